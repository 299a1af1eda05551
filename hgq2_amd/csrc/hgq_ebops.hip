// EBOPs of the layers whose estimate is plain algebra on bit-width tensors - QUnaryFunctionLUT,
// QSoftmax, QMultiHeadAttention - each as ONE launch that reads the quantizers' raw variables and
// leaves the value (uint32 variable), the loss term ebops * beta and the gradients of that term
// with respect to the variables.  (As library calls the same algebra is 10 - 20 launches per layer
// and as many again in the backward pass, each on a few thousand elements.)
//
// One workgroup of 1024 threads; every sum is formed in a fixed order (no atomics).  A gradient entry
// is the sum over the cells that broadcast from it: cells are split over thread groups and combined
// by a tree in LDS, so scalar operands and full tables take the same code.
#include <math.h>

#include "hgq_device.h"
#include "hgq_host.h"

namespace hgq {

#define EB_NT 1024
#define EB_MAX_ROWS 4096  // rows of a softmax / (head, key) pairs held in LDS

struct Bits {
    hgq_bits_desc d;
    __device__ __forceinline__ float raw_sum(uint32_t j) const { return __fadd_rn(rintf(d.i[j]), rintf(d.fb[j])); }
    // bits / fbits of entry j as the quantizer classes define them (see hgq_qbits_fwd)
    __device__ __forceinline__ float entry(uint32_t j) const {
        float b;
        if (d.kbi) {
            b = rintf(d.fb[j]);
        } else {
            const float s = raw_sum(j);
            b = s > 0.f ? s : 0.f;
        }
        if (d.add_mode == 1) b = __fadd_rn(b, (float)d.k[j]);
        else if (d.add_mode == 2) b = __fadd_rn(b, (float)d.k[j] * (b > 0.f ? 1.f : 0.f));
        return b;
    }
    __device__ __forceinline__ uint32_t entry_of(uint32_t cell) const { return (cell / (uint32_t)d.inner) % (uint32_t)d.size; }
    __device__ __forceinline__ float cell(uint32_t c) const { return entry(entry_of(c)); }
    // straight-through rounding: d bits / d i = d bits / d f = [round(i) + round(f) > 0], d bits / d b = 1
    __device__ __forceinline__ void put(uint32_t j, float g) const {
        if (d.kbi) {
            d.g_fb[j] = g;
        } else {
            const float v = raw_sum(j) > 0.f ? g : 0.f;
            d.g_i[j] = v, d.g_fb[j] = v;
        }
    }
};

// Fixed-order sum over the workgroup (double: exact for integer-valued terms far beyond 2**24).
__device__ __forceinline__ double block_sum(double v, double *red) {
    const int t = threadIdx.x;
    red[t] = v;
    __syncthreads();
    for (int o = EB_NT / 2; o > 0; o >>= 1) {
        if (t < o) red[t] += red[t + o];
        __syncthreads();
    }
    const double s = red[0];
    __syncthreads();
    return s;
}

// g[j] = scale * sum over the cells c of entry j of f(c), for every entry of b; n_cells = numel of the tensor b is broadcast to.
template <class F>
__device__ __forceinline__ void entry_grads(const Bits &b, uint32_t n_cells, float scale, F f, double *red) {
    const uint32_t size = (uint32_t)b.d.size, inner = (uint32_t)b.d.inner, per = n_cells / size;  // cells per entry
    uint32_t P2 = 1;
    while (P2 < size && P2 < EB_NT) P2 <<= 1;
    const uint32_t G = EB_NT / P2, jl = threadIdx.x % P2, grp = threadIdx.x / P2;
    for (uint32_t j0 = 0; j0 < size; j0 += P2) {
        const uint32_t j = j0 + jl;
        double s = 0.0;
        if (j < size)
            for (uint32_t c = grp; c < per; c += G) {
                const uint32_t q = c / inner, r = c - q * inner;
                s += (double)f((q * size + j) * inner + r);
            }
        red[threadIdx.x] = s;
        __syncthreads();
        for (uint32_t o = G / 2; o > 0; o >>= 1) {
            if (grp < o) red[threadIdx.x] += red[threadIdx.x + o * P2];
            __syncthreads();
        }
        if (grp == 0 && j < size) b.put(j, (float)red[jl] * scale);
        __syncthreads();
    }
}

// value -> uint32 variable, loss term; returns the factor of the unit-upstream gradients
__device__ __forceinline__ float finish(double raw, float f1, float f2, const float *beta, uint32_t *ebops_u32, float *loss_term) {
    const float e = __fmul_rn(__fmul_rn((float)raw, f1), f2);
    if (threadIdx.x == 0) {
        if (ebops_u32) ebops_u32[0] = (uint32_t)(int64_t)e;
        loss_term[0] = __fmul_rn(e, beta[0]);
    }
    return __fmul_rn(__fmul_rn(beta[0], f2), f1);
}

// QUnaryFunctionLUT: sum over the cells of 2**bits_in * bits_out
__global__ __launch_bounds__(EB_NT) void lut_ebops_kernel(hgq_bits_desc d_in, hgq_bits_desc d_out, uint32_t n, float f1, float f2,
                                                          const float *beta, uint32_t *ebops_u32, float *loss_term) {
    __shared__ double red[EB_NT];
    Bits in{d_in}, out{d_out};
    double part = 0.0;
    for (uint32_t c = threadIdx.x; c < n; c += EB_NT) part += (double)(ldexpf(1.0f, (int)in.cell(c)) * out.cell(c));
    const float gs = finish(block_sum(part, red), f1, f2, beta, ebops_u32, loss_term);
    entry_grads(in, n, gs * HGQ_LN2, [&](uint32_t c) { return ldexpf(1.0f, (int)in.cell(c)) * out.cell(c); }, red);
    entry_grads(out, n, gs, [&](uint32_t c) { return ldexpf(1.0f, (int)in.cell(c)); }, red);
}

// QSoftmax over the last axis of [R, L] (stable form):
//   sum(bits_sub) + sum(bits_exp) - sum_rows min_l bits_exp + sum(bits_exp * bits_inv[row])
// bits_sub: what the maximum is subtracted from (the layer's input quantizer, else the exp table's); may be absent.
__global__ __launch_bounds__(EB_NT) void softmax_ebops_kernel(hgq_bits_desc d_sub, hgq_bits_desc d_exp, hgq_bits_desc d_inv, int has_sub,
                                                              uint32_t R, uint32_t L, float f1, float f2, const float *beta,
                                                              uint32_t *ebops_u32, float *loss_term) {
    __shared__ double red[EB_NT];
    __shared__ float row_min[EB_MAX_ROWS], row_share[EB_MAX_ROWS], row_sum[EB_MAX_ROWS];
    Bits sub{d_sub}, ex{d_exp}, inv{d_inv};
    const uint32_t n = R * L;
    double part = 0.0;
    for (uint32_t r = threadIdx.x; r < R; r += EB_NT) {
        float mn = INFINITY, sm = 0.f, cnt = 0.f;
        for (uint32_t l = 0; l < L; ++l) mn = fminf(mn, ex.cell(r * L + l));
        for (uint32_t l = 0; l < L; ++l) {
            const float v = ex.cell(r * L + l);
            sm += v, cnt += v == mn ? 1.f : 0.f;
        }
        row_min[r] = mn, row_share[r] = 1.f / cnt, row_sum[r] = sm;  // the minimum's gradient is shared by ties
        part += (double)sm - (double)mn + (double)(sm * inv.cell(r));
    }
    if (has_sub)
        for (uint32_t c = threadIdx.x; c < n; c += EB_NT) part += (double)sub.cell(c);
    const float gs = finish(block_sum(part, red), f1, f2, beta, ebops_u32, loss_term);  // (also orders the LDS rows)
    if (has_sub) entry_grads(sub, n, gs, [&](uint32_t) { return 1.f; }, red);
    entry_grads(ex, n, gs, [&](uint32_t c) {
        const uint32_t r = c / L;
        return 1.f + inv.cell(r) - (ex.cell(c) == row_min[r] ? row_share[r] : 0.f);
    }, red);
    entry_grads(inv, R, gs, [&](uint32_t r) { return row_sum[r]; }, red);
}

// QMultiHeadAttention: sum_{t,s,n,h} bq[t,n,h] bk[s,n,h] + sum_{n,t,s,h} ba[n,t,s] bv[s,n,h], through the marginal sums
//   Q[n,h] = sum_t bq, K[n,h] = sum_s bk, A[n,s] = sum_t ba, V[s,n] = sum_h bv.
__global__ __launch_bounds__(EB_NT) void mha_ebops_kernel(hgq_bits_desc d_q, hgq_bits_desc d_k, hgq_bits_desc d_v, hgq_bits_desc d_a, uint32_t T,
                                                          uint32_t S, uint32_t N, uint32_t H, uint32_t Hv, float f1, float f2,
                                                          const float *beta, uint32_t *ebops_u32, float *loss_term) {
    __shared__ double red[EB_NT];
    __shared__ float Qm[EB_NT], Km[EB_NT], Am[EB_MAX_ROWS], Vm[EB_MAX_ROWS];
    Bits bq{d_q}, bk{d_k}, bv{d_v}, ba{d_a};
    const uint32_t NH = N * H, NS = N * S;
    for (uint32_t e = threadIdx.x; e < NH; e += EB_NT) {
        float sq = 0.f, sk = 0.f;
        for (uint32_t t = 0; t < T; ++t) sq += bq.cell(t * NH + e);
        for (uint32_t s = 0; s < S; ++s) sk += bk.cell(s * NH + e);
        Qm[e] = sq, Km[e] = sk;
    }
    for (uint32_t e = threadIdx.x; e < NS; e += EB_NT) {
        const uint32_t n = e / S, s = e - n * S;
        float sa = 0.f, sv = 0.f;
        for (uint32_t t = 0; t < T; ++t) sa += ba.cell((n * T + t) * S + s);
        for (uint32_t h = 0; h < Hv; ++h) sv += bv.cell((s * N + n) * Hv + h);
        Am[e] = sa, Vm[s * N + n] = sv;
    }
    __syncthreads();
    double part = 0.0;
    for (uint32_t e = threadIdx.x; e < NH; e += EB_NT) part += (double)Qm[e] * (double)Km[e];
    for (uint32_t e = threadIdx.x; e < NS; e += EB_NT) {
        const uint32_t n = e / S, s = e - n * S;
        part += (double)Am[e] * (double)Vm[s * N + n];
    }
    const float gs = finish(block_sum(part, red), f1, f2, beta, ebops_u32, loss_term);
    entry_grads(bq, T * NH, gs, [&](uint32_t c) { return Km[c % NH]; }, red);
    entry_grads(bk, S * NH, gs, [&](uint32_t c) { return Qm[c % NH]; }, red);
    entry_grads(bv, S * N * Hv, gs, [&](uint32_t c) {
        const uint32_t s = c / (N * Hv), n = (c / Hv) % N;
        return Am[n * S + s];
    }, red);
    entry_grads(ba, N * T * S, gs, [&](uint32_t c) {
        const uint32_t n = c / (T * S), s = c % S;
        return Vm[s * N + n];
    }, red);
}

static int check_bits(const hgq_bits_desc *d, int64_t n_cells, const char *who, const char *name) {
    if (!d) return fail(HGQ_ERR_ARG, "%s: %s is null", who, name);
    if (d->size < 1 || d->inner < 1 || n_cells % (d->size * d->inner) != 0)
        return fail(HGQ_ERR_ARG, "%s: %s: size=%lld, inner=%lld do not tile %lld cells", who, name, (long long)d->size, (long long)d->inner,
                    (long long)n_cells);
    if (!d->fb || !d->g_fb || (!d->kbi && (!d->i || !d->g_i)) || (d->add_mode && !d->k))
        return fail(HGQ_ERR_ARG, "%s: %s: null pointer", who, name);
    if (d->add_mode < 0 || d->add_mode > 2) return fail(HGQ_ERR_ARG, "%s: %s: add_mode must be 0, 1 or 2", who, name);
    return HGQ_OK;
}

}  // namespace hgq

using namespace hgq;

extern "C" int hgq_lut_ebops(const hgq_bits_desc *bits_in, const hgq_bits_desc *bits_out, int64_t n_cells, float scale, float ebops_factor,
                             const float *beta, uint32_t *ebops_u32, float *loss_term, void *stream) {
    const char *who = "hgq_lut_ebops";
    if (n_cells < 1 || n_cells >= (1ll << 31)) return fail(HGQ_ERR_UNSUPPORTED, "%s: 1 <= n_cells < 2**31 expected", who);
    int rc;
    if ((rc = check_bits(bits_in, n_cells, who, "bits_in")) || (rc = check_bits(bits_out, n_cells, who, "bits_out"))) return rc;
    if (!beta || !loss_term) return fail(HGQ_ERR_ARG, "%s: null pointer", who);
    hipLaunchKernelGGL(lut_ebops_kernel, dim3(1), dim3(EB_NT), 0, (hipStream_t)stream, *bits_in, *bits_out, (uint32_t)n_cells, scale,
                       ebops_factor, beta, ebops_u32, loss_term);
    return check_launch(who);
}

extern "C" int hgq_softmax_ebops(const hgq_bits_desc *bits_sub, const hgq_bits_desc *bits_exp, const hgq_bits_desc *bits_inv, int64_t rows, int L,
                                 float instance_factor, float ebops_factor, const float *beta, uint32_t *ebops_u32, float *loss_term,
                                 void *stream) {
    const char *who = "hgq_softmax_ebops";
    if (rows < 1 || L < 1 || rows > EB_MAX_ROWS || rows * L >= (1ll << 31))
        return fail(HGQ_ERR_UNSUPPORTED, "%s: 1 <= rows <= %d expected, got %lld", who, EB_MAX_ROWS, (long long)rows);
    int rc;
    if (bits_sub && (rc = check_bits(bits_sub, rows * L, who, "bits_sub"))) return rc;
    if ((rc = check_bits(bits_exp, rows * L, who, "bits_exp")) || (rc = check_bits(bits_inv, rows, who, "bits_inv"))) return rc;
    if (!beta || !loss_term) return fail(HGQ_ERR_ARG, "%s: null pointer", who);
    hipLaunchKernelGGL(softmax_ebops_kernel, dim3(1), dim3(EB_NT), 0, (hipStream_t)stream, bits_sub ? *bits_sub : *bits_exp, *bits_exp, *bits_inv,
                       bits_sub ? 1 : 0, (uint32_t)rows, (uint32_t)L, instance_factor, ebops_factor, beta, ebops_u32, loss_term);
    return check_launch(who);
}

extern "C" int hgq_mha_ebops(const hgq_bits_desc *bits_q, const hgq_bits_desc *bits_k, const hgq_bits_desc *bits_v, const hgq_bits_desc *bits_attn,
                             int T, int S, int N, int H, int Hv, float parallel_factor, float ebops_factor, const float *beta,
                             uint32_t *ebops_u32, float *loss_term, void *stream) {
    const char *who = "hgq_mha_ebops";
    if (T < 1 || S < 1 || N < 1 || H < 1 || Hv < 1) return fail(HGQ_ERR_ARG, "%s: bad sizes", who);
    if ((int64_t)N * H > EB_NT || (int64_t)N * S > EB_MAX_ROWS || (int64_t)N * T * S >= (1ll << 31) || (int64_t)(T + S) * N * (H + Hv) >= (1ll << 31))
        return fail(HGQ_ERR_UNSUPPORTED, "%s: N * H <= %d and N * S <= %d expected", who, EB_NT, EB_MAX_ROWS);
    int rc;
    if ((rc = check_bits(bits_q, (int64_t)T * N * H, who, "bits_q")) || (rc = check_bits(bits_k, (int64_t)S * N * H, who, "bits_k")) ||
        (rc = check_bits(bits_v, (int64_t)S * N * Hv, who, "bits_v")) || (rc = check_bits(bits_attn, (int64_t)N * T * S, who, "bits_attn")))
        return rc;
    if (!beta || !loss_term) return fail(HGQ_ERR_ARG, "%s: null pointer", who);
    hipLaunchKernelGGL(mha_ebops_kernel, dim3(1), dim3(EB_NT), 0, (hipStream_t)stream, *bits_q, *bits_k, *bits_v, *bits_attn, (uint32_t)T, (uint32_t)S,
                       (uint32_t)N, (uint32_t)H, (uint32_t)Hv, parallel_factor, ebops_factor, beta, ebops_u32, loss_term);
    return check_launch(who);
}
