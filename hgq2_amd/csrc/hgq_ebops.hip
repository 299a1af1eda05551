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
#define EB_MAX_ROWS 2048     // rows of a softmax / (head, key) pairs held in LDS
#define EB_MAX_ENTRIES 30720  // bit-width entries of all operands of a launch, staged in LDS

// A quantizer's bit-width view, staged once in LDS: bits of entry j at v[j], stored negative (-0.0 for zero) when the
// straight-through gradient of the entry is closed, so that no later step goes back to global memory.
struct Bits {
    hgq_bits_desc d;
    float *v;
    bool norep;     // the entries tile the cells exactly once: no wrap-around in the broadcast rule
    uint32_t step;  // simple layouts: entry = cell * step (1: an entry per cell, 0: one shared entry)
    __device__ __forceinline__ void stage(float *lds, uint32_t n_cells) {
        v = lds;
        norep = (uint64_t)d.size * (uint64_t)d.inner == n_cells;
        step = d.size == 1 ? 0u : 1u;
        const uint32_t size = (uint32_t)d.size;
        // absent operands read something valid that is then ignored: no load sits behind a branch
        const float *ip = d.kbi ? d.fb : d.i;
        const uint8_t *kp = d.add_mode ? d.k : (const uint8_t *)d.fb;
        const bool vec = (size & 3u) == 0 && (((uintptr_t)d.fb | (uintptr_t)ip | (uintptr_t)kp | (uintptr_t)v) & 15u) == 0;
        if (vec) {
            // four entries per 128-bit load, four loads per array in flight
            for (uint32_t j0 = threadIdx.x * 4; j0 < size; j0 += 4 * 4 * EB_NT) {
                f32x4_t iv[4], fv[4];
                uint32_t kv[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const uint32_t j = j0 + u * 4 * EB_NT, jj = j < size ? j : 0;
                    fv[u] = *(const f32x4_t *)(d.fb + jj);
                    iv[u] = *(const f32x4_t *)(ip + jj);
                    kv[u] = *(const uint32_t *)(kp + jj);
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const uint32_t j = j0 + u * 4 * EB_NT;
                    if (j < size) {
                        f32x4_t o;
#pragma unroll
                        for (int c = 0; c < 4; ++c) o[c] = encode(iv[u][c], fv[u][c], (float)((kv[u] >> (8 * c)) & 0xff));
                        *(f32x4_t *)(v + j) = o;
                    }
                }
            }
        } else {
            for (uint32_t j = threadIdx.x; j < size; j += EB_NT) v[j] = encode(ip[j], d.fb[j], (float)kp[j]);
        }
    }
    // bits / fbits as the quantizer classes define them (see hgq_qbits_fwd), negative when the straight-through gradient is closed
    __device__ __forceinline__ float encode(float i, float fb, float k) const {
        float b;
        bool open = true;
        if (d.kbi) {
            b = rintf(fb);
        } else {
            const float sum = __fadd_rn(rintf(i), rintf(fb));
            open = sum > 0.f;
            b = open ? sum : 0.f;
        }
        if (d.add_mode == 1) b = __fadd_rn(b, k);
        else if (d.add_mode == 2) b = __fadd_rn(b, k * (b > 0.f ? 1.f : 0.f));
        return (open || d.kbi) ? b : -b;
    }
    __device__ __forceinline__ float entry(uint32_t j) const { return d.kbi ? v[j] : fabsf(v[j]); }
    // (cell / inner) % size without the divisions in the common layouts (one shared entry; one entry per cell)
    __device__ __forceinline__ uint32_t entry_of(uint32_t cell) const {
        if (d.size == 1) return 0;
        const uint32_t idx = d.inner == 1 ? cell : cell / (uint32_t)d.inner;
        return norep ? idx : idx % (uint32_t)d.size;
    }
    // a single shared entry, read straight from memory (closed-form paths): value and whether its gradient is open
    __device__ __forceinline__ float lone(bool &open) const {
        const float e = encode(d.kbi ? 0.f : d.i[0], d.fb[0], d.add_mode ? (float)d.k[0] : 0.f);
        open = d.kbi || !signbit(e);
        return d.kbi ? e : fabsf(e);
    }
    __device__ __forceinline__ void put_lone(bool open, float g) const {
        if (d.kbi) {
            d.g_fb[0] = g;
        } else {
            d.g_i[0] = open ? g : 0.f, d.g_fb[0] = open ? g : 0.f;
        }
    }
    // GENERIC = false: every operand of the launch has a simple layout; no branch, no division in the loops
    template <bool GENERIC>
    __device__ __forceinline__ float cell(uint32_t c) const {
        return entry(GENERIC ? entry_of(c) : c * step);
    }
    // straight-through rounding: d bits / d i = d bits / d f = [round(i) + round(f) > 0], d bits / d b = 1
    __device__ __forceinline__ void put(uint32_t j, float g) const {
        if (d.kbi) {
            d.g_fb[j] = g;
        } else {
            const float m = signbit(v[j]) ? 0.f : g;
            d.g_i[j] = m, d.g_fb[j] = m;
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
    if (G == 1) {
        // a thread per entry: no exchange between threads
        for (uint32_t j = threadIdx.x; j < size; j += EB_NT) {
            double s = 0.0;
            if (per == 1) {
                s = (double)f(j);
            } else {
                for (uint32_t c = 0; c < per; ++c) {
                    const uint32_t q = c / inner, r = c - q * inner;
                    s += (double)f((q * size + j) * inner + r);
                }
            }
            b.put(j, (float)s * scale);
        }
        return;
    }
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
        if (loss_term) loss_term[0] = __fmul_rn(e, beta[0]);
    }
    return __fmul_rn(__fmul_rn(beta[0], f2), f1);
}

// QUnaryFunctionLUT: sum over the cells of 2**bits_in * bits_out
template <bool GENERIC>
__global__ __launch_bounds__(EB_NT) void lut_ebops_kernel(hgq_bits_desc d_in, hgq_bits_desc d_out, uint32_t n, float f1, float f2,
                                                          const float *beta, uint32_t *ebops_u32, float *loss_term) {
    __shared__ double red[EB_NT];
    extern __shared__ float pool[];
    Bits in{d_in}, out{d_out};
    if (d_in.size == 1 && d_out.size == 1) {
        // one entry each (tables that are not heterogeneous): the sums are n times one term
        if (threadIdx.x == 0) {
            bool oa, ob;
            const float a = in.lone(oa), b = out.lone(ob), p2 = ldexpf(1.0f, (int)a);
            const float gs = finish((double)n * (double)(p2 * b), f1, f2, beta, ebops_u32, loss_term);
            in.put_lone(oa, (float)((double)n * (double)(p2 * b)) * (gs * HGQ_LN2));
            out.put_lone(ob, (float)((double)n * (double)p2) * gs);
        }
        return;
    }
    in.stage(pool, n), out.stage(pool + d_in.size, n);
    __syncthreads();
    double part = 0.0;
    for (uint32_t c = threadIdx.x; c < n; c += EB_NT) part += (double)(ldexpf(1.0f, (int)in.template cell<GENERIC>(c)) * out.template cell<GENERIC>(c));
    const float gs = finish(block_sum(part, red), f1, f2, beta, ebops_u32, loss_term);
    entry_grads(in, n, gs * HGQ_LN2, [&](uint32_t c) { return ldexpf(1.0f, (int)in.template cell<GENERIC>(c)) * out.template cell<GENERIC>(c); }, red);
    entry_grads(out, n, gs, [&](uint32_t c) { return ldexpf(1.0f, (int)in.template cell<GENERIC>(c)); }, red);
}

// Pooling layers: sum over the cells of bits_in, times parallel_factor, divided by n_parallel (a product, then a correctly
// rounded division, as the reference evaluates it left to right)
template <bool GENERIC>
__global__ __launch_bounds__(EB_NT) void sum_ebops_kernel(hgq_bits_desc d_in, uint32_t n, float parallel_factor, float n_parallel, float f2,
                                                          const float *beta, uint32_t *ebops_u32, float *loss_term) {
    __shared__ double red[EB_NT];
    extern __shared__ float pool[];
    Bits in{d_in};
    const bool lone = d_in.size == 1;
    double raw;
    bool oa = false;
    if (lone) {
        if (threadIdx.x != 0) return;
        raw = (double)n * (double)in.lone(oa);
    } else {
        in.stage(pool, n);
        __syncthreads();
        double part = 0.0;
        for (uint32_t c = threadIdx.x; c < n; c += EB_NT) part += (double)in.template cell<GENERIC>(c);
        raw = block_sum(part, red);
    }
    float e = __fmul_rn((float)raw, parallel_factor);
    if (n_parallel != 1.0f) e = __fdiv_rn(e, n_parallel);
    const float gs = __fmul_rn(finish((double)e, 1.0f, f2, beta, ebops_u32, loss_term), parallel_factor / n_parallel);
    if (lone) {
        in.put_lone(oa, (float)(double)n * gs);
        return;
    }
    entry_grads(in, n, gs, [&](uint32_t) { return 1.0f; }, red);
}

// QSoftmax over the last axis of [R, L] (stable form):
//   sum(bits_sub) + sum(bits_exp) - sum_rows min_l bits_exp + sum(bits_exp * bits_inv[row])
// bits_sub: what the maximum is subtracted from (the layer's input quantizer, else the exp table's); may be absent.
template <bool GENERIC>
__global__ __launch_bounds__(EB_NT) void softmax_ebops_kernel(hgq_bits_desc d_sub, hgq_bits_desc d_exp, hgq_bits_desc d_inv, int has_sub,
                                                              uint32_t R, uint32_t L, float f1, float f2, const float *beta,
                                                              uint32_t *ebops_u32, float *loss_term) {
    __shared__ double red[EB_NT];
    __shared__ float row_min[EB_MAX_ROWS], row_share[EB_MAX_ROWS], row_sum[EB_MAX_ROWS];
    extern __shared__ float pool[];
    Bits sub{d_sub}, ex{d_exp}, inv{d_inv};
    const uint32_t n = R * L;
    if (d_exp.size == 1 && d_inv.size == 1 && (!has_sub || d_sub.size == 1)) {
        // one entry each: every row is L equal values (all of them tie for the minimum)
        if (threadIdx.x == 0) {
            bool oe, oi, os = false;
            const float eb = ex.lone(oe), ib = inv.lone(oi), sb = has_sub ? sub.lone(os) : 0.f;
            float sm = 0.f;
            for (uint32_t l = 0; l < L; ++l) sm += eb;
            const double per_row = (double)sm - (double)eb + (double)(sm * ib);
            const float gs = finish((double)R * per_row + (double)n * (double)sb, f1, f2, beta, ebops_u32, loss_term);
            const float share = 1.f / (float)L;
            if (has_sub) sub.put_lone(os, (float)(double)n * gs);
            ex.put_lone(oe, (float)((double)n * (double)(1.f + ib - share)) * gs);
            inv.put_lone(oi, (float)((double)R * (double)sm) * gs);
        }
        return;
    }
    ex.stage(pool, n), inv.stage(pool + d_exp.size, R);
    if (has_sub) sub.stage(pool + d_exp.size + d_inv.size, n);
    __syncthreads();
    double part = 0.0;
    for (uint32_t r = threadIdx.x; r < R; r += EB_NT) {
        float mn = INFINITY, sm = 0.f, cnt = 0.f;
#pragma unroll 8
        for (uint32_t l = 0; l < L; ++l) mn = fminf(mn, ex.template cell<GENERIC>(r * L + l));
#pragma unroll 8
        for (uint32_t l = 0; l < L; ++l) {
            const float v = ex.template cell<GENERIC>(r * L + l);
            sm += v, cnt += v == mn ? 1.f : 0.f;
        }
        row_min[r] = mn, row_share[r] = 1.f / cnt, row_sum[r] = sm;  // the minimum's gradient is shared by ties
        part += (double)sm - (double)mn + (double)(sm * inv.template cell<GENERIC>(r));
    }
    if (has_sub)
        for (uint32_t c = threadIdx.x; c < n; c += EB_NT) part += (double)sub.template cell<GENERIC>(c);
    const float gs = finish(block_sum(part, red), f1, f2, beta, ebops_u32, loss_term);  // (also orders the LDS rows)
    if (has_sub) entry_grads(sub, n, gs, [&](uint32_t) { return 1.f; }, red);
    entry_grads(ex, n, gs, [&](uint32_t c) {
        const uint32_t r = c / L;
        return 1.f + inv.template cell<GENERIC>(r) - (ex.template cell<GENERIC>(c) == row_min[r] ? row_share[r] : 0.f);
    }, red);
    entry_grads(inv, R, gs, [&](uint32_t r) { return row_sum[r]; }, red);
}

// QMultiHeadAttention: sum_{t,s,n,h} bq[t,n,h] bk[s,n,h] + sum_{n,t,s,h} ba[n,t,s] bv[s,n,h], through the marginal sums
//   Q[n,h] = sum_t bq, K[n,h] = sum_s bk, A[n,s] = sum_t ba, V[s,n] = sum_h bv.
// Four workgroups: each forms the marginal sums and the total (the same bits in each), then writes the gradients of one
// of the four operands; the first also writes the value.
template <bool GENERIC>
__global__ __launch_bounds__(EB_NT) void mha_ebops_kernel(hgq_bits_desc d_q, hgq_bits_desc d_k, hgq_bits_desc d_v, hgq_bits_desc d_a, uint32_t T,
                                                          uint32_t S, uint32_t N, uint32_t H, uint32_t Hv, float f1, float f2,
                                                          const float *beta, uint32_t *ebops_u32, float *loss_term) {
    __shared__ double red[EB_NT];
    __shared__ float Qm[EB_NT], Km[EB_NT], Am[EB_MAX_ROWS], Vm[EB_MAX_ROWS];
    extern __shared__ float pool[];
    Bits bq{d_q}, bk{d_k}, bv{d_v}, ba{d_a};
    bq.stage(pool, T * N * H), bk.stage(pool + d_q.size, S * N * H), bv.stage(pool + d_q.size + d_k.size, S * N * Hv);
    ba.stage(pool + d_q.size + d_k.size + d_v.size, N * T * S);
    __syncthreads();
    const uint32_t NH = N * H, NS = N * S;
    for (uint32_t e = threadIdx.x; e < NH; e += EB_NT) {
        float sq = 0.f, sk = 0.f;
#pragma unroll 8
        for (uint32_t t = 0; t < T; ++t) sq += bq.template cell<GENERIC>(t * NH + e);
#pragma unroll 8
        for (uint32_t s = 0; s < S; ++s) sk += bk.template cell<GENERIC>(s * NH + e);
        Qm[e] = sq, Km[e] = sk;
    }
    for (uint32_t e = threadIdx.x; e < NS; e += EB_NT) {
        const uint32_t n = e / S, s = e - n * S;
        float sa = 0.f, sv = 0.f;
#pragma unroll 8
        for (uint32_t t = 0; t < T; ++t) sa += ba.template cell<GENERIC>((n * T + t) * S + s);
#pragma unroll 8
        for (uint32_t h = 0; h < Hv; ++h) sv += bv.template cell<GENERIC>((s * N + n) * Hv + h);
        Am[e] = sa, Vm[s * N + n] = sv;
    }
    __syncthreads();
    double part = 0.0;
    for (uint32_t e = threadIdx.x; e < NH; e += EB_NT) part += (double)Qm[e] * (double)Km[e];
    for (uint32_t e = threadIdx.x; e < NS; e += EB_NT) {
        const uint32_t n = e / S, s = e - n * S;
        part += (double)Am[e] * (double)Vm[s * N + n];
    }
    const bool lead = blockIdx.x == 0;
    const float gs = finish(block_sum(part, red), f1, f2, beta, lead ? ebops_u32 : nullptr, lead ? loss_term : nullptr);
    const FastDiv by_nh(NH), by_nhv(N * Hv), by_hv(Hv), by_n(N), by_ts(T * S), by_s(S);
    const uint32_t which = blockIdx.x, all = gridDim.x == 1;
    if (all || which == 0) entry_grads(bq, T * NH, gs, [&](uint32_t c) { return Km[by_nh.mod(c)]; }, red);
    if (all || which == 1) entry_grads(bk, S * NH, gs, [&](uint32_t c) { return Qm[by_nh.mod(c)]; }, red);
    if (all || which == 2)
        entry_grads(bv, S * N * Hv, gs, [&](uint32_t c) {
            const uint32_t s = by_nhv.div(c), n = by_n.mod(by_hv.div(c));
            return Am[n * S + s];
        }, red);
    if (all || which == 3)
        entry_grads(ba, N * T * S, gs, [&](uint32_t c) {
            const uint32_t n = by_ts.div(c), s = by_s.mod(c);
            return Vm[s * N + n];
        }, red);
}

static int pool_bytes(int64_t entries, const char *who, size_t &bytes) {
    if (entries > EB_MAX_ENTRIES) return fail(HGQ_ERR_UNSUPPORTED, "%s: %lld bit-width entries exceed the %d held in LDS", who, (long long)entries, EB_MAX_ENTRIES);
    bytes = (size_t)entries * sizeof(float);
    return HGQ_OK;
}

template <class K>
static int raise_pool(K kernel, bool &raised, const char *who) {
    if (raised) return HGQ_OK;
    if (hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, EB_MAX_ENTRIES * (int)sizeof(float)) != hipSuccess) {
        (void)hipGetLastError();
        return fail(HGQ_ERR_LAUNCH, "%s: cannot reserve LDS", who);
    }
    raised = true;
    return HGQ_OK;
}

static bool simple_layout(const hgq_bits_desc *d, int64_t n_cells) { return !d || d->size == 1 || (d->size == n_cells && d->inner == 1); }

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
    size_t lds;
    static bool raised = false, raised2 = false;
    if ((rc = pool_bytes(bits_in->size + bits_out->size, who, lds)) || (rc = raise_pool(lut_ebops_kernel<true>, raised, who)) ||
        (rc = raise_pool(lut_ebops_kernel<false>, raised2, who)))
        return rc;
    const bool generic = !(simple_layout(bits_in, n_cells) && simple_layout(bits_out, n_cells));
    hipLaunchKernelGGL(generic ? lut_ebops_kernel<true> : lut_ebops_kernel<false>, dim3(1), dim3(EB_NT), lds, (hipStream_t)stream, *bits_in, *bits_out, (uint32_t)n_cells, scale,
                       ebops_factor, beta, ebops_u32, loss_term);
    return check_launch(who);
}

extern "C" int hgq_sum_ebops(const hgq_bits_desc *bits_in, int64_t n_cells, float parallel_factor, float n_parallel, float ebops_factor,
                             const float *beta, uint32_t *ebops_u32, float *loss_term, void *stream) {
    const char *who = "hgq_sum_ebops";
    if (n_cells < 1 || n_cells >= (1ll << 31)) return fail(HGQ_ERR_UNSUPPORTED, "%s: 1 <= n_cells < 2**31 expected", who);
    if (!(n_parallel > 0.f)) return fail(HGQ_ERR_ARG, "%s: n_parallel must be positive", who);
    int rc;
    if ((rc = check_bits(bits_in, n_cells, who, "bits_in"))) return rc;
    if (!beta || !loss_term) return fail(HGQ_ERR_ARG, "%s: null pointer", who);
    size_t lds;
    static bool raised = false, raised2 = false;
    if ((rc = pool_bytes(bits_in->size, who, lds)) || (rc = raise_pool(sum_ebops_kernel<true>, raised, who)) ||
        (rc = raise_pool(sum_ebops_kernel<false>, raised2, who)))
        return rc;
    const bool generic = !simple_layout(bits_in, n_cells);
    hipLaunchKernelGGL(generic ? sum_ebops_kernel<true> : sum_ebops_kernel<false>, dim3(1), dim3(EB_NT), lds, (hipStream_t)stream, *bits_in,
                       (uint32_t)n_cells, parallel_factor, n_parallel, ebops_factor, beta, ebops_u32, loss_term);
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
    size_t lds;
    static bool raised = false, raised2 = false;
    if ((rc = pool_bytes(bits_exp->size + bits_inv->size + (bits_sub ? bits_sub->size : 0), who, lds)) ||
        (rc = raise_pool(softmax_ebops_kernel<true>, raised, who)) || (rc = raise_pool(softmax_ebops_kernel<false>, raised2, who)))
        return rc;
    const bool generic = !(simple_layout(bits_sub, rows * L) && simple_layout(bits_exp, rows * L) && simple_layout(bits_inv, rows));
    hipLaunchKernelGGL(generic ? softmax_ebops_kernel<true> : softmax_ebops_kernel<false>, dim3(1), dim3(EB_NT), lds, (hipStream_t)stream, bits_sub ? *bits_sub : *bits_exp, *bits_exp, *bits_inv,
                       bits_sub ? 1 : 0, (uint32_t)rows, (uint32_t)L, instance_factor, ebops_factor, beta, ebops_u32, loss_term);
    return check_launch(who);
}

extern "C" int hgq_mha_ebops(const hgq_bits_desc *bits_q, const hgq_bits_desc *bits_k, const hgq_bits_desc *bits_v, const hgq_bits_desc *bits_attn,
                             int T, int S, int N, int H, int Hv, float parallel_factor, float ebops_factor, const float *beta,
                             uint32_t *ebops_u32, float *loss_term, void *stream) {
    const char *who = "hgq_mha_ebops";
    if (T < 1 || S < 1 || N < 1 || H < 1 || Hv < 1) return fail(HGQ_ERR_ARG, "%s: bad sizes", who);
    if ((int64_t)N * H > EB_NT || (int64_t)N * S > EB_MAX_ROWS || (int64_t)N * T * S >= (1ll << 21) || (int64_t)(T + S) * N * (H + Hv) >= (1ll << 21))
        return fail(HGQ_ERR_UNSUPPORTED, "%s: N * H <= %d, N * S <= %d and fewer than 2**21 cells per tensor expected", who, EB_NT, EB_MAX_ROWS);
    int rc;
    if ((rc = check_bits(bits_q, (int64_t)T * N * H, who, "bits_q")) || (rc = check_bits(bits_k, (int64_t)S * N * H, who, "bits_k")) ||
        (rc = check_bits(bits_v, (int64_t)S * N * Hv, who, "bits_v")) || (rc = check_bits(bits_attn, (int64_t)N * T * S, who, "bits_attn")))
        return rc;
    if (!beta || !loss_term) return fail(HGQ_ERR_ARG, "%s: null pointer", who);
    size_t lds;
    static bool raised = false, raised2 = false;
    if ((rc = pool_bytes(bits_q->size + bits_k->size + bits_v->size + bits_attn->size, who, lds)) || (rc = raise_pool(mha_ebops_kernel<true>, raised, who)) ||
        (rc = raise_pool(mha_ebops_kernel<false>, raised2, who)))
        return rc;
    const bool generic = !(simple_layout(bits_q, (int64_t)T * N * H) && simple_layout(bits_k, (int64_t)S * N * H) &&
                           simple_layout(bits_v, (int64_t)S * N * Hv) && simple_layout(bits_attn, (int64_t)N * T * S));
    hipLaunchKernelGGL(generic ? mha_ebops_kernel<true> : mha_ebops_kernel<false>, dim3(4), dim3(EB_NT), lds, (hipStream_t)stream, *bits_q, *bits_k, *bits_v, *bits_attn, (uint32_t)T, (uint32_t)S,
                       (uint32_t)N, (uint32_t)H, (uint32_t)Hv, parallel_factor, ebops_factor, beta, ebops_u32, loss_term);
    return check_launch(who);
}
