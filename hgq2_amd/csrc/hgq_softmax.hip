// Table-driven softmax of QSoftmax / QMultiHeadAttention as one pass over the score tensor.
//
//   d = max(x) - x;  e = Q_exp_out(exp(-Q_exp_in(d) * scale));  s = sum(e);
//   r = Q_inv_out(1 / (Q_inv_in(s) + eps));  y = Q_out(e * r)
//
// A row (the softmax axis, contiguous, L <= 256 elements) lives in the lanes of one wavefront:
// SUB lanes per row (a power of two >= L, or 64 lanes holding EPL elements each), 64 / SUB rows
// side by side.  The four table quantizers have one shared bit-width entry each; the output
// quantizer has a [P, L] table, row r using entry r % P.  A wavefront owns fixed table rows and
// walks along the batch, so the output quantizer's operands, its abs-max tracker and its
// bit-width gradients stay in registers; max / sum over the row are xor-shuffles.
#include <math.h>

#include "hgq_device.h"
#include "hgq_host.h"

namespace hgq {

// A quantizer with a single shared bit-width entry, resolved once per wavefront.
struct SharedQ {
    bool present, training, kbi;
    int rm, om;
    KIF p;
    __device__ __forceinline__ void init(const hgq_qdesc &d) {
        present = d.k != nullptr;
        training = false, kbi = false, rm = 0, om = 0;
        p.k = 0.f, p.i = 0.f, p.f = 0.f;
        if (!present) return;
        const Mode m(d.mode);
        rm = m.round_mode, om = m.overflow_mode, training = m.training, kbi = m.kbi;
        p = resolve_kif(load_k(d.k, 0, m.k_u8), d.i[0], d.fb[0], m.kbi, m.round_params);
    }
    __device__ __forceinline__ float fwd(float x) const { return present ? quantize_dyn(x, p, rm, om, training) : x; }
    // gradients w.r.t. the input and the two stored variables (i and f, or i and b)
    __device__ __forceinline__ void grad(float x, float dy, float &dx, float &di, float &dfb) const {
        if (!present) {
            dx = dy, di = 0.f, dfb = 0.f;
            return;
        }
        quantize_grad_dyn(x, dy, p, rm, om, dx, di, dfb);
        if (kbi) di -= dfb;  // f = b - i
    }
};

// The output quantizer: per-lane operands.
struct LaneQ {
    int rm, om;
    bool present, training, kbi;
    __device__ __forceinline__ void init(const hgq_qdesc &d) {
        present = d.k != nullptr;
        const Mode m(present ? d.mode : 0);
        rm = m.round_mode, om = m.overflow_mode, training = m.training, kbi = m.kbi;
    }
    __device__ __forceinline__ KIF load(const hgq_qdesc &d, int64_t idx) const {
        const Mode m(d.mode);
        return resolve_kif(load_k(d.k, idx, m.k_u8), d.i[idx], d.fb[idx], m.kbi, m.round_params);
    }
};

template <int SUB>
__device__ __forceinline__ float sub_max(float v) {
#pragma unroll
    for (int o = SUB / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
template <int SUB>
__device__ __forceinline__ float sub_sum(float v) {
#pragma unroll
    for (int o = SUB / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_sum(float v) { return sub_sum<64>(v); }
__device__ __forceinline__ uint32_t wave_max_bits(uint32_t v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const uint32_t t = (uint32_t)__shfl_xor((int)v, o, 64);
        v = t > v ? t : v;
    }
    return v;
}

// Work decomposition shared by the forward and backward kernels.
struct SoftmaxPlan {
    int64_t rows;       // number of softmax rows
    int L;              // row length
    int64_t Pq;         // table rows walked by the grid (a multiple of the rows one wavefront takes per step)
    int64_t P_table;    // rows of the output quantizer's bit-width table (1 if shared or absent)
    int64_t n_batches;  // ceil(rows / Pq)
    int64_t PG;         // position groups = Pq / (rows per wavefront step)
    int bpc;            // batches per chunk
    int64_t n_chunks;
    int SUB, EPL, NP;
    __host__ __device__ int64_t n_waves() const { return PG * n_chunks; }
};

#define SM_WAVES_PER_BLOCK 4

template <int SUB, int EPL, int NP>
__global__ __launch_bounds__(64 * SM_WAVES_PER_BLOCK) void qsoftmax_fwd_kernel(
    const float *__restrict__ x, float *__restrict__ y, SoftmaxPlan pl, float scale, float eps, hgq_qdesc d1, hgq_qdesc d2,
    hgq_qdesc d3, hgq_qdesc d4, hgq_qdesc dq, uint32_t *amax1, uint32_t *amax3, uint32_t *amax_o) {
    constexpr int RPW = 64 / SUB;
    const int64_t gw = (int64_t)blockIdx.x * SM_WAVES_PER_BLOCK + (threadIdx.x >> 6);
    if (gw >= pl.n_waves()) return;
    const int lane = threadIdx.x & 63, slot = lane / SUB, col = lane % SUB;
    const int64_t pg = gw % pl.PG, chunk = gw / pl.PG;
    SharedQ q1, q2, q3, q4;
    q1.init(d1), q2.init(d2), q3.init(d3), q4.init(d4);
    LaneQ qo;
    qo.init(dq);
    const int L = pl.L;
    KIF po[NP][EPL];
    uint32_t mo[NP][EPL];
    int64_t pos[NP];
#pragma unroll
    for (int np = 0; np < NP; ++np) {
        pos[np] = (pg * NP + np) * RPW + slot;
#pragma unroll
        for (int e = 0; e < EPL; ++e) {
            mo[np][e] = 0;
            const int c = col + 64 * e;
            po[np][e].k = 0.f, po[np][e].i = 0.f, po[np][e].f = 0.f;
            if (qo.present && c < L) po[np][e] = qo.load(dq, (pos[np] % pl.P_table) * L + c);
        }
    }
    uint32_t m1 = 0, m3 = 0;
    const int64_t b0 = chunk * pl.bpc, b1 = min(pl.n_batches, b0 + pl.bpc);
    for (int64_t b = b0; b < b1; ++b) {
        float xv[NP][EPL];
        bool act[NP][EPL];
#pragma unroll
        for (int np = 0; np < NP; ++np) {
            const int64_t r = b * pl.Pq + pos[np];
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                const int c = col + 64 * e;
                act[np][e] = r < pl.rows && c < L;
                xv[np][e] = act[np][e] ? __builtin_nontemporal_load(x + r * L + c) : -INFINITY;
            }
        }
#pragma unroll
        for (int np = 0; np < NP; ++np) {
            const int64_t r = b * pl.Pq + pos[np];
            float mx = xv[np][0];
#pragma unroll
            for (int e = 1; e < EPL; ++e) mx = fmaxf(mx, xv[np][e]);
            mx = sub_max<SUB>(mx);
            float ev[EPL], s = 0.f;
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                const float d = __fsub_rn(mx, xv[np][e]);
                const float a = q1.fwd(d);
                const float t = expf(__fmul_rn(-a, scale));
                ev[e] = act[np][e] ? q2.fwd(t) : 0.f;
                if (act[np][e]) m1 = max(m1, abs_bits(a));
                s += ev[e];
            }
            s = sub_sum<SUB>(s);
            const float sq = q3.fwd(s);
            const float rr = q4.fwd(__fdiv_rn(1.0f, __fadd_rn(sq, eps)));
            if (r < pl.rows) m3 = max(m3, abs_bits(sq));
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                float yv = __fmul_rn(ev[e], rr);
                if (qo.present) yv = quantize_dyn(yv, po[np][e], qo.rm, qo.om, qo.training);
                if (act[np][e]) {
                    __builtin_nontemporal_store(yv, y + r * L + col + 64 * e);
                    mo[np][e] = max(mo[np][e], abs_bits(yv));
                }
            }
        }
    }
    if (amax1) {
        m1 = wave_max_bits(m1);
        if (lane == 0) atomicMax(amax1, m1);
    }
    if (amax3) {
        m3 = wave_max_bits(m3);
        if (lane == 0) atomicMax(amax3, m3);
    }
    if (amax_o) {
#pragma unroll
        for (int np = 0; np < NP; ++np)
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                const int c = col + 64 * e;
                if (c < L && mo[np][e]) atomicMax(&amax_o[(pos[np] % pl.P_table) * L + c], mo[np][e]);
            }
    }
}

// Backward: recomputes the forward chain from x, then walks it in reverse.  Per-wavefront
// partial sums of the bit-width gradients go to workspace slices that a second kernel adds up
// in a fixed order.
//   workspace = [n_waves, 8] scalar slices | [n_chunks, Pq * L] d/di of Q_out | [n_chunks, Pq * L] d/df of Q_out
template <int SUB, int EPL, int NP>
__global__ __launch_bounds__(64 * SM_WAVES_PER_BLOCK) void qsoftmax_bwd_kernel(
    const float *__restrict__ dy, const float *__restrict__ x, float *__restrict__ dx, SoftmaxPlan pl, float scale,
    float eps, hgq_qdesc d1, hgq_qdesc d2, hgq_qdesc d3, hgq_qdesc d4, hgq_qdesc dq, float *__restrict__ ws) {
    constexpr int RPW = 64 / SUB;
    const int64_t gw = (int64_t)blockIdx.x * SM_WAVES_PER_BLOCK + (threadIdx.x >> 6);
    if (gw >= pl.n_waves()) return;
    const int lane = threadIdx.x & 63, slot = lane / SUB, col = lane % SUB;
    const int64_t pg = gw % pl.PG, chunk = gw / pl.PG;
    SharedQ q1, q2, q3, q4;
    q1.init(d1), q2.init(d2), q3.init(d3), q4.init(d4);
    LaneQ qo;
    qo.init(dq);
    const int L = pl.L;
    KIF po[NP][EPL];
    float goi[NP][EPL], gof[NP][EPL];
    int64_t pos[NP];
#pragma unroll
    for (int np = 0; np < NP; ++np) {
        pos[np] = (pg * NP + np) * RPW + slot;
#pragma unroll
        for (int e = 0; e < EPL; ++e) {
            goi[np][e] = 0.f, gof[np][e] = 0.f;
            const int c = col + 64 * e;
            po[np][e].k = 0.f, po[np][e].i = 0.f, po[np][e].f = 0.f;
            if (qo.present && c < L) po[np][e] = qo.load(dq, (pos[np] % pl.P_table) * L + c);
        }
    }
    float gs[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) gs[j] = 0.f;
    const int64_t b0 = chunk * pl.bpc, b1 = min(pl.n_batches, b0 + pl.bpc);
    for (int64_t b = b0; b < b1; ++b) {
        float xv[NP][EPL], gv[NP][EPL];
        bool act[NP][EPL];
#pragma unroll
        for (int np = 0; np < NP; ++np) {
            const int64_t r = b * pl.Pq + pos[np];
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                const int c = col + 64 * e;
                act[np][e] = r < pl.rows && c < L;
                xv[np][e] = act[np][e] ? __builtin_nontemporal_load(x + r * L + c) : -INFINITY;
                gv[np][e] = act[np][e] ? __builtin_nontemporal_load(dy + r * L + c) : 0.f;
            }
        }
#pragma unroll
        for (int np = 0; np < NP; ++np) {
            const int64_t r = b * pl.Pq + pos[np];
            const bool row_on = r < pl.rows;
            // ---- forward chain
            float mx = xv[np][0];
#pragma unroll
            for (int e = 1; e < EPL; ++e) mx = fmaxf(mx, xv[np][e]);
            mx = sub_max<SUB>(mx);
            float dv[EPL], av[EPL], tv[EPL], ev[EPL], s = 0.f;
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                dv[e] = act[np][e] ? __fsub_rn(mx, xv[np][e]) : 0.f;
                av[e] = q1.fwd(dv[e]);
                tv[e] = expf(__fmul_rn(-av[e], scale));
                ev[e] = act[np][e] ? q2.fwd(tv[e]) : 0.f;
                s += ev[e];
            }
            s = sub_sum<SUB>(s);
            const float sq = q3.fwd(s);
            const float r0 = __fdiv_rn(1.0f, __fadd_rn(sq, eps));
            const float rr = q4.fwd(r0);
            // ---- backward chain
            float g0[EPL], drr = 0.f;
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                const float y0 = __fmul_rn(ev[e], rr);
                float gx = gv[np][e];
                if (qo.present) {
                    float gi, gf;
                    quantize_grad_dyn(y0, gv[np][e], po[np][e], qo.rm, qo.om, gx, gi, gf);
                    if (qo.kbi) gi -= gf;
                    if (act[np][e]) goi[np][e] += gi, gof[np][e] += gf;
                }
                g0[e] = act[np][e] ? gx : 0.f;
                drr += g0[e] * ev[e];
            }
            drr = sub_sum<SUB>(drr);
            float dr0, gi4, gf4, dsq, gi3, gf3, ds;
            q4.grad(r0, drr, dr0, gi4, gf4);
            dsq = dr0 * -(r0 * r0);
            q3.grad(s, dsq, ds, gi3, gf3);
            if (row_on && col == 0) gs[6] += gi4, gs[7] += gf4, gs[4] += gi3, gs[5] += gf3;
            float dd[EPL], dm = 0.f, cnt = 0.f;
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                const float de = g0[e] * rr + ds;
                float dt, gi2, gf2, gi1, gf1;
                q2.grad(tv[e], de, dt, gi2, gf2);
                const float da = -((dt * tv[e]) * scale);
                q1.grad(dv[e], da, dd[e], gi1, gf1);
                if (act[np][e]) {
                    gs[2] += gi2, gs[3] += gf2, gs[0] += gi1, gs[1] += gf1;
                    dm += dd[e];
                    cnt += (xv[np][e] == mx) ? 1.f : 0.f;
                } else {
                    dd[e] = 0.f;
                }
            }
            dm = sub_sum<SUB>(dm);
            cnt = sub_sum<SUB>(cnt);
            const float share = dm / cnt;  // the maximum's gradient is split evenly among ties
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                if (act[np][e]) {
                    const float g = (xv[np][e] == mx) ? share - dd[e] : -dd[e];
                    __builtin_nontemporal_store(g, dx + r * L + col + 64 * e);
                }
            }
        }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const float v = wave_sum(gs[j]);
        if (lane == 0) ws[gw * 8 + j] = v;
    }
    if (qo.present) {
        const int64_t PL = pl.Pq * L;
        float *wi = ws + pl.n_waves() * 8 + chunk * PL;
        float *wf = wi + pl.n_chunks * PL;
#pragma unroll
        for (int np = 0; np < NP; ++np)
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                const int c = col + 64 * e;
                if (c < L) wi[pos[np] * L + c] = goi[np][e], wf[pos[np] * L + c] = gof[np][e];
            }
    }
}

// Fixed-order sums of the backward kernel's slices.
//   block 0: the eight shared-quantizer gradients;  blocks 1..: 64 output-quantizer entries each
__global__ __launch_bounds__(256) void qsoftmax_reduce_kernel(const float *__restrict__ ws, SoftmaxPlan pl, float *g_shared,
                                                              float *g_oi, float *g_of) {
    __shared__ float red[256];
    const int t = threadIdx.x;
    const int64_t nw = pl.n_waves();
    if (blockIdx.x == 0) {
        // thread t sums slice entries j = t % 8 of waves t / 8, t / 8 + 32, ...
        const int j = t & 7;
        float s = 0.f;
        for (int64_t w = t >> 3; w < nw; w += 32) s += ws[w * 8 + j];
        red[t] = s;
        __syncthreads();
        for (int o = 128; o >= 8; o >>= 1) {
            if (t < o) red[t] += red[t + o];
            __syncthreads();
        }
        if (t < 8 && g_shared) g_shared[t] = red[t];
        return;
    }
    if (!g_oi && !g_of) return;
    const int64_t PL = pl.Pq * pl.L, M = pl.P_table * pl.L;
    const int64_t fold = pl.Pq / pl.P_table;  // table rows aliased by several walked rows (shared table)
    const int64_t n_slices = pl.n_chunks * fold;
    const int e_local = t & 63, grp = t >> 6;
    const int64_t e = (int64_t)(blockIdx.x - 1) * 64 + e_local;
    const float *wi = ws + nw * 8, *wf = wi + pl.n_chunks * PL;
    float si = 0.f, sf = 0.f;
    if (e < M) {
        for (int64_t sl = grp; sl < n_slices; sl += 4) {
            const int64_t off = (sl / fold) * PL + (sl % fold) * M + e;
            si += wi[off], sf += wf[off];
        }
    }
    red[t] = si;
    __syncthreads();
    if (grp == 0 && e < M && g_oi) g_oi[e] = (red[e_local] + red[e_local + 64]) + (red[e_local + 128] + red[e_local + 192]);
    __syncthreads();
    red[t] = sf;
    __syncthreads();
    if (grp == 0 && e < M && g_of) g_of[e] = (red[e_local] + red[e_local + 64]) + (red[e_local + 128] + red[e_local + 192]);
}

static int plan_softmax(int64_t rows, int L, int64_t bw_rows, bool has_oq, SoftmaxPlan &pl, const char *who) {
    if (rows < 0 || L < 1) return fail(HGQ_ERR_ARG, "%s: bad sizes", who);
    if (L > 256) return fail(HGQ_ERR_UNSUPPORTED, "%s: rows of up to 256 elements are supported, got %d", who, L);
    int64_t P = has_oq ? bw_rows : 1;
    if (P < 1 || (rows > 0 && rows % P != 0)) return fail(HGQ_ERR_ARG, "%s: rows=%lld is not a multiple of bw_rows=%lld", who, (long long)rows, (long long)P);
    pl.rows = rows, pl.L = L, pl.P_table = P;
    pl.EPL = L <= 64 ? 1 : (L <= 128 ? 2 : 4);
    pl.SUB = L > 32 ? 64 : (L > 16 ? 32 : 16);
    if (P > 1 && P % (64 / pl.SUB) != 0) pl.SUB = 64;  // table rows do not tile the wavefront: one row per wavefront
    const int rpw = 64 / pl.SUB;
    if (P == 1) {
        pl.NP = 4, pl.Pq = rpw * 4;
    } else {
        pl.NP = (P % (rpw * 4) == 0) ? 4 : 1;
        pl.Pq = P;
    }
    pl.PG = pl.Pq / (rpw * pl.NP);
    pl.n_batches = (rows + pl.Pq - 1) / pl.Pq;
    if (pl.n_batches < 1) pl.n_batches = 1;
    // enough wavefronts to fill the device (256 CUs x 4 SIMDs x ~8), each walking >= 4 batches where possible
    const int64_t target = 8192;
    int64_t chunks = (target + pl.PG - 1) / pl.PG;
    if (chunks > pl.n_batches) chunks = pl.n_batches;
    if (chunks < 1) chunks = 1;
    pl.bpc = (int)((pl.n_batches + chunks - 1) / chunks);
    pl.n_chunks = (pl.n_batches + pl.bpc - 1) / pl.bpc;
    return HGQ_OK;
}

static bool desc_ok(const hgq_qdesc *d) { return d == nullptr || d->k == nullptr || (d->i != nullptr && d->fb != nullptr); }
static hgq_qdesc desc_or_none(const hgq_qdesc *d) {
    hgq_qdesc r;
    r.k = nullptr, r.i = nullptr, r.fb = nullptr, r.mode = 0;
    return d ? *d : r;
}

}  // namespace hgq

using namespace hgq;

#define SM_DISPATCH(PLAN, ...)                                                                      \
    do {                                                                                            \
        const int key = (PLAN).SUB * 100 + (PLAN).EPL * 10 + (PLAN).NP;                             \
        switch (key) {                                                                              \
            case 1611: { constexpr int SUB = 16, EPL = 1, NP = 1; __VA_ARGS__; } break;             \
            case 1614: { constexpr int SUB = 16, EPL = 1, NP = 4; __VA_ARGS__; } break;             \
            case 3211: { constexpr int SUB = 32, EPL = 1, NP = 1; __VA_ARGS__; } break;             \
            case 3214: { constexpr int SUB = 32, EPL = 1, NP = 4; __VA_ARGS__; } break;             \
            case 6411: { constexpr int SUB = 64, EPL = 1, NP = 1; __VA_ARGS__; } break;             \
            case 6414: { constexpr int SUB = 64, EPL = 1, NP = 4; __VA_ARGS__; } break;             \
            case 6421: { constexpr int SUB = 64, EPL = 2, NP = 1; __VA_ARGS__; } break;             \
            case 6424: { constexpr int SUB = 64, EPL = 2, NP = 4; __VA_ARGS__; } break;             \
            case 6441: { constexpr int SUB = 64, EPL = 4, NP = 1; __VA_ARGS__; } break;             \
            case 6444: { constexpr int SUB = 64, EPL = 4, NP = 4; __VA_ARGS__; } break;             \
            default: return fail(HGQ_ERR_UNSUPPORTED, "softmax: no kernel for this row layout");    \
        }                                                                                           \
    } while (0)

extern "C" int hgq_qsoftmax_fwd(const float *x, float *y, int64_t rows, int L, int64_t bw_rows, float input_scaler,
                                float eps, const hgq_qdesc *exp_iq, const hgq_qdesc *exp_oq, const hgq_qdesc *inv_iq,
                                const hgq_qdesc *inv_oq, const hgq_qdesc *oq, uint32_t *amax_exp_iq, uint32_t *amax_inv_iq,
                                uint32_t *amax_oq, void *stream) {
    hipStream_t s = (hipStream_t)stream;
    const bool has_oq = oq && oq->k;
    SoftmaxPlan pl;
    int rc = plan_softmax(rows, L, bw_rows, has_oq, pl, "hgq_qsoftmax_fwd");
    if (rc) return rc;
    if (rows == 0) return HGQ_OK;
    if (!x || !y) return fail(HGQ_ERR_ARG, "hgq_qsoftmax_fwd: null pointer");
    if (!desc_ok(exp_iq) || !desc_ok(exp_oq) || !desc_ok(inv_iq) || !desc_ok(inv_oq) || !desc_ok(oq))
        return fail(HGQ_ERR_ARG, "hgq_qsoftmax_fwd: a quantizer descriptor has k but not i / fb");
    if (amax_oq && !has_oq) return fail(HGQ_ERR_ARG, "hgq_qsoftmax_fwd: amax_oq without an output quantizer");
    if (amax_exp_iq && (rc = fill_u32(amax_exp_iq, 0, 1, s))) return rc;
    if (amax_inv_iq && (rc = fill_u32(amax_inv_iq, 0, 1, s))) return rc;
    if (amax_oq && (rc = fill_u32(amax_oq, 0, pl.P_table * L, s))) return rc;
    const unsigned grid = (unsigned)((pl.n_waves() + SM_WAVES_PER_BLOCK - 1) / SM_WAVES_PER_BLOCK);
    SM_DISPATCH(pl, hipLaunchKernelGGL((qsoftmax_fwd_kernel<SUB, EPL, NP>), dim3(grid), dim3(64 * SM_WAVES_PER_BLOCK), 0, s, x, y, pl,
                                       input_scaler, eps, desc_or_none(exp_iq), desc_or_none(exp_oq), desc_or_none(inv_iq),
                                       desc_or_none(inv_oq), desc_or_none(oq), amax_exp_iq, amax_inv_iq, amax_oq));
    return check_launch("hgq_qsoftmax_fwd");
}

extern "C" int64_t hgq_qsoftmax_bwd_workspace(int64_t rows, int L, int64_t bw_rows, int has_oq) {
    SoftmaxPlan pl;
    if (plan_softmax(rows, L, bw_rows, has_oq != 0, pl, "hgq_qsoftmax_bwd_workspace")) return -1;
    return pl.n_waves() * 8 + (has_oq ? 2 * pl.n_chunks * pl.Pq * L : 0);
}

extern "C" int hgq_qsoftmax_bwd(const float *dy, const float *x, float *dx, int64_t rows, int L, int64_t bw_rows,
                                float input_scaler, float eps, const hgq_qdesc *exp_iq, const hgq_qdesc *exp_oq,
                                const hgq_qdesc *inv_iq, const hgq_qdesc *inv_oq, const hgq_qdesc *oq, float *g_shared,
                                float *g_oq_i, float *g_oq_fb, float *workspace, void *stream) {
    hipStream_t s = (hipStream_t)stream;
    const bool has_oq = oq && oq->k;
    SoftmaxPlan pl;
    int rc = plan_softmax(rows, L, bw_rows, has_oq, pl, "hgq_qsoftmax_bwd");
    if (rc) return rc;
    if (!desc_ok(exp_iq) || !desc_ok(exp_oq) || !desc_ok(inv_iq) || !desc_ok(inv_oq) || !desc_ok(oq))
        return fail(HGQ_ERR_ARG, "hgq_qsoftmax_bwd: a quantizer descriptor has k but not i / fb");
    const hgq_qdesc *all[5] = {exp_iq, exp_oq, inv_iq, inv_oq, oq};
    for (const hgq_qdesc *d : all)
        if (d && d->k && !(d->mode & HGQ_MODE_TRAINING))
            return fail(HGQ_ERR_ARG, "hgq_qsoftmax_bwd: the surrogate gradient is defined for training mode only");
    if (rows == 0) {
        if (g_shared && (rc = fill_f32(g_shared, 0.f, 8, s))) return rc;
        if (has_oq && g_oq_i && (rc = fill_f32(g_oq_i, 0.f, pl.P_table * L, s))) return rc;
        if (has_oq && g_oq_fb && (rc = fill_f32(g_oq_fb, 0.f, pl.P_table * L, s))) return rc;
        return HGQ_OK;
    }
    if (!dy || !x || !dx || !workspace) return fail(HGQ_ERR_ARG, "hgq_qsoftmax_bwd: null pointer");
    const unsigned grid = (unsigned)((pl.n_waves() + SM_WAVES_PER_BLOCK - 1) / SM_WAVES_PER_BLOCK);
    SM_DISPATCH(pl, hipLaunchKernelGGL((qsoftmax_bwd_kernel<SUB, EPL, NP>), dim3(grid), dim3(64 * SM_WAVES_PER_BLOCK), 0, s, dy, x, dx,
                                       pl, input_scaler, eps, desc_or_none(exp_iq), desc_or_none(exp_oq), desc_or_none(inv_iq),
                                       desc_or_none(inv_oq), desc_or_none(oq), workspace));
    if ((rc = check_launch("hgq_qsoftmax_bwd"))) return rc;
    const unsigned rgrid = 1 + (has_oq ? (unsigned)((pl.P_table * L + 63) / 64) : 0);
    hipLaunchKernelGGL(qsoftmax_reduce_kernel, dim3(rgrid), dim3(256), 0, s, workspace, pl, g_shared, has_oq ? g_oq_i : nullptr,
                       has_oq ? g_oq_fb : nullptr);
    return check_launch("hgq_qsoftmax_bwd(reduce)");
}
