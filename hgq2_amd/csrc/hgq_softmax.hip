// Table-driven softmax of QSoftmax / QMultiHeadAttention as one pass over the score tensor.
//
//   d = max(x) - x;  e = Q_exp_out(exp(-Q_exp_in(d) * scale));  s = sum(e);
//   r = Q_inv_out(1 / (Q_inv_in(s) + eps));  y = Q_out(e * r)
//
// Layout.  A row (the softmax axis, contiguous, L <= 256 elements) lives in SUB lanes of a
// wavefront, VEC consecutive elements per lane (128-bit accesses when L is a multiple of 4), so a
// wavefront holds 64 / SUB rows side by side and takes NP such groups per step: the row maximum
// and sum are four DPP steps inside a 16-lane row (plus scalar-register reads across rows when a
// row spans several), and the per-row stages (inverse table) are evaluated once for all rows of
// the wavefront.  The four table quantizers have one shared bit-width entry each; the output
// quantizer has a [P, L] table, row r using entry r % P.  A workgroup owns fixed table rows and
// its wavefronts walk along the batch, so the output quantizer's operands, its abs-max tracker
// and its bit-width gradients stay in registers and are combined through LDS once at the end.
#include "hgq_softmax_dev.h"

namespace hgq {

typedef float f32x4 __attribute__((ext_vector_type(4)));
template <int VEC>
__device__ __forceinline__ void row_load(const float *p, float *o) {
    if (VEC == 4) {
        const f32x4 t = __builtin_nontemporal_load((const f32x4 *)p);
        o[0] = t.x, o[1] = t.y, o[2] = t.z, o[3] = t.w;
    } else {
        o[0] = __builtin_nontemporal_load(p);
    }
}
template <int VEC>
__device__ __forceinline__ void row_store(float *p, const float *o) {
    if (VEC == 4) {
        f32x4 t;
        t.x = o[0], t.y = o[1], t.z = o[2], t.w = o[3];
        __builtin_nontemporal_store(t, (f32x4 *)p);
    } else {
        __builtin_nontemporal_store(o[0], p);
    }
}


// Per-wavefront constants of the walk.
template <int SUB, int VEC, int NP>
struct Walk {
    static constexpr int RPW = 64 / SUB;
    int lane, col;
    bool col_on;
    int nb;           // steps of this wavefront
    int64_t stride;   // elements between consecutive steps
    int64_t off[NP];  // element offset of this lane's first element at step 0
    int tcol[NP];     // offset into the output quantizer's table
    int wcol[NP];     // offset into a [Pq, L] slice
    int blim[NP];     // number of steps whose row exists
    __device__ __forceinline__ void init(const SoftmaxPlan &pl) {
        const int wave = threadIdx.x >> 6;
        lane = threadIdx.x & 63;
        const int slot = lane / SUB;
        col = (lane % SUB) * VEC;
        col_on = col < pl.L;
        const int64_t pg = blockIdx.x % pl.PG, chunk = blockIdx.x / pl.PG;
        const int64_t b0 = chunk * pl.bpc + wave, b1 = min(pl.n_batches, chunk * pl.bpc + pl.bpc);
        nb = b0 < b1 ? (int)((b1 - b0 + SM_WPB - 1) / SM_WPB) : 0;
        stride = (int64_t)SM_WPB * pl.Pq * pl.L;
#pragma unroll
        for (int np = 0; np < NP; ++np) {
            const int64_t pos = (pg * NP + np) * RPW + slot;
            const int64_t first = b0 * pl.Pq + pos;
            off[np] = first * pl.L + col;
            tcol[np] = (int)((pos % pl.P_table) * pl.L) + col;
            wcol[np] = (int)(pos * pl.L) + col;
            const int64_t step_rows = (int64_t)SM_WPB * pl.Pq;
            const int64_t left = first < pl.rows ? (pl.rows - first + step_rows - 1) / step_rows : 0;
            blim[np] = (int)min((int64_t)nb, left);
        }
    }
};

template <int SUB, int VEC, int NP, bool TRAIN>
__global__ __launch_bounds__(64 * SM_WPB) void qsoftmax_fwd_kernel(
    const float *__restrict__ x, float *__restrict__ y, SoftmaxPlan pl, float scale, float eps, hgq_qdesc d1, hgq_qdesc d2,
    hgq_qdesc d3, hgq_qdesc d4, hgq_qdesc dq, uint32_t *amax1, uint32_t *amax3, uint32_t *amax_o) {
    __shared__ uint32_t lds_max[SM_WPB][NP * VEC][64];
    __shared__ uint32_t lds_m13[SM_WPB][2];
    __shared__ float lds_tab_e[SM_TABLE];
    Walk<SUB, VEC, NP> wk;
    wk.init(pl);
    SharedQ q1, q2, q3, q4;
    q1.init(d1), q2.init(d2), q3.init(d3), q4.init(d4);
    LaneQ qo;
    qo.init(dq);
    int po[NP][VEC];
    uint32_t mo[NP][VEC];
#pragma unroll
    for (int np = 0; np < NP; ++np)
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            mo[np][e] = 0, po[np][e] = 0;
            if (qo.present && wk.col_on) po[np][e] = qo.load(dq, wk.tcol[np] + e);
        }
    ExpTable tab;
    tab.on = false;
    if (TRAIN) tab.build_fwd(lds_tab_e, q1, q2, scale);
    uint32_t m1 = 0, m3 = 0;
    for (int b = 0; b < wk.nb; ++b) {
        float xv[NP][VEC];
        bool act[NP];
#pragma unroll
        for (int np = 0; np < NP; ++np) {
            act[np] = b < wk.blim[np] && wk.col_on;
#pragma unroll
            for (int e = 0; e < VEC; ++e) xv[np][e] = -INFINITY;
            if (act[np]) row_load<VEC>(x + wk.off[np], xv[np]);
        }
#pragma unroll
        for (int np = 0; np < NP; ++np) {
            float mx = xv[np][0];
#pragma unroll
            for (int e = 1; e < VEC; ++e) mx = fmaxf(mx, xv[np][e]);
            mx = sub_max<SUB>(mx);
            float ev[VEC], s = 0.f;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const float d = act[np] ? __fsub_rn(mx, xv[np][e]) : 0.f;
                float a, ee;
                if (TRAIN && tab.on) {
                    tab.eval_fwd(lds_tab_e, d, q1, q2, scale, a, ee);
                } else {
                    a = q1.fwd<TRAIN>(d);
                    ee = q2.fwd<TRAIN>(ExpTable::t_of(a, scale));
                }
                ev[e] = act[np] ? ee : 0.f;
                m1 = max(m1, abs_bits(a));
                s += ev[e];
            }
            s = sub_sum<SUB>(s);
            const float sq = q3.fwd<TRAIN>(s);
            const float rr = q4.fwd<TRAIN>(__fdiv_rn(1.0f, __fadd_rn(sq, eps)));
            if (b < wk.blim[np]) m3 = max(m3, abs_bits(sq));
            float yv[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                yv[e] = __fmul_rn(ev[e], rr);
                if (qo.present) yv[e] = qo.fwd<TRAIN>(yv[e], po[np][e]);
                if (act[np]) mo[np][e] = max(mo[np][e], abs_bits(yv[e]));
            }
            if (act[np]) row_store<VEC>(y + wk.off[np], yv);
            wk.off[np] += wk.stride;
        }
    }
    // combine the trackers of the workgroup's wavefronts, then one atomic per entry
    const int wave = threadIdx.x >> 6;
    if (amax1 || amax3) {
        m1 = wave_max_bits(m1), m3 = wave_max_bits(m3);
        if (wk.lane == 0) lds_m13[wave][0] = m1, lds_m13[wave][1] = m3;
    }
    if (amax_o) {
#pragma unroll
        for (int np = 0; np < NP; ++np)
#pragma unroll
            for (int e = 0; e < VEC; ++e) lds_max[wave][np * VEC + e][wk.lane] = mo[np][e];
    }
    __syncthreads();
    if (threadIdx.x < 2 && (amax1 || amax3)) {
        uint32_t m = 0;
        for (int w = 0; w < SM_WPB; ++w) m = max(m, lds_m13[w][threadIdx.x]);
        uint32_t *dst = threadIdx.x == 0 ? amax1 : amax3;
        if (dst) atomicMax(dst, m);
    }
    if (amax_o && wave == 0 && wk.col_on) {
#pragma unroll
        for (int np = 0; np < NP; ++np)
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                uint32_t m = 0;
                for (int w = 0; w < SM_WPB; ++w) m = max(m, lds_max[w][np * VEC + e][wk.lane]);
                if (m) atomicMax(&amax_o[wk.tcol[np] + e], m);
            }
    }
}

// Backward: recomputes the forward chain from x, then walks it in reverse.  Partial sums of the
// bit-width gradients go to workspace slices that a second kernel adds up in a fixed order.
//   workspace = [n_blocks, 8] shared-quantizer slices | [n_chunks, Pq * L] d/df of Q_out | [n_chunks, Pq * L] d/di of Q_out
// OQ_GI: the output quantizer saturates, so its integer bits take gradient (else that slice is not written).
template <int SUB, int VEC, int NP, bool OQ_GI>
__global__ __launch_bounds__(64 * SM_WPB) void qsoftmax_bwd_kernel(
    const float *__restrict__ dy, const float *__restrict__ x, float *__restrict__ dx, SoftmaxPlan pl, float scale,
    float eps, hgq_qdesc d1, hgq_qdesc d2, hgq_qdesc d3, hgq_qdesc d4, hgq_qdesc dq, float *__restrict__ ws) {
    __shared__ float lds_g[SM_WPB][NP * VEC][64];
    __shared__ float part[SM_WPB][8];
    __shared__ float lds_tab[4 * SM_TABLE];
    Walk<SUB, VEC, NP> wk;
    wk.init(pl);
    SharedQ q1, q2, q3, q4;
    q1.init(d1), q2.init(d2), q3.init(d3), q4.init(d4);
    LaneQ qo;
    qo.init(dq);
    int po[NP][VEC];
    float gof[NP][VEC], goi[OQ_GI ? NP : 1][VEC];
#pragma unroll
    for (int np = 0; np < NP; ++np)
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            gof[np][e] = 0.f, po[np][e] = 0;
            if (OQ_GI) goi[np][e] = 0.f;
            if (qo.present && wk.col_on) po[np][e] = qo.load(dq, wk.tcol[np] + e);
        }
    float gs[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) gs[j] = 0.f;
    const bool row_lead = wk.col == 0;
    ExpTable tab;
    tab.build_bwd(lds_tab, q1, q2, scale);
    for (int b = 0; b < wk.nb; ++b) {
        float xv[NP][VEC], gv[NP][VEC];
        bool act[NP];
#pragma unroll
        for (int np = 0; np < NP; ++np) {
            act[np] = b < wk.blim[np] && wk.col_on;
#pragma unroll
            for (int e = 0; e < VEC; ++e) xv[np][e] = -INFINITY, gv[np][e] = 0.f;
            if (act[np]) {
                row_load<VEC>(x + wk.off[np], xv[np]);
                row_load<VEC>(dy + wk.off[np], gv[np]);
            }
        }
#pragma unroll
        for (int np = 0; np < NP; ++np) {
            // ---- forward chain
            float mx = xv[np][0];
#pragma unroll
            for (int e = 1; e < VEC; ++e) mx = fmaxf(mx, xv[np][e]);
            mx = sub_max<SUB>(mx);
            float dv[VEC], rv[VEC], ev[VEC], s = 0.f;
            ExpTable::Entry en[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                dv[e] = act[np] ? __fsub_rn(mx, xv[np][e]) : 0.f;
                if (tab.on) {
                    en[e] = tab.eval_bwd(lds_tab, dv[e], q1, q2, scale, rv[e]);
                } else {
                    rv[e] = 0.f;
                    en[e] = ExpTable::entry_of(q1.fwd(dv[e]), q2, scale);
                }
                ev[e] = act[np] ? en[e].e : 0.f;
                s += ev[e];
            }
            s = sub_sum<SUB>(s);
            const float sq = q3.fwd(s);
            const float r0 = __fdiv_rn(1.0f, __fadd_rn(sq, eps));
            const float rr = q4.fwd(r0);
            // ---- backward chain
            float g0[VEC], drr = 0.f;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                float gx = gv[np][e];
                if (qo.present) {
                    float gi, gf;
                    qo.grad(__fmul_rn(ev[e], rr), gv[np][e], po[np][e], gx, gi, gf);
                    gof[np][e] += gf;  // dy is zero on inactive lanes
                    if (OQ_GI) goi[np][e] += gi;
                }
                g0[e] = gx;
                drr += g0[e] * ev[e];
            }
            drr = sub_sum<SUB>(drr);
            float dr0, gi4, gf4, ds, gi3, gf3;
            q4.grad(r0, drr, dr0, gi4, gf4);
            q3.grad(s, dr0 * -(r0 * r0), ds, gi3, gf3);
            if (b < wk.blim[np] && row_lead) gs[6] += gi4, gs[7] += gf4, gs[4] += gi3, gs[5] += gf3;
            float dd[VEC], dm = 0.f, cnt = 0.f;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const float de = g0[e] * rr + ds;
                const float gi2 = en[e].ci * de, gf2 = en[e].cf * de, da = en[e].ca * de;
                float gi1, gf1;
                if (tab.on)
                    tab.grad_q1(dv[e], rv[e], da, q1, dd[e], gi1, gf1);
                else
                    q1.grad(dv[e], da, dd[e], gi1, gf1);
                if (act[np]) {
                    gs[2] += gi2, gs[3] += gf2, gs[0] += gi1, gs[1] += gf1;
                    dm += dd[e];
                    cnt += (xv[np][e] == mx) ? 1.f : 0.f;
                }
            }
            dm = sub_sum<SUB>(dm);
            cnt = sub_sum<SUB>(cnt);
            const float share = dm / cnt;  // the maximum's gradient is split evenly among ties
            float ov[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) ov[e] = (xv[np][e] == mx) ? share - dd[e] : -dd[e];
            if (act[np]) row_store<VEC>(dx + wk.off[np], ov);
            wk.off[np] += wk.stride;
        }
    }
    // shared-quantizer gradients: wavefront sums, then the workgroup's in a fixed order
    const int wave = threadIdx.x >> 6;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const float v = wave_sum(gs[j]);
        if (wk.lane == 0) part[wave][j] = v;
    }
    if (qo.present) {
#pragma unroll
        for (int np = 0; np < NP; ++np)
#pragma unroll
            for (int e = 0; e < VEC; ++e) lds_g[wave][np * VEC + e][wk.lane] = gof[np][e];
    }
    __syncthreads();
    if (threadIdx.x < 8) {
        float s = 0.f;
        for (int w = 0; w < SM_WPB; ++w) s += part[w][threadIdx.x];
        ws[(int64_t)blockIdx.x * 8 + threadIdx.x] = s;
    }
    if (!qo.present) return;
    const int64_t PL = pl.Pq * pl.L;
    const int64_t chunk = blockIdx.x / pl.PG;
    float *wf = ws + pl.n_blocks() * 8 + chunk * PL;
    if (wave == 0 && wk.col_on) {
#pragma unroll
        for (int np = 0; np < NP; ++np)
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                float s = 0.f;
                for (int w = 0; w < SM_WPB; ++w) s += lds_g[w][np * VEC + e][wk.lane];
                wf[wk.wcol[np] + e] = s;
            }
    }
    if (OQ_GI) {
        __syncthreads();
#pragma unroll
        for (int np = 0; np < NP; ++np)
#pragma unroll
            for (int e = 0; e < VEC; ++e) lds_g[wave][np * VEC + e][wk.lane] = goi[np][e];
        __syncthreads();
        float *wi = wf + pl.n_chunks * PL;
        if (wave == 0 && wk.col_on) {
#pragma unroll
            for (int np = 0; np < NP; ++np)
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    float s = 0.f;
                    for (int w = 0; w < SM_WPB; ++w) s += lds_g[w][np * VEC + e][wk.lane];
                    wi[wk.wcol[np] + e] = s;
                }
        }
    }
}

// Fixed-order sums of the backward kernel's slices.
//   block 0: the eight shared-quantizer gradients;  blocks 1..: 64 output-quantizer entries each
__global__ __launch_bounds__(1024) void qsoftmax_reduce_kernel(const float *__restrict__ ws, SoftmaxPlan pl, float *g_shared,
                                                               float *g_oi, float *g_of, int oq_gi) {
    __shared__ float red[1024];
    const int t = threadIdx.x;
    const int64_t nblk = pl.n_blocks();
    if (blockIdx.x == 0) {
        // thread t sums entry j = t % 8 of slices t / 8, t / 8 + 128, ...; eight loads in flight
        const int j = t & 7;
        float s = 0.f;
        int64_t w = t >> 3;
        for (; w + 7 * 128 < nblk; w += 8 * 128) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = ws[(w + u * 128) * 8 + j];
            s += ((v[0] + v[1]) + (v[2] + v[3])) + ((v[4] + v[5]) + (v[6] + v[7]));
        }
        for (; w < nblk; w += 128) s += ws[w * 8 + j];
        red[t] = s;
        __syncthreads();
        for (int o = 512; o >= 8; o >>= 1) {
            if (t < o) red[t] += red[t + o];
            __syncthreads();
        }
        if (t < 8 && g_shared) g_shared[t] = red[t];
        return;
    }
    const int64_t PL = pl.Pq * pl.L, M = pl.P_table * pl.L;
    const int64_t fold = pl.Pq / pl.P_table;  // walked rows that alias one table row (shared table)
    const int64_t n_slices = pl.n_chunks * fold;
    const int e_local = t & 63, grp = t >> 6;  // 16 slice groups x 64 entries
    const int64_t e = (int64_t)(blockIdx.x - 1) * 64 + e_local;
    const float *wf = ws + nblk * 8, *wi = wf + pl.n_chunks * PL;
    float si = 0.f, sf = 0.f;
    if (e < M) {
        // eight loads in flight per thread; the order of the additions is fixed
        int64_t sl = grp;
        for (; sl + 7 * 16 < n_slices; sl += 8 * 16) {
            float vf[8], vi[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int64_t su = sl + u * 16, o = (su / fold) * PL + (su % fold) * M + e;
                vf[u] = wf[o];
                vi[u] = oq_gi ? wi[o] : 0.f;
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) sf += vf[u], si += vi[u];
        }
        for (; sl < n_slices; sl += 16) {
            const int64_t o = (sl / fold) * PL + (sl % fold) * M + e;
            sf += wf[o];
            if (oq_gi) si += wi[o];
        }
    }
    red[t] = sf;
    __syncthreads();
    for (int o = 512; o >= 64; o >>= 1) {
        if (t < o) red[t] += red[t + o];
        __syncthreads();
    }
    if (t < 64 && e < M && g_of) g_of[e] = red[t];
    __syncthreads();
    red[t] = si;
    __syncthreads();
    for (int o = 512; o >= 64; o >>= 1) {
        if (t < o) red[t] += red[t + o];
        __syncthreads();
    }
    if (t < 64 && e < M && g_oi) g_oi[e] = red[t];
}

// Clears up to three tracker arrays in one launch.
__global__ void fill3_u32_kernel(uint32_t *a, int64_t na, uint32_t *b, int64_t nb, uint32_t *c, int64_t nc) {
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < na + nb + nc; t += (int64_t)gridDim.x * blockDim.x) {
        if (t < na) a[t] = 0;
        else if (t < na + nb) b[t - na] = 0;
        else c[t - na - nb] = 0;
    }
}

static int pow2_at_least(int v, int lo) {
    int t = lo;
    while (t < v) t *= 2;
    return t;
}

static int plan_softmax(int64_t rows, int L, int64_t bw_rows, bool has_oq, SoftmaxPlan &pl, const char *who) {
    if (rows < 0 || L < 1) return fail(HGQ_ERR_ARG, "%s: bad sizes", who);
    int64_t P = has_oq ? bw_rows : 1;
    if (P < 1 || (rows > 0 && rows % P != 0))
        return fail(HGQ_ERR_ARG, "%s: rows=%lld is not a multiple of bw_rows=%lld", who, (long long)rows, (long long)P);
    pl.rows = rows, pl.L = L, pl.P_table = P;
    if (L % 4 == 0 && L > 16 && L <= 256) {
        pl.VEC = 4, pl.SUB = pow2_at_least(L / 4, 16);
    } else if (L <= 64) {
        pl.VEC = 1, pl.SUB = pow2_at_least(L, 16);
    } else {
        return fail(HGQ_ERR_UNSUPPORTED, "%s: rows of up to 64 elements, or up to 256 in multiples of 4, are supported, got %d", who, L);
    }
    if (P > 1 && P % (64 / pl.SUB) != 0) {
        // the table rows do not tile the wavefront: fall back to one row per wavefront
        if (pl.VEC == 4 && L > 64)
            return fail(HGQ_ERR_UNSUPPORTED, "%s: bw_rows=%lld must be a multiple of %d for rows of %d elements", who, (long long)P, 64 / pl.SUB, L);
        pl.VEC = 1, pl.SUB = 64;
    }
    const int rpw = 64 / pl.SUB;
    // four row groups per step give a one-element-per-lane wavefront independent work; with four
    // elements per lane that is already there and more would only cost registers
    if (P == 1) {
        pl.NP = pl.VEC == 1 ? 4 : 1, pl.Pq = rpw * pl.NP;
    } else {
        pl.NP = (pl.VEC == 1 && P % (rpw * 4) == 0) ? 4 : 1;
        pl.Pq = P;
    }
    pl.PG = pl.Pq / (rpw * pl.NP);
    pl.n_batches = (rows + pl.Pq - 1) / pl.Pq;
    if (pl.n_batches < 1) pl.n_batches = 1;
    // about 1024 workgroups of 8 wavefronts fill the device; a wavefront should walk >= 4 steps
    const int64_t target = 1024;
    int64_t chunks = (target + pl.PG - 1) / pl.PG;
    const int64_t max_chunks = (pl.n_batches + SM_WPB * 4 - 1) / (SM_WPB * 4);
    if (chunks > max_chunks) chunks = max_chunks;
    if (chunks < 1) chunks = 1;
    pl.bpc = (int)((pl.n_batches + chunks - 1) / chunks);
    pl.n_chunks = (pl.n_batches + pl.bpc - 1) / pl.bpc;
    return HGQ_OK;
}

static bool desc_ok(const hgq_qdesc *d) { return softmax_desc_ok(d); }
static hgq_qdesc desc_or_none(const hgq_qdesc *d) { return softmax_desc_or_none(d); }
static bool aligned16(const void *p) { return ((uintptr_t)p & 15u) == 0; }

int softmax_clear_trackers(uint32_t *a, int64_t na, uint32_t *b, int64_t nb, uint32_t *c, int64_t nc, hipStream_t s) {
    if (!a) na = 0;
    if (!b) nb = 0;
    if (!c) nc = 0;
    if (na + nb + nc == 0) return HGQ_OK;
    const int grid = (int)min((int64_t)1024, (na + nb + nc + 255) / 256);
    hipLaunchKernelGGL(fill3_u32_kernel, dim3(grid), dim3(256), 0, s, a, na, b, nb, c, nc);
    return check_launch("softmax(clear trackers)");
}

int softmax_reduce_slices(const float *ws, const SoftmaxPlan &pl, float *g_shared, float *g_oi, float *g_of, bool has_oq, bool oq_gi,
                          hipStream_t s) {
    const unsigned rgrid = 1 + (has_oq ? (unsigned)((pl.P_table * pl.L + 63) / 64) : 0);
    hipLaunchKernelGGL(qsoftmax_reduce_kernel, dim3(rgrid), dim3(1024), 0, s, ws, pl, g_shared, has_oq ? g_oi : nullptr,
                       has_oq ? g_of : nullptr, (int)oq_gi);
    return check_launch("softmax(reduce slices)");
}

}  // namespace hgq

using namespace hgq;

#define SM_DISPATCH(PLAN, ...)                                                                      \
    do {                                                                                            \
        const int key = (PLAN).SUB * 100 + (PLAN).VEC * 10 + (PLAN).NP;                             \
        switch (key) {                                                                              \
            case 1611: { constexpr int SUB = 16, VEC = 1, NP = 1; __VA_ARGS__; } break;             \
            case 1614: { constexpr int SUB = 16, VEC = 1, NP = 4; __VA_ARGS__; } break;             \
            case 3211: { constexpr int SUB = 32, VEC = 1, NP = 1; __VA_ARGS__; } break;             \
            case 3214: { constexpr int SUB = 32, VEC = 1, NP = 4; __VA_ARGS__; } break;             \
            case 6411: { constexpr int SUB = 64, VEC = 1, NP = 1; __VA_ARGS__; } break;             \
            case 6414: { constexpr int SUB = 64, VEC = 1, NP = 4; __VA_ARGS__; } break;             \
            case 1641: { constexpr int SUB = 16, VEC = 4, NP = 1; __VA_ARGS__; } break;             \
            case 3241: { constexpr int SUB = 32, VEC = 4, NP = 1; __VA_ARGS__; } break;             \
            case 6441: { constexpr int SUB = 64, VEC = 4, NP = 1; __VA_ARGS__; } break;             \
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
    if (pl.VEC == 4 && !(aligned16(x) && aligned16(y))) return fail(HGQ_ERR_ARG, "hgq_qsoftmax_fwd: x and y must be 16-byte aligned");
    if (!desc_ok(exp_iq) || !desc_ok(exp_oq) || !desc_ok(inv_iq) || !desc_ok(inv_oq) || !desc_ok(oq))
        return fail(HGQ_ERR_ARG, "hgq_qsoftmax_fwd: a quantizer descriptor has k but not i / fb");
    if (amax_oq && !has_oq) return fail(HGQ_ERR_ARG, "hgq_qsoftmax_fwd: amax_oq without an output quantizer");
    if (amax_exp_iq || amax_inv_iq || amax_oq) {
        const int64_t n_o = amax_oq ? pl.P_table * L : 0;
        const int grid = (int)min((int64_t)1024, (n_o + 2 + 255) / 256);
        hipLaunchKernelGGL(fill3_u32_kernel, dim3(grid), dim3(256), 0, s, amax_exp_iq, (int64_t)(amax_exp_iq ? 1 : 0), amax_inv_iq,
                           (int64_t)(amax_inv_iq ? 1 : 0), amax_oq, n_o);
        if ((rc = check_launch("hgq_qsoftmax_fwd(clear)"))) return rc;
    }
    // a launch whose quantizers are all in training mode takes the kernel without the inference-only steps
    bool train = true;
    const hgq_qdesc *all[5] = {exp_iq, exp_oq, inv_iq, inv_oq, oq};
    for (const hgq_qdesc *d : all)
        if (d && d->k && !(d->mode & HGQ_MODE_TRAINING)) train = false;
    if (train)
        SM_DISPATCH(pl, hipLaunchKernelGGL((qsoftmax_fwd_kernel<SUB, VEC, NP, true>), dim3((unsigned)pl.n_blocks()), dim3(64 * SM_WPB), 0, s, x, y,
                                           pl, input_scaler, eps, desc_or_none(exp_iq), desc_or_none(exp_oq), desc_or_none(inv_iq),
                                           desc_or_none(inv_oq), desc_or_none(oq), amax_exp_iq, amax_inv_iq, amax_oq));
    else
        SM_DISPATCH(pl, hipLaunchKernelGGL((qsoftmax_fwd_kernel<SUB, VEC, NP, false>), dim3((unsigned)pl.n_blocks()), dim3(64 * SM_WPB), 0, s, x, y,
                                           pl, input_scaler, eps, desc_or_none(exp_iq), desc_or_none(exp_oq), desc_or_none(inv_iq),
                                           desc_or_none(inv_oq), desc_or_none(oq), amax_exp_iq, amax_inv_iq, amax_oq));
    return check_launch("hgq_qsoftmax_fwd");
}

extern "C" int64_t hgq_qsoftmax_bwd_workspace(int64_t rows, int L, int64_t bw_rows, int has_oq) {
    SoftmaxPlan pl;
    if (plan_softmax(rows, L, bw_rows, has_oq != 0, pl, "hgq_qsoftmax_bwd_workspace")) return -1;
    return pl.n_blocks() * 8 + (has_oq ? 2 * pl.n_chunks * pl.Pq * L : 0);
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
    if (pl.VEC == 4 && !(aligned16(x) && aligned16(dy) && aligned16(dx)))
        return fail(HGQ_ERR_ARG, "hgq_qsoftmax_bwd: dy, x and dx must be 16-byte aligned");
    const bool oq_gi = has_oq && ((oq->mode >> 4) & 0xf) != HGQ_WRAP;
    const unsigned grid = (unsigned)pl.n_blocks();
    if (oq_gi)
        SM_DISPATCH(pl, hipLaunchKernelGGL((qsoftmax_bwd_kernel<SUB, VEC, NP, true>), dim3(grid), dim3(64 * SM_WPB), 0, s, dy, x, dx, pl,
                                           input_scaler, eps, desc_or_none(exp_iq), desc_or_none(exp_oq), desc_or_none(inv_iq),
                                           desc_or_none(inv_oq), desc_or_none(oq), workspace));
    else
        SM_DISPATCH(pl, hipLaunchKernelGGL((qsoftmax_bwd_kernel<SUB, VEC, NP, false>), dim3(grid), dim3(64 * SM_WPB), 0, s, dy, x, dx, pl,
                                           input_scaler, eps, desc_or_none(exp_iq), desc_or_none(exp_oq), desc_or_none(inv_iq),
                                           desc_or_none(inv_oq), desc_or_none(oq), workspace));
    if ((rc = check_launch("hgq_qsoftmax_bwd"))) return rc;
    return softmax_reduce_slices(workspace, pl, g_shared, g_oq_i, g_oq_fb, has_oq, oq_gi, s);
}
