// Device-side pieces of the table softmax shared by the softmax kernels and the fused attention
// kernels: quantizers with wavefront-uniform modes, the exp stage as a lookup table, reductions,
// and the slice layout of the bit-width gradients.
#pragma once
#include <math.h>

#include "hgq_device.h"
#include "hgq_host.h"

namespace hgq {

// A quantizer whose mode is uniform over the wavefront, with every mode except inference-time
// WRAP folded into constants so that the per-element code has no mode branches:
//   rounding  r = conv ? rint(t) : floor(t + rc)     (rc = 0.5 for RND, -0 for TRN)
//   overflow  clamp to [lo, hi]; modes that do not saturate use lo = -inf, hi = +inf
// Arithmetic and operation order are those of quantize<> / quantize_grad<> in hgq_device.h.
struct UniQ {
    bool present, conv, sat, sym, kbi, wrap_inf, training;
    float rc;
    __device__ __forceinline__ void init_mode(const hgq_qdesc &d) {
        present = d.k != nullptr;
        const Mode m(present ? d.mode : 0);
        conv = m.round_mode == HGQ_RND_CONV;
        rc = m.round_mode == HGQ_RND ? 0.5f : -0.0f;
        sat = m.overflow_mode != HGQ_WRAP, sym = m.overflow_mode == HGQ_SAT_SYM;
        kbi = m.kbi, training = m.training;
        wrap_inf = present && !sat && !m.training;
    }
    __device__ __forceinline__ float round_at(float x, int fi) const {
        const float t = ldexpf(x, fi);
        const float r = conv ? rintf(t) : floorf(__fadd_rn(t, rc));
        return ldexpf(r, -fi);
    }
    // two's-complement wrap of an already-rounded value (inference only)
    static __device__ __forceinline__ float wrap(float xq, const KIF &p) {
        int st;
        return overflow<HGQ_WRAP>(xq, p, false, st);
    }
};

// One shared bit-width entry: bounds and their derivatives are wavefront constants.
struct SharedQ : UniQ {
    KIF p;
    int fi;
    float hi, lo, gi_hi, gf_hi, gi_lo, gf_lo;
    bool zero;
    __device__ __forceinline__ void init(const hgq_qdesc &d) {
        init_mode(d);
        p.k = 0.f, p.i = 0.f, p.f = 0.f, fi = 0, zero = false;
        hi = INFINITY, lo = -INFINITY, gi_hi = gf_hi = gi_lo = gf_lo = 0.f;
        if (!present) return;
        const Mode m(d.mode);
        p = resolve_kif(load_k(d.k, 0, m.k_u8), d.i[0], d.fb[0], m.kbi, m.round_params);
        fi = (int)p.f;
        zero = !training && !(p.k + p.i + p.f > 0.0f);
        if (sat) {
            const float eps = pow2(-p.f);
            hi = __fsub_rn(pow2(p.i), eps);
            lo = sym ? -p.k * hi : -p.k * pow2(p.i);
            gi_hi = HGQ_LN2 * pow2(p.i), gf_hi = HGQ_LN2 * eps;
            gi_lo = -p.k * gi_hi, gf_lo = sym ? -p.k * gf_hi : 0.f;
        }
        // the values are the same in every lane: pin them to scalar registers
        fi = __builtin_amdgcn_readfirstlane(fi);
        hi = uniform(hi), lo = uniform(lo), gi_hi = uniform(gi_hi), gf_hi = uniform(gf_hi), gi_lo = uniform(gi_lo), gf_lo = uniform(gf_lo);
        p.k = uniform(p.k), p.i = uniform(p.i), p.f = uniform(p.f);
    }
    static __device__ __forceinline__ float uniform(float v) {
        return __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(v)));
    }
    // TRAIN: every quantizer of the launch is in training mode (no wrap, no zeroing of empty words)
    template <bool TRAIN = true>
    __device__ __forceinline__ float fwd(float x) const {
        if (!present) return x;
        const float xq = round_at(x, fi);
        float y = xq > hi ? hi : (xq < lo ? lo : xq);
        if (!TRAIN) {
            if (wrap_inf) y = wrap(xq, p);
            y = zero ? 0.f : y;
        }
        return y;
    }
    // gradients w.r.t. the input and the two stored variables (i and f, or i and b), training mode
    __device__ __forceinline__ void grad(float x, float dy, float &dx, float &di, float &dfb) const {
        if (!present) {
            dx = dy, di = 0.f, dfb = 0.f;
            return;
        }
        const float xq = round_at(x, fi);
        const bool over = xq > hi, under = xq < lo;
        const float ste_f = -HGQ_LN2 * (xq - x) * dy;
        const float oi = over ? gi_hi * dy : 0.f, of = over ? gf_hi * dy : 0.f;
        const float ui = under ? gi_lo * dy : 0.f, uf = under ? gf_lo * dy : 0.f;
        const bool in = !(over || under);
        dx = in ? dy : 0.f;
        di = oi + ui;
        dfb = in ? ste_f : of + uf;
        if (kbi) di -= dfb;  // f = b - i
    }
};

// The output quantizer: operands differ per lane (packed into one register per element: f in
// bits 0-7, i in bits 8-15, both as signed bytes, k in bit 16), the mode is uniform.
struct LaneQ : UniQ {
    __device__ __forceinline__ void init(const hgq_qdesc &d) { init_mode(d); }
    static __device__ __forceinline__ int clamp8(float v) { return (int)fminf(fmaxf(v, -128.f), 127.f); }
    __device__ __forceinline__ int load(const hgq_qdesc &d, int64_t idx) const {
        const Mode m(d.mode);
        const KIF p = resolve_kif(load_k(d.k, idx, m.k_u8), d.i[idx], d.fb[idx], m.kbi, m.round_params);
        return (clamp8(p.f) & 0xff) | ((clamp8(p.i) & 0xff) << 8) | (p.k != 0.f ? 1 << 16 : 0);
    }
    static __device__ __forceinline__ int f_of(int pk) { return (int)(int8_t)(pk & 0xff); }
    static __device__ __forceinline__ int i_of(int pk) { return (int)(int8_t)((pk >> 8) & 0xff); }
    static __device__ __forceinline__ float k_of(int pk) { return (pk >> 16) & 1 ? 1.f : 0.f; }
    template <bool TRAIN>
    __device__ __forceinline__ float fwd(float x, int pk) const {
        const int fi = f_of(pk);
        const float xq = round_at(x, fi);
        float y = xq;
        if (sat) {
            const float k = k_of(pk), pi = ldexpf(1.0f, i_of(pk));
            const float hi = __fsub_rn(pi, ldexpf(1.0f, -fi));
            const float lo = sym ? -k * hi : -k * pi;
            y = xq > hi ? hi : (xq < lo ? lo : xq);
        } else if (!TRAIN && wrap_inf) {
            KIF p;
            p.k = k_of(pk), p.i = (float)i_of(pk), p.f = (float)fi;
            y = wrap(xq, p);
        }
        if (!TRAIN && !training && !(k_of(pk) + (float)(i_of(pk) + fi) > 0.0f)) y = 0.f;
        return y;
    }
    __device__ __forceinline__ void grad(float x, float dy, int pk, float &dx, float &di, float &dfb) const {
        const int fi = f_of(pk);
        const float xq = round_at(x, fi);
        dx = dy, di = 0.f;
        dfb = -HGQ_LN2 * (xq - x) * dy;
        if (sat) {
            const float k = k_of(pk), eps = ldexpf(1.0f, -fi), pi = ldexpf(1.0f, i_of(pk));
            const float hi = __fsub_rn(pi, eps);
            const float lo = sym ? -k * hi : -k * pi;
            const bool over = xq > hi, under = xq < lo;
            if (over || under) {
                const float gi = HGQ_LN2 * pi * dy, gf = HGQ_LN2 * eps * dy;
                dx = 0.f;
                di = (over ? gi : 0.f) + (under ? -k * gi : 0.f);
                dfb = (over ? gf : 0.f) + ((under && sym) ? -k * gf : 0.f);
            }
        }
        if (kbi) di -= dfb;
    }
};

// The exp stage as the lookup table it stands for.  The rounded, saturated argument of the exp
// quantizer is a small non-negative integer code n (d >= 0), and
//     t(n) = exp(-(n * 2**-f) * scale),   e(n) = Q_exp_oq(t(n))
// are functions of n alone: a workgroup tabulates the first SM_TABLE codes in LDS with the same
// device code that evaluates them directly, so looked-up and computed values are identical;
// codes beyond the table (possible only when the exp input quantizer does not saturate) are
// computed in place.
#define SM_TABLE 1024
struct ExpTable {
    float code_max;  // largest code the input quantizer lets through (+inf without saturation)
    bool on;
    __device__ __forceinline__ void init(const SharedQ &q1) {
        // the table needs d -> code to be monotone from 0: an input quantizer whose upper bound is
        // negative (an empty word) keeps the direct evaluation
        on = q1.present && !(q1.hi < 0.f);
        code_max = INFINITY;
        if (on && q1.sat) code_max = SharedQ::uniform(ldexpf(q1.hi, q1.fi));
    }
    static __device__ __forceinline__ float code_of(float d, const SharedQ &q1) {
        return q1.conv ? rintf(ldexpf(d, q1.fi)) : floorf(__fadd_rn(ldexpf(d, q1.fi), q1.rc));
    }
    static __device__ __forceinline__ float t_of(float a, float scale) { return expf(__fmul_rn(-a, scale)); }

    // forward: tab[n] = e(n)
    __device__ __forceinline__ void build_fwd(float *tab, const SharedQ &q1, const SharedQ &q2, float scale) {
        init(q1);
        if (!on) return;
        for (int n = threadIdx.x; n < SM_TABLE; n += blockDim.x) tab[n] = q2.fwd<true>(t_of(ldexpf((float)n, -q1.fi), scale));
        __syncthreads();
    }
    // d >= 0 -> a = Q_exp_iq(d), e
    __device__ __forceinline__ void eval_fwd(const float *tab, float d, const SharedQ &q1, const SharedQ &q2, float scale,
                                             float &a, float &e) const {
        const float rcl = fminf(code_of(d, q1), code_max);
        a = ldexpf(rcl, -q1.fi);
        const unsigned n = (unsigned)(int)rcl;
        e = n < SM_TABLE ? tab[n] : q2.fwd<true>(t_of(a, scale));
    }

    // backward: entry n = (e, d a / d e-gradient, d i2, d fb2) with
    //   da = -((dt * t) * scale) = ca * de,  gi2 = ci * de,  gf2 = cf * de   for the upstream gradient de of e.
    // In LDS the four fields are four planes of SM_TABLE words (field j of code n at tab[j * SM_TABLE + n]): the lanes of a
    // wavefront look up unrelated codes, and 32-bit reads at unrelated addresses cost a fraction of what 128-bit ones do
    // (the banks serve them a word at a time; a 128-bit read needs four neighbouring banks free at once).
    struct Entry {
        float e, ca, ci, cf;
    };
    static __device__ __forceinline__ Entry entry_at(const float *tab, int n) {
        Entry r;
        r.e = tab[n], r.ca = tab[SM_TABLE + n], r.ci = tab[2 * SM_TABLE + n], r.cf = tab[3 * SM_TABLE + n];
        return r;
    }
    static __device__ __forceinline__ Entry entry_of(float a, const SharedQ &q2, float scale) {
        const float t = t_of(a, scale);
        Entry r;
        r.e = q2.fwd<true>(t);
        float dt;
        q2.grad(t, 1.0f, dt, r.ci, r.cf);
        r.ca = -((dt * t) * scale);
        return r;
    }
    __device__ __forceinline__ void build_bwd(float *tab, const SharedQ &q1, const SharedQ &q2, float scale) {
        init(q1);
        if (!on) return;
        for (int n = threadIdx.x; n < SM_TABLE; n += blockDim.x) {
            const Entry en = entry_of(ldexpf((float)n, -q1.fi), q2, scale);
            tab[n] = en.e, tab[SM_TABLE + n] = en.ca, tab[2 * SM_TABLE + n] = en.ci, tab[3 * SM_TABLE + n] = en.cf;
        }
        __syncthreads();
    }
    // d >= 0 -> r = un-saturated code, entry of the saturated code
    __device__ __forceinline__ Entry eval_bwd(const float *tab, float d, const SharedQ &q1, const SharedQ &q2, float scale,
                                              float &r) const {
        r = code_of(d, q1);
        const float rcl = fminf(r, code_max);
        const unsigned n = (unsigned)(int)rcl;
        if (n < SM_TABLE) return entry_at(tab, (int)n);
        return entry_of(ldexpf(rcl, -q1.fi), q2, scale);
    }
    // gradients of the exp input quantizer from the un-saturated code r (no lower violation: d >= 0 >= lo)
    __device__ __forceinline__ void grad_q1(float d, float r, float da, const SharedQ &q1, float &dd, float &gi, float &gf) const {
        const bool over = r > code_max;
        const float xq = ldexpf(r, -q1.fi);
        dd = over ? 0.f : da;
        gi = over ? q1.gi_hi * da : 0.f;
        gf = over ? q1.gf_hi * da : -HGQ_LN2 * (xq - d) * da;
        if (q1.kbi) gi -= gf;
    }
};

template <int SUB>
__device__ __forceinline__ float sub_max(float v) { return sub_reduce<SUB, OpMax>(v); }
template <int SUB>
__device__ __forceinline__ float sub_sum(float v) { return sub_reduce<SUB, OpAdd>(v); }
__device__ __forceinline__ float wave_sum(float v) { return sub_reduce<64, OpAdd>(v); }
__device__ __forceinline__ uint32_t wave_max_bits(uint32_t v) {
    // non-negative floats order like their bit patterns
    return __float_as_uint(sub_reduce<64, OpMax>(__uint_as_float(v)));
}

#define SM_WPB 8  // wavefronts per workgroup

// Work decomposition shared by the forward and backward kernels.  Workgroup (pg, chunk) owns the
// table rows [pg * RI, (pg + 1) * RI) with RI = NP * 64 / SUB and the batches of its chunk;
// wavefront w of the workgroup takes batches b0 + w, b0 + w + SM_WPB, ...
struct SoftmaxPlan {
    int64_t rows;       // number of softmax rows
    int L;              // row length
    int64_t Pq;         // table rows walked by the grid (a multiple of RI)
    int64_t P_table;    // rows of the output quantizer's bit-width table (1 if shared or absent)
    int64_t n_batches;  // ceil(rows / Pq)
    int64_t PG;         // position groups = Pq / RI
    int bpc;            // batches per chunk
    int64_t n_chunks;
    int SUB, VEC, NP;
    __host__ __device__ int64_t n_blocks() const { return PG * n_chunks; }
};

// Host side (hgq_softmax.hip): clears up to three tracker arrays in one launch; adds up the slices
// a backward kernel left in `ws` ([n_blocks, 8] shared-quantizer sums | [n_chunks, Pq * L] d/df |
// [n_chunks, Pq * L] d/di of the output quantizer) in a fixed order.
int softmax_clear_trackers(uint32_t *a, int64_t na, uint32_t *b, int64_t nb, uint32_t *c, int64_t nc, hipStream_t s);
int softmax_reduce_slices(const float *ws, const SoftmaxPlan &pl, float *g_shared, float *g_oi, float *g_of, bool has_oq, bool oq_gi,
                          hipStream_t s);
inline bool softmax_desc_ok(const hgq_qdesc *d) { return d == nullptr || d->k == nullptr || (d->i != nullptr && d->fb != nullptr); }
inline hgq_qdesc softmax_desc_or_none(const hgq_qdesc *d) {
    hgq_qdesc r;
    r.k = nullptr, r.i = nullptr, r.fb = nullptr, r.mode = 0;
    return d ? *d : r;
}

}  // namespace hgq
