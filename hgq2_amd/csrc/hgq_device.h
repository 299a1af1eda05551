// Device-side core of the fixed-point quantizer, shared by every kernel family.
//
// All arithmetic is the same sequence of IEEE-754 fp32 operations the reference's eager
// Keras path performs (scale by an exact power of two, add 0.5, floor, scale back, compare,
// select), so results are bit-identical to it; powers of two are built from the exponent
// (v_ldexp_f32) and never through exp2f/powf/log2f.
#pragma once

#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>

#include "../../include/hgq_hip.h"

#define HGQ_LN2 0.69314718055994530942f

namespace hgq {

struct Mode {
    int round_mode, overflow_mode;
    bool training, kbi, round_params, k_u8, symmetric, tracing, track_input;
    __host__ __device__ explicit Mode(int m)
        : round_mode(m & 0xf), overflow_mode((m >> 4) & 0xf), training(m & HGQ_MODE_TRAINING),
          kbi(m & HGQ_MODE_KBI), round_params(m & HGQ_MODE_ROUND_PARAMS), k_u8(m & HGQ_MODE_K_U8),
          symmetric(m & HGQ_MODE_SYMMETRIC), tracing(m & HGQ_MODE_TRACING), track_input(m & HGQ_MODE_TRACK_INPUT) {}
};

// 2**e for an integer-valued float e (exact, including subnormal results).
__device__ __forceinline__ float pow2(float e) { return ldexpf(1.0f, (int)e); }

template <int RM>
__device__ __forceinline__ float round_scaled(float t) {
    if (RM == HGQ_TRN) return floorf(t);
    if (RM == HGQ_RND) return floorf(__fadd_rn(t, 0.5f));
    return rintf(t);  // RND_CONV: round half to even
}

// xq = R(x * 2**f) / 2**f.  Scaling by ldexp equals the multiply / divide by the fp32 value
// 2**f wherever that value is finite and the result normal.
template <int RM>
__device__ __forceinline__ float fixed_round(float x, float f) {
    const int fi = (int)f;
    return ldexpf(round_scaled<RM>(ldexpf(x, fi)), -fi);
}

__device__ __forceinline__ float load_k(const void *k, int64_t idx, bool k_u8) {
    return k_u8 ? (float)((const uint8_t *)k)[idx] : ((const float *)k)[idx];
}

// Resolve (k, i, f) of one bit-width entry from the stored operands.
struct KIF {
    float k, i, f;
};

__device__ __forceinline__ KIF resolve_kif(float k, float i, float fb, bool kbi, bool round_params) {
    if (round_params) {
        i = rintf(i);
        fb = rintf(fb);
    }
    KIF r;
    r.k = k;
    r.i = i;
    r.f = kbi ? __fsub_rn(fb, i) : fb;
    return r;
}

// Overflow handling of an already-rounded value.  Returns the output; `state` is 0 inside the
// range, bit 0 set above the upper bound, bit 1 set below the lower bound (SAT modes only).
template <int OM>
__device__ __forceinline__ float overflow(float xq, const KIF &p, bool training, int &state) {
    state = 0;
    if (OM == HGQ_WRAP) {
        if (training) return xq;
        const float bias = p.k * pow2(p.i);
        const float ik = __fadd_rn(p.i, p.k);
        const float m = pow2(ik);
        const float a = __fadd_rn(xq, bias);
        // floor-mod by a power of two: a - floor(a / m) * m is exact
        const float q = floorf(ldexpf(a, -(int)ik));
        return __fsub_rn(__fmaf_rn(-q, m, a), bias);
    }
    const float eps = pow2(-p.f);
    const float hi = __fsub_rn(pow2(p.i), eps);
    const float lo = (OM == HGQ_SAT) ? -p.k * pow2(p.i) : -p.k * hi;
    // both comparisons are evaluated: for an empty word (upper bound below the lower bound) a
    // value can violate both, the upper bound wins in the forward and both bounds take gradient
    const bool over = xq > hi, under = xq < lo;
    state = (over ? 1 : 0) | (under ? 2 : 0);
    return over ? hi : (under ? lo : xq);
}

template <int RM, int OM>
__device__ __forceinline__ float quantize(float x, const KIF &p, bool training) {
    int st;
    float y = overflow<OM>(fixed_round<RM>(x, p.f), p, training, st);
    if (!training && !(p.k + p.i + p.f > 0.0f)) y = 0.0f;
    return y;
}

// Surrogate backward of one element (training mode).  Outputs the gradients w.r.t. x, i, f.
template <int RM, int OM>
__device__ __forceinline__ void quantize_grad(float x, float dy, const KIF &p, float &dx, float &di, float &df) {
    const float xq = fixed_round<RM>(x, p.f);
    int st = 0;
    if (OM != HGQ_WRAP) (void)overflow<OM>(xq, p, true, st);
    if (st == 0) {
        dx = dy;
        di = 0.0f;
        df = -HGQ_LN2 * (xq - x) * dy;
    } else {
        dx = 0.0f;
        const float gi = HGQ_LN2 * pow2(p.i) * dy;
        const float gf = HGQ_LN2 * pow2(-p.f) * dy;
        di = 0.0f, df = 0.0f;
        if (st & 1) {
            di += gi;
            df += gf;
        }
        if (st & 2) {
            di += -p.k * gi;
            if (OM == HGQ_SAT_SYM) df += -p.k * gf;
        }
    }
}

// Training-mode forward and surrogate backward of one element from one rounding: y is what quantize<RM, OM>(x, p, true)
// returns and dx / di / df what quantize_grad<RM, OM> returns, bit for bit (same operations in the same order).
template <int RM, int OM>
__device__ __forceinline__ float quantize_with_grad(float x, float dy, const KIF &p, float &dx, float &di, float &df) {
    const float xq = fixed_round<RM>(x, p.f);
    int st = 0;
    float y = xq;
    if (OM != HGQ_WRAP) y = overflow<OM>(xq, p, true, st);
    if (st == 0) {
        dx = dy;
        di = 0.0f;
        df = -HGQ_LN2 * (xq - x) * dy;
    } else {
        dx = 0.0f;
        const float gi = HGQ_LN2 * pow2(p.i) * dy;
        const float gf = HGQ_LN2 * pow2(-p.f) * dy;
        di = 0.0f, df = 0.0f;
        if (st & 1) {
            di += gi;
            df += gf;
        }
        if (st & 2) {
            di += -p.k * gi;
            if (OM == HGQ_SAT_SYM) df += -p.k * gf;
        }
    }
    return y;
}

// Bit pattern of |v| as an unsigned integer: monotone for non-negative floats, so an integer
// atomic max is a float max.  NaN payloads compare above every finite value and propagate.
__device__ __forceinline__ uint32_t abs_bits(float v) { return __float_as_uint(v) & 0x7fffffffu; }


// Runtime-mode forms (for kernels that serve several quantizers with different modes at once).
// Selects, not branches: the mode is uniform over a launch, but a chain of scalar branches per element costs several
// times the two vector instructions it would save (one floor serves TRN and RND, one pair of scalings all three).
__device__ __forceinline__ float fixed_round_dyn(float x, float f, int rm) {
    const int fi = (int)f;
    const float t = ldexpf(x, fi);
    const float down = floorf(rm == HGQ_RND ? __fadd_rn(t, 0.5f) : t);
    return ldexpf(rm == HGQ_RND_CONV ? rintf(t) : down, -fi);
}

__device__ __forceinline__ float quantize_dyn(float x, const KIF &p, int rm, int om, bool training) {
    const float xq = fixed_round_dyn(x, p.f, rm);
    int st;
    float y = om == HGQ_WRAP ? overflow<HGQ_WRAP>(xq, p, training, st)
              : om == HGQ_SAT ? overflow<HGQ_SAT>(xq, p, training, st) : overflow<HGQ_SAT_SYM>(xq, p, training, st);
    if (!training && !(p.k + p.i + p.f > 0.0f)) y = 0.0f;
    return y;
}

__device__ __forceinline__ void quantize_grad_dyn(float x, float dy, const KIF &p, int rm, int om, float &dx, float &di, float &df) {
#define HGQ_QG(RMV, OMV) quantize_grad<RMV, OMV>(x, dy, p, dx, di, df)
    if (om == HGQ_WRAP) {
        if (rm == HGQ_TRN) HGQ_QG(HGQ_TRN, HGQ_WRAP); else if (rm == HGQ_RND) HGQ_QG(HGQ_RND, HGQ_WRAP); else HGQ_QG(HGQ_RND_CONV, HGQ_WRAP);
    } else if (om == HGQ_SAT) {
        if (rm == HGQ_TRN) HGQ_QG(HGQ_TRN, HGQ_SAT); else if (rm == HGQ_RND) HGQ_QG(HGQ_RND, HGQ_SAT); else HGQ_QG(HGQ_RND_CONV, HGQ_SAT);
    } else {
        if (rm == HGQ_TRN) HGQ_QG(HGQ_TRN, HGQ_SAT_SYM); else if (rm == HGQ_RND) HGQ_QG(HGQ_RND, HGQ_SAT_SYM); else HGQ_QG(HGQ_RND_CONV, HGQ_SAT_SYM);
    }
#undef HGQ_QG
}

// ceil(log2(v)) for v > 0 from the exponent field: exact, where log2f is only faithfully rounded.
__device__ __forceinline__ float ceil_log2_exact(float v) {
    if (!(v > 0.0f)) return v == 0.0f ? -INFINITY : NAN;
    if (!(v < INFINITY)) return v;
    int e;
    const float mant = frexpf(v, &e);  // v = mant * 2**e, mant in [0.5, 1)
    return (float)(mant == 0.5f ? e - 1 : e);
}


// ---- buffer loads ------------------------------------------------------------------------
// The hardware returns 0 for an offset outside the descriptor's range, so a lane that must not
// read passes BUF_OOB instead of branching around the load.  (A load inside a branch - and the
// compiler turns `ok ? load : 0` into one - is waited for where it is issued, which serialises
// the loads of a tile and defeats any prefetch.)  `base` must be wave-uniform; ranges are capped
// at 2 GiB, so callers rebase the descriptor per tile for large tensors.
typedef float f32x4_t __attribute__((ext_vector_type(4)));
#define BUF_OOB 0xfffffff0u
__device__ __forceinline__ __amdgpu_buffer_rsrc_t buf_rsrc(const void *base, int64_t bytes) {
    const int64_t cap = 0x7fffffff;
    return __builtin_amdgcn_make_buffer_rsrc((void *)base, 0, (int)(bytes < 0 ? 0 : (bytes > cap ? cap : bytes)), 0x00020000);
}
__device__ __forceinline__ f32x4_t buf_ld4(__amdgpu_buffer_rsrc_t r, uint32_t byte_off) {
    return __builtin_bit_cast(f32x4_t, __builtin_amdgcn_raw_buffer_load_b128(r, byte_off, 0, 0));
}
__device__ __forceinline__ float buf_ld1(__amdgpu_buffer_rsrc_t r, uint32_t byte_off) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, byte_off, 0, 0));
}

// c / d for c < 2**21 through the float reciprocal: (c + 0.5) / d is at least 0.5 / d away from an integer, more than the
// rounding error of the two float operations below that bound.
struct FastDiv {
    uint32_t d;
    float inv;
    __device__ __forceinline__ explicit FastDiv(uint32_t d_) : d(d_), inv(1.0f / (float)d_) {}
    __device__ __forceinline__ uint32_t div(uint32_t c) const { return (uint32_t)(((float)c + 0.5f) * inv); }
    __device__ __forceinline__ uint32_t mod(uint32_t c) const { return c - div(c) * d; }
};

// Stores through a descriptor: a store at BUF_OOB (or anywhere past the descriptor's range) is dropped.
typedef unsigned int u32x4_raw_t __attribute__((__vector_size__(16)));
__device__ __forceinline__ void buf_st4(__amdgpu_buffer_rsrc_t r, uint32_t byte_off, f32x4_t v) {
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_raw_t, v), r, byte_off, 0, 0);
}
__device__ __forceinline__ void buf_st1(__amdgpu_buffer_rsrc_t r, uint32_t byte_off, float v) {
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned int, v), r, byte_off, 0, 0);
}

// ------------------------------------------------------------------------------------------
// all-reduce over groups of SUB consecutive lanes (SUB = 16, 32 or 64): four DPP steps inside
// each 16-lane row (xor 1, xor 2, half-row mirror, row mirror), then the row totals are read
// back through scalar registers
// ------------------------------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v) {
    return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ float lane_value(float v, int lane) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}
struct OpMax {
    static __device__ __forceinline__ float f(float a, float b) { return fmaxf(a, b); }
};
struct OpAdd {
    static __device__ __forceinline__ float f(float a, float b) { return a + b; }
};
template <int SUB, class Op>
__device__ __forceinline__ float sub_reduce(float v) {
    v = Op::f(v, dpp_mov<0xB1>(v));   // quad_perm [1,0,3,2]
    v = Op::f(v, dpp_mov<0x4E>(v));   // quad_perm [2,3,0,1]
    v = Op::f(v, dpp_mov<0x141>(v));  // row_half_mirror
    v = Op::f(v, dpp_mov<0x140>(v));  // row_mirror
    if (SUB == 16) return v;
    const float r0 = lane_value(v, 0), r1 = lane_value(v, 16), r2 = lane_value(v, 32), r3 = lane_value(v, 48);
    const float a = Op::f(r0, r1), b = Op::f(r2, r3);
    if (SUB == 32) return (threadIdx.x & 32) ? b : a;
    return Op::f(a, b);
}
template <int SUB>
__device__ __forceinline__ float row_reduce_sum(float v) { return sub_reduce<SUB, OpAdd>(v); }
template <int SUB>
__device__ __forceinline__ float row_reduce_max(float v) { return sub_reduce<SUB, OpMax>(v); }

typedef float floatx16 __attribute__((ext_vector_type(16)));

// acc += sum over 16 * n_batches contraction steps of A * B on the matrix cores, A at ap[k * sa],
// B at bp[k * sb] (k even; the lane's k parity is already folded into ap / bp).  The sixteen LDS
// operands of a batch of eight instructions are read together, and the next batch's reads are
// issued before the current batch's instructions, so a workgroup that is alone on its CU pays one
// LDS latency per chain instead of one per instruction.  n_batches <= 4 (contractions up to 64); longer ones chain several calls.
__device__ __forceinline__ floatx16 mfma_chain(floatx16 acc, const float *ap, int sa, const float *bp, int sb, int n_batches) {
    float a[8], b[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) a[u] = ap[2 * u * sa], b[u] = bp[2 * u * sb];
#pragma unroll
    for (int bt = 0; bt < 4; ++bt) {
        if (bt < n_batches) {
            float an[8], bn[8];
            if (bt + 1 < n_batches) {
#pragma unroll
                for (int u = 0; u < 8; ++u) an[u] = ap[(16 * (bt + 1) + 2 * u) * sa], bn[u] = bp[(16 * (bt + 1) + 2 * u) * sb];
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u], b[u], acc, 0, 0, 0);
            if (bt + 1 < n_batches) {
#pragma unroll
                for (int u = 0; u < 8; ++u) a[u] = an[u], b[u] = bn[u];
            }
        }
    }
    return acc;
}

// ------------------------------------------------------------------------------------------
// The same chain on the bf16 matrix cores, exactly.  An fp32 number is the sum of three numbers of eight significant
// bits each - its leading bits, the leading bits of what is left, and the rest - and each is a bf16 number (same
// exponent range).  A product of two parts is exact in fp32, so the sum over part pairs of A_p B_q, accumulated in fp32,
// is the contraction with only the accumulation rounded, as in the fp32 instruction.  v_mfma_f32_32x32x16_bf16 takes the
// sixteen contraction steps of a batch in one instruction of half the issue time of ONE fp32 instruction: one to nine
// instructions replace eight.  Quantized operands rarely need more than one part (eight bits) or two (sixteen): a
// wavefront looks at the operands it has just read and multiplies the non-zero parts only (uniform branches).
// Operand layout (64 lanes, eight bf16 per lane): A[i][k]: i = lane % 32, k = 8 (lane / 32) + e; B[k][j] likewise; the
// sum does not depend on which contraction step sits where, so element e of lane half h is step 2 e + h of the batch -
// the LDS reads are those of the fp32 chain.
// ------------------------------------------------------------------------------------------
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

// the three parts of v as fp32 bit patterns whose low halves are zero (a part that is not needed is zero)
__device__ __forceinline__ void bf16_parts(float v, uint32_t &h, uint32_t &m, uint32_t &l) {
    h = __float_as_uint(v) & 0xffff0000u;
    const float r1 = __fsub_rn(v, __uint_as_float(h));  // exact: the low 16 bits of the significand
    m = __float_as_uint(r1) & 0xffff0000u;
    l = __float_as_uint(__fsub_rn(r1, __uint_as_float(m)));  // exact, at most eight significant bits
}
// the high halves of two words as one register of two bf16, `a` first (one byte-permute instruction)
__device__ __forceinline__ uint32_t bf16_pair(uint32_t a, uint32_t b) { return __builtin_amdgcn_perm(b, a, 0x07060302u); }

__device__ __forceinline__ floatx16 mfma_bf16(const u32x4_t &a, const u32x4_t &b, floatx16 acc) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), acc, 0, 0, 0);
}

// The leading parts of eight fp32 operands of a lane (the high halves of the words) and whether that is all of them for
// every lane of the wavefront that counts (`counts` = false: a lane that feeds padding rows, whatever it read).
__device__ __forceinline__ bool bf16_lead8(const float (&v)[8], u32x4_t &p0, bool counts = true) {
    uint32_t low = 0u;
#pragma unroll
    for (int e = 0; e < 8; e += 2) {
        p0[e >> 1] = __builtin_amdgcn_perm(__float_as_uint(v[e + 1]), __float_as_uint(v[e]), 0x07060302u);
        low |= __float_as_uint(v[e]) | __float_as_uint(v[e + 1]);
    }
    return !__any(counts && (low & 0xffffu) != 0u);
}
// The second and third parts; returns whether the third is non-zero in a lane that counts.
__device__ __forceinline__ bool bf16_rest8(const float (&v)[8], u32x4_t &p1, u32x4_t &p2, bool counts = true) {
    uint32_t nz2 = 0u;
#pragma unroll
    for (int e = 0; e < 8; e += 2) {
        uint32_t h0, m0, l0, h1, m1, l1;
        bf16_parts(v[e], h0, m0, l0), bf16_parts(v[e + 1], h1, m1, l1);
        p1[e >> 1] = bf16_pair(m0, m1), p2[e >> 1] = bf16_pair(l0, l1);
        nz2 |= l0 | l1;
    }
    return __any(counts && nz2 != 0u);
}

// One batch of sixteen contraction steps: a[u], b[u] are the operands lane (column / row, half h) would hand to the u-th
// of eight `32x32x2` instructions (step 2 u + h).  FULL_A / FULL_B: that operand is a gradient - arbitrary fp32, all three
// parts taken without looking.  A batch whose part pairs would cost more than the eight fp32 instructions they replace
// (splitting included) is issued as those eight instructions.  a_counts = false: this lane's `a` feeds result rows that are
// never read (padding of a short operand): its values take no part in the choice of the parts, so the choice - and with it
// the order of the additions - depends on the operands alone.
template <bool FULL_A, bool FULL_B>
__device__ __forceinline__ floatx16 mfma_batch_bf16(floatx16 acc, const float (&a)[8], const float (&b)[8], bool a_counts = true) {
    static_assert(!(FULL_A && FULL_B), "one operand of a chain is a quantized tensor");
    u32x4_t pa0, pb0;
    const bool one_a = bf16_lead8(a, pa0, a_counts), one_b = bf16_lead8(b, pb0);
    if (FULL_A || FULL_B) {
        if (FULL_A ? one_b : one_a) {
            // three instructions: the quantized operand's single part against the gradient's three
            u32x4_t p1, p2;
            bf16_rest8(FULL_A ? a : b, p1, p2);
            acc = mfma_bf16(pa0, pb0, acc);
            acc = FULL_A ? mfma_bf16(p1, pb0, acc) : mfma_bf16(pa0, p1, acc);
            acc = FULL_A ? mfma_bf16(p2, pb0, acc) : mfma_bf16(pa0, p2, acc);
        } else {
#pragma unroll
            for (int u = 0; u < 8; ++u) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u], b[u], acc, 0, 0, 0);
        }
    } else if (one_a && one_b) {
        acc = mfma_bf16(pa0, pb0, acc);
    } else if (one_a || one_b) {
        // one side has a single part: up to three instructions
        u32x4_t p1, p2;
        const bool third = bf16_rest8(one_a ? b : a, p1, p2, one_a || a_counts);
        acc = mfma_bf16(pa0, pb0, acc);
        acc = one_a ? mfma_bf16(pa0, p1, acc) : mfma_bf16(p1, pb0, acc);
        if (third) acc = one_a ? mfma_bf16(pa0, p2, acc) : mfma_bf16(p2, pb0, acc);
    } else {
#pragma unroll
        for (int u = 0; u < 8; ++u) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u], b[u], acc, 0, 0, 0);
    }
    return acc;
}

// Two result blocks that share an operand which is a gradient (arbitrary fp32: all three parts): the shared operand is split
// ONCE for both.  SHARED_A: acc0 += a * b0, acc1 += a * b1; else acc0 += a0 * b, acc1 += a1 * b (then `a` is unused and
// b0 / b1 hold a0 / a1).  The other operand of a block takes the bf16 instruction where it has a single part (three
// instructions) and the eight fp32 instructions otherwise, block by block.
template <bool SHARED_A>
__device__ __forceinline__ void mfma_batch2_bf16(floatx16 &acc0, floatx16 &acc1, const float (&sh)[8], const float (&o0)[8],
                                                 const float (&o1)[8]) {
    u32x4_t s0, s1, s2, q0, q1;
    bf16_lead8(sh, s0);
    bf16_rest8(sh, s1, s2);
    const bool one0 = bf16_lead8(o0, q0), one1 = bf16_lead8(o1, q1);
    if (one0) {
        acc0 = SHARED_A ? mfma_bf16(s0, q0, acc0) : mfma_bf16(q0, s0, acc0);
        acc0 = SHARED_A ? mfma_bf16(s1, q0, acc0) : mfma_bf16(q0, s1, acc0);
        acc0 = SHARED_A ? mfma_bf16(s2, q0, acc0) : mfma_bf16(q0, s2, acc0);
    } else {
#pragma unroll
        for (int u = 0; u < 8; ++u)
            acc0 = SHARED_A ? __builtin_amdgcn_mfma_f32_32x32x2f32(sh[u], o0[u], acc0, 0, 0, 0)
                            : __builtin_amdgcn_mfma_f32_32x32x2f32(o0[u], sh[u], acc0, 0, 0, 0);
    }
    if (one1) {
        acc1 = SHARED_A ? mfma_bf16(s0, q1, acc1) : mfma_bf16(q1, s0, acc1);
        acc1 = SHARED_A ? mfma_bf16(s1, q1, acc1) : mfma_bf16(q1, s1, acc1);
        acc1 = SHARED_A ? mfma_bf16(s2, q1, acc1) : mfma_bf16(q1, s2, acc1);
    } else {
#pragma unroll
        for (int u = 0; u < 8; ++u)
            acc1 = SHARED_A ? __builtin_amdgcn_mfma_f32_32x32x2f32(sh[u], o1[u], acc1, 0, 0, 0)
                            : __builtin_amdgcn_mfma_f32_32x32x2f32(o1[u], sh[u], acc1, 0, 0, 0);
    }
}

// Same arguments and LDS reads as mfma_chain, every batch through mfma_batch_bf16: never slower than mfma_chain by more
// than the look at the operands.
template <bool FULL_A, bool FULL_B>
__device__ __forceinline__ floatx16 mfma_chain_bf16(floatx16 acc, const float *ap, int sa, const float *bp, int sb, int n_batches) {
    // (the next batch's operands are not requested ahead as in mfma_chain: the registers that takes spill in the kernels
    // that use this chain, and a batch is a few instructions, not eight, so the other wavefronts cover the LDS latency)
#pragma unroll
    for (int bt = 0; bt < 4; ++bt) {
        if (bt < n_batches) {
            float a[8], b[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) a[u] = ap[(16 * bt + 2 * u) * sa], b[u] = bp[(16 * bt + 2 * u) * sb];
            acc = mfma_batch_bf16<FULL_A, FULL_B>(acc, a, b);
        }
    }
    return acc;
}

}  // namespace hgq

// dispatch a (round_mode, overflow_mode) pair to template arguments
#define HGQ_DISPATCH_RM_OM(RMV, OMV, ...)                                   \
    do {                                                                    \
        switch ((RMV) * 4 + (OMV)) {                                        \
            case HGQ_TRN * 4 + HGQ_WRAP: { constexpr int RM = HGQ_TRN, OM = HGQ_WRAP; __VA_ARGS__; } break;         \
            case HGQ_TRN * 4 + HGQ_SAT: { constexpr int RM = HGQ_TRN, OM = HGQ_SAT; __VA_ARGS__; } break;           \
            case HGQ_TRN * 4 + HGQ_SAT_SYM: { constexpr int RM = HGQ_TRN, OM = HGQ_SAT_SYM; __VA_ARGS__; } break;   \
            case HGQ_RND * 4 + HGQ_WRAP: { constexpr int RM = HGQ_RND, OM = HGQ_WRAP; __VA_ARGS__; } break;         \
            case HGQ_RND * 4 + HGQ_SAT: { constexpr int RM = HGQ_RND, OM = HGQ_SAT; __VA_ARGS__; } break;           \
            case HGQ_RND * 4 + HGQ_SAT_SYM: { constexpr int RM = HGQ_RND, OM = HGQ_SAT_SYM; __VA_ARGS__; } break;   \
            case HGQ_RND_CONV * 4 + HGQ_WRAP: { constexpr int RM = HGQ_RND_CONV, OM = HGQ_WRAP; __VA_ARGS__; } break;       \
            case HGQ_RND_CONV * 4 + HGQ_SAT: { constexpr int RM = HGQ_RND_CONV, OM = HGQ_SAT; __VA_ARGS__; } break;         \
            case HGQ_RND_CONV * 4 + HGQ_SAT_SYM: { constexpr int RM = HGQ_RND_CONV, OM = HGQ_SAT_SYM; __VA_ARGS__; } break; \
            default: return hgq::fail(HGQ_ERR_ARG, "unknown round/overflow mode");                                          \
        }                                                                   \
    } while (0)
