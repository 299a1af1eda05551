// Stochastic rounding (round modes S_RND / S_RND_CONV in training): R(t) = floor(t + u), u uniform in [0, 1).
//
// The reference draws u from a Keras SeedGenerator (src/hgq/quantizer/internal/fixed_point_quantizer.py:56-57,279,404);
// its stream depends on the Keras backend, so no stream can be matched.  Here u comes from the counter-based generator
// Philox4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3", SC'11): element e of a call takes output
// word e % 4 of counter (e / 4, call offset) under key `seed`, and u = (word >> 8) * 2^-24.  The draw of an element is
// a pure function of (seed, offset, e): the backward pass recomputes it, nothing is stored, any grid gives the same bits.
#include "hgq_device.h"
#include "hgq_host.h"

namespace hgq {

__device__ __forceinline__ void philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0, uint32_t k1,
                                              uint32_t (&out)[4]) {
#pragma unroll
    for (int r = 0; r < 10; ++r) {
        const uint32_t lo0 = 0xD2511F53u * c0, hi0 = __umulhi(0xD2511F53u, c0);
        const uint32_t lo1 = 0xCD9E8D57u * c2, hi1 = __umulhi(0xCD9E8D57u, c2);
        const uint32_t n0 = hi1 ^ c1 ^ k0, n2 = hi0 ^ c3 ^ k1;
        c0 = n0, c1 = lo1, c2 = n2, c3 = lo0;
        k0 += 0x9E3779B9u, k1 += 0xBB67AE85u;
    }
    out[0] = c0, out[1] = c1, out[2] = c2, out[3] = c3;
}

__device__ __forceinline__ float srnd_uniform(int64_t e, uint64_t seed, uint64_t offset) {
    uint32_t w[4];
    const uint64_t c = (uint64_t)e >> 2;
    philox4x32_10((uint32_t)c, (uint32_t)(c >> 32), (uint32_t)offset, (uint32_t)(offset >> 32), (uint32_t)seed, (uint32_t)(seed >> 32), w);
    return (float)(w[e & 3] >> 8) * 5.9604644775390625e-08f;  // 2^-24: exact, in [0, 1)
}

__device__ __forceinline__ float srnd_round(float x, float f, float u) {
    const int fi = (int)f;
    return ldexpf(floorf(__fadd_rn(ldexpf(x, fi), u)), -fi);
}

template <int OM>
__global__ __launch_bounds__(256) void srnd_fwd_kernel(const float *__restrict__ x, const void *k, const float *i, const float *fb,
                                                       float *__restrict__ y, uint32_t *amax, uint32_t *anyneg, int64_t n, int64_t bw_size,
                                                       int64_t bw_inner, int mode, uint64_t seed, uint64_t offset, const uint64_t *__restrict__ offset_base,
                                                       uint64_t *__restrict__ used_offset) {
    const Mode m(mode);
    // the draw is (seed, offset + *offset_base): a base in device memory lets a recorded launch draw anew on every replay
    // (the caller advances it between steps); the sum is left for the backward pass, which must repeat this draw
    if (offset_base) offset += offset_base[0];
    if (used_offset && blockIdx.x == 0 && threadIdx.x == 0) used_offset[0] = offset;
    for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < n; e += (int64_t)gridDim.x * 256) {
        const int64_t b = (e / bw_inner) % bw_size;
        const KIF p = resolve_kif(load_k(k, b, m.k_u8), i[b], fb[b], m.kbi, m.round_params);
        int st;
        const float yv = overflow<OM>(srnd_round(x[e], p.f, srnd_uniform(e, seed, offset)), p, true, st);
        y[e] = yv;
        const float tv = m.track_input ? x[e] : yv;
        if (amax) atomicMax(&amax[b], abs_bits(tv));
        if (anyneg && tv < 0.0f) atomicOr(&anyneg[b], 1u);
    }
}

// the surrogate of quantize_grad with the rounded value of the same draw
template <int OM>
__global__ __launch_bounds__(256) void srnd_bwd_kernel(const float *__restrict__ dy, const float *__restrict__ x, const void *k, const float *i,
                                                       const float *fb, float *__restrict__ dx, float *di, float *dfb, int64_t n,
                                                       int64_t bw_size, int64_t bw_inner, int mode, uint64_t seed, uint64_t offset,
                                                       const uint64_t *__restrict__ offset_base) {
    const Mode m(mode);
    if (offset_base) offset += offset_base[0];
    for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < n; e += (int64_t)gridDim.x * 256) {
        const int64_t b = (e / bw_inner) % bw_size;
        const KIF p = resolve_kif(load_k(k, b, m.k_u8), i[b], fb[b], m.kbi, m.round_params);
        const float xq = srnd_round(x[e], p.f, srnd_uniform(e, seed, offset)), g = dy[e];
        int st = 0;
        if (OM != HGQ_WRAP) (void)overflow<OM>(xq, p, true, st);
        float gx, gi = 0.0f, gf = 0.0f;
        if (st == 0) {
            gx = g;
            gf = -HGQ_LN2 * (xq - x[e]) * g;
        } else {
            gx = 0.0f;
            const float ti = HGQ_LN2 * pow2(p.i) * g, tf = HGQ_LN2 * pow2(-p.f) * g;
            if (st & 1) gi += ti, gf += tf;
            if (st & 2) {
                gi += -p.k * ti;
                if (OM == HGQ_SAT_SYM) gf += -p.k * tf;
            }
        }
        if (m.kbi) gi -= gf;
        if (dx) dx[e] = gx;
        if (bw_size == n && bw_inner == 1) {
            if (di) di[e] = gi;
            if (dfb) dfb[e] = gf;
        } else {
            if (di && gi != 0.0f) atomicAdd(&di[b], gi);
            if (dfb && gf != 0.0f) atomicAdd(&dfb[b], gf);
        }
    }
}

static int srnd_check(const char *who, const void *x, const void *k, const void *i, const void *fb, int64_t n, int64_t bw_size, int64_t bw_inner,
                      int mode) {
    if (n < 0 || bw_size < 1 || bw_inner < 1) return fail(HGQ_ERR_ARG, "%s: bad sizes", who);
    if (n > 0 && (!x || !k || !i || !fb)) return fail(HGQ_ERR_ARG, "%s: null pointer", who);
    const Mode m(mode);
    if (m.round_mode != HGQ_S_RND && m.round_mode != HGQ_S_RND_CONV) return fail(HGQ_ERR_ARG, "%s: round mode %d is not a stochastic one", who, m.round_mode);
    if (!m.training) return fail(HGQ_ERR_ARG, "%s: stochastic rounding is a training-mode operation (inference rounds with RND / RND_CONV)", who);
    if (m.overflow_mode != HGQ_WRAP && m.overflow_mode != HGQ_SAT && m.overflow_mode != HGQ_SAT_SYM) return fail(HGQ_ERR_ARG, "%s: unknown overflow mode", who);
    return HGQ_OK;
}

}  // namespace hgq

using namespace hgq;

#define HGQ_SRND_OM(om, CALL)                    \
    do {                                         \
        if ((om) == HGQ_WRAP) CALL(HGQ_WRAP);    \
        else if ((om) == HGQ_SAT) CALL(HGQ_SAT); \
        else CALL(HGQ_SAT_SYM);                  \
    } while (0)

static int srnd_fwd_impl(const char *who, const float *x, const void *k, const float *i, const float *fb, float *y, uint32_t *amax,
                         uint32_t *anyneg, int64_t n, int64_t bw_size, int64_t bw_inner, int mode, uint64_t seed, uint64_t offset,
                         const uint64_t *offset_base, uint64_t *used_offset, void *stream) {
    int rc = srnd_check(who, x, k, i, fb, n, bw_size, bw_inner, mode);
    if (rc) return rc;
    hipStream_t s = (hipStream_t)stream;
    if (amax && (rc = fill_f32((float *)amax, 0.0f, bw_size, s))) return rc;
    if (anyneg && (rc = fill_f32((float *)anyneg, 0.0f, bw_size, s))) return rc;
    if (n == 0 && !used_offset) return HGQ_OK;
    if (n > 0 && !y) return fail(HGQ_ERR_ARG, "%s: null output", who);
    const int grid = persistent_grid((n + 255) / 256, 8);  // (n = 0 with used_offset: one workgroup that only leaves the offset)
#define CALL(OMV) hipLaunchKernelGGL((srnd_fwd_kernel<OMV>), dim3(grid), dim3(256), 0, s, x, k, i, fb, y, amax, anyneg, n, bw_size, bw_inner, mode, seed, offset, offset_base, used_offset)
    HGQ_SRND_OM(Mode(mode).overflow_mode, CALL);
#undef CALL
    return check_launch(who);
}

extern "C" int hgq_quantize_fwd_stochastic(const float *x, const void *k, const float *i, const float *fb, float *y, uint32_t *amax,
                                           uint32_t *anyneg, int64_t n, int64_t bw_size, int64_t bw_inner, int mode, uint64_t seed,
                                           uint64_t offset, void *stream) {
    return srnd_fwd_impl("hgq_quantize_fwd_stochastic", x, k, i, fb, y, amax, anyneg, n, bw_size, bw_inner, mode, seed, offset, nullptr, nullptr,
                         stream);
}

extern "C" int hgq_quantize_fwd_stochastic_at(const float *x, const void *k, const float *i, const float *fb, float *y, uint32_t *amax,
                                              uint32_t *anyneg, int64_t n, int64_t bw_size, int64_t bw_inner, int mode, uint64_t seed,
                                              uint64_t offset, const uint64_t *offset_base, uint64_t *used_offset, void *stream) {
    if (!offset_base || !used_offset) return fail(HGQ_ERR_ARG, "hgq_quantize_fwd_stochastic_at: null pointer");
    return srnd_fwd_impl("hgq_quantize_fwd_stochastic_at", x, k, i, fb, y, amax, anyneg, n, bw_size, bw_inner, mode, seed, offset, offset_base,
                         used_offset, stream);
}

static int srnd_bwd_impl(const char *who, const float *dy, const float *x, const void *k, const float *i, const float *fb, float *dx, float *di,
                         float *dfb, int64_t n, int64_t bw_size, int64_t bw_inner, int mode, uint64_t seed, uint64_t offset,
                         const uint64_t *offset_base, void *stream) {
    int rc = srnd_check(who, x, k, i, fb, n, bw_size, bw_inner, mode);
    if (rc) return rc;
    if (n > 0 && !dy) return fail(HGQ_ERR_ARG, "%s: null pointer", who);
    hipStream_t s = (hipStream_t)stream;
    const bool per_element = bw_size == n && bw_inner == 1;
    if (!per_element || n == 0) {
        if (di && (rc = fill_f32(di, 0.0f, bw_size, s))) return rc;
        if (dfb && (rc = fill_f32(dfb, 0.0f, bw_size, s))) return rc;
    }
    if (n == 0) return HGQ_OK;
    const int grid = persistent_grid((n + 255) / 256, 8);
#define CALL(OMV) hipLaunchKernelGGL((srnd_bwd_kernel<OMV>), dim3(grid), dim3(256), 0, s, dy, x, k, i, fb, dx, di, dfb, n, bw_size, bw_inner, mode, seed, offset, offset_base)
    HGQ_SRND_OM(Mode(mode).overflow_mode, CALL);
#undef CALL
    return check_launch(who);
}

extern "C" int hgq_quantize_bwd_stochastic(const float *dy, const float *x, const void *k, const float *i, const float *fb, float *dx, float *di,
                                           float *dfb, int64_t n, int64_t bw_size, int64_t bw_inner, int mode, uint64_t seed, uint64_t offset,
                                           void *stream) {
    return srnd_bwd_impl("hgq_quantize_bwd_stochastic", dy, x, k, i, fb, dx, di, dfb, n, bw_size, bw_inner, mode, seed, offset, nullptr, stream);
}

extern "C" int hgq_quantize_bwd_stochastic_at(const float *dy, const float *x, const void *k, const float *i, const float *fb, float *dx,
                                              float *di, float *dfb, int64_t n, int64_t bw_size, int64_t bw_inner, int mode, uint64_t seed,
                                              const uint64_t *used_offset, void *stream) {
    if (!used_offset) return fail(HGQ_ERR_ARG, "hgq_quantize_bwd_stochastic_at: null pointer");
    return srnd_bwd_impl("hgq_quantize_bwd_stochastic_at", dy, x, k, i, fb, dx, di, dfb, n, bw_size, bw_inner, mode, seed, 0, used_offset, stream);
}

// counters[j][0] += increments[j]: the draw counters of the seed generators a step used, advanced in one launch
#define SRND_MAX_COUNTERS 32
struct CounterBatch {
    uint64_t *counter[SRND_MAX_COUNTERS];
    uint64_t increment[SRND_MAX_COUNTERS];
    int count;
};
namespace hgq {
__global__ __launch_bounds__(64) void counters_advance_kernel(const CounterBatch b) {
    const int j = threadIdx.x;
    if (j < b.count) b.counter[j][0] += b.increment[j];
}
}  // namespace hgq

extern "C" int hgq_counters_advance(uint64_t *const *counters, const uint64_t *increments, int count, void *stream) {
    if (count < 0 || (count > 0 && (!counters || !increments))) return fail(HGQ_ERR_ARG, "hgq_counters_advance: bad arguments");
    for (int j0 = 0; j0 < count; j0 += SRND_MAX_COUNTERS) {
        CounterBatch b;
        b.count = count - j0 < SRND_MAX_COUNTERS ? count - j0 : SRND_MAX_COUNTERS;
        for (int j = 0; j < b.count; ++j) {
            if (!counters[j0 + j]) return fail(HGQ_ERR_ARG, "hgq_counters_advance: null counter %d", j0 + j);
            for (int u = 0; u < j; ++u)
                if (b.counter[u] == counters[j0 + j]) return fail(HGQ_ERR_ARG, "hgq_counters_advance: counter %d is listed twice", j0 + j);
            b.counter[j] = counters[j0 + j], b.increment[j] = increments[j0 + j];
        }
        hipLaunchKernelGGL(counters_advance_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, b);
        const int rc = check_launch("hgq_counters_advance");
        if (rc) return rc;
    }
    return HGQ_OK;
}
