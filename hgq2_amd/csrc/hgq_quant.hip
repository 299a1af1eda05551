// Fixed-point quantizer kernels: forward, surrogate backward, integer-bit tracking.
//
// Three layouts of the bit-width operands are served:
//   per-element  (bw_size == n)            1-D kernel, 128-bit loads of x, k, i, f
//   shared       (bw_size == 1)            1-D kernel, operands in registers, one reduction per launch
//   per-column   (bw_inner == 1, x = [rows, bw_size])  2-D kernel: a thread owns fixed columns
//                and walks down the rows, so bit-widths and the partial reductions stay in
//                registers; one atomic per column per workgroup at the end
// plus a scalar fallback for bw_inner > 1.
#include <math.h>
#include <stdarg.h>
#include <stdio.h>

#include <mutex>

#include "hgq_device.h"
#include "hgq_host.h"

namespace hgq {

static thread_local char g_err[256] = "";

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

__global__ void fill_u32_kernel(uint32_t *p, uint32_t v, int64_t n) {
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < n; t += (int64_t)gridDim.x * blockDim.x) p[t] = v;
}

int fill_u32(uint32_t *p, uint32_t v, int64_t n, hipStream_t s) {
    if (n <= 0) return HGQ_OK;
    int grid = (int)((n + 255) / 256);
    if (grid > 2048) grid = 2048;
    hipLaunchKernelGGL(fill_u32_kernel, dim3(grid), dim3(256), 0, s, p, v, n);
    return check_launch("fill");
}

// ------------------------------------------------------------------------------------------
// wavefront (64 lanes) and workgroup reductions
// ------------------------------------------------------------------------------------------
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        uint32_t t = (uint32_t)__shfl_xor((int)v, o, 64);
        v = t > v ? t : v;
    }
    return v;
}
__device__ __forceinline__ uint32_t wave_or_u32(uint32_t v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v |= (uint32_t)__shfl_xor((int)v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_sum_f32(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

template <int VEC>
struct VecIO;
template <>
struct VecIO<1> {
    static __device__ __forceinline__ void load(const float *p, int64_t v, float *o) { o[0] = p[v]; }
    static __device__ __forceinline__ void store(float *p, int64_t v, const float *o) { p[v] = o[0]; }
    static __device__ __forceinline__ void load_k(const void *k, int64_t v, bool u8, float *o) { o[0] = hgq::load_k(k, v, u8); }
    static __device__ __forceinline__ void store_u32(uint32_t *p, int64_t v, const uint32_t *o) { p[v] = o[0]; }
};
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// 128-bit accesses.  Loads and stores are non-temporal: every operand is touched once, so the
// caches are bypassed instead of polluted; measured on MI355X this is worth ~10 % of bandwidth.
template <>
struct VecIO<4> {
    static __device__ __forceinline__ void load(const float *p, int64_t v, float *o) {
        const f32x4 t = __builtin_nontemporal_load((const f32x4 *)p + v);
        o[0] = t.x, o[1] = t.y, o[2] = t.z, o[3] = t.w;
    }
    static __device__ __forceinline__ void store(float *p, int64_t v, const float *o) {
        f32x4 t;
        t.x = o[0], t.y = o[1], t.z = o[2], t.w = o[3];
        __builtin_nontemporal_store(t, (f32x4 *)p + v);
    }
    static __device__ __forceinline__ void load_k(const void *k, int64_t v, bool u8, float *o) {
        if (u8) {
            uchar4 t = ((const uchar4 *)k)[v];
            o[0] = t.x, o[1] = t.y, o[2] = t.z, o[3] = t.w;
        } else {
            load((const float *)k, v, o);
        }
    }
    static __device__ __forceinline__ void store_u32(uint32_t *p, int64_t v, const uint32_t *o) {
        u32x4 t;
        t.x = o[0], t.y = o[1], t.z = o[2], t.w = o[3];
        __builtin_nontemporal_store(t, (u32x4 *)p + v);
    }
};

// ------------------------------------------------------------------------------------------
// 1-D kernels: per-element or shared bit-widths
// ------------------------------------------------------------------------------------------
#define Q1D_BS 512

template <int RM, int OM, int VEC, bool SHARED>
__global__ __launch_bounds__(Q1D_BS) void quant_fwd_1d(const float *__restrict__ x, const void *__restrict__ k,
                                                    const float *__restrict__ i, const float *__restrict__ fb,
                                                    float *__restrict__ y, uint32_t *amax, uint32_t *anyneg,
                                                    int64_t nvec, int mode) {
    const Mode m(mode);
    KIF ps;
    if (SHARED) ps = resolve_kif(load_k(k, 0, m.k_u8), i[0], fb[0], m.kbi, m.round_params);
    uint32_t lmax = 0, lneg = 0;
    const bool need_k = !(OM == HGQ_WRAP && m.training), need_i = need_k || m.kbi;
    for (int64_t v = (int64_t)blockIdx.x * Q1D_BS + threadIdx.x; v < nvec; v += (int64_t)gridDim.x * Q1D_BS) {
        float xv[VEC], kv[VEC] = {0.f}, iv[VEC] = {0.f}, fv[VEC], yv[VEC];
        VecIO<VEC>::load(x, v, xv);
        if (!SHARED) {
            // a WRAP quantizer in training mode only rounds: k (and i, unless f = b - i) are dead operands
            if (need_k) VecIO<VEC>::load_k(k, v, m.k_u8, kv);
            if (need_i) VecIO<VEC>::load(i, v, iv);
            VecIO<VEC>::load(fb, v, fv);
        }
        uint32_t ab[VEC], ng[VEC];
#pragma unroll
        for (int c = 0; c < VEC; ++c) {
            const KIF p = SHARED ? ps : resolve_kif(kv[c], iv[c], fv[c], m.kbi, m.round_params);
            yv[c] = quantize<RM, OM>(xv[c], p, m.training);
            const float tv = m.track_input ? xv[c] : yv[c];
            ab[c] = abs_bits(tv);
            ng[c] = tv < 0.0f ? 1u : 0u;
            lmax = ab[c] > lmax ? ab[c] : lmax;
            lneg |= ng[c];
        }
        VecIO<VEC>::store(y, v, yv);
        if (!SHARED) {
            if (amax) VecIO<VEC>::store_u32(amax, v, ab);
            if (anyneg) VecIO<VEC>::store_u32(anyneg, v, ng);
        }
    }
    if (SHARED && (amax || anyneg)) {
        __shared__ uint32_t smax[Q1D_BS / 64], sneg[Q1D_BS / 64];
        lmax = wave_max_u32(lmax);
        lneg = wave_or_u32(lneg);
        if ((threadIdx.x & 63) == 0) smax[threadIdx.x >> 6] = lmax, sneg[threadIdx.x >> 6] = lneg;
        __syncthreads();
        if (threadIdx.x == 0) {
            uint32_t a = smax[0], g = sneg[0];
            for (int w = 1; w < Q1D_BS / 64; ++w) a = smax[w] > a ? smax[w] : a, g |= sneg[w];
            if (amax) atomicMax(amax, a);
            if (anyneg && g) atomicOr(anyneg, 1u);
        }
    }
}

template <int RM, int OM, int VEC, bool SHARED>
__global__ __launch_bounds__(Q1D_BS) void quant_bwd_1d(const float *__restrict__ dy, const float *__restrict__ x,
                                                    const void *__restrict__ k, const float *__restrict__ i,
                                                    const float *__restrict__ fb, float *__restrict__ dx,
                                                    float *di, float *dfb, int64_t nvec, int mode) {
    const Mode m(mode);
    KIF ps;
    if (SHARED) ps = resolve_kif(load_k(k, 0, m.k_u8), i[0], fb[0], m.kbi, m.round_params);
    float si = 0.0f, sf = 0.0f;
    const bool need_k = OM != HGQ_WRAP, need_i = need_k || m.kbi;  // the WRAP surrogate gradient only rounds
    for (int64_t v = (int64_t)blockIdx.x * Q1D_BS + threadIdx.x; v < nvec; v += (int64_t)gridDim.x * Q1D_BS) {
        float gv[VEC], xv[VEC], kv[VEC] = {0.f}, iv[VEC] = {0.f}, fv[VEC], dxv[VEC], div[VEC], dfv[VEC];
        VecIO<VEC>::load(dy, v, gv);
        VecIO<VEC>::load(x, v, xv);
        if (!SHARED) {
            if (need_k) VecIO<VEC>::load_k(k, v, m.k_u8, kv);
            if (need_i) VecIO<VEC>::load(i, v, iv);
            VecIO<VEC>::load(fb, v, fv);
        }
#pragma unroll
        for (int c = 0; c < VEC; ++c) {
            const KIF p = SHARED ? ps : resolve_kif(kv[c], iv[c], fv[c], m.kbi, m.round_params);
            float gi, gf;
            quantize_grad<RM, OM>(xv[c], gv[c], p, dxv[c], gi, gf);
            if (m.kbi) gi -= gf;  // f = b - i
            div[c] = gi, dfv[c] = gf;
            si += gi, sf += gf;
        }
        if (dx) VecIO<VEC>::store(dx, v, dxv);
        if (!SHARED) {
            if (di) VecIO<VEC>::store(di, v, div);
            if (dfb) VecIO<VEC>::store(dfb, v, dfv);
        }
    }
    if (SHARED) {
        __shared__ float ssi[Q1D_BS / 64], ssf[Q1D_BS / 64];
        si = wave_sum_f32(si);
        sf = wave_sum_f32(sf);
        if ((threadIdx.x & 63) == 0) ssi[threadIdx.x >> 6] = si, ssf[threadIdx.x >> 6] = sf;
        __syncthreads();
        if (threadIdx.x == 0) {
            float ti = 0.f, tf = 0.f;
            for (int w = 0; w < Q1D_BS / 64; ++w) ti += ssi[w], tf += ssf[w];
            if (di) atomicAdd(di, ti);
            if (dfb) atomicAdd(dfb, tf);
        }
    }
}

// ------------------------------------------------------------------------------------------
// Per-element bit-widths, fp32 k, no trackers: the standalone-quantizer case.  Nothing but the streams: the training
// flag and the set of live operands are template arguments, the raw variables are always rounded (the identity on
// integer-valued ones), KIF / KBI is a select - no branch sits between the loads.  LIVE bit 0: `i` is read; bit 1: `k`
// is read.  A WRAP quantizer in training mode only rounds, so k is dead there, and i as well unless f = b - i.
//
// U = vectors (128 bits) per lane and array.  U = 1: thread t of the launch takes vector v_begin + t (checked against
// v_end): the form for small inputs and for the remainder behind whole tiles.  U = 2: a wavefront owns 2 KB of every
// array (lane l takes vectors l and l + 64 of the wavefront's tile) and requests them one after the other (see
// HGQ_PE_WAIT below); the launch covers whole tiles only, so no load sits behind a bounds check.  At 4 Mi elements U = 2 puts the whole problem on the device in ONE round of workgroups (1024 workgroups of
// 512 threads = what 256 CUs hold) instead of two rounds that run in step - all load, all store, all retire, all
// start again - and pay the store-acknowledge + launch + first-load latency once more in the middle.
// ------------------------------------------------------------------------------------------
template <int LIVE>
__device__ __forceinline__ KIF pe_kif(const f32x4 &kv, const f32x4 &iv, const f32x4 &fv, int c, bool kbi) {
    KIF p;
    p.k = (LIVE & 2) ? kv[c] : 1.0f;
    p.i = (LIVE & 1) ? rintf(iv[c]) : 0.0f;
    const float fb = rintf(fv[c]);
    p.f = kbi ? __fsub_rn(fb, p.i) : fb;
    return p;
}

template <int U>
__device__ __forceinline__ int64_t pe_first_vector(int64_t v_begin) {
    if (U == 1) return v_begin + (int64_t)blockIdx.x * Q1D_BS + threadIdx.x;
    return v_begin + ((int64_t)blockIdx.x * (Q1D_BS / 64) + (threadIdx.x >> 6)) * (64 * U) + (threadIdx.x & 63);
}

// In the two-vector form every load is waited for before the next one is issued, and every array's pair of stores before
// the next array's: ONE request in flight per wavefront.  The 32 wavefronts of a CU still keep 8 MB in flight across
// the device, which covers the memory latency; more only queues up in front of the memory channels, and the queues cost
// bandwidth - measured on the 3-read 4-write stream at 4 Mi elements: all six loads in flight 22.3 us, pairs 21.3 us,
// one at a time 19.2 us, and 18.8 us with the store pairs waited for as well.  The waits also keep the device in step:
// all wavefronts read the same array at the same time, then the next one, then all write.
#define HGQ_PE_WAIT() asm volatile("s_waitcnt vmcnt(0)" ::: "memory")
#define HGQ_PE_LOAD(dst, src)                                                 \
    _Pragma("unroll") for (int u = 0; u < U; ++u) {                           \
        dst[u] = __builtin_nontemporal_load(src + v0 + 64 * u);               \
        if (U > 1) HGQ_PE_WAIT();                                             \
    }
#define HGQ_PE_STORE(src, dst)                                                \
    do {                                                                      \
        _Pragma("unroll") for (int u = 0; u < U; ++u) __builtin_nontemporal_store(src[u], dst + v0 + 64 * u); \
        if (U > 1) HGQ_PE_WAIT();                                             \
    } while (0)

template <int RM, int OM, bool TRAIN, int LIVE, int U>
__global__ __launch_bounds__(Q1D_BS) void quant_fwd_pe(const f32x4 *__restrict__ x, const f32x4 *__restrict__ k,
                                                       const f32x4 *__restrict__ i, const f32x4 *__restrict__ fb,
                                                       f32x4 *__restrict__ y, int64_t v_begin, int64_t v_end, int kbi) {
    const int64_t v0 = pe_first_vector<U>(v_begin);
    if (U == 1 && v0 >= v_end) return;
    f32x4 xv[U], fv[U], iv[U], kv[U], yv[U];
    HGQ_PE_LOAD(xv, x);
    HGQ_PE_LOAD(fv, fb);
    if (LIVE & 1) HGQ_PE_LOAD(iv, i);
    if (LIVE & 2) HGQ_PE_LOAD(kv, k);
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
        for (int c = 0; c < 4; ++c) yv[u][c] = quantize<RM, OM>(xv[u][c], pe_kif<LIVE>(kv[u], iv[u], fv[u], c, kbi != 0), TRAIN);
    }
    HGQ_PE_STORE(yv, y);
}

template <int RM, int OM, int LIVE, int U>
__global__ __launch_bounds__(Q1D_BS) void quant_bwd_pe(const f32x4 *__restrict__ dy, const f32x4 *__restrict__ x,
                                                       const f32x4 *__restrict__ k, const f32x4 *__restrict__ i,
                                                       const f32x4 *__restrict__ fb, f32x4 *__restrict__ dx,
                                                       f32x4 *__restrict__ di, f32x4 *__restrict__ dfb, int64_t v_begin,
                                                       int64_t v_end, int kbi) {
    const int64_t v0 = pe_first_vector<U>(v_begin);
    if (U == 1 && v0 >= v_end) return;
    f32x4 gv[U], xv[U], fv[U], iv[U], kv[U];
    HGQ_PE_LOAD(gv, dy);
    HGQ_PE_LOAD(xv, x);
    HGQ_PE_LOAD(fv, fb);
    if (LIVE & 1) HGQ_PE_LOAD(iv, i);
    if (LIVE & 2) HGQ_PE_LOAD(kv, k);
    f32x4 gx[U], gi[U], gf[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            float a, b, d;
            quantize_grad<RM, OM>(xv[u][c], gv[u][c], pe_kif<LIVE>(kv[u], iv[u], fv[u], c, kbi != 0), a, b, d);
            if (kbi) b -= d;  // f = b - i
            gx[u][c] = a, gi[u][c] = b, gf[u][c] = d;
        }
    }
    if (dx) HGQ_PE_STORE(gx, dx);
    if (di) HGQ_PE_STORE(gi, di);
    if (dfb) HGQ_PE_STORE(gf, dfb);
}

// Forward and surrogate backward of a training step in ONE pass: x (and k, i where live), f and the upstream gradient
// in; y, dx, di, df out.  The value is rounded once and every operand crosses HBM once: 28 B/elem in WRAP training
// (x, f, dy read; four arrays written) against 12 + 24 for the two separate launches, 36 B/elem with every operand
// live against 20 + 32, and one launch ramp instead of two.
template <int RM, int OM, int LIVE, int U>
__global__ __launch_bounds__(Q1D_BS) void quant_fwd_bwd_pe(const f32x4 *__restrict__ x, const f32x4 *__restrict__ k,
                                                           const f32x4 *__restrict__ i, const f32x4 *__restrict__ fb,
                                                           const f32x4 *__restrict__ dy, f32x4 *__restrict__ y,
                                                           f32x4 *__restrict__ dx, f32x4 *__restrict__ di,
                                                           f32x4 *__restrict__ dfb, int64_t v_begin, int64_t v_end, int kbi) {
    const int64_t v0 = pe_first_vector<U>(v_begin);
    if (U == 1 && v0 >= v_end) return;
    f32x4 xv[U], fv[U], gv[U], iv[U], kv[U];
    HGQ_PE_LOAD(xv, x);
    HGQ_PE_LOAD(fv, fb);
    HGQ_PE_LOAD(gv, dy);
    if (LIVE & 1) HGQ_PE_LOAD(iv, i);
    if (LIVE & 2) HGQ_PE_LOAD(kv, k);
    f32x4 yv[U], gx[U], gi[U], gf[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            float a, b, d;
            yv[u][c] = quantize_with_grad<RM, OM>(xv[u][c], gv[u][c], pe_kif<LIVE>(kv[u], iv[u], fv[u], c, kbi != 0), a, b, d);
            if (kbi) b -= d;  // f = b - i
            gx[u][c] = a, gi[u][c] = b, gf[u][c] = d;
        }
    }
    HGQ_PE_STORE(yv, y);
    if (dx) HGQ_PE_STORE(gx, dx);
    if (di) HGQ_PE_STORE(gi, di);
    if (dfb) HGQ_PE_STORE(gf, dfb);
}

// ------------------------------------------------------------------------------------------
// 2-D kernels: x = [rows, M], one bit-width entry per column
// thread (tx, ty): tx walks column groups of VEC, ty walks rows; TX is a power of two <= 64
// ------------------------------------------------------------------------------------------
// Row batches of the per-column kernels: a thread has QC_U rows of its column group in flight
// (buffer loads; rows past the end of the workgroup's chunk read as zero, which is neutral for
// every reduction below), and a workgroup walks a contiguous chunk of rows so that a column sees
// few workgroups - and few atomics - at the end.
#define QC_U 8
#define QC_BWD_U 8
template <int VEC>
__device__ __forceinline__ void qc_load(const __amdgpu_buffer_rsrc_t rs, uint32_t off, float *o) {
    if (VEC == 4) {
        const f32x4_t t = buf_ld4(rs, off);
        o[0] = t[0], o[1 % VEC] = t[1], o[2 % VEC] = t[2], o[3 % VEC] = t[3];
    } else {
        o[0] = buf_ld1(rs, off);
    }
}

template <int VEC>
__device__ __forceinline__ void qc_store(const __amdgpu_buffer_rsrc_t rs, uint32_t off, const float *v) {
    if (VEC == 4) {
        f32x4_t t;
        t[0] = v[0], t[1] = v[1 % VEC], t[2] = v[2 % VEC], t[3] = v[3 % VEC];
        buf_st4(rs, off, t);
    } else {
        buf_st1(rs, off, v[0]);
    }
}

// TRAIN: the quantizer's training flag as a template argument (the WRAP training branch is decided once, not per element).
// A workgroup's chunk is below 2 GiB, so all index arithmetic inside it is 32-bit and a load and the store of the same
// row share one byte offset; rows past the end of the chunk are dropped by the descriptors' range check.
template <int RM, int OM, int VEC, bool TRAIN>
__global__ __launch_bounds__(256) void quant_fwd_cols(const float *__restrict__ x, const void *__restrict__ k,
                                                      const float *__restrict__ i, const float *__restrict__ fb,
                                                      float *__restrict__ y, uint32_t *amax, uint32_t *anyneg,
                                                      int64_t rows, int64_t M, int TX, int64_t rows_per_wg, int mode, int sliced) {
    const Mode m(mode);
    const int TY = 256 / TX;
    const int tx = threadIdx.x % TX, ty = threadIdx.x / TX;
    const int cg = (int)(M / VEC);
    const int c = (int)blockIdx.x * TX + tx;
    const bool active = c < cg;
    KIF p[VEC];
    uint32_t lmax[VEC];
    float lmin[VEC];  // a negative minimum <=> some tracked value was negative (-0 and NaN are not)
#pragma unroll
    for (int e = 0; e < VEC; ++e) p[e] = KIF{0.f, 0.f, 0.f}, lmax[e] = 0, lmin[e] = 0.f;
    const int64_t row0 = (int64_t)blockIdx.y * rows_per_wg;
    const int n_rows = (int)min(rows - row0, rows_per_wg);
    const __amdgpu_buffer_rsrc_t rs = buf_rsrc(x + row0 * M, (int64_t)n_rows * M * 4);
    const __amdgpu_buffer_rsrc_t rs_y = buf_rsrc(y + row0 * M, (int64_t)n_rows * M * 4);
    const uint32_t row_bytes = (uint32_t)cg * VEC * 4u, trip_rows = (uint32_t)TY * QC_U;
    // byte offset of this thread's element(s) in row `r` of the chunk
    auto offset = [&](int r) { return (active && r < n_rows) ? (uint32_t)r * row_bytes + (uint32_t)c * (VEC * 4u) : BUF_OOB; };
    // the first rows are requested before the bit-width operands: a workgroup is short-lived (often a single
    // trip), and operands first would put two memory round trips end to end
    float xv[QC_U][VEC];
    uint32_t off[QC_U];
#pragma unroll
    for (int u = 0; u < QC_U; ++u) {
        off[u] = offset(ty + TY * u);
        qc_load<VEC>(rs, off[u], xv[u]);
    }
    if (active) {
        float kv[VEC], iv[VEC], fv[VEC];
        VecIO<VEC>::load_k(k, c, m.k_u8, kv);
        VecIO<VEC>::load(i, c, iv);
        VecIO<VEC>::load(fb, c, fv);
#pragma unroll
        for (int e = 0; e < VEC; ++e) p[e] = resolve_kif(kv[e], iv[e], fv[e], m.kbi, m.round_params);
    }
    const bool track_input = m.track_input;
    for (int rb = 0; rb < n_rows; rb += (int)trip_rows) {
        float cur[QC_U][VEC];
        uint32_t cur_off[QC_U];
#pragma unroll
        for (int u = 0; u < QC_U; ++u) {
            cur_off[u] = off[u];
#pragma unroll
            for (int e = 0; e < VEC; ++e) cur[u][e] = xv[u][e];
        }
        // next trip's rows in flight while this one is quantized
#pragma unroll
        for (int u = 0; u < QC_U; ++u) {
            off[u] = offset(rb + (int)trip_rows + ty + TY * u);
            qc_load<VEC>(rs, off[u], xv[u]);
        }
#pragma unroll
        for (int u = 0; u < QC_U; ++u) {
            float yv[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                yv[e] = quantize<RM, OM>(cur[u][e], p[e], TRAIN);
                float tv = track_input ? cur[u][e] : yv[e];
                // rows past the end read as zero; a saturating quantizer whose range excludes zero maps that to a bound,
                // which must not reach the trackers (WRAP keeps zero at zero)
                if (OM != HGQ_WRAP) tv = cur_off[u] != BUF_OOB ? tv : 0.0f;
                const uint32_t ab = abs_bits(tv);
                lmax[e] = ab > lmax[e] ? ab : lmax[e];
                lmin[e] = fminf(lmin[e], tv);
            }
            qc_store<VEC>(rs_y, cur_off[u], yv);
        }
    }
    if (amax || anyneg) {
        __shared__ uint32_t smax[256 * VEC], sneg[256 * VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) smax[threadIdx.x * VEC + e] = lmax[e], sneg[threadIdx.x * VEC + e] = lmin[e] < 0.0f ? 1u : 0u;
        __syncthreads();
        for (int s = TY / 2; s > 0; s >>= 1) {
            if (ty < s) {
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    const uint32_t o = smax[(threadIdx.x + s * TX) * VEC + e];
                    uint32_t &mine = smax[threadIdx.x * VEC + e];
                    mine = o > mine ? o : mine;
                    sneg[threadIdx.x * VEC + e] |= sneg[(threadIdx.x + s * TX) * VEC + e];
                }
            }
            __syncthreads();
        }
        if (ty == 0 && active) {
            if (sliced) {
                // one tracker slice per row chunk, written whole: nothing to clear beforehand, no atomics; the
                // integer-bit update combines the slices
                const int64_t base = (int64_t)blockIdx.y * M + (int64_t)c * VEC;
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    if (amax) amax[base + e] = smax[tx * VEC + e];
                    if (anyneg) anyneg[base + e] = sneg[tx * VEC + e];
                }
            } else {
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    if (amax) atomicMax(&amax[c * VEC + e], smax[tx * VEC + e]);
                    if (anyneg && sneg[tx * VEC + e]) atomicOr(&anyneg[c * VEC + e], 1u);
                }
            }
        }
    }
}

template <int RM, int OM, int VEC>
__global__ __launch_bounds__(256) void quant_bwd_cols(const float *__restrict__ dy, const float *__restrict__ x,
                                                      const void *__restrict__ k, const float *__restrict__ i,
                                                      const float *__restrict__ fb, float *__restrict__ dx, float *di,
                                                      float *dfb, int64_t rows, int64_t M, int TX, int64_t rows_per_wg, int mode,
                                                      float *part) {
    const Mode m(mode);
    const int TY = 256 / TX;
    const int tx = threadIdx.x % TX, ty = threadIdx.x / TX;
    const int cg = (int)(M / VEC);
    const int c = (int)blockIdx.x * TX + tx;
    const bool active = c < cg;
    KIF p[VEC];
    float si[VEC], sf[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) p[e] = KIF{0.f, 0.f, 0.f}, si[e] = 0.0f, sf[e] = 0.0f;
    if (active) {
        float kv[VEC], iv[VEC], fv[VEC];
        VecIO<VEC>::load_k(k, c, m.k_u8, kv);
        VecIO<VEC>::load(i, c, iv);
        VecIO<VEC>::load(fb, c, fv);
#pragma unroll
        for (int e = 0; e < VEC; ++e) p[e] = resolve_kif(kv[e], iv[e], fv[e], m.kbi, m.round_params);
    }
    const int64_t row0 = (int64_t)blockIdx.y * rows_per_wg;
    const int n_rows = (int)min(rows - row0, rows_per_wg);
    // a chunk is below 2 GiB: 32-bit index arithmetic, one byte offset for a row's two loads and its store (rows past
    // the end are dropped by the descriptors' range check)
    const int64_t chunk_bytes = (int64_t)n_rows * M * 4;
    const __amdgpu_buffer_rsrc_t rs_g = buf_rsrc(dy + row0 * M, chunk_bytes), rs_x = buf_rsrc(x + row0 * M, chunk_bytes);
    const __amdgpu_buffer_rsrc_t rs_dx = buf_rsrc(dx ? dx + row0 * M : const_cast<float *>(x), dx ? chunk_bytes : 0);
    const uint32_t row_bytes = (uint32_t)cg * VEC * 4u;
    constexpr int U = QC_BWD_U;  // rows in flight per thread (two operands each)
    for (int rb = 0; rb < n_rows; rb += TY * U) {
        float gv[U][VEC], xv[U][VEC];
        uint32_t off[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int r = rb + ty + TY * u;
            off[u] = (active && r < n_rows) ? (uint32_t)r * row_bytes + (uint32_t)c * (VEC * 4u) : BUF_OOB;
            qc_load<VEC>(rs_g, off[u], gv[u]);
            qc_load<VEC>(rs_x, off[u], xv[u]);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            float dxv[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                float gi, gf;
                quantize_grad<RM, OM>(xv[u][e], gv[u][e], p[e], dxv[e], gi, gf);
                if (m.kbi) gi -= gf;
                si[e] += gi, sf[e] += gf;
            }
            if (dx) qc_store<VEC>(rs_dx, off[u], dxv);  // nothing is issued when the data gradient is not wanted
        }
    }
    __shared__ float ssi[256 * VEC], ssf[256 * VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) ssi[threadIdx.x * VEC + e] = si[e], ssf[threadIdx.x * VEC + e] = sf[e];
    __syncthreads();
    for (int s = TY / 2; s > 0; s >>= 1) {
        if (ty < s) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                ssi[threadIdx.x * VEC + e] += ssi[(threadIdx.x + s * TX) * VEC + e];
                ssf[threadIdx.x * VEC + e] += ssf[(threadIdx.x + s * TX) * VEC + e];
            }
        }
        __syncthreads();
    }
    if (ty == 0 && active) {
        if (part) {
            // slice blockIdx.y of `part`, [df (M) | di (M, only when wanted)], written whole: nothing to clear, no atomics,
            // and the sum over the slices that follows has a fixed order
            float *my = part + (int64_t)blockIdx.y * (di ? 2 * M : M) + c * VEC;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                my[e] = ssf[tx * VEC + e];
                if (di) my[M + e] = ssi[tx * VEC + e];
            }
        } else {
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                if (di) atomicAdd(&di[c * VEC + e], ssi[tx * VEC + e]);
                if (dfb) atomicAdd(&dfb[c * VEC + e], ssf[tx * VEC + e]);
            }
        }
    }
}

// ------------------------------------------------------------------------------------------
// scalar fallback: arbitrary (bw_size, bw_inner); reductions go straight to global atomics
// ------------------------------------------------------------------------------------------
template <int RM, int OM>
__global__ __launch_bounds__(256) void quant_fwd_generic(const float *__restrict__ x, const void *k, const float *i,
                                                         const float *fb, float *__restrict__ y, uint32_t *amax,
                                                         uint32_t *anyneg, int64_t n, int64_t bw_size, int64_t bw_inner,
                                                         int mode) {
    const Mode m(mode);
    for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < n; e += (int64_t)gridDim.x * 256) {
        const int64_t b = (e / bw_inner) % bw_size;
        const KIF p = resolve_kif(load_k(k, b, m.k_u8), i[b], fb[b], m.kbi, m.round_params);
        const float yv = quantize<RM, OM>(x[e], p, m.training);
        y[e] = yv;
        const float tv = m.track_input ? x[e] : yv;
        if (amax) atomicMax(&amax[b], abs_bits(tv));
        if (anyneg && tv < 0.0f) atomicOr(&anyneg[b], 1u);
    }
}

template <int RM, int OM>
__global__ __launch_bounds__(256) void quant_bwd_generic(const float *__restrict__ dy, const float *__restrict__ x,
                                                         const void *k, const float *i, const float *fb,
                                                         float *__restrict__ dx, float *di, float *dfb, int64_t n,
                                                         int64_t bw_size, int64_t bw_inner, int mode) {
    const Mode m(mode);
    for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < n; e += (int64_t)gridDim.x * 256) {
        const int64_t b = (e / bw_inner) % bw_size;
        const KIF p = resolve_kif(load_k(k, b, m.k_u8), i[b], fb[b], m.kbi, m.round_params);
        float gx, gi, gf;
        quantize_grad<RM, OM>(x[e], dy[e], p, gx, gi, gf);
        if (m.kbi) gi -= gf;
        if (dx) dx[e] = gx;
        if (di && gi != 0.0f) atomicAdd(&di[b], gi);
        if (dfb && gf != 0.0f) atomicAdd(&dfb[b], gf);
    }
}

// ------------------------------------------------------------------------------------------
// many small quantizers with per-element bit-widths in one launch (the kernel / bias quantizers of a model: a few
// thousand elements each, every launch of its own costs more than its work)
// ------------------------------------------------------------------------------------------
struct QuantBatch {
    hgq_quant_item item[HGQ_QUANT_BATCH];
};
struct QuantGradBatch {
    hgq_quant_grad_item item[HGQ_QUANT_BATCH];
};

// grid.y = quantizer, grid.x strides over its elements; round and overflow modes are read per item
__global__ __launch_bounds__(256) void quant_fwd_multi_kernel(QuantBatch b) {
    const hgq_quant_item it = b.item[blockIdx.y];
    const Mode m(it.mode);
    for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < it.n; t += (int64_t)gridDim.x * 256) {
        const KIF p = resolve_kif(load_k(it.k, t, m.k_u8), it.i[t], it.fb[t], m.kbi, m.round_params);
        it.y[t] = quantize_dyn(it.x[t], p, m.round_mode, m.overflow_mode, m.training);
    }
}

__global__ __launch_bounds__(256) void quant_bwd_multi_kernel(QuantGradBatch b) {
    const hgq_quant_grad_item it = b.item[blockIdx.y];
    const Mode m(it.mode);
    for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < it.n; t += (int64_t)gridDim.x * 256) {
        const KIF p = resolve_kif(load_k(it.k, t, m.k_u8), it.i[t], it.fb[t], m.kbi, m.round_params);
        float gx, gi, gf;
        quantize_grad_dyn(it.x[t], it.dy ? it.dy[t] : 0.0f, p, m.round_mode, m.overflow_mode, gx, gi, gf);
        if (m.kbi) gi -= gf;
        if (it.dx) it.dx[t] = gx;
        if (it.di) it.di[t] = gi;
        if (it.dfb) it.dfb[t] = gf;
    }
}

// ------------------------------------------------------------------------------------------
// Measurement aid: a plain streaming kernel with a chosen mix of read and written arrays (one 128-bit
// non-temporal access per array per thread, like the per-element quantizer kernels, and no arithmetic to speak
// of).  It calibrates the hardware traffic counters (known bytes) and gives the bandwidth this memory system
// yields for a given read / write mix and size, which is the ceiling the quantizer kernels are measured against.
// ------------------------------------------------------------------------------------------
template <int NR, int NW>
__global__ __launch_bounds__(Q1D_BS) void stream_probe_kernel(const f32x4 *__restrict__ a, const f32x4 *__restrict__ b,
                                                              const f32x4 *__restrict__ c, f32x4 *__restrict__ o0,
                                                              f32x4 *__restrict__ o1, f32x4 *__restrict__ o2,
                                                              f32x4 *__restrict__ o3, int64_t nvec) {
    const int64_t v = (int64_t)blockIdx.x * Q1D_BS + threadIdx.x;
    if (v >= nvec) return;
    f32x4 t = __builtin_nontemporal_load(a + v);
    if (NR > 1) t += __builtin_nontemporal_load(b + v);
    if (NR > 2) t += __builtin_nontemporal_load(c + v);
    __builtin_nontemporal_store(t, o0 + v);
    if (NW > 1) __builtin_nontemporal_store(t * 2.0f, o1 + v);
    if (NW > 2) __builtin_nontemporal_store(t * 3.0f, o2 + v);
    if (NW > 3) __builtin_nontemporal_store(t * 4.0f, o3 + v);
}

// ------------------------------------------------------------------------------------------
// integer-bit tracking
// ------------------------------------------------------------------------------------------
// 1024 threads = 64 entries x 16 slice groups: the abs-max / any-negative trackers arrive as
// `n_parts` slices of [n] (one per producing workgroup) and are combined here.
#define WT_G 16
__device__ __forceinline__ void wrap_track_body(const uint32_t *__restrict__ amax, const uint32_t *__restrict__ anyneg, int n_parts,
                                                float *i_var, const float *__restrict__ fb, uint8_t *k_var, int64_t n, float decay,
                                                float c_lo, float c_hi, int mode, int64_t block) {
    __shared__ uint32_t smax[64 * WT_G], sneg[64 * WT_G];
    const Mode m(mode);
    const int e_local = threadIdx.x & 63, grp = threadIdx.x >> 6;
    const int64_t t = block * 64 + e_local;
    uint32_t mx = 0, ng = 0;
    if (t < n) {
        const int per = (n_parts + WT_G - 1) / WT_G;
        const int g0 = grp * per, g1 = min(n_parts, g0 + per);
        int g = g0;
        for (; g + 8 <= g1; g += 8) {  // independent loads in flight
            uint32_t v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = amax[(int64_t)(g + u) * n + t];
#pragma unroll
            for (int u = 0; u < 8; ++u) mx = v[u] > mx ? v[u] : mx;
            if (anyneg) {
#pragma unroll
                for (int u = 0; u < 8; ++u) ng |= anyneg[(int64_t)(g + u) * n + t];
            }
        }
        for (; g < g1; ++g) {
            const uint32_t a = amax[(int64_t)g * n + t];
            mx = a > mx ? a : mx;
            if (anyneg) ng |= anyneg[(int64_t)g * n + t];
        }
    }
    smax[threadIdx.x] = mx, sneg[threadIdx.x] = ng;
    __syncthreads();
    if (grp != 0 || t >= n) return;
    for (int w = 1; w < WT_G; ++w) {
        const uint32_t a = smax[e_local + 64 * w];
        mx = a > mx ? a : mx;
        ng |= sneg[e_local + 64 * w];
    }
    const float xr = __uint_as_float(mx);
    const float raw_i = i_var[t];
    float mi;
    if (!m.kbi) {
        const float f = rintf(fb[t]);
        mi = ceil_log2_exact(__fadd_rn(xr, pow2(-f)));
    } else {
        const float b = rintf(fb[t]);
        const float eps = 1e-7f;
        const float num = __fadd_rn(xr, eps);
        const float den = __fadd_rn(__fsub_rn(1.0f, pow2(-b)), eps);
        mi = ceil_log2_exact(__fdiv_rn(num, den));  // exact: log2f is only faithfully rounded
        if (!m.symmetric && !(b > 0.0f)) mi = 32.0f;
    }
    float ni;
    if (!m.tracing) {
        ni = fmaxf(__fsub_rn(raw_i, decay), mi);
        if (m.kbi) ni = fminf(fmaxf(ni, c_lo), c_hi);
    } else {
        if (!m.kbi) {
            mi = fminf(fmaxf(mi, c_lo), c_hi);
            ni = fmaxf(rintf(raw_i), mi);
        } else {
            ni = fminf(fmaxf(fmaxf(rintf(raw_i), mi), c_lo), c_hi);
        }
        if (k_var && anyneg && ng) k_var[t] = 1;
    }
    i_var[t] = ni;
}

__global__ __launch_bounds__(64 * WT_G) void wrap_track_i_kernel(const uint32_t *__restrict__ amax,
                                                                 const uint32_t *__restrict__ anyneg, int n_parts,
                                                                 float *i_var, const float *__restrict__ fb, uint8_t *k_var,
                                                                 int64_t n, float decay, float c_lo, float c_hi, int mode) {
    wrap_track_body(amax, anyneg, n_parts, i_var, fb, k_var, n, decay, c_lo, c_hi, mode, blockIdx.x);
}

// The same update for several quantizers in one launch: block b serves the item whose block range holds b.
struct TrackBatch {
    hgq_track_item item[HGQ_TRACK_BATCH];
    int first_block[HGQ_TRACK_BATCH + 1];
    int count;
};

__global__ __launch_bounds__(64 * WT_G) void wrap_track_i_multi_kernel(const TrackBatch b) {
    int t = 0;
    while (t + 1 < b.count && (int)blockIdx.x >= b.first_block[t + 1]) ++t;
    const hgq_track_item &it = b.item[t];
    wrap_track_body(it.amax, it.anyneg, it.n_parts, it.i_var, it.fb, it.k_var, it.m, it.decay, it.c_lo, it.c_hi, it.mode,
                    (int)blockIdx.x - b.first_block[t]);
}

static inline bool aligned16(const void *p) { return ((uintptr_t)p & 15u) == 0; }

static inline int pow2_floor_le64(int64_t v) {
    int t = 1;
    while (t * 2 <= v && t < 64) t *= 2;
    return t;
}

}  // namespace hgq

using namespace hgq;

extern "C" int hgq_version(void) { return 1; }
extern "C" const char *hgq_last_error(void) { return g_err; }

extern "C" int hgq_stream_probe(const float *a, const float *b, const float *c, float *o0, float *o1, float *o2, float *o3,
                                int n_read, int n_write, int64_t n, void *stream) {
    if (n < 4 || n % 4 != 0 || n_read < 1 || n_read > 3 || n_write < 1 || n_write > 4)
        return fail(HGQ_ERR_ARG, "hgq_stream_probe: n must be a positive multiple of 4, 1..3 arrays read, 1..4 written");
    const float *in[3] = {a, b, c};
    float *out[4] = {o0, o1, o2, o3};
    for (int t = 0; t < 4; ++t)
        if ((t < n_read && (!in[t] || !aligned16(in[t]))) || (t < n_write && (!out[t] || !aligned16(out[t]))))
            return fail(HGQ_ERR_ARG, "hgq_stream_probe: arrays must be non-null and 16-byte aligned");
    const int64_t nvec = n / 4, grid = (nvec + Q1D_BS - 1) / Q1D_BS;
    if (grid >= (1ll << 31)) return fail(HGQ_ERR_ARG, "hgq_stream_probe: n too large");
    hipStream_t s = (hipStream_t)stream;
#define HGQ_PROBE(NRV, NWV)                                                                                                    \
    hipLaunchKernelGGL((stream_probe_kernel<NRV, NWV>), dim3((unsigned)grid), dim3(Q1D_BS), 0, s, (const f32x4 *)a, (const f32x4 *)b, \
                       (const f32x4 *)c, (f32x4 *)o0, (f32x4 *)o1, (f32x4 *)o2, (f32x4 *)o3, nvec)
    switch (n_read * 8 + n_write) {
        case 1 * 8 + 1: HGQ_PROBE(1, 1); break;
        case 1 * 8 + 2: HGQ_PROBE(1, 2); break;
        case 1 * 8 + 3: HGQ_PROBE(1, 3); break;
        case 1 * 8 + 4: HGQ_PROBE(1, 4); break;
        case 2 * 8 + 1: HGQ_PROBE(2, 1); break;
        case 2 * 8 + 2: HGQ_PROBE(2, 2); break;
        case 2 * 8 + 3: HGQ_PROBE(2, 3); break;
        case 2 * 8 + 4: HGQ_PROBE(2, 4); break;
        case 3 * 8 + 1: HGQ_PROBE(3, 1); break;
        case 3 * 8 + 2: HGQ_PROBE(3, 2); break;
        case 3 * 8 + 3: HGQ_PROBE(3, 3); break;
        default: HGQ_PROBE(3, 4); break;
    }
#undef HGQ_PROBE
    return check_launch("hgq_stream_probe");
}

extern "C" int hgq_fill_u32(uint32_t *p, uint32_t value, int64_t n, void *stream) {
    if (n < 0 || (n > 0 && !p)) return fail(HGQ_ERR_ARG, "hgq_fill_u32: bad arguments");
    return fill_u32(p, value, n, (hipStream_t)stream);
}

// Row split of the per-column kernels: about four workgroups per CU in total, every workgroup a
// whole number of row batches, and a chunk below 2 GiB (one buffer descriptor per workgroup).
static bool cols_grid(int64_t rows, int64_t M, int batch_rows, int64_t gx, int64_t &gy, int64_t &rows_per_wg) {
    const int64_t n_batches = (rows + batch_rows - 1) / batch_rows;
    int64_t want = (int64_t)persistent_grid(1 << 30, 4) / gx;
    if (want < 1) want = 1;
    gy = n_batches < want ? n_batches : want;
    if (gy < 1) gy = 1;
    int64_t bpw = (n_batches + gy - 1) / gy;                         // batches per workgroup
    const int64_t max_rows = ((1ll << 31) - 1) / (M * 4);             // rows in one descriptor
    if (max_rows < batch_rows) return false;  // absurdly wide rows: the generic kernel takes them
    if (bpw * batch_rows > max_rows) bpw = max_rows / batch_rows;
    rows_per_wg = bpw * batch_rows;
    gy = (rows + rows_per_wg - 1) / rows_per_wg;
    return true;
}

// Launches of the lean per-element kernels over n4 vectors (inside HGQ_DISPATCH_RM_OM: RM, OM, and the locals of the
// entry point).  Whole tiles of two vectors per lane first where that form pays (pe_two_vectors), then the remaining
// vectors - all of them for small inputs - one per thread.
#define HGQ_PE_SPLIT(TWO)                                                                                   \
    const int64_t pe_tiles = (TWO) ? n4 / (2 * Q1D_BS) : 0, pe_main = pe_tiles * 2 * Q1D_BS, pe_rest = n4 - pe_main, \
                  pe_rest_grid = (pe_rest + Q1D_BS - 1) / Q1D_BS
#define HGQ_FWD_PE(TRAINV, LIVEV)                                                                                                    \
    do {                                                                                                                              \
        if (pe_tiles > 0)                                                                                                             \
            hipLaunchKernelGGL((quant_fwd_pe<RM, OM, TRAINV, LIVEV, 2>), dim3((unsigned)pe_tiles), dim3(Q1D_BS), 0, s, (const f32x4 *)x, \
                               (const f32x4 *)k, (const f32x4 *)i, (const f32x4 *)fb, (f32x4 *)y, (int64_t)0, pe_main, (int)m.kbi);   \
        if (pe_rest > 0)                                                                                                              \
            hipLaunchKernelGGL((quant_fwd_pe<RM, OM, TRAINV, LIVEV, 1>), dim3((unsigned)pe_rest_grid), dim3(Q1D_BS), 0, s,            \
                               (const f32x4 *)x, (const f32x4 *)k, (const f32x4 *)i, (const f32x4 *)fb, (f32x4 *)y, pe_main, n4,      \
                               (int)m.kbi);                                                                                           \
    } while (0)
#define HGQ_BWD_PE(LIVEV)                                                                                                             \
    do {                                                                                                                              \
        if (pe_tiles > 0)                                                                                                             \
            hipLaunchKernelGGL((quant_bwd_pe<RM, OM, LIVEV, 2>), dim3((unsigned)pe_tiles), dim3(Q1D_BS), 0, s, (const f32x4 *)dy,     \
                               (const f32x4 *)x, (const f32x4 *)k, (const f32x4 *)i, (const f32x4 *)fb, (f32x4 *)dx, (f32x4 *)di,     \
                               (f32x4 *)dfb, (int64_t)0, pe_main, (int)m.kbi);                                                        \
        if (pe_rest > 0)                                                                                                              \
            hipLaunchKernelGGL((quant_bwd_pe<RM, OM, LIVEV, 1>), dim3((unsigned)pe_rest_grid), dim3(Q1D_BS), 0, s, (const f32x4 *)dy, \
                               (const f32x4 *)x, (const f32x4 *)k, (const f32x4 *)i, (const f32x4 *)fb, (f32x4 *)dx, (f32x4 *)di,     \
                               (f32x4 *)dfb, pe_main, n4, (int)m.kbi);                                                                \
    } while (0)
#define HGQ_FWD_BWD_PE(LIVEV)                                                                                                         \
    do {                                                                                                                              \
        if (pe_tiles > 0)                                                                                                             \
            hipLaunchKernelGGL((quant_fwd_bwd_pe<RM, OM, LIVEV, 2>), dim3((unsigned)pe_tiles), dim3(Q1D_BS), 0, s, (const f32x4 *)x,  \
                               (const f32x4 *)k, (const f32x4 *)i, (const f32x4 *)fb, (const f32x4 *)dy, (f32x4 *)y, (f32x4 *)dx,     \
                               (f32x4 *)di, (f32x4 *)dfb, (int64_t)0, pe_main, (int)m.kbi);                                           \
        if (pe_rest > 0)                                                                                                              \
            hipLaunchKernelGGL((quant_fwd_bwd_pe<RM, OM, LIVEV, 1>), dim3((unsigned)pe_rest_grid), dim3(Q1D_BS), 0, s,                \
                               (const f32x4 *)x, (const f32x4 *)k, (const f32x4 *)i, (const f32x4 *)fb, (const f32x4 *)dy,            \
                               (f32x4 *)y, (f32x4 *)dx, (f32x4 *)di, (f32x4 *)dfb, pe_main, n4, (int)m.kbi);                          \
    } while (0)

// Two vectors per lane pay where they put the whole input on the device in one round of workgroups, or nearly so, and one
// vector per thread would take two to three rounds: measured per size with both forms, the two-vector form is 10 - 17 %
// faster from one to two rounds' worth of vectors (2 Mi - 4 Mi elements on 256 CUs), within +-2 % up to three rounds, and
// 1 - 3 % slower beyond, where the rounds of the one-vector form no longer run in step anyway.  The forward alone has few
// streams and gains only from one and a half rounds on.
static bool pe_two_vectors(int64_t n4, bool many_streams) {
#ifdef HGQ_PE_FORCE_VECTORS
    return HGQ_PE_FORCE_VECTORS == 2;  // measurement builds only
#endif
    const int64_t one_round = (int64_t)persistent_grid(1ll << 40, 1) * 2048;  // threads the device holds at once
    return (many_streams ? n4 >= one_round : 2 * n4 >= 3 * one_round) && n4 <= 3 * one_round;
}

// launch of the per-column forward kernel: vector width and training flag as template arguments
#define HGQ_FWD_COLS_1(VECV, TRAINV, SLICED)                                                                                       \
    hipLaunchKernelGGL((quant_fwd_cols<RM, OM, VECV, TRAINV>), dim3((unsigned)gx, (unsigned)gy), dim3(256), 0, s, x, k, i, fb, y, \
                       amax, anyneg, rows, M, TX, rows_per_wg, mode, SLICED)
#define HGQ_FWD_COLS(SLICED)                                  \
    do {                                                      \
        if (vec && m.training) HGQ_FWD_COLS_1(4, true, SLICED);       \
        else if (vec) HGQ_FWD_COLS_1(4, false, SLICED);               \
        else if (m.training) HGQ_FWD_COLS_1(1, true, SLICED);         \
        else HGQ_FWD_COLS_1(1, false, SLICED);                        \
    } while (0)

extern "C" int hgq_quantize_fwd(const float *x, const void *k, const float *i, const float *fb, float *y,
                                uint32_t *amax, uint32_t *anyneg, int64_t n, int64_t bw_size, int64_t bw_inner,
                                int mode, void *stream) {
    hipStream_t s = (hipStream_t)stream;
    if (n < 0 || bw_size < 1 || bw_inner < 1) return fail(HGQ_ERR_ARG, "hgq_quantize_fwd: bad sizes");
    if (n == 0) return HGQ_OK;
    if (!x || !k || !i || !fb || !y) return fail(HGQ_ERR_ARG, "hgq_quantize_fwd: null pointer");
    if (bw_size * bw_inner > n || n % (bw_size * bw_inner) != 0)
        return fail(HGQ_ERR_ARG, "hgq_quantize_fwd: n=%lld is not a multiple of bw_size*bw_inner", (long long)n);
    const Mode m(mode);
    const bool reduce = bw_size < n;
    if (reduce) {
        int rc;
        if (amax && (rc = fill_u32(amax, 0, bw_size, s))) return rc;
        if (anyneg && (rc = fill_u32(anyneg, 0, bw_size, s))) return rc;
    }
    if (bw_size == n || bw_size == 1) {
        const bool shared = bw_size == 1 && n > 1;
        bool vec = aligned16(x) && aligned16(y) && n >= 4;
        if (!shared) vec = vec && aligned16(i) && aligned16(fb) && ((uintptr_t)k & (m.k_u8 ? 3u : 15u)) == 0 &&
                           (!amax || aligned16(amax)) && (!anyneg || aligned16(anyneg));
        const int64_t n4 = vec ? (n / 4) : 0;
        const int64_t tail0 = n4 * 4, tail = n - tail0;
        // the lean per-element kernel: no trackers, and k either dead or stored as fp32
        const bool k_dead = m.overflow_mode == HGQ_WRAP && m.training;
        const bool lean = !shared && n4 > 0 && !amax && !anyneg && !m.track_input && (k_dead || !m.k_u8) && n4 / Q1D_BS < (1ll << 30);
        HGQ_PE_SPLIT(lean && pe_two_vectors(n4, false));
        HGQ_DISPATCH_RM_OM(m.round_mode, m.overflow_mode, {
            if (lean) {
                if (OM == HGQ_WRAP && m.training) {
                    if (m.kbi) HGQ_FWD_PE(true, 1);
                    else HGQ_FWD_PE(true, 0);
                } else if (m.training) {
                    HGQ_FWD_PE(true, 3);
                } else {
                    HGQ_FWD_PE(false, 3);
                }
            } else if (n4 > 0) {
                const int grid = persistent_grid((n4 + Q1D_BS - 1) / Q1D_BS, 16);
                if (shared)
                    hipLaunchKernelGGL((quant_fwd_1d<RM, OM, 4, true>), dim3(grid), dim3(Q1D_BS), 0, s, x, k, i, fb, y, amax, anyneg, n4, mode);
                else
                    hipLaunchKernelGGL((quant_fwd_1d<RM, OM, 4, false>), dim3(grid), dim3(Q1D_BS), 0, s, x, k, i, fb, y, amax, anyneg, n4, mode);
            }
            if (tail > 0) {
                const int grid = 1;
                if (shared) {
                    hipLaunchKernelGGL((quant_fwd_1d<RM, OM, 1, true>), dim3(grid), dim3(Q1D_BS), 0, s, x + tail0, k, i, fb, y + tail0, amax, anyneg, tail, mode);
                } else {
                    const void *kt = m.k_u8 ? (const void *)((const uint8_t *)k + tail0) : (const void *)((const float *)k + tail0);
                    hipLaunchKernelGGL((quant_fwd_1d<RM, OM, 1, false>), dim3(grid), dim3(Q1D_BS), 0, s, x + tail0, kt, i + tail0, fb + tail0, y + tail0,
                                       amax ? amax + tail0 : nullptr, anyneg ? anyneg + tail0 : nullptr, tail, mode);
                }
            }
        });
        return check_launch("hgq_quantize_fwd");
    }
    if (bw_inner == 1 && bw_size * 4 * 256 * QC_U < (1ll << 31)) {
        const int64_t M = bw_size, rows = n / M;
        const bool vec = (M % 4 == 0) && aligned16(x) && aligned16(y) && aligned16(i) && aligned16(fb) &&
                         ((uintptr_t)k & (m.k_u8 ? 3u : 15u)) == 0;
        const int64_t cg = vec ? M / 4 : M;
        const int TX = pow2_floor_le64(cg), TY = 256 / TX;
        const int64_t gx = (cg + TX - 1) / TX;
        int64_t gy, rows_per_wg;
        cols_grid(rows, M, TY * QC_U, gx, gy, rows_per_wg);
        HGQ_DISPATCH_RM_OM(m.round_mode, m.overflow_mode, {
            HGQ_FWD_COLS(0);
        });
        return check_launch("hgq_quantize_fwd");
    }
    HGQ_DISPATCH_RM_OM(m.round_mode, m.overflow_mode, {
        const int grid = persistent_grid((n + 255) / 256, 8);
        hipLaunchKernelGGL((quant_fwd_generic<RM, OM>), dim3(grid), dim3(256), 0, s, x, k, i, fb, y, amax, anyneg, n, bw_size, bw_inner, mode);
    });
    return check_launch("hgq_quantize_fwd");
}

// Geometry of the per-column kernels for the sliced tracker form (16-byte aligned operands when bw_size is a multiple of 4).
static bool sliced_geometry(int64_t n, int64_t bw_size, int64_t bw_inner, bool &vec, int &TX, int64_t &gx, int64_t &gy, int64_t &rows_per_wg) {
    if (n < 1 || bw_size < 1 || bw_inner != 1 || bw_size >= n || n % bw_size != 0 || bw_size * 4 * 256 * QC_U >= (1ll << 31)) return false;
    vec = bw_size % 4 == 0;
    const int64_t cg = vec ? bw_size / 4 : bw_size;
    TX = pow2_floor_le64(cg);
    gx = (cg + TX - 1) / TX;
    return cols_grid(n / bw_size, bw_size, (256 / TX) * QC_U, gx, gy, rows_per_wg);
}

extern "C" int64_t hgq_quantize_tracker_slices(int64_t n, int64_t bw_size, int64_t bw_inner) {
    bool vec;
    int TX;
    int64_t gx, gy, rows_per_wg;
    return sliced_geometry(n, bw_size, bw_inner, vec, TX, gx, gy, rows_per_wg) ? gy : 0;
}

extern "C" int hgq_quantize_fwd_sliced(const float *x, const void *k, const float *i, const float *fb, float *y, uint32_t *amax,
                                       uint32_t *anyneg, int64_t n_slices, int64_t n, int64_t bw_size, int64_t bw_inner, int mode,
                                       void *stream) {
    hipStream_t s = (hipStream_t)stream;
    bool vec;
    int TX;
    int64_t gx, gy, rows_per_wg;
    if (!sliced_geometry(n, bw_size, bw_inner, vec, TX, gx, gy, rows_per_wg) || gy != n_slices)
        return fail(HGQ_ERR_ARG, "hgq_quantize_fwd_sliced: n_slices must be hgq_quantize_tracker_slices(n, bw_size, bw_inner) > 0");
    if (!x || !k || !i || !fb || !y) return fail(HGQ_ERR_ARG, "hgq_quantize_fwd_sliced: null pointer");
    const Mode m(mode);
    if (vec && !(aligned16(x) && aligned16(y) && aligned16(i) && aligned16(fb) && ((uintptr_t)k & (m.k_u8 ? 3u : 15u)) == 0))
        return fail(HGQ_ERR_ARG, "hgq_quantize_fwd_sliced: operands must be 16-byte aligned when bw_size is a multiple of 4");
    const int64_t M = bw_size, rows = n / M;
    HGQ_DISPATCH_RM_OM(m.round_mode, m.overflow_mode, {
        HGQ_FWD_COLS(1);
    });
    return check_launch("hgq_quantize_fwd_sliced");
}

static unsigned multi_grid_x(int64_t max_n) {
    int64_t gx = (max_n + 1023) / 1024;
    return (unsigned)(gx < 1 ? 1 : (gx > 256 ? 256 : gx));
}

extern "C" int hgq_quantize_fwd_multi(const hgq_quant_item *items, int count, void *stream) {
    if (count < 0 || (count > 0 && !items)) return fail(HGQ_ERR_ARG, "hgq_quantize_fwd_multi: bad arguments");
    for (int base = 0; base < count; base += HGQ_QUANT_BATCH) {
        QuantBatch b;
        const int nb = count - base < HGQ_QUANT_BATCH ? count - base : HGQ_QUANT_BATCH;
        int64_t max_n = 0;
        for (int t = 0; t < nb; ++t) {
            b.item[t] = items[base + t];
            const hgq_quant_item &it = b.item[t];
            if (it.n < 0 || (it.n > 0 && (!it.x || !it.k || !it.i || !it.fb || !it.y)))
                return fail(HGQ_ERR_ARG, "hgq_quantize_fwd_multi: bad item %d", base + t);
            if (it.n > max_n) max_n = it.n;
        }
        if (max_n == 0) continue;
        hipLaunchKernelGGL(quant_fwd_multi_kernel, dim3(multi_grid_x(max_n), (unsigned)nb), dim3(256), 0, (hipStream_t)stream, b);
        int rc = check_launch("hgq_quantize_fwd_multi");
        if (rc) return rc;
    }
    return HGQ_OK;
}

extern "C" int hgq_quantize_bwd_multi(const hgq_quant_grad_item *items, int count, void *stream) {
    if (count < 0 || (count > 0 && !items)) return fail(HGQ_ERR_ARG, "hgq_quantize_bwd_multi: bad arguments");
    for (int base = 0; base < count; base += HGQ_QUANT_BATCH) {
        QuantGradBatch b;
        const int nb = count - base < HGQ_QUANT_BATCH ? count - base : HGQ_QUANT_BATCH;
        int64_t max_n = 0;
        for (int t = 0; t < nb; ++t) {
            b.item[t] = items[base + t];
            const hgq_quant_grad_item &it = b.item[t];
            if (it.n < 0 || (it.n > 0 && (!it.x || !it.k || !it.i || !it.fb)))
                return fail(HGQ_ERR_ARG, "hgq_quantize_bwd_multi: bad item %d", base + t);
            if (!Mode(it.mode).training)
                return fail(HGQ_ERR_ARG, "hgq_quantize_bwd_multi: item %d: the surrogate gradient is defined for training mode only", base + t);
            if (it.n > max_n) max_n = it.n;
        }
        if (max_n == 0) continue;
        hipLaunchKernelGGL(quant_bwd_multi_kernel, dim3(multi_grid_x(max_n), (unsigned)nb), dim3(256), 0, (hipStream_t)stream, b);
        int rc = check_launch("hgq_quantize_bwd_multi");
        if (rc) return rc;
    }
    return HGQ_OK;
}

// Geometry of the per-column backward for the sliced form of the bit-width gradients.
static bool sliced_bwd_geometry(int64_t n, int64_t bw_size, int64_t bw_inner, bool &vec, int &TX, int64_t &gx, int64_t &gy, int64_t &rows_per_wg) {
    if (n < 1 || bw_size < 2 || bw_inner != 1 || bw_size >= n || n % bw_size != 0 || bw_size * 4 * 256 * QC_U >= (1ll << 31)) return false;
    vec = bw_size % 4 == 0;
    const int64_t cg = vec ? bw_size / 4 : bw_size;
    TX = pow2_floor_le64(cg);
    gx = (cg + TX - 1) / TX;
    return cols_grid(n / bw_size, bw_size, (256 / TX) * QC_BWD_U, gx, gy, rows_per_wg);
}

extern "C" int64_t hgq_quantize_bwd_workspace(int64_t n, int64_t bw_size, int64_t bw_inner) {
    bool vec;
    int TX;
    int64_t gx, gy, rows_per_wg;
    return sliced_bwd_geometry(n, bw_size, bw_inner, vec, TX, gx, gy, rows_per_wg) ? gy * 2 * bw_size : 0;
}

extern "C" int64_t hgq_quantize_bwd_slice_count(int64_t n, int64_t bw_size, int64_t bw_inner) {
    bool vec;
    int TX;
    int64_t gx, gy, rows_per_wg;
    return sliced_bwd_geometry(n, bw_size, bw_inner, vec, TX, gx, gy, rows_per_wg) ? gy : 0;
}

static int quantize_bwd_sliced_impl(const float *dy, const float *x, const void *k, const float *i, const float *fb, float *dx,
                                    float *di, float *dfb, float *workspace, int64_t n, int64_t bw_size, int64_t bw_inner,
                                    int mode, void *stream, bool reduce);

extern "C" int hgq_quantize_bwd_sliced(const float *dy, const float *x, const void *k, const float *i, const float *fb, float *dx,
                                       float *di, float *dfb, float *workspace, int64_t n, int64_t bw_size, int64_t bw_inner,
                                       int mode, void *stream) {
    return quantize_bwd_sliced_impl(dy, x, k, i, fb, dx, di, dfb, workspace, n, bw_size, bw_inner, mode, stream, true);
}

extern "C" int hgq_quantize_bwd_slices(const float *dy, const float *x, const void *k, const float *i, const float *fb, float *dx,
                                       int want_di, float *workspace, int64_t n, int64_t bw_size, int64_t bw_inner, int mode,
                                       void *stream) {
    // the kernel takes the two gradient pointers only as "wanted" flags when it writes slices
    return quantize_bwd_sliced_impl(dy, x, k, i, fb, dx, want_di ? workspace : nullptr, workspace, workspace, n, bw_size, bw_inner, mode,
                                    stream, false);
}

static int quantize_bwd_sliced_impl(const float *dy, const float *x, const void *k, const float *i, const float *fb, float *dx,
                                    float *di, float *dfb, float *workspace, int64_t n, int64_t bw_size, int64_t bw_inner,
                                    int mode, void *stream, bool reduce) {
    hipStream_t s = (hipStream_t)stream;
    bool vec;
    int TX;
    int64_t gx, gy, rows_per_wg;
    if (!sliced_bwd_geometry(n, bw_size, bw_inner, vec, TX, gx, gy, rows_per_wg))
        return fail(HGQ_ERR_UNSUPPORTED, "hgq_quantize_bwd_sliced: shape outside the per-column kernels (hgq_quantize_bwd_workspace returns 0 for it)");
    if (!dy || !x || !k || !i || !fb || !dfb || !workspace) return fail(HGQ_ERR_ARG, "hgq_quantize_bwd_sliced: null pointer");
    const Mode m(mode);
    if (!m.training) return fail(HGQ_ERR_ARG, "hgq_quantize_bwd_sliced: the surrogate gradient is defined for training mode only");
    if (vec && !(aligned16(x) && aligned16(dy) && (!dx || aligned16(dx)) && aligned16(i) && aligned16(fb) &&
                 ((uintptr_t)k & (m.k_u8 ? 3u : 15u)) == 0))
        return fail(HGQ_ERR_ARG, "hgq_quantize_bwd_sliced: operands must be 16-byte aligned when bw_size is a multiple of 4");
    const int64_t M = bw_size, rows = n / M;
    HGQ_DISPATCH_RM_OM(m.round_mode, m.overflow_mode, {
        if (vec)
            hipLaunchKernelGGL((quant_bwd_cols<RM, OM, 4>), dim3((unsigned)gx, (unsigned)gy), dim3(256), 0, s, dy, x, k, i, fb, dx, di, dfb, rows, M, TX, rows_per_wg, mode, workspace);
        else
            hipLaunchKernelGGL((quant_bwd_cols<RM, OM, 1>), dim3((unsigned)gx, (unsigned)gy), dim3(256), 0, s, dy, x, k, i, fb, dx, di, dfb, rows, M, TX, rows_per_wg, mode, workspace);
    });
    int rc = check_launch("hgq_quantize_bwd_sliced");
    if (rc || !reduce) return rc;
    return reduce_parts(workspace, (int)gy, di ? 2 * M : M, dfb, M, di, di ? M : 0, nullptr, 0, s);
}

// ------------------------------------------------------------------------------------------
// hgq_quantize_bwd_sliced for callers that cannot allocate: the slices live in a file-scope device array.
// Every GPU the library runs on holds its own copy of the array (HGQ_STATIC_SCRATCH_FLOATS * 4 bytes) until the
// process ends.  In host code the array's NAME is only a handle for hipGetSymbolAddress: the device address is looked
// up once per device and only that pointer is ever handed to a kernel.
// ------------------------------------------------------------------------------------------
static __device__ __align__(256) float scratch[HGQ_STATIC_SCRATCH_FLOATS];

#define HGQ_MAX_DEVICES 64
static std::mutex g_scratch_mutex;
static float *g_scratch_ptr[HGQ_MAX_DEVICES];  // per device: each GPU has the array at its own address

static int static_scratch(float **out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(HGQ_ERR_LAUNCH, "hgq_quantize_bwd_static: hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= HGQ_MAX_DEVICES) return fail(HGQ_ERR_UNSUPPORTED, "hgq_quantize_bwd_static: device index %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));  // with device `dev` current: its copy of the array
        if (e != hipSuccess || !p) return fail(HGQ_ERR_LAUNCH, "hgq_quantize_bwd_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
        g_scratch_ptr[dev] = (float *)p;
    }
    *out = g_scratch_ptr[dev];
    return HGQ_OK;
}

extern "C" int hgq_quantize_bwd_static(const float *dy, const float *x, const void *k, const float *i, const float *fb, float *dx,
                                       float *di, float *dfb, int64_t n, int64_t bw_size, int64_t bw_inner, int mode, void *stream) {
    const int64_t need = hgq_quantize_bwd_workspace(n, bw_size, bw_inner);
    if (need <= 0)
        return fail(HGQ_ERR_UNSUPPORTED, "hgq_quantize_bwd_static: shape outside the per-column kernels (hgq_quantize_bwd_workspace returns 0 for it)");
    if (need > (int64_t)HGQ_STATIC_SCRATCH_FLOATS)
        return fail(HGQ_ERR_ARG, "hgq_quantize_bwd_static: %lld floats of slices needed, the static scratch holds %lld; use hgq_quantize_bwd_sliced with a caller workspace",
                    (long long)need, (long long)HGQ_STATIC_SCRATCH_FLOATS);
    float *ws = nullptr;
    const int rc = static_scratch(&ws);
    if (rc) return rc;
    // every slice entry that the reduction reads is written whole by the kernel before: nothing to clear between calls
    return hgq_quantize_bwd_sliced(dy, x, k, i, fb, dx, di, dfb, ws, n, bw_size, bw_inner, mode, stream);
}

extern "C" int hgq_quantize_bwd(const float *dy, const float *x, const void *k, const float *i, const float *fb,
                                float *dx, float *di, float *dfb, int64_t n, int64_t bw_size, int64_t bw_inner,
                                int mode, void *stream) {
    hipStream_t s = (hipStream_t)stream;
    if (n < 0 || bw_size < 1 || bw_inner < 1) return fail(HGQ_ERR_ARG, "hgq_quantize_bwd: bad sizes");
    if (n == 0) return HGQ_OK;
    if (!dy || !x || !k || !i || !fb) return fail(HGQ_ERR_ARG, "hgq_quantize_bwd: null pointer");
    if (bw_size * bw_inner > n || n % (bw_size * bw_inner) != 0)
        return fail(HGQ_ERR_ARG, "hgq_quantize_bwd: n=%lld is not a multiple of bw_size*bw_inner", (long long)n);
    const Mode m(mode);
    if (!m.training) return fail(HGQ_ERR_ARG, "hgq_quantize_bwd: the surrogate gradient is defined for training mode only");
    if (bw_size < n) {
        int rc;
        if (di && (rc = fill_f32(di, 0.0f, bw_size, s))) return rc;
        if (dfb && (rc = fill_f32(dfb, 0.0f, bw_size, s))) return rc;
    }
    if (bw_size == n || bw_size == 1) {
        const bool shared = bw_size == 1 && n > 1;
        bool vec = aligned16(x) && aligned16(dy) && (!dx || aligned16(dx)) && n >= 4;
        if (!shared) vec = vec && aligned16(i) && aligned16(fb) && ((uintptr_t)k & (m.k_u8 ? 3u : 15u)) == 0 &&
                           (!di || aligned16(di)) && (!dfb || aligned16(dfb));
        const int64_t n4 = vec ? (n / 4) : 0;
        const int64_t tail0 = n4 * 4, tail = n - tail0;
        const bool k_dead = m.overflow_mode == HGQ_WRAP;  // the WRAP surrogate gradient only rounds
        const bool lean = !shared && n4 > 0 && (k_dead || !m.k_u8) && n4 / Q1D_BS < (1ll << 30);
        HGQ_PE_SPLIT(lean && pe_two_vectors(n4, true));
        HGQ_DISPATCH_RM_OM(m.round_mode, m.overflow_mode, {
            if (lean) {
                if (OM == HGQ_WRAP) {
                    if (m.kbi) HGQ_BWD_PE(1);
                    else HGQ_BWD_PE(0);
                } else {
                    HGQ_BWD_PE(3);
                }
            } else if (n4 > 0) {
                const int grid = persistent_grid((n4 + Q1D_BS - 1) / Q1D_BS, 16);
                if (shared)
                    hipLaunchKernelGGL((quant_bwd_1d<RM, OM, 4, true>), dim3(grid), dim3(Q1D_BS), 0, s, dy, x, k, i, fb, dx, di, dfb, n4, mode);
                else
                    hipLaunchKernelGGL((quant_bwd_1d<RM, OM, 4, false>), dim3(grid), dim3(Q1D_BS), 0, s, dy, x, k, i, fb, dx, di, dfb, n4, mode);
            }
            if (tail > 0) {
                const int grid = 1;
                if (shared) {
                    hipLaunchKernelGGL((quant_bwd_1d<RM, OM, 1, true>), dim3(grid), dim3(Q1D_BS), 0, s, dy + tail0, x + tail0, k, i, fb,
                                       dx ? dx + tail0 : nullptr, di, dfb, tail, mode);
                } else {
                    const void *kt = m.k_u8 ? (const void *)((const uint8_t *)k + tail0) : (const void *)((const float *)k + tail0);
                    hipLaunchKernelGGL((quant_bwd_1d<RM, OM, 1, false>), dim3(grid), dim3(Q1D_BS), 0, s, dy + tail0, x + tail0, kt, i + tail0, fb + tail0,
                                       dx ? dx + tail0 : nullptr, di ? di + tail0 : nullptr, dfb ? dfb + tail0 : nullptr, tail, mode);
                }
            }
        });
        return check_launch("hgq_quantize_bwd");
    }
    if (bw_inner == 1 && bw_size * 4 * 256 * QC_U < (1ll << 31)) {
        const int64_t M = bw_size, rows = n / M;
        const bool vec = (M % 4 == 0) && aligned16(x) && aligned16(dy) && (!dx || aligned16(dx)) && aligned16(i) &&
                         aligned16(fb) && ((uintptr_t)k & (m.k_u8 ? 3u : 15u)) == 0;
        const int64_t cg = vec ? M / 4 : M;
        const int TX = pow2_floor_le64(cg), TY = 256 / TX;
        const int64_t gx = (cg + TX - 1) / TX;
        int64_t gy, rows_per_wg;
        cols_grid(rows, M, TY * QC_BWD_U, gx, gy, rows_per_wg);
        HGQ_DISPATCH_RM_OM(m.round_mode, m.overflow_mode, {
            if (vec)
                hipLaunchKernelGGL((quant_bwd_cols<RM, OM, 4>), dim3((unsigned)gx, (unsigned)gy), dim3(256), 0, s, dy, x, k, i, fb, dx, di, dfb, rows, M, TX, rows_per_wg, mode, (float *)nullptr);
            else
                hipLaunchKernelGGL((quant_bwd_cols<RM, OM, 1>), dim3((unsigned)gx, (unsigned)gy), dim3(256), 0, s, dy, x, k, i, fb, dx, di, dfb, rows, M, TX, rows_per_wg, mode, (float *)nullptr);
        });
        return check_launch("hgq_quantize_bwd");
    }
    HGQ_DISPATCH_RM_OM(m.round_mode, m.overflow_mode, {
        const int grid = persistent_grid((n + 255) / 256, 8);
        hipLaunchKernelGGL((quant_bwd_generic<RM, OM>), dim3(grid), dim3(256), 0, s, dy, x, k, i, fb, dx, di, dfb, n, bw_size, bw_inner, mode);
    });
    return check_launch("hgq_quantize_bwd");
}

extern "C" int hgq_quantize_fwd_bwd(const float *x, const void *k, const float *i, const float *fb, const float *dy, float *y,
                                    float *dx, float *di, float *dfb, int64_t n, int64_t bw_size, int64_t bw_inner, int mode,
                                    void *stream) {
    hipStream_t s = (hipStream_t)stream;
    if (n < 0 || bw_size < 1 || bw_inner < 1) return fail(HGQ_ERR_ARG, "hgq_quantize_fwd_bwd: bad sizes");
    if (n == 0) return HGQ_OK;
    if (!x || !k || !i || !fb || !dy || !y) return fail(HGQ_ERR_ARG, "hgq_quantize_fwd_bwd: null pointer");
    if (bw_size * bw_inner > n || n % (bw_size * bw_inner) != 0)
        return fail(HGQ_ERR_ARG, "hgq_quantize_fwd_bwd: n=%lld is not a multiple of bw_size*bw_inner", (long long)n);
    const Mode m(mode);
    if (!m.training) return fail(HGQ_ERR_ARG, "hgq_quantize_fwd_bwd: the surrogate gradient is defined for training mode only");
    if (m.track_input) return fail(HGQ_ERR_ARG, "hgq_quantize_fwd_bwd: no trackers here; HGQ_MODE_TRACK_INPUT has no meaning");
    const bool k_dead = m.overflow_mode == HGQ_WRAP;  // a WRAP quantizer in training mode only rounds
    const bool all16 = aligned16(x) && aligned16(i) && aligned16(fb) && aligned16(dy) && aligned16(y) && (!dx || aligned16(dx)) &&
                       (!di || aligned16(di)) && (!dfb || aligned16(dfb)) && (k_dead || (!m.k_u8 && aligned16(k)));
    const int64_t n4 = n / 4;
    if (bw_size == n && n4 > 0 && all16 && n4 / Q1D_BS < (1ll << 30)) {
        const int64_t tail0 = n4 * 4, tail = n - tail0;
        HGQ_PE_SPLIT(pe_two_vectors(n4, true));
        HGQ_DISPATCH_RM_OM(m.round_mode, m.overflow_mode, {
            if (OM == HGQ_WRAP) {
                if (m.kbi) HGQ_FWD_BWD_PE(1);
                else HGQ_FWD_BWD_PE(0);
            } else {
                HGQ_FWD_BWD_PE(3);
            }
        });
        int rc = check_launch("hgq_quantize_fwd_bwd");
        if (rc || tail == 0) return rc;
        // up to three trailing elements: the general kernels, one workgroup each
        const void *kt = m.k_u8 ? (const void *)((const uint8_t *)k + tail0) : (const void *)((const float *)k + tail0);
        if ((rc = hgq_quantize_fwd(x + tail0, kt, i + tail0, fb + tail0, y + tail0, nullptr, nullptr, tail, tail, 1, mode, stream))) return rc;
        return hgq_quantize_bwd(dy + tail0, x + tail0, kt, i + tail0, fb + tail0, dx ? dx + tail0 : nullptr, di ? di + tail0 : nullptr,
                                dfb ? dfb + tail0 : nullptr, tail, tail, 1, mode, stream);
    }
    // shared or per-column bit-widths, uint8 k with a live k, unaligned operands: the two separate passes
    int rc = hgq_quantize_fwd(x, k, i, fb, y, nullptr, nullptr, n, bw_size, bw_inner, mode, stream);
    if (rc) return rc;
    return hgq_quantize_bwd(dy, x, k, i, fb, dx, di, dfb, n, bw_size, bw_inner, mode, stream);
}

extern "C" int hgq_wrap_track_i(const uint32_t *amax, const uint32_t *anyneg, int n_parts, float *i_var, const float *fb,
                                uint8_t *k_var, int64_t m, float decay, float c_lo, float c_hi, int mode, void *stream) {
    if (m < 0 || n_parts < 1) return fail(HGQ_ERR_ARG, "hgq_wrap_track_i: bad size");
    if (m == 0) return HGQ_OK;
    if (!amax || !i_var || !fb) return fail(HGQ_ERR_ARG, "hgq_wrap_track_i: null pointer");
    hipLaunchKernelGGL(wrap_track_i_kernel, dim3((unsigned)((m + 63) / 64)), dim3(64 * WT_G), 0, (hipStream_t)stream, amax, anyneg, n_parts,
                       i_var, fb, k_var, m, decay, c_lo, c_hi, mode);
    return check_launch("hgq_wrap_track_i");
}

extern "C" int hgq_wrap_track_i_multi(const hgq_track_item *items, int count, void *stream) {
    if (count < 0 || (count > 0 && !items)) return fail(HGQ_ERR_ARG, "hgq_wrap_track_i_multi: bad arguments");
    for (int base = 0; base < count; base += HGQ_TRACK_BATCH) {
        TrackBatch b;
        b.count = 0;
        int64_t blocks = 0;
        const int nb = count - base < HGQ_TRACK_BATCH ? count - base : HGQ_TRACK_BATCH;
        for (int t = 0; t < nb; ++t) {
            const hgq_track_item &it = items[base + t];
            if (it.m < 0 || it.n_parts < 1) return fail(HGQ_ERR_ARG, "hgq_wrap_track_i_multi: bad size in item %d", base + t);
            if (it.m == 0) continue;
            if (!it.amax || !it.i_var || !it.fb) return fail(HGQ_ERR_ARG, "hgq_wrap_track_i_multi: null pointer in item %d", base + t);
            // the items of one launch run concurrently: two updates of one variable would race
            for (int u = 0; u < b.count; ++u)
                if (b.item[u].i_var == it.i_var)
                    return fail(HGQ_ERR_ARG, "hgq_wrap_track_i_multi: items %d and an earlier one update the same variable; pass them in separate calls", base + t);
            b.item[b.count] = it;
            b.first_block[b.count++] = (int)blocks;
            blocks += (it.m + 63) / 64;
            if (blocks > (1 << 24)) return fail(HGQ_ERR_UNSUPPORTED, "hgq_wrap_track_i_multi: too many entries");
        }
        if (b.count == 0) continue;
        for (int t = b.count; t <= HGQ_TRACK_BATCH; ++t) b.first_block[t] = (int)blocks;
        hipLaunchKernelGGL(wrap_track_i_multi_kernel, dim3((unsigned)blocks), dim3(64 * WT_G), 0, (hipStream_t)stream, b);
        int rc = check_launch("hgq_wrap_track_i_multi");
        if (rc) return rc;
    }
    return HGQ_OK;
}
