// QDense / QEinsumDense contraction on quantized operands for gfx950.
//
// Forward: the input tile is quantized while it is staged into LDS (quantize-on-load), the
// quantized kernel tile sits next to it, and fp32 MFMA (v_mfma_f32_32x32x2f32) does the
// contraction; bias and activation are applied in the accumulator registers.  The abs-max the
// WRAP input quantizer tracks is reduced in LDS and flushed once per workgroup.
//
// Backward (K, N <= 64): one pass over (dy, y, x) produces dx, the kernel / bias gradients and
// the input quantizer's fractional-bit gradient.  Per-workgroup partial sums of the kernel
// gradient stay in MFMA accumulators across the grid-stride loop and are flushed with one
// coalesced atomic add per accumulator register at the end.
//
// MFMA 32x32x2 fp32 operand layout (64 lanes): A[i][k]: i = lane % 32, k = lane / 32;
// B[k][j]: k = lane / 32, j = lane % 32; D[i][j] in 16 registers: j = lane % 32,
// i = (r / 4) * 8 + (lane / 32) * 4 + (r % 4).
#include "hgq_device.h"
#include "hgq_host.h"

namespace hgq {

typedef float floatx16 __attribute__((ext_vector_type(16)));

#define FWD_BM 128
#define FWD_BK 32
#define FWD_BN 64
#define AMAX_LDS_MAX 8192

__device__ __forceinline__ int acc_row(int r, int lane) { return (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3); }

template <int RM, int OM, bool QUANT>
__global__ __launch_bounds__(256) void qdense_fwd_kernel(const float *__restrict__ x, const void *__restrict__ k_in,
                                                         const float *__restrict__ i_in, const float *__restrict__ f_in,
                                                         int64_t P, const float *__restrict__ qw,
                                                         const float *__restrict__ qb, float *__restrict__ y,
                                                         uint32_t *amax, int64_t rows, int K, int N, int act, int mode,
                                                         int vec_ok, int amax_lds) {
    __shared__ float xs[FWD_BM][FWD_BK + 1];
    __shared__ float ws[FWD_BK][FWD_BN];
    extern __shared__ uint32_t amax_s[];  // [P*K] when amax_lds

    const Mode m(mode);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n0 = blockIdx.y * FWD_BN;
    const int nw = min(FWD_BN, N - n0);
    const int64_t n_tiles = (rows + FWD_BM - 1) / FWD_BM;
    const int64_t PK = P * (int64_t)K;
    const bool track = QUANT && amax != nullptr && blockIdx.y == 0;

    if (track && amax_lds)
        for (int64_t t = tid; t < PK; t += 256) amax_s[t] = 0;
    __syncthreads();

    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const int64_t r0 = tile * FWD_BM;
        floatx16 acc0 = {0}, acc1 = {0};
        for (int k0 = 0; k0 < K; k0 += FWD_BK) {
            const int kw = min(FWD_BK, K - k0);
            // ---- stage the (quantized) input tile
            if (vec_ok) {
                const int kw4 = kw >> 2;
                for (int id = tid; id < FWD_BM * kw4; id += 256) {
                    const int row = id / kw4, c = (id - row * kw4) << 2;
                    const int64_t gr = r0 + row;
                    float v[4] = {0.f, 0.f, 0.f, 0.f};
                    if (gr < rows) {
                        const float4 t = *(const float4 *)(x + gr * K + k0 + c);
                        v[0] = t.x, v[1] = t.y, v[2] = t.z, v[3] = t.w;
                        if (QUANT) {
                            const int64_t b = (gr % P) * K + k0 + c;
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                const KIF p = resolve_kif(load_k(k_in, b + e, m.k_u8), i_in[b + e], f_in[b + e], m.kbi, m.round_params);
                                v[e] = quantize<RM, OM>(v[e], p, m.training);
                                if (track) {
                                    if (amax_lds) atomicMax(&amax_s[b + e], abs_bits(v[e]));
                                    else atomicMax(&amax[b + e], abs_bits(v[e]));
                                }
                            }
                        }
                    }
#pragma unroll
                    for (int e = 0; e < 4; ++e) xs[row][c + e] = v[e];
                }
            } else {
                for (int id = tid; id < FWD_BM * kw; id += 256) {
                    const int row = id / kw, c = id - row * kw;
                    const int64_t gr = r0 + row;
                    float v = 0.f;
                    if (gr < rows) {
                        v = x[gr * K + k0 + c];
                        if (QUANT) {
                            const int64_t b = (gr % P) * K + k0 + c;
                            const KIF p = resolve_kif(load_k(k_in, b, m.k_u8), i_in[b], f_in[b], m.kbi, m.round_params);
                            v = quantize<RM, OM>(v, p, m.training);
                            if (track) {
                                if (amax_lds) atomicMax(&amax_s[b], abs_bits(v));
                                else atomicMax(&amax[b], abs_bits(v));
                            }
                        }
                    }
                    xs[row][c] = v;
                }
            }
            if (kw < FWD_BK) {
                const int pad = FWD_BK - kw;
                for (int id = tid; id < FWD_BM * pad; id += 256) xs[id / pad][kw + id % pad] = 0.f;
            }
            // ---- stage the kernel tile [BK, BN], zero padded
            for (int id = tid; id < FWD_BK * FWD_BN; id += 256) {
                const int kk = id / FWD_BN, nn = id - kk * FWD_BN;
                ws[kk][nn] = (kk < kw && nn < nw) ? qw[(int64_t)(k0 + kk) * N + n0 + nn] : 0.f;
            }
            __syncthreads();
            const int ksteps = (kw + 1) & ~1;
            const int arow = wave * 32 + (lane & 31), kq = lane >> 5, bcol = lane & 31;
            if (nw > 32) {
                for (int kk = 0; kk < ksteps; kk += 2) {
                    const float a = xs[arow][kk + kq];
                    acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, ws[kk + kq][bcol], acc0, 0, 0, 0);
                    acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, ws[kk + kq][32 + bcol], acc1, 0, 0, 0);
                }
            } else {
                for (int kk = 0; kk < ksteps; kk += 2)
                    acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(xs[arow][kk + kq], ws[kk + kq][bcol], acc0, 0, 0, 0);
            }
            __syncthreads();
        }
        // ---- epilogue: bias, activation, store
        const int col = lane & 31;
#pragma unroll
        for (int blk = 0; blk < 2; ++blk) {
            const int n = n0 + blk * 32 + col;
            if (blk * 32 >= nw || n >= N) continue;
            const float bias = qb ? qb[n] : 0.f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int64_t gr = r0 + wave * 32 + acc_row(r, lane);
                if (gr < rows) {
                    float v = (blk == 0 ? acc0[r] : acc1[r]) + bias;
                    if (act == HGQ_ACT_RELU) v = v > 0.f ? v : 0.f;
                    y[gr * N + n] = v;
                }
            }
        }
    }
    if (track && amax_lds) {
        __syncthreads();
        for (int64_t t = tid; t < PK; t += 256) {
            const uint32_t v = amax_s[t];
            if (v) atomicMax(&amax[t], v);
        }
    }
}

// ------------------------------------------------------------------------------------------
// backward, K <= 64 and N <= 64
// ------------------------------------------------------------------------------------------
#define BWD_BM 64
#define BWD_LD 65
#define DF_LDS_MAX 4096

template <int RM, bool QUANT>
__global__ __launch_bounds__(256) void qdense_bwd_kernel(const float *__restrict__ dy, const float *__restrict__ y,
                                                         const float *__restrict__ x, const float *__restrict__ f_in,
                                                         int64_t P, const float *__restrict__ qw, float *__restrict__ dx,
                                                         float *dqw, float *dqb, float *df_in, int64_t rows, int K, int N,
                                                         int act, int mode, int df_lds) {
    __shared__ float xs[BWD_BM][BWD_LD];   // quantized input tile
    __shared__ float dzs[BWD_BM][BWD_LD];  // gradient at the pre-activation
    __shared__ float ws[64][BWD_LD];       // quantized kernel, zero padded to 64 x 64
    __shared__ float bred[256];
    extern __shared__ float df_s[];  // [P*K] when df_lds

    const Mode m(mode);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int K32 = (K + 31) >> 5, N32 = (N + 31) >> 5;
    const int64_t PK = P * (int64_t)K;
    const int64_t n_tiles = (rows + BWD_BM - 1) / BWD_BM;
    const bool want_df = QUANT && df_in != nullptr;

    for (int id = tid; id < 64 * 64; id += 256) {
        const int kk = id >> 6, nn = id & 63;
        ws[kk][nn] = (kk < K && nn < N) ? qw[(int64_t)kk * N + nn] : 0.f;
    }
    if (want_df && df_lds)
        for (int64_t t = tid; t < PK; t += 256) df_s[t] = 0.f;

    // kernel-gradient block owned by this wave
    const int nblk = K32 * N32;        // 1, 2 or 4 blocks of 32 x 32
    const int wpb = 4 / nblk;          // waves sharing one block
    const int blk = wave / wpb, sub = wave % wpb;
    const int wkb = blk / N32, wnb = blk % N32;
    const int rows_per = BWD_BM / wpb;
    floatx16 accw = {0};
    float accb = 0.f;
    const int bn = tid & 63, bq = tid >> 6;  // bias column / row quarter

    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const int64_t r0 = tile * BWD_BM;
        __syncthreads();  // previous tile fully consumed (and ws / df_s initialised)
        for (int id = tid; id < BWD_BM * 64; id += 256) {
            const int row = id >> 6, c = id & 63;
            const int64_t gr = r0 + row;
            float dz = 0.f, xv = 0.f;
            if (gr < rows) {
                if (c < N) {
                    dz = dy[gr * N + c];
                    if (act == HGQ_ACT_RELU && !(y[gr * N + c] > 0.f)) dz = 0.f;
                }
                if (c < K) {
                    xv = x[gr * K + c];
                    if (QUANT) xv = fixed_round<RM>(xv, m.round_params ? rintf(f_in[(gr % P) * K + c]) : f_in[(gr % P) * K + c]);
                }
            }
            dzs[row][c] = dz;
            xs[row][c] = xv;
        }
        __syncthreads();
        // ---- dx = dz @ qW^T : blocks (row half, k block)
        {
            const int rh = wave & 1, kb = wave >> 1;
            if (kb < K32) {
                floatx16 acc = {0};
                const int arow = rh * 32 + (lane & 31), kq = lane >> 5, wrow = kb * 32 + (lane & 31);
                const int nsteps = N32 * 32;
                for (int nn = 0; nn < nsteps; nn += 2)
                    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(dzs[arow][nn + kq], ws[wrow][nn + kq], acc, 0, 0, 0);
                const int kcol = kb * 32 + (lane & 31);
                float dfsum = 0.f;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int row = rh * 32 + acc_row(r, lane);
                    const int64_t gr = r0 + row;
                    if (gr < rows && kcol < K) {
                        dx[gr * K + kcol] = acc[r];
                        if (want_df) {
                            const float delta = xs[row][kcol] - x[gr * K + kcol];
                            const float g = -HGQ_LN2 * delta * acc[r];
                            if (P == 1) dfsum += g;
                            else if (df_lds) atomicAdd(&df_s[(gr % P) * K + kcol], g);
                            else atomicAdd(&df_in[(gr % P) * K + kcol], g);
                        }
                    }
                }
                if (want_df && P == 1) {
                    dfsum += __shfl_xor(dfsum, 32, 64);
                    if (lane < 32 && kcol < K) {
                        if (df_lds) atomicAdd(&df_s[kcol], dfsum);
                        else atomicAdd(&df_in[kcol], dfsum);
                    }
                }
            }
        }
        // ---- dW += rx^T @ dz : this wave's block, its slice of the tile's rows
        if (dqw) {
            const int rbeg = sub * rows_per;
            const int kq = lane >> 5, c32 = lane & 31;
            for (int rr = rbeg; rr < rbeg + rows_per; rr += 2)
                accw = __builtin_amdgcn_mfma_f32_32x32x2f32(xs[rr + kq][wkb * 32 + c32], dzs[rr + kq][wnb * 32 + c32], accw, 0, 0, 0);
        }
        // ---- bias gradient partial sums
        if (dqb) {
#pragma unroll
            for (int j = 0; j < BWD_BM / 4; ++j) accb += dzs[bq * (BWD_BM / 4) + j][bn];
        }
    }
    // ---- flush
    if (dqw) {
        const int n = wnb * 32 + (lane & 31);
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int k = wkb * 32 + acc_row(r, lane);
            if (k < K && n < N) atomicAdd(&dqw[(int64_t)k * N + n], accw[r]);
        }
    }
    if (dqb) {
        bred[tid] = accb;
        __syncthreads();
        if (tid < 64 && tid < N) atomicAdd(&dqb[tid], bred[tid] + bred[tid + 64] + bred[tid + 128] + bred[tid + 192]);
    }
    if (want_df && df_lds) {
        __syncthreads();
        for (int64_t t = tid; t < PK; t += 256) {
            const float v = df_s[t];
            if (v != 0.f) atomicAdd(&df_in[t], v);
        }
    }
}

static inline bool aligned16(const void *p) { return ((uintptr_t)p & 15u) == 0; }

}  // namespace hgq

using namespace hgq;

extern "C" int hgq_qdense_fwd(const float *x, const void *k_in, const float *i_in, const float *f_in, int64_t bw_rows,
                              const float *qw, const float *qb, float *y, uint32_t *amax, int64_t rows, int K, int N,
                              int act, int mode, void *stream) {
    hipStream_t s = (hipStream_t)stream;
    if (rows < 0 || K < 1 || N < 1 || bw_rows < 0) return fail(HGQ_ERR_ARG, "hgq_qdense_fwd: bad sizes");
    if (rows == 0) return HGQ_OK;
    if (!x || !qw || !y) return fail(HGQ_ERR_ARG, "hgq_qdense_fwd: null pointer");
    if (bw_rows > 0 && (!k_in || !i_in || !f_in)) return fail(HGQ_ERR_ARG, "hgq_qdense_fwd: null bit-width pointer");
    if (act != HGQ_ACT_NONE && act != HGQ_ACT_RELU) return fail(HGQ_ERR_ARG, "hgq_qdense_fwd: unknown activation %d", act);
    if (bw_rows > 0 && rows % bw_rows != 0) return fail(HGQ_ERR_ARG, "hgq_qdense_fwd: rows=%lld not a multiple of bw_rows=%lld", (long long)rows, (long long)bw_rows);
    const Mode m(mode);
    const int64_t PK = bw_rows * (int64_t)K;
    const bool quant = bw_rows > 0;
    int rc;
    if (quant && amax && (rc = fill_u32(amax, 0, PK, s))) return rc;
    const int amax_lds = (quant && amax && PK <= AMAX_LDS_MAX) ? 1 : 0;
    const size_t dyn = amax_lds ? (size_t)PK * 4 : 0;
    const int vec_ok = (K % 4 == 0) && aligned16(x);
    const int64_t n_tiles = (rows + FWD_BM - 1) / FWD_BM;
    const dim3 grid((unsigned)persistent_grid(n_tiles, 4), (unsigned)((N + FWD_BN - 1) / FWD_BN));
    if (!quant) {
        hipLaunchKernelGGL((qdense_fwd_kernel<HGQ_TRN, HGQ_WRAP, false>), grid, dim3(256), dyn, s, x, k_in, i_in, f_in, (int64_t)1, qw, qb, y,
                           amax, rows, K, N, act, mode, vec_ok, amax_lds);
    } else {
        HGQ_DISPATCH_RM_OM(m.round_mode, m.overflow_mode, {
            hipLaunchKernelGGL((qdense_fwd_kernel<RM, OM, true>), grid, dim3(256), dyn, s, x, k_in, i_in, f_in, bw_rows, qw, qb, y, amax, rows,
                               K, N, act, mode, vec_ok, amax_lds);
        });
    }
    return check_launch("hgq_qdense_fwd");
}

extern "C" int hgq_qdense_bwd(const float *dy, const float *y, const float *x, const float *f_in, int64_t bw_rows,
                              const float *qw, float *dx, float *dqw, float *dqb, float *df_in, int64_t rows, int K,
                              int N, int act, int mode, void *stream) {
    hipStream_t s = (hipStream_t)stream;
    if (rows < 0 || K < 1 || N < 1 || bw_rows < 0) return fail(HGQ_ERR_ARG, "hgq_qdense_bwd: bad sizes");
    if (K > 64 || N > 64) return fail(HGQ_ERR_UNSUPPORTED, "hgq_qdense_bwd: K=%d N=%d exceed the fused kernel's 64 x 64", K, N);
    if (!dy || !x || !qw || !dx) return fail(HGQ_ERR_ARG, "hgq_qdense_bwd: null pointer");
    if (act == HGQ_ACT_RELU && !y) return fail(HGQ_ERR_ARG, "hgq_qdense_bwd: relu needs the forward output");
    if (act != HGQ_ACT_NONE && act != HGQ_ACT_RELU) return fail(HGQ_ERR_ARG, "hgq_qdense_bwd: unknown activation %d", act);
    const Mode m(mode);
    const bool quant = bw_rows > 0;
    if (quant && !(m.overflow_mode == HGQ_WRAP && m.training))
        return fail(HGQ_ERR_UNSUPPORTED, "hgq_qdense_bwd: the fused input quantizer must be a training-mode WRAP quantizer");
    if (quant && !f_in) return fail(HGQ_ERR_ARG, "hgq_qdense_bwd: null bit-width pointer");
    if (quant && rows % bw_rows != 0) return fail(HGQ_ERR_ARG, "hgq_qdense_bwd: rows not a multiple of bw_rows");
    const int64_t PK = bw_rows * (int64_t)K;
    int rc;
    if (dqw && (rc = fill_f32(dqw, 0.f, (int64_t)K * N, s))) return rc;
    if (dqb && (rc = fill_f32(dqb, 0.f, N, s))) return rc;
    if (quant && df_in && (rc = fill_f32(df_in, 0.f, PK, s))) return rc;
    if (rows == 0) return HGQ_OK;
    const int df_lds = (quant && df_in && PK <= DF_LDS_MAX) ? 1 : 0;
    const size_t dyn = df_lds ? (size_t)PK * 4 : 0;
    const int64_t n_tiles = (rows + BWD_BM - 1) / BWD_BM;
    const dim3 grid((unsigned)persistent_grid(n_tiles, 3));
    typedef void (*bwd_fn)(const float *, const float *, const float *, const float *, int64_t, const float *, float *, float *,
                           float *, float *, int64_t, int, int, int, int, int);
    bwd_fn fn = nullptr;
    if (!quant) fn = qdense_bwd_kernel<HGQ_TRN, false>;
    else if (m.round_mode == HGQ_TRN) fn = qdense_bwd_kernel<HGQ_TRN, true>;
    else if (m.round_mode == HGQ_RND) fn = qdense_bwd_kernel<HGQ_RND, true>;
    else if (m.round_mode == HGQ_RND_CONV) fn = qdense_bwd_kernel<HGQ_RND_CONV, true>;
    else return fail(HGQ_ERR_ARG, "hgq_qdense_bwd: unknown round mode");
    if (dyn > 8192) {
        // static LDS is ~50 KB; ask once per kernel for the part of the 160 KB LDS beyond the default 64 KB window
        static const void *raised[8] = {nullptr};
        bool done = false;
        int slot = -1;
        for (int t = 0; t < 8; ++t) {
            if (raised[t] == (const void *)fn) done = true;
            if (raised[t] == nullptr && slot < 0) slot = t;
        }
        if (!done) {
            hipError_t e = hipFuncSetAttribute((const void *)fn, hipFuncAttributeMaxDynamicSharedMemorySize, DF_LDS_MAX * 4);
            if (e != hipSuccess) return fail(HGQ_ERR_LAUNCH, "hgq_qdense_bwd: hipFuncSetAttribute: %s", hipGetErrorString(e));
            if (slot >= 0) raised[slot] = (const void *)fn;
        }
    }
    hipLaunchKernelGGL(fn, grid, dim3(256), dyn, s, dy, y, x, f_in, quant ? bw_rows : (int64_t)1, qw, dx, dqw, dqb, df_in, rows, K, N, act,
                       mode, df_lds);
    return check_launch("hgq_qdense_bwd");
}
