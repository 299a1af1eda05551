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


#define FWD_BM 64
#define FWD_BK 32
#define FWD_BN 64
#define AMAX_LDS_MAX 8192
#define MAX_PARTS 512

__device__ __forceinline__ int acc_row(int r, int lane) { return (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3); }

// Workgroup `g` of the row grid owns slice `g` of `amax_part` ([gridDim.x, P*K]): no atomics
// between workgroups, no clearing pass; the integer-bit tracking kernel reduces over the slices.
template <int RM, int OM, bool QUANT>
__global__ __launch_bounds__(256) void qdense_fwd_kernel(const float *__restrict__ x, const void *__restrict__ k_in,
                                                         const float *__restrict__ i_in, const float *__restrict__ f_in,
                                                         int64_t P, const float *__restrict__ qw,
                                                         const float *__restrict__ qb, float *__restrict__ y,
                                                         uint32_t *amax_part, int64_t rows, int K, int N, int act,
                                                         int mode, int vec_ok, int amax_lds) {
    __shared__ float xs[FWD_BM][FWD_BK + 1];
    __shared__ float ws[FWD_BK][FWD_BN];
    extern __shared__ uint32_t amax_s[];  // [P*K] when amax_lds

    const Mode m(mode);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int rh = wave & 1, cb = wave >> 1;  // this wave's 32 x 32 output block of the 64 x 64 tile
    const int n0 = blockIdx.y * FWD_BN;
    const int nw = min(FWD_BN, N - n0);
    const int64_t n_tiles = (rows + FWD_BM - 1) / FWD_BM;
    const int64_t PK = P * (int64_t)K;
    const bool track = QUANT && amax_part != nullptr && blockIdx.y == 0;
    uint32_t *my_amax = track ? amax_part + (int64_t)blockIdx.x * PK : nullptr;

    if (track) {
        if (amax_lds) for (int64_t t = tid; t < PK; t += 256) amax_s[t] = 0;
        else for (int64_t t = tid; t < PK; t += 256) my_amax[t] = 0;
        __threadfence_block();
    }
    __syncthreads();

    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const int64_t r0 = tile * FWD_BM;
        floatx16 acc = {0};
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
                                if (track && P > 1) atomicMax(amax_lds ? &amax_s[b + e] : &my_amax[b + e], abs_bits(v[e]));
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
                            if (track && P > 1) atomicMax(amax_lds ? &amax_s[b] : &my_amax[b], abs_bits(v));
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
            // one bit-width entry per column: column maxima straight from the staged tile
            // (rows past the end were staged as zero, which never raises a maximum)
            if (track && P == 1 && tid < kw) {
                uint32_t mx = 0;
#pragma unroll 8
                for (int r = 0; r < FWD_BM; ++r) {
                    const uint32_t a = abs_bits(xs[r][tid]);
                    mx = a > mx ? a : mx;
                }
                uint32_t *dst = amax_lds ? &amax_s[k0 + tid] : &my_amax[k0 + tid];
                if (mx > *dst) *dst = mx;
            }
            if (cb * 32 < nw) {
                const int ksteps = (kw + 1) & ~1;
                const int arow = rh * 32 + (lane & 31), kq = lane >> 5, bcol = cb * 32 + (lane & 31);
                for (int kk = 0; kk < ksteps; kk += 2)
                    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(xs[arow][kk + kq], ws[kk + kq][bcol], acc, 0, 0, 0);
            }
            __syncthreads();
        }
        // ---- epilogue: bias, activation, store
        const int n = n0 + cb * 32 + (lane & 31);
        if (cb * 32 < nw && n < N) {
            const float bias = qb ? qb[n] : 0.f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int64_t gr = r0 + rh * 32 + acc_row(r, lane);
                if (gr < rows) {
                    float v = acc[r] + bias;
                    if (act == HGQ_ACT_RELU) v = v > 0.f ? v : 0.f;
                    y[gr * N + n] = v;
                }
            }
        }
    }
    if (track && amax_lds) {
        __syncthreads();
        for (int64_t t = tid; t < PK; t += 256) my_amax[t] = amax_s[t];
    }
}

// ------------------------------------------------------------------------------------------
// backward, K <= 64 and N <= 64
// ------------------------------------------------------------------------------------------
#define BWD_BM 64
#define BWD_LD 65
#define DF_LDS_MAX 4096

// Workgroup `g` accumulates its share of the kernel / bias / fractional-bit gradients over the
// tiles it walks and writes them to slice `g` of `part` ([gridDim.x, K*N + N + P*K]); a second
// small kernel sums the slices in a fixed order, so the result is deterministic and no floating
// point atomics are used.
template <int RM, bool QUANT>
__global__ __launch_bounds__(256) void qdense_bwd_kernel(const float *__restrict__ dy, const float *__restrict__ y,
                                                         const float *__restrict__ x, const float *__restrict__ f_in,
                                                         int64_t P, const float *__restrict__ qw, float *__restrict__ dx,
                                                         float *part, int has_bias, int64_t rows, int K, int N, int act,
                                                         int mode, int df_lds) {
    __shared__ float xs[BWD_BM][BWD_LD];   // quantized input tile
    __shared__ float dzs[BWD_BM][BWD_LD];  // gradient at the pre-activation
    __shared__ float ws[64][BWD_LD];       // quantized kernel, zero padded to 64 x 64
    __shared__ float bred[256];
    extern __shared__ float df_s[];  // [P*K] when df_lds

    const Mode m(mode);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int K32 = (K + 31) >> 5, N32 = (N + 31) >> 5;
    const int64_t PK = QUANT ? P * (int64_t)K : 0;
    const int64_t M = (int64_t)K * N + N + PK;
    const int64_t n_tiles = (rows + BWD_BM - 1) / BWD_BM;
    float *my_dw = part + (int64_t)blockIdx.x * M;
    float *my_db = my_dw + (int64_t)K * N;
    float *my_df = my_db + N;

    for (int id = tid; id < 64 * 64; id += 256) {
        const int kk = id >> 6, nn = id & 63;
        ws[kk][nn] = (kk < K && nn < N) ? qw[(int64_t)kk * N + nn] : 0.f;
    }
    if (QUANT) {
        if (df_lds) for (int64_t t = tid; t < PK; t += 256) df_s[t] = 0.f;
        else for (int64_t t = tid; t < PK; t += 256) my_df[t] = 0.f;
        __threadfence_block();
    }

    // kernel-gradient block owned by this wave
    const int nblk = K32 * N32;        // 1, 2 or 4 blocks of 32 x 32
    const int wpb = 4 / nblk;          // waves sharing one block
    const int blk = wave / wpb, sub = wave % wpb;
    const int wkb = blk / N32, wnb = blk % N32;
    const int rows_per = BWD_BM / wpb;
    floatx16 accw = {0}, acc2 = {0};  // acc2: the second block of a wavefront with PAIRS
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
                        if (QUANT) {
                            const float delta = xs[row][kcol] - x[gr * K + kcol];
                            const float g = -HGQ_LN2 * delta * acc[r];
                            if (P == 1) dfsum += g;
                            else atomicAdd(df_lds ? &df_s[(gr % P) * K + kcol] : &my_df[(gr % P) * K + kcol], g);
                        }
                    }
                }
                if (QUANT && P == 1) {
                    dfsum += __shfl_xor(dfsum, 32, 64);
                    if (lane < 32 && kcol < K) atomicAdd(df_lds ? &df_s[kcol] : &my_df[kcol], dfsum);
                }
            }
        }
        // ---- dW += rx^T @ dz : this wave's block, its slice of the tile's rows
        {
            const int rbeg = sub * rows_per;
            const int kq = lane >> 5, c32 = lane & 31;
            accw = mfma_chain(accw, &xs[rbeg + kq][wkb * 32 + c32], BWD_LD, &dzs[rbeg + kq][wnb * 32 + c32], BWD_LD, rows_per / 16);
        }
        // ---- bias gradient partial sums
        if (has_bias) {
#pragma unroll
            for (int j = 0; j < BWD_BM / 4; ++j) accb += dzs[bq * (BWD_BM / 4) + j][bn];
        }
    }
    // ---- write this workgroup's slice.  Waves sharing a kernel-gradient block combine through LDS.
    __syncthreads();
    float *comb = &xs[0][0];  // 64 x 65 floats, free now
    for (int pass = 0; pass < wpb; ++pass) {
        if (sub == pass) {
            const int n = wnb * 32 + (lane & 31);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int k = wkb * 32 + acc_row(r, lane);
                if (pass == 0) comb[k * BWD_LD + n] = accw[r];
                else comb[k * BWD_LD + n] += accw[r];
            }
        }
        __syncthreads();
    }
    for (int id = tid; id < K * N; id += 256) my_dw[id] = comb[(id / N) * BWD_LD + (id % N)];
    bred[tid] = accb;
    __syncthreads();
    if (tid < N) my_db[tid] = has_bias ? bred[tid] + bred[tid + 64] + bred[tid + 128] + bred[tid + 192] : 0.f;
    if (QUANT && df_lds)
        for (int64_t t = tid; t < PK; t += 256) my_df[t] = df_s[t];
}

// ------------------------------------------------------------------------------------------
// streaming variants for the common case: K, N <= 64, K a multiple of 4, the input quantizer (if
// any) on its WRAP training branch (round only) with a bit-width table whose row count divides 64
// ------------------------------------------------------------------------------------------
// A tile is 64 rows, so the table row of a staged element, (tile row) % P, is the same in every
// tile: a thread keeps the fractional bits and the abs-max / gradient accumulators of the elements
// it stages in registers for the whole launch.  The next tile's global loads are issued before
// the current tile's MFMAs, and the staged tile is double buffered (one barrier per tile).
#define FAST_BM 64
#define FAST_LD 65
#define FAST_NJ 4  // 128-bit loads per thread and tile: 64 * K / 4 / 256 <= 4

struct FastMap {
    int row[FAST_NJ], col[FAST_NJ];
    bool on[FAST_NJ];
    __device__ __forceinline__ void init(int W) {  // W = row width in floats, a multiple of 4, at most 64
        const int w4 = W >> 2;
        // id / w4 for id < 1024, w4 <= 16 by a 16-bit reciprocal (exact: id * (ceil(2^16 / w4) - 2^16 / w4) < 2^16 / w4)
        const uint32_t rcp = (65536u + (uint32_t)w4 - 1u) / (uint32_t)w4;
#pragma unroll
        for (int j = 0; j < FAST_NJ; ++j) {
            const int id = threadIdx.x + 256 * j;
            on[j] = id < FAST_BM * w4;
            row[j] = on[j] ? (int)(((uint32_t)id * rcp) >> 16) : 0;
            col[j] = on[j] ? (id - row[j] * w4) << 2 : 0;
        }
    }
};

// Fractional bits of the elements a thread stages, fi[j][e], from the [P, K] table (P a power of two); tix[j] is the
// table entry of slot j's first element.  Every load is issued before any is waited for (a load inside a branch is
// waited for where it is issued, one memory latency per element).
template <bool QUANT>
__device__ __forceinline__ void fast_frac_bits(const float *f_in, int P, int K, const FastMap &mp, bool round_params,
                                               int (&fi)[FAST_NJ][4], int (&tix)[FAST_NJ]) {
    const __amdgpu_buffer_rsrc_t rs_f = buf_rsrc(f_in, QUANT ? (int64_t)P * K * 4 : 0);
    float fv[FAST_NJ][4];
#pragma unroll
    for (int j = 0; j < FAST_NJ; ++j) {
        tix[j] = (mp.row[j] & (P - 1)) * K + mp.col[j];
#pragma unroll
        for (int e = 0; e < 4; ++e) fv[j][e] = QUANT ? buf_ld1(rs_f, mp.on[j] ? (uint32_t)(tix[j] + e) * 4u : BUF_OOB) : 0.f;
    }
#pragma unroll
    for (int j = 0; j < FAST_NJ; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e) fi[j][e] = (int)(round_params ? rintf(fv[j][e]) : fv[j][e]);
}

__device__ __forceinline__ void st4(float *p, const float4 &v) {
    f32x4_t t;
    t.x = v.x, t.y = v.y, t.z = v.z, t.w = v.w;
    *(f32x4_t *)p = t;
}

// Forward.  The kernel matrix never touches LDS: lane (j, h) of a wavefront keeps the 32 entries
// W[2 s + h][column j] it multiplies by in registers for the whole launch.  The input tile sits
// in LDS with its columns permuted (even k first, then odd k) so that the 32 operands of a lane,
// x[row][2 s + h], s = 0 .. 31, are contiguous and are read four at a time; rows are 68 words
// apart, which keeps those 128-bit reads free of bank conflicts.  The output tile goes back
// through LDS so that it leaves as full 128-bit rows.
#define FAST_XLD 68
template <int RM, bool QUANT, int NS4>
__global__ __launch_bounds__(256, 2) void qdense_fwd_fast_kernel(const float *__restrict__ x, const float *__restrict__ f_in,
                                                              int P, const float *__restrict__ qw,
                                                              const float *__restrict__ qb, float *__restrict__ y,
                                                              uint32_t *amax_part, int64_t rows, int K, int N, int act,
                                                              int mode) {
    __shared__ __attribute__((aligned(16))) float xs[2][FAST_BM + 1][FAST_XLD];  // row FAST_BM: sink of the idle staging slots
    __shared__ __attribute__((aligned(16))) float ys[FAST_BM][FAST_XLD];
    const Mode m(mode);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int rh = wave & 1, cb = wave >> 1;
    const int64_t n_tiles = (rows + FAST_BM - 1) / FAST_BM;
    for (int id = tid; id < 2 * (FAST_BM + 1) * FAST_XLD; id += 256) (&xs[0][0][0])[id] = 0.f;  // columns >= K stay zero
    const int arow = rh * 32 + (lane & 31), kq = lane >> 5, bcol = cb * 32 + (lane & 31);
    float wreg[4 * NS4];
#pragma unroll
    for (int sidx = 0; sidx < 4 * NS4; ++sidx) {
        const int k = 2 * sidx + kq;
        wreg[sidx] = (k < K && bcol < N) ? qw[(int64_t)k * N + bcol] : 0.f;
    }
    const float bias = (qb && bcol < N) ? qb[bcol] : 0.f;
    FastMap mp, mo;
    mp.init(K);
    const bool vec_out = (N & 3) == 0 && ((uintptr_t)y & 15u) == 0;
    mo.init(vec_out ? N : 4);
    int fi[FAST_NJ][4], tix[FAST_NJ];
    uint32_t amx[FAST_NJ][4];
    fast_frac_bits<QUANT>(f_in, P, K, mp, m.round_params, fi, tix);
#pragma unroll
    for (int j = 0; j < FAST_NJ; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e) amx[j][e] = 0;
    f32x4_t raw[FAST_NJ];
    uint32_t xoff[FAST_NJ];
#pragma unroll
    for (int j = 0; j < FAST_NJ; ++j) xoff[j] = mp.on[j] ? (uint32_t)(mp.row[j] * K + mp.col[j]) * 4u : BUF_OOB;
    // the descriptor covers the valid rows of one tile: rows past the end read as zero
    auto load_tile = [&](int64_t t) {
        const int64_t r0 = t * FAST_BM, left = rows - r0;
        const __amdgpu_buffer_rsrc_t rs = buf_rsrc(x + r0 * K, (left < FAST_BM ? left : FAST_BM) * K * 4);
#pragma unroll
        for (int j = 0; j < FAST_NJ; ++j) raw[j] = buf_ld4(rs, xoff[j]);
    };
    int64_t tile = blockIdx.x;
    if (tile < n_tiles) load_tile(tile);
    __syncthreads();
    // everything loaded so far (kernel entries, bit-widths) has arrived: no wait on them inside the loop
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    int buf = 0;
    for (; tile < n_tiles; tile += gridDim.x, buf ^= 1) {
        // no branch around a staging slot (a wait inside one would cover every load): idle slots
        // hold zeros and write them to the sink row
#pragma unroll
        for (int j = 0; j < FAST_NJ; ++j) {
            float v[4] = {raw[j][0], raw[j][1], raw[j][2], raw[j][3]};
            if (QUANT) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    v[e] = ldexpf(round_scaled<RM>(ldexpf(v[e], fi[j][e])), -fi[j][e]);
                    amx[j][e] = max(amx[j][e], abs_bits(v[e]));
                }
            }
            // columns k0 .. k0 + 3 -> even ones at k0 / 2, odd ones at 32 + k0 / 2
            float *dst = &xs[buf][mp.on[j] ? mp.row[j] : FAST_BM][mp.col[j] >> 1];
            *(float2 *)dst = make_float2(v[0], v[2]);
            *(float2 *)(dst + 32) = make_float2(v[1], v[3]);
        }
        __syncthreads();
        const int64_t next = tile + gridDim.x;
        if (next < n_tiles) load_tile(next);
        floatx16 acc = {0};
        if (cb * 32 < N) {
            const float *arow_p = &xs[buf][arow][kq * 32];
            // NS4 groups of four k pairs cover K (columns past K are zero on both sides)
            f32x4_t a4[NS4];
#pragma unroll
            for (int s4 = 0; s4 < NS4; ++s4) a4[s4] = *(const f32x4_t *)(arow_p + 4 * s4);
            // the reads stay ahead of the chain (rescheduled, they would share registers and wait for the instructions in between)
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int s4 = 0; s4 < NS4; ++s4)
#pragma unroll
                for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a4[s4][e], wreg[4 * s4 + e], acc, 0, 0, 0);
        }
        const int64_t r0 = tile * FAST_BM;
        if (vec_out) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                float v = acc[r] + bias;
                if (act == HGQ_ACT_RELU) v = v > 0.f ? v : 0.f;
                ys[rh * 32 + acc_row(r, lane)][bcol] = v;
            }
            __syncthreads();
#pragma unroll
            for (int j = 0; j < FAST_NJ; ++j) {
                const int64_t gr = r0 + mo.row[j];
                if (mo.on[j] && gr < rows) {
                    *(f32x4_t *)(y + gr * N + mo.col[j]) = *(const f32x4_t *)&ys[mo.row[j]][mo.col[j]];
                }
            }
        } else if (bcol < N) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int64_t gr = r0 + rh * 32 + acc_row(r, lane);
                if (gr < rows) {
                    float v = acc[r] + bias;
                    if (act == HGQ_ACT_RELU) v = v > 0.f ? v : 0.f;
                    y[gr * N + bcol] = v;
                }
            }
        }
    }
    if (QUANT && amax_part && P == FAST_BM && ((uintptr_t)amax_part & 15u) == 0) {
        // one table row per tile row: every entry of this workgroup's slice has exactly one owner thread
        uint32_t *my = amax_part + (int64_t)blockIdx.x * (P * K);
#pragma unroll
        for (int j = 0; j < FAST_NJ; ++j)
            if (mp.on[j]) {
                uint4 v;
                v.x = amx[j][0], v.y = amx[j][1], v.z = amx[j][2], v.w = amx[j][3];
                *(uint4 *)(my + tix[j]) = v;
            }
    } else if (QUANT && amax_part) {
        // this workgroup's slice: combine the registers of all threads through an LDS table
        const int PK = P * K;
        uint32_t *tab = (uint32_t *)&xs[0][0][0];
        __syncthreads();
        for (int t = tid; t < PK; t += 256) tab[t] = 0;
        __syncthreads();
#pragma unroll
        for (int j = 0; j < FAST_NJ; ++j)
            if (mp.on[j])
#pragma unroll
                for (int e = 0; e < 4; ++e) atomicMax(&tab[tix[j] + e], amx[j][e]);
        __syncthreads();
        uint32_t *my = amax_part + (int64_t)blockIdx.x * PK;
        for (int t = tid; t < PK; t += 256) my[t] = tab[t];
    }
}

// ------------------------------------------------------------------------------------------
// The same contraction on the bf16 matrix cores, exactly.  An fp32 number is the sum of three numbers
// of eight significant bits each - its leading bits, the leading bits of what is left, and the rest -
// and each of them is a bf16 number (same exponent range as fp32).  A product of two such parts is
// exact in fp32, so  x W = sum over part pairs  x_p W_q  accumulated in fp32 is the contraction itself,
// with only the accumulation rounded, as in the fp32 matrix instruction.  v_mfma_f32_32x32x16_bf16 does
// sixteen times the work of v_mfma_f32_32x32x2_f32 per cycle, so even all nine pairs cost about half of
// the fp32 chain - and quantized operands rarely need more than one part (eight bits) or two (sixteen):
// the staging threads note which parts of a tile are non-zero, a wavefront notes it for its kernel
// columns, and only those pairs are issued.
// Operand layout of the 32x32x16 instruction (64 lanes, eight bf16 per lane and operand):
// A[i][k]: i = lane % 32, k = 8 (lane / 32) + e;  B[k][j]: k = 8 (lane / 32) + e, j = lane % 32;  D as for 32x32x2.
// ------------------------------------------------------------------------------------------
// Time stamps of workgroup 0 (measurement builds only: -DDB_PROF): [kernel: 0 forward, 1 backward, 2 statistics' backward][wavefront][event],
// in ticks of the constant-rate counter
#ifdef DB_PROF
__device__ unsigned long long db_prof_stamps[3 * 4 * 32];
#define DB_STAMP(k, i)                                                                                                  \
    do {                                                                                                                \
        if (blockIdx.x == 0 && (threadIdx.x & 63) == 0 && (i) < 32)                                                     \
            db_prof_stamps[((k) * 4 + (threadIdx.x >> 6)) * 32 + (i)] = wall_clock64();                                 \
    } while (0)
#else
#define DB_STAMP(k, i)
#endif

#define BF_LD 72  // bf16 per LDS row: rows 144 bytes apart keep the 128-bit operand reads of 16 consecutive rows on different banks

typedef uint16_t (*bf16_planes_t)[FAST_BM + 1][BF_LD];  // [part][row][k] of one staged tile

// Stages the four 128-bit slots of a thread (quantized first when QUANT) as bf16 parts and records in `need` which of
// the second / third parts of the tile are non-zero (bit 0 / 1).  TRACK: the abs-max of the staged values.
// Four small integers (fractional bits: clamped to a signed byte) in one register.
__device__ __forceinline__ int pack_i8x4(const int (&v)[4]) {
    int r = 0;
#pragma unroll
    for (int e = 0; e < 4; ++e) r |= (max(-128, min(127, v[e])) & 0xff) << (8 * e);
    return r;
}
__device__ __forceinline__ int unpack_i8(int packed, int e) { return (int)(int8_t)((packed >> (8 * e)) & 0xff); }

template <int RM, bool QUANT, bool TRACK>
__device__ __forceinline__ void bf16_stage(const f32x4_t (&raw)[FAST_NJ], const int (&fi)[FAST_NJ][4], const FastMap &mp, bf16_planes_t xp,
                                           uint32_t *need, uint32_t (&amx)[FAST_NJ][4], float (*dlt)[4] = nullptr) {
    float v[FAST_NJ][4];
    uint32_t low = 0u;
#pragma unroll
    for (int j = 0; j < FAST_NJ; ++j) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            v[j][e] = raw[j][e];
            if (QUANT) {
                v[j][e] = ldexpf(round_scaled<RM>(ldexpf(v[j][e], fi[j][e])), -fi[j][e]);
                if (TRACK) amx[j][e] = max(amx[j][e], abs_bits(v[j][e]));
            }
            if (dlt) dlt[j][e] = v[j][e] - raw[j][e];
            low |= __float_as_uint(v[j][e]);
        }
        // leading parts: the high halves of the four words
        const int r = mp.on[j] ? mp.row[j] : FAST_BM;
        *(uint2 *)&xp[0][r][mp.col[j]] = make_uint2(__builtin_amdgcn_perm(__float_as_uint(v[j][1]), __float_as_uint(v[j][0]), 0x07060302u),
                                                   __builtin_amdgcn_perm(__float_as_uint(v[j][3]), __float_as_uint(v[j][2]), 0x07060302u));
    }
    // the other parts only where a wavefront staged a value of more than eight significant bits (uniform branch);
    // all three planes are written either way: every wavefront reads every staging wavefront's rows
    if (__any((low & 0xffffu) != 0u)) {
        uint32_t nz2 = 0u;
#pragma unroll
        for (int j = 0; j < FAST_NJ; ++j) {
            uint32_t h[4], md[4], lo[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                bf16_parts(v[j][e], h[e], md[e], lo[e]);
                nz2 |= lo[e];
            }
            const int r = mp.on[j] ? mp.row[j] : FAST_BM;
            *(uint2 *)&xp[1][r][mp.col[j]] = make_uint2(bf16_pair(md[0], md[1]), bf16_pair(md[2], md[3]));
            *(uint2 *)&xp[2][r][mp.col[j]] = make_uint2(bf16_pair(lo[0], lo[1]), bf16_pair(lo[2], lo[3]));
        }
        const bool third = __any(nz2 != 0u);
        if ((threadIdx.x & 63) == 0) atomicOr(need, third ? 3u : 1u);
    } else {
#pragma unroll
        for (int j = 0; j < FAST_NJ; ++j) {
            const int r = mp.on[j] ? mp.row[j] : FAST_BM;
            *(uint2 *)&xp[1][r][mp.col[j]] = make_uint2(0u, 0u);
            *(uint2 *)&xp[2][r][mp.col[j]] = make_uint2(0u, 0u);
        }
    }
}

// A lane's kernel column (B operand of x W) in parts: wp[part][step] holds k = 16 step + 8 kq + 0 .. 7 of column `col`;
// returns the number of parts the wavefront has to multiply by.
template <int NS>
__device__ __forceinline__ int bf16_kernel_column(const float *__restrict__ qw, int K, int N, int col, int kq, u32x4_t (&wp)[3][NS]) {
    // through a descriptor: entries outside the matrix read as zero and no load sits inside a branch, so all of them
    // are in flight together
    const __amdgpu_buffer_rsrc_t rs_w = buf_rsrc(qw, (int64_t)K * N * 4);
    float wv[NS][8];
#pragma unroll
    for (int st = 0; st < NS; ++st)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int k = 16 * st + 8 * kq + e;
            wv[st][e] = buf_ld1(rs_w, (k < K && col < N) ? (uint32_t)(k * N + col) * 4u : BUF_OOB);
        }
    uint32_t wnz1 = 0u, wnz2 = 0u;
#pragma unroll
    for (int st = 0; st < NS; ++st)
#pragma unroll
        for (int e = 0; e < 8; e += 2) {
            uint32_t h0, m0, l0, h1, m1, l1;
            bf16_parts(wv[st][e], h0, m0, l0), bf16_parts(wv[st][e + 1], h1, m1, l1);
            wp[0][st][e >> 1] = bf16_pair(h0, h1), wp[1][st][e >> 1] = bf16_pair(m0, m1), wp[2][st][e >> 1] = bf16_pair(l0, l1);
            wnz1 |= m0 | m1, wnz2 |= l0 | l1;
        }
    return __any(wnz2 != 0u) ? 3 : (__any(wnz1 != 0u) ? 2 : 1);
}

// acc += x W for this wavefront's 32 x 32 block: row `arow` of the staged tile against the lane's kernel column, over the
// parts that are non-zero on either side, leading parts first (uniform branches).
template <int NS>
__device__ __forceinline__ floatx16 bf16_chain(floatx16 acc, bf16_planes_t xp, int arow, int kq, uint32_t nd, const u32x4_t (&wp)[3][NS], int PW) {
    const int PX = (nd & 2u) ? 3 : ((nd & 1u) ? 2 : 1);
#pragma unroll
    for (int px = 0; px < 3; ++px) {
        if (px < PX) {
            u32x4_t a[NS];
#pragma unroll
            for (int st = 0; st < NS; ++st) a[st] = *(const u32x4_t *)&xp[px][arow][16 * st + 8 * kq];
#pragma unroll
            for (int pw = 0; pw < 3; ++pw) {
                if (pw < PW) {
#pragma unroll
                    for (int st = 0; st < NS; ++st) acc = mfma_bf16(a[st], wp[pw][st], acc);
                }
            }
        }
    }
    return acc;
}

// NS = steps of sixteen k that cover K.
// OQ: the layer's output quantizer (training-mode WRAP: round only, [Po, N] table of fractional bits, same round mode)
// runs on the output tile as it leaves: `y` gets the contraction, `yq` its quantized values, slice blockIdx.x of
// `oamax_part` the abs-max of the quantized values per table entry.
// MEAN (`ymean`; mean_rows = 32 or 64, rows a multiple of it): the output itself is not written; row g of `ymean`
// [rows / mean_rows, N] = the mean of the activated output rows g * mean_rows .. (g + 1) * mean_rows - 1, taken from the
// accumulator registers (a tile holds two groups or one): sixteen rows per lane in order, the two lane halves, then the two
// row halves.  With ReLU, `relu_mask` [rows][2] gets a bit per output - bit c & 31 of word c >> 5 of a row says that column c
// was positive - which is all the backward pass needs of the output.
template <int RM, bool QUANT, int NS, bool OQ = false, bool MEAN = false>
__global__ __launch_bounds__(256, 2) void qdense_fwd_bf16_kernel(const float *__restrict__ x, const float *__restrict__ f_in,
                                                              int P, const float *__restrict__ qw,
                                                              const float *__restrict__ qb, float *__restrict__ y,
                                                              uint32_t *amax_part, int64_t rows, int K, int N, int act,
                                                              int mode, const float *__restrict__ f_out = nullptr, int Po = 1,
                                                              int mode_out = 0, float *__restrict__ yq = nullptr,
                                                              uint32_t *oamax_part = nullptr, float *__restrict__ ymean = nullptr,
                                                              int mean_rows = 0, uint32_t *__restrict__ relu_mask = nullptr) {
    // [buffer][part][row][k]; row FAST_BM: sink of the idle staging slots
    __shared__ __attribute__((aligned(16))) uint16_t xp[2][3][FAST_BM + 1][BF_LD];
    __shared__ __attribute__((aligned(16))) float ys[FAST_BM][FAST_XLD];
    // ymean: column sums of the two row halves of a tile and the tile's ReLU mask words (written out as one contiguous run);
    // two sets in turn - a tile's set is written out behind the NEXT tile's staging barrier, so the tile needs no barrier of its own
    __shared__ float msum[MEAN ? 2 : 1][2][64];
    __shared__ uint32_t mtile[MEAN ? 2 : 1][FAST_BM][2];
    // bit 0 / 1: the staged tile has a non-zero second / third part.  Three slots in rotation: the slot of the tile after
    // next is cleared behind this tile's barrier - its last readers passed that barrier, its next writers come after the next one
    __shared__ uint32_t need[3];
    const Mode m(mode);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int rh = wave & 1, cb = wave >> 1;
    const int64_t n_tiles = (rows + FAST_BM - 1) / FAST_BM;
    // The first tile is asked for before anything else: the kernel matrix, the fractional bits and the LDS clearing below
    // then run under its latency (a launch of few tiles per workgroup is mostly these start-up round trips).
    FastMap mp, mo;
    mp.init(K);
    f32x4_t raw[FAST_NJ];
    uint32_t xoff[FAST_NJ];
#pragma unroll
    for (int j = 0; j < FAST_NJ; ++j) xoff[j] = mp.on[j] ? (uint32_t)(mp.row[j] * K + mp.col[j]) * 4u : BUF_OOB;
    auto load_tile = [&](int64_t t) {
        const int64_t r0 = t * FAST_BM, left = rows - r0;
        const __amdgpu_buffer_rsrc_t rs = buf_rsrc(x + r0 * K, (left < FAST_BM ? left : FAST_BM) * K * 4);
#pragma unroll
        for (int j = 0; j < FAST_NJ; ++j) raw[j] = buf_ld4(rs, xoff[j]);
    };
    int64_t tile = blockIdx.x;
    DB_STAMP(0, 0);
    if (tile < n_tiles) load_tile(tile);
    const int arow = rh * 32 + (lane & 31), kq = lane >> 5, bcol = cb * 32 + (lane & 31);
    u32x4_t wp[3][NS];
    const int PW = bf16_kernel_column<NS>(qw, K, N, bcol, kq, wp);  // parts of the kernel this wavefront multiplies by
    const float bias = (qb && bcol < N) ? qb[bcol] : 0.f;
    // columns from K to the end of the last step of sixteen must read as zero (they are never staged); with K a multiple
    // of 16 every column a matrix instruction reads is staged in every tile and the 56 KB need no clearing
    if (K & 15)
        for (int id = tid; id < 2 * 3 * (FAST_BM + 1) * BF_LD / 2; id += 256) ((uint32_t *)&xp[0][0][0][0])[id] = 0u;
    if (tid < 3) need[tid] = 0u;
    const bool vec_out = (N & 3) == 0 && ((uintptr_t)y & 15u) == 0;
    mo.init(vec_out ? N : 4);
    // fractional bits of the staged elements, four to a register (unpacked per tile: sixteen values and their negations
    // would otherwise each hold a register for the whole launch)
    int fip[FAST_NJ], tix[FAST_NJ];
    uint32_t amx[FAST_NJ][4];
    {
        int fi[FAST_NJ][4];
        fast_frac_bits<QUANT>(f_in, P, K, mp, m.round_params, fi, tix);
#pragma unroll
        for (int j = 0; j < FAST_NJ; ++j) fip[j] = pack_i8x4(fi[j]);
    }
#pragma unroll
    for (int j = 0; j < FAST_NJ; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e) amx[j][e] = 0;
    // OQ: fractional bits of the output elements this thread stores, four to a register, and their trackers
    int fo[OQ ? FAST_NJ : 1], otix[OQ ? FAST_NJ : 1];
    uint32_t oamx[OQ ? FAST_NJ : 1][4];
    if (OQ) {
        int fo4[FAST_NJ][4], ot[FAST_NJ];
        fast_frac_bits<true>(f_out, Po, N, mo, Mode(mode_out).round_params, fo4, ot);
#pragma unroll
        for (int j = 0; j < FAST_NJ; ++j) {
            const int jj = OQ ? j : 0;
            otix[jj] = ot[j];
                        fo[jj] = pack_i8x4(fo4[j]);
#pragma unroll
            for (int e = 0; e < 4; ++e) oamx[jj][e] = 0;
        }
    }
    __syncthreads();
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    DB_STAMP(0, 1);
    int buf = 0, slot = 0;
    [[maybe_unused]] int it_ = 0;
    // ymean: the means and mask words of tile `t`, from set `set` (threads 0 - 127)
    int64_t mean_tile = -1;
    int mean_set = 0;
    auto write_means = [&](int64_t t, int set) __attribute__((always_inline)) {
        if (tid < 2 * 64) {
            const int64_t t0 = t * FAST_BM;
            if (relu_mask && act == HGQ_ACT_RELU && t0 + (tid >> 1) < rows) relu_mask[t0 * 2 + tid] = (&mtile[set][0][0])[tid];
            const int c = tid & 63, h = tid >> 6;
            if (mean_rows == FAST_BM) {
                if (h == 0 && c < N) ymean[t * N + c] = (msum[set][0][c] + msum[set][1][c]) * (1.0f / FAST_BM);
            } else if (c < N && t0 + h * 32 < rows) {
                ymean[(2 * t + h) * N + c] = msum[set][h][c] * (1.0f / 32);
            }
        }
    };
    for (; tile < n_tiles; tile += gridDim.x, buf ^= 1, slot = slot == 2 ? 0 : slot + 1, ++it_) {
        int fi[FAST_NJ][4];
#pragma unroll
        for (int j = 0; j < FAST_NJ; ++j) {
            asm volatile("" : "+v"(fip[j]));
#pragma unroll
            for (int e = 0; e < 4; ++e) fi[j][e] = unpack_i8(fip[j], e);
        }
        bf16_stage<RM, QUANT, QUANT>(raw, fi, mp, xp[buf], &need[slot], amx);
        DB_STAMP(0, 2 + 6 * it_);
        __syncthreads();
        DB_STAMP(0, 3 + 6 * it_);
        if (tid == 0) need[slot == 0 ? 2 : slot - 1] = 0u;  // (slot + 2) % 3
        const int64_t next = tile + gridDim.x;
        if (next < n_tiles) load_tile(next);
        if (MEAN && mean_tile >= 0) write_means(mean_tile, mean_set ^ 1);
        floatx16 acc = {0};
        if (cb * 32 < N) {
            acc = bf16_chain<NS>(acc, xp[buf], arow, kq, need[slot], wp, PW);
        }
        DB_STAMP(0, 4 + 6 * it_);
        const int64_t r0 = tile * FAST_BM;
        if (MEAN) {
            // no branch inside the loop: the mask words are formed whatever the activation and only written out with ReLU
            const bool relu = act == HGQ_ACT_RELU;
            float csum = 0.f;
            uint32_t word[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                float v = acc[r] + bias;
                const bool pos = v > 0.f;
                v = (relu && !pos) ? 0.f : v;
                // lanes 0 - 31 hold 32 columns of one row, lanes 32 - 63 the same columns of the row four below
                const unsigned long long bits = __ballot(pos);
                word[r] = lane >= 32 ? (uint32_t)(bits >> 32) : (uint32_t)bits;
                csum += v;
            }
            if ((lane & 31) == 0) {
#pragma unroll
                for (int r = 0; r < 16; ++r) mtile[mean_set][rh * 32 + acc_row(r, lane)][cb] = word[r];
            }
            csum += __shfl_xor(csum, 32);
            if (lane < 32) msum[mean_set][rh][bcol] = csum;
            // written out behind the next tile's staging barrier (or the one after the loop); this set is written again two
            // tiles on, behind a barrier that the threads who read it now have passed
            mean_tile = tile, mean_set ^= 1;
        } else if (vec_out) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                float v = acc[r] + bias;
                if (act == HGQ_ACT_RELU) v = v > 0.f ? v : 0.f;
                ys[rh * 32 + acc_row(r, lane)][bcol] = v;
            }
            DB_STAMP(0, 5 + 6 * it_);
            __syncthreads();
            DB_STAMP(0, 6 + 6 * it_);
#pragma unroll
            for (int j = 0; j < FAST_NJ; ++j) {
                const int64_t gr = r0 + mo.row[j];
                if (mo.on[j] && gr < rows) {
                    const f32x4_t v4 = *(const f32x4_t *)&ys[mo.row[j]][mo.col[j]];
                    *(f32x4_t *)(y + gr * N + mo.col[j]) = v4;
                    if (OQ) {
                        const int jj = OQ ? j : 0;
                        asm volatile("" : "+v"(fo[jj]));
                        f32x4_t q4;
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const int f = unpack_i8(fo[jj], e);
                            q4[e] = ldexpf(round_scaled<RM>(ldexpf(v4[e], f)), -f);
                            oamx[jj][e] = max(oamx[jj][e], abs_bits(q4[e]));
                        }
                        *(f32x4_t *)(yq + gr * N + mo.col[j]) = q4;
                    }
                }
            }
        } else {
            if (bcol < N) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int64_t gr = r0 + rh * 32 + acc_row(r, lane);
                    if (gr < rows) {
                        float v = acc[r] + bias;
                        if (act == HGQ_ACT_RELU) v = v > 0.f ? v : 0.f;
                        y[gr * N + bcol] = v;
                    }
                }
            }
        }
    }
    DB_STAMP(0, 30);
    if (MEAN && mean_tile >= 0) {
        __syncthreads();
        write_means(mean_tile, mean_set ^ 1);
    }
    if (QUANT && amax_part && P == FAST_BM && ((uintptr_t)amax_part & 15u) == 0) {
        uint32_t *my = amax_part + (int64_t)blockIdx.x * (P * K);
#pragma unroll
        for (int j = 0; j < FAST_NJ; ++j)
            if (mp.on[j]) {
                uint4 v;
                v.x = amx[j][0], v.y = amx[j][1], v.z = amx[j][2], v.w = amx[j][3];
                *(uint4 *)(my + tix[j]) = v;
            }
    } else if (QUANT && amax_part) {
        const int PK = P * K;
        uint32_t *tab = (uint32_t *)&ys[0][0];
        __syncthreads();
        for (int t = tid; t < PK; t += 256) tab[t] = 0;
        __syncthreads();
#pragma unroll
        for (int j = 0; j < FAST_NJ; ++j)
            if (mp.on[j])
#pragma unroll
                for (int e = 0; e < 4; ++e) atomicMax(&tab[tix[j] + e], amx[j][e]);
        __syncthreads();
        uint32_t *my = amax_part + (int64_t)blockIdx.x * PK;
        for (int t = tid; t < PK; t += 256) my[t] = tab[t];
    }
    if (OQ) {  // (launched with 128-bit output rows only)
        const int PN = Po * N;
        uint32_t *my = oamax_part + (int64_t)blockIdx.x * PN;
        if (Po == FAST_BM) {
#pragma unroll
            for (int j = 0; j < FAST_NJ; ++j)
                if (mo.on[j]) {
                    const int jj = OQ ? j : 0;
                    uint4 v;
                    v.x = oamx[jj][0], v.y = oamx[jj][1], v.z = oamx[jj][2], v.w = oamx[jj][3];
                    *(uint4 *)(my + otix[jj]) = v;
                }
        } else {
            uint32_t *tab = (uint32_t *)&ys[0][0];
            __syncthreads();
            for (int t = tid; t < PN; t += 256) tab[t] = 0;
            __syncthreads();
#pragma unroll
            for (int j = 0; j < FAST_NJ; ++j)
                if (mo.on[j])
#pragma unroll
                    for (int e = 0; e < 4; ++e) atomicMax(&tab[otix[OQ ? j : 0] + e], oamx[OQ ? j : 0][e]);
            __syncthreads();
            for (int t = tid; t < PN; t += 256) my[t] = tab[t];
        }
    }
    DB_STAMP(0, 31);
}

// Column statistics of the contraction without writing it: sum_r z and sum_r z^2 of z = x W per
// output column, for the batch statistics of QEinsumDenseBatchnorm.  Same tiling as the forward
// above; a lane keeps the sums of its column over its 16 accumulator rows in registers across
// tiles.  Slice blockIdx.x of `part` is [N sums | N sums of squares].
// QUANT: x is the raw input of a training-mode WRAP quantizer (round only) with a [P, K] table of fractional bits,
// quantized while it is staged exactly as the forward kernel does.
template <int RM, bool QUANT, int NS4>
__global__ __launch_bounds__(256, 2) void dense_moments_fast_kernel(const float *__restrict__ x, const float *__restrict__ f_in, int P,
                                                                   const float *__restrict__ w, float *__restrict__ part,
                                                                   int64_t rows, int K, int N, int mode) {
    __shared__ __attribute__((aligned(16))) float xs[2][FAST_BM + 1][FAST_XLD];
    __shared__ float red[4][64][2];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int rh = wave & 1, cb = wave >> 1;
    const int64_t n_tiles = (rows + FAST_BM - 1) / FAST_BM;
    for (int id = tid; id < 2 * (FAST_BM + 1) * FAST_XLD; id += 256) (&xs[0][0][0])[id] = 0.f;
    const int arow = rh * 32 + (lane & 31), kq = lane >> 5, bcol = cb * 32 + (lane & 31);
    float wreg[4 * NS4];
#pragma unroll
    for (int sidx = 0; sidx < 4 * NS4; ++sidx) {
        const int k = 2 * sidx + kq;
        wreg[sidx] = (k < K && bcol < N) ? w[(int64_t)k * N + bcol] : 0.f;
    }
    FastMap mp;
    mp.init(K);
    int fi[FAST_NJ][4], tix[FAST_NJ];
    fast_frac_bits<QUANT>(f_in, P, K, mp, Mode(mode).round_params, fi, tix);
    f32x4_t raw[FAST_NJ];
    uint32_t xoff[FAST_NJ];
#pragma unroll
    for (int j = 0; j < FAST_NJ; ++j) xoff[j] = mp.on[j] ? (uint32_t)(mp.row[j] * K + mp.col[j]) * 4u : BUF_OOB;
    auto load_tile = [&](int64_t t) {
        const int64_t r0 = t * FAST_BM, left = rows - r0;
        const __amdgpu_buffer_rsrc_t rs = buf_rsrc(x + r0 * K, (left < FAST_BM ? left : FAST_BM) * K * 4);
#pragma unroll
        for (int j = 0; j < FAST_NJ; ++j) raw[j] = buf_ld4(rs, xoff[j]);
    };
    int64_t tile = blockIdx.x;
    if (tile < n_tiles) load_tile(tile);
    __syncthreads();
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    float s1 = 0.f, s2 = 0.f;
    int buf = 0;
    for (; tile < n_tiles; tile += gridDim.x, buf ^= 1) {
#pragma unroll
        for (int j = 0; j < FAST_NJ; ++j) {
            float v[4] = {raw[j][0], raw[j][1], raw[j][2], raw[j][3]};
            if (QUANT) {
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = ldexpf(round_scaled<RM>(ldexpf(v[e], fi[j][e])), -fi[j][e]);
            }
            float *dst = &xs[buf][mp.on[j] ? mp.row[j] : FAST_BM][mp.col[j] >> 1];
            *(float2 *)dst = make_float2(v[0], v[2]);
            *(float2 *)(dst + 32) = make_float2(v[1], v[3]);
        }
        __syncthreads();
        const int64_t next = tile + gridDim.x;
        if (next < n_tiles) load_tile(next);
        if (cb * 32 < N) {
            floatx16 acc = {0};
            const float *arow_p = &xs[buf][arow][kq * 32];
            f32x4_t a4[NS4];
#pragma unroll
            for (int s4 = 0; s4 < NS4; ++s4) a4[s4] = *(const f32x4_t *)(arow_p + 4 * s4);
#pragma unroll
            for (int s4 = 0; s4 < NS4; ++s4)
#pragma unroll
                for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a4[s4][e], wreg[4 * s4 + e], acc, 0, 0, 0);
            // rows past the end were staged as zeros: z = 0 there, which adds nothing
#pragma unroll
            for (int r = 0; r < 16; ++r) s1 += acc[r], s2 += acc[r] * acc[r];
        }
    }
    // a column's sums sit in two lanes (row groups) of two wavefronts (row halves): add them in a fixed order
    red[wave][lane][0] = s1, red[wave][lane][1] = s2;
    __syncthreads();
    if (tid < 2 * N) {
        const int c = tid % N, which = tid / N, wcb = c >> 5, l = c & 31;
        float v = 0.f;
#pragma unroll
        for (int h = 0; h < 2; ++h) v += red[wcb * 2 + h][l][which] + red[wcb * 2 + h][l + 32][which];
        part[(int64_t)blockIdx.x * 2 * N + which * N + c] = v;
    }
}

// The column statistics on the bf16 matrix cores (exact splitting, see qdense_fwd_bf16_kernel).
template <int RM, bool QUANT, int NS>
__global__ __launch_bounds__(256, 2) void dense_moments_bf16_kernel(const float *__restrict__ x, const float *__restrict__ f_in, int P,
                                                                   const float *__restrict__ w, float *__restrict__ part,
                                                                   int64_t rows, int K, int N, int mode) {
    __shared__ __attribute__((aligned(16))) uint16_t xp[2][3][FAST_BM + 1][BF_LD];
    __shared__ float red[4][64][2];
    __shared__ uint32_t need[3];  // three slots in rotation, as in the forward kernel
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int rh = wave & 1, cb = wave >> 1;
    const int64_t n_tiles = (rows + FAST_BM - 1) / FAST_BM;
    if (K & 15)  // (as in the forward kernel: only the columns between K and the next multiple of 16 need zeros)
        for (int id = tid; id < 2 * 3 * (FAST_BM + 1) * BF_LD / 2; id += 256) ((uint32_t *)&xp[0][0][0][0])[id] = 0u;
    if (tid < 3) need[tid] = 0u;
    const int arow = rh * 32 + (lane & 31), kq = lane >> 5, bcol = cb * 32 + (lane & 31);
    u32x4_t wp[3][NS];
    const int PW = bf16_kernel_column<NS>(w, K, N, bcol, kq, wp);
    FastMap mp;
    mp.init(K);
    int fi[FAST_NJ][4], tix[FAST_NJ];
    uint32_t amx[FAST_NJ][4];  // not tracked here
    fast_frac_bits<QUANT>(f_in, P, K, mp, Mode(mode).round_params, fi, tix);
    f32x4_t raw[FAST_NJ];
    uint32_t xoff[FAST_NJ];
#pragma unroll
    for (int j = 0; j < FAST_NJ; ++j) xoff[j] = mp.on[j] ? (uint32_t)(mp.row[j] * K + mp.col[j]) * 4u : BUF_OOB;
    auto load_tile = [&](int64_t t) {
        const int64_t r0 = t * FAST_BM, left = rows - r0;
        const __amdgpu_buffer_rsrc_t rs = buf_rsrc(x + r0 * K, (left < FAST_BM ? left : FAST_BM) * K * 4);
#pragma unroll
        for (int j = 0; j < FAST_NJ; ++j) raw[j] = buf_ld4(rs, xoff[j]);
    };
    int64_t tile = blockIdx.x;
    if (tile < n_tiles) load_tile(tile);
    __syncthreads();
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    float s1 = 0.f, s2 = 0.f;
    int buf = 0, slot = 0;
    for (; tile < n_tiles; tile += gridDim.x, buf ^= 1, slot = slot == 2 ? 0 : slot + 1) {
        bf16_stage<RM, QUANT, false>(raw, fi, mp, xp[buf], &need[slot], amx);
        __syncthreads();
        if (tid == 0) need[slot == 0 ? 2 : slot - 1] = 0u;
        const uint32_t nd = need[slot];
        const int64_t next = tile + gridDim.x;
        if (next < n_tiles) load_tile(next);
        if (cb * 32 < N) {
            floatx16 acc = {0};
            acc = bf16_chain<NS>(acc, xp[buf], arow, kq, nd, wp, PW);
            // rows past the end were staged as zeros: z = 0 there, which adds nothing
#pragma unroll
            for (int r = 0; r < 16; ++r) s1 += acc[r], s2 += acc[r] * acc[r];
        }
    }
    red[wave][lane][0] = s1, red[wave][lane][1] = s2;
    __syncthreads();
    if (tid < 2 * N) {
        const int c = tid % N, which = tid / N, wcb = c >> 5, l = c & 31;
        float v = 0.f;
#pragma unroll
        for (int h = 0; h < 2; ++h) v += red[wcb * 2 + h][l][which] + red[wcb * 2 + h][l + 32][which];
        part[(int64_t)blockIdx.x * 2 * N + which * N + c] = v;
    }
}

// Backward.  Per tile: stage dz = dy (masked by y for ReLU) and the quantized input; dx = dz W^T
// and dW += xq^T dz on MFMA; dx goes back through LDS so that it is stored with 128-bit writes and
// meets the rounding residue (xq - x) of the staging thread for the fractional-bit gradient.
// Slice blockIdx.x of `part` is [K * N | N | P * K].
// STATS: the gradient at the pre-activation is not read but computed in the tile from the upstream
// gradients of the column statistics: dz[r, c] = (gm[c] + 2 z[r, c] gs[c]) / rows with z = x W
// recomputed on the matrix cores (dy = gm, y = gs, both [N]); no activation, no bias, no quantizer.
// BF: the three contractions run on the bf16 matrix cores by exact splitting (mfma_chain_bf16); the gradient operand is
// taken in all three parts without looking, the quantized input and the kernel in as many as they need.
// BCAST (32 or 64, not with STATS, ZVEC only, rows a multiple of it; `bcast` below): the output went through a mean over groups of `bcast` rows
// and dy is the gradient of those means, [rows / bcast, N]: row r of the gradient tile is dy[r / bcast] / bcast, read with a
// zero row stride instead of from a broadcast copy; `y` is then not the output but its ReLU mask, two 32-bit words per row
// (what the forward kernel leaves when it writes the means instead of the output).
// PAIRS (with BF; K and N above 32): wavefronts 0 and 1 take the two row halves of dx (both k blocks: the gradient rows they
// contract are split into bf16 parts once for both), wavefronts 2 and 3 the two column halves of the kernel gradient (both k
// blocks, all rows of the tile) - every gradient value is split twice per tile instead of four times.  A wavefront's two
// blocks live in the same registers either way: reset per tile for dx, kept across the tiles for the kernel gradient.
template <int RM, bool QUANT, bool STATS = false, bool ZVEC = true, bool BF = false, bool PAIRS = false, int BCAST = 0, bool NOACT = false>
__global__ __launch_bounds__(256, 2) void qdense_bwd_fast_kernel(const float *__restrict__ dy, const float *__restrict__ y,
                                                              const float *__restrict__ x, const float *__restrict__ f_in,
                                                              int P, const float *__restrict__ qw, float *__restrict__ dx,
                                                              float *part, int has_bias, int64_t rows, int K, int N, int act,
                                                              int mode, const float *__restrict__ dx_add) {
    constexpr int bcast = BCAST;
    __shared__ float xs[FAST_BM + 1][FAST_LD];   // row FAST_BM: sink of the idle staging slots
    __shared__ float dzs[FAST_BM + 1][FAST_LD];  // dz, then the dx tile
    __shared__ float ws[64][FAST_LD];
    __shared__ float adds[STATS ? FAST_BM + 1 : 1][STATS ? FAST_LD : 1];  // STATS: the tile of dx_add, staged with x
    const bool has_add = STATS && dx_add != nullptr;
    const Mode m(mode);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // (PAIRS is launched with K and N above 32 only: both block counts are 2 and known when the kernel is compiled)
    const int K32 = PAIRS ? 2 : (K + 31) >> 5, N32 = PAIRS ? 2 : (N + 31) >> 5;
    const bool split_n = !PAIRS && K32 == 1 && N32 == 2;
    const int PK = QUANT ? P * K : 0;
    const int64_t M = (int64_t)K * N + N + PK;
    const int64_t n_tiles = (rows + FAST_BM - 1) / FAST_BM;
    float *my_dw = part + (int64_t)blockIdx.x * M;
    float *my_db = my_dw + (int64_t)K * N;
    float *my_df = my_db + N;
    FastMap mx, mz;
    // !ZVEC - N not a multiple of 4, or unaligned gradient rows: the gradient tile is staged in groups of four columns
    // of the width rounded up, each element with a load of its own (columns past N read as zero)
    mx.init(K), mz.init((N + 3) & ~3);
    // fractional bits of the staged elements, four to a register (unpacked per tile: sixteen values and their negations
    // would otherwise each hold a register for the whole launch); loaded in the start-up block below
    int fip[FAST_NJ];
    float gf[FAST_NJ][4];
#pragma unroll
    for (int j = 0; j < FAST_NJ; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e) gf[j][e] = 0.f;
    // kernel-gradient block owned by this wave
    const int nblk = K32 * N32, wpb = 4 / nblk;
    const int blk = wave / wpb, sub = wave % wpb;
    const int wkb = blk / N32, wnb = blk % N32;
    const int rows_per = FAST_BM / wpb;
    floatx16 accw = {0}, acc2 = {0};  // acc2: the second block of a wavefront with PAIRS
    float accb = 0.f;
    const int bn = tid & 63, bq = tid >> 6;
    // NOACT: launched without activation - the forward output is then neither asked for nor kept in registers
    const bool relu = !NOACT && act == HGQ_ACT_RELU;

    f32x4_t rx[FAST_NJ], rg[FAST_NJ], ry[FAST_NJ];
    uint32_t xoff[FAST_NJ], zoff[FAST_NJ];
#pragma unroll
    for (int j = 0; j < FAST_NJ; ++j) {
        xoff[j] = mx.on[j] ? (uint32_t)(mx.row[j] * K + mx.col[j]) * 4u : BUF_OOB;
        zoff[j] = mz.on[j] ? (uint32_t)(mz.row[j] * N + mz.col[j]) * 4u : BUF_OOB;
    }
    int64_t tile = blockIdx.x;
    DB_STAMP(1, 0);
    // descriptors cover the valid rows of one tile (rows past the end read as zero); without ReLU
    // the mask descriptor is empty and is not consulted
    auto load_tile = [&](int64_t t) {
        const int64_t r0 = t * FAST_BM, left = rows - r0, vr = left < FAST_BM ? left : FAST_BM;
        const __amdgpu_buffer_rsrc_t sx = buf_rsrc(x + r0 * K, vr * K * 4);
        const __amdgpu_buffer_rsrc_t sg = STATS ? buf_rsrc(has_add ? dx_add + r0 * K : x, has_add ? vr * K * 4 : 0)
                                          : bcast ? buf_rsrc(dy + (r0 / bcast) * N, ((vr + bcast - 1) / bcast) * N * 4)
                                                  : buf_rsrc(dy + r0 * N, vr * N * 4);
        const __amdgpu_buffer_rsrc_t sy = bcast ? buf_rsrc(relu ? y + r0 * 2 : x, relu ? vr * 2 * 4 : 0)
                                                : buf_rsrc((relu && !STATS) ? y + r0 * N : x, (relu && !STATS) ? vr * N * 4 : 0);
#pragma unroll
        for (int j = 0; j < FAST_NJ; ++j) {
            rx[j] = buf_ld4(sx, xoff[j]);
            if (!STATS) {
                if (ZVEC) {
                    // bcast: every row of a group reads the group's one gradient row
                    const uint32_t goff = !bcast ? zoff[j]
                                          : mz.on[j] ? (uint32_t)((bcast == 32 ? (mz.row[j] >> 5) : 0) * N + mz.col[j]) * 4u : BUF_OOB;
                    rg[j] = buf_ld4(sg, goff);
                    if (NOACT) ry[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
                    else if (bcast) ry[j][0] = buf_ld1(sy, mz.on[j] ? (uint32_t)(mz.row[j] * 2 + (mz.col[j] >> 5)) * 4u : BUF_OOB);  // mask word
                    else ry[j] = buf_ld4(sy, zoff[j]);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const uint32_t off = (mz.on[j] && mz.col[j] + e < N) ? zoff[j] + 4u * e : BUF_OOB;
                        rg[j][e] = buf_ld1(sg, off);
                        ry[j][e] = buf_ld1(sy, off);
                    }
                }
            } else {
                rg[j] = buf_ld4(sg, xoff[j]);  // the other gradient of x, laid out like x (zeros without one)
            }
        }
    };
    const float inv_rows = 1.0f / (float)rows;
    const float gscale = bcast ? 1.0f / (float)bcast : 1.0f;
    // Start-up: the first tile is asked for first, then the kernel matrix and the fractional bits - one round trip for the
    // three of them instead of three in a row (a launch of one or two tiles per workgroup is mostly start-up).
    if (tile < n_tiles) load_tile(tile);
    {
        // all 16 kernel-matrix loads of a thread in flight (one per loop trip would cost a memory latency each)
        const __amdgpu_buffer_rsrc_t rs_w = buf_rsrc(qw, (int64_t)K * N * 4);
        float wv[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) {
            const int id = tid + 256 * u, kk = id >> 6, nn = id & 63;
            wv[u] = buf_ld1(rs_w, (kk < K && nn < N) ? (uint32_t)(kk * N + nn) * 4u : BUF_OOB);
        }
        int fi[FAST_NJ][4], tix[FAST_NJ];
        fast_frac_bits<QUANT>(f_in, P, K, mx, m.round_params, fi, tix);
#pragma unroll
        for (int j = 0; j < FAST_NJ; ++j) fip[j] = pack_i8x4(fi[j]);
#pragma unroll
        for (int u = 0; u < 16; ++u) {
            const int id = tid + 256 * u, kk = id >> 6, nn = id & 63;
            ws[kk][nn] = wv[u];
            xs[kk][nn] = 0.f, dzs[kk][nn] = 0.f;
        }
    }
    __syncthreads();
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): nothing loaded before the loop is waited for inside it
    DB_STAMP(1, 1);
    [[maybe_unused]] int it_ = 0;
    for (; tile < n_tiles; tile += gridDim.x, ++it_) {
        float dlt[FAST_NJ][4];  // xq - x of the elements this thread stages
        __syncthreads();        // previous tile's dx has been read back
        DB_STAMP(1, 2 + 6 * it_);
        // no branch around a staging slot (a wait inside one would cover every load): idle slots
        // hold zeros and write them to the sink row
#pragma unroll
        for (int j = 0; j < FAST_NJ; ++j) {
            const float v[4] = {rx[j][0], rx[j][1], rx[j][2], rx[j][3]};
            const int xr = mx.on[j] ? mx.row[j] : FAST_BM, zr = mz.on[j] ? mz.row[j] : FAST_BM;
            asm volatile("" : "+v"(fip[j]));
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int f = unpack_i8(fip[j], e);
                const float q = QUANT ? ldexpf(round_scaled<RM>(ldexpf(v[e], f)), -f) : v[e];
                dlt[j][e] = q - v[e];
                xs[xr][mx.col[j] + e] = q;
            }
            if (STATS) {
                if (has_add) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) adds[xr][mx.col[j] + e] = rg[j][e];
                }
            } else {
                const float g[4] = {rg[j][0], rg[j][1], rg[j][2], rg[j][3]};
                const float a[4] = {ry[j][0], ry[j][1], ry[j][2], ry[j][3]};
                const uint32_t mbits = __float_as_uint(ry[j][0]) >> (mz.col[j] & 31);  // (BCAST: the mask word of this row and column block)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const bool live = !relu || (bcast ? ((mbits >> e) & 1u) != 0u : a[e] > 0.f);
                    dzs[zr][mz.col[j] + e] = live ? g[e] * gscale : 0.f;
                }
            }
        }
        DB_STAMP(1, 3 + 6 * it_);
        __syncthreads();
        DB_STAMP(1, 4 + 6 * it_);
        if (STATS) {
            // z block (row half, column block) of this wave, then dz into the gradient tile
            const int zrh = wave & 1, zcb = wave >> 1;
            if (zcb < N32) {
                floatx16 z = {0};
                const int arow = zrh * 32 + (lane & 31), kq = lane >> 5, bcol = zcb * 32 + (lane & 31);
                z = BF ? mfma_chain_bf16<false, false>(z, &xs[arow][kq], 1, &ws[kq][bcol], FAST_LD, K32 * 2)
                       : mfma_chain(z, &xs[arow][kq], 1, &ws[kq][bcol], FAST_LD, K32 * 2);
                const float gm = bcol < N ? dy[bcol] : 0.f, gs = bcol < N ? y[bcol] : 0.f;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int row = zrh * 32 + acc_row(r, lane);
                    const bool live = tile * FAST_BM + row < rows && bcol < N;
                    dzs[row][bcol] = live ? (gm + 2.0f * z[r] * gs) * inv_rows : 0.f;
                }
            }
            __syncthreads();
        }
        const int64_t next = tile + gridDim.x;
        const int64_t r0 = tile * FAST_BM;
        if (next < n_tiles) load_tile(next);
        // ---- dx = dz @ qW^T : blocks (row half, k block), kept in registers until dz is no longer needed
        floatx16 acc = {0};
        const int rh = wave & 1, kb = wave >> 1;
        if (PAIRS) {
            const int kq = lane >> 5, c32 = lane & 31;
            if (wave < 2) {
                accw = floatx16{0}, acc2 = floatx16{0};
#pragma unroll
                for (int bt = 0; bt < 4; ++bt) {
                    float a[8], b0[8], b1[8];
#pragma unroll
                    for (int u = 0; u < 8; ++u) {
                        const int n = 16 * bt + 2 * u + kq;
                        a[u] = dzs[wave * 32 + c32][n], b0[u] = ws[c32][n], b1[u] = ws[32 + c32][n];
                    }
                    mfma_batch2_bf16<true>(accw, acc2, a, b0, b1);
                }
            } else {
#pragma unroll
                for (int bt = 0; bt < FAST_BM / 16; ++bt) {
                    float b[8], a0[8], a1[8];
#pragma unroll
                    for (int u = 0; u < 8; ++u) {
                        const int r = 16 * bt + 2 * u + kq;
                        b[u] = dzs[r][(wave - 2) * 32 + c32], a0[u] = xs[r][c32], a1[u] = xs[r][32 + c32];
                    }
                    mfma_batch2_bf16<false>(accw, acc2, b, a0, a1);
                }
            }
        } else if (split_n) {
            // one k block, two column blocks: the two wavefronts of a row half take one half of the contraction each
            const int arow = rh * 32 + (lane & 31), kq = lane >> 5, n0 = kb * 32;
            acc = BF ? mfma_chain_bf16<true, false>(acc, &dzs[arow][n0 + kq], 1, &ws[lane & 31][n0 + kq], 1, 2)
                     : mfma_chain(acc, &dzs[arow][n0 + kq], 1, &ws[lane & 31][n0 + kq], 1, 2);
        } else if (kb < K32) {
            const int arow = rh * 32 + (lane & 31), kq = lane >> 5, wrow = kb * 32 + (lane & 31);
            acc = BF ? mfma_chain_bf16<true, false>(acc, &dzs[arow][kq], 1, &ws[wrow][kq], 1, N32 * 2)
                     : mfma_chain(acc, &dzs[arow][kq], 1, &ws[wrow][kq], 1, N32 * 2);
        }
        // ---- dW += xq^T @ dz : this wave's block, its slice of the tile's rows
        if (!PAIRS) {
            const int rbeg = sub * rows_per;
            const int kq = lane >> 5, c32 = lane & 31;
            accw = BF ? mfma_chain_bf16<false, true>(accw, &xs[rbeg + kq][wkb * 32 + c32], FAST_LD, &dzs[rbeg + kq][wnb * 32 + c32], FAST_LD, rows_per / 16)
                      : mfma_chain(accw, &xs[rbeg + kq][wkb * 32 + c32], FAST_LD, &dzs[rbeg + kq][wnb * 32 + c32], FAST_LD, rows_per / 16);
        }
        if (has_bias) {
#pragma unroll
            for (int j = 0; j < FAST_BM / 4; ++j) accb += dzs[bq * (FAST_BM / 4) + j][bn];
        }
        DB_STAMP(1, 5 + 6 * it_);
        __syncthreads();  // dz and xq consumed: the dx tile takes the place of dz (its second partial sum that of xq)
        DB_STAMP(1, 6 + 6 * it_);
        if (PAIRS) {
            if (wave < 2) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    dzs[wave * 32 + acc_row(r, lane)][lane & 31] = accw[r];
                    dzs[wave * 32 + acc_row(r, lane)][32 + (lane & 31)] = acc2[r];
                }
            }
        } else if (split_n) {
            float(*dst)[FAST_LD] = kb ? xs : dzs;
#pragma unroll
            for (int r = 0; r < 16; ++r) dst[rh * 32 + acc_row(r, lane)][lane & 31] = acc[r];
        } else if (kb < K32) {
            const int kcol = kb * 32 + (lane & 31);
#pragma unroll
            for (int r = 0; r < 16; ++r) dzs[rh * 32 + acc_row(r, lane)][kcol] = acc[r];
        }
        __syncthreads();
        DB_STAMP(1, 7 + 6 * it_);
#pragma unroll
        for (int j = 0; j < FAST_NJ; ++j) {
            if (mx.on[j]) {
                const int64_t gr = r0 + mx.row[j];
                float4 o;
                o.x = dzs[mx.row[j]][mx.col[j]], o.y = dzs[mx.row[j]][mx.col[j] + 1];
                o.z = dzs[mx.row[j]][mx.col[j] + 2], o.w = dzs[mx.row[j]][mx.col[j] + 3];
                if (split_n) {
                    o.x += xs[mx.row[j]][mx.col[j]], o.y += xs[mx.row[j]][mx.col[j] + 1];
                    o.z += xs[mx.row[j]][mx.col[j] + 2], o.w += xs[mx.row[j]][mx.col[j] + 3];
                }
                float4 og = o;  // this contraction's own gradient: the one the rounding residue meets
                if (has_add) {
                    o.x += adds[mx.row[j]][mx.col[j]], o.y += adds[mx.row[j]][mx.col[j] + 1];
                    o.z += adds[mx.row[j]][mx.col[j] + 2], o.w += adds[mx.row[j]][mx.col[j] + 3];
                }
                if (gr < rows) {
                    st4(dx + gr * K + mx.col[j], o);
                    if (QUANT) {
                        gf[j][0] += -HGQ_LN2 * dlt[j][0] * og.x, gf[j][1] += -HGQ_LN2 * dlt[j][1] * og.y;
                        gf[j][2] += -HGQ_LN2 * dlt[j][2] * og.z, gf[j][3] += -HGQ_LN2 * dlt[j][3] * og.w;
                    }
                }
            }
        }
    }
    // ---- write this workgroup's slice.  Waves sharing a kernel-gradient block combine through LDS.
    DB_STAMP(1, 30);
    __syncthreads();
    float *comb = &xs[0][0];
    if (PAIRS) {
        if (wave >= 2) {
            const int n = (wave - 2) * 32 + (lane & 31);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                comb[acc_row(r, lane) * FAST_LD + n] = accw[r];
                comb[(32 + acc_row(r, lane)) * FAST_LD + n] = acc2[r];
            }
        }
        __syncthreads();
    }
    for (int pass = 0; pass < (PAIRS ? 0 : wpb); ++pass) {
        if (sub == pass) {
            const int n = wnb * 32 + (lane & 31);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int k = wkb * 32 + acc_row(r, lane);
                if (pass == 0) comb[k * FAST_LD + n] = accw[r];
                else comb[k * FAST_LD + n] += accw[r];
            }
        }
        __syncthreads();
    }
#pragma unroll 4
    for (int id = tid; id < K * 64; id += 256) {
        const int kk = id >> 6, nn = id & 63;
        if (nn < N) my_dw[kk * N + nn] = comb[kk * FAST_LD + nn];
    }
    float *bred = &ws[0][0];
    __syncthreads();
    bred[tid] = accb;
    __syncthreads();
    if (tid < N) my_db[tid] = has_bias ? bred[tid] + bred[tid + 64] + bred[tid + 128] + bred[tid + 192] : 0.f;
    if (QUANT) {
        // fractional-bit gradient: every (tile row, column) has one owner thread; rows that share a
        // table row are added in row order
        float *gt = &dzs[0][0];
        __syncthreads();
#pragma unroll
        for (int j = 0; j < FAST_NJ; ++j)
            if (mx.on[j])
#pragma unroll
                for (int e = 0; e < 4; ++e) gt[mx.row[j] * FAST_LD + mx.col[j] + e] = gf[j][e];
        __syncthreads();
        if (P <= 16) {
            // few table rows, many tile rows per entry: four threads per entry add a quarter of the tile each (a serial
            // walk over all 64 rows was three microseconds of every launch), then the quarters are added in order
            float *quarter = &xs[0][0];  // (the kernel-gradient block has left it)
            for (int id = tid; id < 4 * P * 64; id += 256) {
                const int c = id & 63, pq = id >> 6, p = pq & (P - 1), q = pq / P;  // (P is a power of two)
                float s = 0.f;
                for (int r = 16 * q + p; r < 16 * q + 16; r += P) s += gt[r * FAST_LD + c];
                quarter[pq * 64 + c] = s;
            }
            __syncthreads();
            for (int id = tid; id < P * 64; id += 256) {
                const int p = id >> 6, c = id & 63;
                if (c < K)
                    my_df[p * K + c] = (quarter[p * 64 + c] + quarter[(P + p) * 64 + c]) + (quarter[(2 * P + p) * 64 + c] + quarter[(3 * P + p) * 64 + c]);
            }
        } else {
#pragma unroll 4
            for (int id = tid; id < P * 64; id += 256) {
                const int p = id >> 6, c = id & 63;
                if (c < K) {
                    float s = 0.f;
                    for (int r = p; r < FAST_BM; r += P) s += gt[r * FAST_LD + c];
                    my_df[p * K + c] = s;
                }
            }
        }
    }
    DB_STAMP(1, 31);
}

// ------------------------------------------------------------------------------------------
// Backward of the column statistics without the pre-activation.  With z = xq W, the upstream gradients gm / gs of the
// column means / means of squares give  dz[r, c] = (gm[c] + 2 z[r, c] gs[c]) / rows,  and both results are functions of
// xq through K x K matrices:
//     dx = dz W^T          = xq A + v,      A = (2 / rows) W diag(gs) W^T,   v = W gm / rows
//     dW = xq^T dz         = (m gm^T + 2 (S W) diag(gs)) / rows,   S = xq^T xq,  m = column sums of xq  (live rows)
// so a tile costs one contraction of the quantized input with A (the kernel above recomputes z, forms dz and contracts it
// twice, each time splitting fresh fp32 values) and one Gram update of the quantized input with itself - operands of one
// bf16 part each in the usual case.  A and v are formed once per workgroup while the first tile is on its way; S W once
// per workgroup at the end.  Slices, arguments and results are those of the STATS form of qdense_bwd_fast_kernel
// (dy = gm, y = gs, no activation, no bias; the [N] section of a slice is zero).
// rep > 1 (a narrow input, K rep = 64): the caller passes the [rows, K] operands as [rows / rep, 64] - the same memory, rep
// rows side by side, the [P, K] table of fractional bits as [P / rep, 64] - and the kernel works on 64-wide rows with
// A' = diag(A, ..., A) and v' = (v, ..., v); S and m are the sums of the diagonal blocks / segments of S' and m'.  A tile
// then holds 64 rep rows of the input, so a narrow layer pays the per-tile latencies a quarter or an eighth as often.
// ------------------------------------------------------------------------------------------
template <int RM, bool QUANT>
__global__ __launch_bounds__(256, 2) void dense_moments_bwd_gram_kernel(const float *__restrict__ gm, const float *__restrict__ gs,
                                                                     const float *__restrict__ x, const float *__restrict__ f_in,
                                                                     int P, const float *__restrict__ w, float *__restrict__ dx,
                                                                     float *part, int64_t rows, int K, int N, int mode,
                                                                     const float *__restrict__ dx_add, int rep) {
    // the quantized input tile, then the dx tile (start-up: A in fp32); rows 68 words apart: 128-bit reads along a row, row
    // FAST_BM the sink of the idle staging slots
    __shared__ __attribute__((aligned(16))) float xs[FAST_BM + 1][FAST_XLD];
    __shared__ float adds[FAST_BM + 1][FAST_LD];  // the tile of dx_add (start-up: W diag(2 gs / rows))
    __shared__ __attribute__((aligned(16))) uint16_t Ap[3][64][BF_LD];  // A in bf16 parts, row j = column j (A is symmetric)
    __shared__ float ws[64][FAST_LD];             // W, zero beyond [K, N]
    __shared__ float vs[64], gms[64], gss[64];
    const bool has_add = dx_add != nullptr;
    const Mode m(mode);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, kq = lane >> 5;
    const int Ko = K / rep;  // rows of W; K is the width of a staged row
    const int K32 = (K + 31) >> 5, N32 = (N + 31) >> 5, Ko32 = (Ko + 31) >> 5;
    const int PK = QUANT ? P * K : 0;
    const int64_t M = (int64_t)Ko * N + N + PK;
    const int64_t n_tiles = (rows + FAST_BM - 1) / FAST_BM;
    float *my_dw = part + (int64_t)blockIdx.x * M;
    float *my_db = my_dw + (int64_t)Ko * N;
    float *my_df = my_db + N;
    const float inv_rows = 1.0f / ((float)rows * (float)rep);  // the statistics are over the rows of the input, not over the staged rows
    FastMap mx;
    mx.init(K);
    int fip[FAST_NJ];
    float gf[FAST_NJ][4];
#pragma unroll
    for (int j = 0; j < FAST_NJ; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e) gf[j][e] = 0.f;
    // Gram block of this wavefront: (k block, j block); with one k block the four wavefronts share it, a quarter of the
    // tile's rows each
    const int gblk = K32 * K32, gpb = 4 / gblk;
    const int gb = wave / gpb, gsub = wave % gpb;
    const int gib = gb / K32, gjb = gb % K32;
    const int grows = FAST_BM / gpb;
    floatx16 accS = {0};
    float accm = 0.f;
    const int bn = tid & 63, bq = tid >> 6;

    f32x4_t rx[FAST_NJ], rg[FAST_NJ];
    uint32_t xoff[FAST_NJ];
#pragma unroll
    for (int j = 0; j < FAST_NJ; ++j) xoff[j] = mx.on[j] ? (uint32_t)(mx.row[j] * K + mx.col[j]) * 4u : BUF_OOB;
    int64_t tile = blockIdx.x;
    auto load_tile = [&](int64_t t) {
        const int64_t r0 = t * FAST_BM, left = rows - r0, vr = left < FAST_BM ? left : FAST_BM;
        const __amdgpu_buffer_rsrc_t sx = buf_rsrc(x + r0 * K, vr * K * 4);
        const __amdgpu_buffer_rsrc_t sg = buf_rsrc(has_add ? dx_add + r0 * K : x, has_add ? vr * K * 4 : 0);
#pragma unroll
        for (int j = 0; j < FAST_NJ; ++j) {
            rx[j] = buf_ld4(sx, xoff[j]);
            rg[j] = buf_ld4(sg, xoff[j]);  // the other gradient of x, laid out like x (zeros without one)
        }
    };
    DB_STAMP(2, 0);
    if (tile < n_tiles) load_tile(tile);
    {
        // start-up under the first tile's latency: W, its scaled copy, the fractional bits; then A and v
        const __amdgpu_buffer_rsrc_t rs_w = buf_rsrc(w, (int64_t)Ko * N * 4);
        const __amdgpu_buffer_rsrc_t rs_m = buf_rsrc(gm, (int64_t)N * 4), rs_s = buf_rsrc(gs, (int64_t)N * 4);
        float wv[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) {
            const int id = tid + 256 * u, kk = id >> 6, nn = id & 63;
            wv[u] = buf_ld1(rs_w, (kk < Ko && nn < N) ? (uint32_t)(kk * N + nn) * 4u : BUF_OOB);
        }
        const float g1 = buf_ld1(rs_m, bn < N ? (uint32_t)bn * 4u : BUF_OOB), g2 = buf_ld1(rs_s, bn < N ? (uint32_t)bn * 4u : BUF_OOB);
        int fi[FAST_NJ][4], tix[FAST_NJ];
        fast_frac_bits<QUANT>(f_in, P, K, mx, m.round_params, fi, tix);
#pragma unroll
        for (int j = 0; j < FAST_NJ; ++j) fip[j] = pack_i8x4(fi[j]);
        const float sc = 2.0f * g2 * inv_rows;  // column bn = id & 63 of every entry this thread holds
#pragma unroll
        for (int u = 0; u < 16; ++u) {
            const int id = tid + 256 * u, kk = id >> 6, nn = id & 63;
            ws[kk][nn] = wv[u];
            adds[kk][nn] = wv[u] * sc;
            xs[kk][nn] = 0.f;
        }
        if (tid < 64) gms[tid] = g1, gss[tid] = g2;  // (zero past N: the loads are out of range there)
        __syncthreads();
        // A block (i block, j block) of this wavefront: sum over n of (W diag)[i][n] W[j][n]; blocks past K are zero
        {
            const int ib = wave & 1, jb = wave >> 1;
            floatx16 a = {0};
            a = mfma_chain(a, &adds[ib * 32 + l32][kq], 1, &ws[jb * 32 + l32][kq], 1, N32 * 2);
#pragma unroll
            for (int r = 0; r < 16; ++r) xs[ib * 32 + acc_row(r, lane)][jb * 32 + l32] = a[r];  // A in fp32, for now
        }
        {
            // v = W gm / rows: four threads per entry, a quarter of the columns each
            float sacc = 0.f;
            for (int n = 16 * bq; n < 16 * bq + 16; ++n) sacc += gms[n] * ws[bn][n];  // (gms is zero past N)
            adds[FAST_BM][0] = 0.f;  // (keeps the sink row defined)
            __syncthreads();         // the scaled copy of W in `adds` has been read by every A block
            adds[bq][bn] = sacc;
            __syncthreads();
            if (tid < 64) vs[tid] = ((adds[0][tid] + adds[1][tid]) + (adds[2][tid] + adds[3][tid])) * inv_rows;
        }
        // A (rep > 1: A' = diag(A, ..., A) and v' = (v, ..., v)) into bf16 parts, 64-bit stores of four entries; then the
        // input tile's place is cleared again: its columns past K must read as zero
        __syncthreads();
        float vv = 0.f;
        const int seg = rep > 1 ? Ko - 1 : 63;  // (rep > 1: Ko is a power of two, entry (kk, nn) of A' is entry (kk & seg, nn & seg) of A)
        if (tid < 64) vv = vs[tid & seg];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int id = tid + 256 * u, kk = id >> 4, n4 = (id & 15) << 2;
            // four consecutive columns lie in one diagonal block or in none (Ko is a multiple of 4)
            const bool in_block = rep > 1 ? (kk & ~seg) == (n4 & ~seg) : (kk < K && n4 < K);
            const f32x4_t a4 = *(const f32x4_t *)&xs[kk & seg][n4 & seg];
            uint32_t h4[4], m4[4], l4[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) bf16_parts(in_block ? a4[e] : 0.f, h4[e], m4[e], l4[e]);
            *(uint2 *)&Ap[0][kk][n4] = make_uint2(bf16_pair(h4[0], h4[1]), bf16_pair(h4[2], h4[3]));
            *(uint2 *)&Ap[1][kk][n4] = make_uint2(bf16_pair(m4[0], m4[1]), bf16_pair(m4[2], m4[3]));
            *(uint2 *)&Ap[2][kk][n4] = make_uint2(bf16_pair(l4[0], l4[1]), bf16_pair(l4[2], l4[3]));
        }
        __syncthreads();
        if (tid < 64) vs[tid] = vv;
#pragma unroll
        for (int u = 0; u < 16; ++u) {
            const int id = tid + 256 * u, kk = id >> 6, nn = id & 63;
            xs[kk][nn] = 0.f;
        }
    }
    __syncthreads();
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): nothing loaded before the loop is waited for inside it
    DB_STAMP(2, 1);
    [[maybe_unused]] int it_ = 0;
    for (; tile < n_tiles; tile += gridDim.x, ++it_) {
        float dlt[FAST_NJ][4];  // xq - x of the elements this thread stages
        __syncthreads();        // the previous tile's dx has been read back
        DB_STAMP(2, 2 + 6 * it_);
#pragma unroll
        for (int j = 0; j < FAST_NJ; ++j) {
            const float v[4] = {rx[j][0], rx[j][1], rx[j][2], rx[j][3]};
            const int xr = mx.on[j] ? mx.row[j] : FAST_BM;
            asm volatile("" : "+v"(fip[j]));
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int f = unpack_i8(fip[j], e);
                const float q = QUANT ? ldexpf(round_scaled<RM>(ldexpf(v[e], f)), -f) : v[e];
                dlt[j][e] = q - v[e];
                xs[xr][mx.col[j] + e] = q;
            }
            if (has_add) {
#pragma unroll
                for (int e = 0; e < 4; ++e) adds[xr][mx.col[j] + e] = rg[j][e];
            }
        }
        DB_STAMP(2, 3 + 6 * it_);
        __syncthreads();
        DB_STAMP(2, 4 + 6 * it_);
        const int64_t next = tile + gridDim.x;
        const int64_t r0 = tile * FAST_BM;
        if (next < n_tiles) load_tile(next);
        // ---- dx = xq A : (row half, k block); the quantized input usually has one bf16 part, A takes all three
        floatx16 acc = {0};
        const int rh = wave & 1, kb = wave >> 1;
        if (kb < K32) {
            // steps 16 bt + 8 kq + 0 .. 7 of a batch sit in one lane (both operands in the same order): the input row is read
            // with two 128-bit loads, A's parts with one each
#pragma unroll
            for (int bt = 0; bt < 4; ++bt) {
                if (bt < K32 * 2) {
                    const f32x4_t a0 = *(const f32x4_t *)&xs[rh * 32 + l32][16 * bt + 8 * kq], a1 = *(const f32x4_t *)&xs[rh * 32 + l32][16 * bt + 8 * kq + 4];
                    const float av[8] = {a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
                    u32x4_t pb[3], pa0;
#pragma unroll
                    for (int q = 0; q < 3; ++q) pb[q] = *(const u32x4_t *)&Ap[q][kb * 32 + l32][16 * bt + 8 * kq];
                    const bool one_a = bf16_lead8(av, pa0);
#pragma unroll
                    for (int q = 0; q < 3; ++q) acc = mfma_bf16(pa0, pb[q], acc);
                    if (!one_a) {
                        u32x4_t p1, p2;
                        const bool third = bf16_rest8(av, p1, p2);
#pragma unroll
                        for (int q = 0; q < 3; ++q) acc = mfma_bf16(p1, pb[q], acc);
                        if (third) {
#pragma unroll
                            for (int q = 0; q < 3; ++q) acc = mfma_bf16(p2, pb[q], acc);
                        }
                    }
                }
            }
        }
        // ---- S += xq^T xq : this wavefront's block over its rows of the tile (rows past the end are zeros)
        accS = mfma_chain_bf16<false, false>(accS, &xs[gsub * grows + kq][gib * 32 + l32], FAST_XLD, &xs[gsub * grows + kq][gjb * 32 + l32], FAST_XLD, grows / 16);
#pragma unroll
        for (int j = 0; j < FAST_BM / 4; ++j) accm += xs[bq * (FAST_BM / 4) + j][bn];
        DB_STAMP(2, 5 + 6 * it_);
        __syncthreads();  // xq consumed: the dx tile takes its place
        DB_STAMP(2, 6 + 6 * it_);
        if (kb < K32) {
#pragma unroll
            for (int r = 0; r < 16; ++r) xs[rh * 32 + acc_row(r, lane)][kb * 32 + l32] = acc[r];
        }
        __syncthreads();
        DB_STAMP(2, 7 + 6 * it_);
#pragma unroll
        for (int j = 0; j < FAST_NJ; ++j) {
            if (mx.on[j]) {
                const int64_t gr = r0 + mx.row[j];
                const f32x4_t t4 = *(const f32x4_t *)&xs[mx.row[j]][mx.col[j]];
                float4 o;
                o.x = t4[0] + vs[mx.col[j]], o.y = t4[1] + vs[mx.col[j] + 1], o.z = t4[2] + vs[mx.col[j] + 2], o.w = t4[3] + vs[mx.col[j] + 3];
                const float4 og = o;  // this contraction's own gradient: the one the rounding residue meets
                if (has_add) {
                    o.x += adds[mx.row[j]][mx.col[j]], o.y += adds[mx.row[j]][mx.col[j] + 1];
                    o.z += adds[mx.row[j]][mx.col[j] + 2], o.w += adds[mx.row[j]][mx.col[j] + 3];
                }
                if (gr < rows) {
                    st4(dx + gr * K + mx.col[j], o);
                    if (QUANT) {
                        gf[j][0] += -HGQ_LN2 * dlt[j][0] * og.x, gf[j][1] += -HGQ_LN2 * dlt[j][1] * og.y;
                        gf[j][2] += -HGQ_LN2 * dlt[j][2] * og.z, gf[j][3] += -HGQ_LN2 * dlt[j][3] * og.w;
                    }
                }
            }
        }
    }
    // ---- this workgroup's slice: S and m through LDS (wavefronts that share a Gram block add in a fixed order), then
    // dW = (m gm^T + 2 (S W) diag(gs)) / rows on the fp32 matrix instruction (both operands are arbitrary fp32)
    DB_STAMP(2, 30);
    __syncthreads();
    float *Ss = &xs[0][0];
    for (int pass = 0; pass < gpb; ++pass) {
        if (gsub == pass) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int k = gib * 32 + acc_row(r, lane), jx = gjb * 32 + l32;
                if (pass == 0) Ss[k * FAST_XLD + jx] = accS[r];
                else Ss[k * FAST_XLD + jx] += accS[r];
            }
        }
        __syncthreads();
    }
    float *bred = &adds[0][0];
    bred[tid] = accm;
    __syncthreads();
    if (tid < 64) vs[tid] = (bred[tid] + bred[tid + 64]) + (bred[tid + 128] + bred[tid + 192]);  // m (v is not needed any more)
    __syncthreads();
    if (rep > 1) {
        // S = sum of the diagonal blocks of S', m = sum of the segments of m', in block order, left in the first block
        for (int id = tid; id < Ko * Ko; id += 256) {
            const int i = id / Ko, jx = id % Ko;
            float sacc = Ss[i * FAST_XLD + jx];
            for (int q = 1; q < rep; ++q) sacc += Ss[(q * Ko + i) * FAST_XLD + q * Ko + jx];
            Ss[i * FAST_XLD + jx] = sacc;
        }
        float macc = 0.f;
        if (tid < Ko)
            for (int q = 0; q < rep; ++q) macc += vs[q * Ko + tid];
        __syncthreads();
        if (tid < Ko) vs[tid] = macc;
        __syncthreads();
    }
    {
        const int nb2 = Ko32 * N32;
        if (wave < nb2) {
            const int wkb = wave / N32, wnb = wave % N32;
            floatx16 t = {0};
            t = mfma_chain(t, &Ss[(wkb * 32 + l32) * FAST_XLD + kq], 1, &ws[kq][wnb * 32 + l32], FAST_LD, Ko32 * 2);
            const int c = wnb * 32 + l32;
            const float g1 = gms[c], g2 = gss[c];
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int k = wkb * 32 + acc_row(r, lane);
                if (k < Ko && c < N) my_dw[k * N + c] = (vs[k] * g1 + 2.0f * g2 * t[r]) * inv_rows;
            }
        }
    }
    if (tid < N) my_db[tid] = 0.f;
    if (QUANT) {
        // fractional-bit gradient: every (tile row, column) has one owner thread; rows that share a table row are
        // added in row order (few table rows: four threads per entry, a quarter of the tile each, as in the kernel above)
        float *gt = &adds[0][0];
        __syncthreads();
#pragma unroll
        for (int j = 0; j < FAST_NJ; ++j)
            if (mx.on[j])
#pragma unroll
                for (int e = 0; e < 4; ++e) gt[mx.row[j] * FAST_LD + mx.col[j] + e] = gf[j][e];
        __syncthreads();
        if (P <= 16) {
            float *quarter = &ws[0][0];  // (W has been used)
            for (int id = tid; id < 4 * P * 64; id += 256) {
                const int c = id & 63, pq = id >> 6, p = pq & (P - 1), q = pq / P;
                float sacc = 0.f;
                for (int r = 16 * q + p; r < 16 * q + 16; r += P) sacc += gt[r * FAST_LD + c];
                quarter[pq * 64 + c] = sacc;
            }
            __syncthreads();
            for (int id = tid; id < P * 64; id += 256) {
                const int p = id >> 6, c = id & 63;
                if (c < K)
                    my_df[p * K + c] = (quarter[p * 64 + c] + quarter[(P + p) * 64 + c]) + (quarter[(2 * P + p) * 64 + c] + quarter[(3 * P + p) * 64 + c]);
            }
        } else {
#pragma unroll 4
            for (int id = tid; id < P * 64; id += 256) {
                const int p = id >> 6, c = id & 63;
                if (c < K) {
                    float sacc = 0.f;
                    for (int r = p; r < FAST_BM; r += P) sacc += gt[r * FAST_LD + c];
                    my_df[p * K + c] = sacc;
                }
            }
        }
    }
    DB_STAMP(2, 31);
}

// out[e] = sum over slices of part[g][e], in slice order.  256 threads = 64 elements x 4 slice groups.
#define RP_G 16  // slice groups per entry: 64 entries x 16 groups = 1024 threads, few dependent load batches per thread
__global__ __launch_bounds__(64 * RP_G) void reduce_parts_kernel(const float *__restrict__ part, int n_parts, int64_t M,
                                                                 float *dqw, int64_t n_dqw, float *dqb, int64_t n_dqb,
                                                                 float *df, int64_t n_df, float scale) {
    __shared__ float red[64 * RP_G];
    const int e_local = threadIdx.x & 63, grp = threadIdx.x >> 6;
    const int64_t e = (int64_t)blockIdx.x * 64 + e_local;
    float s = 0.f;
    if (e < M) {
        const int per = (n_parts + RP_G - 1) / RP_G;
        const int g0 = grp * per, g1 = min(n_parts, g0 + per);
        // eight independent loads in flight per thread: the loop is latency-bound otherwise
        int g = g0;
        for (; g + 8 <= g1; g += 8) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = part[(int64_t)(g + u) * M + e];
            s += ((v[0] + v[1]) + (v[2] + v[3])) + ((v[4] + v[5]) + (v[6] + v[7]));
        }
        for (; g < g1; ++g) s += part[(int64_t)g * M + e];
    }
    red[threadIdx.x] = s;
    __syncthreads();
    if (grp == 0 && e < M) {
        float v = 0.f;  // groups in order
#pragma unroll
        for (int w = 0; w < RP_G; w += 4)
            v += (red[e_local + 64 * w] + red[e_local + 64 * (w + 1)]) + (red[e_local + 64 * (w + 2)] + red[e_local + 64 * (w + 3)]);
        v *= scale;
        if (e < n_dqw) {
            if (dqw) dqw[e] = v;
        } else if (e < n_dqw + n_dqb) {
            if (dqb) dqb[e - n_dqw] = v;
        } else if (df) {
            df[e - n_dqw - n_dqb] = v;
        }
    }
}

int reduce_parts(const float *part, int n_parts, int64_t M, float *dqw, int64_t n_dqw, float *dqb, int64_t n_dqb, float *df,
                 int64_t n_df, hipStream_t s, float scale) {
    hipLaunchKernelGGL(reduce_parts_kernel, dim3((unsigned)((M + 63) / 64)), dim3(64 * RP_G), 0, s, part, n_parts, M, dqw, n_dqw, dqb, n_dqb, df, n_df, scale);
    return check_launch("reduce_parts");
}

// The same reduction for several independent slice sets in one launch: block b serves the set whose block range holds b.
struct ReduceBatch {
    hgq_reduce_item item[HGQ_REDUCE_BATCH];
    int first_block[HGQ_REDUCE_BATCH + 1];
    int count;
};

// quantizers whose upstream gradient IS a reduced segment (the kernel / bias quantizers behind a contraction): their surrogate
// backward runs on the sum as it is formed; attach[t][o] = index into `item` for segment o of slice set t, or -1
struct ReduceQuants {
    hgq_quant_grad_item item[HGQ_REDUCE_QUANTS];
    int8_t attach[HGQ_REDUCE_BATCH][3];
};

template <bool QUANTS>
__global__ __launch_bounds__(64 * RP_G) void reduce_parts_multi_kernel(const ReduceBatch b, const ReduceQuants q) {
    __shared__ float red[64 * RP_G];
    int t = 0;
    while (t + 1 < b.count && (int)blockIdx.x >= b.first_block[t + 1]) ++t;
    const hgq_reduce_item &it = b.item[t];
    const float *__restrict__ part = it.slices;
    const int n_parts = it.n_slices;
    const int64_t M = it.width;
    const int e_local = threadIdx.x & 63, grp = threadIdx.x >> 6;
    const int64_t e = (int64_t)((int)blockIdx.x - b.first_block[t]) * 64 + e_local;
    float s = 0.f;
    if (e < M) {
        const int per = (n_parts + RP_G - 1) / RP_G;
        const int g0 = grp * per, g1 = min(n_parts, g0 + per);
        int g = g0;
        for (; g + 8 <= g1; g += 8) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = part[(int64_t)(g + u) * M + e];
            s += ((v[0] + v[1]) + (v[2] + v[3])) + ((v[4] + v[5]) + (v[6] + v[7]));
        }
        for (; g < g1; ++g) s += part[(int64_t)g * M + e];
    }
    red[threadIdx.x] = s;
    __syncthreads();
    if (grp == 0 && e < M) {
        float v = 0.f;  // groups in order: the same association as reduce_parts_kernel
#pragma unroll
        for (int w = 0; w < RP_G; w += 4)
            v += (red[e_local + 64 * w] + red[e_local + 64 * (w + 1)]) + (red[e_local + 64 * (w + 2)] + red[e_local + 64 * (w + 3)]);
        int64_t off = e;
#pragma unroll
        for (int o = 0; o < 3; ++o) {
            if (off < it.n_out[o]) {
                if (it.out[o]) it.out[o][off] = v;
                if (QUANTS && q.attach[t][o] >= 0) {
                    // (the arithmetic of quant_bwd_multi_kernel on dy = v)
                    const hgq_quant_grad_item &qi = q.item[q.attach[t][o]];
                    const Mode m(qi.mode);
                    const KIF p = resolve_kif(load_k(qi.k, off, m.k_u8), qi.i[off], qi.fb[off], m.kbi, m.round_params);
                    float gx, gi, gf;
                    quantize_grad_dyn(qi.x[off], v, p, m.round_mode, m.overflow_mode, gx, gi, gf);
                    if (m.kbi) gi -= gf;
                    if (qi.dx) qi.dx[off] = gx;
                    if (qi.di) qi.di[off] = gi;
                    if (qi.dfb) qi.dfb[off] = gf;
                }
                break;
            }
            off -= it.n_out[o];
        }
    }
}

static int reduce_slices_impl(const hgq_reduce_item *items, int count, const hgq_quant_grad_item *quants, const int *quant_set,
                              const int *quant_segment, int n_quants, void *stream) {
    const char *who = n_quants ? "hgq_reduce_slices_quant_multi" : "hgq_reduce_slices_multi";
    if (count < 0 || (count > 0 && !items) || n_quants < 0 || (n_quants > 0 && (!quants || !quant_set || !quant_segment)))
        return fail(HGQ_ERR_ARG, "%s: bad arguments", who);
    for (int j = 0; j < n_quants; ++j) {
        const hgq_quant_grad_item &qi = quants[j];
        if (quant_set[j] < 0 || quant_set[j] >= count || quant_segment[j] < 0 || quant_segment[j] > 2 || !qi.x || !qi.k || !qi.i || !qi.fb ||
            qi.n != items[quant_set[j]].n_out[quant_segment[j]])
            return fail(HGQ_ERR_ARG, "%s: quantizer %d does not fit the segment it is attached to", who, j);
        if (!Mode(qi.mode).training) return fail(HGQ_ERR_ARG, "%s: quantizer %d: the surrogate gradient is defined for training mode only", who, j);
    }
    for (int base = 0; base < count; base += HGQ_REDUCE_BATCH) {
        ReduceBatch b;
        ReduceQuants q;
        b.count = count - base < HGQ_REDUCE_BATCH ? count - base : HGQ_REDUCE_BATCH;
        for (int t = 0; t < HGQ_REDUCE_BATCH; ++t) q.attach[t][0] = q.attach[t][1] = q.attach[t][2] = -1;
        int nq = 0;
        for (int j = 0; j < n_quants; ++j) {
            if (quant_set[j] < base || quant_set[j] >= base + b.count) continue;
            if (nq == HGQ_REDUCE_QUANTS) return fail(HGQ_ERR_UNSUPPORTED, "%s: more than %d quantizers on %d slice sets", who, HGQ_REDUCE_QUANTS, HGQ_REDUCE_BATCH);
            if (q.attach[quant_set[j] - base][quant_segment[j]] >= 0) return fail(HGQ_ERR_ARG, "%s: two quantizers on one segment", who);
            q.attach[quant_set[j] - base][quant_segment[j]] = (int8_t)nq;
            q.item[nq++] = quants[j];
        }
        int64_t blocks = 0;
        for (int t = 0; t < b.count; ++t) {
            const hgq_reduce_item &it = items[base + t];
            if (it.n_slices < 1 || it.width < 1 || !it.slices) return fail(HGQ_ERR_ARG, "%s: bad sizes in item %d", who, base + t);
            if (it.n_out[0] < 0 || it.n_out[1] < 0 || it.n_out[2] < 0 || it.n_out[0] + it.n_out[1] + it.n_out[2] != it.width)
                return fail(HGQ_ERR_ARG, "%s: item %d: output lengths do not add up to the slice width", who, base + t);
            b.item[t] = it;
            b.first_block[t] = (int)blocks;
            blocks += (it.width + 63) / 64;
            if (blocks > (1 << 24)) return fail(HGQ_ERR_UNSUPPORTED, "%s: too many columns", who);
        }
        for (int t = b.count; t <= HGQ_REDUCE_BATCH; ++t) b.first_block[t] = (int)blocks;
        if (nq) hipLaunchKernelGGL(reduce_parts_multi_kernel<true>, dim3((unsigned)blocks), dim3(64 * RP_G), 0, (hipStream_t)stream, b, q);
        else hipLaunchKernelGGL(reduce_parts_multi_kernel<false>, dim3((unsigned)blocks), dim3(64 * RP_G), 0, (hipStream_t)stream, b, q);
        int rc = check_launch(who);
        if (rc) return rc;
    }
    return HGQ_OK;
}

extern "C" int hgq_reduce_slices_multi(const hgq_reduce_item *items, int count, void *stream) {
    return reduce_slices_impl(items, count, nullptr, nullptr, nullptr, 0, stream);
}

extern "C" int hgq_reduce_slices_quant_multi(const hgq_reduce_item *items, int count, const hgq_quant_grad_item *quants, const int *quant_set,
                                             const int *quant_segment, int n_quants, void *stream) {
    return reduce_slices_impl(items, count, quants, quant_set, quant_segment, n_quants, stream);
}

static inline bool aligned16(const void *p) { return ((uintptr_t)p & 15u) == 0; }

static inline int row_parts(int64_t rows, int bm) {
    const int64_t n_tiles = (rows + bm - 1) / bm;
    int g = persistent_grid(n_tiles, 2);
    if (g > MAX_PARTS) g = MAX_PARTS;
    return g;
}

}  // namespace hgq

using namespace hgq;

#ifdef DB_PROF
extern "C" int hgq_db_prof_read(unsigned long long *out) {
    return hipMemcpyFromSymbol(out, HIP_SYMBOL(db_prof_stamps), sizeof(unsigned long long) * 3 * 4 * 32) == hipSuccess ? 0 : -2;
}
#endif

// 1: the streaming dense kernels contract on the bf16 matrix cores by exact splitting; 0: on the fp32 ones
static int g_dense_bf16 = 1;
extern "C" int hgq_dense_use_bf16_parts(int on) {
    const int was = g_dense_bf16;
    if (on >= 0) g_dense_bf16 = on ? 1 : 0;
    return was;
}

extern "C" int hgq_qdense_fwd_parts(int64_t rows) { return rows > 0 ? row_parts(rows, FWD_BM) : 1; }

extern "C" int64_t hgq_qdense_bwd_workspace(int64_t rows, int K, int N, int64_t bw_rows) {
    const int64_t M = (int64_t)K * N + N + bw_rows * (int64_t)K;
    return (rows > 0 ? row_parts(rows, BWD_BM) : 1) * M;
}

extern "C" int hgq_qdense_fwd(const float *x, const void *k_in, const float *i_in, const float *f_in, int64_t bw_rows,
                              const float *qw, const float *qb, float *y, uint32_t *amax_part, int64_t rows, int K, int N,
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
    const int amax_lds = (quant && amax_part && PK <= AMAX_LDS_MAX) ? 1 : 0;
    const size_t dyn = amax_lds ? (size_t)PK * 4 : 0;
    const int vec_ok = (K % 4 == 0) && aligned16(x);
    const bool wrap_train = quant && m.overflow_mode == HGQ_WRAP && m.training && !m.kbi;
    const bool fast = (!quant || wrap_train) && K <= 64 && N <= 64 && K % 4 == 0 && aligned16(x) &&
                      (!quant || (bw_rows <= 64 && 64 % bw_rows == 0));
    if (fast) {
        const dim3 fgrid((unsigned)row_parts(rows, FWD_BM));
        const int P = quant ? (int)bw_rows : 1;
#define HGQ_FWD_BF16(NSV) \
    do { \
        if (!quant) hipLaunchKernelGGL((qdense_fwd_bf16_kernel<HGQ_TRN, false, NSV>), fgrid, dim3(256), 0, s, x, f_in, P, qw, qb, y, (uint32_t *)nullptr, rows, K, N, act, mode); \
        else if (m.round_mode == HGQ_TRN) hipLaunchKernelGGL((qdense_fwd_bf16_kernel<HGQ_TRN, true, NSV>), fgrid, dim3(256), 0, s, x, f_in, P, qw, qb, y, amax_part, rows, K, N, act, mode); \
        else if (m.round_mode == HGQ_RND) hipLaunchKernelGGL((qdense_fwd_bf16_kernel<HGQ_RND, true, NSV>), fgrid, dim3(256), 0, s, x, f_in, P, qw, qb, y, amax_part, rows, K, N, act, mode); \
        else hipLaunchKernelGGL((qdense_fwd_bf16_kernel<HGQ_RND_CONV, true, NSV>), fgrid, dim3(256), 0, s, x, f_in, P, qw, qb, y, amax_part, rows, K, N, act, mode); \
    } while (0)
        if (g_dense_bf16) {
            if (K <= 16) HGQ_FWD_BF16(1);
            else if (K <= 32) HGQ_FWD_BF16(2);
            else if (K <= 48) HGQ_FWD_BF16(3);
            else HGQ_FWD_BF16(4);
            return check_launch("hgq_qdense_fwd");
        }
#undef HGQ_FWD_BF16
#define HGQ_FWD_FAST(NS4V) \
    do { \
        if (!quant) hipLaunchKernelGGL((qdense_fwd_fast_kernel<HGQ_TRN, false, NS4V>), fgrid, dim3(256), 0, s, x, f_in, P, qw, qb, y, (uint32_t *)nullptr, rows, K, N, act, mode); \
        else if (m.round_mode == HGQ_TRN) hipLaunchKernelGGL((qdense_fwd_fast_kernel<HGQ_TRN, true, NS4V>), fgrid, dim3(256), 0, s, x, f_in, P, qw, qb, y, amax_part, rows, K, N, act, mode); \
        else if (m.round_mode == HGQ_RND) hipLaunchKernelGGL((qdense_fwd_fast_kernel<HGQ_RND, true, NS4V>), fgrid, dim3(256), 0, s, x, f_in, P, qw, qb, y, amax_part, rows, K, N, act, mode); \
        else hipLaunchKernelGGL((qdense_fwd_fast_kernel<HGQ_RND_CONV, true, NS4V>), fgrid, dim3(256), 0, s, x, f_in, P, qw, qb, y, amax_part, rows, K, N, act, mode); \
    } while (0)
        if (K <= 8) HGQ_FWD_FAST(1);
        else if (K <= 16) HGQ_FWD_FAST(2);
        else if (K <= 32) HGQ_FWD_FAST(4);
        else HGQ_FWD_FAST(8);
#undef HGQ_FWD_FAST
        return check_launch("hgq_qdense_fwd");
    }
    const dim3 grid((unsigned)row_parts(rows, FWD_BM), (unsigned)((N + FWD_BN - 1) / FWD_BN));
    if (!quant) {
        hipLaunchKernelGGL((qdense_fwd_kernel<HGQ_TRN, HGQ_WRAP, false>), grid, dim3(256), dyn, s, x, k_in, i_in, f_in, (int64_t)1, qw, qb, y,
                           (uint32_t *)nullptr, rows, K, N, act, mode, vec_ok, amax_lds);
    } else {
        HGQ_DISPATCH_RM_OM(m.round_mode, m.overflow_mode, {
            hipLaunchKernelGGL((qdense_fwd_kernel<RM, OM, true>), grid, dim3(256), dyn, s, x, k_in, i_in, f_in, bw_rows, qw, qb, y, amax_part,
                               rows, K, N, act, mode, vec_ok, amax_lds);
        });
    }
    return check_launch("hgq_qdense_fwd");
}

// 1 if hgq_qdense_fwd_oq covers the shape and modes
extern "C" int hgq_qdense_fwd_oq_supported(int64_t rows, int K, int N, int64_t bw_rows, int64_t bw_rows_out, int mode, int mode_out) {
    const Mode m(mode), mo(mode_out);
    const bool wrap_in = m.overflow_mode == HGQ_WRAP && m.training && !m.kbi;
    const bool wrap_out = mo.overflow_mode == HGQ_WRAP && mo.training && !mo.kbi;
    return g_dense_bf16 && rows > 0 && K >= 1 && N >= 1 && K <= 64 && N <= 64 && K % 4 == 0 && N % 4 == 0 && wrap_in && wrap_out &&
           m.round_mode == mo.round_mode && (m.round_mode == HGQ_TRN || m.round_mode == HGQ_RND || m.round_mode == HGQ_RND_CONV) &&
           bw_rows > 0 && bw_rows <= 64 && 64 % bw_rows == 0 && rows % bw_rows == 0 &&
           bw_rows_out > 0 && bw_rows_out <= 64 && 64 % bw_rows_out == 0 && rows % bw_rows_out == 0;
}

extern "C" int hgq_qdense_fwd_oq(const float *x, const float *f_in, int64_t bw_rows, const float *qw, const float *qb, const float *f_out,
                                 int64_t bw_rows_out, float *y, float *yq, uint32_t *amax_part, uint32_t *oamax_part, int64_t rows,
                                 int K, int N, int act, int mode, int mode_out, void *stream) {
    hipStream_t s = (hipStream_t)stream;
    if (rows == 0) return HGQ_OK;
    if (!hgq_qdense_fwd_oq_supported(rows, K, N, bw_rows, bw_rows_out, mode, mode_out))
        return fail(HGQ_ERR_UNSUPPORTED, "hgq_qdense_fwd_oq: shape or modes outside the fused output quantizer (see hgq_qdense_fwd_oq_supported)");
    if (!x || !f_in || !qw || !f_out || !y || !yq || !oamax_part) return fail(HGQ_ERR_ARG, "hgq_qdense_fwd_oq: null pointer");
    if (act != HGQ_ACT_NONE && act != HGQ_ACT_RELU) return fail(HGQ_ERR_ARG, "hgq_qdense_fwd_oq: unknown activation %d", act);
    if (!aligned16(x) || !aligned16(y) || !aligned16(yq) || !aligned16(oamax_part))
        return fail(HGQ_ERR_ARG, "hgq_qdense_fwd_oq: x, y, yq and the tracker slices must be 16-byte aligned");
    const Mode m(mode);
    const dim3 fgrid((unsigned)row_parts(rows, FWD_BM));
    const int P = (int)bw_rows, Po = (int)bw_rows_out;
#define HGQ_FWD_OQ(NSV) \
    do { \
        if (m.round_mode == HGQ_TRN) hipLaunchKernelGGL((qdense_fwd_bf16_kernel<HGQ_TRN, true, NSV, true>), fgrid, dim3(256), 0, s, x, f_in, P, qw, qb, y, amax_part, rows, K, N, act, mode, f_out, Po, mode_out, yq, oamax_part); \
        else if (m.round_mode == HGQ_RND) hipLaunchKernelGGL((qdense_fwd_bf16_kernel<HGQ_RND, true, NSV, true>), fgrid, dim3(256), 0, s, x, f_in, P, qw, qb, y, amax_part, rows, K, N, act, mode, f_out, Po, mode_out, yq, oamax_part); \
        else hipLaunchKernelGGL((qdense_fwd_bf16_kernel<HGQ_RND_CONV, true, NSV, true>), fgrid, dim3(256), 0, s, x, f_in, P, qw, qb, y, amax_part, rows, K, N, act, mode, f_out, Po, mode_out, yq, oamax_part); \
    } while (0)
    if (K <= 16) HGQ_FWD_OQ(1);
    else if (K <= 32) HGQ_FWD_OQ(2);
    else if (K <= 48) HGQ_FWD_OQ(3);
    else HGQ_FWD_OQ(4);
#undef HGQ_FWD_OQ
    return check_launch("hgq_qdense_fwd_oq");
}

// 1 if hgq_qdense_fwd_mean covers the shape and mode
extern "C" int hgq_qdense_fwd_mean_supported(int64_t rows, int K, int N, int64_t bw_rows, int64_t mean_rows, int mode) {
    const Mode m(mode);
    const bool quant = bw_rows > 0;
    const bool wrap_in = m.overflow_mode == HGQ_WRAP && m.training && !m.kbi;
    return g_dense_bf16 && rows > 0 && K >= 1 && N >= 1 && K <= 64 && N <= 64 && K % 4 == 0 && N % 4 == 0 &&
           (mean_rows == 32 || mean_rows == 64) && rows % mean_rows == 0 &&
           (!quant || (wrap_in && (m.round_mode == HGQ_TRN || m.round_mode == HGQ_RND || m.round_mode == HGQ_RND_CONV) && bw_rows <= 64 &&
                       64 % bw_rows == 0 && rows % bw_rows == 0));
}

extern "C" int hgq_qdense_fwd_mean(const float *x, const float *f_in, int64_t bw_rows, const float *qw, const float *qb,
                                   uint32_t *relu_mask, float *ymean, uint32_t *amax_part, int64_t rows, int K, int N, int64_t mean_rows,
                                   int act, int mode, void *stream) {
    hipStream_t s = (hipStream_t)stream;
    if (rows == 0) return HGQ_OK;
    if (bw_rows < 0 || !hgq_qdense_fwd_mean_supported(rows, K, N, bw_rows, mean_rows, mode))
        return fail(HGQ_ERR_UNSUPPORTED, "hgq_qdense_fwd_mean: shape or mode outside the fused group mean (see hgq_qdense_fwd_mean_supported)");
    if (!x || !qw || !ymean || (bw_rows > 0 && !f_in)) return fail(HGQ_ERR_ARG, "hgq_qdense_fwd_mean: null pointer");
    if (act != HGQ_ACT_NONE && act != HGQ_ACT_RELU) return fail(HGQ_ERR_ARG, "hgq_qdense_fwd_mean: unknown activation %d", act);
    if (act == HGQ_ACT_RELU && !relu_mask) return fail(HGQ_ERR_ARG, "hgq_qdense_fwd_mean: a ReLU needs the mask array");
    if (!aligned16(x)) return fail(HGQ_ERR_ARG, "hgq_qdense_fwd_mean: x must be 16-byte aligned");
    const Mode m(mode);
    const bool quant = bw_rows > 0;
    const dim3 fgrid((unsigned)row_parts(rows, FWD_BM));
    const int P = quant ? (int)bw_rows : 1, mr = (int)mean_rows;
#define HGQ_FWD_MEAN(NSV) \
    do { \
        if (!quant) hipLaunchKernelGGL((qdense_fwd_bf16_kernel<HGQ_TRN, false, NSV, false, true>), fgrid, dim3(256), 0, s, x, f_in, P, qw, qb, (float *)nullptr, (uint32_t *)nullptr, rows, K, N, act, mode, (const float *)nullptr, 1, 0, (float *)nullptr, (uint32_t *)nullptr, ymean, mr, relu_mask); \
        else if (m.round_mode == HGQ_TRN) hipLaunchKernelGGL((qdense_fwd_bf16_kernel<HGQ_TRN, true, NSV, false, true>), fgrid, dim3(256), 0, s, x, f_in, P, qw, qb, (float *)nullptr, amax_part, rows, K, N, act, mode, (const float *)nullptr, 1, 0, (float *)nullptr, (uint32_t *)nullptr, ymean, mr, relu_mask); \
        else if (m.round_mode == HGQ_RND) hipLaunchKernelGGL((qdense_fwd_bf16_kernel<HGQ_RND, true, NSV, false, true>), fgrid, dim3(256), 0, s, x, f_in, P, qw, qb, (float *)nullptr, amax_part, rows, K, N, act, mode, (const float *)nullptr, 1, 0, (float *)nullptr, (uint32_t *)nullptr, ymean, mr, relu_mask); \
        else hipLaunchKernelGGL((qdense_fwd_bf16_kernel<HGQ_RND_CONV, true, NSV, false, true>), fgrid, dim3(256), 0, s, x, f_in, P, qw, qb, (float *)nullptr, amax_part, rows, K, N, act, mode, (const float *)nullptr, 1, 0, (float *)nullptr, (uint32_t *)nullptr, ymean, mr, relu_mask); \
    } while (0)
    if (K <= 16) HGQ_FWD_MEAN(1);
    else if (K <= 32) HGQ_FWD_MEAN(2);
    else if (K <= 48) HGQ_FWD_MEAN(3);
    else HGQ_FWD_MEAN(4);
#undef HGQ_FWD_MEAN
    return check_launch("hgq_qdense_fwd_mean");
}

extern "C" int64_t hgq_qdense_moments_workspace(int64_t rows, int K, int N, int64_t bw_rows) {
    if (rows < 0 || K < 1 || N < 1 || bw_rows < 0) return -1;
    const int64_t parts = rows > 0 ? row_parts(rows, FAST_BM) : 1;
    const int64_t fwd = parts * 2 * N, bwd = parts * ((int64_t)K * N + N + bw_rows * K);
    return fwd > bwd ? fwd : bwd;
}

extern "C" int64_t hgq_dense_moments_workspace(int64_t rows, int K, int N) { return hgq_qdense_moments_workspace(rows, K, N, 0); }

static int moments_check(const char *who, int64_t rows, int K, int N, const void *x, const float *f_in, int64_t bw_rows, int mode) {
    if (rows < 1 || K < 1 || N < 1 || bw_rows < 0) return fail(HGQ_ERR_ARG, "%s: bad sizes", who);
    if (K > 64 || N > 64 || K % 4 != 0 || N % 4 != 0 || !aligned16(x))
        return fail(HGQ_ERR_UNSUPPORTED, "%s: needs K, N <= 64, multiples of 4, and a 16-byte aligned input (K=%d N=%d)", who, K, N);
    if (bw_rows > 0) {
        const Mode m(mode);
        if (!f_in) return fail(HGQ_ERR_ARG, "%s: null bit-width pointer", who);
        if (!(m.overflow_mode == HGQ_WRAP && m.training && !m.kbi))
            return fail(HGQ_ERR_UNSUPPORTED, "%s: the fused input quantizer must be a training-mode WRAP (k, i, f) quantizer", who);
        if (bw_rows > 64 || 64 % bw_rows != 0 || rows % bw_rows != 0)
            return fail(HGQ_ERR_UNSUPPORTED, "%s: bw_rows=%lld must divide 64 and rows", who, (long long)bw_rows);
        if (m.round_mode != HGQ_TRN && m.round_mode != HGQ_RND && m.round_mode != HGQ_RND_CONV) return fail(HGQ_ERR_ARG, "%s: unknown round mode", who);
    }
    return HGQ_OK;
}

extern "C" int hgq_qdense_moments_fwd(const float *x, const float *f_in, int64_t bw_rows, int mode, const float *w, float *mean,
                                      float *meansq, float *workspace, int64_t rows, int K, int N, void *stream) {
    hipStream_t s = (hipStream_t)stream;
    int rc = moments_check("hgq_qdense_moments_fwd", rows, K, N, x, f_in, bw_rows, mode);
    if (rc) return rc;
    if (!x || !w || !mean || !meansq || !workspace) return fail(HGQ_ERR_ARG, "hgq_qdense_moments_fwd: null pointer");
    const int parts = row_parts(rows, FAST_BM);
    const dim3 grid((unsigned)parts);
    const bool quant = bw_rows > 0;
    const int P = quant ? (int)bw_rows : 1;
    const int rm = Mode(mode).round_mode;
#define HGQ_MOM_BF16(NSV) \
    do { \
        if (!quant) hipLaunchKernelGGL((dense_moments_bf16_kernel<HGQ_TRN, false, NSV>), grid, dim3(256), 0, s, x, f_in, P, w, workspace, rows, K, N, mode); \
        else if (rm == HGQ_TRN) hipLaunchKernelGGL((dense_moments_bf16_kernel<HGQ_TRN, true, NSV>), grid, dim3(256), 0, s, x, f_in, P, w, workspace, rows, K, N, mode); \
        else if (rm == HGQ_RND) hipLaunchKernelGGL((dense_moments_bf16_kernel<HGQ_RND, true, NSV>), grid, dim3(256), 0, s, x, f_in, P, w, workspace, rows, K, N, mode); \
        else hipLaunchKernelGGL((dense_moments_bf16_kernel<HGQ_RND_CONV, true, NSV>), grid, dim3(256), 0, s, x, f_in, P, w, workspace, rows, K, N, mode); \
    } while (0)
#define HGQ_MOM_FAST(NS4V) \
    do { \
        if (!quant) hipLaunchKernelGGL((dense_moments_fast_kernel<HGQ_TRN, false, NS4V>), grid, dim3(256), 0, s, x, f_in, P, w, workspace, rows, K, N, mode); \
        else if (rm == HGQ_TRN) hipLaunchKernelGGL((dense_moments_fast_kernel<HGQ_TRN, true, NS4V>), grid, dim3(256), 0, s, x, f_in, P, w, workspace, rows, K, N, mode); \
        else if (rm == HGQ_RND) hipLaunchKernelGGL((dense_moments_fast_kernel<HGQ_RND, true, NS4V>), grid, dim3(256), 0, s, x, f_in, P, w, workspace, rows, K, N, mode); \
        else hipLaunchKernelGGL((dense_moments_fast_kernel<HGQ_RND_CONV, true, NS4V>), grid, dim3(256), 0, s, x, f_in, P, w, workspace, rows, K, N, mode); \
    } while (0)
    if (g_dense_bf16) {
        if (K <= 16) HGQ_MOM_BF16(1);
        else if (K <= 32) HGQ_MOM_BF16(2);
        else if (K <= 48) HGQ_MOM_BF16(3);
        else HGQ_MOM_BF16(4);
    } else if (K <= 8) HGQ_MOM_FAST(1);
    else if (K <= 16) HGQ_MOM_FAST(2);
    else if (K <= 32) HGQ_MOM_FAST(4);
    else HGQ_MOM_FAST(8);
#undef HGQ_MOM_FAST
#undef HGQ_MOM_BF16
    if ((rc = check_launch("hgq_qdense_moments_fwd"))) return rc;
    // the sums leave the reduction scaled by 1 / rows: mean and mean of squares
    return reduce_parts(workspace, parts, 2 * (int64_t)N, mean, (int64_t)N, meansq, (int64_t)N, nullptr, 0, s, 1.0f / (float)rows);
}

extern "C" int hgq_dense_moments_fwd(const float *x, const float *w, float *mean, float *meansq, float *workspace, int64_t rows,
                                     int K, int N, void *stream) {
    return hgq_qdense_moments_fwd(x, nullptr, 0, 0, w, mean, meansq, workspace, rows, K, N, stream);
}

extern "C" int hgq_qdense_moments_bwd(const float *x, const float *f_in, int64_t bw_rows, int mode, const float *w, const float *dmean,
                                      const float *dmeansq, const float *dx_add, float *dx, float *dw, float *df_in, float *workspace,
                                      int64_t rows, int K, int N, void *stream) {
    hipStream_t s = (hipStream_t)stream;
    int rc = moments_check("hgq_qdense_moments_bwd", rows, K, N, x, f_in, bw_rows, mode);
    if (rc) return rc;
    if (!x || !w || !dmean || !dmeansq || !dx || !workspace) return fail(HGQ_ERR_ARG, "hgq_qdense_moments_bwd: null pointer");
    if (!aligned16(dx) || !aligned16(dx_add)) return fail(HGQ_ERR_UNSUPPORTED, "hgq_qdense_moments_bwd: dx and dx_add must be 16-byte aligned");
    const int parts = row_parts(rows, BWD_BM);
    const bool quant = bw_rows > 0;
    const int P = quant ? (int)bw_rows : 1;
    const int rm = Mode(mode).round_mode;
    const dim3 grid((unsigned)parts);
    // a narrow input as rows of 64: rep rows side by side (the table of fractional bits folds the same way)
    int rep = 1;
    if (g_dense_bf16 && (K == 8 || K == 16 || K == 32) && rows % (64 / K) == 0 && (!quant || bw_rows % (64 / K) == 0)) rep = 64 / K;
#define HGQ_MOM_BWD(RMV, QV) \
    do { \
        if (g_dense_bf16) hipLaunchKernelGGL((dense_moments_bwd_gram_kernel<RMV, QV>), grid, dim3(256), 0, s, dmean, dmeansq, x, f_in, quant ? P / rep : 1, w, dx, workspace, rows / rep, K * rep, N, mode, dx_add, rep); \
        else hipLaunchKernelGGL((qdense_bwd_fast_kernel<RMV, QV, true>), grid, dim3(256), 0, s, dmean, dmeansq, x, f_in, P, w, dx, workspace, 0, rows, K, N, HGQ_ACT_NONE, mode, dx_add); \
    } while (0)
    if (!quant) HGQ_MOM_BWD(HGQ_TRN, false);
    else if (rm == HGQ_TRN) HGQ_MOM_BWD(HGQ_TRN, true);
    else if (rm == HGQ_RND) HGQ_MOM_BWD(HGQ_RND, true);
    else HGQ_MOM_BWD(HGQ_RND_CONV, true);
#undef HGQ_MOM_BWD
    if ((rc = check_launch("hgq_qdense_moments_bwd"))) return rc;
    if (!dw) return HGQ_OK;  // the slices stay in the workspace for the caller's own reduction
    const int64_t PK = bw_rows * (int64_t)K;
    return reduce_parts(workspace, parts, (int64_t)K * N + N + PK, dw, (int64_t)K * N, nullptr, (int64_t)N, quant ? df_in : (float *)nullptr, PK, s);
}

extern "C" int hgq_dense_moments_bwd(const float *x, const float *w, const float *dmean, const float *dmeansq, float *dx, float *dw,
                                     float *workspace, int64_t rows, int K, int N, void *stream) {
    return hgq_qdense_moments_bwd(x, nullptr, 0, 0, w, dmean, dmeansq, nullptr, dx, dw, nullptr, workspace, rows, K, N, stream);
}

// Launches the backward kernel; the slices are reduced here (reduce == true) or left in the workspace for the caller.
static int qdense_bwd_impl(const float *dy, const float *y, const float *x, const float *f_in, int64_t bw_rows, const float *qw, float *dx,
                           float *dqw, float *dqb, float *df_in, float *workspace, int64_t rows, int K, int N, int act, int mode,
                           void *stream, bool reduce, int64_t mean_rows = 0) {
    hipStream_t s = (hipStream_t)stream;
    if (mean_rows != 0 && mean_rows != 32 && mean_rows != 64) return fail(HGQ_ERR_UNSUPPORTED, "hgq_qdense_bwd_mean: groups of 32 or 64 rows only");
    if (mean_rows && rows % mean_rows != 0) return fail(HGQ_ERR_ARG, "hgq_qdense_bwd_mean: rows=%lld not a multiple of mean_rows=%lld", (long long)rows, (long long)mean_rows);
    const int bcast = (int)mean_rows;
    if (rows < 0 || K < 1 || N < 1 || bw_rows < 0) return fail(HGQ_ERR_ARG, "hgq_qdense_bwd: bad sizes");
    if (K > 64 || N > 64) return fail(HGQ_ERR_UNSUPPORTED, "hgq_qdense_bwd: K=%d N=%d exceed the fused kernel's 64 x 64", K, N);
    if (!dy || !x || !qw || !dx || !workspace) return fail(HGQ_ERR_ARG, "hgq_qdense_bwd: null pointer");
    if (act == HGQ_ACT_RELU && !y) return fail(HGQ_ERR_ARG, "hgq_qdense_bwd: relu needs the forward output");
    if (act != HGQ_ACT_NONE && act != HGQ_ACT_RELU) return fail(HGQ_ERR_ARG, "hgq_qdense_bwd: unknown activation %d", act);
    const Mode m(mode);
    const bool quant = bw_rows > 0;
    if (quant && !(m.overflow_mode == HGQ_WRAP && m.training))
        return fail(HGQ_ERR_UNSUPPORTED, "hgq_qdense_bwd: the fused input quantizer must be a training-mode WRAP quantizer");
    if (quant && !f_in) return fail(HGQ_ERR_ARG, "hgq_qdense_bwd: null bit-width pointer");
    if (quant && rows % bw_rows != 0) return fail(HGQ_ERR_ARG, "hgq_qdense_bwd: rows not a multiple of bw_rows");
    const int64_t PK = bw_rows * (int64_t)K;
    const int64_t M = (int64_t)K * N + N + PK;
    if (rows == 0) {
        int rc;
        if (!reduce) return fill_f32(workspace, 0.f, M, s);  // one slice of zeros
        if (dqw && (rc = fill_f32(dqw, 0.f, (int64_t)K * N, s))) return rc;
        if (dqb && (rc = fill_f32(dqb, 0.f, N, s))) return rc;
        if (df_in && (rc = fill_f32(df_in, 0.f, PK, s))) return rc;
        return HGQ_OK;
    }
    const bool fast = K % 4 == 0 && aligned16(x) && aligned16(dx) && (!quant || (bw_rows <= 64 && 64 % bw_rows == 0));
    if (fast) {
        const int parts = row_parts(rows, BWD_BM);
        const int P = quant ? (int)bw_rows : 1;
        const dim3 fgrid((unsigned)parts);
        const bool zvec = N % 4 == 0 && aligned16(dy) && (act != HGQ_ACT_RELU || bcast || aligned16(y));
        if (bcast && !(zvec && g_dense_bf16))
            return fail(HGQ_ERR_UNSUPPORTED, "hgq_qdense_bwd_mean: needs the bf16 matrix instruction, N a multiple of 4 and 16-byte aligned gradients");
#define HGQ_BWD_BCAST(RMV, QV, BC)                                                                                                     \
    do {                                                                                                                               \
        if (K > 32 && N > 32)                                                                                                          \
            hipLaunchKernelGGL((qdense_bwd_fast_kernel<RMV, QV, false, true, true, true, BC>), fgrid, dim3(256), 0, s, dy, y, x, f_in, P, qw, dx, \
                               workspace, dqb ? 1 : 0, rows, K, N, act, mode, (const float *)nullptr);                                 \
        else                                                                                                                           \
            hipLaunchKernelGGL((qdense_bwd_fast_kernel<RMV, QV, false, true, true, false, BC>), fgrid, dim3(256), 0, s, dy, y, x, f_in, P, qw, dx, \
                               workspace, dqb ? 1 : 0, rows, K, N, act, mode, (const float *)nullptr);                                 \
    } while (0)
#define HGQ_BWD_BCAST_RM(BC)                                                                                                           \
    do {                                                                                                                               \
        if (!quant) HGQ_BWD_BCAST(HGQ_TRN, false, BC);                                                                                 \
        else if (m.round_mode == HGQ_TRN) HGQ_BWD_BCAST(HGQ_TRN, true, BC);                                                            \
        else if (m.round_mode == HGQ_RND) HGQ_BWD_BCAST(HGQ_RND, true, BC);                                                            \
        else HGQ_BWD_BCAST(HGQ_RND_CONV, true, BC);                                                                                    \
    } while (0)
#define HGQ_BWD_FAST(RMV, QV)                                                                                                          \
    do {                                                                                                                               \
        if (zvec && g_dense_bf16 && K > 32 && N > 32 && act == HGQ_ACT_NONE)                                                           \
            hipLaunchKernelGGL((qdense_bwd_fast_kernel<RMV, QV, false, true, true, true, 0, true>), fgrid, dim3(256), 0, s, dy, y, x, f_in, P, qw, dx, \
                               workspace, dqb ? 1 : 0, rows, K, N, act, mode, (const float *)nullptr);                                 \
        else if (zvec && g_dense_bf16 && K > 32 && N > 32)                                                                             \
            hipLaunchKernelGGL((qdense_bwd_fast_kernel<RMV, QV, false, true, true, true>), fgrid, dim3(256), 0, s, dy, y, x, f_in, P, qw, dx, workspace, \
                               dqb ? 1 : 0, rows, K, N, act, mode, (const float *)nullptr);                                            \
        else if (zvec && g_dense_bf16)                                                                                                 \
            hipLaunchKernelGGL((qdense_bwd_fast_kernel<RMV, QV, false, true, true>), fgrid, dim3(256), 0, s, dy, y, x, f_in, P, qw, dx, workspace, \
                               dqb ? 1 : 0, rows, K, N, act, mode, (const float *)nullptr);                                            \
        else if (zvec)                                                                                                                 \
            hipLaunchKernelGGL((qdense_bwd_fast_kernel<RMV, QV, false, true>), fgrid, dim3(256), 0, s, dy, y, x, f_in, P, qw, dx, workspace, \
                               dqb ? 1 : 0, rows, K, N, act, mode, (const float *)nullptr);                                            \
        else if (g_dense_bf16)                                                                                                         \
            hipLaunchKernelGGL((qdense_bwd_fast_kernel<RMV, QV, false, false, true>), fgrid, dim3(256), 0, s, dy, y, x, f_in, P, qw, dx, workspace, \
                               dqb ? 1 : 0, rows, K, N, act, mode, (const float *)nullptr);                                            \
        else                                                                                                                           \
            hipLaunchKernelGGL((qdense_bwd_fast_kernel<RMV, QV, false, false>), fgrid, dim3(256), 0, s, dy, y, x, f_in, P, qw, dx, workspace, \
                               dqb ? 1 : 0, rows, K, N, act, mode, (const float *)nullptr);                                            \
    } while (0)
        if (bcast == 64) HGQ_BWD_BCAST_RM(64);
        else if (bcast == 32) HGQ_BWD_BCAST_RM(32);
        else if (!quant) HGQ_BWD_FAST(HGQ_TRN, false);
        else if (m.round_mode == HGQ_TRN) HGQ_BWD_FAST(HGQ_TRN, true);
        else if (m.round_mode == HGQ_RND) HGQ_BWD_FAST(HGQ_RND, true);
        else HGQ_BWD_FAST(HGQ_RND_CONV, true);
#undef HGQ_BWD_FAST
#undef HGQ_BWD_BCAST_RM
#undef HGQ_BWD_BCAST
        int rc = check_launch("hgq_qdense_bwd");
        if (rc || !reduce) return rc;
        return reduce_parts(workspace, parts, M, dqw, (int64_t)K * N, dqb, (int64_t)N, quant ? df_in : (float *)nullptr, PK, s);
    }
    if (bcast) return fail(HGQ_ERR_UNSUPPORTED, "hgq_qdense_bwd_mean: K must be a multiple of 4 and x / dx 16-byte aligned");
    const int df_lds = (quant && PK <= DF_LDS_MAX) ? 1 : 0;
    const size_t dyn = df_lds ? (size_t)PK * 4 : 0;
    const int parts = row_parts(rows, BWD_BM);
    const dim3 grid((unsigned)parts);
    typedef void (*bwd_fn)(const float *, const float *, const float *, const float *, int64_t, const float *, float *, float *, int,
                           int64_t, int, int, int, int, int);
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
    hipLaunchKernelGGL(fn, grid, dim3(256), dyn, s, dy, y, x, f_in, quant ? bw_rows : (int64_t)1, qw, dx, workspace, dqb ? 1 : 0, rows, K, N,
                       act, mode, df_lds);
    int rc = check_launch("hgq_qdense_bwd");
    if (rc || !reduce) return rc;
    hipLaunchKernelGGL(reduce_parts_kernel, dim3((unsigned)((M + 63) / 64)), dim3(64 * RP_G), 0, s, workspace, parts, M, dqw, (int64_t)K * N, dqb,
                       (int64_t)N, quant ? df_in : (float *)nullptr, PK, 1.0f);
    return check_launch("hgq_qdense_bwd(reduce)");
}

extern "C" int hgq_qdense_bwd(const float *dy, const float *y, const float *x, const float *f_in, int64_t bw_rows,
                              const float *qw, float *dx, float *dqw, float *dqb, float *df_in, float *workspace,
                              int64_t rows, int K, int N, int act, int mode, void *stream) {
    return qdense_bwd_impl(dy, y, x, f_in, bw_rows, qw, dx, dqw, dqb, df_in, workspace, rows, K, N, act, mode, stream, true);
}

extern "C" int hgq_qdense_bwd_mean(const float *dmean, const uint32_t *relu_mask, const float *x, const float *f_in, int64_t bw_rows, const float *qw,
                                   float *dx, float *dqw, float *dqb, float *df_in, float *workspace, int64_t rows, int K, int N,
                                   int64_t mean_rows, int act, int mode, void *stream) {
    if (mean_rows <= 0) return fail(HGQ_ERR_ARG, "hgq_qdense_bwd_mean: mean_rows must be positive");
    return qdense_bwd_impl(dmean, (const float *)relu_mask, x, f_in, bw_rows, qw, dx, dqw, dqb, df_in, workspace, rows, K, N, act, mode, stream, true,
                           mean_rows);
}

extern "C" int hgq_qdense_bwd_mean_slices(const float *dmean, const uint32_t *relu_mask, const float *x, const float *f_in, int64_t bw_rows,
                                          const float *qw, float *dx, float *workspace, int has_bias, int64_t rows, int K, int N,
                                          int64_t mean_rows, int act, int mode, void *stream) {
    if (mean_rows <= 0) return fail(HGQ_ERR_ARG, "hgq_qdense_bwd_mean_slices: mean_rows must be positive");
    return qdense_bwd_impl(dmean, (const float *)relu_mask, x, f_in, bw_rows, qw, dx, nullptr, has_bias ? workspace : nullptr, nullptr, workspace, rows,
                           K, N, act, mode, stream, false, mean_rows);
}

extern "C" int hgq_qdense_bwd_slices(const float *dy, const float *y, const float *x, const float *f_in, int64_t bw_rows,
                                     const float *qw, float *dx, float *workspace, int has_bias, int64_t rows, int K, int N, int act,
                                     int mode, void *stream) {
    // the kernels only test the bias pointer for "is there a bias": any non-null value stands for it
    return qdense_bwd_impl(dy, y, x, f_in, bw_rows, qw, dx, nullptr, has_bias ? workspace : nullptr, nullptr, workspace, rows, K, N, act, mode,
                           stream, false);
}
