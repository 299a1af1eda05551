// The two score contractions of QMultiHeadAttention for rank-3 inputs, one workgroup per
// (batch, head) pair, on fp32 MFMA:
//
//   scores[b, n, t, s] = sum_h query[b, t, n, h] * key[b, s, n, h]          ('aecd,abcd->acbe')
//   out[b, t, n, h]    = sum_s probs[b, n, t, s] * value[b, s, n, h]        ('acbe,aecd->abcd')
//
// and their gradients.  query / key / value / out are the projections' outputs in their own
// layout [B, seq, N, H] (rows of one head are N * H floats apart), so no transposed copies are
// made; every operand of a pair (at most 64 x 64) is staged once in LDS and read by the MFMAs
// either way round.  T, S, H <= 64.
//
// MFMA 32x32x2 fp32 operand layout (64 lanes): A[i][k]: i = lane % 32, k = lane / 32;
// B[k][j]: k = lane / 32, j = lane % 32; D[i][j] in 16 registers: j = lane % 32,
// i = (r / 4) * 8 + (lane / 32) * 4 + (r % 4).
#include "hgq_device.h"
#include "hgq_host.h"

namespace hgq {

typedef float floatx16 __attribute__((ext_vector_type(16)));
#define AT_LD 65
typedef float AtTile[64][AT_LD];

__device__ __forceinline__ int at_acc_row(int r, int lane) { return (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3); }

// C block (rb, cb) of sum_k A(i, k) B(k, j), k < K2 (even); TA / TB read the LDS tile transposed.
template <bool TA, bool TB>
__device__ __forceinline__ floatx16 tile_mma(const AtTile &As, const AtTile &Bs, int K2, int rb, int cb, int lane) {
    floatx16 acc = {0};
    const int i = rb * 32 + (lane & 31), j = cb * 32 + (lane & 31), kq = lane >> 5;
    for (int k = 0; k < K2; k += 2) {
        const float a = TA ? As[k + kq][i] : As[i][k + kq];
        const float b = TB ? Bs[j][k + kq] : Bs[k + kq][j];
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc, 0, 0, 0);
    }
    return acc;
}

// Stage a [R, W] operand whose rows are `ld` floats apart into a zero-padded 64 x 64 tile.
__device__ __forceinline__ void stage(AtTile &dst, const float *__restrict__ src, int R, int W, int64_t ld) {
    for (int id = threadIdx.x; id < 64 * 64; id += 256) {
        const int r = id >> 6, c = id & 63;
        dst[r][c] = (r < R && c < W) ? src[(int64_t)r * ld + c] : 0.f;
    }
}

// Store C block (rb, cb) to a [R, W] destination with row stride ld.
__device__ __forceinline__ void store_block(const floatx16 &acc, float *__restrict__ dst, int R, int W, int64_t ld, int rb,
                                            int cb, int lane) {
    const int j = cb * 32 + (lane & 31);
    if (j >= W) return;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int i = rb * 32 + at_acc_row(r, lane);
        if (i < R) dst[(int64_t)i * ld + j] = acc[r];
    }
}

struct AttnDims {
    int B, T, S, N, H;
};

__global__ __launch_bounds__(256) void attn_scores_fwd_kernel(const float *__restrict__ q, const float *__restrict__ k,
                                                              float *__restrict__ scores, AttnDims d) {
    __shared__ AtTile qs, ks;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, rb = wave & 1, cb = wave >> 1;
    const int64_t ld = (int64_t)d.N * d.H;
    for (int64_t pair = blockIdx.x; pair < (int64_t)d.B * d.N; pair += gridDim.x) {
        const int64_t b = pair / d.N, n = pair % d.N;
        __syncthreads();
        stage(qs, q + (b * d.T * d.N + n) * d.H, d.T, d.H, ld);
        stage(ks, k + (b * d.S * d.N + n) * d.H, d.S, d.H, ld);
        __syncthreads();
        const floatx16 acc = tile_mma<false, true>(qs, ks, (d.H + 1) & ~1, rb, cb, lane);
        store_block(acc, scores + pair * d.T * d.S, d.T, d.S, d.S, rb, cb, lane);
    }
}

__global__ __launch_bounds__(256) void attn_combine_fwd_kernel(const float *__restrict__ p, const float *__restrict__ v,
                                                               float *__restrict__ out, AttnDims d) {
    __shared__ AtTile ps, vs;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, rb = wave & 1, cb = wave >> 1;
    const int64_t ld = (int64_t)d.N * d.H;
    for (int64_t pair = blockIdx.x; pair < (int64_t)d.B * d.N; pair += gridDim.x) {
        const int64_t b = pair / d.N, n = pair % d.N;
        __syncthreads();
        stage(ps, p + pair * d.T * d.S, d.T, d.S, d.S);
        stage(vs, v + (b * d.S * d.N + n) * d.H, d.S, d.H, ld);
        __syncthreads();
        if (cb * 32 < d.H) {
            const floatx16 acc = tile_mma<false, false>(ps, vs, (d.S + 1) & ~1, rb, cb, lane);
            store_block(acc, out + (b * d.T * d.N + n) * d.H, d.T, d.H, ld, rb, cb, lane);
        }
    }
}

// dp = dout v^T,  dv = p^T dout
__global__ __launch_bounds__(256) void attn_combine_bwd_kernel(const float *__restrict__ dout, const float *__restrict__ p,
                                                               const float *__restrict__ v, float *__restrict__ dp,
                                                               float *__restrict__ dv, AttnDims d) {
    __shared__ AtTile ps, vs, gs;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, rb = wave & 1, cb = wave >> 1;
    const int64_t ld = (int64_t)d.N * d.H;
    for (int64_t pair = blockIdx.x; pair < (int64_t)d.B * d.N; pair += gridDim.x) {
        const int64_t b = pair / d.N, n = pair % d.N;
        __syncthreads();
        stage(ps, p + pair * d.T * d.S, d.T, d.S, d.S);
        stage(vs, v + (b * d.S * d.N + n) * d.H, d.S, d.H, ld);
        stage(gs, dout + (b * d.T * d.N + n) * d.H, d.T, d.H, ld);
        __syncthreads();
        if (dp) {
            const floatx16 acc = tile_mma<false, true>(gs, vs, (d.H + 1) & ~1, rb, cb, lane);
            store_block(acc, dp + pair * d.T * d.S, d.T, d.S, d.S, rb, cb, lane);
        }
        if (dv && cb * 32 < d.H) {
            const floatx16 acc = tile_mma<true, false>(ps, gs, (d.T + 1) & ~1, rb, cb, lane);
            store_block(acc, dv + (b * d.S * d.N + n) * d.H, d.S, d.H, ld, rb, cb, lane);
        }
    }
}

// dq = ds k,  dk = ds^T q
__global__ __launch_bounds__(256) void attn_scores_bwd_kernel(const float *__restrict__ ds, const float *__restrict__ q,
                                                              const float *__restrict__ k, float *__restrict__ dq,
                                                              float *__restrict__ dk, AttnDims d) {
    __shared__ AtTile ss, qs, ks;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, rb = wave & 1, cb = wave >> 1;
    const int64_t ld = (int64_t)d.N * d.H;
    for (int64_t pair = blockIdx.x; pair < (int64_t)d.B * d.N; pair += gridDim.x) {
        const int64_t b = pair / d.N, n = pair % d.N;
        __syncthreads();
        stage(ss, ds + pair * d.T * d.S, d.T, d.S, d.S);
        stage(qs, q + (b * d.T * d.N + n) * d.H, d.T, d.H, ld);
        stage(ks, k + (b * d.S * d.N + n) * d.H, d.S, d.H, ld);
        __syncthreads();
        if (cb * 32 < d.H) {
            if (dq) {
                const floatx16 acc = tile_mma<false, false>(ss, ks, (d.S + 1) & ~1, rb, cb, lane);
                store_block(acc, dq + (b * d.T * d.N + n) * d.H, d.T, d.H, ld, rb, cb, lane);
            }
            if (dk) {
                const floatx16 acc = tile_mma<true, false>(ss, qs, (d.T + 1) & ~1, rb, cb, lane);
                store_block(acc, dk + (b * d.S * d.N + n) * d.H, d.S, d.H, ld, rb, cb, lane);
            }
        }
    }
}

static int check_dims(int B, int T, int S, int N, int H, const char *who, AttnDims &d) {
    if (B < 0 || T < 1 || S < 1 || N < 1 || H < 1) return fail(HGQ_ERR_ARG, "%s: bad sizes", who);
    if (T > 64 || S > 64 || H > 64)
        return fail(HGQ_ERR_UNSUPPORTED, "%s: sequence lengths and head size up to 64 are supported (T=%d S=%d H=%d)", who, T, S, H);
    d.B = B, d.T = T, d.S = S, d.N = N, d.H = H;
    return HGQ_OK;
}

static unsigned pair_grid(const AttnDims &d) { return (unsigned)persistent_grid((int64_t)d.B * d.N, 16); }

}  // namespace hgq

using namespace hgq;

extern "C" int hgq_attn_scores_fwd(const float *query, const float *key, float *scores, int B, int T, int S, int N, int H,
                                   void *stream) {
    AttnDims d;
    int rc = check_dims(B, T, S, N, H, "hgq_attn_scores_fwd", d);
    if (rc) return rc;
    if (B == 0) return HGQ_OK;
    if (!query || !key || !scores) return fail(HGQ_ERR_ARG, "hgq_attn_scores_fwd: null pointer");
    hipLaunchKernelGGL(attn_scores_fwd_kernel, dim3(pair_grid(d)), dim3(256), 0, (hipStream_t)stream, query, key, scores, d);
    return check_launch("hgq_attn_scores_fwd");
}

extern "C" int hgq_attn_scores_bwd(const float *dscores, const float *query, const float *key, float *dquery, float *dkey,
                                   int B, int T, int S, int N, int H, void *stream) {
    AttnDims d;
    int rc = check_dims(B, T, S, N, H, "hgq_attn_scores_bwd", d);
    if (rc) return rc;
    if (B == 0) return HGQ_OK;
    if (!dscores || !query || !key) return fail(HGQ_ERR_ARG, "hgq_attn_scores_bwd: null pointer");
    hipLaunchKernelGGL(attn_scores_bwd_kernel, dim3(pair_grid(d)), dim3(256), 0, (hipStream_t)stream, dscores, query, key, dquery, dkey, d);
    return check_launch("hgq_attn_scores_bwd");
}

extern "C" int hgq_attn_combine_fwd(const float *probs, const float *value, float *out, int B, int T, int S, int N, int H,
                                    void *stream) {
    AttnDims d;
    int rc = check_dims(B, T, S, N, H, "hgq_attn_combine_fwd", d);
    if (rc) return rc;
    if (B == 0) return HGQ_OK;
    if (!probs || !value || !out) return fail(HGQ_ERR_ARG, "hgq_attn_combine_fwd: null pointer");
    hipLaunchKernelGGL(attn_combine_fwd_kernel, dim3(pair_grid(d)), dim3(256), 0, (hipStream_t)stream, probs, value, out, d);
    return check_launch("hgq_attn_combine_fwd");
}

extern "C" int hgq_attn_combine_bwd(const float *dout, const float *probs, const float *value, float *dprobs, float *dvalue,
                                    int B, int T, int S, int N, int H, void *stream) {
    AttnDims d;
    int rc = check_dims(B, T, S, N, H, "hgq_attn_combine_bwd", d);
    if (rc) return rc;
    if (B == 0) return HGQ_OK;
    if (!dout || !probs || !value) return fail(HGQ_ERR_ARG, "hgq_attn_combine_bwd: null pointer");
    hipLaunchKernelGGL(attn_combine_bwd_kernel, dim3(pair_grid(d)), dim3(256), 0, (hipStream_t)stream, dout, probs, value, dprobs, dvalue, d);
    return check_launch("hgq_attn_combine_bwd");
}
