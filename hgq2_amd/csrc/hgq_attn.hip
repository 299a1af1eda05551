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

typedef float f32x4_a __attribute__((ext_vector_type(4)));

__device__ __forceinline__ int at_acc_row(int r, int lane) { return (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3); }

// An operand tile in LDS: 64 rows of `ld` floats (ld odd, >= padded width + 1), zero padded.
struct Tile {
    float *p;
    int ld;
    __device__ __forceinline__ float at(int r, int c) const { return p[r * ld + c]; }
};
__host__ __device__ inline int tile_ld(int W) { return ((W + 3) & ~3) + 1; }

// C block (rb, cb) of sum_k A(i, k) B(k, j), k < K2 (even); TA / TB read the LDS tile transposed.
template <bool TA, bool TB>
__device__ __forceinline__ floatx16 tile_mma(const Tile &A, const Tile &B, int K2, int rb, int cb, int lane) {
    floatx16 acc = {0};
    const int i = rb * 32 + (lane & 31), j = cb * 32 + (lane & 31), kq = lane >> 5;
    for (int k = 0; k < K2; k += 2) {
        const float a = TA ? A.at(k + kq, i) : A.at(i, k + kq);
        const float b = TB ? B.at(j, k + kq) : B.at(k + kq, j);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc, 0, 0, 0);
    }
    return acc;
}

// Stage a [R, W] operand whose rows are `ld` floats apart into a tile, zero padded to 64 rows and
// to a multiple of 4 columns; 128-bit loads when W is a multiple of 4 and the rows are aligned.
__device__ __forceinline__ void stage(const Tile &t, const float *__restrict__ src, int R, int W, int64_t ld) {
    const int W4 = (W + 3) >> 2;
    const bool vec = (W & 3) == 0 && (ld & 3) == 0 && ((uintptr_t)src & 15u) == 0;
    for (int id = threadIdx.x; id < 64 * W4; id += 256) {
        const int r = id / W4, c = (id - r * W4) << 2;
        float v[4] = {0.f, 0.f, 0.f, 0.f};
        if (r < R) {
            if (vec) {
                const f32x4_a q = __builtin_nontemporal_load((const f32x4_a *)(src + (int64_t)r * ld + c));
                v[0] = q.x, v[1] = q.y, v[2] = q.z, v[3] = q.w;
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (c + e < W) v[e] = src[(int64_t)r * ld + c + e];
            }
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) t.p[r * t.ld + c + e] = v[e];
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

// One workgroup per (batch, head) pair; dynamic LDS holds the operand tiles back to back.
#define AT_PROLOGUE                                                                             \
    extern __shared__ float lds[];                                                              \
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, rb = wave & 1, cb = wave >> 1; \
    const int64_t ld = (int64_t)d.N * d.H;                                                      \
    const int64_t pair = blockIdx.x, b = pair / d.N, n = pair % d.N;                            \
    const int ldh = tile_ld(d.H), lds_ = tile_ld(d.S);                                          \
    (void)lds_, (void)ldh

__global__ __launch_bounds__(256) void attn_scores_fwd_kernel(const float *__restrict__ q, const float *__restrict__ k,
                                                              float *__restrict__ scores, AttnDims d) {
    AT_PROLOGUE;
    const Tile qs = {lds, ldh}, ks = {lds + 64 * ldh, ldh};
    stage(qs, q + (b * d.T * d.N + n) * d.H, d.T, d.H, ld);
    stage(ks, k + (b * d.S * d.N + n) * d.H, d.S, d.H, ld);
    __syncthreads();
    const floatx16 acc = tile_mma<false, true>(qs, ks, (d.H + 1) & ~1, rb, cb, lane);
    store_block(acc, scores + pair * d.T * d.S, d.T, d.S, d.S, rb, cb, lane);
}

__global__ __launch_bounds__(256) void attn_combine_fwd_kernel(const float *__restrict__ p, const float *__restrict__ v,
                                                               float *__restrict__ out, AttnDims d) {
    AT_PROLOGUE;
    const Tile ps = {lds, lds_}, vs = {lds + 64 * lds_, ldh};
    stage(ps, p + pair * d.T * d.S, d.T, d.S, d.S);
    stage(vs, v + (b * d.S * d.N + n) * d.H, d.S, d.H, ld);
    __syncthreads();
    if (cb * 32 < d.H) {
        const floatx16 acc = tile_mma<false, false>(ps, vs, (d.S + 1) & ~1, rb, cb, lane);
        store_block(acc, out + (b * d.T * d.N + n) * d.H, d.T, d.H, ld, rb, cb, lane);
    }
}

// dp = dout v^T,  dv = p^T dout
__global__ __launch_bounds__(256) void attn_combine_bwd_kernel(const float *__restrict__ dout, const float *__restrict__ p,
                                                               const float *__restrict__ v, float *__restrict__ dp,
                                                               float *__restrict__ dv, AttnDims d) {
    AT_PROLOGUE;
    const Tile ps = {lds, lds_}, vs = {lds + 64 * lds_, ldh}, gs = {lds + 64 * lds_ + 64 * ldh, ldh};
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

// dq = ds k,  dk = ds^T q
__global__ __launch_bounds__(256) void attn_scores_bwd_kernel(const float *__restrict__ ds, const float *__restrict__ q,
                                                              const float *__restrict__ k, float *__restrict__ dq,
                                                              float *__restrict__ dk, AttnDims d) {
    AT_PROLOGUE;
    const Tile ss = {lds, lds_}, qs = {lds + 64 * lds_, ldh}, ks = {lds + 64 * lds_ + 64 * ldh, ldh};
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

static int check_dims(int B, int T, int S, int N, int H, const char *who, AttnDims &d) {
    if (B < 0 || T < 1 || S < 1 || N < 1 || H < 1) return fail(HGQ_ERR_ARG, "%s: bad sizes", who);
    if ((int64_t)B * N >= (1ll << 31)) return fail(HGQ_ERR_UNSUPPORTED, "%s: too many (batch, head) pairs", who);
    if (T > 64 || S > 64 || H > 64)
        return fail(HGQ_ERR_UNSUPPORTED, "%s: sequence lengths and head size up to 64 are supported (T=%d S=%d H=%d)", who, T, S, H);
    d.B = B, d.T = T, d.S = S, d.N = N, d.H = H;
    return HGQ_OK;
}

static unsigned pair_grid(const AttnDims &d) { return (unsigned)((int64_t)d.B * d.N); }
static size_t lds_bytes(int n_h, int n_s, const AttnDims &d) { return (size_t)64 * (n_h * tile_ld(d.H) + n_s * tile_ld(d.S)) * sizeof(float); }

}  // namespace hgq

using namespace hgq;

extern "C" int hgq_attn_scores_fwd(const float *query, const float *key, float *scores, int B, int T, int S, int N, int H,
                                   void *stream) {
    AttnDims d;
    int rc = check_dims(B, T, S, N, H, "hgq_attn_scores_fwd", d);
    if (rc) return rc;
    if (B == 0) return HGQ_OK;
    if (!query || !key || !scores) return fail(HGQ_ERR_ARG, "hgq_attn_scores_fwd: null pointer");
    hipLaunchKernelGGL(attn_scores_fwd_kernel, dim3(pair_grid(d)), dim3(256), lds_bytes(2, 0, d), (hipStream_t)stream, query, key, scores, d);
    return check_launch("hgq_attn_scores_fwd");
}

extern "C" int hgq_attn_scores_bwd(const float *dscores, const float *query, const float *key, float *dquery, float *dkey,
                                   int B, int T, int S, int N, int H, void *stream) {
    AttnDims d;
    int rc = check_dims(B, T, S, N, H, "hgq_attn_scores_bwd", d);
    if (rc) return rc;
    if (B == 0) return HGQ_OK;
    if (!dscores || !query || !key) return fail(HGQ_ERR_ARG, "hgq_attn_scores_bwd: null pointer");
    hipLaunchKernelGGL(attn_scores_bwd_kernel, dim3(pair_grid(d)), dim3(256), lds_bytes(2, 1, d), (hipStream_t)stream, dscores, query, key, dquery, dkey, d);
    return check_launch("hgq_attn_scores_bwd");
}

extern "C" int hgq_attn_combine_fwd(const float *probs, const float *value, float *out, int B, int T, int S, int N, int H,
                                    void *stream) {
    AttnDims d;
    int rc = check_dims(B, T, S, N, H, "hgq_attn_combine_fwd", d);
    if (rc) return rc;
    if (B == 0) return HGQ_OK;
    if (!probs || !value || !out) return fail(HGQ_ERR_ARG, "hgq_attn_combine_fwd: null pointer");
    hipLaunchKernelGGL(attn_combine_fwd_kernel, dim3(pair_grid(d)), dim3(256), lds_bytes(1, 1, d), (hipStream_t)stream, probs, value, out, d);
    return check_launch("hgq_attn_combine_fwd");
}

extern "C" int hgq_attn_combine_bwd(const float *dout, const float *probs, const float *value, float *dprobs, float *dvalue,
                                    int B, int T, int S, int N, int H, void *stream) {
    AttnDims d;
    int rc = check_dims(B, T, S, N, H, "hgq_attn_combine_bwd", d);
    if (rc) return rc;
    if (B == 0) return HGQ_OK;
    if (!dout || !probs || !value) return fail(HGQ_ERR_ARG, "hgq_attn_combine_bwd: null pointer");
    hipLaunchKernelGGL(attn_combine_bwd_kernel, dim3(pair_grid(d)), dim3(256), lds_bytes(2, 1, d), (hipStream_t)stream, dout, probs, value, dprobs, dvalue, d);
    return check_launch("hgq_attn_combine_bwd");
}
