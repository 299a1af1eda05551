// Two small row-streaming kernel families that the einsum and batch-normalisation layers need beside the dense kernels:
//
//   grouped dense     y[r, g, :] = act(x[r, g, :] W[g] + bias[g])      x [R, G, K], W [G, K, N], y [R, G, N]
//                     (an einsum whose kernel carries an axis of the input with it, e.g. 'Babc,bcd->Babd': one small
//                     kernel matrix per position b; reference tests/test_dense.py:56, src/hgq/layers/core/einsum_dense.py:72-93)
//   per-channel affine y[r, c] = x[r, c] * s[c] + o[c]                 (QBatchNormalization, reference
//                     src/hgq/layers/batch_normalization.py:184) with d/ds, d/do as fixed-order sums over the rows
//
// and the elementwise arithmetic the Quantizer wrapper puts around its internal quantizer (reference
// src/hgq/quantizer/quantizer.py:49-60): the division by the scaler in front, and behind it the multiplication by the scaler,
// the quantization-noise blend and the affine map as ONE pass each way.
//
// K, N <= 64 per group: the operands of a (row tile, group) pair sit in LDS, every output is one thread's sequential sum
// (a multiplication and an addition per step, in k order), gradients that are sums over the rows leave as one slice per
// workgroup and are added in a fixed order by reduce_parts.  These are HBM-bound shapes; nothing is reshaped to reach the
// matrix cores.
#include "hgq_device.h"
#include "hgq_host.h"

namespace hgq {

#define GD_TR 64    // rows per tile
#define GD_NT 256
#define GD_MAX 64   // K, N per group

__global__ __launch_bounds__(GD_NT) void gdense_fwd_kernel(const float *__restrict__ x, const float *__restrict__ w,
                                                           const float *__restrict__ bias, float *__restrict__ y, int64_t R, int G,
                                                           int K, int N, int act) {
    __shared__ float Ws[GD_MAX][GD_MAX + 1], Xs[GD_TR][GD_MAX + 1], Bs[GD_MAX];
    const int g = blockIdx.y;
    for (int id = threadIdx.x; id < K * N; id += GD_NT) Ws[id / N][id % N] = w[(int64_t)g * K * N + id];
    if (threadIdx.x < N) Bs[threadIdx.x] = bias ? bias[g * N + threadIdx.x] : 0.f;
    const int64_t n_tiles = (R + GD_TR - 1) / GD_TR;
    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const int64_t r0 = tile * GD_TR;
        const int rows = (int)(R - r0 < GD_TR ? R - r0 : GD_TR);
        __syncthreads();  // the previous tile's operands are no longer read (and the kernel matrix is in place)
        for (int id = threadIdx.x; id < rows * K; id += GD_NT) {
            const int r = id / K, k = id - r * K;
            Xs[r][k] = x[((r0 + r) * G + g) * K + k];
        }
        __syncthreads();
        for (int id = threadIdx.x; id < rows * N; id += GD_NT) {
            const int r = id / N, n = id - r * N;
            float acc = 0.f;
            for (int k = 0; k < K; ++k) acc = __fadd_rn(acc, __fmul_rn(Xs[r][k], Ws[k][n]));
            if (bias) acc = __fadd_rn(acc, Bs[n]);
            if (act == HGQ_ACT_RELU) acc = acc > 0.f ? acc : 0.f;
            y[((r0 + r) * G + g) * N + n] = acc;
        }
    }
}

// dx, and one slice [G][K * N + N] of kernel / bias gradient per workgroup column (blockIdx.x); a thread keeps the
// (k, n) entries id = threadIdx.x + j * GD_NT of its group in registers over all tiles of the workgroup.
__global__ __launch_bounds__(GD_NT) void gdense_bwd_kernel(const float *__restrict__ dy, const float *__restrict__ y,
                                                           const float *__restrict__ x, const float *__restrict__ w,
                                                           float *__restrict__ dx, float *__restrict__ part, int64_t R, int G, int K,
                                                           int N, int act, int has_bias) {
    __shared__ float Ws[GD_MAX][GD_MAX + 1], Xs[GD_TR][GD_MAX + 1], Zs[GD_TR][GD_MAX + 1];
    const int g = blockIdx.y;
    for (int id = threadIdx.x; id < K * N; id += GD_NT) Ws[id / N][id % N] = w[(int64_t)g * K * N + id];
    constexpr int PER = GD_MAX * GD_MAX / GD_NT;  // 16 kernel entries per thread at most
    float dw_acc[PER], db_acc = 0.f;
#pragma unroll
    for (int j = 0; j < PER; ++j) dw_acc[j] = 0.f;
    const int64_t n_tiles = (R + GD_TR - 1) / GD_TR;
    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const int64_t r0 = tile * GD_TR;
        const int rows = (int)(R - r0 < GD_TR ? R - r0 : GD_TR);
        __syncthreads();
        for (int id = threadIdx.x; id < rows * K; id += GD_NT) {
            const int r = id / K, k = id - r * K;
            Xs[r][k] = x[((r0 + r) * G + g) * K + k];
        }
        for (int id = threadIdx.x; id < rows * N; id += GD_NT) {
            const int r = id / N, n = id - r * N;
            const int64_t o = ((r0 + r) * G + g) * N + n;
            float z = dy[o];
            if (act == HGQ_ACT_RELU && !(y[o] > 0.f)) z = 0.f;
            Zs[r][n] = z;
        }
        __syncthreads();
        if (dx) {
            for (int id = threadIdx.x; id < rows * K; id += GD_NT) {
                const int r = id / K, k = id - r * K;
                float acc = 0.f;
                for (int n = 0; n < N; ++n) acc = __fadd_rn(acc, __fmul_rn(Zs[r][n], Ws[k][n]));
                dx[((r0 + r) * G + g) * K + k] = acc;
            }
        }
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            const int id = threadIdx.x + j * GD_NT;
            if (id < K * N) {
                const int k = id / N, n = id - k * N;
                float acc = dw_acc[j];
                for (int r = 0; r < rows; ++r) acc = __fadd_rn(acc, __fmul_rn(Xs[r][k], Zs[r][n]));
                dw_acc[j] = acc;
            }
        }
        if (has_bias && threadIdx.x < N) {
            for (int r = 0; r < rows; ++r) db_acc = __fadd_rn(db_acc, Zs[r][threadIdx.x]);
        }
    }
    // slice layout: [G * K * N kernel entries | G * N bias entries]
    float *mine = part + (int64_t)blockIdx.x * ((int64_t)G * K * N + (has_bias ? G * N : 0));
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int id = threadIdx.x + j * GD_NT;
        if (id < K * N) mine[(int64_t)g * K * N + id] = dw_acc[j];
    }
    if (has_bias && threadIdx.x < N) mine[(int64_t)G * K * N + g * N + threadIdx.x] = db_acc;
}

static int gdense_parts(int64_t R, int G) {
    const int64_t n_tiles = (R + GD_TR - 1) / GD_TR;
    int want = persistent_grid(1 << 30, 4) / (G > 0 ? G : 1);
    if (want < 1) want = 1;
    return (int)(n_tiles < want ? (n_tiles > 0 ? n_tiles : 1) : want);
}

// ---- per-channel affine map -----------------------------------------------------------------------------------------
// A thread owns four adjacent channels (one 128-bit access per row) and walks down its row group; C % 4 == 0.
#define AF_NT 256
__global__ __launch_bounds__(AF_NT) void affine_rows_fwd_kernel(const float *__restrict__ x, const float *__restrict__ sc,
                                                                const float *__restrict__ of, float *__restrict__ y, int64_t n4,
                                                                int C4) {
    for (int64_t v = (int64_t)blockIdx.x * AF_NT + threadIdx.x; v < n4; v += (int64_t)gridDim.x * AF_NT) {
        const int c4 = (int)(v % C4);
        const f32x4_t xv = ((const f32x4_t *)x)[v], sv = ((const f32x4_t *)sc)[c4], ov = ((const f32x4_t *)of)[c4];
        f32x4_t o;
#pragma unroll
        for (int c = 0; c < 4; ++c) o[c] = __fadd_rn(__fmul_rn(xv[c], sv[c]), ov[c]);
        ((f32x4_t *)y)[v] = o;
    }
}

// dx = g * s; slices [gridDim.y][2 * C]: per-channel sums of g * x, then of g, over the workgroup's rows.
// thread (tx, ty): tx walks the column groups of four, ty the rows; TX is a power of two <= 64.
__global__ __launch_bounds__(AF_NT) void affine_rows_bwd_kernel(const float *__restrict__ g, const float *__restrict__ x,
                                                                const float *__restrict__ sc, float *__restrict__ dx,
                                                                float *__restrict__ part, int64_t rows, int C, int TX,
                                                                int64_t rows_per_wg) {
    __shared__ float red[2][AF_NT][4];
    const int TY = AF_NT / TX, tx = threadIdx.x % TX, ty = threadIdx.x / TX;
    const int c0 = (blockIdx.x * TX + tx) * 4;
    const bool col_on = c0 < C;
    f32x4_t sv = {0.f, 0.f, 0.f, 0.f}, sgx = {0.f, 0.f, 0.f, 0.f}, sg = {0.f, 0.f, 0.f, 0.f};
    if (col_on) sv = *(const f32x4_t *)(sc + c0);
    const int64_t r_lo = (int64_t)blockIdx.y * rows_per_wg, r_hi = r_lo + rows_per_wg < rows ? r_lo + rows_per_wg : rows;
    if (col_on) {
        for (int64_t r = r_lo + ty; r < r_hi; r += TY) {
            const f32x4_t gv = *(const f32x4_t *)(g + r * C + c0), xv = *(const f32x4_t *)(x + r * C + c0);
            f32x4_t d;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                d[c] = __fmul_rn(gv[c], sv[c]);
                sgx[c] = __fadd_rn(sgx[c], __fmul_rn(gv[c], xv[c]));
                sg[c] = __fadd_rn(sg[c], gv[c]);
            }
            if (dx) *(f32x4_t *)(dx + r * C + c0) = d;
        }
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) red[0][threadIdx.x][c] = sgx[c], red[1][threadIdx.x][c] = sg[c];
    __syncthreads();
    if (ty == 0 && col_on) {
        float *mine = part + (int64_t)blockIdx.y * 2 * C;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            float a = 0.f, b = 0.f;
            for (int j = 0; j < TY; ++j) a = __fadd_rn(a, red[0][j * TX + tx][c]), b = __fadd_rn(b, red[1][j * TX + tx][c]);  // row groups in order
            mine[c0 + c] = a, mine[C + c0 + c] = b;
        }
    }
}

// ---- Quantizer wrapper: every step is one IEEE fp32 operation, in the order the reference's eager code takes them
struct WrapTail {
    float scaler, noise, a0, a1;
    int has_scaler, has_noise, has_affine;
};

__device__ __forceinline__ float wrap_tail_value(float q, float xs, const WrapTail &t) {
    float o = q;
    if (t.has_scaler) o = __fmul_rn(o, t.scaler);
    if (t.has_noise) o = __fadd_rn(xs, __fmul_rn(t.noise, __fsub_rn(o, xs)));
    if (t.has_affine) o = __fadd_rn(__fmul_rn(o, t.a0), t.a1);
    return o;
}

// gradients of the quantizer's output and of the scaled input (the blend reads it) for an upstream gradient g, as autograd
// forms them for the same chain of operations
__device__ __forceinline__ void wrap_tail_grad(float g, const WrapTail &t, float &dq, float &dxs) {
    if (t.has_affine) g = __fmul_rn(g, t.a0);
    dxs = 0.f;
    if (t.has_noise) {
        const float go = __fmul_rn(g, t.noise);
        dxs = __fsub_rn(g, go);
        g = go;
    }
    dq = t.has_scaler ? __fmul_rn(g, t.scaler) : g;
}

// mode 0: y = x / scaler; 1: y = tail(q = x, xs = x2); 2: (y, y2) = gradients of (q, xs) for the upstream gradient x.
// Four elements per thread where the arrays are 16-byte aligned (vec), one otherwise.
__global__ __launch_bounds__(256) void wrap_kernel(const float *__restrict__ x, const float *__restrict__ x2, float *__restrict__ y,
                                                   float *__restrict__ y2, int64_t n, WrapTail t, int mode, int vec) {
    const int64_t stride = (int64_t)gridDim.x * 256, first = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t n4 = vec ? n / 4 : 0;
    for (int64_t v = first; v < n4; v += stride) {
        const f32x4_t a = ((const f32x4_t *)x)[v];
        f32x4_t o, o2 = {0.f, 0.f, 0.f, 0.f};
        if (mode == 0) {
#pragma unroll
            for (int c = 0; c < 4; ++c) o[c] = __fdiv_rn(a[c], t.scaler);
        } else if (mode == 1) {
            const f32x4_t b = t.has_noise ? ((const f32x4_t *)x2)[v] : a;
#pragma unroll
            for (int c = 0; c < 4; ++c) o[c] = wrap_tail_value(a[c], b[c], t);
        } else {
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                float dq, dxs;
                wrap_tail_grad(a[c], t, dq, dxs);
                o[c] = dq, o2[c] = dxs;
            }
            if (y2) ((f32x4_t *)y2)[v] = o2;
        }
        ((f32x4_t *)y)[v] = o;
    }
    for (int64_t e = 4 * n4 + first; e < n; e += stride) {
        const float a = x[e];
        if (mode == 0) {
            y[e] = __fdiv_rn(a, t.scaler);
        } else if (mode == 1) {
            y[e] = wrap_tail_value(a, t.has_noise ? x2[e] : a, t);
        } else {
            float dq, dxs;
            wrap_tail_grad(a, t, dq, dxs);
            y[e] = dq;
            if (y2) y2[e] = dxs;
        }
    }
}

static int wrap_launch(const char *what, const float *x, const float *x2, float *y, float *y2, int64_t n, const WrapTail &t, int mode,
                       void *stream) {
    if (n < 0) return fail(HGQ_ERR_ARG, "%s: negative size", what);
    if (n == 0) return HGQ_OK;
    if (!x || !y) return fail(HGQ_ERR_ARG, "%s: null pointer", what);
    const bool vec = (((uintptr_t)x | (uintptr_t)y | (uintptr_t)(x2 ? x2 : x) | (uintptr_t)(y2 ? y2 : y)) & 15u) == 0;
    const int64_t items = vec ? (n + 3) / 4 : n;
    hipLaunchKernelGGL(wrap_kernel, dim3((unsigned)persistent_grid((items + 255) / 256, 8)), dim3(256), 0, (hipStream_t)stream, x, x2, y, y2, n, t,
                       mode, vec ? 1 : 0);
    return check_launch(what);
}

static void affine_geometry(int64_t rows, int C, int &TX, int &gx, int64_t &gy, int64_t &rows_per_wg) {
    const int cg = C / 4;
    TX = 1;
    while (TX * 2 <= cg && TX < 64) TX *= 2;
    gx = (cg + TX - 1) / TX;
    const int TY = AF_NT / TX;
    int64_t want = (int64_t)persistent_grid(1 << 30, 4) / gx;
    if (want < 1) want = 1;
    const int64_t batches = (rows + TY - 1) / TY;
    gy = batches < want ? (batches > 0 ? batches : 1) : want;
    rows_per_wg = ((batches + gy - 1) / gy) * TY;
    gy = (rows + rows_per_wg - 1) / rows_per_wg;
    if (gy < 1) gy = 1;
}

static inline bool aligned16(const void *p) { return ((uintptr_t)p & 15u) == 0; }

}  // namespace hgq

using namespace hgq;

extern "C" int hgq_gdense_supported(int64_t R, int G, int K, int N) {
    return R >= 0 && G >= 1 && K >= 1 && N >= 1 && K <= GD_MAX && N <= GD_MAX && G <= 65535 && (int64_t)R * G * (K > N ? K : N) < (1ll << 40);
}

extern "C" int hgq_gdense_fwd(const float *x, const float *w, const float *bias, float *y, int64_t R, int G, int K, int N, int act,
                              void *stream) {
    if (!hgq_gdense_supported(R, G, K, N)) return fail(HGQ_ERR_UNSUPPORTED, "hgq_gdense_fwd: R=%lld G=%d K=%d N=%d (K, N <= %d)", (long long)R, G, K, N, GD_MAX);
    if (act != HGQ_ACT_NONE && act != HGQ_ACT_RELU) return fail(HGQ_ERR_ARG, "hgq_gdense_fwd: unknown activation");
    if (R == 0) return HGQ_OK;
    if (!x || !w || !y) return fail(HGQ_ERR_ARG, "hgq_gdense_fwd: null pointer");
    hipLaunchKernelGGL(gdense_fwd_kernel, dim3((unsigned)gdense_parts(R, G), (unsigned)G), dim3(GD_NT), 0, (hipStream_t)stream, x, w, bias, y, R,
                       G, K, N, act);
    return check_launch("hgq_gdense_fwd");
}

extern "C" int64_t hgq_gdense_bwd_workspace(int64_t R, int G, int K, int N, int has_bias) {
    if (!hgq_gdense_supported(R, G, K, N)) return -1;
    return (int64_t)gdense_parts(R, G) * ((int64_t)G * K * N + (has_bias ? G * N : 0));
}

extern "C" int hgq_gdense_bwd(const float *dy, const float *y, const float *x, const float *w, float *dx, float *dw, float *dbias,
                              float *workspace, int64_t R, int G, int K, int N, int act, void *stream) {
    hipStream_t s = (hipStream_t)stream;
    if (!hgq_gdense_supported(R, G, K, N)) return fail(HGQ_ERR_UNSUPPORTED, "hgq_gdense_bwd: R=%lld G=%d K=%d N=%d (K, N <= %d)", (long long)R, G, K, N, GD_MAX);
    if (act != HGQ_ACT_NONE && act != HGQ_ACT_RELU) return fail(HGQ_ERR_ARG, "hgq_gdense_bwd: unknown activation");
    if (!dw) return fail(HGQ_ERR_ARG, "hgq_gdense_bwd: dw is required");
    const int64_t KN = (int64_t)G * K * N, BN = dbias ? (int64_t)G * N : 0;
    if (R == 0) {
        int rc = fill_f32(dw, 0.f, KN, s);
        if (!rc && dbias) rc = fill_f32(dbias, 0.f, BN, s);
        return rc;
    }
    if (!dy || !x || !w || !workspace || (act == HGQ_ACT_RELU && !y)) return fail(HGQ_ERR_ARG, "hgq_gdense_bwd: null pointer");
    const int parts = gdense_parts(R, G);
    hipLaunchKernelGGL(gdense_bwd_kernel, dim3((unsigned)parts, (unsigned)G), dim3(GD_NT), 0, s, dy, y, x, w, dx, workspace, R, G, K, N, act,
                       dbias ? 1 : 0);
    int rc = check_launch("hgq_gdense_bwd");
    if (rc) return rc;
    return reduce_parts(workspace, parts, KN + BN, dw, KN, dbias, BN, nullptr, 0, s);
}

extern "C" int hgq_affine_rows_fwd(const float *x, const float *scale, const float *offset, float *y, int64_t rows, int C, void *stream) {
    if (rows < 0 || C < 4 || C % 4) return fail(HGQ_ERR_UNSUPPORTED, "hgq_affine_rows_fwd: the channel count must be a positive multiple of 4, got %d", C);
    if (rows == 0) return HGQ_OK;
    if (!x || !scale || !offset || !y) return fail(HGQ_ERR_ARG, "hgq_affine_rows_fwd: null pointer");
    if (!(aligned16(x) && aligned16(scale) && aligned16(offset) && aligned16(y))) return fail(HGQ_ERR_ARG, "hgq_affine_rows_fwd: operands must be 16-byte aligned");
    const int64_t n4 = rows * (C / 4);
    hipLaunchKernelGGL(affine_rows_fwd_kernel, dim3((unsigned)persistent_grid((n4 + AF_NT - 1) / AF_NT, 8)), dim3(AF_NT), 0, (hipStream_t)stream, x,
                       scale, offset, y, n4, C / 4);
    return check_launch("hgq_affine_rows_fwd");
}

extern "C" int64_t hgq_affine_rows_bwd_workspace(int64_t rows, int C) {
    if (rows < 0 || C < 4 || C % 4) return -1;
    int TX, gx;
    int64_t gy, rpw;
    affine_geometry(rows > 0 ? rows : 1, C, TX, gx, gy, rpw);
    return gy * 2 * (int64_t)C;
}

extern "C" int hgq_affine_rows_bwd(const float *g, const float *x, const float *scale, float *dx, float *dscale, float *doffset,
                                   float *workspace, int64_t rows, int C, void *stream) {
    hipStream_t s = (hipStream_t)stream;
    if (rows < 0 || C < 4 || C % 4) return fail(HGQ_ERR_UNSUPPORTED, "hgq_affine_rows_bwd: the channel count must be a positive multiple of 4, got %d", C);
    if (rows == 0) {
        int rc = dscale ? fill_f32(dscale, 0.f, C, s) : HGQ_OK;
        if (!rc && doffset) rc = fill_f32(doffset, 0.f, C, s);
        return rc;
    }
    if (!g || !x || !scale || !workspace) return fail(HGQ_ERR_ARG, "hgq_affine_rows_bwd: null pointer");
    if (!(aligned16(g) && aligned16(x) && aligned16(scale) && (!dx || aligned16(dx)))) return fail(HGQ_ERR_ARG, "hgq_affine_rows_bwd: operands must be 16-byte aligned");
    int TX, gx;
    int64_t gy, rpw;
    affine_geometry(rows, C, TX, gx, gy, rpw);
    hipLaunchKernelGGL(affine_rows_bwd_kernel, dim3((unsigned)gx, (unsigned)gy), dim3(AF_NT), 0, s, g, x, scale, dx, workspace, rows, C, TX, rpw);
    int rc = check_launch("hgq_affine_rows_bwd");
    if (rc) return rc;
    return reduce_parts(workspace, (int)gy, 2 * (int64_t)C, dscale, C, doffset, C, nullptr, 0, s);
}

extern "C" int hgq_quantizer_scale_div(const float *x, float *y, int64_t n, float scaler, void *stream) {
    WrapTail t = {scaler, 0.f, 1.f, 0.f, 1, 0, 0};
    return wrap_launch("hgq_quantizer_scale_div", x, nullptr, y, nullptr, n, t, 0, stream);
}

extern "C" int hgq_quantizer_tail_fwd(const float *q, const float *xs, float *out, int64_t n, int has_scaler, float scaler, int has_noise,
                                      float noise, int has_affine, float a0, float a1, void *stream) {
    if (has_noise && !xs) return fail(HGQ_ERR_ARG, "hgq_quantizer_tail_fwd: the noise blend needs the quantizer's input");
    WrapTail t = {scaler, noise, a0, a1, has_scaler ? 1 : 0, has_noise ? 1 : 0, has_affine ? 1 : 0};
    return wrap_launch("hgq_quantizer_tail_fwd", q, xs, out, nullptr, n, t, 1, stream);
}

extern "C" int hgq_quantizer_tail_bwd(const float *g, float *dq, float *dxs, int64_t n, int has_scaler, float scaler, int has_noise,
                                      float noise, int has_affine, float a0, void *stream) {
    if (has_noise && !dxs) return fail(HGQ_ERR_ARG, "hgq_quantizer_tail_bwd: the noise blend sends a gradient to the quantizer's input");
    WrapTail t = {scaler, noise, a0, 0.f, has_scaler ? 1 : 0, has_noise ? 1 : 0, has_affine ? 1 : 0};
    return wrap_launch("hgq_quantizer_tail_bwd", g, nullptr, dq, has_noise ? dxs : nullptr, n, t, 2, stream);
}
