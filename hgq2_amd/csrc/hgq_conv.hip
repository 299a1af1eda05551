// QConv2D contraction (channels-last input, HWIO kernel) as implicit GEMM on fp32 MFMA, and the
// dense contraction of any width as its 1 x 1 special case.
//
//   forward        y[m, f]  = act(sum_k A(m, k) * W[k, f] + b[f])      m = (b, oy, ox), k = (ky, kx, c)
//   data gradient  dx[m', c] = sum_k' Z(m', k') * W[ky, kx, c, f]       m' = (b, iy, ix), k' = (ky, kx, f)
//   weight grad.   dW[k, f] = sum_m A(m, k) * dz[m, f],  db[f] = sum_m dz[m, f]
//
// with dz = dy masked by the activation (y > 0 for ReLU).  A(m, k) is the im2col matrix, never
// materialised: a tile of it is gathered straight into LDS (rows decoded once per tile, the
// column of a thread once per k step), next to the matching tile of the second operand, and
// v_mfma_f32_32x32x2f32 contracts them.  The weight gradient is split along m across
// workgroups; the per-workgroup partial sums go to workspace slices which a second kernel adds
// up in a fixed order (deterministic, no floating-point atomics).
//
// MFMA 32x32x2 fp32 operand layout (64 lanes): A[i][k]: i = lane % 32, k = lane / 32;
// B[k][j]: k = lane / 32, j = lane % 32; D[i][j] in 16 registers: j = lane % 32,
// i = (r / 4) * 8 + (lane / 32) * 4 + (r % 4).
#include "hgq_device.h"
#include "hgq_host.h"

namespace hgq {

typedef float floatx16 __attribute__((ext_vector_type(16)));

#define CV_BK 32

__device__ __forceinline__ int cv_acc_row(int r, int lane) { return (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3); }

struct RowInfo {
    int base;  // pixel index of (b, 0, 0) in the gathered tensor, -1 for rows past the end
    int y0, x0;
};

// Gather descriptor of one k column.
struct ColInfo {
    int ky, kx, ch;
    bool on;
};

// MODE 0: forward im2col gather from the input [B, H, W, C] for output pixels (b, oy, ox).
// MODE 1: transposed gather from dz [B, OH, OW, F] for input pixels (b, iy, ix).
template <int MODE>
__device__ __forceinline__ RowInfo decode_row(int64_t m, int64_t rows, const hgq_conv_geom &g) {
    RowInfo r;
    r.base = -1, r.y0 = 0, r.x0 = 0;
    if (m >= rows) return r;
    if (MODE == 0) {
        const int per = g.OH * g.OW;
        const int b = (int)(m / per), rem = (int)(m - (int64_t)b * per);
        const int oy = rem / g.OW, ox = rem - oy * g.OW;
        r.base = b * g.H * g.W, r.y0 = oy * g.sy - g.py, r.x0 = ox * g.sx - g.px;
    } else {
        const int per = g.H * g.W;
        const int b = (int)(m / per), rem = (int)(m - (int64_t)b * per);
        const int iy = rem / g.W, ix = rem - iy * g.W;
        r.base = b * g.OH * g.OW, r.y0 = iy + g.py, r.x0 = ix + g.px;
    }
    return r;
}

template <int MODE>
__device__ __forceinline__ ColInfo decode_col(int k, int K, const hgq_conv_geom &g, int F) {
    ColInfo c;
    const int depth = MODE == 0 ? g.C : F;
    c.on = k < K;
    const int kk = c.on ? k : 0;
    const int tap = kk / depth;
    c.ch = kk - tap * depth;
    c.ky = tap / g.kw, c.kx = tap - c.ky * g.kw;
    return c;
}

// Element (row, column) of the gathered operand; `mask` (the forward output) applies the ReLU
// derivative in MODE 1.
template <int MODE>
__device__ __forceinline__ float gather(const float *__restrict__ src, const float *__restrict__ mask, const RowInfo &r,
                                        const ColInfo &c, const hgq_conv_geom &g, int F) {
    if (r.base < 0 || !c.on) return 0.f;
    if (MODE == 0) {
        const int iy = r.y0 + c.ky * g.dly, ix = r.x0 + c.kx * g.dlx;
        if ((unsigned)iy >= (unsigned)g.H || (unsigned)ix >= (unsigned)g.W) return 0.f;
        return src[((int64_t)r.base + iy * g.W + ix) * g.C + c.ch];
    } else {
        const int ty = r.y0 - c.ky * g.dly, tx = r.x0 - c.kx * g.dlx;
        if (ty < 0 || tx < 0) return 0.f;
        const int oy = ty / g.sy, ox = tx / g.sx;
        if (oy * g.sy != ty || ox * g.sx != tx || oy >= g.OH || ox >= g.OW) return 0.f;
        const int64_t a = ((int64_t)r.base + oy * g.OW + ox) * F + c.ch;
        const float v = src[a];
        return (mask && !(mask[a] > 0.f)) ? 0.f : v;
    }
}

// Forward (MODE 0, N = F) and data gradient (MODE 1, N = C).  WN = wavefronts along n (1 or 2):
// the workgroup's tile is (128 / WN) x (32 * WN).
template <int MODE, int WN>
__global__ __launch_bounds__(256) void igemm_kernel(const float *__restrict__ src, const float *__restrict__ mask,
                                                    const float *__restrict__ w, const float *__restrict__ bias,
                                                    float *__restrict__ out, hgq_conv_geom g, int F, int64_t rows, int K,
                                                    int N, int act) {
    constexpr int WM = 4 / WN, BM = 32 * WM, BN = 32 * WN;
    __shared__ float as[BM][CV_BK + 1];
    __shared__ float bs[CV_BK][BN + 1];
    __shared__ RowInfo rinfo[BM];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int n0 = blockIdx.y * BN;
    const int64_t n_tiles = (rows + BM - 1) / BM;
    const int acol = tid & 31, arow0 = tid >> 5;  // A staging: fixed column, rows arow0 + 8 j
    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const int64_t r0 = tile * BM;
        __syncthreads();
        if (tid < BM) rinfo[tid] = decode_row<MODE>(r0 + tid, rows, g);
        __syncthreads();
        floatx16 acc = {0};
        for (int k0 = 0; k0 < K; k0 += CV_BK) {
            const ColInfo ci = decode_col<MODE>(k0 + acol, K, g, F);
#pragma unroll 4
            for (int j = 0; j < BM / 8; ++j) {
                const int row = arow0 + 8 * j;
                as[row][acol] = gather<MODE>(src, mask, rinfo[row], ci, g, F);
            }
            // second operand tile [BK, BN]:  MODE 0: W[k, n];  MODE 1: W[tap, n (= c), f] with k = (tap, f)
            for (int id = tid; id < CV_BK * BN; id += 256) {
                int kk, nn;
                if (MODE == 0) kk = id / BN, nn = id - kk * BN;
                else nn = id / CV_BK, kk = id - nn * CV_BK;
                const int k = k0 + kk, n = n0 + nn;
                float v = 0.f;
                if (k < K && n < N) {
                    if (MODE == 0) {
                        v = w[(int64_t)k * N + n];
                    } else {
                        const int tap = k / F, f = k - tap * F;
                        v = w[((int64_t)tap * N + n) * F + f];
                    }
                }
                bs[kk][nn] = v;
            }
            __syncthreads();
            {
                const int arow = wm * 32 + (lane & 31), kq = lane >> 5, bcol = wn * 32 + (lane & 31);
#pragma unroll
                for (int kk = 0; kk < CV_BK; kk += 2)
                    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(as[arow][kk + kq], bs[kk + kq][bcol], acc, 0, 0, 0);
            }
            __syncthreads();
        }
        const int n = n0 + wn * 32 + (lane & 31);
        if (n < N) {
            const float bv = (MODE == 0 && bias) ? bias[n] : 0.f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int64_t m = r0 + wm * 32 + cv_acc_row(r, lane);
                if (m < rows) {
                    float v = acc[r] + bv;
                    if (MODE == 0 && act == HGQ_ACT_RELU) v = v > 0.f ? v : 0.f;
                    out[m * N + n] = v;
                }
            }
        }
    }
}

// Weight / bias gradient.  Workgroup (kt, nt, split): k tile of 32 * WK columns of the im2col
// matrix, n tile of 32 * (4 / WK) filters, rows [split * chunk, (split + 1) * chunk).
// Slice `split` of `part` is [K * F | F].
template <int WK>
__global__ __launch_bounds__(256) void wgrad_kernel(const float *__restrict__ src, const float *__restrict__ dy,
                                                    const float *__restrict__ y, float *__restrict__ part, hgq_conv_geom g,
                                                    int F, int64_t rows, int K, int64_t chunk, int act, int n_ktiles) {
    constexpr int WN = 4 / WK, BKT = 32 * WK, BN = 32 * WN, BMS = 32;
    __shared__ float as[BMS][BKT + 1];
    __shared__ float zs[BMS][BN + 1];
    __shared__ RowInfo rinfo[BMS];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wk = wave / WN, wn = wave % WN;
    const int kt = blockIdx.x % n_ktiles, nt = blockIdx.x / n_ktiles;
    const int k0 = kt * BKT, n0 = nt * BN;
    const int64_t m_begin = (int64_t)blockIdx.y * chunk, m_end = min(rows, m_begin + chunk);
    const int64_t KF = (int64_t)K * F;
    float *my = part + (int64_t)blockIdx.y * (KF + F);
    // A staging: thread owns column tid % BKT, rows tid / BKT + (256 / BKT) j
    const int acol = tid % BKT, arow0 = tid / BKT;
    const ColInfo ci = decode_col<0>(k0 + acol, K, g, F);
    floatx16 acc = {0};
    float bsum = 0.f;
    const int zc = tid % BN, zr0 = tid / BN;  // dz staging: column, first row
    for (int64_t m0 = m_begin; m0 < m_end; m0 += BMS) {
        __syncthreads();
        if (tid < BMS) rinfo[tid] = decode_row<0>(m0 + tid < m_end ? m0 + tid : rows, rows, g);
        __syncthreads();
#pragma unroll 4
        for (int row = arow0; row < BMS; row += 256 / BKT) as[row][acol] = gather<0>(src, nullptr, rinfo[row], ci, g, F);
        for (int row = zr0; row < BMS; row += 256 / BN) {
            const int64_t m = m0 + row;
            const int n = n0 + zc;
            float v = 0.f;
            if (m < m_end && n < F) {
                v = dy[m * F + n];
                if (act == HGQ_ACT_RELU && !(y[m * F + n] > 0.f)) v = 0.f;
            }
            zs[row][zc] = v;
            bsum += v;
        }
        __syncthreads();
        const int kq = lane >> 5, c32 = lane & 31;
#pragma unroll
        for (int mm = 0; mm < BMS; mm += 2)
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(as[mm + kq][wk * 32 + c32], zs[mm + kq][wn * 32 + c32], acc, 0, 0, 0);
    }
    const int n = n0 + wn * 32 + (lane & 31);
    if (n < F) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int k = k0 + wk * 32 + cv_acc_row(r, lane);
            if (k < K) my[(int64_t)k * F + n] = acc[r];
        }
    }
    if (kt == 0) {
        // bias gradient: threads with the same dz column add up in a fixed order
        __syncthreads();
        float *red = &as[0][0];
        red[tid] = bsum;
        __syncthreads();
        if (tid < BN && n0 + tid < F) {
            float s = 0.f;
            for (int j = 0; j < 256 / BN; ++j) s += red[tid + j * BN];
            my[KF + n0 + tid] = s;
        }
    }
}

static int check_geom(const hgq_conv_geom *g, int F, const char *who) {
    if (!g) return fail(HGQ_ERR_ARG, "%s: null geometry", who);
    if (g->B < 0 || g->H < 1 || g->W < 1 || g->C < 1 || g->kh < 1 || g->kw < 1 || g->sy < 1 || g->sx < 1 || g->dly < 1 ||
        g->dlx < 1 || g->OH < 1 || g->OW < 1 || g->py < 0 || g->px < 0 || F < 1)
        return fail(HGQ_ERR_ARG, "%s: bad geometry", who);
    // every source pixel index must fit 31 bits (the kernels decode rows with 32-bit arithmetic)
    if ((int64_t)g->B * g->H * g->W >= (1ll << 31) || (int64_t)g->B * g->OH * g->OW >= (1ll << 31) ||
        (int64_t)g->kh * g->kw * g->C >= (1ll << 30) || (int64_t)g->kh * g->kw * F >= (1ll << 30))
        return fail(HGQ_ERR_UNSUPPORTED, "%s: tensor too large for 32-bit pixel indices", who);
    return HGQ_OK;
}

static int64_t wgrad_splits(int64_t rows, int n_tiles_kn) {
    // enough workgroups to fill the device, at least 128 rows each
    int64_t s = (1024 + n_tiles_kn - 1) / n_tiles_kn;
    const int64_t cap = (rows + 127) / 128;
    if (s > cap) s = cap;
    if (s > 512) s = 512;
    return s < 1 ? 1 : s;
}

}  // namespace hgq

using namespace hgq;

extern "C" int hgq_conv2d_fwd(const float *xq, const float *qw, const float *qb, float *y, const hgq_conv_geom *g, int F,
                              int act, void *stream) {
    int rc = check_geom(g, F, "hgq_conv2d_fwd");
    if (rc) return rc;
    if (act != HGQ_ACT_NONE && act != HGQ_ACT_RELU) return fail(HGQ_ERR_ARG, "hgq_conv2d_fwd: unknown activation %d", act);
    const int64_t rows = (int64_t)g->B * g->OH * g->OW;
    if (rows == 0) return HGQ_OK;
    if (!xq || !qw || !y) return fail(HGQ_ERR_ARG, "hgq_conv2d_fwd: null pointer");
    const int K = g->kh * g->kw * g->C;
    hipStream_t s = (hipStream_t)stream;
    if (F <= 32) {
        const dim3 grid((unsigned)persistent_grid((rows + 127) / 128, 8), 1);
        hipLaunchKernelGGL((igemm_kernel<0, 1>), grid, dim3(256), 0, s, xq, (const float *)nullptr, qw, qb, y, *g, F, rows, K, F, act);
    } else {
        const dim3 grid((unsigned)persistent_grid((rows + 63) / 64, 8), (unsigned)((F + 63) / 64));
        hipLaunchKernelGGL((igemm_kernel<0, 2>), grid, dim3(256), 0, s, xq, (const float *)nullptr, qw, qb, y, *g, F, rows, K, F, act);
    }
    return check_launch("hgq_conv2d_fwd");
}

extern "C" int64_t hgq_conv2d_bwd_workspace(const hgq_conv_geom *g, int F) {
    if (check_geom(g, F, "hgq_conv2d_bwd_workspace")) return -1;
    const int64_t rows = (int64_t)g->B * g->OH * g->OW;
    const int K = g->kh * g->kw * g->C;
    const int wk = F <= 32 ? 4 : 2;
    const int n_kn = ((K + 32 * wk - 1) / (32 * wk)) * ((F + 32 * (4 / wk) - 1) / (32 * (4 / wk)));
    return wgrad_splits(rows, n_kn) * ((int64_t)K * F + F);
}

extern "C" int hgq_conv2d_bwd(const float *dy, const float *y, const float *xq, const float *qw, float *dxq, float *dqw,
                              float *dqb, float *workspace, const hgq_conv_geom *g, int F, int act, void *stream) {
    int rc = check_geom(g, F, "hgq_conv2d_bwd");
    if (rc) return rc;
    if (act != HGQ_ACT_NONE && act != HGQ_ACT_RELU) return fail(HGQ_ERR_ARG, "hgq_conv2d_bwd: unknown activation %d", act);
    hipStream_t s = (hipStream_t)stream;
    const int64_t rows = (int64_t)g->B * g->OH * g->OW, in_rows = (int64_t)g->B * g->H * g->W;
    const int K = g->kh * g->kw * g->C;
    const int64_t KF = (int64_t)K * F;
    if (rows == 0) {
        if (dqw && (rc = fill_f32(dqw, 0.f, KF, s))) return rc;
        if (dqb && (rc = fill_f32(dqb, 0.f, F, s))) return rc;
        if (dxq && (rc = fill_f32(dxq, 0.f, in_rows * g->C, s))) return rc;
        return HGQ_OK;
    }
    if (!dy || !qw || !xq) return fail(HGQ_ERR_ARG, "hgq_conv2d_bwd: null pointer");
    if (act == HGQ_ACT_RELU && !y) return fail(HGQ_ERR_ARG, "hgq_conv2d_bwd: relu needs the forward output");
    const float *mask = act == HGQ_ACT_RELU ? y : nullptr;
    if (dxq) {
        const int Kt = g->kh * g->kw * F;  // contraction length of the data gradient
        if (g->C <= 32) {
            const dim3 grid((unsigned)persistent_grid((in_rows + 127) / 128, 8), 1);
            hipLaunchKernelGGL((igemm_kernel<1, 1>), grid, dim3(256), 0, s, dy, mask, qw, (const float *)nullptr, dxq, *g, F, in_rows, Kt, g->C, act);
        } else {
            const dim3 grid((unsigned)persistent_grid((in_rows + 63) / 64, 8), (unsigned)((g->C + 63) / 64));
            hipLaunchKernelGGL((igemm_kernel<1, 2>), grid, dim3(256), 0, s, dy, mask, qw, (const float *)nullptr, dxq, *g, F, in_rows, Kt, g->C, act);
        }
        if ((rc = check_launch("hgq_conv2d_bwd(data)"))) return rc;
    }
    if (dqw || dqb) {
        if (!workspace) return fail(HGQ_ERR_ARG, "hgq_conv2d_bwd: null workspace");
        const int wk = F <= 32 ? 4 : 2;
        const int n_kt = (K + 32 * wk - 1) / (32 * wk), n_nt = (F + 32 * (4 / wk) - 1) / (32 * (4 / wk));
        const int64_t splits = wgrad_splits(rows, n_kt * n_nt);
        int64_t chunk = (rows + splits - 1) / splits;
        chunk = (chunk + 31) / 32 * 32;
        const dim3 grid((unsigned)(n_kt * n_nt), (unsigned)splits);
        if (wk == 4)
            hipLaunchKernelGGL((wgrad_kernel<4>), grid, dim3(256), 0, s, xq, dy, mask, workspace, *g, F, rows, K, chunk, act, n_kt);
        else
            hipLaunchKernelGGL((wgrad_kernel<2>), grid, dim3(256), 0, s, xq, dy, mask, workspace, *g, F, rows, K, chunk, act, n_kt);
        if ((rc = check_launch("hgq_conv2d_bwd(weights)"))) return rc;
        const int64_t M = KF + F;
        if ((rc = reduce_parts(workspace, (int)splits, M, dqw, KF, dqb, (int64_t)F, nullptr, 0, s))) return rc;
    }
    return HGQ_OK;
}
