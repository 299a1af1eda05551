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
template <int MODE, int WN, bool BF = false>
__global__ __launch_bounds__(256) void igemm_kernel(const float *__restrict__ src, const float *__restrict__ mask,
                                                    const float *__restrict__ w, const float *__restrict__ bias,
                                                    float *__restrict__ out, hgq_conv_geom g, int F, int64_t rows, int K,
                                                    int N, int act, int kchunk) {
    // gridDim.z > 1: split along k; slice z of `out` ([gridDim.z, rows * N]) receives the raw partial sums
    constexpr int WM = 4 / WN, BM = 32 * WM, BN = 32 * WN;
    const bool split = gridDim.z > 1;
    const int k_begin = blockIdx.z * kchunk, k_end = min(K, k_begin + kchunk);
    if (split) out += (int64_t)blockIdx.z * rows * N;
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
        for (int k0 = k_begin; k0 < k_end; k0 += CV_BK) {
            const ColInfo ci = decode_col<MODE>(k0 + acol, k_end, g, F);
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
                if (k < k_end && n < N) {
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
                if (BF) {
                    acc = mfma_chain_bf16<MODE == 1, false>(acc, &as[arow][kq], 1, &bs[kq][bcol], BN + 1, CV_BK / 16);
                } else {
#pragma unroll
                    for (int kk = 0; kk < CV_BK; kk += 2)
                        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(as[arow][kk + kq], bs[kk + kq][bcol], acc, 0, 0, 0);
                }
            }
            __syncthreads();
        }
        const int n = n0 + wn * 32 + (lane & 31);
        if (n < N) {
            const float bv = (MODE == 0 && bias && !split) ? bias[n] : 0.f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int64_t m = r0 + wm * 32 + cv_acc_row(r, lane);
                if (m < rows) {
                    float v = acc[r] + bv;
                    if (MODE == 0 && act == HGQ_ACT_RELU && !split) v = v > 0.f ? v : 0.f;
                    out[m * N + n] = v;
                }
            }
        }
    }
}


// Byte offset of four consecutive k columns (same tap, channels ch .. ch + 3; the depth is a
// multiple of 4) of one row in the gathered tensor, or BUF_OOB where the tap falls outside it:
// the buffer load then returns zeros and no branch surrounds the load.
template <int MODE>
__device__ __forceinline__ uint32_t gather4_offset(const RowInfo &r, const ColInfo &c, const hgq_conv_geom &g, int F) {
    if (r.base < 0 || !c.on) return BUF_OOB;
    if (MODE == 0) {
        const int iy = r.y0 + c.ky * g.dly, ix = r.x0 + c.kx * g.dlx;
        if ((unsigned)iy >= (unsigned)g.H || (unsigned)ix >= (unsigned)g.W) return BUF_OOB;
        return (uint32_t)((r.base + iy * g.W + ix) * g.C + c.ch) * 4u;
    } else {
        const int ty = r.y0 - c.ky * g.dly, tx = r.x0 - c.kx * g.dlx;
        if (ty < 0 || tx < 0) return BUF_OOB;
        const int oy = ty / g.sy, ox = tx / g.sx;
        if (oy * g.sy != ty || ox * g.sx != tx || oy >= g.OH || ox >= g.OW) return BUF_OOB;
        return (uint32_t)((r.base + oy * g.OW + ox) * F + c.ch) * 4u;
    }
}

// The same contraction for a gathered depth (C forward, F data gradient) that is a multiple of 4
// and 16-byte aligned operands.  A row's 32 k columns of a step are read as eight 128-bit loads
// by eight adjacent lanes, the loads of step s + 1 are in flight while the matrix cores work on
// step s (two LDS buffers, one barrier per step), and the A tile sits k-major in LDS with a row
// stride of BM + 2 words: the transposing writes and the operand reads both spread evenly over
// the banks.
template <int MODE, int WN, bool BF = false>
__global__ __launch_bounds__(256) void igemm_vec_kernel(const float *__restrict__ src, const float *__restrict__ mask,
                                                        const float *__restrict__ w, const float *__restrict__ bias,
                                                        float *__restrict__ out, hgq_conv_geom g, int F, int64_t rows, int K,
                                                        int N, int act, int kchunk) {
    constexpr int WM = 4 / WN, BM = 32 * WM, BN = 32 * WN, AS = BM + 2, NP = BM / 32, NB = CV_BK * BN / 256;
    const bool split = gridDim.z > 1;
    const int k_begin = blockIdx.z * kchunk, k_end = min(K, k_begin + kchunk);
    if (split) out += (int64_t)blockIdx.z * rows * N;
    __shared__ float as[2][CV_BK][AS];
    __shared__ float bs[2][CV_BK][BN + 1];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int n0 = blockIdx.y * BN;
    const int64_t n_tiles = (rows + BM - 1) / BM;
    const int q = tid & 7, rbase = tid >> 3;
    const int n_steps = (k_end - k_begin + CV_BK - 1) / CV_BK;
    // the gathered tensor (and the ReLU mask, same shape) as buffer descriptors: the launcher
    // guarantees they are smaller than 2 GiB
    const int64_t src_bytes = (MODE == 0 ? (int64_t)g.B * g.H * g.W * g.C : (int64_t)g.B * g.OH * g.OW * F) * 4;
    const __amdgpu_buffer_rsrc_t rs_src = buf_rsrc(src, src_bytes), rs_mask = buf_rsrc(mask ? mask : src, mask ? src_bytes : 0);
    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const int64_t r0 = tile * BM;
        RowInfo ri[NP];
#pragma unroll
        for (int p = 0; p < NP; ++p) ri[p] = decode_row<MODE>(r0 + rbase + 32 * p, rows, g);
        f32x4_t av[NP], am[NP];
        float bv[NB];
        auto fetch = [&](int k0) {
            const ColInfo ci = decode_col<MODE>(k0 + 4 * q, k_end, g, F);
#pragma unroll
            for (int p = 0; p < NP; ++p) {
                const uint32_t off = gather4_offset<MODE>(ri[p], ci, g, F);
                av[p] = buf_ld4(rs_src, off);
                if (MODE == 1) am[p] = buf_ld4(rs_mask, off);
            }
#pragma unroll
            for (int j = 0; j < NB; ++j) {
                const int id = tid + 256 * j;
                int kk, nn;
                if (MODE == 0) kk = id / BN, nn = id % BN;
                else nn = id / CV_BK, kk = id % CV_BK;
                const int k = k0 + kk, n = n0 + nn;
                float v = 0.f;
                if (k < k_end && n < N) {
                    if (MODE == 0) {
                        v = w[(int64_t)k * N + n];
                    } else {
                        const int tap = k / F, f = k - tap * F;
                        v = w[((int64_t)tap * N + n) * F + f];
                    }
                }
                bv[j] = v;
            }
        };
        auto stash = [&](int buf) {
#pragma unroll
            for (int p = 0; p < NP; ++p) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    float v = av[p][j];
                    if (MODE == 1 && mask && !(am[p][j] > 0.f)) v = 0.f;
                    as[buf][4 * q + j][rbase + 32 * p] = v;
                }
            }
#pragma unroll
            for (int j = 0; j < NB; ++j) {
                const int id = tid + 256 * j;
                if (MODE == 0) bs[buf][id / BN][id % BN] = bv[j];
                else bs[buf][id % CV_BK][id / CV_BK] = bv[j];
            }
        };
        __syncthreads();  // the previous tile's last step may still be reading buffer (n_steps - 1) & 1
        fetch(k_begin);
        stash(0);
        __syncthreads();
        floatx16 acc = {0};
        for (int st = 0; st < n_steps; ++st) {
            const int buf = st & 1;
            const bool more = st + 1 < n_steps;
            if (more) fetch(k_begin + (st + 1) * CV_BK);
            {
                const int arow = wm * 32 + (lane & 31), kq = lane >> 5, bcol = wn * 32 + (lane & 31);
                if (BF) {
                    acc = mfma_chain_bf16<MODE == 1, false>(acc, &as[buf][kq][arow], AS, &bs[buf][kq][bcol], BN + 1, CV_BK / 16);
                } else {
#pragma unroll
                    for (int kk = 0; kk < CV_BK; kk += 2)
                        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(as[buf][kk + kq][arow], bs[buf][kk + kq][bcol], acc, 0, 0, 0);
                }
            }
            if (more) stash(buf ^ 1);
            __syncthreads();
        }
        const int n = n0 + wn * 32 + (lane & 31);
        if (n < N) {
            const float bb = (MODE == 0 && bias && !split) ? bias[n] : 0.f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int64_t m = r0 + wm * 32 + cv_acc_row(r, lane);
                if (m < rows) {
                    float v = acc[r] + bb;
                    if (MODE == 0 && act == HGQ_ACT_RELU && !split) v = v > 0.f ? v : 0.f;
                    out[m * N + n] = v;
                }
            }
        }
    }
}

// y = act(sum of the k-split slices + bias), slices added in order.
__global__ __launch_bounds__(256) void splitk_finish_kernel(const float *__restrict__ part, int n_parts, int64_t n,
                                                            const float *__restrict__ bias, int N, int act,
                                                            float *__restrict__ out) {
    for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < n; e += (int64_t)gridDim.x * 256) {
        float v = 0.f;
        for (int p = 0; p < n_parts; ++p) v += part[(int64_t)p * n + e];
        if (bias) v += bias[e % N];
        if (act == HGQ_ACT_RELU) v = v > 0.f ? v : 0.f;
        out[e] = v;
    }
}

// Data gradient for inputs with few channels (C <= 4, e.g. the image itself), where a matrix-core
// tile would be almost empty.  FP = lanes per pixel (a power of two >= F): lane f of a pixel's
// group keeps the kernel entries W[tap, c, f] in registers, accumulates dz[tap pixel, f] * W over
// the taps with coalesced reads along f, and the group is summed with DPP steps at the end.
#define DG_MAXW 8192
// KH, KW > 0: kernel size known at compile time (all tap loads of a pixel in flight together); 0: any size.
template <int FP, int KH, int KW>
__global__ __launch_bounds__(256) void dgrad_smallc_kernel(const float *__restrict__ dz, const float *__restrict__ mask,
                                                           const float *__restrict__ w, float *__restrict__ out,
                                                           hgq_conv_geom g, int F, int64_t in_rows) {
    constexpr int PPW = 64 / FP;  // pixels per wavefront step
    extern __shared__ float wl[];  // the kernel, kh * kw * C * F floats
    const int lane = threadIdx.x & 63, f = lane % FP, slot = lane / FP;
    const int C = g.C, taps = g.kh * g.kw;
    const bool f_on = f < F;
    for (int t = threadIdx.x; t < taps * C * F; t += 256) wl[t] = w[t];
    __syncthreads();
    const bool unit = g.sy == 1 && g.sx == 1;
    const int64_t wave_id = ((int64_t)blockIdx.x * 256 + threadIdx.x) >> 6, n_waves = ((int64_t)gridDim.x * 256) >> 6;
    for (int64_t m0 = wave_id * PPW; m0 < in_rows; m0 += n_waves * PPW) {
        const int64_t m = m0 + slot;
        const RowInfo r = decode_row<1>(m, in_rows, g);
        float acc[4] = {0.f, 0.f, 0.f, 0.f};
        if (KH > 0) {
            constexpr int NT = KH * KW > 0 ? KH * KW : 1, KWD = KW > 0 ? KW : 1;
            float v[NT], km[NT];
            bool ok[NT];
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const int ky = t / KWD, kx = t % KWD;
                const int ty = r.y0 - ky * g.dly, tx = r.x0 - kx * g.dlx;
                const int oy = unit ? ty : ty / g.sy, ox = unit ? tx : tx / g.sx;
                ok[t] = r.base >= 0 && f_on && ty >= 0 && tx >= 0 && oy * g.sy == ty && ox * g.sx == tx && oy < g.OH && ox < g.OW;
                const int64_t a = ok[t] ? ((int64_t)r.base + oy * g.OW + ox) * F + f : 0;
                v[t] = dz[a];
                km[t] = mask ? mask[a] : 1.f;
            }
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const float vv = (ok[t] && km[t] > 0.f) ? v[t] : 0.f;
                const float *wt = wl + t * C * F + (f_on ? f : 0);
#pragma unroll
                for (int c = 0; c < 4; ++c)
                    if (c < C) acc[c] += vv * wt[c * F];
            }
        } else {
            // three taps at a time, loads issued together and unconditionally (clamped address)
            for (int ky = 0; ky < g.kh; ++ky) {
                const int ty = r.y0 - ky * g.dly;
                const int oy = unit ? ty : ty / g.sy;
                const bool oky = r.base >= 0 && f_on && ty >= 0 && oy * g.sy == ty && oy < g.OH;
                for (int kx0 = 0; kx0 < g.kw; kx0 += 3) {
                    float v[3], km[3];
                    bool ok[3];
#pragma unroll
                    for (int u = 0; u < 3; ++u) {
                        const int kx = kx0 + u;
                        const int tx = r.x0 - kx * g.dlx;
                        const int ox = unit ? tx : tx / g.sx;
                        ok[u] = oky && kx < g.kw && tx >= 0 && ox * g.sx == tx && ox < g.OW;
                        const int64_t a = ok[u] ? ((int64_t)r.base + oy * g.OW + ox) * F + f : 0;
                        v[u] = dz[a];
                        km[u] = mask ? mask[a] : 1.f;
                    }
#pragma unroll
                    for (int u = 0; u < 3; ++u) {
                        const int kx = kx0 + u;
                        if (kx < g.kw) {
                            const float vv = (ok[u] && km[u] > 0.f) ? v[u] : 0.f;
                            const float *wt = wl + (ky * g.kw + kx) * C * F + (f_on ? f : 0);
#pragma unroll
                            for (int c = 0; c < 4; ++c)
                                if (c < C) acc[c] += vv * wt[c * F];
                        }
                    }
                }
            }
        }
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            if (c < C) {
                const float tot = row_reduce_sum<FP>(acc[c]);
                if (f == 0 && m < in_rows) out[m * C + c] = tot;
            }
        }
    }
}

// The same for unit stride and dilation: a workgroup takes an 8 x 32 patch of input pixels,
// stages the (8 + kh - 1) x (32 + kw - 1) patch of dz it needs (masked, read once, coalesced
// along f) in LDS with the pixel stride padded to F + 1, and each thread contracts one pixel
// from LDS.
#define DP_TH 8
#define DP_TW 32
__global__ __launch_bounds__(256) void dgrad_patch_kernel(const float *__restrict__ dz, const float *__restrict__ mask,
                                                          const float *__restrict__ w, float *__restrict__ out,
                                                          hgq_conv_geom g, int F, int tiles_x, int tiles_y) {
    extern __shared__ float lds[];  // [kh * kw * C * F] kernel | [(DP_TH + kh - 1) * (DP_TW + kw - 1)][F + 1] patch
    const int C = g.C, taps = g.kh * g.kw;
    float *wl = lds, *patch = lds + taps * C * F;
    const int PH = DP_TH + g.kh - 1, PW = DP_TW + g.kw - 1, FS = F + 1;
    for (int t = threadIdx.x; t < taps * C * F; t += 256) wl[t] = w[t];
    const int tx = threadIdx.x % DP_TW, ty = threadIdx.x / DP_TW;
    const int64_t n_tiles = (int64_t)g.B * tiles_y * tiles_x;
    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const int b = (int)(tile / (tiles_y * tiles_x)), rem = (int)(tile - (int64_t)b * tiles_y * tiles_x);
        const int iy0 = (rem / tiles_x) * DP_TH, ix0 = (rem % tiles_x) * DP_TW;
        // patch origin in output coordinates: oy = iy + py - ky, ky = kh - 1 .. 0
        const int oy0 = iy0 + g.py - (g.kh - 1), ox0 = ix0 + g.px - (g.kw - 1);
        __syncthreads();
        // 32 lanes along f, 8 pixel columns at a time: no per-element index division
        const int fl = threadIdx.x & 31, pc0 = threadIdx.x >> 5;
        for (int pr = 0; pr < PH; ++pr) {
            const int oy = oy0 + pr;
            const bool row_ok = (unsigned)oy < (unsigned)g.OH;
            for (int pc = pc0; pc < PW; pc += 8) {
                const int ox = ox0 + pc;
                const bool ok = row_ok && (unsigned)ox < (unsigned)g.OW;
                const int64_t a0 = (((int64_t)b * g.OH + oy) * g.OW + ox) * F;
                for (int f = fl; f < F; f += 32) {
                    float v = 0.f;
                    if (ok) {
                        v = dz[a0 + f];
                        if (mask && !(mask[a0 + f] > 0.f)) v = 0.f;
                    }
                    patch[(pr * PW + pc) * FS + f] = v;
                }
            }
        }
        __syncthreads();
        const int iy = iy0 + ty, ix = ix0 + tx;
        if (iy < g.H && ix < g.W) {
            float acc[4] = {0.f, 0.f, 0.f, 0.f};
            for (int ky = 0; ky < g.kh; ++ky)
                for (int kx = 0; kx < g.kw; ++kx) {
                    // oy = iy + py - ky  ->  patch row ty + (kh - 1) - ky
                    const float *pp = patch + ((ty + g.kh - 1 - ky) * PW + (tx + g.kw - 1 - kx)) * FS;
                    const float *wt = wl + (ky * g.kw + kx) * C * F;
                    int f = 0;
                    for (; f + 8 <= F; f += 8) {  // eight LDS reads in flight per operand
                        float v[8];
#pragma unroll
                        for (int u = 0; u < 8; ++u) v[u] = pp[f + u];
#pragma unroll
                        for (int c = 0; c < 4; ++c) {
                            if (c < C) {
                                float wv[8];
#pragma unroll
                                for (int u = 0; u < 8; ++u) wv[u] = wt[c * F + f + u];
#pragma unroll
                                for (int u = 0; u < 8; ++u) acc[c] += v[u] * wv[u];
                            }
                        }
                    }
                    for (; f < F; ++f) {
                        const float v = pp[f];
#pragma unroll
                        for (int c = 0; c < 4; ++c)
                            if (c < C) acc[c] += v * wt[c * F + f];
                    }
                }
            const int64_t o = (((int64_t)b * g.H + iy) * g.W + ix) * C;
            for (int c = 0; c < C; ++c) out[o + c] = acc[c];
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Few input channels (C <= 4: the image itself), at most 32 filters, kernel size known at compile
// time.  A matrix-core tile would be almost empty and the layer is bound by the HBM traffic of the
// [.., F] tensor, so these kernels work on an 8 x 32 pixel tile per workgroup with lanes along
// the filter axis: every access to the F-wide tensor is a coalesced 128-byte row, the small
// operand sits in LDS and is read as a broadcast, the kernel entries of a lane sit in registers.
// ---------------------------------------------------------------------------------------------
#define SC_TH 8
#define SC_TW 32

// UNIT: unit stride and dilation - the patch sizes and every tap offset are compile-time constants (the LDS reads of a
// pixel then differ only in their immediate offsets: no address arithmetic in the loop).
template <int KH, int KW, int C, bool UNIT = false>
__global__ __launch_bounds__(256) void fwd_smallc_kernel(const float *__restrict__ x, const float *__restrict__ w,
                                                         const float *__restrict__ bias, float *__restrict__ out, hgq_conv_geom g,
                                                         int F, int act, int tiles_x, int tiles_y, float *__restrict__ pooled,
                                                         uint8_t *__restrict__ code) {
#pragma clang fp contract(fast)  // multiply-adds of the convolution sum may fuse (see bwd_smallc_kernel)
    constexpr int KC = KH * KW * C;
    extern __shared__ float lds[];  // input patch [XH][XW][C]
    const int sy = UNIT ? 1 : g.sy, sx = UNIT ? 1 : g.sx, dly = UNIT ? 1 : g.dly, dlx = UNIT ? 1 : g.dlx;
    const int XH = (SC_TH - 1) * sy + (KH - 1) * dly + 1, XW = (SC_TW - 1) * sx + (KW - 1) * dlx + 1;
    const int f = threadIdx.x & 31, slot = threadIdx.x >> 5;
    const bool f_on = f < F;
    float wreg[KC];
#pragma unroll
    for (int t = 0; t < KC; ++t) wreg[t] = f_on ? w[t * F + f] : 0.f;
    const float bb = (bias && f_on) ? bias[f] : 0.f;
    const __amdgpu_buffer_rsrc_t rs_x = buf_rsrc(x, (int64_t)g.B * g.H * g.W * C * 4);  // < 2 GiB (checked by the launcher)
    const int64_t n_tiles = (int64_t)g.B * tiles_y * tiles_x;
    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const int b = (int)(tile / (tiles_y * tiles_x)), rem = (int)(tile - (int64_t)b * tiles_y * tiles_x);
        const int oy0 = (rem / tiles_x) * SC_TH, ox0 = (rem % tiles_x) * SC_TW;
        const int iy0 = oy0 * sy - g.py, ix0 = ox0 * sx - g.px;
        __syncthreads();
        const FastDiv d_xw((uint32_t)(XW * C));
        for (int e = threadIdx.x; e < XH * XW * C; e += 256) {
            const int r = (int)d_xw.div((uint32_t)e), q = e - r * XW * C, iy = iy0 + r, ix = ix0 + q / C;
            const bool ok = (unsigned)iy < (unsigned)g.H && (unsigned)ix < (unsigned)g.W;
            lds[e] = buf_ld1(rs_x, ok ? (uint32_t)(((b * g.H + iy) * g.W + ix0) * C + q) * 4u : BUF_OOB);
        }
        __syncthreads();
        const int oy = oy0 + slot;
        if (oy < g.OH) {
            const int n_x = min(SC_TW, g.OW - ox0);
            float *orow = out ? out + (((int64_t)b * g.OH + oy) * g.OW + ox0) * F + f : nullptr;
            // `pooled`: also the 2 x 2 / stride 2 maxima, [B, OH / 2, OW / 2, F].  Tiles start on even rows and columns; a
            // window's two rows are the two halves of one wavefront (slots 2 w and 2 w + 1), its columns two trips of the loop.
            // `code` (same shape, one byte per window and filter): bits 0-1 = the place of the window's first maximum in
            // row-major order, bit 2 = that maximum is positive - all the backward pass needs of the unpooled output.
            const int PHo = g.OH >> 1, PWo = g.OW >> 1;
            const int64_t pbase = (((int64_t)b * PHo + (oy >> 1)) * PWo + (ox0 >> 1)) * F + f;
            float *prow = pooled ? pooled + pbase : nullptr;
            uint8_t *crow = code ? code + pbase : nullptr;
            const bool p_row = pooled && (oy >> 1) < PHo;  // both rows of the window exist: both halves are in this loop
            auto pixel = [&](int tx) -> float {
                const float *xp = lds + (slot * sy * XW + tx * sx) * C;
                float acc = bb;
#pragma unroll
                for (int t = 0; t < KC; ++t) {
                    const int ky = t / (KW * C), kx = (t / C) % KW, c = t % C;
                    acc += xp[(ky * dly * XW + kx * dlx) * C + c] * wreg[t];
                }
                if (act == HGQ_ACT_RELU) acc = acc > 0.f ? acc : 0.f;
                return acc;
            };
            // two pixels - the two columns of a pooling window - per trip: two independent sums in flight
            int tx = 0;
            for (; tx + 1 < n_x; tx += 2) {
                const float left = pixel(tx), acc = pixel(tx + 1);
                if (f_on && orow) orow[(int64_t)tx * F] = left, orow[(int64_t)(tx + 1) * F] = acc;
                if (p_row) {
                    const bool right = acc > left;
                    const float m = right ? acc : left, mo = __shfl_xor(m, 32);
                    const int j = right ? 1 : 0, jo = __shfl_xor(j, 32);
                    if (!(slot & 1) && f_on && ((ox0 + tx) >> 1) < PWo) {
                        const bool lower = mo > m;  // the lower row takes the window only with a larger value
                        const float best = lower ? mo : m;
                        prow[(int64_t)(tx >> 1) * F] = best;
                        if (crow) crow[(int64_t)(tx >> 1) * F] = (uint8_t)((lower ? 2 + jo : j) | (best > 0.f ? 4 : 0));
                    }
                }
            }
            if (tx < n_x) {  // a last column without a window
                const float acc = pixel(tx);
                if (f_on && orow) orow[(int64_t)tx * F] = acc;
            }
        }
    }
}

// Data, weight and bias gradient in one pass over dy (and the forward output for the ReLU mask),
// for unit stride and dilation.  A workgroup takes an 8 x 32 tile of INPUT pixels, stages the
// (8 + KH - 1) x (32 + KW - 1) patch of dz = dy * mask it touches (pixel stride F + 1 words) and
// the matching input patch, then
//   - thread = input pixel contracts the patch with the kernel (data gradient), and
//   - lane = filter, 8 row slots: every OUTPUT pixel is owned by exactly one tile (the patch
//     without its top / left halo; the first tile row / column also owns the pixels above / left
//     of it that exist because of the padding); a lane accumulates dz * x for its KC kernel
//     entries over the owned pixels in registers.
// After its last tile the workgroup adds the 8 slots in slot order and writes slice blockIdx.x of
// `part` ([KC * F | F]); a second kernel adds the slices in order.
// `dyp` (with `mask` = the forward output): the gradient arrives behind a 2 x 2 maximum pooling of stride 2 without
// padding, as [B, PHo, PWo, F]; dz is built from it while the patch is staged (the pooling layer's backward pass - one
// more read of the forward output and a write and a read of a gradient four times the size - does not run).
template <int KH, int KW, int C>
__global__ __launch_bounds__(256) void bwd_smallc_kernel(const float *__restrict__ dy, const float *__restrict__ mask,
                                                         const float *__restrict__ x, const float *__restrict__ w,
                                                         float *__restrict__ dx, float *__restrict__ part, hgq_conv_geom g, int F,
                                                         int tiles_x, int tiles_y, int vec, const float *__restrict__ dyp, int PHo,
                                                         int PWo, int relu, const uint8_t *__restrict__ code) {
    // the multiply-adds of the two contractions below may fuse (the file is built without contraction for the quantizer
    // arithmetic; a convolution sum has no such contract, and unfused it costs two vector instructions per term)
#pragma clang fp contract(fast)
    constexpr int KC = KH * KW * C, PH = SC_TH + KH - 1, PW = SC_TW + KW - 1;
    constexpr int XWS = PW + KW - 1;  // pixels between the rows of the input patch in LDS (at least PW + px: tap offsets are immediates)
    extern __shared__ float lds[];  // kernel [KC * F] | dz patch [PH * PW][F + 1] (reused for the final sum) | input patch
    const int FS = F + 1, XH = PH + g.py, XW = PW + g.px;
    float *zp = lds + ((KC * F + 3) & ~3), *xp = zp + max(PH * PW * FS, SC_TH * (KC + 1) * 32);
    const int tid = threadIdx.x, f = tid & 31, slot = tid >> 5;
    const bool f_on = f < F;
    // whole-tensor buffer descriptors (the launcher guarantees they are smaller than 2 GiB)
    const int64_t dy_bytes = (int64_t)g.B * g.OH * g.OW * F * 4;
    const __amdgpu_buffer_rsrc_t rs_dy = buf_rsrc(dy, dy_bytes), rs_mask = buf_rsrc(mask ? mask : dy, mask ? dy_bytes : 0),
                                 rs_x = buf_rsrc(x, (int64_t)g.B * g.H * g.W * C * 4),
                                 rs_dyp = buf_rsrc(dyp ? dyp : mask, dyp ? (int64_t)g.B * PHo * PWo * F * 4 : 0),
                                 rs_code = buf_rsrc(code ? (const void *)code : (const void *)dy, code ? (int64_t)g.B * PHo * PWo * F : 0);
    float wacc[KC], bacc = 0.f;
#pragma unroll
    for (int t = 0; t < KC; ++t) wacc[t] = 0.f;
    const bool two_step = KC <= F;  // the KC sums of a pixel fit into its dz row
    const int64_t n_tiles = (int64_t)g.B * tiles_y * tiles_x;
    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const int b = (int)(tile / (tiles_y * tiles_x)), rem = (int)(tile - (int64_t)b * tiles_y * tiles_x);
        const int iy0 = (rem / tiles_x) * SC_TH, ix0 = (rem % tiles_x) * SC_TW;
        const int oy0 = iy0 + g.py - (KH - 1), ox0 = ix0 + g.px - (KW - 1);
        __syncthreads();
        // buffer loads (zeros outside the tensor, no branch around a load): all units of a batch are in flight together
        if (dyp && code) {
            // the same units from the forward pass's byte per window and filter (place of the first maximum, and whether it
            // is positive) instead of the four outputs of the window: a sixteenth of the bytes
            const int f4 = F / 4, wpr = PW / 2, n_u = (PH / 2) * wpr * f4;
            const FastDiv d_f4((uint32_t)f4), d_wpr((uint32_t)wpr);
            for (int e0 = 0; e0 < n_u; e0 += 4 * 256) {
                f32x4_t gv[4];
                uint32_t cv[4];
                int dst[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int e = e0 + u * 256 + tid;
                    uint32_t off_g = BUF_OOB;
                    dst[u] = -1;
                    if (e < n_u) {
                        const int wi = (int)d_f4.div((uint32_t)e), f0 = (e - wi * f4) * 4, wr = (int)d_wpr.div((uint32_t)wi), wc = wi - wr * wpr;
                        const int oy = oy0 + 2 * wr, ox = ox0 + 2 * wc;
                        dst[u] = (2 * wr * PW + 2 * wc) * FS + f0;
                        if ((unsigned)oy < (unsigned)(2 * PHo) && (unsigned)ox < (unsigned)(2 * PWo))
                            off_g = (uint32_t)(((b * PHo + (oy >> 1)) * PWo + (ox >> 1)) * F + f0) * 4u;
                    }
                    gv[u] = buf_ld4(rs_dyp, off_g);
                    cv[u] = __float_as_uint(buf_ld1(rs_code, off_g == BUF_OOB ? BUF_OOB : off_g >> 2));
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    if (dst[u] < 0) continue;
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        const uint32_t cb = (cv[u] >> (8 * c)) & 0xffu;
                        const int first = (int)(cb & 3u);
                        const float gz = (!relu || (cb & 4u)) ? gv[u][c] : 0.f;
#pragma unroll
                        for (int j = 0; j < 4; ++j) zp[dst[u] + ((j >> 1) * PW + (j & 1)) * FS + c] = first == j ? gz : 0.f;
                    }
                }
            }
        } else if (dyp) {
            // unit = one pooling window x four filters (the patch starts on a window boundary and holds whole windows:
            // the launcher checks it).  An output pixel takes its window's gradient where it holds the window's first
            // maximum in row-major order - what the pooling kernels do - and, behind a ReLU, is positive.
            const int f4 = F / 4, wpr = PW / 2, n_u = (PH / 2) * wpr * f4;
            const FastDiv d_f4((uint32_t)f4), d_wpr((uint32_t)wpr);
            for (int e0 = 0; e0 < n_u; e0 += 2 * 256) {
                f32x4_t yv[2][4], gv[2];
                int dst[2];
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    const int e = e0 + u * 256 + tid;
                    uint32_t off_g = BUF_OOB, off_y = BUF_OOB;
                    dst[u] = -1;
                    if (e < n_u) {
                        const int wi = (int)d_f4.div((uint32_t)e), f0 = (e - wi * f4) * 4, wr = (int)d_wpr.div((uint32_t)wi), wc = wi - wr * wpr;
                        const int oy = oy0 + 2 * wr, ox = ox0 + 2 * wc;
                        dst[u] = (2 * wr * PW + 2 * wc) * FS + f0;
                        if ((unsigned)oy < (unsigned)(2 * PHo) && (unsigned)ox < (unsigned)(2 * PWo)) {
                            off_g = (uint32_t)(((b * PHo + (oy >> 1)) * PWo + (ox >> 1)) * F + f0) * 4u;
                            off_y = (uint32_t)(((b * g.OH + oy) * g.OW + ox) * F + f0) * 4u;
                        }
                    }
                    gv[u] = buf_ld4(rs_dyp, off_g);
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        yv[u][j] = buf_ld4(rs_mask, off_y == BUF_OOB ? BUF_OOB : off_y + (uint32_t)(((j >> 1) * g.OW + (j & 1)) * F) * 4u);
                }
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    if (dst[u] < 0) continue;
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        float best = yv[u][0][c];
                        int first = 0;
#pragma unroll
                        for (int j = 1; j < 4; ++j)
                            if (yv[u][j][c] > best) best = yv[u][j][c], first = j;
                        const float gz = (!relu || best > 0.f) ? gv[u][c] : 0.f;
#pragma unroll
                        for (int j = 0; j < 4; ++j) zp[dst[u] + ((j >> 1) * PW + (j & 1)) * FS + c] = first == j ? gz : 0.f;
                    }
                }
            }
        } else if (vec) {
            const int upr = PW * F / 4, n_u = PH * upr;
            const FastDiv d_upr((uint32_t)upr), d_f((uint32_t)F);  // no integer division per unit
            for (int e0 = 0; e0 < n_u; e0 += 4 * 256) {
                f32x4_t v[4], m[4];
                int dst[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int e = e0 + u * 256 + tid;
                    uint32_t off = BUF_OOB;
                    dst[u] = -1;
                    if (e < n_u) {
                        const int pr = (int)d_upr.div((uint32_t)e), q = (e - pr * upr) * 4, pc = (int)d_f.div((uint32_t)q), f0 = q - pc * F;
                        const int oy = oy0 + pr, ox = ox0 + pc;
                        dst[u] = (pr * PW + pc) * FS + f0;
                        if ((unsigned)oy < (unsigned)g.OH && (unsigned)ox < (unsigned)g.OW) off = (uint32_t)(((b * g.OH + oy) * g.OW + ox) * F + f0) * 4u;
                    }
                    v[u] = buf_ld4(rs_dy, off);
                    m[u] = buf_ld4(rs_mask, off);
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    if (dst[u] >= 0) {
#pragma unroll
                        for (int j = 0; j < 4; ++j) zp[dst[u] + j] = (!mask || m[u][j] > 0.f) ? v[u][j] : 0.f;
                    }
                }
            }
        } else {
            const int upr = PW * F, n_u = PH * upr;
            const FastDiv d_upr((uint32_t)upr), d_f((uint32_t)F);
            for (int e0 = 0; e0 < n_u; e0 += 8 * 256) {
                float v[8], m[8];
                int dst[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const int e = e0 + u * 256 + tid;
                    uint32_t off = BUF_OOB;
                    dst[u] = -1;
                    if (e < n_u) {
                        const int pr = (int)d_upr.div((uint32_t)e), q = e - pr * upr, pc = (int)d_f.div((uint32_t)q), f0 = q - pc * F;
                        const int oy = oy0 + pr, ox = ox0 + pc;
                        dst[u] = (pr * PW + pc) * FS + f0;
                        if ((unsigned)oy < (unsigned)g.OH && (unsigned)ox < (unsigned)g.OW) off = (uint32_t)(((b * g.OH + oy) * g.OW + ox) * F + f0) * 4u;
                    }
                    v[u] = buf_ld1(rs_dy, off);
                    m[u] = buf_ld1(rs_mask, off);
                }
#pragma unroll
                for (int u = 0; u < 8; ++u)
                    if (dst[u] >= 0) zp[dst[u]] = (!mask || m[u] > 0.f) ? v[u] : 0.f;
            }
        }
        if (part) {
            const FastDiv d_xw((uint32_t)(XW * C));
            for (int e = tid; e < XH * XW * C; e += 256) {
                const int r = (int)d_xw.div((uint32_t)e), q = e - r * XW * C, iy = iy0 - g.py + r, ix = ix0 - g.px + q / C;
                const bool ok = (unsigned)iy < (unsigned)g.H && (unsigned)ix < (unsigned)g.W;
                xp[r * XWS * C + q] = buf_ld1(rs_x, ok ? (uint32_t)(((b * g.H + iy) * g.W + ix) * C + q % C) * 4u : BUF_OOB);
            }
        }
        __syncthreads();
        if (dx && !two_step) {
            const int tx = tid % SC_TW, ty = tid / SC_TW;
            const int iy = iy0 + ty, ix = ix0 + tx;
            if (iy < g.H && ix < g.W) {
                float acc[C];
#pragma unroll
                for (int c = 0; c < C; ++c) acc[c] = 0.f;
#pragma unroll
                for (int ky = 0; ky < KH; ++ky) {
#pragma unroll
                    for (int kx = 0; kx < KW; ++kx) {
                        // oy = iy + py - ky  ->  patch row ty + (KH - 1) - ky
                        const float *pp = zp + ((ty + KH - 1 - ky) * PW + (tx + KW - 1 - kx)) * FS;
                        // kernel entries straight from memory: the address is the same in every lane, so they arrive
                        // through the scalar cache and enter the multiply-adds as scalar operands (no LDS reads for them)
                        const float *wt = w + (ky * KW + kx) * C * F;
                        int ff = 0;
                        for (; ff + 8 <= F; ff += 8) {
                            float v[8];
#pragma unroll
                            for (int u = 0; u < 8; ++u) v[u] = pp[ff + u];
#pragma unroll
                            for (int c = 0; c < C; ++c) {
                                float wv[8];
#pragma unroll
                                for (int u = 0; u < 8; ++u) wv[u] = wt[c * F + ff + u];
#pragma unroll
                                for (int u = 0; u < 8; ++u) acc[c] += v[u] * wv[u];
                            }
                        }
                        for (; ff < F; ++ff) {
                            const float v = pp[ff];
#pragma unroll
                            for (int c = 0; c < C; ++c) acc[c] += v * wt[c * F + ff];
                        }
                    }
                }
                const int64_t o = (((int64_t)b * g.H + iy) * g.W + ix) * C;
#pragma unroll
                for (int c = 0; c < C; ++c) dx[o + c] = acc[c];
            }
        }
        if (part && dyp) {
            // Behind the pooling at most ONE pixel of a 2 x 2 window has a gradient per filter: a lane walks the windows its
            // tile owns (a row slot takes every eighth), finds that pixel from the window's four dz values, and multiplies
            // the one input window under it - a quarter of the multiply-adds of the walk over pixels below.  (Whole windows
            // only have gradient, and the tiles' ownership boundaries fall on window boundaries: kh - 1 and kw - 1 are even.)
            const int pc_lo = ix0 == 0 ? max(0, -ox0) : KW - 1, pc_hi = min(PW, g.OW - ox0);
            const int wr_lo = iy0 == 0 ? max(0, -oy0 / 2) : (KH - 1) / 2, wr_hi = min(PH / 2, (g.OH - oy0 + 1) >> 1);
            const int wc_lo = pc_lo >> 1, ncol = min(PW / 2, (pc_hi + 1) >> 1) - wc_lo, n_w = (wr_hi - wr_lo) * ncol;
            if (ncol > 0 && wr_hi > wr_lo) {
                const FastDiv d_nc((uint32_t)ncol);
                for (int wi = slot; wi < n_w; wi += SC_TH) {
                    const int r = (int)d_nc.div((uint32_t)wi), wr = wr_lo + r, wc = wc_lo + (wi - r * ncol);
                    const float *zq = zp + (2 * wr * PW + 2 * wc) * FS + f;
                    const float z0 = f_on ? zq[0] : 0.f, z1 = f_on ? zq[FS] : 0.f, z2 = f_on ? zq[PW * FS] : 0.f,
                                z3 = f_on ? zq[(PW + 1) * FS] : 0.f;
                    const float z = (z0 + z1) + (z2 + z3);  // one of them at most is not zero
                    const int dyb = (z2 != 0.f || z3 != 0.f) ? 1 : 0, dxb = (z1 != 0.f || z3 != 0.f) ? 1 : 0;
                    bacc += z;
                    const float *xq = xp + ((2 * wr + dyb - (KH - 1) + g.py) * XWS + (2 * wc + dxb - (KW - 1) + g.px)) * C;
#pragma unroll
                    for (int t = 0; t < KC; ++t) wacc[t] += xq[((t / (KW * C)) * XWS + (t / C) % KW) * C + t % C] * z;
                }
            }
        } else if (part) {
            for (int pr = slot; pr < PH; pr += SC_TH) {
                const int oy = oy0 + pr;
                if ((unsigned)oy >= (unsigned)g.OH || !(pr >= KH - 1 || iy0 == 0)) continue;
                const int pc_lo = ix0 == 0 ? max(0, -ox0) : KW - 1, pc_hi = min(PW, g.OW - ox0);
                // input pixel of tap (ky, kx): patch-relative (pr + ky - (KH - 1) + py, pc + kx - (KW - 1) + px).  The KH x KW
                // window of a pixel shares all but one column with its left neighbour's: it lives in registers and takes KH * C
                // new entries per pixel (LDS broadcasts) instead of KC
                const float *xq = xp + ((pr - (KH - 1) + g.py) * XWS + (pc_lo - (KW - 1) + g.px)) * C;
                float xw[KH][KW * C];
#pragma unroll
                for (int ky = 0; ky < KH; ++ky)
#pragma unroll
                    for (int j = 0; j < (KW - 1) * C; ++j) xw[ky][j + C] = xq[ky * XWS * C + j];
                for (int pc = pc_lo; pc < pc_hi; ++pc, xq += C) {
                    const float z = f_on ? zp[(pr * PW + pc) * FS + f] : 0.f;
                    bacc += z;
#pragma unroll
                    for (int ky = 0; ky < KH; ++ky) {
#pragma unroll
                        for (int j = 0; j < (KW - 1) * C; ++j) xw[ky][j] = xw[ky][j + C];
#pragma unroll
                        for (int c = 0; c < C; ++c) xw[ky][(KW - 1) * C + c] = xq[(ky * XWS + KW - 1) * C + c];
                    }
#pragma unroll
                    for (int t = 0; t < KC; ++t) wacc[t] += xw[t / (KW * C)][t % (KW * C)] * z;
                }
            }
        }
        if (dx && two_step) {
            // data gradient in two steps, after the weight gradient has read dz: (1) thread = OUTPUT pixel of the patch
            // contracts its F entries of dz with the kernel - KC sums u[tap] - and writes them over the start of its own dz
            // row (nobody else touches that row); (2) thread = input pixel adds the KH * KW * C sums that meet in it.  One LDS
            // read of dz feeds KC multiply-adds instead of one.
            __syncthreads();
            for (int p = tid; p < PH * PW; p += 256) {
                float *row = zp + p * FS;
                float u[KC];
#pragma unroll
                for (int t = 0; t < KC; ++t) u[t] = 0.f;
                int ff = 0;
                for (; ff + 8 <= F; ff += 8) {
                    float v[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) v[j] = row[ff + j];
#pragma unroll
                    for (int t = 0; t < KC; ++t) {
                        float wv[8];  // the same address in every lane: scalar loads
#pragma unroll
                        for (int j = 0; j < 8; ++j) wv[j] = w[t * F + ff + j];
#pragma unroll
                        for (int j = 0; j < 8; ++j) u[t] += v[j] * wv[j];
                    }
                }
                for (; ff < F; ++ff) {
                    const float v = row[ff];
#pragma unroll
                    for (int t = 0; t < KC; ++t) u[t] += v * w[t * F + ff];
                }
#pragma unroll
                for (int t = 0; t < KC; ++t) row[t] = u[t];
            }
            __syncthreads();
            const int tx = tid % SC_TW, ty = tid / SC_TW;
            const int iy = iy0 + ty, ix = ix0 + tx;
            if (iy < g.H && ix < g.W) {
                float acc[C];
#pragma unroll
                for (int c = 0; c < C; ++c) acc[c] = 0.f;
#pragma unroll
                for (int ky = 0; ky < KH; ++ky)
#pragma unroll
                    for (int kx = 0; kx < KW; ++kx) {
                        // oy = iy + py - ky  ->  patch row ty + (KH - 1) - ky
                        const float *up = zp + ((ty + KH - 1 - ky) * PW + (tx + KW - 1 - kx)) * FS + (ky * KW + kx) * C;
#pragma unroll
                        for (int c = 0; c < C; ++c) acc[c] += up[c];
                    }
                const int64_t o = (((int64_t)b * g.H + iy) * g.W + ix) * C;
#pragma unroll
                for (int c = 0; c < C; ++c) dx[o + c] = acc[c];
            }
        }
    }
    if (part) {
        __syncthreads();
        float *red = zp;  // [slot][KC + 1][32]
#pragma unroll
        for (int t = 0; t < KC; ++t) red[(slot * (KC + 1) + t) * 32 + f] = wacc[t];
        red[(slot * (KC + 1) + KC) * 32 + f] = bacc;
        __syncthreads();
        float *my = part + (int64_t)blockIdx.x * ((int64_t)KC * F + F);
        for (int e = tid; e < (KC + 1) * 32; e += 256) {
            const int t = e >> 5, ff = e & 31;
            if (ff < F) {
                float sacc = 0.f;
                for (int u = 0; u < SC_TH; ++u) sacc += red[(u * (KC + 1) + t) * 32 + ff];
                my[(int64_t)t * F + ff] = sacc;
            }
        }
    }
}

// Weight / bias gradient.  Workgroup (kt, nt, split): k tile of 32 * WK columns of the im2col
// matrix, n tile of 32 * WN filters, rows [split * chunk, (split + 1) * chunk) taken 32 * WS at
// a step, WS wavefronts sharing one output block (combined through LDS at the end);
// WK * WN * WS = 4.  Slice `split` of `part` is [K * F | F].
template <int WK, int WN, int WS, bool BF = false>
__global__ __launch_bounds__(256) void wgrad_kernel(const float *__restrict__ src, const float *__restrict__ dy,
                                                    const float *__restrict__ y, float *__restrict__ part, hgq_conv_geom g,
                                                    int F, int64_t rows, int K, int64_t chunk, int act, int n_ktiles) {
    constexpr int BKT = 32 * WK, BN = 32 * WN, BMS = 32 * WS;
    static_assert(WK * WN * WS == 4, "four wavefronts");
    __shared__ float as[BMS][BKT + 1];
    __shared__ float zs[BMS][BN + 1];
    __shared__ RowInfo rinfo[BMS];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wsub = wave / (WK * WN), wk = (wave / WN) % WK, wn = wave % WN;
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
        const int kq = lane >> 5, c32 = lane & 31, mb = wsub * 32;
        if (BF) {
            acc = mfma_chain_bf16<false, true>(acc, &as[mb + kq][wk * 32 + c32], BKT + 1, &zs[mb + kq][wn * 32 + c32], BN + 1, 2);
        } else {
#pragma unroll
            for (int mm = 0; mm < 32; mm += 2)
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(as[mb + mm + kq][wk * 32 + c32], zs[mb + mm + kq][wn * 32 + c32], acc, 0, 0, 0);
        }
    }
    __syncthreads();
    float *red = &as[0][0];  // BMS * (BKT + 1) >= 4096 floats whenever WS > 1
    if (WS > 1) {
        // the WS wavefronts of an output block add up in wavefront order
        const int blk = wk * WN + wn;  // output block of this wavefront
#pragma unroll
        for (int r = 0; r < 16; ++r) red[((blk * WS + wsub) * 32 + cv_acc_row(r, lane)) * 32 + (lane & 31)] = acc[r];
        __syncthreads();
        if (wsub == 0) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                float v = 0.f;
                for (int u = 0; u < WS; ++u) v += red[((blk * WS + u) * 32 + cv_acc_row(r, lane)) * 32 + (lane & 31)];
                acc[r] = v;
            }
        }
        __syncthreads();
    }
    const int n = n0 + wn * 32 + (lane & 31);
    if (wsub == 0 && n < F) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int k = k0 + wk * 32 + cv_acc_row(r, lane);
            if (k < K) my[(int64_t)k * F + n] = acc[r];
        }
    }
    if (kt == 0) {
        // bias gradient: threads with the same dz column add up in a fixed order
        red[tid] = bsum;
        __syncthreads();
        if (tid < BN && n0 + tid < F) {
            float s = 0.f;
            for (int j = 0; j < 256 / BN; ++j) s += red[tid + j * BN];
            my[KF + n0 + tid] = s;
        }
    }
}

// The weight / bias gradient for C and F multiples of 4 and 16-byte aligned operands: 128-bit
// gathers and dz loads, the loads of row step s + 1 in flight while the matrix cores work on
// step s (two LDS buffers, one barrier per step).  Same tiling and slice layout as wgrad_kernel.
// BF: the contraction on the bf16 matrix instruction over exact bf16 parts (mfma_chain_bf16; dz is an arbitrary fp32 tensor).
// ZS: the filter count is not a multiple of 4 (or dy is not 16-byte aligned): dz and the mask are loaded element by element,
// columns past F as zeros; the gathers of the source stay 128 bits wide.
template <int WK, int WN, int WS, bool BF = false, bool ZS = false>
__global__ __launch_bounds__(256) void wgrad_vec_kernel(const float *__restrict__ src, const float *__restrict__ dy,
                                                        const float *__restrict__ y, float *__restrict__ part, hgq_conv_geom g,
                                                        int F, int64_t rows, int K, int64_t chunk, int act, int n_ktiles) {
    constexpr int BKT = 32 * WK, BN = 32 * WN, BMS = 32 * WS;
    constexpr int AQ = 8 * WK, AP = WS * WK, AR = 32 / WK;  // A: float4 per row, passes per thread, rows per pass
    constexpr int ZQ = 8 * WN, ZP = WS * WN, ZR = 32 / WN;  // dz: the same
    constexpr int AST = BKT + 4, ZST = BN + 4;
    static_assert(WK * WN * WS == 4, "four wavefronts");
    __shared__ float as[2][BMS][AST];
    __shared__ float zs[2][BMS][ZST];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wsub = wave / (WK * WN), wk = (wave / WN) % WK, wn = wave % WN;
    const int kt = blockIdx.x % n_ktiles, nt = blockIdx.x / n_ktiles;
    const int k0 = kt * BKT, n0 = nt * BN;
    const int64_t m_begin = (int64_t)blockIdx.y * chunk, m_end = min(rows, m_begin + chunk);
    const int64_t KF = (int64_t)K * F;
    float *my = part + (int64_t)blockIdx.y * (KF + F);
    const int aq = tid % AQ, ar = tid / AQ, zq = tid % ZQ, zr = tid / ZQ;
    const ColInfo ci = decode_col<0>(k0 + 4 * aq, K, g, F);
    const bool z_on = n0 + 4 * zq < F, relu = act == HGQ_ACT_RELU;
    // whole-tensor buffer descriptors (the launcher guarantees they are smaller than 2 GiB)
    const __amdgpu_buffer_rsrc_t rs_src = buf_rsrc(src, (int64_t)g.B * g.H * g.W * g.C * 4), rs_dy = buf_rsrc(dy, rows * F * 4),
                                 rs_y = buf_rsrc(relu ? y : dy, relu ? rows * F * 4 : 0);
    floatx16 acc = {0};
    f32x4_t bsum = {0.f, 0.f, 0.f, 0.f};
    f32x4_t av[AP], zv[ZP], zm[ZP];
    auto fetch = [&](int64_t m0) {
#pragma unroll
        for (int p = 0; p < AP; ++p) {
            const int64_t m = m0 + ar + AR * p;
            const RowInfo ri = decode_row<0>(m < m_end ? m : rows, rows, g);
            av[p] = buf_ld4(rs_src, gather4_offset<0>(ri, ci, g, F));
        }
#pragma unroll
        for (int p = 0; p < ZP; ++p) {
            const int64_t m = m0 + zr + ZR * p;
            if (ZS) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint32_t off = (m < m_end && n0 + 4 * zq + j < F) ? (uint32_t)(m * F + n0 + 4 * zq + j) * 4u : BUF_OOB;
                    zv[p][j] = buf_ld1(rs_dy, off);
                    zm[p][j] = buf_ld1(rs_y, off);
                }
            } else {
                const uint32_t off = (m < m_end && z_on) ? (uint32_t)(m * F + n0 + 4 * zq) * 4u : BUF_OOB;
                zv[p] = buf_ld4(rs_dy, off);
                zm[p] = buf_ld4(rs_y, off);
            }
        }
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int p = 0; p < AP; ++p) *(f32x4_t *)&as[buf][ar + AR * p][4 * aq] = av[p];
#pragma unroll
        for (int p = 0; p < ZP; ++p) {
            f32x4_t v = zv[p];
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (relu && !(zm[p][j] > 0.f)) v[j] = 0.f;
            bsum += v;
            *(f32x4_t *)&zs[buf][zr + ZR * p][4 * zq] = v;
        }
    };
    const int64_t n_steps = m_end > m_begin ? (m_end - m_begin + BMS - 1) / BMS : 0;
    if (n_steps > 0) {
        fetch(m_begin);
        stash(0);
    }
    __syncthreads();
    for (int64_t st = 0; st < n_steps; ++st) {
        const int buf = (int)(st & 1);
        const bool more = st + 1 < n_steps;
        if (more) fetch(m_begin + (st + 1) * BMS);
        const int kq = lane >> 5, c32 = lane & 31, mb = wsub * 32;
        if (BF) {
            acc = mfma_chain_bf16<false, true>(acc, &as[buf][mb + kq][wk * 32 + c32], AST, &zs[buf][mb + kq][wn * 32 + c32], ZST, 2);
        } else {
#pragma unroll
            for (int mm = 0; mm < 32; mm += 2)
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(as[buf][mb + mm + kq][wk * 32 + c32], zs[buf][mb + mm + kq][wn * 32 + c32], acc, 0, 0, 0);
        }
        if (more) stash(buf ^ 1);
        __syncthreads();
    }
    float *red = &as[0][0][0];  // 2 * BMS * AST >= 4096 floats whenever WS > 1
    if (WS > 1) {
        const int blk = wk * WN + wn;
#pragma unroll
        for (int r = 0; r < 16; ++r) red[((blk * WS + wsub) * 32 + cv_acc_row(r, lane)) * 32 + (lane & 31)] = acc[r];
        __syncthreads();
        if (wsub == 0) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                float v = 0.f;
                for (int u = 0; u < WS; ++u) v += red[((blk * WS + u) * 32 + cv_acc_row(r, lane)) * 32 + (lane & 31)];
                acc[r] = v;
            }
        }
        __syncthreads();
    }
    const int n = n0 + wn * 32 + (lane & 31);
    if (wsub == 0 && n < F) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int k = k0 + wk * 32 + cv_acc_row(r, lane);
            if (k < K) my[(int64_t)k * F + n] = acc[r];
        }
    }
    if (kt == 0) {
        // bias gradient: the threads that share four dz columns add up in a fixed order
#pragma unroll
        for (int j = 0; j < 4; ++j) red[tid * 4 + j] = bsum[j];
        __syncthreads();
        if (tid < BN && n0 + tid < F) {
            float sacc = 0.f;
            for (int u = 0; u < 256 / ZQ; ++u) sacc += red[(u * ZQ + tid / 4) * 4 + tid % 4];
            my[KF + n0 + tid] = sacc;
        }
    }
}

struct WgradCfg {
    int wk, wn, ws;
    int n_kt, n_nt;
};
static WgradCfg wgrad_cfg(int K, int F) {
    WgradCfg c;
    if (F > 32) c.wk = 2, c.wn = 2, c.ws = 1;
    else if (K <= 32) c.wk = 1, c.wn = 1, c.ws = 4;
    else if (K <= 64) c.wk = 2, c.wn = 1, c.ws = 2;
    else c.wk = 4, c.wn = 1, c.ws = 1;
    c.n_kt = (K + 32 * c.wk - 1) / (32 * c.wk), c.n_nt = (F + 32 * c.wn - 1) / (32 * c.wn);
    return c;
}

// k-split of the forward for few output tiles and a long contraction (a wide dense layer on a small batch)
static int fwd_ksplit(int64_t rows, int K, int F) {
    const int64_t tiles = F <= 32 ? (rows + 127) / 128 : ((rows + 63) / 64) * ((F + 63) / 64);
    if (tiles >= 256 || K < 512) return 1;
    int64_t s = 512 / tiles;
    if (s > K / 128) s = K / 128;
    if (s > 64) s = 64;
    return s < 1 ? 1 : (int)s;
}


// EBOPs of a convolution: sum over all output pixels and filters of conv(bits_in, bits_ker), and
// its gradient, without running the convolution:
//     S[tap, c] = sum of bits_in over the input pixels that tap visits,   Wsum[tap, c] = sum_f bits_ker[tap, c, f]
//     total = sum S * Wsum;   d total / d bits_ker[tap, c, f] = S[tap, c];
//     d total / d bits_in[y, x, c] = sum over the taps that visit (y, x) of Wsum[tap, c]
// The pixels a tap visits form a (strided) rectangle, so S is computed separably: column sums
// R[ky][x][c] over the visited rows first, then sums of R over the visited columns.
// One workgroup; every quantity is a sum of small integers, exact in fp32 in any order while below 2^24.
#define CE_MAX 4096   // kh * kw * C
#define CE_MAXR 8192  // kh * W * C
#define CE_MAXV 2048  // H * kh and W * kw
__global__ __launch_bounds__(1024) void conv_ebops_kernel(const float *__restrict__ bits_in, const float *__restrict__ bits_ker,
                                                          hgq_conv_geom g, int F, float *total,
                                                          float *__restrict__ g_in, float *__restrict__ g_ker) {
    __shared__ float S[CE_MAX], R[CE_MAXR];
    __shared__ int Ws[CE_MAX];  // integer sums: native LDS atomics
    __shared__ float red[1024];
    __shared__ unsigned char vy[CE_MAXV], vx[CE_MAXV];  // vy[y * kh + ky]: row y is visited by kernel row ky
    const int t = threadIdx.x, taps = g.kh * g.kw, TC = taps * g.C, WC = g.W * g.C;
    // flat sweeps decode their index with float reciprocals (every swept range is below 2**21: checked by the launcher)
    const FastDiv by_wc((uint32_t)WC), by_f((uint32_t)F), by_c((uint32_t)g.C), by_kw((uint32_t)g.kw);
    for (int e = t; e < TC; e += 1024) Ws[e] = 0;
    for (int e = t; e < g.H * g.kh; e += 1024) {
        const int y = e / g.kh, ky = e - y * g.kh, ty = y + g.py - ky * g.dly;
        vy[e] = ty >= 0 && ty % g.sy == 0 && ty / g.sy < g.OH;
    }
    for (int e = t; e < g.W * g.kw; e += 1024) {
        const int x = e / g.kw, kx = e - x * g.kw, tx = x + g.px - kx * g.dlx;
        vx[e] = tx >= 0 && tx % g.sx == 0 && tx / g.sx < g.OW;
    }
    // R[ky][x][c]: adjacent threads take adjacent (x, c), so every row read is coalesced
    for (int e = t; e < g.kh * WC; e += 1024) {
        const int ky = (int)by_wc.div((uint32_t)e), xc = e - ky * WC;
        float r = 0.f;
        int oy = 0;
        for (; oy + 4 <= g.OH; oy += 4) {
            float v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int iy = (oy + u) * g.sy - g.py + ky * g.dly;
                v[u] = (unsigned)iy < (unsigned)g.H ? bits_in[(int64_t)iy * WC + xc] : 0.f;
            }
            r += (v[0] + v[1]) + (v[2] + v[3]);
        }
        for (; oy < g.OH; ++oy) {
            const int iy = oy * g.sy - g.py + ky * g.dly;
            if ((unsigned)iy < (unsigned)g.H) r += bits_in[(int64_t)iy * WC + xc];
        }
        R[e] = r;
    }
    __syncthreads();
    const int n_w = TC * F;
    for (int e0 = 0; e0 < n_w; e0 += 4 * 1024) {
        float v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int e = e0 + u * 1024 + t;
            v[u] = e < n_w ? bits_ker[e] : 0.f;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int e = e0 + u * 1024 + t;
            if (e < n_w) atomicAdd(&Ws[by_f.div((uint32_t)e)], (int)v[u]);
        }
    }
    for (int e = t; e < TC; e += 1024) {
        const int tap = (int)by_c.div((uint32_t)e), c = e - tap * g.C, ky = (int)by_kw.div((uint32_t)tap), kx = tap - ky * g.kw;
        float sacc = 0.f;
        for (int ox = 0; ox < g.OW; ++ox) {
            const int ix = ox * g.sx - g.px + kx * g.dlx;
            if ((unsigned)ix < (unsigned)g.W) sacc += R[ky * WC + ix * g.C + c];
        }
        S[e] = sacc;
    }
    __syncthreads();
    float part = 0.f;
    for (int e = t; e < TC; e += 1024) part += S[e] * (float)Ws[e];
    red[t] = part;
    __syncthreads();
    for (int o = 512; o > 0; o >>= 1) {
        if (t < o) red[t] += red[t + o];
        __syncthreads();
    }
    if (t == 0) total[0] = red[0];
    if (g_ker)
        for (int e = t; e < n_w; e += 1024) g_ker[e] = S[by_f.div((uint32_t)e)];
    if (g_in) {
        for (int e = t; e < g.H * WC; e += 1024) {
            const int y = (int)by_wc.div((uint32_t)e), xc = e - y * WC, x = (int)by_c.div((uint32_t)xc), c = xc - x * g.C;
            float a = 0.f;
            for (int ky = 0; ky < g.kh; ++ky) {
                if (!vy[y * g.kh + ky]) continue;
                for (int kx = 0; kx < g.kw; ++kx)
                    if (vx[x * g.kw + kx]) a += (float)Ws[(ky * g.kw + kx) * g.C + c];
            }
            g_in[e] = a;
        }
    }
}

// The same estimate straight from the quantizers' raw variables, as one launch for the whole `_compute_ebops` of a
// convolution layer: bits are formed on the fly (hgq_qbits_fwd's rule), the bias term, the scale factors, the uint32
// variable, the loss term ebops * beta and the gradients of that term with respect to the variables (straight-through
// rounding, hgq_qbits_bwd's rule) all come out of it.  Every operand must have one bit-width entry per cell.
__device__ __forceinline__ float ce_bits(const hgq_bits_desc &d, uint32_t j, bool &open) {
    float b;
    open = true;
    if (d.kbi) {
        b = rintf(d.fb[j]);
    } else {
        const float sum = __fadd_rn(rintf(d.i[j]), rintf(d.fb[j]));
        open = sum > 0.f;
        b = open ? sum : 0.f;
    }
    if (d.add_mode == 1) b = __fadd_rn(b, (float)d.k[j]);
    else if (d.add_mode == 2) b = __fadd_rn(b, (float)d.k[j] * (b > 0.f ? 1.f : 0.f));
    return b;
}
__device__ __forceinline__ void ce_put(const hgq_bits_desc &d, uint32_t j, bool open, float g) {
    if (d.kbi) {
        d.g_fb[j] = g;
    } else {
        d.g_i[j] = open ? g : 0.f, d.g_fb[j] = open ? g : 0.f;
    }
}

// The bit-widths of n cells of one operand into LDS, a byte per cell (bits 0-6 the width, bit 7 "open": the straight-through
// gradient is not closed).  Eight cells of a thread per trip, every load of the trip issued before the first value is used:
// one workgroup sweeping an operand a load at a time pays a memory latency per cell and thread.
__device__ __forceinline__ void ce_stage_bits(const hgq_bits_desc &d, int n, unsigned char *dst, int *bad) {
    const bool has_i = !d.kbi, has_k = d.add_mode != 0;
    for (int e0 = 0; e0 < n; e0 += 8 * 1024) {
        float iv[8], fv[8];
        unsigned char kv[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int e = e0 + u * 1024 + (int)threadIdx.x, j = e < n ? e : 0;
            fv[u] = d.fb[j];
            iv[u] = has_i ? d.i[j] : 0.f;
            kv[u] = has_k ? d.k[j] : (unsigned char)0;
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int e = e0 + u * 1024 + (int)threadIdx.x;
            float b;
            bool open = true;
            if (d.kbi) {
                b = rintf(fv[u]);
            } else {
                const float sum = __fadd_rn(rintf(iv[u]), rintf(fv[u]));
                open = sum > 0.f;
                b = open ? sum : 0.f;
            }
            if (d.add_mode == 1) b = __fadd_rn(b, (float)kv[u]);
            else if (d.add_mode == 2) b = __fadd_rn(b, (float)kv[u] * (b > 0.f ? 1.f : 0.f));
            if (e < n) {
                if (!(b >= 0.f && b <= 127.f)) *bad = 1;  // a width a byte cannot hold (a negative `_b`): the sweeps read the variables instead
                dst[e] = (unsigned char)((int)fminf(fmaxf(b, 0.f), 127.f) | (open ? 0x80 : 0));
            }
        }
    }
}

// STAGED: both operands' bit-widths are formed once into dynamic LDS (H W C + kh kw C F bytes) and every later sweep reads
// them there; otherwise (operands too large for that, or a width outside 0 .. 127) every sweep forms them from the variables
// in memory.
template <bool STAGED>
__global__ __launch_bounds__(1024) void conv_ebops_q_kernel(hgq_bits_desc din, hgq_bits_desc dker, hgq_bits_desc dbias, int has_bias,
                                                            hgq_conv_geom g, int F, float conv_scale, float bias_size, float factor,
                                                            const float *beta, uint32_t *ebops_u32, float *loss_term) {
    __shared__ float S[CE_MAX], R[CE_MAXR];
    __shared__ int Ws[CE_MAX];
    __shared__ float red[1024];
    __shared__ unsigned char vy[CE_MAXV], vx[CE_MAXV];
    extern __shared__ unsigned char ce_dyn[];
    const int t = threadIdx.x, taps = g.kh * g.kw, TC = taps * g.C, WC = g.W * g.C;
    unsigned char *bi = ce_dyn, *bk = ce_dyn + ((g.H * WC + 15) & ~15);
    __shared__ int ce_bad;
    bool use_staged = false;
    auto bits_of = [&](const hgq_bits_desc &d, const unsigned char *staged, uint32_t j, bool &open) -> float {
        if (STAGED && use_staged) {
            const unsigned char v = staged[j];
            open = (v & 0x80) != 0;
            return (float)(v & 0x7f);
        }
        return ce_bits(d, j, open);
    };
    if (STAGED) {
        if (t == 0) ce_bad = 0;
        __syncthreads();
        ce_stage_bits(din, g.H * WC, bi, &ce_bad);
        ce_stage_bits(dker, TC * F, bk, &ce_bad);
        __syncthreads();
        use_staged = ce_bad == 0;
    }
    const FastDiv by_wc((uint32_t)WC), by_f((uint32_t)F), by_c((uint32_t)g.C), by_kw((uint32_t)g.kw);
    for (int e = t; e < TC; e += 1024) Ws[e] = 0;
    for (int e = t; e < g.H * g.kh; e += 1024) {
        const int y = e / g.kh, ky = e - y * g.kh, ty = y + g.py - ky * g.dly;
        vy[e] = ty >= 0 && ty % g.sy == 0 && ty / g.sy < g.OH;
    }
    for (int e = t; e < g.W * g.kw; e += 1024) {
        const int x = e / g.kw, kx = e - x * g.kw, tx = x + g.px - kx * g.dlx;
        vx[e] = tx >= 0 && tx % g.sx == 0 && tx / g.sx < g.OW;
    }
    for (int e = t; e < g.kh * WC; e += 1024) {
        const int ky = (int)by_wc.div((uint32_t)e), xc = e - ky * WC;
        float r = 0.f;
        for (int oy = 0; oy < g.OH; ++oy) {
            const int iy = oy * g.sy - g.py + ky * g.dly;
            bool open;
            if ((unsigned)iy < (unsigned)g.H) r += bits_of(din, bi, (uint32_t)(iy * WC + xc), open);
        }
        R[e] = r;
    }
    __syncthreads();
    const int n_w = TC * F;
    for (int e = t; e < n_w; e += 1024) {
        bool open;
        atomicAdd(&Ws[by_f.div((uint32_t)e)], (int)bits_of(dker, bk, (uint32_t)e, open));
    }
    for (int e = t; e < TC; e += 1024) {
        const int tap = (int)by_c.div((uint32_t)e), c = e - tap * g.C, ky = (int)by_kw.div((uint32_t)tap), kx = tap - ky * g.kw;
        float sacc = 0.f;
        for (int ox = 0; ox < g.OW; ++ox) {
            const int ix = ox * g.sx - g.px + kx * g.dlx;
            if ((unsigned)ix < (unsigned)g.W) sacc += R[ky * WC + ix * g.C + c];
        }
        S[e] = sacc;
    }
    __syncthreads();
    float part = 0.f;
    for (int e = t; e < TC; e += 1024) part += S[e] * (float)Ws[e];
    red[t] = part;
    __syncthreads();
    for (int o = 512; o > 0; o >>= 1) {
        if (t < o) red[t] += red[t + o];
        __syncthreads();
    }
    const float conv_total = red[0];
    __syncthreads();
    float bias_sum = 0.f;
    if (has_bias) {
        float bs = 0.f;
        for (int n = t; n < F; n += 1024) {
            bool open;
            bs += ce_bits(dbias, (uint32_t)n, open);
        }
        red[t] = bs;
        __syncthreads();
        for (int o = 512; o > 0; o >>= 1) {
            if (t < o) red[t] += red[t + o];
            __syncthreads();
        }
        bias_sum = red[0];
    }
    // the reference's order: sum(conv) * (pf / n_parallel) + mean(bits_bias) * size, then * ebops_factor
    const float ebops = __fmul_rn(__fadd_rn(__fmul_rn(conv_total, conv_scale), has_bias ? __fmul_rn(__fdiv_rn(bias_sum, (float)F), bias_size) : 0.f), factor);
    const float gs = beta[0] * factor;  // gradients are those of the loss term ebops * beta
    if (t == 0) {
        if (ebops_u32) ebops_u32[0] = (uint32_t)ebops;
        loss_term[0] = ebops * beta[0];
    }
    for (int e = t; e < n_w; e += 1024) {
        bool open;  // a KIF kernel quantizer's width relu(i + f) is flat where i + f <= 0
        (void)bits_of(dker, bk, (uint32_t)e, open);
        ce_put(dker, (uint32_t)e, open, S[by_f.div((uint32_t)e)] * conv_scale * gs);
    }
    for (int e = t; e < g.H * WC; e += 1024) {
        const int y = (int)by_wc.div((uint32_t)e), xc = e - y * WC, x = (int)by_c.div((uint32_t)xc), c = xc - x * g.C;
        float a = 0.f;
        for (int ky = 0; ky < g.kh; ++ky) {
            if (!vy[y * g.kh + ky]) continue;
            for (int kx = 0; kx < g.kw; ++kx)
                if (vx[x * g.kw + kx]) a += (float)Ws[(ky * g.kw + kx) * g.C + c];
        }
        bool open;
        (void)bits_of(din, bi, (uint32_t)e, open);
        ce_put(din, (uint32_t)e, open, a * conv_scale * gs);
    }
    if (has_bias)
        for (int n = t; n < F; n += 1024) {
            bool open;
            (void)ce_bits(dbias, (uint32_t)n, open);
            ce_put(dbias, (uint32_t)n, open, bias_size / (float)F * gs);
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

// Launch plan of the few-channel kernels: which (kh, kw, C) are instantiated, LDS sizes, grid.
static bool smallc_shape(const hgq_conv_geom &g, int F) {
    const bool k33 = g.kh == 3 && g.kw == 3 && g.C >= 1 && g.C <= 4;
    const bool k55 = g.kh == 5 && g.kw == 5 && g.C == 1;
    return (k33 || k55) && F <= 32;
}
static size_t fwd_smallc_lds(const hgq_conv_geom &g) {
    const size_t XH = (size_t)(SC_TH - 1) * g.sy + (size_t)(g.kh - 1) * g.dly + 1, XW = (size_t)(SC_TW - 1) * g.sx + (size_t)(g.kw - 1) * g.dlx + 1;
    return XH * XW * g.C * sizeof(float);
}
static bool fwd_smallc_ok(const hgq_conv_geom &g, int F) {
    return smallc_shape(g, F) && fwd_smallc_lds(g) <= 48 * 1024 && (int64_t)g.B * g.H * g.W * g.C * 4 < (1ll << 31);
}
static size_t bwd_smallc_lds(const hgq_conv_geom &g, int F) {
    const size_t KC = (size_t)g.kh * g.kw * g.C, PH = SC_TH + g.kh - 1, PW = SC_TW + g.kw - 1;
    size_t zp = PH * PW * (F + 1), red = SC_TH * (KC + 1) * 32;
    if (red > zp) zp = red;
    return (((KC * F + 3) & ~(size_t)3) + zp + (PH + g.py) * (PW + g.kw - 1) * g.C) * sizeof(float);  // (input patch rows PW + kw - 1 pixels apart)
}
static bool bwd_smallc_ok(const hgq_conv_geom &g, int F) {
    return smallc_shape(g, F) && g.sy == 1 && g.sx == 1 && g.dly == 1 && g.dlx == 1 && g.py < g.kh && g.px < g.kw &&
           bwd_smallc_lds(g, F) <= 64 * 1024 && (int64_t)g.B * g.OH * g.OW * F * 4 < (1ll << 31) &&
           (int64_t)g.B * g.H * g.W * g.C * 4 < (1ll << 31);
}
static int bwd_smallc_grid(const hgq_conv_geom &g) {
    const int64_t tiles = (int64_t)g.B * ((g.H + SC_TH - 1) / SC_TH) * ((g.W + SC_TW - 1) / SC_TW);
    return persistent_grid(tiles, 3);
}
#define HGQ_SMALLC_DISPATCH(CALL) \
    do { \
        if (g->kh == 5) CALL(5, 5, 1); \
        else if (g->C == 1) CALL(3, 3, 1); \
        else if (g->C == 2) CALL(3, 3, 2); \
        else if (g->C == 3) CALL(3, 3, 3); \
        else CALL(3, 3, 4); \
    } while (0)

static inline bool aligned16(const void *p) { return ((uintptr_t)p & 15u) == 0; }

template <int MODE>
static void launch_igemm(bool vec, bool wide, dim3 grid, hipStream_t s, const float *src, const float *mask, const float *w,
                         const float *bias, float *out, const hgq_conv_geom &g, int F, int64_t rows, int K, int N, int act, int kchunk) {
#define HGQ_IGEMM(BFV) \
    do { \
        if (vec && wide) hipLaunchKernelGGL((igemm_vec_kernel<MODE, 2, BFV>), grid, dim3(256), 0, s, src, mask, w, bias, out, g, F, rows, K, N, act, kchunk); \
        else if (vec) hipLaunchKernelGGL((igemm_vec_kernel<MODE, 1, BFV>), grid, dim3(256), 0, s, src, mask, w, bias, out, g, F, rows, K, N, act, kchunk); \
        else if (wide) hipLaunchKernelGGL((igemm_kernel<MODE, 2, BFV>), grid, dim3(256), 0, s, src, mask, w, bias, out, g, F, rows, K, N, act, kchunk); \
        else hipLaunchKernelGGL((igemm_kernel<MODE, 1, BFV>), grid, dim3(256), 0, s, src, mask, w, bias, out, g, F, rows, K, N, act, kchunk); \
    } while (0)
    // the process-wide choice of matrix instruction (hgq_dense_use_bf16_parts)
    if (hgq_dense_use_bf16_parts(-1)) HGQ_IGEMM(true);
    else HGQ_IGEMM(false);
#undef HGQ_IGEMM
}

// A long contraction onto a handful of filters for few rows (the classifier behind a flattened feature map: 1024 x 3872
// onto 10): an implicit-GEMM tile would be mostly padding and needs a split along k plus a finishing launch.  Here a
// wavefront takes one row and a quarter of k - lanes along k, so the row is read in 256-byte pieces and a lane reads the
// F kernel entries of its k - adds up across its lanes, and the four quarters meet in LDS in a fixed order.  (Measured on
// 1024 x 3872 x 10: 14.8 us; two rows x eight parts of k per workgroup 17.1 us; the kernel matrix read as flat 256-byte
// pieces with the row entries gathered to match 24.4 us; implicit GEMM with split + finishing launch 12.2 + 8.3 us.)
#define SK_ROWS 4
#define SK_SPLIT 4
template <int F>
__global__ __launch_bounds__(1024) void skinny_fwd_kernel(const float *__restrict__ x, const float *__restrict__ w,
                                                          const float *__restrict__ bias, float *__restrict__ y, int64_t rows, int K,
                                                          int act) {
#pragma clang fp contract(fast)  // a contraction sum: multiply-adds may fuse, as in the other contraction kernels
    __shared__ float red[SK_ROWS][SK_SPLIT][F];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int r = wave / SK_SPLIT, sp = wave % SK_SPLIT;
    const int64_t row = (int64_t)blockIdx.x * SK_ROWS + r;
    const int kchunk = (K + SK_SPLIT * 64 - 1) / (SK_SPLIT * 64) * 64;
    const int k_begin = sp * kchunk, k_end = min(K, k_begin + kchunk);
    float acc[F];
#pragma unroll
    for (int n = 0; n < F; ++n) acc[n] = 0.f;
    if (row < rows) {
        const float *xr = x + row * K;
#pragma unroll 4
        for (int k = k_begin + lane; k < k_end; k += 64) {
            const float xv = xr[k];
            const float *wr = w + (int64_t)k * F;
#pragma unroll
            for (int n = 0; n < F; ++n) acc[n] += xv * wr[n];
        }
    }
#pragma unroll
    for (int n = 0; n < F; ++n) {
        float v = acc[n];
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
        if (lane == 0) red[r][sp][n] = v;
    }
    __syncthreads();
    if (threadIdx.x < SK_ROWS * F) {
        const int rr = threadIdx.x / F, n = threadIdx.x % F;
        const int64_t orow = (int64_t)blockIdx.x * SK_ROWS + rr;
        if (orow < rows) {
            float v = red[rr][0][n];
#pragma unroll
            for (int q = 1; q < SK_SPLIT; ++q) v += red[rr][q][n];
            if (bias) v += bias[n];
            if (act == HGQ_ACT_RELU) v = v > 0.f ? v : 0.f;
            y[orow * F + n] = v;
        }
    }
}

}  // namespace hgq

using namespace hgq;

extern "C" int64_t hgq_conv2d_fwd_workspace(const hgq_conv_geom *g, int F) {
    if (check_geom(g, F, "hgq_conv2d_fwd_workspace")) return -1;
    const int64_t rows = (int64_t)g->B * g->OH * g->OW;
    const int ks = fwd_ksplit(rows, g->kh * g->kw * g->C, F);
    return ks > 1 ? (int64_t)ks * rows * F : 0;
}

extern "C" int hgq_conv2d_fwd(const float *xq, const float *qw, const float *qb, float *y, float *workspace,
                              const hgq_conv_geom *g, int F, int act, void *stream) {
    int rc = check_geom(g, F, "hgq_conv2d_fwd");
    if (rc) return rc;
    if (act != HGQ_ACT_NONE && act != HGQ_ACT_RELU) return fail(HGQ_ERR_ARG, "hgq_conv2d_fwd: unknown activation %d", act);
    const int64_t rows = (int64_t)g->B * g->OH * g->OW;
    if (rows == 0) return HGQ_OK;
    if (!xq || !qw || !y) return fail(HGQ_ERR_ARG, "hgq_conv2d_fwd: null pointer");
    const int K = g->kh * g->kw * g->C;
    hipStream_t s = (hipStream_t)stream;
    const int ks = fwd_ksplit(rows, K, F);
    if (ks > 1 && !workspace) return fail(HGQ_ERR_ARG, "hgq_conv2d_fwd: this shape needs the workspace");
    int kchunk = (K + ks - 1) / ks;
    kchunk = (kchunk + CV_BK - 1) / CV_BK * CV_BK;
    const int nz = (K + kchunk - 1) / kchunk;
    float *dst = nz > 1 ? workspace : y;
    if (g->kh == 1 && g->kw == 1 && g->sy == 1 && g->sx == 1 && g->py == 0 && g->px == 0 && g->OH == g->H && g->OW == g->W && F <= 16 &&
        K >= 1024 && rows <= 16384) {
        const dim3 grid((unsigned)((rows + SK_ROWS - 1) / SK_ROWS));
#define HGQ_SKINNY(FV) \
    case FV: hipLaunchKernelGGL((skinny_fwd_kernel<FV>), grid, dim3(1024), 0, s, xq, qw, qb, y, rows, K, act); break
        switch (F) {
            HGQ_SKINNY(1); HGQ_SKINNY(2); HGQ_SKINNY(3); HGQ_SKINNY(4); HGQ_SKINNY(5); HGQ_SKINNY(6); HGQ_SKINNY(7); HGQ_SKINNY(8);
            HGQ_SKINNY(9); HGQ_SKINNY(10); HGQ_SKINNY(11); HGQ_SKINNY(12); HGQ_SKINNY(13); HGQ_SKINNY(14); HGQ_SKINNY(15); HGQ_SKINNY(16);
        }
#undef HGQ_SKINNY
        return check_launch("hgq_conv2d_fwd(few filters, long contraction)");
    }
    if (fwd_smallc_ok(*g, F)) {
        const int tiles_x = (g->OW + SC_TW - 1) / SC_TW, tiles_y = (g->OH + SC_TH - 1) / SC_TH;
        const dim3 grid((unsigned)persistent_grid((int64_t)g->B * tiles_x * tiles_y, 8));
        const size_t lds = fwd_smallc_lds(*g);
#define HGQ_FWD_SC(KH, KW, CC)                                                                                                                      \
    do {                                                                                                                                            \
        if (g->sy == 1 && g->sx == 1 && g->dly == 1 && g->dlx == 1)                                                                                 \
            hipLaunchKernelGGL((fwd_smallc_kernel<KH, KW, CC, true>), grid, dim3(256), lds, s, xq, qw, qb, y, *g, F, act, tiles_x, tiles_y, (float *)nullptr, (uint8_t *)nullptr); \
        else                                                                                                                                        \
            hipLaunchKernelGGL((fwd_smallc_kernel<KH, KW, CC, false>), grid, dim3(256), lds, s, xq, qw, qb, y, *g, F, act, tiles_x, tiles_y, (float *)nullptr, (uint8_t *)nullptr); \
    } while (0)
        HGQ_SMALLC_DISPATCH(HGQ_FWD_SC);
#undef HGQ_FWD_SC
        return check_launch("hgq_conv2d_fwd(few channels)");
    }
    if (nz == 1 && aligned16(xq) && conv_patch_ok(0, *g, F)) return conv_patch_launch(0, xq, nullptr, qw, qb, y, *g, F, act, s);
    const bool vec = g->C % 4 == 0 && aligned16(xq) && (int64_t)g->B * g->H * g->W * g->C * 4 < (1ll << 31);
    if (F <= 32) {
        const dim3 grid((unsigned)persistent_grid((rows + 127) / 128, vec ? 3 : 8), 1, (unsigned)nz);
        launch_igemm<0>(vec, false, grid, s, xq, nullptr, qw, qb, dst, *g, F, rows, K, F, act, kchunk);
    } else {
        const dim3 grid((unsigned)persistent_grid((rows + 63) / 64, vec ? 4 : 8), (unsigned)((F + 63) / 64), (unsigned)nz);
        launch_igemm<0>(vec, true, grid, s, xq, nullptr, qw, qb, dst, *g, F, rows, K, F, act, kchunk);
    }
    if ((rc = check_launch("hgq_conv2d_fwd"))) return rc;
    if (nz > 1) {
        const int64_t n = rows * F;
        hipLaunchKernelGGL(splitk_finish_kernel, dim3((unsigned)persistent_grid((n + 255) / 256, 8)), dim3(256), 0, s, workspace, nz, n, qb, F,
                           act, y);
        return check_launch("hgq_conv2d_fwd(finish)");
    }
    return HGQ_OK;
}

extern "C" int64_t hgq_conv2d_bwd_workspace(const hgq_conv_geom *g, int F) {
    if (check_geom(g, F, "hgq_conv2d_bwd_workspace")) return -1;
    const int64_t rows = (int64_t)g->B * g->OH * g->OW;
    const int K = g->kh * g->kw * g->C;
    const WgradCfg c = wgrad_cfg(K, F);
    int64_t slices = wgrad_splits(rows, c.n_kt * c.n_nt);
    if (bwd_smallc_ok(*g, F) && bwd_smallc_grid(*g) > slices) slices = bwd_smallc_grid(*g);
    if (conv_patch_wgrad_ok(*g, F) && conv_patch_wgrad_slices(*g, F) > slices) slices = conv_patch_wgrad_slices(*g, F);
    return slices * ((int64_t)K * F + F);
}

extern "C" int hgq_conv2d_maxpool_bwd_supported(const hgq_conv_geom *g, int F) {
    if (!g || F < 1) return 0;
    // the kernel's patch of output pixels starts at (8 ty + py - (kh - 1), 32 tx + px - (kw - 1)) and is (8 + kh - 1) x
    // (32 + kw - 1): whole windows when both offsets and both sizes are even
    return bwd_smallc_ok(*g, F) && F % 4 == 0 && g->OH >= 2 && g->OW >= 2 && (g->kh - 1 - g->py) % 2 == 0 &&
           (g->kw - 1 - g->px) % 2 == 0 && (g->kh & 1) && (g->kw & 1) && (int64_t)g->B * g->OH * g->OW > 0;
}

extern "C" int64_t hgq_conv2d_bwd_slice_count(const hgq_conv_geom *g, int F) {
    if (check_geom(g, F, "hgq_conv2d_bwd_slice_count")) return -1;
    const int64_t rows = (int64_t)g->B * g->OH * g->OW;
    if (rows == 0) return 1;
    if (bwd_smallc_ok(*g, F)) return bwd_smallc_grid(*g);
    if (conv_patch_wgrad_ok(*g, F)) return conv_patch_wgrad_slices(*g, F);
    const WgradCfg c = wgrad_cfg(g->kh * g->kw * g->C, F);
    return wgrad_splits(rows, c.n_kt * c.n_nt);
}

// reduce: the slices of the kernel / bias gradient are summed into dqw / dqb; otherwise they stay in `workspace`
// ([hgq_conv2d_bwd_slice_count][kh kw C F + F]) and dqw / dqb only say whether the gradient is wanted
// dyp: the gradient behind a 2 x 2 / stride 2 / unpadded maximum pooling of the output ([B, OH / 2, OW / 2, F]) instead of dy
static int conv2d_bwd_impl(const float *dy, const float *y, const float *xq, const float *qw, float *dxq, float *dqw, float *dqb,
                           float *workspace, const hgq_conv_geom *g, int F, int act, void *stream, bool reduce,
                           const float *dyp = nullptr, const uint8_t *code = nullptr) {
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
    if ((!dy && !dyp) || !qw || !xq) return fail(HGQ_ERR_ARG, "hgq_conv2d_bwd: null pointer");
    if ((act == HGQ_ACT_RELU || dyp) && !y && !code) return fail(HGQ_ERR_ARG, "hgq_conv2d_bwd: relu / pooling need the forward output");
    const float *mask = (act == HGQ_ACT_RELU || dyp) ? y : nullptr;
    if (dyp && !(hgq_conv2d_maxpool_bwd_supported(g, F) && aligned16(dyp) && (code ? ((uintptr_t)code & 3u) == 0 : aligned16(y))))
        return fail(HGQ_ERR_UNSUPPORTED, "hgq_conv2d_maxpool_bwd: shape or alignment not supported (ask hgq_conv2d_maxpool_bwd_supported)");
    if (bwd_smallc_ok(*g, F)) {
        const bool want_w = dqw || dqb;
        if (want_w && !workspace) return fail(HGQ_ERR_ARG, "hgq_conv2d_bwd: null workspace");
        const int tiles_x = (g->W + SC_TW - 1) / SC_TW, tiles_y = (g->H + SC_TH - 1) / SC_TH;
        const int grid = bwd_smallc_grid(*g);
        const size_t lds = bwd_smallc_lds(*g, F);
        const int vec = F % 4 == 0 && aligned16(dy) && (!mask || aligned16(mask));
#define HGQ_BWD_SC(KH, KW, CC) \
    hipLaunchKernelGGL((bwd_smallc_kernel<KH, KW, CC>), dim3((unsigned)grid), dim3(256), lds, s, dy, mask, xq, qw, dxq, want_w ? workspace : (float *)nullptr, *g, F, tiles_x, tiles_y, vec, dyp, g->OH / 2, g->OW / 2, act == HGQ_ACT_RELU, code)
        HGQ_SMALLC_DISPATCH(HGQ_BWD_SC);
#undef HGQ_BWD_SC
        if ((rc = check_launch("hgq_conv2d_bwd(few channels)"))) return rc;
        if (want_w && reduce) return reduce_parts(workspace, grid, KF + F, dqw, KF, dqb, (int64_t)F, nullptr, 0, s);
        return HGQ_OK;
    }
    if (dxq) {
        const int Kt = g->kh * g->kw * F;  // contraction length of the data gradient
        const size_t patch_lds = ((size_t)g->kh * g->kw * g->C * F + (size_t)(DP_TH + g->kh - 1) * (DP_TW + g->kw - 1) * (F + 1)) * sizeof(float);
        if (g->C <= 4 && g->sy == 1 && g->sx == 1 && g->dly == 1 && g->dlx == 1 && patch_lds <= 64 * 1024) {
            const int tiles_x = (g->W + DP_TW - 1) / DP_TW, tiles_y = (g->H + DP_TH - 1) / DP_TH;
            const dim3 grid((unsigned)persistent_grid((int64_t)g->B * tiles_x * tiles_y, 8));
            hipLaunchKernelGGL(dgrad_patch_kernel, grid, dim3(256), patch_lds, s, dy, mask, qw, dxq, *g, F, tiles_x, tiles_y);
        } else if (g->C <= 4 && (int64_t)g->kh * g->kw * g->C * F <= DG_MAXW && F <= 64) {
            const int fp = F <= 16 ? 16 : (F <= 32 ? 32 : 64);
            const dim3 grid((unsigned)persistent_grid((in_rows * fp + 255) / 256, 16));
            const size_t lds = (size_t)g->kh * g->kw * g->C * F * sizeof(float);
            const bool k33 = g->kh == 3 && g->kw == 3;
#define HGQ_DG(FPV) \
    do { \
        if (k33) hipLaunchKernelGGL((dgrad_smallc_kernel<FPV, 3, 3>), grid, dim3(256), lds, s, dy, mask, qw, dxq, *g, F, in_rows); \
        else hipLaunchKernelGGL((dgrad_smallc_kernel<FPV, 0, 0>), grid, dim3(256), lds, s, dy, mask, qw, dxq, *g, F, in_rows); \
    } while (0)
            if (fp == 16) HGQ_DG(16);
            else if (fp == 32) HGQ_DG(32);
            else HGQ_DG(64);
#undef HGQ_DG
        } else if (aligned16(dy) && (!mask || aligned16(mask)) && conv_patch_ok(1, *g, F)) {
            if ((rc = conv_patch_launch(1, dy, mask, qw, nullptr, dxq, *g, F, act, s))) return rc;
        } else {
            const bool vec = F % 4 == 0 && aligned16(dy) && (!mask || aligned16(mask)) && rows * F * 4 < (1ll << 31);
            if (g->C <= 32) {
                const dim3 grid((unsigned)persistent_grid((in_rows + 127) / 128, vec ? 3 : 8), 1);
                launch_igemm<1>(vec, false, grid, s, dy, mask, qw, nullptr, dxq, *g, F, in_rows, Kt, g->C, act, Kt);
            } else {
                const dim3 grid((unsigned)persistent_grid((in_rows + 63) / 64, vec ? 4 : 8), (unsigned)((g->C + 63) / 64));
                launch_igemm<1>(vec, true, grid, s, dy, mask, qw, nullptr, dxq, *g, F, in_rows, Kt, g->C, act, Kt);
            }
        }
        if ((rc = check_launch("hgq_conv2d_bwd(data)"))) return rc;
    }
    if (dqw || dqb) {
        if (!workspace) return fail(HGQ_ERR_ARG, "hgq_conv2d_bwd: null workspace");
        const int64_t M = KF + F;
        // small feature maps: both operands of a band of an image staged once in LDS (the slice count is a function of the
        // shape alone, so operands that are not 16-byte aligned keep it and go through the gathered kernels below)
        const bool patch_shape = conv_patch_wgrad_ok(*g, F);
        const int64_t patch_slices = patch_shape ? conv_patch_wgrad_slices(*g, F) : 0;
        if (patch_shape && aligned16(xq) && aligned16(dy) && (!mask || aligned16(mask))) {
            if ((rc = conv_patch_wgrad_launch(xq, dy, mask, workspace, *g, F, act, s))) return rc;
            if (reduce && (rc = reduce_parts(workspace, (int)patch_slices, M, dqw, KF, dqb, (int64_t)F, nullptr, 0, s))) return rc;
            return HGQ_OK;
        }
        const WgradCfg c = wgrad_cfg(K, F);
        int64_t splits = wgrad_splits(rows, c.n_kt * c.n_nt);
        if (patch_shape) {
            if (splits > patch_slices) splits = patch_slices;
            if (splits < patch_slices && !reduce && (rc = fill_f32(workspace + splits * M, 0.f, (patch_slices - splits) * M, s))) return rc;
        }
        int64_t chunk = (rows + splits - 1) / splits;
        chunk = (chunk + 127) / 128 * 128;
        const dim3 grid((unsigned)(c.n_kt * c.n_nt), (unsigned)splits);
        const bool src_vec = g->C % 4 == 0 && aligned16(xq) && rows * F * 4 < (1ll << 31) && in_rows * g->C * 4 < (1ll << 31);
        const bool z_vec = F % 4 == 0 && aligned16(dy) && (!mask || aligned16(mask));
        const bool vec = src_vec && z_vec;
        const bool bf = hgq_dense_use_bf16_parts(-1) != 0;
#define HGQ_WGRAD(WK, WN, WS) \
    do { \
        if (src_vec && !z_vec && bf) hipLaunchKernelGGL((wgrad_vec_kernel<WK, WN, WS, true, true>), grid, dim3(256), 0, s, xq, dy, mask, workspace, *g, F, rows, K, chunk, act, c.n_kt); \
        else if (src_vec && !z_vec) hipLaunchKernelGGL((wgrad_vec_kernel<WK, WN, WS, false, true>), grid, dim3(256), 0, s, xq, dy, mask, workspace, *g, F, rows, K, chunk, act, c.n_kt); \
        else if (vec && bf) hipLaunchKernelGGL((wgrad_vec_kernel<WK, WN, WS, true>), grid, dim3(256), 0, s, xq, dy, mask, workspace, *g, F, rows, K, chunk, act, c.n_kt); \
        else if (vec) hipLaunchKernelGGL((wgrad_vec_kernel<WK, WN, WS>), grid, dim3(256), 0, s, xq, dy, mask, workspace, *g, F, rows, K, chunk, act, c.n_kt); \
        else if (bf) hipLaunchKernelGGL((wgrad_kernel<WK, WN, WS, true>), grid, dim3(256), 0, s, xq, dy, mask, workspace, *g, F, rows, K, chunk, act, c.n_kt); \
        else hipLaunchKernelGGL((wgrad_kernel<WK, WN, WS>), grid, dim3(256), 0, s, xq, dy, mask, workspace, *g, F, rows, K, chunk, act, c.n_kt); \
    } while (0)
        if (c.wk == 2 && c.wn == 2) HGQ_WGRAD(2, 2, 1);
        else if (c.wk == 1) HGQ_WGRAD(1, 1, 4);
        else if (c.wk == 2) HGQ_WGRAD(2, 1, 2);
        else HGQ_WGRAD(4, 1, 1);
#undef HGQ_WGRAD
        if ((rc = check_launch("hgq_conv2d_bwd(weights)"))) return rc;
        if (reduce && (rc = reduce_parts(workspace, (int)splits, M, dqw, KF, dqb, (int64_t)F, nullptr, 0, s))) return rc;
    }
    return HGQ_OK;
}

extern "C" int hgq_conv2d_bwd(const float *dy, const float *y, const float *xq, const float *qw, float *dxq, float *dqw,
                              float *dqb, float *workspace, const hgq_conv_geom *g, int F, int act, void *stream) {
    return conv2d_bwd_impl(dy, y, xq, qw, dxq, dqw, dqb, workspace, g, F, act, stream, true);
}

extern "C" int hgq_conv2d_bwd_slices(const float *dy, const float *y, const float *xq, const float *qw, float *dxq, float *workspace,
                                     const hgq_conv_geom *g, int F, int act, void *stream) {
    if (!workspace) return fail(HGQ_ERR_ARG, "hgq_conv2d_bwd_slices: null workspace");
    if (g && (int64_t)g->B * g->OH * g->OW == 0) {  // nothing to add up: one slice of zeros
        const int rc = check_geom(g, F, "hgq_conv2d_bwd_slices");
        return rc ? rc : fill_f32(workspace, 0.f, hgq_conv2d_bwd_slice_count(g, F) * ((int64_t)g->kh * g->kw * g->C * F + F), (hipStream_t)stream);
    }
    // the kernels only test the gradient pointers for "is it wanted": any non-null value stands for it
    return conv2d_bwd_impl(dy, y, xq, qw, dxq, workspace, workspace, workspace, g, F, act, stream, false);
}

static int conv2d_maxpool_fwd_impl(const float *xq, const float *qw, const float *qb, float *y, float *yp, uint8_t *code,
                                   const hgq_conv_geom *g, int F, int act, void *stream, const char *who) {
    int rc = check_geom(g, F, who);
    if (rc) return rc;
    if (act != HGQ_ACT_NONE && act != HGQ_ACT_RELU) return fail(HGQ_ERR_ARG, "%s: unknown activation %d", who, act);
    if (!hgq_conv2d_maxpool_bwd_supported(g, F) || !fwd_smallc_ok(*g, F))
        return fail(HGQ_ERR_UNSUPPORTED, "%s: shape not supported (ask hgq_conv2d_maxpool_bwd_supported)", who);
    if (!xq || !qw || (!y && !code) || !yp) return fail(HGQ_ERR_ARG, "%s: null pointer", who);
    hipStream_t s = (hipStream_t)stream;
    const int tiles_x = (g->OW + SC_TW - 1) / SC_TW, tiles_y = (g->OH + SC_TH - 1) / SC_TH;
    const dim3 grid((unsigned)persistent_grid((int64_t)g->B * tiles_x * tiles_y, 8));
    const size_t lds = fwd_smallc_lds(*g);
    // (hgq_conv2d_maxpool_bwd_supported holds only for unit stride and dilation)
#define HGQ_FWD_SC(KH, KW, CC) hipLaunchKernelGGL((fwd_smallc_kernel<KH, KW, CC, true>), grid, dim3(256), lds, s, xq, qw, qb, y, *g, F, act, tiles_x, tiles_y, yp, code)
    HGQ_SMALLC_DISPATCH(HGQ_FWD_SC);
#undef HGQ_FWD_SC
    return check_launch(who);
}

extern "C" int hgq_conv2d_maxpool_fwd(const float *xq, const float *qw, const float *qb, float *y, float *yp, const hgq_conv_geom *g,
                                      int F, int act, void *stream) {
    if (!y) return fail(HGQ_ERR_ARG, "hgq_conv2d_maxpool_fwd: null pointer");
    return conv2d_maxpool_fwd_impl(xq, qw, qb, y, yp, nullptr, g, F, act, stream, "hgq_conv2d_maxpool_fwd");
}

extern "C" int hgq_conv2d_maxpool_fwd_coded(const float *xq, const float *qw, const float *qb, float *yp, uint8_t *code,
                                            const hgq_conv_geom *g, int F, int act, void *stream) {
    if (!code) return fail(HGQ_ERR_ARG, "hgq_conv2d_maxpool_fwd_coded: null pointer");
    return conv2d_maxpool_fwd_impl(xq, qw, qb, nullptr, yp, code, g, F, act, stream, "hgq_conv2d_maxpool_fwd_coded");
}

extern "C" int hgq_conv2d_maxpool_bwd(const float *dyp, const float *y, const float *xq, const float *qw, float *dxq, float *dqw,
                                      float *dqb, float *workspace, const hgq_conv_geom *g, int F, int act, int reduce, void *stream) {
    if (!dyp) return fail(HGQ_ERR_ARG, "hgq_conv2d_maxpool_bwd: null pointer");
    if (!reduce && !workspace) return fail(HGQ_ERR_ARG, "hgq_conv2d_maxpool_bwd: null workspace");
    if (reduce) return conv2d_bwd_impl(nullptr, y, xq, qw, dxq, dqw, dqb, workspace, g, F, act, stream, true, dyp);
    return conv2d_bwd_impl(nullptr, y, xq, qw, dxq, workspace, workspace, workspace, g, F, act, stream, false, dyp);
}

extern "C" int hgq_conv2d_maxpool_bwd_coded(const float *dyp, const uint8_t *code, const float *xq, const float *qw, float *dxq,
                                            float *dqw, float *dqb, float *workspace, const hgq_conv_geom *g, int F, int act, int reduce,
                                            void *stream) {
    if (!dyp || !code) return fail(HGQ_ERR_ARG, "hgq_conv2d_maxpool_bwd_coded: null pointer");
    if (!reduce && !workspace) return fail(HGQ_ERR_ARG, "hgq_conv2d_maxpool_bwd_coded: null workspace");
    if (reduce) return conv2d_bwd_impl(nullptr, nullptr, xq, qw, dxq, dqw, dqb, workspace, g, F, act, stream, true, dyp, code);
    return conv2d_bwd_impl(nullptr, nullptr, xq, qw, dxq, workspace, workspace, workspace, g, F, act, stream, false, dyp, code);
}

extern "C" int hgq_conv2d_ebops(const float *bits_in, const float *bits_ker, const hgq_conv_geom *g, int F, float *total,
                                float *g_bits_in, float *g_bits_ker, void *stream) {
    int rc = check_geom(g, F, "hgq_conv2d_ebops");
    if (rc) return rc;
    if (!bits_in || !bits_ker || !total) return fail(HGQ_ERR_ARG, "hgq_conv2d_ebops: null pointer");
    if ((int64_t)g->kh * g->kw * g->C > CE_MAX || (int64_t)g->kh * g->W * g->C > CE_MAXR || (int64_t)g->H * g->kh > CE_MAXV ||
        (int64_t)g->W * g->kw > CE_MAXV)
        return fail(HGQ_ERR_UNSUPPORTED, "hgq_conv2d_ebops: needs kh * kw * C <= %d, kh * W * C <= %d, H * kh and W * kw <= %d", CE_MAX,
                    CE_MAXR, CE_MAXV);
    if ((int64_t)g->kh * g->kw * g->C * g->OH * g->OW >= (1ll << 31) || (int64_t)g->kh * g->kw * g->C * F >= (1ll << 21) ||
        (int64_t)g->H * g->W * g->C >= (1ll << 21))
        return fail(HGQ_ERR_UNSUPPORTED, "hgq_conv2d_ebops: needs kh * kw * C * F and H * W * C below 2**21 (flat sweeps of one workgroup)");
    hipLaunchKernelGGL(conv_ebops_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, bits_in, bits_ker, *g, F, total, g_bits_in, g_bits_ker);
    return check_launch("hgq_conv2d_ebops");
}

extern "C" int hgq_conv2d_ebops_q(const hgq_bits_desc *bits_in, const hgq_bits_desc *bits_ker, const hgq_bits_desc *bits_bias,
                                  const hgq_conv_geom *g, int F, float conv_scale, float bias_size, float ebops_factor, const float *beta,
                                  uint32_t *ebops_u32, float *loss_term, void *stream) {
    int rc = check_geom(g, F, "hgq_conv2d_ebops_q");
    if (rc) return rc;
    if (!bits_in || !bits_ker || !beta || !loss_term) return fail(HGQ_ERR_ARG, "hgq_conv2d_ebops_q: null pointer");
    if ((int64_t)g->kh * g->kw * g->C > CE_MAX || (int64_t)g->kh * g->W * g->C > CE_MAXR || (int64_t)g->H * g->kh > CE_MAXV ||
        (int64_t)g->W * g->kw > CE_MAXV)
        return fail(HGQ_ERR_UNSUPPORTED, "hgq_conv2d_ebops_q: needs kh * kw * C <= %d, kh * W * C <= %d, H * kh and W * kw <= %d", CE_MAX,
                    CE_MAXR, CE_MAXV);
    const int64_t n_in = (int64_t)g->H * g->W * g->C, n_w = (int64_t)g->kh * g->kw * g->C * F;
    if ((int64_t)g->kh * g->kw * g->C * g->OH * g->OW >= (1ll << 31) || n_w >= (1ll << 21) || n_in >= (1ll << 21))
        return fail(HGQ_ERR_UNSUPPORTED, "hgq_conv2d_ebops_q: needs kh * kw * C * F and H * W * C below 2**21 (flat sweeps of one workgroup)");
    const hgq_bits_desc *ds[3] = {bits_in, bits_ker, bits_bias};
    const int64_t cells[3] = {n_in, n_w, (int64_t)F};
    for (int t = 0; t < 3; ++t) {
        if (!ds[t]) continue;
        if (ds[t]->size != cells[t] || ds[t]->inner != 1)
            return fail(HGQ_ERR_UNSUPPORTED, "hgq_conv2d_ebops_q: operand %d must have one bit-width entry per cell", t);
        if (!ds[t]->fb || !ds[t]->g_fb || (!ds[t]->kbi && (!ds[t]->i || !ds[t]->g_i)) || (ds[t]->add_mode && !ds[t]->k))
            return fail(HGQ_ERR_ARG, "hgq_conv2d_ebops_q: null pointer in operand %d", t);
    }
    hgq_bits_desc none = *bits_ker;
    const size_t staged_bytes = (size_t)((n_in + 15) & ~(int64_t)15) + (size_t)n_w;
    if (staged_bytes <= 60 * 1024) {
        static bool allowed = false;  // (static + dynamic LDS of this kernel pass 64 KiB)
        if (!allowed) {
            if (hipFuncSetAttribute((const void *)conv_ebops_q_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, 60 * 1024) != hipSuccess)
                return fail(HGQ_ERR_LAUNCH, "hgq_conv2d_ebops_q: cannot raise the dynamic LDS limit");
            allowed = true;
        }
        hipLaunchKernelGGL(conv_ebops_q_kernel<true>, dim3(1), dim3(1024), staged_bytes, (hipStream_t)stream, *bits_in, *bits_ker,
                           bits_bias ? *bits_bias : none, bits_bias ? 1 : 0, *g, F, conv_scale, bias_size, ebops_factor, beta, ebops_u32, loss_term);
    } else {
        hipLaunchKernelGGL(conv_ebops_q_kernel<false>, dim3(1), dim3(1024), 0, (hipStream_t)stream, *bits_in, *bits_ker,
                           bits_bias ? *bits_bias : none, bits_bias ? 1 : 0, *g, F, conv_scale, bias_size, ebops_factor, beta, ebops_u32, loss_term);
    }
    return check_launch("hgq_conv2d_ebops_q");
}
