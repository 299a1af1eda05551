// 2-D max / average pooling on channels-last tensors, forward and backward.
//
// One thread per (pixel, channel group): adjacent threads take adjacent channels, so every window
// read is coalesced along the channel axis (128-bit when C is a multiple of 4).  The backward for
// overlapping windows is gather-style - a thread owns an INPUT element and visits the windows that
// contain it - and the one for disjoint windows owns a stride tile; neither uses atomics and
// uncovered border pixels get an exact zero.  Max pooling routes the gradient
// to the first maximum of a window in row-major order (what the library max-pool the reference
// sits on does), recomputed from the forward input.
#include "hgq_device.h"
#include "hgq_host.h"

namespace hgq {

struct PoolGeom {
    int B, H, W, C, ph, pw, sy, sx, py, px, OH, OW;
};

template <int VEC>
struct PV {
    float v[VEC];
};
template <int VEC>
__device__ __forceinline__ PV<VEC> pload(const float *p) {
    PV<VEC> r;
    if (VEC == 4) {
        const float4 t = *(const float4 *)p;
        r.v[0] = t.x, r.v[1 % VEC] = t.y, r.v[2 % VEC] = t.z, r.v[3 % VEC] = t.w;
    } else {
        r.v[0] = *p;
    }
    return r;
}
template <int VEC>
__device__ __forceinline__ void pstore(float *p, const PV<VEC> &r) {
    if (VEC == 4) *(float4 *)p = make_float4(r.v[0], r.v[1 % VEC], r.v[2 % VEC], r.v[3 % VEC]);
    else *p = r.v[0];
}

// MAX: y = max over the window (padding never wins); else the mean over the in-range part of the
// window (Keras / TensorFlow 'same' average pooling excludes the padding from the count).
template <int VEC, bool MAX>
__global__ __launch_bounds__(256) void pool2d_fwd_kernel(const float *__restrict__ x, float *__restrict__ y, PoolGeom g) {
    const int cg = g.C / VEC;
    const int64_t n = (int64_t)g.B * g.OH * g.OW * cg;
    for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < n; t += (int64_t)gridDim.x * 256) {
        const int c = (int)(t % cg) * VEC;
        int64_t pix = t / cg;
        const int ox = (int)(pix % g.OW);
        pix /= g.OW;
        const int oy = (int)(pix % g.OH), b = (int)(pix / g.OH);
        PV<VEC> acc;
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc.v[e] = MAX ? -INFINITY : 0.f;
        int cnt = 0;
        for (int wy = 0; wy < g.ph; ++wy) {
            const int iy = oy * g.sy - g.py + wy;
            if ((unsigned)iy >= (unsigned)g.H) continue;
            for (int wx = 0; wx < g.pw; ++wx) {
                const int ix = ox * g.sx - g.px + wx;
                if ((unsigned)ix >= (unsigned)g.W) continue;
                const PV<VEC> v = pload<VEC>(x + (((int64_t)b * g.H + iy) * g.W + ix) * g.C + c);
#pragma unroll
                for (int e = 0; e < VEC; ++e) acc.v[e] = MAX ? fmaxf(acc.v[e], v.v[e]) : acc.v[e] + v.v[e];
                ++cnt;
            }
        }
        if (!MAX) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) acc.v[e] = acc.v[e] / (float)cnt;
        }
        pstore<VEC>(y + t * VEC, acc);
    }
}

template <int VEC, bool MAX>
__global__ __launch_bounds__(256) void pool2d_bwd_kernel(const float *__restrict__ dy, const float *__restrict__ x,
                                                         float *__restrict__ dx, PoolGeom g) {
    const int cg = g.C / VEC;
    const int64_t n = (int64_t)g.B * g.H * g.W * cg;
    for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < n; t += (int64_t)gridDim.x * 256) {
        const int c = (int)(t % cg) * VEC;
        int64_t pix = t / cg;
        const int ix = (int)(pix % g.W);
        pix /= g.W;
        const int iy = (int)(pix % g.H), b = (int)(pix / g.H);
        PV<VEC> mine;
        if (MAX) mine = pload<VEC>(x + t * VEC);
        PV<VEC> acc;
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc.v[e] = 0.f;
        // windows (oy, ox) that contain (iy, ix): oy * sy - py <= iy < oy * sy - py + ph
        const int oy_hi = min(g.OH - 1, (iy + g.py) / g.sy), ox_hi = min(g.OW - 1, (ix + g.px) / g.sx);
        const int oy_lo = max(0, (iy + g.py - g.ph + g.sy) / g.sy), ox_lo = max(0, (ix + g.px - g.pw + g.sx) / g.sx);
        for (int oy = oy_lo; oy <= oy_hi; ++oy) {
            for (int ox = ox_lo; ox <= ox_hi; ++ox) {
                const PV<VEC> gv = pload<VEC>(dy + (((int64_t)b * g.OH + oy) * g.OW + ox) * g.C + c);
                if (!MAX) {
                    const int y0 = max(0, oy * g.sy - g.py), y1 = min(g.H, oy * g.sy - g.py + g.ph);
                    const int x0 = max(0, ox * g.sx - g.px), x1 = min(g.W, ox * g.sx - g.px + g.pw);
                    const float inv = 1.0f / (float)((y1 - y0) * (x1 - x0));
#pragma unroll
                    for (int e = 0; e < VEC; ++e) acc.v[e] += gv.v[e] * inv;
                    continue;
                }
                // this element takes the window's gradient iff it is the first maximum in row-major order
                bool win[VEC];
#pragma unroll
                for (int e = 0; e < VEC; ++e) win[e] = true;
                for (int wy = 0; wy < g.ph; ++wy) {
                    const int qy = oy * g.sy - g.py + wy;
                    if ((unsigned)qy >= (unsigned)g.H) continue;
                    for (int wx = 0; wx < g.pw; ++wx) {
                        const int qx = ox * g.sx - g.px + wx;
                        if ((unsigned)qx >= (unsigned)g.W || (qy == iy && qx == ix)) continue;
                        const PV<VEC> o = pload<VEC>(x + (((int64_t)b * g.H + qy) * g.W + qx) * g.C + c);
                        const bool before = qy < iy || (qy == iy && qx < ix);
#pragma unroll
                        for (int e = 0; e < VEC; ++e)
                            if (before ? o.v[e] >= mine.v[e] : o.v[e] > mine.v[e]) win[e] = false;
                    }
                }
#pragma unroll
                for (int e = 0; e < VEC; ++e)
                    if (win[e]) acc.v[e] += gv.v[e];
            }
        }
        pstore<VEC>(dx + t * VEC, acc);
    }
}

// Backward for disjoint windows (stride >= pool size, the usual case): a thread owns one stride
// tile of the INPUT - the window in its corner plus the pixels no window covers - so x and dy are
// read once and dx is written once.
template <int VEC, bool MAX>
__global__ __launch_bounds__(256) void pool2d_bwd_tiles_kernel(const float *__restrict__ dy, const float *__restrict__ x,
                                                               float *__restrict__ dx, PoolGeom g, int TH, int TW) {
    const int cg = g.C / VEC;
    const int64_t n = (int64_t)g.B * TH * TW * cg;
    for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < n; t += (int64_t)gridDim.x * 256) {
        const int c = (int)(t % cg) * VEC;
        int64_t r = t / cg;
        const int tx = (int)(r % TW);
        r /= TW;
        const int ty = (int)(r % TH), b = (int)(r / TH);
        const bool valid = ty < g.OH && tx < g.OW;
        const int y0 = ty * g.sy - g.py, x0 = tx * g.sx - g.px;
        PV<VEC> gv;
        int first[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) gv.v[e] = 0.f, first[e] = -1;
        if (valid) {
            gv = pload<VEC>(dy + (((int64_t)b * g.OH + ty) * g.OW + tx) * g.C + c);
            if (MAX) {
                float best[VEC];
#pragma unroll
                for (int e = 0; e < VEC; ++e) best[e] = -INFINITY;
                for (int wy = 0; wy < g.ph; ++wy) {
                    const int iy = y0 + wy;
                    if ((unsigned)iy >= (unsigned)g.H) continue;
                    for (int wx = 0; wx < g.pw; ++wx) {
                        const int ix = x0 + wx;
                        if ((unsigned)ix >= (unsigned)g.W) continue;
                        const PV<VEC> v = pload<VEC>(x + (((int64_t)b * g.H + iy) * g.W + ix) * g.C + c);
#pragma unroll
                        for (int e = 0; e < VEC; ++e)
                            if (v.v[e] > best[e] || first[e] < 0) best[e] = v.v[e], first[e] = wy * g.pw + wx;
                    }
                }
            } else {
                const int ya = max(0, y0), yb = min(g.H, y0 + g.ph), xa = max(0, x0), xb = min(g.W, x0 + g.pw);
                const float inv = 1.0f / (float)((yb - ya) * (xb - xa));
#pragma unroll
                for (int e = 0; e < VEC; ++e) gv.v[e] *= inv;
            }
        }
        for (int ry = 0; ry < g.sy; ++ry) {
            const int iy = y0 + ry;
            if ((unsigned)iy >= (unsigned)g.H) continue;
            for (int rx = 0; rx < g.sx; ++rx) {
                const int ix = x0 + rx;
                if ((unsigned)ix >= (unsigned)g.W) continue;
                const bool in_win = valid && ry < g.ph && rx < g.pw;
                PV<VEC> o;
#pragma unroll
                for (int e = 0; e < VEC; ++e) o.v[e] = in_win && (!MAX || first[e] == ry * g.pw + rx) ? gv.v[e] : 0.f;
                pstore<VEC>(dx + (((int64_t)b * g.H + iy) * g.W + ix) * g.C + c, o);
            }
        }
    }
}

static int check_pool(const int *d, PoolGeom &g, const char *who) {
    g.B = d[0], g.H = d[1], g.W = d[2], g.C = d[3], g.ph = d[4], g.pw = d[5], g.sy = d[6], g.sx = d[7], g.py = d[8], g.px = d[9],
    g.OH = d[10], g.OW = d[11];
    if (g.B < 0 || g.H < 1 || g.W < 1 || g.C < 1 || g.ph < 1 || g.pw < 1 || g.sy < 1 || g.sx < 1 || g.py < 0 || g.px < 0 || g.OH < 1 ||
        g.OW < 1 || g.py >= g.ph || g.px >= g.pw)
        return fail(HGQ_ERR_ARG, "%s: bad geometry", who);
    return HGQ_OK;
}

// ------------------------------------------------------------------------------------------
// mean over the middle axis of [B, P, N] (global average pooling of a channels-last tensor; the mean over the
// particles of the per-particle configuration)
// ------------------------------------------------------------------------------------------
// One workgroup per batch element: thread (c, ty) owns VEC columns and walks rows ty, ty + TY, ... with eight loads
// in flight; the TY partial sums of a column group are added in row-group order through LDS.
template <int VEC>
__global__ __launch_bounds__(256) void mean_mid_fwd_kernel(const float *__restrict__ x, float *__restrict__ y, int P, int N, int TX,
                                                           float inv) {
    __shared__ float red[256 * VEC];
    const int cg = N / VEC, TY = 256 / TX, c0 = threadIdx.x % TX, ty = threadIdx.x / TX;
    const int64_t b = blockIdx.x;
    const __amdgpu_buffer_rsrc_t rs = buf_rsrc(x + b * P * N, (int64_t)P * N * 4);
    for (int cb = 0; cb < cg; cb += TX) {
        const int c = cb + c0;
        const bool on = c < cg;
        float s[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) s[e] = 0.f;
        for (int p0 = ty; p0 < P; p0 += 8 * TY) {
            float v[8][VEC];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int p = p0 + u * TY;
                const uint32_t off = (on && p < P) ? (uint32_t)(p * N + c * VEC) * 4u : BUF_OOB;
                if (VEC == 4) {
                    const f32x4_t t = buf_ld4(rs, off);
                    v[u][0] = t[0], v[u][1 % VEC] = t[1], v[u][2 % VEC] = t[2], v[u][3 % VEC] = t[3];
                } else {
                    v[u][0] = buf_ld1(rs, off);
                }
            }
#pragma unroll
            for (int u = 0; u < 8; ++u)
#pragma unroll
                for (int e = 0; e < VEC; ++e) s[e] += v[u][e];
        }
        __syncthreads();  // the previous column block's sums have been read
#pragma unroll
        for (int e = 0; e < VEC; ++e) red[threadIdx.x * VEC + e] = s[e];
        __syncthreads();
        if (ty == 0 && on) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                float t = 0.f;
                for (int g = 0; g < TY; ++g) t += red[(g * TX + c0) * VEC + e];
                y[b * N + c * VEC + e] = t * inv;
            }
        }
    }
}

template <int VEC>
__global__ __launch_bounds__(256) void mean_mid_bwd_kernel(const float *__restrict__ dy, float *__restrict__ dx, int P, int N, int TX,
                                                           float inv) {
    const int cg = N / VEC, TY = 256 / TX, c0 = threadIdx.x % TX, ty = threadIdx.x / TX;
    const int64_t b = blockIdx.x;
    const __amdgpu_buffer_rsrc_t rs = buf_rsrc(dx + b * P * N, (int64_t)P * N * 4);
    for (int cb = 0; cb < cg; cb += TX) {
        const int c = cb + c0;
        if (c >= cg) continue;
        float g[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) g[e] = dy[b * N + c * VEC + e] * inv;
        for (int p = ty; p < P; p += TY) {
            const uint32_t off = (uint32_t)(p * N + c * VEC) * 4u;
            if (VEC == 4) {
                f32x4_t t;
                t[0] = g[0], t[1] = g[1 % VEC], t[2] = g[2 % VEC], t[3] = g[3 % VEC];
                buf_st4(rs, off, t);
            } else {
                buf_st1(rs, off, g[0]);
            }
        }
    }
}

}  // namespace hgq

using namespace hgq;

extern "C" int hgq_mean_mid_fwd(const float *x, float *y, int64_t B, int64_t P, int64_t N, void *stream) {
    if (B < 0 || P < 1 || N < 1) return fail(HGQ_ERR_ARG, "hgq_mean_mid_fwd: bad sizes");
    if (B == 0) return HGQ_OK;
    if (!x || !y) return fail(HGQ_ERR_ARG, "hgq_mean_mid_fwd: null pointer");
    if (P * N * 4 >= (1ll << 31) || B >= (1ll << 31)) return fail(HGQ_ERR_UNSUPPORTED, "hgq_mean_mid_fwd: one batch element must stay below 2 GiB");
    const bool vec = N % 4 == 0 && ((uintptr_t)x & 15u) == 0;
    const int64_t cg = vec ? N / 4 : N;
    int TX = 1;
    while (TX < cg && TX < 256) TX <<= 1;
    const float inv = 1.0f / (float)P;
    if (vec) hipLaunchKernelGGL(mean_mid_fwd_kernel<4>, dim3((unsigned)B), dim3(256), 0, (hipStream_t)stream, x, y, (int)P, (int)N, TX, inv);
    else hipLaunchKernelGGL(mean_mid_fwd_kernel<1>, dim3((unsigned)B), dim3(256), 0, (hipStream_t)stream, x, y, (int)P, (int)N, TX, inv);
    return check_launch("hgq_mean_mid_fwd");
}

extern "C" int hgq_mean_mid_bwd(const float *dy, float *dx, int64_t B, int64_t P, int64_t N, void *stream) {
    if (B < 0 || P < 1 || N < 1) return fail(HGQ_ERR_ARG, "hgq_mean_mid_bwd: bad sizes");
    if (B == 0) return HGQ_OK;
    if (!dy || !dx) return fail(HGQ_ERR_ARG, "hgq_mean_mid_bwd: null pointer");
    if (P * N * 4 >= (1ll << 31) || B >= (1ll << 31)) return fail(HGQ_ERR_UNSUPPORTED, "hgq_mean_mid_bwd: one batch element must stay below 2 GiB");
    const bool vec = N % 4 == 0 && ((uintptr_t)dx & 15u) == 0;
    const int64_t cg = vec ? N / 4 : N;
    int TX = 1;
    while (TX < cg && TX < 256) TX <<= 1;
    const float inv = 1.0f / (float)P;
    if (vec) hipLaunchKernelGGL(mean_mid_bwd_kernel<4>, dim3((unsigned)B), dim3(256), 0, (hipStream_t)stream, dy, dx, (int)P, (int)N, TX, inv);
    else hipLaunchKernelGGL(mean_mid_bwd_kernel<1>, dim3((unsigned)B), dim3(256), 0, (hipStream_t)stream, dy, dx, (int)P, (int)N, TX, inv);
    return check_launch("hgq_mean_mid_bwd");
}

extern "C" int hgq_pool2d_fwd(const float *x, float *y, const int *geom, int is_max, void *stream) {
    PoolGeom g;
    if (!geom) return fail(HGQ_ERR_ARG, "hgq_pool2d_fwd: null geometry");
    int rc = check_pool(geom, g, "hgq_pool2d_fwd");
    if (rc) return rc;
    if (g.B == 0) return HGQ_OK;
    if (!x || !y) return fail(HGQ_ERR_ARG, "hgq_pool2d_fwd: null pointer");
    const bool vec = g.C % 4 == 0 && ((uintptr_t)x & 15u) == 0 && ((uintptr_t)y & 15u) == 0;
    const int64_t n = (int64_t)g.B * g.OH * g.OW * (vec ? g.C / 4 : g.C);
    const dim3 grid((unsigned)persistent_grid((n + 255) / 256, 32));
    hipStream_t s = (hipStream_t)stream;
    if (vec && is_max) hipLaunchKernelGGL((pool2d_fwd_kernel<4, true>), grid, dim3(256), 0, s, x, y, g);
    else if (vec) hipLaunchKernelGGL((pool2d_fwd_kernel<4, false>), grid, dim3(256), 0, s, x, y, g);
    else if (is_max) hipLaunchKernelGGL((pool2d_fwd_kernel<1, true>), grid, dim3(256), 0, s, x, y, g);
    else hipLaunchKernelGGL((pool2d_fwd_kernel<1, false>), grid, dim3(256), 0, s, x, y, g);
    return check_launch("hgq_pool2d_fwd");
}

extern "C" int hgq_pool2d_bwd(const float *dy, const float *x, float *dx, const int *geom, int is_max, void *stream) {
    PoolGeom g;
    if (!geom) return fail(HGQ_ERR_ARG, "hgq_pool2d_bwd: null geometry");
    int rc = check_pool(geom, g, "hgq_pool2d_bwd");
    if (rc) return rc;
    if (g.B == 0) return HGQ_OK;
    if (!dy || !dx || (is_max && !x)) return fail(HGQ_ERR_ARG, "hgq_pool2d_bwd: null pointer");
    const bool vec = g.C % 4 == 0 && ((uintptr_t)dy & 15u) == 0 && ((uintptr_t)dx & 15u) == 0 && (!is_max || ((uintptr_t)x & 15u) == 0);
    hipStream_t s = (hipStream_t)stream;
    if (g.sy >= g.ph && g.sx >= g.pw) {
        const int TH = (g.H + g.py + g.sy - 1) / g.sy, TW = (g.W + g.px + g.sx - 1) / g.sx;
        const int64_t n = (int64_t)g.B * TH * TW * (vec ? g.C / 4 : g.C);
        const dim3 grid((unsigned)persistent_grid((n + 255) / 256, 32));
        if (vec && is_max) hipLaunchKernelGGL((pool2d_bwd_tiles_kernel<4, true>), grid, dim3(256), 0, s, dy, x, dx, g, TH, TW);
        else if (vec) hipLaunchKernelGGL((pool2d_bwd_tiles_kernel<4, false>), grid, dim3(256), 0, s, dy, x, dx, g, TH, TW);
        else if (is_max) hipLaunchKernelGGL((pool2d_bwd_tiles_kernel<1, true>), grid, dim3(256), 0, s, dy, x, dx, g, TH, TW);
        else hipLaunchKernelGGL((pool2d_bwd_tiles_kernel<1, false>), grid, dim3(256), 0, s, dy, x, dx, g, TH, TW);
        return check_launch("hgq_pool2d_bwd");
    }
    const int64_t n = (int64_t)g.B * g.H * g.W * (vec ? g.C / 4 : g.C);
    const dim3 grid((unsigned)persistent_grid((n + 255) / 256, 32));
    if (vec && is_max) hipLaunchKernelGGL((pool2d_bwd_kernel<4, true>), grid, dim3(256), 0, s, dy, x, dx, g);
    else if (vec) hipLaunchKernelGGL((pool2d_bwd_kernel<4, false>), grid, dim3(256), 0, s, dy, x, dx, g);
    else if (is_max) hipLaunchKernelGGL((pool2d_bwd_kernel<1, true>), grid, dim3(256), 0, s, dy, x, dx, g);
    else hipLaunchKernelGGL((pool2d_bwd_kernel<1, false>), grid, dim3(256), 0, s, dy, x, dx, g);
    return check_launch("hgq_pool2d_bwd");
}
