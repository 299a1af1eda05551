// QConv2D contraction for small feature maps: implicit GEMM on fp32 MFMA with the operands in LDS.
//
// The im2col gather reads every source element kh * kw times; done from global memory that
// traffic, not HBM or the matrix cores, bounds the kernel.  Here a workgroup takes a TH x TW tile
// of pixels of ONE image, stages the source patch the tile touches once (zeros outside the image,
// the ReLU mask applied while staging) with a pixel stride of D + 1 words, keeps the whole kernel
// matrix in LDS, and the matrix cores read both operands from LDS: the A operand of tap (ky, kx)
// is the patch shifted by a per-tap offset, so the inner loop is one LDS read per operand and one
// v_mfma_f32_32x32x2f32, with no index arithmetic and no barrier.
//
//   forward        rows = output pixels, depth D = C, N = F:  patch of the input
//   data gradient  rows = input pixels,  depth D = F, N = C:  patch of dz (unit stride only)
//   weight grad.   contraction over the tile's output pixels; a wavefront owns whole taps and
//                  keeps their [32 x 32] blocks in registers across the tiles of its workgroup
//
// MFMA 32x32x2 fp32 operand layout (64 lanes): A[i][k]: i = lane % 32, k = lane / 32;
// B[k][j]: k = lane / 32, j = lane % 32; D[i][j] in 16 registers: j = lane % 32,
// i = (r / 4) * 8 + (lane / 32) * 4 + (r % 4).
#include "hgq_device.h"
#include "hgq_host.h"

namespace hgq {

#define PG_WS 33  // row stride of the kernel matrix in LDS

__device__ __forceinline__ int pg_acc_row(int r, int lane) { return (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3); }

struct PatchPlan {
    int TH, TW, tiles_y, tiles_x;  // tile of row-space pixels
    int PH, PW, DS;                // patch of source pixels, pixel stride in words
    int D, N;                      // gathered depth, output channels
    int RH, RW, SH, SW;            // row-space and source-space image sizes
};

// Staging of the source patch of one tile: PH * PW pixels of D floats as 128-bit units, unit e of
// a thread = e * NT + thread.  The first PG_MAXU units of a thread are loaded into registers
// (buffer loads, zeros outside the image) while the matrix cores still work on the previous
// tile, and written to LDS afterwards; a larger patch stages the rest in place.
#define PG_MAXU 6
struct PatchRegs {
    f32x4_t v[PG_MAXU], m[PG_MAXU];
};

__device__ __forceinline__ uint32_t patch_unit_offset(const PatchPlan &p, int e, int n_u, int D4, int b, int sy0, int sx0, int &dst) {
    dst = -1;
    if (e >= n_u) return BUF_OOB;
    const int px = e / D4, d4 = e - px * D4, pr = px / p.PW, pc = px - pr * p.PW;
    const int yy = sy0 + pr, xx = sx0 + pc;
    dst = px * p.DS + 4 * d4;
    if ((unsigned)yy < (unsigned)p.SH && (unsigned)xx < (unsigned)p.SW) return (uint32_t)(((b * p.SH + yy) * p.SW + xx) * p.D + 4 * d4) * 4u;
    return BUF_OOB;
}

template <bool MASKED, int NT>
__device__ __forceinline__ void patch_fetch(PatchRegs &r, const __amdgpu_buffer_rsrc_t rs_src, const __amdgpu_buffer_rsrc_t rs_mask,
                                            const PatchPlan &p, int b, int sy0, int sx0) {
    const int D4 = p.D >> 2, n_u = p.PH * p.PW * D4;
#pragma unroll
    for (int u = 0; u < PG_MAXU; ++u) {
        int dst;
        const uint32_t off = patch_unit_offset(p, u * NT + (int)threadIdx.x, n_u, D4, b, sy0, sx0, dst);
        r.v[u] = buf_ld4(rs_src, off);
        if (MASKED) r.m[u] = buf_ld4(rs_mask, off);
    }
}

template <bool MASKED, int NT>
__device__ __forceinline__ void patch_stash(float *patch, const PatchRegs &r, const __amdgpu_buffer_rsrc_t rs_src,
                                            const __amdgpu_buffer_rsrc_t rs_mask, bool use_mask, const PatchPlan &p, int b, int sy0,
                                            int sx0) {
    const int D4 = p.D >> 2, n_u = p.PH * p.PW * D4;
#pragma unroll
    for (int u = 0; u < PG_MAXU; ++u) {
        const int e = u * NT + (int)threadIdx.x;
        if (e < n_u) {
            const int px = e / D4, dst = px * p.DS + 4 * (e - px * D4);
#pragma unroll
            for (int j = 0; j < 4; ++j) patch[dst + j] = (!MASKED || !use_mask || r.m[u][j] > 0.f) ? r.v[u][j] : 0.f;
        }
    }
    // the rest of a large patch, four units in flight
    for (int e0 = PG_MAXU * NT; e0 < n_u; e0 += 4 * NT) {
        f32x4_t v[4], m[4];
        int dst[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const uint32_t off = patch_unit_offset(p, e0 + u * NT + (int)threadIdx.x, n_u, D4, b, sy0, sx0, dst[u]);
            v[u] = buf_ld4(rs_src, off);
            if (MASKED) m[u] = buf_ld4(rs_mask, off);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            if (dst[u] >= 0) {
#pragma unroll
                for (int j = 0; j < 4; ++j) patch[dst[u] + j] = (!MASKED || !use_mask || m[u][j] > 0.f) ? v[u][j] : 0.f;
            }
        }
    }
}

// Position (ty << 16 | tx) of tile row `rr` for a tile TW pixels wide.
__device__ __forceinline__ int tile_pos(int rr, int TW) {
    const int ty = rr / TW;
    return (ty << 16) | (rr - ty * TW);
}
__device__ __forceinline__ int tile_pos_advance(int pos, int by, int TW) {  // by < 32768
    int ty = pos >> 16, tx = (pos & 0xffff) + by;
    while (tx >= TW) tx -= TW, ++ty;
    return (ty << 16) | tx;
}

// MODE 0: forward; MODE 1: data gradient.  NW wavefronts, each owning 32 rows of the tile.
// BF: the contraction runs on the bf16 matrix instruction over exact bf16 parts of the fp32 operands (mfma_chain_bf16: same
// LDS reads, the same values up to the order of the fp32 additions); the source of the data gradient is an arbitrary fp32 tensor.
template <int MODE, int NW, bool BF = false>
__global__ __launch_bounds__(NW * 64) void pgemm_kernel(const float *__restrict__ src, const float *__restrict__ mask,
                                                       const float *__restrict__ w, const float *__restrict__ bias,
                                                       float *__restrict__ out, hgq_conv_geom g, int F, int act, PatchPlan p) {
    constexpr int NT = NW * 64;
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int taps = g.kh * g.kw, K = taps * p.D;
    float *wl = lds, *patch = lds + ((K * PG_WS + 3) & ~3);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, kq = lane >> 5, n = lane & 31;
    const int64_t src_bytes = (int64_t)g.B * p.SH * p.SW * p.D * 4;
    const __amdgpu_buffer_rsrc_t rs_src = buf_rsrc(src, src_bytes), rs_mask = buf_rsrc(mask ? mask : src, mask ? src_bytes : 0);
    const int tiles_per_image = p.tiles_y * p.tiles_x;
    const int64_t n_tiles = (int64_t)g.B * tiles_per_image;
    // source origin of a tile
    auto origin = [&](int64_t tile, int &b, int &ty0, int &tx0, int &sy0, int &sx0) {
        b = (int)(tile / tiles_per_image);
        const int rem = (int)(tile - (int64_t)b * tiles_per_image);
        ty0 = (rem / p.tiles_x) * p.TH, tx0 = (rem % p.tiles_x) * p.TW;
        sy0 = MODE == 0 ? ty0 * g.sy - g.py : ty0 + g.py - (g.kh - 1) * g.dly;
        sx0 = MODE == 0 ? tx0 * g.sx - g.px : tx0 + g.px - (g.kw - 1) * g.dlx;
    };
    PatchRegs pre;
    int64_t tile = blockIdx.x;
    int b, ty0, tx0, sy0, sx0;
    if (tile < n_tiles) {
        origin(tile, b, ty0, tx0, sy0, sx0);
        patch_fetch<MODE == 1, NT>(pre, rs_src, rs_mask, p, b, sy0, sx0);  // in flight during the set-up below
    }
    // kernel matrix B[k = (tap, d)][n] -> wl[k][n], zero for n >= N; eight loads per thread in flight
    // (one load per loop trip would cost a full memory latency each)
    {
        const __amdgpu_buffer_rsrc_t rs_w = buf_rsrc(w, (int64_t)K * p.N * 4);
        const int dshift = (p.D & (p.D - 1)) == 0 ? __builtin_ctz(p.D) : -1;
        for (int id0 = 0; id0 < K * 32; id0 += 8 * NT) {
            float v[8];
            int dst[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int id = id0 + u * NT + tid;
                uint32_t off = BUF_OOB;
                dst[u] = -1;
                if (id < K * 32) {
                    if (MODE == 0) {
                        const int k = id >> 5, nn = id & 31;
                        dst[u] = k * PG_WS + nn;
                        if (nn < p.N) off = (uint32_t)(k * p.N + nn) * 4u;
                    } else {
                        // W[tap][c = n][f = d]: consecutive threads take consecutive f
                        const int r = dshift >= 0 ? id >> dshift : id / p.D, d = id - r * p.D, nn = r & 31, tap = r >> 5;
                        dst[u] = (tap * p.D + d) * PG_WS + nn;
                        if (nn < p.N) off = (uint32_t)((tap * p.N + nn) * F + d) * 4u;
                    }
                }
                v[u] = buf_ld1(rs_w, off);
            }
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (dst[u] >= 0) wl[dst[u]] = v[u];
        }
    }
    // tile-relative position of the row this lane feeds to the matrix cores, and of its 16 result
    // rows (one division, the others follow by stepping)
    const int n_rows = p.TH * p.TW;
    const int r_lane = wave * 32 + (lane & 31);
    int rowbase = 0;
    if (r_lane < n_rows) {
        const int pos = tile_pos(r_lane, p.TW), ty = pos >> 16, tx = pos & 0xffff;
        rowbase = MODE == 0 ? (ty * g.sy * p.PW + tx * g.sx) * p.DS : (ty * p.PW + tx) * p.DS;
    }
    int rpos[16];
    {
        int pos4 = tile_pos(wave * 32 + (lane >> 5) * 4, p.TW);  // row of register 0
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
            int pos = pos4;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int rr = wave * 32 + q4 * 8 + (lane >> 5) * 4 + j;
                rpos[q4 * 4 + j] = rr < n_rows ? pos : -1;
                pos = tile_pos_advance(pos, 1, p.TW);
            }
            pos4 = tile_pos_advance(pos4, 8, p.TW);
        }
    }
    const float bb = (MODE == 0 && bias && n < p.N) ? bias[n] : 0.f;
    for (; tile < n_tiles; tile += gridDim.x) {
        __syncthreads();  // the previous tile's operand reads are done (and, the first time, wl is written)
        patch_stash<MODE == 1, NT>(patch, pre, rs_src, rs_mask, mask != nullptr, p, b, sy0, sx0);
        __syncthreads();
        const int cb = b, cty0 = ty0, ctx0 = tx0;
        const int64_t next = tile + gridDim.x;
        if (next < n_tiles) {
            origin(next, b, ty0, tx0, sy0, sx0);
            patch_fetch<MODE == 1, NT>(pre, rs_src, rs_mask, p, b, sy0, sx0);  // lands while the matrix cores work
        }
        floatx16 acc = {0};
        if (wave * 32 < n_rows) {
            for (int tap = 0; tap < taps; ++tap) {
                const int ky = tap / g.kw, kx = tap - ky * g.kw;
                const int tapoff = MODE == 0 ? (ky * g.dly * p.PW + kx * g.dlx) * p.DS
                                             : ((g.kh - 1 - ky) * g.dly * p.PW + (g.kw - 1 - kx) * g.dlx) * p.DS;
                const float *ap = patch + rowbase + tapoff + kq;
                const float *bp = wl + (tap * p.D + kq) * PG_WS + n;
                // eight depth steps at a time, operands read ahead of the matrix instructions (D is a multiple of 4)
                int d = 0;
                if (BF) {
                    for (; d + 16 <= p.D; d += 16) acc = mfma_chain_bf16<MODE == 1, false>(acc, ap + d, 1, bp + d * PG_WS, PG_WS, 1);
                }
                for (; d + 16 <= p.D; d += 16) {
                    float a[8], bq[8];
#pragma unroll
                    for (int u = 0; u < 8; ++u) a[u] = ap[d + 2 * u], bq[u] = bp[(d + 2 * u) * PG_WS];
#pragma unroll
                    for (int u = 0; u < 8; ++u) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u], bq[u], acc, 0, 0, 0);
                }
                for (; d < p.D; d += 4) {
                    const float a0 = ap[d], a1 = ap[d + 2], b0 = bp[d * PG_WS], b1 = bp[(d + 2) * PG_WS];
                    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b0, acc, 0, 0, 0);
                    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b1, acc, 0, 0, 0);
                }
            }
            if (n < p.N) {
                const int y_end = min(cty0 + p.TH, p.RH);
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    if (rpos[r] < 0) continue;
                    const int ry = cty0 + (rpos[r] >> 16), rx = ctx0 + (rpos[r] & 0xffff);
                    if (ry < y_end && rx < p.RW) {
                        float v = acc[r] + bb;
                        if (MODE == 0 && act == HGQ_ACT_RELU) v = v > 0.f ? v : 0.f;
                        out[(((int64_t)cb * p.RH + ry) * p.RW + rx) * p.N + n] = v;
                    }
                }
            }
        }
    }
}

#define PG_MAX_LDS (80 * 1024)  // two workgroups per CU

static bool plan_patch(int mode, const hgq_conv_geom &g, int F, PatchPlan &p, size_t &lds) {
    p.D = mode == 0 ? g.C : F, p.N = mode == 0 ? F : g.C;
    p.RH = mode == 0 ? g.OH : g.H, p.RW = mode == 0 ? g.OW : g.W;
    p.SH = mode == 0 ? g.H : g.OH, p.SW = mode == 0 ? g.W : g.OW;
    const int64_t K = (int64_t)g.kh * g.kw * p.D;
    if (p.D % 4 != 0 || p.N > 32 || K * PG_WS * 4 > 48 * 1024 || (int64_t)p.RH * p.RW < 32) return false;
    if (mode == 1 && (g.sy != 1 || g.sx != 1)) return false;
    if ((int64_t)g.B * p.SH * p.SW * p.D * 4 >= (1ll << 31) || p.RH >= 32768 || p.RW >= 32768) return false;
    p.DS = p.D + 1;
    p.TW = p.RW < 32 ? p.RW : 32;
    p.tiles_x = (p.RW + p.TW - 1) / p.TW;
    const size_t wbytes = (size_t)((K * PG_WS + 3) & ~3ll) * 4;
    for (int th = 256 / p.TW; th >= 1; --th) {
        const int tiles_y = (p.RH + th - 1) / th;
        p.TH = (p.RH + tiles_y - 1) / tiles_y, p.tiles_y = tiles_y;
        p.PH = mode == 0 ? (p.TH - 1) * g.sy + (g.kh - 1) * g.dly + 1 : p.TH + (g.kh - 1) * g.dly;
        p.PW = mode == 0 ? (p.TW - 1) * g.sx + (g.kw - 1) * g.dlx + 1 : p.TW + (g.kw - 1) * g.dlx;
        lds = wbytes + (size_t)p.PH * p.PW * p.DS * 4;
        if (lds <= PG_MAX_LDS) return (int64_t)p.TH * p.TW >= 16;
    }
    return false;
}

static int patch_grid(const hgq_conv_geom &g, const PatchPlan &p, size_t lds) {
    int per_cu = (int)((160 * 1024) / lds);
    if (per_cu > 4) per_cu = 4;
    if (per_cu < 1) per_cu = 1;
    return persistent_grid((int64_t)g.B * p.tiles_y * p.tiles_x, per_cu);
}

bool conv_patch_ok(int mode, const hgq_conv_geom &g, int F) {
    PatchPlan p;
    size_t lds;
    return plan_patch(mode, g, F, p, lds);
}

int conv_patch_launch(int mode, const float *src, const float *mask, const float *w, const float *bias, float *out,
                      const hgq_conv_geom &g, int F, int act, hipStream_t s) {
    PatchPlan p;
    size_t lds;
    if (!plan_patch(mode, g, F, p, lds)) return fail(HGQ_ERR_UNSUPPORTED, "conv_patch_launch: shape not covered");
    const dim3 grid((unsigned)patch_grid(g, p, lds));
    const bool wide = p.TH * p.TW > 128;  // eight wavefronts of 32 rows
    // more than 64 KiB of dynamic LDS has to be allowed per kernel, once
    static bool allowed = false;
    if (!allowed) {
        const void *kernels[8] = {(const void *)pgemm_kernel<0, 4>, (const void *)pgemm_kernel<0, 8>, (const void *)pgemm_kernel<1, 4>,
                                  (const void *)pgemm_kernel<1, 8>, (const void *)pgemm_kernel<0, 4, true>, (const void *)pgemm_kernel<0, 8, true>,
                                  (const void *)pgemm_kernel<1, 4, true>, (const void *)pgemm_kernel<1, 8, true>};
        for (const void *k : kernels)
            if (hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, PG_MAX_LDS) != hipSuccess)
                return fail(HGQ_ERR_LAUNCH, "conv_patch_launch: cannot raise the dynamic LDS limit");
        allowed = true;
    }
#define PG_LAUNCH(BFV) \
    do { \
        if (mode == 0 && wide) hipLaunchKernelGGL((pgemm_kernel<0, 8, BFV>), grid, dim3(512), lds, s, src, mask, w, bias, out, g, F, act, p); \
        else if (mode == 0) hipLaunchKernelGGL((pgemm_kernel<0, 4, BFV>), grid, dim3(256), lds, s, src, mask, w, bias, out, g, F, act, p); \
        else if (wide) hipLaunchKernelGGL((pgemm_kernel<1, 8, BFV>), grid, dim3(512), lds, s, src, mask, w, bias, out, g, F, act, p); \
        else hipLaunchKernelGGL((pgemm_kernel<1, 4, BFV>), grid, dim3(256), lds, s, src, mask, w, bias, out, g, F, act, p); \
    } while (0)
    if (hgq_dense_use_bf16_parts(-1)) PG_LAUNCH(true);
    else PG_LAUNCH(false);
#undef PG_LAUNCH
    return check_launch("conv_patch_launch");
}

}  // namespace hgq
