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

// Time stamps of workgroup 0 (measurement builds only: -DPG_PROF): [mode][wavefront][event]
#ifdef PG_PROF
__device__ unsigned long long pg_prof_stamps[2 * 8 * 32];
#define PG_STAMP(i)                                                                                                          \
    do {                                                                                                                     \
        if (blockIdx.x == 0 && (threadIdx.x & 63) == 0 && (i) < 32) pg_prof_stamps[(MODE * 8 + (threadIdx.x >> 6)) * 32 + (i)] = wall_clock64(); \
    } while (0)
#else
#define PG_STAMP(i)
#endif

__device__ __forceinline__ int pg_acc_row(int r, int lane) { return (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3); }

struct PatchPlan {
    int TH, TW, tiles_y, tiles_x;  // tile of row-space pixels
    int PH, PW, DS;                // patch of source pixels, pixel stride in words
    int D, N;                      // gathered depth, output channels
    int patch_words;               // LDS words of the patch (fp32 form: PH * PW * DS; bf16 parts: PH * PW * D * 3 / 2)
    int RH, RW, SH, SW;            // row-space and source-space image sizes
};

// Staging of the source patch of one tile: PH * PW pixels of D floats as 128-bit units, unit e of
// a thread = e * NT + thread.  The first PG_MAXU units of a thread are loaded into registers
// (buffer loads, zeros outside the image) while the matrix cores still work on the previous
// tile, and written to LDS afterwards; a larger patch stages the rest in place.
// (A workgroup of eight wavefronts keeps four: its threads are twice as many, and two such workgroups share a CU only
// if a wavefront stays within 128 registers.)
template <int MAXU>
struct PatchRegs {
    f32x4_t v[MAXU], m[MAXU];
    // where unit u of this thread sits in the patch - row << 20 | column << 8 | group of four depths, ~0 past the patch's
    // end: the same for every tile, so the divisions that find it are done once per launch, not once per tile
    uint32_t geo[MAXU];
    template <int NT>
    __device__ __forceinline__ void init(const PatchPlan &p) {
        const int D4 = p.D >> 2, n_u = p.PH * p.PW * D4;
#pragma unroll
        for (int u = 0; u < MAXU; ++u) {
            const int e = u * NT + (int)threadIdx.x, px = e / D4, pr = px / p.PW;
            geo[u] = e < n_u ? ((uint32_t)pr << 20) | ((uint32_t)(px - pr * p.PW) << 8) | (uint32_t)(e - px * D4) : ~0u;
        }
    }
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

template <bool MASKED, int NT, int MAXU>
__device__ __forceinline__ void patch_fetch(PatchRegs<MAXU> &r, const __amdgpu_buffer_rsrc_t rs_src, const __amdgpu_buffer_rsrc_t rs_mask,
                                            const PatchPlan &p, int b, int sy0, int sx0) {
#pragma unroll
    for (int u = 0; u < MAXU; ++u) {
        const uint32_t gq = r.geo[u];
        const int yy = sy0 + (int)(gq >> 20), xx = sx0 + (int)((gq >> 8) & 0xfffu);
        const bool in = gq != ~0u && (unsigned)yy < (unsigned)p.SH && (unsigned)xx < (unsigned)p.SW;
        const uint32_t off = in ? (uint32_t)(((b * p.SH + yy) * p.SW + xx) * p.D + 4 * (int)(gq & 0xffu)) * 4u : BUF_OOB;
        r.v[u] = buf_ld4(rs_src, off);
        if (MASKED) r.m[u] = buf_ld4(rs_mask, off);
    }
}

// The patch in LDS, two forms.  fp32: pixel px, depth d at word px * DS + d (DS = D + 1).  bf16 parts (D = 16, 32 or 64): every
// value as its three exact bf16 parts (hgq_device.h: an fp32 number is the sum of three numbers of eight significant bits),
// split ONCE here instead of at each of the kh * kw reads; a pixel is 3 * D / 8 slots of 16 bytes - part-major, eight
// consecutive depths per slot - so a lane's A operand of a 32x32x16 bf16 instruction is one 128-bit read per part.  Slot
// c of a pixel sits at c ^ ((px >> (4 - j)) & (D / 8 - 1)), j = log2(D / 8): with a pixel stride of 3 * 2**j slots, sixteen
// consecutive pixels then read sixteen different 16-byte bank groups (no padding: the patch and the kernel matrix of a
// 3 x 3 x 32 layer fill the 80 KB that let two workgroups share a CU).
__device__ __forceinline__ void put_unit_f32(float *patch, int DS, int px, int d4, const f32x4_t &v) {
#pragma unroll
    for (int j = 0; j < 4; ++j) patch[px * DS + 4 * d4 + j] = v[j];
}
__device__ __forceinline__ void put_unit_parts(float *patch, int nch, int jbits, int px, int d4, const f32x4_t &v, uint32_t &nz) {
    uint32_t h[4], m[4], l[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) bf16_parts(v[j], h[j], m[j], l[j]);
    const int pos = (d4 >> 1) ^ ((px >> (4 - jbits)) & (nch - 1));
    uint2 *dst = (uint2 *)patch + (px * 3 * nch + pos) * 2 + (d4 & 1);
    dst[0] = uint2{bf16_pair(h[0], h[1]), bf16_pair(h[2], h[3])};
    dst[2 * nch] = uint2{bf16_pair(m[0], m[1]), bf16_pair(m[2], m[3])};
    dst[4 * nch] = uint2{bf16_pair(l[0], l[1]), bf16_pair(l[2], l[3])};
    // which parts the tile needs at all (bit 0: a second part, bit 1: a third one; a third part implies a second)
    nz |= ((m[0] | m[1] | m[2] | m[3]) != 0u ? 1u : 0u) | ((l[0] | l[1] | l[2] | l[3]) != 0u ? 2u : 0u);
}

template <bool MASKED, int NT, int MAXU, bool PARTS>
__device__ __forceinline__ uint32_t patch_stash(float *patch, const PatchRegs<MAXU> &r, const __amdgpu_buffer_rsrc_t rs_src,
                                                const __amdgpu_buffer_rsrc_t rs_mask, bool use_mask, const PatchPlan &p, int b, int sy0,
                                                int sx0) {
    const int D4 = p.D >> 2, n_u = p.PH * p.PW * D4, nch = p.D >> 3, jbits = 31 - __clz(nch);
    uint32_t nz = 0u;
#pragma unroll
    for (int u = 0; u < MAXU; ++u) {
        const uint32_t gq = r.geo[u];
        if (gq != ~0u) {
            const int px = (int)(gq >> 20) * p.PW + (int)((gq >> 8) & 0xfffu), d4 = (int)(gq & 0xffu);
            f32x4_t v;
#pragma unroll
            for (int j = 0; j < 4; ++j) v[j] = (!MASKED || !use_mask || r.m[u][j] > 0.f) ? r.v[u][j] : 0.f;
            if (PARTS) put_unit_parts(patch, nch, jbits, px, d4, v, nz);
            else put_unit_f32(patch, p.DS, px, d4, v);
        }
    }
    // the rest of a large patch, four units in flight
    for (int e0 = MAXU * NT; e0 < n_u; e0 += 4 * NT) {
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
                const int e = e0 + u * NT + (int)threadIdx.x, px = e / D4, d4 = e - px * D4;
                f32x4_t w;
#pragma unroll
                for (int j = 0; j < 4; ++j) w[j] = (!MASKED || !use_mask || m[u][j] > 0.f) ? v[u][j] : 0.f;
                if (PARTS) put_unit_parts(patch, nch, jbits, px, d4, w, nz);
                else put_unit_f32(patch, p.DS, px, d4, w);
            }
        }
    }
    return nz;
}

// One batch of sixteen contraction steps with the A operand already in bf16 parts (n_a of them are not all zero in this
// tile) and B as fp32 values from LDS: B's leading parts are one byte-permute per pair; its further parts are formed only
// where some lane of the wavefront has them.  Every product of two parts is exact in fp32; only the accumulation rounds.
__device__ __forceinline__ floatx16 mfma_batch_parts_a(floatx16 acc, const u32x4_t (&a)[3], int n_a, const float (&b)[8]) {
    u32x4_t pb0;
    const bool one_b = bf16_lead8(b, pb0);
    acc = mfma_bf16(a[0], pb0, acc);
    if (n_a > 1) acc = mfma_bf16(a[1], pb0, acc);
    if (n_a > 2) acc = mfma_bf16(a[2], pb0, acc);
    if (!one_b) {
        u32x4_t p1, p2;
        const bool third = bf16_rest8(b, p1, p2);
        acc = mfma_bf16(a[0], p1, acc);
        if (n_a > 1) acc = mfma_bf16(a[1], p1, acc);
        if (n_a > 2) acc = mfma_bf16(a[2], p1, acc);
        if (third) {
            acc = mfma_bf16(a[0], p2, acc);
            if (n_a > 1) acc = mfma_bf16(a[1], p2, acc);
            if (n_a > 2) acc = mfma_bf16(a[2], p2, acc);
        }
    }
    return acc;
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
// BF = 1: the contraction runs on the bf16 matrix instruction over exact bf16 parts of the fp32 operands, formed at each LDS read
// (mfma_chain_bf16: same LDS reads, the same values up to the order of the fp32 additions); the source of the data gradient
// is an arbitrary fp32 tensor.  BF = 2 (D = 16, 32 or 64): the patch is staged as bf16 parts, see put_unit_parts.
template <int MODE, int NW, int BF = 0>
__global__ __launch_bounds__(NW * 64, NW == 8 ? 4 : 2) void pgemm_kernel(const float *__restrict__ src, const float *__restrict__ mask,
                                                       const float *__restrict__ w, const float *__restrict__ bias,
                                                       float *__restrict__ out, hgq_conv_geom g, int F, int act, PatchPlan p) {
    constexpr int NT = NW * 64;
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int taps = g.kh * g.kw, K = taps * p.D;
    float *wl = lds, *patch = lds + ((K * PG_WS + 3) & ~3);
    uint32_t *part_flags = (uint32_t *)(patch + p.patch_words);  // [2], BF == 2 forward only
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, kq = lane >> 5, n = lane & 31;
    const int64_t src_bytes = (int64_t)g.B * p.SH * p.SW * p.D * 4;
    const __amdgpu_buffer_rsrc_t rs_src = buf_rsrc(src, src_bytes), rs_mask = buf_rsrc(mask ? mask : src, mask ? src_bytes : 0);
    const __amdgpu_buffer_rsrc_t rs_out = buf_rsrc(out, (int64_t)g.B * p.RH * p.RW * p.N * 4);
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
    PatchRegs<(NW == 8 ? 4 : 6)> pre;
    pre.template init<NT>(p);
    int64_t tile = blockIdx.x;
    int b, ty0, tx0, sy0, sx0;
    PG_STAMP(0);
    if (BF == 2 && MODE == 0 && tid < 2) part_flags[tid] = 0u;
    if (tile < n_tiles) {
        origin(tile, b, ty0, tx0, sy0, sx0);
        patch_fetch<MODE == 1, NT>(pre, rs_src, rs_mask, p, b, sy0, sx0);  // in flight during the set-up below
    }
    // kernel matrix B[k = (tap, d)][n] -> wl[k][n], zero for n >= N.  128-bit loads, six or twelve per thread in flight (the matrix
    // is a few tens of KB in L2: what costs is a memory latency per loop trip, so a trip moves 24 or 48 values per thread);
    // a forward kernel matrix whose rows are not a multiple of four values wide goes value by value
    {
        const __amdgpu_buffer_rsrc_t rs_w = buf_rsrc(w, (int64_t)K * p.N * 4);
        const int dshift = (p.D & (p.D - 1)) == 0 ? __builtin_ctz(p.D) : -1;
        if (MODE == 1 || (p.N & 3) == 0) {
            const int D4 = p.D >> 2, n_u = MODE == 0 ? K * 8 : taps * 32 * D4;
            constexpr int WU = NW == 8 ? 6 : 12;  // units of a thread per trip
            for (int id0 = 0; id0 < n_u; id0 += WU * NT) {
                f32x4_t v[WU];
                int dst[WU];
#pragma unroll
                for (int u = 0; u < WU; ++u) {
                    const int id = id0 + u * NT + tid;
                    uint32_t off = BUF_OOB;
                    dst[u] = -1;
                    if (id < n_u) {
                        if (MODE == 0) {
                            const int k = id >> 3, n4 = (id & 7) * 4;
                            dst[u] = k * PG_WS + n4;
                            if (n4 < p.N) off = (uint32_t)(k * p.N + n4) * 4u;
                        } else {
                            // W[tap][c = n][f = d]: consecutive threads take consecutive groups of four f
                            const int r = dshift >= 2 ? id >> (dshift - 2) : id / D4, d = (id - r * D4) * 4, nn = r & 31, tap = r >> 5;
                            dst[u] = (tap * p.D + d) * PG_WS + nn;
                            if (nn < p.N) off = (uint32_t)((tap * p.N + nn) * F + d) * 4u;
                        }
                    }
                    v[u] = buf_ld4(rs_w, off);
                }
#pragma unroll
                for (int u = 0; u < WU; ++u)
                    if (dst[u] >= 0) {
#pragma unroll
                        for (int j = 0; j < 4; ++j) wl[dst[u] + (MODE == 0 ? j : j * PG_WS)] = v[u][j];
                    }
            }
        } else {
            for (int id0 = 0; id0 < K * 32; id0 += 8 * NT) {
                float v[8];
                int dst[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const int id = id0 + u * NT + tid;
                    uint32_t off = BUF_OOB;
                    dst[u] = -1;
                    if (id < K * 32) {
                        const int k = id >> 5, nn = id & 31;
                        dst[u] = k * PG_WS + nn;
                        if (nn < p.N) off = (uint32_t)(k * p.N + nn) * 4u;
                    }
                    v[u] = buf_ld1(rs_w, off);
                }
#pragma unroll
                for (int u = 0; u < 8; ++u)
                    if (dst[u] >= 0) wl[dst[u]] = v[u];
            }
        }
    }
    // tile-relative position of the row this lane feeds to the matrix cores, and of its 16 result
    // rows (one division, the others follow by stepping)
    const int n_rows = p.TH * p.TW;
    const int r_lane = wave * 32 + (lane & 31);
    int rowpix = 0;  // the patch pixel under tap (0, 0) of this lane's row
    if (r_lane < n_rows) {
        const int pos = tile_pos(r_lane, p.TW), ty = pos >> 16, tx = pos & 0xffff;
        rowpix = MODE == 0 ? ty * g.sy * p.PW + tx * g.sx : ty * p.PW + tx;
    }
    const int rowbase = rowpix * p.DS;
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
    PG_STAMP(1);
    int it_ = 0;
    for (; tile < n_tiles; tile += gridDim.x, ++it_) {
        __syncthreads();  // the previous tile's operand reads are done (and, the first time, wl is written)
        PG_STAMP(2 + 8 * it_);
        const uint32_t nz = patch_stash<MODE == 1, NT, (NW == 8 ? 4 : 6), BF == 2>(patch, pre, rs_src, rs_mask, mask != nullptr, p, b, sy0, sx0);
        if (BF == 2 && MODE == 0) {
            const uint32_t any_nz = (__any((nz & 1u) != 0u) ? 1u : 0u) | (__any((nz & 2u) != 0u) ? 2u : 0u);
            if (lane == 0 && any_nz) atomicOr(&part_flags[it_ & 1], any_nz);
        }
        PG_STAMP(3 + 8 * it_);
        __syncthreads();
        PG_STAMP(4 + 8 * it_);
        // parts of the activations this tile needs (the gradient of the data-gradient pass always has three); the other
        // flag word is cleared for the next tile: its last readers passed the barrier at the top of this trip
        int n_a = 3;
        if (BF == 2 && MODE == 0) {
            const uint32_t f = __builtin_amdgcn_readfirstlane(part_flags[it_ & 1]);
            n_a = (f & 2u) ? 3 : ((f & 1u) ? 2 : 1);
            if (tid == 0) part_flags[(it_ + 1) & 1] = 0u;
        }
        const int cb = b, cty0 = ty0, ctx0 = tx0;
        const int64_t next = tile + gridDim.x;
        if (next < n_tiles) {
            origin(next, b, ty0, tx0, sy0, sx0);
            patch_fetch<MODE == 1, NT>(pre, rs_src, rs_mask, p, b, sy0, sx0);  // lands while the matrix cores work
        }
        floatx16 acc = {0};
        PG_STAMP(5 + 8 * it_);
        if (wave * 32 < n_rows) {
            for (int tap = 0; tap < taps; ++tap) {
                const int ky = tap / g.kw, kx = tap - ky * g.kw;
                const int tappix = MODE == 0 ? ky * g.dly * p.PW + kx * g.dlx : (g.kh - 1 - ky) * g.dly * p.PW + (g.kw - 1 - kx) * g.dlx;
                if (BF == 2) {
                    // lane half kq takes depths 8 kq .. 8 kq + 7 of each batch of sixteen: one 128-bit read per part of A
                    const int nch = p.D >> 3, px = rowpix + tappix, sw = (px >> (4 - (31 - __clz(nch)))) & (nch - 1);
                    const u32x4_t *pa = (const u32x4_t *)patch + px * 3 * nch;
                    const float *bp8 = wl + (tap * p.D + 8 * kq) * PG_WS + n;
                    for (int bt = 0; bt < (p.D >> 4); ++bt) {
                        const int pos = (2 * bt + kq) ^ sw;
                        const u32x4_t a[3] = {pa[pos], pa[nch + pos], pa[2 * nch + pos]};
                        float bq[8];
#pragma unroll
                        for (int e = 0; e < 8; ++e) bq[e] = bp8[(16 * bt + e) * PG_WS];
                        acc = mfma_batch_parts_a(acc, a, MODE == 1 ? 3 : n_a, bq);
                    }
                    continue;
                }
                const int tapoff = tappix * p.DS;
                const float *ap = patch + rowbase + tapoff + kq;
                const float *bp = wl + (tap * p.D + kq) * PG_WS + n;
                // eight depth steps at a time, operands read ahead of the matrix instructions (D is a multiple of 4)
                int d = 0;
                if (BF == 1) {
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
            PG_STAMP(6 + 8 * it_);
            {
                // through a descriptor: a row outside the tile or the image, or a column past N, is dropped by its offset
                const int y_end = min(cty0 + p.TH, p.RH);
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int ry = cty0 + (rpos[r] >> 16), rx = ctx0 + (rpos[r] & 0xffff);
                    const bool ok = rpos[r] >= 0 && ry < y_end && rx < p.RW && n < p.N;
                    float v = acc[r] + bb;
                    if (MODE == 0 && act == HGQ_ACT_RELU) v = v > 0.f ? v : 0.f;
                    buf_st1(rs_out, ok ? (uint32_t)(((cb * p.RH + ry) * p.RW + rx) * p.N + n) * 4u : BUF_OOB, v);
                }
            }
            PG_STAMP(7 + 8 * it_);
        }
    }
}

#define PG_MAX_LDS (80 * 1024)  // two workgroups per CU

static bool plan_patch(int mode, const hgq_conv_geom &g, int F, bool parts, PatchPlan &p, size_t &lds) {
    p.D = mode == 0 ? g.C : F, p.N = mode == 0 ? F : g.C;
    p.RH = mode == 0 ? g.OH : g.H, p.RW = mode == 0 ? g.OW : g.W;
    p.SH = mode == 0 ? g.H : g.OH, p.SW = mode == 0 ? g.W : g.OW;
    const int64_t K = (int64_t)g.kh * g.kw * p.D;
    if (p.D % 4 != 0 || p.N > 32 || K * PG_WS * 4 > 48 * 1024 || (int64_t)p.RH * p.RW < 32) return false;
    if (mode == 1 && (g.sy != 1 || g.sx != 1)) return false;
    if ((int64_t)g.B * p.SH * p.SW * p.D * 4 >= (1ll << 31) || p.RH >= 32768 || p.RW >= 32768) return false;
    if ((int64_t)g.B * p.RH * p.RW * p.N * 4 >= (1ll << 31)) return false;
    if (parts && p.D != 16 && p.D != 32 && p.D != 64) return false;
    if (p.D > 1020) return false;  // (a thread's place in the patch is packed into one register: 12 + 12 + 8 bits)
    p.DS = p.D + 1;
    p.TW = p.RW < 32 ? p.RW : 32;
    p.tiles_x = (p.RW + p.TW - 1) / p.TW;
    const size_t wbytes = (size_t)((K * PG_WS + 3) & ~3ll) * 4;
    for (int th = 256 / p.TW; th >= 1; --th) {
        const int tiles_y = (p.RH + th - 1) / th;
        p.TH = (p.RH + tiles_y - 1) / tiles_y, p.tiles_y = tiles_y;
        p.PH = mode == 0 ? (p.TH - 1) * g.sy + (g.kh - 1) * g.dly + 1 : p.TH + (g.kh - 1) * g.dly;
        p.PW = mode == 0 ? (p.TW - 1) * g.sx + (g.kw - 1) * g.dlx + 1 : p.TW + (g.kw - 1) * g.dlx;
        p.patch_words = parts ? p.PH * p.PW * p.D * 3 / 2 : p.PH * p.PW * p.DS;
        lds = wbytes + (size_t)p.patch_words * 4 + 16;  // (+ 16: the two part-flag words behind the patch)
        if (lds <= PG_MAX_LDS) return (int64_t)p.TH * p.TW >= 16 && p.PH < 4096 && p.PW < 4096;
    }
    return false;
}

static int patch_grid(const hgq_conv_geom &g, const PatchPlan &p, size_t lds) {
    int per_cu = (int)((160 * 1024) / lds);
    if (per_cu > 4) per_cu = 4;
    if (per_cu < 1) per_cu = 1;
    return persistent_grid((int64_t)g.B * p.tiles_y * p.tiles_x, per_cu);
}

#ifdef PG_PROF
extern "C" int hgq_pg_prof_read(unsigned long long *out) {
    return hipMemcpyFromSymbol(out, HIP_SYMBOL(pg_prof_stamps), sizeof(unsigned long long) * 2 * 8 * 32) == hipSuccess ? 0 : -2;
}
#endif

bool conv_patch_ok(int mode, const hgq_conv_geom &g, int F) {
    PatchPlan p;
    size_t lds;
    return plan_patch(mode, g, F, false, p, lds);
}

int conv_patch_launch(int mode, const float *src, const float *mask, const float *w, const float *bias, float *out,
                      const hgq_conv_geom &g, int F, int act, hipStream_t s) {
    PatchPlan p;
    size_t lds;
    // the form of the patch: bf16 parts where the matrix cores run on them and the depth allows, else fp32
    const bool bf = hgq_dense_use_bf16_parts(-1) != 0;
    const bool parts = bf && plan_patch(mode, g, F, true, p, lds);
    if (!parts && !plan_patch(mode, g, F, false, p, lds)) return fail(HGQ_ERR_UNSUPPORTED, "conv_patch_launch: shape not covered");
    const dim3 grid((unsigned)patch_grid(g, p, lds));
    const bool wide = p.TH * p.TW > 128;  // eight wavefronts of 32 rows
    // more than 64 KiB of dynamic LDS has to be allowed per kernel, once
    static bool allowed = false;
    if (!allowed) {
        const void *kernels[12] = {(const void *)pgemm_kernel<0, 4, 0>, (const void *)pgemm_kernel<0, 8, 0>, (const void *)pgemm_kernel<1, 4, 0>,
                                   (const void *)pgemm_kernel<1, 8, 0>, (const void *)pgemm_kernel<0, 4, 1>, (const void *)pgemm_kernel<0, 8, 1>,
                                   (const void *)pgemm_kernel<1, 4, 1>, (const void *)pgemm_kernel<1, 8, 1>, (const void *)pgemm_kernel<0, 4, 2>,
                                   (const void *)pgemm_kernel<0, 8, 2>, (const void *)pgemm_kernel<1, 4, 2>, (const void *)pgemm_kernel<1, 8, 2>};
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
    if (parts) PG_LAUNCH(2);
    else if (bf) PG_LAUNCH(1);
    else PG_LAUNCH(0);
#undef PG_LAUNCH
    return check_launch("conv_patch_launch");
}

// ---- weight / bias gradient -------------------------------------------------------------------
// dW[ky][kx][c][f] = sum over output pixels of x[oy + ky - py][ox + kx - px][c] * dz[oy][ox][f]  (unit stride and dilation).
// The gathered form reads every source element kh * kw times through L2 and every dz element once per block of the
// gathered matrix; here a workgroup stages a band of ONE image once - the source patch as fp32 (pixel p of the padded
// raster, XW = OW + kw - 1 pixels wide, at word p * XS), dz laid out on the SAME raster (zeros in the kw - 1 columns past OW,
// ReLU mask applied) - so that the contraction index q runs over the raster and tap (ky, kx) reads source pixel
// q + ky * XW + kx: no index arithmetic in the loop.  dz is an arbitrary fp32 tensor: it is split into its three exact bf16
// parts ONCE while staging, transposed to [part][f][q], so the B operand of a 32x32x16 bf16 instruction (eight consecutive q of
// one filter) is one 128-bit read per part.  Wavefront ky owns the kw taps of kernel row ky for the whole launch (kw
// accumulator blocks [32 c x 32 f] in registers): the taps of a row read the same source values shifted by one pixel, so a
// lane reads a window of 8 + kw - 1 values per batch of sixteen q and packs kw operands from it.  The source is a quantized
// tensor: the wavefront looks at the window and multiplies by its first bf16 part only when the others are zero
// (3 instructions per tap and batch), by two or three parts otherwise (6 / 9) - every product of two parts is exact in fp32,
// only the accumulation rounds.  Slice blockIdx.x of `part` is [kh kw C F | F] (kernel gradient, bias gradient).
#ifdef PG_PROF
__device__ unsigned long long wg_prof_stamps[8 * 32];
#define WG_STAMP(i)                                                                                                     \
    do {                                                                                                                \
        if (blockIdx.x == 0 && (threadIdx.x & 63) == 0 && (i) < 32) wg_prof_stamps[(threadIdx.x >> 6) * 32 + (i)] = clock64(); \
    } while (0)
extern "C" int hgq_wg_prof_read(unsigned long long *out) {
    return hipMemcpyFromSymbol(out, HIP_SYMBOL(wg_prof_stamps), sizeof(unsigned long long) * 8 * 32) == hipSuccess ? 0 : -2;
}
#else
#define WG_STAMP(i)
#endif

struct WgPlan {
    int TH, bands;  // output rows per tile, tiles per image
    int XW, XH;     // the tile's source raster: OW + kw - 1 pixels wide, TH + kh - 1 rows
    int XP, XS;     // pixel slots of the source patch (the windows of the last batch read past the raster: zeros), words per pixel
    int QN, QS;     // contraction length of a tile (TH * XW rounded up to 16), bf16 between the rows of a dz plane
};

template <int KH, int KW>
__global__ __launch_bounds__(64 * KH, 2) void wgrad_patch_kernel(const float *__restrict__ x, const float *__restrict__ dy,
                                                              const float *__restrict__ mask, float *__restrict__ part,
                                                              hgq_conv_geom g, int F, int relu, WgPlan p) {
    constexpr int NT = 64 * KH, WIN = 8 + KW - 1;
    extern __shared__ __attribute__((aligned(16))) float lds[];
    float *xs = lds;                                    // [XP][XS]
    uint32_t *zp = (uint32_t *)(lds + p.XP * p.XS);     // [3][32][QS / 2] pairs of bf16
    const int tid = threadIdx.x, lane = tid & 63, ky = tid >> 6, kq = lane >> 5, c = lane & 31;
    const int C4 = g.C >> 2, QS2 = p.QS >> 1;
    const __amdgpu_buffer_rsrc_t rs_x = buf_rsrc(x, (int64_t)g.B * g.H * g.W * g.C * 4);
    const __amdgpu_buffer_rsrc_t rs_dy = buf_rsrc(dy, (int64_t)g.B * g.OH * g.OW * F * 4);
    const __amdgpu_buffer_rsrc_t rs_m = buf_rsrc(relu ? mask : dy, relu ? (int64_t)g.B * g.OH * g.OW * F * 4 : 0);
    const FastDiv dxw((uint32_t)p.XW), dc4((uint32_t)C4);
    floatx16 acc[KW];
#pragma unroll
    for (int kx = 0; kx < KW; ++kx) acc[kx] = floatx16{0};
    f32x4_t bsum = {0.f, 0.f, 0.f, 0.f};
    const int f4 = tid & 7;  // NT is a multiple of 8: a thread stages the same four filters in every trip
    const bool c_counts = c < g.C;
    const int cc = c_counts ? c : 0;  // lanes past the channel count feed result rows nobody reads
    const int64_t n_tiles = (int64_t)g.B * p.bands;
    const int n_xu = p.XP * C4, n_zu = (p.QN >> 1) * 8;
    // The first XU source units and ZU dz units of a thread are asked for together (one memory latency per tile, not one per
    // unit; the registers are free again when the matrix cores start, and the other workgroups of the CU cover the wait);
    // a larger tile stages the rest in place.
    constexpr int XU = 8, ZU = 3;
    f32x4_t rx[XU], rz[ZU][2], rm[ZU][2];
    auto x_off = [&](int u, int b, int oy0, int th, int &dst) -> uint32_t {
        const uint32_t pix = dc4.div((uint32_t)u), c4 = (uint32_t)u - pix * (uint32_t)C4;
        const uint32_t pr = dxw.div(pix), pc = pix - pr * (uint32_t)p.XW;
        const int yy = oy0 + (int)pr - g.py, xx = (int)pc - g.px;
        const bool in = u < n_xu && (int)pr < th + KH - 1 && (unsigned)yy < (unsigned)g.H && (unsigned)xx < (unsigned)g.W;
        dst = u < n_xu ? (int)pix * p.XS + 4 * (int)c4 : -1;
        return in ? (uint32_t)(((b * g.H + yy) * g.W + xx) * g.C + 4 * (int)c4) * 4u : BUF_OOB;
    };
    auto z_off = [&](int u, int e, int b, int oy0, int th) -> uint32_t {
        const uint32_t q = (uint32_t)((u >> 3) * 2 + e), qr = dxw.div(q), qc = q - qr * (uint32_t)p.XW;
        const bool in = u < n_zu && (int)qr < th && (int)qc < g.OW && 4 * f4 < F;
        return in ? (uint32_t)(((b * g.OH + oy0 + (int)qr) * g.OW + (int)qc) * F + 4 * f4) * 4u : BUF_OOB;
    };
    // one dz unit (q, q + 1 of four filters) into the three planes
    auto z_put = [&](int u, const f32x4_t (&v)[2], const f32x4_t (&m)[2]) {
        if (u >= n_zu) return;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float z[2];
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                z[e] = (relu && !(m[e][j] > 0.f)) ? 0.f : v[e][j];
                bsum[j] += z[e];
            }
            uint32_t h0, m0, l0, h1, m1, l1;
            bf16_parts(z[0], h0, m0, l0), bf16_parts(z[1], h1, m1, l1);
            uint32_t *dst = zp + (4 * f4 + j) * QS2 + (u >> 3);
            dst[0] = bf16_pair(h0, h1), dst[32 * QS2] = bf16_pair(m0, m1), dst[64 * QS2] = bf16_pair(l0, l1);
        }
    };
    auto fetch = [&](int64_t tile) {
        const int b = (int)(tile / p.bands), oy0 = (int)(tile - (int64_t)b * p.bands) * p.TH, th = min(p.TH, g.OH - oy0);
#pragma unroll
        for (int i = 0; i < XU; ++i) {
            int dst;
            rx[i] = buf_ld4(rs_x, x_off(i * NT + tid, b, oy0, th, dst));
        }
#pragma unroll
        for (int i = 0; i < ZU; ++i)
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                const uint32_t off = z_off(i * NT + tid, e, b, oy0, th);
                rz[i][e] = buf_ld4(rs_dy, off);
                rm[i][e] = buf_ld4(rs_m, off);
            }
    };
    WG_STAMP(0);
    int it_ = 0;
    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x, ++it_) {
        const int b = (int)(tile / p.bands), oy0 = (int)(tile - (int64_t)b * p.bands) * p.TH;
        const int th = min(p.TH, g.OH - oy0);
        WG_STAMP(1 + 8 * it_);
        fetch(tile);      // every load of the tile is in flight before the first is waited for
        WG_STAMP(2 + 8 * it_);
        __syncthreads();  // the previous tile's operands are no longer read
        WG_STAMP(3 + 8 * it_);
        // source patch: every slot is written (zeros outside the image and past the raster)
#pragma unroll
        for (int i = 0; i < XU; ++i) {
            const int u = i * NT + tid;
            if (u < n_xu) {
                const uint32_t pix = dc4.div((uint32_t)u), c4 = (uint32_t)u - pix * (uint32_t)C4;
                *(f32x4_t *)(xs + (int)pix * p.XS + 4 * (int)c4) = rx[i];
            }
        }
        for (int u0 = XU * NT; u0 < n_xu; u0 += 4 * NT) {
            f32x4_t v[4];
            int dst[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) v[i] = buf_ld4(rs_x, x_off(u0 + i * NT + tid, b, oy0, th, dst[i]));
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (dst[i] >= 0) *(f32x4_t *)(xs + dst[i]) = v[i];
        }
        WG_STAMP(4 + 8 * it_);
        // dz on the source raster, two neighbouring q of four filters per unit; split into bf16 parts, transposed
#pragma unroll
        for (int i = 0; i < ZU; ++i) z_put(i * NT + tid, rz[i], rm[i]);
        for (int u0 = ZU * NT; u0 < n_zu; u0 += 2 * NT) {
            f32x4_t v[2][2], m[2][2];
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const uint32_t off = z_off(u0 + i * NT + tid, e, b, oy0, th);
                    v[i][e] = buf_ld4(rs_dy, off);
                    m[i][e] = buf_ld4(rs_m, off);
                }
#pragma unroll
            for (int i = 0; i < 2; ++i) z_put(u0 + i * NT + tid, v[i], m[i]);
        }
        WG_STAMP(5 + 8 * it_);
        __syncthreads();
        WG_STAMP(6 + 8 * it_);
        const float *xrow = xs + (8 * kq + ky * p.XW) * p.XS + cc;
        const u32x4_t *zrow = (const u32x4_t *)zp + (c * QS2 + 4 * kq) / 4;  // this lane's filter is c (= lane % 32)
        const int n_bt = (th * p.XW + 15) >> 4;
        for (int bt = 0; bt < n_bt; ++bt) {
            float w[WIN];
#pragma unroll
            for (int e = 0; e < WIN; ++e) w[e] = xrow[(16 * bt + e) * p.XS];
            const u32x4_t b0 = zrow[2 * bt], b1 = zrow[8 * QS2 + 2 * bt], b2 = zrow[16 * QS2 + 2 * bt];
            uint32_t low = 0u;
#pragma unroll
            for (int e = 0; e < WIN; ++e) low |= __float_as_uint(w[e]);
            if (!__any(c_counts && (low & 0xffffu) != 0u)) {
#pragma unroll
                for (int kx = 0; kx < KW; ++kx) {
                    u32x4_t a;
#pragma unroll
                    for (int e = 0; e < 4; ++e) a[e] = bf16_pair(__float_as_uint(w[kx + 2 * e]), __float_as_uint(w[kx + 2 * e + 1]));
                    acc[kx] = mfma_bf16(a, b0, acc[kx]);
                    acc[kx] = mfma_bf16(a, b1, acc[kx]);
                    acc[kx] = mfma_bf16(a, b2, acc[kx]);
                }
            } else {
                uint32_t ph[WIN], pm[WIN], pl[WIN], third = 0u;
#pragma unroll
                for (int e = 0; e < WIN; ++e) {
                    bf16_parts(w[e], ph[e], pm[e], pl[e]);
                    third |= pl[e];
                }
                const bool three = __any(c_counts && third != 0u);
#pragma unroll
                for (int kx = 0; kx < KW; ++kx) {
                    u32x4_t a0, a1, a2;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        a0[e] = bf16_pair(ph[kx + 2 * e], ph[kx + 2 * e + 1]);
                        a1[e] = bf16_pair(pm[kx + 2 * e], pm[kx + 2 * e + 1]);
                        a2[e] = bf16_pair(pl[kx + 2 * e], pl[kx + 2 * e + 1]);
                    }
                    acc[kx] = mfma_bf16(a0, b0, acc[kx]), acc[kx] = mfma_bf16(a0, b1, acc[kx]), acc[kx] = mfma_bf16(a0, b2, acc[kx]);
                    acc[kx] = mfma_bf16(a1, b0, acc[kx]), acc[kx] = mfma_bf16(a1, b1, acc[kx]), acc[kx] = mfma_bf16(a1, b2, acc[kx]);
                    if (three) {
                        acc[kx] = mfma_bf16(a2, b0, acc[kx]), acc[kx] = mfma_bf16(a2, b1, acc[kx]), acc[kx] = mfma_bf16(a2, b2, acc[kx]);
                    }
                }
            }
        }
    }
    WG_STAMP(30);
    float *my = part + (int64_t)blockIdx.x * ((int64_t)KH * KW * g.C * F + F);
    if (c < F) {  // result column = filter
#pragma unroll
        for (int kx = 0; kx < KW; ++kx)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int ch = pg_acc_row(r, lane);
                if (ch < g.C) my[(int64_t)((ky * KW + kx) * g.C + ch) * F + c] = acc[kx][r];
            }
    }
    // bias gradient: the threads that stage the same four filters add up in a fixed order
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 4; ++j) lds[tid * 4 + j] = bsum[j];
    __syncthreads();
    if (tid < 32 && tid < F) {
        float sacc = 0.f;
        for (int u = 0; u < NT / 8; ++u) sacc += lds[(u * 8 + (tid >> 2)) * 4 + (tid & 3)];
        my[(int64_t)KH * KW * g.C * F + tid] = sacc;
    }
    WG_STAMP(31);
}

#define WG_MAX_LDS (53 * 1024)  // three workgroups per CU

static bool plan_wgrad(const hgq_conv_geom &g, int F, WgPlan &p, size_t &lds) {
    if (!((g.kh == 3 && g.kw == 3) || (g.kh == 5 && g.kw == 5))) return false;
    if (g.sy != 1 || g.sx != 1 || g.dly != 1 || g.dlx != 1) return false;
    if (g.C % 4 != 0 || g.C > 32 || F % 4 != 0 || F > 32 || g.B < 1) return false;
    if ((int64_t)g.B * g.H * g.W * g.C * 4 >= (1ll << 31) || (int64_t)g.B * g.OH * g.OW * F * 4 >= (1ll << 31)) return false;
    p.XW = g.OW + g.kw - 1;
    p.XS = (g.C & 7) == 4 ? g.C : g.C + 4;  // 8 * XS = 32 (mod 64) words: the two halves of a wavefront read disjoint banks
    for (int th = g.OH; th >= 1; th = th > 1 ? (th + 1) / 2 : 0) {
        p.TH = th, p.bands = (g.OH + th - 1) / th, p.XH = th + g.kh - 1;
        p.QN = (th * p.XW + 15) & ~15, p.QS = p.QN + 8;
        p.XP = p.QN + (g.kh - 1) * p.XW + g.kw - 1;
        if (p.XP < p.XH * p.XW) p.XP = p.XH * p.XW;
        if (p.XP * (g.C / 4) >= (1 << 20) || p.QN >= (1 << 20)) continue;
        lds = (size_t)p.XP * p.XS * 4 + (size_t)3 * 32 * p.QS * 2;
        if (lds < (size_t)64 * g.kh * 16) lds = (size_t)64 * g.kh * 16;  // the bias sums of the last step
        if (lds <= WG_MAX_LDS) return true;
    }
    return false;
}

bool conv_patch_wgrad_ok(const hgq_conv_geom &g, int F) {
    WgPlan p;
    size_t lds;
    return hgq_dense_use_bf16_parts(-1) != 0 && plan_wgrad(g, F, p, lds);
}

int conv_patch_wgrad_slices(const hgq_conv_geom &g, int F) {
    WgPlan p;
    size_t lds;
    if (!plan_wgrad(g, F, p, lds)) return 0;
    return persistent_grid((int64_t)g.B * p.bands, 2);
}

int conv_patch_wgrad_launch(const float *x, const float *dy, const float *mask, float *part, const hgq_conv_geom &g, int F, int act,
                            hipStream_t s) {
    WgPlan p;
    size_t lds;
    if (!plan_wgrad(g, F, p, lds)) return fail(HGQ_ERR_UNSUPPORTED, "conv_patch_wgrad_launch: shape not covered");
    const dim3 grid((unsigned)conv_patch_wgrad_slices(g, F));
    const int relu = act == HGQ_ACT_RELU && mask != nullptr;
    if (g.kh == 3) hipLaunchKernelGGL((wgrad_patch_kernel<3, 3>), grid, dim3(192), lds, s, x, dy, mask, part, g, F, relu, p);
    else hipLaunchKernelGGL((wgrad_patch_kernel<5, 5>), grid, dim3(320), lds, s, x, dy, mask, part, g, F, relu, p);
    return check_launch("conv_patch_wgrad_launch");
}

}  // namespace hgq
