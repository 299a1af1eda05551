// The attention core of QMultiHeadAttention as one pass each way:
//
//   scores[b, n, t, s] = sum_h query[b, t, n, h] key[b, s, n, h]
//   probs              = table softmax over s (hgq_softmax_dev.h: five quantizers, trackers)
//   out[b, t, n, h]    = sum_s probs[b, n, t, s] value[b, s, n, h]
//
// The [B, N, T, S] tensors never reach memory: the backward pass recomputes scores and softmax
// from query / key / value.  query / key / value / out keep the projections' layout
// [B, seq, N, H].
//
// Work decomposition.  A workgroup of eight wavefronts takes one batch element at a time (all of
// its heads, operands staged once in LDS with coalesced 128-bit loads, the next element's already
// in flight) and walks the batch.  Wavefront u owns head u / TH and the 32 query positions
// u % TH of it for the whole walk, so the output quantizer's operands, its abs-max tracker and its
// bit-width gradients stay in registers.  The wavefront computes the TRANSPOSED score tile
// (key position = MFMA row, query position = MFMA column = lane): a softmax row then lives in the
// registers of lanes t and t + 32, so row maximum and sums are in-register loops plus one
// cross-lane exchange, and the accumulator registers are, as they stand, the B operand of the
// contractions over the key position (out = probs v, dquery = dscores key).  The two contractions
// over the query position (dvalue, dkey) read probs / dscores back from an LDS buffer.
//
// MFMA 32x32x2 fp32 operand layout (64 lanes): A[i][k]: i = lane % 32, k = lane / 32;
// B[k][j]: k = lane / 32, j = lane % 32; D[i][j] in 16 registers: j = lane % 32,
// i = (r / 4) * 8 + (lane / 32) * 4 + (r % 4).  The contraction index of a step is free, so a
// half-wavefront takes one half of the head dimension and reads its operands as 128-bit words.
// Output rows beyond the head size come from whatever the A operand's lanes read; they are never stored.
#include <type_traits>

#include "hgq_softmax_dev.h"

namespace hgq {

#define QA_LD 68    // words between rows of an operand tile in LDS
#define QA_NT 512   // eight wavefronts
#define QA_PAD 64   // readable words after the last operand tile

// Time stamps of workgroup 0 in the backward kernel (measurement builds only: -DQA_PROF): [wavefront][element][event], core clock
#ifdef QA_PROF
__device__ unsigned long long qa_prof_stamps[8 * 4 * 16];
#define QA_STAMP(i)                                                                                                       \
    do {                                                                                                                  \
        if (blockIdx.x == 0 && (threadIdx.x & 63) == 0 && it_ < 4) qa_prof_stamps[((threadIdx.x >> 6) * 4 + it_) * 16 + (i)] = clock64(); \
    } while (0)
#else
#define QA_STAMP(i)
#endif

struct QAttnPlan {
    int B, T, S, N;
    int n_wg;         // workgroup w takes batch elements w, w + n_wg, ...
    int64_t P_table;  // rows of the output quantizer's [P_table, S] table; row (n * T + t) % P_table serves (n, t)
    int bf;           // contractions on the bf16 matrix instruction over exact bf16 parts (mfma_batch_bf16), batch by batch
};

// One operand array of a batch element in flight: up to two 128-bit words per thread.
struct Stage {
    __amdgpu_buffer_rsrc_t rs;
    uint32_t n4;      // 128-bit words per batch element
    uint32_t row4;    // 128-bit words per row
    __device__ __forceinline__ void init(const float *base, int B, int rows, int row_len) {
        rs = buf_rsrc(base, (int64_t)B * rows * row_len * 4);
        n4 = (uint32_t)(rows * row_len) >> 2, row4 = (uint32_t)row_len >> 2;
    }
    __device__ __forceinline__ void fetch(f32x4_t (&r)[2], int b, bool live) const {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const uint32_t i4 = threadIdx.x + u * QA_NT;
            const bool ok = live && i4 < n4;
            r[u] = buf_ld4(rs, ok ? ((uint32_t)b * n4 + i4) * 16u : BUF_OOB);
        }
    }
    // idle slots write their zeros to the sink row after the tile
    __device__ __forceinline__ void stash(float *tile, int sink_row, const f32x4_t (&r)[2]) const {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const uint32_t i4 = threadIdx.x + u * QA_NT;
            const uint32_t row = i4 / row4, c4 = i4 - row * row4;
            const bool ok = i4 < n4;
            *(f32x4_t *)(tile + (ok ? row * QA_LD + c4 * 4 : (uint32_t)sink_row * QA_LD + (threadIdx.x & 15) * 4)) = r[u];
        }
    }
};

__device__ __forceinline__ float xor32(float v) { return __shfl_xor(v, 32); }

// Key position of accumulator register r of score tile st in this half-wavefront.
__device__ __forceinline__ int qa_row(int st, int r, int hf) { return st * 32 + (r >> 2) * 8 + hf * 4 + (r & 3); }

// Transposed score tile of one head: acc[st][r] = sum_h key[s][h] query[t][h], s = qa_row(st, r, hf), t = t0 + lane % 32.
// bf: sixteen contraction steps at a time through mfma_batch_bf16 (FULL_B: b_tile holds a gradient).
template <int HD, int ST, bool FULL_B = false>
__device__ __forceinline__ void score_tiles(const float *a_tile, const float *b_tile, int t0, int col0, int t_l, int hf, floatx16 (&acc)[ST],
                                            bool bf = false) {
    constexpr int HH = HD / 2;
    float b[HH];
#pragma unroll
    for (int g = 0; g < HH / 4; ++g) {
        const f32x4_t v = *(const f32x4_t *)(b_tile + (t0 + t_l) * QA_LD + col0 + hf * HH + 4 * g);
        b[4 * g] = v.x, b[4 * g + 1] = v.y, b[4 * g + 2] = v.z, b[4 * g + 3] = v.w;
    }
#pragma unroll
    for (int st = 0; st < ST; ++st) {
        float a[HH];
#pragma unroll
        for (int g = 0; g < HH / 4; ++g) {
            const f32x4_t v = *(const f32x4_t *)(a_tile + (st * 32 + t_l) * QA_LD + col0 + hf * HH + 4 * g);
            a[4 * g] = v.x, a[4 * g + 1] = v.y, a[4 * g + 2] = v.z, a[4 * g + 3] = v.w;
        }
        floatx16 c = {0};
        if (HH % 8 == 0 && bf) {
#pragma unroll
            for (int j0 = 0; j0 < HH; j0 += 8) {
                float a8[8], b8[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) a8[j] = a[(j0 + j) % HH], b8[j] = b[(j0 + j) % HH];
                c = mfma_batch_bf16<false, FULL_B>(c, a8, b8);
            }
        } else {
#pragma unroll
            for (int j = 0; j < HH; ++j) c = __builtin_amdgcn_mfma_f32_32x32x2f32(a[j], b[j], c, 0, 0, 0);
        }
        acc[st] = c;
    }
}

// D[h][t] = sum_s tile[s][col0 + h] * acc[s][t]: the accumulator registers are the B operand as they stand.
// bf: sixteen contraction steps at a time through mfma_batch_bf16 (FULL_B: the accumulators hold a gradient).
template <int ST, bool FULL_B = false>
__device__ __forceinline__ floatx16 contract_keys(const float *tile, int col0, int t_l, int hf, const floatx16 (&acc)[ST], bool bf = false,
                                                  int hd = 32) {
    floatx16 o = {0};
#pragma unroll
    for (int st = 0; st < ST; ++st) {
        float a[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) a[r] = tile[qa_row(st, r, hf) * QA_LD + col0 + t_l];
        if (bf) {
#pragma unroll
            for (int r0 = 0; r0 < 16; r0 += 8) {
                float a8[8], b8[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) a8[j] = a[r0 + j], b8[j] = acc[st][r0 + j];
                o = mfma_batch_bf16<false, FULL_B>(o, a8, b8, t_l < hd);  // lanes past the head size feed rows nobody reads
            }
        } else {
#pragma unroll
            for (int r = 0; r < 16; ++r) o = __builtin_amdgcn_mfma_f32_32x32x2f32(a[r], acc[st][r], o, 0, 0, 0);
        }
    }
    return o;
}

// D[h][s] = sum_t tile[t][col0 + h] * buf[t][s0 + s], t < 32 * TH (buf rows are QA_LD words apart).  A step pairs
// rows t and t + 8: 8 * QA_LD = 32 (mod 64) words, so the two half-wavefronts read disjoint banks.
// bf: sixteen contraction steps at a time through mfma_batch_bf16 (FULL_A / FULL_B: tile / buf holds a gradient).
template <int TH, bool FULL_A = false, bool FULL_B = false>
__device__ __forceinline__ floatx16 contract_queries(const float *tile, int col0, const float *buf, int s0, int t_l, int hf, bool bf = false,
                                                     int hd = 32) {
    floatx16 o = {0};
#pragma unroll
    for (int j0 = 0; j0 < 16 * TH; j0 += 16) {
        float a[16], b[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const int t = 2 * j0 + (j >> 3) * 16 + (j & 7) + 8 * hf;
            a[j] = tile[t * QA_LD + col0 + t_l];
            b[j] = buf[t * QA_LD + s0 + t_l];
        }
        if (bf) {
#pragma unroll
            for (int h0 = 0; h0 < 16; h0 += 8) {
                float a8[8], b8[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) a8[j] = a[h0 + j], b8[j] = b[h0 + j];
                o = mfma_batch_bf16<FULL_A, FULL_B>(o, a8, b8, t_l < hd);
            }
        } else {
#pragma unroll
            for (int j = 0; j < 16; ++j) o = __builtin_amdgcn_mfma_f32_32x32x2f32(a[j], b[j], o, 0, 0, 0);
        }
    }
    return o;
}

// Rows d < HD of a transposed result (row = head channel, column = position) to dst[pos][d]: four
// consecutive channels per register group.
template <int HD>
__device__ __forceinline__ void store_rows(const floatx16 &o, float *__restrict__ dst, int64_t pos_stride, int pos, int hf) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const int d0 = 8 * g + 4 * hf;
        if (d0 < HD) {
            f32x4_t v;
            v.x = o[4 * g], v.y = o[4 * g + 1], v.z = o[4 * g + 2], v.w = o[4 * g + 3];
            *(f32x4_t *)(dst + (int64_t)pos * pos_stride + d0) = v;
        }
    }
}

// One accumulator tile of a wavefront into its [32 positions][S] block of buf (row = lane % 32).
__device__ __forceinline__ void spill_tile(float *buf, int st, const floatx16 &acc, int t_l, int hf) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        f32x4_t v;
        v.x = acc[4 * g], v.y = acc[4 * g + 1], v.z = acc[4 * g + 2], v.w = acc[4 * g + 3];
        *(f32x4_t *)(buf + t_l * QA_LD + st * 32 + 8 * g + 4 * hf) = v;
    }
}

// The accumulator tiles of a wavefront as a [32 positions][S] block of buf (row = lane % 32).
template <int ST>
__device__ __forceinline__ void spill_tiles(float *buf, const floatx16 (&acc)[ST], int t_l, int hf) {
#pragma unroll
    for (int st = 0; st < ST; ++st)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            f32x4_t v;
            v.x = acc[st][4 * g], v.y = acc[st][4 * g + 1], v.z = acc[st][4 * g + 2], v.w = acc[st][4 * g + 3];
            *(f32x4_t *)(buf + t_l * QA_LD + st * 32 + 8 * g + 4 * hf) = v;
        }
}

// ---- attention masks (reference src/hgq/layers/softmax.py:118-127: scores <- mask * scores - (1 - mask) * 1e9 ahead of
// the maximum, exp <- mask * exp behind the table).  A lane keeps one bit per score it owns: bit r of keep[st] is
// clear where (query t, key qa_row(st, r, hf)) is masked out - by the boolean mask [mask_batch, T, S] (one byte per
// entry, 0 = masked; four consecutive keys per 32-bit load) and / or by the causal rule key <= query.
#define QA_MASKED (-1e9f)
struct QAttnMask {
    const uint8_t *mask;  // null: no boolean mask
    int mask_batch;       // 1: the same mask for every batch element, else B
    int causal;
};

template <int ST>
__device__ __forceinline__ void load_keep(const QAttnMask &mk, int b, int T, int S, int t, int hf, uint32_t (&keep)[ST]) {
#pragma unroll
    for (int st = 0; st < ST; ++st) keep[st] = 0xffffu;
    if (mk.mask) {
        const uint8_t *row = mk.mask + ((int64_t)(mk.mask_batch > 1 ? b : 0) * T + t) * S;
        uint32_t w[ST][4];
#pragma unroll
        for (int st = 0; st < ST; ++st)
#pragma unroll
            for (int g = 0; g < 4; ++g) w[st][g] = *(const uint32_t *)(row + st * 32 + 8 * g + 4 * hf);
#pragma unroll
        for (int st = 0; st < ST; ++st)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                if (((w[st][r >> 2] >> (8 * (r & 3))) & 0xffu) == 0) keep[st] &= ~(1u << r);
    }
    if (mk.causal) {
#pragma unroll
        for (int st = 0; st < ST; ++st)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                if (qa_row(st, r, hf) > t) keep[st] &= ~(1u << r);
    }
}

// ---- the exp stage.  The walk keeps only what turns d = max - x into a table code (ExpCode); the
// table holds the rest.  Arguments the table does not cover - codes beyond SM_TABLE, an exp input
// quantizer with an empty range - are rare and go through out-of-line functions that rebuild the
// two quantizers from their descriptors, which keeps some forty wavefront-uniform values out of
// the loop (they do not fit the scalar registers and would each take a vector register).
struct ExpCode {
    int fi;
    float rc, code_max, gi_hi, gf_hi;
    bool conv, on, kbi;
    __device__ __forceinline__ void init(const SharedQ &q1, const ExpTable &tab) {
        fi = q1.fi, rc = q1.rc, conv = q1.conv, kbi = q1.kbi, gi_hi = q1.gi_hi, gf_hi = q1.gf_hi;
        on = tab.on, code_max = tab.code_max;
    }
    __device__ __forceinline__ float code_of(float d) const {
        const float t = ldexpf(d, fi);
        return conv ? rintf(t) : floorf(__fadd_rn(t, rc));
    }
    // ExpTable::grad_q1 on the kept values
    __device__ __forceinline__ void grad_q1(float d, float r, float da, float &dd, float &gi, float &gf) const {
        const bool over = r > code_max;
        const float xq = ldexpf(r, -fi);
        dd = over ? 0.f : da;
        gi = over ? gi_hi * da : 0.f;
        gf = over ? gf_hi * da : -HGQ_LN2 * (xq - d) * da;
        if (kbi) gi -= gf;
    }
};

__device__ __noinline__ void exp_direct(hgq_qdesc d1, hgq_qdesc d2, float scale, float d, float *a, float *e) {
    SharedQ q1, q2;
    q1.init(d1), q2.init(d2);
    *a = q1.fwd<true>(d);
    *e = q2.fwd<true>(ExpTable::t_of(*a, scale));
}

// gradients through the exp stage for one element: de = upstream gradient of e
__device__ __noinline__ void exp_direct_grad(hgq_qdesc d1, hgq_qdesc d2, float scale, float d, float de, float *dd, float *g4) {
    SharedQ q1, q2;
    q1.init(d1), q2.init(d2);
    ExpTable tab;
    tab.init(q1);
    float gi1, gf1;
    ExpTable::Entry en;
    if (tab.on) {
        const float r = ExpTable::code_of(d, q1);
        en = ExpTable::entry_of(ldexpf(fminf(r, tab.code_max), -q1.fi), q2, scale);
        tab.grad_q1(d, r, en.ca * de, q1, *dd, gi1, gf1);
    } else {
        en = ExpTable::entry_of(q1.fwd(d), q2, scale);
        q1.grad(d, en.ca * de, *dd, gi1, gf1);
    }
    g4[0] = gi1, g4[1] = gf1, g4[2] = en.ci * de, g4[3] = en.cf * de;
}

// Codes of a tile; true if some lane of the wavefront needs the out-of-line path.
__device__ __forceinline__ bool tile_codes(const floatx16 &x, float mx, const ExpCode &ec, float (&raw)[16], float (&cl)[16]) {
    bool big = false;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        raw[r] = ec.code_of(__fsub_rn(mx, x[r]));
        cl[r] = fminf(raw[r], ec.code_max);
        big |= !(cl[r] < (float)SM_TABLE);
    }
    return !ec.on || __any(big);
}

// x <- e of a training-mode tile; tab = table of e (stride words apart); cmax / m1 track the exp input quantizer's output
__device__ __forceinline__ void exp_tile(const float *tab, int stride, const ExpCode &ec, const hgq_qdesc &d1, const hgq_qdesc &d2,
                                         float scale, float mx, floatx16 &x, float &cmax, uint32_t &m1) {
    float raw[16], cl[16];
    if (!tile_codes(x, mx, ec, raw, cl)) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            cmax = fmaxf(cmax, cl[r]);
            x[r] = tab[(int)cl[r] * stride];
        }
        return;
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        if (ec.on && cl[r] < (float)SM_TABLE) {
            cmax = fmaxf(cmax, cl[r]);
            x[r] = tab[(int)cl[r] * stride];
        } else {
            float a, e;
            exp_direct(d1, d2, scale, __fsub_rn(mx, x[r]), &a, &e);
            m1 = max(m1, abs_bits(a));
            x[r] = e;
        }
    }
}

// The output quantizer's operands of this lane's entries (row `row` of the [P, S] table, key positions
// qa_row(st, r, hf)), packed as LaneQ::load packs them.  Four consecutive entries per 128-bit load, and every
// load is issued before the first value is used: entry-by-entry loads would cost a memory round trip each.
template <int ST>
__device__ __forceinline__ void load_oq_entries(const hgq_qdesc &d, int64_t row, int S, int hf, int (&pk)[ST][16]) {
    const Mode m(d.mode);
    f32x4_t iv[ST][4], fv[ST][4], kf[ST][4];
    uint32_t kb[ST][4];
#pragma unroll
    for (int st = 0; st < ST; ++st)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int64_t off = row * S + st * 32 + 8 * g + 4 * hf;
            iv[st][g] = *(const f32x4_t *)(d.i + off);
            fv[st][g] = *(const f32x4_t *)(d.fb + off);
            if (m.k_u8)
                kb[st][g] = *(const uint32_t *)((const uint8_t *)d.k + off);
            else
                kf[st][g] = *(const f32x4_t *)((const float *)d.k + off);
        }
#pragma unroll
    for (int st = 0; st < ST; ++st)
#pragma unroll
        for (int g = 0; g < 4; ++g)
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const float kk = m.k_u8 ? (float)((kb[st][g] >> (8 * c)) & 0xff) : kf[st][g][c];
                const KIF p = resolve_kif(kk, iv[st][g][c], fv[st][g][c], m.kbi, m.round_params);
                pk[st][4 * g + c] = (LaneQ::clamp8(p.f) & 0xff) | ((LaneQ::clamp8(p.i) & 0xff) << 8) | (p.k != 0.f ? 1 << 16 : 0);
            }
}

// OQ_PLAIN: training mode and an output quantizer that only rounds (or none): its fractional bits are
// packed four to a register; otherwise (k, i, f) take a register per element.
template <int HD, int TH, int ST, bool TRAIN, bool OQ_PLAIN, bool MASKED>
__global__ __launch_bounds__(QA_NT) void qattn_fwd_kernel(const float *__restrict__ q, const float *__restrict__ k,
                                                          const float *__restrict__ v, float *__restrict__ out, QAttnPlan pl,
                                                          float scale, float eps, hgq_qdesc d1, hgq_qdesc d2, hgq_qdesc d3,
                                                          hgq_qdesc d4, hgq_qdesc dq, uint32_t *amax1, uint32_t *amax3,
                                                          uint32_t *__restrict__ amax_slices, uint32_t *__restrict__ pair_slices,
                                                          QAttnMask mk) {
    static_assert(TRAIN || !OQ_PLAIN, "the packed form is for training mode");
    extern __shared__ __align__(16) float lds[];
    constexpr int T = 32 * TH, S = 32 * ST, NPO = OQ_PLAIN ? 4 : 16;
    float *Qs = lds, *Ks = Qs + (T + 1) * QA_LD, *Vs = Ks + (S + 1) * QA_LD;
    float *tab_e = Vs + (S + 1) * QA_LD + QA_PAD;
    __shared__ uint32_t lds_m13[QA_NT / 64][2];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, t_l = lane & 31, hf = lane >> 5;
    const int h = wave / TH, th = wave % TH;
    const bool active = h < pl.N;
    const int RL = pl.N * HD, col0 = h * HD, t0 = th * 32;
    const int table_row = (int)((int64_t)(h * T + t0 + t_l) % pl.P_table);

    SharedQ q3, q4;
    q3.init(d3), q4.init(d4);
    LaneQ qo;
    qo.init(dq);
    int po[ST][NPO];
    uint32_t mo[ST][16];
    {
        int pk_[ST][16];
#pragma unroll
        for (int st = 0; st < ST; ++st)
#pragma unroll
            for (int r = 0; r < 16; ++r) pk_[st][r] = 0, mo[st][r] = 0;
        if (qo.present && active) load_oq_entries<ST>(dq, table_row, S, hf, pk_);
#pragma unroll
        for (int st = 0; st < ST; ++st) {
#pragma unroll
            for (int j = 0; j < NPO; ++j) po[st][j] = 0;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                if (OQ_PLAIN)
                    po[st][r >> 2] |= (LaneQ::f_of(pk_[st][r]) & 0xff) << (8 * (r & 3));
                else
                    po[st][r % NPO] = pk_[st][r];
            }
        }
    }
    ExpCode ec;
    {
        SharedQ q1, q2;
        q1.init(d1), q2.init(d2);
        ExpTable tab;
        tab.on = false, tab.code_max = INFINITY;
        if (TRAIN) tab.build_fwd(tab_e, q1, q2, scale);
        ec.init(q1, tab);
    }
    uint32_t m1 = 0, m3 = 0;
    float cmax = 0.f;

    Stage sq_, sk_, sv_;
    sq_.init(q, pl.B, T, RL), sk_.init(k, pl.B, S, RL), sv_.init(v, pl.B, S, RL);
    f32x4_t pq[2], pk[2], pv[2];
    floatx16 o_prev = {0};
    int b_prev = -1;
    int b = blockIdx.x;
    sq_.fetch(pq, b, b < pl.B), sk_.fetch(pk, b, b < pl.B), sv_.fetch(pv, b, b < pl.B);
    for (; b < pl.B; b += pl.n_wg) {
        __syncthreads();  // the previous element's tiles are no longer read
        sq_.stash(Qs, T, pq), sk_.stash(Ks, S, pk), sv_.stash(Vs, S, pv);
        const int nb = b + pl.n_wg;
        sq_.fetch(pq, nb, nb < pl.B), sk_.fetch(pk, nb, nb < pl.B), sv_.fetch(pv, nb, nb < pl.B);
        __syncthreads();
        if (!active) continue;
        // the previous element's output leaves here, a whole element ahead of the wait at the top of the walk
        // (that wait covers every outstanding memory operation, stores included)
        if (b_prev >= 0) store_rows<HD>(o_prev, out + ((int64_t)b_prev * T * pl.N + h) * HD, (int64_t)pl.N * HD, t0 + t_l, hf);
        // the packed operands stay packed: without this the unpacking is hoisted out of the walk and
        // every element's fractional bits (and their negation) take a register for the whole kernel
#pragma unroll
        for (int st = 0; st < ST; ++st)
#pragma unroll
            for (int j = 0; j < NPO; ++j) asm volatile("" : "+v"(po[st][j]));
        uint32_t keep[ST];
        if (MASKED) load_keep<ST>(mk, b, T, S, t0 + t_l, hf, keep);  // (its loads travel with the contraction below)
        floatx16 acc[ST];
        score_tiles<HD, ST>(Ks, Qs, t0, col0, t_l, hf, acc, pl.bf != 0);
        if (MASKED) {
#pragma unroll
            for (int st = 0; st < ST; ++st)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[st][r] = ((keep[st] >> r) & 1u) ? acc[st][r] : QA_MASKED;
        }
        float mx = acc[0][0];
#pragma unroll
        for (int st = 0; st < ST; ++st)
#pragma unroll
            for (int r = 0; r < 16; ++r) mx = fmaxf(mx, acc[st][r]);
        mx = fmaxf(mx, xor32(mx));
        if (TRAIN && MASKED) {
            // a masked score sits 1e9 below the maximum, far outside the table: it takes the table's place of the maximum
            // (code 0) and its exp is replaced by zero; what the exp input quantizer makes of it only matters to its tracker
            bool any_masked = false;
#pragma unroll
            for (int st = 0; st < ST; ++st) {
                floatx16 xm;
#pragma unroll
                for (int r = 0; r < 16; ++r) xm[r] = ((keep[st] >> r) & 1u) ? acc[st][r] : mx;
                exp_tile(tab_e, 1, ec, d1, d2, scale, mx, xm, cmax, m1);
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[st][r] = ((keep[st] >> r) & 1u) ? xm[r] : 0.f;
                any_masked |= keep[st] != 0xffffu;
            }
            if (amax1 && any_masked && mx > QA_MASKED) {
                float a, e;
                exp_direct(d1, d2, scale, __fsub_rn(mx, QA_MASKED), &a, &e);
                m1 = max(m1, abs_bits(a));
            }
        } else if (TRAIN) {
#pragma unroll
            for (int st = 0; st < ST; ++st) exp_tile(tab_e, 1, ec, d1, d2, scale, mx, acc[st], cmax, m1);
        } else {
            SharedQ q1, q2;
            q1.init(d1), q2.init(d2);
#pragma unroll
            for (int st = 0; st < ST; ++st)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const float a = q1.fwd<false>(__fsub_rn(mx, acc[st][r]));
                    m1 = max(m1, abs_bits(a));
                    acc[st][r] = q2.fwd<false>(ExpTable::t_of(a, scale));
                    if (MASKED && !((keep[st] >> r) & 1u)) acc[st][r] = 0.f;
                    if ((r & 3) == 3) __builtin_amdgcn_sched_barrier(0);
                }
        }
        float s = 0.f;
#pragma unroll
        for (int st = 0; st < ST; ++st)
#pragma unroll
            for (int r = 0; r < 16; ++r) s += acc[st][r];
        s += xor32(s);
        const float sq = q3.fwd<TRAIN>(s);
        const float rr = q4.fwd<TRAIN>(__fdiv_rn(1.0f, __fadd_rn(sq, eps)));
        m3 = max(m3, abs_bits(sq));
        // the output quantizer of an element, then its step of out = probs value: the MFMA of one element runs
        // while the next one is quantized (the presence test is hoisted: no branch between the elements)
        floatx16 o = {0};
        if (qo.present && pl.bf) {
            // eight quantized probabilities at a time, then their sixteen contraction steps as one batch
#pragma unroll
            for (int st = 0; st < ST; ++st) {
                float a[16];
#pragma unroll
                for (int r = 0; r < 16; ++r) a[r] = Vs[qa_row(st, r, hf) * QA_LD + col0 + t_l];
#pragma unroll
                for (int r0 = 0; r0 < 16; r0 += 8) {
                    float a8[8], y8[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        const int r = r0 + j;
                        float y = __fmul_rn(acc[st][r], rr);
                        if (OQ_PLAIN)
                            y = qo.round_at(y, (int)(int8_t)((po[st][r >> 2] >> (8 * (r & 3))) & 0xff));
                        else
                            y = qo.fwd<TRAIN>(y, po[st][r % NPO]);
                        mo[st][r] = max(mo[st][r], abs_bits(y));
                        a8[j] = a[r], y8[j] = y;
                    }
                    o = mfma_batch_bf16<false, false>(o, a8, y8, t_l < HD);  // lanes past the head size feed rows nobody reads
                }
            }
        } else if (qo.present) {
#pragma unroll
            for (int st = 0; st < ST; ++st) {
                float a[16];
#pragma unroll
                for (int r = 0; r < 16; ++r) a[r] = Vs[qa_row(st, r, hf) * QA_LD + col0 + t_l];
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    float y = __fmul_rn(acc[st][r], rr);
                    if (OQ_PLAIN)
                        y = qo.round_at(y, (int)(int8_t)((po[st][r >> 2] >> (8 * (r & 3))) & 0xff));
                    else
                        y = qo.fwd<TRAIN>(y, po[st][r % NPO]);
                    mo[st][r] = max(mo[st][r], abs_bits(y));
                    o = __builtin_amdgcn_mfma_f32_32x32x2f32(a[r], y, o, 0, 0, 0);
                    if (OQ_PLAIN) {
                        __builtin_amdgcn_sched_group_barrier(0x002, 11, 0);  // VALU of this element
                        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // its MFMA
                    } else if ((r & 3) == 3) {
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
        } else {
#pragma unroll
            for (int st = 0; st < ST; ++st) {
                float a[16];
#pragma unroll
                for (int r = 0; r < 16; ++r) a[r] = Vs[qa_row(st, r, hf) * QA_LD + col0 + t_l];
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const float y = __fmul_rn(acc[st][r], rr);
                    mo[st][r] = max(mo[st][r], abs_bits(y));
                    o = __builtin_amdgcn_mfma_f32_32x32x2f32(a[r], y, o, 0, 0, 0);
                }
            }
        }
        o_prev = o, b_prev = b;
    }
    if (active && b_prev >= 0) store_rows<HD>(o_prev, out + ((int64_t)b_prev * T * pl.N + h) * HD, (int64_t)pl.N * HD, t0 + t_l, hf);
    m1 = max(m1, abs_bits(ldexpf(cmax, -ec.fi)));
    if (amax1 || amax3) {
        m1 = wave_max_bits(m1), m3 = wave_max_bits(m3);
        if (lane == 0) lds_m13[wave][0] = m1, lds_m13[wave][1] = m3;
        __syncthreads();
        if (threadIdx.x < 2) {
            uint32_t m = 0;
            for (int w = 0; w < QA_NT / 64; ++w) m = max(m, lds_m13[w][threadIdx.x]);
            if (pair_slices) {
                // one pair per workgroup behind the output quantizer's slices; the reduction launch folds them (nothing to clear)
                pair_slices[2 * blockIdx.x + threadIdx.x] = m;
            } else {
                uint32_t *dst = threadIdx.x == 0 ? amax1 : amax3;
                if (dst) atomicMax(dst, m);
            }
        }
    }
    if (amax_slices && active) {
        // every (head, query, key) entry has one owner in the workgroup: a slice per workgroup, no atomics
        uint32_t *dst = amax_slices + ((int64_t)blockIdx.x * pl.N * T + h * T + t0 + t_l) * S;
#pragma unroll
        for (int st = 0; st < ST; ++st)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                uint4 m4;
                m4.x = mo[st][4 * g], m4.y = mo[st][4 * g + 1], m4.z = mo[st][4 * g + 2], m4.w = mo[st][4 * g + 3];
                *(uint4 *)(dst + st * 32 + 8 * g + 4 * hf) = m4;
            }
    }
}

// amax_o[p * S + s] = max over the workgroups' slices and over the walked rows r = p (mod P) of slices[wg][r][s];
// a block takes 64 entries, its 16 thread groups share the (slice, row) pairs.
// pairs (may be null): [n_slices][2] maxima of the two scalar trackers, folded into amax1 / amax3 by the first workgroup
__global__ __launch_bounds__(1024) void qattn_amax_reduce_kernel(const uint32_t *__restrict__ slices, int n_slices, int64_t rows,
                                                                 int S, int64_t P, uint32_t *__restrict__ amax_o,
                                                                 const uint32_t *__restrict__ pairs, uint32_t *amax1, uint32_t *amax3) {
    __shared__ uint32_t red[1024];
    const int t = threadIdx.x, e_local = t & 63, grp = t >> 6;
    if (pairs && blockIdx.x == 0 && t < 128) {
        // wavefront 0 takes the first tracker, wavefront 1 the second
        const int which = t >> 6;
        uint32_t pm = 0;
        for (int i = t & 63; i < n_slices; i += 64) pm = max(pm, pairs[2 * i + which]);
        pm = wave_max_bits(pm);
        uint32_t *dst = which == 0 ? amax1 : amax3;
        if ((t & 63) == 0 && dst) dst[0] = pm;
    }
    const int64_t e = (int64_t)blockIdx.x * 64 + e_local, M = P * S, fold = rows / P;
    uint32_t m = 0;
    if (e < M) {
        const int64_t p = e / S, s = e - p * S;
        // eight loads in flight per thread
        const int64_t n_it = (int64_t)n_slices * fold;
        int64_t it = grp;
        for (; it + 7 * 16 < n_it; it += 8 * 16) {
            uint32_t v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int64_t iu = it + u * 16, sl = iu / fold, r = p + (iu - sl * fold) * P;
                v[u] = slices[(sl * rows + r) * S + s];
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) m = max(m, v[u]);
        }
        for (; it < n_it; it += 16) {
            const int64_t sl = it / fold, r = p + (it - sl * fold) * P;
            m = max(m, slices[(sl * rows + r) * S + s]);
        }
    }
    red[t] = m;
    __syncthreads();
    for (int o = 512; o >= 64; o >>= 1) {
        if (t < o) red[t] = max(red[t], red[t + o]);
        __syncthreads();
    }
    if (t < 64 && e < M) amax_o[e] = red[t];
}

// Backward: slices of the bit-width gradients go to the workspace in the softmax kernels' layout
// ([n_wg, 8] shared-quantizer sums | [n_wg, N * T * S] d/df of the output quantizer).  The output
// quantizer, if present, wraps (only rounds in training): its input gradient is the identity and
// only its fractional bits take gradient; they are packed four to a register.
// BF: the contractions on the bf16 matrix instruction (exact parts) or on the fp32 one - a template argument, not a branch:
// with both forms in one kernel the register allocation spilled 80 bytes per lane more
template <int HD, int TH, int ST, bool MASKED, bool BF>
__global__ __launch_bounds__(QA_NT) void qattn_bwd_kernel(const float *__restrict__ dout, const float *__restrict__ q,
                                                          const float *__restrict__ k, const float *__restrict__ v,
                                                          float *__restrict__ dq_, float *__restrict__ dk_, float *__restrict__ dv_,
                                                          QAttnPlan pl, float scale, float eps, hgq_qdesc d1, hgq_qdesc d2,
                                                          hgq_qdesc d3, hgq_qdesc d4, hgq_qdesc dq, float *__restrict__ ws,
                                                          QAttnMask mk) {
    extern __shared__ __align__(16) float lds[];
    constexpr int T = 32 * TH, S = 32 * ST, NW = QA_NT / 64;
    float *Qs = lds, *Ks = Qs + (T + 1) * QA_LD, *Vs = Ks + (S + 1) * QA_LD, *Gs = Vs + (S + 1) * QA_LD;
    float *Pm = Gs + (T + 1) * QA_LD + QA_PAD;                           // [NW][32][QA_LD]: probs, then dscores
    float *tabp = Pm + NW * 32 * QA_LD;  // [4][SM_TABLE]: planes e, ca, ci, cf of the exp stage's table
    float *tab_e = tabp;
    __shared__ float part[NW][8];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, t_l = lane & 31, hf = lane >> 5;
    const int h = wave / TH, th = wave % TH;
    const bool active = h < pl.N;
    const int RL = pl.N * HD, col0 = h * HD, t0 = th * 32;
    float *my_buf = Pm + wave * 32 * QA_LD;
    const float *head_buf = Pm + (h * TH) * 32 * QA_LD;  // the T rows of this head
    const int table_row = (int)((int64_t)(h * T + t0 + t_l) % pl.P_table);

    SharedQ q3, q4;
    q3.init(d3), q4.init(d4);
    LaneQ qo;
    qo.init(dq);
    int pf[ST][4];  // fractional bits of the output quantizer, element r of a tile in byte r % 4 of pf[st][r / 4]
    float gof[ST][16];
    {
        int pk_[ST][16];
#pragma unroll
        for (int st = 0; st < ST; ++st)
#pragma unroll
            for (int r = 0; r < 16; ++r) pk_[st][r] = 0, gof[st][r] = 0.f;
        if (qo.present && active) load_oq_entries<ST>(dq, table_row, S, hf, pk_);
#pragma unroll
        for (int st = 0; st < ST; ++st)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                pf[st][g] = 0;
#pragma unroll
                for (int c = 0; c < 4; ++c) pf[st][g] |= (LaneQ::f_of(pk_[st][4 * g + c]) & 0xff) << (8 * c);
            }
    }
    float gs[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) gs[j] = 0.f;
    ExpCode ec;
    {
        SharedQ q1, q2;
        q1.init(d1), q2.init(d2);
        ExpTable tab;
        tab.build_bwd(tabp, q1, q2, scale);
        ec.init(q1, tab);
    }

    Stage sq_, sk_, sv_, sg_;
    sq_.init(q, pl.B, T, RL), sk_.init(k, pl.B, S, RL), sv_.init(v, pl.B, S, RL), sg_.init(dout, pl.B, T, RL);
    f32x4_t pq[2], pk[2], pv[2], pg[2];
    floatx16 dk_prev = {0};
    int b_prev = -1;
    int b = blockIdx.x;
    sq_.fetch(pq, b, b < pl.B), sk_.fetch(pk, b, b < pl.B), sv_.fetch(pv, b, b < pl.B), sg_.fetch(pg, b, b < pl.B);
    int it_ = 0;
    for (; b < pl.B; b += pl.n_wg, ++it_) {
        QA_STAMP(0);
        __syncthreads();  // the previous element's tiles and buffers are no longer read
        QA_STAMP(1);
        sq_.stash(Qs, T, pq), sk_.stash(Ks, S, pk), sv_.stash(Vs, S, pv), sg_.stash(Gs, T, pg);
        __syncthreads();
        QA_STAMP(2);
        // the previous element's dkey leaves here, well ahead of the wait at the top of the walk
        if (active && b_prev >= 0) {
#pragma unroll
            for (int st = 0; st < ST; ++st)
                if (st % TH == th) store_rows<HD>(dk_prev, dk_ + ((int64_t)b_prev * S * pl.N + h) * HD, (int64_t)pl.N * HD, st * 32 + t_l, hf);
        }
        floatx16 xs[ST], ga[ST];
        float mx = 0.f, rr = 0.f, ds = 0.f;
        // the packed fractional bits stay packed (see the forward kernel)
#pragma unroll
        for (int st = 0; st < ST; ++st)
#pragma unroll
            for (int g = 0; g < 4; ++g) asm volatile("" : "+v"(pf[st][g]));
        uint32_t keep[ST];
        if (MASKED) {
#pragma unroll
            for (int st = 0; st < ST; ++st) keep[st] = 0xffffu;
        }
        if (active) {
            if (MASKED) load_keep<ST>(mk, b, T, S, t0 + t_l, hf, keep);
            score_tiles<HD, ST>(Ks, Qs, t0, col0, t_l, hf, xs, BF);        // scores, transposed
            score_tiles<HD, ST, true>(Vs, Gs, t0, col0, t_l, hf, ga, BF);  // d probs = dout value^T, transposed
            QA_STAMP(3);
            if (MASKED) {
#pragma unroll
                for (int st = 0; st < ST; ++st)
#pragma unroll
                    for (int r = 0; r < 16; ++r) xs[st][r] = ((keep[st] >> r) & 1u) ? xs[st][r] : QA_MASKED;
            }
            // ---- forward chain: e of every element (kept in the wavefront's buffer), row sum, inverse stage
            mx = xs[0][0];
#pragma unroll
            for (int st = 0; st < ST; ++st)
#pragma unroll
                for (int r = 0; r < 16; ++r) mx = fmaxf(mx, xs[st][r]);
            mx = fmaxf(mx, xor32(mx));
            float s = 0.f;
            {
                float cmax = 0.f;
                uint32_t m1 = 0;
#pragma unroll
                for (int st = 0; st < ST; ++st) {
                    floatx16 ev = xs[st];
                    if (MASKED) {  // masked scores take the maximum's place in the table and give no exp (see the forward kernel)
#pragma unroll
                        for (int r = 0; r < 16; ++r) ev[r] = ((keep[st] >> r) & 1u) ? ev[r] : mx;
                    }
                    exp_tile(tab_e, 1, ec, d1, d2, scale, mx, ev, cmax, m1);
                    if (MASKED) {
#pragma unroll
                        for (int r = 0; r < 16; ++r) ev[r] = ((keep[st] >> r) & 1u) ? ev[r] : 0.f;
                    }
#pragma unroll
                    for (int r = 0; r < 16; ++r) s += ev[r];
                    spill_tile(my_buf, st, ev, t_l, hf);  // e waits in the buffer where its prob will go
                }
            }
            s += xor32(s);
            QA_STAMP(4);
            const float sq = q3.fwd(s);
            const float r0 = __fdiv_rn(1.0f, __fadd_rn(sq, eps));
            rr = q4.fwd(r0);
            // ---- output quantizer and the product; probs go to the buffer as they are formed.  The round mode is the same for
            // the whole launch: one branch here instead of a select per element.  The fractional-bit gradient keeps its factor
            // -ln 2 for the end of the walk (gof holds sum (p - y0) * dprob).
            float drr = 0.f;
            auto oq_stage = [&](auto conv_tag) {
                constexpr bool CONV = decltype(conv_tag)::value;
#pragma unroll
                for (int st = 0; st < ST; ++st)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        float *slot = my_buf + t_l * QA_LD + st * 32 + 8 * g + 4 * hf;
                        const f32x4_t e4 = *(const f32x4_t *)slot;
                        f32x4_t p4;
#pragma unroll
                        for (int c = 0; c < 4; ++c) {
                            const int r = 4 * g + c;
                            const float y0 = __fmul_rn(e4[c], rr);
                            float p = y0;
                            if (qo.present) {
                                const int fi = (int)(int8_t)((pf[st][g] >> (8 * c)) & 0xff);
                                const float t = ldexpf(y0, fi);
                                p = ldexpf(CONV ? rintf(t) : floorf(__fadd_rn(t, qo.rc)), -fi);
                                gof[st][r] = fmaf(p - y0, ga[st][r], gof[st][r]);
                            }
                            p4[c] = p;
                            drr = fmaf(ga[st][r], e4[c], drr);
                        }
                        *(f32x4_t *)slot = p4;
                    }
            };
            if (qo.conv) oq_stage(std::true_type{});
            else oq_stage(std::false_type{});
            drr += xor32(drr);
            float dr0, gi4, gf4, gi3, gf3;
            q4.grad(r0, drr, dr0, gi4, gf4);
            q3.grad(s, dr0 * -(r0 * r0), ds, gi3, gf3);
            if (hf == 0) gs[6] += gi4, gs[7] += gf4, gs[4] += gi3, gs[5] += gf3;
        }
        QA_STAMP(5);
        __syncthreads();  // probs of every head are in the buffers
        QA_STAMP(6);
        if (active) {
            // dvalue[s][h] = sum_t probs[t][s] dout[t][h]: key-position tile st of a head goes to its wavefront st % TH
#pragma unroll
            for (int st = 0; st < ST; ++st)
                if (st % TH == th) {
                    const floatx16 o = contract_queries<TH, true, false>(Gs, col0, head_buf, st * 32, t_l, hf, BF, HD);
                    store_rows<HD>(o, dv_ + ((int64_t)b * S * pl.N + h) * HD, (int64_t)pl.N * HD, st * 32 + t_l, hf);
                }
            QA_STAMP(7);
            // ---- exp stage and the maximum
            float dm = 0.f, cnt = 0.f;
            // the usual exp input quantizer rounds to nearest (or truncates) and does not saturate: its gradient then has no
            // bound terms, d/df = -ln 2 * sum (a - d) * da (the factor waits for the end of the element) and d/di = 0
            const bool plain = ec.on && !ec.conv && ec.code_max == INFINITY;
            float f1 = 0.f;
#pragma unroll
            for (int st = 0; st < ST; ++st) {
                float raw[16], cl[16];
                floatx16 xm = xs[st];  // masked entries: the maximum's code, and no gradient (their exp was multiplied by zero)
                if (MASKED) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) xm[r] = ((keep[st] >> r) & 1u) ? xm[r] : mx;
                }
                if (plain) {
                    bool big = false;
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        raw[r] = floorf(__fadd_rn(ldexpf(__fsub_rn(mx, xm[r]), ec.fi), ec.rc));
                        big |= !(raw[r] < (float)SM_TABLE);
                    }
                    if (!__any(big)) {
#pragma unroll
                        for (int r0_ = 0; r0_ < 16; r0_ += 4) {
                            ExpTable::Entry en[4];
#pragma unroll
                            for (int j = 0; j < 4; ++j) en[j] = ExpTable::entry_at(tabp, (int)raw[r0_ + j]);
#pragma unroll
                            for (int j = 0; j < 4; ++j) {
                                const int r = r0_ + j;
                                const float d = __fsub_rn(mx, xm[r]);
                                const float de = (!MASKED || ((keep[st] >> r) & 1u)) ? fmaf(ga[st][r], rr, ds) : 0.f;
                                const float da = en[j].ca * de;
                                f1 = fmaf(ldexpf(raw[r], -ec.fi) - d, da, f1);
                                gs[2] = fmaf(en[j].ci, de, gs[2]), gs[3] = fmaf(en[j].cf, de, gs[3]);
                                dm += da;
                                ga[st][r] = da;
                            }
                        }
#pragma unroll
                        for (int r = 0; r < 16; ++r) cnt += (xs[st][r] == mx) ? 1.f : 0.f;
                        continue;
                    }
                }
                const bool slow = tile_codes(xm, mx, ec, raw, cl);
#pragma unroll
                for (int r0_ = 0; r0_ < 16; r0_ += 4) {
                    if (!slow) {
                        ExpTable::Entry en[4];
#pragma unroll
                        for (int j = 0; j < 4; ++j) en[j] = ExpTable::entry_at(tabp, (int)cl[r0_ + j]);
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            const int r = r0_ + j;
                            const float d = __fsub_rn(mx, xm[r]);
                            const float de = (!MASKED || ((keep[st] >> r) & 1u)) ? ga[st][r] * rr + ds : 0.f;
                            float dd, gi1, gf1;
                            ec.grad_q1(d, raw[r], en[j].ca * de, dd, gi1, gf1);
                            gs[2] += en[j].ci * de, gs[3] += en[j].cf * de, gs[0] += gi1, gs[1] += gf1;
                            dm += dd;
                            ga[st][r] = dd;
                        }
                    } else {
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            const int r = r0_ + j;
                            float dd, g4[4];
                            exp_direct_grad(d1, d2, scale, __fsub_rn(mx, xm[r]),
                                            (!MASKED || ((keep[st] >> r) & 1u)) ? ga[st][r] * rr + ds : 0.f, &dd, g4);
                            gs[0] += g4[0], gs[1] += g4[1], gs[2] += g4[2], gs[3] += g4[3];
                            dm += dd;
                            ga[st][r] = dd;
                        }
                    }
                }
#pragma unroll
                for (int r = 0; r < 16; ++r) cnt += (xs[st][r] == mx) ? 1.f : 0.f;
            }
            {
                const float gf1 = -HGQ_LN2 * f1;
                gs[1] += gf1;
                if (ec.kbi) gs[0] -= gf1;
            }
            dm += xor32(dm);
            cnt += xor32(cnt);
            const float share = dm / cnt;  // the maximum's gradient is split evenly among ties
#pragma unroll
            for (int st = 0; st < ST; ++st)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    ga[st][r] = (xs[st][r] == mx) ? share - ga[st][r] : -ga[st][r];
                    if (MASKED && !((keep[st] >> r) & 1u)) ga[st][r] = 0.f;  // d (mask * scores - ...) / d scores
                }
        }
        QA_STAMP(8);
        {
            // the next element's operands: issued here, after the register-hungry stages, some eighty MFMAs ahead of their use
            const int nb = b + pl.n_wg;
            sq_.fetch(pq, nb, nb < pl.B), sk_.fetch(pk, nb, nb < pl.B), sv_.fetch(pv, nb, nb < pl.B), sg_.fetch(pg, nb, nb < pl.B);
        }
        if (active) {
            // dquery[t][h] = sum_s dscores[t][s] key[s][h]
            const floatx16 o = contract_keys<ST, true>(Ks, col0, t_l, hf, ga, BF, HD);
            store_rows<HD>(o, dq_ + ((int64_t)b * T * pl.N + h) * HD, (int64_t)pl.N * HD, t0 + t_l, hf);
        }
        QA_STAMP(9);
        __syncthreads();  // dvalue has read the probs
        QA_STAMP(10);
        if (active) spill_tiles<ST>(my_buf, ga, t_l, hf);
        __syncthreads();
        QA_STAMP(11);
        if (active) {
            // dkey[s][h] = sum_t dscores[t][s] query[t][h]
#pragma unroll
            for (int st = 0; st < ST; ++st)
                if (st % TH == th) dk_prev = contract_queries<TH, false, true>(Qs, col0, head_buf, st * 32, t_l, hf, BF, HD);
            b_prev = b;
        }
        QA_STAMP(12);
    }
    if (active && b_prev >= 0) {
#pragma unroll
        for (int st = 0; st < ST; ++st)
            if (st % TH == th) store_rows<HD>(dk_prev, dk_ + ((int64_t)b_prev * S * pl.N + h) * HD, (int64_t)pl.N * HD, st * 32 + t_l, hf);
    }
    // shared-quantizer gradients: wavefront sums, then the workgroup's in a fixed order
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const float vsum = wave_sum(gs[j]);
        if (lane == 0) part[wave][j] = vsum;
    }
    __syncthreads();
    if (threadIdx.x < 8) {
        float s = 0.f;
        for (int w = 0; w < NW; ++w) s += part[w][threadIdx.x];
        ws[(int64_t)blockIdx.x * 8 + threadIdx.x] = s;
    }
    if (!qo.present || !active) return;
    float *wf = ws + (int64_t)pl.n_wg * 8 + (int64_t)blockIdx.x * pl.N * T * S + (int64_t)(h * T + t0 + t_l) * S;
#pragma unroll
    for (int st = 0; st < ST; ++st)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            f32x4_t v4;
            v4.x = -HGQ_LN2 * gof[st][4 * g], v4.y = -HGQ_LN2 * gof[st][4 * g + 1], v4.z = -HGQ_LN2 * gof[st][4 * g + 2], v4.w = -HGQ_LN2 * gof[st][4 * g + 3];
            *(f32x4_t *)(wf + st * 32 + 8 * g + 4 * hf) = v4;
        }
}

#ifdef QA_PROF
extern "C" int hgq_qa_prof_read(unsigned long long *out) {
    return hipMemcpyFromSymbol(out, HIP_SYMBOL(qa_prof_stamps), sizeof(unsigned long long) * 8 * 4 * 16) == hipSuccess ? 0 : -2;
}
#endif

static size_t qattn_lds_bytes(int T, int S, bool bwd) {
    size_t words = (size_t)(T + 1 + 2 * (S + 1)) * QA_LD + QA_PAD;
    if (!bwd) return (words + SM_TABLE) * sizeof(float);
    words += (size_t)(T + 1) * QA_LD + (size_t)(QA_NT / 64) * 32 * QA_LD;
    return words * sizeof(float) + SM_TABLE * sizeof(ExpTable::Entry);
}

// Shapes the kernels take: sequence lengths 32 or 64 (both the same number of tiles), head size 8, 16 or
// 32 for query / key and value alike, every head of a batch element in one workgroup.
static int plan_qattn(int B, int T, int S, int N, int H, int64_t bw_rows, bool has_oq, QAttnPlan &pl, const char *who) {
    if (B < 0 || T < 1 || S < 1 || N < 1 || H < 1) return fail(HGQ_ERR_ARG, "%s: bad sizes", who);
    if (!((T == 32 && S == 32) || (T == 64 && S == 64)))
        return fail(HGQ_ERR_UNSUPPORTED, "%s: query and key sequences of 32 or of 64 positions are supported (T=%d S=%d)", who, T, S);
    if (H != 8 && H != 16 && H != 32) return fail(HGQ_ERR_UNSUPPORTED, "%s: head sizes 8, 16, 32 are supported, got %d", who, H);
    if (N * (T / 32) > QA_NT / 64 || N * H > 64)
        return fail(HGQ_ERR_UNSUPPORTED, "%s: N * T / 32 <= 8 and N * H <= 64 are required (N=%d T=%d H=%d)", who, N, T, H);
    if ((int64_t)B * 64 * N * H * 4 >= (1ll << 31)) return fail(HGQ_ERR_UNSUPPORTED, "%s: operands of 2 GiB or more", who);
    const int64_t P = has_oq ? bw_rows : 1;
    if (P < 1 || ((int64_t)N * T) % P != 0)
        return fail(HGQ_ERR_ARG, "%s: bw_rows=%lld does not divide N * T=%d", who, (long long)P, N * T);
    pl.B = B, pl.T = T, pl.S = S, pl.N = N, pl.P_table = P;
    pl.n_wg = persistent_grid(B > 0 ? B : 1, 1);
    pl.bf = hgq_dense_use_bf16_parts(-1);
    return HGQ_OK;
}

static SoftmaxPlan slices_plan(const QAttnPlan &pl) {
    SoftmaxPlan sp;
    sp.rows = (int64_t)pl.B * pl.N * pl.T, sp.L = pl.S, sp.Pq = (int64_t)pl.N * pl.T, sp.P_table = pl.P_table;
    sp.n_batches = pl.B, sp.PG = 1, sp.bpc = 1, sp.n_chunks = pl.n_wg, sp.SUB = 64, sp.VEC = 1, sp.NP = 1;
    return sp;
}

template <class K>
static int raise_lds(K kernel, size_t bytes, const char *who) {
    if (hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) != hipSuccess) {
        (void)hipGetLastError();
        return fail(HGQ_ERR_LAUNCH, "%s: cannot reserve %zu bytes of LDS", who, bytes);
    }
    return HGQ_OK;
}

static bool aligned16(const void *p) { return ((uintptr_t)p & 15u) == 0; }

static int check_mask(const uint8_t *mask, int mask_batch, int B, const char *who) {
    if (!mask) return HGQ_OK;
    if (mask_batch != 1 && mask_batch != B) return fail(HGQ_ERR_ARG, "%s: mask_batch must be 1 or the batch size, got %d", who, mask_batch);
    if ((uintptr_t)mask & 3u) return fail(HGQ_ERR_ARG, "%s: the mask must be 4-byte aligned", who);
    return HGQ_OK;
}

}  // namespace hgq

using namespace hgq;

#define QA_DISPATCH(H, T, ...)                                                              \
    do {                                                                                    \
        const int qa_key = (H) * 100 + (T);                                                   \
        switch (qa_key) {                                                                   \
            case 832: { constexpr int HD = 8, TH = 1; __VA_ARGS__; } break;                 \
            case 864: { constexpr int HD = 8, TH = 2; __VA_ARGS__; } break;                 \
            case 1632: { constexpr int HD = 16, TH = 1; __VA_ARGS__; } break;               \
            case 1664: { constexpr int HD = 16, TH = 2; __VA_ARGS__; } break;               \
            case 3232: { constexpr int HD = 32, TH = 1; __VA_ARGS__; } break;               \
            case 3264: { constexpr int HD = 32, TH = 2; __VA_ARGS__; } break;               \
            default: return fail(HGQ_ERR_UNSUPPORTED, "attention: no kernel for this shape"); \
        }                                                                                   \
    } while (0)

extern "C" int hgq_qattention_fwd(const float *query, const float *key, const float *value, float *out, int B, int T, int S,
                                  int N, int H, int64_t bw_rows, float input_scaler, float eps, const hgq_qdesc *exp_iq,
                                  const hgq_qdesc *exp_oq, const hgq_qdesc *inv_iq, const hgq_qdesc *inv_oq, const hgq_qdesc *oq,
                                  uint32_t *amax_exp_iq, uint32_t *amax_inv_iq, uint32_t *amax_oq, void *workspace,
                                  const uint8_t *mask, int mask_batch, int causal, void *stream) {
    hipStream_t s = (hipStream_t)stream;
    const bool has_oq = oq && oq->k;
    QAttnPlan pl;
    int rc = plan_qattn(B, T, S, N, H, bw_rows, has_oq, pl, "hgq_qattention_fwd");
    if (rc) return rc;
    if ((rc = check_mask(mask, mask_batch, B, "hgq_qattention_fwd"))) return rc;
    const QAttnMask mk = {mask, mask_batch, causal != 0};
    const bool masked = mask || causal;
    if (!softmax_desc_ok(exp_iq) || !softmax_desc_ok(exp_oq) || !softmax_desc_ok(inv_iq) || !softmax_desc_ok(inv_oq) || !softmax_desc_ok(oq))
        return fail(HGQ_ERR_ARG, "hgq_qattention_fwd: a quantizer descriptor has k but not i / fb");
    if (amax_oq && !has_oq) return fail(HGQ_ERR_ARG, "hgq_qattention_fwd: amax_oq without an output quantizer");
    if (has_oq && !(aligned16(oq->i) && aligned16(oq->fb) && ((uintptr_t)oq->k & 3u) == 0))
        return fail(HGQ_ERR_ARG, "hgq_qattention_fwd: the output quantizer's i / fb must be 16-byte aligned, k 4-byte aligned");
    if (amax_oq && !workspace && B > 0) return fail(HGQ_ERR_ARG, "hgq_qattention_fwd: amax_oq needs the workspace");
    uint32_t *slices = (amax_oq && B > 0) ? (uint32_t *)workspace : nullptr;
    // with the output quantizer's slices there is a reduction launch anyway: it also folds the scalar trackers' per-workgroup
    // maxima, so nothing needs clearing; otherwise the scalar trackers are cleared and updated by atomics
    uint32_t *pairs = slices ? slices + (int64_t)pl.n_wg * N * T * S : nullptr;
    if (!pairs && (rc = softmax_clear_trackers(amax_exp_iq, 1, amax_inv_iq, 1, B == 0 ? amax_oq : nullptr, pl.P_table * S, s))) return rc;
    if (B == 0) return HGQ_OK;
    if (!query || !key || !value || !out) return fail(HGQ_ERR_ARG, "hgq_qattention_fwd: null pointer");
    if (!(aligned16(query) && aligned16(key) && aligned16(value) && aligned16(out)))
        return fail(HGQ_ERR_ARG, "hgq_qattention_fwd: operands must be 16-byte aligned");
    bool train = true;
    const hgq_qdesc *all[5] = {exp_iq, exp_oq, inv_iq, inv_oq, oq};
    for (const hgq_qdesc *d : all)
        if (d && d->k && !(d->mode & HGQ_MODE_TRAINING)) train = false;
    const size_t lds = qattn_lds_bytes(T, S, false);
#define QA_FWD_M(TRAINV, PLAINV, MASKV)                                                                                          \
    QA_DISPATCH(H, T, {                                                                                                         \
        auto kern = qattn_fwd_kernel<HD, TH, TH, TRAINV, PLAINV, MASKV>;                                                        \
        static bool raised = false;                                                                                             \
        if (!raised && (rc = raise_lds(kern, lds, "hgq_qattention_fwd"))) return rc;                                            \
        raised = true;                                                                                                          \
        hipLaunchKernelGGL(kern, dim3(pl.n_wg), dim3(QA_NT), lds, s, query, key, value, out, pl, input_scaler, eps,             \
                           softmax_desc_or_none(exp_iq), softmax_desc_or_none(exp_oq), softmax_desc_or_none(inv_iq),            \
                           softmax_desc_or_none(inv_oq), softmax_desc_or_none(oq), amax_exp_iq, amax_inv_iq, slices, pairs, mk); \
    })
#define QA_FWD(TRAINV, PLAINV)                  \
    do {                                        \
        if (masked) QA_FWD_M(TRAINV, PLAINV, true); \
        else QA_FWD_M(TRAINV, PLAINV, false);   \
    } while (0)
    if (train && (!has_oq || ((oq->mode >> 4) & 0xf) == HGQ_WRAP))
        QA_FWD(true, true);
    else if (train)
        QA_FWD(true, false);
    else
        QA_FWD(false, false);
#undef QA_FWD
#undef QA_FWD_M
    if ((rc = check_launch("hgq_qattention_fwd"))) return rc;
    if (!slices) return HGQ_OK;
    const int64_t entries = pl.P_table * S;
    hipLaunchKernelGGL(qattn_amax_reduce_kernel, dim3((unsigned)((entries + 63) / 64)), dim3(1024), 0, s, slices, pl.n_wg, (int64_t)N * T, S,
                       pl.P_table, amax_oq, (const uint32_t *)pairs, amax_exp_iq, amax_inv_iq);
    return check_launch("hgq_qattention_fwd(trackers)");
}

extern "C" int64_t hgq_qattention_fwd_workspace(int B, int T, int S, int N, int H, int64_t bw_rows, int track_oq) {
    QAttnPlan pl;
    if (plan_qattn(B, T, S, N, H, bw_rows, track_oq != 0, pl, "hgq_qattention_fwd_workspace")) return -1;
    return track_oq ? (int64_t)pl.n_wg * N * T * S + 2 * (int64_t)pl.n_wg : 0;  // slices + a pair of scalar trackers per workgroup
}

extern "C" int64_t hgq_qattention_bwd_workspace(int B, int T, int S, int N, int H, int64_t bw_rows, int has_oq) {
    QAttnPlan pl;
    if (plan_qattn(B, T, S, N, H, bw_rows, has_oq != 0, pl, "hgq_qattention_bwd_workspace")) return -1;
    return (int64_t)pl.n_wg * 8 + (has_oq ? (int64_t)pl.n_wg * N * T * S : 0);
}

extern "C" int hgq_qattention_bwd(const float *dout, const float *query, const float *key, const float *value, float *dquery,
                                  float *dkey, float *dvalue, int B, int T, int S, int N, int H, int64_t bw_rows,
                                  float input_scaler, float eps, const hgq_qdesc *exp_iq, const hgq_qdesc *exp_oq,
                                  const hgq_qdesc *inv_iq, const hgq_qdesc *inv_oq, const hgq_qdesc *oq, float *g_shared,
                                  float *g_oq_i, float *g_oq_fb, float *workspace, const uint8_t *mask, int mask_batch, int causal,
                                  void *stream) {
    hipStream_t s = (hipStream_t)stream;
    const bool has_oq = oq && oq->k;
    QAttnPlan pl;
    int rc = plan_qattn(B, T, S, N, H, bw_rows, has_oq, pl, "hgq_qattention_bwd");
    if (rc) return rc;
    if ((rc = check_mask(mask, mask_batch, B, "hgq_qattention_bwd"))) return rc;
    const QAttnMask mk = {mask, mask_batch, causal != 0};
    if (!softmax_desc_ok(exp_iq) || !softmax_desc_ok(exp_oq) || !softmax_desc_ok(inv_iq) || !softmax_desc_ok(inv_oq) || !softmax_desc_ok(oq))
        return fail(HGQ_ERR_ARG, "hgq_qattention_bwd: a quantizer descriptor has k but not i / fb");
    const hgq_qdesc *all[5] = {exp_iq, exp_oq, inv_iq, inv_oq, oq};
    for (const hgq_qdesc *d : all)
        if (d && d->k && !(d->mode & HGQ_MODE_TRAINING))
            return fail(HGQ_ERR_ARG, "hgq_qattention_bwd: the surrogate gradient is defined for training mode only");
    if (has_oq && !(aligned16(oq->i) && aligned16(oq->fb) && ((uintptr_t)oq->k & 3u) == 0))
        return fail(HGQ_ERR_ARG, "hgq_qattention_bwd: the output quantizer's i / fb must be 16-byte aligned, k 4-byte aligned");
    if (has_oq && (((oq->mode >> 4) & 0xf) != HGQ_WRAP || (oq->mode & HGQ_MODE_KBI)))
        return fail(HGQ_ERR_UNSUPPORTED, "hgq_qattention_bwd: a saturating or (k, b, i) output quantizer takes the separate softmax kernels");
    if (B == 0) {
        if (g_shared && (rc = fill_f32(g_shared, 0.f, 8, s))) return rc;
        if (has_oq && g_oq_i && (rc = fill_f32(g_oq_i, 0.f, pl.P_table * S, s))) return rc;
        if (has_oq && g_oq_fb && (rc = fill_f32(g_oq_fb, 0.f, pl.P_table * S, s))) return rc;
        return HGQ_OK;
    }
    if (!dout || !query || !key || !value || !dquery || !dkey || !dvalue || !workspace)
        return fail(HGQ_ERR_ARG, "hgq_qattention_bwd: null pointer");
    if (!(aligned16(dout) && aligned16(query) && aligned16(key) && aligned16(value) && aligned16(dquery) && aligned16(dkey) &&
          aligned16(dvalue) && aligned16(workspace)))
        return fail(HGQ_ERR_ARG, "hgq_qattention_bwd: operands and workspace must be 16-byte aligned");
    const size_t lds = qattn_lds_bytes(T, S, true);
#define QA_BWD(MASKV, BFV)                                                                                                       \
    QA_DISPATCH(H, T, {                                                                                                          \
        auto kern = qattn_bwd_kernel<HD, TH, TH, MASKV, BFV>;                                                                    \
        static bool raised = false;                                                                                              \
        if (!raised && (rc = raise_lds(kern, lds, "hgq_qattention_bwd"))) return rc;                                             \
        raised = true;                                                                                                           \
        hipLaunchKernelGGL(kern, dim3(pl.n_wg), dim3(QA_NT), lds, s, dout, query, key, value, dquery, dkey, dvalue, pl,          \
                           input_scaler, eps, softmax_desc_or_none(exp_iq), softmax_desc_or_none(exp_oq),                        \
                           softmax_desc_or_none(inv_iq), softmax_desc_or_none(inv_oq), softmax_desc_or_none(oq), workspace, mk); \
    })
    if (pl.bf) {
        if (mask || causal) QA_BWD(true, true);
        else QA_BWD(false, true);
    } else {
        if (mask || causal) QA_BWD(true, false);
        else QA_BWD(false, false);
    }
#undef QA_BWD
    if ((rc = check_launch("hgq_qattention_bwd"))) return rc;
    // a wrapping quantizer's integer bits take no gradient: the reduction writes zeros there
    return softmax_reduce_slices(workspace, slices_plan(pl), g_shared, g_oq_i, g_oq_fb, has_oq, false, s);
}
