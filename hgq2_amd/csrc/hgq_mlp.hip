// One training step of a stack of QDense layers in two launches (three when the quantized weight image has to be
// rebuilt first).
//
// At the layer sizes HGQ targets (tens of units per layer) a training step built from per-layer
// kernels is bound by launch latency, not by HBM or MFMA.  Here the whole data path - every
// layer's input quantizer, contraction, bias, activation, the sparse cross-entropy loss and the
// full backward pass - runs in ONE kernel: the quantized weights of all layers sit in LDS
// (a few tens of KB), a workgroup takes a tile of 64 samples through forward and backward without
// touching HBM in between, and writes its partial gradient sums to a private slice.  A second
// kernel adds the slices in a fixed order and applies, per variable entry, the integer-bit tracking,
// EBOPs (value, variable and gradient), the weight / bias quantizer backward and the SGD update
// with the MonoL1 gradient and the clip constraints folded in; it also leaves the quantized weight
// image of the updated variables for the next step.
//
// HBM traffic per step is the input batch, the labels and the partial slices.
#include "hgq_device.h"
#include "hgq_host.h"

namespace hgq {


#define MLP_BM 64
// Phase time stamps of workgroup 0, one row per wavefront (measurement builds only: -DMLP_PROF)
#ifdef MLP_PROF
__device__ unsigned long long mlp_prof_stamps[8 * 64];
#define MLP_STAMP(i)                                                                                                  \
    do {                                                                                                              \
        if (blockIdx.x == 0 && (threadIdx.x & 63) == 0) mlp_prof_stamps[(threadIdx.x >> 6) * 64 + (i)] = wall_clock64(); \
    } while (0)
#else
#define MLP_STAMP(i)
#endif
// the matrix-core chains: by exact bf16 parts (1) or with the fp32 instruction (0)
#ifndef MLP_BF16
#define MLP_BF16 1
#endif
#if MLP_BF16
#define MLP_CHAIN(FA, FB) mfma_chain_bf16<FA, FB>
#else
#define MLP_CHAIN(FA, FB) mfma_chain
#endif
#define MLP_NT 512  // eight wavefronts: two per SIMD, so the chains of one hide the latencies of the other
#define MLP_LDZ 65

__device__ __forceinline__ int acc_row_(int r, int lane) { return (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3); }

struct MlpLayerDev {
    hgq_mlp_layer h;
    int Kp, Np, ldw;                 // K, N padded to multiples of 32; leading dimension of the LDS kernel
    int off_w, off_qb, off_f;        // LDS offsets (floats)
    int acol;                        // column of this layer's input in the activation arrays
    int p_dw, p_db, p_df, p_amax;    // offsets inside a partial slice
};

struct MlpDev {
    MlpLayerDev l[HGQ_MLP_MAX_LAYERS];
    int n_layers, n_classes;
    int ld_raw, ld_rx;               // leading dimensions of the activation arrays
    int off_raw, off_rx, off_dz0, off_dz1, off_red;  // LDS offsets (floats)
    int p_loss, M;                   // loss slot and slice length
    int acol_out;                    // column of the logits in `raw`
};

__device__ __forceinline__ KIF kbi_entry(const void *k, const float *i, const float *b, int64_t idx, int mode) {
    const Mode m(mode);
    return resolve_kif(load_k(k, idx, m.k_u8), i[idx], b[idx], true, true);
}

// The quantized kernels and biases of all layers and the rounded fractional bits of the input
// quantizers, laid out exactly as the forward/backward kernel keeps them in LDS (zero padded).
// One thread per entry: every workgroup of the main kernel then fetches the finished image with
// a single round of wide loads instead of re-quantizing it behind dozens of dependent loads.
__global__ __launch_bounds__(256) void mlp_prep_kernel(MlpDev d, float *__restrict__ img) {
    const int e = blockIdx.x * 256 + threadIdx.x;
    if (e >= d.off_raw) return;
    int l = 0;
    while (l + 1 < d.n_layers && e >= d.l[l + 1].off_w) ++l;
    const MlpLayerDev &ly = d.l[l];
    const hgq_mlp_layer &h = ly.h;
    float v = 0.f;
    if (e < ly.off_qb) {
        const int id = e - ly.off_w, k = id / ly.ldw, n = id - k * ly.ldw;
        if (k < h.K && n < h.N) {
            const Mode m(h.mode_ker);
            const int64_t t = (int64_t)k * h.N + n;
            v = quantize_dyn(h.w[t], kbi_entry(h.k_ker, h.i_ker, h.b_ker, t, h.mode_ker), m.round_mode, m.overflow_mode, true);
        }
    } else if (e < ly.off_f) {
        const int n = e - ly.off_qb;
        if (n < h.N && h.bias) {
            const Mode m(h.mode_bias);
            v = quantize_dyn(h.bias[n], kbi_entry(h.k_bias, h.i_bias, h.b_bias, n, h.mode_bias), m.round_mode, m.overflow_mode, true);
        }
    } else {
        const int k = e - ly.off_f;
        if (k < h.K) v = rintf(h.f_in[k]);
    }
    img[e] = v;
}

#define MLP_AUX 192  // per layer, after the slices: colsum[64], i_in[64], round(f_in)[64] of the variables BEFORE this step's update

// Snapshot the update pass needs of variables it overwrites: taken by the main kernel (which runs to completion before
// the update pass starts), so that an update workgroup never reads a variable another one is writing.  Row (l, k) is
// computed by one wavefront: colsum = sum_n bits_ker[k, n].
struct MlpSnapRow {
    int l, k;      // layer and row (l < 0: none)
    float cs, i, f;
};

// Row `row` of the snapshot, first half: the loads (one kernel-row entry per lane) are issued and nothing waits for them.
__device__ __forceinline__ MlpSnapRow mlp_snapshot_begin(const MlpDev &d, int row, int lane) {
    MlpSnapRow r;
    r.l = -1, r.k = 0, r.cs = 0.f, r.i = 0.f, r.f = 0.f;
    int base = 0;
    for (int l = 0; l < d.n_layers; ++l) {  // (the layer index stays a loop counter: indexing the kernel-argument
        const hgq_mlp_layer &h = d.l[l].h;  //  structure with a computed value would move it to scratch memory)
        const int k = row - base;
        if (k >= 0 && k < h.K) {
            const Mode mk(h.mode_ker);
            r.l = l, r.k = k;
            if (lane < h.N) {
                r.cs = rintf(h.b_ker[k * h.N + lane]);
                if (mk.overflow_mode == HGQ_SAT) r.cs += load_k(h.k_ker, k * h.N + lane, mk.k_u8);
            }
            r.i = h.i_in[k], r.f = h.f_in[k];
        }
        base += h.K;
    }
    return r;
}

// Second half: the row sum over the lanes (integers: exact in any order) and the three stores.
__device__ __forceinline__ void mlp_snapshot_end(MlpSnapRow r, float *aux, int lane) {
    if (r.l < 0) return;
    float cs = r.cs;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) cs += __shfl_xor(cs, o, 64);
    if (lane == 0) {
        float *a = aux + r.l * MLP_AUX;
        a[r.k] = cs, a[64 + r.k] = r.i, a[128 + r.k] = rintf(r.f);
    }
}

__global__ __launch_bounds__(MLP_NT) void mlp_fwd_bwd_kernel(MlpDev d, const float *__restrict__ img, const float *__restrict__ x,
                                                          const int64_t *__restrict__ labels, int64_t rows,
                                                          float *part, float *aux, uint32_t *loss_words) {
    extern __shared__ float lds[];
    __shared__ float loss_part[MLP_NT / 64];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    MLP_STAMP(0);
    // snapshot for the update pass: workgroup w's last wavefront takes row w, in a forward phase, where it has no other work
    const bool snap_wave = __builtin_amdgcn_readfirstlane(wave) == MLP_NT / 64 - 1;
    if (blockIdx.x == 0 && tid < 4) loss_words[tid] = 0u;  // the update pass adds up and counts its loss pieces here
    const int L = d.n_layers;
    float *raw = lds + d.off_raw, *rx = lds + d.off_rx;
    // [2][L][64] fractional-bit gradient sums: one set per row half of the tile, each entry owned by one wavefront for the
    // whole launch (no atomics: the two halves are added in a fixed order at the end)
    float *dfs = lds + d.off_red;
    uint32_t *amx = (uint32_t *)(lds + d.off_red) + 2 * 64 * HGQ_MLP_MAX_LAYERS;  // [L][64] abs-max of each layer's quantized input
    float *my = part + (int64_t)blockIdx.x * d.M;
    const int64_t n_tiles = (rows + MLP_BM - 1) / MLP_BM;
    const float inv_rows = 1.0f / (float)rows;

    // ---- prologue.  The first input tile's loads are issued ahead of everything else: they travel while the image is
    // fetched (the tile can only be quantized once the image's fractional bits are in LDS, but it need not wait to be asked for)
    const int K0 = d.l[0].h.K, n_el0 = MLP_BM * K0;
    float pre[4];
    {
        const int64_t r0 = (int64_t)blockIdx.x * MLP_BM, left = rows - r0;
        const __amdgpu_buffer_rsrc_t rs = buf_rsrc(x + r0 * K0, (left < MLP_BM ? (left > 0 ? left : 0) : MLP_BM) * K0 * 4);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int id = u * MLP_NT + tid;
            pre[u] = buf_ld1(rs, id < n_el0 ? (uint32_t)id * 4u : BUF_OOB);
        }
    }
    MLP_STAMP(1);
    // fetch the quantized kernels / biases / rounded fractional bits (off_raw is a multiple of 4)
    // (four 128-bit loads per thread in flight: one load per loop trip would cost a memory latency each; the LDS
    // clearing is done while the first batch travels)
    for (int id0 = 0; id0 < d.off_raw; id0 += 4 * 4 * MLP_NT) {
        float4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int id = id0 + (u * MLP_NT + tid) * 4;
            v[u] = *(const float4 *)(img + (id < d.off_raw ? id : 0));
        }
        if (id0 == 0) {
            MLP_STAMP(2);
            // padding columns of rx stay zero for good (rx starts at a multiple of four floats)
            const int n_rx = MLP_BM * d.ld_rx;
            for (int id = tid * 4; id + 3 < n_rx; id += 4 * MLP_NT) *(float4 *)(rx + id) = float4{0.f, 0.f, 0.f, 0.f};
            if (tid < (n_rx & 3)) rx[(n_rx & ~3) + tid] = 0.f;
            for (int id = tid; id < 64 * HGQ_MLP_MAX_LAYERS; id += MLP_NT) dfs[id] = 0.f, dfs[64 * HGQ_MLP_MAX_LAYERS + id] = 0.f, amx[id] = 0u;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int id = id0 + (u * MLP_NT + tid) * 4;
            if (id < d.off_raw) *(float4 *)(lds + id) = v[u];
        }
    }
    __syncthreads();
    MLP_STAMP(3);
    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const bool first = tile == blockIdx.x;
        const int64_t r0 = tile * MLP_BM;
        const int live = (int)(rows - r0 < MLP_BM ? rows - r0 : MLP_BM);  // rows of this tile that exist
        // ---- stage the input tile: raw value, quantized value, abs-max
        MLP_STAMP(60);
        {
            const MlpLayerDev &l0 = d.l[0];
            const int rm = Mode(l0.h.mode_in).round_mode;
            const float *fl = lds + l0.off_f;
            // the tile's rows are contiguous in x: buffer loads, zeros past the last row, four in flight
            const int n_el = n_el0;
            const __amdgpu_buffer_rsrc_t rs = buf_rsrc(x + r0 * K0, live * K0 * 4);
            // id / K0 for id < 64 * 64 and K0 <= 64 as a multiply and a shift (exact: the error term id * (K0 - 1) stays below 2**20)
            const uint32_t by_k0 = ((1u << 20) + (uint32_t)K0 - 1u) / (uint32_t)K0;
            for (int id0 = 0; id0 < n_el; id0 += 4 * MLP_NT) {
                float v[4];
                MLP_STAMP(61);
                if (first && id0 == 0) {
#pragma unroll
                    for (int u = 0; u < 4; ++u) v[u] = pre[u];
                } else {
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        const int id = id0 + u * MLP_NT + tid;
                        v[u] = buf_ld1(rs, id < n_el ? (uint32_t)id * 4u : BUF_OOB);
                    }
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int id = id0 + u * MLP_NT + tid;
                    if (id < n_el) {
                        const int row = (int)(((uint32_t)id * by_k0) >> 20), k = id - row * K0;
                        float q = fixed_round_dyn(v[u], fl[k], rm);
                        q = row < live ? q : 0.f;  // (a row past the end was read as zeros: its abs-max term is zero too)
                        atomicMax(&amx[k], abs_bits(q));
                        raw[row * d.ld_raw + l0.acol + k] = v[u];
                        rx[row * d.ld_rx + l0.acol + k] = q;
                    }
                }
            }
        }
        MLP_STAMP(32);
        __syncthreads();
        MLP_STAMP(4);
        // ================= forward =================
        for (int l = 0; l < L; ++l) {
            const MlpLayerDev &ly = d.l[l];
            const int N = ly.h.N;
            const int rh = wave & 1, cb = wave >> 1;
            if (snap_wave && first && l == 0) {
                // (fewer workgroups than rows - small batches: the remaining rows, one after the other)
                int total = 0;
                for (int j = 0; j < L; ++j) total += d.l[j].h.K;
                for (int row = (int)blockIdx.x; row < total; row += (int)gridDim.x) mlp_snapshot_end(mlp_snapshot_begin(d, row, lane), aux, lane);
            }
            if (wave < 4 && cb * 32 < ly.Np) {
                floatx16 acc = {0};
                const float *ws = lds + ly.off_w;
                const int arow = rh * 32 + (lane & 31), kq = lane >> 5, bcol = cb * 32 + (lane & 31);
                // everything the epilogue needs is asked for ahead of the chain (no branches in between, so the scalar and
                // LDS loads travel together): the bias, and the next layer's input quantizer, which runs on the accumulator
                // registers (for the last layer the values are read and not used)
                const bool last = l + 1 == L;
                const MlpLayerDev &nx = d.l[last ? l : l + 1];
                const int ocol = (last ? d.acol_out : nx.acol) + bcol;
                const int rm = Mode(nx.h.mode_in).round_mode;
                const bool relu = ly.h.act == HGQ_ACT_RELU;
                const float bias = lds[ly.off_qb + bcol], fn = lds[nx.off_f + bcol];
                // input columns and kernel rows are zero padded to a multiple of 32
                acc = MLP_CHAIN(false, false)(acc, rx + arow * d.ld_rx + ly.acol + kq, 1, ws + kq * ly.ldw + bcol, ly.ldw, (ly.h.K + 15) >> 4);
                if (bcol < N) {
                    uint32_t mx = 0;
                    float *raw_o = raw + (rh * 32 + (lane >> 5) * 4) * d.ld_raw + ocol, *rx_o = rx + (rh * 32 + (lane >> 5) * 4) * d.ld_rx + ocol;
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int rr = (r >> 2) * 8 + (r & 3);  // acc_row_(r, lane) - 4 * (lane / 32)
                        float v = acc[r] + bias;
                        v = relu ? (v > 0.f ? v : 0.f) : v;
                        raw_o[rr * d.ld_raw] = v;
                        if (!last) {
                            float q = fixed_round_dyn(v, fn, rm);
                            q = rh * 32 + (lane >> 5) * 4 + rr < live ? q : 0.f;
                            rx_o[rr * d.ld_rx] = q;
                            const uint32_t a = abs_bits(q);
                            mx = a > mx ? a : mx;
                        }
                    }
                    if (!last) {
                        const uint32_t o = (uint32_t)__shfl_xor((int)mx, 32, 64);
                        mx = o > mx ? o : mx;
                        if (lane < 32) atomicMax(&amx[(l + 1) * 64 + bcol], mx);
                    }
                }
            }
            MLP_STAMP(33 + l);
            __syncthreads();
            MLP_STAMP(5 + l);
        }
        // ================= loss: mean sparse categorical cross-entropy from logits =================
        // eight threads per sample, classes j, j + 8, ...: one exponential per thread instead of all of a row's in turn
        float *cur = lds + d.off_dz0, *nxt = lds + d.off_dz1;
        {
            const int C = d.n_classes;
            const int Cp = d.l[L - 1].Np;
            const int row = tid >> 3, j = tid & 7;
            const int64_t gr = r0 + row;
            const float *z = raw + row * d.ld_raw + d.acol_out;
            float *dz = cur + row * MLP_LDZ;
            float lrow = 0.f;
            if (gr < rows) {
                float mx = -INFINITY;
                for (int c = j; c < C; c += 8) mx = fmaxf(mx, z[c]);
                mx = fmaxf(mx, __shfl_xor(mx, 1, 64)), mx = fmaxf(mx, __shfl_xor(mx, 2, 64)), mx = fmaxf(mx, __shfl_xor(mx, 4, 64));
                float se = 0.f;
                for (int c = j; c < C; c += 8) se += expf(z[c] - mx);
                // the same association on every lane of the group (and on every run): pairs, then pairs of pairs
                se += __shfl_xor(se, 1, 64), se += __shfl_xor(se, 2, 64), se += __shfl_xor(se, 4, 64);
                const int lab = (int)labels[gr];
                const bool lab_ok = (unsigned)lab < (unsigned)C;  // a label outside [0, C): NaN loss, no gradient for the sample
                if (j == 0) lrow = lab_ok ? logf(se) - (z[lab_ok ? lab : 0] - mx) : NAN;
                const float inv = 1.0f / se;
                // a relu on the output layer: its mask (z holds the values after the activation)
                const bool mask_out = d.l[L - 1].h.act == HGQ_ACT_RELU;
                for (int c = j; c < Cp; c += 8) {
                    float gz = 0.f;
                    if (c < C && lab_ok) {
                        gz = (expf(z[c] - mx) * inv - (c == lab ? 1.0f : 0.0f)) * inv_rows;
                        if (mask_out && !(z[c] > 0.f)) gz = 0.f;
                    }
                    dz[c] = gz;
                }
            } else {
                for (int c = j; c < Cp; c += 8) dz[c] = 0.f;
            }
            // the tile's loss: the eight samples of a wavefront in lane order, then the wavefronts in order
#pragma unroll
            for (int o = 8; o < 64; o <<= 1) lrow += __shfl_xor(lrow, o, 64);
            if (lane == 0) loss_part[wave] = lrow;
        }
        __syncthreads();
        MLP_STAMP(16);
        if (tid == 0) {
            float t = 0.f;
#pragma unroll
            for (int w = 0; w < MLP_NT / 64; ++w) t += loss_part[w];
            my[d.p_loss] = (first ? 0.f : my[d.p_loss]) + t * inv_rows;
        }
        // ================= backward =================
        // `cur` holds the gradient at this layer's pre-activation (relu mask already applied) in
        // columns [0, Np); both phases only read it, so one barrier per layer is enough.
        for (int l = L - 1; l >= 0; --l) {
            const MlpLayerDev &ly = d.l[l];
            const int K = ly.h.K, N = ly.h.N;
            const int K32 = ly.Kp >> 5, N32 = ly.Np >> 5;
            const int nblk = K32 * N32;
            // ---- kernel gradient: one 32 x 32 block per wave over the whole tile, on waves 4 .. 7
            // (waves 0 .. 3 work on the input gradient at the same time)
            if (wave >= 4 && wave - 4 < nblk) {
                const int wkb = (wave - 4) / N32, wnb = (wave - 4) % N32;
                floatx16 acc = {0};
                const int kq = lane >> 5, c32 = lane & 31;
                acc = MLP_CHAIN(false, true)(acc, rx + kq * d.ld_rx + ly.acol + wkb * 32 + c32, d.ld_rx, cur + kq * MLP_LDZ + wnb * 32 + c32, MLP_LDZ,
                                             MLP_BM / 16);
                MLP_STAMP(48 + (L - 1 - l));
                // through a descriptor of this layer's K x N section: rows past K fall outside it and are dropped, so
                // the sixteen stores (or load - add - store triples) go out back to back, without a branch each
                const int n = wnb * 32 + c32;
                const __amdgpu_buffer_rsrc_t rsw = buf_rsrc(my + ly.p_dw, (int64_t)K * N * 4);
                const uint32_t off0 = (uint32_t)(((wkb * 32 + kq * 4) * N + n) * 4);
                float old[16];
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const uint32_t off = n < N ? off0 + (uint32_t)(((r >> 2) * 8 + (r & 3)) * N * 4) : BUF_OOB;
                    old[r] = first ? 0.f : buf_ld1(rsw, off);
                }
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const uint32_t off = n < N ? off0 + (uint32_t)(((r >> 2) * 8 + (r & 3)) * N * 4) : BUF_OOB;
                    buf_st1(rsw, off, first ? acc[r] : old[r] + acc[r]);
                }
            }
            MLP_STAMP(52 + (L - 1 - l));
            // ---- bias gradient: the last wave is free of kernel-gradient work unless all four blocks exist.  A layer of
            // up to 32 outputs: each half of the wavefront adds 32 rows (in row order), the halves are added last
            if (ly.h.bias && wave == 7) {
                const bool halves = N <= 32;
                const int col = halves ? lane & 31 : lane, ra = halves ? (lane >> 5) * (MLP_BM / 2) : 0, nr = halves ? MLP_BM / 2 : MLP_BM;
                const float *src = cur + ra * MLP_LDZ + (col < N ? col : 0);
                float s0 = 0.f, s1 = 0.f;
#pragma unroll 16
                for (int r = 0; r < nr; r += 2) s0 += src[r * MLP_LDZ], s1 += src[(r + 1) * MLP_LDZ];
                float t = s0 + s1;
                if (halves) t += __shfl_xor(t, 32, 64);
                if (lane < N) {
                    float *dst = my + ly.p_db + lane;
                    *dst = first ? t : *dst + t;
                }
            }
            // ---- input gradient, the relu mask of the layer below, and this layer's fractional-bit gradient
            {
                const int rh = wave & 1, kb = wave >> 1;
                if (wave < 4 && kb < K32) {
                    floatx16 acc = {0};
                    const float *ws = lds + ly.off_w;
                    const int arow = rh * 32 + (lane & 31), kq = lane >> 5, wrow = kb * 32 + (lane & 31);
                    // gradient columns and kernel columns are zero padded to a multiple of 32
                    acc = MLP_CHAIN(true, false)(acc, cur + arow * MLP_LDZ + kq, 1, ws + wrow * ly.ldw + kq, 1, (N + 15) >> 4);
                    MLP_STAMP(56 + (L - 1 - l));
                    const int kcol = kb * 32 + (lane & 31);
                    const bool mask_below = l > 0 && d.l[l - 1].h.act == HGQ_ACT_RELU;
                    // this lane's sixteen rows are rb + {0..3, 8..11, 16..19, 24..27}: all its LDS reads are asked for first
                    const int rb = rh * 32 + (lane >> 5) * 4;
                    const float *raw_i = raw + rb * d.ld_raw + ly.acol + kcol, *rx_i = rx + rb * d.ld_rx + ly.acol + kcol;
                    float *nxt_o = nxt + rb * MLP_LDZ + kcol;
                    float a[16], q[16];
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int rr = (r >> 2) * 8 + (r & 3);
                        a[r] = raw_i[rr * d.ld_raw], q[r] = rx_i[rr * d.ld_rx];
                    }
                    float dfsum = 0.f;
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int rr = (r >> 2) * 8 + (r & 3);
                        const float delta = q[r] - a[r];
                        const float term = -HGQ_LN2 * delta * acc[r];
                        dfsum += (kcol < K && rb + rr < live) ? term : 0.f;
                    }
                    if (l > 0) {  // (nobody reads the gradient at the stack's input)
#pragma unroll
                        for (int r = 0; r < 16; ++r)
                            nxt_o[((r >> 2) * 8 + (r & 3)) * MLP_LDZ] = (kcol < K && (!mask_below || a[r] > 0.f)) ? acc[r] : 0.f;
                    }
                    dfsum += __shfl_xor(dfsum, 32, 64);
                    if (lane < 32 && kcol < K) dfs[(rh * HGQ_MLP_MAX_LAYERS + l) * 64 + kcol] += dfsum;  // this wavefront's own entry
                }
            }
            MLP_STAMP(41 + (L - 1 - l));
            __syncthreads();
            MLP_STAMP(17 + (L - 1 - l));
            float *t = cur;
            cur = nxt;
            nxt = t;
        }
    }
    // ---- this workgroup's abs-max and fractional-bit sums
    MLP_STAMP(30);
    for (int l = 0; l < L; ++l) {
        const MlpLayerDev &ly = d.l[l];
        if (tid < ly.h.K) {
            my[ly.p_df + tid] = dfs[l * 64 + tid] + dfs[(HGQ_MLP_MAX_LAYERS + l) * 64 + tid];
            ((uint32_t *)(my + ly.p_amax))[tid] = amx[l * 64 + tid];
        }
    }
    MLP_STAMP(31);
}

__device__ __forceinline__ float sgd_clip(float w, float g, float lr, float l1, float lo, float hi) {
    return fminf(fmaxf(__fsub_rn(w, __fmul_rn(lr, __fadd_rn(g, l1))), lo), hi);
}

// Second and last launch of a step.  A workgroup is 64 entries x 16 slice groups; its role, from its block index:
//   role 0 (ceil(K N / 64) per layer): 64 kernel entries - their gradient sums over the slices, quantizer backward,
//           SGD + constraints, the next step's image entries;
//   role 1 (one per layer): the bias entries likewise, and the layer's EBOPs (value, variable, loss term);
//   role 2 (one per layer): the input quantizer's fractional bits, and the assignment of its tracked integer bits;
//   last block: the cross-entropy loss slot.
// Every workgroup of a layer also reduces the layer's abs-max section, so each knows the tracked integer bits (hence the
// input bit counts the EBOPs gradients need) without waiting for another workgroup; pre-update values of variables it
// does not own come from the main kernel's snapshot.
#define MLP_RG 16
// The loss is the sum of one piece per workgroup (cross-entropy, a layer's ebops * beta, MonoL1 terms), taken in fixed
// point so that it does not depend on the order in which the workgroups arrive: ONE 64-bit atomic addition per workgroup
// carries its piece (multiples of 2**-28 in bits 12 and up: exact for a piece of magnitude 1/16 and more, within 2**-28
// otherwise) and counts it (bits 0 .. 10); the workgroup whose addition completes the count converts the sum - one
// rounding - and clears the word for the next step.  A piece outside +-2**22 or not finite goes beside the sum: it is
// left in `odd` (an exchange, whose result the addition's operand depends on, so it is in place before it is counted,
// bit 11) and added to the converted sum by the last workgroup; with several such pieces in one step one of them is
// reported (NaN if any is NaN ahead of it in arrival, which no run can tell from another NaN).  The main kernel cleared both words.
#define MLP_LOSS_SCALE 268435456.0f  // 2**28
__device__ __forceinline__ void mlp_loss_piece(float piece, unsigned long long *word, uint32_t *odd, float *loss, int lane) {
    if (lane != 0) return;
    unsigned long long add = 1ull;
    const bool plain = fabsf(piece) < 4194304.0f;  // (false for NaN)
    if (plain) {
        add += (unsigned long long)((long long)(piece * MLP_LOSS_SCALE)) << 12;  // the product is exact, and an integer below 2**50
    } else {
        const uint32_t before = atomicExch(odd, __float_as_uint(piece));
        uint32_t mark = 1u << 11;
        asm volatile("" : "+v"(mark) : "v"(before));
        add += mark;
    }
    const unsigned long long total = atomicAdd(word, add) + add;
    if ((uint32_t)(total & 0x7ffull) != gridDim.x) return;
    float v = (float)((double)((long long)total >> 12) * (1.0 / (double)MLP_LOSS_SCALE));
    if (total & 0x800ull) v += __uint_as_float(atomicExch(odd, 0u));
    loss[0] = v;
    atomicExch(word, 0ull);
}

__global__ __launch_bounds__(64 * MLP_RG) void mlp_reduce_update_kernel(MlpDev d, const float *__restrict__ part, int n_parts,
                                                                        const float *__restrict__ aux, float lr, float *loss, float *img,
                                                                        unsigned long long *loss_word, uint32_t *loss_odd) {
    __shared__ float red[64 * MLP_RG];
    __shared__ uint32_t smx[64 * MLP_RG];
    __shared__ float val[64], bits_in[64], dbits_in[64], new_i[64];
    const int e_local = threadIdx.x & 63, grp = threadIdx.x >> 6;
    const int per = (n_parts + MLP_RG - 1) / MLP_RG;
    const int g0 = grp * per, g1 = min(n_parts, g0 + per);
    // ---- role
    int l = 0, role = 3, j = 0;
    {
        int b = blockIdx.x;
        for (; l < d.n_layers; ++l) {
            const int na = (d.l[l].h.K * d.l[l].h.N + 63) / 64;
            if (b < na + 2) {
                role = b < na ? 0 : (b == na ? 1 : 2);
                j = b;
                break;
            }
            b -= na + 2;
        }
    }
    const bool loss_block = role == 3;
    if (loss_block) l = 0;
    const MlpLayerDev &ly = d.l[l];
    const hgq_mlp_layer &h = ly.h;
    const int K = h.K, N = h.N;
    // ---- this workgroup's 64 gradient sums
    int n_mine, p0;
    if (role == 0) p0 = ly.p_dw + 64 * j, n_mine = min(64, K * N - 64 * j);
    else if (role == 1) p0 = ly.p_db, n_mine = h.bias ? N : 0;
    else if (role == 2) p0 = ly.p_df, n_mine = K;
    else p0 = d.p_loss, n_mine = 1;
    // the variables of the entry this thread will update, requested before the slices (the updates are applied by the
    // first wavefront only; the loads are in flight while all sixteen reduce)
    const int t = e_local;
    const bool mine = grp == 0 && t < n_mine && !loss_block;
    float v_w = 0.f, v_k = 0.f, v_i = 0.f, v_b = 0.f;
    const Mode mk(h.mode_ker), mb(h.mode_bias);
    if (mine) {
        if (role == 0) {
            const int e = 64 * j + t;
            v_w = h.w[e], v_k = load_k(h.k_ker, e, mk.k_u8), v_i = h.i_ker[e], v_b = h.b_ker[e];
        } else if (role == 1) {
            v_w = h.bias[t], v_k = load_k(h.k_bias, t, mb.k_u8), v_i = h.i_bias[t], v_b = h.b_bias[t];
        } else {
            v_w = h.f_in[t];
        }
    }
    // what the first wavefront needs after the reduction is asked for now as well (the snapshot's column sums, tracked
    // integer bits and fractional bits of feature t; beta): loads issued behind the barrier would each cost a trip to memory
    float a_col = 0.f, a_i = 0.f, a_f = 0.f, beta = 0.f;
    if (grp == 0 && !loss_block) {
        const float *ax = aux + l * MLP_AUX + (e_local < K ? e_local : 0);
        a_col = ax[0], a_i = ax[64], a_f = ax[128];
        if (h.beta) beta = h.beta[0];
    }
    // both reductions of a thread (its entry's sums, its feature's abs-max) with all loads of a 16-slice run in flight
    {
        float s = 0.f;
        uint32_t mx = 0;
        const bool have_e = e_local < n_mine, have_a = !loss_block && e_local < K;
        const float *pe = part + p0 + (have_e ? e_local : 0);
        const uint32_t *pa = (const uint32_t *)part + ly.p_amax + (have_a ? e_local : 0);
        for (int g = g0; g < g1; g += 16) {
            float v[16];
            uint32_t a[16];
#pragma unroll
            for (int u = 0; u < 16; ++u) {
                const int64_t row = (int64_t)min(g + u, g1 - 1) * d.M;
                v[u] = pe[row], a[u] = pa[row];
            }
#pragma unroll
            for (int u = 0; u < 16; ++u)
                if (g + u >= g1) v[u] = 0.f, a[u] = 0u;
            s += (((v[0] + v[1]) + (v[2] + v[3])) + ((v[4] + v[5]) + (v[6] + v[7]))) +
                 (((v[8] + v[9]) + (v[10] + v[11])) + ((v[12] + v[13]) + (v[14] + v[15])));
#pragma unroll
            for (int u = 0; u < 16; ++u) mx = max(mx, a[u]);
        }
        red[threadIdx.x] = have_e ? s : 0.f;
        smx[threadIdx.x] = have_a ? mx : 0u;
    }
    __syncthreads();
    if (grp != 0) return;  // one wavefront applies the 64 updates
    {
        float v = 0.f;  // groups in order
#pragma unroll
        for (int w = 0; w < MLP_RG; w += 4)
            v += (red[e_local + 64 * w] + red[e_local + 64 * (w + 1)]) + (red[e_local + 64 * (w + 2)] + red[e_local + 64 * (w + 3)]);
        val[e_local] = v;
        if (!loss_block && e_local < K) {
            uint32_t mx = smx[e_local];
            for (int w = 1; w < MLP_RG; ++w) mx = max(mx, smx[e_local + 64 * w]);
            const float f = a_f;
            const float mi_ = ceil_log2_exact(__fadd_rn(__uint_as_float(mx), pow2(-f)));
            const float ni = fmaxf(__fsub_rn(a_i, h.decay), mi_);
            const float sfi = __fadd_rn(rintf(ni), f);
            float b = sfi > 0.f ? sfi : 0.f;
            const Mode mi(h.mode_in);
            if (mi.overflow_mode == HGQ_SAT) b += load_k(h.k_in, e_local, mi.k_u8);
            new_i[e_local] = ni, bits_in[e_local] = b, dbits_in[e_local] = sfi > 0.f ? 1.f : 0.f;
        } else {
            new_i[e_local] = 0.f, bits_in[e_local] = 0.f, dbits_in[e_local] = 0.f;
        }
    }
    // (one wavefront from here on: its LDS writes above are ordered before its reads below)
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
    __builtin_amdgcn_wave_barrier();
    if (loss_block) {
        if (loss) mlp_loss_piece(val[0], loss_word, loss_odd, loss, t);
        return;
    }
    // d(ebops * beta) / d bits: the chain rule through ((total * par_factor) / n_parallel) * ebops_factor * beta
    const float gs = __fmul_rn(__fdiv_rn(__fmul_rn(beta, h.ebops_factor), h.n_parallel), h.par_factor);
    float reg = 0.f;  // MonoL1 regularisation loss of the trainable bit-width variables (pre-update values)
    float ebops_term = 0.f;  // role 1, lane 0: the layer's ebops * beta
    if (role == 0) {
        const int e = 64 * j + t;
        if (t < n_mine) {
            const int k = e / N;
            const KIF p = resolve_kif(v_k, v_i, v_b, true, true);
            float dw, di, db;
            quantize_grad_dyn(v_w, val[t], p, mk.round_mode, mk.overflow_mode, dw, di, db);
            di -= db;  // f = b - i
            const float w_new = __fsub_rn(v_w, __fmul_rn(lr, dw));
            h.w[e] = w_new;
            reg += h.b_ker_l1 * v_b + (h.train_i_ker ? h.i_ker_l1 * v_i : 0.f);
            const float b_new = sgd_clip(v_b, db + bits_in[k] * gs, lr, h.b_ker_l1, h.b_ker_lo, h.b_ker_hi);
            h.b_ker[e] = b_new;
            float i_new = v_i;
            if (h.train_i_ker) h.i_ker[e] = i_new = sgd_clip(v_i, di, lr, h.i_ker_l1, h.i_ker_lo, h.i_ker_hi);
            // the next step's image entry, from the updated variables (what mlp_prep_kernel would compute)
            img[ly.off_w + k * ly.ldw + (e - k * N)] = quantize_dyn(w_new, resolve_kif(v_k, i_new, b_new, true, true), mk.round_mode,
                                                                    mk.overflow_mode, true);
        }
    } else if (role == 1) {
        float part_e = t < K ? bits_in[t] * a_col : 0.f;
        float bsum = 0.f;
        if (h.bias && t < N) {
            bsum = rintf(v_b);
            if (mb.overflow_mode == HGQ_SAT) bsum += v_k;
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) part_e += __shfl_xor(part_e, o, 64), bsum += __shfl_xor(bsum, o, 64);
        if (t == 0) {
            float total = part_e;
            if (h.bias) total += bsum / (float)N * h.bias_size;
            const float e = __fmul_rn(__fdiv_rn(__fmul_rn(total, h.par_factor), h.n_parallel), h.ebops_factor);
            if (h.ebops) h.ebops[0] = (uint32_t)e;
            ebops_term = e * beta;
        }
        if (h.bias && t < N) {
            const KIF p = resolve_kif(v_k, v_i, v_b, true, true);
            float dw, di, db;
            quantize_grad_dyn(v_w, val[t], p, mb.round_mode, mb.overflow_mode, dw, di, db);
            di -= db;
            const float w_new = __fsub_rn(v_w, __fmul_rn(lr, dw));
            h.bias[t] = w_new;
            reg += h.b_bias_l1 * v_b + (h.train_i_bias ? h.i_bias_l1 * v_i : 0.f);
            const float b_new = sgd_clip(v_b, db + h.bias_size / (float)N * gs, lr, h.b_bias_l1, h.b_bias_lo, h.b_bias_hi);
            h.b_bias[t] = b_new;
            float i_new = v_i;
            if (h.train_i_bias) h.i_bias[t] = i_new = sgd_clip(v_i, di, lr, h.i_bias_l1, h.i_bias_lo, h.i_bias_hi);
            img[ly.off_qb + t] = quantize_dyn(w_new, resolve_kif(v_k, i_new, b_new, true, true), mb.round_mode, mb.overflow_mode, true);
        }
    } else {
        if (t < K) {
            h.i_in[t] = new_i[t];
            reg += h.f_in_l1 * v_w;
            const float f_new = sgd_clip(v_w, val[t] + dbits_in[t] * a_col * gs, lr, h.f_in_l1, h.f_in_lo, h.f_in_hi);
            h.f_in[t] = f_new;
            img[ly.off_f + t] = rintf(f_new);
        }
    }
    if (loss) {
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) reg += __shfl_xor(reg, o, 64);
        mlp_loss_piece(ebops_term + reg, loss_word, loss_odd, loss, t);
    }
}

static int mlp_plan(const hgq_mlp_layer *layers, int n_layers, MlpDev &d, size_t &lds_bytes) {
    if (!layers || n_layers < 1 || n_layers > HGQ_MLP_MAX_LAYERS) return fail(HGQ_ERR_ARG, "hgq_mlp: 1..%d layers", HGQ_MLP_MAX_LAYERS);
    d.n_layers = n_layers;
    int off = 0, acol = 0, p = 0;
    for (int l = 0; l < n_layers; ++l) {
        MlpLayerDev &ly = d.l[l];
        ly.h = layers[l];
        const hgq_mlp_layer &h = ly.h;
        if (h.K < 1 || h.N < 1 || h.K > 64 || h.N > 64) return fail(HGQ_ERR_UNSUPPORTED, "hgq_mlp: layer %d is %d x %d; widths up to 64 are supported", l, h.K, h.N);
        if (l > 0 && h.K != layers[l - 1].N) return fail(HGQ_ERR_ARG, "hgq_mlp: layer %d input width %d != previous output width %d", l, h.K, layers[l - 1].N);
        if (!h.w || !h.k_in || !h.i_in || !h.f_in || !h.k_ker || !h.b_ker || !h.i_ker) return fail(HGQ_ERR_ARG, "hgq_mlp: null pointer in layer %d", l);
        if (h.bias && (!h.k_bias || !h.b_bias || !h.i_bias)) return fail(HGQ_ERR_ARG, "hgq_mlp: null bias quantizer pointer in layer %d", l);
        const Mode mi(h.mode_in), mk(h.mode_ker), mb(h.mode_bias);
        if (mi.kbi || mi.overflow_mode != HGQ_WRAP) return fail(HGQ_ERR_UNSUPPORTED, "hgq_mlp: input quantizers must be KIF WRAP (layer %d)", l);
        if (!mk.kbi || (h.bias && !mb.kbi)) return fail(HGQ_ERR_UNSUPPORTED, "hgq_mlp: kernel / bias quantizers must be KBI (layer %d)", l);
        if (mk.overflow_mode == HGQ_WRAP || (h.bias && mb.overflow_mode == HGQ_WRAP))
            return fail(HGQ_ERR_UNSUPPORTED, "hgq_mlp: WRAP kernel / bias quantizers track their integer bits per call and are not fused (layer %d)", l);
        if (h.act != HGQ_ACT_NONE && h.act != HGQ_ACT_RELU) return fail(HGQ_ERR_ARG, "hgq_mlp: unknown activation in layer %d", l);
        ly.Kp = (h.K + 31) & ~31;
        ly.Np = (h.N + 31) & ~31;
        ly.ldw = ly.Np + 1;
        ly.off_w = off, off += ly.Kp * ly.ldw;
        ly.off_qb = off, off += ly.Np;
        ly.off_f = off, off += ly.Kp;
        ly.acol = acol, acol += ly.Kp;
        ly.p_dw = p, p += h.K * h.N;
        ly.p_db = p, p += h.N;
        ly.p_df = p, p += h.K;
        ly.p_amax = p, p += h.K;
    }
    d.n_classes = layers[n_layers - 1].N;
    d.acol_out = acol;
    d.ld_rx = acol + 1;
    d.ld_raw = acol + d.l[n_layers - 1].Np + 1;
    d.p_loss = p, p += 1;
    d.M = p;
    off = (off + 3) & ~3;
    d.off_raw = off, off += MLP_BM * d.ld_raw;
    d.off_rx = off, off += MLP_BM * d.ld_rx;
    d.off_dz0 = off, off += MLP_BM * MLP_LDZ;
    d.off_dz1 = off, off += MLP_BM * MLP_LDZ;
    d.off_red = off, off += 3 * 64 * HGQ_MLP_MAX_LAYERS;  // fractional-bit sums (two sets) and abs-max, [layers][64] each
    lds_bytes = (size_t)off * 4;
    if (lds_bytes > 160 * 1024 - 512) return fail(HGQ_ERR_UNSUPPORTED, "hgq_mlp: the stack needs %zu bytes of LDS", lds_bytes);
    return HGQ_OK;
}

static inline int mlp_parts(int64_t rows) {
    const int64_t n_tiles = (rows + MLP_BM - 1) / MLP_BM;
    return persistent_grid(n_tiles, 1);
}

}  // namespace hgq

using namespace hgq;

#ifdef MLP_PROF
extern "C" int hgq_mlp_prof_read(unsigned long long *out) {
    return hipMemcpyFromSymbol(out, HIP_SYMBOL(mlp_prof_stamps), sizeof(unsigned long long) * 8 * 64) == hipSuccess ? 0 : -2;
}
#endif

extern "C" int64_t hgq_mlp_workspace(const hgq_mlp_layer *layers, int n_layers, int64_t rows) {
    MlpDev d;
    size_t lds_bytes;
    if (mlp_plan(layers, n_layers, d, lds_bytes)) return -1;
    return (int64_t)(mlp_parts(rows > 0 ? rows : 1) + 1) * d.M + (int64_t)n_layers * MLP_AUX + d.off_raw + 4 + 64;  // (+ 64: the loss words and their alignment)
}

extern "C" int hgq_mlp_train_step_cached(const hgq_mlp_layer *layers, int n_layers, const float *x, const int64_t *labels,
                                         int64_t rows, float lr, float *loss, float *workspace, int image_current, void *stream) {
    hipStream_t s = (hipStream_t)stream;
    MlpDev d;
    size_t lds_bytes;
    int rc = mlp_plan(layers, n_layers, d, lds_bytes);
    if (rc) return rc;
    if (rows < 1 || !x || !labels || !workspace) return fail(HGQ_ERR_ARG, "hgq_mlp_train_step: bad arguments");
    if ((uintptr_t)workspace & 15u) return fail(HGQ_ERR_ARG, "hgq_mlp_train_step: the workspace must be 16-byte aligned");
    static bool raised = false;
    if (!raised) {
        hipError_t e = hipFuncSetAttribute((const void *)mlp_fwd_bwd_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 512);
        if (e != hipSuccess) return fail(HGQ_ERR_LAUNCH, "hgq_mlp_train_step: hipFuncSetAttribute: %s", hipGetErrorString(e));
        raised = true;
    }
    const int parts = mlp_parts(rows);
    // workspace: [image | per-workgroup slices | per-layer snapshot of pre-update variables]; the image comes first so
    // that its place does not depend on the batch size
    float *img = workspace;
    float *slices = workspace + ((d.off_raw + 3) & ~3);
    float *reduced = slices + (int64_t)parts * d.M;
    if (!image_current) {
        hipLaunchKernelGGL(mlp_prep_kernel, dim3((d.off_raw + 255) / 256), dim3(256), 0, s, d, img);
        if ((rc = check_launch("hgq_mlp_train_step(prep)"))) return rc;
    }
    // behind the snapshot: the word the update pass adds its loss pieces into (8-byte aligned) and the word beside it
    uint32_t *loss_words = (uint32_t *)(((uintptr_t)(reduced + (int64_t)n_layers * MLP_AUX) + 7u) & ~(uintptr_t)7u);
    int blocks = 1;
    for (int l = 0; l < n_layers; ++l) blocks += (layers[l].K * layers[l].N + 63) / 64 + 2;
    hipLaunchKernelGGL(mlp_fwd_bwd_kernel, dim3(parts), dim3(MLP_NT), lds_bytes, s, d, img, x, labels, rows, slices, reduced, loss_words);
    if ((rc = check_launch("hgq_mlp_train_step(fwd_bwd)"))) return rc;
    hipLaunchKernelGGL(mlp_reduce_update_kernel, dim3(blocks), dim3(64 * MLP_RG), 0, s, d, slices, parts, reduced, lr, loss, img,
                       (unsigned long long *)loss_words, loss_words + 2);
    return check_launch("hgq_mlp_train_step(update)");
}

extern "C" int hgq_mlp_train_step(const hgq_mlp_layer *layers, int n_layers, const float *x, const int64_t *labels,
                                  int64_t rows, float lr, float *loss, float *workspace, void *stream) {
    return hgq_mlp_train_step_cached(layers, n_layers, x, labels, rows, lr, loss, workspace, 0, stream);
}
