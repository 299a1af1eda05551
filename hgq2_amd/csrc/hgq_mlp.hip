// One training step of a stack of QDense layers in four launches.
//
// At the layer sizes HGQ targets (tens of units per layer) a training step built from per-layer
// kernels is bound by launch latency, not by HBM or MFMA.  Here the whole data path - every
// layer's input quantizer, contraction, bias, activation, the sparse cross-entropy loss and the
// full backward pass - runs in ONE kernel: the quantized weights of all layers sit in LDS
// (a few tens of KB), a workgroup takes a tile of 64 samples through forward and backward without
// touching HBM in between, and writes its partial gradient sums to a private slice.  A second
// kernel adds the slices in a fixed order; a third applies, per layer, the integer-bit tracking,
// EBOPs (value, variable and gradient), the weight / bias quantizer backward and the SGD update
// with the MonoL1 gradient and the clip constraints folded in.
//
// HBM traffic per step is the input batch, the labels and the partial slices.
#include "hgq_device.h"
#include "hgq_host.h"

namespace hgq {


#define MLP_BM 64
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

__global__ __launch_bounds__(MLP_NT) void mlp_fwd_bwd_kernel(MlpDev d, const float *__restrict__ img, const float *__restrict__ x,
                                                          const int64_t *__restrict__ labels, int64_t rows,
                                                          float *part) {
    extern __shared__ float lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int L = d.n_layers;
    float *raw = lds + d.off_raw, *rx = lds + d.off_rx;
    float *dfs = lds + d.off_red;                                 // [L][64] fractional-bit gradient sums
    uint32_t *amx = (uint32_t *)(lds + d.off_red) + 64 * HGQ_MLP_MAX_LAYERS;  // [L][64] abs-max of each layer's quantized input
    float *my = part + (int64_t)blockIdx.x * d.M;
    const int64_t n_tiles = (rows + MLP_BM - 1) / MLP_BM;
    const float inv_rows = 1.0f / (float)rows;

    // ---- prologue: fetch the quantized kernels / biases / rounded fractional bits (off_raw is a multiple of 4)
    // (four 128-bit loads per thread in flight: one load per loop trip would cost a memory latency each)
    for (int id0 = 0; id0 < d.off_raw; id0 += 4 * 4 * MLP_NT) {
        float4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int id = id0 + (u * MLP_NT + tid) * 4;
            v[u] = *(const float4 *)(img + (id < d.off_raw ? id : 0));
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int id = id0 + (u * MLP_NT + tid) * 4;
            if (id < d.off_raw) *(float4 *)(lds + id) = v[u];
        }
    }
    for (int id = tid; id < MLP_BM * d.ld_rx; id += MLP_NT) rx[id] = 0.f;  // padding columns stay zero for good
    for (int id = tid; id < 64 * HGQ_MLP_MAX_LAYERS; id += MLP_NT) dfs[id] = 0.f, amx[id] = 0u;
    __syncthreads();

    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const bool first = tile == blockIdx.x;
        const int64_t r0 = tile * MLP_BM;
        // ---- stage the input tile: raw value, quantized value, abs-max
        {
            const MlpLayerDev &l0 = d.l[0];
            const int K0 = l0.h.K, rm = Mode(l0.h.mode_in).round_mode;
            const float *fl = lds + l0.off_f;
            // the tile's rows are contiguous in x: buffer loads, zeros past the last row, four in flight
            const int64_t left = rows - r0;
            const int n_el = MLP_BM * K0;
            const __amdgpu_buffer_rsrc_t rs = buf_rsrc(x + r0 * K0, (left < MLP_BM ? left : MLP_BM) * K0 * 4);
            for (int id0 = 0; id0 < n_el; id0 += 4 * MLP_NT) {
                float v[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int id = id0 + u * MLP_NT + tid;
                    v[u] = buf_ld1(rs, id < n_el ? (uint32_t)id * 4u : BUF_OOB);
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int id = id0 + u * MLP_NT + tid;
                    if (id < n_el) {
                        const int row = id / K0, k = id - row * K0;
                        float q = 0.f;
                        if (r0 + row < rows) {
                            q = fixed_round_dyn(v[u], fl[k], rm);
                            atomicMax(&amx[k], abs_bits(q));
                        }
                        raw[row * d.ld_raw + l0.acol + k] = v[u];
                        rx[row * d.ld_rx + l0.acol + k] = q;
                    }
                }
            }
        }
        __syncthreads();
        // ================= forward =================
        for (int l = 0; l < L; ++l) {
            const MlpLayerDev &ly = d.l[l];
            const int N = ly.h.N;
            const int rh = wave & 1, cb = wave >> 1;
            if (wave < 4 && cb * 32 < ly.Np) {
                floatx16 acc = {0};
                const float *ws = lds + ly.off_w;
                const int arow = rh * 32 + (lane & 31), kq = lane >> 5, bcol = cb * 32 + (lane & 31);
                // input columns and kernel rows are zero padded to a multiple of 32
                acc = mfma_chain(acc, rx + arow * d.ld_rx + ly.acol + kq, 1, ws + kq * ly.ldw + bcol, ly.ldw, (ly.h.K + 15) >> 4);
                if (bcol < N) {
                    const float bias = lds[ly.off_qb + bcol];
                    const bool last = l + 1 == L;
                    const int ocol = (last ? d.acol_out : d.l[l + 1].acol) + bcol;
                    // the next layer's input quantizer runs here, on the accumulator registers
                    const float fn = last ? 0.f : lds[d.l[l + 1].off_f + bcol];
                    const int rm = last ? 0 : Mode(d.l[l + 1].h.mode_in).round_mode;
                    uint32_t mx = 0;
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int row = rh * 32 + acc_row_(r, lane);
                        float v = acc[r] + bias;
                        if (ly.h.act == HGQ_ACT_RELU) v = v > 0.f ? v : 0.f;
                        raw[row * d.ld_raw + ocol] = v;
                        if (!last) {
                            const float q = (r0 + row < rows) ? fixed_round_dyn(v, fn, rm) : 0.f;
                            rx[row * d.ld_rx + ocol] = q;
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
            __syncthreads();
        }
        // ================= loss: mean sparse categorical cross-entropy from logits =================
        float *cur = lds + d.off_dz0, *nxt = lds + d.off_dz1;
        {
            const int C = d.n_classes;
            const int Cp = d.l[L - 1].Np;
            float lrow = 0.f;
            if (tid < MLP_BM) {
                const int64_t gr = r0 + tid;
                const float *z = raw + tid * d.ld_raw + d.acol_out;
                float *dz = cur + tid * MLP_LDZ;
                if (gr < rows) {
                    float mx = z[0];
                    for (int c = 1; c < C; ++c) mx = fmaxf(mx, z[c]);
                    float se = 0.f;
                    for (int c = 0; c < C; ++c) se += expf(z[c] - mx);
                    const int lab = (int)labels[gr];
                    lrow = logf(se) - (z[lab] - mx);
                    const float inv = 1.0f / se;
                    for (int c = 0; c < C; ++c) dz[c] = (expf(z[c] - mx) * inv - (c == lab ? 1.0f : 0.0f)) * inv_rows;
                    for (int c = C; c < Cp; ++c) dz[c] = 0.f;
                } else {
                    for (int c = 0; c < Cp; ++c) dz[c] = 0.f;
                }
            }
            if (wave == 0) {
#pragma unroll
                for (int o = 32; o > 0; o >>= 1) lrow += __shfl_xor(lrow, o, 64);
                if (lane == 0) my[d.p_loss] = (first ? 0.f : my[d.p_loss]) + lrow * inv_rows;
            }
        }
        __syncthreads();
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
                acc = mfma_chain(acc, rx + kq * d.ld_rx + ly.acol + wkb * 32 + c32, d.ld_rx, cur + kq * MLP_LDZ + wnb * 32 + c32, MLP_LDZ,
                                 MLP_BM / 16);
                const int n = wnb * 32 + c32;
                if (n < N) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int k = wkb * 32 + acc_row_(r, lane);
                        if (k < K) {
                            float *dst = my + ly.p_dw + k * N + n;
                            *dst = first ? acc[r] : *dst + acc[r];
                        }
                    }
                }
            }
            // ---- bias gradient: the last wave is free of kernel-gradient work unless all four blocks exist
            if (ly.h.bias && wave == 7 && lane < N) {
                float s0 = 0.f, s1 = 0.f;
#pragma unroll 8
                for (int r = 0; r < MLP_BM; r += 2) s0 += cur[r * MLP_LDZ + lane], s1 += cur[(r + 1) * MLP_LDZ + lane];
                float *dst = my + ly.p_db + lane;
                *dst = first ? s0 + s1 : *dst + (s0 + s1);
            }
            // ---- input gradient, the relu mask of the layer below, and this layer's fractional-bit gradient
            {
                const int rh = wave & 1, kb = wave >> 1;
                if (wave < 4 && kb < K32) {
                    floatx16 acc = {0};
                    const float *ws = lds + ly.off_w;
                    const int arow = rh * 32 + (lane & 31), kq = lane >> 5, wrow = kb * 32 + (lane & 31);
                    // gradient columns and kernel columns are zero padded to a multiple of 32
                    acc = mfma_chain(acc, cur + arow * MLP_LDZ + kq, 1, ws + wrow * ly.ldw + kq, 1, (N + 15) >> 4);
                    const int kcol = kb * 32 + (lane & 31);
                    const bool mask_below = l > 0 && d.l[l - 1].h.act == HGQ_ACT_RELU;
                    float dfsum = 0.f;
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int row = rh * 32 + acc_row_(r, lane);
                        const float a = raw[row * d.ld_raw + ly.acol + kcol];
                        const float delta = rx[row * d.ld_rx + ly.acol + kcol] - a;
                        if (kcol < K && r0 + row < rows) dfsum += -HGQ_LN2 * delta * acc[r];
                        nxt[row * MLP_LDZ + kcol] = (kcol < K && (!mask_below || a > 0.f)) ? acc[r] : 0.f;
                    }
                    dfsum += __shfl_xor(dfsum, 32, 64);
                    if (lane < 32 && kcol < K) atomicAdd(&dfs[l * 64 + kcol], dfsum);
                }
            }
            __syncthreads();
            float *t = cur;
            cur = nxt;
            nxt = t;
        }
    }
    // ---- this workgroup's abs-max and fractional-bit sums
    for (int l = 0; l < L; ++l) {
        const MlpLayerDev &ly = d.l[l];
        if (tid < ly.h.K) {
            my[ly.p_df + tid] = dfs[l * 64 + tid];
            ((uint32_t *)(my + ly.p_amax))[tid] = amx[l * 64 + tid];
        }
    }
}

#define MLP_AUX 192  // per layer, after the M reduced sums: colsum[64], bits_in[64], dbits_in[64]

// Blocks [0, ceil(M/64)): out[e] = sum over slices of part[g][e] (the abs-max sections are skipped
// here).  Blocks beyond that, one per layer: reduce the layer's abs-max section, track the input
// quantizer's integer bits in place, and leave for the update pass - which must not read variables
// another workgroup is updating - the per-feature bit counts of the input quantizer and the
// per-row sums of the kernel bit counts, all from the pre-update variables.
#define MLP_RG 16  // slice groups per entry: 64 entries x 16 groups = 1024 threads, few loads per thread
__global__ __launch_bounds__(64 * MLP_RG) void mlp_reduce_kernel(MlpDev d, const float *__restrict__ part, int n_parts, float *out,
                                                         float *loss) {
    __shared__ float red[64 * MLP_RG];
    const int e_local = threadIdx.x & 63, grp = threadIdx.x >> 6;
    const int n_main = (d.M + 63) / 64;
    const int per = (n_parts + MLP_RG - 1) / MLP_RG;
    const int g0 = grp * per, g1 = min(n_parts, g0 + per);
    if ((int)blockIdx.x < n_main) {
        const int64_t e = (int64_t)blockIdx.x * 64 + e_local;
        float s = 0.f;
        if (e < d.M) {
            int g = g0;
            for (; g + 8 <= g1; g += 8) {
                float v[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) v[u] = part[(int64_t)(g + u) * d.M + e];
                s += ((v[0] + v[1]) + (v[2] + v[3])) + ((v[4] + v[5]) + (v[6] + v[7]));
            }
            for (; g < g1; ++g) s += part[(int64_t)g * d.M + e];
        }
        red[threadIdx.x] = s;
        __syncthreads();
        if (grp == 0 && e < d.M) {
            float v = 0.f;  // groups in order
#pragma unroll
            for (int w = 0; w < MLP_RG; w += 4)
                v += (red[e_local + 64 * w] + red[e_local + 64 * (w + 1)]) + (red[e_local + 64 * (w + 2)] + red[e_local + 64 * (w + 3)]);
            out[e] = v;
            if (e == d.p_loss && loss) loss[0] = v;
        }
        return;
    }
    const int l = blockIdx.x - n_main;
    const MlpLayerDev &ly = d.l[l];
    const hgq_mlp_layer &h = ly.h;
    const int k = e_local, K = h.K, N = h.N;
    const Mode mk(h.mode_ker), mi(h.mode_in);
    uint32_t mx = 0;
    float cs = 0.f;
    if (k < K) {
        const uint32_t *pa = (const uint32_t *)part + ly.p_amax + k;
        int g = g0;
        for (; g + 8 <= g1; g += 8) {
            uint32_t v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = pa[(int64_t)(g + u) * d.M];
#pragma unroll
            for (int u = 0; u < 8; ++u) mx = max(mx, v[u]);
        }
        for (; g < g1; ++g) mx = max(mx, pa[(int64_t)g * d.M]);
        // this thread's share of row k of the kernel bit counts
        const int nper = (N + MLP_RG - 1) / MLP_RG, n0 = grp * nper, n1 = min(N, n0 + nper);
        for (int n = n0; n < n1; ++n) {
            float bk = rintf(h.b_ker[k * N + n]);
            if (mk.overflow_mode == HGQ_SAT) bk += load_k(h.k_ker, k * N + n, mk.k_u8);
            cs += bk;
        }
    }
    __shared__ uint32_t smx[64 * MLP_RG];
    smx[threadIdx.x] = mx;
    red[threadIdx.x] = cs;
    __syncthreads();
    if (grp == 0 && k < K) {
        for (int w = 1; w < MLP_RG; ++w) mx = max(mx, smx[k + 64 * w]);
        const float f = rintf(h.f_in[k]);
        const float mi_ = ceil_log2_exact(__fadd_rn(__uint_as_float(mx), pow2(-f)));
        const float ni = fmaxf(__fsub_rn(h.i_in[k], h.decay), mi_);
        h.i_in[k] = ni;
        const float sfi = __fadd_rn(rintf(ni), f);
        float b = sfi > 0.f ? sfi : 0.f;
        if (mi.overflow_mode == HGQ_SAT) b += load_k(h.k_in, k, mi.k_u8);
        float *aux = out + d.M + l * MLP_AUX;
        float csum = 0.f;  // integers: exact in any order
        for (int w = 0; w < MLP_RG; ++w) csum += red[k + 64 * w];
        aux[k] = csum;
        aux[64 + k] = b;
        aux[128 + k] = sfi > 0.f ? 1.f : 0.f;
    }
}

__device__ __forceinline__ float sgd_clip(float w, float g, float lr, float l1, float lo, float hi) {
    return fminf(fmaxf(__fsub_rn(w, __fmul_rn(lr, __fadd_rn(g, l1))), lo), hi);
}

#define MLP_UPD_SPLIT 8

// Grid (layers, MLP_UPD_SPLIT).  Each workgroup updates its share of the layer's kernel entries;
// the first one of a layer also owns EBOPs, the bias and the input quantizer's fractional bits.
// Everything a workgroup needs about variables it does not own comes from the reduce pass.
__global__ __launch_bounds__(256) void mlp_update_kernel(MlpDev d, const float *__restrict__ g, float lr, float *loss, float *img) {
    __shared__ float colsum[64];   // sum_n bits_ker[k, n]
    __shared__ float bits_in[64];  // relu(round(i) + round(f)) with the tracked i
    __shared__ float dbits_in[64];
    const MlpLayerDev &ly = d.l[blockIdx.x];
    const hgq_mlp_layer &h = ly.h;
    const int tid = threadIdx.x, K = h.K, N = h.N;
    const bool owner = blockIdx.y == 0;
    const Mode mk(h.mode_ker), mb(h.mode_bias);
    if (tid < 64) {
        const float *aux = g + d.M + blockIdx.x * MLP_AUX;
        colsum[tid] = aux[tid], bits_in[tid] = aux[64 + tid], dbits_in[tid] = aux[128 + tid];
    }
    __syncthreads();
    const float beta = h.beta ? h.beta[0] : 0.f;
    const float gs = h.ebops_scale * beta;  // d(ebops * beta) / d bits
    float reg = 0.f;  // MonoL1 regularisation loss of the trainable bit-width variables (pre-update values)
    if (owner) {
        float part = tid < K ? bits_in[tid] * colsum[tid] : 0.f;
        float bsum = 0.f;
        if (h.bias && tid < N) {
            bsum = rintf(h.b_bias[tid]);
            if (mb.overflow_mode == HGQ_SAT) bsum += load_k(h.k_bias, tid, mb.k_u8);
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) part += __shfl_xor(part, o, 64), bsum += __shfl_xor(bsum, o, 64);
        if (tid == 0) {  // K, N <= 64: wave 0 holds every non-zero term
            float total = part;
            if (h.bias) total += bsum / (float)N * h.bias_size;
            const float e = total * h.ebops_scale;
            if (h.ebops) h.ebops[0] = (uint32_t)e;
            if (loss) atomicAdd(loss, e * beta);
        }
        if (h.bias && tid < N) {
            const KIF p = kbi_entry(h.k_bias, h.i_bias, h.b_bias, tid, h.mode_bias);
            float dw, di, db;
            quantize_grad_dyn(h.bias[tid], g[ly.p_db + tid], p, mb.round_mode, mb.overflow_mode, dw, di, db);
            di -= db;
            h.bias[tid] = __fsub_rn(h.bias[tid], __fmul_rn(lr, dw));
            reg += h.b_bias_l1 * h.b_bias[tid] + (h.train_i_bias ? h.i_bias_l1 * h.i_bias[tid] : 0.f);
            h.b_bias[tid] = sgd_clip(h.b_bias[tid], db + h.bias_size / (float)N * gs, lr, h.b_bias_l1, h.b_bias_lo, h.b_bias_hi);
            if (h.train_i_bias) h.i_bias[tid] = sgd_clip(h.i_bias[tid], di, lr, h.i_bias_l1, h.i_bias_lo, h.i_bias_hi);
            // the next step's image entry, from the updated variables (what mlp_prep_kernel would compute)
            img[ly.off_qb + tid] = quantize_dyn(h.bias[tid], kbi_entry(h.k_bias, h.i_bias, h.b_bias, tid, h.mode_bias), mb.round_mode,
                                                mb.overflow_mode, true);
        }
        if (tid < K) {
            reg += h.f_in_l1 * h.f_in[tid];
            h.f_in[tid] = sgd_clip(h.f_in[tid], g[ly.p_df + tid] + dbits_in[tid] * colsum[tid] * gs, lr, h.f_in_l1, h.f_in_lo, h.f_in_hi);
            img[ly.off_f + tid] = rintf(h.f_in[tid]);
        }
    }
    // quantizer backward of this workgroup's kernel entries, SGD + constraints
    for (int e = blockIdx.y * 256 + tid; e < K * N; e += MLP_UPD_SPLIT * 256) {
        const int k = e / N;
        const KIF p = kbi_entry(h.k_ker, h.i_ker, h.b_ker, e, h.mode_ker);
        float dw, di, db;
        quantize_grad_dyn(h.w[e], g[ly.p_dw + e], p, mk.round_mode, mk.overflow_mode, dw, di, db);
        di -= db;  // f = b - i
        h.w[e] = __fsub_rn(h.w[e], __fmul_rn(lr, dw));
        reg += h.b_ker_l1 * h.b_ker[e] + (h.train_i_ker ? h.i_ker_l1 * h.i_ker[e] : 0.f);
        h.b_ker[e] = sgd_clip(h.b_ker[e], db + bits_in[k] * gs, lr, h.b_ker_l1, h.b_ker_lo, h.b_ker_hi);
        if (h.train_i_ker) h.i_ker[e] = sgd_clip(h.i_ker[e], di, lr, h.i_ker_l1, h.i_ker_lo, h.i_ker_hi);
        img[ly.off_w + k * ly.ldw + (e - k * N)] = quantize_dyn(h.w[e], kbi_entry(h.k_ker, h.i_ker, h.b_ker, e, h.mode_ker), mk.round_mode,
                                                                mk.overflow_mode, true);
    }
    if (loss) {
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) reg += __shfl_xor(reg, o, 64);
        if ((tid & 63) == 0 && reg != 0.f) atomicAdd(loss, reg);
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
    d.off_red = off, off += 2 * 64 * HGQ_MLP_MAX_LAYERS;  // fractional-bit sums and abs-max, [layers][64] each
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

extern "C" int64_t hgq_mlp_workspace(const hgq_mlp_layer *layers, int n_layers, int64_t rows) {
    MlpDev d;
    size_t lds_bytes;
    if (mlp_plan(layers, n_layers, d, lds_bytes)) return -1;
    return (int64_t)(mlp_parts(rows > 0 ? rows : 1) + 1) * d.M + (int64_t)n_layers * MLP_AUX + d.off_raw + 4;
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
    // workspace: [image | per-workgroup slices | reduced sums + per-layer aux]; the image comes first so
    // that its place does not depend on the batch size
    float *img = workspace;
    float *slices = workspace + ((d.off_raw + 3) & ~3);
    float *reduced = slices + (int64_t)parts * d.M;
    if (!image_current) {
        hipLaunchKernelGGL(mlp_prep_kernel, dim3((d.off_raw + 255) / 256), dim3(256), 0, s, d, img);
        if ((rc = check_launch("hgq_mlp_train_step(prep)"))) return rc;
    }
    hipLaunchKernelGGL(mlp_fwd_bwd_kernel, dim3(parts), dim3(MLP_NT), lds_bytes, s, d, img, x, labels, rows, slices);
    if ((rc = check_launch("hgq_mlp_train_step(fwd_bwd)"))) return rc;
    hipLaunchKernelGGL(mlp_reduce_kernel, dim3((d.M + 63) / 64 + n_layers), dim3(64 * MLP_RG), 0, s, d, slices, parts, reduced, loss);
    if ((rc = check_launch("hgq_mlp_train_step(reduce)"))) return rc;
    hipLaunchKernelGGL(mlp_update_kernel, dim3(n_layers, MLP_UPD_SPLIT), dim3(256), 0, s, d, reduced, lr, loss, img);
    return check_launch("hgq_mlp_train_step(update)");
}

extern "C" int hgq_mlp_train_step(const hgq_mlp_layer *layers, int n_layers, const float *x, const int64_t *labels,
                                  int64_t rows, float lr, float *loss, float *workspace, void *stream) {
    return hgq_mlp_train_step_cached(layers, n_layers, x, labels, rows, lr, loss, workspace, 0, stream);
}
