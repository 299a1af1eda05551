// One training step of a stack of QDense layers in three launches.
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

typedef float floatx16 __attribute__((ext_vector_type(16)));

#define MLP_BM 64
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

__global__ __launch_bounds__(256) void mlp_fwd_bwd_kernel(MlpDev d, const float *__restrict__ x,
                                                          const int64_t *__restrict__ labels, int64_t rows,
                                                          float *part) {
    extern __shared__ float lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int L = d.n_layers;
    float *raw = lds + d.off_raw, *rx = lds + d.off_rx, *red = lds + d.off_red;
    float *my = part + (int64_t)blockIdx.x * d.M;
    const int64_t n_tiles = (rows + MLP_BM - 1) / MLP_BM;
    const float inv_rows = 1.0f / (float)rows;

    // ---- prologue: quantize every layer's kernel and bias into LDS (zero padded), round f
    for (int l = 0; l < L; ++l) {
        const MlpLayerDev &ly = d.l[l];
        const Mode mk(ly.h.mode_ker), mb(ly.h.mode_bias);
        float *ws = lds + ly.off_w;
        for (int id = tid; id < ly.Kp * ly.ldw; id += 256) {
            const int k = id / ly.ldw, n = id - k * ly.ldw;
            float v = 0.f;
            if (k < ly.h.K && n < ly.h.N) {
                const int64_t e = (int64_t)k * ly.h.N + n;
                v = quantize_dyn(ly.h.w[e], kbi_entry(ly.h.k_ker, ly.h.i_ker, ly.h.b_ker, e, ly.h.mode_ker), mk.round_mode,
                                 mk.overflow_mode, true);
            }
            ws[id] = v;
        }
        for (int n = tid; n < ly.Np; n += 256) {
            float v = 0.f;
            if (n < ly.h.N && ly.h.bias)
                v = quantize_dyn(ly.h.bias[n], kbi_entry(ly.h.k_bias, ly.h.i_bias, ly.h.b_bias, n, ly.h.mode_bias), mb.round_mode,
                                 mb.overflow_mode, true);
            lds[ly.off_qb + n] = v;
        }
        for (int k = tid; k < ly.Kp; k += 256) lds[ly.off_f + k] = k < ly.h.K ? rintf(ly.h.f_in[k]) : 0.f;
    }
    for (int id = tid; id < MLP_BM * d.ld_raw; id += 256) raw[id] = 0.f;
    __syncthreads();

    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const bool first = tile == blockIdx.x;
        const int64_t r0 = tile * MLP_BM;
        // ---- stage the input batch tile
        {
            const int K0 = d.l[0].h.K;
            for (int id = tid; id < MLP_BM * K0; id += 256) {
                const int row = id / K0, k = id - row * K0;
                const int64_t gr = r0 + row;
                raw[row * d.ld_raw + d.l[0].acol + k] = gr < rows ? x[gr * K0 + k] : 0.f;
            }
        }
        __syncthreads();
        // ================= forward =================
        for (int l = 0; l < L; ++l) {
            const MlpLayerDev &ly = d.l[l];
            const int K = ly.h.K, N = ly.h.N;
            const int rm = Mode(ly.h.mode_in).round_mode;
            const float *fl = lds + ly.off_f;
            for (int id = tid; id < MLP_BM * ly.Kp; id += 256) {
                const int row = id / ly.Kp, k = id - row * ly.Kp;
                float v = 0.f;
                if (k < K && r0 + row < rows) v = fixed_round_dyn(raw[row * d.ld_raw + ly.acol + k], fl[k], rm);
                rx[row * d.ld_rx + ly.acol + k] = v;
            }
            __syncthreads();
            if (tid < K) {  // abs-max of the quantized input, per feature
                uint32_t mx = 0;
#pragma unroll 8
                for (int r = 0; r < MLP_BM; ++r) {
                    const uint32_t a = abs_bits(rx[r * d.ld_rx + ly.acol + tid]);
                    mx = a > mx ? a : mx;
                }
                uint32_t *dst = (uint32_t *)(my + ly.p_amax) + tid;
                if (first || mx > *dst) *dst = mx;
            }
            {
                const int rh = wave & 1, cb = wave >> 1;
                if (cb * 32 < ly.Np) {
                    floatx16 acc = {0};
                    const float *ws = lds + ly.off_w;
                    const int arow = rh * 32 + (lane & 31), kq = lane >> 5, bcol = cb * 32 + (lane & 31);
                    for (int kk = 0; kk < ly.Kp; kk += 2)
                        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(rx[arow * d.ld_rx + ly.acol + kk + kq], ws[(kk + kq) * ly.ldw + bcol], acc, 0, 0, 0);
                    if (bcol < N) {
                        const float bias = lds[ly.off_qb + bcol];
                        const int ocol = (l + 1 < L ? d.l[l + 1].acol : d.acol_out) + bcol;
#pragma unroll
                        for (int r = 0; r < 16; ++r) {
                            float v = acc[r] + bias;
                            if (ly.h.act == HGQ_ACT_RELU) v = v > 0.f ? v : 0.f;
                            raw[(rh * 32 + acc_row_(r, lane)) * d.ld_raw + ocol] = v;
                        }
                    }
                }
            }
            __syncthreads();
        }
        // ================= loss: mean sparse categorical cross-entropy from logits =================
        float *cur = lds + d.off_dz0, *nxt = lds + d.off_dz1;
        {
            const int C = d.n_classes;
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
                    for (int c = C; c < 64; ++c) dz[c] = 0.f;
                } else {
                    for (int c = 0; c < 64; ++c) dz[c] = 0.f;
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
        for (int l = L - 1; l >= 0; --l) {
            const MlpLayerDev &ly = d.l[l];
            const int K = ly.h.K, N = ly.h.N;
            const int K32 = ly.Kp >> 5, N32 = ly.Np >> 5;
            if (ly.h.act == HGQ_ACT_RELU) {
                const int ocol = l + 1 < L ? d.l[l + 1].acol : d.acol_out;
                for (int id = tid; id < MLP_BM * N; id += 256) {
                    const int row = id / N, n = id - row * N;
                    if (!(raw[row * d.ld_raw + ocol + n] > 0.f)) cur[row * MLP_LDZ + n] = 0.f;
                }
                __syncthreads();
            }
            for (int id = tid; id < ly.Kp; id += 256) red[id] = 0.f;  // fractional-bit gradient of this layer's input
            // ---- kernel gradient: one 32 x 32 block per wave over the whole tile
            {
                const int nblk = K32 * N32;
                if (wave < nblk) {
                    const int wkb = wave / N32, wnb = wave % N32;
                    floatx16 acc = {0};
                    const int kq = lane >> 5, c32 = lane & 31;
                    for (int rr = 0; rr < MLP_BM; rr += 2)
                        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(rx[(rr + kq) * d.ld_rx + ly.acol + wkb * 32 + c32],
                                                                   cur[(rr + kq) * MLP_LDZ + wnb * 32 + c32], acc, 0, 0, 0);
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
            }
            // ---- bias gradient
            if (tid < N) {
                float s = 0.f;
#pragma unroll 8
                for (int r = 0; r < MLP_BM; ++r) s += cur[r * MLP_LDZ + tid];
                float *dst = my + ly.p_db + tid;
                *dst = first ? s : *dst + s;
            }
            __syncthreads();  // red zeroed, cur fully read by the bias sums before nxt/cur swap matters
            // ---- input gradient and the fractional-bit gradient of the input quantizer
            {
                const int rh = wave & 1, kb = wave >> 1;
                if (kb < K32) {
                    floatx16 acc = {0};
                    const float *ws = lds + ly.off_w;
                    const int arow = rh * 32 + (lane & 31), kq = lane >> 5, wrow = kb * 32 + (lane & 31);
                    for (int nn = 0; nn < ly.Np; nn += 2)
                        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(cur[arow * MLP_LDZ + nn + kq], ws[wrow * ly.ldw + nn + kq], acc, 0, 0, 0);
                    const int kcol = kb * 32 + (lane & 31);
                    float dfsum = 0.f;
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int row = rh * 32 + acc_row_(r, lane);
                        nxt[row * MLP_LDZ + kcol] = acc[r];
                        const float delta = rx[row * d.ld_rx + ly.acol + kcol] - raw[row * d.ld_raw + ly.acol + kcol];
                        if (kcol < K && r0 + row < rows) dfsum += -HGQ_LN2 * delta * acc[r];
                    }
                    dfsum += __shfl_xor(dfsum, 32, 64);
                    if (lane < 32 && kcol < K) atomicAdd(&red[kcol], dfsum);
                }
            }
            __syncthreads();
            if (tid < K) {
                float *dst = my + ly.p_df + tid;
                *dst = first ? red[tid] : *dst + red[tid];
            }
            // columns [Kp, 64) of the next gradient tile must read as zero for a narrower next layer
            if (ly.Kp < 64)
                for (int id = tid; id < MLP_BM * (64 - ly.Kp); id += 256) {
                    const int row = id / (64 - ly.Kp), c = ly.Kp + id % (64 - ly.Kp);
                    nxt[row * MLP_LDZ + c] = 0.f;
                }
            __syncthreads();
            float *t = cur;
            cur = nxt;
            nxt = t;
        }
    }
}

// out[e] = combination over slices of part[g][e]: float sum, or unsigned max inside the abs-max sections
__global__ __launch_bounds__(256) void mlp_reduce_kernel(MlpDev d, const float *__restrict__ part, int n_parts, float *out) {
    __shared__ float red[256];
    const int e_local = threadIdx.x & 63, grp = threadIdx.x >> 6;
    const int64_t e = (int64_t)blockIdx.x * 64 + e_local;
    bool is_max = false;
    for (int l = 0; l < d.n_layers; ++l) is_max |= (e >= d.l[l].p_amax && e < d.l[l].p_amax + d.l[l].h.K);
    float s = 0.f;
    uint32_t mx = 0;
    if (e < d.M) {
        const int per = (n_parts + 3) / 4;
        const int g0 = grp * per, g1 = min(n_parts, g0 + per);
        int g = g0;
        for (; g + 8 <= g1; g += 8) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = part[(int64_t)(g + u) * d.M + e];
            if (is_max) {
#pragma unroll
                for (int u = 0; u < 8; ++u) mx = max(mx, __float_as_uint(v[u]));
            } else {
                s += ((v[0] + v[1]) + (v[2] + v[3])) + ((v[4] + v[5]) + (v[6] + v[7]));
            }
        }
        for (; g < g1; ++g) {
            const float v = part[(int64_t)g * d.M + e];
            if (is_max) mx = max(mx, __float_as_uint(v));
            else s += v;
        }
    }
    red[threadIdx.x] = is_max ? __uint_as_float(mx) : s;
    __syncthreads();
    if (grp == 0 && e < d.M) {
        if (is_max) {
            uint32_t m = __float_as_uint(red[e_local]);
            for (int w = 1; w < 4; ++w) m = max(m, __float_as_uint(red[e_local + 64 * w]));
            out[e] = __uint_as_float(m);
        } else {
            out[e] = (red[e_local] + red[e_local + 64]) + (red[e_local + 128] + red[e_local + 192]);
        }
    }
}

__device__ __forceinline__ float sgd_clip(float w, float g, float lr, float l1, float lo, float hi) {
    return fminf(fmaxf(__fsub_rn(w, __fmul_rn(lr, __fadd_rn(g, l1))), lo), hi);
}

// One workgroup per layer.  All gradients are formed from the pre-update variables (phase 1 and 2
// only read), then every variable is updated (phase 3).
__global__ __launch_bounds__(256) void mlp_update_kernel(MlpDev d, const float *__restrict__ g, float lr, float *loss) {
    __shared__ float colsum[64];   // sum_n bits_ker[k, n]
    __shared__ float bits_in[64];  // relu(round(i) + round(f)) with the tracked i
    __shared__ float dbits_in[64];
    __shared__ float redbuf[4];
    const MlpLayerDev &ly = d.l[blockIdx.x];
    const hgq_mlp_layer &h = ly.h;
    const int tid = threadIdx.x, K = h.K, N = h.N;
    const Mode mk(h.mode_ker), mb(h.mode_bias), mi(h.mode_in);
    // ---- phase 1: integer-bit tracking of the input quantizer, then bit counts
    if (tid < K) {
        const float f = rintf(h.f_in[tid]);
        const float mi_ = ceil_log2_exact(__fadd_rn(g[ly.p_amax + tid], pow2(-f)));
        const float ni = fmaxf(__fsub_rn(h.i_in[tid], h.decay), mi_);
        h.i_in[tid] = ni;
        const float s = __fadd_rn(rintf(ni), f);
        float b = s > 0.f ? s : 0.f;
        dbits_in[tid] = s > 0.f ? 1.f : 0.f;
        if (mi.overflow_mode == HGQ_SAT) b += load_k(h.k_in, tid, mi.k_u8);
        bits_in[tid] = b;
        float cs = 0.f;
        for (int n = 0; n < N; ++n) {
            float bk = rintf(h.b_ker[tid * N + n]);
            if (mk.overflow_mode == HGQ_SAT) bk += load_k(h.k_ker, tid * N + n, mk.k_u8);
            cs += bk;
        }
        colsum[tid] = cs;
    }
    __syncthreads();
    // ---- phase 2: EBOPs value
    float part = tid < K ? bits_in[tid] * colsum[tid] : 0.f;
    float bsum = 0.f;
    if (h.bias && tid < N) {
        bsum = rintf(h.b_bias[tid]);
        if (mb.overflow_mode == HGQ_SAT) bsum += load_k(h.k_bias, tid, mb.k_u8);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) part += __shfl_xor(part, o, 64), bsum += __shfl_xor(bsum, o, 64);
    if ((tid & 63) == 0) redbuf[tid >> 6] = part;  // K, N <= 64: only wave 0 holds non-zero terms
    __syncthreads();
    const float beta = h.beta ? h.beta[0] : 0.f;
    if (tid == 0) {
        float total = redbuf[0];
        if (h.bias) total += bsum / (float)N * h.bias_size;
        const float e = total * h.ebops_scale;
        if (h.ebops) h.ebops[0] = (uint32_t)e;
        if (loss) atomicAdd(loss, e * beta + (blockIdx.x == 0 ? g[d.p_loss] : 0.f));
    }
    const float gs = h.ebops_scale * beta;  // d(ebops * beta) / d bits
    float reg = 0.f;  // MonoL1 regularisation loss of the trainable bit-width variables (pre-update values)
    // ---- phase 3: quantizer backward of kernel and bias, SGD + constraints on every variable
    for (int e = tid; e < K * N; e += 256) {
        const int k = e / N;
        const KIF p = kbi_entry(h.k_ker, h.i_ker, h.b_ker, e, h.mode_ker);
        float dw, di, db;
        quantize_grad_dyn(h.w[e], g[ly.p_dw + e], p, mk.round_mode, mk.overflow_mode, dw, di, db);
        di -= db;  // f = b - i
        h.w[e] = __fsub_rn(h.w[e], __fmul_rn(lr, dw));
        reg += h.b_ker_l1 * h.b_ker[e] + (h.train_i_ker ? h.i_ker_l1 * h.i_ker[e] : 0.f);
        h.b_ker[e] = sgd_clip(h.b_ker[e], db + bits_in[k] * gs, lr, h.b_ker_l1, h.b_ker_lo, h.b_ker_hi);
        if (h.train_i_ker) h.i_ker[e] = sgd_clip(h.i_ker[e], di, lr, h.i_ker_l1, h.i_ker_lo, h.i_ker_hi);
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
    }
    if (tid < K) {
        reg += h.f_in_l1 * h.f_in[tid];
        h.f_in[tid] = sgd_clip(h.f_in[tid], g[ly.p_df + tid] + dbits_in[tid] * colsum[tid] * gs, lr, h.f_in_l1, h.f_in_lo, h.f_in_hi);
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
    d.off_raw = off, off += MLP_BM * d.ld_raw;
    d.off_rx = off, off += MLP_BM * d.ld_rx;
    d.off_dz0 = off, off += MLP_BM * MLP_LDZ;
    d.off_dz1 = off, off += MLP_BM * MLP_LDZ;
    d.off_red = off, off += 64;
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
    return (int64_t)(mlp_parts(rows > 0 ? rows : 1) + 1) * d.M;
}

extern "C" int hgq_mlp_train_step(const hgq_mlp_layer *layers, int n_layers, const float *x, const int64_t *labels,
                                  int64_t rows, float lr, float *loss, float *workspace, void *stream) {
    hipStream_t s = (hipStream_t)stream;
    MlpDev d;
    size_t lds_bytes;
    int rc = mlp_plan(layers, n_layers, d, lds_bytes);
    if (rc) return rc;
    if (rows < 1 || !x || !labels || !workspace) return fail(HGQ_ERR_ARG, "hgq_mlp_train_step: bad arguments");
    static bool raised = false;
    if (!raised) {
        hipError_t e = hipFuncSetAttribute((const void *)mlp_fwd_bwd_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 512);
        if (e != hipSuccess) return fail(HGQ_ERR_LAUNCH, "hgq_mlp_train_step: hipFuncSetAttribute: %s", hipGetErrorString(e));
        raised = true;
    }
    const int parts = mlp_parts(rows);
    float *reduced = workspace + (int64_t)parts * d.M;
    if (loss && (rc = fill_f32(loss, 0.f, 1, s))) return rc;
    hipLaunchKernelGGL(mlp_fwd_bwd_kernel, dim3(parts), dim3(256), lds_bytes, s, d, x, labels, rows, workspace);
    if ((rc = check_launch("hgq_mlp_train_step(fwd_bwd)"))) return rc;
    hipLaunchKernelGGL(mlp_reduce_kernel, dim3((d.M + 63) / 64), dim3(256), 0, s, d, workspace, parts, reduced);
    if ((rc = check_launch("hgq_mlp_train_step(reduce)"))) return rc;
    hipLaunchKernelGGL(mlp_update_kernel, dim3(n_layers), dim3(256), 0, s, d, reduced, lr, loss);
    return check_launch("hgq_mlp_train_step(update)");
}
