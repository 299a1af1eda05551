// Training-step kernels around the contractions: EBOPs of a dense contraction (value and
// gradient in one pass), sparse categorical cross-entropy (value and gradient in one pass),
// SGD update with the bit-width constraint and MonoL1 gradient folded in.
#include <math.h>

#include "hgq_device.h"
#include "hgq_host.h"

namespace hgq {

__device__ __forceinline__ float block_sum_256(float v, float *scratch4) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    if ((threadIdx.x & 63) == 0) scratch4[threadIdx.x >> 6] = v;
    __syncthreads();
    v = scratch4[0] + scratch4[1] + scratch4[2] + scratch4[3];
    __syncthreads();
    return v;
}

// bits of one entry and the derivative of bits w.r.t. the fractional / total-bits variable
__device__ __forceinline__ float entry_bits(const void *k, const float *i, const float *fb, int64_t idx, const Mode &m,
                                            float &dbits) {
    float b;
    if (m.kbi) {
        b = rintf(fb[idx]);
        dbits = 1.0f;
    } else {
        const float s = __fadd_rn(rintf(i[idx]), rintf(fb[idx]));
        b = s > 0.0f ? s : 0.0f;
        dbits = s > 0.0f ? 1.0f : 0.0f;
    }
    if (m.overflow_mode == HGQ_SAT) b += load_k(k, idx, m.k_u8);
    return b;
}

#define HGQ_EBOPS_MAXK 4096

#define HGQ_EBOPS_NT 1024

__device__ __forceinline__ float block_sum_ebops(float v, float *scratch16) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    if ((threadIdx.x & 63) == 0) scratch16[threadIdx.x >> 6] = v;
    __syncthreads();
    float s = 0.0f;
#pragma unroll
    for (int w = 0; w < HGQ_EBOPS_NT / 64; ++w) s += scratch16[w];
    __syncthreads();
    return s;
}

// One workgroup of 1024 threads.  Bit-widths are integers, so the per-row / per-column sums are
// accumulated with integer LDS atomics over flat, coalesced sweeps (exact in any order).
__device__ __forceinline__ void dense_ebops_body(const uint32_t *amax_part, int n_parts, float decay,
                                                 const float *beta, float *loss_term,
                                                 const void *k_in, float *i_in, const float *f_in,
                                                 int64_t P, int K, int N, const void *k_ker,
                                                 const float *b_ker, const void *k_bias, const float *b_bias,
                                                 float par_factor, float n_parallel, float ebops_factor, float bias_size, int mode_in, int mode_ker, int mode_bias,
                                                 float *ebops, uint32_t *ebops_u32, float *g_f_in,
                                                 float *g_b_ker, float *g_b_bias) {
    constexpr int NT = HGQ_EBOPS_NT;
    // bit-widths are integers: the sums are accumulated with native integer LDS atomics
    __shared__ int colsum[HGQ_EBOPS_MAXK];  // sum_n bits_ker[k, n]
    __shared__ int insum[HGQ_EBOPS_MAXK];   // sum_p bits_in[p, k]
    __shared__ float red[NT / 64];
    const Mode mi(mode_in), mk(mode_ker), mb(mode_bias);
    const int t = threadIdx.x;
    // with beta the gradients are those of the loss term ebops * beta
    // the chain rule walks ((total * par_factor) / n_parallel) * ebops_factor (* beta) back one operation at a time
    const float gscale = __fmul_rn(__fdiv_rn(__fmul_rn(beta ? beta[0] : 1.0f, ebops_factor), n_parallel), par_factor);
    const int64_t PK = P * K;
    for (int k = t; k < K; k += NT) colsum[k] = 0, insum[k] = 0;
    if (amax_part) {
        // integer-bit tracking of the (KIF, WRAP, training) input quantizer, before its bits are read:
        // _i <- max(_i - decay, ceil(log2(max|x_q| + 2**-f)))
        // NT threads = `ne` entries x `ng` slice groups per pass, combined through LDS
        __shared__ uint32_t tmax[NT];
        int ne = 1;
        while (ne < NT && ne < PK) ne <<= 1;
        const int ng = NT / ne, el = t % ne, grp = t / ne;
        const int per = (n_parts + ng - 1) / ng;
        for (int64_t e0 = 0; e0 < PK; e0 += ne) {
            const int64_t e = e0 + el;
            uint32_t mx = 0;
            if (e < PK) {
                const int g0 = grp * per, g1 = min(n_parts, g0 + per);
                int g = g0;
                for (; g + 8 <= g1; g += 8) {
                    uint32_t v[8];
#pragma unroll
                    for (int u = 0; u < 8; ++u) v[u] = amax_part[(int64_t)(g + u) * PK + e];
#pragma unroll
                    for (int u = 0; u < 8; ++u) mx = v[u] > mx ? v[u] : mx;
                }
                for (; g < g1; ++g) {
                    const uint32_t a = amax_part[(int64_t)g * PK + e];
                    mx = a > mx ? a : mx;
                }
            }
            tmax[t] = mx;
            __syncthreads();
            if (grp == 0 && e < PK) {
                for (int w = 1; w < ng; ++w) mx = tmax[el + w * ne] > mx ? tmax[el + w * ne] : mx;
                const float mi_ = ceil_log2_exact(__fadd_rn(__uint_as_float(mx), pow2(-rintf(f_in[e]))));
                i_in[e] = fmaxf(__fsub_rn(i_in[e], decay), mi_);
            }
            __syncthreads();
        }
        __threadfence_block();
    }
    __syncthreads();
    const int64_t KN = (int64_t)K * N;
    // kernel entries in blocks of 4 * NT: loaded with consecutive lanes on consecutive entries, handed over through
    // LDS so that a thread adds a contiguous run of four before it touches a row's sum - one LDS atomic per (thread,
    // row) instead of one per entry (up to 64 lanes on one address serialise)
    __shared__ int sbits[4 * NT];
    for (int64_t blk = 0; blk < KN; blk += 4 * NT) {
        float b[4], d;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int64_t e = blk + u * NT + t;
            b[u] = entry_bits(k_ker, nullptr, b_ker, e < KN ? e : 0, mk, d);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) sbits[u * NT + t] = (int)b[u];
        __syncthreads();
        const int64_t e0 = blk + 4 * (int64_t)t;
        if (e0 < KN) {
            const int4 v = *(const int4 *)&sbits[4 * t];
            const int vals[4] = {v.x, v.y, v.z, v.w};
            int k = (int)(e0 / N), rem = (int)(e0 - (int64_t)k * N), acc = 0;
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                if (e0 + u < KN) {
                    acc += vals[u];
                    if (++rem == N) {
                        atomicAdd(&colsum[k], acc);
                        acc = 0, rem = 0, ++k;
                    }
                }
            }
            if (acc) atomicAdd(&colsum[k], acc);
        }
        __syncthreads();
    }
    __syncthreads();
    for (int64_t e = t; e < PK; e += NT) {
        float d;
        const int k = (int)(e % K);
        const float b = entry_bits(k_in, i_in, f_in, e, mi, d);
        atomicAdd(&insum[k], (int)b);
        if (g_f_in) g_f_in[e] = d * (float)colsum[k] * gscale;
    }
    __syncthreads();
    float part = 0.0f;
    for (int k = t; k < K; k += NT) part += (float)insum[k] * (float)colsum[k];
    float total = block_sum_ebops(part, red);
    if (g_b_ker)
        for (int64_t e = t; e < KN; e += NT) g_b_ker[e] = (float)insum[e / N] * gscale;
    if (b_bias) {
        float bs = 0.0f, d;
        for (int n = t; n < N; n += NT) {
            bs += entry_bits(k_bias, nullptr, b_bias, n, mb, d);
            if (g_b_bias) g_b_bias[n] = bias_size / (float)N * gscale;
        }
        bs = block_sum_ebops(bs, red);
        total += bs / (float)N * bias_size;
    }
    if (t == 0) {
        const float e = __fmul_rn(__fdiv_rn(__fmul_rn(total, par_factor), n_parallel), ebops_factor);
        ebops[0] = e;
        if (ebops_u32) ebops_u32[0] = (uint32_t)e;
        if (loss_term && beta) loss_term[0] = e * beta[0];
    }
}

__global__ __launch_bounds__(HGQ_EBOPS_NT) void dense_ebops_kernel(const uint32_t *amax_part, int n_parts, float decay,
                                                          const float *beta, float *loss_term,
                                                          const void *k_in, float *i_in, const float *f_in,
                                                          int64_t P, int K, int N, const void *k_ker,
                                                          const float *b_ker, const void *k_bias, const float *b_bias,
                                                          float par_factor, float n_parallel, float ebops_factor, float bias_size, int mode_in, int mode_ker, int mode_bias,
                                                          float *ebops, uint32_t *ebops_u32, float *g_f_in,
                                                          float *g_b_ker, float *g_b_bias) {
    dense_ebops_body(amax_part, n_parts, decay, beta, loss_term, k_in, i_in, f_in, P, K, N, k_ker, b_ker, k_bias, b_bias, par_factor, n_parallel, ebops_factor,
                     bias_size, mode_in, mode_ker, mode_bias, ebops, ebops_u32, g_f_in, g_b_ker, g_b_bias);
}

// the layers of a model, one workgroup each: the estimates depend on the bit-width variables only, so they can all be
// computed at the end of the forward pass in one launch instead of one single-workgroup launch per layer
struct DenseEbopsBatch {
    hgq_dense_ebops_item item[HGQ_EBOPS_BATCH];
};
__global__ __launch_bounds__(HGQ_EBOPS_NT) void dense_ebops_multi_kernel(DenseEbopsBatch b) {
    const hgq_dense_ebops_item &it = b.item[blockIdx.x];
    dense_ebops_body(it.amax_part, it.n_parts, it.decay, it.beta, it.loss_term, it.k_in, it.i_in, it.f_in, it.P, it.K, it.N, it.k_ker,
                     it.b_ker, it.k_bias, it.b_bias, it.par_factor, it.n_parallel, it.ebops_factor, it.bias_size, it.mode_in, it.mode_ker, it.mode_bias, it.ebops, it.ebops_u32,
                     it.g_f_in, it.g_b_ker, it.g_b_bias);
}

// Mean squared error: per-workgroup partial sums (fixed order inside a workgroup), added in order
// by one wavefront of a second launch: the loss does not depend on scheduling.
#define MSE_PARTS 1024
// dpred (may be null): also receives the gradient for a unit upstream gradient, (pred - target) * two_over_n, the value
// mse_bwd_kernel gives for g = 1
__global__ __launch_bounds__(256) void mse_partial_kernel(const float *__restrict__ pred, const float *__restrict__ target, int64_t n,
                                                          float *__restrict__ part, float *__restrict__ dpred, float two_over_n) {
    __shared__ float red[4];
    float acc = 0.f;
    const int64_t n4 = n >> 2, stride = (int64_t)gridDim.x * 256;
    // four vectors of a thread per trip, every load of the trip in flight before the first is used
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    for (; i + 3 * stride < n4; i += 4 * stride) {
        f32x4_t p[4], t[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            p[u] = ((const f32x4_t *)pred)[i + u * stride];
            t[u] = target ? ((const f32x4_t *)target)[i + u * stride] : f32x4_t{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const f32x4_t d = p[u] - t[u];
            acc += (d[0] * d[0] + d[1] * d[1]) + (d[2] * d[2] + d[3] * d[3]);
            if (dpred) ((f32x4_t *)dpred)[i + u * stride] = d * two_over_n;
        }
    }
    for (; i < n4; i += stride) {
        const f32x4_t p = ((const f32x4_t *)pred)[i];
        const f32x4_t t = target ? ((const f32x4_t *)target)[i] : f32x4_t{0.f, 0.f, 0.f, 0.f};
        const f32x4_t d = p - t;
        acc += (d[0] * d[0] + d[1] * d[1]) + (d[2] * d[2] + d[3] * d[3]);
        if (dpred) ((f32x4_t *)dpred)[i] = d * two_over_n;
    }
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
        const int64_t i = (n4 << 2) + threadIdx.x;
        const float d = pred[i] - (target ? target[i] : 0.f);
        acc += d * d;
        if (dpred) dpred[i] = d * two_over_n;
    }
    acc = block_sum_256(acc, red);
    if (threadIdx.x == 0) part[blockIdx.x] = acc;
}

__global__ __launch_bounds__(64) void mse_finish_kernel(const float *__restrict__ part, int n_parts, float inv_n, float *loss) {
    float acc = 0.f;
    for (int i = threadIdx.x; i < n_parts; i += 64) acc += part[i];
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o, 64);
    if (threadIdx.x == 0) loss[0] = acc * inv_n;
}

// dpred = g * 2 (pred - target) / n, g read from device memory
__global__ __launch_bounds__(256) void mse_bwd_kernel(const float *__restrict__ pred, const float *__restrict__ target,
                                                      const float *__restrict__ g, float two_over_n, int64_t n, float *__restrict__ dpred) {
    const float c = g[0] * two_over_n;
    const int64_t n4 = n >> 2, stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += stride) {
        const f32x4_t p = ((const f32x4_t *)pred)[i];
        const f32x4_t t = target ? ((const f32x4_t *)target)[i] : f32x4_t{0.f, 0.f, 0.f, 0.f};
        ((f32x4_t *)dpred)[i] = (p - t) * c;
    }
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
        const int64_t i = (n4 << 2) + threadIdx.x;
        dpred[i] = (pred[i] - (target ? target[i] : 0.f)) * c;
    }
}

// Batch-norm folding of QEinsumDenseBatchnorm for a [K, N] kernel normalised over its N outputs:
//     var = second - mean^2 (second = mean of squares) or var = second;  scaler = gamma / sqrt(var + eps)
//     fused_w[k, n] = w[k, n] * scaler[n];   fused_b[n] = bias[n] + (-mean[n] * scaler[n])
// and, when moving statistics are given, their momentum update.  One thread per kernel entry; the
// first K-row also writes the per-column results.  IEEE division and square root, reference order.
__device__ __forceinline__ float bn_var(float mean, float second, int is_meansq) {
    return is_meansq ? __fsub_rn(second, __fmul_rn(mean, mean)) : second;
}

// QUANT: the kernel and bias quantizers (per-element bit-widths, no trackers) follow in the same thread: fused_w / fused_b
// then receive the QUANTIZED values (the folded ones are products the backward pass forms again, bit for bit).
template <bool QUANT>
__global__ __launch_bounds__(256) void bn_fold_fwd_kernel(const float *__restrict__ w, const float *__restrict__ bias,
                                                          const float *__restrict__ gamma, const float *__restrict__ mean,
                                                          const float *__restrict__ second, int is_meansq, float eps,
                                                          float *__restrict__ fused_w, float *__restrict__ fused_b, float *moving_mean,
                                                          float *moving_var, float momentum, float one_minus_momentum, int K, int N,
                                                          hgq_qdesc qk, hgq_qdesc qb) {
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= (int64_t)K * N) return;
    const int n = (int)(e % N);
    const float var = bn_var(mean[n], second[n], is_meansq);
    const float scaler = __fdiv_rn(gamma ? gamma[n] : 1.0f, __fsqrt_rn(__fadd_rn(var, eps)));
    float fw = __fmul_rn(w[e], scaler);
    if (QUANT) {
        const Mode mk(qk.mode);
        fw = quantize_dyn(fw, resolve_kif(load_k(qk.k, e, mk.k_u8), qk.i[e], qk.fb[e], mk.kbi, mk.round_params), mk.round_mode,
                          mk.overflow_mode, mk.training);
    }
    fused_w[e] = fw;
    if (e < N) {
        float fb = __fadd_rn(bias[n], __fmul_rn(-mean[n], scaler));
        if (QUANT) {
            const Mode mb(qb.mode);
            fb = quantize_dyn(fb, resolve_kif(load_k(qb.k, n, mb.k_u8), qb.i[n], qb.fb[n], mb.kbi, mb.round_params), mb.round_mode,
                              mb.overflow_mode, mb.training);
        }
        fused_b[n] = fb;
        if (moving_mean) moving_mean[n] = __fadd_rn(__fmul_rn(moving_mean[n], momentum), __fmul_rn(mean[n], one_minus_momentum));
        if (moving_var) moving_var[n] = __fadd_rn(__fmul_rn(moving_var[n], momentum), __fmul_rn(var, one_minus_momentum));
    }
}

// Gradients of the folding.  Thread (column n, row group r of 4) walks kernel rows r, r + 4, ... with all its loads in
// flight (coalesced across columns); the four partial sums of a column meet in LDS in group order:
//   dw = d_fw * scaler;  dscaler = sum_k d_fw * w - d_fb * mean;  dbias = d_fb;
//   dgamma = dscaler / sqrt(var + eps);  dvar = -dscaler * gamma / (2 (var + eps)^(3/2));
//   dmean = -d_fb * scaler (- 2 mean dvar when var comes from the mean of squares);  dsecond = dvar.
// QUANT: d_fw / d_fb are the gradients at the QUANTIZED folded kernel / bias; each passes its quantizer's surrogate
// gradient first (the folded value is formed again from w and the scaler), whose bit-width parts go to dik / dfk [K, N]
// and dib / dfbb [N].
// CB columns per workgroup, 256 / CB row groups: the quantizer form takes 16 columns per workgroup (its work per element is
// an order of magnitude more than the folding's, and a kernel of 64 columns would otherwise run on one CU).
template <bool QUANT, int CB>
__global__ __launch_bounds__(256) void bn_fold_bwd_kernel(const float *__restrict__ w, const float *__restrict__ gamma,
                                                          const float *__restrict__ mean, const float *__restrict__ second,
                                                          int is_meansq, float eps, const float *__restrict__ d_fw,
                                                          const float *__restrict__ d_fb, float *__restrict__ dw, float *dbias,
                                                          float *dgamma, float *dmean, float *dsecond, int K, int N,
                                                          const float *__restrict__ bias, hgq_qdesc qk, hgq_qdesc qb,
                                                          float *__restrict__ dik, float *__restrict__ dfk, float *dib, float *dfbb) {
    constexpr int RG = 256 / CB, BNF_ROWS = 64 / RG;  // row groups; rows per thread and trip (64 rows per trip)
    __shared__ float part[RG][CB];
    const int nl = threadIdx.x % CB, grp = threadIdx.x / CB, n = blockIdx.x * CB + nl;
    const bool col = n < N;
    const float g = (gamma && col) ? gamma[n] : 1.0f, m = col ? mean[n] : 0.f;
    const float ve = bn_var(m, col ? second[n] : 1.0f, is_meansq) + eps, sd = __fsqrt_rn(ve);
    const float scaler = __fdiv_rn(g, sd);
    const int64_t bytes = (int64_t)K * N * 4;
    const __amdgpu_buffer_rsrc_t rs_g = buf_rsrc(d_fw, bytes), rs_w = buf_rsrc(w, bytes), rs_dw = buf_rsrc(dw, bytes);
    float ds = 0.f;
    for (int k0 = grp; k0 < K; k0 += RG * BNF_ROWS) {
        float gv[BNF_ROWS], wv[BNF_ROWS];
        uint32_t off[BNF_ROWS];
#pragma unroll
        for (int u = 0; u < BNF_ROWS; ++u) {
            const int k = k0 + RG * u;
            off[u] = (col && k < K) ? (uint32_t)(k * N + n) * 4u : BUF_OOB;  // rows / columns past the end read as zero
            gv[u] = buf_ld1(rs_g, off[u]);
            wv[u] = buf_ld1(rs_w, off[u]);
        }
        if (QUANT) {
            const Mode mk(qk.mode);
            const __amdgpu_buffer_rsrc_t rs_i = buf_rsrc(qk.i, bytes), rs_f = buf_rsrc(qk.fb, bytes);
            const __amdgpu_buffer_rsrc_t rs_di = buf_rsrc(dik, bytes), rs_df = buf_rsrc(dfk, bytes);
            // every operand of the trip is requested before the first is used (a load behind a branch is waited for on the spot)
            const __amdgpu_buffer_rsrc_t rs_k = buf_rsrc(qk.k, mk.k_u8 ? bytes / 4 : bytes);
            float iv[BNF_ROWS], fv[BNF_ROWS], kv[BNF_ROWS];
#pragma unroll
            for (int u = 0; u < BNF_ROWS; ++u) {
                iv[u] = buf_ld1(rs_i, off[u]), fv[u] = buf_ld1(rs_f, off[u]);
                if (mk.k_u8) kv[u] = (float)__builtin_amdgcn_raw_buffer_load_b8(rs_k, off[u] == BUF_OOB ? BUF_OOB : off[u] >> 2, 0, 0);
                else kv[u] = buf_ld1(rs_k, off[u]);
            }
#pragma unroll
            for (int u = 0; u < BNF_ROWS; ++u) {
                const int k = k0 + RG * u;
                if (col && k < K) {
                    const KIF p = resolve_kif(kv[u], iv[u], fv[u], mk.kbi, mk.round_params);
                    float gx, gi, gf;
                    quantize_grad_dyn(__fmul_rn(wv[u], scaler), gv[u], p, mk.round_mode, mk.overflow_mode, gx, gi, gf);
                    if (mk.kbi) gi -= gf;
                    buf_st1(rs_di, off[u], gi), buf_st1(rs_df, off[u], gf);
                    gv[u] = gx;
                }
            }
        }
#pragma unroll
        for (int u = 0; u < BNF_ROWS; ++u) {
            ds += gv[u] * wv[u];
            buf_st1(rs_dw, off[u], gv[u] * scaler);
        }
    }
    part[grp][nl] = ds;
    __syncthreads();
    if (grp != 0 || !col) return;
    ds = part[0][nl];
#pragma unroll
    for (int r = 1; r < RG; ++r) ds += part[r][nl];  // groups in order
    float gb = d_fb[n];
    if (QUANT) {
        const Mode mb(qb.mode);
        const KIF p = resolve_kif(load_k(qb.k, n, mb.k_u8), qb.i[n], qb.fb[n], mb.kbi, mb.round_params);
        float gx, gi, gf;
        quantize_grad_dyn(__fadd_rn(bias[n], __fmul_rn(-m, scaler)), gb, p, mb.round_mode, mb.overflow_mode, gx, gi, gf);
        if (mb.kbi) gi -= gf;
        dib[n] = gi, dfbb[n] = gf;
        gb = gx;
    }
    ds -= gb * m;
    const float dvar = -ds * g / (2.0f * ve * sd);
    if (dbias) dbias[n] = gb;
    if (dgamma) dgamma[n] = ds / sd;
    if (dsecond) dsecond[n] = dvar;
    if (dmean) dmean[n] = -gb * scaler - (is_meansq ? 2.0f * m * dvar : 0.f);
}

// Bit-widths of a quantizer from its raw variables, in one launch each way (the host formula is a
// chain of round / add / relu / cast launches per quantizer and step):
//   KIF:  b = relu(rint(i) + rint(f));   KBI:  b = rint(fb)
//   add_mode 0: b;  1: b + k (SAT `bits`, non-WRAP `fbits`);  2: b + k * (b > 0) (WRAP `fbits`)
// Straight-through rounding: d b / d i = d b / d f = [rint(i) + rint(f) > 0] (KIF), d b / d fb = 1 (KBI).
__global__ __launch_bounds__(256) void qbits_fwd_kernel(const uint8_t *__restrict__ k, const float *__restrict__ i,
                                                        const float *__restrict__ fb, int64_t n, int kbi, int add_mode,
                                                        float *__restrict__ out) {
    for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < n; e += (int64_t)gridDim.x * 256) {
        float b;
        if (kbi) {
            b = rintf(fb[e]);
        } else {
            const float sum = __fadd_rn(rintf(i[e]), rintf(fb[e]));
            b = sum > 0.f ? sum : 0.f;
        }
        if (add_mode == 1) b = __fadd_rn(b, (float)k[e]);
        else if (add_mode == 2) b = __fadd_rn(b, (float)k[e] * (b > 0.f ? 1.f : 0.f));
        out[e] = b;
    }
}

__global__ __launch_bounds__(256) void qbits_bwd_kernel(const float *__restrict__ g, const float *__restrict__ i,
                                                        const float *__restrict__ fb, int64_t n, int kbi, float *__restrict__ di,
                                                        float *__restrict__ dfb) {
    for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < n; e += (int64_t)gridDim.x * 256) {
        if (kbi) {
            dfb[e] = g[e];
        } else {
            const float v = __fadd_rn(rintf(i[e]), rintf(fb[e])) > 0.f ? g[e] : 0.f;
            di[e] = v, dfb[e] = v;
        }
    }
}

// The tail of QLayerBase's call wrapper on a scalar: ebops <- ebops * factor, the uint32 variable,
// and the loss term ebops * beta, in one launch (and its gradient in another).
__global__ void ebops_finish_fwd_kernel(const float *ebops, float factor, const float *beta, uint32_t *ebops_u32, float *out) {
    const float e = __fmul_rn(ebops[0], factor);
    if (ebops_u32) ebops_u32[0] = (uint32_t)(int64_t)e;
    out[0] = __fmul_rn(e, beta[0]);
}
__global__ void ebops_finish_bwd_kernel(const float *g, const float *beta, float factor, float *d_ebops) {
    d_ebops[0] = __fmul_rn(__fmul_rn(g[0], beta[0]), factor);
}

// one thread per row; C is small (class count)
// `state` = {sum (64-bit fixed point, two words), finished workgroups, a workgroup's sum was not finite}: all zero at the
// start and left zero at the end.  The workgroups' sums meet as INTEGERS (2^-40 units): integer addition does not depend on
// the order in which they arrive, so the loss is the same in every run and in every replay of a recorded step (a float
// atomic would round differently with every arrival order).  state == NULL: a single workgroup, no meeting at all.
#define CE_FIX 1099511627776.0f  // 2^40: a sum of up to 2^22 in magnitude keeps 2^-40 resolution in 63 bits
__global__ __launch_bounds__(256) void sparse_ce_kernel(const float *__restrict__ logits,
                                                        const int64_t *__restrict__ labels, float *loss,
                                                        float *__restrict__ dlogits, int64_t rows, int C, uint32_t *state) {
    __shared__ float red[4];
    const float inv_rows = 1.0f / (float)rows;
    float acc = 0.0f;
    for (int64_t r = (int64_t)blockIdx.x * 256 + threadIdx.x; r < rows; r += (int64_t)gridDim.x * 256) {
        const float *z = logits + r * C;
        float mx = z[0];
        for (int c = 1; c < C; ++c) mx = fmaxf(mx, z[c]);
        float se = 0.0f;
        for (int c = 0; c < C; ++c) se += expf(z[c] - mx);
        const float lse = logf(se);
        const int64_t lab = labels[r];
        // a label outside [0, C) (an ignore index, 1-based labels) reads nothing: the loss becomes NaN, the row's gradient zero
        const bool lab_ok = (uint64_t)lab < (uint64_t)C;
        acc += lab_ok ? lse - (z[lab_ok ? lab : 0] - mx) : NAN;
        if (dlogits) {
            float *d = dlogits + r * C;
            const float inv = 1.0f / se;
            for (int c = 0; c < C; ++c) d[c] = lab_ok ? (expf(z[c] - mx) * inv - (c == lab ? 1.0f : 0.0f)) * inv_rows : 0.0f;
        }
    }
    acc = block_sum_256(acc, red);
    if (threadIdx.x == 0) {
        const float part = acc * inv_rows;
        if (!state) {
            loss[0] = part;  // (launched as one workgroup)
            return;
        }
        // All four words are only ever touched by device-scope atomics, which are performed where all workgroups meet (not
        // in a cache that would need a write-back).  The ticket is drawn with an operand that depends on the value the
        // sum's atomic RETURNS, so it cannot leave this wavefront before this workgroup's part has been added: whoever
        // draws the last ticket finds every part in the sum.  (A fence of workgroup scope between two non-returning
        // atomics orders nothing for other workgroups; one of device scope costs a cache write-back, ~2 us here.)
        const bool finite = fabsf(part) < 4194304.0f;  // (false for NaN too)
        unsigned long long *sum = (unsigned long long *)state;
        unsigned long long before = atomicAdd(sum, finite ? (unsigned long long)(long long)rintf(part * CE_FIX) : 0ull);
        if (!finite) before += atomicOr(state + 3, 1u);
        uint32_t one = 1u;
        asm volatile("" : "+v"(one) : "v"((uint32_t)before));
        if (atomicAdd(state + 2, one) == gridDim.x - 1) {
            // every other workgroup has added its part
            const long long total = (long long)atomicExch(sum, 0ull);
            const uint32_t bad = atomicExch(state + 3, 0u);
            loss[0] = bad ? NAN : (float)((double)total * (1.0 / (double)CE_FIX));
            atomicExch(state + 2, 0u);
        }
    }
}

// The next batch of a data set that lives in device memory: row r of the batch is row order[pos + r] of the source (samples
// and labels alike), pos = state[0].  The workgroup that finishes last - every other one has read pos by then - moves pos
// on by `batch` and clears the ticket word state[1], so a recorded launch draws batch after batch as it is replayed.
// Positions past the end read the last row (the caller resets pos before that happens).  Rows are whole 32-bit words;
// VEC: 128-bit accesses (row sizes multiples of 16 bytes, aligned arrays).
template <bool VEC>
__global__ __launch_bounds__(256) void gather_batch_kernel(const uint32_t *__restrict__ x_src, int64_t x_words,
                                                           const uint32_t *__restrict__ y_src, int64_t y_words,
                                                           const int64_t *__restrict__ order, unsigned long long *state,
                                                           uint32_t *__restrict__ x_dst, uint32_t *__restrict__ y_dst, int64_t batch,
                                                           int64_t n_rows) {
    __shared__ int64_t spos;
    if (threadIdx.x == 0) spos = (int64_t)__hip_atomic_load(state, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    const int64_t pos = spos;
    const int64_t first = (int64_t)blockIdx.x * 256 + threadIdx.x, stride = (int64_t)gridDim.x * 256;
    auto source_row = [&](int64_t r) {
        int64_t p = pos + r;
        p = p < n_rows ? p : n_rows - 1;
        int64_t s = order[p < 0 ? 0 : p];
        return s < 0 ? 0 : (s < n_rows ? s : n_rows - 1);
    };
    const int64_t xw = VEC ? x_words / 4 : x_words;
    for (int64_t e = first; e < batch * xw; e += stride) {
        const int64_t r = e / xw, c = e - r * xw, s = source_row(r);
        if (VEC) ((u32x4_t *)x_dst)[r * xw + c] = ((const u32x4_t *)x_src)[s * xw + c];
        else x_dst[r * xw + c] = x_src[s * xw + c];
    }
    for (int64_t e = first; e < batch * y_words; e += stride) {
        const int64_t r = e / y_words, c = e - r * y_words;
        y_dst[e] = y_src[source_row(r) * y_words + c];
    }
    __syncthreads();  // every thread of this workgroup has read pos
    if (threadIdx.x == 0) {
        uint32_t *ticket = (uint32_t *)(state + 1);
        if (atomicAdd(ticket, 1u) == gridDim.x - 1) {
            atomicExch(state, (unsigned long long)(pos + batch));
            atomicExch(ticket, 0u);
        }
    }
}

__global__ __launch_bounds__(256) void sgd_kernel(float *__restrict__ w, const float *__restrict__ g, int64_t n,
                                                  float lr, float l1, float lo, float hi) {
    for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < n; t += (int64_t)gridDim.x * 256) {
        const float v = __fsub_rn(w[t], __fmul_rn(lr, __fadd_rn(g[t], l1)));
        w[t] = fminf(fmaxf(v, lo), hi);
    }
}

struct SgdBatch {
    hgq_sgd_item item[HGQ_SGD_BATCH];
};
struct SumBatch {
    const float *term[HGQ_SUM_BATCH];
};

// grid.y = variable, grid.x strides over its elements; the descriptors travel as a kernel argument
// n_sum > 0: the first thread of the launch also adds the scalars of `sums` in list order into sum_out (the step's loss
// terms: the update does not read them, they only ride along instead of taking a launch of their own)
__global__ __launch_bounds__(256) void sgd_multi_kernel(SgdBatch b, float lr, SumBatch sums, int n_sum, float *sum_out) {
    if (n_sum > 0 && blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) {
        float v = sums.term[0][0];
        for (int t = 1; t < n_sum; ++t) v = __fadd_rn(v, sums.term[t][0]);
        sum_out[0] = v;
    }
    const hgq_sgd_item it = b.item[blockIdx.y];
    float sc[HGQ_SGD_SIDES];
#pragma unroll
    for (int s = 0; s < HGQ_SGD_SIDES; ++s) sc[s] = (it.side[s] && it.side_scale[s]) ? it.side_scale[s][0] : 1.0f;
    for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < it.n; t += (int64_t)gridDim.x * 256) {
        float g = it.g ? it.g[t] : 0.0f;
#pragma unroll
        for (int s = 0; s < HGQ_SGD_SIDES; ++s)
            if (it.side[s]) g = __fadd_rn(g, __fmul_rn(sc[s], it.side[s][t]));
        const float v = __fsub_rn(it.w[t], __fmul_rn(lr, __fadd_rn(g, it.l1)));
        it.w[t] = fminf(fmaxf(v, it.lo), it.hi);
    }
}


// ------------------------------------------------------------------------------------------
// per-column first and second moments of a [rows, N] matrix (batch-normalisation statistics)
// ------------------------------------------------------------------------------------------
// A thread owns VEC adjacent columns and walks down the rows; the workgroup's TY row groups are
// combined through LDS and written to slice blockIdx.y of `part` ([gridDim.y, 2 * N]: sums, then
// sums of squares), which reduce_parts adds up in a fixed order.
template <int VEC>
__global__ __launch_bounds__(256) void col_moments_kernel(const float *__restrict__ x, int64_t rows, int N, int TX,
                                                          float *__restrict__ part) {
    __shared__ float s1[256 * VEC], s2[256 * VEC];
    const int TY = 256 / TX;
    const int tx = threadIdx.x % TX, ty = threadIdx.x / TX;
    const int64_t cg = N / VEC;
    const int64_t c = (int64_t)blockIdx.x * TX + tx;
    float a1[VEC], a2[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) a1[e] = 0.f, a2[e] = 0.f;
    if (c < cg) {
        for (int64_t r = (int64_t)blockIdx.y * TY + ty; r < rows; r += (int64_t)gridDim.y * TY) {
            float v[VEC];
            if (VEC == 4) {
                const float4 t = *(const float4 *)(x + (r * cg + c) * 4);
                v[0] = t.x, v[1 % VEC] = t.y, v[2 % VEC] = t.z, v[3 % VEC] = t.w;
            } else {
                v[0] = x[r * cg + c];
            }
#pragma unroll
            for (int e = 0; e < VEC; ++e) a1[e] += v[e], a2[e] += v[e] * v[e];
        }
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) s1[threadIdx.x * VEC + e] = a1[e], s2[threadIdx.x * VEC + e] = a2[e];
    __syncthreads();
    for (int st = TY / 2; st > 0; st >>= 1) {
        if (ty < st) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                s1[threadIdx.x * VEC + e] += s1[(threadIdx.x + st * TX) * VEC + e];
                s2[threadIdx.x * VEC + e] += s2[(threadIdx.x + st * TX) * VEC + e];
            }
        }
        __syncthreads();
    }
    if (ty == 0 && c < cg) {
        float *my = part + (int64_t)blockIdx.y * 2 * N;
#pragma unroll
        for (int e = 0; e < VEC; ++e) my[c * VEC + e] = s1[tx * VEC + e], my[N + c * VEC + e] = s2[tx * VEC + e];
    }
}

// dx[r, c] = (dmean[c] + 2 x[r, c] dmeansq[c]) / rows
__global__ __launch_bounds__(256) void col_moments_bwd_kernel(const float *__restrict__ x, const float *__restrict__ dmean,
                                                              const float *__restrict__ dmeansq, int64_t n, int N,
                                                              float inv_rows, float *__restrict__ dx) {
    for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < n; e += (int64_t)gridDim.x * 256) {
        const int c = (int)(e % N);
        dx[e] = (dmean[c] + 2.0f * x[e] * dmeansq[c]) * inv_rows;
    }
}

}  // namespace hgq

using namespace hgq;

static int sgd_update_multi_impl(const hgq_sgd_item *items, int count, float lr, const float *const *terms, int n_terms, float *sum_out,
                                 void *stream) {
    if (count < 0 || (count > 0 && !items)) return fail(HGQ_ERR_ARG, "hgq_sgd_update_multi: bad arguments");
    SumBatch sums;
    for (int t = 0; t < HGQ_SUM_BATCH; ++t) sums.term[t] = t < n_terms ? terms[t] : nullptr;
    bool summed = n_terms == 0;
    for (int base = 0; base < count; base += HGQ_SGD_BATCH) {
        SgdBatch b;
        const int nb = count - base < HGQ_SGD_BATCH ? count - base : HGQ_SGD_BATCH;
        int64_t max_n = 0;
        for (int t = 0; t < nb; ++t) {
            b.item[t] = items[base + t];
            bool any = b.item[t].g != nullptr;
            for (int sd = 0; sd < HGQ_SGD_SIDES; ++sd) any = any || b.item[t].side[sd] != nullptr;
            if (b.item[t].n < 0 || (b.item[t].n > 0 && (!b.item[t].w || !any)))
                return fail(HGQ_ERR_ARG, "hgq_sgd_update_multi: bad item %d", base + t);
            if (b.item[t].n > max_n) max_n = b.item[t].n;
        }
        if (max_n == 0) continue;
        int64_t gx = (max_n + 1023) / 1024;
        if (gx > 512) gx = 512;
        hipLaunchKernelGGL(sgd_multi_kernel, dim3((unsigned)gx, (unsigned)nb), dim3(256), 0, (hipStream_t)stream, b, lr, sums, summed ? 0 : n_terms,
                           sum_out);
        summed = true;
        int rc = check_launch("hgq_sgd_update_multi");
        if (rc) return rc;
    }
    if (!summed) return hgq_sum_scalars(terms, n_terms, sum_out, stream);  // nothing to update: the sum alone
    return HGQ_OK;
}

extern "C" int hgq_sgd_update_multi(const hgq_sgd_item *items, int count, float lr, void *stream) {
    return sgd_update_multi_impl(items, count, lr, nullptr, 0, nullptr, stream);
}

extern "C" int hgq_sgd_update_multi_sum(const hgq_sgd_item *items, int count, float lr, const float *const *terms, int n_terms,
                                        float *sum_out, void *stream) {
    if (n_terms < 1 || n_terms > HGQ_SUM_BATCH || !terms || !sum_out)
        return fail(HGQ_ERR_ARG, "hgq_sgd_update_multi_sum: 1 <= n_terms <= %d terms and an output are expected", HGQ_SUM_BATCH);
    for (int t = 0; t < n_terms; ++t)
        if (!terms[t]) return fail(HGQ_ERR_ARG, "hgq_sgd_update_multi_sum: null term %d", t);
    return sgd_update_multi_impl(items, count, lr, terms, n_terms, sum_out, stream);
}

namespace hgq {
// one thread: the terms are added in list order, exactly as a chain of scalar additions would
__global__ void sum_scalars_kernel(SumBatch b, int count, float *out) {
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        float v = b.term[0][0];
        for (int t = 1; t < count; ++t) v = __fadd_rn(v, b.term[t][0]);
        out[0] = v;
    }
}
}  // namespace hgq

extern "C" int hgq_sum_scalars(const float *const *terms, int count, float *out, void *stream) {
    if (!terms || !out || count < 1 || count > HGQ_SUM_BATCH) return fail(HGQ_ERR_ARG, "hgq_sum_scalars: 1 <= count <= %d terms expected", HGQ_SUM_BATCH);
    SumBatch b;
    for (int t = 0; t < count; ++t) {
        if (!terms[t]) return fail(HGQ_ERR_ARG, "hgq_sum_scalars: null term %d", t);
        b.term[t] = terms[t];
    }
    for (int t = count; t < HGQ_SUM_BATCH; ++t) b.term[t] = nullptr;
    hipLaunchKernelGGL(sum_scalars_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, b, count, out);
    return check_launch("hgq_sum_scalars");
}

extern "C" int hgq_dense_ebops(const uint32_t *amax_part, int n_parts, float decay, const float *beta, float *loss_term,
                               const void *k_in, float *i_in, const float *f_in, int64_t P, int K, int N,
                               const void *k_ker, const float *b_ker, const void *k_bias, const float *b_bias,
                               float par_factor, float n_parallel, float ebops_factor, float bias_size, int mode_in, int mode_ker, int mode_bias, float *ebops,
                               uint32_t *ebops_u32, float *g_f_in, float *g_b_ker, float *g_b_bias, void *stream) {
    if (P < 1 || K < 1 || N < 1) return fail(HGQ_ERR_ARG, "hgq_dense_ebops: bad sizes");
    if (!i_in || !f_in || !b_ker || !ebops || !k_in || !k_ker) return fail(HGQ_ERR_ARG, "hgq_dense_ebops: null pointer");
    if (K > HGQ_EBOPS_MAXK) return fail(HGQ_ERR_UNSUPPORTED, "hgq_dense_ebops: K=%d > %d", K, HGQ_EBOPS_MAXK);
    if (!(Mode(mode_ker).kbi) || (b_bias && !(Mode(mode_bias).kbi))) return fail(HGQ_ERR_UNSUPPORTED, "hgq_dense_ebops: kernel/bias bit-widths must use the KBI parametrisation");
    if (amax_part && (n_parts < 1 || Mode(mode_in).kbi || Mode(mode_in).overflow_mode != HGQ_WRAP))
        return fail(HGQ_ERR_ARG, "hgq_dense_ebops: fused tracking is for KIF WRAP input quantizers");
    if (amax_part && P * K * n_parts > 16384) {
        // many tracker slices: combine them with one thread group per entry across the device first
        int rc = hgq_wrap_track_i(amax_part, nullptr, n_parts, i_in, f_in, nullptr, P * K, decay, 0.0f, 0.0f,
                                  mode_in & ~(HGQ_MODE_TRACING | HGQ_MODE_SYMMETRIC), stream);
        if (rc) return rc;
        amax_part = nullptr;
    }
    hipLaunchKernelGGL(dense_ebops_kernel, dim3(1), dim3(HGQ_EBOPS_NT), 0, (hipStream_t)stream, amax_part, n_parts, decay, beta, loss_term, k_in,
                       i_in, f_in, P, K, N, k_ker, b_ker,
                       k_bias, b_bias, par_factor, n_parallel, ebops_factor, bias_size, mode_in, mode_ker, mode_bias, ebops, ebops_u32, g_f_in, g_b_ker,
                       g_b_bias);
    return check_launch("hgq_dense_ebops");
}

extern "C" int hgq_dense_ebops_multi(const hgq_dense_ebops_item *items, int count, void *stream) {
    if (count < 0 || (count > 0 && !items)) return fail(HGQ_ERR_ARG, "hgq_dense_ebops_multi: bad arguments");
    for (int base = 0; base < count; base += HGQ_EBOPS_BATCH) {
        DenseEbopsBatch b;
        hgq_track_item tracks[HGQ_EBOPS_BATCH];
        int n_tracks = 0;
        const int nb = count - base < HGQ_EBOPS_BATCH ? count - base : HGQ_EBOPS_BATCH;
        for (int t = 0; t < nb; ++t) {
            const hgq_dense_ebops_item &it = items[base + t];
            if (it.P < 1 || it.K < 1 || it.N < 1) return fail(HGQ_ERR_ARG, "hgq_dense_ebops_multi: bad sizes in item %d", base + t);
            if (!it.i_in || !it.f_in || !it.b_ker || !it.ebops || !it.k_in || !it.k_ker)
                return fail(HGQ_ERR_ARG, "hgq_dense_ebops_multi: null pointer in item %d", base + t);
            if (it.K > HGQ_EBOPS_MAXK) return fail(HGQ_ERR_UNSUPPORTED, "hgq_dense_ebops_multi: K=%d > %d", it.K, HGQ_EBOPS_MAXK);
            if (!(Mode(it.mode_ker).kbi) || (it.b_bias && !(Mode(it.mode_bias).kbi)))
                return fail(HGQ_ERR_UNSUPPORTED, "hgq_dense_ebops_multi: kernel/bias bit-widths must use the KBI parametrisation");
            if (it.amax_part && (it.n_parts < 1 || Mode(it.mode_in).kbi || Mode(it.mode_in).overflow_mode != HGQ_WRAP))
                return fail(HGQ_ERR_ARG, "hgq_dense_ebops_multi: fused tracking is for KIF WRAP input quantizers");
            // the items of one launch run concurrently: an update of integer bits another item reads or updates would race
            for (int u = 0; u < t; ++u)
                if (b.item[u].i_in == it.i_in && (it.amax_part || items[base + u].amax_part))
                    return fail(HGQ_ERR_ARG, "hgq_dense_ebops_multi: items %d and %d share integer bits one of them updates; pass them in separate calls", base + u, base + t);
            b.item[t] = it;
            if (it.amax_part && it.P * it.K * it.n_parts > 16384) {
                // many tracker slices: combine them with one thread group per entry across the device first (all such
                // layers in one launch)
                hgq_track_item &tr = tracks[n_tracks++];
                tr.amax = it.amax_part, tr.anyneg = nullptr, tr.n_parts = it.n_parts, tr.i_var = it.i_in, tr.fb = it.f_in, tr.k_var = nullptr;
                tr.m = it.P * it.K, tr.decay = it.decay, tr.c_lo = 0.0f, tr.c_hi = 0.0f;
                tr.mode = it.mode_in & ~(HGQ_MODE_TRACING | HGQ_MODE_SYMMETRIC);
                b.item[t].amax_part = nullptr;
            }
        }
        if (n_tracks) {
            int rc = hgq_wrap_track_i_multi(tracks, n_tracks, stream);
            if (rc) return rc;
        }
        hipLaunchKernelGGL(dense_ebops_multi_kernel, dim3((unsigned)nb), dim3(HGQ_EBOPS_NT), 0, (hipStream_t)stream, b);
        int rc = check_launch("hgq_dense_ebops_multi");
        if (rc) return rc;
    }
    return HGQ_OK;
}

extern "C" int hgq_sparse_ce_fwd_bwd(const float *logits, const int64_t *labels, float *loss, float *dlogits,
                                     int64_t rows, int C, uint32_t *state, void *stream) {
    if (rows < 1 || C < 1) return fail(HGQ_ERR_ARG, "hgq_sparse_ce_fwd_bwd: bad sizes");
    if (!logits || !labels || !loss) return fail(HGQ_ERR_ARG, "hgq_sparse_ce_fwd_bwd: null pointer");
    hipStream_t s = (hipStream_t)stream;
    if (state && ((uintptr_t)state & 7u)) return fail(HGQ_ERR_ARG, "hgq_sparse_ce_fwd_bwd: state must be 8-byte aligned");
    const int grid = state ? persistent_grid((rows + 255) / 256, 4) : 1;
    hipLaunchKernelGGL(sparse_ce_kernel, dim3(grid), dim3(256), 0, s, logits, labels, loss, dlogits, rows, C, state);
    return check_launch("hgq_sparse_ce_fwd_bwd");
}

extern "C" int hgq_gather_batch(const void *x_src, int64_t x_row_bytes, const void *y_src, int64_t y_row_bytes, const int64_t *order,
                                void *state, void *x_dst, void *y_dst, int64_t batch, int64_t n_rows, void *stream) {
    if (batch < 1 || n_rows < 1 || x_row_bytes < 4 || y_row_bytes < 0 || (x_row_bytes & 3) || (y_row_bytes & 3))
        return fail(HGQ_ERR_ARG, "hgq_gather_batch: sizes must be positive and rows whole 32-bit words");
    if (batch * (x_row_bytes + y_row_bytes) >= (1ll << 40)) return fail(HGQ_ERR_UNSUPPORTED, "hgq_gather_batch: batch too large");
    if (!x_src || !x_dst || !order || !state || (y_row_bytes && (!y_src || !y_dst))) return fail(HGQ_ERR_ARG, "hgq_gather_batch: null pointer");
    if (((uintptr_t)x_src | (uintptr_t)x_dst | (uintptr_t)y_src | (uintptr_t)y_dst) & 3u)
        return fail(HGQ_ERR_ARG, "hgq_gather_batch: arrays must be 4-byte aligned");
    if (((uintptr_t)state | (uintptr_t)order) & 7u) return fail(HGQ_ERR_ARG, "hgq_gather_batch: order and state must be 8-byte aligned");
    const bool vec = (x_row_bytes & 15) == 0 && ((((uintptr_t)x_src | (uintptr_t)x_dst)) & 15u) == 0;
    const int64_t items = batch * (vec ? x_row_bytes / 16 : x_row_bytes / 4);
    const dim3 grid((unsigned)persistent_grid((items + 255) / 256, 8));
    if (vec)
        hipLaunchKernelGGL(gather_batch_kernel<true>, grid, dim3(256), 0, (hipStream_t)stream, (const uint32_t *)x_src, x_row_bytes / 4,
                           (const uint32_t *)y_src, y_row_bytes / 4, order, (unsigned long long *)state, (uint32_t *)x_dst, (uint32_t *)y_dst, batch, n_rows);
    else
        hipLaunchKernelGGL(gather_batch_kernel<false>, grid, dim3(256), 0, (hipStream_t)stream, (const uint32_t *)x_src, x_row_bytes / 4,
                           (const uint32_t *)y_src, y_row_bytes / 4, order, (unsigned long long *)state, (uint32_t *)x_dst, (uint32_t *)y_dst, batch, n_rows);
    return check_launch("hgq_gather_batch");
}

extern "C" int hgq_ebops_finish_fwd(const float *ebops, float factor, const float *beta, uint32_t *ebops_u32, float *out, void *stream) {
    if (!ebops || !beta || !out) return fail(HGQ_ERR_ARG, "hgq_ebops_finish_fwd: null pointer");
    hipLaunchKernelGGL(ebops_finish_fwd_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, ebops, factor, beta, ebops_u32, out);
    return check_launch("hgq_ebops_finish_fwd");
}

extern "C" int hgq_ebops_finish_bwd(const float *g, const float *beta, float factor, float *d_ebops, void *stream) {
    if (!g || !beta || !d_ebops) return fail(HGQ_ERR_ARG, "hgq_ebops_finish_bwd: null pointer");
    hipLaunchKernelGGL(ebops_finish_bwd_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, g, beta, factor, d_ebops);
    return check_launch("hgq_ebops_finish_bwd");
}

extern "C" int hgq_qbits_fwd(const uint8_t *k, const float *i, const float *fb, int64_t n, int kbi, int add_mode, float *out,
                             void *stream) {
    if (n < 0 || add_mode < 0 || add_mode > 2) return fail(HGQ_ERR_ARG, "hgq_qbits_fwd: bad arguments");
    if (n == 0) return HGQ_OK;
    if (!fb || !out || (!kbi && !i) || (add_mode && !k)) return fail(HGQ_ERR_ARG, "hgq_qbits_fwd: null pointer");
    hipLaunchKernelGGL(qbits_fwd_kernel, dim3((unsigned)persistent_grid((n + 255) / 256, 8)), dim3(256), 0, (hipStream_t)stream, k, i, fb, n, kbi,
                       add_mode, out);
    return check_launch("hgq_qbits_fwd");
}

extern "C" int hgq_qbits_bwd(const float *g, const float *i, const float *fb, int64_t n, int kbi, float *di, float *dfb, void *stream) {
    if (n < 0) return fail(HGQ_ERR_ARG, "hgq_qbits_bwd: bad size");
    if (n == 0) return HGQ_OK;
    if (!g || !dfb || (!kbi && (!i || !fb || !di))) return fail(HGQ_ERR_ARG, "hgq_qbits_bwd: null pointer");
    hipLaunchKernelGGL(qbits_bwd_kernel, dim3((unsigned)persistent_grid((n + 255) / 256, 8)), dim3(256), 0, (hipStream_t)stream, g, i, fb, n, kbi,
                       di, dfb);
    return check_launch("hgq_qbits_bwd");
}

extern "C" int hgq_bn_fold_fwd(const float *w, const float *bias, const float *gamma, const float *mean, const float *second,
                               int is_meansq, float eps, float *fused_w, float *fused_b, float *moving_mean, float *moving_var,
                               float momentum, float one_minus_momentum, int K, int N, void *stream) {
    if (K < 1 || N < 1) return fail(HGQ_ERR_ARG, "hgq_bn_fold_fwd: bad sizes");
    if (!w || !bias || !mean || !second || !fused_w || !fused_b) return fail(HGQ_ERR_ARG, "hgq_bn_fold_fwd: null pointer");
    const int64_t n = (int64_t)K * N;
    hipLaunchKernelGGL(bn_fold_fwd_kernel<false>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, w, bias, gamma, mean,
                       second, is_meansq, eps, fused_w, fused_b, moving_mean, moving_var, momentum, one_minus_momentum, K, N, hgq_qdesc{},
                       hgq_qdesc{});
    return check_launch("hgq_bn_fold_fwd");
}

static int fold_quant_check(const hgq_qdesc *qk, const hgq_qdesc *qb, const char *who) {
    if (!qk || !qb || !qk->k || !qk->i || !qk->fb || !qb->k || !qb->i || !qb->fb) return fail(HGQ_ERR_ARG, "%s: null quantizer operand", who);
    for (const hgq_qdesc *q : {qk, qb}) {
        const Mode m(q->mode);
        if (!m.training) return fail(HGQ_ERR_ARG, "%s: training-mode quantizers only", who);
        if (m.overflow_mode == HGQ_WRAP) return fail(HGQ_ERR_UNSUPPORTED, "%s: WRAP quantizers track their integer bits per call and are not fused", who);
    }
    return HGQ_OK;
}

extern "C" int hgq_bn_fold_quant_fwd(const float *w, const float *bias, const float *gamma, const float *mean, const float *second,
                                     int is_meansq, float eps, const hgq_qdesc *qk, const hgq_qdesc *qb, float *qw, float *qbias,
                                     float *moving_mean, float *moving_var, float momentum, float one_minus_momentum, int K, int N,
                                     void *stream) {
    if (K < 1 || N < 1) return fail(HGQ_ERR_ARG, "hgq_bn_fold_quant_fwd: bad sizes");
    if (!w || !bias || !mean || !second || !qw || !qbias) return fail(HGQ_ERR_ARG, "hgq_bn_fold_quant_fwd: null pointer");
    const int rc = fold_quant_check(qk, qb, "hgq_bn_fold_quant_fwd");
    if (rc) return rc;
    const int64_t n = (int64_t)K * N;
    hipLaunchKernelGGL(bn_fold_fwd_kernel<true>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, w, bias, gamma, mean,
                       second, is_meansq, eps, qw, qbias, moving_mean, moving_var, momentum, one_minus_momentum, K, N, *qk, *qb);
    return check_launch("hgq_bn_fold_quant_fwd");
}

extern "C" int hgq_bn_fold_bwd(const float *w, const float *gamma, const float *mean, const float *second, int is_meansq, float eps,
                               const float *d_fw, const float *d_fb, float *dw, float *dbias, float *dgamma, float *dmean,
                               float *dsecond, int K, int N, void *stream) {
    if (K < 1 || N < 1) return fail(HGQ_ERR_ARG, "hgq_bn_fold_bwd: bad sizes");
    if (!w || !mean || !second || !d_fw || !d_fb || !dw) return fail(HGQ_ERR_ARG, "hgq_bn_fold_bwd: null pointer");
    if ((int64_t)K * N * 4 >= (1ll << 31)) return fail(HGQ_ERR_UNSUPPORTED, "hgq_bn_fold_bwd: the kernel matrix must be smaller than 2 GiB");
    hipLaunchKernelGGL((bn_fold_bwd_kernel<false, 64>), dim3((unsigned)((N + 63) / 64)), dim3(256), 0, (hipStream_t)stream, w, gamma, mean, second,
                       is_meansq, eps, d_fw, d_fb, dw, dbias, dgamma, dmean, dsecond, K, N, (const float *)nullptr, hgq_qdesc{}, hgq_qdesc{},
                       (float *)nullptr, (float *)nullptr, (float *)nullptr, (float *)nullptr);
    return check_launch("hgq_bn_fold_bwd");
}

extern "C" int hgq_bn_fold_quant_bwd(const float *w, const float *bias, const float *gamma, const float *mean, const float *second,
                                     int is_meansq, float eps, const hgq_qdesc *qk, const hgq_qdesc *qb, const float *d_qw,
                                     const float *d_qb, float *dw, float *dbias, float *dgamma, float *dmean, float *dsecond, float *di_k,
                                     float *dfb_k, float *di_b, float *dfb_b, int K, int N, void *stream) {
    if (K < 1 || N < 1) return fail(HGQ_ERR_ARG, "hgq_bn_fold_quant_bwd: bad sizes");
    if (!w || !bias || !mean || !second || !d_qw || !d_qb || !dw || !di_k || !dfb_k || !di_b || !dfb_b)
        return fail(HGQ_ERR_ARG, "hgq_bn_fold_quant_bwd: null pointer");
    if ((int64_t)K * N * 4 >= (1ll << 31)) return fail(HGQ_ERR_UNSUPPORTED, "hgq_bn_fold_quant_bwd: the kernel matrix must be smaller than 2 GiB");
    const int rc = fold_quant_check(qk, qb, "hgq_bn_fold_quant_bwd");
    if (rc) return rc;
    hipLaunchKernelGGL((bn_fold_bwd_kernel<true, 16>), dim3((unsigned)((N + 15) / 16)), dim3(256), 0, (hipStream_t)stream, w, gamma, mean, second,
                       is_meansq, eps, d_qw, d_qb, dw, dbias, dgamma, dmean, dsecond, K, N, bias, *qk, *qb, di_k, dfb_k, di_b, dfb_b);
    return check_launch("hgq_bn_fold_quant_bwd");
}

extern "C" int64_t hgq_mse_workspace(void) { return MSE_PARTS; }

extern "C" int hgq_mse_fwd(const float *pred, const float *target, float *loss, float *workspace, int64_t n, void *stream) {
    if (n < 1) return fail(HGQ_ERR_ARG, "hgq_mse_fwd: bad size");
    if (!pred || !loss || !workspace) return fail(HGQ_ERR_ARG, "hgq_mse_fwd: null pointer");
    if (((uintptr_t)pred & 15u) || ((uintptr_t)target & 15u)) return fail(HGQ_ERR_ARG, "hgq_mse_fwd: operands must be 16-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    int grid = persistent_grid(((n >> 2) + 255) / 256, 4);
    if (grid > MSE_PARTS) grid = MSE_PARTS;
    hipLaunchKernelGGL(mse_partial_kernel, dim3(grid), dim3(256), 0, s, pred, target, n, workspace, (float *)nullptr, 0.f);
    int rc = check_launch("hgq_mse_fwd");
    if (rc) return rc;
    hipLaunchKernelGGL(mse_finish_kernel, dim3(1), dim3(64), 0, s, workspace, grid, 1.0f / (float)n, loss);
    return check_launch("hgq_mse_fwd(finish)");
}

extern "C" int hgq_mse_fwd_bwd(const float *pred, const float *target, float *loss, float *dpred, float *workspace, int64_t n, void *stream) {
    if (n < 1) return fail(HGQ_ERR_ARG, "hgq_mse_fwd_bwd: bad size");
    if (!pred || !loss || !dpred || !workspace) return fail(HGQ_ERR_ARG, "hgq_mse_fwd_bwd: null pointer");
    if (((uintptr_t)pred & 15u) || ((uintptr_t)target & 15u) || ((uintptr_t)dpred & 15u))
        return fail(HGQ_ERR_ARG, "hgq_mse_fwd_bwd: operands must be 16-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    int grid = persistent_grid(((n >> 2) + 255) / 256, 4);
    if (grid > MSE_PARTS) grid = MSE_PARTS;
    hipLaunchKernelGGL(mse_partial_kernel, dim3(grid), dim3(256), 0, s, pred, target, n, workspace, dpred, 2.0f / (float)n);
    int rc = check_launch("hgq_mse_fwd_bwd");
    if (rc) return rc;
    hipLaunchKernelGGL(mse_finish_kernel, dim3(1), dim3(64), 0, s, workspace, grid, 1.0f / (float)n, loss);
    return check_launch("hgq_mse_fwd_bwd(finish)");
}

extern "C" int hgq_mse_bwd(const float *pred, const float *target, const float *g, float *dpred, int64_t n, void *stream) {
    if (n < 1) return fail(HGQ_ERR_ARG, "hgq_mse_bwd: bad size");
    if (!pred || !g || !dpred) return fail(HGQ_ERR_ARG, "hgq_mse_bwd: null pointer");
    if (((uintptr_t)pred & 15u) || ((uintptr_t)target & 15u) || ((uintptr_t)dpred & 15u))
        return fail(HGQ_ERR_ARG, "hgq_mse_bwd: operands must be 16-byte aligned");
    const int grid = persistent_grid(((n >> 2) + 255) / 256, 8);
    hipLaunchKernelGGL(mse_bwd_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream, pred, target, g, 2.0f / (float)n, n, dpred);
    return check_launch("hgq_mse_bwd");
}

extern "C" int hgq_sgd_update(float *w, const float *g, int64_t n, float lr, float l1, float lo, float hi, void *stream) {
    if (n < 0) return fail(HGQ_ERR_ARG, "hgq_sgd_update: bad size");
    if (n == 0) return HGQ_OK;
    if (!w || !g) return fail(HGQ_ERR_ARG, "hgq_sgd_update: null pointer");
    const int grid = persistent_grid((n + 255) / 256, 8);
    hipLaunchKernelGGL(sgd_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream, w, g, n, lr, l1, lo, hi);
    return check_launch("hgq_sgd_update");
}

static inline int moments_layout(int64_t rows, int N, bool vec, int &TX, int64_t &gx, int64_t &gy) {
    const int64_t cg = vec ? N / 4 : N;
    TX = 1;
    while (TX * 2 <= cg && TX < 64) TX *= 2;
    const int TY = 256 / TX;
    gx = (cg + TX - 1) / TX;
    gy = (rows + TY - 1) / TY;
    int64_t cap = (int64_t)persistent_grid(1 << 30, 4) / gx;
    if (cap > 256) cap = 256;
    if (gy > cap) gy = cap < 1 ? 1 : cap;
    return 0;
}

extern "C" int64_t hgq_col_moments_workspace(int64_t rows, int N) {
    if (rows < 0 || N < 1) return -1;
    int TX;
    int64_t gx, gy;
    moments_layout(rows, N, N % 4 == 0, TX, gx, gy);
    return gy * 2 * N;
}

extern "C" int hgq_col_moments_fwd(const float *x, int64_t rows, int N, float *mean, float *meansq, float *workspace,
                                   void *stream) {
    hipStream_t s = (hipStream_t)stream;
    if (rows < 1 || N < 1) return fail(HGQ_ERR_ARG, "hgq_col_moments_fwd: bad sizes");
    if (!x || !mean || !meansq || !workspace) return fail(HGQ_ERR_ARG, "hgq_col_moments_fwd: null pointer");
    const bool vec = N % 4 == 0 && ((uintptr_t)x & 15u) == 0;
    int TX;
    int64_t gx, gy;
    moments_layout(rows, N, N % 4 == 0, TX, gx, gy);
    if (!vec && N % 4 == 0) moments_layout(rows, N, false, TX, gx, gy), gy = hgq_col_moments_workspace(rows, N) / (2 * N);
    if (vec)
        hipLaunchKernelGGL((col_moments_kernel<4>), dim3((unsigned)gx, (unsigned)gy), dim3(256), 0, s, x, rows, N, TX, workspace);
    else
        hipLaunchKernelGGL((col_moments_kernel<1>), dim3((unsigned)gx, (unsigned)gy), dim3(256), 0, s, x, rows, N, TX, workspace);
    int rc = check_launch("hgq_col_moments_fwd");
    if (rc) return rc;
    return reduce_parts(workspace, (int)gy, 2 * (int64_t)N, mean, N, meansq, N, nullptr, 0, s, 1.0f / (float)rows);
}

extern "C" int hgq_col_moments_bwd(const float *x, const float *dmean, const float *dmeansq, int64_t rows, int N, float *dx,
                                   void *stream) {
    if (rows < 0 || N < 1) return fail(HGQ_ERR_ARG, "hgq_col_moments_bwd: bad sizes");
    if (rows == 0) return HGQ_OK;
    if (!x || !dmean || !dmeansq || !dx) return fail(HGQ_ERR_ARG, "hgq_col_moments_bwd: null pointer");
    const int64_t n = rows * N;
    hipLaunchKernelGGL(col_moments_bwd_kernel, dim3((unsigned)persistent_grid((n + 255) / 256, 16)), dim3(256), 0, (hipStream_t)stream, x, dmean,
                       dmeansq, n, N, 1.0f / (float)rows, dx);
    return check_launch("hgq_col_moments_bwd");
}
