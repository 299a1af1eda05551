/*
 * hgq_hip.h - C ABI of libhgq_hip.so: the HGQ2 quantized-training hot path on MI355X (gfx950).
 *
 * The reference (calad0i/HGQ2) is pure Python and has no FFI; the seam these entry points sit
 * behind is the stateless quantizer callable it imports from the third-party package
 * `quantizers` and the chains of eager keras.ops calls inside its layers.  Each declaration
 * cites the reference code it replaces (paths relative to the reference root).
 *
 * Conventions
 *   - every pointer is a DEVICE pointer to contiguous memory, fp32 unless stated otherwise;
 *   - the library never allocates, never frees and never synchronises; all work is enqueued on
 *     `stream` (a hipStream_t passed as void*; NULL = the default stream);
 *   - every function returns HGQ_OK (0) or a negative HGQ_ERR_* code; hgq_last_error() returns a
 *     thread-local description of the last failure;
 *   - outputs that are reductions (bit-width gradients, abs-max trackers) are cleared by the
 *     entry point itself with a fill kernel (safe under HIP graph capture), then accumulated;
 *   - bit-width operands (k, i, f or b) must hold integer-valued floats after the optional
 *     rounding selected by HGQ_MODE_ROUND_PARAMS; powers of two are formed exactly from them;
 *   - the entry points keep no state between calls, with two exceptions that are named where they are declared:
 *     hgq_dense_use_bf16_parts (ONE process-wide switch: which matrix instruction the contractions issue; it
 *     changes instruction selection only, results stay the fp32 contraction) and the per-GPU scratch array of
 *     hgq_quantize_bwd_static.
 *
 * Bit-width broadcasting: element `e` of a tensor with `n` elements uses bit-width entry
 * `(e / bw_inner) % bw_size`.  bw_size == n, bw_inner == 1 is the per-element case;
 * bw_size == 1 a single shared bit-width; a tensor [B, ...] with bit-widths [1, ...] has
 * bw_size = n / B, bw_inner = 1.
 */
#ifndef HGQ_HIP_H
#define HGQ_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HGQ_OK 0
#define HGQ_ERR_ARG (-1)         /* null pointer, negative size, unknown mode */
#define HGQ_ERR_LAUNCH (-2)      /* the HIP runtime refused a launch; see hgq_last_error() */
#define HGQ_ERR_UNSUPPORTED (-3) /* shape outside what the kernel family covers */

/* rounding modes (low nibble of `mode`) */
#define HGQ_TRN 0
#define HGQ_RND 1
#define HGQ_RND_CONV 2
#define HGQ_S_RND 3      /* stochastic in training (hgq_quantize_*_stochastic); RND otherwise */
#define HGQ_S_RND_CONV 4 /* stochastic in training; RND_CONV otherwise */
/* overflow modes (second nibble of `mode`) */
#define HGQ_WRAP 0
#define HGQ_SAT 1
#define HGQ_SAT_SYM 2

#define HGQ_MODE(round_mode, overflow_mode) ((round_mode) | ((overflow_mode) << 4))
#define HGQ_MODE_TRAINING (1 << 8)     /* training-mode forward: WRAP is round-only, no zeroing of empty words */
#define HGQ_MODE_KBI (1 << 9)          /* third bit-width operand is b (total bits); f = b - i */
#define HGQ_MODE_ROUND_PARAMS (1 << 10) /* operands are the raw trainable variables: round half-even first */
#define HGQ_MODE_K_U8 (1 << 11)        /* k operand is uint8 (the reference's `_k` variable dtype) */
#define HGQ_MODE_SYMMETRIC (1 << 12)   /* hgq_wrap_track_i: the symmetric minimal-i formula */
#define HGQ_MODE_TRACING (1 << 13)     /* hgq_wrap_track_i: calibration ("tracing") update rule */
#define HGQ_MODE_TRACK_INPUT (1 << 14) /* hgq_quantize_fwd: amax / anyneg observe x instead of y (KBI WRAP tracks the un-rounded input) */

#define HGQ_ACT_NONE 0
#define HGQ_ACT_RELU 1

int hgq_version(void);
const char *hgq_last_error(void);

/*
 * Fixed-point quantizer, forward.  Replaces the callable returned by
 * quantizers.fixed_point._fixed_point_ops._get_fixed_quantizer(round_mode, overflow_mode),
 * i.e. `q(x, k, i, f, training, seed_gen)` and `q.round(x, f, ...)` (imported at
 * src/hgq/quantizer/internal/fixed_point_quantizer.py:9, called at :147, :288, :305, :405),
 * together with the broadcast of k/i/f and the inference-time zeroing around it
 * (fixed_point_quantizer.py:142-150) and the `round_conv` of the raw variables (:250,:254,:441,:445).
 *
 *   y      [n]        quantized values
 *   amax   [bw_size]  optional (NULL to skip): max |y| over the elements sharing each bit-width
 *                     entry, as the uint32 bit pattern of a non-negative float - the reduction of
 *                     DefaultBitwidthMapper.x_to_bw_absmax (src/hgq/quantizer/internal/base.py:185-186)
 *   anyneg [bw_size]  optional: 1 where any y < 0 (x_to_bw_sign, internal/base.py:188-189)
 */
int hgq_quantize_fwd(const float *x, const void *k, const float *i, const float *fb, float *y,
                     uint32_t *amax, uint32_t *anyneg, int64_t n, int64_t bw_size, int64_t bw_inner,
                     int mode, void *stream);

/*
 * hgq_quantize_fwd with the trackers as slices: when bit-widths are shared along the leading axis only
 * (bw_inner == 1, bw_size < n) the kernel can leave one abs-max / any-negative slice per row chunk instead of
 * combining them with atomics; hgq_wrap_track_i takes the slices as they are (n_parts = n_slices), nothing has
 * to be cleared first.  hgq_quantize_tracker_slices returns the slice count for a shape (0: use hgq_quantize_fwd).
 *   amax / anyneg [n_slices, bw_size] (either may be NULL).  Operands 16-byte aligned when bw_size % 4 == 0.
 */
int64_t hgq_quantize_tracker_slices(int64_t n, int64_t bw_size, int64_t bw_inner);
int hgq_quantize_fwd_sliced(const float *x, const void *k, const float *i, const float *fb, float *y, uint32_t *amax, uint32_t *anyneg,
                            int64_t n_slices, int64_t n, int64_t bw_size, int64_t bw_inner, int mode, void *stream);

/*
 * Fixed-point quantizer, surrogate backward (training mode only).  Replaces the custom
 * gradients of the same third-party callable plus autograd through broadcast_to (the sum over
 * the homogeneous axes) and through `f = b - i` for the KBI parametrisation
 * (fixed_point_quantizer.py:256-265).
 *
 *   dx  [n];  di, dfb [bw_size]  (either may be NULL to skip).  With HGQ_MODE_KBI `dfb` is the
 *   gradient w.r.t. b and `di` the total gradient w.r.t. i (direct - via f).
 */
/*
 * hgq_quantize_bwd with the bit-width gradients summed in a fixed order: when bit-widths are shared along the leading
 * axis only (bw_inner == 1, 1 < bw_size < n) every row chunk leaves a slice of partial sums in `workspace`
 * (hgq_quantize_bwd_workspace floats; 0: the shape is not handled here, use hgq_quantize_bwd) and a second launch adds
 * the slices in order - no atomics, nothing to clear, the same bits on every run.  dfb is required, di and dx optional.
 */
int64_t hgq_quantize_bwd_workspace(int64_t n, int64_t bw_size, int64_t bw_inner);
int hgq_quantize_bwd_sliced(const float *dy, const float *x, const void *k, const float *i, const float *fb, float *dx, float *di,
                            float *dfb, float *workspace, int64_t n, int64_t bw_size, int64_t bw_inner, int mode, void *stream);
/*
 * The first launch of hgq_quantize_bwd_sliced alone: `workspace` keeps hgq_quantize_bwd_slice_count() slices, each
 * [dfb (bw_size) | di (bw_size, only with want_di)], for a caller that adds the slice sets of several quantizers of a
 * backward pass in one launch (hgq_reduce_slices_multi) - their sums are first read by the optimizer.
 */
int64_t hgq_quantize_bwd_slice_count(int64_t n, int64_t bw_size, int64_t bw_inner);
int hgq_quantize_bwd_slices(const float *dy, const float *x, const void *k, const float *i, const float *fb, float *dx, int want_di,
                            float *workspace, int64_t n, int64_t bw_size, int64_t bw_inner, int mode, void *stream);

/*
 * Stochastic rounding: the training-mode forward and surrogate backward of round modes S_RND / S_RND_CONV
 * (src/hgq/quantizer/internal/fixed_point_quantizer.py:56-57,279,288,404-405: `q(..., seed_gen)`,
 * `q.round(x, f, stochastic, seed_gen)`): R(t) = floor(t + u) with u uniform in [0, 1), then the overflow mode.
 * The reference's draws come from a Keras SeedGenerator, whose stream is backend-specific; here element e of a call
 * draws u = (word e % 4 of Philox4x32-10(counter = (e / 4, offset), key = seed) >> 8) * 2^-24, so a call is a pure
 * function of (seed, offset): pass the same pair to the backward, and a new offset to every forward call.
 * Outside training these round modes are the deterministic RND / RND_CONV: call hgq_quantize_fwd with that mode.
 *   amax / anyneg [bw_size] optional trackers as in hgq_quantize_fwd.  di / dfb [bw_size]: with shared bit-widths the
 *   sums are accumulated with float atomics (the last bits depend on the order of arrival).
 */
int hgq_quantize_fwd_stochastic(const float *x, const void *k, const float *i, const float *fb, float *y, uint32_t *amax, uint32_t *anyneg,
                                int64_t n, int64_t bw_size, int64_t bw_inner, int mode, uint64_t seed, uint64_t offset, void *stream);
int hgq_quantize_bwd_stochastic(const float *dy, const float *x, const void *k, const float *i, const float *fb, float *dx, float *di,
                                float *dfb, int64_t n, int64_t bw_size, int64_t bw_inner, int mode, uint64_t seed, uint64_t offset,
                                void *stream);
/*
 * The same pair with the draw's offset partly in device memory, so that a launch recorded into a HIP graph draws anew on
 * every replay: the forward uses offset + offset_base[0] and leaves that sum in used_offset[0]; the backward repeats the draw
 * named by used_offset[0].  hgq_counters_advance adds increments[j] to counters[j][0] (any number, 32 per launch; a counter
 * may be listed once): a trainer calls it once per step with the number of draws each seed generator made, which is the
 * advance keras.random.SeedGenerator makes on the host (reference src/hgq/quantizer/internal/fixed_point_quantizer.py:56-57,
 * :142-150).  Same shapes, modes and errors as the pair above.
 */
int hgq_quantize_fwd_stochastic_at(const float *x, const void *k, const float *i, const float *fb, float *y, uint32_t *amax,
                                   uint32_t *anyneg, int64_t n, int64_t bw_size, int64_t bw_inner, int mode, uint64_t seed,
                                   uint64_t offset, const uint64_t *offset_base, uint64_t *used_offset, void *stream);
int hgq_quantize_bwd_stochastic_at(const float *dy, const float *x, const void *k, const float *i, const float *fb, float *dx, float *di,
                                   float *dfb, int64_t n, int64_t bw_size, int64_t bw_inner, int mode, uint64_t seed,
                                   const uint64_t *used_offset, void *stream);
int hgq_counters_advance(uint64_t *const *counters, const uint64_t *increments, int count, void *stream);

/*
 * Measurement aid (no counterpart in the reference): o_j[e] = (j + 1) * (a[e] (+ b[e]) (+ c[e])) for the first n_write
 * (1..4) outputs and n_read (1..3) inputs, one 128-bit non-temporal access per array per thread.  4 * (n_read + n_write) * n
 * bytes cross HBM per launch and nothing else: used to scale the hardware traffic counters and as the bandwidth a plain
 * streaming kernel of a given read / write mix reaches at a given size.  n a multiple of 4, arrays 16-byte aligned.
 */
int hgq_stream_probe(const float *a, const float *b, const float *c, float *o0, float *o1, float *o2, float *o3, int n_read,
                     int n_write, int64_t n, void *stream);

/*
 * hgq_quantize_bwd_sliced without a workspace argument.  This entry point has no counterpart in the reference.  It is
 * for callers that cannot allocate device memory around the call: code running under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc.  The slices go to a device array that is part of the library's code object
 * (HGQ_STATIC_SCRATCH_FLOATS floats = 1 MiB, held on every GPU the library runs on until the process ends); the call
 * allocates and frees nothing.  Same arguments, results (bit for bit) and errors as hgq_quantize_bwd_sliced, plus
 * HGQ_ERR_ARG when hgq_quantize_bwd_workspace(n, bw_size, bw_inner) exceeds HGQ_STATIC_SCRATCH_FLOATS.
 * All calls on one GPU share that GPU's array: calls that overlap on one GPU (different streams or threads) race;
 * calls on one stream are ordered.  Nothing needs clearing between calls: every slice entry read is written first.
 */
#define HGQ_STATIC_SCRATCH_FLOATS (1 << 18)
int hgq_quantize_bwd_static(const float *dy, const float *x, const void *k, const float *i, const float *fb, float *dx, float *di,
                            float *dfb, int64_t n, int64_t bw_size, int64_t bw_inner, int mode, void *stream);

/*
 * Many quantizers with per-element bit-widths (bw_size == n, no trackers) in one launch each way: the kernel and bias
 * quantizers of a model (src/hgq/layers/core/dense.py:72-79 `self.kq(self._kernel)`, `self.bq(self.bias)` and the same
 * in the other layers) depend on the variables only, so all of them can run before the first layer and their gradients
 * after the last.  Per item the arithmetic is that of hgq_quantize_fwd / hgq_quantize_bwd with bw_size == n; each item
 * carries its own HGQ_MODE(...) bits.  Descriptors are read on the host and travel as launch arguments (safe under HIP
 * graph capture).  Backward: dy NULL = zero upstream gradient; dx, di, dfb may each be NULL.
 */
#define HGQ_QUANT_BATCH 32
typedef struct {
    const float *x;
    const void *k;
    const float *i, *fb;
    float *y;
    int64_t n;
    int mode;
} hgq_quant_item;
typedef struct {
    const float *dy, *x;
    const void *k;
    const float *i, *fb;
    float *dx, *di, *dfb;
    int64_t n;
    int mode;
} hgq_quant_grad_item;
int hgq_quantize_fwd_multi(const hgq_quant_item *items, int count, void *stream);
int hgq_quantize_bwd_multi(const hgq_quant_grad_item *items, int count, void *stream);

int hgq_quantize_bwd(const float *dy, const float *x, const void *k, const float *i, const float *fb,
                     float *dx, float *di, float *dfb, int64_t n, int64_t bw_size, int64_t bw_inner,
                     int mode, void *stream);

/*
 * Training-mode forward and surrogate backward of the fixed-point quantizer in one launch, for callers that hold the
 * upstream gradient when they quantize (the standalone quantizer step: `y = q(x, k, i, f, training=True)` followed by
 * the custom gradients of the same callable, src/hgq/quantizer/internal/fixed_point_quantizer.py:142-150,401-429).
 * Results are those of hgq_quantize_fwd (HGQ_MODE_TRAINING, no trackers) and hgq_quantize_bwd on the same operands,
 * bit for bit.  With per-element bit-widths (bw_size == n), 16-byte aligned operands and an fp32 or dead k every
 * operand crosses HBM once: x, f, dy read and y, dx, di, dfb written (28 B per element) for a WRAP quantizer, whose
 * training branch reads neither k nor i; 36 B per element with every operand live.  Other layouts run the two passes.
 *   y [n] required; dx [n], di, dfb [bw_size] may each be NULL.  HGQ_MODE_TRAINING must be set.
 */
int hgq_quantize_fwd_bwd(const float *x, const void *k, const float *i, const float *fb, const float *dy, float *y, float *dx,
                         float *di, float *dfb, int64_t n, int64_t bw_size, int64_t bw_inner, int mode, void *stream);

/*
 * Integer-bit tracking of WRAP quantizers.  Replaces minimal_i_given_xf / minimal_i_given_xb
 * (fixed_point_quantizer.py:16-31) and the `_i.assign(...)` recurrences of
 * FixedPointQuantizerKIF.call (:406-422) and FixedPointQuantizerKBI.call (:280-300).
 *
 *   amax / anyneg [n_parts, m]: trackers as produced by hgq_quantize_fwd (n_parts = 1) or by
 *   hgq_qdense_fwd (one slice per producing workgroup); they are combined here.
 *   i_var [m]  in/out: the raw `_i` variable;   fb [m]: raw `_f` (KIF) or `_b` (KBI)
 *   training : i_var <- max(i_var - decay, minimal_i)            (KBI: then clipped to [c_lo, c_hi])
 *   tracing  : i_var <- max(round(i_var), clip(minimal_i)),  k_var |= anyneg   (k_var uint8, optional)
 */
int hgq_wrap_track_i(const uint32_t *amax, const uint32_t *anyneg, int n_parts, float *i_var, const float *fb,
                     uint8_t *k_var, int64_t m, float decay, float c_lo, float c_hi, int mode, void *stream);

/*
 * The same update for several quantizers in one launch.  In a training step each WRAP quantizer of a model updates
 * its integer bits right after its own forward (fixed_point_quantizer.py:406-413); the updates are independent of
 * each other and nothing in the forward pass reads them before the EBOPs estimates do, so a caller may collect them.
 * Items with the fields of hgq_wrap_track_i; up to HGQ_TRACK_BATCH per launch, more are split over launches.
 * The items of a launch run concurrently: two items of one launch that name the same i_var are refused (HGQ_ERR_ARG) - the
 * repeated updates of a quantizer that several layers share go into successive calls.
 */
#define HGQ_TRACK_BATCH 16
typedef struct {
    const uint32_t *amax, *anyneg;
    int32_t n_parts;
    float *i_var;
    const float *fb;
    uint8_t *k_var;
    int64_t m;
    float decay, c_lo, c_hi;
    int32_t mode;
} hgq_track_item;
int hgq_wrap_track_i_multi(const hgq_track_item *items, int count, void *stream);

/*
 * QDense / QEinsumDense contraction, forward, with the input quantizer fused into the operand
 * load.  Replaces `ops.matmul(self.iq(inputs), self.qkernel) + self.qbias` and the activation
 * (src/hgq/layers/core/dense.py:60-68; einsum_dense.py:72-83 for equations that reshape to a
 * GEMM), including the abs-max reduction the WRAP input quantizer needs
 * (fixed_point_quantizer.py:405-408).
 *
 *   x [rows, K];  k_in/i_in/f_in [bw_rows, K] input-quantizer operands (row r uses entry
 *   r % bw_rows); bw_rows == 0 means x is used as is;  qw [K, N] quantized kernel;
 *   qb [N] quantized bias or NULL;  y [rows, N];
 *   amax_part [hgq_qdense_fwd_parts(rows), bw_rows*K] optional: per-workgroup slices of the
 *   abs-max tracker (no atomics, no clearing pass), to be handed to hgq_wrap_track_i.
 *   `mode` selects the input quantizer (any round / overflow mode, training or inference);
 *   act is HGQ_ACT_*.
 */
int hgq_qdense_fwd_parts(int64_t rows);
/*
 * The streaming kernels (K, N <= 64) contract on the bf16 matrix cores: every fp32 operand is split exactly into up to
 * three bf16 parts (8 + 8 + 8 significant bits), the products of parts are exact in fp32 and are accumulated in fp32,
 * and only the non-zero parts are multiplied - quantized operands of up to 8 bits need one part, up to 16 bits two.
 * The convolution and attention kernels take the same choice (sixteen contraction steps at a time: one bf16 instruction
 * where both operands have one part, three where one of them is a gradient, the eight fp32 instructions otherwise).
 * Same values as the fp32 matrix instruction up to the order of the fp32 accumulation.  `on` = 0 selects the fp32
 * instruction instead, 1 the bf16 parts (default), a negative value changes nothing; returns the previous setting.
 * Process-wide, not synchronised with launches in flight on other threads.
 */
int hgq_dense_use_bf16_parts(int on);
/*
 * hgq_qdense_fwd with the layer's output quantizer run on the output tile as it leaves (reference
 * src/hgq/layers/core/base.py:106-116: `return self.oq(r, training=training)` after the layer's call): `y` gets
 * act(q_in(x) W + b), `yq` its quantized values, slice w of `oamax_part` ([hgq_qdense_fwd_parts(rows)][bw_rows_out * N]
 * words, every slice written whole) the abs-max bit patterns of the quantized values per table entry, for
 * hgq_wrap_track_i.  Covers what hgq_qdense_fwd_oq_supported says: both quantizers KIF on their WRAP training branch
 * (round only) with the same round mode, fractional-bit tables [bw_rows, K] and [bw_rows_out, N] whose row counts divide
 * 64 and the rows, K and N multiples of 4 up to 64, the bf16-part kernels selected; HGQ_ERR_UNSUPPORTED otherwise
 * (run hgq_qdense_fwd and hgq_quantize_fwd then).  The gradient is the two separate ones: hgq_quantize_bwd* on (dyq, y),
 * which passes dyq through unchanged, then hgq_qdense_bwd.
 */
int hgq_qdense_fwd_oq_supported(int64_t rows, int K, int N, int64_t bw_rows, int64_t bw_rows_out, int mode, int mode_out);
int hgq_qdense_fwd_oq(const float *x, const float *f_in, int64_t bw_rows, const float *qw, const float *qb, const float *f_out,
                      int64_t bw_rows_out, float *y, float *yq, uint32_t *amax_part, uint32_t *oamax_part, int64_t rows, int K,
                      int N, int act, int mode, int mode_out, void *stream);
int hgq_qdense_fwd(const float *x, const void *k_in, const float *i_in, const float *f_in, int64_t bw_rows,
                   const float *qw, const float *qb, float *y, uint32_t *amax_part, int64_t rows, int K, int N,
                   int act, int mode, void *stream);
/*
 * hgq_qdense_fwd followed by a mean over groups of `mean_rows` consecutive rows, in one launch: a contraction layer whose
 * output [batch, positions, N] goes straight into a mean over the positions (reference src/hgq/layers/core/einsum_dense.py:72-83
 * and src/hgq/layers/einsum_dense_batchnorm.py:185-212 for the layer; the mean is the host framework's
 * GlobalAveragePooling1D behind it).  The output itself is not written: row g of `ymean` [rows / mean_rows, N] = the mean of
 * the activated output rows g * mean_rows .. (g + 1) * mean_rows - 1, summed in a fixed order from the accumulator registers,
 * and with HGQ_ACT_RELU `relu_mask` [rows][2] (32-bit words) gets what the backward pass needs of the output: bit c & 31 of
 * word c >> 5 of a row = column c was positive (NULL without ReLU).  `f_in` / `bw_rows` / `amax_part` as in hgq_qdense_fwd
 * (bw_rows = 0: no input quantizer).  Covers what hgq_qdense_fwd_mean_supported says: mean_rows 32 or 64 dividing the rows,
 * K and N multiples of 4 up to 64, the input quantizer none or KIF on its WRAP training branch with a table whose row count
 * divides 64 and the rows, the bf16-part kernels selected; HGQ_ERR_UNSUPPORTED otherwise (run hgq_qdense_fwd and
 * hgq_mean_mid_fwd then).
 *
 * hgq_qdense_bwd_mean / hgq_qdense_bwd_mean_slices: hgq_qdense_bwd / hgq_qdense_bwd_slices for that pair, from the gradient
 * of the means `dmean` [rows / mean_rows, N] and the mask: row r of the gradient the contraction sees is
 * dmean[r / mean_rows] / mean_rows where the mask bit is set (everywhere without ReLU), read from `dmean` directly (no
 * [rows, N] broadcast copy is made).  All other arguments as in hgq_qdense_bwd(_slices).
 */
int hgq_qdense_fwd_mean_supported(int64_t rows, int K, int N, int64_t bw_rows, int64_t mean_rows, int mode);
int hgq_qdense_fwd_mean(const float *x, const float *f_in, int64_t bw_rows, const float *qw, const float *qb, uint32_t *relu_mask,
                        float *ymean, uint32_t *amax_part, int64_t rows, int K, int N, int64_t mean_rows, int act, int mode,
                        void *stream);
int hgq_qdense_bwd_mean(const float *dmean, const uint32_t *relu_mask, const float *x, const float *f_in, int64_t bw_rows, const float *qw,
                        float *dx, float *dqw, float *dqb, float *df_in, float *workspace, int64_t rows, int K, int N,
                        int64_t mean_rows, int act, int mode, void *stream);
int hgq_qdense_bwd_mean_slices(const float *dmean, const uint32_t *relu_mask, const float *x, const float *f_in, int64_t bw_rows,
                               const float *qw, float *dx, float *workspace, int has_bias, int64_t rows, int K, int N,
                               int64_t mean_rows, int act, int mode, void *stream);

/*
 * QDense / QEinsumDense contraction, backward: autograd of the same expression.
 *   dx [rows, K] gradient w.r.t. the un-quantized input (straight-through);
 *   dqw [K, N], dqb [N] (NULL if no bias): gradients w.r.t. the quantized kernel / bias;
 *   df_in [bw_rows*K]: gradient w.r.t. the input quantizer's fractional bits (NULL if bw_rows == 0);
 *   workspace: hgq_qdense_bwd_workspace(rows, K, N, bw_rows) floats of scratch for the
 *   per-workgroup partial sums, which a second kernel adds up in a fixed order (deterministic).
 * Supported: K <= 64 and N <= 64, training-mode WRAP input quantizer (round-only).
 */
int64_t hgq_qdense_bwd_workspace(int64_t rows, int K, int N, int64_t bw_rows);
int hgq_qdense_bwd(const float *dy, const float *y, const float *x, const float *f_in, int64_t bw_rows,
                   const float *qw, float *dx, float *dqw, float *dqb, float *df_in, float *workspace,
                   int64_t rows, int K, int N, int act, int mode, void *stream);

/*
 * The same backward in two halves, for a caller that reduces the slices of several layers in one launch: the kernel
 * gradient of a layer is first read by the backward of its kernel quantizer, which in a training step runs after the
 * backward of every layer (the quantizers depend on the variables only: src/hgq/layers/core/dense.py:72-79).
 *   hgq_qdense_bwd_slices: writes dx and leaves n = hgq_qdense_bwd_workspace(...) / width slices of
 *   width = K*N + N + bw_rows*K floats in `workspace`: [dqw | dqb | df_in] partial sums per workgroup
 *   (the dqb segment is undefined when has_bias == 0).
 *   hgq_reduce_slices_multi: out[0] | out[1] | out[2] (lengths n_out[0..2], summing to `width`; a NULL pointer skips
 *   that segment) = sum over the slices, in slice order and with the association hgq_qdense_bwd uses, so both routes
 *   give the same bits.  Up to HGQ_REDUCE_BATCH sets per launch, more are split over launches.
 */
#define HGQ_REDUCE_BATCH 16
typedef struct {
    const float *slices; /* [n_slices, width] */
    int32_t n_slices;
    int64_t width;
    float *out[3];
    int64_t n_out[3];
} hgq_reduce_item;
int hgq_qdense_bwd_slices(const float *dy, const float *y, const float *x, const float *f_in, int64_t bw_rows,
                          const float *qw, float *dx, float *workspace, int has_bias, int64_t rows, int K, int N, int act,
                          int mode, void *stream);
int hgq_reduce_slices_multi(const hgq_reduce_item *items, int count, void *stream);
/*
 * hgq_reduce_slices_multi with the backward of quantizers whose upstream gradient is one of the reduced segments - the kernel
 * and bias quantizers behind a contraction (src/hgq/layers/core/dense.py:60-68: `qkernel = self.kq(self.kernel)`) - run on
 * the sums as they are formed: quantizer j (hgq_quant_grad_item, its `dy` ignored, n = the segment's length, per-element
 * bit-widths) reads segment quant_segment[j] of slice set quant_set[j] and writes dx / di / dfb exactly as
 * hgq_quantize_bwd_multi would from the reduced array.  At most HGQ_REDUCE_QUANTS quantizers per HGQ_REDUCE_BATCH consecutive
 * slice sets, one per segment; a segment's own output pointer may then be NULL.
 */
#define HGQ_REDUCE_QUANTS 24
int hgq_reduce_slices_quant_multi(const hgq_reduce_item *items, int count, const hgq_quant_grad_item *quants, const int *quant_set,
                                  const int *quant_segment, int n_quants, void *stream);

/*
 * EBOPs of a dense contraction and its gradient.  Replaces QDense._compute_ebops
 * (src/hgq/layers/core/dense.py:70-80) / QEinsumDense._compute_ebops for GEMM-shaped equations
 * (einsum_dense.py:85-93) evaluated on bit-width tensors, i.e.
 *     ebops = (sum_p sum_k bits_in[p,k] * sum_n bits_ker[k,n] + mean(bits_bias) * bias_size)
 *             * par_factor / n_parallel * ebops_factor
 * evaluated left to right in fp32 with a correctly rounded division, as the reference's
 * `ebops * self.parallelization_factor / self.n_parallel` (dense.py:80) followed by `* self.ebops_factor`
 * (base.py:102) is: a single precomputed factor can land one ulp away, and the cast to uint32 then one count away.
 * The gradients are scaled in the order the chain rule walks those operations back.
 * with bits_in = relu(round(i_in)+round(f_in)) (+k for SAT), bits_ker / bits_bias = round(b) (+k for SAT).
 *
 *   ebops [1] fp32;  ebops_u32 [1] optional: the value cast to uint32 (the `_ebops` variable,
 *   src/hgq/layers/core/base.py:103);  g_f_in [P*K], g_b_ker [K*N], g_b_bias [N]: d ebops / d variable;
 *   beta [1], loss_term [1] optional: loss_term = ebops * beta (the add_loss term, base.py:104);
 *   when beta is given the three gradient outputs are d loss_term / d variable (scaled by beta).
 *   amax_part [n_parts, P*K] optional: when given, the input quantizer's integer bits are first
 *   tracked in place in i_in exactly as hgq_wrap_track_i does in training mode with `decay`
 *   (the reference updates `_i` in the layer call before EBOPs are computed, base.py:94-104);
 *   meant for small P*K*n_parts - the single workgroup walks all slices.
 */
int hgq_dense_ebops(const uint32_t *amax_part, int n_parts, float decay, const float *beta, float *loss_term,
                    const void *k_in, float *i_in, const float *f_in, int64_t P, int K, int N,
                    const void *k_ker, const float *b_ker, const void *k_bias, const float *b_bias,
                    float par_factor, float n_parallel, float ebops_factor, float bias_size, int mode_in, int mode_ker,
                    int mode_bias, float *ebops,
                    uint32_t *ebops_u32, float *g_f_in, float *g_b_ker, float *g_b_bias, void *stream);

/*
 * hgq_dense_ebops for several layers in one launch (one workgroup per item; argument meaning as above).  The estimate of a
 * layer depends on bit-width variables only (src/hgq/layers/core/base.py:100: shapes (1,) + shape[1:]), so the layers of
 * a model can be served together once the forward pass has produced every input quantizer's abs-max slices.
 * Descriptors are read on the host and travel as launch arguments (safe under HIP graph capture).
 * The items of a launch (HGQ_EBOPS_BATCH consecutive items) run concurrently: two of them may share `i_in` only if neither
 * tracks (amax_part NULL in both), else HGQ_ERR_ARG - a quantizer shared by several layers is updated by each layer's
 * call in turn (src/hgq/layers/attn/mha.py:205-210), so such layers go into successive calls.
 */
#define HGQ_EBOPS_BATCH 16
typedef struct {
    const uint32_t *amax_part;
    int n_parts;
    float decay;
    const float *beta;
    float *loss_term;
    const void *k_in;
    float *i_in;
    const float *f_in;
    int64_t P;
    int K, N;
    const void *k_ker;
    const float *b_ker;
    const void *k_bias;
    const float *b_bias;
    float par_factor, n_parallel, ebops_factor, bias_size;
    int mode_in, mode_ker, mode_bias;
    float *ebops;
    uint32_t *ebops_u32;
    float *g_f_in, *g_b_ker, *g_b_bias;
} hgq_dense_ebops_item;
int hgq_dense_ebops_multi(const hgq_dense_ebops_item *items, int count, void *stream);

/*
 * Mean squared error, the regression loss HGQ models are trained with through Keras
 * (`loss='mse'`; the reference has no loss code of its own).  target may be NULL (zeros).
 *   loss [1] = mean((pred - target)^2) over n elements, summed in a fixed order;
 *   workspace: hgq_mse_workspace() floats.
 *   hgq_mse_bwd: dpred = g[0] * 2 (pred - target) / n with the upstream gradient g read on the device.
 * Operands must be 16-byte aligned.
 */
int64_t hgq_mse_workspace(void);
int hgq_mse_fwd(const float *pred, const float *target, float *loss, float *workspace, int64_t n, void *stream);
int hgq_mse_bwd(const float *pred, const float *target, const float *g, float *dpred, int64_t n, void *stream);
/* Loss and, in the same pass over pred / target, the gradient for a unit upstream gradient: dpred = 2 (pred - target) / n
 * (what hgq_mse_bwd gives for g = 1); a caller with another upstream gradient scales it. */
int hgq_mse_fwd_bwd(const float *pred, const float *target, float *loss, float *dpred, float *workspace, int64_t n, void *stream);

/*
 * Mean sparse categorical cross-entropy from logits, forward and gradient in one pass.
 *   logits [rows, C]; labels [rows] int64;  loss [1] = mean_r(-log softmax(logits_r)[label_r]);
 *   dlogits [rows, C] = (softmax - onehot) / rows.
 *   state: four 32-bit words, 8-byte aligned, that are zero when the call starts; the kernel leaves them zero again (the
 *   workgroup that finishes last takes the sum out and clears them), so one allocation zeroed once serves every later
 *   call and no launch clears anything.  The workgroups' sums meet as 64-bit fixed-point integers, so the loss does not
 *   depend on the order in which they arrive: every run and every replay of a recorded step gives the same bits.  Calls
 *   that overlap in time need separate words.  NULL: one workgroup computes the whole sum (slower for many rows).
 *   A workgroup's share of the mean beyond 2^22 in magnitude (or not finite) makes the loss NaN.
 */
int hgq_sparse_ce_fwd_bwd(const float *logits, const int64_t *labels, float *loss, float *dlogits, int64_t rows,
                          int C, uint32_t *state, void *stream);

/*
 * The batch feed of an epoch loop over a data set that lives in device memory (what `model.fit(x, y, batch_size=,
 * shuffle=)` of the reference's users does on the host, reference tests/base.py:313-331): row r of the batch =
 * row order[pos + r] of the source, for the samples (x_row_bytes per row) and the labels (y_row_bytes per row; 0 and NULL
 * pointers: none) alike; pos = the first of the two 64-bit words of `state`, moved on by `batch` when the launch ends, so
 * that a launch recorded in a HIP graph draws batch after batch as the graph is replayed.  The caller writes the
 * permutation (or 0 .. n_rows - 1) into `order` and zeroes `state` when an epoch starts, and launches at most
 * n_rows / batch times per epoch; positions past the end read the last row.  Row sizes are multiples of 4 bytes;
 * `order` and `state` 8-byte aligned.  Launches that share `state` must not overlap in time.
 */
int hgq_gather_batch(const void *x_src, int64_t x_row_bytes, const void *y_src, int64_t y_row_bytes, const int64_t *order, void *state,
                     void *x_dst, void *y_dst, int64_t batch, int64_t n_rows, void *stream);

/*
 * Plain SGD update with the reference's post-update constraint and MonoL1 regulariser folded in.
 * Replaces `optimizer.apply` + Constraint.__call__ (src/hgq/constraints/__init__.py:19-21) +
 * the gradient of MonoL1 (src/hgq/regularizers/__init__.py:13-14) for one variable:
 *     w <- clip(w - lr * (g + l1), lo, hi)          (pass lo = -inf, hi = +inf for no constraint)
 */
int hgq_sgd_update(float *w, const float *g, int64_t n, float lr, float l1, float lo, float hi, void *stream);

/*
 * The same update for many variables in one launch (descriptors are read on the host and travel
 * to the kernel as launch arguments, so the call is safe under HIP graph capture).
 *
 * A variable's gradient may arrive in several pieces: `g` (NULL = none) plus up to HGQ_SGD_SIDES further contributions
 * `side[s]` of the same length, each multiplied by the device scalar `side_scale[s][0]` (NULL = 1):
 *     grad = g + sum_s side_scale[s] * side[s];   w <- clip(w - lr * (grad + l1), lo, hi)
 * In the reference a bit-width variable collects its gradient from its quantizer's backward and from every EBOPs term
 * it enters (src/hgq/layers/core/base.py:100-104), and autograd adds the pieces one launch at a time; here the
 * pieces are added where they are consumed.
 */
#define HGQ_SGD_BATCH 28
#define HGQ_SGD_SIDES 4
typedef struct {
    float *w;
    const float *g;
    int64_t n;
    float l1, lo, hi;
    const float *side[HGQ_SGD_SIDES];
    const float *side_scale[HGQ_SGD_SIDES];
} hgq_sgd_item;
int hgq_sgd_update_multi(const hgq_sgd_item *items, int count, float lr, void *stream);

/*
 * out[0] = ((terms[0][0] + terms[1][0]) + terms[2][0]) + ... : the scalar loss terms of a step (user loss, one
 * `add_loss` term per layer - src/hgq/layers/core/base.py:102-110 - and the variable regularizers) added in list
 * order, as Keras adds them one at a time, in one launch.  `terms` is a HOST array of `count` device pointers
 * (1 <= count <= HGQ_SUM_BATCH); they travel as launch arguments, so the call is safe under HIP graph capture.
 */
#define HGQ_SUM_BATCH 64
int hgq_sum_scalars(const float *const *terms, int count, float *out, void *stream);
/* hgq_sgd_update_multi with hgq_sum_scalars riding along in its (first) launch: a training step's loss terms, which the
 * update does not read, are added up for the caller's report without a launch of their own. */
int hgq_sgd_update_multi_sum(const hgq_sgd_item *items, int count, float lr, const float *const *terms, int n_terms, float *sum_out,
                             void *stream);

/*
 * One training step (forward, mean sparse categorical cross-entropy from logits, backward, SGD)
 * of a stack of QDense layers in two launches (three when the quantized weight image is rebuilt).  It performs, in the same order and with the
 * same arithmetic, what the per-layer entry points above do when the reference's call stack
 * (src/hgq/layers/core/base.py:88-110 around src/hgq/layers/core/dense.py:60-80, then the
 * optimizer and the constraints) is followed layer by layer: input quantizer (KIF, WRAP,
 * training branch, fixed_point_quantizer.py:401-413) with its integer-bit tracking, kernel / bias
 * quantizers (KBI, SAT or SAT_SYM), contraction, bias, activation, EBOPs * beta added to the loss
 * and assigned to `ebops`, MonoL1 gradient, SGD update, clip constraints.
 *
 * Limits: up to HGQ_MLP_MAX_LAYERS layers, widths up to 64, bit-widths shared along the batch
 * axis for inputs and individual per weight.  All variables are updated in place.
 *   x [rows, layers[0].K];  labels [rows] int64 in [0, layers[n-1].N);
 *   loss [1] optional: cross-entropy + sum of ebops * beta + the MonoL1 terms of the trainable bit-widths;
 *   workspace: hgq_mlp_workspace(layers, n_layers, rows) floats.
 */
#define HGQ_MLP_MAX_LAYERS 8
typedef struct {
    int K, N, act;                    /* input width, output width, HGQ_ACT_* */
    int mode_in, mode_ker, mode_bias; /* HGQ_MODE(...) | HGQ_MODE_KBI | HGQ_MODE_K_U8 as applicable */
    float *w, *bias;                  /* kernel [K, N]; bias [N] or NULL */
    const void *k_in;                 /* input quantizer variables, [K] */
    float *i_in, *f_in;
    const void *k_ker;                /* kernel quantizer variables, [K, N] */
    float *b_ker, *i_ker;
    const void *k_bias;               /* bias quantizer variables, [N] (NULL without bias) */
    float *b_bias, *i_bias;
    float decay;                      /* i_decay_speed of the input quantizer */
    const float *beta;                /* the layer's beta variable [1] */
    uint32_t *ebops;                  /* the layer's ebops variable [1] */
    float par_factor, n_parallel, ebops_factor; /* ebops = sum * par_factor / n_parallel * ebops_factor, left to right */
    float bias_size;                  /* number of bias additions: prod(shape[:-1]) * N for shape (1, ..., K) */
    /* MonoL1 coefficient and clip bounds of each trainable bit-width variable (-inf / +inf for none) */
    float f_in_l1, f_in_lo, f_in_hi;
    float b_ker_l1, b_ker_lo, b_ker_hi, i_ker_l1, i_ker_lo, i_ker_hi;
    float b_bias_l1, b_bias_lo, b_bias_hi, i_bias_l1, i_bias_lo, i_bias_hi;
    int train_i_ker, train_i_bias;    /* integer bits of SAT / SAT_SYM quantizers are trainable */
} hgq_mlp_layer;
int64_t hgq_mlp_workspace(const hgq_mlp_layer *layers, int n_layers, int64_t rows);
int hgq_mlp_train_step(const hgq_mlp_layer *layers, int n_layers, const float *x, const int64_t *labels,
                       int64_t rows, float lr, float *loss, float *workspace, void *stream);
/*
 * The same step for a caller that owns the variables between steps.  The update pass leaves the
 * quantized kernels / biases / rounded fractional bits of the UPDATED variables at the start of the
 * workspace (the image the next step's forward reads); with image_current != 0 the step uses it
 * instead of quantizing the variables again.  Pass 0 on the first step, after any change to a
 * variable from outside, and whenever the workspace or the layer descriptors differ from the previous
 * call's.  workspace must be 16-byte aligned.
 */
int hgq_mlp_train_step_cached(const hgq_mlp_layer *layers, int n_layers, const float *x, const int64_t *labels,
                              int64_t rows, float lr, float *loss, float *workspace, int image_current, void *stream);

/*
 * Table-driven softmax, forward.  Replaces QSoftmax.call for the stable form without a mask
 * (src/hgq/layers/softmax.py:119-136) together with the two QUnaryFunctionLUT tables it calls
 * (src/hgq/layers/activation.py:58-61 and the input / output quantizers the layer wrapper applies
 * around them, src/hgq/layers/core/base.py:88-116), i.e. for every row of L contiguous elements
 *     d = max(x) - x;  e = Q_exp_oq(exp(-Q_exp_iq(d) * input_scaler));  s = sum(e);
 *     r = Q_inv_oq(1 / (Q_inv_iq(s) + eps));  y = Q_oq(e * r)
 * which the reference evaluates as about ten full passes over the score tensor
 * (QMultiHeadAttention._compute_attention, src/hgq/layers/attn/mha.py:386-416 builds it with
 * input_scaler = 1 / sqrt(key_dim)).
 *
 * A quantizer is described by its raw variables and mode bits; k == NULL (or a NULL descriptor)
 * means the stage has no quantizer.  The four table quantizers have ONE bit-width entry each
 * (the reference's default, allow_heterogeneous_table = False, softmax.py:59-63); the output
 * quantizer has a [bw_rows, L] table, row r using table row r % bw_rows (bw_rows = 1 for a
 * table shared by all rows).  L <= 256.
 *
 *   x, y [rows, L];
 *   amax_exp_iq [1], amax_inv_iq [1], amax_oq [bw_rows * L]  optional: max |.| of the values the
 *   respective quantizer produced, as uint32 bit patterns (for hgq_wrap_track_i; pass them for
 *   KIF quantizers on their WRAP training branch, where the quantizer output is the rounded value).
 */
typedef struct {
    const void *k;   /* keep-negative variable (fp32, or uint8 with HGQ_MODE_K_U8); NULL = no quantizer */
    const float *i;  /* integer-bits variable */
    const float *fb; /* fractional-bits (KIF) or total-bits (HGQ_MODE_KBI) variable */
    int mode;        /* HGQ_MODE(round, overflow) | HGQ_MODE_* flags */
} hgq_qdesc;
int hgq_qsoftmax_fwd(const float *x, float *y, int64_t rows, int L, int64_t bw_rows, float input_scaler, float eps,
                     const hgq_qdesc *exp_iq, const hgq_qdesc *exp_oq, const hgq_qdesc *inv_iq, const hgq_qdesc *inv_oq,
                     const hgq_qdesc *oq, uint32_t *amax_exp_iq, uint32_t *amax_inv_iq, uint32_t *amax_oq, void *stream);

/*
 * Table-driven softmax, backward (training mode): autograd of the expression above, including
 * the even split of the row maximum's gradient among ties (torch.amax) and the surrogate
 * gradients of the five quantizers.  The forward chain is recomputed from x.
 *
 *   dy, x, dx [rows, L];
 *   g_shared [8]: d loss / d (i, fb) of exp_iq, exp_oq, inv_iq, inv_oq in that order (fb = f or b;
 *                 with HGQ_MODE_KBI the i entry is the total gradient, direct minus via f = b - i);
 *   g_oq_i, g_oq_fb [bw_rows * L]: the same for the output quantizer (either may be NULL);
 *   workspace: hgq_qsoftmax_bwd_workspace(rows, L, bw_rows, has_oq) floats for the per-wavefront
 *   partial sums, which a second kernel adds up in a fixed order (deterministic).
 */
int64_t hgq_qsoftmax_bwd_workspace(int64_t rows, int L, int64_t bw_rows, int has_oq);
int hgq_qsoftmax_bwd(const float *dy, const float *x, float *dx, int64_t rows, int L, int64_t bw_rows, float input_scaler,
                     float eps, const hgq_qdesc *exp_iq, const hgq_qdesc *exp_oq, const hgq_qdesc *inv_iq,
                     const hgq_qdesc *inv_oq, const hgq_qdesc *oq, float *g_shared, float *g_oq_i, float *g_oq_fb,
                     float *workspace, void *stream);

/*
 * QConv2D contraction, forward.  Replaces `self.convolution_op(qinputs, self.qkernel)`, the bias
 * add and the activation of QBaseConv.call (src/hgq/layers/conv.py:72-89; the Keras torch backend
 * transposes to channels-first around a library convolution) with an implicit GEMM that reads the
 * channels-last tensors in place.  With a 1 x 1 geometry (H = W = kh = kw = 1, C = K) it is the
 * dense contraction of any width, `ops.matmul(qinputs, self.qkernel) + self.qbias`
 * (src/hgq/layers/core/dense.py:60-68), used where K or N exceeds the fused dense kernels.
 *
 *   xq [B, H, W, C] quantized input;  qw [kh, kw, C, F] quantized kernel;  qb [F] or NULL;
 *   y [B, OH, OW, F];  output pixel (oy, ox) reads input rows oy * sy - py + ky * dly (columns alike),
 *   positions outside the input contribute zero ('same' padding: py, px = the top / left pad);
 *   workspace: hgq_conv2d_fwd_workspace(g, F) floats (0 for most shapes; a long contraction with few
 *   output tiles is split along k and the slices are added by a second kernel), may be NULL if 0.
 *   A 1 x 1 geometry with at most 16384 rows, a contraction of 1024 or more and at most 16 filters (a classifier behind a
 *   flattened feature map) runs in one launch that does not touch the workspace.
 */
typedef struct {
    int B, H, W, C;   /* input: batch, height, width, channels */
    int kh, kw;       /* kernel height, width */
    int sy, sx;       /* strides */
    int py, px;       /* zero padding before the first row / column */
    int dly, dlx;     /* dilation */
    int OH, OW;       /* output height, width */
} hgq_conv_geom;
int64_t hgq_conv2d_fwd_workspace(const hgq_conv_geom *g, int F);
int hgq_conv2d_fwd(const float *xq, const float *qw, const float *qb, float *y, float *workspace, const hgq_conv_geom *g,
                   int F, int act, void *stream);

/*
 * QConv2D contraction, backward: autograd of the expression above.
 *   dy, y [B, OH, OW, F] (y only for HGQ_ACT_RELU);  dxq [B, H, W, C] gradient w.r.t. the quantized
 *   input (NULL to skip);  dqw [kh, kw, C, F], dqb [F] gradients w.r.t. the quantized kernel / bias
 *   (NULL to skip);  workspace: hgq_conv2d_bwd_workspace(g, F) floats for the per-workgroup partial
 *   sums of the weight gradient, added up in a fixed order by a second kernel.
 */
int64_t hgq_conv2d_bwd_workspace(const hgq_conv_geom *g, int F);
int hgq_conv2d_bwd(const float *dy, const float *y, const float *xq, const float *qw, float *dxq, float *dqw, float *dqb,
                   float *workspace, const hgq_conv_geom *g, int F, int act, void *stream);
/*
 * hgq_conv2d_bwd without the sum over the slices: dxq is written, the kernel / bias gradient stays in `workspace` as
 * hgq_conv2d_bwd_slice_count(g, F) slices of [kh kw C F | F] floats (every slice written whole), for a caller that adds the
 * slices of several layers in one launch (hgq_reduce_slices_multi).  Same reference lines as hgq_conv2d_bwd.
 */
int64_t hgq_conv2d_bwd_slice_count(const hgq_conv_geom *g, int F);
int hgq_conv2d_bwd_slices(const float *dy, const float *y, const float *xq, const float *qw, float *dxq, float *workspace,
                          const hgq_conv_geom *g, int F, int act, void *stream);
/*
 * hgq_conv2d_bwd for a convolution whose output is read by a 2 x 2 maximum pooling of stride 2 without padding and by
 * nothing else (QConv2D followed by MaxPooling2D - the Keras layer the reference's models put behind it, e.g.
 * /root/reference/tests/test_layers/test_pool.py:16-40 for the pooling semantics): `dyp` is the gradient of the POOLED
 * output, [B, OH / 2, OW / 2, F]; the gradient of the convolution's output - dyp where a pixel holds its window's first
 * maximum in row-major order (what hgq_pool2d_bwd does), zero elsewhere and in a trailing odd row / column - is formed
 * while the kernel stages its tiles, so the pooling's own backward pass does not run.  `y` (the convolution's output) is
 * always read.  reduce = 0: the kernel / bias gradient stays in `workspace` as slices (hgq_conv2d_bwd_slices), else it is
 * summed into dqw / dqb.  hgq_conv2d_maxpool_bwd_supported: 1 where the few-input-channel kernel takes the shape with F a
 * multiple of 4 (kernels of odd size; 'valid', or a 'same' padding that keeps the tiles on window boundaries);
 * HGQ_ERR_UNSUPPORTED otherwise, and for dyp / y not aligned to 16 bytes.
 * hgq_conv2d_maxpool_fwd (same shapes): hgq_conv2d_fwd that also writes the pooled output yp [B, OH / 2, OW / 2, F] from
 * the values it has in registers (hgq_pool2d_fwd's result without its pass over y).
 */
int hgq_conv2d_maxpool_bwd_supported(const hgq_conv_geom *g, int F);
int hgq_conv2d_maxpool_fwd(const float *xq, const float *qw, const float *qb, float *y, float *yp, const hgq_conv_geom *g, int F,
                           int act, void *stream);
int hgq_conv2d_maxpool_bwd(const float *dyp, const float *y, const float *xq, const float *qw, float *dxq, float *dqw, float *dqb,
                           float *workspace, const hgq_conv_geom *g, int F, int act, int reduce, void *stream);
/*
 * The same pair with the unpooled output replaced by what the backward pass needs of it: `code`
 * [B, OH / 2, OW / 2, F], one byte per pooling window and filter - bits 0-1 the place (row-major, 0..3) of the window's
 * first maximum, bit 2 set where that maximum is positive.  The forward pass writes yp and code and never writes the
 * unpooled tensor (four times yp's size); the backward pass reads dyp and code.  Results are those of
 * hgq_conv2d_maxpool_fwd / _bwd bit for bit.  code must be 4-byte aligned.  Same shapes and errors otherwise.
 * (No counterpart in the reference, whose Keras layers keep the unpooled tensor: reference src/hgq/layers/conv.py:72-102.)
 */
int hgq_conv2d_maxpool_fwd_coded(const float *xq, const float *qw, const float *qb, float *yp, uint8_t *code,
                                 const hgq_conv_geom *g, int F, int act, void *stream);
int hgq_conv2d_maxpool_bwd_coded(const float *dyp, const uint8_t *code, const float *xq, const float *qw, float *dxq, float *dqw,
                                 float *dqb, float *workspace, const hgq_conv_geom *g, int F, int act, int reduce, void *stream);

/*
 * One quantizer's bit-width view for the EBOPs entry points below: `bits` / `fbits` as hgq_qbits_fwd forms
 * them from the raw variables, broadcast to a tensor of n cells by the rule entry = (cell / inner) % size.
 * g_i / g_fb [size] receive the gradient of the LOSS TERM (ebops * beta, unit upstream gradient) with
 * respect to the variables, through the straight-through rounding of hgq_qbits_bwd (g_i unused for kbi).
 */
typedef struct hgq_bits_desc {
    const uint8_t *k; /* uint8 keep-negative flags; may be NULL when add_mode == 0 */
    const float *i;   /* NULL for the (k, b, i) kind */
    const float *fb;
    int64_t size, inner;
    int kbi, add_mode;
    float *g_i, *g_fb;
} hgq_bits_desc;

/*
 * EBOPs of layers whose estimate is algebra on bit-width tensors, one launch each: value * factors ->
 * uint32 variable (may be NULL), loss_term[0] = ebops * beta, gradients into the descriptors.
 *   hgq_lut_ebops      QUnaryFunctionLUT._compute_ebops (src/hgq/layers/activation.py:101-104):
 *                      sum over n_cells of 2**bits_in * bits_out, times `scale` (1e-4), times ebops_factor.
 *   hgq_softmax_ebops  QSoftmax._compute_ebops, stable form (src/hgq/layers/softmax.py:177-206) for a softmax over
 *                      the last axis of [rows, L]: sum(bits_sub) + sum(bits_exp) - sum_rows min_l bits_exp +
 *                      sum(bits_exp * bits_inv[row]), times instance_factor, times ebops_factor; bits_inv is
 *                      laid out over the rows; bits_sub may be NULL.  rows <= 2048.
 *   hgq_mha_ebops      QMultiHeadAttention._compute_ebops (src/hgq/layers/attn/mha.py:507-524) for rank-3 inputs:
 *                      sum bits_q[t,n,h] bits_k[s,n,h] + sum bits_attn[n,t,s] bits_v[s,n,h]; cells of q / k / v in
 *                      [seq, N, H] order, of attn in [N, T, S] order.  N * H <= 1024, N * S <= 2048.
 *   hgq_sum_ebops      the pooling layers' QBasePooling._compute_ebops (src/hgq/layers/pooling.py:28-30): sum over
 *                      n_cells of bits_in, times parallel_factor, divided by n_parallel (a product, then a correctly
 *                      rounded division; no division when n_parallel is 1), times ebops_factor.
 * Every sum is formed in a fixed order; values are exact while they stay below 2**53.  The operands' entries are
 * staged in LDS: at most 30720 over all operands of a call (HGQ_ERR_UNSUPPORTED beyond, as for the other limits).
 */
int hgq_sum_ebops(const hgq_bits_desc *bits_in, int64_t n_cells, float parallel_factor, float n_parallel, float ebops_factor,
                  const float *beta, uint32_t *ebops_u32, float *loss_term, void *stream);
int hgq_lut_ebops(const hgq_bits_desc *bits_in, const hgq_bits_desc *bits_out, int64_t n_cells, float scale, float ebops_factor,
                  const float *beta, uint32_t *ebops_u32, float *loss_term, void *stream);
int hgq_softmax_ebops(const hgq_bits_desc *bits_sub, const hgq_bits_desc *bits_exp, const hgq_bits_desc *bits_inv, int64_t rows, int L,
                      float instance_factor, float ebops_factor, const float *beta, uint32_t *ebops_u32, float *loss_term, void *stream);
int hgq_mha_ebops(const hgq_bits_desc *bits_q, const hgq_bits_desc *bits_k, const hgq_bits_desc *bits_v, const hgq_bits_desc *bits_attn, int T,
                  int S, int N, int H, int Hv, float parallel_factor, float ebops_factor, const float *beta, uint32_t *ebops_u32,
                  float *loss_term, void *stream);

/*
 * The whole QBaseConv._compute_ebops (src/hgq/layers/conv.py:91-102) and the scalar tail of the call wrapper
 * (src/hgq/layers/core/base.py:101-104) from the quantizers' raw variables, in one launch:
 *     ebops = (sum(conv(bits_in, bits_ker)) * conv_scale + mean(bits_bias) * bias_size) * ebops_factor
 * by the closed form of hgq_conv2d_ebops; uint32 variable (may be NULL), loss_term[0] = ebops * beta, gradients of the
 * loss term into the descriptors.  Every operand needs one bit-width entry per cell (size = cells, inner = 1):
 * bits_in over [H, W, C], bits_ker over [kh, kw, C, F], bits_bias (may be NULL) over [F]; limits as hgq_conv2d_ebops.
 */
int hgq_conv2d_ebops_q(const hgq_bits_desc *bits_in, const hgq_bits_desc *bits_ker, const hgq_bits_desc *bits_bias,
                       const hgq_conv_geom *g, int F, float conv_scale, float bias_size, float ebops_factor, const float *beta,
                       uint32_t *ebops_u32, float *loss_term, void *stream);

/*
 * The scalar tail of QLayerBase.call (src/hgq/layers/core/base.py:101-104):
 *     ebops = ebops * ebops_factor;  self._ebops.assign(cast(ebops, uint32));  loss term = ebops * beta
 * forward writes the uint32 variable (may be NULL) and out [1]; backward: d_ebops = (g * beta) * factor.
 */
int hgq_ebops_finish_fwd(const float *ebops, float factor, const float *beta, uint32_t *ebops_u32, float *out, void *stream);
int hgq_ebops_finish_bwd(const float *g, const float *beta, float factor, float *d_ebops, void *stream);

/*
 * Bit-widths of a quantizer from its raw variables: the `b`, `bits` and `fbits` properties of
 * FixedPointQuantizerKIF / KBI (src/hgq/quantizer/internal/fixed_point_quantizer.py:60-79,
 * :206-215, :311-320) in one launch, with the straight-through gradient of round_conv.
 *   KIF (kbi = 0): b = relu(rint(i) + rint(fb));   KBI (kbi = 1): b = rint(fb) (i unused)
 *   add_mode 0: b;  1: b + k;  2: b + k * (b > 0).   k is the uint8 keep-negative variable.
 *   backward: KIF di = dfb = g * [rint(i) + rint(fb) > 0];  KBI dfb = g (di untouched).
 */
int hgq_qbits_fwd(const uint8_t *k, const float *i, const float *fb, int64_t n, int kbi, int add_mode, float *out, void *stream);
int hgq_qbits_bwd(const float *g, const float *i, const float *fb, int64_t n, int kbi, float *di, float *dfb, void *stream);

/*
 * Batch-norm folding of QEinsumDenseBatchnorm.get_fused_qkernel_and_qbias
 * (src/hgq/layers/einsum_dense_batchnorm.py:160-172) for a [K, N] kernel normalised over its N
 * outputs, before the kernel / bias quantizers:
 *     var = second - mean^2 if is_meansq else second;   scaler = gamma / sqrt(var + eps)   (gamma NULL = 1)
 *     fused_w[k, n] = w[k, n] * scaler[n];   fused_b[n] = bias[n] - mean[n] * scaler[n]
 * With moving_mean / moving_var (each may be NULL) the forward also applies the momentum update of
 * QEinsumDenseBatchnorm.call (:113-117): m <- m * momentum + batch * one_minus_momentum.
 * The backward returns the gradients w.r.t. w, bias, gamma, mean and `second` (any of dbias, dgamma,
 * dmean, dsecond may be NULL).
 */
int hgq_bn_fold_fwd(const float *w, const float *bias, const float *gamma, const float *mean, const float *second, int is_meansq,
                    float eps, float *fused_w, float *fused_b, float *moving_mean, float *moving_var, float momentum,
                    float one_minus_momentum, int K, int N, void *stream);
int hgq_bn_fold_bwd(const float *w, const float *gamma, const float *mean, const float *second, int is_meansq, float eps,
                    const float *d_fw, const float *d_fb, float *dw, float *dbias, float *dgamma, float *dmean, float *dsecond,
                    int K, int N, void *stream);
/*
 * The folding with the kernel and bias quantizers behind it in the same launch each way (reference
 * src/hgq/layers/einsum_dense_batchnorm.py:158-211, get_fused_qkernel_and_qbias: fold, then `self.kq(...)`, `self.bq(...)`).
 * qk / qb: training-mode quantizers with per-element bit-widths ([K, N] and [N]) and no trackers (SAT / SAT_SYM).
 * Forward: qw = q_k(w s), qbias = q_b(bias - mean s), moving statistics updated as by hgq_bn_fold_fwd.  Backward: d_qw /
 * d_qb are the gradients at the quantized values; each passes its quantizer's surrogate gradient (bit-width parts to
 * di_k / dfb_k [K, N] and di_b / dfb_b [N], the folded values formed again from w, bias and the statistics), then the
 * folding's own gradient as in hgq_bn_fold_bwd.  Values and gradients equal the two separate launches'.
 */
int hgq_bn_fold_quant_fwd(const float *w, const float *bias, const float *gamma, const float *mean, const float *second, int is_meansq,
                          float eps, const hgq_qdesc *qk, const hgq_qdesc *qb, float *qw, float *qbias, float *moving_mean,
                          float *moving_var, float momentum, float one_minus_momentum, int K, int N, void *stream);
int hgq_bn_fold_quant_bwd(const float *w, const float *bias, const float *gamma, const float *mean, const float *second, int is_meansq,
                          float eps, const hgq_qdesc *qk, const hgq_qdesc *qb, const float *d_qw, const float *d_qb, float *dw,
                          float *dbias, float *dgamma, float *dmean, float *dsecond, float *di_k, float *dfb_k, float *di_b,
                          float *dfb_b, int K, int N, void *stream);

/*
 * Batch statistics of the un-quantized pre-activation z = x W of QEinsumDenseBatchnorm.call
 * (src/hgq/layers/einsum_dense_batchnorm.py:99-124) WITHOUT materialising z: the contraction and the
 * column sums run in one pass over x.
 *   x [rows, K];  w [K, N] (the un-quantized kernel);  mean, meansq [N] = mean_r z, mean_r z^2;
 *   backward: with dz[r, c] = (dmean[c] + 2 z[r, c] dmeansq[c]) / rows,  dx = dz W^T,  dw = x^T dz - evaluated without z
 *   on the default matrix instruction:  dx = x A + v,  A = (2 / rows) W diag(dmeansq) W^T,  v = W dmean / rows;
 *   dw = (m dmean^T + 2 (S W) diag(dmeansq)) / rows  with  S = x^T x  and m the column sums of x.
 *   workspace: hgq_dense_moments_workspace(rows, K, N) floats (per-workgroup slices, fixed-order sum).
 * K, N <= 64 and multiples of 4; x (and dx) 16-byte aligned; otherwise HGQ_ERR_UNSUPPORTED and the
 * caller uses hgq_qdense_fwd + hgq_col_moments_fwd.
 */
int64_t hgq_dense_moments_workspace(int64_t rows, int K, int N);
int hgq_dense_moments_fwd(const float *x, const float *w, float *mean, float *meansq, float *workspace, int64_t rows, int K,
                          int N, void *stream);
int hgq_dense_moments_bwd(const float *x, const float *w, const float *dmean, const float *dmeansq, float *dx, float *dw,
                          float *workspace, int64_t rows, int K, int N, void *stream);

/*
 * The same with the layer's input quantizer applied while x is staged (QEinsumDenseBatchnorm.call quantizes its
 * input once, :101-102, and contracts it twice): x is the RAW input, f_in the raw fractional-bit variable of a
 * training-mode WRAP (k, i, f) quantizer laid out as a [bw_rows, K] table (row r of x uses table row r % bw_rows,
 * bw_rows divides 64), mode its HGQ_MODE(...) bits.  The quantized input is never written; the backward returns dx
 * with respect to the raw input (straight-through) and df_in [bw_rows * K], this contraction's share of the
 * fractional-bit gradient.  bw_rows == 0: no quantizer (the entry points above).
 * dx_add (may be null): [rows, K], 16-byte aligned, added to dx while it is written - the gradient x receives from its
 * other use, the output contraction, so that the two need no separate accumulation pass; it does not enter df_in.
 * dw == NULL in the backward: the kernel / fractional-bit gradient is left in `workspace` as hgq_qdense_bwd_workspace(rows,
 * K, N, bw_rows) / (K N + N + bw_rows K) slices of [K N | N (unused) | bw_rows K] floats for the caller's own reduction
 * (hgq_reduce_slices_multi).
 */
int64_t hgq_qdense_moments_workspace(int64_t rows, int K, int N, int64_t bw_rows);
int hgq_qdense_moments_fwd(const float *x, const float *f_in, int64_t bw_rows, int mode, const float *w, float *mean, float *meansq,
                           float *workspace, int64_t rows, int K, int N, void *stream);
int hgq_qdense_moments_bwd(const float *x, const float *f_in, int64_t bw_rows, int mode, const float *w, const float *dmean,
                           const float *dmeansq, const float *dx_add, float *dx, float *dw, float *df_in, float *workspace,
                           int64_t rows, int K, int N, void *stream);

/*
 * Per-column mean and mean of squares of a [rows, N] matrix, and the gradient of both.  Replaces
 * `ops.mean(x, axis)` / `ops.mean(ops.square(x), axis)` and their autograd in
 * QEinsumDenseBatchnorm.call (src/hgq/layers/einsum_dense_batchnorm.py:99-124, the batch
 * statistics of the un-quantized pre-activation) when the normalised axes are the trailing ones.
 *   mean, meansq [N];  workspace: hgq_col_moments_workspace(rows, N) floats (partial sums per
 *   workgroup, added in a fixed order);  dx[r, c] = (dmean[c] + 2 x[r, c] dmeansq[c]) / rows.
 */
int64_t hgq_col_moments_workspace(int64_t rows, int N);
int hgq_col_moments_fwd(const float *x, int64_t rows, int N, float *mean, float *meansq, float *workspace, void *stream);
int hgq_col_moments_bwd(const float *x, const float *dmean, const float *dmeansq, int64_t rows, int N, float *dx,
                        void *stream);

/*
 * The two score contractions of QMultiHeadAttention._compute_attention for rank-3 inputs
 * (src/hgq/layers/attn/mha.py:418-470; einsum strings built by Keras, imported at mha.py:10):
 *     scores[b, n, t, s] = sum_h query[b, t, n, h] * key[b, s, n, h]        'aecd,abcd->acbe'
 *     out[b, t, n, h]    = sum_s probs[b, n, t, s] * value[b, s, n, h]      'acbe,aecd->abcd'
 * and their autograd, reading the projections in their own [B, seq, N, H] layout (the reference
 * path permutes and copies around a batched library GEMM).  T, S, H <= 64.
 *   query / dquery [B, T, N, H];  key, value / dkey, dvalue [B, S, N, H];  scores, probs and their
 *   gradients [B, N, T, S];  out / dout [B, T, N, H].  Gradient outputs may be NULL to skip.
 */
int hgq_attn_scores_fwd(const float *query, const float *key, float *scores, int B, int T, int S, int N, int H, void *stream);
int hgq_attn_scores_bwd(const float *dscores, const float *query, const float *key, float *dquery, float *dkey, int B, int T,
                        int S, int N, int H, void *stream);
int hgq_attn_combine_fwd(const float *probs, const float *value, float *out, int B, int T, int S, int N, int H, void *stream);
int hgq_attn_combine_bwd(const float *dout, const float *probs, const float *value, float *dprobs, float *dvalue, int B, int T,
                         int S, int N, int H, void *stream);

/*
 * The attention core of QMultiHeadAttention._compute_attention (src/hgq/layers/attn/mha.py:418-470) with
 * the table softmax of QSoftmax.call (src/hgq/layers/softmax.py:121-141) in one pass each way:
 *     out = combine(qsoftmax(scores(query, key)), value)
 * scores and probabilities are never written: the backward pass recomputes them from query / key /
 * value.  Quantizer descriptors, trackers, g_shared / g_oq_i / g_oq_fb and bw_rows (rows of the output
 * quantizer's [bw_rows, S] table; row (n * T + t) % bw_rows serves head n, query position t; must
 * divide N * T) are those of hgq_qsoftmax_fwd / _bwd.  Supported: T = S = 32 or 64, H = 8, 16 or 32
 * (query / key and value alike), N * T / 32 <= 8, N * H <= 64, an output quantizer that does not
 * saturate and is not of the (k, b, i) kind in the backward pass; anything else returns
 * HGQ_ERR_UNSUPPORTED (the workspace queries return -1) and the caller composes hgq_attn_scores_*,
 * hgq_qsoftmax_* and hgq_attn_combine_*.  Operands and workspaces 16-byte aligned.  The forward
 * workspace (needed with amax_oq only) holds one abs-max slice per workgroup: entries are combined by a
 * second launch, not by atomics.
 * Masks (QSoftmax.call with `mask`, src/hgq/layers/softmax.py:118-127; `use_causal_mask` and `attention_mask` of
 * QMultiHeadAttention.call, src/hgq/layers/attn/mha.py:439-461): `mask` (may be NULL) is a boolean mask
 * [mask_batch, T, S], one byte per entry, 0 = masked out, shared by all heads, mask_batch = 1 or B, 4-byte aligned;
 * `causal` != 0 masks key positions beyond the query position as well.  A masked score becomes -1e9 ahead of the row
 * maximum and its exp is multiplied by zero behind the table, as the reference does; it takes no gradient.
 */
int hgq_qattention_fwd(const float *query, const float *key, const float *value, float *out, int B, int T, int S, int N, int H,
                       int64_t bw_rows, float input_scaler, float eps, const hgq_qdesc *exp_iq, const hgq_qdesc *exp_oq,
                       const hgq_qdesc *inv_iq, const hgq_qdesc *inv_oq, const hgq_qdesc *oq, uint32_t *amax_exp_iq,
                       uint32_t *amax_inv_iq, uint32_t *amax_oq, void *workspace, const uint8_t *mask, int mask_batch, int causal,
                       void *stream);
int64_t hgq_qattention_fwd_workspace(int B, int T, int S, int N, int H, int64_t bw_rows, int track_oq); /* 4-byte words */
int64_t hgq_qattention_bwd_workspace(int B, int T, int S, int N, int H, int64_t bw_rows, int has_oq);
int hgq_qattention_bwd(const float *dout, const float *query, const float *key, const float *value, float *dquery, float *dkey,
                       float *dvalue, int B, int T, int S, int N, int H, int64_t bw_rows, float input_scaler, float eps,
                       const hgq_qdesc *exp_iq, const hgq_qdesc *exp_oq, const hgq_qdesc *inv_iq, const hgq_qdesc *inv_oq,
                       const hgq_qdesc *oq, float *g_shared, float *g_oq_i, float *g_oq_fb, float *workspace, const uint8_t *mask,
                       int mask_batch, int causal, void *stream);

/*
 * Grouped dense contraction: one small kernel matrix per group g (an axis that input, kernel and output share), the
 * form of QEinsumDense equations such as 'Babc,bcd->Babd' (reference tests/test_dense.py:56; the einsum and its
 * autograd of src/hgq/layers/core/einsum_dense.py:72-93 on already quantized operands):
 *     y[r, g, n] = act(sum_k x[r, g, k] * w[g, k, n] + bias[g, n])
 *   x [R, G, K], w [G, K, N], bias [G, N] or NULL, y / dy [R, G, N]; K, N <= 64 (hgq_gdense_supported), act HGQ_ACT_*.
 *   Backward: dx [R, G, K] (NULL to skip), dw [G, K, N], dbias [G, N] or NULL; y is read for the relu mask only;
 *   workspace: hgq_gdense_bwd_workspace floats (per-workgroup slices, added in a fixed order).
 */
int hgq_gdense_supported(int64_t R, int G, int K, int N);
int hgq_gdense_fwd(const float *x, const float *w, const float *bias, float *y, int64_t R, int G, int K, int N, int act, void *stream);
int64_t hgq_gdense_bwd_workspace(int64_t R, int G, int K, int N, int has_bias);
int hgq_gdense_bwd(const float *dy, const float *y, const float *x, const float *w, float *dx, float *dw, float *dbias, float *workspace,
                   int64_t R, int G, int K, int N, int act, void *stream);

/*
 * Per-channel affine map of QBatchNormalization.call (src/hgq/layers/batch_normalization.py:184,
 * `inputs * qscale + qoffset`, a multiplication and then an addition) over the trailing axis, and its gradients:
 *     y[r, c] = x[r, c] * scale[c] + offset[c];  dx = g * scale;  dscale[c] = sum_r g x;  doffset[c] = sum_r g
 *   C a positive multiple of 4, operands 16-byte aligned; dx / dscale / doffset may be NULL; workspace:
 *   hgq_affine_rows_bwd_workspace floats (slices of the two sums, added in a fixed order).
 */
int hgq_affine_rows_fwd(const float *x, const float *scale, const float *offset, float *y, int64_t rows, int C, void *stream);
int64_t hgq_affine_rows_bwd_workspace(int64_t rows, int C);
int hgq_affine_rows_bwd(const float *g, const float *x, const float *scale, float *dx, float *dscale, float *doffset, float *workspace,
                        int64_t rows, int C, void *stream);

/*
 * The arithmetic Quantizer.call puts around its internal quantizer (src/hgq/quantizer/quantizer.py:49-60), every step one
 * IEEE fp32 operation in the reference's order:
 *   hgq_quantizer_scale_div:  y = x / scaler                                   (`inputs = inputs / self.scaler`, :50-51)
 *   hgq_quantizer_tail_fwd:   o = q; o = o * scaler (has_scaler);  o = xs + noise * (o - xs) (has_noise: the
 *                             quantization-noise blend of training calls, xs = the quantizer's input);  o = o * a0 + a1
 *                             (has_affine)                                      (:54-59) - one pass for whichever are set
 *   hgq_quantizer_tail_bwd:   the gradients of (q, xs) for the upstream gradient g, formed as reverse-mode differentiation
 *                             of that chain forms them: g' = g * a0; dxs = g' - g' * noise, g'' = g' * noise; dq = g'' * scaler.
 *                             dxs is written only with has_noise (it may be NULL otherwise).
 * Any n, any alignment (128-bit accesses when every array is 16-byte aligned).
 */
int hgq_quantizer_scale_div(const float *x, float *y, int64_t n, float scaler, void *stream);
int hgq_quantizer_tail_fwd(const float *q, const float *xs, float *out, int64_t n, int has_scaler, float scaler, int has_noise,
                           float noise, int has_affine, float a0, float a1, void *stream);
int hgq_quantizer_tail_bwd(const float *g, float *dq, float *dxs, int64_t n, int has_scaler, float scaler, int has_noise, float noise,
                           int has_affine, float a0, void *stream);

/*
 * 2-D max / average pooling on channels-last tensors, forward and backward.  Replaces the Keras
 * MaxPooling2D / AveragePooling2D `call` that QMaxPooling2D / QAveragePooling2D apply to the
 * quantized input (src/hgq/layers/pooling.py:23-47; the Keras torch backend transposes to
 * channels-first around the library pooling) and its autograd.
 *   geom = {B, H, W, C, pool_h, pool_w, stride_y, stride_x, pad_top, pad_left, OH, OW};
 *   x, dx [B, H, W, C];  y, dy [B, OH, OW, C].  Max pooling sends the gradient to the first maximum
 *   of a window in row-major order; average pooling divides by the number of in-range elements.
 */
int hgq_pool2d_fwd(const float *x, float *y, const int *geom, int is_max, void *stream);
int hgq_pool2d_bwd(const float *dy, const float *x, float *dx, const int *geom, int is_max, void *stream);

/*
 * Mean over the middle axis: y[b, n] = mean_p x[b, p, n] and its gradient dx[b, p, n] = dy[b, n] / P.  Replaces
 * `ops.mean(x, axis)` of the global average pooling layers on channels-last tensors
 * (src/hgq/layers/pooling.py:23-47 wrap keras.layers.GlobalAveragePooling1D / 2D; the spatial axes are the middle
 * ones and collapse into P) and the mean over the particles of the per-particle configuration.  A row's partial sums
 * are added in a fixed order.  One batch element (P * N floats) must be smaller than 2 GiB.
 */
int hgq_mean_mid_fwd(const float *x, float *y, int64_t B, int64_t P, int64_t N, void *stream);
int hgq_mean_mid_bwd(const float *dy, float *dx, int64_t B, int64_t P, int64_t N, void *stream);

/*
 * EBOPs of a convolution and their gradient.  Replaces `ops.sum(self.convolution_op(bw_inp, bw_ker))`
 * of QBaseConv._compute_ebops (src/hgq/layers/conv.py:91-102), evaluated on the bit-width tensors of
 * one sample, by its closed form (no convolution is run): every kernel tap visits a rectangle of
 * input pixels, so the sum factorises per (tap, channel).
 *   bits_in [H, W, C];  bits_ker [kh, kw, C, F];  total [1];  g_bits_in [H, W, C], g_bits_ker
 *   [kh, kw, C, F] = d total / d bits (either may be NULL).  g->B is ignored.  Needs kh * kw * C <= 4096,
 *   kh * W * C <= 8192, H * kh <= 2048, W * kw <= 2048, kh * kw * C * F < 2**21 and H * W * C < 2**21
 *   (HGQ_ERR_UNSUPPORTED otherwise).
 */
int hgq_conv2d_ebops(const float *bits_in, const float *bits_ker, const hgq_conv_geom *g, int F, float *total,
                     float *g_bits_in, float *g_bits_ker, void *stream);

/* Fill kernel (graph-capture safe replacement for a memset). */
int hgq_fill_u32(uint32_t *p, uint32_t value, int64_t n, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* HGQ_HIP_H */
