/*
 * odl_fp8.h - C ABI of the MI355X (gfx950) FP8 Linear kernels.
 *
 * This is the native boundary under the FP8 AMP Linear path of Optimus-DL.  In
 * the reference that boundary is the call into a third-party CUDA library:
 *   optimus_dl/modules/model_transforms/transformer_engine.py:97-108
 *       (TELinear builds and calls te.pytorch.Linear: amax, cast, cast+transpose,
 *        FP8 GEMM for fwd / dgrad / wgrad)
 *   optimus_dl/modules/amp/fp8.py:279-306,337-340,357-360
 *       (recipe objects and the autocast contexts whose exit refreshes the scales)
 * Each entry point below names the step of that call it stands in for.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless the comment says "host";
 *   - matrices are dense row-major; `rows`/`cols` are in elements;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream);
 *     nothing here synchronises with the host or allocates memory;
 *   - return value 0 = launched; non-zero = refused, nothing was launched, and
 *     odl_fp8_last_error() (host string, thread-local) says why;
 *   - 8-bit codes are OCP FP8: E4M3 ("fn": no Inf, 0x7F/0xFF = NaN, max 448) and
 *     E5M2 (max 57344).  Conversion is round-to-nearest-even after an explicit
 *     clamp to +-max; NaN inputs give 0x7F with the input's sign bit.
 */
#ifndef ODL_FP8_H
#define ODL_FP8_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *odl_stream_t;

enum odl_fp8_format { ODL_FP8_E4M3 = 0, ODL_FP8_E5M2 = 1 };
enum odl_scale_mode { ODL_SCALE_TENSOR = 0, ODL_SCALE_ROW = 1, ODL_SCALE_COL = 2 };
enum odl_dtype { ODL_BF16 = 0, ODL_F32 = 1 };
enum odl_amax_algo { ODL_AMAX_MAX = 0, ODL_AMAX_MOST_RECENT = 1 };

enum odl_status {
    ODL_OK = 0,
    ODL_ERR_ARG = 1,      /* bad enum / null pointer / negative size */
    ODL_ERR_SHAPE = 2,    /* shape or alignment the kernels do not support */
    ODL_ERR_LAUNCH = 3    /* HIP reported an error at launch */
};

/* ABI version of this header (15); bumped when a signature changes or an entry point is added. */
int odl_fp8_abi_version(void);

/*
 * Per-device set-up, for the device that is current on the calling thread: looks up the addresses of the two small
 * objects in the library's device image (the partial maxima of odl_fp8_cast_dynamic_noalloc, the unit scale of the
 * block-scaled GEMMs; hipGetSymbolAddress) and the device's compute-unit count.  Every entry point that needs them
 * makes the same lookups on its first call on a device, so this call is optional -- except for callers that will
 * make such a first call under HIP stream capture, where the lookup is not allowed: they call this once per device
 * beforehand.  No counterpart in the reference (its backend initialises itself on import).  Idempotent, launches nothing.
 */
int odl_fp8_init_device(void);

/* Last error message of the calling host thread ("" if none). */
const char *odl_fp8_last_error(void);

/*
 * amax = max |x| of a [rows, cols] matrix, as fp32.
 *   mode TENSOR -> amax_out[1], ROW -> amax_out[rows], COL -> amax_out[cols]
 *   accumulate != 0: amax_out = max(amax_out, amax(x)) (used to fold several
 *   tensors, or microbatches, into one history slot); otherwise overwritten.
 * NaN in x yields NaN.  Stands in for the amax reduction inside the
 * quantisation step of te.pytorch.Linear (transformer_engine.py:106).
 */
int odl_fp8_amax(const void *x, int src_dtype, int64_t rows, int64_t cols, int mode,
                 float *amax_out, int accumulate, odl_stream_t stream);

/*
 * scale[i]     = fp8_max(fmt) / amax[i] / 2^margin   (IEEE fp32 division)
 * scale_inv[i] = 1 / scale[i]
 * amax[i] that is 0, negative, NaN or Inf gives scale 1; an infinite quotient
 * gives FLT_MAX.  This is the "current scaling" rule (recipe "tensorwise",
 * fp8.py:289-294) applied to n independent amaxes.
 */
int odl_fp8_scale_from_amax(const float *amax, int64_t n, int fmt, int margin,
                            float *scale, float *scale_inv, odl_stream_t stream);

/*
 * Per-tensor amax and the scale derived from it in ONE launch: what the recipe
 * "tensorwise" (current scaling, fp8.py:289-294) does to every tensor before its cast.
 * Results are those of odl_fp8_amax(mode TENSOR, accumulate 0) followed by
 * odl_fp8_scale_from_amax(n = 1).  scale_inv may be NULL.
 * workspace: two 32-bit words of device memory that are zero before the first
 * call; the kernel leaves them zero, so one workspace serves every call that is
 * ordered on the same stream.  Calls that may overlap need a workspace each.
 */
int odl_fp8_amax_scale(const void *x, int src_dtype, int64_t rows, int64_t cols, int fmt, int margin,
                       float *amax_out, float *scale, float *scale_inv, uint32_t *workspace,
                       odl_stream_t stream);

/*
 * Current scaling ("tensorwise", fp8.py:289-294) of one tensor in two launches and no other:
 *   odl_fp8_amax_parts  : ODL_FP8_AMAX_PARTS partial maxima of |x| (unused entries 0),
 *                         written without atomics;
 *   odl_fp8_cast_dynamic: every block reduces the partials, derives
 *                         scale = fp8_max(fmt) / amax / 2^margin (rules of odl_fp8_scale_from_amax)
 *                         and casts; out (row-major codes) and out_t (transposed codes) may
 *                         each be NULL, not both; dyn_out[3] receives {amax, scale, 1/scale}.
 * The codes and the three numbers equal those of odl_fp8_amax + odl_fp8_scale_from_amax +
 * odl_fp8_cast / odl_fp8_cast_transpose, bit for bit.
 */
#define ODL_FP8_AMAX_PARTS 512
int odl_fp8_amax_parts(const void *x, int src_dtype, int64_t rows, int64_t cols, float *parts,
                       odl_stream_t stream);
int odl_fp8_cast_dynamic(const void *x, int src_dtype, int64_t rows, int64_t cols, const float *parts,
                         int fmt, int margin, uint8_t *out, uint8_t *out_t, float *dyn_out,
                         odl_stream_t stream);

/*
 * MANY tensors per launch: every weight of a model after an optimizer step (what te.pytorch.Linear does per
 * weight and forward, transformer_engine.py:106; `fp8.param`, optim/config.py:36-37, asks for weights that are kept
 * quantised between steps).  Results per tensor are those of the single-tensor calls, bit for bit.
 *   odl_fp8_mt_tensor : one tensor; the table of n of them is read by the kernels from DEVICE memory.
 *   odl_fp8_multi_plan: host only.  Checks a HOST copy of the table (rows a positive multiple of 16, cols of 8;
 *                       x, out_t, parts 16-byte aligned, out 8-byte, no NULL; `scale` non-NULL for the delayed phase)
 *                       and writes the work list of a phase, pairs {tensor, local index} of int32, into `work` (host
 *                       memory, room for `capacity` pairs; NULL or too small: only counts).  Returns the number of
 *                       pairs, -1 on error.  Tables and work lists depend on addresses and shapes only: build them
 *                       once, copy them to the device.
 *   current scaling (recipe "tensorwise"), two launches:
 *     odl_fp8_multi_amax_parts  (phase ODL_MT_AMAX): parts of every tensor <- its partial maxima;
 *     odl_fp8_multi_cast_dynamic (phase ODL_MT_CAST): codes, transposed codes and dyn_out = {amax, scale, 1/scale}
 *                       of every tensor as odl_fp8_amax_parts + odl_fp8_cast_dynamic give them; one format and
 *                       margin for all.
 *   delayed scaling (recipe "delayed"), one launch:
 *     odl_fp8_multi_cast_delayed (phase ODL_MT_CAST_DELAYED): codes and transposed codes with the scale in force
 *                       (*scale), block maxima folded into parts (accumulated, as odl_fp8_cast_delayed does),
 *                       dyn_out[1] = scale, dyn_out[2] = 1/scale.
 * Nothing is allocated; the device tables are not validated again at launch.
 */
typedef struct odl_fp8_mt_tensor {
    const void *x;      /* source [rows, cols], src_dtype */
    uint8_t *out;       /* codes [rows, cols] */
    uint8_t *out_t;     /* codes [cols, rows] */
    float *parts;       /* ODL_FP8_AMAX_PARTS floats */
    float *dyn_out;     /* 3 floats */
    const float *scale; /* delayed scaling: 1 float, the scale in force; NULL for current scaling */
    int64_t rows, cols;
    int32_t src_dtype;  /* odl_dtype */
    int32_t reserved;   /* 0 */
} odl_fp8_mt_tensor;    /* 72 bytes */
enum odl_mt_phase { ODL_MT_AMAX = 0, ODL_MT_CAST = 1, ODL_MT_CAST_DELAYED = 2 };
int64_t odl_fp8_multi_plan(const odl_fp8_mt_tensor *tensors_host, int64_t n, int phase, int32_t *work_host, int64_t capacity);
int odl_fp8_multi_amax_parts(const odl_fp8_mt_tensor *tensors_dev, const int32_t *work_dev, int64_t n_work, odl_stream_t stream);
int odl_fp8_multi_cast_dynamic(const odl_fp8_mt_tensor *tensors_dev, const int32_t *work_dev, int64_t n_work, int fmt, int margin,
                               odl_stream_t stream);
int odl_fp8_multi_cast_delayed(const odl_fp8_mt_tensor *tensors_dev, const int32_t *work_dev, int64_t n_work, int fmt,
                               odl_stream_t stream);

/*
 * odl_fp8_amax_parts + odl_fp8_cast_dynamic in one call that ALLOCATES NOTHING and takes no workspace:
 * the partial maxima go through a 2 KB array that is part of the library's device image (one copy per
 * GPU, held until the process ends).  It has no counterpart in the reference; it is for callers that
 * cannot allocate device memory or carry a workspace around: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  out, out_t, dyn_out and the results are those of
 * odl_fp8_cast_dynamic, bit for bit.  rows * cols above ODL_FP8_NOALLOC_MAX_ELEMS is refused with
 * ODL_ERR_SHAPE (use the two calls above with a buffer of your own).
 * Every call on a GPU uses that GPU's one array: calls that may overlap on the same GPU (different
 * streams, or different host threads without ordering between their streams) race on it and must be
 * ordered by the caller; calls on one stream are safe.  The first call on a device looks up the array's
 * address (hipGetSymbolAddress): make it, or odl_fp8_init_device, once outside of graph capture.
 */
#define ODL_FP8_NOALLOC_MAX_ELEMS ((int64_t)1 << 31)
int odl_fp8_cast_dynamic_noalloc(const void *x, int src_dtype, int64_t rows, int64_t cols, int fmt, int margin,
                                 uint8_t *out, uint8_t *out_t, float *dyn_out, odl_stream_t stream);

/*
 * odl_fp8_amax_parts that also adds up the columns: colsum[c] = sum over rows of x[r, c] in fp32.
 * For the grad_output of a Linear with a bias, whose bias gradient is that sum (the `db` of
 * te.pytorch.Linear's backward, transformer_engine.py:97-108): dY is read by this pass and by the
 * cast, not a third time.  The sum is formed from per-lane, per-block and per-slab partial sums in
 * a fixed order (reproducible on one device).  rows, cols > 0; cols a multiple of 8 (bf16) / 4
 * (fp32) and at most 512 * 256 (bf16) / 512 * 128 (fp32).
 * workspace: ODL_FP8_COLSUM_WORKSPACE floats of device memory, contents irrelevant.
 */
#define ODL_FP8_COLSUM_WORKSPACE (512 * 256)
int odl_fp8_amax_parts_colsum(const void *x, int src_dtype, int64_t rows, int64_t cols, float *parts,
                              float *colsum, float *workspace, odl_stream_t stream);

/*
 * The rowwise recipe needs every tensor twice: scaled per row for the GEMM that contracts
 * its columns, and scaled per column, transposed, for the GEMM that contracts its rows.
 *   odl_fp8_amax_rowcol: amax_row[rows] and amax_col[cols] in one pass over x;
 *   odl_fp8_cast_rowcol: out[rows, cols] = codes with scale_row, out_t[cols, rows] = codes
 *                        with scale_col, one pass; scale = fp8_max(fmt) / amax / 2^margin per
 *                        row / column (rules of odl_fp8_scale_from_amax); the scales and their
 *                        inverses are written to s_row, s_row_inv, s_col, s_col_inv.
 * Results equal those of odl_fp8_amax (ROW, COL) + odl_fp8_scale_from_amax + odl_fp8_cast (ROW)
 * + odl_fp8_cast_transpose (COL), bit for bit.  No counterpart in the reference (its recipes
 * stop at per-tensor and block scaling, fp8.py:58-61); this is the "rowwise" extension.
 */
int odl_fp8_amax_rowcol(const void *x, int src_dtype, int64_t rows, int64_t cols, float *amax_row,
                        float *amax_col, odl_stream_t stream);
int odl_fp8_cast_rowcol(const void *x, int src_dtype, int64_t rows, int64_t cols, const float *amax_row,
                        const float *amax_col, int fmt, int margin, uint8_t *out, uint8_t *out_t,
                        float *s_row, float *s_row_inv, float *s_col, float *s_col_inv,
                        odl_stream_t stream);

/*
 * Producers that hand the partial maxima of their OUTPUT to odl_fp8_cast_dynamic, so that the
 * tensor they write is quantised without an amax pass of its own.  parts has
 * ODL_FP8_AMAX_PARTS entries, as with odl_fp8_amax_parts.  All tensors are dense, bf16 unless
 * said otherwise, 16-byte aligned; rows * cols (SwiGLU) or cols (RMSNorm) a multiple of 8.
 *
 * The arithmetic is fixed to the last bit (IEEE fp32 operations in a stated order, no hardware
 * approximations), so a CPU restatement reproduces every output exactly:
 *   sigmoid(g): t = clamp(-g, -80, 80); k = rint(t * 1.44269504f);
 *               r = fma(k, -0.693359375f, t); r = fma(k, 2.12194440e-4f, r);
 *               p = Horner by fma of {1.9875691500e-4f, 1.3981999507e-3f, 8.3334519073e-3f,
 *                   4.1665795894e-2f, 1.6666665459e-1f, 5.0000001201e-1f} in r;
 *               e = (fma(p, r * r, r) + 1) * 2^k; d = 1 + e;
 *               y = bits(0x7EF311C7 - bits(d)); three times y = fma(y, fma(-d, y, 1), y);
 *               result y, 0 where -g > 80, NaN for NaN.
 *
 * odl_fp8_swiglu_amax_parts: h = bf16( bf16(gate * sigmoid(gate)) * up ), the value of
 *   silu(w1(x)) * w2(x) computed in bf16 (optimus_dl/modules/model/blocks/mlp.py:73-76);
 *   parts = partial maxima of |h|.
 * odl_fp8_swiglu_bwd_amax_parts: the gradients autograd derives for that expression in bf16:
 *   d_up   = bf16( dh * bf16(gate * sigmoid(gate)) )
 *   d_gate = bf16( bf16(dh * up) * (sig * fma(gate, 1 - sig, 1)) ),  sig = sigmoid(gate)
 *   with the partial maxima of |d_gate| and |d_up|.
 * odl_fp8_rmsnorm_amax_parts: y = bf16( (x * rstd) * weight ), rstd[r] = 1 / sqrt(sum_r / cols + eps)
 *   (IEEE sqrt and division), the RMSNorm of optimus_dl/modules/model/blocks/layer_norms.py:86-119;
 *   sum_r = sum of squares of row r in this order: lane l of 64 adds, by fma, the elements of the
 *   8-element chunks l, l + 64, l + 128, ... in ascending order; the 64 lane sums are then combined
 *   by the butterfly acc[l] += acc[l ^ off], off = 32, 16, 8, 4, 2, 1.  x is bf16 or fp32
 *   (src_dtype), weight fp32[cols], 8 <= cols <= 8192.  rstd[rows] is kept for the backward.
 */
int odl_fp8_swiglu_amax_parts(const void *gate, const void *up, int64_t rows, int64_t cols, void *h,
                              float *parts, odl_stream_t stream);
int odl_fp8_swiglu_bwd_amax_parts(const void *dh, const void *gate, const void *up, int64_t rows,
                                  int64_t cols, void *dgate, void *dup, float *parts_dgate,
                                  float *parts_dup, odl_stream_t stream);
int odl_fp8_rmsnorm_amax_parts(const void *x, int src_dtype, const float *weight, int64_t rows,
                               int64_t cols, float eps, void *y, float *rstd, float *parts,
                               odl_stream_t stream);

/*
 * Backward of that RMSNorm (what autograd derives for layer_norms.py:86-119), dy in bf16:
 *   xh = x * rstd, t = dy * weight, c = sum_row(t * xh) / cols
 *   dx = rstd * fma(-xh, c, t), rounded once to the dtype of x (src_dtype)
 *   Row sums of the backward kernels (this one and the LayerNorm one): the 8-element chunk k of a row
 *   belongs to wave (k / 64) % 4 and lane k % 64 of a 4-wave block; a lane adds its chunks in ascending
 *   order (t * xh by fma, elements in order), the 64 lanes of a wave are combined by the butterfly
 *   acc[l] += acc[l ^ off], off = 32 .. 1, and the four waves as ((s0 + s1) + s2) + s3.
 *   dweight[col] = sum over rows of dy * xh, fp32 (per-lane sums over the rows of a block, then the
 *   blocks' slabs in a fixed order: reproducible from run to run on one device)
 * workspace: ODL_FP8_RMSNORM_BWD_SLABS * cols floats of device memory, contents irrelevant.
 */
#define ODL_FP8_RMSNORM_BWD_SLABS 512
int odl_fp8_rmsnorm_bwd(const void *dy, const void *x, int src_dtype, const float *weight,
                        const float *rstd, int64_t rows, int64_t cols, void *dx, float *dweight,
                        float *workspace, odl_stream_t stream);

/*
 * LayerNorm (F.layer_norm over the last axis, optimus_dl/modules/model/blocks/layer_norms.py:21-47
 * and torch.nn.LayerNorm, both of which the reference's transform replaces,
 * transformer_engine.py:338-352) with the partial maxima of its output, and its backward.
 * Forward: row split and summation order of the RMSNorm forward; backward: those of the RMSNorm
 * backward; 8 <= cols <= 4096.
 *   mean = sum(x) / cols; d = x - mean; rstd = 1 / sqrt(sum(d * d) / cols + eps)  (d * d added by fma)
 *   y    = bf16( ((d * rstd) * weight) + bias ), bias may be NULL
 *   backward (dy bf16): xh = d * rstd, t = dy * weight, c1 = sum(t) / cols, c2 = sum(t * xh) / cols,
 *   dx = rstd * fma(-xh, c2, t - c1) in the dtype of x; dweight = sum_rows dy * xh and
 *   dbias = sum_rows dy, fp32, fixed-order partial sums.  dbias must be dweight + cols (one
 *   buffer of 2 * cols floats); workspace: 2 * ODL_FP8_RMSNORM_BWD_SLABS * cols floats.
 */
int odl_fp8_layernorm_amax_parts(const void *x, int src_dtype, const float *weight, const float *bias,
                                 int64_t rows, int64_t cols, float eps, void *y, float *mean,
                                 float *rstd, float *parts, odl_stream_t stream);
int odl_fp8_layernorm_bwd(const void *dy, const void *x, int src_dtype, const float *weight,
                          const float *mean, const float *rstd, int64_t rows, int64_t cols, void *dx,
                          float *dweight, float *dbias, float *workspace, odl_stream_t stream);

/*
 * Exact (erf) GELU between c_fc and c_proj of a GPT-2 MLP (optimus_dl/modules/model/blocks/mlp.py:141-157,
 * nn.GELU()), bf16 in and out, with the partial maxima of the output, and its backward.  GELU of a
 * bf16 value is a function of 16 bits, so both run from a table that odl_fp8_gelu_table fills once
 * (ODL_FP8_GELU_TABLE_BYTES of device memory owned by the caller; double-precision evaluation):
 *   fwd[x] = bf16( float( x * Phi(x) ) ),  Phi(x) = erfc(-x / sqrt 2) / 2
 *   bwd[x] = float( Phi(x) + x * exp(-x^2 / 2) / sqrt(2 pi) )
 *   odl_fp8_gelu_amax_parts     : y  = fwd[x];                  parts = partial maxima of |y|
 *   odl_fp8_gelu_bwd_amax_parts : dx = bf16( dy * bwd[x] );     parts = partial maxima of |dx|
 * rows * cols a multiple of 8, 16-byte aligned pointers.
 */
#define ODL_FP8_GELU_TABLE_BYTES (65536 * 2 + 65536 * 4)
int odl_fp8_gelu_table(void *table, odl_stream_t stream);
int odl_fp8_gelu_amax_parts(const void *x, int64_t rows, int64_t cols, const void *table, void *y,
                            float *parts, odl_stream_t stream);
int odl_fp8_gelu_bwd_amax_parts(const void *dy, const void *x, int64_t rows, int64_t cols,
                                const void *table, void *dx, float *parts, odl_stream_t stream);

/*
 * out[r,c] = fp8( clamp( fp32(x[r,c]) * s , +-max ) ), s = scale[0] | scale[r] | scale[c].
 * amax_out (may be NULL): *amax_out = max(*amax_out, max|x|), for delayed scaling,
 * where the cast uses an older scale while this step's amax is recorded.
 * Stands in for the cast inside te.pytorch.Linear (transformer_engine.py:106).
 */
int odl_fp8_cast(const void *x, int src_dtype, int64_t rows, int64_t cols,
                 const float *scale, int mode, int fmt,
                 uint8_t *out, float *amax_out, odl_stream_t stream);

/*
 * Same cast, also written transposed: out_t[c,r] = out[r,c] (out may be NULL
 * when only the transposed copy is wanted).  The transposed copies are what
 * dgrad (W^T) and wgrad (dY^T, X^T) contract over.
 */
int odl_fp8_cast_transpose(const void *x, int src_dtype, int64_t rows, int64_t cols,
                           const float *scale, int mode, int fmt,
                           uint8_t *out, uint8_t *out_t, float *amax_out, odl_stream_t stream);

/*
 * The cast of the delayed-scaling recipe in one launch (recipe "delayed", fp8.py:279-288; the cast inside
 * te.pytorch.Linear, transformer_engine.py:106, under that recipe): codes with the per-tensor scale in force
 * (scale[0], device memory), row-major (out), transposed (out_t) or both (either may be NULL, not both);
 *   amax_parts    : ODL_FP8_AMAX_PARTS floats (or NULL: nothing is recorded).  Block b folds its maximum of |x|
 *                   into amax_parts[b % ODL_FP8_AMAX_PARTS] (integer atomicMax of the magnitude bits, spread
 *                   over many words instead of one); the entries are NOT cleared first, so several casts of
 *                   one step accumulate.  odl_fp8_delayed_update folds and clears them.
 *   scale_inv_out : 1 float (or NULL) <- 1 / scale[0] (IEEE division), the factor for the GEMM, in storage
 *                   that the refresh after the step does not touch.
 */
int odl_fp8_cast_delayed(const void *x, int src_dtype, int64_t rows, int64_t cols, const float *scale, int fmt,
                         uint8_t *out, uint8_t *out_t, float *amax_parts, float *scale_inv_out, odl_stream_t stream);

/*
 * C[M,N] = (A[M,K] . B[N,K]^T) * (sa_inv[i] * sb_inv[j]) (+ bias[j]), fp32
 * accumulate on the MFMA units, rounded once to out_dtype (bf16 or fp32).
 *   a, b     : FP8 codes, K contiguous ("NT"); fmt_a / fmt_b may differ
 *   sa_inv   : 1 value (sa_n == 1) or M values; sb_inv: 1 or N values
 *   bias     : NULL or N fp32 values (bias_dtype must be ODL_F32), added in fp32
 *              before the single rounding to out_dtype
 *   accumulate : 0: C is overwritten.  Non-zero: C = C + product, the old value of C joining the fp32 sum
 *              after the bias, i.e. out = round(fl(fl(fl(acc * s) + bias) + C_old)): ONE rounding to out_dtype.
 *              This is the accumulate flag of the backend's GEMM: the weight gradient of a microbatch added
 *              into the gradient buffer (gradient accumulation,
 *              optimus_dl/recipe/train/mixins/execution/iteration_mixin.py:332), and the data gradients of
 *              Linears fed by one tensor (q/k/v, gate/up) summed without a separate pass.  Such a call runs on
 *              the kernels whose tiles end in a separate output phase (the old values are requested one slab of
 *              32 rows ahead), not on the streaming kernel.
 * Covers fwd (A=Xq, B=Wq), dgrad (A=dYq, B=Wq^T) and wgrad (A=dYq^T, B=Xq^T):
 * the three GEMMs of te.pytorch.Linear forward/backward.
 * K must be a multiple of 16; any M, N >= 1.
 */
int odl_fp8_gemm_nt(const uint8_t *a, const uint8_t *b, int64_t M, int64_t N, int64_t K,
                    int fmt_a, int fmt_b,
                    const float *sa_inv, int64_t sa_n, const float *sb_inv, int64_t sb_n,
                    const void *bias, int bias_dtype,
                    void *c, int out_dtype, int accumulate, odl_stream_t stream);

/*
 * A sum of such products in one call:
 *   C[M, N] = sum over s < pairs of (A_s[M, K[s]] . B_s[N, K[s]]^T) * (sa_inv[s][0] * sb_inv[s][0])
 * a, b, sa_inv, sb_inv: HOST arrays of `pairs` device pointers, K a host array of `pairs` lengths (all read
 * during the call); one scale per operand, no bias, out_dtype ODL_BF16 or ODL_F32, C is overwritten.  This is
 * the data gradient of Linears that are fed one tensor, dX = sum_s dY_s . W_s (q / k / v of the reference's
 * attention block, optimus_dl/modules/model/blocks/attention.py:317-319; gate / up of its gated MLP,
 * optimus_dl/modules/model/blocks/mlp.py:76-78): te.pytorch.Linear computes one dgrad per Linear and autograd
 * adds them up; here the streaming kernel runs the contraction through all pairs on one set of accumulators,
 * multiplying them by (scale product of pair s) / (scale product of pair s + 1) where it passes from one pair
 * to the next, and applies the last pair's scale product in its epilogue:
 *   C = round(((acc_0 r_0 + acc_1) r_1 + ... + acc_last) s_last), every step in fp32, ONE rounding to out_dtype.
 * That route is taken for 2 .. 4 pairs with M % 128 == 0, N % 128 == 0, every K[s] % 256 == 0 and >= 512 and
 * every operand under 2 GiB.  Anything else (up to 64 pairs, K[s] % 16 == 0) runs as one odl_fp8_gemm_nt per
 * pair, the second and later ones with accumulate set: one rounding to out_dtype per pair.  The two routes
 * agree within those roundings and bit for bit where every partial sum and every scale ratio is exact
 * (powers of two).
 */
int odl_fp8_gemm_nt_sum(int pairs, const uint8_t *const *a, const uint8_t *const *b, const int64_t *K,
                        int64_t M, int64_t N, int fmt_a, int fmt_b, const float *const *sa_inv,
                        const float *const *sb_inv, void *c, int out_dtype, odl_stream_t stream);

/*
 * The same product for operands that need no transposed copy.  layout_a / layout_b say how an
 * operand is stored: ODL_K_FAST = [rows, K] row-major (what odl_fp8_gemm_nt takes), ODL_K_SLOW =
 * [K, rows] row-major.  With per-tensor scaling the three GEMMs of te.pytorch.Linear then read the
 * row-major codes of X [M,K], W [N,K] and dY [M,N] directly:
 *   fwd   Y  = X . W^T      a = X  (K_FAST), b = W  (K_FAST)
 *   dgrad dX = dY . W       a = dY (K_FAST), b = W  (K_SLOW: contraction over N, W is [N, K])
 *   wgrad dW = dY^T . X     a = dY (K_SLOW), b = X  (K_SLOW: contraction over M)
 * Results equal those of odl_fp8_gemm_nt on the transposed copies bit for bit (same order of
 * accumulation).  One scale per operand, no bias, out_dtype ODL_BF16 or ODL_F32 (weight gradients
 * of fp32 master weights); M, N, K multiples of 256, K >= 512: anything else is refused with
 * ODL_ERR_SHAPE (make the transposed copy and use odl_fp8_gemm_nt).  There is no accumulate flag here
 * (only the streaming kernel reads K-slow operands): C = C + product with such operands is
 * odl_fp8_gemm_splitk with accumulate set, which takes a single run as well.
 */
enum odl_operand_layout { ODL_K_FAST = 0, ODL_K_SLOW = 1 };
int odl_fp8_gemm_layouts(const uint8_t *a, const uint8_t *b, int64_t M, int64_t N, int64_t K,
                         int fmt_a, int fmt_b, int layout_a, int layout_b, const float *sa_inv,
                         const float *sb_inv, void *c, int out_dtype, odl_stream_t stream);

/*
 * The same product for an output of few 256 x 256 tiles and a long contraction (weight gradients of
 * small layers, the input gradient of a vocabulary-sized head): K is cut into `splits` runs that are
 * computed side by side as unscaled fp32 partial results in `workspace` ([splits, M, N] floats,
 * caller-owned, no other use while the call is in flight on its stream), then added in run order,
 * scaled (sa_n / sb_n as for odl_fp8_gemm_nt), biased (fp32, may be NULL) and rounded once.  The sum
 * is therefore taken in a different order than by odl_fp8_gemm_nt: equal within fp32 rounding,
 * bit-identical where every partial sum is exact.  odl_fp8_gemm_split_count proposes `splits`
 * for a shape (1 = not worth splitting; k_slow != 0: an operand will be passed K-slow); any 2 <= splits <= 64 that leaves every run at least 512
 * long is accepted.  M, N, K multiples of 128 (256 for an operand stored K-slow), K-run >= 512.
 * accumulate != 0: the second kernel adds the old value of C to the sum before the one rounding
 * (C = C + product, as for odl_fp8_gemm_nt); splits == 1 is then accepted too, which is how a product
 * with an operand stored K-slow (a weight gradient that reads dY as stored) is added into C.
 * No counterpart in the reference, whose GEMMs are cuBLASLt's choice inside te.pytorch.Linear.
 */
int odl_fp8_gemm_split_count(int64_t M, int64_t N, int64_t K, int k_slow);
int odl_fp8_gemm_splitk(const uint8_t *a, const uint8_t *b, int64_t M, int64_t N, int64_t K,
                        int fmt_a, int fmt_b, int layout_a, int layout_b,
                        const float *sa_inv, int64_t sa_n, const float *sb_inv, int64_t sb_n,
                        const float *bias, void *c, int out_dtype, int accumulate, int splits,
                        void *workspace, int64_t workspace_bytes, odl_stream_t stream);

/*
 * Delayed-scaling bookkeeping for R tensor roles with H history slots each
 * (recipe "delayed", fp8.py:279-288; runs where the reference leaves its
 * autocast context, fp8.py:337-340,357-360).
 *   history [H,R] fp32 with leading dimension ld >= R (element (h,r) at h*ld + r),
 *   row 0 = newest amax (written by the casts of the step)
 *   a = max over the column (ODL_AMAX_MAX) or history[0] (ODL_AMAX_MOST_RECENT)
 *   history <- roll(history, -1 along H); history[0] <- 0
 *   scale[r] = fp8_max(fmt[r]) / a / 2^margin, kept when a is 0/NaN/Inf; Inf -> FLT_MAX
 *   scale_inv[r] = 1 / scale[r]
 *   fmt: R ints (odl_fp8_format) in device memory.
 *   amax_parts (or NULL): [R, ODL_FP8_AMAX_PARTS] partial maxima recorded by odl_fp8_cast_delayed, role r at
 *   amax_parts + r * ODL_FP8_AMAX_PARTS, 16-byte aligned; history[0, r] <- max(history[0, r], max of the
 *   role's entries) before anything else, and the entries are cleared for the next step.
 * One launch for all R roles; the cost grows with H * R (the roll moves the whole history), not with a chain
 * of H dependent reads per role.
 */
int odl_fp8_delayed_update(float *history, int64_t H, int64_t R, int64_t ld,
                           float *scale, float *scale_inv, const int *fmt,
                           int margin, int algo, float *amax_parts, odl_stream_t stream);

/*
 * Testing / tuning / introspection (host only).  odl_fp8_gemm_set_variant pins the GEMM kernel variant
 * for calls made from the CALLING HOST THREAD only (thread-local, like odl_fp8_last_error): -1 =
 * automatic choice by shape (the state every thread starts in); otherwise an index <
 * odl_fp8_gemm_num_variants().  It exists for tests that cross-check the kernels against each other
 * and for tuning sweeps; production callers never call it, and nothing else in the library is
 * mutable process state.  odl_fp8_gemm_variant_name returns a short description ("256x256x128 w4 s2").
 */
int odl_fp8_gemm_num_variants(void);
const char *odl_fp8_gemm_variant_name(int variant);
int odl_fp8_gemm_set_variant(int variant);
/*
 * BENCH-ONLY hook; a production build may compile it out (-DODL_FP8_NO_BENCH_HOOKS removes the entry point and the
 * two clock reads it switches on in the streaming kernel).  Host thread-local, like odl_fp8_gemm_set_variant; NULL
 * switches it off: launch i of the streaming GEMM kernel made from this thread afterwards writes record i % capacity
 * of records_dev, 4 x uint64 = {shader-clock counter, 100 MHz counter} on entry and on exit of the kernel's first
 * wave.  (exit - entry) of the first over (exit - entry) of the second, times 100 MHz, is the average shader clock
 * the board granted that launch.  No counterpart in the reference.
 */
#ifndef ODL_FP8_NO_BENCH_HOOKS
int odl_fp8_gemm_set_clock_probe(uint64_t *records_dev, int capacity);
#endif

/* ---------------------------------------------------------------------------------------------------------------
 * MXFP8: blocks of 32 consecutive elements along the contraction axis share one power-of-two scale, stored as an
 * E8M0 byte (value 2^(byte - 127); 0xFF = NaN).  Replaces, for the recipe string "mxfp8", what the reference hands to
 * its backend as MXFP8BlockScaling (optimus_dl/modules/amp/fp8.py:301-306) around the same Linear
 * (optimus_dl/modules/model/blocks/layers/linear.py:55-86).  The conversion rule is the one of the OCP Microscaling
 * Formats specification v1.0, section 6.3: shared exponent = floor(log2(block amax)) - emax_elem (8 for E4M3, 15 for
 * E5M2), clamped to [-127, 127]; elements = rne(clamp(v / 2^shared, +-fp8_max)); a block of zeros gets byte 0, a block
 * that holds Inf or NaN gets 0xFF.  There is no amax pass and no scale state: one kernel reads x once.
 *
 *   out    [rows, cols]      codes, blocks along the columns;  scales   for [rows, cols / 32] blocks   (cols % 32 == 0)
 *   out_t  [cols, rows]      codes of x^T, blocks along the rows of x;  scales_t for [cols, rows / 32] blocks   (rows % 32 == 0)
 * Either pair may be NULL (both members together).  cols % 8 == 0, x and out_t 16-byte aligned, out 8-byte aligned.
 *
 * Scale bytes of R rows x B blocks are stored in one of two layouts (chosen per output):
 *   ODL_MX_SCALES_ROWMAJOR  [R][B]: byte (r, b) at r * B + b
 *   ODL_MX_SCALES_KSTEP     [B / 4][R][4]: byte (r, b) at ((b / 4) * R + r) * 4 + b % 4; needs B % 4 == 0 (the blocked axis a
 *                           multiple of 128).  The 4 scales a row needs for one 128-byte K step of a GEMM are one dword, and
 *                           the dwords of consecutive rows are consecutive: a GEMM tile fetches its scales for a step as
 *                           one contiguous run.  The streaming GEMM kernel takes only this layout.
 *
 * scale_rule: how the shared exponent of a block follows from its amax.
 *   ODL_MX_SCALE_FLOOR  floor(log2 amax) - emax_elem: the formula of the OCP specification (section 6.3).  A block whose amax
 *                       lies in the top eighth of its binade (mantissa above 1.75) saturates: amax itself, and anything
 *                       beyond fp8_max * 2^shared, becomes +-fp8_max, up to 12.5 % off.
 *   ODL_MX_SCALE_CEIL   ceil(log2(amax / fp8_max)): the smallest power of two that brings amax inside the format, i.e. the
 *                       floor plus one where amax's mantissa exceeds 1.75; nothing saturates, and such a block loses one bit
 *                       of resolution instead.  This is what a quantiser computes that converts amax / fp8_max to E8M0 with
 *                       rounding up, which is how the backend behind the reference's `recipe: mxfp8` is published to work.
 */
#define ODL_MX_SCALES_ROWMAJOR 0
#define ODL_MX_SCALES_KSTEP 1
#define ODL_MX_SCALE_FLOOR 0
#define ODL_MX_SCALE_CEIL 1
int odl_fp8_mx_cast(const void *x, int src_dtype, int64_t rows, int64_t cols, int fmt, uint8_t *out, uint8_t *scales,
                    int scales_layout, uint8_t *out_t, uint8_t *scales_t, int scales_t_layout, int scale_rule, odl_stream_t stream);

/*
 * C[M, N] = sum over blocks kb of 2^(sa[m, kb] - 127) * 2^(sb[n, kb] - 127) * dot(A[m, 32 kb .. +32], B[n, 32 kb .. +32])
 * (+ bias[n]), accumulated in fp32 by the scaled MFMA (V_MFMA_SCALE_F32_32X32X64_F8F6F4 applies the two block scales to
 * the products), one rounding to out_dtype.  a [M, K], b [N, K] codes; sa, sb the scale bytes of the M x K / 32 and
 * N x K / 32 blocks, both in `scales_layout`; K % 32 == 0; a, b, c and bias 16-byte aligned.  With K-step-major scales,
 * M % 128 == 0, N % 128 == 0, K >= 512 and enough tiles to fill the chip the persistent streaming kernel runs (the one of
 * odl_fp8_gemm_nt, with the scale dwords riding beside the operand loads); K % 128 == 0 with 4-byte aligned scale arrays
 * otherwise runs an LDS-tiled kernel; other shapes a plain one-wave-per-tile kernel.  The first call on a device looks up a
 * constant in the library's device image (hipGetSymbolAddress): make it outside of stream capture.  accumulate: as for
 * odl_fp8_gemm_nt (C = C + product, one rounding; not on the streaming kernel).
 */
int odl_fp8_mx_gemm_nt(const uint8_t *a, const uint8_t *sa, const uint8_t *b, const uint8_t *sb, int scales_layout, int64_t M,
                       int64_t N, int64_t K, int fmt_a, int fmt_b, const float *bias, void *c, int out_dtype, int accumulate,
                       odl_stream_t stream);

/*
 * odl_fp8_mx_gemm_nt with K cut into `splits` runs that are computed side by side, for outputs of few tiles and a long
 * contraction (weight gradients of small layers), exactly as odl_fp8_gemm_splitk does for per-tensor scales
 * (odl_fp8_gemm_split_count says when and how many): fp32 partial results in `workspace` (splits * M * N floats, 16-byte
 * aligned, caller-owned), added in run order, bias added, one rounding.  K-step-major scales only; M, N, K multiples of
 * 128; every run at least 512 long.
 */
int odl_fp8_mx_gemm_splitk(const uint8_t *a, const uint8_t *sa, const uint8_t *b, const uint8_t *sb, int64_t M, int64_t N, int64_t K,
                           int fmt_a, int fmt_b, const float *bias, void *c, int out_dtype, int accumulate, int splits, void *workspace,
                           int64_t workspace_bytes, odl_stream_t stream);

/*
 * The cast of the "blockwise" recipe (what the reference hands to its backend as Float8BlockScaling,
 * optimus_dl/modules/amp/fp8.py:295-300): blocks of 128 elements along the contraction axis for activations and gradients
 * (two_d = 0: one scale per row and 128 columns for `out`, one per column and 128 rows for `out_t`), blocks of 128 x 128
 * for weights (two_d = 1: both outputs share the block's scale).  Scale of a block = fp8_max / amax / 2^margin (the rule of
 * odl_fp8_scale_from_amax; 1 when the amax is 0, NaN or Inf) rounded DOWN to a power of two, so nothing saturates;
 * elements = rne(clamp(v * scale)).  The inverse of such a scale is an E8M0 byte (254 - exponent field), and a 128-block is
 * four MX blocks with the same byte: `scales` / `scales_t` are written in the ODL_MX_SCALES_KSTEP layout ([cols / 128][rows]
 * and [rows / 128][cols] dwords of four equal bytes), and odl_fp8_mx_gemm_nt multiplies the results as they are.
 * rows and cols multiples of 128; x and the codes 16-byte aligned.  Either pair may be NULL.
 */
int odl_fp8_block_cast(const void *x, int src_dtype, int64_t rows, int64_t cols, int fmt, int margin, int two_d, uint8_t *out,
                       uint8_t *scales, uint8_t *out_t, uint8_t *scales_t, odl_stream_t stream);


#ifdef __cplusplus
}
#endif
#endif /* ODL_FP8_H */
