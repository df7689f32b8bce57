/*
 * CPU oracle for the FP8 Linear path.  TEST INFRASTRUCTURE ONLY: nothing in the
 * shipped package may include, link or call this file; it exists so that the
 * HIP kernels can be checked against an independent, plain-C restatement.
 *
 * What it restates.  The reference repository holds no FP8 arithmetic of its
 * own: optimus_dl/modules/model_transforms/transformer_engine.py:97-108 and
 * optimus_dl/modules/amp/fp8.py:254-306,337-340 forward everything to NVIDIA
 * Transformer Engine (pyproject.toml:80-82, pinned 2.15.0 in uv.lock:5728-5757,
 * not vendored).  The arithmetic below therefore follows the published
 * definitions that library implements:
 *   - OCP 8-bit floating point (E4M3 "fn" flavour, E5M2), round to nearest even
 *   - amax = max |x|; scale = fp8_max / amax / 2^margin (IEEE fp32 division)
 *   - cast = rne( clamp( fp32(x) * scale, +-fp8_max ) )
 *   - emulated GEMM: upcast the 8-bit codes to fp32, accumulate in fp32,
 *     multiply by the product of the inverse scales, round to bf16
 *   - delayed scaling: amax history ring, scale refreshed from max / most recent
 *
 * How each function is pinned (see tests/test_oracle_*.py):
 *   encode/decode : 256-entry decode tables from the format definition;
 *                   nearest-value brute force in float64; torch CPU
 *                   Tensor.to(float8_*) as the library routine (all bf16
 *                   patterns and a strided sweep of all fp32 exponents)
 *   amax / scale  : closed forms (max, IEEE division) against numpy/torch
 *   cast          : composition of the two above, against torch CPU
 *   cast_transpose: byte identity with cast followed by a transpose
 *   gemm          : float64 brute force on tiny shapes, exact special cases
 *                   (one-hot and power-of-two operands), torch._scaled_mm
 *   delayed update: hand-worked ring-buffer sequences and window properties.
 *                   The roll/update ORDER follows the documented behaviour of
 *                   the third-party library and cannot be checked against it
 *                   offline: parity unpinned for that ordering.
 *   mxfp8         : the OCP Microscaling v1.0 conversion formula restated in
 *                   float64 and with torch routines, hand-worked blocks,
 *                   power-of-two invariance (tests/test_oracle_mx.py).  The
 *                   third-party library's own rounding of the shared exponent
 *                   cannot be checked offline: parity unpinned for that choice.
 *   blockwise     : "the per-tensor rule on every block, scale rounded down to
 *                   a power of two" against the cast / scale functions above
 *                   block by block, a torch restatement, hand-worked blocks
 *                   (tests/test_oracle_block.py).  Parity unpinned likewise for
 *                   the third-party library's rounding of the block scale.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>
#include <float.h>
#include <stdlib.h>

#define ORACLE_API __attribute__((visibility("default")))

enum { FMT_E4M3 = 0, FMT_E5M2 = 1 };
enum { SCALE_TENSOR = 0, SCALE_ROW = 1, SCALE_COL = 2 };

static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline float bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

/* fp32 -> bf16, round to nearest even, NaN kept quiet (what torch does). */
static inline uint16_t f32_to_bf16(float f) {
    uint32_t u = f32_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

/*
 * Generic IEEE-style narrowing of an fp32 bit pattern to an 8-bit float with
 * `mbits` mantissa bits and exponent bias `bias`, round to nearest even, done
 * in integer arithmetic.  Returns the magnitude code WITHOUT overflow handling
 * (the caller maps too-large codes to NaN / Inf as the format demands).
 */
static uint32_t narrow_magnitude(uint32_t abs_bits, int mbits, int bias) {
    int e = (int)(abs_bits >> 23);
    uint32_t m = abs_bits & 0x7fffffu;
    if (e == 0) return 0;                       /* fp32 subnormal: far below any fp8 subnormal */
    int E = e - 127 + bias;                     /* biased target exponent */
    uint32_t full = m | 0x800000u;              /* 24-bit significand, value = full * 2^(e-150) */
    int shift = 23 - mbits;                     /* bits dropped for a normal result */
    uint32_t base;
    if (E >= 1) {
        base = ((uint32_t)E << mbits) | (m >> shift);
        full = m;                               /* remainder comes from the fraction only */
    } else {
        shift += 1 - E;                         /* subnormal target: drop more bits */
        if (shift > 25) return 0;               /* less than half of the smallest subnormal */
        base = full >> shift;                   /* shift <= 25 keeps this well defined */
    }
    uint32_t rem  = full & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (base & 1u))) base += 1;  /* carry may bump the exponent: intended */
    return base;
}

/* OCP E4M3 (finite-only "fn"): bias 7, max 448 = 0x7E, 0x7F = NaN, no Inf.
 * Non-saturating: anything that rounds past 448 becomes NaN (torch CPU cast). */
ORACLE_API uint8_t oracle_f32_to_e4m3(float f) {
    uint32_t u = f32_bits(f);
    uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
    uint32_t a = u & 0x7fffffffu;
    if (a >= 0x7f800000u) return sign | 0x7f;             /* Inf and NaN */
    uint32_t c = narrow_magnitude(a, 3, 7);
    if (c >= 0x7f) c = 0x7f;
    return sign | (uint8_t)c;
}

/* OCP E5M2: bias 15, max 57344 = 0x7B, 0x7C = Inf, 0x7D..0x7F = NaN.
 * Non-saturating: overflow goes to Inf.  NaN maps to 0x7F (torch CPU cast). */
ORACLE_API uint8_t oracle_f32_to_e5m2(float f) {
    uint32_t u = f32_bits(f);
    uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return sign | 0x7f;
    if (a == 0x7f800000u) return sign | 0x7c;
    uint32_t c = narrow_magnitude(a, 2, 15);
    if (c >= 0x7c) c = 0x7c;
    return sign | (uint8_t)c;
}

ORACLE_API float oracle_e4m3_to_f32(uint8_t c) {
    int e = (c >> 3) & 0xf, m = c & 7;
    float v;
    if (e == 0xf && m == 7) v = NAN;
    else if (e == 0) v = ldexpf((float)m, -9);             /* m/8 * 2^-6 */
    else v = ldexpf(1.0f + (float)m / 8.0f, e - 7);
    return (c & 0x80) ? -v : v;
}

ORACLE_API float oracle_e5m2_to_f32(uint8_t c) {
    int e = (c >> 2) & 0x1f, m = c & 3;
    float v;
    if (e == 0x1f) v = m ? NAN : INFINITY;
    else if (e == 0) v = ldexpf((float)m, -16);            /* m/4 * 2^-14 */
    else v = ldexpf(1.0f + (float)m / 4.0f, e - 15);
    return (c & 0x80) ? -v : v;
}

static inline float fp8_max_of(int fmt) { return fmt == FMT_E5M2 ? 57344.0f : 448.0f; }
static inline uint8_t encode(float v, int fmt) {
    return fmt == FMT_E5M2 ? oracle_f32_to_e5m2(v) : oracle_f32_to_e4m3(v);
}
static inline float decode(uint8_t c, int fmt) {
    return fmt == FMT_E5M2 ? oracle_e5m2_to_f32(c) : oracle_e4m3_to_f32(c);
}

ORACLE_API void oracle_encode_f32(const float *x, int64_t n, int fmt, uint8_t *out) {
    for (int64_t i = 0; i < n; ++i) out[i] = encode(x[i], fmt);
}
ORACLE_API void oracle_decode(const uint8_t *c, int64_t n, int fmt, float *out) {
    for (int64_t i = 0; i < n; ++i) out[i] = decode(c[i], fmt);
}

/* max that propagates NaN, like torch.amax. */
static inline float nanmax(float a, float b) {
    if (a != a) return a;
    if (b != b) return b;
    return a > b ? a : b;
}

/* amax over a bf16 matrix [rows, cols] (row-major).
 * mode SCALE_TENSOR -> out[1], SCALE_ROW -> out[rows], SCALE_COL -> out[cols]. */
ORACLE_API void oracle_amax_bf16(const uint16_t *x, int64_t rows, int64_t cols, int mode, float *out) {
    int64_t n_out = mode == SCALE_TENSOR ? 1 : (mode == SCALE_ROW ? rows : cols);
    for (int64_t i = 0; i < n_out; ++i) out[i] = 0.0f;
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t c = 0; c < cols; ++c) {
            float a = fabsf(bf16_to_f32(x[r * cols + c]));
            int64_t o = mode == SCALE_TENSOR ? 0 : (mode == SCALE_ROW ? r : c);
            out[o] = nanmax(out[o], a);
        }
}

/* scale = fp8_max / amax / 2^margin as IEEE fp32; `fallback` when amax is not a
 * positive finite number; an infinite quotient is replaced by FLT_MAX. */
ORACLE_API float oracle_scale(float amax, int fmt, int margin, float fallback) {
    if (!(amax > 0.0f) || isinf(amax)) return fallback;      /* catches NaN, 0, negatives, Inf */
    volatile float s = fp8_max_of(fmt) / amax;               /* volatile: no excess precision */
    s = ldexpf(s, -margin);
    if (isinf(s)) s = FLT_MAX;
    return s;
}

ORACLE_API float oracle_scale_inv(float scale) {
    volatile float r = 1.0f / scale;
    return r;
}

static inline uint8_t quantise(uint16_t xb, float scale, int fmt) {
    float x = bf16_to_f32(xb);
    if (x != x) return (uint8_t)(((xb >> 8) & 0x80u) | 0x7fu);
    volatile float y = x * scale;                            /* one fp32 multiply */
    float m = fp8_max_of(fmt), v = y;
    if (v > m) v = m;
    if (v < -m) v = -m;
    if (v != v) return (uint8_t)(((xb >> 8) & 0x80u) | 0x7fu);  /* 0*inf cannot occur (scale finite) */
    return encode(v, fmt);
}

/* cast of a bf16 matrix with per-tensor / per-row / per-column scale. */
ORACLE_API void oracle_cast_bf16(const uint16_t *x, int64_t rows, int64_t cols, const float *scale,
                                 int mode, int fmt, uint8_t *out) {
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t c = 0; c < cols; ++c) {
            float s = mode == SCALE_TENSOR ? scale[0] : (mode == SCALE_ROW ? scale[r] : scale[c]);
            out[r * cols + c] = quantise(x[r * cols + c], s, fmt);
        }
}

/* out_t[c, r] = cast(x)[r, c]  (the copy wgrad/dgrad contract over) */
ORACLE_API void oracle_cast_transpose_bf16(const uint16_t *x, int64_t rows, int64_t cols, const float *scale,
                                           int mode, int fmt, uint8_t *out, uint8_t *out_t) {
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t c = 0; c < cols; ++c) {
            float s = mode == SCALE_TENSOR ? scale[0] : (mode == SCALE_ROW ? scale[r] : scale[c]);
            uint8_t q = quantise(x[r * cols + c], s, fmt);
            if (out) out[r * cols + c] = q;
            out_t[c * rows + r] = q;
        }
}

/*
 * Emulated FP8 GEMM, "NT": C[M,N] = A[M,K] * B[N,K]^T, operands are 8-bit codes.
 * fp32 accumulate over k in ascending order; epilogue multiplies by
 * (sa_inv * sb_inv) with sa_inv scalar (sa_n == 1) or per-row of A (sa_n == M),
 * sb_inv scalar or per-row of B (sb_n == N); then rounds to bf16.
 * If c_f32 is not NULL the un-rounded fp32 result is stored there as well.
 */
ORACLE_API void oracle_gemm_nt(const uint8_t *a, const uint8_t *b, int64_t M, int64_t N, int64_t K,
                               int fmt_a, int fmt_b, const float *sa_inv, int64_t sa_n,
                               const float *sb_inv, int64_t sb_n, uint16_t *c_bf16, float *c_f32) {
    float lut_a[256], lut_b[256];
    for (int i = 0; i < 256; ++i) { lut_a[i] = decode((uint8_t)i, fmt_a); lut_b[i] = decode((uint8_t)i, fmt_b); }
    /* built with -ffp-contract=off; the product of two 8-bit floats is exact in
     * fp32 (at most 8 significant bits), so only the additions round */
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < M; ++i)
        for (int64_t j = 0; j < N; ++j) {
            float acc = 0.0f;
            for (int64_t k = 0; k < K; ++k) acc += lut_a[a[i * K + k]] * lut_b[b[j * K + k]];
            volatile float s = (sa_n == 1 ? sa_inv[0] : sa_inv[i]) * (sb_n == 1 ? sb_inv[0] : sb_inv[j]);
            volatile float v = acc * s;
            if (c_f32) c_f32[i * N + j] = v;
            if (c_bf16) c_bf16[i * N + j] = f32_to_bf16(v);
        }
}

/*
 * MXFP8 (recipe "mxfp8", optimus_dl/modules/amp/fp8.py:301-306 -> the third-party library's MXFP8BlockScaling): blocks of 32
 * consecutive elements along the contraction axis share a power-of-two scale, stored as one E8M0 byte (value 2^(byte - 127)).
 * The conversion follows the OCP Microscaling Formats (MX) specification v1.0, section 6.3:
 *   shared_exp = floor(log2(max |v|)) - emax_elem      (emax_elem: 8 for E4M3, 15 for E5M2), clamped to [-127, 127]
 *   scale byte = shared_exp + 127; a block of zeros gets byte 0; a block holding a NaN or an infinity gets 0xFF
 *   element    = rne( clamp( v * 2^-shared_exp, +-fp8_max ) )    (saturating, as every cast of this library)
 * The third-party library rounds the shared exponent its own way (towards larger scales, so that nothing saturates);
 * that choice cannot be checked offline: parity unpinned against it, pinned against the specification's formula.
 */
static inline int emax_elem(int fmt) { return fmt == FMT_E5M2 ? 15 : 8; }

/* rule 0: the specification's floor (above).  rule 1: the exponent rounded UP, shared_exp = ceil(log2(amax / fp8_max)), the
 * smallest power of two that brings the block's amax inside the format, so that no element saturates (the convention of
 * quantisers that derive the scale byte from amax / fp8_max with a round-up conversion to E8M0).  fp8_max = 1.75 * 2^emax for
 * both formats, so with amax = m * 2^e, 1 <= m < 2: ceil(log2(amax / fp8_max)) = e - emax + (m > 1.75 ? 1 : 0). */
ORACLE_API void oracle_mx_quantise_bf16(const uint16_t *x, int64_t rows, int64_t cols, int fmt, int rule, uint8_t *codes, uint8_t *scales) {
    const int64_t nb = cols / 32;
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t b = 0; b < nb; ++b) {
            const uint16_t *v = x + r * cols + b * 32;
            uint32_t mag = 0;
            for (int i = 0; i < 32; ++i) { uint32_t m = (uint32_t)(v[i] & 0x7fffu) << 16; if (m > mag) mag = m; }
            uint8_t sb;
            float mul;
            if (mag >= 0x7f800000u) { sb = 0xff; mul = 1.0f; }                 /* Inf / NaN in the block */
            else if (mag == 0) { sb = 0; mul = 1.0f; }
            else {
                int e;                                                            /* floor(log2(amax)), subnormals included */
                (void)frexpf(bits_f32(mag), &e);
                int se = (e - 1) - emax_elem(fmt);
                if (rule == 1 && frexpf(bits_f32(mag), &e) > 0.875f) se += 1;        /* frexp's mantissa is m / 2 */
                if (se < -127) se = -127;
                if (se > 127) se = 127;
                sb = (uint8_t)(se + 127);
                mul = ldexpf(1.0f, -se);                                          /* 2^-se: exact, at most 2^127 */
            }
            scales[r * nb + b] = sb;
            for (int i = 0; i < 32; ++i) codes[r * cols + b * 32 + i] = quantise(v[i], mul, fmt);
        }
}

/* C[M,N] = sum over 32-blocks kb of 2^(sa[m,kb] - 127 + sb[n,kb] - 127) * dot(A[m, kb], B[n, kb]); fp32 accumulation, block dots
 * added in ascending kb; a scale byte 0xFF makes the result NaN.  bias (fp32, may be NULL) is added before the rounding. */
ORACLE_API void oracle_mx_gemm_nt(const uint8_t *a, const uint8_t *sa, const uint8_t *b, const uint8_t *sb, int64_t M, int64_t N,
                                  int64_t K, int fmt_a, int fmt_b, const float *bias, uint16_t *c_bf16, float *c_f32) {
    float lut_a[256], lut_b[256];
    for (int i = 0; i < 256; ++i) { lut_a[i] = decode((uint8_t)i, fmt_a); lut_b[i] = decode((uint8_t)i, fmt_b); }
    const int64_t nb = K / 32;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < M; ++i)
        for (int64_t j = 0; j < N; ++j) {
            float acc = 0.0f;
            for (int64_t kb = 0; kb < nb; ++kb) {
                float dot = 0.0f;
                for (int k = 0; k < 32; ++k) dot += lut_a[a[i * K + kb * 32 + k]] * lut_b[b[j * K + kb * 32 + k]];
                const uint8_t ea = sa[i * nb + kb], eb = sb[j * nb + kb];
                if (ea == 0xff || eb == 0xff) { acc = NAN; continue; }
                volatile float term = ldexpf(dot, (int)ea + (int)eb - 254);
                acc += term;
            }
            volatile float v = bias ? acc + bias[j] : acc;
            if (c_f32) c_f32[i * N + j] = v;
            if (c_bf16) c_bf16[i * N + j] = f32_to_bf16(v);
        }
}

/*
 * Blockwise recipe (the reference's "blockwise", optimus_dl/modules/amp/fp8.py:295-300, which hands its backend a
 * Float8BlockScaling recipe: 1 x 128 blocks along the contraction axis for activations and gradients, 128 x 128 blocks
 * for weights, power-of-two scales).  Restated as: the per-tensor rule of oracle_scale applied to the amax of each block
 * of block_r x block_c elements, the result rounded DOWN to a power of two (mantissa cleared; a subnormal result becomes
 * 2^-126), elements = rne(clamp(v * scale)).  Rounding down keeps amax * scale <= fp8_max: nothing saturates.  The inverse
 * of such a scale is an E8M0 byte, 254 - (exponent field of the scale); a block whose amax is 0, NaN or Inf keeps scale 1
 * (byte 127).  The backend's own rounding of the scale cannot be checked here: parity unpinned for that choice; everything
 * else is pinned by tests/test_oracle_block.py.
 *   codes [rows, cols]; scale_bytes [rows / block_r, cols / block_c]
 */
ORACLE_API void oracle_block_quantise_bf16(const uint16_t *x, int64_t rows, int64_t cols, int64_t block_r, int64_t block_c,
                                           int fmt, int margin, uint8_t *codes, uint8_t *scale_bytes) {
    const int64_t nbr = rows / block_r, nbc = cols / block_c;
    for (int64_t br = 0; br < nbr; ++br)
        for (int64_t bc = 0; bc < nbc; ++bc) {
            uint32_t mag = 0;
            for (int64_t r = 0; r < block_r; ++r)
                for (int64_t c = 0; c < block_c; ++c) {
                    uint32_t m = (uint32_t)(x[(br * block_r + r) * cols + bc * block_c + c] & 0x7fffu) << 16;
                    if (m > mag) mag = m;                                  /* NaN patterns sort above Inf */
                }
            float s = oracle_scale(bits_f32(mag), fmt, margin, 1.0f);
            uint32_t sb = f32_bits(s) & 0xff800000u;
            if ((sb >> 23) == 0) sb = 0x00800000u;
            s = bits_f32(sb);
            scale_bytes[br * nbc + bc] = (uint8_t)(254u - (sb >> 23));
            for (int64_t r = 0; r < block_r; ++r)
                for (int64_t c = 0; c < block_c; ++c) {
                    const int64_t i = (br * block_r + r) * cols + bc * block_c + c;
                    codes[i] = quantise(x[i], s, fmt);
                }
        }
}

/*
 * Delayed-scaling bookkeeping for R roles with a history of H steps each,
 * history stored [H, R] row-major with row 0 = the newest amax (written by the
 * cast kernels of the step that just ran).
 *   a      = max over the column (algo 0, "max") or history[0] (algo 1, "most_recent")
 *   roll   : history <- roll(history, -1 along H); history[0] <- 0
 *   scale  = fp8_max/a/2^margin, unchanged when a is 0 / NaN / Inf; Inf -> FLT_MAX
 *   scale_inv = 1/scale
 */
ORACLE_API void oracle_delayed_update(float *history, int64_t H, int64_t R, float *scale, float *scale_inv,
                                      const int *fmt, int margin, int algo) {
    for (int64_t r = 0; r < R; ++r) {
        float a = history[r];
        if (algo == 0)
            for (int64_t h = 1; h < H; ++h) a = nanmax(a, history[h * R + r]);
        /* roll by -1: row h takes row h+1, last row takes old row 0, then row 0 is cleared */
        float first = history[r];
        for (int64_t h = 0; h + 1 < H; ++h) history[h * R + r] = history[(h + 1) * R + r];
        history[(H - 1) * R + r] = first;
        history[r] = 0.0f;
        scale[r] = oracle_scale(a, fmt[r], margin, scale[r]);
        scale_inv[r] = oracle_scale_inv(scale[r]);
    }
}

/* ------------------------------------------------------------------------------------------
 * Producers either side of the Linear: SwiGLU (optimus_dl/modules/model/blocks/mlp.py:73-76,
 * `silu(w1(x)) * w2(x)` evaluated in bf16 under autocast, and the gradients autograd derives
 * for it) and RMSNorm (optimus_dl/modules/model/blocks/layer_norms.py:86-119).  The reference
 * leaves both to PyTorch; the kernels fix the arithmetic to the last bit (documented in the C
 * header of the library) and this is the same sequence of IEEE fp32 operations in plain C.
 * Pinned in tests/test_oracle_fused.py: sigmoid against float64 over ALL bf16 inputs,
 * SwiGLU forward / backward against torch's bf16 silu, multiplication and autograd on the CPU
 * (equal up to one bf16 unit in a small fraction of elements, since torch's exp differs in the
 * last fp32 bits), RMSNorm against the float64 closed form and against torch in fp32.
 * Built with -ffp-contract=off: every fused multiply-add below is an explicit fmaf().
 */
static float recip_newton(float d) {
    float y = bits_f32(0x7EF311C7u - f32_bits(d));
    y = fmaf(y, fmaf(-d, y, 1.0f), y);
    y = fmaf(y, fmaf(-d, y, 1.0f), y);
    y = fmaf(y, fmaf(-d, y, 1.0f), y);
    return y;
}

ORACLE_API float oracle_sigmoid(float g) {
    if (g != g) return g;
    float t = -g;
    int zero = t > 80.0f;
    if (t < -80.0f) t = -80.0f;
    if (zero) t = 80.0f;
    float kf = rintf(t * 1.44269504f);                 /* ties to even (default rounding mode) */
    float r = fmaf(kf, -0.693359375f, t);
    r = fmaf(kf, 2.12194440e-4f, r);
    float p = 1.9875691500e-4f;
    p = fmaf(p, r, 1.3981999507e-3f);
    p = fmaf(p, r, 8.3334519073e-3f);
    p = fmaf(p, r, 4.1665795894e-2f);
    p = fmaf(p, r, 1.6666665459e-1f);
    p = fmaf(p, r, 5.0000001201e-1f);
    float z = r * r;
    float y = fmaf(p, z, r) + 1.0f;
    float e = y * bits_f32((uint32_t)((int)kf + 127) << 23);
    float s = recip_newton(1.0f + e);
    return zero ? 0.0f : s;
}

static inline float round_bf16(float f) { return bf16_to_f32(f32_to_bf16(f)); }

ORACLE_API void oracle_swiglu_fwd(const uint16_t *gate, const uint16_t *up, int64_t n, uint16_t *h) {
    for (int64_t i = 0; i < n; ++i) {
        float g = bf16_to_f32(gate[i]), u = bf16_to_f32(up[i]);
        float s = round_bf16(g * oracle_sigmoid(g));
        h[i] = f32_to_bf16(s * u);
    }
}

ORACLE_API void oracle_swiglu_bwd(const uint16_t *dh, const uint16_t *gate, const uint16_t *up, int64_t n,
                                  uint16_t *dgate, uint16_t *dup) {
    for (int64_t i = 0; i < n; ++i) {
        float d = bf16_to_f32(dh[i]), g = bf16_to_f32(gate[i]), u = bf16_to_f32(up[i]);
        float sig = oracle_sigmoid(g);
        float s = round_bf16(g * sig);
        dup[i] = f32_to_bf16(d * s);
        float ds = round_bf16(d * u);
        float dsilu = sig * fmaf(g, 1.0f - sig, 1.0f);
        dgate[i] = f32_to_bf16(ds * dsilu);
    }
}

/* x: bf16 (src 0) or fp32 (src 1), [rows, cols], cols % 8 == 0; the summation order is the one the
 * C header of the library states (64 lanes, 8-element chunks dealt round-robin, xor butterfly). */
ORACLE_API void oracle_rmsnorm(const void *x, int src, const float *weight, int64_t rows, int64_t cols, float eps,
                               uint16_t *y, float *rstd_out) {
    const int64_t nchunk = cols / 8;
    for (int64_t r = 0; r < rows; ++r) {
        float acc[64];
        for (int l = 0; l < 64; ++l) {
            float a = 0.0f;
            for (int64_t c = l; c < nchunk; c += 64)
                for (int e = 0; e < 8; ++e) {
                    int64_t idx = r * cols + c * 8 + e;
                    float v = src == 0 ? bf16_to_f32(((const uint16_t *)x)[idx]) : ((const float *)x)[idx];
                    a = fmaf(v, v, a);
                }
            acc[l] = a;
        }
        for (int off = 32; off > 0; off >>= 1) {
            float nxt[64];
            for (int l = 0; l < 64; ++l) nxt[l] = acc[l] + acc[l ^ off];
            memcpy(acc, nxt, sizeof(acc));
        }
        float mean = acc[0] / (float)cols;
        float rstd = 1.0f / sqrtf(mean + eps);
        rstd_out[r] = rstd;
        for (int64_t c = 0; c < cols; ++c) {
            int64_t idx = r * cols + c;
            float v = src == 0 ? bf16_to_f32(((const uint16_t *)x)[idx]) : ((const float *)x)[idx];
            y[idx] = f32_to_bf16((v * rstd) * weight[c]);
        }
    }
}

/* Backward of the RMSNorm above for bf16 dy.  dx follows the library's stated sequence of IEEE
 * operations (bit-exact target); d_weight is accumulated in double here, because the library only
 * promises a fixed but device-dependent order of fp32 partial sums (tolerance target).  Pinned in
 * tests/test_oracle_fused.py against torch autograd of the reference module's expression. */
static float lane_butterfly(float *acc) {
    for (int off = 32; off > 0; off >>= 1) {
        float nxt[64];
        for (int l = 0; l < 64; ++l) nxt[l] = acc[l] + acc[l ^ off];
        memcpy(acc, nxt, 64 * sizeof(float));
    }
    return acc[0];
}

static inline float load_src(const void *x, int src, int64_t idx) {
    return src == 0 ? bf16_to_f32(((const uint16_t *)x)[idx]) : ((const float *)x)[idx];
}

/* Row sums of the backward kernels: the 8-element chunk c of a row belongs to wave (c / 64) % 4, lane c % 64;
 * a lane adds its chunks in ascending order (elements in order), the 64 lanes of a wave are combined by the
 * xor butterfly, the four waves as ((s0 + s1) + s2) + s3.  term(idx, which) is the summand of element idx. */
typedef float (*row_term_fn)(const void *ctx, int64_t idx, int which);
static float row_sum_4waves(const void *ctx, row_term_fn term, int which, int64_t r, int64_t cols) {
    const int64_t nchunk = cols / 8;
    float wave_sum[4];
    for (int w = 0; w < 4; ++w) {
        float acc[64];
        for (int l = 0; l < 64; ++l) {
            float a = 0.0f;
            for (int64_t c = (int64_t)w * 64 + l; c < nchunk; c += 256)
                for (int e = 0; e < 8; ++e) {
                    int64_t idx = r * cols + c * 8 + e;
                    float t = term(ctx, idx, 0);
                    if (which == 0) a = a + t;                       /* plain sum of t */
                    else a = fmaf(t, term(ctx, idx, 1), a);          /* sum of t * xh by fma */
                }
            acc[l] = a;
        }
        wave_sum[w] = lane_butterfly(acc);
    }
    return ((wave_sum[0] + wave_sum[1]) + wave_sum[2]) + wave_sum[3];
}

struct norm_ctx { const uint16_t *dy; const void *x; int src; const float *weight; float mean, rstd; int64_t cols; };
static float norm_term(const void *vctx, int64_t idx, int which) {
    const struct norm_ctx *c = (const struct norm_ctx *)vctx;
    if (which == 0) return bf16_to_f32(c->dy[idx]) * c->weight[idx % c->cols];
    return (load_src(c->x, c->src, idx) - c->mean) * c->rstd;
}
static float rms_term(const void *vctx, int64_t idx, int which) {
    const struct norm_ctx *c = (const struct norm_ctx *)vctx;
    if (which == 0) return bf16_to_f32(c->dy[idx]) * c->weight[idx % c->cols];
    return load_src(c->x, c->src, idx) * c->rstd;
}

ORACLE_API void oracle_rmsnorm_bwd(const uint16_t *dy, const void *x, int src, const float *weight, const float *rstd_in,
                                   int64_t rows, int64_t cols, void *dx, float *dweight) {
    double *dw = (double *)calloc((size_t)cols, sizeof(double));
    for (int64_t r = 0; r < rows; ++r) {
        const float rstd = rstd_in[r];
        struct norm_ctx ctx = {dy, x, src, weight, 0.0f, rstd, cols};
        const float cmean = row_sum_4waves(&ctx, rms_term, 1, r, cols) / (float)cols;
        for (int64_t c = 0; c < cols; ++c) {
            int64_t idx = r * cols + c;
            float xh = load_src(x, src, idx) * rstd;
            float d = bf16_to_f32(dy[idx]);
            float o = rstd * fmaf(-xh, cmean, d * weight[c]);
            if (src == 0) ((uint16_t *)dx)[idx] = f32_to_bf16(o); else ((float *)dx)[idx] = o;
            dw[c] += (double)d * (double)xh;
        }
    }
    for (int64_t c = 0; c < cols; ++c) dweight[c] = (float)dw[c];
    free(dw);
}

/* LayerNorm (F.layer_norm, optimus_dl/modules/model/blocks/layer_norms.py:21-47) in the library's
 * stated order of IEEE operations, and its backward (dx bit-exact target; d_weight / d_bias summed
 * in double: tolerance targets).  Pinned in tests/test_oracle_fused.py against float64 closed
 * forms, torch's F.layer_norm and autograd, and exact special cases. */
ORACLE_API void oracle_layernorm(const void *x, int src, const float *weight, const float *bias, int64_t rows, int64_t cols,
                                 float eps, uint16_t *y, float *mean_out, float *rstd_out) {
    const int64_t nchunk = cols / 8;
    for (int64_t r = 0; r < rows; ++r) {
        float acc[64];
        for (int l = 0; l < 64; ++l) {
            float a = 0.0f;
            for (int64_t c = l; c < nchunk; c += 64)
                for (int e = 0; e < 8; ++e) a = a + load_src(x, src, r * cols + c * 8 + e);
            acc[l] = a;
        }
        const float mean = lane_butterfly(acc) / (float)cols;
        for (int l = 0; l < 64; ++l) {
            float a = 0.0f;
            for (int64_t c = l; c < nchunk; c += 64)
                for (int e = 0; e < 8; ++e) {
                    float d = load_src(x, src, r * cols + c * 8 + e) - mean;
                    a = fmaf(d, d, a);
                }
            acc[l] = a;
        }
        const float var = lane_butterfly(acc) / (float)cols;
        const float rstd = 1.0f / sqrtf(var + eps);
        mean_out[r] = mean;
        rstd_out[r] = rstd;
        for (int64_t c = 0; c < cols; ++c) {
            float o = ((load_src(x, src, r * cols + c) - mean) * rstd) * weight[c];
            if (bias) o = o + bias[c];
            y[r * cols + c] = f32_to_bf16(o);
        }
    }
}

ORACLE_API void oracle_layernorm_bwd(const uint16_t *dy, const void *x, int src, const float *weight, const float *mean_in,
                                     const float *rstd_in, int64_t rows, int64_t cols, void *dx, float *dweight, float *dbias) {
    double *dw = (double *)calloc((size_t)cols * 2, sizeof(double));
    for (int64_t r = 0; r < rows; ++r) {
        const float mean = mean_in[r], rstd = rstd_in[r];
        struct norm_ctx ctx = {dy, x, src, weight, mean, rstd, cols};
        const float c1 = row_sum_4waves(&ctx, norm_term, 0, r, cols) / (float)cols;
        const float c2 = row_sum_4waves(&ctx, norm_term, 1, r, cols) / (float)cols;
        for (int64_t c = 0; c < cols; ++c) {
            int64_t idx = r * cols + c;
            float xh = (load_src(x, src, idx) - mean) * rstd;
            float d = bf16_to_f32(dy[idx]);
            float o = rstd * fmaf(-xh, c2, d * weight[c] - c1);
            if (src == 0) ((uint16_t *)dx)[idx] = f32_to_bf16(o); else ((float *)dx)[idx] = o;
            dw[c] += (double)d * (double)xh;
            dw[cols + c] += (double)d;
        }
    }
    for (int64_t c = 0; c < cols; ++c) { dweight[c] = (float)dw[c]; dbias[c] = (float)dw[cols + c]; }
    free(dw);
}

/* Exact (erf) GELU of a bf16 input, nn.GELU() in optimus_dl/modules/model/blocks/mlp.py:141-157, and
 * its derivative, evaluated in double precision with libm and rounded once to float (then bf16 for
 * the forward): the definition of the library's lookup table.  Pinned in tests/test_oracle_fused.py
 * against torch's F.gelu and autograd over every bf16 input (torch evaluates 1 + erf(x / sqrt 2) in
 * float, which loses the far negative tail: there the comparison is absolute). */
ORACLE_API void oracle_gelu_fwd(const uint16_t *x, int64_t n, uint16_t *y) {
    for (int64_t i = 0; i < n; ++i) {
        double v = (double)bf16_to_f32(x[i]);
        double cdf = 0.5 * erfc(-v * 0.70710678118654752440);
        y[i] = f32_to_bf16((float)(v * cdf));
    }
}

ORACLE_API void oracle_gelu_bwd(const uint16_t *dy, const uint16_t *x, int64_t n, uint16_t *dx) {
    for (int64_t i = 0; i < n; ++i) {
        double v = (double)bf16_to_f32(x[i]);
        double cdf = 0.5 * erfc(-v * 0.70710678118654752440);
        double pdf = exp(-0.5 * v * v) * 0.39894228040143267794;
        float d = (float)(cdf + v * pdf);
        dx[i] = f32_to_bf16(bf16_to_f32(dy[i]) * d);
    }
}
