// FP8 GEMM entry point: argument checks, kernel choice, and the generic kernel.
//
//   C[M,N] = (A[M,K] . B[N,K]^T) * (sa_inv[i] * sb_inv[j]) (+ bias[j])
//
// Both operands are K-contiguous 8-bit codes ("NT").  Kernels:
//   gemm_tiled.hip : BM x BN block tiles through two LDS stages
//   gemm_pipe.hip  : 256x256 tile, one wave per SIMD, explicit software pipeline
//   gemm_stream.hip: the same pipeline running across tile boundaries, epilogue under the
//                    next tile's MFMAs (M, N, K multiples of 128); with a split over K for
//                    outputs of few tiles, summed by splitk_reduce_kernel below
//   here           : generic one-wave-per-32x32-tile kernel for any M, N, K % 16 == 0
#include "gemm_common.h"

namespace odl {

// ---------------------------------------------------------------- generic kernel
template <int FA, int FB>
__global__ __launch_bounds__(64) void gemm_nt_generic_kernel(const GemmArgs g) {
    const int64_t tile = blockIdx.x;
    const int64_t m0 = (tile % g.tiles_m) * 32, n0 = (tile / g.tiles_m) * 32;
    const int lane = threadIdx.x, lr = lane % 32, lg = lane / 32;
    const uint8_t *pa = g.a + min(m0 + lr, g.M - 1) * g.K;
    const uint8_t *pb = g.b + min(n0 + lr, g.N - 1) * g.K;
    v16f acc;
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = 0.0f;
    const v4i zero = {0, 0, 0, 0};
    for (int64_t k0 = 0; k0 < g.K; k0 += 64) {
        const int64_t k = k0 + 32 * lg;                         // K % 16 == 0: each 16-byte chunk is wholly in or out
        const v4i a_lo = k < g.K ? *reinterpret_cast<const v4i *>(pa + k) : zero;
        const v4i a_hi = k + 16 < g.K ? *reinterpret_cast<const v4i *>(pa + k + 16) : zero;
        const v4i b_lo = k < g.K ? *reinterpret_cast<const v4i *>(pb + k) : zero;
        const v4i b_hi = k + 16 < g.K ? *reinterpret_cast<const v4i *>(pb + k + 16) : zero;
        const v8i af = {a_lo.x, a_lo.y, a_lo.z, a_lo.w, a_hi.x, a_hi.y, a_hi.z, a_hi.w};
        const v8i bf = {b_lo.x, b_lo.y, b_lo.z, b_lo.w, b_hi.x, b_hi.y, b_hi.z, b_hi.w};
        acc = mfma_32x32x64<FB, FA>(bf, af, acc);
    }
    if (g.out_dtype == ODL_BF16) store_tile<true, false>(g, acc, m0 + lr, n0 + 4 * lg);
    else store_tile<false, false>(g, acc, m0 + lr, n0 + 4 * lg);
}

// ---------------------------------------------------------------- sum of K splits
// out[m, n] = ((p_0 + p_1) + ... + p_{S-1})[m, n] * (sa[m] * sb[n]) (+ bias[n]), fp32 throughout, one
// rounding to the output type; the partial results are added in split order, so the result does not
// depend on how the splits were scheduled.  Four consecutive columns per lane (N % 4 == 0).
template <bool OUT_BF16>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float *__restrict__ parts, int splits, int64_t M, int64_t N,
                                                            const float *__restrict__ sa, int sa_vec, const float *__restrict__ sb,
                                                            int sb_vec, const float *__restrict__ bias, void *__restrict__ out,
                                                            int accumulate) {
    const int64_t quads = M * N / 4, slice = M * N;
    for (int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; q < quads; q += (int64_t)gridDim.x * blockDim.x) {
        const int64_t e = q * 4, m = e / N, n = e % N;
        typedef float f32x4 __attribute__((ext_vector_type(4)));
        f32x4 acc = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(parts + e));
        for (int s = 1; s < splits; ++s) {
            const f32x4 p = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(parts + s * slice + e));
            acc.x = acc.x + p.x; acc.y = acc.y + p.y; acc.z = acc.z + p.z; acc.w = acc.w + p.w;
        }
        const float a = sa[m * sa_vec];
        float v[4] = {acc.x * (a * sb[n * sb_vec]), acc.y * (a * sb[(n + 1) * sb_vec]), acc.z * (a * sb[(n + 2) * sb_vec]),
                      acc.w * (a * sb[(n + 3) * sb_vec])};
        if (bias) {
#pragma unroll
            for (int j = 0; j < 4; ++j) v[j] = v[j] + bias[n + j];
        }
        if constexpr (OUT_BF16) {
            u32x2 *dst = reinterpret_cast<u32x2 *>(reinterpret_cast<uint16_t *>(out) + e);
            if (accumulate) {                          // out = out + product: the old value joins the fp32 sum, one rounding
                const u32x2 old = *dst;
                v[0] = v[0] + bf16_lo(old.x); v[1] = v[1] + bf16_hi(old.x); v[2] = v[2] + bf16_lo(old.y); v[3] = v[3] + bf16_hi(old.y);
            }
            *dst = u32x2{pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
        } else {
            float4 *dst = reinterpret_cast<float4 *>(reinterpret_cast<float *>(out) + e);
            if (accumulate) {
                const float4 old = *dst;
                v[0] = v[0] + old.x; v[1] = v[1] + old.y; v[2] = v[2] + old.z; v[3] = v[3] + old.w;
            }
            *dst = float4{v[0], v[1], v[2], v[3]};
        }
    }
}

// ------------------------------------------------------------------- host side
struct Variant {
    const char *name;
    int bm, bn, threads;     // bm == 0: generic kernel
    float eff;               // relative per-tile efficiency used by the automatic choice
};

static const Variant kVariants[] = {
    {"generic 32x32 (1 wave, no LDS)", 0, 0, 64, 0.05f},
    {"256x256x128 4 waves (128x128 per wave)", 256, 256, 256, 0.25f},
    {"256x256x128 8 waves (128x64 per wave)", 256, 256, 512, 1.00f},
    {"256x128x128 4 waves (128x64 per wave)", 256, 128, 256, 0.85f},
    {"128x128x128 4 waves (64x64 per wave)", 128, 128, 256, 0.70f},
    {"256x256x128 4 waves, software-pipelined, persistent (K % 256 == 0)", 256, 256, 256, 1.10f},
    {"256x256x128 4 waves, software-pipelined, one tile per block", 256, 256, 256, 0.50f},
    {"256x256x128 4 waves, streaming across tiles, folded epilogue (M, N, K multiples of 128)", 256, 256, 256, 1.25f},
};
constexpr int kPipeVariant = 5, kPipeOneTileVariant = 6, kStreamVariant = 7;
constexpr int kNumVariants = sizeof(kVariants) / sizeof(kVariants[0]);
// Forced kernel variant of the calling host thread (-1: choose by shape).  Thread-local: a test or a tuning
// sweep that pins a variant cannot change the kernels another thread (e.g. the autograd worker) launches.
static thread_local int t_forced_variant = -1;
// Clock probe of the calling host thread (see odl_fp8_gemm_set_clock_probe): launch i of the streaming kernel writes
// record i % capacity.
static thread_local unsigned long long *t_clock_probe = nullptr;
static thread_local int t_clock_capacity = 0, t_clock_next = 0;

template <int FA, int FB>
static void launch_generic_fmt(const GemmArgs &g, hipStream_t stream) {
    hipLaunchKernelGGL((gemm_nt_generic_kernel<FA, FB>), dim3((unsigned)(g.tiles_m * g.tiles_n)), dim3(64), 0, stream, g);
}

static void launch_gemm_generic(int fa, int fb, const GemmArgs &g, hipStream_t stream) {
    if (fa == ODL_FP8_E4M3 && fb == ODL_FP8_E4M3) launch_generic_fmt<ODL_FP8_E4M3, ODL_FP8_E4M3>(g, stream);
    else if (fa == ODL_FP8_E5M2 && fb == ODL_FP8_E4M3) launch_generic_fmt<ODL_FP8_E5M2, ODL_FP8_E4M3>(g, stream);
    else if (fa == ODL_FP8_E4M3 && fb == ODL_FP8_E5M2) launch_generic_fmt<ODL_FP8_E4M3, ODL_FP8_E5M2>(g, stream);
    else launch_generic_fmt<ODL_FP8_E5M2, ODL_FP8_E5M2>(g, stream);
}

static int cu_count() { return device_cu_count(); }

static int choose_variant(int64_t M, int64_t N, bool stream_ok) {
    const int cus = cu_count();
    // an output of at most cus / 2 tiles of 256 x 256 leaves half the chip idle with the big tiles: the 128 x 128
    // kernel (two blocks per compute unit) spreads it four times wider (measured 15-20 % faster than either
    // 256-wide kernel at 8192 x 1024, 8192 x 768 and 2048 x 4096 outputs, K = 768 .. 4096)
    if (((M + 255) / 256) * ((N + 255) / 256) * 2 <= cus) return 4;
    int best = 2;
    double best_score = -1.0;
    for (int v = 2; v < kNumVariants; ++v) {                       // variant 1 (one wave per SIMD) only by explicit request
        if (v == kStreamVariant && !stream_ok) continue;
        const Variant &cfg = kVariants[v];
        const int64_t tiles = ((M + cfg.bm - 1) / cfg.bm) * ((N + cfg.bn - 1) / cfg.bn);
        const int per_cu = cfg.bm * cfg.bn >= 256 * 256 ? 1 : (cfg.bm * cfg.bn >= 256 * 128 ? 1 : 2);
        const int64_t slots = (int64_t)cus * per_cu;
        const int64_t rounds = (tiles + slots - 1) / slots;
        const double useful = (double)M * N / ((double)rounds * slots * cfg.bm * cfg.bn);
        const double score = useful * cfg.eff;
        if (score > best_score) { best_score = score; best = v; }
    }
    return best;
}

}  // namespace odl

using namespace odl;

extern "C" int odl_fp8_gemm_num_variants(void) { return kNumVariants; }

extern "C" const char *odl_fp8_gemm_variant_name(int variant) {
    return (variant >= 0 && variant < kNumVariants) ? kVariants[variant].name : "";
}

void odl::launch_splitk_reduce(const float *workspace, int splits, int64_t M, int64_t N, const float *sa, int sa_vec, const float *sb,
                               int sb_vec, const float *bias, void *c, int out_dtype, int accumulate, hipStream_t stream) {
    const int64_t quads = M * N / 4;
    int64_t blocks = (quads + 255) / 256;
    if (blocks > 4 * (int64_t)cu_count()) blocks = 4 * (int64_t)cu_count();
    if (out_dtype == ODL_BF16)
        hipLaunchKernelGGL((splitk_reduce_kernel<true>), dim3((unsigned)blocks), dim3(256), 0, stream, workspace, splits, M, N, sa, sa_vec, sb,
                           sb_vec, bias, c, accumulate);
    else
        hipLaunchKernelGGL((splitk_reduce_kernel<false>), dim3((unsigned)blocks), dim3(256), 0, stream, workspace, splits, M, N, sa, sa_vec, sb,
                           sb_vec, bias, c, accumulate);
}

void odl::attach_clock_probe(GemmArgs &g) {
    if (!t_clock_probe) return;
    g.clock_out = t_clock_probe + 4 * (size_t)(t_clock_next % t_clock_capacity);
    ++t_clock_next;
}

#ifndef ODL_FP8_NO_BENCH_HOOKS
extern "C" int odl_fp8_gemm_set_clock_probe(uint64_t *records_dev, int capacity) {
    if (records_dev && capacity < 1) return set_error(ODL_ERR_ARG, "odl_fp8_gemm_set_clock_probe: capacity %d", capacity);
    t_clock_probe = reinterpret_cast<unsigned long long *>(records_dev);
    t_clock_capacity = records_dev ? capacity : 0;
    t_clock_next = 0;
    return ODL_OK;
}
#endif

extern "C" int odl_fp8_gemm_set_variant(int variant) {
    if (variant < -1 || variant >= kNumVariants) return set_error(ODL_ERR_ARG, "odl_fp8_gemm_set_variant: %d out of range", variant);
    t_forced_variant = variant;
    return ODL_OK;
}

extern "C" int odl_fp8_gemm_nt(const uint8_t *a, const uint8_t *b, int64_t M, int64_t N, int64_t K, int fmt_a, int fmt_b,
                               const float *sa_inv, int64_t sa_n, const float *sb_inv, int64_t sb_n, const void *bias,
                               int bias_dtype, void *c, int out_dtype, int accumulate, odl_stream_t stream_) {
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    if (!a || !b || !c || !sa_inv || !sb_inv) return set_error(ODL_ERR_ARG, "odl_fp8_gemm_nt: null pointer");
    if (M < 0 || N < 0 || K < 0) return set_error(ODL_ERR_ARG, "odl_fp8_gemm_nt: negative size");
    if ((fmt_a != ODL_FP8_E4M3 && fmt_a != ODL_FP8_E5M2) || (fmt_b != ODL_FP8_E4M3 && fmt_b != ODL_FP8_E5M2))
        return set_error(ODL_ERR_ARG, "odl_fp8_gemm_nt: formats %d, %d", fmt_a, fmt_b);
    if (sa_n != 1 && sa_n != M) return set_error(ODL_ERR_ARG, "odl_fp8_gemm_nt: sa_n=%lld is neither 1 nor M", (long long)sa_n);
    if (sb_n != 1 && sb_n != N) return set_error(ODL_ERR_ARG, "odl_fp8_gemm_nt: sb_n=%lld is neither 1 nor N", (long long)sb_n);
    if (out_dtype != ODL_BF16 && out_dtype != ODL_F32) return set_error(ODL_ERR_ARG, "odl_fp8_gemm_nt: out_dtype %d", out_dtype);
    if (bias && bias_dtype != ODL_F32) return set_error(ODL_ERR_ARG, "odl_fp8_gemm_nt: bias must be fp32 (bias_dtype %d)", bias_dtype);
    if (K % 16 != 0) return set_error(ODL_ERR_SHAPE, "odl_fp8_gemm_nt: K=%lld must be a multiple of 16", (long long)K);
    if ((reinterpret_cast<uintptr_t>(a) & 15) || (reinterpret_cast<uintptr_t>(b) & 15))
        return set_error(ODL_ERR_SHAPE, "odl_fp8_gemm_nt: operands must be 16-byte aligned");
    if (reinterpret_cast<uintptr_t>(c) & 15) return set_error(ODL_ERR_SHAPE, "odl_fp8_gemm_nt: output must be 16-byte aligned");
    if ((sa_n > 1 && (reinterpret_cast<uintptr_t>(sa_inv) & 15)) || (sb_n > 1 && (reinterpret_cast<uintptr_t>(sb_inv) & 15)) ||
        (bias && (reinterpret_cast<uintptr_t>(bias) & 15)))
        return set_error(ODL_ERR_SHAPE, "odl_fp8_gemm_nt: scale vectors and bias must be 16-byte aligned");
    if (M == 0 || N == 0) return ODL_OK;

    const bool tiled_ok = K >= 128 && K % 128 == 0 && (double)M * (double)K < 4294967296.0 && (double)N * (double)K < 4294967296.0;
    // the pipelined and the streaming kernel address rows with 32-bit byte offsets
    const bool lim32 = (double)(M + 256) * (double)K < 2147483648.0 && (double)(N + 256) * (double)K < 2147483648.0;
    // C = C + product is an epilogue of the kernels whose tiles end in a separate output phase; the streaming kernel
    // stores a tile under the next tile's MFMAs, where nothing can wait for the old values of C
    const bool stream_ok = tiled_ok && lim32 && M % 128 == 0 && N % 128 == 0 && K >= 512 && !accumulate;
    int variant = t_forced_variant >= 0 ? t_forced_variant : (tiled_ok ? choose_variant(M, N, stream_ok) : 0);
    if (variant != 0 && !tiled_ok) variant = 0;
    // the pipelined kernel walks K in pairs of 128-byte steps
    const bool pipe_ok = tiled_ok && K % 256 == 0 && lim32;
    if ((variant == kPipeVariant || variant == kPipeOneTileVariant) && !pipe_ok) variant = 2;

    GemmArgs g;
    g.a = a; g.b = b; g.c = c; g.sa = sa_inv; g.sb = sb_inv; g.bias = bias;
    g.M = M; g.N = N; g.K = K;
    g.sa_vec = sa_n == M && M != 1;
    g.sb_vec = sb_n == N && N != 1;
    g.out_dtype = out_dtype;
    g.accumulate = accumulate != 0;
    const int bm = variant == 0 ? 32 : kVariants[variant].bm, bn = variant == 0 ? 32 : kVariants[variant].bn;
    const int64_t tm = (M + bm - 1) / bm, tn = (N + bn - 1) / bn;
    if (tm * tn > 0x7ffffff0LL) return set_error(ODL_ERR_SHAPE, "odl_fp8_gemm_nt: too many tiles");
    g.tiles_m = (int)tm; g.tiles_n = (int)tn;

    if (variant == kStreamVariant && !(stream_ok && gemm_stream_accepts(g))) {
        // the streaming kernel wants M, N in multiples of 128: next best kernel instead
        variant = pipe_ok ? kPipeVariant : 2;
    }
    if (variant == 0) launch_gemm_generic(fmt_a, fmt_b, g, stream);
    else if (variant == kPipeVariant) launch_gemm_pipe(fmt_a, fmt_b, g, cu_count(), stream);
    else if (variant == kPipeOneTileVariant) launch_gemm_pipe(fmt_a, fmt_b, g, 1 << 30, stream);
    else if (variant == kStreamVariant) { attach_clock_probe(g); launch_gemm_stream(fmt_a, fmt_b, g, cu_count(), stream); }
    else launch_gemm_tiled(variant, fmt_a, fmt_b, g, stream);
    return check_launch("odl_fp8_gemm_nt");
}

extern "C" int odl_fp8_gemm_nt_sum(int pairs, const uint8_t *const *a, const uint8_t *const *b, const int64_t *K, int64_t M, int64_t N,
                                   int fmt_a, int fmt_b, const float *const *sa_inv, const float *const *sb_inv, void *c,
                                   int out_dtype, odl_stream_t stream_) {
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    if (pairs < 1 || pairs > 64) return set_error(ODL_ERR_ARG, "odl_fp8_gemm_nt_sum: %d operand pairs (1 .. 64)", pairs);
    if (!a || !b || !K || !sa_inv || !sb_inv || !c) return set_error(ODL_ERR_ARG, "odl_fp8_gemm_nt_sum: null pointer");
    if (M < 0 || N < 0) return set_error(ODL_ERR_ARG, "odl_fp8_gemm_nt_sum: negative size");
    if ((fmt_a != ODL_FP8_E4M3 && fmt_a != ODL_FP8_E5M2) || (fmt_b != ODL_FP8_E4M3 && fmt_b != ODL_FP8_E5M2))
        return set_error(ODL_ERR_ARG, "odl_fp8_gemm_nt_sum: formats %d, %d", fmt_a, fmt_b);
    if (out_dtype != ODL_BF16 && out_dtype != ODL_F32) return set_error(ODL_ERR_ARG, "odl_fp8_gemm_nt_sum: out_dtype %d", out_dtype);
    for (int s = 0; s < pairs; ++s) {
        if (!a[s] || !b[s] || !sa_inv[s] || !sb_inv[s]) return set_error(ODL_ERR_ARG, "odl_fp8_gemm_nt_sum: null pointer in pair %d", s);
        if (K[s] <= 0 || K[s] % 16 != 0)
            return set_error(ODL_ERR_SHAPE, "odl_fp8_gemm_nt_sum: K[%d]=%lld must be a positive multiple of 16", s, (long long)K[s]);
        if ((reinterpret_cast<uintptr_t>(a[s]) & 15) || (reinterpret_cast<uintptr_t>(b[s]) & 15))
            return set_error(ODL_ERR_SHAPE, "odl_fp8_gemm_nt_sum: operands must be 16-byte aligned (pair %d)", s);
    }
    if (reinterpret_cast<uintptr_t>(c) & 15) return set_error(ODL_ERR_SHAPE, "odl_fp8_gemm_nt_sum: output must be 16-byte aligned");
    if (M == 0 || N == 0) return ODL_OK;

    // one launch of the streaming kernel when every pair suits it ...
    if (pairs <= 4 && (t_forced_variant < 0 || t_forced_variant == kStreamVariant)) {
        GemmArgs g;
        GemmPairs gp;
        g.a = a[0]; g.b = b[0]; g.c = c; g.sa = sa_inv[0]; g.sb = sb_inv[0]; g.bias = nullptr;
        g.M = M; g.N = N; g.K = K[0];
        g.sa_vec = 0; g.sb_vec = 0;
        g.out_dtype = out_dtype;
        g.tiles_m = (int)((M + 255) / 256); g.tiles_n = (int)((N + 255) / 256);
        gp.count = pairs;
        bool fits = true;
        for (int s = 0; s < pairs; ++s) {
            fits = fits && K[s] < 2147483648LL;
            gp.k[s] = (int)K[s]; gp.a[s] = a[s]; gp.b[s] = b[s]; gp.sa[s] = sa_inv[s]; gp.sb[s] = sb_inv[s];
        }
        if (fits && (pairs > 1 || t_forced_variant == kStreamVariant) && gemm_stream_accepts_pairs(g, gp)) {
            launch_gemm_stream_pairs(fmt_a, fmt_b, g, gp, cu_count(), stream);
            return check_launch("odl_fp8_gemm_nt_sum");
        }
    }
    // ... otherwise a GEMM per pair, the second and later ones adding into C (one rounding to the output type per pair)
    for (int s = 0; s < pairs; ++s) {
        const int rc = odl_fp8_gemm_nt(a[s], b[s], M, N, K[s], fmt_a, fmt_b, sa_inv[s], 1, sb_inv[s], 1, nullptr, ODL_F32, c, out_dtype,
                                       s > 0, stream_);
        if (rc != ODL_OK) return rc;
    }
    return ODL_OK;
}

extern "C" int odl_fp8_gemm_layouts(const uint8_t *a, const uint8_t *b, int64_t M, int64_t N, int64_t K, int fmt_a, int fmt_b,
                                    int layout_a, int layout_b, const float *sa_inv, const float *sb_inv, void *c,
                                    int out_dtype, odl_stream_t stream_) {
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    if (!a || !b || !c || !sa_inv || !sb_inv) return set_error(ODL_ERR_ARG, "odl_fp8_gemm_layouts: null pointer");
    if ((fmt_a != ODL_FP8_E4M3 && fmt_a != ODL_FP8_E5M2) || (fmt_b != ODL_FP8_E4M3 && fmt_b != ODL_FP8_E5M2))
        return set_error(ODL_ERR_ARG, "odl_fp8_gemm_layouts: formats %d, %d", fmt_a, fmt_b);
    if ((layout_a != ODL_K_FAST && layout_a != ODL_K_SLOW) || (layout_b != ODL_K_FAST && layout_b != ODL_K_SLOW))
        return set_error(ODL_ERR_ARG, "odl_fp8_gemm_layouts: layouts %d, %d", layout_a, layout_b);
    if (out_dtype != ODL_BF16 && out_dtype != ODL_F32) return set_error(ODL_ERR_ARG, "odl_fp8_gemm_layouts: out_dtype %d", out_dtype);
    if ((reinterpret_cast<uintptr_t>(a) & 15) || (reinterpret_cast<uintptr_t>(b) & 15) || (reinterpret_cast<uintptr_t>(c) & 15))
        return set_error(ODL_ERR_SHAPE, "odl_fp8_gemm_layouts: operands and output must be 16-byte aligned");
    GemmArgs g;
    g.a = a; g.b = b; g.c = c; g.sa = sa_inv; g.sb = sb_inv; g.bias = nullptr;
    g.M = M; g.N = N; g.K = K;
    g.sa_vec = 0; g.sb_vec = 0;
    g.out_dtype = out_dtype;
    g.ta = layout_a == ODL_K_SLOW;
    g.tb = layout_b == ODL_K_SLOW;
    const bool sizes_ok = M > 0 && N > 0 && K >= 512 && M % 256 == 0 && N % 256 == 0 && K % 256 == 0 &&
                          (double)(M + 256) * (double)K < 2147483648.0 && (double)(N + 256) * (double)K < 2147483648.0;
    if (!sizes_ok) return set_error(ODL_ERR_SHAPE, "odl_fp8_gemm_layouts: M, N, K must be multiples of 256 (K >= 512) and each operand under 2 GiB; got %lld x %lld x %lld", (long long)M, (long long)N, (long long)K);
    g.tiles_m = (int)(M / 256); g.tiles_n = (int)(N / 256);
    if (!gemm_stream_accepts(g)) return set_error(ODL_ERR_SHAPE, "odl_fp8_gemm_layouts: shape not taken by the streaming kernel");
    attach_clock_probe(g);
    launch_gemm_stream(fmt_a, fmt_b, g, cu_count(), stream);
    return check_launch("odl_fp8_gemm_layouts");
}

// How many runs to cut K into for an output of few tiles (1 = do not split).  A model in microseconds, fitted to
// measurements on this GPU (outputs 768 x 768 .. 8192 x 1024, K = 8192 .. 151936):
//   one launch, 256 x 256 tiles : 0.92 us per K step of 128 (few compute units busy: high clock) + 3 steps of overhead
//   one launch, 128 x 128 tiles : 0.55 us per step where every block has a compute unit to itself (the four-stage form
//                                 of the kernel), 0.62 with two blocks per unit (what odl_fp8_gemm_nt takes for outputs
//                                 of <= cus / 2 big tiles); it reads every operand panel twice as often
//   split                       : 0.96 us per step of a run + 9 us (pipeline fill, the fp32 epilogue, the second launch)
//                                 + the partial results, splits x M x N floats written and read back, at 2.7 TB/s in all
//   each bounded below by its operand traffic (tiles x panel bytes) at about 12 TB/s out of the caches.
// The runs of a split must fit the compute units at once, and a split must win by 10 %.
// k_slow: an operand is stored with the contraction index slow (odl_fp8_gemm_layouts), which only the streaming
// kernel reads: the 128 x 128 kernel is then not an alternative.
extern "C" int odl_fp8_gemm_split_count(int64_t M, int64_t N, int64_t K, int k_slow) {
    if (M <= 0 || N <= 0 || M % 128 || N % 128 || K % 128 || K < 2048) return 1;
    const int64_t tiles = ((M + 255) / 256) * ((N + 255) / 256);
    const int cus = cu_count();
    const int64_t steps = K / 128;
    int64_t most = cus / tiles;
    if (most > 16) most = 16;
    const double traffic_us = (double)tiles * 512.0 * (double)K / 12.0e6;
    double whole = 0.92 * ((double)steps + 3.0);
    if (whole < traffic_us) whole = traffic_us;
    if (tiles * 2 <= cus && !k_slow) {
        const int64_t small_tiles = ((M + 127) / 128) * ((N + 127) / 128);
        double small = (small_tiles <= cus ? 0.55 : 0.62) * ((double)steps + 3.0);
        const double small_traffic_us = (double)small_tiles * 256.0 * (double)K / 12.0e6;
        if (small < small_traffic_us) small = small_traffic_us;
        if (small < whole) whole = small;
    }
    double best = whole;
    int best_splits = 1;
    for (int64_t splits = 2; splits <= most; ++splits) {
        const int64_t per = ((steps + splits - 1) / splits + 1) & ~(int64_t)1;
        const int64_t last = steps - (splits - 1) * per;
        if (per < 8 || last < 4) continue;
        double run = 0.96 * (double)per + 9.0;
        if (run < traffic_us) run = traffic_us;
        const double cost = run + (double)splits * (double)M * (double)N * 4.0 / 2.7e6;
        if (cost < 0.90 * whole && cost < best) { best = cost; best_splits = (int)splits; }
    }
    return best_splits;
}

extern "C" int odl_fp8_gemm_splitk(const uint8_t *a, const uint8_t *b, int64_t M, int64_t N, int64_t K, int fmt_a, int fmt_b,
                                   int layout_a, int layout_b, const float *sa_inv, int64_t sa_n, const float *sb_inv,
                                   int64_t sb_n, const float *bias, void *c, int out_dtype, int accumulate, int splits, void *workspace,
                                   int64_t workspace_bytes, odl_stream_t stream_) {
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    if (!a || !b || !c || !sa_inv || !sb_inv || !workspace) return set_error(ODL_ERR_ARG, "odl_fp8_gemm_splitk: null pointer");
    if ((fmt_a != ODL_FP8_E4M3 && fmt_a != ODL_FP8_E5M2) || (fmt_b != ODL_FP8_E4M3 && fmt_b != ODL_FP8_E5M2))
        return set_error(ODL_ERR_ARG, "odl_fp8_gemm_splitk: formats %d, %d", fmt_a, fmt_b);
    if ((layout_a != ODL_K_FAST && layout_a != ODL_K_SLOW) || (layout_b != ODL_K_FAST && layout_b != ODL_K_SLOW))
        return set_error(ODL_ERR_ARG, "odl_fp8_gemm_splitk: layouts %d, %d", layout_a, layout_b);
    if (out_dtype != ODL_BF16 && out_dtype != ODL_F32) return set_error(ODL_ERR_ARG, "odl_fp8_gemm_splitk: out_dtype %d", out_dtype);
    if (sa_n != 1 && sa_n != M) return set_error(ODL_ERR_ARG, "odl_fp8_gemm_splitk: sa_n=%lld is neither 1 nor M", (long long)sa_n);
    if (sb_n != 1 && sb_n != N) return set_error(ODL_ERR_ARG, "odl_fp8_gemm_splitk: sb_n=%lld is neither 1 nor N", (long long)sb_n);
    if ((reinterpret_cast<uintptr_t>(a) & 15) || (reinterpret_cast<uintptr_t>(b) & 15) || (reinterpret_cast<uintptr_t>(c) & 15) ||
        (reinterpret_cast<uintptr_t>(workspace) & 15))
        return set_error(ODL_ERR_SHAPE, "odl_fp8_gemm_splitk: operands, output and workspace must be 16-byte aligned");
    const int ta = layout_a == ODL_K_SLOW, tb = layout_b == ODL_K_SLOW;
    const bool sizes_ok = M > 0 && N > 0 && M % (ta ? 256 : 128) == 0 && N % (tb ? 256 : 128) == 0 && K % 128 == 0 &&
                          (double)(M + 256) * (double)K < 2147483648.0 && (double)(N + 256) * (double)K < 2147483648.0;
    if (!sizes_ok)
        return set_error(ODL_ERR_SHAPE, "odl_fp8_gemm_splitk: M, N, K must be multiples of 128 (256 for an operand stored K-slow) and each operand under 2 GiB; got %lld x %lld x %lld", (long long)M, (long long)N, (long long)K);
    const int64_t steps = K / 128;
    const int64_t per = ((steps + splits - 1) / (splits > 0 ? splits : 1) + 1) & ~(int64_t)1;
    // what the kernel needs to be correct: every run at least four K steps (its load pipeline is two steps deep and runs
    // in pairs).  odl_fp8_gemm_split_count proposes only runs of eight steps and more, which is where a split pays.
    // one "run" is allowed with accumulate: the way to add a product with an operand stored K-slow into C
    if (splits < (accumulate ? 1 : 2) || splits > 64 || per < 4 || steps - (splits - 1) * per < 4)
        return set_error(ODL_ERR_ARG, "odl_fp8_gemm_splitk: %d splits of K=%lld leave a run shorter than 512 (or fewer than 2 splits without accumulate)", splits, (long long)K);
    if (workspace_bytes < (int64_t)splits * M * N * 4)
        return set_error(ODL_ERR_ARG, "odl_fp8_gemm_splitk: workspace of %lld bytes, %lld needed", (long long)workspace_bytes,
                         (long long)splits * M * N * 4);
    GemmArgs g;
    g.a = a; g.b = b; g.c = workspace; g.sa = sa_inv; g.sb = sb_inv; g.bias = nullptr;
    g.M = M; g.N = N; g.K = K;
    g.sa_vec = 0; g.sb_vec = 0;
    g.out_dtype = ODL_F32;
    g.ta = ta; g.tb = tb;
    g.splits = splits; g.split_steps = (int)per;
    g.tiles_m = (int)((M + 255) / 256); g.tiles_n = (int)((N + 255) / 256);
    if (!gemm_stream_accepts(g)) return set_error(ODL_ERR_SHAPE, "odl_fp8_gemm_splitk: shape not taken by the streaming kernel");
    attach_clock_probe(g);
    launch_gemm_stream(fmt_a, fmt_b, g, cu_count(), stream);
    const int sa_vec = sa_n == M && M != 1, sb_vec = sb_n == N && N != 1;
    if (splits == 1) {
        // a single run is an ordinary launch: the kernel applies the tensor scales itself, the second kernel adds C
        const float *one = unit_scale_for_current_device("odl_fp8_gemm_splitk");
        if (!one) return ODL_ERR_LAUNCH;
        launch_splitk_reduce((const float *)workspace, 1, M, N, one, 0, one, 0, bias, c, out_dtype, accumulate != 0, stream);
        return check_launch("odl_fp8_gemm_splitk");
    }
    launch_splitk_reduce((const float *)workspace, splits, M, N, sa_inv, sa_vec, sb_inv, sb_vec, bias, c, out_dtype, accumulate != 0, stream);
    return check_launch("odl_fp8_gemm_splitk");
}
