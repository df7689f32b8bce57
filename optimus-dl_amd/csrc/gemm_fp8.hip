// FP8 GEMM for gfx950 on the f8f6f4 MFMA units.
//
//   C[M,N] = (A[M,K] . B[N,K]^T) * (sa_inv[i] * sb_inv[j]) (+ bias[j])
//
// Both operands are K-contiguous 8-bit codes ("NT"), which is what the MFMA
// wants: each lane feeds 32 consecutive K-bytes of one row.  fwd, dgrad and
// wgrad of the Linear all arrive in this form because the cast+transpose kernel
// has already produced the K-major copies.
//
// Tiled kernel (the fast path):
//   * block tile BM x BN, K step 128 bytes, two LDS stages (2 x (BM+BN) x 128 B);
//   * global -> LDS with global_load_lds_dwordx4 (no VGPR round trip).  One wave
//     instruction fills 8 rows x 128 B; the 16-byte chunks of a row are stored
//     XOR-swizzled (chunk ^ f(row)) by permuting the *global* addresses, so the
//     later 128-bit LDS reads of 32 different rows hit different banks;
//   * V_MFMA_F32_32X32X64_F8F6F4, operands swapped (B first) so every lane ends
//     up with 4 consecutive output columns of one row -> 8-byte bf16 stores;
//   * the two stages are separate __shared__ objects and the K loop is unrolled
//     by two, so the compiler can prove that the loads in flight into one stage
//     do not alias the LDS reads of the other (no vmcnt stall in front of them);
//   * block id -> tile mapping is XCD-aware: ids are dealt round-robin to the 8
//     XCDs by the hardware, so tile = (id % 8) * chunk + id / 8 keeps each XCD on
//     a contiguous run of tiles, walked in groups of GM rows for L2 reuse.
// Generic kernel: one wave per 32x32 tile straight from global memory; any
// M, N and K % 16 == 0.  Used for shapes the tiled kernel refuses.
#include "common.h"

namespace odl {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

struct GemmArgs {
    const uint8_t *a, *b;
    void *c;
    const float *sa, *sb;
    const void *bias;
    int64_t M, N, K;
    int sa_vec, sb_vec;          // 0 = one value, 1 = one per row of A / B
    int out_dtype;               // bias, when present, is fp32
    int tiles_m, tiles_n;
};

__device__ __forceinline__ int swz(int row) { return (row ^ (row >> 3)) & 7; }

// D[i][j] += sum_k first[i][k] * second[j][k]; lane l supplies row l%32 and the
// K-bytes [32*(l/32), +32) of both operands.  F1 / F2: 0 = E4M3, 1 = E5M2.
template <int F1, int F2>
__device__ __forceinline__ v16f mfma_32x32x64(v8i first, v8i second, v16f acc) {
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(first, second, acc, F1, F2, 0, 0, 0, 0);
}

// Epilogue for one 32x32 accumulator tile in the swapped layout: this lane holds
// row m and columns n_base + 8*q + {0..3}, q = 0..3, in acc[4q .. 4q+3].
// value = acc * (sa_inv[m] * sb_inv[n]) (+ bias[n]), each step rounded to fp32,
// then one rounding to the output type.  sa/sb are read with stride 0 (one value)
// or 1 (one per row / column), which removes the per-element branch.
// INTERIOR: the whole block tile is inside the matrix and N % 4 == 0, so no
// bounds checks and vector stores throughout.
template <bool OUT_BF16, bool INTERIOR>
__device__ __forceinline__ void store_tile(const GemmArgs &g, const v16f &acc, int64_t m, int64_t n_base) {
    if (!INTERIOR && m >= g.M) return;
    const float sa = g.sa[m * g.sa_vec];
    const float *bias = reinterpret_cast<const float *>(g.bias);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const int64_t n = n_base + 8 * q;
        if (!INTERIOR && n >= g.N) continue;
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int64_t ne = (INTERIOR || n + e < g.N) ? n + e : g.N - 1;
            const float s = sa * g.sb[ne * g.sb_vec];
            v[e] = acc[4 * q + e] * s;
            if (bias) v[e] = v[e] + bias[ne];
        }
        if constexpr (OUT_BF16) {
            uint16_t *c = reinterpret_cast<uint16_t *>(g.c) + m * g.N + n;
            if (INTERIOR || (n + 3 < g.N && (g.N & 3) == 0)) {
                u32x2 pk = {f32_to_bf16_bits(v[0]) | (f32_to_bf16_bits(v[1]) << 16),
                            f32_to_bf16_bits(v[2]) | (f32_to_bf16_bits(v[3]) << 16)};
                *reinterpret_cast<u32x2 *>(c) = pk;
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (n + e < g.N) c[e] = (uint16_t)f32_to_bf16_bits(v[e]);
            }
        } else {
            float *c = reinterpret_cast<float *>(g.c) + m * g.N + n;
            if (INTERIOR || (n + 3 < g.N && (g.N & 3) == 0)) {
                *reinterpret_cast<float4 *>(c) = float4{v[0], v[1], v[2], v[3]};
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (n + e < g.N) c[e] = v[e];
            }
        }
    }
}

// ------------------------------------------------------------------ tiled kernel
template <int BM, int BN, int WAVES_M, int WAVES_N, int FA, int FB>
__global__ __launch_bounds__(WAVES_M *WAVES_N * 64) void gemm_nt_tiled_kernel(const GemmArgs g) {
    constexpr int NW = WAVES_M * WAVES_N;
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N, TM = WM / 32, TN = WN / 32;
    constexpr int A_BYTES = BM * 128, B_BYTES = BN * 128, STAGE = A_BYTES + B_BYTES;
    constexpr int LA = BM / 8 / NW, LB = BN / 8 / NW;    // 1 KB load instructions per wave per stage
    constexpr int GM = 8;                                 // tile rows walked together
    static_assert(BM % (8 * NW) == 0 && BN % (8 * NW) == 0, "tile rows must split evenly over the waves");
    static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile must be a multiple of the 32x32 MFMA");

    __shared__ __attribute__((aligned(1024))) uint8_t lds0[STAGE];
    __shared__ __attribute__((aligned(1024))) uint8_t lds1[STAGE];

    // ---- which tile (XCD-aware, grouped)
    const int total = g.tiles_m * g.tiles_n;
    const int per_xcd = (total + 7) / 8;
    const int pid = (int)(blockIdx.x % 8) * per_xcd + (int)(blockIdx.x / 8);
    if (pid >= total) return;
    const int in_group = GM * g.tiles_n;
    const int first_m = (pid / in_group) * GM;
    const int group_rows = min(g.tiles_m - first_m, GM);
    const int tile_m = first_m + (pid % in_group) % group_rows;
    const int tile_n = (pid % in_group) / group_rows;
    const int64_t m0 = (int64_t)tile_m * BM, n0 = (int64_t)tile_n * BN;

    const int lane = threadIdx.x % 64;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    const int wm0 = (wave / WAVES_N) * WM, wn0 = (wave % WAVES_N) * WN;
    const int KT = (int)(g.K / 128);

    // ---- global -> LDS: per-lane source offsets (rows past the edge re-read the last row)
    uint32_t off_a[LA], off_b[LB];
#pragma unroll
    for (int j = 0; j < LA; ++j) {
        const int row = (wave + j * NW) * 8 + lane / 8;
        const int64_t gr = min(m0 + row, g.M - 1);
        off_a[j] = (uint32_t)(gr * g.K + (((lane % 8) ^ swz(row)) << 4));
    }
#pragma unroll
    for (int j = 0; j < LB; ++j) {
        const int row = (wave + j * NW) * 8 + lane / 8;
        const int64_t gr = min(n0 + row, g.N - 1);
        off_b[j] = (uint32_t)(gr * g.K + (((lane % 8) ^ swz(row)) << 4));
    }
    auto issue = [&](uint8_t *lds, int kt) {
        const uint8_t *ga = g.a + (int64_t)kt * 128, *gb = g.b + (int64_t)kt * 128;
#pragma unroll
        for (int j = 0; j < LA; ++j)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(ga + off_a[j]),
                                             (__attribute__((address_space(3))) void *)(lds + (wave + j * NW) * 1024), 16, 0, 0);
#pragma unroll
        for (int j = 0; j < LB; ++j)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(gb + off_b[j]),
                                             (__attribute__((address_space(3))) void *)(lds + A_BYTES + (wave + j * NW) * 1024), 16, 0, 0);
    };

    // ---- LDS -> MFMA operands
    const int lr = lane % 32, lg = lane / 32;
    int a_off[TM], a_sw[TM], b_off[TN], b_sw[TN];
#pragma unroll
    for (int t = 0; t < TM; ++t) { const int row = wm0 + 32 * t + lr; a_off[t] = row * 128; a_sw[t] = swz(row); }
#pragma unroll
    for (int u = 0; u < TN; ++u) { const int row = wn0 + 32 * u + lr; b_off[u] = A_BYTES + row * 128; b_sw[u] = swz(row); }

    v16f acc[TM][TN];
#pragma unroll
    for (int t = 0; t < TM; ++t)
#pragma unroll
        for (int u = 0; u < TN; ++u)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[t][u][e] = 0.0f;

    auto compute = [&](const uint8_t *lds) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int c = 4 * h + 2 * lg;                       // first of this lane's two 16-byte chunks
            v8i af[TM], bf[TN];
#pragma unroll
            for (int t = 0; t < TM; ++t) {
                const uint8_t *p = lds + a_off[t];
                const v4i lo = *reinterpret_cast<const v4i *>(p + ((c ^ a_sw[t]) << 4));
                const v4i hi = *reinterpret_cast<const v4i *>(p + (((c + 1) ^ a_sw[t]) << 4));
                af[t] = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
            }
#pragma unroll
            for (int u = 0; u < TN; ++u) {
                const uint8_t *p = lds + b_off[u];
                const v4i lo = *reinterpret_cast<const v4i *>(p + ((c ^ b_sw[u]) << 4));
                const v4i hi = *reinterpret_cast<const v4i *>(p + (((c + 1) ^ b_sw[u]) << 4));
                bf[u] = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
            }
#pragma unroll
            for (int t = 0; t < TM; ++t)
#pragma unroll
                for (int u = 0; u < TN; ++u) acc[t][u] = mfma_32x32x64<FB, FA>(bf[u], af[t], acc[t][u]);
        }
    };

    // ---- main loop, two K-steps per trip so each stage is a fixed LDS object
    issue(lds0, 0);
    for (int kt = 0; kt < KT; kt += 2) {
        __builtin_amdgcn_s_waitcnt(0x0F70);                     // vmcnt(0): my loads into lds0 have landed
        __syncthreads();                                        // everyone's have, and lds1 is no longer being read
        if (kt + 1 < KT) issue(lds1, kt + 1);
        compute(lds0);
        if (kt + 1 < KT) {
            __builtin_amdgcn_s_waitcnt(0x0F70);
            __syncthreads();
            if (kt + 2 < KT) issue(lds0, kt + 2);
            compute(lds1);
        }
    }

    // ---- epilogue (uniform choice per block: output type, interior or edge tile)
    const bool interior = m0 + BM <= g.M && n0 + BN <= g.N && (g.N & 3) == 0;
#define ODL_EPILOGUE(BF, INT)                                                                                  \
    _Pragma("unroll") for (int t = 0; t < TM; ++t) _Pragma("unroll") for (int u = 0; u < TN; ++u)              \
        store_tile<BF, INT>(g, acc[t][u], m0 + wm0 + 32 * t + lr, n0 + wn0 + 32 * u + 4 * lg)
    if (g.out_dtype == ODL_BF16) {
        if (interior) { ODL_EPILOGUE(true, true); } else { ODL_EPILOGUE(true, false); }
    } else {
        if (interior) { ODL_EPILOGUE(false, true); } else { ODL_EPILOGUE(false, false); }
    }
#undef ODL_EPILOGUE
}

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
};
constexpr int kNumVariants = sizeof(kVariants) / sizeof(kVariants[0]);
static int g_forced_variant = -1;

template <int FA, int FB>
static void launch_variant(int variant, const GemmArgs &g, hipStream_t stream) {
    const int total = g.tiles_m * g.tiles_n;
    const unsigned grid = (unsigned)(((total + 7) / 8) * 8);
    switch (variant) {
    case 1: hipLaunchKernelGGL((gemm_nt_tiled_kernel<256, 256, 2, 2, FA, FB>), dim3(grid), dim3(256), 0, stream, g); break;
    case 2: hipLaunchKernelGGL((gemm_nt_tiled_kernel<256, 256, 2, 4, FA, FB>), dim3(grid), dim3(512), 0, stream, g); break;
    case 3: hipLaunchKernelGGL((gemm_nt_tiled_kernel<256, 128, 2, 2, FA, FB>), dim3(grid), dim3(256), 0, stream, g); break;
    case 4: hipLaunchKernelGGL((gemm_nt_tiled_kernel<128, 128, 2, 2, FA, FB>), dim3(grid), dim3(256), 0, stream, g); break;
    default: hipLaunchKernelGGL((gemm_nt_generic_kernel<FA, FB>), dim3((unsigned)total), dim3(64), 0, stream, g); break;
    }
}

static int cu_count() {
    static int cus = 0;
    if (cus == 0) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess) cus = prop.multiProcessorCount;
        if (cus <= 0) cus = 256;
    }
    return cus;
}

static int choose_variant(int64_t M, int64_t N) {
    const int cus = cu_count();
    int best = 2;
    double best_score = -1.0;
    for (int v = 2; v < kNumVariants; ++v) {                    // variant 1 (one wave per SIMD) only by explicit request
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

extern "C" int odl_fp8_gemm_set_variant(int variant) {
    if (variant < -1 || variant >= kNumVariants) return set_error(ODL_ERR_ARG, "odl_fp8_gemm_set_variant: %d out of range", variant);
    g_forced_variant = variant;
    return ODL_OK;
}

extern "C" int odl_fp8_gemm_nt(const uint8_t *a, const uint8_t *b, int64_t M, int64_t N, int64_t K, int fmt_a, int fmt_b,
                               const float *sa_inv, int64_t sa_n, const float *sb_inv, int64_t sb_n, const void *bias,
                               int bias_dtype, void *c, int out_dtype, odl_stream_t stream_) {
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
    const int out_align = out_dtype == ODL_BF16 ? 8 : 16;
    if (reinterpret_cast<uintptr_t>(c) & (out_align - 1)) return set_error(ODL_ERR_SHAPE, "odl_fp8_gemm_nt: output must be %d-byte aligned", out_align);
    if (M == 0 || N == 0) return ODL_OK;

    const bool tiled_ok = K >= 128 && K % 128 == 0 && (double)M * (double)K < 4294967296.0 && (double)N * (double)K < 4294967296.0;
    int variant = g_forced_variant >= 0 ? g_forced_variant : (tiled_ok ? choose_variant(M, N) : 0);
    if (variant != 0 && !tiled_ok) variant = 0;

    GemmArgs g;
    g.a = a; g.b = b; g.c = c; g.sa = sa_inv; g.sb = sb_inv; g.bias = bias;
    g.M = M; g.N = N; g.K = K;
    g.sa_vec = sa_n == M && M != 1;
    g.sb_vec = sb_n == N && N != 1;
    g.out_dtype = out_dtype;
    const int bm = variant == 0 ? 32 : kVariants[variant].bm, bn = variant == 0 ? 32 : kVariants[variant].bn;
    const int64_t tm = (M + bm - 1) / bm, tn = (N + bn - 1) / bn;
    if (tm * tn > 0x7ffffff0LL) return set_error(ODL_ERR_SHAPE, "odl_fp8_gemm_nt: too many tiles");
    g.tiles_m = (int)tm; g.tiles_n = (int)tn;

    if (fmt_a == ODL_FP8_E4M3 && fmt_b == ODL_FP8_E4M3) launch_variant<ODL_FP8_E4M3, ODL_FP8_E4M3>(variant, g, stream);
    else if (fmt_a == ODL_FP8_E5M2 && fmt_b == ODL_FP8_E4M3) launch_variant<ODL_FP8_E5M2, ODL_FP8_E4M3>(variant, g, stream);
    else if (fmt_a == ODL_FP8_E4M3 && fmt_b == ODL_FP8_E5M2) launch_variant<ODL_FP8_E4M3, ODL_FP8_E5M2>(variant, g, stream);
    else launch_variant<ODL_FP8_E5M2, ODL_FP8_E5M2>(variant, g, stream);
    return check_launch("odl_fp8_gemm_nt");
}
