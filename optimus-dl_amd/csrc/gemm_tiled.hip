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
//   * launches of at most one 128 x 128 tile per compute unit use four stages and eight waves instead (three K steps of
//     loads in flight; see the STAGES == 4 branch);
//   * block id -> tile mapping is XCD-aware: ids are dealt round-robin to the 8
//     XCDs by the hardware, so tile = (id % 8) * chunk + id / 8 keeps each XCD on
//     a contiguous run of tiles, walked in groups of GM rows for L2 reuse.
// Generic kernel: one wave per 32x32 tile straight from global memory; any
// M, N and K % 16 == 0.  Used for shapes the tiled kernel refuses.
#include "gemm_common.h"

namespace odl {

// ------------------------------------------------------------------ tiled kernel
template <int BM, int BN, int WAVES_M, int WAVES_N, int FA, int FB, int STAGES = 2>
__global__ __launch_bounds__(WAVES_M *WAVES_N * 64) void gemm_nt_tiled_kernel(const GemmArgs g) {
    static_assert(STAGES == 2 || STAGES == 4, "two LDS stages, or four for launches of at most one block per compute unit");
    constexpr int NW = WAVES_M * WAVES_N;
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N, TM = WM / 32, TN = WN / 32;
    constexpr int A_BYTES = BM * 128, B_BYTES = BN * 128, STAGE = A_BYTES + B_BYTES;
    constexpr int LA = BM / 8 / NW, LB = BN / 8 / NW;    // 1 KB load instructions per wave per stage
    constexpr int GM = 8;                                 // tile rows walked together
    static_assert(BM % (8 * NW) == 0 && BN % (8 * NW) == 0, "tile rows must split evenly over the waves");
    static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile must be a multiple of the 32x32 MFMA");

    __shared__ __attribute__((aligned(1024))) uint8_t lds0[STAGE];
    __shared__ __attribute__((aligned(1024))) uint8_t lds1[STAGE];
    __shared__ __attribute__((aligned(1024))) uint8_t lds2[STAGES == 4 ? STAGE : 1024];
    __shared__ __attribute__((aligned(1024))) uint8_t lds3[STAGES == 4 ? STAGE : 1024];

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

    if constexpr (STAGES == 4) {
        // A block that has a compute unit to itself cannot hide the latency of its loads behind another block's MFMAs:
        // with two stages a load has one step's compute (0.25 us) to arrive from the L2 or beyond, and the block waits
        // out the rest every step.  Four stages keep three steps of loads in flight.  A wave's loads complete in order,
        // so "stage kt has landed" is "at most the loads of the later stages are outstanding": vmcnt(2, 1 or 0 stages).
        // Loads, waits and barriers are written as instructions here: the compiler, shown direct-to-LDS loads into four
        // buffers, puts a wait for ALL of them in front of every LDS read (it tracks only a few such loads apart), and
        // __syncthreads() carries a fence that does the same; either is the two-stage kernel again.  The "memory"
        // clobber of the barrier keeps the LDS reads of a stage behind it.
        constexpr int PER = LA + LB;                            // direct-to-LDS instructions of a wave per stage
        static_assert(2 * PER <= 63, "the counter holds 63 loads");
        auto lds_addr_of = [](const uint8_t *p) { return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) uint8_t *)p; };
        auto dma = [](const uint8_t *src, uint32_t lds_addr) {  // 64 lanes x 16 bytes land at lds_addr + lane * 16
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_addr), "v"(src));
        };
        auto fetch = [&](uint8_t *lds, int kt) {
            const uint8_t *ga = g.a + (int64_t)kt * 128, *gb = g.b + (int64_t)kt * 128;
            const uint32_t base = lds_addr_of(lds);
#pragma unroll
            for (int j = 0; j < LA; ++j) dma(ga + off_a[j], base + (wave + j * NW) * 1024);
#pragma unroll
            for (int j = 0; j < LB; ++j) dma(gb + off_b[j], base + A_BYTES + (wave + j * NW) * 1024);
        };
        auto phase = [&](const uint8_t *cur, uint8_t *refill, int kt) {
            // everyone's loads of stage kt are in, and everyone has read stage kt - 1
            if (kt + 2 < KT) asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(2 * PER) : "memory");
            else if (kt + 1 < KT) asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(PER) : "memory");
            else asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
            if (kt + 3 < KT) fetch(refill, kt + 3);             // into the stage that step kt - 1 used
            compute(cur);
        };
        fetch(lds0, 0);
        if (KT > 1) fetch(lds1, 1);
        if (KT > 2) fetch(lds2, 2);
        for (int kt = 0; kt < KT; kt += 4) {
            phase(lds0, lds3, kt);
            if (kt + 1 < KT) phase(lds1, lds0, kt + 1);
            if (kt + 2 < KT) phase(lds2, lds1, kt + 2);
            if (kt + 3 < KT) phase(lds3, lds2, kt + 3);
        }
    } else {
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
    }

    // ---- epilogue (uniform choice per block: staged through LDS for interior tiles, direct stores at the edges)
    const bool interior = m0 + BM <= g.M && n0 + BN <= g.N;
    constexpr int EPI_BYTES = 32 * (TN * 32 * 4 + 16);      // one wave's staging region, fp32 worst case
    static_assert(NW * EPI_BYTES <= 2 * STAGE, "epilogue staging must fit in the operand stages");
    if (interior && (g.N % 8) == 0) {
        __syncthreads();
        uint8_t *wave_lds = (wave * EPI_BYTES + EPI_BYTES <= STAGE) ? lds0 + wave * EPI_BYTES
                                                                    : lds1 + (wave - STAGE / EPI_BYTES) * EPI_BYTES;
        if (g.accumulate) {
            if (g.out_dtype == ODL_BF16) epilogue_staged_accumulate<true, TM, TN, 1>(g, acc, wave_lds, m0 + wm0, n0 + wn0, lane);
            else epilogue_staged_accumulate<false, TM, TN, 1>(g, acc, wave_lds, m0 + wm0, n0 + wn0, lane);
        } else if (g.out_dtype == ODL_BF16) epilogue_staged<true, TM, TN, TN>(g, acc, wave_lds, m0 + wm0, n0 + wn0, lane);
        else epilogue_staged<false, TM, TN, TN>(g, acc, wave_lds, m0 + wm0, n0 + wn0, lane);
    } else {
#define ODL_EPILOGUE(BF)                                                                                       \
    _Pragma("unroll") for (int t = 0; t < TM; ++t) _Pragma("unroll") for (int u = 0; u < TN; ++u)              \
        store_tile<BF, false>(g, acc[t][u], m0 + wm0 + 32 * t + lr, n0 + wn0 + 32 * u + 4 * lg)
        if (g.out_dtype == ODL_BF16) { ODL_EPILOGUE(true); } else { ODL_EPILOGUE(false); }
#undef ODL_EPILOGUE
    }
}


template <int FA, int FB>
static void launch_tiled_fmt(int variant, const GemmArgs &g, hipStream_t stream) {
    const int total = g.tiles_m * g.tiles_n;
    const unsigned grid = (unsigned)(((total + 7) / 8) * 8);
    switch (variant) {
    case 1: hipLaunchKernelGGL((gemm_nt_tiled_kernel<256, 256, 2, 2, FA, FB>), dim3(grid), dim3(256), 0, stream, g); break;
    case 2: hipLaunchKernelGGL((gemm_nt_tiled_kernel<256, 256, 2, 4, FA, FB>), dim3(grid), dim3(512), 0, stream, g); break;
    case 3: hipLaunchKernelGGL((gemm_nt_tiled_kernel<256, 128, 2, 2, FA, FB>), dim3(grid), dim3(256), 0, stream, g); break;
    default:
        // at most one block per compute unit: the four-stage form (128 KB of LDS, which leaves room for one block only)
        if (total <= device_cu_count())
            hipLaunchKernelGGL((gemm_nt_tiled_kernel<128, 128, 2, 4, FA, FB, 4>), dim3(grid), dim3(512), 0, stream, g);
        else
            hipLaunchKernelGGL((gemm_nt_tiled_kernel<128, 128, 2, 2, FA, FB>), dim3(grid), dim3(256), 0, stream, g);
        break;
    }
}

void launch_gemm_tiled(int variant, int fa, int fb, const GemmArgs &g, hipStream_t stream) {
    if (fa == ODL_FP8_E4M3 && fb == ODL_FP8_E4M3) launch_tiled_fmt<ODL_FP8_E4M3, ODL_FP8_E4M3>(variant, g, stream);
    else if (fa == ODL_FP8_E5M2 && fb == ODL_FP8_E4M3) launch_tiled_fmt<ODL_FP8_E5M2, ODL_FP8_E4M3>(variant, g, stream);
    else if (fa == ODL_FP8_E4M3 && fb == ODL_FP8_E5M2) launch_tiled_fmt<ODL_FP8_E4M3, ODL_FP8_E5M2>(variant, g, stream);
    else launch_tiled_fmt<ODL_FP8_E5M2, ODL_FP8_E5M2>(variant, g, stream);
}

}  // namespace odl
