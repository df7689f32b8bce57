// FP8 GEMM, 256x256 block tile, 4 waves (one per SIMD, 128x128 each), explicit
// software pipeline.  C = (A[M,K] . B[N,K]^T) * scales, K % 256 == 0.
//
// Why one wave per SIMD: a 128x128 wave tile needs 256 accumulator registers
// (the whole AGPR half of the unified 512-entry file) but halves the LDS traffic
// per flop compared with two 128x64 waves.  With nothing else on the SIMD to hide
// a stall, the wave has to keep the MFMA pipe fed by itself:
//
//   per K step of 128 bytes (two halves h0, h1 of 64 bytes = one MFMA K each)
//     phase A : 16 MFMAs on register buffer 0 (step kt, h0)
//               interleaved with the 16 LDS reads of (kt, h1) into buffer 1
//     wait vmcnt(0) + lgkmcnt(0), s_barrier      <- the ONLY sync per K step:
//               step kt+1 has landed in the other LDS stage (it was requested a
//               whole step ago) and everybody is done reading this stage
//     phase B : 16 MFMAs on buffer 1 (kt, h1)
//               interleaved with the 16 LDS reads of (kt+1, h0) into buffer 0
//               and the 16 direct-to-LDS loads of step kt+2 into this stage
//
//   so MFMAs that do not depend on anything after the barrier are always
//   available when the barrier is crossed, and every LDS read has ~1000 cycles
//   of MFMA work in front of its first use.
//
// Global -> LDS: buffer_load_dwordx4 ... lds.  The per-lane byte offset is a
// loop-invariant VGPR, the K position is the scalar offset, the buffer resource's
// size makes rows past the end of the matrix read as zero: no per-load address
// arithmetic at all.  LDS layout as in gemm_tiled.hip (16-byte chunks of a 128-byte
// row XOR-swizzled with f(row) = (row ^ row>>3) & 7); because 32-row tile steps
// only flip bit 2 of f, each operand needs just 4 per-lane LDS address registers,
// everything else is an immediate.
//
// The four LDS regions (A/B x stage 0/1) are separate __shared__ objects so that
// the compiler can see that loads in flight into one stage never alias the reads
// of the other, and does not fence them with vmcnt waits.
#include "gemm_common.h"

#include <type_traits>

namespace odl {

namespace {

constexpr int BM = 256, BN = 256, NW = 4, WM = 128, WN = 128, TM = 4, TN = 4;
constexpr int REGION = 256 * 128;          // bytes of one operand in one stage
constexpr int LOADS = 256 / 8 / NW;        // 1 KB direct-to-LDS loads per wave per operand per stage
constexpr int GM = 8;

constexpr unsigned MASK_MFMA = 0x008, MASK_VMEM = 0x010, MASK_DS_RD = 0x100;   // sched_group_barrier classes

typedef __attribute__((address_space(3))) void *lds_ptr_t;

template <int FA, int FB>
__global__ __launch_bounds__(256) void gemm_nt_pipe_kernel(const GemmArgs g) {
    __shared__ __attribute__((aligned(1024))) uint8_t sA0[REGION];
    __shared__ __attribute__((aligned(1024))) uint8_t sB0[REGION];
    __shared__ __attribute__((aligned(1024))) uint8_t sA1[REGION];
    __shared__ __attribute__((aligned(1024))) uint8_t sB1[REGION];

    // ---- tile (XCD-aware, grouped): see gemm_tiled.hip
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
    const int wm0 = (wave / 2) * WM, wn0 = (wave % 2) * WN;
    const int KT = (int)(g.K / 128);
#ifdef ODL_GEMM_TRACE
    uint64_t t_entry; asm volatile("s_memtime %0\n\ts_waitcnt lgkmcnt(0)" : "=s"(t_entry));
#endif

    // ---- global -> LDS
    const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc((void *)g.a, 0, (int)(g.M * g.K), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc((void *)g.b, 0, (int)(g.N * g.K), 0x00020000);
    int voff_a[LOADS], voff_b[LOADS];
#pragma unroll
    for (int j = 0; j < LOADS; ++j) {
        const int row = (wave + j * NW) * 8 + lane / 8;
        const int sw = ((lane % 8) ^ swz(row)) << 4;
        voff_a[j] = (int)((m0 + row) * g.K) + sw;          // rows past M land beyond num_records -> zeros
        voff_b[j] = (int)((n0 + row) * g.K) + sw;
    }
    auto issue = [&](uint8_t *sa, uint8_t *sb, int kt) {
        const int soff = kt * 128;
#pragma unroll
        for (int j = 0; j < LOADS; ++j) {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (lds_ptr_t)(sa + (wave + j * NW) * 1024), 16, voff_a[j], soff, 0, 0);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, (lds_ptr_t)(sb + (wave + j * NW) * 1024), 16, voff_b[j], soff, 0, 0);
        }
    };

    // ---- L2 prefetch.  About one line in six of a K step misses this XCD's L2 (the 32
    // tiles running on an XCD share rows, but every row has to arrive once), and a miss
    // costs more than the one K step the LDS stages can cover.  So each lane touches one
    // 128-byte line of the step PF ahead with a load whose value is never used: 2 loads
    // per wave per step pull all 512 lines of that step into L2 long before the
    // direct-to-LDS loads ask for them.  They are issued AFTER the DMA loads of the same
    // phase, so "vmcnt(2)" still means "every DMA load has landed".
    constexpr int PF = 4;
    const uint8_t *pf_a = g.a + min(m0 + wave * 64 + lane, g.M - 1) * g.K;
    const uint8_t *pf_b = g.b + min(n0 + wave * 64 + lane, g.N - 1) * g.K;
    int pfv_a = 0, pfv_b = 0;
    auto prefetch = [&](int kt) {
        const int kp = min(kt, KT - 1) * 128;
        // "use" the values fetched one step ago (long since returned) so that the loads stay in the program
        asm volatile("" ::"v"(pfv_a), "v"(pfv_b));
        pfv_a = *reinterpret_cast<const int *>(pf_a + kp);
        pfv_b = *reinterpret_cast<const int *>(pf_b + kp);
    };

    // ---- LDS -> registers.  chunk(t, h, e) = ((2*lg + e) ^ s0) ^ 4*(h ^ (t & 1))
    const int lr = lane % 32, lg = lane / 32;
    int ra[2][2], rb[2][2];                     // [e][h ^ (t & 1)] byte offsets inside a region (tile 0)
    {
        const int rowa = wm0 + lr, rowb = wn0 + lr;
        const int s0a = swz(rowa), s0b = swz(rowb);
#pragma unroll
        for (int e = 0; e < 2; ++e)
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                ra[e][p] = rowa * 128 + (((((2 * lg + e) ^ s0a)) ^ (4 * p)) << 4);
                rb[e][p] = rowb * 128 + (((((2 * lg + e) ^ s0b)) ^ (4 * p)) << 4);
            }
    }
    auto read_a = [&](const uint8_t *sa, int t, int h) -> v8i {
        const v4i lo = *reinterpret_cast<const v4i *>(sa + ra[0][h ^ (t & 1)] + t * 4096);
        const v4i hi = *reinterpret_cast<const v4i *>(sa + ra[1][h ^ (t & 1)] + t * 4096);
        return v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    };
    auto read_b = [&](const uint8_t *sb, int u, int h) -> v8i {
        const v4i lo = *reinterpret_cast<const v4i *>(sb + rb[0][h ^ (u & 1)] + u * 4096);
        const v4i hi = *reinterpret_cast<const v4i *>(sb + rb[1][h ^ (u & 1)] + u * 4096);
        return v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    };

    v16f acc[TM][TN];
#pragma unroll
    for (int t = 0; t < TM; ++t)
#pragma unroll
        for (int u = 0; u < TN; ++u)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[t][u][e] = 0.0f;

    v8i a0[TM], b0[TN], a1[TM], b1[TN];         // register buffers 0 (h0) and 1 (h1)

    auto mfma_all = [&](v8i (&fa)[TM], v8i (&fb)[TN]) {
#pragma unroll
        for (int t = 0; t < TM; ++t)
#pragma unroll
            for (int u = 0; u < TN; ++u) acc[t][u] = mfma_32x32x64<FB, FA>(fb[u], fa[t], acc[t][u]);
    };

#ifdef ODL_GEMM_TRACE
    // development aid: cycle stamps around the per-step wait and barrier, kept in three VGPRs (lane = K step)
    uint32_t tr_a = 0, tr_b = 0, tr_c = 0;
#define ODL_STAMP_ISSUE(var) uint64_t var; asm volatile("s_memtime %0" : "=s"(var))
#define ODL_STAMP_SYNC(var) uint64_t var; asm volatile("s_memtime %0\n\ts_waitcnt lgkmcnt(0)" : "=s"(var))
#endif

    // One K step.  cur / nxt = LDS stage holding step kt / kt+1.
    auto step = [&](uint8_t *sa_cur, uint8_t *sb_cur, uint8_t *sa_nxt, uint8_t *sb_nxt, int kt, auto read_next, auto load_g) {
        // phase A
#pragma unroll
        for (int t = 0; t < TM; ++t) a1[t] = read_a(sa_cur, t, 1);
#pragma unroll
        for (int u = 0; u < TN; ++u) b1[u] = read_b(sb_cur, u, 1);
        mfma_all(a0, b0);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            __builtin_amdgcn_sched_group_barrier(MASK_MFMA, 1, 0);
            __builtin_amdgcn_sched_group_barrier(MASK_DS_RD, 2, 0);
        }
        __builtin_amdgcn_sched_group_barrier(MASK_MFMA, 8, 0);

        __builtin_amdgcn_sched_barrier(0);      // keep all 16 MFMAs of phase A in front of the wait: they cover the LDS latency
#ifdef ODL_GEMM_TRACE
        ODL_STAMP_SYNC(t_a);
#endif
        // my DMA for kt+1 has landed (the 2 younger prefetch loads may still be out), my LDS reads returned
        __builtin_amdgcn_s_waitcnt(0x0072);     // vmcnt(2) lgkmcnt(0)
#ifdef ODL_GEMM_TRACE
        ODL_STAMP_SYNC(t_b);
#endif
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
#ifdef ODL_GEMM_TRACE
        ODL_STAMP_SYNC(t_c);
        tr_a = lane == (kt & 63) ? (uint32_t)t_a : tr_a;
        tr_b = lane == (kt & 63) ? (uint32_t)t_b : tr_b;
        tr_c = lane == (kt & 63) ? (uint32_t)t_c : tr_c;
#endif
        __builtin_amdgcn_sched_barrier(0);

        // phase B
        if constexpr (decltype(read_next)::value) {
#pragma unroll
            for (int t = 0; t < TM; ++t) a0[t] = read_a(sa_nxt, t, 0);
#pragma unroll
            for (int u = 0; u < TN; ++u) b0[u] = read_b(sb_nxt, u, 0);
        }
        if constexpr (decltype(load_g)::value) {
            issue(sa_cur, sb_cur, kt + 2);
            prefetch(kt + 2 + PF);
        }
        mfma_all(a1, b1);
        if constexpr (decltype(read_next)::value && decltype(load_g)::value) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                __builtin_amdgcn_sched_group_barrier(MASK_MFMA, 1, 0);
                __builtin_amdgcn_sched_group_barrier(MASK_DS_RD, 2, 0);
                __builtin_amdgcn_sched_group_barrier(MASK_VMEM, 1, 0);
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                __builtin_amdgcn_sched_group_barrier(MASK_MFMA, 1, 0);
                __builtin_amdgcn_sched_group_barrier(MASK_VMEM, 1, 0);
            }
            __builtin_amdgcn_sched_group_barrier(MASK_VMEM, 2, 0);      // the two prefetch loads go last
        }
    };
    using yes = std::integral_constant<bool, true>;
    using no = std::integral_constant<bool, false>;

    // ---- prologue: steps 0 and 1 requested, step 0 awaited, (0, h0) in registers
    issue(sA0, sB0, 0);
    issue(sA1, sB1, 1);                          // KT >= 2 (host-checked)
    for (int k = 2; k < 2 + PF; ++k) prefetch(k);
    __builtin_amdgcn_s_waitcnt(0x0F70);          // vmcnt(0)
    __syncthreads();
#pragma unroll
    for (int t = 0; t < TM; ++t) a0[t] = read_a(sA0, t, 0);
#pragma unroll
    for (int u = 0; u < TN; ++u) b0[u] = read_b(sB0, u, 0);

    // ---- main loop: KT is even; the last two steps load nothing new
    for (int kt = 0; kt < KT - 2; kt += 2) {
        step(sA0, sB0, sA1, sB1, kt, yes{}, yes{});
        step(sA1, sB1, sA0, sB0, kt + 1, yes{}, yes{});
    }
    step(sA0, sB0, sA1, sB1, KT - 2, yes{}, no{});
    step(sA1, sB1, sA0, sB0, KT - 1, no{}, no{});

#ifdef ODL_GEMM_TRACE
    uint64_t t_loop_end; asm volatile("s_memtime %0\n\ts_waitcnt lgkmcnt(0)" : "=s"(t_loop_end));
    if (g.trace) {
        uint32_t *t = g.trace + ((size_t)blockIdx.x * NW + wave) * 3 * 64;
        t[lane] = tr_a; t[64 + lane] = tr_b; t[128 + lane] = tr_c;
    }
#endif
    // ---- epilogue
    const bool interior = m0 + BM <= g.M && n0 + BN <= g.N;
    const bool staged = interior && (g.N % 8) == 0;
    if (staged) {
        __syncthreads();                             // every wave is done with the operand stages: reuse them
        uint8_t *wave_lds = wave == 0 ? sA0 : (wave == 1 ? sB0 : (wave == 2 ? sA1 : sB1));
        if (g.out_dtype == ODL_BF16) epilogue_staged<true, TM, TN, TN>(g, acc, wave_lds, m0 + wm0, n0 + wn0, lane);
        else epilogue_staged<false, TM, TN, TN>(g, acc, wave_lds, m0 + wm0, n0 + wn0, lane);
    } else {
#define ODL_EPILOGUE(BF)                                                                                       \
    _Pragma("unroll") for (int t = 0; t < TM; ++t) _Pragma("unroll") for (int u = 0; u < TN; ++u)              \
        store_tile<BF, false>(g, acc[t][u], m0 + wm0 + 32 * t + lr, n0 + wn0 + 32 * u + 4 * lg)
        if (g.out_dtype == ODL_BF16) { ODL_EPILOGUE(true); } else { ODL_EPILOGUE(false); }
#undef ODL_EPILOGUE
    }
#ifdef ODL_GEMM_TRACE
    if (g.trace) {
        __builtin_amdgcn_s_waitcnt(0x0070);
        uint64_t t_exit; asm volatile("s_memtime %0\n\ts_waitcnt lgkmcnt(0)" : "=s"(t_exit));
        uint64_t *t64 = reinterpret_cast<uint64_t *>(g.trace + (size_t)gridDim.x * NW * 3 * 64) + ((size_t)blockIdx.x * NW + wave) * 4;
        if (lane == 0) { t64[0] = t_entry; t64[1] = t_loop_end; t64[2] = t_exit; t64[3] = __builtin_amdgcn_s_getreg((4 << 11) | 20 /*XCC_ID*/) ; }
    }
#endif
}

template <int FA, int FB>
void launch_fmt(const GemmArgs &g, hipStream_t stream) {
    const int total = g.tiles_m * g.tiles_n;
    const unsigned grid = (unsigned)(((total + 7) / 8) * 8);
    hipLaunchKernelGGL((gemm_nt_pipe_kernel<FA, FB>), dim3(grid), dim3(256), 0, stream, g);
}

}  // namespace

void launch_gemm_pipe(int fa, int fb, const GemmArgs &g, hipStream_t stream) {
    if (fa == ODL_FP8_E4M3 && fb == ODL_FP8_E4M3) launch_fmt<ODL_FP8_E4M3, ODL_FP8_E4M3>(g, stream);
    else if (fa == ODL_FP8_E5M2 && fb == ODL_FP8_E4M3) launch_fmt<ODL_FP8_E5M2, ODL_FP8_E4M3>(g, stream);
    else if (fa == ODL_FP8_E4M3 && fb == ODL_FP8_E5M2) launch_fmt<ODL_FP8_E4M3, ODL_FP8_E5M2>(g, stream);
    else launch_fmt<ODL_FP8_E5M2, ODL_FP8_E5M2>(g, stream);
}

}  // namespace odl
