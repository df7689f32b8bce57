// FP8 GEMM, 256x256 block tile, 4 waves (one per SIMD, 128x128 each), explicit
// software pipeline, persistent over tiles.  C = (A[M,K] . B[N,K]^T) * scales,
// K % 256 == 0.
//
// Why one wave per SIMD: a 128x128 wave tile needs 256 accumulator registers
// (the whole AGPR half of the unified 512-entry file) but halves the LDS traffic
// per flop compared with two 128x64 waves.  With nothing else on the SIMD to hide
// a stall, the wave has to keep the MFMA pipe fed by itself:
//
//   per K step of 128 bytes (two halves h0, h1 of 64 bytes = one MFMA K each)
//     phase A : 16 MFMAs on register buffer 0 (step kt, h0)
//               interleaved with the 16 LDS reads of (kt, h1) into buffer 1
//     wait vmcnt(2) + lgkmcnt(0), s_barrier      <- the ONLY sync per K step:
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
// Persistent: one block per CU walks its share of the tiles.  When the K loop of a
// tile ends, the first two K steps of the NEXT tile are requested before the
// epilogue starts, so the latency of a tile's first loads (HBM: several
// microseconds) and the drain of the output stores overlap each other instead of
// both being paid per tile.  The epilogue therefore stages through its own small
// LDS region (the operand stages are already being refilled).
//
// Global -> LDS: buffer_load_dwordx4 ... lds.  The per-lane byte offset is a
// loop-invariant VGPR, the K position is the scalar offset, the buffer resource's
// size makes rows past the end of the matrix read as zero: no per-load address
// arithmetic at all.  LDS layout as in gemm_tiled.hip (16-byte chunks of a 128-byte
// row XOR-swizzled with f(row) = (row ^ row>>3) & 7); because 32-row tile steps
// only flip bit 2 of f, each operand needs just 4 per-lane LDS address registers,
// everything else is an immediate.
//
// Every vector-memory load of the K loop is issued from inline asm, and every wait
// on the vector-memory counter is written out by hand: the counter retires in issue
// order, which lets the loop wait for "all but the youngest n" operations (the previous
// tile's output stores), something the compiler's own bookkeeping cannot express across
// the tile loop.  Instruction order inside a phase
// is pinned with sched_barrier so that each MFMA is followed by its share of LDS
// reads and loads.
#include "gemm_common.h"

#include <type_traits>

namespace odl {

namespace {

constexpr int BM = 256, BN = 256, NW = 4, WM = 128, WN = 128, TM = 4, TN = 4;
constexpr int REGION = 256 * 128;          // bytes of one operand in one stage
constexpr int LOADS = 256 / 8 / NW;        // 1 KB direct-to-LDS loads per wave per operand per stage
constexpr int GM = 8;
constexpr int EPI_BYTES = 32 * (128 + 16); // one wave's epilogue slab: 32 rows x 128 bytes (+16 pad)
static_assert(staged_epilogue_bytes<true, 2>() == EPI_BYTES && staged_epilogue_bytes<false, 1>() == EPI_BYTES, "slab size");

typedef __attribute__((address_space(3))) void *lds_ptr_t;

// ACC: the form for C = C + product (g.accumulate).  A kernel of its own, so that the registers its epilogue needs for
// the old values of C do not weigh on the ordinary one; its direct-to-LDS loads carry the wait states that a scalar
// register restored from a spill needs before a vector-memory instruction reads it (this form does spill scalars).
template <int FA, int FB, bool ACC>
__global__ __launch_bounds__(256) void gemm_nt_pipe_kernel(const GemmArgs g) {
    __shared__ __attribute__((aligned(1024))) uint8_t sA0[REGION];
    __shared__ __attribute__((aligned(1024))) uint8_t sB0[REGION];
    __shared__ __attribute__((aligned(1024))) uint8_t sA1[REGION];
    __shared__ __attribute__((aligned(1024))) uint8_t sB1[REGION];
    __shared__ __attribute__((aligned(16))) uint8_t sEpi[NW * EPI_BYTES];

    const int lane = threadIdx.x % 64;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    const int wm0 = (wave / 2) * WM, wn0 = (wave % 2) * WN;
    const int lr = lane % 32, lg = lane / 32;
    const int KT = (int)(g.K / 128);

    // ---- which tiles: block ids are dealt round-robin to the 8 XCDs, so the blocks of
    // one XCD (id % 8) walk one contiguous chunk of the grouped tile order together
    const int total = g.tiles_m * g.tiles_n;
    const int per_xcd = (total + 7) / 8;
    const int xcd = (int)(blockIdx.x % 8), stride = (int)(gridDim.x / 8);
    const int pid_end = min((xcd + 1) * per_xcd, total);
    int pid = xcd * per_xcd + (int)(blockIdx.x / 8);
    if (pid >= pid_end) return;

    // ---- per-tile addressing.  The tile's origin lives in the buffer resources (base =
    // first row of the tile, size = what is left of the matrix, so rows past the end read
    // as zero); the per-lane offsets are the same for every tile and for both operands.
    int64_t m0 = 0, n0 = 0, next_m0 = 0, next_n0 = 0;
    v4i rsrc_a, rsrc_b, next_a, next_b;           // raw buffer descriptors (base, stride 0, bytes, format)
    auto tile_origin = [&](int p, int64_t &tm0, int64_t &tn0) {
        const int in_group = GM * g.tiles_n;
        const int first_m = (p / in_group) * GM;
        const int group_rows = min(g.tiles_m - first_m, GM);
        tm0 = (int64_t)(first_m + (p % in_group) % group_rows) * BM;
        tn0 = (int64_t)((p % in_group) / group_rows) * BN;
    };
    auto rsrc_for = [&](const uint8_t *base, int64_t row0, int64_t rows) -> v4i {
        const uint64_t addr = reinterpret_cast<uint64_t>(base + row0 * g.K);
        return v4i{(int)(uint32_t)addr, (int)(uint32_t)(addr >> 32), (int)((rows - row0) * g.K), 0x00020000};
    };
    int voff[LOADS];
#pragma unroll
    for (int j = 0; j < LOADS; ++j) {
        const int row = (wave + j * NW) * 8 + lane / 8;
        voff[j] = row * (int)g.K + (((lane % 8) ^ swz(row)) << 4);
    }
    // one 1 KB direct-to-LDS load: 64 lanes x 16 bytes land at lds_addr + lane * 16
    auto dma = [&](const v4i &rsrc, uint32_t lds_addr, int vo, int so) {
        if constexpr (ACC)
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 4\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                         ::"s"(lds_addr), "v"(vo), "s"(rsrc), "s"(so));
        else
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                     ::"s"(lds_addr), "v"(vo), "s"(rsrc), "s"(so));
    };
    auto lds_addr_of = [](const uint8_t *p) { return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) uint8_t *)p; };
    // load j of a stage: j < LOADS -> operand A, else operand B
    auto issue_one = [&](uint8_t *sa, uint8_t *sb, int kt, int j) {
        if (j < LOADS) dma(rsrc_a, lds_addr_of(sa) + (wave + j * NW) * 1024, voff[j], kt * 128);
        else dma(rsrc_b, lds_addr_of(sb) + (wave + (j - LOADS) * NW) * 1024, voff[j - LOADS], kt * 128);
    };
    auto issue = [&](uint8_t *sa, uint8_t *sb, int kt) {
#pragma unroll
        for (int j = 0; j < 2 * LOADS; ++j) issue_one(sa, sb, kt, j);
    };

    bool has_next = false;

    // ---- LDS -> registers.  chunk(t, h, e) = ((2*lg + e) ^ s0) ^ 4*(h ^ (t & 1))
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
    v8i a0[TM], b0[TN], a1[TM], b1[TN];         // register buffers 0 (h0) and 1 (h1)

    auto mfma_all = [&](v8i (&fa)[TM], v8i (&fb)[TN]) {
#pragma unroll
        for (int t = 0; t < TM; ++t)
#pragma unroll
            for (int u = 0; u < TN; ++u) acc[t][u] = mfma_32x32x64<FB, FA>(fb[u], fa[t], acc[t][u]);
    };

    // One K step.  cur / nxt = LDS stage holding step kt / kt+1.  MFMA i works on tile
    // (t, u) = (i / 4, i % 4); fragment f < 4 is A tile f, f >= 4 is B tile f - 4.
    auto step = [&](uint8_t *sa_cur, uint8_t *sb_cur, uint8_t *sa_nxt, uint8_t *sb_nxt, int kt, auto read_next, auto load_g) {
        // phase A: MFMAs on buffer 0, the 8 fragments of (kt, h1) stream into buffer 1 behind the first 8
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            acc[i / 4][i % 4] = mfma_32x32x64<FB, FA>(b0[i % 4], a0[i / 4], acc[i / 4][i % 4]);
            if (i < 4) a1[i] = read_a(sa_cur, i, 1);
            else if (i < 8) b1[i - 4] = read_b(sb_cur, i - 4, 1);
            __builtin_amdgcn_sched_barrier(0);
        }
        // my DMA for kt+1 has landed, my LDS reads returned
        __builtin_amdgcn_s_waitcnt(0x0070);     // vmcnt(0) lgkmcnt(0)
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);

        // phase B: MFMAs on buffer 1; (kt+1, h0) streams into buffer 0; step kt+2 is requested into this stage
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            acc[i / 4][i % 4] = mfma_32x32x64<FB, FA>(b1[i % 4], a1[i / 4], acc[i / 4][i % 4]);
            if constexpr (decltype(read_next)::value) {
                if (i < 4) a0[i] = read_a(sa_nxt, i, 0);
                else if (i < 8) b0[i - 4] = read_b(sb_nxt, i - 4, 0);
            }
            if constexpr (decltype(load_g)::value) {
                issue_one(sa_cur, sb_cur, kt + 2, i);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    using yes = std::integral_constant<bool, true>;
    using no = std::integral_constant<bool, false>;

    // ---- first tile: steps 0 and 1 requested (KT >= 2, host-checked) and awaited
    tile_origin(pid, m0, n0);
    rsrc_a = rsrc_for(g.a, m0, g.M);
    rsrc_b = rsrc_for(g.b, n0, g.N);
    next_a = rsrc_a;
    next_b = rsrc_b;
    issue(sA0, sB0, 0);
    issue(sA1, sB1, 1);
    __builtin_amdgcn_s_waitcnt(0x0F70);          // vmcnt(0)

    while (true) {
        const int64_t cm0 = m0, cn0 = n0;        // this tile's origin, kept for the epilogue
        const int next_pid = pid + stride;
        has_next = next_pid < pid_end;
        if (has_next) {
            tile_origin(next_pid, next_m0, next_n0);
            next_a = rsrc_for(g.a, next_m0, g.M);
            next_b = rsrc_for(g.b, next_n0, g.N);
        }

        // Steps 0 and 1 of this tile have landed.  The vector-memory counter retires in issue
        // order, and behind those 32 loads this wave has issued at least 32 output stores of
        // the previous tile ("at most 32
        // outstanding" = the loads are in; for the first tile everything was awaited above),
        // while the stores of the previous tile may still be draining.  (The staged epilogue
        // issues 32 or 64 stores; the edge-tile path ends with a full wait.)
        __builtin_amdgcn_s_waitcnt(0x8F70);      // vmcnt(32): bits 3:0 = 0, bits 15:14 = 2
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
#pragma unroll
        for (int t = 0; t < TM; ++t) a0[t] = read_a(sA0, t, 0);
#pragma unroll
        for (int u = 0; u < TN; ++u) b0[u] = read_b(sB0, u, 0);
#pragma unroll
        for (int t = 0; t < TM; ++t)
#pragma unroll
            for (int u = 0; u < TN; ++u)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[t][u][e] = 0.0f;

        // ---- K loop: KT is even; the last two steps load nothing new
        for (int kt = 0; kt < KT - 2; kt += 2) {
            step(sA0, sB0, sA1, sB1, kt, yes{}, yes{});
            step(sA1, sB1, sA0, sB0, kt + 1, yes{}, yes{});
        }
        step(sA0, sB0, sA1, sB1, KT - 2, yes{}, no{});
        step(sA1, sB1, sA0, sB0, KT - 1, no{}, no{});

        // Every wave passed the barrier of the last step after its final operand read, so
        // the stages are free: request the next tile's first two steps before the epilogue.
        if (has_next) {
            pid = next_pid;
            m0 = next_m0;
            n0 = next_n0;
            rsrc_a = next_a;
            rsrc_b = next_b;
            issue(sA0, sB0, 0);
            issue(sA1, sB1, 1);
        }
        __builtin_amdgcn_sched_barrier(0);       // the loads stay in front of every store of the epilogue

        // ---- epilogue of the tile just finished.  The lane / wave ids are laundered through
        // empty asm so that the compiler computes the epilogue's addresses here, instead of
        // once before the tile loop: kept across the K loop they would spill, and every
        // scratch reload would wait on the vector-memory counter, i.e. on the output stores.
        int lane_e = lane, wave_e = wave;
        asm volatile("" : "+v"(lane_e));
        asm volatile("" : "+s"(wave_e));
        const bool interior = cm0 + BM <= g.M && cn0 + BN <= g.N;
        if (interior && (g.N % 8) == 0) {
            uint8_t *wave_lds = sEpi + wave_e * EPI_BYTES;
            const int64_t mw = cm0 + (wave_e / 2) * WM, nw = cn0 + (wave_e % 2) * WN;
            if constexpr (ACC) {
                if (g.out_dtype == ODL_BF16) epilogue_staged_accumulate<true, TM, TN, 1>(g, acc, wave_lds, mw, nw, lane_e);
                else epilogue_staged_accumulate<false, TM, TN, 1>(g, acc, wave_lds, mw, nw, lane_e);
            } else if (g.out_dtype == ODL_BF16) epilogue_staged<true, TM, TN, 2>(g, acc, wave_lds, mw, nw, lane_e);
            else epilogue_staged<false, TM, TN, 1>(g, acc, wave_lds, mw, nw, lane_e);
        } else {
#define ODL_EPILOGUE(BF)                                                                                       \
    _Pragma("unroll") for (int t = 0; t < TM; ++t) _Pragma("unroll") for (int u = 0; u < TN; ++u)              \
        store_tile<BF, false>(g, acc[t][u], cm0 + wm0 + 32 * t + lr, cn0 + wn0 + 32 * u + 4 * lg)
            if (g.out_dtype == ODL_BF16) { ODL_EPILOGUE(true); } else { ODL_EPILOGUE(false); }
#undef ODL_EPILOGUE
            // this path issues a data-dependent number of stores: do not count on them below
            __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
        }
        if (!has_next) break;
    }
}

template <int FA, int FB>
void launch_fmt(const GemmArgs &g, int blocks_per_xcd, hipStream_t stream) {
    if (g.accumulate) hipLaunchKernelGGL((gemm_nt_pipe_kernel<FA, FB, true>), dim3((unsigned)(8 * blocks_per_xcd)), dim3(256), 0, stream, g);
    else hipLaunchKernelGGL((gemm_nt_pipe_kernel<FA, FB, false>), dim3((unsigned)(8 * blocks_per_xcd)), dim3(256), 0, stream, g);
}

}  // namespace

// One block per CU at most (the kernel needs ~150 KB of LDS), 8 | grid so that the
// round-robin placement gives every XCD the same number of blocks.
void launch_gemm_pipe(int fa, int fb, const GemmArgs &g, int num_cus, hipStream_t stream) {
    const int total = g.tiles_m * g.tiles_n;
    const int per_xcd = (total + 7) / 8;
    int bpx = num_cus / 8;
    if (bpx < 1) bpx = 1;
    if (bpx > per_xcd) bpx = per_xcd;
    if (fa == ODL_FP8_E4M3 && fb == ODL_FP8_E4M3) launch_fmt<ODL_FP8_E4M3, ODL_FP8_E4M3>(g, bpx, stream);
    else if (fa == ODL_FP8_E5M2 && fb == ODL_FP8_E4M3) launch_fmt<ODL_FP8_E5M2, ODL_FP8_E4M3>(g, bpx, stream);
    else if (fa == ODL_FP8_E4M3 && fb == ODL_FP8_E5M2) launch_fmt<ODL_FP8_E4M3, ODL_FP8_E5M2>(g, bpx, stream);
    else launch_fmt<ODL_FP8_E5M2, ODL_FP8_E5M2>(g, bpx, stream);
}

}  // namespace odl
