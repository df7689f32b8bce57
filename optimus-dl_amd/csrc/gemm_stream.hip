// FP8 GEMM, 256x256 block tile, 4 waves (one per SIMD, 128x128 each), persistent,
// with the epilogue of every tile folded under the first MFMAs of the next one.
// C = (A[M,K] . B[N,K]^T) * (sa_inv * sb_inv) (+ bias) in bf16 or fp32, for the shapes training uses:
// M % 128 == 0, N % 128 == 0, K % 128 == 0, K >= 512; scales per tensor or per row of A / B.
// Everything else goes to gemm_pipe.hip, whose K step this kernel shares:
//
//   per K step of 128 bytes (two halves h0, h1 of 64 bytes = one MFMA K each)
//     phase A : 16 MFMAs on register buffer 0 (step kt, h0)
//               interleaved with the 16 LDS reads of (kt, h1) into buffer 1
//     wait vmcnt + lgkmcnt(0), s_barrier         <- the only sync per K step
//     phase B : 16 MFMAs on buffer 1 (kt, h1)
//               interleaved with the 16 LDS reads of (kt+1, h0) into buffer 0
//               and the 16 direct-to-LDS loads of step kt+2 into this stage
//
// What is different here:
//
// * The load pipeline does not stop at a tile boundary.  The last two K steps of a
//   tile request the first two of the block's next tile (its last tile requests from
//   an empty buffer, which reads as zero without touching memory), so the whole
//   kernel is one uniform stream of steps and no tile ever waits for its first loads.
//
// * With one wave per SIMD nobody else can use the MFMA pipe while a wave converts
//   and stores its 128x128 results (about a sixth of a tile's time).  So phase A of a
//   tile's step 0 starts each 32x32 sub-tile from a zero C operand, and just before
//   MFMA i is issued the previous tile's sub-tile i is read out of the accumulators,
//   scaled, rounded to bf16 (v_cvt_pk_bf16_f32) and written to a private LDS slab;
//   after every second MFMA the slab (32 rows x 64 columns) is read back along the
//   rows and leaves as full 128-byte lines.  The conversion runs on the vector ALU
//   while the matrix pipe works on the MFMA just issued.  After a block's last tile
//   the same phase runs once more on operands nobody uses, only to store that tile.
//
// * The tile loop is rotated so that the accumulators are read (by the vector ALU)
//   in the same straight-line block in which the last MFMAs of the tile define them:
//   the loop body is [phase B of step 0, steps 1 .. KT-1, folded phase A of the next
//   tile].  Across the loop edge the accumulators are only ever MFMA operands.
//
// Vector-memory counter: all loads and stores of the loop are inline asm and every
// wait is written by hand.  The counter retires in issue order, so "vmcnt(n)" means
// "everything but the youngest n operations has completed":
//   step 0 : younger than the loads of step 1 are the 32 output stores of the folded
//            epilogue                                 -> vmcnt(32)
//            (fp32 output: 64 stores, and the counter field ends at 63 -> vmcnt(63), which also
//            waits for the first of those stores, issued a thousand cycles earlier)
//   others : nothing is younger than the loads of step kt+1            -> vmcnt(0)
// (An L2 prefetch, one lane per 128-byte line a few steps ahead, was tried and removed: the
// scattered loads occupy the texture path that the direct-to-LDS loads need, 14 % of the K loop.)
//
// Two compile-time switches exist for measuring where the energy of a launch goes (never defined in the shipped
// build; the results are wrong on purpose): ODL_EXP_SAME_PANELS makes every tile read the operand panels of tile
// (0, 0), so that nothing comes from beyond the L2; ODL_EXP_HALF_LDS_READS makes the second K half of a step
// multiply the fragments of the first again, which halves the LDS-to-register traffic.
#include "gemm_common.h"

#include <type_traits>

namespace odl {

namespace {

constexpr int BM = 256, BN = 256, NW = 4, WM = 128, WN = 128, TM = 4, TN = 4;
constexpr int REGION = 256 * 128;          // bytes of one operand in one stage
constexpr int LOADS = 256 / 8 / NW;        // 1 KB direct-to-LDS loads per wave per operand per stage
constexpr int GM = 8;
constexpr int PITCH = 128 + 8;             // slab row: 64 bf16 + 8 bytes, see phase_a_fold
constexpr int SLAB = 32 * PITCH;           // one wave's epilogue slab
typedef float f32x4 __attribute__((ext_vector_type(4)));

// TA / TB: the operand is stored with the contraction index as the SLOW axis ([K, M] resp. [K, N]
// row-major) instead of the fast one.  A stage then holds 128 K-rows of 256 bytes; the 1 KB loads
// bring 4 such rows each, and fragments are read with ds_read_b64_tr_b8, which hands every lane
// of a 16-lane group one byte column of an 8 x 16 byte block (8 consecutive K for its own row).
// The 16-byte chunks of a K-row are placed at chunk ^ 2 (k & 7): the 8 rows x 32 bytes that the two
// 16-lane groups of a half-wave read together then cover all 16 chunk positions = all 64 banks once
// (with chunk ^ (k & 7) the two groups met in the same 8 positions: 2 extra cycles per read, measured).  Same K order, same accumulation, same bits
// as the other layout: wgrad and dgrad no longer need transposed copies of their operands.
// F32: fp32 output (weight gradients of fp32 master weights).  A 32 x 32 sub-tile is then a whole slab
// (32 rows of 128 bytes) and leaves right after its own MFMA: 64 stores per wave and tile instead of 32.
// EPI: 0 = one scale per operand; 1 = a scale per row of A and / or per row of B (rowwise recipe);
// 2 = the same plus an fp32 bias per output column.
// MX: block-scaled operands (32 K-bytes share an E8M0 scale byte, applied by the MFMA itself).  g.mx_sa / g.mx_sb hold
// the scale bytes K-step-major: dword [kstep][row] = the 4 scale bytes of row `row` in the 128-byte K step `kstep`.
// Per K step a wave brings 64 such dwords of A and 64 of B to LDS with two 256-byte loads issued beside the operand
// loads of the same step, placed so that a lane finds the dwords of its 4 fragment rows (32 apart) side by side: one
// 16-byte LDS read per operand and step, made in phase B of the step before.  Lanes 32..63 shift the dword right by 8:
// byte 0 / byte 2 are then the scales a lane supplies in phase A / phase B (the MFMA takes the scale of K 0..31 from
// lanes 0..31 and of K 32..63 from lanes 32..63, and a lane's registers 0..3 / 4..7 as K 16 g.. / 32 + 16 g..).
template <int FB, int FA, bool MX, int H>
__device__ __forceinline__ v16f mma_step(const v8i &b, const v8i &a, const v16f &c, int eb, int ea) {
    if constexpr (MX) return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b, a, c, FB, FA, 2 * H, eb, 2 * H, ea);
    else return mfma_32x32x64<FB, FA>(b, a, c);
}

// SEG: the contraction runs over gp.count operand pairs with a scale product each (the data gradients of Linears that are
// fed one tensor: dX = sum_s dY_s . W_s).  A block stays on its tile through all pairs; the load pipeline crosses from one
// pair to the next exactly as it crosses from one tile to the next (other descriptors, other row pitch), and where a tile
// ends with a fold, a pair ends with the accumulators multiplied by (scale product of this pair) / (that of the next)
// under the first MFMAs of the next pair.  After the last pair the fold applies the last pair's scale product, so
// C = ((acc_0 r_0 + acc_1) r_1 + ...) s_last in fp32 with one rounding to the output type.
template <int FA, int FB, bool TA, bool TB, bool F32, int EPI, bool MX, bool SEG>
__device__ __forceinline__ void gemm_nt_stream_body(const GemmArgs &g, const GemmPairs &gp) {
    static_assert(!MX || (!TA && !TB && EPI != 1), "block scales: both operands stored [rows, K], no scale vectors");
    static_assert(!SEG || (!TA && !TB && EPI == 0 && !MX), "operand pairs: both stored [rows, K], one scale each");
    constexpr int ESZ = F32 ? 4 : 2;
    constexpr int VEC_BYTES = 3 * 128 * 4;     // per wave: 128 row scales, 128 column scales, 128 bias values
    __shared__ __attribute__((aligned(1024))) uint8_t sA0[REGION];
    __shared__ __attribute__((aligned(1024))) uint8_t sB0[REGION];
    __shared__ __attribute__((aligned(1024))) uint8_t sA1[REGION];
    __shared__ __attribute__((aligned(1024))) uint8_t sB1[REGION];
    __shared__ __attribute__((aligned(16))) uint8_t sEpi[NW * SLAB];
    __shared__ __attribute__((aligned(16))) uint8_t sVec[EPI > 0 ? NW * VEC_BYTES : 16];
    __shared__ __attribute__((aligned(16))) uint32_t sScale[MX ? 2 * 512 : 4];     // [stage][A rows 0..255 | B rows 0..255], permuted
    __shared__ float sRatio[4];

    const int lane = threadIdx.x % 64;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    const int wm0 = (wave / 2) * WM, wn0 = (wave % 2) * WN;
    const int lr = lane % 32, lg = lane / 32;
    // K steps of 128 bytes come in pairs (two LDS stages): an odd count is rounded up, and the padding
    // step is requested through the empty descriptor, so it multiplies zeros.  With g.splits > 1 a work item
    // is (tile, split): the steps [split * split_steps, + split_steps) of that tile, written as an fp32
    // partial result to slice `split` of the workspace that g.c then points to.
    int KT = 0;
    bool padded = false;
    const int tiles = g.tiles_m * g.tiles_n;
    auto item_steps = [&](int p, int &first_step, int &kt, bool &pad) {
        first_step = __builtin_amdgcn_readfirstlane((p / tiles) * g.split_steps);
        const int real = min(g.split_steps, (int)(g.K / 128) - first_step);
        kt = (real + 1) & ~1;
        pad = kt != real;
    };

    // ---- which items: block ids are dealt round-robin to the 8 XCDs, so the blocks of
    // one XCD (id % 8) walk one contiguous chunk of the grouped tile order together
    const int total = tiles * g.splits;
    const int per_xcd = (total + 7) / 8;
    const int xcd = (int)(blockIdx.x % 8), stride = (int)(gridDim.x / 8);
    const int pid_end = min((xcd + 1) * per_xcd, total);
    int pid = xcd * per_xcd + (int)(blockIdx.x / 8);
    if (pid >= pid_end) return;
#ifdef ODL_FP8_NO_BENCH_HOOKS
    constexpr bool stamps = false;
#else
    const bool stamps = g.clock_out != nullptr && blockIdx.x == 0 && threadIdx.x == 0;   // bench-only clock probe
#endif
    if (stamps) {
        g.clock_out[0] = clock64();
        g.clock_out[1] = wall_clock64();
    }

    // ---- per-tile addressing: the tile's origin lives in the buffer resources, the
    // per-lane offsets are the same for every tile and for both operands
    const v4i empty = {0, 0, 0, 0x00020000};      // zero bytes: loads read as zero, stores are dropped
    auto tile_origin = [&](int item, int &tm0, int &tn0) {
        const int p = item % tiles;
        const int in_group = GM * g.tiles_n;
        const int first_m = (p / in_group) * GM;
        const int group_rows = min(g.tiles_m - first_m, GM);
        // (integer division runs on the vector unit: readfirstlane states that the results are uniform)
        tm0 = __builtin_amdgcn_readfirstlane((first_m + (p % in_group) % group_rows) * BM);
        tn0 = __builtin_amdgcn_readfirstlane(((p % in_group) / group_rows) * BN);
    };
    // descriptor of an operand for the tile rows from row0 on and the K steps from first_step on
    auto rsrc_for = [&](const uint8_t *base, int row0, int64_t rows, bool transposed, int first_step, int nk) -> v4i {
        // an operand is smaller than 2 GiB (checked by the caller): 32-bit products, which stay scalar
        const int k0 = first_step * 128, nrows = (int)rows;
        if (transposed) {                          // [K, rows] storage: the tile starts at column row0 of K-row k0
            const uint64_t addr = reinterpret_cast<uint64_t>(base) + (uint32_t)(k0 * nrows + row0);
            return v4i{(int)(uint32_t)addr, (int)(uint32_t)(addr >> 32), (nk - k0) * nrows - row0, 0x00020000};
        }
        const uint64_t addr = reinterpret_cast<uint64_t>(base) + (uint32_t)(row0 * nk + k0);
        return v4i{(int)(uint32_t)addr, (int)(uint32_t)(addr >> 32), (nrows - row0) * nk - k0, 0x00020000};
    };
    // per-lane source offsets of the LOADS 1 KB loads of a stage
    int voff_a[LOADS], voff_b[LOADS];
#pragma unroll
    for (int j = 0; j < LOADS; ++j) {
        const int row = (wave + j * NW) * 8 + lane / 8;                   // K fast: 8 rows of 128 bytes per load
        const int nt = row * (SEG ? gp.k[0] : (int)g.K) + (((lane % 8) ^ swz(row)) << 4);
        const int kb = (wave + j * NW) * 4 + lane / 16;                   // K slow: 4 K-rows of 256 bytes per load
        const int chunk = ((lane % 16) ^ ((kb & 7) << 1)) << 4;
        voff_a[j] = TA ? kb * (int)g.M + chunk : nt;
        voff_b[j] = TB ? kb * (int)g.N + chunk : nt;
    }
    // SEG: the same offsets for operands of another row length (both stored [rows, K])
    auto set_voffs = [&](int nk) {
#pragma unroll
        for (int j = 0; j < LOADS; ++j) {
            const int row = (wave + j * NW) * 8 + lane / 8;
            voff_a[j] = voff_b[j] = row * nk + (((lane % 8) ^ swz(row)) << 4);
        }
    };
    const int kstep_a = TA ? 128 * (int)g.M : 128, kstep_b = TB ? 128 * (int)g.N : 128;   // bytes between K steps
    // one 1 KB direct-to-LDS load: 64 lanes x 16 bytes land at lds_addr + lane * 16
    auto dma = [&](const v4i &rsrc, uint32_t lds_addr, int vo, int so) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                     ::"s"(lds_addr), "v"(vo), "s"(rsrc), "s"(so));
    };
    auto lds_addr_of = [](const uint8_t *p) { return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) uint8_t *)p; };
    // load j of a stage: j < LOADS -> operand A, else operand B
    auto issue_one = [&](uint8_t *sa, uint8_t *sb, const v4i &da, const v4i &db, int kstep, int j) {

        if (j < LOADS) dma(da, lds_addr_of(sa) + (wave + j * NW) * 1024, voff_a[j], kstep * kstep_a);
        else dma(db, lds_addr_of(sb) + (wave + (j - LOADS) * NW) * 1024, voff_b[j - LOADS], kstep * kstep_b);
    };

    int m0 = 0, n0 = 0;
    v4i rsrc_a, rsrc_b, next_a, next_b;           // raw buffer descriptors (base, stride 0, bytes, format)


    // one 256-byte direct-to-LDS load: 64 lanes x 4 bytes land at lds_addr + lane * 4
    auto dma4 = [](const v4i &rsrc, uint32_t lds_addr, int vo, int so) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 4\n\tbuffer_load_dword %1, %2, %3 offen lds"
                     ::"s"(lds_addr), "v"(vo), "s"(rsrc), "s"(so));
    };
    // ---- block scales (MX).  One descriptor per operand covers the whole array; a tile and a K step are reached through
    // the scalar offset, and a load that must deliver nothing (rows outside the matrix, the padding step, no next tile)
    // gets the size field cleared.  Of each operand this wave fetches 64 dwords per step: LDS dword d = 64 wave + lane
    // holds tile row 128 (d / 128) + 32 (d % 4) + (d % 128) / 4, so that rows r, r + 32, r + 64, r + 96 of a wave tile
    // lie side by side.
    auto whole_scales = [&](const uint8_t *p, int64_t rows) -> v4i {
        const uint64_t addr = reinterpret_cast<uint64_t>(p);
        return v4i{(int)(uint32_t)addr, (int)(uint32_t)(addr >> 32), (int)((uint32_t)(g.K / 128) * (uint32_t)rows * 4u), 0x00020000};
    };
    const v4i whole_sa = MX ? whole_scales(g.mx_sa, g.M) : empty, whole_sb = MX ? whole_scales(g.mx_sb, g.N) : empty;
    const int sc_d = 64 * wave + lane;
    const int sc_voff = (128 * (sc_d / 128) + 32 * (sc_d % 4) + (sc_d % 128) / 4) * 4;
    const int sc_region = 128 * (wave / 2);       // first tile row of the 128 rows this wave fetches from (both operands)
    int sc_off_a = 0, sc_off_b = 0, sc_next_a = 0, sc_next_b = 0;                    // bytes to (tile row 0, the item's first K step)
    int sc_in_a = 0, sc_in_b = 0, sc_nin_a = 0, sc_nin_b = 0;                        // 1: those 128 rows exist (kept as
    // integers and applied by multiplication: selects on loop-carried flags do not stay scalar code)
    auto scale_origin = [&](int tm0, int tn0, int first_step, int &oa, int &ob, int &ia, int &ib) {
        oa = (first_step * (int)g.M + tm0) * 4;
        ob = (first_step * (int)g.N + tn0) * 4;
        ia = tm0 + sc_region < (int)g.M ? 1 : 0;
        ib = tn0 + sc_region < (int)g.N ? 1 : 0;
    };
    // one operand's 64 scale dwords of a K step (which: 0 = A, 1 = B)
    auto issue_scale = [&](int which, int stage, int ok, int off, int kstep) {
        v4i d = which ? whole_sb : whole_sa;
        d.z = __builtin_amdgcn_readfirstlane(d.z * ok);
        off = __builtin_amdgcn_readfirstlane(off);
        const uint32_t dst = lds_addr_of(reinterpret_cast<const uint8_t *>(sScale)) + (stage * 512 + which * 256 + 64 * wave) * 4;
        dma4(d, dst, sc_voff, off + kstep * (int)(which ? g.N : g.M) * 4);
    };
    auto issue_scales = [&](int stage, int ok_a, int ok_b, int off_a, int off_b, int kstep) {
        issue_scale(0, stage, ok_a, off_a, kstep);
        issue_scale(1, stage, ok_b, off_b, kstep);
    };
    int sca[2][4] = {}, scb[2][4] = {};           // [K step parity][fragment]: this lane's scale dwords, already shifted
    // in two parts, so that the shift (which waits for the data) can sit a few MFMAs after the read
    v4i sc_raw_a = {0, 0, 0, 0}, sc_raw_b = {0, 0, 0, 0};
    auto fetch_scales = [&](int stage) {
        const uint32_t *base = sScale + stage * 512;
        sc_raw_a = *reinterpret_cast<const v4i *>(base + 128 * (wave / 2) + 4 * lr);
        sc_raw_b = *reinterpret_cast<const v4i *>(base + 256 + 128 * (wave % 2) + 4 * lr);
    };
    auto place_a = [&](int (&ea)[4]) {
#pragma unroll
        for (int t = 0; t < 4; ++t) ea[t] = (int)((uint32_t)sc_raw_a[t] >> (8 * lg));
    };
    auto place_b = [&](int (&eb)[4]) {
#pragma unroll
        for (int t = 0; t < 4; ++t) eb[t] = (int)((uint32_t)sc_raw_b[t] >> (8 * lg));
    };
    auto place_scales = [&](int (&ea)[4], int (&eb)[4]) {
        place_a(ea);
        place_b(eb);
    };
    auto read_scales = [&](int stage, int (&ea)[4], int (&eb)[4]) {
        fetch_scales(stage);
        place_scales(ea, eb);
    };

    // ---- LDS -> registers.  chunk(t, h, e) = ((2*lg + e) ^ s0) ^ 4*(h ^ (t & 1))   (block scales: lg + 2*e)
    int ra[2][2], rb[2][2];                     // [e][h ^ (t & 1)] byte offsets inside a region (tile 0)
    {
        const int rowa = wm0 + lr, rowb = wn0 + lr;
        const int s0a = swz(rowa), s0b = swz(rowb);
#pragma unroll
        for (int e = 0; e < 2; ++e)
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                // which 32 of the 64 K-bytes of a half a lane takes is free without block scales (both operands agree);
                // with them the instruction's own order decides: registers 0..3 = chunk lg, registers 4..7 = chunk 2 + lg
                const int chunk = MX ? lg + 2 * e : 2 * lg + e;
                ra[e][p] = rowa * 128 + ((((chunk ^ s0a)) ^ (4 * p)) << 4);
                rb[e][p] = rowb * 128 + ((((chunk ^ s0b)) ^ (4 * p)) << 4);
            }
    }
    // K-slow layout: fragment t covers tile rows row0 + 32 t .. + 31 = the 16-byte chunks c0 + 2t, c0 + 2t + 1
    // of a K-row; a lane of a 16-lane group addresses K-row 32 lg + (lane % 16) / 2 (+ 8p, + 64h) and the
    // 8-byte half lane % 2 of chunk (c0 + 2t) ^ 2 (k & 7).  c0 has bits 0 and 3 only, so the t-dependence
    // is an XOR on the address.
    const int tj = (lane % 16) / 2;
    const int tra = (lg * 32 + tj) * 256 + ((((wm0 / 16) + (lr / 16)) ^ (tj << 1)) << 4) + (lane % 2) * 8;
    const int trb = (lg * 32 + tj) * 256 + ((((wn0 / 16) + (lr / 16)) ^ (tj << 1)) << 4) + (lane % 2) * 8;
    auto read_tr = [&](const uint8_t *sx, int lane_off, int t, int h) -> v8i {
        typedef int v2i_t __attribute__((ext_vector_type(2)));
        const uint32_t base = lds_addr_of(sx) + (uint32_t)(lane_off ^ (t << 5)) + h * 64 * 256;
        v2i_t p[4];
#pragma unroll
        for (int q = 0; q < 4; ++q)
            p[q] = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) v2i_t *)(base + q * 8 * 256));
        return v8i{p[0].x, p[0].y, p[1].x, p[1].y, p[2].x, p[2].y, p[3].x, p[3].y};
    };
    auto read_a = [&](const uint8_t *sa, int t, int h) -> v8i {
        if constexpr (TA) return read_tr(sa, tra, t, h);
        const v4i lo = *reinterpret_cast<const v4i *>(sa + ra[0][h ^ (t & 1)] + t * 4096);
        const v4i hi = *reinterpret_cast<const v4i *>(sa + ra[1][h ^ (t & 1)] + t * 4096);
        return v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    };
    auto read_b = [&](const uint8_t *sb, int u, int h) -> v8i {
        if constexpr (TB) return read_tr(sb, trb, u, h);
        const v4i lo = *reinterpret_cast<const v4i *>(sb + rb[0][h ^ (u & 1)] + u * 4096);
        const v4i hi = *reinterpret_cast<const v4i *>(sb + rb[1][h ^ (u & 1)] + u * 4096);
        return v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    };

    v16f acc[TM][TN];
    v8i a0[TM], b0[TN], a1[TM], b1[TN];         // register buffers 0 (h0) and 1 (h1)
    const v16f zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

    // ---- output side of the folded epilogue
    const int n2 = (int)g.N * ESZ;                // bytes per output row
    const int c_soff0 = (wm0 * (int)g.N + wn0) * ESZ;
    auto uniform = [](float v) { return bits_to_float((uint32_t)__builtin_amdgcn_readfirstlane((int)float_to_bits(v))); };
    // SEG: between pair s and s + 1 the accumulators take sRatio[s] = (scale product of s) / (that of s + 1); kept in
    // LDS (read once per pair) rather than in scalar registers, of which the K loop leaves none to spare
    if constexpr (SEG) {
        const int s = (int)threadIdx.x;
        if (s + 1 < gp.count) sRatio[s] = (gp.sa[s][0] * gp.sb[s][0]) / (gp.sa[s + 1][0] * gp.sb[s + 1][0]);
        // (first read after the K loop of the first pair, many barriers from here)
    }
    const float s_tensor = g.splits > 1 ? 1.0f :       // partial results leave unscaled
        SEG ? uniform(gp.sa[gp.count - 1][0] * gp.sb[gp.count - 1][0]) : uniform(g.sa[0] * g.sb[0]);
    // M and N are multiples of 128 = the wave tile: in the last tile row / column of a matrix that is not a
    // multiple of 256 a wave is either wholly inside or wholly outside.  One that is outside computes on the
    // zeros that the bounded operand loads deliver and stores through the empty descriptor (nothing is written).
    auto wave_inside = [&](int tm0, int tn0) { return tm0 + wm0 < (int)g.M && tn0 + wn0 < (int)g.N; };
    auto rsrc_out = [&](int item, int tm0, int tn0) -> v4i {
        const int split = __builtin_amdgcn_readfirstlane(item / tiles);
        const uint64_t addr = reinterpret_cast<uint64_t>(reinterpret_cast<uint8_t *>(g.c) +
                                                         ((int64_t)split * g.M * g.N + (int64_t)tm0 * g.N + tn0) * ESZ);
        const v4i whole = {(int)(uint32_t)addr, (int)(uint32_t)(addr >> 32), (int)0x80000000u, 0x00020000};
        return wave_inside(tm0, tn0) ? whole : empty;
    };
    // `us`: the slab's position in the wave tile's row, in slabs of 128 bytes
    auto store_slab = [](const u32x4 (&data)[4], int vo, const v4i &rsrc, int so_base, int row_bytes, int t, int us) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int so = so_base + (32 * t + 8 * j) * row_bytes + 128 * us;
            // s_nop 4: a scalar register written by a vector instruction (the compiler restores
            // spilled scalars that way) must not be read by a vector-memory instruction for 5
            // cycles, and the compiler does not look inside asm statements for that hazard.
            // nt: the output is not an operand of the next kernel; stored normally it sits dirty in the
            // memory-side cache and its write-back competes with the amax / cast pass that follows
            asm volatile("s_nop 4\n\tbuffer_store_dwordx4 %0, %1, %2, %3 offen nt" ::"v"(data[j]), "v"(vo), "s"(rsrc), "s"(so));
        }
    };
    auto lds_w = [](uint32_t addr) { return (__attribute__((address_space(3))) u32x2 *)addr; };
    auto lds_r = [](uint32_t addr) -> u32x4 {   // 16 bytes as two 8-byte reads: slab rows are only 8-byte aligned
        const u32x2 lo = *(const __attribute__((address_space(3))) u32x2 *)addr;
        const u32x2 hi = *(const __attribute__((address_space(3))) u32x2 *)(addr + 8);
        return u32x4{lo.x, lo.y, hi.x, hi.y};
    };

    // phase A of a step: MFMA i works on sub-tile (t, u) = (i / 4, i % 4); the 8 fragments of
    // (kt, h1) stream into buffer 1 behind the first 8 MFMAs.
    auto phase_a = [&](const uint8_t *sa_cur, const uint8_t *sb_cur, const int par) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            acc[i / 4][i % 4] = mma_step<FB, FA, MX, 0>(b0[i % 4], a0[i / 4], acc[i / 4][i % 4], scb[par][i % 4], sca[par][i / 4]);
#ifdef ODL_EXP_HALF_LDS_READS         // experiment: the second K half multiplies the fragments of the first again
            if (i < 4) a1[i] = a0[i];
            else if (i < 8) b1[i - 4] = b0[i - 4];
#else
            if (i < 4) a1[i] = read_a(sa_cur, i, 1);
            else if (i < 8) b1[i - 4] = read_b(sb_cur, i - 4, 1);
#endif
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    // phase A of step 0 of the first tile: accumulators start from zero
    auto phase_a_first = [&](const uint8_t *sa_cur, const uint8_t *sb_cur) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            acc[i / 4][i % 4] = mma_step<FB, FA, MX, 0>(b0[i % 4], a0[i / 4], zero16, scb[0][i % 4], sca[0][i / 4]);
            if (i < 4) a1[i] = read_a(sa_cur, i, 1);
            else if (i < 8) b1[i - 4] = read_b(sb_cur, i - 4, 1);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    // SEG, phase A of step 0 of a later operand pair of the same tile: the accumulators carry on, multiplied by the
    // ratio of the two pairs' scale products (sub-tile i while MFMA i - 1 runs)
    auto phase_a_rescale = [&](const uint8_t *sa_cur, const uint8_t *sb_cur, const int pair) {
        const float ratio = sRatio[pair];
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            // (the statement makes this read of the accumulators another one than the fold's, for the compiler: it would
            // otherwise read them out once, ahead of the branch between the two, into registers that do not exist)
            asm volatile("" : "+a"(acc[i / 4][i % 4]));
            v16f carried;
#pragma unroll
            for (int e = 0; e < 16; ++e) carried[e] = acc[i / 4][i % 4][e] * ratio;
            acc[i / 4][i % 4] = mma_step<FB, FA, MX, 0>(b0[i % 4], a0[i / 4], carried, scb[0][i % 4], sca[0][i / 4]);
            if (i < 4) a1[i] = read_a(sa_cur, i, 1);
            else if (i < 8) b1[i - 4] = read_b(sb_cur, i - 4, 1);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    // phase A of step 0 of a later tile (or the drain after the last one): the finished tile
    // leaves through `rsrc_c` while its accumulators are restarted from zero.
    //   bf16: sub-tiles (t, u), (t, u + 1) make one slab of 32 rows x 64 columns; it is read back after
    //         the odd one and stored one MFMA later
    //   fp32: every sub-tile is a slab of 32 rows x 32 floats, read back at once and stored one MFMA later
    // EPI > 0: the wave's slices of the scale vectors (and of the bias) were brought to LDS by
    // `request_vectors`; those of sub-tile i + 1 are read while MFMA i runs.
    auto phase_a_fold = [&](const uint8_t *sa_cur, const uint8_t *sb_cur, const v4i &rsrc_c) {
        // addresses are derived here (laundered ids), not kept in registers across the K loop
        int lane_e = lane, wave_e = wave;
        asm volatile("" : "+v"(lane_e));
        asm volatile("" : "+s"(wave_e));
        const uint32_t slab = lds_addr_of(sEpi) + wave_e * SLAB;
        const uint32_t epi_w = slab + (lane_e % 32) * PITCH + (lane_e / 32) * (F32 ? 16 : 8);
        const uint32_t epi_r = slab + (lane_e / 8) * PITCH + (lane_e % 8) * 16;
        const int c_voff = (lane_e / 8) * n2 + (lane_e % 8) * 16;
        const uint32_t vec_row = lds_addr_of(sVec) + wave_e * VEC_BYTES + (lane_e % 32) * 4;          // sa of row lr
        const uint32_t vec_col = lds_addr_of(sVec) + wave_e * VEC_BYTES + 512 + (lane_e / 32) * 16;   // sb of columns 4 lg ..
        float sa_next = 0.0f;
        f32x4 sb_next[4], bias_next[4];
        auto read_vectors = [&](int t, int u) {
            sa_next = *(const __attribute__((address_space(3))) float *)(vec_row + t * 128);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                sb_next[q] = *(const __attribute__((address_space(3))) f32x4 *)(vec_col + u * 128 + q * 32);
                if constexpr (EPI == 2) bias_next[q] = *(const __attribute__((address_space(3))) f32x4 *)(vec_col + 512 + u * 128 + q * 32);
            }
        };
        if constexpr (EPI > 0) read_vectors(0, 0);
        u32x4 back[4];
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int t = i / 4, u = i % 4;
            float v[16];
            if constexpr (EPI > 0) {
#pragma unroll
                for (int q = 0; q < 4; ++q)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        v[4 * q + e] = acc[t][u][4 * q + e] * (sa_next * sb_next[q][e]);
                        if constexpr (EPI == 2) v[4 * q + e] = v[4 * q + e] + bias_next[q][e];
                    }
            } else {
#pragma unroll
                for (int e = 0; e < 16; ++e) v[e] = acc[t][u][e] * s_tensor;
            }
            uint32_t pk[8];
            if constexpr (!F32) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    pk[2 * q] = pack_bf16x2(v[4 * q], v[4 * q + 1]);
                    pk[2 * q + 1] = pack_bf16x2(v[4 * q + 2], v[4 * q + 3]);
                }
            }
            acc[t][u] = mma_step<FB, FA, MX, 0>(b0[u], a0[t], zero16, scb[0][u], sca[0][t]);
            if constexpr (EPI > 0) {
                if (i < 15) read_vectors((i + 1) / 4, (i + 1) % 4);
            }
            if constexpr (F32) {
                if (i > 0) store_slab(back, c_voff, rsrc_c, c_soff0, n2, (i - 1) / 4, (i - 1) % 4);
                // lane (lr, lg) holds columns 8q + 4lg + {0..3} of row lr: 16 bytes at 32q + 16lg, as two 8-byte
                // writes (the row pitch of 34 dwords spreads the 32 rows of a half-wave over all 64 banks)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    *lds_w(epi_w + q * 32) = u32x2{float_to_bits(v[4 * q]), float_to_bits(v[4 * q + 1])};
                    *lds_w(epi_w + q * 32 + 8) = u32x2{float_to_bits(v[4 * q + 2]), float_to_bits(v[4 * q + 3])};
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) back[j] = lds_r(epi_r + j * 8 * PITCH);
            } else {
                // lane (lr, lg) holds columns 8q + 4lg + {0..3} of row lr of the sub-tile.  With a row
                // pitch of 34 dwords the 8-byte writes of 16 consecutive rows cover all 32 banks once,
                // and so do the 8-byte halves of the row-wise reads of two consecutive rows.
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    *lds_w(epi_w + (u & 1) * 64 + q * 16) = u32x2{pk[2 * q], pk[2 * q + 1]};
                if (u & 1) {
                    // slab complete: 8 lanes cover a row with 16 bytes each, 8 rows per instruction.
                    // LDS operations of a wave execute in order, so the next writes cannot overtake these reads.
#pragma unroll
                    for (int j = 0; j < 4; ++j) back[j] = lds_r(epi_r + j * 8 * PITCH);
                } else if (i > 0) {
                    store_slab(back, c_voff, rsrc_c, c_soff0, n2, (i - 2) / 4, ((i - 2) % 4) / 2);   // completed one MFMA ago
                }
            }
            if (i < 4) a1[i] = read_a(sa_cur, i, 1);
            else if (i < 8) b1[i - 4] = read_b(sb_cur, i - 4, 1);
            __builtin_amdgcn_sched_barrier(0);
        }
        store_slab(back, c_voff, rsrc_c, c_soff0, n2, 3, F32 ? 3 : 1);
        __builtin_amdgcn_sched_barrier(0);
    };
    // EPI > 0: this wave's 128 row scales, 128 column scales (and 128 bias values) of the tile at (tm0, tn0)
    // go straight to LDS, 64 floats per load.  A vector that is a single value is read with stride 0; the
    // loads are issued one K step before the tile ends and are covered by that step's vmcnt(0).
    auto request_vectors = [&](int tm0, int tn0) {
        const uint32_t dst = lds_addr_of(sVec) + wave * VEC_BYTES;
        auto rsrc_vec = [](const void *p, int64_t count) -> v4i {
            const uint64_t addr = reinterpret_cast<uint64_t>(p);
            return v4i{(int)(uint32_t)addr, (int)(uint32_t)(addr >> 32), (int)(count * 4), 0x00020000};
        };
        // the bounds of a descriptor cover the per-lane offset only, not the scalar one: a wave outside the matrix
        // must not request its (non-existent) slices at all
        const bool inside = wave_inside(tm0, tn0);
        const v4i ra_ = inside ? rsrc_vec(g.sa, g.sa_vec ? g.M : 1) : empty, rb_ = inside ? rsrc_vec(g.sb, g.sb_vec ? g.N : 1) : empty;
        const int va = lane * 4 * g.sa_vec, vb = lane * 4 * g.sb_vec;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            dma4(ra_, dst + j * 256, va, (tm0 + wm0 + 64 * j) * 4 * g.sa_vec);
            dma4(rb_, dst + 512 + j * 256, vb, (tn0 + wn0 + 64 * j) * 4 * g.sb_vec);
        }
        if constexpr (EPI == 2) {
            const v4i rc_ = inside ? rsrc_vec(g.bias, g.N) : empty;
#pragma unroll
            for (int j = 0; j < 2; ++j) dma4(rc_, dst + 1024 + j * 256, lane * 4, (tn0 + wn0 + 64 * j) * 4);
        }
    };
    auto sync = [&](bool after_fold) {
        if (after_fold) __builtin_amdgcn_s_waitcnt(F32 ? 0xC07F : 0x8070);   // vmcnt(63 | 32) lgkmcnt(0)
        else __builtin_amdgcn_s_waitcnt(0x0070);                     // vmcnt(0)  lgkmcnt(0)
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
    };
    // phase B: MFMAs on buffer 1; (kt+1, h0) streams into buffer 0; step kt+2 is requested into
    // the stage just consumed -- from the next tile when this tile has no such step
    auto phase_b = [&](uint8_t *sa_cur, uint8_t *sb_cur, const uint8_t *sa_nxt, const uint8_t *sb_nxt, int kt, const int par) {
        const bool nx = kt + 2 >= KT;
        const bool pad = padded && kt + 3 == KT;                  // the step requested is the padding step
        // (a nested select between three descriptors is not compiled as scalar code; the padding step
        // instead clears the size field, which makes every load of the step read zeros)
        v4i la = nx ? next_a : rsrc_a, lb = nx ? next_b : rsrc_b;
        la.z = pad && !nx ? 0 : la.z;
        lb.z = pad && !nx ? 0 : lb.z;
        const int koff = nx ? kt + 2 - KT : kt + 2;               // K step to request
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            acc[i / 4][i % 4] = mma_step<FB, FA, MX, 1>(b1[i % 4], a1[i / 4], acc[i / 4][i % 4], scb[par][i % 4], sca[par][i / 4]);
            if (i < 4) a0[i] = read_a(sa_nxt, i, 0);
            else if (i < 8) b0[i - 4] = read_b(sb_nxt, i - 4, 0);
            issue_one(sa_cur, sb_cur, la, lb, koff, i);
            if constexpr (MX) {
                // the scales of step kt + 1 arrived with its operands; those of the step requested above go to the stage
                // whose dwords every wave read one phase B ago
                // spread over the MFMA slots that carry no fragment reads (i >= 8), one small piece each: a slot has room
                // for about a dozen instructions beside its MFMA
                const int live = pad && !nx ? 0 : 1;
                if (i == 8) fetch_scales(par ^ 1);
                if (i == 9) issue_scale(0, par, (nx ? sc_nin_a : sc_in_a) * live, nx ? sc_next_a : sc_off_a, koff);
                if (i == 10) issue_scale(1, par, (nx ? sc_nin_b : sc_in_b) * live, nx ? sc_next_b : sc_off_b, koff);
                if (i == 12) place_a(sca[par ^ 1]);
                if (i == 14) place_b(scb[par ^ 1]);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    auto step = [&](uint8_t *sa_cur, uint8_t *sb_cur, uint8_t *sa_nxt, uint8_t *sb_nxt, int kt, const int par) {
        phase_a(sa_cur, sb_cur, par);
        sync(false);
        phase_b(sa_cur, sb_cur, sa_nxt, sb_nxt, kt, par);
    };

    // ---- first tile: steps 0 and 1 requested and awaited, then phase A of step 0
    tile_origin(pid, m0, n0);
    int seg = 0;                                  // SEG: the operand pair the block is on
    if constexpr (SEG) {
        KT = gp.k[0] / 128;                    // an even number of steps, at least 4 (checked by the caller)
        rsrc_a = rsrc_for(gp.a[0], m0, g.M, false, 0, gp.k[0]);
        rsrc_b = rsrc_for(gp.b[0], n0, g.N, false, 0, gp.k[0]);
    } else {
        int first_step = 0;
        item_steps(pid, first_step, KT, padded);
        rsrc_a = rsrc_for(g.a, m0, g.M, TA, first_step, (int)g.K);
        rsrc_b = rsrc_for(g.b, n0, g.N, TB, first_step, (int)g.K);
        if constexpr (MX) scale_origin(m0, n0, first_step, sc_off_a, sc_off_b, sc_in_a, sc_in_b);
    }
    next_a = empty;
    next_b = empty;
#pragma unroll
    for (int j = 0; j < 2 * LOADS; ++j) issue_one(sA0, sB0, rsrc_a, rsrc_b, 0, j);
#pragma unroll
    for (int j = 0; j < 2 * LOADS; ++j) issue_one(sA1, sB1, rsrc_a, rsrc_b, 1, j);
    if constexpr (MX) {
        issue_scales(0, sc_in_a, sc_in_b, sc_off_a, sc_off_b, 0);
        issue_scales(1, sc_in_a, sc_in_b, sc_off_a, sc_off_b, 1);
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);          // vmcnt(0)
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if constexpr (MX) read_scales(0, sca[0], scb[0]);
#pragma unroll
    for (int t = 0; t < TM; ++t) a0[t] = read_a(sA0, t, 0);
#pragma unroll
    for (int u = 0; u < TN; ++u) b0[u] = read_b(sB0, u, 0);
    phase_a_first(sA0, sB0);

    // One trip: the rest of the current item (a tile; SEG: one operand pair of a tile) and phase A of the next.
    // ENDS: the item ends its tile (always, without SEG).  -> whether the block has another item.
    auto trip = [&](auto ends_tile) -> bool {
        constexpr bool tile_ends = decltype(ends_tile)::value;
        // the block's next tile, if any (scalar work only; no branches around vector code).  SEG: the next operand pair
        // of this tile, or the first pair of the next tile
        const int next_seg = tile_ends ? 0 : seg + 1;
        const int next_pid = tile_ends ? pid + stride : pid;
        const bool has_next = next_pid < pid_end;
        int next_m0 = 0, next_n0 = 0, next_first = 0, next_kt = 0;
        bool next_padded = false;
        tile_origin(has_next ? next_pid : pid, next_m0, next_n0);
        const int next_nk = SEG ? gp.k[next_seg] : (int)g.K;
        if constexpr (SEG) next_kt = next_nk / 128;
        else item_steps(has_next ? next_pid : pid, next_first, next_kt, next_padded);
        const uint8_t *const base_a = SEG ? gp.a[next_seg] : g.a, *const base_b = SEG ? gp.b[next_seg] : g.b;
#ifdef ODL_EXP_SAME_PANELS            // experiment: every tile reads the operand panels of tile (0, 0): all traffic stays in the L2
        const v4i na = rsrc_for(base_a, 0, g.M, TA, next_first, next_nk), nb = rsrc_for(base_b, 0, g.N, TB, next_first, next_nk);
#else
        const v4i na = rsrc_for(base_a, next_m0, g.M, TA, next_first, next_nk), nb = rsrc_for(base_b, next_n0, g.N, TB, next_first, next_nk);
#endif
        next_a = has_next ? na : empty;
        next_b = has_next ? nb : empty;
        if constexpr (MX) {
            scale_origin(next_m0, next_n0, next_first, sc_next_a, sc_next_b, sc_nin_a, sc_nin_b);
            sc_nin_a *= has_next ? 1 : 0;
            sc_nin_b *= has_next ? 1 : 0;
        }

        // ---- rest of step 0 (its phase A ran at the end of the previous trip), then steps 1 .. KT-1.
        // The first trip's step 0 and every drained tile's step 0 carry 32 stores (dropped ones
        // count too), the first tile's none: vmcnt(32) is then simply satisfied earlier.
        // SEG: a later pair of a tile follows a rescale, which stores nothing: every load must have landed
        if (SEG && seg > 0) sync(false);
        else sync(true);
        phase_b(sA0, sB0, sA1, sB1, 0, 0);
        step(sA1, sB1, sA0, sB0, 1, 1);
        for (int kt = 2; kt < KT - 2; kt += 2) {
            step(sA0, sB0, sA1, sB1, kt, 0);
            step(sA1, sB1, sA0, sB0, kt + 1, 1);
        }
        // the two steps that follow request the next item's first two: its row pitch from here on
        if constexpr (SEG) set_voffs(next_nk);
        step(sA0, sB0, sA1, sB1, KT - 2, 0);
        if constexpr (EPI > 0) request_vectors(m0, n0);
        step(sA1, sB1, sA0, sB0, KT - 1, 1);

        // ---- the tile is finished; buffer 0 already holds the next tile's first fragments.
        // Phase A of the next tile's step 0 stores this tile.  Without a next tile the same
        // phase runs on whatever the empty buffer delivered, only for its stores.
        const v4i rsrc_c = rsrc_out(pid, m0, n0);
        pid = next_pid;
        KT = next_kt;
        padded = next_padded;
        m0 = next_m0;
        n0 = next_n0;
        rsrc_a = next_a;
        rsrc_b = next_b;
        sc_off_a = sc_next_a;
        sc_off_b = sc_next_b;
        sc_in_a = sc_nin_a;
        sc_in_b = sc_nin_b;
        const int pair = seg;
        seg = next_seg;
        if constexpr (tile_ends) phase_a_fold(sA0, sB0, rsrc_c);
        else phase_a_rescale(sA0, sB0, pair);
        return has_next;
    };
    if constexpr (SEG) {
        // two copies of the trip, one ending in the rescale and one in the fold, instead of a branch between the two at
        // the end of one: with the branch the compiler does not keep the accumulators where they are (it spills them)
        while (true) {
            while (seg + 1 < gp.count) trip(std::false_type{});
            if (!trip(std::true_type{})) break;
        }
    } else {
        while (trip(std::true_type{})) {
        }
    }
    if (stamps) {
        g.clock_out[2] = clock64();
        g.clock_out[3] = wall_clock64();
    }
}

template <int FA, int FB, bool TA, bool TB, bool F32, int EPI, bool MX = false>
__global__ __launch_bounds__(256) void gemm_nt_stream_kernel(const GemmArgs g) {
    gemm_nt_stream_body<FA, FB, TA, TB, F32, EPI, MX, false>(g, GemmPairs{});
}

// the same kernel over several operand pairs (see SEG above)
template <int FA, int FB, bool F32>
__global__ __launch_bounds__(256) void gemm_nt_stream_pairs_kernel(const GemmArgs g, const GemmPairs gp) {
    gemm_nt_stream_body<FA, FB, false, false, F32, 0, false, true>(g, gp);
}

template <int FA, int FB, bool F32>
void launch_out(const GemmArgs &g, int blocks_per_xcd, hipStream_t stream) {
    const dim3 grid((unsigned)(8 * blocks_per_xcd)), block(256);
    const bool vectors = g.splits == 1 && (g.bias || g.sa_vec || g.sb_vec);     // partial results carry no scales
    if (g.mx_sa) {
        if (vectors) hipLaunchKernelGGL((gemm_nt_stream_kernel<FA, FB, false, false, F32, 2, true>), grid, block, 0, stream, g);
        else hipLaunchKernelGGL((gemm_nt_stream_kernel<FA, FB, false, false, F32, 0, true>), grid, block, 0, stream, g);
    } else if (vectors && g.bias) hipLaunchKernelGGL((gemm_nt_stream_kernel<FA, FB, false, false, F32, 2>), grid, block, 0, stream, g);
    else if (vectors) hipLaunchKernelGGL((gemm_nt_stream_kernel<FA, FB, false, false, F32, 1>), grid, block, 0, stream, g);
    else if (g.ta && g.tb) hipLaunchKernelGGL((gemm_nt_stream_kernel<FA, FB, true, true, F32, 0>), grid, block, 0, stream, g);
    else if (g.tb) hipLaunchKernelGGL((gemm_nt_stream_kernel<FA, FB, false, true, F32, 0>), grid, block, 0, stream, g);
    else if (g.ta) hipLaunchKernelGGL((gemm_nt_stream_kernel<FA, FB, true, false, F32, 0>), grid, block, 0, stream, g);
    else hipLaunchKernelGGL((gemm_nt_stream_kernel<FA, FB, false, false, F32, 0>), grid, block, 0, stream, g);
}

template <int FA, int FB>
void launch_fmt(const GemmArgs &g, int blocks_per_xcd, hipStream_t stream) {
    if (g.out_dtype == ODL_F32 || g.splits > 1) launch_out<FA, FB, true>(g, blocks_per_xcd, stream);
    else launch_out<FA, FB, false>(g, blocks_per_xcd, stream);
}

}  // namespace

// Shapes this kernel takes (the caller checks the 32-bit offset limits shared with gemm_pipe.hip).
// An operand stored [K, rows] must fill whole tiles: the loads of a partial tile would run past the
// end of its last K-row.  One stored [rows, K] may end after half a tile (see wave_inside).
bool gemm_stream_accepts(const GemmArgs &g) {
    const double esz = (g.out_dtype == ODL_F32 || g.splits > 1) ? 4.0 : 2.0;
    const bool vectors = g.splits == 1 && (g.sa_vec || g.sb_vec || g.bias != nullptr);   // only with both operands stored [rows, K]
    if (g.mx_sa && (g.ta || g.tb || g.sa_vec || g.sb_vec || !g.mx_sb)) return false;
    return !g.accumulate && (g.out_dtype == ODL_BF16 || g.out_dtype == ODL_F32) && !(vectors && (g.ta || g.tb)) &&
           g.M % (g.ta ? BM : WM) == 0 && g.N % (g.tb ? BN : WN) == 0 && g.K % 128 == 0 && g.K >= 512 && (double)g.N * esz * (BM + 8) < 2147483648.0;
}

// Operand pairs: each a whole even number of K steps, four at least (the load pipeline is two steps deep and crosses
// from one pair to the next in its last two), every operand addressed with 32-bit byte offsets.
bool gemm_stream_accepts_pairs(const GemmArgs &g, const GemmPairs &gp) {
    const double esz = g.out_dtype == ODL_F32 ? 4.0 : 2.0;
    if (gp.count < 1 || gp.count > 4 || g.accumulate || g.ta || g.tb || g.sa_vec || g.sb_vec || g.bias || g.mx_sa || g.mx_sb || g.splits > 1)
        return false;
    for (int s = 0; s < gp.count; ++s) {
        const int k = gp.k[s];
        if (!gp.a[s] || !gp.b[s] || !gp.sa[s] || !gp.sb[s] || k < 512 || k % 256 != 0) return false;
        if ((double)(g.M + 256) * k >= 2147483648.0 || (double)(g.N + 256) * k >= 2147483648.0) return false;
    }
    return (g.out_dtype == ODL_BF16 || g.out_dtype == ODL_F32) && g.M > 0 && g.N > 0 && g.M % WM == 0 && g.N % WN == 0 &&
           (double)g.N * esz * (BM + 8) < 2147483648.0;
}

// One block per CU at most (the kernel needs ~150 KB of LDS), 8 | grid so that the
// round-robin placement gives every XCD the same number of blocks.
void launch_gemm_stream(int fa, int fb, const GemmArgs &args, int num_cus, hipStream_t stream) {
    GemmArgs g = args;
    if (g.splits <= 1) {
        g.splits = 1;
        g.split_steps = ((int)(g.K / 128) + 1) & ~1;
    }
    const int total = g.tiles_m * g.tiles_n * g.splits;
    const int per_xcd = (total + 7) / 8;
    int bpx = num_cus / 8;
    if (bpx < 1) bpx = 1;
    if (bpx > per_xcd) bpx = per_xcd;
    if (fa == ODL_FP8_E4M3 && fb == ODL_FP8_E4M3) launch_fmt<ODL_FP8_E4M3, ODL_FP8_E4M3>(g, bpx, stream);
    else if (fa == ODL_FP8_E5M2 && fb == ODL_FP8_E4M3) launch_fmt<ODL_FP8_E5M2, ODL_FP8_E4M3>(g, bpx, stream);
    else if (fa == ODL_FP8_E4M3 && fb == ODL_FP8_E5M2) launch_fmt<ODL_FP8_E4M3, ODL_FP8_E5M2>(g, bpx, stream);
    else launch_fmt<ODL_FP8_E5M2, ODL_FP8_E5M2>(g, bpx, stream);
}

namespace {

template <int FA, int FB>
void launch_pairs_fmt(const GemmArgs &g, const GemmPairs &gp, int blocks_per_xcd, hipStream_t stream) {
    const dim3 grid((unsigned)(8 * blocks_per_xcd)), block(256);
    if (g.out_dtype == ODL_F32) hipLaunchKernelGGL((gemm_nt_stream_pairs_kernel<FA, FB, true>), grid, block, 0, stream, g, gp);
    else hipLaunchKernelGGL((gemm_nt_stream_pairs_kernel<FA, FB, false>), grid, block, 0, stream, g, gp);
}

}  // namespace

void launch_gemm_stream_pairs(int fa, int fb, const GemmArgs &args, const GemmPairs &gp, int num_cus, hipStream_t stream) {
    GemmArgs g = args;
    g.splits = 1;
    g.split_steps = 0;
    const int per_xcd = (g.tiles_m * g.tiles_n + 7) / 8;
    int bpx = num_cus / 8;
    if (bpx < 1) bpx = 1;
    if (bpx > per_xcd) bpx = per_xcd;
    if (fa == ODL_FP8_E4M3 && fb == ODL_FP8_E4M3) launch_pairs_fmt<ODL_FP8_E4M3, ODL_FP8_E4M3>(g, gp, bpx, stream);
    else if (fa == ODL_FP8_E5M2 && fb == ODL_FP8_E4M3) launch_pairs_fmt<ODL_FP8_E5M2, ODL_FP8_E4M3>(g, gp, bpx, stream);
    else if (fa == ODL_FP8_E4M3 && fb == ODL_FP8_E5M2) launch_pairs_fmt<ODL_FP8_E4M3, ODL_FP8_E5M2>(g, gp, bpx, stream);
    else launch_pairs_fmt<ODL_FP8_E5M2, ODL_FP8_E5M2>(g, gp, bpx, stream);
}

}  // namespace odl
