// Block-scaled FP8 on gfx950.  MXFP8: blocks of 32 consecutive elements along the contraction axis share a power-of-two
// scale (one E8M0 byte, value 2^(byte - 127)), and the MFMA applies the scales itself (V_MFMA_SCALE_F32_32X32X64_F8F6F4:
// the 64 K-bytes of a row that one instruction consumes are two blocks, each with its scale byte).  The blockwise recipe
// (128-element and 128 x 128 blocks with power-of-two scales) rides on the same GEMMs: its cast writes every block's byte
// four times.
//
//   odl_fp8_mx_cast       : x [rows, cols] -> codes + scale bytes with the blocks along the columns (`out`, `scales`)
//                           and / or, transposed, with the blocks along the rows (`out_t`, `scales_t`); one pass over x,
//                           no amax pass before it: the scale of a block is found inside the tile.
//   odl_fp8_block_cast    : the same for the blockwise recipe.
//   odl_fp8_mx_gemm_nt    : C[M, N] = sum over blocks kb of 2^(sa[m, kb] + sb[n, kb] - 254) * dot(A[m, kb], B[n, kb]); the
//                           streaming kernel of gemm_stream.hip with block scales where the shape allows, else the
//                           tiled or the plain kernel of this file.
//   odl_fp8_mx_gemm_splitk: the same with K cut into runs (outputs of few tiles).
//
// Operand layout of the instruction, measured (one nonzero byte at a time against two different block scales): of the
// 8 registers a lane supplies for row (lane % 32), registers 0..3 are the 16 K-bytes [16 g, 16 g + 16) and registers
// 4..7 the 16 K-bytes [32 + 16 g, 32 + 16 g + 16), g = lane / 32; the products of registers 0..3 of ALL lanes (K 0..31)
// take the scale byte supplied by lanes 0..31, those of registers 4..7 (K 32..63) the byte supplied by lanes 32..63.
//
// Conversion rule (OCP Microscaling Formats v1.0, 6.3): shared exponent = floor(log2(block amax)) - emax of the element
// format (8 for E4M3, 15 for E5M2), clamped to [-127, 127]; elements = rne(clamp(v * 2^-shared, +-fp8_max)).  A block of
// zeros gets byte 0, a block holding Inf / NaN gets 0xFF (a NaN scale: the products it enters are NaN).  The element
// conversion is one instruction per two elements (the scaled conversions of gfx950, see cvt_scaled_bf16x2); only blocks
// that hold Inf / NaN are converted step by step.
#include <hip/hip_runtime.h>

#include "common.h"
#include "ct_tile.h"
#include "gemm_common.h"

namespace odl {

constexpr int kMxBlock = 32;
constexpr int kMxThreads = 256;

// Where the scale byte of (row, block) lives.  Row-major: [rows][blocks].  K-step-major: [blocks / 4][rows][4], i.e.
// the 4 bytes a row needs for one 128-byte K step of a GEMM are one dword and the dwords of consecutive rows are
// consecutive: what the GEMM kernels fetch per step is contiguous (blocks % 4 == 0).
__device__ __forceinline__ int64_t mx_scale_at(int kstep_major, int64_t row, int64_t block, int64_t rows, int64_t blocks) {
    return kstep_major ? ((block >> 2) * rows + row) * 4 + (block & 3) : row * blocks + block;
}

template <int FMT> struct MxEmax { static constexpr int value = FMT == ODL_FP8_E5M2 ? 15 : 8; };

// magnitude bits (fp32 layout) of a block's amax -> scale byte and the multiplier 2^-shared
// rule 0 (ODL_MX_SCALE_FLOOR): floor(log2 amax) - emax.  rule 1 (ODL_MX_SCALE_CEIL): ceil(log2(amax / fp8_max)); fp8_max is
// 1.75 * 2^emax in both formats, so that is one more than the floor exactly when amax's mantissa exceeds 1.75.
template <int FMT>
__device__ __forceinline__ void mx_scale_of(uint32_t amax_bits, int rule, uint32_t &byte, float &mul) {
    if (amax_bits >= 0x7f800000u) { byte = 0xffu; mul = 1.0f; return; }     // Inf / NaN in the block
    if (amax_bits == 0) { byte = 0u; mul = 1.0f; return; }
    // floor(log2): the exponent field, or for a subnormal (only bf16 / fp32 subnormal inputs) the position of its top bit
    int e = (int)(amax_bits >> 23) - 127;
    if ((amax_bits >> 23) == 0) e = -127 - (__builtin_clz(amax_bits) - 9);   // mantissa bit 22 is 2^-127
    int se = e - MxEmax<FMT>::value;
    // (a subnormal amax ends at the lower clamp whatever its mantissa; its mantissa field is not normalised)
    se += (rule != 0 && (amax_bits & 0x7fffffu) > 0x600000u && (amax_bits >> 23) != 0) ? 1 : 0;
    se = se < -127 ? -127 : se;                                            // (the upper clamp cannot be reached: e <= 127)
    byte = (uint32_t)(se + 127);
    mul = bits_to_float((uint32_t)(127 - se) << 23);                       // 2^-se, 127 - se in [8, 254]
}

// Maxima across lanes without the LDS crossbar: DPP inside a row of 16 lanes, and the two swap instructions of gfx950
// (v_permlane16_swap exchanges the odd rows of one register with the even rows of another, v_permlane32_swap the wave's
// halves: applied to two copies of a value they leave "mine" in one and "my partner's" in the other).
template <int CTRL>
__device__ __forceinline__ uint32_t max_with_dpp(uint32_t m) {
    return max(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, CTRL, 0xf, 0xf, false));
}
// over the 4 lanes l ^ {0, 1, 2, 3}
__device__ __forceinline__ uint32_t max_quad(uint32_t m) {
    m = max_with_dpp<0xB1>(m);            // quad_perm [1, 0, 3, 2]
    return max_with_dpp<0x4E>(m);         // quad_perm [2, 3, 0, 1]
}
// over the 8 lanes l ^ {0, 8, 16, 24, 32, 40, 48, 56}
__device__ __forceinline__ uint32_t max_stride8(uint32_t m) {
    m = max_with_dpp<0x128>(m);           // row_ror:8 = lane ^ 8 inside a row of 16
    const auto r = __builtin_amdgcn_permlane16_swap(m, m, false, false);
    m = max(r[0], r[1]);
    const auto q = __builtin_amdgcn_permlane32_swap(m, m, false, false);
    return max(q[0], q[1]);
}

// the same for a pair of 16-bit magnitudes per lane
__device__ __forceinline__ uint32_t max_stride8_u16x2(uint32_t m) {
    m = max_u16x2(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x128, 0xf, 0xf, false));
    const auto r = __builtin_amdgcn_permlane16_swap(m, m, false, false);
    m = max_u16x2(r[0], r[1]);
    const auto q = __builtin_amdgcn_permlane32_swap(m, m, false, false);
    return max_u16x2(q[0], q[1]);
}

// gfx950's scaled conversions: two bf16 (or two floats) divided by 2^(E - 127), E = the exponent field of `scale` (an
// E8M0 byte sitting where a float keeps its exponent; mantissa and sign are ignored and E = 0 acts as 2^-127), rounded
// to nearest even into the two FP8 bytes of the low (HIGH = false) or the high half of `old`.  With MODE.FP16_OVFL set
// (saturate_fp8_conversions) a result beyond the format's largest value becomes that value.  Measured on all 65536
// bf16 inputs, both sources and both formats, at 16 exponents from 0 to 254: bit for bit round(clamp(v * 2^(127 - E))),
// the rule of the block-scaled casts, for every input except NaN (0xFF / 0xFE whatever the sign), which the kernels
// therefore keep away from these instructions.
typedef short v2i16_t __attribute__((ext_vector_type(2)));
typedef __bf16 v2bf16_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ void saturate_fp8_conversions() {
    __builtin_amdgcn_s_setreg(1 | (23 << 6) | (0 << 11), 1);          // hwreg(HW_REG_MODE, 23, 1) = FP16_OVFL, this wave only
}

template <int FMT, bool HIGH>
__device__ __forceinline__ uint32_t cvt_scaled_bf16x2(uint32_t old, uint32_t pair, float scale) {
    const v2i16_t o = __builtin_bit_cast(v2i16_t, old);
    const v2bf16_t v = __builtin_bit_cast(v2bf16_t, pair);
    if constexpr (FMT == ODL_FP8_E4M3) return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(o, v, scale, HIGH));
    else return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf8_bf16(o, v, scale, HIGH));
}

template <int FMT, bool HIGH>
__device__ __forceinline__ uint32_t cvt_scaled_f32x2(uint32_t old, float a, float b, float scale) {
    const v2i16_t o = __builtin_bit_cast(v2i16_t, old);
    if constexpr (FMT == ODL_FP8_E4M3) return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(o, a, b, scale, HIGH));
    else return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf8_f32(o, a, b, scale, HIGH));
}

// four codes from two dwords of bf16 pairs (SRC bf16: p0, p1) or four floats (SRC fp32: p0 .. p3 as bits), one scale
template <int SRC, int FMT>
__device__ __forceinline__ uint32_t cvt_scaled4(uint32_t p0, uint32_t p1, uint32_t p2, uint32_t p3, float scale) {
    if constexpr (SRC == ODL_BF16) {
        return cvt_scaled_bf16x2<FMT, true>(cvt_scaled_bf16x2<FMT, false>(0u, p0, scale), p1, scale);
    } else {
        return cvt_scaled_f32x2<FMT, true>(cvt_scaled_f32x2<FMT, false>(0u, bits_to_float(p0), bits_to_float(p1), scale),
                                           bits_to_float(p2), bits_to_float(p3), scale);
    }
}

// 128 x 64 tile per block of 256 lanes, lane (tx, ty) owns rows 4 ty .. 4 ty + 3 and two groups of 4 columns as in
// cast_transpose_kernel: bf16 source, columns 8 tx .. 8 tx + 7, so a block along the columns (32 of them) is held by 4
// neighbouring lanes; fp32 source, columns 4 tx .. + 3 and 32 + 4 tx .. + 3 (every load instruction contiguous over the
// 8 lanes of a row), so the first groups of the 8 lanes are one block and the second groups the other.  A block along
// the rows (32 of them) is held by the 8 lanes of a wave that share tx.  All maxima are exchanges inside the wave.
template <int SRC, int FMT, bool WANT_ROW, bool WANT_COL>
__global__ __launch_bounds__(kMxThreads) void mx_cast_kernel(const void *__restrict__ x, int64_t rows, int64_t cols,
                                                              uint8_t *__restrict__ out, uint8_t *__restrict__ scales,
                                                              uint8_t *__restrict__ out_t, uint8_t *__restrict__ scales_t,
                                                              int layout, int layout_t, int rule) {
    __shared__ __attribute__((aligned(16))) uint8_t tile[kTileC * kTileR];
    // K-step-major scale bytes leave the block as whole runs: the tile's 4 row blocks are one dword per column (256
    // contiguous bytes per tile), its 2 column blocks one 16-bit half of a dword per row.  Stored a byte at a time from
    // the lanes that hold them they were hundreds of masked one-byte writes per tile and cost a tenth of the kernel.
    __shared__ __attribute__((aligned(16))) uint8_t stage_t[kTileC * 4];
    __shared__ __attribute__((aligned(16))) uint8_t stage_r[kTileR * 2];
    saturate_fp8_conversions();
    constexpr int ESZ = SRC == ODL_BF16 ? 2 : 4;
    const int tx = threadIdx.x % 8, ty = threadIdx.x / 8;
    const int64_t tiles_r = (rows + kTileR - 1) / kTileR, tiles_c = (cols + kTileC - 1) / kTileC;
    // (K-step-major implies whole dwords: cols % 128 == 0 for `scales`, rows % 128 == 0 for `scales_t`; host-checked)
    const bool staged_r = WANT_ROW && WANT_COL && layout == ODL_MX_SCALES_KSTEP;
    const bool staged_t = WANT_COL && layout_t == ODL_MX_SCALES_KSTEP;
    int64_t tr, tc;
    ct_tile_of(blockIdx.x, tiles_r, tiles_c, tr, tc);
    const int kA = SRC == ODL_BF16 ? tx * 8 : tx * 4, kB = SRC == ODL_BF16 ? tx * 8 + 4 : 32 + tx * 4;   // tile columns of the two groups
    const int64_t r0 = tr * kTileR + ty * 4, cA = tc * kTileC + kA, cB = tc * kTileC + kB;
    // cols % 32 == 0 where codes along the rows are wanted, % 8 otherwise (host-checked): a group of 4 is in or out as a whole
    const bool okA = cA < cols, okB = cB < cols;
    [[maybe_unused]] auto col_of = [&](int j) { return j < 4 ? cA + j : cB + j - 4; };      // matrix column of the lane's column j

    // The patch stays in registers as loaded (bf16: 4 dwords a row) and is widened row by row where it is used; magnitudes
    // of bf16 pairs are compared as packed 16-bit integers, two columns at a time.
    constexpr int DW = SRC == ODL_BF16 ? 4 : 8;
    uint32_t raw[4][DW];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const bool row_ok = (r0 + i) < rows;
        const char *row = reinterpret_cast<const char *>(x) + (r0 + i) * cols * ESZ;
#pragma unroll
        for (int h = 0; h < DW / 4; ++h) {
            const bool ok = row_ok && (h == 0 ? okA : okB);
            const u32x4 v = ok ? __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(row + (h == 0 ? cA : cB) * ESZ)) : u32x4{0, 0, 0, 0};
            raw[i][4 * h] = v.x; raw[i][4 * h + 1] = v.y; raw[i][4 * h + 2] = v.z; raw[i][4 * h + 3] = v.w;
        }
    }
    auto widen = [&](int i, float (&f)[8]) {
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            if constexpr (SRC == ODL_BF16) f[q] = (q & 1) ? bf16_hi(raw[i][q / 2]) : bf16_lo(raw[i][q / 2]);
            else f[q] = bits_to_float(raw[i][q]);
        }
    };

    if constexpr (WANT_ROW) {
        const int64_t nb = cols / kMxBlock;
        uint32_t row_pairs[2] = {0u, 0u};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            // m / byte / mul: of the block that holds the lane's first group; m_b / byte_b / mul_b: of its second group's
            uint32_t m = 0, m_b = 0;
            if constexpr (SRC == ODL_BF16) {
                uint32_t m2 = max_u16x2(max_u16x2(abs_bf16x2(raw[i][0]), abs_bf16x2(raw[i][1])), max_u16x2(abs_bf16x2(raw[i][2]), abs_bf16x2(raw[i][3])));
                m = max_quad(fold_u16x2_to_f32bits(m2));                 // the 4 lanes tx = 4 b .. 4 b + 3 hold the block
                m_b = m;
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) { m = max(m, raw[i][j] & 0x7fffffffu); m_b = max(m_b, raw[i][4 + j] & 0x7fffffffu); }
                m = max_with_dpp<0x141>(max_quad(m));                    // all 8 lanes of the row (row_half_mirror joins the quads)
                m_b = max_with_dpp<0x141>(max_quad(m_b));
            }
            uint32_t byte, byte_b;
            float mul, mul_b;
            mx_scale_of<FMT>(m, rule, byte, mul);
            if constexpr (SRC == ODL_BF16) { byte_b = byte; mul_b = mul; }
            else mx_scale_of<FMT>(m_b, rule, byte_b, mul_b);
            if ((r0 + i) < rows) {
                uint32_t lo, hi;
                if (__builtin_expect(max(m, m_b) >= 0x7f800000u, 0)) {  // only a block whose amax is Inf / NaN can hold a NaN
                    float f[8];
                    widen(i, f);
                    lo = quantise4<FMT>(f[0], f[1], f[2], f[3], mul, mul, mul, mul);
                    hi = quantise4<FMT>(f[4], f[5], f[6], f[7], mul_b, mul_b, mul_b, mul_b);
                } else {                                                // the hardware divides by 2^(byte - 127) and saturates
                    const float e8 = bits_to_float(byte << 23), e8_b = bits_to_float(byte_b << 23);
                    if constexpr (SRC == ODL_BF16) {
                        lo = cvt_scaled4<SRC, FMT>(raw[i][0], raw[i][1], 0u, 0u, e8);
                        hi = cvt_scaled4<SRC, FMT>(raw[i][2], raw[i][3], 0u, 0u, e8);
                    } else {
                        lo = cvt_scaled4<SRC, FMT>(raw[i][0], raw[i][1], raw[i][2], raw[i][3], e8);
                        hi = cvt_scaled4<SRC, FMT>(raw[i][4], raw[i][5], raw[i][6], raw[i][7], e8_b);
                    }
                }
                if constexpr (SRC == ODL_BF16) {
                    if (okA) *reinterpret_cast<u32x2 *>(out + (r0 + i) * cols + cA) = u32x2{lo, hi};
                } else {
                    if (okA) *reinterpret_cast<uint32_t *>(out + (r0 + i) * cols + cA) = lo;
                    if (okB) *reinterpret_cast<uint32_t *>(out + (r0 + i) * cols + cB) = hi;
                }
                if (staged_r) {
                    // both bytes of the row in one lane (bf16: row_shl:4 hands lane l the value of lane l + 4, which holds
                    // the row's second block); the lane's four rows then go to LDS as one 8-byte write
                    uint32_t second = byte_b;
                    if constexpr (SRC == ODL_BF16) second = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)byte, 0x104, 0xf, 0xf, false);
                    row_pairs[i / 2] |= (byte | (second << 8)) << (16 * (i & 1));
                } else if constexpr (SRC == ODL_BF16) {
                    if ((tx & 3) == 0 && okA) scales[mx_scale_at(layout, r0 + i, cA / kMxBlock, rows, nb)] = (uint8_t)byte;
                } else if (tx == 0) {
                    if (okA) scales[mx_scale_at(layout, r0 + i, cA / kMxBlock, rows, nb)] = (uint8_t)byte;
                    if (okB) scales[mx_scale_at(layout, r0 + i, cB / kMxBlock, rows, nb)] = (uint8_t)byte_b;
                }
            }
        }
        if (staged_r && tx == 0) *reinterpret_cast<u32x2 *>(&stage_r[ty * 8]) = u32x2{row_pairs[0], row_pairs[1]};
    }

    if constexpr (WANT_COL) {
        const int64_t nbt = rows / kMxBlock;
        float mul_c[8], e8_c[8];
        uint32_t col_bytes[2] = {0u, 0u};                                // the scale bytes of the lane's 8 columns, packed
        uint32_t cmax[8];                                                // fp32 magnitude bits per column, over the 32 rows
        if constexpr (SRC == ODL_BF16) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                uint32_t m2 = max_u16x2(max_u16x2(abs_bf16x2(raw[0][q]), abs_bf16x2(raw[1][q])), max_u16x2(abs_bf16x2(raw[2][q]), abs_bf16x2(raw[3][q])));
                m2 = max_stride8_u16x2(m2);                              // the 8 lanes of the wave with this tx: 32 rows
                cmax[2 * q] = m2 << 16;
                cmax[2 * q + 1] = m2 & 0xffff0000u;
            }
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j)
                cmax[j] = max_stride8(max(max(raw[0][j] & 0x7fffffffu, raw[1][j] & 0x7fffffffu), max(raw[2][j] & 0x7fffffffu, raw[3][j] & 0x7fffffffu)));
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            uint32_t byte;
            mx_scale_of<FMT>(cmax[j], rule, byte, mul_c[j]);
            e8_c[j] = bits_to_float(byte << 23);
            // rows % 32 == 0 (host-checked): a row block is inside the matrix as a whole or not at all
            col_bytes[j / 4] |= byte << (8 * (j % 4));
            if (!staged_t && (ty & 7) == 0 && (j < 4 ? okA : okB) && r0 < rows)
                scales_t[mx_scale_at(layout_t, col_of(j), r0 / kMxBlock, cols, nbt)] = (uint8_t)byte;
        }
        // staged: the wave's row block is one plane of 64 bytes, a lane's two groups of 4 columns a 4-byte write each
        if (staged_t && (ty & 7) == 0) {
            *reinterpret_cast<uint32_t *>(&stage_t[(ty / 8) * kTileC + kA]) = col_bytes[0];
            *reinterpret_cast<uint32_t *>(&stage_t[(ty / 8) * kTileC + kB]) = col_bytes[1];
        }
        uint32_t worst = 0;                                              // Inf / NaN in any of the lane's 8 column blocks?
#pragma unroll
        for (int j = 0; j < 8; ++j) worst = max(worst, cmax[j]);
        uint32_t tl[4], th[4];                                           // tl[k] / th[k]: rows 4 ty .. + 3 of column k / 4 + k
        if (__builtin_expect(worst >= 0x7f800000u, 0)) {
            uint32_t lo[4], hi[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float f[8];
                widen(i, f);
                lo[i] = quantise4<FMT>(f[0], f[1], f[2], f[3], mul_c[0], mul_c[1], mul_c[2], mul_c[3]);
                hi[i] = quantise4<FMT>(f[4], f[5], f[6], f[7], mul_c[4], mul_c[5], mul_c[6], mul_c[7]);
            }
            transpose4x4(lo, tl);
            transpose4x4(hi, th);
        } else {
            // the four rows of one column side by side are the operands of one pair of conversions: the codes come out
            // transposed (bf16: the two halves of the rows' dwords are regrouped per column first)
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                uint32_t t;
                if constexpr (SRC == ODL_BF16) {
                    const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
                    const uint32_t r01 = __builtin_amdgcn_perm(raw[1][j / 2], raw[0][j / 2], sel);
                    const uint32_t r23 = __builtin_amdgcn_perm(raw[3][j / 2], raw[2][j / 2], sel);
                    t = cvt_scaled4<SRC, FMT>(r01, r23, 0u, 0u, e8_c[j]);
                } else {
                    t = cvt_scaled4<SRC, FMT>(raw[0][j], raw[1][j], raw[2][j], raw[3][j], e8_c[j]);
                }
                if (j < 4) tl[j] = t; else th[j - 4] = t;
            }
        }
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            *reinterpret_cast<uint32_t *>(&tile[ct_lds_write_off(kA + k, ty)]) = tl[k];
            *reinterpret_cast<uint32_t *>(&tile[ct_lds_write_off(kB + k, ty)]) = th[k];
        }
        __syncthreads();
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            const int chunk = threadIdx.x + it * kMxThreads;
            const int k = chunk / 8, m16 = chunk % 8;
            const int64_t oc = tc * kTileC + k, orow = tr * kTileR + m16 * 16;
            if (oc < cols && orow < rows)
                __builtin_nontemporal_store(ct_lds_read(tile, k, m16), reinterpret_cast<u32x4 *>(out_t + oc * rows + orow));
        }
        // the staged scale bytes: dword [tile row][column] of scales_t from the first wave, the 16-bit half
        // [tile column / 2][row] of scales from the next two
        if (staged_t && threadIdx.x < kTileC) {
            const int64_t oc = tc * kTileC + threadIdx.x;
            const int c = threadIdx.x;
            if (oc < cols && tr * kTileR < rows)
                reinterpret_cast<uint32_t *>(scales_t)[tr * cols + oc] = (uint32_t)stage_t[c] | ((uint32_t)stage_t[kTileC + c] << 8) |
                                                                         ((uint32_t)stage_t[2 * kTileC + c] << 16) | ((uint32_t)stage_t[3 * kTileC + c] << 24);
        }
        if (staged_r && threadIdx.x >= 64 && threadIdx.x < 64 + kTileR) {
            const int r = threadIdx.x - 64;
            const int64_t orow = tr * kTileR + r;
            if (orow < rows && tc * kTileC < cols)
                reinterpret_cast<uint16_t *>(scales)[((tc >> 1) * rows + orow) * 2 + (tc & 1)] = reinterpret_cast<const uint16_t *>(stage_r)[r];
        }
    }
}

// ------------------------------------------------------------------ blockwise recipe
// Blocks of 128 along the contraction axis (activations, gradients) or of 128 x 128 (weights), each with the per-tensor
// scale rule applied to its amax and rounded down to a power of two.  The inverse of such a scale is an E8M0 byte, and a
// 128-block is four MX blocks with the same byte: the kernel writes that byte four times as the dword [K step][row] of
// the K-step-major layout, and the MXFP8 GEMMs serve this recipe unchanged.
template <int FMT>
__device__ __forceinline__ void block_scale_of(uint32_t amax_bits, int margin, uint32_t &dword, float &mul) {
    const float s = scale_rule(bits_to_float(amax_bits), Fp8Lim<FMT>::max, margin, 1.0f);
    uint32_t b = float_to_bits(s) & 0xff800000u;                     // the power of two below (s > 0 always)
    if ((b >> 23) == 0) b = 0x00800000u;
    mul = bits_to_float(b);
    dword = (254u - (b >> 23)) * 0x01010101u;
}

// Byte offset of (column, dword of 4 rows) in the transposed 128 x 128 tile: two halves of 64 columns, each laid out as the
// 64-column tile of ct_tile.h (a 256-byte line per pair of columns, rotated by 16 bytes per 8 columns), the second half
// rotated by 16 bytes more.  The dword writes of a half-wave (8 column groups of 16 x 4 row groups) then differ mod 32,
// and the 16-byte reads stay aligned with 16 consecutive lanes reading one whole line.
__device__ __forceinline__ int block_col_slot(int col) { return col + 4 * (col >> 5); }

__device__ __forceinline__ int block_lds_off(int col, int dw) {
    const int half = col >> 6, c = col & 63;
    // (the last term separates the lanes tx and tx + 1 of an fp32 source, whose columns 4 tx + k share c >> 3; for a bf16
    // source it is the same for all lanes of an instruction)
    return half * 8192 + (c >> 1) * 256 + ((((c & 1) * 32) + dw + 4 * (c >> 3) + 4 * half + 16 * ((c >> 2) & 1)) & 63) * 4;
}

// 128 x 128 tile per block of 256 lanes; lane (tx = lane % 8, ty = lane / 8) owns rows 4 ty .. 4 ty + 3 and four groups
// of 4 columns: bf16 source, columns 8 tx .. 8 tx + 7 and 64 + 8 tx .. 64 + 8 tx + 7; fp32 source, columns 4 tx + 32 g ..
// + 3 for g = 0 .. 3.  That way the 8 lanes of a tile row read 128 contiguous bytes with each load instruction:
// non-temporal loads are not merged across instructions, and a lane that reads its 32 (64) bytes of a row as
// neighbouring 16-byte pieces leaves every instruction a half (quarter) of each 64-byte request (a read-only loop over
// 8192 x 14336 bf16 measured 5.1 TB/s that way against 6.2 TB/s with contiguous instructions).  TWO_D: one scale for the whole tile (weights); else one per row of the tile for the row-major
// codes and one per column for the transposed codes.  rows, cols multiples of 128.
template <int SRC, int FMT, bool TWO_D, bool WANT_ROW, bool WANT_COL>
__global__ __launch_bounds__(256, SRC == ODL_BF16 ? 8 : 4) void block_cast_kernel(const void *__restrict__ x, int64_t rows, int64_t cols, int margin,
                                                         uint8_t *__restrict__ out, uint32_t *__restrict__ scales,
                                                         uint8_t *__restrict__ out_t, uint32_t *__restrict__ scales_t) {
    __shared__ __attribute__((aligned(16))) uint8_t tile[WANT_COL ? 128 * 128 : 16];
    // red and col_e8 hold one value per column at block_col_slot(column): every 32 columns sit four dwords further on.
    // The 8-byte write of the column maxima is served 16 lanes at a time over 32 banks (measured: with the 8 lanes tx
    // on dwords 8 tx + j, lanes tx and tx + 4 met, 4 conflict cycles per wave); with the pitch the 16 lanes (8 tx, two
    // neighbouring column pairs each) cover 32 consecutive dwords.  The 16-byte reads of col_e8 stay on 32 different banks.
    __shared__ __attribute__((aligned(16))) uint32_t red[4][144];       // per wave: column maxima (1-D), or slot 0: the wave's maximum (2-D)
    __shared__ __attribute__((aligned(16))) float col_e8[144];          // per column: its E8M0 byte where a float keeps its exponent
    __shared__ int odd_tile;                                       // 1-D blocks: some column of the tile holds Inf / NaN
    __shared__ uint32_t row_dw[128];                               // 1-D blocks, both outputs: the scale dwords of the tile's rows
    saturate_fp8_conversions();
    constexpr int ESZ = SRC == ODL_BF16 ? 2 : 4, DW = 16 * ESZ / 4;
    const int tx = threadIdx.x % 8, ty = threadIdx.x / 8, wave = threadIdx.x / 64;
    const int64_t tiles_r = rows / 128, tiles_c = cols / 128;
    int64_t tr, tc;
    ct_tile_of(blockIdx.x, tiles_r, tiles_c, tr, tc);
    const int64_t r0 = tr * 128 + ty * 4;
    // first tile column of the lane's group g of 4 columns; raw[i] holds the groups in this order
    auto group_col = [&](int g) { return SRC == ODL_BF16 ? 8 * tx + 4 * (g & 1) + 64 * (g >> 1) : 4 * tx + 32 * g; };

    uint32_t raw[4][DW];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const char *row = reinterpret_cast<const char *>(x) + ((r0 + i) * cols + tc * 128) * ESZ;
#pragma unroll
        for (int h = 0; h < DW / 4; ++h) {
            const int byte = 16 * tx + 128 * h;
            const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(row + byte));
            raw[i][4 * h] = v.x; raw[i][4 * h + 1] = v.y; raw[i][4 * h + 2] = v.z; raw[i][4 * h + 3] = v.w;
        }
    }
    auto widen4 = [&](int i, int g, float (&f)[4]) {            // the lane's column group g of row i
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            if constexpr (SRC == ODL_BF16) f[q] = (q & 1) ? bf16_hi(raw[i][2 * g + q / 2]) : bf16_lo(raw[i][2 * g + q / 2]);
            else f[q] = bits_to_float(raw[i][4 * g + q]);
        }
    };
    // magnitude bits (fp32 layout) of row i over the lane's 16 columns
    auto row_mag = [&](int i) -> uint32_t {
        if constexpr (SRC == ODL_BF16) {
            uint32_t m2 = 0;
#pragma unroll
            for (int d = 0; d < DW; ++d) m2 = max_u16x2(m2, abs_bf16x2(raw[i][d]));
            return fold_u16x2_to_f32bits(m2);
        } else {
            uint32_t m = 0;
#pragma unroll
            for (int d = 0; d < DW; ++d) m = max(m, raw[i][d] & 0x7fffffffu);
            return m;
        }
    };

    // A block whose amax is Inf / NaN (the only kind that can hold a NaN) goes through quantise4, which gives NaN its code;
    // every other block through the hardware's scaled conversions, which divide by 2^(byte - 127) and saturate.
    auto e8_of = [](uint32_t dword) { return bits_to_float((dword & 0xffu) << 23); };
    auto mul_of = [](float e8) { return bits_to_float((254u - (float_to_bits(e8) >> 23)) << 23); };     // byte <= 253
    float e8_all = 1.0f;
    uint32_t m_all = 0;
    if constexpr (TWO_D) {
        uint32_t m = max(max(row_mag(0), row_mag(1)), max(row_mag(2), row_mag(3)));
        m = wave_max_u32(m);
        if (threadIdx.x % 64 == 0) red[wave][0] = m;
        __syncthreads();
        m_all = max(max(red[0][0], red[1][0]), max(red[2][0], red[3][0]));
        uint32_t dword;
        float mul;
        block_scale_of<FMT>(m_all, margin, dword, mul);
        e8_all = e8_of(dword);
        if (threadIdx.x < 128) {
            if (WANT_ROW) scales[tc * rows + tr * 128 + threadIdx.x] = dword;
            if (WANT_COL) scales_t[tr * cols + tc * 128 + threadIdx.x] = dword;
        }
    }

    if constexpr (WANT_ROW) {
        [[maybe_unused]] uint32_t keep_row = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float e8 = e8_all;
            uint32_t m = m_all;
            if constexpr (!TWO_D) {
                m = max_quad(row_mag(i));
                m = max_with_dpp<0x141>(m);                              // row_half_mirror: lane l <-> 7 - l of its 8: the other quad
                uint32_t dword;
                float mul;
                block_scale_of<FMT>(m, margin, dword, mul);
                e8 = e8_of(dword);
                // with the transposed output to follow, the tile's 128 row dwords leave as one 512-byte run after the next
                // barrier: lane tx = i of the 8 that hold the row keeps it, and the lanes tx < 4 store one dword each
                if constexpr (WANT_COL) { if (tx == i) keep_row = dword; }
                else if (tx == 0) scales[tc * rows + r0 + i] = dword;
            }
            uint32_t q[4];
            if (__builtin_expect(m >= 0x7f800000u, 0)) {
                const float mul = mul_of(e8);
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    float f[4];
                    widen4(i, g, f);
                    q[g] = quantise4<FMT>(f[0], f[1], f[2], f[3], mul, mul, mul, mul);
                }
            } else {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    if constexpr (SRC == ODL_BF16) q[g] = cvt_scaled4<SRC, FMT>(raw[i][2 * g], raw[i][2 * g + 1], 0u, 0u, e8);
                    else q[g] = cvt_scaled4<SRC, FMT>(raw[i][4 * g], raw[i][4 * g + 1], raw[i][4 * g + 2], raw[i][4 * g + 3], e8);
                }
            }
            uint8_t *o = out + (r0 + i) * cols + tc * 128;
            if constexpr (SRC == ODL_BF16) {
                *reinterpret_cast<u32x2 *>(o + group_col(0)) = u32x2{q[0], q[1]};
                *reinterpret_cast<u32x2 *>(o + group_col(2)) = u32x2{q[2], q[3]};
            } else {
#pragma unroll
                for (int g = 0; g < 4; ++g) *reinterpret_cast<uint32_t *>(o + group_col(g)) = q[g];
            }
        }
        if constexpr (!TWO_D && WANT_COL) { if (tx < 4) row_dw[ty * 4 + tx] = keep_row; }
    }

    if constexpr (WANT_COL) {
        bool plain = m_all < 0x7f800000u;                                // no Inf / NaN anywhere in the tile
        if constexpr (!TWO_D) {
            // column maxima: over the lane's 4 rows, over the 8 lanes of the wave with this tx (32 rows), over the 4 waves.
            // After the exchange all 8 lanes with this tx hold the maxima of the lane's 8 column pairs; lane p = ty & 7 of
            // them keeps pair p, so the wave stores its 128 maxima with ONE 8-byte write per lane that covers the row of
            // `red` exactly (eight writes of 8 lanes each were counted as one conflict cycle apiece)
            const int p = ty & 7;
            uint32_t keep_lo = 0, keep_hi = 0;
#pragma unroll
            for (int d = 0; d < DW; ++d) {
                uint32_t m;
                if constexpr (SRC == ODL_BF16) {
                    m = max_u16x2(max_u16x2(abs_bf16x2(raw[0][d]), abs_bf16x2(raw[1][d])), max_u16x2(abs_bf16x2(raw[2][d]), abs_bf16x2(raw[3][d])));
                    m = max_stride8_u16x2(m);
                    if (p == d) { keep_lo = m << 16; keep_hi = m & 0xffff0000u; }
                } else {
                    m = max(max(raw[0][d] & 0x7fffffffu, raw[1][d] & 0x7fffffffu), max(raw[2][d] & 0x7fffffffu, raw[3][d] & 0x7fffffffu));
                    m = max_stride8(m);
                    if (p == d / 2) { if (d & 1) keep_hi = m; else keep_lo = m; }
                }
            }
            *reinterpret_cast<u32x2 *>(&red[wave][block_col_slot(group_col(p / 2) + 2 * (p & 1))]) = u32x2{keep_lo, keep_hi};
            if (threadIdx.x == 0) odd_tile = 0;
            __syncthreads();
            if (threadIdx.x < 128) {
                const int slot = block_col_slot(threadIdx.x);
                const uint32_t m = max(max(red[0][slot], red[1][slot]), max(red[2][slot], red[3][slot]));
                uint32_t dword;
                float mul;
                block_scale_of<FMT>(m, margin, dword, mul);
                col_e8[slot] = e8_of(dword);
                scales_t[tr * cols + tc * 128 + threadIdx.x] = dword;
                if constexpr (WANT_ROW) scales[tc * rows + tr * 128 + threadIdx.x] = row_dw[threadIdx.x];
                if (m >= 0x7f800000u) odd_tile = 1;                      // (every writer writes the same value)
            }
            __syncthreads();
            plain = odd_tile == 0;
        }
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            float ec[4] = {e8_all, e8_all, e8_all, e8_all};
            if constexpr (!TWO_D) {
                const float4 v = *reinterpret_cast<const float4 *>(&col_e8[block_col_slot(group_col(g))]);
                ec[0] = v.x; ec[1] = v.y; ec[2] = v.z; ec[3] = v.w;
            }
            uint32_t t[4];
            if (__builtin_expect(!plain, 0)) {
                uint32_t q[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float f[4];
                    widen4(i, g, f);
                    q[i] = quantise4<FMT>(f[0], f[1], f[2], f[3], mul_of(ec[0]), mul_of(ec[1]), mul_of(ec[2]), mul_of(ec[3]));
                }
                transpose4x4(q, t);                                      // t[k] = rows 4 ty .. + 3 of column 16 tx + 4 g + k
            } else {
                // the four rows of a column side by side feed one pair of conversions: the codes come out transposed
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const int c = 4 * g + k;
                    if constexpr (SRC == ODL_BF16) {
                        const uint32_t sel = (c & 1) ? 0x07060302u : 0x05040100u;
                        const uint32_t r01 = __builtin_amdgcn_perm(raw[1][c / 2], raw[0][c / 2], sel);
                        const uint32_t r23 = __builtin_amdgcn_perm(raw[3][c / 2], raw[2][c / 2], sel);
                        t[k] = cvt_scaled4<SRC, FMT>(r01, r23, 0u, 0u, ec[k]);
                    } else {
                        t[k] = cvt_scaled4<SRC, FMT>(raw[0][c], raw[1][c], raw[2][c], raw[3][c], ec[k]);
                    }
                }
            }
#pragma unroll
            for (int k = 0; k < 4; ++k) *reinterpret_cast<uint32_t *>(&tile[block_lds_off(group_col(g) + k, ty)]) = t[k];
        }
        __syncthreads();
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            const int chunk = threadIdx.x + it * 256;
            const int col = chunk / 8, m16 = chunk % 8;
            const u32x4 v = *reinterpret_cast<const u32x4 *>(&tile[block_lds_off(col, 4 * m16)]);
            __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(out_t + (tc * 128 + col) * rows + tr * 128 + m16 * 16));
        }
    }
}

// ------------------------------------------------------------------ GEMM, tiled
// The structure of gemm_nt_tiled_kernel (two LDS stages of BM + BN rows x 128 bytes, direct-to-LDS loads, swizzled
// 16-byte chunks, MFMA operands swapped so that a lane ends up with 4 consecutive output columns) plus the scale
// bytes: per K step of 128 bytes a row has 4 of them (one dword); every thread of the block fetches the dword of one
// row of A or B for the NEXT step with that step's operand loads, like them straight into LDS;
// a lane reads the dword of each of its rows and shifts it right by 8 bits when it sits in the upper half of the
// wave, so that byte 0 / byte 2 are the scales it supplies in the first / second MFMA of the step (lanes 0..31: blocks 0
// and 2 of the step, lanes 32..63: blocks 1 and 3).
template <int BM, int BN, int WAVES_M, int WAVES_N, int FA, int FB, bool KS, int STAGES = 2>
__global__ __launch_bounds__(WAVES_M *WAVES_N * 64) void mx_gemm_tiled_kernel(const GemmArgs g, const uint8_t *__restrict__ sa,
                                                                              const uint8_t *__restrict__ sb) {
    static_assert(STAGES == 2 || STAGES == 4, "two LDS stages, or four for launches of at most one block per compute unit");
    constexpr int NW = WAVES_M * WAVES_N, NT = NW * 64;
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N, TM = WM / 32, TN = WN / 32;
    constexpr int A_BYTES = BM * 128, B_BYTES = BN * 128, STAGE = A_BYTES + B_BYTES;
    constexpr int LA = BM / 8 / NW, LB = BN / 8 / NW;
    constexpr int GM = 8;
    static_assert(BM + BN <= NT && (BM + BN) % 64 == 0, "one scale dword per thread of the first (BM + BN) / 64 waves: BM threads serve A, the next BN serve B");
    constexpr int SCALE_WAVES = (BM + BN) / 64;

    __shared__ __attribute__((aligned(1024))) uint8_t lds0[STAGE];
    __shared__ __attribute__((aligned(1024))) uint8_t lds1[STAGE];
    __shared__ __attribute__((aligned(1024))) uint8_t lds2[STAGES == 4 ? STAGE : 1024];
    __shared__ __attribute__((aligned(1024))) uint8_t lds3[STAGES == 4 ? STAGE : 1024];
    __shared__ __attribute__((aligned(256))) uint32_t sc0[BM + BN];
    __shared__ __attribute__((aligned(256))) uint32_t sc1[BM + BN];
    __shared__ __attribute__((aligned(256))) uint32_t sc2[STAGES == 4 ? BM + BN : 64];
    __shared__ __attribute__((aligned(256))) uint32_t sc3[STAGES == 4 ? BM + BN : 64];

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
    const int64_t nb = g.K / kMxBlock;

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
    // the scale dword this thread fetches per step: thread i < BM that of A row i, the others that of B row i - BM (rows
    // past the edge re-read the last row); K-step-major: the dword of step kt is [kt][row], row-major: dword kt of the
    // row's nb bytes.  It travels like the operands, straight into the stage's scale slots (64 lanes x 4 bytes land at
    // the wave's 256 bytes), and is complete when the operand loads of the stage are.
    const bool mine_a = (int)threadIdx.x < BM;
    const int64_t my_row = mine_a ? min(m0 + (int64_t)threadIdx.x, g.M - 1) : min(n0 + min((int64_t)threadIdx.x - BM, (int64_t)BN - 1), g.N - 1);
    const uint32_t *my_scales = reinterpret_cast<const uint32_t *>(mine_a ? sa : sb) + (KS ? my_row : my_row * (nb / 4));
    const int64_t my_step = KS ? (mine_a ? g.M : g.N) : 1;
    auto issue = [&](uint8_t *lds, uint32_t *sc, int kt) {
        const uint8_t *ga = g.a + (int64_t)kt * 128, *gb = g.b + (int64_t)kt * 128;
#pragma unroll
        for (int j = 0; j < LA; ++j)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(ga + off_a[j]),
                                             (__attribute__((address_space(3))) void *)(lds + (wave + j * NW) * 1024), 16, 0, 0);
#pragma unroll
        for (int j = 0; j < LB; ++j)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(gb + off_b[j]),
                                             (__attribute__((address_space(3))) void *)(lds + A_BYTES + (wave + j * NW) * 1024), 16, 0, 0);
        if (wave < SCALE_WAVES)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(my_scales + kt * my_step),
                                             (__attribute__((address_space(3))) void *)(sc + wave * 64), 4, 0, 0);
    };

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

    auto compute = [&](const uint8_t *lds, const uint32_t *sc) {
        int esa[TM], esb[TN];                       // this lane's scale bytes: byte 0 for the first K half, byte 2 for the second
#pragma unroll
        for (int t = 0; t < TM; ++t) esa[t] = (int)(sc[wm0 + 32 * t + lr] >> (8 * lg));
#pragma unroll
        for (int u = 0; u < TN; ++u) esb[u] = (int)(sc[BM + wn0 + 32 * u + lr] >> (8 * lg));
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int c = 4 * h + lg;               // 16-byte chunks c (first block) and c + 2 (second block) of the row
            v8i af[TM], bf[TN];
#pragma unroll
            for (int t = 0; t < TM; ++t) {
                const uint8_t *p = lds + a_off[t];
                const v4i lo = *reinterpret_cast<const v4i *>(p + ((c ^ a_sw[t]) << 4));
                const v4i hi = *reinterpret_cast<const v4i *>(p + (((c + 2) ^ a_sw[t]) << 4));
                af[t] = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
            }
#pragma unroll
            for (int u = 0; u < TN; ++u) {
                const uint8_t *p = lds + b_off[u];
                const v4i lo = *reinterpret_cast<const v4i *>(p + ((c ^ b_sw[u]) << 4));
                const v4i hi = *reinterpret_cast<const v4i *>(p + (((c + 2) ^ b_sw[u]) << 4));
                bf[u] = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
            }
#pragma unroll
            for (int t = 0; t < TM; ++t)
#pragma unroll
                for (int u = 0; u < TN; ++u) {
                    if (h == 0) acc[t][u] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bf[u], af[t], acc[t][u], FB, FA, 0, esb[u], 0, esa[t]);
                    else acc[t][u] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bf[u], af[t], acc[t][u], FB, FA, 2, esb[u], 2, esa[t]);
                }
        }
    };

    if constexpr (STAGES == 4) {
        // The four-stage form of gemm_nt_tiled_kernel (a block alone on its compute unit keeps three K steps of loads in
        // flight); loads, waits and barriers written as instructions for the reasons given there.  The waves that also
        // fetch scale dwords have one more load per stage to count.
        constexpr int PER = LA + LB;
        static_assert(2 * (PER + 1) <= 63, "the counter holds 63 loads");
        auto lds_addr_of = [](const void *p) { return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) uint8_t *)p; };
        auto dma16 = [](const uint8_t *src, uint32_t lds_addr) {
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_addr), "v"(src));
        };
        auto dma4 = [](const uint32_t *src, uint32_t lds_addr) {
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" ::"s"(lds_addr), "v"(src));
        };
        auto fetch = [&](uint8_t *lds, uint32_t *sc, int kt) {
            const uint8_t *ga = g.a + (int64_t)kt * 128, *gb = g.b + (int64_t)kt * 128;
            const uint32_t base = lds_addr_of(lds);
#pragma unroll
            for (int j = 0; j < LA; ++j) dma16(ga + off_a[j], base + (wave + j * NW) * 1024);
#pragma unroll
            for (int j = 0; j < LB; ++j) dma16(gb + off_b[j], base + A_BYTES + (wave + j * NW) * 1024);
            if (wave < SCALE_WAVES) dma4(my_scales + kt * my_step, lds_addr_of(sc) + wave * 256);
        };
        auto phase = [&](const uint8_t *cur, const uint32_t *cur_sc, uint8_t *refill, uint32_t *refill_sc, int kt) {
            if (wave < SCALE_WAVES) {
                if (kt + 2 < KT) asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(2 * (PER + 1)) : "memory");
                else if (kt + 1 < KT) asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(PER + 1) : "memory");
                else asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
            } else {
                if (kt + 2 < KT) asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(2 * PER) : "memory");
                else if (kt + 1 < KT) asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(PER) : "memory");
                else asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
            }
            if (kt + 3 < KT) fetch(refill, refill_sc, kt + 3);
            compute(cur, cur_sc);
        };
        fetch(lds0, sc0, 0);
        if (KT > 1) fetch(lds1, sc1, 1);
        if (KT > 2) fetch(lds2, sc2, 2);
        for (int kt = 0; kt < KT; kt += 4) {
            phase(lds0, sc0, lds3, sc3, kt);
            if (kt + 1 < KT) phase(lds1, sc1, lds0, sc0, kt + 1);
            if (kt + 2 < KT) phase(lds2, sc2, lds1, sc1, kt + 2);
            if (kt + 3 < KT) phase(lds3, sc3, lds2, sc2, kt + 3);
        }
    } else {
    issue(lds0, sc0, 0);
    for (int kt = 0; kt < KT; kt += 2) {
        __builtin_amdgcn_s_waitcnt(0x0F70);                     // vmcnt(0): my loads into lds0 and sc0 have landed
        __syncthreads();
        if (kt + 1 < KT) issue(lds1, sc1, kt + 1);
        compute(lds0, sc0);
        if (kt + 1 < KT) {
            __builtin_amdgcn_s_waitcnt(0x0F70);
            __syncthreads();
            if (kt + 2 < KT) issue(lds0, sc0, kt + 2);
            compute(lds1, sc1);
        }
    }
    }

    const bool interior = m0 + BM <= g.M && n0 + BN <= g.N;
    constexpr int EPI_BYTES = 32 * (TN * 32 * 4 + 16);
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

// ------------------------------------------------------------------ GEMM, any shape with K % 32 == 0
// One wave per 32 x 32 output tile, operands and scale bytes straight from global memory, 64 K-bytes per trip; a last
// half trip (K % 64 == 32) feeds zeros as the second block.
template <int FA, int FB>
__global__ __launch_bounds__(64) void mx_gemm_generic_kernel(const GemmArgs g, const uint8_t *__restrict__ sa, const uint8_t *__restrict__ sb,
                                                             int kstep_major) {
    const int lane = threadIdx.x, lr = lane % 32, lg = lane / 32;
    const int64_t m0 = (int64_t)blockIdx.y * 32, n0 = (int64_t)blockIdx.x * 32;
    const int64_t ra = min(m0 + lr, g.M - 1), rb = min(n0 + lr, g.N - 1), nb = g.K / kMxBlock;
    v16f acc;
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = 0.0f;
    for (int64_t k = 0; k < g.K; k += 64) {
        const bool second = k + 32 < g.K;                           // false in the half trip at the end
        const v4i zero = {0, 0, 0, 0};
        const v4i *pa = reinterpret_cast<const v4i *>(g.a + ra * g.K + k + 16 * lg), *pb = reinterpret_cast<const v4i *>(g.b + rb * g.K + k + 16 * lg);
        const v4i a0 = pa[0], b0 = pb[0], a1 = second ? pa[2] : zero, b1 = second ? pb[2] : zero;
        const v8i af = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w}, bf = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
        int ea = 127, eb = 127;                                     // lanes 0..31: scale of block k / 32, lanes 32..63: of the next
        if (lg == 0 || second) {
            ea = sa[mx_scale_at(kstep_major, ra, k / kMxBlock + lg, g.M, nb)];
            eb = sb[mx_scale_at(kstep_major, rb, k / kMxBlock + lg, g.N, nb)];
        }
        acc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bf, af, acc, FB, FA, 0, eb, 0, ea);
    }
    if (g.out_dtype == ODL_BF16) store_tile<true, false>(g, acc, m0 + lr, n0 + 4 * lg);
    else store_tile<false, false>(g, acc, m0 + lr, n0 + 4 * lg);
}

}  // namespace odl

// The epilogues multiply by *g.sa * *g.sb: a 1.0f that is part of the library's device image (one copy per GPU; the name is
// only a handle for hipGetSymbolAddress, the address the kernels take is looked up once per device).
static __device__ float mx_unit_scale = 1.0f;

namespace odl {

const float *unit_scale_for_current_device(const char *who) {
    constexpr int kMaxDevices = 64;
    static const float *cached[kMaxDevices] = {};
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) { set_error(ODL_ERR_LAUNCH, "%s: hipGetDevice: %s", who, hipGetErrorString(e)); return nullptr; }
    const float *ptr = __atomic_load_n(&cached[dev], __ATOMIC_ACQUIRE);
    if (!ptr) {
        void *addr = nullptr;
        e = hipGetSymbolAddress(&addr, HIP_SYMBOL(mx_unit_scale));
        if (e != hipSuccess || !addr) { set_error(ODL_ERR_LAUNCH, "%s: hipGetSymbolAddress on device %d: %s", who, dev, hipGetErrorString(e)); return nullptr; }
        ptr = static_cast<const float *>(addr);
        __atomic_store_n(&cached[dev], ptr, __ATOMIC_RELEASE);
    }
    return ptr;
}

template <int SRC, int FMT>
static void launch_mx_cast(const void *x, int64_t rows, int64_t cols, uint8_t *out, uint8_t *scales, uint8_t *out_t, uint8_t *scales_t,
                           int layout, int layout_t, int rule, hipStream_t stream) {
    const int64_t g = ((rows + kTileR - 1) / kTileR) * ((cols + kTileC - 1) / kTileC);
#define ODL_MX(R, C) hipLaunchKernelGGL((mx_cast_kernel<SRC, FMT, R, C>), dim3((unsigned)g), dim3(kMxThreads), 0, stream, x, rows, cols, out, scales, out_t, scales_t, layout, layout_t, rule)
    if (out && out_t) ODL_MX(true, true);
    else if (out) ODL_MX(true, false);
    else ODL_MX(false, true);
#undef ODL_MX
}

template <int FA, int FB, bool KS>
static void launch_mx_tiled(const GemmArgs &g, const uint8_t *sa, const uint8_t *sb, int cus, hipStream_t stream) {
    GemmArgs t = g;
    // 256 x 256 tiles (8 waves of 128 x 64) when they fill the chip, else 128 x 128 (two blocks per compute unit)
    const int64_t big = ((g.M + 255) / 256) * ((g.N + 255) / 256);
    if (big >= cus) {
        t.tiles_m = (int)((g.M + 255) / 256); t.tiles_n = (int)((g.N + 255) / 256);
        const unsigned grid = (unsigned)(((t.tiles_m * t.tiles_n + 7) / 8) * 8);
        hipLaunchKernelGGL((mx_gemm_tiled_kernel<256, 256, 2, 4, FA, FB, KS>), dim3(grid), dim3(512), 0, stream, t, sa, sb);
    } else {
        t.tiles_m = (int)((g.M + 127) / 128); t.tiles_n = (int)((g.N + 127) / 128);
        const unsigned grid = (unsigned)(((t.tiles_m * t.tiles_n + 7) / 8) * 8);
        // at most one block per compute unit: eight waves and four stages (see gemm_nt_tiled_kernel)
        if (t.tiles_m * t.tiles_n <= cus)
            hipLaunchKernelGGL((mx_gemm_tiled_kernel<128, 128, 2, 4, FA, FB, KS, 4>), dim3(grid), dim3(512), 0, stream, t, sa, sb);
        else
            hipLaunchKernelGGL((mx_gemm_tiled_kernel<128, 128, 2, 2, FA, FB, KS>), dim3(grid), dim3(256), 0, stream, t, sa, sb);
    }
}

// kernel: 0 = one wave per 32 x 32 tile, 1 = LDS-tiled, 2 = the streaming kernel of gemm_stream.hip with block scales
template <int FA, int FB>
static void launch_mx_gemm(const GemmArgs &g, const uint8_t *sa, const uint8_t *sb, int kernel, int kstep_major, int cus, hipStream_t stream) {
    if (kernel == 2) {
        GemmArgs t = g;
        t.mx_sa = sa; t.mx_sb = sb;
        t.tiles_m = (int)((g.M + 255) / 256); t.tiles_n = (int)((g.N + 255) / 256);
        attach_clock_probe(t);
        launch_gemm_stream(FA, FB, t, cus, stream);
    } else if (kernel == 1) {
        if (kstep_major) launch_mx_tiled<FA, FB, true>(g, sa, sb, cus, stream);
        else launch_mx_tiled<FA, FB, false>(g, sa, sb, cus, stream);
    } else {
        hipLaunchKernelGGL((mx_gemm_generic_kernel<FA, FB>), dim3((unsigned)((g.N + 31) / 32), (unsigned)((g.M + 31) / 32)), dim3(64), 0, stream, g, sa, sb,
                           kstep_major);
    }
}

template <int SRC, int FMT, bool TWO_D>
static void launch_block_cast(const void *x, int64_t rows, int64_t cols, int margin, uint8_t *out, uint8_t *scales, uint8_t *out_t,
                              uint8_t *scales_t, hipStream_t stream) {
    const dim3 grid((unsigned)((rows / 128) * (cols / 128))), block(256);
    uint32_t *s = reinterpret_cast<uint32_t *>(scales), *st = reinterpret_cast<uint32_t *>(scales_t);
#define ODL_BLK(R, C) hipLaunchKernelGGL((block_cast_kernel<SRC, FMT, TWO_D, R, C>), grid, block, 0, stream, x, rows, cols, margin, out, s, out_t, st)
    if (out && out_t) ODL_BLK(true, true);
    else if (out) ODL_BLK(true, false);
    else ODL_BLK(false, true);
#undef ODL_BLK
}

}  // namespace odl

using namespace odl;

extern "C" int odl_fp8_mx_cast(const void *x, int src_dtype, int64_t rows, int64_t cols, int fmt, uint8_t *out, uint8_t *scales,
                               int scales_layout, uint8_t *out_t, uint8_t *scales_t, int scales_t_layout, int scale_rule,
                               odl_stream_t stream_) {
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    if (rows < 0 || cols < 0) return set_error(ODL_ERR_ARG, "odl_fp8_mx_cast: negative shape");
    if (scale_rule != ODL_MX_SCALE_FLOOR && scale_rule != ODL_MX_SCALE_CEIL) return set_error(ODL_ERR_ARG, "odl_fp8_mx_cast: scale_rule %d", scale_rule);
    if (src_dtype != ODL_BF16 && src_dtype != ODL_F32) return set_error(ODL_ERR_ARG, "odl_fp8_mx_cast: src_dtype %d", src_dtype);
    if (fmt != ODL_FP8_E4M3 && fmt != ODL_FP8_E5M2) return set_error(ODL_ERR_ARG, "odl_fp8_mx_cast: fmt %d", fmt);
    if (rows * cols == 0) return ODL_OK;
    if ((out == nullptr) != (scales == nullptr) || (out_t == nullptr) != (scales_t == nullptr))
        return set_error(ODL_ERR_ARG, "odl_fp8_mx_cast: codes and scale bytes of a layout go together");
    if (!out && !out_t) return set_error(ODL_ERR_ARG, "odl_fp8_mx_cast: neither layout asked for");
    auto bad_layout = [](int l) { return l != ODL_MX_SCALES_ROWMAJOR && l != ODL_MX_SCALES_KSTEP; };
    if ((out && bad_layout(scales_layout)) || (out_t && bad_layout(scales_t_layout)))
        return set_error(ODL_ERR_ARG, "odl_fp8_mx_cast: scale layouts %d, %d", scales_layout, scales_t_layout);
    if ((out && scales_layout == ODL_MX_SCALES_KSTEP && cols % 128 != 0) || (out_t && scales_t_layout == ODL_MX_SCALES_KSTEP && rows % 128 != 0))
        return set_error(ODL_ERR_SHAPE, "odl_fp8_mx_cast: K-step-major scales need the blocked axis to be a multiple of 128 (%lld x %lld)",
                         (long long)rows, (long long)cols);
    if (!x) return set_error(ODL_ERR_ARG, "odl_fp8_mx_cast: x is null");
    if (cols % 8 != 0 || (out && cols % kMxBlock != 0) || (out_t && rows % kMxBlock != 0))
        return set_error(ODL_ERR_SHAPE, "odl_fp8_mx_cast: %lld x %lld: the blocked axis must be a multiple of 32 (cols for out, rows for out_t) and cols of 8",
                         (long long)rows, (long long)cols);
    auto mis = [](const void *p, uintptr_t a) { return p && (reinterpret_cast<uintptr_t>(p) & (a - 1)); };
    if (mis(x, 16) || mis(out, 8) || mis(out_t, 16)) return set_error(ODL_ERR_SHAPE, "odl_fp8_mx_cast: x and out_t must be 16-byte aligned, out 8-byte");
    const int64_t tiles = ((rows + kTileR - 1) / kTileR) * ((cols + kTileC - 1) / kTileC);
    if (tiles > 0x7fffffffLL) return set_error(ODL_ERR_SHAPE, "odl_fp8_mx_cast: too many tiles for one launch");
    if (src_dtype == ODL_BF16) {
        if (fmt == ODL_FP8_E4M3) launch_mx_cast<ODL_BF16, ODL_FP8_E4M3>(x, rows, cols, out, scales, out_t, scales_t, scales_layout, scales_t_layout, scale_rule, stream);
        else launch_mx_cast<ODL_BF16, ODL_FP8_E5M2>(x, rows, cols, out, scales, out_t, scales_t, scales_layout, scales_t_layout, scale_rule, stream);
    } else {
        if (fmt == ODL_FP8_E4M3) launch_mx_cast<ODL_F32, ODL_FP8_E4M3>(x, rows, cols, out, scales, out_t, scales_t, scales_layout, scales_t_layout, scale_rule, stream);
        else launch_mx_cast<ODL_F32, ODL_FP8_E5M2>(x, rows, cols, out, scales, out_t, scales_t, scales_layout, scales_t_layout, scale_rule, stream);
    }
    return check_launch("odl_fp8_mx_cast");
}

extern "C" int odl_fp8_mx_gemm_nt(const uint8_t *a, const uint8_t *sa, const uint8_t *b, const uint8_t *sb, int scales_layout, int64_t M,
                                  int64_t N, int64_t K, int fmt_a, int fmt_b, const float *bias, void *c, int out_dtype, int accumulate, odl_stream_t stream_) {
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    if (M < 0 || N < 0 || K < 0) return set_error(ODL_ERR_ARG, "odl_fp8_mx_gemm_nt: negative shape");
    if ((fmt_a != ODL_FP8_E4M3 && fmt_a != ODL_FP8_E5M2) || (fmt_b != ODL_FP8_E4M3 && fmt_b != ODL_FP8_E5M2))
        return set_error(ODL_ERR_ARG, "odl_fp8_mx_gemm_nt: formats %d, %d", fmt_a, fmt_b);
    if (out_dtype != ODL_BF16 && out_dtype != ODL_F32) return set_error(ODL_ERR_ARG, "odl_fp8_mx_gemm_nt: out_dtype %d", out_dtype);
    if (M == 0 || N == 0) return ODL_OK;
    if (!a || !sa || !b || !sb || !c) return set_error(ODL_ERR_ARG, "odl_fp8_mx_gemm_nt: null pointer");
    if (K == 0 || K % kMxBlock != 0) return set_error(ODL_ERR_SHAPE, "odl_fp8_mx_gemm_nt: K = %lld must be a positive multiple of 32", (long long)K);
    if (scales_layout != ODL_MX_SCALES_ROWMAJOR && scales_layout != ODL_MX_SCALES_KSTEP)
        return set_error(ODL_ERR_ARG, "odl_fp8_mx_gemm_nt: scales_layout %d", scales_layout);
    const int ks = scales_layout == ODL_MX_SCALES_KSTEP;
    if (ks && K % 128 != 0) return set_error(ODL_ERR_SHAPE, "odl_fp8_mx_gemm_nt: K-step-major scales need K %% 128 == 0 (K = %lld)", (long long)K);
    auto mis = [](const void *p, uintptr_t al) { return (reinterpret_cast<uintptr_t>(p) & (al - 1)) != 0; };
    if (mis(a, 16) || mis(b, 16) || mis(c, 16) || (bias && mis(bias, 16)))
        return set_error(ODL_ERR_SHAPE, "odl_fp8_mx_gemm_nt: operands, output and bias must be 16-byte aligned");
    const float *one = unit_scale_for_current_device("odl_fp8_mx_gemm_nt");
    if (!one) return ODL_ERR_LAUNCH;
    GemmArgs g{};
    g.a = a; g.b = b; g.c = c; g.sa = one; g.sb = one; g.bias = bias;
    g.M = M; g.N = N; g.K = K; g.sa_vec = 0; g.sb_vec = 0; g.out_dtype = out_dtype;
    g.accumulate = accumulate != 0;
    // the tiled and the streaming kernel address rows with 32-bit offsets and read whole scale dwords (4 blocks = one
    // 128-byte K step); the streaming kernel wants the scales K-step-major and the shapes of gemm_stream_accepts, and
    // pays only when more than half the compute units get one of its 256 x 256 tiles (at exactly half, outputs of
    // 8192 x 1024, the 128 x 128 kernel is 3 us faster at K = 1024 .. 3072, as for the per-tensor GEMMs)
    const bool lim32 = (double)(M + 256) * (double)K < 2147483648.0 && (double)(N + 256) * (double)K < 2147483648.0;
    const bool tiled = K % 128 == 0 && !mis(sa, 4) && !mis(sb, 4) && lim32 && M >= 32 && N >= 32;
    GemmArgs probe = g;
    probe.mx_sa = sa; probe.mx_sb = sb;
    const int cus = device_cu_count();
    const bool stream_ok = !accumulate && ks && tiled && ((M + 255) / 256) * ((N + 255) / 256) * 2 > cus && gemm_stream_accepts(probe);
    const int kernel = stream_ok ? 2 : (tiled ? 1 : 0);
#define ODL_MXG(FA_, FB_) launch_mx_gemm<FA_, FB_>(g, sa, sb, kernel, ks, cus, stream)
    if (fmt_a == ODL_FP8_E4M3 && fmt_b == ODL_FP8_E4M3) ODL_MXG(ODL_FP8_E4M3, ODL_FP8_E4M3);
    else if (fmt_a == ODL_FP8_E5M2 && fmt_b == ODL_FP8_E4M3) ODL_MXG(ODL_FP8_E5M2, ODL_FP8_E4M3);
    else if (fmt_a == ODL_FP8_E4M3 && fmt_b == ODL_FP8_E5M2) ODL_MXG(ODL_FP8_E4M3, ODL_FP8_E5M2);
    else ODL_MXG(ODL_FP8_E5M2, ODL_FP8_E5M2);
#undef ODL_MXG
    return check_launch("odl_fp8_mx_gemm_nt");
}

extern "C" int odl_fp8_block_cast(const void *x, int src_dtype, int64_t rows, int64_t cols, int fmt, int margin, int two_d, uint8_t *out,
                                  uint8_t *scales, uint8_t *out_t, uint8_t *scales_t, odl_stream_t stream_) {
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    if (rows < 0 || cols < 0) return set_error(ODL_ERR_ARG, "odl_fp8_block_cast: negative shape");
    if (src_dtype != ODL_BF16 && src_dtype != ODL_F32) return set_error(ODL_ERR_ARG, "odl_fp8_block_cast: src_dtype %d", src_dtype);
    if (fmt != ODL_FP8_E4M3 && fmt != ODL_FP8_E5M2) return set_error(ODL_ERR_ARG, "odl_fp8_block_cast: fmt %d", fmt);
    if (margin < -64 || margin > 64) return set_error(ODL_ERR_ARG, "odl_fp8_block_cast: margin %d", margin);
    if (rows * cols == 0) return ODL_OK;
    if ((out == nullptr) != (scales == nullptr) || (out_t == nullptr) != (scales_t == nullptr))
        return set_error(ODL_ERR_ARG, "odl_fp8_block_cast: codes and scale bytes of a layout go together");
    if (!out && !out_t) return set_error(ODL_ERR_ARG, "odl_fp8_block_cast: neither layout asked for");
    if (!x) return set_error(ODL_ERR_ARG, "odl_fp8_block_cast: x is null");
    if (rows % 128 != 0 || cols % 128 != 0)
        return set_error(ODL_ERR_SHAPE, "odl_fp8_block_cast: %lld x %lld: both sizes must be multiples of 128", (long long)rows, (long long)cols);
    auto mis = [](const void *p, uintptr_t a) { return p && (reinterpret_cast<uintptr_t>(p) & (a - 1)); };
    if (mis(x, 16) || mis(out, 16) || mis(out_t, 16) || mis(scales, 4) || mis(scales_t, 4))
        return set_error(ODL_ERR_SHAPE, "odl_fp8_block_cast: x and the codes must be 16-byte aligned, the scale arrays 4-byte");
    if ((rows / 128) * (cols / 128) > 0x7fffffffLL) return set_error(ODL_ERR_SHAPE, "odl_fp8_block_cast: too many tiles for one launch");
#define ODL_BLK(S, F) \
    do { if (two_d) launch_block_cast<S, F, true>(x, rows, cols, margin, out, scales, out_t, scales_t, stream); \
         else launch_block_cast<S, F, false>(x, rows, cols, margin, out, scales, out_t, scales_t, stream); } while (0)
    if (src_dtype == ODL_BF16) { if (fmt == ODL_FP8_E4M3) ODL_BLK(ODL_BF16, ODL_FP8_E4M3); else ODL_BLK(ODL_BF16, ODL_FP8_E5M2); }
    else { if (fmt == ODL_FP8_E4M3) ODL_BLK(ODL_F32, ODL_FP8_E4M3); else ODL_BLK(ODL_F32, ODL_FP8_E5M2); }
#undef ODL_BLK
    return check_launch("odl_fp8_block_cast");
}

// The block-scaled GEMM with K cut into `splits` runs computed side by side (outputs of few tiles and a long contraction:
// weight gradients of small layers), as odl_fp8_gemm_splitk does for per-tensor scales: every run leaves an fp32 partial
// result in the caller's workspace, a second kernel adds them in run order, adds the bias and rounds once.
extern "C" int odl_fp8_mx_gemm_splitk(const uint8_t *a, const uint8_t *sa, const uint8_t *b, const uint8_t *sb, int64_t M, int64_t N, int64_t K,
                                      int fmt_a, int fmt_b, const float *bias, void *c, int out_dtype, int accumulate, int splits, void *workspace,
                                      int64_t workspace_bytes, odl_stream_t stream_) {
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    if (!a || !sa || !b || !sb || !c || !workspace) return set_error(ODL_ERR_ARG, "odl_fp8_mx_gemm_splitk: null pointer");
    if ((fmt_a != ODL_FP8_E4M3 && fmt_a != ODL_FP8_E5M2) || (fmt_b != ODL_FP8_E4M3 && fmt_b != ODL_FP8_E5M2))
        return set_error(ODL_ERR_ARG, "odl_fp8_mx_gemm_splitk: formats %d, %d", fmt_a, fmt_b);
    if (out_dtype != ODL_BF16 && out_dtype != ODL_F32) return set_error(ODL_ERR_ARG, "odl_fp8_mx_gemm_splitk: out_dtype %d", out_dtype);
    auto mis = [](const void *p, uintptr_t al) { return (reinterpret_cast<uintptr_t>(p) & (al - 1)) != 0; };
    if (mis(a, 16) || mis(b, 16) || mis(c, 16) || mis(workspace, 16) || mis(sa, 4) || mis(sb, 4) || (bias && mis(bias, 16)))
        return set_error(ODL_ERR_SHAPE, "odl_fp8_mx_gemm_splitk: operands, output, workspace and bias must be 16-byte aligned, scales 4-byte");
    const bool sizes_ok = M > 0 && N > 0 && M % 128 == 0 && N % 128 == 0 && K % 128 == 0 &&
                          (double)(M + 256) * (double)K < 2147483648.0 && (double)(N + 256) * (double)K < 2147483648.0;
    if (!sizes_ok)
        return set_error(ODL_ERR_SHAPE, "odl_fp8_mx_gemm_splitk: M, N, K must be multiples of 128 and each operand under 2 GiB; got %lld x %lld x %lld",
                         (long long)M, (long long)N, (long long)K);
    const int64_t steps = K / 128;
    const int64_t per = ((steps + splits - 1) / (splits > 0 ? splits : 1) + 1) & ~(int64_t)1;
    if (splits < 2 || splits > 64 || per < 4 || steps - (splits - 1) * per < 4)
        return set_error(ODL_ERR_ARG, "odl_fp8_mx_gemm_splitk: %d splits of K=%lld leave a run shorter than 512", splits, (long long)K);
    if (workspace_bytes < (int64_t)splits * M * N * 4)
        return set_error(ODL_ERR_ARG, "odl_fp8_mx_gemm_splitk: workspace of %lld bytes, %lld needed", (long long)workspace_bytes,
                         (long long)splits * M * N * 4);
    const float *one = unit_scale_for_current_device("odl_fp8_mx_gemm_splitk");
    if (!one) return ODL_ERR_LAUNCH;
    GemmArgs g{};
    g.a = a; g.b = b; g.c = workspace; g.sa = one; g.sb = one; g.bias = nullptr;
    g.M = M; g.N = N; g.K = K; g.sa_vec = 0; g.sb_vec = 0; g.out_dtype = ODL_F32;
    g.splits = splits; g.split_steps = (int)per;
    g.mx_sa = sa; g.mx_sb = sb;
    g.tiles_m = (int)((M + 255) / 256); g.tiles_n = (int)((N + 255) / 256);
    if (!gemm_stream_accepts(g)) return set_error(ODL_ERR_SHAPE, "odl_fp8_mx_gemm_splitk: shape not taken by the streaming kernel");
    attach_clock_probe(g);
    launch_gemm_stream(fmt_a, fmt_b, g, device_cu_count(), stream);
    launch_splitk_reduce((const float *)workspace, splits, M, N, one, 0, one, 0, bias, c, out_dtype, accumulate != 0, stream);
    return check_launch("odl_fp8_mx_gemm_splitk");
}
