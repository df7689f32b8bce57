// The 128 x 64 tile shared by the kernels that write FP8 codes both row-major and transposed: tile size, the order in
// which blocks take tiles, the LDS placement of the transposed tile and the in-register 4 x 4 byte transpose.
#pragma once

#include "common.h"

namespace odl {

constexpr int kTileR = 128, kTileC = 64;

// Order in which consecutive blocks take tiles: panels of kCtPanel tile rows, down the rows of a panel first.
// Blocks that run at the same time then write neighbouring 128-byte pieces of the same rows of the
// transposed output instead of pieces that lie a whole output row (a power of two for the usual token
// counts) apart; measured alone at 8192 x 4096 / 8192 x 14336: 28.6 -> 25.8 us, 90.3 -> 85.1 us.
constexpr int kCtPanel = 16;
__device__ __forceinline__ void ct_tile_of(int64_t id, int64_t tiles_r, int64_t tiles_c, int64_t &tr, int64_t &tc) {
    const int64_t pn = id / (kCtPanel * tiles_c), local = id % (kCtPanel * tiles_c);
    const int64_t gl = min((int64_t)kCtPanel, tiles_r - pn * kCtPanel);
    tr = pn * kCtPanel + local % gl;
    tc = local / gl;
}

// LDS placement of the transposed tile.  Measured on gfx950 (counting conflict cycles of single instructions):
// a 4-byte access is served 32 lanes per cycle and its lanes must differ in (dword address mod 32); 8- and 16-byte
// accesses are served 32 / 16 lanes per cycle over 64 four-byte banks.  The tile is kept as 32 lines of 256 bytes,
// one per PAIR of tile columns (even column in the first 128 bytes), each line rotated by 16 bytes per group of 8
// columns:
//   * the dword writes of a half-wave (8 column groups x 4 consecutive row groups) differ mod 32,
//   * the 16-byte reads stay aligned (ds_read_b128), and 16 consecutive lanes read one whole line.
// Offsets in bytes; `ty` is the lane's group of 4 rows (0..31), `m16` a chunk of 16 rows (0..7).
// (the second term separates lanes whose columns 4 tx + k share col >> 3, the layout of an fp32 source; where a lane's
// columns are 8 tx + k it is the same for all lanes of an instruction)
__device__ __forceinline__ int ct_lds_rot(int col) { return 4 * (col >> 3) + 16 * ((col >> 2) & 1); }
__device__ __forceinline__ int ct_lds_write_off(int col, int ty) {
    return (col >> 1) * 256 + ((((col & 1) * 32) + ty + ct_lds_rot(col)) & 63) * 4;
}
__device__ __forceinline__ int ct_lds_read_off(int col, int m16) {
    return (col >> 1) * 256 + ((((col & 1) * 32) + m16 * 4 + ct_lds_rot(col)) & 63) * 4;
}
// 16 bytes of rows m16*16.. of tile column col
__device__ __forceinline__ u32x4 ct_lds_read(const uint8_t *tile, int col, int m16) {
    return *reinterpret_cast<const u32x4 *>(&tile[ct_lds_read_off(col, m16)]);
}

// 4x4 byte transpose: in a[j] byte k  ->  out t[k] byte j
__device__ __forceinline__ void transpose4x4(const uint32_t a[4], uint32_t t[4]) {
    // v_perm_b32(hi, lo, sel): result byte i = bytes{hi:lo}[sel byte i], lo = bytes 0..3, hi = 4..7
    const uint32_t p01_lo = __builtin_amdgcn_perm(a[1], a[0], 0x05010400u);  // a0.b0 a1.b0 a0.b1 a1.b1
    const uint32_t p01_hi = __builtin_amdgcn_perm(a[1], a[0], 0x07030602u);  // a0.b2 a1.b2 a0.b3 a1.b3
    const uint32_t p23_lo = __builtin_amdgcn_perm(a[3], a[2], 0x05010400u);
    const uint32_t p23_hi = __builtin_amdgcn_perm(a[3], a[2], 0x07030602u);
    t[0] = __builtin_amdgcn_perm(p23_lo, p01_lo, 0x05040100u);               // a0.b0 a1.b0 a2.b0 a3.b0
    t[1] = __builtin_amdgcn_perm(p23_lo, p01_lo, 0x07060302u);
    t[2] = __builtin_amdgcn_perm(p23_hi, p01_hi, 0x05040100u);
    t[3] = __builtin_amdgcn_perm(p23_hi, p01_hi, 0x07060302u);
}

}  // namespace odl
