// Memory-bound half of the FP8 Linear path for gfx950: amax reductions,
// scale-and-cast, fused cast+transpose, and the scale bookkeeping kernels.
//
// All of these are bound by HBM bandwidth.  Design rules used throughout:
//   * 128-bit global loads, several in flight per lane before the first use;
//   * 64-lane wavefront reductions through DPP shuffles, one LDS slot per wave,
//     one atomic per block (amax is a max, so any reduction tree is exact);
//   * grids sized to a few waves of blocks per CU so all 8 XCDs stay busy and
//     the tail is short.
#include "common.h"
#include "ct_tile.h"

#include <float.h>

namespace odl {

// Row-major FP8 codes are stored with ordinary (cache-allocating) stores: the GEMM that reads them
// is the next kernel and finds them in the memory-side cache (measured: -3 % GEMM time inside a step).
// Transposed codes are read much later (wgrad): they are stored non-temporally.
#define ODL_CODE_STORE(val, ptr) (*(ptr) = (val))
constexpr int kThreads = 256;
// Kernels that end in one atomicMax per block use fat blocks and a small grid:
// same-address atomics from different XCDs retire one at a time (~8 ns each).
constexpr int kFatThreads = 1024;

__device__ __forceinline__ u32x4 load16(const void *p) { return *reinterpret_cast<const u32x4 *>(p); }

// ---------------------------------------------------------------- fill (tiny)
__global__ void fill_f32_kernel(float *p, int64_t n, float v) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}



// Optional tail of the per-tensor amax kernel: the block that finishes last turns the
// amax into scale and 1/scale, so current scaling needs no second launch.  `ws` is two
// dwords {amax bits, tickets}, zero on entry; the last block leaves them zero again.
struct FusedScale {
    uint32_t *ws;
    float *scale, *scale_inv;
    float fp8_max;
    int margin;
};

// ------------------------------------------------------------ amax, per tensor
// x viewed as n16 chunks of 16 bytes plus a scalar tail.  Each lane keeps UNROLL
// loads in flight; magnitudes are reduced as integer bit patterns.
// The amax kernels read with ordinary (cache-allocating) loads on purpose: the cast
// that follows reads the same tensor again, and finds it in the 256 MB memory-side
// cache if this pass left it there.  With non-temporal loads this pass is a little
// faster but the cast runs at HBM speed (measured: 159 -> 124 us for the pair on a
// 235 MB tensor).
// OUT: 0 = atomicMax into out[0]; 1 = fused scale (see FusedScale); 2 = out[blockIdx] = this block's
// maximum, no atomics at all: the cast that follows reduces the kAmaxParts partials itself.
constexpr int kAmaxParts = ODL_FP8_AMAX_PARTS;

// Maximum of |x| over the 16-byte chunks i0, i0 + stride, ... < n16 of x, as fp32 magnitude bits; UNROLL loads
// in flight per lane.
template <int SRC, int UNROLL>
__device__ __forceinline__ uint32_t amax_chunks(const void *__restrict__ x, int64_t n16, int64_t i0, int64_t stride) {
    const u32x4 *p = reinterpret_cast<const u32x4 *>(x);
    int64_t i = i0;
    uint32_t m0 = 0, m1 = 0, m2 = 0, m3 = 0;
    for (; i + (UNROLL - 1) * stride < n16; i += UNROLL * stride) {
        u32x4 v[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) v[u] = p[i + u * stride];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            if constexpr (SRC == ODL_BF16) {
                m0 = max_u16x2(m0, abs_bf16x2(v[u].x));
                m1 = max_u16x2(m1, abs_bf16x2(v[u].y));
                m2 = max_u16x2(m2, abs_bf16x2(v[u].z));
                m3 = max_u16x2(m3, abs_bf16x2(v[u].w));
            } else {
                m0 = max(m0, v[u].x & 0x7fffffffu);
                m1 = max(m1, v[u].y & 0x7fffffffu);
                m2 = max(m2, v[u].z & 0x7fffffffu);
                m3 = max(m3, v[u].w & 0x7fffffffu);
            }
        }
    }
    // the rest (fewer than UNROLL chunks for this lane) as one more batch of loads with the missing ones left out:
    // taken one at a time they were up to UNROLL - 1 memory latencies in a row at the end of every block
    if (i < n16) {
        u32x4 v[UNROLL - 1];
#pragma unroll
        for (int u = 0; u < UNROLL - 1; ++u) v[u] = (i + u * stride < n16) ? p[i + u * stride] : u32x4{0, 0, 0, 0};
#pragma unroll
        for (int u = 0; u < UNROLL - 1; ++u) {
            if constexpr (SRC == ODL_BF16) {
                m0 = max_u16x2(m0, abs_bf16x2(v[u].x));
                m1 = max_u16x2(m1, abs_bf16x2(v[u].y));
                m2 = max_u16x2(m2, abs_bf16x2(v[u].z));
                m3 = max_u16x2(m3, abs_bf16x2(v[u].w));
            } else {
                m0 = max(m0, v[u].x & 0x7fffffffu);
                m1 = max(m1, v[u].y & 0x7fffffffu);
                m2 = max(m2, v[u].z & 0x7fffffffu);
                m3 = max(m3, v[u].w & 0x7fffffffu);
            }
        }
    }
    if constexpr (SRC == ODL_BF16) return fold_u16x2_to_f32bits(max_u16x2(max_u16x2(m0, m1), max_u16x2(m2, m3)));
    else return max(max(m0, m1), max(m2, m3));
}

template <int SRC, int UNROLL, int OUT>
__global__ __launch_bounds__(kFatThreads) void amax_tensor_kernel(const void *__restrict__ x, int64_t n,
                                                                   float *__restrict__ out, const FusedScale fs) {
    __shared__ uint32_t red[kFatThreads / kWave];
    constexpr int EPC = SRC == ODL_BF16 ? 8 : 4;          // elements per 16-byte chunk
    const int64_t n16 = n / EPC;
    uint32_t m = amax_chunks<SRC, UNROLL>(x, n16, (int64_t)blockIdx.x * kFatThreads + threadIdx.x, (int64_t)gridDim.x * kFatThreads);
    // scalar tail (fewer than EPC elements), done by one thread
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        for (int64_t t = n16 * EPC; t < n; ++t) {
            uint32_t b;
            if constexpr (SRC == ODL_BF16) b = ((uint32_t) reinterpret_cast<const uint16_t *>(x)[t] & 0x7fffu) << 16;
            else b = reinterpret_cast<const uint32_t *>(x)[t] & 0x7fffffffu;
            m = max(m, b);
        }
    }
    m = block_max_u32(m, red);
    if constexpr (OUT == 2) {
        if (threadIdx.x == 0) out[blockIdx.x] = bits_to_float(m);
        if (blockIdx.x == 0)                                  // entries no block owns
            for (int i = (int)gridDim.x + threadIdx.x; i < kAmaxParts; i += kFatThreads) out[i] = 0.0f;
    } else if constexpr (OUT == 0) {
        if (threadIdx.x == 0 && m != 0) atomicMax(reinterpret_cast<uint32_t *>(out), m);
    } else if (threadIdx.x == 0) {
        // Device-scope atomics are performed at the point of coherence, and one that returns a
        // value has been performed when the value arrives.  The ticket is made to depend on the
        // value returned by the max, so it is drawn after the max has landed: no fence (which would
        // write back this XCD's whole L2) is needed to order the two.
        uint32_t prev = atomicMax(fs.ws, m);
        uint32_t one = 1u;
        asm volatile("" : "+v"(one) : "v"(prev));
        if (atomicAdd(fs.ws + 1, one) == gridDim.x - 1) {     // every other block has drawn its ticket
            const float amax = bits_to_float(atomicExch(fs.ws, 0u));
            atomicExch(fs.ws + 1, 0u);
            const float sc = scale_rule(amax, fs.fp8_max, fs.margin, 1.0f);
            out[0] = amax;
            fs.scale[0] = sc;
            if (fs.scale_inv) fs.scale_inv[0] = __fdiv_rn(1.0f, sc);
        }
    }
}

// element-at-a-time variant for pointers that are not 16-byte aligned
template <int SRC>
__global__ __launch_bounds__(kThreads) void amax_tensor_scalar_kernel(const void *__restrict__ x, int64_t n,
                                                                       float *__restrict__ out) {
    __shared__ uint32_t red[kThreads / kWave];
    uint32_t m = 0;
    for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += (int64_t)gridDim.x * kThreads) {
        uint32_t b;
        if constexpr (SRC == ODL_BF16) b = ((uint32_t) reinterpret_cast<const uint16_t *>(x)[i] & 0x7fffu) << 16;
        else b = reinterpret_cast<const uint32_t *>(x)[i] & 0x7fffffffu;
        m = max(m, b);
    }
    m = block_max_u32(m, red);
    if (threadIdx.x == 0 && m != 0) atomicMax(reinterpret_cast<uint32_t *>(out), m);
}

// ---------------------------------------------------------------- amax, per row
// One wavefront per row, kThreads/64 rows per block.  Handles any cols; the
// 16-byte path is used for the aligned middle of the row.
template <int SRC, bool ACC>
__global__ __launch_bounds__(kThreads) void amax_row_kernel(const void *__restrict__ x, int64_t rows, int64_t cols,
                                                             float *__restrict__ out) {
    constexpr int ESZ = SRC == ODL_BF16 ? 2 : 4;
    constexpr int EPC = 16 / ESZ;
    const int lane = threadIdx.x % kWave;
    const int64_t row = (int64_t)blockIdx.x * (kThreads / kWave) + threadIdx.x / kWave;
    if (row >= rows) return;
    const char *base = reinterpret_cast<const char *>(x) + row * cols * ESZ;
    // elements before the first 16-byte boundary
    int64_t head = ((16 - (reinterpret_cast<uintptr_t>(base) & 15)) & 15) / ESZ;
    if (head > cols) head = cols;
    const int64_t n16 = (cols - head) / EPC;
    auto elem_bits = [&](int64_t c) -> uint32_t {
        if constexpr (SRC == ODL_BF16) return ((uint32_t) reinterpret_cast<const uint16_t *>(base)[c] & 0x7fffu) << 16;
        else return reinterpret_cast<const uint32_t *>(base)[c] & 0x7fffffffu;
    };
    uint32_t m = 0;
    for (int64_t c = lane; c < head; c += kWave) m = max(m, elem_bits(c));
    for (int64_t c = head + n16 * EPC + lane; c < cols; c += kWave) m = max(m, elem_bits(c));
    const u32x4 *p = reinterpret_cast<const u32x4 *>(base + head * ESZ);
    uint32_t a0 = 0, a1 = 0, a2 = 0, a3 = 0;
    int64_t i = lane;
    for (; i + 3 * kWave < n16; i += 4 * kWave) {
        u32x4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = p[i + u * kWave];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            if constexpr (SRC == ODL_BF16) {
                a0 = max_u16x2(a0, abs_bf16x2(v[u].x)); a1 = max_u16x2(a1, abs_bf16x2(v[u].y));
                a2 = max_u16x2(a2, abs_bf16x2(v[u].z)); a3 = max_u16x2(a3, abs_bf16x2(v[u].w));
            } else {
                a0 = max(a0, v[u].x & 0x7fffffffu); a1 = max(a1, v[u].y & 0x7fffffffu);
                a2 = max(a2, v[u].z & 0x7fffffffu); a3 = max(a3, v[u].w & 0x7fffffffu);
            }
        }
    }
    for (; i < n16; i += kWave) {
        u32x4 v = p[i];
        if constexpr (SRC == ODL_BF16) {
            a0 = max_u16x2(a0, abs_bf16x2(v.x)); a1 = max_u16x2(a1, abs_bf16x2(v.y));
            a2 = max_u16x2(a2, abs_bf16x2(v.z)); a3 = max_u16x2(a3, abs_bf16x2(v.w));
        } else {
            a0 = max(a0, v.x & 0x7fffffffu); a1 = max(a1, v.y & 0x7fffffffu);
            a2 = max(a2, v.z & 0x7fffffffu); a3 = max(a3, v.w & 0x7fffffffu);
        }
    }
    if constexpr (SRC == ODL_BF16) m = max(m, fold_u16x2_to_f32bits(max_u16x2(max_u16x2(a0, a1), max_u16x2(a2, a3))));
    else m = max(m, max(max(a0, a1), max(a2, a3)));
    m = wave_max_u32(m);
    if (lane == 0) {
        uint32_t *o = reinterpret_cast<uint32_t *>(out) + row;
        if constexpr (ACC) { if (m > *o) *o = m; }     // one writer per row: plain read-modify-write
        else *o = m;
    }
}

// ------------------------------------------------------------- amax, per column
// Block = 32 column-lanes x 8 row-lanes; each lane owns CPL consecutive columns
// (one 16-byte load) and walks ROWS_PER_BLOCK rows in steps of 8.  Column maxima
// are combined through LDS, then one atomicMax per column per block.
template <int SRC>
__global__ __launch_bounds__(kThreads) void amax_col_kernel(const void *__restrict__ x, int64_t rows, int64_t cols,
                                                             int rows_per_block, float *__restrict__ out) {
    constexpr int ESZ = SRC == ODL_BF16 ? 2 : 4;
    constexpr int CPL = 16 / ESZ;                 // columns per lane
    constexpr int CW = 32 * CPL;                  // columns per block
    __shared__ uint32_t red[8][CW + 1];
    const int tx = threadIdx.x % 32, ty = threadIdx.x / 32;
    const int64_t c0 = (int64_t)blockIdx.x * CW + tx * CPL;
    const int64_t r0 = (int64_t)blockIdx.y * rows_per_block;
    const int64_t r1 = min(rows, r0 + rows_per_block);
    uint32_t m[CPL];
#pragma unroll
    for (int j = 0; j < CPL; ++j) m[j] = 0;
    const char *base = reinterpret_cast<const char *>(x);
    if (c0 + CPL <= cols) {                        // host guarantees cols % CPL == 0 and 16-byte rows
        int64_t r = r0 + ty;
        for (; r + 24 < r1; r += 32) {
            u32x4 v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = *reinterpret_cast<const u32x4 *>(base + ((r + 8 * u) * cols + c0) * ESZ);
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                uint32_t w[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    if constexpr (SRC == ODL_BF16) {
                        uint32_t a = abs_bf16x2(w[q]);
                        m[2 * q] = max(m[2 * q], (a & 0xffffu) << 16);
                        m[2 * q + 1] = max(m[2 * q + 1], a & 0xffff0000u);
                    } else {
                        m[q] = max(m[q], w[q] & 0x7fffffffu);
                    }
                }
            }
        }
        for (; r < r1; r += 8) {
            u32x4 v = *reinterpret_cast<const u32x4 *>(base + (r * cols + c0) * ESZ);
            uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                if constexpr (SRC == ODL_BF16) {
                    uint32_t a = abs_bf16x2(w[q]);
                    m[2 * q] = max(m[2 * q], (a & 0xffffu) << 16);
                    m[2 * q + 1] = max(m[2 * q + 1], a & 0xffff0000u);
                } else {
                    m[q] = max(m[q], w[q] & 0x7fffffffu);
                }
            }
        }
    }
#pragma unroll
    for (int j = 0; j < CPL; ++j) red[ty][tx * CPL + j] = m[j];
    __syncthreads();
    for (int c = threadIdx.x; c < CW; c += kThreads) {
        uint32_t v = 0;
#pragma unroll
        for (int y = 0; y < 8; ++y) v = max(v, red[y][c]);
        const int64_t col = (int64_t)blockIdx.x * CW + c;
        if (col < cols && v != 0) atomicMax(reinterpret_cast<uint32_t *>(out) + col, v);
    }
}

// ----------------------------------------------------- amax, per row AND per column
// One pass for the rowwise recipe, which scales a tensor along its rows for one GEMM and along
// its columns for another.  Same lane tile as amax_col_kernel; in addition every loaded 16-byte
// piece is folded to one value and reduced over the 32 lanes that share its row (xor shuffles stay
// inside a 32-lane half), and the first lane of the half does one atomicMax per row and block.
// Both outputs accumulate (atomicMax): the caller zeroes them.
template <int SRC>
__global__ __launch_bounds__(kThreads) void amax_rowcol_kernel(const void *__restrict__ x, int64_t rows, int64_t cols,
                                                                int rows_per_block, float *__restrict__ out_row,
                                                                float *__restrict__ out_col) {
    constexpr int ESZ = SRC == ODL_BF16 ? 2 : 4;
    constexpr int CPL = 16 / ESZ;                 // columns per lane
    constexpr int CW = 32 * CPL;                  // columns per block
    __shared__ uint32_t red[8][CW + 1];
    const int tx = threadIdx.x % 32, ty = threadIdx.x / 32;
    const int64_t c0 = (int64_t)blockIdx.x * CW + tx * CPL;
    const int64_t r0 = (int64_t)blockIdx.y * rows_per_block;
    const int64_t r1 = min(rows, r0 + rows_per_block);
    const bool col_ok = c0 + CPL <= cols;          // host guarantees cols % CPL == 0 and 16-byte rows
    uint32_t m[CPL];
#pragma unroll
    for (int j = 0; j < CPL; ++j) m[j] = 0;
    const char *base = reinterpret_cast<const char *>(x);
    // every lane walks the same rows (the shuffles need all 32 lanes of a row); r1 - r0 is a multiple of 8
    // except in the last slab, where rows past the end load nothing
    for (int64_t rb = r0; rb < r1; rb += 32) {
        u32x4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int64_t r = rb + ty + 8 * u;
            v[u] = (col_ok && r < r1) ? *reinterpret_cast<const u32x4 *>(base + (r * cols + c0) * ESZ) : u32x4{0, 0, 0, 0};
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const uint32_t w[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
            uint32_t rowmax = 0;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                if constexpr (SRC == ODL_BF16) {
                    const uint32_t a = abs_bf16x2(w[q]);
                    const uint32_t lo = (a & 0xffffu) << 16, hi = a & 0xffff0000u;
                    m[2 * q] = max(m[2 * q], lo);
                    m[2 * q + 1] = max(m[2 * q + 1], hi);
                    rowmax = max(rowmax, max(lo, hi));
                } else {
                    const uint32_t a = w[q] & 0x7fffffffu;
                    m[q] = max(m[q], a);
                    rowmax = max(rowmax, a);
                }
            }
#pragma unroll
            for (int off = 16; off > 0; off >>= 1) {
                const uint32_t o = (uint32_t)__shfl_xor((int)rowmax, off, kWave);
                rowmax = rowmax > o ? rowmax : o;
            }
            const int64_t r = rb + ty + 8 * u;
            if (tx == 0 && r < r1 && rowmax != 0) atomicMax(reinterpret_cast<uint32_t *>(out_row) + r, rowmax);
        }
    }
#pragma unroll
    for (int j = 0; j < CPL; ++j) red[ty][tx * CPL + j] = m[j];
    __syncthreads();
    for (int c = threadIdx.x; c < CW; c += kThreads) {
        uint32_t v = 0;
#pragma unroll
        for (int y = 0; y < 8; ++y) v = max(v, red[y][c]);
        const int64_t col = (int64_t)blockIdx.x * CW + c;
        if (col < cols && v != 0) atomicMax(reinterpret_cast<uint32_t *>(out_col) + col, v);
    }
}

// generic column amax for shapes the vector kernel refuses: one thread per column strip
template <int SRC>
__global__ void amax_col_scalar_kernel(const void *__restrict__ x, int64_t rows, int64_t cols, int rows_per_block,
                                       float *__restrict__ out) {
    const int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= cols) return;
    const int64_t r0 = (int64_t)blockIdx.y * rows_per_block, r1 = min(rows, r0 + rows_per_block);
    uint32_t m = 0;
    for (int64_t r = r0; r < r1; ++r) {
        uint32_t b;
        if constexpr (SRC == ODL_BF16) b = ((uint32_t) reinterpret_cast<const uint16_t *>(x)[r * cols + c] & 0x7fffu) << 16;
        else b = reinterpret_cast<const uint32_t *>(x)[r * cols + c] & 0x7fffffffu;
        m = max(m, b);
    }
    if (m != 0) atomicMax(reinterpret_cast<uint32_t *>(out) + c, m);
}

// ------------------------------------------------------------- scale from amax
__global__ void scale_from_amax_kernel(const float *__restrict__ amax, int64_t n, float fp8_max, int margin,
                                       float *__restrict__ scale, float *__restrict__ scale_inv) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float s = scale_rule(amax[i], fp8_max, margin, 1.0f);
    scale[i] = s;
    if (scale_inv) scale_inv[i] = __fdiv_rn(1.0f, s);
}

// Delayed-scaling refresh of R roles: amax = max over the window (or the newest entry), history rolled by -1
// with row 0 cleared, scale and 1/scale by the scale rule.  `parts` (optional) holds kAmaxParts partial maxima
// per role that the casts of this step recorded: they are folded into row 0 first and cleared.
// A block owns 16 roles; its 256 lanes are 16 lanes per role.  The roll runs in place: lane `seg` of a role
// moves rows [seg*S, (seg+1)*S) down by one, reading ahead of its own writes; the one row that a neighbouring
// lane overwrites (the last of the segment) is read before a block-wide barrier.  History lengths of 1024
// (the reference's default) cost 64 rows per lane instead of a chain of 1024 dependent loads.
constexpr int kUpdRoles = 16, kUpdSegs = kThreads / kUpdRoles;

__global__ __launch_bounds__(kThreads) void delayed_update_kernel(float *__restrict__ history, int64_t H, int64_t R, int64_t ld,
                                                                  float *__restrict__ scale, float *__restrict__ scale_inv,
                                                                  const int *__restrict__ fmt, int margin, int algo,
                                                                  float *__restrict__ parts) {
    __shared__ uint32_t s_part[kUpdRoles];
    __shared__ uint32_t s_max[kUpdSegs][kUpdRoles];
    const int64_t r_base = (int64_t)blockIdx.x * kUpdRoles;
    // ---- partial maxima of this step: 16 lanes per role, 8 x 16 bytes per lane
    {
        const int role = threadIdx.x / kUpdSegs, lane = threadIdx.x % kUpdSegs;
        const int64_t r = r_base + role;
        uint32_t m = 0;
        if (parts && r < R) {
            u32x4 *p = reinterpret_cast<u32x4 *>(parts + r * kAmaxParts);
            u32x4 v[kAmaxParts / 4 / kUpdSegs];
#pragma unroll
            for (int j = 0; j < kAmaxParts / 4 / kUpdSegs; ++j) v[j] = p[lane + kUpdSegs * j];
#pragma unroll
            for (int j = 0; j < kAmaxParts / 4 / kUpdSegs; ++j) {
                m = max(m, max(max(v[j].x & 0x7fffffffu, v[j].y & 0x7fffffffu), max(v[j].z & 0x7fffffffu, v[j].w & 0x7fffffffu)));
                p[lane + kUpdSegs * j] = u32x4{0, 0, 0, 0};
            }
        }
#pragma unroll
        for (int off = kUpdSegs / 2; off > 0; off >>= 1) m = max(m, (uint32_t)__shfl_xor((int)m, off, kUpdSegs));
        if (lane == 0) s_part[role] = m;
    }
    __syncthreads();
    // ---- the roll: lane (c, seg) owns rows [lo, hi) of role r
    const int c = threadIdx.x % kUpdRoles, seg = threadIdx.x / kUpdRoles;
    const int64_t r = r_base + c;
    const bool valid = r < R;
    const int64_t S = (H + kUpdSegs - 1) / kUpdSegs;
    const int64_t lo = seg * S, hi = min(H, lo + S);
    const bool has_rows = valid && lo < hi;
    // amaxes are >= 0 or NaN: the integer maximum of the magnitude bits keeps a NaN
    // (what is stored back are the entries as they were, sign and NaN payload included)
    uint32_t first = 0, first_mag = 0, tail = 0, abits = 0;
    if (has_rows) tail = float_to_bits(history[(hi - 1) * ld + r]);
    if (valid && seg == 0) {
        first = float_to_bits(history[r]);
        first_mag = first & 0x7fffffffu;
        if (s_part[c] > first_mag) first = first_mag = s_part[c];
    }
    __syncthreads();                                          // every segment's last row is in a register
    if (has_rows) {
        abits = tail & 0x7fffffffu;
        constexpr int kAhead = 8;
        int64_t h = max(lo, (int64_t)1);                      // row 0 moves to row H - 1 (below), not down
        for (; h + kAhead <= hi - 1; h += kAhead) {
            uint32_t v[kAhead];
#pragma unroll
            for (int u = 0; u < kAhead; ++u) v[u] = float_to_bits(history[(h + u) * ld + r]);
#pragma unroll
            for (int u = 0; u < kAhead; ++u) {
                abits = max(abits, v[u] & 0x7fffffffu);
                history[(h + u - 1) * ld + r] = (h + u == 1) ? 0.0f : bits_to_float(v[u]);
            }
        }
        for (; h < hi - 1; ++h) {
            const uint32_t v = float_to_bits(history[h * ld + r]);
            abits = max(abits, v & 0x7fffffffu);
            history[(h - 1) * ld + r] = h == 1 ? 0.0f : bits_to_float(v);
        }
        if (hi - 1 >= 1) history[(hi - 2) * ld + r] = hi - 1 == 1 ? 0.0f : bits_to_float(tail);   // the row read before the barrier
    }
    s_max[seg][c] = abits;
    __syncthreads();
    if (valid && seg == 0) {
        // row 0 held this step's amax (seg 0 read it as its tail when S == 1, as `first` always)
        uint32_t window = first_mag;
        if (algo == ODL_AMAX_MAX)
            for (int g = 0; g < kUpdSegs; ++g) window = max(window, s_max[g][c]);
        history[(H - 1) * ld + r] = bits_to_float(first);
        history[r] = 0.0f;                                    // also when H == 1: the only row starts the next step empty
        const float fmax = fmt[r] == ODL_FP8_E5M2 ? 57344.0f : 448.0f;
        const float sc = scale_rule(bits_to_float(window), fmax, margin, scale[r]);
        scale[r] = sc;
        scale_inv[r] = __fdiv_rn(1.0f, sc);
    }
}

// ------------------------------------------------- current scaling inside the cast
// MODE == kScaleParts: `scale` points at kAmaxParts partial maxima (amax_tensor_kernel<.., 2>).
// Every block reduces them (2 KB from L2), derives the per-tensor scale, and block 0 records
// {amax, scale, 1/scale} in dyn_out for the GEMM: no kernel between the amax pass and the cast.
constexpr int kScaleParts = 3;

template <int FMT>
__device__ __forceinline__ float dynamic_scale(const float *__restrict__ parts, int margin, float *__restrict__ dyn_out,
                                               uint32_t *red, bool record) {
    __shared__ float s_bcast;
    uint32_t m = 0;
    for (int i = threadIdx.x; i < kAmaxParts; i += blockDim.x) m = max(m, float_to_bits(parts[i]));
    m = block_max_u32(m, red);
    if (threadIdx.x == 0) {
        const float amax = bits_to_float(m);
        const float sc = scale_rule(amax, Fp8Lim<FMT>::max, margin, 1.0f);
        s_bcast = sc;
        if (record && dyn_out) {
            dyn_out[0] = amax;
            dyn_out[1] = sc;
            dyn_out[2] = __fdiv_rn(1.0f, sc);
        }
    }
    __syncthreads();
    return s_bcast;
}

// one block: the same reduction for the element-at-a-time route
template <int FMT>
__global__ __launch_bounds__(kThreads) void parts_to_scale_kernel(const float *__restrict__ parts, int margin, float *__restrict__ dyn_out) {
    __shared__ uint32_t red[kThreads / kWave];
    dynamic_scale<FMT>(parts, margin, dyn_out, red, true);
}

// Per-tensor scale given (delayed scaling): the first block also hands back 1/scale, the factor the GEMM
// multiplies by, in storage of the caller's.  The scale itself is refreshed in place after the step; a GEMM
// of this step, or its backward, must not read the refreshed value.
__device__ __forceinline__ void record_scale_inv(float s, float *__restrict__ scale_inv_out) {
    if (scale_inv_out && blockIdx.x == 0 && threadIdx.x == 0) scale_inv_out[0] = __fdiv_rn(1.0f, s);
}

// ------------------------------------------------------------------------ cast
// A wave works on spans of 1024 elements: VP load instructions, each of which has the 64 lanes read 1024 contiguous
// bytes (lane l takes the 16-byte piece h * 64 + l of the span with instruction h), one store per piece.  A lane
// that instead read its 16 elements as neighbouring 16-byte pieces would leave every instruction a half (bf16) or a
// quarter (fp32) of each 64-byte request, and non-temporal loads are not merged across instructions: fp32 sources ran
// at 0.49 of the HBM peak that way (4096 x 14336, bf16 0.68).  cols % 16 == 0 and 16-byte aligned pointers
// (host-checked), so a piece never crosses a row.
template <int SRC, int FMT, int MODE, bool AMAX>
__global__ __launch_bounds__(AMAX ? kFatThreads : kThreads) void cast_kernel(const void *__restrict__ x, int64_t rows, int64_t cols,
                                                         const float *__restrict__ scale, uint8_t *__restrict__ out,
                                                         float *__restrict__ amax_out, int margin, float *__restrict__ dyn_out,
                                                         int amax_mask) {
    constexpr int kT = AMAX ? kFatThreads : kThreads;
    __shared__ uint32_t red[kT / kWave];
    const int64_t n = rows * cols;
    float s_t = 1.0f;
    if constexpr (MODE == ODL_SCALE_TENSOR) {
        s_t = scale[0];
        record_scale_inv(s_t, dyn_out);
    }
    if constexpr (MODE == kScaleParts) s_t = dynamic_scale<FMT>(scale, margin, dyn_out, red, blockIdx.x == 0);
    uint32_t am = 0;
    constexpr int VP = SRC == ODL_BF16 ? 2 : 4;              // 16-byte pieces per lane and span
    constexpr int EPP = SRC == ODL_BF16 ? 8 : 4;             // elements per piece
    constexpr int U = SRC == ODL_BF16 ? 2 : 1;               // spans in flight per wave
    const int lane = threadIdx.x % kWave;
    // one piece: EPP elements from element index e on
    auto one = [&](const int64_t e, const u32x4 v) {
        float f[8];
        if constexpr (SRC == ODL_BF16) {
            const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                f[2 * q] = bf16_lo(w[q]);
                f[2 * q + 1] = bf16_hi(w[q]);
                if constexpr (AMAX) am = max_u16x2(am, abs_bf16x2(w[q]));
            }
        } else {
            f[0] = bits_to_float(v.x); f[1] = bits_to_float(v.y); f[2] = bits_to_float(v.z); f[3] = bits_to_float(v.w);
            f[4] = f[5] = f[6] = f[7] = 0.0f;
            if constexpr (AMAX) am = max(am, max(max(v.x & 0x7fffffffu, v.y & 0x7fffffffu), max(v.z & 0x7fffffffu, v.w & 0x7fffffffu)));
        }
        float sc[8];
        if constexpr (MODE == ODL_SCALE_TENSOR || MODE == kScaleParts) {
#pragma unroll
            for (int j = 0; j < 8; ++j) sc[j] = s_t;
        } else if constexpr (MODE == ODL_SCALE_ROW) {
            const float sr = scale[e / cols];
#pragma unroll
            for (int j = 0; j < 8; ++j) sc[j] = sr;
        } else {
            const float4 *sp = reinterpret_cast<const float4 *>(scale + e % cols);
#pragma unroll
            for (int u = 0; u < EPP / 4; ++u) { float4 t = sp[u]; sc[4 * u] = t.x; sc[4 * u + 1] = t.y; sc[4 * u + 2] = t.z; sc[4 * u + 3] = t.w; }
        }
        const uint32_t lo = quantise4<FMT>(f[0], f[1], f[2], f[3], sc[0], sc[1], sc[2], sc[3]);
        if constexpr (SRC == ODL_BF16) {
            const uint32_t hi = quantise4<FMT>(f[4], f[5], f[6], f[7], sc[4], sc[5], sc[6], sc[7]);
            ODL_CODE_STORE((u32x2{lo, hi}), reinterpret_cast<u32x2 *>(out + e));
        } else {
            ODL_CODE_STORE(lo, reinterpret_cast<uint32_t *>(out + e));
        }
    };
    const char *px = reinterpret_cast<const char *>(x);
    constexpr int ESZ = SRC == ODL_BF16 ? 2 : 4;
    const int64_t nspan = (n + 1023) / 1024;
    const int64_t stride = (int64_t)gridDim.x * (kT / kWave);
    int64_t sp = (int64_t)blockIdx.x * (kT / kWave) + threadIdx.x / kWave;
    for (; sp + (U - 1) * stride < nspan; sp += U * stride) {
        u32x4 v[U][VP];
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int h = 0; h < VP; ++h) {
                const int64_t e = (sp + u * stride) * 1024 + (h * kWave + lane) * EPP;
                v[u][h] = e < n ? __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(px + e * ESZ)) : u32x4{0, 0, 0, 0};
            }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int h = 0; h < VP; ++h) {
                const int64_t e = (sp + u * stride) * 1024 + (h * kWave + lane) * EPP;
                if (e < n) one(e, v[u][h]);
            }
    }
    for (; sp < nspan; sp += stride) {
        u32x4 v[VP];
#pragma unroll
        for (int h = 0; h < VP; ++h) {
            const int64_t e = sp * 1024 + (h * kWave + lane) * EPP;
            v[h] = e < n ? __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(px + e * ESZ)) : u32x4{0, 0, 0, 0};
        }
#pragma unroll
        for (int h = 0; h < VP; ++h) {
            const int64_t e = sp * 1024 + (h * kWave + lane) * EPP;
            if (e < n) one(e, v[h]);
        }
    }
    if constexpr (AMAX) {
        if constexpr (SRC == ODL_BF16) am = fold_u16x2_to_f32bits(am);
        am = block_max_u32(am, red);
        if (threadIdx.x == 0 && am != 0) atomicMax(reinterpret_cast<uint32_t *>(amax_out) + (blockIdx.x & amax_mask), am);
    }
}

// element-at-a-time cast (+ optional transposed copy) for any shape / alignment
template <int SRC, int FMT>
__global__ __launch_bounds__(kThreads) void cast_generic_kernel(const void *__restrict__ x, int64_t rows, int64_t cols,
                                                                 const float *__restrict__ scale, int mode,
                                                                 uint8_t *__restrict__ out, uint8_t *__restrict__ out_t,
                                                                 float *__restrict__ amax_out) {
    __shared__ uint32_t red[kThreads / kWave];
    uint32_t am = 0;
    const int64_t n = rows * cols;
    for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += (int64_t)gridDim.x * kThreads) {
        const int64_t r = i / cols, c = i % cols;
        float f;
        if constexpr (SRC == ODL_BF16) f = bits_to_float((uint32_t) reinterpret_cast<const uint16_t *>(x)[i] << 16);
        else f = reinterpret_cast<const float *>(x)[i];
        am = max(am, float_to_bits(f) & 0x7fffffffu);
        const float s = mode == ODL_SCALE_TENSOR ? scale[0] : (mode == ODL_SCALE_ROW ? scale[r] : scale[c]);
        const uint8_t q = (uint8_t)(quantise4<FMT>(f, 0.f, 0.f, 0.f, s, 1.f, 1.f, 1.f) & 0xffu);
        if (out) out[i] = q;
        if (out_t) out_t[c * rows + r] = q;
    }
    if (amax_out) {
        am = block_max_u32(am, red);
        if (threadIdx.x == 0 && am != 0) atomicMax(reinterpret_cast<uint32_t *>(amax_out), am);
    }
}

// -------------------------------------------------------------- cast+transpose
// Tile = 128 rows x 64 cols of x per block of 256 lanes.  A lane owns 4 rows x 8 columns: bf16 source, columns
// 8 tx .. 8 tx + 7 (one 16-byte load a row); fp32 source, columns 4 tx .. 4 tx + 3 and 32 + 4 tx .. 32 + 4 tx + 3 (two
// loads a row, each of which has the 8 lanes of a row read 128 contiguous bytes: non-temporal loads are not merged
// across instructions, and with a lane's 32 bytes side by side every instruction used half of each 64-byte request;
// 4096 x 14336 fp32 ran at 0.55 of the HBM peak that way).  The row-major codes leave as
// 8-byte (fp32 source: two 4-byte) stores (a wave covers whole 64-byte row segments); the transposed codes
// go through a 4x4 byte transpose in registers (v_perm_b32) and an LDS tile
// [64 cols][128 rows] so that they leave as 16-byte stores along the row axis:
// both outputs are written in full 64/128-byte segments.  (Tile helpers: ct_tile.h.)
//
// One 128 x 64 tile (tr, tc) of x: convert, write the row-major codes, transpose through `tile` (LDS), write the
// transposed codes.  `st` is the per-tensor scale (modes TENSOR and parts), `scale` the vector of the ROW / COL modes.
// Ends after the transposed stores: a caller that reuses `tile` puts a barrier in between.
// first tile column of the lane's group g (0 / 1) of 4 columns
template <int SRC>
__device__ __forceinline__ int ct_group_col(int tx, int g) { return SRC == ODL_BF16 ? tx * 8 + 4 * g : tx * 4 + 32 * g; }

// the lane's 8 elements of row r: columns cA .. cA + 3 and cB .. cB + 3 (bf16: cB = cA + 4, one load)
template <int SRC>
__device__ __forceinline__ void ct_load_row(const void *__restrict__ x, int64_t r, int64_t rows, int64_t cols, int64_t cA, int64_t cB,
                                            bool okA, bool okB, u32x4 (&raw)[SRC == ODL_BF16 ? 1 : 2]) {
    constexpr int ESZ = SRC == ODL_BF16 ? 2 : 4;
    const bool row_ok = r < rows;
    const char *row = reinterpret_cast<const char *>(x) + r * cols * ESZ;
    raw[0] = (okA && row_ok) ? __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(row + cA * ESZ)) : u32x4{0, 0, 0, 0};
    if constexpr (SRC != ODL_BF16)
        raw[1] = (okB && row_ok) ? __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(row + cB * ESZ)) : u32x4{0, 0, 0, 0};
}

// the lane's 8 row-major codes of row r
template <int SRC>
__device__ __forceinline__ void ct_store_row(uint8_t *__restrict__ out, int64_t r, int64_t rows, int64_t cols, int64_t cA, int64_t cB,
                                             bool okA, bool okB, uint32_t lo, uint32_t hi) {
    if (r >= rows) return;
    if constexpr (SRC == ODL_BF16) {
        if (okA) ODL_CODE_STORE((u32x2{lo, hi}), reinterpret_cast<u32x2 *>(out + r * cols + cA));
    } else {
        if (okA) ODL_CODE_STORE(lo, reinterpret_cast<uint32_t *>(out + r * cols + cA));
        if (okB) ODL_CODE_STORE(hi, reinterpret_cast<uint32_t *>(out + r * cols + cB));
    }
}

template <int SRC, int FMT, int MODE, bool AMAX, bool WRITE_ROWMAJOR>
__device__ __forceinline__ void ct_one_tile(const void *__restrict__ x, int64_t rows, int64_t cols, const float *__restrict__ scale,
                                            float st, uint8_t *__restrict__ out, uint8_t *__restrict__ out_t, int64_t tr,
                                            int64_t tc, uint8_t *tile, uint32_t &am) {
    constexpr int ESZ = SRC == ODL_BF16 ? 2 : 4;
    const int tx = threadIdx.x % 8;                 // 8 lanes across 64 columns
    const int ty = threadIdx.x / 8;                 // 32 lane-rows, 4 rows each
    // tile columns of the lane's two groups of 4 (codes lo / hi below)
    const int kA = ct_group_col<SRC>(tx, 0), kB = ct_group_col<SRC>(tx, 1);
    const int64_t r0 = tr * kTileR + ty * 4, cA = tc * kTileC + kA, cB = tc * kTileC + kB;
    const bool okA = cA < cols, okB = cB < cols;    // cols % 8 == 0 (host-checked), so a group of 4 is in or out as a whole

    float s_col[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) s_col[j] = 1.0f;
    if constexpr (MODE == ODL_SCALE_TENSOR || MODE == kScaleParts) {
#pragma unroll
        for (int j = 0; j < 8; ++j) s_col[j] = st;
    } else if constexpr (MODE == ODL_SCALE_COL) {
        if (okA) {
            const float4 t0 = *reinterpret_cast<const float4 *>(scale + cA);
            s_col[0] = t0.x; s_col[1] = t0.y; s_col[2] = t0.z; s_col[3] = t0.w;
        }
        if (okB) {
            const float4 t1 = *reinterpret_cast<const float4 *>(scale + cB);
            s_col[4] = t1.x; s_col[5] = t1.y; s_col[6] = t1.z; s_col[7] = t1.w;
        }
    }

    // ---- load the 4 x 8 patch (rows beyond the matrix read as zero)
    u32x4 raw[4][ESZ / 2];
#pragma unroll
    for (int i = 0; i < 4; ++i) ct_load_row<SRC>(x, r0 + i, rows, cols, cA, cB, okA, okB, raw[i]);

    uint32_t lo[4], hi[4];                          // codes of columns 0..3 / 4..7 for each of the 4 rows
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        float f[8];
        if constexpr (SRC == ODL_BF16) {
            uint32_t w[4] = {raw[i][0].x, raw[i][0].y, raw[i][0].z, raw[i][0].w};
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                f[2 * q] = bf16_lo(w[q]);
                f[2 * q + 1] = bf16_hi(w[q]);
                if constexpr (AMAX) am = max_u16x2(am, abs_bf16x2(w[q]));
            }
        } else {
            uint32_t w[8] = {raw[i][0].x, raw[i][0].y, raw[i][0].z, raw[i][0].w, raw[i][1].x, raw[i][1].y, raw[i][1].z, raw[i][1].w};
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                f[q] = bits_to_float(w[q]);
                if constexpr (AMAX) am = max(am, w[q] & 0x7fffffffu);
            }
        }
        float s[8];
        if constexpr (MODE == ODL_SCALE_ROW) {
            const float sr = (r0 + i) < rows ? scale[r0 + i] : 1.0f;
#pragma unroll
            for (int j = 0; j < 8; ++j) s[j] = sr;
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) s[j] = s_col[j];
        }
        lo[i] = quantise4<FMT>(f[0], f[1], f[2], f[3], s[0], s[1], s[2], s[3]);
        hi[i] = quantise4<FMT>(f[4], f[5], f[6], f[7], s[4], s[5], s[6], s[7]);
        if constexpr (WRITE_ROWMAJOR) ct_store_row<SRC>(out, r0 + i, rows, cols, cA, cB, okA, okB, lo[i], hi[i]);
    }

    // ---- transpose in registers, stage through LDS
    uint32_t tl[4], th[4];
    transpose4x4(lo, tl);                           // tl[k] = rows r0..r0+3 of column c0+k
    transpose4x4(hi, th);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        *reinterpret_cast<uint32_t *>(&tile[ct_lds_write_off(kA + k, ty)]) = tl[k];
        *reinterpret_cast<uint32_t *>(&tile[ct_lds_write_off(kB + k, ty)]) = th[k];
    }
    __syncthreads();
    // 64 tile-columns x 8 chunks of 16 rows = 512 chunks, two per lane
#pragma unroll
    for (int it = 0; it < 2; ++it) {
        const int chunk = threadIdx.x + it * kThreads;
        const int k = chunk / 8, m16 = chunk % 8;
        const int64_t oc = tc * kTileC + k, orow = tr * kTileR + m16 * 16;
        if (oc < cols && orow < rows) {             // rows % 16 == 0 (host-checked)
            const u32x4 v = ct_lds_read(tile, k, m16);
            __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(out_t + oc * rows + orow));
        }
    }
}

template <int SRC, int FMT, int MODE, bool AMAX, bool WRITE_ROWMAJOR>
__global__ __launch_bounds__(kThreads) void cast_transpose_kernel(const void *__restrict__ x, int64_t rows, int64_t cols,
                                                                   const float *__restrict__ scale,
                                                                   uint8_t *__restrict__ out, uint8_t *__restrict__ out_t,
                                                                   float *__restrict__ amax_out, int margin, float *__restrict__ dyn_out,
                                                                   int amax_mask) {
    __shared__ __attribute__((aligned(16))) uint8_t tile[kTileC * kTileR];
    __shared__ uint32_t red[kThreads / kWave];
    float st = 1.0f;
    if constexpr (MODE == kScaleParts) st = dynamic_scale<FMT>(scale, margin, dyn_out, red, blockIdx.x == 0);
    if constexpr (MODE == ODL_SCALE_TENSOR) {
        st = scale[0];
        record_scale_inv(st, dyn_out);
    }
    const int64_t tiles_c = (cols + kTileC - 1) / kTileC;
    const int64_t ntiles = tiles_c * ((rows + kTileR - 1) / kTileR);
    uint32_t am = 0;
    // With a maximum folded into one word the grid is small and each block walks several tiles, so
    // that the kernel ends in few atomics; otherwise one tile per block.
    for (int64_t tile_id = blockIdx.x; tile_id < ntiles; tile_id += gridDim.x) {
        // Tiles are walked from the end of the tensor: the amax pass that ran just before read it front
        // to back, so its tail is what the memory-side cache still holds.
        int64_t tr, tc;
        ct_tile_of(ntiles - 1 - tile_id, (rows + kTileR - 1) / kTileR, tiles_c, tr, tc);
        ct_one_tile<SRC, FMT, MODE, AMAX, WRITE_ROWMAJOR>(x, rows, cols, scale, st, out, out_t, tr, tc, tile, am);
        if (tile_id + gridDim.x < ntiles) __syncthreads();  // the LDS tile is reused by the next trip
    }
    if constexpr (AMAX) {
        if constexpr (SRC == ODL_BF16) am = fold_u16x2_to_f32bits(am);
        am = block_max_u32(am, red);
        if (threadIdx.x == 0 && am != 0) atomicMax(reinterpret_cast<uint32_t *>(amax_out) + (blockIdx.x & amax_mask), am);
    }
}

// ----------------------------------------------------------------- host helpers
// ---------------------------------------- cast for the rowwise recipe, both operands at once
// out   [rows, cols] = codes scaled per ROW    (scale derived from amax_row)
// out_t [cols, rows] = codes scaled per COLUMN (scale derived from amax_col), transposed
// One read of x instead of the two that a cast and a cast+transpose would make.  The 128 row
// scales and 64 column scales of a tile are derived once per block (IEEE division) and kept in
// LDS; the blocks of the first tile column / row also record 1/scale for the GEMM epilogues.
template <int SRC, int FMT>
__global__ __launch_bounds__(kThreads) void cast_rowcol_kernel(const void *__restrict__ x, int64_t rows, int64_t cols,
                                                                const float *__restrict__ amax_row, const float *__restrict__ amax_col,
                                                                int margin, uint8_t *__restrict__ out, uint8_t *__restrict__ out_t,
                                                                float *__restrict__ s_row_out, float *__restrict__ s_row_inv,
                                                                float *__restrict__ s_col_out, float *__restrict__ s_col_inv) {
    __shared__ __attribute__((aligned(16))) uint8_t tile[kTileC * kTileR];
    __shared__ float s_row[kTileR], s_col[kTileC];
    constexpr int ESZ = SRC == ODL_BF16 ? 2 : 4;
    const int tx = threadIdx.x % 8;                 // 8 lanes across 64 columns
    const int ty = threadIdx.x / 8;                 // 32 lane-rows, 4 rows each
    const int64_t tiles_c = (cols + kTileC - 1) / kTileC;
    int64_t tr, tc;
    ct_tile_of(blockIdx.x, (rows + kTileR - 1) / kTileR, tiles_c, tr, tc);
    if (threadIdx.x < kTileR) {
        const int64_t r = tr * kTileR + threadIdx.x;
        const float sc = r < rows ? scale_rule(amax_row[r], Fp8Lim<FMT>::max, margin, 1.0f) : 1.0f;
        s_row[threadIdx.x] = sc;
        if (tc == 0 && r < rows) { s_row_out[r] = sc; s_row_inv[r] = __fdiv_rn(1.0f, sc); }
    } else if (threadIdx.x < kTileR + kTileC) {
        const int64_t c = tc * kTileC + (threadIdx.x - kTileR);
        const float sc = c < cols ? scale_rule(amax_col[c], Fp8Lim<FMT>::max, margin, 1.0f) : 1.0f;
        s_col[threadIdx.x - kTileR] = sc;
        if (tr == 0 && c < cols) { s_col_out[c] = sc; s_col_inv[c] = __fdiv_rn(1.0f, sc); }
    }
    __syncthreads();
    const int kA = ct_group_col<SRC>(tx, 0), kB = ct_group_col<SRC>(tx, 1);     // the lane's columns, as in ct_one_tile
    const int64_t r0 = tr * kTileR + ty * 4, cA = tc * kTileC + kA, cB = tc * kTileC + kB;
    const bool okA = cA < cols, okB = cB < cols;    // cols % 8 == 0 (host-checked)
    float sc_col[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) { sc_col[j] = s_col[kA + j]; sc_col[4 + j] = s_col[kB + j]; }

    u32x4 raw[4][ESZ / 2];
#pragma unroll
    for (int i = 0; i < 4; ++i) ct_load_row<SRC>(x, r0 + i, rows, cols, cA, cB, okA, okB, raw[i]);
    uint32_t lo[4], hi[4];                          // column-scaled codes of columns 0..3 / 4..7 for each of the 4 rows
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        float f[8];
        if constexpr (SRC == ODL_BF16) {
            const uint32_t w[4] = {raw[i][0].x, raw[i][0].y, raw[i][0].z, raw[i][0].w};
#pragma unroll
            for (int q = 0; q < 4; ++q) { f[2 * q] = bf16_lo(w[q]); f[2 * q + 1] = bf16_hi(w[q]); }
        } else {
            const uint32_t w[8] = {raw[i][0].x, raw[i][0].y, raw[i][0].z, raw[i][0].w, raw[i][1].x, raw[i][1].y, raw[i][1].z, raw[i][1].w};
#pragma unroll
            for (int q = 0; q < 8; ++q) f[q] = bits_to_float(w[q]);
        }
        const float sr = s_row[ty * 4 + i];
        const uint32_t rlo = quantise4<FMT>(f[0], f[1], f[2], f[3], sr, sr, sr, sr);
        const uint32_t rhi = quantise4<FMT>(f[4], f[5], f[6], f[7], sr, sr, sr, sr);
        ct_store_row<SRC>(out, r0 + i, rows, cols, cA, cB, okA, okB, rlo, rhi);
        lo[i] = quantise4<FMT>(f[0], f[1], f[2], f[3], sc_col[0], sc_col[1], sc_col[2], sc_col[3]);
        hi[i] = quantise4<FMT>(f[4], f[5], f[6], f[7], sc_col[4], sc_col[5], sc_col[6], sc_col[7]);
    }
    // ---- transpose in registers, stage through LDS (as in cast_transpose_kernel)
    uint32_t tl[4], th[4];
    transpose4x4(lo, tl);
    transpose4x4(hi, th);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        *reinterpret_cast<uint32_t *>(&tile[ct_lds_write_off(kA + k, ty)]) = tl[k];
        *reinterpret_cast<uint32_t *>(&tile[ct_lds_write_off(kB + k, ty)]) = th[k];
    }
    __syncthreads();
#pragma unroll
    for (int it = 0; it < 2; ++it) {
        const int chunk = threadIdx.x + it * kThreads;
        const int k = chunk / 8, m16 = chunk % 8;
        const int64_t oc = tc * kTileC + k, orow = tr * kTileR + m16 * 16;
        if (oc < cols && orow < rows) {             // rows % 16 == 0 (host-checked)
            const u32x4 v = ct_lds_read(tile, k, m16);
            __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(out_t + oc * rows + orow));
        }
    }
}

static inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

static int num_cus() { return device_cu_count(); }

static int64_t grid_for(int64_t work_items, int per_block, int blocks_per_cu) {
    int64_t need = (work_items + per_block - 1) / per_block;
    int64_t cap = (int64_t)num_cus() * blocks_per_cu;
    return need < 1 ? 1 : (need < cap ? need : cap);
}

}  // namespace odl

using namespace odl;

extern "C" int odl_fp8_amax(const void *x, int src_dtype, int64_t rows, int64_t cols, int mode, float *amax_out,
                            int accumulate, odl_stream_t stream_) {
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    if (rows < 0 || cols < 0) return set_error(ODL_ERR_ARG, "odl_fp8_amax: negative shape %lld x %lld", (long long)rows, (long long)cols);
    if ((!x && rows * cols > 0) || !amax_out) return set_error(ODL_ERR_ARG, "odl_fp8_amax: null pointer");
    if (src_dtype != ODL_BF16 && src_dtype != ODL_F32) return set_error(ODL_ERR_ARG, "odl_fp8_amax: src_dtype %d", src_dtype);
    if (mode < ODL_SCALE_TENSOR || mode > ODL_SCALE_COL) return set_error(ODL_ERR_ARG, "odl_fp8_amax: mode %d", mode);
    const int64_t n_out = mode == ODL_SCALE_TENSOR ? 1 : (mode == ODL_SCALE_ROW ? rows : cols);
    const int64_t n = rows * cols;
    const bool atomic_path = mode != ODL_SCALE_ROW;
    if (n_out > 0 && (!accumulate) && (atomic_path || n == 0))
        hipLaunchKernelGGL(fill_f32_kernel, dim3((unsigned)((n_out + 255) / 256)), dim3(256), 0, stream, amax_out, n_out, 0.0f);
    if (n == 0) return check_launch("odl_fp8_amax(fill)");
    const int esz = src_dtype == ODL_BF16 ? 2 : 4;
    if (mode == ODL_SCALE_TENSOR) {
        if (aligned16(x)) {
            const int64_t g = grid_for(n * esz / 16, kFatThreads * 4, 2);
            if (src_dtype == ODL_BF16) hipLaunchKernelGGL((amax_tensor_kernel<ODL_BF16, 4, 0>), dim3((unsigned)g), dim3(kFatThreads), 0, stream, x, n, amax_out, FusedScale{});
            else hipLaunchKernelGGL((amax_tensor_kernel<ODL_F32, 4, 0>), dim3((unsigned)g), dim3(kFatThreads), 0, stream, x, n, amax_out, FusedScale{});
        } else {
            const int64_t g = grid_for(n, kThreads * 8, 8);
            if (src_dtype == ODL_BF16) hipLaunchKernelGGL((amax_tensor_scalar_kernel<ODL_BF16>), dim3((unsigned)g), dim3(kThreads), 0, stream, x, n, amax_out);
            else hipLaunchKernelGGL((amax_tensor_scalar_kernel<ODL_F32>), dim3((unsigned)g), dim3(kThreads), 0, stream, x, n, amax_out);
        }
    } else if (mode == ODL_SCALE_ROW) {
        const int64_t g = (rows + (kThreads / kWave) - 1) / (kThreads / kWave);
        if (g > 0x7fffffffLL) return set_error(ODL_ERR_SHAPE, "odl_fp8_amax: too many rows");
#define ODL_ROW(SRC) \
        if (accumulate) hipLaunchKernelGGL((amax_row_kernel<SRC, true>), dim3((unsigned)g), dim3(kThreads), 0, stream, x, rows, cols, amax_out); \
        else hipLaunchKernelGGL((amax_row_kernel<SRC, false>), dim3((unsigned)g), dim3(kThreads), 0, stream, x, rows, cols, amax_out);
        if (src_dtype == ODL_BF16) { ODL_ROW(ODL_BF16) } else { ODL_ROW(ODL_F32) }
#undef ODL_ROW
    } else {
        const int cpl = 16 / esz, cw = 32 * cpl;
        // enough row-slabs for ~8 blocks per CU, each at least 64 rows tall
        int64_t col_blocks = (cols + cw - 1) / cw;
        int64_t want_slabs = ((int64_t)num_cus() * 8 + col_blocks - 1) / col_blocks;
        int64_t rpb = (rows + want_slabs - 1) / want_slabs;
        rpb = ((rpb + 31) / 32) * 32;
        if (rpb < 64) rpb = 64;
        const int64_t slabs = (rows + rpb - 1) / rpb;
        if (slabs > 65535) return set_error(ODL_ERR_SHAPE, "odl_fp8_amax: too many row slabs");
        if (aligned16(x) && cols % cpl == 0) {
            if (src_dtype == ODL_BF16) hipLaunchKernelGGL((amax_col_kernel<ODL_BF16>), dim3((unsigned)col_blocks, (unsigned)slabs), dim3(kThreads), 0, stream, x, rows, cols, (int)rpb, amax_out);
            else hipLaunchKernelGGL((amax_col_kernel<ODL_F32>), dim3((unsigned)col_blocks, (unsigned)slabs), dim3(kThreads), 0, stream, x, rows, cols, (int)rpb, amax_out);
        } else {
            const int64_t gx = (cols + 255) / 256;
            if (src_dtype == ODL_BF16) hipLaunchKernelGGL((amax_col_scalar_kernel<ODL_BF16>), dim3((unsigned)gx, (unsigned)slabs), dim3(256), 0, stream, x, rows, cols, (int)rpb, amax_out);
            else hipLaunchKernelGGL((amax_col_scalar_kernel<ODL_F32>), dim3((unsigned)gx, (unsigned)slabs), dim3(256), 0, stream, x, rows, cols, (int)rpb, amax_out);
        }
    }
    return check_launch("odl_fp8_amax");
}

extern "C" int odl_fp8_amax_scale(const void *x, int src_dtype, int64_t rows, int64_t cols, int fmt, int margin, float *amax_out,
                                  float *scale, float *scale_inv, uint32_t *workspace, odl_stream_t stream_) {
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    if (rows < 0 || cols < 0) return set_error(ODL_ERR_ARG, "odl_fp8_amax_scale: negative shape %lld x %lld", (long long)rows, (long long)cols);
    if ((!x && rows * cols > 0) || !amax_out || !scale || !workspace) return set_error(ODL_ERR_ARG, "odl_fp8_amax_scale: null pointer");
    if (src_dtype != ODL_BF16 && src_dtype != ODL_F32) return set_error(ODL_ERR_ARG, "odl_fp8_amax_scale: src_dtype %d", src_dtype);
    if (fmt != ODL_FP8_E4M3 && fmt != ODL_FP8_E5M2) return set_error(ODL_ERR_ARG, "odl_fp8_amax_scale: fmt %d", fmt);
    const int64_t n = rows * cols;
    if (n == 0 || !aligned16(x)) {
        // nothing to read, or a pointer the vector kernel cannot take: the two-launch route
        int rc = odl_fp8_amax(x, src_dtype, rows, cols, ODL_SCALE_TENSOR, amax_out, 0, stream_);
        if (rc != ODL_OK) return rc;
        return odl_fp8_scale_from_amax(amax_out, 1, fmt, margin, scale, scale_inv, stream_);
    }
    const int esz = src_dtype == ODL_BF16 ? 2 : 4;
    const int64_t g = grid_for(n * esz / 16, kFatThreads * 4, 2);
    const FusedScale fs{workspace, scale, scale_inv, fmt == ODL_FP8_E5M2 ? 57344.0f : 448.0f, margin};
    if (src_dtype == ODL_BF16) hipLaunchKernelGGL((amax_tensor_kernel<ODL_BF16, 4, 1>), dim3((unsigned)g), dim3(kFatThreads), 0, stream, x, n, amax_out, fs);
    else hipLaunchKernelGGL((amax_tensor_kernel<ODL_F32, 4, 1>), dim3((unsigned)g), dim3(kFatThreads), 0, stream, x, n, amax_out, fs);
    return check_launch("odl_fp8_amax_scale");
}

extern "C" int odl_fp8_scale_from_amax(const float *amax, int64_t n, int fmt, int margin, float *scale, float *scale_inv,
                                       odl_stream_t stream_) {
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    if (!amax || !scale) return set_error(ODL_ERR_ARG, "odl_fp8_scale_from_amax: null pointer");
    if (fmt != ODL_FP8_E4M3 && fmt != ODL_FP8_E5M2) return set_error(ODL_ERR_ARG, "odl_fp8_scale_from_amax: fmt %d", fmt);
    if (n < 0) return set_error(ODL_ERR_ARG, "odl_fp8_scale_from_amax: n < 0");
    if (n == 0) return ODL_OK;
    hipLaunchKernelGGL(scale_from_amax_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, amax, n,
                       fmt == ODL_FP8_E5M2 ? 57344.0f : 448.0f, margin, scale, scale_inv);
    return check_launch("odl_fp8_scale_from_amax");
}

extern "C" int odl_fp8_delayed_update(float *history, int64_t H, int64_t R, int64_t ld, float *scale, float *scale_inv,
                                      const int *fmt, int margin, int algo, float *amax_parts, odl_stream_t stream_) {
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    if (!history || !scale || !scale_inv || !fmt) return set_error(ODL_ERR_ARG, "odl_fp8_delayed_update: null pointer");
    if (H < 1 || R < 0 || ld < R) return set_error(ODL_ERR_ARG, "odl_fp8_delayed_update: H=%lld R=%lld ld=%lld", (long long)H, (long long)R, (long long)ld);
    if (algo != ODL_AMAX_MAX && algo != ODL_AMAX_MOST_RECENT) return set_error(ODL_ERR_ARG, "odl_fp8_delayed_update: algo %d", algo);
    if (amax_parts && !aligned16(amax_parts)) return set_error(ODL_ERR_ARG, "odl_fp8_delayed_update: amax_parts must be 16-byte aligned");
    if (R == 0) return ODL_OK;
    hipLaunchKernelGGL(delayed_update_kernel, dim3((unsigned)((R + kUpdRoles - 1) / kUpdRoles)), dim3(kThreads), 0, stream, history, H, R,
                       ld, scale, scale_inv, fmt, margin, algo, amax_parts);
    return check_launch("odl_fp8_delayed_update");
}

namespace odl {

template <int SRC, int FMT, int MODE>
static void launch_cast(const void *x, int64_t rows, int64_t cols, const float *scale, uint8_t *out, float *amax_out,
                        hipStream_t stream, int margin = 0, float *dyn_out = nullptr, int amax_mask = 0) {
    if (amax_out) {
        const int64_t g = grid_for(rows * cols / 16, kFatThreads, 2);
        hipLaunchKernelGGL((cast_kernel<SRC, FMT, MODE, true>), dim3((unsigned)g), dim3(kFatThreads), 0, stream, x, rows, cols, scale, out, amax_out, margin, dyn_out, amax_mask);
    } else {
        const int64_t g = grid_for(rows * cols / 16, kThreads, 16);
        hipLaunchKernelGGL((cast_kernel<SRC, FMT, MODE, false>), dim3((unsigned)g), dim3(kThreads), 0, stream, x, rows, cols, scale, out, amax_out, margin, dyn_out, amax_mask);
    }
}

template <int SRC, int FMT>
static void launch_cast_mode(int mode, const void *x, int64_t rows, int64_t cols, const float *scale, uint8_t *out,
                             float *amax_out, hipStream_t stream) {
    if (mode == ODL_SCALE_TENSOR) launch_cast<SRC, FMT, ODL_SCALE_TENSOR>(x, rows, cols, scale, out, amax_out, stream);
    else if (mode == ODL_SCALE_ROW) launch_cast<SRC, FMT, ODL_SCALE_ROW>(x, rows, cols, scale, out, amax_out, stream);
    else launch_cast<SRC, FMT, ODL_SCALE_COL>(x, rows, cols, scale, out, amax_out, stream);
}

template <int SRC, int FMT>
static void launch_generic(const void *x, int64_t rows, int64_t cols, const float *scale, int mode, uint8_t *out,
                           uint8_t *out_t, float *amax_out, hipStream_t stream) {
    const int64_t g = grid_for(rows * cols, kThreads * 4, 8);
    hipLaunchKernelGGL((cast_generic_kernel<SRC, FMT>), dim3((unsigned)g), dim3(kThreads), 0, stream, x, rows, cols, scale, mode, out, out_t, amax_out);
}

template <int SRC, int FMT, int MODE>
static void launch_ct(const void *x, int64_t rows, int64_t cols, const float *scale, uint8_t *out, uint8_t *out_t,
                      float *amax_out, hipStream_t stream, int margin = 0, float *dyn_out = nullptr, int amax_mask = 0) {
    int64_t g = ((rows + kTileR - 1) / kTileR) * ((cols + kTileC - 1) / kTileC);
    // maxima folded into ONE word: few blocks that walk several tiles each, so that the kernel ends in few
    // atomics on that word; spread over many words (amax_mask != 0), one tile per block as without a maximum
    if (amax_out && amax_mask == 0 && g > (int64_t)num_cus() * 4) g = (int64_t)num_cus() * 4;
#define ODL_CT(AM, RM) hipLaunchKernelGGL((cast_transpose_kernel<SRC, FMT, MODE, AM, RM>), dim3((unsigned)g), dim3(kThreads), 0, stream, x, rows, cols, scale, out, out_t, amax_out, margin, dyn_out, amax_mask)
    if (amax_out) { if (out) ODL_CT(true, true); else ODL_CT(true, false); }
    else { if (out) ODL_CT(false, true); else ODL_CT(false, false); }
#undef ODL_CT
}

template <int SRC, int FMT>
static void launch_ct_mode(int mode, const void *x, int64_t rows, int64_t cols, const float *scale, uint8_t *out,
                           uint8_t *out_t, float *amax_out, hipStream_t stream) {
    if (mode == ODL_SCALE_TENSOR) launch_ct<SRC, FMT, ODL_SCALE_TENSOR>(x, rows, cols, scale, out, out_t, amax_out, stream);
    else if (mode == ODL_SCALE_ROW) launch_ct<SRC, FMT, ODL_SCALE_ROW>(x, rows, cols, scale, out, out_t, amax_out, stream);
    else launch_ct<SRC, FMT, ODL_SCALE_COL>(x, rows, cols, scale, out, out_t, amax_out, stream);
}

static int check_cast_args(const char *who, const void *x, int src_dtype, int64_t rows, int64_t cols, const float *scale,
                           int mode, int fmt) {
    if (rows < 0 || cols < 0) return set_error(ODL_ERR_ARG, "%s: negative shape", who);
    if ((!x || !scale) && rows * cols > 0) return set_error(ODL_ERR_ARG, "%s: null pointer", who);
    if (src_dtype != ODL_BF16 && src_dtype != ODL_F32) return set_error(ODL_ERR_ARG, "%s: src_dtype %d", who, src_dtype);
    if (mode < ODL_SCALE_TENSOR || mode > ODL_SCALE_COL) return set_error(ODL_ERR_ARG, "%s: mode %d", who, mode);
    if (fmt != ODL_FP8_E4M3 && fmt != ODL_FP8_E5M2) return set_error(ODL_ERR_ARG, "%s: fmt %d", who, fmt);
    return ODL_OK;
}

}  // namespace odl

#define ODL_DISPATCH_SRC_FMT(FN, ...)                                             \
    do {                                                                          \
        if (src_dtype == ODL_BF16) {                                              \
            if (fmt == ODL_FP8_E4M3) FN<ODL_BF16, ODL_FP8_E4M3>(__VA_ARGS__);     \
            else FN<ODL_BF16, ODL_FP8_E5M2>(__VA_ARGS__);                         \
        } else {                                                                  \
            if (fmt == ODL_FP8_E4M3) FN<ODL_F32, ODL_FP8_E4M3>(__VA_ARGS__);      \
            else FN<ODL_F32, ODL_FP8_E5M2>(__VA_ARGS__);                          \
        }                                                                         \
    } while (0)

extern "C" int odl_fp8_cast(const void *x, int src_dtype, int64_t rows, int64_t cols, const float *scale, int mode, int fmt,
                            uint8_t *out, float *amax_out, odl_stream_t stream_) {
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    if (int e = check_cast_args("odl_fp8_cast", x, src_dtype, rows, cols, scale, mode, fmt)) return e;
    if (rows * cols == 0) return ODL_OK;
    if (!out) return set_error(ODL_ERR_ARG, "odl_fp8_cast: out is null");
    const bool fast = cols % 16 == 0 && aligned16(x) && aligned16(out) && (mode != ODL_SCALE_COL || aligned16(scale));
    if (fast) ODL_DISPATCH_SRC_FMT(launch_cast_mode, mode, x, rows, cols, scale, out, amax_out, stream);
    else ODL_DISPATCH_SRC_FMT(launch_generic, x, rows, cols, scale, mode, out, (uint8_t *)nullptr, amax_out, stream);
    return check_launch("odl_fp8_cast");
}

extern "C" int odl_fp8_cast_transpose(const void *x, int src_dtype, int64_t rows, int64_t cols, const float *scale, int mode,
                                      int fmt, uint8_t *out, uint8_t *out_t, float *amax_out, odl_stream_t stream_) {
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    if (int e = check_cast_args("odl_fp8_cast_transpose", x, src_dtype, rows, cols, scale, mode, fmt)) return e;
    if (rows * cols == 0) return ODL_OK;
    if (!out_t) return set_error(ODL_ERR_ARG, "odl_fp8_cast_transpose: out_t is null");
    const int64_t tiles = ((rows + kTileR - 1) / kTileR) * ((cols + kTileC - 1) / kTileC);
    const bool fast = cols % 8 == 0 && rows % 16 == 0 && aligned16(x) && aligned16(out_t) &&
                      (!out || (reinterpret_cast<uintptr_t>(out) & 7) == 0) &&
                      (mode != ODL_SCALE_COL || aligned16(scale)) && tiles <= 0x7fffffffLL;
    if (fast) ODL_DISPATCH_SRC_FMT(launch_ct_mode, mode, x, rows, cols, scale, out, out_t, amax_out, stream);
    else ODL_DISPATCH_SRC_FMT(launch_generic, x, rows, cols, scale, mode, out, out_t, amax_out, stream);
    return check_launch("odl_fp8_cast_transpose");
}

namespace odl {
__global__ void scale_inv_kernel(const float *__restrict__ scale, float *__restrict__ scale_inv_out) {
    scale_inv_out[0] = __fdiv_rn(1.0f, scale[0]);
}

template <int SRC, int FMT>
static void launch_delayed(const void *x, int64_t rows, int64_t cols, const float *scale, uint8_t *out, uint8_t *out_t,
                           float *amax_parts, float *scale_inv_out, bool fast, hipStream_t stream) {
    if (!fast) {
        // element-at-a-time route: the whole maximum goes into amax_parts[0]
        launch_generic<SRC, FMT>(x, rows, cols, scale, ODL_SCALE_TENSOR, out, out_t, amax_parts, stream);
        if (scale_inv_out) hipLaunchKernelGGL(scale_inv_kernel, dim3(1), dim3(1), 0, stream, scale, scale_inv_out);
    } else if (out_t) {
        launch_ct<SRC, FMT, ODL_SCALE_TENSOR>(x, rows, cols, scale, out, out_t, amax_parts, stream, 0, scale_inv_out, kAmaxParts - 1);
    } else {
        launch_cast<SRC, FMT, ODL_SCALE_TENSOR>(x, rows, cols, scale, out, amax_parts, stream, 0, scale_inv_out, kAmaxParts - 1);
    }
}
}  // namespace odl

extern "C" int odl_fp8_cast_delayed(const void *x, int src_dtype, int64_t rows, int64_t cols, const float *scale, int fmt,
                                    uint8_t *out, uint8_t *out_t, float *amax_parts, float *scale_inv_out, odl_stream_t stream_) {
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    if (int e = check_cast_args("odl_fp8_cast_delayed", x, src_dtype, rows, cols, scale, ODL_SCALE_TENSOR, fmt)) return e;
    if (!scale) return set_error(ODL_ERR_ARG, "odl_fp8_cast_delayed: scale is null");
    if (rows * cols == 0) {                       // nothing to cast and nothing to record: only the inverse scale
        if (scale_inv_out) hipLaunchKernelGGL(scale_inv_kernel, dim3(1), dim3(1), 0, stream, scale, scale_inv_out);
        return check_launch("odl_fp8_cast_delayed");
    }
    if (!out && !out_t) return set_error(ODL_ERR_ARG, "odl_fp8_cast_delayed: out and out_t are both null");
    const int64_t tiles = ((rows + kTileR - 1) / kTileR) * ((cols + kTileC - 1) / kTileC);
    const bool fast = out_t ? (cols % 8 == 0 && rows % 16 == 0 && aligned16(x) && aligned16(out_t) &&
                               (!out || (reinterpret_cast<uintptr_t>(out) & 7) == 0) && tiles <= 0x7fffffffLL)
                            : (cols % 16 == 0 && aligned16(x) && aligned16(out));
    ODL_DISPATCH_SRC_FMT(launch_delayed, x, rows, cols, scale, out, out_t, amax_parts, scale_inv_out, fast, stream);
    return check_launch("odl_fp8_cast_delayed");
}

namespace odl {

template <int SRC, int FMT>
static void launch_dynamic(const void *x, int64_t rows, int64_t cols, const float *parts, int margin, uint8_t *out,
                           uint8_t *out_t, float *dyn_out, bool fast, hipStream_t stream) {
    if (!fast) {
        // element-at-a-time route: scale first (one block), then the generic kernel reads it from dyn_out[1]
        hipLaunchKernelGGL((parts_to_scale_kernel<FMT>), dim3(1), dim3(kThreads), 0, stream, parts, margin, dyn_out);
        launch_generic<SRC, FMT>(x, rows, cols, dyn_out + 1, ODL_SCALE_TENSOR, out, out_t, nullptr, stream);
    } else if (out_t) {
        launch_ct<SRC, FMT, kScaleParts>(x, rows, cols, parts, out, out_t, nullptr, stream, margin, dyn_out);
    } else {
        launch_cast<SRC, FMT, kScaleParts>(x, rows, cols, parts, out, nullptr, stream, margin, dyn_out);
    }
}

}  // namespace odl

extern "C" int odl_fp8_amax_parts(const void *x, int src_dtype, int64_t rows, int64_t cols, float *parts, odl_stream_t stream_) {
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    if (rows < 0 || cols < 0) return set_error(ODL_ERR_ARG, "odl_fp8_amax_parts: negative shape %lld x %lld", (long long)rows, (long long)cols);
    if ((!x && rows * cols > 0) || !parts) return set_error(ODL_ERR_ARG, "odl_fp8_amax_parts: null pointer");
    if (src_dtype != ODL_BF16 && src_dtype != ODL_F32) return set_error(ODL_ERR_ARG, "odl_fp8_amax_parts: src_dtype %d", src_dtype);
    const int64_t n = rows * cols;
    if (n == 0 || !aligned16(x)) {
        // nothing to read, or a pointer the vector kernel cannot take: everything into parts[0]
        hipLaunchKernelGGL(fill_f32_kernel, dim3((kAmaxParts + 255) / 256), dim3(256), 0, stream, parts, (int64_t)kAmaxParts, 0.0f);
        if (n == 0) return check_launch("odl_fp8_amax_parts(fill)");
        return odl_fp8_amax(x, src_dtype, rows, cols, ODL_SCALE_TENSOR, parts, 1, stream_);
    }
    const int esz = src_dtype == ODL_BF16 ? 2 : 4;
    int64_t g = grid_for(n * esz / 16, kFatThreads * 4, 2);
    if (g > kAmaxParts) g = kAmaxParts;
    if (src_dtype == ODL_BF16) hipLaunchKernelGGL((amax_tensor_kernel<ODL_BF16, 4, 2>), dim3((unsigned)g), dim3(kFatThreads), 0, stream, x, n, parts, FusedScale{});
    else hipLaunchKernelGGL((amax_tensor_kernel<ODL_F32, 4, 2>), dim3((unsigned)g), dim3(kFatThreads), 0, stream, x, n, parts, FusedScale{});
    return check_launch("odl_fp8_amax_parts");
}

extern "C" int odl_fp8_cast_dynamic(const void *x, int src_dtype, int64_t rows, int64_t cols, const float *parts, int fmt, int margin,
                                    uint8_t *out, uint8_t *out_t, float *dyn_out, odl_stream_t stream_) {
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    if (int e = check_cast_args("odl_fp8_cast_dynamic", x, src_dtype, rows, cols, parts, ODL_SCALE_TENSOR, fmt)) return e;
    if (!parts || !dyn_out) return set_error(ODL_ERR_ARG, "odl_fp8_cast_dynamic: null pointer");
    if (rows * cols == 0) {                       // nothing to cast: only the three numbers
        if (fmt == ODL_FP8_E4M3) hipLaunchKernelGGL((parts_to_scale_kernel<ODL_FP8_E4M3>), dim3(1), dim3(kThreads), 0, stream, parts, margin, dyn_out);
        else hipLaunchKernelGGL((parts_to_scale_kernel<ODL_FP8_E5M2>), dim3(1), dim3(kThreads), 0, stream, parts, margin, dyn_out);
        return check_launch("odl_fp8_cast_dynamic(empty)");
    }
    if (!out && !out_t) return set_error(ODL_ERR_ARG, "odl_fp8_cast_dynamic: out and out_t are both null");
    bool fast;
    if (out_t) {
        const int64_t tiles = ((rows + kTileR - 1) / kTileR) * ((cols + kTileC - 1) / kTileC);
        fast = cols % 8 == 0 && rows % 16 == 0 && aligned16(x) && aligned16(out_t) && (!out || (reinterpret_cast<uintptr_t>(out) & 7) == 0) &&
               tiles <= 0x7fffffffLL && rows * cols > 0;
    } else {
        fast = cols % 16 == 0 && aligned16(x) && aligned16(out) && rows * cols > 0;
    }
    ODL_DISPATCH_SRC_FMT(launch_dynamic, x, rows, cols, parts, margin, out, out_t, dyn_out, fast, stream);
    return check_launch("odl_fp8_cast_dynamic");
}

// ------------------------------------------------ current scaling of many tensors in two launches
// All weights of a model per optimizer step: one amax launch and one cast+transpose launch instead of a pair per
// weight.  The tensors are described by a table in device memory (odl_fp8_mt_tensor); a second table lists the work
// items, (tensor, local index) pairs, one per block: the blocks of the amax pass, the 128 x 64 tiles of the cast.
// Both tables depend only on addresses and shapes, so a caller builds them once (odl_fp8_multi_plan).
namespace odl {

// blocks of the amax pass for a tensor of n16 16-byte chunks: one per 64 KB, at most one per partial maximum
__host__ __device__ inline int mt_amax_blocks(int64_t n16) {
    const int64_t nb = (n16 + 4095) / 4096;
    return nb < 1 ? 1 : (nb > kAmaxParts ? kAmaxParts : (int)nb);
}

__global__ __launch_bounds__(kFatThreads) void multi_amax_kernel(const odl_fp8_mt_tensor *__restrict__ tensors,
                                                                  const int32_t *__restrict__ work) {
    __shared__ uint32_t red[kFatThreads / kWave];
    const int32_t t = work[2 * (int64_t)blockIdx.x], b = work[2 * (int64_t)blockIdx.x + 1];
    const odl_fp8_mt_tensor e = tensors[t];
    const int64_t n16 = e.rows * e.cols / (e.src_dtype == ODL_BF16 ? 8 : 4);
    const int nb = mt_amax_blocks(n16);
    const int64_t i0 = (int64_t)b * kFatThreads + threadIdx.x, stride = (int64_t)nb * kFatThreads;
    uint32_t m = e.src_dtype == ODL_BF16 ? amax_chunks<ODL_BF16, 4>(e.x, n16, i0, stride) : amax_chunks<ODL_F32, 4>(e.x, n16, i0, stride);
    m = block_max_u32(m, red);
    if (threadIdx.x == 0) e.parts[b] = bits_to_float(m);
    if (b == 0)                                                   // entries no block owns
        for (int i = nb + threadIdx.x; i < kAmaxParts; i += kFatThreads) e.parts[i] = 0.0f;
}

template <int FMT>
__global__ __launch_bounds__(kThreads) void multi_cast_dynamic_kernel(const odl_fp8_mt_tensor *__restrict__ tensors,
                                                                       const int32_t *__restrict__ work, int margin) {
    __shared__ __attribute__((aligned(16))) uint8_t tile[kTileC * kTileR];
    __shared__ uint32_t red[kThreads / kWave];
    const int32_t t = work[2 * (int64_t)blockIdx.x], local = work[2 * (int64_t)blockIdx.x + 1];
    const odl_fp8_mt_tensor e = tensors[t];
    const float st = dynamic_scale<FMT>(e.parts, margin, e.dyn_out, red, local == 0);
    const int64_t tiles_r = (e.rows + kTileR - 1) / kTileR, tiles_c = (e.cols + kTileC - 1) / kTileC;
    int64_t tr, tc;
    ct_tile_of(tiles_r * tiles_c - 1 - local, tiles_r, tiles_c, tr, tc);
    uint32_t am = 0;
    if (e.src_dtype == ODL_BF16) ct_one_tile<ODL_BF16, FMT, kScaleParts, false, true>(e.x, e.rows, e.cols, nullptr, st, e.out, e.out_t, tr, tc, tile, am);
    else ct_one_tile<ODL_F32, FMT, kScaleParts, false, true>(e.x, e.rows, e.cols, nullptr, st, e.out, e.out_t, tr, tc, tile, am);
}

template <int FMT>
__global__ __launch_bounds__(kThreads) void multi_cast_delayed_kernel(const odl_fp8_mt_tensor *__restrict__ tensors,
                                                                       const int32_t *__restrict__ work) {
    __shared__ __attribute__((aligned(16))) uint8_t tile[kTileC * kTileR];
    __shared__ uint32_t red[kThreads / kWave];
    const int32_t t = work[2 * (int64_t)blockIdx.x], local = work[2 * (int64_t)blockIdx.x + 1];
    const odl_fp8_mt_tensor e = tensors[t];
    const float st = e.scale[0];
    if (local == 0 && threadIdx.x == 0) {
        e.dyn_out[1] = st;
        e.dyn_out[2] = __fdiv_rn(1.0f, st);
    }
    const int64_t tiles_r = (e.rows + kTileR - 1) / kTileR, tiles_c = (e.cols + kTileC - 1) / kTileC;
    int64_t tr, tc;
    ct_tile_of(tiles_r * tiles_c - 1 - local, tiles_r, tiles_c, tr, tc);
    uint32_t am = 0;
    if (e.src_dtype == ODL_BF16) {
        ct_one_tile<ODL_BF16, FMT, ODL_SCALE_TENSOR, true, true>(e.x, e.rows, e.cols, nullptr, st, e.out, e.out_t, tr, tc, tile, am);
        am = fold_u16x2_to_f32bits(am);
    } else {
        ct_one_tile<ODL_F32, FMT, ODL_SCALE_TENSOR, true, true>(e.x, e.rows, e.cols, nullptr, st, e.out, e.out_t, tr, tc, tile, am);
    }
    am = block_max_u32(am, red);
    if (threadIdx.x == 0 && am != 0) atomicMax(reinterpret_cast<uint32_t *>(e.parts) + (local & (kAmaxParts - 1)), am);
}

}  // namespace odl

extern "C" int64_t odl_fp8_multi_plan(const odl_fp8_mt_tensor *tensors, int64_t n, int phase, int32_t *work, int64_t capacity) {
    if (n < 0 || (!tensors && n > 0)) { set_error(ODL_ERR_ARG, "odl_fp8_multi_plan: bad table (n = %lld)", (long long)n); return -1; }
    if (phase != ODL_MT_AMAX && phase != ODL_MT_CAST && phase != ODL_MT_CAST_DELAYED) { set_error(ODL_ERR_ARG, "odl_fp8_multi_plan: phase %d", phase); return -1; }
    int64_t count = 0;
    for (int64_t t = 0; t < n; ++t) {
        const odl_fp8_mt_tensor &e = tensors[t];
        if (e.src_dtype != ODL_BF16 && e.src_dtype != ODL_F32) { set_error(ODL_ERR_ARG, "odl_fp8_multi_plan: tensor %lld: src_dtype %d", (long long)t, e.src_dtype); return -1; }
        if (e.rows <= 0 || e.cols <= 0 || e.rows % 16 || e.cols % 8) {
            set_error(ODL_ERR_SHAPE, "odl_fp8_multi_plan: tensor %lld is %lld x %lld; rows must be a positive multiple of 16, cols of 8", (long long)t, (long long)e.rows, (long long)e.cols);
            return -1;
        }
        if (!e.x || !e.out || !e.out_t || !e.parts || !e.dyn_out || !aligned16(e.x) || !aligned16(e.out_t) || !aligned16(e.parts) ||
            (reinterpret_cast<uintptr_t>(e.out) & 7)) {
            set_error(ODL_ERR_ARG, "odl_fp8_multi_plan: tensor %lld: null or misaligned pointer (x, out_t, parts: 16 bytes; out: 8)", (long long)t);
            return -1;
        }
        if (phase == ODL_MT_CAST_DELAYED && !e.scale) { set_error(ODL_ERR_ARG, "odl_fp8_multi_plan: tensor %lld: the delayed phase needs `scale`", (long long)t); return -1; }
        const int64_t items = phase == ODL_MT_AMAX ? mt_amax_blocks(e.rows * e.cols / (e.src_dtype == ODL_BF16 ? 8 : 4))
                                                   : ((e.rows + kTileR - 1) / kTileR) * ((e.cols + kTileC - 1) / kTileC);
        if (t > 0x7fffffffLL || items > 0x7fffffffLL) { set_error(ODL_ERR_SHAPE, "odl_fp8_multi_plan: tensor %lld is too large", (long long)t); return -1; }
        if (work && count + items <= capacity)
            for (int64_t i = 0; i < items; ++i) { work[2 * (count + i)] = (int32_t)t; work[2 * (count + i) + 1] = (int32_t)i; }
        count += items;
    }
    if (count > 0x7fffffffLL) { set_error(ODL_ERR_SHAPE, "odl_fp8_multi_plan: %lld work items exceed one launch", (long long)count); return -1; }
    return count;
}

extern "C" int odl_fp8_multi_amax_parts(const odl_fp8_mt_tensor *tensors_dev, const int32_t *work_dev, int64_t n_work, odl_stream_t stream_) {
    if (n_work < 0 || n_work > 0x7fffffffLL) return set_error(ODL_ERR_ARG, "odl_fp8_multi_amax_parts: n_work %lld", (long long)n_work);
    if (n_work == 0) return ODL_OK;
    if (!tensors_dev || !work_dev) return set_error(ODL_ERR_ARG, "odl_fp8_multi_amax_parts: null table");
    hipLaunchKernelGGL(multi_amax_kernel, dim3((unsigned)n_work), dim3(kFatThreads), 0, reinterpret_cast<hipStream_t>(stream_), tensors_dev, work_dev);
    return check_launch("odl_fp8_multi_amax_parts");
}

extern "C" int odl_fp8_multi_cast_delayed(const odl_fp8_mt_tensor *tensors_dev, const int32_t *work_dev, int64_t n_work, int fmt,
                                          odl_stream_t stream_) {
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    if (n_work < 0 || n_work > 0x7fffffffLL) return set_error(ODL_ERR_ARG, "odl_fp8_multi_cast_delayed: n_work %lld", (long long)n_work);
    if (fmt != ODL_FP8_E4M3 && fmt != ODL_FP8_E5M2) return set_error(ODL_ERR_ARG, "odl_fp8_multi_cast_delayed: fmt %d", fmt);
    if (n_work == 0) return ODL_OK;
    if (!tensors_dev || !work_dev) return set_error(ODL_ERR_ARG, "odl_fp8_multi_cast_delayed: null table");
    if (fmt == ODL_FP8_E4M3) hipLaunchKernelGGL((multi_cast_delayed_kernel<ODL_FP8_E4M3>), dim3((unsigned)n_work), dim3(kThreads), 0, stream, tensors_dev, work_dev);
    else hipLaunchKernelGGL((multi_cast_delayed_kernel<ODL_FP8_E5M2>), dim3((unsigned)n_work), dim3(kThreads), 0, stream, tensors_dev, work_dev);
    return check_launch("odl_fp8_multi_cast_delayed");
}

extern "C" int odl_fp8_multi_cast_dynamic(const odl_fp8_mt_tensor *tensors_dev, const int32_t *work_dev, int64_t n_work, int fmt, int margin,
                                          odl_stream_t stream_) {
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    if (n_work < 0 || n_work > 0x7fffffffLL) return set_error(ODL_ERR_ARG, "odl_fp8_multi_cast_dynamic: n_work %lld", (long long)n_work);
    if (fmt != ODL_FP8_E4M3 && fmt != ODL_FP8_E5M2) return set_error(ODL_ERR_ARG, "odl_fp8_multi_cast_dynamic: fmt %d", fmt);
    if (n_work == 0) return ODL_OK;
    if (!tensors_dev || !work_dev) return set_error(ODL_ERR_ARG, "odl_fp8_multi_cast_dynamic: null table");
    if (fmt == ODL_FP8_E4M3) hipLaunchKernelGGL((multi_cast_dynamic_kernel<ODL_FP8_E4M3>), dim3((unsigned)n_work), dim3(kThreads), 0, stream, tensors_dev, work_dev, margin);
    else hipLaunchKernelGGL((multi_cast_dynamic_kernel<ODL_FP8_E5M2>), dim3((unsigned)n_work), dim3(kThreads), 0, stream, tensors_dev, work_dev, margin);
    return check_launch("odl_fp8_multi_cast_dynamic");
}

// ------------------------------------------------ current scaling without a caller-side workspace
// The partial maxima that odl_fp8_amax_parts hands to odl_fp8_cast_dynamic normally live in a buffer the
// caller allocates.  Callers that cannot allocate (code under HIP graph capture, serving loops) use this
// array instead: one copy per GPU, held until the process ends.  In host code the array's NAME is only a
// handle for hipGetSymbolAddress; the address that kernels, copies and fills take is the pointer that
// call returns, looked up once per device with that device current and kept in `g_scratch_ptr`.
static __device__ __align__(256) float scratch[ODL_FP8_AMAX_PARTS];

namespace odl {

constexpr int kMaxScratchDevices = 64;
static float *g_scratch_ptr[kMaxScratchDevices] = {};

// Device address of `scratch` on the device that is current on this thread (nullptr + error text on failure).
// Two threads that resolve the same device at once store the same pointer.
float *scratch_for_current_device(const char *who) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) { set_error(ODL_ERR_LAUNCH, "%s: hipGetDevice: %s", who, hipGetErrorString(e)); return nullptr; }
    if (dev < 0 || dev >= kMaxScratchDevices) { set_error(ODL_ERR_ARG, "%s: device ordinal %d is not below %d", who, dev, kMaxScratchDevices); return nullptr; }
    float *ptr = __atomic_load_n(&g_scratch_ptr[dev], __ATOMIC_ACQUIRE);
    if (!ptr) {
        void *addr = nullptr;
        e = hipGetSymbolAddress(&addr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !addr) {
            set_error(ODL_ERR_LAUNCH, "%s: hipGetSymbolAddress(scratch) on device %d: %s", who, dev, hipGetErrorString(e));
            return nullptr;
        }
        ptr = static_cast<float *>(addr);
        __atomic_store_n(&g_scratch_ptr[dev], ptr, __ATOMIC_RELEASE);
    }
    return ptr;
}

}  // namespace odl

extern "C" int odl_fp8_cast_dynamic_noalloc(const void *x, int src_dtype, int64_t rows, int64_t cols, int fmt, int margin,
                                            uint8_t *out, uint8_t *out_t, float *dyn_out, odl_stream_t stream_) {
    if (int e = check_cast_args("odl_fp8_cast_dynamic_noalloc", x, src_dtype, rows, cols, reinterpret_cast<const float *>(x), ODL_SCALE_TENSOR, fmt)) return e;
    if (!dyn_out) return set_error(ODL_ERR_ARG, "odl_fp8_cast_dynamic_noalloc: dyn_out is null");
    if (rows * cols > 0 && !out && !out_t) return set_error(ODL_ERR_ARG, "odl_fp8_cast_dynamic_noalloc: out and out_t are both null");
    // rows, cols >= 0 here; the product is formed in floating point so that it cannot wrap
    if ((double)rows * (double)cols > (double)ODL_FP8_NOALLOC_MAX_ELEMS)
        return set_error(ODL_ERR_SHAPE, "odl_fp8_cast_dynamic_noalloc: %lld x %lld elements exceed the limit of %lld of the entry point that "
                         "allocates nothing; use odl_fp8_amax_parts + odl_fp8_cast_dynamic with a workspace of your own",
                         (long long)rows, (long long)cols, (long long)ODL_FP8_NOALLOC_MAX_ELEMS);
    float *parts = scratch_for_current_device("odl_fp8_cast_dynamic_noalloc");
    if (!parts) return ODL_ERR_LAUNCH;
    // the amax pass writes all ODL_FP8_AMAX_PARTS entries (unused ones as 0), so what the last call left is overwritten
    if (int e = odl_fp8_amax_parts(x, src_dtype, rows, cols, parts, stream_)) return e;
    return odl_fp8_cast_dynamic(x, src_dtype, rows, cols, parts, fmt, margin, out, out_t, dyn_out, stream_);
}

// ------------------------------------------------------------------ rowwise recipe, fused passes
static bool rowcol_fast(const void *x, int64_t rows, int64_t cols) {
    return rows > 0 && cols > 0 && aligned16(x) && cols % 8 == 0 && rows % 16 == 0;
}

extern "C" int odl_fp8_amax_rowcol(const void *x, int src_dtype, int64_t rows, int64_t cols, float *amax_row, float *amax_col,
                                   odl_stream_t stream_) {
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    if (rows < 0 || cols < 0) return set_error(ODL_ERR_ARG, "odl_fp8_amax_rowcol: negative shape");
    if ((!x && rows * cols > 0) || (!amax_row && rows > 0) || (!amax_col && cols > 0)) return set_error(ODL_ERR_ARG, "odl_fp8_amax_rowcol: null pointer");
    if (src_dtype != ODL_BF16 && src_dtype != ODL_F32) return set_error(ODL_ERR_ARG, "odl_fp8_amax_rowcol: src_dtype %d", src_dtype);
    if (!rowcol_fast(x, rows, cols)) {
        int rc = odl_fp8_amax(x, src_dtype, rows, cols, ODL_SCALE_ROW, amax_row, 0, stream_);
        if (rc != ODL_OK) return rc;
        return odl_fp8_amax(x, src_dtype, rows, cols, ODL_SCALE_COL, amax_col, 0, stream_);
    }
    hipLaunchKernelGGL(fill_f32_kernel, dim3((unsigned)((rows + 255) / 256)), dim3(256), 0, stream, amax_row, rows, 0.0f);
    hipLaunchKernelGGL(fill_f32_kernel, dim3((unsigned)((cols + 255) / 256)), dim3(256), 0, stream, amax_col, cols, 0.0f);
    const int esz = src_dtype == ODL_BF16 ? 2 : 4;
    const int cw = 32 * (16 / esz);
    const int64_t col_blocks = (cols + cw - 1) / cw;
    int64_t want_slabs = ((int64_t)num_cus() * 8 + col_blocks - 1) / col_blocks;
    int64_t rpb = (rows + want_slabs - 1) / want_slabs;
    rpb = ((rpb + 31) / 32) * 32;
    if (rpb < 64) rpb = 64;
    const int64_t slabs = (rows + rpb - 1) / rpb;
    if (slabs > 65535) return set_error(ODL_ERR_SHAPE, "odl_fp8_amax_rowcol: too many row slabs");
    if (src_dtype == ODL_BF16) hipLaunchKernelGGL((amax_rowcol_kernel<ODL_BF16>), dim3((unsigned)col_blocks, (unsigned)slabs), dim3(kThreads), 0, stream, x, rows, cols, (int)rpb, amax_row, amax_col);
    else hipLaunchKernelGGL((amax_rowcol_kernel<ODL_F32>), dim3((unsigned)col_blocks, (unsigned)slabs), dim3(kThreads), 0, stream, x, rows, cols, (int)rpb, amax_row, amax_col);
    return check_launch("odl_fp8_amax_rowcol");
}

template <int SRC, int FMT>
static void launch_rowcol(const void *x, int64_t rows, int64_t cols, const float *amax_row, const float *amax_col, int margin,
                          uint8_t *out, uint8_t *out_t, float *s_row, float *s_row_inv, float *s_col, float *s_col_inv, hipStream_t stream) {
    const int64_t g = ((rows + kTileR - 1) / kTileR) * ((cols + kTileC - 1) / kTileC);
    hipLaunchKernelGGL((cast_rowcol_kernel<SRC, FMT>), dim3((unsigned)g), dim3(kThreads), 0, stream, x, rows, cols, amax_row, amax_col,
                       margin, out, out_t, s_row, s_row_inv, s_col, s_col_inv);
}

extern "C" int odl_fp8_cast_rowcol(const void *x, int src_dtype, int64_t rows, int64_t cols, const float *amax_row,
                                   const float *amax_col, int fmt, int margin, uint8_t *out, uint8_t *out_t, float *s_row,
                                   float *s_row_inv, float *s_col, float *s_col_inv, odl_stream_t stream_) {
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    if (rows < 0 || cols < 0) return set_error(ODL_ERR_ARG, "odl_fp8_cast_rowcol: negative shape");
    if (src_dtype != ODL_BF16 && src_dtype != ODL_F32) return set_error(ODL_ERR_ARG, "odl_fp8_cast_rowcol: src_dtype %d", src_dtype);
    if (fmt != ODL_FP8_E4M3 && fmt != ODL_FP8_E5M2) return set_error(ODL_ERR_ARG, "odl_fp8_cast_rowcol: fmt %d", fmt);
    if ((rows > 0 && (!amax_row || !s_row || !s_row_inv)) || (cols > 0 && (!amax_col || !s_col || !s_col_inv)))
        return set_error(ODL_ERR_ARG, "odl_fp8_cast_rowcol: null scale pointer");
    if (rows * cols > 0 && (!x || !out || !out_t)) return set_error(ODL_ERR_ARG, "odl_fp8_cast_rowcol: null pointer");
    const int64_t tiles = ((rows + kTileR - 1) / kTileR) * ((cols + kTileC - 1) / kTileC);
    const bool fast = rowcol_fast(x, rows, cols) && aligned16(out_t) && (reinterpret_cast<uintptr_t>(out) & 7) == 0 && tiles <= 0x7fffffffLL;
    if (!fast) {
        // the step-by-step route: scales first, then the two casts
        int rc = odl_fp8_scale_from_amax(amax_row, rows, fmt, margin, s_row, s_row_inv, stream_);
        if (rc == ODL_OK) rc = odl_fp8_scale_from_amax(amax_col, cols, fmt, margin, s_col, s_col_inv, stream_);
        if (rc == ODL_OK && rows * cols > 0) rc = odl_fp8_cast(x, src_dtype, rows, cols, s_row, ODL_SCALE_ROW, fmt, out, nullptr, stream_);
        if (rc == ODL_OK && rows * cols > 0) rc = odl_fp8_cast_transpose(x, src_dtype, rows, cols, s_col, ODL_SCALE_COL, fmt, nullptr, out_t, nullptr, stream_);
        return rc;
    }
    ODL_DISPATCH_SRC_FMT(launch_rowcol, x, rows, cols, amax_row, amax_col, margin, out, out_t, s_row, s_row_inv, s_col, s_col_inv, stream);
    return check_launch("odl_fp8_cast_rowcol");
}
