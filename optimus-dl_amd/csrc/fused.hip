// Producers of FP8 Linear inputs that also deliver the partial maxima of what they write, so
// that the current-scaling quantisation of their output needs no amax pass of its own:
//   SwiGLU forward    h  = silu(gate) * up                        (input of the down projection)
//   SwiGLU backward   d_gate, d_up from d_h                        (grad_outputs of gate / up)
//   RMSNorm forward   y  = x * rsqrt(mean(x^2) + eps) * weight     (input of q/k/v, gate/up)
// plus the RMSNorm backward and the amax pass that also yields the bias gradient (column sums).
// All are bound by HBM bandwidth.  Elementwise results and per-row reductions are written so that
// a plain-C restatement gives the same bits: fused multiply-adds are spelled out, nothing is left
// to contraction, no hardware approximation (v_exp_f32, v_rcp_f32, v_rsq_f32) is used.  Sums over
// rows (d_weight, column sums) are fp32 partial sums in a fixed order.
#include "common.h"

#pragma clang fp contract(off)

namespace odl {

constexpr int kFusedThreads = 1024;
constexpr int kParts = ODL_FP8_AMAX_PARTS;

// 1 / d for 1 <= d < 2^120: integer first guess, three Newton steps in fused multiply-adds.
__device__ __forceinline__ float recip_newton(float d) {
    float y = bits_to_float(0x7EF311C7u - float_to_bits(d));
    y = __fmaf_rn(y, __fmaf_rn(-d, y, 1.0f), y);
    y = __fmaf_rn(y, __fmaf_rn(-d, y, 1.0f), y);
    y = __fmaf_rn(y, __fmaf_rn(-d, y, 1.0f), y);
    return y;
}

// logistic function 1 / (1 + exp(-g)): range reduction by ln 2 in two pieces, degree-5 polynomial
// for (exp(r) - 1 - r) / r^2, exact scaling by 2^k, reciprocal as above.  A NaN argument is
// evaluated as 0 here (every use below multiplies by the argument again, which restores the NaN).
__device__ __forceinline__ float sigmoid_det(float g) {
    float t = (g != g) ? 0.0f : -g;
    const bool zero = t > 80.0f;                 // exp(-g) beyond 2^115: the quotient is taken as 0
    t = __builtin_amdgcn_fmed3f(t, -80.0f, 80.0f);
    const float kf = __builtin_rintf(__fmul_rn(t, 1.44269504f));
    float r = __fmaf_rn(kf, -0.693359375f, t);
    r = __fmaf_rn(kf, 2.12194440e-4f, r);
    float p = 1.9875691500e-4f;
    p = __fmaf_rn(p, r, 1.3981999507e-3f);
    p = __fmaf_rn(p, r, 8.3334519073e-3f);
    p = __fmaf_rn(p, r, 4.1665795894e-2f);
    p = __fmaf_rn(p, r, 1.6666665459e-1f);
    p = __fmaf_rn(p, r, 5.0000001201e-1f);
    const float z = __fmul_rn(r, r);
    const float y = __fadd_rn(__fmaf_rn(p, z, r), 1.0f);
    const float e = __fmul_rn(y, bits_to_float((uint32_t)((int)kf + 127) << 23));
    const float s = recip_newton(__fadd_rn(1.0f, e));
    return zero ? 0.0f : s;
}

// Roundings to bf16 use the hardware's round-to-nearest-even conversion of a pair (subnormal
// results are kept: the kernels run with fp32 denormals enabled).

// h = bf16( bf16(g * sigmoid(g)) * u ), the two roundings of silu(gate) * up evaluated in bf16, for
// the two elements of a packed pair
__device__ __forceinline__ uint32_t swiglu_fwd_pair(uint32_t gw, uint32_t uw) {
    const float g0 = bf16_lo(gw), g1 = bf16_hi(gw);
    const uint32_t s = pack_bf16x2(__fmul_rn(g0, sigmoid_det(g0)), __fmul_rn(g1, sigmoid_det(g1)));
    return pack_bf16x2(__fmul_rn(bf16_lo(s), bf16_lo(uw)), __fmul_rn(bf16_hi(s), bf16_hi(uw)));
}

// d_up = bf16(dh * s), d_gate = bf16( bf16(dh * u) * (sig * (1 + g * (1 - sig))) ), s = bf16(g * sig)
__device__ __forceinline__ void swiglu_bwd_pair(uint32_t dw, uint32_t gw, uint32_t uw, uint32_t &dg, uint32_t &du) {
    const float g0 = bf16_lo(gw), g1 = bf16_hi(gw), d0 = bf16_lo(dw), d1 = bf16_hi(dw);
    const float sig0 = sigmoid_det(g0), sig1 = sigmoid_det(g1);
    const uint32_t s = pack_bf16x2(__fmul_rn(g0, sig0), __fmul_rn(g1, sig1));
    du = pack_bf16x2(__fmul_rn(d0, bf16_lo(s)), __fmul_rn(d1, bf16_hi(s)));
    const uint32_t ds = pack_bf16x2(__fmul_rn(d0, bf16_lo(uw)), __fmul_rn(d1, bf16_hi(uw)));
    const float ds0 = __fmul_rn(sig0, __fmaf_rn(g0, __fsub_rn(1.0f, sig0), 1.0f));
    const float ds1 = __fmul_rn(sig1, __fmaf_rn(g1, __fsub_rn(1.0f, sig1), 1.0f));
    dg = pack_bf16x2(__fmul_rn(bf16_lo(ds), ds0), __fmul_rn(bf16_hi(ds), ds1));
}

__device__ __forceinline__ uint32_t pack2(float a, float b) { return pack_bf16x2(a, b); }

// ------------------------------------------------------------------ SwiGLU forward
// n8 chunks of 8 bf16 (16 bytes) per operand; two chunks per lane in flight.  parts[blockIdx] =
// this block's max |h|; entries no block owns are zeroed by block 0.
__global__ __launch_bounds__(kFusedThreads) void swiglu_fwd_kernel(const u32x4 *__restrict__ gate, const u32x4 *__restrict__ up,
                                                                    int64_t n8, u32x4 *__restrict__ h, float *__restrict__ parts) {
    __shared__ uint32_t red[kFusedThreads / kWave];
    const int64_t stride = (int64_t)gridDim.x * kFusedThreads;
    uint32_t am = 0;
    auto one = [&](const u32x4 gv, const u32x4 uv) -> u32x4 {
        const uint32_t gw[4] = {gv.x, gv.y, gv.z, gv.w}, uw[4] = {uv.x, uv.y, uv.z, uv.w};
        uint32_t o[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            o[q] = swiglu_fwd_pair(gw[q], uw[q]);
            am = max_u16x2(am, abs_bf16x2(o[q]));
        }
        return u32x4{o[0], o[1], o[2], o[3]};
    };
    int64_t i = (int64_t)blockIdx.x * kFusedThreads + threadIdx.x;
    for (; i + stride < n8; i += 2 * stride) {
        const u32x4 g0 = __builtin_nontemporal_load(gate + i), u0 = __builtin_nontemporal_load(up + i);
        const u32x4 g1 = __builtin_nontemporal_load(gate + i + stride), u1 = __builtin_nontemporal_load(up + i + stride);
        h[i] = one(g0, u0);
        h[i + stride] = one(g1, u1);
    }
    for (; i < n8; i += stride) h[i] = one(__builtin_nontemporal_load(gate + i), __builtin_nontemporal_load(up + i));
    am = block_max_u32(fold_u16x2_to_f32bits(am), red);
    if (threadIdx.x == 0) parts[blockIdx.x] = bits_to_float(am);
    if (blockIdx.x == 0)
        for (int j = (int)gridDim.x + threadIdx.x; j < kParts; j += kFusedThreads) parts[j] = 0.0f;
}

// ----------------------------------------------------------------- SwiGLU backward
__global__ __launch_bounds__(kFusedThreads) void swiglu_bwd_kernel(const u32x4 *__restrict__ dh, const u32x4 *__restrict__ gate,
                                                                    const u32x4 *__restrict__ up, int64_t n8,
                                                                    u32x4 *__restrict__ dgate, u32x4 *__restrict__ dup,
                                                                    float *__restrict__ parts_dg, float *__restrict__ parts_du) {
    __shared__ uint32_t red[kFusedThreads / kWave];
    const int64_t stride = (int64_t)gridDim.x * kFusedThreads;
    uint32_t am_g = 0, am_u = 0;
    for (int64_t i = (int64_t)blockIdx.x * kFusedThreads + threadIdx.x; i < n8; i += stride) {
        const u32x4 dv = __builtin_nontemporal_load(dh + i), gv = __builtin_nontemporal_load(gate + i),
                    uv = __builtin_nontemporal_load(up + i);
        const uint32_t dw[4] = {dv.x, dv.y, dv.z, dv.w}, gw[4] = {gv.x, gv.y, gv.z, gv.w}, uw[4] = {uv.x, uv.y, uv.z, uv.w};
        uint32_t og[4], ou[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            swiglu_bwd_pair(dw[q], gw[q], uw[q], og[q], ou[q]);
            am_g = max_u16x2(am_g, abs_bf16x2(og[q]));
            am_u = max_u16x2(am_u, abs_bf16x2(ou[q]));
        }
        dgate[i] = u32x4{og[0], og[1], og[2], og[3]};
        dup[i] = u32x4{ou[0], ou[1], ou[2], ou[3]};
    }
    am_g = block_max_u32(fold_u16x2_to_f32bits(am_g), red);
    __syncthreads();                               // red is reused
    am_u = block_max_u32(fold_u16x2_to_f32bits(am_u), red);
    if (threadIdx.x == 0) {
        parts_dg[blockIdx.x] = bits_to_float(am_g);
        parts_du[blockIdx.x] = bits_to_float(am_u);
    }
    if (blockIdx.x == 0)
        for (int j = (int)gridDim.x + threadIdx.x; j < kParts; j += kFusedThreads) { parts_dg[j] = 0.0f; parts_du[j] = 0.0f; }
}

// ------------------------------------------------------------------- RMSNorm forward
// One wavefront per row, rows handed out round-robin over all waves of the grid.  A lane holds
// CPL chunks of 8 elements (chunk index = lane + 64 * j), so the row is read once.  Sum of
// squares: per lane in element order by fused multiply-add, then the xor butterfly 32,16,..,1
// (a + b is commutative, so every lane ends with the same bits).
//   rstd = 1 / sqrt(sum / cols + eps)      (IEEE sqrt and division)
//   y    = bf16( (x * rstd) * weight )     (two fp32 products, one rounding)
// Rows up to 64 * 8 * 8 elements keep a lane's share in few registers and run in fat blocks (one
// row per wave and trip, many rows in flight per CU); wider rows use 256-lane blocks.

template <int SRC>
__device__ __forceinline__ void unpack8(const u32x4 *raw, float f[8]) {
    if constexpr (SRC == ODL_BF16) {
        const uint32_t w[4] = {raw[0].x, raw[0].y, raw[0].z, raw[0].w};
#pragma unroll
        for (int q = 0; q < 4; ++q) { f[2 * q] = bf16_lo(w[q]); f[2 * q + 1] = bf16_hi(w[q]); }
    } else {
        f[0] = bits_to_float(raw[0].x); f[1] = bits_to_float(raw[0].y); f[2] = bits_to_float(raw[0].z); f[3] = bits_to_float(raw[0].w);
        f[4] = bits_to_float(raw[1].x); f[5] = bits_to_float(raw[1].y); f[6] = bits_to_float(raw[1].z); f[7] = bits_to_float(raw[1].w);
    }
}

template <int SRC, int CPL, int kRmsThreads>
__global__ __launch_bounds__(kRmsThreads) void rmsnorm_fwd_kernel(const void *__restrict__ x, const float *__restrict__ weight,
                                                                   int64_t rows, int64_t cols, float eps,
                                                                   uint16_t *__restrict__ y, float *__restrict__ rstd_out,
                                                                   float *__restrict__ parts) {
    __shared__ uint32_t red[kRmsThreads / kWave];
    constexpr int VPC = SRC == ODL_BF16 ? 1 : 2;            // 16-byte vectors per chunk of 8 elements
    // Short rows: a wave takes RB consecutive rows per trip, so that as many loads are in flight per lane as for a long
    // row and the RB reductions (a chain of dependent cross-lane steps and two divisions each) overlap one another.
    constexpr int RB = CPL <= 2 ? 4 : (CPL <= 4 ? 2 : 1);
    const int lane = threadIdx.x % kWave;
    const int64_t wave = (int64_t)blockIdx.x * (kRmsThreads / kWave) + threadIdx.x / kWave;
    const int64_t nwave = (int64_t)gridDim.x * (kRmsThreads / kWave);
    const int64_t nchunk = cols / 8;
    uint32_t am = 0;
    for (int64_t row0 = wave * RB; row0 < rows; row0 += nwave * RB) {
        u32x4 raw[RB][CPL][VPC];
#pragma unroll
        for (int b = 0; b < RB; ++b)
#pragma unroll
            for (int j = 0; j < CPL; ++j) {
                const int64_t c = lane + (int64_t)kWave * j;
                const u32x4 *p = reinterpret_cast<const u32x4 *>(x) + ((row0 + b) * nchunk + c) * VPC;
#pragma unroll
                for (int h = 0; h < VPC; ++h) raw[b][j][h] = (c < nchunk && row0 + b < rows) ? __builtin_nontemporal_load(p + h) : u32x4{0, 0, 0, 0};
            }
        float acc[RB], rstd[RB];
#pragma unroll
        for (int b = 0; b < RB; ++b) {
            acc[b] = 0.0f;
#pragma unroll
            for (int j = 0; j < CPL; ++j) {
                float f[8];
                unpack8<SRC>(raw[b][j], f);
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[b] = __fmaf_rn(f[e], f[e], acc[b]);
            }
        }
#pragma unroll
        for (int off = kWave / 2; off > 0; off >>= 1)
#pragma unroll
            for (int b = 0; b < RB; ++b) acc[b] = __fadd_rn(acc[b], __shfl_xor(acc[b], off, kWave));
#pragma unroll
        for (int b = 0; b < RB; ++b) {
            const float mean = __fdiv_rn(acc[b], (float)cols);
            rstd[b] = __fdiv_rn(1.0f, __builtin_sqrtf(__fadd_rn(mean, eps)));
            if (lane == 0 && row0 + b < rows) rstd_out[row0 + b] = rstd[b];
        }
#pragma unroll
        for (int j = 0; j < CPL; ++j) {
            const int64_t c = lane + (int64_t)kWave * j;
            if (c < nchunk) {
                const float4 w0 = *reinterpret_cast<const float4 *>(weight + c * 8), w1 = *reinterpret_cast<const float4 *>(weight + c * 8 + 4);
                const float w[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
#pragma unroll
                for (int b = 0; b < RB; ++b) {
                    if (row0 + b < rows) {
                        float f[8];
                        unpack8<SRC>(raw[b][j], f);
                        uint32_t o[4];
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            o[q] = pack2(__fmul_rn(__fmul_rn(f[2 * q], rstd[b]), w[2 * q]), __fmul_rn(__fmul_rn(f[2 * q + 1], rstd[b]), w[2 * q + 1]));
                            am = max_u16x2(am, abs_bf16x2(o[q]));
                        }
                        reinterpret_cast<u32x4 *>(y)[(row0 + b) * nchunk + c] = u32x4{o[0], o[1], o[2], o[3]};
                    }
                }
            }
        }
    }
    am = block_max_u32(fold_u16x2_to_f32bits(am), red);
    if (threadIdx.x == 0) parts[blockIdx.x] = bits_to_float(am);
    if (blockIdx.x == 0)
        for (int j = (int)gridDim.x + threadIdx.x; j < kParts; j += kRmsThreads) parts[j] = 0.0f;
}

// Rows of at most 256 elements (per-head q / k norms): LPR <= 32 lanes hold a row, a wave works on 64 / LPR rows
// per trip.  The row sum is the same per-lane fma chain and the xor butterfly over the row's lanes; the steps
// 32 .. LPR of the full butterfly would add exact zeros, so rstd and y are the same bits as from the kernel above.
template <int SRC, int LPR>
__global__ __launch_bounds__(kFusedThreads) void rmsnorm_fwd_narrow_kernel(const void *__restrict__ x, const float *__restrict__ weight,
                                                                            int64_t rows, int64_t cols, float eps,
                                                                            uint16_t *__restrict__ y, float *__restrict__ rstd_out,
                                                                            float *__restrict__ parts) {
    __shared__ uint32_t red[kFusedThreads / kWave];
    constexpr int VPC = SRC == ODL_BF16 ? 1 : 2, RPW = kWave / LPR;
    const int lane = threadIdx.x % kWave, c = lane % LPR;
    const int64_t wave = (int64_t)blockIdx.x * (kFusedThreads / kWave) + threadIdx.x / kWave;
    const int64_t nwave = (int64_t)gridDim.x * (kFusedThreads / kWave);
    const int64_t nchunk = cols / 8;
    const bool ok = c < nchunk;
    float w[8];
    {
        const float4 w0 = ok ? *reinterpret_cast<const float4 *>(weight + c * 8) : float4{0, 0, 0, 0};
        const float4 w1 = ok ? *reinterpret_cast<const float4 *>(weight + c * 8 + 4) : float4{0, 0, 0, 0};
        w[0] = w0.x; w[1] = w0.y; w[2] = w0.z; w[3] = w0.w; w[4] = w1.x; w[5] = w1.y; w[6] = w1.z; w[7] = w1.w;
    }
    uint32_t am = 0;
    for (int64_t row0 = wave * RPW; row0 < rows; row0 += nwave * RPW) {      // uniform per wave: every lane shuffles
        const int64_t row = row0 + lane / LPR;
        const bool live = ok && row < rows;
        u32x4 raw[VPC];
        const u32x4 *p = reinterpret_cast<const u32x4 *>(x) + (row * nchunk + c) * VPC;
#pragma unroll
        for (int h = 0; h < VPC; ++h) raw[h] = live ? __builtin_nontemporal_load(p + h) : u32x4{0, 0, 0, 0};
        float f[8];
        unpack8<SRC>(raw, f);
        float acc = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) acc = __fmaf_rn(f[e], f[e], acc);
#pragma unroll
        for (int off = LPR / 2; off > 0; off >>= 1) acc = __fadd_rn(acc, __shfl_xor(acc, off, kWave));
        const float mean = __fdiv_rn(acc, (float)cols);
        const float rstd = __fdiv_rn(1.0f, __builtin_sqrtf(__fadd_rn(mean, eps)));
        if (c == 0 && row < rows) rstd_out[row] = rstd;
        if (live) {
            uint32_t o[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                o[q] = pack2(__fmul_rn(__fmul_rn(f[2 * q], rstd), w[2 * q]), __fmul_rn(__fmul_rn(f[2 * q + 1], rstd), w[2 * q + 1]));
                am = max_u16x2(am, abs_bf16x2(o[q]));
            }
            reinterpret_cast<u32x4 *>(y)[row * nchunk + c] = u32x4{o[0], o[1], o[2], o[3]};
        }
    }
    am = block_max_u32(fold_u16x2_to_f32bits(am), red);
    if (threadIdx.x == 0) parts[blockIdx.x] = bits_to_float(am);
    if (blockIdx.x == 0)
        for (int j = (int)gridDim.x + threadIdx.x; j < kParts; j += kFusedThreads) parts[j] = 0.0f;
}

__device__ __forceinline__ float wave_sum_butterfly(float acc) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) acc = __fadd_rn(acc, __shfl_xor(acc, off, kWave));
    return acc;
}

// the same butterfly on N independent values, step by step across all of them (the N chains overlap)
template <int N>
__device__ __forceinline__ void wave_sum_butterfly_n(float (&acc)[N]) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1)
#pragma unroll
        for (int b = 0; b < N; ++b) acc[b] = __fadd_rn(acc[b], __shfl_xor(acc[b], off, kWave));
}

// ------------------------------------------------------- RMSNorm / LayerNorm backward
// One BLOCK of four waves per row, rows dealt round-robin to the blocks; the next row's loads are in
// flight while the current one is worked on.  The 8-element chunk c of a row belongs to wave
// (c / 64) % 4, lane c % 64, slot c / 256, so a lane owns the same columns in every row: the weights
// of those columns stay in registers and d_weight / d_bias are plain per-lane sums over the rows of
// the block (no reduction inside the block), written as one slab per block and added up over the
// blocks by rmsnorm_bwd_reduce_kernel.
//   xh = (x - mean) * rstd   (RMSNorm: x * rstd),   t = dy * weight
//   row sums  S1 = sum t (LayerNorm only), S2 = sum t * xh: per lane over its slots in ascending order and
//   the elements of a chunk in order (t * xh by fma), xor butterfly 32..1 inside the wave, then the four
//   wave sums as ((s0 + s1) + s2) + s3;  c1 = S1 / cols, c2 = S2 / cols
//   dx = rstd * fma(-xh, c2, t - c1)   (RMSNorm: rstd * fma(-xh, c2, t)), rounded once to the dtype of x.
constexpr int kRmsBwdThreads = 256;

template <int SRC, bool LN, int CPLW>
__global__ __launch_bounds__(kRmsBwdThreads) void norm_bwd_kernel(const u32x4 *__restrict__ dy, const void *__restrict__ x,
                                                                   const float *__restrict__ weight, const float *__restrict__ mean_in,
                                                                   const float *__restrict__ rstd_in, int64_t rows, int64_t cols,
                                                                   void *__restrict__ dx, float *__restrict__ slabs) {
    __shared__ float rsum[2][2][kRmsBwdThreads / kWave];
    constexpr int VPC = SRC == ODL_BF16 ? 1 : 2;
    constexpr int NS = LN ? 2 : 1;                            // accumulator sets per lane (d_weight, d_bias)
    const int lane = threadIdx.x % kWave, wv = threadIdx.x / kWave;
    const int64_t nchunk = cols / 8;
    int64_t chunk[CPLW];
    float wreg[CPLW][8], dw[CPLW][8], db[LN ? CPLW : 1][8];
#pragma unroll
    for (int j = 0; j < CPLW; ++j) {
        chunk[j] = (int64_t)(j * 4 + wv) * kWave + lane;
        const bool ok = chunk[j] < nchunk;
        const float4 w0 = ok ? *reinterpret_cast<const float4 *>(weight + chunk[j] * 8) : float4{0, 0, 0, 0};
        const float4 w1 = ok ? *reinterpret_cast<const float4 *>(weight + chunk[j] * 8 + 4) : float4{0, 0, 0, 0};
        wreg[j][0] = w0.x; wreg[j][1] = w0.y; wreg[j][2] = w0.z; wreg[j][3] = w0.w;
        wreg[j][4] = w1.x; wreg[j][5] = w1.y; wreg[j][6] = w1.z; wreg[j][7] = w1.w;
#pragma unroll
        for (int e = 0; e < 8; ++e) { dw[j][e] = 0.0f; if constexpr (LN) db[j][e] = 0.0f; }
    }
    // Two rows are in flight beside the one being worked on (PF register sets, used in turn): a block spends about one
    // memory latency per row whatever it computes, so what is in flight per compute unit sets the rate
    // (LayerNorm, 8192 x 4096, one row in flight: 44.2 us).
    constexpr int PF = CPLW <= 2 ? 2 : 1;
    u32x4 nx[PF][CPLW][VPC], nd[PF][CPLW];
    auto fetch = [&](int s, int64_t row) {
#pragma unroll
        for (int j = 0; j < CPLW; ++j) {
            const bool ok = chunk[j] < nchunk && row < rows;
            const u32x4 *p = reinterpret_cast<const u32x4 *>(x) + (row * nchunk + chunk[j]) * VPC;
#pragma unroll
            for (int h = 0; h < VPC; ++h) nx[s][j][h] = ok ? __builtin_nontemporal_load(p + h) : u32x4{0, 0, 0, 0};
            nd[s][j] = ok ? __builtin_nontemporal_load(dy + row * nchunk + chunk[j]) : u32x4{0, 0, 0, 0};
        }
    };
#pragma unroll
    for (int s = 0; s < PF; ++s) fetch(s, blockIdx.x + (int64_t)s * gridDim.x);
    auto one_row = [&](int s, int64_t row, int par) {
        u32x4 xr[CPLW][VPC], dr[CPLW];
#pragma unroll
        for (int j = 0; j < CPLW; ++j) {
#pragma unroll
            for (int h = 0; h < VPC; ++h) xr[j][h] = nx[s][j][h];
            dr[j] = nd[s][j];
        }
        fetch(s, row + (int64_t)PF * gridDim.x);              // rows past the end load nothing
        const float rstd = rstd_in[row];
        const float mean = LN ? mean_in[row] : 0.0f;
        float a1 = 0.0f, a2 = 0.0f;
#pragma unroll
        for (int j = 0; j < CPLW; ++j) {
            if (chunk[j] < nchunk) {
                float xf[8], df[8];
                unpack8<SRC>(xr[j], xf);
                unpack8<ODL_BF16>(&dr[j], df);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float xh = LN ? __fmul_rn(__fsub_rn(xf[e], mean), rstd) : __fmul_rn(xf[e], rstd);
                    const float t = __fmul_rn(df[e], wreg[j][e]);
                    if constexpr (LN) a1 = __fadd_rn(a1, t);
                    a2 = __fmaf_rn(t, xh, a2);
                    dw[j][e] = __fmaf_rn(df[e], xh, dw[j][e]);
                    if constexpr (LN) db[j][e] = __fadd_rn(db[j][e], df[e]);
                }
            }
        }
        if constexpr (LN) {
            float both[2] = {a1, a2};                         // the two chains side by side; each is the butterfly it was
            wave_sum_butterfly_n<2>(both);
            a1 = both[0]; a2 = both[1];
        } else {
            a2 = wave_sum_butterfly(a2);
        }
        if (lane == 0) { rsum[par][1][wv] = a2; if constexpr (LN) rsum[par][0][wv] = a1; }
        __syncthreads();
        const float c2 = __fdiv_rn(__fadd_rn(__fadd_rn(__fadd_rn(rsum[par][1][0], rsum[par][1][1]), rsum[par][1][2]), rsum[par][1][3]), (float)cols);
        float c1 = 0.0f;
        if constexpr (LN) c1 = __fdiv_rn(__fadd_rn(__fadd_rn(__fadd_rn(rsum[par][0][0], rsum[par][0][1]), rsum[par][0][2]), rsum[par][0][3]), (float)cols);
#pragma unroll
        for (int j = 0; j < CPLW; ++j) {
            if (chunk[j] < nchunk) {
                float xf[8], df[8], o[8];
                unpack8<SRC>(xr[j], xf);
                unpack8<ODL_BF16>(&dr[j], df);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float xh = LN ? __fmul_rn(__fsub_rn(xf[e], mean), rstd) : __fmul_rn(xf[e], rstd);
                    const float t = __fmul_rn(df[e], wreg[j][e]);
                    o[e] = __fmul_rn(rstd, __fmaf_rn(-xh, c2, LN ? __fsub_rn(t, c1) : t));
                }
                if constexpr (SRC == ODL_BF16) {
                    reinterpret_cast<u32x4 *>(dx)[row * nchunk + chunk[j]] =
                        u32x4{pack2(o[0], o[1]), pack2(o[2], o[3]), pack2(o[4], o[5]), pack2(o[6], o[7])};
                } else {
                    float4 *q = reinterpret_cast<float4 *>(dx) + (row * nchunk + chunk[j]) * 2;
                    q[0] = float4{o[0], o[1], o[2], o[3]};
                    q[1] = float4{o[4], o[5], o[6], o[7]};
                }
            }
        }
    };
    // (the row is the same for the whole block, so every lane meets the barrier inside one_row or none does; rsum is used
    // in turn: a lane may still read the sums of row i while another writes those of row i + 1)
    for (int64_t row = blockIdx.x; row < rows; row += (int64_t)PF * gridDim.x) {
#pragma unroll
        for (int s = 0; s < PF; ++s)
            if (row + (int64_t)s * gridDim.x < rows) one_row(s, row + (int64_t)s * gridDim.x, PF == 1 ? (int)((row / gridDim.x) & 1) : s);
    }
    // every lane owns its columns: the block's slab needs no reduction
    float *slab = slabs + (int64_t)blockIdx.x * NS * cols;
#pragma unroll
    for (int j = 0; j < CPLW; ++j) {
        if (chunk[j] < nchunk) {
            float4 *q = reinterpret_cast<float4 *>(slab + chunk[j] * 8);
            q[0] = float4{dw[j][0], dw[j][1], dw[j][2], dw[j][3]};
            q[1] = float4{dw[j][4], dw[j][5], dw[j][6], dw[j][7]};
            if constexpr (LN) {
                float4 *qb = reinterpret_cast<float4 *>(slab + cols + chunk[j] * 8);
                qb[0] = float4{db[j][0], db[j][1], db[j][2], db[j][3]};
                qb[1] = float4{db[j][4], db[j][5], db[j][6], db[j][7]};
            }
        }
    }
}

// Rows of at most 512 elements (the per-head q / k norms of Qwen3: 128): a row fits LPR <= 64 lanes, so a wave
// works on 64 / LPR rows at a time and never meets the other waves (no barrier per row).  Row sums: the same
// per-lane order, then the xor butterfly over the row's LPR lanes only; the steps 32 .. LPR of the wide kernel's
// butterfly and its three other wave sums would add exact zeros, so dx is the same bits.  d_weight / d_bias: per-lane
// sums over the rows a lane sees, combined over the block's row groups through LDS in group order.
template <int SRC, bool LN, int LPR>
__global__ __launch_bounds__(kRmsBwdThreads) void norm_bwd_narrow_kernel(const u32x4 *__restrict__ dy, const void *__restrict__ x,
                                                                          const float *__restrict__ weight, const float *__restrict__ mean_in,
                                                                          const float *__restrict__ rstd_in, int64_t rows, int64_t cols,
                                                                          void *__restrict__ dx, float *__restrict__ slabs) {
    constexpr int VPC = SRC == ODL_BF16 ? 1 : 2;
    constexpr int NS = LN ? 2 : 1;
    constexpr int RPW = kWave / LPR, RPB = (kRmsBwdThreads / kWave) * RPW;      // rows per wave / per block and pass
    __shared__ float part[NS][RPB][LPR * 8];
    const int lane = threadIdx.x % kWave, wv = threadIdx.x / kWave;
    const int grp = wv * RPW + lane / LPR, c = lane % LPR;
    const int64_t nchunk = cols / 8;
    const bool ok = c < nchunk;
    float wreg[8], dw[8], db[8];
    {
        const float4 w0 = ok ? *reinterpret_cast<const float4 *>(weight + c * 8) : float4{0, 0, 0, 0};
        const float4 w1 = ok ? *reinterpret_cast<const float4 *>(weight + c * 8 + 4) : float4{0, 0, 0, 0};
        wreg[0] = w0.x; wreg[1] = w0.y; wreg[2] = w0.z; wreg[3] = w0.w;
        wreg[4] = w1.x; wreg[5] = w1.y; wreg[6] = w1.z; wreg[7] = w1.w;
#pragma unroll
        for (int e = 0; e < 8; ++e) { dw[e] = 0.0f; db[e] = 0.0f; }
    }
    u32x4 nx[VPC], nd;
    auto fetch = [&](int64_t row) {
        const bool in = ok && row < rows;
        const u32x4 *p = reinterpret_cast<const u32x4 *>(x) + (row * nchunk + c) * VPC;
#pragma unroll
        for (int h = 0; h < VPC; ++h) nx[h] = in ? __builtin_nontemporal_load(p + h) : u32x4{0, 0, 0, 0};
        nd = in ? __builtin_nontemporal_load(dy + row * nchunk + c) : u32x4{0, 0, 0, 0};
    };
    const int64_t stride = (int64_t)gridDim.x * RPB;
    int64_t row = (int64_t)blockIdx.x * RPB + grp;
    fetch(row);
    // every lane of a wave runs the same number of passes (the shuffles need all of them): rows past the end are zeros
    for (int64_t base = (int64_t)blockIdx.x * RPB; base < rows; base += stride, row += stride) {
        u32x4 xr[VPC];
#pragma unroll
        for (int h = 0; h < VPC; ++h) xr[h] = nx[h];
        const u32x4 dr = nd;
        fetch(row + stride);
        const bool live = row < rows;
        const float rstd = live ? rstd_in[row] : 0.0f;
        const float mean = (LN && live) ? mean_in[row] : 0.0f;
        float xf[8], df[8], xh[8], t[8];
        unpack8<SRC>(xr, xf);
        unpack8<ODL_BF16>(&dr, df);
        float a1 = 0.0f, a2 = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            xh[e] = LN ? __fmul_rn(__fsub_rn(xf[e], mean), rstd) : __fmul_rn(xf[e], rstd);
            t[e] = __fmul_rn(df[e], wreg[e]);
            if constexpr (LN) a1 = __fadd_rn(a1, t[e]);
            a2 = __fmaf_rn(t[e], xh[e], a2);
            dw[e] = __fmaf_rn(df[e], xh[e], dw[e]);
            if constexpr (LN) db[e] = __fadd_rn(db[e], df[e]);
        }
#pragma unroll
        for (int off = LPR / 2; off > 0; off >>= 1) {
            a2 = __fadd_rn(a2, __shfl_xor(a2, off, kWave));
            if constexpr (LN) a1 = __fadd_rn(a1, __shfl_xor(a1, off, kWave));
        }
        const float c2 = __fdiv_rn(a2, (float)cols), c1 = LN ? __fdiv_rn(a1, (float)cols) : 0.0f;
        if (ok && live) {
            float o[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = __fmul_rn(rstd, __fmaf_rn(-xh[e], c2, LN ? __fsub_rn(t[e], c1) : t[e]));
            if constexpr (SRC == ODL_BF16) {
                reinterpret_cast<u32x4 *>(dx)[row * nchunk + c] = u32x4{pack2(o[0], o[1]), pack2(o[2], o[3]), pack2(o[4], o[5]), pack2(o[6], o[7])};
            } else {
                float4 *q = reinterpret_cast<float4 *>(dx) + (row * nchunk + c) * 2;
                q[0] = float4{o[0], o[1], o[2], o[3]};
                q[1] = float4{o[4], o[5], o[6], o[7]};
            }
        }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        part[0][grp][c * 8 + e] = dw[e];
        if constexpr (LN) part[1][grp][c * 8 + e] = db[e];
    }
    __syncthreads();
    float *slab = slabs + (int64_t)blockIdx.x * NS * cols;
    for (int col = threadIdx.x; col < NS * cols; col += kRmsBwdThreads) {
        const int set = col >= cols ? 1 : 0, cc = col - set * (int)cols;
        float acc = part[set][0][cc];
#pragma unroll
        for (int r = 1; r < RPB; ++r) acc = __fadd_rn(acc, part[set][r][cc]);
        slab[col] = acc;
    }
}

// Rows of 513 .. 1024 elements (the model widths 768 and 1024): one WAVE per row and trip, four rows per block in
// flight, no barrier per row.  Lane l holds the chunks l and 64 + l, i.e. what lane l of waves 0 and 1 of the
// block-per-row kernel holds (with SETS = 4, rows up to 2048, the kernel needs 300 registers and was measured
// slower than the block-per-row kernel: not used); the row sums are formed the same way (one butterfly per set of 64 chunks,
// then ((s0 + s1) + s2) + s3), so dx is the same bits.  d_weight / d_bias: per-lane sums over the rows a wave sees,
// the block's four waves combined through LDS in wave order, one slab per block.
template <int SRC, bool LN, int SETS>
__global__ __launch_bounds__(kRmsBwdThreads) void norm_bwd_wave_kernel(const u32x4 *__restrict__ dy, const void *__restrict__ x,
                                                                        const float *__restrict__ weight, const float *__restrict__ mean_in,
                                                                        const float *__restrict__ rstd_in, int64_t rows, int64_t cols,
                                                                        void *__restrict__ dx, float *__restrict__ slabs) {
    constexpr int VPC = SRC == ODL_BF16 ? 1 : 2;
    constexpr int NS = LN ? 2 : 1, NW = kRmsBwdThreads / kWave;
    __shared__ float part[NS][NW][kWave * 8];
    const int lane = threadIdx.x % kWave, wv = threadIdx.x / kWave;
    const int64_t nchunk = cols / 8;
    float wreg[SETS][8], dw[SETS][8], db[LN ? SETS : 1][8];
#pragma unroll
    for (int j = 0; j < SETS; ++j) {
        const int64_t c = j * kWave + lane;
        const bool ok = c < nchunk;
        const float4 w0 = ok ? *reinterpret_cast<const float4 *>(weight + c * 8) : float4{0, 0, 0, 0};
        const float4 w1 = ok ? *reinterpret_cast<const float4 *>(weight + c * 8 + 4) : float4{0, 0, 0, 0};
        wreg[j][0] = w0.x; wreg[j][1] = w0.y; wreg[j][2] = w0.z; wreg[j][3] = w0.w;
        wreg[j][4] = w1.x; wreg[j][5] = w1.y; wreg[j][6] = w1.z; wreg[j][7] = w1.w;
#pragma unroll
        for (int e = 0; e < 8; ++e) { dw[j][e] = 0.0f; if constexpr (LN) db[j][e] = 0.0f; }
    }
    u32x4 nx[SETS][VPC], nd[SETS];
    auto fetch = [&](int64_t row) {
#pragma unroll
        for (int j = 0; j < SETS; ++j) {
            const int64_t c = j * kWave + lane;
            const bool in = c < nchunk && row < rows;
            const u32x4 *p = reinterpret_cast<const u32x4 *>(x) + (row * nchunk + c) * VPC;
#pragma unroll
            for (int h = 0; h < VPC; ++h) nx[j][h] = in ? __builtin_nontemporal_load(p + h) : u32x4{0, 0, 0, 0};
            nd[j] = in ? __builtin_nontemporal_load(dy + row * nchunk + c) : u32x4{0, 0, 0, 0};
        }
    };
    const int64_t stride = (int64_t)gridDim.x * NW;
    int64_t row = (int64_t)blockIdx.x * NW + wv;
    fetch(row);
    for (; row < rows; row += stride) {                       // uniform per wave
        u32x4 xr[SETS][VPC], dr[SETS];
#pragma unroll
        for (int j = 0; j < SETS; ++j) {
#pragma unroll
            for (int h = 0; h < VPC; ++h) xr[j][h] = nx[j][h];
            dr[j] = nd[j];
        }
        fetch(row + stride);
        const float rstd = rstd_in[row];
        const float mean = LN ? mean_in[row] : 0.0f;
        float s1[SETS], s2[SETS];
#pragma unroll
        for (int j = 0; j < SETS; ++j) {
            float xf[8], df[8];
            unpack8<SRC>(xr[j], xf);
            unpack8<ODL_BF16>(&dr[j], df);
            float a1 = 0.0f, a2 = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float xh = LN ? __fmul_rn(__fsub_rn(xf[e], mean), rstd) : __fmul_rn(xf[e], rstd);
                const float t = __fmul_rn(df[e], wreg[j][e]);
                if constexpr (LN) a1 = __fadd_rn(a1, t);
                a2 = __fmaf_rn(t, xh, a2);
                dw[j][e] = __fmaf_rn(df[e], xh, dw[j][e]);
                if constexpr (LN) db[j][e] = __fadd_rn(db[j][e], df[e]);
            }
            s2[j] = wave_sum_butterfly(a2);
            s1[j] = LN ? wave_sum_butterfly(a1) : 0.0f;
        }
        float t2 = s2[0], t1 = s1[0];
#pragma unroll
        for (int j = 1; j < 4; ++j) {                         // the block-per-row kernel always adds four wave sums
            t2 = __fadd_rn(t2, j < SETS ? s2[j] : 0.0f);
            if constexpr (LN) t1 = __fadd_rn(t1, j < SETS ? s1[j] : 0.0f);
        }
        const float c2 = __fdiv_rn(t2, (float)cols), c1 = LN ? __fdiv_rn(t1, (float)cols) : 0.0f;
#pragma unroll
        for (int j = 0; j < SETS; ++j) {
            const int64_t c = j * kWave + lane;
            if (c < nchunk) {
                float xf[8], df[8], o[8];
                unpack8<SRC>(xr[j], xf);
                unpack8<ODL_BF16>(&dr[j], df);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float xh = LN ? __fmul_rn(__fsub_rn(xf[e], mean), rstd) : __fmul_rn(xf[e], rstd);
                    const float t = __fmul_rn(df[e], wreg[j][e]);
                    o[e] = __fmul_rn(rstd, __fmaf_rn(-xh, c2, LN ? __fsub_rn(t, c1) : t));
                }
                if constexpr (SRC == ODL_BF16) {
                    reinterpret_cast<u32x4 *>(dx)[row * nchunk + c] = u32x4{pack2(o[0], o[1]), pack2(o[2], o[3]), pack2(o[4], o[5]), pack2(o[6], o[7])};
                } else {
                    float4 *q = reinterpret_cast<float4 *>(dx) + (row * nchunk + c) * 2;
                    q[0] = float4{o[0], o[1], o[2], o[3]};
                    q[1] = float4{o[4], o[5], o[6], o[7]};
                }
            }
        }
    }
    // one set of 64 chunks at a time through LDS: the four waves' sums of a column are added in wave order
    float *slab = slabs + (int64_t)blockIdx.x * NS * cols;
#pragma unroll
    for (int j = 0; j < SETS; ++j) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            part[0][wv][lane * 8 + e] = dw[j][e];
            if constexpr (LN) part[1][wv][lane * 8 + e] = db[j][e];
        }
        __syncthreads();
        for (int i = threadIdx.x; i < NS * kWave * 8; i += kRmsBwdThreads) {
            const int set = i / (kWave * 8), cc = i % (kWave * 8);
            const int64_t col = (int64_t)j * kWave * 8 + cc;
            if (col < cols) {
                float acc = part[set][0][cc];
#pragma unroll
                for (int w = 1; w < NW; ++w) acc = __fadd_rn(acc, part[set][w][cc]);
                slab[set * cols + col] = acc;
            }
        }
        __syncthreads();
    }
}

// ------------------------------------------------------------------------ LayerNorm
// Same work split and summation order as the RMSNorm kernels.  Forward, per row:
//   mean = sum(x) / cols;  d = x - mean;  rstd = 1 / sqrt(sum(d * d) / cols + eps)   (d * d by fma)
//   y = bf16( ((d * rstd) * weight) + bias )          (bias may be absent)
// The backward is norm_bwd_kernel<.., LN = true, ..> above (slabs hold d_weight in [0, cols) and d_bias in
// [cols, 2 cols) of each block's row).
// Wide rows (CPL == 8): weight and bias are staged in LDS once per block.  Read from global memory in the output pass, the
// compiler hoists the loads of all eight chunks above the reductions, which takes 144 registers and leaves room for one
// 512-lane block per compute unit; from LDS a bf16 row needs 128 and two blocks fit (an fp32 row, twice the registers
// of input, keeps one block).
template <int SRC, int CPL, int THREADS>
__global__ __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu((CPL == 8 && SRC == ODL_BF16) ? 4 : 1, 8))) void layernorm_fwd_kernel(const void *__restrict__ x, const float *__restrict__ weight,
                                                                 const float *__restrict__ bias, int64_t rows, int64_t cols, float eps,
                                                                 uint16_t *__restrict__ y, float *__restrict__ mean_out,
                                                                 float *__restrict__ rstd_out, float *__restrict__ parts) {
    __shared__ uint32_t red[THREADS / kWave];
    constexpr bool kStage = CPL == 8;
    __shared__ __attribute__((aligned(16))) float s_w[kStage ? CPL * kWave * 8 : 4], s_b[kStage ? CPL * kWave * 8 : 4];
    if constexpr (kStage) {
        for (int64_t c = threadIdx.x; c < cols; c += THREADS) {
            s_w[c] = weight[c];
            s_b[c] = bias ? bias[c] : 0.0f;
        }
        __syncthreads();
    }
    constexpr int VPC = SRC == ODL_BF16 ? 1 : 2;
    constexpr int RB = CPL <= 2 ? 2 : 1;                    // rows per wave and trip, as in rmsnorm_fwd_kernel (more would spill here)
    const int lane = threadIdx.x % kWave;
    const int64_t wave = (int64_t)blockIdx.x * (THREADS / kWave) + threadIdx.x / kWave;
    const int64_t nwave = (int64_t)gridDim.x * (THREADS / kWave);
    const int64_t nchunk = cols / 8;
    uint32_t am = 0;
    for (int64_t row0 = wave * RB; row0 < rows; row0 += nwave * RB) {
        u32x4 raw[RB][CPL][VPC];
#pragma unroll
        for (int b = 0; b < RB; ++b)
#pragma unroll
            for (int j = 0; j < CPL; ++j) {
                const int64_t c = lane + (int64_t)kWave * j;
                const u32x4 *p = reinterpret_cast<const u32x4 *>(x) + ((row0 + b) * nchunk + c) * VPC;
#pragma unroll
                for (int h = 0; h < VPC; ++h) raw[b][j][h] = (c < nchunk && row0 + b < rows) ? __builtin_nontemporal_load(p + h) : u32x4{0, 0, 0, 0};
            }
        float acc[RB], mean[RB], rstd[RB];
#pragma unroll
        for (int b = 0; b < RB; ++b) {
            acc[b] = 0.0f;
#pragma unroll
            for (int j = 0; j < CPL; ++j) {
                float f[8];
                unpack8<SRC>(raw[b][j], f);
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[b] = __fadd_rn(acc[b], f[e]);
            }
        }
        wave_sum_butterfly_n<RB>(acc);
#pragma unroll
        for (int b = 0; b < RB; ++b) {
            mean[b] = __fdiv_rn(acc[b], (float)cols);
            acc[b] = 0.0f;
#pragma unroll
            for (int j = 0; j < CPL; ++j) {
                if (lane + (int64_t)kWave * j < nchunk) {      // padding chunks must not contribute (0 - mean)^2
                    float f[8];
                    unpack8<SRC>(raw[b][j], f);
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const float d = __fsub_rn(f[e], mean[b]);
                        acc[b] = __fmaf_rn(d, d, acc[b]);
                    }
                }
            }
        }
        wave_sum_butterfly_n<RB>(acc);
#pragma unroll
        for (int b = 0; b < RB; ++b) {
            const float var = __fdiv_rn(acc[b], (float)cols);
            rstd[b] = __fdiv_rn(1.0f, __builtin_sqrtf(__fadd_rn(var, eps)));
            if (lane == 0 && row0 + b < rows) { mean_out[row0 + b] = mean[b]; rstd_out[row0 + b] = rstd[b]; }
        }
#pragma unroll
        for (int j = 0; j < CPL; ++j) {
            const int64_t c = lane + (int64_t)kWave * j;
            if (c < nchunk) {
                const float *wp = kStage ? s_w : weight, *bp = kStage ? s_b : bias;
                const float4 w0 = *reinterpret_cast<const float4 *>(wp + c * 8), w1 = *reinterpret_cast<const float4 *>(wp + c * 8 + 4);
                const float w[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
                float bv[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
                if (bias) {
                    const float4 b0 = *reinterpret_cast<const float4 *>(bp + c * 8), b1 = *reinterpret_cast<const float4 *>(bp + c * 8 + 4);
                    bv[0] = b0.x; bv[1] = b0.y; bv[2] = b0.z; bv[3] = b0.w; bv[4] = b1.x; bv[5] = b1.y; bv[6] = b1.z; bv[7] = b1.w;
                }
#pragma unroll
                for (int b = 0; b < RB; ++b) {
                    if (row0 + b < rows) {
                        float f[8], o[8];
                        unpack8<SRC>(raw[b][j], f);
#pragma unroll
                        for (int e = 0; e < 8; ++e) o[e] = __fmul_rn(__fmul_rn(__fsub_rn(f[e], mean[b]), rstd[b]), w[e]);
                        if (bias) {
#pragma unroll
                            for (int e = 0; e < 8; ++e) o[e] = __fadd_rn(o[e], bv[e]);
                        }
                        uint32_t pk[4];
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            pk[q] = pack2(o[2 * q], o[2 * q + 1]);
                            am = max_u16x2(am, abs_bf16x2(pk[q]));
                        }
                        reinterpret_cast<u32x4 *>(y)[(row0 + b) * nchunk + c] = u32x4{pk[0], pk[1], pk[2], pk[3]};
                    }
                }
            }
        }
    }
    am = block_max_u32(fold_u16x2_to_f32bits(am), red);
    if (threadIdx.x == 0) parts[blockIdx.x] = bits_to_float(am);
    if (blockIdx.x == 0)
        for (int j = (int)gridDim.x + threadIdx.x; j < kParts; j += THREADS) parts[j] = 0.0f;
}

// slabs -> d_weight: a block owns 64 columns; 16 groups of lanes each add every 16th slab (8 loads in
// flight), the groups are combined through LDS in group order.  The order is fixed by the code.
__global__ __launch_bounds__(1024) void rmsnorm_bwd_reduce_kernel(const float *__restrict__ slabs, int nslab, int64_t cols,
                                                                   float *__restrict__ dw) {
    __shared__ float part[16][64];
    const int cx = threadIdx.x % 64, grp = threadIdx.x / 64;
    const int64_t c = (int64_t)blockIdx.x * 64 + cx;
    float a = 0.0f;
    if (c < cols) {
        int b = grp;
        for (; b + 7 * 16 < nslab; b += 8 * 16) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = slabs[(int64_t)(b + u * 16) * cols + c];
#pragma unroll
            for (int u = 0; u < 8; ++u) a = __fadd_rn(a, v[u]);
        }
        for (; b < nslab; b += 16) a = __fadd_rn(a, slabs[(int64_t)b * cols + c]);
    }
    part[grp][cx] = a;
    __syncthreads();
    if (grp == 0 && c < cols) {
        float t = part[0][cx];
#pragma unroll
        for (int g = 1; g < 16; ++g) t = __fadd_rn(t, part[g][cx]);
        dw[c] = t;
    }
}

static inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// slabs [nslab][cols] -> out[cols]
static void launch_slab_reduce(const float *slabs, int nslab, int64_t cols, float *out, hipStream_t stream) {
    hipLaunchKernelGGL(rmsnorm_bwd_reduce_kernel, dim3((unsigned)((cols + 63) / 64)), dim3(1024), 0, stream, slabs, nslab, cols, out);
}

// ------------------------------------------------ partial maxima + column sums in one pass
// For the grad_output of a Linear with a bias: the amax pass of its quantisation also adds up the
// columns (the bias gradient), so dY is not read a third time.  Block = 32 column-lanes (8 bf16 /
// 4 fp32 columns each) x 32 row-lanes; a lane adds its columns over rows ty, ty + 32, ... of the
// block's row slab in fp32, the 32 row-lanes are combined through LDS in order, and the block
// writes one slab row of column sums; rmsnorm_bwd_reduce_kernel adds the slabs in order.
template <int SRC>
__global__ __launch_bounds__(kFusedThreads) void amax_colsum_kernel(const void *__restrict__ x, int64_t rows, int64_t cols,
                                                                     int rows_per_block, float *__restrict__ parts,
                                                                     float *__restrict__ slabs) {
    constexpr int ESZ = SRC == ODL_BF16 ? 2 : 4;
    constexpr int CPL = 16 / ESZ;                 // columns per lane
    constexpr int CW = 32 * CPL;                  // columns per block
    __shared__ float sums[32][CW + 1];
    __shared__ uint32_t red[kFusedThreads / kWave];
    const int tx = threadIdx.x % 32, ty = threadIdx.x / 32;
    const int64_t c0 = (int64_t)blockIdx.x * CW + tx * CPL;
    const int64_t r0 = (int64_t)blockIdx.y * rows_per_block;
    const int64_t r1 = r0 + rows_per_block < rows ? r0 + rows_per_block : rows;
    const bool col_ok = c0 + CPL <= cols;          // host guarantees cols % CPL == 0
    float acc[CPL];
#pragma unroll
    for (int j = 0; j < CPL; ++j) acc[j] = 0.0f;
    uint32_t am = 0;
    const char *base = reinterpret_cast<const char *>(x);
    auto take = [&](const u32x4 v) {
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            if constexpr (SRC == ODL_BF16) {
                acc[2 * q] = __fadd_rn(acc[2 * q], bf16_lo(w[q]));
                acc[2 * q + 1] = __fadd_rn(acc[2 * q + 1], bf16_hi(w[q]));
                am = max_u16x2(am, abs_bf16x2(w[q]));
            } else {
                acc[q] = __fadd_rn(acc[q], bits_to_float(w[q]));
                am = max(am, w[q] & 0x7fffffffu);
            }
        }
    };
    if (col_ok) {
        int64_t r = r0 + ty;
        for (; r + 96 < r1; r += 128) {
            u32x4 v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = *reinterpret_cast<const u32x4 *>(base + ((r + 32 * u) * cols + c0) * ESZ);
#pragma unroll
            for (int u = 0; u < 4; ++u) take(v[u]);
        }
        for (; r < r1; r += 32) take(*reinterpret_cast<const u32x4 *>(base + (r * cols + c0) * ESZ));
    }
#pragma unroll
    for (int j = 0; j < CPL; ++j) sums[ty][tx * CPL + j] = acc[j];
    if constexpr (SRC == ODL_BF16) am = fold_u16x2_to_f32bits(am);
    am = block_max_u32(am, red);                   // has the barrier that also publishes sums[][]
    const int64_t slab = blockIdx.y;
    for (int c = threadIdx.x; c < CW; c += kFusedThreads) {
        float t = sums[0][c];
#pragma unroll
        for (int y = 1; y < 32; ++y) t = __fadd_rn(t, sums[y][c]);
        const int64_t col = (int64_t)blockIdx.x * CW + c;
        if (col < cols) slabs[slab * cols + col] = t;
    }
    const int bid = blockIdx.y * gridDim.x + blockIdx.x, nblk = gridDim.x * gridDim.y;
    if (threadIdx.x == 0) parts[bid] = bits_to_float(am);
    if (bid == 0)
        for (int j = nblk + threadIdx.x; j < kParts; j += kFusedThreads) parts[j] = 0.0f;
}

// ------------------------------------------------------------------------------ GELU
// The exact (erf) GELU of a bf16 input is a function of 16 bits: a table, made once per device by
// gelu_table_kernel in double precision, holds for every bf16 pattern x
//   fwd[x] = bf16( float( x * Phi(x) ) )            Phi(x) = erfc(-x / sqrt 2) / 2
//   bwd[x] = float( Phi(x) + x * phi(x) )           phi(x) = exp(-x^2 / 2) / sqrt(2 pi)
// (65536 bf16 values, then 65536 floats: 384 KB).  The kernels gather:
//   y = fwd[x],   dx = bf16( dy * bwd[x] ),   each with the partial maxima of what it writes.
constexpr int kGeluFwdBytes = 65536 * 2;

__global__ void gelu_table_kernel(uint16_t *__restrict__ fwd, float *__restrict__ bwd) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= 65536u) return;
    const double x = (double)bits_to_float(i << 16);
    const double cdf = 0.5 * erfc(-x * 0.70710678118654752440);
    const double pdf = exp(-0.5 * x * x) * 0.39894228040143267794;
    fwd[i] = (uint16_t)f32_to_bf16_bits((float)(x * cdf));
    bwd[i] = (float)(cdf + x * pdf);
}

// The gathers are served from LDS for the inputs that occur: a window of the table, the bf16 patterns with
// exponent fields kGeluExpLo .. kGeluExpHi - 1 (2^-31 <= |x| < 2^8) of both signs, is copied into LDS by every block
// (20 KB of the forward table, 39 KB of the backward one); zeros, denormals, tiny and huge inputs go to the full
// table in global memory.  One L2 access per element held the kernels to 40 % / 50 % of the HBM rate.
constexpr int kGeluExpLo = 96, kGeluExpHi = 135;
constexpr uint32_t kGeluWinLo = kGeluExpLo << 7, kGeluWin = (kGeluExpHi - kGeluExpLo) << 7;   // 4992 magnitudes per sign

template <typename T>
__device__ __forceinline__ void gelu_window_to_lds(const T *__restrict__ table, T *win) {
    for (uint32_t i = threadIdx.x; i < 2 * kGeluWin; i += kFusedThreads) {
        const uint32_t sign = i >= kGeluWin ? 1u : 0u;
        win[i] = table[(sign << 15) | (kGeluWinLo + i - sign * kGeluWin)];
    }
    __syncthreads();
}

template <typename T>
__device__ __forceinline__ T gelu_lookup(uint32_t bits16, const T *win, const T *__restrict__ table) {
    const uint32_t t = (bits16 & 0x7fffu) - kGeluWinLo;
    if (t < kGeluWin) return win[t + (bits16 >> 15) * kGeluWin];
    return table[bits16];
}

__global__ __launch_bounds__(kFusedThreads) void gelu_fwd_kernel(const u32x4 *__restrict__ x, int64_t n8, const uint16_t *__restrict__ fwd,
                                                                  u32x4 *__restrict__ y, float *__restrict__ parts) {
    __shared__ uint32_t red[kFusedThreads / kWave];
    __shared__ uint16_t win[2 * kGeluWin];
    gelu_window_to_lds(fwd, win);
    const int64_t stride = (int64_t)gridDim.x * kFusedThreads;
    uint32_t am = 0;
    constexpr int U = 2;                                   // 16-byte chunks in flight per lane
    int64_t i = (int64_t)blockIdx.x * kFusedThreads + threadIdx.x;
    auto one = [&](const u32x4 v, int64_t at) {
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
        uint32_t o[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            o[q] = (uint32_t)gelu_lookup(w[q] & 0xffffu, win, fwd) | ((uint32_t)gelu_lookup(w[q] >> 16, win, fwd) << 16);
            am = max_u16x2(am, abs_bf16x2(o[q]));
        }
        y[at] = u32x4{o[0], o[1], o[2], o[3]};
    };
    for (; i + (U - 1) * stride < n8; i += U * stride) {
        u32x4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = __builtin_nontemporal_load(x + i + u * stride);
#pragma unroll
        for (int u = 0; u < U; ++u) one(v[u], i + u * stride);
    }
    for (; i < n8; i += stride) one(__builtin_nontemporal_load(x + i), i);
    am = block_max_u32(fold_u16x2_to_f32bits(am), red);
    if (threadIdx.x == 0) parts[blockIdx.x] = bits_to_float(am);
    if (blockIdx.x == 0)
        for (int j = (int)gridDim.x + threadIdx.x; j < kParts; j += kFusedThreads) parts[j] = 0.0f;
}

__global__ __launch_bounds__(kFusedThreads) void gelu_bwd_kernel(const u32x4 *__restrict__ dy, const u32x4 *__restrict__ x, int64_t n8,
                                                                  const float *__restrict__ bwd, u32x4 *__restrict__ dx,
                                                                  float *__restrict__ parts) {
    __shared__ uint32_t red[kFusedThreads / kWave];
    __shared__ float win[2 * kGeluWin];
    gelu_window_to_lds(bwd, win);
    const int64_t stride = (int64_t)gridDim.x * kFusedThreads;
    uint32_t am = 0;
    constexpr int U = 2;
    int64_t i = (int64_t)blockIdx.x * kFusedThreads + threadIdx.x;
    auto one = [&](const u32x4 v, const u32x4 d, int64_t at) {
        const uint32_t w[4] = {v.x, v.y, v.z, v.w}, dw[4] = {d.x, d.y, d.z, d.w};
        uint32_t o[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            o[q] = pack2(__fmul_rn(bf16_lo(dw[q]), gelu_lookup(w[q] & 0xffffu, win, bwd)),
                         __fmul_rn(bf16_hi(dw[q]), gelu_lookup(w[q] >> 16, win, bwd)));
            am = max_u16x2(am, abs_bf16x2(o[q]));
        }
        dx[at] = u32x4{o[0], o[1], o[2], o[3]};
    };
    for (; i + (U - 1) * stride < n8; i += U * stride) {
        u32x4 v[U], d[U];
#pragma unroll
        for (int u = 0; u < U; ++u) { v[u] = __builtin_nontemporal_load(x + i + u * stride); d[u] = __builtin_nontemporal_load(dy + i + u * stride); }
#pragma unroll
        for (int u = 0; u < U; ++u) one(v[u], d[u], i + u * stride);
    }
    for (; i < n8; i += stride) one(__builtin_nontemporal_load(x + i), __builtin_nontemporal_load(dy + i), i);
    am = block_max_u32(fold_u16x2_to_f32bits(am), red);
    if (threadIdx.x == 0) parts[blockIdx.x] = bits_to_float(am);
    if (blockIdx.x == 0)
        for (int j = (int)gridDim.x + threadIdx.x; j < kParts; j += kFusedThreads) parts[j] = 0.0f;
}


// at most two fat blocks per CU, and never more blocks than there are partial maxima
static int grid_cap() {
    const int cus = device_cu_count();
    return cus * 2 < kParts ? cus * 2 : kParts;
}

}  // namespace odl

using namespace odl;

extern "C" int odl_fp8_swiglu_amax_parts(const void *gate, const void *up, int64_t rows, int64_t cols, void *h, float *parts,
                                         odl_stream_t stream_) {
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    if (rows < 0 || cols < 0) return set_error(ODL_ERR_ARG, "odl_fp8_swiglu_amax_parts: negative shape");
    const int64_t n = rows * cols;
    if (!parts || (n > 0 && (!gate || !up || !h))) return set_error(ODL_ERR_ARG, "odl_fp8_swiglu_amax_parts: null pointer");
    if (n % 8 != 0 || !aligned16(gate) || !aligned16(up) || !aligned16(h))
        return set_error(ODL_ERR_SHAPE, "odl_fp8_swiglu_amax_parts: rows*cols must be a multiple of 8 and the pointers 16-byte aligned");
    const int64_t n8 = n / 8;
    int64_t g = (n8 + 2 * kFusedThreads - 1) / (2 * kFusedThreads);
    g = g < 1 ? 1 : (g < grid_cap() ? g : grid_cap());
    hipLaunchKernelGGL(swiglu_fwd_kernel, dim3((unsigned)g), dim3(kFusedThreads), 0, stream, reinterpret_cast<const u32x4 *>(gate),
                       reinterpret_cast<const u32x4 *>(up), n8, reinterpret_cast<u32x4 *>(h), parts);
    return check_launch("odl_fp8_swiglu_amax_parts");
}

extern "C" int odl_fp8_swiglu_bwd_amax_parts(const void *dh, const void *gate, const void *up, int64_t rows, int64_t cols,
                                             void *dgate, void *dup, float *parts_dgate, float *parts_dup, odl_stream_t stream_) {
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    if (rows < 0 || cols < 0) return set_error(ODL_ERR_ARG, "odl_fp8_swiglu_bwd_amax_parts: negative shape");
    const int64_t n = rows * cols;
    if (!parts_dgate || !parts_dup || (n > 0 && (!dh || !gate || !up || !dgate || !dup)))
        return set_error(ODL_ERR_ARG, "odl_fp8_swiglu_bwd_amax_parts: null pointer");
    if (n % 8 != 0 || !aligned16(dh) || !aligned16(gate) || !aligned16(up) || !aligned16(dgate) || !aligned16(dup))
        return set_error(ODL_ERR_SHAPE, "odl_fp8_swiglu_bwd_amax_parts: rows*cols must be a multiple of 8 and the pointers 16-byte aligned");
    const int64_t n8 = n / 8;
    int64_t g = (n8 + kFusedThreads - 1) / kFusedThreads;
    g = g < 1 ? 1 : (g < grid_cap() ? g : grid_cap());
    hipLaunchKernelGGL(swiglu_bwd_kernel, dim3((unsigned)g), dim3(kFusedThreads), 0, stream, reinterpret_cast<const u32x4 *>(dh),
                       reinterpret_cast<const u32x4 *>(gate), reinterpret_cast<const u32x4 *>(up), n8,
                       reinterpret_cast<u32x4 *>(dgate), reinterpret_cast<u32x4 *>(dup), parts_dgate, parts_dup);
    return check_launch("odl_fp8_swiglu_bwd_amax_parts");
}

extern "C" int odl_fp8_rmsnorm_amax_parts(const void *x, int src_dtype, const float *weight, int64_t rows, int64_t cols, float eps,
                                          void *y, float *rstd, float *parts, odl_stream_t stream_) {
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    if (rows < 0 || cols < 0) return set_error(ODL_ERR_ARG, "odl_fp8_rmsnorm_amax_parts: negative shape");
    if (src_dtype != ODL_BF16 && src_dtype != ODL_F32) return set_error(ODL_ERR_ARG, "odl_fp8_rmsnorm_amax_parts: src_dtype %d", src_dtype);
    if (!parts || (rows > 0 && !rstd) || (rows * cols > 0 && (!x || !weight || !y)))
        return set_error(ODL_ERR_ARG, "odl_fp8_rmsnorm_amax_parts: null pointer");
    if (cols < 8 || cols % 8 != 0 || cols > 8192 || !aligned16(x) || !aligned16(y) || !aligned16(weight))
        return set_error(ODL_ERR_SHAPE, "odl_fp8_rmsnorm_amax_parts: cols must be a multiple of 8 in [8, 8192] and the pointers 16-byte aligned");
    if (cols <= 256) {                                        // several rows per wave
        const int lpr = cols <= 64 ? 8 : (cols <= 128 ? 16 : 32), rpb = (kFusedThreads / kWave) * (kWave / lpr);
        int64_t gn = (rows + rpb - 1) / rpb;
        gn = gn < 1 ? 1 : (gn < grid_cap() ? gn : grid_cap());
#define ODL_RMSF(SRC, LPR) hipLaunchKernelGGL((rmsnorm_fwd_narrow_kernel<SRC, LPR>), dim3((unsigned)gn), dim3(kFusedThreads), 0, stream, x, weight, rows, cols, eps, reinterpret_cast<uint16_t *>(y), rstd, parts)
#define ODL_RMSF_SRC(LPR) do { if (src_dtype == ODL_BF16) ODL_RMSF(ODL_BF16, LPR); else ODL_RMSF(ODL_F32, LPR); } while (0)
        if (lpr == 8) ODL_RMSF_SRC(8);
        else if (lpr == 16) ODL_RMSF_SRC(16);
        else ODL_RMSF_SRC(32);
#undef ODL_RMSF_SRC
#undef ODL_RMSF
        return check_launch("odl_fp8_rmsnorm_amax_parts");
    }
    const int64_t cpl = (cols / 8 + kWave - 1) / kWave;
    // fp32 rows of 5 .. 8 chunks a lane (64 registers of input per row) allow four waves per SIMD: as 1024-lane blocks that
    // is one block per compute unit, which reads, then writes, then makes room for the next; two 512-lane blocks per unit
    // overlap one's stores with the other's loads (8192 x 4096: 43.4 -> 40.4 us; bf16 rows measured no difference)
    const int threads = cpl <= 4 ? kFusedThreads : (cpl <= 8 ? (src_dtype == ODL_BF16 ? kFusedThreads : 512) : 256);
    const int rows_per_block = (threads / kWave) * (cpl <= 2 ? 4 : (cpl <= 4 ? 2 : 1));   // RB rows per wave and trip
    int64_t g = (rows + rows_per_block - 1) / rows_per_block;
    g = g < 1 ? 1 : (g < grid_cap() ? g : grid_cap());
#define ODL_RMS(SRC, CPL, THR) hipLaunchKernelGGL((rmsnorm_fwd_kernel<SRC, CPL, THR>), dim3((unsigned)g), dim3(THR), 0, stream, x, weight, rows, cols, eps, reinterpret_cast<uint16_t *>(y), rstd, parts)
#define ODL_RMS_SRC(CPL, THR) do { if (src_dtype == ODL_BF16) ODL_RMS(ODL_BF16, CPL, THR); else ODL_RMS(ODL_F32, CPL, THR); } while (0)
    if (cpl <= 2) ODL_RMS_SRC(2, kFusedThreads);
    else if (cpl <= 4) ODL_RMS_SRC(4, kFusedThreads);
    else if (cpl <= 8 && src_dtype == ODL_BF16) ODL_RMS(ODL_BF16, 8, kFusedThreads);
    else if (cpl <= 8) ODL_RMS(ODL_F32, 8, 512);
    else ODL_RMS_SRC(16, 256);
#undef ODL_RMS_SRC
#undef ODL_RMS
    return check_launch("odl_fp8_rmsnorm_amax_parts");
}

extern "C" int odl_fp8_rmsnorm_bwd(const void *dy, const void *x, int src_dtype, const float *weight, const float *rstd, int64_t rows,
                                   int64_t cols, void *dx, float *dweight, float *workspace, odl_stream_t stream_) {
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    if (rows < 0 || cols < 0) return set_error(ODL_ERR_ARG, "odl_fp8_rmsnorm_bwd: negative shape");
    if (src_dtype != ODL_BF16 && src_dtype != ODL_F32) return set_error(ODL_ERR_ARG, "odl_fp8_rmsnorm_bwd: src_dtype %d", src_dtype);
    if (!dweight || !workspace || !weight || (rows > 0 && !rstd) || (rows * cols > 0 && (!dy || !x || !dx)))
        return set_error(ODL_ERR_ARG, "odl_fp8_rmsnorm_bwd: null pointer");
    if (cols < 8 || cols % 8 != 0 || cols > 8192 || !aligned16(x) || !aligned16(dy) || !aligned16(dx) || !aligned16(weight))
        return set_error(ODL_ERR_SHAPE, "odl_fp8_rmsnorm_bwd: cols must be a multiple of 8 in [8, 8192] and the pointers 16-byte aligned");
    int64_t g = rows < 1 ? 1 : (rows < ODL_FP8_RMSNORM_BWD_SLABS ? rows : ODL_FP8_RMSNORM_BWD_SLABS);
    if (cols <= 512) {                                        // a row fits one wave: several rows per wave
        const int lpr = cols <= 64 ? 8 : (cols <= 128 ? 16 : (cols <= 256 ? 32 : 64)), rpb = (kRmsBwdThreads / kWave) * (kWave / lpr);
        g = (rows + rpb - 1) / rpb;
        g = g < 1 ? 1 : (g < ODL_FP8_RMSNORM_BWD_SLABS ? g : ODL_FP8_RMSNORM_BWD_SLABS);
#define ODL_RMSN(SRC, LPR) hipLaunchKernelGGL((norm_bwd_narrow_kernel<SRC, false, LPR>), dim3((unsigned)g), dim3(kRmsBwdThreads), 0, stream, reinterpret_cast<const u32x4 *>(dy), x, weight, (const float *)nullptr, rstd, rows, cols, dx, workspace)
#define ODL_RMSN_SRC(LPR) do { if (src_dtype == ODL_BF16) ODL_RMSN(ODL_BF16, LPR); else ODL_RMSN(ODL_F32, LPR); } while (0)
        if (lpr == 8) ODL_RMSN_SRC(8);
        else if (lpr == 16) ODL_RMSN_SRC(16);
        else if (lpr == 32) ODL_RMSN_SRC(32);
        else ODL_RMSN_SRC(64);
#undef ODL_RMSN_SRC
#undef ODL_RMSN
        launch_slab_reduce(workspace, (int)g, cols, dweight, stream);
        return check_launch("odl_fp8_rmsnorm_bwd");
    }
    if (cols <= 1024) {                                       // a wave per row, four rows per block in flight
        const int64_t rpb = kRmsBwdThreads / kWave;
        g = (rows + rpb - 1) / rpb;
        g = g < 1 ? 1 : (g < ODL_FP8_RMSNORM_BWD_SLABS ? g : ODL_FP8_RMSNORM_BWD_SLABS);
#define ODL_RMSW(SRC, SETS) hipLaunchKernelGGL((norm_bwd_wave_kernel<SRC, false, SETS>), dim3((unsigned)g), dim3(kRmsBwdThreads), 0, stream, reinterpret_cast<const u32x4 *>(dy), x, weight, (const float *)nullptr, rstd, rows, cols, dx, workspace)
#define ODL_RMSW_SRC(SETS) do { if (src_dtype == ODL_BF16) ODL_RMSW(ODL_BF16, SETS); else ODL_RMSW(ODL_F32, SETS); } while (0)
        ODL_RMSW_SRC(2);
#undef ODL_RMSW_SRC
#undef ODL_RMSW
        launch_slab_reduce(workspace, (int)g, cols, dweight, stream);
        return check_launch("odl_fp8_rmsnorm_bwd");
    }
    const int64_t cplw = (cols / 8 + kRmsBwdThreads - 1) / kRmsBwdThreads;
#define ODL_RMSB(SRC, CPLW) hipLaunchKernelGGL((norm_bwd_kernel<SRC, false, CPLW>), dim3((unsigned)g), dim3(kRmsBwdThreads), 0, stream, reinterpret_cast<const u32x4 *>(dy), x, weight, (const float *)nullptr, rstd, rows, cols, dx, workspace)
#define ODL_RMSB_SRC(CPLW) do { if (src_dtype == ODL_BF16) ODL_RMSB(ODL_BF16, CPLW); else ODL_RMSB(ODL_F32, CPLW); } while (0)
    if (cplw <= 1) ODL_RMSB_SRC(1);
    else if (cplw <= 2) ODL_RMSB_SRC(2);
    else ODL_RMSB_SRC(4);
#undef ODL_RMSB_SRC
#undef ODL_RMSB
    launch_slab_reduce(workspace, (int)g, cols, dweight, stream);
    return check_launch("odl_fp8_rmsnorm_bwd");
}

extern "C" int odl_fp8_amax_parts_colsum(const void *x, int src_dtype, int64_t rows, int64_t cols, float *parts, float *colsum,
                                         float *workspace, odl_stream_t stream_) {
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    if (rows <= 0 || cols <= 0) return set_error(ODL_ERR_ARG, "odl_fp8_amax_parts_colsum: empty or negative shape");
    if (!x || !parts || !colsum || !workspace) return set_error(ODL_ERR_ARG, "odl_fp8_amax_parts_colsum: null pointer");
    if (src_dtype != ODL_BF16 && src_dtype != ODL_F32) return set_error(ODL_ERR_ARG, "odl_fp8_amax_parts_colsum: src_dtype %d", src_dtype);
    const int cpl = src_dtype == ODL_BF16 ? 8 : 4, cw = 32 * cpl;
    const int64_t col_blocks = (cols + cw - 1) / cw;
    if (cols % cpl != 0 || !aligned16(x) || col_blocks > kParts)
        return set_error(ODL_ERR_SHAPE, "odl_fp8_amax_parts_colsum: cols must be a multiple of %d and at most %d, x 16-byte aligned", cpl, kParts * cw);
    int64_t slabs = kParts / col_blocks;                      // one partial maximum per block
    int64_t rpb = (rows + slabs - 1) / slabs;
    rpb = ((rpb + 31) / 32) * 32;
    slabs = (rows + rpb - 1) / rpb;
    if (src_dtype == ODL_BF16) hipLaunchKernelGGL((amax_colsum_kernel<ODL_BF16>), dim3((unsigned)col_blocks, (unsigned)slabs), dim3(kFusedThreads), 0, stream, x, rows, cols, (int)rpb, parts, workspace);
    else hipLaunchKernelGGL((amax_colsum_kernel<ODL_F32>), dim3((unsigned)col_blocks, (unsigned)slabs), dim3(kFusedThreads), 0, stream, x, rows, cols, (int)rpb, parts, workspace);
    launch_slab_reduce(workspace, (int)slabs, cols, colsum, stream);
    return check_launch("odl_fp8_amax_parts_colsum");
}

extern "C" int odl_fp8_layernorm_amax_parts(const void *x, int src_dtype, const float *weight, const float *bias, int64_t rows,
                                            int64_t cols, float eps, void *y, float *mean, float *rstd, float *parts,
                                            odl_stream_t stream_) {
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    if (rows < 0 || cols < 0) return set_error(ODL_ERR_ARG, "odl_fp8_layernorm_amax_parts: negative shape");
    if (src_dtype != ODL_BF16 && src_dtype != ODL_F32) return set_error(ODL_ERR_ARG, "odl_fp8_layernorm_amax_parts: src_dtype %d", src_dtype);
    if (!parts || (rows > 0 && (!rstd || !mean)) || (rows * cols > 0 && (!x || !weight || !y)))
        return set_error(ODL_ERR_ARG, "odl_fp8_layernorm_amax_parts: null pointer");
    if (cols < 8 || cols % 8 != 0 || cols > 4096 || !aligned16(x) || !aligned16(y) || !aligned16(weight) || !aligned16(bias))
        return set_error(ODL_ERR_SHAPE, "odl_fp8_layernorm_amax_parts: cols must be a multiple of 8 in [8, 4096] and the pointers 16-byte aligned");
    const int64_t cpl = (cols / 8 + kWave - 1) / kWave;
    const int threads = cpl <= 4 ? kFusedThreads : 512;     // wider rows need more than the 128 registers of a 1024-lane block
    const int rows_per_block = (threads / kWave) * (cpl <= 2 ? 2 : 1);   // RB rows per wave and trip
    int64_t g = (rows + rows_per_block - 1) / rows_per_block;
    g = g < 1 ? 1 : (g < grid_cap() ? g : grid_cap());
#define ODL_LN(SRC, CPL, THR) hipLaunchKernelGGL((layernorm_fwd_kernel<SRC, CPL, THR>), dim3((unsigned)g), dim3(THR), 0, stream, x, weight, bias, rows, cols, eps, reinterpret_cast<uint16_t *>(y), mean, rstd, parts)
#define ODL_LN_SRC(CPL, THR) do { if (src_dtype == ODL_BF16) ODL_LN(ODL_BF16, CPL, THR); else ODL_LN(ODL_F32, CPL, THR); } while (0)
    if (cpl <= 2) ODL_LN_SRC(2, kFusedThreads);
    else if (cpl <= 4) ODL_LN_SRC(4, kFusedThreads);
    else ODL_LN_SRC(8, 512);
#undef ODL_LN_SRC
#undef ODL_LN
    return check_launch("odl_fp8_layernorm_amax_parts");
}

extern "C" int odl_fp8_layernorm_bwd(const void *dy, const void *x, int src_dtype, const float *weight, const float *mean,
                                     const float *rstd, int64_t rows, int64_t cols, void *dx, float *dweight, float *dbias,
                                     float *workspace, odl_stream_t stream_) {
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    if (rows < 0 || cols < 0) return set_error(ODL_ERR_ARG, "odl_fp8_layernorm_bwd: negative shape");
    if (src_dtype != ODL_BF16 && src_dtype != ODL_F32) return set_error(ODL_ERR_ARG, "odl_fp8_layernorm_bwd: src_dtype %d", src_dtype);
    if (!dweight || !dbias || !workspace || !weight || (rows > 0 && (!rstd || !mean)) || (rows * cols > 0 && (!dy || !x || !dx)))
        return set_error(ODL_ERR_ARG, "odl_fp8_layernorm_bwd: null pointer");
    if (dbias != dweight + cols) return set_error(ODL_ERR_ARG, "odl_fp8_layernorm_bwd: dbias must follow dweight (dweight + cols)");
    if (cols < 8 || cols % 8 != 0 || cols > 4096 || !aligned16(x) || !aligned16(dy) || !aligned16(dx) || !aligned16(weight))
        return set_error(ODL_ERR_SHAPE, "odl_fp8_layernorm_bwd: cols must be a multiple of 8 in [8, 4096] and the pointers 16-byte aligned");
    int64_t g = rows < 1 ? 1 : (rows < ODL_FP8_RMSNORM_BWD_SLABS ? rows : ODL_FP8_RMSNORM_BWD_SLABS);
    if (cols <= 512) {                                        // a row fits one wave: several rows per wave
        const int lpr = cols <= 64 ? 8 : (cols <= 128 ? 16 : (cols <= 256 ? 32 : 64)), rpb = (kRmsBwdThreads / kWave) * (kWave / lpr);
        g = (rows + rpb - 1) / rpb;
        g = g < 1 ? 1 : (g < ODL_FP8_RMSNORM_BWD_SLABS ? g : ODL_FP8_RMSNORM_BWD_SLABS);
#define ODL_LNN(SRC, LPR) hipLaunchKernelGGL((norm_bwd_narrow_kernel<SRC, true, LPR>), dim3((unsigned)g), dim3(kRmsBwdThreads), 0, stream, reinterpret_cast<const u32x4 *>(dy), x, weight, mean, rstd, rows, cols, dx, workspace)
#define ODL_LNN_SRC(LPR) do { if (src_dtype == ODL_BF16) ODL_LNN(ODL_BF16, LPR); else ODL_LNN(ODL_F32, LPR); } while (0)
        if (lpr == 8) ODL_LNN_SRC(8);
        else if (lpr == 16) ODL_LNN_SRC(16);
        else if (lpr == 32) ODL_LNN_SRC(32);
        else ODL_LNN_SRC(64);
#undef ODL_LNN_SRC
#undef ODL_LNN
        launch_slab_reduce(workspace, (int)g, 2 * cols, dweight, stream);
        return check_launch("odl_fp8_layernorm_bwd");
    }
    if (cols <= 1024) {                                       // a wave per row, four rows per block in flight
        const int64_t rpb = kRmsBwdThreads / kWave;
        g = (rows + rpb - 1) / rpb;
        g = g < 1 ? 1 : (g < ODL_FP8_RMSNORM_BWD_SLABS ? g : ODL_FP8_RMSNORM_BWD_SLABS);
#define ODL_LNW(SRC, SETS) hipLaunchKernelGGL((norm_bwd_wave_kernel<SRC, true, SETS>), dim3((unsigned)g), dim3(kRmsBwdThreads), 0, stream, reinterpret_cast<const u32x4 *>(dy), x, weight, mean, rstd, rows, cols, dx, workspace)
#define ODL_LNW_SRC(SETS) do { if (src_dtype == ODL_BF16) ODL_LNW(ODL_BF16, SETS); else ODL_LNW(ODL_F32, SETS); } while (0)
        ODL_LNW_SRC(2);
#undef ODL_LNW_SRC
#undef ODL_LNW
        launch_slab_reduce(workspace, (int)g, 2 * cols, dweight, stream);
        return check_launch("odl_fp8_layernorm_bwd");
    }
    const int64_t cplw = (cols / 8 + kRmsBwdThreads - 1) / kRmsBwdThreads;
#define ODL_LNB(SRC, CPLW) hipLaunchKernelGGL((norm_bwd_kernel<SRC, true, CPLW>), dim3((unsigned)g), dim3(kRmsBwdThreads), 0, stream, reinterpret_cast<const u32x4 *>(dy), x, weight, mean, rstd, rows, cols, dx, workspace)
#define ODL_LNB_SRC(CPLW) do { if (src_dtype == ODL_BF16) ODL_LNB(ODL_BF16, CPLW); else ODL_LNB(ODL_F32, CPLW); } while (0)
    if (cplw <= 1) ODL_LNB_SRC(1);
    else ODL_LNB_SRC(2);
#undef ODL_LNB_SRC
#undef ODL_LNB
    // slabs are rows of 2 * cols sums (d_weight, d_bias); dweight and dbias are adjacent, so one reduction writes both
    launch_slab_reduce(workspace, (int)g, 2 * cols, dweight, stream);
    return check_launch("odl_fp8_layernorm_bwd");
}

extern "C" int odl_fp8_gelu_table(void *table, odl_stream_t stream_) {
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    if (!table || !aligned16(table)) return set_error(ODL_ERR_ARG, "odl_fp8_gelu_table: null or misaligned table");
    hipLaunchKernelGGL(gelu_table_kernel, dim3(65536 / 256), dim3(256), 0, stream, reinterpret_cast<uint16_t *>(table),
                       reinterpret_cast<float *>(reinterpret_cast<uint8_t *>(table) + kGeluFwdBytes));
    return check_launch("odl_fp8_gelu_table");
}

extern "C" int odl_fp8_gelu_amax_parts(const void *x, int64_t rows, int64_t cols, const void *table, void *y, float *parts,
                                       odl_stream_t stream_) {
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    if (rows < 0 || cols < 0) return set_error(ODL_ERR_ARG, "odl_fp8_gelu_amax_parts: negative shape");
    const int64_t n = rows * cols;
    if (!parts || !table || (n > 0 && (!x || !y))) return set_error(ODL_ERR_ARG, "odl_fp8_gelu_amax_parts: null pointer");
    if (n % 8 != 0 || !aligned16(x) || !aligned16(y) || !aligned16(table))
        return set_error(ODL_ERR_SHAPE, "odl_fp8_gelu_amax_parts: rows*cols must be a multiple of 8 and the pointers 16-byte aligned");
    const int64_t n8 = n / 8;
    int64_t g = (n8 + kFusedThreads - 1) / kFusedThreads;
    g = g < 1 ? 1 : (g < grid_cap() ? g : grid_cap());
    hipLaunchKernelGGL(gelu_fwd_kernel, dim3((unsigned)g), dim3(kFusedThreads), 0, stream, reinterpret_cast<const u32x4 *>(x), n8,
                       reinterpret_cast<const uint16_t *>(table), reinterpret_cast<u32x4 *>(y), parts);
    return check_launch("odl_fp8_gelu_amax_parts");
}

extern "C" int odl_fp8_gelu_bwd_amax_parts(const void *dy, const void *x, int64_t rows, int64_t cols, const void *table, void *dx,
                                           float *parts, odl_stream_t stream_) {
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    if (rows < 0 || cols < 0) return set_error(ODL_ERR_ARG, "odl_fp8_gelu_bwd_amax_parts: negative shape");
    const int64_t n = rows * cols;
    if (!parts || !table || (n > 0 && (!x || !dy || !dx))) return set_error(ODL_ERR_ARG, "odl_fp8_gelu_bwd_amax_parts: null pointer");
    if (n % 8 != 0 || !aligned16(x) || !aligned16(dy) || !aligned16(dx) || !aligned16(table))
        return set_error(ODL_ERR_SHAPE, "odl_fp8_gelu_bwd_amax_parts: rows*cols must be a multiple of 8 and the pointers 16-byte aligned");
    const int64_t n8 = n / 8;
    int64_t g = (n8 + kFusedThreads - 1) / kFusedThreads;
    g = g < 1 ? 1 : (g < grid_cap() ? g : grid_cap());
    hipLaunchKernelGGL(gelu_bwd_kernel, dim3((unsigned)g), dim3(kFusedThreads), 0, stream, reinterpret_cast<const u32x4 *>(dy),
                       reinterpret_cast<const u32x4 *>(x), n8,
                       reinterpret_cast<const float *>(reinterpret_cast<const uint8_t *>(table) + kGeluFwdBytes),
                       reinterpret_cast<u32x4 *>(dx), parts);
    return check_launch("odl_fp8_gelu_bwd_amax_parts");
}
