// Shared device helpers for the gfx950 FP8 kernels: packed bf16 handling,
// hardware FP8 conversion with the clamp / NaN rules of the C ABI, and
// wavefront (64-lane) + LDS reductions.
#pragma once

#include <hip/hip_runtime.h>
#include <float.h>
#include <stdint.h>

#include "../../include/odl_fp8.h"

namespace odl {

constexpr int kWave = 64;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));

int set_error(int code, const char *fmt, ...);   // defined in api.hip
int check_launch(const char *what);              // hipGetLastError -> status
int device_cu_count();                           // compute units of the CURRENT device (cached per device, api.hip)
// Device addresses of the two objects in the library's device image, for the CURRENT device (looked up once per device
// with hipGetSymbolAddress, which must not run under stream capture; odl_fp8_init_device makes both lookups):
float *scratch_for_current_device(const char *who);            // quant.hip: partial maxima of the entry point that allocates nothing
const float *unit_scale_for_current_device(const char *who);   // mx.hip: the 1.0f the block-scaled GEMM epilogues multiply by

__device__ __forceinline__ float bits_to_float(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t float_to_bits(float f) { return __builtin_bit_cast(uint32_t, f); }

// low / high bf16 of a packed dword, widened to fp32 (exact)
__device__ __forceinline__ float bf16_lo(uint32_t w) { return bits_to_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return bits_to_float(w & 0xffff0000u); }

// fp32 -> bf16 bits, round to nearest even, NaN stays a quiet NaN
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    uint32_t u = float_to_bits(f);
    uint32_t r = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
    return (f != f) ? ((u >> 16) | 0x40u) : r;
}

// two fp32 -> packed bf16 (lo = a, hi = b) with the hardware's round-to-nearest-even conversion
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{a, b}, bf16x2));   // v_cvt_pk_bf16_f32
}

template <int FMT> struct Fp8Lim;
template <> struct Fp8Lim<ODL_FP8_E4M3> { static constexpr float max = 448.0f; };
template <> struct Fp8Lim<ODL_FP8_E5M2> { static constexpr float max = 57344.0f; };

// Two fp32 -> two FP8 codes packed into the low or high half of `old`.
// The clamp makes the result independent of the hardware's overflow mode.
template <int FMT, bool HI>
__device__ __forceinline__ uint32_t cvt_pk(float a, float b, uint32_t old) {
    constexpr float m = Fp8Lim<FMT>::max;
    a = __builtin_amdgcn_fmed3f(a, -m, m);
    b = __builtin_amdgcn_fmed3f(b, -m, m);
    if constexpr (FMT == ODL_FP8_E4M3)
        return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, (int)old, HI);
    else
        return (uint32_t)__builtin_amdgcn_cvt_pk_bf8_f32(a, b, (int)old, HI);
}

// Four scaled values -> one dword of codes (byte i = value i).
// NaN inputs are patched afterwards to 0x7F | sign: med3 does not keep NaN.
template <int FMT>
__device__ __forceinline__ uint32_t quantise4(float x0, float x1, float x2, float x3,
                                              float s0, float s1, float s2, float s3) {
    uint32_t r = 0;
    r = cvt_pk<FMT, false>(x0 * s0, x1 * s1, r);
    r = cvt_pk<FMT, true>(x2 * s2, x3 * s3, r);
    if (__builtin_expect((x0 != x0) | (x1 != x1) | (x2 != x2) | (x3 != x3), 0)) {
        if (x0 != x0) r = (r & 0xffffff00u) | (0x7fu | ((float_to_bits(x0) >> 24) & 0x80u));
        if (x1 != x1) r = (r & 0xffff00ffu) | ((0x7fu | ((float_to_bits(x1) >> 24) & 0x80u)) << 8);
        if (x2 != x2) r = (r & 0xff00ffffu) | ((0x7fu | ((float_to_bits(x2) >> 24) & 0x80u)) << 16);
        if (x3 != x3) r = (r & 0x00ffffffu) | ((0x7fu | ((float_to_bits(x3) >> 24) & 0x80u)) << 24);
    }
    return r;
}

// scale = fp8_max / amax / 2^margin with the guards of the C ABI
__device__ __forceinline__ float scale_rule(float amax, float fp8_max, int margin, float fallback) {
    if (!(amax > 0.0f) || __builtin_isinf(amax)) return fallback;
    float s = __fdiv_rn(fp8_max, amax);                     // IEEE division, not the fast reciprocal
    s = ldexpf(s, -margin);
    if (__builtin_isinf(s)) s = FLT_MAX;
    return s;
}

// The same for values known to hold no NaN (the caller has their amax): no patching.
template <int FMT>
__device__ __forceinline__ uint32_t quantise4_finite(float x0, float x1, float x2, float x3, float s0, float s1, float s2, float s3) {
    uint32_t r = 0;
    r = cvt_pk<FMT, false>(x0 * s0, x1 * s1, r);
    return cvt_pk<FMT, true>(x2 * s2, x3 * s3, r);
}

// |x| bit pattern of a packed pair of bf16, per 16-bit half.  For bf16 (and
// fp32) the magnitude ordering equals the unsigned ordering of these bits, and
// every NaN pattern sorts above Inf, so an unsigned max propagates NaN.
__device__ __forceinline__ uint32_t abs_bf16x2(uint32_t w) { return w & 0x7fff7fffu; }

__device__ __forceinline__ uint32_t max_u16x2(uint32_t a, uint32_t b) {
    u16x2 r = __builtin_elementwise_max(__builtin_bit_cast(u16x2, a), __builtin_bit_cast(u16x2, b));
    return __builtin_bit_cast(uint32_t, r);
}

// fold a packed pair of bf16 magnitudes into fp32 bits of the larger one
__device__ __forceinline__ uint32_t fold_u16x2_to_f32bits(uint32_t w) {
    uint32_t lo = w & 0xffffu, hi = w >> 16;
    return (lo > hi ? lo : hi) << 16;
}

__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
        uint32_t o = (uint32_t)__shfl_xor((int)v, off, kWave);
        v = v > o ? v : o;
    }
    return v;
}

// Block-wide max of fp32 magnitude bits; result valid in thread 0.
// `red` is LDS scratch with one slot per wave.
__device__ __forceinline__ uint32_t block_max_u32(uint32_t v, uint32_t *red) {
    v = wave_max_u32(v);
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    const int nwave = (blockDim.x + kWave - 1) / kWave;
    if (lane == 0) red[wave] = v;
    __syncthreads();
    if (wave == 0) {
        v = lane < nwave ? red[lane] : 0u;
        v = wave_max_u32(v);
    }
    return v;
}

}  // namespace odl
