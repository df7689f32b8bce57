// Measurement aids for bench.py: not part of the FP8 library's ABI (a library of their own, libodl_probe.so).
//
//   odl_probe_mfma_loop   : the FP8 MFMA of the GEMM kernels (32x32x64, 16 accumulator tiles per wave, one wave per
//                           SIMD, nothing but registers) issued back to back, with operands that are all zero or
//                           spread like quantised Gaussian data: the matrix pipe's rate with no memory system behind
//                           it, and how it depends on what the operands hold.
//   odl_probe_mfma_loop_scaled : the same with the block-scaled form of the instruction (MXFP8).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../optimus-dl_amd/csrc/gemm_common.h"

namespace {

__device__ __forceinline__ uint32_t mix(uint32_t x) {
    x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
    return x;
}

// four E4M3 codes with random sign and mantissa and an exponent field of 3..9 (values of 2^-4 .. 2^2 times 1.x):
// roughly what a Gaussian tensor scaled to the format's range holds
__device__ __forceinline__ uint32_t gaussian_like_codes(uint32_t seed) {
    uint32_t w = 0;
#pragma unroll
    for (int b = 0; b < 4; ++b) {
        const uint32_t h = mix(seed * 4 + b);
        const uint32_t code = ((h & 1u) << 7) | ((3u + (h >> 1) % 7u) << 3) | ((h >> 8) & 7u);
        w |= code << (8 * b);
    }
    return w;
}

// SCALED: the block-scaled form of the instruction (an E8M0 scale byte per lane and operand, as the MXFP8 GEMM issues it)
template <bool SCALED>
__global__ __launch_bounds__(256) void mfma_loop_kernel(int random_operands, int iters, float *sink, uint64_t *cycles) {
    using namespace odl;
    // scale bytes 119 .. 134 (2^-8 .. 2^7) when the operands are random, 127 (1.0) otherwise
    const int sc = random_operands ? (int)(119u + (mix(blockIdx.x * 256 + threadIdx.x) & 15u)) : 127;
    v8i a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            const uint32_t seed = ((blockIdx.x * 256 + threadIdx.x) * 8 + i) * 16 + r;
            a[i][r] = random_operands ? (int)gaussian_like_codes(seed) : 0;
            b[i][r] = random_operands ? (int)gaussian_like_codes(seed ^ 0x9e3779b9u) : 0;
        }
    v16f acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
    const uint64_t c0 = clock64(), t0 = wall_clock64();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            if constexpr (SCALED)
                acc[i / 4][i % 4] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b[i % 4], a[i / 4], acc[i / 4][i % 4], 0, 0, 0, sc, 0, sc ^ 3);
            else
                acc[i / 4][i % 4] = mfma_32x32x64<0, 0>(b[i % 4], a[i / 4], acc[i / 4][i % 4]);
        }
    }
    const uint64_t c1 = clock64(), t1 = wall_clock64();
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) s += acc[i][j][r];
    if (s == 123.456f) sink[0] = s;                      // keeps the accumulators alive
    if (threadIdx.x == 0) {
        cycles[2 * blockIdx.x] = c1 - c0;
        cycles[2 * blockIdx.x + 1] = t1 - t0;
    }
}

}  // namespace

// blocks x 4 waves x iters x 16 MFMAs of 2 * 32 * 32 * 64 flop.  cycles_dev: [blocks][2] = {shader clocks, 100 MHz ticks}
// spent in the loop by each block's first wave.
extern "C" int odl_probe_mfma_loop(int random_operands, int iters, int blocks, float *sink_dev, uint64_t *cycles_dev, void *stream) {
    if (iters < 1 || blocks < 1 || !sink_dev || !cycles_dev) return -1;
    hipLaunchKernelGGL(mfma_loop_kernel<false>, dim3(blocks), dim3(256), 0, reinterpret_cast<hipStream_t>(stream), random_operands, iters,
                       sink_dev, cycles_dev);
    return (int)hipGetLastError();
}

// The same loop with the block-scaled form of the instruction.
extern "C" int odl_probe_mfma_loop_scaled(int random_operands, int iters, int blocks, float *sink_dev, uint64_t *cycles_dev, void *stream) {
    if (iters < 1 || blocks < 1 || !sink_dev || !cycles_dev) return -1;
    hipLaunchKernelGGL(mfma_loop_kernel<true>, dim3(blocks), dim3(256), 0, reinterpret_cast<hipStream_t>(stream), random_operands, iters,
                       sink_dev, cycles_dev);
    return (int)hipGetLastError();
}
