// Shared pieces of the FP8 GEMM kernels: argument block, LDS swizzle, the MFMA
// wrapper and the scaling epilogue.
#pragma once

#include "common.h"

namespace odl {


typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

struct GemmArgs {
    const uint8_t *a, *b;
    void *c;
    const float *sa, *sb;
    const void *bias;
    int64_t M, N, K;
    int sa_vec, sb_vec;          // 0 = one value, 1 = one per row of A / B
    int out_dtype;               // bias, when present, is fp32
    int accumulate = 0;          // C = C + product (one rounding) instead of C = product; not in the streaming kernel
    int tiles_m, tiles_n;
    int ta = 0, tb = 0;          // operand stored [K, M] / [K, N] (contraction index slow); streaming kernel only
    // streaming kernel only: splits > 1 cuts K into `splits` runs of `split_steps` 128-byte steps (an even number;
    // the last run may be shorter) and `c` is an fp32 workspace [splits, M, N] of unscaled partial results
    int splits = 1, split_steps = 0;
    // streaming kernel only, measurement aid: when set, the first wave of block 0 writes {shader-clock counter,
    // 100 MHz counter} on entry and on exit (4 x uint64): the average clock the board granted this launch
    unsigned long long *clock_out = nullptr;
    // streaming kernel only: block scales of A and B (E8M0 bytes, one per 32 K-bytes), stored K-step-major:
    // dword [K / 128][rows] = the 4 scale bytes of a row in one 128-byte K step.  Set: the MFMAs apply them.
    const uint8_t *mx_sa = nullptr, *mx_sb = nullptr;
};

// A contraction that runs over several operand pairs (streaming kernel only):
// C = sum_s (A_s . B_s^T) * (sa_s * sb_s), A_s [M, k[s]] and B_s [N, k[s]] with the contraction index fast, one scale per
// operand.  Passed beside GemmArgs, whose a, b, sa, sb and K are then not read.
struct GemmPairs {
    int count = 0;
    int k[4] = {0, 0, 0, 0};
    const uint8_t *a[4] = {nullptr, nullptr, nullptr, nullptr}, *b[4] = {nullptr, nullptr, nullptr, nullptr};
    const float *sa[4] = {nullptr, nullptr, nullptr, nullptr}, *sb[4] = {nullptr, nullptr, nullptr, nullptr};
};

__device__ __forceinline__ int swz(int row) { return (row ^ (row >> 3)) & 7; }

// D[i][j] += sum_k first[i][k] * second[j][k]; lane l supplies row l%32 and 32 K-bytes
// of both operands (which 32 does not matter as long as both operands use the same ones;
// the instruction itself takes registers 0..3 as K [16 g, +16) and 4..7 as K [32 + 16 g, +16),
// g = l/32, which only the block-scaled kernels in mx.hip depend on).  F1 / F2: 0 = E4M3, 1 = E5M2.
template <int F1, int F2>
__device__ __forceinline__ v16f mfma_32x32x64(v8i first, v8i second, v16f acc) {
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(first, second, acc, F1, F2, 0, 0, 0, 0);
}

// Epilogue for one 32x32 accumulator tile in the swapped layout: this lane holds
// row m and columns n_base + 8*q + {0..3}, q = 0..3, in acc[4q .. 4q+3].
// value = acc * (sa_inv[m] * sb_inv[n]) (+ bias[n]), each step rounded to fp32,
// then one rounding to the output type.  sa/sb are read with stride 0 (one value)
// or 1 (one per row / column), which removes the per-element branch.
// INTERIOR: the whole block tile is inside the matrix and N % 4 == 0, so no
// bounds checks and vector stores throughout.
template <bool OUT_BF16, bool INTERIOR>
__device__ __forceinline__ void store_tile(const GemmArgs &g, const v16f &acc, int64_t m, int64_t n_base) {
    if (!INTERIOR && m >= g.M) return;
    const float sa = g.sa[m * g.sa_vec];
    const float *bias = reinterpret_cast<const float *>(g.bias);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const int64_t n = n_base + 8 * q;
        if (!INTERIOR && n >= g.N) continue;
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int64_t ne = (INTERIOR || n + e < g.N) ? n + e : g.N - 1;
            const float s = sa * g.sb[ne * g.sb_vec];
            v[e] = acc[4 * q + e] * s;
            if (bias) v[e] = v[e] + bias[ne];
        }
        if constexpr (OUT_BF16) {
            uint16_t *c = reinterpret_cast<uint16_t *>(g.c) + m * g.N + n;
            if (INTERIOR || (n + 3 < g.N && (g.N & 3) == 0)) {
                if (g.accumulate) {
                    const u32x2 old = *reinterpret_cast<const u32x2 *>(c);
                    v[0] = v[0] + bits_to_float(old.x << 16); v[1] = v[1] + bits_to_float(old.x & 0xffff0000u);
                    v[2] = v[2] + bits_to_float(old.y << 16); v[3] = v[3] + bits_to_float(old.y & 0xffff0000u);
                }
                u32x2 pk = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
                *reinterpret_cast<u32x2 *>(c) = pk;
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (n + e < g.N) c[e] = (uint16_t)f32_to_bf16_bits(g.accumulate ? v[e] + bits_to_float((uint32_t)c[e] << 16) : v[e]);
            }
        } else {
            float *c = reinterpret_cast<float *>(g.c) + m * g.N + n;
            if (INTERIOR || (n + 3 < g.N && (g.N & 3) == 0)) {
                if (g.accumulate) {
                    const float4 old = *reinterpret_cast<const float4 *>(c);
                    v[0] = v[0] + old.x; v[1] = v[1] + old.y; v[2] = v[2] + old.z; v[3] = v[3] + old.w;
                }
                *reinterpret_cast<float4 *>(c) = float4{v[0], v[1], v[2], v[3]};
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (n + e < g.N) c[e] = g.accumulate ? v[e] + c[e] : v[e];
            }
        }
    }
}


// ---------------------------------------------------------------- staged epilogue
// Output path for a wave tile that lies wholly inside the matrix.  The MFMA leaves
// each lane with 4-column fragments of 32 different rows, which as direct stores
// touch 32 cache lines per instruction.  Instead every slab of 32 rows x (TNS*32)
// columns of the wave tile is scaled, rounded and written to a private LDS region
// (rows padded by 16 bytes), then read back 16 bytes per lane along the rows and
// stored so that a wave instruction writes whole 128-byte lines.
//   value = acc * (sa_inv[m] * sb_inv[n]) (+ bias[n]); fp32 steps, one final rounding.
// Requires: N % 8 == 0, n_wave % 8 == 0, 16-byte aligned output / scale vectors / bias,
// and that nobody else touches `wave_lds` (staged_epilogue_bytes<> bytes).  LDS
// operations of one wave execute in order, so write -> read -> next write needs no barrier.
template <bool OUT_BF16, int TNS>
constexpr int staged_epilogue_bytes() { return 32 * (TNS * 32 * (OUT_BF16 ? 2 : 4) + 16); }

template <bool OUT_BF16, int TM, int TN, int TNS>
__device__ __forceinline__ void epilogue_staged(const GemmArgs &g, v16f (&acc)[TM][TN], uint8_t *wave_lds,
                                                int64_t m_wave, int64_t n_wave, int lane) {
    static_assert(TN % TNS == 0, "slab width must divide the wave tile");
    constexpr int ESZ = OUT_BF16 ? 2 : 4;
    constexpr int ROW_BYTES = TNS * 32 * ESZ, PITCH = ROW_BYTES + 16;
    constexpr int LPR = ROW_BYTES / 16;            // lanes that cover one slab row with 16 bytes each
    constexpr int RPI = 64 / LPR;                  // rows per store instruction
    const int lr = lane % 32, lg = lane / 32;
    const bool vec = g.sa_vec | g.sb_vec | (g.bias != nullptr);
    const float s_tensor = g.sa[0] * g.sb[0];
    const float *bias = reinterpret_cast<const float *>(g.bias);
    uint8_t *out = reinterpret_cast<uint8_t *>(g.c);
#pragma unroll
    for (int t = 0; t < TM; ++t) {
        float sa = 1.0f;
        if (vec) sa = g.sa[(m_wave + 32 * t + lr) * g.sa_vec];
#pragma unroll
        for (int us = 0; us < TN; us += TNS) {
#pragma unroll
            for (int uu = 0; uu < TNS; ++uu) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int col = 32 * uu + 8 * q + 4 * lg;    // first of this lane's 4 columns inside the slab
                    float v[4];
                    if (vec) {
                        const int64_t n = n_wave + 32 * us + col;
                        float sb[4] = {g.sb[0], g.sb[0], g.sb[0], g.sb[0]};
                        if (g.sb_vec) { const float4 t4 = *reinterpret_cast<const float4 *>(g.sb + n); sb[0] = t4.x; sb[1] = t4.y; sb[2] = t4.z; sb[3] = t4.w; }
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] = acc[t][us + uu][4 * q + e] * (sa * sb[e]);
                        if (bias) { const float4 b4 = *reinterpret_cast<const float4 *>(bias + n); v[0] = v[0] + b4.x; v[1] = v[1] + b4.y; v[2] = v[2] + b4.z; v[3] = v[3] + b4.w; }
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] = acc[t][us + uu][4 * q + e] * s_tensor;
                    }
                    uint8_t *dst = wave_lds + lr * PITCH + col * ESZ;
                    if constexpr (OUT_BF16) *reinterpret_cast<u32x2 *>(dst) = u32x2{pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
                    else *reinterpret_cast<float4 *>(dst) = float4{v[0], v[1], v[2], v[3]};
                }
            }
#pragma unroll
            for (int i = 0; i < 32 / RPI; ++i) {
                const int r = i * RPI + lane / LPR, chunk = lane % LPR;
                const u32x4 val = *reinterpret_cast<const u32x4 *>(wave_lds + r * PITCH + chunk * 16);
                uint8_t *dst = out + ((m_wave + 32 * t + r) * g.N + n_wave + 32 * us) * ESZ + chunk * 16;
                // non-temporal: the output is not read by the next kernel, and written through the memory-side
                // cache it would still be draining to HBM while the next (memory-bound) kernel runs
                __builtin_nontemporal_store(val, reinterpret_cast<u32x4 *>(dst));
            }
        }
    }
}

// The same output path for C = C + product: the slab is staged as fp32 whatever the output type (the sum is rounded
// once), TNS sub-tiles wide (32 * (TNS * 128 + 16) bytes of `wave_lds`), and a lane that has read back four values of
// a row adds the four old values of C, which it requested one slab earlier (the loads of slab k + 1 are in flight
// while slab k is scaled, staged and stored).  Ordinary stores: what is accumulated into is read again.
template <bool OUT_BF16, int TM, int TN, int TNS>
__device__ __forceinline__ void epilogue_staged_accumulate(const GemmArgs &g, v16f (&acc)[TM][TN], uint8_t *wave_lds,
                                                           int64_t m_wave, int64_t n_wave, int lane) {
    static_assert(TN % TNS == 0, "slab width must divide the wave tile");
    constexpr int ESZ = OUT_BF16 ? 2 : 4;
    constexpr int ROW_BYTES = TNS * 32 * 4, PITCH = ROW_BYTES + 16;
    constexpr int LPR = ROW_BYTES / 16;            // lanes that cover one slab row with four floats each
    constexpr int RPI = 64 / LPR, NI = 32 / RPI;   // rows per instruction, instructions per slab
    constexpr int SLABS = TM * (TN / TNS);
    const int lr = lane % 32, lg = lane / 32;
    const bool vec = g.sa_vec | g.sb_vec | (g.bias != nullptr);
    const float s_tensor = g.sa[0] * g.sb[0];
    const float *bias = reinterpret_cast<const float *>(g.bias);
    uint8_t *out = reinterpret_cast<uint8_t *>(g.c);
    auto c_ptr = [&](int slab, int i) -> uint8_t * {   // where this lane's four values of instruction i of a slab live
        const int t = slab / (TN / TNS), us = (slab % (TN / TNS)) * TNS;
        const int r = i * RPI + lane / LPR, chunk = lane % LPR;
        return out + ((m_wave + 32 * t + r) * g.N + n_wave + 32 * us + 4 * chunk) * ESZ;
    };
    auto fetch_old = [&](float (&old)[NI][4], int slab) {
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            if constexpr (OUT_BF16) {
                const u32x2 o = *reinterpret_cast<const u32x2 *>(c_ptr(slab, i));
                old[i][0] = bits_to_float(o.x << 16); old[i][1] = bits_to_float(o.x & 0xffff0000u);
                old[i][2] = bits_to_float(o.y << 16); old[i][3] = bits_to_float(o.y & 0xffff0000u);
            } else {
                const float4 o = *reinterpret_cast<const float4 *>(c_ptr(slab, i));
                old[i][0] = o.x; old[i][1] = o.y; old[i][2] = o.z; old[i][3] = o.w;
            }
        }
    };
    float old[2][NI][4];
    fetch_old(old[0], 0);
#pragma unroll
    for (int slab = 0; slab < SLABS; ++slab) {
        const int t = slab / (TN / TNS), us = (slab % (TN / TNS)) * TNS;
        if (slab + 1 < SLABS) fetch_old(old[(slab + 1) & 1], slab + 1);
        float sa = 1.0f;
        if (vec) sa = g.sa[(m_wave + 32 * t + lr) * g.sa_vec];
#pragma unroll
        for (int uu = 0; uu < TNS; ++uu) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int col = 32 * uu + 8 * q + 4 * lg;    // first of this lane's 4 columns inside the slab
                float v[4];
                if (vec) {
                    const int64_t n = n_wave + 32 * us + col;
                    float sb[4] = {g.sb[0], g.sb[0], g.sb[0], g.sb[0]};
                    if (g.sb_vec) { const float4 t4 = *reinterpret_cast<const float4 *>(g.sb + n); sb[0] = t4.x; sb[1] = t4.y; sb[2] = t4.z; sb[3] = t4.w; }
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = acc[t][us + uu][4 * q + e] * (sa * sb[e]);
                    if (bias) { const float4 b4 = *reinterpret_cast<const float4 *>(bias + n); v[0] = v[0] + b4.x; v[1] = v[1] + b4.y; v[2] = v[2] + b4.z; v[3] = v[3] + b4.w; }
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = acc[t][us + uu][4 * q + e] * s_tensor;
                }
                *reinterpret_cast<float4 *>(wave_lds + lr * PITCH + col * 4) = float4{v[0], v[1], v[2], v[3]};
            }
        }
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const int r = i * RPI + lane / LPR, chunk = lane % LPR;
            const float4 val = *reinterpret_cast<const float4 *>(wave_lds + r * PITCH + chunk * 16);
            const float (&o)[4] = old[slab & 1][i];
            const float w[4] = {o[0] + val.x, o[1] + val.y, o[2] + val.z, o[3] + val.w};
            if constexpr (OUT_BF16) *reinterpret_cast<u32x2 *>(c_ptr(slab, i)) = u32x2{pack_bf16x2(w[0], w[1]), pack_bf16x2(w[2], w[3])};
            else *reinterpret_cast<float4 *>(c_ptr(slab, i)) = float4{w[0], w[1], w[2], w[3]};
        }
    }
}

// launchers implemented in gemm_tiled.hip / gemm_pipe.hip / gemm_stream.hip (fa, fb: odl_fp8_format of A and B)
void launch_gemm_tiled(int variant, int fa, int fb, const GemmArgs &g, hipStream_t stream);
void launch_gemm_pipe(int fa, int fb, const GemmArgs &g, int num_cus, hipStream_t stream);
bool gemm_stream_accepts(const GemmArgs &g);
void launch_gemm_stream(int fa, int fb, const GemmArgs &g, int num_cus, hipStream_t stream);
bool gemm_stream_accepts_pairs(const GemmArgs &g, const GemmPairs &pairs);
void launch_gemm_stream_pairs(int fa, int fb, const GemmArgs &g, const GemmPairs &pairs, int num_cus, hipStream_t stream);
// gemm_fp8.hip: hands the calling thread's clock-probe record (odl_fp8_gemm_set_clock_probe), if any, to a streaming launch
void attach_clock_probe(GemmArgs &g);
// gemm_fp8.hip: out = (sum of the `splits` fp32 partial results in `workspace`, in split order) * (sa x sb) (+ bias), one rounding
void launch_splitk_reduce(const float *workspace, int splits, int64_t M, int64_t N, const float *sa, int sa_vec, const float *sb, int sb_vec,
                          const float *bias, void *c, int out_dtype, int accumulate, hipStream_t stream);

}  // namespace odl
