// Issue-rate calibration of the vector ALU: what one wave64 instruction of a given kind costs on
// this GPU when every SIMD is kept full, measured by a loop of independent chains of that
// instruction.  The assignment kernel's selection (v_and_or_b32, v_min3_i32, v_med3_i32) is priced
// with these rates; v_fma_f32 is the rate the published fp32 vector peak is made of.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace vq {

constexpr int kCalibChains = 8;   // independent dependency chains per lane
constexpr int kCalibUnroll = 4;   // instructions per chain and loop iteration

// OP 0: v_fma_f32, 1: v_min3_i32, 2: v_med3_i32, 3: v_and_or_b32, 4: v_add_u32.
// Grid: any; every wave issues iters * kCalibChains * kCalibUnroll instructions of the kind.
template <int OP>
__global__ void __launch_bounds__(256) k_calib_valu(int iters, uint32_t seed, uint32_t *__restrict__ sink) {
    uint32_t a[kCalibChains];
#pragma unroll
    for (int u = 0; u < kCalibChains; ++u) a[u] = seed + threadIdx.x * 2654435761u + u;
    uint32_t b = seed ^ 0x3f800001u, c = seed | 0x00ffff00u;
    asm volatile("" : "+v"(b), "+v"(c));  // operands in vector registers, opaque to the compiler
    for (int i = 0; i < iters; ++i) {
#pragma unroll
        for (int r = 0; r < kCalibUnroll; ++r) {
#pragma unroll
            for (int u = 0; u < kCalibChains; ++u) {
                if constexpr (OP == 0)
                    asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(a[u]) : "v"(b), "v"(c));
                else if constexpr (OP == 1)
                    asm volatile("v_min3_i32 %0, %0, %1, %2" : "+v"(a[u]) : "v"(b), "v"(c));
                else if constexpr (OP == 2)
                    asm volatile("v_med3_i32 %0, %0, %1, %2" : "+v"(a[u]) : "v"(b), "v"(c));
                else if constexpr (OP == 3)
                    asm volatile("v_and_or_b32 %0, %0, %1, %2" : "+v"(a[u]) : "v"(b), "v"(c));
                else
                    asm volatile("v_add_u32 %0, %0, %1" : "+v"(a[u]) : "v"(b));
            }
        }
    }
    uint32_t x = 0;
#pragma unroll
    for (int u = 0; u < kCalibChains; ++u) x ^= a[u];
    if (x == 0x12345677u) sink[0] = x;  // keeps the chains alive; practically never taken
}

// ---- do matrix and vector instructions of a SIMD overlap? ---------------------------------------
// MODE 0: workgroups of 8 waves; waves 0-3 issue chains of v_mfma_f32_32x32x16_bf16, waves 4-7
//         chains of v_min3_i32 (n_mfma / n_valu instructions per wave; 0 = the wave leaves at once).
//         The waves of a workgroup are dealt to the four SIMDs of its compute unit in turn, so with 4
//         workgroups per compute unit every SIMD holds 4 waves of each kind: the two kinds come from
//         different waves of the same SIMD.  (Kinds by workgroup index would not do: workgroups are
//         dealt round-robin to the 8 XCDs, and even and odd ones never meet.)  Every wave counts
//         itself in where[kind * 4 + its SIMD's number], which the host checks to be balanced.
// MODE 1: every wave issues both, interleaved in one instruction stream: per loop iteration 4
//         matrix instructions on 4 independent accumulators and 4 * VPM v_min3_i32 on 8 independent
//         chains (nothing depends on anything of the other kind).
// Timed alone (the other count 0) and together: together = max(alone, alone) means the two pipes
// run side by side, together = sum means they take turns.
typedef float calib_f16 __attribute__((ext_vector_type(16)));
typedef __bf16 calib_bf8 __attribute__((ext_vector_type(8)));

template <int MODE, int VPM>
__global__ void __launch_bounds__(MODE == 0 ? 512 : 256) k_calib_overlap(int n_mfma, int n_valu, uint32_t seed,
                                                                         uint32_t *__restrict__ sink,
                                                                         uint32_t *__restrict__ where) {
    uint32_t a[kCalibChains];
#pragma unroll
    for (int u = 0; u < kCalibChains; ++u) a[u] = seed + threadIdx.x * 2654435761u + u;
    uint32_t b = seed ^ 0x3f800001u, c = seed | 0x00ffff00u;
    asm volatile("" : "+v"(b), "+v"(c));
    calib_f16 acc[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int t = 0; t < 16; ++t) acc[u][t] = 0.0f;
    typedef uint32_t calib_u4 __attribute__((ext_vector_type(4)));
    calib_u4 opa = {0x3f803f80u, 0x3f803f80u, 0u, 0u}, opb = {0x3f803f80u, 0u, 0x3f803f80u, 0u};
    asm volatile("" : "+v"(opa), "+v"(opb));
    const calib_bf8 A = __builtin_bit_cast(calib_bf8, opa), B = __builtin_bit_cast(calib_bf8, opb);
    if constexpr (MODE == 0) {
        const int kind = (int)(threadIdx.x >> 8);  // waves 0-3: matrix, waves 4-7: vector
        if ((threadIdx.x & 63) == 0) {
            // HW_ID (hardware register 4), bits 5:4: the SIMD this wave runs on
            const uint32_t simd = __builtin_amdgcn_s_getreg(4 | (4 << 6) | (1 << 11));
            atomicAdd(where + kind * 4 + (simd & 3u), 1u);
        }
        if (kind == 0) {
            for (int i = 0; i < n_mfma; i += 4) {
#pragma unroll
                for (int u = 0; u < 4; ++u) acc[u] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(A, B, acc[u], 0, 0, 0);
            }
        } else {
            for (int i = 0; i < n_valu; i += kCalibChains * kCalibUnroll) {
#pragma unroll
                for (int r = 0; r < kCalibUnroll; ++r)
#pragma unroll
                    for (int u = 0; u < kCalibChains; ++u)
                        asm volatile("v_min3_i32 %0, %0, %1, %2" : "+v"(a[u]) : "v"(b), "v"(c));
            }
        }
    } else {
        // one stream: n_mfma counts the matrix instructions; n_valu != 0 switches the vector ones on,
        // n_mfma == 0 with n_valu != 0 runs the vector instructions of n_valu / VPM loop steps alone
        const bool with_m = n_mfma > 0, with_v = n_valu > 0;
        const int steps = with_m ? n_mfma / 4 : n_valu / (4 * VPM);
        if (with_m && with_v) {
            for (int i = 0; i < steps; ++i) {
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    acc[u] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(A, B, acc[u], 0, 0, 0);
#pragma unroll
                    for (int v = 0; v < VPM; ++v)
                        asm volatile("v_min3_i32 %0, %0, %1, %2" : "+v"(a[(u * VPM + v) % kCalibChains]) : "v"(b), "v"(c));
                }
            }
        } else if (with_m) {
            for (int i = 0; i < steps; ++i) {
#pragma unroll
                for (int u = 0; u < 4; ++u) acc[u] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(A, B, acc[u], 0, 0, 0);
            }
        } else {
            for (int i = 0; i < steps; ++i) {
#pragma unroll
                for (int u = 0; u < 4; ++u)
#pragma unroll
                    for (int v = 0; v < VPM; ++v)
                        asm volatile("v_min3_i32 %0, %0, %1, %2" : "+v"(a[(u * VPM + v) % kCalibChains]) : "v"(b), "v"(c));
            }
        }
    }
    uint32_t x = 0;
#pragma unroll
    for (int u = 0; u < kCalibChains; ++u) x ^= a[u];
    float f = 0.0f;
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int t = 0; t < 16; ++t) f += acc[u][t];
    if (x == 0x12345677u && f == 1.2345f) sink[0] = x;  // keeps both kinds alive; practically never taken
}

}  // namespace vq
