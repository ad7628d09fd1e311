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

}  // namespace vq
