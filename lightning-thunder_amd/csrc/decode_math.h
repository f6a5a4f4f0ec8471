// Arithmetic that the decode-step kernels (decode_glue.hip) and the epilogues of the decode-shape matmul kernels
// share, so that a step computes the same bits whichever of the two does the work.  bf16 in and out, fp32
// arithmetic; self-contained.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace nf4x {

__device__ __forceinline__ float bf16_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

// round to nearest even; NaN is quieted
__device__ __forceinline__ uint32_t f32_to_bf16(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
    u += 0x7fffu + ((u >> 16) & 1u);
    return u >> 16;
}

__device__ __forceinline__ float round_bf16(float f) { return bf16_to_f32(f32_to_bf16(f)); }

// SiLU(gate) * up with the roundings of a bf16 SiLU followed by a bf16 product: bf16(bf16(silu(g)) * u), as bits
__device__ __forceinline__ uint32_t silu_mul_bf16(float g, float u) {
    return f32_to_bf16(round_bf16(g / (1.0f + __expf(-g))) * u);
}

// residual add: bf16(x + d)
__device__ __forceinline__ float resid_add(float x, float d) { return round_bf16(x + d); }

}  // namespace nf4x
