// Shared device helpers for the OMMX store / decode kernels (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/ommx_hip.h"

namespace ommx {

// bf16 bit pattern -> fp32 (exact).
__device__ __forceinline__ float bf16_to_f32(uint16_t b) {
    return __uint_as_float(static_cast<uint32_t>(b) << 16);
}

// fp32 -> bf16 bit pattern, round to nearest even; finite inputs only.
__device__ __forceinline__ uint16_t f32_to_bf16_rne(float x) {
    uint32_t u = __float_as_uint(x);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return static_cast<uint16_t>(u >> 16);
}

// fp32 -> bf16 as torch's `.to(torch.bfloat16)` does for any input: round to nearest even,
// infinities kept, NaN made quiet.
__device__ __forceinline__ uint16_t f32_to_bf16_any(float x) {
    const uint32_t u = __float_as_uint(x);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return static_cast<uint16_t>((u >> 16) | 0x0040u);
    return f32_to_bf16_rne(x);
}

__device__ __forceinline__ bool is_finite_f32(float x) {
    return (__float_as_uint(x) & 0x7F800000u) != 0x7F800000u;
}

// FP4 E2M1 magnitudes indexed by the low three code bits (exp<<1 | mant).
__device__ __forceinline__ float fp4_level(uint32_t code3) {
    // 0, .5, 1, 1.5, 2, 3, 4, 6
    const float m = (code3 & 1u) ? 1.5f : 1.0f;
    const uint32_t e = code3 >> 1;
    const float nrm = m * __uint_as_float((126u + e) << 23);   // m * 2^(e-1)
    return e == 0 ? 0.5f * static_cast<float>(code3 & 1u) : nrm;
}

void set_error(const char* msg);

}  // namespace ommx
