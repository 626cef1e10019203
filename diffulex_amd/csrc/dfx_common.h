// Shared helpers for the gfx950 kernels: status codes, vector types, bf16 bit helpers.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/diffulex_amd.h"

#define DFX_HD __host__ __device__ __forceinline__
#define DFX_D __device__ __forceinline__

namespace dfx {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

DFX_HD float bf16_bits_to_f32(uint16_t b) {
    union { uint32_t u; float f; } c;
    c.u = static_cast<uint32_t>(b) << 16;
    return c.f;
}

// Round-to-nearest-even fp32 -> bf16 bits (NaN kept quiet).
DFX_HD uint16_t f32_to_bf16_bits(float f) {
    union { uint32_t u; float f; } c;
    c.f = f;
    if ((c.u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((c.u >> 16) | 0x40u);
    const uint32_t lsb = (c.u >> 16) & 1u;
    return static_cast<uint16_t>((c.u + 0x7fffu + lsb) >> 16);
}

static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

static inline int launch_status() {
    return hipGetLastError() == hipSuccess ? DFX_OK : DFX_ERR_LAUNCH;
}

}  // namespace dfx
