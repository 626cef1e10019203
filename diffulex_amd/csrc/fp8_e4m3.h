// OCP FP8 E4M3 (e4m3fn) conversions in integer arithmetic, usable on host and device.
//
// The store path quantises with these (not with the hardware convert) so that the
// result is defined bit for bit by this file:
//     code = rne_e4m3fn( clamp( x / scale, -448, +448 ) )
// with an IEEE fp32 division.
#pragma once

#include "dfx_common.h"

namespace dfx {

// fp32 -> e4m3fn code, round to nearest even.  Magnitudes that round above 448
// give the NaN code, like a non-saturating library cast; quantise_e4m3 clamps first.
DFX_HD uint8_t f32_to_e4m3fn(float f) {
    union { uint32_t u; float f; } c;
    c.f = f;
    const uint32_t sign = (c.u >> 24) & 0x80u;
    const uint32_t mag = c.u & 0x7fffffffu;
    if (mag > 0x7f800000u) return static_cast<uint8_t>(sign | 0x7fu);
    uint32_t code;
    if (mag >= 0x3c800000u) {  // >= 2^-6: normal e4m3 number
        const uint32_t lsb = (mag >> 20) & 1u;
        const uint32_t r = (mag + 0x7ffffu + lsb) >> 20;  // (exp8 << 3) | m3, carry into exp
        code = r - ((127u - 7u) << 3);
        if (code > 0x7eu) code = 0x7fu;
    } else {  // multiples of 2^-9; the scaling is exact, rint is RNE
        union { uint32_t u; float f; } m;
        m.u = mag;
#if defined(__HIP_DEVICE_COMPILE__)
        code = static_cast<uint32_t>(__builtin_rintf(m.f * 512.0f));
#else
        code = static_cast<uint32_t>(__builtin_nearbyintf(m.f * 512.0f));
#endif
    }
    return static_cast<uint8_t>(sign | code);
}

DFX_HD float e4m3fn_to_f32(uint8_t code) {
    const uint32_t e = (code >> 3) & 0xfu;
    const uint32_t m = code & 0x7u;
    union { uint32_t u; float f; } c;
    if (e == 0) {
        c.f = static_cast<float>(m) * 0.001953125f;  // m * 2^-9
    } else if (e == 15 && m == 7) {
        c.u = 0x7fc00000u;
    } else {
        c.u = ((e + 120u) << 23) | (m << 20);
    }
    if (code & 0x80u) c.u |= 0x80000000u;
    return c.f;
}

DFX_HD uint8_t quantise_e4m3(float x, float scale) {
    float y = x / scale;
    if (y == y) y = y > 448.0f ? 448.0f : (y < -448.0f ? -448.0f : y);
    return f32_to_e4m3fn(y);
}

DFX_D uint32_t quantise_pair(uint32_t two_bf16, float scale) {
    const uint8_t lo = quantise_e4m3(bf16_bits_to_f32(static_cast<uint16_t>(two_bf16 & 0xffffu)), scale);
    const uint8_t hi = quantise_e4m3(bf16_bits_to_f32(static_cast<uint16_t>(two_bf16 >> 16)), scale);
    return static_cast<uint32_t>(lo) | (static_cast<uint32_t>(hi) << 8);
}

// 8 bf16 (16 bytes) -> 8 e4m3 codes (8 bytes)
DFX_D u32x2 quantise8(u32x4 v, float scale) {
    u32x2 r;
    r.x = quantise_pair(v.x, scale) | (quantise_pair(v.y, scale) << 16);
    r.y = quantise_pair(v.z, scale) | (quantise_pair(v.w, scale) << 16);
    return r;
}

}  // namespace dfx
