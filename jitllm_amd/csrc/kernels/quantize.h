// Activation quantizer: f32 -> int8 with one f32 scale per 32 elements and one
// integer sum per 16, bit for bit what the reference's PackActivationsInto
// produces (jit/gpu/kernels/pack.go:474-525; device twin elem.go:76-170):
//
//   amax over the block's window (32..256 elements, clamped to the vector),
//   d = amax / 127 and inv = 1 / d, both correctly rounded f32 divisions,
//   q = round-half-away-from-zero(f32(x * inv)),
//   as[b] = d, sum16[h] = sum of q over 16 elements (stored as f32, exact).
//
// One thread owns one 16-element half-block; the window's amax is combined
// across the 2*per lanes that share it with cross-lane xor shuffles, so a
// window never leaves a 16-lane row.
#pragma once
#include "common.h"

#pragma clang fp contract(off)

// |v| as an integer bit pattern: comparing these orders the magnitudes exactly
// as the reference's sign-cleared integer compare does (NaNs included).
__device__ __forceinline__ u32 abs_bits(float v) { return __float_as_uint(v) & 0x7FFFFFFFu; }

// amax bits over this thread's 16 values (all zero when the half-block is past
// the end of the vector).
__device__ __forceinline__ u32 half_block_amax(const f32x4 v[4]) {
    u32 m = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        m = max(m, abs_bits(v[i].x));
        m = max(m, abs_bits(v[i].y));
        m = max(m, abs_bits(v[i].z));
        m = max(m, abs_bits(v[i].w));
    }
    return m;
}

// Combine amax over the 2*per consecutive lanes of a window (per = window/32,
// a power of two <= 8).  Lanes of one window are aligned to 2*per.
__device__ __forceinline__ u32 window_amax(u32 m, int per) {
    for (int x = 1; x < 2 * per; x <<= 1) m = max(m, (u32)__shfl_xor((int)m, x, JL_WAVE));
    return m;
}

// Quantize 16 values with the window's amax.  q[4] = 16 int8 packed little
// endian; returns the scale d and the integer sum.
__device__ __forceinline__ void quantize_half_block(const f32x4 v[4], u32 amax_bits, u32 q[4],
                                                    float& d_out, i32& sum_out) {
    float amax = __uint_as_float(amax_bits);
    float d = amax / 127.0f;
    float inv = d != 0.0f ? 1.0f / d : 0.0f;
    i32 sum = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        i32 a = (i32)__builtin_roundf(v[i].x * inv);
        i32 b = (i32)__builtin_roundf(v[i].y * inv);
        i32 c = (i32)__builtin_roundf(v[i].z * inv);
        i32 e = (i32)__builtin_roundf(v[i].w * inv);
        q[i] = (u32)(a & 0xFF) | ((u32)(b & 0xFF) << 8) | ((u32)(c & 0xFF) << 16) | ((u32)e << 24);
        sum += a + b + c + e;
    }
    d_out = d;
    sum_out = sum;
}
