// Activation quantizer: f32 -> int8 with one f32 scale per 32 elements and one
// integer sum per 16, bit for bit what the reference's PackActivationsInto
// produces (jit/gpu/kernels/pack.go:474-525; device twin elem.go:76-170):
//
//   amax over the block's window (32..256 elements, clamped to the vector),
//   d = amax / 127 and inv = 1 / d, both correctly rounded f32 divisions,
//   q = round-half-away-from-zero(f32(x * inv)),
//   as[b] = d, sum16[h] = sum of q over 16 elements (stored as f32, exact).
//
// One thread owns four consecutive elements.  A 16-element half-block is a
// quad of lanes, a 32-element block eight lanes, a window 8*per lanes, so the
// window's amax and the half-block sums are combined with DPP lane moves.
#pragma once
#include "common.h"

#pragma clang fp contract(off)

// |v| as an integer bit pattern: comparing these orders the magnitudes exactly
// as the reference's sign-cleared integer compare does.
__device__ __forceinline__ u32 abs_bits(float v) { return __float_as_uint(v) & 0x7FFFFFFFu; }

template <int CTRL>
__device__ __forceinline__ u32 dpp_max_u32(u32 m) {
    return max(m, (u32)dpp_i32<CTRL, 0xf>(0, (i32)m));
}

// amax bits over the 8*per consecutive lanes of a window (per = window/32, a power
// of two <= 8); lanes of one window are aligned to 8*per.
__device__ __forceinline__ u32 window_amax(u32 m, int per) {
    m = dpp_max_u32<JL_DPP_QUAD_XOR1>(m);
    m = dpp_max_u32<JL_DPP_QUAD_XOR2>(m);
    m = dpp_max_u32<JL_DPP_ROW_HALF_MIRROR>(m);  // 8 lanes = one 32-element block
    if (per >= 2) m = dpp_max_u32<JL_DPP_ROW_MIRROR>(m);
    if (per >= 4) m = max(m, (u32)__shfl_xor((int)m, 16, JL_WAVE));
    if (per >= 8) m = max(m, (u32)__shfl_xor((int)m, 32, JL_WAVE));
    return m;
}

// The whole-wavefront (256-element window) amax without LDS traffic: DPP maxima
// within and across the 16-lane rows, then lane 63's value read back as a scalar.
__device__ __forceinline__ u32 wave_amax_256(u32 m) {
    m = dpp_max_u32<JL_DPP_QUAD_XOR1>(m);
    m = dpp_max_u32<JL_DPP_QUAD_XOR2>(m);
    m = dpp_max_u32<JL_DPP_ROW_HALF_MIRROR>(m);
    m = dpp_max_u32<JL_DPP_ROW_MIRROR>(m);
    m = max(m, (u32)dpp_i32<JL_DPP_ROW_BCAST15, 0xa>(0, (i32)m));
    m = max(m, (u32)dpp_i32<JL_DPP_ROW_BCAST31, 0xc>(0, (i32)m));
    return (u32)__builtin_amdgcn_readlane((i32)m, 63);
}

// The gated activation of a feed-forward block, silu(g) = g / (1 + e^-g)
// (jit/gpu/kernels/elem.go:813-818).  The exponential is the hardware's (one ulp or so), so the
// quotient is taken with the hardware reciprocal as well (one ulp) instead of a correctly
// rounded division of a value that is not: ten vector instructions less per element in a
// quantizer that every workgroup runs over the whole activation.
__device__ __forceinline__ float silu_f32(float g) { return g * __builtin_amdgcn_rcpf(1.0f + __expf(-g)); }

// Round half away from zero for |p| < 2^22, exactly: adding 0.5 - 2^-25 (the
// largest f32 below one half) cannot carry a value below n + 0.5 up to n + 1,
// and carries every value at or above it; the conversion then truncates.
__device__ __forceinline__ i32 round_half_away(float p) {
    const float c = __uint_as_float(0x3EFFFFFFu);
    return (i32)(p + __builtin_copysignf(c, p));
}

// Quantize this thread's four values with the window's amax.  Returns the four
// int8 packed little endian, the scale d, and the sum over the 16-element
// half-block (identical in the four lanes of the quad).
__device__ __forceinline__ u32 quantize4(f32x4 v, u32 amax_bits, float& d_out, i32& sum16_out) {
    float amax = __uint_as_float(amax_bits);
    float d = amax / 127.0f;
    float inv = d != 0.0f ? 1.0f / d : 0.0f;
    i32 a = round_half_away(v.x * inv), b = round_half_away(v.y * inv);
    i32 c = round_half_away(v.z * inv), e = round_half_away(v.w * inv);
    u32 q = (u32)(a & 0xFF) | ((u32)(b & 0xFF) << 8) | ((u32)(c & 0xFF) << 16) | ((u32)e << 24);
    i32 s = a + b + c + e;
    s += dpp_i32<JL_DPP_QUAD_XOR1, 0xf>(0, s);
    s += dpp_i32<JL_DPP_QUAD_XOR2, 0xf>(0, s);
    d_out = d;
    sum16_out = s;
    return q;
}
