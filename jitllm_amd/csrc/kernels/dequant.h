// Dequantize GGUF blocks to f32, bit for bit the reference's Dequant32
// (format/quant/dequant.go:148-174, :367-397, :443-470).  Products are rounded
// to f32 one at a time in the reference's order; nothing is fused.
#pragma once
#include "common.h"

#pragma clang fp contract(off)

static const __device__ int8_t kMxfp4Values[16] = {0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12};

// One thread per element; n elements of type `type` from src.
__device__ __forceinline__ float dequant_elem(int type, const uint8_t* src, size_t i) {
    switch (type) {
    case JL_Q8_0: {
        const uint8_t* blk = src + (i / 32) * 34;
        return (float)(int8_t)blk[2 + (i % 32)] * half_bits_to_f32(ld2(blk));
    }
    case JL_MXFP4: {
        const uint8_t* blk = src + (i / 32) * 17;
        int j = (int)(i % 32);
        uint8_t b = blk[1 + (j & 15)];
        int code = j < 16 ? (b & 0xF) : (b >> 4);
        // 2^(e-128): exact through ldexp, subnormal results included
        return ldexpf((float)kMxfp4Values[code], (int)blk[0] - 128);
    }
    case JL_Q4_K: {
        const uint8_t* blk = src + (i / 256) * 144;
        int e = (int)(i % 256), s = e / 32, l = e % 32;
        float d = half_bits_to_f32(ld2(blk)), dmin = half_bits_to_f32(ld2(blk + 2));
        u32 s0 = *(const u32*)(blk + 4), s1 = *(const u32*)(blk + 8), s2 = *(const u32*)(blk + 12);
        u32 sc, m;
        scale_min_k4(s, s0, s1, s2, sc, m);
        uint8_t b = blk[16 + (s / 2) * 32 + l];
        float q = (float)((s & 1) ? (b >> 4) : (b & 0xF));
        float d1 = d * (float)sc, min1 = dmin * (float)m;
        float p = d1 * q;
        return p - min1;
    }
    case JL_Q6_K: {
        const uint8_t* blk = src + (i / 256) * 210;
        int e = (int)(i % 256), n = e / 128, r = e % 128, quarter = r / 32, l = r % 32;
        const uint8_t* ql = blk + n * 64;
        const uint8_t* qh = blk + 128 + n * 32;
        uint8_t lo = ql[l + (quarter & 1) * 32];
        int nib = quarter >= 2 ? (lo >> 4) : (lo & 0xF);
        int q = (nib | (((qh[l] >> (2 * quarter)) & 3) << 4)) - 32;
        float d = half_bits_to_f32(ld2(blk + 208));
        float sc = (float)(int8_t)blk[192 + n * 8 + l / 16 + 2 * quarter];
        float ds = d * sc;
        return ds * (float)q;
    }
    }
    return 0.f;
}
