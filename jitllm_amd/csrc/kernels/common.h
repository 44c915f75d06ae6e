// Device-side helpers shared by every kernel of the code object (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef uint32_t u32;
typedef int32_t i32;
typedef u32 u32x2 __attribute__((ext_vector_type(2)));
typedef u32 u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// ggml type numbers (the reference's quant.Type, format/quant/types.go:14-55)
#define JL_Q8_0 8
#define JL_Q4_K 12
#define JL_Q6_K 14
#define JL_MXFP4 39

#define JL_WAVE 64

// Loads of 2-byte-aligned block fields.  The amdhsa target runs with unaligned
// global access enabled, so these lower to single wide loads.
struct __attribute__((packed, aligned(2))) u32x4_a2 { u32x4 v; };
struct __attribute__((packed, aligned(2))) u32x2_a2 { u32x2 v; };
struct __attribute__((packed, aligned(2))) u32_a2 { u32 v; };

__device__ __forceinline__ u32x4 ld16_a2(const uint8_t* p) { return ((const u32x4_a2*)p)->v; }
__device__ __forceinline__ u32x2 ld8_a2(const uint8_t* p) { return ((const u32x2_a2*)p)->v; }
__device__ __forceinline__ u32 ld4_a2(const uint8_t* p) { return ((const u32_a2*)p)->v; }
__device__ __forceinline__ u32x4 ld16(const uint8_t* p) { return *(const u32x4*)p; }
__device__ __forceinline__ uint16_t ld2(const uint8_t* p) { return *(const uint16_t*)p; }

// IEEE binary16 -> f32, exact for every pattern including subnormals
// (format/quant/dequant.go:15-32); the hardware conversion is exact.
__device__ __forceinline__ float half_bits_to_f32(uint16_t h) {
    return (float)__builtin_bit_cast(_Float16, h);
}

// Four signed int8 products accumulated into an int32 (v_dot4_i32_i8).
__device__ __forceinline__ i32 dot4(u32 a, u32 b, i32 c) {
    return __builtin_amdgcn_sdot4((i32)a, (i32)b, c, false);
}

// Data-parallel-primitive lane moves (DPP): the value of another lane of the
// same 16-lane row, or of the previous row's last lane, with no LDS traffic.
#define JL_DPP_QUAD_XOR1 0xB1      // quad_perm [1,0,3,2]
#define JL_DPP_QUAD_XOR2 0x4E      // quad_perm [2,3,0,1]
#define JL_DPP_ROW_HALF_MIRROR 0x141
#define JL_DPP_ROW_MIRROR 0x140
#define JL_DPP_ROW_BCAST15 0x142
#define JL_DPP_ROW_BCAST31 0x143

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ i32 dpp_i32(i32 old, i32 v) {
    return __builtin_amdgcn_update_dpp(old, v, CTRL, ROW_MASK, 0xf, false);
}
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_f32(float v) {  // lanes outside ROW_MASK read 0
    return __builtin_bit_cast(float, dpp_i32<CTRL, ROW_MASK>(0, __builtin_bit_cast(i32, v)));
}

// Sum over the 64 lanes of a wavefront with DPP adds; the total lands in lane 63
// (and in every lane of the last 16-lane row).
__device__ __forceinline__ float wave_sum_to_lane63(float v) {
    v += dpp_f32<JL_DPP_QUAD_XOR1, 0xf>(v);
    v += dpp_f32<JL_DPP_QUAD_XOR2, 0xf>(v);
    v += dpp_f32<JL_DPP_ROW_HALF_MIRROR, 0xf>(v);
    v += dpp_f32<JL_DPP_ROW_MIRROR, 0xf>(v);       // every lane: its row's sum
    v += dpp_f32<JL_DPP_ROW_BCAST15, 0xa>(v);      // rows 1,3 += rows 0,2
    v += dpp_f32<JL_DPP_ROW_BCAST31, 0xc>(v);      // rows 2,3 += rows 0+1
    return v;
}

// Workgroup barrier that orders LDS traffic only.  __syncthreads() carries a
// release fence that also drains every outstanding global load, which would
// throw away the register prefetch that is meant to stay in flight across it.
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// Q4_K / Q5_K 6-bit scale and minimum of sub-block j from the 12 packed bytes,
// given as three little-endian words (format/quant/dequant.go:360-365).
__device__ __forceinline__ void scale_min_k4(int j, u32 s0, u32 s1, u32 s2, u32& sc, u32& m) {
    // bytes 0-3 = s0, 4-7 = s1, 8-11 = s2
    if (j < 4) {
        sc = (s0 >> (8 * j)) & 63;
        m = (s1 >> (8 * j)) & 63;
    } else {
        int i = j - 4;
        u32 b8 = (s2 >> (8 * i)) & 0xFF;
        sc = (b8 & 0xF) | (((s0 >> (8 * i + 6)) & 3) << 4);
        m = (b8 >> 4) | (((s1 >> (8 * i + 6)) & 3) << 4);
    }
}
