// MXFP4 weights (32 e2m1 codes + one E8M0 exponent per block, 17 bytes) against
// bf16 activations, f32 accumulate: out[t][r] = sum_k W[r][k] * x[t][k].
//
// A code times its block scale is T[code] * 2^(e-128) with |T| in {0,1,2,3,4,6,8,12}
// (format/quant/dequant.go:159-174, :268): at most two significant bits, so the
// dequantized weight is EXACT in bf16, and bf16 x bf16 products are exact in the
// f32 accumulator of v_mfma_f32_32x32x16_bf16.  The result is therefore the
// reference's "dequantize, then f32 matmul" up to f32 summation order.  The
// hardware's scaled fp4 -> bf16 conversion does the decode, two codes an
// instruction; the block scale is its power-of-two scale operand.
//
// GEMM: 128 tokens x 128 rows per workgroup, K in stages of 128 (four blocks a
// row), both operands staged through double-buffered LDS with a register
// prefetch one stage ahead.  A short-row matvec serves a handful of tokens.
#pragma once
#include "args.h"
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

#define JL_MX_TILE 128
#define JL_MX_KSTAGE 128
#define JL_MX_STRIDE 136  // bf16 per LDS row: 128 + 8 pad (272 B, an odd multiple of 16 B)
#define JL_MX_STAGE_ELEMS (JL_MX_TILE * JL_MX_STRIDE)

struct __attribute__((packed, aligned(1))) u32x4_a1 { u32x4 v; };
__device__ __forceinline__ u32x4 ld16_a1(const uint8_t* p) { return ((const u32x4_a1*)p)->v; }

// 2^(e-127) as an f32 scale: e2m1 values are half the doubled table, so
// T[code] * 2^(e-128) = e2m1(code) * 2^(e-127).  e = 0 gives 2^-127 (subnormal).
__device__ __forceinline__ float mx_scale(uint8_t e) {
    return e ? __uint_as_float((u32)e << 23) : __uint_as_float(0x00400000u);
}

// One block: 16 bytes of codes (byte j = element j in the low nibble, element j+16
// in the high) -> 32 bf16 in element order, as four 16-byte groups.
__device__ __forceinline__ void mx_dequant_block(u32x4 q, float scale, u32x4 out[4]) {
#pragma unroll
    for (int w = 0; w < 4; w++) {
        // bytes 4w..4w+3: pair i = (element 4w+i, element 4w+i+16)
        u32 p0 = __builtin_bit_cast(u32, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q[w], scale, 0));
        u32 p1 = __builtin_bit_cast(u32, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q[w], scale, 1));
        u32 p2 = __builtin_bit_cast(u32, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q[w], scale, 2));
        u32 p3 = __builtin_bit_cast(u32, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q[w], scale, 3));
        // low halves = elements 4w..4w+3, high halves = elements 4w+16..4w+19
        u32 lo01 = __builtin_amdgcn_perm(p1, p0, 0x05040100u), lo23 = __builtin_amdgcn_perm(p3, p2, 0x05040100u);
        u32 hi01 = __builtin_amdgcn_perm(p1, p0, 0x07060302u), hi23 = __builtin_amdgcn_perm(p3, p2, 0x07060302u);
        // group g holds elements 8g..8g+7: w = 0,1 fill groups 0 (low) and 2 (high); w = 2,3 groups 1 and 3
        const int g = w >> 1, h = (w & 1) * 2;
        out[g][h] = lo01; out[g][h + 1] = lo23;
        out[g + 2][h] = hi01; out[g + 2][h + 1] = hi23;
    }
}

struct MxWRegs {
    u32x4 q[2];
    uint8_t e[2];
};

__device__ __forceinline__ void mx_load_w(const MxGemmArgs& p, int row, int stage, int pr, MxWRegs& r) {
    const int nblk = p.k / 32;
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int b = stage * 4 + 2 * pr + i;
        const uint8_t* blk = p.w + (size_t)row * p.row_bytes + (size_t)min(b, nblk - 1) * 17;
        r.e[i] = blk[0];
        r.q[i] = ld16_a1(blk + 1);
        if (b >= nblk) r.q[i] = u32x4{0, 0, 0, 0};  // past the end of K: zero codes
    }
}

__device__ __forceinline__ void mx_store_w(const MxWRegs& r, int row, int pr, __bf16* sw) {
#pragma unroll
    for (int i = 0; i < 2; i++) {
        u32x4 o[4];
        mx_dequant_block(r.q[i], mx_scale(r.e[i]), o);
        __bf16* dst = sw + row * JL_MX_STRIDE + (2 * pr + i) * 32;
#pragma unroll
        for (int g = 0; g < 4; g++) *(u32x4*)(dst + 8 * g) = o[g];
    }
}

struct MxARegs {
    u32x4 c[8];
};

__device__ __forceinline__ void mx_load_a(const MxGemmArgs& p, int t0, int stage, int tid, MxARegs& r) {
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const int c = tid + 256 * i, tok = c >> 4, ch = c & 15;
        const int kk = stage * JL_MX_KSTAGE + ch * 8;
        const bool ok = t0 + tok < p.ntok && kk < p.k;
        const uint16_t* src = p.x + (size_t)min(t0 + tok, p.ntok - 1) * p.k + min(kk, p.k - 8);
        u32x4 v = *(const u32x4*)src;
        r.c[i] = ok ? v : u32x4{0, 0, 0, 0};
    }
}

__device__ __forceinline__ void mx_store_a(const MxARegs& r, int tid, __bf16* sa) {
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const int c = tid + 256 * i, tok = c >> 4, ch = c & 15;
        *(u32x4*)(sa + tok * JL_MX_STRIDE + ch * 8) = r.c[i];
    }
}

__device__ __forceinline__ void mx_lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

__device__ __forceinline__ void mx_gemm_body(const MxGemmArgs& p, uint8_t* smem) {
    __bf16* sA = (__bf16*)smem;
    __bf16* sW = sA + 2 * JL_MX_STAGE_ELEMS;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int t0 = blockIdx.x * JL_MX_TILE, r0 = blockIdx.y * JL_MX_TILE;
    // a small grid is widened along K: workgroup z takes a contiguous run of the K
    // stages and writes its partial sums to its own slab, summed afterwards in order
    const int all_stages = (p.k + JL_MX_KSTAGE - 1) / JL_MX_KSTAGE;
    const int per_split = (all_stages + p.nsplit - 1) / p.nsplit;
    const int s_lo = min((int)blockIdx.z * per_split, all_stages), s_hi = min(s_lo + per_split, all_stages);
    const int nstages = s_hi - s_lo;
    float* outp = p.nsplit > 1 ? p.part + (size_t)blockIdx.z * p.ntok * p.nrows : p.out;
    const int wrow = min(r0 + (tid >> 1), p.nrows - 1), pr = tid & 1;
    const int wt = (wave >> 1) * 64, wr = (wave & 1) * 64;
    const int arow = lane & 31, kg = lane >> 5;

    f32x16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.f;

    MxWRegs wreg;
    MxARegs areg;
    if (nstages > 0) {
        mx_load_w(p, wrow, s_lo, pr, wreg);
        mx_load_a(p, t0, s_lo, tid, areg);
        mx_store_w(wreg, tid >> 1, pr, sW);
        mx_store_a(areg, tid, sA);
    }
    if (nstages > 1) {
        mx_load_w(p, wrow, s_lo + 1, pr, wreg);
        mx_load_a(p, t0, s_lo + 1, tid, areg);
    }
    mx_lds_barrier();

    for (int st = 0; st < nstages; st++) {
        const int buf = st & 1;
        const __bf16* a = sA + buf * JL_MX_STAGE_ELEMS;
        const __bf16* w = sW + buf * JL_MX_STAGE_ELEMS;
        if (st + 1 < nstages) {
            mx_store_w(wreg, tid >> 1, pr, sW + (buf ^ 1) * JL_MX_STAGE_ELEMS);
            mx_store_a(areg, tid, sA + (buf ^ 1) * JL_MX_STAGE_ELEMS);
            if (st + 2 < nstages) {
                mx_load_w(p, wrow, s_lo + st + 2, pr, wreg);
                mx_load_a(p, t0, s_lo + st + 2, tid, areg);
            }
        }
#pragma unroll
        for (int ks = 0; ks < JL_MX_KSTAGE / 16; ks++) {
            bf16x8 af[2], wf[2];
#pragma unroll
            for (int i = 0; i < 2; i++) {
                af[i] = *(const bf16x8*)(a + (wt + 32 * i + arow) * JL_MX_STRIDE + 16 * ks + 8 * kg);
                wf[i] = *(const bf16x8*)(w + (wr + 32 * i + arow) * JL_MX_STRIDE + 16 * ks + 8 * kg);
            }
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], wf[j], acc[i][j], 0, 0, 0);
        }
        mx_lds_barrier();
    }
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int r = r0 + wr + 32 * j + arow;
        if (r >= p.nrows) continue;
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const int t = t0 + wt + 32 * i + 8 * (e >> 2) + 4 * kg + (e & 3);
                if (t < p.ntok) outp[(size_t)t * p.nrows + r] = acc[i][j][e];
            }
    }
}

// A few tokens (ntok <= 8): one wavefront per row, lane l takes blocks l, l+64, ...;
// weights decode to f32 pairs, activations (bf16 in global memory) widen to f32.
__device__ __forceinline__ void mx_matvec_body(const MxGemmArgs& p) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
    const int row = blockIdx.x * nwaves + wave;
    if (row >= p.nrows) return;
    const int nblk = p.k / 32;
    float acc[8];
#pragma unroll
    for (int t = 0; t < 8; t++) acc[t] = 0.f;
    for (int b = lane; b < nblk; b += 64) {
        const uint8_t* blk = p.w + (size_t)row * p.row_bytes + (size_t)b * 17;
        const float scale = mx_scale(blk[0]);
        const u32x4 q = ld16_a1(blk + 1);
        float wv[32];
#pragma unroll
        for (int w = 0; w < 4; w++) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                f32x2 pr;
                switch (i) {
                case 0: pr = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(q[w], scale, 0); break;
                case 1: pr = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(q[w], scale, 1); break;
                case 2: pr = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(q[w], scale, 2); break;
                default: pr = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(q[w], scale, 3); break;
                }
                wv[4 * w + i] = pr.x;
                wv[4 * w + i + 16] = pr.y;
            }
        }
#pragma unroll
        for (int t = 0; t < 8; t++) {
            if (t < p.ntok) {
                const uint16_t* xt = p.x + (size_t)t * p.k + (size_t)b * 32;
                float s = 0.f;
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    u32x4 v = ((const u32x4*)xt)[c];
#pragma unroll
                    for (int d = 0; d < 4; d++) {
                        s = fmaf(wv[8 * c + 2 * d], __uint_as_float(v[d] << 16), s);
                        s = fmaf(wv[8 * c + 2 * d + 1], __uint_as_float(v[d] & 0xFFFF0000u), s);
                    }
                }
                acc[t] += s;
            }
        }
    }
#pragma unroll
    for (int t = 0; t < 8; t++) {
        if (t < p.ntok) {
            float v = wave_sum_to_lane63(acc[t]);
            if (lane == 63) p.out[(size_t)t * p.nrows + row] = v;
        }
    }
}

// grid = ceil(n / 256), block = 256
__device__ __forceinline__ void sum_parts_body(const SumPartsArgs& p) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= p.n) return;
    float s = p.part[i];
    for (int z = 1; z < p.nsplit; z++) s += p.part[(size_t)z * p.n + i];
    p.out[i] = s;
}
