// Prefill GEMM over Q4_K weights: out[t][r] = sum_k W[r][k] * x[t][k], many tokens.
//
// Arithmetic (the reference's quantized-activation form with the k-quant window
// of 256, jit/cpu/matvec.go:46-62, so one activation scale d_a per token and
// super-block; per (token, row) it is the decode matvec's value,
// jit/cpu/packedgemm.go:54-58):
//
//   out[t][r] = sum_sb d_a[t,sb] * ( d[r,sb]    * P[t,r,sb]  -  dmin[r,sb] * M[t,r,sb] )
//   P = sum_{s,l} (sc[r,s] * q[r,s,l]) * a[t,s,l]          sub-blocks s, elements l
//   M = sum_s      m[r,s] * A[t,s],   A[t,s] = sum_l a[t,s,l]
//
// P and M are sums of products of small integers, so they run EXACTLY on the
// f16 matrix cores (v_mfma_f32_32x32x16_f16): sc*q <= 945 and |a| <= 127 are
// f16 values, products and partial sums are exact in the f32 accumulator.  A is
// split as 64*A_hi + A_lo so both parts and 64*m are f16 values too.  Scales
// change every 32 weights, which would force an f32 epilogue per 32-deep MFMA
// step on the int8 cores; folding the 6-bit sub-block scale into the f16 operand
// moves the epilogue out to once per 256, where the matrix cores hide it.
//
// Layout.  A workgroup of eight wavefronts (two per SIMD) owns a 128-token x 128-row
// tile and walks K in half super-blocks (a "stage": 128 weights, plus the 16 minimum
// columns in the second half).  Tokens are the matrix instruction's M dimension, so a
// lane owns one weight row (its scales are scalars) and output stores run along rows.
// A wavefront computes 32 tokens x 64 rows.
//   Weights go through LDS: the 512 threads dequantize a stage from HBM into f16
// (magic-number nibble unpack with packed-f16 FMAs, eight K values per 32-bit word of
// nibbles), two stages double-buffered, the loads of the stage after next in flight in
// registers.  The dequantization is spread between a stage's matrix instructions.
//   Activations do not touch LDS.  The prep kernel writes them in matrix-fragment order
// -- for every (stage, 32 tokens, K-step) the 64 lanes' 16-byte operands back to back --
// so a wavefront's operand for its 32 tokens is one fully coalesced 1 KiB load, issued
// a whole stage ahead into a ring of registers.  That removes the largest LDS writer
// and half the LDS reads: LDS writes run at a third of the read rate on this part, and
// with both operands staged the kernel was bound by them.
//   Every wavefront does the same work, so the two on a SIMD cover each other: while
// one dequantizes or runs the super-block epilogue, the other feeds the matrix core.
#pragma once
#include "args.h"
#include "common.h"
#include "quantize.h"

// Phase marker for profiling builds; expands to nothing in the product.
#ifndef JL_TRACE
#define JL_TRACE(i)
#endif

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

#define JL_GEMM_TILE 128          // tokens per workgroup (rows: 64 per group of four wavefronts)
#define JL_GEMM_STRIDE 152        // f16 per LDS row of a stage: 144 used + 8 pad (304 B, odd multiple of 16 B)
// Activation fragments: 64 lanes x 8 f16 each; nine per (stage, 32 tokens): eight
// K-steps and the minimum columns (used in second halves only).
#define JL_GEMM_AFRAG_HALFS 512
#define JL_GEMM_ASTAGE_FRAGS 9

// K position (within a stage's 128 weights) of nibble pair i of 32-bit word c of a
// 64-element group: word c holds bytes 4c..4c+3; byte b's low nibble is element
// 4c+b of the group's first sub-block, its high nibble the same element of the
// second.  The unpack below emits, per word, the eight values
//   (b0.lo, b2.lo, b0.hi, b2.hi, b1.lo, b3.lo, b1.hi, b3.hi)
// and the prep kernel writes activations in the same order.

// -------------------------------------------------------------------- prep
// x [ntok][k] f32 -> bq [2*nsb stages][tok_pad/32][9 fragments][64 lanes][8] f16 and
// da [nsb][tok_pad] f32.  Position pos (0..143) of token t in a stage is K-step pos/16,
// lane 32*((pos/8)%2) + t%32, element pos%8: positions 0..127 are the stage's weights in
// the order the unpack emits them, 128..135 the sub-block sums' low parts, 136..143
// their high parts.  One wavefront per (token, super-block); lane l owns elements 4l..4l+3.
__device__ __forceinline__ _Float16* gemm_a_pos(_Float16* bq, int stage, int t, int tok_pad, int pos) {
    const size_t frag = ((size_t)stage * (tok_pad >> 5) + (t >> 5)) * JL_GEMM_ASTAGE_FRAGS + (pos >> 4);
    return bq + frag * JL_GEMM_AFRAG_HALFS + (32 * ((pos >> 3) & 1) + (t & 31)) * 8 + (pos & 7);
}

__device__ __forceinline__ void gemm_prep_q4k_body(const GemmPrepArgs& p) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sb = blockIdx.x;
    const int t = blockIdx.y * 4 + wave;
    if (t >= p.tok_pad) return;
    f32x4 v = f32x4{0.f, 0.f, 0.f, 0.f};
    if (t < p.ntok) v = ((const f32x4*)(p.x + (size_t)t * p.k + (size_t)sb * 256))[lane];
    u32 m = max(max(abs_bits(v.x), abs_bits(v.y)), max(abs_bits(v.z), abs_bits(v.w)));
    u32 amax = window_amax(m, 8);
    float d;
    i32 sum16;
    u32 q = quantize4(v, amax, d, sum16);
    // sub-block (32 elements = 8 lanes) sum from the two half-block sums
    i32 a32 = sum16 + dpp_i32<JL_DPP_ROW_HALF_MIRROR, 0xf>(0, sum16);
    const int g = lane >> 4, hi = (lane >> 3) & 1, c = lane & 7;
    const int base = 8 * (8 * (g & 1) + c) + 2 * hi;
    _Float16* bq = (_Float16*)p.bq;
    f16x2 p02 = {(_Float16)(float)(int8_t)(q & 0xFF), (_Float16)(float)(int8_t)((q >> 16) & 0xFF)};
    f16x2 p13 = {(_Float16)(float)(int8_t)((q >> 8) & 0xFF), (_Float16)(float)(int8_t)(q >> 24)};
    *(f16x2*)gemm_a_pos(bq, sb * 2 + (g >> 1), t, p.tok_pad, base) = p02;
    *(f16x2*)gemm_a_pos(bq, sb * 2 + (g >> 1), t, p.tok_pad, base + 4) = p13;
    if ((lane & 7) == 0) {
        const int s = lane >> 3;
        *gemm_a_pos(bq, sb * 2 + 1, t, p.tok_pad, 128 + s) = (_Float16)(float)(a32 & 63);  // A = 64*A_hi + A_lo, 0 <= A_lo < 64
        *gemm_a_pos(bq, sb * 2 + 1, t, p.tok_pad, 136 + s) = (_Float16)(float)(a32 >> 6);  // arithmetic shift: floor
    }
    if (lane == 0) p.da[(size_t)sb * p.tok_pad + t] = d;
}

// -------------------------------------------------------------------- main
template <int V> struct GemmIntC { static constexpr int value = V; };

// One stage of weights for a thread: row = tid/4, hh = (tid/2)%2 selects the 64-element
// group (2*half + hh) of the super-block, wq = tid%2 the half of its 32 nibble bytes
// (four 32-bit words).
struct GemmWRegs {
    u32x4 hdr;
    u32x4 q;
};

__device__ __forceinline__ void gemm_load_w(const GemmArgs& p, int row, int sb, int g, int wq, GemmWRegs& r) {
    const uint8_t* blk = p.w + (size_t)row * p.row_bytes + (size_t)sb * 144;
    r.hdr = ld16(blk);
    r.q = ld16(blk + 16 + 32 * g + 16 * wq);
}

// (1024 + n) as f16 for the nibble in bits 0-3 of each 16-bit half.  mask and magic
// (0x000F000F, 0x64006400) are passed in registers so the pair is one and-or instruction.
__device__ __forceinline__ f16x2 nib_pair(u32 w, int shift, u32 mask, u32 magic) {
    u32 v = ((w >> shift) & mask) | magic;
    return __builtin_bit_cast(f16x2, v);
}

// Dequantizing a thread's stage share into LDS is cut into pieces so that it can be
// spread between the matrix instructions of a stage: the scale operands first, then
// one 32-bit word of nibbles (eight K values, one 16-byte LDS write) at a time, and in a
// second half the 16 minimum columns and the row's (d, dmin).
struct GemmWScale {
    f16x2 mlo, mhi, alo, ahi;
    u32 mask, magic;
    _Float16* dst;
};

__device__ __forceinline__ void gemm_w_scale(const GemmWRegs& r, int row, int hh, int wq, int half,
                                             _Float16* sw, GemmWScale& k) {
    const int g = 2 * half + hh;
    // scales of sub-blocks 2g (low nibbles) and 2g+1 (high nibbles), straight from the
    // packed bytes (format/quant/dequant.go:360-365)
    u32 slo, shi;
    const int sh = 16 * (g & 1);
    const u32 A = r.hdr.y >> sh, C = r.hdr.w >> sh;
    if (half == 0) {
        slo = A & 63;
        shi = (A >> 8) & 63;
    } else {
        slo = (C & 0xF) | (((A >> 6) & 3) << 4);
        shi = ((C >> 8) & 0xF) | (((A >> 14) & 3) << 4);
    }
    const _Float16 flo = (_Float16)(float)slo, fhi = (_Float16)(float)shi;
    k.mlo = f16x2{flo, flo};
    k.mhi = f16x2{fhi, fhi};
    const _Float16 nlo = (_Float16)(-1024.0f * (float)slo), nhi = (_Float16)(-1024.0f * (float)shi);
    k.alo = f16x2{nlo, nlo};
    k.ahi = f16x2{nhi, nhi};
    k.mask = 0x000F000Fu;
    k.magic = 0x64006400u;
    asm volatile("" : "+v"(k.mask), "+v"(k.magic));   // keep them in vector registers
    k.dst = sw + row * JL_GEMM_STRIDE + 64 * hh + 32 * wq;
}

// word c (0..3) of the thread's four
__device__ __forceinline__ void gemm_w_word(const GemmWRegs& r, const GemmWScale& k, int c) {
    const u32 w = r.q[c];
    // (1024+n)*sc - 1024*sc = sc*n, exact in f16 (<= 945) through the fused multiply-add
    f16x2 p0 = __builtin_elementwise_fma(nib_pair(w, 0, k.mask, k.magic), k.mlo, k.alo);
    f16x2 p1 = __builtin_elementwise_fma(nib_pair(w, 4, k.mask, k.magic), k.mhi, k.ahi);
    f16x2 p2 = __builtin_elementwise_fma(nib_pair(w, 8, k.mask, k.magic), k.mlo, k.alo);
    f16x2 p3 = __builtin_elementwise_fma(nib_pair(w, 12, k.mask, k.magic), k.mhi, k.ahi);
    u32x4 o = {__builtin_bit_cast(u32, p0), __builtin_bit_cast(u32, p1), __builtin_bit_cast(u32, p2),
               __builtin_bit_cast(u32, p3)};
    *(u32x4*)(k.dst + 8 * c) = o;
}

// second halves, threads with wq == 0: hh = 0 writes m_s (pairs with A_lo), hh = 1
// writes 64*m_s (pairs with A_hi); hh = 0 also the row's (d, dmin)
__device__ __forceinline__ void gemm_w_mins(const GemmWRegs& r, int row, int hh, _Float16* sw, float* sscale) {
    const float mul = hh ? 64.0f : 1.0f;
    f16x8 mm;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        u32 scj, mnj;
        scale_min_k4(j, r.hdr.y, r.hdr.z, r.hdr.w, scj, mnj);
        mm[j] = (_Float16)((float)mnj * mul);
    }
    *(f16x8*)(sw + row * JL_GEMM_STRIDE + 128 + 8 * hh) = mm;
    if (hh == 0) {
        sscale[2 * row] = half_bits_to_f32((uint16_t)(r.hdr.x & 0xFFFF));
        sscale[2 * row + 1] = half_bits_to_f32((uint16_t)(r.hdr.x >> 16));
    }
}

// RH = groups of four wavefronts in the workgroup, each group 64 rows: RH = 2 is the
// 128 x 128 tile on eight wavefronts; RH = 1 a 128-token x 64-row tile on four, of which
// two workgroups share a CU -- they drift apart, so one's vector phases (dequantization,
// epilogue) fall under the other's matrix instructions.
// grid = (tok_pad/128, ceil(nrows/(64*RH))), block = 256*RH, dynamic LDS = two weight
// stages [64*RH][152] f16 + row scales [2][64*RH][2] + token scales [2][128].
template <int RH>
__device__ __forceinline__ void gemm_q4k_body(const GemmArgs& p, uint8_t* smem) {
    constexpr int ROWS = 64 * RH, JL_GEMM_STAGE_HALFS = ROWS * JL_GEMM_STRIDE;
    _Float16* sW = (_Float16*)smem;
    float* sScale = (float*)(sW + 2 * JL_GEMM_STAGE_HALFS);
    float* sDa = sScale + 2 * 2 * ROWS;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int tg = wave & 3, rh = wave >> 2;   // this wavefront: tokens 32*tg.., rows 64*rh..
    const int t0 = blockIdx.x * JL_GEMM_TILE, r0 = blockIdx.y * ROWS;
    const int nsteps = 2 * (p.k / 256);
    // this thread's share of a weight stage
    const int srow = tid >> 2, hh = (tid >> 1) & 1, wq = tid & 1;
    const int wrow = min(r0 + srow, p.nrows - 1);
    const int arow = lane & 31, kg = lane >> 5;
    // fragment (step, ks) of this wavefront's 32 tokens
    const size_t ngrp = (size_t)(p.tok_pad >> 5), mygrp = (size_t)(t0 >> 5) + tg;
    auto a_frag = [&](int step, int ks) {
        return ((const f16x8*)p.bq)[(((size_t)step * ngrp + mygrp) * JL_GEMM_ASTAGE_FRAGS + ks) * 64 + lane];
    };

    f32x16 out[2], accP[2];
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
        for (int e = 0; e < 16; e++) out[j][e] = 0.f;

    // prologue: stage 0 of the weights into LDS, stage 1 into registers; the first
    // stage's activation fragments into the ring
    GemmWRegs wa, wb;   // stages alternate between the two register sets
    gemm_load_w(p, wrow, 0, hh, wq, wa);
    f16x8 aring[8], aaug;
#pragma unroll
    for (int ks = 0; ks < 8; ks++) aring[ks] = a_frag(0, ks);
    aaug = aring[0];
    {
        GemmWScale k0;
        gemm_w_scale(wa, srow, hh, wq, 0, sW, k0);
#pragma unroll
        for (int c = 0; c < 4; c++) gemm_w_word(wa, k0, c);
    }
    gemm_load_w(p, wrow, 0, 2 + hh, wq, wa);
    float da_reg = p.da[t0 + (tid & (JL_GEMM_TILE - 1))];
    lds_barrier();

    // One stage.  HALF is the stage's half of its super-block; wcur holds the next
    // stage's weights (loaded a stage ago), wnxt receives the stage after that.
    auto stage = [&](auto HALF, int step, GemmWRegs& wcur, GemmWRegs& wnxt) {
        constexpr int half = decltype(HALF)::value;
        const int sb = step >> 1;
        const _Float16* w = sW + half * JL_GEMM_STAGE_HALFS;
        const bool has_next = step + 1 < nsteps;
        constexpr int nhalf = half ^ 1;
        const int nsbi = (step + 1) >> 1;
        _Float16* wnext = sW + nhalf * JL_GEMM_STAGE_HALFS;
        JL_TRACE(0);
        // the loads of the stage after next go out first: a whole stage of matrix work
        // covers their latency (that stage has this stage's half)
        {
            const int s2 = min(step + 2, nsteps - 1);
            gemm_load_w(p, wrow, s2 >> 1, 2 * half + hh, wq, wnxt);
        }
        // The next weight stage sits in registers; its dequantization into LDS is spread
        // over this stage's K-steps, one word after every second K-step's matrix
        // instructions, so the vector work runs under the matrix core.
        GemmWScale wsc;
        gemm_w_scale(wcur, srow, hh, wq, nhalf, wnext, wsc);
        JL_TRACE(1);
        // matrix work: per K-step one activation fragment (already in the ring) against
        // the two row groups' weight fragments, fetched from LDS a K-step ahead; the ring
        // slot is refilled with the next stage's fragment as soon as it has been used
        const _Float16* wp0 = w + (64 * rh + arow) * JL_GEMM_STRIDE + 8 * kg;
        const int nstep = min(step + 1, nsteps - 1);
        f16x8 wf[2][2];
#pragma unroll
        for (int j = 0; j < 2; j++) wf[0][j] = *(const f16x8*)(wp0 + 32 * j * JL_GEMM_STRIDE);
        __builtin_amdgcn_sched_barrier(0);
        JL_TRACE(2);
#pragma unroll
        for (int ks = 0; ks < 8; ks++) {
            if (ks + 1 < 8) {
#pragma unroll
                for (int j = 0; j < 2; j++)
                    wf[(ks + 1) & 1][j] = *(const f16x8*)(wp0 + 32 * j * JL_GEMM_STRIDE + 16 * (ks + 1));
            }
            __builtin_amdgcn_sched_barrier(0);
            // (a super-block's first instruction starts from a zero accumulator operand)
            const f32x16 czero = {0};
#pragma unroll
            for (int j = 0; j < 2; j++)
                accP[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(aring[ks], wf[ks & 1][j],
                                                                 (half == 0 && ks == 0) ? czero : accP[j], 0, 0, 0);
            aring[ks] = a_frag(nstep, ks);
            if (ks == 0 && nhalf == 1) aaug = a_frag(nstep, 8);
            if (has_next && (ks & 1)) gemm_w_word(wcur, wsc, ks >> 1);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (has_next && nhalf == 1) {
            if (wq == 0) gemm_w_mins(wcur, srow, hh, wnext, sScale + (nsbi & 1) * 2 * ROWS);
            if (tid < JL_GEMM_TILE) sDa[(nsbi & 1) * JL_GEMM_TILE + tid] = da_reg;
        }
        if (half == 1) {
            // the token scales of the next super-block (written to LDS during its first half)
            const int sb2 = min(sb + 1, p.k / 256 - 1);
            da_reg = p.da[(size_t)sb2 * p.tok_pad + t0 + (tid & (JL_GEMM_TILE - 1))];
        }
        JL_TRACE(3);
        if (half == 1) {
            // the 16 minimum columns: M, then the super-block's epilogue
            //   out += d_a * (d * P - dmin * M)
            const f32x16 zero = {0};
            const float* ssc = sScale + (sb & 1) * 2 * ROWS + 2 * 64 * rh;
            const float* sda = sDa + (sb & 1) * JL_GEMM_TILE + 32 * tg;
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const float dd = ssc[2 * (32 * j + arow)];
                const float dmin = ssc[2 * (32 * j + arow) + 1];
                const f16x8 wm = *(const f16x8*)(wp0 + 32 * j * JL_GEMM_STRIDE + 128);
                const f32x16 accM = __builtin_amdgcn_mfma_f32_32x32x16_f16(aaug, wm, zero, 0, 0, 0);
#pragma unroll
                for (int e = 0; e < 16; e++) {
                    const int tk = 8 * (e >> 2) + 4 * kg + (e & 3);
                    const float u = fmaf(dd, accP[j][e], -(dmin * accM[e]));
                    out[j][e] = fmaf(sda[tk], u, out[j][e]);
                }
            }
        }
        JL_TRACE(4);
        lds_barrier();
        JL_TRACE(5);
    };
    for (int step = 0; step < nsteps; step += 2) {
        stage(GemmIntC<0>{}, step, wa, wb);
        stage(GemmIntC<1>{}, step + 1, wb, wa);
    }

    // store: lane = row (contiguous in memory), register = token
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int r = r0 + 64 * rh + 32 * j + arow;
        if (r >= p.nrows) continue;
#pragma unroll
        for (int e = 0; e < 16; e++) {
            const int t = t0 + 32 * tg + 8 * (e >> 2) + 4 * kg + (e & 3);
            if (t < p.ntok) p.out[(size_t)t * p.nrows + r] = out[j][e];
        }
    }
}
