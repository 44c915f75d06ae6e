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
// their high parts.
// grid = (k/256, tok_pad/32), block = 256 (or 1024): 32 tokens of one super-block.  Each wavefront
// quantizes eight (two) tokens (lane l owns elements 4l..4l+3) into LDS; then every wavefront
// assembles whole fragments, 16 bytes a lane and 1 KiB contiguous a store.
#define JL_GEMM_PREP_LDS_WORDS (32 * 65 + 32 * 8)
// One group of 32 tokens, one super-block: load(tl) returns this lane's four elements
// (4*lane .. 4*lane+3 of the super-block) of token tl of the group, zeros for a token that
// does not exist.  grp of ngrp groups; da is laid [nsb][32*ngrp].
// NW wavefronts a workgroup (4, or 16 where few tokens make the grid small and the chain of
// tokens a wavefront quantizes one after the other is the kernel's length).
// PL: the K order of the plane-reading kernels.  There a 32-bit word of nibbles holds eight
// weights of ONE sub-block (byte b of word w: element 4w+b in the low nibble, element 4w+b+16
// in the high nibble, jit/gpu/kernels/pack.go:210-239), so vector v = 2*ks + kg of a stage is
// word v%4 of the stage's sub-block v/4, and its eight values pair with the activations of
// elements 4w + (0, 2, 16, 18, 1, 3, 17, 19) of that sub-block.
// FOLD: the fragments hold f16(q * d_a), the token's scale folded into the operand (the form of
// kernels/gemm_q4k_fold.h: one rounding to f16 more than the exact form, no sums fragment).
template <int NW, bool PL = false, bool FOLD = false, class Load>
__device__ __forceinline__ void gemm_prep_group(u32* lds, int sb, int grp, int ngrp, uint16_t* bqp, float* dap,
                                                Load load) {
    constexpr int TPW = 32 / NW, FPW = 16 / NW;   // tokens and fragments per wavefront
    u32* sq = lds;                       // [32 tokens][65]: 64 words of int8 + 1 pad (bank spread)
    i32* sA = (i32*)(lds + 32 * 65);     // [32 tokens][8 sub-block sums]
    float* sD = (float*)(lds + JL_GEMM_PREP_LDS_WORDS);   // FOLD: [32 tokens] scales
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    f32x4 v[TPW];
#pragma unroll
    for (int i = 0; i < TPW; i++) v[i] = load(wave * TPW + i);
#pragma unroll
    for (int i = 0; i < TPW; i++) {
        const int tl = wave * TPW + i;
        const u32 m = max(max(abs_bits(v[i].x), abs_bits(v[i].y)), max(abs_bits(v[i].z), abs_bits(v[i].w)));
        const u32 amax = wave_amax_256(m);
        float d;
        i32 sum16;
        const u32 q = quantize4(v[i], amax, d, sum16);
        // sub-block (32 elements = 8 lanes) sum from the two half-block sums
        const i32 a32 = sum16 + dpp_i32<JL_DPP_ROW_HALF_MIRROR, 0xf>(0, sum16);
        sq[tl * 65 + lane] = q;
        if ((lane & 7) == 0) sA[tl * 8 + (lane >> 3)] = a32;
        if (lane == 0) dap[(size_t)sb * (32 * ngrp) + grp * 32 + tl] = d;
        if (FOLD && lane == 0) sD[tl] = d;
    }
    __syncthreads();
    const int tl = lane & 31, kg = lane >> 5;
    u32x4* dst = (u32x4*)bqp;
    const float dtl = FOLD ? sD[tl] : 1.0f;
#pragma unroll
    for (int i = 0; i < FPW; i++) {
        const int pi = wave * FPW + i, h = pi >> 3, ks = pi & 7;
        // vector (group g, word c): low nibbles' partners are elements 4c.. of sub-block 2g,
        // high nibbles' partners the same elements of sub-block 2g+1
        u32 lo, hi;
        if (PL) {
            const int v = 2 * ks + kg, sub = 4 * h + (v >> 2), w = v & 3;
            lo = sq[tl * 65 + 8 * sub + w];
            hi = sq[tl * 65 + 8 * sub + 4 + w];
        } else {
            const int g = 2 * h + (ks >> 2), c = 2 * (ks & 3) + kg;
            lo = sq[tl * 65 + 16 * g + c];
            hi = sq[tl * 65 + 16 * g + 8 + c];
        }
        auto f = [&](u32 w, int b) {
            const float q = (float)(int8_t)(w >> (8 * b));
            return (_Float16)(FOLD ? q * dtl : q);
        };
        const f16x8 o = {f(lo, 0), f(lo, 2), f(hi, 0), f(hi, 2), f(lo, 1), f(lo, 3), f(hi, 1), f(hi, 3)};
        dst[(((size_t)(2 * sb + h) * ngrp + grp) * JL_GEMM_ASTAGE_FRAGS + ks) * 64 + lane] =
            __builtin_bit_cast(u32x4, o);
    }
    if (!FOLD && wave == 0) {
        // A = 64*A_hi + A_lo with 0 <= A_lo < 64 (arithmetic shift: floor); lanes 0-31 carry
        // the low parts, lanes 32-63 the high parts
        f16x8 o;
#pragma unroll
        for (int s8 = 0; s8 < 8; s8++) {
            const i32 a32 = sA[tl * 8 + s8];
            o[s8] = (_Float16)(float)(kg ? (a32 >> 6) : (a32 & 63));
        }
        dst[(((size_t)(2 * sb + 1) * ngrp + grp) * JL_GEMM_ASTAGE_FRAGS + 8) * 64 + lane] =
            __builtin_bit_cast(u32x4, o);
    }
}

template <int NW, bool PL = false, bool FOLD = false>
__device__ __forceinline__ void gemm_prep_q4k_body(const GemmPrepArgs& p, u32* lds) {
    const int lane = threadIdx.x & 63;
    const int sb = blockIdx.x, grp = blockIdx.y;
    gemm_prep_group<NW, PL, FOLD>(lds, sb, grp, p.tok_pad >> 5, p.bq, p.da, [&](int tl) {
        const int t = grp * 32 + tl;
        f32x4 v = f32x4{0.f, 0.f, 0.f, 0.f};
        if (t < p.ntok) v = ((const f32x4*)(p.x + (size_t)t * p.k + (size_t)sb * 256))[lane];
        return v;
    });
}

// -------------------------------------------------------------------- main
template <int V> struct GemmIntC { static constexpr int value = V; };

// f(GemmIntC<I>{}) for I = 0..N-1 with I a compile-time constant inside f: register arrays
// indexed by it stay in registers.
template <int I, int N, class F>
__device__ __forceinline__ void gemm_static_for(F&& f) {
    if constexpr (I < N) {
        f(GemmIntC<I>{});
        gemm_static_for<I + 1, N>(f);
    }
}

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

// The same registers from packed planes (jit/gpu/kernels/pack.go:52-247): thread = (row, sub-block
// of the stage).  hdr = (d | dmin << 16, the three words of the 96-bit stream of 6-bit scales
// and minimums: scale of sub-block j at bit 12 j, its minimum at bit 12 j + 6); q = the four
// words of the sub-block's nibbles.  Every load is a 32-bit word a lane, consecutive rows in
// consecutive lanes: 256 contiguous bytes an instruction.  row: relative to the launch's first.
__device__ __forceinline__ void gemm_load_w_planes(const GemmArgs& p, int row, int sb, int sub, GemmWRegs& r) {
    const size_t st = (size_t)p.pstride;
    const size_t sup = (size_t)(p.psb0 + sb);
    const u32* d = p.pd + sup * st + p.prow0;
    const u32* sc = p.psc + sup * 3 * st + p.prow0;
    const u32* q = p.pqs + (sup * 8 + sub) * 4 * st + p.prow0;
    r.hdr = u32x4{d[row], sc[row], sc[st + row], sc[2 * st + row]};
    r.q = u32x4{q[row], q[st + row], q[2 * st + row], q[3 * st + row]};
}

// Field f (six bits at bit 6 f) of the 96-bit stream in hdr.y, hdr.z, hdr.w (scstream.go:32-52).
__device__ __forceinline__ u32 gemm_stream_field(const u32x4& hdr, int f) {
    const int b = 6 * f, wi = b >> 5, sh = b & 31;
    const u32 lo = wi == 0 ? hdr.y : wi == 1 ? hdr.z : hdr.w;
    const u32 hi = wi == 0 ? hdr.z : wi == 1 ? hdr.w : 0u;
    return __builtin_amdgcn_alignbit(hi, lo, sh) & 63u;
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

// the same for a thread of the plane form: all eight nibbles of a word belong to sub-block
// `sub` of the super-block, the row's K positions 32 * (sub % 4) .. of the stage
__device__ __forceinline__ void gemm_w_scale_planes(const GemmWRegs& r, int row, int sub, _Float16* sw, GemmWScale& k) {
    const u32 sc = gemm_stream_field(r.hdr, 2 * sub);
    const _Float16 f = (_Float16)(float)sc, n = (_Float16)(-1024.0f * (float)sc);
    k.mlo = k.mhi = f16x2{f, f};
    k.alo = k.ahi = f16x2{n, n};
    k.mask = 0x000F000Fu;
    k.magic = 0x64006400u;
    asm volatile("" : "+v"(k.mask), "+v"(k.magic));
    k.dst = sw + row * JL_GEMM_STRIDE + 32 * (sub & 3);
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

// plane form: sub-block threads 0 (m_s, and the row's d and dmin) and 1 (64 * m_s) of a row
__device__ __forceinline__ void gemm_w_mins_planes(const GemmWRegs& r, int row, int hh, _Float16* sw, float* sscale) {
    const float mul = hh ? 64.0f : 1.0f;
    f16x8 mm;
#pragma unroll
    for (int j = 0; j < 8; j++) mm[j] = (_Float16)((float)gemm_stream_field(r.hdr, 2 * j + 1) * mul);
    *(f16x8*)(sw + row * JL_GEMM_STRIDE + 128 + 8 * hh) = mm;
    if (hh == 0) {
        sscale[2 * row] = half_bits_to_f32((uint16_t)(r.hdr.x & 0xFFFF));
        sscale[2 * row + 1] = half_bits_to_f32((uint16_t)(r.hdr.x >> 16));
    }
}

// A grid too small for the chip is widened along K: workgroup z takes sb_per super-blocks
// and writes its partial sums to slab z; the slabs are added in order afterwards.
__device__ __forceinline__ void gemm_split_slice(GemmArgs& p) {
    if (p.sb_per == 0) return;
    const int sb0 = blockIdx.z * p.sb_per;
    const int n = min(p.sb_per, p.k / 256 - sb0);
    p.w += (size_t)sb0 * 144;
    p.psb0 += sb0;
    p.bq += (size_t)2 * sb0 * (p.tok_pad >> 5) * (JL_GEMM_ASTAGE_FRAGS * JL_GEMM_AFRAG_HALFS);
    p.da += (size_t)sb0 * p.tok_pad;
    p.k = 256 * n;
    p.out += (size_t)blockIdx.z * p.ntok * p.out_stride;
}

// RH = groups of four wavefronts in the workgroup, each group 64 rows: RH = 2 is the
// 128 x 128 tile on eight wavefronts; RH = 1 a 128-token x 64-row tile on four, of which
// two workgroups share a CU -- they drift apart, so one's vector phases (dequantization,
// epilogue) fall under the other's matrix instructions.
// grid = (tok_pad/128, ceil(nrows/(64*RH))), block = 256*RH, dynamic LDS = two weight
// stages [64*RH][152] f16 + row scales [2][64*RH][2] + token scales [2][128].
// t0, r0: the tile's first token and row (a grouped launch places tiles per expert).
// SKIP: a wavefront whose 32 tokens all lie past ntok takes its share of the dequantization
// and the barriers and leaves the matrix work out (ragged tiles of a grouped launch).
// PL (RH = 1 only): the weights come from packed planes.  Thread = (row = lane, sub-block of the
// stage = wavefront); the stage's K order is the planes' (the prep kernel's PL order), the rest
// of the kernel is the same.
template <int RH, bool SKIP = false, bool PL = false>
__device__ __forceinline__ void gemm_q4k_body(const GemmArgs& p, uint8_t* smem, int t0, int r0) {
    static_assert(!PL || RH == 1, "the plane form is the four-wavefront tile");
    constexpr int ROWS = 64 * RH, JL_GEMM_STAGE_HALFS = ROWS * JL_GEMM_STRIDE;
    _Float16* sW = (_Float16*)smem;
    float* sScale = (float*)(sW + 2 * JL_GEMM_STAGE_HALFS);
    float* sDa = sScale + 2 * 2 * ROWS;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int tg = wave & 3, rh = wave >> 2;   // this wavefront: tokens 32*tg.., rows 64*rh..
    const bool live = !SKIP || t0 + 32 * (__builtin_amdgcn_readfirstlane(wave) & 3) < p.ntok;   // wavefront-uniform
    const int nsteps = 2 * (p.k / 256);
    // this thread's share of a weight stage
    const int srow = PL ? lane : tid >> 2, hh = PL ? (wave & 1) : (tid >> 1) & 1, wq = tid & 1;
    const int psub = __builtin_amdgcn_readfirstlane(wave) & 3;   // plane form: its sub-block of a stage
    const int wrow = min(r0 + srow, p.nrows - 1);
    auto load_w = [&](int sb, int half, GemmWRegs& r) {
        if (PL) gemm_load_w_planes(p, wrow, sb, 4 * half + psub, r);
        else gemm_load_w(p, wrow, sb, 2 * half + hh, wq, r);
    };
    auto w_scale = [&](const GemmWRegs& r, int half, _Float16* sw, GemmWScale& k) {
        if (PL) gemm_w_scale_planes(r, srow, 4 * half + psub, sw, k);
        else gemm_w_scale(r, srow, hh, wq, half, sw, k);
    };
    const int arow = lane & 31, kg = lane >> 5;
    // fragment (step, ks) of this wavefront's 32 tokens
    // (a tile may reach past the last group of the workspace: such tokens are never stored)
    const size_t ngrp = (size_t)(p.tok_pad >> 5), mygrp = min((size_t)(t0 >> 5) + tg, ngrp - 1);
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
    // The loads go out in the order the loop issues them -- a stage's weights, the next stage's,
    // the activation fragments in K order, the token scale; the loop's head adds the stage after
    // that.  The wait the compiler puts before a register's first use in the loop is the smaller
    // of the counts on the two ways in: with stage 1's weights requested last here, every
    // first half-stage waited for the weights its own head had just requested.
    GemmWRegs wa, wb;   // stages alternate between the two register sets
    load_w(0, 0, wb);
    load_w(0, 1, wa);
    __builtin_amdgcn_sched_barrier(0);
    f16x8 aring[8], aaug;
#pragma unroll
    for (int ks = 0; ks < 8; ks++) {
        aring[ks] = a_frag(0, ks);
        __builtin_amdgcn_sched_barrier(0);
    }
    aaug = aring[0];
    const int da_tok = min(t0 + (tid & (JL_GEMM_TILE - 1)), p.tok_pad - 1);
    float da_reg = p.da[da_tok];
    __builtin_amdgcn_sched_barrier(0);
    {
        GemmWScale k0;
        w_scale(wb, 0, sW, k0);
#pragma unroll
        for (int c = 0; c < 4; c++) gemm_w_word(wb, k0, c);
    }
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
        // the loads of the stage after next go out first: a whole stage of matrix work
        // covers their latency (that stage has this stage's half)
        {
            const int s2 = min(step + 2, nsteps - 1);
            load_w(s2 >> 1, half, wnxt);
        }
        // The next weight stage sits in registers; its dequantization into LDS is spread
        // over this stage's K-steps, one word after every second K-step's matrix
        // instructions, so the vector work runs under the matrix core.
        GemmWScale wsc;
        w_scale(wcur, nhalf, wnext, wsc);
        // (all four header words stay live to here: d and dmin are read only by the stage that
        // writes the minimum columns, and a word nobody reads is handed out as a temporary while
        // its load is still in flight -- writing it then waits for the load just requested)
        asm volatile("" ::"v"(wcur.hdr));
        // matrix work: per K-step one activation fragment (already in the ring) against
        // the two row groups' weight fragments, fetched from LDS a K-step ahead; the ring
        // slot is refilled with the next stage's fragment as soon as it has been used
        const _Float16* wp0 = w + (64 * rh + arow) * JL_GEMM_STRIDE + 8 * kg;
        const int nstep = min(step + 1, nsteps - 1);
        f16x8 wf[2][2];
        if (live) {
#pragma unroll
            for (int j = 0; j < 2; j++) wf[0][j] = *(const f16x8*)(wp0 + 32 * j * JL_GEMM_STRIDE);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ks = 0; ks < 8; ks++) {
            if (live) {
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
            }
            if (has_next && (ks & 1)) gemm_w_word(wcur, wsc, ks >> 1);
            // a matrix instruction, vector work under it, the second (two in a row would park
            // the vector work behind the second for its whole length)
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, 6, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (has_next && nhalf == 1) {
            if (PL) {
                if (psub < 2) gemm_w_mins_planes(wcur, srow, psub, wnext, sScale + (nsbi & 1) * 2 * ROWS);
            } else if (wq == 0) {
                gemm_w_mins(wcur, srow, hh, wnext, sScale + (nsbi & 1) * 2 * ROWS);
            }
            if (tid < JL_GEMM_TILE) sDa[(nsbi & 1) * JL_GEMM_TILE + tid] = da_reg;
        }
        if (half == 1) {
            // the token scales of the next super-block (written to LDS during its first half)
            const int sb2 = min(sb + 1, p.k / 256 - 1);
            da_reg = p.da[(size_t)sb2 * p.tok_pad + da_tok];
        }
        if (half == 1 && live) {
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
        lds_barrier();
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
            if (t < p.ntok) p.out[(size_t)t * p.out_stride + r] = out[j][e];
        }
    }
}

// ------------------------------------------------------------- wide form
// What bounds the tiles above, measured: (1) the vector L1 path of a CU moves 64 bytes a
// clock, a quarter of what LDS reads deliver, and carries the activation fragments; a
// wavefront that owns 64 rows uses each fragment for only two matrix instructions.  (2) A
// matrix instruction hides about four vector instructions issued beside it and nothing
// more, and wavefronts that meet at a barrier every stage run their vector phases (scale
// decode, minimum columns, the super-block epilogue) together, with the matrix cores idle.
//
// Here a wavefront owns 32 tokens x ALL 128 rows of the workgroup's tile, so a fragment
// feeds four matrix instructions, and the eight wavefronts of a workgroup share one
// dequantization of the weights over 256 tokens.  A stage is cut into 16 slots of two
// matrix instructions (tile pair jh = slot/8, K-step ks = slot%8) and ALL vector work is
// dealt out over the slots, a dozen instructions each:
//   * the epilogue of a super-block runs one quarter tile per slot: tiles 0,1 under the
//     second half's matrix instructions for tiles 2,3, and tiles 2,3 under the NEXT
//     super-block's first-half instructions for tiles 0,1 (its accumulators are not
//     restarted before slot 8); minimum columns and scales are kept per super-block parity
//     so the deferred half still finds them;
//   * the next stage's weights are dequantized in the other eight slots: scales in the
//     first, a word of nibbles in every odd one, the minimum columns in the even ones.
// grid = (tok_pad/256, ceil(nrows/128)), block = 512 (one workgroup per CU, two wavefronts
// per SIMD), dynamic LDS = JL_GEMM_WIDE_LDS_BYTES.  tok_pad is a multiple of 256.
#define JL_GEMM_WIDE_TOK 256
#define JL_GEMM_WROW 136   // f16 per weight row of a stage: 128 + 8 (272 B: rows advance four banks)
#define JL_GEMM_MROW 24    // f16 per row of minimum columns: 16 + 8
#define JL_GEMM_WIDE_LDS_BYTES (2 * 128 * JL_GEMM_WROW * 2 + 2 * 128 * JL_GEMM_MROW * 2 + 2 * 128 * 2 * 4 + 2 * 256 * 4)

// The 16 six-bit scales and minimums of a Q4_K super-block as bytes of four words
// (format/quant/dequant.go:360-365, four at a time).
struct GemmScaleBytes {
    u32 sc_lo, sc_hi, mn_lo, mn_hi;   // sub-blocks 0-3 and 4-7
};
__device__ __forceinline__ GemmScaleBytes gemm_scale_bytes(u32 s0, u32 s1, u32 s2) {
    GemmScaleBytes r;
    r.sc_lo = s0 & 0x3F3F3F3Fu;
    r.mn_lo = s1 & 0x3F3F3F3Fu;
    r.sc_hi = (s2 & 0x0F0F0F0Fu) | ((s0 >> 2) & 0x30303030u);
    r.mn_hi = ((s2 >> 4) & 0x0F0F0F0Fu) | ((s1 >> 2) & 0x30303030u);
    return r;
}

// Multipliers and addends that turn the magic-number nibbles into sc*q: low nibbles read
// (1024 + q), high nibbles are left in place and read (1024 + 16 q), so their multiplier
// is sc/16 and their addend -64 sc; every product and sum is exact in f16.
struct GemmWideScale {
    f16x2 mlo, alo, mhi, ahi;
    _Float16* dst;
};
__device__ __forceinline__ void gemm_wide_scale(const u32x4& hdr, int hh, int half, GemmWideScale& k) {
    // sub-blocks 2g (low nibbles) and 2g+1 (high nibbles), g = 2*half + hh
    const u32 word = half ? ((hdr.w & 0x0F0F0F0Fu) | ((hdr.y >> 2) & 0x30303030u)) : (hdr.y & 0x3F3F3F3Fu);
    const u32 pair = word >> (16 * hh);
    const float flo = (float)(pair & 0xFF), fhi = (float)((pair >> 8) & 0xFF);
    const _Float16 hlo = (_Float16)flo, hhi16 = (_Float16)(fhi * 0.0625f);
    const _Float16 nlo = (_Float16)(-1024.0f * flo), nhi = (_Float16)(-64.0f * fhi);
    k.mlo = f16x2{hlo, hlo};
    k.alo = f16x2{nlo, nlo};
    k.mhi = f16x2{hhi16, hhi16};
    k.ahi = f16x2{nhi, nhi};
}
// plane form: all eight nibbles of a word belong to sub-block `sub` of the super-block
__device__ __forceinline__ void gemm_wide_scale_planes(const u32x4& hdr, int sub, GemmWideScale& k) {
    const float f = (float)gemm_stream_field(hdr, 2 * sub);
    const _Float16 hlo = (_Float16)f, hhi16 = (_Float16)(f * 0.0625f);
    const _Float16 nlo = (_Float16)(-1024.0f * f), nhi = (_Float16)(-64.0f * f);
    k.mlo = f16x2{hlo, hlo};
    k.alo = f16x2{nlo, nlo};
    k.mhi = f16x2{hhi16, hhi16};
    k.ahi = f16x2{nhi, nhi};
}
__device__ __forceinline__ void gemm_wide_word(u32 w, const GemmWideScale& k, int c, u32 mask_lo, u32 mask_hi,
                                               u32 magic) {
    const u32 w8 = w >> 8;
    auto nib = [&](u32 v, u32 mask) { return __builtin_bit_cast(f16x2, (v & mask) | magic); };
    // (b0.lo, b2.lo), (b0.hi, b2.hi), (b1.lo, b3.lo), (b1.hi, b3.hi)
    const f16x2 p0 = __builtin_elementwise_fma(nib(w, mask_lo), k.mlo, k.alo);
    const f16x2 p1 = __builtin_elementwise_fma(nib(w, mask_hi), k.mhi, k.ahi);
    const f16x2 p2 = __builtin_elementwise_fma(nib(w8, mask_lo), k.mlo, k.alo);
    const f16x2 p3 = __builtin_elementwise_fma(nib(w8, mask_hi), k.mhi, k.ahi);
    const u32x4 o = {__builtin_bit_cast(u32, p0), __builtin_bit_cast(u32, p1), __builtin_bit_cast(u32, p2),
                     __builtin_bit_cast(u32, p3)};
    *(u32x4*)(k.dst + 8 * c) = o;
}

// PL: the weights come from packed planes; thread = (row = 64 * (wavefront % 2) + lane, sub-block
// of the stage = wavefront / 2), the stage's K order is the planes' (the prep kernel's PL order).
template <bool PL = false>
__device__ __forceinline__ void gemm_q4k_wide_body(const GemmArgs& p, uint8_t* smem) {
    constexpr int ROWS = 128, TOK = JL_GEMM_WIDE_TOK, STAGE_HALFS = ROWS * JL_GEMM_WROW;
    constexpr int MIN_HALFS = ROWS * JL_GEMM_MROW;
    _Float16* sW = (_Float16*)smem;                 // [2 stages][128][136]
    _Float16* sMin = sW + 2 * STAGE_HALFS;          // [2 super-block parities][128][24]
    float* sScale = (float*)(sMin + 2 * MIN_HALFS); // [2][128][2]  (d, dmin)
    float* sDa = sScale + 2 * 2 * ROWS;             // [2][256]

    const int tid = threadIdx.x, lane = tid & 63;
    const int tg = __builtin_amdgcn_readfirstlane(tid >> 6);   // wavefront tg: tokens 32*tg..
    const int t0 = blockIdx.x * TOK, r0 = blockIdx.y * ROWS;
    const int nsteps = 2 * (p.k / 256);
    const int psub = tg >> 1;   // plane form: this thread's sub-block of a stage
    const int srow = PL ? 64 * (tg & 1) + lane : tid >> 2, hh = PL ? (psub & 1) : (tid >> 1) & 1, wq = tid & 1;
    const int arow = lane & 31, kg = lane >> 5;
    // Addresses are a uniform 64-bit base (scalar registers) plus a 32-bit lane offset.
    // Activation fragment (step, ks) of this wavefront's 32 tokens:
    const size_t astride = (size_t)(p.tok_pad >> 5) * (JL_GEMM_ASTAGE_FRAGS * 1024);   // bytes per stage
    const char* abase = (const char*)p.bq + ((size_t)(t0 >> 5) + tg) * (JL_GEMM_ASTAGE_FRAGS * 1024);
    const unsigned aoff = lane * 16;
    auto a_frag = [&](int step, int ks) {
        return *(const f16x8*)(abase + (size_t)step * astride + ks * 1024 + aoff);
    };
    // This thread's share of a weight stage: 16 bytes of nibbles and the block header.
    const uint8_t* wbase = p.w + (size_t)r0 * p.row_bytes;
    const unsigned woff = (unsigned)(min(r0 + srow, p.nrows - 1) - r0) * (unsigned)p.row_bytes;
    const unsigned wqoff = woff + 16 + 32 * hh + 16 * wq;
    const int prow = min(r0 + srow, p.nrows - 1);
    auto load_w = [&](int step, GemmWRegs& r) {
        if (PL) {
            gemm_load_w_planes(p, prow, step >> 1, 4 * (step & 1) + psub, r);
        } else {
            const uint8_t* blk = wbase + (size_t)(step >> 1) * 144 + 64 * (step & 1);
            r.hdr = ld16(blk - 64 * (step & 1) + woff);
            r.q = ld16(blk + wqoff);
        }
    };
    u32 mask_lo = 0x000F000Fu, mask_hi = 0x00F000F0u, magic = 0x64006400u;
    asm volatile("" : "+v"(mask_lo), "+v"(mask_hi), "+v"(magic));   // keep them in vector registers
    const int wdst = PL ? srow * JL_GEMM_WROW + 32 * psub : srow * JL_GEMM_WROW + 64 * hh + 32 * wq;

    f32x16 out[4], accP[4];
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
        for (int e = 0; e < 16; e++) out[j][e] = 0.f;

    // prologue: stage 0 of the weights into LDS, stage 1 into registers, the first
    // activation fragments into the ring
    GemmWRegs wa, wb;
    load_w(0, wa);
    f16x8 aring[8], aaug;
#pragma unroll
    for (int ks = 0; ks < 8; ks++) aring[ks] = a_frag(0, ks);
    aaug = a_frag(min(1, nsteps - 1), 8);
    {
        GemmWideScale k0;
        if (PL) gemm_wide_scale_planes(wa.hdr, psub, k0);
        else gemm_wide_scale(wa.hdr, hh, 0, k0);
        k0.dst = sW + wdst;
#pragma unroll
        for (int c = 0; c < 4; c++) gemm_wide_word(wa.q[c], k0, c, mask_lo, mask_hi, magic);
    }
    load_w(min(1, nsteps - 1), wa);
    float da_reg = p.da[t0 + (tid & (TOK - 1))];
    lds_barrier();

    // One quarter (four tokens per lane) of tile `tile`'s epilogue, out += d_a * (d * P - dmin * M),
    // with the scales of super-block parity eb.
    f32x16 accM;
    float2 esc;   // (d, dmin) of the tile's row
    auto ep_quarter = [&](auto TILE, auto I, const f32x4& dav) __attribute__((always_inline)) {
        constexpr int tile = decltype(TILE)::value, i = decltype(I)::value;
#pragma unroll
        for (int e4 = 0; e4 < 4; e4++) {
            const int e = 4 * i + e4;
            const float u = fmaf(esc.x, accP[tile][e], -(esc.y * accM[e]));
            out[tile][e] = fmaf(dav[e4], u, out[tile][e]);
        }
    };

    auto stage = [&](auto HALF, auto FIRST, int step, GemmWRegs& wcur, GemmWRegs& wnxt) {
        constexpr int half = decltype(HALF)::value;
        constexpr bool first = decltype(FIRST)::value != 0;
        constexpr int nhalf = half ^ 1;
        constexpr int ep_jh = half;            // tile pair whose slots carry the epilogue
        constexpr bool has_ep = half == 1 || !first;
        constexpr int ej0 = half ? 0 : 2;      // its tiles: 0,1 of this super-block / 2,3 of the last
        const int sb = step >> 1;
        const int eb = (half ? sb : sb - 1) & 1;
        const _Float16* w = sW + half * STAGE_HALFS;
        _Float16* wnext = sW + nhalf * STAGE_HALFS;
        const int nstep = min(step + 1, nsteps - 1);
        load_w(min(step + 2, nsteps - 1), wnxt);
        const _Float16* wp0 = w + arow * JL_GEMM_WROW + 8 * kg;
        const _Float16* mp0 = sMin + eb * MIN_HALFS + arow * JL_GEMM_MROW + 8 * kg;
        const float* scp = sScale + eb * 2 * ROWS + 2 * arow;
        const float* dap = sDa + eb * TOK + 32 * tg + 4 * kg;
        auto w_frag = [&](int slot, int j) {
            return *(const f16x8*)(wp0 + 32 * (2 * (slot >> 3) + j) * JL_GEMM_WROW + 16 * (slot & 7));
        };
        f16x8 wf[2][2], wm;
        f32x4 dav[2];   // token scales of an epilogue slot, read from LDS a slot ahead
        GemmWideScale wsc;
        wsc.dst = wnext + wdst;
#pragma unroll
        for (int j = 0; j < 2; j++) wf[0][j] = w_frag(0, j);
        if (has_ep && ep_jh == 0) {
            dav[0] = *(const f32x4*)dap;
            wm = *(const f16x8*)(mp0 + 32 * ej0 * JL_GEMM_MROW);
            esc = *(const float2*)(scp + 2 * 32 * ej0);
        }
        __builtin_amdgcn_sched_barrier(0);
        gemm_static_for<0, 16>([&](auto SLOT) __attribute__((always_inline)) {
            constexpr int slot = decltype(SLOT)::value, jh = slot >> 3, ks = slot & 7;
            constexpr bool ep = has_ep && jh == ep_jh;
            constexpr bool ep_next = has_ep && slot + 1 < 16 && ((slot + 1) >> 3) == ep_jh;
            // the next slot's token scales first: the wait that guards them then leaves the
            // weight fragments (read after them, used a slot later) in flight
            if (ep_next) dav[(slot + 1) & 1] = *(const f32x4*)(dap + 8 * ((ks + 1) & 3));
            if (slot + 1 < 16) {
#pragma unroll
                for (int j = 0; j < 2; j++) wf[(slot + 1) & 1][j] = w_frag(slot + 1, j);
            }
            // a slot ahead of a tile's first quarter: its minimum columns and row scales
            if (has_ep && ep_jh == 1 && slot == 7) {
                wm = *(const f16x8*)(mp0 + 32 * ej0 * JL_GEMM_MROW);
                esc = *(const float2*)(scp + 2 * 32 * ej0);
            }
            if (ep && ks == 3) wm = *(const f16x8*)(mp0 + 32 * (ej0 + 1) * JL_GEMM_MROW);   // (the first tile's M is done with it)
            if (ep && ks == 4) esc = *(const float2*)(scp + 2 * 32 * (ej0 + 1));
            __builtin_amdgcn_sched_barrier(0);
            const f32x16 czero = {0};
            if (ep && (ks & 3) == 0) {
                // the tile's M = sum m_s A_s, ahead of this slot's instructions so that it is
                // ready when the vector work below asks for it
                accM = __builtin_amdgcn_mfma_f32_32x32x16_f16(aaug, wm, czero, 0, 0, 0);
            }
#pragma unroll
            for (int j = 0; j < 2; j++)
                accP[2 * jh + j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                    aring[ks], wf[slot & 1][j], (half == 0 && ks == 0) ? czero : accP[2 * jh + j], 0, 0, 0);
            if (jh == 1) {
                aring[ks] = a_frag(nstep, ks);
                if (ks == 0 && nhalf == 1) aaug = a_frag(nstep, 8);
            }
            if (ep) {
                ep_quarter(GemmIntC<ej0 + (ks >> 2)>{}, GemmIntC<(ks & 3)>{}, dav[slot & 1]);
            } else if (jh != ep_jh) {
                // the next stage's weights: wcur -> f16 -> LDS
                if (ks == 0) {
                    if (PL) gemm_wide_scale_planes(wcur.hdr, 4 * nhalf + psub, wsc);
                    else gemm_wide_scale(wcur.hdr, hh, nhalf, wsc);
                }
                if (ks & 1) gemm_wide_word(wcur.q[ks >> 1], wsc, ks >> 1, mask_lo, mask_hi, magic);
                if (nhalf == 1) {
                    // a first half also lays down its super-block's minimum columns and scales
                    // (no branches on the lane here: the four threads of a row that share an
                    // address write the same value, which costs nothing and keeps the slot
                    // one basic block)
                    if (ks == 4) {
                        // hh = 0 writes m_s (pairs with A_lo), hh = 1 writes 64*m_s (pairs with A_hi)
                        const float mul = hh ? 64.0f : 1.0f;
                        f16x8 mm;
                        if (PL) {
#pragma unroll
                            for (int j = 0; j < 8; j++)
                                mm[j] = (_Float16)((float)gemm_stream_field(wcur.hdr, 2 * j + 1) * mul);
                        } else {
                            const GemmScaleBytes sbytes = gemm_scale_bytes(wcur.hdr.y, wcur.hdr.z, wcur.hdr.w);
#pragma unroll
                            for (int b = 0; b < 4; b++) {
                                mm[b] = (_Float16)((float)((sbytes.mn_lo >> (8 * b)) & 0xFF) * mul);
                                mm[4 + b] = (_Float16)((float)((sbytes.mn_hi >> (8 * b)) & 0xFF) * mul);
                            }
                        }
                        *(f16x8*)(sMin + (sb & 1) * MIN_HALFS + srow * JL_GEMM_MROW + 8 * hh) = mm;
                    }
                    if (ks == 6) {
                        float2 dd = {half_bits_to_f32((uint16_t)(wcur.hdr.x & 0xFFFF)),
                                     half_bits_to_f32((uint16_t)(wcur.hdr.x >> 16))};
                        *(float2*)(sScale + (sb & 1) * 2 * ROWS + 2 * srow) = dd;
                        sDa[(sb & 1) * TOK + (tid & (TOK - 1))] = da_reg;
                    }
                }
            }
            // Issue order inside the slot.  A wavefront issues in order, and a matrix
            // instruction waits at issue until the one before it has left the matrix core: two
            // in a row park the vector work behind the second for its whole length, and vector
            // work ahead of them that waits on an LDS read parks the matrix core.  So: a matrix
            // instruction, half of the vector work under it, the second, the rest.
            if (ep && (ks & 3) == 0) {
                __builtin_amdgcn_sched_group_barrier(0x008, 3, 0);   // M first: the vector work reads it
            } else {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, 6, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            }
            __builtin_amdgcn_sched_group_barrier(0x002, 48, 0);
            __builtin_amdgcn_sched_barrier(0);
        });
        if (half == 1) {
            const int sb2 = min(sb + 1, p.k / 256 - 1);
            da_reg = p.da[(size_t)sb2 * p.tok_pad + t0 + (tid & (TOK - 1))];
        }
        lds_barrier();
    };
    stage(GemmIntC<0>{}, GemmIntC<1>{}, 0, wa, wb);
    stage(GemmIntC<1>{}, GemmIntC<0>{}, 1, wb, wa);
    for (int step = 2; step < nsteps; step += 2) {
        stage(GemmIntC<0>{}, GemmIntC<0>{}, step, wa, wb);
        stage(GemmIntC<1>{}, GemmIntC<0>{}, step + 1, wb, wa);
    }
    // tiles 2,3 of the last super-block
    {
        const int eb = (p.k / 256 - 1) & 1;
        const f32x16 czero = {0};
        gemm_static_for<2, 4>([&](auto TILE) __attribute__((always_inline)) {
            constexpr int tile = decltype(TILE)::value;
            const f16x8 wm = *(const f16x8*)(sMin + eb * MIN_HALFS + (32 * tile + arow) * JL_GEMM_MROW + 8 * kg);
            esc = *(const float2*)(sScale + eb * 2 * ROWS + 2 * (32 * tile + arow));
            accM = __builtin_amdgcn_mfma_f32_32x32x16_f16(aaug, wm, czero, 0, 0, 0);
            gemm_static_for<0, 4>([&](auto I) __attribute__((always_inline)) {
                constexpr int i = decltype(I)::value;
                ep_quarter(TILE, I, *(const f32x4*)(sDa + eb * TOK + 32 * tg + 4 * kg + 8 * i));
            });
        });
    }

#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int r = r0 + 32 * j + arow;
        if (r >= p.nrows) continue;
#pragma unroll
        for (int e = 0; e < 16; e++) {
            const int t = t0 + 32 * tg + 8 * (e >> 2) + 4 * kg + (e & 3);
            if (t < p.ntok) p.out[(size_t)t * p.out_stride + r] = out[j][e];
        }
    }
}

// ------------------------------------------------------------- two-pass form
// With several token tiles per weight tile the dequantization above is repeated for every
// one of them, and it is vector work that the matrix cores wait for (an MFMA hides about
// half of the vector instructions issued beside it, and the fused kernel issues nine per
// MFMA).  From a few hundred tokens on it is cheaper to expand the weights ONCE per call
// into f16 fragments in a workspace (2 bytes per weight, written and re-read at HBM/L2
// speed) and run a matrix kernel whose only vector work is the super-block epilogue.
// The values are the same integers either way, so both forms give the same sums.
#define JL_GEMM_W16_STAGE_VECS 1152   // 16-byte vectors per (64 rows, stage): 16 weight fragments + 2 of minimums

// grid = (k/256, nrows_pad/32), block = 256: 32 rows of one super-block.  The blocks are
// read coalesced into LDS, then thread (row = tid%32, c = tid/32) expands word c of each of
// the four 64-element groups: one 16-byte vector each, 1 KiB contiguous per wavefront.
__device__ __forceinline__ void gemm_w16_prep_q4k_body(const GemmW16PrepArgs& p, u32* raw) {
    const int tid = threadIdx.x, sb = blockIdx.x, tile32 = blockIdx.y;
    const int nst = 2 * (p.k / 256);
    for (int idx = tid; idx < 32 * 9; idx += 256) {
        const int rl = idx / 9, v = idx - 9 * rl;
        const int row = min(tile32 * 32 + rl, p.nrows - 1);
        const u32x4 t = ld16(p.w + (size_t)row * p.row_bytes + (size_t)sb * 144 + 16 * v);
        u32* d = raw + rl * 37 + 4 * v;   // 37-word rows: lanes of a wavefront hit distinct banks
        d[0] = t.x; d[1] = t.y; d[2] = t.z; d[3] = t.w;
    }
    __syncthreads();
    const int rl = tid & 31, c = tid >> 5;
    const u32* rr = raw + rl * 37;
    const u32 s0 = rr[1], s1 = rr[2], s2 = rr[3];
    const int rg = tile32 & 1;
    u32x4* dst = (u32x4*)p.w16 + ((size_t)(tile32 >> 1) * nst + 2 * sb) * JL_GEMM_W16_STAGE_VECS;
#pragma unroll
    for (int g = 0; g < 4; g++) {
        u32 sclo, schi, mlo, mhi;
        scale_min_k4(2 * g, s0, s1, s2, sclo, mlo);
        scale_min_k4(2 * g + 1, s0, s1, s2, schi, mhi);
        const u32 w = rr[4 + 8 * g + c];
        // the order gemm_w_word emits: (b0.lo, b2.lo, b0.hi, b2.hi, b1.lo, b3.lo, b1.hi, b3.hi)
        f16x8 v;
        v[0] = (_Float16)(float)(sclo * (w & 15));
        v[1] = (_Float16)(float)(sclo * ((w >> 16) & 15));
        v[2] = (_Float16)(float)(schi * ((w >> 4) & 15));
        v[3] = (_Float16)(float)(schi * ((w >> 20) & 15));
        v[4] = (_Float16)(float)(sclo * ((w >> 8) & 15));
        v[5] = (_Float16)(float)(sclo * ((w >> 24) & 15));
        v[6] = (_Float16)(float)(schi * ((w >> 12) & 15));
        v[7] = (_Float16)(float)(schi * (w >> 28));
        const int ks = 4 * (g & 1) + (c >> 1);
        dst[(size_t)(g >> 1) * JL_GEMM_W16_STAGE_VECS + (2 * ks + rg) * 64 + 32 * (c & 1) + rl] =
            __builtin_bit_cast(u32x4, v);
    }
    if (c < 2) {   // c = 0: m_s (pairs with A_lo), c = 1: 64*m_s (pairs with A_hi)
        const float mul = c ? 64.0f : 1.0f;
        f16x8 mm;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            u32 scj, mnj;
            scale_min_k4(j, s0, s1, s2, scj, mnj);
            mm[j] = (_Float16)((float)mnj * mul);
        }
        dst[JL_GEMM_W16_STAGE_VECS + (16 + rg) * 64 + 32 * c + rl] = __builtin_bit_cast(u32x4, mm);
    } else if (c == 2) {
        float* o = p.wsc + 2 * ((size_t)sb * p.nrows_pad + tile32 * 32 + rl);
        o[0] = half_bits_to_f32((uint16_t)(rr[0] & 0xFFFF));
        o[1] = half_bits_to_f32((uint16_t)(rr[0] >> 16));
    }
}

// grid = 8 * ceil(nrt/8) * ntt workgroups of 256 threads, dynamic LDS = two weight stages
// of 1152 vectors + token scales [2][128].  Workgroups are dealt to the eight XCDs in turn,
// so workgroup L takes row tile 8*(L/8/ntt) + L%8 and token tile (L/8)%ntt: all token tiles
// of a row tile run on one XCD and its L2 fetches the expanded weights once.
// A wavefront computes 32 tokens x 64 rows exactly as in the fused kernel; a weight stage
// is a plain copy, global -> registers (a stage ahead) -> LDS in fragment order, four
// vectors per thread spread between the K-steps.
__device__ __forceinline__ void gemm_q4k_w16_body(const GemmW16Args& p, uint8_t* smem) {
    u32x4* sW = (u32x4*)smem;
    float* sDa = (float*)(sW + 2 * JL_GEMM_W16_STAGE_VECS);
    const int tid = threadIdx.x, lane = tid & 63, tg = tid >> 6;
    const int L = blockIdx.x, idx = L >> 3;
    const int tt = idx % p.ntt, rt = (idx / p.ntt) * 8 + (L & 7);
    if (rt >= p.nrt) return;
    const int t0 = tt * JL_GEMM_TILE, r0 = rt * 64;
    const int nsteps = 2 * (p.k / 256);
    const u32x4* wsrc = (const u32x4*)p.w16 + (size_t)rt * nsteps * JL_GEMM_W16_STAGE_VECS;
    const int arow = lane & 31, kg = lane >> 5;
    // (a tile may reach past the last group of the workspace: such tokens are never stored)
    const size_t ngrp = (size_t)(p.tok_pad >> 5), mygrp = min((size_t)(t0 >> 5) + tg, ngrp - 1);
    auto a_frag = [&](int step, int ks) {
        return ((const f16x8*)p.bq)[(((size_t)step * ngrp + mygrp) * JL_GEMM_ASTAGE_FRAGS + ks) * 64 + lane];
    };

    f32x16 out[2], accP[2];
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
        for (int e = 0; e < 16; e++) out[j][e] = 0.f;

    // prologue: stage 0 into LDS, stage 1 into registers, the first activation fragments
    u32x4 wv[4], wvaug;
#pragma unroll
    for (int i = 0; i < 4; i++) wv[i] = wsrc[tid + 256 * i];
    f16x8 aring[8], aaug;
#pragma unroll
    for (int ks = 0; ks < 8; ks++) aring[ks] = a_frag(0, ks);
    aaug = aring[0];
#pragma unroll
    for (int i = 0; i < 4; i++) sW[tid + 256 * i] = wv[i];
    {
        const int s1 = min(1, nsteps - 1);
#pragma unroll
        for (int i = 0; i < 4; i++) wv[i] = wsrc[(size_t)s1 * JL_GEMM_W16_STAGE_VECS + tid + 256 * i];
        wvaug = wsrc[(size_t)s1 * JL_GEMM_W16_STAGE_VECS + 1024 + (tid & 127)];
    }
    const int da_tok = min(t0 + (tid & (JL_GEMM_TILE - 1)), p.tok_pad - 1);
    float da_reg = p.da[da_tok];
    lds_barrier();

    auto stage = [&](auto HALF, int step) {
        constexpr int half = decltype(HALF)::value;
        constexpr int nhalf = half ^ 1;
        const int sb = step >> 1;
        const u32x4* cur = sW + half * JL_GEMM_W16_STAGE_VECS;
        u32x4* nxt = sW + nhalf * JL_GEMM_W16_STAGE_VECS;
        const int nstep = min(step + 1, nsteps - 1);
        const u32x4* w2 = wsrc + (size_t)min(step + 2, nsteps - 1) * JL_GEMM_W16_STAGE_VECS;
        float sc2[2][2];
        if (half == 1) {
            // the rows' (d, dmin) for this super-block's epilogue
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const float* s = p.wsc + 2 * ((size_t)sb * p.nrows_pad + r0 + 32 * j + arow);
                sc2[j][0] = s[0];
                sc2[j][1] = s[1];
            }
        }
        f16x8 wf[2][2];
#pragma unroll
        for (int j = 0; j < 2; j++) wf[0][j] = __builtin_bit_cast(f16x8, cur[j * 64 + lane]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ks = 0; ks < 8; ks++) {
            if (ks + 1 < 8) {
#pragma unroll
                for (int j = 0; j < 2; j++)
                    wf[(ks + 1) & 1][j] = __builtin_bit_cast(f16x8, cur[(2 * (ks + 1) + j) * 64 + lane]);
            }
            __builtin_amdgcn_sched_barrier(0);
            const f32x16 czero = {0};
#pragma unroll
            for (int j = 0; j < 2; j++)
                accP[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(aring[ks], wf[ks & 1][j],
                                                                 (half == 0 && ks == 0) ? czero : accP[j], 0, 0, 0);
            aring[ks] = a_frag(nstep, ks);
            if (ks == 0 && nhalf == 1) aaug = a_frag(nstep, 8);
            if (ks & 1) {
                // one vector of the next stage into LDS, its register refilled for the stage after
                const int i = ks >> 1;
                nxt[tid + 256 * i] = wv[i];
                wv[i] = w2[tid + 256 * i];
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if (nhalf == 1) {
            // the next stage is a second half: its minimum columns and the token scales
            if (tid < 128) nxt[1024 + tid] = wvaug;
            if (tid < JL_GEMM_TILE) sDa[(sb & 1) * JL_GEMM_TILE + tid] = da_reg;
        } else {
            wvaug = w2[1024 + (tid & 127)];
            const int sb2 = min(sb + 1, p.k / 256 - 1);
            da_reg = p.da[(size_t)sb2 * p.tok_pad + da_tok];
        }
        if (half == 1) {
            const f32x16 zero = {0};
            const float* sda = sDa + (sb & 1) * JL_GEMM_TILE + 32 * tg;
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const f16x8 wm = __builtin_bit_cast(f16x8, cur[(16 + j) * 64 + lane]);
                const f32x16 accM = __builtin_amdgcn_mfma_f32_32x32x16_f16(aaug, wm, zero, 0, 0, 0);
#pragma unroll
                for (int e = 0; e < 16; e++) {
                    const int tk = 8 * (e >> 2) + 4 * kg + (e & 3);
                    const float u = fmaf(sc2[j][0], accP[j][e], -(sc2[j][1] * accM[e]));
                    out[j][e] = fmaf(sda[tk], u, out[j][e]);
                }
            }
        }
        lds_barrier();
    };
    for (int step = 0; step < nsteps; step += 2) {
        stage(GemmIntC<0>{}, step);
        stage(GemmIntC<1>{}, step + 1);
    }

#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int r = r0 + 32 * j + arow;
        if (r >= p.nrows) continue;
#pragma unroll
        for (int e = 0; e < 16; e++) {
            const int t = t0 + 32 * tg + 8 * (e >> 2) + 4 * kg + (e & 3);
            if (t < p.ntok) p.out[(size_t)t * p.nrows + r] = out[j][e];
        }
    }
}

// ------------------------------------------------------------- few tokens
// Up to 64 tokens (speculative decoding, small batches, the first tokens of a prompt): the
// weights are read once at the decode matvec's pace and nothing else should cost anything.
// The tiles above stage weights through LDS behind workgroup barriers, need a K split with a
// second launch to fill the chip, and idle most of a 32- or 128-token tile.  Here:
//   * the matrix instruction is v_mfma_f32_16x16x32_f16: 16 tokens x 16 rows, K = 32; a
//     workgroup owns 16 rows and ALL tokens, so 4096 rows are 256 workgroups;
//   * its eight wavefronts split K (wavefront w takes super-blocks w, w + 8, ...), each with
//     its own accumulators; the eight partial tiles meet in LDS at the end and are added in
//     wavefront order: one launch, no atomics, no second pass;
//   * weights go from memory straight into the operand registers: lane (row r = lane % 16,
//     kq = lane / 16) loads the 16 bytes at 16 + 64 G + 16 kq of its row's block (G = 0, 1:
//     the super-block's halves), four 32-bit words, and word j is its operand for the
//     half's K-step j after the usual unpack (eight nibbles -> eight f16 values sc * q);
//   * the activations are the prefill GEMM's fragments, read where they lie: word j of lane
//     kq is word c = 4 (kq % 2) + j of the 64-element group g = 2 G + kq / 2, whose partner
//     values sit in fragment ks = 4 (kq / 2) + c / 2, lane-half c % 2 of stage 2 sb + G.
// The arithmetic per super-block is the other forms': out += d_a * (d * P - dmin * M), P and M
// exact on the matrix cores (M through one 16x16x16 instruction over the sixteen minimum
// columns).  grid = ceil(nrows / 16), block = 512, static LDS = 8 x NT x 1 KiB.
// Measured and not kept: two 16-row groups a workgroup (an activation operand then feeds two
// instructions: no faster at 14336 rows, slower at 4096 where it halves the grid), and
// copying the rows' blocks into LDS with coalesced loads first (slower by a microsecond).
// Every load is a buffer load: a descriptor on the operand's base, a per-lane byte offset
// formed once (the lane's row, its quarter of a K-step) and a scalar offset for everything
// that moves (super-block, half, K-step, token tile), so the address arithmetic runs on the
// scalar unit: at sixteen tokens the vector unit is the busiest part of this kernel.  The
// host declines matrices of 4 GiB and more.
template <int NT>   // NT tiles of 16 tokens: tok_pad = 32 * ceil(NT / 2) covers them
__device__ __forceinline__ void gemm_q4k_few_body(const GemmArgs& p, float* part) {
    typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r16 = lane & 15, kq = lane >> 4;
    const int r0 = blockIdx.x * 16;
    const int nsb = p.k / 256;
    const u32 ngrp = (u32)(p.tok_pad >> 5);
    const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc((void*)p.w, 0, -1, 0x00020000);
    const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc((void*)p.bq, 0, -1, 0x00020000);
    const __amdgpu_buffer_rsrc_t rd = __builtin_amdgcn_make_buffer_rsrc((void*)p.da, 0, -1, 0x00020000);
    const u32 vrow = (u32)min(r0 + r16, p.nrows - 1) * (u32)p.row_bytes;   // this lane's row
    const u32 vq = vrow + 16u + 16u * (u32)kq;                               // its 16 bytes of a half
    // its operand in a fragment: K-steps 4 (kq/2) + 2 (kq%2) + j/2, lane 32 (j%2) + 16 (tile%2) + r16
    const u32 va = ((u32)(4 * (kq >> 1) + 2 * (kq & 1)) * 64u + (u32)r16) * 16u;
    const u32 vm = ((u32)(32 * (kq >> 1) + r16)) * 16u + 8u * (u32)(kq & 1);   // in the sums' fragment
    const u32 vd = 16u * (u32)kq;                                             // its four tokens' scales

    f32x4 out[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) out[t] = f32x4{0.f, 0.f, 0.f, 0.f};

    struct W { u32x4 hdr, q[2]; };
    auto load_w = [&](int sb, W& w) {
        const u32 so = (u32)sb * 144u;
        w.hdr = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rw, vrow, so, 0));
        w.q[0] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rw, vq, so, 0));
        w.q[1] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rw, vq + 64u, so, 0));
    };
    // activation operands of half G of super-block sb: [K-step j][token tile]
    auto load_a = [&](int sb, int G, f16x8* af) {
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int t = 0; t < NT; t++) {
                const u32 so = ((((u32)(2 * sb + G) * ngrp + (u32)(t >> 1)) * JL_GEMM_ASTAGE_FRAGS + (u32)(j >> 1)) * 64u +
                                32u * (u32)(j & 1) + 16u * (u32)(t & 1)) * 16u;
                af[j * NT + t] = __builtin_bit_cast(f16x8, __builtin_amdgcn_raw_buffer_load_b128(rb, va, so, 0));
            }
    };
    u32 mask = 0x000F000Fu, magic = 0x64006400u;
    asm volatile("" : "+v"(mask), "+v"(magic));

    W wcur, wnxt;
    if (wave < nsb) load_w(wave, wcur);
    for (int sb = wave; sb < nsb; sb += 8) {
        if (sb + 8 < nsb) load_w(sb + 8, wnxt);
        f32x4 accP[NT];
#pragma unroll
        for (int t = 0; t < NT; t++) accP[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int G = 0; G < 2; G++) {
            // the half's operands go out together; left to itself the scheduler sinks each load
            // next to its use and the loop becomes a chain of waits
            f16x8 af[4 * NT];
            load_a(sb, G, af);
            __builtin_amdgcn_sched_barrier(0);
            // scales of sub-blocks 2s (low nibbles) and 2s+1 (high nibbles), s = 2G + kq/2,
            // straight from the packed bytes (format/quant/dequant.go:360-365)
            const int sh = 16 * (kq >> 1);
            const u32 A = wcur.hdr.y >> sh, C = wcur.hdr.w >> sh;
            u32 slo, shi;
            if (G == 0) {
                slo = A & 63;
                shi = (A >> 8) & 63;
            } else {
                slo = (C & 0xF) | (((A >> 6) & 3) << 4);
                shi = ((C >> 8) & 0xF) | (((A >> 14) & 3) << 4);
            }
            const _Float16 flo = (_Float16)(float)slo, fhi = (_Float16)(float)shi;
            const _Float16 nlo = (_Float16)(-1024.0f * (float)slo), nhi = (_Float16)(-1024.0f * (float)shi);
            const f16x2 mlo = {flo, flo}, mhi = {fhi, fhi}, alo = {nlo, nlo}, ahi = {nhi, nhi};
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const u32 w = wcur.q[G][j];
                // (1024+n)*sc - 1024*sc = sc*n, exact in f16 (<= 945) through the fused multiply-add
                const f16x2 p0 = __builtin_elementwise_fma(nib_pair(w, 0, mask, magic), mlo, alo);
                const f16x2 p1 = __builtin_elementwise_fma(nib_pair(w, 4, mask, magic), mhi, ahi);
                const f16x2 p2 = __builtin_elementwise_fma(nib_pair(w, 8, mask, magic), mlo, alo);
                const f16x2 p3 = __builtin_elementwise_fma(nib_pair(w, 12, mask, magic), mhi, ahi);
                const f16x8 wf = {p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
#pragma unroll
                for (int t = 0; t < NT; t++)
                    accP[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[j * NT + t], wf, accP[t], 0, 0, 0);
            }
        }
        // minimum columns: K = 16 = (m_0..m_7 against the sums' low parts, 64 m_0..m_7 against
        // their high parts); lane kq holds columns 4 kq .. 4 kq + 3
        f16x4 wm;
        {
            const float mul = (kq >> 1) ? 64.0f : 1.0f;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                u32 scj, mnj;
                scale_min_k4(4 * (kq & 1) + i, wcur.hdr.y, wcur.hdr.z, wcur.hdr.w, scj, mnj);
                wm[i] = (_Float16)((float)mnj * mul);
            }
        }
        const float dd = half_bits_to_f32((uint16_t)(wcur.hdr.x & 0xFFFF));
        const float dmin = half_bits_to_f32((uint16_t)(wcur.hdr.x >> 16));
#pragma unroll
        for (int t = 0; t < NT; t++) {
            // the sums' fragment (index 8 of the super-block's second stage): lanes 0-31 low
            // parts, 32-63 high parts, eight sub-blocks each
            const u32 som = ((((u32)(2 * sb + 1) * ngrp + (u32)(t >> 1)) * JL_GEMM_ASTAGE_FRAGS + 8u) * 64u +
                             16u * (u32)(t & 1)) * 16u;
            const f16x4 am = __builtin_bit_cast(f16x4, __builtin_amdgcn_raw_buffer_load_b64(rb, vm, som, 0));
            const f32x4 accM = __builtin_amdgcn_mfma_f32_16x16x16f16(am, wm, f32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
            // this lane's four tokens: 16 t + 4 kq + i
            const f32x4 da = __builtin_bit_cast(
                f32x4, __builtin_amdgcn_raw_buffer_load_b128(rd, vd, ((u32)sb * (u32)p.tok_pad + 16u * (u32)t) * 4u, 0));
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float u = fmaf(dd, accP[t][i], -(dmin * accM[i]));
                out[t][i] = fmaf(da[i], u, out[t][i]);
            }
        }
        wcur = wnxt;
    }

    // the eight K shares, added in wavefront order; part [wave][tile][lane] of four floats
    f32x4* pv = (f32x4*)part;
#pragma unroll
    for (int t = 0; t < NT; t++) pv[(wave * NT + t) * 64 + lane] = out[t];
    __syncthreads();
    for (int o = tid; o < NT * 64; o += 512) {
        f32x4 s = pv[o];
#pragma unroll
        for (int w = 1; w < 8; w++) {
            const f32x4 v = pv[w * NT * 64 + o];
            s = f32x4{s.x + v.x, s.y + v.y, s.z + v.z, s.w + v.w};
        }
        const int t = o >> 6, l = o & 63, r = r0 + (l & 15);
        if (r < p.nrows) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int tok = 16 * t + 4 * (l >> 4) + i;
                if (tok < p.ntok) p.out[(size_t)tok * p.out_stride + r] = s[i];
            }
        }
    }
}

// The same scheme on v_mfma_f32_32x32x16_f16 for 65..128 tokens, where the tiled forms still
// need a K split with a second launch: a workgroup owns 32 rows and 64 tokens (NT tiles of
// 32; grid.y = groups of 64 tokens, which read the weights again from L2), its eight
// wavefronts split K.  Lane (row r = lane % 32, half = lane / 32) loads the 16 bytes at
// 16 + 32 g + 16 half of its row's block for each 64-element group g: words c = 4 half + j,
// and word j is its operand for the group's K-step j; the partner activations sit in
// fragment ks = 4 (g % 2) + 2 half + j / 2, lane-half j % 2 of stage 2 sb + g / 2.
// grid = (ceil(nrows / 32), ceil(ntok / 64)), block = 512, static LDS = 8 x NT x 4 KiB.
// The kernel takes ~150 registers, one workgroup a CU; a build held to 128 (operands loaded a
// K-step at a time, no weight prefetch) spilled and ran 1.5x slower, so the host sends only
// grids of at most one and a half workgroups a CU here.
template <int NT>
__device__ __forceinline__ void gemm_q4k_few32_body(const GemmArgs& p, float* part) {
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r32 = lane & 31, half = lane >> 5;
    const int r0 = blockIdx.x * 32, t0 = blockIdx.y * 64;
    const int nsb = p.k / 256;
    const u32 ngrp = (u32)(p.tok_pad >> 5), grp0 = (u32)(t0 >> 5);
    const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc((void*)p.w, 0, -1, 0x00020000);
    const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc((void*)p.bq, 0, -1, 0x00020000);
    const __amdgpu_buffer_rsrc_t rd = __builtin_amdgcn_make_buffer_rsrc((void*)p.da, 0, -1, 0x00020000);
    const u32 vrow = (u32)min(r0 + r32, p.nrows - 1) * (u32)p.row_bytes;
    const u32 vq = vrow + 16u + 16u * (u32)half;
    const u32 va = ((u32)(2 * half) * 64u + (u32)r32) * 16u;   // fragment 2 half (+ j / 2), lane r32 (+ 32 (j % 2))
    const u32 vm = (u32)lane * 16u;                            // the sums' fragment as it lies
    const u32 vd = 16u * (u32)half;                            // tokens 4 half .. 4 half + 3 of each eight

    f32x16 out[NT];
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int e = 0; e < 16; e++) out[t][e] = 0.f;

    struct W { u32x4 hdr, q[4]; };
    auto load_w = [&](int sb, W& w) {
        const u32 so = (u32)sb * 144u;
        w.hdr = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rw, vrow, so, 0));
#pragma unroll
        for (int g = 0; g < 4; g++)
            w.q[g] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rw, vq + 32u * (u32)g, so, 0));
    };
    u32 mask = 0x000F000Fu, magic = 0x64006400u;
    asm volatile("" : "+v"(mask), "+v"(magic));

    W wcur, wnxt;
    if (wave < nsb) load_w(wave, wcur);
    for (int sb = wave; sb < nsb; sb += 8) {
        if (sb + 8 < nsb) load_w(sb + 8, wnxt);
        f32x16 accP[NT];
#pragma unroll
        for (int g = 0; g < 4; g++) {
            // activation operands of the group: [K-step j][token tile]
            f16x8 af[4 * NT];
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int t = 0; t < NT; t++) {
                    const u32 so = ((((u32)(2 * sb + (g >> 1)) * ngrp + grp0 + (u32)t) * JL_GEMM_ASTAGE_FRAGS +
                                     (u32)(4 * (g & 1) + (j >> 1))) * 64u + 32u * (u32)(j & 1)) * 16u;
                    af[j * NT + t] = __builtin_bit_cast(f16x8, __builtin_amdgcn_raw_buffer_load_b128(rb, va, so, 0));
                }
            __builtin_amdgcn_sched_barrier(0);   // the group's loads go out together, not one before each use
            // scales of sub-blocks 2g (low nibbles) and 2g+1 (high nibbles), straight from the
            // packed bytes (format/quant/dequant.go:360-365)
            const int sh = 16 * (g & 1);
            const u32 A = wcur.hdr.y >> sh, C = wcur.hdr.w >> sh;
            u32 slo, shi;
            if ((g >> 1) == 0) {
                slo = A & 63;
                shi = (A >> 8) & 63;
            } else {
                slo = (C & 0xF) | (((A >> 6) & 3) << 4);
                shi = ((C >> 8) & 0xF) | (((A >> 14) & 3) << 4);
            }
            const _Float16 flo = (_Float16)(float)slo, fhi = (_Float16)(float)shi;
            const _Float16 nlo = (_Float16)(-1024.0f * (float)slo), nhi = (_Float16)(-1024.0f * (float)shi);
            const f16x2 mlo = {flo, flo}, mhi = {fhi, fhi}, alo = {nlo, nlo}, ahi = {nhi, nhi};
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const u32 w = wcur.q[g][j];
                // (1024+n)*sc - 1024*sc = sc*n, exact in f16 (<= 945) through the fused multiply-add
                const f16x2 p0 = __builtin_elementwise_fma(nib_pair(w, 0, mask, magic), mlo, alo);
                const f16x2 p1 = __builtin_elementwise_fma(nib_pair(w, 4, mask, magic), mhi, ahi);
                const f16x2 p2 = __builtin_elementwise_fma(nib_pair(w, 8, mask, magic), mlo, alo);
                const f16x2 p3 = __builtin_elementwise_fma(nib_pair(w, 12, mask, magic), mhi, ahi);
                const f16x8 wf = {p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
                const f32x16 czero = {0};
#pragma unroll
                for (int t = 0; t < NT; t++)
                    accP[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[j * NT + t], wf, (g == 0 && j == 0) ? czero : accP[t],
                                                                     0, 0, 0);
            }
        }
        // minimum columns: lanes 0-31 hold m_0..m_7 (against the sums' low parts), lanes 32-63
        // 64 m_0..m_7 (against their high parts)
        f16x8 wm;
        {
            const float mul = half ? 64.0f : 1.0f;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                u32 scj, mnj;
                scale_min_k4(j, wcur.hdr.y, wcur.hdr.z, wcur.hdr.w, scj, mnj);
                wm[j] = (_Float16)((float)mnj * mul);
            }
        }
        const float dd = half_bits_to_f32((uint16_t)(wcur.hdr.x & 0xFFFF));
        const float dmin = half_bits_to_f32((uint16_t)(wcur.hdr.x >> 16));
#pragma unroll
        for (int t = 0; t < NT; t++) {
            const u32 som = ((((u32)(2 * sb + 1) * ngrp + grp0 + (u32)t) * JL_GEMM_ASTAGE_FRAGS + 8u) * 64u) * 16u;
            const f16x8 am = __builtin_bit_cast(f16x8, __builtin_amdgcn_raw_buffer_load_b128(rb, vm, som, 0));
            const f32x16 zero = {0};
            const f32x16 accM = __builtin_amdgcn_mfma_f32_32x32x16_f16(am, wm, zero, 0, 0, 0);
#pragma unroll
            for (int q = 0; q < 4; q++) {
                // tokens 8 q + 4 half + i of the tile
                const f32x4 da = __builtin_bit_cast(
                    f32x4, __builtin_amdgcn_raw_buffer_load_b128(
                               rd, vd, ((u32)sb * (u32)p.tok_pad + (u32)t0 + 32u * (u32)t + 8u * (u32)q) * 4u, 0));
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int e = 4 * q + i;
                    const float u = fmaf(dd, accP[t][e], -(dmin * accM[e]));
                    out[t][e] = fmaf(da[i], u, out[t][e]);
                }
            }
        }
        wcur = wnxt;
    }

    // the eight K shares, added in wavefront order; part [wave][tile][register][lane]
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int e = 0; e < 16; e++) part[((wave * NT + t) * 16 + e) * 64 + lane] = out[t][e];
    __syncthreads();
    for (int o = tid; o < NT * 1024; o += 512) {
        float s = part[o];
#pragma unroll
        for (int w = 1; w < 8; w++) s += part[w * NT * 1024 + o];
        const int t = o >> 10, e = (o >> 6) & 15, l = o & 63, r = r0 + (l & 31);
        const int tok = t0 + 32 * t + 8 * (e >> 2) + 4 * (l >> 5) + (e & 3);
        if (r < p.nrows && tok < p.ntok) p.out[(size_t)tok * p.out_stride + r] = s;
    }
}
