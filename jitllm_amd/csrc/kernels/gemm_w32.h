// Prefill GEMM with the activation window of 32 (the window of a model that holds a type
// with 32-element blocks, jit/cpu/matvec.go:46-62), Q8_0, Q6_K and Q4_K weights.  Per (token,
// row) it is the decode matvec's value (format/quant/dequant.go:148-157, :443-470 and :360-397
// for the weights, jit/cpu/packedgemm.go:54-58 for the identity with the matvec):
//
//   out[t][r] = sum_b d[r,b] * d_a[t,b] * P[t,r,b],   P = sum_{l<32} q[r,b,l] * a[t,b,l]
//
// P is a sum of products of int8 values and runs exactly on the f16 matrix cores
// (v_mfma_f32_32x32x16_f16, two K-steps a block); both scales change every 32 weights, so
// the f32 epilogue runs once per block: two vector instructions an output element per two
// matrix instructions, which is what bounds the kernel (the matrix cores wait).
// Q6_K: q is sc * (q6 - 32) with the int8 sub-block scale split into two exact f16 operands
// as in gemm_q6k.h (two planes in LDS, four matrix instructions a K-step pair and tile), d
// the super-block's.
// Q4_K: q is the nibble, d the product d * sc of the 32-element sub-block, and the minimum
// joins as  - (dmin * m) * (d_a * sum of the block's activations), the second factor from
// the prep: a third vector instruction an element.
//
// Activation prep (gemm_prep_w32_body): x [ntok][k] f32 -> bq [k/128 stages][tok_pad/32]
// [8 K-steps][64 lanes][8] f16 and da [k/32][tok_pad] f32.  Lane (t = lane%32, kg = lane/32)
// of K-step ks holds K positions 16*ks + 8*kg + (0, 2, 1, 3, 4, 6, 5, 7) of the stage: the
// order in which the byte unpack below emits a 32-bit word of weights.
// grid = (ceil(k/256), tok_pad/32), block = 256.
//
// Matrix kernel: a workgroup of four wavefronts owns 128 tokens x 64 rows, a wavefront 32
// tokens x 64 rows.  Per stage (128 weights = four blocks a row) the 256 threads turn 64 rows
// into f16 in LDS (thread = row, block: 32 bytes, xor 0x80 and the 1024 + byte trick), with
// the rows' block scales and the tile's token scales beside them; then every wavefront runs
// its sixteen matrix instructions, the block epilogue after every second K-step.  Workgroups
// that share a CU cover each other's vector phases.  Q6_K: thread = row, 32-element run of the
// half super-block (ql nibbles + two qh bits, two sub-block scales).
// grid = (tok_pad/128, ceil(nrows/64), K splits), block = 256, dynamic LDS =
// JL_GEMM32_LDS_BYTES(planes), planes = 1 (Q8_0, Q4_K) or 2 (Q6_K).
#pragma once
#include "gemm_q4k.h"

#define JL_GEMM32_FRAGS 8
#define JL_GEMM32_LDS_BYTES(planes) ((planes) * 64 * JL_GEMM_STRIDE * 2 + 2 * 64 * 4 * 4 + 2 * 4 * JL_GEMM_TILE * 4)

__device__ __forceinline__ void gemm_prep_w32_body(const GemmPrepArgs& p, u32* sq) {
    // sq [32 tokens][65]: 64 words of int8 + 1 pad (bank spread)
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int ch = blockIdx.x, grp = blockIdx.y, ngrp = p.tok_pad >> 5;
    const int e0 = ch * 256 + 4 * lane;   // this lane's four elements
    f32x4 v[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const int t = grp * 32 + wave * 8 + i;
        v[i] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (t < p.ntok && e0 < p.k) v[i] = *(const f32x4*)(p.x + (size_t)t * p.k + e0);
    }
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const int tl = wave * 8 + i;
        const u32 m = max(max(abs_bits(v[i].x), abs_bits(v[i].y)), max(abs_bits(v[i].z), abs_bits(v[i].w)));
        const u32 amax = window_amax(m, 1);
        float d;
        i32 sum16;
        sq[tl * 65 + lane] = quantize4(v[i], amax, d, sum16);
        // the block's sum from its two half-block sums (eight lanes a block)
        const i32 a32 = sum16 + dpp_i32<JL_DPP_ROW_HALF_MIRROR, 0xf>(0, sum16);
        if ((lane & 7) == 0 && e0 < p.k) {
            const size_t at = (size_t)(ch * 8 + (lane >> 3)) * p.tok_pad + grp * 32 + tl;
            p.da[at] = d;
            if (p.dsum) p.dsum[at] = d * (float)a32;
        }
    }
    __syncthreads();
    const int tl = lane & 31, kg = lane >> 5;
    u32x4* dst = (u32x4*)p.bq;
    const int nstage = p.k / 128;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int pi = wave * 4 + i, h = pi >> 3, ks = pi & 7;
        const int stage = 2 * ch + h;
        if (stage >= nstage) continue;
        const int w0 = 32 * h + 4 * ks + 2 * kg;
        const u32 lo = sq[tl * 65 + w0], hi = sq[tl * 65 + w0 + 1];
        auto f = [](u32 w, int b) { return (_Float16)(float)(int8_t)(w >> (8 * b)); };
        const f16x8 o = {f(lo, 0), f(lo, 2), f(lo, 1), f(lo, 3), f(hi, 0), f(hi, 2), f(hi, 1), f(hi, 3)};
        dst[(((size_t)stage * ngrp + grp) * JL_GEMM32_FRAGS + ks) * 64 + lane] = __builtin_bit_cast(u32x4, o);
    }
}

struct Gemm32Raw {
    u32x4 q0, q1;   // Q8_0: the block's 32 int8; Q6_K: the run's 32 ql bytes
    u32x4 h0, h1;   // Q6_K: the half's 32 qh bytes
    u32 d;          // Q8_0: the block's f16 scale; Q6_K: d | the run's two int8 scales << 16
    float da[2];    // two of the stage's 4 x 128 token scales
    float ds[2];    // Q4_K: and of its d_a * block sums
};

template <int TYPE>
__device__ __forceinline__ void gemm_w32_body(const GemmArgs& p0, uint8_t* smem) {
    constexpr bool Q6 = TYPE == JL_Q6_K, Q4 = TYPE == JL_Q4_K;
    constexpr int NPL = Q6 ? 2 : 1;
    constexpr int SB_BYTES = Q6 ? 210 : 144;   // k-quants: a stage is half a super-block
    GemmArgs p = p0;
    if (p.sb_per) {   // K split: sb_per stages to a workgroup (k-quants: an even number), partial sums to slab z
        const int s0 = blockIdx.z * p.sb_per;
        const int n = min(p.sb_per, p.k / 128 - s0);
        p.w += Q6 || Q4 ? (size_t)(s0 / 2) * SB_BYTES : (size_t)s0 * 4 * 34;
        if (Q4) p.dsum += (size_t)s0 * 4 * p.tok_pad;
        p.bq += (size_t)s0 * (p.tok_pad >> 5) * (JL_GEMM32_FRAGS * JL_GEMM_AFRAG_HALFS);
        p.da += (size_t)s0 * 4 * p.tok_pad;
        p.k = 128 * n;
        p.out += (size_t)blockIdx.z * p.ntok * p.out_stride;
    }
    const int t0 = blockIdx.x * JL_GEMM_TILE, r0 = blockIdx.y * 64;
    _Float16* sW = (_Float16*)smem;                            // [planes][64][JL_GEMM_STRIDE]
    float* sD = (float*)(sW + NPL * 64 * JL_GEMM_STRIDE);      // [64 rows][4 blocks]
    float* sD2 = sD + 64 * 4;                                  // Q4_K: dmin * m, [64 rows][4 blocks]
    float* sDa = sD2 + 64 * 4;                                 // [4 blocks][128 tokens]
    float* sDs = sDa + 4 * JL_GEMM_TILE;                       // Q4_K: d_a * block sum, [4 blocks][128 tokens]
    const int tid = threadIdx.x, lane = tid & 63;
    const int tg = __builtin_amdgcn_readfirstlane(tid >> 6);   // this wavefront: tokens 32*tg..
    const bool live = t0 + 32 * tg < p.ntok;                   // else no token of its 32 exists
    const int arow = lane & 31, kg = lane >> 5;
    const int nsteps = p.k / 128;
    // this thread's share of a weight stage: one block (run) of one row
    const int srow = tid >> 2, qb = tid & 3;
    const uint8_t* wrow = p.w + (size_t)min(r0 + srow, p.nrows - 1) * p.row_bytes;
    const float* dsrc = p.da + (size_t)(tid >> 7) * p.tok_pad + t0 + (tid & 127);   // blocks tid/128 and + 2
    auto load_raw = [&](int step, Gemm32Raw& r) {
        if constexpr (Q6) {
            const uint8_t* blk = wrow + (size_t)(step >> 1) * 210;
            const int n = step & 1;
            r.q0 = ld16_a2(blk + 64 * n + 32 * (qb & 1));
            r.q1 = ld16_a2(blk + 64 * n + 32 * (qb & 1) + 16);
            r.h0 = ld16_a2(blk + 128 + 32 * n);
            r.h1 = ld16_a2(blk + 128 + 32 * n + 16);
            r.d = (u32)ld2(blk + 208) | ((u32)ld2(blk + 192 + 8 * n + 2 * qb) << 16);
        } else if constexpr (Q4) {
            // sub-block 4 * n + qb: nibble qb % 2 of the 32 bytes of group 2 * n + qb / 2
            const uint8_t* blk = wrow + (size_t)(step >> 1) * 144;
            const int g = 2 * (step & 1) + (qb >> 1);
            r.h0 = ld16_a2(blk);
            r.q0 = ld16_a2(blk + 16 + 32 * g);
            r.q1 = ld16_a2(blk + 32 + 32 * g);
            r.d = (u32)(4 * (step & 1) + qb);
            r.ds[0] = (p.dsum + (dsrc - p.da))[(size_t)(4 * step) * p.tok_pad];
            r.ds[1] = (p.dsum + (dsrc - p.da))[(size_t)(4 * step + 2) * p.tok_pad];
        } else {
            const uint8_t* blk = wrow + (size_t)(4 * step + qb) * 34;
            r.d = ld2(blk);
            r.q0 = ld16_a2(blk + 2);
            r.q1 = ld16_a2(blk + 18);
        }
        r.da[0] = dsrc[(size_t)(4 * step) * p.tok_pad];
        r.da[1] = dsrc[(size_t)(4 * step + 2) * p.tok_pad];
    };
    u32 m8 = Q6 || Q4 ? 0x000F000Fu : 0x00FF00FFu, m2 = 0x00300030u, magic = 0x64006400u;
    asm volatile("" : "+v"(m8), "+v"(m2), "+v"(magic));   // keep them in vector registers
    _Float16* dst = sW + srow * JL_GEMM_STRIDE + 32 * qb;
    auto dequant = [&](const Gemm32Raw& r) {
        auto word = [](f16x2 v) { return __builtin_bit_cast(u32, v); };
        if constexpr (Q6) {
            // run qb of the half: nibble qb/2 of the ql bytes, qh bits 2*qb; elements 0-15 and
            // 16-31 are sub-blocks with their own scale, each split as 2 * (sc >> 1) + (sc & 1)
            const f16x2 off = {(_Float16)-1056.0f, (_Float16)-1056.0f};
            const int nsh = 4 * (qb >> 1), hsh = 2 * qb;
#pragma unroll
            for (int half = 0; half < 2; half++) {
                const i32 sc = (i32)(int8_t)(r.d >> (16 + 8 * half));
                const _Float16 s2 = (_Float16)(float)(2 * (sc >> 1)), s0 = (_Float16)(float)(sc & 1);
                const f16x2 S2 = {s2, s2}, S0 = {s0, s0};
                const u32x4 ql = half ? r.q1 : r.q0, qh = half ? r.h1 : r.h0;
#pragma unroll
                for (int i = 0; i < 2; i++) {
                    f16x2 t[4];
#pragma unroll
                    for (int c = 0; c < 2; c++) {
                        const u32 wn = ql[2 * i + c] >> nsh;
                        // the two high bits of an element at bits 4-5 of its 16-bit half
                        const u32 wh = (qh[2 * i + c] >> hsh) << 4;
                        const u32 v02 = (wh & m2) | ((wn & m8) | magic);
                        const u32 v13 = ((wh >> 8) & m2) | (((wn >> 8) & m8) | magic);
                        t[2 * c] = __builtin_bit_cast(f16x2, v02) + off;      // (1024 + q) - 1056: exact
                        t[2 * c + 1] = __builtin_bit_cast(f16x2, v13) + off;
                    }
                    const u32x4 oa = {word(t[0] * S2), word(t[1] * S2), word(t[2] * S2), word(t[3] * S2)};
                    const u32x4 ob = {word(t[0] * S0), word(t[1] * S0), word(t[2] * S0), word(t[3] * S0)};
                    *(u32x4*)(dst + 16 * half + 8 * i) = oa;
                    *(u32x4*)(dst + 64 * JL_GEMM_STRIDE + 16 * half + 8 * i) = ob;
                }
            }
            sD[srow * 4 + qb] = half_bits_to_f32((uint16_t)(r.d & 0xFFFF));
        } else if constexpr (Q4) {
            const f16x2 off = {(_Float16)-1024.0f, (_Float16)-1024.0f};
            const int nsh = 4 * (qb & 1);
            // nibbles of bytes (b0, b2) and (b1, b3) of a word as 1024 + q, then q: exact
            auto pair = [&](u32 w) {
                const u32 v = (w & m8) | magic;
                return word(__builtin_bit_cast(f16x2, v) + off);
            };
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const u32 wa = (i < 2 ? r.q0[2 * i] : r.q1[2 * i - 4]) >> nsh;
                const u32 wb = (i < 2 ? r.q0[2 * i + 1] : r.q1[2 * i - 3]) >> nsh;
                const u32x4 o = {pair(wa), pair(wa >> 8), pair(wb), pair(wb >> 8)};
                *(u32x4*)(dst + 8 * i) = o;
            }
            u32 sc, mn;
            scale_min_k4((int)r.d, r.h0.y, r.h0.z, r.h0.w, sc, mn);
            sD[srow * 4 + qb] = half_bits_to_f32((uint16_t)(r.h0.x & 0xFFFF)) * (float)sc;
            sD2[srow * 4 + qb] = half_bits_to_f32((uint16_t)(r.h0.x >> 16)) * (float)mn;
            sDs[tid] = r.ds[0];
            sDs[256 + tid] = r.ds[1];
        } else {
            const f16x2 off = {(_Float16)-1152.0f, (_Float16)-1152.0f};
            // bytes (b0, b2) and (b1, b3) of a word as 1024 + (q + 128), then q: exact
            auto pair = [&](u32 w) {
                const u32 v = (w & m8) | magic;
                return word(__builtin_bit_cast(f16x2, v) + off);
            };
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const u32 wa = (i < 2 ? r.q0[2 * i] : r.q1[2 * i - 4]) ^ 0x80808080u;
                const u32 wb = (i < 2 ? r.q0[2 * i + 1] : r.q1[2 * i - 3]) ^ 0x80808080u;
                const u32x4 o = {pair(wa), pair(wa >> 8), pair(wb), pair(wb >> 8)};
                *(u32x4*)(dst + 8 * i) = o;
            }
            sD[srow * 4 + qb] = half_bits_to_f32((uint16_t)r.d);
        }
        sDa[tid] = r.da[0];
        sDa[256 + tid] = r.da[1];
    };
    // fragment (step, ks) of this wavefront's 32 tokens
    const size_t ngrp = (size_t)(p.tok_pad >> 5), mygrp = (size_t)(t0 >> 5) + tg;
    auto a_frag = [&](int step, int ks) {
        return ((const f16x8*)p.bq)[(((size_t)step * ngrp + mygrp) * JL_GEMM32_FRAGS + ks) * 64 + lane];
    };

    f32x16 out[2], acc[2];
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
        for (int e = 0; e < 16; e++) out[j][e] = 0.f;

    Gemm32Raw raw;
    load_raw(0, raw);
    f16x8 aring[8];
    if (live) {
#pragma unroll
        for (int ks = 0; ks < 8; ks++) aring[ks] = a_frag(0, ks);
    }
    for (int step = 0; step < nsteps; step++) {
        dequant(raw);
        load_raw(min(step + 1, nsteps - 1), raw);   // a whole stage of matrix work covers the latency
        lds_barrier();
        if (live) {
            const int nstep = min(step + 1, nsteps - 1);
            const _Float16* w0 = sW + arow * JL_GEMM_STRIDE + 8 * kg;
            const f32x16 czero = {0};
#pragma unroll
            for (int b = 0; b < 4; b++) {
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    const int ks = 2 * b + h;
                    f16x8 wf[NPL][2];
#pragma unroll
                    for (int pl = 0; pl < NPL; pl++)
#pragma unroll
                        for (int j = 0; j < 2; j++)
                            wf[pl][j] = *(const f16x8*)(w0 + (pl * 64 + 32 * j) * JL_GEMM_STRIDE + 16 * ks);
#pragma unroll
                    for (int j = 0; j < 2; j++) {
                        acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(aring[ks], wf[0][j], h ? acc[j] : czero, 0, 0, 0);
                        if constexpr (Q6) acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(aring[ks], wf[1][j], acc[j], 0, 0, 0);
                    }
                    aring[ks] = a_frag(nstep, ks);
                }
                // out += d_a * (d * P) for the block
                f32x4 dav[4];
#pragma unroll
                for (int i = 0; i < 4; i++) dav[i] = *(const f32x4*)(sDa + b * JL_GEMM_TILE + 32 * tg + 8 * i + 4 * kg);
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    const float dd = sD[(32 * j + arow) * 4 + b];
#pragma unroll
                    for (int e = 0; e < 16; e++) out[j][e] = fmaf(dav[e >> 2][e & 3], dd * acc[j][e], out[j][e]);
                }
                if constexpr (Q4) {
                    f32x4 dsv[4];
#pragma unroll
                    for (int i = 0; i < 4; i++) dsv[i] = *(const f32x4*)(sDs + b * JL_GEMM_TILE + 32 * tg + 8 * i + 4 * kg);
#pragma unroll
                    for (int j = 0; j < 2; j++) {
                        const float nm = -sD2[(32 * j + arow) * 4 + b];
#pragma unroll
                        for (int e = 0; e < 16; e++) out[j][e] = fmaf(dsv[e >> 2][e & 3], nm, out[j][e]);
                    }
                }
            }
        }
        lds_barrier();
    }
    if (!live) return;
    // store: lane = row (contiguous in memory), register = token
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int r = r0 + 32 * j + arow;
        if (r >= p.nrows) continue;
#pragma unroll
        for (int e = 0; e < 16; e++) {
            const int t = t0 + 32 * tg + 8 * (e >> 2) + 4 * kg + (e & 3);
            if (t < p.ntok) p.out[(size_t)t * p.out_stride + r] = out[j][e];
        }
    }
}
