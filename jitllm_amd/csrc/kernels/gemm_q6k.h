// Prefill GEMM over Q6_K weights with the k-quant activation window of 256 (the window a
// model has when every matvec type is a k-quant, jit/cpu/matvec.go:46-62: a Q4_K_M file's
// Q6_K tensors).  Per (token, row) it is the decode matvec's value (format/quant/dequant.go:
// 443-470 for the weights, jit/cpu/packedgemm.go:54-58 for the identity with the matvec):
//
//   out[t][r] = sum_sb d_a[t,sb] * d[r,sb] * P[t,r,sb]
//   P = sum_{s,l} sc[r,s] * (q[r,s,l] - 32) * a[t,s,l]        16 sub-blocks s of 16 elements l
//
// P is a sum of products of small integers and runs exactly on the f16 matrix cores, as in
// the Q4_K kernel (gemm_q4k.h), with one difference: |sc * (q - 32)| reaches 4096 and f16
// holds odd integers only up to 2048.  So the scale is split, sc = 2 * (sc >> 1) + (sc & 1),
// and a weight becomes two f16 operands, 2 * (sc >> 1) * (q - 32) (even, <= 4096) and
// (sc & 1) * (q - 32): two matrix instructions a K-step into the same accumulator.  No
// minimum term: the zero point 32 is inside the operand.
//
// The K order inside a stage (half a super-block) is the Q4_K kernel's, so the activation
// fragments are the same prep kernel's: a 64-element group g = 2 * half + hh of the stage
// is the pair of 32-element runs (ql low or high nibbles by hh; first and second 32 bytes
// of the half's ql), word c of a run's sixteen-byte share holds elements 4c..4c+3, and the
// eight values of a word go out as (a0, a2, b0, b2, a1, a3, b1, b3), a from the first run,
// b from the second.
//
// A workgroup of four wavefronts owns 128 tokens x 64 rows; a wavefront 32 tokens x 64 rows.
// Per stage the 256 threads dequantize 64 rows x 128 weights into the two operand planes in
// LDS (thread = row, hh, half of the run: one 16-element sub-block of each run, so its two
// scales are scalars), the next stage's bytes already on their way; then every wavefront
// runs 32 matrix instructions against its activation fragments, which come from the
// workspace into a register ring a stage ahead.  Two workgroups share a CU and cover each
// other's vector phases.
// grid = (tok_pad/128, ceil(nrows/64), K splits), block = 256, dynamic LDS = JL_GEMM6_LDS_BYTES.
#pragma once
#include "gemm_q4k.h"

#define JL_GEMM6_LDS_BYTES (2 * 64 * JL_GEMM_STRIDE * 2)

struct Gemm6Raw {
    u32x4 qla, qlb, qh;
    u32 sc;   // the four int8 scales 8n + 4hh .. + 3
};

// K split: workgroup z takes sb_per super-blocks and writes its partial sums to slab z
__device__ __forceinline__ void gemm_q6k_split_slice(GemmArgs& p) {
    if (p.sb_per == 0) return;
    const int sb0 = blockIdx.z * p.sb_per;
    const int n = min(p.sb_per, p.k / 256 - sb0);
    p.w += (size_t)sb0 * 210;
    p.bq += (size_t)2 * sb0 * (p.tok_pad >> 5) * (JL_GEMM_ASTAGE_FRAGS * JL_GEMM_AFRAG_HALFS);
    p.da += (size_t)sb0 * p.tok_pad;
    p.k = 256 * n;
    p.out += (size_t)blockIdx.z * p.ntok * p.out_stride;
}

// t0, r0: the tile's first token and row.  SKIP (a grouped launch, which places tiles per expert and
// leaves many of them ragged): a wavefront whose tokens all lie past ntok loads and computes
// nothing.  Without it every wavefront walks the same loop (one without tokens works on the last
// group's fragments and stores nothing): the compiler sets the wait before a register's first use
// to the smallest count over all ways to get there, and with a branch round the matrix work the
// wait in front of the dequantization drained the fragment loads at every stage's head.
template <bool SKIP = false>
__device__ __forceinline__ void gemm_q6k_body(const GemmArgs& p, uint8_t* smem, int t0, int r0) {
    _Float16* sA = (_Float16*)smem;                 // [64][JL_GEMM_STRIDE]: 2 * (sc >> 1) * (q - 32)
    _Float16* sB = sA + 64 * JL_GEMM_STRIDE;        // (sc & 1) * (q - 32)
    const int tid = threadIdx.x, lane = tid & 63;
    const int tg = __builtin_amdgcn_readfirstlane(tid >> 6);   // this wavefront: tokens 32*tg..
    const bool live = !SKIP || t0 + 32 * tg < p.ntok;          // (SKIP) else no token of its 32 exists
    const int arow = lane & 31, kg = lane >> 5;
    const int nsb = p.k / 256, nsteps = 2 * nsb;
    // this thread's share of a weight stage
    const int srow = tid >> 2, hh = (tid >> 1) & 1, wq = tid & 1;
    const uint8_t* wrow = p.w + (size_t)min(r0 + srow, p.nrows - 1) * p.row_bytes;
    auto load_raw = [&](int step, Gemm6Raw& r) {
        const uint8_t* blk = wrow + (size_t)(step >> 1) * 210;
        const int n = step & 1;
        r.qla = ld16_a2(blk + 64 * n + 16 * wq);
        r.qlb = ld16_a2(blk + 64 * n + 32 + 16 * wq);
        r.qh = ld16_a2(blk + 128 + 32 * n + 16 * wq);
        r.sc = ld4_a2(blk + 192 + 8 * n + 4 * hh);
    };
    u32 m4 = 0x000F000Fu, m2 = 0x00300030u, magic = 0x64006400u;
    asm volatile("" : "+v"(m4), "+v"(m2), "+v"(magic));   // keep them in vector registers
    _Float16* dstA = sA + srow * JL_GEMM_STRIDE + 64 * hh + 32 * wq;
    _Float16* dstB = sB + srow * JL_GEMM_STRIDE + 64 * hh + 32 * wq;
    auto dequant = [&](const Gemm6Raw& r) {
        const i32 sa = (i32)(int8_t)(r.sc >> (8 * wq)), sb_ = (i32)(int8_t)(r.sc >> (8 * (2 + wq)));
        const _Float16 a2 = (_Float16)(float)(2 * (sa >> 1)), a0 = (_Float16)(float)(sa & 1);
        const _Float16 b2 = (_Float16)(float)(2 * (sb_ >> 1)), b0 = (_Float16)(float)(sb_ & 1);
        const f16x2 A2 = {a2, a2}, A0 = {a0, a0}, B2 = {b2, b2}, B0 = {b0, b0};
        const f16x2 off = {(_Float16)-1056.0f, (_Float16)-1056.0f};
        const int nsh = 4 * hh;
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const u32 wa = r.qla[c] >> nsh, wb = r.qlb[c] >> nsh;
            // the two high bits of an element, moved to bits 4-5 of its 16-bit half
            const u32 wh = hh ? r.qh[c] : r.qh[c] << 4;
            // (1024 + q) as f16, then q - 32: exact
            auto val = [&](u32 nib, u32 hi) {
                const u32 v = (hi & m2) | ((nib & m4) | magic);
                return __builtin_bit_cast(f16x2, v) + off;
            };
            const f16x2 ta02 = val(wa, wh), tb02 = val(wb, wh >> 2);
            const f16x2 ta13 = val(wa >> 8, wh >> 8), tb13 = val(wb >> 8, wh >> 10);
            auto word = [](f16x2 v) { return __builtin_bit_cast(u32, v); };
            const u32x4 oa = {word(ta02 * A2), word(tb02 * B2), word(ta13 * A2), word(tb13 * B2)};
            const u32x4 ob = {word(ta02 * A0), word(tb02 * B0), word(ta13 * A0), word(tb13 * B0)};
            *(u32x4*)(dstA + 8 * c) = oa;
            *(u32x4*)(dstB + 8 * c) = ob;
        }
    };
    // fragment (step, ks) of this wavefront's 32 tokens
    const size_t ngrp = (size_t)(p.tok_pad >> 5), mygrp = min((size_t)(t0 >> 5) + tg, ngrp - 1);
    auto a_frag = [&](int step, int ks) {
        return ((const f16x8*)p.bq)[(((size_t)step * ngrp + mygrp) * JL_GEMM_ASTAGE_FRAGS + ks) * 64 + lane];
    };
    // the rows of this lane's two output tiles: their super-block scale d
    const uint8_t* drow[2];
#pragma unroll
    for (int j = 0; j < 2; j++) drow[j] = p.w + (size_t)min(r0 + 32 * j + arow, p.nrows - 1) * p.row_bytes + 208;
    const float* dap = p.da + min(t0 + 32 * tg, p.tok_pad - 32) + 4 * kg;

    f32x16 out[2], acc[2];
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
        for (int e = 0; e < 16; e++) out[j][e] = 0.f;

    // Before the loop the loads go out in the loop's order: the weights, then the fragments in K order.
    Gemm6Raw raw;
    load_raw(0, raw);
    __builtin_amdgcn_sched_barrier(0);
    f16x8 aring[8];
    if (live) {
#pragma unroll
        for (int ks = 0; ks < 8; ks++) {
            aring[ks] = a_frag(0, ks);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    // One stage (half a super-block; the half is a compile-time constant, so the loads that
    // only the second half needs are no branch in the loop).
    auto stage = [&](auto HALF, int step) {
        constexpr int half = decltype(HALF)::value;
        const int sb = step >> 1;
        dequant(raw);
        load_raw(min(step + 1, nsteps - 1), raw);   // a whole stage of matrix work covers the latency
        uint16_t dbits[2] = {0, 0};
        f32x4 dav[4];
        if (half == 1 && live) {
#pragma unroll
            for (int j = 0; j < 2; j++) dbits[j] = ld2(drow[j] + (size_t)sb * 210);
#pragma unroll
            for (int i = 0; i < 4; i++) dav[i] = *(const f32x4*)(dap + (size_t)sb * p.tok_pad + 8 * i);
        }
        __builtin_amdgcn_sched_barrier(0);
        lds_barrier();
        if (live) {
            const int nstep = min(step + 1, nsteps - 1);
            const _Float16* wa0 = sA + arow * JL_GEMM_STRIDE + 8 * kg;
            const _Float16* wb0 = sB + arow * JL_GEMM_STRIDE + 8 * kg;
            const f32x16 czero = {0};
#pragma unroll
            for (int ks = 0; ks < 8; ks++) {
                f16x8 wfa[2], wfb[2];
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    wfa[j] = *(const f16x8*)(wa0 + 32 * j * JL_GEMM_STRIDE + 16 * ks);
                    wfb[j] = *(const f16x8*)(wb0 + 32 * j * JL_GEMM_STRIDE + 16 * ks);
                }
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    // (a super-block's first instruction starts from a zero accumulator operand)
                    acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(aring[ks], wfa[j],
                                                                    (half == 0 && ks == 0) ? czero : acc[j], 0, 0, 0);
                    acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(aring[ks], wfb[j], acc[j], 0, 0, 0);
                }
                // the next stage's fragment for this slot, requested HERE (left to itself the
                // scheduler gathers all eight behind the last matrix instruction, a trip to L2
                // before the next stage can start)
                aring[ks] = a_frag(nstep, ks);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (half) {
                // out += d_a * (d * P) for the super-block
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    const float dd = half_bits_to_f32(dbits[j]);
#pragma unroll
                    for (int e = 0; e < 16; e++) out[j][e] = fmaf(dav[e >> 2][e & 3], dd * acc[j][e], out[j][e]);
                }
            }
        }
        lds_barrier();
    };
    for (int step = 0; step < nsteps; step += 2) {
        stage(GemmIntC<0>{}, step);
        stage(GemmIntC<1>{}, step + 1);
    }
    if (SKIP && !live) return;
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
