// Prefill GEMM over Q4_K weights with the scales FOLDED into the f16 operands (an opt-in form).
//
// The exact forms (gemm_q4k.h) keep the integers apart from the scales,
//   out = sum_sb d_a * (d * P - dmin * M),
// and pay for it with three vector instructions an output element per super-block, a second
// accumulator set and a matrix instruction for M.  Here the operands carry the scales,
//   W16[r][k] = f16(d * sc * q - dmin * m)          the dequantized weight, rounded to f16
//   A16[t][k] = f16(d_a * a)                         the quantized activation, dequantized and rounded
//   out[t][r] = sum_k W16 * A16                      f32 accumulation on the matrix cores, all of K
// so a workgroup is a plain GEMM tile with on-the-fly dequantization: no epilogue, no minimum
// columns, one accumulator set.  The activations are still quantized to int8 first, as the
// reference's path does (jit/cpu/matvec.go:46-62); what differs from the exact forms is two
// roundings to f16 (2^-12 relative each, and the sub-block's f16(d * sc) and f16(dmin * m)
// shared by its 32 weights): rel-L2 against the exact result a few 1e-4, inside the path's 1e-3
// and measured wherever it is timed.  A weight whose |d| * 945 + |dmin| * 63 passes the f16 range
// cannot be folded: the host checks a matrix's scales before it uses this form.
//
// The dequantization: q as an exact f16 first ((nibble | 0x6400) reads 1024 + q; minus 1024),
// then ONE packed fma per pair, q * f16(d * sc) - f16(dmin * m), rounded once.  (The exact
// forms' trick of folding the 1024 into the addend would round it at the addend's magnitude.)
#pragma once
#include "gemm_q4k.h"

struct GemmFoldScale {
    f16x2 mlo, alo, mhi, ahi;
    _Float16* dst;
};

// sub-blocks 2g (low nibbles) and 2g + 1 (high nibbles), g = 2 * half + hh, of a GGUF header
__device__ __forceinline__ void gemm_fold_scale(const u32x4& hdr, int hh, int half, GemmFoldScale& k) {
    const float d = half_bits_to_f32((uint16_t)(hdr.x & 0xFFFF)), dmin = half_bits_to_f32((uint16_t)(hdr.x >> 16));
    const u32 sword = half ? ((hdr.w & 0x0F0F0F0Fu) | ((hdr.y >> 2) & 0x30303030u)) : (hdr.y & 0x3F3F3F3Fu);
    const u32 mword = half ? (((hdr.w >> 4) & 0x0F0F0F0Fu) | ((hdr.z >> 2) & 0x30303030u)) : (hdr.z & 0x3F3F3F3Fu);
    const u32 sp = sword >> (16 * hh), mp = mword >> (16 * hh);
    const _Float16 slo = (_Float16)(d * (float)(sp & 0xFF)), shi = (_Float16)(d * (float)((sp >> 8) & 0xFF) * 0.0625f);
    const _Float16 nlo = (_Float16)(-(dmin * (float)(mp & 0xFF))), nhi = (_Float16)(-(dmin * (float)((mp >> 8) & 0xFF)));
    k.mlo = f16x2{slo, slo};
    k.alo = f16x2{nlo, nlo};
    k.mhi = f16x2{shi, shi};   // high nibbles stay in place and read 16 q
    k.ahi = f16x2{nhi, nhi};
}
// plane form: all eight nibbles of a word belong to sub-block `sub`
__device__ __forceinline__ void gemm_fold_scale_planes(const u32x4& hdr, int sub, GemmFoldScale& k) {
    const float d = half_bits_to_f32((uint16_t)(hdr.x & 0xFFFF)), dmin = half_bits_to_f32((uint16_t)(hdr.x >> 16));
    const float sc = (float)gemm_stream_field(hdr, 2 * sub), m = (float)gemm_stream_field(hdr, 2 * sub + 1);
    const _Float16 slo = (_Float16)(d * sc), shi = (_Float16)(d * sc * 0.0625f), n = (_Float16)(-(dmin * m));
    k.mlo = f16x2{slo, slo};
    k.alo = f16x2{n, n};
    k.mhi = f16x2{shi, shi};
    k.ahi = f16x2{n, n};
}
// one 32-bit word of nibbles -> eight f16 weights -> 16 bytes of LDS at k.dst + 8 c
__device__ __forceinline__ void gemm_fold_word(u32 w, const GemmFoldScale& k, int c, u32 mask_lo, u32 mask_hi, u32 magic,
                                               f16x2 neg) {
    const u32 w8 = w >> 8;
    auto nib = [&](u32 v, u32 mask) { return __builtin_bit_cast(f16x2, (v & mask) | magic) + neg; };
    // (b0.lo, b2.lo), (b0.hi, b2.hi), (b1.lo, b3.lo), (b1.hi, b3.hi): the exact forms' K order
    const f16x2 p0 = __builtin_elementwise_fma(nib(w, mask_lo), k.mlo, k.alo);
    const f16x2 p1 = __builtin_elementwise_fma(nib(w, mask_hi), k.mhi, k.ahi);
    const f16x2 p2 = __builtin_elementwise_fma(nib(w8, mask_lo), k.mlo, k.alo);
    const f16x2 p3 = __builtin_elementwise_fma(nib(w8, mask_hi), k.mhi, k.ahi);
    const u32x4 o = {__builtin_bit_cast(u32, p0), __builtin_bit_cast(u32, p1), __builtin_bit_cast(u32, p2),
                     __builtin_bit_cast(u32, p3)};
    *(u32x4*)(k.dst + 8 * c) = o;
}

// The wide tile: 256 tokens x 128 rows a workgroup, 512 threads, a wavefront 32 tokens x all 128
// rows; the exact wide form's staging (two weight stages of half a super-block in LDS, the
// threads' shares, the activation ring a stage ahead, the fragments' addresses) with nothing but
// matrix instructions and the next stage's dequantization in the loop.  Weight fragments are read
// three slots ahead (the exact form has registers for one).
// grid = (tok_pad/256, ceil(nrows/128)), block = 512, dynamic LDS = JL_GEMM_FOLD_LDS_BYTES.
#define JL_GEMM_FOLD_LDS_BYTES (2 * 128 * JL_GEMM_WROW * 2)
template <bool PL = false>
__device__ __forceinline__ void gemm_q4k_fold_wide_body(const GemmArgs& p, uint8_t* smem) {
    constexpr int ROWS = 128, TOK = JL_GEMM_WIDE_TOK, STAGE_HALFS = ROWS * JL_GEMM_WROW, AHEAD = 3;
    _Float16* sW = (_Float16*)smem;   // [2 stages][128][136]
    const int tid = threadIdx.x, lane = tid & 63;
    const int tg = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int t0 = blockIdx.x * TOK, r0 = blockIdx.y * ROWS;
    const int nsteps = 2 * (p.k / 256);
    const int psub = tg >> 1;
    const int srow = PL ? 64 * (tg & 1) + lane : tid >> 2, hh = PL ? (psub & 1) : (tid >> 1) & 1, wq = tid & 1;
    const int arow = lane & 31, kg = lane >> 5;
    const size_t astride = (size_t)(p.tok_pad >> 5) * (JL_GEMM_ASTAGE_FRAGS * 1024);
    const char* abase = (const char*)p.bq + ((size_t)(t0 >> 5) + tg) * (JL_GEMM_ASTAGE_FRAGS * 1024);
    const unsigned aoff = lane * 16;
    auto a_frag = [&](int step, int ks) { return *(const f16x8*)(abase + (size_t)step * astride + ks * 1024 + aoff); };
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
    u32 mask_lo = 0x000F000Fu, mask_hi = 0x00F000F0u, magic = 0x64006400u, negbits = 0xE400E400u;   // -1024, -1024
    asm volatile("" : "+v"(mask_lo), "+v"(mask_hi), "+v"(magic), "+v"(negbits));
    const f16x2 neg = __builtin_bit_cast(f16x2, negbits);
    const int wdst = PL ? srow * JL_GEMM_WROW + 32 * psub : srow * JL_GEMM_WROW + 64 * hh + 32 * wq;
    auto scale_of = [&](const GemmWRegs& r, int step, GemmFoldScale& k) {
        if (PL) gemm_fold_scale_planes(r.hdr, 4 * (step & 1) + psub, k);
        else gemm_fold_scale(r.hdr, hh, step & 1, k);
    };

    f32x16 out[4];
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
        for (int e = 0; e < 16; e++) out[j][e] = 0.f;

    // The loads before the loop are issued in the loop's own order (a stage's weights, then the
    // activation fragments, then the next weights at the loop's head): the wait the compiler puts
    // before a register's first use is the smaller of the counts on the two ways into the loop,
    // and a shorter queue on the way in would drain the loop's queue every other stage.
    GemmWRegs wa, wb;
    load_w(0, wb);
    load_w(min(1, nsteps - 1), wa);
    __builtin_amdgcn_sched_barrier(0);
    f16x8 aring[8];
#pragma unroll
    for (int ks = 0; ks < 8; ks++) aring[ks] = a_frag(0, ks);
    __builtin_amdgcn_sched_barrier(0);
    {
        GemmFoldScale k0;
        scale_of(wb, 0, k0);
        asm volatile("" ::"v"(wb.hdr));   // see the loop
        k0.dst = sW + wdst;
#pragma unroll
        for (int c = 0; c < 4; c++) gemm_fold_word(wb.q[c], k0, c, mask_lo, mask_hi, magic, neg);
    }
    lds_barrier();

    auto stage = [&](auto HALF, int step, GemmWRegs& wcur, GemmWRegs& wnxt) {
        constexpr int half = decltype(HALF)::value;
        const _Float16* w = sW + half * STAGE_HALFS;
        _Float16* wnext = sW + (half ^ 1) * STAGE_HALFS;
        const int nstep = min(step + 1, nsteps - 1);
        load_w(min(step + 2, nsteps - 1), wnxt);
        const _Float16* wp0 = w + arow * JL_GEMM_WROW + 8 * kg;
        // unit u = (K-step u / 4, row tile u % 4): one fragment, one matrix instruction
        auto w_frag = [&](int u) { return *(const f16x8*)(wp0 + 32 * (u & 3) * JL_GEMM_WROW + 16 * (u >> 2)); };
        f16x8 wf[4];
        GemmFoldScale wsc;
        wsc.dst = wnext + wdst;
#pragma unroll
        for (int u = 0; u < AHEAD; u++) wf[u] = w_frag(u);
        __builtin_amdgcn_sched_barrier(0);
        gemm_static_for<0, 32>([&](auto U) __attribute__((always_inline)) {
            constexpr int u = decltype(U)::value, ks = u >> 2, j = u & 3;
            if (u + AHEAD < 32) wf[(u + AHEAD) & 3] = w_frag(u + AHEAD);
            out[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(aring[ks], wf[u & 3], out[j], 0, 0, 0);
            if (j == 3) aring[ks] = a_frag(nstep, ks);
            // the next stage's weights: the scales under the first K-step, a word under every
            // second one after it
            if (u == 1) {
                scale_of(wcur, half ^ 1, wsc);   // the last stage decodes a stage nobody reads
                // all four header words stay live to here: a word the scales of this half do not
                // read would otherwise be handed out as a temporary while its load is in flight,
                // and writing it waits for the load
                asm volatile("" ::"v"(wcur.hdr));
            }
            if (j == 1 && (ks & 1) == 1) gemm_fold_word(wcur.q[ks >> 1], wsc, ks >> 1, mask_lo, mask_hi, magic, neg);
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, 12, 0);
            __builtin_amdgcn_sched_barrier(0);
        });
        lds_barrier();
    };
    for (int step = 0; step < nsteps; step += 2) {
        stage(GemmIntC<0>{}, step, wa, wb);
        stage(GemmIntC<1>{}, step + 1, wb, wa);
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

// The same tile for four wavefronts: a wavefront owns 64 tokens x all 128 rows, so a weight
// fragment read from LDS feeds TWO matrix instructions (the one limit of the eight-wavefront
// form: a fragment of its own for every instruction is all the LDS can deliver) and the running
// sums are 128 registers -- which the exact forms cannot afford beside their integer sums.  Two
// workgroups a CU.  A thread dequantizes 64 weights a stage (row = tid / 2, the half's 64-element
// group tid % 2: header and 32 bytes of nibbles).
// grid = (tok_pad/256, ceil(nrows/128)), block = 256, dynamic LDS = JL_GEMM_FOLD_LDS_BYTES.
struct GemmFoldWRegs {
    u32x4 hdr, q0, q1;
};
__device__ __forceinline__ void gemm_q4k_fold_wide4_body(const GemmArgs& p, uint8_t* smem) {
    constexpr int ROWS = 128, TOK = JL_GEMM_WIDE_TOK, STAGE_HALFS = ROWS * JL_GEMM_WROW, AHEAD = 3;
    _Float16* sW = (_Float16*)smem;   // [2 stages][128][136]
    const int tid = threadIdx.x, lane = tid & 63;
    const int tg = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int t0 = blockIdx.x * TOK, r0 = blockIdx.y * ROWS;
    const int nsteps = 2 * (p.k / 256);
    const int srow = tid >> 1, hh = tid & 1;
    const int arow = lane & 31, kg = lane >> 5;
    const size_t astride = (size_t)(p.tok_pad >> 5) * (JL_GEMM_ASTAGE_FRAGS * 1024);
    const char* abase = (const char*)p.bq + ((size_t)(t0 >> 5) + 2 * tg) * (JL_GEMM_ASTAGE_FRAGS * 1024);
    const unsigned aoff = lane * 16;
    auto a_frag = [&](int step, int ks, int h) {
        return *(const f16x8*)(abase + (size_t)step * astride + h * (JL_GEMM_ASTAGE_FRAGS * 1024) + ks * 1024 + aoff);
    };
    const uint8_t* wbase = p.w + (size_t)r0 * p.row_bytes;
    const unsigned woff = (unsigned)(min(r0 + srow, p.nrows - 1) - r0) * (unsigned)p.row_bytes;
    const unsigned wqoff = woff + 16 + 32 * hh;
    auto load_w = [&](int step, GemmFoldWRegs& r) {
        const uint8_t* blk = wbase + (size_t)(step >> 1) * 144;
        r.hdr = ld16(blk + woff);
        r.q0 = ld16(blk + 64 * (step & 1) + wqoff);
        r.q1 = ld16(blk + 64 * (step & 1) + wqoff + 16);
    };
    u32 mask_lo = 0x000F000Fu, mask_hi = 0x00F000F0u, magic = 0x64006400u, negbits = 0xE400E400u;   // -1024, -1024
    asm volatile("" : "+v"(mask_lo), "+v"(mask_hi), "+v"(magic), "+v"(negbits));
    const f16x2 neg = __builtin_bit_cast(f16x2, negbits);
    const int wdst = srow * JL_GEMM_WROW + 64 * hh;
    auto word_of = [&](const GemmFoldWRegs& r, int c) { return c < 4 ? r.q0[c & 3] : r.q1[c & 3]; };

    f32x16 out[2][4];
#pragma unroll
    for (int h = 0; h < 2; h++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) out[h][j][e] = 0.f;

    // loads before the loop in the loop's own order, as in the eight-wavefront form
    GemmFoldWRegs wa, wb;
    load_w(0, wb);
    load_w(min(1, nsteps - 1), wa);
    __builtin_amdgcn_sched_barrier(0);
    // activation fragments four K-steps (32 matrix instructions) ahead: a whole stage ahead, as
    // the eight-wavefront form has them, would spill
    f16x8 aring[4][2];
#pragma unroll
    for (int ks = 0; ks < 4; ks++)
#pragma unroll
        for (int h = 0; h < 2; h++) aring[ks][h] = a_frag(0, ks, h);
    __builtin_amdgcn_sched_barrier(0);
    {
        GemmFoldScale k0;
        gemm_fold_scale(wb.hdr, hh, 0, k0);
        asm volatile("" ::"v"(wb.hdr));   // see the loop
        k0.dst = sW + wdst;
#pragma unroll
        for (int c = 0; c < 8; c++) gemm_fold_word(word_of(wb, c), k0, c, mask_lo, mask_hi, magic, neg);
    }
    lds_barrier();

    auto stage = [&](auto HALF, int step, GemmFoldWRegs& wcur, GemmFoldWRegs& wnxt) {
        constexpr int half = decltype(HALF)::value;
        const _Float16* w = sW + half * STAGE_HALFS;
        _Float16* wnext = sW + (half ^ 1) * STAGE_HALFS;
        const int nstep = min(step + 1, nsteps - 1);
        load_w(min(step + 2, nsteps - 1), wnxt);
        const _Float16* wp0 = w + arow * JL_GEMM_WROW + 8 * kg;
        // fragment f = (K-step f / 4, row tile f % 4): two matrix instructions, one a token half
        auto w_frag = [&](int f) { return *(const f16x8*)(wp0 + 32 * (f & 3) * JL_GEMM_WROW + 16 * (f >> 2)); };
        f16x8 wf[4];
        GemmFoldScale wsc;
        wsc.dst = wnext + wdst;
#pragma unroll
        for (int f = 0; f < AHEAD; f++) wf[f] = w_frag(f);
        __builtin_amdgcn_sched_barrier(0);
        gemm_static_for<0, 32>([&](auto F) __attribute__((always_inline)) {
            constexpr int f = decltype(F)::value, ks = f >> 2, j = f & 3;
            if (f + AHEAD < 32) wf[(f + AHEAD) & 3] = w_frag(f + AHEAD);
#pragma unroll
            for (int h = 0; h < 2; h++)
                out[h][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(aring[ks & 3][h], wf[f & 3], out[h][j], 0, 0, 0);
            if (j == 3) {
#pragma unroll
                for (int h = 0; h < 2; h++) aring[ks & 3][h] = ks < 4 ? a_frag(step, ks + 4, h) : a_frag(nstep, ks - 4, h);
            }
            // the next stage's weights: the scales under the first fragment, a word under the
            // second fragment of every K-step
            if (f == 0) {
                gemm_fold_scale(wcur.hdr, hh, (half ^ 1), wsc);
                asm volatile("" ::"v"(wcur.hdr));   // as in the eight-wavefront form
            }
            if (j == 1) gemm_fold_word(word_of(wcur, ks), wsc, ks, mask_lo, mask_hi, magic, neg);
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, 8, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, 24, 0);
            __builtin_amdgcn_sched_barrier(0);
        });
        lds_barrier();
    };
    for (int step = 0; step < nsteps; step += 2) {
        stage(GemmIntC<0>{}, step, wa, wb);
        stage(GemmIntC<1>{}, step + 1, wb, wa);
    }

#pragma unroll
    for (int h = 0; h < 2; h++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int r = r0 + 32 * j + arow;
            if (r >= p.nrows) continue;
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const int t = t0 + 64 * tg + 32 * h + 8 * (e >> 2) + 4 * kg + (e & 3);
                if (t < p.ntok) p.out[(size_t)t * p.out_stride + r] = out[h][j][e];
            }
        }
}
