// Prefill GEMM over Q4_K weights, the form for grids that the 256-token x 128-row tile
// cannot fill without cutting K across workgroups (jit/cpu/packedgemm.go:37-75 is the
// reference's weight-stationary kernel; engine/nn/packedmm.go:23-139 its driver).
//
// A workgroup owns 128 tokens x 64 rows over the WHOLE of K, so a matmul of 512 tokens x
// 4096 rows is 256 workgroups, one a CU, and nothing is left to add afterwards.  Its eight
// wavefronts are two groups of four: group kh walks half of the super-blocks with the
// machinery of the wide tile (gemm_q4k.h) -- its own double-buffered weight stages in LDS,
// dequantized by its 256 threads between its matrix instructions; activation fragments from
// L2 straight into a register ring a stage ahead -- and wavefront (tg, kh) accumulates
// 32 tokens x 64 rows.  The two groups' sums meet in LDS at the end, group 0's first, so the
// result does not depend on timing.
//
// The super-block epilogue  out += d_a * (d * P - dmin * M)  of super-block s runs under the
// matrix instructions of super-block s + 1: P has two register sets, by super-block parity,
// and so have the minimum columns, the row scales and the token scales in LDS.  Tile 0's
// epilogue takes the even slots of the next super-block's first stage, tile 1's those of its
// second stage; the odd slots carry the next stage's dequantization.
#pragma once
#include "gemm_q4k.h"

#define JL_GEMM_K2_TOK 128
#define JL_GEMM_K2_ROWS 64
// per group: two weight stages [64][136] f16, minimum columns [2][64][24] f16, row scales
// [2][64][2] f32, token scales [2][128] f32
#define JL_GEMM_K2_GROUP_BYTES \
    (2 * JL_GEMM_K2_ROWS * JL_GEMM_WROW * 2 + 2 * JL_GEMM_K2_ROWS * JL_GEMM_MROW * 2 + 2 * JL_GEMM_K2_ROWS * 2 * 4 + \
     2 * JL_GEMM_K2_TOK * 4)
#define JL_GEMM_K2_LDS_BYTES (2 * JL_GEMM_K2_GROUP_BYTES)

// grid = (tok_pad/128, ceil(nrows/64)), block = 512, dynamic LDS = JL_GEMM_K2_LDS_BYTES.
// k/256 is a multiple of four (each group walks an even number of super-blocks).
// PL: the weights come from packed planes; thread = (row = lane, sub-block of the stage =
// wavefront of the group), the stage's K order is the planes' (the prep kernel's PL order).
template <bool PL = false>
__device__ __forceinline__ void gemm_q4k_k2_body(const GemmArgs& p, uint8_t* smem) {
    constexpr int ROWS = JL_GEMM_K2_ROWS, TOK = JL_GEMM_K2_TOK, STAGE_HALFS = ROWS * JL_GEMM_WROW;
    constexpr int MIN_HALFS = ROWS * JL_GEMM_MROW;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int tg = wave & 3, kh = wave >> 2;
    uint8_t* gmem = smem + kh * JL_GEMM_K2_GROUP_BYTES;
    _Float16* sW = (_Float16*)gmem;                  // [2 stages][64][136]
    _Float16* sMin = sW + 2 * STAGE_HALFS;           // [2 parities][64][24]
    float* sScale = (float*)(sMin + 2 * MIN_HALFS);  // [2][64][2]  (d, dmin)
    float* sDa = sScale + 2 * 2 * ROWS;              // [2][128]

    const int t0 = blockIdx.x * TOK, r0 = blockIdx.y * ROWS;
    const int nsbg = (p.k / 256) >> 1, sb0 = kh * nsbg;   // this group's super-blocks
    const int nsteps = 2 * nsbg;
    const int gt = tid & 255;                             // thread of the group
    const int psub = tg;   // plane form: this thread's sub-block of a stage
    const int srow = PL ? lane : gt >> 2, hh = PL ? (psub & 1) : (gt >> 1) & 1, wq = gt & 1;
    const int arow = lane & 31, kg = lane >> 5;

    // activation fragment (stage of the group, K-step) of this wavefront's 32 tokens: a uniform
    // base plus the lane's 16 bytes
    const size_t astride = (size_t)(p.tok_pad >> 5) * (JL_GEMM_ASTAGE_FRAGS * 1024);
    const char* abase = (const char*)p.bq + ((size_t)(t0 >> 5) + tg) * (JL_GEMM_ASTAGE_FRAGS * 1024) +
                        (size_t)(2 * sb0) * astride;
    const unsigned aoff = lane * 16;
    auto a_frag = [&](int step, int ks) {
        return *(const f16x8*)(abase + (size_t)step * astride + ks * 1024 + aoff);
    };
    // this thread's share of a weight stage: the block header and 16 bytes of nibbles
    const uint8_t* wbase = p.w + (size_t)r0 * p.row_bytes + (size_t)sb0 * 144;
    const unsigned woff = (unsigned)(min(r0 + srow, p.nrows - 1) - r0) * (unsigned)p.row_bytes;
    const unsigned wqoff = woff + 16 + 32 * hh + 16 * wq;
    const int prow = min(r0 + srow, p.nrows - 1);
    auto load_w = [&](int step, GemmWRegs& r) {
        if (PL) {
            gemm_load_w_planes(p, prow, sb0 + (step >> 1), 4 * (step & 1) + psub, r);
        } else {
            const uint8_t* blk = wbase + (size_t)(step >> 1) * 144;
            r.hdr = ld16(blk + woff);
            r.q = ld16(blk + 64 * (step & 1) + wqoff);
        }
    };
    auto w_scale = [&](const u32x4& hdr, int half, GemmWideScale& k) __attribute__((always_inline)) {
        if (PL) gemm_wide_scale_planes(hdr, 4 * half + psub, k);
        else gemm_wide_scale(hdr, hh, half, k);
    };
    u32 mask_lo = 0x000F000Fu, mask_hi = 0x00F000F0u, magic = 0x64006400u;
    asm volatile("" : "+v"(mask_lo), "+v"(mask_hi), "+v"(magic));   // keep them in vector registers
    const int wdst = PL ? srow * JL_GEMM_WROW + 32 * psub : srow * JL_GEMM_WROW + 64 * hh + 32 * wq;
    const float* dag = p.da + (size_t)sb0 * p.tok_pad + t0 + (gt & (TOK - 1));

    f32x16 out[2], accP[2][2];
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
        for (int e = 0; e < 16; e++) out[j][e] = 0.f;

    // prologue: stage 0 of the weights into LDS, stage 1 into registers, the first
    // activation fragments into the ring
    GemmWRegs wa, wb;
    load_w(0, wa);
    f16x8 aring[8], aaug[2];
#pragma unroll
    for (int ks = 0; ks < 8; ks++) aring[ks] = a_frag(0, ks);
    aaug[0] = aaug[1] = aring[0];   // (each is loaded a stage before its first use)
    {
        GemmWideScale k0;
        w_scale(wa.hdr, 0, k0);
        k0.dst = sW + wdst;
#pragma unroll
        for (int c = 0; c < 4; c++) gemm_wide_word(wa.q[c], k0, c, mask_lo, mask_hi, magic);
    }
    load_w(1, wa);
    float da_reg = dag[0];
    lds_barrier();

    f32x16 accM;
    float2 esc;
    // a quarter (four tokens a lane) of a tile's epilogue with the scales of parity epar
    auto ep_quarter = [&](auto EPAR, auto TILE, auto I, const f32x4& dav) __attribute__((always_inline)) {
        constexpr int epar = decltype(EPAR)::value, tile = decltype(TILE)::value, i = decltype(I)::value;
#pragma unroll
        for (int e4 = 0; e4 < 4; e4++) {
            const int e = 4 * i + e4;
            const float u = fmaf(esc.x, accP[epar][tile][e], -(esc.y * accM[e]));
            out[tile][e] = fmaf(dav[e4], u, out[tile][e]);
        }
    };

    // One stage: half `half` of the group's super-block step / 2, whose parity is par.
    auto stage = [&](auto HALF, auto PAR, auto FIRST, int step, GemmWRegs& wcur, GemmWRegs& wnxt) {
        constexpr int half = decltype(HALF)::value, par = decltype(PAR)::value;
        constexpr bool has_ep = decltype(FIRST)::value == 0;
        constexpr int nhalf = half ^ 1, epar = par ^ 1;
        const int sbl = step >> 1;
        const _Float16* w = sW + half * STAGE_HALFS;
        _Float16* wnext = sW + nhalf * STAGE_HALFS;
        const int nstep = min(step + 1, nsteps - 1);
        load_w(min(step + 2, nsteps - 1), wnxt);
        const _Float16* wp0 = w + arow * JL_GEMM_WROW + 8 * kg;
        // the epilogue under this stage: tile `half` of the super-block before
        const _Float16* mp = sMin + epar * MIN_HALFS + (32 * half + arow) * JL_GEMM_MROW + 8 * kg;
        const float* scp = sScale + epar * 2 * ROWS + 2 * (32 * half + arow);
        const float* dap = sDa + epar * TOK + 32 * tg + 4 * kg;
        auto w_frag = [&](int ks, int j) { return *(const f16x8*)(wp0 + 32 * j * JL_GEMM_WROW + 16 * ks); };
        f16x8 wf[2][2], wm;
        f32x4 dav;
        GemmWideScale wsc;
        wsc.dst = wnext + wdst;
#pragma unroll
        for (int j = 0; j < 2; j++) wf[0][j] = w_frag(0, j);
        if (has_ep) {
            wm = *(const f16x8*)mp;
            esc = *(const float2*)scp;
            dav = *(const f32x4*)dap;
        }
        __builtin_amdgcn_sched_barrier(0);
        gemm_static_for<0, 8>([&](auto KS) __attribute__((always_inline)) {
            constexpr int ks = decltype(KS)::value;
            constexpr bool ep = has_ep && (ks & 1) == 0;
            if (ks + 1 < 8) {
#pragma unroll
                for (int j = 0; j < 2; j++) wf[(ks + 1) & 1][j] = w_frag(ks + 1, j);
            }
            __builtin_amdgcn_sched_barrier(0);
            const f32x16 czero = {0};
            if (ep && ks == 0) accM = __builtin_amdgcn_mfma_f32_32x32x16_f16(aaug[epar], wm, czero, 0, 0, 0);
#pragma unroll
            for (int j = 0; j < 2; j++)
                accP[par][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                    aring[ks], wf[ks & 1][j], (half == 0 && ks == 0) ? czero : accP[par][j], 0, 0, 0);
            aring[ks] = a_frag(nstep, ks);
            if (ks == 0 && nhalf == 1) aaug[par] = a_frag(nstep, 8);
            if (ep) ep_quarter(GemmIntC<epar>{}, GemmIntC<half>{}, GemmIntC<(ks >> 1)>{}, dav);
            // the next quarter's token scales, a slot ahead of their use
            if (has_ep && (ks & 1) && ks + 1 < 8) dav = *(const f32x4*)(dap + 8 * ((ks + 1) >> 1));
            // the next stage's weights: wcur -> f16 -> LDS
            if (ks == 0) w_scale(wcur.hdr, nhalf, wsc);
            if (ks & 1) gemm_wide_word(wcur.q[ks >> 1], wsc, ks >> 1, mask_lo, mask_hi, magic);
            if (nhalf == 1) {
                // a first half also lays down its super-block's minimum columns and scales (no
                // branch on the lane: threads that share an address write the same value)
                if (ks == 2) {
                    const float mul = hh ? 64.0f : 1.0f;   // hh = 0: m_s (meets A_lo), 1: 64 m_s (meets A_hi)
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
                    *(f16x8*)(sMin + par * MIN_HALFS + srow * JL_GEMM_MROW + 8 * hh) = mm;
                }
                if (ks == 6) {
                    float2 dd = {half_bits_to_f32((uint16_t)(wcur.hdr.x & 0xFFFF)),
                                 half_bits_to_f32((uint16_t)(wcur.hdr.x >> 16))};
                    *(float2*)(sScale + par * 2 * ROWS + 2 * srow) = dd;
                    sDa[par * TOK + (gt & (TOK - 1))] = da_reg;
                }
            }
            // issue order inside the slot: a matrix instruction, part of the vector work under
            // it, the second, the rest (two in a row would park the vector work behind the second)
            if (ep && ks == 0) {
                __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);   // M first: the vector work reads it
                __builtin_amdgcn_sched_group_barrier(0x002, 8, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            } else {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, 7, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            }
            __builtin_amdgcn_sched_group_barrier(0x002, 48, 0);
            __builtin_amdgcn_sched_barrier(0);
        });
        if (half == 1) da_reg = dag[(size_t)min(sbl + 1, nsbg - 1) * p.tok_pad];
        lds_barrier();
    };
    stage(GemmIntC<0>{}, GemmIntC<0>{}, GemmIntC<1>{}, 0, wa, wb);
    stage(GemmIntC<1>{}, GemmIntC<0>{}, GemmIntC<1>{}, 1, wb, wa);
    stage(GemmIntC<0>{}, GemmIntC<1>{}, GemmIntC<0>{}, 2, wa, wb);
    stage(GemmIntC<1>{}, GemmIntC<1>{}, GemmIntC<0>{}, 3, wb, wa);
    for (int step = 4; step < nsteps; step += 4) {
        stage(GemmIntC<0>{}, GemmIntC<0>{}, GemmIntC<0>{}, step, wa, wb);
        stage(GemmIntC<1>{}, GemmIntC<0>{}, GemmIntC<0>{}, step + 1, wb, wa);
        stage(GemmIntC<0>{}, GemmIntC<1>{}, GemmIntC<0>{}, step + 2, wa, wb);
        stage(GemmIntC<1>{}, GemmIntC<1>{}, GemmIntC<0>{}, step + 3, wb, wa);
    }
    // the last super-block's epilogue (its parity is 1)
    {
        const f32x16 czero = {0};
        gemm_static_for<0, 2>([&](auto TILE) __attribute__((always_inline)) {
            constexpr int tile = decltype(TILE)::value;
            const f16x8 wm = *(const f16x8*)(sMin + MIN_HALFS + (32 * tile + arow) * JL_GEMM_MROW + 8 * kg);
            esc = *(const float2*)(sScale + 2 * ROWS + 2 * (32 * tile + arow));
            accM = __builtin_amdgcn_mfma_f32_32x32x16_f16(aaug[1], wm, czero, 0, 0, 0);
            gemm_static_for<0, 4>([&](auto I) __attribute__((always_inline)) {
                constexpr int i = decltype(I)::value;
                ep_quarter(GemmIntC<1>{}, TILE, I, *(const f32x4*)(sDa + TOK + 32 * tg + 4 * kg + 8 * i));
            });
        });
    }

    // The two groups' sums meet in LDS: group kh hands over the tile it does not store
    // (tile 1 - kh) and adds the other group's share of tile kh, group 0's term first.
    // (the loop's last barrier is behind every wavefront and the last epilogue reads no weight
    // stage, so group 0's stages can be written over)
    float* xch = (float*)smem;   // [2 groups][4 wavefronts][16][64] f32
    {
        float* mine = xch + ((kh * 4 + tg) * 16) * 64 + lane;
        gemm_static_for<0, 2>([&](auto TILE) __attribute__((always_inline)) {
            constexpr int tile = decltype(TILE)::value;
            if (tile != kh) {
#pragma unroll
                for (int e = 0; e < 16; e++) mine[e * 64] = out[tile][e];
            }
        });
    }
    lds_barrier();
    {
        const float* theirs = xch + (((kh ^ 1) * 4 + tg) * 16) * 64 + lane;
        gemm_static_for<0, 2>([&](auto TILE) __attribute__((always_inline)) {
            constexpr int tile = decltype(TILE)::value;
            if (tile == kh) {
                const int r = r0 + 32 * tile + arow;
#pragma unroll
                for (int e = 0; e < 16; e++) {
                    const float o = theirs[e * 64];
                    const float s = kh == 0 ? out[tile][e] + o : o + out[tile][e];
                    const int t = t0 + 32 * tg + 8 * (e >> 2) + 4 * kg + (e & 3);
                    if (r < p.nrows && t < p.ntok) p.out[(size_t)t * p.out_stride + r] = s;
                }
            }
        });
    }
}
