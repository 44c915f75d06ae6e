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
// GEMM: 128 tokens x 128 rows per workgroup, K in stages of 256 (eight blocks a
// row); weights are decoded through double-buffered LDS, activations are laid out
// in matrix-fragment order by a prep kernel and go straight into registers.  A
// short-row matvec serves a handful of tokens.
#pragma once
#include "args.h"
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

template <int V> struct MxIntC { static constexpr int value = V; };


struct __attribute__((packed, aligned(1))) u32x4_a1 { u32x4 v; };
__device__ __forceinline__ u32x4 ld16_a1(const uint8_t* p) { return ((const u32x4_a1*)p)->v; }

// 2^(e-127) as an f32 scale: e2m1 values are half the doubled table, so
// T[code] * 2^(e-128) = e2m1(code) * 2^(e-127).  e = 0 gives 2^-127 (subnormal).
__device__ __forceinline__ float mx_scale(uint8_t e) {
    return e ? __uint_as_float((u32)e << 23) : __uint_as_float(0x00400000u);
}

// Half a block: words (2h, 2h+1) of the 16 code bytes (byte j = element j in the low
// nibble, element j+16 in the high) -> elements 8h..8h+7 and 16+8h..16+8h+7 as bf16, two
// 16-byte groups.
__device__ __forceinline__ void mx_dequant_half(u32 q0, u32 q1, float scale, u32x4& lo, u32x4& hi) {
    const u32 q[2] = {q0, q1};
#pragma unroll
    for (int w = 0; w < 2; w++) {
        // bytes 4w..4w+3 of the half: pair i = (element 4w+i, element 4w+i+16)
        u32 p0 = __builtin_bit_cast(u32, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q[w], scale, 0));
        u32 p1 = __builtin_bit_cast(u32, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q[w], scale, 1));
        u32 p2 = __builtin_bit_cast(u32, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q[w], scale, 2));
        u32 p3 = __builtin_bit_cast(u32, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q[w], scale, 3));
        lo[2 * w] = __builtin_amdgcn_perm(p1, p0, 0x05040100u);
        lo[2 * w + 1] = __builtin_amdgcn_perm(p3, p2, 0x05040100u);
        hi[2 * w] = __builtin_amdgcn_perm(p1, p0, 0x07060302u);
        hi[2 * w + 1] = __builtin_amdgcn_perm(p3, p2, 0x07060302u);
    }
}

__device__ __forceinline__ void mx_lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

#define JL_MX_TILE 128
#define JL_MX_KSTAGE 256   // eight blocks a row
#define JL_MX_STRIDE 264   // bf16 per LDS row: 256 + 8 pad (528 B: rows advance four banks)
#define JL_MX_STAGE_ELEMS (JL_MX_TILE * JL_MX_STRIDE)

// ---------------------------------------------------------------- activation prep
// grid = (ceil(k/256), tok_pad/32), block = 256: 32 tokens of one K stage.  Rows are read
// coalesced (32 lanes cover a token's 512 bytes), turned through LDS, and written as whole
// fragments, 1 KiB contiguous a wavefront.
__device__ __forceinline__ void mx_prep_body(const MxPrepArgs& p, u32x4* lds) {
    const int tid = threadIdx.x, st = blockIdx.x, grp = blockIdx.y;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int c = tid + 256 * i, tl = c >> 5, ch = c & 31;   // token, 16-byte chunk of its 512 bytes
        const int t = grp * 32 + tl, kk = st * JL_MX_KSTAGE + 8 * ch;
        u32x4 v = {0, 0, 0, 0};
        if (t < p.ntok && kk < p.k) v = *(const u32x4*)(p.x + (size_t)t * p.k + kk);
        lds[tl * 33 + ch] = v;   // 33-vector rows: the turned reads below spread over the banks
    }
    __syncthreads();
    u32x4* dst = (u32x4*)p.xf + ((size_t)st * (p.tok_pad >> 5) + grp) * (16 * 64);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int f = (tid >> 6) * 4 + i, lane = tid & 63;       // fragment ks = f, lane = 32*kg + token
        dst[f * 64 + lane] = lds[(lane & 31) * 33 + 2 * f + (lane >> 5)];
    }
}

// ---------------------------------------------------------------- GEMM
// One stage of weights for a thread: two blocks (rows 8*i + lane/8 of its wavefront's 16,
// block lane%8 of the row's eight): a wavefront's load covers eight rows x 136 contiguous
// bytes, sixteen cache lines instead of one per lane.
struct MxWRegs {
    u32x4 q[2];
    uint8_t e[2];
};

__device__ __forceinline__ void mx_load_w(const MxGemmArgs& p, int r0, int wave, int lane, int stage, MxWRegs& r) {
    const int nblk = p.k / 32;
    const int b = stage * 8 + (lane & 7);
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int row = min(r0 + wave * 16 + 8 * i + (lane >> 3), p.nrows - 1);
        const uint8_t* blk = p.w + (size_t)row * p.row_bytes + (size_t)min(b, nblk - 1) * 17;
        r.e[i] = blk[0];
        r.q[i] = ld16_a1(blk + 1);
        // (a block past the end of K reads the row's last block again; the decode zeroes its codes.
        // Zeroing them here is a select on the loaded words, and the wait for the load comes to
        // stand right behind the load: every stage then began with a whole trip to memory)
    }
}

// grid = (tok_pad/128, ceil(nrows/(32*NJ)), nsplit), block = 512, dynamic LDS = two weight
// stages [128][264] bf16.  NJ = 4: 128 tokens x 128 rows a workgroup; NJ = 3: 128 x 96, for
// shapes whose 128-row tiles would leave a quarter of the CUs without one (2880 rows x 1024
// tokens: 184 tiles of 128 rows, 240 of 96).  The shape this serves gives about as many
// tiles as the chip has CUs, so a tile gets EIGHT wavefronts, two per SIMD to cover each
// other's waits: wavefront (tg, kh) owns 32 tokens x all 32*NJ rows (NJ 32 x 32
// accumulators) over the K-steps of parity kh, and the two parities are added through LDS
// at the end, kh = 0 first.  Activation fragments come from the prepared workspace into a
// register ring a stage ahead (1 KiB coalesced loads), each feeding NJ matrix
// instructions; all eight wavefronts share one decode of the weights through LDS.  A stage
// (256 K) is 8*NJ matrix instructions per wavefront with their weight fragments fetched six
// instructions ahead and the next stage's weights decoded half a block at a time in
// between, their registers loaded two stages ahead.
template <int NJ>
__device__ __forceinline__ void mx_gemm_body(const MxGemmArgs& p, uint8_t* smem) {
    constexpr int ROWS = 32 * NJ, UNITS = 8 * NJ, AHEAD = 6;
    __bf16* sW = (__bf16*)smem;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int tg = wave & 3, kh = wave >> 2;
    const int t0 = blockIdx.x * JL_MX_TILE, r0 = blockIdx.y * ROWS;
    // a small grid is widened along K: workgroup z takes a contiguous run of the K
    // stages and writes its partial sums to its own slab, summed afterwards in order
    const int all_stages = (p.k + JL_MX_KSTAGE - 1) / JL_MX_KSTAGE;
    const int per_split = (all_stages + p.nsplit - 1) / p.nsplit;
    const int s_lo = min((int)blockIdx.z * per_split, all_stages), s_hi = min(s_lo + per_split, all_stages);
    float* outp = p.nsplit > 1 ? p.part + (size_t)blockIdx.z * p.ntok * p.nrows : p.out;
    const int arow = lane & 31, kg = lane >> 5;
    // activation fragment (stage, K-step 2*ks2 + kh) of this wavefront's 32 tokens: uniform base + lane
    const size_t astride = (size_t)(p.tok_pad >> 5) * (16 * 1024);
    const char* abase = (const char*)p.x + ((size_t)(t0 >> 5) + tg) * (16 * 1024) + kh * 1024;
    const unsigned aoff = lane * 16;
    auto a_frag = [&](int stage, int ks2) {
        return *(const bf16x8*)(abase + (size_t)stage * astride + ks2 * 2048 + aoff);
    };
    // this wavefront decodes rows 16*wave .. 16*wave+15 of the tile (none if the tile is shorter)
    const bool decodes = wave * 16 < ROWS;   // uniform
    const int wdst = (wave * 16 + (lane >> 3)) * JL_MX_STRIDE + (lane & 7) * 32;

    f32x16_t acc[NJ];
#pragma unroll
    for (int j = 0; j < NJ; j++)
#pragma unroll
        for (int e = 0; e < 16; e++) acc[j][e] = 0.f;

    const int nblk = p.k / 32;
    auto decode_half = [&](const MxWRegs& r, int i, int h, __bf16* buf, int stg) {
        // block i of the thread's two, words (2h, 2h+1): elements 8h.. and 16+8h..
        // (stg: the stage r holds; its blocks past the end of K decode as zero codes)
        const bool past = stg * 8 + (lane & 7) >= nblk;
        u32x4 lo, hi;
        mx_dequant_half(past ? 0u : r.q[i][2 * h], past ? 0u : r.q[i][2 * h + 1], mx_scale(r.e[i]), lo, hi);
        __bf16* dst = buf + wdst + 8 * i * JL_MX_STRIDE + 8 * h;
        *(u32x4*)dst = lo;
        *(u32x4*)(dst + 16) = hi;
    };

    // The loads before the loop go out in the loop's own order (a stage's weights, the next
    // stage's, then the activation fragments; the loop's head adds the stage after that): the
    // wait the compiler puts before a register's first use in the loop is the smaller of the
    // counts on the two ways in, and with the second stage's weights requested last here it made
    // every other stage wait for the weights its own head had just requested.
    MxWRegs wa, wb;
    bf16x8 aring[8];
    const int last = max(s_hi - 1, s_lo);
    if (decodes) {
        mx_load_w(p, r0, wave, lane, s_lo, wb);
        mx_load_w(p, r0, wave, lane, min(s_lo + 1, last), wa);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int ks2 = 0; ks2 < 8; ks2++) {
        aring[ks2] = a_frag(s_lo, ks2);
        __builtin_amdgcn_sched_barrier(0);   // in K order, as the loop requests them
    }
    if (decodes) {
#pragma unroll
        for (int i = 0; i < 2; i++) {
            decode_half(wb, i, 0, sW, s_lo);
            decode_half(wb, i, 1, sW, s_lo);
        }
    }
    mx_lds_barrier();

    auto stage = [&](auto BUF, int st, MxWRegs& wcur, MxWRegs& wnxt) {
        constexpr int buf = decltype(BUF)::value;
        const __bf16* w = sW + buf * JL_MX_STAGE_ELEMS;
        __bf16* wnext = sW + (buf ^ 1) * JL_MX_STAGE_ELEMS;
        const int nst = min(st + 1, last);
        if (decodes) mx_load_w(p, r0, wave, lane, min(st + 2, last), wnxt);
        const __bf16* wp0 = w + arow * JL_MX_STRIDE + 8 * kg + 16 * kh;
        // unit u = matrix instruction (K-step u / NJ, row tile u % NJ)
        auto w_frag = [&](int u) {
            return *(const bf16x8*)(wp0 + 32 * (u % NJ) * JL_MX_STRIDE + 32 * (u / NJ));
        };
        bf16x8 wf[8];
#pragma unroll
        for (int u = 0; u < AHEAD; u++) wf[u] = w_frag(u);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < UNITS; u++) {
            const int ks2 = u / NJ, j = u % NJ;
            if (u + AHEAD < UNITS) wf[(u + AHEAD) & 7] = w_frag(u + AHEAD);
            __builtin_amdgcn_sched_barrier(0);
            acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(aring[ks2], wf[u & 7], acc[j], 0, 0, 0);
            if (j == NJ - 1) {
                aring[ks2] = a_frag(nst, ks2);
                // half a block of the next stage's weights in every second K-step
                if (decodes && (ks2 & 1)) decode_half(wcur, ks2 >> 2, (ks2 >> 1) & 1, wnext, nst);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        mx_lds_barrier();
    };
    for (int st = s_lo; st < s_hi; st += 2) {
        stage(MxIntC<0>{}, st, wa, wb);
        if (st + 1 < s_hi) stage(MxIntC<1>{}, st + 1, wb, wa);
    }

    // the two K parities meet in LDS (the weight stages are done with): [tg][tile][16][64] f32
    float* sAcc = (float*)smem + (size_t)tg * (NJ * 16 * 64) + lane;
    if (kh == 1) {
#pragma unroll
        for (int j = 0; j < NJ; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) sAcc[(j * 16 + e) * 64] = acc[j][e];
    }
    __syncthreads();
    if (kh == 1) return;
#pragma unroll
    for (int j = 0; j < NJ; j++) {
        const int r = r0 + 32 * j + arow;
#pragma unroll
        for (int e = 0; e < 16; e++) {
            const float v = acc[j][e] + sAcc[(j * 16 + e) * 64];
            const int t = t0 + 32 * tg + 8 * (e >> 2) + 4 * kg + (e & 3);
            if (r < p.nrows && t < p.ntok) outp[(size_t)t * p.nrows + r] = v;
        }
    }
}

// A few tokens (ntok <= 8): one wavefront per row, lane l takes blocks l, l+64, ...
// A conversion turns a code byte into the bf16 pair (element j, element j + 16), exact; the
// matching activation pair is picked out of two of the block's words with one byte permute,
// and v_dot2_f32_bf16 adds the pair's two products to the f32 sum: three vector instructions
// for two weights per token where widening everything to f32 took five.
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
        bf16x2 wp[16];   // wp[4w + i] = (element 4w + i, element 4w + i + 16)
#pragma unroll
        for (int w = 0; w < 4; w++) {
            wp[4 * w + 0] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q[w], scale, 0);
            wp[4 * w + 1] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q[w], scale, 1);
            wp[4 * w + 2] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q[w], scale, 2);
            wp[4 * w + 3] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q[w], scale, 3);
        }
#pragma unroll
        for (int t = 0; t < 8; t++) {
            if (t < p.ntok) {
                const u32x4* xt = (const u32x4*)(p.x + (size_t)t * p.k + (size_t)b * 32);
                u32 X[16];   // X[j] = (element 2j, element 2j + 1)
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    const u32x4 v = xt[c];
                    X[4 * c] = v.x; X[4 * c + 1] = v.y; X[4 * c + 2] = v.z; X[4 * c + 3] = v.w;
                }
                float s = 0.f;
#pragma unroll
                for (int e = 0; e < 16; e++) {
                    // (x[e], x[e + 16]): the same half of words e/2 and e/2 + 8
                    const u32 xp = __builtin_amdgcn_perm(X[e / 2 + 8], X[e / 2], (e & 1) ? 0x07060302u : 0x05040100u);
                    s = __builtin_amdgcn_fdot2_f32_bf16(wp[e], __builtin_bit_cast(bf16x2, xp), s, false);
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

// One token: the activation is the same for every row, so a lane keeps its blocks' activation
// pairs in registers (already in the conversions' pair order) and the wavefront walks RPW rows
// with them: the activation is read and permuted once per wavefront instead of once per row, and
// all the rows' weight loads go out before the first row is decoded.
// NBI = blocks a lane holds (lane l: blocks l, l + 64, ...: k <= 2048 * NBI).
// grid = ceil(nrows / (nwaves * RPW)), block = 64 * nwaves (the library launches one wavefront a workgroup)
template <int NBI>
__device__ __forceinline__ void mx_matvec1_body(const MxGemmArgs& p) {
    constexpr int RPW = JL_MX1_RPW;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
    const int row0 = (blockIdx.x * nwaves + wave) * RPW;
    if (row0 >= p.nrows) return;
    const int nblk = p.k / 32;
    u32x4 q[RPW][NBI];
    uint8_t e[RPW][NBI];
#pragma unroll
    for (int r = 0; r < RPW; r++) {
        const uint8_t* wrow = p.w + (size_t)min(row0 + r, p.nrows - 1) * p.row_bytes;
#pragma unroll
        for (int u = 0; u < NBI; u++) {
            const uint8_t* blk = wrow + (size_t)min(lane + 64 * u, nblk - 1) * 17;
            e[r][u] = blk[0];
            q[r][u] = ld16_a1(blk + 1);
        }
    }
    bf16x2 xp[NBI][16];   // xp[u][e] = (x[32b + e], x[32b + e + 16]) of block b = lane + 64u
#pragma unroll
    for (int u = 0; u < NBI; u++) {
        const int b = lane + 64 * u;
        const u32x4* xt = (const u32x4*)(p.x + (size_t)min(b, nblk - 1) * 32);
        u32 X[16];
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const u32x4 v = b < nblk ? xt[c] : u32x4{0u, 0u, 0u, 0u};   // a block past the row's end adds nothing
            X[4 * c] = v.x; X[4 * c + 1] = v.y; X[4 * c + 2] = v.z; X[4 * c + 3] = v.w;
        }
#pragma unroll
        for (int i = 0; i < 16; i++)
            xp[u][i] = __builtin_bit_cast(bf16x2, __builtin_amdgcn_perm(X[i / 2 + 8], X[i / 2],
                                                                         (i & 1) ? 0x07060302u : 0x05040100u));
    }
#pragma unroll
    for (int r = 0; r < RPW; r++) {
        float s = 0.f;
#pragma unroll
        for (int u = 0; u < NBI; u++) {
            const float scale = mx_scale(e[r][u]);
#pragma unroll
            for (int w = 0; w < 4; w++) {
                s = __builtin_amdgcn_fdot2_f32_bf16(__builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q[r][u][w], scale, 0), xp[u][4 * w + 0], s, false);
                s = __builtin_amdgcn_fdot2_f32_bf16(__builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q[r][u][w], scale, 1), xp[u][4 * w + 1], s, false);
                s = __builtin_amdgcn_fdot2_f32_bf16(__builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q[r][u][w], scale, 2), xp[u][4 * w + 2], s, false);
                s = __builtin_amdgcn_fdot2_f32_bf16(__builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q[r][u][w], scale, 3), xp[u][4 * w + 3], s, false);
            }
        }
        const float v = wave_sum_to_lane63(s);
        if (lane == 63 && row0 + r < p.nrows) p.out[row0 + r] = v;
    }
}

// The same handful of tokens over packed planes (jit/gpu/kernels/pack.go:543-575).  A lane
// takes a row, so the four code words and the exponent word of a block are consecutive
// across RL lanes; the 64 / RL lane groups of a wavefront, and the wavefronts of a workgroup,
// take the blocks of K in turn (a slice each).  RL = 64: the activations are the same for
// every lane and come as scalar operands; RL = 32 / 16: more, smaller workgroups for a
// matrix of few rows, the activations as vector loads a lane group shares.  The slices' sums
// are added in a fixed order: across a wavefront's lane groups, then the wavefronts in turn
// through LDS (red: [nwaves][8][RL] floats).
// AHEAD blocks at a time: all their loads go out before the first is decoded, so a slice's
// few blocks cost one trip to memory and not one each.
// grid = ceil(nrows/RL), block = 64 * nwaves
template <int RL, int AHEAD>
__device__ __forceinline__ void mx_planes_matvec_body(const MxPlanesArgs& p, float* red) {
    constexpr int G = 64 / RL;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int rlane = lane % RL;
    const int slice = G == 1 ? wave : wave * G + lane / RL, nsl = p.nwaves * G;
    const int rl = blockIdx.x * RL + rlane;
    const bool live = rl < p.nrows;
    const size_t n = (size_t)p.stride;
    const size_t r = (size_t)p.row0 + (live ? rl : p.nrows - 1);   // idle lanes re-read the last row
    const int nblk = p.k / 32, sh = 8 * (int)(r & 3);
    const size_t dwords = (n + 3) / 4;
    float acc[8];
#pragma unroll
    for (int t = 0; t < 8; t++) acc[t] = 0.f;
    for (int base = 0; base < nblk; base += AHEAD * nsl) {
        const int b0 = base + slice;
        u32 q[AHEAD][4], dd[AHEAD];
#pragma unroll
        for (int u = 0; u < AHEAD; u++) {
            const int b = b0 + u * nsl < nblk ? b0 + u * nsl : nblk - 1;
            const u32* qp = p.qs + (size_t)b * 4 * n + r;
#pragma unroll
            for (int w = 0; w < 4; w++) q[u][w] = qp[(size_t)w * n];
            dd[u] = p.d[(size_t)b * dwords + (r >> 2)];
        }
#pragma unroll
        for (int u = 0; u < AHEAD; u++) {
            const int b = b0 + u * nsl;
            if (b < nblk) {
                const float scale = mx_scale((uint8_t)(((dd[u] >> sh) & 0xFF) + 1));
                float wv[32];
#pragma unroll
                for (int w = 0; w < 4; w++) {
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        f32x2 pr;
                        switch (i) {
                        case 0: pr = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(q[u][w], scale, 0); break;
                        case 1: pr = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(q[u][w], scale, 1); break;
                        case 2: pr = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(q[u][w], scale, 2); break;
                        default: pr = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(q[u][w], scale, 3); break;
                        }
                        wv[4 * w + i] = pr.x;
                        wv[4 * w + i + 16] = pr.y;
                    }
                }
#pragma unroll
                for (int t = 0; t < 8; t++) {
                    if (t < p.ntok) {
                        const u32* xt = p.x + (((size_t)t * p.k + (size_t)b * 32) >> 1);
                        float s = 0.f;
#pragma unroll
                        for (int c4 = 0; c4 < 4; c4++) {
                            u32 v[4];
                            if constexpr (G == 1) {
#pragma unroll
                                for (int j = 0; j < 4; j++) v[j] = xt[4 * c4 + j];
                            } else {
                                const u32x4 vv = ((const u32x4*)xt)[c4];
#pragma unroll
                                for (int j = 0; j < 4; j++) v[j] = vv[j];
                            }
#pragma unroll
                            for (int j = 0; j < 4; j++) {
                                s = fmaf(wv[8 * c4 + 2 * j], __uint_as_float(v[j] << 16), s);
                                s = fmaf(wv[8 * c4 + 2 * j + 1], __uint_as_float(v[j] & 0xFFFF0000u), s);
                            }
                        }
                        acc[t] += s;
                    }
                }
            }
        }
    }
    // a wavefront's lane groups first (lanes RL apart hold the same row), then the wavefronts
    // in order through LDS
#pragma unroll
    for (int t = 0; t < 8; t++) {
        if (t < p.ntok) {
            float s = acc[t];
            if constexpr (G >= 2) s += __shfl_xor(s, 32);
            if constexpr (G >= 4) s += __shfl_xor(s, 16);
            if (lane < RL) red[(wave * 8 + t) * RL + rlane] = s;
        }
    }
    __syncthreads();
    // one thread per (token, row) adds the wavefronts' sums
    for (int i = threadIdx.x; i < p.ntok * RL; i += blockDim.x) {
        const int t = i / RL, rr = i % RL;
        float s = red[t * RL + rr];
        for (int w = 1; w < p.nwaves; w++) s += red[(w * 8 + t) * RL + rr];
        if ((int)(blockIdx.x * RL + rr) < p.nrows) p.out[(size_t)t * p.nrows + blockIdx.x * RL + rr] = s;
    }
}

// ------------------------------------------------- the GEMM over packed planes
// More than a handful of tokens over MX4 planes, nothing restored: a lane of the matrix
// instruction's weight operand is (row = lane % 32, kg = lane / 32), and with the planes laid
// [block][word][row] its eight K values of a 16-deep step are ONE plane word -- word 2s + kg of
// the block for the block's step s -- read coalesced (32 consecutive rows) and decoded by four
// conversions with the block's scale.  The word holds elements 4w..4w+3 in its low nibbles and
// 4w+16..4w+19 in its high ones, and a conversion gives a byte's pair, so the operand's K order
// is 4w, 4w+16, 4w+1, 4w+17, ...; the prep kernel lays the activation fragments out in that order.
// A workgroup owns 64 tokens x 64 rows (2 x 2 tiles) and its four wavefronts take the K-steps of
// 64 (two blocks) in turn: many small workgroups, so a CU holds enough wavefronts to cover the
// trip to memory; the four partial tiles meet in LDS in wavefront order, wavefront w finishing
// tile w (red: [wavefront][tile][16][64] floats).
//
// Tile of workgroup L in a 1-D grid of 8 * ceil(tiles / 8): the hardware deals consecutive
// workgroups round the eight XCDs, each with an L2 of its own, so XCD x = L % 8 is given a
// contiguous run of the token-major tile order -- its workgroups share a few token tiles, whose
// activation fragments then stay in that L2 while the row tiles walk past.  False: no tile.
__device__ __forceinline__ bool mx_xcd_tile(int ntt64, int nrt, int& tt, int& rt) {
    const int tiles = ntt64 * nrt, per = (tiles + 7) / 8;
    const int g = (int)(blockIdx.x & 7) * per + (int)(blockIdx.x >> 3);
    if ((int)(blockIdx.x >> 3) >= per || g >= tiles) return false;
    tt = g / nrt;
    rt = g - tt * nrt;
    return true;
}

// prep: grid = (ceil(K-steps / 4), tok_pad / 32), block = 256: a wavefront per (K-step, 32 tokens)
__device__ __forceinline__ void mx_planes_prep_body(const MxPlanesPrepArgs& p) {
    const int lane = threadIdx.x & 63, nks = (p.k + 63) / 64, ntt = p.tok_pad / 32;
    const int ks = blockIdx.x * 4 + (threadIdx.x >> 6), tile = blockIdx.y;
    if (ks >= nks) return;
    const int t = 32 * tile + (lane & 31), kg = lane >> 5, nblk = p.k / 32;
    u32x4* dst = (u32x4*)p.xa + ((size_t)ks * ntt + tile) * 4 * 64 + lane;
#pragma unroll
    for (int s4 = 0; s4 < 4; s4++) {
        const int b = 2 * ks + (s4 >> 1), w = 2 * (s4 & 1) + kg;
        u32x4 v = u32x4{0u, 0u, 0u, 0u};
        if (t < p.ntok && b < nblk) {
            const uint16_t* src = p.x + (size_t)t * p.k + (size_t)b * 32 + 4 * w;
            const u32x2 lo = *(const u32x2*)src, hi = *(const u32x2*)(src + 16);
            // elements (4w, 4w+1 | 4w+2, 4w+3) and (4w+16, 4w+17 | 4w+18, 4w+19), interleaved
            v.x = (lo.x & 0xFFFFu) | (hi.x << 16);
            v.y = (lo.x >> 16) | (hi.x & 0xFFFF0000u);
            v.z = (lo.y & 0xFFFFu) | (hi.y << 16);
            v.w = (lo.y >> 16) | (hi.y & 0xFFFF0000u);
        }
        dst[(size_t)s4 * 64] = v;
    }
}

// grid = 8 * ceil(tiles / 8) (mx_xcd_tile), block = 256, dynamic LDS = 64 KiB
__device__ __forceinline__ void mx_planes_gemm_body(const MxPlanesGemmArgs& p, float* red) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    int tt, rt;
    if (!mx_xcd_tile(p.tok_pad / 64, (p.nrows + 63) / 64, tt, rt)) return;
    const int t0 = tt * 64, r0 = rt * 64;
    const int nblk = p.k / 32, nks = (p.k + 63) / 64, ntt = p.tok_pad / 32, kg = lane >> 5;
    const size_t n = (size_t)p.stride, dwords = (n + 3) / 4;
    // every load is a uniform base (scalar registers) plus a 32-bit lane offset
    u32 qoff[2][2], doff[2];
    int sh[2];
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const u32 row = (u32)p.row0 + (u32)min(r0 + 32 * j + (lane & 31), p.nrows - 1);
        sh[j] = 8 * (int)(row & 3);
        doff[j] = row >> 2;
#pragma unroll
        for (int s = 0; s < 2; s++) qoff[j][s] = (u32)(2 * s + kg) * (u32)p.stride + row;
    }
    // [row tile][matrix K-step], [row tile][block]; past: the K-step's second block lies beyond K
    // (its codes are zeroed where they are used: a select on the loaded words here would put the
    // wait for the load right behind the load)
    struct WOps { u32 q[2][4]; u32 d[2][2]; bool past; };
    struct AOps { u32x4 a[2][4]; };                // [token tile][matrix K-step]
    auto load_w = [&](int ks, WOps& o) {
        ks = min(ks, nks - 1);
        o.past = 2 * ks + 1 >= nblk;       // the second block of a last, half K-step (uniform)
#pragma unroll
        for (int bi = 0; bi < 2; bi++) {
            const int b = 2 * ks + bi;
            const size_t bc = (size_t)min(b, nblk - 1);
            const u32* qb = p.qs + bc * 4 * n;
            const u32* db = p.d + bc * dwords;
#pragma unroll
            for (int j = 0; j < 2; j++) {
#pragma unroll
                for (int s = 0; s < 2; s++) {
                    o.q[j][2 * bi + s] = qb[qoff[j][s]];
                }
                o.d[j][bi] = db[doff[j]];
            }
        }
    };
    const u32 aoff = (u32)lane * 4;
    auto load_a = [&](int ks, AOps& o) {
        ks = min(ks, nks - 1);
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const u32* ab = p.xa + ((size_t)ks * ntt + (t0 >> 5) + i) * (4 * 64 * 4);
#pragma unroll
            for (int s4 = 0; s4 < 4; s4++) o.a[i][s4] = *(const u32x4*)(ab + aoff + s4 * 256);
        }
    };
    f32x16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.f;
    auto compute = [&](const WOps& wo, const AOps& ao) {
#pragma unroll
        for (int s4 = 0; s4 < 4; s4++) {
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const float scale = mx_scale((uint8_t)(((wo.d[j][s4 >> 1] >> sh[j]) & 0xFF) + 1));
                const u32 q = (s4 >> 1) && wo.past ? 0u : wo.q[j][s4];
                u32x4 wb;
                wb.x = __builtin_bit_cast(u32, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q, scale, 0));
                wb.y = __builtin_bit_cast(u32, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q, scale, 1));
                wb.z = __builtin_bit_cast(u32, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q, scale, 2));
                wb.w = __builtin_bit_cast(u32, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q, scale, 3));
                const bf16x8 wf = __builtin_bit_cast(bf16x8, wb);
#pragma unroll
                for (int i = 0; i < 2; i++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, ao.a[i][s4]), wf,
                                                                         acc[i][j], 0, 0, 0);
            }
        }
    };
    // Operand sets in rotation -- three of weights (from HBM: loaded two K-steps before their
    // use), two of activations (from L2: one K-step) -- and the loop unrolled by six so that no
    // set is ever copied (a copy would wait for the load it copies).
    WOps w0, w1, w2;
    AOps a0, a1;
    load_w(wave, w0);
    load_a(wave, a0);
    load_w(wave + 4, w1);
    // (the barrier keeps a step's requests in front of its matrix work: left to itself the
    // scheduler moved fragment loads down to just before their use, a whole trip to memory each)
#define JL_MXP_STEP(N, WL, AL, WC, AC)                   \
    load_w(wave + 4 * (n + (N) + 2), WL);                \
    load_a(wave + 4 * (n + (N) + 1), AL);                \
    __builtin_amdgcn_sched_barrier(0);                   \
    if (n + (N) < my_steps) compute(WC, AC);             \
    __builtin_amdgcn_sched_barrier(0);
    const int my_steps = (nks - wave + 3) / 4;   // K-steps wave, wave + 4, ... (uniform)
    for (int n = 0; n < my_steps; n += 6) {
        JL_MXP_STEP(0, w2, a1, w0, a0)
        JL_MXP_STEP(1, w0, a0, w1, a1)
        JL_MXP_STEP(2, w1, a1, w2, a0)
        JL_MXP_STEP(3, w2, a0, w0, a1)
        JL_MXP_STEP(4, w0, a1, w1, a0)
        JL_MXP_STEP(5, w1, a0, w2, a1)
    }
#undef JL_MXP_STEP
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) red[((wave * 4 + 2 * i + j) * 16 + e) * 64 + lane] = acc[i][j][e];
    __syncthreads();
    const int i = wave >> 1, j = wave & 1;
    const int r = r0 + 32 * j + (lane & 31);
#pragma unroll
    for (int e = 0; e < 16; e++) {
        float s = red[((0 * 4 + wave) * 16 + e) * 64 + lane];
#pragma unroll
        for (int w = 1; w < 4; w++) s += red[((w * 4 + wave) * 16 + e) * 64 + lane];
        const int t = t0 + 32 * i + 8 * (e >> 2) + 4 * kg + (e & 3);
        if (r < p.nrows && t < p.ntok) p.out[(size_t)t * p.nrows + r] = s;
    }
}

// ------------------------------------------------- block-scaled form (opt-in)
// v_mfma_scale_f32_32x32x64_f8f6f4 takes MXFP4 as it is stored: 32 e2m1 codes a lane (one
// block: row = lane % 32, block of the K-step = lane / 32, position = nibble index) and the
// block's E8M0 exponent as the lane's scale.  The other operand cannot be bf16: the activations are quantized to MX fp8
// (e4m3, a power-of-two scale per token and block of 32, chosen so the block's largest value
// stays below 448), which costs about three bits of every activation -- so this form is never
// the default and reports its error beside its time.  The codes of a block are stored byte j =
// (element j, element j + 16), so the activation block is laid out in that order too:
// position 2j holds element j, position 2j + 1 element j + 16.
typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef short i16x2 __attribute__((ext_vector_type(2)));

// grid = (ceil(K-steps / 4), tok_pad / 32), block = 256: a wavefront per (K-step of 64, 32 tokens)
__device__ __forceinline__ void mx_scaled_prep_body(const MxScaledPrepArgs& p) {
    const int lane = threadIdx.x & 63, nks = (p.k + 63) / 64, ntt = p.tok_pad / 32;
    const int ks = blockIdx.x * 4 + (threadIdx.x >> 6), tile = blockIdx.y;
    if (ks >= nks) return;
    const int t = 32 * tile + (lane & 31), b = 2 * ks + (lane >> 5);
    float v[32];
    float amax = 0.f;
    if (t < p.ntok && b < p.k / 32) {
        const u32x4* src = (const u32x4*)(p.x + (size_t)t * p.k + (size_t)b * 32);
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const u32x4 w = src[c];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                v[8 * c + 2 * j] = __uint_as_float(w[j] << 16);
                v[8 * c + 2 * j + 1] = __uint_as_float(w[j] & 0xFFFF0000u);
            }
        }
#pragma unroll
        for (int i = 0; i < 32; i++) amax = fmaxf(amax, fabsf(v[i]));
    } else {
#pragma unroll
        for (int i = 0; i < 32; i++) v[i] = 0.f;
    }
    // scale 2^(sb - 127): the largest value lands in [224, 448]
    const u32 bits = __float_as_uint(amax);
    int sb = (int)((bits >> 23) & 0xFF) - 8 + ((bits & 0x7FFFFFu) > 0x600000u ? 1 : 0);
    sb = amax == 0.f ? 127 : min(max(sb, 1), 254);
    const float scale = __uint_as_float((u32)sb << 23);
    u32 w[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        i16x2 r = {0, 0};
        r = __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(r, v[2 * i], v[2 * i + 16], scale, false);
        r = __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(r, v[2 * i + 1], v[2 * i + 17], scale, true);
        w[i] = __builtin_bit_cast(u32, r);
    }
    // An 8-bit operand keeps, in lane (token, g), positions 16g .. 16g+15 of BOTH blocks of the
    // K-step (first block in the low four registers); the block's scale stays with lane
    // (token, block).  So the two lanes of a token trade half a block.
    const int g = lane >> 5;
    u32 got[4];
#pragma unroll
    for (int i = 0; i < 4; i++) got[i] = __shfl_xor(g ? w[i] : w[4 + i], 32);
    const size_t frag = (size_t)ks * ntt + tile;
    u32x4* dst = (u32x4*)(p.xa + (frag * 64 + lane) * 8);
    dst[0] = g ? u32x4{got[0], got[1], got[2], got[3]} : u32x4{w[0], w[1], w[2], w[3]};
    dst[1] = g ? u32x4{w[4], w[5], w[6], w[7]} : u32x4{got[0], got[1], got[2], got[3]};
    p.xs[frag * 64 + lane] = (uint8_t)sb;
}

// grid = 8 * ceil(tiles / 8) (mx_xcd_tile), block = 256, LDS = 64 KiB: a workgroup owns 64 tokens x
// 64 rows (2 x 2 tiles of 32 x 32) and its four wavefronts take the K-steps of 64 in turn --
// many small workgroups, so that a CU holds enough wavefronts to cover the trip to memory, which
// is all a loop of loads and matrix instructions has to hide.  Weights come straight from the
// planes (a lane a row: coalesced), activations from the prepared fragments, both two K-steps
// ahead of their use; the four partial tiles are added in wavefront order through LDS
// (red: [wavefront][tile][16][64] floats), wavefront w finishing tile w.
__device__ __forceinline__ void mx_scaled_gemm_body(const MxScaledGemmArgs& p, float* red) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    int tt, rt;
    if (!mx_xcd_tile(p.tok_pad / 64, (p.nrows + 63) / 64, tt, rt)) return;
    const int t0 = tt * 64, r0 = rt * 64;
    const int nblk = p.k / 32, nks = (p.k + 63) / 64, ntt = p.tok_pad / 32;
    const size_t n = (size_t)p.stride, dwords = (n + 3) / 4;
    size_t row[2];
    int sh[2];
#pragma unroll
    for (int j = 0; j < 2; j++) {
        row[j] = (size_t)p.row0 + min(r0 + 32 * j + (lane & 31), p.nrows - 1);
        sh[j] = 8 * (int)(row[j] & 3);
    }
    struct Ops { i32x8 a[2]; u32 sa[2]; i32x8 b[2]; u32 sb[2]; };
    auto load = [&](int ks, Ops& o) {
        ks = min(ks, nks - 1);
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const size_t frag = (size_t)ks * ntt + (t0 >> 5) + i;
            const u32x4* src = (const u32x4*)(p.xa + (frag * 64 + lane) * 8);
            const u32x4 lo = src[0], hi = src[1];
            o.a[i] = i32x8{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
            o.sa[i] = p.xs[frag * 64 + lane];
        }
        const int b = 2 * ks + (lane >> 5);
        const bool past = b >= nblk;   // the second block of a last, half K-step
        const size_t bc = (size_t)(past ? nblk - 1 : b);
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const u32* qp = p.qs + bc * 4 * n + row[j];
            u32 q[4];
#pragma unroll
            for (int w = 0; w < 4; w++) q[w] = past ? 0u : qp[(size_t)w * n];
            o.b[j] = i32x8{(int)q[0], (int)q[1], (int)q[2], (int)q[3], 0, 0, 0, 0};
            o.sb[j] = ((p.d[bc * dwords + (row[j] >> 2)] >> sh[j]) + 1) & 0xFF;
        }
    };
    f32x16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.f;
    auto compute = [&](const Ops& o) {
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 2; j++)
                acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(o.a[i], o.b[j], acc[i][j], 0, 4, 0,
                                                                             (int)o.sa[i], 0, (int)o.sb[j]);
    };
    // three operand sets in rotation, the loop unrolled by three so that no set is ever copied
    // (a copy would wait for the load it copies)
    Ops o0, o1, o2;
    load(wave, o0);
    load(wave + 4, o1);
    for (int ks = wave; ks < nks; ks += 12) {
        load(ks + 8, o2);
        compute(o0);
        if (ks + 4 >= nks) break;
        load(ks + 12, o0);
        compute(o1);
        if (ks + 8 >= nks) break;
        load(ks + 16, o1);
        compute(o2);
    }
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) red[((wave * 4 + 2 * i + j) * 16 + e) * 64 + lane] = acc[i][j][e];
    __syncthreads();
    const int i = wave >> 1, j = wave & 1, kg = lane >> 5;
    const int r = r0 + 32 * j + (lane & 31);
#pragma unroll
    for (int e = 0; e < 16; e++) {
        float s = red[((0 * 4 + wave) * 16 + e) * 64 + lane];
#pragma unroll
        for (int w = 1; w < 4; w++) s += red[((w * 4 + wave) * 16 + e) * 64 + lane];
        const int t = t0 + 32 * i + 8 * (e >> 2) + 4 * kg + (e & 3);
        if (r < p.nrows && t < p.ntok) p.out[(size_t)t * p.nrows + r] = s;
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

// ---------------------------------------------------------------- few tokens
// 9..64 tokens: the weights (4.4 MB at 2880 x 2880) should be read once and nothing else
// should cost; the tiled GEMM above needs a K split with a second launch there.  The scheme
// of the Q4_K few-token kernel: v_mfma_f32_16x16x32_bf16 (16 tokens x 16 rows, K = 32), a
// workgroup owns 16 rows and all tokens, its eight wavefronts split K and meet in LDS.
// K is walked in groups of four blocks (128 weights).  Lane (row r = lane % 16, kq = lane / 16)
// loads block 4 G + kq of its row whole (16 code bytes + the exponent) and K-step j of the
// group takes code word j of every lane: a step mixes four blocks, each lane converting its
// word with its own block's scale (the hardware conversion takes the scale per lane).  Word
// j, byte i decodes to elements 4j+i and 16+4j+i of the block, so the lane's operand is
//   (e[4j], e[16+4j], e[4j+1], e[16+4j+1], e[4j+2], e[16+4j+2], e[4j+3], e[16+4j+3])
// and the prep kernel below lays the activations out in exactly that order.
//
// prep: x bf16 [ntok][k] -> xf [ceil(k/128) groups][4 steps][ntiles][64 lanes][8] bf16;
// grid = (ceil(k/128), ntiles), block = 256 (thread = step j, lane); zeros past ntok and k.
__device__ __forceinline__ void mx_prep_few_body(const MxPrepArgs& p) {
    const int G = blockIdx.x, tile = blockIdx.y, ntiles = gridDim.y;
    const int j = threadIdx.x >> 6, lane = threadIdx.x & 63, t = tile * 16 + (lane & 15), kq = lane >> 4;
    const int k0 = 128 * G + 32 * kq + 4 * j;   // elements k0..k0+3 and k0+16..k0+19
    typedef uint16_t u16x4 __attribute__((ext_vector_type(4)));
    u16x4 lo = {0, 0, 0, 0}, hi = {0, 0, 0, 0};
    if (t < p.ntok && k0 < p.k) {   // k % 32 == 0: a block is inside K or outside it
        const uint16_t* src = p.x + (size_t)t * p.k + k0;
        lo = *(const u16x4*)src;
        hi = *(const u16x4*)(src + 16);
    }
    typedef uint16_t u16x8 __attribute__((ext_vector_type(8)));
    const u16x8 o = {lo[0], hi[0], lo[1], hi[1], lo[2], hi[2], lo[3], hi[3]};
    ((u16x8*)p.xf)[(((size_t)G * 4 + j) * ntiles + tile) * 64 + lane] = o;
}

// grid = ceil(nrows / 16), block = 512, static LDS = 8 x NT x 1 KiB; p.x is the prep's
// workspace, p.tok_pad = 16 * NT.
template <int NT>
__device__ __forceinline__ void mx_few_body(const MxGemmArgs& p, float* part) {
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r16 = lane & 15, kq = lane >> 4;
    const int r0 = blockIdx.x * 16;
    const int nblk = p.k / 32, ngroups = (nblk + 3) / 4;
    const uint8_t* wrow = p.w + (size_t)min(r0 + r16, p.nrows - 1) * p.row_bytes;
    const u32x4* xf = (const u32x4*)p.x;

    f32x4 out[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) out[t] = f32x4{0.f, 0.f, 0.f, 0.f};

    struct W { u32x4 q; u32 e; };
    auto load_w = [&](int G, W& w) {
        const int b = 4 * G + kq;
        const uint8_t* blk = wrow + (size_t)min(b, nblk - 1) * 17;
        w.e = blk[0];
        w.q = ld16_a1(blk + 1);
        // (a block past the end of K reads the row's last block; its codes are zeroed where they
        // are used.  A select on the loaded words here puts the wait for the load right behind
        // the load, and so does a copy of one register set into the other at the loop's end: the
        // loop is unrolled over the two sets instead)
    };
    auto group = [&](int G, const W& wcur) {
        // the group's sixteen NT activation operands go out together; left to itself the
        // scheduler sinks each load next to its use and the loop becomes a chain of waits
        bf16x8 af[4 * NT];
#pragma unroll
        for (int i = 0; i < 4 * NT; i++)
            af[i] = __builtin_bit_cast(bf16x8, xf[((size_t)G * 4 * NT + i) * 64 + lane]);
        __builtin_amdgcn_sched_barrier(0);
        const float scale = mx_scale((uint8_t)wcur.e);
        const bool past = 4 * G + kq >= nblk;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const u32 q = past ? 0u : wcur.q[j];
            const u32x4 wv = {__builtin_bit_cast(u32, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q, scale, 0)),
                              __builtin_bit_cast(u32, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q, scale, 1)),
                              __builtin_bit_cast(u32, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q, scale, 2)),
                              __builtin_bit_cast(u32, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q, scale, 3))};
            const bf16x8 wf = __builtin_bit_cast(bf16x8, wv);
#pragma unroll
            for (int t = 0; t < NT; t++)
                out[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[j * NT + t], wf, out[t], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    // A wavefront's groups are wave, wave + 8, ...: four of them (all of K = 4096) have their weights
    // requested together before the first group's fragments, so the weights make ONE trip to memory
    // a wavefront; a group's matrix work is far too short to cover the next group's trip.
    for (int G0 = wave; G0 < ngroups; G0 += 32) {
        W w[4];
#pragma unroll
        for (int i = 0; i < 4; i++)
            if (G0 + 8 * i < ngroups) load_w(G0 + 8 * i, w[i]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 4; i++)
            if (G0 + 8 * i < ngroups) group(G0 + 8 * i, w[i]);
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
                if (tok < p.ntok) p.out[(size_t)tok * p.nrows + r] = s[i];
            }
        }
    }
}
