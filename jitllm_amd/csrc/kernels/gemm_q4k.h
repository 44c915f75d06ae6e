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
// Layout.  A workgroup owns a 128-token x 128-row tile and walks K in half
// super-blocks (a "stage": 128 weights, plus the 16 minimum columns in the first
// half).  Weights are dequantized from HBM straight into an LDS stage as f16
// (magic-number nibble unpack with packed-f16 FMAs, eight K values per 32-bit
// word of nibbles); activations were laid out by the prep kernel in exactly the
// stage's LDS image -- same K permutation, same padding -- so their stage is one
// contiguous copy.  Two stages are double-buffered.  Four consumer wavefronts each compute 64 tokens x 64 rows as
// 2x2 MFMA tiles while four producer wavefronts fill the next stage; tokens are the MFMA M dimension so a lane owns one weight row
// (its scales are scalars) and output stores run along rows.
#pragma once
#include "args.h"
#include "common.h"
#include "quantize.h"

// Phase marker for profiling builds; expands to nothing in the product.
#ifndef JL_TRACE
#define JL_TRACE(i)
#endif
#ifndef JL_GEMM_SKIP_PRODUCER
#define JL_GEMM_SKIP_PRODUCER 0
#define JL_GEMM_SKIP_CONSUMER 0
#endif

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

#define JL_GEMM_TILE 128          // tokens and rows per workgroup
#define JL_GEMM_STRIDE 152        // f16 per LDS row of a stage: 144 used + 8 pad (304 B, odd multiple of 16 B)
#define JL_GEMM_STAGE_HALFS (JL_GEMM_TILE * JL_GEMM_STRIDE)
#define JL_GEMM_STAGE_BYTES (JL_GEMM_STAGE_HALFS * 2)

// Workgroup barrier that orders LDS traffic only.  __syncthreads() carries a
// release fence that also drains every outstanding global load, which would
// throw away the register prefetch that is meant to stay in flight across it.
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// K position (within a stage's 128 weights) of nibble pair i of 32-bit word c of a
// 64-element group: word c holds bytes 4c..4c+3; byte b's low nibble is element
// 4c+b of the group's first sub-block, its high nibble the same element of the
// second.  The unpack below emits, per word, the eight values
//   (b0.lo, b2.lo, b0.hi, b2.hi, b1.lo, b3.lo, b1.hi, b3.hi)
// and the prep kernel writes activations in the same order.

// -------------------------------------------------------------------- prep
// x [ntok][k] f32 -> bq [nsb][2][tok_pad][152] f16 and da [nsb][tok_pad] f32.
// One wavefront per (token, super-block); lane l owns elements 4l..4l+3.
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
    _Float16* dst = (_Float16*)p.bq + ((size_t)(sb * 2 + (g >> 1)) * p.tok_pad + t) * JL_GEMM_STRIDE;
    const int base = 8 * (8 * (g & 1) + c) + 2 * hi;
    f16x2 p02 = {(_Float16)(float)(int8_t)(q & 0xFF), (_Float16)(float)(int8_t)((q >> 16) & 0xFF)};
    f16x2 p13 = {(_Float16)(float)(int8_t)((q >> 8) & 0xFF), (_Float16)(float)(int8_t)(q >> 24)};
    *(f16x2*)(dst + base) = p02;
    *(f16x2*)(dst + base + 4) = p13;
    if ((lane & 7) == 0) {
        const int s = lane >> 3;
        _Float16* aug = (_Float16*)p.bq + ((size_t)(sb * 2 + 1) * p.tok_pad + t) * JL_GEMM_STRIDE + 128;
        aug[s] = (_Float16)(float)(a32 & 63);       // A = 64*A_hi + A_lo, 0 <= A_lo < 64
        aug[8 + s] = (_Float16)(float)(a32 >> 6);   // arithmetic shift: floor
    }
    if (lane == 0) p.da[(size_t)sb * p.tok_pad + t] = d;
}

// -------------------------------------------------------------------- main
// One stage of weights for this thread: row = tid/2, hh = tid%2 selects the
// 64-element group (2*half + hh) of the super-block.
struct GemmWRegs {
    u32x4 hdr;
    u32x4 q[2];
};

__device__ __forceinline__ void gemm_load_w(const GemmArgs& p, int row, int sb, int g, GemmWRegs& r) {
    const uint8_t* blk = p.w + (size_t)row * p.row_bytes + (size_t)sb * 144;
    r.hdr = ld16(blk);
    r.q[0] = ld16(blk + 16 + 32 * g);
    r.q[1] = ld16(blk + 32 + 32 * g);
}

// (1024 + n) as f16 for the nibble in bits 0-3 of each 16-bit half
__device__ __forceinline__ f16x2 nib_pair(u32 w, int shift) {
    u32 v = ((w >> shift) & 0x000F000Fu) | 0x64006400u;
    return __builtin_bit_cast(f16x2, v);
}

// Dequantize one thread's stage share into LDS: 8 words of nibbles -> 8 K-groups
// of eight f16 (sc*q); in the first half also the 16 minimum columns and the
// row's (d, dmin).
__device__ __forceinline__ void gemm_store_w(const GemmWRegs& r, int row, int hh, int half, _Float16* sw,
                                             float* sscale) {
    const int g = 2 * half + hh;
    // scales of sub-blocks 2g (low nibbles) and 2g+1 (high nibbles), straight from the
    // packed bytes (format/quant/dequant.go:360-365)
    u32 slo, shi;
    {
        const int sh = 16 * (g & 1);
        const u32 A = r.hdr.y >> sh, C = r.hdr.w >> sh;
        if (half == 0) {
            slo = A & 63;
            shi = (A >> 8) & 63;
        } else {
            slo = (C & 0xF) | (((A >> 6) & 3) << 4);
            shi = ((C >> 8) & 0xF) | (((A >> 14) & 3) << 4);
        }
    }
    const _Float16 flo = (_Float16)(float)slo, fhi = (_Float16)(float)shi;
    const f16x2 mlo = {flo, flo}, mhi = {fhi, fhi};
    const _Float16 nlo = (_Float16)(-1024.0f * (float)slo), nhi = (_Float16)(-1024.0f * (float)shi);
    const f16x2 alo = {nlo, nlo}, ahi = {nhi, nhi};
    _Float16* dst = sw + row * JL_GEMM_STRIDE + 64 * hh;
#pragma unroll
    for (int c = 0; c < 8; c++) {
        const u32 w = c < 4 ? r.q[0][c] : r.q[1][c - 4];
        // (1024+n)*sc - 1024*sc = sc*n, exact in f16 (<= 945) through the fused multiply-add
        f16x2 p0 = __builtin_elementwise_fma(nib_pair(w, 0), mlo, alo);
        f16x2 p1 = __builtin_elementwise_fma(nib_pair(w, 4), mhi, ahi);
        f16x2 p2 = __builtin_elementwise_fma(nib_pair(w, 8), mlo, alo);
        f16x2 p3 = __builtin_elementwise_fma(nib_pair(w, 12), mhi, ahi);
        u32x4 o = {__builtin_bit_cast(u32, p0), __builtin_bit_cast(u32, p1), __builtin_bit_cast(u32, p2),
                   __builtin_bit_cast(u32, p3)};
        *(u32x4*)(dst + 8 * c) = o;
    }
    if (half == 1) {
        // minimum columns: hh = 0 writes m_s (pairs with A_lo), hh = 1 writes 64*m_s (pairs with A_hi)
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
}

// One activation stage is 128 tokens x 304 B, contiguous in HBM in exactly its LDS
// image: 2432 vectors of 16 B.  All 512 threads carry it through registers, loaded one
// step ahead -- the 256 consumer threads four vectors each (their registers are nearly
// all accumulators), the 256 producer threads the other 1408.  Plain vector loads issue
// in a few cycles each, where the direct global->LDS form costs the issuing wavefront
// about 150 cycles an instruction, and spread over every wavefront the copy hides under
// the consumers' matrix instructions.
#define JL_GEMM_STAGE_VECS (JL_GEMM_STAGE_BYTES / 16)
template <int N, int FIRST>
struct GemmARegs {
    u32x4 v[N];
    // tid = index within the role (0..255)
    __device__ __forceinline__ void load(const _Float16* src, int tid) {
        const u32x4* s = (const u32x4*)src;
#pragma unroll
        for (int i = 0; i < N; i++) v[i] = s[min(FIRST + tid + 256 * i, JL_GEMM_STAGE_VECS - 1)];
    }
    __device__ __forceinline__ void store(_Float16* dst, int tid) const {
        u32x4* d = (u32x4*)dst;
#pragma unroll
        for (int i = 0; i < N; i++)
            if (FIRST + 256 * (i + 1) <= JL_GEMM_STAGE_VECS || FIRST + tid + 256 * i < JL_GEMM_STAGE_VECS)
                d[FIRST + tid + 256 * i] = v[i];
    }
};
typedef GemmARegs<4, 0> GemmARegsConsumer;      // vectors 0 .. 1023
typedef GemmARegs<6, 1024> GemmARegsProducer;   // vectors 1024 .. 2431

// Producer wavefronts (four): HBM -> registers -> (dequantize) -> LDS, one stage ahead
// of the consumers, with the stage after that in flight in registers.
__device__ __forceinline__ void gemm_producer(const GemmArgs& p, _Float16* sA, _Float16* sW, float* sScale,
                                              float* sDa, int tid, int t0, int r0, int nsteps) {
    const int wrow = min(r0 + (tid >> 1), p.nrows - 1), hh = tid & 1;
    auto a_src = [&](int step) {
        return (const _Float16*)p.bq + ((size_t)step * p.tok_pad + t0) * JL_GEMM_STRIDE;
    };
    GemmWRegs wreg;
    GemmARegsProducer areg;
    areg.load(a_src(0), tid);
    gemm_load_w(p, wrow, 0, hh, wreg);
    areg.store(sA, tid);
    gemm_store_w(wreg, tid >> 1, hh, 0, sW, sScale);
    areg.load(a_src(min(1, nsteps - 1)), tid);
    gemm_load_w(p, wrow, 0, 2 + hh, wreg);
    float da_reg = p.da[t0 + (tid & (JL_GEMM_TILE - 1))];
    lds_barrier();
    for (int step = 0; step < nsteps; step++) {
        JL_TRACE(0);
        if (step + 1 < nsteps && !JL_GEMM_SKIP_PRODUCER) {
            const int nb = (step & 1) ^ 1, nhalf = (step + 1) & 1, nsbi = (step + 1) >> 1;
            // (a) the next stage, loaded into registers a step ago, goes to LDS.  A second
            // half also carries the super-block's row scales and token scales.
#ifdef JL_TRACE_PRODUCER
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            JL_TRACE(1);
#endif
            areg.store(sA + nb * JL_GEMM_STAGE_HALFS, tid);
#ifdef JL_TRACE_PRODUCER
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            JL_TRACE(2);
#endif
            gemm_store_w(wreg, tid >> 1, hh, nhalf, sW + nb * JL_GEMM_STAGE_HALFS,
                         sScale + (nsbi & 1) * 2 * JL_GEMM_TILE);
            if (nhalf == 1 && tid < JL_GEMM_TILE) sDa[(nsbi & 1) * JL_GEMM_TILE + tid] = da_reg;
#ifdef JL_TRACE_PRODUCER
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            JL_TRACE(3);
#else
            JL_TRACE(1);
#endif
            // (b) issue the loads of the stage after it
            const int s2 = min(step + 2, nsteps - 1);
            areg.load(a_src(s2), tid);
            gemm_load_w(p, wrow, s2 >> 1, 2 * (s2 & 1) + hh, wreg);
            da_reg = p.da[(size_t)(s2 >> 1) * p.tok_pad + t0 + (tid & (JL_GEMM_TILE - 1))];
        }
#ifndef JL_TRACE_PRODUCER
        JL_TRACE(2);
        JL_TRACE(3);
#endif
        JL_TRACE(4);
        // the next stage is complete in LDS once every producer has passed here; the
        // register loads of (b) stay in flight across the barrier
        lds_barrier();
        JL_TRACE(5);
    }
}

// Consumer wavefronts (four, one 64-token x 64-row corner each): LDS -> matrix cores,
// fragments fetched a K-step ahead of the instructions that use them; once per
// super-block the minimum columns and the epilogue  out += d_a * (d * P - dmin * M).
__device__ __forceinline__ void gemm_consumer(const GemmArgs& p, _Float16* sA, const _Float16* sW,
                                              const float* sScale, const float* sDa, int wave, int lane,
                                              int t0, int r0, int nsteps) {
    const int wt = ((wave >> 1) & 1) * 64, wr = (wave & 1) * 64;
    const int arow = lane & 31, kg = lane >> 5;
    f32x16 out[2][2], accP[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) out[i][j][e] = 0.f;
    // this wavefront's share of the activation copy
    const int atid = threadIdx.x;  // consumers are threads 0..255
    auto a_src = [&](int step) {
        return (const _Float16*)p.bq + ((size_t)step * p.tok_pad + t0) * JL_GEMM_STRIDE;
    };
    GemmARegsConsumer areg;
    areg.load(a_src(0), atid);
    areg.store(sA, atid);
    areg.load(a_src(min(1, nsteps - 1)), atid);
    lds_barrier();
    for (int step = 0; step < nsteps; step++) {
        const int buf = step & 1, half = step & 1, sb = step >> 1;
        const _Float16* a = sA + buf * JL_GEMM_STAGE_HALFS;
        const _Float16* w = sW + buf * JL_GEMM_STAGE_HALFS;
        JL_TRACE(0);
        if (step + 1 < nsteps) {
            areg.store(sA + (buf ^ 1) * JL_GEMM_STAGE_HALFS, atid);
            areg.load(a_src(min(step + 2, nsteps - 1)), atid);
        }
        JL_TRACE(1);
        JL_TRACE(2);
        if (!JL_GEMM_SKIP_CONSUMER) {
            if (half == 0) {
#pragma unroll
                for (int i = 0; i < 2; i++)
#pragma unroll
                    for (int j = 0; j < 2; j++)
#pragma unroll
                        for (int e = 0; e < 16; e++) accP[i][j][e] = 0.f;
            }
            const _Float16* ap0 = a + (wt + arow) * JL_GEMM_STRIDE + 8 * kg;
            const _Float16* wp0 = w + (wr + arow) * JL_GEMM_STRIDE + 8 * kg;
            f16x8 af[2][2], wf[2][2];
            auto fetch = [&](int slot, int ks) {
#pragma unroll
                for (int i = 0; i < 2; i++) {
                    af[slot][i] = *(const f16x8*)(ap0 + 32 * i * JL_GEMM_STRIDE + 16 * ks);
                    wf[slot][i] = *(const f16x8*)(wp0 + 32 * i * JL_GEMM_STRIDE + 16 * ks);
                }
            };
            fetch(0, 0);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int ks = 0; ks < 8; ks++) {
                // K-step 8 of a second half is the sixteen minimum columns
                // (the scheduling fences keep the fetch a K-step ahead of its use; left
                // alone the compiler re-reads fragments right before the instruction needing them)
                if (ks + 1 < 8 || half == 1) fetch((ks + 1) & 1, ks + 1);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i = 0; i < 2; i++)
#pragma unroll
                    for (int j = 0; j < 2; j++)
                        accP[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[ks & 1][i], wf[ks & 1][j], accP[i][j], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
            JL_TRACE(3);
            if (half == 1) {
                const f32x16 zero = {0};
                const float* ssc = sScale + (sb & 1) * 2 * JL_GEMM_TILE;
                const float* sda = sDa + (sb & 1) * JL_GEMM_TILE;
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    const float dd = ssc[2 * (wr + 32 * j + arow)];
                    const float dmin = ssc[2 * (wr + 32 * j + arow) + 1];
#pragma unroll
                    for (int i = 0; i < 2; i++) {
                        const f32x16 accM = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[0][i], wf[0][j], zero, 0, 0, 0);
#pragma unroll
                        for (int e = 0; e < 16; e++) {
                            const int tk = wt + 32 * i + 8 * (e >> 2) + 4 * kg + (e & 3);
                            const float u = fmaf(dd, accP[i][j][e], -(dmin * accM[e]));
                            out[i][j][e] = fmaf(sda[tk], u, out[i][j][e]);
                        }
                    }
                }
            }
        }
        JL_TRACE(4);
        lds_barrier();
        JL_TRACE(5);
    }
    // store: lane = row (contiguous in memory), register = token
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int r = r0 + wr + 32 * j + arow;
        if (r >= p.nrows) continue;
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const int t = t0 + wt + 32 * i + 8 * (e >> 2) + 4 * kg + (e & 3);
                if (t < p.ntok) p.out[(size_t)t * p.nrows + r] = out[i][j][e];
            }
    }
}

__device__ __forceinline__ void gemm_q4k_body(const GemmArgs& p, uint8_t* smem) {
    // LDS: activation stages [2], weight stages [2], row scales [2][128][2], token scales [2][128]
    _Float16* sA = (_Float16*)smem;
    _Float16* sW = sA + 2 * JL_GEMM_STAGE_HALFS;
    float* sScale = (float*)(sW + 2 * JL_GEMM_STAGE_HALFS);
    float* sDa = sScale + 2 * 2 * JL_GEMM_TILE;
    // Eight wavefronts, two per SIMD: wavefronts 0-3 are consumers, 4-7 producers, so a
    // SIMD always has vector work from its producer to issue under its consumer's matrix
    // instructions.  The two roles are separate loops (their registers never coexist) that
    // meet at the same barriers: one after the prologue, one per stage.
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int t0 = blockIdx.x * JL_GEMM_TILE, r0 = blockIdx.y * JL_GEMM_TILE;
    const int nsteps = 2 * (p.k / 256);
    if (wave >= 4) gemm_producer(p, sA, sW, sScale, sDa, threadIdx.x & 255, t0, r0, nsteps);
    else gemm_consumer(p, sA, sW, sScale, sDa, wave, lane, t0, r0, nsteps);
}
