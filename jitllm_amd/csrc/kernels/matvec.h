// Decode matvec over row-major GGUF blocks: out[r] = sum_k W[r][k] * x[k].
//
// What it computes is the reference's quantized-activation form
// (jit/gpu/kernels/matvec.go:1121-1271, jit/cpu/packedfused.go:200-362): the
// activation is int8 with one f32 scale d_a per 32 elements, each sub-block's
// dot product is an exact int32, and
//     out[r] += d_a * (scale * dot - bias * sum_a)
// with (scale, bias) = (d*sc, dmin*m) for Q4_K, (d*sc, 32*scale) for Q6_K and
// (d, 0) for Q8_0.  Only the f32 summation order differs from the reference.
//
// Shape of the kernel: HBM-bound, so everything is arranged to put the whole
// weight matrix in flight at once.  A wavefront owns RPW rows; a row is cut
// into "slots" (one 64-element group of a Q4_K super-block, one quarter of a
// Q6_K super-block, one Q8_0 block) and lane l takes slots l, l+64, ... so a
// wavefront's 128-bit loads walk a row contiguously.  The int8 activations
// live in LDS, staged once per workgroup -- either copied from a quantizer's
// output or, in the fused form, quantized in place from f32 x while the first
// weight loads are still in flight.  Per-row partial sums are reduced across
// the 64 lanes with cross-lane shuffles.
#pragma once
#include "args.h"
#include "common.h"
#include "quantize.h"

struct __attribute__((packed, aligned(4))) u32x4_a4 { u32x4 v; };   // a 16-byte load on a 4-byte boundary

// Activation staging area in LDS: int8 a[k], then f32 da[k/32], then f32 s16[k/16].
struct ActLds {
    const uint8_t* a;
    const float* da;
    const float* s16;
    const uint8_t* a2;   // the Q8_0 pair form only: a second copy of a[], two bytes further on
};

// Bytes of LDS the staging area needs for a k-element activation.
#define JL_ACT_LDS_BYTES(k) ((k) + ((k) / 32) * 4 + ((k) / 16) * 4)
// the grouped kernels' RMSNorm: up to sixteen partial sums and the scale, behind the staging area
#define JL_NORM_LDS_BYTES 160
// ... and with the second copy of the int8 values that the Q8_0 pair form reads (k % 64 == 0)
#define JL_ACT_LDS_BYTES_SHIFTED(k) (JL_ACT_LDS_BYTES(k) + (k) + 16)

__device__ __forceinline__ ActLds act_lds_views(uint8_t* smem, int k) {
    ActLds v;
    v.a = smem;
    v.da = (const float*)(smem + k);
    v.s16 = (const float*)(smem + k + (k / 32) * 4);
    v.a2 = smem + JL_ACT_LDS_BYTES(k);   // 16-byte aligned when k % 64 == 0
    return v;
}

// Stage pre-quantized activations (global) into LDS.  k % 32 == 0.
// Layouts of the staging area.  JL_STAGE_SHIFTED: also the copy two bytes further on
// (a2[i + 2] = a[i]), written as two 16-bit halves.  JL_STAGE_Q6K: the half-block sums as the
// Q6_K slot wants them -- the integer -32 * sum (the zero point of a 6-bit weight times the
// sum, what its dot-product accumulator starts from), and the eight sums of a 128-element
// half laid (j, q) -> 4 j + q for the sum of elements 32 q + 16 j .., so that the four runs of
// a slot are one 16-byte read.
#define JL_STAGE_PLAIN 0
#define JL_STAGE_SHIFTED 1
#define JL_STAGE_Q6K 2
__device__ __forceinline__ int stage_q6k_sum_index(int h) {   // h = element / 16
    const int p = h & 7;
    return (h & ~7) + ((p & 1) << 2) + (p >> 1);
}

template <int SH = JL_STAGE_PLAIN>
__device__ __forceinline__ void stage_act_copy(uint8_t* smem, const int8_t* q, const float* as,
                                               const float* s16, int k, int nthreads) {
    u32* a = (u32*)smem;
    float* da = (float*)(smem + k);
    float* ss = (float*)(smem + k + (k / 32) * 4);
    for (int i = threadIdx.x; i < k / 4; i += nthreads) {
        const u32 v = ((const u32*)q)[i];
        a[i] = v;
        if (SH == JL_STAGE_SHIFTED) {
            uint16_t* h = (uint16_t*)(smem + JL_ACT_LDS_BYTES(k)) + 2 * i + 1;
            h[0] = (uint16_t)v;
            h[1] = (uint16_t)(v >> 16);
        }
    }
    for (int i = threadIdx.x; i < k / 32; i += nthreads) da[i] = as[i];
    for (int i = threadIdx.x; i < k / 16; i += nthreads) {
        if (SH == JL_STAGE_Q6K) ((i32*)ss)[stage_q6k_sum_index(i)] = -32 * (i32)s16[i];
        else ss[i] = s16[i];
    }
}

// Quantize one float4 of x (element group g4, i.e. elements 4*g4 .. 4*g4+3) into the
// LDS staging area; every lane of a wavefront must call it together (DPP).
template <int SH = JL_STAGE_PLAIN>
__device__ __forceinline__ void stage_quantize4(uint8_t* smem, int k, int per, int g4, f32x4 v) {
    u32* a = (u32*)smem;
    float* da = (float*)(smem + k);
    float* ss = (float*)(smem + k + (k / 32) * 4);
    const bool live = g4 < k / 4;
    u32 m = max(max(abs_bits(v.x), abs_bits(v.y)), max(abs_bits(v.z), abs_bits(v.w)));
    u32 amax = per == 8 ? wave_amax_256(live ? m : 0u) : window_amax(live ? m : 0u, per);
    float d;
    i32 sum;
    u32 q = quantize4(v, amax, d, sum);
    if (live) {
        a[g4] = q;
        if (SH == JL_STAGE_SHIFTED) {
            uint16_t* h = (uint16_t*)(smem + JL_ACT_LDS_BYTES(k)) + 2 * g4 + 1;
            h[0] = (uint16_t)q;
            h[1] = (uint16_t)(q >> 16);
        }
        if ((g4 & 3) == 0) {
            if (SH == JL_STAGE_Q6K) ((i32*)ss)[stage_q6k_sum_index(g4 >> 2)] = -32 * sum;
            else ss[g4 >> 2] = (float)sum;
        }
        if ((g4 & 7) == 0) da[g4 >> 3] = d;
    }
}

// Quantize f32 x into the LDS staging area (same bits as the standalone
// quantizer).  k % 32 == 0, blockDim.x % 64 == 0, per = window / 32.  `first` is
// this thread's first float4 of x, loaded by the caller ahead of time.
// This thread's first XP float4 groups of x (groups tid, tid + nthreads, ...), loaded
// together so that their latency is paid once, under the first weight loads (a loop that
// loads and quantizes a group at a time waits out a load per pass: at k = 14336 three and a
// half passes, about two microseconds before the first row could start).
// XP = 1 for a vector of at most one group a thread (no loads it has no use for go out ahead
// of the weights), 4 for longer ones: the body is compiled for both and chosen once, at its top.
template <int XP>
__device__ __forceinline__ void load_x_groups(const float* x, int k, int nthreads, f32x4 (&xs)[XP]) {
    const int n4 = k / 4;
#pragma unroll
    for (int i = 0; i < XP; i++) xs[i] = ((const f32x4*)x)[min((int)threadIdx.x + i * nthreads, n4 - 1)];
}

template <int SH, int XP>
__device__ __forceinline__ void stage_act_quantize(uint8_t* smem, const float* x, int k, int per,
                                                   const f32x4 (&first)[XP], int nthreads) {
    const int n4 = k / 4;
    const int n4_pad = (n4 + 63) & ~63;  // whole wavefronts take part in the lane exchanges
    int g4 = threadIdx.x;
#pragma unroll
    for (int i = 0; i < XP; i++, g4 += nthreads)
        if (g4 < n4_pad) stage_quantize4<SH>(smem, k, per, g4, first[i]);   // (a group past n4 is not stored)
    for (; g4 < n4_pad; g4 += nthreads) {
        f32x4 v = g4 < n4 ? ((const f32x4*)x)[g4] : f32x4{0.f, 0.f, 0.f, 0.f};
        stage_quantize4<SH>(smem, k, per, g4, v);
    }
}

// ---------------------------------------------------------------- Q4_K slot
// slot = (super-block sb, group g of 64 elements): 32 bytes of nibbles whose
// low halves are sub-block 2g and high halves sub-block 2g+1
// (format/quant/dequant.go:367-397).
struct SlotActQ4K {
    u32x4 lo[2], hi[2];  // int8 activations of sub-block 2g / 2g+1
    float da_lo, da_hi;  // their scales
    float s_lo, s_hi;    // their integer sums
};

__device__ __forceinline__ void load_act_q4k(const ActLds& A, int slot, SlotActQ4K& s) {
    int e0 = slot * 64;  // first element of the group
    const u32x4* a = (const u32x4*)(A.a + e0);
    s.lo[0] = a[0]; s.lo[1] = a[1]; s.hi[0] = a[2]; s.hi[1] = a[3];
    s.da_lo = A.da[e0 / 32];
    s.da_hi = A.da[e0 / 32 + 1];
    s.s_lo = A.s16[e0 / 16] + A.s16[e0 / 16 + 1];
    s.s_hi = A.s16[e0 / 16 + 2] + A.s16[e0 / 16 + 3];
}

struct SlotWQ4K {
    u32x4 hdr;    // f16 d, f16 dmin, 12 scale bytes
    u32x4 q[2];   // 32 bytes of nibbles
};

__device__ __forceinline__ void load_w_q4k(const uint8_t* row, int slot, SlotWQ4K& w) {
    const uint8_t* blk = row + (size_t)(slot >> 2) * 144;
    w.hdr = ld16(blk);
    const uint8_t* qs = blk + 16 + (slot & 3) * 32;
    w.q[0] = ld16(qs);
    w.q[1] = ld16(qs + 16);
}

// A slot's weights with the scale arithmetic done: what stays the same when the
// slot meets several activations (the columns of a mixture-of-experts pass).
struct PrepQ4K {
    u32x4 lo[2], hi[2];    // nibbles of sub-blocks 2g / 2g+1 as bytes
    float dsc_lo, dsc_hi;  // d * sc of sub-blocks 2g, 2g+1
    float dm_lo, dm_hi;    // dmin * m
};

__device__ __forceinline__ void prep_q4k(const SlotWQ4K& w, int g, PrepQ4K& P) {
    float d = half_bits_to_f32((uint16_t)(w.hdr.x & 0xFFFF));
    float dmin = half_bits_to_f32((uint16_t)(w.hdr.x >> 16));
    // 6-bit scale/min pairs of sub-blocks 2g and 2g+1, branch-free
    int sh = 16 * (g & 1);
    u32 A = w.hdr.y >> sh, B = w.hdr.z >> sh, C = w.hdr.w >> sh;
    u32 sc_lo, sc_hi, m_lo, m_hi;
    if (g < 2) {
        sc_lo = A & 63; sc_hi = (A >> 8) & 63;
        m_lo = B & 63;  m_hi = (B >> 8) & 63;
    } else {
        sc_lo = (C & 0xF) | (((A >> 6) & 3) << 4);
        sc_hi = ((C >> 8) & 0xF) | (((A >> 14) & 3) << 4);
        m_lo = ((C >> 4) & 0xF) | (((B >> 6) & 3) << 4);
        m_hi = ((C >> 12) & 0xF) | (((B >> 14) & 3) << 4);
    }
#pragma unroll
    for (int i = 0; i < 2; i++) {
        P.lo[i] = w.q[i] & 0x0F0F0F0Fu;
        P.hi[i] = (w.q[i] >> 4) & 0x0F0F0F0Fu;
    }
    P.dsc_lo = d * (float)sc_lo; P.dsc_hi = d * (float)sc_hi;
    P.dm_lo = dmin * (float)m_lo; P.dm_hi = dmin * (float)m_hi;
}

__device__ __forceinline__ float dotp_q4k(const PrepQ4K& w, const SlotActQ4K& s) {
    i32 dl = 0, dh = 0;
#pragma unroll
    for (int i = 0; i < 2; i++) {
        dl = dot4(w.lo[i].x, s.lo[i].x, dl);
        dl = dot4(w.lo[i].y, s.lo[i].y, dl);
        dl = dot4(w.lo[i].z, s.lo[i].z, dl);
        dl = dot4(w.lo[i].w, s.lo[i].w, dl);
        dh = dot4(w.hi[i].x, s.hi[i].x, dh);
        dh = dot4(w.hi[i].y, s.hi[i].y, dh);
        dh = dot4(w.hi[i].z, s.hi[i].z, dh);
        dh = dot4(w.hi[i].w, s.hi[i].w, dh);
    }
    float v_lo = (float)dl * w.dsc_lo - s.s_lo * w.dm_lo;
    float v_hi = (float)dh * w.dsc_hi - s.s_hi * w.dm_hi;
    return fmaf(v_lo, s.da_lo, v_hi * s.da_hi);
}

__device__ __forceinline__ float dot_q4k(const SlotWQ4K& w, int g, const SlotActQ4K& s) {
    PrepQ4K P;
    prep_q4k(w, g, P);
    return dotp_q4k(P, s);
}

// ---------------------------------------------------------------- Q8_0 slot
// slot = one 34-byte block: f16 d, 32 int8 (format/quant/dequant.go:148-157).
struct SlotActQ8 {
    u32x4 a[2];
    float da;
};

__device__ __forceinline__ void load_act_q8(const ActLds& A, int slot, SlotActQ8& s) {
    const u32x4* a = (const u32x4*)(A.a + slot * 32);
    s.a[0] = a[0]; s.a[1] = a[1];
    s.da = A.da[slot];
}

struct SlotWQ8 {
    u32x4 q[2];
    uint16_t d;
};

__device__ __forceinline__ void load_w_q8(const uint8_t* row, int slot, SlotWQ8& w) {
    const uint8_t* blk = row + (size_t)slot * 34;
    w.d = ld2(blk);
    w.q[0] = ld16_a2(blk + 2);
    w.q[1] = ld16_a2(blk + 18);
}

struct PrepQ8 {
    u32x4 q[2];
    float d;
};

__device__ __forceinline__ void prep_q8(const SlotWQ8& w, PrepQ8& P) {
    P.q[0] = w.q[0]; P.q[1] = w.q[1];
    P.d = half_bits_to_f32(w.d);
}

__device__ __forceinline__ float dotp_q8(const PrepQ8& w, const SlotActQ8& s) {
    i32 dt = 0;
#pragma unroll
    for (int i = 0; i < 2; i++) {
        dt = dot4(w.q[i].x, s.a[i].x, dt);
        dt = dot4(w.q[i].y, s.a[i].y, dt);
        dt = dot4(w.q[i].z, s.a[i].z, dt);
        dt = dot4(w.q[i].w, s.a[i].w, dt);
    }
    return (float)dt * w.d * s.da;
}

__device__ __forceinline__ float dot_q8(const SlotWQ8& w, const SlotActQ8& s) {
    PrepQ8 P;
    prep_q8(w, P);
    return dotp_q8(P, s);
}

// ------------------------------------------------- Q8_0, two blocks a slot
// A 34-byte block leaves every second block's int8 values two bytes off a 32-bit boundary,
// and a 16-byte load that is only 2-byte aligned is served at about three quarters of the
// rate of one that is 4-byte aligned (a pure read of 62 MB: 14.2 against 11.2 us).  Two blocks
// are 68 bytes, so a slot of two blocks is seventeen 4-byte-aligned words
//   w0 = d0 | q0[0..1] << 16,  w1..w7 = q0[2..29],  w8 = q0[30..31] | d1 << 16,  w9..w16 = q1[0..31].
// Block 1's values sit on word boundaries.  Block 0's sit two bytes into theirs: they meet a
// second copy of the activations laid two bytes further on (ActLds.a2, so that word m of it is
// a[4m-2 .. 4m+1]), with the scale halves of w0 and w8 masked off.
// Rows must be 4-byte aligned and k a multiple of 64.
#define JL_Q8_0P 1008   // (not a ggml type: the kernel form's tag)
struct SlotActQ8P {
    u32x4 s[2];   // a[-2 .. 29] of block 0, as the shifted copy has them
    u32 s8;       // a[30 .. 33]
    u32x4 a[2];   // a[0 .. 31] of block 1
    float da0, da1;
};

__device__ __forceinline__ void load_act_q8p(const ActLds& A, int slot, SlotActQ8P& s) {
    const u32* a2 = (const u32*)A.a2 + 16 * slot;
    s.s[0] = *(const u32x4*)a2;
    s.s[1] = *(const u32x4*)(a2 + 4);
    s.s8 = a2[8];
    const u32x4* a = (const u32x4*)(A.a + slot * 64 + 32);
    s.a[0] = a[0]; s.a[1] = a[1];
    s.da0 = A.da[2 * slot];
    s.da1 = A.da[2 * slot + 1];
}

struct SlotWQ8P {
    u32x4 q[4];
    u32 t;
};

__device__ __forceinline__ void load_w_q8p(const uint8_t* row, int slot, SlotWQ8P& w) {
    const uint8_t* blk = row + (size_t)slot * 68;
#pragma unroll
    for (int i = 0; i < 4; i++) w.q[i] = ((const u32x4_a4*)(blk + 16 * i))->v;
    w.t = *(const u32*)(blk + 64);
}

__device__ __forceinline__ float dot_q8p(const SlotWQ8P& w, const SlotActQ8P& s) {
    i32 t0 = dot4(w.q[0].x & 0xFFFF0000u, s.s[0].x, 0);
    t0 = dot4(w.q[0].y, s.s[0].y, t0);
    t0 = dot4(w.q[0].z, s.s[0].z, t0);
    t0 = dot4(w.q[0].w, s.s[0].w, t0);
    t0 = dot4(w.q[1].x, s.s[1].x, t0);
    t0 = dot4(w.q[1].y, s.s[1].y, t0);
    t0 = dot4(w.q[1].z, s.s[1].z, t0);
    t0 = dot4(w.q[1].w, s.s[1].w, t0);
    t0 = dot4(w.q[2].x & 0x0000FFFFu, s.s8, t0);
    i32 t1 = dot4(w.q[2].y, s.a[0].x, 0);
    t1 = dot4(w.q[2].z, s.a[0].y, t1);
    t1 = dot4(w.q[2].w, s.a[0].z, t1);
    t1 = dot4(w.q[3].x, s.a[0].w, t1);
    t1 = dot4(w.q[3].y, s.a[1].x, t1);
    t1 = dot4(w.q[3].z, s.a[1].y, t1);
    t1 = dot4(w.q[3].w, s.a[1].z, t1);
    t1 = dot4(w.t, s.a[1].w, t1);
    const float d0 = half_bits_to_f32((uint16_t)(w.q[0].x & 0xFFFF));
    const float d1 = half_bits_to_f32((uint16_t)(w.q[2].x >> 16));
    return (float)t0 * d0 * s.da0 + (float)t1 * d1 * s.da1;
}

// ---------------------------------------------------------------- Q6_K slot
// slot = (super-block sb, half n, 16-run j): ql[16] (low nibbles = sub-block
// 8n+j, high = 8n+4+j), ql[32+16] (sub-blocks 8n+2+j / 8n+6+j) and qh[16] (two
// bits for each of the four), format/quant/dequant.go:443-470.  Each of the
// four 16-element runs is a whole sub-block with its own int8 scale.
struct SlotActQ6K {
    u32x4 a[4];   // runs at elements 128n + 32q + 16j, q = 0..3
    float da[4];
    float s[4];
};

__device__ __forceinline__ void load_act_q6k(const ActLds& A, int slot, SlotActQ6K& s) {
    int sb = slot >> 2, n = (slot >> 1) & 1, j = slot & 1;
    int e0 = sb * 256 + n * 128 + j * 16;
#pragma unroll
    for (int q = 0; q < 4; q++) {
        int e = e0 + 32 * q;
        s.a[q] = *(const u32x4*)(A.a + e);
        s.da[q] = A.da[e / 32];
        s.s[q] = A.s16[e / 16];
    }
}

struct SlotWQ6K {
    u32x4 qla, qlb, qh;
    u32 sc;       // four int8 scales, byte q = sub-block 8n + 2q + j
    uint16_t d;
};

__device__ __forceinline__ void load_w_q6k(const uint8_t* row, int slot, SlotWQ6K& w) {
    int sb = slot >> 2, n = (slot >> 1) & 1, j = slot & 1;
    const uint8_t* blk = row + (size_t)sb * 210;
    w.qla = ld16_a2(blk + n * 64 + j * 16);
    w.qlb = ld16_a2(blk + n * 64 + 32 + j * 16);
    w.qh = ld16_a2(blk + 128 + n * 32 + j * 16);
    // the half's eight int8 scales in one load; bytes j, j+2, j+4, j+6 are this slot's
    const u32x2 s8 = ld8_a2(blk + 192 + n * 8);
    const u32 lo = (s8.x >> (8 * j)) & 0x00FF00FFu, hi = (s8.y >> (8 * j)) & 0x00FF00FFu;
    w.sc = (lo & 0xFF) | ((lo >> 8) & 0xFF00) | ((hi & 0xFF) << 16) | ((hi >> 16) << 24);
    w.d = ld2(blk + 208);
}

// (Reading each 16-byte field as five 4-byte-aligned words moved down by a funnel shift, so
// that no load of an odd super-block is only 2-byte aligned, measured slower: eight load
// instructions a slot instead of five, 14.0 against 13.6 us at 4096 x 14336.)
__device__ __forceinline__ i32 dot16(u32x4 q, u32x4 a) {
    i32 t = dot4(q.x, a.x, 0);
    t = dot4(q.y, a.y, t);
    t = dot4(q.z, a.z, t);
    return dot4(q.w, a.w, t);
}

// The same slot over the staging layout JL_STAGE_Q6K: the four runs' scales and (already
// multiplied by the zero point) sums are one 16-byte read each, the dot products accumulate
// onto the sums as integers, and the block scale d multiplies the slot's total once.
#define JL_Q6_KS 1014   // (not a ggml type: the kernel form's tag)
struct SlotActQ6KS {
    u32x4 a[4];
    f32x4 da;
    u32x4 s;      // int32: -32 * sum of each run
};

__device__ __forceinline__ void load_act_q6ks(const ActLds& A, int slot, SlotActQ6KS& s) {
    const int h = slot >> 1, j = slot & 1;   // half-super-block h = 2 sb + n
    const u32x4* a = (const u32x4*)(A.a + h * 128 + j * 16);
    s.a[0] = a[0]; s.a[1] = a[2]; s.a[2] = a[4]; s.a[3] = a[6];
    s.da = *(const f32x4*)(A.da + 4 * h);
    s.s = *(const u32x4*)((const u32*)A.s16 + 8 * h + 4 * j);
}

__device__ __forceinline__ i32 dot16_acc(u32x4 q, u32x4 a, i32 t) {
    t = dot4(q.x, a.x, t);
    t = dot4(q.y, a.y, t);
    t = dot4(q.z, a.z, t);
    return dot4(q.w, a.w, t);
}

__device__ __forceinline__ float dot_q6ks(const SlotWQ6K& w, const SlotActQ6KS& s) {
    const u32 M4 = 0x0F0F0F0Fu, M2 = 0x30303030u;
    const u32x4 q0 = (w.qla & M4) | ((w.qh << 4) & M2);
    const u32x4 q1 = (w.qlb & M4) | ((w.qh << 2) & M2);
    const u32x4 q2 = ((w.qla >> 4) & M4) | (w.qh & M2);
    const u32x4 q3 = ((w.qlb >> 4) & M4) | ((w.qh >> 2) & M2);
    // value = d * sc * (q - 32): the zero point is in the accumulator's start
    const float t0 = (float)dot16_acc(q0, s.a[0], (i32)s.s.x) * (float)(int8_t)(w.sc & 0xFF);
    const float t1 = (float)dot16_acc(q1, s.a[1], (i32)s.s.y) * (float)(int8_t)((w.sc >> 8) & 0xFF);
    const float t2 = (float)dot16_acc(q2, s.a[2], (i32)s.s.z) * (float)(int8_t)((w.sc >> 16) & 0xFF);
    const float t3 = (float)dot16_acc(q3, s.a[3], (i32)s.s.w) * (float)(int8_t)(w.sc >> 24);
    float acc = t0 * s.da.x;
    acc = fmaf(t1, s.da.y, acc);
    acc = fmaf(t2, s.da.z, acc);
    acc = fmaf(t3, s.da.w, acc);
    return acc * half_bits_to_f32(w.d);
}

struct PrepQ6K {
    u32x4 q[4];   // the four 16-element runs as bytes 0..63
    float sc[4];  // d * int8 scale of each run
};

__device__ __forceinline__ void prep_q6k(const SlotWQ6K& w, PrepQ6K& P) {
    const u32 M4 = 0x0F0F0F0Fu, M2 = 0x30303030u;
    P.q[0] = (w.qla & M4) | ((w.qh << 4) & M2);
    P.q[1] = (w.qlb & M4) | ((w.qh << 2) & M2);
    P.q[2] = ((w.qla >> 4) & M4) | (w.qh & M2);
    P.q[3] = ((w.qlb >> 4) & M4) | ((w.qh >> 2) & M2);
    float d = half_bits_to_f32(w.d);
    P.sc[0] = d * (float)(int8_t)(w.sc & 0xFF);
    P.sc[1] = d * (float)(int8_t)((w.sc >> 8) & 0xFF);
    P.sc[2] = d * (float)(int8_t)((w.sc >> 16) & 0xFF);
    P.sc[3] = d * (float)(int8_t)(w.sc >> 24);
}

__device__ __forceinline__ float dotp_q6k(const PrepQ6K& w, const SlotActQ6K& s) {
    float acc = 0.f;
    // value = d*sc*(q-32): the zero point goes through the activation sum
#pragma unroll
    for (int j = 0; j < 4; j++) {
        float t = (float)(dot16(w.q[j], s.a[j])) - 32.f * s.s[j];
        acc = fmaf(t * w.sc[j], s.da[j], acc);
    }
    return acc;
}

__device__ __forceinline__ float dot_q6k(const SlotWQ6K& w, const SlotActQ6K& s) {
    PrepQ6K P;
    prep_q6k(w, P);
    return dotp_q6k(P, s);
}

// ------------------------------------------------------------- the kernel
__device__ constexpr int stage_layout_of(int type) {
    return type == JL_Q8_0P ? JL_STAGE_SHIFTED : type == JL_Q6_KS ? JL_STAGE_Q6K : JL_STAGE_PLAIN;
}
template <int TYPE> struct SlotTraits;
template <> struct SlotTraits<JL_Q4_K> {
    typedef SlotActQ4K Act; typedef SlotWQ4K W;
    static constexpr int kElems = 64;
    static __device__ __forceinline__ void load_act(const ActLds& A, int s, Act& a) { load_act_q4k(A, s, a); }
    static __device__ __forceinline__ void load_w(const uint8_t* row, int s, W& w) { load_w_q4k(row, s, w); }
    static __device__ __forceinline__ float dot(const W& w, int s, const Act& a) { return dot_q4k(w, s & 3, a); }
    typedef PrepQ4K Prep;
    static __device__ __forceinline__ void prep(const W& w, int s, Prep& P) { prep_q4k(w, s & 3, P); }
    static __device__ __forceinline__ float dotp(const Prep& P, const Act& a) { return dotp_q4k(P, a); }
};
template <> struct SlotTraits<JL_Q8_0> {
    typedef SlotActQ8 Act; typedef SlotWQ8 W;
    static constexpr int kElems = 32;
    static __device__ __forceinline__ void load_act(const ActLds& A, int s, Act& a) { load_act_q8(A, s, a); }
    static __device__ __forceinline__ void load_w(const uint8_t* row, int s, W& w) { load_w_q8(row, s, w); }
    static __device__ __forceinline__ float dot(const W& w, int, const Act& a) { return dot_q8(w, a); }
    typedef PrepQ8 Prep;
    static __device__ __forceinline__ void prep(const W& w, int, Prep& P) { prep_q8(w, P); }
    static __device__ __forceinline__ float dotp(const Prep& P, const Act& a) { return dotp_q8(P, a); }
};
template <> struct SlotTraits<JL_Q8_0P> {
    typedef SlotActQ8P Act; typedef SlotWQ8P W;
    static constexpr int kElems = 64;
    static __device__ __forceinline__ void load_act(const ActLds& A, int s, Act& a) { load_act_q8p(A, s, a); }
    static __device__ __forceinline__ void load_w(const uint8_t* row, int s, W& w) { load_w_q8p(row, s, w); }
    static __device__ __forceinline__ float dot(const W& w, int, const Act& a) { return dot_q8p(w, a); }
};
template <> struct SlotTraits<JL_Q6_KS> {
    typedef SlotActQ6KS Act; typedef SlotWQ6K W;
    static constexpr int kElems = 64;
    static __device__ __forceinline__ void load_act(const ActLds& A, int s, Act& a) { load_act_q6ks(A, s, a); }
    static __device__ __forceinline__ void load_w(const uint8_t* row, int s, W& w) { load_w_q6k(row, s, w); }
    static __device__ __forceinline__ float dot(const W& w, int, const Act& a) { return dot_q6ks(w, a); }
};
template <> struct SlotTraits<JL_Q6_K> {
    typedef SlotActQ6K Act; typedef SlotWQ6K W;
    static constexpr int kElems = 64;
    static __device__ __forceinline__ void load_act(const ActLds& A, int s, Act& a) { load_act_q6k(A, s, a); }
    static __device__ __forceinline__ void load_w(const uint8_t* row, int s, W& w) { load_w_q6k(row, s, w); }
    static __device__ __forceinline__ float dot(const W& w, int, const Act& a) { return dot_q6k(w, a); }
    typedef PrepQ6K Prep;
    static __device__ __forceinline__ void prep(const W& w, int, Prep& P) { prep_q6k(w, P); }
    static __device__ __forceinline__ float dotp(const Prep& P, const Act& a) { return dotp_q6k(P, a); }
};


// The row loop of one wavefront: rows r0, r0 + group_stride, ... (RPW at a time), each row's
// slots dealt to the lanes in chunks of 64.  w holds the first step's weights, loaded by the
// caller before the activation was staged; every later step's loads are issued when the step
// begins, and the dozen or so wavefronts of a CU cover each other's latency.  (A two-deep
// pipeline -- the next step's weight loads issued BEFORE the current step's dot products, into
// a second register set -- measured slower for every type but Q4_K, where they tie: more loads
// in flight per wavefront do not help a kernel that is not waiting on latency.  Kept behind a
// run-time switch it also cost the plain loop, so it is gone.  So did requesting all four chunks
// of a long row before the activation is staged: Q6_K 4096 x 14336 13.4 -> 16.3 us, and 13.3 ->
// 14.7 with the loads' issue order pinned and the waits checked in the assembly (15, 10, 5, 0
// loads left in flight before the four dot products): a CU returns its loads in the order they
// were issued, so the last wavefront's first chunk arrives behind the first wavefront's last.)
// store(row, total) receives a finished row in lane 63.
template <int TYPE, int RPW, class Store>
__device__ __forceinline__ void matvec_rows(const uint8_t* w0, int row_bytes, const ActLds& A, int nrows, int r0,
                                            int group_stride, int nslots, int lane,
                                            typename SlotTraits<TYPE>::W (&w)[RPW], Store store) {
    typedef SlotTraits<TYPE> T;
    float acc[RPW];
#pragma unroll
    for (int j = 0; j < RPW; j++) acc[j] = 0.f;
    bool preloaded = true;
    for (; r0 < nrows; r0 += group_stride) {
        for (int slot = lane; slot < nslots; slot += 64) {
            if (!preloaded) {
#pragma unroll
                for (int j = 0; j < RPW; j++)
                    T::load_w(w0 + (size_t)min(r0 + j, nrows - 1) * row_bytes, slot, w[j]);
            }
            preloaded = false;
            typename T::Act a;
            T::load_act(A, slot, a);
#pragma unroll
            for (int j = 0; j < RPW; j++) acc[j] += T::dot(w[j], slot, a);
        }
        preloaded = false;
#pragma unroll
        for (int j = 0; j < RPW; j++) {
            const float t = wave_sum_to_lane63(acc[j]);
            if (lane == 63 && r0 + j < nrows) store(r0 + j, t);
            acc[j] = 0.f;
        }
    }
}

// Weight of a residual add: alpha, or alpha * sigmoid(logit) when the add is gated by a
// logit in device memory (a shared expert's contribution, engine/model/moe.go:401-497;
// sigma(x) = 1/(1+exp(-x)) in f64, narrowed once, internal/oracle/moe.go:361-370).
__device__ __forceinline__ float resid_weight(float alpha, const float* gate) {
    if (!gate) return alpha;
    return alpha * (float)(1.0 / (1.0 + exp(-(double)*gate)));
}

// One wavefront computes RPW rows at a time and strides over the row groups of
// a persistent grid.  The first group's weight loads are issued before the
// activation is staged, so HBM latency overlaps the quantizer; after that each
// group is load -> dot -> cross-lane reduce, and the wavefronts of a CU (two
// workgroups of eight, or one of sixteen) cover each other's memory latency.
// RES: the residual add rides on the store (entry points of their own: with the add and its
// gate's f64 exponential compiled into the plain kernel behind a branch, the plain matvecs ran
// 10-20 % slower, Q8_0 14336 x 4096 14.2 against 11.8 us).
// PQ: the activation comes quantized (MatVecArgs.q / as / s16) and is only copied into LDS.
template <int TYPE, int RPW, int XP, bool RES, bool PQ>
__device__ __forceinline__ void matvec_body_xp(const MatVecArgs& p, uint8_t* smem) {
    typedef SlotTraits<TYPE> T;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = p.nwaves;
    const int nslots = p.k / T::kElems;
    const int rows_per_block = nwaves * RPW;
    const int group_stride = p.ngroups * rows_per_block;
    const ActLds A = act_lds_views(smem, p.k);
    int r0 = blockIdx.x * rows_per_block + wave * RPW;

    // The activation loads go first, for the whole workgroup: a CU serves its vector
    // loads in the order they were issued whichever wavefront issued them, so every
    // wavefront issues its x load, the workgroup meets at a barrier that waits for no
    // data, and only then do the weight loads go out.  The quantizer starts as soon as x
    // is back while the first weight loads are still in flight.
    f32x4 x0[XP];
#pragma unroll
    for (int i = 0; i < XP; i++) x0[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    if constexpr (!PQ) {
        load_x_groups<XP>(p.x, p.k, nwaves * 64, x0);
        __builtin_amdgcn_s_barrier();
    }

    typename T::W w[RPW];
    {
        const int s = min(lane, nslots - 1);
#pragma unroll
        for (int j = 0; j < RPW; j++)
            T::load_w(p.w + (size_t)min(r0 + j, p.nrows - 1) * p.row_bytes, s, w[j]);
    }
    constexpr int SH = stage_layout_of(TYPE);
    if constexpr (!PQ) stage_act_quantize<SH, XP>(smem, p.x, p.k, p.per, x0, nwaves * 64);
    else stage_act_copy<SH>(smem, p.q, p.as, p.s16, p.k, nwaves * 64);
    lds_barrier();   // orders the LDS staging only: the weight loads stay in flight

    if constexpr (RES) {
        float* const resid = p.resid;
        matvec_rows<TYPE, RPW>(p.w, p.row_bytes, A, p.nrows, r0, group_stride, nslots, lane, w, [&](int r, float t) {
            p.out[r] = t;
            resid[r] += resid_weight(p.alpha, p.resid_gate) * t;
        });
    } else {
        matvec_rows<TYPE, RPW>(p.w, p.row_bytes, A, p.nrows, r0, group_stride, nslots, lane, w,
                               [&](int r, float t) { p.out[r] = t; });
    }
}

// XP = 1: a vector of at most one float4 group a thread; 4: longer ones (the host picks the
// entry point; one body compiled for both behind a branch ran the short-vector case 10 % slower).
template <int TYPE, int RPW, int XP = 1, bool RES = false, bool PQ = false>
__device__ __forceinline__ void matvec_body(const MatVecArgs& p, uint8_t* smem) {
    matvec_body_xp<TYPE, RPW, XP, RES, PQ>(p, smem);
}

// Several matvecs of one type in one launch: grid = (row groups, matrices).  Each
// workgroup stages its matrix's activation (shared, or its own at xstride; optionally
// silu(x) * x2 formed on the way into the quantizer) and then is the single-matrix
// kernel with one row per wavefront.  The reference runs such sets as one pool region:
// q/k/v or gate/up of a block (MatVecPackedGroup, engine/nn/packedgroup.go:13-51), a
// mixture's experts at decode (MatVecPackedMulti / MatVecPackedGatherAct,
// engine/nn/packedmulti.go:24,84,93); on this machine the saving is the per-launch cost.
// Sum over the 64 lanes in f64, butterfly order (every lane gets the sum).
__device__ __forceinline__ double wave_sum_f64(double v) {
#pragma unroll
    for (int m = 1; m < 64; m <<= 1) v += __shfl_xor(v, m, 64);
    return v;
}

// XP = 0: the activation comes quantized (MatVecMultiArgs.q / as / s16, one for all matrices):
// a long gated activation is formed and quantized once by the quantizer kernel instead of by
// every workgroup (silu and its division for 14336 elements in each of 256 workgroups cost the
// down projection of a feed-forward block 6 of its 20 us).
// RES: matrix 0's rows are added into the residual as they are made (entry points of their own,
// like the single-matrix kernel's).
template <int TYPE, int XP, bool RES>
__device__ __forceinline__ void matvec_multi_body_xp(const MatVecMultiArgs& p, uint8_t* smem, int row_bytes) {
    typedef SlotTraits<TYPE> T;
    const int y = blockIdx.y;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = p.nwaves;
    const int nthreads = nwaves * 64;
    const int nrows = p.nrows[y];
    const int nslots = p.k / T::kElems;
    const int group_stride = p.ngroups * nwaves;
    const ActLds A = act_lds_views(smem, p.k);
    int r0 = blockIdx.x * nwaves + wave;
    if ((int)blockIdx.x * nwaves >= nrows) return;   // uniform: this matrix has fewer row groups
    const uint8_t* w0 = p.w[y];
    if constexpr (XP == 0) {
        typename T::W w[1];
        T::load_w(w0 + (size_t)min(r0, nrows - 1) * row_bytes, min(lane, nslots - 1), w[0]);
        stage_act_copy<stage_layout_of(TYPE)>(smem, p.q, p.as, p.s16, p.k, nthreads);
        lds_barrier();
        float* const outp = p.out[y];
        if constexpr (RES) {
            float* const resid = y == 0 ? p.resid : nullptr;
            matvec_rows<TYPE, 1>(w0, row_bytes, A, nrows, r0, group_stride, nslots, lane, w, [&](int r, float t) {
                outp[r] = t;
                if (resid) resid[r] += resid_weight(p.alpha, p.resid_gate) * t;
            });
        } else {
            matvec_rows<TYPE, 1>(w0, row_bytes, A, nrows, r0, group_stride, nslots, lane, w,
                                 [&](int r, float t) { outp[r] = t; });
        }
        return;
    } else {
    const float* x = p.x + (size_t)y * p.xstride;
    const float* x2 = p.x2 ? p.x2 + (size_t)y * p.xstride : nullptr;

    const int n4 = p.k / 4, n4_pad = (n4 + 63) & ~63;
    f32x4 x0[XP], u0[XP];
    load_x_groups<XP>(x, p.k, nthreads, x0);
    if (x2) load_x_groups<XP>(x2, p.k, nthreads, u0);
    else {
#pragma unroll
        for (int i = 0; i < XP; i++) u0[i] = f32x4{1.f, 1.f, 1.f, 1.f};
    }
    f32x4 nw0[XP];   // the norm weights of the same groups
#pragma unroll
    for (int i = 0; i < XP; i++) nw0[i] = f32x4{1.f, 1.f, 1.f, 1.f};
    if (p.norm_w) load_x_groups<XP>(p.norm_w, p.k, nthreads, nw0);
    __builtin_amdgcn_s_barrier();   // activation loads of the whole workgroup go out first
    typename T::W w[1];
    T::load_w(w0 + (size_t)min(r0, nrows - 1) * row_bytes, min(lane, nslots - 1), w[0]);
    // RMSNorm ahead of the quantizer (the reference's RMSNormQuantRows, jit/gpu/kernels/
    // elem.go:252-267, with its host arithmetic, internal/oracle/oracle.go:230-240): the sum
    // of squares in f64, scale = 1/sqrt(sum/k + eps), y = f32(f64(x) * scale * f64(w)).
    // Every workgroup forms the sum itself: k floats are cheaper than a launch.
    double nscale = 0.0;
    if (p.norm_w) {
        double ss = 0.0;
        int g4 = threadIdx.x;
#pragma unroll
        for (int i = 0; i < XP; i++, g4 += nthreads) {
            const f32x4 v = x0[i];
            if (g4 < n4) ss += (double)v.x * v.x + (double)v.y * v.y + (double)v.z * v.z + (double)v.w * v.w;
        }
        for (; g4 < n4; g4 += nthreads) {
            const f32x4 v = ((const f32x4*)x)[g4];
            ss += (double)v.x * v.x + (double)v.y * v.y + (double)v.z * v.z + (double)v.w * v.w;
        }
        ss = wave_sum_f64(ss);
        // nwaves partial sums and the scale, behind the staging area (JL_NORM_LDS_BYTES more of
        // dynamic LDS).  One wavefront turns the sum into the scale: the f64 division and square
        // root are a hundred dependent instructions, and sixteen wavefronts taking them side by
        // side on four SIMDs made the launch 1.3 us longer than one taking them for all.
        double* red = (double*)(smem + (((TYPE == JL_Q8_0P ? JL_ACT_LDS_BYTES_SHIFTED(p.k) : JL_ACT_LDS_BYTES(p.k)) + 15) & ~15));
        if (lane == 0) red[wave] = ss;
        lds_barrier();                 // (orders LDS only: the first weight loads stay in flight)
        if (wave == 0) {
            double tot = 0.0;
            for (int i = 0; i < nwaves; i++) tot += red[i];
            if (lane == 0) red[nwaves] = 1.0 / __builtin_sqrt(tot / (double)p.k + (double)p.norm_eps);
        }
        lds_barrier();
        nscale = red[nwaves];
    }
    auto stage_group = [&](int g4, f32x4 v, f32x4 u, f32x4 nw) __attribute__((always_inline)) {
        if (p.norm_w) {
            v = f32x4{(float)((double)v.x * nscale * (double)nw.x), (float)((double)v.y * nscale * (double)nw.y),
                      (float)((double)v.z * nscale * (double)nw.z), (float)((double)v.w * nscale * (double)nw.w)};
            if (p.norm_out && blockIdx.x == 0 && y == 0 && g4 < n4) ((f32x4*)p.norm_out)[g4] = v;
        }
        if (x2) v = f32x4{silu_f32(v.x) * u.x, silu_f32(v.y) * u.y, silu_f32(v.z) * u.z, silu_f32(v.w) * u.w};
        stage_quantize4<stage_layout_of(TYPE)>(smem, p.k, p.per, g4, v);
    };
    {
        int g4 = threadIdx.x;
#pragma unroll
        for (int i = 0; i < XP; i++, g4 += nthreads)
            if (g4 < n4_pad) stage_group(g4, x0[i], u0[i], nw0[i]);
        for (; g4 < n4_pad; g4 += nthreads)
            stage_group(g4, ((const f32x4*)x)[min(g4, n4 - 1)],
                        x2 ? ((const f32x4*)x2)[min(g4, n4 - 1)] : f32x4{1.f, 1.f, 1.f, 1.f},
                        p.norm_w ? ((const f32x4*)p.norm_w)[min(g4, n4 - 1)] : f32x4{1.f, 1.f, 1.f, 1.f});
    }
    lds_barrier();

    float* const outp = p.out[y];
    // (a second step of weights requested ahead of the staging, for the launches with an RMSNorm or
    // a gated activation in front, measured slower: gate + up 26.2 -> 32.8 us, down 14.5 -> 16.9)
    if constexpr (RES) {
        float* const resid = y == 0 ? p.resid : nullptr;
        matvec_rows<TYPE, 1>(w0, row_bytes, A, nrows, r0, group_stride, nslots, lane, w, [&](int r, float t) {
            outp[r] = t;
            if (resid) resid[r] += resid_weight(p.alpha, p.resid_gate) * t;
        });
    } else {
        matvec_rows<TYPE, 1>(w0, row_bytes, A, nrows, r0, group_stride, nslots, lane, w,
                             [&](int r, float t) { outp[r] = t; });
    }
    }
}

template <int TYPE, int XP = 1, bool RES = true>
__device__ __forceinline__ void matvec_multi_body(const MatVecMultiArgs& p, uint8_t* smem, int row_bytes) {
    matvec_multi_body_xp<TYPE, XP, RES>(p, smem, row_bytes);
}
