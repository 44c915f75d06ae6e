// The reference's device weight layout ("packed planes") and the decode matvec
// over it.
//
// Layout (jit/gpu/kernels/pack.go:52-386, matvec.go:137-166, scstream.go:8-42):
// three planes of u32 words, each [unit][row] with the row index fastest, so the
// word a row needs for one unit sits beside the same word of the next row:
//   QS  per sub-block `pw` primary words (4-bit: byte b of word w = element 4w+b
//       in the low nibble and element 4w+b+sub/2 in the high nibble; 8-bit: raw
//       bytes), then `hw` secondary words (Q6_K: byte j holds the top two bits of
//       elements j, 4+j, 8+j, 12+j at bits 0,2,4,6);
//   D   one word per (super-block, row) = d | dmin<<16 for the k-quants; Q8_0
//       keeps two rows' f16 in one word (index super*ceil(rows/2) + row/2);
//   SC  Q4_K: three words per (super-block, row) holding sixteen 6-bit fields
//       sc0,m0,sc1,m1,... as one 96-bit little-endian stream; Q6_K: one byte
//       per 16-element sub-block, int8 scale + 128, four to a word.
// A matrix may be a row range of a larger buffer: `stride` is the buffer's row
// count and `row0` the first row (engine/nn/device.go:70-80).
//
// The matvec puts rows on lanes: a wavefront takes RW rows (64, 32 or 16) and one
// 256-element chunk of k at a time, the 64/RW lane groups splitting the chunk's
// sub-blocks, so every load is a run of RW consecutive words and no cross-lane
// reduction is needed for the dot products.  Each wavefront quantizes just its
// own 256 activations (a whole quantization window) into a private corner of LDS
// while its weight loads are in flight; the only workgroup barrier is the one
// before the final sum over the wavefronts' partial results.
#pragma once
#include "args.h"
#include "common.h"
#include "quantize.h"

#pragma clang fp contract(off)

// ------------------------------------------------------------------ pack
// One thread per (row, super-block); Q8_0's "super-block" is its 32-element block.
// grid = (ceil(nrows/256), k/unit), block = 256.

__device__ __forceinline__ void sc_stream_put(u32 ws[3], int field, u32 v) {
    const int bit = field * 6, w = bit >> 5, b = bit & 31;
    ws[w] |= v << b;
    if (b > 26) ws[w + 1] |= v >> (32 - b);
}

__device__ __forceinline__ void pack_q4k(const PackArgs& p, int r, int sb) {
    const int nsb = p.k / 256;
    const u32* blk = (const u32*)(p.src + ((size_t)r * nsb + sb) * 144);
    const size_t n = (size_t)p.nrows;
    p.d[(size_t)sb * n + r] = blk[0];
    const u32 s0 = blk[1], s1 = blk[2], s2 = blk[3];
    u32 ws[3] = {0u, 0u, 0u};
#pragma unroll
    for (int s = 0; s < 8; s++) {
        u32 sc, m;
        scale_min_k4(s, s0, s1, s2, sc, m);
        sc_stream_put(ws, 2 * s, sc);
        sc_stream_put(ws, 2 * s + 1, m);
    }
#pragma unroll
    for (int w = 0; w < 3; w++) p.sc[((size_t)sb * 3 + w) * n + r] = ws[w];
    const u32 M = 0x0F0F0F0Fu;
#pragma unroll
    for (int g = 0; g < 4; g++) {
        u32 G[8];
#pragma unroll
        for (int j = 0; j < 8; j++) G[j] = blk[4 + g * 8 + j];
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const size_t even = ((size_t)(sb * 8 + 2 * g) * 4 + w) * n + r;
            const size_t odd = ((size_t)(sb * 8 + 2 * g + 1) * 4 + w) * n + r;
            p.qs[even] = (G[w] & M) | ((G[w + 4] & M) << 4);
            p.qs[odd] = ((G[w] >> 4) & M) | (G[w + 4] & ~M);
        }
    }
}

__device__ __forceinline__ void pack_q6k(const PackArgs& p, int r, int sb) {
    const int nsb = p.k / 256;
    const uint8_t* blk = p.src + ((size_t)r * nsb + sb) * 210;
    const size_t n = (size_t)p.nrows;
    p.d[(size_t)sb * n + r] = (u32)ld2(blk + 208);
    for (int j = 0; j < 4; j++) {
        u32 v = 0;
        for (int b = 0; b < 4; b++) v |= (u32)(uint8_t)((int)(int8_t)blk[192 + 4 * j + b] + 128) << (8 * b);
        p.sc[((size_t)sb * 4 + j) * n + r] = v;
    }
    for (int s = 0; s < 16; s++) {
        const int half = s >> 3, grp = (s & 7) >> 1, run = s & 1;
        const uint8_t* ql = blk + half * 64 + (grp & 1) * 32 + run * 16;
        const uint8_t* qh = blk + 128 + half * 32 + run * 16;
        uint8_t nib[16], top[16];
        for (int l = 0; l < 16; l++) {
            nib[l] = grp >= 2 ? (uint8_t)(ql[l] >> 4) : (uint8_t)(ql[l] & 0xF);
            top[l] = (uint8_t)((qh[l] >> (2 * grp)) & 3);
        }
        u32 w0 = 0, w1 = 0, h = 0;
        for (int j = 0; j < 4; j++) {
            w0 |= (u32)(nib[j] | (nib[j + 8] << 4)) << (8 * j);
            w1 |= (u32)(nib[4 + j] | (nib[12 + j] << 4)) << (8 * j);
            h |= (u32)(top[j] | (top[4 + j] << 2) | (top[8 + j] << 4) | (top[12 + j] << 6)) << (8 * j);
        }
        const size_t base = ((size_t)(sb * 16 + s) * 3) * n + r;
        p.qs[base] = w0;
        p.qs[base + n] = w1;
        p.qs[base + 2 * n] = h;
    }
}

__device__ __forceinline__ void pack_q8_0(const PackArgs& p, int r, int b) {
    const int nb = p.k / 32;
    const uint8_t* blk = p.src + ((size_t)r * nb + b) * 34;
    const size_t n = (size_t)p.nrows;
#pragma unroll
    for (int w = 0; w < 8; w++) p.qs[((size_t)b * 8 + w) * n + r] = ld4_a2(blk + 2 + 4 * w);
    if ((r & 1) == 0) {  // two rows share a word of the D plane
        u32 v = (u32)ld2(blk);
        if (r + 1 < p.nrows) v |= (u32)ld2(blk + (size_t)nb * 34) << 16;
        p.d[(size_t)b * ((n + 1) / 2) + (r >> 1)] = v;
    }
}

// MXFP4 (jit/gpu/kernels/pack.go:395-420, :543-575): a block's 16 code bytes are the four QS
// words as they lie (byte j = element j in the low nibble, element j+16 in the high); the D
// plane holds the E8M0 exponent minus one, a byte a row, four rows a word, so that the byte
// shifted left 23 is the f32 scale of the doubled code table.  Exponents 0, 1 and 255 have no
// such byte: a block that carries one and a code other than +-0 raises the flag.
__device__ __forceinline__ void pack_mxfp4(const PackArgs& p, int r, int b) {
    const int nb = p.k / 32;
    const size_t n = (size_t)p.nrows, step = (size_t)nb * 17;
    const uint8_t* blk = p.src + ((size_t)r * nb + b) * 17;
    const u32x4 q = ld16_a1(blk + 1);
#pragma unroll
    for (int w = 0; w < 4; w++) p.qs[((size_t)b * 4 + w) * n + r] = q[w];
    const u32 e = blk[0];
    if ((e < 2 || e == 255) && ((q[0] | q[1] | q[2] | q[3]) & 0x77777777u)) *p.flag = 1;
    if ((r & 3) == 0) {
        u32 v = (e - 1) & 0xFF;
#pragma unroll
        for (int i = 1; i < 4; i++)
            if (r + i < p.nrows) v |= (((u32)blk[i * step] - 1) & 0xFF) << (8 * i);
        p.d[(size_t)b * ((n + 3) / 4) + (r >> 2)] = v;
    }
}

__device__ __forceinline__ void pack_weights_body(const PackArgs& p) {
    const int r = blockIdx.x * 256 + threadIdx.x, u = blockIdx.y;
    if (r >= p.nrows) return;
    if (p.type == JL_Q4_K) pack_q4k(p, r, u);
    else if (p.type == JL_Q6_K) pack_q6k(p, r, u);
    else if (p.type == JL_MXFP4) pack_mxfp4(p, r, u);
    else pack_q8_0(p, r, u);
}

// The inverse for Q4_K: planes (row range row0.. of a buffer of `stride` rows) back
// to GGUF row-major super-blocks, bit for bit.  The 12 scale bytes are the sixteen
// 6-bit values in ggml's arrangement (format/quant/dequant.go:360-365).
__device__ __forceinline__ void unpack_q4k_body(const UnpackArgs& p) {
    const int rl = blockIdx.x * 256 + threadIdx.x, sb = blockIdx.y;
    if (rl >= p.nrows) return;
    const size_t n = (size_t)p.stride, r = (size_t)p.row0 + rl;
    const int nsb = p.k / 256;
    u32* blk = (u32*)(p.dst + ((size_t)rl * nsb + sb) * 144);
    blk[0] = p.d[(size_t)sb * n + r];
    u32 ws[3];
#pragma unroll
    for (int w = 0; w < 3; w++) ws[w] = p.sc[((size_t)sb * 3 + w) * n + r];
    const uint64_t lo = ws[0] | ((uint64_t)ws[1] << 32), hi = ws[1] | ((uint64_t)ws[2] << 32);
    u32 sc[8], m[8];
#pragma unroll
    for (int s = 0; s < 8; s++) {
        const int bit = 12 * s;
        const u32 f = bit < 32 ? (u32)(lo >> bit) : (u32)(hi >> (bit - 32));
        sc[s] = f & 63;
        m[s] = (f >> 6) & 63;
    }
    u32 s0 = 0, s1 = 0, s2 = 0;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        s0 |= (sc[j] | ((sc[j + 4] >> 4) << 6)) << (8 * j);
        s1 |= (m[j] | ((m[j + 4] >> 4) << 6)) << (8 * j);
        s2 |= ((sc[j + 4] & 0xF) | ((m[j + 4] & 0xF) << 4)) << (8 * j);
    }
    blk[1] = s0; blk[2] = s1; blk[3] = s2;
    const u32 M = 0x0F0F0F0Fu;
#pragma unroll
    for (int g = 0; g < 4; g++)
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const u32 e = p.qs[((size_t)(sb * 8 + 2 * g) * 4 + w) * n + r];
            const u32 o = p.qs[((size_t)(sb * 8 + 2 * g + 1) * 4 + w) * n + r];
            blk[4 + g * 8 + w] = (e & M) | ((o & M) << 4);
            blk[4 + g * 8 + 4 + w] = ((e >> 4) & M) | (o & ~M);
        }
}

// The inverse for Q6_K (pack_q6k above): one thread per (row, super-block).  Per (half, run)
// the four sub-blocks 8*half + 2*grp + run share sixteen ql bytes pairwise (grp and grp + 2:
// low and high nibbles) and sixteen qh bytes all four (two bits each); a plane word holds the
// nibbles of elements j and j + 8 (w0) or 4 + j and 12 + j (w1) in byte j, the bit-pair word
// the top bits of elements j, 4 + j, 8 + j, 12 + j.  Blocks are 210 bytes: 2-byte aligned stores.
__device__ __forceinline__ void st4_a2(uint8_t* p, u32 v) { ((u32_a2*)p)->v = v; }

__device__ __forceinline__ void unpack_q6k_body(const UnpackArgs& p) {
    const int rl = blockIdx.x * 256 + threadIdx.x, sb = blockIdx.y;
    if (rl >= p.nrows) return;
    const size_t n = (size_t)p.stride, r = (size_t)p.row0 + rl;
    const int nsb = p.k / 256;
    uint8_t* blk = p.dst + ((size_t)rl * nsb + sb) * 210;
    *(uint16_t*)(blk + 208) = (uint16_t)p.d[(size_t)sb * n + r];
#pragma unroll
    for (int j = 0; j < 4; j++)   // int8 scales are stored + 128
        st4_a2(blk + 192 + 4 * j, p.sc[((size_t)sb * 4 + j) * n + r] ^ 0x80808080u);
    const u32 M = 0x0F0F0F0Fu, T = 0x03030303u;
#pragma unroll
    for (int half = 0; half < 2; half++)
#pragma unroll
        for (int run = 0; run < 2; run++) {
            u32 N[4][4], H[4];   // [grp][four elements] nibbles in bytes; bit-pair words
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const size_t base = ((size_t)(sb * 16 + half * 8 + 2 * g + run) * 3) * n + r;
                const u32 w0 = p.qs[base], w1 = p.qs[base + n];
                H[g] = p.qs[base + 2 * n];
                N[g][0] = w0 & M; N[g][2] = (w0 >> 4) & M;
                N[g][1] = w1 & M; N[g][3] = (w1 >> 4) & M;
            }
#pragma unroll
            for (int i = 0; i < 4; i++) {
                st4_a2(blk + half * 64 + run * 16 + 4 * i, N[0][i] | (N[2][i] << 4));
                st4_a2(blk + half * 64 + 32 + run * 16 + 4 * i, N[1][i] | (N[3][i] << 4));
                u32 q = 0;
#pragma unroll
                for (int g = 0; g < 4; g++) q |= ((H[g] >> (2 * i)) & T) << (2 * g);
                st4_a2(blk + 128 + half * 32 + run * 16 + 4 * i, q);
            }
        }
}

// The inverse for Q8_0 (pack_q8_0 above): one thread per (row, block); two rows share a word
// of the D plane.
__device__ __forceinline__ void unpack_q8_0_body(const UnpackArgs& p) {
    const int rl = blockIdx.x * 256 + threadIdx.x, b = blockIdx.y;
    if (rl >= p.nrows) return;
    const size_t n = (size_t)p.stride, r = (size_t)p.row0 + rl;
    const int nb = p.k / 32;
    uint8_t* blk = p.dst + ((size_t)rl * nb + b) * 34;
    const u32 dd = p.d[(size_t)b * ((n + 1) / 2) + (r >> 1)];
    *(uint16_t*)blk = (uint16_t)(r & 1 ? dd >> 16 : dd);
#pragma unroll
    for (int w = 0; w < 8; w++) st4_a2(blk + 2 + 4 * w, p.qs[((size_t)b * 8 + w) * n + r]);
}

// The inverse for MXFP4 (pack_mxfp4 above): one thread per (row, block).
struct __attribute__((packed, aligned(1))) u32x4_st1 { u32x4 v; };
__device__ __forceinline__ void unpack_mxfp4_body(const UnpackArgs& p) {
    const int rl = blockIdx.x * 256 + threadIdx.x, b = blockIdx.y;
    if (rl >= p.nrows) return;
    const size_t n = (size_t)p.stride, r = (size_t)p.row0 + rl;
    const int nb = p.k / 32;
    uint8_t* blk = p.dst + ((size_t)rl * nb + b) * 17;
    const u32 dd = p.d[(size_t)b * ((n + 3) / 4) + (r >> 2)];
    blk[0] = (uint8_t)(((dd >> (8 * (r & 3))) & 0xFF) + 1);
    u32x4 q;
#pragma unroll
    for (int w = 0; w < 4; w++) q[w] = p.qs[((size_t)b * 4 + w) * n + r];
    ((u32x4_st1*)(blk + 1))->v = q;
}

// ---------------------------------------------------------------- matvec

// A wavefront's private LDS: 256 int8 activations, 8 scales, 16 half-block sums.
#define JL_PK_WAVE_LDS 384
// Dynamic LDS of a workgroup of `nw` wavefronts: the private areas, then the
// partial sums [nw][64], rows one word apart in banks.
#define JL_PK_RED_STRIDE 65
#define JL_PK_LDS_BYTES(nw) ((nw) * (JL_PK_WAVE_LDS + JL_PK_RED_STRIDE * 4))

struct PkAct {
    const u32x4* a;    // int8 activations of the chunk, 16 per vector
    const float* da;   // [8]
    const float* ss;   // [16]
};

// NB = 32-element blocks of the chunk one lane covers (8, 4 or 2).
template <int NB> struct PkWQ4K { u32 q[NB][4]; u32 d; u32 sc[3]; };
template <int NB> struct PkWQ8 { u32 q[NB][8]; u32 d[NB]; };
template <int NB> struct PkWQ6K { u32 q[2 * NB][3]; u32 sc[(2 * NB + 3) / 4]; u32 d; };

template <int NB>
__device__ __forceinline__ void pk_load(const PackedMatVecArgs& p, int c, int b0, int row, PkWQ4K<NB>& w) {
    const size_t st = (size_t)p.stride;
    w.d = p.d[(size_t)c * st + row];
#pragma unroll
    for (int j = 0; j < 3; j++) w.sc[j] = p.sc[((size_t)c * 3 + j) * st + row];
    const u32* qs = p.qs + (size_t)(c * 8 + b0) * 4 * st + row;
#pragma unroll
    for (int i = 0; i < NB; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) w.q[i][j] = qs[(size_t)(i * 4 + j) * st];
}

template <int NB>
__device__ __forceinline__ float pk_dot(const PackedMatVecArgs&, const PkWQ4K<NB>& w, int, int b0, int,
                                        const PkAct& A) {
    const u32 M = 0x0F0F0F0Fu;
    const float d = half_bits_to_f32((uint16_t)(w.d & 0xFFFF));
    const float dmin = half_bits_to_f32((uint16_t)(w.d >> 16));
    const uint64_t lo = w.sc[0] | ((uint64_t)w.sc[1] << 32), hi = w.sc[1] | ((uint64_t)w.sc[2] << 32);
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < NB; i++) {
        const int s = b0 + i, bit = 12 * s;
        const u32 f = bit < 32 ? (u32)(lo >> bit) : (u32)(hi >> (bit - 32));
        const u32 sc = f & 63, m = (f >> 6) & 63;
        const u32x4 a0 = A.a[2 * s], a1 = A.a[2 * s + 1];
        i32 dt = dot4(w.q[i][0] & M, a0.x, 0);
        dt = dot4(w.q[i][1] & M, a0.y, dt);
        dt = dot4(w.q[i][2] & M, a0.z, dt);
        dt = dot4(w.q[i][3] & M, a0.w, dt);
        dt = dot4((w.q[i][0] >> 4) & M, a1.x, dt);
        dt = dot4((w.q[i][1] >> 4) & M, a1.y, dt);
        dt = dot4((w.q[i][2] >> 4) & M, a1.z, dt);
        dt = dot4((w.q[i][3] >> 4) & M, a1.w, dt);
        const float sa = A.ss[2 * s] + A.ss[2 * s + 1];
        const float v = (float)dt * (d * (float)sc) - sa * (dmin * (float)m);
        acc = fmaf(v, A.da[s], acc);
    }
    return acc;
}

template <int NB>
__device__ __forceinline__ void pk_load(const PackedMatVecArgs& p, int c, int b0, int row, PkWQ8<NB>& w) {
    const size_t st = (size_t)p.stride, dst = (st + 1) / 2;
    const int nb = p.k / 32;
#pragma unroll
    for (int i = 0; i < NB; i++) {
        const int B = min(c * 8 + b0 + i, nb - 1);
        w.d[i] = p.d[(size_t)B * dst + (row >> 1)];
        const u32* qs = p.qs + (size_t)B * 8 * st + row;
#pragma unroll
        for (int j = 0; j < 8; j++) w.q[i][j] = qs[(size_t)j * st];
    }
}

template <int NB>
__device__ __forceinline__ float pk_dot(const PackedMatVecArgs& p, const PkWQ8<NB>& w, int c, int b0, int row,
                                        const PkAct& A) {
    const int nb = p.k / 32;
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < NB; i++) {
        const int s = b0 + i;
        const u32x4 a0 = A.a[2 * s], a1 = A.a[2 * s + 1];
        i32 dt = dot4(w.q[i][0], a0.x, 0);
        dt = dot4(w.q[i][1], a0.y, dt);
        dt = dot4(w.q[i][2], a0.z, dt);
        dt = dot4(w.q[i][3], a0.w, dt);
        dt = dot4(w.q[i][4], a1.x, dt);
        dt = dot4(w.q[i][5], a1.y, dt);
        dt = dot4(w.q[i][6], a1.z, dt);
        dt = dot4(w.q[i][7], a1.w, dt);
        const float d = half_bits_to_f32((uint16_t)(w.d[i] >> (16 * (row & 1))));
        const float v = (float)dt * d * A.da[s];
        if (c * 8 + s < nb) acc += v;   // a short last chunk has fewer blocks
    }
    return acc;
}

template <int NB>
__device__ __forceinline__ void pk_load(const PackedMatVecArgs& p, int c, int b0, int row, PkWQ6K<NB>& w) {
    const size_t st = (size_t)p.stride;
    const int s0 = 2 * b0;   // first 16-element sub-block of this lane's share
    w.d = p.d[(size_t)c * st + row];
#pragma unroll
    for (int j = 0; j < (2 * NB + 3) / 4; j++) w.sc[j] = p.sc[((size_t)(c * 16 + s0) / 4 + j) * st + row];
    const u32* qs = p.qs + (size_t)(c * 16 + s0) * 3 * st + row;
#pragma unroll
    for (int i = 0; i < 2 * NB; i++)
#pragma unroll
        for (int j = 0; j < 3; j++) w.q[i][j] = qs[(size_t)(i * 3 + j) * st];
}

template <int NB>
__device__ __forceinline__ float pk_dot(const PackedMatVecArgs&, const PkWQ6K<NB>& w, int, int b0, int,
                                        const PkAct& A) {
    const u32 M4 = 0x0F0F0F0Fu, M2 = 0x30303030u;
    const float d = half_bits_to_f32((uint16_t)(w.d & 0xFFFF));
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < 2 * NB; i++) {
        const int s = 2 * b0 + i;
        const u32x4 a = A.a[s];
        const u32 w0 = w.q[i][0], w1 = w.q[i][1], h = w.q[i][2];
        i32 dt = dot4((w0 & M4) | ((h << 4) & M2), a.x, 0);
        dt = dot4((w1 & M4) | ((h << 2) & M2), a.y, dt);
        dt = dot4(((w0 >> 4) & M4) | (h & M2), a.z, dt);
        dt = dot4(((w1 >> 4) & M4) | ((h >> 2) & M2), a.w, dt);
        // value = d*sc*(q-32): the zero point goes through the activation sum
        const float t = (float)dt - 32.f * A.ss[s];
        const i32 sc = (i32)((w.sc[i >> 2] >> (8 * (i & 3))) & 0xFF) - 128;
        acc = fmaf(t * (d * (float)sc), A.da[s >> 1], acc);
    }
    return acc;
}

template <int TYPE, int NB> struct PkTraits;
template <int NB> struct PkTraits<JL_Q4_K, NB> { typedef PkWQ4K<NB> W; };
template <int NB> struct PkTraits<JL_Q8_0, NB> { typedef PkWQ8<NB> W; };
template <int NB> struct PkTraits<JL_Q6_K, NB> { typedef PkWQ6K<NB> W; };

// A chunk's activation as the lane holds it between the load and the staging: four
// f32 values (fused form), or in the split form four int8 in .x, a scale in .y (lanes
// 0-7) and a half-block sum in .z (lanes 0-15).  Loads are unconditional at clamped
// addresses, so nothing between them makes the compiler wait for data; what lies past
// the end of the vector is zeroed when the chunk is staged.
// The gated form carries the gate's partner beside it.
template <bool GATED> struct PkX { f32x4 v; };
template <> struct PkX<true> { f32x4 v, u; };

template <bool FUSED, bool GATED>
__device__ __forceinline__ void pk_load_x(const PackedMatVecArgs& p, int c, int lane, PkX<GATED>& X) {
    const int g4 = min(c * 64 + lane, p.k / 4 - 1);
    if (FUSED) {
        X.v = ((const f32x4*)p.x)[g4];
        if constexpr (GATED) X.u = ((const f32x4*)p.x2)[g4];   // the gate's partner, or the norm's weights
    } else {
        X.v.x = __uint_as_float(((const u32*)p.q)[g4]);
        X.v.y = p.as[min(c * 8 + (lane & 7), p.k / 32 - 1)];
        X.v.z = p.s16[min(c * 16 + (lane & 15), p.k / 16 - 1)];
        X.v.w = 0.f;
    }
}

// Quantize (or copy) the chunk's activation into the wavefront's private LDS area.
// NORM: the second operand is the RMSNorm weight and nscale the row's 1/rms; the normed
// value is f32(f64(x) * nscale * f64(w)), the reference's host arithmetic
// (internal/oracle/oracle.go:230-240).
template <bool FUSED, bool GATED, bool NORM = false>
__device__ __forceinline__ void pk_stage_x(const PackedMatVecArgs& p, int c, int lane, const PkX<GATED>& X, uint8_t* my,
                                           double nscale = 0.0, bool write_norm = false) {
    u32* a_w = (u32*)my;
    float* da_w = (float*)(my + 256);
    float* ss_w = (float*)(my + 288);
    const bool live = c * 64 + lane < p.k / 4;
    if (FUSED) {
        f32x4 xv = live ? X.v : f32x4{0.f, 0.f, 0.f, 0.f};
        if constexpr (NORM) {
            const f32x4 nw = X.u;
            xv = f32x4{(float)((double)xv.x * nscale * (double)nw.x), (float)((double)xv.y * nscale * (double)nw.y),
                       (float)((double)xv.z * nscale * (double)nw.z), (float)((double)xv.w * nscale * (double)nw.w)};
            if (write_norm && live) ((f32x4*)p.norm_out)[c * 64 + lane] = xv;
        } else if constexpr (GATED) {
            const f32x4 u = live ? X.u : f32x4{0.f, 0.f, 0.f, 0.f};
            xv = f32x4{silu_f32(xv.x) * u.x, silu_f32(xv.y) * u.y, silu_f32(xv.z) * u.z, silu_f32(xv.w) * u.w};
        }
        u32 m = max(max(abs_bits(xv.x), abs_bits(xv.y)), max(abs_bits(xv.z), abs_bits(xv.w)));
        const u32 amax = p.per == 8 ? wave_amax_256(m) : window_amax(m, p.per);
        float d;
        i32 sum;
        const u32 qv = quantize4(xv, amax, d, sum);
        a_w[lane] = qv;
        if ((lane & 3) == 0) ss_w[lane >> 2] = (float)sum;
        if ((lane & 7) == 0) da_w[lane >> 3] = d;
    } else {
        a_w[lane] = live ? __float_as_uint(X.v.x) : 0u;
        if (lane < 8) da_w[lane] = X.v.y;
        if (lane < 16) ss_w[lane] = X.v.z;
    }
    // The area is private to this wavefront, whose LDS operations complete in
    // order: only the compiler has to be kept from moving reads above the writes.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// grid = ceil(nrows / RW) workgroups of 64..1024 threads; dynamic LDS =
// JL_PK_LDS_BYTES(wavefronts).  Needs k % 32 == 0 (k % 256 == 0 for the k-quants).
//
// Order of the memory requests: a CU's vector loads are served in the order they were
// issued, whichever wavefront issued them, so an activation load that goes out after
// another wavefront's weight loads comes back behind them.  Every wavefront therefore
// issues the activation loads of its first XPRE chunks (as many as registers allow),
// the workgroup meets at a barrier that waits for no data, and only then do the weight
// loads go out: the small activation comes back first and is quantized while the
// weights stream in.
//
// The partial sums [wavefront][lane] are added up by RW*16 threads at once: thread
// (row r, j) takes wavefront j's KP partials of row r, and the sixteen j of a row sit
// in one 16-lane DPP row, so the sum over wavefronts is four lane-exchange adds.
//
// NORM (an RMSNorm in front of the quantizer, the reference's RMSNormQuantRows,
// jit/gpu/kernels/elem.go:252-267): every workgroup forms the row's sum of squares itself,
// in f64, before anything else; k floats from L2 are cheaper than a launch.  The norm's
// weights ride in the gate partner's registers (p.x2), so NORM implies the two-operand load.
// (The first chunk's weights requested before the reduction instead of after it measured slower
// both ways it was tried, us for the gated block over planes: 44.7 -> 54.4 with __syncthreads() in
// the reduction, whose fence waits for every load in flight; 45.0 -> 46.7 with barriers that order
// LDS only: the activation's quantization then no longer runs under the weights' way from memory.)
template <int TYPE, int RW, int XPRE, bool FUSED, bool GATED = false, bool NORM = false>
__device__ __forceinline__ void packed_matvec_body(const PackedMatVecArgs& p, uint8_t* smem) {
    static_assert(!NORM || (FUSED && GATED), "the norm's weights ride in the second operand");
    constexpr int KP = 64 / RW, NB = 8 / KP;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = p.nwaves;
    // Workgroups are dealt to the eight XCDs round robin; give each XCD a contiguous
    // range of row groups so neighbouring row runs meet in one L2.
    int g = blockIdx.x;
    const int ng = p.ngroups;
    if ((ng & 7) == 0) g = (g & 7) * (ng >> 3) + (g >> 3);
    const int rl = lane % RW, part = lane / RW, b0 = part * NB;
    const int row = p.row0 + min(g * RW + rl, p.nrows - 1);

    uint8_t* my = smem + wave * JL_PK_WAVE_LDS;
    PkAct A;
    A.a = (const u32x4*)my;
    A.da = (const float*)(my + 256);
    A.ss = (const float*)(my + 288);

    const int nchunks = (p.k + 255) / 256;
    PkX<GATED> X[XPRE];
#pragma unroll
    for (int i = 0; i < XPRE; i++) pk_load_x<FUSED, GATED>(p, wave + i * nwaves, lane, X[i]);
    double nscale = 0.0;
    bool write_norm = false;
    if constexpr (NORM) {
        const int n4 = p.k / 4, nthreads = nwaves * 64;
        double ss = 0.0;
        auto sq = [&](const f32x4& v) {
            ss += (double)v.x * v.x + (double)v.y * v.y + (double)v.z * v.z + (double)v.w * v.w;
        };
        // chunk wave + i * nwaves of lane `lane` is element threadIdx.x + i * nthreads
#pragma unroll
        for (int i = 0; i < XPRE; i++)
            if ((int)threadIdx.x + i * nthreads < n4) sq(X[i].v);
        for (int g4 = threadIdx.x + XPRE * nthreads; g4 < n4; g4 += nthreads) sq(((const f32x4*)p.x)[g4]);
        ss = wave_sum_f64(ss);
        double* nred = (double*)(smem + nwaves * JL_PK_WAVE_LDS);   // the partial-sum area, not in use yet
        if (lane == 0) nred[wave] = ss;
        __syncthreads();
        double tot = 0.0;
        for (int i = 0; i < nwaves; i++) tot += nred[i];
        __syncthreads();                                            // all have read before the area is reused
        nscale = 1.0 / __builtin_sqrt(tot / (double)p.k + (double)p.norm_eps);
        write_norm = p.norm_out != nullptr && blockIdx.x == 0;
    } else {
        __builtin_amdgcn_s_barrier();
    }

    float acc = 0.f;
    auto chunk = [&](int c, const PkX<GATED>& Xc) {
        typename PkTraits<TYPE, NB>::W w;
        pk_load<NB>(p, c, b0, row, w);
        pk_stage_x<FUSED, GATED, NORM>(p, c, lane, Xc, my, nscale, write_norm);
        acc += pk_dot<NB>(p, w, c, b0, row, A);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    };
#pragma unroll
    for (int i = 0; i < XPRE; i++) {
        const int c = wave + i * nwaves;
        if (c < nchunks) chunk(c, X[i]);
    }
    for (int c = wave + XPRE * nwaves; c < nchunks; c += nwaves) {
        PkX<GATED> Xc;
        pk_load_x<FUSED, GATED>(p, c, lane, Xc);
        chunk(c, Xc);
    }

    float* red = (float*)(smem + nwaves * JL_PK_WAVE_LDS);
    red[wave * JL_PK_RED_STRIDE + lane] = acc;
    __syncthreads();
    const int j = threadIdx.x & 15;
    for (int r = threadIdx.x >> 4; r < RW; r += nwaves * 4) {
        float t = 0.f;
        if (j < nwaves) {
#pragma unroll
            for (int q = 0; q < KP; q++) t += red[j * JL_PK_RED_STRIDE + q * RW + r];
        }
        t += dpp_f32<JL_DPP_QUAD_XOR1, 0xf>(t);
        t += dpp_f32<JL_DPP_QUAD_XOR2, 0xf>(t);
        t += dpp_f32<JL_DPP_ROW_HALF_MIRROR, 0xf>(t);
        t += dpp_f32<JL_DPP_ROW_MIRROR, 0xf>(t);
        if (j == 0 && g * RW + r < p.nrows) {
            p.out[g * RW + r] = t;
            if (p.resid) p.resid[g * RW + r] += p.alpha * t;
        }
    }
}

// Matrix blockIdx.y of a multi launch as a single packed matvec.
template <int TYPE, int RW, int XPRE, bool GATED, bool NORM = false>
__device__ __forceinline__ void packed_matvec_multi_body(const PackedMultiArgs& m, uint8_t* smem) {
    const int y = blockIdx.y;
    PackedMatVecArgs p;
    p.out = m.out[y]; p.qs = m.qs[y]; p.d = m.d[y]; p.sc = m.sc[y];
    p.x = m.x + (size_t)y * m.xstride;
    p.x2 = NORM ? m.norm_w : GATED ? m.x2 + (size_t)y * m.xstride : nullptr;
    p.norm_out = NORM && y == 0 ? m.norm_out : nullptr; p.norm_eps = m.norm_eps;
    p.q = nullptr; p.as = nullptr; p.s16 = nullptr;
    p.nrows = m.nrows; p.k = m.k; p.row0 = m.row0[y]; p.stride = m.stride;
    p.per = m.per; p.nwaves = m.nwaves; p.ngroups = m.ngroups;
    p.resid = y == 0 ? m.resid : nullptr;
    p.alpha = y == 0 && m.resid ? resid_weight(m.alpha, m.resid_gate) : 0.f;
    packed_matvec_body<TYPE, RW, XPRE, true, GATED, NORM>(p, smem);
}
