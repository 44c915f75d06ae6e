/*
 * jl_oracle.c -- TEST INFRASTRUCTURE ONLY (see jl_oracle.h).
 *
 * Plain-C restatement of the reference arithmetic of jitllm's quantized-weight
 * matmul path.  Scalar, no SIMD, no cleverness; each function names the
 * reference lines it follows.  Compile with -ffp-contract=off so that no
 * product is fused into an FMA the reference does not have.
 */
#include "jl_oracle.h"
#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ types */

/* format/quant/types.go:61-85 */
int jlo_block_elems(int type) {
    switch (type) {
    case JLO_Q8_0: return 32;
    case JLO_Q4_K: return 256;
    case JLO_Q5_K: return 256;
    case JLO_Q6_K: return 256;
    case JLO_MXFP4: return 32;
    }
    return 0;
}
int jlo_block_bytes(int type) {
    switch (type) {
    case JLO_Q8_0: return 34;
    case JLO_Q4_K: return 144;
    case JLO_Q5_K: return 176;
    case JLO_Q6_K: return 210;
    case JLO_MXFP4: return 17;
    }
    return 0;
}

static uint16_t rd16(const uint8_t *p) { return (uint16_t)(p[0] | (p[1] << 8)); }
static float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

/* ------------------------------------------------------------- half codec */

/* format/quant/dequant.go:15-32.  Every binary16 is exact in f32. */
float jlo_half_to_f32(uint16_t u) {
    double sign = (u & 0x8000) ? -1.0 : 1.0;
    int e = (u >> 10) & 0x1f, mant = u & 0x3ff;
    if (e == 0) return (float)(sign * (double)mant * ldexp(1.0, -24));
    if (e == 0x1f) return mant ? NAN : (float)(sign * INFINITY);
    return (float)(sign * (double)(1024 + mant) * ldexp(1.0, e - 25));
}

/* format/quant/dequant.go:478-517 (EncodeHalf), round to nearest even. */
uint16_t jlo_f32_to_half(float f) {
    uint32_t b = f32_bits(f);
    uint16_t sign = (uint16_t)((b >> 16) & 0x8000);
    int32_t e8 = (int32_t)((b >> 23) & 0xFF);
    uint32_t man = b & 0x7FFFFF;
    if (e8 == 0xFF) return (uint16_t)(sign | (man ? 0x7E00 : 0x7C00));
    int32_t e = e8 - 127 + 15;
    if (e >= 0x1F) return (uint16_t)(sign | 0x7C00);
    if (e <= 0) {
        if (e < -10) return sign;
        man |= 0x800000;
        uint32_t shift = (uint32_t)(14 - e);
        uint32_t h = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1);
        uint32_t half = 1u << (shift - 1);
        if (rem > half || (rem == half && (h & 1))) h++;
        return (uint16_t)(sign | h);
    }
    uint16_t h = (uint16_t)((e << 10) | (man >> 13));
    uint32_t rem = man & 0x1FFF;
    if (rem > 0x1000 || (rem == 0x1000 && (h & 1))) h++;
    return (uint16_t)(sign | h);
}

/* ---------------------------------------------------------------- dequant */

/* format/quant/dequant.go:360-365 */
static void scale_min_k4(int j, const uint8_t *q, uint8_t *sc, uint8_t *m) {
    if (j < 4) {
        *sc = q[j] & 63;
        *m = q[j + 4] & 63;
    } else {
        *sc = (uint8_t)((q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4));
        *m = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    }
}

/* format/quant/dequant.go:268 */
static const int8_t mxfp4_values[16] = {0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12};

/* format/quant/dequant.go:148-157 */
static void dequant_q8_0(const uint8_t *src, float *dst, size_t blocks) {
    for (size_t b = 0; b < blocks; b++) {
        const uint8_t *blk = src + b * 34;
        double d = jlo_half_to_f32(rd16(blk));
        for (int j = 0; j < 32; j++) dst[b * 32 + j] = (float)((double)(int8_t)blk[2 + j] * d);
    }
}

/* format/quant/dequant.go:159-174 */
static void dequant_mxfp4(const uint8_t *src, float *dst, size_t blocks) {
    for (size_t b = 0; b < blocks; b++) {
        const uint8_t *blk = src + b * 17;
        double d = ldexp(1.0, (int)blk[0] - 128);
        for (int j = 0; j < 16; j++) {
            dst[b * 32 + j] = (float)((double)mxfp4_values[blk[1 + j] & 0xF] * d);
            dst[b * 32 + j + 16] = (float)((double)mxfp4_values[blk[1 + j] >> 4] * d);
        }
    }
}

/* format/quant/dequant.go:367-397.  The products d*sc and dmin*m are rounded
 * to f32, then d1*q is rounded to f32, then the subtraction. */
static void dequant_q4_k(const uint8_t *src, float *dst, size_t blocks) {
    for (size_t b = 0; b < blocks; b++) {
        const uint8_t *blk = src + b * 144;
        float d = jlo_half_to_f32(rd16(blk));
        float dmin = jlo_half_to_f32(rd16(blk + 2));
        const uint8_t *scales = blk + 4, *qs = blk + 16;
        float *out = dst + b * 256;
        int o = 0, is = 0;
        for (int j = 0; j < 256; j += 64) {
            const uint8_t *q = qs + j / 2;
            uint8_t sc1, m1, sc2, m2;
            scale_min_k4(is, scales, &sc1, &m1);
            scale_min_k4(is + 1, scales, &sc2, &m2);
            volatile float d1 = d * (float)sc1, min1 = dmin * (float)m1;
            volatile float d2 = d * (float)sc2, min2 = dmin * (float)m2;
            for (int l = 0; l < 32; l++) {
                volatile float p = d1 * (float)(q[l] & 0xF);
                out[o++] = p - min1;
            }
            for (int l = 0; l < 32; l++) {
                volatile float p = d2 * (float)(q[l] >> 4);
                out[o++] = p - min2;
            }
            is += 2;
        }
    }
}

/* format/quant/dequant.go:399-441.  Q4_K's scales; the fifth bit of element l of 64-group g
 * is bit 2g (first half) / 2g+1 (second half) of qh[l]: the same 32 bytes serve all four
 * groups.  Not a type of the matmul path: it is here because it is the one format with a
 * secondary (high-bit) plane whose packed bytes the reference wrote into a fixture. */
static void dequant_q5_k(const uint8_t *src, float *dst, size_t blocks) {
    for (size_t b = 0; b < blocks; b++) {
        const uint8_t *blk = src + b * 176;
        float d = jlo_half_to_f32(rd16(blk));
        float dmin = jlo_half_to_f32(rd16(blk + 2));
        const uint8_t *scales = blk + 4, *qh = blk + 16, *qs = blk + 48;
        float *out = dst + b * 256;
        int o = 0, is = 0;
        uint8_t u1 = 1, u2 = 2;
        for (int j = 0; j < 256; j += 64) {
            const uint8_t *ql = qs + j / 2;
            uint8_t sc1, m1, sc2, m2;
            scale_min_k4(is, scales, &sc1, &m1);
            scale_min_k4(is + 1, scales, &sc2, &m2);
            volatile float d1 = d * (float)sc1, min1 = dmin * (float)m1;
            volatile float d2 = d * (float)sc2, min2 = dmin * (float)m2;
            for (int l = 0; l < 32; l++) {
                int32_t v = (ql[l] & 0xF) + ((qh[l] & u1) ? 16 : 0);
                volatile float p = d1 * (float)v;
                out[o++] = p - min1;
            }
            for (int l = 0; l < 32; l++) {
                int32_t v = (ql[l] >> 4) + ((qh[l] & u2) ? 16 : 0);
                volatile float p = d2 * (float)v;
                out[o++] = p - min2;
            }
            is += 2;
            u1 = (uint8_t)(u1 << 2);
            u2 = (uint8_t)(u2 << 2);
        }
    }
}

/* format/quant/dequant.go:443-470.  (d*sc)*q, left to right in f32. */
static void dequant_q6_k(const uint8_t *src, float *dst, size_t blocks) {
    for (size_t b = 0; b < blocks; b++) {
        const uint8_t *blk = src + b * 210;
        float d = jlo_half_to_f32(rd16(blk + 208));
        float *out = dst + b * 256;
        for (int n = 0; n < 256; n += 128) {
            const uint8_t *ql = blk + n / 2, *qh = blk + 128 + n / 4;
            const int8_t *sc = (const int8_t *)(blk + 192 + n / 16);
            float *y = out + n;
            for (int l = 0; l < 32; l++) {
                int is = l / 16;
                int32_t q1 = (int32_t)(int8_t)((ql[l] & 0xF) | (((qh[l] >> 0) & 3) << 4)) - 32;
                int32_t q2 = (int32_t)(int8_t)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32;
                int32_t q3 = (int32_t)(int8_t)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
                int32_t q4 = (int32_t)(int8_t)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
                volatile float s1 = d * (float)sc[is + 0], s2 = d * (float)sc[is + 2];
                volatile float s3 = d * (float)sc[is + 4], s4 = d * (float)sc[is + 6];
                y[l + 0] = s1 * (float)q1;
                y[l + 32] = s2 * (float)q2;
                y[l + 64] = s3 * (float)q3;
                y[l + 96] = s4 * (float)q4;
            }
        }
    }
}

/* format/quant/dequant.go:50-69 */
int jlo_dequant(int type, const uint8_t *src, float *dst, size_t n) {
    int be = jlo_block_elems(type);
    if (be == 0 || n % (size_t)be != 0) return -1;
    size_t blocks = n / (size_t)be;
    switch (type) {
    case JLO_Q8_0: dequant_q8_0(src, dst, blocks); return 0;
    case JLO_Q4_K: dequant_q4_k(src, dst, blocks); return 0;
    case JLO_Q5_K: dequant_q5_k(src, dst, blocks); return 0;
    case JLO_Q6_K: dequant_q6_k(src, dst, blocks); return 0;
    case JLO_MXFP4: dequant_mxfp4(src, dst, blocks); return 0;
    }
    return -1;
}

/* ------------------------------------------------------- packed layout */

/* jit/gpu/kernels/matvec.go:137-166 (qtab), the rows this path uses. */
typedef struct {
    int bits, hi, sub, block_b, block_e, per_super, sc_off;
    float bias_k;
    int bias_array, signed_q, e8m0, codes;
} qinfo;

static int qinfo_of(int type, qinfo *qi) {
    memset(qi, 0, sizeof *qi);
    switch (type) {
    case JLO_Q8_0:
        qi->bits = 8; qi->sub = 32; qi->block_b = 34; qi->block_e = 32; qi->per_super = 1;
        qi->signed_q = 1; return 0;
    case JLO_Q4_K:
        qi->bits = 4; qi->sub = 32; qi->bias_array = 1; qi->block_b = 144; qi->block_e = 256;
        qi->per_super = 8; return 0;
    case JLO_Q5_K:   /* a 4-bit primary plane plus a one-bit secondary plane, the two-plane form Q6_K uses */
        qi->bits = 4; qi->hi = 1; qi->sub = 32; qi->bias_array = 1; qi->block_b = 176; qi->block_e = 256;
        qi->per_super = 8; return 0;
    case JLO_Q6_K:
        qi->bits = 4; qi->hi = 2; qi->sub = 16; qi->bias_k = 32; qi->block_b = 210;
        qi->block_e = 256; qi->per_super = 16; qi->sc_off = -128; return 0;
    case JLO_MXFP4:
        qi->bits = 4; qi->sub = 32; qi->bias_k = 12; qi->block_b = 17; qi->block_e = 32;
        qi->per_super = 1; qi->e8m0 = 1; qi->codes = 1; return 0;
    }
    return -1;
}

/* jit/gpu/kernels/scstream.go:24 */
static int sc_stream(const qinfo *qi) { return qi->bias_array && qi->per_super == 8; }

/* jit/gpu/kernels/pack.go:543-556 */
static int d_slots(const qinfo *qi) {
    if (qi->e8m0) return 4;
    if (qi->bias_array) return 1;
    if (qi->per_super == 1) return 2;
    return 1;
}

/* jit/gpu/kernels/pack.go:570-575 */
static void d_index(const qinfo *qi, int super, int nrows, int r, size_t *idx, int *slot) {
    int n = d_slots(qi);
    if (n > 1) {
        *idx = (size_t)super * (size_t)((nrows + n - 1) / n) + (size_t)(r / n);
        *slot = r % n;
    } else {
        *idx = (size_t)super * (size_t)nrows + (size_t)r;
        *slot = 0;
    }
}

/* jit/gpu/kernels/scstream.go:32-42 */
static void sc_field(int sub, int min, int *w, int *b, int *hi) {
    int f = 2 * sub + (min ? 1 : 0);
    *w = f * 6 / 32;
    *b = f * 6 % 32;
    *hi = *b > 26 ? *b - 26 : 0;
}
/* jit/gpu/kernels/scstream.go:46-52 */
static uint8_t sc_value(const uint32_t ws[3], int sub, int min) {
    int w, b, hi;
    sc_field(sub, min, &w, &b, &hi);
    if (hi == 0) return (uint8_t)((ws[w] << (26 - b)) >> 26);
    return (uint8_t)((ws[w] >> b) | ((ws[w + 1] << (32 - hi)) >> 26));
}
/* jit/gpu/kernels/scstream.go:55-61 */
static void sc_put(uint32_t ws[3], int sub, int min, uint8_t v) {
    int w, b, hi;
    sc_field(sub, min, &w, &b, &hi);
    ws[w] |= (uint32_t)(v & 63) << b;
    if (hi > 0) ws[w + 1] |= (uint32_t)(v & 63) >> (6 - hi);
}

/* jit/gpu/kernels/pack.go:580-621 */
int jlo_packed_words(int type, int nrows, int k, size_t *nq, size_t *nd, size_t *nsc) {
    qinfo qi;
    if (qinfo_of(type, &qi) < 0) return -1;
    int unit = qi.sub * qi.per_super;
    if (k <= 0 || nrows <= 0 || k % unit != 0) return -1;
    size_t nsub = (size_t)(k / qi.sub);
    *nq = (size_t)nrows * nsub * (size_t)(qi.sub * (qi.bits + qi.hi) / 32);
    size_t nsuper = nsub / (size_t)qi.per_super;
    int n = d_slots(&qi);
    *nd = n > 1 ? nsuper * (size_t)((nrows + n - 1) / n) : nsuper * (size_t)nrows;
    *nsc = 0;
    if (sc_stream(&qi)) *nsc = (size_t)nrows * nsuper * 3;
    else if (qi.per_super > 1) {
        size_t per = qi.bias_array ? 2 : 4;
        *nsc = (size_t)nrows * ((nsub + per - 1) / per);
    }
    return 0;
}

/* jit/gpu/kernels/pack.go:252-386 (extract), the four formats on this path.
 * Returns the raw d / dmin bits and the integer scale / min of sub-block s. */
static void extract(int type, const uint8_t *blk, int s, int32_t *q, uint16_t *dbits,
                    uint16_t *dminbits, uint8_t *sc, uint8_t *m) {
    *dbits = 0; *dminbits = 0; *sc = 0; *m = 0;
    switch (type) {
    case JLO_Q8_0:
        for (int l = 0; l < 32; l++) q[l] = (int8_t)blk[2 + l];
        *dbits = rd16(blk);
        return;
    case JLO_MXFP4:
        for (int l = 0; l < 16; l++) {
            q[l] = blk[1 + l] & 0xF;
            q[l + 16] = blk[1 + l] >> 4;
        }
        *dbits = (uint16_t)(uint8_t)(blk[0] - 1); /* e8m0Store, pack.go:395 */
        return;
    case JLO_Q4_K: {
        scale_min_k4(s, blk + 4, sc, m);
        const uint8_t *grp = blk + 16 + (s / 2) * 32;
        for (int l = 0; l < 32; l++) q[l] = (s % 2 == 0) ? (grp[l] & 0xF) : (grp[l] >> 4);
        *dbits = rd16(blk);
        *dminbits = rd16(blk + 2);
        return;
    }
    case JLO_Q5_K: {   /* pack.go:332-349 */
        scale_min_k4(s, blk + 4, sc, m);
        const uint8_t *qh = blk + 16, *ql = blk + 48 + (s / 2) * 32;
        for (int l = 0; l < 32; l++) {
            int32_t v = (s % 2 == 1) ? (ql[l] >> 4) : (ql[l] & 0xF);
            if (qh[l] & (1u << s)) v += 16;
            q[l] = v;
        }
        *dbits = rd16(blk);
        *dminbits = rd16(blk + 2);
        return;
    }
    case JLO_Q6_K: {
        *sc = (uint8_t)((int)(int8_t)blk[192 + s] + 128);
        int g = s / 8, e0 = (s % 8) * 16;
        const uint8_t *ql = blk + g * 64, *qh = blk + 128 + g * 32;
        for (int l = 0; l < 16; l++) {
            int e = e0 + l;
            int lo = e % 32, sh = 2 * (e / 32);
            uint8_t nib = ql[lo + (e / 32) % 2 * 32];
            nib = (e / 32 >= 2) ? (uint8_t)(nib >> 4) : (uint8_t)(nib & 0xF);
            q[l] = (int32_t)nib | (int32_t)(((qh[lo] >> sh) & 3) << 4);
        }
        *dbits = rd16(blk + 208);
        return;
    }
    }
}

/* jit/gpu/kernels/pack.go:210-239 (packSub) */
static void pack_sub(uint32_t *qs, const int32_t *q, const qinfo *qi, int si, int nrows, int r) {
    int pw = qi->sub * qi->bits / 32, hw = qi->sub * qi->hi / 32;
    uint8_t out[32];
    memset(out, 0, sizeof out);
    if (qi->bits < 8) {
        int n = qi->sub / (8 / qi->bits);
        for (int l = 0; l < qi->sub; l++)
            out[l % n] |= (uint8_t)(((uint8_t)q[l] & (uint8_t)((1u << qi->bits) - 1))
                                    << (qi->bits * (l / n)));
    } else {
        for (int l = 0; l < qi->sub; l++) out[l] = (uint8_t)(int8_t)q[l];
    }
    if (hw > 0) {
        int lanes = 8 / qi->hi;
        for (int l = 0; l < qi->sub; l++) {
            int g = l / 4;
            int b = pw * 4 + (g / lanes) * 4 + l % 4;
            out[b] |= (uint8_t)((uint8_t)(q[l] >> qi->bits) << (qi->hi * (g % lanes)));
        }
    }
    for (int w = 0; w < pw + hw; w++) {
        uint32_t v = (uint32_t)out[4 * w] | ((uint32_t)out[4 * w + 1] << 8) |
                     ((uint32_t)out[4 * w + 2] << 16) | ((uint32_t)out[4 * w + 3] << 24);
        qs[((size_t)si * (size_t)(pw + hw) + (size_t)w) * (size_t)nrows + (size_t)r] = v;
    }
}

/* jit/gpu/kernels/pack.go:407-420 */
static int mxfp4_refuse(const uint8_t *src, size_t nbytes) {
    for (size_t b = 0; b + 17 <= nbytes; b += 17) {
        uint8_t e = src[b];
        if (e >= 2 && e != 0xFF) continue;
        for (int i = 1; i < 17; i++)
            if (src[b + i] & 0x77) return -2;
    }
    return 0;
}

/* jit/gpu/kernels/pack.go:52-199 (PackWeightsInto, packRows) */
int jlo_pack_weights(int type, const uint8_t *src, int nrows, int k, uint32_t *qs,
                     uint32_t *d, uint32_t *sc) {
    qinfo qi;
    size_t nq, nd, nsc;
    if (qinfo_of(type, &qi) < 0) return -1;
    if (k % qi.block_e != 0) return -1;
    if (jlo_packed_words(type, nrows, k, &nq, &nd, &nsc) < 0) return -1;
    int nsuper = k / qi.block_e;
    if (type == JLO_MXFP4 && mxfp4_refuse(src, (size_t)nrows * nsuper * qi.block_b) < 0) return -2;
    memset(d, 0, nd * 4);
    if (nsc) memset(sc, 0, nsc * 4);
    int32_t q[32];
    int per_super_blk = qi.block_e / qi.sub;
    for (int r = 0; r < nrows; r++) {
        for (int sb = 0; sb < nsuper; sb++) {
            const uint8_t *blk = src + ((size_t)r * nsuper + sb) * (size_t)qi.block_b;
            for (int s = 0; s < per_super_blk; s++) {
                uint16_t dbits, dminbits;
                uint8_t sci, mi;
                extract(type, blk, s, q, &dbits, &dminbits, &sci, &mi);
                int si = sb * per_super_blk + s;
                pack_sub(qs, q, &qi, si, nrows, r);
                int sup = si / qi.per_super;
                size_t di;
                int slot;
                d_index(&qi, sup, nrows, r, &di, &slot);
                switch (d_slots(&qi)) {
                case 4: d[di] |= (uint32_t)dbits << (8 * slot); break;
                case 2: d[di] |= (uint32_t)dbits << (16 * slot); break;
                default: d[di] |= (uint32_t)dbits | ((uint32_t)dminbits << 16);
                }
                if (nsc) {
                    if (sc_stream(&qi)) {
                        uint32_t ws[3] = {0, 0, 0};
                        sc_put(ws, s, 0, sci);
                        sc_put(ws, s, 1, mi);
                        for (int w = 0; w < 3; w++)
                            sc[((size_t)sup * 3 + w) * (size_t)nrows + r] |= ws[w];
                    } else if (qi.bias_array) {
                        int w = si / 2, lane = si % 2;
                        sc[(size_t)w * nrows + r] |=
                            ((uint32_t)sci << (lane * 16)) | ((uint32_t)mi << (lane * 16 + 8));
                    } else {
                        int w = si / 4, lane = si % 4;
                        sc[(size_t)w * nrows + r] |= (uint32_t)sci << (lane * 8);
                    }
                }
            }
        }
    }
    return 0;
}

/* internal/oracle/packed.go:66-79 (dScale) */
static void d_scale(const qinfo *qi, const uint32_t *d, int super, int nrows, int r,
                    float *scale, float *dmin) {
    size_t di;
    int slot;
    d_index(qi, super, nrows, r, &di, &slot);
    uint32_t dw = d[di];
    *dmin = 0;
    switch (d_slots(qi)) {
    case 4: *scale = bits_f32((uint32_t)(uint8_t)(dw >> (8 * slot)) << 23); return;
    case 2: *scale = jlo_half_to_f32((uint16_t)(dw >> (16 * slot))); return;
    }
    *scale = jlo_half_to_f32((uint16_t)dw);
    *dmin = jlo_half_to_f32((uint16_t)(dw >> 16));
}

/* internal/oracle/packed.go:41-49 (hiPlane) */
static uint32_t hi_plane(const uint32_t *qs, const qinfo *qi, size_t base, int nrows, int pw, int l) {
    if (qi->hi == 0) return 0;
    int lanes = 8 / qi->hi, g = l / 4;
    uint32_t v = qs[base + (size_t)(pw + g / lanes) * nrows];
    return (v >> (8 * (l % 4) + qi->hi * (g % lanes))) & ((1u << qi->hi) - 1);
}

/* One sub-block's (scale, bias) in the normalised form value = scale*Q - bias,
 * internal/oracle/packed.go:124-153. */
static void sub_scale_bias(const qinfo *qi, const uint32_t *d, const uint32_t *sc, int si,
                           int nrows, int r, float *scale_out, float *bias_out) {
    int super = si / qi->per_super;
    float scale, dmin, bias = 0;
    d_scale(qi, d, super, nrows, r, &scale, &dmin);
    if (sc_stream(qi)) {
        uint32_t ws[3];
        for (int w = 0; w < 3; w++) ws[w] = sc[((size_t)super * 3 + w) * nrows + r];
        uint8_t scv = sc_value(ws, si % 8, 0), mv = sc_value(ws, si % 8, 1);
        volatile float s2 = scale * (float)((int32_t)scv + qi->sc_off);
        scale = s2;
        volatile float b2 = dmin * (float)mv;
        bias = b2;
    } else if (qi->per_super > 1) {
        int per_word = qi->bias_array ? 2 : 4, stride = qi->bias_array ? 16 : 8;
        uint32_t sw = sc[(size_t)(si / per_word) * nrows + r];
        int sh = (si % per_word) * stride;
        volatile float s2 = scale * (float)((int32_t)((sw >> sh) & 0xFF) + qi->sc_off);
        scale = s2;
        if (qi->bias_array) {
            volatile float b2 = dmin * (float)((sw >> (sh + 8)) & 0xFF);
            bias = b2;
        }
    } else if (qi->bias_array) {
        bias = dmin;
    }
    if (!qi->bias_array) {
        volatile float b2 = scale * qi->bias_k;
        bias = b2;
    }
    *scale_out = scale;
    *bias_out = bias;
}

/* jit/gpu/kernels/matvec.go:169-175 (mxfp4Codes = MXFP4Values + 12) */
static uint32_t code_of(const qinfo *qi, uint32_t q) {
    return qi->codes ? (uint32_t)(mxfp4_values[q] + 12) : q;
}

/* Walks one row of the planes; calls back element by element.  Shared by
 * RowPacked and MatVecPackedRows, which are the same loop in the reference
 * (internal/oracle/packed.go:124-188 and :228-279). */
static void row_walk(const qinfo *qi, const uint32_t *qs, const uint32_t *d, const uint32_t *sc,
                     int r, int nrows, int k, float *dst /* k values */) {
    int nsub = k / qi->sub;
    int pw = qi->sub * qi->bits / 32, hw = qi->sub * qi->hi / 32, words = pw + hw;
    for (int si = 0; si < nsub; si++) {
        float scale, bias;
        sub_scale_bias(qi, d, sc, si, nrows, r, &scale, &bias);
        size_t base = (size_t)si * words * nrows + r;
        int e0 = si * qi->sub;
        if (qi->bits < 8) {
            int fields = 8 / qi->bits, h = qi->sub / fields;
            uint32_t mask = (1u << qi->bits) - 1;
            for (int w = 0; w < pw; w++) {
                uint32_t v = qs[base + (size_t)w * nrows];
                for (int b = 0; b < 4; b++) {
                    uint32_t by = v >> (8 * b);
                    for (int f = 0; f < fields; f++) {
                        int l = w * 4 + b + f * h;
                        uint32_t q = code_of(qi, (by >> (qi->bits * f)) & mask) |
                                     (hi_plane(qs, qi, base, nrows, pw, l) << 4);
                        volatile float p = scale * (float)q;
                        dst[e0 + l] = p - bias;
                    }
                }
            }
            continue;
        }
        for (int w = 0; w < pw; w++) {
            uint32_t v = qs[base + (size_t)w * nrows];
            for (int b = 0; b < 4; b++) {
                uint8_t by = (uint8_t)(v >> (8 * b));
                float q = qi->signed_q ? (float)(int8_t)by : (float)by;
                volatile float p = scale * q;
                dst[e0 + w * 4 + b] = p - bias;
            }
        }
    }
}

/* internal/oracle/packed.go:199-281 */
int jlo_row_packed(float *dst, int type, const uint32_t *qs, const uint32_t *d,
                   const uint32_t *sc, int r, int nrows, int k) {
    qinfo qi;
    if (qinfo_of(type, &qi) < 0 || k % qi.block_e != 0) return -1;
    if (r < 0 || r >= nrows) return -1;
    row_walk(&qi, qs, d, sc, r, nrows, k, dst);
    return 0;
}

/* internal/oracle/packed.go:87-192: acc += (scale*q - bias) * x[e], f32, in the
 * element order the reader visits (words, bytes, fields). */
int jlo_matvec_packed_rows(float *out, int type, const uint32_t *qs, const uint32_t *d,
                           const uint32_t *sc, const float *x, int nrows, int k, int lo,
                           int hi) {
    qinfo qi;
    if (qinfo_of(type, &qi) < 0 || k % qi.block_e != 0) return -1;
    if (lo < 0 || hi < lo || hi > nrows) return -1;
    float *row = (float *)malloc((size_t)k * sizeof(float));
    if (!row) return -1;
    int pw = qi.sub * qi.bits / 32;
    for (int r = lo; r < hi; r++) {
        row_walk(&qi, qs, d, sc, r, nrows, k, row);
        volatile float acc = 0;
        int nsub = k / qi.sub;
        for (int si = 0; si < nsub; si++) {
            int e0 = si * qi.sub;
            if (qi.bits < 8) {
                int fields = 8 / qi.bits, h = qi.sub / fields;
                for (int w = 0; w < pw; w++)
                    for (int b = 0; b < 4; b++)
                        for (int f = 0; f < fields; f++) {
                            int l = w * 4 + b + f * h;
                            volatile float p = row[e0 + l] * x[e0 + l];
                            acc = acc + p;
                        }
            } else {
                for (int l = 0; l < qi.sub; l++) {
                    volatile float p = row[e0 + l] * x[e0 + l];
                    acc = acc + p;
                }
            }
        }
        out[r] = acc;
    }
    free(row);
    return 0;
}

/* ------------------------------------------------------- row-major matvec */

/* internal/oracle/oracle.go:23-61: Dequant32 then a Neumaier-compensated f32 dot. */
int jlo_matvec(float *out, int type, const uint8_t *w, const float *x, int nrows, int k) {
    int be = jlo_block_elems(type), bb = jlo_block_bytes(type);
    if (be == 0 || k % be != 0) return -1;
    size_t row_bytes = (size_t)(k / be) * (size_t)bb;
    float *row = (float *)malloc((size_t)k * sizeof(float));
    if (!row) return -1;
    for (int r = 0; r < nrows; r++) {
        jlo_dequant(type, w + (size_t)r * row_bytes, row, (size_t)k);
        volatile float sum = 0, comp = 0;
        for (int i = 0; i < k; i++) {
            volatile float p = row[i] * x[i];
            volatile float t = sum + p;
            if (fabsf(sum) >= fabsf(p)) {
                volatile float u = sum - t;
                volatile float v = u + p;
                comp = comp + v;
            } else {
                volatile float u = p - t;
                volatile float v = u + sum;
                comp = comp + v;
            }
            sum = t;
        }
        out[r] = sum + comp;
    }
    free(row);
    return 0;
}

int jlo_matvec_f64(double *out, int type, const uint8_t *w, const float *x, int nrows, int k) {
    int be = jlo_block_elems(type), bb = jlo_block_bytes(type);
    if (be == 0 || k % be != 0) return -1;
    size_t row_bytes = (size_t)(k / be) * (size_t)bb;
    float *row = (float *)malloc((size_t)k * sizeof(float));
    if (!row) return -1;
    for (int r = 0; r < nrows; r++) {
        jlo_dequant(type, w + (size_t)r * row_bytes, row, (size_t)k);
        double s = 0;
        for (int i = 0; i < k; i++) s += (double)row[i] * (double)x[i];
        out[r] = s;
    }
    free(row);
    return 0;
}

/* -------------------------------------------------- activation quantizer */

/* Shared core of internal/oracle/quantize.go:80-119 and
 * jit/gpu/kernels/pack.go:474-525: amax over the block's window (clamped to
 * the vector), d = amax/127, inv = 1/d (both IEEE f32 divisions),
 * q = round-half-away(f32(v*inv)). */
static void quant_block(const float *x, int k, int b, int window, int8_t *q, float *d_out) {
    int per = window / 32;
    if (per < 1) per = 1;
    int w0 = (b / per) * per * 32, w1 = w0 + per * 32;
    if (w1 > k) w1 = k;
    uint32_t amax_bits = 0;
    for (int i = w0; i < w1; i++) {
        uint32_t u = f32_bits(x[i]) & 0x7FFFFFFFu;
        if (u > amax_bits) amax_bits = u;
    }
    float amax = bits_f32(amax_bits);
    volatile float d = amax / 127.0f;
    volatile float inv = 0;
    if (d != 0) inv = 1.0f / d;
    for (int i = 0; i < 32; i++) {
        volatile float p = x[b * 32 + i] * inv;
        q[i] = (int8_t)(int)round((double)p); /* math.Round: half away from zero */
    }
    *d_out = d;
}

/* jit/gpu/kernels/pack.go:474-525 */
int jlo_quantize_act(int8_t *q, float *as, float *sum16, const float *x, int k, int window) {
    if (k % 32 != 0) return -1;
    for (int b = 0; b < k / 32; b++) {
        float d;
        quant_block(x, k, b, window, q + b * 32, &d);
        int lo = 0, hi = 0;
        for (int i = 0; i < 16; i++) lo += q[b * 32 + i];
        for (int i = 16; i < 32; i++) hi += q[b * 32 + i];
        as[b] = d;
        sum16[2 * b] = (float)lo;
        sum16[2 * b + 1] = (float)hi;
    }
    return 0;
}

/* internal/oracle/quantize.go:80-119 and :53-61 */
int jlo_quantize_q8_window(int8_t *q, float *pairs, float *half, const float *x, int k,
                           double biasC, int window) {
    if (k % 32 != 0) return -1;
    for (int b = 0; b < k / 32; b++) {
        float d;
        quant_block(x, k, b, window, q + b * 32, &d);
        int sum = 0;
        for (int i = 0; i < 32; i++) sum += q[b * 32 + i];
        pairs[2 * b] = d;
        pairs[2 * b + 1] = (float)(-(double)sum * biasC / 8);
    }
    if (half)
        for (int h = 0; h * 16 + 16 <= k; h++) {
            int s = 0;
            for (int i = 0; i < 16; i++) s += q[h * 16 + i];
            half[h] = (float)(-(double)s * biasC / 4);
        }
    return 0;
}

/* jit/cpu/matvec.go:78-105 */
double jlo_bias_c(int type) {
    qinfo qi;
    if (qinfo_of(type, &qi) < 0) return 0;
    if (qi.bias_array) return 1;
    if (qi.signed_q) return 128;
    return qi.bias_k;
}

/* ----------------------------- like-for-like int8-activation evaluators */

/* One GGUF row -> per sub-block integer quants Q (after the code table, before
 * the zero point), via the same extract the packer uses. */
typedef struct { float d, dmin; int sc, m; } subscale;

static void row_sub(int type, const qinfo *qi, const uint8_t *row, int si, int32_t *q,
                    subscale *ss) {
    int per_blk = qi->block_e / qi->sub;
    const uint8_t *blk = row + (size_t)(si / per_blk) * qi->block_b;
    uint16_t dbits, dminbits;
    uint8_t sc, m;
    extract(type, blk, si % per_blk, q, &dbits, &dminbits, &sc, &m);
    if (qi->e8m0) ss->d = bits_f32((uint32_t)(uint8_t)dbits << 23);
    else ss->d = jlo_half_to_f32(dbits);
    ss->dmin = jlo_half_to_f32(dminbits);
    ss->sc = (int)sc + qi->sc_off;
    ss->m = m;
    if (qi->codes)
        for (int l = 0; l < qi->sub; l++) q[l] = mxfp4_values[q[l]] + 12;
}

/* value = d_a * (scale*dot - bias*sum_a), summed over sub-blocks, all in f64
 * from the exact integer dot and the f32-representable factors. */
int jlo_matvec_q8act_f64(double *out, int type, const uint8_t *w, const int8_t *qa,
                         const float *as, int nrows, int k) {
    qinfo qi;
    if (qinfo_of(type, &qi) < 0 || k % qi.block_e != 0) return -1;
    size_t row_bytes = (size_t)(k / qi.block_e) * qi.block_b;
    int nsub = k / qi.sub;
    int32_t q[32];
    for (int r = 0; r < nrows; r++) {
        const uint8_t *row = w + (size_t)r * row_bytes;
        double acc = 0;
        for (int si = 0; si < nsub; si++) {
            subscale ss;
            row_sub(type, &qi, row, si, q, &ss);
            int64_t dot = 0, suma = 0;
            for (int l = 0; l < qi.sub; l++) {
                int a = qa[si * qi.sub + l];
                dot += (int64_t)q[l] * a;
                suma += a;
            }
            double scale = (double)ss.d, bias;
            if (qi.per_super > 1) scale *= (double)ss.sc;
            if (qi.bias_array) bias = (double)ss.dmin * (double)ss.m;
            else bias = scale * (double)qi.bias_k;
            double da = as[(si * qi.sub) / 32];
            acc += da * (scale * (double)dot - bias * (double)suma);
        }
        out[r] = acc;
    }
    return 0;
}

/* jit/gpu/kernels/matvec.go:1121-1271, one row, sub-blocks in k order:
 *   bias array (Q4_K): v = f32(dot)*scale - sum_a*(dmin*f32(m))
 *   biasK == 0 (Q8_0): v = f32(dot)*scale
 *   otherwise        : v = scale*fma(-biasK, sum_a, f32(dot))
 *   acc = fma(v, d_a, acc)
 * scale = d*f32(sc) for the k-quants, d otherwise. */
int jlo_matvec_q8act_f32(float *out, int type, const uint8_t *w, const int8_t *qa,
                         const float *as, const float *sum16, int nrows, int k) {
    qinfo qi;
    if (qinfo_of(type, &qi) < 0 || k % qi.block_e != 0) return -1;
    size_t row_bytes = (size_t)(k / qi.block_e) * qi.block_b;
    int nsub = k / qi.sub;
    int32_t q[32];
    for (int r = 0; r < nrows; r++) {
        const uint8_t *row = w + (size_t)r * row_bytes;
        float acc = 0;
        for (int si = 0; si < nsub; si++) {
            subscale ss;
            row_sub(type, &qi, row, si, q, &ss);
            int32_t dot = 0;
            for (int l = 0; l < qi.sub; l++) dot += q[l] * (int32_t)qa[si * qi.sub + l];
            volatile float suma;
            if (qi.sub == 16) suma = sum16[si];
            else suma = sum16[2 * si] + sum16[2 * si + 1];
            volatile float scale = ss.d;
            if (qi.per_super > 1) scale = ss.d * (float)ss.sc;
            volatile float v;
            if (qi.bias_array) {
                volatile float bias = ss.dmin * (float)ss.m;
                volatile float t1 = (float)dot * scale;
                volatile float t2 = suma * bias;
                v = t1 - t2;
            } else if (qi.bias_k == 0) {
                v = (float)dot * scale;
            } else {
                volatile float t = fmaf(-qi.bias_k, suma, (float)dot);
                v = scale * t;
            }
            acc = fmaf(v, as[(si * qi.sub) / 32], acc);
        }
        out[r] = acc;
    }
    return 0;
}

/* ------------------------------------------------------------------- MoE */

/* internal/oracle/moe.go:332-359 (moeLexTopK, no fault): k largest, descending,
 * lowest index wins a tie, NaN never eligible.  Returns how many were found. */
static int lex_topk(const float *v, int n, int k, int32_t *out) {
    float prev_val = 0;
    int prev_idx = -1, found = 0;
    for (int i = 0; i < k; i++) {
        int best = -1;
        float best_val = 0;
        for (int e = 0; e < n; e++) {
            float x = v[e];
            if (x != x) continue;
            if (i > 0 && !(x < prev_val || (x == prev_val && e > prev_idx))) continue;
            if (best < 0 || x > best_val) { best = e; best_val = x; }
        }
        if (best < 0) break;
        out[found++] = best;
        prev_val = best_val;
        prev_idx = best;
    }
    return found;
}

/* internal/oracle/oracle.go:230-240 (RMSNorm32): the sum of squares and the scale in f64,
 * in element order; y[i] = f32(f64(x[i]) * scale * f64(w[i])). */
void jlo_rmsnorm32(float *y, const float *x, const float *w, int n, double eps) {
    double sum = 0;
    for (int i = 0; i < n; i++) sum += (double)x[i] * (double)x[i];
    double scale = 1 / sqrt(sum / (double)n + eps);
    for (int i = 0; i < n; i++) y[i] = (float)((double)x[i] * scale * (double)w[i]);
}

/* jit/gpu/kernels/moe.go:843-917 (routerMatVec): the router's logits, out[t][r] = sum_i
 * W[r][i] * x[t][i] in f32 in the device kernel's order.  128 threads a row: thread j adds
 * the products of i = j, j + 128, ... one after the other over ceil(k/128) trips (product
 * rounded, then added; a trip past k adds +0), then the partial sums meet in a binary
 * tree, thread j taking thread j + s at s = 64, 32, ..., 1.  W is f32, or f16 when f16 != 0
 * (decoded exactly).  No golden vector of the reference covers the order; the tests pin it
 * with crafted cancellation cases whose answer under this order is known by hand. */
void jlo_router_logits(float *out, const void *w, int f16, const float *x, int rows, int k, int ntok) {
    const float *wf = (const float *)w;
    const uint16_t *wh = (const uint16_t *)w;
    for (int t = 0; t < ntok; t++)
        for (int r = 0; r < rows; r++) {
            float part[128];
            for (int j = 0; j < 128; j++) {
                float acc = 0.f;
                for (int i0 = 0; i0 < k; i0 += 128) {
                    int i = i0 + j, ic = i < k ? i : k - 1;
                    size_t e = (size_t)r * k + ic;
                    float wv = f16 ? jlo_half_to_f32(wh[e]) : wf[e];
                    float prod = wv * x[(size_t)t * k + ic];
                    acc = acc + (i < k ? prod : 0.f);
                }
                part[j] = acc;
            }
            for (int s = 64; s >= 1; s >>= 1)
                for (int j = 0; j < s; j++) part[j] = part[j] + part[j + s];
            out[(size_t)t * rows + r] = part[0];
        }
}

/* internal/oracle/oracle.go:244-265 (Softmax32) then internal/oracle/moe.go:197-327
 * with Norm = true, Scale = 1, no bias, no groups, no expert scales. */
int jlo_moe_route(const float *logits, int n, int k, int32_t *sel, float *wt, int32_t *ord,
                  float *owt) {
    if (n <= 0 || k <= 0 || k > n) return -1;
    float *scores = (float *)malloc((size_t)n * sizeof(float));
    if (!scores) return -1;
    float mx = logits[0];
    for (int i = 1; i < n; i++)
        if (logits[i] > mx) mx = logits[i];
    double sum = 0;
    for (int i = 0; i < n; i++) {
        double e = exp((double)logits[i] - (double)mx);
        scores[i] = (float)e;
        sum += e;
    }
    double inv = 1 / sum;
    for (int i = 0; i < n; i++) scores[i] = (float)((double)scores[i] * inv);

    int found = lex_topk(scores, n, k, sel);
    for (int i = 0; i < found; i++) ord[i] = sel[i];
    for (int i = 1; i < found; i++)
        for (int j = i; j > 0 && ord[j] < ord[j - 1]; j--) {
            int32_t t = ord[j]; ord[j] = ord[j - 1]; ord[j - 1] = t;
        }
    volatile float s = 0;
    for (int i = 0; i < found; i++) s = s + scores[sel[i]];
    s = s + 1e-20f; /* moeSumFloor */
    for (int i = 0; i < found; i++) wt[i] = scores[sel[i]] / s;
    for (int i = 0; i < found; i++)
        for (int j = 0; j < found; j++)
            if (sel[j] == ord[i]) owt[i] = wt[j];
    free(scores);
    return found;
}

/* jit/gpu/tier/grouppairs_test.go:91-122 */
int jlo_group_pairs(const uint32_t *sel, int rows, int k, int n_exp, int unit, uint32_t *perm,
                    uint32_t *col_e, uint32_t *pos, int ncols) {
    int *count = (int *)calloc((size_t)n_exp, sizeof(int));
    int *start = (int *)calloc((size_t)n_exp, sizeof(int));
    if (!count || !start) { free(count); free(start); return -1; }
    for (int r = 0; r < rows; r++)
        for (int s = 0; s < k; s++) count[sel[r * (k + 1) + s]]++;
    int c = 0;
    for (int e = 0; e < n_exp; e++) {
        start[e] = c;
        c += (count[e] + unit - 1) / unit * unit;
    }
    if (c > ncols) { free(count); free(start); return -1; }
    for (int i = 0; i < ncols; i++) { perm[i] = (uint32_t)rows; col_e[i] = 0; }
    for (int e = 0; e < n_exp; e++)
        for (int j = start[e]; j < start[e] + (count[e] + unit - 1) / unit * unit; j++)
            col_e[j] = (uint32_t)e;
    for (int r = 0; r < rows; r++)
        for (int s = 0; s < k; s++) {
            uint32_t e = sel[r * (k + 1) + s];
            int j = start[e]++;
            perm[j] = (uint32_t)r;
            pos[r * k + s] = (uint32_t)j;
        }
    free(count);
    free(start);
    return c;
}
