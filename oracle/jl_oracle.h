/*
 * jl_oracle.h -- TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C, CPU restatement of the arithmetic of jitllm's quantized-weight
 * matmul path.  It exists so the HIP kernels can be checked against it; it is
 * never linked into, imported by or called from the product library.  Every
 * function cites the reference file:line it follows.
 *
 * Pinning status (what independently fixes each function):
 *   half codecs        all 65,536 patterns vs numpy float16
 *   dequant            libggml / gguf-py golden vectors held by the reference's
 *                      own tests (Q4_K, Q6_K, Q8_0, MXFP4), uint32 equality
 *   pack (Q4_K, Q5_K)  byte equality with planes written by the reference's
 *                      container writer (v29 fixture, k = 256): Q4_K pins the primary
 *                      nibble plane, the D word and the 96-bit SC stream; Q5_K (kept in
 *                      the oracle for this purpose only) pins the SECONDARY plane half of
 *                      packSub -- byte pw*4 + (g/lanes)*4 + l%4, shift hi*(g%lanes) --
 *                      which Q6_K shares with hi = 2, and its reader (RowPacked of the
 *                      packed q5_k_tiny blocks == the libggml golden values)
 *   pack (Q6_K, Q8_0,  round trip RowPacked(pack(src)) == dequant(src) on the
 *         MXFP4)       golden blocks, an independently written numpy reader,
 *                      closed-form plane sizes; that reader's indexing is also what
 *                      the reference's own independent gate restates
 *                      (jit/gpu/kernels/realpack_test.go:67-195, checkPack), so two
 *                      texts inside the reference agree with it.  What stays "parity
 *                      unpinned" (held by reading those texts, no bytes the reference wrote):
 *                      Q6_K's SC bytes (int8 + 128, four a word), Q8_0's D pairing
 *                      (two rows' f16 a word), MXFP4's D bytes (e - 1, four rows a word)
 *   act quantizer      numpy float32 brute force incl. rounding-boundary cases
 *   matvec evaluators  brute force on hand-decoded blocks; agreement between
 *                      the three independent forms (f32 dequant + Neumaier,
 *                      packed reader, int8-activation f64 form)
 *   MoE router / group brute force on tiny cases, edge cases of the reference
 *   RMSNorm32          a hand-computed case, exact rational arithmetic, unit mean
 *                      square, power-of-two scaling, the large-eps limit
 *   router logits      the ORDER of the f32 sum by cancellation cases worked out
 *                      by hand (2^24 absorbs a lone +1, not a +2); the VALUE
 *                      against f64, exact small integers, f16 == f32 weights;
 *                      the reference holds no golden vector for the order
 *   weight quantizers  NOT an oracle function: the reference has none for
 *                      Q4_K/Q6_K/MXFP4 ("parity unpinned" for the quantizer;
 *                      matmul parity is measured on the quantized bytes)
 */
#ifndef JL_ORACLE_H
#define JL_ORACLE_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ggml type numbers, format/quant/types.go:14-55 */
/* (Q5_K is not a type of the matmul path; it is here to pin the secondary-plane half of the
 * packer against bytes the reference wrote, see the pinning table above) */
enum { JLO_Q8_0 = 8, JLO_Q4_K = 12, JLO_Q5_K = 13, JLO_Q6_K = 14, JLO_MXFP4 = 39 };

/* format/quant/types.go:61-85 */
int jlo_block_elems(int type);
int jlo_block_bytes(int type);

/* format/quant/dequant.go:15-32 and :478-517 */
float    jlo_half_to_f32(uint16_t h);
uint16_t jlo_f32_to_half(float f);

/* format/quant/dequant.go:50 (Dequant32); n = number of elements */
int jlo_dequant(int type, const uint8_t *src, float *dst, size_t n);

/* jit/gpu/kernels/pack.go:580 (PackedWords) */
int jlo_packed_words(int type, int nrows, int k, size_t *nq, size_t *nd, size_t *nsc);
/* jit/gpu/kernels/pack.go:52 (PackWeightsInto); <0 on refusal (MXFP4 exponents) */
int jlo_pack_weights(int type, const uint8_t *src, int nrows, int k,
                     uint32_t *qs, uint32_t *d, uint32_t *sc);
/* internal/oracle/packed.go:199 (RowPacked) */
int jlo_row_packed(float *dst, int type, const uint32_t *qs, const uint32_t *d,
                   const uint32_t *sc, int r, int nrows, int k);
/* internal/oracle/packed.go:87 (MatVecPackedRows): f32, sequential */
int jlo_matvec_packed_rows(float *out, int type, const uint32_t *qs, const uint32_t *d,
                           const uint32_t *sc, const float *x, int nrows, int k,
                           int lo, int hi);

/* internal/oracle/oracle.go:23 (MatVec): Dequant32 + Neumaier f32 dot */
int jlo_matvec(float *out, int type, const uint8_t *w, const float *x, int nrows, int k);
/* same operands, plain f64 dot of Dequant32(w) with x (the "dequant + matmul" bar) */
int jlo_matvec_f64(double *out, int type, const uint8_t *w, const float *x, int nrows, int k);

/* jit/gpu/kernels/pack.go:474 (PackActivationsInto), device form:
 * q int8[k], as f32[k/32], sum16 f32[k/16] */
int jlo_quantize_act(int8_t *q, float *as, float *sum16, const float *x, int k, int window);
/* internal/oracle/quantize.go:80 (QuantizeQ8Window) + :53 (QuantizeHalfSums), host form:
 * pairs f32[2*k/32], half f32[k/16] (may be NULL) */
int jlo_quantize_q8_window(int8_t *q, float *pairs, float *half, const float *x, int k,
                           double biasC, int window);
/* jit/cpu/matvec.go:78-105 */
double jlo_bias_c(int type);

/* Like-for-like evaluators over int8 activations (q, as) and GGUF weight bytes.
 * f64: exact-order-free value every kernel form is held to at NMSE <= 1e-10
 *      (jit/cpu/matvec_test.go:15-18, jit/gpu/backend/matvec_test.go:16-21).
 * f32: the device form's own f32 order, jit/gpu/kernels/matvec.go:1121-1271. */
int jlo_matvec_q8act_f64(double *out, int type, const uint8_t *w, const int8_t *q,
                         const float *as, int nrows, int k);
int jlo_matvec_q8act_f32(float *out, int type, const uint8_t *w, const int8_t *q,
                         const float *as, const float *sum16, int nrows, int k);

/* internal/oracle/moe.go:197-327 with Norm = true, no bias/groups (Qwen3-MoE):
 * logits[n] -> softmax -> top-k (score desc, index asc) -> renormalised weights.
 * sel[k], wt[k] in selection order; ord[k], owt[k] ascending expert id. */
void jlo_rmsnorm32(float *y, const float *x, const float *w, int n, double eps);
void jlo_router_logits(float *out, const void *w, int f16, const float *x, int rows, int k, int ntok);
int jlo_moe_route(const float *logits, int n, int k, int32_t *sel, float *wt,
                  int32_t *ord, float *owt);
/* jit/gpu/tier/grouppairs_test.go:91-122 (groupPairs); returns used columns */
int jlo_group_pairs(const uint32_t *sel, int rows, int k, int n_exp, int unit,
                    uint32_t *perm, uint32_t *col_e, uint32_t *pos, int ncols);

#ifdef __cplusplus
}
#endif
#endif
