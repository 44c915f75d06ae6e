/*
 * jlmi.h -- C ABI of the MI355X (gfx950) quantized-weight matmul path.
 *
 * This is the boundary a host program binds (cgo, ctypes, dlopen): plain
 * pointers and sizes, no C++ or framework types.  Each entry point names the
 * interface of the reference engine it stands behind.  The library loads one
 * gfx950 code object with hipModuleLoad and launches its kernels on HIP
 * streams; there is no CPU fallback inside it.
 *
 * Result convention (the reference's device seam returns a bool, "served" or
 * "declined, run the host path"; engine/nn/device.go:18-31):
 *     JL_OK        served: the output is complete
 *     JL_DECLINED  not served (unsupported type or shape); nothing was written,
 *                  the caller runs its own path.  Never an approximation.
 *     < 0          failure (bad argument, HIP error); jl_last_error() says what
 *
 * Two families of entry points:
 *   host-pointer  (jl_matvec, jl_matmul, ...): operands are host memory, the
 *       library owns device residency of weights keyed on the host pointer,
 *       exactly the contract of nn.Device.MatVec.  Synchronous.
 *   device-pointer (*_dev): operands are device memory of the context's
 *       device, work is enqueued on the given hipStream_t (void*; NULL = the
 *       context's own stream) and not waited for.  This is what a resident
 *       engine and the benchmarks call: no PCIe in the loop.
 *
 * Weight types are ggml type numbers (format/quant/types.go:14-55).
 * Matrices: W is [nrows][k] (k = input features, contiguous), x is [ntok][k],
 * out is [ntok][nrows] -- the reference's layouts (engine/nn/packedmm.go:23).
 */
#ifndef JLMI_H
#define JLMI_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define JL_OK 0
#define JL_DECLINED 1
#define JL_ERR_ARG (-1)
#define JL_ERR_HIP (-2)
#define JL_ERR_NOMEM (-3)

#define JL_TYPE_F32 0   /* router weights only (jl_moe_logits_dev) */
#define JL_TYPE_F16 1
#define JL_TYPE_Q8_0 8
#define JL_TYPE_Q4_K 12
#define JL_TYPE_Q6_K 14
#define JL_TYPE_MXFP4 39

typedef struct jl_ctx jl_ctx;

/* Per-context options; the library reads no environment variables, like the
 * reference's per-instance options (engine/nn/options.go:7-13). */
typedef struct jl_options {
    int device;              /* HIP device ordinal; < 0: a context bound to no device --
                                its host-side bookkeeping works (residency keys, the
                                forget queue, the lock), every entry point that needs
                                the GPU fails with JL_ERR_HIP */
    int act_window;          /* activation amax window: 32 or 256; 0 = 32 */
    const char *code_object; /* path of the gfx950 code object; NULL = the file
                                jlmi_gfx950.hsaco beside the library */
} jl_options;

/* Creates a context: selects the device, creates a stream, hipModuleLoad()s the
 * code object and resolves every kernel.  Replaces opening a backend device
 * (jit/gpu/hip/hipapi.go:43-114, jit/gpu/backend/backend.go:60-78). */
int jl_ctx_create(jl_ctx **out, const jl_options *opts);
void jl_ctx_destroy(jl_ctx *ctx);

/* Name of the HIP runtime library the context calls (resolved with dlopen; a
 * runtime the process already holds is reused), "" when none could be loaded.
 * The reference reaches its drivers the same way (jit/gpu/hip/hipapi.go:43-72). */
const char *jl_hip_runtime(void);

/* Text of the last failure on this context (or of the last failed
 * jl_ctx_create when ctx is NULL).  Valid until the next call. */
const char *jl_last_error(const jl_ctx *ctx);

/* nn.ActWindower.SetActWindow (engine/nn/device.go:39-44, :1566-1568): the amax
 * window of the activation quantizer, 32 or 256 (jit/cpu/matvec.go:46-62). */
int jl_set_act_window(jl_ctx *ctx, int window);

/* The context's own stream as a hipStream_t. */
void *jl_stream(jl_ctx *ctx);
int jl_synchronize(jl_ctx *ctx);

/* Kernel-shape overrides for measurement and the parity tests: key is one of "matvec.rpw"
 * (rows per wavefront: 1, 2, 4), "matvec.block" (threads per workgroup), "matvec.grid"
 * (workgroups), "matvec.q8pair" (2: Q8_0
 * rows one block a lane-slot even where the two-block form with 4-byte-aligned loads applies),
 * "matvec.xpre" (1 / 4: float4 groups of the activation a thread loads ahead of its weights),
 * "matvec.act_split" (1: a group's gated activation is formed and quantized once, by a launch of
 * its own, instead of by every workgroup), "gemm.min_tok"
 * (fewest tokens sent to the matrix-core GEMM), "gemm.form" (1: 128 x 64 tiles, 2: 256 x 128
 * tiles, 3: two-pass, 4 / 5: the few-token forms, 6: 128 x 64 tiles over the whole of K on two
 * groups of wavefronts, 9: token by token), "gemm.rows" (64 or 128),
 * "gemm.split" (K slices), "gemm.prep" (4: the four-wavefront activation prep), "gemm.planes"
 * (2: restore rows from planes before the GEMM), "packed.rw" (rows per wavefront of the
 * packed-plane matvec: 16, 32, 64), "packed.block" (its threads per workgroup), "moe.shares"
 * (row shares an expert's matrix is split into), "moe.form" (grouped matmul: 1 dot products,
 * 2 / 3 groups of 32 / 16 columns on the matrix cores, 4 the prefill tile per expert),
 * "moe.group16" (form 3: 1 a prep kernel quantizes the columns, 2 the matrix kernel does, 3 groups
 * of 32 columns),
 * "moe.chunk" (form 3: super-blocks a step, 1-3),
 * "moe.group" / "moe.logits" / "moe.q6k_cols" / "moe.waves" / "moe.lpr" (forms of the mixture
 * block's other kernels),
 * "mxfp4.split" (K slices of the MXFP4 GEMM), "mxfp4.rows" (96 or 128 rows a tile; 1: the
 * general decode matvec also for one token), "mxfp4.planes" (packed MXFP4: 2 restores rows
 * first, 3 the plane GEMM whatever the grid, 64 / 32 / 16 rows a workgroup of the plane
 * matvec); value 0 restores the built-in choice.  These change launch shapes and f32 summation
 * order only.  Two keys change values, both off unless set: "mxfp4.scaled" = 1 runs
 * jl_matmul_mxfp4_packed_bf16_dev on the block-scaled fp8 x fp4 matrix instruction, which
 * quantizes the activations to MX fp8 (rel-L2 about 2.7e-2 against the bf16 activations);
 * "gemm.fold" = 1 lets the Q4_K prefill GEMM of jl_matmul_dev run its 256 x 128 tiles on
 * operands that carry the scales (weights d * sc * q - dmin * m and activations d_a * a, each
 * rounded to f16; rel-L2 about 7e-4 against the exact forms, inside the path's 1e-3), for the
 * matrices jl_fold_admit_dev has admitted and no others ("gemm.fold_waves": 4 or 8 wavefronts a
 * workgroup).  Mirrors the reference's per-instance tuning knobs (engine/nn/options.go:67-118). */
int jl_set_tuning(jl_ctx *ctx, const char *key, int value);

/* Kernels this context has launched so far: how callers and tests check that a grouped
 * call was one launch, the point of the reference's grouped forms
 * (engine/nn/packedgroup.go:13-20). */
unsigned long long jl_launch_count(const jl_ctx *ctx);

/* Measurement only; no counterpart in the reference.  What a single launch costs on this
 * machine before any arithmetic, so a kernel's time can be set beside it: kind 0 launches
 * an empty kernel, kind 1 a kernel that only reads nbytes of device memory at src (16-byte
 * aligned; every thread keeps eight 128-bit loads in flight) and stores nothing; kind 2
 * holds the stream for nbytes MICROSECONDS (<= 100000) on one wavefront that touches no
 * memory -- a benchmark enqueues it in front of a timed window so that the window's
 * launches are all queued before the first starts; kinds 3 and 4 price the matrix cores:
 * every wavefront issues nbytes ROUNDS (<= 1000000) of four independent 32x32x16 f16 matrix
 * instructions on registers, kind 4 with five f32 multiply-adds after each (the vector load
 * of the prefill GEMM's loop) -- 4 * 32768 flops a round a wavefront.  grid and block <= 0
 * pick two 1024-thread workgroups per CU (kinds 0 and 1), one 512-thread workgroup per CU
 * (kinds 3 and 4). */
int jl_probe_dev(jl_ctx *ctx, int kind, const void *src, size_t nbytes, int grid, int block,
                 void *stream);

/* ---- host-pointer seam ------------------------------------------------ */

/* nn.Device.MatVec (engine/nn/device.go:23-31; call site engine/nn/jit.go:935-940):
 * out[0:nrows] = W x, W = raw GGUF row-major bytes.  Residency is keyed on the
 * pointer w: the first offer uploads, later offers of the same pointer reuse
 * the device copy, so w must stay put and unchanged until jl_forget. */
int jl_matvec(jl_ctx *ctx, float *out, int type, const void *w, size_t wbytes,
              const float *x, int nrows, int k);

/* nn.CopyForgetter.Forget (engine/nn/device.go:1570-1581): drop any device copy
 * keyed inside [p, p+n).  Callable from any thread, also from inside a page-in that
 * this context's own upload started: it queues the range under a lock of its own that no
 * launch or upload holds, and never blocks.  If the context is free at that moment the
 * queue is applied at once (the copies are freed now); if another thread's call, or this
 * thread's own, holds the context, the next host-pointer call applies it before it looks
 * its weight up (the reference applies or queues the same way, jit/gpu/tier/forget.go:20-49);
 * jl_ctx_destroy frees what is left.  A range of DEVICE addresses withdraws the matrices
 * jl_fold_admit_dev admitted inside it. */
int jl_forget(jl_ctx *ctx, const void *p, size_t n);

/* Threads.  The host-pointer entry points (no _dev in the name) may be called from any
 * thread: each holds the context's lock for its whole synchronous run.  The *_dev entry
 * points take no lock and share the context's workspaces (activation fragments, K-split
 * slabs, the mixture block's lists, the flag word of jl_pack_weights_dev and
 * jl_fold_admit_dev): a context's *_dev calls are made by one thread at a time, on one stream
 * at a time, as the reference's tier makes its device calls (jit/gpu/tier/tier.go:2831-2843);
 * give each thread that launches concurrently a context of its own.
 *
 * The lock the host-pointer entry points hold for their whole synchronous run (the
 * reference's tier serialises the same way, jit/gpu/tier/tier.go:2831-2843), for a
 * caller that needs several of them to run as one.  Not recursive: a host-pointer call
 * between lock and unlock on the same thread deadlocks; *_dev calls and jl_forget take
 * no such lock. */
int jl_ctx_lock(jl_ctx *ctx);
int jl_ctx_unlock(jl_ctx *ctx);

/* Device copies the context holds for the host-pointer seam, after applying queued
 * forgets (takes the context lock). */
size_t jl_resident_count(jl_ctx *ctx);

/* JIT.MatMul over raw GGUF bytes (engine/nn/matmul.go:27): x [ntok][k] ->
 * out [ntok][nrows].  Each token is quantized on its own. */
int jl_matmul(jl_ctx *ctx, float *out, int type, const void *w, size_t wbytes,
              const float *x, int nrows, int k, int ntok);

/* ---- packed planes, host pointers ------------------------------------- */

/* kernels.PackedWords (jit/gpu/kernels/pack.go:580-621): u32 words of the QS, D and
 * SC planes of an nrows x k matrix.  Pure host arithmetic; JL_DECLINED for a type
 * or k the planes are not defined for. */
int jl_packed_words(int type, int nrows, int k, size_t *nq, size_t *nd, size_t *nsc);

/* JIT.MatVecPacked (engine/nn/packed.go:24): rows row .. row+nrows of planes that
 * hold `stride` rows (nn.Packed{QS,D,SC,Row,Stride}, engine/nn/device.go:70-80).
 * Residency of the three planes is keyed on the pointer qs, as for jl_matvec. */
int jl_matvec_packed(jl_ctx *ctx, float *out, int type, const uint32_t *qs, const uint32_t *d,
                     const uint32_t *sc, int row, int stride, const float *x, int nrows, int k);

/* JIT.MatMulPacked (engine/nn/packedmm.go:23): x [ntok][k] -> out [ntok][nrows]. */
int jl_matmul_packed(jl_ctx *ctx, float *out, int type, const uint32_t *qs, const uint32_t *d,
                     const uint32_t *sc, int row, int stride, const float *x, int nrows, int k,
                     int ntok);

/* ---- device-pointer entry points -------------------------------------- */

/* The activation quantizer (jit/gpu/kernels/elem.go:76-170, pack.go:474-525):
 * x [ntok][k] f32 -> q [ntok][k] int8, as [ntok][k/32] f32 scales,
 * sum16 [ntok][k/16] f32 integer sums.  k % 32 == 0; x, q 16-byte aligned. */
int jl_quantize_act_dev(jl_ctx *ctx, const float *x, int ntok, int k, int8_t *q,
                        float *as, float *sum16, void *stream);

/* quant.Dequant32 (format/quant/dequant.go:50): n elements of GGUF blocks -> f32,
 * bit-identical to the reference decoder. */
int jl_dequant_dev(jl_ctx *ctx, int type, const void *src, float *dst, size_t n,
                   void *stream);

/* JIT.MatVec / MatVecPacked semantics on resident operands (engine/nn/jit.go:916,
 * packed.go:24): quantizes x (fused into the matvec kernel) and computes
 * out[0:nrows].  w = GGUF row-major bytes, 16-byte aligned; x 16-byte aligned. */
int jl_matvec_dev(jl_ctx *ctx, float *out, int type, const void *w, const float *x,
                  int nrows, int k, void *stream);

/* The same matvec over activations already quantized by jl_quantize_act_dev
 * (the reference caches them across matvecs that share x, engine/nn/packed.go:282). */
int jl_matvec_q8_dev(jl_ctx *ctx, float *out, int type, const void *w, const int8_t *q,
                     const float *as, const float *sum16, int nrows, int k, void *stream);

/* Several decode matvecs in one launch -- on this machine a launch costs as much as
 * streaming 10 MB, so a block's projections belong together.
 *
 * jl_matvec_group_dev is JIT.MatVecPackedGroup (engine/nn/packedgroup.go:13-51) over GGUF
 * row-major weights: n <= JL_MAX_GROUP matrices (a block's q, k, v; its gate and up; a
 * single projection) read ONE activation x[0:k]; out[i] gets rows[i] rows of w[i] (type
 * type[i]).  act_up, when set, makes the activation silu(x) * act_up, formed on the way
 * into the quantizer (x is left as it was).  resid, when set, takes matrix 0's rows as
 * they are made: resid[r] += alpha * out[0][r]; resid_gate, when set, points at one logit in
 * device memory and the weight becomes alpha * sigmoid(*resid_gate) -- a shared expert's
 * contribution (engine/model/moe.go:401-497; sigma in f64 narrowed once,
 * internal/oracle/moe.go:361-370; the logit is jl_moe_logits_dev with one expert row).
 * norm_w, when set, puts an RMSNorm in
 * front of everything, the reference's RMSNormQuantRows (jit/gpu/kernels/elem.go:252-267)
 * with the arithmetic of its host form (internal/oracle/oracle.go:230-240): the activation
 * is f32(f64(x) * 1/sqrt(mean(x^2) + norm_eps) * f64(norm_w)), mean in f64; norm_out, when
 * set, receives that normed vector.  One launch, whatever the mix of types (the reference's
 * MatVecSegments, jit/gpu/kernels/matvec.go:1411-1431). */
#define JL_MAX_GROUP 4
typedef struct jl_mv_group {
    int n;
    float *out[JL_MAX_GROUP];
    int type[JL_MAX_GROUP];
    const void *w[JL_MAX_GROUP];
    int rows[JL_MAX_GROUP];
    const float *x;
    int k;
    const float *act_up;
    float *resid;
    float alpha;
    const float *resid_gate;
    const float *norm_w;
    float norm_eps;
    float *norm_out;
} jl_mv_group;
int jl_matvec_group_dev(jl_ctx *ctx, const jl_mv_group *g, void *stream);

/* JIT.MatVecPackedMulti (engine/nn/packedmulti.go:24): m <= 16 matrices of one type and
 * shape sharing one activation (a mixture's experts' gate and up at decode). */
int jl_matvec_multi_dev(jl_ctx *ctx, float *const *outs, int type, const void *const *ws,
                        const float *x, int nrows, int k, int m, void *stream);

/* JIT.MatVecPackedGather / GatherAct (engine/nn/packedmulti.go:84,93): m <= 16 matrices,
 * matrix j with its own activation x[j*xstride : j*xstride+k] (a mixture's down
 * projections); up, when given, makes it silu(x_j) * up[j*xstride : ...]. */
int jl_matvec_gather_dev(jl_ctx *ctx, float *const *outs, int type, const void *const *ws,
                         const float *x, size_t xstride, const float *up, int nrows, int k,
                         int m, void *stream);

/* The same three operations over packed planes, as the reference runs them
 * (engine/nn/packedmulti.go:24,84,93 take []*Packed): matrix j reads planes qs[j], d[j],
 * sc[j] (sc may be null for Q8_0) from row row0[j] of a buffer of `stride` rows -- an
 * expert's sheet inside its bank's pages is the bank's plane pointers with row0 =
 * expert * nrows (device.go:70-80, format/jlm/write.go:165-180) -- and the activation
 * x[j*xstride : j*xstride+k] (xstride 0: one shared activation); up, when given, makes it
 * silu(x_j) * up_j; resid, when given, takes matrix 0's rows as they are made,
 * resid[r] += alpha * out[0][r] (MVGroup.Resid, engine/nn/packedgroup.go:32-36), alpha
 * times sigmoid(*resid_gate) when resid_gate is given, as in jl_matvec_group_dev; norm_w,
 * when given (never together with up: JL_DECLINED), puts RMSNorm(x_j, norm_w, norm_eps) in
 * front of the quantizer (RMSNormQuantRows, jit/gpu/kernels/elem.go:252-267, with the host
 * arithmetic of internal/oracle/oracle.go:230-240) and norm_out, if not null, receives
 * matrix 0's normed activation.  m <= 16, one launch. */
int jl_matvec_packed_multi_dev(jl_ctx *ctx, float *const *outs, int type, const uint32_t *const *qs,
                               const uint32_t *const *d, const uint32_t *const *sc, const int *row0,
                               int stride, const float *x, size_t xstride, const float *up, float *resid,
                               float alpha, const float *resid_gate, const float *norm_w, float norm_eps,
                               float *norm_out, int nrows, int k, int m, void *stream);

/* JIT.MatVecPackedMulti / MatVecPackedGather / MatVecPackedGatherAct as the reference's callers
 * have them, over HOST memory (engine/nn/packedmulti.go:24,84,93): m matrices of one type and
 * shape, matrix j's planes qs[j], d[j], sc[j] (sc, or an entry of it, may be null for Q8_0) read
 * from row row0[j] of a buffer of `stride` rows, outs[j] receiving nrows floats.  xstride 0 is
 * Multi (every matrix reads x[0:k]); xstride >= k is Gather (matrix j reads x[j*xstride :
 * j*xstride+k]); up, when given, is GatherAct with act = JL_ACT_SILU (matrix j reads
 * silu(x_j) * up_j; another act: JL_DECLINED).  The planes are uploaded on first use and stay
 * resident, keyed on their qs pointer, until jl_forget over it, as for jl_matvec_packed.  One
 * launch per sixteen matrices; returns after the results are in outs.  m < 2 is declined, as the
 * reference declines it ("one matrix is not a batch").  Unlike the reference's GatherAct, which
 * forms the gated product in place in x, x is left as it was. */
#define JL_ACT_SILU 0   /* kernels.ActSiLU, jit/gpu/kernels/actkind.go:14 */
int jl_matvec_packed_multi(jl_ctx *ctx, float *const *outs, int type, const uint32_t *const *qs,
                           const uint32_t *const *d, const uint32_t *const *sc, const int *row0, int stride,
                           const float *x, size_t xstride, const float *up, int act, int nrows, int k,
                           int m);

/* JIT.MatVecPackedGroup over HOST memory (engine/nn/packedgroup.go:18-51, MVGroup): n <=
 * JL_MAX_GROUP packed matvecs that read one activation x[0:k] -- a block's q, k and v, its gate
 * and up, or one projection -- matrix i of type types[i] with rows[i] rows from row row[i] of
 * planes holding stride[i] rows (0: rows[i], as MVGroup's Packed.Stride).  act_up, when given,
 * makes the activation silu(x) * act_up (act = JL_ACT_SILU; x is left as it was, MVGroup.ActUp);
 * resid, when given, takes matrix 0's rows as they are made, resid[r] += alpha * outs[0][r]
 * (MVGroup.Resid / Alpha).  Nothing runs unless every matrix can be served (JL_DECLINED
 * otherwise), as the reference returns false having run nothing.  Matrices of one type and row
 * count that follow one another share a launch. */
int jl_matvec_packed_group(jl_ctx *ctx, int n, float *const *outs, const int *types,
                           const uint32_t *const *qs, const uint32_t *const *d, const uint32_t *const *sc,
                           const int *row, const int *stride, const int *rows, const float *x, int k,
                           const float *act_up, int act, float *resid, float alpha);

/* JIT.MatMulPacked / MatMul semantics on resident operands (engine/nn/packedmm.go:23,
 * matmul.go:27): x [ntok][k] f32 -> out [ntok][nrows], every token quantized on
 * its own.  Q4_K with the 256 window runs the matrix-core GEMM (quantize-and-
 * lay-out kernel, then the GEMM kernel, in a workspace the context owns); other
 * cases run one fused matvec launch per token, which the reference also falls
 * back to (engine/model/prefill.go:1036-1041).  The workspace grows on demand
 * (a device allocation); jl_reserve sizes it ahead of time. */
int jl_matmul_dev(jl_ctx *ctx, float *out, int type, const void *w, const float *x,
                  int nrows, int k, int ntok, void *stream);

/* nn.LayerDevice.Reserve(maxRows, maxK) (engine/nn/device.go:1096-1176): size the
 * prefill workspace for up to max_tok tokens of max_k features now, so later
 * calls allocate nothing. */
int jl_reserve(jl_ctx *ctx, int max_tok, int max_k);

/* nn.LayerDevice.PrepLayer / Layers / ReleaseLayers (engine/nn/device.go:1096-1176) for the
 * matmul part of a block: a block's feed-forward weights are handed over ONCE and the block is
 * then run by handle, so that no weight pointer crosses the boundary per call.  (Attention,
 * rotary tables, KV migration and the head are other parts of that interface and not of this
 * path.)
 *
 * jl_prep_layer uploads block li's weights from HOST memory (LayerPlan + LayerWeights) and keeps
 * them until jl_release_layers: JL_DECLINED when a type or shape has no kernel or the block does
 * not fit in device memory -- the reference then runs that block and every later one on the
 * CPU.  Preparing a block again replaces it.
 *   kind JL_LAYER_DENSE: the gated feed-forward block  resid += W_down (silu(W_gate h) * W_up h);
 *       gate and up of `type` [n_ffn][n_embd], down of `down_type` [n_embd][n_ffn].  norm_w, when
 *       set, is an RMSNorm in front of gate and up (h = RMSNorm(x, norm_w, norm_eps), as in
 *       jl_matvec_group_dev).
 *   kind JL_LAYER_MOE: the routed block of jl_moe_ffn_types_dev behind its own router: router
 *       f32 [n_expert][n_embd], softmax and top-k_used (jl_moe_logits_dev, jl_moe_route_dev), banks
 *       of n_expert sheets.
 *   packed = 0: gate / up / down point at GGUF row-major bytes (a bank: its sheets back to back);
 *   packed = 1: they point at a jl_host_planes each, the three packed planes of the matrix (of a
 *       bank: ONE plane set of n_expert * rows rows, an expert's sheet a row range of it).
 *
 * jl_layer_ffn_dev runs block li for n rows: h [n][n_embd] in, resid [n][n_embd] updated, both in
 * device memory (they may be one buffer, as they are for a block with its norm in front: every
 * launch that reads a row of h has been enqueued before the one that adds to it).  One row runs the
 * decode kernels (two launches for a dense block), more rows the grouped kernels of the mixture
 * block (a dense block is a mixture of one expert that every row selects with weight 1; with
 * norm_w set its rows run one at a time).  The values are those of the pointer-form entry points
 * on the same operands, bit for bit.  Workspaces are the context's (calls on one context are
 * serialized by the caller).
 *
 * jl_release_layers frees blocks lo .. hi-1 (those that are prepared). */
#define JL_LAYER_DENSE 0
#define JL_LAYER_MOE 1
typedef struct jl_host_planes {
    const uint32_t *qs, *d, *sc;   /* host memory; sc may be null for Q8_0 */
} jl_host_planes;
typedef struct jl_layer_plan {
    int kind;
    int type, down_type;
    int n_embd, n_ffn;
    int packed;
    const void *gate, *up, *down;
    const float *norm_w;           /* dense only; may be null */
    float norm_eps;
    int n_expert, k_used;          /* mixture only */
    const float *router;           /* mixture only */
} jl_layer_plan;
int jl_prep_layer(jl_ctx *ctx, int li, const jl_layer_plan *plan);
int jl_layer_ffn_dev(jl_ctx *ctx, int li, const float *h, float *resid, int n, void *stream);
int jl_release_layers(jl_ctx *ctx, int lo, int hi);
/* blocks resident now */
int jl_layer_count(jl_ctx *ctx);

/* The same for one call shape, exactly: walks the launch path of jl_matmul_dev
 * (packed = 0), jl_matmul_packed_dev (packed = 1) or, for type MXFP4,
 * jl_matmul_mxfp4_bf16_dev / jl_matmul_mxfp4_packed_bf16_dev, for this type, shape and the
 * context's current activation window (and tuning) with
 * launching switched off, so every workspace that call would grow -- activation
 * fragments, rows restored from planes, K-split partial sums -- has its size
 * afterwards and the call itself allocates nothing.  Returns what the call would. */
int jl_reserve_shape(jl_ctx *ctx, int type, int nrows, int k, int ntok, int packed);

/* jl_matmul_dev for callers that cannot allocate.  It has no counterpart in the reference:
 * it exists for code under HIP graph capture, tight serving loops and harnesses that forbid
 * hipMalloc.  Same operands, same values, same launches as jl_matmul_dev, but every
 * workspace the call needs (activation fragments, K-split partial sums) is carved from ONE
 * static device array of jl_static_scratch_bytes() bytes (64 MiB) that each GPU holds from
 * library load to process exit; the call allocates nothing, frees nothing and waits for
 * nothing.  A shape whose workspaces do not fit is refused with JL_ERR_NOMEM before
 * anything is launched (jl_last_error says how many bytes it needed).  Every call on a GPU
 * shares that GPU's array, which keeps the last call's contents: the kernels write all they
 * read, so nothing needs clearing, but calls that OVERLAP on one GPU (two streams, two
 * contexts, two threads) race on it -- order them on one stream. */
int jl_matmul_static_dev(jl_ctx *ctx, float *out, int type, const void *w, const float *x,
                         int nrows, int k, int ntok, void *stream);
size_t jl_static_scratch_bytes(void);

/* kernels.PackWeightsInto (jit/gpu/kernels/pack.go:52-199) on the device: GGUF
 * row-major blocks -> the three planes [unit][row] (sizes from jl_packed_words; sc may
 * be NULL for Q8_0 and MXFP4).  Q4_K, Q6_K, Q8_0 and MXFP4; the result is byte for byte
 * the reference's.  src 4-byte aligned for Q4_K, 2-byte for Q6_K and Q8_0.
 * MXFP4 (pack.go:395-420): the D plane holds the E8M0 exponent minus one, four rows a
 * word, and a matrix with a block of exponent 0, 1 or 255 whose codes are not all +-0 is
 * refused as the reference's mxfp4Refuse refuses it: JL_DECLINED, the planes' contents
 * then undefined.  To learn that, the MXFP4 call alone waits for its kernel. */
int jl_pack_weights_dev(jl_ctx *ctx, int type, const void *src, int nrows, int k, uint32_t *qs,
                        uint32_t *d, uint32_t *sc, void *stream);

/* Admits a Q4_K matrix in device memory (GGUF rows, 4-byte aligned) to the folded-scale GEMM
 * form that "gemm.fold" = 1 switches on: checks that no super-block's weights can pass the f16
 * range (|d| * 945 + |dmin| * 63 <= 65504, finite), waits for that check, and remembers the
 * matrix by its address, rows and k.  JL_DECLINED for scales outside the range (and for another
 * type): such a matrix keeps the exact forms whatever the key says.  A call made once after
 * the weights are in place; jl_forget over the matrix's address range withdraws it, and a
 * matrix rewritten in place is admitted again by a new call.  Activations beyond the f16
 * range give non-finite outputs in the folded form, as in any f16 GEMM.  No counterpart in
 * the reference, whose kernels keep the scales apart (engine/nn/matmul.go:27-189). */
int jl_fold_admit_dev(jl_ctx *ctx, int type, const void *w, int nrows, int k, void *stream);

/* The inverse permutation for Q4_K, Q6_K, Q8_0 and MXFP4: rows row .. row+nrows of the
 * planes back to GGUF blocks in dst (nrows * k/256 * 144 bytes, 4-byte aligned; Q6_K 210
 * bytes a super-block, Q8_0 34 bytes a block of 32, 2-byte aligned; MXFP4 17 bytes a block
 * of 32, any alignment, sc ignored), bit for bit. */
int jl_unpack_weights_dev(jl_ctx *ctx, int type, const uint32_t *qs, const uint32_t *d,
                          const uint32_t *sc, int row, int stride, int nrows, int k, void *dst,
                          void *stream);

/* JIT.MatVecPacked on resident planes (engine/nn/packed.go:24-198; device twin
 * jit/gpu/kernels/matvec.go:1121-1271): quantizes x inside the kernel and computes
 * out[0:nrows] for rows row .. row+nrows of planes holding `stride` rows.  An expert
 * sheet of a bank is its own set of planes (format/jlm/write.go:123-140): pass the
 * sheet's plane pointers with row 0. */
int jl_matvec_packed_dev(jl_ctx *ctx, float *out, int type, const uint32_t *qs, const uint32_t *d,
                         const uint32_t *sc, int row, int stride, const float *x, int nrows,
                         int k, void *stream);

/* The same over activations already quantized by jl_quantize_act_dev. */
int jl_matvec_packed_q8_dev(jl_ctx *ctx, float *out, int type, const uint32_t *qs,
                            const uint32_t *d, const uint32_t *sc, int row, int stride,
                            const int8_t *q, const float *as, const float *sum16, int nrows,
                            int k, void *stream);

/* JIT.MatMulPacked on resident planes (engine/nn/packedmm.go:23-139).  Q4_K with the
 * 256 window and enough tokens restores the row range to GGUF order in a workspace the
 * context owns and runs the matrix-core GEMM on it; other cases run one packed matvec
 * launch per token. */
int jl_matmul_packed_dev(jl_ctx *ctx, float *out, int type, const uint32_t *qs, const uint32_t *d,
                         const uint32_t *sc, int row, int stride, const float *x, int nrows,
                         int k, int ntok, void *stream);

/* MXFP4 weights (GGUF type 39: 32 e2m1 codes + one E8M0 exponent per block) against
 * bf16 activations with f32 accumulation: x [ntok][k] bf16 -> out [ntok][nrows] f32.
 * The value is the reference's Dequant32 (format/quant/dequant.go:159-174) followed by
 * an f32 matmul: dequantized MXFP4 weights are exact in bf16, so only the f32
 * summation order differs.  The reference's own device path instead feeds e2m1 codes
 * to its int8 kernels through a code table (jit/gpu/kernels/matvec.go:137-175). */
int jl_matmul_mxfp4_bf16_dev(jl_ctx *ctx, float *out, const void *w, const uint16_t *x,
                             int nrows, int k, int ntok, void *stream);

/* The same over packed MXFP4 planes (jit/gpu/kernels/pack.go:543-575: QS the code bytes
 * four words a block, D the exponent minus one four rows a word; sizes from
 * jl_packed_words, no SC plane): rows row .. row+nrows of planes of `stride` rows.  Up to
 * 8 tokens read the planes where they lie, a lane a row; so do more tokens when tiles of
 * 64 tokens x 64 rows give at least half the CUs a workgroup (a plane word is a lane's
 * eight K values of the matrix instruction's weight operand); the shapes between restore
 * the row range to GGUF blocks in a workspace the context owns and run the few-token and
 * tiled forms on it.  The value of a block is that of the GGUF block it was packed from. */
int jl_matmul_mxfp4_packed_bf16_dev(jl_ctx *ctx, float *out, const uint32_t *qs, const uint32_t *d,
                                    int row, int stride, const uint16_t *x, int nrows, int k,
                                    int ntok, void *stream);

/* ---- mixture of experts (device pointers) ----------------------------- */

/* The router's logits (kernels.RouterMatVecTok, jit/gpu/kernels/moe.go:820-917):
 * logits[t][r] = sum_i W[r][i] * x[t][i], W [n_expert][k] in f32 (JL_TYPE_F32) or f16
 * (JL_TYPE_F16, Mixtral's ffn_gate_inp), the one matrix of a mixture block that is not
 * quantized.  f32 arithmetic in that kernel's order (128 strided partial sums, then a
 * binary tree), so the logits are bit for bit what the reference's device path routes on. */
int jl_moe_logits_dev(jl_ctx *ctx, float *logits, int wtype, const void *w, const float *x,
                      int n_expert, int k, int ntok, void *stream);

/* The router (kernels.ExpertRoute, jit/gpu/kernels/moe.go:562; specification
 * oracle.MoERouter, internal/oracle/moe.go:197-327, with Softmax32, oracle.go:244-265):
 * per row, softmax over all n_expert logits (f64 exp and sum, scores narrowed to f32), the
 * k_used largest by (score descending, index ascending), weights = score / (sum of the
 * selected scores in selection order + 1e-20).  Fills sel [rows][sel_stride] (first k_used
 * of each row) and wt [rows][k_used].  n_expert <= 1024, k_used <= 16. */
int jl_moe_route_dev(jl_ctx *ctx, const float *logits, int rows, int n_expert, int k_used,
                     uint32_t *sel, int sel_stride, float *wt, void *stream);

/* The grouping the device tier runs before a batched mixture (kernels.ExpertGroup*,
 * jit/gpu/kernels/moesort.go:12-31; specification groupPairs,
 * jit/gpu/tier/grouppairs_test.go:91-122, with unit 1): sel [rows][sel_stride] holds
 * each row's k_used expert ids first.  Fills start [n_expert+1] (first column of each
 * expert's run), perm [rows*k_used] (column -> row) and pos [rows*k_used]
 * (pair r*k_used+s -> column); experts ascending, pairs in (row, slot) order. */
int jl_moe_group_dev(jl_ctx *ctx, const uint32_t *sel, int sel_stride, int rows, int k_used,
                     int n_expert, uint32_t *start, uint32_t *perm, uint32_t *pos, void *stream);

/* MUL_MAT_ID over sorted columns (the Experts/Slots/SlotAct forms of kernels.MatVec,
 * jit/gpu/kernels/matvec.go:330-343, :788-836; host forms MatVecPackedMulti / GatherAct,
 * engine/nn/packedmulti.go:24,93): for every column c of expert e,
 *   out0[c][0:nrows] = bank0 sheet e . act(c)   (and out1 / bank1 when given),
 * act(c) = x[src[c]] (src NULL: x[c]) or silu(x[..]) * x2[..] when x2 is given.  A bank
 * is n_expert sheets of nrows x k GGUF rows back to back.  ncols = start[n_expert], the
 * number of columns (rows * k_used).  Activations are quantized per column exactly as
 * jl_matvec_dev does, once, into a workspace the context owns (grown on demand). */
int jl_moe_matvec_dev(jl_ctx *ctx, float *out0, float *out1, int type, const void *bank0,
                      const void *bank1, const float *x, const float *x2, const uint32_t *src,
                      const uint32_t *start, int n_expert, int ncols, int nrows, int k,
                      void *stream);

/* kernels.ExpertCombineGrouped (jit/gpu/kernels/moegroup.go:38-68) with the host path's
 * order (engine/model/moe.go:127-134, :752-759): resid[r] += sum of wt[r][s] *
 * y[pos[r*k_used+s]] over the row's experts in ascending expert id. */
int jl_moe_combine_dev(jl_ctx *ctx, float *resid, const float *y, const float *wt,
                       const uint32_t *sel, int sel_stride, const uint32_t *pos, int rows,
                       int k_used, int n_embd, void *stream);

/* One routed feed-forward block, moeBatchFrom / moeBatchExpert
 * (engine/model/moe.go:510-761): group, gate and up in one launch, act(gate)*up fused
 * into the down launch's quantizer, combine into resid [rows][n_embd] (accumulated).
 * gate/up banks: n_expert sheets of n_ffn x n_embd; down bank: n_embd x n_ffn.
 * Intermediates live in a workspace the context owns (grown on demand). */
int jl_moe_ffn_dev(jl_ctx *ctx, float *resid, int type, const void *gate_bank,
                   const void *up_bank, const void *down_bank, const float *x,
                   const uint32_t *sel, int sel_stride, const float *wt, int rows, int k_used,
                   int n_expert, int n_ffn, int n_embd, void *stream);

/* A mixture's bank as packed planes, the way a container holds it (nn.Packed.Sheet / Sheets,
 * engine/nn/device.go:70-80; format/jlm/write.go:123-180, read.go:447-469): qs, d, sc are
 * expert 0's planes in device memory.
 *   sheet_bytes > 0: every expert's sheet was packed on its own and expert e's three planes
 *       start sheet_bytes * e bytes after expert 0's (a container's expert page size; a
 *       sheet holds `stride` rows, normally the expert's own row count);
 *   sheet_bytes == 0: the bank is ONE plane set of `stride` rows and expert e is rows
 *       e * nrows .. of it (Packed.Row / Stride). */
typedef struct jl_packed_bank {
    const uint32_t *qs, *d, *sc;
    size_t sheet_bytes;
    int stride;
} jl_packed_bank;

/* jl_moe_ffn_dev over HOST memory: resid [rows][n_embd] (read, accumulated, written back), the
 * three banks as GGUF bytes (uploaded on first use and resident, each keyed on its pointer, until
 * jl_forget over it), x [rows][n_embd], sel [rows][sel_stride] and wt [rows][k_used] as the host
 * router made them (engine/model/moe.go:697-761).  Returns after resid is back in host memory. */
int jl_moe_grouped(jl_ctx *ctx, float *resid, int type, const void *gate_bank, const void *up_bank,
                   const void *down_bank, const float *x, const uint32_t *sel, int sel_stride,
                   const float *wt, int rows, int k_used, int n_expert, int n_ffn, int n_embd);

/* jl_moe_matvec_dev over banks of packed planes: the per-expert matrix-core tile reads every
 * sheet where it lies (Q4_K with the activation window of 256; anything else JL_DECLINED).
 * bank1 / out1 may be null; both banks must share one layout (sheet_bytes, stride). */
int jl_moe_matvec_packed_dev(jl_ctx *ctx, float *out0, float *out1, int type,
                             const jl_packed_bank *bank0, const jl_packed_bank *bank1, const float *x,
                             const float *x2, const uint32_t *src, const uint32_t *start, int n_expert,
                             int ncols, int nrows, int k, void *stream);

/* jl_moe_ffn_dev over banks of packed planes (moeBatchFrom over a container's expert pages,
 * engine/model/moe.go:510-761): gate and up banks hold n_ffn x n_embd sheets, the down bank
 * n_embd x n_ffn sheets. */
int jl_moe_ffn_packed_dev(jl_ctx *ctx, float *resid, int type, const jl_packed_bank *gate,
                          const jl_packed_bank *up, const jl_packed_bank *down, const float *x,
                          const uint32_t *sel, int sel_stride, const float *wt, int rows, int k_used,
                          int n_expert, int n_ffn, int n_embd, void *stream);

/* The same block with the down bank in a type of its own: every expert tensor carries its
 * own quant.Type in the reference (nn.Weight.T, engine/nn/device.go:47-58; a Q4_K_M file
 * holds Q4_K gate and up sheets beside Q6_K down sheets). */
int jl_moe_ffn_types_dev(jl_ctx *ctx, float *resid, int type, int down_type, const void *gate_bank,
                         const void *up_bank, const void *down_bank, const float *x,
                         const uint32_t *sel, int sel_stride, const float *wt, int rows,
                         int k_used, int n_expert, int n_ffn, int n_embd, void *stream);

/* The whole mixture block for rows rows, router included (engine/model/moe.go:697-761 from the
 * hidden state on): jl_moe_logits_dev (router f32 or f16, [n_expert][n_embd]), jl_moe_route_dev,
 * then jl_moe_ffn_types_dev on that selection, in one call and bit for bit.  sel
 * [rows][k_used + 1] and wt [rows][k_used] receive the routing when given (null: kept in the
 * context's workspace, like the logits). */
int jl_moe_block_dev(jl_ctx *ctx, float *resid, int type, int down_type, const void *gate_bank,
                     const void *up_bank, const void *down_bank, int router_type, const void *router,
                     const float *x, int rows, int k_used, int n_expert, int n_ffn, int n_embd,
                     uint32_t *sel, float *wt, void *stream);

/* The same over banks of packed planes (jl_moe_ffn_packed_dev behind the router). */
int jl_moe_block_packed_dev(jl_ctx *ctx, float *resid, int type, const jl_packed_bank *gate,
                            const jl_packed_bank *up, const jl_packed_bank *down, int router_type,
                            const void *router, const float *x, int rows, int k_used, int n_expert,
                            int n_ffn, int n_embd, uint32_t *sel, float *wt, void *stream);

#ifdef __cplusplus
}
#endif
#endif
