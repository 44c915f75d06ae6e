// Kernel argument blocks, shared by the device code and the host launcher.
// Plain C layouts: the host passes each struct by value as the kernel's single
// parameter.
#pragma once
#include <stdint.h>

struct MatVecArgs {
    float* out;          // [nrows]
    const uint8_t* w;    // GGUF row-major blocks
    const float* x;      // f32 activations (fused quantize) or null
    const int8_t* q;     // pre-quantized activations (split form) or null
    const float* as;     // [k/32] activation scales
    const float* s16;    // [k/16] activation sums
    int nrows, k;
    int row_bytes;
    int per;             // activation window / 32 (fused form)
    int nwaves;          // wavefronts per workgroup (the launch's block / 64)
    int ngroups;         // workgroups (the launch's grid)
    float* resid;        // optional: resid[r] += alpha * out[r] (times sigmoid(*resid_gate) when resid_gate is set)
    const float* resid_gate;
    float alpha;
};

// Several decode matvecs of one type in one launch (grid y = matrix): matrix i computes
// out[i][0:nrows[i]] = w[i] . act(i), act(i) = x + i*xstride (xstride 0: one shared
// activation), optionally silu(x) * (x2 + i*xstride); matrix 0 may also add
// alpha * out[0] into resid.
#define JL_MAX_MULTI 16
struct MatVecMultiArgs {
    float* out[JL_MAX_MULTI];
    const uint8_t* w[JL_MAX_MULTI];
    int nrows[JL_MAX_MULTI];
    const float* x;
    const float* x2;     // null: plain activation
    float* resid;        // null: none
    float alpha;
    const float* resid_gate;   // null, or one logit: the residual weight is alpha * sigmoid(*resid_gate)
    size_t xstride;      // elements
    int k, row_bytes, per, nwaves, ngroups;
    // the mixed-type kernel only: each matrix's type (JL_TYPE_*) and bytes per row
    int type[JL_MAX_MULTI];
    int row_bytes_of[JL_MAX_MULTI];
    // the _q entry points: one activation for every matrix, quantized beforehand (x unused)
    const int8_t* q;
    const float* as;
    const float* s16;
    const float* norm_w; // null: none; else the activation is RMSNorm(x) * norm_w first
    float* norm_out;     // optional: the normed activation, written once
    float norm_eps;
};

// Activation preparation for the Q4_K prefill GEMM: quantize x and lay it out
// in matrix-fragment order, bq [k/128 stages][tok_pad/32][9][64][8] f16, da [k/256][tok_pad].
struct GemmPrepArgs {
    const float* x;      // [ntok][k]
    uint16_t* bq;        // f16 bits
    float* da;
    int ntok, tok_pad, k;
    float* dsum = nullptr;   // window 32, optional: d_a * (sum of the block's int8) [k/32][tok_pad]
};

struct GemmArgs {
    float* out;          // [ntok][out_stride]; a launch may cover a slice of the rows
    const uint8_t* w;    // GGUF row-major Q4_K (of the slice)
    const uint16_t* bq;
    const float* da;
    int nrows, k, ntok, tok_pad;   // nrows of the slice
    int row_bytes;
    int out_stride;      // floats between tokens in out
    int sb_per;          // K split: super-blocks per blockIdx.z (0 = whole K), out = slab z of [gridDim.z][ntok][out_stride]
    const float* dsum = nullptr;   // window 32, Q4_K: the prep's d_a * block sums
    // the weights as packed planes (the kernels' plane forms; w is unused then): QS, D and SC
    // planes of a buffer of pstride rows, this launch's first row at prow0 (nrows counted from
    // it), its first super-block psb0 (a K split moves it)
    const uint32_t* pqs = nullptr;
    const uint32_t* pd = nullptr;
    const uint32_t* psc = nullptr;
    int prow0 = 0, pstride = 0, psb0 = 0;
};

// Mixture block on the matrix cores (Q4_K, activation window 256).  An expert's columns are
// cut into groups of 32; group g of expert e has the workspace slot start[e]/32 + e + g
// (distinct for distinct groups, below ncols/32 + n_expert + 1 = nslots).  The prep kernel
// gathers, quantizes and lays out the groups' activations as the prefill GEMM's fragments,
// bq [k/128 stages][nslots][9][64 lanes][8] f16 and da [k/256][32*nslots]; the matrix kernel
// meets them with the expert's sheet, out[mat][column][nrows].
//
// Most (expert, group) pairs of a grid sized for the fullest expert are empty, and an empty
// workgroup still costs its dispatch, so the kernels walk a work list instead, written by
// jl_moe_worklist from start[]: wl[0] = number of 128-column tiles, wl[4 + s] = expert of
// slot s (all ones: unused), wl[4 + nslots + t] = tile t as expert | (tile of the expert << 16).
struct MoeWorklistArgs {
    const uint32_t* start;
    uint32_t* wl;
    int n_expert, nslots;
};

struct MoeGemmPrepArgs {
    const float* x;       // [.][k]
    const float* x2;      // optional: activation is silu(x) * x2
    const uint32_t* src;  // optional: column -> row of x (identity when null)
    const uint32_t* start;
    const uint32_t* wl;
    uint16_t* bq;
    float* da;
    int k, nslots;
};

struct MoeGemmArgs {
    float* out[2];
    const uint8_t* bank[2];
    const uint16_t* bq;
    const float* da;
    const uint32_t* start;
    const uint32_t* wl;
    size_t sheet_bytes;
    int nrows, k, row_bytes, nslots, nmat;
    // the banks as packed planes (plane form of the tile kernel; bank[] unused): expert e's planes
    // are pqs / pd / psc [mat] + e * sheet_words (u32 words; 0 when the bank is ONE plane set), its
    // first row e * row_step inside them (0 when every expert has its own sheet), pstride rows a
    // plane set
    const uint32_t* pqs[2] = {nullptr, nullptr};
    const uint32_t* pd[2] = {nullptr, nullptr};
    const uint32_t* psc[2] = {nullptr, nullptr};
    size_t sheet_words = 0;
    int row_step = 0, pstride = 0;
};

// Grouped expert matmul, sixteen columns a group (moe_g16_body).  Column group g of expert e is
// slot (start[e] >> 4) + e + g of the prepared workspace; a slot holds, for every super-block,
// JL_MOE_G16_SB_WORDS words: eight matrix fragments of 64 lanes x 16 bytes (half, K-step), the
// sub-block sums' fragment (32 lanes x 16 bytes) and the sixteen columns' scales.
#define JL_MX1_RPW 2   // rows a wavefront of the one-token MXFP4 matvec walks (2880 x 2880: 1 / 2 / 3 / 4 rows 4.46 / 4.18 / 4.22 / 4.30 us)
#define JL_MOE_G16_SB_WORDS 2192
#define JL_MOE_G16_LDS_WORDS 2224   // the same in LDS, the fragments 65 vectors apart
struct MoeG16PrepArgs {
    const float* x;
    const float* x2;        // null: plain activation
    const uint32_t* src;    // null: column c reads row c
    const uint32_t* start;  // [n_expert + 1]
    uint32_t* ws;
    int k, n_expert, ncols;
};
struct MoeG16Args {
    float* out[2];
    const uint8_t* bank[2];
    const uint32_t* ws;
    const uint32_t* start;
    size_t sheet_bytes;
    int nrows, k, row_bytes;
    int tiles_wg;           // tiles of sixteen rows a workgroup owns
    int blocks, nmat, n_expert, nwaves;   // row blocks an (expert, matrix); wavefronts a workgroup
    // the banks as packed planes (plane form; bank[] and sheet_bytes unused): expert e's planes are
    // pqs / pd / psc [mat] + e * sheet_words (u32 words; 0 when the bank is ONE plane set), its first
    // row e * row_step inside them (0 when every expert has its own sheet), pstride rows a plane set
    const uint32_t* pqs[2] = {nullptr, nullptr};
    const uint32_t* pd[2] = {nullptr, nullptr};
    const uint32_t* psc[2] = {nullptr, nullptr};
    size_t sheet_words = 0;
    int row_step = 0, pstride = 0;
    // fused form: the columns are quantized by the matrix kernel itself (ws unused)
    const float* x = nullptr;
    const float* x2 = nullptr;
    const uint32_t* src = nullptr;
};

// Two-pass form of the Q4_K prefill GEMM.  Pass one expands the weights once per call into
// f16 matrix fragments, w16 [ceil(nrows/64)][k/128 stages][18 fragments][64 lanes] 16-byte
// vectors (fragment 2*ks+g: K-step ks of the tile's row group g; 16+g: the minimum columns,
// meaningful in second halves) and wsc [k/256][nrows_pad] (d, dmin); pass two is the matrix
// kernel with nothing left to dequantize.
struct GemmW16PrepArgs {
    const uint8_t* w;    // GGUF row-major Q4_K
    void* w16;           // 16-byte vectors
    float* wsc;          // pairs (d, dmin)
    int nrows, nrows_pad, k, row_bytes;
};

struct GemmW16Args {
    float* out;          // [ntok][nrows]
    const void* w16;
    const float* wsc;
    const uint16_t* bq;
    const float* da;
    int nrows, nrows_pad, k, ntok, tok_pad;
    int ntt, nrt;        // token tiles (128) and row tiles (64)
};

// Mixture-of-experts grouping: sel [rows][sel_stride] expert ids (the first k_used of
// each row are the selection) -> start [n_expert+1], perm [rows*k_used] (column ->
// row), pos [rows*k_used] (pair -> column).
struct MoeGroupArgs {
    const uint32_t* sel;
    uint32_t* start;
    uint32_t* perm;
    uint32_t* pos;
    int sel_stride, rows, k_used, n_expert;
};

// Router: softmax over all experts, the k largest by (score descending, index ascending),
// weights = selected scores over their sum.  sel [rows][sel_stride] (first k_used filled),
// wt [rows][k_used].
struct MoeRouteArgs {
    const float* logits;    // [rows][n_expert]
    uint32_t* sel;
    float* wt;
    int n_expert, k_used, sel_stride;
};

// Router logits: logits[t][r] = sum_i W[r][i] * x[t][i], W f32 or f16 (the one matrix of a
// mixture block that is not quantized).
struct MoeLogitsArgs {
    const void* w;          // [n_expert][k], f32 or f16
    const float* x;         // [ntok][k]
    float* logits;          // [ntok][n_expert]
    int n_expert, k, ntok, f16;
};

// Column activations of a mixture pass: column c reads x[src(c)] (or silu(x[src(c)]) *
// x2[src(c)]) and is quantized like any activation vector: q [ncols][k] int8,
// as [ncols][k/32], s16 [ncols][k/16].
struct MoeQuantArgs {
    const float* x;
    const float* x2;        // null: plain activation
    const uint32_t* src;    // null: column c reads row c
    int8_t* q;
    float* as;
    float* s16;
    int k, per;
    // chunked form (q, as, s16 unused): column c's 256-element chunk i as 88 consecutive words at
    // chunked + (c * k/256 + i) * 88 -- 64 of int8 values, 8 scales, 16 half-block sums -- so a
    // reader addresses everything it needs of a (column, chunk) from one base
    uint32_t* chunked = nullptr;
};

// Grouped expert matvec over columns sorted by expert: out[m][c][0:nrows] =
// bank[m] sheet(expert of c) . column c, columns already quantized (MoeQuantArgs).
struct MoeMatVecArgs {
    float* out[2];
    const uint8_t* bank[2];
    const int8_t* q;
    const float* as;
    const float* s16;
    const uint32_t* start;  // [n_expert + 1]
    size_t sheet_bytes;
    int nrows, k, row_bytes;
    int nwaves;             // wavefronts per workgroup
    int shares;             // workgroups one (expert, matrix) is split into, by rows
};

// The same over banks of packed planes (moe_matvec_planes_body): expert e's planes are
// pqs / pd / psc [m] + e * sheet_words (u32 words; 0 when a bank is ONE plane set), its first
// row e * row_step inside them (0 when every expert has a sheet of its own), pstride rows a
// plane set.
struct MoePlanesArgs {
    float* out[2];
    const uint32_t* pqs[2];
    const uint32_t* pd[2];
    const uint32_t* psc[2];
    const uint32_t* chunked;   // the columns, quantized in the chunked form (MoeQuantArgs.chunked)
    const uint32_t* start;  // [n_expert + 1]
    size_t sheet_words;
    int row_step, pstride;
    int nrows, k;
    int nwaves;             // wavefronts per workgroup: they split the 256-element chunks of K
};

struct MoeCombineArgs {
    float* resid;           // [rows][n_embd], accumulated into
    const float* y;         // [ncols][n_embd]
    const float* wt;        // [rows][k_used]
    const uint32_t* sel;    // [rows][sel_stride]
    const uint32_t* pos;    // [rows*k_used]
    int sel_stride, k_used, n_embd;
};

// MXFP4 weights x bf16 activations: out [ntok][nrows] f32.
// bf16 activations x [ntok][k] -> matrix fragments xf [ceil(k/256) stages][tok_pad/32][16]
// [64 lanes][8 bf16]: fragment ks of a stage holds, for lane 32*kg + t%32, the eight values
// x[t][256*stage + 16*ks + 8*kg ..]; tokens past ntok and K past k are zero.
struct MxPrepArgs {
    const uint16_t* x;
    uint16_t* xf;
    int ntok, tok_pad, k;
};

struct MxGemmArgs {
    float* out;
    const uint8_t* w;     // GGUF row-major MXFP4 blocks (17 bytes per 32)
    const uint16_t* x;    // bf16 bits: [ntok][k] for the matvec, fragment order (MxPrepArgs) for the GEMM
    int tok_pad;          // GEMM: tokens padded to whole tiles of 128
    int nrows, k, ntok;
    int row_bytes;
    int nsplit;           // workgroups along K (grid z); > 1: partial sums go to part
    float* part;          // [nsplit][ntok][nrows], summed by jl_sum_parts
};

// MXFP4 planes x a handful of bf16 tokens: rows row0 .. row0+nrows of planes of `stride` rows.
struct MxPlanesArgs {
    float* out;           // [ntok][nrows]
    const uint32_t* qs;   // [k/32][4][stride]: a block's 16 code bytes, four words
    const uint32_t* d;    // [k/32][ceil(stride/4)]: E8M0 exponent minus one, four rows a word
    const uint32_t* x;    // [ntok][k] bf16 bits, read two a word
    int nrows, k, ntok, row0, stride;
    int nwaves;           // wavefronts of a workgroup; they split the blocks of K
};

// MXFP4 planes x bf16, more than a handful of tokens, the planes read where they lie:
// activation fragments in the planes' K order.
struct MxPlanesPrepArgs {
    const uint16_t* x;    // [ntok][k] bf16 bits
    uint32_t* xa;         // [K-step of 64][token tile of 32][4 matrix K-steps][64 lanes][4 words]
    int ntok, tok_pad, k;
};

struct MxPlanesGemmArgs {
    float* out;           // [ntok][nrows]
    const uint32_t* qs;   // rows row0 .. row0+nrows of planes of `stride` rows
    const uint32_t* d;
    const uint32_t* xa;
    int nrows, k, ntok, tok_pad, row0, stride;
};

// The opt-in block-scaled form: activations as MX fp8 (e4m3 codes, one E8M0 scale a token and
// block of 32) in the operand order of the 32x32x64 scaled matrix instruction.
struct MxScaledPrepArgs {
    const uint16_t* x;    // [ntok][k] bf16 bits
    uint32_t* xa;         // [K-step][token tile][64 lanes][8 words]
    uint8_t* xs;          // [K-step][token tile][64 lanes]
    int ntok, tok_pad, k;
};

struct MxScaledGemmArgs {
    float* out;           // [ntok][nrows]
    const uint32_t* qs;   // MXFP4 planes, rows row0 .. row0+nrows of `stride`
    const uint32_t* d;
    const uint32_t* xa;
    const uint8_t* xs;
    int nrows, k, ntok, tok_pad, row0, stride;
};

// out[i] = part[0][i] + part[1][i] + ... in that order.
struct SumPartsArgs {
    float* out;
    const float* part;
    size_t n;
    int nsplit;
};

// GGUF row-major blocks -> the reference's device planes (and back, for Q4_K).
struct PackArgs {
    const uint8_t* src;   // [nrows][k / block] GGUF blocks
    uint32_t* qs;
    uint32_t* d;
    uint32_t* sc;         // null for formats without a scale plane
    int nrows, k, type;
    uint32_t* flag;       // MXFP4: set to 1 when a block's exponent cannot be stored (else untouched)
};

// Scale range of a Q4_K matrix for the folded-scale GEMM (kernels/gemm_q4k_fold.h).
struct FoldRangeArgs {
    const uint8_t* w;     // GGUF super-blocks, 144 bytes each
    size_t nblocks;
    uint32_t* flag;       // set to 1 when a super-block's weights can pass the f16 range (else untouched)
};

struct UnpackArgs {
    uint8_t* dst;         // [nrows][k/256] Q4_K super-blocks
    const uint32_t* qs;
    const uint32_t* d;
    const uint32_t* sc;
    int nrows, k, row0, stride;
};

// Decode matvec over the planes: rows row0 .. row0+nrows of a buffer of `stride` rows.
struct PackedMatVecArgs {
    float* out;           // [nrows]
    const uint32_t* qs;
    const uint32_t* d;
    const uint32_t* sc;
    const float* x;       // f32 activations (fused quantize) or null
    const int8_t* q;      // pre-quantized activations or null
    const float* as;
    const float* s16;
    int nrows, k, row0, stride;
    int per;              // activation window / 32
    int nwaves;           // wavefronts per workgroup (the launch's block / 64)
    int ngroups;          // workgroups (the launch's grid.x)
    const float* x2;      // gated kernels only: the activation is silu(x) * x2
    float* resid;         // null: none; else resid[r] += alpha * out[r]
    float alpha;
    float* norm_out;      // norm kernels only: null, or where the normed activation goes
    float norm_eps;
};

// Several packed matvecs of one type and shape in one launch, grid = (row groups,
// matrices): matrix y has its own planes and first row (an expert's sheet inside its bank's
// planes: the same plane pointers, row0 = expert * rows) and reads x + y * xstride.
struct PackedMultiArgs {
    float* out[JL_MAX_MULTI];
    const uint32_t* qs[JL_MAX_MULTI];
    const uint32_t* d[JL_MAX_MULTI];
    const uint32_t* sc[JL_MAX_MULTI];
    int row0[JL_MAX_MULTI];
    const float* x;
    const float* x2;      // null: plain activation
    size_t xstride;       // elements
    int nrows, k, stride, per, nwaves, ngroups;
    float* resid;         // null: none; else resid[r] += alpha * out[0][r] (matrix 0 only)
    float alpha;
    const float* resid_gate;    // null, or one logit: the residual weight is alpha * sigmoid(*resid_gate)
    const float* norm_w;  // norm kernels only: RMSNorm weights [k]; every x_j is normed ahead of its quantizer
    float* norm_out;      // null, or where matrix 0's normed activation goes
    float norm_eps;
};
