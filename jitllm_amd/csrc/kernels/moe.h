// Grouped (ragged) expert matmul for a mixture-of-experts block.
//
// The reference routes every row, then works expert-major: gather the rows that
// chose expert e, gate/up GEMMs, act(gate)*up, down GEMM, and add w*y back into
// the row (engine/model/moe.go:697-761); its device twin sorts the (row, slot)
// pairs by expert into columns and runs MUL_MAT_ID-style kernels over the
// sorted columns (jit/gpu/kernels/moesort.go:12-31, moegroup.go:18-68,
// matvec.go:330-343).  Here:
//
//   moe_group      (row, slot) pairs -> columns sorted by expert, pairs in
//                  (row, slot) order inside an expert: start[e], perm[col],
//                  pos[pair]  (jit/gpu/tier/grouppairs_test.go:91-122, unit 1)
//   moe_quant      every column's activation, x[src(c)] or act(gate)*up, quantized
//                  once like any activation vector
//   moe_matvec     for every column c of expert e: out[c] = W_e . column c, the
//                  decode matvec's arithmetic per column.  One workgroup owns
//                  (expert, row share): it stages up to eight of the expert's
//                  quantized columns in LDS and streams the expert's weight rows
//                  once for all of them, so a sheet is read from HBM once however
//                  many rows chose it.
//   moe_combine    resid[r] += sum_s w[r][s] * y[pos[r][s]], experts in ascending
//                  id order as the host path adds them (engine/model/moe.go:127-134)
//
// A weight row is cut into the same slots as the decode matvec; a row takes LPR
// lanes (the next power of two >= slots per row, so K = 2048 uses 32 lanes and a
// wavefront works on two rows, K = 768 uses 16 and four rows).
#pragma once
#include "args.h"
#include "common.h"
#include "matvec.h"
#include "gemm_q4k.h"

// Phase marker for profiling builds; expands to nothing in the product.
#ifndef JL_MOE_TRACE
#define JL_MOE_TRACE(i)
#endif

#define JL_MOE_TB 8  // columns of one expert processed per pass over its rows
#define JL_MOE_U 2   // row groups of 64/LPR rows a wavefront step covers
#define JL_MOE_GROUP_KEYS 16384  // (row, slot) pairs the grouping kernel holds in LDS

// ------------------------------------------------------------------- routing
// One wavefront per row (n_expert <= 1024: sixteen experts a lane).  The reference's
// router (internal/oracle/oracle.go:244-265 Softmax32, moe.go:197-327 with Norm, no bias,
// no groups): exp and the sum in f64, scores narrowed to f32, then k rounds of "largest
// score not yet taken, lowest index on a tie", weights = score / (sum in selection order
// + 1e-20).  The f64 sum is taken as a butterfly over the lanes, so it can differ from the
// reference's sequential sum in its last bit; after narrowing to f32 that moves a score
// only when it sits on a rounding boundary.
// Reductions over the 64 lanes by DPP lane moves (a shuffle through the LDS crossbar costs
// ~100 cycles and the router is a chain of them): quad swaps, the two row mirrors, then
// row broadcasts; lane 63 ends up with the result and it is read back as a scalar.
#define JL_ROUTE_STEPS(STEP)                                                                         \
    STEP(JL_DPP_QUAD_XOR1, 0xf) STEP(JL_DPP_QUAD_XOR2, 0xf) STEP(JL_DPP_ROW_HALF_MIRROR, 0xf)        \
    STEP(JL_DPP_ROW_MIRROR, 0xf) STEP(JL_DPP_ROW_BCAST15, 0xa) STEP(JL_DPP_ROW_BCAST31, 0xc)

__device__ __forceinline__ float route_wave_max(float v) {
    const i32 ninf = __builtin_bit_cast(i32, -__builtin_inff());
#define STEP(C, M) v = fmaxf(v, __builtin_bit_cast(float, dpp_i32<C, M>(ninf, __builtin_bit_cast(i32, v))));
    JL_ROUTE_STEPS(STEP)
#undef STEP
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(i32, v), 63));
}

__device__ __forceinline__ double route_wave_sum(double v) {
#define STEP(C, M)                                                                                   \
    {                                                                                                \
        const uint64_t b = __builtin_bit_cast(uint64_t, v);                                                    \
        const u32 lo = (u32)dpp_i32<C, M>(0, (i32)(u32)b), hi = (u32)dpp_i32<C, M>(0, (i32)(u32)(b >> 32)); \
        v += __builtin_bit_cast(double, ((uint64_t)hi << 32) | lo);                                       \
    }
    JL_ROUTE_STEPS(STEP)
#undef STEP
    const uint64_t b = __builtin_bit_cast(uint64_t, v);
    const u32 lo = (u32)__builtin_amdgcn_readlane((i32)(u32)b, 63), hi = (u32)__builtin_amdgcn_readlane((i32)(u32)(b >> 32), 63);
    return __builtin_bit_cast(double, ((uint64_t)hi << 32) | lo);
}

// (key, index) of the largest key, lowest index on a tie; key = -1 where a lane has none.
__device__ __forceinline__ void route_wave_argmax(i32& key, i32& idx) {
#define STEP(C, M)                                                                                   \
    {                                                                                                \
        const i32 ok = dpp_i32<C, M>(-1, key), oi = dpp_i32<C, M>(0x7fffffff, idx);                  \
        const bool take = ok > key || (ok == key && oi < idx);                                       \
        key = take ? ok : key;                                                                       \
        idx = take ? oi : idx;                                                                       \
    }
    JL_ROUTE_STEPS(STEP)
#undef STEP
    key = __builtin_amdgcn_readlane(key, 63);
    idx = __builtin_amdgcn_readlane(idx, 63);
}

// NG: experts a lane at most (n_expert <= 64 * NG).  The router is one wavefront a row, a dependent
// chain of f64 arithmetic, and every expert slot a lane does not need still costs a clamped load, its
// compares and a skipped branch in each loop: 128 experts in the sixteen-a-lane form 8.1 us, in the
// two-a-lane form 5.6.
template <int NG = 16>
__device__ __forceinline__ void moe_route_body(const MoeRouteArgs& p) {
    const int lane = threadIdx.x & 63, n = p.n_expert;
    const size_t row = blockIdx.x;
    const float* lg = p.logits + row * (size_t)n;
    float v[NG];
    float mx = -__builtin_inff();
#pragma unroll
    for (int i = 0; i < NG; i++) {
        const int e = lane + 64 * i;
        v[i] = e < n ? lg[min(e, n - 1)] : -__builtin_inff();
        if (v[i] > mx) mx = v[i];
    }
    mx = route_wave_max(mx);
    double sum = 0.0;
    float sc[NG];
#pragma unroll
    for (int i = 0; i < NG; i++) {
        const int e = lane + 64 * i;
        double ex = 0.0;
        if (64 * i < n) ex = e < n ? exp((double)v[i] - (double)mx) : 0.0;   // (uniform: whole groups of 64 past n are skipped)
        sc[i] = (float)ex;
        sum += ex;
    }
    sum = route_wave_sum(sum);
    const double inv = 1.0 / sum;
#pragma unroll
    for (int i = 0; i < NG; i++) sc[i] = (float)((double)sc[i] * inv);

    // Scores are >= 0, so their bit patterns order as integers; -1 marks "none".
    i32 prev_key = 0, prev_idx = -1;
    float total = 0.f;
    float chosen = 0.f;   // lane r keeps the r-th selected score
    int found = 0;
    for (int r = 0; r < p.k_used && r < 16; r++) {
        // this lane's best eligible score (index ascending within a lane, so the first
        // of equal values is kept)
        i32 bk = -1, bi = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < NG; i++) {
            if (64 * i >= n) continue;   // uniform
            const int e = lane + 64 * i;
            const float x = sc[i];
            const i32 xk = __builtin_bit_cast(i32, x);
            const bool ok = e < n && x == x && (r == 0 || xk < prev_key || (xk == prev_key && e > prev_idx));
            if (ok && xk > bk) { bk = xk; bi = e; }
        }
        route_wave_argmax(bk, bi);
        if (bi == 0x7fffffff) break;
        if (lane == 0) p.sel[row * p.sel_stride + r] = (u32)bi;
        const float bv = __builtin_bit_cast(float, bk);
        if (lane == r) chosen = bv;
        total = total + bv;          // selection order, as the reference adds them
        prev_key = bk;
        prev_idx = bi;
        found = r + 1;
    }
    total = total + 1e-20f;
    if (lane < found) p.wt[row * p.k_used + lane] = chosen / total;
}

// ------------------------------------------------------------------ grouping
// A stable counting sort of the (row, slot) pairs by expert in one workgroup of 1024
// threads.  The threads form NSEG segments x NEXP experts (NEXP = n_expert rounded up
// to a power of two): thread (seg, e) counts expert e's pairs in its contiguous segment
// of the pair list, a prefix over (e, seg) turns counts into first columns, and the
// same thread then walks its segment again handing out columns in order.  No atomics,
// so inside an expert the order is (row, slot).
__device__ __forceinline__ void moe_group_body(const MoeGroupArgs& p, u32* scount, uint16_t* skeys) {
    const int npairs = p.rows * p.k_used;
    int nexp = 1;
    while (nexp < p.n_expert) nexp <<= 1;
    const int nseg = 1024 / nexp;
    const int e = threadIdx.x & (nexp - 1), seg = threadIdx.x / nexp;
    // segments are whole groups of eight pairs so the staged keys are read eight at a time
    const int per_seg = ((npairs + nseg - 1) / nseg + 7) & ~7;
    const int lo = min(seg * per_seg, npairs), hi = min(lo + per_seg, npairs);
    auto key_global = [&](int i) { return p.sel[(i / p.k_used) * p.sel_stride + i % p.k_used]; };
    // the pair list is walked twice by every segment: keep it in LDS when it fits
    // (padded to a multiple of eight with an id no expert has)
    const bool staged = npairs <= JL_MOE_GROUP_KEYS;
    if (staged) {
        const int padded = (npairs + 7) & ~7;
        for (int i = threadIdx.x; i < padded; i += 1024)
            skeys[i] = i < npairs ? (uint16_t)min(key_global(i), 0xFFFFu) : (uint16_t)0xFFFF;
        __syncthreads();
    }
    typedef uint16_t u16x8 __attribute__((ext_vector_type(8)));
    u32 cnt = 0;
    if (e < p.n_expert) {
        if (staged) {
            for (int i = lo; i < hi; i += 8) {
                const u16x8 v = *(const u16x8*)(skeys + i);
#pragma unroll
                for (int b = 0; b < 8; b++) cnt += v[b] == (uint16_t)e;
            }
        } else {
            for (int i = lo; i < hi; i++) cnt += key_global(i) == (u32)e;
        }
    }
    // Inclusive scan of the 1024 counts laid out expert-major (so a running sum is the
    // column order): the counts change places through LDS, every wavefront scans its 64 with
    // lane moves, and the sixteen wavefront totals are added up by whoever needs them.
    const int me = e * nseg + seg;
    u32* src = scount;            // [1024] counts in scan order, then the scanned values
    u32* tot = scount + 1024;     // [16] wavefront totals
    src[me] = cnt;
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    u32 v = src[threadIdx.x];
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const u32 o = __shfl_up(v, off, 64);
        if (lane >= off) v += o;
    }
    if (lane == 63) tot[wave] = v;
    __syncthreads();
    for (int w = 0; w < wave; w++) v += tot[w];
    src[threadIdx.x] = v;
    __syncthreads();
    const u32 before = src[me] - cnt;
    if (e < p.n_expert) {
        if (seg == 0) p.start[e] = before;
        if (e == p.n_expert - 1 && seg == nseg - 1) p.start[p.n_expert] = before + cnt;
        u32 col = before;
        auto place = [&](int i) {
            p.perm[col] = (u32)(i / p.k_used);
            p.pos[i] = col;
            col++;
        };
        if (staged) {
            for (int i = lo; i < hi; i += 8) {
                const u16x8 v = *(const u16x8*)(skeys + i);
#pragma unroll
                for (int b = 0; b < 8; b++)
                    if (v[b] == (uint16_t)e) place(i + b);
            }
        } else {
            for (int i = lo; i < hi; i++)
                if (key_global(i) == (u32)e) place(i);
        }
    }
}

// The same sort in time linear in the pairs (the form above compares every pair with every
// expert, all on one CU: 11 us at 512 pairs and 128 experts, 234 us at 16,384 pairs).  The
// pair list is cut into sixteen contiguous shares, one per wavefront, walked in runs of 64.
// Inside a run every lane finds the lanes that hold its expert with one ballot per bit of the
// expert id, which gives its rank among them and their number; the share's running count of
// the expert (an LDS table the wavefront owns, so its accesses execute in order) gives the
// pairs before the run.  A thread per expert then turns the sixteen share counts into offsets,
// the expert totals are scanned, and a pair's column is its expert's first column + the
// expert's pairs in earlier shares + its rank in its own share: (row, slot) order inside an
// expert, no atomics.  The rank waits in pos[] between the passes (the same thread writes
// and reads it).  grid = 1, block = 1024, dynamic LDS = JL_MOE_GROUP2_LDS(nexp).
#define JL_MOE_GROUP2_LDS(nexp) (16 * (nexp) * 2 + ((nexp) + 1 + 16) * 4)
// CNT: the type of a share's per-expert counts and of their running sums over the sixteen
// shares: uint16_t while the whole pair list has at most 65535 pairs (no sum can pass that),
// u32 above.  Dynamic LDS = 16 * nexp * sizeof(CNT) + (nexp + 17) * 4.
template <typename CNT>
__device__ __forceinline__ void moe_group2_body(const MoeGroupArgs& p, uint8_t* smem) {
    const int npairs = p.rows * p.k_used, nexp = p.n_expert;
    const int nruns = (npairs + 63) / 64, runs_per = (nruns + 15) / 16;
    CNT* scnt = (CNT*)smem;                                            // [16][nexp]
    u32* sstart = (u32*)(scnt + 16 * nexp);                            // [nexp + 1]
    u32* stot = sstart + nexp + 1;                                     // [16] wavefront totals
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int nbits = 0;
    while ((1 << nbits) < nexp) nbits++;
    for (int i = tid; i < 16 * nexp; i += 1024) scnt[i] = 0;
    __syncthreads();
    const uint64_t lt = lane ? (~0ull >> (64 - lane)) : 0ull;   // lanes below this one
    CNT* mine = scnt + wave * nexp;
    const int run_lo = min(wave * runs_per, nruns), run_hi = min(run_lo + runs_per, nruns);
    auto key_of = [&](int i) { return p.sel[(i / p.k_used) * p.sel_stride + i % p.k_used]; };
    for (int run = run_lo; run < run_hi; run++) {
        const int i = run * 64 + lane;
        u32 e = 0;
        bool valid = i < npairs;
        if (valid) {
            e = key_of(i);
            valid = e < (u32)nexp;   // an id no expert has: the pair is left out, as in the form above
        }
        uint64_t m = __ballot(valid);
        for (int b = 0; b < nbits; b++) {
            const bool bit = (e >> b) & 1;
            const uint64_t bal = __ballot(bit);
            m &= bit ? bal : ~bal;
        }
        if (valid) {
            const u32 before = mine[e];
            p.pos[i] = before + (u32)__builtin_popcountll(m & lt);
            if ((m & lt) == 0) mine[e] = (CNT)(before + (u32)__builtin_popcountll(m));
        }
    }
    __syncthreads();
    // per expert: counts of successive shares -> pairs in earlier shares; the total goes to the scan
    u32 total = 0;
    if (tid < nexp) {
#pragma unroll
        for (int w = 0; w < 16; w++) {
            const u32 c = scnt[w * nexp + tid];
            scnt[w * nexp + tid] = (CNT)total;
            total += c;
        }
    }
    // exclusive scan of the totals over experts (thread = expert; nexp <= 1024)
    u32 v = total;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const u32 o = __shfl_up(v, off, 64);
        if (lane >= off) v += o;
    }
    if (lane == 63) stot[wave] = v;
    __syncthreads();
    for (int w = 0; w < wave; w++) v += stot[w];
    if (tid < nexp) {
        sstart[tid] = v - total;
        p.start[tid] = v - total;
        if (tid == nexp - 1) p.start[nexp] = v;
    }
    __syncthreads();
    for (int run = run_lo; run < run_hi; run++) {
        const int i = run * 64 + lane;
        if (i >= npairs) continue;
        const u32 e = key_of(i);
        if (e >= (u32)nexp) continue;
        const u32 col = sstart[e] + mine[e] + p.pos[i];
        p.perm[col] = (u32)(i / p.k_used);
        p.pos[i] = col;
    }
}

// Sum over the LPR consecutive lanes of a row group (LPR = 16, 32 or 64); the
// total is valid in the group's last lane.
template <int LPR>
__device__ __forceinline__ float group_sum(float v) {
    v += dpp_f32<JL_DPP_QUAD_XOR1, 0xf>(v);
    v += dpp_f32<JL_DPP_QUAD_XOR2, 0xf>(v);
    if (LPR >= 8) v += dpp_f32<JL_DPP_ROW_HALF_MIRROR, 0xf>(v);
    if (LPR >= 16) v += dpp_f32<JL_DPP_ROW_MIRROR, 0xf>(v);
    if (LPR >= 32) v += dpp_f32<JL_DPP_ROW_BCAST15, 0xa>(v);
    if (LPR >= 64) v += dpp_f32<JL_DPP_ROW_BCAST31, 0xc>(v);
    return v;
}

// ------------------------------------------------- grouped matvec, packed planes
// The dot-product form over banks of packed planes, for a handful of columns an expert (a small
// prefill batch through a mixture: 64 rows top-8 of 128 experts is four columns an expert).
// The planes put a word of one row beside the same word of the next row, so rows go on LANES:
// a workgroup owns 64 rows of one expert's sheet, its wavefronts split K in chunks of 256
// elements (one super-block), and a lane loads its row's share of a chunk -- 32 words of
// nibbles, three of scales, one of (d, dmin), every load 256 contiguous bytes a wavefront --
// exactly once, whatever the number of columns.  The chunk's scale arithmetic is done once;
// then the expert's columns pass by, eight at a time.  A column's int8 values, scales and sums
// are the SAME for every lane of the wavefront (all lanes work on the same chunk), so they are
// read through the scalar cache into scalar registers and meet the weights as scalar operands
// of the dot instructions: no LDS traffic, no staging, no barrier inside the loop.  The column
// quantizer lays a (column, chunk) out as 88 consecutive words for this reader
// (MoeQuantArgs.chunked), read as 32-bit words and bit-cast: the kernel stores floats, and a
// float load that a float store might alias would not be made a scalar load.  The wavefronts'
// partial sums meet in LDS at the end and are added in wavefront order.
// (A form with one wavefront a workgroup walking all of K, its scalar loads pipelined by hand,
// measured 2.1x slower at the 128-expert shape: few, long wavefronts expose every scalar
// round trip, many short ones cover each other.)
// Q4_K.  grid = (ceil(nrows/64), n_expert, matrices), block = 64 * nwaves (<= 8),
// dynamic LDS = nwaves * JL_MOEP_TB * 64 * 4.
#define JL_MOEP_TB 8   // columns a pass

__device__ __forceinline__ void moe_matvec_planes_body(const MoePlanesArgs& p, uint8_t* smem) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), nwaves = p.nwaves;
    const int e = blockIdx.y, mat = blockIdx.z;
    // (the same in every lane: in scalar registers, so that what depends on them is scalar too)
    const u32 c_lo = (u32)__builtin_amdgcn_readfirstlane((int)p.start[e]);
    const u32 c_hi = (u32)__builtin_amdgcn_readfirstlane((int)p.start[e + 1]);
    if (c_lo == c_hi) return;   // nobody chose this expert (uniform across the workgroup)
    const int r_l = blockIdx.x * 64 + lane;
    const size_t st = (size_t)p.pstride;
    const size_t row = (size_t)e * p.row_step + min(r_l, p.nrows - 1);
    const size_t ew = (size_t)e * p.sheet_words;
    const u32* pqs = p.pqs[mat] + ew + row;
    const u32* pd = p.pd[mat] + ew + row;
    const u32* psc = p.psc[mat] + ew + row;
    float* red = (float*)smem;   // [nwaves][JL_MOEP_TB][64]
    const int nchunks = p.k / 256;
    const u32 M = 0x0F0F0F0Fu;

    for (u32 c0 = c_lo; c0 < c_hi; c0 += JL_MOEP_TB) {
        const int ncol = (int)min((u32)JL_MOEP_TB, c_hi - c0);   // uniform
        float acc[JL_MOEP_TB];
#pragma unroll
        for (int j = 0; j < JL_MOEP_TB; j++) acc[j] = 0.f;
        for (int c = wave; c < nchunks; c += nwaves) {
            // this row's chunk: (d, dmin), the 96-bit stream of 6-bit scales and minimums, 8 x 4 words
            const u32 dw = pd[(size_t)c * st];
            const u32 s0 = psc[(size_t)(3 * c) * st], s1 = psc[(size_t)(3 * c + 1) * st], s2 = psc[(size_t)(3 * c + 2) * st];
            u32 wq[8][4];
#pragma unroll
            for (int s = 0; s < 8; s++)
#pragma unroll
                for (int w = 0; w < 4; w++) wq[s][w] = pqs[(size_t)((c * 8 + s) * 4 + w) * st];
            const float d = half_bits_to_f32((uint16_t)(dw & 0xFFFF)), dmin = half_bits_to_f32((uint16_t)(dw >> 16));
            const uint64_t lo = s0 | ((uint64_t)s1 << 32), hi = s1 | ((uint64_t)s2 << 32);
            float dsc[8], dm[8];
#pragma unroll
            for (int s = 0; s < 8; s++) {
                const int bit = 12 * s;
                const u32 f = bit < 32 ? (u32)(lo >> bit) : (u32)(hi >> (bit - 32));
                dsc[s] = d * (float)(f & 63);
                dm[s] = dmin * (float)((f >> 6) & 63);
            }
#pragma unroll
            for (int j = 0; j < JL_MOEP_TB; j++) {
                if (j < ncol) {   // uniform
                    // column c0 + j, chunk c: the same address in every lane -> scalar loads, one
                    // base and immediate offsets
                    const u32* cb = p.chunked + ((size_t)(c0 + j) * nchunks + c) * 88;
                    float t = acc[j];
#pragma unroll
                    for (int s = 0; s < 8; s++) {
                        i32 dt = 0;
#pragma unroll
                        for (int w = 0; w < 4; w++) {
                            dt = dot4(wq[s][w] & M, cb[8 * s + w], dt);
                            dt = dot4((wq[s][w] >> 4) & M, cb[8 * s + 4 + w], dt);
                        }
                        const float sa = __uint_as_float(cb[72 + 2 * s]) + __uint_as_float(cb[73 + 2 * s]);
                        const float v = (float)dt * dsc[s] - sa * dm[s];
                        t = fmaf(v, __uint_as_float(cb[64 + s]), t);
                    }
                    acc[j] = t;
                }
            }
        }
        // the wavefronts' shares of K meet in LDS and are added in wavefront order
#pragma unroll
        for (int j = 0; j < JL_MOEP_TB; j++) red[(wave * JL_MOEP_TB + j) * 64 + lane] = acc[j];
        __syncthreads();
        for (int i = threadIdx.x; i < ncol * 64; i += nwaves * 64) {
            const int j = i >> 6, l = i & 63;
            float sum = red[j * 64 + l];
            for (int w = 1; w < nwaves; w++) sum += red[(w * JL_MOEP_TB + j) * 64 + l];
            const int r = blockIdx.x * 64 + l;
            if (r < p.nrows) p.out[mat][(size_t)(c0 + j) * p.nrows + r] = sum;
        }
        __syncthreads();   // red is free for the next pass
    }
}

// --------------------------------------------------------- column activations
// grid = (ceil(k/4/256), ncols), block = 256: one thread per four elements of a column.
__device__ __forceinline__ void moe_quant_body(const MoeQuantArgs& p) {
    const size_t c = blockIdx.y;
    const size_t src = p.src ? p.src[c] : c;
    const int g4 = blockIdx.x * 256 + threadIdx.x;
    const bool live = g4 < p.k / 4;
    f32x4 v = f32x4{0.f, 0.f, 0.f, 0.f};
    if (live) {
        v = ((const f32x4*)(p.x + src * (size_t)p.k))[g4];
        if (p.x2) {
            f32x4 u = ((const f32x4*)(p.x2 + src * (size_t)p.k))[g4];
            v = f32x4{silu_f32(v.x) * u.x, silu_f32(v.y) * u.y, silu_f32(v.z) * u.z, silu_f32(v.w) * u.w};
        }
    }
    u32 m = max(max(abs_bits(v.x), abs_bits(v.y)), max(abs_bits(v.z), abs_bits(v.w)));
    u32 amax = window_amax(live ? m : 0u, p.per);
    float d;
    i32 sum;
    u32 qq = quantize4(v, amax, d, sum);
    if (live && p.chunked) {
        const int within = g4 & 63;
        u32* cb = p.chunked + (c * (size_t)(p.k / 256) + (size_t)(g4 >> 6)) * 88;
        cb[within] = qq;
        if ((g4 & 3) == 0) cb[72 + (within >> 2)] = __float_as_uint((float)sum);
        if ((g4 & 7) == 0) cb[64 + (within >> 3)] = __float_as_uint(d);
    } else if (live) {
        ((u32*)(p.q + c * (size_t)p.k))[g4] = qq;
        if ((g4 & 3) == 0) p.s16[c * (size_t)(p.k / 16) + (g4 >> 2)] = (float)sum;
        if ((g4 & 7) == 0) p.as[c * (size_t)(p.k / 32) + (g4 >> 3)] = d;
    }
}

// ------------------------------------------------------------- grouped matvec
// grid = (shares, n_expert, matrices), block = nwaves * 64, dynamic LDS = JL_MOE_TB
// staged columns.  A workgroup owns (expert, matrix, row share).  It copies up to eight
// of the expert's quantized columns into LDS and streams its rows once for all of them.
// A wavefront works in steps of 64/LPR rows (one slot per lane): it decodes the step's
// scales and nibbles once, meets every staged column with them, and has the next step's
// loads in flight meanwhile.  k % 256 == 0.
template <int TYPE, int LPR>
__device__ __forceinline__ void moe_matvec_body(const MoeMatVecArgs& p, uint8_t* smem) {
    typedef SlotTraits<TYPE> T;
    constexpr int RW = 64 / LPR, U = JL_MOE_U;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = p.nwaves;
    const int nthreads = nwaves * 64;
    const int e = blockIdx.y, mat = blockIdx.z;
    JL_MOE_TRACE(0);
    const u32 c_lo = p.start[e], c_hi = p.start[e + 1];
    if (c_lo == c_hi) return;  // nobody chose this expert (uniform across the workgroup)
    JL_MOE_TRACE(1);
    const int nslots = p.k / T::kElems;
    const int slot = lane % LPR, rw = lane / LPR;
    const int share = (p.nrows + p.shares - 1) / p.shares;
    const int row_lo = blockIdx.x * share, row_hi = min(row_lo + share, p.nrows);
    if (row_lo >= row_hi) return;
    const uint8_t* sheet = p.bank[mat] + (size_t)e * p.sheet_bytes;
    float* out = p.out[mat];
    const int act_bytes = (JL_ACT_LDS_BYTES(p.k) + 15) & ~15;
    // steps of this wavefront: row groups (U * RW rows, stride nwaves of them) x slot groups
    const int nsl = (nslots + LPR - 1) / LPR;
    const int ngroups = (row_hi - row_lo - wave * U * RW + nwaves * U * RW - 1) / (nwaves * U * RW);  // may be <= 0
    const int nsteps = max(ngroups, 0) * nsl;
    // step it = (row group it / nsl, slot group it % nsl); the pair is carried along the loop
    const int row_first = row_lo + wave * U * RW + rw, row_stride = nwaves * U * RW;
    auto load_step = [&](int row0, int sg, typename T::W (&w)[U]) {
        const int s = min(slot + sg * LPR, nslots - 1);
#pragma unroll
        for (int u = 0; u < U; u++)
            T::load_w(sheet + (size_t)min(row0 + u * RW, row_hi - 1) * p.row_bytes, s, w[u]);
    };

    typename T::W w_next[U];

    for (u32 c0 = c_lo; c0 < c_hi; c0 += JL_MOE_TB) {
        const int ncol = min((u32)JL_MOE_TB, c_hi - c0);
        // stage the pass's columns: int8 values, scales and sums, 16 bytes at a time
        {
            const int nq = p.k / 16, na = p.k / 128, ns = p.k / 64, per_col = nq + na + ns;
            for (int i = threadIdx.x; i < ncol * per_col; i += nthreads) {
                const int j = i / per_col, o = i - j * per_col;
                const size_t c = c0 + j;
                u32x4* dst = (u32x4*)(smem + (size_t)j * act_bytes);
                if (o < nq) {
                    dst[o] = ((const u32x4*)(p.q + c * (size_t)p.k))[o];
                } else if (o < nq + na) {
                    ((u32x4*)((uint8_t*)dst + p.k))[o - nq] = ((const u32x4*)(p.as + c * (size_t)(p.k / 32)))[o - nq];
                } else {
                    ((u32x4*)((uint8_t*)dst + p.k + (p.k / 32) * 4))[o - nq - na] =
                        ((const u32x4*)(p.s16 + c * (size_t)(p.k / 16)))[o - nq - na];
                }
            }
        }
        // the first step's weights are requested behind the staging loads (loads are served
        // in order) and stay in flight across the barrier, which orders LDS only
        if (nsteps > 0) load_step(row_first, 0, w_next);
        lds_barrier();
        JL_MOE_TRACE(2);
        float acc[JL_MOE_TB][U];
#pragma unroll
        for (int j = 0; j < JL_MOE_TB; j++)
#pragma unroll
            for (int u = 0; u < U; u++) acc[j][u] = 0.f;
        int row0 = row_first, sg = 0;   // this step's first row of the lane and its slot group
        for (int it = 0; it < nsteps; it++) {
            typename T::Prep P[U];
            const int s = slot + sg * LPR, sc = min(s, nslots - 1);
            const bool live = s < nslots;
            const bool last_sg = sg == nsl - 1;
            const int row_n = last_sg ? row0 + row_stride : row0, sg_n = last_sg ? 0 : sg + 1;
#pragma unroll
            for (int u = 0; u < U; u++) T::prep(w_next[u], sc, P[u]);
            if (it + 1 < nsteps) load_step(row_n, sg_n, w_next);
#pragma unroll
            for (int j = 0; j < JL_MOE_TB; j++) {
                if (j < ncol) {
                    typename T::Act a;
                    T::load_act(act_lds_views(smem + (size_t)j * act_bytes, p.k), sc, a);
#pragma unroll
                    for (int u = 0; u < U; u++) {
                        const float v = T::dotp(P[u], a);
                        acc[j][u] += live ? v : 0.f;
                    }
                }
                // one column's activation in registers at a time
                asm volatile("" ::: "memory");
                __builtin_amdgcn_sched_barrier(0);
            }
            if (last_sg) {  // the rows' last slot group: reduce and store
#pragma unroll
                for (int j = 0; j < JL_MOE_TB; j++)
#pragma unroll
                    for (int u = 0; u < U; u++) {
                        if (j < ncol) {
                            const int r = row0 + u * RW;
                            float t = group_sum<LPR>(acc[j][u]);
                            if (slot == LPR - 1 && r < row_hi) out[(size_t)(c0 + j) * p.nrows + r] = t;
                        }
                        acc[j][u] = 0.f;
                    }
            }
            row0 = row_n;
            sg = sg_n;
        }
        JL_MOE_TRACE(3);
        __syncthreads();
    }
    JL_MOE_TRACE(4);
}

// ------------------------------------------------- grouped matmul on the matrix cores
// The dot-product kernel above pays for every (weight, column) pair in vector instructions.
// With Q4_K weights and the k-quant activation window the prefill GEMM's exact f16
// arithmetic applies (gemm_q4k.h): a group of up to 32 of an expert's columns is one
// matrix operand, and the vector work is the dequantization alone, whatever the group holds.
//
// Work list: grid = 1, block = 1024.  Expert e owns the slots from start[e]/32 + e up to the
// next expert's first; the leading ceil(columns / 32) of them are its groups, the rest stay
// unused, so every slot is written exactly once.  The 128-column tiles are numbered by a
// running sum over the experts (wavefront scans, wavefront totals through LDS).
__device__ __forceinline__ void moe_worklist_body(const MoeWorklistArgs& p, u32* tot) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    u32* slot_e = p.wl + 4;
    u32* tiles = p.wl + 4 + p.nslots;
    u32 base = 0;
    for (int e0 = 0; e0 < p.n_expert; e0 += 1024) {
        const int e = e0 + (int)threadIdx.x;
        u32 nt = 0, c_lo = 0, ncol = 0;
        if (e < p.n_expert) {
            c_lo = p.start[e];
            const u32 c_hi = p.start[e + 1];
            ncol = c_hi - c_lo;
            nt = (ncol + 127) >> 7;
            const u32 s0 = (c_lo >> 5) + (u32)e, ng = (ncol + 31) >> 5;
            const u32 s1 = e + 1 < p.n_expert ? (c_hi >> 5) + (u32)e + 1 : (u32)p.nslots;
            for (u32 s = s0; s < s1; s++) slot_e[s] = s - s0 < ng ? (u32)e : 0xFFFFFFFFu;
        }
        u32 v = nt;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const u32 o = __shfl_up(v, off, 64);
            if (lane >= off) v += o;
        }
        __syncthreads();   // the totals of the previous round have been read
        if (lane == 63) tot[wave] = v;
        __syncthreads();
        u32 round = 0;
        for (int w = 0; w < 16; w++) {
            if (w < wave) v += tot[w];
            round += tot[w];
        }
        const u32 first = base + v - nt;
        for (u32 j = 0; j < nt; j++) tiles[first + j] = (u32)e | (j << 16);
        base += round;
    }
    if (threadIdx.x == 0) p.wl[0] = base;
}

// Activation prep: grid = (k/256, nslots), block = 256: one group of 32 columns, one
// super-block; tokens past the expert's last column are zeros.
// PL: the K order of the plane-reading tile kernel (gemm_q4k.h).
template <bool PL = false>
__device__ __forceinline__ void moe_gemm_prep_body(const MoeGemmPrepArgs& p, u32* lds) {
    const int lane = threadIdx.x & 63;
    const int sb = blockIdx.x, slot = blockIdx.y;
    const u32 eu = p.wl[4 + slot];
    if (eu == 0xFFFFFFFFu) return;   // uniform across the workgroup
    const int e = (int)eu;
    const u32 c_lo = p.start[e], c_hi = p.start[e + 1];
    const u32 c0 = c_lo + 32 * (u32)(slot - ((int)(c_lo >> 5) + e));
    gemm_prep_group<4, PL>(lds, sb, slot, p.nslots, p.bq, p.da, [&](int tl) {
        f32x4 v = f32x4{0.f, 0.f, 0.f, 0.f};
        const u32 c = c0 + tl;
        if (c < c_hi) {
            const size_t row = p.src ? p.src[c] : c;
            v = ((const f32x4*)(p.x + row * (size_t)p.k + (size_t)sb * 256))[lane];
            if (p.x2) {
                const f32x4 u = ((const f32x4*)(p.x2 + row * (size_t)p.k + (size_t)sb * 256))[lane];
                v = f32x4{silu_f32(v.x) * u.x, silu_f32(v.y) * u.y, silu_f32(v.z) * u.z, silu_f32(v.w) * u.w};
            }
        }
        return v;
    });
}

// Matrix kernel: grid = (ceil(nrows/256), nslots, matrices), block = 256, dynamic
// LDS = 4 * JL_MOEG_WAVE_LDS.  A wavefront owns 32 columns x 64 rows and shares nothing
// with its neighbours -- the columns are the same for the whole workgroup, the rows are its
// own -- so it keeps a private LDS buffer to turn its dequantized weights into matrix
// fragments and no workgroup barrier is needed: LDS operations of one wavefront execute in
// order.  Per stage (half a super-block) it dequantizes 64 rows x 128 weights (lane =
// (row%16, 16-byte chunk), four rows a lane), then runs 16 matrix instructions against the
// group's activation fragments, which come from the workspace into a register ring a stage
// ahead; the weights of the next stage are in flight in registers meanwhile.  Two
// workgroups share a CU and cover each other's vector phases.
#define JL_MOEG_WROW 136   // f16 per weight row: 128 + 8 (272 B: rows advance four banks)
#define JL_MOEG_MROW 16    // f16 per row of minimum columns
#define JL_MOEG_WAVE_LDS (64 * JL_MOEG_WROW * 2 + 64 * JL_MOEG_MROW * 2 + 64 * 2 * 4)

__device__ __forceinline__ void moe_gemm_q4k_body(const MoeGemmArgs& p, uint8_t* smem) {
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int slot = blockIdx.y, mat = blockIdx.z;
    const u32 eu = p.wl[4 + slot];
    if (eu == 0xFFFFFFFFu) return;
    const int e = (int)eu;
    const u32 c_lo = p.start[e], c_hi = p.start[e + 1];
    const u32 c0 = c_lo + 32 * (u32)(slot - ((int)(c_lo >> 5) + e));
    const int ncol = min(32, (int)(c_hi - c0));
    const int r0 = blockIdx.x * 256 + wave * 64;
    if (r0 >= p.nrows) return;   // (no workgroup barrier below)
    _Float16* sW = (_Float16*)(smem + (size_t)wave * JL_MOEG_WAVE_LDS);
    _Float16* sMin = sW + 64 * JL_MOEG_WROW;
    float* sSc = (float*)(sMin + 64 * JL_MOEG_MROW);

    const int nsb = p.k / 256, nsteps = 2 * nsb;
    const int arow = lane & 31, kg = lane >> 5;
    const int drow = lane >> 2, chunk = lane & 3, hh = chunk >> 1, wq_ = chunk & 1;
    // weights: uniform base + 32-bit lane offsets, rows clamped to the sheet
    const uint8_t* sheet = p.bank[mat] + (size_t)e * p.sheet_bytes;
    unsigned woff[4];
#pragma unroll
    for (int i = 0; i < 4; i++) woff[i] = (unsigned)min(r0 + 16 * i + drow, p.nrows - 1) * (unsigned)p.row_bytes;
    // activation fragment (step, ks) of the group: uniform base + lane
    const size_t astride = (size_t)p.nslots * (JL_GEMM_ASTAGE_FRAGS * 1024);
    const char* abase = (const char*)p.bq + (size_t)slot * (JL_GEMM_ASTAGE_FRAGS * 1024);
    const unsigned aoff = lane * 16;
    auto a_frag = [&](int step, int ks) {
        return *(const f16x8*)(abase + (size_t)step * astride + ks * 1024 + aoff);
    };
    const float* dabase = p.da + (size_t)slot * 32 + 4 * kg;
    u32 mask_lo = 0x000F000Fu, mask_hi = 0x00F000F0u, magic = 0x64006400u;
    asm volatile("" : "+v"(mask_lo), "+v"(mask_hi), "+v"(magic));

    f32x16 out[2], accP[2];
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
        for (int el = 0; el < 16; el++) out[j][el] = 0.f;

    // Weights are streamed once from HBM and a stage is short, so their loads run three
    // stages ahead (four register sets in rotation) and the block headers a whole
    // super-block ahead: one stage of lookahead is less than the memory latency under load.
    u32x4 hdr[2][4], wq[4][4];
    f16x8 aring[8], aaug;
    auto load_hdr = [&](int sb, u32x4 (&h)[4]) {
#pragma unroll
        for (int i = 0; i < 4; i++) h[i] = ld16(sheet + (size_t)sb * 144 + woff[i]);
    };
    auto load_q = [&](int step, u32x4 (&q)[4]) {
        const uint8_t* b = sheet + (size_t)(step >> 1) * 144 + 16 + 64 * (step & 1) + 16 * chunk;
#pragma unroll
        for (int i = 0; i < 4; i++) q[i] = ld16(b + woff[i]);
    };
    load_hdr(0, hdr[0]);
    load_q(0, wq[0]);
    load_q(min(1, nsteps - 1), wq[1]);
    load_q(min(2, nsteps - 1), wq[2]);
    load_hdr(min(1, nsb - 1), hdr[1]);
#pragma unroll
    for (int ks = 0; ks < 8; ks++) aring[ks] = a_frag(0, ks);
    aaug = a_frag(1, 8);

    // STEP4 = step % 4 names the register sets: weights wq[STEP4], headers hdr[(STEP4 / 2)]
    auto stage = [&](auto STEP4, int step) {
        constexpr int s4 = decltype(STEP4)::value, half = s4 & 1, hs = s4 >> 1;
        const int sb = step >> 1;
        const int nstep = min(step + 1, nsteps - 1);
        load_q(min(step + 3, nsteps - 1), wq[(s4 + 3) & 3]);
        // dequantize this stage into the wavefront's buffer
#pragma unroll
        for (int i = 0; i < 4; i++) {
            GemmWideScale sc;
            gemm_wide_scale(hdr[hs][i], hh, half, sc);
            sc.dst = sW + (16 * i + drow) * JL_MOEG_WROW + 64 * hh + 32 * wq_;
#pragma unroll
            for (int c = 0; c < 4; c++) gemm_wide_word(wq[s4][i][c], sc, c, mask_lo, mask_hi, magic);
            if (half == 0) {
                // the super-block's minimum columns (even chunks: m_s, odd: 64 m_s) and (d, dmin);
                // lanes that share an address store the same value
                const GemmScaleBytes sbytes = gemm_scale_bytes(hdr[hs][i].y, hdr[hs][i].z, hdr[hs][i].w);
                const float mul = wq_ ? 64.0f : 1.0f;
                f16x8 mm;
#pragma unroll
                for (int b = 0; b < 4; b++) {
                    mm[b] = (_Float16)((float)((sbytes.mn_lo >> (8 * b)) & 0xFF) * mul);
                    mm[4 + b] = (_Float16)((float)((sbytes.mn_hi >> (8 * b)) & 0xFF) * mul);
                }
                *(f16x8*)(sMin + (16 * i + drow) * JL_MOEG_MROW + 8 * wq_) = mm;
                float2 dd = {half_bits_to_f32((uint16_t)(hdr[hs][i].x & 0xFFFF)),
                             half_bits_to_f32((uint16_t)(hdr[hs][i].x >> 16))};
                *(float2*)(sSc + 2 * (16 * i + drow)) = dd;
            }
        }
        // this super-block's headers are done with after its second half: fetch those of the
        // super-block after next into their place
        if (half == 1) load_hdr(min(sb + 2, nsb - 1), hdr[hs]);
        // matrix work: fragments a K-step ahead; the ring slot is refilled for the next stage
        f32x4 dav[4];
        if (half == 1) {   // the group's token scales, for the epilogue below
#pragma unroll
            for (int i = 0; i < 4; i++) dav[i] = *(const f32x4*)(dabase + (size_t)sb * (32 * p.nslots) + 8 * i);
        }
        const _Float16* wp0 = sW + arow * JL_MOEG_WROW + 8 * kg;
        f16x8 wf[2][2];
#pragma unroll
        for (int j = 0; j < 2; j++) wf[0][j] = *(const f16x8*)(wp0 + 32 * j * JL_MOEG_WROW);
#pragma unroll
        for (int ks = 0; ks < 8; ks++) {
            if (ks + 1 < 8) {
#pragma unroll
                for (int j = 0; j < 2; j++)
                    wf[(ks + 1) & 1][j] = *(const f16x8*)(wp0 + 32 * j * JL_MOEG_WROW + 16 * (ks + 1));
            }
            const f32x16 czero = {0};
#pragma unroll
            for (int j = 0; j < 2; j++)
                accP[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(aring[ks], wf[ks & 1][j],
                                                                 (half == 0 && ks == 0) ? czero : accP[j], 0, 0, 0);
            aring[ks] = a_frag(nstep, ks);
        }
        if (half == 1) {
            // out += d_a * (d * P - dmin * M) for the super-block
            const f32x16 czero = {0};
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const f16x8 wm = *(const f16x8*)(sMin + (32 * j + arow) * JL_MOEG_MROW + 8 * kg);
                const float2 esc = *(const float2*)(sSc + 2 * (32 * j + arow));
                const f32x16 accM = __builtin_amdgcn_mfma_f32_32x32x16_f16(aaug, wm, czero, 0, 0, 0);
#pragma unroll
                for (int el = 0; el < 16; el++) {
                    const float u = fmaf(esc.x, accP[j][el], -(esc.y * accM[el]));
                    out[j][el] = fmaf(dav[el >> 2][el & 3], u, out[j][el]);
                }
            }
            aaug = a_frag(min(step + 2, nsteps - 1), 8);
        }
    };
    for (int step = 0; step < nsteps; step += 4) {
        stage(GemmIntC<0>{}, step);
        stage(GemmIntC<1>{}, step + 1);
        if (step + 2 < nsteps) {   // uniform
            stage(GemmIntC<2>{}, step + 2);
            stage(GemmIntC<3>{}, step + 3);
        }
    }

    float* outm = p.out[mat];
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int r = r0 + 32 * j + arow;
#pragma unroll
        for (int el = 0; el < 16; el++) {
            const int t = 8 * (el >> 2) + 4 * kg + (el & 3);
            if (r < p.nrows && t < ncol) outm[(size_t)(c0 + t) * p.nrows + r] = out[j][el];
        }
    }
}

// ------------------------------------ grouped matmul, sixteen columns a group, no weight staging
// A handful of columns an expert (a small prefill batch through a wide mixture) is too few for
// the 32-column tile above and too many for the dot-product kernel, which pays every (weight,
// column) pair in vector instructions.  Here a group is up to sixteen columns and the matrix
// instruction is the 16 x 16 x 32 one: tokens are its M, sixteen weight rows its N, and a lane
// (row j = lane % 16, kg = lane / 16) supplies eight K values a step.  The K order of a step is
// free as long as both operands agree, so it is chosen to be what the lane's own 32-byte load
// of nibbles decodes to: lane (j, kg) loads group kg of the super-block of row j (32 bytes: low
// nibbles sub-block 2 kg, high nibbles sub-block 2 kg + 1), and word ks of it, unpacked as in
// the prefill GEMM (b0.lo, b2.lo, b0.hi, b2.hi, b1.lo, b3.lo, b1.hi, b3.hi),
// IS the lane's operand of K-step ks.  Weights therefore go HBM -> registers -> matrix core:
// no LDS staging, no barrier in the loop.  The prep kernel writes the columns in the matching
// order.  The group's activation fragments for the whole of K sit in LDS (JL_MOE_G16_SB_WORDS
// words a super-block), filled once per (workgroup, group); columns the group does not have are
// filled with zeros, so the workspace needs none.
//
// Prep: grid = ceil(ncols / 4), block = 256: a wavefront owns one column.  It finds the column's
// expert by counting the experts whose first column is not after it (one load of start[] a lane,
// ballots; the expert's first column is the largest start not after the column, a lane
// reduction, not a second trip to memory), then quantizes the column's super-blocks four at a
// time (lane l owns elements 4l..4l+3; the four loads go out together) and writes, per
// super-block, the 32 sixteen-byte pieces of the column's fragments, the two pieces of its
// sub-block sums (low six bits, the rest) and its scale.  (A wavefront a super-block, 65,536
// short wavefronts at 1024 rows, was bound by their dependent loads: 36 us where this takes 26.)
// KO: the K order of the matrix kernel's weights: 0 Q4_K GGUF rows, 1 Q4_K packed planes, 2 Q6_K GGUF rows
template <int KO = 0>
__device__ __forceinline__ void moe_g16_prep_body(const MoeG16PrepArgs& p, u32* lds) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const u32 c = blockIdx.x * 4 + wave;
    if (c >= (u32)p.ncols) return;   // whole wavefronts; no workgroup barrier below
    const int nsb = p.k / 256;
    const size_t row = p.src ? p.src[c] : c;
    u32 cnt = 0, c_lo = 0;
    for (int base = 0; base <= p.n_expert; base += 64) {
        const int idx = base + lane;
        const u32 s = idx <= p.n_expert ? p.start[idx] : 0xFFFFFFFFu;
        const bool le = s <= c;
        cnt += (u32)__builtin_popcountll(__ballot(le));
        c_lo = max(c_lo, le ? s : 0u);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) c_lo = max(c_lo, (u32)__shfl_xor((int)c_lo, off, 64));
    const int e = (int)cnt - 1;
    const u32 rel = c - c_lo;
    const size_t slot = (size_t)(c_lo >> 4) + (size_t)e + (rel >> 4);
    const int i = (int)(rel & 15);
    u32* sq = lds + wave * 72;   // the wavefront's own: 64 words of int8, 8 sub-block sums
    const f32x4* xr = (const f32x4*)(p.x + row * (size_t)p.k);
    const f32x4* ur = p.x2 ? (const f32x4*)(p.x2 + row * (size_t)p.k) : nullptr;
    for (int sb0 = 0; sb0 < nsb; sb0 += 4) {
        f32x4 vv[4], uu[4];
#pragma unroll
        for (int b = 0; b < 4; b++) {
            const int sb = min(sb0 + b, nsb - 1);
            vv[b] = xr[sb * 64 + lane];
            uu[b] = f32x4{0.f, 0.f, 0.f, 0.f};
            if (ur) uu[b] = ur[sb * 64 + lane];
        }
#pragma unroll
        for (int b = 0; b < 4; b++) {
            const int sb = sb0 + b;
            if (sb >= nsb) break;   // uniform
            f32x4 v = vv[b];
            if (ur) v = f32x4{silu_f32(v.x) * uu[b].x, silu_f32(v.y) * uu[b].y, silu_f32(v.z) * uu[b].z, silu_f32(v.w) * uu[b].w};
            const u32 m = max(max(abs_bits(v.x), abs_bits(v.y)), max(abs_bits(v.z), abs_bits(v.w)));
            const u32 amax = wave_amax_256(m);
            float d;
            i32 sum16;
            const u32 q = quantize4(v, amax, d, sum16);
            const i32 a32 = sum16 + dpp_i32<JL_DPP_ROW_HALF_MIRROR, 0xf>(0, sum16);
            sq[lane] = q;
            if ((lane & 7) == 0) sq[64 + (lane >> 3)] = (u32)a32;
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // LDS operations of a wavefront execute in order
            u32* blk = p.ws + (slot * nsb + sb) * JL_MOE_G16_SB_WORDS;
            if (lane < 32) {
                const int ks = lane >> 2, kg = lane & 3;
                // GGUF sheets: word ks of group kg pairs elements 4 ks.. of sub-blocks 2 kg and 2 kg + 1;
                // packed planes: K-step ks is word ks % 4 of sub-block 2 kg + ks / 4, whose low nibbles
                // are elements 4 w.. and whose high nibbles elements 4 w + 16.. of that one sub-block
                // Q6_K rows: lane group kg = (half n, half-run c), K-step ks = (nibble hh, word w): the
                // word of the run of elements 128 n + 64 hh + 16 c + 4 w.. and of the run 32 further on
                const int psub = 2 * kg + (ks >> 2), pw = ks & 3;
                const int q6 = 32 * (kg >> 1) + 16 * (ks >> 2) + 4 * (kg & 1) + (ks & 3);
                const u32 lo = KO == 2 ? sq[q6] : KO == 1 ? sq[8 * psub + pw] : sq[16 * kg + ks];
                const u32 hi = KO == 2 ? sq[q6 + 8] : KO == 1 ? sq[8 * psub + 4 + pw] : sq[16 * kg + 8 + ks];
                auto f = [](u32 w, int b2) { return (_Float16)(float)(int8_t)(w >> (8 * b2)); };
                const f16x8 o = {f(lo, 0), f(lo, 2), f(hi, 0), f(hi, 2), f(lo, 1), f(lo, 3), f(hi, 1), f(hi, 3)};
                ((u32x4*)blk)[ks * 64 + 16 * kg + i] = __builtin_bit_cast(u32x4, o);
            } else if (lane < 34) {
                const int kg = lane - 32;
                f16x8 o;
#pragma unroll
                for (int s8 = 0; s8 < 8; s8++) {
                    const i32 a = (i32)sq[64 + s8];
                    o[s8] = (_Float16)(float)(kg ? (a >> 6) : (a & 63));
                }
                ((u32x4*)blk)[512 + 16 * kg + i] = __builtin_bit_cast(u32x4, o);
            } else if (lane == 34) {
                blk[2176 + i] = __float_as_uint(d);
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the reads above, before the next task's writes
        }
    }
}

// One 32-bit word of nibbles as a matrix operand: the prefill GEMM's unpack, kept in registers.
__device__ __forceinline__ f16x8 moe_g16_word(u32 w, const GemmWideScale& k, u32 mask_lo, u32 mask_hi, u32 magic) {
    const u32 w8 = w >> 8;
    auto nib = [&](u32 v, u32 mask) { return __builtin_bit_cast(f16x2, (v & mask) | magic); };
    const f16x2 p0 = __builtin_elementwise_fma(nib(w, mask_lo), k.mlo, k.alo);
    const f16x2 p1 = __builtin_elementwise_fma(nib(w, mask_hi), k.mhi, k.ahi);
    const f16x2 p2 = __builtin_elementwise_fma(nib(w8, mask_lo), k.mlo, k.alo);
    const f16x2 p3 = __builtin_elementwise_fma(nib(w8, mask_hi), k.mhi, k.ahi);
    const u32x4 o = {__builtin_bit_cast(u32, p0), __builtin_bit_cast(u32, p1), __builtin_bit_cast(u32, p2),
                     __builtin_bit_cast(u32, p3)};
    return __builtin_bit_cast(f16x8, o);
}

// Matrix kernel: grid = 8 * ceil(n_expert / 8) * blocks * matrices (one dimension), block =
// 64 * nwaves, dynamic LDS = (k/256) * JL_MOE_G16_LDS_WORDS * 4 + 16.  Workgroups go round the eight
// XCDs in the order of their ids, so id % 8 names the XCD: expert e is worked on by XCD e % 8
// alone, its (matrix, row block) workgroups one after the other there, and the group's fragments
// are fetched into one L2 once.  A workgroup owns tiles_wg tiles of sixteen rows of the
// expert's sheet and walks the expert's column groups; its wavefronts take the tiles one after
// the other from a counter in LDS.  A step is (tile, chunk of CH super-blocks): CH * 144 contiguous bytes of
// each of the tile's rows, requested in one go a whole step ahead (two register sets), so a
// cache line is used up by the step that fetched it and only the line at a chunk's border is
// touched twice.  Per super-block: eight K-steps, then the epilogue into the tile's four sums.
// FUSED: no prep kernel and no workspace -- the workgroup quantizes its group's columns itself
// (a wavefront per (column, super-block), the prep kernel's arithmetic) straight into the LDS
// fragments, behind the first weight loads.  Every workgroup of the expert repeats that, which
// pays while an expert has a handful of columns: two launches less a call.  FUSED = 1: plain
// columns, 2: silu(x) * x2.  NT = 2: a group is 32 columns, two token tiles whose fragments sit
// in LDS one behind the other (two workspace slots), and a decoded word meets both: an expert of
// 17-32 columns reads its sheet once.
template <int CH, int FUSED, int KO = 0, int NT = 1>
__device__ __forceinline__ void moe_g16_body(const MoeG16Args& p, uint8_t* smem) {
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    JL_MOE_TRACE(0);
    const int nwaves = p.nwaves, nthreads = 64 * nwaves;
    const int per_e = p.blocks * p.nmat;
    const int xcd = blockIdx.x & 7, q = blockIdx.x >> 3;
    const int e = xcd + 8 * (q / per_e), sub = q % per_e;
    if (e >= p.n_expert) return;
    const int mat = sub / p.blocks, blk = sub % p.blocks;
    const u32 c_lo = p.start[e], c_hi = p.start[e + 1];
    if (c_lo == c_hi) return;   // nobody chose this expert (uniform across the workgroup)
    const int nsb = p.k / 256, nch = (nsb + CH - 1) / CH;
    const int tiles = (p.nrows + 15) >> 4;
    const int tile_base = blk * p.tiles_wg;
    const int ntw = min(tiles, tile_base + p.tiles_wg) - tile_base;   // tiles of this workgroup
    const int j = lane & 15, kg = lane >> 4;
    constexpr bool PL = KO == 1, Q6 = KO == 2;
    const uint8_t* sheet = PL ? nullptr : p.bank[mat] + (size_t)e * p.sheet_bytes;
    u32 mask_lo = 0x000F000Fu, mask_hi = 0x00F000F0u, magic = 0x64006400u;
    asm volatile("" : "+v"(mask_lo), "+v"(mask_hi), "+v"(magic));
    u32x4* sA4 = (u32x4*)smem;
    const float* sAf = (const float*)smem;
    static_assert(NT == 1 || FUSED == 0, "two token tiles a group take their fragments from the prep kernel");
    u32* next_tile = (u32*)smem + (size_t)NT * nsb * JL_MOE_G16_LDS_WORDS;   // behind the fragments
    const int RV = nsb * (JL_MOE_G16_LDS_WORDS / 4);   // vectors of one token tile's fragments (NT = 2: two regions)
    float* outm = p.out[mat];
    // LDS vectors a super-block: eight fragments 65 vectors apart (64 used: a column's pieces, one
    // a fragment, then spread over sixteen banks when the fused form writes them), the sums' 32, the
    // scales' 4; WS: vectors a super-block of the prep kernel's workspace
    constexpr int V = JL_MOE_G16_LDS_WORDS / 4, WS = JL_MOE_G16_SB_WORDS / 4;

    // a step's registers: header and two vectors of nibbles a super-block (Q6_K: the scales' eight
    // bytes and d in the header, the two runs' low nibbles, and a third vector of high bits)
    constexpr int NQ = Q6 ? 3 : 2;
    u32x4 hd[2][CH], wq[2][CH][NQ];
    // step (tile ti of the workgroup's range, chunk ch) into a register set
    // PL (packed planes): the header is the row's (d, dmin) word and its three words of 6-bit fields,
    // the lane's eight words are sub-blocks 2 kg and 2 kg + 1 (four words each); every load
    // instruction reads four runs of sixteen consecutive rows
    const size_t pst = (size_t)p.pstride;
    const u32* pl_qs = PL ? p.pqs[mat] + (size_t)e * p.sheet_words + (size_t)e * p.row_step : nullptr;
    const u32* pl_d = PL ? p.pd[mat] + (size_t)e * p.sheet_words + (size_t)e * p.row_step : nullptr;
    const u32* pl_sc = PL ? p.psc[mat] + (size_t)e * p.sheet_words + (size_t)e * p.row_step : nullptr;
    auto load_step = [&](int ti, int ch, u32x4 (&h)[CH], u32x4 (&q)[CH][NQ]) {
        const int row = min(16 * (tile_base + ti) + j, p.nrows - 1);
        if (Q6) {
            // lane (j, kg): half n = kg / 2 of the super-block, half-run c = kg % 2: sixteen bytes of each
            // run's nibbles and of the high bits, the half's eight scales, d
            const uint8_t* b = sheet + (size_t)row * p.row_bytes;
            const int n = kg >> 1, c = kg & 1;
#pragma unroll
            for (int s = 0; s < CH; s++) {
                const uint8_t* bs = b + (size_t)min(ch * CH + s, nsb - 1) * 210;
                q[s][0] = ld16_a2(bs + 64 * n + 16 * c);
                q[s][1] = ld16_a2(bs + 64 * n + 32 + 16 * c);
                q[s][NQ - 1] = ld16_a2(bs + 128 + 32 * n + 16 * c);
                h[s] = u32x4{ld4_a2(bs + 192 + 8 * n), ld4_a2(bs + 196 + 8 * n), (u32)ld2(bs + 208), 0u};
            }
            return;
        }
        if (PL) {
#pragma unroll
            for (int s = 0; s < CH; s++) {
                const size_t sbi = (size_t)min(ch * CH + s, nsb - 1);
                h[s] = u32x4{pl_d[sbi * pst + row], pl_sc[(3 * sbi) * pst + row], pl_sc[(3 * sbi + 1) * pst + row],
                             pl_sc[(3 * sbi + 2) * pst + row]};
#pragma unroll
                for (int hh = 0; hh < 2; hh++) {
                    const u32* b = pl_qs + ((sbi * 8 + 2 * kg + hh) * 4) * pst + row;
                    q[s][hh] = u32x4{b[0], b[pst], b[2 * pst], b[3 * pst]};
                }
            }
            return;
        }
        const uint8_t* b = sheet + (size_t)row * p.row_bytes;
#pragma unroll
        for (int s = 0; s < CH; s++) {
            const uint8_t* bs = b + (size_t)min(ch * CH + s, nsb - 1) * 144;
            h[s] = ld16(bs);
            q[s][0] = ld16(bs + 16 + 32 * kg);
            q[s][1] = ld16(bs + 32 + 32 * kg);
        }
    };

    for (u32 c0 = c_lo; c0 < c_hi; c0 += 16 * NT) {
        const int ncg = min(16 * NT, (int)(c_hi - c0));
        const size_t slot = (size_t)(c_lo >> 4) + (size_t)e + ((c0 - c_lo) >> 4);
        // FUSED: the group's source rows, one a lane, and the first eight (column, super-block)
        // tasks of this wavefront requested ahead of the weights, which have the longer way and
        // would hold them up (a wavefront's loads return in order)
        constexpr bool X2 = FUSED == 2;           // columns are silu(x) * x2 (the down projection's)
        // tasks of a wavefront in flight: 32 (K = 768: ten columns) or 64 a workgroup of eight.  Slots past
        // the last task repeat its load (a slot that requested nothing would make every wait that follows
        // count as if none had: 104.5 -> 105.9 us for the 64-row block), and a repeated load still takes
        // its place in the queue in front of the weights, so there are no more slots than a handful of
        // columns needs (sixteen and eight: 108.0 us)
        constexpr int TB = X2 ? 4 : 8;
        const int ntask = ncg * nsb;
        // task / nsb for task < 16 * nsb <= 1024 as a multiplication (a division is ~30 instructions)
        const u32 nsb_inv = 65536u / (u32)nsb + 1u;
        u32 rowv = 0;
        f32x4 xv[TB], xu[X2 ? TB : 1];
        auto issue = [&](int t0) {
#pragma unroll
            for (int b = 0; b < TB; b++) {
                const int task = min(t0 + b * nwaves, ntask - 1);
                const int i = (int)(((u32)task * nsb_inv) >> 16), sb = task - i * nsb;
                const size_t row = (size_t)__shfl(rowv, i, 64);
                xv[b] = ((const f32x4*)(p.x + row * (size_t)p.k + (size_t)sb * 256))[lane];
                if (X2) xu[X2 ? b : 0] = ((const f32x4*)(p.x2 + row * (size_t)p.k + (size_t)sb * 256))[lane];
            }
        };
        if (FUSED) {
            if (lane < ncg) rowv = p.src ? p.src[c0 + lane] : c0 + (u32)lane;
            issue(wave);
        }
        if (wave < ntw) load_step(wave, 0, hd[0], wq[0]);
        if (c0 != c_lo) __syncthreads();   // the previous group's fragments have been read
        if (tid == 0) *next_tile = (u32)nwaves;   // tiles 0 .. nwaves - 1 are the wavefronts' first ones
        if (FUSED) {
            // zeros where the group has no column (fragments and sums; the scales are not read there)
            const int total = nsb * WS;
            for (int idx = tid; idx < total; idx += nthreads) {
                const int sb = idx / WS, o = idx - sb * WS;
                if (o < 544 && (o & 15) >= ncg) sA4[sb * V + (o < 512 ? o + (o >> 6) : o + 8)] = u32x4{0u, 0u, 0u, 0u};
            }
            u32* sAw = (u32*)smem;
            _Float16* sAh = (_Float16*)smem;
            float* sAfw = (float*)smem;
            for (int t0 = wave; t0 < ntask; t0 += TB * nwaves) {
                if (t0 != wave) issue(t0);
#pragma unroll
                for (int b = 0; b < TB; b++) {
                    const int task = t0 + b * nwaves;
                    if (task < ntask) {   // uniform
                        const int i = (int)(((u32)task * nsb_inv) >> 16), sb = task - i * nsb;
                        f32x4 w = xv[b];
                        if (X2) {
                            const f32x4 u = xu[X2 ? b : 0];
                            w = f32x4{silu_f32(w.x) * u.x, silu_f32(w.y) * u.y, silu_f32(w.z) * u.z, silu_f32(w.w) * u.w};
                        }
                        const u32 m = max(max(abs_bits(w.x), abs_bits(w.y)), max(abs_bits(w.z), abs_bits(w.w)));
                        const u32 amax = wave_amax_256(m);
                        float d;
                        i32 sum16;
                        const u32 q = quantize4(w, amax, d, sum16);
                        const i32 a32 = sum16 + dpp_i32<JL_DPP_ROW_HALF_MIRROR, 0xf>(0, sum16);
                        // lane l holds word l of the super-block: sub-block l / 8 (group kg, low or
                        // high nibbles' partner), K-step l % 8; its bytes go to two f16 pairs
                        // (planes: word l % 4 of sub-block l / 8, low nibbles' partner where
                        // l % 8 < 4; K-step 4 (sub % 2) + l % 4 of group sub / 2)
                        // (Q6_K: l = 32 n + 16 hh + 8 r + 4 c + w: group 2 n + c, K-step 4 hh + w, run r)
                        const int sub = lane >> 3;
                        const int kg = Q6 ? 2 * (lane >> 5) + ((lane >> 2) & 1) : sub >> 1;
                        const int ks = Q6 ? 4 * ((lane >> 4) & 1) + (lane & 3) : PL ? 4 * (sub & 1) + (lane & 3) : lane & 7;
                        const int hi = Q6 ? (lane >> 3) & 1 : PL ? (lane >> 2) & 1 : sub & 1;
                        auto f = [](u32 x, int b2) { return (_Float16)(float)(int8_t)(x >> (8 * b2)); };
                        const f16x2 p02 = {f(q, 0), f(q, 2)}, p13 = {f(q, 1), f(q, 3)};
                        const int vec = sb * V + ks * 65 + 16 * kg + i;
                        sAw[vec * 4 + hi] = __builtin_bit_cast(u32, p02);
                        sAw[vec * 4 + 2 + hi] = __builtin_bit_cast(u32, p13);
                        if ((lane & 7) == 0) {
                            sAh[(sb * V + 520 + i) * 8 + sub] = (_Float16)(float)(a32 & 63);
                            sAh[(sb * V + 520 + 16 + i) * 8 + sub] = (_Float16)(float)(a32 >> 6);
                        }
                        if (lane == 0) sAfw[(sb * V + 552) * 4 + i] = d;
                    }
                }
            }
        } else {
            // twelve loads in flight a thread (all of K = 2048 at 512 threads): the fill is one round
            // trip to L2, not one a vector
            constexpr int NB = 12;
            const int total = nsb * WS;
#pragma unroll
            for (int r = 0; r < NT; r++) {
                const int ncr = min(16, max(0, ncg - 16 * r));   // columns of token tile r
                const u32x4* src = (const u32x4*)(p.ws + (slot + r) * nsb * JL_MOE_G16_SB_WORDS);
                for (int base = tid; base < total; base += NB * nthreads) {
                    u32x4 val[NB];
#pragma unroll
                    for (int u = 0; u < NB; u++) {
                        const int idx = base + u * nthreads, o = idx % WS;
                        // fragments: lane = o % 64, its column o % 16; sums: (o - 512) % 16; scales: all
                        const bool have = idx < total && (o >= 544 ? ncr > 0 : (o & 15) < ncr);
                        val[u] = u32x4{0u, 0u, 0u, 0u};
                        if (have) val[u] = src[idx];
                    }
#pragma unroll
                    for (int u = 0; u < NB; u++) {
                        const int idx = base + u * nthreads, sb = idx / WS, o = idx - sb * WS;
                        if (idx < total) sA4[r * RV + sb * V + (o < 512 ? o + (o >> 6) : o + 8)] = val[u];
                    }
                }
            }
        }
        __syncthreads();
        JL_MOE_TRACE(1);
        f32x4 out[NT];
#pragma unroll
        for (int r = 0; r < NT; r++) out[r] = f32x4{0.f, 0.f, 0.f, 0.f};
        // Tiles are handed out as the wavefronts get to them (a counter in LDS): the SIMD issues
        // its oldest wavefront first, so with a fixed share each the young ones fall behind and
        // run the last tenth of the kernel alone.  A wavefront knows its next tile a tile ahead.
        auto take = [&]() {
            u32 v = 0;
            if (lane == 0) v = __hip_atomic_fetch_add(next_tile, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            return (int)__builtin_amdgcn_readfirstlane(v);
        };
        int ti = wave, ch = 0;   // this step's tile and chunk
        int ti_n = ti < ntw ? take() : ntw;
        auto step = [&](auto PAR) {
            constexpr int cur = decltype(PAR)::value;
            const bool last_ch = ch == nch - 1;
            const int t_n = last_ch ? ti_n : ti, ch_n = last_ch ? 0 : ch + 1;
            load_step(min(t_n, ntw - 1), ch_n, hd[cur ^ 1], wq[cur ^ 1]);
#pragma unroll
            for (int s = 0; s < CH; s++) {
                const int sb = ch * CH + s;
                if (sb < nsb) {   // uniform
                    f32x4 accP[NT];
                    if (Q6) {
                        // sc * (q - 32) reaches 4096 and f16 holds odd integers only up to 2048: the scale
                        // is split, sc = 2 (sc >> 1) + (sc & 1), two operands and two matrix instructions
                        // a K-step into the same sums (gemm_q6k.h); the zero point is inside the operand
                        const int c = kg & 1;
                        u32 m4 = 0x000F000Fu, m2 = 0x00300030u;
                        asm volatile("" : "+v"(m4), "+v"(m2));
                        const f16x2 off = {(_Float16)-1056.0f, (_Float16)-1056.0f};
                        // the super-block's fragments and token scales requested from LDS in one go (see below)
                        u32x4 af[8][NT];
                        f32x4 dav[NT];
#pragma unroll
                        for (int ks = 0; ks < 8; ks++)
#pragma unroll
                            for (int r = 0; r < NT; r++) af[ks][r] = sA4[r * RV + sb * V + ks * 65 + lane];
#pragma unroll
                        for (int r = 0; r < NT; r++) dav[r] = *(const f32x4*)(sAf + ((size_t)r * RV + sb * V + 552) * 4 + 4 * kg);
                        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                        for (int ks = 0; ks < 8; ks++) {
                            const int hh = ks >> 2, w = ks & 3;
                            // the two runs' scales: bytes c and 2 + c of the half's word hh
                            const u32 scw = hh ? hd[cur][s].y : hd[cur][s].x;
                            const i32 sa = (i32)(int8_t)(scw >> (8 * c)), sb_ = (i32)(int8_t)(scw >> (8 * (2 + c)));
                            const _Float16 a2 = (_Float16)(float)(2 * (sa >> 1)), a0 = (_Float16)(float)(sa & 1);
                            const _Float16 b2 = (_Float16)(float)(2 * (sb_ >> 1)), b0 = (_Float16)(float)(sb_ & 1);
                            const f16x2 A2 = {a2, a2}, A0 = {a0, a0}, B2 = {b2, b2}, B0 = {b0, b0};
                            const u32 wa = wq[cur][s][0][w] >> (4 * hh), wb = wq[cur][s][1][w] >> (4 * hh);
                            const u32 whq = wq[cur][s][NQ - 1][w];
                            const u32 wh = hh ? whq : whq << 4;   // an element's two high bits at bits 4-5 of its half
                            auto val = [&](u32 nib, u32 hi2) {
                                const u32 v = (hi2 & m2) | ((nib & m4) | magic);
                                return __builtin_bit_cast(f16x2, v) + off;
                            };
                            const f16x2 ta02 = val(wa, wh), tb02 = val(wb, wh >> 2);
                            const f16x2 ta13 = val(wa >> 8, wh >> 8), tb13 = val(wb >> 8, wh >> 10);
                            auto word = [](f16x2 v) { return __builtin_bit_cast(u32, v); };
                            const u32x4 oa = {word(ta02 * A2), word(tb02 * B2), word(ta13 * A2), word(tb13 * B2)};
                            const u32x4 ob = {word(ta02 * A0), word(tb02 * B0), word(ta13 * A0), word(tb13 * B0)};
                            const f32x4 czero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                            for (int r = 0; r < NT; r++) {
                                const f16x8 a = __builtin_bit_cast(f16x8, af[ks][r]);
                                accP[r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, __builtin_bit_cast(f16x8, oa),
                                                                                 ks == 0 ? czero : accP[r], 0, 0, 0);
                                accP[r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, __builtin_bit_cast(f16x8, ob), accP[r], 0, 0, 0);
                            }
                        }
                        // out += d_a * (d * P) for the super-block
                        const float dd = half_bits_to_f32((uint16_t)(hd[cur][s].z & 0xFFFF));
#pragma unroll
                        for (int r = 0; r < NT; r++)
#pragma unroll
                            for (int el = 0; el < 4; el++) out[r][el] = fmaf(dav[r][el], dd * accP[r][el], out[r][el]);
                    } else {
                    GemmWideScale sc, sc1;
                    if (PL) {
                        gemm_wide_scale_planes(hd[cur][s], 2 * kg, sc);
                        gemm_wide_scale_planes(hd[cur][s], 2 * kg + 1, sc1);
                    } else {
                        gemm_wide_scale(hd[cur][s], kg & 1, kg >> 1, sc);
                    }
                    // the super-block's fragments, sums and token scales are requested from LDS in one
                    // go: read one K-step at a time, each matrix instruction waited a full LDS latency
                    // behind its own read, with two wavefronts a SIMD to hide it
                    u32x4 af[8][NT], augw[NT];
                    f32x4 dav[NT];
#pragma unroll
                    for (int ks = 0; ks < 8; ks++)
#pragma unroll
                        for (int r = 0; r < NT; r++) af[ks][r] = sA4[r * RV + sb * V + ks * 65 + lane];
#pragma unroll
                    for (int r = 0; r < NT; r++) {
                        augw[r] = sA4[r * RV + sb * V + 520 + (lane & 31)];
                        dav[r] = *(const f32x4*)(sAf + ((size_t)r * RV + sb * V + 552) * 4 + 4 * kg);
                    }
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int ks = 0; ks < 8; ks++) {
                        const f16x8 b = moe_g16_word(wq[cur][s][ks >> 2][ks & 3], PL && ks >= 4 ? sc1 : sc, mask_lo, mask_hi, magic);
                        const f32x4 czero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                        for (int r = 0; r < NT; r++)
                            accP[r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, af[ks][r]), b,
                                                                             ks == 0 ? czero : accP[r], 0, 0, 0);
                    }
                    // out += d_a * (d * P - dmin * M) for the super-block
                    const float mul = kg == 0 ? 1.0f : (kg == 1 ? 64.0f : 0.0f);
                    f16x8 mm;
                    if (PL) {
#pragma unroll
                        for (int b = 0; b < 8; b++) mm[b] = (_Float16)((float)gemm_stream_field(hd[cur][s], 2 * b + 1) * mul);
                    } else {
                        const GemmScaleBytes sbytes = gemm_scale_bytes(hd[cur][s].y, hd[cur][s].z, hd[cur][s].w);
#pragma unroll
                        for (int b = 0; b < 4; b++) {
                            mm[b] = (_Float16)((float)((sbytes.mn_lo >> (8 * b)) & 0xFF) * mul);
                            mm[4 + b] = (_Float16)((float)((sbytes.mn_hi >> (8 * b)) & 0xFF) * mul);
                        }
                    }
                    const float dd = half_bits_to_f32((uint16_t)(hd[cur][s].x & 0xFFFF));
                    const float dmin = half_bits_to_f32((uint16_t)(hd[cur][s].x >> 16));
#pragma unroll
                    for (int r = 0; r < NT; r++) {
                        // lanes 32-63 (kg 2, 3) meet minimum columns of zero, so what they hold of the sums does not count
                        const f16x8 aug = __builtin_bit_cast(f16x8, augw[r]);
                        const f32x4 czero = {0.f, 0.f, 0.f, 0.f};
                        const f32x4 accM = __builtin_amdgcn_mfma_f32_16x16x32_f16(aug, mm, czero, 0, 0, 0);
#pragma unroll
                        for (int el = 0; el < 4; el++) {
                            const float uu = fmaf(dd, accP[r][el], -(dmin * accM[el]));
                            out[r][el] = fmaf(dav[r][el], uu, out[r][el]);
                        }
                    }
                    }
                }
            }
            if (last_ch) {   // the tile is done: store its 16 rows x ncg columns
                const int r = 16 * (tile_base + ti) + j;
#pragma unroll
                for (int tt = 0; tt < NT; tt++)
#pragma unroll
                    for (int el = 0; el < 4; el++) {
                        const int tok = 16 * tt + 4 * kg + el;
                        if (r < p.nrows && tok < ncg) outm[(size_t)(c0 + tok) * p.nrows + r] = out[tt][el];
                        out[tt][el] = 0.f;
                    }
            }
            if (last_ch) {
                ti = ti_n;
                if (ti < ntw) ti_n = take();
            }
            ch = ch_n;
        };
        bool first = true;
        while (ti < ntw) {   // uniform
            step(GemmIntC<0>{});
            if (first) JL_MOE_TRACE(2);
            first = false;
            if (ti < ntw) step(GemmIntC<1>{});
        }
        JL_MOE_TRACE(3);
    }
}

// resid[r][n] += sum over the row's k_used experts, ascending expert id, of
// wt[r][s] * y[pos[r*k_used+s]][n].  grid = (ceil(n_embd/4/256), rows): a thread owns four
// columns of a row.  The first k_used threads rank the row's slots by expert id and lay weights
// and positions out in that order in LDS, so every thread adds in the reference's order
// without sorting anything itself.
__device__ __forceinline__ void moe_combine_body(const MoeCombineArgs& p, float* swt, u32* spos) {
    const int r = blockIdx.y, ku = p.k_used, tid = threadIdx.x;
    if (tid < ku) {
        const u32 mine = p.sel[r * p.sel_stride + tid];
        int rank = 0;   // a stable rank: equal ids (not a valid routing) keep their slot order
        for (int j = 0; j < ku; j++) {
            const u32 other = p.sel[r * p.sel_stride + j];
            rank += other < mine || (other == mine && j < tid);
        }
        swt[rank] = p.wt[r * ku + tid];
        spos[rank] = p.pos[r * ku + tid];
    }
    __syncthreads();
    const int n4 = p.n_embd >> 2, n = blockIdx.x * 256 + tid;
    if (n >= n4) return;
    f32x4* res = (f32x4*)(p.resid + (size_t)r * p.n_embd) + n;
    f32x4 acc = *res;
    // eight experts' rows requested together (a loop of load, add, load, ... is a chain of trips to
    // memory), added in ascending expert order as before
    for (int i0 = 0; i0 < ku; i0 += 8) {
        f32x4 y[8];
#pragma unroll
        for (int b = 0; b < 8; b++) {
            const int i = min(i0 + b, ku - 1);
            y[b] = ((const f32x4*)(p.y + (size_t)spos[i] * p.n_embd))[n];
        }
#pragma unroll
        for (int b = 0; b < 8; b++) {
            if (i0 + b < ku) {   // uniform
                const float w = swt[i0 + b];
                acc = f32x4{acc.x + w * y[b].x, acc.y + w * y[b].y, acc.z + w * y[b].z, acc.w + w * y[b].w};
            }
        }
    }
    *res = acc;
}

// ---------------------------------------------------------------- router logits
// logits[t][r] = sum_i W[r][i] * x[t][i] in f32, with the summation order of the reference's
// device kernel (jit/gpu/kernels/moe.go:843-917) so that the bits are its bits: thread j of
// 128 adds the products of i = j, j + 128, ... one after the other (product rounded, then
// the sum; a ragged tail adds +0), and the 128 partial sums meet in a binary tree, thread j
// taking thread j + s at s = 64, 32, ..., 1.  One workgroup per expert row and group of
// JL_LOGITS_TOK tokens: the row is read once for all of them.
// With many tokens the launch is bound by re-reading x from L2 for every expert row (2048
// tokens x 128 experts x k = 2048: 114 us), so there a workgroup takes EB = 8 expert rows
// for its eight tokens and every x value loaded meets eight weights (grid.x = ceil(rows/EB)).
#define JL_LOGITS_TOK 8
template <int EB>
__device__ __forceinline__ void moe_logits_body(const MoeLogitsArgs& p, float* part) {
    const int r0 = blockIdx.x * EB, t0 = blockIdx.y * JL_LOGITS_TOK, tid = threadIdx.x;
    const int nt = min(JL_LOGITS_TOK, p.ntok - t0), k = p.k;
    float acc[EB][JL_LOGITS_TOK];
#pragma unroll
    for (int e = 0; e < EB; e++)
#pragma unroll
        for (int t = 0; t < JL_LOGITS_TOK; t++) acc[e][t] = 0.f;
    // a trip: element i0 + tid of every row and token; the ragged last trip (k % 128 != 0) adds +0 where
    // the row has ended, the whole ones carry neither the select nor the clamp (a third of the
    // loop's vector instructions, and the kernel issues vector instructions most of its time)
    auto trip = [&](int i0, auto RAGGED) {
        constexpr bool ragged = decltype(RAGGED)::value != 0;
        const int i = i0 + tid, ic = ragged ? min(i, k - 1) : i;
        float w[EB], xv[JL_LOGITS_TOK];
#pragma unroll
        for (int e = 0; e < EB; e++) {
            const size_t at = (size_t)min(r0 + e, p.n_expert - 1) * k + ic;
            w[e] = p.f16 ? half_bits_to_f32(((const uint16_t*)p.w)[at]) : ((const float*)p.w)[at];
        }
#pragma unroll
        for (int t = 0; t < JL_LOGITS_TOK; t++) xv[t] = p.x[(size_t)(t0 + min(t, nt - 1)) * k + ic];
#pragma unroll
        for (int e = 0; e < EB; e++)
#pragma unroll
            for (int t = 0; t < JL_LOGITS_TOK; t++) {
                const float prod = w[e] * xv[t];
                acc[e][t] = acc[e][t] + (!ragged || i < k ? prod : 0.f);
            }
    };
    const int kfull = k & ~127;
    // unrolled so that the loads of several trips are in flight together; the sums stay in order
#pragma unroll EB == 1 ? 16 : 2
    // (the eight-row form keeps the select in every trip: without it the same loop measured 34.4 us
    // against 29.3 at 1024 tokens, the one-row form 5.96 against 6.8 at 64)
    for (int i0 = 0; i0 < kfull; i0 += 128) trip(i0, GemmIntC<EB == 1 ? 0 : 1>{});
    if (kfull < k) trip(kfull, GemmIntC<1>{});
    // The tree, one token per 16 lanes: lane j of a token's row takes the partial sums the
    // tree would bring to thread j by s = 16 (levels 64, 32, 16: seven adds in tree order),
    // then levels 8..1 are lane moves inside the 16-lane row (lane j reads lane j + s).
    // One expert row at a time through part [token][128] (a buffer per row would cost the
    // eight-row form its wavefronts per CU).
    static_assert(JL_LOGITS_TOK == 8, "eight tokens x sixteen lanes = the workgroup");
    const int tk = tid >> 4, j = tid & 15;
#pragma unroll
    for (int e = 0; e < EB; e++) {
        if (e) __syncthreads();
#pragma unroll
        for (int t = 0; t < JL_LOGITS_TOK; t++) part[t * 128 + tid] = acc[e][t];
        __syncthreads();
        const float* q = part + tk * 128 + j;
        const float a0 = q[0] + q[64], a32 = q[32] + q[96], a16 = q[16] + q[80], a48 = q[48] + q[112];
        const float b0 = a0 + a32, b16 = a16 + a48;
        float v = b0 + b16;
        v = v + dpp_f32<0x108, 0xf>(v);   // row_shl:8
        v = v + dpp_f32<0x104, 0xf>(v);   // row_shl:4
        v = v + dpp_f32<0x102, 0xf>(v);   // row_shl:2
        v = v + dpp_f32<0x101, 0xf>(v);   // row_shl:1
        if (j == 0 && tk < nt && r0 + e < p.n_expert) p.logits[(size_t)(t0 + tk) * p.n_expert + r0 + e] = v;
    }
}
