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
//   moe_matvec     for every column c of expert e: out[c] = W_e . x[src(c)], the
//                  decode matvec's arithmetic per column.  One workgroup owns
//                  (expert, row share): it quantizes the expert's activations
//                  into LDS once (optionally act(gate)*up first) and streams the
//                  expert's weight rows once for up to eight columns at a time,
//                  so a sheet is read from HBM once however many rows chose it.
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

#define JL_MOE_TB 8  // columns of one expert processed per pass over its rows

// ------------------------------------------------------------------ grouping
// One workgroup; thread e owns expert e and scans the pairs in order, which makes
// the within-expert order (row, slot) with no atomics.
__device__ __forceinline__ void moe_group_body(const MoeGroupArgs& p, u32* scount) {
    const int e = threadIdx.x;
    const int npairs = p.rows * p.k_used;
    u32 cnt = 0;
    if (e < p.n_expert)
        for (int i = 0; i < npairs; i++) cnt += p.sel[(i / p.k_used) * p.sel_stride + i % p.k_used] == (u32)e;
    scount[e] = e < p.n_expert ? cnt : 0;
    __syncthreads();
    if (e < p.n_expert) {
        u32 start = 0;
        for (int j = 0; j < e; j++) start += scount[j];
        p.start[e] = start;
        if (e == p.n_expert - 1) p.start[p.n_expert] = start + cnt;
        u32 col = start;
        for (int i = 0; i < npairs; i++) {
            const int r = i / p.k_used, s = i % p.k_used;
            if (p.sel[r * p.sel_stride + s] == (u32)e) {
                p.perm[col] = (u32)r;
                p.pos[i] = col;
                col++;
            }
        }
    }
}

// Sum over the LPR consecutive lanes of a row group (LPR = 16, 32 or 64); the
// total is valid in the group's last lane.
template <int LPR>
__device__ __forceinline__ float group_sum(float v) {
    v += dpp_f32<JL_DPP_QUAD_XOR1, 0xf>(v);
    v += dpp_f32<JL_DPP_QUAD_XOR2, 0xf>(v);
    v += dpp_f32<JL_DPP_ROW_HALF_MIRROR, 0xf>(v);
    v += dpp_f32<JL_DPP_ROW_MIRROR, 0xf>(v);
    if (LPR >= 32) v += dpp_f32<JL_DPP_ROW_BCAST15, 0xa>(v);
    if (LPR >= 64) v += dpp_f32<JL_DPP_ROW_BCAST31, 0xc>(v);
    return v;
}

__device__ __forceinline__ float silu_f32(float g) { return g / (1.0f + __expf(-g)); }

// Quantize one column's activation (k floats, optionally silu(x)*x2) into the LDS
// staging area `smem`; called by whole wavefronts, n4_pad a multiple of 64.
__device__ __forceinline__ void moe_stage_column(uint8_t* smem, const float* x, const float* x2, int k,
                                                 int per, int tid, int nthreads) {
    const int n4 = k / 4, n4_pad = (n4 + 63) & ~63;
    for (int g4 = tid; g4 < n4_pad; g4 += nthreads) {
        f32x4 v = f32x4{0.f, 0.f, 0.f, 0.f};
        if (g4 < n4) {
            v = ((const f32x4*)x)[g4];
            if (x2) {
                f32x4 u = ((const f32x4*)x2)[g4];
                v = f32x4{silu_f32(v.x) * u.x, silu_f32(v.y) * u.y, silu_f32(v.z) * u.z, silu_f32(v.w) * u.w};
            }
        }
        stage_quantize4(smem, k, per, g4, v);
    }
}

template <int TYPE, int LPR>
__device__ __forceinline__ void moe_matvec_body(const MoeMatVecArgs& p, uint8_t* smem) {
    typedef SlotTraits<TYPE> T;
    constexpr int RW = 64 / LPR;  // weight rows per wavefront step
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
    const int e = blockIdx.y, mat = blockIdx.z;
    const u32 c_lo = p.start[e], c_hi = p.start[e + 1];
    if (c_lo == c_hi) return;  // nobody chose this expert (uniform across the workgroup)
    const int nslots = p.k / T::kElems;
    const int slot = lane % LPR, rw = lane / LPR;
    const bool live = slot < nslots;
    // this workgroup's share of the rows
    const int share = (p.nrows + gridDim.x - 1) / gridDim.x;
    const int row_lo = blockIdx.x * share, row_hi = min(row_lo + share, p.nrows);
    const uint8_t* sheet = p.bank[mat] + (size_t)e * p.sheet_bytes;
    float* out = p.out[mat];
    const int act_bytes = (JL_ACT_LDS_BYTES(p.k) + 15) & ~15;

    for (u32 c0 = c_lo; c0 < c_hi; c0 += JL_MOE_TB) {
        const int ncol = min((u32)JL_MOE_TB, c_hi - c0);
        // stage the pass's columns: two wavefront groups of 512 threads work on two columns at a time
        {
            const int half = threadIdx.x >= 512 ? 1 : 0, nth = blockDim.x >= 1024 ? 512 : blockDim.x;
            const int ngroups = blockDim.x >= 1024 ? 2 : 1;
            for (int j = (ngroups == 2 ? half : 0); j < ncol; j += ngroups) {
                const u32 c = c0 + j;
                const size_t src = p.src ? p.src[c] : c;
                moe_stage_column(smem + (size_t)j * act_bytes, p.x + src * p.k,
                                 p.x2 ? p.x2 + src * p.k : nullptr, p.k, p.per,
                                 ngroups == 2 ? (int)threadIdx.x - 512 * half : (int)threadIdx.x, nth);
            }
        }
        __syncthreads();
        for (int r0 = row_lo + wave * RW; r0 < row_hi; r0 += nwaves * RW) {
            const int r = min(r0 + rw, row_hi - 1);
            float acc[JL_MOE_TB];
#pragma unroll
            for (int j = 0; j < JL_MOE_TB; j++) acc[j] = 0.f;
            for (int s = slot; s < nslots; s += LPR) {
                typename T::W w;
                T::load_w(sheet + (size_t)r * p.row_bytes, s, w);
#pragma unroll
                for (int j = 0; j < JL_MOE_TB; j++) {
                    if (j < ncol) {
                        typename T::Act a;
                        T::load_act(act_lds_views(smem + (size_t)j * act_bytes, p.k), s, a);
                        acc[j] += T::dot(w, s, a);
                    }
                }
            }
#pragma unroll
            for (int j = 0; j < JL_MOE_TB; j++) {
                if (j < ncol) {
                    float t = group_sum<LPR>(live ? acc[j] : 0.f);
                    if (slot == LPR - 1 && r0 + rw < row_hi) out[(size_t)(c0 + j) * p.nrows + r0 + rw] = t;
                }
            }
        }
        __syncthreads();
    }
}

// resid[r][n] += sum over the row's k_used experts, ascending expert id, of
// wt[r][s] * y[pos[r*k_used+s]][n].  One thread per (row, n).
__device__ __forceinline__ void moe_combine_body(const MoeCombineArgs& p) {
    const int n = blockIdx.x * blockDim.x + threadIdx.x;
    const int r = blockIdx.y;
    if (n >= p.n_embd) return;
    // order the row's slots by expert id (k_used is small: insertion sort in registers)
    int order[16];
    const int ku = p.k_used;
    for (int s = 0; s < ku; s++) order[s] = s;
    for (int i = 1; i < ku; i++)
        for (int j = i; j > 0 && p.sel[r * p.sel_stride + order[j]] < p.sel[r * p.sel_stride + order[j - 1]]; j--) {
            int t = order[j]; order[j] = order[j - 1]; order[j - 1] = t;
        }
    float acc = p.resid[(size_t)r * p.n_embd + n];
    for (int i = 0; i < ku; i++) {
        const int s = order[i];
        acc += p.wt[r * ku + s] * p.y[(size_t)p.pos[r * ku + s] * p.n_embd + n];
    }
    p.resid[(size_t)r * p.n_embd + n] = acc;
}
