// The gfx950 code object: every kernel entry point the C ABI launches through
// hipModuleLaunchKernel.  Built with
//   hipcc --genco --offload-arch=gfx950 -O3 -ffp-contract=off ...
// Entry points are extern "C" so the host can look them up by name.
#include "common.h"
#include "dequant.h"
#include "matvec.h"
#include "quantize.h"

extern __shared__ __attribute__((aligned(16))) uint8_t jl_smem[];

// ------------------------------------------------------------- quantizer
// x [ntok][k] f32 -> q [ntok][k] int8, as [ntok][k/32], sum16 [ntok][k/16].
// grid = (ceil(k/16/256), ntok), block = 256: one thread per 16 elements.
extern "C" __global__ __launch_bounds__(256) void jl_quantize_act(
    const float* __restrict__ x, int8_t* __restrict__ q, float* __restrict__ as,
    float* __restrict__ sum16, int k, int per) {
    const size_t tok = blockIdx.y;
    const int hb = blockIdx.x * 256 + threadIdx.x;
    const int nhb = k / 16;
    const bool live = hb < nhb;
    const f32x4* xt = (const f32x4*)(x + tok * (size_t)k);
    f32x4 v[4];
#pragma unroll
    for (int i = 0; i < 4; i++) v[i] = live ? xt[hb * 4 + i] : f32x4{0.f, 0.f, 0.f, 0.f};
    u32 amax = window_amax(half_block_amax(v), per);
    u32 qq[4];
    float d;
    i32 sum;
    quantize_half_block(v, amax, qq, d, sum);
    if (live) {
        ((u32x4*)(q + tok * (size_t)k))[hb] = u32x4{qq[0], qq[1], qq[2], qq[3]};
        sum16[tok * (size_t)nhb + hb] = (float)sum;
        if ((hb & 1) == 0) as[tok * (size_t)(k / 32) + (hb >> 1)] = d;
    }
}

// --------------------------------------------------------------- dequant
extern "C" __global__ __launch_bounds__(256) void jl_dequant(
    const uint8_t* __restrict__ src, float* __restrict__ dst, size_t n, int type) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) dst[i] = dequant_elem(type, src, i);
}

// ---------------------------------------------------------------- matvec
#define JL_MATVEC_KERNEL(NAME, TYPE, RPW, NI)                                        \
    extern "C" __global__ __launch_bounds__(1024) void NAME(MatVecArgs p) {          \
        matvec_body<TYPE, RPW, NI>(p, jl_smem);                                      \
    }

// (type, rows per wavefront, unrolled slot iterations per lane); only shapes that
// stay inside 128 VGPRs, so a 1024-thread workgroup fits.
#define K(T, TYPE, R, N) JL_MATVEC_KERNEL(jl_matvec_##T##_r##R##_n##N, TYPE, R, N)
K(q4k, JL_Q4_K, 1, 0) K(q4k, JL_Q4_K, 2, 0) K(q4k, JL_Q4_K, 4, 0)
K(q4k, JL_Q4_K, 1, 1) K(q4k, JL_Q4_K, 2, 1) K(q4k, JL_Q4_K, 4, 1)
K(q4k, JL_Q4_K, 1, 2) K(q4k, JL_Q4_K, 2, 2)
K(q8_0, JL_Q8_0, 1, 0) K(q8_0, JL_Q8_0, 2, 0) K(q8_0, JL_Q8_0, 4, 0)
K(q8_0, JL_Q8_0, 1, 1) K(q8_0, JL_Q8_0, 2, 1) K(q8_0, JL_Q8_0, 4, 1)
K(q8_0, JL_Q8_0, 1, 2) K(q8_0, JL_Q8_0, 2, 2) K(q8_0, JL_Q8_0, 1, 4)
K(q6k, JL_Q6_K, 1, 0) K(q6k, JL_Q6_K, 2, 0)
K(q6k, JL_Q6_K, 1, 1) K(q6k, JL_Q6_K, 2, 1) K(q6k, JL_Q6_K, 4, 1)
#undef K
