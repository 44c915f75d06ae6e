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
};

// Activation preparation for the Q4_K prefill GEMM: quantize x and lay it out
// as the GEMM's LDS stages, bq [k/256][2][tok_pad][152] f16, da [k/256][tok_pad].
struct GemmPrepArgs {
    const float* x;      // [ntok][k]
    uint16_t* bq;        // f16 bits
    float* da;
    int ntok, tok_pad, k;
};

struct GemmArgs {
    float* out;          // [ntok][nrows]
    const uint8_t* w;    // GGUF row-major Q4_K
    const uint16_t* bq;
    const float* da;
    int nrows, k, ntok, tok_pad;
    int row_bytes;
};
