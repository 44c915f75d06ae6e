// The static device workspace behind jl_matmul_static_dev (scratch.hip).
#pragma once
#include <stddef.h>

// Its size: enough for every Q4_K / Q6_K / Q8_0 prefill matmul up to 512 tokens of 4096
// features against 14336 rows (activation fragments 4.7 MiB, K-split partial sums up to 32 MiB)
// and for 2048 tokens of 4096 features wherever no K split is needed (fragments 18.1 MiB).
// The array is part of the library's device image: every GPU the process touches holds it from
// the moment the library is loaded, used or not.
#define JL_STATIC_SCRATCH_BYTES ((size_t)64 << 20)

extern "C" int jl_static_scratch_get(int device, void** ptr, size_t* bytes, const char** err);
