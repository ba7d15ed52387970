// MFMA path (5 <= M) of the GGUF Q4_0 / Q8_0 / Q5_K / Q6_K GEMVs: the weight-streaming
// skinny kernel instantiated for those formats (fp16 activations).
#pragma once
#include <hip/hip_runtime.h>

namespace qlin {

// fmt: 3 = Q4_0, 4 = Q8_0, 5 = Q5_K, 6 = Q6_K (the format numbers of gemv_rows.hpp).
// h = tile-shuffled high bits (Q5_K / Q6_K), z = mins (Q5_K); otherwise null.
// Rows are processed 64 at a time, each pass streaming the weight once.
int gguf_skinny(int fmt, const void* x, const void* w, const void* h, const void* s, const void* z, void* out,
                int M, int N, int K, hipStream_t st);

// Whether gguf_skinny would run the register-resident K-sliced kernel (Q4_0 / Q8_0, few rows,
// K % 128 == 0): with 3 or 4 rows that kernel is ahead of the row kernel for Q4_0.
bool gguf_skinny_resident(int fmt, int M, int K);

}  // namespace qlin
