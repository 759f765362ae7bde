// prefill.h -- launchers of the multi-token prefill kernels (prefill.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>

namespace mg {

// Rows of `in` [T,K] (RMS-normalised with `gain` when it is not NULL) split into two bf16 planes, a = hi + lo.
hipError_t launch_split_rows(const float* in, const float* gain, float eps, int T, int K, void* hi, void* lo, hipStream_t s);
// silu(gate) * up over n elements, written as the hi/lo split.
hipError_t launch_swiglu_split(const float* gate, const float* up, size_t n, void* hi, void* lo, hipStream_t s);
// RoPE on q rows in place; rotated k rows and v rows stored into cache rows pos0 .. pos0+T-1.
hipError_t launch_rope_store_rows(float* q, const float* k, const float* v, float* Kc, float* Vc, const float* cosTab,
                                  const float* sinTab, int pos0, int T, int dim, int kvDim, int headDim, hipStream_t s);
// Embedding rows of T tokens: kind 0 = Q8 row * scale, 1 = fp16 table, 2 = fp32 table.
hipError_t launch_embed_rows(int kind, const void* table, const float* scales, const int* tokens, float* x, int T, int dim,
                             int vocab, hipStream_t s);
// Y[T,N] (+)= (Ahi + Alo)[T,K] . W[N,K]^T * scales[n] (+ bias[n]); K a multiple of 32.
hipError_t launch_gemm_q8(const void* Ahi, const void* Alo, const void* W, const float* scales, const float* bias, float* Y,
                          int T, int N, int K, int residual, hipStream_t s);

}  // namespace mg
