// prefill.h -- launchers of the multi-token prefill kernels (prefill.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>

namespace mg {

// Elements of one bf16 plane of split activations for T rows of K (blocks of 128 rows x 64 k).
inline size_t split_plane_elems(int T, int K) { return (size_t)((T + 127) / 128) * 128 * (size_t)((K + 63) / 64) * 64; }
// Rows of `in` [T,K] (RMS-normalised with `gain` when it is not NULL) split into two bf16 planes, a = hi + lo,
// stored block by block in the order the GEMM reads them.
hipError_t launch_split_rows(const float* in, const float* gain, float eps, int T, int K, void* hi, void* lo, hipStream_t s);
// silu(gate) * up over [T,K], written as the hi/lo split.
hipError_t launch_swiglu_split(const float* gate, const float* up, int T, int K, void* hi, void* lo, hipStream_t s);
// RoPE on q rows in place; rotated k rows and v rows stored into cache rows pos0 .. pos0+T-1 (fp32 or fp16 caches).
hipError_t launch_rope_store_rows(float* q, const float* k, const float* v, void* Kc, void* Vc, int kvHalf, const float* cosTab,
                                  const float* sinTab, int pos0, int T, int dim, int kvDim, int headDim, hipStream_t s);
// Causal attention of T query rows [T,dim] (rotated) at positions pos0.. over cache rows [0, pos0+T); out [T,dim]
// and/or its hi/lo split for K = dim in launch_split_rows's layout (either may be NULL, not both).  The cache rows
// are first split into bf16 hi/lo planes in kvSplit, a workspace of prefill_kv_split_bytes(pos0 + T, kvDim) bytes
// (16-byte aligned) that the launch owns until it has finished.
size_t prefill_kv_split_bytes(int rows, int kvDim);
hipError_t launch_prefill_attention(const float* q, const void* Kc, const void* Vc, int kvHalf, void* kvSplit, float* out,
                                    void* splitHi, void* splitLo, int T, int pos0, int rowLimit, int dim, int kvDim, int nHeads,
                                    int nKVHeads, int headDim, hipStream_t s);
// Embedding rows of T tokens: kind 0 = Q8 row * scale, 1 = fp16 table, 2 = fp32 table, 3 = Q4_0 split-layout row.
hipError_t launch_embed_rows(int kind, const void* table, const float* scales, const int* tokens, float* x, int T, int dim,
                             int vocab, hipStream_t s);
// One launch: for each of up to three weight matrices, Y[T,N] (+)= (Ahi + Alo)[T,K] . W[N,K]^T * scales[n] (+ bias[n]).
// q4 = 0: W int8 [N,K] with float scales[N].  q4 = 1: W is Q4_0 in the split layout (16-byte nibble groups
// [N, K/32], then fp16 d [N, K/32]), scales NULL.
// K a multiple of 32; W, Ahi, Alo 16-byte aligned; Ahi/Alo in the blocked layout of launch_split_rows.
struct GemmSeg { const signed char* W; const float* scales; const float* bias; float* Y; int N; int tile0; };
struct GemmParams {
    GemmSeg seg[3];
    int nseg;
    const unsigned short* Ahi;
    const unsigned short* Alo;
    int T, K;
    int q4;
    float* partial;   // workspace of gemm_partial_floats() floats for K-split partial sums (NULL: never split K)
    // Optional (one matrix, residual form): when K was split, the kernel that sums the splits into Y also
    // writes the hi/lo split of the finished rows, RMS-normalised with nextGain (NULL: plain), for the
    // projection that follows -- into nextHi/nextLo, in launch_split_rows's layout for K = N.
    const float* nextGain;
    float nextEps;
    unsigned short* nextHi;
    unsigned short* nextLo;
    // Optional (q | k | v in one launch, plain form): when K was split, the kernel that sums the splits
    // also applies RoPE to the q and k rows and stores the k / v rows into the caches at pos0 + row
    // (what launch_rope_store_rows does); seg[0].Y still receives the rotated q rows, seg[1].Y / seg[2].Y
    // are not written then.
    void* ropeKc;
    void* ropeVc;
    const float* ropeCos;
    const float* ropeSin;
    int ropePos0, ropeHeadDim, ropeKvHalf;
    // Optional (gate | up in one launch, plain form): nextSwiglu != 0 asks for silu(gate) * up
    // (mongoose.cu:949-956) written as the hi/lo split for K = N into nextHi/nextLo (what launch_swiglu_split
    // does); seg[0].Y / seg[1].Y are not written when the launcher could do that (wroteNext = 1).
    int nextSwiglu;
    // filled by the launcher
    int nTiles, splitK, stepsPerSplit, ldPartial;
    int wroteNext;    // 1: nextHi/nextLo were written; 0: the caller still has to split Y's rows itself
    int wroteRope;    // 1: q rows rotated and K/V rows stored; 0: the caller still has to call launch_rope_store_rows
};
size_t gemm_partial_floats();
hipError_t launch_gemm_q8(GemmParams& p, int residual, hipStream_t s);

}  // namespace mg
