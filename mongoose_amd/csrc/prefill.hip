// prefill.hip -- multi-token prefill for the Q8 path: the one place where the
// work is a dense GEMM, so it runs on the matrix cores (MFMA).
//
// Y[T,N] = A[T,K] . W[N,K]^T with W int8 (per-row scale) and A fp32.  An int8
// value is exact in bf16, so the weights go to the matrix cores without loss;
// an fp32 activation is split into two bf16 terms a = hi + lo (|a - hi - lo| <=
// 2^-16 |a|), which costs two MFMAs per tile instead of one and keeps the
// result within ~1e-5 of the fp32 decode path (a single bf16 term would be off
// by ~4e-3).  Accumulation is fp32; the row scale is applied once at the end.
// Reference semantics: the same layer as the decode step, applied to T rows
// (causal attention as kernels/mongoose.cu:251-353 does for training).
#include "kernels.h"
#include "prefill.h"

namespace mg {

typedef short short4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int PWG = 256;

__device__ __forceinline__ unsigned short f32_to_bf16_rne(float f) {
    unsigned u = __builtin_bit_cast(unsigned, f);
    u += 0x7fffu + ((u >> 16) & 1u);          // round to nearest even (inputs are finite)
    return (unsigned short)(u >> 16);
}
__device__ __forceinline__ float bf16_to_f32(unsigned short h) {
    return __builtin_bit_cast(float, (unsigned)h << 16);
}
__device__ __forceinline__ float block_sum256(float v, float* red) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float t = (red[0] + red[1]) + (red[2] + red[3]);
    __syncthreads();
    return t;
}

// Row-wise: optional RMSNorm (x * 1/sqrt(mean(x^2)+eps) * g, the decode step's
// order of operations), then the hi/lo bf16 split.  One workgroup per row.
__global__ __launch_bounds__(PWG) void split_rows_kernel(const float* in, const float* gain, float eps, int K,
                                                        unsigned short* hi, unsigned short* lo) {
    __shared__ float red[4];
    const float* x = in + (size_t)blockIdx.x * K;
    float rs = 1.0f;
    if (gain) {
        float ss = 0.f;
        for (int i = threadIdx.x; i < K; i += PWG) ss += x[i] * x[i];
        float tot = block_sum256(ss, red);
        rs = 1.0f / sqrtf(tot / (float)K + eps);
    }
    for (int i = threadIdx.x; i < K; i += PWG) {
        float a = gain ? x[i] * rs * gain[i] : x[i];
        unsigned short h = f32_to_bf16_rne(a);
        hi[(size_t)blockIdx.x * K + i] = h;
        lo[(size_t)blockIdx.x * K + i] = f32_to_bf16_rne(a - bf16_to_f32(h));
    }
}
hipError_t launch_split_rows(const float* in, const float* gain, float eps, int T, int K, void* hi, void* lo, hipStream_t s) {
    if (T <= 0) return hipSuccess;
    hipLaunchKernelGGL(split_rows_kernel, dim3(T), dim3(PWG), 0, s, in, gain, eps, K,
                       static_cast<unsigned short*>(hi), static_cast<unsigned short*>(lo));
    return hipGetLastError();
}

// SiLU(gate)*up (mongoose.cu:949-956) over [T, n], written as the hi/lo split the down GEMM reads.
__global__ void swiglu_split_kernel(const float* gate, const float* up, size_t n, unsigned short* hi, unsigned short* lo) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float g = gate[i];
    float a = g * (1.0f / (1.0f + expf(-g))) * up[i];
    unsigned short h = f32_to_bf16_rne(a);
    hi[i] = h;
    lo[i] = f32_to_bf16_rne(a - bf16_to_f32(h));
}
hipError_t launch_swiglu_split(const float* gate, const float* up, size_t n, void* hi, void* lo, hipStream_t s) {
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(swiglu_split_kernel, dim3((unsigned)((n + PWG - 1) / PWG)), dim3(PWG), 0, s, gate, up, n,
                       static_cast<unsigned short*>(hi), static_cast<unsigned short*>(lo));
    return hipGetLastError();
}

// RoPE (mongoose.cu:991-1006) on the q and k rows of T positions and the K/V
// rows stored into the caches (mongoose.cu:1644-1647).  One workgroup per row.
__global__ void rope_store_rows_kernel(float* q, const float* k, const float* v, float* Kc, float* Vc,
                                       const float* cosTab, const float* sinTab, int pos0, int dim, int kvDim, int headDim) {
    const int t = blockIdx.x, pos = pos0 + t, half = headDim / 2;
    const float* c = cosTab + (size_t)pos * half;
    const float* s = sinTab + (size_t)pos * half;
    float* qr = q + (size_t)t * dim;
    for (int i = threadIdx.x; i < dim / 2; i += blockDim.x) {
        int h = i / half, j = i % half;
        float x0 = qr[h * headDim + j], x1 = qr[h * headDim + half + j];
        qr[h * headDim + j] = x0 * c[j] - x1 * s[j];
        qr[h * headDim + half + j] = x0 * s[j] + x1 * c[j];
    }
    const float* kr = k + (size_t)t * kvDim;
    const float* vr = v + (size_t)t * kvDim;
    float* kd = Kc + (size_t)pos * kvDim;
    float* vd = Vc + (size_t)pos * kvDim;
    for (int i = threadIdx.x; i < kvDim / 2; i += blockDim.x) {
        int h = i / half, j = i % half;
        float x0 = kr[h * headDim + j], x1 = kr[h * headDim + half + j];
        kd[h * headDim + j] = x0 * c[j] - x1 * s[j];
        kd[h * headDim + half + j] = x0 * s[j] + x1 * c[j];
    }
    for (int i = threadIdx.x; i < kvDim; i += blockDim.x) vd[i] = vr[i];
}
hipError_t launch_rope_store_rows(float* q, const float* k, const float* v, float* Kc, float* Vc, const float* cosTab,
                                  const float* sinTab, int pos0, int T, int dim, int kvDim, int headDim, hipStream_t s) {
    if (T <= 0) return hipSuccess;
    hipLaunchKernelGGL(rope_store_rows_kernel, dim3(T), dim3(PWG), 0, s, q, k, v, Kc, Vc, cosTab, sinTab, pos0, dim, kvDim, headDim);
    return hipGetLastError();
}

// Embedding rows of T tokens from the tied Q8 table (kind 0) or an fp16 (1) / fp32 (2) table.
__global__ void embed_rows_kernel(int kind, const void* table, const float* scales, const int* tokens, float* x, int dim, int vocab) {
    int tok = tokens[blockIdx.x];
    tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
    float* o = x + (size_t)blockIdx.x * dim;
    for (int i = threadIdx.x; i < dim; i += blockDim.x) {
        if (kind == 0) o[i] = (float)static_cast<const signed char*>(table)[(size_t)tok * dim + i] * scales[tok];
        else if (kind == 1) o[i] = (float)__builtin_bit_cast(_Float16, static_cast<const unsigned short*>(table)[(size_t)tok * dim + i]);
        else o[i] = static_cast<const float*>(table)[(size_t)tok * dim + i];
    }
}
hipError_t launch_embed_rows(int kind, const void* table, const float* scales, const int* tokens, float* x, int T, int dim,
                             int vocab, hipStream_t s) {
    if (T <= 0) return hipSuccess;
    hipLaunchKernelGGL(embed_rows_kernel, dim3(T), dim3(PWG), 0, s, kind, table, scales, tokens, x, dim, vocab);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// GEMM on v_mfma_f32_32x32x8_bf16_1k.  Workgroup tile 128 (T) x 128 (N), K in
// steps of 32; four waves as 2x2, each 64x64 = 2x2 MFMA blocks, hi and lo
// activations against the same weight fragment.  Fragment layouts (lane l):
//   A: row l%32, k = 4*(l/32)..+3        B: col l%32, k = 4*(l/32)..+3
//   C: col l%32, rows 8*(i/4) + 4*(l/32) + i%4 for i = 0..15
// ---------------------------------------------------------------------------
constexpr int BM = 128, BN = 128, BK = 32;
constexpr int A_STRIDE = 40;   // bf16 per LDS row (80 bytes: 16-byte aligned, spreads banks)
constexpr int B_STRIDE = 48;   // bytes per LDS row of int8 weights

template <int EPI>   // 0: Y = acc*scale (+bias)   1: Y += acc*scale (residual in place)
__global__ __launch_bounds__(PWG) void gemm_q8_bf16x2_kernel(const unsigned short* Ahi, const unsigned short* Alo,
                                                            const signed char* W, const float* scales, const float* bias,
                                                            float* Y, int T, int N, int K) {
    __shared__ __attribute__((aligned(16))) unsigned short sAh[BM * A_STRIDE];
    __shared__ __attribute__((aligned(16))) unsigned short sAl[BM * A_STRIDE];
    __shared__ __attribute__((aligned(16))) signed char sB[BN * B_STRIDE];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;

    // global -> LDS assignment: A: row = tid/4 + 64*r, 16-byte segment tid%4 ; B: row = tid/2, segment tid%2
    const int aRow = tid >> 2, aSeg = tid & 3;
    const int bRow = tid >> 1, bSeg = tid & 1;
    const int bRowG = min(n0 + bRow, N - 1);

    float16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.f;

    int4 gAh[2], gAl[2], gB;
    auto gload = [&](int k0) {
#pragma unroll
        for (int r = 0; r < 2; r++) {
            int row = min(m0 + aRow + 64 * r, T - 1);
            gAh[r] = *reinterpret_cast<const int4*>(Ahi + (size_t)row * K + k0 + aSeg * 8);
            gAl[r] = *reinterpret_cast<const int4*>(Alo + (size_t)row * K + k0 + aSeg * 8);
        }
        gB = *reinterpret_cast<const int4*>(W + (size_t)bRowG * K + k0 + bSeg * 16);
    };
    gload(0);
    for (int k0 = 0; k0 < K; k0 += BK) {
        __syncthreads();                       // previous step's fragments are consumed
#pragma unroll
        for (int r = 0; r < 2; r++) {
            *reinterpret_cast<int4*>(&sAh[(aRow + 64 * r) * A_STRIDE + aSeg * 8]) = gAh[r];
            *reinterpret_cast<int4*>(&sAl[(aRow + 64 * r) * A_STRIDE + aSeg * 8]) = gAl[r];
        }
        *reinterpret_cast<int4*>(&sB[bRow * B_STRIDE + bSeg * 16]) = gB;
        __syncthreads();
        if (k0 + BK < K) gload(k0 + BK);       // next tile in flight while this one is multiplied
#pragma unroll
        for (int ks = 0; ks < BK / 8; ks++) {
            const int kk = ks * 8 + 4 * (lane >> 5);
            short4_t b[2];
#pragma unroll
            for (int j = 0; j < 2; j++) {
                int w = *reinterpret_cast<const int*>(&sB[(wn * 64 + j * 32 + (lane & 31)) * B_STRIDE + kk]);
                // int8 -> float -> bf16: exact, the float's low 16 bits are zero
                unsigned f0 = __builtin_bit_cast(unsigned, (float)(int)(signed char)(w & 0xff));
                unsigned f1 = __builtin_bit_cast(unsigned, (float)(int)(signed char)((w >> 8) & 0xff));
                unsigned f2 = __builtin_bit_cast(unsigned, (float)(int)(signed char)((w >> 16) & 0xff));
                unsigned f3 = __builtin_bit_cast(unsigned, (float)(w >> 24));
                b[j][0] = (short)(f0 >> 16); b[j][1] = (short)(f1 >> 16);
                b[j][2] = (short)(f2 >> 16); b[j][3] = (short)(f3 >> 16);
            }
#pragma unroll
            for (int i = 0; i < 2; i++) {
                const int arow = (wm * 64 + i * 32 + (lane & 31)) * A_STRIDE + kk;
                short4_t ah = *reinterpret_cast<const short4_t*>(&sAh[arow]);
                short4_t al = *reinterpret_cast<const short4_t*>(&sAl[arow]);
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(ah, b[j], acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(al, b[j], acc[i][j], 0, 0, 0);
                }
            }
        }
    }
    // epilogue
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int n = n0 + wn * 64 + j * 32 + (lane & 31);
        if (n >= N) continue;
        const float sc = scales[n];
        const float bi = bias ? bias[n] : 0.f;
#pragma unroll
        for (int i = 0; i < 2; i++) {
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const int m = m0 + wm * 64 + i * 32 + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
                if (m < T) {
                    float v = acc[i][j][e] * sc + bi;
                    float* dst = Y + (size_t)m * N + n;
                    if (EPI == 1) v = *dst + v;
                    *dst = v;
                }
            }
        }
    }
}

hipError_t launch_gemm_q8(const void* Ahi, const void* Alo, const void* W, const float* scales, const float* bias, float* Y,
                          int T, int N, int K, int residual, hipStream_t s) {
    if (T <= 0 || N <= 0) return hipSuccess;
    if (K % BK != 0) return hipErrorInvalidValue;
    dim3 grid((N + BN - 1) / BN, (T + BM - 1) / BM);
    if (residual)
        hipLaunchKernelGGL((gemm_q8_bf16x2_kernel<1>), grid, dim3(PWG), 0, s, static_cast<const unsigned short*>(Ahi),
                           static_cast<const unsigned short*>(Alo), static_cast<const signed char*>(W), scales, bias, Y, T, N, K);
    else
        hipLaunchKernelGGL((gemm_q8_bf16x2_kernel<0>), grid, dim3(PWG), 0, s, static_cast<const unsigned short*>(Ahi),
                           static_cast<const unsigned short*>(Alo), static_cast<const signed char*>(W), scales, bias, Y, T, N, K);
    return hipGetLastError();
}

}  // namespace mg
