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

// The split activations are stored in the order the GEMM walks them: blocks of
// 128 rows x 64 k (16 KB per plane), block (t/128, k/64) at ((t/128)*ceil(K/64) + k/64) * 8192
// elements, so one K step of a workgroup is one contiguous read.
__device__ __forceinline__ size_t tiled_index(int t, int k, int K) {
    const int ksteps = (K + 63) >> 6;
    return ((size_t)(t >> 7) * ksteps + (k >> 6)) * 8192 + (size_t)(t & 127) * 64 + (k & 63);
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
        const size_t o = tiled_index(blockIdx.x, i, K);
        hi[o] = h;
        lo[o] = f32_to_bf16_rne(a - bf16_to_f32(h));
    }
}
hipError_t launch_split_rows(const float* in, const float* gain, float eps, int T, int K, void* hi, void* lo, hipStream_t s) {
    if (T <= 0) return hipSuccess;
    hipLaunchKernelGGL(split_rows_kernel, dim3(T), dim3(PWG), 0, s, in, gain, eps, K,
                       static_cast<unsigned short*>(hi), static_cast<unsigned short*>(lo));
    return hipGetLastError();
}

// SiLU(gate)*up (mongoose.cu:949-956) over [T, n], written as the hi/lo split the down GEMM reads.
__global__ void swiglu_split_kernel(const float* gate, const float* up, int K, unsigned short* hi, unsigned short* lo) {
    const int t = blockIdx.y;
    const int k = blockIdx.x * blockDim.x + threadIdx.x;
    if (k >= K) return;
    float g = gate[(size_t)t * K + k];
    float a = g * (1.0f / (1.0f + expf(-g))) * up[(size_t)t * K + k];
    unsigned short h = f32_to_bf16_rne(a);
    const size_t o = tiled_index(t, k, K);
    hi[o] = h;
    lo[o] = f32_to_bf16_rne(a - bf16_to_f32(h));
}
hipError_t launch_swiglu_split(const float* gate, const float* up, int T, int K, void* hi, void* lo, hipStream_t s) {
    if (T <= 0 || K <= 0) return hipSuccess;
    hipLaunchKernelGGL(swiglu_split_kernel, dim3((unsigned)((K + PWG - 1) / PWG), (unsigned)T), dim3(PWG), 0, s, gate, up, K,
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
// GEMM on v_mfma_f32_32x32x16_bf16.  Workgroup tile BM (T) x 128 (N), K in
// steps of 64; four waves as 2x2, each (BM/2)x64 = (BM/64)x2 MFMA blocks, the
// hi and the lo activation term against the same weight fragment.  Fragment
// layouts (lane l):
//   A: row l%32, k = 8*(l/32)..+7        B: col l%32, k = 8*(l/32)..+7
//   C: col l%32, rows 8*(i/4) + 4*(l/32) + i%4 for i = 0..15
// Up to three weight matrices (q/k/v, gate/up) share one launch.  Workgroups
// that share a weight tile are placed on one XCD (ids congruent mod 8), so the
// tile comes into that XCD's L2 once.
// ---------------------------------------------------------------------------
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
constexpr int BN = 128, BK = 64;
constexpr int A_STRIDE = BK + 8;    // bf16 per LDS row (144 bytes)
constexpr int B_STRIDE = BK + 16;   // bytes per LDS row of int8 weights (80)

__device__ __forceinline__ unsigned pack_bf16_exact(float lo, float hi) {
    // both floats hold small integers: their low 16 bits are zero, truncation is exact
    return (__builtin_bit_cast(unsigned, lo) >> 16) | (__builtin_bit_cast(unsigned, hi) & 0xffff0000u);
}

template <int BM, int EPI>   // EPI 0: Y = acc*scale (+bias)   1: Y += acc*scale (residual in place)
__global__ __launch_bounds__(PWG) void gemm_q8_bf16x2_kernel(GemmParams p) {
    constexpr int MI = BM / 64;                  // 32-row MFMA blocks per wave
    constexpr int AR = BM / 32;                  // 16-byte segments per thread and A plane (BM*8 segments / 256)
    __shared__ __attribute__((aligned(16))) unsigned short sAh[BM * A_STRIDE];
    __shared__ __attribute__((aligned(16))) unsigned short sAl[BM * A_STRIDE];
    __shared__ __attribute__((aligned(16))) signed char sB[BN * B_STRIDE];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int numM = (p.T + BM - 1) / BM;
    const int L = blockIdx.x;
    const int grp = L / (8 * numM), rem = L % (8 * numM);
    const int nTile = grp * 8 + (rem & 7), mTile = rem >> 3;
    if (nTile >= p.nTiles) return;
    int sgi = 0;
    if (p.nseg > 1 && nTile >= p.seg[1].tile0) sgi = 1;
    if (p.nseg > 2 && nTile >= p.seg[2].tile0) sgi = 2;
    const GemmSeg sg = p.seg[sgi];
    const int N = sg.N, K = p.K, T = p.T;
    const int m0 = mTile * BM, n0 = (nTile - sg.tile0) * BN;

    // global -> LDS: A row = tid/8 + 32*r, segment tid%8 (8 bf16) ; B row = tid/4 + 64*r, segment tid%4 (16 int8)
    const int aRow = tid >> 3, aSeg = tid & 7;
    const int bRow = tid >> 2, bSeg = tid & 3;
    const unsigned short* aHiP[AR]; const unsigned short* aLoP[AR];
    const int ksteps = (K + BK - 1) / BK;
#pragma unroll
    for (int r = 0; r < AR; r++) {         // rows past T exist in the padded planes; their results are dropped
        const int row = m0 + aRow + 32 * r;
        const size_t o = (size_t)(row >> 7) * ksteps * 8192 + (size_t)(row & 127) * 64 + aSeg * 8;
        aHiP[r] = p.Ahi + o;
        aLoP[r] = p.Alo + o;
    }
    const signed char* bP[2];
#pragma unroll
    for (int r = 0; r < 2; r++) bP[r] = sg.W + (size_t)min(n0 + bRow + 64 * r, N - 1) * K + bSeg * 16;

    float16_t acc[MI][2];
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.f;

    int4 gAh[AR], gAl[AR], gB[2];
    const int4 zero4 = make_int4(0, 0, 0, 0);
    auto gload = [&](int k0) {       // K is a multiple of 32: a last half step reads zeros past the end
        const bool okA = k0 + aSeg * 8 < K, okB = k0 + bSeg * 16 < K;
#pragma unroll
        for (int r = 0; r < AR; r++) {
            gAh[r] = okA ? *reinterpret_cast<const int4*>(aHiP[r] + (size_t)k0 * 128) : zero4;   // 8192 elements per K step
            gAl[r] = okA ? *reinterpret_cast<const int4*>(aLoP[r] + (size_t)k0 * 128) : zero4;
        }
#pragma unroll
        for (int r = 0; r < 2; r++) gB[r] = okB ? *reinterpret_cast<const int4*>(bP[r] + k0) : zero4;
    };
    gload(0);
    for (int k0 = 0; k0 < K; k0 += BK) {
        __syncthreads();                       // the previous step's fragments are consumed
#pragma unroll
        for (int r = 0; r < AR; r++) {
            *reinterpret_cast<int4*>(&sAh[(aRow + 32 * r) * A_STRIDE + aSeg * 8]) = gAh[r];
            *reinterpret_cast<int4*>(&sAl[(aRow + 32 * r) * A_STRIDE + aSeg * 8]) = gAl[r];
        }
#pragma unroll
        for (int r = 0; r < 2; r++) *reinterpret_cast<int4*>(&sB[(bRow + 64 * r) * B_STRIDE + bSeg * 16]) = gB[r];
        __syncthreads();
        if (k0 + BK < K) gload(k0 + BK);       // next tile in flight while this one is multiplied
#pragma unroll
        for (int ks = 0; ks < BK / 16; ks++) {
            const int kk = ks * 16 + 8 * (lane >> 5);
            bf16x8_t b[2];
#pragma unroll
            for (int j = 0; j < 2; j++) {
                int2 w = *reinterpret_cast<const int2*>(&sB[(wn * 64 + j * 32 + (lane & 31)) * B_STRIDE + kk]);
                uint4 u;
                u.x = pack_bf16_exact((float)(signed char)(w.x), (float)(signed char)(w.x >> 8));
                u.y = pack_bf16_exact((float)(signed char)(w.x >> 16), (float)(w.x >> 24));
                u.z = pack_bf16_exact((float)(signed char)(w.y), (float)(signed char)(w.y >> 8));
                u.w = pack_bf16_exact((float)(signed char)(w.y >> 16), (float)(w.y >> 24));
                b[j] = __builtin_bit_cast(bf16x8_t, u);
            }
#pragma unroll
            for (int i = 0; i < MI; i++) {
                const int arow = (wm * (BM / 2) + i * 32 + (lane & 31)) * A_STRIDE + kk;
                bf16x8_t ah = *reinterpret_cast<const bf16x8_t*>(&sAh[arow]);
                bf16x8_t al = *reinterpret_cast<const bf16x8_t*>(&sAl[arow]);
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, b[j], acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al, b[j], acc[i][j], 0, 0, 0);
                }
            }
        }
    }
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int n = n0 + wn * 64 + j * 32 + (lane & 31);
        if (n >= N) continue;
        const float sc = sg.scales[n];
        const float bi = sg.bias ? sg.bias[n] : 0.f;
#pragma unroll
        for (int i = 0; i < MI; i++) {
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const int m = m0 + wm * (BM / 2) + i * 32 + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
                if (m < T) {
                    float v = acc[i][j][e] * sc + bi;
                    float* dst = sg.Y + (size_t)m * N + n;
                    if (EPI == 1) v = *dst + v;
                    *dst = v;
                }
            }
        }
    }
}

hipError_t launch_gemm_q8(GemmParams& p, int residual, hipStream_t s) {
    if (p.T <= 0 || p.nseg < 1 || p.nseg > 3) return p.T <= 0 ? hipSuccess : hipErrorInvalidValue;
    if (p.K <= 0 || p.K % 32 != 0) return hipErrorInvalidValue;
    int tiles = 0;
    for (int i = 0; i < p.nseg; i++) {
        if (p.seg[i].N <= 0) return hipErrorInvalidValue;
        p.seg[i].tile0 = tiles;
        tiles += (p.seg[i].N + BN - 1) / BN;
    }
    p.nTiles = tiles;
    // 128-row tiles once they fill the chip, 64-row tiles below that
    const int numM128 = (p.T + 127) / 128;
    const bool big = (long long)numM128 * tiles >= 512;
    const int numM = big ? numM128 : (p.T + 63) / 64;
    dim3 grid((unsigned)(((tiles + 7) / 8) * 8 * numM));
    if (big) {
        if (residual) hipLaunchKernelGGL((gemm_q8_bf16x2_kernel<128, 1>), grid, dim3(PWG), 0, s, p);
        else hipLaunchKernelGGL((gemm_q8_bf16x2_kernel<128, 0>), grid, dim3(PWG), 0, s, p);
    } else {
        if (residual) hipLaunchKernelGGL((gemm_q8_bf16x2_kernel<64, 1>), grid, dim3(PWG), 0, s, p);
        else hipLaunchKernelGGL((gemm_q8_bf16x2_kernel<64, 0>), grid, dim3(PWG), 0, s, p);
    }
    return hipGetLastError();
}

}  // namespace mg
