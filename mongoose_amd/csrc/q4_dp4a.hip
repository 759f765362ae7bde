// q4_dp4a.hip -- the integer form of the Q4_0 matvec: the activation vector is quantized to int8 blocks once and the
// dot products run on the packed int8 dot instruction (v_dot4_i32_i8), as the reference's dp4a kernels do
// (kernels.go:66-70, 985-1017; dispatch cuda_fused_infer_q4.go:611-673).
//
// The reference's CUDA bodies of these kernels are not in its tree; what its Go side fixes is the calling sequence and
// the size of the scratch buffer, (K/32)*40 bytes (cuda_fused_infer.go:176): 40 bytes per block of 32 activations,
// "Q8_1 blocks" (kernels.go:993).  The block here is GGML's Q8_1 with fp32 fields:
//     float d = max|x| / 127;  float s = d * sum(q);  int8 q[32] = round-half-away(x / d)      (zero block: d = s = 0)
// and a row of block_q4_0 weights against it is GGML's vec_dot_q4_0_q8_1:
//     out[r] = sum_b  f32(d4[r,b]) * ( d8[b] * sum_i nib[r,b,i] * q[b,i]  -  8 * s8[b] )
// with nib the unsigned nibbles in GGML element order (low nibble of byte j = element j, high nibble = element j+16).
// The integer sums are exact; only the activation rounding distinguishes the result from the fp32-activation matvec.
#include "kernels.h"
#include "device_util.h"

namespace mg {

// One thread per block of 32 activations (a vector has at most a few hundred blocks, a batch a few thousand).
__global__ __launch_bounds__(WG) void q8_quantize_act_kernel(const float* __restrict__ act, unsigned char* __restrict__ out, int nBlocks) {
    const int b = blockIdx.x * WG + threadIdx.x;
    if (b >= nBlocks) return;
    const float4* x4 = reinterpret_cast<const float4*>(act + (size_t)b * 32);
    float4 v[8];
#pragma unroll
    for (int i = 0; i < 8; i++) v[i] = x4[i];
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < 8; i++) amax = fmaxf(fmaxf(fmaxf(amax, fabsf(v[i].x)), fabsf(v[i].y)), fmaxf(fabsf(v[i].z), fabsf(v[i].w)));
    const float d = amax / 127.0f;
    const float id = d != 0.f ? 1.0f / d : 0.f;
    int q[8];
    int sum = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const int a = (int)roundf(v[i].x * id), b1 = (int)roundf(v[i].y * id), c = (int)roundf(v[i].z * id), e = (int)roundf(v[i].w * id);
        sum += a + b1 + c + e;
        q[i] = (a & 0xff) | ((b1 & 0xff) << 8) | ((c & 0xff) << 16) | ((e & 0xff) << 24);
    }
    unsigned char* o = out + (size_t)b * 40;                  // 8-byte aligned (the buffer is, and 40 is a multiple of 8)
    *reinterpret_cast<float2*>(o) = make_float2(d, d * (float)sum);
    int2* oq = reinterpret_cast<int2*>(o + 8);
#pragma unroll
    for (int i = 0; i < 4; i++) oq[i] = make_int2(q[2 * i], q[2 * i + 1]);
}

// A wave per row, a lane per block and step of 64 blocks.  PLANAR: the split layout of the context's resident matrices
// (nibble groups [N, K/32] of 16 bytes, then fp16 d [N, K/32]); otherwise raw GGUF 18-byte blocks (2-byte aligned).
// grid.y = vectors of the batch: activations q8 + y * (K/32) * 40, results out + y * N.
template <bool PLANAR>
__global__ __launch_bounds__(WG) void q4_0_dp4a_kernel(const unsigned char* __restrict__ w, const unsigned char* __restrict__ q8,
                                                       float* __restrict__ out, int N, int K) {
    const int lane = threadIdx.x & 63;
    const int r = blockIdx.x * (WG / 64) + (threadIdx.x >> 6);
    if (r >= N) return;
    const int nb = K >> 5;
    const unsigned char* a = q8 + (size_t)blockIdx.y * nb * 40;
    float acc = 0.f;
    for (int b = lane; b < nb; b += 64) {
        unsigned x[4];
        unsigned short hd;
        if (PLANAR) {
            const uint4 g = reinterpret_cast<const uint4*>(w)[(size_t)r * nb + b];
            x[0] = g.x; x[1] = g.y; x[2] = g.z; x[3] = g.w;
            hd = reinterpret_cast<const unsigned short*>(w + (size_t)N * (K >> 1))[(size_t)r * nb + b];
        } else {
            const unsigned short* h = reinterpret_cast<const unsigned short*>(w + ((size_t)r * nb + b) * 18);
            hd = h[0];
#pragma unroll
            for (int i = 0; i < 4; i++) x[i] = (unsigned)h[1 + 2 * i] | ((unsigned)h[2 + 2 * i] << 16);
        }
        const unsigned char* ab = a + (size_t)b * 40;
        const float2 ds = *reinterpret_cast<const float2*>(ab);
        const int2* aq = reinterpret_cast<const int2*>(ab + 8);
        int qv[8];
#pragma unroll
        for (int i = 0; i < 4; i++) { const int2 t = aq[i]; qv[2 * i] = t.x; qv[2 * i + 1] = t.y; }
        int sumi = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            sumi = __builtin_amdgcn_sdot4((int)(x[i] & 0x0f0f0f0fu), qv[i], sumi, false);             // elements 4i .. 4i+3
            sumi = __builtin_amdgcn_sdot4((int)((x[i] >> 4) & 0x0f0f0f0fu), qv[4 + i], sumi, false);   // elements 16+4i .. 16+4i+3
        }
        acc += half_bits_to_float(hd) * (ds.x * (float)sumi - 8.0f * ds.y);
    }
    acc = wave_sum(acc);
    if (lane == 0) out[(size_t)blockIdx.y * N + r] = acc;
}

hipError_t launch_q8_quantize_act(const float* act, void* q8out, int K, int batch, hipStream_t s) {
    if (K <= 0 || K % 32 || batch <= 0 || ((uintptr_t)act & 15) || ((uintptr_t)q8out & 7)) return hipErrorInvalidValue;
    const long long nBlocks = (long long)(K / 32) * batch;
    if (nBlocks > (1ll << 30)) return hipErrorInvalidValue;
    hipLaunchKernelGGL(q8_quantize_act_kernel, dim3((unsigned)((nBlocks + WG - 1) / WG)), dim3(WG), 0, s, act,
                       static_cast<unsigned char*>(q8out), (int)nBlocks);
    return hipGetLastError();
}

hipError_t launch_q4_0_dp4a(const void* w, bool planar, const void* q8, float* out, int N, int K, int batch, hipStream_t s) {
    if (N <= 0 || K <= 0 || K % 32 || batch <= 0 || batch > 65535 || ((uintptr_t)q8 & 7) || ((uintptr_t)w & (planar ? 15 : 1)))
        return hipErrorInvalidValue;
    const dim3 grid((unsigned)((N + WG / 64 - 1) / (WG / 64)), (unsigned)batch);
    if (planar) hipLaunchKernelGGL(q4_0_dp4a_kernel<true>, grid, dim3(WG), 0, s, static_cast<const unsigned char*>(w),
                                   static_cast<const unsigned char*>(q8), out, N, K);
    else hipLaunchKernelGGL(q4_0_dp4a_kernel<false>, grid, dim3(WG), 0, s, static_cast<const unsigned char*>(w),
                            static_cast<const unsigned char*>(q8), out, N, K);
    return hipGetLastError();
}

// (max, lowest index) of contiguous slices of a vector, one per workgroup: the partials argmax_finish takes.
__global__ __launch_bounds__(WG) void argmax_slices_kernel(const float* __restrict__ x, int n, float* __restrict__ pv, int* __restrict__ pi) {
    __shared__ float sv[WG / 64];
    __shared__ int si[WG / 64];
    const int per = (n + gridDim.x - 1) / gridDim.x;
    const int i0 = blockIdx.x * per, i1 = min(n, i0 + per);
    float v = -INFINITY;
    int idx = INT_MAX;
    for (int i = i0 + threadIdx.x; i < i1; i += WG) argmax_pick(v, idx, x[i], i);
    wave_argmax(v, idx);
    if ((threadIdx.x & 63) == 0) { sv[threadIdx.x >> 6] = v; si[threadIdx.x >> 6] = idx; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int k = 1; k < WG / 64; k++) argmax_pick(v, idx, sv[k], si[k]);
        pv[blockIdx.x] = v;
        pi[blockIdx.x] = idx;
    }
}
hipError_t launch_argmax_slices(const float* x, int n, int nparts, float* pv, int* pi, hipStream_t s) {
    if (n <= 0 || nparts <= 0) return hipErrorInvalidValue;
    hipLaunchKernelGGL(argmax_slices_kernel, dim3((unsigned)nparts), dim3(WG), 0, s, x, n, pv, pi);
    return hipGetLastError();
}

}  // namespace mg
