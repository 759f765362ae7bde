// kernels.hip -- gfx950 device code for mongoose's batch-1 quantized decode
// step: dequantizing matvec (Q8 per-row scale, GGUF Q4_0), RMSNorm, RoPE,
// GQA decode attention over an fp32 KV cache, SwiGLU, embedding gather and
// greedy argmax.  Reference arithmetic: kernels/mongoose.cu (cited per kernel).
//
// Everything here is HBM-bound byte streaming.  The matvec reads each weight
// byte once with 16-byte loads, keeps the activation vector in LDS in a
// conflict-free "planar" order, accumulates in fp32 and applies the row scale
// once in the epilogue; norm, bias, residual, SiLU*mul and argmax are folded
// into its prologue/epilogue so a layer is five launches instead of seventeen.
#include "kernels.h"
#include <limits.h>
#include <math.h>

namespace mg {

constexpr int WG = 256;

// ---------------------------------------------------------------------------
// wave64 / workgroup reductions
// ---------------------------------------------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
// Sum over the 256 threads of a workgroup; every thread gets the result.
// red: 4 floats of LDS.  Two barriers, so red can be reused right after.
__device__ __forceinline__ float block_sum(float v, float* red) {
    v = wave_sum(v);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float t = (red[0] + red[1]) + (red[2] + red[3]);
    __syncthreads();
    return t;
}
__device__ __forceinline__ float block_max(float v, float* red) {
    v = wave_max(v);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float t = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    __syncthreads();
    return t;
}

// ---------------------------------------------------------------------------
// Activation vector in LDS.  A lane that owns weight chunk c (CH consecutive
// weights) needs activations [c*CH, c*CH+CH).  Stored linearly, neighbouring
// lanes would read float4s CH*4 bytes apart and collide on LDS banks, so the
// vector is stored as CH/4 planes: plane p holds, for every chunk c, the float4
// a[c*CH+4p .. +3] at float4 index p*nch + c.  Lane reads are then 16 bytes
// apart: conflict free.
// ---------------------------------------------------------------------------
template <int CH>
__device__ __forceinline__ int act_slot4(int k4, int nch) {   // k4 = k/4 -> float4 index
    constexpr int P = CH / 4;
    int c = k4 / P, p = k4 % P;
    return p * nch + c;
}

template <int CH>
__device__ void stage_activation(const MvParams& p, int pro, float4* a4, float* red) {
    const int K4 = p.K >> 2;
    const int nch = p.K / CH;
    const int tid = threadIdx.x;
    if (pro == PRO_PLAIN) {
        const float4* x4 = reinterpret_cast<const float4*>(p.act);
        for (int i = tid; i < K4; i += WG) a4[act_slot4<CH>(i, nch)] = x4[i];
    } else if (pro == PRO_RMS) {
        // mongoose.cu:145-174 / cpu.go:36-47: x * (1/sqrt(mean(x^2)+eps)) * g
        const float4* x4 = reinterpret_cast<const float4*>(p.act);
        const float4* g4 = reinterpret_cast<const float4*>(p.gain);
        float ss = 0.f;
        for (int i = tid; i < K4; i += WG) {
            float4 v = x4[i];
            ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
        }
        float tot = block_sum(ss, red);
        float rs = 1.0f / sqrtf(tot / (float)p.K + p.eps);
        for (int i = tid; i < K4; i += WG) {
            float4 v = x4[i], g = g4[i], o;
            o.x = v.x * rs * g.x; o.y = v.y * rs * g.y; o.z = v.z * rs * g.z; o.w = v.w * rs * g.w;
            a4[act_slot4<CH>(i, nch)] = o;
        }
    } else {
        // Combine split-KV attention partials: out = sum_s e^(m_s-M) acc_s / sum_s e^(m_s-M) l_s
        int pos = p.state ? p.state->pos : p.posImm;
        int len = pos + 1;
        int splitLen = attn_split_len(len, p.smax, p.minSplit);
        int nsplit = (len + splitLen - 1) / splitLen;
        const int hd4 = p.headDim >> 2;
        for (int i = tid; i < K4; i += WG) {
            int h = i / hd4, d4 = i % hd4;
            const float* pm = p.pm + (size_t)h * p.smax;
            const float* pl = p.pl + (size_t)h * p.smax;
            float M = pm[0];
            for (int s = 1; s < nsplit; s++) M = fmaxf(M, pm[s]);
            float den = 0.f;
            float4 num = make_float4(0.f, 0.f, 0.f, 0.f);
            for (int s = 0; s < nsplit; s++) {
                float w = nsplit == 1 ? 1.0f : expf(pm[s] - M);
                den += w * pl[s];
                float4 a = reinterpret_cast<const float4*>(p.pacc + ((size_t)h * p.smax + s) * p.headDim)[d4];
                num.x += w * a.x; num.y += w * a.y; num.z += w * a.z; num.w += w * a.w;
            }
            float4 o;
            o.x = num.x / den; o.y = num.y / den; o.z = num.z / den; o.w = num.w / den;
            a4[act_slot4<CH>(i, nch)] = o;
        }
    }
}

// ---------------------------------------------------------------------------
// Chunk dot products
// ---------------------------------------------------------------------------
__device__ __forceinline__ float dot4_i8(int w, float4 a, float acc) {
    acc = fmaf((float)(int)(signed char)(w & 0xff), a.x, acc);
    acc = fmaf((float)(int)(signed char)((w >> 8) & 0xff), a.y, acc);
    acc = fmaf((float)(int)(signed char)((w >> 16) & 0xff), a.z, acc);
    acc = fmaf((float)(w >> 24), a.w, acc);
    return acc;
}
// sum over 4 bytes of a * (nibble - 8); n holds one nibble per byte (0..15)
__device__ __forceinline__ float dot4_nib(unsigned n, float4 a, float acc) {
    acc = fmaf((float)(n & 0xff) - 8.0f, a.x, acc);
    acc = fmaf((float)((n >> 8) & 0xff) - 8.0f, a.y, acc);
    acc = fmaf((float)((n >> 16) & 0xff) - 8.0f, a.z, acc);
    acc = fmaf((float)(n >> 24) - 8.0f, a.w, acc);
    return acc;
}
__device__ __forceinline__ float half_bits_to_float(unsigned short h) {
    return (float)__builtin_bit_cast(_Float16, h);
}

template <int WF> struct Fmt;
template <> struct Fmt<WF_Q8> {
    static constexpr int CH = 16;
    struct Row { const int4* w; };
    __device__ static Row row(const MvSeg& s, int r, int K) {
        return Row{reinterpret_cast<const int4*>(static_cast<const char*>(s.w) + (size_t)r * K)};
    }
    struct Chunk { int4 w; };
    __device__ static Chunk load(const Row& r, int c) { return Chunk{r.w[c]}; }
    __device__ static float dot(const Chunk& ck, const float4* a4, int nch, int c, float acc) {
        acc = dot4_i8(ck.w.x, a4[c], acc);
        acc = dot4_i8(ck.w.y, a4[nch + c], acc);
        acc = dot4_i8(ck.w.z, a4[2 * nch + c], acc);
        acc = dot4_i8(ck.w.w, a4[3 * nch + c], acc);
        return acc;
    }
};
// Q4_0: per block s = sum_i act_i*(nib_i-8), then acc += s * f32(d)
// (kernels/infer.metal:63-75); element order: low nibble of byte j = element
// j, high nibble = element j+16 (kernels/q4_simd.metal:6-19, GGML).
__device__ __forceinline__ float dot_q4_block(int4 w, float d, const float4* a4, int nch, int c, float acc) {
    float s = 0.f;
    unsigned q;
    q = (unsigned)w.x; s = dot4_nib(q & 0x0f0f0f0fu, a4[c], s);           s = dot4_nib((q >> 4) & 0x0f0f0f0fu, a4[4 * nch + c], s);
    q = (unsigned)w.y; s = dot4_nib(q & 0x0f0f0f0fu, a4[nch + c], s);     s = dot4_nib((q >> 4) & 0x0f0f0f0fu, a4[5 * nch + c], s);
    q = (unsigned)w.z; s = dot4_nib(q & 0x0f0f0f0fu, a4[2 * nch + c], s); s = dot4_nib((q >> 4) & 0x0f0f0f0fu, a4[6 * nch + c], s);
    q = (unsigned)w.w; s = dot4_nib(q & 0x0f0f0f0fu, a4[3 * nch + c], s); s = dot4_nib((q >> 4) & 0x0f0f0f0fu, a4[7 * nch + c], s);
    return fmaf(s, d, acc);
}
template <> struct Fmt<WF_Q4P> {
    static constexpr int CH = 32;
    struct Row { const int4* qs; const unsigned short* d; };
    __device__ static Row row(const MvSeg& s, int r, int K) {
        const char* base = static_cast<const char*>(s.w);
        const char* dplane = base + (size_t)s.rows * (K >> 1);
        return Row{reinterpret_cast<const int4*>(base + (size_t)r * (K >> 1)),
                   reinterpret_cast<const unsigned short*>(dplane) + (size_t)r * (K >> 5)};
    }
    struct Chunk { int4 w; unsigned short d; };
    __device__ static Chunk load(const Row& r, int c) { return Chunk{r.qs[c], r.d[c]}; }
    __device__ static float dot(const Chunk& ck, const float4* a4, int nch, int c, float acc) {
        return dot_q4_block(ck.w, half_bits_to_float(ck.d), a4, nch, c, acc);
    }
};
template <> struct Fmt<WF_Q4RAW> {
    static constexpr int CH = 32;
    struct Row { const unsigned short* b; };   // 18-byte blocks, 2-byte aligned
    __device__ static Row row(const MvSeg& s, int r, int K) {
        return Row{reinterpret_cast<const unsigned short*>(static_cast<const char*>(s.w) + (size_t)r * (K >> 5) * 18)};
    }
    struct Chunk { int4 w; unsigned short d; };
    __device__ static Chunk load(const Row& r, int c) {
        const unsigned short* b = r.b + (size_t)c * 9;
        Chunk ck;
        ck.d = b[0];
        ck.w.x = (int)((unsigned)b[1] | ((unsigned)b[2] << 16));
        ck.w.y = (int)((unsigned)b[3] | ((unsigned)b[4] << 16));
        ck.w.z = (int)((unsigned)b[5] | ((unsigned)b[6] << 16));
        ck.w.w = (int)((unsigned)b[7] | ((unsigned)b[8] << 16));
        return ck;
    }
    __device__ static float dot(const Chunk& ck, const float4* a4, int nch, int c, float acc) {
        return dot_q4_block(ck.w, half_bits_to_float(ck.d), a4, nch, c, acc);
    }
};

// ---------------------------------------------------------------------------
// The matvec.  One "group" is NR rows that share every activation read.
// KS == 1: each of the 4 waves owns a group and strides K by 64 chunks.
// KS == 4: the 4 waves share one group and stride K by 256 chunks (few rows,
//          long K: keeps every CU loading).
// ---------------------------------------------------------------------------
template <int WF, int NR, int KS>
__global__ __launch_bounds__(WG) void matvec_kernel(MvParams p, int pro, int epi) {
    using F = Fmt<WF>;
    constexpr int CH = F::CH;
    extern __shared__ float4 a4[];
    __shared__ float red[4];
    __shared__ float part[4][NR];
    __shared__ float bestV[4];
    __shared__ int bestI[4];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nch = p.K / CH;

    stage_activation<CH>(p, pro, a4, red);
    __syncthreads();

    float myBestV = -INFINITY;
    int myBestI = INT_MAX;

    const int gStart = KS == 1 ? blockIdx.x * 4 + wave : blockIdx.x;
    const int gStep = KS == 1 ? gridDim.x * 4 : gridDim.x;
    const int c0 = KS == 1 ? lane : (int)threadIdx.x;
    constexpr int cStep = KS == 1 ? 64 : 256;

    for (int g = gStart; g < p.ngroups; g += gStep) {
        // resolve the NR rows of this group
        int segOf[NR], rowOf[NR];
        bool valid[NR];
        typename F::Row rows[NR];
        if (epi == EPI_SWIGLU) {
            constexpr int H = NR / 2 > 0 ? NR / 2 : 1;
#pragma unroll
            for (int i = 0; i < NR; i++) {
                segOf[i] = i < H ? 0 : 1;
                rowOf[i] = g * H + (i < H ? i : i - H);
                valid[i] = rowOf[i] < p.seg[0].rows;
            }
        } else {
            int s = 0;
            if (p.nseg > 1 && g >= p.segGroup0[1]) s = 1;
            if (p.nseg > 2 && g >= p.segGroup0[2]) s = 2;
            int r0 = (g - p.segGroup0[s]) * NR;
#pragma unroll
            for (int i = 0; i < NR; i++) {
                segOf[i] = s;
                rowOf[i] = r0 + i;
                valid[i] = rowOf[i] < p.seg[s].rows;
            }
        }
#pragma unroll
        for (int i = 0; i < NR; i++) {
            int r = valid[i] ? rowOf[i] : 0;          // clamp: loads stay in bounds, result dropped
            rows[i] = F::row(p.seg[segOf[i]], r, p.K);
        }

        float acc[NR];
#pragma unroll
        for (int i = 0; i < NR; i++) acc[i] = 0.f;

#pragma unroll 2
        for (int c = c0; c < nch; c += cStep) {
            typename F::Chunk ck[NR];
#pragma unroll
            for (int i = 0; i < NR; i++) ck[i] = F::load(rows[i], c);
#pragma unroll
            for (int i = 0; i < NR; i++) acc[i] = F::dot(ck[i], a4, nch, c, acc[i]);
        }

#pragma unroll
        for (int i = 0; i < NR; i++) acc[i] = wave_sum(acc[i]);

        bool finisher = true;
        if (KS == 4) {
            if (lane == 0) {
#pragma unroll
                for (int i = 0; i < NR; i++) part[wave][i] = acc[i];
            }
            __syncthreads();
            finisher = wave == 0;
            if (finisher) {
#pragma unroll
                for (int i = 0; i < NR; i++) acc[i] = (part[0][i] + part[1][i]) + (part[2][i] + part[3][i]);
            }
        }

        if (finisher) {
            // lane i finishes row i
            float v = acc[0];
            int seg = segOf[0], r = rowOf[0];
            bool ok = valid[0];
#pragma unroll
            for (int i = 1; i < NR; i++) {
                if (lane == i) { v = acc[i]; seg = segOf[i]; r = rowOf[i]; ok = valid[i]; }
            }
            if (epi == EPI_SWIGLU) {
                constexpr int H = NR / 2 > 0 ? NR / 2 : 1;
                float u = acc[H < NR ? H : 0];
#pragma unroll
                for (int i = 1; i < H; i++) if (lane == i) u = acc[(H + i) < NR ? (H + i) : 0];
                if (lane < H && ok) {
                    float gs = 1.0f, us = 1.0f;
                    if (WF == WF_Q8) {
                        gs = static_cast<const float*>(p.seg[0].aux)[r];
                        us = static_cast<const float*>(p.seg[1].aux)[r];
                    }
                    float gv = v * gs, uv = u * us;
                    // mongoose.cu:949-956
                    float sig = 1.0f / (1.0f + expf(-gv));
                    p.seg[0].out[r] = gv * sig * uv;
                }
            } else if (lane < NR && ok) {
                const MvSeg& sg = p.seg[seg];
                if (WF == WF_Q8) {
                    float sc = static_cast<const float*>(sg.aux)[r];
                    if (p.div127) sc = sc / 127.0f;     // mongoose.cu:1561
                    v *= sc;
                }
                if (sg.bias) v += sg.bias[r];
                if (epi == EPI_RESID) v = p.resid[r] + v;
                sg.out[r] = v;
                if (epi == EPI_ARGMAX) {
                    if (v > myBestV || (v == myBestV && r < myBestI)) { myBestV = v; myBestI = r; }
                }
            }
        }
        if (KS == 4) __syncthreads();
    }

    if (epi == EPI_ARGMAX) {
        // lanes 0..NR-1 of each finishing wave hold candidates
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            float ov = __shfl_xor(myBestV, o, 64);
            int oi = __shfl_xor(myBestI, o, 64);
            if (ov > myBestV || (ov == myBestV && oi < myBestI)) { myBestV = ov; myBestI = oi; }
        }
        if (lane == 0) { bestV[wave] = myBestV; bestI[wave] = myBestI; }
        __syncthreads();
        if (threadIdx.x == 0) {
            float bv = bestV[0]; int bi = bestI[0];
            for (int w = 1; w < 4; w++)
                if (bestV[w] > bv || (bestV[w] == bv && bestI[w] < bi)) { bv = bestV[w]; bi = bestI[w]; }
            p.amaxVal[blockIdx.x] = bv;
            p.amaxIdx[blockIdx.x] = bi;
        }
    }
}

MvConfig pick_config(int wf, int epi, int totalRows, int K) {
    const int CH = wf == WF_Q8 ? 16 : 32;
    const int nch = K / CH;
    MvConfig c;
    c.ks = 1;
    // Long rows and few of them: split K over the workgroup.
    if (nch > 128 && totalRows <= 8192) c.ks = 4;
    if (epi == EPI_SWIGLU) {
        // totalRows counts gate rows; each group carries a gate and an up row
        c.nr = totalRows >= 8192 ? 4 : 2;
    } else if (c.ks == 4) {
        c.nr = totalRows >= 4096 ? 2 : 1;
    } else {
        c.nr = totalRows >= 16384 ? 4 : (totalRows >= 4096 ? 2 : 1);
    }
    c.grid = 0;   // filled by the launcher from the group count
    return c;
}

template <int WF, int NR, int KS>
static hipError_t launch_t(MvParams& p, int pro, int epi, int grid, hipStream_t s) {
    size_t lds = (size_t)p.K * sizeof(float);
    hipLaunchKernelGGL((matvec_kernel<WF, NR, KS>), dim3(grid), dim3(WG), lds, s, p, pro, epi);
    return hipGetLastError();
}

template <int WF>
static hipError_t launch_wf(MvParams& p, int pro, int epi, const MvConfig& c, hipStream_t s) {
    if (c.ks == 4) {
        if (c.nr == 1) return launch_t<WF, 1, 4>(p, pro, epi, c.grid, s);
        if (c.nr == 2) return launch_t<WF, 2, 4>(p, pro, epi, c.grid, s);
        return launch_t<WF, 4, 4>(p, pro, epi, c.grid, s);
    }
    if (c.nr == 1) return launch_t<WF, 1, 1>(p, pro, epi, c.grid, s);
    if (c.nr == 2) return launch_t<WF, 2, 1>(p, pro, epi, c.grid, s);
    return launch_t<WF, 4, 1>(p, pro, epi, c.grid, s);
}

hipError_t launch_matvec(int wf, int epi, int pro, MvParams& p, MvConfig* cfgInOut, hipStream_t s) {
    const int CH = wf == WF_Q8 ? 16 : 32;
    if (p.K <= 0 || p.K % CH != 0 || (size_t)p.K * 4 > 64 * 1024) return hipErrorInvalidValue;
    int total = 0;
    for (int i = 0; i < p.nseg; i++) total += p.seg[i].rows;
    MvConfig c = (cfgInOut && cfgInOut->nr > 0) ? *cfgInOut
                                                : pick_config(wf, epi, epi == EPI_SWIGLU ? p.seg[0].rows : total, p.K);
    if (epi == EPI_SWIGLU) {
        if (p.nseg != 2 || p.seg[0].rows != p.seg[1].rows) return hipErrorInvalidValue;
        if (c.nr < 2) c.nr = 2;
        int h = c.nr / 2;
        p.ngroups = (p.seg[0].rows + h - 1) / h;
        p.segGroup0[0] = 0; p.segGroup0[1] = p.ngroups; p.segGroup0[2] = p.ngroups;
    } else {
        int g = 0;
        for (int i = 0; i < 3; i++) {
            p.segGroup0[i] = g;
            if (i < p.nseg) g += (p.seg[i].rows + c.nr - 1) / c.nr;
        }
        p.ngroups = g;
    }
    if (p.ngroups == 0) return hipSuccess;
    int wgs = c.ks == 1 ? (p.ngroups + 3) / 4 : p.ngroups;
    int cap = 2048;
    if (c.grid <= 0 || c.grid > wgs) c.grid = wgs < cap ? wgs : cap;
    if (cfgInOut) *cfgInOut = c;
    if (wf == WF_Q8) return launch_wf<WF_Q8>(p, pro, epi, c, s);
    if (wf == WF_Q4P) return launch_wf<WF_Q4P>(p, pro, epi, c, s);
    return launch_wf<WF_Q4RAW>(p, pro, epi, c, s);
}

// Any K, any alignment: one wave per row, byte loads.  Only used by the
// per-op ABI when the fast kernel's preconditions (K % 16, 16-byte aligned
// rows) do not hold.
__global__ __launch_bounds__(WG) void matvec_generic_q8_kernel(const float* act, const signed char* w, const float* scales,
                                                               float* out, int N, int K, int div127) {
    int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    int lane = threadIdx.x & 63;
    if (row >= N) return;
    const signed char* wr = w + (size_t)row * K;
    float sum = 0.f;
    for (int k = lane; k < K; k += 64) sum = fmaf(act[k], (float)wr[k], sum);
    sum = wave_sum(sum);
    if (lane == 0) {
        float sc = scales[row];
        if (div127) sc = sc / 127.0f;
        out[row] = sum * sc;
    }
}
hipError_t launch_matvec_generic_q8(const float* act, const void* w, const float* scales, float* out, int N, int K,
                                    int div127, hipStream_t s) {
    if (N <= 0) return hipSuccess;
    hipLaunchKernelGGL(matvec_generic_q8_kernel, dim3((N + 3) / 4), dim3(WG), 0, s, act,
                       static_cast<const signed char*>(w), scales, out, N, K, div127);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// Decode attention (mongoose.cu:856-933), split over the KV range.
// One workgroup = one KV head (all its GQA query heads, so K/V rows are read
// once) x one split of the positions.  Online softmax over 256-position
// tiles; scores: one lane per position; P.V: one lane per float4 of the head.
// Fused form also applies RoPE (mongoose.cu:991-1006) to q and the new k and
// stores the new k/v rows (mongoose.cu:1644-1647).
// ---------------------------------------------------------------------------
template <int HD, int GMAX>
__global__ __launch_bounds__(WG) void attn_decode_kernel(AttnParams p) {
    constexpr int LPR = HD / 4;        // lanes per V row
    constexpr int TG = WG / LPR;       // position groups in the P.V phase
    constexpr int HALF = HD / 2;
    __shared__ float4 q_s4[GMAX * HD / 4];
    __shared__ float sc[GMAX][WG];
    __shared__ float red[4];
    __shared__ float4 accbuf[TG][GMAX][LPR];
    float* q_s = reinterpret_cast<float*>(q_s4);

    const int tid = threadIdx.x;
    const int G = p.nHeads / p.nKVHeads;
    const int nChunks = (G + GMAX - 1) / GMAX;
    const int kvh = blockIdx.x / nChunks;
    const int chunk = blockIdx.x % nChunks;
    const int h0 = kvh * G + chunk * GMAX;
    const int gn = min(GMAX, G - chunk * GMAX);
    const int split = blockIdx.y;

    const int pos = p.state ? p.state->pos : p.posImm;
    const int len = pos + 1;
    int splitLen, nsplit;
    if (p.direct) { splitLen = len; nsplit = 1; }
    else {
        splitLen = attn_split_len(len, p.smax, p.minSplit);
        nsplit = (len + splitLen - 1) / splitLen;
    }
    if (split >= nsplit) return;
    const int t0 = split * splitLen;
    const int t1 = min(len, t0 + splitLen);
    const int kvOff = kvh * HD;

    // q (rotated when fused) -> LDS
    for (int i = tid; i < gn * HALF; i += WG) {
        int g = i / HALF, j = i % HALF;
        float x0 = p.q[(h0 + g) * HD + j];
        float x1 = p.q[(h0 + g) * HD + HALF + j];
        if (p.fused) {
            float c = p.cosTab[(size_t)pos * HALF + j], s = p.sinTab[(size_t)pos * HALF + j];
            q_s[g * HD + j] = x0 * c - x1 * s;
            q_s[g * HD + HALF + j] = x0 * s + x1 * c;
        } else {
            q_s[g * HD + j] = x0;
            q_s[g * HD + HALF + j] = x1;
        }
    }
    // new k/v row: the split that contains `pos` stores it, then reads it back
    // like any other row (same workgroup: visible after the barrier).
    if (p.fused && t1 == len) {
        for (int j = tid; j < HALF; j += WG) {
            float c = p.cosTab[(size_t)pos * HALF + j], s = p.sinTab[(size_t)pos * HALF + j];
            float x0 = p.kNew[kvOff + j], x1 = p.kNew[kvOff + HALF + j];
            p.Kc[(size_t)pos * p.kvDim + kvOff + j] = x0 * c - x1 * s;
            p.Kc[(size_t)pos * p.kvDim + kvOff + HALF + j] = x0 * s + x1 * c;
            p.Vc[(size_t)pos * p.kvDim + kvOff + j] = p.vNew[kvOff + j];
            p.Vc[(size_t)pos * p.kvDim + kvOff + HALF + j] = p.vNew[kvOff + HALF + j];
        }
    }
    __threadfence_block();
    __syncthreads();

    const float scale = 1.0f / sqrtf((float)HD);     // mongoose.cu:867 rsqrtf(headDim)
    float m[GMAX], l[GMAX];
    float4 acc[GMAX];
#pragma unroll
    for (int g = 0; g < GMAX; g++) { m[g] = -INFINITY; l[g] = 0.f; acc[g] = make_float4(0.f, 0.f, 0.f, 0.f); }

    const int tg = tid / LPR, dl = tid % LPR;

    for (int tile = t0; tile < t1; tile += WG) {
        const int t = tile + tid;
        const bool active = t < t1;
        float s[GMAX];
#pragma unroll
        for (int g = 0; g < GMAX; g++) s[g] = 0.f;
        if (active) {
            const float4* krow = reinterpret_cast<const float4*>(p.Kc + (size_t)t * p.kvDim + kvOff);
#pragma unroll 8
            for (int d4 = 0; d4 < HD / 4; d4++) {
                float4 kv = krow[d4];
#pragma unroll
                for (int g = 0; g < GMAX; g++) {
                    if (g < gn) {
                        float4 qv = q_s4[g * (HD / 4) + d4];
                        s[g] = fmaf(qv.x, kv.x, s[g]);
                        s[g] = fmaf(qv.y, kv.y, s[g]);
                        s[g] = fmaf(qv.z, kv.z, s[g]);
                        s[g] = fmaf(qv.w, kv.w, s[g]);
                    }
                }
            }
        }
#pragma unroll
        for (int g = 0; g < GMAX; g++) {
            if (g < gn) {                                  // gn is uniform: barriers inside are safe
                float sv = active ? s[g] * scale : -INFINITY;
                float tmax = block_max(sv, red);
                float mNew = fmaxf(m[g], tmax);
                float corr = expf(m[g] - mNew);            // first tile: exp(-inf) = 0
                float pv = active ? expf(sv - mNew) : 0.f;
                sc[g][tid] = pv;
                float tsum = block_sum(pv, red);
                l[g] = l[g] * corr + tsum;
                acc[g].x *= corr; acc[g].y *= corr; acc[g].z *= corr; acc[g].w *= corr;
                m[g] = mNew;
            }
        }
        __syncthreads();
        const int tileLen = min(WG, t1 - tile);
        for (int tt = tg; tt < tileLen; tt += TG) {
            float4 v = reinterpret_cast<const float4*>(p.Vc + (size_t)(tile + tt) * p.kvDim + kvOff)[dl];
#pragma unroll
            for (int g = 0; g < GMAX; g++) {
                if (g < gn) {
                    float w = sc[g][tt];
                    acc[g].x = fmaf(w, v.x, acc[g].x);
                    acc[g].y = fmaf(w, v.y, acc[g].y);
                    acc[g].z = fmaf(w, v.z, acc[g].z);
                    acc[g].w = fmaf(w, v.w, acc[g].w);
                }
            }
        }
        __syncthreads();
    }

#pragma unroll
    for (int g = 0; g < GMAX; g++) if (g < gn) accbuf[tg][g][dl] = acc[g];
    __syncthreads();
    for (int i = tid; i < gn * LPR; i += WG) {
        int g = i / LPR, d4 = i % LPR;
        float4 r = accbuf[0][g][d4];
        for (int k = 1; k < TG; k++) {
            float4 a = accbuf[k][g][d4];
            r.x += a.x; r.y += a.y; r.z += a.z; r.w += a.w;
        }
        // m[], l[] are replicated in every thread; pick g's with a select chain
        float lg = l[0], mg_ = m[0];
#pragma unroll
        for (int k = 1; k < GMAX; k++) if (g == k) { lg = l[k]; mg_ = m[k]; }
        int h = h0 + g;
        if (p.direct) {
            float4 o;
            o.x = r.x / lg; o.y = r.y / lg; o.z = r.z / lg; o.w = r.w / lg;
            reinterpret_cast<float4*>(p.out + (size_t)h * HD)[d4] = o;
        } else {
            reinterpret_cast<float4*>(p.pacc + ((size_t)h * p.smax + split) * HD)[d4] = r;
            if (d4 == 0) {
                p.pm[(size_t)h * p.smax + split] = mg_;
                p.pl[(size_t)h * p.smax + split] = lg;
            }
        }
    }
}

template <int HD>
static hipError_t launch_attn_hd(const AttnParams& p, int maxSplits, hipStream_t s) {
    int G = p.nHeads / p.nKVHeads;
    int gmax = G >= 8 ? 8 : (G > 2 ? (G > 4 ? 8 : 4) : (G == 2 ? 2 : 1));
    int nChunks = (G + gmax - 1) / gmax;
    dim3 grid(p.nKVHeads * nChunks, maxSplits);
    switch (gmax) {
    case 1: hipLaunchKernelGGL((attn_decode_kernel<HD, 1>), grid, dim3(WG), 0, s, p); break;
    case 2: hipLaunchKernelGGL((attn_decode_kernel<HD, 2>), grid, dim3(WG), 0, s, p); break;
    case 4: hipLaunchKernelGGL((attn_decode_kernel<HD, 4>), grid, dim3(WG), 0, s, p); break;
    default: hipLaunchKernelGGL((attn_decode_kernel<HD, 8>), grid, dim3(WG), 0, s, p); break;
    }
    return hipGetLastError();
}

hipError_t launch_attention(const AttnParams& p, hipStream_t s) {
    if (p.nKVHeads <= 0 || p.nHeads % p.nKVHeads != 0) return hipErrorInvalidValue;
    int splits = p.direct ? 1 : p.smax;
    if (p.headDim == 64) return launch_attn_hd<64>(p, splits, s);
    if (p.headDim == 128) return launch_attn_hd<128>(p, splits, s);
    return hipErrorInvalidValue;
}

// ---------------------------------------------------------------------------
// Small per-op kernels (the reference's one-launch-per-op path)
// ---------------------------------------------------------------------------
// mongoose.cu:145-174
__global__ __launch_bounds__(WG) void rmsnorm_out_kernel(const float* in, float* out, const float* w, int dim, float eps) {
    __shared__ float red[4];
    const float* x = in + (size_t)blockIdx.x * dim;
    float* o = out + (size_t)blockIdx.x * dim;
    float ss = 0.f;
    for (int i = threadIdx.x; i < dim; i += WG) ss += x[i] * x[i];
    float tot = block_sum(ss, red);
    float rs = 1.0f / sqrtf(tot / (float)dim + eps);
    for (int i = threadIdx.x; i < dim; i += WG) o[i] = x[i] * rs * w[i];
}
hipError_t launch_rmsnorm_out(const float* in, float* out, const float* w, int seqLen, int dim, float eps, hipStream_t s) {
    if (seqLen <= 0) return hipSuccess;
    hipLaunchKernelGGL(rmsnorm_out_kernel, dim3(seqLen), dim3(WG), 0, s, in, out, w, dim, eps);
    return hipGetLastError();
}

// mongoose.cu:991-1006
__global__ void rope_kernel(float* x, const float* cosTab, const float* sinTab, int dim, int headDim, int nHeads) {
    int pos = blockIdx.x;
    int half = headDim / 2;
    for (int i = threadIdx.x; i < nHeads * half; i += blockDim.x) {
        int h = i / half, j = i % half;
        size_t base = (size_t)pos * dim + (size_t)h * headDim;
        float c = cosTab[(size_t)pos * half + j], s = sinTab[(size_t)pos * half + j];
        float x0 = x[base + j], x1 = x[base + half + j];
        x[base + j] = x0 * c - x1 * s;
        x[base + half + j] = x0 * s + x1 * c;
    }
}
hipError_t launch_rope(float* x, const float* cosTab, const float* sinTab, int seqLen, int dim, int headDim, int nHeads, hipStream_t s) {
    if (seqLen <= 0) return hipSuccess;
    hipLaunchKernelGGL(rope_kernel, dim3(seqLen), dim3(WG), 0, s, x, cosTab, sinTab, dim, headDim, nHeads);
    return hipGetLastError();
}

// mongoose.cu:1644-1647
__global__ void kv_cache_write_kernel(float* cache, const float* src, int pos, int kvDim) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < kvDim) cache[(size_t)pos * kvDim + i] = src[i];
}
hipError_t launch_kv_cache_write(float* cache, const float* src, int pos, int kvDim, hipStream_t s) {
    hipLaunchKernelGGL(kv_cache_write_kernel, dim3((kvDim + WG - 1) / WG), dim3(WG), 0, s, cache, src, pos, kvDim);
    return hipGetLastError();
}

// mongoose.cu:949-956
__global__ void silu_gate_mul_kernel(const float* gate, const float* up, float* out, int n) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        float g = gate[i];
        float sig = 1.0f / (1.0f + expf(-g));
        out[i] = g * sig * up[i];
    }
}
hipError_t launch_silu_gate_mul(const float* gate, const float* up, float* out, int n, hipStream_t s) {
    if (n <= 0) return hipSuccess;
    hipLaunchKernelGGL(silu_gate_mul_kernel, dim3((n + WG - 1) / WG), dim3(WG), 0, s, gate, up, out, n);
    return hipGetLastError();
}

// mongoose.cu:212-219
__global__ void add_inplace_kernel(float* a, const float* b, int n) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) a[i] += b[i];
}
hipError_t launch_add_inplace(float* a, const float* b, int n, hipStream_t s) {
    if (n <= 0) return hipSuccess;
    hipLaunchKernelGGL(add_inplace_kernel, dim3((n + WG - 1) / WG), dim3(WG), 0, s, a, b, n);
    return hipGetLastError();
}

// mongoose.cu:1052-1064
__global__ void embed_gather_f32_kernel(float* out, const float* embed, const int* tokens, int dim) {
    int p = blockIdx.x;
    int tok = tokens[p];
    for (int i = threadIdx.x; i < dim; i += blockDim.x) out[(size_t)p * dim + i] = embed[(size_t)tok * dim + i];
}
hipError_t launch_embed_gather_f32(float* out, const float* embed, const int* tokens, int seqLen, int dim, hipStream_t s) {
    if (seqLen <= 0) return hipSuccess;
    hipLaunchKernelGGL(embed_gather_f32_kernel, dim3(seqLen), dim3(WG), 0, s, out, embed, tokens, dim);
    return hipGetLastError();
}

// mongoose.cu:1475-1487 (div127) and the per-row-scale form q*s
__global__ void dequant_q8_kernel(const signed char* w, const float* scales, float* out, int cols, int div127) {
    int row = blockIdx.x;
    float s = scales[row];
    if (div127) s = s / 127.0f;
    for (int j = threadIdx.x; j < cols; j += blockDim.x)
        out[(size_t)row * cols + j] = (float)w[(size_t)row * cols + j] * s;
}
hipError_t launch_dequant_q8(const void* w, const float* scales, float* out, int rows, int cols, int div127, hipStream_t s) {
    if (rows <= 0) return hipSuccess;
    hipLaunchKernelGGL(dequant_q8_kernel, dim3(rows), dim3(WG), 0, s, static_cast<const signed char*>(w), scales, out, cols, div127);
    return hipGetLastError();
}

// GGML dequantize_row_q4_0 on raw 18-byte blocks
__global__ void dequant_q4_0_kernel(const unsigned char* w, float* out, size_t nblocks) {
    size_t b = (size_t)blockIdx.x * (blockDim.x / 16) + threadIdx.x / 16;
    int j = threadIdx.x % 16;
    if (b >= nblocks) return;
    const unsigned char* y = w + b * 18;
    unsigned short hb = (unsigned short)(y[0] | (y[1] << 8));
    float d = half_bits_to_float(hb);
    unsigned char q = y[2 + j];
    out[b * 32 + j] = (float)((int)(q & 0x0f) - 8) * d;
    out[b * 32 + 16 + j] = (float)((int)(q >> 4) - 8) * d;
}
hipError_t launch_dequant_q4_0(const void* w, float* out, int rows, int cols, hipStream_t s) {
    size_t nb = (size_t)rows * (cols / 32);
    if (nb == 0) return hipSuccess;
    size_t grid = (nb + 15) / 16;
    hipLaunchKernelGGL(dequant_q4_0_kernel, dim3((unsigned)grid), dim3(WG), 0, s, static_cast<const unsigned char*>(w), out, nb);
    return hipGetLastError();
}

// raw GGUF rows -> nibbles plane then fp16 d plane
__global__ void q4_0_repack_kernel(const unsigned short* raw, unsigned short* planar, size_t nblocks) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;    // one thread per 2 bytes of nibbles
    size_t b = i / 8;
    int j = (int)(i % 8);
    if (b >= nblocks) return;
    planar[b * 8 + j] = raw[b * 9 + 1 + j];
    if (j == 0) planar[nblocks * 8 + b] = raw[b * 9];
}
hipError_t launch_q4_0_repack(const void* raw, void* planar, int N, int K, hipStream_t s) {
    size_t nb = (size_t)N * (K / 32);
    if (nb == 0) return hipSuccess;
    size_t threads = nb * 8;
    hipLaunchKernelGGL(q4_0_repack_kernel, dim3((unsigned)((threads + WG - 1) / WG)), dim3(WG), 0, s,
                       static_cast<const unsigned short*>(raw), static_cast<unsigned short*>(planar), nb);
    return hipGetLastError();
}

__global__ void fill_zero_kernel(unsigned* p, size_t nwords, unsigned char* tail, int ntail) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < nwords; i += stride) p[i] = 0u;
    if (blockIdx.x == 0 && (int)threadIdx.x < ntail) tail[threadIdx.x] = 0;
}
hipError_t launch_fill_zero(void* ptr, size_t bytes, hipStream_t s) {
    if (bytes == 0) return hipSuccess;
    if (((uintptr_t)ptr & 3) != 0) return hipMemsetAsync(ptr, 0, bytes, s);
    size_t nwords = bytes / 4;
    int ntail = (int)(bytes % 4);
    size_t blocks = (nwords + WG - 1) / WG;
    if (blocks > 4096) blocks = 4096;
    if (blocks == 0) blocks = 1;
    hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)blocks), dim3(WG), 0, s, static_cast<unsigned*>(ptr), nwords,
                       static_cast<unsigned char*>(ptr) + nwords * 4, ntail);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// Token-level stages that the reference leaves to its caller
// ---------------------------------------------------------------------------
__global__ void embed_token_kernel(int kind, const void* table, const float* scales, const StepState* state,
                                   float* x, int dim, int vocab) {
    int tok = state->token;
    if (tok < 0) tok = 0;
    if (tok >= vocab) tok = vocab - 1;
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= dim) return;
    if (kind == 0) {
        const signed char* q = static_cast<const signed char*>(table) + (size_t)tok * dim;
        x[i] = (float)q[i] * scales[tok];
    } else if (kind == 1) {
        const unsigned short* t = static_cast<const unsigned short*>(table) + (size_t)tok * dim;
        x[i] = half_bits_to_float(t[i]);
    } else if (kind == 2) {
        x[i] = static_cast<const float*>(table)[(size_t)tok * dim + i];
    } else {
        const unsigned char* base = static_cast<const unsigned char*>(table);
        const unsigned char* qs = base + (size_t)tok * (dim >> 1);
        const unsigned short* dpl = reinterpret_cast<const unsigned short*>(base + (size_t)vocab * (dim >> 1)) + (size_t)tok * (dim >> 5);
        int b = i >> 5, j = i & 31;
        unsigned char q = qs[b * 16 + (j & 15)];
        int nib = j < 16 ? (q & 0x0f) : (q >> 4);
        x[i] = (float)(nib - 8) * half_bits_to_float(dpl[b]);
    }
}
hipError_t launch_embed_token(int kind, const void* table, const float* scales, const StepState* state, float* x,
                              int dim, int vocab, hipStream_t s) {
    hipLaunchKernelGGL(embed_token_kernel, dim3((dim + WG - 1) / WG), dim3(WG), 0, s, kind, table, scales, state, x, dim, vocab);
    return hipGetLastError();
}

__global__ __launch_bounds__(WG) void argmax_finish_kernel(const float* pv, const int* pi, int nparts, StepState* state,
                                                           const int* prompt, int* history, int historyCap, int vocab) {
    __shared__ float bv[WG];
    __shared__ int bi[WG];
    float v = -INFINITY;
    int idx = INT_MAX;
    for (int i = threadIdx.x; i < nparts; i += WG) {
        float ov = pv[i]; int oi = pi[i];
        if (ov > v || (ov == v && oi < idx)) { v = ov; idx = oi; }
    }
    bv[threadIdx.x] = v; bi[threadIdx.x] = idx;
    __syncthreads();
    for (int o = WG / 2; o > 0; o >>= 1) {
        if ((int)threadIdx.x < o) {
            float ov = bv[threadIdx.x + o]; int oi = bi[threadIdx.x + o];
            if (ov > bv[threadIdx.x] || (ov == bv[threadIdx.x] && oi < bi[threadIdx.x])) { bv[threadIdx.x] = ov; bi[threadIdx.x] = oi; }
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        int tok = bi[0];
        if (tok < 0 || tok >= vocab) tok = 0;
        int np = state->pos + 1;
        int next = tok;
        if (prompt && np < state->nPrompt) next = prompt[np];
        int cnt = state->count;
        if (history && cnt < historyCap) history[cnt] = tok;
        state->count = cnt + 1;
        state->token = next;
        state->pos = np;
    }
}
hipError_t launch_argmax_finish(const float* pv, const int* pi, int nparts, StepState* state, const int* prompt,
                                int* history, int historyCap, int vocab, hipStream_t s) {
    hipLaunchKernelGGL(argmax_finish_kernel, dim3(1), dim3(WG), 0, s, pv, pi, nparts, state, prompt, history, historyCap, vocab);
    return hipGetLastError();
}

__global__ void set_state_kernel(StepState* state, int pos, int token, int count, int nPrompt) {
    state->pos = pos; state->token = token; state->count = count; state->nPrompt = nPrompt;
}
hipError_t launch_set_state(StepState* state, int pos, int token, int count, int nPrompt, hipStream_t s) {
    hipLaunchKernelGGL(set_state_kernel, dim3(1), dim3(1), 0, s, state, pos, token, count, nPrompt);
    return hipGetLastError();
}

__global__ void advance_prompt_kernel(StepState* state, const int* prompt) {
    int np = state->pos + 1;
    state->pos = np;
    if (np < state->nPrompt) state->token = prompt[np];
}
hipError_t launch_advance_prompt(StepState* state, const int* prompt, hipStream_t s) {
    hipLaunchKernelGGL(advance_prompt_kernel, dim3(1), dim3(1), 0, s, state, prompt);
    return hipGetLastError();
}

}  // namespace mg
