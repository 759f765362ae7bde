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
#include "device_util.h"

namespace mg {

// ---------------------------------------------------------------------------
// Activation vector in LDS.  A lane owns a weight chunk of 16 weights: 16
// consecutive int8 (Q8), or half a Q4_0 block = 8 bytes whose low nibbles are
// elements 8h..8h+7 of the block and whose high nibbles are elements
// 16+8h..16+8h+7.  Stored linearly, neighbouring lanes would read float4s 64
// bytes apart and collide on LDS banks, so the vector is stored as 4 planes:
// plane p holds, for every chunk c, one float4 of the chunk's activations at
// float4 index p*nch + c.  Lane reads are then 16 bytes apart: conflict free.
// ---------------------------------------------------------------------------
template <int WF>
__device__ __forceinline__ int act_slot4(int k4, int nch) {   // k4 = k/4 -> float4 index
    if (WF == WF_Q8) {
        return (k4 & 3) * nch + (k4 >> 2);
    } else {
        // k4 = 8*block + r4; r4: 0,1 lo-half0  2,3 lo-half1  4,5 hi-half0  6,7 hi-half1
        int blk = k4 >> 3, r4 = k4 & 7;
        int hi = r4 >> 2, h = (r4 >> 1) & 1, q = r4 & 1;
        return (hi * 2 + q) * nch + blk * 2 + h;
    }
}

// All global loads of a prologue are issued before anything waits on them; the
// caller has already issued its first weight loads, so the activation latency
// and the weight latency overlap instead of adding up.
// SHORT: the caller knows K <= 4 * WG (one float4 a thread at most): no loops, no long-vector path.
template <int WF, int PRO, bool SHORT = false>
__device__ __forceinline__ float stage_activation(const MvParams& p, float4* a4, float* red) {
    const int K4 = p.K >> 2;
    const int nch = p.K / 16;
    const int tid = threadIdx.x;
    if (PRO == PRO_PLAIN) {
        const float4* x4 = reinterpret_cast<const float4*>(p.act);
        if (SHORT) {
            if (tid < K4) a4[act_slot4<WF>(tid, nch)] = x4[tid];
        } else if (K4 <= 4 * WG) {
            for (int i = tid; i < K4; i += WG) a4[act_slot4<WF>(i, nch)] = x4[i];
        } else {
            // Long vectors (down projection, K = 14336): every load of a batch is issued before the
            // first LDS store, so a batch costs one memory round trip; a load-store loop pays one per
            // few iterations.
            constexpr int B = 16;
            for (int base = 0; base < K4; base += B * WG) {
                float4 v[B];
#pragma unroll
                for (int u = 0; u < B; u++) {
                    v[u] = make_float4(0.f, 0.f, 0.f, 0.f);
                    if (base + u * WG < K4) v[u] = x4[min(base + u * WG + tid, K4 - 1)];   // uniform test
                }
#pragma unroll
                for (int u = 0; u < B; u++) {
                    const int i = base + u * WG + tid;
                    if (i < K4) a4[act_slot4<WF>(i, nch)] = v[u];
                }
            }
        }
        __syncthreads();
        return 1.0f;
    }
    // RMSNorm (mongoose.cu:145-174 / cpu.go:36-47): x * (1/sqrt(mean(x^2)+eps)) * g.  The vector
    // staged is x*g; the common factor 1/rms is returned and applied to each finished row, so
    // nothing waits for the sum of squares before the weights can be consumed: one barrier
    // covers both the staged vector and the partial sums.
    const float4* x4 = reinterpret_cast<const float4*>(p.act);
    const float4* g4 = reinterpret_cast<const float4*>(p.gain);
    float ss = 0.f;
    for (int i = tid; i < (SHORT ? min(K4, WG) : K4); i += WG) {      // SHORT: at most one pass
        float4 v = x4[i], g = g4[i], o;
        ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
        o.x = v.x * g.x; o.y = v.y * g.y; o.z = v.z * g.z; o.w = v.w * g.w;
        a4[act_slot4<WF>(i, nch)] = o;
    }
    ss = wave_sum(ss);
    if ((tid & 63) == 0) red[tid >> 6] = ss;
    __syncthreads();
    float tot = (red[0] + red[1]) + (red[2] + red[3]);
    return __builtin_amdgcn_rsqf(tot * __builtin_amdgcn_rcpf((float)p.K) + p.eps);   // 1 ulp each; the reference's rsqrtf (mongoose.cu:170) is no closer
}

// av[0..3]: the chunk's activations (4 float4), asum: their sum (Q4 only).
template <int WF> struct Fmt;
template <> struct Fmt<WF_Q8> {
    struct Row { const int4* w; };
    __device__ static Row row(const MvSeg& s, int r, int K) {
        return Row{reinterpret_cast<const int4*>(static_cast<const char*>(s.w) + (size_t)r * K)};
    }
    struct Chunk { int4 w; };
    __device__ static Chunk load(const Row& r, int c) { return Chunk{r.w[c]}; }
    __device__ static float dot(const Chunk& ck, const float4 (&av)[4], float, float acc) {
        acc = dot4_i8(ck.w.x, av[0], acc);
        acc = dot4_i8(ck.w.y, av[1], acc);
        acc = dot4_i8(ck.w.z, av[2], acc);
        acc = dot4_i8(ck.w.w, av[3], acc);
        return acc;
    }
};
template <> struct Fmt<WF_Q4P> {
    struct Row { const int2* qs; const unsigned short* d; };
    __device__ static Row row(const MvSeg& s, int r, int K) {
        const char* base = static_cast<const char*>(s.w);
        const char* dplane = base + (size_t)s.rows * (K >> 1);
        return Row{reinterpret_cast<const int2*>(base + (size_t)r * (K >> 1)),
                   reinterpret_cast<const unsigned short*>(dplane) + (size_t)r * (K >> 5)};
    }
    struct Chunk { int2 w; unsigned short d; };
    __device__ static Chunk load(const Row& r, int c) { return Chunk{r.qs[c], r.d[c >> 1]}; }
    __device__ static float dot(const Chunk& ck, const float4 (&av)[4], float asum, float acc) {
        return dot_q4_half(ck.w, half_bits_to_float(ck.d), av, asum, acc);
    }
};
template <> struct Fmt<WF_Q4RAW> {
    struct Row { const unsigned short* b; };   // 18-byte blocks, 2-byte aligned
    __device__ static Row row(const MvSeg& s, int r, int K) {
        return Row{reinterpret_cast<const unsigned short*>(static_cast<const char*>(s.w) + (size_t)r * (K >> 5) * 18)};
    }
    struct Chunk { int2 w; unsigned short d; };
    __device__ static Chunk load(const Row& r, int c) {
        const unsigned short* b = r.b + (size_t)(c >> 1) * 9;
        const unsigned short* h = b + 1 + (c & 1) * 4;
        Chunk ck;
        ck.d = b[0];
        ck.w.x = (int)((unsigned)h[0] | ((unsigned)h[1] << 16));
        ck.w.y = (int)((unsigned)h[2] | ((unsigned)h[3] << 16));
        return ck;
    }
    __device__ static float dot(const Chunk& ck, const float4 (&av)[4], float asum, float acc) {
        return dot_q4_half(ck.w, half_bits_to_float(ck.d), av, asum, acc);
    }
};

// ---------------------------------------------------------------------------
// The matvec.  A "group" is NR rows that share every activation read; KS == 1:
// each of the 4 waves owns a group (64 lanes stride K), KS == 4: the 4 waves
// share one group (256 lanes stride K; few rows, long K).
//
// Work of a wave is a stream of items (group, chunk iteration).  Items are
// loaded D ahead of the one being consumed (register ring), the first D of
// them before the activation vector is even staged, so the kernel's critical
// path is one memory latency, not prologue + weights + scales in sequence.
// Per-row epilogue operands (scale, bias, residual, RoPE factors) ride in the
// same ring.
// ---------------------------------------------------------------------------
struct RowRef { int seg; int row; bool valid; };

// Every workgroup of the launch fills its share of [x, x + words) with 0xFFFFFFFF (16 bytes a store).
__device__ __forceinline__ void fill_unset(unsigned* x, unsigned words) {
    if (!x) return;
    const unsigned n4 = words >> 2;
    const uint4 v = make_uint4(0xFFFFFFFFu, 0xFFFFFFFFu, 0xFFFFFFFFu, 0xFFFFFFFFu);
    for (unsigned i = blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += gridDim.x * blockDim.x) reinterpret_cast<uint4*>(x)[i] = v;
}

template <int NR, int EPI>
__device__ __forceinline__ RowRef resolve_row(const MvParams& p, int g, int i) {
    RowRef r;
    if (EPI == EPI_SWIGLU) {
        constexpr int H = NR / 2 > 0 ? NR / 2 : 1;
        r.seg = i < H ? 0 : 1;
        r.row = g * H + (i < H ? i : i - H);
        r.valid = r.row < p.seg[0].rows;
    } else if (EPI == EPI_QKV) {
        // pairs (j, j + headDim/2) of one head for q and k, consecutive rows for v
        int s = 0;
        if (g >= p.segGroup0[1]) s = 1;
        if (g >= p.segGroup0[2]) s = 2;
        int gi = g - p.segGroup0[s];
        r.seg = s;
        if (s < 2) {
            // headDim is a power of two (checked by the launcher): gi = head * half + j
            const int half = p.headDim >> 1;
            const int j = gi & (half - 1);
            r.row = ((gi - j) << 1) + j + (i ? half : 0);
        } else {
            r.row = gi * 2 + i;
        }
        r.valid = r.row < p.seg[s].rows;
    } else {
        int s = 0;
        if (p.nseg > 1 && g >= p.segGroup0[1]) s = 1;
        if (p.nseg > 2 && g >= p.segGroup0[2]) s = 2;
        r.seg = s;
        r.row = (g - p.segGroup0[s]) * NR + i;
        r.valid = r.row < p.seg[s].rows;
    }
    return r;
}

template <int WF, int NR, int KS, int PRO, int EPI, bool EARLY = false, bool ONCE = false>
__global__ __launch_bounds__(WG) void matvec_kernel(MvParams p) {
    using F = Fmt<WF>;
    constexpr int LPG = KS == 1 ? 64 : WG;           // lanes per group
    // items in flight per wave; ONCE: the launcher knows that no wave has more than one item (short
    // rows, one round of workgroups), and the ring with its unrolled slots shrinks to one: a quarter of
    // the code for a launch that runs every instruction once
    constexpr int D = (ONCE && KS == 1) ? (EARLY ? 2 : 1) : (NR >= 4 ? 2 : 4);      // with EARLY (K of 1025..2048): two chunk passes
    extern __shared__ float4 a4[];
    __shared__ float red[4];
    __shared__ float part[4][NR];
    __shared__ float bestV[4];
    __shared__ int bestI[4];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lig = KS == 1 ? lane : (int)threadIdx.x;       // lane within the group
    const int nch = p.K / 16;
    const int iters = (nch + LPG - 1) / LPG;
    const int gStart = KS == 1 ? blockIdx.x * 4 + wave : blockIdx.x;
    const int gStep = KS == 1 ? gridDim.x * 4 : gridDim.x;
    const int myGroups = gStart >= p.ngroups ? 0 : ((ONCE && KS == 1) ? 1 : (p.ngroups - gStart + gStep - 1) / gStep);
    const int nItems = myGroups * iters;

    if (EPI == EPI_ARGMAX) fill_unset(p.xreset, p.xresetWords);

    int pos = 0;
    if (EPI == EPI_QKV) {
        // not `state ? state->pos : posImm`: that selects between a global address and the kernel-argument
        // address, i.e. a flat load, and the kernel's first scalar/LDS wait then sits behind it.  A vector
        // load issued ahead of the weights instead: it is back before they are, and nothing waits for it alone.
        pos = p.posImm;
        if (p.state) pos = __hip_atomic_load(&p.state->pos, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }

    typename F::Chunk ring[D][NR];
    float rSc[D], rBi[D], rRe[D], rCs[D], rSn[D];            // epilogue operands of the lane's row

    // (group, chunk iteration) of the next item to issue and of the next item to consume:
    // advanced step by step, no division in the loop
    int gI = gStart, itI = 0, gC = gStart, itC = 0;
    auto issue = [&](int slot, int item) {
        if (item >= nItems) return;
        const int g = gI;
        const int it = itI;
        if (++itI == iters) { itI = 0; gI += gStep; }
        const int c = lig + it * LPG;
#pragma unroll
        for (int i = 0; i < NR; i++) {
            RowRef rr = resolve_row<NR, EPI>(p, g, i);
            if (c < nch) ring[slot][i] = F::load(F::row(p.seg[rr.seg], rr.valid ? rr.row : 0, p.K), c);
        }
        if (it == 0) {
            rSc[slot] = 1.0f; rBi[slot] = 0.f; rRe[slot] = 0.f; rCs[slot] = 1.0f; rSn[slot] = 0.f;
            if (lane < NR) {
                RowRef rr = resolve_row<NR, EPI>(p, g, lane < NR ? lane : 0);
                if (rr.valid) {
                    const MvSeg& sg = p.seg[rr.seg];
                    if (WF == WF_Q8) rSc[slot] = static_cast<const float*>(sg.aux)[rr.row];
                    if (sg.bias) rBi[slot] = sg.bias[rr.row];
                    if (EPI == EPI_RESID) rRe[slot] = p.resid[rr.row];
                    if (EPI == EPI_QKV && rr.seg < 2 && lane == 0) {
                        const int j = (g - p.segGroup0[rr.seg]) & ((p.headDim >> 1) - 1);
                        rCs[slot] = p.cosRow[j];
                        rSn[slot] = p.sinRow[j];
                    }
                }
            }
        }
    };

    // Vectors of 1025..4096 elements (two to four float4 per thread): all of a thread's pieces of the
    // vector (and of the norm gain) are requested in one batch, ahead of the first weights, and held in
    // registers -- one memory round trip; the load-then-store loop of stage_activation pays one per
    // piece.  (A single piece gains nothing from this and costs registers: measured slower at K = 896.)
    constexpr int SB = 4;                             // float4 per thread held across the weight issue
    const int K4 = p.K >> 2;
    constexpr bool early = EARLY;                     // chosen by the launcher: KS == 1 and WG < K/4 <= SB*WG
    float4 sx[SB], sgn[SB];
    if (early) {
        const float4* x4 = reinterpret_cast<const float4*>(p.act);
        const float4* g4 = reinterpret_cast<const float4*>(p.gain);
#pragma unroll
        for (int u = 0; u < SB; u++) {
            sx[u] = make_float4(0.f, 0.f, 0.f, 0.f);
            sgn[u] = sx[u];
            if (u * WG < K4) {                                        // uniform: whole rounds past the end issue nothing
                const int i = min((int)threadIdx.x + u * WG, K4 - 1);
                sx[u] = x4[i];
                if (PRO == PRO_RMS) sgn[u] = g4[i];
            }
        }
    }

    // first weight loads go out before the activation vector is staged
#pragma unroll
    for (int s = 0; s < D; s++) issue(s, s);

    // K split over the workgroup and at most two chunk rounds: a thread only ever meets its own one or
    // two chunks of the vector, so it reads them straight into registers -- no LDS copy, no barrier,
    // and no more bytes than staging reads.  (With KS == 1 every wave would read the whole vector
    // itself, four times the requests: measured slower.)
    constexpr bool CAN_DIRECT = KS == 4 && PRO == PRO_PLAIN;
    const bool direct = CAN_DIRECT && (ONCE || iters <= 2);      // ONCE with KS == 4: the launcher has checked iters <= 2
    float4 avr[2][4];
    float rs = 1.0f;
    if (direct) {
        const float4* x4 = reinterpret_cast<const float4*>(p.act);
#pragma unroll
        for (int it = 0; it < 2; it++) {
            const int c = min(lig + it * LPG, nch - 1);
            if (WF == WF_Q8) {
#pragma unroll
                for (int pl = 0; pl < 4; pl++) avr[it][pl] = x4[c * 4 + pl];
            } else {
                // half block h of block blk: planes 0,1 meet its low nibbles (elements 8h..8h+7),
                // planes 2,3 its high nibbles (16+8h..16+8h+7), as act_slot4 lays them out
                const int base = (c >> 1) * 8 + (c & 1) * 2;
                avr[it][0] = x4[base]; avr[it][1] = x4[base + 1];
                avr[it][2] = x4[base + 4]; avr[it][3] = x4[base + 5];
            }
        }
    } else if (early) {
        // stage_activation's arithmetic on the registers loaded above
        float ss = 0.f;
#pragma unroll
        for (int u = 0; u < SB; u++) {
            const int i = threadIdx.x + u * WG;
            if (i < K4) {
                float4 v = sx[u];
                if (PRO == PRO_RMS) {
                    ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
                    v.x *= sgn[u].x; v.y *= sgn[u].y; v.z *= sgn[u].z; v.w *= sgn[u].w;
                }
                a4[act_slot4<WF>(i, nch)] = v;
            }
        }
        if (PRO == PRO_RMS) {
            ss = wave_sum(ss);
            if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
        }
        __syncthreads();
        if (PRO == PRO_RMS) rs = 1.0f / sqrtf(((red[0] + red[1]) + (red[2] + red[3])) / (float)p.K + p.eps);
    } else {
        rs = stage_activation<WF, PRO, ONCE && KS == 1 && !EARLY>(p, a4, red);     // one-item launches have K <= 1024
    }

    float myBestV = -INFINITY;
    int myBestI = INT_MAX;
    float acc[NR];
#pragma unroll
    for (int i = 0; i < NR; i++) acc[i] = 0.f;
    float sc = 1.0f, bi = 0.f, re = 0.f, cs = 1.0f, sn = 0.f;

    for (int base = 0; base < nItems; base += D) {
#pragma unroll
        for (int s = 0; s < D; s++) {
            const int item = base + s;
            if (item < nItems) {
                const int g = gC;
                const int it = itC;
                if (++itC == iters) { itC = 0; gC += gStep; }
                const int c = lig + it * LPG;
                if (c < nch) {
                    float4 av[4];
                    if (CAN_DIRECT && direct) {
#pragma unroll
                        for (int pl = 0; pl < 4; pl++) av[pl] = it == 0 ? avr[0][pl] : avr[1][pl];
                    } else {
#pragma unroll
                        for (int pl = 0; pl < 4; pl++) av[pl] = a4[pl * nch + c];
                    }
                    float asum = 0.f;
                    if (WF != WF_Q8) {
                        float4 t;
                        t.x = (av[0].x + av[1].x) + (av[2].x + av[3].x);
                        t.y = (av[0].y + av[1].y) + (av[2].y + av[3].y);
                        t.z = (av[0].z + av[1].z) + (av[2].z + av[3].z);
                        t.w = (av[0].w + av[1].w) + (av[2].w + av[3].w);
                        asum = (t.x + t.y) + (t.z + t.w);
                    }
#pragma unroll
                    for (int i = 0; i < NR; i++) acc[i] = F::dot(ring[s][i], av, asum, acc[i]);
                }
                // operands arrive with the group's first item and are held until its last
                if (it == 0) { sc = rSc[s]; bi = rBi[s]; re = rRe[s]; cs = rCs[s]; sn = rSn[s]; }
                if (it == iters - 1) {
                    // ---- group finished: reduce and write ----
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
                        float v = acc[0];
#pragma unroll
                        for (int i = 1; i < NR; i++) if (lane == i) v = acc[i];
                        if (WF == WF_Q8) {
                            if (p.div127) sc = sc / 127.0f;      // mongoose.cu:1561
                            v *= sc;
                        }
                        if (PRO == PRO_RMS) v *= rs;
                        v += bi;
                        RowRef rr = resolve_row<NR, EPI>(p, g, lane < NR ? lane : 0);
                        if (EPI == EPI_SWIGLU) {
                            constexpr int H = NR / 2 > 0 ? NR / 2 : 1;
                            const float u = dpp_f<0x100 + H>(v);               // row_shl:H -- lane l reads lane l + H (the up row)
                            if (lane < H && rr.valid) {
                                float sig = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-v * 1.4426950408889634f));   // mongoose.cu:949-956
                                p.seg[0].out[rr.row] = v * sig * u;
                            }
                        } else if (EPI == EPI_QKV) {
                            const float v1 = dpp_f<0x101>(v);                  // row_shl:1 -- lane 0 reads lane 1 (the pair's second row)
                            if (lane == 0 && rr.valid) {
                                const MvSeg& sg = p.seg[rr.seg];
                                float o0, o1;
                                int i1;
                                if (rr.seg < 2) {                               // mongoose.cu:991-1006
                                    o0 = v * cs - v1 * sn;
                                    o1 = v * sn + v1 * cs;
                                    i1 = rr.row + (p.headDim >> 1);
                                } else {                                        // mongoose.cu:1644-1647
                                    o0 = v; o1 = v1;
                                    i1 = rr.row + 1 < sg.rows ? rr.row + 1 : rr.row;
                                }
                                if (rr.seg > 0 && p.kvHalf) {                   // fp16 cache rows
                                    _Float16* dst = reinterpret_cast<_Float16*>(sg.out) + (size_t)pos * p.kvDim;
                                    dst[i1] = (_Float16)o1;
                                    dst[rr.row] = (_Float16)o0;
                                } else {
                                    float* dst = rr.seg == 0 ? sg.out : sg.out + (size_t)pos * p.kvDim;
                                    dst[i1] = o1;
                                    dst[rr.row] = o0;
                                }
                            }
                        } else if (lane < NR && rr.valid) {
                            if (EPI == EPI_RESID) v = re + v;
                            p.seg[rr.seg].out[rr.row] = v;
                            if (EPI == EPI_ARGMAX) {
                                if (v > myBestV || (v == myBestV && rr.row < myBestI)) { myBestV = v; myBestI = rr.row; }
                            }
                        }
                    }
                    if (KS == 4) __syncthreads();
#pragma unroll
                    for (int i = 0; i < NR; i++) acc[i] = 0.f;
                }
            }
            issue(s, item + D);
        }
    }

    if (EPI == EPI_ARGMAX) {
        wave_argmax(myBestV, myBestI);
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

// Tall matrix of short rows (lm_head of a small model: K <= 1024*CH, so CH wave passes cover a row):
// a lane meets the same 16*CH activations in every row, so they are read from LDS once and stay in
// registers, and the loop is nothing but "four row loads, four dots, four reductions".  No ring:
// the loads of the waves a SIMD holds overlap each other.  Arithmetic and order are
// matvec_kernel's, so the two give the same bits.
template <int EPI, int CH, int NR>
__global__ __launch_bounds__(WG) void matvec_rows_q8_kernel(MvParams p) {
    extern __shared__ float4 a4[];
    __shared__ float red[4];
    __shared__ float bestV[4];
    __shared__ int bestI[4];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nch = p.K / 16;
    const int nrows = p.seg[0].rows;
    const char* __restrict__ w = static_cast<const char*>(p.seg[0].w);
    const float* __restrict__ scales = static_cast<const float*>(p.seg[0].aux);
    float* __restrict__ out = p.seg[0].out;
    const int gStep = gridDim.x * 4;

    int g = blockIdx.x * 4 + wave;
    int4 v[NR * CH];
    float scl = 0.f;
    auto fetch = [&](int gg) {
#pragma unroll
        for (int i = 0; i < NR; i++) {
            const int r = gg * NR + i;
#pragma unroll
            for (int ch = 0; ch < CH; ch++) {
                v[i * CH + ch] = make_int4(0, 0, 0, 0);
                if (r < nrows && lane + ch * 64 < nch) v[i * CH + ch] = *reinterpret_cast<const int4*>(w + (size_t)r * p.K + (lane + ch * 64) * 16);
            }
        }
        scl = 0.f;
        if (lane < NR && gg * NR + lane < nrows) scl = scales[gg * NR + lane];
    };
    if (g * NR < nrows) fetch(g);                    // the first rows go out before the vector is staged
    if (EPI == EPI_ARGMAX) fill_unset(p.xreset, p.xresetWords);

    const float rs = stage_activation<WF_Q8, PRO_RMS>(p, a4, red);
    float4 av[CH * 4];
#pragma unroll
    for (int ch = 0; ch < CH; ch++)
#pragma unroll
        for (int pl = 0; pl < 4; pl++) av[ch * 4 + pl] = lane + ch * 64 < nch ? a4[pl * nch + lane + ch * 64] : make_float4(0.f, 0.f, 0.f, 0.f);

    float myBestV = -INFINITY;
    int myBestI = INT_MAX;
    for (; g * NR < nrows; g += gStep) {
        float acc[NR];
#pragma unroll
        for (int i = 0; i < NR; i++) {
            float a = 0.f;
#pragma unroll
            for (int ch = 0; ch < CH; ch++) {
                a = dot4_i8(v[i * CH + ch].x, av[ch * 4], a); a = dot4_i8(v[i * CH + ch].y, av[ch * 4 + 1], a);
                a = dot4_i8(v[i * CH + ch].z, av[ch * 4 + 2], a); a = dot4_i8(v[i * CH + ch].w, av[ch * 4 + 3], a);
            }
            acc[i] = a;
            if (CH > 1) asm volatile("" : "+v"(acc[i]));    // finished here, not sunk below the next loads
        }
        const float sc = scl;
        const int gNext = g + gStep;
        if (gNext * NR < nrows) fetch(gNext);
#pragma unroll
        for (int i = 0; i < NR; i++) acc[i] = wave_sum(acc[i]);
        float val = acc[0];
#pragma unroll
        for (int i = 1; i < NR; i++) if (lane == i) val = acc[i];
        const int r = g * NR + lane;
        if (lane < NR && r < nrows) {
            val *= sc;
            val *= rs;
            out[r] = val;
            if (EPI == EPI_ARGMAX) {
                if (val > myBestV || (val == myBestV && r < myBestI)) { myBestV = val; myBestI = r; }
            }
        }
    }
    if (EPI == EPI_ARGMAX) {
        wave_argmax(myBestV, myBestI);
        if (lane == 0) { bestV[wave] = myBestV; bestI[wave] = myBestI; }
        __syncthreads();
        if (threadIdx.x == 0) {
            float bv = bestV[0]; int bi = bestI[0];
            for (int k = 1; k < 4; k++)
                if (bestV[k] > bv || (bestV[k] == bv && bestI[k] < bi)) { bv = bestV[k]; bi = bestI[k]; }
            p.amaxVal[blockIdx.x] = bv;
            p.amaxIdx[blockIdx.x] = bi;
        }
    }
}

// The same for Q4_0 rows in the split layout (K <= 1024): a lane owns one whole block (16 bytes of
// nibbles + its fp16 d), so a row takes K/32 <= 32 lanes and each half of the wave streams its own
// row; the lane's 32 activations and the two -8*sum terms stay in registers.
template <int EPI>
__global__ __launch_bounds__(WG) void matvec_rows_q4_kernel(MvParams p) {
    constexpr int NR = 4;                            // row pairs per step
    extern __shared__ float4 a4[];
    __shared__ float red[4];
    __shared__ float bestV[4];
    __shared__ int bestI[4];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int half = lane >> 5, bl = lane & 31;
    const int nblk = p.K / 32;
    const int nch = p.K / 16;
    const int nrows = p.seg[0].rows;
    const char* __restrict__ qs = static_cast<const char*>(p.seg[0].w);
    const unsigned short* __restrict__ dpl = reinterpret_cast<const unsigned short*>(qs + (size_t)nrows * (p.K >> 1));
    float* __restrict__ out = p.seg[0].out;
    const bool live = bl < nblk;
    const int gStep = gridDim.x * 4;

    int g = blockIdx.x * 4 + wave;
    int4 v[NR];
    unsigned short dh[NR];
    auto fetch = [&](int gg) {
#pragma unroll
        for (int i = 0; i < NR; i++) {
            const int r = (gg * NR + i) * 2 + half;
            v[i] = make_int4(0, 0, 0, 0);
            dh[i] = 0;
            if (r < nrows && live) {
                v[i] = *reinterpret_cast<const int4*>(qs + (size_t)r * (p.K >> 1) + bl * 16);
                dh[i] = dpl[(size_t)r * nblk + bl];
            }
        }
    };
    if (g * NR * 2 < nrows) fetch(g);
    if (EPI == EPI_ARGMAX) fill_unset(p.xreset, p.xresetWords);

    const float rs = stage_activation<WF_Q4P, PRO_RMS>(p, a4, red);
    // half block h of the lane's block: low nibbles meet lo[h][0..1], high nibbles hi[h][0..1]
    float4 avh[2][4];
    float asum[2];
#pragma unroll
    for (int h = 0; h < 2; h++) {
#pragma unroll
        for (int pl = 0; pl < 4; pl++) avh[h][pl] = live ? a4[pl * nch + bl * 2 + h] : make_float4(0.f, 0.f, 0.f, 0.f);
        float4 t;
        t.x = (avh[h][0].x + avh[h][1].x) + (avh[h][2].x + avh[h][3].x);
        t.y = (avh[h][0].y + avh[h][1].y) + (avh[h][2].y + avh[h][3].y);
        t.z = (avh[h][0].z + avh[h][1].z) + (avh[h][2].z + avh[h][3].z);
        t.w = (avh[h][0].w + avh[h][1].w) + (avh[h][2].w + avh[h][3].w);
        asum[h] = (t.x + t.y) + (t.z + t.w);
    }

    float myBestV = -INFINITY;
    int myBestI = INT_MAX;
#pragma nounroll
    for (; g * NR * 2 < nrows; g += gStep) {
        float acc[NR];
#pragma unroll
        for (int i = 0; i < NR; i++) {
            const float d = half_bits_to_float(dh[i]);
            float a = dot_q4_half(make_int2(v[i].x, v[i].y), d, avh[0], asum[0], 0.f);
            acc[i] = dot_q4_half(make_int2(v[i].z, v[i].w), d, avh[1], asum[1], a);
            asm volatile("" : "+v"(acc[i]));            // the row's sum is finished here, not sunk below the next loads
        }
        const int gNext = g + gStep;
        if (gNext * NR * 2 < nrows) fetch(gNext);
        float val = 0.f;
#pragma unroll
        for (int i = 0; i < NR; i++) {
            float a = acc[i];                        // sum over the 32 lanes of this half
            a += dpp_f<0xB1>(a); a += dpp_f<0x4E>(a); a += dpp_f<0x124>(a); a += dpp_f<0x128>(a);
            { float b = a; row_swap16(a, b); a += b; }
            if (bl == i) val = a;
        }
        const int r = (g * NR + bl) * 2 + half;
        if (bl < NR && r < nrows) {
            val *= rs;
            out[r] = val;
            if (EPI == EPI_ARGMAX) {
                if (val > myBestV || (val == myBestV && r < myBestI)) { myBestV = val; myBestI = r; }
            }
        }
    }
    if (EPI == EPI_ARGMAX) {
        wave_argmax(myBestV, myBestI);
        if (lane == 0) { bestV[wave] = myBestV; bestI[wave] = myBestI; }
        __syncthreads();
        if (threadIdx.x == 0) {
            float bv = bestV[0]; int bi = bestI[0];
            for (int k = 1; k < 4; k++)
                if (bestV[k] > bv || (bestV[k] == bv && bestI[k] < bi)) { bv = bestV[k]; bi = bestI[k]; }
            p.amaxVal[blockIdx.x] = bv;
            p.amaxIdx[blockIdx.x] = bi;
        }
    }
}

// Launch shape from measurements on MI355X (cold weights, all benchmark shapes):
// two rows per wave group is the best default, one for matrices of at most 1024 rows,
// four for very tall ones (lm_head), and the K split over the workgroup only pays for long rows with
// too few of them to give every CU a wave otherwise.
MvConfig pick_config(int wf, int epi, int totalRows, int K) {
    const int nch = K / 16;
    MvConfig c;
    c.ks = (nch > 128 && totalRows <= 2048) ? 4 : 1;
    if (epi == EPI_QKV) {
        c.nr = 2;
    } else if (epi == EPI_SWIGLU) {
        // totalRows counts gate rows; each group carries gate and up rows
        // short rows (K <= 1024): two gate and two up rows a wave group (Qwen Q4_0 step -2.8 %, Q8 -0.3 %);
        // neutral at K = 2048, 2 % slower at K = 4096
        c.nr = (totalRows >= 32768 || K <= 1024) ? 4 : 2;
    } else if (c.ks == 4) {
        c.nr = 4;
    } else {
        // few rows (Wo of a small model): one row a wave spreads them over twice the workgroups
        c.nr = totalRows >= 65536 ? 4 : (totalRows <= 1024 ? 1 : 2);
    }
    c.grid = 0;   // filled by the launcher from the group count
    return c;
}

template <int WF, int NR, int KS, int PRO, int EPI>
static hipError_t launch_t(MvParams& p, int grid, hipStream_t s) {
    size_t lds = (size_t)p.K * sizeof(float);
    const int K4 = p.K >> 2;
    // only for the launch shapes the decode step itself picks: NR 2, fused epilogues
    if constexpr (KS == 1 && NR == 2 && WF != WF_Q4RAW && (EPI == EPI_QKV || EPI == EPI_SWIGLU || EPI == EPI_RESID)) {
        if (K4 > WG && K4 <= 4 * WG) {                // a variant of its own: the batch costs registers the short vectors need not pay
            if (p.K / 16 <= 128 && p.ngroups <= grid * 4) {          // and one row group a wave in two chunk passes: two load slots, no ring
                hipLaunchKernelGGL((matvec_kernel<WF, NR, KS, PRO, EPI, true, true>), dim3(grid), dim3(WG), lds, s, p);
                return hipGetLastError();
            }
            hipLaunchKernelGGL((matvec_kernel<WF, NR, KS, PRO, EPI, true>), dim3(grid), dim3(WG), lds, s, p);
            return hipGetLastError();
        }
    }
    if constexpr (KS == 1 && WF != WF_Q4RAW && (EPI == EPI_QKV || EPI == EPI_SWIGLU || EPI == EPI_RESID) &&
                  (NR <= 2 || EPI == EPI_SWIGLU)) {
        if (p.K / 16 <= 64 && p.ngroups <= grid * 4) {           // one chunk pass a row (16 weights a lane), one group a wave
            hipLaunchKernelGGL((matvec_kernel<WF, NR, KS, PRO, EPI, false, true>), dim3(grid), dim3(WG), lds, s, p);
            return hipGetLastError();
        }
    }
    if constexpr (KS == 4 && NR == 4 && WF != WF_Q4RAW && PRO == PRO_PLAIN && EPI == EPI_RESID) {
        if (p.K / 16 <= 2 * WG) {                                // registers hold the thread's one or two chunks: no staging path
            hipLaunchKernelGGL((matvec_kernel<WF, NR, KS, PRO, EPI, false, true>), dim3(grid), dim3(WG), 0, s, p);   // nothing is staged in LDS
            return hipGetLastError();
        }
    }
    hipLaunchKernelGGL((matvec_kernel<WF, NR, KS, PRO, EPI>), dim3(grid), dim3(WG), lds, s, p);
    return hipGetLastError();
}

#define MV_CASE(NRV, KSV)                                                           \
    if (c.nr == NRV && c.ks == KSV) return launch_t<WF, NRV, KSV, PRO, EPI>(p, c.grid, s);

template <int WF, int PRO, int EPI>
static hipError_t launch_pe(MvParams& p, const MvConfig& c, hipStream_t s) {
    if (EPI == EPI_QKV) {
        MV_CASE(2, 1) MV_CASE(2, 4)
    } else if (EPI == EPI_SWIGLU) {
        MV_CASE(2, 1) MV_CASE(2, 4) MV_CASE(4, 1) MV_CASE(4, 4)
    } else {
        MV_CASE(1, 1) MV_CASE(1, 4) MV_CASE(2, 1) MV_CASE(2, 4) MV_CASE(4, 1) MV_CASE(4, 4)
    }
    return hipErrorInvalidValue;
}
#undef MV_CASE

template <int WF>
static hipError_t launch_wf(int pro, int epi, MvParams& p, const MvConfig& c, hipStream_t s) {
    if (pro == PRO_PLAIN && epi == EPI_STORE) return launch_pe<WF, PRO_PLAIN, EPI_STORE>(p, c, s);
    if (WF == WF_Q4RAW) return hipErrorInvalidValue;             // raw GGUF rows: per-op entry point only
    if (pro == PRO_RMS && epi == EPI_QKV) return launch_pe<WF == WF_Q4RAW ? WF_Q4P : WF, PRO_RMS, EPI_QKV>(p, c, s);
    if (pro == PRO_RMS && epi == EPI_SWIGLU) return launch_pe<WF == WF_Q4RAW ? WF_Q4P : WF, PRO_RMS, EPI_SWIGLU>(p, c, s);
    if (pro == PRO_PLAIN && epi == EPI_RESID) return launch_pe<WF == WF_Q4RAW ? WF_Q4P : WF, PRO_PLAIN, EPI_RESID>(p, c, s);
    if (pro == PRO_RMS && epi == EPI_ARGMAX) return launch_pe<WF == WF_Q4RAW ? WF_Q4P : WF, PRO_RMS, EPI_ARGMAX>(p, c, s);
    return hipErrorInvalidValue;
}

// Row grouping and grid of a launch: fills p.ngroups / p.segGroup0 and c (what launch_matvec runs with,
// the short-row lm_head kernels aside).
static hipError_t resolve_matvec(int wf, int epi, MvParams& p, const MvConfig* cfgInOut, MvConfig& c) {
    const int CH = wf == WF_Q8 ? 16 : 32;
    if (p.K <= 0 || p.K % CH != 0 || (size_t)p.K * 4 > 64 * 1024) return hipErrorInvalidValue;
    int total = 0;
    for (int i = 0; i < p.nseg; i++) total += p.seg[i].rows;
    c = (cfgInOut && cfgInOut->nr > 0) ? *cfgInOut
                                                : pick_config(wf, epi, epi == EPI_SWIGLU ? p.seg[0].rows : total, p.K);
    if (epi == EPI_SWIGLU) {
        if (p.nseg != 2 || p.seg[0].rows != p.seg[1].rows) return hipErrorInvalidValue;
        if (c.nr < 2) c.nr = 2;
        int h = c.nr / 2;
        p.ngroups = (p.seg[0].rows + h - 1) / h;
        p.segGroup0[0] = 0; p.segGroup0[1] = p.ngroups; p.segGroup0[2] = p.ngroups;
    } else if (epi == EPI_QKV) {
        // q and k rows pair up inside a head, so both need whole heads; v rows pair up consecutively
        if (p.nseg != 3 || p.headDim < 2 || (p.headDim & (p.headDim - 1)) || p.seg[0].rows % p.headDim ||
            p.seg[1].rows % p.headDim || p.seg[2].rows % 2)
            return hipErrorInvalidValue;
        c.nr = 2;
        int g = 0;
        for (int i = 0; i < 3; i++) { p.segGroup0[i] = g; g += p.seg[i].rows / 2; }
        p.ngroups = g;
    } else {
        int g = 0;
        for (int i = 0; i < 3; i++) {
            p.segGroup0[i] = g;
            if (i < p.nseg) g += (p.seg[i].rows + c.nr - 1) / c.nr;
        }
        p.ngroups = g;
    }
    if (p.ngroups == 0) return hipSuccess;
    const int wgs = c.ks == 1 ? (p.ngroups + 3) / 4 : p.ngroups;
    const int cap = epi == EPI_ARGMAX ? 1024 : 2048;      // one argmax partial per workgroup
    if (c.grid <= 0 || c.grid > wgs) {
        // every workgroup stages the activation vector: beyond the cap each takes several groups,
        // the same number each (an uneven last round leaves most of the chip idle)
        const int rounds = (wgs + cap - 1) / cap;
        c.grid = epi == EPI_ARGMAX ? (wgs < cap ? wgs : cap) : (wgs + rounds - 1) / rounds;
    }
    return hipSuccess;
}

hipError_t launch_matvec(int wf, int epi, int pro, MvParams& p, MvConfig* cfgInOut, hipStream_t s) {
    MvConfig c{0, 0, 0};
    hipError_t e = resolve_matvec(wf, epi, p, cfgInOut, c);
    if (e != hipSuccess) return e;
    if (p.ngroups == 0) return hipSuccess;
    int wgs;
    const int cap = epi == EPI_ARGMAX ? 1024 : 2048;
    if (wf == WF_Q8 && pro == PRO_RMS && epi == EPI_ARGMAX && p.nseg == 1 && !p.seg[0].bias && !p.div127 &&
        p.K / 16 <= 128 && c.ks == 1 && !(cfgInOut && cfgInOut->nr > 0)) {
        c.nr = 4;
        wgs = ((p.seg[0].rows + 3) / 4 + 3) / 4;
        c.grid = wgs < cap ? wgs : cap;
        if (cfgInOut) *cfgInOut = c;
        const size_t lds = (size_t)p.K * sizeof(float);
        if (p.K / 16 <= 64) hipLaunchKernelGGL((matvec_rows_q8_kernel<EPI_ARGMAX, 1, 4>), dim3(c.grid), dim3(WG), lds, s, p);
        else hipLaunchKernelGGL((matvec_rows_q8_kernel<EPI_ARGMAX, 2, 4>), dim3(c.grid), dim3(WG), lds, s, p);
        return hipGetLastError();
    }
    if (wf == WF_Q4P && pro == PRO_RMS && epi == EPI_ARGMAX && p.nseg == 1 && !p.seg[0].bias &&
        p.K / 32 <= 32 && c.ks == 1 && !(cfgInOut && cfgInOut->nr > 0)) {
        c.nr = 8;
        wgs = ((p.seg[0].rows + 7) / 8 + 3) / 4;
        c.grid = wgs < cap ? wgs : cap;
        if (cfgInOut) *cfgInOut = c;
        hipLaunchKernelGGL((matvec_rows_q4_kernel<EPI_ARGMAX>), dim3(c.grid), dim3(WG), (size_t)p.K * sizeof(float), s, p);
        return hipGetLastError();
    }
    if (cfgInOut) *cfgInOut = c;
    if (wf == WF_Q8) return launch_wf<WF_Q8>(pro, epi, p, c, s);
    if (wf == WF_Q4P) return launch_wf<WF_Q4P>(pro, epi, p, c, s);
    return launch_wf<WF_Q4RAW>(pro, epi, p, c, s);
}

size_t plan_matvec_prefetch(int wf, int epi, int pro, const MvParams& pin, PfJob& job, size_t limitBytes) {
    if (wf != WF_Q8 && wf != WF_Q4P) return 0;
    MvParams p = pin;
    MvConfig c{0, 0, 0};
    if (resolve_matvec(wf, epi, p, nullptr, c) != hipSuccess || p.ngroups == 0) return 0;
    const int wgs = c.ks == 1 ? (p.ngroups + 3) / 4 : p.ngroups;
    // several rounds of workgroups: workgroup b also takes groups b + grid, b + 2 grid, ..., which are
    // runs of its XCD only when grid is a multiple of 8
    if (c.grid != wgs && (c.grid & 7)) return 0;
    const size_t rowBytes = wf == WF_Q8 ? (size_t)p.K : (size_t)p.K / 2 + p.K / 16;
    size_t total = 0;
    for (int i = 0; i < p.nseg; i++) total += (size_t)p.seg[i].rows * rowBytes;
    const bool partial = limitBytes > 0 && limitBytes < total;
    if (partial && epi == EPI_QKV) return 0;         // q, k and v rows do not come in one order
    size_t takenBytes = 0;
    PfJob j = job;
    auto region = [&](const void* base, size_t bytes, size_t runBytes, int xoff) {
        if (j.nregion >= PF_MAX_REGIONS || bytes == 0 || bytes >= (1ull << 31)) return false;
        j.region[j.nregion++] = PfRegion{static_cast<const char*>(base), (unsigned)bytes, (unsigned)runBytes, xoff & 7,
                                         (int)((bytes + runBytes - 1) / runBytes), 0};
        return true;
    };
    auto flat = [&](const void* base, size_t bytes) {
        if (!base || bytes == 0) return true;
        if (j.nregion >= PF_MAX_REGIONS || bytes >= (1ull << 31)) return false;
        j.region[j.nregion++] = PfRegion{static_cast<const char*>(base), (unsigned)bytes, 1024u, -1, (int)((bytes + 1023) / 1024), 0};
        return true;
    };
    for (int i = 0; i < p.nseg; i++) {
        // rows of one workgroup are consecutive (q/k: two such pieces half a head apart, whose run
        // indices differ by a multiple of 8 once a head has 64 rows or more)
        int run, xoff;
        const int perWG = c.ks == 1 ? 4 : 1;         // row groups a workgroup takes
        if (epi == EPI_SWIGLU) {
            run = perWG * (c.nr / 2); xoff = 0;
        } else if (epi == EPI_QKV) {
            if (c.ks != 1 || p.headDim < 64 || (p.segGroup0[i] & 3)) return 0;
            run = i < 2 ? 4 : 8; xoff = p.segGroup0[i] >> 2;
        } else {
            if (c.ks == 1 && (p.segGroup0[i] & 3)) return 0;
            run = perWG * c.nr; xoff = c.ks == 1 ? p.segGroup0[i] >> 2 : p.segGroup0[i];
        }
        const size_t allRows = p.seg[i].rows;
        size_t rows = allRows;
        if (partial) {
            // the first rows of every segment (the workgroups that start first), whole sets of 8 runs
            const size_t set = (size_t)run * 8;
            rows = limitBytes / p.nseg / rowBytes / set * set;
            if (rows == 0) return 0;
            if (rows > allRows) rows = allRows;
        }
        const char* w = static_cast<const char*>(p.seg[i].w);
        if (wf == WF_Q8) {
            if (!region(w, rows * p.K, (size_t)run * p.K, xoff) || !flat(p.seg[i].aux, rows * 4)) return 0;
        } else {
            if (!region(w, rows * (p.K / 2), (size_t)run * (p.K / 2), xoff) ||
                !region(w + allRows * (p.K / 2), rows * (p.K / 16), (size_t)run * (p.K / 16), xoff))
                return 0;
        }
        if (!flat(p.seg[i].bias, rows * 4)) return 0;
        takenBytes += rows * rowBytes;
    }
    if (pro == PRO_RMS && !flat(p.gain, (size_t)p.K * 4)) return 0;
    job = j;
    return takenBytes;
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
// One workgroup = one KV head x up to GMAX of its GQA query heads (K/V rows are
// read once for all of them) x one split of the positions.  q arrives rotated
// and the K/V rows of the current position are already in the caches (the QKV
// matvec's epilogue did both).  The split geometry is fixed per context, so the
// first tile's K and V rows are requested before the position is known (rows
// past the end are clamped and masked): the critical path is one memory latency.
//
// K and V use the same register layout: a row of the head is spread over 16
// lanes (one DPP row; HD/64 float4s each, lanes 16 bytes apart: coalesced), and
// a thread holds the tile's rows tg + u*16.  A score is the lane's partial
// product reduced over the row's lanes by DPP; every lane
// of a row ends up with the score, which is exactly where P.V needs it -- the
// probabilities never leave registers.  A wave keeps its own running maximum
// (no barrier per tile); the running sum and the output stay per-thread
// partials over the thread's own rows and are reduced once at the end, where
// the waves' partials are weighted by exp(wave maximum - workgroup maximum).
// With several splits the last workgroup of a column to finish combines the
// partials, so the output is always the final [dim] vector.
// ---------------------------------------------------------------------------
// One float4 of a cache row: fp32 rows are read as they are, fp16 rows as 8 bytes and widened.
template <bool KVH>
__device__ __forceinline__ float4 ld_kv4(const void* base, size_t idx4) {
    if (!KVH) return static_cast<const float4*>(base)[idx4];
    typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
    const half4_t h = static_cast<const half4_t*>(base)[idx4];
    return make_float4((float)h[0], (float)h[1], (float)h[2], (float)h[3]);
}

// A helper workgroup of the attention launch (grid rows past the splits): its waves fetch their share
// of one region each into this XCD's L2.  Two scalar loads (the wave table, one region) come before
// the first fetch; the loads go straight into a 1 KB scrap area of LDS that nothing reads
// (global_load_lds_dwordx4: no destination register that a late load could overwrite), and none is
// waited for before the last one is out.
__device__ __forceinline__ void prefetch_helper(const PfJob& job, int firstFlat, int nWaves) {
    const int lane = threadIdx.x & 63;
    const int flatId = blockIdx.x + blockIdx.y * gridDim.x;      // dispatch order: XCD = flatId & 7
    const int x = flatId & 7;
    const int first = firstFlat + ((x - firstFlat) & 7);         // first helper on this XCD
    const int rank = (flatId - first) >> 3;                      // this workgroup among the XCD's helpers
    if (rank >= job.wgsPerXcd) return;
    const int hw = rank * nWaves + __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    int r = 0;
#pragma unroll
    for (int i = 1; i < PF_MAX_REGIONS; i++)
        if (i < job.nregion && hw >= job.waveStart[i]) r = i;
    const int lw = hw - job.waveStart[r];
    const int nw = job.waveStart[r + 1] - job.waveStart[r];
    if (lw >= nw) return;
    const PfRegion R = job.region[r];
    const unsigned end = (R.bytes + 15u) & ~15u;
    const int nruns = R.nruns;
    const int q0 = R.xoff < 0 ? 0 : (x - R.xoff) & 7;
    const int qs = R.xoff < 0 ? 1 : 8;                           // runs q0, q0 + qs, ...
    // long runs are shared by 2^splitLog2 waves (every wave gets about the same number of loads)
    const int sub = lw & ((1 << R.splitLog2) - 1);
    const int grp = lw >> R.splitLog2;
    const int ngrp = nw >> R.splitLog2;
    if (grp >= ngrp) return;
    __shared__ int4 scrap[64];
    for (int q = q0 + qs * grp; q < nruns; q += qs * ngrp) {
        const unsigned b0 = (unsigned)q * R.runBytes;
        unsigned b1 = b0 + R.runBytes;
        b1 = b1 < end ? (b1 + 15u) & ~15u : end;
        for (unsigned o = (b0 & ~15u) + (unsigned)sub * 1024 + lane * 16; o < b1; o += 1024u << R.splitLog2)
            __builtin_amdgcn_global_load_lds(reinterpret_cast<const int4*>(R.base + o), scrap, 16, 0, 0);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

template <int HD, int GMAX, bool KVH, int AWG = WG>
__global__ __launch_bounds__(AWG) void attn_decode_kernel(AttnParams p) {
    if (blockIdx.y >= p.smax) {                          // uniform: a whole workgroup is either a helper or not
        prefetch_helper(p.pf, p.smax * gridDim.x, AWG / 64);
        return;
    }
    constexpr int NWV = AWG / 64;      // waves: 4, or more for the one-head workgroups of short contexts (fewer rows per thread)
    constexpr int LPR = 16;            // lanes per K/V row: one DPP row
    constexpr int NF = HD / 64;        // float4s of a row per lane (float4 index j*16 + dl)
    constexpr int TG = AWG / LPR;      // rows in flight per load step (16 or 32)
    constexpr int VU = 16 / NF / (AWG / WG);   // rows per thread and tile
    constexpr int TILE = TG * VU;      // positions per tile (256 for head size 64, 128 for 128)
    __shared__ float wred[GMAX][NWV];                  // the waves' running maxima, for the final combination
    __shared__ float4 accbuf[NWV][GMAX][HD / 4];
    __shared__ float lbuf[NWV][GMAX];
    __shared__ int lastFlag;

    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int G = p.nHeads / p.nKVHeads;
    const int nChunks = (G + GMAX - 1) / GMAX;
    const int kvh = blockIdx.x / nChunks;
    const int chunk = blockIdx.x % nChunks;
    const int h0 = kvh * G + chunk * GMAX;
    const int gn = min(GMAX, G - chunk * GMAX);
    const int split = blockIdx.y;
    const int kvOff = kvh * HD;
    const int tg = tid / LPR, dl = tid % LPR;
    const int t0 = p.splitLen > 0 ? split * p.splitLen : 0;
    const int lastRow = p.rowLimit - 1;
    const size_t rowStride = (size_t)p.kvDim / 4;
    const size_t colOff = (size_t)kvOff / 4 + dl;      // float4 index of this lane's first piece inside a row

    // ---- everything that does not need the position goes out first ----
    float4 q4[GMAX][NF];
#pragma unroll
    for (int g = 0; g < GMAX; g++)             // heads past gn work on zeros and are dropped at the end
#pragma unroll
        for (int j = 0; j < NF; j++) {
            q4[g][j] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (g < gn) q4[g][j] = reinterpret_cast<const float4*>(p.q + (size_t)(h0 + g) * HD)[j * 16 + dl];
        }
    // K and V rows alternate in issue order, lowest rows first: the load unit works through them in
    // that order, and a short context only waits for the rows it has (the rest is never looked at).
    float4 kreg[VU][NF], vreg[VU][NF];
#pragma unroll
    for (int u = 0; u < VU; u++) {
#pragma unroll
        for (int j = 0; j < NF; j++) kreg[u][j] = ld_kv4<KVH>(p.Kc, (size_t)min(t0 + tg + u * TG, lastRow) * rowStride + colOff + j * 16);
#pragma unroll
        for (int j = 0; j < NF; j++) vreg[u][j] = ld_kv4<KVH>(p.Vc, (size_t)min(t0 + tg + u * TG, lastRow) * rowStride + colOff + j * 16);
    }

    const int pos = p.state ? p.state->pos : p.posImm;     // compiles to a branch and a scalar load (checked)
    const int len = pos + 1;
    if (t0 >= len) return;                                 // this split holds no position yet
    const int nsplit = p.splitLen > 0 ? (len + p.splitLen - 1) / p.splitLen : 1;
    const int t1 = p.splitLen > 0 ? min(len, t0 + p.splitLen) : len;

    const float scale = 1.0f / sqrtf((float)HD);     // mongoose.cu:867 rsqrtf(headDim)
    float m[GMAX], l[GMAX];                           // m: the wave's running max; l, acc: this thread's rows only
    float4 acc[GMAX][NF];
#pragma unroll
    for (int g = 0; g < GMAX; g++) {
        m[g] = -INFINITY; l[g] = 0.f;
#pragma unroll
        for (int j = 0; j < NF; j++) acc[g][j] = make_float4(0.f, 0.f, 0.f, 0.f);
    }

    for (int tile = t0; tile < t1; tile += TILE) {
        if (tile != t0) {
#pragma unroll
            for (int u = 0; u < VU; u++) {
#pragma unroll
                for (int j = 0; j < NF; j++) kreg[u][j] = ld_kv4<KVH>(p.Kc, (size_t)min(tile + tg + u * TG, lastRow) * rowStride + colOff + j * 16);
#pragma unroll
                for (int j = 0; j < NF; j++) vreg[u][j] = ld_kv4<KVH>(p.Vc, (size_t)min(tile + tg + u * TG, lastRow) * rowStride + colOff + j * 16);
            }
        }
        const int live = t1 - tile;                        // positions of this tile that exist (uniform)
        float sc[GMAX][VU], tmaxg[GMAX];
#pragma unroll
        for (int g = 0; g < GMAX; g++) {
            float tmax = -INFINITY;
#pragma unroll
            for (int u = 0; u < VU; u++) {
                sc[g][u] = -INFINITY;
                if (u * TG >= live) continue;              // whole row step past the end: its loads are not waited for
                float d = 0.f;
#pragma unroll
                for (int j = 0; j < NF; j++) {
                    d = fmaf(q4[g][j].x, kreg[u][j].x, d);
                    d = fmaf(q4[g][j].y, kreg[u][j].y, d);
                    d = fmaf(q4[g][j].z, kreg[u][j].z, d);
                    d = fmaf(q4[g][j].w, kreg[u][j].w, d);
                }
                d = row_sum16(d);
                sc[g][u] = (tile + tg + u * TG < t1) ? d * scale : -INFINITY;
                tmax = fmaxf(tmax, sc[g][u]);
            }
            tmaxg[g] = tg_max(tmax);                       // the wave's maximum: no other wave is asked
        }
#pragma unroll
        for (int g = 0; g < GMAX; g++) {
            const float mNew = fmaxf(m[g], tmaxg[g]);
            const float mRef = mNew == -INFINITY ? 0.f : mNew;     // a wave none of whose rows exist yet
            const float corr = exp_neg(m[g] - mRef);       // first tile: exp(-inf) = 0
            m[g] = mNew;
            float ps = 0.f;
#pragma unroll
            for (int j = 0; j < NF; j++) { acc[g][j].x *= corr; acc[g][j].y *= corr; acc[g][j].z *= corr; acc[g][j].w *= corr; }
#pragma unroll
            for (int u = 0; u < VU; u++) {
                if (u * TG >= live) continue;
                const float pv = exp_neg(sc[g][u] - mRef); // masked rows: exp(-inf) = 0
                ps += pv;
#pragma unroll
                for (int j = 0; j < NF; j++) {
                    acc[g][j].x = fmaf(pv, vreg[u][j].x, acc[g][j].x);
                    acc[g][j].y = fmaf(pv, vreg[u][j].y, acc[g][j].y);
                    acc[g][j].z = fmaf(pv, vreg[u][j].z, acc[g][j].z);
                    acc[g][j].w = fmaf(pv, vreg[u][j].w, acc[g][j].w);
                }
            }
            l[g] = l[g] * corr + ps;
        }
    }

    // ---- reduce the per-thread partials over the row groups: in the wave, then across waves ----
#pragma unroll
    for (int g = 0; g < GMAX; g++) {
#pragma unroll
        for (int j = 0; j < NF; j++) {
            acc[g][j].x = tg_sum(acc[g][j].x); acc[g][j].y = tg_sum(acc[g][j].y);
            acc[g][j].z = tg_sum(acc[g][j].z); acc[g][j].w = tg_sum(acc[g][j].w);
            if ((tid & 63) < LPR) accbuf[wave][g][j * 16 + dl] = acc[g][j];
        }
        l[g] = tg_sum(l[g]);
        if ((tid & 63) == 0) { lbuf[wave][g] = l[g]; wred[g][wave] = m[g]; }
    }
    __syncthreads();
    constexpr int F4 = HD / 4;                             // float4s of a head
    for (int i = tid; i < gn * F4; i += AWG) {
        int g = i / F4, d4 = i % F4;
        // every wave kept its own running maximum: the workgroup's is the greatest of them (finite, the
        // split holds at least one position), and a wave's sums count with exp(its maximum - that)
        float mg_ = wred[g][0];
#pragma unroll
        for (int k = 1; k < NWV; k++) mg_ = fmaxf(mg_, wred[g][k]);
        float4 r = make_float4(0.f, 0.f, 0.f, 0.f);
        float lg = 0.f;                                    // lbuf holds lane 0's column of each wave: every row's probability exactly once
#pragma unroll
        for (int k = 0; k < NWV; k++) {
            const float w = exp_neg(wred[g][k] - mg_);     // a wave without rows: exp(-inf) = 0
            const float4 a = accbuf[k][g][d4];
            r.x = fmaf(w, a.x, r.x); r.y = fmaf(w, a.y, r.y); r.z = fmaf(w, a.z, r.z); r.w = fmaf(w, a.w, r.w);
            lg = fmaf(w, lbuf[k][g], lg);
        }
        int h = h0 + g;
        if (nsplit == 1) {
            float4 o;
            const float il = __builtin_amdgcn_rcpf(lg);
            o.x = r.x * il; o.y = r.y * il; o.z = r.z * il; o.w = r.w * il;
            reinterpret_cast<float4*>(p.out + (size_t)h * HD)[d4] = o;
        } else {
            float* pa = p.pacc + ((size_t)h * p.smax + split) * HD + d4 * 4;
            st_agent(pa, r.x); st_agent(pa + 1, r.y); st_agent(pa + 2, r.z); st_agent(pa + 3, r.w);
            if (d4 == 0) {
                st_agent(p.pm + (size_t)h * p.smax + split, mg_);
                st_agent(p.pl + (size_t)h * p.smax + split, lg);
            }
        }
    }
    if (nsplit == 1) return;

    // ---- several splits: the last workgroup of this column combines ----
    // The partials were stored write-through at agent scope, so "release" is just waiting
    // for those stores to be acknowledged; a full release fence would also write back the
    // whole L2 from every workgroup, which serialises them.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) {
        int old = __hip_atomic_fetch_add(p.counters + blockIdx.x, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        lastFlag = (old == nsplit - 1);
    }
    __syncthreads();
    if (!lastFlag) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");     // drop cached copies of the other workgroups' partials
    // The workgroup's threads form NG groups of IT = GMAX*F4 items (head, float4 of the head); group q
    // merges the splits q, q+NG, ... 16 at a time -- all 48 loads of a batch are issued before the first
    // is used, one memory round trip a batch, and up to 16*NG splits need only one -- and the NG results
    // of an item are folded through LDS with the same running-maximum rescale.
    constexpr int IT = GMAX * F4;
    constexpr int NG = AWG / IT;
    __shared__ float4 cnum[AWG];
    __shared__ float cM[AWG], cden[AWG];
    {
        const int q = tid / IT, i = tid % IT;
        const int g = i / F4, d4 = i % F4;
        const int h = h0 + min(g, gn - 1);                           // heads past gn repeat the last one, dropped below
        const float* pm = p.pm + (size_t)h * p.smax;
        const float* pl = p.pl + (size_t)h * p.smax;
        const float4* pa = reinterpret_cast<const float4*>(p.pacc + (size_t)h * p.smax * HD) + d4;
        float M = -INFINITY, den = 0.f;
        float4 num = make_float4(0.f, 0.f, 0.f, 0.f);
        for (int s0 = q; s0 < nsplit; s0 += 16 * NG) {
            float pmv[16], plv[16];
            float4 pav[16];
#pragma unroll
            for (int u = 0; u < 16; u++) {
                const int sidx = min(s0 + u * NG, nsplit - 1);      // clamped, unconditional: stays in registers
                pmv[u] = pm[sidx]; plv[u] = pl[sidx]; pav[u] = pa[(size_t)sidx * F4];
            }
            float bm = -INFINITY;
#pragma unroll
            for (int u = 0; u < 16; u++) if (s0 + u * NG < nsplit) bm = fmaxf(bm, pmv[u]);
            const float Mn = fmaxf(M, bm);
            const float c = exp_neg(M - Mn);                           // first batch: exp(-inf) = 0
            den *= c; num.x *= c; num.y *= c; num.z *= c; num.w *= c;
            M = Mn;
#pragma unroll
            for (int u = 0; u < 16; u++) {
                if (s0 + u * NG < nsplit) {
                    const float w = exp_neg(pmv[u] - M);
                    den = fmaf(w, plv[u], den);
                    num.x = fmaf(w, pav[u].x, num.x); num.y = fmaf(w, pav[u].y, num.y);
                    num.z = fmaf(w, pav[u].z, num.z); num.w = fmaf(w, pav[u].w, num.w);
                }
            }
        }
        cM[tid] = M; cden[tid] = den; cnum[tid] = num;              // a group without splits leaves (-inf, 0, 0)
        __syncthreads();
        if (q == 0 && g < gn) {
            float Mt = cM[i];
#pragma unroll
            for (int k = 1; k < NG; k++) Mt = fmaxf(Mt, cM[k * IT + i]);
            float dt = 0.f;
            float4 nt = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int k = 0; k < NG; k++) {
                const float w = exp_neg(cM[k * IT + i] - Mt);           // empty group: exp(-inf) = 0
                const float4 a = cnum[k * IT + i];
                dt = fmaf(w, cden[k * IT + i], dt);
                nt.x = fmaf(w, a.x, nt.x); nt.y = fmaf(w, a.y, nt.y); nt.z = fmaf(w, a.z, nt.z); nt.w = fmaf(w, a.w, nt.w);
            }
            float4 o;
            o.x = nt.x / dt; o.y = nt.y / dt; o.z = nt.z / dt; o.w = nt.w / dt;
            reinterpret_cast<float4*>(p.out + (size_t)h * HD)[d4] = o;
        }
    }
    if (tid == 0) __hip_atomic_store(p.counters + blockIdx.x, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Query heads handled per workgroup.  Long contexts: the whole GQA group (K/V
// rows are fetched from HBM once).  Short contexts are latency-bound and the
// K/V rows of a layer sit in L2, so the group is spread over more workgroups.
static int attention_gmax(int G, int heads) {
    int want = heads > 0 ? heads : G;
    if (want > G) want = G;
    return want >= 3 ? 4 : (want == 2 ? 2 : 1);      // scores of GMAX heads x 16 rows live in registers: at most 4
}

template <int HD, bool KVH>
static hipError_t launch_attn_hd(const AttnParams& pin, hipStream_t s) {
    AttnParams p = pin;
    int G = p.nHeads / p.nKVHeads;
    int gmax = attention_gmax(G, p.headsPerWG);
    int nChunks = (G + gmax - 1) / gmax;
    const int cols = p.nKVHeads * nChunks;
    const int wavesPerWG = gmax == 1 ? 8 : 4;
    p.pf.rows = 0;
    if (p.pf.helperWaves > 0 && p.pf.nregion > 0) {
        // helper workgroups: the same number on every XCD (a few of the last grid row stay idle); the
        // XCD's helper waves are shared out over the regions by the loads an XCD issues for each
        const int rows = (p.pf.helperWaves + wavesPerWG * cols - 1) / (wavesPerWG * cols);
        const int perXcd = rows * cols / 8;
        const int W = perXcd * wavesPerWG;
        if (W >= p.pf.nregion) {
            double share[PF_MAX_REGIONS], total = 0.0;
            for (int i = 0; i < p.pf.nregion; i++) {
                // in load instructions (1 KB a wave): a region of short runs needs as many as one of long runs
                const PfRegion& R = p.pf.region[i];
                share[i] = (double)((R.runBytes + 1023) / 1024) * (R.xoff < 0 ? R.nruns : (R.nruns + 7) / 8);
                total += share[i];
            }
            int spare = W - p.pf.nregion, at = 0;        // one wave each, the rest by share
            double acc = 0.0;
            for (int i = 0; i < p.pf.nregion; i++) {
                p.pf.waveStart[i] = at;
                const int before = (int)(acc / total * spare + 0.5);
                acc += share[i];
                at += 1 + (int)(acc / total * spare + 0.5) - before;
            }
            p.pf.waveStart[p.pf.nregion] = at;
            for (int i = 0; i < p.pf.nregion; i++) {
                PfRegion& R = p.pf.region[i];
                const int nw = p.pf.waveStart[i + 1] - p.pf.waveStart[i];
                const int runsHere = R.xoff < 0 ? R.nruns : (R.nruns + 7) / 8;
                const int pieces = (int)((R.runBytes + 1023) / 1024);
                int s2 = 0;
                while ((nw >> s2) > runsHere && (2 << s2) <= pieces) s2++;
                R.splitLog2 = s2;
            }
            p.pf.rows = rows;
            p.pf.wgsPerXcd = perXcd;
        }
    }
    dim3 grid(cols, p.smax + p.pf.rows);
    switch (gmax) {
    case 1: hipLaunchKernelGGL((attn_decode_kernel<HD, 1, KVH, 2 * WG>), grid, dim3(2 * WG), 0, s, p); break;
    case 2: hipLaunchKernelGGL((attn_decode_kernel<HD, 2, KVH>), grid, dim3(WG), 0, s, p); break;
    default: hipLaunchKernelGGL((attn_decode_kernel<HD, 4, KVH>), grid, dim3(WG), 0, s, p); break;
    }
    return hipGetLastError();
}

// Columns of workgroups an attention launch uses (size of the counter array).
int attention_columns(int nHeads, int nKVHeads, int headsPerWG) {
    int G = nHeads / nKVHeads;
    int gmax = attention_gmax(G, headsPerWG);
    return nKVHeads * ((G + gmax - 1) / gmax);
}

hipError_t launch_attention(const AttnParams& p, hipStream_t s) {
    if (p.nKVHeads <= 0 || p.nHeads % p.nKVHeads != 0 || p.rowLimit <= 0 || p.smax < 1) return hipErrorInvalidValue;
    const int tile = p.headDim == 128 ? WG / 2 : WG;
    if (p.smax > 1 && (p.splitLen <= 0 || p.splitLen % tile != 0 || !p.counters || !p.pm || !p.pl || !p.pacc)) return hipErrorInvalidValue;
    if (p.headDim == 64) return p.kvHalf ? launch_attn_hd<64, true>(p, s) : launch_attn_hd<64, false>(p, s);
    if (p.headDim == 128) return p.kvHalf ? launch_attn_hd<128, true>(p, s) : launch_attn_hd<128, false>(p, s);
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

// mongoose.cu:372-404: out = rmsnorm(a + b, w).  The sum goes into out first and is scaled in place,
// so out may be a or b.
__global__ __launch_bounds__(WG) void fused_add_rmsnorm_kernel(const float* a, const float* b, float* out, const float* w,
                                                               int dim, float eps) {
    __shared__ float red[4];
    const float* ar = a + (size_t)blockIdx.x * dim;
    const float* br = b + (size_t)blockIdx.x * dim;
    float* o = out + (size_t)blockIdx.x * dim;
    float ss = 0.f;
    for (int i = threadIdx.x; i < dim; i += WG) {
        const float v = ar[i] + br[i];
        o[i] = v;
        ss += v * v;
    }
    float tot = block_sum(ss, red);
    float rs = 1.0f / sqrtf(tot / (float)dim + eps);
    for (int i = threadIdx.x; i < dim; i += WG) o[i] = o[i] * rs * w[i];      // a thread re-reads only what it wrote
}
hipError_t launch_fused_add_rmsnorm(const float* a, const float* b, float* out, const float* w, int seqLen, int dim, float eps,
                                    hipStream_t s) {
    if (seqLen <= 0) return hipSuccess;
    hipLaunchKernelGGL(fused_add_rmsnorm_kernel, dim3(seqLen), dim3(WG), 0, s, a, b, out, w, dim, eps);
    return hipGetLastError();
}

// mongoose.cu:1598-1630: per-row-scale 4-bit weights, two per byte in sequence (low nibble = element
// 2k, high nibble = element 2k+1), value (nib - 8) * (scales[row] / 7).  One wave per row; a lane
// takes four bytes (eight weights) at a time when rows are word-aligned, single bytes otherwise.
__global__ __launch_bounds__(WG) void q4_rowscale_matvec_kernel(const float* act, const unsigned char* w, const float* scales,
                                                                float* out, int N, int K, int words) {
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (row >= N) return;
    const int halfK = K / 2;
    const unsigned char* wr = w + (size_t)row * halfK;
    float sum = 0.f;
    int k0 = 0;
    if (words) {
        const unsigned* w4 = reinterpret_cast<const unsigned*>(wr);
        const int nw = halfK / 4;
        for (int i = lane; i < nw; i += 64) {
            const unsigned q = w4[i];
            const float* a = act + (size_t)i * 8;
#pragma unroll
            for (int b = 0; b < 4; b++) {
                const unsigned byte = (q >> (8 * b)) & 0xffu;
                sum = fmaf(a[2 * b], (float)((int)(byte & 0xfu) - 8), sum);
                sum = fmaf(a[2 * b + 1], (float)((int)(byte >> 4) - 8), sum);
            }
        }
        k0 = nw * 4;
    }
    for (int k = k0 + lane; k < halfK; k += 64) {
        const unsigned byte = wr[k];
        sum = fmaf(act[2 * k], (float)((int)(byte & 0xfu) - 8), sum);
        sum = fmaf(act[2 * k + 1], (float)((int)(byte >> 4) - 8), sum);
    }
    sum = wave_sum(sum);
    if (lane == 0) out[row] = sum * (scales[row] / 7.0f);
}
hipError_t launch_q4_rowscale_matvec(const float* act, const void* w, const float* scales, float* out, int N, int K, hipStream_t s) {
    if (N <= 0 || K <= 0) return hipSuccess;
    if (K & 1) return hipErrorInvalidValue;
    const int words = ((K / 2) % 4 == 0 && ((uintptr_t)w & 3) == 0) ? 1 : 0;
    hipLaunchKernelGGL(q4_rowscale_matvec_kernel, dim3((N + 3) / 4), dim3(WG), 0, s, act, static_cast<const unsigned char*>(w),
                       scales, out, N, K, words);
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
__global__ void kv_cache_write_f16_kernel(_Float16* cache, const float* src, int pos, int kvDim) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < kvDim) cache[(size_t)pos * kvDim + i] = (_Float16)src[i];
}
hipError_t launch_kv_cache_write_f16(void* cache, const float* src, int pos, int kvDim, hipStream_t s) {
    hipLaunchKernelGGL(kv_cache_write_f16_kernel, dim3((kvDim + WG - 1) / WG), dim3(WG), 0, s, static_cast<_Float16*>(cache), src, pos, kvDim);
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
    if (((uintptr_t)ptr & 3) != 0) {
        // unaligned start: the bytes up to the next word boundary by the same kernel (a fill kernel, not a
        // memset node, so that the call stays safe inside a captured graph), then the aligned rest
        const size_t head = 4 - ((uintptr_t)ptr & 3);
        const size_t n = head < bytes ? head : bytes;
        hipLaunchKernelGGL(fill_zero_kernel, dim3(1), dim3(WG), 0, s, static_cast<unsigned*>(nullptr), (size_t)0,
                           static_cast<unsigned char*>(ptr), (int)n);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess || n == bytes) return e;
        ptr = static_cast<unsigned char*>(ptr) + n;
        bytes -= n;
    }
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
__device__ __forceinline__ void embed_element(int kind, const void* table, const float* scales, int tok, float* x, int dim, int vocab, int i) {
    x[i] = embed_value(kind, table, scales, tok, dim, vocab, i);
}
// Row `tok` of the table into e.out, by the whole workgroup.
__device__ __forceinline__ void embed_gather(const EmbedRef& e, int tok) {
    if (!e.out) return;
    if (tok < 0) tok = 0;
    if (tok >= e.vocab) tok = e.vocab - 1;
    for (int i = threadIdx.x; i < e.dim; i += blockDim.x) embed_element(e.kind, e.table, e.scales, tok, e.out, e.dim, e.vocab, i);
}
__global__ void embed_token_kernel(int kind, const void* table, const float* scales, const StepState* state,
                                   float* x, int dim, int vocab) {
    int tok = state->token;
    if (tok < 0) tok = 0;
    if (tok >= vocab) tok = vocab - 1;
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= dim) return;
    embed_element(kind, table, scales, tok, x, dim, vocab, i);
}
hipError_t launch_embed_token(int kind, const void* table, const float* scales, const StepState* state, float* x,
                              int dim, int vocab, hipStream_t s) {
    hipLaunchKernelGGL(embed_token_kernel, dim3((dim + WG - 1) / WG), dim3(WG), 0, s, kind, table, scales, state, x, dim, vocab);
    return hipGetLastError();
}

// cos/sin row of position `pos` -> rope.cur (cos then sin), by the whole workgroup
__device__ __forceinline__ void copy_rope_row(const RopeCur& rope, int pos) {
    if (!rope.cur) return;
    if (pos >= rope.maxSeq) pos = rope.maxSeq - 1;
    for (int j = threadIdx.x; j < rope.half; j += blockDim.x) {
        rope.cur[j] = rope.cosTab[(size_t)pos * rope.half + j];
        rope.cur[rope.half + j] = rope.sinTab[(size_t)pos * rope.half + j];
    }
}

__global__ __launch_bounds__(WG) void argmax_finish_kernel(const float* pv, const int* pi, int nparts, StepState* state,
                                                           const int* prompt, int* history, int historyCap, int vocab,
                                                           RopeCur rope, EmbedRef emb) {
    __shared__ float bv[WG / 64];
    __shared__ int bi[WG / 64];
    __shared__ int nextTok;
    const int np = state->pos + 1;
    copy_rope_row(rope, np);
    float v = -INFINITY;
    int idx = INT_MAX;
    for (int i = threadIdx.x; i < nparts; i += WG) {
        float ov = pv[i]; int oi = pi[i];
        if (ov > v || (ov == v && oi < idx)) { v = ov; idx = oi; }
    }
    // inside the wave without LDS, then the four waves' results through it: one barrier instead of nine
    wave_argmax(v, idx);
    if ((threadIdx.x & 63) == 0) { bv[threadIdx.x >> 6] = v; bi[threadIdx.x >> 6] = idx; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < WG / 64; w++) argmax_pick(v, idx, bv[w], bi[w]);
        int tok = idx;
        if (tok < 0 || tok >= vocab) tok = 0;
        int next = tok;
        if (prompt && np < state->nPrompt) next = prompt[np];
        int cnt = state->count;
        if (history && cnt < historyCap) history[cnt] = tok;
        state->count = cnt + 1;
        state->token = next;
        state->pos = np;
        nextTok = next;
    }
    if (emb.out) {                                   // uniform: the next step's embedding, one launch saved
        __syncthreads();
        embed_gather(emb, nextTok);
    }
}
hipError_t launch_argmax_finish(const float* pv, const int* pi, int nparts, StepState* state, const int* prompt,
                                int* history, int historyCap, int vocab, RopeCur rope, EmbedRef emb, hipStream_t s) {
    hipLaunchKernelGGL(argmax_finish_kernel, dim3(1), dim3(WG), 0, s, pv, pi, nparts, state, prompt, history, historyCap, vocab, rope, emb);
    return hipGetLastError();
}

__global__ void set_state_kernel(StepState* state, int pos, int token, int count, int nPrompt, RopeCur rope) {
    copy_rope_row(rope, pos);
    if (threadIdx.x == 0) { state->pos = pos; state->token = token; state->count = count; state->nPrompt = nPrompt; }
}
hipError_t launch_set_state(StepState* state, int pos, int token, int count, int nPrompt, RopeCur rope, hipStream_t s) {
    hipLaunchKernelGGL(set_state_kernel, dim3(1), dim3(64), 0, s, state, pos, token, count, nPrompt, rope);
    return hipGetLastError();
}

__global__ void advance_prompt_kernel(StepState* state, const int* prompt, RopeCur rope, EmbedRef emb) {
    int np = state->pos + 1;
    copy_rope_row(rope, np);
    const int tok = np < state->nPrompt ? prompt[np] : state->token;      // every thread reads the same words
    if (emb.out) embed_gather(emb, tok);
    __syncthreads();                                 // every wave has read the old position before it changes
    if (threadIdx.x == 0) {
        state->pos = np;
        state->token = tok;
    }
}
hipError_t launch_advance_prompt(StepState* state, const int* prompt, RopeCur rope, EmbedRef emb, hipStream_t s) {
    hipLaunchKernelGGL(advance_prompt_kernel, dim3(1), dim3(emb.out ? WG : 64), 0, s, state, prompt, rope, emb);
    return hipGetLastError();
}

// Holds the stream until the host sets *flag (or the tick limit passes), so
// that the host can queue a whole batch of launches ahead of the GPU.  One
// lane; always exits.
__global__ void signal_mailbox_kernel(unsigned* counter, unsigned value) {
    // the stream orders this kernel behind the stage's launches; the fence makes their writes
    // visible to the host before the counter moves
    __atomic_thread_fence(__ATOMIC_SEQ_CST);
    __hip_atomic_store(counter, value, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}
hipError_t launch_signal_mailbox(unsigned* counter, unsigned value, hipStream_t s) {
    hipLaunchKernelGGL(signal_mailbox_kernel, dim3(1), dim3(1), 0, s, counter, value);
    return hipGetLastError();
}

__global__ void gate_kernel(const volatile int* flag, long long limitTicks) {
    const long long t0 = wall_clock64();
    while (__hip_atomic_load(const_cast<const int*>(flag), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) == 0) {
        if (wall_clock64() - t0 > limitTicks) break;
        __builtin_amdgcn_s_sleep(32);
    }
}
hipError_t launch_gate(const int* flag, long long limitTicks, hipStream_t s) {
    hipLaunchKernelGGL(gate_kernel, dim3(1), dim3(1), 0, s, flag, limitTicks);
    return hipGetLastError();
}

}  // namespace mg
