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
template <typename KVT>
__global__ void rope_store_rows_kernel(float* q, const float* k, const float* v, KVT* Kc, KVT* Vc,
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
    KVT* kd = Kc + (size_t)pos * kvDim;
    KVT* vd = Vc + (size_t)pos * kvDim;
    for (int i = threadIdx.x; i < kvDim / 2; i += blockDim.x) {
        int h = i / half, j = i % half;
        float x0 = kr[h * headDim + j], x1 = kr[h * headDim + half + j];
        kd[h * headDim + j] = (KVT)(x0 * c[j] - x1 * s[j]);
        kd[h * headDim + half + j] = (KVT)(x0 * s[j] + x1 * c[j]);
    }
    for (int i = threadIdx.x; i < kvDim; i += blockDim.x) vd[i] = (KVT)vr[i];
}
hipError_t launch_rope_store_rows(float* q, const float* k, const float* v, void* Kc, void* Vc, int kvHalf, const float* cosTab,
                                  const float* sinTab, int pos0, int T, int dim, int kvDim, int headDim, hipStream_t s) {
    if (T <= 0) return hipSuccess;
    if (kvHalf)
        hipLaunchKernelGGL(rope_store_rows_kernel<_Float16>, dim3(T), dim3(PWG), 0, s, q, k, v, static_cast<_Float16*>(Kc),
                           static_cast<_Float16*>(Vc), cosTab, sinTab, pos0, dim, kvDim, headDim);
    else
        hipLaunchKernelGGL(rope_store_rows_kernel<float>, dim3(T), dim3(PWG), 0, s, q, k, v, static_cast<float*>(Kc),
                           static_cast<float*>(Vc), cosTab, sinTab, pos0, dim, kvDim, headDim);
    return hipGetLastError();
}

// Embedding rows of T tokens from the tied Q8 table (kind 0), an fp16 (1) / fp32 (2) table, or the
// tied Q4_0 table in the split layout (3).
__global__ void embed_rows_kernel(int kind, const void* table, const float* scales, const int* tokens, float* x, int dim, int vocab) {
    int tok = tokens[blockIdx.x];
    tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
    float* o = x + (size_t)blockIdx.x * dim;
    for (int i = threadIdx.x; i < dim; i += blockDim.x) {
        if (kind == 0) o[i] = (float)static_cast<const signed char*>(table)[(size_t)tok * dim + i] * scales[tok];
        else if (kind == 1) o[i] = (float)__builtin_bit_cast(_Float16, static_cast<const unsigned short*>(table)[(size_t)tok * dim + i]);
        else if (kind == 2) o[i] = static_cast<const float*>(table)[(size_t)tok * dim + i];
        else {
            const unsigned char* base = static_cast<const unsigned char*>(table);
            const int nb = dim >> 5, b = i >> 5, e = i & 31;
            const unsigned char byte = base[((size_t)tok * nb + b) * 16 + (e & 15)];
            const int nib = e < 16 ? (byte & 15) : (byte >> 4);
            const unsigned short dh = reinterpret_cast<const unsigned short*>(base + (size_t)vocab * (dim >> 1))[(size_t)tok * nb + b];
            o[i] = (float)(nib - 8) * (float)__builtin_bit_cast(_Float16, dh);
        }
    }
}
hipError_t launch_embed_rows(int kind, const void* table, const float* scales, const int* tokens, float* x, int T, int dim,
                             int vocab, hipStream_t s) {
    if (T <= 0) return hipSuccess;
    hipLaunchKernelGGL(embed_rows_kernel, dim3(T), dim3(PWG), 0, s, kind, table, scales, tokens, x, dim, vocab);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// Causal attention over T query rows (mongoose.cu:251-353 for a training
// sequence; here against the KV caches, query t at position pos0 + t), on the
// bf16 matrix instruction v_mfma_f32_16x16x32_bf16 with every fp32 operand
// split into two bf16 terms (x = hi + lo, |x - hi - lo| <= 2^-16 |x|) and
// three products per pair of operands (hi.hi + hi.lo + lo.hi; lo.lo is below
// 2^-16 of the result).
//
// The cache rows are split once per layer by kv_split_kernel into planes the
// matrix instruction reads as they lie: K hi / lo as [row][kvDim], and V hi /
// lo transposed, [kvh * HD + d][row], the rows of each group of 32 in the order
// the P operand holds them (below).  Rows past pos0 + T, up to the next
// multiple of 32, are written as zeros.
//
// A workgroup = 8 waves = 4 slots x 2 tile parities.  The slots are the query
// heads of one KV head (4 of them; fewer heads a KV head: the slots are shared
// out over neighbouring blocks of 16 queries instead), so all waves want the
// same K / V tiles: each step brings two 32-position tiles into LDS by direct
// global -> LDS loads (double-buffered: the next pair is requested before the
// current one is multiplied), and every wave reads its operands from there.
// A wave keeps its own running max / sum / output over the tiles of its
// parity; the two parities of a slot are combined at the end.
//
// Transposed, so that the softmax statistics of a query stay in four lanes
// (C layout of a 16 x 16 block: lane l holds column l%16, rows 4*(l/16) + e):
//   S^T[kpos][q] = K . Q^T    A = K rows (lane: row l%16, 8 d of quarter l/16 of a 32-d step), B = Q^T in registers
//   O^T[d][q]    = V^T . P^T  A = V^T rows, B = the S^T accumulators themselves: as the B operand a lane
//                             holds k slots 8*(l/16) + j, j = 0..7, and it has S^T for tile positions
//                             16*(j/4) + 4*(l/16) + j%4 -- the order V^T is stored in.
// LDS: planes of 16 rows x 64 bytes (a 32-d step of 16 K rows; 32 positions of 16 V^T rows), the 16-byte
// piece p of row r at p ^ ((r>>1)&3): the fragment reads (lane l: row l%16, piece l/16) are conflict-free.
// ---------------------------------------------------------------------------
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void split8(const float (&v)[8], bf16x8_t& h, bf16x8_t& l) {
    unsigned short hs[8], ls[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        hs[i] = f32_to_bf16_rne(v[i]);
        ls[i] = f32_to_bf16_rne(v[i] - bf16_to_f32(hs[i]));
    }
    uint4 uh, ul;
    uh.x = hs[0] | ((unsigned)hs[1] << 16); uh.y = hs[2] | ((unsigned)hs[3] << 16);
    uh.z = hs[4] | ((unsigned)hs[5] << 16); uh.w = hs[6] | ((unsigned)hs[7] << 16);
    ul.x = ls[0] | ((unsigned)ls[1] << 16); ul.y = ls[2] | ((unsigned)ls[3] << 16);
    ul.z = ls[4] | ((unsigned)ls[5] << 16); ul.w = ls[6] | ((unsigned)ls[7] << 16);
    h = __builtin_bit_cast(bf16x8_t, uh);
    l = __builtin_bit_cast(bf16x8_t, ul);
}

// grid (rowsPad / 32, nKVHeads, 2), (HD, 4) threads: thread (d, w) takes column kvh * HD + d of a quarter of the 32
// rows of K (z = 0: rows 8w .. 8w+7) or V (z = 1: the eight rows whose values make up 16-byte piece w of the column's
// transposed group)
template <typename KVT>
__global__ void kv_split_kernel(const KVT* Kc, const KVT* Vc, int rows, int kvDim, int HD, unsigned short* Khi,
                                unsigned short* Klo, unsigned short* VThi, unsigned short* VTlo, int vtStride) {
    const int g = blockIdx.x, col = blockIdx.y * HD + threadIdx.x, w = threadIdx.y;
    if (blockIdx.z == 0) {
#pragma unroll
        for (int t = 0; t < 8; t++) {
            const int r = g * 32 + 8 * w + t;
            const size_t o = (size_t)r * kvDim + col;
            const float k = r < rows ? (float)Kc[o] : 0.f;
            const unsigned short kh = f32_to_bf16_rne(k);
            Khi[o] = kh;
            Klo[o] = f32_to_bf16_rne(k - bf16_to_f32(kh));
        }
        return;
    }
    // position i of the tile sits at k slot 8 * ((i >> 2) & 3) + (i & 3) + 4 * (i >> 4): piece w holds positions
    // 4w .. 4w+3 and 16+4w .. 16+4w+3
    unsigned short vh[8], vl[8];
#pragma unroll
    for (int t = 0; t < 8; t++) {
        const int i = t < 4 ? 4 * w + t : 16 + 4 * w + (t - 4);
        const int r = g * 32 + i;
        const float v = r < rows ? (float)Vc[(size_t)r * kvDim + col] : 0.f;
        vh[t] = f32_to_bf16_rne(v);
        vl[t] = f32_to_bf16_rne(v - bf16_to_f32(vh[t]));
    }
    uint4* dh = reinterpret_cast<uint4*>(VThi + (size_t)col * vtStride + g * 32);
    uint4* dl = reinterpret_cast<uint4*>(VTlo + (size_t)col * vtStride + g * 32);
    dh[w] = make_uint4(vh[0] | ((unsigned)vh[1] << 16), vh[2] | ((unsigned)vh[3] << 16),
                       vh[4] | ((unsigned)vh[5] << 16), vh[6] | ((unsigned)vh[7] << 16));
    dl[w] = make_uint4(vl[0] | ((unsigned)vl[1] << 16), vl[2] | ((unsigned)vl[3] << 16),
                       vl[4] | ((unsigned)vl[5] << 16), vl[6] | ((unsigned)vl[7] << 16));
}

template <int HD>
__global__ __launch_bounds__(512) void prefill_attn_kernel(const float* q, const unsigned short* Khi, const unsigned short* Klo,
                                                          const unsigned short* VThi, const unsigned short* VTlo, int vtStride,
                                                          float* out, unsigned short* hi, unsigned short* lo, int T, int pos0,
                                                          int dim, int kvDim, int nHeads, int nKVHeads, int HS, int parts) {
    constexpr int NS = HD / 32;                // 32-wide steps of the head dimension
    constexpr int DB = HD / 16;                // 16-wide blocks of the head dimension
    constexpr int PL = HD * 64;                // bytes of one plane of a tile: 32 rows x HD bf16 (K), HD rows x 32 bf16 (V^T)
    constexpr int TILE_BYTES = 4 * PL;         // K hi, K lo, V^T hi, V^T lo
    constexpr int BUF_BYTES = 2 * TILE_BYTES;  // the two tiles of a step
    constexpr int OS = 17;                     // row stride (floats) of a wave's [d][16 q] partial output
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    __shared__ float wm[8][16], wl[8][16];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int slot = wave >> 1, ph = wave & 1;
    const int QB = 4 / HS;                                   // blocks of 16 queries a workgroup covers
    const int QH = nHeads / nKVHeads;
    const int kvh = blockIdx.y / parts, part = blockIdx.y % parts;
    const int hIn = part * HS + slot % HS;                   // this wave's query head within the KV head's group
    const int qblk = ((int)gridDim.x - 1 - (int)blockIdx.x) * QB + slot / HS;     // the longest causal ranges start first
    const int q0 = qblk * 16;
    const bool active = hIn < QH && q0 < T;
    const int head = kvh * QH + min(hIn, QH - 1);
    const int fr = lane & 15, fq = lane >> 4;
    const int myq = min(q0 + fr, T - 1);                    // this lane's query row (clamped rows are never stored)
    const int qpos = pos0 + myq;
    const float scale = 1.0f / sqrtf((float)HD);

    // Q^T operand: step ds holds Q[myq][32 ds + 8 fq .. + 7]
    bf16x8_t qh[NS], ql[NS];
    {
        const float* qr = q + (size_t)myq * dim + (size_t)head * HD + 8 * fq;
#pragma unroll
        for (int ds = 0; ds < NS; ds++) {
            const float4 a = *reinterpret_cast<const float4*>(qr + 32 * ds), b = *reinterpret_cast<const float4*>(qr + 32 * ds + 4);
            const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
            split8(v, qh[ds], ql[ds]);
        }
    }
    float4_t o[DB];
#pragma unroll
    for (int b = 0; b < DB; b++)
#pragma unroll
        for (int e = 0; e < 4; e++) o[b][e] = 0.f;
    float m = -INFINITY, l = 0.f;

    // the workgroup walks the tiles its furthest query sees; a wave skips the tiles past its own block's range
    const int wgLast = pos0 + min(((int)gridDim.x - 1 - (int)blockIdx.x) * QB * 16 + QB * 16 - 1, T - 1);
    const int wgTiles = wgLast / 32 + 1, nSteps = (wgTiles + 1) / 2;
    const int myLast = pos0 + min(q0 + 15, T - 1);
    const int myTiles = active ? myLast / 32 + 1 : 0;

    // loads of a step: wave w brings plane w%4 (K hi, K lo, V^T hi, V^T lo) of tile w/4: DB wave-loads of 1 KB
    const int ltile = wave >> 2, lplane = wave & 3;
    const int lr = lane >> 2, lpiece = (lane & 3) ^ ((lr >> 1) & 3);
    const unsigned short* lsrc = lplane == 0 ? Khi : lplane == 1 ? Klo : lplane == 2 ? VThi : VTlo;
    auto issue = [&](int step, int buf) __attribute__((always_inline)) {
        const int tile = min(2 * step + ltile, wgTiles - 1);
        const int t0 = tile * 32;
        unsigned char* dst = lds + buf * BUF_BYTES + ltile * TILE_BYTES + lplane * PL;
#pragma unroll
        for (int i = 0; i < DB; i++) {
            const unsigned short* src;
            if (lplane < 2) src = lsrc + (size_t)(t0 + 16 * (i & 1) + lr) * kvDim + (size_t)kvh * HD + (i >> 1) * 32 + lpiece * 8;     // plane (ds = i/2, rows 16 (i%2) ..)
            else src = lsrc + (size_t)(kvh * HD + 16 * i + lr) * vtStride + t0 + lpiece * 8;                                        // d block i
            __builtin_amdgcn_global_load_lds(src, reinterpret_cast<int4*>(dst + i * 1024), 16, 0, 0);
        }
    };
    const unsigned foff = fr * 64 + ((fq ^ ((fr >> 1) & 3)) * 16);

    issue(0, 0);
    for (int step = 0; step < nSteps; step++) {
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");     // this step's tiles have landed; the other buffer is free
        if (step + 1 < nSteps) issue(step + 1, (step + 1) & 1);
        const int tile = 2 * step + ph;
        if (tile >= myTiles) continue;
        const int t0 = tile * 32;
        const unsigned char* base = lds + (step & 1) * BUF_BYTES + ph * TILE_BYTES;
        float4_t sT[2], sX[2];                           // hi.hi and the two cross terms: two chains for the matrix pipe
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
            for (int e = 0; e < 4; e++) { sT[kb][e] = 0.f; sX[kb][e] = 0.f; }
#pragma unroll
        for (int ds = 0; ds < NS; ds++)
#pragma unroll
            for (int kb = 0; kb < 2; kb++) {
                const bf16x8_t ah = *reinterpret_cast<const bf16x8_t*>(base + (ds * 2 + kb) * 1024 + foff);
                const bf16x8_t al = *reinterpret_cast<const bf16x8_t*>(base + PL + (ds * 2 + kb) * 1024 + foff);
                sT[kb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ah, qh[ds], sT[kb], 0, 0, 0);
                sX[kb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ah, ql[ds], sX[kb], 0, 0, 0);
                sX[kb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(al, qh[ds], sX[kb], 0, 0, 0);
            }
        // causal mask, online softmax: a query's 32 scores are in the four lanes l%16 = its column
        float sv[8];
        float tmax = -INFINITY;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int kpos = t0 + 16 * (j >> 2) + 4 * fq + (j & 3);
            sv[j] = kpos <= qpos ? (sT[j >> 2][j & 3] + sX[j >> 2][j & 3]) * scale : -INFINITY;
            tmax = fmaxf(tmax, sv[j]);
        }
        tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
        const float mNew = fmaxf(m, tmax);
        const float corr = m == -INFINITY ? 0.f : expf(m - mNew);
        float psum = 0.f;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            sv[j] = sv[j] == -INFINITY ? 0.f : expf(sv[j] - mNew);
            psum += sv[j];
        }
        psum += __shfl_xor(psum, 16, 64);
        psum += __shfl_xor(psum, 32, 64);
        l = l * corr + psum;
        m = mNew;
#pragma unroll
        for (int b = 0; b < DB; b++)
#pragma unroll
            for (int e = 0; e < 4; e++) o[b][e] *= corr;
        bf16x8_t pH, pL;
        split8(sv, pH, pL);
        // O^T += V^T . P^T
#pragma unroll
        for (int b = 0; b < DB; b++) {
            const bf16x8_t vh = *reinterpret_cast<const bf16x8_t*>(base + 2 * PL + b * 1024 + foff);
            const bf16x8_t vl = *reinterpret_cast<const bf16x8_t*>(base + 3 * PL + b * 1024 + foff);
            o[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vh, pH, o[b], 0, 0, 0);
            o[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vh, pL, o[b], 0, 0, 0);
            o[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vl, pH, o[b], 0, 0, 0);
        }
    }
    // ---- combine the two parities of every slot: O^T partials through LDS, [d][q] with row stride 17 ----
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");     // every wave is done with the tiles
    float* part_ = reinterpret_cast<float*>(lds) + wave * (HD * OS);
#pragma unroll
    for (int b = 0; b < DB; b++)
#pragma unroll
        for (int e = 0; e < 4; e++) part_[(16 * b + 4 * fq + e) * OS + fr] = o[b][e];
    if (fq == 0) { wm[wave][fr] = m; wl[wave][fr] = l; }
    __syncthreads();
    for (int i = tid; i < 4 * 16 * HD; i += 512) {
        const int sl = i / (16 * HD), qq = (i / HD) % 16, d = i % HD;
        const int hI = part * HS + sl % HS, qrow = (((int)gridDim.x - 1 - (int)blockIdx.x) * QB + sl / HS) * 16 + qq;
        if (hI >= QH || qrow >= T) continue;
        const int w0 = sl * 2, w1 = sl * 2 + 1;
        const float M = fmaxf(wm[w0][qq], wm[w1][qq]);
        const float g0 = wm[w0][qq] == -INFINITY ? 0.f : expf(wm[w0][qq] - M);
        const float g1 = wm[w1][qq] == -INFINITY ? 0.f : expf(wm[w1][qq] - M);
        const float* P0 = reinterpret_cast<const float*>(lds) + w0 * (HD * OS);
        const float* P1 = reinterpret_cast<const float*>(lds) + w1 * (HD * OS);
        const float num = fmaf(g1, P1[d * OS + qq], g0 * P0[d * OS + qq]);
        const float den = fmaf(g1, wl[w1][qq], g0 * wl[w0][qq]);
        const float v = num / den;
        const int hd = (kvh * QH + hI) * HD + d;
        if (out) out[(size_t)qrow * dim + hd] = v;
        if (hi) {            // the output projection's hi/lo split, written here instead of by a pass of its own
            const unsigned short h = f32_to_bf16_rne(v);
            const size_t o2 = tiled_index(qrow, hd, dim);
            hi[o2] = h;
            lo[o2] = f32_to_bf16_rne(v - bf16_to_f32(h));
        }
    }
}

size_t prefill_kv_split_bytes(int rows, int kvDim) {
    const size_t rowsPad = ((size_t)rows + 31) / 32 * 32;
    return 4 * rowsPad * (size_t)kvDim * sizeof(unsigned short);
}

template <int HD>
static hipError_t launch_attn(dim3 grid, hipStream_t s, const float* q, const unsigned short* Khi, const unsigned short* Klo,
                              const unsigned short* VThi, const unsigned short* VTlo, int vtStride, float* out, unsigned short* hi,
                              unsigned short* lo, int T, int pos0, int dim, int kvDim, int nHeads, int nKVHeads, int HS, int parts) {
    constexpr int bytes = 2 * 2 * 4 * HD * 64;             // two buffers of two tiles of four planes (HD = 128: 128 KB)
    static_assert(8 * HD * 17 * 4 <= bytes, "the partial outputs reuse the tile buffers");
    static bool raised = false;                            // the default cap on dynamic LDS is 64 KB
    if (!raised) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&prefill_attn_kernel<HD>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
        if (e != hipSuccess) return e;
        raised = true;
    }
    hipLaunchKernelGGL((prefill_attn_kernel<HD>), grid, dim3(512), bytes, s, q, Khi, Klo, VThi, VTlo, vtStride, out, hi, lo, T, pos0,
                       dim, kvDim, nHeads, nKVHeads, HS, parts);
    return hipGetLastError();
}

hipError_t launch_prefill_attention(const float* q, const void* Kc, const void* Vc, int kvHalf, void* kvSplit, float* out,
                                    void* splitHi, void* splitLo, int T, int pos0, int rowLimit, int dim, int kvDim, int nHeads,
                                    int nKVHeads, int headDim, hipStream_t s) {
    if (T <= 0) return hipSuccess;
    if ((!out && !splitHi) || (splitHi == nullptr) != (splitLo == nullptr) || !kvSplit) return hipErrorInvalidValue;
    unsigned short* hi = static_cast<unsigned short*>(splitHi);
    unsigned short* lo = static_cast<unsigned short*>(splitLo);
    if (nKVHeads <= 0 || nHeads % nKVHeads != 0 || pos0 < 0 || pos0 + T > rowLimit || dim != nHeads * headDim ||
        kvDim != nKVHeads * headDim || (headDim != 64 && headDim != 128)) return hipErrorInvalidValue;
    const int rows = pos0 + T, rowsPad = (rows + 31) / 32 * 32;
    const size_t plane = (size_t)rowsPad * kvDim;
    unsigned short* Khi = static_cast<unsigned short*>(kvSplit);
    unsigned short *Klo = Khi + plane, *VThi = Klo + plane, *VTlo = VThi + plane;
    const dim3 sgrid((unsigned)(rowsPad / 32), (unsigned)nKVHeads, 2);
    if (kvHalf) hipLaunchKernelGGL((kv_split_kernel<_Float16>), sgrid, dim3(headDim, 4), 0, s, static_cast<const _Float16*>(Kc),
                                   static_cast<const _Float16*>(Vc), rows, kvDim, headDim, Khi, Klo, VThi, VTlo, rowsPad);
    else hipLaunchKernelGGL((kv_split_kernel<float>), sgrid, dim3(headDim, 4), 0, s, static_cast<const float*>(Kc),
                            static_cast<const float*>(Vc), rows, kvDim, headDim, Khi, Klo, VThi, VTlo, rowsPad);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    // four slots a workgroup: the query heads of a KV head, or (fewer than 3 heads a KV head) heads x neighbouring query blocks
    const int QH = nHeads / nKVHeads;
    const int HS = QH >= 3 ? 4 : QH, QB = 4 / HS, parts = (QH + HS - 1) / HS;
    const int qblocks = (T + 15) / 16;
    dim3 grid((unsigned)((qblocks + QB - 1) / QB), (unsigned)(nKVHeads * parts));
    if (headDim == 64) return launch_attn<64>(grid, s, q, Khi, Klo, VThi, VTlo, rowsPad, out, hi, lo, T, pos0, dim, kvDim, nHeads, nKVHeads, HS, parts);
    return launch_attn<128>(grid, s, q, Khi, Klo, VThi, VTlo, rowsPad, out, hi, lo, T, pos0, dim, kvDim, nHeads, nKVHeads, HS, parts);
}

// ---------------------------------------------------------------------------
// GEMM on v_mfma_f32_32x32x16_bf16, K in steps of 64; each wave owns 32-row x
// 32-column MFMA blocks and issues the hi and the lo activation term against
// the same weight fragment.  Fragment layouts (lane l):
//   A: row l%32, k = 8*(l/32)..+7        B: col l%32, k = 8*(l/32)..+7
//   C: col l%32, rows 8*(i/4) + 4*(l/32) + i%4 for i = 0..15
// Up to three weight matrices (q/k/v, gate/up) share one launch.  Workgroups
// that share a weight tile are placed on one XCD (ids congruent mod 8), so the
// tile comes into that XCD's L2 once.
// ---------------------------------------------------------------------------
constexpr int BK = 64;
constexpr int A_STRIDE = BK + 8;    // bf16 per LDS row (144 bytes)
constexpr int B_STRIDE = BK + 16;   // bytes per LDS row of int8 weights (80)

__device__ __forceinline__ unsigned pack_bf16_exact(float lo, float hi) {
    // both floats hold small integers: their low 16 bits are zero, truncation is exact
    // (one v_perm_b32: bytes 2, 3 of lo, then bytes 2, 3 of hi)
    return __builtin_amdgcn_perm(__builtin_bit_cast(unsigned, hi), __builtin_bit_cast(unsigned, lo), 0x07060302u);
}

// Workgroup tile BM x BN with NT threads: NT/64 waves as (NT/64)/(BN/64) x (BN/64), each wave
// (BM/WM) x 64.  The L2-to-CU traffic per flop falls with the tile size (A costs 4 bytes an
// element, W one), and it is that traffic which bounds the kernel: 256 x 256 tiles with 1024
// threads where the problem is large enough, 64/128 x 128 with 256 threads for short prompts.
// MODE 0: Y = acc*scale (+bias)   1: Y += acc*scale   2: raw partial sums of one K split into p.partial
//
// Q4 = 1 reads Q4_0 weights in the split layout (16-byte nibble groups [N, K/32], then fp16 d
// [N, K/32]).  nibble - 8 is exact in bf16; the block scale cannot be folded into a bf16 weight
// without loss, so each 32-k block is multiplied into a scratch accumulator (two MFMA steps, hi and
// lo) and added to the running sums as d * scratch: 16 FMAs per MFMA block and Q4_0 block.  Element
// order in a block (GGML): low nibble of byte j = element j, high nibble = element j + 16, so the 8
// consecutive elements a fragment needs are the low or the high nibbles of 8 consecutive bytes.
template <int Q4, int BM, int BN, int NT, int MODE>
__global__ __launch_bounds__(NT) void gemm_q8_bf16x2_kernel(GemmParams p) {
    constexpr int WN = BN / 64, WM = (NT / 64) / WN;
    constexpr int MI = BM / WM / 32;             // 32-row MFMA blocks per wave
    constexpr int AR = BM * 8 / NT;              // 16-byte segments per thread and A plane
    constexpr int WSEG = Q4 ? 2 : 4;             // 16-byte segments of W per row and K step
    constexpr int BR = BN * WSEG / NT > 0 ? BN * WSEG / NT : 1;
    constexpr int WSTRIDE = Q4 ? 48 : B_STRIDE;  // bytes per LDS row of W
    static_assert(MI >= 1 && AR >= 1, "tile too small for the thread count");
    static_assert(BN * WSEG % NT == 0 || BN * WSEG < NT, "W segments do not divide over the threads");
    __shared__ __attribute__((aligned(16))) unsigned short sAh[BM * A_STRIDE];
    __shared__ __attribute__((aligned(16))) unsigned short sAl[BM * A_STRIDE];
    __shared__ __attribute__((aligned(16))) signed char sB[BN * WSTRIDE];
    __shared__ float sD[Q4 ? BN * 2 : 1];         // Q4_0: the step's two block scales of every row

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int numM = (p.T + BM - 1) / BM;
    const int L = blockIdx.x;
    const int grp = L / (8 * numM), rem = L % (8 * numM);
    const int nTile = grp * 8 + (rem & 7), mTile = rem >> 3;
    if (nTile >= p.nTiles) return;
    int sgi = 0;
    if (MODE != 3) {
        if (p.nseg > 1 && nTile >= p.seg[1].tile0) sgi = 1;
        if (p.nseg > 2 && nTile >= p.seg[2].tile0) sgi = 2;
    }
    GemmSeg sg = p.seg[0];                       // selected by value: indexing the argument array by a
    if (sgi == 1) sg = p.seg[1];                 // run-time index would copy it into scratch memory
    if (sgi == 2) sg = p.seg[2];
    const int N = sg.N, K = p.K, T = p.T;
    // MODE 3 (gate | up -> silu(gate) * up): a tile is BN/2 columns of the output; its BN weight rows
    // alternate in blocks of 32 between the gate and the up matrix, so a wave's two 32-column MFMA
    // blocks are the gate and the up values of the same 32 columns.
    const int m0 = mTile * BM, n0 = MODE == 3 ? nTile * (BN / 2) : (nTile - sg.tile0) * BN;
    // weight row (and matrix) behind local row lr of the tile
    auto wrow = [&](int lr) { return MODE == 3 ? n0 + (lr >> 6) * 32 + (lr & 31) : n0 + lr; };
    auto wmat = [&](int lr) { return MODE == 3 && ((lr >> 5) & 1) ? p.seg[1].W : sg.W; };
    const int ksteps = (K + BK - 1) / BK;
    const int stepBeg = MODE == 2 ? blockIdx.y * p.stepsPerSplit : 0;
    const int stepEnd = MODE == 2 ? min(ksteps, stepBeg + p.stepsPerSplit) : ksteps;

    // global -> LDS: A row = tid/8 (+NT/8 per pass), segment tid%8 (8 bf16) ; W row = tid/4 (+NT/4), segment tid%4 (16 int8)
    const int aRow = tid >> 3, aSeg = tid & 7;
    const int bRow = Q4 ? tid >> 1 : tid >> 2, bSeg = Q4 ? tid & 1 : tid & 3;
    const bool bActive = bRow < BN;                  // Q4_0 with more threads than segments: the rest only load A
    const unsigned short* aHiP[AR]; const unsigned short* aLoP[AR];
    const int planeRows = ((T + 127) >> 7) << 7;     // the planes are padded to whole 128-row blocks, not to BM
#pragma unroll
    for (int r = 0; r < AR; r++) {         // rows in [T, planeRows) exist in the planes; their results are dropped
        const int row = min(m0 + aRow + (NT / 8) * r, planeRows - 1);
        const size_t o = (size_t)(row >> 7) * ksteps * 8192 + (size_t)(row & 127) * 64 + aSeg * 8;
        aHiP[r] = p.Ahi + o;
        aLoP[r] = p.Alo + o;
    }
    const signed char* bP[BR];
#pragma unroll
    for (int r = 0; r < BR; r++) {
        const int lr = bRow + (NT / WSEG) * r;
        const int row = min(wrow(lr), N - 1);
        const signed char* Wm = wmat(lr);
        bP[r] = Q4 ? Wm + ((size_t)row * (K >> 5) + bSeg) * 16 : Wm + (size_t)row * K + bSeg * 16;
    }
    // Q4_0: thread t < BN also fetches row t's two block scales of the step
    const unsigned short* dP = nullptr;
    if (Q4 && tid < BN)
        dP = reinterpret_cast<const unsigned short*>(wmat(tid) + (size_t)N * (K >> 1)) + (size_t)min(wrow(tid), N - 1) * (K >> 5);

    float16_t acc[MI][2];
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.f;

    int4 gAh[AR], gAl[AR], gB[BR];
    unsigned short gD[2] = {0, 0};
    // K is a multiple of 32: a last half step reads zeros past the end.  The load itself is never
    // conditional (`ok ? *p : zero` made the compiler select between p and the address of a private
    // zero, i.e. a flat load that is waited for at once and staged through scratch memory): a
    // segment past the end re-reads the step's first segment and is zeroed afterwards.
    // (A macro rather than a lambda: with the staging arrays captured by reference the compiler kept
    // them in scratch memory in some instantiations.)
#define MG_GEMM_GLOAD(K0)                                                                                   \
    do {                                                                                                    \
        const int k0_ = (K0);                                                                               \
        const bool okA_ = k0_ + aSeg * 8 < K;                                                               \
        const bool okB_ = bActive && (Q4 ? k0_ + bSeg * 32 < K : k0_ + bSeg * 16 < K);                      \
        const int aBack_ = okA_ ? 0 : aSeg * 8;      /* elements back to segment 0 of the step */           \
        const int bBack_ = okB_ ? 0 : bSeg * 16;     /* bytes back to segment 0 of the step */              \
        _Pragma("unroll") for (int r = 0; r < AR; r++) {                                                    \
            gAh[r] = *reinterpret_cast<const int4*>(aHiP[r] + (size_t)k0_ * 128 - aBack_);                  \
            gAl[r] = *reinterpret_cast<const int4*>(aLoP[r] + (size_t)k0_ * 128 - aBack_);                  \
            if (!okA_) { gAh[r] = make_int4(0, 0, 0, 0); gAl[r] = make_int4(0, 0, 0, 0); }                  \
        }                                                                                                   \
        _Pragma("unroll") for (int r = 0; r < BR; r++) {                                                    \
            gB[r] = *reinterpret_cast<const int4*>(bP[r] + (Q4 ? k0_ >> 1 : k0_) - bBack_);                 \
            if (!okB_) gB[r] = make_int4(0, 0, 0, 0);                                                       \
        }                                                                                                   \
        if (Q4 && dP) {                                                                                     \
            gD[0] = dP[k0_ >> 5];                                                                           \
            gD[1] = k0_ + 32 < K ? dP[(k0_ >> 5) + 1] : (unsigned short)0;                                  \
        }                                                                                                   \
    } while (0)
    if (stepBeg < stepEnd) MG_GEMM_GLOAD(stepBeg * BK);
    for (int step = stepBeg; step < stepEnd; step++) {
        __syncthreads();                       // the previous step's fragments are consumed
#pragma unroll
        for (int r = 0; r < AR; r++) {
            *reinterpret_cast<int4*>(&sAh[(aRow + (NT / 8) * r) * A_STRIDE + aSeg * 8]) = gAh[r];
            *reinterpret_cast<int4*>(&sAl[(aRow + (NT / 8) * r) * A_STRIDE + aSeg * 8]) = gAl[r];
        }
#pragma unroll
        for (int r = 0; r < BR; r++)
            if (bActive) *reinterpret_cast<int4*>(&sB[(bRow + (NT / WSEG) * r) * WSTRIDE + bSeg * 16]) = gB[r];
        if (Q4 && tid < BN) {
            sD[tid * 2] = (float)__builtin_bit_cast(_Float16, gD[0]);
            sD[tid * 2 + 1] = (float)__builtin_bit_cast(_Float16, gD[1]);
        }
        __syncthreads();
        if (step + 1 < stepEnd) MG_GEMM_GLOAD((step + 1) * BK);       // next tile in flight while this one is multiplied
        if (Q4) {
            float16_t zero16;
#pragma unroll
            for (int e = 0; e < 16; e++) zero16[e] = 0.f;
#pragma unroll
            for (int bl = 0; bl < 2; bl++) {               // the step's two Q4_0 blocks
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    const int nrow = wn * 64 + j * 32 + (lane & 31);
                    const float d = sD[nrow * 2 + bl];
                    // this lane's 8 elements of each 16-k half: e = 16*h2 + 8*(lane/32) -> bytes (e & 8).., nibble e >= 16
                    bf16x8_t b[2];
#pragma unroll
                    for (int h2 = 0; h2 < 2; h2++) {
                        const int e0 = 16 * h2 + 8 * (lane >> 5);
                        const int2 w = *reinterpret_cast<const int2*>(&sB[nrow * WSTRIDE + bl * 16 + (e0 & 8)]);
                        const unsigned sh = h2 ? 4u : 0u;   // elements 16..31 are the high nibbles
                        const unsigned n0v = ((unsigned)w.x >> sh) & 0x0f0f0f0fu, n1v = ((unsigned)w.y >> sh) & 0x0f0f0f0fu;
                        uint4 u;
                        u.x = pack_bf16_exact((float)(n0v & 0xff) - 8.0f, (float)((n0v >> 8) & 0xff) - 8.0f);
                        u.y = pack_bf16_exact((float)((n0v >> 16) & 0xff) - 8.0f, (float)(n0v >> 24) - 8.0f);
                        u.z = pack_bf16_exact((float)(n1v & 0xff) - 8.0f, (float)((n1v >> 8) & 0xff) - 8.0f);
                        u.w = pack_bf16_exact((float)((n1v >> 16) & 0xff) - 8.0f, (float)(n1v >> 24) - 8.0f);
                        b[h2] = __builtin_bit_cast(bf16x8_t, u);
                    }
#pragma unroll
                    for (int i = 0; i < MI; i++) {
                        float16_t t = zero16;
#pragma unroll
                        for (int h2 = 0; h2 < 2; h2++) {
                            const int arow = (wm * (BM / WM) + i * 32 + (lane & 31)) * A_STRIDE + bl * 32 + h2 * 16 + 8 * (lane >> 5);
                            bf16x8_t ah = *reinterpret_cast<const bf16x8_t*>(&sAh[arow]);
                            bf16x8_t al = *reinterpret_cast<const bf16x8_t*>(&sAl[arow]);
                            t = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, b[h2], t, 0, 0, 0);
                            t = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al, b[h2], t, 0, 0, 0);
                        }
#pragma unroll
                        for (int e = 0; e < 16; e++) acc[i][j][e] = fmaf(d, t[e], acc[i][j][e]);
                    }
                }
            }
        } else {
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
                const int arow = (wm * (BM / WM) + i * 32 + (lane & 31)) * A_STRIDE + kk;
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
    }
    if (MODE == 3) {
        const int n = n0 + wn * 32 + (lane & 31);
        if (n < N) {
            const float scg = Q4 ? 1.0f : p.seg[0].scales[n], scu = Q4 ? 1.0f : p.seg[1].scales[n];
            const float big = p.seg[0].bias ? p.seg[0].bias[n] : 0.f, biu = p.seg[1].bias ? p.seg[1].bias[n] : 0.f;
#pragma unroll
            for (int i = 0; i < MI; i++)
#pragma unroll
                for (int e = 0; e < 16; e++) {
                    const int m = m0 + wm * (BM / WM) + i * 32 + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
                    if (m < T) {
                        const float g = acc[i][0][e] * scg + big, u = acc[i][1][e] * scu + biu;
                        const float a = g * (1.0f / (1.0f + expf(-g))) * u;        // mongoose.cu:949-956
                        const unsigned short h = f32_to_bf16_rne(a);
                        const size_t o = tiled_index(m, n, N);
                        p.nextHi[o] = h;
                        p.nextLo[o] = f32_to_bf16_rne(a - bf16_to_f32(h));
                    }
                }
        }
        return;
    }
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int nl = wn * 64 + j * 32 + (lane & 31);
        const int n = n0 + nl;
        if (MODE == 2) {
            // partial[split][m][column in the concatenated, tile-padded column space]
            float* dst = p.partial + ((size_t)blockIdx.y * T) * p.ldPartial + (size_t)nTile * BN + nl;
#pragma unroll
            for (int i = 0; i < MI; i++)
#pragma unroll
                for (int e = 0; e < 16; e++) {
                    const int m = m0 + wm * (BM / WM) + i * 32 + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
                    if (m < T) dst[(size_t)m * p.ldPartial] = acc[i][j][e];
                }
        } else if (n < N) {      // no `continue` in this loop: it must unroll, or acc is indexed at run time (scratch)
            const float sc = Q4 ? 1.0f : sg.scales[n];
            const float bi = sg.bias ? sg.bias[n] : 0.f;
#pragma unroll
            for (int i = 0; i < MI; i++) {
#pragma unroll
                for (int e = 0; e < 16; e++) {
                    const int m = m0 + wm * (BM / WM) + i * 32 + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
                    if (m < T) {
                        float v = acc[i][j][e] * sc + bi;
                        float* dst = sg.Y + (size_t)m * N + n;
                        if (MODE == 1) v = *dst + v;
                        *dst = v;
                    }
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------
// The large Q8 tile: 256 x 256, 512 threads (4 x 2 waves of 64 rows x 128
// columns), v_mfma_f32_16x16x32_bf16, a three-stage LDS ring with K steps of 32
// and one barrier per step.  Measured on the gate|up shape (512 x 28672 x 4096):
// the matrix pipe and ordinary vector instructions of a SIMD do not overlap
// here (busy cycles add up), so the loop carries as few of the latter as it
// can, and under this load the chip clocks near 1.8 GHz, where the 16x16x32
// form sustains 2.2 PFLOP/s on random operands against 1.84 for 32x32x16.
//
// * The activation planes (A hi, A lo: 16 KB a stage each) come by direct global -> LDS loads
//   (global_load_lds_dwordx4: no registers, no LDS store instructions), issued two steps ahead.  A wave's load
//   lands as 1 KB of consecutive 16-byte slots, so the layout is made on the global side: slot s of a
//   load holds row r = first + s/4 and piece (s%4) ^ ((r>>1)&3) of the row's 64 bytes.
// * The weights come through registers, 16 int8 a thread and step, requested five steps ahead (their
//   rows come from HBM, the activations from L2), and are converted to bf16 once per workgroup --
//   not once per wave that multiplies them -- into the stage's third plane, same layout.
// * A fragment read is ds_read_b128 with lane l at row l%16, piece l/16: with the XOR by (row>>1)&3
//   it is served without bank conflicts (4 cycles an instruction; (row>>2)&3 or none: 8).
// * s_waitcnt / s_barrier are written out: the compiler's __syncthreads() waits for every outstanding
//   load, including the ones issued for later steps.  Loads complete in order, five are issued per
//   step (A x 4, W), so "at most five outstanding" at the top of step s means A(s) and W(s+1) landed.
// The K steps of a workgroup must be a multiple of 4 (the register ring is unrolled by hand).
// ---------------------------------------------------------------------------
constexpr int RK = 32, RS = 3;
constexpr int RING_PLANE = 256 * 64;                      // 256 rows x 32 bf16
constexpr int RING_STAGE_BYTES = 3 * RING_PLANE;          // A hi, A lo, W as bf16

// the 32-bit LDS address of a pointer into __shared__ memory
__device__ __forceinline__ unsigned lds_offset(const void* p) {
    return (unsigned)(size_t)(__attribute__((address_space(3))) const void*)p;
}

__device__ __forceinline__ bf16x8_t cvt8_i8_bf16(int lo, int hi) {
    uint4 u;
    u.x = pack_bf16_exact((float)(signed char)(lo), (float)(signed char)(lo >> 8));
    u.y = pack_bf16_exact((float)(signed char)(lo >> 16), (float)(lo >> 24));
    u.z = pack_bf16_exact((float)(signed char)(hi), (float)(signed char)(hi >> 8));
    u.w = pack_bf16_exact((float)(signed char)(hi >> 16), (float)(hi >> 24));
    return __builtin_bit_cast(bf16x8_t, u);
}

template <int MODE>
__global__ __launch_bounds__(512) void gemm_q8_ring_kernel(GemmParams p) {
    constexpr int BM = 256, BN = 256;
    extern __shared__ __attribute__((aligned(16))) unsigned char ring[];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;             // 4 x 2 waves, each 64 rows x 128 columns
    const int numM = (p.T + BM - 1) / BM;
    const int L = blockIdx.x;
    const int grp = L / (8 * numM), rem = L % (8 * numM);
    const int nTile = grp * 8 + (rem & 7), mTile = rem >> 3;
    if (nTile >= p.nTiles) return;
    GemmSeg sg = p.seg[0];
    if (MODE != 3) {
        if (p.nseg > 1 && nTile >= p.seg[1].tile0) sg = p.seg[1];
        if (p.nseg > 2 && nTile >= p.seg[2].tile0) sg = p.seg[2];
    }
    const int N = sg.N, K = p.K, T = p.T;
    // MODE 3 (gate | up -> silu(gate) * up): a tile is 128 columns of the output; its 256 weight rows
    // alternate in blocks of 32 between the gate and the up matrix, so a wave holds the gate and the
    // up values of the same columns (blocks j and j + 2) and the product needs no exchange.
    const int m0 = mTile * BM, n0 = MODE == 3 ? nTile * 128 : (nTile - sg.tile0) * BN;
    const int ksteps = K / RK;
    const int ks64 = (K + 63) / 64;                       // the split planes are blocked in 64-k steps
    const int stepBeg = MODE == 2 ? blockIdx.y * p.stepsPerSplit * 2 : 0;
    const int stepEnd = MODE == 2 ? min(ksteps, stepBeg + p.stepsPerSplit * 2) : ksteps;
    const int planeRows = ((T + 127) >> 7) << 7;

    // A: the wave's two loads per plane cover rows 32 wave + 16 u + lane/4, u = 0, 1
    unsigned aOff[2];                                     // in elements of a plane (< 2^32)
#pragma unroll
    for (int u = 0; u < 2; u++) {
        const int rl = 32 * wave + 16 * u + (lane >> 2);
        const int seg = (lane & 3) ^ ((rl >> 1) & 3);
        const int rg = min(m0 + rl, planeRows - 1);
        aOff[u] = (unsigned)(rg >> 7) * (unsigned)ks64 * 8192u + (unsigned)(rg & 127) * 64u + (unsigned)seg * 8u;
    }
    // W: thread t -> tile row t/2, 16 weights (t%2)*16 .. +15 of the step = pieces 2 (t%2) and 2 (t%2) + 1 of the row
    const int bRowL = tid >> 1, bQ = (tid & 1) * 2;
    const signed char* bG;
    if (MODE == 3) {
        const int blk = bRowL >> 5;
        const int wrow = min(n0 + (blk >> 1) * 32 + (bRowL & 31), N - 1);
        bG = ((blk & 1) ? p.seg[1].W : p.seg[0].W) + (size_t)wrow * K + bQ * 8;
    } else {
        bG = sg.W + (size_t)min(n0 + bRowL, N - 1) * K + bQ * 8;
    }
    const unsigned bDst0 = 2 * RING_PLANE + bRowL * 64 + ((bQ ^ ((bRowL >> 1) & 3)) * 16);
    const unsigned bDst1 = 2 * RING_PLANE + bRowL * 64 + (((bQ + 1) ^ ((bRowL >> 1) & 3)) * 16);
    const int fr = lane & 15, fq = lane >> 4;
    const unsigned offA = (wm * 64 + fr) * 64 + ((fq ^ ((fr >> 1) & 3)) * 16);
    const unsigned offW = 2 * RING_PLANE + (wn * 128 + fr) * 64 + ((fq ^ ((fr >> 1) & 3)) * 16);

    auto issueA = [&](int step, int stage) __attribute__((always_inline)) {
        const int st = min(step, ksteps - 1);            // past the end: a harmless reload that keeps the counters uniform
        unsigned char* base = ring + stage * RING_STAGE_BYTES + wave * 2048;
        const size_t ko = (size_t)(st >> 1) * 8192 + (st & 1) * 32;
        if constexpr (MODE == 3) {
            // A uniform base in scalar registers and a 32-bit byte offset a lane that never changes: written out, because the
            // compiler's own form of this load adds the two in vector registers for every load (the matrix pipe and the other
            // vector instructions of a SIMD do not overlap, so those additions came out of the multiplications' time).  M0
            // carries the LDS address of the wave's first slot.
            const unsigned short* ah = p.Ahi + ko;
            const unsigned short* al = p.Alo + ko;
            const unsigned l0 = lds_offset(base);
            asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(l0), "v"(aOff[0] * 2u), "s"(ah));
            asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(l0 + 1024u), "v"(aOff[1] * 2u), "s"(ah));
            asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(l0 + (unsigned)RING_PLANE), "v"(aOff[0] * 2u), "s"(al));
            asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(l0 + (unsigned)RING_PLANE + 1024u), "v"(aOff[1] * 2u), "s"(al));
        } else {
            // (K split or short launches: the compiler's form of the same loads schedules better there -- measured)
            __builtin_amdgcn_global_load_lds(p.Ahi + aOff[0] + ko, reinterpret_cast<int4*>(base), 16, 0, 0);
            __builtin_amdgcn_global_load_lds(p.Ahi + aOff[1] + ko, reinterpret_cast<int4*>(base + 1024), 16, 0, 0);
            __builtin_amdgcn_global_load_lds(p.Alo + aOff[0] + ko, reinterpret_cast<int4*>(base + RING_PLANE), 16, 0, 0);
            __builtin_amdgcn_global_load_lds(p.Alo + aOff[1] + ko, reinterpret_cast<int4*>(base + RING_PLANE + 1024), 16, 0, 0);
        }
    };
    auto loadW = [&](int step) __attribute__((always_inline)) {
        return *reinterpret_cast<const int4*>(bG + (size_t)min(step, ksteps - 1) * RK);
    };
    auto putW = [&](int4 w, int stage) __attribute__((always_inline)) {
        *reinterpret_cast<bf16x8_t*>(ring + stage * RING_STAGE_BYTES + bDst0) = cvt8_i8_bf16(w.x, w.y);
        *reinterpret_cast<bf16x8_t*>(ring + stage * RING_STAGE_BYTES + bDst1) = cvt8_i8_bf16(w.z, w.w);
    };

    float4_t acc[4][8];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 8; j++)
#pragma unroll
            for (int e = 0; e < 4; e++) acc[i][j][e] = 0.f;

    auto multiply = [&](int stage) __attribute__((always_inline)) {
        const unsigned char* base = ring + stage * RING_STAGE_BYTES;
        bf16x8_t b[8];
#pragma unroll
        for (int j = 0; j < 8; j++) b[j] = *reinterpret_cast<const bf16x8_t*>(base + offW + j * 1024);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const bf16x8_t ah = *reinterpret_cast<const bf16x8_t*>(base + offA + i * 1024);
            const bf16x8_t al = *reinterpret_cast<const bf16x8_t*>(base + RING_PLANE + offA + i * 1024);
#pragma unroll
            for (int j = 0; j < 8; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ah, b[j], acc[i][j], 0, 0, 0);
#pragma unroll
            for (int j = 0; j < 8; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(al, b[j], acc[i][j], 0, 0, 0);
        }
    };

    // W of the first four steps into the register ring, the first converted at once
    int4 w0 = loadW(stepBeg), w1 = loadW(stepBeg + 1), w2 = loadW(stepBeg + 2), w3 = loadW(stepBeg + 3);
    asm volatile("s_waitcnt vmcnt(3)" ::: "memory");
    putW(w0, 0);
    issueA(stepBeg, 0);
    w0 = loadW(stepBeg + 4);
    issueA(stepBeg + 1, 1);
    int stage = 0;
    // step s: A(s) and W(s+1) have landed; barrier; W(s+1) -> stage s+1; request W(s+5) and A(s+2); multiply stage s
#define MG_RING_STEP(WS, S)                                                                          \
    {                                                                                                \
        asm volatile("s_waitcnt vmcnt(5) lgkmcnt(0)\n\ts_barrier" ::: "memory");                     \
        const int s1 = stage + 1 == RS ? 0 : stage + 1;                                              \
        const int s2 = s1 + 1 == RS ? 0 : s1 + 1;                                                    \
        putW(WS, s1);                                                                                \
        WS = loadW((S) + 5);                                                                         \
        issueA((S) + 2, s2);                                                                         \
        multiply(stage);                                                                             \
        stage = s1;                                                                                  \
    }
    for (int step = stepBeg; step < stepEnd; step += 4) {
        MG_RING_STEP(w1, step)
        MG_RING_STEP(w2, step + 1)
        MG_RING_STEP(w3, step + 2)
        MG_RING_STEP(w0, step + 3)
    }
#undef MG_RING_STEP
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");     // the trailing reloads must not outlive the workgroup's LDS

    // C layout of the 16 x 16 blocks: lane l holds column l%16, rows 4*(l/16) + e
    const int mrow = m0 + wm * 64 + 4 * (lane >> 4);
    if (MODE == 3 && n0 + 128 <= N) {
        // A whole tile of columns: the 256 x 128 results are the four 128-row x 64-k blocks (rb, kb) of each split plane,
        // 16 KB of consecutive addresses each.  They are gathered in the ring's LDS in that order (the 32-byte pair of
        // pieces of a row XOR-ed with row bits, so that the four row groups of a wave's store fall into different banks)
        // and leave as whole rows of 128 bytes, 16 bytes a lane -- not as 2-byte stores to four rows an instruction.
        __syncthreads();                                  // every wave is through with the last stage
#pragma unroll
        for (int jj = 0; jj < 4; jj++) {
            const int jg = (jj >> 1) * 4 + (jj & 1);      // gate blocks 0, 1, 4, 5; the up values of the same columns in jg + 2
            const int c = (wn * 2 + (jj >> 1)) * 32 + (jj & 1) * 16 + (lane & 15);
            const int n = n0 + c;
            const float scg = p.seg[0].scales[n], scu = p.seg[1].scales[n];
            const float big = p.seg[0].bias ? p.seg[0].bias[n] : 0.f, biu = p.seg[1].bias ? p.seg[1].bias[n] : 0.f;
            const int kb = c >> 6, pc = (c & 63) >> 3;    // 64-k block of the column, its 16-byte piece there
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int r = wm * 64 + i * 16 + 4 * (lane >> 4) + e;          // row of the tile
                    const float g = acc[i][jg][e] * scg + big, u = acc[i][jg + 2][e] * scu + biu;
                    const float a = g * (1.0f / (1.0f + expf(-g))) * u;            // mongoose.cu:949-956
                    const unsigned short h = f32_to_bf16_rne(a);
                    const int rl = r & 127;
                    const unsigned o = ((r >> 7) * 2 + kb) * 16384 + rl * 128 + ((((pc >> 1) ^ ((rl >> 2) & 3)) << 1) | (pc & 1)) * 16 + (c & 7) * 2;
                    *reinterpret_cast<unsigned short*>(ring + o) = h;
                    *reinterpret_cast<unsigned short*>(ring + 65536 + o) = f32_to_bf16_rne(a - bf16_to_f32(h));
                }
        }
        __syncthreads();
        const int ksN = (N + 63) >> 6;
#pragma unroll
        for (int q = 0; q < 16; q++) {
            const int ch = q * 512 + tid;                 // 16-byte chunk: plane, block, row, piece
            const int plane = ch >> 12, blk = (ch >> 10) & 3, off = ch & 1023;
            const int rl = off >> 3, pc = off & 7;
            const int rbG = (m0 >> 7) + (blk >> 1);
            if (rbG * 128 >= planeRows) continue;         // (uniform in the wave: a chunk row is 8 lanes)
            const uint4 v = *reinterpret_cast<const uint4*>(ring + plane * 65536 + blk * 16384 + rl * 128 +
                                                            ((((pc >> 1) ^ ((rl >> 2) & 3)) << 1) | (pc & 1)) * 16);
            unsigned short* dst = (plane ? p.nextLo : p.nextHi) + ((size_t)rbG * ksN + (n0 >> 6) + (blk & 1)) * 8192 + (size_t)off * 8;
            *reinterpret_cast<uint4*>(dst) = v;
        }
        return;
    }
    if (MODE == 3) {
#pragma unroll
        for (int jj = 0; jj < 4; jj++) {
            const int jg = (jj >> 1) * 4 + (jj & 1);      // gate blocks 0, 1, 4, 5; the up values of the same columns in jg + 2
            const int n = n0 + (wn * 2 + (jj >> 1)) * 32 + (jj & 1) * 16 + (lane & 15);
            if (n >= N) continue;
            const float scg = p.seg[0].scales[n], scu = p.seg[1].scales[n];
            const float big = p.seg[0].bias ? p.seg[0].bias[n] : 0.f, biu = p.seg[1].bias ? p.seg[1].bias[n] : 0.f;
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int m = mrow + i * 16 + e;
                    if (m < T) {
                        const float g = acc[i][jg][e] * scg + big, u = acc[i][jg + 2][e] * scu + biu;
                        const float a = g * (1.0f / (1.0f + expf(-g))) * u;        // mongoose.cu:949-956
                        const unsigned short h = f32_to_bf16_rne(a);
                        const size_t o = tiled_index(m, n, N);
                        p.nextHi[o] = h;
                        p.nextLo[o] = f32_to_bf16_rne(a - bf16_to_f32(h));
                    }
                }
        }
        return;
    }
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const int nl = wn * 128 + j * 16 + (lane & 15);
        const int n = n0 + nl;
        if (MODE == 2) {
            float* dst = p.partial + ((size_t)blockIdx.y * T) * p.ldPartial + (size_t)nTile * BN + nl;
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int m = mrow + i * 16 + e;
                    if (m < T) dst[(size_t)m * p.ldPartial] = acc[i][j][e];
                }
            continue;
        }
        if (n >= N) continue;
        const float sc = sg.scales[n];
        const float bi = sg.bias ? sg.bias[n] : 0.f;
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int m = mrow + i * 16 + e;
                if (m < T) {
                    float v = acc[i][j][e] * sc + bi;
                    float* dst = sg.Y + (size_t)m * N + n;
                    if (MODE == 1) v = *dst + v;
                    *dst = v;
                }
            }
    }
}

template <int MODE>
static hipError_t launch_ring(const GemmParams& p, dim3 grid, hipStream_t s) {
    constexpr int bytes = RS * RING_STAGE_BYTES;          // 144 KB of the CU's 160 KB
    static bool raised = false;                            // the default cap on dynamic LDS is 64 KB
    if (!raised) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_q8_ring_kernel<MODE>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
        if (e != hipSuccess) return e;
        raised = true;
    }
    hipLaunchKernelGGL((gemm_q8_ring_kernel<MODE>), grid, dim3(512), bytes, s, p);
    return hipGetLastError();
}

// Sum of the K splits in split order (so the result does not depend on which workgroup
// finished first), then scale, bias and the optional residual.
__global__ __launch_bounds__(PWG) void gemm_reduce_kernel(GemmParams p, int BN, int residual) {
    const int c = blockIdx.x * PWG + threadIdx.x;      // column in the padded column space
    const int m = blockIdx.y;
    if (c >= p.ldPartial) return;
    const int tile = c / BN;
    int sgi = 0;
    if (p.nseg > 1 && tile >= p.seg[1].tile0) sgi = 1;
    if (p.nseg > 2 && tile >= p.seg[2].tile0) sgi = 2;
    GemmSeg sg = p.seg[0];
    if (sgi == 1) sg = p.seg[1];
    if (sgi == 2) sg = p.seg[2];
    const int n = c - sg.tile0 * BN;
    if (n >= sg.N) return;
    const float* src = p.partial + (size_t)m * p.ldPartial + c;
    float v = 0.f;
    for (int s = 0; s < p.splitK; s++) v += src[(size_t)s * p.T * p.ldPartial];
    v = v * (sg.scales ? sg.scales[n] : 1.0f) + (sg.bias ? sg.bias[n] : 0.f);
    float* dst = sg.Y + (size_t)m * sg.N + n;
    if (residual) v = *dst + v;
    *dst = v;
}

// The same for one matrix in residual form, one workgroup per row, with the row kept in registers:
// x = Y + scale * (sum of the splits) + bias is stored, and the next projection's (RMSNorm +) hi/lo
// split of x is written straight away (split_rows_kernel's arithmetic, term by term).  N <= 16384.
__global__ __launch_bounds__(PWG) void gemm_reduce_norm_split_kernel(GemmParams p) {
    constexpr int MAXV = 16;                            // float4 per thread
    __shared__ float red[4];
    const int m = blockIdx.x;
    const GemmSeg sg = p.seg[0];
    const int N = sg.N;
    const size_t plane = (size_t)p.T * p.ldPartial;
    const float4* src = reinterpret_cast<const float4*>(p.partial + (size_t)m * p.ldPartial);
    float4* y4 = reinterpret_cast<float4*>(sg.Y + (size_t)m * N);
    float4 x[MAXV];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < MAXV; i++) {
        const int c4 = threadIdx.x + i * PWG;
        if (c4 * 4 >= N) continue;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        int s = 0;
        for (; s + 4 <= p.splitK; s += 4) {             // four loads in flight, added in split order
            const float4 a = src[(size_t)s * plane / 4 + c4], b = src[(size_t)(s + 1) * plane / 4 + c4];
            const float4 c = src[(size_t)(s + 2) * plane / 4 + c4], d = src[(size_t)(s + 3) * plane / 4 + c4];
            v.x += a.x; v.y += a.y; v.z += a.z; v.w += a.w;
            v.x += b.x; v.y += b.y; v.z += b.z; v.w += b.w;
            v.x += c.x; v.y += c.y; v.z += c.z; v.w += c.w;
            v.x += d.x; v.y += d.y; v.z += d.z; v.w += d.w;
        }
        for (; s < p.splitK; s++) {
            const float4 a = src[(size_t)s * plane / 4 + c4];
            v.x += a.x; v.y += a.y; v.z += a.z; v.w += a.w;
        }
        float4 sc = make_float4(1.f, 1.f, 1.f, 1.f), bi = make_float4(0.f, 0.f, 0.f, 0.f);
        if (sg.scales) sc = reinterpret_cast<const float4*>(sg.scales)[c4];
        if (sg.bias) bi = reinterpret_cast<const float4*>(sg.bias)[c4];
        const float4 r = y4[c4];
        v.x = r.x + (v.x * sc.x + bi.x); v.y = r.y + (v.y * sc.y + bi.y);
        v.z = r.z + (v.z * sc.z + bi.z); v.w = r.w + (v.w * sc.w + bi.w);
        y4[c4] = v;
        x[i] = v;
        ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
    }
    float rs = 1.0f;
    if (p.nextGain) rs = 1.0f / sqrtf(block_sum256(ss, red) / (float)N + p.nextEps);
#pragma unroll
    for (int i = 0; i < MAXV; i++) {
        const int c4 = threadIdx.x + i * PWG;
        if (c4 * 4 >= N) continue;
        float a[4] = {x[i].x, x[i].y, x[i].z, x[i].w};
        if (p.nextGain) {
            const float4 g = reinterpret_cast<const float4*>(p.nextGain)[c4];
            a[0] = a[0] * rs * g.x; a[1] = a[1] * rs * g.y; a[2] = a[2] * rs * g.z; a[3] = a[3] * rs * g.w;
        }
        unsigned short h[4], l[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            h[e] = f32_to_bf16_rne(a[e]);
            l[e] = f32_to_bf16_rne(a[e] - bf16_to_f32(h[e]));
        }
        const size_t o = tiled_index(m, c4 * 4, N);      // four consecutive k stay inside one 64-k block
        *reinterpret_cast<uint2*>(p.nextHi + o) = make_uint2((unsigned)h[0] | ((unsigned)h[1] << 16), (unsigned)h[2] | ((unsigned)h[3] << 16));
        *reinterpret_cast<uint2*>(p.nextLo + o) = make_uint2((unsigned)l[0] | ((unsigned)l[1] << 16), (unsigned)l[2] | ((unsigned)l[3] << 16));
    }
}

// q | k | v: the row's sums go to LDS (scale and bias applied), then RoPE on q and k
// (mongoose.cu:991-1006) and the K/V rows into the caches (mongoose.cu:1644-1647), as
// rope_store_rows_kernel does them.  One workgroup per row; dynamic LDS = (dim + 2*kvDim) floats.
template <typename KVT>
__global__ __launch_bounds__(PWG) void gemm_reduce_qkv_rope_kernel(GemmParams p, int BN) {
    extern __shared__ float row[];
    const int m = blockIdx.x;
    const int dim = p.seg[0].N, kvDim = p.seg[1].N;
    const size_t plane = (size_t)p.T * p.ldPartial / 4;
    const float4* src = reinterpret_cast<const float4*>(p.partial + (size_t)m * p.ldPartial);
    for (int c4 = threadIdx.x; c4 * 4 < p.ldPartial; c4 += PWG) {
        const int tile = c4 * 4 / BN;
        int sgi = 0;
        if (tile >= p.seg[1].tile0) sgi = 1;
        if (tile >= p.seg[2].tile0) sgi = 2;
        GemmSeg sg = p.seg[0];
        if (sgi == 1) sg = p.seg[1];
        if (sgi == 2) sg = p.seg[2];
        const int n = c4 * 4 - sg.tile0 * BN;
        if (n >= sg.N) continue;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        int s = 0;
        for (; s + 4 <= p.splitK; s += 4) {             // four loads in flight, added in split order
            const float4 a = src[(size_t)s * plane + c4], b = src[(size_t)(s + 1) * plane + c4];
            const float4 c = src[(size_t)(s + 2) * plane + c4], d = src[(size_t)(s + 3) * plane + c4];
            v.x += a.x; v.y += a.y; v.z += a.z; v.w += a.w;
            v.x += b.x; v.y += b.y; v.z += b.z; v.w += b.w;
            v.x += c.x; v.y += c.y; v.z += c.z; v.w += c.w;
            v.x += d.x; v.y += d.y; v.z += d.z; v.w += d.w;
        }
        for (; s < p.splitK; s++) {
            const float4 a = src[(size_t)s * plane + c4];
            v.x += a.x; v.y += a.y; v.z += a.z; v.w += a.w;
        }
        float4 sc = make_float4(1.f, 1.f, 1.f, 1.f), bi = make_float4(0.f, 0.f, 0.f, 0.f);
        if (sg.scales) sc = *reinterpret_cast<const float4*>(sg.scales + n);
        if (sg.bias) bi = *reinterpret_cast<const float4*>(sg.bias + n);
        v.x = v.x * sc.x + bi.x; v.y = v.y * sc.y + bi.y; v.z = v.z * sc.z + bi.z; v.w = v.w * sc.w + bi.w;
        const int base = sgi == 0 ? 0 : (sgi == 1 ? dim : dim + kvDim);
        *reinterpret_cast<float4*>(&row[base + n]) = v;
    }
    __syncthreads();
    const int headDim = p.ropeHeadDim, half = headDim / 2, pos = p.ropePos0 + m;
    const float* c = p.ropeCos + (size_t)pos * half;
    const float* s = p.ropeSin + (size_t)pos * half;
    float* qr = p.seg[0].Y + (size_t)m * dim;
    for (int i = threadIdx.x; i < dim / 2; i += PWG) {
        const int h = i / half, j = i % half;
        const float x0 = row[h * headDim + j], x1 = row[h * headDim + half + j];
        qr[h * headDim + j] = x0 * c[j] - x1 * s[j];
        qr[h * headDim + half + j] = x0 * s[j] + x1 * c[j];
    }
    KVT* kd = static_cast<KVT*>(p.ropeKc) + (size_t)pos * kvDim;
    KVT* vd = static_cast<KVT*>(p.ropeVc) + (size_t)pos * kvDim;
    const float* kr = row + dim;
    const float* vr = row + dim + kvDim;
    for (int i = threadIdx.x; i < kvDim / 2; i += PWG) {
        const int h = i / half, j = i % half;
        const float x0 = kr[h * headDim + j], x1 = kr[h * headDim + half + j];
        kd[h * headDim + j] = (KVT)(x0 * c[j] - x1 * s[j]);
        kd[h * headDim + half + j] = (KVT)(x0 * s[j] + x1 * c[j]);
    }
    for (int i = threadIdx.x; i < kvDim; i += PWG) vd[i] = (KVT)vr[i];
}

// gate | up: sums of the splits, scale/bias, silu(gate) * up, hi/lo split.  Grid (columns / 256, rows).
__global__ __launch_bounds__(PWG) void gemm_reduce_swiglu_split_kernel(GemmParams p, int BN) {
    const int n = blockIdx.x * PWG + threadIdx.x;
    const int m = blockIdx.y;
    const int N = p.seg[0].N;
    if (n >= N) return;
    const size_t plane = (size_t)p.T * p.ldPartial;
    const float* sg_ = p.partial + (size_t)m * p.ldPartial + n;
    const float* su_ = sg_ + (size_t)p.seg[1].tile0 * BN;
    float g = 0.f, u = 0.f;
    int s = 0;
    for (; s + 2 <= p.splitK; s += 2) {
        const float g0 = sg_[(size_t)s * plane], g1 = sg_[(size_t)(s + 1) * plane];
        const float u0 = su_[(size_t)s * plane], u1 = su_[(size_t)(s + 1) * plane];
        g += g0; g += g1; u += u0; u += u1;
    }
    for (; s < p.splitK; s++) { g += sg_[(size_t)s * plane]; u += su_[(size_t)s * plane]; }
    g = g * (p.seg[0].scales ? p.seg[0].scales[n] : 1.0f) + (p.seg[0].bias ? p.seg[0].bias[n] : 0.f);
    u = u * (p.seg[1].scales ? p.seg[1].scales[n] : 1.0f) + (p.seg[1].bias ? p.seg[1].bias[n] : 0.f);
    const float a = g * (1.0f / (1.0f + expf(-g))) * u;
    const unsigned short h = f32_to_bf16_rne(a);
    const size_t o = tiled_index(m, n, N);
    p.nextHi[o] = h;
    p.nextLo[o] = f32_to_bf16_rne(a - bf16_to_f32(h));
}

// Sums the splits (and, where the caller asked for it and the shape allows, does the row-wise step that follows).
static void launch_reduce(GemmParams& p, int BN, int residual, hipStream_t s) {
    const int N = p.seg[0].N;
    if (p.nseg == 1 && residual && p.nextHi && p.nextLo && N % 4 == 0 && N <= 16 * 4 * PWG) {
        hipLaunchKernelGGL(gemm_reduce_norm_split_kernel, dim3((unsigned)p.T), dim3(PWG), 0, s, p);
        p.wroteNext = 1;
        return;
    }
    if (p.nseg == 3 && !residual && p.ropeKc && p.ropeVc && p.seg[1].N == p.seg[2].N && p.seg[0].N % 4 == 0 &&
        p.seg[1].N % 4 == 0 && p.ropeHeadDim > 0 && p.seg[0].N % p.ropeHeadDim == 0 && p.seg[1].N % p.ropeHeadDim == 0) {
        const size_t lds = (size_t)(p.seg[0].N + 2 * p.seg[1].N) * sizeof(float);
        if (lds <= 48 * 1024) {
            if (p.ropeKvHalf) hipLaunchKernelGGL(gemm_reduce_qkv_rope_kernel<_Float16>, dim3((unsigned)p.T), dim3(PWG), lds, s, p, BN);
            else hipLaunchKernelGGL(gemm_reduce_qkv_rope_kernel<float>, dim3((unsigned)p.T), dim3(PWG), lds, s, p, BN);
            p.wroteRope = 1;
            return;
        }
    }
    if (p.nseg == 2 && !residual && p.nextSwiglu && p.nextHi && p.nextLo && p.seg[0].N == p.seg[1].N) {
        hipLaunchKernelGGL(gemm_reduce_swiglu_split_kernel, dim3((unsigned)((p.seg[0].N + PWG - 1) / PWG), (unsigned)p.T), dim3(PWG), 0,
                           s, p, BN);
        p.wroteNext = 1;
        return;
    }
    hipLaunchKernelGGL(gemm_reduce_kernel, dim3((unsigned)((p.ldPartial + PWG - 1) / PWG), (unsigned)p.T), dim3(PWG), 0, s, p, BN,
                       residual);
}

size_t gemm_partial_floats() { return (size_t)320 * 256 * 256; }

template <int Q4>
static hipError_t launch_gemm_fmt(GemmParams& p, int residual, hipStream_t s) {
    auto count = [&](int bn) {
        int tiles = 0;
        for (int i = 0; i < p.nseg; i++) { p.seg[i].tile0 = tiles; tiles += (p.seg[i].N + bn - 1) / bn; }
        p.nTiles = tiles;
        return tiles;
    };
    // the large configuration: Q8 256 x 256 with 1024 threads; Q4_0 128 x 256 with 512 (it needs the
    // scratch accumulator and more fragment registers than 1024 threads leave)
    constexpr int BMB = Q4 ? 128 : 256, NTB = Q4 ? 512 : 1024;
    const int ksteps = (p.K + BK - 1) / BK;
    p.splitK = 1; p.stepsPerSplit = ksteps;
    const bool ringOk = p.K % 128 == 0;          // the ring kernel takes its K steps four at a time
    if (!Q4 && ringOk && p.T > 128 && p.nseg == 2 && !residual && p.nextSwiglu && p.nextHi && p.nextLo && p.seg[0].N == p.seg[1].N) {
        // gate | up with enough 128-column tiles to fill the chip without splitting K: the GEMM's own
        // epilogue forms silu(gate) * up and writes its hi/lo split
        const int tiles = (p.seg[0].N + 127) / 128;
        const int numM = (p.T + 255) / 256;
        if (tiles * numM >= 160) {
            p.nTiles = tiles;
            dim3 grid((unsigned)(((tiles + 7) / 8) * 8 * numM), 1);
            hipError_t e = launch_ring<3>(p, grid, s);
            if (e == hipSuccess) p.wroteNext = 1;
            return e;
        }
    }
    if (p.T > 128) {
        // K is split until about one workgroup per CU exists (each split keeps >= 8 steps).  Worth it
        // when the tiles alone nearly fill the chip or K can be split; otherwise the small tiles below
        // give more workgroups (short K, narrow N: latency-bound either way).
        const int tiles = count(256);
        const int numM = (p.T + BMB - 1) / BMB;
        const int wgs = tiles * numM;
        int S = 1;
        if (p.partial && wgs < 160) {
            S = (224 + wgs / 2) / wgs;
            if (S > ksteps / 8) S = ksteps / 8;
            if (S < 1) S = 1;
            while (S > 1 && (size_t)S * p.T * tiles * 256 > gemm_partial_floats()) S--;
        }
        // ... and only if that launch then has a workgroup for (nearly) every CU: a down projection of a
        // small model (N = 896: 8 tiles, 9 splits) is better off on the small tiles, which split K further
        if ((wgs >= 96 || S >= 2) && wgs * S >= 200) {
            dim3 grid((unsigned)(((tiles + 7) / 8) * 8 * numM), 1);
            if (S > 1) {
                p.stepsPerSplit = (ksteps + S - 1) / S;
                if (!Q4 && ringOk) p.stepsPerSplit = (p.stepsPerSplit + 1) & ~1;      // 64-k steps: an even count = 32-k steps in fours
                S = (ksteps + p.stepsPerSplit - 1) / p.stepsPerSplit;
                grid.y = (unsigned)S;
                p.splitK = S; p.ldPartial = tiles * 256;
                if (Q4 || !ringOk) {
                    hipLaunchKernelGGL((gemm_q8_bf16x2_kernel<Q4, BMB, 256, NTB, 2>), grid, dim3(NTB), 0, s, p);
                } else {
                    hipError_t e = launch_ring<2>(p, grid, s);
                    if (e != hipSuccess) return e;
                }
                launch_reduce(p, 256, residual, s);
                return hipGetLastError();
            }
            if (Q4 || !ringOk) {
                if (residual) hipLaunchKernelGGL((gemm_q8_bf16x2_kernel<Q4, BMB, 256, NTB, 1>), grid, dim3(NTB), 0, s, p);
                else hipLaunchKernelGGL((gemm_q8_bf16x2_kernel<Q4, BMB, 256, NTB, 0>), grid, dim3(NTB), 0, s, p);
                return hipGetLastError();
            } else {
                return residual ? launch_ring<1>(p, grid, s) : launch_ring<0>(p, grid, s);
            }
        }
    }
    if constexpr (Q4 != 0) {
        // Q4_0 in between: the 128 x 256 tiles, K not split, where they give at least a workgroup for
        // every other CU (gate | up of a small model): half the L2-to-CU bytes per flop of the small tile.
        // (For Q8 the small tiles measured faster at this size.)
        if (p.T > 128) {
            const bool swiglu = p.nseg == 2 && !residual && p.nextSwiglu && p.nextHi && p.nextLo && p.seg[0].N == p.seg[1].N;
            const int tilesM = swiglu ? (p.seg[0].N + 127) / 128 : count(256);
            const int numM = (p.T + 127) / 128;
            if (tilesM * numM >= 128) {
                p.nTiles = tilesM;
                dim3 grid((unsigned)(((tilesM + 7) / 8) * 8 * numM), 1);
                if (swiglu) {
                    hipLaunchKernelGGL((gemm_q8_bf16x2_kernel<Q4, 128, 256, 512, 3>), grid, dim3(512), 0, s, p);
                    p.wroteNext = 1;
                } else if (residual) {
                    hipLaunchKernelGGL((gemm_q8_bf16x2_kernel<Q4, 128, 256, 512, 1>), grid, dim3(512), 0, s, p);
                } else {
                    hipLaunchKernelGGL((gemm_q8_bf16x2_kernel<Q4, 128, 256, 512, 0>), grid, dim3(512), 0, s, p);
                }
                return hipGetLastError();
            }
        }
    }
    const int tiles = count(128);
    const int numM = (p.T + 63) / 64;
    dim3 grid((unsigned)(((tiles + 7) / 8) * 8 * numM), 1);
    // These shapes are bound by the memory latency of each K step (one workgroup per CU or fewer, one
    // step of lookahead), so K is split as well, down to 4 steps a piece, until a few workgroups share
    // every CU and cover each other's waits.
    const int wgs = tiles * numM;
    int S = 1;
    if (p.partial && wgs < 512 && ksteps >= 8) {
        S = (768 + wgs - 1) / wgs;
        if (S > ksteps / 4) S = ksteps / 4;
        while (S > 1 && (size_t)S * p.T * tiles * 128 > gemm_partial_floats()) S--;
    }
    if (S > 1) {
        p.stepsPerSplit = (ksteps + S - 1) / S;
        S = (ksteps + p.stepsPerSplit - 1) / p.stepsPerSplit;
        grid.y = (unsigned)S;
        p.splitK = S; p.ldPartial = tiles * 128;
        hipLaunchKernelGGL((gemm_q8_bf16x2_kernel<Q4, 64, 128, 256, 2>), grid, dim3(PWG), 0, s, p);
        launch_reduce(p, 128, residual, s);
    } else if (residual) {
        hipLaunchKernelGGL((gemm_q8_bf16x2_kernel<Q4, 64, 128, 256, 1>), grid, dim3(PWG), 0, s, p);
    } else if (p.nseg == 2 && p.nextSwiglu && p.nextHi && p.nextLo && p.seg[0].N == p.seg[1].N) {
        // gate | up, K not split: silu(gate) * up and its hi/lo split in the GEMM's own epilogue
        p.nTiles = (p.seg[0].N + 63) / 64;
        dim3 g3((unsigned)(((p.nTiles + 7) / 8) * 8 * numM), 1);
        hipLaunchKernelGGL((gemm_q8_bf16x2_kernel<Q4, 64, 128, 256, 3>), g3, dim3(PWG), 0, s, p);
        p.wroteNext = 1;
    } else {
        hipLaunchKernelGGL((gemm_q8_bf16x2_kernel<Q4, 64, 128, 256, 0>), grid, dim3(PWG), 0, s, p);
    }
    return hipGetLastError();
}

hipError_t launch_gemm_q8(GemmParams& p, int residual, hipStream_t s) {
    if (p.T <= 0 || p.nseg < 1 || p.nseg > 3) return p.T <= 0 ? hipSuccess : hipErrorInvalidValue;
    if (p.K <= 0 || p.K % 32 != 0) return hipErrorInvalidValue;
    for (int i = 0; i < p.nseg; i++) if (p.seg[i].N <= 0) return hipErrorInvalidValue;
    p.wroteNext = 0;
    p.wroteRope = 0;
    return p.q4 ? launch_gemm_fmt<1>(p, residual, s) : launch_gemm_fmt<0>(p, residual, s);
}

}  // namespace mg
