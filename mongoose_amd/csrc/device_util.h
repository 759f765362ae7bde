// device_util.h -- device helpers shared by the kernel files: wave64 / workgroup reductions through DPP
// and the gfx950 permlane swaps, and the per-chunk dot products of the dequantizing matvec.
#pragma once
#include <hip/hip_runtime.h>
#include <limits.h>
#include <math.h>

namespace mg {

constexpr int WG = 256;

// ---------------------------------------------------------------------------
// wave64 / workgroup reductions
// ---------------------------------------------------------------------------
// Lane exchange inside a row of 16 lanes through DPP (no LDS traffic):
// quad_perm [1,0,3,2] = 0xB1, quad_perm [2,3,0,1] = 0x4E, row_ror:4 = 0x124, row_ror:8 = 0x128.
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
// Exchange between the four rows of 16 lanes, in the VALU instead of through the LDS crossbar
// (ds_bpermute): v_permlane16_swap exchanges the odd rows of its first operand with the even rows of
// its second, v_permlane32_swap the upper half of the first with the lower half of the second.  With
// the same value in both operands the two results are (own, partner) or (partner, own) in every lane:
// their sum / maximum is v combined with the lane 16 (32) away, and since both operations are
// commutative the bits are those of v op shfl_xor(v, 16 / 32).
__device__ __forceinline__ void row_swap16(float& a, float& b) {
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ void row_swap32(float& a, float& b) {
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ float rows_sum(float v) {      // over lanes l, l^16, l^32, l^48
    float a = v, b = v;
    row_swap16(a, b);
    a = a + b; b = a;
    row_swap32(a, b);
    return a + b;
}
__device__ __forceinline__ float rows_max(float v) {
    float a = v, b = v;
    row_swap16(a, b);
    a = fmaxf(a, b); b = a;
    row_swap32(a, b);
    return fmaxf(a, b);
}
// Greatest value of the wave and, among equals, its lowest index, in every lane: the combination is
// symmetric and idempotent, so it does not matter which of the two operands is the lane's own.
__device__ __forceinline__ void argmax_pick(float& v, int& i, float ov, int oi) {
    if (ov > v || (ov == v && oi < i)) { v = ov; i = oi; }
}
template <int CTRL>
__device__ __forceinline__ int dpp_i(int v) { return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true); }
__device__ __forceinline__ void wave_argmax(float& v, int& i) {
    float va = v, vb = v;
    float ia = __builtin_bit_cast(float, i), ib = ia;
    row_swap32(va, vb); row_swap32(ia, ib);
    v = va; i = __builtin_bit_cast(int, ia);
    argmax_pick(v, i, vb, __builtin_bit_cast(int, ib));
    va = v; vb = v; ia = __builtin_bit_cast(float, i); ib = ia;
    row_swap16(va, vb); row_swap16(ia, ib);
    v = va; i = __builtin_bit_cast(int, ia);
    argmax_pick(v, i, vb, __builtin_bit_cast(int, ib));
    argmax_pick(v, i, dpp_f<0x128>(v), dpp_i<0x128>(i));     // row_ror:8, row_ror:4, then the quad
    argmax_pick(v, i, dpp_f<0x124>(v), dpp_i<0x124>(i));
    argmax_pick(v, i, dpp_f<0x4E>(v), dpp_i<0x4E>(i));
    argmax_pick(v, i, dpp_f<0xB1>(v), dpp_i<0xB1>(i));
}
__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_f<0xB1>(v);
    v += dpp_f<0x4E>(v);
    v += dpp_f<0x124>(v);
    v += dpp_f<0x128>(v);
    return rows_sum(v);
}
// Two sums over the wave for the price of little more than one: the first exchange folds them into one register
// (lanes 0..31 carry a, lanes 32..63 carry b), the rest reduces within the halves.  Returns sum(a) in lanes 0..31 and
// sum(b) in lanes 32..63.
__device__ __forceinline__ float wave_sum2(float a, float b) {
    row_swap32(a, b);                      // a: [a low half | b low half], b: [a high half | b high half]
    float t = a + b;
    float x = t, y = t;
    row_swap16(x, y);
    t = x + y;
    t += dpp_f<0xB1>(t);
    t += dpp_f<0x4E>(t);
    t += dpp_f<0x124>(t);
    t += dpp_f<0x128>(t);
    return t;
}
__device__ __forceinline__ float lane_value(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_f<0xB1>(v));
    v = fmaxf(v, dpp_f<0x4E>(v));
    v = fmaxf(v, dpp_f<0x124>(v));
    v = fmaxf(v, dpp_f<0x128>(v));
    return rows_max(v);
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
// Chunk dot products
// ---------------------------------------------------------------------------
__device__ __forceinline__ float dot4_i8(int w, float4 a, float acc) {
    acc = fmaf((float)(int)(signed char)(w & 0xff), a.x, acc);
    acc = fmaf((float)(int)(signed char)((w >> 8) & 0xff), a.y, acc);
    acc = fmaf((float)(int)(signed char)((w >> 16) & 0xff), a.z, acc);
    acc = fmaf((float)(w >> 24), a.w, acc);
    return acc;
}
// sum over 4 bytes of a * nibble; n holds one nibble per byte (0..15).  The -8
// offset of Q4_0 is applied once per chunk from the sum of its activations.
template <int B>
__device__ __forceinline__ float cvt_ubyte(unsigned n) {
    // v_cvt_f32_ubyteN straight from the masked dword: one convert per weight; written out
    // because the compiler otherwise re-derives every nibble with its own bit-field extract
    float f;
    if (B == 0) asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(f) : "v"(n));
    else if (B == 1) asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(f) : "v"(n));
    else if (B == 2) asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(f) : "v"(n));
    else asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(f) : "v"(n));
    return f;
}
__device__ __forceinline__ float dot4_nib(unsigned n, float4 a, float acc) {
    acc = fmaf(cvt_ubyte<0>(n), a.x, acc);
    acc = fmaf(cvt_ubyte<1>(n), a.y, acc);
    acc = fmaf(cvt_ubyte<2>(n), a.z, acc);
    acc = fmaf(cvt_ubyte<3>(n), a.w, acc);
    return acc;
}
__device__ __forceinline__ float half_bits_to_float(unsigned short h) {
    return (float)__builtin_bit_cast(_Float16, h);
}

// Q4_0 half block: s = sum_i act_i*nib_i - 8*sum_i act_i, then acc += s * f32(d)
// (block form kernels/infer.metal:63-75; the -8 folded as kernels/q4_simd.metal:6-19
// does).  Element order: low nibble of byte j = element j, high nibble = element
// j+16 of the block (GGML).
__device__ __forceinline__ float dot_q4_half(int2 w, float d, const float4 (&av)[4], float asum, float acc) {
    float s = -8.0f * asum;
    unsigned q;
    q = (unsigned)w.x; s = dot4_nib(q & 0x0f0f0f0fu, av[0], s); s = dot4_nib((q >> 4) & 0x0f0f0f0fu, av[2], s);
    q = (unsigned)w.y; s = dot4_nib(q & 0x0f0f0f0fu, av[1], s); s = dot4_nib((q >> 4) & 0x0f0f0f0fu, av[3], s);
    return fmaf(s, d, acc);
}
// The sum of a chunk's 16 activations, in the order every Q4_0 path uses.
__device__ __forceinline__ float chunk_act_sum(const float4 (&av)[4]) {
    float4 t;
    t.x = (av[0].x + av[1].x) + (av[2].x + av[3].x);
    t.y = (av[0].y + av[1].y) + (av[2].y + av[3].y);
    t.z = (av[0].z + av[1].z) + (av[2].z + av[3].z);
    t.w = (av[0].w + av[1].w) + (av[2].w + av[3].w);
    return (t.x + t.y) + (t.z + t.w);
}

// Element i of token tok's embedding row.  kind 0: int8 rows [vocab, dim] times the row's scale (a tied Q8 lm_head),
// 1: fp16 table, 2: fp32 table, 3: Q4_0 in the split layout (nibble plane [vocab, dim/2], then the fp16 d plane).
__device__ __forceinline__ float embed_value(int kind, const void* table, const float* scales, int tok, int dim, int vocab, int i) {
    if (kind == 0) {
        const signed char* q = static_cast<const signed char*>(table) + (size_t)tok * dim;
        return (float)q[i] * scales[tok];
    }
    if (kind == 1) return half_bits_to_float((static_cast<const unsigned short*>(table) + (size_t)tok * dim)[i]);
    if (kind == 2) return static_cast<const float*>(table)[(size_t)tok * dim + i];
    const unsigned char* base = static_cast<const unsigned char*>(table);
    const unsigned char* qs = base + (size_t)tok * (dim >> 1);
    const unsigned short* dpl = reinterpret_cast<const unsigned short*>(base + (size_t)vocab * (dim >> 1)) + (size_t)tok * (dim >> 5);
    const int b = i >> 5, j = i & 31;
    const unsigned char q = qs[b * 16 + (j & 15)];
    const int nib = j < 16 ? (q & 0x0f) : (q >> 4);
    return (float)(nib - 8) * half_bits_to_float(dpl[b]);
}

// ---------------------------------------------------------------------------
// Agent-scope accesses and the decode attention's row helpers
// ---------------------------------------------------------------------------
__device__ __forceinline__ float ld_agent(const float* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_agent(float* p, float v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Sum over the 16 lanes (one DPP row) that hold a K/V row.  Every step adds a lane's value to its
// mirror partner's (quad_perm, then row_half_mirror = 0x141, row_mirror = 0x140), so both partners
// compute the same commutative sum: all lanes of the row end with the same bits, which keeps
// exp(score - max) identical across the lanes that apply it.
__device__ __forceinline__ float row_sum16(float v) {
    v += dpp_f<0xB1>(v);
    v += dpp_f<0x4E>(v);
    v += dpp_f<0x141>(v);
    v += dpp_f<0x140>(v);
    return v;
}
// combine a per-thread value over the four row groups (tg) that share a wave
__device__ __forceinline__ float tg_max(float v) { return rows_max(v); }
__device__ __forceinline__ float tg_sum(float v) { return rows_sum(v); }

// exp(x) for x <= 0 as one multiply and the hardware's 2^x (1 ulp; the product x * log2(e) adds
// |x| * 2^-24 relative, 2e-6 at x = -20): the library's expf is a dozen instructions, and a thread
// of the decode attention, at one or two waves a SIMD, pays the latency of every one of them.
__device__ __forceinline__ float exp_neg(float x) { return __builtin_amdgcn_exp2f(x * 1.4426950408889634f); }

}  // namespace mg
