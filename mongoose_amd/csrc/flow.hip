// flow.hip -- all layers of a batch-1 decode step in one persistent launch (see flow.h).
//
// Arithmetic per phase is that of the separate launches (kernels.hip): RMSNorm folded into the staged
// vector and the row epilogue, int8 rows against fp32 activations with fp32 accumulation, RoPE on (j, j+hd/2)
// pairs, softmax with a running maximum, SiLU(g)*u, residual adds (cuda_fused_infer.go:414-444,
// cuda_fused_stream.go:319-321, kernels/mongoose.cu:145-174, 856-933, 949-956, 991-1006, 1556-1585).
//
// Hand-over protocol.  Every vector that one phase produces and the next consumes lives in the exchange
// area, one block per layer.  Before the launch every float there is XSENT (a NaN pattern no arithmetic
// here produces: results equal to it are canonicalised on the way out).  Producers store at agent scope
// (write-through, visible to the other XCDs' loads that bypass their L2); consumers load at agent scope
// and repeat until nothing they need is XSENT.  A workgroup only ever waits for phases that precede its
// own in the same fixed order, so with all workgroups resident every wait ends; every wait is bounded by
// a time limit all the same, after which the workgroup stops waiting (results are then garbage and
// *err is set, which the host checks).
#include <cstddef>
#include "flow.h"
#include "device_util.h"

namespace mg {

constexpr unsigned XSENT = 0xFFFFFFFFu;
constexpr int FWAVES = 8;                 // waves of a workgroup (two a SIMD: a wave's instruction latencies are covered by its partner)
constexpr int FWG = 64 * FWAVES;
typedef float f4 __attribute__((ext_vector_type(4)));

// The pointers of the layer table are read from memory, so the compiler takes them for generic pointers and loads
// through them with FLAT instructions, which count as LDS operations as well (a wait for an LDS read then also waits
// for the weights in flight).  What is loaded through them is loaded through explicitly global pointers instead.
typedef int gv4i __attribute__((ext_vector_type(4)));
typedef int gv2i __attribute__((ext_vector_type(2)));
template <bool GL>
__device__ __forceinline__ int4 ldg_i4(const void* p, size_t i) {
    if (!GL) return static_cast<const int4*>(p)[i];
    const gv4i t = ((const gv4i __attribute__((address_space(1)))*)p)[i];
    return make_int4(t.x, t.y, t.z, t.w);
}
template <bool GL>
__device__ __forceinline__ int2 ldg_i2(const void* p, size_t i) {
    if (!GL) return static_cast<const int2*>(p)[i];
    const gv2i t = ((const gv2i __attribute__((address_space(1)))*)p)[i];
    return make_int2(t.x, t.y);
}
template <bool GL>
__device__ __forceinline__ unsigned short ldg_u16(const void* p, size_t i) {
    if (!GL) return static_cast<const unsigned short*>(p)[i];
    return ((const unsigned short __attribute__((address_space(1)))*)p)[i];
}
template <bool GL>
__device__ __forceinline__ void stg_f(float* p, size_t i, float v) {
    if (!GL) { p[i] = v; return; }
    ((float __attribute__((address_space(1)))*)p)[i] = v;
}
template <bool GL>
__device__ __forceinline__ float ldg_f(const float* p, size_t i) {
    if (!GL) return p[i];
    return ((const float __attribute__((address_space(1)))*)p)[i];
}
template <bool GL>
__device__ __forceinline__ float4 ldg_f4(const void* p, size_t i) {
    if (!GL) return static_cast<const float4*>(p)[i];
    const f4 t = ((const f4 __attribute__((address_space(1)))*)p)[i];
    return make_float4(t.x, t.y, t.z, t.w);
}

__device__ __forceinline__ bool unset(float v) { return __builtin_bit_cast(unsigned, v) == XSENT; }
__device__ __forceinline__ float canon(float v) { return unset(v) ? __builtin_bit_cast(float, 0x7FC00000u) : v; }
__device__ __forceinline__ bool ready4(f4 v) { return !(unset(v.x) || unset(v.y) || unset(v.z) || unset(v.w)); }

struct Waiter {
    long long limit;
    int* err;
    bool dead;
    const f4* idle;      // a line nothing writes during the launch (see poll_batch)
    __device__ __forceinline__ void fail() {
        dead = true;
        __hip_atomic_store(err, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
};

// 16-byte agent-scope load (bypasses this XCD's L2) / store (write-through)
__device__ __forceinline__ f4 ldx4(const f4* p) {
    f4 v;
    asm volatile("global_load_dwordx4 %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=&v"(v) : "v"(p) : "memory");
    return v;
}
__device__ __forceinline__ void stx4(f4* p, f4 v) {
    v.x = canon(v.x); v.y = canon(v.y); v.z = canon(v.z); v.w = canon(v.w);
    asm volatile("global_store_dwordx4 %0, %1, off sc1" : : "v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ void stx(float* p, float v) { st_agent(p, canon(v)); }

__device__ __forceinline__ f4 poll4(const f4* p, Waiter& w) {
    f4 v = ldx4(p);
    if (ready4(v) || w.dead) return v;
    const long long t0 = wall_clock64();
    for (;;) {
        v = ldx4(p);
        if (ready4(v)) break;
        if (wall_clock64() - t0 > w.limit) { w.fail(); break; }
    }
    return v;
}
__device__ __forceinline__ float poll1(const float* p, Waiter& w) {
    float v = ld_agent(p);
    if (!unset(v) || w.dead) return v;
    const long long t0 = wall_clock64();
    for (;;) {
        v = ld_agent(p);
        if (!unset(v)) break;
        if (wall_clock64() - t0 > w.limit) { w.fail(); break; }
    }
    return v;
}
// Three pieces with all their loads in flight at once: one memory round trip instead of three.
// Loads and the wait for them are one asm statement -- with the wait in a statement of its own the
// compiler is free to copy a destination register between the two, i.e. before the data has arrived.
__device__ __forceinline__ void ldx4_3(const f4* const (&p)[3], f4 (&v)[3]) {
    asm volatile("global_load_dwordx4 %0, %3, off sc1\n\tglobal_load_dwordx4 %1, %4, off sc1\n\t"
                 "global_load_dwordx4 %2, %5, off sc1\n\ts_waitcnt vmcnt(0)"
                 : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]) : "v"(p[0]), "v"(p[1]), "v"(p[2]) : "memory");
}
__device__ __forceinline__ unsigned unset1(float v) { return __builtin_bit_cast(unsigned, v) == XSENT ? 1u : 0u; }
__device__ __forceinline__ unsigned unset4(f4 v) { return unset1(v.x) | unset1(v.y) | unset1(v.z) | unset1(v.w); }
// A KV split's partial for one 16-byte piece of the attention output: accumulator piece, maximum and sum of its head,
// asked for together (one round trip), repeated until all three are there.
__device__ __forceinline__ void poll_partial(const f4* pa, const float* pm, const float* pl, f4& a, float& m, float& l, Waiter& w) {
    long long t0 = 0;
    bool timing = false;
    for (;;) {
        asm volatile("global_load_dwordx4 %0, %3, off sc1\n\tglobal_load_dword %1, %4, off sc1\n\t"
                     "global_load_dword %2, %5, off sc1\n\ts_waitcnt vmcnt(0)"
                     : "=&v"(a), "=&v"(m), "=&v"(l) : "v"(pa), "v"(pm), "v"(pl) : "memory");
        const unsigned missing = unset4(a) | unset1(m) | unset1(l);
        if (!missing || w.dead) break;
        if (!timing) { timing = true; t0 = wall_clock64(); }
        else if (wall_clock64() - t0 > w.limit) { w.fail(); break; }
    }
}
// A layer's table entry, read one layer ahead: lane i loads word i (the entry is in HBM and cold; read at the top of
// its layer it would hold up every wave of the launch).
__device__ __forceinline__ unsigned layer_words(const FlowLayer* t, int l, int lane) {
    static_assert(sizeof(FlowLayer) <= 64 * 4, "one word a lane");
    const unsigned* q = reinterpret_cast<const unsigned*>(t + l);
    return q[lane < (int)(sizeof(FlowLayer) / 4) ? lane : 0];
}
template <class T>
__device__ __forceinline__ T* lane_ptr(unsigned v, int word) {
    const unsigned lo = (unsigned)__builtin_amdgcn_readlane((int)v, word), hi = (unsigned)__builtin_amdgcn_readlane((int)v, word + 1);
    return reinterpret_cast<T*>(((unsigned long long)hi << 32) | lo);
}
// The fields of a layer's entry are picked out of the lanes where they are used, two readlanes a pointer, not all at the
// top of the layer: 21 pointers held in scalar registers across a layer's phases, on top of the launch's parameters, are
// more than the scalar file has, and the compiler then parks them in lanes of a vector register of its own and fetches
// them back one by one -- some 60 lane writes and over 100 lane reads a layer and wave.
struct LayerView {
    unsigned v;
#define FL_FIELD(T, field) __device__ __forceinline__ T* field() const { return lane_ptr<T>(v, (int)(offsetof(FlowLayer, field) / 4)); }
    FL_FIELD(const float, g1) FL_FIELD(const float, g2)
    FL_FIELD(const signed char, wq) FL_FIELD(const signed char, wk) FL_FIELD(const signed char, wv) FL_FIELD(const signed char, wo)
    FL_FIELD(const signed char, gate) FL_FIELD(const signed char, up) FL_FIELD(const signed char, down)
    FL_FIELD(const float, sq) FL_FIELD(const float, sk) FL_FIELD(const float, sv) FL_FIELD(const float, so)
    FL_FIELD(const float, sgate) FL_FIELD(const float, sup) FL_FIELD(const float, sdown)
    FL_FIELD(const float, bq) FL_FIELD(const float, bk) FL_FIELD(const float, bv)
    FL_FIELD(float, Kc) FL_FIELD(float, Vc)
#undef FL_FIELD
};
// The tail's operands (FlowTail), read the same way: one word a lane, fields picked out where they are used.
__device__ __forceinline__ unsigned tail_words(const FlowTail* t, int lane) {
    static_assert(sizeof(FlowTail) <= 64 * 4, "one word a lane");
    const unsigned* q = reinterpret_cast<const unsigned*>(t);
    return q[lane < (int)(sizeof(FlowTail) / 4) ? lane : 0];
}
#define TW_PTR(T, field) lane_ptr<T>(tw, (int)(offsetof(FlowTail, field) / 4))
#define TW_INT(field) __builtin_amdgcn_readlane((int)tw, (int)(offsetof(FlowTail, field) / 4))

// An argmax partial: value (low word) and index (high word) travel as one 8-byte store and one 8-byte load; a
// workgroup's partial has a 128-byte line of its own (FLOW_AMAX_STRIDE floats), written once a token.
__device__ __forceinline__ void store_arg(float* slot, float v, int i) {
    const unsigned long long w = (unsigned long long)__builtin_bit_cast(unsigned, canon(v)) | ((unsigned long long)(unsigned)i << 32);
    asm volatile("global_store_dwordx2 %0, %1, off sc1" : : "v"(slot), "v"(w) : "memory");
}
struct ArgPart { float v; int i; };
__device__ __forceinline__ ArgPart poll_arg(const float* p, Waiter& w) {
    unsigned long long x;
    long long t0 = 0;
    bool timing = false;
    for (;;) {
        asm volatile("global_load_dwordx2 %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=&v"(x) : "v"(p) : "memory");
        const unsigned missing = ((unsigned)x == XSENT ? 1u : 0u) | ((unsigned)(x >> 32) == XSENT ? 1u : 0u);
        if (!missing || w.dead) break;
        if (!timing) { timing = true; t0 = wall_clock64(); }
        else if (wall_clock64() - t0 > w.limit) { w.fail(); break; }
        for (int z = 0; z < 4; z++) __builtin_amdgcn_s_sleep(2);
    }
    return ArgPart{__builtin_bit_cast(float, (unsigned)x), (int)(unsigned)(x >> 32)};
}

constexpr int PB = 3;        // float4 pieces a thread polls at once (a round of the 512 threads covers 6144 floats)
// Every polling loop here has one shape: a straight loop around ONE asm statement (a fixed number of loads and their
// wait), whose results are tested together as one word; nothing inside the loop chooses between asm statements.
// poll_batch always asks for PB pieces: a thread with fewer pieces of the vector left (n < PB) points the others at its
// workgroup's idle line (Waiter::idle: memory that nothing writes during the launch, so those loads hit in the L2
// and never in a line that producers are storing to) and ignores what comes back.  A thread with no piece at all
// asks for nothing: clamped to the vector's last piece instead, hundreds of threads of every workgroup would re-read
// that one line while its producers are still storing to it.
// SINGLE (fixed where the kernel variant is chosen): the vector has at most one piece a thread (512 pieces), and the
// loop asks for one.
// PAUSE: whether attempts are spaced (see below); the merge of attention partials, which a few lines' worth of threads
// wait for, asks again at once.
template <bool SINGLE, bool PAUSE = true>
__device__ __forceinline__ void poll_batch(const f4* const (&ptr)[PB], f4 (&v)[PB], int n, Waiter& w) {
    static_assert(PB == 3, "the readiness word below names three pieces");
    long long t0 = 0;
    bool timing = false;
    if (n <= 0) return;
    if constexpr (SINGLE) {
        for (;;) {
            v[0] = ldx4(ptr[0]);
            if (!unset4(v[0]) || w.dead) break;
            if (!timing) { timing = true; t0 = wall_clock64(); }
            else if (wall_clock64() - t0 > w.limit) { w.fail(); break; }
            for (int z = 0; z < 4; z++) __builtin_amdgcn_s_sleep(2);
        }
        return;
    }
    for (;;) {
        ldx4_3(ptr, v);
        const unsigned missing = unset4(v[0]) | (n > 1 ? unset4(v[1]) : 0u) | (n > 2 ? unset4(v[2]) : 0u);
        if (!missing || w.dead) break;
        if (!timing) { timing = true; t0 = wall_clock64(); }
        else if (wall_clock64() - t0 > w.limit) { w.fail(); break; }
        // 256 workgroups re-reading a vector load the lines its producers are still storing to, so attempts are spaced;
        // the space is also the spread of the moments at which the workgroups notice the vector, and the phase ends with
        // the last of them.  512 clocks (~0.25 us): against 1024, 1.9 % of the step at the 0.5B shape (Q8), 0.45 % at 8B,
        // nothing at 0.5B Q4_0, -0.3 % at 1.1B; none at all and 256 are within 0.3 % of it at the 0.5B shape.
        if (PAUSE) for (int z = 0; z < 4; z++) __builtin_amdgcn_s_sleep(2);
    }
}

// Maxima and sums of up to PB KV splits of one head, all asked for in one round trip (a thread with fewer splits points
// the rest at the idle line and ignores them).
__device__ __forceinline__ void poll_ml(const float* const (&pm)[PB], const float* const (&pl)[PB], float (&m)[PB], float (&l)[PB], int n, Waiter& w) {
    static_assert(PB == 3, "three splits a round");
    long long t0 = 0;
    bool timing = false;
    for (;;) {
        asm volatile("global_load_dword %0, %6, off sc1\n\tglobal_load_dword %1, %7, off sc1\n\tglobal_load_dword %2, %8, off sc1\n\t"
                     "global_load_dword %3, %9, off sc1\n\tglobal_load_dword %4, %10, off sc1\n\tglobal_load_dword %5, %11, off sc1\n\t"
                     "s_waitcnt vmcnt(0)"
                     : "=&v"(m[0]), "=&v"(m[1]), "=&v"(m[2]), "=&v"(l[0]), "=&v"(l[1]), "=&v"(l[2])
                     : "v"(pm[0]), "v"(pm[1]), "v"(pm[2]), "v"(pl[0]), "v"(pl[1]), "v"(pl[2]) : "memory");
        const unsigned missing = unset1(m[0]) | unset1(l[0]) | (n > 1 ? unset1(m[1]) | unset1(l[1]) : 0u) | (n > 2 ? unset1(m[2]) | unset1(l[2]) : 0u);
        if (!missing || w.dead) break;
        if (!timing) { timing = true; t0 = wall_clock64(); }
        else if (wall_clock64() - t0 > w.limit) { w.fail(); break; }
    }
}
// The same for up to eight pieces (the 8B shape's down projection takes 14336 staged values: seven pieces a thread,
// three rounds of poll_batch -- three dependent round trips; this is one).
constexpr int PBW = 8;
__device__ __forceinline__ void ldx4_w(const f4* const (&p)[PBW], f4 (&v)[PBW], int n) {
    switch (n) {
    case 1:
        asm volatile("global_load_dwordx4 %0, %1, off sc1\n\ts_waitcnt vmcnt(0)"
                     : "=&v"(v[0]) : "v"(p[0]) : "memory");
        break;
    case 2:
        asm volatile("global_load_dwordx4 %0, %2, off sc1\n\tglobal_load_dwordx4 %1, %3, off sc1\n\ts_waitcnt vmcnt(0)"
                     : "=&v"(v[0]), "=&v"(v[1]) : "v"(p[0]), "v"(p[1]) : "memory");
        break;
    case 3:
        asm volatile("global_load_dwordx4 %0, %3, off sc1\n\tglobal_load_dwordx4 %1, %4, off sc1\n\tglobal_load_dwordx4 %2, %5, off sc1\n\ts_waitcnt vmcnt(0)"
                     : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]) : "v"(p[0]), "v"(p[1]), "v"(p[2]) : "memory");
        break;
    case 4:
        asm volatile("global_load_dwordx4 %0, %4, off sc1\n\tglobal_load_dwordx4 %1, %5, off sc1\n\tglobal_load_dwordx4 %2, %6, off sc1\n\tglobal_load_dwordx4 %3, %7, off sc1\n\ts_waitcnt vmcnt(0)"
                     : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3]) : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]) : "memory");
        break;
    case 5:
        asm volatile("global_load_dwordx4 %0, %5, off sc1\n\tglobal_load_dwordx4 %1, %6, off sc1\n\tglobal_load_dwordx4 %2, %7, off sc1\n\tglobal_load_dwordx4 %3, %8, off sc1\n\tglobal_load_dwordx4 %4, %9, off sc1\n\ts_waitcnt vmcnt(0)"
                     : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3]), "=&v"(v[4]) : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]), "v"(p[4]) : "memory");
        break;
    case 6:
        asm volatile("global_load_dwordx4 %0, %6, off sc1\n\tglobal_load_dwordx4 %1, %7, off sc1\n\tglobal_load_dwordx4 %2, %8, off sc1\n\tglobal_load_dwordx4 %3, %9, off sc1\n\tglobal_load_dwordx4 %4, %10, off sc1\n\tglobal_load_dwordx4 %5, %11, off sc1\n\ts_waitcnt vmcnt(0)"
                     : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3]), "=&v"(v[4]), "=&v"(v[5]) : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]), "v"(p[4]), "v"(p[5]) : "memory");
        break;
    case 7:
        asm volatile("global_load_dwordx4 %0, %7, off sc1\n\tglobal_load_dwordx4 %1, %8, off sc1\n\tglobal_load_dwordx4 %2, %9, off sc1\n\tglobal_load_dwordx4 %3, %10, off sc1\n\tglobal_load_dwordx4 %4, %11, off sc1\n\tglobal_load_dwordx4 %5, %12, off sc1\n\tglobal_load_dwordx4 %6, %13, off sc1\n\ts_waitcnt vmcnt(0)"
                     : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3]), "=&v"(v[4]), "=&v"(v[5]), "=&v"(v[6]) : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]), "v"(p[4]), "v"(p[5]), "v"(p[6]) : "memory");
        break;
    case 8:
        asm volatile("global_load_dwordx4 %0, %8, off sc1\n\tglobal_load_dwordx4 %1, %9, off sc1\n\tglobal_load_dwordx4 %2, %10, off sc1\n\tglobal_load_dwordx4 %3, %11, off sc1\n\tglobal_load_dwordx4 %4, %12, off sc1\n\tglobal_load_dwordx4 %5, %13, off sc1\n\tglobal_load_dwordx4 %6, %14, off sc1\n\tglobal_load_dwordx4 %7, %15, off sc1\n\ts_waitcnt vmcnt(0)"
                     : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3]), "=&v"(v[4]), "=&v"(v[5]), "=&v"(v[6]), "=&v"(v[7]) : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]), "v"(p[4]), "v"(p[5]), "v"(p[6]), "v"(p[7]) : "memory");
        break;
    default: break;
    }
}
template <int N>
__device__ __forceinline__ void poll_fixed_w(const f4* const (&ptr)[PBW], f4 (&v)[PBW], Waiter& w) {
    long long t0 = 0;
    bool timing = false;
    for (;;) {
        ldx4_w(ptr, v, N);
        unsigned missing = 0;
#pragma unroll
        for (int i = 0; i < N; i++) missing |= unset4(v[i]);
        if (!missing || w.dead) break;
        if (!timing) { timing = true; t0 = wall_clock64(); }
        else if (wall_clock64() - t0 > w.limit) { w.fail(); break; }
        for (int z = 0; z < 8; z++) __builtin_amdgcn_s_sleep(2);
    }
}
__device__ __forceinline__ void poll_batch_w(const f4* const (&ptr)[PBW], f4 (&v)[PBW], int n, Waiter& w) {
    static_assert(PBW == 8, "one case per batch size");
    switch (n < PBW ? n : PBW) {
    case 1: poll_fixed_w<1>(ptr, v, w); break;
    case 2: poll_fixed_w<2>(ptr, v, w); break;
    case 3: poll_fixed_w<3>(ptr, v, w); break;
    case 4: poll_fixed_w<4>(ptr, v, w); break;
    case 5: poll_fixed_w<5>(ptr, v, w); break;
    case 6: poll_fixed_w<6>(ptr, v, w); break;
    case 7: poll_fixed_w<7>(ptr, v, w); break;
    case 8: poll_fixed_w<8>(ptr, v, w); break;
    default: break;
    }
}

// planar LDS layout of an activation vector for 16-weight chunks (as the matvec kernels use): lane c reads
// a4[pl * nch + c], pl = 0..3.  Q8: a chunk is 16 consecutive weights, float4 k4 of the vector sits at
// (k4 & 3) * nch + (k4 >> 2).  Q4_0: a chunk is half a block (8 bytes: low nibbles = elements 8h..8h+7 of the block,
// high nibbles = elements 16+8h..16+8h+7), planes 0/1 its low-nibble float4s, planes 2/3 its high-nibble ones.
template <bool Q4>
__device__ __forceinline__ int slot4(int k4, int nch) {
    if (!Q4) return (k4 & 3) * nch + (k4 >> 2);
    const int blk = k4 >> 3, r4 = k4 & 7;
    return ((r4 >> 2) * 2 + (r4 & 1)) * nch + blk * 2 + ((r4 >> 1) & 1);
}
__device__ __forceinline__ float4 tof4(f4 v) { return make_float4(v.x, v.y, v.z, v.w); }

// x (optionally polled) -> LDS as x * gain; returns 1/rms.  Leaves with a barrier done.
// SINGLE: K <= 2048, one piece a thread
template <bool GL, bool Q4, bool SINGLE>
__device__ __forceinline__ float stage_rms(const float* x, bool polled, const float* gain, int K, float eps, float4* a4,
                                           float* red, Waiter& w) {
    const int K4 = K >> 2, nch = K >> 4, tid = threadIdx.x;
    const f4* x4 = reinterpret_cast<const f4*>(x);
    const float4* g4 = reinterpret_cast<const float4*>(gain);
    __syncthreads();                                   // the previous phase's readers of a4 are done
    float ss = 0.f;
    for (int base = 0; base < K4; base += FWG * PB) {
        f4 v[PB];
        float4 g[PB];
        const f4* ptr[PB];
#pragma unroll
        for (int u = 0; u < PB; u++) {
            const int i = base + u * FWG + tid;
            ptr[u] = i < K4 ? x4 + i : w.idle;
            g[u] = ldg_f4<GL>(g4, min(i, K4 - 1));
        }
        const int np = max(0, min(PB, (K4 - base - tid + FWG - 1) / FWG));      // this thread's pieces of the round
#pragma unroll
        for (int u = 0; u < PB; u++) v[u] = f4{0.f, 0.f, 0.f, 0.f};
        if (polled) {
            poll_batch<SINGLE>(ptr, v, np, w);
        } else {
#pragma unroll
            for (int u = 0; u < PB; u++) if (u < np) v[u] = *ptr[u];
        }
#pragma unroll
        for (int u = 0; u < PB; u++) {
            const int i = base + u * FWG + tid;
            if (i < K4) {
                ss += v[u].x * v[u].x + v[u].y * v[u].y + v[u].z * v[u].z + v[u].w * v[u].w;
                a4[slot4<Q4>(i, nch)] = make_float4(v[u].x * g[u].x, v[u].y * g[u].y, v[u].z * g[u].z, v[u].w * g[u].w);
            }
        }
    }
    ss = wave_sum(ss);
    if ((tid & 63) == 0) red[tid >> 6] = ss;
    __syncthreads();
    float tot = 0.f;
#pragma unroll
    for (int k = 0; k < FWAVES; k++) tot += red[k];
    return __builtin_amdgcn_rsqf(tot * __builtin_amdgcn_rcpf((float)K) + eps);
}

// polled x -> LDS.  Leaves with a barrier done.
template <bool Q4, bool SINGLE>
__device__ __forceinline__ void stage_plain(const float* x, int K, float4* a4, Waiter& w) {
    const int K4 = K >> 2, nch = K >> 4, tid = threadIdx.x;
    const f4* x4 = reinterpret_cast<const f4*>(x);
    __syncthreads();
    for (int base = 0; base < K4; base += FWG * PB) {
        f4 v[PB];
        const f4* ptr[PB];
#pragma unroll
        for (int u = 0; u < PB; u++) { const int i = base + u * FWG + tid; ptr[u] = i < K4 ? x4 + i : w.idle; v[u] = f4{0.f, 0.f, 0.f, 0.f}; }
        poll_batch<SINGLE>(ptr, v, max(0, min(PB, (K4 - base - tid + FWG - 1) / FWG)), w);
#pragma unroll
        for (int u = 0; u < PB; u++) {
            const int i = base + u * FWG + tid;
            if (i < K4) a4[slot4<Q4>(i, nch)] = tof4(v[u]);
        }
    }
    __syncthreads();
}

// stage_plain with up to eight pieces a thread in one round trip.
template <bool Q4>
__device__ __forceinline__ void stage_plain_w(const float* x, int K, float4* a4, Waiter& w) {
    const int K4 = K >> 2, nch = K >> 4, tid = threadIdx.x;
    const f4* x4 = reinterpret_cast<const f4*>(x);
    __syncthreads();
    for (int base = 0; base < K4; base += FWG * PBW) {
        f4 v[PBW];
        const f4* ptr[PBW];
#pragma unroll
        for (int u = 0; u < PBW; u++) { ptr[u] = x4 + min(base + u * FWG + tid, K4 - 1); v[u] = f4{0.f, 0.f, 0.f, 0.f}; }
        poll_batch_w(ptr, v, max(0, min(PBW, (K4 - base - tid + FWG - 1) / FWG)), w);
#pragma unroll
        for (int u = 0; u < PBW; u++) {
            const int i = base + u * FWG + tid;
            if (i < K4) a4[slot4<Q4>(i, nch)] = tof4(v[u]);
        }
    }
    __syncthreads();
}

// A weight row: Q8 16-byte chunks of int8; Q4_0 (split layout: all nibble groups of the matrix, then all fp16 d)
// 8-byte half blocks and the row of d, one per two chunks.
struct WRow { const signed char* w; const unsigned short* d; };

template <bool Q4>
__device__ __forceinline__ WRow wrow(const signed char* W, const float* aux, int r, int K) {
    if (Q4) return WRow{W + (size_t)r * (K >> 1), reinterpret_cast<const unsigned short*>(aux) + (size_t)r * (K >> 5)};
    return WRow{W + (size_t)r * K, nullptr};
}
// chunks c0 + lane + i*64 of a row (clamped inside the row: loads are unconditional); a Q4_0 chunk travels as
// {nibbles, nibbles, d bits, -}
template <bool GL, bool Q4, int CB>
__device__ __forceinline__ void ld_row(WRow row, int nch, int lane, int c0, int4 (&wr)[CB]) {
#pragma unroll
    for (int i = 0; i < CB; i++) {
        const int c = min(c0 + lane + i * 64, nch - 1);
        if (Q4) {
            const int2 q = ldg_i2<GL>(row.w, c);
            wr[i] = make_int4(q.x, q.y, (int)ldg_u16<GL>(row.d, c >> 1), 0);
        } else {
            wr[i] = ldg_i4<GL>(row.w, c);
        }
    }
}
template <bool Q4, int NR, int CB>
__device__ __forceinline__ void dot_rows(const int4 (&wr)[NR][CB], const float4* a4, int nch, int lane, int c0, float (&acc)[NR]) {
#pragma unroll
    for (int i = 0; i < CB; i++) {
        const int c = c0 + lane + i * 64;
        if (c < nch) {
            const float4 av[4] = {a4[c], a4[nch + c], a4[2 * nch + c], a4[3 * nch + c]};
            if (Q4) {
                const float asum = chunk_act_sum(av);
#pragma unroll
                for (int r = 0; r < NR; r++)
                    acc[r] = dot_q4_half(make_int2(wr[r][i].x, wr[r][i].y), half_bits_to_float((unsigned short)wr[r][i].z), av, asum, acc[r]);
            } else {
#pragma unroll
                for (int r = 0; r < NR; r++) {
                    float a = acc[r];
                    a = dot4_i8(wr[r][i].x, av[0], a); a = dot4_i8(wr[r][i].y, av[1], a);
                    a = dot4_i8(wr[r][i].z, av[2], a); a = dot4_i8(wr[r][i].w, av[3], a);
                    acc[r] = a;
                }
            }
        }
    }
}
// the same over the chunks [.., cHi) of a row only (a row shared by two waves); nch stays the stride of the staged planes
template <bool GL, bool Q4, int CB>
__device__ __forceinline__ void ld_row_rng(WRow row, int cHi, int lane, int c0, int4 (&wr)[CB]) {
#pragma unroll
    for (int i = 0; i < CB; i++) {
        const int c = min(c0 + lane + i * 64, cHi - 1);
        if (Q4) {
            const int2 q = ldg_i2<GL>(row.w, c);
            wr[i] = make_int4(q.x, q.y, (int)ldg_u16<GL>(row.d, c >> 1), 0);
        } else {
            wr[i] = ldg_i4<GL>(row.w, c);
        }
    }
}
template <bool Q4, int CB>
__device__ __forceinline__ float dot_row_rng(const int4 (&wr)[CB], const float4* a4, int nch, int cHi, int lane, int c0, float acc) {
#pragma unroll
    for (int i = 0; i < CB; i++) {
        const int c = c0 + lane + i * 64;
        if (c < cHi) {
            const float4 av[4] = {a4[c], a4[nch + c], a4[2 * nch + c], a4[3 * nch + c]};
            if (Q4) {
                acc = dot_q4_half(make_int2(wr[i].x, wr[i].y), half_bits_to_float((unsigned short)wr[i].z), av, chunk_act_sum(av), acc);
            } else {
                acc = dot4_i8(wr[i].x, av[0], acc); acc = dot4_i8(wr[i].y, av[1], acc);
                acc = dot4_i8(wr[i].z, av[2], acc); acc = dot4_i8(wr[i].w, av[3], acc);
            }
        }
    }
    return acc;
}
// the rest of rows longer than the prefetched batch
template <bool GL, bool Q4, int NR, int CB>
__device__ __forceinline__ void dot_rows_tail(const WRow (&rows)[NR], const float4* a4, int nch, int lane, float (&acc)[NR]) {
    for (int c0 = CB * 64; c0 < nch; c0 += CB * 64) {
        int4 wr[NR][CB];
#pragma unroll
        for (int r = 0; r < NR; r++) ld_row<GL, Q4, CB>(rows[r], nch, lane, c0, wr[r]);
        dot_rows<Q4, NR, CB>(wr, a4, nch, lane, c0, acc);
    }
}

// ---------------------------------------------------------------------------------------------------------------
// Prefetch role.  The last workgroups of the launch compute nothing: they read the rows that the computing
// workgroups of their own XCD are going to want, one phase to one layer ahead of them, so that those find their
// weights in the XCD's L2 instead of in HBM.  (The computing workgroups cannot do this for themselves: a CU's loads
// come back in order, so the polls of a hand-over would queue behind their own prefetch.)  The dispatcher places
// workgroup i on XCD i & 7; the eight waves of computing workgroup w take rows 8g .. 8g+7 of a matrix for every run
// g with g % nC == w, so with nC a multiple of 8 run g belongs to XCD g & 7.
// ---------------------------------------------------------------------------------------------------------------
// The fetches are loads straight into LDS (global_load_lds_dwordx4: 1 KB a wave and instruction, no destination
// register), all into one 1 KB scrap area that nothing reads: nothing the compiler allocates can be overwritten
// by a load that returns late, whatever it does with its registers between the issue and the wait.
struct Prefetcher {
    int x, rank, nRank, tid;     // XCD, this workgroup among the XCD's prefetchers, their number, thread
    int4* scrap;                 // LDS, 1 KB
    // bytes [b0, b1) of base, 16 bytes a thread and step; b0 a multiple of 16, the tail rounded down
    __device__ __forceinline__ void span(const char* base, size_t b0, size_t b1) {
        b1 &= ~(size_t)15;
        for (size_t o = b0 + (size_t)tid * 16; o < b1; o += (size_t)FWG * 16)
            __builtin_amdgcn_global_load_lds(reinterpret_cast<const int4*>(base + o), scrap, 16, 0, 0);
    }
    // runs of `run` rows of rowBytes each; run g of the matrix goes to XCD g & 7, then to the XCD's prefetchers in turn
    __device__ __forceinline__ void rows(const void* base, size_t rowBytes, int nRows, int run) {
        if (!base) return;
        const size_t total = (size_t)nRows * rowBytes, rb = (size_t)run * rowBytes;
        const int nRuns = (nRows + run - 1) / run;
        for (int g = x + 8 * rank; g < nRuns; g += 8 * nRank) {
            const size_t b0 = (size_t)g * rb;
            span(static_cast<const char*>(base), b0 & ~(size_t)15, b0 + rb < total ? b0 + rb : total);
        }
    }
    // a small array every workgroup of the XCD reads (scales, gains, biases): the XCD's first prefetcher takes it whole
    __device__ __forceinline__ void whole(const void* base, size_t bytes) {
        if (!base || rank != 0) return;
        span(static_cast<const char*>(base), 0, bytes);
    }
    // everything requested so far has landed (in the L2 on its way): nothing of it can arrive in the scrap area later
    __device__ __forceinline__ void drain() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
};

constexpr int FLOW_MAX_ROUNDS = 8;   // rows of a matrix a wave takes at most (rounds of all waves over the matrix)
constexpr int CBF = 6;       // ... per row of K = ffnDim (rows up to 6144 weights in one batch)
constexpr int NIB = 24 / FWAVES;   // gate/up items (a gate row and its up row) a wave holds in flight
constexpr int NID = 8 / FWAVES;    // down rows a wave holds in flight

// CBD: chunks a lane prefetches per row of K = dim (1: rows of up to 1024 weights in one batch, 2: up to 2048)
// RING: gate | up and down stream their rows through a ring of register sets (rows of more than 2048 weights)
// GQA: an attention workgroup takes all query heads of a KV head (contexts too long for one workgroup a query head)
// Q4: the seven matrices of a layer are Q4_0 in the split layout (the table's scale pointers then hold the d planes)
// TRACE: the launch records its per-workgroup timeline (FlowParams::trace); the variants without it carry neither the
//        trace points' instructions nor their scalar registers (1.2 % of the step at the 0.5B and 1.1B shapes)
// FIX: 0 = the sizes come with the launch; low three bits 1, 2, 3 = the sizes of a known model shape (FlowFixedShape) are
//      constants of the variant instead of launch parameters held in scalar registers and laundered at every token and layer:
//      addresses, trip counts and divisions fold (0.5B shape: 0.3294 -> 0.3231 ms a token).  Bit 8: the caches hold fp16 rows;
//      bit 16: the launch runs whole tokens (FlowParams::nTokens > 0).  Same formulas over the same rows; results agree with
//      the other variants' to rounding (the compiler contracts and schedules differently).  launch_flow_layers picks them.
struct FlowFixedShape { int dim, kvDim, ffn, nHeads, nKVHeads, headDim, downSplit, dedicated; };
__host__ __device__ constexpr FlowFixedShape flow_fixed_shape(int fix) {
    return fix == 1 ? FlowFixedShape{896, 128, 4864, 14, 2, 64, 1, 1}      // Qwen2.5-0.5B
         : fix == 2 ? FlowFixedShape{2048, 256, 5632, 32, 4, 64, 0, 0}     // TinyLlama-1.1B
         : fix == 3 ? FlowFixedShape{4096, 1024, 14336, 32, 8, 128, 0, 0}  // Llama-3-8B
                    : FlowFixedShape{0, 0, 0, 0, 0, 0, 0, 0};
}
// The part of a layer's exchange area whose layout follows from the sizes alone: q, current K row, current V row, hidden
// after attention, SwiGLU vector, layer output, merged attention output, and where the KV splits' partial slots begin.
__host__ __device__ constexpr FlowGeometry flow_geometry_head(int dim, int kvDim, int ffn) {
    FlowGeometry g{};
    int o = 0;
    g.offQ = o; o += (dim + 63) & ~63;
    g.offKc = o; o += (kvDim + 63) & ~63;
    g.offVc = o; o += (kvDim + 63) & ~63;
    g.offX1 = o; o += (dim + 63) & ~63;
    g.offM = o; o += (ffn + 63) & ~63;
    g.offX2 = o; o += (dim + 63) & ~63;
    g.offAttn = o; o += (dim + 63) & ~63;          // attention output merged over the splits (grouped attention only)
    g.offPacc = o;
    return g;
}

template <int HD, int CBD, bool RING, bool GQA, bool Q4, bool TRACE, int FIX = 0>
__global__ __launch_bounds__(FWG) void flow_layers_kernel(FlowParams p) {
    extern __shared__ float4 a4[];                     // the staged activation vector, max(dim, ffn) floats
    __shared__ float red[FWAVES];
    constexpr int QHMAX = GQA ? FLOW_GQA_MAX : 1;
    // Rows of up to 1024 weights are requested whole before a hand-over and multiplied after all of them have arrived:
    // no load is in flight across an LDS read, and the generic loads measure 1.6 % faster there (0.5B shape); longer
    // rows stream (remainders, rings), and the explicitly global loads measure 1.7 % (1.1B) and 2.7 % (8B) faster.
    constexpr bool GL = CBD > 1;
    __shared__ float4 sqkv[2 + QHMAX][HD / 4];         // K and V row of the current position, q of the workgroup's heads
    __shared__ float4 accbuf[QHMAX][FWAVES][HD / 4];   // per query head of the workgroup: the waves' partial outputs, sums, maxima
    __shared__ float lbuf[QHMAX][FWAVES], wred[QHMAX][FWAVES];
    __shared__ float outbuf[FLOW_MAX_ROUNDS][FWAVES];                // a phase's results of the workgroup, stored by one wave as whole 32-byte runs
    __shared__ int4 pfScrap[64];                       // where the prefetching loads land (never read)
    __shared__ float tailV[FWAVES];                    // the tail's argmax: the waves' best values and indices
    __shared__ int tailI[FWAVES];
    __shared__ unsigned tailCtr;                       // the tail's lm_head: next item of the workgroup to hand out (long rows)

    int tid = threadIdx.x, lane = tid & 63;
    int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nC = p.nCompute;                         // workgroups that compute; those after them prefetch
    int gw = blockIdx.x * FWAVES + wave;               // this wave among all computing waves of the launch
    const int W = nC * FWAVES;
    // The rows of a workgroup's eight waves are consecutive (row = base + wave + k W), so their results go out as runs
    // of eight floats in one store instruction of wave 0 instead of eight single-float stores from eight waves: a line
    // of a handed-over vector is then written 4 times, not 32, while 256 workgroups keep re-reading it.
    // Lane k < nk of every wave holds the value of its row k; all waves of the workgroup call this together.
    // rowOff: offset of this round's rows from the first round's (the same for all waves).
    auto store_runs = [&](float val, int nk, int nI, int rowOff, float* dst, float* dst2) {
        if (lane < nk) outbuf[lane][wave] = val;
        __syncthreads();
        if (wave == 0 && lane < nk * FWAVES) {
            const int k = lane / FWAVES, wv = lane % FWAVES;
            const int r = blockIdx.x * FWAVES + wv + k * W + rowOff;
            if (r < nI) {
                const float o = outbuf[k][wv];
                stx(dst + r, o);
                if (dst2) dst2[r] = o;
            }
        }
    };
    constexpr bool FX = FIX != 0;
    constexpr FlowFixedShape FS = flow_fixed_shape(FIX & 7);
    static_assert(!FX || FS.headDim == HD, "the fixed shape's head size is the variant's");
    int dim = FX ? FS.dim : p.dim, kvDim = FX ? FS.kvDim : p.kvDim, ffn = FX ? FS.ffn : p.ffn;
    const int nHeadsV = FX ? FS.nHeads : p.nHeads, nKVHeadsV = FX ? FS.nKVHeads : p.nKVHeads;
    // (known shapes: whether two waves share a row of the down projection follows from the sizes and the launch's 2048
    // waves; the caches hold fp32 rows unless the variant's code says fp16 -- both are branches between whole code paths)
    // Measured per variant, ms a token with / without: 0.5B Q8 0.3141 / 0.3230, 8B 1.558 / 1.561 (fp16 rows at 4,000
    // positions 1.841 / 1.847), 0.5B Q4_0 0.3235 / 0.3230, 1.1B 0.378 / 0.372 -- the last two keep them in registers.
    constexpr bool FXF = FX && (((FIX & 7) == 1 && !Q4) || (FIX & 7) == 3);
    constexpr bool FXD = FX && (FIX & 7) == 1;        // (0.5B Q4_0 0.3267 -> 0.3204 ms a token, Q8 0.3141 -> 0.3138; the others gain nothing)
    // whether workgroups past the computing ones prefetch (then none prefetches while idle during the attention): of the
    // two roles a known shape has one, the other's code is not in its variant
    const bool hasPrefetchers = FXD ? FS.dedicated != 0 : nC != (int)gridDim.x;
    // (1.1B: the row sharing alone as a constant 0.3734 -> 0.3695 ms a token, the row format alone 0.3818)
    const bool downSplitV = (FXF || (FIX & 7) == 2) ? FS.downSplit != 0 : p.downSplit != 0;
    const bool kvHalfV = FXF ? (FIX & 8) != 0 : p.kvHalf != 0;
    int nchD = dim >> 4, nchF = ffn >> 4;
    FlowGeometry G = p.geo;
    // (A known shape: these are constants, not scalar registers -- 0.5B Q4_0 0.330 -> 0.3235 ms a token, 1.1B 0.3755 -> 0.372,
    // 0.5B Q8 and 8B unchanged.)
    if constexpr (FX) {
        constexpr FlowGeometry GH = flow_geometry_head(FS.dim, FS.kvDim, FS.ffn);
        G.offQ = GH.offQ; G.offKc = GH.offKc; G.offVc = GH.offVc; G.offX1 = GH.offX1; G.offM = GH.offM; G.offX2 = GH.offX2;
        G.offAttn = GH.offAttn; G.offPacc = GH.offPacc;
    }
    // (the idle lines follow the error word's 256 bytes: 16 lines of 128 bytes, two workgroups of an XCD on each)
    Waiter wt{p.limitTicks, p.err, false, reinterpret_cast<const f4*>(reinterpret_cast<const char*>(p.err) + 256 + ((blockIdx.x >> 3) & 15) * 128)};

    // attention geometry (decode attention of kernels.hip with one query head per workgroup): a thread group of 16
    // lanes holds a K/V row, a thread VU rows of its workgroup's tile of FLOW_TILE positions.  (Measured on the 0.5B
    // shape at 100-200 positions: tiles of 128 beat 256 by 5 %, and beat 64 and 32, whose extra partials cost more to
    // merge than the rows save; a kernel that can also take tiles of 256 is 2-3 % slower at every context for the
    // unrolled code alone.)
    constexpr int LPR = 16, NF = HD / 64, TG = FWG / LPR, VU = FLOW_TILE / TG, TILE = FLOW_TILE;
    const int half = HD >> 1;

    // timing trace (diagnostic): slot b of layer l, per workgroup, in ticks of the 100 MHz wall clock
#define FLOW_TRACE(b) do { if constexpr (TRACE) { if (p.trace && tid == 0 && (int)blockIdx.x < nC) \
        p.trace[((size_t)(l - p.l0) * FLOW_TRACE_SLOTS + (b)) * nC + blockIdx.x] = wall_clock64(); } } while (0)
    // the exchange area as a buffer resource: agent-scope loads that the compiler keeps track of (used where many are
    // wanted in flight together)
    const __amdgpu_buffer_rsrc_t xrsrc = __builtin_amdgcn_make_buffer_rsrc(p.xchg, 0, (int)((size_t)p.nLayersTotal * G.stride * 4 * (p.nTokens > 0 ? 2 : 1)), 0x00020000);
    unsigned lw = layer_words(p.layers, p.l0, lane);

    // Token mode (p.nTokens > 0): the launch runs whole tokens -- the embedding of the token in the device state, all
    // layers, and the tail (final norm, lm_head, greedy argmax; cuda_fused_infer.go:446-450 and what the reference's
    // caller does with the logits), nTokens of them, every token's successor chosen on the device.  The exchange area
    // then has two halves, used by even and by odd positions: during a token's tail all workgroups reset the other
    // half for the token after it.  (Nothing of the token before is read any more once a workgroup has got there:
    // every workgroup reads every workgroup's argmax partial, so a token starts only when all are through the last.)
    // (known shapes, bit 16 of FIX: the launch runs whole tokens -- the layers-only form's code is not in the variant)
    const bool tokens = (FIX & 16) ? true : p.nTokens > 0;
    const int nTok = tokens ? p.nTokens : 1;
    const unsigned tw = tokens ? tail_words(p.tail, lane) : 0u;
    int pos = p.state ? p.state->pos : p.posImm;
    int tok = tokens ? p.state->token : 0;
    const int count0 = tokens ? p.state->count : 0, nPrompt = tokens ? p.state->nPrompt : 0;
    const size_t halfFloats = (size_t)p.nLayersTotal * G.stride;
    float* const xemb = reinterpret_cast<float*>(a4) + (dim > ffn ? dim : ffn);      // the token's embedding (token mode)
    for (int tk = 0; tk < nTok; tk++) {
        // Nothing that depends on the thread or on the shape is to be computed once for all tokens and kept in registers
        // across the whole launch (hundreds of addresses and offsets otherwise are): every token derives them again.
        asm volatile("" : "+v"(tid), "+v"(lane));
        if constexpr (FX) asm volatile("" : "+s"(wave), "+s"(gw));
        else asm volatile("" : "+s"(wave), "+s"(gw), "+s"(dim), "+s"(kvDim), "+s"(ffn), "+s"(nchD), "+s"(nchF));
        float* const xb = p.xchg + (tokens ? (size_t)(pos & 1) * halfFloats : (size_t)0);
        const unsigned xoff = tokens ? (unsigned)((size_t)(pos & 1) * halfFloats) : 0u;
        if constexpr (!GQA) {
            // the plain variant on a geometry laid out for grouped attention: a position past what a workgroup per query head
            // and split covers is the host's mistake, and is reported instead of computed wrongly
            if (G.gqa && nHeadsV * (pos / TILE + 1) > nC && blockIdx.x == 0 && tid == 0)
                __hip_atomic_store(p.err, 3, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        const float* cosRow = p.cosRow;
        const float* sinRow = p.sinRow;
        if (tokens) {
            cosRow = TW_PTR(const float, cosTab) + (size_t)pos * half;
            sinRow = TW_PTR(const float, sinTab) + (size_t)pos * half;
            const void* et = TW_PTR(const void, embTable);
            const float* es = TW_PTR(const float, embScales);
            const int ek = TW_INT(embKind), vocab = TW_INT(vocab);
            __syncthreads();                               // the token before has no reader of xemb left
            const int tc = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
            for (int i = tid; i < dim; i += FWG) xemb[i] = embed_value(ek, et, es, tc, dim, vocab, i);
            __syncthreads();
        }

        if (hasPrefetchers && (int)blockIdx.x >= nC) {
            // ---- prefetch role (see Prefetcher): per layer three jobs, each released by a vector of the layer before ----
            const int pi = (int)blockIdx.x - nC;
            Prefetcher pf{pi & 7, pi >> 3, ((int)gridDim.x - nC) >> 3, tid, pfScrap};
            const size_t rbD = Q4 ? dim >> 1 : dim, rbF = Q4 ? ffn >> 1 : ffn;      // bytes of a row of dim / of ffn weights
            const size_t rdD = dim >> 4, rdF = ffn >> 4;                             // ... of its fp16 d values (Q4_0)
            const int halfHd = HD >> 1;
            for (int l = p.l0; l < p.l1; l++) {
                LayerView L{lw};
                if (l + 1 < p.l1) lw = layer_words(p.layers, l + 1, lane);
                else if (tk + 1 < nTok) lw = layer_words(p.layers, p.l0, lane);
                const float* Xp = xb + (size_t)(l - 1) * G.stride;               // the layer before (not for the first)
                // (Measured at the 0.5B shape: releasing every job a phase earlier or later, and 24 to 48 prefetching
                // workgroups, all give the same step time within 0.5 %; 16 are too few, 64 cost more than they bring.)
                auto release = [&](int off) {
                    pf.drain();                // the job before has landed
                    if (l == p.l0) return;
                    if (tid == 0) (void)poll1(Xp + off, wt);
                    __syncthreads();
                };
                release(G.offX1);              // the layer before is past its Wo: q | k | v and Wo of this one
                {
                    const int nq = dim >> 1, nk = kvDim >> 1, nI = nq + 2 * nk;
                    for (int g = pf.x + 8 * pf.rank; g * 8 < nI; g += 8 * pf.nRank) {
                        const int item = g * 8;
                        const signed char* Wm; const float* aux; int a0, a1;
                        if (item < nq) { Wm = L.wq(); aux = L.sq(); const int jj = item % halfHd; a0 = (item - jj) * 2 + jj; a1 = a0 + halfHd; }
                        else if (item < nq + nk) { Wm = L.wk(); aux = L.sk(); const int i2 = item - nq; const int jj = i2 % halfHd; a0 = (i2 - jj) * 2 + jj; a1 = a0 + halfHd; }
                        else { Wm = L.wv(); aux = L.sv(); a0 = (item - nq - nk) * 2; a1 = a0 + 8; }
                        const char* wb = reinterpret_cast<const char*>(Wm);
                        pf.span(wb, (size_t)a0 * rbD, (size_t)(a0 + 8) * rbD);
                        pf.span(wb, (size_t)a1 * rbD, (size_t)(a1 + 8) * rbD);
                        if (Q4) {
                            const char* db = reinterpret_cast<const char*>(aux);
                            pf.span(db, ((size_t)a0 * rdD) & ~(size_t)15, (size_t)(a0 + 8) * rdD);
                            pf.span(db, ((size_t)a1 * rdD) & ~(size_t)15, (size_t)(a1 + 8) * rdD);
                        }
                    }
                    if (!Q4) { pf.whole(L.sq(), (size_t)dim * 4); pf.whole(L.sk(), (size_t)kvDim * 4); pf.whole(L.sv(), (size_t)kvDim * 4); }
                    pf.whole(L.bq(), (size_t)dim * 4); pf.whole(L.bk(), (size_t)kvDim * 4); pf.whole(L.bv(), (size_t)kvDim * 4);
                    pf.whole(L.g1(), (size_t)dim * 4);
                    pf.rows(L.wo(), rbD, dim, 8);
                    if (Q4) pf.rows(L.so(), rdD, dim, 8); else pf.whole(L.so(), (size_t)dim * 4);
                    // the K / V rows of the earlier positions (the attention workgroups of every XCD read them; the row of the
                    // current position comes through the exchange area), while they are a small part of an L2: 0.5B shape at
                    // positions 16 .. 216 0.3766 -> 0.3710 ms a token
                    const size_t kvBytes = (size_t)pos * kvDim * (kvHalfV ? 2 : 4);
                    if (kvBytes <= ((size_t)512 << 10)) { pf.whole(L.Kc(), kvBytes); pf.whole(L.Vc(), kvBytes); }
                }
                release(G.offM);               // ... past its gate | up: gate | up of this one
                pf.rows(L.gate(), rbD, ffn, 8);
                pf.rows(L.up(), rbD, ffn, 8);
                if (Q4) { pf.rows(L.sgate(), rdD, ffn, 8); pf.rows(L.sup(), rdD, ffn, 8); }
                else { pf.whole(L.sgate(), (size_t)ffn * 4); pf.whole(L.sup(), (size_t)ffn * 4); }
                pf.whole(L.g2(), (size_t)dim * 4);
                release(G.offX2);              // ... done: the down projection of this one
                const int drun = downSplitV ? FWAVES / 2 : FWAVES;      // rows of the down projection a workgroup takes
                pf.rows(L.down(), rbF, dim, drun);
                if (Q4) pf.rows(L.sdown(), rdF, dim, drun); else pf.whole(L.sdown(), (size_t)dim * 4);
            }
            pf.drain();
        } else {
            for (int l = p.l0; l < p.l1; l++) {
                // (the same per layer: offsets that do not depend on the layer would otherwise be kept across all phases, and
                // the phases' own working sets then no longer fit the registers)
                asm volatile("" : "+v"(tid), "+v"(lane));
                if constexpr (FX) asm volatile("" : "+s"(wave), "+s"(gw));
        else asm volatile("" : "+s"(wave), "+s"(gw), "+s"(dim), "+s"(kvDim), "+s"(ffn), "+s"(nchD), "+s"(nchF));
                LayerView L{lw};
                if (l + 1 < p.l1) lw = layer_words(p.layers, l + 1, lane);
                else if (tk + 1 < nTok) lw = layer_words(p.layers, p.l0, lane);
                FLOW_TRACE(0);
                float* X = xb + (size_t)l * G.stride;
                const bool first = l == p.l0;
                const float* xin = first ? (tokens ? xemb : p.hidden) : xb + (size_t)(l - 1) * G.stride + G.offX2;

                // ------------------------------------------------------------------ q | k | v
                {
                    const int nq = dim >> 1, nk = kvDim >> 1, nI = nq + 2 * nk;       // RoPE pairs of q, of k; row pairs of v
                    if (blockIdx.x * FWAVES < nI) {
                        // The first NPI items of a wave are requested whole (CBQ chunks a lane and row) before the input is waited for;
                        // further items, and chunks past CBQ, are read where they are used.
                        constexpr int NPI = 1, CBQ = CBD;
                        int4 wr[NPI][2][CBQ];
                        WRow rows[NPI][2];
                        int kind[NPI], r0[NPI], r1[NPI];
                        float e0[NPI], e1[NPI];                  // per-lane epilogue operands: lanes 0/1 scale and bias, lane 2 cos and sin
                        auto resolve = [&](int4 (&w)[2][CBQ], WRow (&rw)[2], int& kd, int& a0, int& a1, float& f0, float& f1, int item) {
                            const signed char* Wm; const float* sc; const float* bias;
                            if (item < nq) { kd = 0; Wm = L.wq(); sc = L.sq(); bias = L.bq(); const int jj = item % half; a0 = (item - jj) * 2 + jj; a1 = a0 + half; }
                            else if (item < nq + nk) { kd = 1; Wm = L.wk(); sc = L.sk(); bias = L.bk(); const int i2 = item - nq; const int jj = i2 % half; a0 = (i2 - jj) * 2 + jj; a1 = a0 + half; }
                            else { kd = 2; Wm = L.wv(); sc = L.sv(); bias = L.bv(); a0 = (item - nq - nk) * 2; a1 = a0 + 1; }
                            rw[0] = wrow<Q4>(Wm, sc, a0, dim); rw[1] = wrow<Q4>(Wm, sc, a1, dim);
                            ld_row<GL, Q4, CBQ>(rw[0], nchD, lane, 0, w[0]);
                            ld_row<GL, Q4, CBQ>(rw[1], nchD, lane, 0, w[1]);
                            f0 = 1.f; f1 = 0.f;
                            if (lane < 2) {
                                const int r = lane ? a1 : a0;
                                if (!Q4) f0 = ldg_f<GL>(sc, r);
                                if (bias) f1 = ldg_f<GL>(bias, r);
                            }
                            if (lane == 2 && kd < 2) { const int jj = a0 % half; f0 = cosRow[jj]; f1 = sinRow[jj]; }
                        };
                        // the pair of every wave of the workgroup (lane 0: both values) out as runs by wave 0; `it` the wave's item
                        auto put_pair = [&](float o0, float o1, int it) {
                            // the eight waves' rows are consecutive (first rows of the pairs, and second rows)
                            if (it != gw) __syncthreads();              // outbuf is free again
                            if (lane == 0) { outbuf[0][wave] = o0; outbuf[1][wave] = o1; }
                            __syncthreads();
                            if (wave == 0 && lane < 2 * FWAVES) {
                                const int k = lane / FWAVES, wv = lane % FWAVES, item = it + wv;
                                if (item < nI) {
                                    int kk, a0, a1;
                                    if (item < nq) { kk = 0; const int jj = item % half; a0 = (item - jj) * 2 + jj; a1 = a0 + half; }
                                    else if (item < nq + nk) { kk = 1; const int i2 = item - nq; const int jj = i2 % half; a0 = (i2 - jj) * 2 + jj; a1 = a0 + half; }
                                    else { kk = 2; a0 = (item - nq - nk) * 2; a1 = a0 + 1; }
                                    const int r = k ? a1 : a0;
                                    const float o = outbuf[k][wv];
                                    if (kk == 0) {
                                        stx(X + G.offQ + r, o);
                                    } else {                                              // mongoose.cu:1644-1647, and the hand-over copy
                                        // (write-through: the next token of the same launch reads the row on other XCDs)
                                        float oc = o;
                                        if (kvHalfV) {           // fp16 rows: rounded where written; the hand-over copy carries the rounded value
                                            const _Float16 hv = (_Float16)o;
                                            oc = (float)hv;
                                            const _Float16* dst = reinterpret_cast<const _Float16*>(kk == 1 ? L.Kc() : L.Vc()) + (size_t)pos * kvDim + r;
                                            const unsigned bits = __builtin_bit_cast(unsigned short, hv);
                                            asm volatile("global_store_short %0, %1, off sc1" : : "v"(dst), "v"(bits) : "memory");
                                        } else {
                                            st_agent((kk == 1 ? L.Kc() : L.Vc()) + (size_t)pos * kvDim + r, o);
                                        }
                                        stx(X + (kk == 1 ? G.offKc : G.offVc) + r, oc);
                                    }
                                }
                            }
                        };
                        // one item of every wave of the workgroup: dot, epilogue, the results out as runs by wave 0
                        auto finish = [&](const int4 (&w)[2][CBQ], const WRow (&rw)[2], int kd, float f0, float f1, float rs, int it) {
                            float acc[2] = {0.f, 0.f};
                            dot_rows<Q4, 2, CBQ>(w, a4, nchD, lane, 0, acc);
                            if (nchD > CBQ * 64) dot_rows_tail<GL, Q4, 2, CBQ>(rw, a4, nchD, lane, acc);
                            const float t = wave_sum2(acc[0], acc[1]);
                            float v = lane == 1 ? lane_value(t, 32) : t;
                            v = v * f0;                                                  // row scale (lanes 0 and 1)
                            v = v * rs;
                            v = v + f1;
                            const float v1 = dpp_f<0x101>(v);                            // lane 0 reads lane 1: the pair's second row
                            const float cs = dpp_f<0x102>(f0), sn = dpp_f<0x102>(f1);    // lane 0 reads lane 2
                            float o0 = v, o1 = v1;
                            if (kd < 2) { o0 = v * cs - v1 * sn; o1 = v * sn + v1 * cs; }            // mongoose.cu:991-1006
                            put_pair(o0, o1, it);
                        };
                        if constexpr (RING) {
                            // Rows of more than 2048 weights: a wave's items (one or two row pairs of 16 KB at the 8B shape) stream
                            // through a ring of register sets in steps of 2 x 128 chunks, as gate | up's rows do, two steps
                            // requested before the input is waited for and every later one two steps ahead of its use.  Requested
                            // whole-or-not-at-all (half of the first pair ahead, the rest where it is used) the phase ran into one
                            // HBM latency after the other: 2 % of the 8B shape's step.
                            // (Measured and not kept: single rows as items, dealt round the waves evenly -- three rows a wave at
                            // the 8B shape instead of two pairs on half the waves and one on the others -- with the pairs' halves
                            // meeting in LDS for the rotation.  HBM is shared by the whole chip, so the waves with two pairs speed
                            // up once the others are done, and a third round of barriers and stores costs more than the balance
                            // brings: 1.648 against 1.638 ms a token at 8B, +5 % at the 1.1B shape, whose pairs fit one round and
                            // whose rows need two.)
                            constexpr int RD = 3, CB = 2;
                            int4 ring[RD][2][CB];
                            float ef0[RD], ef1[RD];                  // the step's item's epilogue operands, as e0 / e1 above
                            const int nRounds = (nI - (int)blockIdx.x * FWAVES + W - 1) / W;      // items of the workgroup's first wave
                            const int nb = (nchD + 64 * CB - 1) / (64 * CB);
                            const int T = nRounds * nb;
                            auto issueStep = [&](int4 (&set)[2][CB], float& f0, float& f1, int st) {
                                const int sc2 = min(st, T - 1);                      // past the end: the last step again (uniform loop)
                                const int k = sc2 / nb, b = sc2 - k * nb;
                                const int item = min(gw + k * W, nI - 1);            // (a wave past the last item repeats it and stores nothing)
                                const signed char* Wm; const float* sc; const float* bias; int kd, a0, a1;
                                if (item < nq) { kd = 0; Wm = L.wq(); sc = L.sq(); bias = L.bq(); const int jj = item % half; a0 = (item - jj) * 2 + jj; a1 = a0 + half; }
                                else if (item < nq + nk) { kd = 1; Wm = L.wk(); sc = L.sk(); bias = L.bk(); const int i2 = item - nq; const int jj = i2 % half; a0 = (i2 - jj) * 2 + jj; a1 = a0 + half; }
                                else { kd = 2; Wm = L.wv(); sc = L.sv(); bias = L.bv(); a0 = (item - nq - nk) * 2; a1 = a0 + 1; }
                                ld_row<true, Q4, CB>(wrow<Q4>(Wm, sc, a0, dim), nchD, lane, b * CB * 64, set[0]);
                                ld_row<true, Q4, CB>(wrow<Q4>(Wm, sc, a1, dim), nchD, lane, b * CB * 64, set[1]);
                                f0 = 1.f; f1 = 0.f;
                                if (lane < 2) {
                                    const int r = lane ? a1 : a0;
                                    if (!Q4) f0 = ldg_f<true>(sc, r);
                                    if (bias) f1 = ldg_f<true>(bias, r);
                                }
                                if (lane == 2 && kd < 2) { const int jj = a0 % half; f0 = ldg_f<true>(cosRow, jj); f1 = ldg_f<true>(sinRow, jj); }
                            };
#pragma unroll
                            for (int j = 0; j < RD - 1; j++) issueStep(ring[j], ef0[j], ef1[j], j);
                            const float rs = stage_rms<GL, Q4, false>(xin, !first, L.g1(), dim, p.eps, a4, red, wt);
                            FLOW_TRACE(1);
                            float acc[2] = {0.f, 0.f};
                            for (int s0 = 0; s0 < T; s0 += RD) {
#pragma unroll
                                for (int j = 0; j < RD; j++) {
                                    const int st = s0 + j;
                                    issueStep(ring[(j + RD - 1) % RD], ef0[(j + RD - 1) % RD], ef1[(j + RD - 1) % RD], st + RD - 1);
                                    if (st < T) {                                        // uniform in the workgroup
                                        const int k = st / nb, b = st - k * nb;
                                        dot_rows<Q4, 2, CB>(ring[j], a4, nchD, lane, b * CB * 64, acc);
                                        if (b == nb - 1) {
                                            const int it = gw + k * W;
                                            const int kd = it < nq ? 0 : (it < nq + nk ? 1 : 2);
                                            const float t = wave_sum2(acc[0], acc[1]);
                                            acc[0] = 0.f; acc[1] = 0.f;
                                            float v = lane == 1 ? lane_value(t, 32) : t;
                                            v = v * ef0[j];
                                            v = v * rs;
                                            v = v + ef1[j];
                                            const float v1 = dpp_f<0x101>(v);
                                            const float cs = dpp_f<0x102>(ef0[j]), sn = dpp_f<0x102>(ef1[j]);
                                            float o0 = v, o1 = v1;
                                            if (kd < 2) { o0 = v * cs - v1 * sn; o1 = v * sn + v1 * cs; }            // mongoose.cu:991-1006
                                            put_pair(o0, o1, it);
                                        }
                                    }
                                }
                            }
                        } else {
#pragma unroll
                        for (int q = 0; q < NPI; q++) {
                            kind[q] = 0; r0[q] = 0; r1[q] = 0; e0[q] = 0.f; e1[q] = 0.f; rows[q][0] = wrow<Q4>(L.wq(), L.sq(), 0, dim); rows[q][1] = rows[q][0];
                            if (gw + q * W < nI) resolve(wr[q], rows[q], kind[q], r0[q], r1[q], e0[q], e1[q], gw + q * W);
                        }
                        const float rs = stage_rms<GL, Q4, !RING>(xin, !first, L.g1(), dim, p.eps, a4, red, wt);
                        FLOW_TRACE(1);
#pragma unroll
                        for (int q = 0; q < NPI; q++)
                            if (blockIdx.x * FWAVES + q * W < nI) finish(wr[q], rows[q], kind[q], e0[q], e1[q], rs, gw + q * W);      // uniform in the workgroup
                        for (int it = gw + NPI * W; it - wave < nI; it += W) {         // it - wave: the same for all waves of the workgroup
                            if (it < nI) resolve(wr[0], rows[0], kind[0], r0[0], r1[0], e0[0], e1[0], it);
                            finish(wr[0], rows[0], kind[0], e0[0], e1[0], rs, it);
                        }
                        }
                    }
                }

                FLOW_TRACE(2);
                // ------------------------------------------------------------------ attention: one (head, KV split) per workgroup
                // grouped only while a workgroup per query head and split would not fit the launch (positions far into a long context)
                const bool grouped = GQA && nHeadsV * (pos / TILE + 1) > nC;
                {
                    const int nsplit = pos / TILE + 1;
                    // Grouped: the query heads of a KV head are shared out over as many workgroups as the launch has left for
                    // them at this position (each loads the K / V rows once and takes its heads in turn), so a workgroup takes as
                    // few heads as possible: qhMax heads a workgroup, `sub` workgroups a KV head and split.
                    const int Gq = nHeadsV / nKVHeadsV;
                    int qhMax = 1, sub = Gq;
                    if (grouped) {
                        qhMax = Gq; sub = 1;
                        const int live = nsplit < G.smax ? nsplit : G.smax;
                        for (int q = 2; q < Gq; q++) {
                            const int sb = (Gq + q - 1) / q;
                            if (nKVHeadsV * sb * live <= nC) { qhMax = q; sub = sb; break; }
                        }
                    }
                    const int unit = grouped ? nKVHeadsV * sub : nHeadsV;
                    const int split = blockIdx.x / unit, hu = blockIdx.x % unit;
                    const int hg = grouped ? hu % sub : 0;                         // which of the KV head's groups of query heads
                    const int QH = grouped ? min(qhMax, Gq - hg * qhMax) : 1;      // query heads of this workgroup
                    // Workgroups with no attention to do (and no partials to merge per head) read, into their XCD's L2, rows that the
                    // XCD's workgroups will want after it -- their next poll, for the attention's partials, is microseconds away, and
                    // HBM would be idle meanwhile.  p.idleWoRows: Wo (rows of more than 2048 weights, of which a wave requests only
                    // the first half-row ahead); p.idleGateUpRows: the leading rows of gate and of up -- all of them where both
                    // matrices fit the L2s (1.1B shape: 0.465 -> 0.436 ms a token; the down projection on top overflows the L2s:
                    // 0.470), else half of the first round of rows, which is what a phase waits for before it streams (8B shape
                    // with both: 1.845 -> 1.790; the whole first round 1.804, a quarter 1.800).
                    // Only while at least half the launch is idle (short contexts), and only without dedicated prefetchers.
                    if (!hasPrefetchers && (p.idleWoRows > 0 || p.idleGateUpRows > 0)) {
                        const int live = nsplit < G.smax ? nsplit : G.smax;
                        int nBusy = unit * live;
                        if (grouped && nBusy < nHeadsV) nBusy = nHeadsV;
                        nBusy = (nBusy + 7) & ~7;
                        if ((int)blockIdx.x >= nBusy && 2 * ((int)gridDim.x - nBusy) >= (int)gridDim.x) {
                            Prefetcher pf{(int)blockIdx.x & 7, ((int)blockIdx.x - nBusy) >> 3, ((int)gridDim.x - nBusy) >> 3, tid, pfScrap};
                            const size_t rbD = Q4 ? dim >> 1 : dim, rdD = dim >> 4;
                            // (a workgroup without q | k | v rows gets here at the top of the layer; holding it back until q | k | v is
                            // through measures slower: 1.1B shape 0.453 against 0.435 ms a token)
                            if (p.idleWoRows > 0) {
                                pf.rows(L.wo(), rbD, p.idleWoRows, 8);
                                if (Q4) pf.rows(L.so(), rdD, p.idleWoRows, 8);
                            }
                            if (p.idleGateUpRows > 0) {
                                pf.rows(L.gate(), rbD, p.idleGateUpRows, 8);
                                pf.rows(L.up(), rbD, p.idleGateUpRows, 8);
                                if (Q4) { pf.rows(L.sgate(), rdD, p.idleGateUpRows, 8); pf.rows(L.sup(), rdD, p.idleGateUpRows, 8); }
                            }
                            pf.drain();
                        }
                    }
                    if (split < G.smax && split < nsplit) {
                        const int kvh = grouped ? hu / sub : hu / Gq;
                        const int h0 = grouped ? kvh * Gq + hg * qhMax : hu;
                        const int tg = tid / LPR, dl = tid % LPR;
                        const int t0 = split * TILE;
                        const int len = pos + 1;
                        const int t1 = min(len, t0 + TILE);
                        const size_t rowStride = (size_t)kvDim / 4;
                        const size_t colOff = (size_t)(kvh * HD) / 4 + dl;
                        const float4* Kc4 = reinterpret_cast<const float4*>(L.Kc());
                        const float4* Vc4 = reinterpret_cast<const float4*>(L.Vc());
                        float4 kreg[VU][NF], vreg[VU][NF];
                        // Only rows of earlier positions are read from the caches (the current one comes through the exchange
                        // area, the loads of later ones go to the idle line): a cache line is never fetched into an L2 before its
                        // row has been written -- in token mode that row is written later in this same launch, by a workgroup of
                        // another XCD, and a line fetched early would be served stale from then on.
                        const float4* idle4 = reinterpret_cast<const float4*>(wt.idle) + dl;
                        if (kvHalfV) {
                            // fp16 rows: a lane's piece is four halves (8 bytes), widened as it arrives
                            typedef _Float16 h4 __attribute__((ext_vector_type(4)));
                            const int2* Kh = reinterpret_cast<const int2*>(L.Kc());
                            const int2* Vh = reinterpret_cast<const int2*>(L.Vc());
                            const int2* idle2 = reinterpret_cast<const int2*>(wt.idle) + dl;
                            auto widen = [](int2 b) {
                                const h4 h = __builtin_bit_cast(h4, b);
                                return make_float4((float)h[0], (float)h[1], (float)h[2], (float)h[3]);
                            };
#pragma unroll
                            for (int u = 0; u < VU; u++) {
                                const int row = t0 + tg + u * TG;
                                const size_t ro = (size_t)row * rowStride + colOff;
                                const int2* kp = row < pos ? Kh + ro : idle2;
                                const int2* vp = row < pos ? Vh + ro : idle2;
#pragma unroll
                                for (int j = 0; j < NF; j++) kreg[u][j] = widen(ldg_i2<GL>(kp, j * 16));
#pragma unroll
                                for (int j = 0; j < NF; j++) vreg[u][j] = widen(ldg_i2<GL>(vp, j * 16));
                            }
                        } else {
#pragma unroll
                        for (int u = 0; u < VU; u++) {
                            const int row = t0 + tg + u * TG;
                            const size_t ro = (size_t)row * rowStride + colOff;
                            const float4* kp = row < pos ? Kc4 + ro : idle4;
                            const float4* vp = row < pos ? Vc4 + ro : idle4;
#pragma unroll
                            for (int j = 0; j < NF; j++) kreg[u][j] = ldg_f4<GL>(kp, j * 16);
#pragma unroll
                            for (int j = 0; j < NF; j++) vreg[u][j] = ldg_f4<GL>(vp, j * 16);
                        }
                        }
                        __syncthreads();
                        if (tid < (2 + QH) * (HD / 4)) {
                            const int which = tid / (HD / 4), i = tid % (HD / 4);
                            const float* src = which >= 2 ? X + G.offQ + (h0 + which - 2) * HD : X + (which == 0 ? G.offKc : G.offVc) + kvh * HD;
                            sqkv[which][i] = tof4(poll4(reinterpret_cast<const f4*>(src) + i, wt));
                        }
                        __syncthreads();
                        FLOW_TRACE(3);
                        const int live = t1 - t0;
                        const float scale = 1.0f / sqrtf((float)HD);
#pragma unroll
                        for (int u = 0; u < VU; u++) {
                            if (t0 + tg + u * TG == pos) {          // the current position's rows come from this launch, not from the cache
#pragma unroll
                                for (int j = 0; j < NF; j++) { kreg[u][j] = sqkv[0][j * 16 + dl]; vreg[u][j] = sqkv[1][j * 16 + dl]; }
                            }
                        }
                        for (int hi = 0; hi < QH; hi++) {          // the heads of the KV head in turn, on the same K / V registers
                        float4 q4[NF];
#pragma unroll
                        for (int j = 0; j < NF; j++) q4[j] = sqkv[2 + hi][j * 16 + dl];
                        float sc[VU];
                        float tmax = -INFINITY;
#pragma unroll
                        for (int u = 0; u < VU; u++) {
                            sc[u] = -INFINITY;
                            if (u * TG >= live) continue;
                            const int row = t0 + tg + u * TG;
                            float d = 0.f;
#pragma unroll
                            for (int j = 0; j < NF; j++) {
                                d = fmaf(q4[j].x, kreg[u][j].x, d); d = fmaf(q4[j].y, kreg[u][j].y, d);
                                d = fmaf(q4[j].z, kreg[u][j].z, d); d = fmaf(q4[j].w, kreg[u][j].w, d);
                            }
                            d = row_sum16(d);
                            sc[u] = row < t1 ? d * scale : -INFINITY;
                            tmax = fmaxf(tmax, sc[u]);
                        }
                        const float m = tg_max(tmax);               // the wave's maximum
                        const float mRef = m == -INFINITY ? 0.f : m;
                        float4 acc[NF];
#pragma unroll
                        for (int j = 0; j < NF; j++) acc[j] = make_float4(0.f, 0.f, 0.f, 0.f);
                        float lsum = 0.f;
#pragma unroll
                        for (int u = 0; u < VU; u++) {
                            if (u * TG >= live) continue;
                            const float pv = exp_neg(sc[u] - mRef);
                            lsum += pv;
#pragma unroll
                            for (int j = 0; j < NF; j++) {
                                acc[j].x = fmaf(pv, vreg[u][j].x, acc[j].x); acc[j].y = fmaf(pv, vreg[u][j].y, acc[j].y);
                                acc[j].z = fmaf(pv, vreg[u][j].z, acc[j].z); acc[j].w = fmaf(pv, vreg[u][j].w, acc[j].w);
                            }
                        }
#pragma unroll
                        for (int j = 0; j < NF; j++) {
                            acc[j].x = tg_sum(acc[j].x); acc[j].y = tg_sum(acc[j].y); acc[j].z = tg_sum(acc[j].z); acc[j].w = tg_sum(acc[j].w);
                            if (lane < LPR) accbuf[hi][wave][j * 16 + dl] = acc[j];
                        }
                        lsum = tg_sum(lsum);
                        if (lane == 0) { lbuf[hi][wave] = lsum; wred[hi][wave] = m; }
                        }
                        // the waves' partials of all the workgroup's heads combined together: one barrier, a thread per head and piece
                        __syncthreads();
                        if (tid < QH * (HD / 4)) {
                            const int hq = tid / (HD / 4), i = tid % (HD / 4), h = h0 + hq;
                            float mg_ = wred[hq][0];
#pragma unroll
                            for (int k = 1; k < FWAVES; k++) mg_ = fmaxf(mg_, wred[hq][k]);
                            f4 r = {0.f, 0.f, 0.f, 0.f};
                            float lg = 0.f;
#pragma unroll
                            for (int k = 0; k < FWAVES; k++) {
                                const float wk = exp_neg(wred[hq][k] - mg_);
                                const float4 a = accbuf[hq][k][i];
                                r.x = fmaf(wk, a.x, r.x); r.y = fmaf(wk, a.y, r.y); r.z = fmaf(wk, a.z, r.z); r.w = fmaf(wk, a.w, r.w);
                                lg = fmaf(wk, lbuf[hq][k], lg);
                            }
                            stx4(reinterpret_cast<f4*>(X + G.offPacc + (size_t)split * dim + h * HD) + i, r);
                            if (i == 0) {
                                stx(X + G.offPm + split * nHeadsV + h, mg_);
                                stx(X + G.offPl + split * nHeadsV + h, lg);
                            }
                        }
                    }
                }

                if (grouped) {
                    // Long contexts, tens of KV splits: merged once per head, by workgroup h for head h (every thread a 16-byte piece
                    // and every eighth split, eight splits' loads in flight together, then combined through LDS), and handed on as
                    // one vector -- every consumer merging all partials itself re-reads tens of KB per workgroup and layer.
                    if ((int)blockIdx.x < nHeadsV) {
                        constexpr int P4 = HD / 4, SG = FWG / P4;          // pieces of a head, split groups (thread = piece x group)
                        __shared__ float4 mnum[SG][P4];
                        __shared__ float mM[SG][P4], mden[SG][P4];
                        const int h = blockIdx.x, i = tid % P4, sg = tid / P4;
                        const int ns = min(pos / TILE + 1, G.smax);
                        const unsigned Xo = xoff + (unsigned)l * G.stride;
                        float M = -INFINITY, den = 0.f;
                        f4 num = {0.f, 0.f, 0.f, 0.f};
                        constexpr int MBG = 4;
                        for (int s1 = sg; s1 < ns; s1 += SG * MBG) {
                            f4 a[MBG];
                            float ms[MBG], ls[MBG];
                            long long t0w = 0;
                            bool timing = false;
                            for (;;) {
                                unsigned missing = 0;
#pragma unroll
                                for (int j = 0; j < MBG; j++) {
                                    const int sj = min(s1 + j * SG, ns - 1);
                                    a[j] = __builtin_bit_cast(f4, __builtin_amdgcn_raw_buffer_load_b128(xrsrc, (Xo + G.offPacc + (unsigned)sj * dim + h * HD + i * 4) * 4u, 0, 16));
                                    ms[j] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xrsrc, (Xo + G.offPm + sj * nHeadsV + h) * 4u, 0, 16));
                                    ls[j] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xrsrc, (Xo + G.offPl + sj * nHeadsV + h) * 4u, 0, 16));
                                }
#pragma unroll
                                for (int j = 0; j < MBG; j++) missing |= unset4(a[j]) | unset1(ms[j]) | unset1(ls[j]);
                                if (!missing || wt.dead) break;
                                if (!timing) { timing = true; t0w = wall_clock64(); }
                                else if (wall_clock64() - t0w > wt.limit) { wt.fail(); break; }
                                for (int z = 0; z < 4; z++) __builtin_amdgcn_s_sleep(2);
                            }
#pragma unroll
                            for (int j = 0; j < MBG; j++) {
                                if (s1 + j * SG < ns) {
                                    const float Mn = fmaxf(M, ms[j]);
                                    const float c = exp_neg(M - Mn), wgt = exp_neg(ms[j] - Mn);
                                    den = den * c + wgt * ls[j];
                                    num.x = num.x * c + wgt * a[j].x; num.y = num.y * c + wgt * a[j].y;
                                    num.z = num.z * c + wgt * a[j].z; num.w = num.w * c + wgt * a[j].w;
                                    M = Mn;
                                }
                            }
                        }
                        mnum[sg][i] = tof4(num); mM[sg][i] = M; mden[sg][i] = den;
                        __syncthreads();
                        if (tid < P4) {
                            float Mg = mM[0][tid];
                            for (int g2 = 1; g2 < SG; g2++) Mg = fmaxf(Mg, mM[g2][tid]);
                            float dn = 0.f;
                            f4 nm = {0.f, 0.f, 0.f, 0.f};
                            for (int g2 = 0; g2 < SG; g2++) {
                                const float wgt = exp_neg(mM[g2][tid] - Mg);     // a group without splits has M = -inf: weight 0
                                const float4 a = mnum[g2][tid];
                                dn = fmaf(wgt, mden[g2][tid], dn);
                                nm.x = fmaf(wgt, a.x, nm.x); nm.y = fmaf(wgt, a.y, nm.y); nm.z = fmaf(wgt, a.z, nm.z); nm.w = fmaf(wgt, a.w, nm.w);
                            }
                            const float il = __builtin_amdgcn_rcpf(dn);
                            stx4(reinterpret_cast<f4*>(X + G.offAttn + h * HD) + tid, f4{nm.x * il, nm.y * il, nm.z * il, nm.w * il});
                        }
                    }
                }
                FLOW_TRACE(4);
                // ------------------------------------------------------------------ Wo + residual
                {
                    const int nI = dim;
                    if (blockIdx.x * FWAVES < nI) {
                        int it = gw;
                        int4 wr[1][CBD];
                        WRow rows[1] = {wrow<Q4>(L.wo(), L.so(), 0, dim)};
                        float e0 = 0.f, e1 = 0.f;
                        auto resolve = [&](int item) {
                            rows[0] = wrow<Q4>(L.wo(), L.so(), item, dim);
                            ld_row<GL, Q4, CBD>(rows[0], nchD, lane, 0, wr[0]);
                            if (lane == 0) {
                                e0 = Q4 ? 1.f : ldg_f<GL>(L.so(), item);
                                e1 = first ? xin[item] : poll1(xin + item, wt);         // there already if this workgroup staged it for q | k | v
                            }
                        };
                        // (Long rows streamed through a register ring here as in q | k | v, two steps requested ahead of the merge,
                        // measure 1.6 % slower at the 8B shape: the merge's polls wait for every load issued before them, and a
                        // whole row in flight from HBM holds them up longer than the half row does.)
                        if (it < nI) resolve(it);
                        // stage the attention output: merge the KV splits' partials (running maximum, as the split-KV combine)
                        if (grouped) {
                            stage_plain<Q4, !RING>(X + G.offAttn, dim, a4, wt);      // merged per head above
                        } else {
                        __syncthreads();
                        {
                            const int nsplit = pos / TILE + 1;
                            const int ns = nsplit < G.smax ? nsplit : G.smax;
                            for (int i = tid; i < (dim >> 2); i += FWG) {
                                const int h = (i * 4) / HD;
                                float M = -INFINITY, den = 0.f;
                                f4 num = {0.f, 0.f, 0.f, 0.f};
                                auto mergeIn = [&](f4 a, float ms, float ls) {
                                    const float Mn = fmaxf(M, ms);
                                    const float c = exp_neg(M - Mn);                        // first split: exp(-inf) = 0
                                    const float wgt = exp_neg(ms - Mn);
                                    den = den * c + wgt * ls;
                                    num.x = num.x * c + wgt * a.x; num.y = num.y * c + wgt * a.y;
                                    num.z = num.z * c + wgt * a.z; num.w = num.w * c + wgt * a.w;
                                    M = Mn;
                                };
                                // Up to PB splits a round: their accumulator pieces are waited for together (they are spread
                                // over many lines), then their maxima and sums are fetched together, once the accumulators are
                                // there -- all heads' maxima and sums of a split share a line, and a line that 50,000 threads
                                // keep re-reading takes its producer's store late (asked for in the same round as the
                                // accumulators, by every thread and every attempt, they cost the 0.5B shape 2 us a layer).
                                // Two round trips after the last partial has landed, however many splits (one by one they
                                // were one more per split: 4 % of the step at 1000 positions).
                                const float* idle1 = reinterpret_cast<const float*>(wt.idle);
                                if (ns == 1) {                             // uniform in the launch; one split: no loads to spare
                                    f4 a;
                                    float ms, ls;
                                    const f4* pa = reinterpret_cast<const f4*>(X + G.offPacc) + i;
                                    a = poll4(pa, wt);
                                    poll_partial(pa, X + G.offPm + h, X + G.offPl + h, a, ms, ls, wt);
                                    mergeIn(a, ms, ls);
                                } else
                                for (int s0 = 0; s0 < ns; s0 += PB) {
                                    const int nbt = min(PB, ns - s0);
                                    const f4* pa[PB];
                                    const float* pm[PB];
                                    const float* pl[PB];
                                    f4 a[PB];
                                    float ms[PB], ls[PB];
#pragma unroll
                                    for (int u = 0; u < PB; u++) {
                                        const bool on = u < nbt;
                                        pa[u] = on ? reinterpret_cast<const f4*>(X + G.offPacc + (size_t)(s0 + u) * dim) + i : wt.idle;
                                        pm[u] = on ? X + G.offPm + (s0 + u) * nHeadsV + h : idle1;
                                        pl[u] = on ? X + G.offPl + (s0 + u) * nHeadsV + h : idle1;
                                        a[u] = f4{0.f, 0.f, 0.f, 0.f};
                                    }
                                    poll_batch<false, false>(pa, a, nbt, wt);
                                    poll_ml(pm, pl, ms, ls, nbt, wt);
#pragma unroll
                                    for (int u = 0; u < PB; u++) if (u < nbt) mergeIn(a[u], ms[u], ls[u]);
                                }
                                const float il = __builtin_amdgcn_rcpf(den);
                                a4[slot4<Q4>(i, nchD)] = make_float4(num.x * il, num.y * il, num.z * il, num.w * il);
                            }
                        }
                        __syncthreads();
                        }
                        FLOW_TRACE(5);
                        for (; it < nI; it += W) {
                            if (it != gw) resolve(it);
                            float acc[1] = {0.f};
                            dot_rows<Q4, 1, CBD>(wr, a4, nchD, lane, 0, acc);
                            if (nchD > CBD * 64) dot_rows_tail<GL, Q4, 1, CBD>(rows, a4, nchD, lane, acc);
                            const float v = wave_sum(acc[0]);
                            if (it != gw) __syncthreads();              // outbuf is free again
                            store_runs(e1 + v * e0, 1, nI, it - gw, X + G.offX1, nullptr);
                        }
                    }
                }

                FLOW_TRACE(6);
                // ------------------------------------------------------------------ gate | up, SiLU(g) * u
                {
                    const int nI = ffn;
                    if constexpr (RING) {
                        // Long rows, several items a wave: the rows stream through a ring of register sets, the loads of step
                        // s + RD - 1 are issued before step s is multiplied (a step = one item's two rows x CB chunks a lane).
                        if (blockIdx.x * FWAVES < nI) {
                            constexpr int RD = 3, CB = 2;
                            int4 ring[RD][2][CB];
                            const int nItems = gw < nI ? (nI - gw + W - 1) / W : 0;
                            const int nb = (nchD + 64 * CB - 1) / (64 * CB);
                            const int T = nItems * nb;
                            auto issueStep = [&](int4 (&set)[2][CB], int st) {
                                const int sc = min(st, T - 1);                       // past the end: the last step again (uniform loop)
                                const int k = sc / nb, b = sc - k * nb;
                                const int row = gw + k * W;
                                ld_row<GL, Q4, CB>(wrow<Q4>(L.gate(), L.sgate(), row, dim), nchD, lane, b * CB * 64, set[0]);
                                ld_row<GL, Q4, CB>(wrow<Q4>(L.up(), L.sup(), row, dim), nchD, lane, b * CB * 64, set[1]);
                            };
                            float sg = 0.f, su = 0.f;
                            if (T > 0) {
#pragma unroll
                                for (int j = 0; j < RD - 1; j++) issueStep(ring[j], j);
                                if (lane < nItems) { const int r = gw + lane * W; sg = Q4 ? 1.f : ldg_f<GL>(L.sgate(), r); su = Q4 ? 1.f : ldg_f<GL>(L.sup(), r); }
                            }
                            const float rs = stage_rms<GL, Q4, !RING>(X + G.offX1, true, L.g2(), dim, p.eps, a4, red, wt);
                            FLOW_TRACE(7);
                            float acc[2] = {0.f, 0.f};
                            float g = 0.f, u = 0.f;
                            for (int s0 = 0; s0 < T; s0 += RD) {
#pragma unroll
                                for (int j = 0; j < RD; j++) {
                                    const int st = s0 + j;
                                    issueStep(ring[(j + RD - 1) % RD], st + RD - 1);
                                    if (st < T) {                                        // uniform in the wave
                                        const int k = st / nb, b = st - k * nb;
                                        dot_rows<Q4, 2, CB>(ring[j], a4, nchD, lane, b * CB * 64, acc);
                                        if (b == nb - 1) {
                                            const float t = wave_sum2(acc[0], acc[1]);
                                            const float v0 = lane_value(t, 0), v1 = lane_value(t, 32);
                                            if (lane == k) { g = v0; u = v1; }
                                            acc[0] = 0.f; acc[1] = 0.f;
                                        }
                                    }
                                }
                            }
                            g = g * sg; g = g * rs;
                            u = u * su; u = u * rs;
                            const float sig = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-g * 1.4426950408889634f));   // mongoose.cu:949-956
                            store_runs(g * sig * u, (nI + W - 1) / W, nI, 0, X + G.offM, nullptr);
                        }
                    } else
                    if (blockIdx.x * FWAVES < nI) {
                        int4 wr[NIB][2][CBD];
                        float sg = 0.f, su = 0.f;
                        auto issue = [&](int it0) {
#pragma unroll
                            for (int k = 0; k < NIB; k++) {
                                const int r = it0 + k * W;
                                if (r < nI) {                                           // uniform in the wave
                                    ld_row<GL, Q4, CBD>(wrow<Q4>(L.gate(), L.sgate(), r, dim), nchD, lane, 0, wr[k][0]);
                                    ld_row<GL, Q4, CBD>(wrow<Q4>(L.up(), L.sup(), r, dim), nchD, lane, 0, wr[k][1]);
                                }
                            }
                            if (lane < NIB) { const int r = min(it0 + lane * W, nI - 1); sg = Q4 ? 1.f : ldg_f<GL>(L.sgate(), r); su = Q4 ? 1.f : ldg_f<GL>(L.sup(), r); }
                        };
                        if (gw < nI) issue(gw);
                        const float rs = stage_rms<GL, Q4, !RING>(X + G.offX1, true, L.g2(), dim, p.eps, a4, red, wt);
                        FLOW_TRACE(7);
                        for (int it0 = gw; it0 < nI; it0 += NIB * W) {
                            if (it0 != gw) issue(it0);
                            float g = 0.f, u = 0.f;
#pragma unroll
                            for (int k = 0; k < NIB; k++) {
                                float acc[2] = {0.f, 0.f};
                                if (it0 + k * W < nI) {                                 // uniform in the wave
                                    dot_rows<Q4, 2, CBD>(wr[k], a4, nchD, lane, 0, acc);
                                    if (nchD > CBD * 64) {
                                        const int r = it0 + k * W;
                                        const WRow rows[2] = {wrow<Q4>(L.gate(), L.sgate(), r, dim), wrow<Q4>(L.up(), L.sup(), r, dim)};
                                        dot_rows_tail<GL, Q4, 2, CBD>(rows, a4, nchD, lane, acc);
                                    }
                                    const float t = wave_sum2(acc[0], acc[1]);
                                    acc[0] = lane_value(t, 0);
                                    acc[1] = lane_value(t, 32);
                                }
                                if (lane == k) { g = acc[0]; u = acc[1]; }
                            }
                            g = g * sg; g = g * rs;
                            u = u * su; u = u * rs;
                            const float sig = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-g * 1.4426950408889634f));   // mongoose.cu:949-956
                            if (it0 != gw) __syncthreads();             // outbuf is free again
                            store_runs(g * sig * u, NIB, nI, it0 - gw, X + G.offM, nullptr);
                        }
                    }
                }

                FLOW_TRACE(8);
                // ------------------------------------------------------------------ down + residual
                {
                    const int nI = dim;
                    if constexpr (RING) {
                        if (blockIdx.x * FWAVES < nI) {
                            constexpr int RD = 3, CB = 4;
                            int4 ring[RD][1][CB];
                            const int nItems = gw < nI ? (nI - gw + W - 1) / W : 0;
                            const int nb = (nchF + 64 * CB - 1) / (64 * CB);
                            const int T = nItems * nb;
                            auto issueStep = [&](int4 (&set)[1][CB], int st) {
                                const int sc = min(st, T - 1);
                                const int k = sc / nb, b = sc - k * nb;
                                ld_row<GL, Q4, CB>(wrow<Q4>(L.down(), L.sdown(), gw + k * W, ffn), nchF, lane, b * CB * 64, set[0]);
                            };
                            float e0 = 0.f, e1 = 0.f;
                            if (T > 0) {
                                if (lane < nItems) { const int r = gw + lane * W; e0 = Q4 ? 1.f : ldg_f<GL>(L.sdown(), r); e1 = poll1(X + G.offX1 + r, wt); }
#pragma unroll
                                for (int j = 0; j < RD - 1; j++) issueStep(ring[j], j);
                            }
                            stage_plain_w<Q4>(X + G.offM, ffn, a4, wt);
                            FLOW_TRACE(9);
                            float acc[1] = {0.f};
                            float v = 0.f;
                            for (int s0 = 0; s0 < T; s0 += RD) {
#pragma unroll
                                for (int j = 0; j < RD; j++) {
                                    const int st = s0 + j;
                                    issueStep(ring[(j + RD - 1) % RD], st + RD - 1);
                                    if (st < T) {                                        // uniform in the wave
                                        const int k = st / nb, b = st - k * nb;
                                        dot_rows<Q4, 1, CB>(ring[j], a4, nchF, lane, b * CB * 64, acc);
                                        if (b == nb - 1) {
                                            const float v0 = wave_sum(acc[0]);
                                            if (lane == k) v = v0;
                                            acc[0] = 0.f;
                                        }
                                    }
                                }
                            }
                            store_runs(e1 + v * e0, (nI + W - 1) / W, nI, 0, X + G.offX2, l == p.l1 - 1 ? p.hidden : nullptr);
                        }
                    } else if (downSplitV) {
                        // Few rows (at most half as many as computing waves): a row is shared by two neighbouring waves of a
                        // workgroup, each taking half of its chunks, and every workgroup with rows has half as many -- the
                        // multiplications of this phase, its longest rows, take half as long (0.5B shape 0.366 -> 0.360 ms a
                        // token).  One round.
                        if ((int)blockIdx.x * (FWAVES / 2) < nI) {
                            constexpr int CBH = CBF / 2;
                            const int row = min(gw >> 1, nI - 1), hf = wave & 1;
                            const int nHalf = (nchF + 1) >> 1;
                            const int c0 = hf ? nHalf : 0, cHi = hf ? nchF : nHalf;
                            const WRow rw = wrow<Q4>(L.down(), L.sdown(), row, ffn);
                            int4 wr[CBH];
                            ld_row_rng<GL, Q4, CBH>(rw, cHi, lane, c0, wr);
                            float e0 = 0.f, e1 = 0.f;
                            if (wave == 0 && lane < FWAVES / 2) {
                                const int r = min((int)blockIdx.x * (FWAVES / 2) + lane, nI - 1);
                                e0 = Q4 ? 1.f : ldg_f<GL>(L.sdown(), r);
                                e1 = poll1(X + G.offX1 + r, wt);
                            }
                            stage_plain<Q4, false>(X + G.offM, ffn, a4, wt);
                            FLOW_TRACE(9);
                            float acc = dot_row_rng<Q4, CBH>(wr, a4, nchF, cHi, lane, c0, 0.f);
                            for (int cc = c0 + CBH * 64; cc < cHi; cc += CBH * 64) {
                                ld_row_rng<GL, Q4, CBH>(rw, cHi, lane, cc, wr);
                                acc = dot_row_rng<Q4, CBH>(wr, a4, nchF, cHi, lane, cc, acc);
                            }
                            acc = wave_sum(acc);
                            if (lane == 0) outbuf[0][wave] = acc;
                            __syncthreads();
                            if (wave == 0 && lane < FWAVES / 2) {
                                const int r = (int)blockIdx.x * (FWAVES / 2) + lane;
                                if (r < nI) {
                                    const float o = e1 + (outbuf[0][2 * lane] + outbuf[0][2 * lane + 1]) * e0;
                                    stx(X + G.offX2 + r, o);
                                    if (l == p.l1 - 1) p.hidden[r] = o;
                                }
                            }
                        }
                    } else
                    if (blockIdx.x * FWAVES < nI) {
                        int4 wr[NID][1][CBF];
                        float e0 = 0.f, e1 = 0.f;
                        auto issue = [&](int it0) {
#pragma unroll
                            for (int k = 0; k < NID; k++) {
                                const int r = it0 + k * W;
                                if (r < nI) ld_row<GL, Q4, CBF>(wrow<Q4>(L.down(), L.sdown(), r, ffn), nchF, lane, 0, wr[k][0]);      // uniform in the wave
                            }
                            if (lane < NID) { const int r = min(it0 + lane * W, nI - 1); e0 = Q4 ? 1.f : ldg_f<GL>(L.sdown(), r); e1 = poll1(X + G.offX1 + r, wt); }
                        };
                        if (gw < nI) issue(gw);
                        stage_plain<Q4, false>(X + G.offM, ffn, a4, wt);
                        FLOW_TRACE(9);
                        for (int it0 = gw; it0 < nI; it0 += NID * W) {
                            if (it0 != gw) issue(it0);
                            float v = 0.f;
#pragma unroll
                            for (int k = 0; k < NID; k++) {
                                float acc[1] = {0.f};
                                if (it0 + k * W < nI) {
                                    dot_rows<Q4, 1, CBF>(wr[k], a4, nchF, lane, 0, acc);
                                    if (nchF > CBF * 64) {
                                        const WRow rows[1] = {wrow<Q4>(L.down(), L.sdown(), it0 + k * W, ffn)};
                                        dot_rows_tail<GL, Q4, 1, CBF>(rows, a4, nchF, lane, acc);
                                    }
                                    acc[0] = wave_sum(acc[0]);
                                }
                                if (lane == k) v = acc[0];
                            }
                            if (it0 != gw) __syncthreads();             // outbuf is free again
                            store_runs(e1 + v * e0, NID, nI, it0 - gw, X + G.offX2, l == p.l1 - 1 ? p.hidden : nullptr);
                        }
                    }
                }
                FLOW_TRACE(10);
            }
        }

        if (tokens) {
            // ---------------------------------------------------------------------------------------------- the tail
            // All workgroups of the launch, the prefetching ones included.  Rows of the lm_head in items of NRT, item g to
            // wave g % WA; a wave's items stream through a ring of register sets as gate | up's do.
            const int l = p.l1;                             // (trace: the tail is recorded as one more layer)
            FLOW_TRACE(0);
            const int np = pos + 1;
            const int gwA = blockIdx.x * FWAVES + wave, WA = (int)gridDim.x * FWAVES;
            const signed char* lmW = TW_PTR(const signed char, lmW);
            const float* lmAux = TW_PTR(const float, lmAux);
            const int vocab = TW_INT(vocab);
            float* logits = TW_PTR(float, logits);
            float* amax = TW_PTR(float, amax);
            constexpr int NRT = (RING || CBD > 1) ? 2 : 4, CBT = RING ? 2 : CBD, RDT = 3;
            int4 ring[RDT][NRT][CBT];
            float scl[RDT];
            const int nItemsAll = (vocab + NRT - 1) / NRT;
            float bestV = -INFINITY;
            int bestI = INT_MAX;
            float acc[NRT];
#pragma unroll
            for (int i = 0; i < NRT; i++) acc[i] = 0.f;
            // an item's NRT sums -> logits and the lane's running best; lane i < NRT ends up with row r0 + i
            auto finishItem = [&](int r0, float sc, float rs) {
                float val;
                if constexpr (NRT == 4) {
                    const float t01 = wave_sum2(acc[0], acc[1]), t23 = wave_sum2(acc[2], acc[3]);
                    val = lane_value(t01, 0);
                    if (lane == 1) val = lane_value(t01, 32);
                    if (lane == 2) val = lane_value(t23, 0);
                    if (lane == 3) val = lane_value(t23, 32);
                } else {
                    const float t01 = wave_sum2(acc[0], acc[1]);
                    val = lane_value(t01, 0);
                    if (lane == 1) val = lane_value(t01, 32);
                }
                val = val * sc;
                val = val * rs;
                const int r = r0 + lane;
                if (lane < NRT && r < vocab) {
                    stg_f<true>(logits, (size_t)r, val);
                    if (val > bestV || (val == bestV && r < bestI)) { bestV = val; bestI = r; }
                }
#pragma unroll
                for (int i = 0; i < NRT; i++) acc[i] = 0.f;
            };
            auto resetOther = [&]() {
                // the other half of the exchange area, and this workgroup's argmax slot there, for the token after this one
                const f4 sent = {__builtin_bit_cast(float, XSENT), __builtin_bit_cast(float, XSENT), __builtin_bit_cast(float, XSENT), __builtin_bit_cast(float, XSENT)};
                f4* o4 = reinterpret_cast<f4*>(p.xchg + (size_t)(np & 1) * halfFloats);
                for (size_t i = (size_t)blockIdx.x * FWG + tid; i < halfFloats / 4; i += (size_t)gridDim.x * FWG)
                    asm volatile("global_store_dwordx4 %0, %1, off sc1" : : "v"(o4 + i), "v"(sent) : "memory");
                if (tid == 0) {
                    st_agent(amax + ((size_t)(np & 1) * gridDim.x + blockIdx.x) * FLOW_AMAX_STRIDE, sent.x);
                    st_agent(amax + ((size_t)(np & 1) * gridDim.x + blockIdx.x) * FLOW_AMAX_STRIDE + 1, sent.x);
                }
            };
            const float* xfin = xb + (size_t)(p.l1 - 1) * G.stride + G.offX2;
            // A wave's items (item g to wave g % WA) stream through the ring in steps, as gate | up's rows do, through
            // explicitly global loads whatever the layers' phases use: the ring's loads stay in flight across the LDS reads
            // of the steps before them, and the hand-over before the loop does not wait for the first steps' rows (generic
            // loads here cost the 0.5B shape 2.5 % of its step).
            // Measured and not kept, both at the 0.5B shape: handing the items of a workgroup out to its waves as they fall
            // free, from a counter in LDS (the waves of a workgroup then end together, but the launch ends when its slowest
            // workgroup does, 2-3 us after the mean, as before: 0.3511 against 0.3475 ms a token); and handing the last fifth
            // of the items out across workgroups, from counters bumped by atomics that stay in an XCD's L2, one claim an item
            // made a step ahead of its use.  Atomics on one address complete at some 40 a microsecond: one counter an XCD
            // (256 waves) made the phase 15 us longer, eight an XCD brought the last workgroup 1.5 us closer to the median
            // and still cost 1.7 % of the step against this static mapping (0.3481 against 0.3422 ms).
            const int nb = (nchD + 64 * CBT - 1) / (64 * CBT);
            if constexpr (RING) {
                // Rows of more than 2048 weights (8B shape: 100 us of lm_head): the items of a workgroup -- its waves' first,
                // second, ... items by the mapping above, numbered q = 8 round + slot -- are handed to its waves as they fall
                // free, from a counter in LDS, after the two that every wave requests before the input is waited for.  The
                // waves of a workgroup then end within one item of each other; by the fixed mapping the last wave of the
                // median workgroup ended 13 us after its first.  (Shorter rows: 2 % slower at the 0.5B shape, 12 % with Q4_0
                // matrices, 0.4 % faster at 1.1B -- the fixed mapping stays there.)
                if (tid == 0) tailCtr = 2 * FWAVES;                   // (stage_rms below has a barrier before any wave claims)
                auto itemOf = [&](int q) { return (int)blockIdx.x * FWAVES + (q & (FWAVES - 1)) + (q / FWAVES) * WA; };
                int gI = itemOf(wave), bI = 0, taken = 1;             // the step to issue next: item, block of columns
                int gS[RDT], bS[RDT];
                auto issueStep = [&](int4 (&set)[NRT][CBT], float& sc, int& gs, int& bs) {
                    gs = gI; bs = bI;
                    const int r0 = min(gI, nItemsAll - 1) * NRT;      // past the end: the last item again (uniform loop)
#pragma unroll
                    for (int i = 0; i < NRT; i++)
                        ld_row<true, Q4, CBT>(wrow<Q4>(lmW, lmAux, min(r0 + i, vocab - 1), dim), nchD, lane, bI * CBT * 64, set[i]);
                    sc = Q4 ? 1.f : ldg_f<true>(lmAux, min(r0 + (lane < NRT ? lane : 0), vocab - 1));
                    if (++bI == nb) {
                        bI = 0;
                        if (gI < nItemsAll) {                             // (a wave stops at its first item past the end: later claims are later items)
                            int q = FWAVES * taken + wave;
                            if (taken >= 2) {
                                unsigned c = 0;
                                if (lane == 0) c = __hip_atomic_fetch_add(&tailCtr, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                                q = __builtin_amdgcn_readfirstlane((int)c);
                            }
                            gI = itemOf(q);
                            taken++;
                        }
                    }
                };
#pragma unroll
                for (int j = 0; j < RDT - 1; j++) issueStep(ring[j], scl[j], gS[j], bS[j]);
                resetOther();
                const float rs = stage_rms<GL, Q4, !RING>(xfin, true, TW_PTR(const float, finalGain), dim, p.eps, a4, red, wt);
                FLOW_TRACE(1);
                // (The loop is left at the bottom of a whole round of the ring only: with a way out after every step, the
                // compiler's count of the loads in flight at the top of a round would be that of the shortest way there, and
                // its waits would drain the ring.  A wave whose items end inside a round issues the round's other steps idle.)
                for (bool more = true; more;) {
#pragma unroll
                    for (int j = 0; j < RDT; j++) {
                        constexpr int RDTm = RDT - 1;
                        issueStep(ring[(j + RDTm) % RDT], scl[(j + RDTm) % RDT], gS[(j + RDTm) % RDT], bS[(j + RDTm) % RDT]);
                        if (gS[j] < nItemsAll) {                             // uniform in the wave
                            dot_rows<Q4, NRT, CBT>(ring[j], a4, nchD, lane, bS[j] * CBT * 64, acc);
                            if (bS[j] == nb - 1) finishItem(gS[j] * NRT, scl[j], rs);
                        }
                    }
                    more = gS[RDT - 1] < nItemsAll;
                }
            } else {
            const int nItems = gwA < nItemsAll ? (nItemsAll - gwA + WA - 1) / WA : 0;
            const int Tn = nItems * nb;
            auto issueStep = [&](int4 (&set)[NRT][CBT], float& sc, int st) {
                const int s2 = min(st, Tn - 1);                      // past the end: the last step again (uniform loop)
                const int k = s2 / nb, b = s2 - k * nb;
                const int r0 = (gwA + k * WA) * NRT;
#pragma unroll
                for (int i = 0; i < NRT; i++)
                    ld_row<true, Q4, CBT>(wrow<Q4>(lmW, lmAux, min(r0 + i, vocab - 1), dim), nchD, lane, b * CBT * 64, set[i]);
                sc = Q4 ? 1.f : ldg_f<true>(lmAux, min(r0 + (lane < NRT ? lane : 0), vocab - 1));
            };
            if (Tn > 0) {
#pragma unroll
                for (int j = 0; j < RDT - 1; j++) issueStep(ring[j], scl[j], j);
            }
            resetOther();
            const float rs = stage_rms<GL, Q4, true>(xfin, true, TW_PTR(const float, finalGain), dim, p.eps, a4, red, wt);
            FLOW_TRACE(1);
            for (int s0 = 0; s0 < Tn; s0 += RDT) {
#pragma unroll
                for (int j = 0; j < RDT; j++) {
                    const int st = s0 + j;
                    issueStep(ring[(j + RDT - 1) % RDT], scl[(j + RDT - 1) % RDT], st + RDT - 1);
                    if (st < Tn) {                                       // uniform in the wave
                        const int k = st / nb, b = st - k * nb;
                        dot_rows<Q4, NRT, CBT>(ring[j], a4, nchD, lane, b * CBT * 64, acc);
                        if (b == nb - 1) finishItem((gwA + k * WA) * NRT, scl[j], rs);
                    }
                }
            }
            }
            FLOW_TRACE(2);
            // argmax exchange: the workgroup's best (value, lowest index) goes out once its own stores (the reset above among
            // them) have been acknowledged; then every workgroup reads all of them and picks the token for itself
            wave_argmax(bestV, bestI);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            if (lane == 0) { tailV[wave] = bestV; tailI[wave] = bestI; }
            __syncthreads();
            FLOW_TRACE(4);
            {
                float v = tailV[0];
                int ix = tailI[0];
#pragma unroll
                for (int k = 1; k < FWAVES; k++) argmax_pick(v, ix, tailV[k], tailI[k]);
                if (tid == 0) {
                    float* slot = amax + ((size_t)(pos & 1) * gridDim.x + blockIdx.x) * FLOW_AMAX_STRIDE;
                    store_arg(slot, v, ix);
                }
            }
            float pv = -INFINITY;
            int pix = INT_MAX;
            for (int i = tid; i < (int)gridDim.x; i += FWG) {
                const ArgPart pr = poll_arg(amax + ((size_t)(pos & 1) * gridDim.x + i) * FLOW_AMAX_STRIDE, wt);
                argmax_pick(pv, pix, pr.v, pr.i);
            }
            FLOW_TRACE(5);
            wave_argmax(pv, pix);
            __syncthreads();                                 // every thread has read the waves' bests above
            if (lane == 0) { tailV[wave] = pv; tailI[wave] = pix; }
            __syncthreads();
            float tv = tailV[0];
            int ti = tailI[0];
#pragma unroll
            for (int k = 1; k < FWAVES; k++) argmax_pick(tv, ti, tailV[k], tailI[k]);
            if (ti < 0 || ti >= vocab) ti = 0;               // (a wait ran out: whatever it is, it stays a token)
            FLOW_TRACE(3);
            const int* prompt = TW_PTR(const int, prompt);
            if (blockIdx.x == 0 && tid == 0) {
                int* history = TW_PTR(int, history);
                if (history && count0 + tk < TW_INT(historyCap)) history[count0 + tk] = ti;
            }
            tok = (prompt && np < nPrompt) ? prompt[np] : ti;
            pos = np;
        }
    }   // tokens of the launch
    if (tokens && blockIdx.x == 0) {
        // the device state and the RoPE row of the next position, as the separate launches' last kernel leaves them
        StepState* stw = TW_PTR(StepState, state);
        float* rc = TW_PTR(float, ropeCur);
        const int pr = pos < p.maxSeq ? pos : p.maxSeq - 1;
        if (rc) {
            for (int j = tid; j < half; j += FWG) {
                rc[j] = TW_PTR(const float, cosTab)[(size_t)pr * half + j];
                rc[half + j] = TW_PTR(const float, sinTab)[(size_t)pr * half + j];
            }
        }
        if (tid == 0) { stw->pos = pos; stw->token = tok; stw->count = count0 + nTok; }
    }
}

FlowGeometry flow_geometry(int dim, int kvDim, int ffn, int nHeads, int nKVHeads, int headDim, int maxSeq, int grid) {
    FlowGeometry g{};
    // partial slots: one per FLOW_TILE positions, at most as many as the workgroups of the launch can serve.  One
    // workgroup a query head where that covers the context (the shorter phase), else one a KV head, taking all its
    // query heads in turn on one load of the K / V rows.
    const int want = (maxSeq + FLOW_TILE - 1) / FLOW_TILE;
    g.gqa = (nHeads > 0 && want > grid / nHeads && nKVHeads > 0 && nHeads / nKVHeads > 1 && nHeads / nKVHeads <= FLOW_GQA_MAX) ? 1 : 0;
    const int unit = g.gqa ? nKVHeads : nHeads;
    g.smax = want;
    if (unit > 0 && g.smax > grid / unit) g.smax = grid / unit;
    if (g.smax < 1) g.smax = 1;
    // the vectors whose place depends on the sizes alone come first (a variant with a known shape has them as constants),
    // the partial slots, which grow with the context, last
    auto up64 = [](int v) { return (v + 63) & ~63; };
    const FlowGeometry h = flow_geometry_head(dim, kvDim, ffn);
    g.offQ = h.offQ; g.offKc = h.offKc; g.offVc = h.offVc; g.offX1 = h.offX1; g.offM = h.offM; g.offX2 = h.offX2;
    g.offAttn = h.offAttn; g.offPacc = h.offPacc;
    int o = g.offPacc + up64(g.smax * dim);
    g.offPm = o; o += up64(g.smax * nHeads);
    g.offPl = o; o += up64(g.smax * nHeads);
    g.stride = o;
    return g;
}

// Of `cus` resident workgroups, how many prefetch instead of computing (a multiple of 8: the same number on every
// XCD).  They pay where a layer is a chain of latencies rather than a stream of bytes: a layer's share of an XCD must
// fit its 4 MB L2 beside the share in use (beyond that the prefetched lines push each other out: 1.1B shape 0.453 ->
// 0.494 ms/token with them), and no phase may need more rounds of the computing waves than it would with all
// workgroups computing (8B shape: eight rounds of gate | up instead of seven).  layerBytes: weights of one layer.
int flow_prefetch_workgroups(int cus, size_t layerBytes, int dim, int kvDim, int ffn) {
    const int n = 32;
    if (cus < 128 || cus % 8 || layerBytes / 8 > ((size_t)5 << 19)) return 0;       // 2.5 MB an XCD
    auto rounds = [](int items, int wgs) { return (items + wgs * FWAVES - 1) / (wgs * FWAVES); };
    const int items[3] = {dim / 2 + kvDim, dim, ffn};                               // q | k | v pairs, Wo / down rows, gate | up rows
    for (int it : items) if (rounds(it, cus - n) != rounds(it, cus)) return 0;
    return n;
}

int flow_min_grid(int nHeads, int nKVHeads, const FlowGeometry& g) { return (g.gqa ? nKVHeads : nHeads) * g.smax; }
// one workgroup per (query head, tile): the slots cover the context
bool flow_context_fits(int maxSeq, const FlowGeometry& g) { return (long long)FLOW_TILE * g.smax >= maxSeq; }

bool flow_grid_fits(int ffn, int nHeads, const FlowGeometry& g, int nCompute) {
    if (nCompute <= 0) return false;
    if ((ffn + nCompute * FWAVES - 1) / (nCompute * FWAVES) > FLOW_MAX_ROUNDS) return false;
    if (g.gqa && nHeads > nCompute) return false;
    return true;
}

bool flow_shape_supported(int dim, int kvDim, int ffn, int nHeads, int nKVHeads, int headDim) {
    if (headDim != 64 && headDim != 128) return false;
    // LDS: the staged vector (dynamic, up to 60 KB) beside the kernel's own arrays (4 to 7 KB; 33 to 52 KB in the
    // variants with grouped attention, which keep every query head's partials) stays inside the CU's 160 KB
    if (dim % 16 || ffn % 16 || kvDim % 16 || dim > 15360 || ffn > 15360) return false;
    if (nKVHeads <= 0 || nHeads % nKVHeads || nHeads * headDim != dim || nKVHeads * headDim != kvDim) return false;
    return true;
}

hipError_t launch_flow_layers(const FlowParams& p, int grid, hipStream_t s) {
    if (!flow_shape_supported(p.dim, p.kvDim, p.ffn, p.nHeads, p.nKVHeads, p.headDim)) return hipErrorInvalidValue;
    const int nC = p.nCompute;
    if (nC <= 0 || nC > grid || ((grid - nC) && (nC % 8 || (grid - nC) % 8))) return hipErrorInvalidValue;
    if (p.l0 < 0 || p.l1 <= p.l0 || p.l1 > p.nLayersTotal || nC < flow_min_grid(p.nHeads, p.nKVHeads, p.geo) ||
        !flow_context_fits(p.maxSeq, p.geo) || !p.layers || !p.xchg || !p.err || !p.hidden ||
        !flow_grid_fits(p.ffn, p.nHeads, p.geo, nC) || (size_t)p.nLayersTotal * p.geo.stride * 4 >= (1ull << 31))
        return hipErrorInvalidValue;
    if (p.nTokens > 0 && (!p.tail || !p.state || p.l0 != 0 || p.l1 != p.nLayersTotal || p.nTokens > p.maxSeq ||
                          flow_lds_bytes(p.dim, p.ffn, p.headDim, p.geo.gqa, true) > ((size_t)160 << 10)))
        return hipErrorInvalidValue;
    const size_t lds = (size_t)((p.dim > p.ffn ? p.dim : p.ffn) + (p.nTokens > 0 ? p.dim : 0)) * sizeof(float);
    const bool wide = p.dim > 1024, ring = p.dim > 2048, gqa = p.geo.gqa != 0 && p.gqaCode != 0;
#define FLOW_LAUNCH(HDv, CBv, RGv, GQv, Q4v) do { \
        if (p.trace) hipLaunchKernelGGL((flow_layers_kernel<HDv, CBv, RGv, GQv, Q4v, true>), dim3(grid), dim3(FWG), lds, s, p); \
        else hipLaunchKernelGGL((flow_layers_kernel<HDv, CBv, RGv, GQv, Q4v, false>), dim3(grid), dim3(FWG), lds, s, p); } while (0)
#define FLOW_LAUNCH_G(HDv, CBv, RGv) do { \
        if (p.q4) { if (gqa) FLOW_LAUNCH(HDv, CBv, RGv, true, true); else FLOW_LAUNCH(HDv, CBv, RGv, false, true); } \
        else { if (gqa) FLOW_LAUNCH(HDv, CBv, RGv, true, false); else FLOW_LAUNCH(HDv, CBv, RGv, false, false); } } while (0)
    // the variants with a known shape's sizes compiled in (launches of exactly that shape, unless switched off)
    int fix = 0;
    if (!p.generic)
        for (int k = 1; k <= 3 && !fix; k++) {
            const FlowFixedShape fs = flow_fixed_shape(k);
            if (p.dim == fs.dim && p.kvDim == fs.kvDim && p.ffn == fs.ffn && p.nHeads == fs.nHeads && p.nKVHeads == fs.nKVHeads &&
                p.headDim == fs.headDim && (p.downSplit != 0) == (fs.downSplit != 0) && (k != 1 || (nC != grid) == (fs.dedicated != 0))) fix = k;
        }
#define FLOW_LAUNCH_F(HDv, CBv, RGv, GQv, Q4v, FXv) do { \
        if (p.trace) hipLaunchKernelGGL((flow_layers_kernel<HDv, CBv, RGv, GQv, Q4v, true, FXv>), dim3(grid), dim3(FWG), lds, s, p); \
        else hipLaunchKernelGGL((flow_layers_kernel<HDv, CBv, RGv, GQv, Q4v, false, FXv>), dim3(grid), dim3(FWG), lds, s, p); } while (0)
    if (fix == 1 && !gqa && !p.kvHalf) {
        if (p.q4) FLOW_LAUNCH_F(64, 1, false, false, true, 1);
        else if (p.nTokens > 0 && !p.trace)             // (whole tokens as a constant: 0.3140 -> 0.3130 ms a token; slower in the other variants)
            hipLaunchKernelGGL((flow_layers_kernel<64, 1, false, false, false, false, 17>), dim3(grid), dim3(FWG), lds, s, p);
        else FLOW_LAUNCH_F(64, 1, false, false, false, 1);
    } else if (fix == 2 && !gqa && !p.q4 && !p.kvHalf) {
        FLOW_LAUNCH_F(64, 2, false, false, false, 2);
    } else if (fix == 3 && !p.q4 && !p.kvHalf) {
        if (gqa) FLOW_LAUNCH_F(128, 2, true, true, false, 3);
        else FLOW_LAUNCH_F(128, 2, true, false, false, 3);
    } else if (fix == 3 && !p.q4 && gqa) {              // fp16 K / V rows at a long context
        FLOW_LAUNCH_F(128, 2, true, true, false, 11);
    } else if (p.headDim == 64) {
        if (ring) FLOW_LAUNCH_G(64, 2, true);
        else if (wide) FLOW_LAUNCH_G(64, 2, false);
        else FLOW_LAUNCH_G(64, 1, false);
    } else {
        if (ring) FLOW_LAUNCH_G(128, 2, true);
        else if (wide) FLOW_LAUNCH_G(128, 2, false);
        else FLOW_LAUNCH_G(128, 1, false);
    }
#undef FLOW_LAUNCH_F
#undef FLOW_LAUNCH_G
#undef FLOW_LAUNCH
    return hipGetLastError();
}

__global__ void flow_reset_kernel(uint4* x, size_t n4) {
    const uint4 sent = make_uint4(XSENT, XSENT, XSENT, XSENT);
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += (size_t)gridDim.x * blockDim.x) x[i] = sent;
}
hipError_t launch_flow_reset(float* xchg, const FlowGeometry& g, int l0, int l1, hipStream_t s) {
    if (l1 <= l0) return hipSuccess;
    const size_t n4 = (size_t)(l1 - l0) * g.stride / 4;
    size_t blocks = (n4 + WG - 1) / WG;
    if (blocks > 1024) blocks = 1024;
    hipLaunchKernelGGL(flow_reset_kernel, dim3((unsigned)blocks), dim3(WG), 0, s,
                       reinterpret_cast<uint4*>(xchg + (size_t)l0 * g.stride), n4);
    return hipGetLastError();
}

size_t flow_xchg_floats(const FlowGeometry& g, int nLayers, int grid) {
    return (size_t)2 * nLayers * g.stride + (size_t)2 * grid * FLOW_AMAX_STRIDE;
}
hipError_t launch_flow_reset_all(float* xchg, const FlowGeometry& g, int nLayers, int grid, hipStream_t s) {
    const size_t n4 = flow_xchg_floats(g, nLayers, grid) / 4;
    size_t blocks = (n4 + WG - 1) / WG;
    if (blocks > 1024) blocks = 1024;
    hipLaunchKernelGGL(flow_reset_kernel, dim3((unsigned)blocks), dim3(WG), 0, s, reinterpret_cast<uint4*>(xchg), n4);
    return hipGetLastError();
}
size_t flow_lds_bytes(int dim, int ffn, int headDim, int gqa, bool tokenMode) {
    const size_t own = headDim == 64 ? (gqa ? (34u << 10) : (5u << 10)) : (gqa ? (53u << 10) : (8u << 10));
    return own + (size_t)((dim > ffn ? dim : ffn) + (tokenMode ? dim : 0)) * sizeof(float);
}

}  // namespace mg
