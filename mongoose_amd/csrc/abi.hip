// abi.hip -- the C entry points a dlsym table or cgo block binds: the device
// memory shim (cuda_tensor.go:19-52) and one launch per decode op with the
// reference's symbol names and argument order (kernels.go:12-72).
#include "../../include/mongoose_hip.h"
#include "kernels.h"
#include "prefill.h"
#include "fused_infer.h"

#include <atomic>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

// Scratch memory of mg_q8_gemm_noalloc: the two bf16 planes of the split activations live in this
// array instead of a caller's workspace.  Every GPU the library runs on holds its own copy for the life
// of the process.  In host code the name is only a handle: the device address is looked up once per
// device (scratch_on_current_device) and that pointer is what kernels and copies are given.
#define MG_NOALLOC_SCRATCH_BYTES (8u << 20)
static __device__ __align__(256) unsigned char scratch[MG_NOALLOC_SCRATCH_BYTES];

namespace {
std::atomic<int> g_lastErr{0};
constexpr int kMaxDevices = 64;
std::mutex g_scratchMu;
void* g_scratchPtr[kMaxDevices] = {};
// Device address of `scratch` on the current device (looked up on the first call per device).
hipError_t scratch_on_current_device(void** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lk(g_scratchMu);
    if (!g_scratchPtr[dev]) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        if (!ptr) return hipErrorInvalidSymbol;
        g_scratchPtr[dev] = ptr;
    }
    *out = g_scratchPtr[dev];
    return hipSuccess;
}
inline void note(hipError_t e) {
    if (e != hipSuccess) g_lastErr.store((int)e);
}
inline hipStream_t S(void* s) { return static_cast<hipStream_t>(s); }
inline bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }
}  // namespace

extern "C" {

void* tw_gpu_alloc(size_t bytes) {
    void* ptr = nullptr;
    hipError_t e = hipMalloc(&ptr, bytes ? bytes : 1);
    if (e != hipSuccess) {
        std::fprintf(stderr, "[HIP OOM] hipMalloc(%zu bytes / %.1f MB) failed: %s\n", bytes,
                     (double)bytes / (1024 * 1024), hipGetErrorString(e));
        (void)hipGetLastError();
        return nullptr;
    }
    return ptr;
}
void tw_gpu_free(void* ptr) { if (ptr) note(hipFree(ptr)); }
void tw_gpu_upload(void* dst, const void* src, size_t bytes) { if (bytes) note(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice)); }
void tw_gpu_download(void* dst, const void* src, size_t bytes) { if (bytes) note(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost)); }
void tw_gpu_zero(void* ptr, size_t bytes) { if (bytes) note(hipMemset(ptr, 0, bytes)); }
void* tw_gpu_alloc_pinned(size_t bytes) {
    void* ptr = nullptr;
    if (hipHostMalloc(&ptr, bytes ? bytes : 1, hipHostMallocDefault) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
    return ptr;
}
void tw_gpu_free_pinned(void* ptr) { if (ptr) note(hipHostFree(ptr)); }

int tw_hip_init_device(int device) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || device < 0 || device >= n) { (void)hipGetLastError(); return -1; }
    if (hipSetDevice(device) != hipSuccess) { (void)hipGetLastError(); return -1; }
    // set-up work that later calls must not have to do: the address of the no-allocation entry
    // point's scratch array on this device
    void* ptr = nullptr;
    if (scratch_on_current_device(&ptr) != hipSuccess) { (void)hipGetLastError(); return -1; }
    return 0;
}
int tw_hip_device_info(char* name, size_t nameLen, uint64_t* totalMem) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) { (void)hipGetLastError(); return -1; }
    if (name && nameLen) {          // some driver stacks leave the marketing name empty: fall back to the ISA name
        std::strncpy(name, prop.name[0] ? prop.name : prop.gcnArchName, nameLen - 1);
        name[nameLen - 1] = 0;
    }
    if (totalMem) *totalMem = (uint64_t)prop.totalGlobalMem;
    return 0;
}

void mongoose_rmsnorm_out_eps(const float* in, float* out, const float* w, int seqLen, int dim, float eps, void* stream) {
    note(mg::launch_rmsnorm_out(in, out, w, seqLen, dim, eps, S(stream)));
}
void mongoose_rmsnorm_out(const float* in, float* out, const float* w, int seqLen, int dim, void* stream) {
    mongoose_rmsnorm_out_eps(in, out, w, seqLen, dim, 1e-6f, stream);     // mongoose.cu:170
}

// kernels.go:12, mongoose.cu:16-50: in place, eps 1e-6 (mongoose.cu:47).
void mongoose_rmsnorm(float* x, const float* w, int seqLen, int dim, void* stream) {
    note(mg::launch_rmsnorm_out(x, x, w, seqLen, dim, 1e-6f, S(stream)));     // every thread reads an element before it writes it
}
// kernels.go:20, mongoose.cu:372-404.
void mongoose_fused_add_rmsnorm(const float* a, const float* b, float* out, const float* w, int seqLen, int dim, void* stream) {
    note(mg::launch_fused_add_rmsnorm(a, b, out, w, seqLen, dim, 1e-6f, S(stream)));
}
void mongoose_fused_add_rmsnorm_eps(const float* a, const float* b, float* out, const float* w, int seqLen, int dim, float eps,
                                    void* stream) {
    note(mg::launch_fused_add_rmsnorm(a, b, out, w, seqLen, dim, eps, S(stream)));
}
// kernels.go:63, mongoose.cu:1598-1640.
void mongoose_q4_matvec(const float* act, const void* w_packed, const float* scales, float* out, int N, int K, void* stream) {
    note(mg::launch_q4_rowscale_matvec(act, w_packed, scales, out, N, K, S(stream)));
}

static void q8_matvec_any(const float* act, const void* w, const float* scales, float* out, int N, int K, int div127, void* stream) {
    if (N <= 0 || K <= 0) return;
    if (K % 16 == 0 && K * 4 <= 64 * 1024 && aligned16(w) && aligned16(act)) {
        mg::MvParams p{};
        p.seg[0] = mg::MvSeg{w, scales, nullptr, out, N};
        p.nseg = 1; p.K = K; p.act = act; p.div127 = div127;
        note(mg::launch_matvec(mg::WF_Q8, mg::EPI_STORE, mg::PRO_PLAIN, p, nullptr, S(stream)));
    } else {
        note(mg::launch_matvec_generic_q8(act, w, scales, out, N, K, div127, S(stream)));
    }
}
void mongoose_q8_matvec(const float* act, const void* w, const float* scales, float* out, int N, int K, void* stream) {
    q8_matvec_any(act, w, scales, out, N, K, 1, stream);
}
void mongoose_q8_matvec_rowscale(const float* act, const void* w, const float* scales, float* out, int N, int K, void* stream) {
    q8_matvec_any(act, w, scales, out, N, K, 0, stream);
}

void mongoose_q4_0_matvec(const float* act, const void* w, float* out, int N, int K, void* stream) {
    if (N <= 0 || K <= 0) return;
    if (K % 32 != 0 || K * 4 > 64 * 1024 || !aligned16(act) || ((uintptr_t)w & 1u)) { note(hipErrorInvalidValue); return; }
    mg::MvParams p{};
    p.seg[0] = mg::MvSeg{w, nullptr, nullptr, out, N};
    p.nseg = 1; p.K = K; p.act = act;
    note(mg::launch_matvec(mg::WF_Q4RAW, mg::EPI_STORE, mg::PRO_PLAIN, p, nullptr, S(stream)));
}
void mongoose_q4_0_repack(const void* w, void* planar, int N, int K, void* stream) {
    if (K % 32 != 0 || ((uintptr_t)w & 1u) || ((uintptr_t)planar & 1u)) { note(hipErrorInvalidValue); return; }
    note(mg::launch_q4_0_repack(w, planar, N, K, S(stream)));
}
void mongoose_q4_0_matvec_planar(const float* act, const void* planar, float* out, int N, int K, void* stream) {
    if (N <= 0 || K <= 0) return;
    if (K % 32 != 0 || K * 4 > 64 * 1024 || !aligned16(act) || !aligned16(planar)) { note(hipErrorInvalidValue); return; }
    mg::MvParams p{};
    p.seg[0] = mg::MvSeg{planar, nullptr, nullptr, out, N};
    p.nseg = 1; p.K = K; p.act = act;
    note(mg::launch_matvec(mg::WF_Q4P, mg::EPI_STORE, mg::PRO_PLAIN, p, nullptr, S(stream)));
}

// kernels.go:66-70, 985-1017: the integer (dp4a) forms of the Q4_0 matvec.  The reference's CUDA bodies are not in
// its tree; block format and arithmetic are documented in q4_dp4a.hip.
void mongoose_q8_quantize_act(const float* act, void* q8_out, int K, void* stream) {
    if (K <= 0) return;
    note(mg::launch_q8_quantize_act(act, q8_out, K, 1, S(stream)));
}
void mongoose_q8_quantize_act_batch(const float* acts, void* q8_out, int K, int B, void* stream) {
    if (K <= 0 || B <= 0) return;
    note(mg::launch_q8_quantize_act(acts, q8_out, K, B, S(stream)));
}
void mongoose_q4_0_matvec_dp4a_preq(const void* w, const void* q8_act, float* out, int N, int K, void* stream) {
    if (N <= 0 || K <= 0) return;
    note(mg::launch_q4_0_dp4a(w, false, q8_act, out, N, K, 1, S(stream)));
}
void mongoose_q4_0_matvec_dp4a(const float* act, const void* w, float* out, int N, int K, void* q8_scratch, void* stream) {
    if (N <= 0 || K <= 0) return;
    hipError_t e = mg::launch_q8_quantize_act(act, q8_scratch, K, 1, S(stream));
    if (e == hipSuccess) e = mg::launch_q4_0_dp4a(w, false, q8_scratch, out, N, K, 1, S(stream));
    note(e);
}
void mongoose_q4_0_matvec_dp4a_batch(const void* w, const void* q8_acts, float* out, int N, int K, int B, void* stream) {
    if (N <= 0 || K <= 0 || B <= 0) return;
    note(mg::launch_q4_0_dp4a(w, false, q8_acts, out, N, K, B, S(stream)));
}

void mongoose_rope(float* x, const float* cosTab, const float* sinTab, int seqLen, int dim, int headDim, int nHeads, void* stream) {
    note(mg::launch_rope(x, cosTab, sinTab, seqLen, dim, headDim, nHeads, S(stream)));
}
void mongoose_kv_cache_write(float* cache, const float* src, int pos, int kvDim, void* stream) {
    note(mg::launch_kv_cache_write(cache, src, pos, kvDim, S(stream)));
}
void mongoose_decode_attention(const float* Q, const float* K, const float* V, float* out, int cacheLen, int dim, int kvDim,
                               int nHeads, int nKVHeads, void* stream) {
    if (cacheLen <= 0 || nHeads <= 0) return;
    mg::AttnParams p{};
    p.q = Q; p.Kc = K; p.Vc = V;
    p.posImm = cacheLen - 1;
    p.rowLimit = cacheLen;
    p.kvDim = kvDim; p.nHeads = nHeads; p.nKVHeads = nKVHeads;
    p.headDim = dim / nHeads;                                    // mongoose.cu:939
    p.out = out; p.smax = 1; p.splitLen = 0;
    note(mg::launch_attention(p, S(stream)));
}
void mongoose_silu_gate_mul(const float* gate, const float* up, float* out, int n, void* stream) {
    note(mg::launch_silu_gate_mul(gate, up, out, n, S(stream)));
}
void mongoose_add_inplace(float* a, const float* b, int n, void* stream) {
    note(mg::launch_add_inplace(a, b, n, S(stream)));
}
void mongoose_embed_gather(float* out, const float* embed, const int* tokens, int seqLen, int dim, void* stream) {
    note(mg::launch_embed_gather_f32(out, embed, tokens, seqLen, dim, S(stream)));
}
void mongoose_dequant_int8_to_fp32(const void* w, const float* scales, float* out, int rows, int cols, void* stream) {
    note(mg::launch_dequant_q8(w, scales, out, rows, cols, 1, S(stream)));
}
void mongoose_dequant_q8_rowscale(const void* w, const float* scales, float* out, int rows, int cols, void* stream) {
    note(mg::launch_dequant_q8(w, scales, out, rows, cols, 0, S(stream)));
}
void mongoose_dequant_q4_0(const void* w, float* out, int rows, int cols, void* stream) {
    note(mg::launch_dequant_q4_0(w, out, rows, cols, S(stream)));
}
void mongoose_q8_gemm(const float* act, const void* w, const float* scales, const float* bias, float* out, int T, int N,
                      int K, int accumulate, void* workspace, size_t workspaceBytes, void* stream) {
    const size_t plane = mg::split_plane_elems(T, K > 0 ? K : 64) * 2;     // a multiple of 16 KB
    if (T < 0 || N < 0 || K <= 0 || K % 32 != 0 || !workspace || workspaceBytes < 2 * plane ||
        ((uintptr_t)workspace & 15) || ((uintptr_t)w & 15)) { note(hipErrorInvalidValue); return; }
    void* hi = workspace;
    void* lo = static_cast<char*>(workspace) + plane;
    note(mg::launch_split_rows(act, nullptr, 0.f, T, K, hi, lo, S(stream)));
    if (T == 0 || N == 0) return;
    mg::GemmParams g{};
    g.seg[0] = mg::GemmSeg{static_cast<const signed char*>(w), scales, bias, out, N, 0};
    g.nseg = 1; g.T = T; g.K = K;
    g.Ahi = static_cast<const unsigned short*>(hi); g.Alo = static_cast<const unsigned short*>(lo);
    note(mg::launch_gemm_q8(g, accumulate, S(stream)));
}
// mongoose_q8_gemm with the split planes in the library's static scratch array: no allocation of any
// kind on this path (no hipMalloc / hipFree, no workspace from the caller).
int mg_q8_gemm_noalloc(const float* act, const void* w, const float* scales, const float* bias, float* out, int T, int N,
                       int K, int accumulate, void* stream) {
    if (T < 0 || N < 0 || K <= 0 || K % 32 != 0 || !act || !w || !scales || !out || ((uintptr_t)w & 15)) {
        mg::set_error("mg_q8_gemm_noalloc: bad argument (K must be a positive multiple of 32, w 16-byte aligned)");
        return MG_E_ARG;
    }
    const size_t plane = mg::split_plane_elems(T, K) * 2;
    if (2 * plane > MG_NOALLOC_SCRATCH_BYTES) {
        mg::set_error("mg_q8_gemm_noalloc: 4 * roundup(T,128) * roundup(K,64) = " + std::to_string(2 * plane) +
                      " bytes of split activations exceed the static scratch of " + std::to_string(MG_NOALLOC_SCRATCH_BYTES) +
                      " bytes; use mongoose_q8_gemm with a workspace");
        return MG_E_ARG;
    }
    if (T == 0 || N == 0) return MG_OK;
    void* base = nullptr;
    hipError_t e = scratch_on_current_device(&base);
    if (e != hipSuccess) {
        mg::set_error(std::string("mg_q8_gemm_noalloc: scratch address lookup failed: ") + hipGetErrorString(e));
        (void)hipGetLastError();
        return MG_E_HIP;
    }
    void* hi = base;
    void* lo = static_cast<char*>(base) + plane;
    e = mg::launch_split_rows(act, nullptr, 0.f, T, K, hi, lo, S(stream));
    if (e == hipSuccess) {
        mg::GemmParams g{};
        g.seg[0] = mg::GemmSeg{static_cast<const signed char*>(w), scales, bias, out, N, 0};
        g.nseg = 1; g.T = T; g.K = K;
        g.Ahi = static_cast<const unsigned short*>(hi); g.Alo = static_cast<const unsigned short*>(lo);
        e = mg::launch_gemm_q8(g, accumulate, S(stream));
    }
    if (e != hipSuccess) {
        mg::set_error(std::string("mg_q8_gemm_noalloc: launch failed: ") + hipGetErrorString(e));
        (void)hipGetLastError();
        return MG_E_HIP;
    }
    return MG_OK;
}
size_t mg_q8_gemm_noalloc_max_bytes(void) { return MG_NOALLOC_SCRATCH_BYTES; }

void mongoose_copy(void* dst, const void* src, size_t bytes, void* stream) {
    if (bytes) note(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, S(stream)));
}
void mongoose_zero(void* ptr, size_t bytes, void* stream) {
    note(mg::launch_fill_zero(ptr, bytes, S(stream)));
}
void mongoose_sync(void* stream) { note(hipStreamSynchronize(S(stream))); }

// Measurement helper: average duration of the Q8 / Q4_0 matvec at one shape,
// launched `iters` times over `copies` separate weight buffers in rotation (so
// that with copies * bytes larger than the caches every launch streams from
// HBM).  nr/ks/grid = 0 picks the library's own configuration.
int mg_bench_matvec(int wf, int N, int K, int nr, int ks, int grid, int copies, int iters, float* avgUs) {
    if ((wf != mg::WF_Q8 && wf != mg::WF_Q4P) || N <= 0 || K <= 0 || K % 32 || copies < 1 || iters < 1 || !avgUs) return MG_E_ARG;
    size_t wbytes = wf == mg::WF_Q8 ? (size_t)N * K : (size_t)N * (K / 32) * 18;
    std::vector<void*> w(copies, nullptr);
    void* slab = nullptr;
    float *scales = nullptr, *act = nullptr, *out = nullptr;
    hipStream_t st = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    int rc = MG_OK;
    auto ok = [&](hipError_t e) { if (e != hipSuccess) { rc = MG_E_HIP; (void)hipGetLastError(); } return e == hipSuccess; };
    do {
        if (!ok(hipStreamCreateWithFlags(&st, hipStreamNonBlocking))) break;
        if (!ok(hipEventCreate(&e0)) || !ok(hipEventCreate(&e1))) break;
        // one slab for all copies (as the context's weight arena is laid out), 256-byte aligned slices
        size_t slice = (wbytes + 255) & ~(size_t)255;
        if (!ok(hipMalloc(&slab, slice * copies)) || !ok(hipMemset(slab, 0x11, slice * copies))) break;
        for (int c = 0; c < copies; c++) w[c] = static_cast<char*>(slab) + slice * c;
        if (!ok(hipMalloc((void**)&scales, (size_t)N * 4)) || !ok(hipMalloc((void**)&act, (size_t)K * 4)) ||
            !ok(hipMalloc((void**)&out, (size_t)N * 4))) break;
        if (!ok(hipMemset(scales, 0, (size_t)N * 4)) || !ok(hipMemset(act, 0, (size_t)K * 4))) break;
        mg::MvConfig cfg{nr, ks ? ks : 1, grid};
        auto launch = [&](int c) {
            mg::MvParams p{};
            p.seg[0] = mg::MvSeg{w[c], scales, nullptr, out, N};
            p.nseg = 1; p.K = K; p.act = act;
            mg::MvConfig use = cfg;
            return mg::launch_matvec(wf, mg::EPI_STORE, mg::PRO_PLAIN, p, nr > 0 ? &use : nullptr, st);
        };
        for (int c = 0; c < copies && rc == MG_OK; c++) ok(launch(c));
        if (rc != MG_OK || !ok(hipStreamSynchronize(st))) break;
        if (!ok(hipEventRecord(e0, st))) break;
        for (int i = 0; i < iters && rc == MG_OK; i++) ok(launch(i % copies));
        if (rc != MG_OK || !ok(hipEventRecord(e1, st)) || !ok(hipEventSynchronize(e1))) break;
        float ms = 0.f;
        if (!ok(hipEventElapsedTime(&ms, e0, e1))) break;
        *avgUs = ms * 1000.0f / (float)iters;
    } while (0);
    if (slab) (void)hipFree(slab);
    if (scales) (void)hipFree(scales);
    if (act) (void)hipFree(act);
    if (out) (void)hipFree(out);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (st) (void)hipStreamDestroy(st);
    return rc;
}

int mongoose_check(void) {
    hipError_t e = hipGetLastError();
    int rec = g_lastErr.exchange(0);
    return rec ? rec : (int)e;
}

}  // extern "C"
