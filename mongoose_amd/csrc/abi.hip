// abi.hip -- the C entry points a dlsym table or cgo block binds: the device
// memory shim (cuda_tensor.go:19-52) and one launch per decode op with the
// reference's symbol names and argument order (kernels.go:12-72).
#include "../../include/mongoose_hip.h"
#include "kernels.h"

#include <atomic>
#include <cstdio>
#include <cstring>

namespace {
std::atomic<int> g_lastErr{0};
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
    return hipSetDevice(device) == hipSuccess ? 0 : -1;
}
int tw_hip_device_info(char* name, size_t nameLen, uint64_t* totalMem) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) { (void)hipGetLastError(); return -1; }
    if (name && nameLen) { std::strncpy(name, prop.name, nameLen - 1); name[nameLen - 1] = 0; }
    if (totalMem) *totalMem = (uint64_t)prop.totalGlobalMem;
    return 0;
}

void mongoose_rmsnorm_out_eps(const float* in, float* out, const float* w, int seqLen, int dim, float eps, void* stream) {
    note(mg::launch_rmsnorm_out(in, out, w, seqLen, dim, eps, S(stream)));
}
void mongoose_rmsnorm_out(const float* in, float* out, const float* w, int seqLen, int dim, void* stream) {
    mongoose_rmsnorm_out_eps(in, out, w, seqLen, dim, 1e-6f, stream);     // mongoose.cu:170
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
void mongoose_copy(void* dst, const void* src, size_t bytes, void* stream) {
    if (bytes) note(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, S(stream)));
}
void mongoose_zero(void* ptr, size_t bytes, void* stream) {
    note(mg::launch_fill_zero(ptr, bytes, S(stream)));
}
void mongoose_sync(void* stream) { note(hipStreamSynchronize(S(stream))); }

int mongoose_check(void) {
    hipError_t e = hipGetLastError();
    int rec = g_lastErr.exchange(0);
    return rec ? rec : (int)e;
}

}  // extern "C"
