// fused_infer.hip -- HIPFusedInference and the mg_* C entry points over it.
// Host code only (no kernels here); compiled with hipcc for the runtime API.
#include "fused_infer.h"
#include <mutex>
#include "../../include/mongoose_hip.h"
#include "host_util.h"
#include "prefill.h"

#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>

namespace mg {

static thread_local std::string g_err;
void set_error(const std::string& s) { g_err = s; }
const std::string& get_error() { return g_err; }

#define HIPCHK(expr)                                                                      \
    do {                                                                                  \
        hipError_t e_ = (expr);                                                           \
        if (e_ != hipSuccess) {                                                           \
            set_error(std::string(#expr) + ": " + hipGetErrorString(e_));                 \
            (void)hipGetLastError();                                                      \
            return MG_E_HIP;                                                              \
        }                                                                                 \
    } while (0)

#define ARGCHK(cond, msg)                                                                 \
    do {                                                                                  \
        if (!(cond)) { set_error(msg); return MG_E_ARG; }                                 \
    } while (0)

HIPFusedInference* HIPFusedInference::New(int dim, int kvDim, int headDim, int nHeads, int nKVHeads, int ffnDim,
                                          int vocabSize, int nLayers, int maxSeq, double ropeTheta, float eps) {
    if (dim <= 0 || kvDim <= 0 || nHeads <= 0 || nKVHeads <= 0 || ffnDim <= 0 || vocabSize <= 0 || nLayers <= 0 ||
        maxSeq <= 0) { set_error("mg_create: non-positive dimension"); return nullptr; }
    if (headDim != 64 && headDim != 128) { set_error("mg_create: headDim must be 64 or 128"); return nullptr; }
    if (nHeads * headDim != dim || nKVHeads * headDim != kvDim || nHeads % nKVHeads != 0) {
        set_error("mg_create: dim/kvDim must equal heads*headDim and nHeads must be a multiple of nKVHeads");
        return nullptr;
    }
    if (dim % 32 != 0 || ffnDim % 32 != 0 || dim > 16384 || ffnDim > 16384) {
        set_error("mg_create: dim and ffnDim must be multiples of 32 and at most 16384");
        return nullptr;
    }
    int ndev = 0;
    if (hipGetDeviceCount(&ndev) != hipSuccess || ndev == 0) {
        (void)hipGetLastError();
        set_error("mg_create: no HIP device");
        return nullptr;
    }
    auto* f = new HIPFusedInference();
    f->dim = dim; f->kvDim = kvDim; f->headDim = headDim; f->nHeads = nHeads; f->nKVHeads = nKVHeads;
    f->ffnDim = ffnDim; f->vocabSize = vocabSize; f->nLayers = nLayers; f->maxSeq = maxSeq;
    f->ropeTheta = ropeTheta; f->eps = eps;
    f->layers.resize(nLayers);
    f->layerSlabs.resize(nLayers);
    {
        // slot offsets inside a layer slab, each slot sized for its largest format (Q8: bytes + row scales)
        size_t off = 0;
        for (int w = 0; w < 12; w++) {
            size_t rows = 0, cols = 0;
            switch (w) {
            case 1: case 7: rows = dim; cols = dim; break;
            case 2: case 3: rows = kvDim; cols = dim; break;
            case 9: case 10: rows = ffnDim; cols = dim; break;
            case 11: rows = dim; cols = ffnDim; break;
            case 5: case 6: rows = kvDim; break;
            default: rows = dim; break;
            }
            f->slotOff[w] = off;
            off += cols ? alignUp256(rows * cols) + alignUp256(rows * 4) : alignUp256(rows * 4);
        }
        f->layerSlabBytes = off;
    }
    f->kCache.assign(nLayers, nullptr);
    f->vCache.assign(nLayers, nullptr);

    auto fail = [&](const char* what) -> HIPFusedInference* {
        if (get_error().empty()) set_error(what);
        delete f;
        return nullptr;
    };
    if (hipStreamCreateWithFlags(&f->stream, hipStreamNonBlocking) != hipSuccess) return fail("stream create failed");
    if (hipEventCreate(&f->ev0) != hipSuccess || hipEventCreate(&f->ev1) != hipSuccess) return fail("event create failed");
    // L3 bridge: 64-byte mailbox line + the hidden state, pinned (cuda_fused_infer.go:204-217)
    if (hipHostMalloc(reinterpret_cast<void**>(&f->l3), 64 + (size_t)dim * 4, hipHostMallocDefault) != hipSuccess)
        return fail("L3 bridge allocation failed");
    std::memset(f->l3, 0, 64 + (size_t)dim * 4);
    if (hipStreamCreateWithFlags(&f->copyStream, hipStreamNonBlocking) != hipSuccess ||
        hipEventCreateWithFlags(&f->computeDone, hipEventDisableTiming) != hipSuccess)
        return fail("L3 copy stream create failed");

    // Every device buffer of the context comes out of a few large slabs (one for the scratch
    // and tables, one per layer of weights, one for the head, one per KV range): large
    // contiguous mappings keep the address-translation cost of a cold weight read low, which
    // is a measurable part of a small matvec's latency.
    const int half0 = headDim / 2;
    const int attnTile = headDim == 128 ? 128 : 256;      // positions per attention tile
    f->splitLen = attnTile * ((maxSeq + attnTile * 64 - 1) / (attnTile * 64));      // at most 64 splits
    f->smax = (maxSeq + f->splitLen - 1) / f->splitLen;
    // query heads of a GQA group per attention workgroup: one while the K/V rows of a layer sit in L2
    // anyway, two up to 8k positions (four heads a workgroup measured 20 us against 16 us at 2k-4k
    // positions of the 0.5B and 1.1B shapes, no difference at Llama-3-8B's), the whole group beyond,
    // where every extra pass over the rows is HBM traffic
    f->attnHeadsPerWG = maxSeq <= 1024 ? 1 : (maxSeq <= 8192 ? 2 : 0);
    f->amaxParts = 4096;
    {
        size_t floats = (size_t)7 * dim + 2 * (size_t)kvDim + 3 * (size_t)ffnDim + vocabSize +
                        2 * (size_t)maxSeq * half0 + (size_t)nHeads * f->smax * (headDim + 2) + headDim + f->amaxParts;
        size_t ints = (size_t)f->amaxParts + 2 * ((size_t)maxSeq + 1) + 64 + attention_columns(nHeads, nKVHeads, 1);
        size_t bytes = (floats + ints) * 4 + 64 * 256;
        if (f->scratch.init(bytes) != 0) return fail("scratch alloc failed");
        if (hipMemsetAsync(f->scratch.base, 0, bytes, f->stream) != hipSuccess || hipStreamSynchronize(f->stream) != hipSuccess)
            return fail("scratch clear failed");
    }
    auto takeF = [&](float*& p, size_t n) { p = static_cast<float*>(f->scratch.take(n * 4)); return p != nullptr; };
    auto takeI = [&](int*& p, size_t n) { p = static_cast<int*>(f->scratch.take(n * 4)); return p != nullptr; };
    bool ok = takeF(f->hidden[0], dim) && takeF(f->hidden[1], dim) && takeF(f->logits, vocabSize) && takeF(f->normed, dim) &&
              takeF(f->Q, dim) && takeF(f->K, kvDim) && takeF(f->V, kvDim) && takeF(f->attnOut, dim) && takeF(f->proj, dim) &&
              takeF(f->normed2, dim) && takeF(f->gatePre, ffnDim) && takeF(f->upOut, ffnDim) && takeF(f->ffnMid, ffnDim) &&
              takeF(f->cosTab, (size_t)maxSeq * half0) && takeF(f->sinTab, (size_t)maxSeq * half0) &&
              takeF(f->pm, (size_t)nHeads * f->smax) && takeF(f->pl, (size_t)nHeads * f->smax) &&
              takeF(f->pacc, (size_t)nHeads * f->smax * headDim) && takeF(f->ropeCur, headDim) &&
              takeF(f->amaxVal, f->amaxParts) && takeI(f->amaxIdx, f->amaxParts) &&
              takeI(f->attnCounters, attention_columns(nHeads, nKVHeads, 1)) &&
              takeI(f->dHistory, (size_t)maxSeq + 1) && takeI(f->dPrompt, (size_t)maxSeq + 1);
    if (ok) { f->dState = static_cast<StepState*>(f->scratch.take(sizeof(StepState))); ok = f->dState != nullptr; }
    if (!ok) return fail("scratch slab too small");

    // RoPE tables, cuda_fused_infer.go:181-192: angle in double, stored as float.
    const int half = headDim / 2;
    std::vector<float> cosD((size_t)maxSeq * half), sinD((size_t)maxSeq * half);
    std::vector<double> freq(half);
    for (int j = 0; j < half; j++) freq[j] = 1.0 / std::pow(ropeTheta, (double)(2 * j) / (double)headDim);
    for (int pos = 0; pos < maxSeq; pos++) {
        for (int j = 0; j < half; j++) {
            double angle = (double)pos * freq[j];
            cosD[(size_t)pos * half + j] = (float)std::cos(angle);
            sinD[(size_t)pos * half + j] = (float)std::sin(angle);
        }
    }
    if (hipMemcpy(f->cosTab, cosD.data(), cosD.size() * 4, hipMemcpyHostToDevice) != hipSuccess ||
        hipMemcpy(f->sinTab, sinD.data(), sinD.size() * 4, hipMemcpyHostToDevice) != hipSuccess) return fail("rope upload");

    void* hp = nullptr;
    if (hipHostMalloc(&hp, sizeof(StepState), hipHostMallocDefault) != hipSuccess) return fail("pinned alloc");
    f->hState = static_cast<StepState*>(hp);
    if (hipHostMalloc(&hp, 64, hipHostMallocCoherent | hipHostMallocMapped) != hipSuccess) return fail("pinned alloc");
    f->hGate = static_cast<int*>(hp);
    *f->hGate = 1;
    if (hipHostMalloc(&hp, sizeof(int) * ((size_t)maxSeq + 1), hipHostMallocDefault) != hipSuccess) return fail("pinned alloc");
    f->hTokens = static_cast<int*>(hp);

    f->built = true;
    return f;
}

int Slab::init(size_t bytes) {
    release();
    void* v = nullptr;
    HIPCHK(hipMalloc(&v, bytes ? bytes : 256));
    base = static_cast<char*>(v); size = bytes; used = 0;
    return MG_OK;
}
void* Slab::take(size_t bytes) {
    size_t off = alignUp256(used);
    if (!base || off + bytes > size) return nullptr;
    used = off + bytes;
    return base + off;
}
void Slab::release() {
    if (base) (void)hipFree(base);
    base = nullptr; size = used = 0;
}

// Device address of a weight slot (allocating the layer's / head's slab on first use).
int HIPFusedInference::slotAddr(int idx, char** out) {
    if (idx < nLayers * 12) {
        Slab& sl = layerSlabs[idx / 12];
        if (!sl.base) { int rc = sl.init(layerSlabBytes); if (rc) return rc; }
        *out = sl.base + slotOff[idx % 12];
        return MG_OK;
    }
    if (!headSlab.base) {
        int rc = headSlab.init(alignUp256((size_t)dim * 4) + alignUp256((size_t)vocabSize * dim) + alignUp256((size_t)vocabSize * 4));
        if (rc) return rc;
    }
    *out = headSlab.base + (idx == nLayers * 12 ? 0 : alignUp256((size_t)dim * 4));
    return MG_OK;
}

HIPFusedInference::~HIPFusedInference() {
    releaseFlow();
    for (HIPFusedInference** ref : backrefs) *ref = nullptr;
    if (stream) (void)hipStreamSynchronize(stream);
    invalidateGraphs();
    scratch.release();
    headSlab.release();
    prefillSlab.release();
    prefillKVSlab.release();
    for (auto& sl : layerSlabs) sl.release();
    for (auto& sl : kvSlabs) sl.release();
    if (embedTable) (void)hipFree(embedTable);
    if (q8Scratch) (void)hipFree(q8Scratch);
    if (dFlowLayers) (void)hipFree(dFlowLayers);
    if (flowXchg) (void)hipFree(flowXchg);
    if (dFlowTail) (void)hipFree(dFlowTail);
    if (dFlowErr) (void)hipFree(dFlowErr);
    if (hFlowErr) (void)hipHostFree(hFlowErr);
    if (hState) (void)hipHostFree(hState);
    if (hGate) (void)hipHostFree(hGate);
    if (hTokens) (void)hipHostFree(hTokens);
    for (hipEvent_t e : profEvents) (void)hipEventDestroy(e);
    if (copyStream) { (void)hipStreamSynchronize(copyStream); (void)hipStreamDestroy(copyStream); }
    if (computeDone) (void)hipEventDestroy(computeDone);
    if (l3) (void)hipHostFree(l3);
    if (ev0) (void)hipEventDestroy(ev0);
    if (ev1) (void)hipEventDestroy(ev1);
    if (stream) (void)hipStreamDestroy(stream);
}

int HIPFusedInference::invalidateGraphs() {
    graphGeneration++;
    flowTableDirty = true;          // whatever invalidates the graphs may have moved a weight or a cache
    if (execFull) { (void)hipGraphExecDestroy(execFull); execFull = nullptr; }
    if (execPrompt) { (void)hipGraphExecDestroy(execPrompt); execPrompt = nullptr; }
    if (graphFull) { (void)hipGraphDestroy(graphFull); graphFull = nullptr; }
    if (graphPrompt) { (void)hipGraphDestroy(graphPrompt); graphPrompt = nullptr; }
    return MG_OK;
}

// Slot map, cuda_fused_infer.go:241-272.
DevMat* HIPFusedInference::matSlot(int idx, int* rows, int* cols) {
    if (idx < 0) return nullptr;
    if (idx < nLayers * 12) {
        LayerWeights& L = layers[idx / 12];
        switch (idx % 12) {
        case 1: *rows = dim; *cols = dim; return &L.wq;
        case 2: *rows = kvDim; *cols = dim; return &L.wk;
        case 3: *rows = kvDim; *cols = dim; return &L.wv;
        case 7: *rows = dim; *cols = dim; return &L.wo;
        case 9: *rows = ffnDim; *cols = dim; return &L.gate;
        case 10: *rows = ffnDim; *cols = dim; return &L.up;
        case 11: *rows = dim; *cols = ffnDim; return &L.down;
        default: return nullptr;
        }
    }
    if (idx == nLayers * 12 + 1) { *rows = vocabSize; *cols = dim; return &lmHead; }
    return nullptr;
}

int HIPFusedInference::setVec(int idx, float*& dst, const float* data, size_t n, size_t expect) {
    ARGCHK(n == expect, "SetWeight: wrong element count for a norm/bias slot");
    char* addr = nullptr;
    int rc = slotAddr(idx, &addr);
    if (rc) return rc;
    HIPCHK(hipStreamSynchronize(stream));
    HIPCHK(hipMemcpy(addr, data, expect * sizeof(float), hipMemcpyHostToDevice));
    dst = reinterpret_cast<float*>(addr);
    return MG_OK;
}

int HIPFusedInference::uploadMat(int idx, DevMat& m, int rows, int cols, const int8_t* q, const float* scales) {
    HIPCHK(hipStreamSynchronize(stream));
    invalidateGraphs();
    char* addr = nullptr;
    int rc = slotAddr(idx, &addr);
    if (rc) return rc;
    m = DevMat();
    HIPCHK(hipMemcpy(addr, q, (size_t)rows * cols, hipMemcpyHostToDevice));
    char* sc = addr + alignUp256((size_t)rows * cols);
    HIPCHK(hipMemcpy(sc, scales, (size_t)rows * 4, hipMemcpyHostToDevice));
    m.w = addr; m.scales = reinterpret_cast<float*>(sc);
    m.kind = WF_Q8; m.rows = rows; m.cols = cols;
    m.bytes = (size_t)rows * cols + (size_t)rows * 4;
    return MG_OK;
}

int HIPFusedInference::uploadMatQ4(int idx, DevMat& m, int rows, int cols, const uint8_t* raw, size_t nbytes) {
    ARGCHK(cols % 32 == 0, "SetWeightQ4_0: cols must be a multiple of 32");
    size_t expect = (size_t)rows * (cols / 32) * 18;          // cuda_q4_0.go:16-19
    ARGCHK(nbytes == expect, "SetWeightQ4_0: byte count is not rows*(cols/32)*18");
    HIPCHK(hipStreamSynchronize(stream));
    invalidateGraphs();
    char* addr = nullptr;
    int rc = slotAddr(idx, &addr);
    if (rc) return rc;
    m = DevMat();
    std::vector<uint8_t> planar(expect);
    repack_q4_0_host(raw, rows, cols, planar.data());
    HIPCHK(hipMemcpy(addr, planar.data(), expect, hipMemcpyHostToDevice));
    m.w = addr; m.kind = WF_Q4P; m.rows = rows; m.cols = cols; m.bytes = expect;
    return MG_OK;
}

int HIPFusedInference::SetWeight(int idx, const float* data, size_t n) {
    if (!built) return MG_E_NOT_BUILT;
    ARGCHK(data != nullptr && idx >= 0 && idx < NumWeights(), "SetWeight: bad slot or NULL data");
    int rows = 0, cols = 0;
    DevMat* m = matSlot(idx, &rows, &cols);
    if (m) {
        ARGCHK(n == (size_t)rows * cols, "SetWeight: wrong element count for a matrix slot");
        std::vector<int8_t> q((size_t)rows * cols);
        std::vector<float> sc(rows);
        mg_quantize_q8(data, rows, cols, quantRounding, q.data(), sc.data());
        return uploadMat(idx, *m, rows, cols, q.data(), sc.data());
    }
    if (idx == nLayers * 12) return setVec(idx, finalNorm, data, n, dim);
    LayerWeights& L = layers[idx / 12];
    switch (idx % 12) {
    case 0: return setVec(idx, L.norm1, data, n, dim);
    case 8: return setVec(idx, L.norm2, data, n, dim);
    case 4: invalidateGraphs(); return setVec(idx, L.bq, data, n, dim);
    case 5: invalidateGraphs(); return setVec(idx, L.bk, data, n, kvDim);
    case 6: invalidateGraphs(); return setVec(idx, L.bv, data, n, kvDim);
    }
    set_error("SetWeight: unreachable slot");
    return MG_E_ARG;
}

int HIPFusedInference::SetWeightQ8(int idx, const int8_t* q, const float* scales) {
    if (!built) return MG_E_NOT_BUILT;
    int rows = 0, cols = 0;
    DevMat* m = matSlot(idx, &rows, &cols);
    ARGCHK(m && q && scales, "SetWeightQ8: not a matrix slot or NULL data");
    return uploadMat(idx, *m, rows, cols, q, scales);
}

int HIPFusedInference::SetWeightQ4_0(int idx, const uint8_t* q4Data, size_t nbytes) {
    if (!built) return MG_E_NOT_BUILT;
    int rows = 0, cols = 0;
    DevMat* m = matSlot(idx, &rows, &cols);
    // cuda_fused_infer_q4.go:52,66,78: norm, bias and final-norm slots are not Q4 and are ignored
    if (!m) return (idx >= 0 && idx < NumWeights()) ? MG_OK : MG_E_ARG;
    ARGCHK(q4Data != nullptr, "SetWeightQ4_0: NULL data");
    return uploadMatQ4(idx, *m, rows, cols, q4Data, nbytes);
}

int HIPFusedInference::SetEmbeddingF16(const uint16_t* table) {
    if (!built) return MG_E_NOT_BUILT;
    ARGCHK(table, "SetEmbeddingF16: NULL table");
    HIPCHK(hipStreamSynchronize(stream));
    invalidateGraphs();
    if (embedTable) { (void)hipFree(embedTable); embedTable = nullptr; }
    size_t bytes = (size_t)vocabSize * dim * 2;
    HIPCHK(hipMalloc(&embedTable, bytes));
    HIPCHK(hipMemcpy(embedTable, table, bytes, hipMemcpyHostToDevice));
    embedKind = 1;
    return MG_OK;
}

int HIPFusedInference::SetEmbeddingF32(const float* table) {
    if (!built) return MG_E_NOT_BUILT;
    ARGCHK(table, "SetEmbeddingF32: NULL table");
    HIPCHK(hipStreamSynchronize(stream));
    invalidateGraphs();
    if (embedTable) { (void)hipFree(embedTable); embedTable = nullptr; }
    size_t bytes = (size_t)vocabSize * dim * 4;
    HIPCHK(hipMalloc(&embedTable, bytes));
    HIPCHK(hipMemcpy(embedTable, table, bytes, hipMemcpyHostToDevice));
    embedKind = 2;
    return MG_OK;
}

int HIPFusedInference::SetLayerRange(int layerStart, int layerEnd) {
    if (!built) return MG_E_NOT_BUILT;
    ARGCHK(layerStart >= 0 && layerStart <= layerEnd, "SetLayerRange: bad range");
    int need = 0;
    for (int l = layerStart; l < layerEnd && l < nLayers; l++) if (!kCache[l]) need++;
    if (need == 0) return MG_OK;
    invalidateGraphs();
    const size_t per = alignUp256((size_t)maxSeq * kvDim * (kvHalf ? 2 : 4));
    kvSlabs.emplace_back();
    Slab& sl = kvSlabs.back();
    int rc = sl.init(per * 2 * need);
    if (rc) { kvSlabs.pop_back(); return rc; }
    // on the stream the kernels run on (a non-blocking stream does not order itself behind the NULL stream)
    HIPCHK(hipMemsetAsync(sl.base, 0, sl.size, stream));
    HIPCHK(hipStreamSynchronize(stream));
    for (int l = layerStart; l < layerEnd && l < nLayers; l++) {
        if (kCache[l]) continue;
        kCache[l] = static_cast<float*>(sl.take(per));
        vCache[l] = static_cast<float*>(sl.take(per));
    }
    return MG_OK;
}

// KV rows in fp16 halve the attention's bytes (the step toward the compressed caches the reference
// only declares hooks for, kernels.go:71-72).  The choice fixes the allocation, so it comes first.
int HIPFusedInference::SetKVFormat(int fmt) {
    if (!built) return MG_E_NOT_BUILT;
    ARGCHK(fmt == 0 || fmt == 1, "SetKVFormat: 0 (fp32) or 1 (fp16)");
    if (fmt == kvHalf) return MG_OK;
    if (!kvSlabs.empty()) { set_error("SetKVFormat: call before SetLayerRange (the caches are already allocated)"); return MG_E_STATE; }
    invalidateGraphs();
    kvHalf = fmt;
    return MG_OK;
}

// cuda_fused_infer.go:530-537 uploads zeros over K only; V is cleared as well
// here (a fresh sequence never reads V rows it has not written).
int HIPFusedInference::ResetKV() {
    if (!built) return MG_E_NOT_BUILT;
    // on the context's own stream: it is non-blocking, so a fill on the NULL stream would not be ordered
    // before the launches that follow; ResetKV is never part of a captured graph
    for (int l = 0; l < nLayers; l++) {
        if (kCache[l]) HIPCHK(hipMemsetAsync(kCache[l], 0, (size_t)maxSeq * kvDim * (kvHalf ? 2 : 4), stream));
        if (vCache[l]) HIPCHK(hipMemsetAsync(vCache[l], 0, (size_t)maxSeq * kvDim * (kvHalf ? 2 : 4), stream));
    }
    HIPCHK(hipStreamSynchronize(stream));
    return MG_OK;
}

uint64_t HIPFusedInference::WeightBytesPerToken() const {
    uint64_t b = 0;
    for (const auto& L : layers) {
        b += L.wq.bytes + L.wk.bytes + L.wv.bytes + L.wo.bytes + L.gate.bytes + L.up.bytes + L.down.bytes;
        if (L.norm1) b += (uint64_t)dim * 4;
        if (L.norm2) b += (uint64_t)dim * 4;
    }
    b += lmHead.bytes;
    if (finalNorm) b += (uint64_t)dim * 4;
    return b;
}

// While the instrumented graph is being captured: an event before the launch
// of class `cls` (the previous launch's end).  No-op otherwise.
int HIPFusedInference::mark(int cls) {
    if (!profiling) return MG_OK;
    // an event opens the interval of a wanted class and closes the interval of the one before it
    const bool opens = cls >= 0 && cls < 8 && ((profMask >> cls) & 1);
    const bool closes = profLast >= 0 && profLast < 8 && ((profMask >> profLast) & 1);
    profLast = cls;
    if (!opens && !closes) return MG_OK;
    if (!opens) cls = 8;                      // interval that follows is not measured
    hipEvent_t e = nullptr;
    HIPCHK(hipEventCreate(&e));
    profEvents.push_back(e);
    profClass.push_back(cls);
    HIPCHK(hipEventRecord(e, stream));
    return MG_OK;
}

RopeCur HIPFusedInference::ropeRef() const {
    return RopeCur{cosTab, sinTab, ropeCur, headDim / 2, maxSeq};
}

static bool layerComplete(const LayerWeights& L) {
    return L.norm1 && L.norm2 && L.wq.w && L.wk.w && L.wv.w && L.wo.w && L.gate.w && L.up.w && L.down.w;
}

// One launch per reference op, in the reference's order
// (cuda_fused_infer.go:417-443; bias adds cuda_fused_stream.go:319-321).
int HIPFusedInference::enqueueLayerPerOp(const LayerWeights& L, int layer, int pos) {
    float* h = hidden[hiddenIdx];
    const int half = headDim / 2;
    // requant: the activation vector is quantized into the int8 scratch first (false: it still holds this vector's
    // blocks -- the reference quantizes once for q, k, v and once for gate, up: cuda_fused_infer_q4.go:161-173, 208-212)
    auto mv = [&](const DevMat& m, const float* act, float* out, bool requant = true) -> hipError_t {
        if (q4ActQuant && m.kind == WF_Q4P) {                  // q4Matvec / q4MatvecPreq, cuda_fused_infer_q4.go:611-673
            if (requant) { hipError_t e = launch_q8_quantize_act(act, q8Scratch, m.cols, 1, stream); if (e != hipSuccess) return e; }
            return launch_q4_0_dp4a(m.w, true, q8Scratch, out, m.rows, m.cols, 1, stream);
        }
        MvParams p{};
        p.seg[0] = MvSeg{m.w, m.scales, nullptr, out, m.rows};
        p.nseg = 1; p.K = m.cols; p.act = act;
        return launch_matvec(m.kind, EPI_STORE, PRO_PLAIN, p, nullptr, stream);
    };
    HIPCHK(launch_rmsnorm_out(h, normed, L.norm1, 1, dim, eps, stream));
    HIPCHK(mv(L.wq, normed, Q));
    HIPCHK(mv(L.wk, normed, K, L.wq.kind != WF_Q4P));
    HIPCHK(mv(L.wv, normed, V, L.wq.kind != WF_Q4P));
    if (L.bq) HIPCHK(launch_add_inplace(Q, L.bq, dim, stream));
    if (L.bk) HIPCHK(launch_add_inplace(K, L.bk, kvDim, stream));
    if (L.bv) HIPCHK(launch_add_inplace(V, L.bv, kvDim, stream));
    const float* cosRow = cosTab + (size_t)pos * half;      // cuda_fused_infer.go:423-424
    const float* sinRow = sinTab + (size_t)pos * half;
    HIPCHK(launch_rope(Q, cosRow, sinRow, 1, dim, headDim, nHeads, stream));
    HIPCHK(launch_rope(K, cosRow, sinRow, 1, kvDim, headDim, nKVHeads, stream));
    if (kvHalf) {
        HIPCHK(launch_kv_cache_write_f16(kCache[layer], K, pos, kvDim, stream));
        HIPCHK(launch_kv_cache_write_f16(vCache[layer], V, pos, kvDim, stream));
    } else {
        HIPCHK(launch_kv_cache_write(kCache[layer], K, pos, kvDim, stream));
        HIPCHK(launch_kv_cache_write(vCache[layer], V, pos, kvDim, stream));
    }
    AttnParams a{};
    a.kvHalf = kvHalf;
    a.q = Q; a.Kc = kCache[layer]; a.Vc = vCache[layer]; a.posImm = pos; a.rowLimit = maxSeq;
    a.kvDim = kvDim; a.nHeads = nHeads; a.nKVHeads = nKVHeads; a.headDim = headDim;
    a.out = attnOut; a.smax = 1; a.splitLen = 0;
    HIPCHK(launch_attention(a, stream));
    HIPCHK(mv(L.wo, attnOut, proj));
    HIPCHK(launch_add_inplace(h, proj, dim, stream));
    HIPCHK(launch_rmsnorm_out(h, normed2, L.norm2, 1, dim, eps, stream));
    HIPCHK(mv(L.gate, normed2, gatePre));
    HIPCHK(mv(L.up, normed2, upOut, L.gate.kind != WF_Q4P));
    HIPCHK(launch_silu_gate_mul(gatePre, upOut, ffnMid, ffnDim, stream));
    HIPCHK(mv(L.down, ffnMid, proj));
    HIPCHK(launch_add_inplace(h, proj, dim, stream));
    return MG_OK;
}

// Five launches a layer: [norm1 + QKV + bias + RoPE + KV-cache write] [attention]
// [Wo + residual] [norm2 + gate/up + SiLU*mul] [down + residual].
// Operands of the four matvec launches of a layer (what is launched and what the prefetch plan describes).
MvParams HIPFusedInference::qkvParams(const LayerWeights& L, int layer, const StepState* st, int posImm) const {
    MvParams p{};
    p.K = dim; p.act = hidden[hiddenIdx]; p.gain = L.norm1; p.eps = eps;
    p.seg[0] = MvSeg{L.wq.w, L.wq.scales, L.bq, Q, dim};
    p.seg[1] = MvSeg{L.wk.w, L.wk.scales, L.bk, kCache[layer], kvDim};
    p.seg[2] = MvSeg{L.wv.w, L.wv.scales, L.bv, vCache[layer], kvDim};
    p.nseg = 3;
    p.headDim = headDim; p.kvDim = kvDim; p.kvHalf = kvHalf;
    p.state = st; p.posImm = posImm;
    const int half = headDim / 2;
    p.cosRow = st ? ropeCur : cosTab + (size_t)posImm * half;
    p.sinRow = st ? ropeCur + half : sinTab + (size_t)posImm * half;
    return p;
}
MvParams HIPFusedInference::woParams(const LayerWeights& L) const {
    MvParams p{};
    float* h = hidden[hiddenIdx];
    p.seg[0] = MvSeg{L.wo.w, L.wo.scales, nullptr, h, dim};
    p.nseg = 1; p.K = dim; p.act = attnOut; p.resid = h;
    return p;
}
MvParams HIPFusedInference::gateUpParams(const LayerWeights& L) const {
    MvParams p{};
    p.seg[0] = MvSeg{L.gate.w, L.gate.scales, nullptr, ffnMid, ffnDim};
    p.seg[1] = MvSeg{L.up.w, L.up.scales, nullptr, nullptr, ffnDim};
    p.nseg = 2; p.K = dim; p.act = hidden[hiddenIdx]; p.gain = L.norm2; p.eps = eps;
    return p;
}
MvParams HIPFusedInference::downParams(const LayerWeights& L) const {
    MvParams p{};
    float* h = hidden[hiddenIdx];
    p.seg[0] = MvSeg{L.down.w, L.down.scales, nullptr, h, dim};
    p.nseg = 1; p.K = ffnDim; p.act = ffnMid; p.resid = h;
    return p;
}

// What the idle part of layer `layer`'s attention launch fetches into L2: the launches that follow it,
// in their order -- Wo, gate|up, down, the next layer's q|k|v and Wo -- as long as the helpers can
// have it in before the attention itself is done (a budget in bytes) and the lines will still be
// there when they are wanted (what flows through the L2s in between stays under their size).  A
// launch too large for what is left of the budget is taken in part -- the rows its first
// workgroups read, which fills the idle start of that launch -- and ends the list.  A layer small
// enough for its successor's Wo to stay gets that one instead of its own (which came with the
// launch before): it need not be in by the end of this launch.
void HIPFusedInference::planPrefetch(const LayerWeights& L, const LayerWeights* next, int layer, PfJob& job) const {
    job = PfJob{};
    if (execMode != 1 && execMode != 3 && execMode != 4) return;
    const size_t budget = (size_t)12 << 20;       // measured: 10.6 MB make the attention launch 0.3 us longer, 15 MB 3 us
    const size_t l2 = (size_t)24 << 20;           // of 8 x 4 MB
    const LayerWeights* N = nullptr;
    if (next && layer + 1 < nLayers) {
        const LayerWeights& C = *next;
        const bool uniform = C.wq.kind == C.wk.kind && C.wk.kind == C.wv.kind && C.gate.kind == C.up.kind;
        if (layerComplete(C) && uniform && kCache[layer + 1]) N = &C;
    }
    const size_t nextQkv = N ? N->wq.bytes + N->wk.bytes + N->wv.bytes : 0;
    const bool nextWoStays = N && L.wo.bytes + L.gate.bytes + L.up.bytes + L.down.bytes + nextQkv + N->wo.bytes <= l2;
    // the regions wanted last are listed first: they go to the helper workgroups that start first
    // (measured: 0.3 % of the step against the other order)
    PfJob late{}, soon{};
    size_t taken = 0, flowed = 0;
    bool open = true;                              // nothing after a launch that was taken in part or not at all
    const size_t minPart = (size_t)4 << 20;       // a launch that does not fit is taken in part (its first rows) if that much room is left
    auto considerFor = [&](PfJob& j, size_t bytes, bool needWhole, auto&& plan) {
        const size_t room = budget > taken ? budget - taken : 0;
        if (open && flowed + (bytes < room ? bytes : room) <= l2 && (bytes <= room || (!needWhole && room >= minPart))) {
            PfJob k = j;
            const size_t got = plan(k, bytes <= room ? (size_t)0 : room);
            if (got && late.nregion + soon.nregion + (k.nregion - j.nregion) <= PF_MAX_REGIONS) { j = k; taken += got; }
            if (bytes > room) open = false;
        }
        flowed += bytes;
    };
    if (nextWoStays) flowed += L.wo.bytes;
    else considerFor(soon, L.wo.bytes, false, [&](PfJob& k, size_t lim) { return plan_matvec_prefetch(L.wo.kind, EPI_RESID, PRO_PLAIN, woParams(L), k, lim); });
    considerFor(soon, L.gate.bytes + L.up.bytes, false,
                [&](PfJob& k, size_t lim) { return plan_matvec_prefetch(L.gate.kind, EPI_SWIGLU, PRO_RMS, gateUpParams(L), k, lim); });
    considerFor(soon, L.down.bytes, true, [&](PfJob& k, size_t lim) { return plan_matvec_prefetch(L.down.kind, EPI_RESID, PRO_PLAIN, downParams(L), k, lim); });
    if (N) {
        considerFor(late, nextQkv, true, [&](PfJob& k, size_t lim) { return plan_matvec_prefetch(N->wq.kind, EPI_QKV, PRO_RMS, qkvParams(*N, layer + 1, nullptr, 0), k, lim); });
        if (nextWoStays)
            considerFor(late, N->wo.bytes, true, [&](PfJob& k, size_t lim) { return plan_matvec_prefetch(N->wo.kind, EPI_RESID, PRO_PLAIN, woParams(*N), k, lim); });
    }
    PfJob j = late;
    for (int i = 0; i < soon.nregion && j.nregion < PF_MAX_REGIONS; i++) j.region[j.nregion++] = soon.region[i];
    if (j.nregion == 0) return;
    j.helperWaves = 960;          // measured: half as many are too slow, twice as many disturb the attention workgroups
    job = j;
}

int HIPFusedInference::enqueueLayerFused(const LayerWeights& L, int layer, const StepState* st, int posImm) {
    if (mark(1)) return MG_E_HIP;
    {
        MvParams p = qkvParams(L, layer, st, posImm);
        HIPCHK(launch_matvec(L.wq.kind, EPI_QKV, PRO_RMS, p, nullptr, stream));
    }
    if (mark(2)) return MG_E_HIP;
    {
        AttnParams a{};
        a.kvHalf = kvHalf;
        a.q = Q; a.Kc = kCache[layer]; a.Vc = vCache[layer];
        a.state = st; a.posImm = posImm; a.rowLimit = maxSeq;
        a.kvDim = kvDim; a.nHeads = nHeads; a.nKVHeads = nKVHeads; a.headDim = headDim;
        a.smax = smax; a.splitLen = splitLen; a.headsPerWG = attnHeadsPerWG;
        a.pm = pm; a.pl = pl; a.pacc = pacc; a.counters = attnCounters; a.out = attnOut;
        // the weights this launch was given (a streamed layer's device copy is not the resident slot), and the
        // resident successor only when this layer is the resident one itself
        const bool resident = &L == &layers[layer];
        planPrefetch(L, resident && layer + 1 < nLayers ? &layers[layer + 1] : nullptr, layer, a.pf);
        HIPCHK(launch_attention(a, stream));
    }
    if (mark(3)) return MG_E_HIP;
    {
        MvParams p = woParams(L);
        HIPCHK(launch_matvec(L.wo.kind, EPI_RESID, PRO_PLAIN, p, nullptr, stream));
    }
    if (mark(4)) return MG_E_HIP;
    {
        MvParams p = gateUpParams(L);
        HIPCHK(launch_matvec(L.gate.kind, EPI_SWIGLU, PRO_RMS, p, nullptr, stream));
    }
    if (mark(5)) return MG_E_HIP;
    {
        MvParams p = downParams(L);
        HIPCHK(launch_matvec(L.down.kind, EPI_RESID, PRO_PLAIN, p, nullptr, stream));
    }
    return MG_OK;
}

// ---- all layers of a step in one persistent launch (flow.hip) ----
// Two such launches at once on one GPU could each hold part of the CUs and wait for workgroups that cannot start,
// until their waits run out.  So on every device one context at a time uses the launch: the first that needs it, until
// it is destroyed or set to another mode; the others run the fused launches meanwhile.
static std::mutex g_flowOwnerMutex;
static const HIPFusedInference* g_flowOwner[64] = {};
static bool claim_flow(const HIPFusedInference* f, int dev) {
    if (dev < 0 || dev >= 64) return false;
    std::lock_guard<std::mutex> lk(g_flowOwnerMutex);
    if (!g_flowOwner[dev]) g_flowOwner[dev] = f;
    return g_flowOwner[dev] == f;
}
void HIPFusedInference::releaseFlow() {
    bool owner = false;
    {
        std::lock_guard<std::mutex> lk(g_flowOwnerMutex);
        for (auto& o : g_flowOwner) if (o == this) owner = true;
    }
    if (!owner) return;
    // the launch changes hands only once this context's last one has ended: the next owner's launch must not meet it on the GPU
    if (stream) (void)hipStreamSynchronize(stream);
    std::lock_guard<std::mutex> lk(g_flowOwnerMutex);
    for (auto& o : g_flowOwner) if (o == this) o = nullptr;
}

// The reference's integer Q4_0 matvecs in the op-by-op loop (exec mode 0): activations quantized to int8 blocks.
int HIPFusedInference::SetQ4ActQuant(int on) {
    if (!built) return MG_E_NOT_BUILT;
    if (on && execMode != 0) { set_error("SetQ4ActQuant: only the op-by-op loop (exec mode 0) has the integer matvecs"); return MG_E_STATE; }
    if (on && !q8Scratch) {
        const int q8MaxK = std::max(dim, ffnDim);                      // cuda_fused_infer.go:175-176
        HIPCHK(hipMalloc(&q8Scratch, (size_t)(q8MaxK / 32 + 1) * 40));
    }
    q4ActQuant = on != 0;
    return MG_OK;
}

// Modes 3 and 4 lay the launch out for different numbers of computing workgroups: drop what was sized for the other
// (ensureFlow builds it again).
void HIPFusedInference::flowRegeometry() {
    if (!dFlowLayers) return;
    if (stream) (void)hipStreamSynchronize(stream);
    (void)hipFree(dFlowLayers); dFlowLayers = nullptr;
    if (flowXchg) { (void)hipFree(flowXchg); flowXchg = nullptr; }
    if (dFlowTail) { (void)hipFree(dFlowTail); dFlowTail = nullptr; }
    if (dFlowErr) { (void)hipFree(dFlowErr); dFlowErr = nullptr; }
    if (hFlowErr) { (void)hipHostFree(hFlowErr); hFlowErr = nullptr; }
    if (flowTrace) { (void)hipFree(flowTrace); flowTrace = nullptr; }
    flowGrid = 0; flowCompute = 0;
}

// Of cus resident workgroups, how many compute: all but the prefetchers where the attention phase (one workgroup per
// head and KV split) then still covers the context, else all of them; 0 if the launch cannot cover it at all.
int HIPFusedInference::flowComputeWgs(int cus) const {
    size_t layerBytes = 0;
    if (!layers.empty()) {
        const LayerWeights& L = layers[0];
        layerBytes = L.wq.bytes + L.wk.bytes + L.wv.bytes + L.wo.bytes + L.gate.bytes + L.up.bytes + L.down.bytes;
    }
    const int pf = execMode == 4 ? 0 : flow_prefetch_workgroups(cus, layerBytes, dim, kvDim, ffnDim);
    const int tries[2] = {cus - pf, cus};
    for (int nC : tries) {
        const FlowGeometry g = flow_geometry(dim, kvDim, ffnDim, nHeads, nKVHeads, headDim, maxSeq, nC);
        // (the same limits as launch_flow_layers checks: a shape it would refuse runs the fused launches instead)
        if (flow_min_grid(nHeads, nKVHeads, g) <= nC && flow_context_fits(maxSeq, g) && flow_grid_fits(ffnDim, nHeads, g, nC) &&
            (size_t)nLayers * g.stride * 4 < (1ull << 31)) return nC;
    }
    return 0;
}

bool HIPFusedInference::flowEligible(int l0, int l1) const {
    if ((execMode != 3 && execMode != 4) || flowBroken) return false;
    if (!flow_shape_supported(dim, kvDim, ffnDim, nHeads, nKVHeads, headDim)) return false;
    if (l1 > nLayers) l1 = nLayers;
    if (l0 < 0 || l0 >= l1) return false;
    for (int l = l0; l < l1; l++) {
        const LayerWeights& L = layers[l];
        if (!layerComplete(L) || !kCache[l] || !vCache[l]) return false;
        // one format for all matrices of all layers: Q8, or Q4_0 in the split layout (whole blocks: rows of a multiple of 32)
        const DevMat* ms[7] = {&L.wq, &L.wk, &L.wv, &L.wo, &L.gate, &L.up, &L.down};
        const int kind = layers[l0].wq.kind;
        if (kind != WF_Q8 && kind != WF_Q4P) return false;
        for (const DevMat* m : ms) if (m->kind != kind || (kind == WF_Q4P && m->cols % 32)) return false;
    }
    // one workgroup per CU, all resident at once; a (query head, KV split) per workgroup in the attention phase
    int cus = flowGrid;
    if (cus == 0) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) { (void)hipGetLastError(); return false; }
        cus = prop.multiProcessorCount;
    }
    if (flowComputeWgs(cus) == 0) return false;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) { (void)hipGetLastError(); return false; }
    return claim_flow(this, dev);
}

int HIPFusedInference::ensureFlow() {
    if (!dFlowLayers) {
        int dev = 0;
        hipDeviceProp_t prop;
        HIPCHK(hipGetDevice(&dev));
        HIPCHK(hipGetDeviceProperties(&prop, dev));
        flowGrid = prop.multiProcessorCount;
        flowCompute = flowComputeWgs(flowGrid);
        flowGeo = flow_geometry(dim, kvDim, ffnDim, nHeads, nKVHeads, headDim, maxSeq, flowCompute);
        void* v = nullptr;
        HIPCHK(hipMalloc(&v, sizeof(FlowLayer) * (size_t)nLayers));
        dFlowLayers = static_cast<FlowLayer*>(v);
        HIPCHK(hipMalloc(&v, sizeof(float) * flow_xchg_floats(flowGeo, nLayers, flowGrid)));
        flowXchg = static_cast<float*>(v);
        HIPCHK(launch_flow_reset_all(flowXchg, flowGeo, nLayers, flowGrid, stream));
        HIPCHK(hipMalloc(&v, sizeof(FlowTail)));
        dFlowTail = static_cast<FlowTail*>(v);
        HIPCHK(hipMalloc(&v, FLOW_ERR_BYTES));
        dFlowErr = static_cast<int*>(v);
        HIPCHK(hipMemsetAsync(dFlowErr, 0, FLOW_ERR_BYTES, stream));
        HIPCHK(hipHostMalloc(&v, 64, hipHostMallocDefault));
        hFlowErr = static_cast<int*>(v);
        *hFlowErr = 0;
        flowTableDirty = true;
    }
    if (flowTableDirty) {
        std::vector<FlowLayer> t((size_t)nLayers);
        for (int l = 0; l < nLayers; l++) {
            const LayerWeights& L = layers[l];
            FlowLayer& F = t[l];
            F = FlowLayer{};
            F.g1 = L.norm1; F.g2 = L.norm2;
            auto w8 = [](const DevMat& m) { return static_cast<const signed char*>(m.w); };
            // Q8: the per-row scales; Q4_0: the fp16 d plane, which follows the nibble plane [rows, cols/2]
            auto aux = [](const DevMat& m) -> const float* {
                if (m.kind != WF_Q4P) return m.scales;
                return reinterpret_cast<const float*>(static_cast<const char*>(m.w) + (size_t)m.rows * (m.cols >> 1));
            };
            F.wq = w8(L.wq); F.wk = w8(L.wk); F.wv = w8(L.wv); F.wo = w8(L.wo); F.gate = w8(L.gate); F.up = w8(L.up); F.down = w8(L.down);
            F.sq = aux(L.wq); F.sk = aux(L.wk); F.sv = aux(L.wv); F.so = aux(L.wo);
            F.sgate = aux(L.gate); F.sup = aux(L.up); F.sdown = aux(L.down);
            F.bq = L.bq; F.bk = L.bk; F.bv = L.bv;
            F.Kc = kCache[l]; F.Vc = vCache[l];
        }
        FlowTail T{};
        if (finalNorm && lmHead.w) {
            T.finalGain = finalNorm;
            T.lmW = static_cast<const signed char*>(lmHead.w);
            T.lmAux = lmHead.kind == WF_Q4P
                          ? reinterpret_cast<const float*>(static_cast<const char*>(lmHead.w) + (size_t)lmHead.rows * (lmHead.cols >> 1))
                          : lmHead.scales;
            T.logits = logits;
            if (embedKind == 1 || embedKind == 2) { T.embKind = embedKind; T.embTable = embedTable; }
            else { T.embKind = lmHead.kind == WF_Q8 ? 0 : 3; T.embTable = lmHead.w; T.embScales = lmHead.scales; }
            T.cosTab = cosTab; T.sinTab = sinTab;
            T.state = dState; T.history = dHistory; T.historyCap = maxSeq + 1; T.prompt = dPrompt;
            T.amax = flow_amax_area(flowXchg, flowGeo, nLayers);
            T.ropeCur = ropeCur;
            T.vocab = vocabSize;
        }
        HIPCHK(hipStreamSynchronize(stream));
        HIPCHK(hipMemcpy(dFlowLayers, t.data(), sizeof(FlowLayer) * (size_t)nLayers, hipMemcpyHostToDevice));
        HIPCHK(hipMemcpy(dFlowTail, &T, sizeof(FlowTail), hipMemcpyHostToDevice));
        flowTableDirty = false;
    }
    return MG_OK;
}

// Diagnostic: per-workgroup timestamps of the persistent launch (flow.h: FLOW_TRACE_SLOTS per layer).  enable != 0
// starts recording (graphs are re-captured with the trace pointer), out != NULL copies the last launch's ticks
// [layer][slot][workgroup] (100 MHz wall clock), dims gets {layers, slots, workgroups}; enable == 0 stops.
int HIPFusedInference::FlowTrace(int enable, long long* out, size_t cap, int* dims) {
    if (!flowEligible(0, nLayers)) { set_error("flow trace: the persistent launch is not in use for this model (exec mode, weight kinds, shape)"); return MG_E_STATE; }
    if (int rc = ensureFlow()) return rc;
    // one more block than layers: the tail of a token (FlowTailTrace)
    const size_t n = (size_t)nLayers * FLOW_TRACE_SLOTS * (size_t)flowCompute, nAll = (size_t)(nLayers + 1) * FLOW_TRACE_SLOTS * (size_t)flowCompute;
    HIPCHK(hipStreamSynchronize(stream));
    if (dims) { dims[0] = nLayers; dims[1] = FLOW_TRACE_SLOTS; dims[2] = flowCompute; }
    if (enable && !flowTrace) {
        void* v = nullptr;
        HIPCHK(hipMalloc(&v, sizeof(long long) * nAll));
        flowTrace = static_cast<long long*>(v);
        HIPCHK(hipMemsetAsync(v, 0, sizeof(long long) * nAll, stream));
        HIPCHK(hipStreamSynchronize(stream));
        invalidateGraphs();
    }
    if (out && flowTrace) {
        if (cap < n) { set_error("flow trace: buffer too small"); return MG_E_ARG; }
        HIPCHK(hipMemcpy(out, flowTrace, sizeof(long long) * n, hipMemcpyDeviceToHost));
    }
    if (!enable && flowTrace) {
        invalidateGraphs();
        (void)hipFree(flowTrace);
        flowTrace = nullptr;
    }
    return MG_OK;
}

// The tail's part of the trace (FLOW_TAIL_TRACE_NAMES: six points) of the last token a launch ran, while the trace is
// enabled: ticks [point][workgroup]; dims gets {4, workgroups}.
int HIPFusedInference::FlowTailTrace(long long* out, size_t cap, int* dims) {
    if (!flowTrace || !flowTailEligible()) { set_error("flow tail trace: enable the trace first (and the launch must run whole tokens)"); return MG_E_STATE; }
    const size_t n = (size_t)6 * flowCompute;
    if (dims) { dims[0] = 6; dims[1] = flowCompute; }
    if (!out) return MG_OK;
    if (cap < n) { set_error("flow tail trace: buffer too small"); return MG_E_ARG; }
    HIPCHK(hipStreamSynchronize(stream));
    HIPCHK(hipMemcpy(out, flowTrace + (size_t)nLayers * FLOW_TRACE_SLOTS * (size_t)flowCompute, sizeof(long long) * n, hipMemcpyDeviceToHost));
    return MG_OK;
}

int HIPFusedInference::enqueueLayersFlow(int l0, int l1, const StepState* st, int posImm, bool resetFirst, int nTokens) {
    if (l1 > nLayers) l1 = nLayers;
    FlowParams p{};
    p.layers = dFlowLayers; p.l0 = l0; p.l1 = l1; p.nLayersTotal = nLayers;
    p.dim = dim; p.kvDim = kvDim; p.ffn = ffnDim; p.nHeads = nHeads; p.nKVHeads = nKVHeads; p.headDim = headDim; p.maxSeq = maxSeq;
    p.q4 = layers[l0].wq.kind == WF_Q4P ? 1 : 0;
    p.nCompute = flowCompute;
    p.kvHalf = kvHalf;
    p.downSplit = (dim <= 2048 && 2 * dim <= flowCompute * 8 && ffnDim >= 2048) ? 1 : 0;
    {
        // attention-idle prefetch: Wo where a wave holds only part of its rows ahead (rows of more than 2048 weights); of
        // gate and up the leading rows that fit the L2s beside what is in use, 2.5 MB an XCD (1.1B shape: 5120 of 5632
        // rows 0.423 ms a token, all of them 0.431, 4096 0.435), where that is most of them; else half of their first
        // round of rows
        const LayerWeights& L0 = layers[l0];
        p.idleWoRows = dim > 2048 ? dim : 0;
        const int firstRound = std::min(ffnDim, flowCompute * 8);
        const size_t rowBytes = ffnDim > 0 ? (L0.gate.bytes + L0.up.bytes) / (size_t)ffnDim : 1;      // a gate row and its up row
        const int fit = (int)std::min<size_t>((size_t)ffnDim, (((size_t)5 << 19) * 8) / (rowBytes ? rowBytes : 1)) & ~63;
        p.idleGateUpRows = (L0.gate.bytes + L0.up.bytes) / 8 <= ((size_t)3 << 20) ? fit : (firstRound / 2) & ~63;
    }
    p.eps = eps;
    p.state = st; p.posImm = posImm;
    const int half = headDim / 2;
    p.cosRow = st ? ropeCur : cosTab + (size_t)posImm * half;
    p.sinRow = st ? ropeCur + half : sinTab + (size_t)posImm * half;
    p.hidden = hidden[hiddenIdx];
    p.xchg = flowXchg; p.geo = flowGeo;
    p.err = dFlowErr;
    p.limitTicks = flowLimitTicks;
    {
        // the last position this launch can reach, where the host knows it: the plain attention variant serves while a
        // workgroup per query head and KV split fits the launch, also in a context laid out for grouped attention
        long long posMax = -1;
        if (!st) posMax = posImm;
        else if (statePosHost >= 0) posMax = (long long)statePosHost + (nTokens > 0 ? nTokens - 1 : 0);
        p.gqaCode = (posMax < 0 || (long long)nHeads * (posMax / FLOW_TILE + 1) > flowCompute) ? 1 : 0;
        p.generic = flowGeneric ? 1 : 0;
        if (st && nTokens > 0 && statePosHost >= 0) statePosHost += nTokens;          // whole tokens advance the device state
        else if (st) statePosHost = -1;                                               // (what follows this launch advances it)
    }
    p.trace = flowTrace;
    if (nTokens > 0) { p.nTokens = nTokens; p.tail = dFlowTail; }
    if (resetFirst) HIPCHK(launch_flow_reset(flowXchg, flowGeo, l0, l1, stream));
    if (mark(1)) return MG_E_HIP;
    HIPCHK(launch_flow_layers(p, flowGrid, stream));
    return MG_OK;
}

// nTokens whole tokens from the device state in one launch: embedding, layers, final norm, lm_head, argmax; the
// exchange area must be in its reset state for the first token's position (setState), the launch leaves it so for
// the position after its last.
int HIPFusedInference::enqueueTokensFlow(int nTokens) {
    return enqueueLayersFlow(0, nLayers, dState, 0, false, nTokens);
}

// Whole tokens in the launch need: the tail's operands set, the lm_head in the layers' format, room in LDS for the
// embedding beside the staged vector.
bool HIPFusedInference::flowTailEligible() const {
    if (!flowTail || !flowEligible(0, nLayers)) return false;
    if (!finalNorm || !lmHead.w || lmHead.kind != layers[0].wq.kind || lmHead.cols != dim || lmHead.rows != vocabSize) return false;
    if (lmHead.kind == WF_Q4P && dim % 32) return false;
    const FlowGeometry g = flowGrid ? flowGeo : flow_geometry(dim, kvDim, ffnDim, nHeads, nKVHeads, headDim, maxSeq, 8);
    const int gqa = flowGrid ? flowGeo.gqa : 1;        // before the launch is set up: the larger bound
    (void)g;
    return flow_lds_bytes(dim, ffnDim, headDim, gqa, true) <= ((size_t)160 << 10);
}

int HIPFusedInference::SetTokensPerLaunch(int n) {
    if (n < 1 || n > 4096) { set_error("tokens per launch must be between 1 and 4096"); return MG_E_ARG; }
    tokensPerLaunch = n;
    return MG_OK;
}

// Sets the device-resident step state; where the persistent launch runs whole tokens, also leaves its exchange area
// reset (a token expects the half of its position's parity so, and resets the other for its successor).
int HIPFusedInference::setState(int pos, int token, int count, int nPrompt) {
    HIPCHK(launch_set_state(dState, pos, token, count, nPrompt, ropeRef(), stream));
    statePosHost = pos;
    if (flowXchg && (execMode == 3 || execMode == 4)) HIPCHK(launch_flow_reset_all(flowXchg, flowGeo, nLayers, flowGrid, stream));
    return MG_OK;
}

// nTokens decode steps from the device state: runs of tokens inside the persistent launch where that is in use, else
// graph replays or eager launches of single tokens.
bool HIPFusedInference::runsInLaunch(bool useGraph) const { return useGraph && tokensPerLaunch > 1 && flowTailEligible(); }

int HIPFusedInference::decodeRun(int nTokens, bool useGraph) {
    if (runsInLaunch(useGraph)) {
        int rc = ensureFlow();
        for (int done = 0; done < nTokens && rc == MG_OK;) {
            const int n = std::min(tokensPerLaunch, nTokens - done);
            rc = enqueueTokensFlow(n);
            done += n;
        }
        return rc;
    }
    for (int i = 0; i < nTokens; i++) {
        statePosHost = -1;                          // (advanced on the device by launches that do not tell the host)
        if (useGraph) HIPCHK(hipGraphLaunch(execFull, stream));
        else { int rc = enqueueToken(true); if (rc) return rc; }
    }
    return MG_OK;
}

// After a synchronisation: did a wait of the persistent launch give up?  (Its workgroups were then not all
// resident at once -- a GPU shared with other work, fewer CUs than reported.)  The step's results are not
// valid; later steps use the separate launches.
int HIPFusedInference::checkFlowError() {
    if (!dFlowErr) return MG_OK;
    HIPCHK(hipMemcpy(hFlowErr, dFlowErr, sizeof(int), hipMemcpyDeviceToHost));
    if (*hFlowErr == 0) return MG_OK;
    const int code = *hFlowErr;
    *hFlowErr = 0;
    HIPCHK(hipMemsetAsync(dFlowErr, 0, sizeof(int), stream));
    HIPCHK(hipStreamSynchronize(stream));
    flowBroken = true;
    releaseFlow();
    invalidateGraphs();
    if (code == 3)
        set_error("persistent layer launch: the variant without grouped attention was given a position it does not cover; "
                  "this step's results are invalid, later steps use the separate launches");
    else
        set_error("persistent layer launch: a wait between phases ran into its time limit (workgroups not all resident at once?); "
                  "this step's results are invalid, later steps use the separate launches");
    return MG_E_HIP;
}

int HIPFusedInference::enqueueLayer(const LayerWeights& L, int layer, const StepState* st, int posImm) {
    if (!kCache[layer] || !vCache[layer]) { set_error("layer has no KV cache: call SetLayerRange first"); return MG_E_STATE; }
    if (!layerComplete(L)) { set_error("layer weights incomplete"); return MG_E_STATE; }
    // the fused QKV and gate/up launches read their matrices with one kernel: same format needed
    const bool uniform = L.wq.kind == L.wk.kind && L.wk.kind == L.wv.kind && L.gate.kind == L.up.kind;
    if (execMode == 0 || !uniform) {
        if (st) { set_error("per-op launches need a host-side position (mixed weight formats in a layer, or exec mode 0)"); return MG_E_STATE; }
        return enqueueLayerPerOp(L, layer, posImm);
    }
    return enqueueLayerFused(L, layer, st, posImm);
}

// Final norm + lm_head (cuda_fused_infer.go:446-448) with the per-workgroup
// argmax folded into the matvec epilogue.
int HIPFusedInference::enqueueFinal(bool withArgmax) {
    if (withArgmax) statePosHost = -1;              // (the argmax's last kernel advances the device state)
    if (!finalNorm || !lmHead.w) { set_error("final norm / lm_head not set"); return MG_E_STATE; }
    if (execMode == 0 && q4ActQuant && lmHead.kind == WF_Q4P) {
        // the reference's tail with its integer matvec (cuda_fused_infer_q4.go:600-601): norm, quantize, lm_head; then
        // the argmax over the finished logits
        HIPCHK(launch_rmsnorm_out(hidden[hiddenIdx], normed, finalNorm, 1, dim, eps, stream));
        HIPCHK(launch_q8_quantize_act(normed, q8Scratch, dim, 1, stream));
        HIPCHK(launch_q4_0_dp4a(lmHead.w, true, q8Scratch, logits, vocabSize, dim, 1, stream));
        if (withArgmax) {
            const int parts = std::max(1, std::min(std::min(amaxParts, 256), (vocabSize + 255) / 256));
            HIPCHK(launch_argmax_slices(logits, vocabSize, parts, amaxVal, amaxIdx, stream));
            HIPCHK(launch_argmax_finish(amaxVal, amaxIdx, parts, dState, nullptr, dHistory, maxSeq + 1, vocabSize, ropeRef(), embedRef(), stream));
        }
        return MG_OK;
    }
    MvParams p{};
    p.seg[0] = MvSeg{lmHead.w, lmHead.scales, nullptr, logits, vocabSize};
    p.nseg = 1; p.K = dim; p.act = hidden[hiddenIdx]; p.gain = finalNorm; p.eps = eps;
    p.amaxVal = amaxVal; p.amaxIdx = amaxIdx;
    if (fuseEmbed && flowEligible(0, nLayers)) {
        // inside the captured token: the lm_head launch also leaves the exchange area of the persistent
        // layer launch in its "nothing written yet" state for the next token (one launch saved)
        p.xreset = reinterpret_cast<unsigned*>(flowXchg);
        p.xresetWords = (unsigned)((size_t)nLayers * flowGeo.stride);
    }
    MvConfig c{0, 0, 0};
    if (mark(6)) return MG_E_HIP;
    HIPCHK(launch_matvec(lmHead.kind, EPI_ARGMAX, PRO_RMS, p, &c, stream));
    if (mark(7)) return MG_E_HIP;
    if (withArgmax) {
        if (c.grid > amaxParts) { set_error("argmax partial buffer too small"); return MG_E_STATE; }
        HIPCHK(launch_argmax_finish(amaxVal, amaxIdx, c.grid, dState, nullptr, dHistory, maxSeq + 1, vocabSize, ropeRef(), embedRef(), stream));
    }
    return MG_OK;
}

int HIPFusedInference::PartialStep(const float* hiddenIn, int pos, int layerStart, int layerEnd, float* hiddenOut,
                                   float* logitsOut) {
    if (!built) return MG_E_NOT_BUILT;
    ARGCHK(pos >= 0 && pos < maxSeq, "PartialStep: pos out of range");
    ARGCHK(layerStart >= 0, "PartialStep: negative layerStart");
    float* h = hidden[hiddenIdx];
    if (hiddenIn) {
        HIPCHK(hipStreamSynchronize(stream));
        HIPCHK(hipMemcpy(h, hiddenIn, (size_t)dim * 4, hipMemcpyHostToDevice));      // :395
    }
    const bool flow = flowEligible(layerStart, layerEnd);
    if (flow) {
        int rc = ensureFlow();
        if (rc == 0) rc = enqueueLayersFlow(layerStart, layerEnd, nullptr, pos, true);
        if (rc) return rc;
    } else {
        for (int l = layerStart; l < layerEnd && l < nLayers; l++) {
            if (!layers[l].norm1) continue;                                           // :415
            int rc = enqueueLayer(layers[l], l, nullptr, pos);
            if (rc) return rc;
        }
    }
    if (layerEnd >= nLayers && logitsOut && finalNorm) {                              // :446
        int rc = enqueueFinal(false);
        if (rc) return rc;
        HIPCHK(hipStreamSynchronize(stream));
        HIPCHK(hipMemcpy(logitsOut, logits, (size_t)vocabSize * 4, hipMemcpyDeviceToHost));
        rc = checkFlowError();
        if (rc) return rc;
    }
    if (hiddenOut && layerEnd < nLayers) {                                            // :452
        HIPCHK(hipStreamSynchronize(stream));
        HIPCHK(hipMemcpy(hiddenOut, h, (size_t)dim * 4, hipMemcpyDeviceToHost));
        int rc = checkFlowError();
        if (rc) return rc;
    }
    // Nothing read back: the launches stay queued (the reference does not sync here either) -- except after a
    // persistent launch, whose waits may have run out: that is reported by the call whose step it spoiled.
    if (flow && !(layerEnd >= nLayers && logitsOut && finalNorm) && !(hiddenOut && layerEnd < nLayers)) {
        HIPCHK(hipStreamSynchronize(stream));
        return checkFlowError();
    }
    return MG_OK;
}

// ---- L3 bridge and mailbox (cuda_fused_infer.go:556-737) ----
int HIPFusedInference::QueueHiddenToL3() {
    if (!built) return MG_E_NOT_BUILT;
    HIPCHK(hipEventRecord(computeDone, stream));
    HIPCHK(hipStreamWaitEvent(copyStream, computeDone, 0));
    HIPCHK(hipMemcpyAsync(l3 + 64, hidden[hiddenIdx], (size_t)dim * 4, hipMemcpyDeviceToHost, copyStream));
    return MG_OK;
}

int HIPFusedInference::WaitL3() {
    if (!built) return MG_E_NOT_BUILT;
    HIPCHK(hipStreamSynchronize(copyStream));
    return MG_OK;
}

const float* HIPFusedInference::GetL3Hidden() const {
    return l3 ? reinterpret_cast<const float*>(l3 + 64) : nullptr;
}

int HIPFusedInference::SignalMailbox() {
    if (!built) return MG_E_NOT_BUILT;
    mailboxSignaled++;
    HIPCHK(launch_signal_mailbox(reinterpret_cast<unsigned*>(l3), mailboxSignaled, stream));
    return MG_OK;
}

int HIPFusedInference::WaitMailbox(int timeoutMs) {
    if (!built) return MG_E_NOT_BUILT;
    ARGCHK(timeoutMs > 0, "WaitMailbox: timeout must be positive");
    if (mailboxSignaled < mailboxExpected) { set_error("WaitMailbox: no signal queued for this stage"); return MG_E_STATE; }
    volatile unsigned* counter = reinterpret_cast<volatile unsigned*>(l3);
    const auto t0 = std::chrono::steady_clock::now();
    while (*counter < mailboxExpected) {
        if (std::chrono::steady_clock::now() - t0 > std::chrono::milliseconds(timeoutMs)) {
            set_error("WaitMailbox: timed out");
            return MG_E_HIP;
        }
    }
    mailboxExpected++;
    return MG_OK;
}

int HIPFusedInference::SwapHiddenBuffer() {
    if (!built) return MG_E_NOT_BUILT;
    HIPCHK(hipStreamSynchronize(stream));
    hiddenIdx = 1 - hiddenIdx;
    return invalidateGraphs();                // captured launches point at the other buffer
}

int HIPFusedInference::StepLayerResident(int layer, int pos, const float* hiddenIn, float* preOut, float* postOut,
                                         float* logitsOut) {
    if (!built) return MG_E_NOT_BUILT;
    ARGCHK(layer >= 0 && layer < nLayers && pos >= 0 && pos < maxSeq, "StepLayerResident: bad layer or pos");
    float* h = hidden[hiddenIdx];
    if (layer == 0) {
        ARGCHK(hiddenIn, "StepLayerResident: layer 0 needs hiddenIn");
        HIPCHK(hipStreamSynchronize(stream));
        HIPCHK(hipMemcpy(h, hiddenIn, (size_t)dim * 4, hipMemcpyHostToDevice));
    }
    if (preOut) {
        HIPCHK(hipStreamSynchronize(stream));
        HIPCHK(hipMemcpy(preOut, h, (size_t)dim * 4, hipMemcpyDeviceToHost));
    }
    int rc = enqueueLayer(layers[layer], layer, nullptr, pos);
    if (rc) return rc;
    if (postOut) {
        HIPCHK(hipStreamSynchronize(stream));
        HIPCHK(hipMemcpy(postOut, h, (size_t)dim * 4, hipMemcpyDeviceToHost));
    }
    if (logitsOut) {
        rc = enqueueFinal(false);
        if (rc) return rc;
        HIPCHK(hipStreamSynchronize(stream));
        HIPCHK(hipMemcpy(logitsOut, logits, (size_t)vocabSize * 4, hipMemcpyDeviceToHost));
    }
    HIPCHK(hipStreamSynchronize(stream));
    return MG_OK;
}

int HIPFusedInference::ExportHidden(float* out) {
    if (!built) return MG_E_NOT_BUILT;
    ARGCHK(out, "ExportHidden: NULL out");
    HIPCHK(hipStreamSynchronize(stream));
    HIPCHK(hipMemcpy(out, hidden[hiddenIdx], (size_t)dim * 4, hipMemcpyDeviceToHost));
    return checkFlowError();
}

int HIPFusedInference::enqueueEmbed() {
    float* h = hidden[hiddenIdx];
    if (mark(0)) return MG_E_HIP;
    if (embedKind == 1 || embedKind == 2) {
        HIPCHK(launch_embed_token(embedKind, embedTable, nullptr, dState, h, dim, vocabSize, stream));
    } else {
        if (!lmHead.w) { set_error("no embedding table and no lm_head to tie to"); return MG_E_STATE; }
        int kind = lmHead.kind == WF_Q8 ? 0 : 3;
        HIPCHK(launch_embed_token(kind, lmHead.w, lmHead.scales, dState, h, dim, vocabSize, stream));
    }
    return MG_OK;
}

// One whole token from the device-resident state.
// Inside the captured graphs the embedding of the next token is written by the kernel that chooses
// it (argmax finish / prompt advance), one launch fewer a token: a graph then starts from a hidden
// buffer that already holds its token's embedding, and whoever sets the state by hand before a
// graph launch embeds once (primeGraph).  After graph launches the hidden buffer holds that next
// embedding, not the last hidden state; launches outside the graphs keep the separate embed kernel.
EmbedRef HIPFusedInference::embedRef() const {
    EmbedRef e{};
    if (!fuseEmbed) return e;
    if (embedKind == 1 || embedKind == 2) { e.kind = embedKind; e.table = embedTable; }
    else { e.kind = lmHead.kind == WF_Q8 ? 0 : 3; e.table = lmHead.w; e.scales = lmHead.scales; }
    e.out = hidden[hiddenIdx]; e.dim = dim; e.vocab = vocabSize;
    return e;
}
int HIPFusedInference::primeGraph() {
    // (a captured token leaves the exchange area reset for its successor; the first one finds it so from setState)
    return enqueueEmbed();
}

int HIPFusedInference::enqueueToken(bool withHead) {
    if (withHead && flowTailEligible()) {          // the whole token is one launch
        int rc = ensureFlow();
        return rc ? rc : enqueueTokensFlow(1);
    }
    int rc = fuseEmbed ? MG_OK : enqueueEmbed();
    if (rc) return rc;
    const bool flow = flowEligible(0, nLayers);
    if (flow) {
        rc = ensureFlow();
        if (rc == 0) rc = enqueueLayersFlow(0, nLayers, dState, 0, !fuseEmbed);
        if (rc) return rc;
    } else {
        for (int l = 0; l < nLayers; l++) {
            rc = enqueueLayer(layers[l], l, dState, 0);
            if (rc) return rc;
        }
    }
    if (withHead) return enqueueFinal(true);
    statePosHost = -1;
    HIPCHK(launch_advance_prompt(dState, dPrompt, ropeRef(), embedRef(), stream));
    // no lm_head launch to leave the exchange area reset for the next launch: a captured prompt step does it itself,
    // and so does any prompt step where whole tokens run in the launch (they expect to find it so)
    if (flow && (fuseEmbed || flowTailEligible())) HIPCHK(launch_flow_reset(flowXchg, flowGeo, 0, nLayers, stream));
    return MG_OK;
}

static int checkReady(HIPFusedInference* f) {
    for (int l = 0; l < f->nLayers; l++) {
        if (!layerComplete(f->layers[l])) { set_error("decode: layer weights incomplete"); return MG_E_STATE; }
        if (!f->kCache[l]) { set_error("decode: KV cache missing, call SetLayerRange(0, nLayers)"); return MG_E_STATE; }
    }
    if (!f->finalNorm || !f->lmHead.w) { set_error("decode: final norm / lm_head not set"); return MG_E_STATE; }
    return MG_OK;
}

int HIPFusedInference::DecodeToken(int token, int pos, int* nextToken, float* logitsOut) {
    if (!built) return MG_E_NOT_BUILT;
    ARGCHK(pos >= 0 && pos < maxSeq && token >= 0 && token < vocabSize, "DecodeToken: token or pos out of range");
    int rc = checkReady(this);
    if (rc) return rc;
    { int rcs = setState(pos, token, 0, 0); if (rcs) return rcs; }
    if (execMode == 0) {
        rc = enqueueEmbed();
        if (rc) return rc;
        for (int l = 0; l < nLayers; l++) {
            rc = enqueueLayerPerOp(layers[l], l, pos);
            if (rc) return rc;
        }
        rc = enqueueFinal(true);
    } else {
        rc = enqueueToken(true);
    }
    if (rc) return rc;
    HIPCHK(hipMemcpyAsync(hTokens, dHistory, sizeof(int), hipMemcpyDeviceToHost, stream));
    HIPCHK(hipStreamSynchronize(stream));
    if (nextToken) *nextToken = hTokens[0];
    if (logitsOut) HIPCHK(hipMemcpy(logitsOut, logits, (size_t)vocabSize * 4, hipMemcpyDeviceToHost));
    return checkFlowError();
}

int HIPFusedInference::GraphCapture() {
    if (!built) return MG_E_NOT_BUILT;
    int rc = checkReady(this);
    if (rc) return rc;
    const bool flow = flowEligible(0, nLayers);
    if (execFull && execPrompt && graphsUseFlow == flow) return MG_OK;     // (the launch may have changed hands since the capture)
    invalidateGraphs();
    graphsUseFlow = flow;
    if (flow) { rc = ensureFlow(); if (rc) return rc; }     // allocations and uploads come before the capture
    HIPCHK(hipStreamSynchronize(stream));
    statePosHost = -1;                              // a captured launch is replayed at any position: the variant that covers all
    for (int which = 0; which < 2; which++) {
        HIPCHK(hipStreamBeginCapture(stream, hipStreamCaptureModeRelaxed));
        fuseEmbed = true;
        rc = enqueueToken(which == 0);
        fuseEmbed = false;
        hipGraph_t g = nullptr;
        hipError_t e = hipStreamEndCapture(stream, &g);
        if (rc) { if (g) (void)hipGraphDestroy(g); return rc; }
        HIPCHK(e);
        hipGraphExec_t ex = nullptr;
        HIPCHK(hipGraphInstantiate(&ex, g, nullptr, nullptr, 0));
        if (which == 0) { graphFull = g; execFull = ex; } else { graphPrompt = g; execPrompt = ex; }
    }
    return MG_OK;
}

// ---- graphs over a range of layers (cuda_graph.go:286-388, 554-598, 650-739) ----
// The reference bakes pos into the kernel arguments and re-captures or updates the executable graph per token
// (:673-714); here the position is read from device memory, so one capture serves every position.
int HIPFusedInference::LayerGraphCapture(LayerGraph& lg) {
    if (!built) return MG_E_NOT_BUILT;
    ARGCHK(lg.l0 >= 0 && lg.l1 > lg.l0 && lg.l1 <= nLayers, "CaptureGraph: layer range outside the model");
    for (int l = lg.l0; l < lg.l1; l++) {
        if (!layerComplete(layers[l])) { set_error("CaptureGraph: layer weights incomplete"); return MG_E_STATE; }
        if (!kCache[l]) { set_error("CaptureGraph: KV cache missing, call SetLayerRange first"); return MG_E_STATE; }
    }
    if (execMode == 0) { set_error("CaptureGraph: the per-op launches (exec mode 0) take their position from the host and are not captured"); return MG_E_STATE; }
    LayerGraphDestroy(lg);
    const bool flow = flowEligible(lg.l0, lg.l1);
    if (flow) { int rc = ensureFlow(); if (rc) return rc; }          // allocations and uploads come before the capture
    HIPCHK(hipStreamSynchronize(stream));
    statePosHost = -1;                              // (replayed at any position)
    HIPCHK(hipStreamBeginCapture(stream, hipStreamCaptureModeRelaxed));
    int rc = MG_OK;
    if (flow) rc = enqueueLayersFlow(lg.l0, lg.l1, dState, 0, true);
    else for (int l = lg.l0; l < lg.l1 && rc == MG_OK; l++) rc = enqueueLayer(layers[l], l, dState, 0);
    hipGraph_t g = nullptr;
    hipError_t e = hipStreamEndCapture(stream, &g);
    if (rc) { if (g) (void)hipGraphDestroy(g); return rc; }
    HIPCHK(e);
    hipGraphExec_t ex = nullptr;
    e = hipGraphInstantiate(&ex, g, nullptr, nullptr, 0);
    if (e != hipSuccess) { (void)hipGraphDestroy(g); HIPCHK(e); }
    lg.g = g; lg.ex = ex; lg.hiddenIdx = hiddenIdx; lg.generation = graphGeneration;
    return MG_OK;
}

int HIPFusedInference::LayerGraphLaunch(LayerGraph& lg, int pos) {
    if (!built) return MG_E_NOT_BUILT;
    ARGCHK(pos >= 0 && pos < maxSeq, "graph Launch: pos out of range");
    // a graph captured before a weight, a cache, the mode or the hidden buffer changed points at the old operands
    if (!lg.ex || lg.generation != graphGeneration || lg.hiddenIdx != hiddenIdx) {
        int rc = LayerGraphCapture(lg);
        if (rc) return rc;
    }
    HIPCHK(launch_set_state(dState, pos, 0, 0, 0, ropeRef(), stream));
    statePosHost = -1;
    HIPCHK(hipGraphLaunch(lg.ex, stream));
    return MG_OK;
}

void HIPFusedInference::LayerGraphDestroy(LayerGraph& lg) {
    if (lg.ex) { (void)hipGraphExecDestroy(lg.ex); lg.ex = nullptr; }
    if (lg.g) { (void)hipGraphDestroy(lg.g); lg.g = nullptr; }
}

int HIPFusedInference::UploadHidden(const float* data) {
    if (!built) return MG_E_NOT_BUILT;
    ARGCHK(data, "UploadHidden: NULL data");
    HIPCHK(hipStreamSynchronize(stream));
    HIPCHK(hipMemcpy(hidden[hiddenIdx], data, (size_t)dim * 4, hipMemcpyHostToDevice));
    return MG_OK;
}

// cuda_graph.go:554-598: the eager path and the graph on the same input at position 0, largest difference below 1e-3.
int HIPFusedInference::ValidateGraphCapture(const float* hiddenIn, int layerStart, int layerEnd, float* maxDiff) {
    if (!built) return MG_E_NOT_BUILT;
    ARGCHK(hiddenIn, "ValidateGraphCapture: NULL hiddenIn");
    std::vector<float> ref((size_t)dim), got((size_t)dim);
    int rc = ResetKV();
    if (rc) return rc;
    rc = PartialStep(hiddenIn, 0, layerStart, layerEnd, nullptr, nullptr);
    if (rc == 0) rc = ExportHidden(ref.data());
    if (rc) return rc;
    rc = ResetKV();
    if (rc) return rc;
    LayerGraph lg;
    lg.l0 = layerStart; lg.l1 = layerEnd < nLayers ? layerEnd : nLayers;
    rc = LayerGraphCapture(lg);
    if (rc == 0) rc = UploadHidden(hiddenIn);
    if (rc == 0) rc = LayerGraphLaunch(lg, 0);
    if (rc == 0) rc = ExportHidden(got.data());
    LayerGraphDestroy(lg);
    if (rc) return rc;
    float md = 0.f;
    for (int i = 0; i < dim; i++) {
        const float d = std::fabs(ref[(size_t)i] - got[(size_t)i]);
        if (!(d <= md)) md = d;                 // a NaN difference counts as the largest
    }
    if (maxDiff) *maxDiff = md;
    return MG_OK;
}

int HIPFusedInference::GraphLaunch(int token, int pos, int* nextToken) {
    if (!built) return MG_E_NOT_BUILT;
    ARGCHK(pos >= 0 && pos < maxSeq && token >= 0 && token < vocabSize, "GraphLaunch: token or pos out of range");
    int rc = GraphCapture();
    if (rc) return rc;
    { int rcs = setState(pos, token, 0, 0); if (rcs) return rcs; }
    rc = primeGraph();
    if (rc) return rc;
    statePosHost = -1;
    HIPCHK(hipGraphLaunch(execFull, stream));
    HIPCHK(hipMemcpyAsync(hTokens, dHistory, sizeof(int), hipMemcpyDeviceToHost, stream));
    HIPCHK(hipStreamSynchronize(stream));
    if (nextToken) *nextToken = hTokens[0];
    return checkFlowError();
}

int HIPFusedInference::GraphValidate(int token, int pos, float* maxAbsDiff) {
    if (!built) return MG_E_NOT_BUILT;
    std::vector<float> a(vocabSize), b(vocabSize);
    int t0 = -1, t1 = -1;
    int saved = execMode;
    if (execMode == 0) execMode = 1;         // the per-op launches are not captured: compare the graph with the fused launches
    int rc = DecodeToken(token, pos, &t0, a.data());
    execMode = saved;
    if (rc) return rc;
    rc = GraphLaunch(token, pos, &t1);
    if (rc) return rc;
    HIPCHK(hipMemcpy(b.data(), logits, (size_t)vocabSize * 4, hipMemcpyDeviceToHost));
    float md = 0.f;
    for (int i = 0; i < vocabSize; i++) md = std::fmax(md, std::fabs(a[i] - b[i]));
    if (t0 != t1) md = std::fmax(md, 1.0f);
    if (maxAbsDiff) *maxAbsDiff = md;
    return MG_OK;
}

int HIPFusedInference::Generate(const int* prompt, int nPrompt, int nDecode, int* outTokens, bool useGraph) {
    if (!built) return MG_E_NOT_BUILT;
    ARGCHK(prompt && nPrompt >= 1 && nDecode >= 0 && outTokens, "Generate: bad arguments");
    ARGCHK(nPrompt + nDecode <= maxSeq + 1 && nPrompt <= maxSeq, "Generate: prompt + decode exceeds maxSeq");
    for (int i = 0; i < nPrompt; i++) ARGCHK(prompt[i] >= 0 && prompt[i] < vocabSize, "Generate: prompt token out of range");
    int rc = checkReady(this);
    if (rc) return rc;
    if (execMode == 0) {
        // per-op mode: host-driven loop, one synchronisation per token
        int tok = prompt[0];
        for (int pos = 0; pos < nPrompt - 1 + nDecode; pos++) {
            int next = -1;
            rc = DecodeToken(tok, pos, &next, nullptr);
            if (rc) return rc;
            if (pos + 1 < nPrompt) tok = prompt[pos + 1];
            else { outTokens[pos + 1 - nPrompt] = next; tok = next; }
        }
        return MG_OK;
    }
    // (where runs of tokens go into one launch no graph is needed: the prompt steps are launched one by one)
    const bool graphs = useGraph && !runsInLaunch(useGraph);
    if (graphs) { rc = GraphCapture(); if (rc) return rc; }
    HIPCHK(hipStreamSynchronize(stream));
    HIPCHK(hipMemcpy(dPrompt, prompt, sizeof(int) * (size_t)nPrompt, hipMemcpyHostToDevice));
    { int rcs = setState(0, prompt[0], 0, nPrompt); if (rcs) return rcs; }
    if (graphs) { rc = primeGraph(); if (rc) return rc; }
    for (int i = 0; i < nPrompt - 1; i++) {
        if (graphs) HIPCHK(hipGraphLaunch(execPrompt, stream));
        else { rc = enqueueToken(false); if (rc) return rc; }
    }
    statePosHost = nPrompt - 1;                     // one position a prompt step since setState(0, ..)
    rc = decodeRun(nDecode, useGraph);
    if (rc) return rc;
    if (nDecode > 0) HIPCHK(hipMemcpyAsync(hTokens, dHistory, sizeof(int) * (size_t)nDecode, hipMemcpyDeviceToHost, stream));
    HIPCHK(hipStreamSynchronize(stream));
    for (int i = 0; i < nDecode; i++) outTokens[i] = hTokens[i];
    return checkFlowError();
}

int HIPFusedInference::TimedDecode(int token, int pos, int steps, bool useGraph, float* elapsedMs) {
    if (!built) return MG_E_NOT_BUILT;
    ARGCHK(steps >= 1 && pos >= 0 && pos + steps <= maxSeq && token >= 0 && token < vocabSize, "TimedDecode: bad arguments");
    int rc = checkReady(this);
    if (rc) return rc;
    const bool graphs = useGraph && !runsInLaunch(useGraph);
    if (graphs) { rc = GraphCapture(); if (rc) return rc; }
    if (runsInLaunch(useGraph)) { rc = ensureFlow(); if (rc) return rc; }      // (allocations before the timed region)
    { int rcs = setState(pos, token, 0, 0); if (rcs) return rcs; }
    if (graphs) { rc = primeGraph(); if (rc) return rc; }
    HIPCHK(hipStreamSynchronize(stream));
    HIPCHK(hipEventRecord(ev0, stream));
    rc = decodeRun(steps, useGraph);
    if (rc) return rc;
    HIPCHK(hipEventRecord(ev1, stream));
    HIPCHK(hipEventSynchronize(ev1));
    float ms = 0.f;
    HIPCHK(hipEventElapsedTime(&ms, ev0, ev1));
    if (elapsedMs) *elapsedMs = ms;
    return checkFlowError();
}

// Per-launch-class durations inside a token.  Events cannot be read back from
// graph nodes, so the same launches are issued eagerly with an event between
// every two of them -- behind a gate kernel that holds the stream until the
// host has queued the whole batch, so the GPU never waits for the host.
// classMs[c] = mean milliseconds from the end of the previous launch to the
// end of a launch of class c (0 embed, 1 norm+QKV, 2 attention, 3 Wo,
// 4 gate/up, 5 down, 6 lm_head, 7 argmax finish); classLaunches[c] = launches per token.
int HIPFusedInference::ProfileDecode(int token, int pos, int steps, unsigned classMask, float* classMs, int* classLaunches) {
    if (!built) return MG_E_NOT_BUILT;
    ARGCHK(steps >= 1 && steps <= 64 && pos >= 0 && pos + steps <= maxSeq && token >= 0 && token < vocabSize &&
           classMs && classLaunches, "ProfileDecode: bad arguments (1 <= steps <= 64)");
    int rc = checkReady(this);
    if (rc) return rc;
    HIPCHK(hipStreamSynchronize(stream));
    for (hipEvent_t e : profEvents) (void)hipEventDestroy(e);
    profEvents.clear(); profClass.clear();
    int* gate = hGate;
    *reinterpret_cast<volatile int*>(gate) = 0;
    { int rcs = setState(pos, token, 0, 0); if (rcs) return rcs; }
    HIPCHK(launch_gate(gate, 100LL * 1000 * 500, stream));   // at most 0.5 s
    profiling = true;
    profMask = classMask ? classMask : 0xffu;
    profLast = -1;
    for (int i = 0; i < steps && rc == 0; i++) {
        rc = enqueueToken(true);
        if (rc == 0) rc = mark(8);
    }
    profiling = false;
    *reinterpret_cast<volatile int*>(gate) = 1;
    HIPCHK(hipStreamSynchronize(stream));
    if (rc) return rc;
    double acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    int cnt[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (size_t k = 0; k + 1 < profEvents.size(); k++) {
        int c = profClass[k];
        if (c < 0 || c >= 8) continue;
        float ms = 0.f;
        HIPCHK(hipEventElapsedTime(&ms, profEvents[k], profEvents[k + 1]));
        acc[c] += ms; cnt[c]++;
    }
    for (int c = 0; c < 8; c++) {
        classMs[c] = cnt[c] ? (float)(acc[c] / cnt[c]) : 0.f;
        classLaunches[c] = cnt[c] / steps;
    }
    for (hipEvent_t e : profEvents) (void)hipEventDestroy(e);
    profEvents.clear(); profClass.clear();
    return MG_OK;
}

// ---------------------------------------------------------------------------
// Batched prefill (Q8): the layer of the decode step applied to T rows at
// once, the seven projections as MFMA GEMMs.
// ---------------------------------------------------------------------------
int HIPFusedInference::ensurePrefill(int rows, int kvRows) {
    const int kvPad = (kvRows + 31) / 32 * 32;
    if (kvPad > prefillKVCap) {                 // the attention's hi/lo planes of the cache rows [0, pos0 + T)
        HIPCHK(hipStreamSynchronize(stream));
        prefillKVSlab.release();
        const int want = std::min((maxSeq + 31) / 32 * 32, std::max(kvPad, 2 * prefillKVCap));
        prefillKVCap = 0;
        const size_t bytes = prefill_kv_split_bytes(want, kvDim);
        int rc = prefillKVSlab.init(bytes + 256);
        if (rc) return rc;
        pfKVSplit = prefillKVSlab.take(bytes);
        if (!pfKVSplit) { set_error("prefill KV slab too small"); return MG_E_STATE; }
        prefillKVCap = want;
    }
    if (rows <= prefillCap) return MG_OK;
    HIPCHK(hipStreamSynchronize(stream));
    prefillSlab.release();
    prefillCap = 0;
    const size_t T = ((size_t)rows + 127) / 128 * 128;
    const size_t plane = split_plane_elems((int)T, ffnDim > dim ? ffnDim : dim) * 2;
    size_t bytes = alignUp256(T * 4) + 2 * alignUp256(T * dim * 4) + 2 * alignUp256(T * kvDim * 4) +
                   2 * alignUp256(T * ffnDim * 4) + 4 * alignUp256(plane) + alignUp256(gemm_partial_floats() * 4) + 16 * 256;
    int rc = prefillSlab.init(bytes);
    if (rc) return rc;
    pfTokens = static_cast<int*>(prefillSlab.take(T * 4));
    pfX = static_cast<float*>(prefillSlab.take(T * dim * 4));
    pfQ = static_cast<float*>(prefillSlab.take(T * dim * 4));
    pfK = static_cast<float*>(prefillSlab.take(T * kvDim * 4));
    pfV = static_cast<float*>(prefillSlab.take(T * kvDim * 4));
    pfGate = static_cast<float*>(prefillSlab.take(T * ffnDim * 4));
    pfUp = static_cast<float*>(prefillSlab.take(T * ffnDim * 4));
    pfHi = prefillSlab.take(plane);
    pfLo = prefillSlab.take(plane);
    pfHi2 = prefillSlab.take(plane);      // second pair: written by the gate|up GEMM's own epilogue while it still reads the first
    pfLo2 = prefillSlab.take(plane);
    pfPartial = static_cast<float*>(prefillSlab.take(gemm_partial_floats() * 4));
    if (!pfTokens || !pfX || !pfQ || !pfK || !pfV || !pfGate || !pfUp || !pfHi || !pfLo || !pfHi2 || !pfLo2 || !pfPartial) {
        set_error("prefill slab too small");
        return MG_E_STATE;
    }
    prefillCap = (int)T;
    return MG_OK;
}

int HIPFusedInference::Prefill(const int* tokens, int nTokens, int pos0, int* nextToken, float* logitsOut, float* elapsedMs) {
    if (!built) return MG_E_NOT_BUILT;
    ARGCHK(tokens && nTokens >= 1 && pos0 >= 0 && pos0 + nTokens <= maxSeq, "Prefill: bad token count or position");
    for (int i = 0; i < nTokens; i++) ARGCHK(tokens[i] >= 0 && tokens[i] < vocabSize, "Prefill: token out of range");
    int rc = checkReady(this);
    if (rc) return rc;
    for (const auto& L : layers) {
        // q/k/v and gate/up share a launch: one weight format each
        if (L.wq.kind != L.wk.kind || L.wk.kind != L.wv.kind || L.gate.kind != L.up.kind) {
            set_error("Prefill: q/k/v (and gate/up) of a layer must share one weight format");
            return MG_E_UNSUPPORTED;
        }
    }
    rc = ensurePrefill(nTokens, pos0 + nTokens);
    if (rc) return rc;
    const int T = nTokens;
    HIPCHK(hipStreamSynchronize(stream));
    HIPCHK(hipMemcpy(pfTokens, tokens, sizeof(int) * (size_t)T, hipMemcpyHostToDevice));
    HIPCHK(hipEventRecord(ev0, stream));
    if (embedKind == 1 || embedKind == 2) {
        HIPCHK(launch_embed_rows(embedKind, embedTable, nullptr, pfTokens, pfX, T, dim, vocabSize, stream));
    } else {
        HIPCHK(launch_embed_rows(lmHead.kind == WF_Q8 ? 0 : 3, lmHead.w, lmHead.scales, pfTokens, pfX, T, dim, vocabSize, stream));
    }
    bool normSplitDone = false;
    for (int l = 0; l < nLayers; l++) {
        const LayerWeights& L = layers[l];
        auto seg = [](const DevMat& m, const float* bias, float* y) {
            return GemmSeg{static_cast<const signed char*>(m.w), m.scales, bias, y, m.rows, 0};
        };
        GemmParams g{};
        g.T = T; g.Ahi = static_cast<const unsigned short*>(pfHi); g.Alo = static_cast<const unsigned short*>(pfLo);
        g.partial = pfPartial;
        // (the previous layer's down projection may already have written this split)
        if (!normSplitDone) HIPCHK(launch_split_rows(pfX, L.norm1, eps, T, dim, pfHi, pfLo, stream));
        g.K = dim; g.nseg = 3; g.q4 = L.wq.kind == WF_Q4P;
        g.seg[0] = seg(L.wq, L.bq, pfQ); g.seg[1] = seg(L.wk, L.bk, pfK); g.seg[2] = seg(L.wv, L.bv, pfV);
        // where K is split, the kernel that sums the splits also rotates q/k and stores the K/V rows
        g.ropeKc = kCache[l]; g.ropeVc = vCache[l]; g.ropeCos = cosTab; g.ropeSin = sinTab;
        g.ropePos0 = pos0; g.ropeHeadDim = headDim; g.ropeKvHalf = kvHalf;
        HIPCHK(launch_gemm_q8(g, 0, stream));
        if (!g.wroteRope)
            HIPCHK(launch_rope_store_rows(pfQ, pfK, pfV, kCache[l], vCache[l], kvHalf, cosTab, sinTab, pos0, T, dim, kvDim, headDim, stream));
        g.ropeKc = nullptr; g.ropeVc = nullptr;
        // the attention writes its rows as the hi/lo split the output projection reads
        HIPCHK(launch_prefill_attention(pfQ, kCache[l], vCache[l], kvHalf, pfKVSplit, nullptr, pfHi, pfLo, T, pos0, maxSeq, dim, kvDim, nHeads,
                                        nKVHeads, headDim, stream));
        g.K = dim; g.nseg = 1; g.q4 = L.wo.kind == WF_Q4P; g.seg[0] = seg(L.wo, nullptr, pfX);
        // where K is split, the kernel that sums the splits also writes norm2's split of the new rows
        g.nextGain = L.norm2; g.nextEps = eps;
        g.nextHi = static_cast<unsigned short*>(pfHi); g.nextLo = static_cast<unsigned short*>(pfLo);
        HIPCHK(launch_gemm_q8(g, 1, stream));
        if (!g.wroteNext) HIPCHK(launch_split_rows(pfX, L.norm2, eps, T, dim, pfHi, pfLo, stream));
        g.nextGain = nullptr; g.nextHi = nullptr; g.nextLo = nullptr;
        g.K = dim; g.nseg = 2; g.q4 = L.gate.kind == WF_Q4P; g.seg[0] = seg(L.gate, nullptr, pfGate); g.seg[1] = seg(L.up, nullptr, pfUp);
        // silu(gate) * up and its hi/lo split come out of the GEMM's epilogue or of the kernel that sums its K splits
        // (into the second pair of planes: the GEMM is still reading the first)
        g.nextSwiglu = 1; g.nextHi = static_cast<unsigned short*>(pfHi2); g.nextLo = static_cast<unsigned short*>(pfLo2);
        HIPCHK(launch_gemm_q8(g, 0, stream));
        if (!g.wroteNext) HIPCHK(launch_swiglu_split(pfGate, pfUp, T, ffnDim, pfHi2, pfLo2, stream));
        g.nextSwiglu = 0; g.nextHi = nullptr; g.nextLo = nullptr;
        g.Ahi = static_cast<const unsigned short*>(pfHi2); g.Alo = static_cast<const unsigned short*>(pfLo2);
        g.K = ffnDim; g.nseg = 1; g.q4 = L.down.kind == WF_Q4P; g.seg[0] = seg(L.down, nullptr, pfX);
        if (l + 1 < nLayers) {                  // ... and here the next layer's norm1 split
            g.nextGain = layers[l + 1].norm1; g.nextEps = eps;
            g.nextHi = static_cast<unsigned short*>(pfHi); g.nextLo = static_cast<unsigned short*>(pfLo);
        }
        HIPCHK(launch_gemm_q8(g, 1, stream));
        normSplitDone = g.wroteNext != 0;
        g.Ahi = static_cast<const unsigned short*>(pfHi); g.Alo = static_cast<const unsigned short*>(pfLo);
    }
    // the last position continues on the decode path: final norm, lm_head, greedy token, state -> pos0 + T
    HIPCHK(hipMemcpyAsync(hidden[hiddenIdx], pfX + (size_t)(T - 1) * dim, (size_t)dim * 4, hipMemcpyDeviceToDevice, stream));
    { int rcs = setState(pos0 + T - 1, tokens[T - 1], 0, 0); if (rcs) return rcs; }
    rc = enqueueFinal(true);
    if (rc) return rc;
    statePosHost = pos0 + T;                        // where the argmax's last kernel leaves the state
    HIPCHK(hipEventRecord(ev1, stream));
    HIPCHK(hipMemcpyAsync(hTokens, dHistory, sizeof(int), hipMemcpyDeviceToHost, stream));
    HIPCHK(hipStreamSynchronize(stream));
    if (nextToken) *nextToken = hTokens[0];
    if (logitsOut) HIPCHK(hipMemcpy(logitsOut, logits, (size_t)vocabSize * 4, hipMemcpyDeviceToHost));
    if (elapsedMs) HIPCHK(hipEventElapsedTime(elapsedMs, ev0, ev1));
    return MG_OK;
}

// Prompt through the GEMM path, then nDecode - 1 graph replays from the device state it left.
int HIPFusedInference::GeneratePrefill(const int* prompt, int nPrompt, int nDecode, int* outTokens) {
    if (!built) return MG_E_NOT_BUILT;
    ARGCHK(prompt && nPrompt >= 1 && nDecode >= 1 && outTokens, "GeneratePrefill: bad arguments");
    ARGCHK(nPrompt + nDecode <= maxSeq + 1, "GeneratePrefill: prompt + decode exceeds maxSeq");
    const bool graphs = !runsInLaunch(true);
    int rc = graphs ? GraphCapture() : MG_OK;
    if (rc) return rc;
    rc = Prefill(prompt, nPrompt, 0, nullptr, nullptr, nullptr);
    if (rc) return rc;
    if (nDecode > 1 && graphs) { rc = primeGraph(); if (rc) return rc; }
    rc = decodeRun(nDecode - 1, true);
    if (rc) return rc;
    HIPCHK(hipMemcpyAsync(hTokens, dHistory, sizeof(int) * (size_t)nDecode, hipMemcpyDeviceToHost, stream));
    HIPCHK(hipStreamSynchronize(stream));
    for (int i = 0; i < nDecode; i++) outTokens[i] = hTokens[i];
    return checkFlowError();
}

}  // namespace mg

// ---------------------------------------------------------------------------
// C entry points
// ---------------------------------------------------------------------------
using mg::HIPFusedInference;

extern "C" {

const char* mg_last_error(void) { return mg::get_error().c_str(); }

mg_ctx* mg_create(int dim, int kvDim, int headDim, int nHeads, int nKVHeads, int ffnDim, int vocabSize, int nLayers,
                  int maxSeq, double ropeTheta, float eps) {
    mg::set_error("");
    HIPFusedInference* f = HIPFusedInference::New(dim, kvDim, headDim, nHeads, nKVHeads, ffnDim, vocabSize, nLayers,
                                                  maxSeq, ropeTheta, eps);
    if (!f) return nullptr;
    return new mg_ctx{f};
}
struct mg_layer_graph { mg_ctx* c; mg::HIPFusedInference::LayerGraph lg; };
void mg_destroy(mg_ctx* c) {
    if (!c) return;
    for (mg_layer_graph* g : c->layerGraphs) { if (c->f) c->f->LayerGraphDestroy(g->lg); g->c = nullptr; }
    delete c->f;
    delete c;
}

#define CTX(c) if (!(c) || !(c)->f) { mg::set_error("NULL context"); return MG_E_NOT_BUILT; } HIPFusedInference* f = (c)->f

int mg_num_weights(const mg_ctx* c) { return c && c->f ? c->f->NumWeights() : 0; }
int mg_set_weight(mg_ctx* c, int idx, const float* data, size_t n) { CTX(c); return f->SetWeight(idx, data, n); }
int mg_set_weight_q8(mg_ctx* c, int idx, const int8_t* q, const float* scales) { CTX(c); return f->SetWeightQ8(idx, q, scales); }
int mg_set_weight_q4_0(mg_ctx* c, int idx, const uint8_t* d, size_t n) { CTX(c); return f->SetWeightQ4_0(idx, d, n); }
int mg_set_quant_rounding(mg_ctx* c, int mode) {
    CTX(c);
    if (mode != 0 && mode != 1) { mg::set_error("rounding mode must be 0 or 1"); return MG_E_ARG; }
    f->quantRounding = mode;
    return MG_OK;
}
int mg_set_embedding_f16(mg_ctx* c, const uint16_t* t) { CTX(c); return f->SetEmbeddingF16(t); }
int mg_set_embedding_f32(mg_ctx* c, const float* t) { CTX(c); return f->SetEmbeddingF32(t); }
int mg_set_layer_range(mg_ctx* c, int a, int b) { CTX(c); return f->SetLayerRange(a, b); }
int mg_reset_kv(mg_ctx* c) { CTX(c); return f->ResetKV(); }
int mg_set_kv_format(mg_ctx* c, int fmt) { CTX(c); return f->SetKVFormat(fmt); }
int mg_partial_step(mg_ctx* c, const float* hiddenIn, int pos, int l0, int l1, float* hiddenOut, float* logitsOut) {
    CTX(c); return f->PartialStep(hiddenIn, pos, l0, l1, hiddenOut, logitsOut);
}
int mg_step_layer_resident(mg_ctx* c, int layer, int pos, const float* hiddenIn, float* preOut, float* postOut, float* logitsOut) {
    CTX(c); return f->StepLayerResident(layer, pos, hiddenIn, preOut, postOut, logitsOut);
}
int mg_export_hidden(mg_ctx* c, float* out) { CTX(c); return f->ExportHidden(out); }
int mg_queue_hidden_to_l3(mg_ctx* c) { CTX(c); return f->QueueHiddenToL3(); }
int mg_wait_l3(mg_ctx* c) { CTX(c); return f->WaitL3(); }
const float* mg_get_l3_hidden(mg_ctx* c) { return c && c->f ? c->f->GetL3Hidden() : nullptr; }
int mg_signal_mailbox(mg_ctx* c) { CTX(c); return f->SignalMailbox(); }
int mg_wait_mailbox(mg_ctx* c, int timeoutMs) { CTX(c); return f->WaitMailbox(timeoutMs); }
int mg_swap_hidden_buffer(mg_ctx* c) { CTX(c); return f->SwapHiddenBuffer(); }
int mg_hidden_idx(mg_ctx* c) { CTX(c); return f->hiddenIdx; }
int mg_set_exec_mode(mg_ctx* c, int mode) {
    CTX(c);
    if (mode < 0 || mode > 4) { mg::set_error("exec mode must be 0, 1, 2, 3 or 4"); return MG_E_ARG; }
    f->SetExecMode(mode);
    return MG_OK;
}
int mg_set_q4_act_quant(mg_ctx* c, int on) { CTX(c); return f->SetQ4ActQuant(on); }
int mg_decode_token(mg_ctx* c, int token, int pos, int* next, float* logitsOut) { CTX(c); return f->DecodeToken(token, pos, next, logitsOut); }
int mg_generate(mg_ctx* c, const int* prompt, int nPrompt, int nDecode, int* out, int useGraph) {
    CTX(c); return f->Generate(prompt, nPrompt, nDecode, out, useGraph != 0);
}
int mg_graph_capture(mg_ctx* c) { CTX(c); return f->GraphCapture(); }
int mg_graph_launch(mg_ctx* c, int token, int pos, int* next) { CTX(c); return f->GraphLaunch(token, pos, next); }
int mg_graph_validate(mg_ctx* c, int token, int pos, float* md) { CTX(c); return f->GraphValidate(token, pos, md); }
mg_layer_graph* mg_layer_graph_capture(mg_ctx* c, int layerStart, int layerEnd, int streamCount, int pipelineBreak, int pos) {
    if (!c || !c->f) { mg::set_error("NULL context"); return nullptr; }
    if (streamCount == 0) streamCount = 1;                                   // cuda_graph.go:316
    if (streamCount != 1 && streamCount != 2) { mg::set_error("CaptureGraph: unsupported StreamCount (use 1 or 2)"); return nullptr; }
    if (streamCount == 2 && (pipelineBreak <= layerStart || pipelineBreak >= layerEnd)) {   // :396-400
        mg::set_error("CaptureGraph: PipelineBreak must lie between LayerStart and LayerEnd");
        return nullptr;
    }
    if (pos < 0 || pos >= c->f->maxSeq) { mg::set_error("CaptureGraph: pos out of range"); return nullptr; }
    mg_layer_graph* g = new mg_layer_graph{c, {}};
    g->lg.l0 = layerStart; g->lg.l1 = layerEnd;
    if (c->f->LayerGraphCapture(g->lg) != MG_OK) { delete g; return nullptr; }
    c->layerGraphs.push_back(g);
    return g;
}
static bool live(mg_layer_graph* g) {
    if (!g) { mg::set_error("NULL graph"); return false; }
    if (!g->c) { mg::set_error("graph: its context was destroyed"); return false; }
    return true;
}
int mg_layer_graph_launch(mg_layer_graph* g, int pos) {
    if (!live(g)) return MG_E_STATE;
    return g->c->f->LayerGraphLaunch(g->lg, pos);
}
int mg_layer_graph_update_and_launch(mg_layer_graph* g, int pos) {
    if (!live(g)) return 0;
    return g->c->f->LayerGraphLaunch(g->lg, pos) == MG_OK ? 1 : 0;
}
void mg_layer_graph_destroy(mg_layer_graph* g) {
    if (!g) return;
    if (g->c) {
        g->c->f->LayerGraphDestroy(g->lg);
        auto& v = g->c->layerGraphs;
        for (size_t i = 0; i < v.size(); i++) if (v[i] == g) { v.erase(v.begin() + (long)i); break; }
    }
    delete g;
}
int mg_upload_hidden(mg_ctx* c, const float* data) { CTX(c); return f->UploadHidden(data); }
int mg_read_hidden(mg_ctx* c, float* out) { CTX(c); return f->ExportHidden(out); }
int mg_validate_graph_capture(mg_ctx* c, const float* hiddenIn, int layerStart, int layerEnd, float* maxDiff) {
    CTX(c);
    float md = 0.f;
    int rc = f->ValidateGraphCapture(hiddenIn, layerStart, layerEnd, &md);
    if (maxDiff) *maxDiff = md;
    if (rc) return rc;
    return md < 0.001f ? 1 : 0;
}
int mg_has_graph_kernel(void) { return 1; }
int mg_timed_decode(mg_ctx* c, int token, int pos, int steps, int useGraph, float* ms) {
    CTX(c); return f->TimedDecode(token, pos, steps, useGraph != 0, ms);
}
int mg_profile_decode(mg_ctx* c, int token, int pos, int steps, unsigned classMask, float* classMs, int* classLaunches) {
    CTX(c); return f->ProfileDecode(token, pos, steps, classMask, classMs, classLaunches);
}
int mg_prefill(mg_ctx* c, const int* tokens, int nTokens, int pos0, int* next, float* logitsOut, float* ms) {
    CTX(c); return f->Prefill(tokens, nTokens, pos0, next, logitsOut, ms);
}
int mg_generate_prefill(mg_ctx* c, const int* prompt, int nPrompt, int nDecode, int* out) {
    CTX(c); return f->GeneratePrefill(prompt, nPrompt, nDecode, out);
}
// Inspection of the persistent layer launch's exchange area after a step (for tests): copies layer `layer`'s
// block into out (cap floats) and writes its geometry {stride, offQ, offKc, offVc, offPacc, offPm, offPl,
// offX1, offM, offX2, smax} into geo[11].  MG_E_STATE when that launch has not been set up.
int mg_flow_exchange(mg_ctx* c, int layer, float* out, size_t cap, int* geo) {
    CTX(c);
    if (!f->flowXchg || layer < 0 || layer >= f->nLayers) { mg::set_error("mg_flow_exchange: no exchange area (or bad layer)"); return MG_E_STATE; }
    const mg::FlowGeometry& g = f->flowGeo;
    if (geo) {
        const int v[11] = {g.stride, g.offQ, g.offKc, g.offVc, g.offPacc, g.offPm, g.offPl, g.offX1, g.offM, g.offX2, g.smax};
        for (int i = 0; i < 11; i++) geo[i] = v[i];
    }
    if (out) {
        if (hipStreamSynchronize(f->stream) != hipSuccess) return MG_E_HIP;
        const size_t n = cap < (size_t)g.stride ? cap : (size_t)g.stride;
        if (hipMemcpy(out, f->flowXchg + (size_t)layer * g.stride, n * 4, hipMemcpyDeviceToHost) != hipSuccess) return MG_E_HIP;
    }
    return MG_OK;
}
int mg_flow_in_use(mg_ctx* c) {
    if (!c || !c->f) return 0;
    return c->f->FlowInUse() ? 1 : 0;
}
int mg_flow_tail_in_use(mg_ctx* c) {
    if (!c || !c->f) return 0;
    return c->f->FlowTailInUse() ? 1 : 0;
}
int mg_set_flow_tail(mg_ctx* c, int on) { CTX(c); f->SetFlowTail(on); return MG_OK; }
int mg_set_flow_generic(mg_ctx* c, int on) { CTX(c); f->SetFlowGeneric(on); return MG_OK; }
int mg_set_tokens_per_launch(mg_ctx* c, int n) { CTX(c); return f->SetTokensPerLaunch(n); }
int mg_tokens_per_launch(mg_ctx* c) { return c && c->f ? c->f->tokensPerLaunch : 0; }
int mg_flow_tail_trace(mg_ctx* c, long long* out, size_t cap, int* dims) { CTX(c); return f->FlowTailTrace(out, cap, dims); }
int mg_flow_set_wait_limit(mg_ctx* c, long long ticks) {
    CTX(c);
    f->SetFlowWaitLimit(ticks);
    return MG_OK;
}
int mg_flow_trace(mg_ctx* c, int enable, long long* out, size_t cap, int* dims) {
    CTX(c);
    return f->FlowTrace(enable, out, cap, dims);
}
uint64_t mg_weight_bytes_per_token(const mg_ctx* c) { return c && c->f ? c->f->WeightBytesPerToken() : 0; }
uint64_t mg_kv_bytes_at(const mg_ctx* c, int pos) { return c && c->f ? c->f->KVBytesAt(pos) : 0; }

}  // extern "C"
