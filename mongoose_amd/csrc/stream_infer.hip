// stream_infer.hip -- HIPStreamInfer: decode with layer weights streamed from
// host memory, for models larger than device memory.  Counterpart of
// CUDAStreamInfer (cuda_fused_stream.go:98-726): two device weight sets, two
// pinned staging buffers, and a three-way overlap per layer of
//   host copy (layer i+2 -> pinned)  ||  DMA (layer i+1 -> device)  ||  compute (layer i).
// The layer arithmetic is the resident path's (stepLayer :277-356 = the
// 17-op body plus the three bias adds at :319-321).
//
// Differences by design: one DMA per layer instead of twelve (the staging
// buffer already has the device layout), and the Q4_0 rows are regrouped into
// the split nibble/scale layout while they are being copied into the pinned
// buffer, so the fast matvec kernel reads them with aligned 16-byte loads at
// no extra pass over the data.
#include "fused_infer.h"
#include "../../include/mongoose_hip.h"
#include "host_util.h"

#include <algorithm>
#include <cstring>
#include <vector>

namespace mg {

#define SHIPCHK(expr)                                                                     \
    do {                                                                                  \
        hipError_t e_ = (expr);                                                           \
        if (e_ != hipSuccess) {                                                           \
            set_error(std::string(#expr) + ": " + hipGetErrorString(e_));                 \
            (void)hipGetLastError();                                                      \
            return MG_E_HIP;                                                              \
        }                                                                                 \
    } while (0)

static size_t alignUp(size_t v) { return (v + 255) & ~(size_t)255; }

class HIPStreamInfer {
public:
    HIPFusedInference* f = nullptr;
    // byte offsets of the 12 tensors inside a layer blob, slot order
    // norm1,wq,wk,wv,bq,bk,bv,wo,norm2,gate,up,down (cuda_fused_stream.go:216-242)
    size_t off[12];
    size_t nbytes[12];
    size_t layerSize = 0;
    char* dev[2] = {nullptr, nullptr};
    char* pinned[2] = {nullptr, nullptr};
    hipStream_t uploadStream = nullptr;
    hipEvent_t uploadDone[2] = {nullptr, nullptr};
    hipEvent_t computeDone[2] = {nullptr, nullptr};
    LayerWeights view[2];

    ~HIPStreamInfer() {
        if (f) {                                   // still alive: no longer tell it about this object
            auto& br = f->backrefs;
            br.erase(std::remove(br.begin(), br.end(), &f), br.end());
        }
        if (f && f->stream) (void)hipStreamSynchronize(f->stream);
        if (uploadStream) { (void)hipStreamSynchronize(uploadStream); (void)hipStreamDestroy(uploadStream); }
        for (int i = 0; i < 2; i++) {
            if (dev[i]) (void)hipFree(dev[i]);
            if (pinned[i]) (void)hipHostFree(pinned[i]);
            if (uploadDone[i]) (void)hipEventDestroy(uploadDone[i]);
            if (computeDone[i]) (void)hipEventDestroy(computeDone[i]);
        }
    }

    int matShape(int k, int* rows, int* cols) const {
        switch (k) {
        case 1: *rows = f->dim; *cols = f->dim; return 1;
        case 2: case 3: *rows = f->kvDim; *cols = f->dim; return 1;
        case 7: *rows = f->dim; *cols = f->dim; return 1;
        case 9: case 10: *rows = f->ffnDim; *cols = f->dim; return 1;
        case 11: *rows = f->dim; *cols = f->ffnDim; return 1;
        }
        return 0;
    }

    int build() {
        size_t o = 0;
        for (int k = 0; k < 12; k++) {
            int r, c;
            if (matShape(k, &r, &c)) nbytes[k] = (size_t)r * (c / 32) * 18;
            else if (k == 5 || k == 6) nbytes[k] = (size_t)f->kvDim * 4;
            else nbytes[k] = (size_t)f->dim * 4;
            off[k] = o;
            o += alignUp(nbytes[k]);
        }
        layerSize = o;
        SHIPCHK(hipStreamCreateWithFlags(&uploadStream, hipStreamNonBlocking));
        for (int i = 0; i < 2; i++) {
            void* p = nullptr;
            SHIPCHK(hipMalloc(&p, layerSize));
            dev[i] = static_cast<char*>(p);
            SHIPCHK(hipHostMalloc(&p, layerSize, hipHostMallocDefault));     // cuda_fused_stream.go:170-180
            pinned[i] = static_cast<char*>(p);
            std::memset(pinned[i], 0, layerSize);
            SHIPCHK(hipEventCreateWithFlags(&uploadDone[i], hipEventDisableTiming));
            SHIPCHK(hipEventCreateWithFlags(&computeDone[i], hipEventDisableTiming));
            LayerWeights& L = view[i];
            char* b = dev[i];
            L.norm1 = reinterpret_cast<float*>(b + off[0]);
            L.bq = reinterpret_cast<float*>(b + off[4]);
            L.bk = reinterpret_cast<float*>(b + off[5]);
            L.bv = reinterpret_cast<float*>(b + off[6]);
            L.norm2 = reinterpret_cast<float*>(b + off[8]);
            DevMat* ms[12] = {nullptr, &L.wq, &L.wk, &L.wv, nullptr, nullptr, nullptr, &L.wo, nullptr, &L.gate, &L.up, &L.down};
            for (int k = 0; k < 12; k++) {
                int r, c;
                if (!ms[k] || !matShape(k, &r, &c)) continue;
                ms[k]->kind = WF_Q4P; ms[k]->w = b + off[k]; ms[k]->scales = nullptr;
                ms[k]->rows = r; ms[k]->cols = c; ms[k]->bytes = nbytes[k];
            }
        }
        return MG_OK;
    }

    // stageLayerToPinned, cuda_fused_stream.go:200-247 (NULL bias -> zeros).  The seven matrices are cut
    // into pieces of 8192 blocks and regrouped by all worker threads in one parallel region.
    int stage(int set, const void* const* ptrs, const int32_t* sizes) {
        static const int matIdx[7] = {1, 2, 3, 7, 9, 10, 11};        // order of layerSizes[i*7+m] (:571-598)
        constexpr size_t PIECE = 8192;
        char* dst = pinned[set];
        struct Job { const uint8_t* src; uint8_t* out; size_t nb, b0, b1; };
        std::vector<Job> jobs;
        for (int m = 0; m < 7; m++) {
            int k = matIdx[m];
            if (!ptrs[k]) { set_error("StreamForwardToken: NULL matrix pointer"); return MG_E_ARG; }
            if ((size_t)sizes[m] != nbytes[k]) { set_error("StreamForwardToken: layerSizes entry is not rows*(cols/32)*18"); return MG_E_ARG; }
            int r, c;
            matShape(k, &r, &c);
            const size_t nb = (size_t)r * (c / 32);
            for (size_t b0 = 0; b0 < nb; b0 += PIECE)
                jobs.push_back(Job{static_cast<const uint8_t*>(ptrs[k]), reinterpret_cast<uint8_t*>(dst + off[k]), nb, b0,
                                   std::min(nb, b0 + PIECE)});
        }
        parallel_jobs(jobs.size(), [&](size_t j) {
            const Job& jb = jobs[j];
            repack_q4_0_blocks(jb.src, jb.nb, jb.b0, jb.b1, jb.out);
        });
        for (int k : {0, 8}) {
            if (!ptrs[k]) { set_error("StreamForwardToken: NULL norm pointer"); return MG_E_ARG; }
            std::memcpy(dst + off[k], ptrs[k], nbytes[k]);
        }
        for (int k : {4, 5, 6}) {
            if (ptrs[k]) std::memcpy(dst + off[k], ptrs[k], nbytes[k]);
            else std::memset(dst + off[k], 0, nbytes[k]);
        }
        return MG_OK;
    }

    // StreamForwardToken, cuda_fused_stream.go:559-670
    int forward(int pos, const float* embHidden, int nLayers, const void* const* layerPtrs, const int32_t* layerSizes,
                float* logitsOut) {
        if (!f) { set_error("StreamForwardToken: the context this object was built on has been destroyed"); return MG_E_STATE; }
        if (!embHidden || !layerPtrs || !layerSizes) { set_error("StreamForwardToken: NULL argument"); return MG_E_ARG; }
        if (nLayers < 1 || nLayers > f->nLayers || pos < 0 || pos >= f->maxSeq) { set_error("StreamForwardToken: bad nLayers or pos"); return MG_E_ARG; }
        for (int l = 0; l < nLayers; l++)
            if (!f->kCache[l]) { set_error("StreamForwardToken: KV cache missing, call SetLayerRange"); return MG_E_STATE; }
        hipStream_t cs = f->stream;
        SHIPCHK(hipStreamSynchronize(cs));
        SHIPCHK(hipStreamSynchronize(uploadStream));
        SHIPCHK(hipMemcpy(f->hidden[f->hiddenIdx], embHidden, (size_t)f->dim * 4, hipMemcpyHostToDevice));

        int rc = stage(0, layerPtrs, layerSizes);
        if (rc) return rc;
        SHIPCHK(hipMemcpyAsync(dev[0], pinned[0], layerSize, hipMemcpyHostToDevice, uploadStream));
        SHIPCHK(hipEventRecord(uploadDone[0], uploadStream));
        if (nLayers > 1) {
            rc = stage(1, layerPtrs + 12, layerSizes + 7);
            if (rc) return rc;
        }
        for (int i = 0; i < nLayers; i++) {
            const int set = i & 1, other = set ^ 1;
            if (i + 1 < nLayers) {
                // device set `other` was last read by layer i-1
                if (i >= 1) SHIPCHK(hipStreamWaitEvent(uploadStream, computeDone[other], 0));
                SHIPCHK(hipMemcpyAsync(dev[other], pinned[other], layerSize, hipMemcpyHostToDevice, uploadStream));
                SHIPCHK(hipEventRecord(uploadDone[other], uploadStream));
            }
            SHIPCHK(hipStreamWaitEvent(cs, uploadDone[set], 0));
            rc = f->enqueueLayer(view[set], i, nullptr, pos);
            if (rc) return rc;
            SHIPCHK(hipEventRecord(computeDone[set], cs));
            if (i + 2 < nLayers) {
                // pinned[set] is free once its DMA (layer i) has finished
                SHIPCHK(hipEventSynchronize(uploadDone[set]));
                rc = stage(set, layerPtrs + (size_t)(i + 2) * 12, layerSizes + (size_t)(i + 2) * 7);
                if (rc) return rc;
            }
        }
        if (logitsOut) {                                                   // stepFinal :469-484
            rc = f->enqueueFinal(false);
            if (rc) return rc;
            SHIPCHK(hipStreamSynchronize(cs));
            SHIPCHK(hipMemcpy(logitsOut, f->logits, (size_t)f->vocabSize * 4, hipMemcpyDeviceToHost));
        }
        SHIPCHK(hipStreamSynchronize(cs));
        SHIPCHK(hipStreamSynchronize(uploadStream));
        return MG_OK;
    }
};

}  // namespace mg

struct mg_stream { mg::HIPStreamInfer* s; };

extern "C" {

mg_stream* mg_stream_build(mg_ctx* ctx) {
    if (!ctx || !ctx->f) { mg::set_error("mg_stream_build: NULL context"); return nullptr; }
    if (ctx->f->dim % 32 || ctx->f->ffnDim % 32) { mg::set_error("mg_stream_build: Q4_0 needs dims % 32 == 0"); return nullptr; }
    auto* s = new mg::HIPStreamInfer();
    s->f = ctx->f;
    ctx->f->backrefs.push_back(&s->f);
    if (s->build() != MG_OK) { delete s; return nullptr; }
    return new mg_stream{s};
}

void mg_stream_destroy(mg_stream* s) {
    if (s) { delete s->s; delete s; }
}

int mg_stream_forward_token(mg_stream* s, int pos, const float* embHidden, int nLayers, const void* const* layerPtrs,
                            const int32_t* layerSizes, float* logitsOut) {
    if (!s || !s->s) { mg::set_error("mg_stream_forward_token: NULL stream object"); return MG_E_NOT_BUILT; }
    return s->s->forward(pos, embHidden, nLayers, layerPtrs, layerSizes, logitsOut);
}

}  // extern "C"
