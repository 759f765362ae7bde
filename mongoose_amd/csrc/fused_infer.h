// fused_infer.h -- HIPFusedInference: the MI355X counterpart of the Go type
// CUDAFusedInference (cuda_fused_infer.go:56-142).  It owns the quantized
// weights, the fp32 KV caches, the scratch vectors and the RoPE tables, and
// runs the batch-1 decode step.  Method names follow the Go methods they
// stand in for; the mg_* C functions are thin wrappers over them.
#pragma once
#include "kernels.h"
#include "flow.h"

#include <cstdint>
#include <string>
#include <vector>

namespace mg {

struct DevMat {
    int kind = -1;          // -1 none, WF_Q8, WF_Q4P
    void* w = nullptr;      // Q8: int8 [rows, cols]; Q4P: nibble plane + fp16 d plane
    float* scales = nullptr;
    int rows = 0, cols = 0;
    size_t bytes = 0;       // bytes a token reads from this matrix (weights + scales)
};

inline size_t alignUp256(size_t v) { return (v + 255) & ~(size_t)255; }

// One device allocation handed out in 256-byte aligned pieces.
struct Slab {
    char* base = nullptr;
    size_t size = 0, used = 0;
    int init(size_t bytes);
    void* take(size_t bytes);
    void release();
};

struct LayerWeights {
    float* norm1 = nullptr;
    float* norm2 = nullptr;
    float* bq = nullptr;
    float* bk = nullptr;
    float* bv = nullptr;
    DevMat wq, wk, wv, wo, gate, up, down;
};

void set_error(const std::string& s);
const std::string& get_error();

class HIPFusedInference {
public:
    // NewCUDAFusedInference, cuda_fused_infer.go:144-229
    static HIPFusedInference* New(int dim, int kvDim, int headDim, int nHeads, int nKVHeads, int ffnDim,
                                  int vocabSize, int nLayers, int maxSeq, double ropeTheta, float eps);
    ~HIPFusedInference();

    int NumWeights() const { return nLayers * 12 + 2; }                           // :231
    int SetWeight(int idx, const float* data, size_t n);                          // :241
    int SetWeightQ8(int idx, const int8_t* q, const float* scales);
    int SetWeightQ4_0(int idx, const uint8_t* q4Data, size_t nbytes);             // cuda_fused_infer_q4.go:46
    int SetEmbeddingF16(const uint16_t* table);
    int SetEmbeddingF32(const float* table);
    int SetLayerRange(int layerStart, int layerEnd);                              // :542
    int ResetKV();                                                                // :530
    int PartialStep(const float* hiddenIn, int pos, int layerStart, int layerEnd,
                    float* hiddenOut, float* logitsOut);                          // :392, :456, q4:92, q4:272
    int StepLayerResident(int layer, int pos, const float* hiddenIn, float* preOut,
                          float* postOut, float* logitsOut);                      // cuda_fused_infer_q4.go:451
    int ExportHidden(float* out);                                                 // :235
    int DecodeToken(int token, int pos, int* nextToken, float* logitsOut);
    int Generate(const int* prompt, int nPrompt, int nDecode, int* outTokens, bool useGraph);
    int GraphCapture();                                                           // cuda_graph.go:315
    int GraphLaunch(int token, int pos, int* nextToken);                          // cuda_graph.go:663
    int GraphValidate(int token, int pos, float* maxAbsDiff);                     // cuda_graph.go:554
    int TimedDecode(int token, int pos, int steps, bool useGraph, float* elapsedMs);
    int ProfileDecode(int token, int pos, int steps, unsigned classMask, float* classMs, int* classLaunches);
    // Batched prefill of nTokens positions starting at pos0 (Q8 weights): fills the KV caches,
    // leaves the last position's hidden state, logits and greedy token, and the device step
    // state ready for the decode that follows.
    int Prefill(const int* tokens, int nTokens, int pos0, int* nextToken, float* logitsOut, float* elapsedMs);
    int GeneratePrefill(const int* prompt, int nPrompt, int nDecode, int* outTokens);
    uint64_t WeightBytesPerToken() const;
    uint64_t KVBytesAt(int pos) const { return (uint64_t)2 * nLayers * (uint64_t)(pos + 1) * kvDim * (kvHalf ? 2 : 4); }
    // L3 bridge (cuda_fused_infer.go:118-131, :556-737): a pinned host buffer, [0:4] mailbox counter,
    // [64:] hidden state, for handing a pipeline stage's output to the host without a device sync.
    int QueueHiddenToL3();                    // :688  copy stream waits for compute, then D2H into the bridge
    int WaitL3();                             // :709  waits for the copy stream only
    const float* GetL3Hidden() const;         // :725  host view of the bridge's hidden state
    int SignalMailbox();                      // :558  kernel behind the stage's last launch bumps the counter
    int WaitMailbox(int timeoutMs);           // :575  host polls the counter
    int SwapHiddenBuffer();                   // :737
    bool HasL3() const { return l3 != nullptr; }
    int SetKVFormat(int fmt);                 // 0: fp32 rows (the reference's layout), 1: fp16 rows
    int kvHalf = 0;

    int quantRounding = 0;
    // 0: one launch per reference op; 1: fused launches; 2: fused, attention launches without the L2 prefetch
    // helpers; 3: all layers of a step in one persistent launch where the model allows it (else as 1).
    int execMode = 3;
    int SetQ4ActQuant(int on);
    void SetExecMode(int mode) {
        if (mode != execMode) invalidateGraphs();
        if ((mode == 3 || mode == 4) && mode != execMode) flowRegeometry();    // the two differ in the launch's geometry
        if (mode == 3 || mode == 4) flowBroken = false;      // asked for again by name: a wait that ran out earlier no longer bars it
        execMode = mode;
        if (mode != 0) q4ActQuant = false;      // only the op-by-op loop has the integer matvecs
        if (mode != 3 && mode != 4) releaseFlow();
    }
    void flowRegeometry();
    void releaseFlow();

    // shape
    int dim, kvDim, headDim, nHeads, nKVHeads, ffnDim, vocabSize, nLayers, maxSeq;
    double ropeTheta;
    float eps;

    // used by the streaming front end
    // Objects that keep a pointer to this context (stream front ends) register where they keep it; the
    // destructor clears those pointers, so that destroying the context first leaves them inert.
    std::vector<HIPFusedInference**> backrefs;
    hipStream_t stream = nullptr;
    std::vector<LayerWeights> layers;
    std::vector<float*> kCache, vCache;
    float* hidden[2] = {nullptr, nullptr};
    int hiddenIdx = 0;
    int enqueueLayer(const LayerWeights& L, int layer, const StepState* st, int posImm);
    int enqueueFinal(bool withArgmax);
    float* logits = nullptr;
    float* finalNorm = nullptr;
    DevMat lmHead;

private:
    HIPFusedInference() = default;
    bool built = false;
    int invalidateGraphs();
    int uploadMat(int idx, DevMat& m, int rows, int cols, const int8_t* q, const float* scales);
    int uploadMatQ4(int idx, DevMat& m, int rows, int cols, const uint8_t* raw, size_t nbytes);
    int setVec(int idx, float*& dst, const float* data, size_t n, size_t expect);
    int slotAddr(int idx, char** out);
    Slab scratch, headSlab, prefillSlab, prefillKVSlab;
    int prefillCap = 0;             // rows the prefill buffers hold
    int prefillKVCap = 0;           // cache rows the attention's split planes hold
    void* pfKVSplit = nullptr;
    int* pfTokens = nullptr;
    float *pfX = nullptr, *pfQ = nullptr, *pfK = nullptr, *pfV = nullptr, *pfGate = nullptr, *pfUp = nullptr;
    void *pfHi = nullptr, *pfLo = nullptr, *pfHi2 = nullptr, *pfLo2 = nullptr;
    float* pfPartial = nullptr;
    int ensurePrefill(int rows, int kvRows);
    std::vector<Slab> layerSlabs, kvSlabs;
    size_t slotOff[12] = {0};
    size_t layerSlabBytes = 0;
    DevMat* matSlot(int idx, int* rows, int* cols);
    int enqueueLayerFused(const LayerWeights& L, int layer, const StepState* st, int posImm);
    MvParams qkvParams(const LayerWeights& L, int layer, const StepState* st, int posImm) const;
    MvParams woParams(const LayerWeights& L) const;
    MvParams gateUpParams(const LayerWeights& L) const;
    MvParams downParams(const LayerWeights& L) const;
    void planPrefetch(const LayerWeights& L, const LayerWeights* next, int layer, PfJob& job) const;
    EmbedRef embedRef() const;
    int primeGraph();
    bool fuseEmbed = false;      // set while the graphs are captured
    int enqueueLayerPerOp(const LayerWeights& L, int layer, int pos);
    int enqueueEmbed();
    // persistent layer launch (flow.hip)
public:
    FlowGeometry flowGeo{};
    float* flowXchg = nullptr;
    long long* flowTrace = nullptr;
    int FlowTrace(int enable, long long* out, size_t cap, int* dims);
    // Graphs over a range of layers (cuda_graph.go:315-388, 663-714): hidden state in, hidden state out.
    struct LayerGraph {
        int l0 = 0, l1 = 0, hiddenIdx = 0;
        unsigned generation = 0;
        hipGraph_t g = nullptr;
        hipGraphExec_t ex = nullptr;
    };
    int LayerGraphCapture(LayerGraph& lg);                 // (re)captures lg.l0 .. lg.l1 on the context's stream
    int LayerGraphLaunch(LayerGraph& lg, int pos);         // sets the device position, replays; asynchronous
    void LayerGraphDestroy(LayerGraph& lg);
    int UploadHidden(const float* data);                   // cuda_graph.go:650
    int ValidateGraphCapture(const float* hiddenIn, int layerStart, int layerEnd, float* maxDiff);   // :554-598
    bool FlowInUse() const { return flowEligible(0, nLayers); }
    long long flowLimitTicks = 5000000;       // per wait of the persistent launch: 50 ms of the 100 MHz wall clock
    void SetFlowWaitLimit(long long ticks) { invalidateGraphs(); flowLimitTicks = ticks; }
    int statePosHost = -1;                    // the device state's position where the host knows it (set with the state, advanced
                                              // with whole tokens run in the persistent launch), else -1
    // Whole tokens inside the persistent launch (embedding, layers, final norm, lm_head, argmax): on where the model
    // allows it; tokensPerLaunch of them in one launch where a caller asks for a run of tokens (Generate, TimedDecode,
    // GeneratePrefill), 1 = a launch (or a graph replay) per token.
    bool flowTail = true;
    int tokensPerLaunch = 64;
    void SetFlowTail(int on) { invalidateGraphs(); flowTail = on != 0; }
    bool flowGeneric = false;    // never the persistent launch's variants with a known shape's sizes compiled in
    void SetFlowGeneric(int on) { invalidateGraphs(); flowGeneric = on != 0; }
    int SetTokensPerLaunch(int n);
    bool FlowTailInUse() const { return flowTailEligible(); }
    int FlowTailTrace(long long* out, size_t cap, int* dims);
private:
    FlowLayer* dFlowLayers = nullptr;
    int* dFlowErr = nullptr;
    int* hFlowErr = nullptr;        // pinned
    int flowGrid = 0;         // workgroups of the persistent launch (one per CU)
    int flowCompute = 0;      // ... of which compute (the others prefetch weights)
    bool flowTableDirty = true;
    bool flowBroken = false;        // a wait ran into its limit once: the separate launches are used from then on
    bool flowEligible(int l0, int l1) const;
    bool flowTailEligible() const;
    FlowTail* dFlowTail = nullptr;
    int enqueueTokensFlow(int nTokens);
    int decodeRun(int nTokens, bool useGraph);      // nTokens decode steps from the device state
    bool runsInLaunch(bool useGraph) const;         // ... as runs of tokens inside the persistent launch
    int setState(int pos, int token, int count, int nPrompt);
    int flowComputeWgs(int cus) const;
    bool q4ActQuant = false;      // exec mode 0: Q4_0 matrices through the int8-activation matvecs
    void* q8Scratch = nullptr;    // (max(dim, ffnDim)/32)*40 bytes of activation blocks (cuda_fused_infer.go:175-179)
    int ensureFlow();
    int enqueueLayersFlow(int l0, int l1, const StepState* st, int posImm, bool resetFirst, int nTokens = 0);
    int checkFlowError();
    int enqueueToken(bool withHead);      // embed -> layers -> final(+argmax) / advance, all from device state

    // scratch (cuda_fused_infer.go:56-69, :626)
    float *normed = nullptr, *Q = nullptr, *K = nullptr, *V = nullptr, *attnOut = nullptr, *proj = nullptr;
    float *normed2 = nullptr, *gatePre = nullptr, *upOut = nullptr, *ffnMid = nullptr;
    float *cosTab = nullptr, *sinTab = nullptr;
    // split-KV attention partials
    float *pm = nullptr, *pl = nullptr, *pacc = nullptr;
    int smax = 1, splitLen = 256, attnHeadsPerWG = 0;
    int* attnCounters = nullptr;
    float* ropeCur = nullptr;        // cos then sin row of the device-resident position
    RopeCur ropeRef() const;
    // embedding table (optional)
    int embedKind = -1;       // -1: tied lm_head
    void* embedTable = nullptr;
    // token-level state
    StepState* dState = nullptr;
    StepState* hState = nullptr;    // pinned mirror
    int* hGate = nullptr;           // pinned flag the timing gate kernel polls
    float* amaxVal = nullptr;
    int* amaxIdx = nullptr;
    int amaxParts = 0;
    int* dHistory = nullptr;
    int* dPrompt = nullptr;
    int* hTokens = nullptr;         // pinned
    bool graphsUseFlow = false;       // the whole-token graphs were captured with the persistent layer launch
    unsigned graphGeneration = 0;     // bumped by whatever makes captured graphs stale (weights, caches, modes)
    hipGraph_t graphFull = nullptr, graphPrompt = nullptr;
    hipGraphExec_t execFull = nullptr, execPrompt = nullptr;
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    // L3 bridge
    char* l3 = nullptr;               // pinned: [0:4] mailbox counter, [64:64+dim*4] hidden
    hipStream_t copyStream = nullptr;
    hipEvent_t computeDone = nullptr;
    unsigned mailboxSignaled = 0, mailboxExpected = 1;
    // instrumented run: an event between every two launches of a token
    std::vector<hipEvent_t> profEvents;
    std::vector<int> profClass;       // class of the launch that follows event i
    bool profiling = false;
    unsigned profMask = 0xffu;
    int profLast = -1;
    int mark(int cls);
};

}  // namespace mg

// the opaque handle of the C ABI
struct mg_layer_graph;
struct mg_ctx {
    mg::HIPFusedInference* f;
    std::vector<mg_layer_graph*> layerGraphs;      // live graph objects: they outlive the context as dead handles
};
