// flow.h -- the layers of a decode step as ONE persistent launch (flow.hip).
//
// A small model's token is ~120 dependent phases of a few microseconds each; as separate launches every
// phase pays a kernel boundary and starts with cold registers.  Here one workgroup per CU stays resident
// for all layers of the token and the phases hand their vectors over through a small exchange area in
// device memory: a producer stores its floats write-through, a consumer polls the vector it needs until
// no element is the "not written yet" pattern.  No barrier across the grid and no atomics: a phase costs
// one store-to-load hand-over, and a wave requests its next weights before it starts to wait.
#pragma once
#include "kernels.h"

namespace mg {

// Per-layer operands, a table in device memory.  Q8 weights: int8 rows + per-row float scales.  Q4_0 weights (all
// seven matrices of every layer, split layout): the matrix pointer is the nibble plane [N, K/2] and the scale pointer
// holds the address of the fp16 d plane [N, K/32] that follows it.
struct FlowLayer {
    const float* g1;
    const float* g2;
    const signed char* wq; const signed char* wk; const signed char* wv; const signed char* wo;
    const signed char* gate; const signed char* up; const signed char* down;
    const float* sq; const float* sk; const float* sv; const float* so;
    const float* sgate; const float* sup; const float* sdown;
    const float* bq; const float* bk; const float* bv;      // optional (NULL)
    float* Kc; float* Vc;                                    // caches [maxSeq, kvDim]: fp32, or fp16 (FlowParams::kvHalf)
};

// Operands of the tail of a token (final norm, lm_head, greedy argmax, the next token's embedding), a struct in device
// memory.  The lm_head has the format of the layers' matrices (pointer pair as in FlowLayer).
struct FlowTail {
    const float* finalGain;
    const signed char* lmW; const float* lmAux;
    float* logits;               // [vocab], every token's logits (the last token's remain)
    const void* embTable;        // embKind 0: the lm_head's int8 rows (embScales = its row scales), 1: fp16 table,
    const float* embScales;      //         2: fp32 table, 3: the lm_head's Q4_0 planes
    const float* cosTab; const float* sinTab;    // [maxSeq, headDim/2]
    StepState* state;            // read at the start (pos, token, count, nPrompt), written at the end of the launch
    int* history;                // greedy tokens go to history[count ..]
    const int* prompt;           // while pos + 1 < nPrompt the next token is prompt[pos + 1] (optional)
    float* amax;                 // argmax exchange: [2][grid] slots of FLOW_AMAX_STRIDE floats (value, index, rest unused),
                                 // part of the exchange allocation
    float* ropeCur;              // cos then sin row of the position after the launch (optional)
    int embKind, vocab, historyCap;
};

// Exchange area: per layer one block of `stride` floats holding, at the offsets below, the rotated query,
// the K and V rows of the current position, the attention partials of up to smax KV splits (accumulator,
// maximum, sum), the hidden state after the attention block, the SwiGLU vector and the layer's output.
// Every float is the pattern 0xFFFFFFFF until its producer has written it.
constexpr int FLOW_GQA_MAX = 8;        // query heads a KV head may have for the grouped attention
constexpr int FLOW_TILE = 128;         // positions of an attention tile: one workgroup per (query head, tile)
struct FlowGeometry {
    int stride;
    int offQ, offKc, offVc, offPacc, offPm, offPl, offX1, offM, offX2, offAttn;
    int smax;
    int gqa;         // 1: an attention workgroup per (KV head, split) taking all its query heads; 0: per (query head, split)
};
FlowGeometry flow_geometry(int dim, int kvDim, int ffn, int nHeads, int nKVHeads, int headDim, int maxSeq, int grid);
bool flow_context_fits(int maxSeq, const FlowGeometry& g);

constexpr size_t FLOW_ERR_BYTES = 4096;
constexpr int FLOW_AMAX_STRIDE = 32;   // floats between two workgroups' argmax slots: a 128-byte line each

// Trace slots of a layer, in program order: when thread 0 of a workgroup passed the point.
constexpr int FLOW_TRACE_SLOTS = 11;
#define FLOW_TRACE_NAMES "layer-top", "qkv-input-staged", "qkv-done", "q-k-v-rows-in", "attention-done", "attention-merged", \
                         "wo-done", "gate-up-input-staged", "gate-up-done", "down-input-staged", "down-done"

struct FlowParams {
    const FlowLayer* layers;     // indexed by layer
    int l0, l1;                  // layers [l0, l1)
    int nLayersTotal;            // layers the table and the exchange area hold
    int dim, kvDim, ffn, nHeads, nKVHeads, headDim, maxSeq;
    int q4;                      // 0: Q8 matrices, 1: Q4_0 matrices in the split layout
    int idleWoRows, idleGateUpRows;   // leading rows of Wo / of gate and up that workgroups idle during the attention read into the L2s
    int downSplit;               // the down projection's rows are shared by two waves each (few rows, long ones)
    int kvHalf;                  // the caches hold fp16 rows (rounded where written, widened where read)
    int nCompute;                // workgroups 0 .. nCompute-1 compute (geo is laid out for them), the rest of the grid prefetches
    float eps;
    const StepState* state;      // position source (NULL -> posImm)
    int posImm;
    const float* cosRow;         // cos / sin row of the position [headDim/2]
    const float* sinRow;
    float* hidden;               // input of layer l0 and output of layer l1-1 [dim]
    float* xchg;                 // exchange area, geo.stride floats per layer (indexed by layer)
    FlowGeometry geo;
    int* err;                    // FLOW_ERR_BYTES of zeros: word 0 is set to 1 when a wait ran into its time limit; bytes
                                 // 256 .. 2304 are the idle lines (never written; polls with nothing to ask for go there)
    long long limitTicks;        // per wait, in ticks of the 100 MHz wall clock
    long long* trace;            // optional (diagnostic): wall-clock ticks [layer][FLOW_TRACE_SLOTS][workgroup], see FLOW_TRACE_NAMES;
                                 // in token mode one more "layer" for the tail: FLOW_TAIL_TRACE_NAMES
    int nTokens;                 // 0: layers [l0, l1) of one step, hidden in and out; n >= 1: token mode -- n whole tokens from the
                                 // device state on (all layers; xchg holds two halves and the argmax exchange; state != NULL)
    const FlowTail* tail;        // token mode
    int gqaCode;                 // geo.gqa only: 1 = a position of this launch may need the grouped attention (the variant that can do
                                 // it is launched); 0 = none does (positions below nCompute / nHeads tiles): the plain variant, which
                                 // is faster there, runs on the same geometry and reports a position past its reach as error 3
    int generic;                 // 1: never a variant with a known shape's sizes compiled in (comparisons, tests)
};
#define FLOW_TAIL_TRACE_NAMES "tail-top", "final-input-staged", "lm-head-done", "token-known", "all-waves-done", "partials-in"

// Of `cus` workgroups that can be resident at once, how many the launch sets aside to prefetch weights into the L2s
// (0 where that does not pay: layers too large for the L2s, or a phase that would need another round of the waves).
int flow_prefetch_workgroups(int cus, size_t layerBytes, int dim, int kvDim, int ffn);
// Computing workgroups the launch needs at least (one per query head and KV split) for this shape.
int flow_min_grid(int nHeads, int nKVHeads, const FlowGeometry& g);
bool flow_shape_supported(int dim, int kvDim, int ffn, int nHeads, int nKVHeads, int headDim);
// With nCompute computing workgroups: no phase needs more rounds of the waves than the kernel holds results for, and
// the grouped attention has a workgroup per query head for its merge.
bool flow_grid_fits(int ffn, int nHeads, const FlowGeometry& g, int nCompute);
// grid workgroups of 512 threads, all of which must be resident at once (grid <= CUs x resident workgroups per CU);
// grid - p.nCompute of them prefetch (0, or a multiple of 8 with nCompute a multiple of 8 as well).
hipError_t launch_flow_layers(const FlowParams& p, int grid, hipStream_t s);
// Fills the blocks of layers [l0, l1) (of the first half) with the "not written yet" pattern.
hipError_t launch_flow_reset(float* xchg, const FlowGeometry& g, int l0, int l1, hipStream_t s);
// Floats of the whole exchange allocation: two halves of nLayers blocks (token mode alternates between them; launches
// over a range of layers use the first) and the argmax exchange [2][grid] pairs behind them.
size_t flow_xchg_floats(const FlowGeometry& g, int nLayers, int grid);
inline float* flow_amax_area(float* xchg, const FlowGeometry& g, int nLayers) { return xchg + (size_t)2 * nLayers * g.stride; }
// ... all of it (before the first token-mode launch after the position was set by the host).
hipError_t launch_flow_reset_all(float* xchg, const FlowGeometry& g, int nLayers, int grid, hipStream_t s);
// LDS a workgroup of the launch takes (an upper bound: dynamic part plus the variant's own arrays); token mode keeps
// the token's embedding beside the staged vector.  Must stay within the CU's 160 KB.
size_t flow_lds_bytes(int dim, int ffn, int headDim, int gqa, bool tokenMode);

}  // namespace mg
