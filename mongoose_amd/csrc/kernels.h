// kernels.h -- launcher prototypes shared by the C ABI (abi.hip) and the
// fused-inference context (fused_infer.hip).  Device code lives in kernels.hip.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mg {

// Weight formats the matvec kernel reads.
enum WeightFormat {
    WF_Q8 = 0,      // int8 [N,K] + per-row float scale
    WF_Q4P = 1,     // Q4_0 split layout: nibbles [N,K/2] then fp16 d [N,K/32]
    WF_Q4RAW = 2,   // raw GGUF block_q4_0, 18-byte blocks
};

// How the activation vector reaches LDS.
enum Prologue {
    PRO_PLAIN = 0,  // act[K] copied
    PRO_RMS = 1,    // act = rmsnorm(x, gain, eps)
};

// What happens to each finished row.
enum Epilogue {
    EPI_STORE = 0,   // out[r] = v (+ bias[r])
    EPI_RESID = 1,   // out[r] = resid[r] + v
    EPI_SWIGLU = 2,  // seg0 = gate, seg1 = up: out[r] = silu(g) * u
    EPI_ARGMAX = 3,  // out[r] = v and a per-workgroup running (max, index)
    EPI_QKV = 4,     // seg0 = q, seg1 = k, seg2 = v: bias, RoPE on q/k, k/v stored into the caches at pos
};

// Device-resident step state, so that a captured graph needs no new arguments
// per token (what tw_graph_params was meant for, cuda_graph.go:181-205).
struct StepState {
    int pos;        // position of the token being processed
    int token;      // its id
    int count;      // tokens emitted so far into the history buffer
    int nPrompt;    // prompt length (tokens < nPrompt come from the prompt buffer)
};

struct MvSeg {
    const void* w;        // weights (format WF)
    const void* aux;      // Q8: float scales[rows]; Q4P: unused (d follows the nibbles); Q4RAW: unused
    const float* bias;    // optional
    float* out;
    int rows;
};

struct MvParams {
    MvSeg seg[3];
    int nseg;
    int K;
    int ngroups;          // row groups over all segments
    int segGroup0[3];     // first group of each segment
    // prologue
    const float* act;     // PRO_PLAIN: activation; PRO_RMS: x
    const float* gain;
    float eps;
    // EPI_QKV: cos/sin row of the current position [headDim/2] (no dependence on the
    // position load); seg1.out / seg2.out are the K / V caches [maxSeq, kvDim], row `pos` is written
    const StepState* state;  // position source (may be NULL -> posImm)
    int posImm;
    const float* cosRow;
    const float* sinRow;
    int headDim, kvDim;
    int kvHalf;           // EPI_QKV: the caches hold fp16 (seg1/seg2.out point at them all the same)
    // epilogue
    const float* resid;
    int div127;           // Q8: multiply by scales[r]/127 instead of scales[r]
    float* amaxVal;       // EPI_ARGMAX partials [gridDim.x]
    int* amaxIdx;
    // EPI_ARGMAX, optional: xresetWords 32-bit words at xreset (a multiple of 4, 16-byte aligned) are filled
    // with 0xFFFFFFFF by the launch's workgroups -- the exchange area of the persistent layer launch, which
    // must read "nothing written yet" before the next token
    unsigned* xreset;
    unsigned xresetWords;
};

struct MvConfig { int nr; int ks; int grid; };

MvConfig pick_config(int wf, int epi, int totalRows, int K);
// Launch the matvec; returns hipSuccess or the launch error.  cfgInOut may be
// NULL or have nr == 0 (pick automatically); the configuration used, with the
// grid size, is written back.
hipError_t launch_matvec(int wf, int epi, int pro, MvParams& p, MvConfig* cfgInOut, hipStream_t s);

// What later launches of the step will read, for workgroups that have nothing else to do: the decode
// attention of a small model keeps a handful of CUs busy, the rest of its launch pulls the next
// matrices into L2.  Workgroup i of a launch runs on XCD i & 7 and every XCD has an L2 of its own, so
// weights are described in runs: run r of a region (bytes [r * runBytes, (r + 1) * runBytes)) will be
// read by a workgroup on XCD (xoff + r) & 7 and is fetched by a helper on that XCD.  A region with
// xoff < 0 (scales, gains, biases) is read by every workgroup and fetched on every XCD.
struct PfRegion { const char* base; unsigned bytes; unsigned runBytes; int xoff; int nruns; int splitLog2; };   // 2^splitLog2 waves share a run (set by the launcher)
constexpr int PF_MAX_REGIONS = 28;
struct PfJob {
    PfRegion region[PF_MAX_REGIONS];
    int nregion;
    int helperWaves;      // waves to spread the job over (0: no helpers); the launcher turns it into
    int rows;             // rows of helper workgroups appended to the attention grid,
    int wgsPerXcd;        // helper workgroups that take part on each XCD, and
    int waveStart[PF_MAX_REGIONS + 1];   // region r is fetched by waves waveStart[r] .. waveStart[r+1]-1 of an XCD's helper waves
};
// Appends what launch_matvec(wf, epi, ..., p) will read and returns its weight bytes; 0 (job unchanged)
// when that launch does not keep rows on fixed XCDs (rounds of workgroups that are not a multiple of 8,
// formats without a fast kernel) or the job is full.  limitBytes > 0 and below the launch's bytes: only
// the first rows of each matrix, as many as fit (not for the q|k|v launch).
size_t plan_matvec_prefetch(int wf, int epi, int pro, const MvParams& p, PfJob& job, size_t limitBytes = 0);

struct AttnParams {
    const float* q;       // [dim], rotated
    const float* Kc;      // [rowLimit, kvDim], row pos already written
    const float* Vc;
    const StepState* state;   // position source (NULL -> posImm)
    int posImm;
    int rowLimit;         // rows that may be touched (maxSeq, or cacheLen for the per-op call)
    int kvDim, nHeads, nKVHeads, headDim;
    int splitLen;         // positions per split, fixed for the context (multiple of 256); 0 = one split
    int smax;             // number of splits launched
    float* pm; float* pl; float* pacc;   // partials [nHeads, smax(, headDim)] when smax > 1
    int* counters;        // one per workgroup column, zero between launches (smax > 1)
    int headsPerWG;       // query heads of a GQA group per workgroup (0 = the whole group, in chunks of up to 4)
    float* out;           // [dim]
    int kvHalf;           // Kc / Vc hold fp16 instead of fp32 (same [row, kvDim] indexing)
    PfJob pf;             // pf.rows > 0: grid rows smax .. smax + pf.rows - 1 are prefetch helpers
};
hipError_t launch_attention(const AttnParams& p, hipStream_t s);
int attention_columns(int nHeads, int nKVHeads, int headsPerWG);

hipError_t launch_rmsnorm_out(const float* in, float* out, const float* w, int seqLen, int dim, float eps, hipStream_t s);
hipError_t launch_fused_add_rmsnorm(const float* a, const float* b, float* out, const float* w, int seqLen, int dim, float eps, hipStream_t s);
hipError_t launch_q4_rowscale_matvec(const float* act, const void* w, const float* scales, float* out, int N, int K, hipStream_t s);
hipError_t launch_rope(float* x, const float* cosTab, const float* sinTab, int seqLen, int dim, int headDim, int nHeads, hipStream_t s);
hipError_t launch_kv_cache_write(float* cache, const float* src, int pos, int kvDim, hipStream_t s);
hipError_t launch_kv_cache_write_f16(void* cache, const float* src, int pos, int kvDim, hipStream_t s);
hipError_t launch_silu_gate_mul(const float* gate, const float* up, float* out, int n, hipStream_t s);
hipError_t launch_add_inplace(float* a, const float* b, int n, hipStream_t s);
hipError_t launch_embed_gather_f32(float* out, const float* embed, const int* tokens, int seqLen, int dim, hipStream_t s);
hipError_t launch_dequant_q8(const void* w, const float* scales, float* out, int rows, int cols, int div127, hipStream_t s);
hipError_t launch_dequant_q4_0(const void* w, float* out, int rows, int cols, hipStream_t s);
hipError_t launch_q4_0_repack(const void* raw, void* planar, int N, int K, hipStream_t s);
hipError_t launch_matvec_generic_q8(const float* act, const void* w, const float* scales, float* out, int N, int K, int div127, hipStream_t s);
hipError_t launch_fill_zero(void* ptr, size_t bytes, hipStream_t s);

// q4_dp4a.hip: int8 activation blocks (40 bytes per 32 activations: float d, float d*sum(q), int8 q[32]) and the
// Q4_0 matvec on the packed int8 dot instruction.  batch vectors / results are contiguous.
hipError_t launch_q8_quantize_act(const float* act, void* q8out, int K, int batch, hipStream_t s);
hipError_t launch_q4_0_dp4a(const void* w, bool planar, const void* q8, float* out, int N, int K, int batch, hipStream_t s);
hipError_t launch_argmax_slices(const float* x, int n, int nparts, float* pv, int* pi, hipStream_t s);

// Embedding row of state->token into x[dim]: kind 0 = Q8 row * scale (tied
// lm_head), 1 = fp16 table, 2 = fp32 table, 3 = Q4_0 split-layout row.
hipError_t launch_embed_token(int kind, const void* table, const float* scales, const StepState* state,
                              float* x, int dim, int vocab, hipStream_t s);
// Reduce the lm_head partials to a token, append it to the history and
// advance the step state (next token comes from the prompt while pos+1 < nPrompt).
// Every kernel that sets the position also copies that position's cos/sin row
// into rope.cur (cos then sin, headDim/2 each), so that the next token's
// kernels read it without first waiting for the position.
struct RopeCur { const float* cosTab; const float* sinTab; float* cur; int half; int maxSeq; };
// Where the token-advancing kernels also leave the embedding row of the token they have just chosen
// (out == NULL: they do not).  kind as in launch_embed_token.
struct EmbedRef { int kind; const void* table; const float* scales; float* out; int dim; int vocab; };
hipError_t launch_argmax_finish(const float* pv, const int* pi, int nparts, StepState* state,
                                const int* prompt, int* history, int historyCap, int vocab, RopeCur rope, EmbedRef emb, hipStream_t s);
hipError_t launch_set_state(StepState* state, int pos, int token, int count, int nPrompt, RopeCur rope, hipStream_t s);
// Advance state without an lm_head (prompt positions): pos++, token = prompt[pos].
hipError_t launch_advance_prompt(StepState* state, const int* prompt, RopeCur rope, EmbedRef emb, hipStream_t s);

// Pipeline-stage mailbox (SignalMailbox, cuda_fused_infer.go:558): stores `value` into a counter in
// host-visible memory once everything queued before it on the stream has finished.
hipError_t launch_signal_mailbox(unsigned* counter, unsigned value, hipStream_t s);

// Stream gate for timing runs: waits for *flag != 0 (host-pinned) or limitTicks of the 100 MHz wall clock.
hipError_t launch_gate(const int* flag, long long limitTicks, hipStream_t s);

}  // namespace mg
