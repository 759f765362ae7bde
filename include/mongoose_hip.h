/*
 * mongoose_hip.h -- C ABI of libmongoose_hip.so, the MI355X (gfx950) backend
 * for mongoose's batch-1 fused quantized decode path.
 *
 * Plain C: pointers, sizes and ints only.  A "device pointer" is memory
 * obtained from tw_gpu_alloc (or any hipMalloc); `stream` is a hipStream_t
 * passed as void* (NULL = the default stream), exactly where the reference
 * passes a cudaStream_t.  Reference paths are relative to the mongoose
 * checkout.
 *
 * Three groups, mirroring what the reference's cgo blocks bind:
 *   1. tw_gpu_*        device memory shim            (cuda_tensor.go:19-52)
 *   2. mongoose_*      one launch per decode op      (kernels.go:12-72, 150-226;
 *                                                     bodies kernels/mongoose.cu)
 *   3. mg_*            fused-inference context: what CUDAFusedInference,
 *                      CUDAStreamInfer and CUDAGraph do behind their Go methods
 *                      (cuda_fused_infer.go, cuda_fused_infer_q4.go,
 *                       cuda_q4_0.go, cuda_fused_stream.go, cuda_graph.go)
 *
 * Error convention.  The reference's kernels return void and report nothing;
 * its Go methods return -1 when the object is not built.  Here mongoose_*
 * keep the void signatures (so a dlsym table binds them unchanged) and record
 * failures for mongoose_check(); mg_* return 0 on success and a negative
 * MG_E_* code otherwise, with text in mg_last_error().
 */
#ifndef MONGOOSE_HIP_H
#define MONGOOSE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MG_OK            0
#define MG_E_NOT_BUILT  (-1)   /* same value the Go methods return when !built */
#define MG_E_ARG        (-2)
#define MG_E_HIP        (-3)
#define MG_E_STATE      (-4)
#define MG_E_UNSUPPORTED (-5)

/* ------------------------------------------------------------------ */
/* 1. Device memory shim                      cuda_tensor.go:19-52      */
/* ------------------------------------------------------------------ */
void* tw_gpu_alloc(size_t bytes);                               /* :19-28  NULL on failure (message on stderr) */
void  tw_gpu_free(void* ptr);                                   /* :30-32 */
void  tw_gpu_upload(void* dst, const void* src, size_t bytes);  /* :34-36  synchronous H2D */
void  tw_gpu_download(void* dst, const void* src, size_t bytes);/* :38-40  synchronous D2H */
void  tw_gpu_zero(void* ptr, size_t bytes);                     /* :42-44 */
void* tw_gpu_alloc_pinned(size_t bytes);                        /* :47-52  page-locked host memory */
void  tw_gpu_free_pinned(void* ptr);
/* cuda.go:30-56 tw_cuda_init_device: select device, 0 on success. */
int   tw_hip_init_device(int device);
/* cuda.go:58-75: device name / total memory. */
int   tw_hip_device_info(char* name, size_t nameLen, uint64_t* totalMem);

/* ------------------------------------------------------------------ */
/* 2. Per-op kernels                           kernels.go:12-72         */
/*    Same symbol names and argument order as libmongoose_kernels.so.   */
/* ------------------------------------------------------------------ */

/* kernels.go:13, mongoose.cu:145-179.  out = in * rsqrt(mean(in^2)+1e-6) * w, per row of [seqLen, dim]. */
void mongoose_rmsnorm_out(const float* in, float* out, const float* w, int seqLen, int dim, void* stream);
/* Same with eps as an argument (cpu.go:36 and the Metal path take it as a
 * parameter; the CUDA kernel hard-codes 1e-6). */
void mongoose_rmsnorm_out_eps(const float* in, float* out, const float* w, int seqLen, int dim, float eps, void* stream);

/* kernels.go:12, mongoose.cu:16-50.  In place: x = x * rsqrt(mean(x^2)+1e-6) * w, per row of [seqLen, dim]
 * (what TRMSNorm binds, kernel_tensor.go:23-26). */
void mongoose_rmsnorm(float* x, const float* w, int seqLen, int dim, void* stream);
/* kernels.go:20, mongoose.cu:372-404.  out = rmsnorm(a + b, w), eps 1e-6; out may be a or b.
 * The _eps form takes eps as an argument (as mongoose_rmsnorm_out_eps does). */
void mongoose_fused_add_rmsnorm(const float* a, const float* b, float* out, const float* w, int seqLen, int dim, void* stream);
void mongoose_fused_add_rmsnorm_eps(const float* a, const float* b, float* out, const float* w, int seqLen, int dim, float eps, void* stream);

/* kernels.go:62, mongoose.cu:1556-1595.  out[r] = sum_k act[k]*w[r,k] * (scales[r]/127):
 * the reference kernel's convention, `scales` holding per-row absmax
 * (producer: mongoose_requant_fp32_to_int8, mongoose.cu:1501-1545). */
void mongoose_q8_matvec(const float* act, const void* w_int8, const float* scales, float* out, int N, int K, void* stream);
/* Per-row-scale form: out[r] = sum_k act[k]*w[r,k] * scales[r], with
 * scales[r] = absmax/127 as quantizeQ8 stores them (cuda_fused_infer.go:373-374,
 * metal_impl_darwin.m:5533-5535).  This is what the mg_* context uses. */
void mongoose_q8_matvec_rowscale(const float* act, const void* w_int8, const float* scales, float* out, int N, int K, void* stream);

/* kernels.go:63, mongoose.cu:1598-1640.  Per-row-scale 4-bit weights (what TQ8Matvec binds for
 * Q8Weight.Q4, kernel_tensor.go:34-40; not GGUF Q4_0): w_packed is [N, K/2] bytes, low nibble =
 * element 2k, high nibble = element 2k+1, value (nib-8) * scales[r]/7.  K even. */
void mongoose_q4_matvec(const float* act, const void* w_packed, const float* scales, float* out, int N, int K, void* stream);

/* kernels.go:65.  w is raw GGUF block_q4_0 (18-byte blocks: fp16 d, 16 bytes of
 * nibbles; low nibble = element j, high nibble = element j+16; value (nib-8)*d),
 * rows of K/32 blocks (cuda_q4_0.go:13-17).  fp32 activations, fp32 accumulate. */
void mongoose_q4_0_matvec(const float* act, const void* w_q4_0, float* out, int N, int K, void* stream);
/* Device-side repack of raw GGUF rows into the split layout the fast kernel
 * reads: N*K/2 bytes of nibbles (16 per block, rows contiguous) followed by
 * N*K/32 fp16 scales.  `planar` needs N*K/2 + N*K/16 bytes. */
void mongoose_q4_0_repack(const void* w_q4_0, void* planar, int N, int K, void* stream);
void mongoose_q4_0_matvec_planar(const float* act, const void* planar, float* out, int N, int K, void* stream);

/* The integer ("dp4a") forms of the Q4_0 matvec: kernels.go:66-70 (typedefs, same argument order), wrappers
 * kernels.go:985-1017, dispatch cuda_fused_infer_q4.go:611-673.  The reference's CUDA bodies of these five are not
 * in its tree; its Go side fixes the calling sequence and the scratch size, (K/32)*40 bytes
 * (cuda_fused_infer.go:176), "Q8_1 blocks" (kernels.go:993).  Here a block of 32 activations is
 *     { float d = max|x|/127;  float s = d * sum(q);  int8 q[32] = round-half-away(x/d) }      (40 bytes)
 * and a row of block_q4_0 weights against it is GGML's vec_dot_q4_0_q8_1,
 *     out[r] = sum_b f32(d4) * (d8 * sum_i nib_i * q_i - 8 * s8),
 * on the packed int8 dot instruction.  Results differ from mongoose_q4_0_matvec by the activation rounding only
 * (about 1e-2 relative on N(0,1) activations).  q8 buffers: 8-byte aligned, (K/32)*40 bytes a vector; batch forms
 * take B contiguous vectors and write out[B, N]. */
void mongoose_q8_quantize_act(const float* act, void* q8_out, int K, void* stream);
void mongoose_q8_quantize_act_batch(const float* acts, void* q8_out, int K, int B, void* stream);
void mongoose_q4_0_matvec_dp4a(const float* act, const void* w_q4_0, float* out, int N, int K, void* q8_scratch, void* stream);
void mongoose_q4_0_matvec_dp4a_preq(const void* w_q4_0, const void* q8_act, float* out, int N, int K, void* stream);
void mongoose_q4_0_matvec_dp4a_batch(const void* w_q4_0, const void* q8_acts, float* out, int N, int K, int B, void* stream);

/* kernels.go:31, mongoose.cu:991-1013.  In place on x[seqLen, dim]; rotate-half
 * pairs (j, j+headDim/2); row `pos` of x uses table row `pos`. */
void mongoose_rope(float* x, const float* cosTab, const float* sinTab, int seqLen, int dim, int headDim, int nHeads, void* stream);
/* kernels.go:64, mongoose.cu:1644-1653.  cache[pos*kvDim + i] = src[i]. */
void mongoose_kv_cache_write(float* cache, const float* src, int pos, int kvDim, void* stream);
/* kernels.go:38, mongoose.cu:856-945.  Single query against [cacheLen, kvDim] caches, GQA. */
void mongoose_decode_attention(const float* Q, const float* K, const float* V, float* out,
                               int cacheLen, int dim, int kvDim, int nHeads, int nKVHeads, void* stream);
/* kernels.go:29, mongoose.cu:949-960.  out = gate * sigmoid(gate) * up. */
void mongoose_silu_gate_mul(const float* gate, const float* up, float* out, int n, void* stream);
/* kernels.go:17, mongoose.cu:212-219.  a += b. */
void mongoose_add_inplace(float* a, const float* b, int n, void* stream);
/* kernels.go:34, mongoose.cu:1052-1064.  out[p,:] = embed[tokens[p],:] (fp32 table). */
void mongoose_embed_gather(float* out, const float* embed, const int* tokens, int seqLen, int dim, void* stream);
/* kernels.go:41, mongoose.cu:1475-1499 (absmax convention: q * scales[r]/127). */
void mongoose_dequant_int8_to_fp32(const void* w_int8, const float* scales, float* out, int rows, int cols, void* stream);
/* q * scales[r] (per-row-scale convention) and GGUF Q4_0 blocks -> fp32. */
void mongoose_dequant_q8_rowscale(const void* w_int8, const float* scales, float* out, int rows, int cols, void* stream);
void mongoose_dequant_q4_0(const void* w_q4_0, float* out, int rows, int cols, void* stream);
/* kernels.go:24-26, mongoose.cu:356-368. */
/* out[T,N] (+)= act[T,K] . w[N,K]^T * scales[n] (+ bias[n]) on the matrix cores:
 * the multi-row form of mongoose_q8_matvec_rowscale, used by the batched
 * prefill.  The reference's nearest op is its dequantize-then-cuBLAS route
 * (mongoose_dequant_int8_to_fp32, mongoose.cu:1489, followed by MatMul,
 * cuda.go:230); here the int8 weights are read directly.  workspace: device
 * memory of at least 4 * roundup(T,128) * roundup(K,64) bytes for the two bf16
 * planes of the split activations.  K a multiple of 32; w and workspace
 * 16-byte aligned. */
void mongoose_q8_gemm(const float* act, const void* w, const float* scales, const float* bias, float* out, int T, int N,
                      int K, int accumulate, void* workspace, size_t workspaceBytes, void* stream);
/* No counterpart in the reference.  mongoose_q8_gemm for callers that cannot allocate and have no
 * workspace to hand over (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc): the two bf16 planes of the split activations are written into a static device array
 * of mg_q8_gemm_noalloc_max_bytes() = 8 MiB inside the library, so the call allocates nothing.
 * Limit: 4 * roundup(T,128) * roundup(K,64) <= 8 MiB (e.g. 512 x 4096, 128 x 16384); larger shapes
 * return MG_E_ARG with the sizes in mg_last_error().  Results are those of mongoose_q8_gemm bit
 * for bit.  All calls on one GPU share that GPU's array: calls that overlap in time on one GPU
 * (different streams or threads) race; serialise them.  Nothing in the array has to start at zero
 * (rows and k past the ends of the input are either not read or their results are dropped), so it
 * is not cleared between calls.  The array's device address is looked up once per device, by
 * tw_hip_init_device or by the first call on that device -- make one of the two before a capture
 * begins.  Returns MG_OK, MG_E_ARG or MG_E_HIP. */
int mg_q8_gemm_noalloc(const float* act, const void* w, const float* scales, const float* bias, float* out, int T, int N,
                       int K, int accumulate, void* stream);
size_t mg_q8_gemm_noalloc_max_bytes(void);
void mongoose_copy(void* dst, const void* src, size_t bytes, void* stream);
void mongoose_zero(void* ptr, size_t bytes, void* stream);
void mongoose_sync(void* stream);
/* kernels.go:326-330 (CUDACheck -> cudaPeekAtLastError): 0 when no launch has
 * failed since the last call, else the HIP error code; clears the record. */
int  mongoose_check(void);

/* ------------------------------------------------------------------ */
/* 3. Fused-inference context                                           */
/* ------------------------------------------------------------------ */
typedef struct mg_ctx mg_ctx;

/* NewCUDAFusedInference, cuda_fused_infer.go:144-229.  eps is the RMSNorm
 * epsilon (a parameter here; cpu.go:36).  NULL on failure. */
mg_ctx* mg_create(int dim, int kvDim, int headDim, int nHeads, int nKVHeads, int ffnDim,
                  int vocabSize, int nLayers, int maxSeq, double ropeTheta, float eps);
void    mg_destroy(mg_ctx* ctx);
const char* mg_last_error(void);

/* NumWeights, cuda_fused_infer.go:231-233: nLayers*12 + 2.  Slot map (:241-272):
 * l*12 + {0 norm1, 1 wq, 2 wk, 3 wv, 4 bq, 5 bk, 6 bv, 7 wo, 8 norm2, 9 gate,
 * 10 up, 11 down}; nLayers*12 final norm; nLayers*12+1 lm_head. */
int mg_num_weights(const mg_ctx* ctx);

/* SetWeight, cuda_fused_infer.go:241-272 + quantizeQ8 :363-390: fp32 in; matrix
 * slots are quantized to per-row int8 on the host and uploaded, norm gains
 * are uploaded as fp32.  Unlike the resident CUDA path (:255 skips them) bias
 * slots 4/5/6 are kept and added before RoPE, as cuda_fused_stream.go:319-321. */
int mg_set_weight(mg_ctx* ctx, int idx, const float* data, size_t n);
/* Already-quantized rows (same layout quantizeQ8 produces). */
int mg_set_weight_q8(mg_ctx* ctx, int idx, const int8_t* q, const float* scales);
/* SetWeightQ4_0, cuda_fused_infer_q4.go:46-90 + UploadQ4_0 cuda_q4_0.go:15-26:
 * raw GGUF block_q4_0 bytes, rows*(cols/32)*18. */
int mg_set_weight_q4_0(mg_ctx* ctx, int idx, const uint8_t* q4Data, size_t nbytes);
/* Q8 rounding used by mg_set_weight: 0 = truncate toward zero
 * (cuda_fused_infer.go:378), 1 = round half away from zero
 * (metal_impl_darwin.m:5776-5778).  Default 0. */
int mg_set_quant_rounding(mg_ctx* ctx, int mode);

/* Embedding table for mg_decode_token / mg_generate (the reference leaves the
 * lookup to its caller).  Without one, the lm_head row is used (tied weights). */
int mg_set_embedding_f16(mg_ctx* ctx, const uint16_t* table /* [vocab, dim] */);
int mg_set_embedding_f32(mg_ctx* ctx, const float* table /* [vocab, dim] */);

/* SetLayerRange :542-554 (allocates the fp32 KV caches of the owned layers),
 * ResetKV :530-537. */
int mg_set_layer_range(mg_ctx* ctx, int layerStart, int layerEnd);
int mg_reset_kv(mg_ctx* ctx);
/* KV cache row format: 0 = fp32 (the reference's layout, cuda_fused_infer.go:546),
 * 1 = fp16 rows (rounded to nearest even when a row is written; scores, softmax
 * and P.V stay fp32).  The reference only declares hooks for compressed caches
 * (kernels.go:71-72, no kernel source), so fp16 is this backend's own first step
 * in that direction: half the attention bytes at long context.  Must be called
 * before mg_set_layer_range (MG_E_STATE afterwards).  The per-op launches
 * (mongoose_kv_cache_write, mongoose_decode_attention) keep fp32 caches. */
int mg_set_kv_format(mg_ctx* ctx, int format);

/* PartialStep :392-452 / PartialStepQ4 cuda_fused_infer_q4.go:92.  hiddenIn
 * [dim] host floats, or NULL for the ...Continue forms (:456, q4:272) that keep
 * the device-resident hidden state.  logitsOut [vocab] is written when
 * layerEnd >= nLayers and it is not NULL; hiddenOut [dim] when
 * layerEnd < nLayers and it is not NULL. */
int mg_partial_step(mg_ctx* ctx, const float* hiddenIn, int pos, int layerStart, int layerEnd,
                    float* hiddenOut, float* logitsOut);
/* StepLayerResident, cuda_fused_infer_q4.go:451-605: one layer, with host
 * snapshots of the hidden state before (preOut) and after (postOut) it;
 * hiddenIn is uploaded when layer == 0; logitsOut as above. */
int mg_step_layer_resident(mg_ctx* ctx, int layer, int pos, const float* hiddenIn,
                           float* preOut, float* postOut, float* logitsOut);
/* ExportHidden :235-239.  The hidden state after mg_partial_step / mg_step_layer_resident /
 * mg_decode_token.  After launches of the captured graph (mg_graph_launch, mg_generate with
 * useGraph) the buffer already holds the next token's embedding instead. */
int mg_export_hidden(mg_ctx* ctx, float* out /* [dim] */);

/* L3 bridge and mailbox, cuda_fused_infer.go:118-131 and :556-737: every context owns a pinned host
 * buffer ([0:4] mailbox counter, [64:] hidden state) for handing a pipeline stage's output to the
 * host while the compute stream runs on.  mg_partial_step with both outputs NULL only queues the
 * stage's launches; then either
 *   mg_queue_hidden_to_l3 (QueueHiddenToL3 :688: the copy stream waits for the launches queued so
 *   far and copies the hidden state into the bridge), mg_wait_l3 (WaitL3 :709: waits for that copy
 *   only) and mg_get_l3_hidden (GetL3Hidden :725: host pointer to the dim floats), or
 *   mg_signal_mailbox (SignalMailbox :558: a kernel behind the stage's last launch moves the
 *   counter) and mg_wait_mailbox (WaitMailbox :575: the host polls the counter; here with a
 *   timeout in milliseconds, MG_E_HIP when it expires, MG_E_STATE when no signal is outstanding).
 * mg_swap_hidden_buffer (SwapHiddenBuffer :737) alternates the device hidden buffer, mg_hidden_idx
 * (HiddenIdx :603) returns which of the two is current. */
int mg_queue_hidden_to_l3(mg_ctx* ctx);
int mg_wait_l3(mg_ctx* ctx);
const float* mg_get_l3_hidden(mg_ctx* ctx);
int mg_signal_mailbox(mg_ctx* ctx);
int mg_wait_mailbox(mg_ctx* ctx, int timeoutMs);
int mg_swap_hidden_buffer(mg_ctx* ctx);
int mg_hidden_idx(mg_ctx* ctx);

/* Execution mode of the layer loop: 0 = one launch per reference op, in the
 * reference's order (cuda_fused_infer.go:417-443, 17 launches a layer);
 * 1 = fused launches (five a layer); 2 = fused launches whose attention launch does not
 * also fetch the following matrices into L2 with its idle workgroups (for a GPU
 * shared with other work); 3 = all layers of a step in ONE persistent launch whose
 * workgroups hand their vectors over through device memory, wherever the model allows it
 * (all matrices of the layers Q8, or all Q4_0; fp32 KV rows, heads of 64 or 128, a context of at most
 * 128 x floor(CUs / nKVHeads) positions -- an attention workgroup per query head and 128 positions where
 * that covers the context, else per KV head -- with at most 8 query heads a KV head; otherwise as mode 1).
 * In mode 3, 32 of the launch's workgroups compute nothing and instead read the weights that the others
 * will want next into the L2s, where a layer is small enough for that to pay (0.5B shape: 8 % faster);
 * 4 = mode 3 with every workgroup computing (bit-identical results; for comparison).
 * A new context is in mode 3 (measured against mode 1: 0.5B shape 56 % more tokens per second, 1.1B
 * shape 59 %, 8B shape 20 %, also at contexts of thousands of positions).
 * On every device one context at a time uses the persistent launch -- the first that needs it, until it is
 * destroyed or set to another mode; other contexts run the fused launches meanwhile (two such launches at
 * once could each hold part of the CUs and wait for workgroups that cannot start).
 * The persistent launch needs all its workgroups resident at once: on a GPU shared with
 * other kernels its waits can run into their time limit; the call then returns MG_E_HIP,
 * and the context continues with the fused launches.  All modes give the same results to
 * rounding. */
int mg_set_exec_mode(mg_ctx* ctx, int mode);

/* q4Matvec / q4MatvecPreq / q8QuantizeAct, cuda_fused_infer_q4.go:611-673: in the op-by-op loop (exec mode 0; any
 * other mode: MG_E_STATE) Q4_0 matrices are multiplied in the integer form -- the activation vector quantized to
 * int8 blocks (once for q, k, v and once for gate, up, as :161-173 and :208-212 do), then the packed int8 dot
 * products of mongoose_q4_0_matvec_dp4a_preq; Wo, down and lm_head quantize their own input (:197, :222, :601).
 * Off by default: the result carries the activation rounding (logits within about 1e-2 of the fp32-activation
 * path, not within its 1e-3 bar), which is why the fused and persistent launches keep fp32 activations.  Setting
 * another exec mode switches it off. */
int mg_set_q4_act_quant(mg_ctx* ctx, int on);

/* Whole token on the device: embedding gather -> layers -> final norm ->
 * lm_head -> greedy argmax (lowest index on ties).  logitsOut may be NULL. */
int mg_decode_token(mg_ctx* ctx, int token, int pos, int* nextToken, float* logitsOut);
/* Greedy generation: prompt tokens occupy positions 0..nPrompt-1, then
 * nDecode tokens are produced; outTokens [nDecode].  useGraph != 0 replays a
 * captured hipGraph per token (CaptureGraph / Launch, cuda_graph.go:315-669);
 * the position and the token stay in device memory between steps. */
int mg_generate(mg_ctx* ctx, const int* prompt, int nPrompt, int nDecode, int* outTokens, int useGraph);

/* Whole-token graphs (embedding gather .. argmax), the form the decode loop replays: capture once;
 * every launch advances the device-resident position by one.  mg_graph_validate replays one step both
 * ways and returns the largest absolute logit difference (the reference's criterion is < 1e-3,
 * cuda_graph.go:590-597).  No counterpart in the reference, whose graphs stop at the hidden state. */
int mg_graph_capture(mg_ctx* ctx);
int mg_graph_launch(mg_ctx* ctx, int token, int pos, int* nextToken);
int mg_graph_validate(mg_ctx* ctx, int token, int pos, float* maxAbsDiff);

/* CUDAGraph, cuda_graph.go:286-739: a captured graph over the layers [layerStart, layerEnd) that takes
 * the current hidden buffer as input and leaves its output there.
 *
 * mg_layer_graph_capture  = (*CUDAFusedInference).CaptureGraph(GraphCaptureConfig{LayerStart, LayerEnd,
 *     StreamCount, PipelineBreak}, pos), cuda_graph.go:315-498.  StreamCount 0 means 1 (:316); other
 *     values than 1 and 2 and a PipelineBreak outside (LayerStart, LayerEnd) with StreamCount 2 return
 *     NULL as there (:323, :396-400).  The reference's two-stream form runs stage B after stage A (an
 *     event joins them), so its result is that of one stream; here both forms are one capture on the
 *     context's stream.  pos is checked and otherwise unused: the kernels read the position from device
 *     memory, so one capture serves every position.
 * mg_layer_graph_launch   = (*CUDAGraph).Launch(pos), :663-669: writes the position, replays.
 *     Asynchronous on the context's stream like the reference's; mg_read_hidden / mg_export_hidden wait.
 * mg_layer_graph_update_and_launch = (*CUDAFusedInference).UpdateAndLaunch(g, pos), :673-714: returns 1
 *     (true) or 0.  The reference re-captures and updates the executable graph because pos is baked
 *     into its kernel arguments; here it is the same as a launch.
 * A graph whose operands went stale (a weight or cache replaced, the exec mode or the hidden buffer
 *     switched) is re-captured by its next launch.  Exec mode 0 (host-side positions) is not captured.
 * mg_layer_graph_destroy  = (*CUDAGraph).Destroy(), :716-739; a graph may be destroyed after its context.
 * mg_upload_hidden / mg_read_hidden = UploadHidden / ReadHidden, :650-658.
 * mg_validate_graph_capture = ValidateGraphCapture(hiddenIn, layerStart, layerEnd), :554-598: resets the
 *     KV cache, runs the range eagerly and through a fresh graph at position 0 on the same input, stores
 *     the largest absolute difference in *maxDiff and returns 1 when it is below 1e-3 (the reference's
 *     true), 0 when not, or a negative error code.  ValidateMultiStreamGraph (:603-647) is the same call.
 * mg_has_graph_kernel = HasGraphKernel(), :281: always 1 (the kernels here all take a device position). */
typedef struct mg_layer_graph mg_layer_graph;
mg_layer_graph* mg_layer_graph_capture(mg_ctx* ctx, int layerStart, int layerEnd, int streamCount, int pipelineBreak, int pos);
int mg_layer_graph_launch(mg_layer_graph* g, int pos);
int mg_layer_graph_update_and_launch(mg_layer_graph* g, int pos);
void mg_layer_graph_destroy(mg_layer_graph* g);
int mg_upload_hidden(mg_ctx* ctx, const float* data /* [dim] */);
int mg_read_hidden(mg_ctx* ctx, float* out /* [dim] */);
int mg_validate_graph_capture(mg_ctx* ctx, const float* hiddenIn, int layerStart, int layerEnd, float* maxDiff);
int mg_has_graph_kernel(void);

/* Timed decode for measurement: runs `steps` graph (or eager) decode steps
 * starting at device state (token, pos), bracketed by events on the context's
 * stream; returns elapsed milliseconds.  Inputs are resident before the timed
 * region starts. */
int mg_timed_decode(mg_ctx* ctx, int token, int pos, int steps, int useGraph, float* elapsedMs);

/* Per-launch-class timing inside a token, for the roofline report: `steps`
 * (<= 64) tokens from (token, pos) are issued launch by launch with an event
 * between every two launches, queued behind a gate so that the GPU never
 * waits for the host.  classMs[8] = mean milliseconds per launch
 * of class {0 embedding gather, 1 norm+QKV(+bias), 2 RoPE+KV write+attention,
 * 3 Wo+residual, 4 norm+gate/up+SiLU*mul, 5 down+residual, 6 final norm+lm_head
 * (+argmax partials), 7 argmax finish}; classLaunches[8] = launches per token.
 * classMask selects the classes to bracket (bit c = class c, 0 = all): every
 * event costs the stream a few microseconds, so one class alone is measured
 * closest to its kernel time. */
int mg_profile_decode(mg_ctx* ctx, int token, int pos, int steps, unsigned classMask, float* classMs, int* classLaunches);

/* Batched prefill -- the multi-token counterpart of the decode step, for the
 * prompt.  The reference has no batched prompt path: a caller feeds the prompt
 * through PartialStep one position at a time (cuda_fused_infer.go:392), and it has
 * GEMM-shaped launches only on its training path (cuda.go:230 MatMul via cuBLAS);
 * here the seven projections of a layer over nTokens rows are MFMA GEMMs that
 * read the int8 weights exactly (int8 is exact in bf16) against activations
 * split into two bf16 terms, so the result stays within ~1e-5 of the
 * token-by-token path.  Q4_0 weights are multiplied block by block (nibble - 8
 * is exact in bf16; the fp16 block scale is applied in fp32).  q/k/v, and
 * gate/up, of a layer must share one format (MG_E_UNSUPPORTED otherwise).
 * Positions pos0 .. pos0+nTokens-1 of the KV caches are written; the last
 * position goes through final norm, lm_head and argmax: *nextToken, logitsOut
 * [vocab] (both optional), and the device step state is left at pos0+nTokens
 * with that token, so mg_generate-style graph replays can follow.  elapsedMs
 * (optional) is the device time of the whole call measured with events. */
int mg_prefill(mg_ctx* ctx, const int* tokens, int nTokens, int pos0, int* nextToken, float* logitsOut, float* elapsedMs);
/* mg_generate with the prompt run through mg_prefill (nDecode >= 1). */
int mg_generate_prefill(mg_ctx* ctx, const int* prompt, int nPrompt, int nDecode, int* outTokens);

/* Measurement helper: mean microseconds of one dequantizing matvec launch at
 * shape [N, K] (wf 0 = Q8 per-row scale, 1 = Q4_0 split layout), over `iters`
 * launches that rotate through `copies` weight buffers (choose copies so that
 * copies * bytes exceeds the on-chip caches and every launch streams from
 * HBM).  nr (rows per wave group), ks (1 or 4: waves sharing a row group) and
 * grid = 0 use the library's own configuration. */
int mg_bench_matvec(int wf, int N, int K, int nr, int ks, int grid, int copies, int iters, float* avgUs);

/* Exec mode 3 hands vectors from phase to phase through an exchange area in device memory; this copies
 * layer `layer`'s block as the last step left it (cap floats at most) and describes it: geo[11] =
 * {floats per layer, offsets of q, current K row, current V row, attention partial accumulators
 * [smax, dim], their maxima [smax, nHeads], their sums [smax, nHeads], hidden after the attention
 * block, SwiGLU vector, layer output, smax}.  A float never written reads 0xFFFFFFFF.  For tests. */
int mg_flow_exchange(mg_ctx* ctx, int layer, float* out, size_t cap, int* geo);

/* 1 when a step over all layers goes through the persistent launch of exec mode 3 (mode, model and
 * context as they are now), else 0. */
int mg_flow_in_use(mg_ctx* ctx);

/* Timing diagnostic of exec mode 3: with enable != 0 every persistent launch records, per layer and
 * workgroup, when thread 0 passed each of 11 points (layer top; q|k|v input staged; q|k|v done; q, K, V
 * rows in; attention done; attention merged; Wo done; gate|up input staged; gate|up done; down input
 * staged; down done) in ticks of the 100 MHz wall clock.  out != NULL receives the last launch's ticks
 * [layer][point][workgroup] (cap int64 at least layers x 11 x workgroups), dims[3] = {layers, 11,
 * workgroups}.  enable == 0 stops and frees.  No counterpart in the reference; MG_E_STATE when the
 * persistent launch is not in use for the model. */
int mg_flow_trace(mg_ctx* ctx, int enable, long long* out, size_t cap, int* dims);

/* Whole tokens inside the persistent launch.  Where the launch is in use (mg_flow_in_use), the lm_head has
 * the layers' weight format and final norm and lm_head are set, a token's embedding gather, its layers, the
 * final norm, the lm_head matvec and the greedy argmax (cuda_fused_infer.go:446-450 plus what the
 * reference's caller does with the logits) all run in that one launch, and the calls that ask for a run
 * of tokens (mg_generate with useGraph, mg_timed_decode with useGraph, mg_generate_prefill) put up to
 * `n` tokens into each launch (default 64): the next token is chosen on the device and the launch goes on
 * with it.  n = 1: a launch (or a replay of the captured one-launch graph) per token.
 * mg_set_flow_tail(ctx, 0) goes back to separate lm_head and argmax launches behind the layers' launch
 * (for comparisons).  mg_flow_tail_in_use: 1 when tokens run that way as things stand.
 * mg_flow_tail_trace: with mg_flow_trace enabled, the tail's six points (tail top; final norm input
 * staged; lm_head done by the workgroup's first wave; token known; lm_head done by all its waves; all
 * workgroups' argmax partials in) of the last token a launch ran, ticks [point][workgroup], dims[2] =
 * {6, workgroups}.  No counterparts in the reference. */
int mg_set_flow_tail(mg_ctx* ctx, int on);
int mg_set_tokens_per_launch(mg_ctx* ctx, int n);
/* The persistent launch has variants with the sizes of known model shapes compiled in (Qwen2.5-0.5B, TinyLlama-1.1B,
 * Llama-3-8B: hidden size, K/V row, FFN width, head counts as constants instead of launch parameters); a context of
 * exactly such a shape takes them: same formulas over the same rows (results agree to rounding), 1-2 % faster.  on != 0: this context only takes
 * the variants whose sizes come with the launch (comparisons, tests).  No counterpart in the reference. */
int mg_set_flow_generic(mg_ctx* ctx, int on);
int mg_tokens_per_launch(mg_ctx* ctx);
int mg_flow_tail_in_use(mg_ctx* ctx);
int mg_flow_tail_trace(mg_ctx* ctx, long long* out, size_t cap, int* dims);

/* Time limit of each wait inside the persistent launch, in ticks of the 100 MHz wall clock (default
 * 5,000,000 = 50 ms).  A workgroup whose wait runs out stops waiting for the rest of the launch, the
 * launch ends normally with an error flag set, the call that issued it returns MG_E_HIP and the
 * context goes on with the fused launches.  A limit below zero makes every wait that is not satisfied
 * at once give up: the way the tests reach that path.  No counterpart in the reference. */
int mg_flow_set_wait_limit(mg_ctx* ctx, long long ticks);

/* Bytes of weights, scales and norm gains one token reads (the figure the
 * bandwidth roofline is computed from), and the KV bytes read at position pos. */
uint64_t mg_weight_bytes_per_token(const mg_ctx* ctx);
uint64_t mg_kv_bytes_at(const mg_ctx* ctx, int pos);

/* ------------------------------------------------------------------ */
/* Streaming inference (weights larger than device memory)              */
/* CUDAStreamInfer, cuda_fused_stream.go:98-726                         */
/* ------------------------------------------------------------------ */
typedef struct mg_stream mg_stream;
/* StreamBuild :127-198: two device weight sets + two pinned staging buffers.  The object uses the
 * context's stream and scratch; destroy it before the context.  If the context goes first the
 * object becomes inert: mg_stream_forward_token returns MG_E_STATE and mg_stream_destroy still
 * releases its own buffers. */
mg_stream* mg_stream_build(mg_ctx* ctx);
void       mg_stream_destroy(mg_stream* s);
/* StreamForwardToken :559-670.  layerPtrs[i*12+k] are host pointers to the
 * tensors of layer i in slot order (norm1, wq, wk, wv, bq, bk, bv, wo, norm2,
 * gate, up, down; bias pointers may be NULL), layerSizes[i*7+m] the byte sizes
 * of its seven Q4_0 matrices (wq, wk, wv, wo, gate, up, down).  The final norm
 * and lm_head come from the context (slots nLayers*12, +1). */
int mg_stream_forward_token(mg_stream* s, int pos, const float* embHidden, int nLayers,
                            const void* const* layerPtrs, const int32_t* layerSizes,
                            float* logitsOut);

/* ------------------------------------------------------------------ */
/* Host-side helpers shared with the loaders                            */
/* ------------------------------------------------------------------ */
/* quantizeQ8 (cuda_fused_infer.go:363-390) on the host; mode as mg_set_quant_rounding. */
void mg_quantize_q8(const float* w, int rows, int cols, int mode, int8_t* q, float* scales);
/* GGML quantize_row_q4_0 over rows*(cols/32) blocks -> 18-byte blocks. */
void mg_quantize_q4_0(const float* w, int rows, int cols, uint8_t* blocks);
uint16_t mg_f32_to_f16(float f);
float    mg_f16_to_f32(uint16_t h);
/* Deterministic synthetic weights: n samples of N(0, std) for stream (seed, idx),
 * identical on every machine (integer generator + fixed-order arithmetic). */
void mg_synth_normal(uint64_t seed, uint64_t idx, float std, float* out, size_t n);
/* n uniform ints in [0, bound). */
void mg_synth_tokens(uint64_t seed, uint64_t idx, int bound, int* out, size_t n);

#ifdef __cplusplus
}
#endif
#endif /* MONGOOSE_HIP_H */
