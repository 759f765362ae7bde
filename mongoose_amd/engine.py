"""Host-side mirror of mongoose's Go API for the fused quantized decode path.

Same names, argument meaning and error behaviour as the Go types they stand
in for, so that tests read like the reference's:

    HIP / NewHIP               Engine + the TensorEngine memory calls
                               (engine.go:7-29, tensor.go:29-49, cuda.go:198-223)
    Tensor                     tensor.go:15-89
    K* functions               kernels.go:600-1136 wrappers over the per-op launches
    HIPFusedInference          CUDAFusedInference (cuda_fused_infer.go,
                               cuda_fused_infer_q4.go, cuda_fused_infer_stub.go:7-49)
    HIPStreamInfer             CUDAStreamInfer (cuda_fused_stream.go)

Everything here is a thin ctypes call into libmongoose_hip.so; there is no
computation in Python and no CPU fallback.
"""
import ctypes

import numpy as np

from .lib import lib, last_error

_f = ctypes.POINTER(ctypes.c_float)
_i = ctypes.POINTER(ctypes.c_int)


def _fp(a):
    return a.ctypes.data_as(_f) if a is not None else None


def _ip(a):
    return a.ctypes.data_as(_i) if a is not None else None


def _as_f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


class Tensor:
    """Device buffer owned by an engine (tensor.go:15-27)."""

    def __init__(self, eng, ptr, nbytes, shape):
        self.eng, self._ptr, self.nbytes, self.Shape = eng, ptr, nbytes, list(shape)

    def DevicePtr(self):
        return self._ptr

    def Size(self):
        n = 1
        for s in self.Shape:
            n *= s
        return n

    def Release(self):
        if self._ptr:
            lib.tw_gpu_free(self._ptr)
            self._ptr = None


def ptrAdd(ptr, nbytes):
    """kernel_tensor.go:9-11."""
    return ctypes.c_void_p(ptr.value + nbytes if isinstance(ptr, ctypes.c_void_p) else ptr + nbytes)


class HIP:
    """The engine object NewHIP() returns (cuda.go:198-223 for CUDA)."""

    def __init__(self, name, vram):
        self._name, self._vram = name, vram

    def Name(self):
        return "hip/" + self._name

    def VRAM(self):
        return self._vram

    # TensorEngine memory calls (cuda_tensor.go:563-627, 980-990)
    def FromHost(self, data, shape):
        a = _as_f32(data)
        ptr = lib.tw_gpu_alloc(a.nbytes)
        if not ptr:
            return None
        lib.tw_gpu_upload(ptr, a.ctypes.data, a.nbytes)
        return Tensor(self, ptr, a.nbytes, shape)

    def Zeros(self, shape):
        n = int(np.prod(shape))
        ptr = lib.tw_gpu_alloc(n * 4)
        if not ptr:
            return None
        lib.tw_gpu_zero(ptr, n * 4)
        return Tensor(self, ptr, n * 4, shape)

    def ToHost(self, t):
        out = np.empty(t.Size(), dtype=np.float32)
        lib.tw_gpu_download(out.ctypes.data, t.DevicePtr(), out.nbytes)
        return out

    def UploadInto(self, t, data):
        a = _as_f32(data)
        lib.tw_gpu_upload(t.DevicePtr(), a.ctypes.data, a.nbytes)

    def UploadRawBytes(self, data):
        a = np.ascontiguousarray(data).view(np.uint8).ravel()
        ptr = lib.tw_gpu_alloc(a.nbytes)
        if not ptr:
            return None
        lib.tw_gpu_upload(ptr, a.ctypes.data, a.nbytes)
        return Tensor(self, ptr, a.nbytes, [a.nbytes])

    def DownloadRawBytes(self, t, nbytes=None):
        out = np.empty(nbytes if nbytes is not None else t.nbytes, dtype=np.uint8)
        lib.tw_gpu_download(out.ctypes.data, t.DevicePtr(), out.nbytes)
        return out

    def UploadQ4_0(self, q4Data, rows, cols):
        """cuda_q4_0.go:15-26: raw GGUF block_q4_0 bytes."""
        return self.UploadRawBytes(np.asarray(q4Data, dtype=np.uint8)[: rows * (cols // 32) * 18])


def NewHIP(device=0):
    """nil (None) when no device is present, as NewCUDA (cuda.go:209-217)."""
    if lib.tw_hip_init_device(device) != 0:
        return None
    name = ctypes.create_string_buffer(256)
    mem = ctypes.c_uint64(0)
    if lib.tw_hip_device_info(name, 256, ctypes.byref(mem)) != 0:
        return None
    return HIP(name.value.decode(), mem.value)


def KernelsLoaded():
    return True


# ---- kernels.go:600-1136 style wrappers (default stream, void) ----
def _p(x):
    return x.DevicePtr() if isinstance(x, Tensor) else x


def KRMSNormOut(inp, out, w, seqLen, dim):
    lib.mongoose_rmsnorm_out(_p(inp), _p(out), _p(w), seqLen, dim, None)


def KRMSNormOutEps(inp, out, w, seqLen, dim, eps):
    lib.mongoose_rmsnorm_out_eps(_p(inp), _p(out), _p(w), seqLen, dim, eps, None)


def KRMSNorm(x, w, seqLen, dim):
    """kernels.go:601: in place."""
    lib.mongoose_rmsnorm(_p(x), _p(w), seqLen, dim, None)


def KFusedAddRMSNorm(a, b, out, w, seqLen, dim):
    """kernels.go:641: out = rmsnorm(a + b, w)."""
    lib.mongoose_fused_add_rmsnorm(_p(a), _p(b), _p(out), _p(w), seqLen, dim, None)


def KFusedAddRMSNormEps(a, b, out, w, seqLen, dim, eps):
    lib.mongoose_fused_add_rmsnorm_eps(_p(a), _p(b), _p(out), _p(w), seqLen, dim, eps, None)


def KQ4Matvec(act, w, scales, out, N, K):
    """kernels.go:947: per-row-scale 4-bit weights (not GGUF Q4_0)."""
    lib.mongoose_q4_matvec(_p(act), _p(w), _p(scales), _p(out), N, K, None)


def KQ8Matvec(act, w, scales, out, N, K):
    lib.mongoose_q8_matvec(_p(act), _p(w), _p(scales), _p(out), N, K, None)


def KQ8MatvecRowScale(act, w, scales, out, N, K):
    lib.mongoose_q8_matvec_rowscale(_p(act), _p(w), _p(scales), _p(out), N, K, None)


def KQ4_0Matvec(act, w, out, N, K):
    lib.mongoose_q4_0_matvec(_p(act), _p(w), _p(out), N, K, None)


def KQ4_0Repack(w, planar, N, K):
    lib.mongoose_q4_0_repack(_p(w), _p(planar), N, K, None)


def KQ4_0MatvecPlanar(act, planar, out, N, K):
    lib.mongoose_q4_0_matvec_planar(_p(act), _p(planar), _p(out), N, K, None)


def KQ8QuantizeAct(act, q8Out, K):
    """kernels.go:993-996: fp32 activations -> int8 blocks, (K/32)*40 bytes."""
    lib.mongoose_q8_quantize_act(_p(act), _p(q8Out), K, None)


def KQ8QuantizeActBatch(acts, q8Out, K, B):
    """kernels.go:1011-1014."""
    lib.mongoose_q8_quantize_act_batch(_p(acts), _p(q8Out), K, B, None)


def KQ4_0MatvecDP4A(act, w, out, scratch, N, K):
    """kernels.go:985-988 (scratch: (K/32)*40 bytes)."""
    lib.mongoose_q4_0_matvec_dp4a(_p(act), _p(w), _p(out), N, K, _p(scratch), None)


def KQ4_0MatvecDP4APreq(w, q8Act, out, N, K):
    """kernels.go:998-1001."""
    lib.mongoose_q4_0_matvec_dp4a_preq(_p(w), _p(q8Act), _p(out), N, K, None)


def KQ4_0MatvecDP4ABatch(w, q8Acts, out, N, K, B):
    """kernels.go:1006-1009."""
    lib.mongoose_q4_0_matvec_dp4a_batch(_p(w), _p(q8Acts), _p(out), N, K, B, None)


def KRoPE(x, cos, sin, seqLen, dim, headDim, nHeads):
    lib.mongoose_rope(_p(x), _p(cos), _p(sin), seqLen, dim, headDim, nHeads, None)


def KKVCacheWrite(cache, src, pos, kvDim):
    lib.mongoose_kv_cache_write(_p(cache), _p(src), pos, kvDim, None)


def KDecodeAttention(Q, K, V, out, cacheLen, dim, kvDim, nHeads, nKVHeads):
    lib.mongoose_decode_attention(_p(Q), _p(K), _p(V), _p(out), cacheLen, dim, kvDim, nHeads, nKVHeads, None)


def KSiLUGateMul(gate, up, out, n):
    lib.mongoose_silu_gate_mul(_p(gate), _p(up), _p(out), n, None)


def KAddInPlace(a, b, n):
    lib.mongoose_add_inplace(_p(a), _p(b), n, None)


def KEmbedGather2(out, embed, tokens, seqLen, dim):
    lib.mongoose_embed_gather(_p(out), _p(embed), _p(tokens), seqLen, dim, None)


def KDequantInt8ToFP32(w, scales, out, rows, cols):
    lib.mongoose_dequant_int8_to_fp32(_p(w), _p(scales), _p(out), rows, cols, None)


def KDequantQ8RowScale(w, scales, out, rows, cols):
    lib.mongoose_dequant_q8_rowscale(_p(w), _p(scales), _p(out), rows, cols, None)


def KDequantQ4_0(w, out, rows, cols):
    lib.mongoose_dequant_q4_0(_p(w), _p(out), rows, cols, None)


def KCopy(dst, src, nbytes):
    lib.mongoose_copy(_p(dst), _p(src), nbytes, None)


def KZero(ptr, nbytes):
    lib.mongoose_zero(_p(ptr), nbytes, None)


def KSync():
    lib.mongoose_sync(None)


# ---- kernel_tensor.go:14-94: the tensor-typed helpers over the K* set ----
class Q8Weight:
    """kernel_tensor.go:14-21."""

    def __init__(self, Data, Scales, Rows, Cols, Q4=False):
        self.Data, self.Scales, self.Rows, self.Cols, self.Q4 = Data, Scales, Rows, Cols, Q4


def TRMSNorm(x, weight, seqLen, dim):
    KRMSNorm(x, weight, seqLen, dim)                          # kernel_tensor.go:23-26


def TRMSNormOut(inp, out, weight, seqLen, dim):
    KRMSNormOut(inp, out, weight, seqLen, dim)                # :28-31


def TQ8Matvec(act, w, out):
    """kernel_tensor.go:33-41: the 4-bit or the 8-bit kernel by w.Q4."""
    if w.Q4:
        KQ4Matvec(act, w.Data, w.Scales, out, w.Rows, w.Cols)
    else:
        KQ8Matvec(act, w.Data, w.Scales, out, w.Rows, w.Cols)


def TRoPE(x, cos, sin, seqLen, dim, headDim, nHeads):
    KRoPE(x, cos, sin, seqLen, dim, headDim, nHeads)          # :43-46


def TDecodeAttention(q, kCache, vCache, out, cacheLen, dim, kvDim, numHeads, numKVHeads):
    KDecodeAttention(q, kCache, vCache, out, cacheLen, dim, kvDim, numHeads, numKVHeads)   # :48-53


def TSiLUGateMul(gate, up, out, n):
    KSiLUGateMul(gate, up, out, n)                            # :55-58


def TCopy(dst, src, nbytes):
    KCopy(dst, src, nbytes)                                   # :60-63


def TCopyAt(dst, dstByteOffset, src, nbytes):
    KCopy(_p(dst) + dstByteOffset, src, nbytes)               # :65-69


def TAddInPlace(a, b, n):
    KAddInPlace(a, b, n)                                      # :71-74


def TRoPEAt(x, cosTable, sinTable, byteOffset, seqLen, dim, headDim, nHeads):
    """kernel_tensor.go:76-79: the table row of a position is passed as a byte offset."""
    KRoPE(x, _p(cosTable) + byteOffset, _p(sinTable) + byteOffset, seqLen, dim, headDim, nHeads)


def TDecodeAttentionKV(q, kCache, vCache, out, cacheLen, dim, kvDim, numHeads, numKVHeads):
    KDecodeAttention(q, kCache, vCache, out, cacheLen, dim, kvDim, numHeads, numKVHeads)   # :81-85


def TZero(t, nBytes):
    KZero(t, nBytes)                                          # :92-95


def PackInt8ToFloat32(q):
    """kernel_tensor.go:97-106: int8 bytes viewed as float32 words (padded to a multiple of four)."""
    b = np.ascontiguousarray(q, dtype=np.int8).view(np.uint8).ravel()
    buf = np.zeros((b.size + 3) // 4 * 4, np.uint8)
    buf[:b.size] = b
    return buf.view(np.float32)


def HIPCheck():
    """kernels.go:732-736 CUDACheck: 0 when no launch failed."""
    return lib.mongoose_check()


# ---- host helpers ----
def quantize_q8(w, mode=0):
    w = _as_f32(w)
    rows, cols = w.shape
    q = np.empty((rows, cols), dtype=np.int8)
    s = np.empty(rows, dtype=np.float32)
    lib.mg_quantize_q8(_fp(w), rows, cols, mode, q.ctypes.data_as(ctypes.POINTER(ctypes.c_int8)), _fp(s))
    return q, s


def quantize_q4_0(w):
    w = _as_f32(w)
    rows, cols = w.shape
    out = np.empty(rows * (cols // 32) * 18, dtype=np.uint8)
    lib.mg_quantize_q4_0(_fp(w), rows, cols, out.ctypes.data_as(ctypes.POINTER(ctypes.c_uint8)))
    return out


def synth_normal(seed, idx, std, shape):
    out = np.empty(shape, dtype=np.float32)
    lib.mg_synth_normal(seed, idx, std, _fp(out), out.size)
    return out


def synth_tokens(seed, idx, bound, n):
    out = np.empty(n, dtype=np.int32)
    lib.mg_synth_tokens(seed, idx, bound, _ip(out), n)
    return out


class GraphCaptureConfig:
    """cuda_graph.go:292-298."""

    def __init__(self, LayerStart=0, LayerEnd=0, StreamCount=1, PipelineBreak=0):
        self.LayerStart, self.LayerEnd, self.StreamCount, self.PipelineBreak = LayerStart, LayerEnd, StreamCount, PipelineBreak


class HIPGraph:
    """CUDAGraph, cuda_graph.go:300-310: a captured graph over a range of layers."""

    def __init__(self, handle, cfg):
        self._h, self.config = handle, cfg

    def Launch(self, pos):
        """cuda_graph.go:663: asynchronous; ReadHidden / ExportHidden wait for it."""
        if not self._h:
            return -1
        return lib.mg_layer_graph_launch(self._h, pos)

    def Destroy(self):
        """cuda_graph.go:716."""
        if self._h:
            lib.mg_layer_graph_destroy(self._h)
            self._h = None


def HasGraphKernel():
    """cuda_graph.go:281."""
    return lib.mg_has_graph_kernel() != 0


class HIPFusedInference:
    """Method set of CUDAFusedInference (cuda_fused_infer_stub.go:11-49)."""

    def __init__(self, handle, shape):
        self._h = handle
        (self.dim, self.kvDim, self.headDim, self.nHeads, self.nKVHeads, self.ffnDim, self.vocabSize,
         self.nLayers, self.maxSeq) = shape

    def Close(self):
        if self._h:
            lib.mg_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.Close()
        except Exception:
            pass

    def NumWeights(self):
        return lib.mg_num_weights(self._h)

    def SetWeight(self, idx, data):
        a = _as_f32(data).ravel()
        return lib.mg_set_weight(self._h, idx, _fp(a), a.size)

    def SetWeightQ8(self, idx, q, scales):
        q = np.ascontiguousarray(q, dtype=np.int8)
        s = _as_f32(scales)
        return lib.mg_set_weight_q8(self._h, idx, q.ctypes.data_as(ctypes.POINTER(ctypes.c_int8)), _fp(s))

    def SetWeightQ4_0(self, idx, q4Data):
        a = np.ascontiguousarray(q4Data, dtype=np.uint8).ravel()
        return lib.mg_set_weight_q4_0(self._h, idx, a.ctypes.data_as(ctypes.POINTER(ctypes.c_uint8)), a.size)

    def SetQuantRounding(self, mode):
        return lib.mg_set_quant_rounding(self._h, mode)

    def SetEmbeddingF16(self, table):
        a = np.ascontiguousarray(table).view(np.uint16)
        return lib.mg_set_embedding_f16(self._h, a.ctypes.data_as(ctypes.POINTER(ctypes.c_uint16)))

    def SetEmbeddingF32(self, table):
        a = _as_f32(table)
        return lib.mg_set_embedding_f32(self._h, _fp(a))

    def SetLayerRange(self, layerStart, layerEnd):
        return lib.mg_set_layer_range(self._h, layerStart, layerEnd)

    def SetKVFormat(self, fmt):
        """0 = fp32 KV rows, 1 = fp16; before SetLayerRange."""
        return lib.mg_set_kv_format(self._h, fmt)

    def ResetKV(self):
        return lib.mg_reset_kv(self._h)

    def SetExecMode(self, mode):
        """0 = one launch per reference op, 1 = fused launches, 2 = fused without the L2 prefetch helpers,
        3 (default) = all layers in one persistent launch where the model allows it, 4 = mode 3 without the
        workgroups that prefetch weights."""
        return lib.mg_set_exec_mode(self._h, mode)

    def SetQ4ActQuant(self, on):
        """cuda_fused_infer_q4.go:611-673: Q4_0 matrices through the int8-activation (dp4a) matvecs; exec mode 0 only."""
        return lib.mg_set_q4_act_quant(self._h, 1 if on else 0)

    # L3 bridge and mailbox (cuda_fused_infer.go:556-737)
    def QueueHiddenToL3(self):
        return lib.mg_queue_hidden_to_l3(self._h)

    def WaitL3(self):
        return lib.mg_wait_l3(self._h)

    def GetL3Hidden(self):
        """Host view (no copy) of the bridge's hidden state; valid after QueueHiddenToL3 + WaitL3."""
        p = lib.mg_get_l3_hidden(self._h)
        return np.ctypeslib.as_array(p, shape=(self.dim,)) if p else None

    def HasL3(self):
        return bool(lib.mg_get_l3_hidden(self._h))

    def SignalMailbox(self):
        return lib.mg_signal_mailbox(self._h)

    def WaitMailbox(self, timeoutMs=2000):
        return lib.mg_wait_mailbox(self._h, timeoutMs)

    def SwapHiddenBuffer(self):
        return lib.mg_swap_hidden_buffer(self._h)

    def HiddenIdx(self):
        return lib.mg_hidden_idx(self._h)

    def PartialStep(self, hiddenIn, pos, layerStart, layerEnd, hiddenOut, logitsOut):
        h = _as_f32(hiddenIn) if hiddenIn is not None else None
        return lib.mg_partial_step(self._h, _fp(h), pos, layerStart, layerEnd, _fp(hiddenOut), _fp(logitsOut))

    def PartialStepContinue(self, pos, layerStart, layerEnd, hiddenOut, logitsOut):
        return lib.mg_partial_step(self._h, None, pos, layerStart, layerEnd, _fp(hiddenOut), _fp(logitsOut))

    # the Q4 step is the same entry point: the weight format is a property of each matrix
    PartialStepQ4 = PartialStep
    PartialStepQ4Continue = PartialStepContinue

    def StepLayerResident(self, layer, pos, hiddenIn, preOut, postOut, logitsOut):
        h = _as_f32(hiddenIn) if hiddenIn is not None else None
        return lib.mg_step_layer_resident(self._h, layer, pos, _fp(h), _fp(preOut), _fp(postOut), _fp(logitsOut))

    def ExportHidden(self):
        out = np.empty(self.dim, dtype=np.float32)
        rc = lib.mg_export_hidden(self._h, _fp(out))
        return out if rc == 0 else None

    def DecodeToken(self, token, pos, logitsOut=None):
        nxt = ctypes.c_int(-1)
        rc = lib.mg_decode_token(self._h, token, pos, ctypes.byref(nxt), _fp(logitsOut))
        return rc, nxt.value

    def Generate(self, prompt, nDecode, useGraph=True):
        p = np.ascontiguousarray(prompt, dtype=np.int32)
        out = np.empty(max(nDecode, 1), dtype=np.int32)
        rc = lib.mg_generate(self._h, _ip(p), p.size, nDecode, _ip(out), 1 if useGraph else 0)
        return rc, out[:nDecode]

    def CaptureTokenGraph(self):
        """mg_graph_capture: the whole-token graphs (embedding gather .. argmax) that Generate / GraphLaunch replay."""
        return lib.mg_graph_capture(self._h)

    def GraphLaunch(self, token, pos):
        nxt = ctypes.c_int(-1)
        rc = lib.mg_graph_launch(self._h, token, pos, ctypes.byref(nxt))
        return rc, nxt.value

    def ValidateGraph(self, token, pos):
        md = ctypes.c_float(0)
        rc = lib.mg_graph_validate(self._h, token, pos, ctypes.byref(md))
        return rc, md.value

    # ---- CUDAGraph mirror, cuda_graph.go:286-739 ----
    def CaptureGraph(self, cfg, pos):
        """(*CUDAFusedInference).CaptureGraph(cfg, pos), cuda_graph.go:315: a HIPGraph over cfg.LayerStart ..
        cfg.LayerEnd, or None (error text in last_error())."""
        h = lib.mg_layer_graph_capture(self._h, cfg.LayerStart, cfg.LayerEnd, cfg.StreamCount, cfg.PipelineBreak, pos)
        return HIPGraph(h, cfg) if h else None

    def UpdateAndLaunch(self, g, pos):
        """cuda_graph.go:673: True when the graph was launched at pos."""
        return bool(g._h) and lib.mg_layer_graph_update_and_launch(g._h, pos) == 1

    def UploadHidden(self, data):
        """cuda_graph.go:650."""
        d = np.ascontiguousarray(data, dtype=np.float32)
        assert d.size == self.dim
        return lib.mg_upload_hidden(self._h, _fp(d))

    def ReadHidden(self):
        """cuda_graph.go:655: the current hidden buffer (waits for the stream)."""
        out = np.empty(self.dim, dtype=np.float32)
        return out if lib.mg_read_hidden(self._h, _fp(out)) == 0 else None

    def ValidateGraphCapture(self, hiddenIn, layerStart, layerEnd):
        """cuda_graph.go:554-598: eager and graph output of the range at position 0 differ by less than 1e-3.
        Returns (ok, maxDiff)."""
        d = np.ascontiguousarray(hiddenIn, dtype=np.float32)
        md = ctypes.c_float(0)
        rc = lib.mg_validate_graph_capture(self._h, _fp(d), layerStart, layerEnd, ctypes.byref(md))
        return rc == 1, md.value

    def ValidateMultiStreamGraph(self, hiddenIn, layerStart, layerEnd, pipelineBreak):
        """cuda_graph.go:603-647.  The two-stream graph of the reference is sequential (stage B waits for stage A),
        so this is ValidateGraphCapture with the break checked."""
        if pipelineBreak <= layerStart or pipelineBreak >= layerEnd:
            return False, float("nan")
        return self.ValidateGraphCapture(hiddenIn, layerStart, layerEnd)

    def TestMinimalCapture(self):
        """cuda_graph.go:536: the graph API works on this runtime (a one-layer capture and replay)."""
        g = self.CaptureGraph(GraphCaptureConfig(0, 1), 0)
        if g is None:
            return False
        g.Destroy()
        return True

    def TimedDecode(self, token, pos, steps, useGraph=True):
        ms = ctypes.c_float(0)
        rc = lib.mg_timed_decode(self._h, token, pos, steps, 1 if useGraph else 0, ctypes.byref(ms))
        return rc, ms.value

    def ProfileDecode(self, token, pos, steps, classMask=0):
        ms = np.zeros(8, dtype=np.float32)
        n = np.zeros(8, dtype=np.int32)
        rc = lib.mg_profile_decode(self._h, token, pos, steps, classMask, _fp(ms), _ip(n))
        return rc, ms, n

    def Prefill(self, tokens, pos0=0, wantLogits=False):
        """Batched prefill of `tokens` at positions pos0.. ; returns (rc, nextToken, logits or None, device ms)."""
        toks = np.ascontiguousarray(tokens, dtype=np.int32)
        nxt = ctypes.c_int(-1)
        ms = ctypes.c_float(0.0)
        logits = np.zeros(self.vocabSize, dtype=np.float32) if wantLogits else None
        rc = lib.mg_prefill(self._h, _ip(toks), len(toks), pos0, ctypes.byref(nxt),
                            _fp(logits) if wantLogits else None, ctypes.byref(ms))
        return rc, nxt.value, logits, ms.value

    def GeneratePrefill(self, prompt, nDecode):
        p = np.ascontiguousarray(prompt, dtype=np.int32)
        out = np.zeros(max(nDecode, 1), dtype=np.int32)
        rc = lib.mg_generate_prefill(self._h, _ip(p), len(p), nDecode, _ip(out))
        return rc, out[:nDecode]

    def FlowExchange(self, layer):
        """The persistent layer launch's exchange block of `layer` after the last step, as a dict of named
        vectors (tests); None when that launch is not in use."""
        geo = np.zeros(11, dtype=np.int32)
        if not self.FlowInUse() or lib.mg_flow_exchange(self._h, layer, None, 0, _ip(geo)) != 0:
            return None
        buf = np.empty(int(geo[0]), dtype=np.float32)
        if lib.mg_flow_exchange(self._h, layer, _fp(buf), buf.size, _ip(geo)) != 0:
            return None
        stride, oq, okc, ovc, opa, opm, opl, ox1, om, ox2, smax = [int(x) for x in geo]
        kv = self.kvDim
        return {"q": buf[oq:oq + self.dim], "k": buf[okc:okc + kv], "v": buf[ovc:ovc + kv],
                "pacc": buf[opa:opa + smax * self.dim].reshape(smax, self.dim),
                "pm": buf[opm:opm + smax * self.nHeads].reshape(smax, self.nHeads),
                "pl": buf[opl:opl + smax * self.nHeads].reshape(smax, self.nHeads),
                "x1": buf[ox1:ox1 + self.dim], "m": buf[om:om + self.ffnDim], "x2": buf[ox2:ox2 + self.dim], "smax": smax}

    FLOW_TRACE_POINTS = ("layer-top", "qkv-input-staged", "qkv-done", "q-k-v-rows-in", "attention-done", "attention-merged",
                         "wo-done", "gate-up-input-staged", "gate-up-done", "down-input-staged", "down-done")

    def FlowTrace(self, enable=True, read=False):
        """Timing diagnostic of the persistent layer launch (mg_flow_trace).  enable starts / stops recording;
        read=True returns the last launch's ticks (10 ns) as an int64 array [layer, point, workgroup]."""
        dims = np.zeros(3, dtype=np.int32)
        rc = lib.mg_flow_trace(self._h, 1 if enable else 0, None, 0, _ip(dims))
        if rc != 0 or not read:
            return rc, None
        buf = np.zeros(int(dims[0]) * int(dims[1]) * int(dims[2]), dtype=np.int64)
        rc = lib.mg_flow_trace(self._h, 1, buf.ctypes.data_as(ctypes.POINTER(ctypes.c_longlong)), buf.size, _ip(dims))
        return rc, buf.reshape(int(dims[0]), int(dims[1]), int(dims[2]))

    def FlowInUse(self):
        """True when a step over all layers goes through the persistent layer launch."""
        return lib.mg_flow_in_use(self._h) == 1

    FLOW_TAIL_TRACE_POINTS = ("tail-top", "final-input-staged", "lm-head-done", "token-known", "all-waves-done", "partials-in")

    def FlowTailInUse(self):
        """True when whole tokens (embedding .. argmax) run inside the persistent launch."""
        return lib.mg_flow_tail_in_use(self._h) == 1

    def SetFlowTail(self, on):
        return lib.mg_set_flow_tail(self._h, 1 if on else 0)

    def SetFlowGeneric(self, on):
        """on: only the persistent launch's variants whose sizes come with the launch (none with a known shape's compiled in)."""
        return lib.mg_set_flow_generic(self._h, 1 if on else 0)

    def SetTokensPerLaunch(self, n):
        return lib.mg_set_tokens_per_launch(self._h, int(n))

    def TokensPerLaunch(self):
        return lib.mg_tokens_per_launch(self._h)

    def FlowTailTrace(self):
        """Ticks (10 ns) [point, workgroup] of the tail of the last token a launch ran (trace enabled)."""
        dims = np.zeros(2, dtype=np.int32)
        rc = lib.mg_flow_tail_trace(self._h, None, 0, _ip(dims))
        if rc != 0:
            return rc, None
        buf = np.zeros(int(dims[0]) * int(dims[1]), dtype=np.int64)
        rc = lib.mg_flow_tail_trace(self._h, buf.ctypes.data_as(ctypes.POINTER(ctypes.c_longlong)), buf.size, _ip(dims))
        return rc, buf.reshape(int(dims[0]), int(dims[1]))

    def SetFlowWaitLimit(self, ticks):
        """Per-wait time limit of the persistent layer launch in 10 ns ticks (negative: give up at once)."""
        return lib.mg_flow_set_wait_limit(self._h, int(ticks))

    def WeightBytesPerToken(self):
        return lib.mg_weight_bytes_per_token(self._h)

    def KVBytesAt(self, pos):
        return lib.mg_kv_bytes_at(self._h, pos)

    def StreamBuild(self):
        h = lib.mg_stream_build(self._h)
        return HIPStreamInfer(h, self) if h else None


def NewHIPFusedInference(eng, dim, kvDim, headDim, nHeads, nKVHeads, ffnDim, vocabSize, nLayers, maxSeq,
                         ropeTheta, eps=1e-6):
    """NewCUDAFusedInference (cuda_fused_infer.go:144): None on failure."""
    if eng is None:
        return None
    h = lib.mg_create(dim, kvDim, headDim, nHeads, nKVHeads, ffnDim, vocabSize, nLayers, maxSeq,
                      float(ropeTheta), float(eps))
    if not h:
        return None
    return HIPFusedInference(h, (dim, kvDim, headDim, nHeads, nKVHeads, ffnDim, vocabSize, nLayers, maxSeq))


class HIPStreamInfer:
    """CUDAStreamInfer (cuda_fused_stream.go:98-126)."""

    def __init__(self, handle, parent):
        self._h, self._parent = handle, parent

    def Close(self):
        if self._h:
            lib.mg_stream_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.Close()
        except Exception:
            pass

    def StreamForwardToken(self, pos, embHidden, nLayers, layerPtrs, layerSizes, logitsOut):
        """layerPtrs: list of nLayers*12 numpy arrays or None; layerSizes: nLayers*7 ints."""
        keep = [np.ascontiguousarray(a) if a is not None else None for a in layerPtrs]
        arr = (ctypes.c_void_p * len(keep))(*[a.ctypes.data if a is not None else None for a in keep])
        sizes = np.ascontiguousarray(layerSizes, dtype=np.int32)
        h = _as_f32(embHidden)
        return lib.mg_stream_forward_token(self._h, pos, _fp(h), nLayers, arr,
                                           sizes.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)), _fp(logitsOut))


def KQ8GemmNoAlloc(act, w, scales, bias, out, T, N, K, accumulate):
    """KQ8Gemm without a workspace: the split planes live in the library's static scratch array."""
    return lib.mg_q8_gemm_noalloc(_p(act), _p(w), _p(scales), _p(bias) if bias is not None else None, _p(out), T, N, K,
                                  1 if accumulate else 0, None)


def KQ8Gemm(act, w, scales, bias, out, T, N, K, accumulate, workspace, workspaceBytes):
    """Multi-row form of KQ8MatvecRowScale on the matrix cores (out[T,N] (+)= act[T,K] . w[N,K]^T * scales + bias)."""
    lib.mongoose_q8_gemm(_p(act), _p(w), _p(scales), _p(bias) if bias is not None else None, _p(out), T, N, K,
                         1 if accumulate else 0, _p(workspace), workspaceBytes, None)
