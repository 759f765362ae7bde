"""ctypes loader for libmongoose_hip.so (the C ABI declared in include/mongoose_hip.h).

There is no fallback: if the library has not been built, importing this module
raises.  Build it with ``python -m mongoose_amd.build``.
"""
import ctypes
import os
from ctypes import (POINTER, c_char_p, c_double, c_float, c_int, c_int8, c_int32, c_size_t, c_uint8,
                    c_uint16, c_uint64, c_void_p)

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libmongoose_hip.so")

if not os.path.exists(LIB_PATH):
    raise ImportError(
        f"{LIB_PATH} is missing: the HIP library has not been built "
        "(run `python -m mongoose_amd.build`); there is no CPU fallback")

lib = ctypes.CDLL(LIB_PATH, mode=ctypes.RTLD_GLOBAL)

_f = POINTER(c_float)
_i = POINTER(c_int)


def _sig(name, restype, *argtypes):
    fn = getattr(lib, name)
    fn.restype = restype
    fn.argtypes = list(argtypes)
    return fn


# 1. memory shim
_sig("tw_gpu_alloc", c_void_p, c_size_t)
_sig("tw_gpu_free", None, c_void_p)
_sig("tw_gpu_upload", None, c_void_p, c_void_p, c_size_t)
_sig("tw_gpu_download", None, c_void_p, c_void_p, c_size_t)
_sig("tw_gpu_zero", None, c_void_p, c_size_t)
_sig("tw_gpu_alloc_pinned", c_void_p, c_size_t)
_sig("tw_gpu_free_pinned", None, c_void_p)
_sig("tw_hip_init_device", c_int, c_int)
_sig("tw_hip_device_info", c_int, c_char_p, c_size_t, POINTER(c_uint64))

# 2. per-op kernels (device pointers are passed as void*)
_p = c_void_p
_sig("mongoose_rmsnorm_out", None, _p, _p, _p, c_int, c_int, _p)
_sig("mongoose_rmsnorm_out_eps", None, _p, _p, _p, c_int, c_int, c_float, _p)
_sig("mongoose_rmsnorm", None, _p, _p, c_int, c_int, _p)
_sig("mongoose_fused_add_rmsnorm", None, _p, _p, _p, _p, c_int, c_int, _p)
_sig("mongoose_fused_add_rmsnorm_eps", None, _p, _p, _p, _p, c_int, c_int, c_float, _p)
_sig("mongoose_q4_matvec", None, _p, _p, _p, _p, c_int, c_int, _p)
_sig("mongoose_q8_matvec", None, _p, _p, _p, _p, c_int, c_int, _p)
_sig("mongoose_q8_matvec_rowscale", None, _p, _p, _p, _p, c_int, c_int, _p)
_sig("mongoose_q4_0_matvec", None, _p, _p, _p, c_int, c_int, _p)
_sig("mongoose_q4_0_repack", None, _p, _p, c_int, c_int, _p)
_sig("mongoose_q4_0_matvec_planar", None, _p, _p, _p, c_int, c_int, _p)
_sig("mongoose_rope", None, _p, _p, _p, c_int, c_int, c_int, c_int, _p)
_sig("mongoose_kv_cache_write", None, _p, _p, c_int, c_int, _p)
_sig("mongoose_decode_attention", None, _p, _p, _p, _p, c_int, c_int, c_int, c_int, c_int, _p)
_sig("mongoose_silu_gate_mul", None, _p, _p, _p, c_int, _p)
_sig("mongoose_add_inplace", None, _p, _p, c_int, _p)
_sig("mongoose_embed_gather", None, _p, _p, _p, c_int, c_int, _p)
_sig("mongoose_dequant_int8_to_fp32", None, _p, _p, _p, c_int, c_int, _p)
_sig("mongoose_dequant_q8_rowscale", None, _p, _p, _p, c_int, c_int, _p)
_sig("mongoose_dequant_q4_0", None, _p, _p, c_int, c_int, _p)
_sig("mongoose_q8_quantize_act", None, _p, _p, c_int, _p)
_sig("mongoose_q8_quantize_act_batch", None, _p, _p, c_int, c_int, _p)
_sig("mongoose_q4_0_matvec_dp4a", None, _p, _p, _p, c_int, c_int, _p, _p)
_sig("mongoose_q4_0_matvec_dp4a_preq", None, _p, _p, _p, c_int, c_int, _p)
_sig("mongoose_q4_0_matvec_dp4a_batch", None, _p, _p, _p, c_int, c_int, c_int, _p)
_sig("mongoose_q8_gemm", None, _p, _p, _p, _p, _p, c_int, c_int, c_int, c_int, _p, c_size_t, _p)
_sig("mg_q8_gemm_noalloc", c_int, _p, _p, _p, _p, _p, c_int, c_int, c_int, c_int, _p)
_sig("mg_q8_gemm_noalloc_max_bytes", c_size_t)
_sig("mongoose_copy", None, _p, _p, c_size_t, _p)
_sig("mongoose_zero", None, _p, c_size_t, _p)
_sig("mongoose_sync", None, _p)
_sig("mongoose_check", c_int)

# 3. fused-inference context
_sig("mg_create", c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_double, c_float)
_sig("mg_destroy", None, c_void_p)
_sig("mg_last_error", c_char_p)
_sig("mg_num_weights", c_int, c_void_p)
_sig("mg_set_weight", c_int, c_void_p, c_int, _f, c_size_t)
_sig("mg_set_weight_q8", c_int, c_void_p, c_int, POINTER(c_int8), _f)
_sig("mg_set_weight_q4_0", c_int, c_void_p, c_int, POINTER(c_uint8), c_size_t)
_sig("mg_set_q4_act_quant", c_int, c_void_p, c_int)
_sig("mg_set_quant_rounding", c_int, c_void_p, c_int)
_sig("mg_set_embedding_f16", c_int, c_void_p, POINTER(c_uint16))
_sig("mg_set_embedding_f32", c_int, c_void_p, _f)
_sig("mg_set_layer_range", c_int, c_void_p, c_int, c_int)
_sig("mg_reset_kv", c_int, c_void_p)
_sig("mg_set_kv_format", c_int, c_void_p, c_int)
_sig("mg_partial_step", c_int, c_void_p, _f, c_int, c_int, c_int, _f, _f)
_sig("mg_step_layer_resident", c_int, c_void_p, c_int, c_int, _f, _f, _f, _f)
_sig("mg_export_hidden", c_int, c_void_p, _f)
_sig("mg_set_exec_mode", c_int, c_void_p, c_int)
_sig("mg_queue_hidden_to_l3", c_int, c_void_p)
_sig("mg_wait_l3", c_int, c_void_p)
_sig("mg_get_l3_hidden", _f, c_void_p)
_sig("mg_signal_mailbox", c_int, c_void_p)
_sig("mg_wait_mailbox", c_int, c_void_p, c_int)
_sig("mg_swap_hidden_buffer", c_int, c_void_p)
_sig("mg_hidden_idx", c_int, c_void_p)
_sig("mg_decode_token", c_int, c_void_p, c_int, c_int, _i, _f)
_sig("mg_generate", c_int, c_void_p, _i, c_int, c_int, _i, c_int)
_sig("mg_graph_capture", c_int, c_void_p)
_sig("mg_graph_launch", c_int, c_void_p, c_int, c_int, _i)
_sig("mg_graph_validate", c_int, c_void_p, c_int, c_int, _f)
_sig("mg_layer_graph_capture", c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int)
_sig("mg_layer_graph_launch", c_int, c_void_p, c_int)
_sig("mg_layer_graph_update_and_launch", c_int, c_void_p, c_int)
_sig("mg_layer_graph_destroy", None, c_void_p)
_sig("mg_upload_hidden", c_int, c_void_p, _f)
_sig("mg_read_hidden", c_int, c_void_p, _f)
_sig("mg_validate_graph_capture", c_int, c_void_p, _f, c_int, c_int, _f)
_sig("mg_has_graph_kernel", c_int)
_sig("mg_timed_decode", c_int, c_void_p, c_int, c_int, c_int, c_int, _f)
_sig("mg_profile_decode", c_int, c_void_p, c_int, c_int, c_int, ctypes.c_uint, _f, _i)
_sig("mg_prefill", c_int, c_void_p, _i, c_int, c_int, _i, _f, _f)
_sig("mg_generate_prefill", c_int, c_void_p, _i, c_int, c_int, _i)
_sig("mg_bench_matvec", c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, _f)
_sig("mg_flow_exchange", c_int, c_void_p, c_int, _f, c_size_t, _i)
_sig("mg_flow_in_use", c_int, c_void_p)
_sig("mg_flow_tail_in_use", c_int, c_void_p)
_sig("mg_set_flow_tail", c_int, c_void_p, c_int)
_sig("mg_set_flow_generic", c_int, c_void_p, c_int)
_sig("mg_set_tokens_per_launch", c_int, c_void_p, c_int)
_sig("mg_tokens_per_launch", c_int, c_void_p)
_sig("mg_flow_tail_trace", c_int, c_void_p, ctypes.POINTER(ctypes.c_longlong), c_size_t, _i)
_sig("mg_flow_set_wait_limit", c_int, c_void_p, ctypes.c_longlong)
_sig("mg_flow_trace", c_int, c_void_p, c_int, ctypes.POINTER(ctypes.c_longlong), c_size_t, _i)
_sig("mg_weight_bytes_per_token", c_uint64, c_void_p)
_sig("mg_kv_bytes_at", c_uint64, c_void_p, c_int)
_sig("mg_stream_build", c_void_p, c_void_p)
_sig("mg_stream_destroy", None, c_void_p)
_sig("mg_stream_forward_token", c_int, c_void_p, c_int, _f, c_int, POINTER(c_void_p), POINTER(c_int32), _f)

# host helpers
_sig("mg_quantize_q8", None, _f, c_int, c_int, c_int, POINTER(c_int8), _f)
_sig("mg_quantize_q4_0", None, _f, c_int, c_int, POINTER(c_uint8))
_sig("mg_f32_to_f16", c_uint16, c_float)
_sig("mg_f16_to_f32", c_float, c_uint16)
_sig("mg_synth_normal", None, c_uint64, c_uint64, c_float, _f, c_size_t)
_sig("mg_synth_tokens", None, c_uint64, c_uint64, c_int, _i, c_size_t)


def last_error():
    return lib.mg_last_error().decode()
