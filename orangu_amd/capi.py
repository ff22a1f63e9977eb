"""ctypes declarations of ``include/orangu_mi355x.h``.

Loads the in-tree ``liborangu_mi355x.so``.  There is no fallback: if the library is missing or a
call fails, an exception is raised.
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "liborangu_mi355x.so")

OGM_OK = 0
STATUS = {0: "OGM_OK", -1: "OGM_ERR_INVALID", -2: "OGM_ERR_UNSUPPORTED", -3: "OGM_ERR_NO_DEVICE",
          -4: "OGM_ERR_HIP", -5: "OGM_ERR_OOM"}

# every symbol the header declares
SYMBOLS = [
    "ogm_init", "ogm_destroy", "ogm_last_error", "ogm_device_name", "ogm_supports_type",
    "ogm_supports", "ogm_block_layout", "ogm_repacked_size", "ogm_repack_host",
    "ogm_unrepack_host", "ogm_weight_upload", "ogm_weight_download", "ogm_weight_free",
    "ogm_weight_info", "ogm_matmul", "ogm_matmul_decode", "ogm_matmul_batch", "ogm_matmul_dev",
    "ogm_quantize_act", "ogm_dump_block_sums", "ogm_f16_to_f32", "ogm_set_tuning",
    "ogm_last_kernel", "ogm_act_quantize_dev", "ogm_matmul_act_dev", "ogm_matmul_multi_dev", "ogm_matmul_multi_act_dev",
    "ogm_llama_create", "ogm_llama_destroy", "ogm_llama_kv_write", "ogm_llama_kv_read", "ogm_llama_decode", "ogm_llama_decode_dev",
    "ogm_llama_debug_hidden", "ogm_dequant_rows", "ogm_llama_generate", "ogm_llama_load_gguf", "ogm_llama_prefill", "ogm_llama_prefill_tokens", "ogm_llama_hidden_states",
    "ogm_gguf_open", "ogm_gguf_parse", "ogm_gguf_close", "ogm_gguf_last_error", "ogm_gguf_info",
    "ogm_gguf_meta_u64", "ogm_gguf_meta_f64", "ogm_gguf_meta_string", "ogm_gguf_meta_array",
    "ogm_gguf_find_tensor", "ogm_gguf_tensor", "ogm_gguf_tensor_data", "ogm_gguf_matrix",
    "ogm_gguf_upload_matrix", "ogm_argmax", "ogm_matmul_dev_static", "ogm_quantize_act_tokens", "ogm_llama_debug_capture", "ogm_llama_debug_act", "ogm_debug_attn_stamps", "ogm_llama_forward_all_logits",
    "ogm_weights_read_probe", "ogm_time_host_calls", "ogm_empty_launch", "ogm_scratch_bytes", "ogm_act_quantize_decode_dev", "ogm_enqueue_repeated",
]


class OgmError(RuntimeError):
    def __init__(self, status: int, where: str, detail: str = ""):
        self.status = status
        super().__init__(f"{where}: {STATUS.get(status, status)}" + (f" ({detail})" if detail else ""))


class OgmLlamaConfig(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("n_layer", "n_embd", "n_head", "n_head_kv", "head_dim", "n_ff",
                                          "n_vocab", "rope_dim", "max_ctx")] + \
               [("rms_eps", C.c_float), ("rope_freq_base", C.c_float), ("rope_neox", C.c_uint32),
                ("rope_freq_factors", C.c_void_p)]


class OgmLlamaLayer(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in ("wq", "wk", "wv", "wo", "w_gate", "w_up", "w_down",
                                          "attn_norm", "ffn_norm", "q_bias", "k_bias", "v_bias",
                                          "q_norm", "k_norm")]


class OgmOp(C.Structure):
    _fields_ = [("w", C.c_void_p), ("x", C.c_void_p), ("n_tokens", C.c_uint32), ("y", C.c_void_p)]


_lib = None


def load_library() -> C.CDLL:
    """Loads the built library, building nothing.  Raises if it is absent."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise OgmError(-3, "load_library", f"{LIB_PATH} is not built; run __graft_entry__.build()")
    L = C.CDLL(LIB_PATH)
    vp, sz, u32, u64 = C.c_void_p, C.c_size_t, C.c_uint32, C.c_uint64
    L.ogm_init.argtypes = [C.c_int, C.POINTER(vp)]
    L.ogm_destroy.argtypes = [vp]
    L.ogm_destroy.restype = None
    L.ogm_last_error.argtypes = [vp]
    L.ogm_last_error.restype = C.c_char_p
    L.ogm_device_name.argtypes = [vp, C.c_char_p, sz]
    L.ogm_supports_type.argtypes = [u32]
    L.ogm_supports.argtypes = [u32, u32]
    L.ogm_block_layout.argtypes = [u32, C.POINTER(u32), C.POINTER(u32)]
    L.ogm_repacked_size.argtypes = [u32, u32, u32]
    L.ogm_repacked_size.restype = sz
    L.ogm_repack_host.argtypes = [u32, vp, sz, u32, u32, vp]
    L.ogm_unrepack_host.argtypes = [u32, vp, sz, u32, u32, vp]
    L.ogm_weight_upload.argtypes = [vp, u32, vp, sz, u32, u32, u64, u64, C.POINTER(vp)]
    L.ogm_weight_download.argtypes = [vp, vp, vp, sz]
    L.ogm_weight_free.argtypes = [vp, vp]
    L.ogm_weight_info.argtypes = [vp, C.POINTER(u32), C.POINTER(u32), C.POINTER(u32), C.POINTER(sz)]
    L.ogm_matmul.argtypes = [vp, vp, vp, u32, vp]
    L.ogm_matmul_decode.argtypes = [vp, vp, vp, u32, vp]
    L.ogm_matmul_batch.argtypes = [vp, C.POINTER(OgmOp), sz, C.c_int, u32]
    L.ogm_matmul_dev.argtypes = [vp, vp, vp, u32, vp, C.c_int, vp]
    L.ogm_matmul_dev_static.argtypes = [vp, vp, vp, u32, vp, C.c_int, vp]
    L.ogm_act_quantize_dev.argtypes = [vp, u32, vp, u32, u32, vp]
    L.ogm_act_quantize_decode_dev.argtypes = [vp, u32, vp, u32, u32, vp]
    L.ogm_matmul_act_dev.argtypes = [vp, vp, u32, vp, C.c_int, vp]
    L.ogm_matmul_multi_dev.argtypes = [vp, C.POINTER(vp), sz, vp, u32, C.POINTER(vp), C.c_int, vp]
    L.ogm_matmul_multi_act_dev.argtypes = [vp, C.POINTER(vp), sz, u32, C.POINTER(vp), C.c_int, vp]
    L.ogm_weights_read_probe.argtypes = [vp, C.POINTER(vp), sz, vp]
    L.ogm_empty_launch.argtypes = [vp, u32, vp]
    L.ogm_scratch_bytes.argtypes = [vp]
    L.ogm_scratch_bytes.restype = sz
    L.ogm_enqueue_repeated.argtypes = [vp, C.c_int, C.POINTER(vp), sz, sz, u32, C.POINTER(vp), C.c_int, u32, u32, vp]
    L.ogm_time_host_calls.argtypes = [vp, C.POINTER(OgmOp), sz, sz, C.POINTER(u32), sz, u32, C.POINTER(C.c_double)]
    L.ogm_llama_create.argtypes = [vp, C.POINTER(OgmLlamaConfig), C.POINTER(OgmLlamaLayer), vp, vp, C.POINTER(vp)]
    L.ogm_llama_destroy.argtypes = [vp, vp]
    L.ogm_llama_destroy.restype = None
    L.ogm_llama_kv_write.argtypes = [vp, vp, u32, u32, u32, vp, vp]
    L.ogm_llama_kv_read.argtypes = [vp, vp, u32, u32, u32, vp, vp]
    L.ogm_llama_prefill.argtypes = [vp, vp, vp, u32, u32, vp, vp]
    L.ogm_llama_prefill_tokens.argtypes = [vp, vp, vp, vp, u32, u32, vp, vp]
    L.ogm_llama_hidden_states.argtypes = [vp, vp, vp, vp, vp, u32, vp]
    L.ogm_llama_load_gguf.argtypes = [vp, vp, u32, C.POINTER(vp), C.POINTER(vp), C.POINTER(OgmLlamaConfig)]
    L.ogm_llama_decode.argtypes = [vp, vp, vp, u32, vp, vp]
    L.ogm_llama_decode_dev.argtypes = [vp, vp, vp, u32, vp, vp, vp]
    L.ogm_llama_debug_hidden.argtypes = [vp, vp, vp]
    L.ogm_dequant_rows.argtypes = [vp, vp, u32, u32, vp]
    L.ogm_llama_generate.argtypes = [vp, vp, vp, u32, u32, u32, vp, vp]
    L.ogm_gguf_open.argtypes = [C.c_char_p, u64, C.POINTER(vp), C.c_char_p, sz]
    L.ogm_gguf_parse.argtypes = [vp, sz, C.POINTER(vp), C.c_char_p, sz]
    L.ogm_gguf_close.argtypes = [vp]
    L.ogm_gguf_close.restype = None
    L.ogm_gguf_last_error.argtypes = [vp]
    L.ogm_gguf_last_error.restype = C.c_char_p
    L.ogm_gguf_info.argtypes = [vp, C.POINTER(u32), C.POINTER(u64), C.POINTER(u64), C.POINTER(u64), C.POINTER(u64)]
    L.ogm_gguf_meta_u64.argtypes = [vp, C.c_char_p, C.POINTER(u64)]
    L.ogm_gguf_meta_f64.argtypes = [vp, C.c_char_p, C.POINTER(C.c_double)]
    L.ogm_gguf_meta_string.argtypes = [vp, C.c_char_p, C.POINTER(C.c_char_p), C.POINTER(sz)]
    L.ogm_gguf_meta_array.argtypes = [vp, C.c_char_p, C.POINTER(u32), C.POINTER(u64)]
    L.ogm_gguf_find_tensor.argtypes = [vp, C.c_char_p]
    L.ogm_gguf_find_tensor.restype = C.c_int64
    L.ogm_gguf_tensor.argtypes = [vp, u64, C.POINTER(C.c_char_p), C.POINTER(u32), C.POINTER(u64), C.POINTER(u32),
                                  C.POINTER(u64)]
    L.ogm_gguf_tensor_data.argtypes = [vp, u64, C.POINTER(vp), C.POINTER(u64)]
    L.ogm_gguf_matrix.argtypes = [vp, C.c_char_p, C.POINTER(u32), C.POINTER(u32), C.POINTER(u32), C.POINTER(sz),
                                  C.POINTER(vp)]
    L.ogm_gguf_upload_matrix.argtypes = [vp, vp, C.c_char_p, C.POINTER(vp)]
    L.ogm_quantize_act.argtypes = [vp, C.c_int, vp, sz, vp, vp, vp]
    L.ogm_dump_block_sums.argtypes = [vp, vp, vp, u32, vp, vp]
    L.ogm_f16_to_f32.argtypes = [vp, vp, sz, vp]
    L.ogm_argmax.argtypes = [vp, vp, u32, C.POINTER(u32)]
    L.ogm_quantize_act_tokens.argtypes = [vp, C.c_int, vp, u32, u32, vp, vp, vp, vp, vp]
    L.ogm_llama_debug_capture.argtypes = [vp, vp, C.c_int]
    L.ogm_llama_debug_act.argtypes = [vp, vp, u32, vp, vp, C.POINTER(u32), C.POINTER(u32)]
    L.ogm_debug_attn_stamps.argtypes = [vp, vp, sz]
    L.ogm_llama_forward_all_logits.argtypes = [vp, vp, vp, vp, vp, u32, u32, vp, vp]
    L.ogm_set_tuning.argtypes = [vp, C.c_char_p, C.c_int]
    L.ogm_last_kernel.argtypes = [vp]
    L.ogm_last_kernel.restype = C.c_char_p
    _lib = L
    return L
