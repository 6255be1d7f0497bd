"""ctypes bindings of libllmcu.so: the HIP C-ABI (include/llmcu_hip.h) and the
reference-shaped host layer (include/llama3_host.h).

There is no CPU fallback: every function here needs the built library, and the
kernel entry points need an MI355X.  A missing library raises ImportError-like
RuntimeError at load time with the build command.
"""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libllmcu.so")

LLM_OK, LLM_ERR_INVALID, LLM_ERR_HIP, LLM_ERR_NO_DEVICE = 0, 1, 2, 3


class LlmError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("llmcu error %d: %s" % (code, msg))
        self.code = code


class ModelConfig(C.Structure):
    _fields_ = [
        ("n_layers", C.c_int), ("d_model", C.c_int), ("n_heads", C.c_int), ("n_kv_heads", C.c_int),
        ("head_dim", C.c_int), ("ffn_dim", C.c_int), ("vocab", C.c_int), ("max_pos", C.c_int),
        ("rms_eps", C.c_double), ("rope_theta", C.c_float),
    ]

    def as_dict(self):
        return {k: getattr(self, k) for k, _ in self._fields_}


class Tensor(C.Structure):
    _fields_ = [
        ("ndim", C.POINTER(C.c_int)), ("mem_len", C.POINTER(C.c_int)), ("shape", C.POINTER(C.c_int)),
        ("bf16_tensor", C.POINTER(C.c_uint16)),
        ("d_ndim", C.c_void_p), ("d_mem_len", C.c_void_p), ("d_shape", C.c_void_p),
        ("d_bf16_tensor", C.c_void_p), ("d_fp16_tensor", C.c_void_p),
    ]


_TP = C.POINTER(Tensor)


class Llama3Layer(C.Structure):
    _fields_ = [
        ("layernum", C.c_int),
        ("input_layernorm", _TP), ("mlp_down_proj", _TP), ("mlp_gate_proj", _TP), ("mlp_up_proj", _TP),
        ("post_attention_layernorm", _TP), ("self_attn_k_proj", _TP), ("self_attn_o_proj", _TP),
        ("self_attn_q_proj", _TP), ("self_attn_v_proj", _TP),
    ]


class Llama3(C.Structure):
    _fields_ = [
        ("embed_tokens", _TP), ("lm_head", _TP), ("norm", _TP),
        ("layers", C.POINTER(C.POINTER(Llama3Layer))), ("n_layers", C.c_int), ("device_slab", C.c_void_p),
    ]


class CudaCache(C.Structure):
    _fields_ = [
        ("PN_X", _TP), ("Q", _TP), ("K", _TP), ("V", _TP),
        ("d_attention_score_cache", C.c_void_p), ("d_feedforward_cache_upgate", C.c_void_p),
        ("d_token_probdist", C.c_void_p), ("h_token_probdist", C.POINTER(C.c_uint16)),
        ("f_token_probdist", C.POINTER(C.c_float)), ("engine", C.c_void_p),
    ]


class GenStats(C.Structure):
    _fields_ = [("prefill_ms", C.c_double), ("decode_ms", C.c_double), ("n_prompt", C.c_int),
                ("n_decode_steps", C.c_int)]


# name -> (restype, argtypes); every symbol declared in include/*.h
_vp, _i, _sz, _u64 = C.c_void_p, C.c_int, C.c_size_t, C.c_uint64
HIP_ABI = {
    "llm_last_error": (C.c_char_p, []),
    "llm_device_count": (_i, [C.POINTER(_i)]),
    "llm_init": (_i, [_i]),
    "llm_device_name": (_i, [C.c_char_p, _sz]),
    "llm_device_cu_count": (_i, [C.POINTER(_i)]),
    "llm_malloc": (_i, [C.POINTER(_vp), _sz]),
    "llm_free": (_i, [_vp]),
    "llm_mem_info": (_i, [C.POINTER(_sz), C.POINTER(_sz)]),
    "llm_malloc_host": (_i, [C.POINTER(_vp), _sz]),
    "llm_free_host": (_i, [_vp]),
    "llm_memcpy_h2d": (_i, [_vp, _vp, _sz, _vp]),
    "llm_memcpy_d2h": (_i, [_vp, _vp, _sz, _vp]),
    "llm_memcpy_d2d": (_i, [_vp, _vp, _sz, _vp]),
    "llm_fill_zero": (_i, [_vp, _sz, _vp]),
    "llm_stream_create": (_i, [C.POINTER(_vp)]),
    "llm_stream_destroy": (_i, [_vp]),
    "llm_stream_sync": (_i, [_vp]),
    "llm_device_sync": (_i, []),
    "llm_event_create": (_i, [C.POINTER(_vp)]),
    "llm_event_destroy": (_i, [_vp]),
    "llm_event_record": (_i, [_vp, _vp]),
    "llm_event_sync": (_i, [_vp]),
    "llm_event_elapsed_ms": (_i, [_vp, _vp, C.POINTER(C.c_float)]),
    "llm_graph_capture_begin": (_i, [_vp]),
    "llm_graph_capture_end": (_i, [_vp, C.POINTER(_vp)]),
    "llm_graph_launch": (_i, [_vp, _vp]),
    "llm_graph_destroy": (_i, [_vp]),
    "llm_bf16_to_fp16": (_i, [_vp, _vp, _sz, _vp]),
    "llm_embed_gather": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "llm_rmsnorm": (_i, [_vp, _vp, _vp, _i, _i, C.c_double, _vp]),
    "llm_add_residual": (_i, [_vp, _vp, _sz, _vp]),
    "llm_rope_table_host": (_i, [_vp, _i, _i, C.c_float]),
    "llm_rope": (_i, [_vp, _i, _i, _i, _i, _i, _vp, _vp, _i, _vp]),
    "llm_rope_kv_append": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _vp, _vp, _i, _vp]),
    "llm_rope_k_append": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _vp, _i, _vp]),
    "llm_linear": (_i, [_vp, _i, _vp, _vp, _i, _vp, _i, _i, _i, _i, _vp]),
    "llm_linear_unsplit_fallbacks": (C.c_long, []),
    "llm_linear_swiglu": (_i, [_vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "llm_norm_linear": (_i, [_vp, _vp, C.c_double, _vp, _vp, _i, _i, _vp]),
    "llm_norm_linear_swiglu": (_i, [_vp, _vp, C.c_double, _vp, _vp, _vp, _i, _i, _vp]),
    "llm_embed_norm_linear": (_i, [_vp, _vp, _vp, _i, _vp, _vp, C.c_double, _vp, _vp, _i, _i, _vp]),
    "llm_attn_decode_rope": (_i, [_vp, _vp, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _i, _vp, _vp]),
    "llm_attn_decode_rope_batch": (_i, [_vp, _i, _vp, _vp, _vp, _i, _vp, _i, _vp, _i, _i, _i, _i, _vp, _vp]),
    "llm_attn_decode_rope_batch_dev": (_i, [_vp, _i, _vp, _sz, _i, _i, _vp, _i, _vp, _i, _i, _i, _i, _vp, _vp]),
    "llm_attn_oproj_supported": (_i, [_i, _i, _i, _i]),
    "llm_attn_oproj_buffer_init": (_i, [_vp, _i, _vp]),
    "llm_attn_decode_rope_oproj": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _i, _vp, _vp, _vp, _i, _vp, _i, _vp]),
    "llm_sample_candidates_bytes": (_sz, [_i, _i]),
    "llm_sample_candidates_head_bytes": (_sz, [_i]),
    "llm_sample_candidates_max_vocab": (_i, []),
    "llm_sample_candidates": (_i, [_vp, _vp, _i, _i, _vp, _vp]),
    "llm_attn_decode_rope_long": (_i, [_vp, _vp, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _i, _vp, _vp]),
    "llm_attn_long_oproj_supported": (_i, [_i, _i, _i, _i]),
    "llm_attn_decode_rope_long_oproj": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _i, _vp, _i, _vp]),
    "llm_norm_lmhead_argmax": (_i, [_vp, _vp, C.c_double, _vp, _vp, _vp, _vp, _vp, _i, _i, _vp, _vp]),
    "llm_attn_decode_workspace_bytes": (_sz, [_i, _i]),
    "llm_attn_decode": (_i, [_vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _i, _vp, _vp]),
    "llm_attn_decode_noalloc_max_bytes": (_sz, []),
    "llm_attn_decode_noalloc": (_i, [_vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _i, _vp]),
    "llm_attn_prefill": (_i, [_vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "llm_attn_prefill_rope_q_supported": (_i, [_i, _i, _i, _i, _i]),
    "llm_attn_prefill_rope_q": (_i, [_vp, _i, _vp, _vp, _vp, _i, _i, _i, _vp, _i, _i, _i, _i, _vp]),
    "llm_lmhead_workspace_bytes": (_sz, [_i]),
    "llm_lmhead_argmax": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _vp, _vp]),
    "llm_argmax_f16": (_i, [_vp, _i, _vp, _vp, _vp]),
    "llm_argmax_f16_rows": (_i, [_vp, _i, _i, _i, _vp, _vp, _vp]),
}
_LP, _CP = C.POINTER(Llama3), C.POINTER(CudaCache)
HOST_ABI = {
    "init_llama3": (_LP, [_i]),
    "free_llama3": (None, [_LP]),
    "_free_tensor": (None, [_TP]),
    "load_safetensor_weights": (None, [_LP, C.c_char_p]),
    "to_cuda": (None, [_LP]),
    "load_safetensor_weights_streaming": (None, [_LP, C.POINTER(C.c_char_p), _i]),
    "init_cache": (_CP, [_LP]),
    "tokens_to_cuda": (C.POINTER(_i), [C.POINTER(_i), _i, _TP]),
    "inference": (_i, [_LP, _TP, C.POINTER(_i), C.POINTER(_i), _CP]),
    "llama3_config_8b": (ModelConfig, []),
    "llama3_config_tiny": (ModelConfig, []),
    "init_cache_cfg": (_CP, [_LP, C.POINTER(ModelConfig)]),
    "free_cache": (None, [_CP]),
    "llama3_prefill": (_i, [_LP, _CP, C.POINTER(_i), _i]),
    "llama3_decode": (_i, [_LP, _CP, _i]),
    "llama3_cache_reset": (None, [_CP]),
    "llama3_cache_pos": (_i, [_CP]),
    "llama3_decode_batch": (None, [_LP, C.POINTER(_CP), C.POINTER(_i), _i, C.POINTER(_i)]),
    "llama3_read_batch_logits": (None, [_CP, _i, _vp]),
    "llama3_generate": (_i, [_LP, _CP, C.POINTER(_i), _i, _i, C.POINTER(_i), C.POINTER(GenStats)]),
    "llama3_set_hidden_trace": (None, [_CP, _vp]),
    "llama3_read_logits": (None, [_CP, _vp]),
    "llama3_set_hidden_inject": (None, [_CP, _vp]),
    "llama3_set_use_graph": (None, [_CP, _i]),
    "llama3_set_handover": (None, [_CP, _i, _i]),
    "llama3_handover_stats": (None, [_CP, C.POINTER(C.c_long), C.POINTER(C.c_long), C.POINTER(_i)]),
    "llama3_test_mark_handover_timeout": (None, [_CP]),
    "llama3_set_error_handler": (None, [_vp]),
    "seeded_normal_bf16": (None, [_u64, _u64, _sz, C.c_float, _vp]),
    "seeded_tokens": (None, [_u64, _i, _i, _vp]),
    "seeded_unit_table_bf16": (C.POINTER(C.c_uint16), [C.c_float]),
    "seeded_fill_model": (None, [_LP, C.POINTER(ModelConfig), _u64]),
    "seeded_write_safetensors": (_i, [C.POINTER(ModelConfig), _u64, C.c_char_p]),
    "seeded_tensor_id": (_u64, [_i, _i]),
    "load_tokenizer": (_vp, []),
    "load_tokenizer_from": (_vp, [C.c_char_p, _i]),
    "free_tokenizer": (None, [_vp, _i]),
    "tokenize": (C.POINTER(_i), [_vp, C.c_char_p]),
    "read_tokenizer_json": (_vp, [_vp, C.c_char_p]),
    "_get_file_size": (C.c_long, [C.c_char_p]),
    "init_trienode": (_vp, []),
    "_build_trie": (None, [_vp, C.c_char_p, _i]),
    "_find_child": (_i, [_vp, C.c_char, C.POINTER(_vp)]),
    "_memexpand_child_nodes": (None, [_vp]),
    "_build_decoder": (None, [_vp, C.c_char_p, _i]),
    "llama3_chat_prompt": (_vp, [C.c_char_p]),
    "sample_next_token": (_i, [_vp, _vp]),
    "sample_next_token_reference": (_i, [_vp, _vp]),
    "temperature_softmax": (_vp, [_vp, _vp, C.c_float]),
    "_compare_desc": (_i, [_vp, _vp]),
    "top_k_sampling": (_i, [_vp, _i]),
    "top_p_sampling": (_i, [_vp, C.c_float]),
    "llama3_sampler_config": (None, [_i, C.c_float, _i, C.c_float]),
    "llama3_set_sampling": (None, [_CP, _i]),
    "llama3_set_device_sampling": (None, [_CP, _i]),
    "llama3_sampler_draw_counts": (None, [_CP, C.POINTER(C.c_long), C.POINTER(C.c_long)]),
    "llama3_sample_device_logits": (_i, [_CP, _vp]),
    "llama3_cache_sampler_config": (None, [_CP, C.c_float, _i, C.c_float]),
    "llama3_sample_with": (_i, [_i, C.c_float, _i, C.c_float, _vp, _vp]),
}

_lib = None


def lib():
    """Loads libllmcu.so (never builds it: build with `python llm.cu_amd/build.py`)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("%s is missing: run `python llm.cu_amd/build.py` (hipcc, gfx950); "
                               "there is no CPU fallback" % LIB_PATH)
        L = C.CDLL(LIB_PATH, mode=C.RTLD_GLOBAL)
        for table in (HIP_ABI, HOST_ABI):
            for name, (res, args) in table.items():
                fn = getattr(L, name)  # AttributeError if the symbol is not exported
                fn.restype = res
                fn.argtypes = args
        _lib = L
    return _lib


def check(code):
    if code != LLM_OK:
        raise LlmError(code, lib().llm_last_error().decode("utf-8", "replace"))


def device_count():
    n = C.c_int(0)
    lib().llm_device_count(C.byref(n))
    return n.value


_inited = False


def init(device=0):
    global _inited
    check(lib().llm_init(device))
    _inited = True


def require_gpu():
    if not _inited:
        init(0)


# ---- device memory as numpy-facing buffers -----------------------------------
class DevBuf:
    """A device allocation with a numpy dtype/shape attached."""

    def __init__(self, shape, dtype):
        require_gpu()
        self.shape = tuple(int(s) for s in (shape if isinstance(shape, (tuple, list)) else (shape,)))
        self.dtype = np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize
        p = C.c_void_p()
        check(lib().llm_malloc(C.byref(p), self.nbytes))
        self.ptr = p.value

    @classmethod
    def from_host(cls, a):
        a = np.ascontiguousarray(a)
        b = cls(a.shape, a.dtype)
        b.upload(a)
        return b

    def upload(self, a):
        a = np.ascontiguousarray(a, dtype=self.dtype)
        assert a.nbytes == self.nbytes, (a.shape, self.shape)
        check(lib().llm_memcpy_h2d(self.ptr, a.ctypes.data, self.nbytes, None))

    def download(self):
        out = np.empty(self.shape, self.dtype)
        check(lib().llm_memcpy_d2h(out.ctypes.data, self.ptr, self.nbytes, None))
        return out

    def zero(self):
        check(lib().llm_fill_zero(self.ptr, self.nbytes, None))
        check(lib().llm_device_sync())

    def free(self):
        if self.ptr:
            lib().llm_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def sync():
    check(lib().llm_device_sync())
