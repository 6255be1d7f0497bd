"""Python face of the C++ host layer (include/llama3_host.h): the same calls a
C++ caller of the reference makes -- init_llama3, load_safetensor_weights /
seeded_fill_model, to_cuda, init_cache, inference -- plus the KV-cached
prefill / decode / generate extensions."""
import ctypes as C

import numpy as np

from . import capi
from .capi import GenStats, ModelConfig, lib

LAYER_SLOTS = ("input_layernorm", "mlp_down_proj", "mlp_gate_proj", "mlp_up_proj",
               "post_attention_layernorm", "self_attn_k_proj", "self_attn_o_proj",
               "self_attn_q_proj", "self_attn_v_proj")


def config(name="tiny", **over):
    c = lib().llama3_config_8b() if name == "8b" else lib().llama3_config_tiny()
    for k, v in over.items():
        setattr(c, k, v)
    return c


def seeded_normal_bf16(seed, tensor_id, n, sigma=0.02):
    out = np.empty(n, np.uint16)
    lib().seeded_normal_bf16(seed, tensor_id, n, sigma, out.ctypes.data)
    return out


def seeded_tokens(seed, n, vocab):
    out = np.empty(n, np.int32)
    lib().seeded_tokens(seed, n, vocab, out.ctypes.data)
    return out


def _host_tensor(t):
    """bf16 payload of a host Tensor as a numpy view (before to_cuda frees it)."""
    t = t.contents
    n = t.mem_len[0]
    shape = tuple(t.shape[i] for i in range(t.ndim[0]))
    return np.ctypeslib.as_array(t.bf16_tensor, shape=(n,)).reshape(shape)


class Model:
    """init_llama3 + weights on the host; to_device() moves and converts them."""

    def __init__(self, cfg):
        self.cfg = cfg
        self.handle = lib().init_llama3(cfg.n_layers)
        self.on_device = False

    @classmethod
    def seeded(cls, cfg, seed):
        m = cls(cfg)
        lib().seeded_fill_model(m.handle, C.byref(cfg), seed)
        return m

    @classmethod
    def from_files(cls, cfg, paths):
        m = cls(cfg)
        for p in paths:
            lib().load_safetensor_weights(m.handle, p.encode())
        return m

    @classmethod
    def from_files_streaming(cls, cfg, paths):
        """Headers first, then every tensor through pinned staging buffers straight to the device."""
        capi.require_gpu()
        m = cls(cfg)
        arr = (C.c_char_p * len(paths))(*[p.encode() for p in paths])
        lib().load_safetensor_weights_streaming(m.handle, arr, len(paths))
        m.on_device = True
        return m

    def host_bf16(self):
        """dict of numpy views on the host bf16 payloads (valid until to_device)."""
        assert not self.on_device
        h = self.handle.contents
        out = {"embed": _host_tensor(h.embed_tokens), "lm_head": _host_tensor(h.lm_head),
               "norm": _host_tensor(h.norm)}
        for s in LAYER_SLOTS:
            out[s] = [_host_tensor(getattr(h.layers[l].contents, s)) for l in range(self.cfg.n_layers)]
        return out

    def to_device(self):
        capi.require_gpu()
        lib().to_cuda(self.handle)
        self.on_device = True
        return self

    def device_fp16(self, tensor_ptr):
        t = tensor_ptr.contents
        n = t.mem_len[0]
        out = np.empty(n, np.uint16)
        capi.check(lib().llm_memcpy_d2h(out.ctypes.data, t.d_fp16_tensor, n * 2, None))
        return out.reshape(tuple(t.shape[i] for i in range(t.ndim[0])))

    def close(self):
        if self.handle:
            lib().free_llama3(self.handle)
            self.handle = None


class Engine:
    """init_cache_cfg + the token loop."""

    def __init__(self, model, cfg=None, use_graph=True):
        assert model.on_device
        self.model = model
        self.cfg = cfg or model.cfg
        self.cache = lib().init_cache_cfg(model.handle, C.byref(self.cfg))
        lib().llama3_set_use_graph(self.cache, 1 if use_graph else 0)

    def reset(self):
        lib().llama3_cache_reset(self.cache)

    @property
    def pos(self):
        return lib().llama3_cache_pos(self.cache)

    def _trace(self, n):
        buf = np.empty((self.cfg.n_layers, n, self.cfg.d_model), np.uint16)
        lib().llama3_set_hidden_trace(self.cache, buf.ctypes.data)
        return buf

    def prefill(self, tokens, want_hidden=False, inject=None):
        """inject: [n_layers, n, d] uint16 hidden states; layer l >= 1 starts from inject[l-1]."""
        tokens = np.ascontiguousarray(tokens, dtype=np.int32)
        hidden = self._trace(tokens.size) if want_hidden else None
        if inject is not None:
            inject = np.ascontiguousarray(inject, dtype=np.uint16)
            assert inject.shape == (self.cfg.n_layers, tokens.size, self.cfg.d_model)
            lib().llama3_set_hidden_inject(self.cache, inject.ctypes.data)
        tok = lib().llama3_prefill(self.model.handle, self.cache,
                                   tokens.ctypes.data_as(C.POINTER(C.c_int)), tokens.size)
        return tok, hidden

    def decode(self, token, want_hidden=False, inject=None):
        hidden = self._trace(1) if want_hidden else None
        if inject is not None:
            inject = np.ascontiguousarray(inject, dtype=np.uint16)
            assert inject.shape == (self.cfg.n_layers, 1, self.cfg.d_model)
            lib().llama3_set_hidden_inject(self.cache, inject.ctypes.data)
        tok = lib().llama3_decode(self.model.handle, self.cache, int(token))
        return tok, hidden

    def logits(self):
        out = np.empty(self.cfg.vocab, np.uint16)
        lib().llama3_read_logits(self.cache, out.ctypes.data)
        return out

    def generate(self, prompt, n_decode):
        prompt = np.ascontiguousarray(prompt, dtype=np.int32)
        out = np.empty(n_decode, np.int32)
        st = GenStats()
        lib().llama3_generate(self.model.handle, self.cache, prompt.ctypes.data_as(C.POINTER(C.c_int)),
                              prompt.size, n_decode, out.ctypes.data_as(C.POINTER(C.c_int)), C.byref(st))
        return out, st

    def inference(self, tokens, d_tokens=None):
        """The reference's call: tokens[0] = n + 1, ids in tokens[1..n].  d_tokens: the device int
        array of tokens_to_cuda (a capi.DevBuf of at least 2048 int32), or None."""
        n = len(tokens)
        arr = np.zeros(2049, np.int32)
        arr[0] = n + 1
        arr[1:n + 1] = tokens
        dt = C.cast(d_tokens.ptr, C.POINTER(C.c_int)) if d_tokens is not None else None
        return lib().inference(self.model.handle, None, dt, arr.ctypes.data_as(C.POINTER(C.c_int)), self.cache)

    def host_logits(self):
        """CudaCache.h_token_probdist: the fp16 logits inference() left on the host."""
        return np.ctypeslib.as_array(self.cache.contents.h_token_probdist, shape=(self.cfg.vocab,)).copy()

    def sampler_config(self, temperature, top_k, top_p):
        lib().llama3_cache_sampler_config(self.cache, temperature, top_k, top_p)

    @staticmethod
    def decode_batch(engines, tokens):
        """One step for several sequences (one Engine each, same model and configuration); returns the greedy ids."""
        B = len(engines)
        caches = (capi.HOST_ABI["init_cache"][0] * B)(*[e.cache for e in engines])
        tok = (C.c_int * B)(*[int(t) for t in tokens])
        out = (C.c_int * B)()
        lib().llama3_decode_batch(engines[0].model.handle, caches, tok, B, out)
        return [int(x) for x in out]

    def batch_logits(self, b):
        out = np.empty(self.cfg.vocab, np.uint16)
        lib().llama3_read_batch_logits(self.cache, b, out.ctypes.data)
        return out

    def set_handover(self, on, spin_limit=-1):
        """Attention + output projection of a decode step in one launch (on) or one launch per operation."""
        lib().llama3_set_handover(self.cache, 1 if on else 0, spin_limit)

    def handover_stats(self):
        """(waits that gave up, steps redone, hand-over launches in use)"""
        t, r, a = C.c_long(0), C.c_long(0), C.c_int(0)
        lib().llama3_handover_stats(self.cache, C.byref(t), C.byref(r), C.byref(a))
        return t.value, r.value, bool(a.value)

    def mark_handover_timeout(self):
        lib().llama3_test_mark_handover_timeout(self.cache)

    def set_device_sampling(self, on):
        lib().llama3_set_device_sampling(self.cache, 1 if on else 0)

    def sampler_draw_counts(self):
        """(draws decided from device-selected candidates, draws made by the host path)"""
        d, h = C.c_long(0), C.c_long(0)
        lib().llama3_sampler_draw_counts(self.cache, C.byref(d), C.byref(h))
        return d.value, h.value

    def sample_device_logits(self, logits):
        """The cache's sampler on fp16 logits given as a host array (uploaded) or a DevBuf."""
        buf = logits if isinstance(logits, capi.DevBuf) else capi.DevBuf.from_host(
            np.ascontiguousarray(logits, dtype=np.uint16))
        return lib().llama3_sample_device_logits(self.cache, buf.ptr)

    def set_sampling(self, on):
        """inference() returns the reference's temperature/top-k/top-p sample (True) or the argmax (False)."""
        lib().llama3_set_sampling(self.cache, 1 if on else 0)

    def close(self):
        if self.cache:
            lib().free_cache(self.cache)
            self.cache = None
