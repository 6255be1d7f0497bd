"""ctypes binding of the CPU oracle (oracle/oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py.  The product never imports this module.

All tensors are numpy uint16 arrays holding fp16 (or bf16) bit patterns.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

ORC_REF16 = 0
ORC_FP32 = 1
ORC_REF16_REV = 2


class OrcConfig(C.Structure):
    _fields_ = [
        ("n_layers", C.c_int),
        ("d_model", C.c_int),
        ("n_heads", C.c_int),
        ("n_kv_heads", C.c_int),
        ("head_dim", C.c_int),
        ("ffn_dim", C.c_int),
        ("vocab", C.c_int),
        ("max_pos", C.c_int),
        ("rms_eps", C.c_double),
        ("rope_theta", C.c_float),
    ]


_PP = C.POINTER(C.c_void_p)


class OrcWeights(C.Structure):
    _fields_ = [
        ("embed", C.c_void_p),
        ("lm_head", C.c_void_p),
        ("norm", C.c_void_p),
        ("input_ln", _PP),
        ("post_ln", _PP),
        ("wq", _PP),
        ("wk", _PP),
        ("wv", _PP),
        ("wo", _PP),
        ("wgate", _PP),
        ("wup", _PP),
        ("wdown", _PP),
    ]


def build(force=False):
    """Compile liboracle.so with gcc (building the checker is not using it)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "liboracle.so"])
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_LIB_PATH)
        vp, i32, sz = C.c_void_p, C.c_int, C.c_size_t
        L.orc_f32_to_f16_soft.restype = C.c_uint16
        L.orc_f32_to_f16_soft.argtypes = [C.c_float]
        L.orc_f32_to_f16.restype = C.c_uint16
        L.orc_f32_to_f16.argtypes = [C.c_float]
        L.orc_f16_to_f32_soft.restype = C.c_float
        L.orc_f16_to_f32_soft.argtypes = [C.c_uint16]
        L.orc_f16_to_f32.restype = C.c_float
        L.orc_f16_to_f32.argtypes = [C.c_uint16]
        L.orc_bf16_to_fp16.argtypes = [vp, vp, sz]
        L.orc_embed.argtypes = [vp, vp, i32, i32, vp]
        L.orc_rmsnorm.argtypes = [vp, vp, i32, i32, C.c_double, vp]
        L.orc_rmsnorm.restype = i32
        L.orc_add.argtypes = [vp, vp, sz]
        L.orc_linear.argtypes = [vp, vp, i32, i32, i32, vp]
        L.orc_linear_swiglu.argtypes = [vp, vp, vp, i32, i32, i32, vp]
        L.orc_rope.argtypes = [vp, i32, i32, i32, i32, C.c_float]
        L.orc_attention.argtypes = [vp, vp, vp, i32, i32, i32, i32, i32, vp]
        L.orc_attention_materialized.argtypes = [vp, vp, vp, i32, i32, i32, i32, vp]
        L.orc_argmax_f16.argtypes = [vp, i32]
        L.orc_argmax_f16.restype = i32
        L.orc_model_new.argtypes = [C.POINTER(OrcConfig), C.POINTER(OrcWeights), i32]
        L.orc_model_new.restype = vp
        L.orc_model_free.argtypes = [vp]
        L.orc_model_reset.argtypes = [vp]
        L.orc_model_pos.argtypes = [vp]
        L.orc_model_pos.restype = i32
        L.orc_model_forward.argtypes = [vp, vp, i32, vp, vp]
        L.orc_model_forward.restype = i32
        L.orc_model_forward_recompute.argtypes = [C.POINTER(OrcConfig), C.POINTER(OrcWeights), vp,
                                                  i32, vp, vp]
        L.orc_model_forward_recompute.restype = i32
        L.orc_num_threads.restype = i32
        L.orc_rand_seed.argtypes = [vp, C.c_uint]
        L.orc_rand_next.argtypes = [vp]
        L.orc_rand_next.restype = i32
        L.orc_sample.argtypes = [vp, i32, C.c_float, i32, C.c_float, vp]
        L.orc_sample.restype = i32
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def _u16(a):
    a = np.ascontiguousarray(a)
    assert a.dtype == np.uint16, a.dtype
    return a


# ---- helpers between numpy float16 and bit patterns -------------------
def f16_bits(a):
    return np.ascontiguousarray(np.asarray(a, dtype=np.float16)).view(np.uint16)


def bits_f16(a):
    return np.ascontiguousarray(a).view(np.float16)


# ---- single ops ---------------------------------------------------------
def bf16_to_fp16(src):
    src = _u16(src)
    dst = np.empty_like(src)
    lib().orc_bf16_to_fp16(_p(src), _p(dst), src.size)
    return dst


def embed(table, ids):
    table = _u16(table)
    ids = np.ascontiguousarray(ids, dtype=np.int32)
    out = np.empty((ids.size, table.shape[1]), np.uint16)
    lib().orc_embed(_p(table), _p(ids), ids.size, table.shape[1], _p(out))
    return out


def rmsnorm(x, gain, eps=1e-5):
    x = _u16(x)
    gain = _u16(gain)
    T, d = x.shape
    out = np.empty_like(x)
    rc = lib().orc_rmsnorm(_p(x), _p(gain), T, d, eps, _p(out))
    if rc != 0:
        raise ValueError("orc_rmsnorm: d/4 must be a power of two")
    return out


def add(x, res):
    x = _u16(x).copy()
    res = _u16(res)
    lib().orc_add(_p(x), _p(res), x.size)
    return x


def linear(x, w):
    x = _u16(x)
    w = _u16(w)
    T, K = x.shape
    N = w.shape[0]
    assert w.shape[1] == K
    out = np.empty((T, N), np.uint16)
    lib().orc_linear(_p(x), _p(w), T, N, K, _p(out))
    return out


def linear_swiglu(x, wgate, wup):
    x = _u16(x)
    wgate = _u16(wgate)
    wup = _u16(wup)
    T, K = x.shape
    N = wgate.shape[0]
    out = np.empty((T, N), np.uint16)
    lib().orc_linear_swiglu(_p(x), _p(wgate), _p(wup), T, N, K, _p(out))
    return out


def rope(buf, n_heads, head_dim, pos0=0, theta=500000.0):
    buf = _u16(buf).copy()
    T = buf.shape[0]
    assert buf.size == T * n_heads * head_dim
    lib().orc_rope(_p(buf), T, n_heads, head_dim, pos0, theta)
    return buf


def attention(q, k, v, pos0, n_heads, n_kv_heads, head_dim):
    q, k, v = _u16(q), _u16(k), _u16(v)
    Tq = q.shape[0]
    assert k.shape[0] >= pos0 + Tq
    out = np.empty_like(q)
    lib().orc_attention(_p(q), _p(k), _p(v), Tq, pos0, n_heads, n_kv_heads, head_dim, _p(out))
    return out


def attention_materialized(q, k, v, n_heads, n_kv_heads, head_dim):
    q, k, v = _u16(q), _u16(k), _u16(v)
    out = np.empty_like(q)
    lib().orc_attention_materialized(_p(q), _p(k), _p(v), q.shape[0], n_heads, n_kv_heads,
                                     head_dim, _p(out))
    return out


def argmax_f16(logits):
    logits = _u16(logits)
    return lib().orc_argmax_f16(_p(logits), logits.size)


# ---- whole model ----------------------------------------------------------
_LAYER_KEYS = ("input_ln", "post_ln", "wq", "wk", "wv", "wo", "wgate", "wup", "wdown")


def _pack_weights(weights, n_layers):
    """weights: dict with 'embed','lm_head','norm' (uint16 arrays of fp16 bits)
    and per-layer lists under _LAYER_KEYS.  Returns (OrcWeights, keepalive)."""
    keep = []
    W = OrcWeights()
    for k in ("embed", "lm_head", "norm"):
        a = _u16(weights[k])
        keep.append(a)
        setattr(W, k, a.ctypes.data)
    for k in _LAYER_KEYS:
        arrs = [_u16(a) for a in weights[k]]
        assert len(arrs) == n_layers
        ptrs = (C.c_void_p * n_layers)(*[a.ctypes.data for a in arrs])
        keep.extend(arrs)
        keep.append(ptrs)
        setattr(W, k, C.cast(ptrs, _PP))
    return W, keep


def make_config(cfg):
    return OrcConfig(cfg["n_layers"], cfg["d_model"], cfg["n_heads"], cfg["n_kv_heads"],
                     cfg["head_dim"], cfg["ffn_dim"], cfg["vocab"], cfg["max_pos"],
                     cfg.get("rms_eps", 1e-5), cfg.get("rope_theta", 500000.0))


class Model:
    """KV-cached oracle model.  forward(tokens) appends tokens and returns
    (next_token, hidden [L, n, d] uint16 or None, logits [vocab] uint16)."""

    def __init__(self, cfg, weights, mode=ORC_REF16):
        self.cfg = dict(cfg)
        self._c = make_config(cfg)
        self._w, self._keep = _pack_weights(weights, cfg["n_layers"])
        self._h = lib().orc_model_new(C.byref(self._c), C.byref(self._w), mode)

    def close(self):
        if self._h:
            lib().orc_model_free(self._h)
            self._h = None

    def __del__(self):
        self.close()

    def reset(self):
        lib().orc_model_reset(self._h)

    @property
    def pos(self):
        return lib().orc_model_pos(self._h)

    def forward(self, tokens, want_hidden=False):
        tokens = np.ascontiguousarray(tokens, dtype=np.int32)
        n = tokens.size
        hidden = (np.empty((self.cfg["n_layers"], n, self.cfg["d_model"]), np.uint16)
                  if want_hidden else None)
        logits = np.empty(self.cfg["vocab"], np.uint16)
        tok = lib().orc_model_forward(self._h, _p(tokens), n, _p(hidden), _p(logits))
        if tok < 0:
            raise ValueError("orc_model_forward: position overflow")
        return tok, hidden, logits

    def generate(self, prompt, n_decode):
        out = []
        tok, _, _ = self.forward(prompt)
        out.append(tok)
        for _ in range(n_decode - 1):
            tok, _, _ = self.forward([tok])
            out.append(tok)
        return out


def forward_recompute(cfg, weights, tokens, want_hidden=False):
    c = make_config(cfg)
    W, keep = _pack_weights(weights, cfg["n_layers"])
    tokens = np.ascontiguousarray(tokens, dtype=np.int32)
    T = tokens.size
    hidden = np.empty((cfg["n_layers"], T, cfg["d_model"]), np.uint16) if want_hidden else None
    logits = np.empty(cfg["vocab"], np.uint16)
    tok = lib().orc_model_forward_recompute(C.byref(c), C.byref(W), _p(tokens), T, _p(hidden),
                                            _p(logits))
    del keep
    return tok, hidden, logits


def weights_from_bf16(h):
    """fp16 weight dict for Model() from the host bf16 payloads of a not-yet-uploaded model (the dict
    llm.cu_amd's engine.Model.host_bf16() returns): the oracle's own BF16->FP16 over the same bits the GPU
    will convert."""
    conv = lambda a: bf16_to_fp16(np.ascontiguousarray(a).reshape(-1)).reshape(a.shape)
    return {
        "embed": conv(h["embed"]), "lm_head": conv(h["lm_head"]), "norm": conv(h["norm"]),
        "input_ln": [conv(a) for a in h["input_layernorm"]],
        "post_ln": [conv(a) for a in h["post_attention_layernorm"]],
        "wq": [conv(a) for a in h["self_attn_q_proj"]],
        "wk": [conv(a) for a in h["self_attn_k_proj"]],
        "wv": [conv(a) for a in h["self_attn_v_proj"]],
        "wo": [conv(a) for a in h["self_attn_o_proj"]],
        "wgate": [conv(a) for a in h["mlp_gate_proj"]],
        "wup": [conv(a) for a in h["mlp_up_proj"]],
        "wdown": [conv(a) for a in h["mlp_down_proj"]],
    }


def num_threads():
    return lib().orc_num_threads()


class Rand:
    """The oracle's private copy of glibc rand() (state seeded like srand(seed))."""

    def __init__(self, seed=1):
        self._s = (C.c_int32 * 36)()
        lib().orc_rand_seed(self._s, seed)

    def next(self):
        return lib().orc_rand_next(self._s)


def sample(logits, rng, temperature=0.7, top_k=50, top_p=0.9):
    logits = _u16(logits)
    return lib().orc_sample(_p(logits), logits.size, temperature, top_k, top_p, rng._s)
