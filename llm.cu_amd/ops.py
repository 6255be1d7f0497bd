"""numpy-in / numpy-out wrappers of the kernel entry points (one C-ABI call
each).  Arrays are uint16 fp16/bf16 bit patterns unless noted.  Used by the
parity tests and the micro-benchmarks; the token loop itself lives in the C++
host layer (engine.py binds it)."""
import ctypes as C

import numpy as np

from . import capi
from .capi import DevBuf, check, lib


def _u16(a):
    a = np.ascontiguousarray(a)
    if a.dtype == np.float16:
        a = a.view(np.uint16)
    assert a.dtype == np.uint16, a.dtype
    return a


def bf16_to_fp16(src):
    src = _u16(src)
    d_src, d_dst = DevBuf.from_host(src), DevBuf(src.shape, np.uint16)
    check(lib().llm_bf16_to_fp16(d_src.ptr, d_dst.ptr, src.size, None))
    return d_dst.download()


def embed_gather(table, ids):
    table = _u16(table)
    ids = np.ascontiguousarray(ids, dtype=np.int32)
    vocab, d = table.shape
    d_t, d_i, d_o = DevBuf.from_host(table), DevBuf.from_host(ids), DevBuf((ids.size, d), np.uint16)
    check(lib().llm_embed_gather(d_t.ptr, d_i.ptr, None, d_o.ptr, ids.size, d, vocab, None))
    return d_o.download()


def rmsnorm(x, gain, eps=1e-5, inplace=False):
    x, gain = _u16(x), _u16(gain)
    T, d = x.shape
    d_x, d_g = DevBuf.from_host(x), DevBuf.from_host(gain)
    d_y = d_x if inplace else DevBuf(x.shape, np.uint16)
    check(lib().llm_rmsnorm(d_x.ptr, d_g.ptr, d_y.ptr, T, d, eps, None))
    return d_y.download()


def add_residual(x, res):
    x, res = _u16(x), _u16(res)
    d_x, d_r = DevBuf.from_host(x), DevBuf.from_host(res)
    check(lib().llm_add_residual(d_x.ptr, d_r.ptr, x.size, None))
    return d_x.download()


def rope_table(max_pos, head_dim, theta=500000.0):
    tab = np.empty((max_pos, head_dim // 2, 2), np.float32)
    check(lib().llm_rope_table_host(tab.ctypes.data, max_pos, head_dim, theta))
    return tab


def rope(buf, n_heads, head_dim, pos0=0, theta=500000.0, max_pos=None):
    buf = _u16(buf)
    T = buf.shape[0]
    stride = buf.size // T
    max_pos = max_pos or (pos0 + T + 63) // 64 * 64
    d_b = DevBuf.from_host(buf)
    d_t = DevBuf.from_host(rope_table(max_pos, head_dim, theta))
    check(lib().llm_rope(d_b.ptr, T, n_heads, head_dim, stride, pos0, None, d_t.ptr, max_pos, None))
    return d_b.download()


def linear(x, w, residual=None, ldo=None, inplace=False):
    """ldo: row stride of the output buffer in elements (default N); the columns beyond N are not returned.
    inplace: the residual buffer is also the output buffer, as in the engine (x += projection)."""
    x, w = _u16(x), _u16(w)
    T, K = x.shape
    N = w.shape[0]
    ldo = N if ldo is None else ldo
    d_x, d_w = DevBuf.from_host(x), DevBuf.from_host(w)
    if inplace:
        assert residual is not None and ldo == N
        d_o = d_r = DevBuf.from_host(_u16(residual))
    else:
        d_o = DevBuf((T, ldo), np.uint16)
        d_r = DevBuf.from_host(_u16(residual)) if residual is not None else None
    check(lib().llm_linear(d_x.ptr, K, d_w.ptr, d_r.ptr if d_r else None, N, d_o.ptr, ldo, T, N, K, None))
    return np.ascontiguousarray(d_o.download()[:, :N])


def linear_swiglu(x, wgate, wup, ldo=None):
    x, wgate, wup = _u16(x), _u16(wgate), _u16(wup)
    T, K = x.shape
    N = wgate.shape[0]
    ldo = N if ldo is None else ldo
    d_x, d_g, d_u = DevBuf.from_host(x), DevBuf.from_host(wgate), DevBuf.from_host(wup)
    d_o = DevBuf((T, ldo), np.uint16)
    check(lib().llm_linear_swiglu(d_x.ptr, K, d_g.ptr, d_u.ptr, d_o.ptr, ldo, T, N, K, None))
    return np.ascontiguousarray(d_o.download()[:, :N])


def kv_layout(k, v, n_kv_heads, head_dim, max_pos):
    """token-major k, v [P, Hkv*hd] -> cache layouts K [Hkv][max_pos][hd], V [Hkv][hd][max_pos]."""
    k, v = _u16(k), _u16(v)
    P = k.shape[0]
    kc = np.zeros((n_kv_heads, max_pos, head_dim), np.uint16)
    vc = np.zeros((n_kv_heads, head_dim, max_pos), np.uint16)
    kc[:, :P, :] = k.reshape(P, n_kv_heads, head_dim).transpose(1, 0, 2)
    vc[:, :, :P] = v.reshape(P, n_kv_heads, head_dim).transpose(1, 2, 0)
    return kc, vc


def rope_kv_append(qkv, n_heads, n_kv_heads, head_dim, pos0, max_pos, theta=500000.0, kc=None, vc=None):
    """Returns (qkv after the in-place Q rotation, K cache, V cache)."""
    qkv = _u16(qkv)
    T = qkv.shape[0]
    kc = np.zeros((n_kv_heads, max_pos, head_dim), np.uint16) if kc is None else _u16(kc)
    vc = np.zeros((n_kv_heads, head_dim, max_pos), np.uint16) if vc is None else _u16(vc)
    d_q, d_k, d_v = DevBuf.from_host(qkv), DevBuf.from_host(kc), DevBuf.from_host(vc)
    d_t = DevBuf.from_host(rope_table(max_pos, head_dim, theta))
    check(lib().llm_rope_kv_append(d_q.ptr, d_k.ptr, d_v.ptr, T, n_heads, n_kv_heads, head_dim, pos0, None,
                                   d_t.ptr, max_pos, None))
    return d_q.download(), d_k.download(), d_v.download()


def rope_k_append_attn_prefill(qkv, n_heads, n_kv_heads, head_dim, pos0, max_pos, theta=500000.0, kc=None, vc=None):
    """The prompt pass's attention step with the queries rotated inside the attention kernel: K rotated into the
    cache, V stored, then llm_attn_prefill_rope_q on the queries as they are.  Returns (out [T, Hq*hd], qkv
    afterwards, K cache, V cache)."""
    qkv = _u16(qkv)
    T = qkv.shape[0]
    kc = np.zeros((n_kv_heads, max_pos, head_dim), np.uint16) if kc is None else _u16(kc)
    vc = np.zeros((n_kv_heads, head_dim, max_pos), np.uint16) if vc is None else _u16(vc)
    d_q, d_k, d_v = DevBuf.from_host(qkv), DevBuf.from_host(kc), DevBuf.from_host(vc)
    d_t = DevBuf.from_host(rope_table(max_pos, head_dim, theta))
    d_o = DevBuf((T, n_heads * head_dim), np.uint16)
    check(lib().llm_rope_k_append(d_q.ptr, d_k.ptr, d_v.ptr, T, n_heads, n_kv_heads, head_dim, pos0, d_t.ptr, max_pos, None))
    check(lib().llm_attn_prefill_rope_q(d_q.ptr, qkv.shape[1], d_k.ptr, d_v.ptr, d_o.ptr, n_heads * head_dim, T, pos0, d_t.ptr,
                                        n_heads, n_kv_heads, head_dim, max_pos, None))
    return d_o.download(), d_q.download(), d_k.download(), d_v.download()


def attn_decode(q, kc, vc, ctx, n_heads, n_kv_heads, head_dim, repeats=1):
    q, kc, vc = _u16(q), _u16(kc), _u16(vc)
    max_pos = kc.shape[1]
    d_q, d_k, d_v = DevBuf.from_host(q), DevBuf.from_host(kc), DevBuf.from_host(vc)
    d_o = DevBuf((n_heads * head_dim,), np.uint16)
    wsb = (lib().llm_attn_decode_workspace_bytes(n_heads, head_dim) + 3) // 4 * 4
    d_ws = DevBuf((wsb // 4,), np.uint32)
    d_ws.zero()
    for _ in range(repeats):  # the workspace is reusable without clearing
        check(lib().llm_attn_decode(d_q.ptr, d_k.ptr, d_v.ptr, d_o.ptr, ctx, None, n_heads, n_kv_heads, head_dim,
                                    max_pos, d_ws.ptr, None))
    return d_o.download()


def attn_decode_noalloc(q, kc, vc, ctx, n_heads, n_kv_heads, head_dim):
    """llm_attn_decode_noalloc: the library's built-in scratch instead of a workspace argument."""
    q, kc, vc = _u16(q), _u16(kc), _u16(vc)
    max_pos = kc.shape[1]
    d_q, d_k, d_v = DevBuf.from_host(q), DevBuf.from_host(kc), DevBuf.from_host(vc)
    d_o = DevBuf((n_heads * head_dim,), np.uint16)
    check(lib().llm_attn_decode_noalloc(d_q.ptr, d_k.ptr, d_v.ptr, d_o.ptr, ctx, None, n_heads, n_kv_heads,
                                        head_dim, max_pos, None))
    return d_o.download()


def sample_candidates(logits, exp_table, k):
    """llm_sample_candidates.  Returns (denominator float32, flag, ranges added one by one,
    probabilities float32[n], indices int32[n]) with n = k, or 0 when the flag is set."""
    logits = _u16(logits).reshape(-1)
    table = np.ascontiguousarray(exp_table, dtype=np.float32)
    assert table.size == 65536
    d_l, d_t = DevBuf.from_host(logits), DevBuf.from_host(table)
    d_o = DevBuf((lib().llm_sample_candidates_bytes(logits.size, k) // 4,), np.uint32)
    check(lib().llm_sample_candidates(d_l.ptr, d_t.ptr, logits.size, k, d_o.ptr, None))
    o = d_o.download()
    n = int(o[1])
    pairs = o[4:4 + 2 * n].reshape(n, 2)
    return (o[0:1].view(np.float32)[0], int(o[2]), int(o[3]), pairs[:, 0].copy().view(np.float32),
            pairs[:, 1].copy().view(np.int32))


def attn_prefill(q, kc, vc, pos0, n_heads, n_kv_heads, head_dim):
    q, kc, vc = _u16(q), _u16(kc), _u16(vc)
    T = q.shape[0]
    ldq = q.size // T
    max_pos = kc.shape[1]
    d_q, d_k, d_v = DevBuf.from_host(q), DevBuf.from_host(kc), DevBuf.from_host(vc)
    d_o = DevBuf((T, n_heads * head_dim), np.uint16)
    check(lib().llm_attn_prefill(d_q.ptr, ldq, d_k.ptr, d_v.ptr, d_o.ptr, n_heads * head_dim, T, pos0, n_heads,
                                 n_kv_heads, head_dim, max_pos, None))
    return d_o.download()


def lmhead_argmax(x, w):
    """Returns (token, logits uint16[vocab])."""
    x, w = _u16(x).reshape(-1), _u16(w)
    vocab, K = w.shape
    d_x, d_w = DevBuf.from_host(x), DevBuf.from_host(w)
    d_l, d_t = DevBuf((vocab,), np.uint16), DevBuf((1,), np.int32)
    d_ws = DevBuf((lib().llm_lmhead_workspace_bytes(vocab),), np.uint8)
    check(lib().llm_lmhead_argmax(d_x.ptr, d_w.ptr, d_l.ptr, d_t.ptr, None, None, vocab, K, d_ws.ptr, None))
    return int(d_t.download()[0]), d_l.download()


def argmax_f16(logits):
    logits = _u16(logits).reshape(-1)
    d_l, d_t = DevBuf.from_host(logits), DevBuf((1,), np.int32)
    d_ws = DevBuf((lib().llm_lmhead_workspace_bytes(logits.size),), np.uint8)
    check(lib().llm_argmax_f16(d_l.ptr, logits.size, d_t.ptr, d_ws.ptr, None))
    return int(d_t.download()[0])


def argmax_f16_rows(logits):
    """argmax of every row of a 2-D fp16 array in one call."""
    logits = _u16(logits)
    rows, n = logits.shape
    d_l, d_t = DevBuf.from_host(logits), DevBuf((rows,), np.int32)
    d_ws = DevBuf((rows * min(1024, (n + 255) // 256) * 8,), np.uint8)
    check(lib().llm_argmax_f16_rows(d_l.ptr, n, rows, n, d_t.ptr, d_ws.ptr, None))
    return d_t.download()


class Timer:
    """HIP-event timing of repeated launches on one stream."""

    def __init__(self):
        capi.require_gpu()
        self.stream = C.c_void_p()
        check(lib().llm_stream_create(C.byref(self.stream)))
        self.e0, self.e1 = C.c_void_p(), C.c_void_p()
        check(lib().llm_event_create(C.byref(self.e0)))
        check(lib().llm_event_create(C.byref(self.e1)))

    def time(self, fn, iters=20, warmup=3):
        """fn(stream) issues the launches; returns mean milliseconds per call."""
        for _ in range(warmup):
            fn(self.stream)
        check(lib().llm_stream_sync(self.stream))
        check(lib().llm_event_record(self.e0, self.stream))
        for _ in range(iters):
            fn(self.stream)
        check(lib().llm_event_record(self.e1, self.stream))
        check(lib().llm_event_sync(self.e1))
        ms = C.c_float(0)
        check(lib().llm_event_elapsed_ms(self.e0, self.e1, C.byref(ms)))
        return ms.value / iters


def norm_linear(x, gain, w, eps=1e-5):
    x, gain, w = _u16(x).reshape(-1), _u16(gain), _u16(w)
    N, K = w.shape
    d_x, d_g, d_w, d_o = DevBuf.from_host(x), DevBuf.from_host(gain), DevBuf.from_host(w), DevBuf((1, N), np.uint16)
    check(lib().llm_norm_linear(d_x.ptr, d_g.ptr, eps, d_w.ptr, d_o.ptr, N, K, None))
    return d_o.download()


def embed_norm_linear(table, ids, offset, gain, w, eps=1e-5):
    """Returns (out [1, N], the gathered row [K]) for the id at ids[offset] (offset None: ids[0])."""
    table, gain, w = _u16(table), _u16(gain), _u16(w)
    vocab, K = table.shape
    N = w.shape[0]
    d_t, d_g, d_w = DevBuf.from_host(table), DevBuf.from_host(gain), DevBuf.from_host(w)
    d_ids = DevBuf.from_host(np.ascontiguousarray(ids, dtype=np.int32))
    d_off = DevBuf.from_host(np.array([offset], dtype=np.int32)) if offset is not None else None
    d_x, d_o = DevBuf((K,), np.uint16), DevBuf((1, N), np.uint16)
    check(lib().llm_embed_norm_linear(d_t.ptr, d_ids.ptr, d_off.ptr if d_off else None, vocab, d_x.ptr, d_g.ptr, eps,
                                      d_w.ptr, d_o.ptr, N, K, None))
    return d_o.download(), d_x.download()


def norm_linear_swiglu(x, gain, wgate, wup, eps=1e-5):
    x, gain, wgate, wup = _u16(x).reshape(-1), _u16(gain), _u16(wgate), _u16(wup)
    N, K = wgate.shape
    d_x, d_g = DevBuf.from_host(x), DevBuf.from_host(gain)
    d_a, d_b, d_o = DevBuf.from_host(wgate), DevBuf.from_host(wup), DevBuf((1, N), np.uint16)
    check(lib().llm_norm_linear_swiglu(d_x.ptr, d_g.ptr, eps, d_a.ptr, d_b.ptr, d_o.ptr, N, K, None))
    return d_o.download()


def norm_lmhead_argmax(x, gain, w, eps=1e-5):
    x, gain, w = _u16(x).reshape(-1), _u16(gain), _u16(w)
    vocab, K = w.shape
    d_x, d_g, d_w = DevBuf.from_host(x), DevBuf.from_host(gain), DevBuf.from_host(w)
    d_l, d_t = DevBuf((vocab,), np.uint16), DevBuf((1,), np.int32)
    d_ws = DevBuf((lib().llm_lmhead_workspace_bytes(vocab),), np.uint8)
    check(lib().llm_norm_lmhead_argmax(d_x.ptr, d_g.ptr, eps, d_w.ptr, d_l.ptr, d_t.ptr, None, None, vocab, K,
                                       d_ws.ptr, None))
    return int(d_t.download()[0]), d_l.download()


def attn_decode_rope(qkv, kc, vc, pos, n_heads, n_kv_heads, head_dim, theta=500000.0, repeats=1, long_form=False):
    """Returns (out [Hq*hd], K cache, V cache) after rope + append + attention at position pos;
    long_form selects the two-launch span/merge kernels."""
    qkv, kc, vc = _u16(qkv).reshape(-1), _u16(kc), _u16(vc)
    max_pos = kc.shape[1]
    d_q, d_k, d_v = DevBuf.from_host(qkv), DevBuf.from_host(kc), DevBuf.from_host(vc)
    d_o = DevBuf((n_heads * head_dim,), np.uint16)
    d_t = DevBuf.from_host(rope_table(max_pos, head_dim, theta))
    wsb = (lib().llm_attn_decode_workspace_bytes(n_heads, head_dim) + 3) // 4 * 4
    d_ws = DevBuf((wsb // 4,), np.uint32)
    d_ws.zero()
    for _ in range(repeats):
        fn = lib().llm_attn_decode_rope_long if long_form else lib().llm_attn_decode_rope
        check(fn(d_q.ptr, d_k.ptr, d_v.ptr, d_o.ptr, pos, None, d_t.ptr, n_heads, n_kv_heads,
                 head_dim, max_pos, d_ws.ptr, None))
    return d_o.download(), d_k.download(), d_v.download()


def attn_decode_rope_oproj(qkv, kc, vc, pos, n_heads, n_kv_heads, head_dim, w, residual=None, theta=500000.0, repeats=1,
                           long_form=False, spin_limit=-1):
    """llm_attn_decode_rope_oproj (long_form: llm_attn_decode_rope_long_oproj): returns (attention output [Hq*hd],
    projection output [N], K cache, V cache, timeouts).  Each repeat starts from the same caches and uses the next
    buffer of a two-buffer ring.  spin_limit >= 0 shortens the projection workgroups' bounded wait (the repeats are
    then not compared with one another: a wait that gave up leaves an invalid projection, which the count reports)."""
    qkv, kc, vc, w = _u16(qkv).reshape(-1), _u16(kc), _u16(vc), _u16(w)
    max_pos = kc.shape[1]
    N = w.shape[0]
    qd = n_heads * head_dim
    d_q, d_t = DevBuf.from_host(qkv), DevBuf.from_host(rope_table(max_pos, head_dim, theta))
    d_w = DevBuf.from_host(w)
    ring = DevBuf((2, qd), np.uint16)
    check(lib().llm_attn_oproj_buffer_init(ring.ptr, 2 * qd, None))
    tmo = DevBuf((1,), np.int32)
    tmo.zero()
    wsb = (lib().llm_attn_decode_workspace_bytes(n_heads, head_dim) + 3) // 4 * 4
    d_ws = DevBuf((wsb // 4,), np.uint32)
    d_ws.zero()
    res = None
    for r in range(repeats):
        d_k, d_v = DevBuf.from_host(kc), DevBuf.from_host(vc)
        d_o = DevBuf.from_host(_u16(residual).reshape(-1)) if residual is not None else DevBuf((N,), np.uint16)
        cur, nxt = ring.ptr + 2 * qd * (r % 2), ring.ptr + 2 * qd * ((r + 1) % 2)
        if long_form:
            check(lib().llm_attn_decode_rope_long_oproj(d_q.ptr, d_k.ptr, d_v.ptr, cur, nxt, pos, None, d_t.ptr, n_heads,
                                                        n_kv_heads, head_dim, max_pos, d_ws.ptr, d_w.ptr,
                                                        d_o.ptr if residual is not None else None, d_o.ptr, N, tmo.ptr,
                                                        spin_limit, None))
        else:
            check(lib().llm_attn_decode_rope_oproj(d_q.ptr, d_k.ptr, d_v.ptr, cur, nxt, pos, None, d_t.ptr, n_heads, n_kv_heads,
                                                   head_dim, max_pos, d_w.ptr, d_o.ptr if residual is not None else None,
                                                   d_o.ptr, N, tmo.ptr, spin_limit, None))
        out = (ring.download()[r % 2].copy(), d_o.download(), d_k.download(), d_v.download())
        assert spin_limit >= 0 or res is None or all(np.array_equal(x, y) for x, y in zip(res, out)), "repeat %d differs" % r
        res = out
    return res + (int(tmo.download()[0]),)
