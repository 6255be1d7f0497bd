"""The reference's host sampler (src/inference/inference.cu:1030-1161): the oracle's restatement is pinned
against libc (its private rand() stream), against an independent float32 numpy derivation of the
two-pass rule, and by the rule's own invariants; the shipped sampler (same names as the reference) is then
compared with the oracle draw for draw.  CPU only."""
import ctypes as C

import numpy as np

from oracle import pyoracle as orc
from tests import helpers as H


def _logits(rng, vocab, scale=3.0):
    return H.bits(scale * rng.standard_normal(vocab))


def test_private_rand_stream_is_glibc_rand():
    libc = C.CDLL("libc.so.6")
    libc.rand.restype = C.c_int
    for seed in (1, 2, 12345):
        libc.srand(seed)
        r = orc.Rand(seed)
        assert [r.next() for _ in range(2000)] == [libc.rand() for _ in range(2000)]
    libc.srand(1)


def _numpy_rule(logits_bits, draws, temperature=0.7, top_k=50, top_p=0.9):
    """Independent derivation, vectorised float32: sort, renormalise the head k, cut the nucleus on the
    renormalised head, draw with the SECOND number (the first belongs to the discarded top-k pick)."""
    f = np.float32
    e = np.exp((H.f16(logits_bits).astype(f) / f(temperature))).astype(f)
    total = f(0)
    for v in e:  # the reference's running float sum, in index order
        total = f(total + v)
    p = (e / total).astype(f)
    order = np.argsort(-p, kind="stable")
    head = p[order[:top_k]]
    s = f(0)
    for v in head:
        s = f(s + v)
    head = (head / s).astype(f)
    c = f(0)
    cut = len(head) - 1
    for i, v in enumerate(head):
        c = f(c + v)
        if c >= f(top_p):
            cut = i
            break
    nuc = (head[:cut + 1] / c).astype(f)
    r = f(f(draws[1]) / f(2147483647.0))
    c = f(0)
    for i, v in enumerate(nuc):
        c = f(c + v)
        if r < c:
            return int(order[i])
    return int(order[0])


def test_oracle_sampler_matches_independent_numpy_rule():
    rng = np.random.default_rng(0)
    for case in range(40):
        vocab = int(rng.integers(60, 700))
        lg = _logits(rng, vocab)
        # distinct probabilities only: qsort's order among equal keys is not part of the rule
        if len(np.unique(H.f16(lg))) != vocab:
            lg = H.bits(np.sort(rng.standard_normal(vocab) * 3)[rng.permutation(vocab)] + np.arange(vocab) * 1e-2)
            if len(np.unique(H.f16(lg))) != vocab:
                continue
        seed = 100 + case
        probe = orc.Rand(seed)
        draws = [probe.next(), probe.next()]
        got = orc.sample(lg, orc.Rand(seed))
        assert got == _numpy_rule(lg, draws), case


def test_sampler_invariants():
    rng = np.random.default_rng(1)
    vocab = 5000
    lg = _logits(rng, vocab)
    order = np.argsort(-H.f16(lg).astype(np.float64), kind="stable")
    r = orc.Rand(7)
    picks = [orc.sample(lg, r) for _ in range(300)]
    assert set(picks) <= set(order[:50].tolist())          # never outside the top-k head
    assert len(set(picks)) > 1                              # and not degenerate
    # a dominant logit is always chosen; so is the argmax when the nucleus is a single entry
    spike = lg.copy()
    spike[1234] = H.bits(np.array([40.0]))[0]
    assert all(orc.sample(spike, r) == 1234 for _ in range(20))
    assert all(orc.sample(lg, r, top_p=1e-6) == int(order[0]) for _ in range(20))
    # two draws per call: the stream position after n calls is 2n
    a, b = orc.Rand(3), orc.Rand(3)
    for _ in range(5):
        orc.sample(lg, a)
    for _ in range(10):
        b.next()
    assert a.next() == b.next()
    # low temperature sharpens towards the argmax, high temperature spreads
    cold = [orc.sample(lg, r, temperature=0.25) for _ in range(100)]
    warm = [orc.sample(lg, r, temperature=2.0) for _ in range(100)]
    assert cold.count(int(order[0])) > warm.count(int(order[0])) + 20
    # the reference does not subtract the maximum: exp overflows for logit/temperature > 88.7, every
    # probability becomes NaN or 0, no comparison succeeds and the pick degenerates to the first entry
    hot = H.bits(np.linspace(-5, 12, vocab))
    assert len({orc.sample(hot, r, temperature=0.05) for _ in range(10)}) == 1


def test_shipped_sampler_equals_oracle_draw_for_draw(pkg):
    lib = pkg.lib()
    libc = C.CDLL("libc.so.6")
    rng = np.random.default_rng(2)
    for vocab, n in ((4096, 40), (128256, 4)):
        lib.llama3_sampler_config(vocab, 0.7, 50, 0.9)
        libc.srand(1)  # the reference never seeds: the stream of srand(1)
        r = orc.Rand(1)
        scratch = np.empty(vocab, np.float32)
        for _ in range(n):
            lg = _logits(rng, vocab, scale=2.0)
            got = lib.sample_next_token(scratch.ctypes.data, lg.ctypes.data)
            assert got == orc.sample(lg, r)
            assert abs(float(scratch.sum()) - 1.0) < 1e-3  # tensor[] holds the normalised probabilities
    # other settings, including the branches that fall back to a uniform pick
    lib.llama3_sampler_config(4096, 1.3, 0, 0.5)
    libc.srand(9)
    r = orc.Rand(9)
    scratch = np.empty(4096, np.float32)
    for _ in range(10):
        lg = _logits(rng, 4096)
        assert lib.sample_next_token(scratch.ctypes.data, lg.ctypes.data) == orc.sample(lg, r, 1.3, 0, 0.5)
    lib.llama3_sampler_config(4096, 0.7, 50, 0.0)
    libc.srand(9)
    r = orc.Rand(9)
    for _ in range(10):
        lg = _logits(rng, 4096)
        assert lib.sample_next_token(scratch.ctypes.data, lg.ctypes.data) == orc.sample(lg, r, 0.7, 50, 0.0)
    # overflow quirk: same degenerate pick on both sides
    lib.llama3_sampler_config(4096, 0.05, 50, 0.9)
    hot = H.bits(np.linspace(-5, 12, 4096))
    libc.srand(4)
    assert lib.sample_next_token(scratch.ctypes.data, hot.ctypes.data) == orc.sample(hot, orc.Rand(4), 0.05, 50, 0.9)
    lib.llama3_sampler_config(128256, 0.7, 50, 0.9)
    libc.srand(1)


def test_shipped_half_widening_all_patterns(pkg):
    # temperature 1: tensor[i] * sum == exp(logit): checks the fp16 -> fp32 widening on every finite pattern <= 11
    lib = pkg.lib()
    allbits = np.arange(65536, dtype=np.uint16)
    with np.errstate(invalid="ignore"):
        vals = H.f16(allbits).astype(np.float32)
    keep = np.isfinite(vals) & (np.abs(vals) <= 11.0)
    lg = np.ascontiguousarray(allbits[keep])
    lib.llama3_sampler_config(lg.size, 1.0, 50, 0.9)
    scratch = np.empty(lg.size, np.float32)
    arr = lib.temperature_softmax(scratch.ctypes.data, lg.ctypes.data, C.c_float(1.0))
    C.CDLL("libc.so.6").free(C.c_void_p(arr))
    want = np.exp(vals[keep].astype(np.float64))
    # ratios to the largest entry cancel the rounding of the float running sum
    assert np.allclose(scratch / scratch.max(), want / want.max(), rtol=1e-6, atol=0)
    assert abs(float(scratch.astype(np.float64).sum()) - 1.0) < 1e-4
    lib.llama3_sampler_config(128256, 0.7, 50, 0.9)


def test_exponentials_are_single_precision_as_in_a_cpp_translation_unit(pkg):
    """inference.cu:1048 writes exp(float): compiled as C++ (nvcc on a .cu file) that is the float overload, not
    a promotion to double.  Over every finite fp16 logit at temperature 0.7 the two readings differ in the last
    bit for some patterns; the shipped temperature_softmax matches the single-precision reading bit for bit
    (libm's expf, the running float sum in index order, then the division) and not the double one."""
    lib = pkg.lib()
    libm = C.CDLL("libm.so.6")
    libm.expf.restype, libm.expf.argtypes = C.c_float, [C.c_float]
    libm.exp.restype, libm.exp.argtypes = C.c_double, [C.c_double]
    f = np.float32
    allbits = np.arange(65536, dtype=np.uint16)
    with np.errstate(invalid="ignore"):
        vals = H.f16(allbits).astype(f)
    keep = np.isfinite(vals) & (np.abs(vals) <= 20.0)
    lg = np.ascontiguousarray(allbits[keep][::7])          # a few thousand patterns
    scaled = (H.f16(lg).astype(f) / f(0.7)).astype(f)
    single = np.array([libm.expf(float(x)) for x in scaled], dtype=f)
    double = np.array([libm.exp(float(x)) for x in scaled]).astype(f)
    differ = int(np.count_nonzero(single != double))
    assert differ > 0                                        # otherwise this test could not tell the readings apart

    def probabilities(e):
        total = f(0)
        for v in e:
            total = f(total + v)
        return (e / total).astype(f)

    lib.llama3_sampler_config(lg.size, 0.7, 50, 0.9)
    scratch = np.empty(lg.size, f)
    arr = lib.temperature_softmax(scratch.ctypes.data, lg.ctypes.data, C.c_float(0.7))
    C.CDLL("libc.so.6").free(C.c_void_p(arr))
    lib.llama3_sampler_config(128256, 0.7, 50, 0.9)
    assert np.array_equal(scratch, probabilities(single))
    assert not np.array_equal(scratch, probabilities(double))


def test_fast_head_selection_equals_the_full_sort_path(pkg):
    """sample_next_token() selects only the top-k head; sample_next_token_reference() is the reference's
    call sequence with the full qsort.  fp16 logits at vocabulary size tie constantly, so the order among
    equal probabilities is exercised on every draw."""
    import time
    lib = pkg.lib()
    libc = C.CDLL("libc.so.6")
    rng = np.random.default_rng(5)
    for vocab, n, scale in ((300, 200, 1.0), (4096, 100, 0.5), (128256, 6, 2.0), (128256, 3, 0.01)):
        lib.llama3_sampler_config(vocab, 0.7, 50, 0.9)
        scratch = np.empty(vocab, np.float32)
        cases = [_logits(rng, vocab, scale) for _ in range(n)]
        libc.srand(11)
        t0 = time.time()
        fast = [lib.sample_next_token(scratch.ctypes.data, lg.ctypes.data) for lg in cases]
        t1 = time.time()
        libc.srand(11)
        full = [lib.sample_next_token_reference(scratch.ctypes.data, lg.ctypes.data) for lg in cases]
        t2 = time.time()
        assert fast == full
        print("vocab %d: head selection %.3f ms per token, full sort %.3f ms" % (vocab, 1e3 * (t1 - t0) / n, 1e3 * (t2 - t1) / n))
    lib.llama3_sampler_config(128256, 0.7, 50, 0.9)
    libc.srand(1)


def test_two_vocabularies_interleaved_do_not_share_settings(pkg):
    """The settings-carrying sampler reads no process-wide state: draws for a 4096-entry and a
    128256-entry vocabulary alternate on exactly-sized buffers while the process-wide setting names a
    third size, and each equals the oracle's draw."""
    lib = pkg.lib()
    libc = C.CDLL("libc.so.6")
    rng = np.random.default_rng(8)
    lib.llama3_sampler_config(777, 0.7, 50, 0.9)
    libc.srand(3)
    r = orc.Rand(3)
    for i in range(8):
        vocab = (4096, 128256)[i % 2]
        lg = _logits(rng, vocab, scale=2.0)
        scratch = np.empty(vocab, np.float32)
        got = lib.llama3_sample_with(vocab, 0.7, 50, 0.9, scratch.ctypes.data, lg.ctypes.data)
        assert got == orc.sample(lg, r)
    lib.llama3_sampler_config(128256, 0.7, 50, 0.9)
    libc.srand(1)


def test_sampler_sources_under_address_sanitizer(tmp_path):
    """The host sampler compiled with -fsanitize=address (host code only) and driven with two
    vocabulary sizes alternately on heap buffers of exactly those sizes, through the settings-carrying
    call and through the reference-named call after llama3_sampler_config: any read or write past a
    buffer aborts the program."""
    import os
    import shutil
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    src = os.path.join(root, "llm.cu_amd", "src")
    main = tmp_path / "main.cpp"
    main.write_text(r'''
#include <cstdio>
#include <cstdlib>
#include <vector>
#include "llama3_host.h"
extern "C" const char *llm_last_error(void) { return ""; }  // the kernel library is not part of this build
int main() {
    const int sizes[2] = {4096, 128256};
    long acc = 0;
    for (int it = 0; it < 6; ++it) {
        const int v = sizes[it % 2];
        std::vector<llm_half> lg(v);
        std::vector<float> scratch(v);
        for (int i = 0; i < v; ++i) lg[i] = (llm_half)(0x3000 + (i * 2654435761u >> 20) % 0x0c00); // 0.125 .. 4
        acc += llama3_sample_with(v, 0.7f, 50, 0.9f, scratch.data(), lg.data());
        acc += llama3_sample_with(v, 1.3f, 0, 0.5f, scratch.data(), lg.data());   // full-sort path
        llama3_sampler_config(v, 0.7f, 50, 0.9f);
        acc += sample_next_token(scratch.data(), lg.data());
        acc += sample_next_token_reference(scratch.data(), lg.data());
    }
    printf("ok %ld\n", acc);
    return 0;
}
''')
    exe = tmp_path / "sampler_asan"
    cmd = [shutil.which("g++") or "g++", "-O1", "-g", "-std=c++17", "-fsanitize=address", "-fno-omit-frame-pointer",
           "-fopenmp", "-I", os.path.join(root, "include"), "-I", src, str(main),
           os.path.join(src, "inference", "sampler.cpp"), os.path.join(src, "common", "fail.cpp"), "-o", str(exe)]
    subprocess.check_call(cmd)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0", LD_PRELOAD="")
    out = subprocess.run([str(exe)], env=env, capture_output=True, text=True, timeout=120)
    assert out.returncode == 0 and out.stdout.startswith("ok"), out.stderr[-2000:]
