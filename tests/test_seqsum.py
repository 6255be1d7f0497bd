"""The parallel form of the sampler's float32 running sum (llm.cu_amd/csrc/seqsum.hpp, compiled for the CPU)
against the plain loop it replaces: numpy's float32 accumulate adds one element after the other, as the
reference's softmax denominator does (src/inference/inference.cu:1049-1056)."""
import ctypes as C
import os
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def seqlib(tmp_path_factory):
    out = tmp_path_factory.mktemp("seqsum") / "libseqsum_host.so"
    subprocess.run(["g++", "-O2", "-std=c++17", "-shared", "-fPIC", "-I", os.path.join(ROOT, "llm.cu_amd", "csrc"),
                    os.path.join(ROOT, "tests", "native", "seqsum_host.cpp"), "-o", str(out)], check=True)
    lib = C.CDLL(str(out))
    lib.seqsum_segments.restype = C.c_float
    lib.seqsum_segments.argtypes = [C.c_void_p, C.c_int, C.c_int, C.POINTER(C.c_int)]
    lib.seqsum_composed.restype = C.c_float
    lib.seqsum_composed.argtypes = [C.c_void_p, C.c_int, C.c_int, C.POINTER(C.c_int)]
    return lib


def loop_sum(x):
    return np.add.accumulate(x.astype(np.float32), dtype=np.float32)[-1] if x.size else np.float32(0)


def cases():
    rng = np.random.default_rng(7)
    out = []
    for n in (1, 2, 63, 1000, 4097, 128256):
        lg = rng.normal(0, 3, n).astype(np.float16).astype(np.float32)
        out.append(("softmax numerators, temperature 0.7", np.exp(lg / np.float32(0.7)).astype(np.float32)))
    out.append(("one dominant entry in the middle", np.exp(np.r_[rng.normal(0, 1, 5000), 30.0, rng.normal(0, 1, 5000)]).astype(np.float32)))
    out.append(("ties everywhere: halves of the unit", np.r_[np.float32(2 ** 20), np.full(50000, 0.0625, np.float32)]))
    out.append(("odd multiples of half a unit", np.r_[np.float32(2 ** 23 + 1), np.tile(np.array([0.5, 1.5, 2.5, 0.5], np.float32), 3000)]))
    out.append(("powers of two of every size", (2.0 ** rng.integers(-140, 60, 30000)).astype(np.float32)))
    out.append(("all equal", np.full(128256, np.exp(np.float32(1.0)), np.float32)))
    out.append(("denormals and zeros first", np.r_[np.zeros(300, np.float32), np.full(500, 1e-44, np.float32), rng.random(5000).astype(np.float32)]))
    out.append(("wide dynamic range, increasing", np.sort(np.exp(rng.uniform(-80, 80, 40000))).astype(np.float32)))
    out.append(("wide dynamic range, decreasing", np.sort(np.exp(rng.uniform(-80, 80, 40000)))[::-1].astype(np.float32).copy()))
    out.append(("mantissas with few bits", (rng.integers(1, 8, 60000) * 2.0 ** rng.integers(-12, 4, 60000)).astype(np.float32)))
    return out


@pytest.mark.parametrize("seg_len", [1, 7, 126, 1000])
def test_segment_scheme_equals_the_sequential_loop(seqlib, seg_len):
    for name, x in cases():
        x = np.ascontiguousarray(x, np.float32)
        nseq = C.c_int(0)
        got = seqlib.seqsum_segments(x.ctypes.data, x.size, seg_len, C.byref(nseq))
        want = loop_sum(x)
        assert np.float32(got).view(np.uint32) == np.float32(want).view(np.uint32), (name, seg_len, got, want)
        n_seg = -(-x.size // seg_len)
        if x.size >= 4097 and seg_len == 126 and "range" not in name and "powers" not in name and "dominant" not in name:
            # the fall-back is the exception, not the rule: a handful of binade changes
            assert nseq.value <= 40, (name, nseq.value, n_seg)


def test_a_wrong_tie_rule_would_be_caught(tmp_path):
    """The cases do exercise ties and their parity rule: the same scheme with ties always rounded up differs."""
    src = open(os.path.join(ROOT, "llm.cu_amd", "csrc", "seqsum.hpp")).read()
    assert "c0 = (m.a0 + X) & 1u;" in src and "c1 = (1u + m.a1 + X) & 1u;" in src
    (tmp_path / "seqsum.hpp").write_text(src.replace("c0 = (m.a0 + X) & 1u;", "c0 = 1;")
                                         .replace("c1 = (1u + m.a1 + X) & 1u;", "c1 = 1;"))
    out = tmp_path / "libseqsum_wrong.so"
    subprocess.run(["g++", "-O2", "-std=c++17", "-shared", "-fPIC", "-I", str(tmp_path),
                    os.path.join(ROOT, "tests", "native", "seqsum_host.cpp"), "-o", str(out)], check=True)
    lib = C.CDLL(str(out))
    lib.seqsum_segments.restype = C.c_float
    lib.seqsum_segments.argtypes = [C.c_void_p, C.c_int, C.c_int, C.POINTER(C.c_int)]
    wrong = 0
    for name, x in cases():
        x = np.ascontiguousarray(x, np.float32)
        got = lib.seqsum_segments(x.ctypes.data, x.size, 126, None)
        wrong += np.float32(got).view(np.uint32) != np.float32(loop_sum(x)).view(np.uint32)
    assert wrong >= 4


def test_composition_in_tree_order(seqlib):
    rng = np.random.default_rng(3)
    for trial in range(200):
        es = int(rng.integers(100, 160))
        s0 = np.float32(2.0 ** (es - 127) * (1 + rng.random() * 0.5))
        u = np.float32(2.0 ** (es - 150))
        n = int(rng.integers(1, 300))
        # multiples of a quarter unit: a tie in a quarter of the additions, increments that keep s in its binade
        x = (rng.integers(0, 24, n) * 0.25 * float(u)).astype(np.float32)
        arr = np.ascontiguousarray(np.r_[s0, x], np.float32)
        ok = C.c_int(0)
        got = seqlib.seqsum_composed(arr.ctypes.data, n, es, C.byref(ok))
        want = loop_sum(arr)
        if int(np.float32(want).view(np.uint32)) >> 23 != es:
            assert ok.value == 0
        else:
            assert ok.value == 1 and np.float32(got).view(np.uint32) == np.float32(want).view(np.uint32), (trial, got, want)
