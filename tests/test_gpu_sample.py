"""llm_sample_candidates against the host loop it stands in for (ref src/inference/inference.cu:1043-1072):
the float32 denominator accumulated in index order, probabilities by float32 division, and the first k
entries of a stable descending sort -- all compared bit for bit with numpy, whose float32 accumulate and
divide are the same IEEE operations the host code performs."""
import numpy as np
import pytest

from tests import helpers as H

pytestmark = pytest.mark.gpu


def host_table(temperature):
    h = np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32)
    with np.errstate(over="ignore", invalid="ignore", divide="ignore"):
        return np.exp(h / np.float32(temperature)).astype(np.float32)


def expect(logits_bits, table, k):
    x = table[logits_bits.astype(np.int64)]
    denom = np.add.accumulate(x, dtype=np.float32)[-1]
    p = (x / denom).astype(np.float32)
    order = np.lexsort((np.arange(p.size), -p.astype(np.float64)))[:k]  # probability descending, index ascending
    return denom, p[order], order.astype(np.int32)


def check(gpu, logits_bits, table, k, name):
    denom, flag, one_by_one, p, idx = gpu.ops.sample_candidates(logits_bits, table, k)
    w_denom, w_p, w_idx = expect(logits_bits, table, k)
    assert flag == 0, name
    assert np.float32(denom).view(np.uint32) == np.float32(w_denom).view(np.uint32), (name, denom, w_denom)
    order = np.lexsort((idx, -p.astype(np.float64)))
    assert np.array_equal(idx[order], w_idx), name
    assert np.array_equal(p[order].view(np.uint32), w_p.view(np.uint32)), name
    return one_by_one


def order_keys():
    """The 16-bit key that orders fp16 bit patterns like their values (-0 with +0), as int64[65536]."""
    b = np.arange(65536, dtype=np.int64)
    key = np.where(b & 0x8000, 0x7fff - (b & 0x7fff), 0x8000 + b)
    key[0x8000] = 0x8000
    return key


def bits_of(values):
    return np.asarray(values, np.float32).astype(np.float16).view(np.uint16)


def test_candidates_on_model_like_logits(gpu):
    rng = np.random.default_rng(0)
    table = host_table(0.7)
    for vocab, k in ((128256, 50), (128256, 1), (128256, 1000), (4096, 50), (1000, 7), (1025, 1024), (2, 1)):
        lg = bits_of(rng.normal(0, 3, vocab))
        n1 = check(gpu, lg, table, k, ("normal", vocab, k))
        assert n1 <= 200, n1  # groups of 8 entries added one by one: the start and the binade changes, not the rule


def test_candidates_with_ties_and_colliding_probabilities(gpu):
    rng = np.random.default_rng(1)
    table = host_table(0.7)
    vocab = 128256
    check(gpu, bits_of(np.zeros(vocab)), table, 50, "all equal")
    check(gpu, bits_of(rng.integers(-2, 3, vocab) * 0.5), table, 50, "five levels")
    check(gpu, bits_of(np.where(rng.random(vocab) < 0.5, 0.0, -0.0)), table, 50, "signed zeros")
    lg = bits_of(rng.normal(0, 1, vocab))
    lg[rng.integers(0, vocab, 40)] = bits_of([9.0])[0]  # 40 equal leaders, k cuts through what follows
    check(gpu, lg, table, 50, "equal leaders")
    check(gpu, lg, table, 30, "k inside the equal leaders")
    # a monotone table with plateaus: distinct logits, same probability -- the cut must follow the probability
    key = order_keys()
    finite = (np.arange(65536) & 0x7fff) <= 0x7c00
    plateau = np.where(finite, (key // 64 * 64).astype(np.float32) + 1.0, np.float32(np.nan)).astype(np.float32)
    lgp = rng.integers(0x3000, 0x4400, vocab).astype(np.uint16)  # positive halves between 0.125 and 4
    for k in (1, 13, 50, 333):
        check(gpu, lgp, plateau, k, ("plateaus", k))
    # numerators one ulp apart under a denominator with a larger mantissa: the division merges neighbours
    ulps = (key - 0xB000).clip(0, 6000).astype(np.float32)
    close = (np.float32(1.9) + ulps * np.spacing(np.float32(1.9))).astype(np.float32)
    close = np.where(finite, close, np.float32(np.nan)).astype(np.float32)
    x = close[lgp.astype(np.int64)]
    p = (x / np.add.accumulate(x, dtype=np.float32)[-1]).astype(np.float32)
    assert np.unique(p).size < np.unique(x).size  # the case does what it is built for
    for k in (50, 2000):
        check(gpu, lgp, close, k, ("merged neighbours", k))


def test_candidates_over_a_wide_range_of_magnitudes(gpu):
    rng = np.random.default_rng(2)
    vocab = 128256
    # temperature 0.05: exp spans the float32 range, the denominator changes binade again and again, early
    # entries vanish next to later ones, some table entries are denormal
    table = host_table(0.05)
    lg = bits_of(np.clip(rng.normal(0, 1.2, vocab), -4.0, 4.0))
    assert np.isfinite(table[lg.astype(np.int64)]).all()
    check(gpu, lg, table, 50, "temperature 0.05")
    lg_sorted = bits_of(np.sort(np.clip(rng.normal(0, 1.2, vocab), -4.0, 4.0)))
    n1 = check(gpu, lg_sorted, table, 50, "ascending logits")
    check(gpu, lg_sorted[::-1].copy(), table, 50, "descending logits")
    print("ranges added one by one on ascending logits:", n1)
    f = H.f16(np.arange(65536, dtype=np.uint16))
    with np.errstate(invalid="ignore"):
        tiny = np.where(f >= 2.0, np.float32(3e-44), np.where(f >= 1.0, np.float32(1e-44), np.float32(0)))
    tiny = np.where(np.isnan(f), np.float32(np.nan), tiny).astype(np.float32)
    check(gpu, bits_of(rng.choice([1.0, 2.0], vocab)), tiny, 50, "denormal numerators")


def test_candidates_report_what_they_cannot_decide(gpu):
    rng = np.random.default_rng(3)
    table = host_table(0.7)
    lg = bits_of(rng.normal(0, 3, 4096))
    bad = lg.copy()
    bad[77] = 0x7e00  # NaN logit
    assert gpu.ops.sample_candidates(bad, table, 50)[1] == 1
    inf = lg.copy()
    inf[5] = bits_of([60000.0])[0]  # exp overflows to infinity
    assert gpu.ops.sample_candidates(inf, table, 50)[1] == 1
    assert gpu.ops.sample_candidates(lg, np.zeros(65536, np.float32), 50)[1] == 1  # zero denominator
    L = gpu.lib()
    buf = gpu.capi.DevBuf((4096,), np.uint16)
    tab = gpu.capi.DevBuf((65536,), np.float32)
    out = gpu.capi.DevBuf((1024,), np.uint32)
    assert L.llm_sample_candidates(buf.ptr, tab.ptr, 4096, 0, out.ptr, None) == gpu.capi.LLM_ERR_INVALID
    assert L.llm_sample_candidates(buf.ptr, tab.ptr, 4096, 4096, out.ptr, None) == gpu.capi.LLM_ERR_INVALID
    assert L.llm_sample_candidates(None, tab.ptr, 4096, 5, out.ptr, None) == gpu.capi.LLM_ERR_INVALID


def _sampling_engine(gpu, vocab):
    cfg = gpu.engine.config("tiny", max_pos=64, vocab=vocab)
    model = gpu.engine.Model.seeded(cfg, 7).to_device()
    return cfg, model, gpu.engine.Engine(model, cfg)


def test_device_assisted_draws_equal_the_host_sampler_and_the_oracle(gpu):
    """The cache's sampler on device-resident logits: candidates from the device, draw on the host.  For
    the same rand() stream the ids equal the oracle's restatement of sample_next_token and the library's
    all-host sampler, at the full vocabulary, on logits with many equal values (where the order of equal
    probabilities decides) and at other settings."""
    import ctypes as C
    from oracle import pyoracle as orc
    libc = C.CDLL("libc.so.6")
    vocab = 128256
    cfg, model, eng = _sampling_engine(gpu, vocab)
    rng = np.random.default_rng(5)
    cases = [("normal", bits_of(rng.normal(0, 3, vocab))),
             ("few levels", bits_of(rng.integers(-3, 4, vocab) * 0.25)),
             ("all equal", bits_of(np.zeros(vocab))),
             ("equal leaders", bits_of(np.where(rng.random(vocab) < 0.001, 8.0, rng.normal(0, 1, vocab)))),
             ("flat with one peak", bits_of(np.r_[np.zeros(vocab - 1), 6.0]))]
    settings = [(0.7, 50, 0.9), (1.3, 5, 0.5), (0.2, 200, 0.99), (0.7, 1, 0.9)]
    for temperature, top_k, top_p in settings:
        eng.sampler_config(temperature, top_k, top_p)
        for name, lg in cases:
            dev = gpu.capi.DevBuf.from_host(lg)
            seed = 1000 + top_k
            libc.srand(seed)
            got = [eng.sample_device_logits(dev) for _ in range(8)]
            rnd = orc.Rand(seed)
            want = [orc.sample(lg, rnd, temperature, top_k, top_p) for _ in range(8)]
            assert got == want, (name, temperature, top_k, top_p, got, want)
            libc.srand(seed)
            scratch = np.empty(vocab, np.float32)
            host = [gpu.lib().llama3_sample_with(vocab, temperature, top_k, top_p, scratch.ctypes.data, lg.ctypes.data)
                    for _ in range(8)]
            assert host == want, (name, "host path")
    dev_draws, host_draws = eng.sampler_draw_counts()
    assert dev_draws == len(settings) * len(cases) * 8 and host_draws == 0
    # what the device cannot decide goes to the host path, same ids
    eng.sampler_config(0.7, 50, 0.9)
    nan = cases[0][1].copy()
    nan[123] = 0x7e00
    libc.srand(3)
    got = eng.sample_device_logits(nan)
    assert eng.sampler_draw_counts() == (dev_draws, 1)
    libc.srand(3)
    assert got == eng.sample_device_logits(nan)
    # settings that can reach the tail of the sorted array are the host's from the start
    eng.sampler_config(0.7, 50, 1.0)
    libc.srand(4)
    got = eng.sample_device_logits(cases[0][1])
    assert got == orc.sample(cases[0][1], orc.Rand(4), 0.7, 50, 1.0)
    assert eng.sampler_draw_counts() == (dev_draws, 3)
    libc.srand(1)
    eng.close()
    model.close()


def test_inference_samples_through_the_device_selection(gpu):
    """inference() with the reference's sampler on: draws come from device-selected candidates, equal the
    oracle's, and equal those of the same cache with the device selection turned off."""
    import ctypes as C
    from oracle import pyoracle as orc
    libc = C.CDLL("libc.so.6")
    cfg, model, eng = _sampling_engine(gpu, 4096)
    eng.set_sampling(True)
    prompt = [int(t) for t in gpu.engine.seeded_tokens(3, 10, cfg.vocab)]
    runs = []
    for device in (True, False):
        eng.reset()
        eng.set_device_sampling(device)
        libc.srand(11)
        rnd = orc.Rand(11)
        seq = list(prompt)
        for _ in range(12):
            tok = eng.inference(seq)
            assert tok == orc.sample(eng.host_logits(), rnd)
            seq.append(tok)
        runs.append(seq)
    assert runs[0] == runs[1]
    assert eng.sampler_draw_counts() == (12, 12)
    libc.srand(1)
    eng.close()
    model.close()
