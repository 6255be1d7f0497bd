"""Static check of llm.cu_amd/csrc/decode_fused.hip, on the CPU: its streaming loop issues the weight loads as
instructions and waits for them with an explicit count, so the compiler knows nothing about loads in flight.
The invariant it relies on: a register that a weight load will write is neither read nor written by any other
instruction until a wait that covers the load has executed.  The kernel is compiled to assembly for gfx950
and every instantiation is scanned."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"


def _regs(tok):
    m = re.match(r"v\[(\d+):(\d+)\]", tok)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(r"v(\d+)$", tok)
    return {int(m.group(1))} if m else set()


def _scan(lines):
    """Returns (weight loads found, violations) for one kernel's instruction list, in text order."""
    idx = [i for i, l in enumerate(lines) if re.search(r"global_load_dwordx4 .* nt", l)]
    if not idx:
        return 0, ["no weight loads found"]
    pending, bad = [], []  # pending: destination register sets of loads not yet covered by a wait, oldest first
    for i in range(idx[0], min(len(lines), idx[-1] + 400)):
        l = lines[i].split(";")[0].strip()
        if not l or l.endswith(":") or l.startswith("."):
            continue
        op, _, rest = l.partition(" ")
        toks = [t.strip() for t in rest.replace(",", " ").split()]
        if op == "global_load_dwordx4" and " nt" in l:
            used = set().union(*[_regs(t) for t in toks[1:]]) if len(toks) > 1 else set()
            bad += ["line %d: address uses a register in flight: %s" % (i, l) for p in pending if p & used]
            pending.append(_regs(toks[0]))
            continue
        if op == "s_waitcnt" and "vmcnt" in l:
            n = int(re.search(r"vmcnt\((\d+)\)", l).group(1))
            pending = pending[len(pending) - n:] if 0 < n < len(pending) else ([] if n == 0 else pending)
            continue
        if op.startswith("scratch_") and pending:
            bad.append("line %d: spill traffic inside the streaming loop: %s" % (i, l))
        used = set().union(*[_regs(t) for t in toks]) if toks else set()
        bad += ["line %d: touches a register in flight: %s" % (i, l) for p in pending if p & used]
    return len(idx), bad


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc is not installed")
def test_streaming_loop_never_touches_a_register_in_flight(tmp_path):
    src = os.path.join(ROOT, "llm.cu_amd", "csrc", "decode_fused.hip")
    out = tmp_path / "decode_fused.s"
    subprocess.check_call([HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off", "-Xclang",
                           "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument",
                           "-I", os.path.join(ROOT, "include"), "-I", os.path.join(ROOT, "llm.cu_amd", "csrc"),
                           "-S", "--cuda-device-only", src, "-o", str(out)], stderr=subprocess.DEVNULL)
    text = open(out).read().split("\n")
    starts = [i for i, l in enumerate(text) if re.match(r"_Z19decode_fused_kernel\w+:", l)]
    assert len(starts) >= 6
    for s in starts:
        end = next(i for i in range(s, len(text)) if "s_endpgm" in text[i])
        n, bad = _scan(text[s:end + 1])
        assert n == 24, (text[s], n)          # three ring stages of eight loads
        assert not bad, (text[s], bad[:5])
