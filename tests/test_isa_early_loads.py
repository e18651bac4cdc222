"""Static check of the generated-operand modes of the weight-streaming kernel (llmmm_amd/csrc/fp8_skinny.hip).

Those kernels request the data of their A operand with inline-assembly loads in front of the ring prologue and wait for it
with a hand-counted ``s_waitcnt vmcnt(n)``.  The compiler does not know these loads are in flight, so the scheme is only
sound if it leaves their destination registers alone until that wait: no copy out of them, no reuse, pairwise distinct.
This test compiles the file to gfx950 assembly (the build's own flags) and checks exactly that for every instantiation."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _regs(tok):
    m = re.match(r"v\[(\d+):(\d+)\]", tok)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(r"v(\d+)$", tok)
    return {int(m.group(1))} if m else set()


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="hipcc not available")
def test_early_load_registers_are_untouched_until_the_counted_wait(tmp_path):
    import importlib.util
    spec = importlib.util.spec_from_file_location("_llmmm_build", os.path.join(ROOT, "llmmm_amd", "build.py"))
    build = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(build)
    out = str(tmp_path / "fp8_skinny.s")
    cmd = ["hipcc"] + build.COMMON + build.SOURCES["fp8_skinny.hip"] + ["-I", os.path.join(ROOT, "include"), "-S", "--cuda-device-only",
                                                                       os.path.join(build.CSRC, "fp8_skinny.hip"), "-o", out]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert res.returncode == 0, res.stdout[-2000:]
    lines = open(out).read().split("\n")
    checked = 0
    for idx, line in enumerate(lines):
        m = re.match(r"(_ZN5llmmm17fp8_skinny_kernelILi1ELi\dELi\dELi\d+ELi([12])E\w+):\s", line)
        if not m:
            continue
        name, mode = m.group(1), int(m.group(2))
        end = next(i for i in range(idx, len(lines)) if "s_endpgm" in lines[i])
        body = lines[idx:end]
        first_ring = next(i for i, x in enumerate(body) if "global_load_lds" in x)
        wait = next(i for i, x in enumerate(body) if i > first_ring and re.search(r"s_waitcnt vmcnt", x))
        dests = []
        for i, x in enumerate(body[:first_ring]):
            mm = re.match(r"\s+global_load_dwordx[24] (v\[\d+:\d+\]),", x)
            if mm:
                dests.append((i, _regs(mm.group(1))))
        assert len(dests) == (8 if mode == 1 else 36), (name, len(dests))  # 4 tasks x (gate, up) / 3 chunks x (residual, w, 10 planes)
        seen = set()
        for i, r in dests:
            assert not (seen & r), "%s: two early loads share registers %s" % (name, sorted(seen & r))
            seen |= r
        # the wait behind the ring prologue allows exactly the ring's loads to stay in flight
        ring_loads = sum(1 for x in body[first_ring:wait] if "global_load_lds" in x)
        n = re.search(r"vmcnt\((\d+)\)", body[wait])
        assert n and int(n.group(1)) == ring_loads, (name, body[wait], ring_loads)
        assert not any(re.match(r"\s+(global|buffer|flat)_load", x) and "global_load_lds" not in x for x in body[first_ring:wait]), name
        for i, x in enumerate(body[:wait]):
            toks = re.findall(r"v\[\d+:\d+\]|v\d+", x)
            if re.match(r"\s+global_load_dwordx[24]", x):
                toks = toks[1:]  # its own destination
            for t in toks:
                for di, dr in dests:
                    assert not (i > di and _regs(t) & dr), "%s: '%s' touches an early-load register before the wait" % (name, x.strip())
        checked += 1
    assert checked == 18, checked  # swiglu: 3 outputs x 3 ring depths; rmsnorm: 3 hidden types x 3 ring depths
