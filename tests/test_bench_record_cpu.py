"""bench.py's record without a GPU: the final line stays compact and strict JSON, and `roofline.traffic` is tied to the
counter summaries under profiles/ by the hash of the kernel source they were taken on."""
import hashlib
import importlib.util
import json
import math
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def bench():
    spec = importlib.util.spec_from_file_location("_bench_under_test", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_non_finite_numbers_become_null(bench):
    rec = {"a": float("nan"), "b": [1.0, float("inf"), {"c": -float("inf")}], "d": 2.5, "e": "x", "f": None}
    out = bench._finite(rec)
    assert out == {"a": None, "b": [1.0, None, {"c": None}], "d": 2.5, "e": "x", "f": None}
    json.loads(json.dumps(out, allow_nan=False))  # strict JSON: raises on NaN / Infinity


def test_a_full_record_stays_compact(bench):
    """A record with every field the GPU run fills in, 24 target rows included, is well under the size the driver reads whole."""
    targets = {"decode_%s_m%d%s" % (n, m, s): {"us": 123.45, "frac": 0.1234, "target": 0.6, "kernels": 2}
               for n in ("qkv", "o", "gate_up", "down") for m in (1, 16) for s in ("", "_pre", "_bf16_pre")}
    targets.update(fp16_4096={"us": 108.12, "frac": 0.5085, "target": 0.75, "kernels": 1}, fp8_fused_4096={"us": 56.13, "frac": 0.49, "target": 0.7, "kernels": 1})
    roof = {"bound": "mfma", "achieved": 1271.123456789, "peak": 2500.0, "unit": "TFLOP/s", "frac": 0.508449, "traffic": 235.1e6, "traffic_source": "profiles/x.txt",
            "algorithmic_bytes": 100663296.0, "kernel": "fp16_gemm_kernel<f16,256,256,row-major B>", "sclk_mhz": 1898.0, "power_w": 1375.0, "peak_at_clock": 1977.0,
            "frac_at_clock": 0.646, "peak_measured": 2100.0, "frac_of_measured": 0.6, "targets": targets, "targets_note": "x" * 160}
    line = {"metric": "TFLOPS (% of MI355X FP8/FP16 MFMA peak) at 4096³; HBM GB/s at M≤16 decode", "value": 1271.1, "unit": "TFLOP/s", "n_gpus": 1,
            "steps": 20, "warmup": 5, "ms_per_step": 0.10812, "wall_ms_per_step": 0.1083, "timing": "y" * 120, "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "f16", "data": "synthetic", "config": {"workload": "z" * 120, "M": 4096, "N": 4096, "K": 4096}, "roofline": roof,
            "cpu_baseline": {"value": 0.025, "unit": "TFLOP/s", "cores": 16, "kind": "port", "sample": "w" * 160}}
    assert len(json.dumps(bench._finite(line), allow_nan=False)) < 6000


def test_traffic_comes_from_a_profile_of_the_same_source(bench, tmp_path, monkeypatch):
    # the committed summaries either match the sources in the tree or yield None with a reason: never a stale figure
    for wl, (fname, src) in bench.TRAFFIC_PROFILES.items():
        value, why = bench.measured_traffic(wl)
        text = open(os.path.join(ROOT, "profiles", fname)).read()
        m = re.search(r"sha256\(%s\) = ([0-9a-f]{64})" % re.escape(src), text)
        fresh = bool(m) and m.group(1) == hashlib.sha256(open(os.path.join(ROOT, "llmmm_amd", "csrc", src), "rb").read()).hexdigest()
        assert (value is not None) == fresh, (wl, why)
        if value is not None:
            assert 1e6 < value < 1e10 and why == "profiles/" + fname
    assert bench.measured_traffic("decode_o_m1") == (None, "no counter summary for this workload")
    # a tree whose kernel source differs from the one the summary names
    fake = tmp_path / "repo"
    (fake / "profiles").mkdir(parents=True)
    (fake / "llmmm_amd" / "csrc").mkdir(parents=True)
    (fake / "llmmm_amd" / "csrc" / "fp16_gemm.hip").write_text("// kernel, version 1\n")
    h = hashlib.sha256(b"// kernel, version 1\n").hexdigest()
    (fake / "profiles" / "fp16_gemm_kernel_4096.txt").write_text("  traffic = 235.1 MB per launch vs 100.7 MB algorithmic\nsha256(fp16_gemm.hip) = %s\n" % h)
    monkeypatch.setattr(bench, "HERE", str(fake))
    assert bench.measured_traffic("fp16_gemm_4096") == (235.1e6, "profiles/fp16_gemm_kernel_4096.txt")
    (fake / "llmmm_amd" / "csrc" / "fp16_gemm.hip").write_text("// kernel, version 2\n")
    value, why = bench.measured_traffic("fp16_gemm_4096")
    assert value is None and "another version" in why
    (fake / "profiles" / "fp16_gemm_kernel_4096.txt").unlink()
    assert bench.measured_traffic("fp16_gemm_4096")[0] is None
