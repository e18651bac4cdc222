#!/usr/bin/env python3
"""Benchmark of the matrix-multiplication hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu] [--no-shapes]

A "step" is one GEMM launch through the C ABI (``libllmmm.so``) on inputs already resident in
HBM.  The headline workload is the FP16 GEMM at M=N=K=4096 (A ~ N(0,1), B ~ N(0,0.02), seed 2,
fp32 accumulation, fp16 output, one kernel, no split-K); ``value`` is its TFLOP/s
(2*M*N*K / time).  The LAST line of stdout is the record: one compact strict-JSON object (a few KB) with
  * ``roofline``: the dominant kernel against MI355X's published dense MFMA peak (or HBM peak
    for the decode shapes), from HIP events recorded on the launch stream around the timed
    region; ``roofline.targets``: FP16 4096^3, FP8 fused 4096^3 and the decode projections at M = 1 and 16,
    each with its microseconds and fraction of the published peak;
  * ``cpu_baseline``: the CPU oracle (a port of the reference's Kahan GEMM, test/kahan.cu:16-26)
    timed on this host's cores on a bounded sample of the same workload.
The lines before it, one JSON object each with a ``detail`` key, carry the per-shape table (``shapes``), the
side-by-side vendor-library comparison, the measured peaks, the other CPU baselines and the full target rows.
"""
import argparse
import json
import os
import sys
import time

import numpy as np
import torch

PEAK_TFLOPS = {"f16": 2500.0, "bf16": 2500.0, "fp8": 5000.0}  # MI355X dense MFMA, published
PEAK_HBM_GBS = 8000.0
PREHEAT_S = 0.25  # seconds of untimed launches before the warm-up steps of every measurement

# HBM bytes per launch of the dominant kernel come from rocprofv3 FETCH_SIZE + WRITE_SIZE counter runs of these same
# workloads (counters cannot be read from inside this process).  The summaries under profiles/ carry the result
# ("traffic = X MB per launch") and the SHA-256 of the kernel source file they were taken on; a summary whose hash is
# not that of the source in this tree is stale and yields traffic = null.
HERE = os.path.dirname(os.path.abspath(__file__))
TRAFFIC_PROFILES = {
    "fp16_gemm_4096": ("fp16_gemm_kernel_4096.txt", "fp16_gemm.hip"),
    "fp8_gemm_fused_4096": ("fp8_gemm_kernel_fused_4096.txt", "fp8_gemm.hip"),
    "decode_gate_up_m1": ("fp8_skinny_kernel_gate_up_m1.txt", "fp8_skinny.hip"),
    "decode_gate_up_m1_pre": ("fp8_skinny_kernel_gate_up_m1_preshuffled.txt", "fp8_skinny.hip"),
    "decode_o_m16_pre": ("fp8_strip_kernel_fused_quant_o_m16.txt", "fp8_skinny.hip"),
    "decode_o_m1_bf16_pre": ("fp8_strip_kernel_o_m1.txt", "fp8_skinny.hip"),
}


def source_sha256(name):
    import hashlib
    with open(os.path.join(HERE, "llmmm_amd", "csrc", name), "rb") as f:
        return hashlib.sha256(f.read()).hexdigest()


def measured_traffic(workload):
    """(bytes per launch, note) from the counter summary of this workload, or (None, why not)."""
    import re
    if workload not in TRAFFIC_PROFILES:
        return None, "no counter summary for this workload"
    fname, src = TRAFFIC_PROFILES[workload]
    try:
        text = open(os.path.join(HERE, "profiles", fname)).read()
    except OSError:
        return None, "profiles/%s missing" % fname
    mt = re.search(r"traffic = ([0-9.]+) MB per launch", text)
    mh = re.search(r"sha256\(%s\) = ([0-9a-f]{64})" % re.escape(src), text)
    if not mt or not mh:
        return None, "profiles/%s carries no traffic figure or no source hash" % fname
    if mh.group(1) != source_sha256(src):
        return None, "profiles/%s was taken on another version of %s" % (fname, src)
    return float(mt.group(1)) * 1e6, "profiles/%s" % fname


QWEN3_4B = {"qkv": (6144, 2560), "o": (2560, 4096), "gate_up": (19456, 2560), "down": (2560, 9728)}


TIMED_BATCHES = 7      # batches of `steps` launches timed one after the other; the median is reported
SETTLE_S = 0.06        # untimed replays of a captured graph before the timed ones (the clocks drop during capture)
LAST_SPREAD = {}       # min / max over the timed batches of the most recent _events_ms call, ms per step


def _events_ms(fn, steps, warmup, graph=False):
    """Duration of one call of fn: the median over TIMED_BATCHES batches of `steps` calls, each batch bracketed by HIP
    events on torch's current stream (the stream every launch below is enqueued on); the batches are enqueued back to
    back with no host synchronisation between them, so the GPU never idles inside the timed region.  With graph=True
    (every GEMM workload) a batch is one replay of a HIP graph of `steps` launches, so that kernels are timed back to
    back on the GPU instead of at the pace of the Python launch loop."""
    # Untimed pre-heat: the GPU's clocks take tens of milliseconds of sustained load to settle, far
    # longer than a handful of warm-up launches of a ~100 us kernel; time the settled state.
    t_heat = time.perf_counter()
    while time.perf_counter() - t_heat < PREHEAT_S:
        for _ in range(20):
            fn()
        torch.cuda.synchronize()
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(TIMED_BATCHES)]
    if graph:
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for _ in range(steps):
                fn()
        t_settle, n = time.perf_counter(), 0
        while n < 3 or time.perf_counter() - t_settle < SETTLE_S:  # graph upload, and the clocks back up after the idle capture
            g.replay()
            n += 1
            if n % 8 == 0:
                torch.cuda.synchronize()
        batch = g.replay
    else:
        def batch():
            for _ in range(steps):
                fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for e0, e1 in ev:
        e0.record()
        batch()
        e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / TIMED_BATCHES
    per = sorted(e0.elapsed_time(e1) / steps for e0, e1 in ev)
    LAST_SPREAD.update(min=per[0], max=per[-1])
    return per[len(per) // 2], wall_ms / steps


def sample_clock_power(step, seconds=1.2):
    """Shader clock and socket power while `step` runs back to back for `seconds` (outside any timed region): medians of
    the driver's sysfs readings (pp_dpm_sclk's active level, hwmon power1_input), None where the files cannot be read.
    The published MFMA peaks are quoted at 2400 MHz; at the board's power limit a GEMM runs below that clock."""
    import glob
    import threading
    import time

    def read():
        mhz = watts = None
        for path in glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk"):
            try:
                for ln in open(path).read().splitlines():
                    if "*" in ln:
                        mhz = float(ln.split(":")[1].lower().replace("mhz", "").replace("*", "").strip())
            except (OSError, ValueError, IndexError):
                pass
        for path in glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_input") + glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_average"):
            try:
                watts = int(open(path).read()) / 1e6
                break
            except (OSError, ValueError):
                pass
        return mhz, watts

    samples, stop = [], threading.Event()

    def poll():
        while not stop.is_set():
            samples.append(read())
            time.sleep(0.1)

    for _ in range(50):
        step()
    torch.cuda.synchronize()
    th = threading.Thread(target=poll)
    t0 = time.time()
    th.start()
    while time.time() - t0 < seconds:
        for _ in range(100):
            step()
        torch.cuda.synchronize()
    stop.set()
    th.join()
    samples = samples[len(samples) // 3:]  # the clock settles within the first few hundred milliseconds
    mhz = sorted(x[0] for x in samples if x[0] is not None)
    watts = sorted(x[1] for x in samples if x[1] is not None)
    return {"sclk_mhz": mhz[len(mhz) // 2] if mhz else None, "power_w": watts[len(watts) // 2] if watts else None, "samples": len(samples)}


def _finite(x):
    """x with every float that strict JSON cannot carry (NaN, +-Inf) replaced by None."""
    if isinstance(x, float):
        return x if np.isfinite(x) else None
    if isinstance(x, dict):
        return {k: _finite(v) for k, v in x.items()}
    if isinstance(x, (list, tuple)):
        return [_finite(v) for v in x]
    if isinstance(x, (np.floating, np.integer)):
        return _finite(x.item())
    return x


def emit_detail(name, obj):
    """One JSON object on a line of its own, ahead of the final record."""
    print(json.dumps(_finite({"detail": name, **obj}), allow_nan=False), flush=True)


def fp16_inputs(M, N, K, dtype=torch.float16, seed=2):
    g = torch.Generator(device="cuda").manual_seed(seed)
    A = torch.randn((M, K), generator=g, device="cuda", dtype=torch.float32).to(dtype)
    B = (torch.randn((K, N), generator=g, device="cuda", dtype=torch.float32) * 0.02).to(dtype)
    return A, B


def fp8_inputs(M, N, K, seed=3, copies=1):
    """Activations N(0,1) with 1% of the K channels x20, weights N(0,0.02); quantised on the GPU by
    the library's own quantiser (1x128 for A, 128x128 for Bt).  `copies` distinct weight buffers."""
    import llmmm_amd
    g = torch.Generator(device="cuda").manual_seed(seed)
    A = torch.randn((M, K), generator=g, device="cuda", dtype=torch.float32)
    nout = max(1, (K + 99) // 100)
    cols = torch.randperm(K, generator=g, device="cuda")[:nout]
    A[:, cols] *= 20.0
    Aq, As = llmmm_amd.quantize_activation(A)
    weights = []
    for c in range(copies):
        Wt = torch.randn((N, K), generator=g, device="cuda", dtype=torch.float32) * 0.02
        weights.append(llmmm_amd.quantize_weight(Wt))
        del Wt
    return Aq, As, weights


def bench_fp16(M, N, K, steps, warmup, dtype=torch.float16, b_transposed=False, clock=False):
    import llmmm_amd
    A, B = fp16_inputs(M, N, K, dtype)
    if b_transposed:
        B = B.t().contiguous()
    C = torch.empty((M, N), dtype=dtype, device="cuda")
    ms, wall = _events_ms(lambda: llmmm_amd.fp16_gemm(A, B, C, b_transposed=b_transposed), steps, warmup, graph=True)
    flops = 2.0 * M * N * K
    r = {"ms": ms, "wall_ms": wall, "tflops": flops / ms * 1e-9, "bytes": 2.0 * (M * K + K * N + M * N), "ms_min": LAST_SPREAD.get("min"),
         "ms_max": LAST_SPREAD.get("max")}
    if clock:
        r["clock"] = sample_clock_power(lambda: llmmm_amd.fp16_gemm(A, B, C, b_transposed=b_transposed))
    return r, (A, B, C)


def fp8_bytes(M, N, K, out):
    b = M * K + N * K + 4.0 * (M * K / 128 + (N / 128) * (K / 128))
    if out == "swiglu":
        b += M * N / 2 + 4.0 * M * N / 256
    elif out == "fp8q":
        b += M * N + 4.0 * M * N / 128
    elif out == "bf16":
        b += 2.0 * M * N
    else:
        b += 4.0 * M * N
    return b


def bench_fp8(M, N, K, out, steps, warmup, rotate_bytes=0, preshuffled=False, clock=False):
    """out in {"f32","bf16","fp8q"}.  With rotate_bytes > 0 the launches cycle through enough
    distinct weight copies to exceed that many bytes, so weights stream from HBM, not from cache.
    preshuffled: the weights are permuted once, outside the timed region, into MFMA operand order."""
    import llmmm_amd
    from llmmm_amd import _lib
    copies = 1
    if rotate_bytes:
        copies = max(2, int(np.ceil(rotate_bytes / float(N * K))))
    Aq, As, weights = fp8_inputs(M, N, K, copies=copies)
    if preshuffled:
        weights = [(llmmm_amd.preshuffle_weight(bq), bs) for bq, bs in weights]
    kind = {"f32": _lib.OUT_F32, "bf16": _lib.OUT_BF16, "fp8q": _lib.OUT_FP8Q, "swiglu": _lib.OUT_FP8Q_SWIGLU}[out]
    cdt = {"f32": torch.float32, "bf16": torch.bfloat16, "fp8q": torch.uint8, "swiglu": torch.uint8}[out]
    n_out = N // 2 if out == "swiglu" else N
    C = torch.empty((M, n_out), dtype=cdt, device="cuda")
    Cs = torch.empty((max(1, n_out // 128), M), dtype=torch.float32, device="cuda")
    ws = llmmm_amd.make_workspace(kind, M, N, K)
    fns = {"f32": llmmm_amd.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32,
           "bf16": llmmm_amd.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_bf16}
    state = {"i": 0}

    def step():
        Bq, Bs = weights[state["i"] % copies]
        state["i"] += 1
        if out == "swiglu":
            llmmm_amd.fp8_gemm_blockwise_quant_A_1x128__B_128x128__swiglu__C_1x128__output_fp8(Aq, As, Bq, Bs, C, Cs, M, N, K, workspace=ws,
                                                                                               b_preshuffled=preshuffled)
        elif out == "fp8q":
            llmmm_amd.fp8_gemm_blockwise_quant_A_1x128__B_128x128__C_1x128__output_fp8(Aq, As, Bq, Bs, C, Cs, M, N, K, workspace=ws,
                                                                                       b_preshuffled=preshuffled)
        else:
            fns[out](Aq, As, Bq, Bs, C, M, N, K, workspace=ws, b_preshuffled=preshuffled)

    ms, wall = _events_ms(step, steps, warmup, graph=True)
    flops = 2.0 * M * N * K
    nbytes = fp8_bytes(M, N, K, out)
    tile, split = llmmm_amd.query_config(kind, M, N, K)
    kernel = ("fp8_skinny_kernel split_k=%d%s" % (split, " + fp8_splitk_reduce_kernel" if split > 1 else "")) if tile == _lib.TILE_SKINNY else \
        "fp8_strip_kernel" if tile == _lib.TILE_STRIP else "fp8_gemm_kernel tile %d split_k %d" % (tile, split)
    r = {"ms": ms, "wall_ms": wall, "tflops": flops / ms * 1e-9, "gbs": nbytes / ms * 1e-6, "bytes": nbytes, "tile": tile,
         "split_k": split, "weight_copies": copies, "kernel": kernel, "ms_min": LAST_SPREAD.get("min"), "ms_max": LAST_SPREAD.get("max")}
    if clock:
        r["clock"] = sample_clock_power(step)
    return r


def bench_mlp_chain(M, steps, warmup, hidden=2560, inter=9728, rotate_bytes=768 << 20):
    """Qwen3-4B MLP block at decode-sized M: hidden state bf16 [M, hidden] -> RMSNorm+quant -> gate_up (N = 2*inter)
    with SwiGLU output -> down (bf16 out).  Algorithmic bytes: both weight matrices once."""
    import llmmm_amd
    from llmmm_amd import _lib
    g = torch.Generator(device="cuda").manual_seed(11)
    per_copy = 3 * inter * hidden
    copies = max(2, int(np.ceil(rotate_bytes / float(per_copy))))
    weights = []
    for _ in range(copies):
        Wgu = torch.randn((2 * inter, hidden), generator=g, device="cuda") * 0.02
        Wd = torch.randn((hidden, inter), generator=g, device="cuda") * 0.02
        gq, gs = llmmm_amd.quantize_weight(Wgu)
        dq, ds = llmmm_amd.quantize_weight(Wd)
        weights.append((llmmm_amd.preshuffle_weight(gq), gs, llmmm_amd.preshuffle_weight(dq), ds))
        del Wgu, Wd, gq, dq
    x = torch.randn((M, hidden), generator=g, device="cuda").to(torch.bfloat16)
    wn = torch.ones(hidden, device="cuda")
    Aq = torch.empty((M, hidden), dtype=torch.uint8, device="cuda")
    As = torch.empty((hidden // 128, M), dtype=torch.float32, device="cuda")
    Hq = torch.empty((M, inter), dtype=torch.uint8, device="cuda")
    Hs = torch.empty((inter // 128, M), dtype=torch.float32, device="cuda")
    Y = torch.empty((M, hidden), dtype=torch.bfloat16, device="cuda")
    ws1 = llmmm_amd.make_workspace(_lib.OUT_FP8Q_SWIGLU, M, 2 * inter, hidden)
    ws2 = llmmm_amd.make_workspace(_lib.OUT_BF16, M, hidden, inter)
    state = {"i": 0}

    def step():
        gq, gs, dq, ds = weights[state["i"] % copies]
        state["i"] += 1
        rc = _lib.lib.llmmm_rmsnorm_quant_fp8(_lib.DTYPE_BF16, x.data_ptr(), wn.data_ptr(), 1e-6, Aq.data_ptr(), As.data_ptr(), M, hidden,
                                              torch.cuda.current_stream().cuda_stream)
        assert rc == 0
        llmmm_amd.fp8_gemm_blockwise_quant_A_1x128__B_128x128__swiglu__C_1x128__output_fp8(Aq, As, gq, gs, Hq, Hs, M, 2 * inter, hidden, workspace=ws1,
                                                                                           b_preshuffled=True)
        llmmm_amd.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_bf16(Hq, Hs, dq, ds, Y, M, hidden, inter, workspace=ws2, b_preshuffled=True)

    ms, _ = _events_ms(step, steps, warmup, graph=True)
    return {"name": "qwen3_4b_mlp_block_m%d" % M, "M": M, "hidden": hidden, "intermediate": inter, "us": ms * 1e3,
            "hbm_gbs": per_copy / ms * 1e-6, "frac_of_hbm_peak": per_copy / ms * 1e-6 / PEAK_HBM_GBS, "weight_copies": copies,
            "launches": "rmsnorm+quant, gate_up+swiglu (+reduce), down (+reduce)"}


def bench_proj_add_norm(name, M, steps, warmup, rotate_bytes=768 << 20):
    """A projection back to the hidden size (o or down of Qwen3-4B) with the decoder block's epilogue: residual add, the next
    RMSNorm and the 1x128 quantisation.  Timed fused (one entry point: GEMM into fp32 planes + one epilogue kernel) and as
    separate launches (GEMM with bf16 output, torch add, rmsnorm+quant)."""
    import llmmm_amd
    N, K = QWEN3_4B[name]
    copies = max(2, int(np.ceil(rotate_bytes / float(N * K)))) if M <= 128 else 1
    Aq, As, weights = fp8_inputs(M, N, K, copies=copies)
    weights = [(llmmm_amd.preshuffle_weight(bq), bs) for bq, bs in weights]
    g = torch.Generator(device="cuda").manual_seed(5)
    res = torch.randn((M, N), generator=g, device="cuda").to(torch.bfloat16)
    hid = torch.empty_like(res)
    Y = torch.empty_like(res)
    wn = torch.ones(N, device="cuda")
    ws = torch.empty(int(llmmm_amd._lib.lib.llmmm_fp8_gemm_add_rmsnorm_quant_workspace(M, N, K)), dtype=torch.uint8, device="cuda")
    ws2 = llmmm_amd.make_workspace(llmmm_amd._lib.OUT_BF16, M, N, K)
    state = {"i": 0}

    def fused():
        bq, bs = weights[state["i"] % copies]
        state["i"] += 1
        llmmm_amd.fp8_gemm_add_rmsnorm_quant(Aq, As, bq, bs, res, hid, wn, 1e-6, M, N, K, workspace=ws, b_preshuffled=True)

    def separate():
        bq, bs = weights[state["i"] % copies]
        state["i"] += 1
        llmmm_amd.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_bf16(Aq, As, bq, bs, Y, M, N, K, workspace=ws2, b_preshuffled=True)
        torch.add(Y, res, out=hid)
        llmmm_amd.rmsnorm_quantize_activation(hid, wn, 1e-6)

    ms_f, _ = _events_ms(fused, steps, warmup, graph=True)
    ms_s, _ = _events_ms(separate, steps, warmup, graph=True)
    nbytes = fp8_bytes(M, N, K, "fp8q") + 4.0 * M * N  # + residual in, hidden out (bf16 each)
    return {"name": "qwen3_4b_%s_add_rmsnorm_quant_m%d" % (name, M), "M": M, "N": N, "K": K, "us": ms_f * 1e3, "us_separate_launches": ms_s * 1e3,
            "hbm_gbs": nbytes / ms_f * 1e-6, "frac_of_hbm_peak": nbytes / ms_f * 1e-6 / PEAK_HBM_GBS, "tflops": 2.0 * M * N * K / ms_f * 1e-9,
            "weight_copies": copies}


def bench_qkv_rope(M, steps, warmup, rotate_bytes=768 << 20):
    """The Qwen3-4B QKV projection (32 query, 8 key/value heads of 128) with per-head RMSNorm and RoPE fused behind it, bf16
    output, beside the plain bf16-output GEMM of the same shape (which still needs a norm + rope kernel after it)."""
    import llmmm_amd
    N, K = QWEN3_4B["qkv"]
    n_q, n_kv = 32, 8
    copies = max(2, int(np.ceil(rotate_bytes / float(N * K)))) if M <= 128 else 1
    Aq, As, weights = fp8_inputs(M, N, K, copies=copies)
    weights = [(llmmm_amd.preshuffle_weight(bq), bs) for bq, bs in weights]
    w = torch.ones(128, device="cuda")
    inv = 1e6 ** (-torch.arange(64, device="cuda", dtype=torch.float64) / 64)
    ang = torch.arange(4096, device="cuda", dtype=torch.float64)[:, None] * inv[None, :]
    cos, sin = torch.cos(ang).float().contiguous(), torch.sin(ang).float().contiguous()
    pos = torch.arange(M, device="cuda", dtype=torch.int32)
    ws = torch.empty(max(16, int(llmmm_amd._lib.lib.llmmm_fp8_gemm_qkv_rope_workspace(M, N, K))), dtype=torch.uint8, device="cuda")
    ws2 = llmmm_amd.make_workspace(llmmm_amd._lib.OUT_BF16, M, N, K)
    Y = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    state = {"i": 0}

    def fused():
        bq, bs = weights[state["i"] % copies]
        state["i"] += 1
        llmmm_amd.fp8_gemm_qkv_rope(Aq, As, bq, bs, w, w, 1e-6, cos, sin, pos, n_q, n_kv, M, N, K, workspace=ws, b_preshuffled=True)

    def plain():
        bq, bs = weights[state["i"] % copies]
        state["i"] += 1
        llmmm_amd.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_bf16(Aq, As, bq, bs, Y, M, N, K, workspace=ws2, b_preshuffled=True)

    ms_f, _ = _events_ms(fused, steps, warmup, graph=True)
    ms_p, _ = _events_ms(plain, steps, warmup, graph=True)
    nbytes = fp8_bytes(M, N, K, "bf16")
    return {"name": "qwen3_4b_qkv_norm_rope_m%d" % M, "M": M, "N": N, "K": K, "us": ms_f * 1e3, "us_plain_bf16_gemm": ms_p * 1e3,
            "hbm_gbs": nbytes / ms_f * 1e-6, "frac_of_hbm_peak": nbytes / ms_f * 1e-6 / PEAK_HBM_GBS, "tflops": 2.0 * M * N * K / ms_f * 1e-9,
            "weight_copies": copies}


def bench_decoder_layer(M, steps, warmup, rotate_bytes=768 << 20, consumer_side=False):
    """The GEMM side of one Qwen3-4B decoder layer at decode-sized M with no elementwise launch between the projections
    (attention is not part of this library; a fixed quantised stand-in feeds O).  Pre-shuffled weights, rotated over distinct
    copies so that they stream from HBM.  Algorithmic bytes: the four weight matrices once (100.9 MB).
      producer side: QKV + per-head RMSNorm + RoPE -> O + residual + RMSNorm + quant -> gate_up (fp32 out for M <= 4, the down
                     kernel then makes silu(gate) * up itself; SwiGLU output otherwise) -> down + residual + RMSNorm + quant
      consumer side (M <= 2): O and down stop at their fp32 planes; the next projection's kernel (gate_up; the next layer's QKV)
                     sums them, adds the residual, normalises and quantises its own operand: five kernels per layer"""
    import llmmm_amd
    from llmmm_amd import _lib
    hidden, inter, n_q, n_kv = 2560, 9728, 32, 8
    shapes = {"qkv": (6144, hidden), "o": (hidden, 4096), "gate_up": (2 * inter, hidden), "down": (hidden, inter)}
    per_copy = sum(n * k for n, k in shapes.values())
    copies = max(2, int(np.ceil(rotate_bytes / float(per_copy))))
    g = torch.Generator(device="cuda").manual_seed(13)
    weights = []
    for _ in range(copies):
        layer = {}
        for name, (n, k) in shapes.items():
            W = torch.randn((n, k), generator=g, device="cuda") * 0.02
            q, sc = llmmm_amd.quantize_weight(W)
            layer[name] = (llmmm_amd.preshuffle_weight(q), sc)
            del W, q
        weights.append(layer)
    h0 = torch.randn((M, hidden), generator=g, device="cuda").to(torch.bfloat16)
    h1, h2 = torch.empty_like(h0), torch.zeros_like(h0)
    wn = torch.ones(hidden, device="cuda")
    wh = torch.ones(128, device="cuda")
    Aq, As = llmmm_amd.rmsnorm_quantize_activation(h0, wn, 1e-6)
    attn_q, attn_s = llmmm_amd.quantize_activation(torch.randn((M, 4096), generator=g, device="cuda"))
    inv = 1e6 ** (-torch.arange(64, device="cuda", dtype=torch.float64) / 64)
    ang = torch.arange(4096, device="cuda", dtype=torch.float64)[:, None] * inv[None, :]
    cos, sin = torch.cos(ang).float().contiguous(), torch.sin(ang).float().contiguous()
    pos = torch.full((M,), 1234, device="cuda", dtype=torch.int32)
    Hq = torch.empty((M, inter), dtype=torch.uint8, device="cuda")
    Hs = torch.empty((inter // 128, M), dtype=torch.float32, device="cuda")
    G32 = torch.empty((M, 2 * inter), dtype=torch.float32, device="cuda")
    planes_o = torch.zeros((16, M, hidden), dtype=torch.float32, device="cuda")
    planes_d = torch.zeros((16, M, hidden), dtype=torch.float32, device="cuda")
    ws = torch.empty(32 << 20, dtype=torch.uint8, device="cuda")
    ws_gu = llmmm_amd.make_workspace(_lib.OUT_FP8Q_SWIGLU, M, *shapes["gate_up"])
    state = {"i": 0, "s_d": 10}

    def producer_step():
        L = weights[state["i"] % copies]
        state["i"] += 1
        llmmm_amd.fp8_gemm_qkv_rope(Aq, As, L["qkv"][0], L["qkv"][1], wh, wh, 1e-6, cos, sin, pos, n_q, n_kv, M, 6144, hidden, workspace=ws, b_preshuffled=True)
        q2, s2 = llmmm_amd.fp8_gemm_add_rmsnorm_quant(attn_q, attn_s, L["o"][0], L["o"][1], h0, h1, wn, 1e-6, M, hidden, 4096, workspace=ws, b_preshuffled=True)
        if M <= 4:
            llmmm_amd.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(q2, s2, L["gate_up"][0], L["gate_up"][1], G32, M, 2 * inter, hidden,
                                                                               b_preshuffled=True)
            llmmm_amd.fp8_gemm_add_rmsnorm_quant(G32, None, L["down"][0], L["down"][1], h1, h2, wn, 1e-6, M, hidden, inter, workspace=ws, b_preshuffled=True,
                                                 a_swiglu=True)
        else:
            llmmm_amd.fp8_gemm_blockwise_quant_A_1x128__B_128x128__swiglu__C_1x128__output_fp8(q2, s2, L["gate_up"][0], L["gate_up"][1], Hq, Hs, M, 2 * inter,
                                                                                               hidden, workspace=ws_gu, b_preshuffled=True)
            llmmm_amd.fp8_gemm_add_rmsnorm_quant(Hq, Hs, L["down"][0], L["down"][1], h1, h2, wn, 1e-6, M, hidden, inter, workspace=ws, b_preshuffled=True)

    def consumer_step():
        L = weights[state["i"] % copies]
        state["i"] += 1
        # this layer's QKV reads the previous layer's down planes (h2 = the residual they are added to, h0 = the new hidden state)
        a_qkv = llmmm_amd.PlanesRmsnorm(planes_d, state["s_d"], h2, h0, wn, 1e-6)
        llmmm_amd.fp8_gemm_qkv_rope(a_qkv, None, L["qkv"][0], L["qkv"][1], wh, wh, 1e-6, cos, sin, pos, n_q, n_kv, M, 6144, hidden, workspace=ws, b_preshuffled=True)
        _, s_o = llmmm_amd.fp8_gemm_planes(attn_q, attn_s, L["o"][0], L["o"][1], M, hidden, 4096, planes=planes_o, b_preshuffled=True)
        a_gu = llmmm_amd.PlanesRmsnorm(planes_o, s_o, h0, h1, wn, 1e-6)
        llmmm_amd.fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32(a_gu, None, L["gate_up"][0], L["gate_up"][1], G32, M, 2 * inter, hidden, b_preshuffled=True)
        _, state["s_d"] = llmmm_amd.fp8_gemm_planes(G32, None, L["down"][0], L["down"][1], M, hidden, inter, planes=planes_d, b_preshuffled=True, a_swiglu=True,
                                                   workspace=ws)

    ms, _ = _events_ms(consumer_step if consumer_side else producer_step, steps, warmup, graph=True)
    if consumer_side:
        launches = "qkv on norm(down planes + residual) +norm+rope (2 kernels), o planes (1), gate_up fp32 on norm(o planes + residual) (1), down planes on silu(gate)*up (1)"
    elif M <= 4:
        launches = "qkv+norm+rope (2 kernels), o+add+norm+quant (2), gate_up fp32 (1), down on silu(gate)*up +add+norm+quant (2)"
    else:
        launches = "qkv+norm+rope (2 kernels), o+add+norm+quant (2), gate_up+swiglu (2), down+add+norm+quant (2)"
    return {"name": "qwen3_4b_decoder_layer_gemms_m%d%s" % (M, "_consumer_side" if consumer_side else ""), "M": M, "us": ms * 1e3, "weight_bytes": per_copy,
            "hbm_gbs": per_copy / ms * 1e-6, "frac_of_hbm_peak": per_copy / ms * 1e-6 / PEAK_HBM_GBS, "weight_copies": copies,
            "launches": launches + "; attention not included"}


def measured_peaks():
    """What this GPU sustains, next to the nominal peaks: register-only MFMA loops (the counterpart of the reference's
    test_fp8_peak_work, examples/005.fp8.test.cu:19-71) on zero and on random operands, and a streaming read."""
    from llmmm_amd import _lib
    lib = _lib.lib
    sink = torch.zeros(4, device="cuda")
    out = {}
    g = torch.Generator(device="cuda").manual_seed(5)
    pats = {
        "f16": (_lib.DTYPE_F16, torch.randn(16384, generator=g, device="cuda").to(torch.float16).view(torch.uint8)),
        "bf16": (_lib.DTYPE_BF16, torch.randn(16384, generator=g, device="cuda").to(torch.bfloat16).view(torch.uint8)),
        "fp8": (_lib.PROBE_FP8, (torch.randint(0, 0x78, (32768,), generator=g, device="cuda", dtype=torch.uint8)
                                 | (torch.randint(0, 2, (32768,), generator=g, device="cuda", dtype=torch.uint8) << 7))),
    }
    wgs, iters = 1024, 2000
    for name, (kind, rnd) in pats.items():
        for label, ops in (("zero", torch.zeros(32768, dtype=torch.uint8, device="cuda")), ("random", rnd)):
            def step():
                assert lib.llmmm_probe_mfma(kind, ops.data_ptr(), sink.data_ptr(), wgs, iters, torch.cuda.current_stream().cuda_stream) == 0
            ms, _ = _events_ms(step, 10, 2, graph=False)
            out["mfma_%s_%s_operands_tflops" % (name, label)] = lib.llmmm_probe_mfma_flops(kind, wgs, iters) / ms * 1e-9
    buf = torch.empty(1 << 30, dtype=torch.uint8, device="cuda").random_(0, 255)

    def read_step():
        assert lib.llmmm_probe_hbm_read(buf.data_ptr(), buf.numel(), sink.data_ptr(), 2048, torch.cuda.current_stream().cuda_stream) == 0
    ms, _ = _events_ms(read_step, 20, 3, graph=False)
    out["hbm_read_1gib_gbs"] = buf.numel() / ms * 1e-6
    out["note"] = ("register-only v_mfma loops, 1024 workgroups x 8 waves (16x16x32 f16/bf16, 16x16x128 fp8); zero operands run at the "
                   "full clock, random operands at the power-limited one; hbm_read: 1 GiB read once, nothing written")
    return out


def bench_read_ceiling(nbytes_per_copy, workgroups, steps, warmup, rotate_bytes=768 << 20):
    """A bare streaming read (llmmm_probe_hbm_read: nothing computed, nothing written) of as many bytes as one launch of a
    decode GEMM reads weights, by as many workgroups of the same size, over rotating buffers, timed exactly like the GEMM:
    the time below which no kernel of that launch shape can get on this part."""
    from llmmm_amd import _lib
    nbytes = int(nbytes_per_copy) // 16 * 16
    copies = max(2, int(np.ceil(rotate_bytes / float(nbytes))))
    bufs = [torch.empty(nbytes, dtype=torch.uint8, device="cuda").random_(0, 255) for _ in range(copies)]
    sink = torch.zeros(4, device="cuda")
    state = {"i": 0}

    def step():
        b = bufs[state["i"] % copies]
        state["i"] += 1
        assert _lib.lib.llmmm_probe_hbm_read(b.data_ptr(), nbytes, sink.data_ptr(), workgroups, torch.cuda.current_stream().cuda_stream) == 0

    ms, _ = _events_ms(step, steps, warmup, graph=True)
    return ms


def bench_targets(steps, warmup, headline=None):
    """The three figures the metric names, each against its published peak: FP16 GEMM and FP8 fused GEMM at 4096^3 (MFMA),
    and the four Qwen3-4B projections at M = 1 and 16 with fused C quantisation (HBM; weights rotated over more copies than
    the caches hold).  The decode rows also carry the time of a bare read of the same weight bytes by the same number of
    workgroups (read_us) and the fraction of that ceiling the GEMM reaches."""
    import llmmm_amd
    from llmmm_amd import _lib
    t = {}
    if headline is None:
        x, _ = bench_fp16(4096, 4096, 4096, steps, warmup)
        headline = x
    t["fp16_4096"] = {"us": round(headline["ms"] * 1e3, 2), "tflops": round(headline["tflops"], 1), "frac": round(headline["tflops"] / PEAK_TFLOPS["f16"], 4),
                      "target": 0.75, "kernel": "fp16_gemm_kernel<f16,256,256>"}
    x = bench_fp8(4096, 4096, 4096, "fp8q", steps, warmup)
    t["fp8_fused_4096"] = {"us": round(x["ms"] * 1e3, 2), "tflops": round(x["tflops"], 1), "frac": round(x["tflops"] / PEAK_TFLOPS["fp8"], 4),
                           "target": 0.70, "kernel": "fp8_gemm_kernel<256,256,fp8q>"}
    dsteps = max(steps, 200)  # microsecond kernels: enough launches per batch for the event clock
    for name, (n, k) in QWEN3_4B.items():
        read_ms = {}
        for m in (1, 16):
            for pre in (False, True):
                x = bench_fp8(m, n, k, "fp8q", dsteps, warmup, rotate_bytes=768 << 20, preshuffled=pre)
                split = max(1, x["split_k"])
                wgs = (n // 128) * split
                if wgs not in read_ms:
                    read_ms[wgs] = bench_read_ceiling(n * k, wgs, dsteps, warmup)
                e = {"us": round(x["ms"] * 1e3, 2), "gbs": round(x["gbs"], 1), "frac": round(x["gbs"] / PEAK_HBM_GBS, 4), "target": 0.60,
                     "kernel": x["kernel"], "read_us": round(read_ms[wgs] * 1e3, 2),
                     "frac_of_read_ceiling": round(read_ms[wgs] / x["ms"], 4)}
                t["decode_%s_m%d%s" % (name, m, "_pre" if pre else "")] = e
            if name != "gate_up":
                # the same projection with bf16 output (no 1x128 groups): one launch of the column-strip kernel where the library picks it
                x = bench_fp8(m, n, k, "bf16", dsteps, warmup, rotate_bytes=768 << 20, preshuffled=True)
                wgs = n // 16 if x["tile"] == _lib.TILE_STRIP else (n // 128) * max(1, x["split_k"])
                if wgs not in read_ms:
                    read_ms[wgs] = bench_read_ceiling(n * k, wgs, dsteps, warmup)
                t["decode_%s_m%d_bf16_pre" % (name, m)] = {"us": round(x["ms"] * 1e3, 2), "gbs": round(x["gbs"], 1), "frac": round(x["gbs"] / PEAK_HBM_GBS, 4),
                                                           "target": 0.60, "kernel": x["kernel"], "read_us": round(read_ms[wgs] * 1e3, 2),
                                                           "frac_of_read_ceiling": round(read_ms[wgs] / x["ms"], 4)}
            torch.cuda.empty_cache()
    t["note"] = ("us = median of %d batches; frac = achieved / published peak (2500 TFLOP/s f16, 5000 fp8, 8000 GB/s); decode: algorithmic bytes of the "
                 "GEMM (fused C quantisation; _bf16: bf16 output) / us, _pre = weights pre-shuffled offline; read_us = bare read of the same weight bytes by the same workgroup count" % TIMED_BATCHES)
    return t


def phase_accounting(kind, M=4096, N=4096, K=4096, launches=40):
    """Where one launch of the 256 x 256 tile kernel spends its time (llmmm_probe_*_gemm_phases: the product kernel with clock
    readings at five points of every wave).  Runs `launches` instrumented launches back to back (the clocks settle), reads the
    stamps of the last one and returns per-phase times over all waves, in microseconds of the 100 MHz clock and in shader cycles."""
    import llmmm_amd
    from llmmm_amd import _lib
    lib = _lib.lib
    nbytes = lib.llmmm_probe_phases_bytes(M, N)
    stamps = torch.zeros(nbytes // 8, dtype=torch.int64, device="cuda")
    if kind == "fp8":
        Aq, As, weights = fp8_inputs(M, N, K)
        Bq, Bs = weights[0]
        C = torch.empty((M, N), dtype=torch.uint8, device="cuda")
        Cs = torch.empty((N // 128, M), dtype=torch.float32, device="cuda")

        def probe():
            assert lib.llmmm_probe_fp8_gemm_phases(Aq.data_ptr(), As.data_ptr(), Bq.data_ptr(), Bs.data_ptr(), C.data_ptr(), Cs.data_ptr(), M, N, K,
                                                   stamps.data_ptr(), nbytes, torch.cuda.current_stream().cuda_stream) == 0

        def plain():
            llmmm_amd.fp8_gemm_blockwise_quant_A_1x128__B_128x128__C_1x128__output_fp8(Aq, As, Bq, Bs, C, Cs, M, N, K, tile=_lib.TILE_256x256)
    else:
        A, B = fp16_inputs(M, N, K)
        C = torch.empty((M, N), dtype=torch.float16, device="cuda")

        def probe():
            assert lib.llmmm_probe_fp16_gemm_phases(_lib.DTYPE_F16, A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, stamps.data_ptr(), nbytes,
                                                    torch.cuda.current_stream().cuda_stream) == 0

        def plain():
            llmmm_amd.fp16_gemm(A, B, C, tile=_lib.TILE_256x256)
    ms_plain, _ = _events_ms(plain, launches, 5, graph=True)
    ms_probe, _ = _events_ms(probe, launches, 5, graph=True)
    torch.cuda.synchronize()
    rec = stamps.cpu().numpy().reshape(-1, 12).astype(np.float64)
    t = rec[:, :10].reshape(-1, 5, 2)  # [wave, point, (100 MHz ticks, shader cycles)]
    real, cyc = t[:, :, 0], t[:, :, 1]
    wait_cy, load_wait_cy = rec[:, 10], rec[:, 11]
    t0 = real[:, 0].min()
    names = ["prologue (entry -> first operands in LDS)", "K loop", "epilogue (amax / convert / staging / stores issued)", "store drain (stores acknowledged)"]
    out = {"kernel_us_uninstrumented": ms_plain * 1e3, "kernel_us_instrumented": ms_probe * 1e3, "waves": int(t.shape[0]),
           "first_wave_start_to_last_wave_end_us": (real[:, 4].max() - t0) / 100.0, "wave_start_spread_us": (real[:, 0].max() - t0) / 100.0, "phases": []}
    for p, name in enumerate(names):
        d_us = (real[:, p + 1] - real[:, p]) / 100.0
        d_cy = cyc[:, p + 1] - cyc[:, p]
        out["phases"].append({"phase": name, "us_median": float(np.median(d_us)), "us_mean": float(d_us.mean()), "us_min": float(d_us.min()), "us_max": float(d_us.max()),
                              "cycles_median": float(np.median(d_cy))})
    whole_cy = cyc[:, 4] - cyc[:, 0]
    whole_us = (real[:, 4] - real[:, 0]) / 100.0
    out["wave_lifetime_us_median"] = float(np.median(whole_us))
    out["shader_mhz_from_stamps"] = float(np.median(whole_cy / whole_us))
    loop_cy = float(np.median(cyc[:, 2] - cyc[:, 1]))
    slices = K // 128 if kind == "fp8" else K // 32
    out["k_loop_cycles_per_stage"] = loop_cy / slices
    # a SIMD holds two waves; per stage each issues 32 MFMAs of 32 cycles (fp8 16x16x128, a 128-K slice) or of 16 cycles (f16 16x16x32, K = 32)
    out["k_loop_wait_cycles_per_stage"] = float(np.median(wait_cy)) / slices
    out["k_loop_load_wait_cycles_per_stage"] = float(np.median(load_wait_cy)) / slices
    # per SIMD (its two waves are records w and w + 4 of a workgroup: waves are dealt to the four SIMDs in turn): the cycles
    # per stage in which BOTH of its waves sit in a wait cannot be read off the sums, but their minimum bounds it from above
    w8 = wait_cy.reshape(-1, 8)
    out["k_loop_wait_cycles_per_stage_less_waiting_wave_of_a_simd"] = float(np.median(np.minimum(w8[:, :4], w8[:, 4:]))) / slices
    ideal = 2048.0 if kind == "fp8" else 1024.0
    out["k_loop_ideal_cycles_per_stage"] = ideal
    out["k_loop_matrix_pipe_share"] = ideal / out["k_loop_cycles_per_stage"]
    return out


def cpu_baseline(M, N, K, rows):
    """The CPU oracle on this host's cores, bounded samples of the GPU workloads: the Kahan GEMM (the headline's
    reference, a port of test/kahan.cu:16-26) on the first `rows` rows of the FP16 workload, and beside it the
    double-accumulate loop (test/kahan.cu:48-55) and the blockwise FP8 GEMM + fused re-quantisation
    (examples/005.fp8.mm.cu:885-902, examples/005.fp8.mm.opt.cu:401-462) on a 256-row slab of the 4096^3 FP8 workload."""
    import oracle
    rng = np.random.default_rng(2)
    A = rng.standard_normal((rows, K), dtype=np.float32).astype(np.float16).astype(np.float32)
    B = (rng.standard_normal((K, N), dtype=np.float32) * 0.02).astype(np.float16).astype(np.float32)
    oracle.kahan_gemm(A[:8], B)  # warm the thread pool
    t0 = time.perf_counter()
    oracle.kahan_gemm(A, B)
    dt = time.perf_counter() - t0
    out = {"value": 2.0 * rows * N * K / dt * 1e-12, "unit": "TFLOP/s", "cores": oracle.num_threads(), "kind": "port",
           "sample": "oracle Kahan fp32 GEMM (port of test/kahan.cu:16-26) on the first %d of %d rows of the same "
                     "M=N=K=4096 fp16 workload, %.1f s" % (rows, M, dt)}
    drows = min(rows, 1024)
    t0 = time.perf_counter()
    oracle.double_gemm(A[:drows], B)
    dt2 = time.perf_counter() - t0
    srows = 256
    X = rng.standard_normal((srows, K), dtype=np.float32)
    X[:, rng.choice(K, max(1, -(-K // 100)), replace=False)] *= np.float32(20.0)
    W = rng.standard_normal((N, K), dtype=np.float32) * np.float32(0.02)
    Aq, As = oracle.quant_fp8(X, 1, True)
    Bq, Bs = oracle.quant_fp8(W, 128, False)
    t0 = time.perf_counter()
    oracle.requant_c_1x128(oracle.fp8_gemm(Aq, As, Bq, Bs, promote=128))
    dt3 = time.perf_counter() - t0
    out["others"] = [
        {"name": "double_accumulate_gemm", "value": 2.0 * drows * N * K / dt2 * 1e-12, "unit": "TFLOP/s", "cores": oracle.num_threads(), "kind": "port",
         "sample": "oracle double-accumulate GEMM (port of test/kahan.cu:48-55) on the first %d rows of the same workload, %.1f s" % (drows, dt2)},
        {"name": "fp8_blockwise_gemm_fused_quant", "value": 2.0 * srows * N * K / dt3 * 1e-12, "unit": "TFLOP/s", "cores": oracle.num_threads(), "kind": "port",
         "sample": "oracle FP8 blockwise GEMM (per-128 promotion) + 1x128 re-quantisation of C on a %d-row slab of the M=N=K=4096 FP8 workload "
                   "(A ~ N(0,1) with 1%% outlier channels, B ~ N(0,0.02)), %.1f s" % (srows, dt3)},
    ]
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=500)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default="fp16_gemm_4096",
                    help="fp16_gemm_4096 (headline) | fp16_gemm_2048x19456x2560 | fp8_gemm_fused_4096 | fp8_gemm_bf16_4096 | bf16_gemm_4096 | "
                         "decode_<qkv|o|gate_up|down>_m<M>[_bf16][_pre] (_bf16: bf16 output instead of fused C quant; _pre: weights pre-shuffled offline) | "
                         "fp16_gemm_4096_k<K> | fp8_gemm_fused_4096_k<K> (M = N = 4096 on another K) | prefill_<qkv|o|gate_up|down>_m<M> | "
                         "prefill_gate_up_swiglu_m<M> | fused_<o|down>_add_norm_m<M> | fused_qkv_rope_m<M> | layer_[consumer_]m<M> | copy_1g (counter calibration only) | "
                         "phases_fp8_4096 | phases_fp16_4096 (where a launch of the tile kernel spends its time; prints a table)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--no-shapes", action="store_true", help="skip the per-shape table")
    ap.add_argument("--no-peaks", action="store_true", help="skip the measured-peak probes")
    ap.add_argument("--no-targets", action="store_true", help="skip the compact table of the metric's three figures")
    ap.add_argument("--cpu-rows", type=int, default=4096)
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (every box has one GPU); run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    torch.cuda.set_device(0)
    import llmmm_amd  # noqa: F401  raises if libllmmm.so is missing

    w = args.workload
    M = N = K = 4096
    if w == "copy_1g":
        # Calibration aid for hardware-counter runs: a plain device copy that reads 1 GiB and writes
        # 1 GiB per step, so a counter's reading can be scaled to bytes.
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda").random_(0, 255)
        dst = torch.empty_like(src)
        ms, _ = _events_ms(lambda: dst.copy_(src), args.steps, args.warmup)
        print(json.dumps({"workload": "copy_1g", "read_bytes": 1 << 30, "write_bytes": 1 << 30, "ms_per_step": ms,
                          "gbs": 2.0 * (1 << 30) / ms * 1e-6}))
        return
    if w in ("phases_fp8_4096", "phases_fp16_4096"):
        kind = "fp8" if "fp8" in w else "fp16"
        r = phase_accounting(kind)
        print("phase accounting, %s 256 x 256 tile kernel, M = N = K = 4096 (one tile per CU, 8 waves per tile)" % ("FP8 fused-quant" if kind == "fp8" else "FP16"))
        print("kernel time per launch (HIP events, graph of back-to-back launches): %.2f us; the instrumented build: %.2f us" %
              (r["kernel_us_uninstrumented"], r["kernel_us_instrumented"]))
        print("first wave's start to last wave's end: %.2f us; wave starts spread over %.2f us; median wave lifetime %.2f us; shader clock %.0f MHz" %
              (r["first_wave_start_to_last_wave_end_us"], r["wave_start_spread_us"], r["wave_lifetime_us_median"], r["shader_mhz_from_stamps"]))
        print("%-62s %9s %9s %9s %9s %12s" % ("phase (per wave, %d waves)" % r["waves"], "median us", "mean us", "min us", "max us", "median cyc"))
        for p in r["phases"]:
            print("%-62s %9.2f %9.2f %9.2f %9.2f %12.0f" % (p["phase"], p["us_median"], p["us_mean"], p["us_min"], p["us_max"], p["cycles_median"]))
        print("K loop: %.0f cycles per stage against %.0f with the matrix pipe always busy (two waves per SIMD, 32 MFMAs each per stage): %.1f %%" %
              (r["k_loop_cycles_per_stage"], r["k_loop_ideal_cycles_per_stage"], 100 * r["k_loop_matrix_pipe_share"]))
        print("of which a wave waits %.0f cycles per stage (%.0f for its own loads to land, the rest for the other waves at the barrier);"
              % (r["k_loop_wait_cycles_per_stage"], r["k_loop_load_wait_cycles_per_stage"]))
        print("the less-waiting wave of each SIMD's pair: %.0f cycles per stage (an upper bound on the time a SIMD has no wave to issue from)"
              % r["k_loop_wait_cycles_per_stage_less_waiting_wave_of_a_simd"])
        print(json.dumps({"workload": w, **r}))
        return
    import re as _re
    mk = _re.fullmatch(r"(fp16_gemm_4096|fp8_gemm_fused_4096)_k(\d+)", w)
    if mk:  # the headline kernels on a shorter or longer K (counter runs: what scales with K and what does not)
        w, K = mk.group(1), int(mk.group(2))
    if w in ("fp16_gemm_4096", "bf16_gemm_4096"):
        dt = torch.float16 if w.startswith("fp16") else torch.bfloat16
        r, _ = bench_fp16(M, N, K, args.steps, args.warmup, dt, clock=True)
        dtype, peak = ("f16" if dt == torch.float16 else "bf16"), PEAK_TFLOPS["f16"]
        roof = {"bound": "mfma", "achieved": r["tflops"], "peak": peak, "unit": "TFLOP/s", "frac": r["tflops"] / peak, "traffic": None,
                "kernel": "fp16_gemm_kernel<%s,256,256,row-major B>" % dtype}
        value, unit = r["tflops"], "TFLOP/s"
        cfg = {"workload": "FP16 GEMM %s A~N(0,1) B~N(0,0.02) seed 2, fp32 accumulate, %s out, "
                           "single kernel, no split-K" % ("M=N=K=4096" if K == 4096 else "M=N=4096 K=%d" % K, dtype), "M": M, "N": N, "K": K}
    elif w == "fp16_gemm_2048x19456x2560":
        # 608 tiles of 256 x 256: two whole rounds of the chip and 96 tiles -- the launch of two tile shapes
        M, N, K = 2048, 19456, 2560
        r, _ = bench_fp16(M, N, K, args.steps, args.warmup, torch.float16, clock=True)
        dtype, peak = "f16", PEAK_TFLOPS["f16"]
        roof = {"bound": "mfma", "achieved": r["tflops"], "peak": peak, "unit": "TFLOP/s", "frac": r["tflops"] / peak, "traffic": None,
                "kernel": "fp16_gemm_hybrid_kernel<f16, row-major B>: 512 tiles of 256 x 256 + 192 of 128 x 256"}
        value, unit = r["tflops"], "TFLOP/s"
        cfg = {"workload": "FP16 GEMM M=2048 N=19456 K=2560 (the Qwen3-4B gate_up shape) A~N(0,1) B~N(0,0.02) seed 2, fp16 out", "M": M, "N": N, "K": K}
    elif w in ("fp8_gemm_fused_4096", "fp8_gemm_bf16_4096"):
        out = "fp8q" if "fused" in w else "bf16"
        r = bench_fp8(M, N, K, out, args.steps, args.warmup, clock=True)
        dtype, peak = "fp8", PEAK_TFLOPS["fp8"]
        roof = {"bound": "mfma", "achieved": r["tflops"], "peak": peak, "unit": "TFLOP/s", "frac": r["tflops"] / peak, "traffic": None,
                "kernel": "fp8_gemm_kernel<256,256,%s>" % out}
        value, unit = r["tflops"], "TFLOP/s"
        cfg = {"workload": "FP8 e4m3 blockwise GEMM %s (A 1x128, B 128x128 scales), output %s" % ("M=N=K=4096" if K == 4096 else "M=N=4096 K=%d" % K, out),
               "M": M, "N": N, "K": K}
    elif w.startswith("layer_"):
        import re
        mo = re.fullmatch(r"layer_(consumer_)?m(\d+)", w)
        if not mo or (mo.group(1) and int(mo.group(2)) > 2):
            print("unknown workload", w, file=sys.stderr)
            sys.exit(2)
        M = int(mo.group(2))
        x = bench_decoder_layer(M, args.steps, args.warmup, consumer_side=bool(mo.group(1)))
        N, K = 0, 0
        r = {"ms": x["us"] * 1e-3, "wall_ms": x["us"] * 1e-3, "bytes": float(x["weight_bytes"])}
        dtype = "fp8"
        roof = {"bound": "hbm", "achieved": x["hbm_gbs"], "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": x["hbm_gbs"] / PEAK_HBM_GBS, "traffic": None,
                "kernel": "fp8_skinny_kernel x 4 projections + second kernels"}
        value, unit = x["hbm_gbs"], "GB/s"
        cfg = {"workload": "GEMM side of one Qwen3-4B decoder layer at M=%d: %s; pre-shuffled weights rotated over %d copies"
                           % (M, x["launches"], x["weight_copies"]), "M": M}
    elif w.startswith("fused_"):
        import re
        mo = re.fullmatch(r"fused_(o|down)_add_norm_m(\d+)|fused_qkv_rope_m(\d+)", w)
        if not mo:
            print("unknown workload", w, file=sys.stderr)
            sys.exit(2)
        if mo.group(1):
            name, M = mo.group(1), int(mo.group(2))
            x = bench_proj_add_norm(name, M, args.steps, args.warmup)
            what = "%s projection + residual add + RMSNorm + 1x128 quantisation (bf16 hidden state)" % name
            nbytes = fp8_bytes(M, x["N"], x["K"], "fp8q") + 4.0 * M * x["N"]
        else:
            name, M = "qkv", int(mo.group(3))
            x = bench_qkv_rope(M, args.steps, args.warmup)
            what = "QKV projection + per-head RMSNorm + RoPE, bf16 output"
            nbytes = fp8_bytes(M, x["N"], x["K"], "bf16")
        N, K = x["N"], x["K"]
        r = {"ms": x["us"] * 1e-3, "wall_ms": x["us"] * 1e-3, "bytes": nbytes}
        dtype = "fp8"
        if M <= 128:
            roof = {"bound": "hbm", "achieved": x["hbm_gbs"], "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": x["hbm_gbs"] / PEAK_HBM_GBS, "traffic": None,
                    "kernel": "fp8_skinny_kernel + fused second kernel"}
            value, unit = x["hbm_gbs"], "GB/s"
        else:
            roof = {"bound": "mfma", "achieved": x["tflops"], "peak": PEAK_TFLOPS["fp8"], "unit": "TFLOP/s", "frac": x["tflops"] / PEAK_TFLOPS["fp8"],
                    "traffic": None, "kernel": "fp8_gemm_kernel with the fused epilogue"}
            value, unit = x["tflops"], "TFLOP/s"
        cfg = {"workload": "Qwen3-4B %s, M=%d N=%d K=%d, pre-shuffled weights rotated over %d copies; the same work as separate launches: %.2f us"
                           % (what, M, N, K, x["weight_copies"], x.get("us_separate_launches", x.get("us_plain_bf16_gemm", 0.0))), "M": M, "N": N, "K": K}
    elif w.startswith("decode_"):
        import re
        mo = re.fullmatch(r"decode_(qkv|o|gate_up|down)_m(\d+)(_bf16)?(_pre)?", w)
        if not mo:
            print("unknown workload", w, file=sys.stderr)
            sys.exit(2)
        name, M = mo.group(1), int(mo.group(2))
        N, K = QWEN3_4B[name]
        out = "bf16" if mo.group(3) else "fp8q"
        pre = mo.group(4) is not None
        r = bench_fp8(M, N, K, out, args.steps, args.warmup, rotate_bytes=768 << 20, preshuffled=pre)
        dtype = "fp8"
        roof = {"bound": "hbm", "achieved": r["gbs"], "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": r["gbs"] / PEAK_HBM_GBS, "traffic": None,
                "kernel": r["kernel"]}
        value, unit = r["gbs"], "GB/s"
        cfg = {"workload": "Qwen3-4B %s projection, FP8 blockwise GEMM, %s, M=%d N=%d K=%d, %s weights rotated over %d "
                           "copies" % (name, "bf16 output" if out == "bf16" else "fused C quant", M, N, K, "pre-shuffled" if pre else "row-major", r["weight_copies"]),
               "M": M, "N": N, "K": K}
    elif w.startswith("prefill_"):
        import re
        mo = re.fullmatch(r"prefill_(qkv|o|gate_up|down)(_swiglu)?_m(\d+)", w)
        if not mo or (mo.group(2) and mo.group(1) != "gate_up"):
            print("unknown workload", w, file=sys.stderr)
            sys.exit(2)
        name, M = mo.group(1), int(mo.group(3))
        N, K = QWEN3_4B[name]
        out = "swiglu" if mo.group(2) else "fp8q"
        r = bench_fp8(M, N, K, out, args.steps, args.warmup, clock=True)
        dtype, peak = "fp8", PEAK_TFLOPS["fp8"]
        roof = {"bound": "mfma", "achieved": r["tflops"], "peak": peak, "unit": "TFLOP/s", "frac": r["tflops"] / peak, "traffic": None,
                "kernel": "fp8_gemm_kernel tile %d split_k %d, output %s" % (r["tile"], r["split_k"], out)}
        value, unit = r["tflops"], "TFLOP/s"
        cfg = {"workload": "Qwen3-4B %s projection at M=%d (N=%d K=%d), FP8 blockwise GEMM, output %s" % (name, M, N, K, out), "M": M, "N": N, "K": K}
    else:
        print("unknown workload", w, file=sys.stderr)
        sys.exit(2)

    if mk:
        roof["traffic"], roof["traffic_source"] = None, "no counter summary for this workload"
    else:
        roof["traffic"], roof["traffic_source"] = measured_traffic(w)
    roof["algorithmic_bytes"] = r["bytes"]
    clk = r.get("clock") if isinstance(r, dict) else None
    if clk and clk.get("sclk_mhz") and roof["bound"] == "mfma":
        # the published peak is quoted at 2400 MHz; under the board's power limit the kernel runs at a lower clock
        roof["sclk_mhz"], roof["power_w"] = clk["sclk_mhz"], clk["power_w"]
        roof["peak_at_clock"] = roof["peak"] * clk["sclk_mhz"] / 2400.0
        roof["frac_at_clock"] = roof["achieved"] / roof["peak_at_clock"]
    line = {
        "metric": "TFLOPS (% of MI355X FP8/FP16 MFMA peak) at 4096\u00b3; HBM GB/s at M\u226416 decode",
        "value": value, "unit": unit, "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": r["ms"],
        "wall_ms_per_step": r["wall_ms"], "timing": "median of %d HIP-graph replays of `steps` launches, events per replay; min %.5f max %.5f ms per step"
        % (TIMED_BATCHES, r.get("ms_min") or r["ms"], r.get("ms_max") or r["ms"]), "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": dtype,
        "data": "synthetic", "config": cfg, "roofline": roof,
    }

    if not args.no_shapes:
        shapes = []
        s2, w2 = max(10, args.steps // 2), max(3, args.warmup // 2)
        sd = max(2 * s2, 100)  # launches per batch for the microsecond-scale kernels (M <= 128)
        if w != "fp16_gemm_4096":
            x, _ = bench_fp16(4096, 4096, 4096, s2, w2)
            shapes.append({"name": "fp16_gemm_4096", "ms": x["ms"], "tflops": x["tflops"], "frac_of_fp16_peak": x["tflops"] / PEAK_TFLOPS["f16"]})
        x, _ = bench_fp16(4096, 4096, 4096, s2, w2, torch.bfloat16)
        shapes.append({"name": "bf16_gemm_4096", "ms": x["ms"], "tflops": x["tflops"], "frac_of_fp16_peak": x["tflops"] / PEAK_TFLOPS["f16"]})
        x, _ = bench_fp16(1024, 1024, 1024, s2, w2)
        shapes.append({"name": "fp16_gemm_1024", "ms": x["ms"], "tflops": x["tflops"], "frac_of_fp16_peak": x["tflops"] / PEAK_TFLOPS["f16"]})
        x, _ = bench_fp16(1024, 1024, 1024, s2, w2, b_transposed=True)
        shapes.append({"name": "fp16_gemm_1024_bt", "ms": x["ms"], "tflops": x["tflops"], "frac_of_fp16_peak": x["tflops"] / PEAK_TFLOPS["f16"]})
        for out in ("bf16", "fp8q"):
            x = bench_fp8(4096, 4096, 4096, out, s2, w2)
            shapes.append({"name": "fp8_gemm_4096_" + out, "ms": x["ms"], "tflops": x["tflops"], "frac_of_fp8_peak": x["tflops"] / PEAK_TFLOPS["fp8"]})
        for name, (n, k) in QWEN3_4B.items():
            for m, pre in ((1, False), (1, True), (16, False), (16, True), (128, False), (128, True), (2048, False), (2048, True)):
                x = bench_fp8(m, n, k, "fp8q", sd if m <= 128 else s2, w2, rotate_bytes=(768 << 20) if m <= 128 else 0, preshuffled=pre)
                e = {"name": "qwen3_4b_%s_m%d%s" % (name, m, "_preshuffled" if pre else ""), "M": m, "N": n, "K": k, "us": x["ms"] * 1e3, "tflops": x["tflops"],
                     "frac_of_fp8_peak": x["tflops"] / PEAK_TFLOPS["fp8"], "tile": x["tile"], "split_k": x["split_k"]}
                if m <= 128:
                    e.update({"hbm_gbs": x["gbs"], "frac_of_hbm_peak": x["gbs"] / PEAK_HBM_GBS, "weight_copies": x["weight_copies"]})
                if m <= 16 and pre:
                    # the same launch on one weight copy: served from the L2 / memory-side cache instead of HBM ("hot" next to the
                    # "cold" figure above, which rotates over more copies than the caches hold)
                    xh = bench_fp8(m, n, k, "fp8q", sd, w2, rotate_bytes=0, preshuffled=True)
                    e["us_hot_cache"] = xh["ms"] * 1e3
                if m > 128 and not pre:
                    # "us" above re-reads one weight copy, which stays in the memory-side cache; in a model a layer's weights come
                    # from HBM every time: the same launch rotated over more copies than the caches hold
                    xc = bench_fp8(m, n, k, "fp8q", s2, w2, rotate_bytes=768 << 20)
                    e["us_weights_from_hbm"] = xc["ms"] * 1e3
                shapes.append(e)
                torch.cuda.empty_cache()
        # the gate_up projection with the SwiGLU activation fused in front of the C quantisation (output N/2 wide)
        n, k = QWEN3_4B["gate_up"]
        for m in (1, 16, 128, 2048):
            x = bench_fp8(m, n, k, "swiglu", sd if m <= 128 else s2, w2, rotate_bytes=(768 << 20) if m <= 128 else 0)
            e = {"name": "qwen3_4b_gate_up_swiglu_m%d" % m, "M": m, "N": n, "K": k, "us": x["ms"] * 1e3, "tflops": x["tflops"],
                 "frac_of_fp8_peak": x["tflops"] / PEAK_TFLOPS["fp8"], "tile": x["tile"], "split_k": x["split_k"]}
            if m <= 128:
                e.update({"hbm_gbs": x["gbs"], "frac_of_hbm_peak": x["gbs"] / PEAK_HBM_GBS, "weight_copies": x["weight_copies"]})
            shapes.append(e)
            torch.cuda.empty_cache()
        # RMSNorm fused in front of the activation quantiser, bf16 hidden states of the Qwen3-4B width (HBM-bound: 3 B per element)
        for m in (16, 2048, 16384):
            xh = torch.randn((m, 2560), device="cuda", dtype=torch.bfloat16)
            wn = torch.ones(2560, device="cuda")
            qh = torch.empty((m, 2560), device="cuda", dtype=torch.uint8)
            sh = torch.empty((20, m), device="cuda", dtype=torch.float32)

            def norm_step():
                rc = llmmm_amd._lib.lib.llmmm_rmsnorm_quant_fp8(llmmm_amd._lib.DTYPE_BF16, xh.data_ptr(), wn.data_ptr(), 1e-6, qh.data_ptr(),
                                                                sh.data_ptr(), m, 2560, torch.cuda.current_stream().cuda_stream)
                assert rc == 0

            ms_, _ = _events_ms(norm_step, s2, w2, graph=True)
            nb = m * 2560 * 3.0 + m * 20 * 4.0
            shapes.append({"name": "rmsnorm_quant_bf16_m%d_k2560" % m, "M": m, "K": 2560, "us": ms_ * 1e3, "hbm_gbs": nb / ms_ * 1e-6,
                           "frac_of_hbm_peak": nb / ms_ * 1e-6 / PEAK_HBM_GBS})
        # The blockwise quantiser (examples/005.fp8.mm.cu:439-563) on the 4096^2 operands of the FP8 workload: activations
        # 1x128 with transposed scales, weights 128x128.  Algorithmic bytes: 4 read + 1 written per element, plus the scales.
        xq = torch.randn((4096, 4096), device="cuda")
        qq = torch.empty((4096, 4096), device="cuda", dtype=torch.uint8)
        for qname, qm, ns in (("quant_1x128_4096x4096", 1, 32 * 4096), ("quant_128x128_4096x4096", 128, 32 * 32)):
            sq = torch.empty(ns, device="cuda")
            ms_, _ = _events_ms(lambda: llmmm_amd.fp8_blockwise_symmetric_quantization(xq, qq, sq, 4096, 4096, qm, 128, qm == 1), s2, w2, graph=True)
            nb = 4096.0 * 4096.0 * 5.0 + ns * 4.0
            shapes.append({"name": qname, "us": ms_ * 1e3, "hbm_gbs": nb / ms_ * 1e-6, "frac_of_hbm_peak": nb / ms_ * 1e-6 / PEAK_HBM_GBS})
        del xq, qq
        # One decoder MLP block as three launches: RMSNorm+quant -> gate_up GEMM with fused SwiGLU output -> down GEMM
        # (bf16 output), weights pre-shuffled and rotated over distinct copies so that they stream from HBM.
        for m in (1, 16):
            shapes.append(bench_mlp_chain(m, sd, w2))
            torch.cuda.empty_cache()
        # o / down projection + residual add + next RMSNorm + quantisation in one entry point, beside the same work as separate launches
        for name in ("o", "down"):
            for m in (1, 16, 128, 2048):
                shapes.append(bench_proj_add_norm(name, m, sd if m <= 128 else s2, w2))
                torch.cuda.empty_cache()
        # QKV projection + per-head RMSNorm + RoPE in one entry point, beside the plain bf16-output GEMM
        for m in (1, 16, 128, 2048):
            shapes.append(bench_qkv_rope(m, sd if m <= 128 else s2, w2))
            torch.cuda.empty_cache()
        # the GEMM side of a whole decoder layer through the four fused entry points
        for m, cs in ((1, False), (1, True), (2, True), (16, False)):
            shapes.append(bench_decoder_layer(m, sd, w2, consumer_side=cs))
            torch.cuda.empty_cache()
        emit_detail("shapes", {"shapes": shapes})

    if not args.no_shapes:
        # Side-by-side comparison only (never part of the product or of `value`): the vendor library behind torch.matmul
        # (hipBLASLt) on the same FP16 inputs, timed the same way.
        comp = {}
        for (m, n, k) in ((4096, 4096, 4096), (1024, 1024, 1024)):
            A, B = fp16_inputs(m, n, k)
            C = torch.empty((m, n), dtype=torch.float16, device="cuda")
            ms_, _ = _events_ms(lambda: torch.matmul(A, B, out=C), max(10, args.steps // 2), max(3, args.warmup // 2), graph=True)
            comp["torch_matmul_fp16_%d_tflops" % m] = 2.0 * m * n * k / ms_ * 1e-9
            comp["torch_matmul_fp16_%d_us" % m] = ms_ * 1e3
        # a shape whose 256 x 256 tiles end in a partly filled round (608 tiles: the two-shape launch), the two non-square shapes
        # of the reference's own test (test/fp16_mm_test.cc:98-103) and a long-K projection, beside the vendor library
        for m, n, k in ((2048, 19456, 2560), (4096, 6144, 2048), (4096, 2048, 12288), (2048, 2560, 9728)):
            A, B = fp16_inputs(m, n, k)
            C = torch.empty((m, n), dtype=torch.float16, device="cuda")
            ms_, _ = _events_ms(lambda: llmmm_amd.fp16_gemm(A, B, C), max(10, args.steps // 5), max(3, args.warmup // 5), graph=True)
            comp["fp16_gemm_%dx%dx%d_tflops" % (m, n, k)] = 2.0 * m * n * k / ms_ * 1e-9
            ms_, _ = _events_ms(lambda: torch.matmul(A, B, out=C), max(10, args.steps // 5), max(3, args.warmup // 5), graph=True)
            comp["torch_matmul_fp16_%dx%dx%d_tflops" % (m, n, k)] = 2.0 * m * n * k / ms_ * 1e-9
            del A, B, C
        try:
            # the vendor library's FP8 GEMM (one scale per tensor, bf16 out: a simpler contract than 1x128 / 128x128 blocks)
            g8 = torch.Generator(device="cuda").manual_seed(7)
            a8 = torch.randn((4096, 4096), generator=g8, device="cuda").to(torch.float8_e4m3fn)
            b8 = torch.randn((4096, 4096), generator=g8, device="cuda").to(torch.float8_e4m3fn).t()  # column-major operand
            one = torch.ones((), device="cuda")
            ms_, _ = _events_ms(lambda: torch._scaled_mm(a8, b8, scale_a=one, scale_b=one, out_dtype=torch.bfloat16), max(10, args.steps // 2),
                                max(3, args.warmup // 2), graph=True)
            comp["torch_scaled_mm_fp8_tensorwise_4096_tflops"] = 2.0 * 4096 ** 3 / ms_ * 1e-9
            comp["torch_scaled_mm_fp8_tensorwise_4096_us"] = ms_ * 1e3
        except Exception as e:  # not every build of the vendor library has the kernel
            comp["torch_scaled_mm_fp8_tensorwise_4096_tflops"] = None
            comp["torch_scaled_mm_error"] = str(e)[:160]
        comp["note"] = "hipBLASLt via torch.matmul / torch._scaled_mm, same timing method; reported for comparison only"
        emit_detail("comparison", comp)
    if not args.no_peaks:
        # the same kernel against what this very part sustains: random-operand MFMA rate / streaming read rate
        mp = measured_peaks()
        emit_detail("measured_peaks", mp)
        key = {"f16": "mfma_f16_random_operands_tflops", "bf16": "mfma_bf16_random_operands_tflops", "fp8": "mfma_fp8_random_operands_tflops"}[dtype]
        roof["peak_measured"] = mp["hbm_read_1gib_gbs"] if roof["bound"] == "hbm" else mp[key]
        roof["frac_of_measured"] = roof["achieved"] / roof["peak_measured"]
    if not args.no_cpu:
        cb = cpu_baseline(4096, 4096, 4096, args.cpu_rows)
        emit_detail("cpu_baseline_others", {"others": cb.pop("others")})
        line["cpu_baseline"] = cb
    else:
        line["cpu_baseline"] = None
    if not args.no_targets:
        # all three figures of the metric, measured in this run: the full rows (read ceilings, GB/s, kernels) go out as a
        # detail line, the final line keeps microseconds, the fraction of the published peak and the number of kernels
        tg = bench_targets(max(20, args.steps), max(3, args.warmup), headline=r if w == "fp16_gemm_4096" else None)
        emit_detail("targets", tg)
        roof["targets"] = {k: {"us": v["us"], "frac": v["frac"], "target": v["target"], "kernels": v["kernel"].count("+") + 1}
                           for k, v in tg.items() if isinstance(v, dict)}
        roof["targets_note"] = "frac = achieved / published peak (2500 TFLOP/s f16, 5000 fp8, 8000 GB/s for decode_*); _pre = pre-shuffled weights, _bf16 = bf16 output"
    # The last line of stdout is the record: strict JSON, a few KB.  Everything else was printed above it, one JSON
    # object per line, each with a "detail" key.
    print(json.dumps(_finite(line), allow_nan=False), flush=True)


if __name__ == "__main__":
    main()
