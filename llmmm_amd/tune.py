"""Offline auto-tune driver: measures every candidate configuration of the FP8 GEMM for a list
of shapes on the GPU at hand and writes ``csrc/tune_table.h`` (compiled into ``libllmmm.so``).

    python -m llmmm_amd.tune [--write] [--write-file PATH] [--m 1,16,128,2048] [--shape N,K ...]

The reference only hints at such an interface (``tune(N, K)`` in src/mm/fp32/impl.h:20-23, a
stub that throws).  Candidates: for M <= 128 the split-K factor of the weight-streaming kernel; for 32 < M < 128 also a
single row of 128 x 128 tiles (a row tail) and its splits; for M % 128 == 0 the MFMA tiles (M = 128 tries both); for the
FP16 / BF16 GEMM all five tiles.  Timing: HIP events around a HIP graph of back-to-back launches
that rotate over enough weight copies to defeat the caches -- at every M: in a model the weights of a
projection are never in cache when its GEMM starts, and at prefill sizes the best tile for cached weights can be
a quarter slower on cold ones (2560 x 9728 at M = 2048: 128 x 128 tiles 59.9 us cached / 84.7 cold, 256 x 128 tiles
61.3 / 62.5; every tile row re-reads the weights, and tall tiles halve the re-reads).  Without ``--write`` the table is only printed.  ``--write-file PATH`` writes the same
results as a text file that the library reads at run time when ``LLMMM_TUNE_FILE=PATH`` is set (its entries come
before the compiled-in table; no rebuild), e.g. for the projection shapes of another model: ``--shape 4096,14336``.
"""
import argparse
import os
import sys

import torch

from . import _lib, mm

QWEN3_4B = {"qkv": (6144, 2560), "o": (2560, 4096), "gate_up": (19456, 2560), "down": (2560, 9728)}
HERE = os.path.dirname(os.path.abspath(__file__))


def _time_ms(fn, iters, graph, batches=5):
    """ms per call: the median over `batches` event-bracketed batches of `iters` calls (one graph replay each when graph)."""
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    if graph:
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for _ in range(iters):
                fn()
        for _ in range(3):
            g.replay()
        batch = g.replay
    else:
        def batch():
            for _ in range(iters):
                fn()
    torch.cuda.synchronize()
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(batches)]
    for e0, e1 in ev:
        e0.record()
        batch()
        e1.record()
    torch.cuda.synchronize()
    return sorted(e0.elapsed_time(e1) for e0, e1 in ev)[batches // 2] / iters


def _inputs(M, N, K, copies):
    g = torch.Generator(device="cuda").manual_seed(1)
    X = torch.randn((M, K), generator=g, device="cuda")
    Aq, As = mm.quantize_activation(X)
    weights = []
    for _ in range(copies):
        W = torch.randn((N, K), generator=g, device="cuda") * 0.02
        weights.append(mm.quantize_weight(W))
        del W
    return Aq, As, weights


def tune_shape(M, N, K, iters=40, rotate_bytes=768 << 20, verbose=True):
    """Returns (best_tile, best_split, {candidate: ms})."""
    skinny = M <= 128
    copies = max(2, -(-rotate_bytes // (N * K)))
    Aq, As, weights = _inputs(M, N, K, copies)
    Cq = torch.empty((M, N), dtype=torch.uint8, device="cuda")
    Cs = torch.empty((N // 128, M), dtype=torch.float32, device="cuda")
    kb = K // 128
    tile_splits = [x for x in (1, 2, 3, 4, 5, 6, 8) if x <= max(1, kb // 2)]
    max_split = min(32, kb) if skinny else max(tile_splits)
    ws = torch.empty(max_split * M * N * 4, dtype=torch.uint8, device="cuda")  # partial planes
    cands = []
    if skinny:
        kb = K // 128
        cands = [(_lib.TILE_SKINNY, s) for s in sorted({1, 2, 3, 4, 5, 6, 8, 10, 12, 16, 19, 20, 24, 32, kb, kb // 2}) if 1 <= s <= min(32, kb)]
    if 32 < M < 128:  # a single row of 128 x 128 tiles whose last rows are not stored
        cands += [(_lib.TILE_128x128, x) for x in tile_splits if x == 1 or (N // 128) * x <= 640]
    if M % 128 == 0:
        dims = {_lib.TILE_256x256: (256, 256), _lib.TILE_128x256: (128, 256), _lib.TILE_256x128: (256, 128), _lib.TILE_128x128: (128, 128)}
        cands = (cands if skinny else []) + [(t, x) for t, (bm, bn) in dims.items() if M % bm == 0 and N % bn == 0
                                                          for x in tile_splits if x == 1 or (M // bm) * (N // bn) * x <= 640]
    results = {}
    for tile, split in cands:
        state = {"i": 0}

        def step():
            Bq, Bs = weights[state["i"] % copies]
            state["i"] += 1
            mm.fp8_gemm_blockwise_quant_A_1x128__B_128x128__C_1x128__output_fp8(Aq, As, Bq, Bs, Cq, Cs, M, N, K, workspace=ws, tile=tile,
                                                                                split_k=split)
        results[(tile, split)] = _time_ms(step, iters, graph=True)
    best = pick_best(results)
    if verbose:
        print("M=%d N=%d K=%d:" % (M, N, K), " ".join("%s/%d:%.1fus" % (t, s, v * 1e3) for (t, s), v in sorted(results.items())),
              "-> best", best, flush=True)
    return best[0], best[1], results


def pick_best(results, tolerance=0.02):
    """The candidate to record: among those within `tolerance` of the fastest (run-to-run noise), the one with the fewest
    splits -- fewer fp32 planes in the workspace -- and then the fastest."""
    floor = min(results.values())
    near = [c for c, v in results.items() if v <= floor * (1.0 + tolerance)]
    return min(near, key=lambda c: (c[1], results[c]))


FP16_SHAPES = [(1024, 1024, 1024), (2048, 2048, 2048), (4096, 4096, 4096), (4096, 6144, 2048), (4096, 2048, 12288), (2048, 19456, 2560),
               (2048, 2560, 9728)]  # the benchmark shapes, those of test/fp16_mm_test.cc:96-103 and two Qwen3-4B prefill projections
FP16_TILES = {_lib.TILE_256x256: (256, 256), _lib.TILE_128x256: (128, 256), _lib.TILE_256x128: (256, 128), _lib.TILE_128x128: (128, 128),
              _lib.TILE_64x128: (64, 128)}


def tune_fp16_shape(M, N, K, iters=40, dtype=torch.float16, verbose=True):
    """The FP16 / BF16 GEMM's tile for one shape: (best_tile, {tile: ms}) over the tiles that divide it."""
    g = torch.Generator(device="cuda").manual_seed(2)
    A = torch.randn((M, K), generator=g, device="cuda").to(dtype)
    B = (torch.randn((K, N), generator=g, device="cuda") * 0.02).to(dtype)
    C = torch.empty((M, N), dtype=dtype, device="cuda")
    results = {}
    for tile, (bm, bn) in FP16_TILES.items():
        if M % bm or N % bn:
            continue
        results[tile] = _time_ms(lambda: mm.fp16_gemm(A, B, C, tile=tile), iters, graph=True)
    best = min(results, key=results.get)
    if verbose:
        print("fp16 M=%d N=%d K=%d:" % (M, N, K), " ".join("%d:%.1fus" % (t, v * 1e3) for t, v in sorted(results.items())), "-> best", best, flush=True)
    return best, results


def render_table(skinny_rows, tile_rows, fp16_rows):
    out = ["// Offline auto-tune results, compiled in.  Regenerate with `python -m llmmm_amd.tune --write` on an",
           "// MI355X; shapes that are not listed fall back to the heuristics in capi.cpp.",
           "// (The reference only sketches this interface: `tune(N, K)` in src/mm/fp32/impl.h:20-23.)",
           "#pragma once", '#include "kernels.h"', "", "namespace llmmm {", "",
           "struct SkinnyTune {", "  int m_max;  // entry applies to M <= m_max (entries are ordered by m_max per shape)", "  int N, K;", "  int split_k;", "};",
           "struct TileTune {", "  int M, N, K;", "  int tile;", "  int split_k;  // 0 = heuristic", "};", "",
           "// FP8 weight-streaming kernel (M <= 128).", "static const SkinnyTune kSkinnyTune[] = {"]
    out += ["  {%d, %d, %d, %d}," % r for r in skinny_rows]
    out += ["};", "", "// FP8 MFMA tile kernels (M % 128 == 0).", "static const TileTune kTileTune[] = {"]
    out += ["  {%d, %d, %d, %d, %d}," % r for r in tile_rows]
    out += ["};", "", "// FP16/BF16 MFMA tile kernels.", "static const TileTune kFp16TileTune[] = {"]
    out += ["  {%d, %d, %d, %d, %d}," % r for r in fp16_rows]
    out += ["};", "", "}  // namespace llmmm", ""]
    return "\n".join(out)


def render_file(skinny_rows, tile_rows, fp16_rows):
    """The run-time form of the table (LLMMM_TUNE_FILE): one entry per line, '#' comments."""
    out = ["# llmmm tune file: entries override the table compiled into libllmmm.so (set LLMMM_TUNE_FILE to this path)",
           "# skinny <m_max> <N> <K> <split_k> | tile <M> <N> <K> <tile id> <split_k> | fp16 <M> <N> <K> <tile id>"]
    out += ["skinny %d %d %d %d" % r for r in skinny_rows]
    out += ["tile %d %d %d %d %d" % r for r in tile_rows]
    out += ["fp16 %d %d %d %d" % r[:4] for r in fp16_rows]
    return "\n".join(out) + "\n"


def parse_header(text):
    """The rows of a rendered tune_table.h: (skinny_rows, tile_rows, fp16_rows)."""
    import re
    out = {"kSkinnyTune": [], "kTileTune": [], "kFp16TileTune": []}
    for name in out:
        body = re.search(r"%s\[\] = \{(.*?)\};" % name, text, re.S)
        if body:
            out[name] = [tuple(int(v) for v in row.split(",")) for row in re.findall(r"\{([-\d, ]+)\}", body.group(1))]
    return out["kSkinnyTune"], out["kTileTune"], out["kFp16TileTune"]


def parse_file(text):
    """Inverse of render_file: (skinny_rows, tile_rows, fp16_rows); lines that are not entries are skipped, as the library does."""
    skinny, tile, fp16 = [], [], []
    for line in text.splitlines():
        f = line.split("#", 1)[0].split()
        try:
            if len(f) == 5 and f[0] == "skinny":
                skinny.append(tuple(int(x) for x in f[1:]))
            elif len(f) == 6 and f[0] == "tile":
                tile.append(tuple(int(x) for x in f[1:]))
            elif len(f) == 5 and f[0] == "fp16":
                fp16.append(tuple(int(x) for x in f[1:]) + (1,))
        except ValueError:
            pass
    return skinny, tile, fp16


def merge_rows(base, additions):
    """base and every element of additions: (skinny_rows, tile_rows, fp16_rows).  Rows are keyed by (m_max | M, N, K); a later
    row replaces an earlier one with the same key.  Weight-streaming rows come out ordered by (N, K, m_max), as the lookup
    (first entry with M <= m_max) needs them; the other tables keep their order, new keys behind the old ones."""
    out = []
    for idx in range(3):
        rows = {}
        for src in [base] + list(additions):
            for r in src[idx]:
                rows[tuple(r[:3])] = tuple(r)
        vals = list(rows.values())
        if idx == 0:
            vals.sort(key=lambda r: (r[1], r[2], r[0]))
        out.append(vals)
    return tuple(out)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--write", action="store_true", help="rewrite csrc/tune_table.h with the results")
    ap.add_argument("--m", default="1,16,32,64,96,128,256,512,1024,2048")
    ap.add_argument("--iters", type=int, default=40)
    ap.add_argument("--write-file", metavar="PATH", help="write the results as a run-time tune file (LLMMM_TUNE_FILE)")
    ap.add_argument("--shape", action="append", metavar="N,K", help="tune this weight shape instead of the Qwen3-4B projections (repeatable)")
    ap.add_argument("--fp16-shape", action="append", metavar="M,N,K", help="tune the FP16 / BF16 GEMM's tile for this shape instead of the built-in list (repeatable)")
    ap.add_argument("--fp16-only", action="store_true", help="tune only the FP16 / BF16 shapes (the FP8 rows keep the compiled-in values)")
    ap.add_argument("--merge-file", metavar="PATH", action="append",
                    help="no measurement: merge the entries of this tune file (as --write-file wrote it; repeatable) into csrc/tune_table.h, "
                         "an entry of the file replacing the table's entry for the same key")
    args = ap.parse_args()
    if args.merge_file:
        path = os.path.join(HERE, "csrc", "tune_table.h")
        merged = merge_rows(parse_header(open(path).read()), [parse_file(open(f).read()) for f in args.merge_file])
        with open(path, "w") as f:
            f.write(render_table(*merged))
        print("merged %s into csrc/tune_table.h -- rebuild with `python llmmm_amd/build.py`" % ", ".join(args.merge_file), file=sys.stderr)
        return
    torch.cuda.set_device(0)
    ms = [int(x) for x in args.m.split(",")]
    shapes = QWEN3_4B
    if args.shape:
        shapes = {"%sx%s" % tuple(x.split(",")): tuple(int(v) for v in x.split(",")) for x in args.shape}
    skinny_rows, tile_rows = [], ([] if args.shape else [(4096, 4096, 4096, _lib.TILE_256x256, 1)])
    if args.fp16_only:
        skinny_rows, tile_rows, _ = parse_header(open(os.path.join(HERE, "csrc", "tune_table.h")).read())
        shapes = {}
    for name, (N, K) in shapes.items():
        for M in ms:
            tile, split, _ = tune_shape(M, N, K, iters=args.iters)
            if tile == _lib.TILE_SKINNY:
                skinny_rows.append((M, N, K, split))  # speaks for every M up to this one that no smaller entry covers
            else:
                tile_rows.append((M, N, K, tile, split))
            torch.cuda.empty_cache()
    skinny_rows.sort(key=lambda r: (r[1], r[2], r[0]))
    fp16_shapes = [tuple(int(v) for v in x.split(",")) for x in args.fp16_shape] if args.fp16_shape else ([] if args.shape else FP16_SHAPES)
    fp16_rows = [(M, N, K, tune_fp16_shape(M, N, K, iters=args.iters)[0], 1) for M, N, K in fp16_shapes]
    text = render_table(skinny_rows, tile_rows, fp16_rows)
    print(text)
    if args.write_file:
        with open(args.write_file, "w") as f:
            f.write(render_file(skinny_rows, tile_rows, fp16_rows))
        print("wrote %s -- use it with LLMMM_TUNE_FILE=%s" % (args.write_file, args.write_file), file=sys.stderr)
    if args.write and not args.shape:
        with open(os.path.join(HERE, "csrc", "tune_table.h"), "w") as f:
            f.write(text)
        print("wrote csrc/tune_table.h -- rebuild with `python llmmm_amd/build.py`", file=sys.stderr)


if __name__ == "__main__":
    main()
