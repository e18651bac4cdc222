"""The tune tables without a GPU: the header `llmmm_amd.tune --write` renders compiles, the run-time file it writes
round-trips through its parser, and a library started with LLMMM_TUNE_FILE takes the file's entries before its
compiled-in table; shapes near a tuned one inherit its tile."""
import os
import subprocess
import sys
import textwrap

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _rows():
    skinny = [(16, 4096, 14336, 7), (127, 4096, 14336, 4)]
    tile = [(2048, 4096, 14336, 0, 1), (256, 2560, 4096, 3, 2)]
    fp16 = [(2048, 2048, 2048, 3, 1)]
    return skinny, tile, fp16


def test_rendered_header_compiles(tmp_path):
    from llmmm_amd import tune
    text = tune.render_table(*_rows())
    csrc = os.path.join(ROOT, "llmmm_amd", "csrc")
    (tmp_path / "tune_table.h").write_text(text)
    (tmp_path / "kernels.h").write_text('#include "%s"\n' % os.path.join(csrc, "kernels.h"))
    (tmp_path / "use.cpp").write_text('#include "tune_table.h"\nint n() { return (int)(sizeof(llmmm::kSkinnyTune) / sizeof(llmmm::kSkinnyTune[0]) + '
                                      'sizeof(llmmm::kTileTune) / sizeof(llmmm::kTileTune[0]) + sizeof(llmmm::kFp16TileTune) / sizeof(llmmm::kFp16TileTune[0])); }\n')
    res = subprocess.run(["hipcc", "-x", "hip", "--offload-arch=gfx950", "-fsyntax-only", "-std=c++17", "-I", str(tmp_path), str(tmp_path / "use.cpp")],
                         stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert res.returncode == 0, res.stdout
    # and the committed table is what the renderer makes of its own rows
    cur = open(os.path.join(csrc, "tune_table.h")).read()
    assert "static const SkinnyTune kSkinnyTune[]" in cur and "static const TileTune kFp16TileTune[]" in cur


def test_tune_file_round_trip_and_override(tmp_path):
    from llmmm_amd import tune
    skinny, tile, fp16 = _rows()
    text = tune.render_file(skinny, tile, fp16)
    assert tune.parse_file(text) == (skinny, tile, fp16)
    assert tune.parse_file(text + "nonsense 1 2 3\ntile 1 2\n# comment\n") == (skinny, tile, fp16)
    path = tmp_path / "tune.txt"
    path.write_text(text + "tile 128 128 128 99 1\nbogus\n")  # an unknown tile id and a stray word: ignored, with a warning
    prog = textwrap.dedent("""
        import ctypes, sys
        sys.path.insert(0, %r)
        import llmmm_amd
        from llmmm_amd import _lib
        q = lambda *a: llmmm_amd.query_config(_lib.OUT_FP8Q, *a)
        # (M = 12 and 24: beyond the sizes that run in column strips, where the split of the weight-streaming kernel shows)
        print(q(12, 4096, 14336), q(100, 4096, 14336), q(2048, 4096, 14336), q(256, 2560, 4096), q(24, 2560, 4096), q(3072, 4096, 14336)[0])
    """ % ROOT)
    env = dict(os.environ, LLMMM_TUNE_FILE=str(path))
    res = subprocess.run([sys.executable, "-c", prog], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, env=env)
    assert res.returncode == 0, res.stderr
    # file entries: split 7 up to M = 16, split 4 up to 127; the 256-row entry of the file replaces the built-in one (split 4 -> 2);
    # shapes the file does not name keep the built-in choice; M = 3072 inherits the tile tuned at M = 2048
    assert res.stdout.split("\n")[0] == "(8, 7) (8, 4) (0, 1) (3, 2) (8, 8) 0", res.stdout
    assert "not a tune entry" in res.stderr
    res = subprocess.run([sys.executable, "-c", prog], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, env=dict(os.environ, LLMMM_TUNE_FILE=""))
    assert res.returncode == 0 and "(3, 3) (8, 8)" in res.stdout, res.stdout + res.stderr


def test_shapes_near_a_tuned_one_inherit_its_tile():
    import llmmm_amd
    from llmmm_amd import _lib
    q = lambda *a: llmmm_amd.query_config(_lib.OUT_FP8Q, *a)
    assert q(2048, 19456, 2560) == (_lib.TILE_256x256, 1)
    assert q(3072, 19456, 2560)[0] == _lib.TILE_256x256      # 1.5 x the tuned M: the tuned tile, the heuristic's split
    assert q(1536, 2560, 9728)[0] == _lib.TILE_256x128       # between the entries at 1024 and 2048 (both 256 x 128)
    assert q(128, 6144, 2560)[0] == _lib.TILE_SKINNY         # M = 128 stays with its weight-streaming entry, not the tile tuned at 256
    assert q(96, 6144, 2560)[0] == _lib.TILE_SKINNY


def test_the_compiled_in_header_parses_back_to_what_renders_it():
    """--fp16-only keeps the FP8 rows of csrc/tune_table.h: parse_header must read exactly what render_table wrote."""
    import os
    from llmmm_amd import tune
    path = os.path.join(os.path.dirname(tune.__file__), "csrc", "tune_table.h")
    text = open(path).read()
    skinny, tile, fp16 = tune.parse_header(text)
    assert skinny and tile and fp16 and all(len(r) == 4 for r in skinny) and all(len(r) == 5 for r in tile + fp16)
    assert tune.render_table(skinny, tile, fp16).rstrip() == text.rstrip()


def test_entries_for_fewer_than_128_rows(tmp_path):
    """A tile entry with M < 128 names a row tail of 128 x 128 tiles for exactly that M; a weight-streaming entry whose m_max
    lies between 65 and 127 goes before the row-tail tiles that M = 128 would hand down."""
    path = tmp_path / "tune.txt"
    path.write_text("tile 80 4096 4096 3 2\ntile 128 4096 4096 3 1\ntile 72 4096 4096 0 1\nskinny 100 8192 4096 3\ntile 128 8192 4096 3 1\n")
    prog = textwrap.dedent("""
        import sys
        sys.path.insert(0, %r)
        import llmmm_amd
        from llmmm_amd import _lib
        q = lambda *a: llmmm_amd.query_config(_lib.OUT_FP8Q, *a)
        print(q(80, 4096, 4096), q(96, 4096, 4096), q(72, 4096, 4096), q(128, 4096, 4096), q(256, 4096, 4096)[0], q(90, 8192, 4096), q(110, 8192, 4096))
    """ % ROOT)
    res = subprocess.run([sys.executable, "-c", prog], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, env=dict(os.environ, LLMMM_TUNE_FILE=str(path)))
    assert res.returncode == 0, res.stderr
    # 80 rows: its own entry; 96 and 72 rows: what M = 128 hands down (the 256 x 256 entry for 72 rows cannot be a row tail);
    # 256 rows: not the 80-row entry; 90 rows of the other shape: the streaming entry, 110 rows: beyond its m_max -> tiles
    assert res.stdout.strip() == "(3, 2) (3, 1) (3, 1) (3, 1) 3 (8, 3) (3, 1)", res.stdout


def test_bad_file_entries_are_dropped_not_obeyed(tmp_path):
    """An entry whose tile does not divide its shape, and a line longer than the parser's buffer (whose tail looks like an
    entry of its own), are ignored with a warning: the shapes they name are served by the built-in table or the heuristic
    as if the file did not mention them."""
    import torch
    path = tmp_path / "tune.txt"
    long_line = "tile 128 4096 4096 3 1" + " " * 280 + "skinny 32 4096 4096 9"
    path.write_text("fp16 384 384 256 0\ntile 384 4096 4096 0 1\n" + long_line + "\nskinny 32 5120 4096 6\n")
    prog = textwrap.dedent("""
        import ctypes, sys
        sys.path.insert(0, %r)
        import llmmm_amd
        from llmmm_amd import _lib
        q = lambda *a: llmmm_amd.query_config(_lib.OUT_FP8Q, *a)
        fake = ctypes.c_void_p(0x1000)
        rc = _lib.lib.llmmm_fp16_gemm(0, fake, fake, fake, 384, 384, 256, 0, None) if not __import__("torch").cuda.is_available() else -1
        print(q(24, 4096, 4096)[1] != 9, q(384, 4096, 4096)[0] != _lib.TILE_256x256, q(24, 5120, 4096), rc)
    """ % ROOT)
    res = subprocess.run([sys.executable, "-c", prog], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, env=dict(os.environ, LLMMM_TUNE_FILE=str(path)))
    assert res.returncode == 0, res.stderr
    out = res.stdout.split()
    assert out[:2] == ["True", "True"], res.stdout
    assert "(8, 6)" in res.stdout            # the entry behind the long line is still read
    assert "line too long" in res.stderr and res.stderr.count("not a tune entry") == 2
    if not torch.cuda.is_available():
        assert out[-1] == "5", res.stdout    # the FP16 call gets as far as the launch (no device here): not "not aligned"


def test_pick_best_prefers_fewer_splits_within_the_noise():
    """Among candidates within 2 % of the fastest the driver records the one with the fewest splits (fewer fp32 planes)."""
    from llmmm_amd import tune
    assert tune.pick_best({(3, 3): 15.7, (3, 4): 15.7, (2, 8): 15.5, (0, 1): 24.0}) == (3, 3)
    assert tune.pick_best({(0, 1): 196.3, (0, 3): 194.3, (2, 1): 288.0}) == (0, 1)
    assert tune.pick_best({(3, 1): 85.0, (2, 1): 62.5, (1, 1): 66.5}) == (2, 1)          # a real difference is a real difference
    assert tune.pick_best({(8, 4): 6.65, (8, 5): 6.60, (8, 8): 7.4}) == (8, 4)
