"""The oracle under AddressSanitizer + UndefinedBehaviorSanitizer: every entry point on ragged shapes with buffers of
exactly the documented sizes (oracle/sanitize_check.c).  Host code only."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_oracle_is_clean_under_asan_and_ubsan():
    odir = os.path.join(ROOT, "oracle")
    res = subprocess.run(["make", "-C", odir, "-B", "sanitize_check"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert res.returncode == 0, res.stdout
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:verify_asan_link_order=0", OMP_NUM_THREADS="4")
    res = subprocess.run([os.path.join(odir, "sanitize_check")], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env, timeout=300)
    assert res.returncode == 0 and "sanitize ok" in res.stdout, res.stdout[-3000:]
