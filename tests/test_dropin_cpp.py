"""The C++ drop-in shims (include/llmmm/mm/...): they compile against the C ABI with the reference's
signatures (CPU check) and pass the reference's closed-form known-answer tests on a GPU."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "cpp", "dropin_test")


def test_shims_compile_and_link():
    from llmmm_amd import build
    out = build.build_dropin_test()
    assert os.path.exists(out)


@pytest.mark.gpu
def test_dropin_known_answers_on_gpu():
    assert os.path.exists(BIN), "tests/cpp/dropin_test has not been built (python llmmm_amd/build.py)"
    res = subprocess.run([BIN], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    print(res.stdout)
    assert res.returncode == 0 and "DROPIN OK" in res.stdout, res.stdout
