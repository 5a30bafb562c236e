"""Builds the oracle with AddressSanitizer + UBSan (host code only) and runs a driver over every
entry point: out-of-bounds block indexing or signed overflow in the restatement would abort it."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.skipif(shutil.which("gcc") is None, reason="needs gcc")
def test_oracle_under_asan_ubsan(tmp_path):
    exe = str(tmp_path / "orc_sanitize")
    src = [os.path.join(ROOT, "oracle", f) for f in ("sanitize_driver.c", "psn_oracle.c")]
    subprocess.check_call(["gcc", "-O1", "-g", "-std=c11", "-fopenmp", "-ffp-contract=off", "-fno-omit-frame-pointer",
                           "-fsanitize=address,undefined", "-fno-sanitize-recover=all", "-static-libasan", "-o", exe, *src, "-lm"])
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=1", OMP_NUM_THREADS="2")
    out = subprocess.run([exe], env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert out.returncode == 0 and "ok" in out.stdout, out.stdout
