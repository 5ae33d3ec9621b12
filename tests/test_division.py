"""The per-token activation quantiser divides by the row scale through a reciprocal and one correction
step (gemlite_amd/csrc/actquant.hip, `div_by_row_scale`).  `division_check.c` runs that sequence against
the IEEE division for every (value, amax) pair of fp16 / bf16 inputs, for both quantisation ranges."""
import os
import shutil
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def checker(tmp_path_factory):
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc")
    exe = str(tmp_path_factory.mktemp("div") / "division_check")
    # no -ffast-math: the division and the fused multiply-adds must be the IEEE ones; -mfma so that fmaf is one instruction
    subprocess.run([gcc, "-O2", "-mfma", "-fopenmp", "-o", exe, os.path.join(HERE, "division_check.c"), "-lm"], check=True)
    return exe


@pytest.mark.parametrize("qmax", [127, 448])
@pytest.mark.parametrize("bf16", [0, 1])
def test_reciprocal_with_one_correction_equals_ieee_division(checker, bf16, qmax):
    env = dict(os.environ, OMP_NUM_THREADS=str(min(8, os.cpu_count() or 1)))
    out = subprocess.run([checker, str(bf16), str(qmax)], check=True, capture_output=True, text=True, env=env).stdout.split()
    pairs, bad = int(out[0]), int(out[1])
    assert pairs > 1_000_000_000   # about half of 65536 x 32768
    assert bad == 0
