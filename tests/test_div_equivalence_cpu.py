"""Builds and runs tests/div_equivalence.c: the exhaustive host proof that the two-operation quotient
of the quantize kernels' fast path, fma(x, k1, x * k2), always has the E2M1 code of the IEEE
quotient x / s the reference rounds (src/quantization/quant_ops.py:57-71), for every divisor
mantissa (NVFP4), for the MXFP4 constants k1 = 0.75, k2 = -1.5 * 2^-26 over every x, and that
a / 6 by Markstein's correction is correctly rounded and equals the reference's fl(fl(2a)/12)."""
import os
import re
import shutil
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.mark.skipif(shutil.which("gcc") is None, reason="needs gcc")
def test_fast_path_quotient_has_the_code_of_the_ieee_quotient(tmp_path):
    exe = str(tmp_path / "div_equivalence")
    subprocess.check_call(["gcc", "-O2", "-mfma", "-ffp-contract=off", "-fopenmp",
                           os.path.join(HERE, "div_equivalence.c"), "-o", exe, "-lm"])
    run = subprocess.run([exe], capture_output=True, text=True, timeout=600)
    out = run.stdout
    assert run.returncode == 0, out
    nv = re.search(r"nv: (\d+) comparisons, (\d+) code mismatches, largest distance to the IEEE quotient (\d+) ulp", out)
    mx = re.search(r"mx: (\d+) comparisons, (\d+) code mismatches, largest distance to the IEEE quotient (\d+) ulp", out)
    d6 = re.search(r"div6: (\d+) wrong Markstein quotients, (\d+) differences", out)
    assert int(nv.group(1)) == (1 << 23) * 7 * 17 and int(nv.group(2)) == 0 and int(nv.group(3)) <= 2
    assert int(mx.group(1)) > 60_000_000 and int(mx.group(2)) == 0 and int(mx.group(3)) <= 2
    assert int(d6.group(1)) == 0 and int(d6.group(2)) == 0
