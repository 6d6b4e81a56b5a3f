"""The block estimate's three-instruction division (pbs_attn_amd/csrc/pbs_div.h) against the `/` operator, on the host,
for every bf16-representable dividend: tests/c_abi/div_check.c includes the header the kernel includes."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("head_dim", [128, 64, 256])
def test_division_by_sqrt_head_dim_equals_ieee_division_for_every_bf16_dividend(tmp_path, head_dim):
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc")
    exe = str(tmp_path / "div_check")
    # -ffp-contract=off: the reference quotient and the products must not be fused by the host compiler
    subprocess.run([gcc, "-std=c99", "-O2", "-ffp-contract=off", os.path.join(ROOT, "tests", "c_abi", "div_check.c"),
                    "-o", exe, "-lm"], check=True)
    run = subprocess.run([exe, str(head_dim)], capture_output=True, text=True)
    assert run.returncode == 0, run.stdout
    assert run.stdout.strip() == "ok 65536"
