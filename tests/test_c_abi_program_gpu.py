"""The C ABI from a program that is neither Python nor torch: examples/c_abi_cdist.cpp,
built next to the library by kermac_amd._build, computes an L1 distance matrix and a
Laplace kernel matrix through kmc_build_kernel and checks them itself against a
double-precision host loop (rtol 1e-5); its exit status is the verdict."""
import subprocess
from pathlib import Path

import pytest

pytestmark = pytest.mark.gpu

PROGRAM = Path(__file__).resolve().parents[1] / "kermac_amd" / "_lib" / "c_abi_cdist"


@pytest.mark.parametrize("shape", [(), ("130", "257", "33"), ("2048", "1500", "512")])
def test_c_program_through_the_abi(shape):
    if not PROGRAM.exists():
        pytest.fail(f"{PROGRAM} is missing: build it with `python -m kermac_amd._build`")
    done = subprocess.run([str(PROGRAM), *shape], capture_output=True, text=True, timeout=120)
    print(done.stdout, done.stderr, flush=True)
    assert done.returncode == 0, done.stdout + done.stderr
    assert "ok" in done.stdout.splitlines()[-1]
