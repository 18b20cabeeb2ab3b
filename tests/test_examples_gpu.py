"""The command-line examples carry the reference's switches (examples/cdist.py:5-36,
examples/cdist_grad.py:6-18, examples/build_a_kernel.py:6-14 of the reference) and
`import kermac` like the reference's own scripts: run each once at a small size, as a
user would, and check exit status and the errors they print."""
import re
import subprocess
import sys
from pathlib import Path

import pytest

pytestmark = pytest.mark.gpu

ROOT = Path(__file__).resolve().parents[1]


def run_example(name, *arguments):
    command = [sys.executable, str(ROOT / "examples" / name), *arguments]
    print(" ".join(command), flush=True)
    done = subprocess.run(command, capture_output=True, text=True, timeout=240, cwd=str(ROOT))
    print(done.stdout, flush=True)
    assert done.returncode == 0, f"{name} exited with {done.returncode}:\n{done.stderr[-2000:]}"
    return done.stdout


def numbers_after(text, label):
    found = [float(x) for x in re.findall(re.escape(label) + r"\s*([0-9.]+e[-+][0-9]+)", text)]
    assert found, f"no '{label}' in the output:\n{text}"
    return found


def test_cdist_example_with_the_reference_switches(device):
    text = run_example("cdist.py", "-m", "1000", "-n", "900", "-k", "64", "-l", "2", "-p", "1.3", "-t", "nnt",
                       "--warmup", "1", "--iters", "2")
    assert "kermac.cdist" in text and "torch.cdist" in text
    assert max(numbers_after(text, "RMSE")) < 1e-4 and max(numbers_after(text, "max abs")) < 1e-4
    assert numbers_after(text, "kermac vs float64 torch.cdist on a 512 x 512 slab: max rel err")[0] < 1e-4
    text = run_example("cdist.py", "-m", "300", "-n", "200", "-k", "33", "-l", "1", "-p", "2.0", "-s", "-a", "-d",
                       "--skip_numeric_compare", "--iters", "1")
    assert "RMSE" not in text
    text = run_example("cdist.py", "-m", "300", "-n", "200", "-k", "33", "-p", "1.0", "--skip_torch", "--iters", "1")
    assert "torch.cdist" not in text


def test_cdist_grad_example_with_the_reference_switches(device):
    text = run_example("cdist_grad.py", "-m", "300", "-n", "40", "-o", "16", "-k", "500", "-l", "2", "-p", "2.0",
                       "--warmup", "1", "--iters", "2")
    assert numbers_after(text, "Root Mean Squared Error:")[0] < 1e-4
    assert numbers_after(text, "Max Absolute Error:")[0] < 1e-3       # sums of 500 products of N(0,1) values
    assert numbers_after(text, "max abs error / mean |truth| =")[0] < 1e-4
    text = run_example("cdist_grad.py", "-m", "200", "-n", "24", "-o", "3", "-k", "300", "-l", "1", "-p", "1.0",
                       "--skip_torch_einsum")
    assert numbers_after(text, "max abs error / mean |truth| =")[0] < 1e-4
    assert "Cannot compare" in text


def test_build_a_kernel_and_broadcast_examples(device, tmp_path, monkeypatch):
    monkeypatch.setenv("KERMAC_AMD_CACHE_DIR", str(tmp_path))           # the run-time compiled descriptors
    text = run_example("build_a_kernel.py", "-m", "400", "-n", "300", "-k", "24")
    errors = numbers_after(text, "relative to max |torch|")
    assert len(errors) == 9 and max(errors) < 1e-4, errors
    text = run_example("build_a_kernel.py", "-m", "130", "-n", "70", "-k", "8", "-s", "-a")
    assert "difference to torch" not in text


def test_broadcast_kernel_example(device):
    """The reference's examples/broadcast_kernel.py: per-batch bandwidths with a regularised diagonal moved by the offsets
    3 and 1 (its result for out=None has 1 + regularization at [n + 2, n] and nowhere else), then per-batch p and
    regularization."""
    text = run_example("broadcast_kernel.py", "-n", "700", "-k", "6")
    assert "(2, 700, 700)" in text and "(4, 700, 700)" in text
    found = re.search(r"elements \[n \+ 2, n\] that hold 1 \+ regularization = 11: (\d+) of (\d+); elsewhere: (\d+)", text)
    assert found, text
    assert found.group(1) == found.group(2) == str(2 * 698) and found.group(3) == "0"
    assert numbers_after(text, "largest deviation of the diagonals from 1 + regularization:")[0] < 1e-6
