"""The command-line comparison in the shape of the reference's kernel-test.py (BATCH=1, HEADS=8, fp16, D=64;
kernel-test.py:6-8) runs and its last column, the largest absolute difference between this package's
result and the naive fp16 matmul + masked softmax on the GPU (kernel-test.py:37-40, 50-51), stays within
the fp16 bar of 2e-2."""
import importlib.util
import os

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_kernel_test_cli(dev, capsys):
    path = os.path.join(ROOT, "customize-block-sparse-attention-with-triton_amd", "kernel_test.py")
    spec = importlib.util.spec_from_file_location("kernel_test_cli", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    mod.main(["--seq-len", "6400", "--heads", "8", "--reps", "3"])
    rows = [l for l in capsys.readouterr().out.splitlines() if l.startswith("| [6400")]
    assert len(rows) == 2                                   # ratios 0.1 and 1.0
    for row in rows:
        cells = [c.strip() for c in row.strip("|").split("|")]
        assert float(cells[2]) > 0 and float(cells[3]) > 0   # seconds, including / excluding the preprocessing
        assert float(cells[6]) <= 2e-2                       # max abs diff against the naive path
