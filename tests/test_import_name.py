"""The reference's import line, unchanged, in a fresh interpreter that only has the
install location on its path (kernel_test.py:6), and -- on a GPU -- its call
(kernel_test.py:254-259)."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _fresh(code, cwd):
    env = dict(os.environ, PYTHONPATH=ROOT)
    return subprocess.run([sys.executable, "-c", code], cwd=cwd, env=env, stdout=subprocess.PIPE,
                          stderr=subprocess.STDOUT, text=True, timeout=300)


def test_import_int4matmul_in_a_fresh_interpreter(tmp_path):
    r = _fresh("import torch\nimport int4matmul\n"
               "names = ['quant_matmul', 'weight_matrix_packing'] + [f'quant_int{b}_linear_mult{s}' for b in (4, 3, 2) for s in ('', '_mtx', '_vec')]\n"
               "assert all(callable(getattr(int4matmul, n)) for n in names)\n"
               "assert type(int4matmul.quant_matmul).__name__ == 'builtin_function_or_method'\n"
               "import int4matmul as again\nassert again is int4matmul\nprint('ok', len(names))", str(tmp_path))
    assert r.returncode == 0 and r.stdout.strip().endswith("ok 11"), r.stdout


@pytest.mark.gpu
def test_reference_call_convention_in_a_fresh_interpreter(tmp_path):
    code = """
import torch
import int4matmul
import numpy as np
import sys
from oracle import oracle as O
p = O.make_problem(K=1024, S=1024, M=1, bits=4, group_size=64, seed=0)
dev = "cuda:0"
t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
matrix, states, scales, zeros = t(p["matrix"]), t(p["states"]), t(p["scales"]), t(p["zeros"])
outs = torch.zeros((1, 1, 1024), dtype=torch.float16, device=dev)
int4matmul.quant_matmul(4, outs, matrix, states, scales, zeros, 64, None)
torch.cuda.synchronize()
w32 = O.dequantize_matrix_fp32(4, p["matrix"], p["scales"], p["zeros"], 64)
err = O.max_rel_error(O.matmul_fp32(p["states"][0], w32), outs.cpu().numpy()[0])
assert err < 1e-2, err
print("ok")
"""
    r = _fresh(code, str(tmp_path))
    assert r.returncode == 0 and r.stdout.strip().endswith("ok"), r.stdout
