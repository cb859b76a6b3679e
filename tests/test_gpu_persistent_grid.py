"""The persistent (work-pulling) GEMV grid, which is off by default: a child process with
BHI_PERSIST=2 forces it for every batch-1 launch and checks it against fp32 products and
against the static grid's weights (needs a GPU)."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CHILD = r"""
import sys, torch
sys.path.insert(0, %(root)r); sys.path.insert(0, %(root)r + '/tests')
import torch.nn.functional as F
from helpers import gaussian_weight, student_t_weight, special_values_weight
from bf16_huffman_infer_amd.functional import ANSWeight, HuffmanWeight, linear_grouped
dev = torch.device('cuda', 0)
cases = [(gaussian_weight, 256, 1024, None), (student_t_weight, 128, 512, 2), (gaussian_weight, 4096, 4096, None),
         (special_values_weight, 256, 1280, None), (gaussian_weight, 18944, 3584, None), (gaussian_weight, 3584, 18944, None)]
for cls in (HuffmanWeight, ANSWeight):
    for make, M, K, n in cases:
        w = make(M, K, seed=5)
        if make is special_values_weight:
            w = w.float().nan_to_num(0.0, 0.0, 0.0).clamp(-1, 1).bfloat16()
        mod = (cls.compress(w) if n is None else cls.compress_split_n(w, n=n)).to(dev)
        x = torch.randn(1, K, generator=torch.Generator().manual_seed(11)).bfloat16().to(dev)
        y = F.linear(x, mod)
        ref = x.float() @ w.to(dev).float().T
        torch.testing.assert_close(y.float(), ref, rtol=1e-2, atol=1e-3)
        print('ok', cls.__name__, M, K, flush=True)
# a group of two, more tasks than resident wavefronts: units are pulled
ws = [HuffmanWeight.compress(gaussian_weight(18944, 3584, seed=s)).to(dev) for s in (1, 2)]
x = torch.randn(1, 3584, generator=torch.Generator().manual_seed(3)).bfloat16().to(dev)
for y, w in zip(linear_grouped(x, ws), ws):
    ref = x.float() @ w.get_weight().float().T
    torch.testing.assert_close(y.float(), ref, rtol=1e-2, atol=1e-3)
print('ok group', flush=True)
"""


def test_persistent_grid_matches_fp32(cuda):
    env = dict(os.environ, BHI_PERSIST="2")
    proc = subprocess.run([sys.executable, "-u", "-c", CHILD % {"root": ROOT}], env=env, capture_output=True, text=True,
                          timeout=600)
    assert proc.returncode == 0, proc.stdout[-2000:] + proc.stderr[-4000:]
    assert proc.stdout.count("ok") == 13
