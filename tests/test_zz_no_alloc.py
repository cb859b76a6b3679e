"""The entry point that allocates nothing (bhi_gemm_bf16_huffman_static) against the one that
takes a workspace, through the C ABI: same bits, on two calls in a row, the second smaller."""
import ctypes

import pytest
import torch

from helpers import gaussian_weight, student_t_weight

pytestmark = pytest.mark.gpu


def _member(mod, y):
    from bf16_huffman_infer_amd import _lib
    mem = (_lib.GemvMember * 1)()
    m = mem[0]
    m.A_rem, m.A_exp, m.exp_words = mod.rem.data_ptr(), mod.exp.data_ptr(), mod.exp.numel()
    m.Y, m.offsets = y.data_ptr(), mod.offsets.data_ptr()
    m.table, m.table_bytes, m.header = mod.LUT1.data_ptr(), mod.LUT1.numel(), mod.code_lengths.data_ptr()
    m.M = mod.rem.shape[1]
    return mem


def test_static_workspace_entry_matches_the_workspace_entry(cuda):
    from bf16_huffman_infer_amd import _lib
    from bf16_huffman_infer_amd.functional import HuffmanWeight
    lib = _lib.load()
    stream = torch.cuda.current_stream().cuda_stream
    cases = [(student_t_weight, 4096, 12288, 16), (gaussian_weight, 1024, 4096, 9)]      # both cut along K; the second is smaller
    for make, M, K, rows in cases:
        w = make(M, K, seed=M)
        mod = HuffmanWeight.compress(w).cuda()
        split_k, _, Ks = mod.rem.shape
        need = lib.bhi_gemm_workspace_bytes(split_k, M, Ks, rows)
        assert 0 < need <= lib.bhi_gemm_static_workspace_bytes()
        x = torch.randn(rows, K, generator=torch.Generator().manual_seed(rows)).bfloat16().cuda()
        want = torch.empty(rows, M, dtype=torch.bfloat16, device="cuda")
        ws = torch.zeros(need, dtype=torch.uint8, device="cuda")
        _lib.check(lib.bhi_gemm_bf16_huffman(_member(mod, want), x.data_ptr(), split_k, Ks, rows, ws.data_ptr(), need, stream), "gemm")
        got = torch.full_like(want, float("nan"))
        _lib.check(lib.bhi_gemm_bf16_huffman_static(_member(mod, got), x.data_ptr(), split_k, Ks, rows, stream), "gemm static")
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16))
        ref = x.float() @ w.cuda().float().T
        torch.testing.assert_close(got.float(), ref, rtol=1e-2, atol=1e-3)


def test_static_workspace_entry_rejects_what_does_not_fit(cuda):
    """6400 x 12288 (three splits of 4096 columns) at 32 rows is cut into 3 K slices: 2.46 MB of
    partial sums, more than the built-in workspace holds.  The entry point says so before it
    touches any buffer (the pointers given here are placeholders)."""
    from bf16_huffman_infer_amd import _lib
    lib = _lib.load()
    M, split_k, Ks, rows = 6400, 3, 4096, 32
    need = lib.bhi_gemm_workspace_bytes(split_k, M, Ks, rows)
    assert need > lib.bhi_gemm_static_workspace_bytes() == 1024 + (2 << 20)
    dummy = torch.zeros(4096, dtype=torch.int32, device="cuda")
    mem = (_lib.GemvMember * 1)()
    m = mem[0]
    m.A_rem = m.A_exp = m.Y = m.offsets = m.table = m.header = dummy.data_ptr()
    m.exp_words, m.table_bytes, m.M = 1 << 28, 8192, M
    rc = lib.bhi_gemm_bf16_huffman_static(mem, dummy.data_ptr(), split_k, Ks, rows, torch.cuda.current_stream().cuda_stream)
    assert rc == -1 and b"built-in workspace" in lib.bhi_last_error_string()
