"""RMSNorm and SiLU*mul in front of the grouped GEMV, and the residual behind it (needs a GPU):
fused == this package's unfused kernels + plain GEMV, bit for bit; both close to PyTorch's ops."""
import pytest
import torch
import torch.nn.functional as F

from helpers import gaussian_weight, student_t_weight

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-2, 1e-3


def _cls(algo):
    from bf16_huffman_infer_amd.functional import ANSWeight, HuffmanWeight, NibbleWeight
    return {"huffman": HuffmanWeight, "ans": ANSWeight, "nibble": NibbleWeight}[algo]


def _bits(t):
    return t.contiguous().view(torch.int16)


@pytest.mark.parametrize("rows", [1, 2, 3, 4, 7])
def test_rms_norm_kernel_against_torch(cuda, rows):
    from bf16_huffman_infer_amd import ops
    g = torch.Generator().manual_seed(rows)
    x = (torch.randn(rows, 4096, generator=g) * 3).bfloat16().cuda()
    gamma = (1 + 0.1 * torch.randn(4096, generator=g)).bfloat16().cuda()
    got = ops.rms_norm(x, gamma, 1e-6)
    want = (x.float() * torch.rsqrt(x.float().pow(2).mean(-1, keepdim=True) + 1e-6) * gamma.float())
    # one BF16 rounding of the fp32 result: half a step of relative error
    torch.testing.assert_close(got.float(), want, rtol=2.0 ** -8, atol=1e-6)
    torch.testing.assert_close(got.float(), F.rms_norm(x, (4096,), gamma, 1e-6).float(), rtol=2.0 ** -6, atol=1e-5)


def test_silu_mul_kernel_against_torch(cuda):
    from bf16_huffman_infer_amd import ops
    g = torch.Generator().manual_seed(3)
    gate = (torch.randn(3, 12288, generator=g) * 2).bfloat16().cuda()
    up = torch.randn(3, 12288, generator=g).bfloat16().cuda()
    got = ops.silu_mul(gate, up)
    want = F.silu(gate) * up
    same = (_bits(got) == _bits(want)).float().mean().item()
    assert same > 0.999                                    # exp is evaluated differently: a rare last-place flip of the BF16 silu
    torch.testing.assert_close(got.float(), want.float(), rtol=2.0 ** -6, atol=1e-6)


@pytest.mark.parametrize("algo", ["huffman", "ans"])
@pytest.mark.parametrize("rows", [1, 2, 3, 4])
def test_norm_in_front_of_grouped_gemv(cuda, algo, rows):
    """q/k/v of a decoder layer: RMSNorm(x) * gamma, then three products -- one launch."""
    from bf16_huffman_infer_amd import ops
    from bf16_huffman_infer_amd.functional import linear_grouped
    K, Ms = 2048, (512, 128, 128)
    ws = [(gaussian_weight if i % 2 == 0 else student_t_weight)(M, K, seed=40 + i) for i, M in enumerate(Ms)]
    mods = [_cls(algo).compress(w).cuda() for w in ws]
    g = torch.Generator().manual_seed(rows)
    x = (torch.randn(rows, K, generator=g) * 2).bfloat16().cuda()
    gamma = (1 + 0.1 * torch.randn(K, generator=g)).bfloat16().cuda()
    fused = linear_grouped(x, mods, input_norm=(gamma, 1e-6))
    h = ops.rms_norm(x, gamma, 1e-6)
    unfused = linear_grouped(h, mods)
    for w, a, b in zip(ws, fused, unfused):
        assert torch.equal(_bits(a), _bits(b))
        ref = h.float() @ w.cuda().float().T
        torch.testing.assert_close(a.float(), ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("algo", ["huffman", "ans"])
@pytest.mark.parametrize("rows", [1, 4])
@pytest.mark.parametrize("M,K", [(512, 3072), (4096, 12288)])
def test_gate_product_in_front_and_residual_behind(cuda, algo, rows, M, K):
    """down_proj of a decoder layer: x + W (silu(gate) * up) -- one launch."""
    from bf16_huffman_infer_amd import ops
    from bf16_huffman_infer_amd.functional import linear_grouped
    w = gaussian_weight(M, K, seed=M)
    mod = _cls(algo).compress(w).cuda()
    g = torch.Generator().manual_seed(rows + M)
    gate = (torch.randn(rows, K, generator=g) * 1.5).bfloat16().cuda()
    up = torch.randn(rows, K, generator=g).bfloat16().cuda()
    res = torch.randn(rows, M, generator=g).bfloat16().cuda()
    fused, = linear_grouped(up, [mod], input_gate=gate, residuals=[res])
    h = ops.silu_mul(gate, up)
    plain, = linear_grouped(h, [mod])
    assert torch.equal(_bits(fused), _bits(plain + res))        # a separate BF16 addition gives the same bits
    prod = h.float() @ w.cuda().float().T
    bound = ATOL + RTOL * (prod + res.float()).abs() + 2.0 ** -8 * prod.abs()
    assert ((fused.float() - (prod + res.float())).abs() <= bound).all()


@pytest.mark.parametrize("algo", ["huffman", "nibble"])
def test_more_rows_or_other_codecs_run_the_unfused_kernels(cuda, algo):
    from bf16_huffman_infer_amd import ops
    from bf16_huffman_infer_amd.functional import linear_grouped
    K, M, rows = 1024, 256, 6
    mod = _cls(algo).compress(gaussian_weight(M, K, seed=5)).cuda()
    g = torch.Generator().manual_seed(1)
    x = torch.randn(rows, K, generator=g).bfloat16().cuda()
    gamma = (1 + 0.1 * torch.randn(K, generator=g)).bfloat16().cuda()
    a, = linear_grouped(x, [mod], input_norm=(gamma, 1e-5))
    b, = linear_grouped(ops.rms_norm(x, gamma, 1e-5), [mod])
    assert torch.equal(_bits(a), _bits(b))
    gate = torch.randn(rows, K, generator=g).bfloat16().cuda()
    a, = linear_grouped(x, [mod], input_gate=gate)
    b, = linear_grouped(ops.silu_mul(gate, x), [mod])
    assert torch.equal(_bits(a), _bits(b))
