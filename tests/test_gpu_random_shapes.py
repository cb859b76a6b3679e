"""Seeded sweep over shapes, weight distributions, codecs and batch sizes: decode is
lossless, the fused GEMV agrees with fp32, a group of two equals two launches."""
import random

import pytest
import torch

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-2, 1e-3      # the tolerance the fused GEMV is held to everywhere


def _weight(kind, M, K, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    if kind == "gauss":
        return (torch.randn(M, K, generator=g, device="cuda") * 0.02).bfloat16()
    if kind == "t3":
        torch.manual_seed(seed)
        return (torch.distributions.StudentT(3.0).sample((M, K)) * 0.0115).bfloat16().cuda()
    if kind == "bits":                       # every exponent, escapes everywhere; not meant to be multiplied
        w = torch.randint(-32768, 32767, (M, K), generator=g, device="cuda", dtype=torch.int16).view(torch.bfloat16)
        return torch.where(torch.isfinite(w.float()), w, torch.zeros_like(w))
    if kind == "wide":                       # per-row scales over many octaves
        return (torch.randn(M, K, generator=g, device="cuda")
                * torch.exp(2 * torch.randn(M, 1, generator=g, device="cuda"))).bfloat16()
    return torch.full((M, K), 0.5, device="cuda").bfloat16()


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_random_shapes(cuda, seed):
    from bf16_huffman_infer_amd.functional import ANSWeight, HuffmanWeight, NibbleWeight, linear_grouped
    from bf16_huffman_infer_amd.utils import get_block_size_n
    rng = random.Random(seed)
    widths = []
    for k in range(384, 8192 + 1, 128):
        try:
            get_block_size_n(torch.empty(1, k, device="meta"))
            widths.append(k)
        except RuntimeError:
            pass
    for it in range(25):
        K, M, bs = rng.choice(widths), 128 * rng.randint(1, 24), rng.randint(1, 8)
        kind = rng.choice(["gauss", "t3", "bits", "wide", "const"])
        cls = rng.choice([HuffmanWeight, ANSWeight, NibbleWeight])
        case = f"seed {seed} case {it}: {cls.__name__} {kind} {M}x{K} batch {bs}"
        w = _weight(kind, M, K, 100 * seed + it)
        mod = cls.compress(w).cuda()
        assert torch.equal(mod.get_weight().view(torch.int16), w.view(torch.int16)), case
        x = torch.randn(bs, K, generator=torch.Generator(device="cuda").manual_seed(it), device="cuda").bfloat16()
        y = torch.nn.functional.linear(x, mod)
        if kind != "bits":
            ref = x.float() @ w.float().T
            torch.testing.assert_close(y.float(), ref, rtol=RTOL, atol=ATOL, msg=case)
        if it % 3 == 0:
            other = cls.compress(w.flip(0).contiguous()).cuda()
            a, b = linear_grouped(x, [mod, other], [None, None])
            assert torch.equal(a.view(torch.int16), y.view(torch.int16)), case
            assert torch.equal(b.view(torch.int16), torch.nn.functional.linear(x, other).view(torch.int16)), case
