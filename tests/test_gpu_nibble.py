"""HIP nibble (fixed-width) path against the oracle and against the original tensors."""
import numpy as np
import pytest
import torch

from helpers import bits_of, gaussian_weight, random_bits_weight, special_values_weight, student_t_weight

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-2, 1e-3

MAKERS = {
    "gauss": gaussian_weight,
    "t3": student_t_weight,
    "bits": random_bits_weight,
    "special": special_values_weight,
    "zeros": lambda M, K, seed=0: torch.zeros(M, K, dtype=torch.bfloat16),
}


def _compress(w, n=None):
    from bf16_huffman_infer_amd.functional import NibbleWeight
    return NibbleWeight.compress(w) if n is None else NibbleWeight.compress_split_n(w, n=n)


@pytest.mark.parametrize("kind,M,K,n", [
    ("gauss", 128, 384, None), ("gauss", 256, 512, 2), ("t3", 128, 1024, None), ("bits", 128, 384, None),
    ("special", 256, 1280, None), ("zeros", 128, 384, None), ("gauss", 1024, 4096, None), ("gauss", 128, 2048, 4),
    ("t3", 128, 16384, 1),
])
def test_encoder_matches_oracle_and_decodes(cuda, kind, M, K, n):
    from bf16_huffman_infer_amd.utils import get_block_size_n
    from oracle import planes, wave64
    w = MAKERS[kind](M, K, seed=3)
    mod = _compress(w, n)
    split_k = n or get_block_size_n(w)[0]
    _, exp = planes.split_bf16(bits_of(w))
    base = wave64.nibble_base(np.bincount(exp.reshape(-1), minlength=256))
    assert int(mod.LUT[0]) == base and mod.LUT.dtype == torch.int32 and mod.LUT.numel() == 256
    want = wave64.encode_nibble(bits_of(w), split_k, base)
    assert np.array_equal(want["rem"], mod.rem.numpy())
    assert np.array_equal(want["offsets"], mod.offsets.numpy())
    assert np.array_equal(want["exp"], mod.exp.numpy())
    got = mod.cuda().get_weight()
    assert torch.equal(got.view(torch.int16).cpu(), w.view(torch.int16))


@pytest.mark.parametrize("bs", [1, 2, 4, 5, 8])
@pytest.mark.parametrize("kind,M,K,n", [("gauss", 256, 1024, None), ("t3", 128, 512, 2), ("special", 128, 384, None)])
def test_fused_gemv_matches_fp32(cuda, kind, M, K, n, bs):
    w = MAKERS[kind](M, K, seed=5)
    if kind == "special":
        w = (w.float().nan_to_num(0.0, 0.0, 0.0).clamp(-1, 1)).bfloat16()
    mod = _compress(w, n).cuda()
    g = torch.Generator().manual_seed(11)
    x = torch.randn(bs, K, generator=g).bfloat16().cuda()
    y = torch.nn.functional.linear(x, mod)
    ref = x.float() @ w.cuda().float().T
    torch.testing.assert_close(y.float(), ref, rtol=RTOL, atol=ATOL)


def test_convert_fallback_and_state_dict(cuda):
    from bf16_huffman_infer_amd.functional import (CompressedLinear, NibbleWeight, convert,
                                                   load_compressed_state_dict)
    lin = torch.nn.Linear(512, 256, bias=True).bfloat16()
    with torch.no_grad():
        lin.weight.copy_(gaussian_weight(256, 512, seed=9))
    ref = lin.weight.detach().clone()
    out = convert(lin, "probe", algo="nibble")
    assert isinstance(out, CompressedLinear) and type(out.weight) is NibbleWeight
    ratio = sum(b.numel() * b.element_size() for b in out.weight.buffers()) / (2 * ref.numel())
    assert ratio < 0.80
    sd = {"0." + k: v.clone() for k, v in out.state_dict().items()}
    with torch.device("meta"):
        fresh = torch.nn.Sequential(torch.nn.Linear(512, 256, bias=True)).bfloat16()
    load_compressed_state_dict(fresh, sd)
    assert type(fresh[0].weight) is NibbleWeight
    fresh.cuda()
    assert torch.equal(fresh[0].weight.get_weight().cpu().view(torch.int16), ref.view(torch.int16))
    x = torch.randn(12, 512).bfloat16().cuda()              # > 8 rows: decode + GEMM
    torch.testing.assert_close(fresh(x).float(), torch.nn.functional.linear(x, ref.cuda(), lin.bias.cuda()).float(),
                               rtol=RTOL, atol=ATOL)
