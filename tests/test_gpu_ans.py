"""HIP rANS path against the oracle and against the original tensors (needs a GPU)."""
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
    from bf16_huffman_infer_amd.functional import ANSWeight
    return ANSWeight.compress(w) if n is None else ANSWeight.compress_split_n(w, n=n)


@pytest.mark.parametrize("kind,M,K,n", [
    ("gauss", 128, 384, None), ("gauss", 256, 512, 2), ("t3", 128, 1024, None), ("bits", 128, 384, None),
    ("special", 256, 1280, None), ("zeros", 128, 384, None), ("gauss", 1024, 4096, None), ("gauss", 128, 2048, 4),
])
def test_encoder_matches_oracle_and_decodes(cuda, kind, M, K, n):
    """HIP encoder == numpy encoder bit for bit; HIP decoder == original tensor."""
    from bf16_huffman_infer_amd.utils import get_block_size_n
    from oracle import planes, ref_tables, wave64
    w = MAKERS[kind](M, K, seed=3)
    mod = _compress(w, n)
    split_k = n or get_block_size_n(w)[0]
    assert tuple(mod.rem.shape) == (split_k, M, K // split_k) and mod.rem.dtype == torch.uint8
    assert tuple(mod.offsets.shape) == (split_k, M) and mod.offsets.dtype == torch.int32
    assert mod.exp.dtype == torch.int32 and mod.LUT.dtype == torch.int32 and mod.LUT.numel() == 256

    _, exp = planes.split_bf16(bits_of(w))
    freq, cum, lut = ref_tables.ans_tables(np.bincount(exp.reshape(-1), minlength=256), 8)
    assert np.array_equal(lut, mod.LUT.numpy())
    want = wave64.encode_ans(bits_of(w), split_k, freq, cum)
    assert np.array_equal(want["rem"], mod.rem.numpy())
    assert np.array_equal(want["offsets"], mod.offsets.numpy())
    assert np.array_equal(want["exp"], mod.exp.numpy())

    mod = mod.cuda()
    got = mod.get_weight()
    assert got.shape == w.shape and got.dtype == torch.bfloat16
    assert torch.equal(got.view(torch.int16).cpu(), w.view(torch.int16))


@pytest.mark.parametrize("bs", [1, 2, 4, 5, 8])
@pytest.mark.parametrize("kind,M,K,n", [("gauss", 256, 1024, None), ("t3", 128, 512, 2)])
def test_fused_gemv_matches_fp32(cuda, kind, M, K, n, bs):
    w = MAKERS[kind](M, K, seed=5)
    mod = _compress(w, n).cuda()
    g = torch.Generator().manual_seed(11)
    x = torch.randn(bs, K, generator=g).bfloat16().cuda()
    y = torch.nn.functional.linear(x, mod)
    assert y.shape == (bs, M) and y.dtype == torch.bfloat16
    ref = x.float() @ w.cuda().float().T
    torch.testing.assert_close(y.float(), ref, rtol=RTOL, atol=ATOL)


def test_large_batch_falls_back_to_decode_then_gemm(cuda):
    from bf16_huffman_infer_amd.functional import CompressedLinear
    w = gaussian_weight(256, 512, seed=7)
    lin = CompressedLinear(_compress(w), None).cuda()
    for rows in (12, 40):                                    # matrix-core kernel; decode to BF16 + dense GEMM
        x = torch.randn(rows, 512).bfloat16().cuda()
        torch.testing.assert_close(lin(x).float(), torch.nn.functional.linear(x, w.cuda()).float(), rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("algo", ["huffman", "ans", "smallest"])
def test_convert_picks_codec_and_is_lossless(cuda, algo):
    from bf16_huffman_infer_amd.functional import ANSWeight, CompressedLinear, HuffmanWeight, convert
    lin = torch.nn.Linear(512, 256, bias=True).bfloat16()
    with torch.no_grad():
        lin.weight.copy_(gaussian_weight(256, 512, seed=9))
    ref = lin.weight.detach().clone()
    out = convert(lin, "probe", algo=algo)
    assert isinstance(out, CompressedLinear)
    want = {"huffman": HuffmanWeight, "ans": ANSWeight}.get(algo)
    if want is not None:
        assert type(out.weight) is want
    else:
        sizes = {cls: sum(b.numel() * b.element_size() for b in cls.compress(ref).buffers())
                 for cls in (HuffmanWeight, ANSWeight)}
        assert type(out.weight) is min(sizes, key=sizes.get)
    out = out.cuda()
    assert torch.equal(out.weight.get_weight().view(torch.int16).cpu(), ref.view(torch.int16))


def test_state_dict_of_a_converted_model_loads_into_a_fresh_one(cuda):
    from bf16_huffman_infer_amd.functional import ANSWeight, HuffmanWeight, convert, load_compressed_state_dict

    def make():
        torch.manual_seed(4)
        return torch.nn.Sequential(torch.nn.Linear(512, 384, bias=True), torch.nn.SiLU(),
                                   torch.nn.Linear(384, 256, bias=False), torch.nn.LayerNorm(256)).bfloat16()

    model = make()
    with torch.no_grad():
        model[0].weight.copy_(gaussian_weight(384, 512, seed=1))
        model[2].weight.copy_(student_t_weight(256, 384, seed=2))
    x = torch.randn(3, 512).bfloat16().cuda()
    want_dense = model.cuda()(x)
    model.cpu()
    model[0] = convert(model[0], "0", algo="huffman")
    model[2] = convert(model[2], "2", algo="ans")
    assert isinstance(model[0].weight, HuffmanWeight) and isinstance(model[2].weight, ANSWeight)
    sd = {k: v.clone() for k, v in model.state_dict().items()}
    assert "0.weight.rem" in sd and "2.weight.LUT" in sd and "0.bias" in sd
    want = model.cuda()(x)

    with torch.device("meta"):
        fresh = make()
    missing = load_compressed_state_dict(fresh, sd)
    assert not missing.missing_keys and not missing.unexpected_keys
    assert isinstance(fresh[0].weight, HuffmanWeight) and isinstance(fresh[2].weight, ANSWeight)
    got = fresh.cuda()(x)
    assert torch.equal(got, want)
    torch.testing.assert_close(got.float(), want_dense.float(), rtol=5e-2, atol=5e-2)
