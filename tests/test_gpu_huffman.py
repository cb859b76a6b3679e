"""HIP Huffman path against the oracle and against the original tensors (needs a GPU)."""
import numpy as np
import pytest
import torch

from helpers import (bits_of, gaussian_weight, pair_counts, random_bits_weight, special_values_weight,
                     student_t_weight)

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-2, 1e-3        # GEMV tolerance against fp32 accumulation of the same BF16 operands

MAKERS = {
    "gauss": gaussian_weight,
    "t3": student_t_weight,
    "bits": random_bits_weight,
    "special": special_values_weight,
    "zeros": lambda M, K, seed=0: torch.zeros(M, K, dtype=torch.bfloat16),
}


def _compress(w, n=None):
    from bf16_huffman_infer_amd.functional import HuffmanWeight
    return HuffmanWeight.compress(w) if n is None else HuffmanWeight.compress_split_n(w, n=n)


@pytest.mark.parametrize("kind,M,K,n", [
    ("gauss", 128, 384, None), ("gauss", 256, 512, 2), ("t3", 128, 1024, None), ("bits", 128, 384, None),
    ("special", 256, 1280, None), ("zeros", 128, 128 * 3, None), ("gauss", 1024, 4096, None),
    ("gauss", 128, 2048, 4),
])
def test_encoder_matches_oracle_and_decodes(cuda, kind, M, K, n):
    """HIP encoder == numpy encoder bit for bit; HIP decoder == original tensor."""
    from bf16_huffman_infer_amd.huffman import LUTHuffmanEncoder
    from bf16_huffman_infer_amd.utils import get_block_size_n
    from oracle import wave64
    w = MAKERS[kind](M, K, seed=3)
    mod = _compress(w, n)
    split_k = n or get_block_size_n(w)[0]
    assert tuple(mod.rem.shape) == (split_k, M, K // split_k) and mod.rem.dtype == torch.uint8
    assert tuple(mod.offsets.shape) == (split_k, M) and mod.offsets.dtype == torch.int32
    assert mod.exp.dtype == torch.int32 and mod.LUT1.numel() == 8192

    codec = LUTHuffmanEncoder()
    codec.build_lut(pair_counts(bits_of(w)))
    assert np.array_equal(codec.LUT1, mod.LUT1.numpy())
    want = wave64.encode(bits_of(w), split_k, codec.enc_table)
    assert np.array_equal(want["rem"], mod.rem.numpy())
    assert np.array_equal(want["offsets"], mod.offsets.numpy())
    assert np.array_equal(want["exp"], mod.exp.numpy())

    mod = mod.cuda()
    got = mod.get_weight()
    assert got.shape == w.shape and got.dtype == torch.bfloat16
    assert torch.equal(got.view(torch.int16).cpu(), w.view(torch.int16))


@pytest.mark.parametrize("bs", [1, 2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("kind,M,K,n", [("gauss", 256, 1024, None), ("t3", 128, 512, 2), ("bits", 128, 384, None)])
def test_fused_gemv_matches_fp32(cuda, kind, M, K, n, bs):
    w = MAKERS[kind](M, K, seed=5)
    if kind == "bits":                      # keep the reference product finite
        w = (w.float().nan_to_num(0.0, 0.0, 0.0).clamp(-1, 1)).bfloat16()
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
    bias = torch.randn(256).bfloat16()
    lin = CompressedLinear(_compress(w), torch.nn.Parameter(bias, requires_grad=False)).cuda()
    x = torch.randn(8, 5, 512).bfloat16().cuda()            # 40 rows: decode to BF16, then a dense GEMM
    y = lin(x)
    ref = torch.nn.functional.linear(x, w.cuda(), bias.cuda())
    assert y.shape == (8, 5, 256)
    torch.testing.assert_close(y.float(), ref.float(), rtol=RTOL, atol=ATOL)
    # 15 rows (matrix-core kernel) and 5 rows (GEMV): the bias is added to the BF16-rounded
    # product, as the reference's `output += bias` does, so where the two cancel the product's
    # rounding step (2**-8 of its magnitude) is what is left
    prod = x.float() @ w.cuda().float().T
    for rows in (x[:3], x[:1]):
        got = lin(rows).float()
        want = prod[:rows.shape[0]] + bias.cuda().float()
        bound = ATOL + RTOL * want.abs() + 2.0 ** -8 * prod[:rows.shape[0]].abs()
        assert ((got - want).abs() <= bound).all()


def test_ops_reject_cpu_tensors_and_big_batch(cuda):
    from bf16_huffman_infer_amd import ops
    mod = _compress(gaussian_weight(128, 384, seed=1))
    y = torch.empty(128, 384, dtype=torch.bfloat16)
    with pytest.raises((RuntimeError, NotImplementedError)):
        ops.huffman_decode(mod.rem, mod.exp, y, mod.offsets, mod.LUT1, mod.LUT2, mod.LUT3, mod.LUT4, mod.code_lengths)
    mod = mod.cuda()
    x = torch.zeros(9, 1, 384, dtype=torch.bfloat16, device="cuda")
    out = torch.empty(9, 128, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(RuntimeError, match="batch"):
        ops.gemv_bf16_huffman(mod.rem, mod.exp, x, out, mod.offsets, mod.LUT1, mod.LUT2, mod.LUT3, mod.LUT4,
                              mod.code_lengths)


@pytest.mark.parametrize("algo", ["huffman", "ans"])
@pytest.mark.parametrize("kind,M,K", [
    ("gauss", 4096, 4096), ("gauss", 4608, 3584), ("gauss", 3584, 3584), ("gauss", 18944, 3584),
    ("gauss", 3584, 18944), ("t3", 12288, 4096), ("t3", 4096, 12288),
])
def test_full_size_layers_round_trip(cuda, algo, kind, M, K):
    """The layer shapes of the benchmark configurations at full size: the decoded weight is
    the original bit for bit, and the fused GEMV agrees with a matmul on that weight."""
    from bf16_huffman_infer_amd.functional import ANSWeight, HuffmanWeight
    g = torch.Generator(device="cuda").manual_seed(M + K)
    if kind == "gauss":
        w = (torch.randn(M, K, generator=g, device="cuda") * 0.02).bfloat16()
    else:
        torch.manual_seed(M + K)
        w = (torch.distributions.StudentT(3.0).sample((M, K)) * (0.02 / 3 ** 0.5)).bfloat16().cuda()
    mod = (HuffmanWeight if algo == "huffman" else ANSWeight).compress(w).cuda()
    assert torch.equal(mod.get_weight().view(torch.int16), w.view(torch.int16))
    ratio = sum(b.numel() * b.element_size() for b in mod.buffers()) / (2 * M * K)
    # short tasks (7 steps for 4608x3584) pay the 64-bit rANS state flush per lane
    assert ratio < (0.75 if algo == "huffman" else 0.78), ratio
    from bf16_huffman_infer_amd.functional import mv_ans, mv_huffman
    for bs in range(1, 9):
        x = torch.randn(bs, K, generator=g, device="cuda").bfloat16()
        ref = x.float() @ w.float().T
        # what F.linear chooses for this shape and row count (the GEMV, or the matrix-core kernel) ...
        y = torch.nn.functional.linear(x, mod)
        torch.testing.assert_close(y.float(), ref, rtol=RTOL, atol=ATOL)
        # ... and the fused GEMV itself at every batch, which is what the reference's op is
        if algo == "huffman":
            y = mv_huffman(mod.rem, mod.exp, x, mod.offsets, mod.LUT1, mod.LUT2, mod.LUT3, mod.LUT4, mod.code_lengths)
        else:
            y = mv_ans(mod.rem, mod.exp, x, mod.offsets, mod.LUT)
        torch.testing.assert_close(y.float(), ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("algo", ["huffman", "nibble"])
def test_vocabulary_sized_weight(cuda, algo):
    """151936 rows (the lm_head of the decoder configuration): 37 984 row groups, the largest
    M of any configuration; row and byte indices go past 2**27 and 2**29."""
    from bf16_huffman_infer_amd.functional import HuffmanWeight, NibbleWeight
    M, K = 151936, 4096
    g = torch.Generator(device="cuda").manual_seed(5)
    w = (torch.randn(M, K, generator=g, device="cuda") * 0.02).bfloat16()
    mod = (HuffmanWeight if algo == "huffman" else NibbleWeight).compress(w).cuda()
    got = mod.get_weight()
    assert torch.equal(got.view(torch.int16), w.view(torch.int16))
    del got
    x = torch.randn(2, K, generator=g, device="cuda").bfloat16()
    y = torch.nn.functional.linear(x, mod)
    ref = x.float() @ w.float().T
    torch.testing.assert_close(y.float(), ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("algo", ["huffman", "ans"])
def test_long_incompressible_tasks_outrun_the_row_ring(cuda, algo):
    """128-step tasks whose exponents are uniform over 39 values: every pair costs about
    10.6 bits, lanes consume rows faster than a segment stages them, so windows have to be
    read from global memory behind the staged rows.  Decode and GEMV must not care."""
    from bf16_huffman_infer_amd.functional import ANSWeight, HuffmanWeight
    g = torch.Generator().manual_seed(21)
    M, K = 128, 16384
    exp = torch.randint(90, 129, (M, K), generator=g, dtype=torch.int32)
    rem = torch.randint(0, 256, (M, K), generator=g, dtype=torch.int32)
    bits = ((rem << 8) & 0x8000) | (rem & 0x7F) | (exp << 7)
    w = bits.to(torch.int16).view(torch.bfloat16)
    mod = (HuffmanWeight if algo == "huffman" else ANSWeight).compress_split_n(w, n=1).cuda()
    words_per_lane_step = (mod.exp.numel() - 2048) / (M // 4 * 128 * 64)
    assert words_per_lane_step > 1.05, "the input no longer outruns the ring"
    assert torch.equal(mod.get_weight().view(torch.int16).cpu(), w.view(torch.int16))
    x = torch.randn(3, K, generator=g).bfloat16().cuda()
    y = torch.nn.functional.linear(x, mod)
    ref = x.float() @ w.cuda().float().T
    torch.testing.assert_close(y.float(), ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("algo", ["huffman", "ans", "nibble"])
def test_hip_encoders_reproduce_the_format_digests(cuda, algo):
    """HIP-compressed buffers of the seeded matrices hash to the committed digests of the
    stream format (tests/golden/wave64_digests.json, written by the numpy model)."""
    import hashlib
    import importlib.util
    import json
    import os
    from bf16_huffman_infer_amd.functional import ANSWeight, HuffmanWeight, NibbleWeight
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    spec = importlib.util.spec_from_file_location("make_wave64_digests", os.path.join(here, "make_wave64_digests.py"))
    gen = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(gen)
    want = json.load(open(os.path.join(here, "wave64_digests.json")))
    sha = lambda t: hashlib.sha256(t.contiguous().cpu().numpy().tobytes()).hexdigest()
    cls = {"huffman": HuffmanWeight, "ans": ANSWeight, "nibble": NibbleWeight}[algo]
    for kind, M, K, split_k, seed in gen.CASES:
        w = MAKERS[kind](M, K, seed=seed)
        mod = cls.compress_split_n(w, n=split_k)
        ref = want[f"{kind}_{M}x{K}_split{split_k}_seed{seed}"][algo]
        assert mod.exp.numel() == ref["exp_words"]
        assert (sha(mod.rem), sha(mod.exp), sha(mod.offsets)) == (ref["rem"], ref["exp"], ref["offsets"])
        if algo == "huffman":
            assert sha(mod.LUT1) == ref["table"]
        elif algo == "nibble":
            assert str(int(mod.LUT[0])) == ref["table"]


@pytest.mark.parametrize("kind", ["gauss", "t3", "bits", "special", "zeros"])
def test_pair_histogram_shortcut_equals_the_full_histogram(cuda, kind):
    """The rank-compressed pair histogram of the converter equals a plain 65536-bin count."""
    from bf16_huffman_infer_amd.functional import HuffmanWeight
    from bf16_huffman_infer_amd.utils import split_bf16
    w = MAKERS[kind](256, 1024, seed=9)
    _, exp = split_bf16(w.cuda())
    got = HuffmanWeight._pair_counts(exp)
    assert got.dtype == torch.int64 and got.shape == (65536,)
    assert np.array_equal(got.cpu().numpy(), pair_counts(bits_of(w)))


def test_linear_with_no_rows(cuda):
    """An input without rows gives an output without rows (and launches nothing)."""
    mod = _compress(gaussian_weight(128, 1024, seed=1)).cuda()
    y = torch.nn.functional.linear(torch.empty(0, 1024, dtype=torch.bfloat16, device="cuda"), mod)
    assert y.shape == (0, 128) and y.dtype == torch.bfloat16
    y = torch.nn.functional.linear(torch.empty(2, 0, 1024, dtype=torch.bfloat16, device="cuda"), mod)
    assert y.shape == (2, 0, 128)


def test_stream_read_helper(cuda):
    """The load-only measurement kernel: reads whole 1 KB loads per wavefront, rejects bad arguments."""
    from bf16_huffman_infer_amd import _lib
    lib = _lib.load()
    buf = torch.zeros(1 << 20, dtype=torch.uint8, device="cuda")
    sink = torch.zeros(1, dtype=torch.int32, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    for nt in (0, 1):
        assert lib.bhi_stream_read(buf.data_ptr(), buf.numel(), 64, nt, sink.data_ptr(), st) == 1 << 20
        assert lib.bhi_stream_read(buf.data_ptr(), (1 << 20) - 1, 64, nt, sink.data_ptr(), st) == (1 << 20) - 64 * 1024
    assert lib.bhi_stream_read(buf.data_ptr(), 100, 64, 1, sink.data_ptr(), st) == 0          # nothing to launch
    torch.cuda.synchronize()
    assert sink.item() == 0
    assert lib.bhi_stream_read(buf.data_ptr(), buf.numel(), 6, 1, sink.data_ptr(), st) < 0
    assert lib.bhi_stream_read(None, buf.numel(), 64, 1, sink.data_ptr(), st) < 0


def test_convert_keeps_the_dense_layer_when_compression_does_not_shrink_it(cuda, capsys):
    """Weights of random bits have nothing to compress: ratio >= 1, and ``convert`` hands back the
    original ``nn.Linear`` with the reference's warning (reference functional.py:362-365, 370-373)."""
    from bf16_huffman_infer_amd.functional import convert
    lin = torch.nn.Linear(512, 256, bias=False).bfloat16()
    w = random_bits_weight(256, 512, seed=9)
    # finite values only (the output check multiplies), still 16 random bits of entropy minus the clamp
    lin.weight.data = w.float().nan_to_num(0.0, 0.0, 0.0).bfloat16()
    out = convert(lin, "probe", algo="huffman")
    text = capsys.readouterr().out
    assert out is lin and isinstance(out, torch.nn.Linear)
    assert "ratio" in text and "Fallback to regular nn.Linear" in text
