"""Grouped launches (several weights, one X): same bits as the single launches they replace."""
import ctypes

import pytest
import torch
from torch import nn

from helpers import gaussian_weight, student_t_weight

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-2, 1e-3


def _cls(algo):
    from bf16_huffman_infer_amd.functional import ANSWeight, HuffmanWeight, NibbleWeight
    return {"huffman": HuffmanWeight, "ans": ANSWeight, "nibble": NibbleWeight}[algo]


def _linear(w, bias=None):
    lin = nn.Linear(w.shape[1], w.shape[0], bias=bias is not None)
    lin.weight.data = w.clone()
    if bias is not None:
        lin.bias.data = bias.clone()
    return lin.bfloat16()


@pytest.mark.parametrize("algo", ["huffman", "ans", "nibble"])
@pytest.mark.parametrize("bs", [1, 3, 8])
@pytest.mark.parametrize("K,Ms", [(1024, (512, 128, 128)), (2048, (256, 384)), (4096, (128, 128, 256, 1024))])
def test_grouped_equals_single_launches(cuda, algo, bs, K, Ms):
    from bf16_huffman_infer_amd.functional import linear_grouped
    ws = [(gaussian_weight if i % 2 == 0 else student_t_weight)(M, K, seed=20 + i) for i, M in enumerate(Ms)]
    mods = [_cls(algo).compress(w).cuda() for w in ws]
    biases = [None] * len(ws)
    biases[1] = torch.randn(Ms[1], generator=torch.Generator().manual_seed(2)).bfloat16().cuda()
    x = torch.randn(bs, K, generator=torch.Generator().manual_seed(7)).bfloat16().cuda()
    got = linear_grouped(x, mods, biases)
    for w, mod, b, y in zip(ws, mods, biases, got):
        single = torch.nn.functional.linear(x, mod, b)
        assert torch.equal(y.view(torch.int16), single.view(torch.int16))
        prod = x.float() @ w.cuda().float().T
        if b is None:
            torch.testing.assert_close(y.float(), prod, rtol=RTOL, atol=ATOL)
        else:
            # The bias is added to the BF16-ROUNDED product (the reference's `output += bias`,
            # functional.py:403-404): where product and bias cancel, the product's rounding
            # step (2**-8 of its magnitude) is all that is left of the result, so the bound
            # carries that step on top of the flat tolerance.
            ref = prod + b.float()
            bound = ATOL + RTOL * ref.abs() + 2.0 ** -8 * prod.abs()
            worst = ((y.float() - ref).abs() - bound).max().item()
            assert worst <= 0, f"biased member off by {worst} beyond its bound"


@pytest.mark.parametrize("algo", ["huffman", "ans"])
@pytest.mark.parametrize("bs", [5, 6, 8])
def test_group_of_layers_that_prefer_the_matrix_cores(cuda, algo, bs):
    """Two 10240x3584 weights from six rows on: every member goes through the matrix-core kernel
    (one launch each), with the bits of its own ``F.linear`` call and a bias added in the kernel;
    at five rows the group stays one GEMV launch."""
    from bf16_huffman_infer_amd.functional import linear_grouped, prefers_matrix_cores
    assert prefers_matrix_cores(6, 10240, 3584) and not prefers_matrix_cores(5, 10240, 3584)
    M, K = 10240, 3584
    ws = [gaussian_weight(M, K, seed=41).cuda(), student_t_weight(M, K, seed=42).cuda()]
    mods = [_cls(algo).compress(w).cuda() for w in ws]
    biases = [None, torch.randn(M, generator=torch.Generator().manual_seed(3)).bfloat16().cuda() * 0.1]
    x = torch.randn(bs, K, generator=torch.Generator().manual_seed(8)).bfloat16().cuda()
    outs = [torch.empty(bs, M, dtype=torch.bfloat16, device="cuda") for _ in ws]
    got = linear_grouped(x, mods, biases, outs=outs)
    for w, mod, b, y, o in zip(ws, mods, biases, got, outs):
        assert y.data_ptr() == o.data_ptr()
        single = torch.nn.functional.linear(x, mod, b)
        assert torch.equal(y.view(torch.int16), single.view(torch.int16))
        prod = x.float() @ w.float().T
        ref = prod if b is None else prod + b.float()
        bound = ATOL + RTOL * ref.abs() + (0 if b is None else 2.0 ** -8) * prod.abs()
        assert ((y.float() - ref).abs() - bound).max().item() <= 0


@pytest.mark.parametrize("algo", ["huffman", "ans", "nibble"])
@pytest.mark.parametrize("bs", [1, 5])
def test_oversubscribed_group_of_long_tasks(cuda, algo, bs):
    """Two 12800x3072 weights are 2 x 3200 tasks of 24 steps: more wavefronts than the GPU
    holds at once, which is the case the library serves with its long-segment kernels; a
    weight alone runs the short-segment ones.  Same arithmetic, same order: equal bits."""
    from bf16_huffman_infer_amd import _lib
    from bf16_huffman_infer_amd.functional import linear_grouped
    M, K = 12800, 3072
    assert _lib.load().bhi_chunks_per_group(M, K, 1) == 1 and 2 * (M // 4) > 6144 and K // 128 >= 24
    g = torch.Generator(device="cuda").manual_seed(11)
    ws = [(torch.randn(M, K, generator=g, device="cuda") * 0.02).bfloat16() for _ in range(2)]
    mods = [_cls(algo).compress(w).cuda() for w in ws]
    x = torch.randn(bs, K, generator=g, device="cuda").bfloat16()
    got = linear_grouped(x, mods, [None, None])
    for w, mod, y in zip(ws, mods, got):
        single = torch.nn.functional.linear(x, mod)
        assert torch.equal(y.view(torch.int16), single.view(torch.int16))
        ref = x.float() @ w.float().T
        torch.testing.assert_close(y.float(), ref, rtol=RTOL, atol=ATOL)


def test_grouped_split_k_and_leading_dims(cuda):
    from bf16_huffman_infer_amd.functional import HuffmanWeight, linear_grouped
    K = 12288                                          # split_k = 3
    ws = [gaussian_weight(128, K, seed=1), gaussian_weight(256, K, seed=2)]
    mods = [HuffmanWeight.compress(w).cuda() for w in ws]
    assert mods[0].rem.shape[0] == 3
    x = torch.randn(2, 2, K, generator=torch.Generator().manual_seed(3)).bfloat16().cuda()
    got = linear_grouped(x, mods)
    for mod, y in zip(mods, got):
        assert y.shape == (2, 2, mod.rem.shape[1])
        assert torch.equal(y, torch.nn.functional.linear(x, mod))


class _Attn(nn.Module):
    def __init__(self, K=1024):
        super().__init__()
        g = torch.Generator().manual_seed(0)
        self.q_proj = _linear(gaussian_weight(512, K, seed=1), torch.randn(512, generator=g).bfloat16())
        self.k_proj = _linear(gaussian_weight(128, K, seed=2))
        self.v_proj = _linear(gaussian_weight(128, K, seed=3))
        self.gate_proj = _linear(gaussian_weight(256, K, seed=4))
        self.up_proj = _linear(gaussian_weight(256, K, seed=5))

    def forward(self, x):
        q, k, v = self.q_proj(x), self.k_proj(x), self.v_proj(x)
        return torch.cat((q, k, v, torch.nn.functional.silu(self.gate_proj(x)) * self.up_proj(x)), -1)


def _count_launches(fn):
    from bf16_huffman_infer_amd import ops
    calls = {"grouped": 0, "single": 0}
    real_grouped, real_single = ops.gemv_bf16_grouped, ops.gemv_bf16_huffman
    import bf16_huffman_infer_amd.functional as F_

    def grouped(*a, **k):
        calls["grouped"] += 1
        return real_grouped(*a, **k)

    def single(*a, **k):
        calls["single"] += 1
        return real_single(*a, **k)
    F_.gemv_bf16_grouped, F_.gemv_bf16_huffman = grouped, single
    try:
        out = fn()
    finally:
        F_.gemv_bf16_grouped, F_.gemv_bf16_huffman = real_grouped, real_single
    return out, calls


def test_parallelize_qkv_model_groups_and_matches(cuda):
    from bf16_huffman_infer_amd import convert_all_linear
    from bf16_huffman_infer_amd.cudastream_utils import get_parallelize_qkv_model
    model = _Attn()
    convert_all_linear(model, min_out_features=0, progress=False)
    model.cuda()
    grouped = get_parallelize_qkv_model(model)
    assert model.q_proj._group is None and grouped.q_proj._group is not None
    assert grouped.q_proj.weight.rem is model.q_proj.weight.rem            # tensors are shared
    assert grouped.k_proj._group is grouped.q_proj._group and grouped.up_proj._group is grouped.gate_proj._group
    x = torch.randn(1, 1, 1024, generator=torch.Generator().manual_seed(9)).bfloat16().cuda()
    want, c0 = _count_launches(lambda: model(x))
    got, c1 = _count_launches(lambda: grouped(x))
    # un-tied: q_proj has a bias and takes the grouped entry point as a group of one
    assert c0 == {"grouped": 1, "single": 4} and c1 == {"grouped": 2, "single": 0}
    assert torch.equal(got, want)
    # more than 8 rows: every member takes its own decode + GEMM path
    xl = torch.randn(12, 1024, generator=torch.Generator().manual_seed(10)).bfloat16().cuda()
    assert torch.equal(grouped(xl), model(xl))


def test_group_member_called_out_of_pattern(cuda):
    from bf16_huffman_infer_amd import convert_all_linear
    from bf16_huffman_infer_amd.cudastream_utils import parallelize_qkv
    model = _Attn()
    convert_all_linear(model, min_out_features=0, progress=False)
    model.cuda()
    plain = {n: getattr(model, n) for n in ("q_proj", "k_proj", "v_proj")}
    x1 = torch.randn(2, 1024, generator=torch.Generator().manual_seed(1)).bfloat16().cuda()
    x2 = torch.randn(2, 1024, generator=torch.Generator().manual_seed(2)).bfloat16().cuda()
    want = {n: (m(x1), m(x2)) for n, m in plain.items()}
    assert parallelize_qkv(model)
    # follower first, follower on another tensor than the leader, leader twice in a row
    assert torch.equal(model.v_proj(x2), want["v_proj"][1])
    assert torch.equal(model.q_proj(x1), want["q_proj"][0])
    assert torch.equal(model.k_proj(x2), want["k_proj"][1])
    assert torch.equal(model.q_proj(x2), want["q_proj"][1])
    assert torch.equal(model.v_proj(x2), want["v_proj"][1])
    assert torch.equal(model.k_proj(x2), want["k_proj"][1])
    assert torch.equal(model.k_proj(x2), want["k_proj"][1])               # already collected: own launch


def test_mixed_codecs_are_not_grouped(cuda):
    from bf16_huffman_infer_amd.functional import convert
    from bf16_huffman_infer_amd.cudastream_utils import parallelize_qkv, parallelize_gate_up
    model = _Attn()
    for n, algo in (("q_proj", "huffman"), ("k_proj", "ans"), ("v_proj", "huffman"), ("gate_proj", "nibble")):
        setattr(model, n, convert(getattr(model, n), n, algo=algo))
    model.cuda()
    assert not parallelize_qkv(model) and model.q_proj._group is None
    assert not parallelize_gate_up(model)                                 # up_proj is still an nn.Linear


def test_grouped_in_graph_replays(cuda):
    from bf16_huffman_infer_amd import convert_all_linear
    from bf16_huffman_infer_amd.cudagraph_utils import GraphedCallable
    from bf16_huffman_infer_amd.cudastream_utils import parallelize_qkv_model
    model = _Attn()
    convert_all_linear(model, min_out_features=0, progress=False)
    model.cuda()
    parallelize_qkv_model(model)
    x = torch.zeros(1, 1024, dtype=torch.bfloat16, device="cuda")
    step = GraphedCallable(model, (x,))
    for seed in range(3):
        x.copy_(torch.randn(1, 1024, generator=torch.Generator().manual_seed(seed)).bfloat16())
        eager = model(x).clone()
        torch.cuda.synchronize()
        assert torch.equal(step(x), eager)


def test_grouped_rejections(cuda):
    from bf16_huffman_infer_amd import _lib
    from bf16_huffman_infer_amd.functional import ANSWeight, HuffmanWeight, linear_grouped
    a = HuffmanWeight.compress(gaussian_weight(128, 1024, seed=1)).cuda()
    b = HuffmanWeight.compress(gaussian_weight(128, 2048, seed=2)).cuda()
    c = ANSWeight.compress(gaussian_weight(128, 1024, seed=3)).cuda()
    x = torch.randn(1, 1024).bfloat16().cuda()
    with pytest.raises(RuntimeError, match="share split_k and Ks"):
        linear_grouped(x, [a, b])
    with pytest.raises(RuntimeError, match="one codec"):
        linear_grouped(x, [a, c])
    with pytest.raises(RuntimeError, match="1 to 4"):
        linear_grouped(x, [a] * 5)
    with pytest.raises(RuntimeError, match="at most 8 rows"):
        linear_grouped(torch.randn(9, 1024).bfloat16().cuda(), [a, a])
    lib = _lib.load()
    members = (_lib.GemvMember * 1)()
    assert lib.bhi_gemv_bf16_huffman_grouped(members, 0, x.data_ptr(), 1, 1024, 1, None) != 0
    assert lib.bhi_gemv_bf16_huffman_grouped(members, 1, x.data_ptr(), 1, 1024, 1, None) != 0     # null members
    assert b"null pointer" in lib.bhi_last_error_string()
    assert lib.bhi_gemv_bf16_huffman_grouped(None, 1, x.data_ptr(), 1, 1024, 1, None) != 0


@pytest.mark.parametrize("algo", ["huffman", "ans", "nibble"])
@pytest.mark.parametrize("bs,M,K", [(1, 256, 1024), (4, 128, 12288), (8, 512, 2048)])
def test_bias_in_the_kernel_equals_a_separate_bf16_add(cuda, algo, bs, M, K):
    """The reference adds the bias with a separate BF16 `output += bias` (functional.py:403-404);
    the kernel's last store must give those bits (K=12288: three splits, summed across wavefronts)."""
    w = gaussian_weight(M, K, seed=31)
    mod = _cls(algo).compress(w).cuda()
    b = (torch.randn(M, generator=torch.Generator().manual_seed(5)) * 0.5).bfloat16().cuda()
    x = torch.randn(bs, K, generator=torch.Generator().manual_seed(6)).bfloat16().cuda()
    two_step = torch.nn.functional.linear(x, mod)
    two_step += b[None, :]
    fused = torch.nn.functional.linear(x, mod, b)
    assert torch.equal(fused.view(torch.int16), two_step.view(torch.int16))
