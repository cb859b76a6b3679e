"""Fused decode + matrix-core product for 9..32 rows (needs a GPU): against an fp32 matmul of
the same BF16 operands, and against the decode-then-GEMM path it replaces."""
import pytest
import torch

from helpers import gaussian_weight, student_t_weight

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-2, 1e-3


def _cls(algo):
    from bf16_huffman_infer_amd.functional import ANSWeight, HuffmanWeight
    return {"huffman": HuffmanWeight, "ans": ANSWeight}[algo]


@pytest.mark.parametrize("algo", ["huffman", "ans"])
@pytest.mark.parametrize("rows", [9, 12, 16, 17, 25, 32])
@pytest.mark.parametrize("make,M,K,n", [(gaussian_weight, 256, 1024, None), (student_t_weight, 128, 512, 2),
                                        (gaussian_weight, 1024, 4096, None), (student_t_weight, 384, 1536, 4)])
def test_fused_product_matches_fp32(cuda, algo, rows, make, M, K, n):
    w = make(M, K, seed=5)
    mod = (_cls(algo).compress(w) if n is None else _cls(algo).compress_split_n(w, n=n)).cuda()
    x = torch.randn(rows, K, generator=torch.Generator().manual_seed(rows)).bfloat16().cuda()
    y = torch.nn.functional.linear(x, mod)
    assert y.shape == (rows, M) and y.dtype == torch.bfloat16
    ref = x.float() @ w.cuda().float().T
    torch.testing.assert_close(y.float(), ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("algo", ["huffman", "ans"])
def test_fused_product_with_bias_and_leading_dims(cuda, algo):
    from bf16_huffman_infer_amd.functional import CompressedLinear
    w = gaussian_weight(256, 512, seed=7)
    bias = (torch.randn(256, generator=torch.Generator().manual_seed(1)) * 0.1).bfloat16()
    lin = CompressedLinear(_cls(algo).compress(w), torch.nn.Parameter(bias, requires_grad=False)).cuda()
    x = torch.randn(3, 5, 512, generator=torch.Generator().manual_seed(2)).bfloat16().cuda()      # 15 rows
    y = lin(x)
    assert y.shape == (3, 5, 256)
    # the reference's arithmetic: BF16 product, then a BF16 `+= bias`
    want = (x.float() @ w.cuda().float().T).bfloat16() + bias.cuda()
    torch.testing.assert_close(y.float(), want.float(), rtol=RTOL, atol=ATOL + 2.0 ** -8 * 0.5)


@pytest.mark.parametrize("algo", ["huffman", "ans"])
@pytest.mark.parametrize("M,K", [(12288, 4096), (4096, 12288)])
@pytest.mark.parametrize("rows", [16, 32])
def test_full_size_fallback_shapes(cuda, algo, M, K, rows):
    """The two layer shapes of the large-batch configuration, Student-t weights: fused product
    against fp32, and the decoded weight bit for bit."""
    torch.manual_seed(M + K)
    w = (torch.distributions.StudentT(3.0).sample((M, K)) * (0.02 / 3 ** 0.5)).bfloat16().cuda()
    mod = _cls(algo).compress(w).cuda()
    assert torch.equal(mod.get_weight().view(torch.int16), w.view(torch.int16))
    x = torch.randn(rows, K, generator=torch.Generator().manual_seed(3)).bfloat16().cuda()
    y = torch.nn.functional.linear(x, mod)
    ref = x.float() @ w.float().T
    torch.testing.assert_close(y.float(), ref, rtol=RTOL, atol=ATOL)
    # twice in a row: the workspace counters are back at zero after every launch
    y2 = torch.nn.functional.linear(x, mod)
    assert torch.equal(y.view(torch.int16), y2.view(torch.int16))


@pytest.mark.parametrize("algo", ["huffman", "ans"])
@pytest.mark.parametrize("rows", [3, 12, 20, 32])
@pytest.mark.parametrize("M,K", [(128, 512), (640, 2048), (1408, 1024), (12160, 512), (12416, 512)])
def test_row_counts_that_fill_no_whole_block(cuda, algo, rows, M, K):
    """M / 4 row groups that are no multiple of the 12 a block may hold (the last block repeats the
    last group and stores nothing for the repeats), with and without K slices; 12160 rows at up to
    16 rows of X and every case above 16 take blocks of 12."""
    from bf16_huffman_infer_amd import ops
    w = gaussian_weight(M, K, seed=M + rows)
    mod = _cls(algo).compress(w).cuda()
    x = torch.randn(rows, K, generator=torch.Generator().manual_seed(rows)).bfloat16().cuda()
    y = torch.full((rows, M), float("nan"), dtype=torch.bfloat16, device="cuda")
    guard = torch.full((4096,), 7.0, dtype=torch.bfloat16, device="cuda")       # allocated right behind y
    ops.gemm_bf16(mod, x.view(rows, *mod.rem.shape[::2]), y)
    ref = x.float() @ w.cuda().float().T
    torch.testing.assert_close(y.float(), ref, rtol=RTOL, atol=ATOL)
    assert bool((guard == 7.0).all())


@pytest.mark.parametrize("algo", ["huffman", "ans"])
@pytest.mark.parametrize("rows", [3, 16, 32])
@pytest.mark.parametrize("Ms", [(2048, 4096, 2560), (1024, 1024, 1024), (8192, 8320)])
def test_grouped_product(cuda, algo, rows, Ms):
    """Up to four weights in one grid (8704 and 16512 rows: the grouped entry point; 3072 rows: too few,
    one launch per member), with a bias on one member and a residual on another: against fp32, and bit
    for bit against the members' own launches where those are not cut along K either."""
    from bf16_huffman_infer_amd import _lib, ops
    K = 1024
    ws = [gaussian_weight(M, K, seed=60 + i) for i, M in enumerate(Ms)]
    mods = [_cls(algo).compress(w).cuda() for w in ws]
    x = torch.randn(rows, K, generator=torch.Generator().manual_seed(rows)).bfloat16().cuda()
    x3 = x.view(rows, *mods[0].rem.shape[::2])
    biases = [None] * len(Ms)
    biases[0] = (torch.randn(Ms[0], generator=torch.Generator().manual_seed(1)) * 0.1).bfloat16().cuda()
    residuals = [None] * len(Ms)
    residuals[-1] = torch.randn(rows, Ms[-1], generator=torch.Generator().manual_seed(2)).bfloat16().cuda()
    ys = [torch.full((rows, M), float("nan"), dtype=torch.bfloat16, device="cuda") for M in Ms]
    ops.gemm_bf16_grouped(mods, x3, ys, biases, residuals)
    for w, mod, b, r, y in zip(ws, mods, biases, residuals, ys):
        want = (x.float() @ w.cuda().float().T).bfloat16()
        if b is not None:
            want = want + b
        if r is not None:
            want = want + r
        torch.testing.assert_close(y.float(), want.float(), rtol=RTOL, atol=ATOL + 2.0 ** -7 * want.float().abs().max().item())
        sk, M, Ks = mod.rem.shape
        if _lib.load().bhi_gemm_workspace_bytes(sk, M, Ks, rows) == 0:
            single = torch.empty_like(y)
            ops.gemm_bf16(mod, x3, single, b, residual=r)
            assert torch.equal(single.view(torch.int16), y.view(torch.int16))


def test_grouped_product_rejections(cuda):
    from bf16_huffman_infer_amd import _lib, ops
    w = gaussian_weight(1024, 1024, seed=3)
    a, b = _cls("huffman").compress(w).cuda(), _cls("ans").compress(w).cuda()
    x = torch.randn(16, 1, 1024).bfloat16().cuda()
    ys = [torch.empty(16, 1024, dtype=torch.bfloat16, device="cuda") for _ in range(2)]
    with pytest.raises(RuntimeError, match="one codec"):
        ops.gemm_bf16_grouped([a, b], x, ys)
    with pytest.raises(RuntimeError, match="1 to 4"):
        ops.gemm_bf16_grouped([a] * 5, x, ys * 3)
    # the C entry point refuses a group it would have to cut along K
    members = (_lib.GemvMember * 2)()
    for m, y in zip(members, ys):
        ops._fill_member(m, a, y, None, a.rem)
    rc = _lib.load().bhi_gemm_bf16_huffman_grouped(members, 2, x.data_ptr(), 1, 1024, 16, None)
    assert rc != 0 and b"one by one" in _lib.load().bhi_last_error_string()


def test_more_than_32_rows_still_decode_then_gemm(cuda):
    w = gaussian_weight(256, 512, seed=7)
    mod = _cls("huffman").compress(w).cuda()
    x = torch.randn(40, 512, generator=torch.Generator().manual_seed(2)).bfloat16().cuda()
    y = torch.nn.functional.linear(x, mod)
    torch.testing.assert_close(y, torch.nn.functional.linear(x, w.cuda()))


def test_k_slice_hand_over_survives_hundreds_of_alternating_launches(cuda):
    """Two K-sliced shapes take turns on ONE workspace, a few hundred launches with no host
    synchronisation in between: every result must have the bits of the first one (a partial sum
    read before its store had landed, or a counter left non-zero, would show as a difference)."""
    torch.manual_seed(3)
    cases = []
    for M, K, rows in ((1024, 4096, 16), (512, 6144, 32)):
        w = gaussian_weight(M, K, seed=M)
        mod = _cls("huffman").compress(w).cuda()
        x = torch.randn(rows, K, generator=torch.Generator().manual_seed(rows)).bfloat16().cuda()
        first = torch.nn.functional.linear(x, mod)
        torch.testing.assert_close(first.float(), x.float() @ w.cuda().float().T, rtol=RTOL, atol=ATOL)
        cases.append((mod, x, first))
    from bf16_huffman_infer_amd import _lib
    for mod, x, _ in cases:
        sk, M, Ks = mod.rem.shape
        assert _lib.load().bhi_gemm_workspace_bytes(sk, M, Ks, x.shape[0]) > 0, "the case must be cut along K"
    outs = []
    for i in range(300):
        mod, x, _ = cases[i % 2]
        outs.append(torch.nn.functional.linear(x, mod))
    torch.cuda.synchronize()
    for i, y in enumerate(outs):
        assert torch.equal(y.view(torch.int16), cases[i % 2][2].view(torch.int16)), f"launch {i} differs from the first"


def test_workspaces_belong_to_one_stream_each(cuda):
    from bf16_huffman_infer_amd import ops
    w = gaussian_weight(1024, 4096, seed=9)
    mod = _cls("huffman").compress(w).cuda()
    x = torch.randn(16, 4096, generator=torch.Generator().manual_seed(1)).bfloat16().cuda()
    want = torch.nn.functional.linear(x, mod)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        got = torch.nn.functional.linear(x, mod)
    side.synchronize()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    here = ops._workspaces[(x.device, torch.cuda.current_stream().cuda_stream)][-1]
    there = ops._workspaces[(x.device, side.cuda_stream)][-1]
    assert here.data_ptr() != there.data_ptr()


@pytest.mark.parametrize("algo", ["huffman", "ans"])
def test_capture_on_a_stream_without_a_workspace(cuda, algo):
    """A 16-row product recorded on a stream that has no workspace yet (torch captures on a stream of
    its own): the workspace is allocated from the graph's pool, its fill is a node of the graph, and
    every replay gives the eager bits -- with the program's own eager work between the replays."""
    w = gaussian_weight(1024, 4096, seed=11)
    mod = _cls(algo).compress(w).cuda()
    x = torch.randn(16, 4096, generator=torch.Generator().manual_seed(4)).bfloat16().cuda()
    eager = torch.nn.functional.linear(x, mod)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = torch.nn.functional.linear(x, mod)
    for i in range(3):
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), eager.view(torch.int16)), f"replay {i}"
        again = torch.nn.functional.linear(x, mod)
        assert torch.equal(again.view(torch.int16), eager.view(torch.int16))


def test_built_in_workspace_on_request(cuda):
    """``static_workspace=True``: nothing is allocated, eagerly or under capture, and the bits are the same."""
    from bf16_huffman_infer_amd import ops
    w = gaussian_weight(1024, 4096, seed=12)
    mod = _cls("huffman").compress(w).cuda()
    x = torch.randn(16, 1, 4096, generator=torch.Generator().manual_seed(5)).bfloat16().cuda()
    want = torch.nn.functional.linear(x.view(16, 4096), mod)
    got = torch.empty_like(want)
    ops.gemm_bf16(mod, x, got, static_workspace=True)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    graph = torch.cuda.CUDAGraph()
    rec = torch.empty_like(want)
    with torch.cuda.graph(graph):
        ops.gemm_bf16(mod, x, rec, static_workspace=True)
    for i in range(2):
        rec.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(rec.view(torch.int16), want.view(torch.int16)), f"replay {i}"
    with pytest.raises(RuntimeError, match="Huffman"):
        ops.gemm_bf16(_cls("ans").compress(w).cuda(), x, got, static_workspace=True)
