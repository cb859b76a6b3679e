"""The one-token attention launch (needs a GPU): against the same step written with torch
operations -- fp32 RMSNorm and rotation, BF16 q/k/cache, fp32 scores and softmax, BF16 weights."""
import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu


def tables(max_len, d, theta=1e6, device="cuda"):
    inv = 1.0 / (theta ** (torch.arange(0, d, 2, device=device).float() / d))
    ang = torch.arange(max_len, device=device).float()[:, None] * inv[None, :]
    return torch.cat((ang.cos(), ang.cos()), -1).contiguous(), torch.cat((-ang.sin(), ang.sin()), -1).contiguous()


def torch_step(qk, v, w, cos, sin, pos, k_cache, v_cache, q_heads, kv_heads, eps):
    d = qk.shape[-1]
    p = int(pos.item())
    x = F.rms_norm(qk.float(), (d,), None, eps)
    if w is not None:
        x = x * w
    turned = x.view(-1, 2, d // 2).flip(1).reshape(-1, d)
    x = x * cos[p] + turned * sin[p]
    x[:q_heads] *= d ** -0.5
    x = x.bfloat16()
    k_cache[:, p] = x[q_heads:]
    v_cache[:, p] = v
    q = x[:q_heads].view(kv_heads, q_heads // kv_heads, d).float()
    scores = q @ k_cache[:, :p + 1].float().transpose(1, 2)
    weights = torch.softmax(scores, -1).bfloat16().float()
    return (weights @ v_cache[:, :p + 1].float()).view(q_heads, d)


@pytest.mark.parametrize("q_heads,kv_heads", [(32, 8), (4, 2), (8, 8)])
@pytest.mark.parametrize("max_len,positions", [(1024, (0, 1, 5, 255, 256, 257, 700, 1023)), (300, (0, 299)), (4096, (3000,))])
@pytest.mark.parametrize("with_weight", [True, False])
def test_matches_the_torch_formulation(cuda, q_heads, kv_heads, max_len, positions, with_weight):
    from bf16_huffman_infer_amd import ops
    d = 128
    g = torch.Generator(device="cuda").manual_seed(q_heads * 1000 + max_len)
    cos, sin = tables(max_len, d)
    w = (1 + 0.1 * torch.randn(q_heads + kv_heads, d, generator=g, device="cuda")).bfloat16() if with_weight else None
    for p in positions:
        kc = torch.randn(kv_heads, max_len, d, generator=g, device="cuda").bfloat16()
        vc = torch.randn(kv_heads, max_len, d, generator=g, device="cuda").bfloat16()
        qk = (torch.randn(q_heads + kv_heads, d, generator=g, device="cuda") * 3).bfloat16()
        v = torch.randn(kv_heads, d, generator=g, device="cuda").bfloat16()
        pos = torch.tensor([p], device="cuda")
        kc_ref, vc_ref = kc.clone(), vc.clone()
        want = torch_step(qk, v, w, cos, sin, pos, kc_ref, vc_ref, q_heads, kv_heads, 1e-6)
        got = ops.decode_attention(qk, v, w, cos, sin, pos, kc, vc, eps=1e-6)
        # the caches: only slot p changed; v bit for bit, k within one BF16 step (fp32 rounding order of the rotation)
        assert torch.equal(vc.view(torch.int16), vc_ref.view(torch.int16)), p
        untouched = torch.ones(max_len, dtype=torch.bool, device="cuda")
        untouched[p] = False
        assert torch.equal(kc[:, untouched].view(torch.int16), kc_ref[:, untouched].view(torch.int16)), p
        torch.testing.assert_close(kc[:, p].float(), kc_ref[:, p].float(), rtol=2 ** -7, atol=1e-3)
        torch.testing.assert_close(got.float(), want, rtol=2e-2, atol=2e-2, msg=lambda m: f"pos {p}: {m}")


def test_follows_the_position_inside_a_recorded_graph(cuda):
    from bf16_huffman_infer_amd import ops
    q_heads, kv_heads, d, max_len = 8, 2, 128, 512
    g = torch.Generator(device="cuda").manual_seed(5)
    cos, sin = tables(max_len, d)
    kc = torch.zeros(kv_heads, max_len, d, dtype=torch.bfloat16, device="cuda")
    vc = torch.zeros_like(kc)
    qk = torch.zeros(q_heads + kv_heads, d, dtype=torch.bfloat16, device="cuda")
    v = torch.zeros(kv_heads, d, dtype=torch.bfloat16, device="cuda")
    pos = torch.zeros(1, dtype=torch.int64, device="cuda")
    out = torch.empty(q_heads, d, dtype=torch.bfloat16, device="cuda")
    ops.decode_attention(qk, v, None, cos, sin, pos, kc, vc, out=out)
    torch.cuda.synchronize()
    kc.zero_(); vc.zero_()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        ops.decode_attention(qk, v, None, cos, sin, pos, kc, vc, out=out)
        pos.add_(1)
    kc.zero_(); vc.zero_(); pos.zero_()
    kc_ref, vc_ref = kc.clone(), vc.clone()
    for step in range(40):
        qk.copy_((torch.randn(qk.shape, generator=g, device="cuda") * 2).bfloat16())
        v.copy_(torch.randn(v.shape, generator=g, device="cuda").bfloat16())
        want = torch_step(qk, v, None, cos, sin, torch.tensor([step]), kc_ref, vc_ref, q_heads, kv_heads, 1e-6)
        graph.replay()
        torch.cuda.synchronize()
        assert int(pos.item()) == step + 1
        torch.testing.assert_close(out.float(), want, rtol=2e-2, atol=2e-2, msg=lambda m: f"step {step}: {m}")
        kc_ref.copy_(kc)            # keep the reference cache on the kernel's (BF16-step close) k values


def test_rejections(cuda):
    from bf16_huffman_infer_amd import ops
    cos, sin = tables(64, 128)
    kc = torch.zeros(2, 64, 128, dtype=torch.bfloat16, device="cuda")
    qk = torch.zeros(6, 128, dtype=torch.bfloat16, device="cuda")
    v = torch.zeros(2, 128, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(RuntimeError, match="pos"):
        ops.decode_attention(qk, v, None, cos, sin, torch.zeros(1, dtype=torch.int64), kc, kc.clone())
    with pytest.raises(RuntimeError, match="cos and sin"):
        ops.decode_attention(qk, v, None, cos[:32], sin, torch.zeros(1, dtype=torch.int64, device="cuda"), kc, kc.clone())
    with pytest.raises(RuntimeError, match="head dimension"):
        c64, s64 = tables(64, 64)
        ops.decode_attention(qk[:, :64].contiguous(), v[:, :64].contiguous(), None, c64, s64,
                             torch.zeros(1, dtype=torch.int64, device="cuda"), kc[..., :64].contiguous(), kc[..., :64].contiguous())
