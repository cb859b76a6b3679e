"""The benchmark's Qwen3-shaped decoder and the graph capture of its step."""
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import bench_decode as bd  # noqa: E402

SMALL = dict(layers=2, hidden=256, intermediate=512, q_heads=4, kv_heads=2, head_dim=64, vocab=1024, max_len=64)


def test_decoder_matches_transformers_qwen3():
    """Same weights in transformers' Qwen3ForCausalLM give the same logits (bf16 noise)."""
    from transformers import Qwen3Config, Qwen3ForCausalLM
    c = bd.Config(**SMALL)
    m = bd.build(c, torch.device("cpu"))
    cfg = Qwen3Config(hidden_size=c.hidden, intermediate_size=c.intermediate, num_hidden_layers=c.layers,
                      num_attention_heads=c.q_heads, num_key_value_heads=c.kv_heads, head_dim=c.head_dim,
                      vocab_size=c.vocab, max_position_embeddings=c.max_len, rope_theta=c.rope_theta,
                      rms_norm_eps=c.eps, tie_word_embeddings=False)
    hf = Qwen3ForCausalLM(cfg).bfloat16().eval()
    sd = hf.state_dict()
    with torch.no_grad():
        sd["model.embed_tokens.weight"].copy_(m.embed.weight)
        sd["lm_head.weight"].copy_(m.lm_head.weight)
        for i, b in enumerate(m.blocks):
            for n in ("q_proj", "k_proj", "v_proj", "o_proj"):
                sd[f"model.layers.{i}.self_attn.{n}.weight"].copy_(getattr(b, n).weight)
            for n in ("gate_proj", "up_proj", "down_proj"):
                sd[f"model.layers.{i}.mlp.{n}.weight"].copy_(getattr(b, n).weight)
        ids = torch.randint(0, c.vocab, (7,), generator=torch.Generator().manual_seed(0))
        ref = hf(input_ids=ids[None]).logits[0]
        got = []
        for t in ids.tolist():
            m.token.fill_(t)
            got.append(m.step()[0].clone())
    got = torch.stack(got)
    torch.testing.assert_close(got.float(), ref.float(), rtol=0, atol=0.05)
    # the same token wherever the reference's best logit leads its second best by more than the noise
    # (q and k stay in fp32 from the RMSNorm to the end of the rotation here, transformers rounds in between)
    top = ref.float().topk(2, -1).values
    clear = (top[:, 0] - top[:, 1]) > 0.1
    assert clear.any()
    assert torch.equal(got.argmax(-1)[clear], ref.argmax(-1)[clear])


@pytest.mark.gpu
@pytest.mark.parametrize("algo", [None, "huffman", "ans"])
def test_graphed_step_replays_match_eager(cuda, algo):
    """The recorded step, replayed token after token (with eager work and synchronisation
    in between), generates exactly what the eager step generates -- raw and compressed."""
    from bf16_huffman_infer_amd import convert_all_linear
    c = bd.Config(layers=2, hidden=512, intermediate=1024, q_heads=4, kv_heads=2, head_dim=128, vocab=4096, max_len=64)
    model = bd.build(c, torch.device("cuda", 0))
    if algo:
        convert_all_linear(model, min_out_features=0, progress=False, algo=algo)
        model.to("cuda")
        names = {type(m).__name__ for m in model.modules()}
        assert ("HuffmanWeight" if algo == "huffman" else "ANSWeight") in names and "Linear" not in names
    prompt = torch.randint(0, c.vocab, (5,), generator=torch.Generator().manual_seed(2))
    eager, _ = bd.generate(model, prompt, 20, graphed=False)
    for _ in range(3):
        torch.cuda.synchronize()
        scratch = torch.randn(256, 256, device="cuda") @ torch.randn(256, 256, device="cuda")   # eager work between replays
        graphed, _ = bd.generate(model, prompt, 20, graphed=True)
        assert torch.equal(eager, graphed)
    del scratch


@pytest.mark.gpu
def test_get_graphed_model_on_transformers_qwen3(cuda):
    """The reference's entry point on a transformers model: graphed generate == eager generate."""
    from transformers import Qwen3Config, Qwen3ForCausalLM, StaticCache
    from bf16_huffman_infer_amd import convert_all_linear, get_graphed_model
    cfg = Qwen3Config(hidden_size=512, intermediate_size=1024, num_hidden_layers=2, num_attention_heads=4,
                      num_key_value_heads=2, head_dim=128, vocab_size=4096, max_position_embeddings=128,
                      tie_word_embeddings=False)
    torch.manual_seed(0)
    model = Qwen3ForCausalLM(cfg).bfloat16().eval()
    convert_all_linear(model, min_out_features=0, progress=False, algo="huffman")
    model.cuda()
    assert any(type(m).__name__ == "HuffmanWeight" for m in model.modules())
    ids = torch.randint(0, 4096, (1, 6), generator=torch.Generator().manual_seed(3)).cuda()
    want = model.generate(ids, max_new_tokens=12, min_new_tokens=12, do_sample=False)
    cache = StaticCache(config=cfg, max_cache_len=1024)
    graphed = get_graphed_model(model, cache)
    for _ in range(3):
        got = graphed.generate(ids, max_new_tokens=12, min_new_tokens=12, do_sample=False)
        assert torch.equal(got, want)


@pytest.mark.gpu
def test_graphed_step_replays_are_identical_and_match_eager_on_transformers_qwen3(cuda):
    """Same tokens from the same cache state: every replay of the recorded step gives the
    same logits bit for bit (first replay included), and they agree with the model's own
    eager one-token forward over a static cache of the same length."""
    from transformers import Qwen3Config, Qwen3ForCausalLM, StaticCache
    from bf16_huffman_infer_amd import get_graphed_model
    cfg = Qwen3Config(hidden_size=512, intermediate_size=1024, num_hidden_layers=2, num_attention_heads=8,
                      num_key_value_heads=2, head_dim=128, vocab_size=4096, max_position_embeddings=2048,
                      tie_word_embeddings=False)
    torch.manual_seed(1)
    model = Qwen3ForCausalLM(cfg).bfloat16().eval().cuda()
    ids = torch.randint(0, 4096, (1, 16), generator=torch.Generator().manual_seed(3)).cuda()
    toks = [7, 99, 1234, 4000]

    def run(m, cache):
        cache.reset()
        outs = []
        with torch.no_grad():
            outs.append(m(input_ids=ids, past_key_values=cache, use_cache=True).logits[0, -1].float().clone())
            for t in toks:
                tok = torch.full((1, 1), t, device="cuda")
                outs.append(m(input_ids=tok, past_key_values=cache, use_cache=True).logits[0, -1].float().clone())
        return outs

    eager = run(model, StaticCache(config=cfg, max_cache_len=1024))
    cache = StaticCache(config=cfg, max_cache_len=1024)
    graphed = get_graphed_model(model, cache)
    runs = [run(graphed, cache) for _ in range(3)]
    for r in runs[1:]:
        assert all(torch.equal(a, b) for a, b in zip(runs[0], r))
    for a, b in zip(runs[0], eager):
        torch.testing.assert_close(a, b, rtol=0, atol=0.08)


@pytest.mark.gpu
def test_parallelize_qkv_model_on_transformers_qwen3(cuda):
    """The reference's benchmark recipe, get_graphed_model(get_parallelize_qkv_model(model), cache):
    transformers' attention and MLP call q/k/v and gate/up one after the other on one tensor, so
    every layer runs two grouped launches, and generation is unchanged."""
    from transformers import Qwen3Config, Qwen3ForCausalLM, StaticCache
    import bf16_huffman_infer_amd.functional as fn
    from bf16_huffman_infer_amd import convert_all_linear, get_graphed_model
    from bf16_huffman_infer_amd.cudastream_utils import get_parallelize_qkv_model
    cfg = Qwen3Config(hidden_size=512, intermediate_size=1024, num_hidden_layers=2, num_attention_heads=4,
                      num_key_value_heads=2, head_dim=128, vocab_size=4096, max_position_embeddings=128,
                      tie_word_embeddings=False)
    torch.manual_seed(0)
    model = Qwen3ForCausalLM(cfg).bfloat16().eval()
    convert_all_linear(model, min_out_features=0, progress=False, algo="huffman")
    model.cuda()
    ids = torch.randint(0, 4096, (1, 6), generator=torch.Generator().manual_seed(3)).cuda()
    want = model.generate(ids, max_new_tokens=12, min_new_tokens=12, do_sample=False)
    grouped = get_parallelize_qkv_model(model)
    assert model.model.layers[0].self_attn.q_proj._group is None
    assert grouped.model.layers[1].mlp.up_proj._group is grouped.model.layers[1].mlp.gate_proj._group is not None

    calls = {"grouped": 0, "single": 0}
    real_grouped, real_single = fn.gemv_bf16_grouped, fn.gemv_bf16_huffman

    def count_grouped(*a, **k):
        calls["grouped"] += 1
        return real_grouped(*a, **k)

    def count_single(*a, **k):
        calls["single"] += 1
        return real_single(*a, **k)
    fn.gemv_bf16_grouped, fn.gemv_bf16_huffman = count_grouped, count_single
    try:
        with torch.no_grad():
            one = grouped(input_ids=ids[:, :1]).logits
    finally:
        fn.gemv_bf16_grouped, fn.gemv_bf16_huffman = real_grouped, real_single
    # per layer: q/k/v and gate/up grouped, o_proj and down_proj alone; lm_head alone
    assert calls == {"grouped": 2 * cfg.num_hidden_layers, "single": 2 * cfg.num_hidden_layers + 1}
    with torch.no_grad():
        assert torch.equal(one, model(input_ids=ids[:, :1]).logits)
    assert torch.equal(grouped.generate(ids, max_new_tokens=12, min_new_tokens=12, do_sample=False), want)
    cache = StaticCache(config=cfg, max_cache_len=1024)
    graphed = get_graphed_model(grouped, cache)
    for _ in range(2):
        assert torch.equal(graphed.generate(ids, max_new_tokens=12, min_new_tokens=12, do_sample=False), want)


@pytest.mark.gpu
def test_graphed_callable_keeps_closed_over_tensors_alive(cuda):
    """A recorded function reads the tensors it closes over by address; the callable must keep
    them alive after the scope that built it is gone (they used to be freed and their memory
    reused, and replays read whatever landed there)."""
    import gc
    from bf16_huffman_infer_amd.cudagraph_utils import GraphedCallable

    def make():
        table = torch.arange(1024, device="cuda", dtype=torch.float32)

        def fn(x):
            return x + table
        return GraphedCallable(fn, (torch.zeros(1024, device="cuda"),))

    step = make()
    gc.collect()
    junk = [torch.full((1024,), 7.0, device="cuda") for _ in range(256)]      # same size class as the table
    out = step(torch.ones(1024, device="cuda"))
    torch.cuda.synchronize()
    assert torch.equal(out, torch.arange(1024, device="cuda", dtype=torch.float32) + 1)
    del junk
