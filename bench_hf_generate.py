"""The reference's own benchmark protocol on a transformers model (examples/benchmark.py).

``get_graphed_model(get_parallelize_qkv_model(model), cache).generate(...)`` on a
``Qwen3ForCausalLM`` of Qwen3-8B's architecture, raw BF16 first, then after
``convert_all_linear(model, min_out_features=0)``; 256 new tokens at batch 1, static KV
cache 1024, best wall time of three whole ``generate`` calls (prefill and the Python of
``generate`` included, as the reference measures it, ``examples/benchmark.py:37-44``).

Two things differ from the reference's script, both forced by running offline: weights
are random (N(0, 0.02), seeded) instead of a downloaded checkpoint, and the prompt is 16
random token ids instead of a tokenised sentence.

    python bench_hf_generate.py [--layers 36] [--tokens 256] [--algo smallest]

Prints one JSON line.
"""
import argparse
import json
import sys
from time import monotonic

import torch


def build(layers: int, device):
    from transformers import Qwen3Config, Qwen3ForCausalLM
    cfg = Qwen3Config(hidden_size=4096, intermediate_size=12288, num_hidden_layers=layers, num_attention_heads=32,
                      num_key_value_heads=8, head_dim=128, vocab_size=151936, max_position_embeddings=40960,
                      rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=False)
    with torch.device("meta"):
        model = Qwen3ForCausalLM(cfg)
    model = model.to(torch.bfloat16).to_empty(device=device).eval()
    g = torch.Generator(device=device).manual_seed(0)
    with torch.no_grad():
        for name, p in model.named_parameters():
            if name.endswith("norm.weight"):
                p.fill_(1.0)
            else:
                p.copy_((torch.randn(p.shape, generator=g, device=device) * 0.02).to(p.dtype))
        # to_empty leaves the rotary table uninitialised (and .to(bfloat16) narrowed it): rebuild
        # it in float32, as a checkpoint load would leave it
        rope = getattr(cfg, "rope_parameters", None) or {}
        theta = float(rope.get("rope_theta", getattr(cfg, "rope_theta", 1000000.0)))
        inv_freq = 1.0 / (theta ** (torch.arange(0, cfg.head_dim, 2, dtype=torch.int64, device=device).float() / cfg.head_dim))
        for m in model.modules():
            if "inv_freq" in dict(m.named_buffers(recurse=False)):
                m.register_buffer("inv_freq", inv_freq.clone(), persistent=False)
                if hasattr(m, "original_inv_freq"):
                    m.original_inv_freq = inv_freq.clone()
    return model, cfg


def best_generate(graphed, ids, tokens, repeats):
    outs, times = [], []
    for _ in range(repeats):
        torch.cuda.synchronize()
        start = monotonic()
        out = graphed.generate(ids, max_new_tokens=tokens, min_new_tokens=tokens, do_sample=False)
        torch.cuda.synchronize()
        times.append(monotonic() - start)
        outs.append(out)
    assert all(torch.equal(outs[0], o) for o in outs), "generation is not reproducible"
    return outs[0], min(times)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--layers", type=int, default=36)
    ap.add_argument("--tokens", type=int, default=256)
    ap.add_argument("--prompt", type=int, default=16)
    ap.add_argument("--algo", default="smallest", choices=["huffman", "ans", "smallest", "nibble"])
    ap.add_argument("--repeats", type=int, default=3)
    args = ap.parse_args()
    if not torch.cuda.is_available():
        sys.exit("bench_hf_generate.py needs a GPU")
    from transformers import StaticCache
    from bf16_huffman_infer_amd import _lib, convert_all_linear, get_model_size
    from bf16_huffman_infer_amd.cudagraph_utils import get_graphed_model
    from bf16_huffman_infer_amd.cudastream_utils import get_parallelize_qkv_model
    _lib.load()
    device = torch.device("cuda", 0)
    model, cfg = build(args.layers, device)
    ids = torch.randint(0, cfg.vocab_size, (1, args.prompt), generator=torch.Generator().manual_seed(1)).to(device)
    cache = StaticCache(config=cfg, max_cache_len=1024)

    raw_size = get_model_size(model)
    graphed = get_graphed_model(get_parallelize_qkv_model(model), cache)
    raw_ids, raw_s = best_generate(graphed, ids, args.tokens, args.repeats)
    print(f"raw BF16: {raw_s:.2f} s for {args.tokens} tokens", flush=True)
    del graphed

    t0 = monotonic()
    convert_all_linear(model, min_out_features=0, progress=False, algo=args.algo)
    model.to(device)
    convert_s = monotonic() - t0
    new_size = get_model_size(model)
    graphed = get_graphed_model(get_parallelize_qkv_model(model), cache)
    new_ids, new_s = best_generate(graphed, ids, args.tokens, args.repeats)
    same = int((raw_ids[0] == new_ids[0]).long().cumprod(0).sum().item()) - args.prompt
    print(json.dumps({
        "protocol": "reference examples/benchmark.py: get_graphed_model(get_parallelize_qkv_model(model), cache).generate, "
                    "best wall time of the whole call",
        "model": f"transformers Qwen3ForCausalLM, Qwen3-8B architecture, {args.layers} layers, random init N(0,0.02)",
        "algo": args.algo, "tokens": args.tokens, "prompt": args.prompt,
        "raw_seconds": round(raw_s, 3), "compressed_seconds": round(new_s, 3),
        "raw_tokens_per_s": round(args.tokens / raw_s, 2), "compressed_tokens_per_s": round(args.tokens / new_s, 2),
        "compressed_over_raw": round(raw_s / new_s, 4),
        "raw_gib": round(raw_size / 2**30, 3), "compressed_gib": round(new_size / 2**30, 3),
        "footprint_ratio": round(new_size / raw_size, 4),
        "common_prefix_new_tokens": same, "convert_seconds": round(convert_s, 1),
    }))


if __name__ == "__main__":
    main()
