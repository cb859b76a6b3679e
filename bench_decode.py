"""Greedy decode of a random-init Qwen3-8B-shaped decoder, raw BF16 against compressed.

The decoder below is the Qwen3 architecture (RMSNorm, grouped-query attention with
per-head q/k RMSNorm and rotary embedding, SwiGLU MLP, untied lm_head) written so that one
decode step is a pure function of device tensors: the position, the current token and the
KV cache live on the GPU and the step updates them itself, so the step can be recorded
into one HIP graph and replayed back to back with no host interaction.  Every projection
is an ``nn.Linear``: ``convert_all_linear`` swaps them for compressed modules in place.

Protocol (bs=1): 16 random prompt ids, then 256 greedy tokens, static KV cache of 1024
slots; tokens/s is taken over the 256 decode steps (prompt excluded), best of 3.

Prints one JSON line with raw and compressed tokens/s, their ratio, the footprints from
``get_model_size`` and a teacher-forced comparison: the compressed model is fed the RAW
model's tokens and its logits are compared, at every step, with the raw model's and with a
third run of the raw weights in which every linear layer is an fp32 matmul (``gold``).
Decoding is lossless, but the summation order of a product differs between the library
GEMV of the raw model and the fused kernels, every layer rounds to BF16, and 36 random-init
layers amplify a one-step difference; the yardstick is therefore how far the raw BF16 model
itself is from ``gold``: the compressed model must stay within twice that distance.  (Greedy
ids of a random-init model are a coin toss between near-equal logits, which is why the
length of their common prefix is reported but proves nothing.)
"""
import argparse
import json
import os
import sys
import time

import torch
import torch.nn.functional as F
from torch import nn

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)


class Config:
    def __init__(self, layers=36, hidden=4096, intermediate=12288, q_heads=32, kv_heads=8, head_dim=128,
                 vocab=151936, max_len=1024, rope_theta=1e6, eps=1e-6):
        self.__dict__.update(locals())
        del self.__dict__["self"]


def rms_norm(x, weight, eps):
    return F.rms_norm(x, (x.shape[-1],), weight, eps)


class Block(nn.Module):
    def __init__(self, c: Config):
        super().__init__()
        self.c = c
        self.q_proj = nn.Linear(c.hidden, c.q_heads * c.head_dim, bias=False)
        self.k_proj = nn.Linear(c.hidden, c.kv_heads * c.head_dim, bias=False)
        self.v_proj = nn.Linear(c.hidden, c.kv_heads * c.head_dim, bias=False)
        self.o_proj = nn.Linear(c.q_heads * c.head_dim, c.hidden, bias=False)
        self.gate_proj = nn.Linear(c.hidden, c.intermediate, bias=False)
        self.up_proj = nn.Linear(c.hidden, c.intermediate, bias=False)
        self.down_proj = nn.Linear(c.intermediate, c.hidden, bias=False)
        # per-head RMSNorm weights of q and k, stacked so that both are normalised and
        # rotated in one pass: [q_heads + kv_heads, head_dim]
        self.qk_norm = nn.Parameter(torch.ones(c.q_heads + c.kv_heads, c.head_dim))
        self.input_norm = nn.Parameter(torch.ones(c.hidden))
        self.post_norm = nn.Parameter(torch.ones(c.hidden))

    fused = False            # set by fuse_neighbours() once every projection is compressed

    kernel_attention = True  # the library's one-launch attention step; False: the same step in torch operations

    def attend(self, qk, v, pos, rot, k_cache, v_cache):
        """Per-head RMSNorm and rotary embedding of q and k ([q_heads + kv_heads, head_dim], as
        projected), cache update at ``pos``, attention of the one query over the visible slots.
        ``rot = (cos, sin, hidden, cos_table, sin_table)``: this position's cosines and signed
        sines for every head (the softmax scale already in the q rows) and 0 / -inf over the cache
        slots, all fp32 and computed once per token, and the tables they were taken from.
        Scores and softmax in fp32; the four query heads that share a key/value head form one
        matrix product with it (no expanded copies of the cache)."""
        c = self.c
        cos, sin, hidden, cos_table, sin_table = rot
        if self.kernel_attention and qk.is_cuda and c.head_dim == 128:
            from bf16_huffman_infer_amd.ops import decode_attention
            return decode_attention(qk, v.view(c.kv_heads, c.head_dim), self.qk_norm, cos_table, sin_table, pos,
                                    k_cache, v_cache, eps=c.eps).view(1, c.q_heads * c.head_dim)
        x = F.rms_norm(qk.float(), (c.head_dim,), None, c.eps) * self.qk_norm
        turned = x.view(-1, 2, c.head_dim // 2).flip(1).view(-1, c.head_dim)       # (x1, x2) -> (x2, x1)
        x = torch.addcmul(x * cos, turned, sin).to(qk.dtype)
        k_cache.index_copy_(1, pos, x[c.q_heads:, None, :])                          # [kv, max_len, d]
        v_cache.index_copy_(1, pos, v.view(c.kv_heads, 1, c.head_dim))
        q = x[:c.q_heads].view(c.kv_heads, c.q_heads // c.kv_heads, c.head_dim)
        if q.is_cuda:
            scores = torch.bmm(q, k_cache.transpose(1, 2), out_dtype=torch.float32) + hidden
        else:
            scores = torch.bmm(q.float(), k_cache.float().transpose(1, 2)) + hidden
        weights = torch.softmax(scores, -1).to(qk.dtype)
        return torch.bmm(weights, v_cache).view(1, c.q_heads * c.head_dim)

    def forward(self, x, pos, rot, k_cache, v_cache):
        c = self.c
        if self.fused:
            return self.forward_fused(x, pos, rot, k_cache, v_cache)
        h = rms_norm(x, self.input_norm, c.eps)
        qk = torch.cat((self.q_proj(h), self.k_proj(h)), -1).view(c.q_heads + c.kv_heads, c.head_dim)
        a = self.attend(qk, self.v_proj(h), pos, rot, k_cache, v_cache)
        x = x + self.o_proj(a)
        h = rms_norm(x, self.post_norm, c.eps)
        return x + self.down_proj(F.silu(self.gate_proj(h)) * self.up_proj(h))


def _forward_fused(self, x, pos, rot, k_cache, v_cache):
    """The same layer with the pieces next to a linear inside its launch: the RMSNorm in front of
    q/k/v, silu(gate) * up in front of down_proj, both residual additions behind o_proj and
    down_proj, q and k written side by side (no concatenation).  The RMSNorm in front of gate/up
    stays a kernel of its own: inside that launch, the largest of the layer, it costs 6.3 us,
    more than the 5.4 us kernel it replaces (2.3 us inside q/k/v)."""
    from bf16_huffman_infer_amd.functional import linear_grouped
    c = self.c
    nq, nk = c.q_heads * c.head_dim, c.kv_heads * c.head_dim
    qk = torch.empty(1, nq + nk, dtype=x.dtype, device=x.device)
    v = torch.empty(1, nk, dtype=x.dtype, device=x.device)
    linear_grouped(x, [self.q_proj.weight, self.k_proj.weight, self.v_proj.weight], input_norm=(self.input_norm, c.eps),
                   outs=[qk[:, :nq], qk[:, nq:], v])
    a = self.attend(qk.view(c.q_heads + c.kv_heads, c.head_dim), v, pos, rot, k_cache, v_cache)
    x, = linear_grouped(a, [self.o_proj.weight], residuals=[x])
    gate, up = linear_grouped(rms_norm(x, self.post_norm, c.eps), [self.gate_proj.weight, self.up_proj.weight])
    x, = linear_grouped(up, [self.down_proj.weight], input_gate=gate, residuals=[x])
    return x


Block.forward_fused = _forward_fused


def fuse_neighbours(model) -> int:
    """Switches every block whose seven projections are compressed with one codec (Huffman or
    rANS, no bias) to :func:`_forward_fused`; returns how many blocks that is."""
    from bf16_huffman_infer_amd.functional import CompressedLinear, NibbleWeight
    n = 0
    for blk in model.blocks:
        mods = [blk.q_proj, blk.k_proj, blk.v_proj, blk.o_proj, blk.gate_proj, blk.up_proj, blk.down_proj]
        ok = all(isinstance(m, CompressedLinear) and m.bias is None and not isinstance(m.weight, NibbleWeight) for m in mods)
        ok = ok and len({type(m.weight) for m in mods[:3]}) == 1 and type(mods[4].weight) is type(mods[5].weight)
        blk.fused = bool(ok)
        n += int(ok)
    return n


def greedy(logits):
    """argmax over the vocabulary in two small stages.  A single reduction over 150k values
    makes torch use its multi-block reduce, whose semaphore buffer is cleared by a memset
    node when recorded into a graph; two stages of at most a few thousand values each stay
    within one block per output and record kernels only."""
    n = logits.shape[-1]
    width = 256
    pad = (-n) % width
    v = F.pad(logits.view(-1), (0, pad), value=float("-inf")).view(-1, width)
    best, col = v.max(-1)
    row = best.argmax(0, keepdim=True)
    return row * width + col.index_select(0, row)


class Decoder(nn.Module):
    def __init__(self, c: Config):
        super().__init__()
        self.c = c
        self.embed = nn.Embedding(c.vocab, c.hidden)
        self.blocks = nn.ModuleList(Block(c) for _ in range(c.layers))
        self.norm = nn.Parameter(torch.ones(c.hidden))
        self.lm_head = nn.Linear(c.hidden, c.vocab, bias=False)

    def init_state(self, device):
        c = self.c
        inv = 1.0 / (c.rope_theta ** (torch.arange(0, c.head_dim, 2, device=device).float() / c.head_dim))
        ang = torch.arange(c.max_len, device=device).float()[:, None] * inv[None, :]
        # per position: cosines twice, sines with the sign of the rotate-half convention
        # (out = x * cos + swap_halves(x) * sin), one row per head with the softmax scale in the q rows
        cos, sin = torch.cat((ang.cos(), ang.cos()), -1), torch.cat((-ang.sin(), ang.sin()), -1)      # [max_len, d]
        scale = torch.ones(c.q_heads + c.kv_heads, 1, device=device)
        scale[:c.q_heads] = c.head_dim ** -0.5
        self.head_scale = scale
        self.cos, self.sin = cos, sin
        self.k_cache = torch.zeros(c.layers, c.kv_heads, c.max_len, c.head_dim, dtype=torch.bfloat16, device=device)
        self.v_cache = torch.zeros_like(self.k_cache)
        self.slots = torch.arange(c.max_len, device=device)
        self.pos = torch.zeros(1, dtype=torch.int64, device=device)
        self.token = torch.zeros(1, dtype=torch.int64, device=device)
        self.out = torch.zeros(c.max_len, dtype=torch.int64, device=device)

    def step(self):
        """One token: consumes ``token`` at ``pos``, stores the greedy next token in ``token``
        and ``out[pos]``, advances ``pos``.  Device tensors only."""
        pos = self.pos
        x = self.embed(self.token.clamp(0, self.c.vocab - 1))            # [1, hidden]
        rot = (self.cos.index_select(0, pos) * self.head_scale, self.sin.index_select(0, pos) * self.head_scale,
               torch.where(self.slots <= pos, 0.0, float("-inf")).view(1, 1, -1), self.cos, self.sin)
        for i, blk in enumerate(self.blocks):
            x = blk(x, pos, rot, self.k_cache[i], self.v_cache[i])
        logits = self.lm_head(rms_norm(x, self.norm, self.c.eps))
        nxt = greedy(logits)
        self.out.index_copy_(0, pos, nxt)
        self.token.copy_(nxt)
        self.pos.add_(1).clamp_(max=self.c.max_len - 1)                  # a replay past the cache stays in range
        return logits


def build(c: Config, device, seed=0):
    """Random-init on the device: N(0, 0.02) for every matrix, ones for the norms."""
    with torch.device("meta"):
        model = Decoder(c)
    model = model.to_empty(device=device).bfloat16()
    g = torch.Generator(device=device).manual_seed(seed)
    with torch.no_grad():
        for name, p in model.named_parameters():
            if not name.endswith("norm"):
                p.copy_((torch.randn(p.shape, generator=g, device=device) * 0.02).bfloat16())
            else:
                p.fill_(1.0)
    model.eval()
    model.init_state(device)
    return model


def teacher_forced_logits(model: Decoder, tokens: torch.Tensor):
    """Logits [len(tokens), vocab] (BF16) of ``model`` consuming ``tokens`` one at a time from an
    empty cache, through the recorded step.  ``tokens`` is a device tensor of ids."""
    step = model._graph
    out = torch.empty(len(tokens), model.c.vocab, dtype=torch.bfloat16, device=tokens.device)
    with torch.no_grad():
        model.k_cache.zero_(); model.v_cache.zero_(); model.pos.zero_()
        for i in range(len(tokens)):
            model.token.copy_(tokens[i:i + 1])
            out[i] = step.replay().view(-1)
    return out


def gold_logits(model: Decoder, tokens: torch.Tensor):
    """The same as :func:`teacher_forced_logits` with every ``nn.Linear`` computed as an fp32
    matmul of the BF16 operands (eager, no graph): the reference both BF16 paths approximate."""
    patched = []
    for m in model.modules():
        if isinstance(m, nn.Linear):
            m.forward = (lambda x, m=m: (x.float() @ m.weight.float().T).to(x.dtype))
            patched.append(m)
    out = torch.empty(len(tokens), model.c.vocab, dtype=torch.bfloat16, device=tokens.device)
    try:
        with torch.no_grad():
            model.k_cache.zero_(); model.v_cache.zero_(); model.pos.zero_()
            for i in range(len(tokens)):
                model.token.copy_(tokens[i:i + 1])
                out[i] = model.step().view(-1)
    finally:
        for m in patched:
            del m.forward
    return out


def generate(model: Decoder, prompt: torch.Tensor, new_tokens: int, graphed=True):
    """Returns (ids of the new tokens, seconds spent on the ``new_tokens`` decode steps)."""
    from bf16_huffman_infer_amd.cudagraph_utils import GraphedCallable
    c = model.c
    assert len(prompt) + new_tokens <= c.max_len
    step = getattr(model, "_graph", None)
    if graphed and step is None:
        model.pos.fill_(c.max_len - 1)                                   # record at the last slot
        step = model._graph = GraphedCallable(lambda: model.step(), ())
    run = step.replay if graphed else (lambda: model.step())
    with torch.no_grad():
        model.k_cache.zero_(); model.v_cache.zero_(); model.pos.zero_()
        for t in prompt.tolist():                                        # prompt: one token at a time
            model.token.fill_(t)
            run()
        first = int(model.pos.item())                                    # == len(prompt); token now holds the first new id
        torch.cuda.synchronize()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(new_tokens):
            run()
        stop.record()
        torch.cuda.synchronize()
    ids = model.out[first - 1:first - 1 + new_tokens + 1].clone()        # out[p] = token chosen after consuming position p
    return ids, start.elapsed_time(stop) * 1e-3


def parse_args(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--layers", type=int, default=36)
    ap.add_argument("--tokens", type=int, default=256)
    ap.add_argument("--prompt", type=int, default=16)
    ap.add_argument("--algo", default="smallest", choices=["huffman", "ans", "smallest", "nibble"])
    ap.add_argument("--repeats", type=int, default=3)
    ap.add_argument("--small", action="store_true", help="tiny shapes (smoke run)")
    ap.add_argument("--no-group", action="store_true", help="q/k/v and gate/up as separate launches")
    ap.add_argument("--no-fuse", action="store_true", help="norms, silu*mul and residual additions as separate PyTorch kernels")
    ap.add_argument("--torch-attention", action="store_true",
                    help="norm, rotation, cache update and attention of a layer as torch operations (14 kernels) instead "
                         "of the library's one launch")
    ap.add_argument("--profile", action="store_true",
                    help="only the compressed model as it is served (grouped, fused), one run of --tokens tokens, no raw "
                         "model and no logit comparison: the run to put under rocprofv3 --kernel-trace")
    ap.add_argument("--gold-steps", type=int, default=64,
                    help="teacher-forced steps also run with fp32 matmuls of the raw weights (0: skip)")
    return ap.parse_args(argv)


def run(args) -> dict:
    if not torch.cuda.is_available():
        sys.exit("bench_decode.py needs a GPU")
    from bf16_huffman_infer_amd import _lib, convert_all_linear, get_model_size
    _lib.load()
    device = torch.device("cuda", 0)
    c = Config(layers=args.layers)
    if args.small:
        c = Config(layers=2, hidden=512, intermediate=1024, q_heads=4, kv_heads=2, head_dim=128, vocab=4096)
    Block.kernel_attention = not args.torch_attention
    model = build(c, device)
    g = torch.Generator().manual_seed(1)
    prompt = torch.randint(0, c.vocab, (args.prompt,), generator=g)

    def best(model):
        runs = [generate(model, prompt, args.tokens) for _ in range(args.repeats)]
        assert all(torch.equal(runs[0][0], r[0]) for r in runs), "generation is not reproducible"
        return runs[0][0], min(r[1] for r in runs)

    if args.profile:
        from bf16_huffman_infer_amd.cudastream_utils import parallelize_qkv_model
        convert_all_linear(model, min_out_features=0, progress=False, algo=args.algo)
        model.to(device)
        if not args.no_group:
            parallelize_qkv_model(model)
            if not args.no_fuse:
                fuse_neighbours(model)
        torch.cuda.synchronize()
        _, secs = generate(model, prompt, args.tokens)
        return {"workload": "compressed model only (profile run)", "algo": args.algo, "layers": c.layers, "tokens": args.tokens,
                "prompt": args.prompt, "library_launches_per_token": 4 * c.layers + 1 if not args.no_group else 7 * c.layers + 1,
                "compressed_tokens_per_s": round(args.tokens / secs, 2), "compressed_ms_per_token": round(secs / args.tokens * 1e3, 4)}

    raw_size = get_model_size(model)
    raw_ids, raw_s = best(model)
    print(f"raw BF16: {args.tokens / raw_s:.1f} tok/s, {raw_size / 2**30:.2f} GiB", file=sys.stderr, flush=True)
    forced = torch.cat((prompt.to(device), raw_ids[:-1]))               # what the raw model consumed, step by step
    raw_logits = teacher_forced_logits(model, forced)
    gold = gold_logits(model, forced[:args.gold_steps]) if args.gold_steps > 0 else None

    del model._graph
    t0 = time.time()
    convert_all_linear(model, min_out_features=0, progress=False, algo=args.algo)
    model.to(device)
    convert_s = time.time() - t0
    kinds = {}
    for m in model.modules():
        if type(m).__name__ in ("HuffmanWeight", "ANSWeight", "NibbleWeight"):
            kinds[type(m).__name__] = kinds.get(type(m).__name__, 0) + 1
    new_size = get_model_size(model)
    new_ids, new_s = best(model)
    single_s = None
    if not args.no_group:
        # the reference's benchmark runs get_parallelize_qkv_model on the converted model
        # (examples/benchmark.py:60); here that ties q/k/v and gate/up into grouped launches
        from bf16_huffman_infer_amd.cudastream_utils import parallelize_qkv_model
        single_s = new_s
        del model._graph
        parallelize_qkv_model(model)
        grouped_ids, new_s = best(model)
        assert torch.equal(grouped_ids, new_ids), "grouped launches changed the generated tokens"
    grouped_s, fused_blocks = None, 0
    if not args.no_group and not args.no_fuse:
        fused_blocks = fuse_neighbours(model)
        if fused_blocks:
            grouped_s = new_s
            del model._graph
            new_ids, new_s = best(model)
    same = int((raw_ids == new_ids).long().cumprod(0).sum().item())
    new_logits = teacher_forced_logits(model, forced)

    def step_max(x, y):
        return (x.float() - y.float()).abs().max(-1).values

    per_step = step_max(new_logits, raw_logits)
    scale = raw_logits.float().abs().max().item()
    agree = (new_logits.float().argmax(-1) == raw_logits.float().argmax(-1)).float().mean().item()
    forced_report = {"steps": int(per_step.numel()), "compressed_vs_raw_max_abs_dlogit": round(per_step.max().item(), 5),
                     "compressed_vs_raw_mean_of_step_max": round(per_step.mean().item(), 5),
                     "max_abs_logit": round(scale, 3), "same_argmax_fraction": round(agree, 4)}
    if gold is not None:
        n = gold.shape[0]
        raw_gold, new_gold = step_max(raw_logits[:n], gold), step_max(new_logits[:n], gold)
        bound = 2.0 * raw_gold.max().item()
        forced_report.update({
            "gold": f"first {n} steps with every linear an fp32 matmul of the raw BF16 weights",
            "raw_vs_gold_max_abs_dlogit": round(raw_gold.max().item(), 5),
            "compressed_vs_gold_max_abs_dlogit": round(new_gold.max().item(), 5),
            "raw_vs_gold_mean_of_step_max": round(raw_gold.mean().item(), 5),
            "compressed_vs_gold_mean_of_step_max": round(new_gold.mean().item(), 5),
            "bound": "compressed_vs_gold_max <= 2 * raw_vs_gold_max", "bound_value": round(bound, 5),
            "within_bound": bool(new_gold.max().item() <= bound)})
    del raw_logits, new_logits, gold
    return {
        "workload": f"Qwen3-8B-shaped decoder ({c.layers} layers, hidden {c.hidden}, intermediate {c.intermediate}, "
                    f"{c.q_heads}/{c.kv_heads} heads, vocab {c.vocab}), random init N(0,0.02), bs=1, "
                    f"{args.prompt}-token prompt, {args.tokens} greedy tokens, static KV {c.max_len}, hipGraph step",
        "algo": args.algo, "modules": kinds,
        "attention": ("torch operations: 14 kernels per layer" if args.torch_attention else
                      "one launch per layer (RMSNorm and rotation of q/k, cache update, softmax(qk)v), raw and compressed alike"),
        "raw_tokens_per_s": round(args.tokens / raw_s, 2), "compressed_tokens_per_s": round(args.tokens / new_s, 2),
        "compressed_over_raw": round(raw_s / new_s, 4),
        "launches": ("q/k/v and gate/up one launch each" if single_s is not None else "one launch per linear")
                    + (f"; RMSNorm, silu*mul and the residual additions inside the launches in {fused_blocks} blocks"
                       if grouped_s is not None else ""),
        "compressed_tokens_per_s_single_launches": None if single_s is None else round(args.tokens / single_s, 2),
        "compressed_tokens_per_s_grouped_unfused": None if grouped_s is None else round(args.tokens / grouped_s, 2),
        "raw_ms_per_token": round(raw_s / args.tokens * 1e3, 4), "compressed_ms_per_token": round(new_s / args.tokens * 1e3, 4),
        "raw_gib": round(raw_size / 2**30, 3), "compressed_gib": round(new_size / 2**30, 3),
        "footprint_ratio": round(new_size / raw_size, 4),
        "common_prefix_tokens": same, "tokens": args.tokens + 1, "convert_seconds": round(convert_s, 1),
        "teacher_forced": forced_report,
    }


def main():
    print(json.dumps(run(parse_args()), allow_nan=False))


if __name__ == "__main__":
    main()
