"""Fused decode-GEMV benchmark on one MI355X.

Workload: the linear layers of one Qwen2.5-7B decoder block (q/k/v fused 3584->4608,
o 3584->3584, gate and up 3584->18944, down 18944->3584), BF16 weights iid N(0, 0.02)
from a seed, Huffman-compressed, batch 1.  One step = one fused decode-GEMV launch per
layer.  Two independently seeded copies of the block alternate between steps so that
the 256 MB last-level cache cannot serve the weights.

Prints one JSON line: whole-block GB/s on compressed bytes, with the roofline of the
dominant kernel (the 18944x3584 GEMV) and the CPU baseline (the reference's layout and
decoder restated in numpy + a host matmul, timed on this machine).
"""
import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
LAYERS = [("qkv_proj", 4608, 3584), ("o_proj", 3584, 3584), ("gate_proj", 18944, 3584),
          ("up_proj", 18944, 3584), ("down_proj", 3584, 18944)]
COPIES = 2
# A token of Qwen2.5-7B is 28 decoder blocks, and serving records the whole token as one graph:
# the timed graphs hold that many block steps (alternating over the COPIES weight sets).  With
# two steps per graph the replay's own start weighs 2.3 us on every step (71.8 against 69.5 us).
STEPS_PER_GRAPH = 28
GRAPH_ROTATIONS = 4       # the single-layer graphs go this many times round their clones, for the same reason
ROTATE_BYTES = 640 << 20
CLOCK_WARMUP_S = 0.06
STD = 0.02
# HBM bytes per launch of the dominant kernel, from rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE
# runs of this script, each scaled by the same counter's reading for the 256 MiB calibration
# copy below.  Keyed by (algo, batch, launch): "single" = one 18944x3584 matrix, "group" =
# gate_proj + up_proj in one launch, "lm_head" = the 152064x3584 launch.  The readings belong
# to the kernel sources whose digest is recorded with them: when the sources have changed
# since, `traffic` is reported as null.
MEASURED_TRAFFIC_SOURCES = "e8b3f419c1ba9e66"
MEASURED_TRAFFIC = {("huffman", 1, "single"): 93800000, ("huffman", 1, "group"): 189020000,
                    ("huffman", 1, "lm_head"): 758480000}


def kernel_sources_digest() -> str:
    """SHA-256 (first 16 hex digits) over the HIP sources the library is built from."""
    import hashlib
    src = os.path.join(ROOT, "bf16_huffman_infer_amd", "csrc")
    h = hashlib.sha256()
    for name in sorted(os.listdir(src)):
        if name.endswith((".h", ".hip")):
            with open(os.path.join(src, name), "rb") as f:
                h.update(name.encode() + b"\0" + f.read())
    return h.hexdigest()[:16]


def measured_traffic(key):
    return MEASURED_TRAFFIC.get(key) if kernel_sources_digest() == MEASURED_TRAFFIC_SOURCES else None


def make_weight(M, K, seed, device):
    g = torch.Generator(device=device).manual_seed(seed)
    return (torch.randn(M, K, generator=g, device=device) * STD).bfloat16()


def weight_bytes(mod) -> int:
    return sum(b.nelement() * b.element_size() for b in mod.buffers())


def gemv_bytes(mod, bs, M, K) -> int:
    """Algorithmic bytes of one fused GEMV: every weight-module buffer once + X + Y."""
    return weight_bytes(mod) + bs * K * 2 + bs * M * 2


def build_block(algo, device, copy):
    from bf16_huffman_infer_amd.functional import ANSWeight, HuffmanWeight, NibbleWeight
    cls = {"huffman": HuffmanWeight, "ans": ANSWeight, "nibble": NibbleWeight}
    mods = []
    for i, (name, M, K) in enumerate(LAYERS):
        w = make_weight(M, K, 1000 * copy + i, device)
        if algo == "smallest":                      # what convert(..., algo='smallest') keeps: the smaller of the two
            mods.append(min((HuffmanWeight.compress(w), ANSWeight.compress(w)), key=weight_bytes).to(device))
        else:
            mods.append(cls[algo].compress(w).to(device))
        del w
    return mods


LM_HEAD = (152064, 3584)      # the model's largest linear: vocabulary x hidden


def lm_head(args, device):
    """The same kernel on the model's lm_head, one launch of 38016 tasks (six times what the
    GPU holds at once), so that launch, first fill and the last blocks weigh little: what the
    kernel sustains when a launch is long enough.  Two clones alternate (375 MB each, more
    than the 256 MB last-level cache)."""
    import copy
    import torch.nn.functional as F
    from bf16_huffman_infer_amd.functional import ANSWeight, HuffmanWeight, NibbleWeight
    M, K = LM_HEAD
    cls = {"huffman": HuffmanWeight, "ans": ANSWeight, "nibble": NibbleWeight}[args.algo]
    w = make_weight(M, K, 77, device)
    mod = cls.compress(w).to(device)
    del w
    mods = [mod, copy.deepcopy(mod)]
    x = torch.randn(args.batch, K, device=device).bfloat16()
    st = {"i": 0}

    def one():
        F.linear(x, mods[st["i"] % 2])
        st["i"] += 1
    t = time_launches(one, max(60, args.steps // 2), args.warmup, launches_per_graph=2)
    nbytes = gemv_bytes(mod, args.batch, M, K)
    return {"shape": f"{M}x{K}", "tasks": M // 4, "bytes_per_launch": nbytes, "us_per_launch": round(t * 1e6, 2),
            "achieved": round(nbytes / t / 1e9, 1), "frac": round(nbytes / t / 1e9 / HBM_PEAK_GBS, 4),
            "traffic": measured_traffic((args.algo, args.batch, "lm_head")),
            "compression_ratio": round(weight_bytes(mod) / (2 * M * K), 4)}


def sweep(args, device, huffman_blocks):
    """The same block step at other batches and with the other codecs: GB/s on compressed bytes,
    fraction of the HBM peak, compressed/raw ratio.  ``smallest`` keeps, per layer, whichever of
    the Huffman and rANS forms is smaller (gate_proj and up_proj are launched as one group only
    when they ended up with the same codec)."""
    import torch.nn.functional as F
    from bf16_huffman_infer_amd.functional import linear_grouped
    raw_bytes = sum(M * K * 2 for _, M, K in LAYERS)
    out = []
    cases = [("huffman", b) for b in (2, 4, 8)] + [("ans", b) for b in (1, 8)] + [("smallest", b) for b in (1, 8)]
    built = {"huffman": huffman_blocks}
    for algo, bs in cases:
        if algo not in built:
            built[algo] = [build_block(algo, device, c) for c in range(COPIES)]
        blocks = built[algo]
        xs = [torch.randn(bs, K, device=device).bfloat16() for _, _, K in LAYERS]
        groupable = all(type(b[2]) is type(b[3]) for b in blocks)
        state = {"i": 0}

        def step():
            mods = blocks[state["i"] % COPIES]
            state["i"] += 1
            F.linear(xs[0], mods[0])
            F.linear(xs[1], mods[1])
            if groupable:
                linear_grouped(xs[2], [mods[2], mods[3]])
            else:
                F.linear(xs[2], mods[2])
                F.linear(xs[3], mods[3])
            F.linear(xs[4], mods[4])
        sec = time_launches(step, args.steps, args.warmup, launches_per_graph=STEPS_PER_GRAPH)
        nbytes = sum(gemv_bytes(m, bs, M, K) for m, (_, M, K) in zip(blocks[0], LAYERS))
        out.append({"algo": algo, "batch": bs, "ms_per_step": round(sec * 1e3, 5), "GBps": round(nbytes / sec / 1e9, 1),
                    "frac": round(nbytes / sec / 1e9 / HBM_PEAK_GBS, 4),
                    "compression_ratio": round(sum(weight_bytes(m) for m in blocks[0]) / raw_bytes, 4),
                    "codecs": sorted({type(m).__name__ for m in blocks[0]})})
    return out


ROUNDS = 5


def time_launches(fn, n, warmup, launches_per_graph=1, rounds=ROUNDS, spread=None):
    """Seconds per call of ``fn``: the median of ``rounds`` timed regions of exactly ``n`` calls each.
    ``fn`` is captured into a HIP graph (as the decode step is in serving, and as the
    reference's own benchmark does with CUDA graphs) so that the Python dispatch cost of the
    op wrappers is not what gets timed; the graph holds ``launches_per_graph`` consecutive
    calls, and a second, shorter graph holds the ``n % launches_per_graph`` calls that remain.
    ``spread``, a dict, receives the fastest and the slowest round."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2 * min(launches_per_graph, 4)):
            fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    def record(calls):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for _ in range(calls):
                fn()
        return g
    n = max(1, n)
    per = min(launches_per_graph, n)
    replays, rest = divmod(n, per)
    graph = record(per)
    tail = record(rest) if rest else None
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    for _ in range(max(1, warmup // per)):
        graph.replay()
    # After any idle period (building the next layer's clones is one) the GPU needs about
    # 25 ms of continuous work to reach its steady clocks: the first launches run 10 %
    # slower (25.0 -> 22.4 us on 18944x3584).  A decoder runs for seconds, so the steady
    # state is what counts: keep the graph running, untimed, for CLOCK_WARMUP_S first.
    start.record()
    graph.replay()
    stop.record()
    torch.cuda.synchronize()
    once = max(start.elapsed_time(stop) * 1e-3, 1e-6)
    for _ in range(int(CLOCK_WARMUP_S / once) + 1):
        graph.replay()
    if tail is not None:
        tail.replay()
    torch.cuda.synchronize()
    times = []
    for _ in range(max(1, rounds)):
        start.record()
        for _ in range(replays):
            graph.replay()
        if tail is not None:
            tail.replay()
        stop.record()
        torch.cuda.synchronize()
        times.append(start.elapsed_time(stop) * 1e-3 / n)
    times.sort()
    if spread is not None:
        spread.update(rounds=len(times), calls_per_round=n, calls_per_graph=per, min=times[0], max=times[-1])
    return times[len(times) // 2]


def load_only(launch_bytes, args, device):
    """The ceiling measured in the same run: a kernel that only loads the bytes of one
    18944x3584 launch (as many wavefronts as that layer has tasks, four 16-byte loads in
    flight per lane, nothing kept), rotating over >= 640 MB like the per-layer timings."""
    from bf16_huffman_infer_amd import _lib
    lib = _lib.load()
    waves = 18944 // 4                                   # one wavefront per task of the layer
    n = max(2, -(-ROTATE_BYTES // launch_bytes))
    stride = -(-launch_bytes // 256) * 256
    buf = torch.empty(n * stride, dtype=torch.uint8, device=device).random_(0, 255)
    sink = torch.zeros(1, dtype=torch.int32, device=device)
    res = {"wavefronts": waves, "unit": "GB/s"}
    for name, nt in (("non_temporal", 1), ("plain", 0)):
        st = {"i": 0, "bytes": 0}

        def one(st=st, nt=nt):
            i = st["i"] % n
            st["i"] += 1
            got = lib.bhi_stream_read(buf.data_ptr() + i * stride, launch_bytes, waves, nt, sink.data_ptr(),
                                      torch.cuda.current_stream().cuda_stream)
            if got <= 0:
                raise RuntimeError(f"bhi_stream_read failed: {got}")
            st["bytes"] = got
        t = time_launches(one, max(100, args.steps), args.warmup, launches_per_graph=n)
        res[name] = round(st["bytes"] / t / 1e9, 1)
        res["bytes_per_launch"] = st["bytes"]
        res[f"us_per_launch_{name}"] = round(t * 1e6, 2)
    res["frac_of_peak"] = round(res["non_temporal"] / HBM_PEAK_GBS, 4)
    return res


def cpu_baseline(rows=18944, K=3584, reps=5):
    """Reference layout + reference decoder (numpy) + host matmul on a slice of gate_proj."""
    import numpy as np
    from oracle import planes, ref_layout, ref_tables
    g = torch.Generator().manual_seed(2)
    w = (torch.randn(rows, K, generator=g) * STD).bfloat16()
    bits = w.view(torch.int16).numpy().view(np.uint16)
    _, exp = planes.split_bf16(bits)
    luts, lens, codes = ref_tables.build_cascade_luts(np.bincount(exp.reshape(-1), minlength=256))
    enc = ref_layout.encode(bits, 1, "huffman", codes)
    x = torch.randn(1, K, generator=g).bfloat16()
    nbytes = enc["rem"].nbytes + enc["exp"].nbytes + enc["offsets"].nbytes + 5 * 256 + K * 2 + rows * 2
    times = []
    for _ in range(reps):
        t = time.perf_counter()
        dec = ref_layout.decode_huffman(enc["rem"], enc["exp"], enc["offsets"], luts, lens)
        t_dec = time.perf_counter() - t
        wd = torch.from_numpy(dec.view(np.int16)).view(torch.bfloat16)
        t = time.perf_counter()
        y = (x.float() @ wd.float().T).bfloat16()
        t_mm = time.perf_counter() - t
        times.append((t_dec + t_mm, t_dec, t_mm))
    assert np.array_equal(dec, bits), "CPU baseline decoder is not lossless"
    times.sort()
    total, t_dec, t_mm = times[len(times) // 2]
    return {
        "value": round(nbytes / total / 1e9, 4), "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
        "sample": f"gate_proj ({rows}x{K}) of the workload, reference layout, median of {reps} passes "
                  f"({sum(t[0] for t in times):.1f}s of CPU work); numpy decode {t_dec:.2f}s (1 thread) + torch matmul "
                  f"{t_mm * 1e3:.1f}ms ({torch.get_num_threads()} threads); os.cpu_count()={os.cpu_count()}",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--batch", type=int, default=1)
    ap.add_argument("--algo", default="huffman", choices=["huffman", "ans", "nibble"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-group", action="store_true", help="gate_proj and up_proj as two launches")
    ap.add_argument("--no-sweep", action="store_true", help="skip the other batches / codecs")
    ap.add_argument("--no-fallback", action="store_true", help="skip the 16- and 32-row fused matrix product")
    ap.add_argument("--no-decode", action="store_true", help="skip the 36-layer decoder (tokens/s)")
    ap.add_argument("--no-lm-head", action="store_true", help="skip the 152064x3584 launch")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path, run with --gpus 1")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")

    from bf16_huffman_infer_amd import _lib
    _lib.load()                                   # fail before any work if the HIP library is missing
    import torch.nn.functional as F
    from bf16_huffman_infer_amd.functional import linear_grouped

    device = torch.device("cuda", 0)
    bs = args.batch
    blocks = [build_block(args.algo, device, c) for c in range(COPIES)]
    xs = [torch.randn(bs, K, device=device).bfloat16() for _, _, K in LAYERS]
    block_bytes = sum(gemv_bytes(m, bs, M, K) for m, (_, M, K) in zip(blocks[0], LAYERS))
    raw_bytes = sum(M * K * 2 for _, M, K in LAYERS)

    # parity gate inside the benchmark: one layer must decode bit-exactly
    w0 = make_weight(LAYERS[1][1], LAYERS[1][2], 1, device)
    assert torch.equal(blocks[0][1].get_weight().view(torch.int16), w0.view(torch.int16)), "decode is not lossless"
    del w0

    # A plain device copy of known size (256 MiB read, 256 MiB written).  It is not timed;
    # it gives hardware-counter runs of this script a kernel whose HBM traffic is known,
    # against which the FETCH_SIZE / WRITE_SIZE readings of the GEMV kernel are scaled.
    cal = torch.zeros(64 << 20, dtype=torch.int32, device=device)
    cal.clone()
    del cal

    state = {"i": 0}

    def step_single():
        mods = blocks[state["i"] % COPIES]
        state["i"] += 1
        for m, x in zip(mods, xs):
            F.linear(x, m)

    # gate_proj and up_proj multiply the same activations: one grouped launch, as in a
    # decoder whose projections were tied by cudastream_utils.parallelize_qkv_model
    def step_grouped():
        mods = blocks[state["i"] % COPIES]
        state["i"] += 1
        F.linear(xs[0], mods[0])
        F.linear(xs[1], mods[1])
        linear_grouped(xs[2], [mods[2], mods[3]])
        F.linear(xs[4], mods[4])

    spread = {}
    sec_single = time_launches(step_single, args.steps, args.warmup, launches_per_graph=STEPS_PER_GRAPH, spread=spread)
    sec = sec_single if args.no_group else time_launches(step_grouped, args.steps, args.warmup, launches_per_graph=STEPS_PER_GRAPH,
                                                         spread=spread)
    gbs = block_bytes / sec / 1e9

    # Per-layer timing and the roofline of the dominant kernel.  A layer alone must not be
    # served by the 256 MB last-level cache either: it rotates over clones of its module
    # (same bytes at different addresses) that add up to at least ROTATE_BYTES.
    import copy

    def rotating(mod):
        n = max(2, -(-ROTATE_BYTES // weight_bytes(mod)))
        return [mod] + [copy.deepcopy(mod) for _ in range(n - 1)]

    per_layer = {}
    t_dom = None
    for li, (name, M, K) in enumerate(LAYERS):
        if li == 3:                               # up_proj is gate_proj's twin: same shape, same kernel
            per_layer[name] = per_layer["gate_proj"]
            continue
        mods = rotating(blocks[0][li])
        st = {"i": 0}

        def one(li=li, st=st, mods=mods):
            F.linear(xs[li], mods[st["i"] % len(mods)])
            st["i"] += 1
        per_layer[name] = time_launches(one, max(100, args.steps), args.warmup, launches_per_graph=GRAPH_ROTATIONS * len(mods))
        if li == 2:
            t_single = per_layer[name]
            # the launch that dominates the step: gate_proj and up_proj as one group, again
            # rotating over clones (of both) so that no cache level holds the weights
            ups = rotating(blocks[0][3])[:len(mods)]
            sg = {"i": 0}

            def pair(sg=sg, mods=mods, ups=ups):
                i = sg["i"] % len(ups)
                linear_grouped(xs[2], [mods[i], ups[i]])
                sg["i"] += 1
            t_group = time_launches(pair, max(100, args.steps), args.warmup, launches_per_graph=GRAPH_ROTATIONS * len(ups))
            del ups
        del mods
    single_bytes = gemv_bytes(blocks[0][2], bs, LAYERS[2][1], LAYERS[2][2])
    group_bytes = single_bytes + gemv_bytes(blocks[0][3], bs, LAYERS[3][1], LAYERS[3][2]) - bs * LAYERS[3][2] * 2  # X once
    if args.no_group:
        dom_bytes, t_dom, dom_name = single_bytes, t_single, "18944x3584"
    else:
        dom_bytes, t_dom, dom_name = group_bytes, t_group, "group of two 18944x3584 (gate_proj + up_proj)"
    achieved = dom_bytes / t_dom / 1e9

    out = {
        "metric": "fused decode-GEMV GB/s (compressed bytes, % HBM peak); bs=1 tokens/s",
        "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(sec * 1e3, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"Qwen2.5-7B decoder-block linears (qkv 4608x3584, o 3584x3584, gate/up 18944x3584, "
                               f"down 3584x18944), N(0,0.02) seeded, algo={args.algo}, batch={bs}, {COPIES} "
                               f"alternating weight copies, "
                               f"{'5 launches' if args.no_group else '4 launches (gate+up grouped)'} per step"},
        # ms_per_step is the median of this many timed regions of --steps steps; fastest and slowest beside it
        "ms_per_step_rounds": {"rounds": spread["rounds"], "steps_per_round": spread["calls_per_round"],
                               "min": round(spread["min"] * 1e3, 5), "max": round(spread["max"] * 1e3, 5)},
        "clock_warmup_ms": CLOCK_WARMUP_S * 1e3,   # untimed replays before every timed region, on top of --warmup
        "ms_per_step_single_launches": round(sec_single * 1e3, 5),
        "pct_hbm_peak": round(100 * gbs / HBM_PEAK_GBS, 2),
        "compressed_bytes_per_step": block_bytes, "compression_ratio": round(
            sum(weight_bytes(m) for m in blocks[0]) / raw_bytes, 4),
        "block_steps_per_s": round(1.0 / sec, 1),
        # DERIVED, not measured: 28 such blocks make one Qwen2.5-7B token (attention, norms, embedding and
        # lm_head not included); the measured tokens/s of a whole decoder is in "decode"
        "bs1_tokens_per_s_28_blocks_derived": round(1.0 / sec / 28, 1),
        "us_per_layer": {k: round(v * 1e6, 2) for k, v in per_layer.items()},
        "roofline": {"bound": "hbm", "kernel": f"bhi::gemv_kernel<bhi::{dict(huffman='HuffCodec', ans='AnsCodec', nibble='NibbleCodec')[args.algo]}, {bs}, 4, {2 if args.no_group else 4}> "
                               f"{dom_name}",
                     "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": measured_traffic((args.algo, bs, "single" if args.no_group else "group")),
                     "bytes_per_launch": dom_bytes, "us_per_launch": round(t_dom * 1e6, 2)},
        # the same kernel launched for one 18944x3584 matrix alone
        "single_launch": {"achieved": round(single_bytes / t_single / 1e9, 1),
                          "frac": round(single_bytes / t_single / 1e9 / HBM_PEAK_GBS, 4),
                          "traffic": measured_traffic((args.algo, bs, "single")),
                          "bytes_per_launch": single_bytes, "us_per_launch": round(t_single * 1e6, 2)},
    }
    out["roofline"]["traffic_from"] = (f"rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this script on kernel sources "
                                       f"{MEASURED_TRAFFIC_SOURCES}; sources now {kernel_sources_digest()}")
    out["load_only"] = load_only(single_bytes, args, device)
    del per_layer
    if not args.no_sweep and args.algo == "huffman" and bs == 1:
        out["sweep"] = sweep(args, device, blocks)
    del blocks
    torch.cuda.empty_cache()
    if not args.no_lm_head:
        out["lm_head"] = lm_head(args, device)
        torch.cuda.empty_cache()
    if not args.no_fallback:
        # more than 8 rows of X: the fused decode + matrix-core product beside decode-to-BF16 + dense GEMM
        from bench_fallback import measure
        out["fallback"] = measure(device, with_library_gemm=True, steps=max(50, args.steps // 2))
        torch.cuda.empty_cache()
    if not args.no_decode:
        # the tokens/s half of the metric, measured: Qwen3-8B-shaped decoder, 36 layers, algo=smallest,
        # recorded step, 256 greedy tokens; teacher-forced logits against the raw model
        import bench_decode
        out["decode"] = bench_decode.run(bench_decode.parse_args([]))
        torch.cuda.empty_cache()
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out, allow_nan=False))


if __name__ == "__main__":
    main()
