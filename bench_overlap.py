"""Can the weight stream of launch N+1 start while launch N drains?  Two measurements on the
Qwen2.5-7B block step of ``bench.py`` (batch 1, Huffman), both with committed entry points only:

* ``side_branch``: the recorded graph forks before every GEMV launch; the side stream reads the
  first ``cap`` bytes of the NEXT launch's weights (``bhi_stream_read``, the library's load-only
  kernel) while the main stream runs the current launch, and joins at the end of the step.
  The weights do not depend on the activations, so the read is legal at any time; whether it
  pays is a question of what the GPU does with two kernels of one graph at once.
* ``warm_in_line``: the same read on the main stream, right in front of the launch that uses the
  bytes (no overlap at all): what a launch gains from finding its first ``cap`` bytes in the
  last-level cache, and what the extra kernel costs.

One JSON line per variant: us per block step and GB/s on the block's compressed bytes.

    python bench_overlap.py [--steps 200]
"""
import argparse
import json
import statistics

import torch
import torch.nn.functional as F

import bench
from bf16_huffman_infer_amd import _lib
from bf16_huffman_infer_amd.functional import linear_grouped


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--rounds", type=int, default=7)
    args = ap.parse_args()
    lib = _lib.load()
    dev = torch.device("cuda", 0)
    blocks = [bench.build_block("huffman", dev, c) for c in range(bench.COPIES)]
    xs = [torch.randn(1, K, device=dev).bfloat16() for _, _, K in bench.LAYERS]
    sink = torch.zeros(1, dtype=torch.int32, device=dev)
    block_bytes = sum(bench.gemv_bytes(m, 1, M, K) for m, (_, M, K) in zip(blocks[0], bench.LAYERS))

    def launches(mods):
        # the four launches of a step with the weight modules each of them reads
        return [(lambda: F.linear(xs[0], mods[0]), [mods[0]]),
                (lambda: F.linear(xs[1], mods[1]), [mods[1]]),
                (lambda: linear_grouped(xs[2], [mods[2], mods[3]]), [mods[2], mods[3]]),
                (lambda: F.linear(xs[4], mods[4]), [mods[4]])]

    def read(mods, cap, waves, stream):
        left = cap
        for m in mods:
            for t in (m.rem, m.exp):
                n = min(left, t.numel() * t.element_size()) // (waves * 1024) * (waves * 1024)
                if n <= 0:
                    continue
                got = lib.bhi_stream_read(t.data_ptr(), n, waves, 0, sink.data_ptr(), stream.cuda_stream)
                assert got > 0, got
                left -= n

    def graph_of(mode, cap, waves):
        side = torch.cuda.Stream()

        def body():
            main_stream = torch.cuda.current_stream()
            seq = [l for c in range(bench.COPIES) for l in launches(blocks[c])]
            for i, (fn, mods) in enumerate(seq):
                if mode == "side_branch":
                    side.wait_stream(main_stream)
                    read(seq[(i + 1) % len(seq)][1], cap, waves, side)
                elif mode == "warm_in_line":
                    read(mods, cap, waves, main_stream)
                fn()
            if mode == "side_branch":
                main_stream.wait_stream(side)
        warm = torch.cuda.Stream()
        warm.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(warm):
            body()
        torch.cuda.current_stream().wait_stream(warm)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            body()
        return g

    variants = {"base": ("none", 0, 512)}
    for cap in (2 << 20, 16 << 20, 1 << 30):
        variants[f"side_branch_{cap >> 20}MiB"] = ("side_branch", cap, 1024)
    for cap in (2 << 20, 16 << 20):
        variants[f"warm_in_line_{cap >> 20}MiB"] = ("warm_in_line", cap, 1024)
    graphs = {k: graph_of(*v) for k, v in variants.items()}
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for g in graphs.values():                      # steady clocks before anything is timed
        for _ in range(300):
            g.replay()
    torch.cuda.synchronize()
    replays = max(1, args.steps // bench.COPIES)
    times = {k: [] for k in graphs}
    for _ in range(args.rounds):                   # variants take turns, round by round
        for k, g in graphs.items():
            for _ in range(10):
                g.replay()
            start.record()
            for _ in range(replays):
                g.replay()
            stop.record()
            torch.cuda.synchronize()
            times[k].append(start.elapsed_time(stop) * 1e3 / (replays * bench.COPIES))
    for k, v in times.items():
        med = statistics.median(v)
        print(json.dumps({"variant": k, "us_per_step": round(med, 2), "GBps": round(block_bytes / med / 1e3, 1),
                          "min_us": round(min(v), 2), "max_us": round(max(v), 2), "rounds": len(v),
                          "steps_per_graph": bench.COPIES}), flush=True)


if __name__ == "__main__":
    main()
