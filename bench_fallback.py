"""More than 8 rows of X: the fused decode + matrix-core product (9..32 rows) beside the
path it replaces, decode the compressed weight to BF16, then a dense BF16 GEMM.

Workload: 12288x4096 and 4096x12288 linears with heavy-tailed weights (Student-t, nu=3,
scaled to std 0.02: long codes and escapes), batch 16 and 32.  For each: the decode kernel
alone (GB/s on compressed bytes read + BF16 bytes written), the GEMM alone (TFLOP/s and the
fraction of the 2.5 PFLOP/s dense BF16 peak; at batch b the GEMM cannot exceed b/312 of
that peak even with perfect streaming of the weight), the two together as the reference's
path runs them (``F.linear(x, module.get_weight())``), and the fused kernel that
``F.linear(x, module)`` now takes: time, GB/s on compressed bytes + X + Y, and its MFMA
utilisation (useful flops: the 4x4x4 blocks are full, every product counts).  Every layer rotates over clones adding up to 640 MB so
that the last-level cache does not serve the weights.  One JSON line per (shape, batch).
"""
import copy
import json
import os
import sys

import torch
import torch.nn.functional as F

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
from bench import ROTATE_BYTES, time_launches, weight_bytes  # noqa: E402

MFMA_PEAK_TFLOPS = 2500.0


def student_t(M, K, seed, device):
    g = torch.Generator(device="cpu").manual_seed(seed)
    t = torch.distributions.StudentT(3.0)
    torch.manual_seed(seed)
    w = t.sample((M, K)) * (0.02 / 3 ** 0.5)
    return w.bfloat16().to(device)


def measure(device, shapes=((12288, 4096), (4096, 12288)), batches=(16, 32), with_library_gemm=True, steps=100):
    """One dict per (shape, batch); ``with_library_gemm=False`` skips the timings of the decode
    kernel alone and of the dense GEMM alone."""
    from bf16_huffman_infer_amd.functional import HuffmanWeight
    results = []
    for (M, K) in shapes:
        w = student_t(M, K, 7, device)
        mod = HuffmanWeight.compress(w).to(device)
        assert torch.equal(mod.get_weight().view(torch.int16), w.view(torch.int16)), "decode is not lossless"
        n = max(2, -(-ROTATE_BYTES // weight_bytes(mod)))
        mods = [mod] + [copy.deepcopy(mod) for _ in range(n - 1)]
        dense = [w] + [w.clone() for _ in range(max(2, -(-ROTATE_BYTES // (2 * M * K))) - 1)]
        st = {"i": 0}

        def decode_only():
            mods[st["i"] % len(mods)].get_weight()
            st["i"] += 1
        t_dec = time_launches(decode_only, steps, 10, launches_per_graph=len(mods)) if with_library_gemm else None
        dec_bytes = weight_bytes(mod) + 2 * M * K
        for bs in batches:
            x = torch.randn(bs, K, device=device).bfloat16()

            def gemm_only():
                F.linear(x, dense[st["i"] % len(dense)])
                st["i"] += 1

            def fallback():
                m = mods[st["i"] % len(mods)]
                F.linear(x, m.get_weight())
                st["i"] += 1

            def fused():
                F.linear(x, mods[st["i"] % len(mods)])
                st["i"] += 1
            t_gemm = time_launches(gemm_only, steps, 10, launches_per_graph=len(dense)) if with_library_gemm else None
            t_all = time_launches(fallback, steps, 10, launches_per_graph=len(mods))
            t_fused = time_launches(fused, steps, 10, launches_per_graph=len(mods))
            flops = 2.0 * bs * M * K
            fused_bytes = weight_bytes(mod) + 2 * bs * (M + K)
            results.append({
                "shape": f"{M}x{K}", "batch": bs, "weights": "Student-t nu=3, std 0.02",
                "compressed_ratio": round(weight_bytes(mod) / (2 * M * K), 4),
                # (None: the timings of the two kernels alone were skipped)
                "decode_us": t_dec and round(t_dec * 1e6, 2), "decode_GBps": t_dec and round(dec_bytes / t_dec / 1e9, 1),
                "decode_frac_of_hbm_peak": t_dec and round(dec_bytes / t_dec / 8e12, 4),
                "gemm_us": t_gemm and round(t_gemm * 1e6, 2), "gemm_TFLOPs": t_gemm and round(flops / t_gemm / 1e12, 2),
                "mfma_utilisation": t_gemm and round(flops / t_gemm / 1e12 / MFMA_PEAK_TFLOPS, 5),
                "mfma_cap_at_this_batch": round(bs / 312.5, 4),
                "decode_then_gemm_us": round(t_all * 1e6, 2),
                "fused_us": round(t_fused * 1e6, 2), "fused_GBps": round(fused_bytes / t_fused / 1e9, 1),
                "fused_frac_of_hbm_peak": round(fused_bytes / t_fused / 8e12, 4),
                "fused_TFLOPs": round(flops / t_fused / 1e12, 2),
                "fused_mfma_utilisation": round(flops / t_fused / 1e12 / MFMA_PEAK_TFLOPS, 5),
            })
        del mods, dense
    return results


def main():
    if not torch.cuda.is_available():
        sys.exit("bench_fallback.py needs a GPU")
    from bf16_huffman_infer_amd import _lib
    _lib.load()
    for r in measure(torch.device("cuda", 0)):
        print(json.dumps(r, allow_nan=False), flush=True)


if __name__ == "__main__":
    main()
