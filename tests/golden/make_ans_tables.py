"""Writes ans_tables.json: histogram -> quantised rANS frequencies, produced by the
reference's own table builder (bf16_huffman_infer/ans.py:6-80, RANSEncoder with
precision 8).  Runs only where the reference checkout is present; the committed JSON is
what the tests read.

The exact hand-out order of the rounding fix-up (ties between equal remainders) is the
one thing about these tables that invariants alone do not pin, hence the vectors.
"""
import types
import json
import os
import sys

import numpy as np

REF = "/root/reference/bf16_huffman_infer/ans.py"
HERE = os.path.dirname(os.path.abspath(__file__))


def histograms():
    rng = np.random.default_rng(20240607)
    out = {}
    # exponent histogram of N(0, 0.02) BF16 weights (1M samples)
    import torch
    g = torch.Generator().manual_seed(3)
    w = (torch.randn(1 << 20, generator=g) * 0.02).bfloat16().view(torch.int16).numpy().view(np.uint16)
    out["gaussian_exponents"] = np.bincount((w >> 7) & 0xFF, minlength=256)
    # heavy tail: Student-t nu=3
    t = torch.distributions.StudentT(3.0).sample((1 << 20,)) * (0.02 / 3 ** 0.5)
    w = t.bfloat16().view(torch.int16).numpy().view(np.uint16)
    out["student_t_exponents"] = np.bincount((w >> 7) & 0xFF, minlength=256)
    # many equal counts: every remainder ties
    out["uniform_200"] = np.concatenate([np.full(200, 7), np.zeros(56, dtype=np.int64)])
    # all 256 symbols present, one dominant (forces the take-back branch)
    c = rng.integers(1, 4, size=256)
    c[17] = 100000
    out["dominant_plus_255_rare"] = c
    # the documented sample of ans.py:152
    out["readme_sample"] = np.bincount([1, 2, 3, 3, 2, 12, 13, 11, 1, 8, 1, 7, 1, 6, 1, 1], minlength=256)
    return {k: [int(x) for x in v] for k, v in out.items()}


def main():
    # Run the SOURCE text: the import machinery would pick the reference's shipped bytecode
    # cache (__pycache__/*.pyc) whenever its header matches the source file.
    mod = types.ModuleType("reference_ans")
    mod.__file__ = REF
    with open(REF) as fh:
        exec(compile(fh.read(), REF, "exec"), mod.__dict__)
    import torch
    torch.manual_seed(11)
    vectors = {}
    for name, counts in histograms().items():
        enc = mod.RANSEncoder(counts, precision=8)
        vectors[name] = {"counts": counts, "freq": [int(f) for f in enc.freq], "cum": [int(c) for c in enc.cum]}
    with open(os.path.join(HERE, "ans_tables.json"), "w") as f:
        json.dump(vectors, f, separators=(",", ":"))
    print("wrote", len(vectors), "vectors")


if __name__ == "__main__":
    sys.exit(main())
