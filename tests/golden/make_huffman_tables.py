"""Writes huffman_tables.json: exponent histogram -> the reference's decomposed decode
tables (LUT1..LUT4, code_lengths) and codes, produced by the reference's own builder
(bf16_huffman_infer/huffman.py:347-361).  Runs only where the reference checkout is
present; the committed JSON is what the tests read.

The vectors pin the table-fill rule and the decoder cascade of the numpy restatement
against real reference tables (its heap tie-breaks and perturbation trajectory cannot be
derived from invariants).
"""
import types
import json
import os
import sys

import numpy as np
import torch

REF = "/root/reference/bf16_huffman_infer/huffman.py"
HERE = os.path.dirname(os.path.abspath(__file__))


def exponent_histogram(values: torch.Tensor) -> np.ndarray:
    w = values.bfloat16().view(torch.int16).numpy().view(np.uint16)
    return np.bincount((w >> 7) & 0xFF, minlength=256)


def histograms():
    g = torch.Generator().manual_seed(5)
    out = {"gaussian_exponents": exponent_histogram(torch.randn(1 << 22, generator=g) * 0.02)}
    torch.manual_seed(6)
    t = torch.distributions.StudentT(3.0).sample((1 << 22,)) * (0.02 / 3 ** 0.5)
    out["student_t_exponents"] = exponent_histogram(t)
    # powers of two: a 30-level tree, so codes reach the fourth byte table.  (Deeper
    # inputs, e.g. 34 Fibonacci weights, make the reference's length limiter give up with
    # an AssertionError at huffman.py:121 -- it lowers the weight of the deepest symbol,
    # which cannot shorten its code.)
    c = np.zeros(256, dtype=np.int64)
    c[100:130] = 2 ** np.arange(30)
    out["powers_of_two_30"] = c
    u = np.zeros(256, dtype=np.int64)
    u[:] = 3
    out["flat_256"] = u
    return {k: [int(x) for x in v] for k, v in out.items()}


def main():
    # Run the SOURCE text: the import machinery would pick the reference's shipped bytecode
    # cache (__pycache__/*.pyc) whenever its header matches the source file.
    mod = types.ModuleType("reference_huffman")
    mod.__file__ = REF
    with open(REF) as fh:
        exec(compile(fh.read(), REF, "exec"), mod.__dict__)
    vectors = {}
    for name, counts in histograms().items():
        enc = mod.LUTHuffmanEncoder()
        enc.build_lut(np.asarray(counts))
        vectors[name] = {
            "counts": counts,
            "LUT1": [int(x) for x in enc.LUT1], "LUT2": [int(x) for x in enc.LUT2],
            "LUT3": [int(x) for x in enc.LUT3], "LUT4": [int(x) for x in enc.LUT4],
            "code_lengths": [int(x) for x in enc.code_lengths],
            "codes": {str(s): c for s, c in sorted(enc.huffman_codes.items())},
        }
    with open(os.path.join(HERE, "huffman_tables.json"), "w") as f:
        json.dump(vectors, f, separators=(",", ":"))
    print("wrote", len(vectors), "vectors")


if __name__ == "__main__":
    sys.exit(main())
