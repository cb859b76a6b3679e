"""Writes wave64_digests.json: SHA-256 of the compressed buffers (rem, exp, offsets and the
decode table) of small seeded matrices in this package's stream format, for the three codecs.

The digests freeze the format: a change of the layout, of the chunking rule, of a table
builder's tie-breaks or of an encoder shows up as a different digest both in the numpy model
(`oracle/wave64.py`, CPU test) and in the HIP encoders (GPU test).  Regenerate only with a
format revision:  python tests/golden/make_wave64_digests.py
"""
import hashlib
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

CASES = [("gauss", 128, 1024, 1, 3), ("t3", 128, 768, 2, 4), ("bits", 128, 384, 1, 5), ("gauss", 1024, 4096, 1, 6)]


def sha(a: np.ndarray) -> str:
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def digests():
    from helpers import bits_of, gaussian_weight, pair_counts, random_bits_weight, student_t_weight
    from bf16_huffman_infer_amd.ans import RANSEncoder
    from bf16_huffman_infer_amd.huffman import LUTHuffmanEncoder
    from oracle import planes, wave64
    makers = {"gauss": gaussian_weight, "t3": student_t_weight, "bits": random_bits_weight}
    out = {}
    for kind, M, K, split_k, seed in CASES:
        bits = bits_of(makers[kind](M, K, seed=seed))
        _, exp = planes.split_bf16(bits)
        counts = np.bincount(exp.reshape(-1), minlength=256)
        entry = {}
        huff = LUTHuffmanEncoder()
        huff.build_lut(pair_counts(bits))
        enc = wave64.encode(bits, split_k, huff.enc_table)
        entry["huffman"] = {"rem": sha(enc["rem"]), "exp": sha(enc["exp"]), "offsets": sha(enc["offsets"]),
                            "table": sha(huff.LUT1), "exp_words": int(enc["exp"].size)}
        ans = RANSEncoder(counts.tolist(), precision=8)
        freq, cum = np.array(ans.freq, dtype=np.int64), np.array(ans.cum, dtype=np.int64)
        enc = wave64.encode_ans(bits, split_k, freq, cum)
        entry["ans"] = {"rem": sha(enc["rem"]), "exp": sha(enc["exp"]), "offsets": sha(enc["offsets"]),
                        "table": sha(freq.astype(np.int32)), "exp_words": int(enc["exp"].size)}
        base = wave64.nibble_base(counts)
        enc = wave64.encode_nibble(bits, split_k, base)
        entry["nibble"] = {"rem": sha(enc["rem"]), "exp": sha(enc["exp"]), "offsets": sha(enc["offsets"]),
                           "table": str(base), "exp_words": int(enc["exp"].size)}
        out[f"{kind}_{M}x{K}_split{split_k}_seed{seed}"] = entry
    return out


if __name__ == "__main__":
    with open(os.path.join(HERE, "wave64_digests.json"), "w") as f:
        json.dump(digests(), f, indent=1, sort_keys=True)
    print("wrote wave64_digests.json")
