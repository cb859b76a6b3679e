"""Host-side code construction for the Huffman path.

Counterpart of the reference's ``LUTHuffmanEncoder.build_lut``
(``bf16_huffman_infer/huffman.py:347-361``), redesigned for a 64-lane decoder: the
coded alphabet is the set of exponent *pairs* ``a | b<<8`` (two horizontally adjacent
weights), every code is at most 11 bits long, and one 2048-entry table resolves the
next 11 stream bits to both exponents at once.  The reference instead limits single
symbol codes to 32 bits and perturbs the frequencies until the codes fit four
256-entry byte tables (``huffman.py:84-218``); that cascade costs two dependent
shared-memory reads per exponent, here one read yields two exponents.

Pairs that are too rare to deserve a code share one ESC code; their two raw bytes
travel in a side list of the stream, so the in-band cost of any pair is bounded by
11 bits and the decoder's bit window never overflows.
"""
from typing import Dict, Tuple, Union

import numpy as np
import torch

TABLE_BITS = 11
ESC_FLAG = 1 << 31
ESC_INDEX = 65536
ESC_SIDE_BITS = 32            # one stream word per escaped pair
MAX_CODED = 1536              # never give more than this many pairs a code of their own
ESC_FREE_SHIFT = 5            # an escape-free code may be 1/32 longer than the shortest one


def package_merge(weights, max_len: int):
    """Optimal code lengths under a length limit (Larmore-Hirschberg package-merge).

    ``weights``: positive numbers, at most ``2**max_len`` of them.  Returns a list of
    lengths with Kraft sum 1 (for two or more symbols).
    """
    n = len(weights)
    assert 2 <= n <= (1 << max_len)
    order = sorted(range(n), key=lambda i: (weights[i], i))
    # a node is (weight, left, right) for a package or (weight, symbol) for a leaf
    leaves = [(weights[i], i) for i in order]
    cur = leaves
    for _ in range(max_len - 1):
        packs = [(cur[j][0] + cur[j + 1][0], cur[j], cur[j + 1]) for j in range(0, len(cur) - 1, 2)]
        merged, i, j = [], 0, 0
        while i < n and j < len(packs):
            if leaves[i][0] <= packs[j][0]:
                merged.append(leaves[i]); i += 1
            else:
                merged.append(packs[j]); j += 1
        merged.extend(leaves[i:])
        merged.extend(packs[j:])
        cur = merged
    lengths = [0] * n
    stack = list(cur[:2 * n - 2])
    while stack:
        node = stack.pop()
        if len(node) == 2:
            lengths[node[1]] += 1
        else:
            stack.append(node[1]); stack.append(node[2])
    return lengths


def _bit_reverse(v: int, n: int) -> int:
    r = 0
    for _ in range(n):
        r = (r << 1) | (v & 1)
        v >>= 1
    return r


class LUTHuffmanEncoder:
    """Pair-alphabet, 11-bit-limited canonical Huffman code with its two tables.

    After :meth:`build_lut`:

    * ``enc_table``  uint32 ``[65537]``: ``code | len<<16`` per pair (0 = escaped), ESC in
      slot 65536; code bits are emitted LSB first.
    * ``dec_table``  uint32 ``[2048]``: ``len | a<<7 | b<<23`` (``| 1<<31`` for ESC): the two
      exponents already sit at their BF16 bit positions of a packed pair.
    * ``LUT1``       the decode table viewed as uint8 ``[8192]`` -- the module buffer.
    * ``LUT2..LUT4`` uint8 ``[256]`` filled with 255: the reference's deeper cascade
      levels have no job when no code is longer than the first-level window.
    * ``code_lengths`` uint8 ``[256]``: a format header (version, table bits, ESC length,
      whether any pair of the histogram is escaped).
    """

    def __init__(self, max_code_length: int = TABLE_BITS):
        assert max_code_length == TABLE_BITS
        self.max_code_length = max_code_length
        self.enc_table = np.zeros(ESC_INDEX + 1, dtype=np.uint32)
        self.dec_table = np.zeros(1 << TABLE_BITS, dtype=np.uint32)
        self.LUT2 = np.full(256, 255, dtype=np.uint8)
        self.LUT3 = np.full(256, 255, dtype=np.uint8)
        self.LUT4 = np.full(256, 255, dtype=np.uint8)
        self.code_lengths = np.zeros(256, dtype=np.uint8)
        self.expected_bits = 0

    @property
    def LUT1(self) -> np.ndarray:
        return self.dec_table.view(np.uint8)

    @property
    def huffman_codes(self) -> Dict[int, str]:
        """pair id (or 65536 for ESC) -> code as a bit string in stream order."""
        out = {}
        for p in np.nonzero(self.enc_table >> 16)[0]:
            code, ln = int(self.enc_table[p]) & 0xFFFF, int(self.enc_table[p]) >> 16
            out[int(p)] = ''.join('1' if (code >> i) & 1 else '0' for i in range(ln))
        return out

    @staticmethod
    def _lengths_for(counts: np.ndarray, coded: np.ndarray) -> Tuple[list, int]:
        """Code lengths for ``coded`` pairs + ESC, and the total cost in bits."""
        esc_count = int(counts.sum() - counts[coded].sum())
        weights = [int(c) for c in counts[coded]] + [max(esc_count, 1)]
        lengths = package_merge(weights, TABLE_BITS)
        bits = sum(w * l for w, l in zip(weights[:-1], lengths[:-1]))
        bits += esc_count * (lengths[-1] + ESC_SIDE_BITS)
        return lengths, bits

    def build_lut(self, frequencies: Union[np.ndarray, torch.Tensor]) -> None:
        """``frequencies``: 65536 pair counts, index ``a | b<<8``."""
        if torch.is_tensor(frequencies):
            frequencies = frequencies.cpu().numpy()
        counts = np.asarray(frequencies, dtype=np.int64).reshape(-1)
        assert counts.shape == (65536,) and counts.min() >= 0

        present = np.nonzero(counts)[0]
        present = present[np.argsort(-counts[present], kind='stable')]      # most frequent first
        # candidate cut-offs: everything, or only pairs seen at least 2/4/16 times
        best = free = last = None
        for thr in (1, 2, 4, 16):
            coded = present[counts[present] >= thr][:MAX_CODED]
            if len(coded) == 0:
                coded = present[:1]
            if last is not None and len(coded) == last:
                continue
            last = len(coded)
            lengths, bits = self._lengths_for(counts, coded)
            if len(coded) == len(present):
                free = (coded, lengths, bits)           # every pair has a code: nothing escapes
            if best is None or bits < best[2]:
                best = (coded, lengths, bits)
        # A matrix whose header says "no escapes" is decoded by kernels without the escape
        # test: one test and one branch less in every step, 6-9 % of a fused GEMV.  Rare
        # pairs crowd the 11-bit code space, so the escape-free code is a little longer
        # (2 % on Gaussian weights); it is taken unless it costs more than 1/32.
        if free is not None and free[2] <= best[2] + (best[2] >> ESC_FREE_SHIFT):
            best = free
        coded, lengths, self.expected_bits = best

        # canonical assignment: shorter codes first, ties by pair id, ESC last in its class
        ids = [int(p) for p in coded] + [ESC_INDEX]
        order = sorted(range(len(ids)), key=lambda i: (lengths[i], ids[i]))
        self.enc_table[:] = 0
        self.dec_table[:] = 0
        code, prev_len = 0, lengths[order[0]]
        filled = np.zeros(1 << TABLE_BITS, dtype=bool)
        for i in order:
            ln = lengths[i]
            code <<= (ln - prev_len)
            prev_len = ln
            rev = _bit_reverse(code, ln)
            sym = ids[i]
            self.enc_table[sym] = rev | (ln << 16)
            idx = rev + (np.arange(1 << (TABLE_BITS - ln)) << ln)
            if sym == ESC_INDEX:
                self.dec_table[idx] = ln | ESC_FLAG
            else:
                self.dec_table[idx] = ln | ((sym & 0xFF) << 7) | ((sym >> 8) << 23)
            filled[idx] = True
            code += 1
        assert filled.all() and code == (1 << prev_len), "code is not complete"

        self.code_lengths[:] = 0
        self.code_lengths[0] = 2                      # format version
        self.code_lengths[1] = TABLE_BITS
        self.code_lengths[2] = int(self.enc_table[ESC_INDEX]) >> 16
        self.code_lengths[3] = 1 if int(counts.sum() - counts[coded].sum()) > 0 else 0   # escapes occur
