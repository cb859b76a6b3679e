"""The reference's two table builders, restated (oracle; test infrastructure only).

* ``build_cascade_luts(counts)`` -- the DFloat11-style decomposed Huffman tables of
  ``bf16_huffman_infer/huffman.py``: a Huffman code of at most 32 bits whose codes are
  written root-bit-first into the stream (``:66-82``, bit 0 of the code integer is the
  root branch), adjusted by frequency perturbation until (a) no code is longer than 32
  bits (``:84-123``: the rarest longest symbol is set to weight 1, then 0.5) and (b) no
  two codes of the same byte level claim the same entry of that level's 256-entry table
  (``:125-218``: the most frequent offender gets 1.5x weight), then the table fill of
  ``:220-280``: a code of length L lives in level T = ceil(L/8), indexed by its T-th
  byte with the unused high bits enumerated; 255 marks a miss.
* ``ans_tables(counts, precision)`` -- ``bf16_huffman_infer/ans.py:6-80``: frequencies
  quantised to sum ``2**precision`` (round-half-even, zero -> 1, fix-up in remainder
  order), exclusive prefix ``cum`` and the packed decode word
  ``(sym<<24)|(freq<<12)|rem`` of ``functional.py:286-295``.

Pins.  Huffman: the cascade decodes every code back to its symbol (checked by
``decode_code`` over all symbols), codes are prefix-free with Kraft sum 1, lengths are
within 1 bit of entropy on unperturbed inputs.  The exact tie-breaking of the
reference's heap is NOT reproduced (it does not affect decoded weights):
"parity unpinned" for byte-identical tables.  rANS: the worked example of ``ans.py:152``
(counts x16 exactly -> freq {1:96, 2:32, 3:32, 6..13:16}), sum/positivity/prefix
invariants, slot bijection.
"""
import heapq
from typing import Dict, List, Tuple

import numpy as np


def _huffman_lengths_and_codes(weights: Dict[int, float]) -> Dict[int, Tuple[int, int]]:
    """symbol -> (code integer with the root branch in bit 0, length)."""
    heap = [(w, s, None, None) for s, w in weights.items() if w > 0]
    if len(heap) == 1:
        return {heap[0][1]: (0, 1)}
    heapq.heapify(heap)
    tick = 1 << 20
    while len(heap) > 1:
        a = heapq.heappop(heap)
        b = heapq.heappop(heap)
        tick += 1
        heapq.heappush(heap, (a[0] + b[0], tick, a, b))
    codes: Dict[int, Tuple[int, int]] = {}
    stack = [(heap[0], 0, 0)]
    while stack:
        node, code, depth = stack.pop()
        if node[2] is None:
            codes[node[1]] = (code, depth)
        else:
            stack.append((node[2], code, depth + 1))                  # left branch = bit 0
            stack.append((node[3], code | (1 << depth), depth + 1))   # right branch = bit 1
    return codes


def _limit_length(weights: Dict[int, float], max_len: int = 32) -> Dict[int, float]:
    w = dict(weights)
    for _ in range(50):
        codes = _huffman_lengths_and_codes(w)
        longest = max(l for _, l in codes.values())
        if longest <= max_len:
            return w
        worst = sorted((s for s, (_, l) in codes.items() if l == longest), key=lambda s: w[s])
        for s in worst:
            if w[s] > 1:
                w[s] = 1
                break
        else:
            w[worst[0]] = 0.5
    raise AssertionError("length limit not reached")


def _level_slots(code: int, length: int) -> Tuple[int, np.ndarray]:
    level = (length - 1) // 8
    byte = (code >> (8 * level)) & 0xFF
    used = length - 8 * level
    return level, byte + (np.arange(1 << (8 - used)) << used)


def build_cascade_luts(counts: np.ndarray, strict: bool = False):
    """counts[256] -> (LUT[4][256] uint8, code_lengths[256] uint8, codes {sym: (code, len)}).

    ``strict=False`` is the reference's rule: only two codes of the SAME level may not
    share a slot.  That leaves a hole the reference does not check: a code of level T
    whose earlier byte t < T happens to equal a populated slot of level t is resolved
    too early by the decoder cascade.  ``strict=True`` also treats those as clashes.
    """
    w = {int(s): float(c) for s, c in enumerate(counts) if c > 0}
    w = _limit_length(w)
    for _ in range(40 if strict else 20):
        codes = _huffman_lengths_and_codes(w)
        claims: List[Dict[int, List[int]]] = [dict() for _ in range(4)]
        for s, (code, length) in codes.items():
            level, slots = _level_slots(code, length)
            for slot in slots:
                claims[level].setdefault(int(slot), []).append(s)
        clashes = [syms for lvl in claims for syms in lvl.values() if len(syms) > 1]
        if strict:
            for s, (code, length) in codes.items():
                for t in range((length - 1) // 8):
                    early = claims[t].get((code >> (8 * t)) & 0xFF)
                    if early and t > 0:          # level 0 cannot alias: the code is prefix-free
                        clashes.append(early + [s])
        if not clashes:
            break
        for syms in clashes:
            top = max(syms, key=lambda s: w[s])
            w[top] *= 1.5
        w = _limit_length(w)
    else:
        raise AssertionError("table conflicts not resolved")
    luts = np.full((4, 256), 255, dtype=np.uint8)
    lens = np.zeros(256, dtype=np.uint8)
    for s, (code, length) in codes.items():
        lens[s] = length
        level, slots = _level_slots(code, length)
        luts[level, slots] = s
    return luts, lens, codes


def decode_code(luts: np.ndarray, lens: np.ndarray, window: int) -> Tuple[int, int]:
    """The decoder rule of ``src/kernel.cu:370-377`` on a 32-bit window: (symbol, length)."""
    for level in range(4):
        s = int(luts[level, (window >> (8 * level)) & 0xFF])
        if s != 255:
            return s, int(lens[s])
    raise AssertionError("window matches no table level")


def ans_tables(counts, precision: int = 8):
    """counts[256] -> (freq[256], cum[256], lut[2**precision] int32 packed)."""
    base = 1 << precision
    present = [(s, int(c)) for s, c in enumerate(counts) if c > 0]
    total = sum(c for _, c in present)
    scaled, rema = {}, []
    for s, c in present:
        exact = c * base / total
        q = int(round(exact)) or 1
        scaled[s] = q
        rema.append((exact - q, s))
    cur = sum(scaled.values())
    if cur < base:
        rema.sort(reverse=True)
        while cur < base:
            for _, s in rema:
                if cur == base:
                    break
                scaled[s] += 1
                cur += 1
    elif cur > base:
        rema.sort()
        while cur > base:
            for _, s in rema:
                if cur == base:
                    break
                if scaled[s] > 1:
                    scaled[s] -= 1
                    cur -= 1
    freq = np.array([scaled.get(s, 0) for s in range(256)], dtype=np.int64)
    cum = np.cumsum(freq) - freq
    lut = np.zeros(base, dtype=np.int64)
    for s in range(256):
        for r in range(int(freq[s])):
            lut[cum[s] + r] = (s << 24) | (int(freq[s]) << 12) | r
    return freq, cum, lut.astype(np.uint32).view(np.int32)
