"""Host-side table construction for the rANS path.

Counterpart of the reference's ``RANSEncoder.__init__`` / ``_normalize``
(``bf16_huffman_infer/ans.py:6-80``): symbol counts are quantised to frequencies that
sum to ``2**precision`` with every present symbol keeping at least one slot, ``cum`` is
their exclusive prefix sum and ``decode_lut[slot] = (symbol, freq, slot - cum[symbol])``.
The quantisation follows the reference's rule so both produce the same tables from the
same histogram: round half to even, lift zeros to one, then hand out (or take back) the
difference one slot at a time in order of rounding remainder.

Only the tables live here; encoding and decoding run in the HIP kernels.
"""
from typing import Dict, List, Mapping, Sequence, Tuple, Union


class RANSEncoder:
    def __init__(self, freq: Union[Mapping[int, int], Sequence[int]], precision: int = 8):
        if not 1 <= precision <= 12:
            raise ValueError("precision must be in [1, 12]")
        if not isinstance(freq, Mapping):
            freq = {s: int(f) for s, f in enumerate(freq) if f > 0}
        if not freq:
            raise ValueError("freq must not be empty")
        self.precision = precision
        self.base = 1 << precision
        self.mask = self.base - 1

        scaled = self._normalize(freq)
        self.freq: List[int] = [scaled.get(s, 0) for s in range(256)]
        self.cum: List[int] = []
        running = 0
        for f in self.freq:
            self.cum.append(running)
            running += f
        self.decode_lut: List[Tuple[int, int, int]] = [
            (s, f, r) for s, f in enumerate(self.freq) for r in range(f)
        ]

    def _normalize(self, freq: Mapping[int, int]) -> Dict[int, int]:
        total = sum(freq.values())
        if total <= 0:
            raise ValueError("sum of frequencies must be positive")
        if len(freq) > self.base:
            raise ValueError("more symbols than slots")
        scaled: Dict[int, int] = {}
        remainders = []
        for sym, count in freq.items():
            if count <= 0:
                raise ValueError(f"frequency of symbol {sym} must be positive")
            exact = count * self.base / total
            slots = max(int(round(exact)), 1)          # round() is round-half-even
            scaled[sym] = slots
            remainders.append((exact - slots, sym))

        current = sum(scaled.values())
        if current < self.base:
            remainders.sort(reverse=True)               # most under-served first
            while current < self.base:
                for _, sym in remainders:
                    if current == self.base:
                        break
                    scaled[sym] += 1
                    current += 1
        elif current > self.base:
            remainders.sort()                           # most over-served first
            while current > self.base:
                for _, sym in remainders:
                    if current == self.base:
                        break
                    if scaled[sym] > 1:
                        scaled[sym] -= 1
                        current -= 1
        assert sum(scaled.values()) == self.base
        return scaled
