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
        """Counts -> slots summing to ``2**precision`` (same result as the reference's
        fix-up loop, written as whole passes over the symbols in remainder order)."""
        total = sum(freq.values())
        if total <= 0:
            raise ValueError("sum of frequencies must be positive")
        if len(freq) > self.base:
            raise ValueError("more symbols than slots")
        if min(freq.values()) <= 0:
            bad = min(freq, key=freq.get)
            raise ValueError(f"frequency of symbol {bad} must be positive")

        exact = {s: c * self.base / total for s, c in freq.items()}
        slots = {s: max(int(round(v)), 1) for s, v in exact.items()}     # round() is half-to-even
        missing = self.base - sum(slots.values())
        if missing > 0:
            # most under-served symbol first; every pass hands one slot to each symbol
            order = sorted(slots, key=lambda s: (exact[s] - slots[s], s), reverse=True)
            rounds, extra = divmod(missing, len(order))
            for i, s in enumerate(order):
                slots[s] += rounds + (1 if i < extra else 0)
        elif missing < 0:
            # most over-served symbol first; a symbol never drops below one slot
            order = sorted(slots, key=lambda s: (exact[s] - slots[s], s))
            surplus = -missing
            while surplus:
                for s in order:
                    if surplus and slots[s] > 1:
                        slots[s] -= 1
                        surplus -= 1
        assert sum(slots.values()) == self.base
        return slots
