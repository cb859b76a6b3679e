"""Compressed-weight modules, conversion and the ``F.linear`` dispatch.

Public surface of the reference's ``bf16_huffman_infer/functional.py``:
``HuffmanWeight``, ``ANSWeight``, ``CompressedLinear``, ``convert``,
``convert_all_linear``, ``linear_huffman`` (plus ``linear_ans``, ``mv_huffman``,
``mv_ans``).  Module buffers keep the reference's names and dtypes
(``rem, exp, offsets, LUT1..LUT4, code_lengths`` / ``rem, exp, offsets, LUT``), the
bytes inside ``rem``/``exp``/``offsets``/``LUT1`` follow the wave64 layout of this
package's HIP kernels.
"""
from typing import Optional

import torch
from torch import Tensor, nn
import torch.nn.functional as F
from tqdm import tqdm

from . import _lib
from .ans import RANSEncoder
from .huffman import LUTHuffmanEncoder
from . import ops as _ops
from .ops import (GEMM_MAX_ROWS, ans_decode, ans_encode, ans_encode_capacity, encode_capacity, gemm_bf16,
                  gemm_bf16_grouped,
                  gemv_bf16_ans, gemv_bf16_grouped, gemv_bf16_huffman, gemv_bf16_nibble, huffman_decode, huffman_encode,
                  nibble_decode, nibble_encode, nibble_encode_capacity)
from .utils import get_block_size_n, split_bf16

ANS_PRECISION = 8
MAX_FUSED_BATCH = 8
GROUP_ROWS = 4
STEP_COLS = 128
LANES = 64
LANE_COLS = 8
ENCODE_PART_BYTES = 256 << 20       # scratch bound per encode call

__all__ = [
    "linear_huffman",
    "linear_ans",
    "linear_nibble",
    "linear_grouped",
    "LinearGroup",
    "HuffmanWeight",
    "ANSWeight",
    "NibbleWeight",
    "CompressedLinear",
    "convert_all_linear",
    "convert",
    "load_compressed_state_dict",
    "check_layout",
]


def _lane_order(plane: Tensor, split_k: int) -> Tensor:
    """[M, K] byte plane -> [split_k, G, S, 64, 8]: (split, row group, step, lane, column)."""
    M, K = plane.shape
    Ks = K // split_k
    G, S = M // GROUP_ROWS, Ks // STEP_COLS
    x = plane.view(G, GROUP_ROWS, split_k, S, STEP_COLS // LANE_COLS, LANE_COLS)     # g i k t b j
    return x.permute(2, 0, 3, 4, 1, 5).reshape(split_k, G, S, LANES, LANE_COLS)


def _promote_single_split(A_rem: Tensor, offsets: Tensor):
    """A weight stored without the leading split dimension (``rem`` ``[M, N]``, ``offsets`` one
    rank lower as well) is a single split: the reference's ``mv_*`` accept that older form
    (``functional.py:33-36, 421-424``)."""
    if A_rem.dim() == 2:
        A_rem = A_rem[None, :, :]
        if offsets.dim() == 1:
            offsets = offsets[None, :]
    return A_rem, offsets


def _check_weight_call(A_rem: Tensor, A_exp: Tensor, X: Tensor):
    split_k, M, N = A_rem.shape
    assert M % 128 == 0
    assert N % 128 == 0
    assert X.dim() == 3 and X.size(-1) == N
    assert X.dtype == torch.bfloat16
    assert A_rem.device.type == A_exp.device.type == X.device.type == 'cuda'
    assert A_rem.device == A_exp.device == X.device


def mv_huffman(
    A_rem: Tensor, A_exp: Tensor, X: Tensor,
    offsets: Tensor,
    LUT1: Tensor, LUT2: Tensor, LUT3: Tensor, LUT4: Tensor,
    code_lengths: Tensor,
) -> Tensor:
    """Y[b, :] = W @ X[b, :] for b < 8 with W held compressed (reference ``functional.py:28-63``)."""
    A_rem, offsets = _promote_single_split(A_rem, offsets)
    split_k, M, N = A_rem.shape
    X = X.view(-1, split_k, N)
    _check_weight_call(A_rem, A_exp, X)
    Y = torch.empty((X.size(0), M), dtype=torch.bfloat16, device=A_rem.device)
    gemv_bf16_huffman(A_rem.contiguous(), A_exp.contiguous(), X.contiguous(), Y, offsets.contiguous(),
                      LUT1.contiguous(), LUT2.contiguous(), LUT3.contiguous(), LUT4.contiguous(),
                      code_lengths.contiguous())
    return Y


def mv_ans(A_rem: Tensor, A_exp: Tensor, X: Tensor, offsets: Tensor, LUT: Tensor) -> Tensor:
    """rANS counterpart of :func:`mv_huffman` (reference ``functional.py:414-444``)."""
    A_rem, offsets = _promote_single_split(A_rem, offsets)
    split_k, M, N = A_rem.shape
    X = X.view(-1, split_k, N)
    _check_weight_call(A_rem, A_exp, X)
    Y = torch.empty((X.size(0), M), dtype=torch.bfloat16, device=A_rem.device)
    gemv_bf16_ans(A_rem.contiguous(), A_exp.contiguous(), X.contiguous(), Y, offsets.contiguous(), LUT.contiguous())
    return Y


class HuffmanWeight(nn.Module):
    """A BF16 weight ``[M, K]`` stored as a raw sign/mantissa plane plus a Huffman-coded
    exponent stream.  Passing the module as the weight of ``F.linear`` runs the fused
    kernels (reference ``functional.py:66-242``)."""

    def __init__(
        self,
        rem: Tensor,
        exp: Tensor,
        offsets: Tensor,
        LUT1: Tensor,
        LUT2: Tensor,
        LUT3: Tensor,
        LUT4: Tensor,
        code_lengths: Tensor,
    ):
        super().__init__()
        self.rem = nn.Buffer(rem)
        self.exp = nn.Buffer(exp)
        self.offsets = nn.Buffer(offsets)
        self.LUT1 = nn.Buffer(LUT1)
        self.LUT2 = nn.Buffer(LUT2)
        self.LUT3 = nn.Buffer(LUT3)
        self.LUT4 = nn.Buffer(LUT4)
        self.code_lengths = nn.Buffer(code_lengths)

    def kwargs(self) -> dict[str, Tensor]:
        return dict(self.named_buffers())

    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        if func is not F.linear:
            return NotImplemented
        return linear_huffman(*args, **(kwargs or {}))

    def _empty_weight(self) -> Tensor:
        split_k, M, Ks = self.rem.shape
        assert self.rem.device.type == 'cuda'
        return torch.empty((M, split_k * Ks), dtype=torch.bfloat16, device=self.rem.device)

    def get_weight(self) -> Tensor:
        """The original BF16 weight, bit for bit."""
        weight = self._empty_weight()
        huffman_decode(self.rem, self.exp, weight, self.offsets,
                       self.LUT1, self.LUT2, self.LUT3, self.LUT4, self.code_lengths)
        return weight

    # ------------------------------------------------------------------ compression
    @classmethod
    def get_codec(cls, a: Tensor) -> LUTHuffmanEncoder:
        """One code per weight matrix, built from the histogram of exponent pairs."""
        device = torch.device('cuda', 0)
        _, exp = split_bf16(a.detach().to(device))
        counts = cls._pair_counts(exp)
        codec = LUTHuffmanEncoder()
        codec.build_lut(counts.cpu())
        return codec

    @staticmethod
    def _pair_counts(exp: Tensor) -> Tensor:
        """int64 [65536]: occurrences of every exponent pair ``a | b << 8`` (a = even column).

        A histogram over 65536 bins runs on global atomics (25 ms for a 4096x12288 layer); real
        weights use a few dozen exponent values, so the pairs are counted over the ranks of
        the values that occur (at most 64 x 64 bins, which the histogram kernel keeps in
        shared memory) and scattered back."""
        single = torch.bincount(exp.flatten().to(torch.int32), minlength=256)
        present = torch.nonzero(single).flatten()                      # exponent values that occur, ascending
        a, b = exp[:, 0::2], exp[:, 1::2]
        if present.numel() > 64:
            pairs = a.to(torch.int32) | (b.to(torch.int32) << 8)
            return torch.bincount(pairs.flatten(), minlength=65536)
        rank = torch.zeros(256, dtype=torch.int32, device=exp.device)
        rank[present] = torch.arange(present.numel(), dtype=torch.int32, device=exp.device)
        dense = rank[a.to(torch.int64)] | (rank[b.to(torch.int64)] << 6)
        small = torch.bincount(dense.flatten(), minlength=4096)        # [rank_b * 64 + rank_a]
        counts = torch.zeros(65536, dtype=torch.int64, device=exp.device)
        ra, rb = torch.meshgrid(torch.arange(present.numel(), device=exp.device),
                                torch.arange(present.numel(), device=exp.device), indexing='ij')
        counts[(present[ra] | (present[rb] << 8)).flatten()] = small[(ra | (rb << 6)).flatten()]
        return counts

    @classmethod
    def get_lut_kwargs(cls, codec: LUTHuffmanEncoder) -> dict[str, Tensor]:
        return {
            'LUT1': torch.from_numpy(codec.LUT1.copy()),
            'LUT2': torch.from_numpy(codec.LUT2.copy()),
            'LUT3': torch.from_numpy(codec.LUT3.copy()),
            'LUT4': torch.from_numpy(codec.LUT4.copy()),
            'code_lengths': torch.from_numpy(codec.code_lengths.copy()),
        }

    @classmethod
    def capacity(cls, n_steps: int) -> int:
        return encode_capacity(n_steps)

    @classmethod
    def compress_groups(cls, x: Tensor, codec) -> tuple[Tensor, Tensor]:
        """x: uint8 ``[tasks, steps*512]`` lane-ordered exponents of equally long tasks ->
        (streams int32 ``[tasks, capacity]``, words used per task)."""
        device = x.device
        n_steps = x.size(1) // (LANES * LANE_COLS)
        out = torch.zeros(x.size(0), cls.capacity(n_steps), dtype=torch.int32, device=device)
        lengths = torch.zeros(x.size(0), dtype=torch.int32, device=device)
        table = torch.from_numpy(codec.enc_table.view('int32').copy()).to(device)
        huffman_encode(x, table, out, lengths)
        return out, lengths

    @classmethod
    def compress_split_n(cls, a: Tensor, n: int = 2):
        """Compress ``a`` with ``n`` column splits (the reference's ``compress_split_n``,
        ``functional.py:195-238``)."""
        assert a.dim() == 2 and a.dtype == torch.bfloat16
        a = a.detach()
        M, K = a.shape
        assert M % 128 == 0 and K % n == 0 and (K // n) % STEP_COLS == 0, a.shape
        Ks = K // n
        S, G = Ks // STEP_COLS, M // GROUP_ROWS
        device = torch.device('cuda', 0)
        lib = _lib.load()
        consts = _lib.constants()
        nc = lib.bhi_chunks_per_group(M, Ks, n)

        codec = cls.get_codec(a)
        rem, exp = split_bf16(a.to(device))
        rem = _lane_order(rem, n).reshape(n, M, Ks).contiguous()
        sym = _lane_order(exp, n)                                           # [n, G, S, 64, 8]
        del exp

        lengths = torch.zeros(n, G, nc, dtype=torch.int64, device=device)
        pieces = []                                                          # (chunk, first task, streams, lengths)
        for c in range(nc):
            t0, t1 = (S * c) // nc, (S * (c + 1)) // nc
            tasks = sym[:, :, t0:t1].reshape(n * G, (t1 - t0) * LANES * LANE_COLS)
            per_call = max(1, ENCODE_PART_BYTES // (4 * cls.capacity(t1 - t0)))
            for first in range(0, n * G, per_call):
                out, ln = cls.compress_groups(tasks[first:first + per_call].contiguous(), codec)
                used = int(ln.max().item())
                pieces.append((c, first, out[:, :used].clone(), ln.to(torch.int64)))
                lengths.view(n * G, nc)[first:first + ln.numel(), c] = ln
        del sym

        total = int(lengths.sum().item())
        assert total + consts['tail_pad_words'] < 2 ** 31, "exponent stream too large for int32 offsets"
        starts = (torch.cumsum(lengths.flatten(), 0) - lengths.flatten()).view(n * G, nc)
        words = torch.zeros(total + consts['tail_pad_words'], dtype=torch.int32, device=device)
        for c, first, out, ln in pieces:
            cols = torch.arange(out.size(1), device=device)[None, :]
            keep = cols < ln[:, None]
            dest = (starts[first:first + ln.numel(), c][:, None] + cols)[keep]
            words[dest] = out[keep]
        offsets = torch.zeros(n, G, GROUP_ROWS, dtype=torch.int32, device=device)
        offsets[:, :, :nc] = starts.view(n, G, nc).to(torch.int32)

        return cls(
            rem=rem.cpu(),
            exp=words.cpu(),
            offsets=offsets.view(n, M).cpu(),
            **cls.get_lut_kwargs(codec),
        )

    @classmethod
    def compress(cls, a: Tensor):
        return cls.compress_split_n(a, n=get_block_size_n(a)[0])


class ANSWeight(HuffmanWeight):
    """Same planes and stream layout with an interleaved rANS exponent stream
    (reference ``functional.py:245-310``)."""

    def __init__(self, rem: Tensor, exp: Tensor, offsets: Tensor, LUT: Tensor):
        nn.Module.__init__(self)
        self.rem = nn.Buffer(rem)
        self.exp = nn.Buffer(exp)
        self.offsets = nn.Buffer(offsets)
        self.LUT = nn.Buffer(torch.as_tensor(LUT))

    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        if func is not F.linear:
            return NotImplemented
        return linear_ans(*args, **(kwargs or {}))

    def get_weight(self) -> Tensor:
        weight = self._empty_weight()
        ans_decode(self.rem, self.exp, weight, self.offsets, self.LUT)
        return weight

    @classmethod
    def get_codec(cls, a: Tensor) -> RANSEncoder:
        device = torch.device('cuda', 0)
        _, exp = split_bf16(a.detach().to(device))
        counts = torch.bincount(exp.flatten().to(torch.int32), minlength=256)
        return RANSEncoder(counts.tolist(), precision=ANS_PRECISION)

    @classmethod
    def get_lut_kwargs(cls, codec: RANSEncoder) -> dict[str, Tensor]:
        lut = torch.tensor(codec.decode_lut, dtype=torch.int32)
        return {'LUT': (lut[:, 0] << 24) | (lut[:, 1] << 12) | lut[:, 2]}

    @classmethod
    def capacity(cls, n_steps: int) -> int:
        return ans_encode_capacity(n_steps)

    @classmethod
    def compress_groups(cls, x: Tensor, codec: RANSEncoder) -> tuple[Tensor, Tensor]:
        device = x.device
        n_steps = x.size(1) // (LANES * LANE_COLS)
        out = torch.zeros(x.size(0), cls.capacity(n_steps), dtype=torch.int32, device=device)
        lengths = torch.zeros(x.size(0), dtype=torch.int32, device=device)
        freq = torch.tensor(codec.freq, dtype=torch.int32, device=device)
        cum = torch.tensor(codec.cum, dtype=torch.int32, device=device)
        ans_encode(x, freq, cum, out, lengths)
        return out, lengths


class NibbleCodec:
    """Per-matrix parameters of the fixed-width code: the start of the 15-wide exponent
    window that covers the most weights, and whether anything falls outside it."""

    WINDOW = 15

    def __init__(self, counts: Tensor):
        counts = counts.to(torch.int64).cpu()
        assert counts.numel() == 256
        cover = counts.unfold(0, self.WINDOW, 1).sum(-1)          # cover[b] = counts[b : b + 15]
        # base + 15 (the escape nibble) must stay below 256: the decoder adds the base to four
        # nibbles with one 32-bit add, and a carry would spill into the neighbouring exponent
        cover = cover[:256 - self.WINDOW]
        self.base = int(torch.argmax(cover).item())               # first best window
        self.has_escapes = int(cover[self.base].item()) != int(counts.sum().item())


class NibbleWeight(ANSWeight):
    """Same planes and task layout with a fixed-width exponent code: 4 bits per exponent
    (offset from a per-matrix base, escape list for outliers).  Not one of the reference's
    codecs: about nine percent larger than the Huffman form and noticeably faster to
    multiply with, because its decoder has no tables, cursors or serial dependencies."""

    MAGIC = 0x4E494242          # LUT[2]: tells this module's LUT from a rANS slot table (whose frequency field is <= 256)

    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        if func is not F.linear:
            return NotImplemented
        return linear_nibble(*args, **(kwargs or {}))

    def get_weight(self) -> Tensor:
        weight = self._empty_weight()
        nibble_decode(self.rem, self.exp, weight, self.offsets, self.LUT)
        return weight

    @classmethod
    def get_codec(cls, a: Tensor) -> NibbleCodec:
        device = torch.device('cuda', 0)
        _, exp = split_bf16(a.detach().to(device))
        return NibbleCodec(torch.bincount(exp.flatten().to(torch.int32), minlength=256))

    @classmethod
    def get_lut_kwargs(cls, codec: NibbleCodec) -> dict[str, Tensor]:
        lut = torch.zeros(256, dtype=torch.int32)
        lut[0], lut[1], lut[2] = codec.base, int(codec.has_escapes), cls.MAGIC
        return {'LUT': lut}

    @classmethod
    def capacity(cls, n_steps: int) -> int:
        return nibble_encode_capacity(n_steps)

    @classmethod
    def compress_groups(cls, x: Tensor, codec: NibbleCodec) -> tuple[Tensor, Tensor]:
        device = x.device
        n_steps = x.size(1) // (LANES * LANE_COLS)
        out = torch.zeros(x.size(0), cls.capacity(n_steps), dtype=torch.int32, device=device)
        lengths = torch.zeros(x.size(0), dtype=torch.int32, device=device)
        nibble_encode(x, cls.get_lut_kwargs(codec)['LUT'].to(device), out, lengths)
        return out, lengths


class CompressedLinear(nn.Module):
    def __init__(self, weight: HuffmanWeight, bias: Optional[Tensor]) -> None:
        super().__init__()
        self.weight = weight
        self.bias = bias
        self._group = None          # a LinearGroup when this module shares launches with siblings

    def forward(self, input: Tensor) -> Tensor:
        group = getattr(self, '_group', None)
        if group is not None:
            return group.forward(self, input)
        return F.linear(input, self.weight, self.bias)


def linear_grouped(input: Tensor, weights, biases=None, *, residuals=None, input_norm=None, input_gate=None,
                   outs=None) -> list:
    """``[F.linear(h, w, b) (+ r) for w, b, r in zip(weights, biases, residuals)]`` in ONE launch, where
    ``h`` is ``input``, or -- so that the layer in front of the linears needs no kernel of its own --

    * ``input_norm=(gamma, eps)``: ``h = rms_norm(input) * gamma`` (RMSNorm in front of q/k/v or gate/up),
    * ``input_gate=gate``: ``h = silu(gate) * input`` (the SwiGLU product in front of down_proj).

    ``weights`` are up to four compressed weights of one class with the same
    ``in_features`` split (``rem.shape[0]`` and ``rem.shape[2]``); ``input`` has at most
    8 rows after flattening.  ``residuals[i]`` (shaped like output ``i``) is added last, as a
    separate BF16 addition would; ``outs[i]`` (bf16 ``[rows, M_i]``, contiguous -- a column slice of a
    one-row buffer qualifies) receives output ``i`` instead of a new tensor.  This is what the q/k/v (or gate/up) projections of a
    decoder layer need: the reference overlaps them on parallel streams
    (``cudastream_utils.py:8-47``), here they are one grid.  Up to 4 rows (Huffman, rANS) the
    norm / gate product happens inside the kernel; otherwise it runs as this package's own
    elementwise kernel first -- the same arithmetic, the same bits.
    """
    assert input.dim() >= 2, input
    assert input_norm is None or input_gate is None, "one transform of the input at a time"
    shape = input.shape
    x = input.flatten(0, -2)
    if x.size(0) > MAX_FUSED_BATCH:
        raise RuntimeError(f'linear_grouped takes at most {MAX_FUSED_BATCH} rows, got {x.size(0)}')
    first = weights[0]
    split_k, _, N = first.rem.shape
    mode, aux, eps = _ops.X_PLAIN, None, 0.0
    if input_norm is not None or input_gate is not None:
        fusable = x.size(0) <= _ops.X_TRANSFORM_MAX_ROWS and not isinstance(first, NibbleWeight)
        if input_norm is not None:
            gamma, eps = input_norm
            gamma = gamma.detach()
            if fusable:
                mode, aux = _ops.X_RMS, gamma.contiguous()
            else:
                x = _ops.rms_norm(x, gamma, eps)
        else:
            gate = input_gate.flatten(0, -2)
            assert gate.shape == x.shape, (gate.shape, x.shape)
            if fusable:
                mode, aux = _ops.X_SILU_MUL, gate.contiguous()
            else:
                x = _ops.silu_mul(gate, x)
    x = x.view(-1, split_k, N)
    _check_weight_call(first.rem, first.exp, x)
    if outs is not None:
        ys = [o.view(x.size(0), w.rem.shape[1]) for o, w in zip(outs, weights)]
    else:
        ys = [torch.empty((x.size(0), w.rem.shape[1]), dtype=torch.bfloat16, device=x.device) for w in weights]
    if biases is not None:
        biases = [None if b is None else b.detach().contiguous() for b in biases]
    if residuals is not None:
        residuals = [None if r is None else r.detach().reshape(x.size(0), -1).contiguous() for r in residuals]
    total = sum(w.rem.shape[1] for w in weights)
    if (mode == _ops.X_PLAIN and not isinstance(first, NibbleWeight)
            and (all(prefers_matrix_cores(x.size(0), w.rem.shape[1], split_k * N) for w in weights)
                 or prefers_matrix_cores(x.size(0), total, split_k * N))):
        # layers this large -- or this large together -- are faster through the matrix-core kernel
        gemm_bf16_grouped(weights, x.contiguous(), ys, biases, residuals)
    else:
        gemv_bf16_grouped(weights, x.contiguous(), ys, biases, residuals, mode, aux, float(eps))
    return [y.unflatten(0, shape[:-1]) for y in ys]


class LinearGroup:
    """Sibling :class:`CompressedLinear` modules that a model always calls one after the
    other on the same input tensor (q/k/v of an attention block, gate/up of an MLP).

    The call of the first member computes every member's output in one grouped launch
    and keeps the others until their own call collects them.  Whatever does not fit that
    pattern -- more than 8 rows, a member called alone or on another tensor, weights of
    different codecs or splits -- runs each member's ordinary path.  Grouping changes the
    number of launches and, where members that are large only together move to the matrix-core
    kernel (:func:`prefers_matrix_cores`), the order of the fp32 sums: a last bit of BF16 here
    and there, nothing else.
    """

    def __init__(self, members):
        self.members = list(members)
        for m in self.members:
            if not isinstance(m, CompressedLinear):
                raise TypeError('LinearGroup takes CompressedLinear modules')
        if not 2 <= len(self.members) <= 4:
            raise ValueError('a group has 2 to 4 members')
        first = self.members[0].weight
        self.uniform = all(type(m.weight) is type(first) and m.weight.rem.shape[0] == first.rem.shape[0]
                           and m.weight.rem.shape[2] == first.rem.shape[2] for m in self.members)
        self._input = None
        self._outputs = None
        for m in self.members:
            m._group = self

    def _biases_fit(self, input: Tensor) -> bool:
        """The grouped launch adds BF16 biases on the input's device; anything else takes the
        members' own path (``output += bias``), as an ungrouped module would."""
        return all(m.bias is None or (m.bias.dtype == torch.bfloat16 and m.bias.device == input.device)
                   for m in self.members)

    def dissolve(self) -> None:
        for m in self.members:
            m._group = None

    def forward(self, module: CompressedLinear, input: Tensor) -> Tensor:
        index = next(i for i, m in enumerate(self.members) if m is module)
        if index == 0:
            self._input = self._outputs = None
            rows = input.numel() // input.shape[-1] if input.dim() >= 2 else MAX_FUSED_BATCH + 1
            if self.uniform and input.is_cuda and rows <= MAX_FUSED_BATCH and self._biases_fit(input):
                self._outputs = linear_grouped(input, [m.weight for m in self.members],
                                               [m.bias for m in self.members])
                self._input = input
                return self._outputs[0]
        elif self._input is input and self._outputs is not None:
            out = self._outputs[index]
            self._outputs[index] = None
            if index == len(self.members) - 1:
                self._input = self._outputs = None
            if out is not None:
                return out
        return F.linear(input, module.weight, module.bias)


def _weight_bytes(w: nn.Module) -> int:
    return sum(b.nelement() * b.element_size() for b in w.buffers())


def convert(linear: nn.Linear, name, disable_precision_check=True, algo='huffman') -> nn.Module:
    """Compress one ``nn.Linear`` (reference ``functional.py:323-375``).

    Returns the original module when compression does not shrink it or when the decoded
    weight is not bit-identical; with ``disable_precision_check=False`` also when one
    random GEMV deviates by 2 % or more from the dense layer.
    """
    assert algo in ('huffman', 'ans', 'smallest', 'nibble')
    if algo == 'huffman':
        weight = HuffmanWeight.compress(linear.weight)
    elif algo == 'ans':
        weight = ANSWeight.compress(linear.weight)
    elif algo == 'nibble':
        weight = NibbleWeight.compress(linear.weight)
    else:
        weight = min([HuffmanWeight.compress(linear.weight), ANSWeight.compress(linear.weight)], key=_weight_bytes)

    module = CompressedLinear(weight=weight, bias=linear.bias)
    ori_size = linear.weight.nelement() * linear.weight.element_size()
    ratio = _weight_bytes(module.weight) / ori_size

    linear.cuda()
    module.cuda()
    x = torch.randn(1, linear.in_features, dtype=torch.bfloat16, device='cuda')
    with torch.no_grad():
        y1 = linear(x)
        y2 = module(x)
        lossless = torch.equal(module.weight.get_weight().view(torch.int16), linear.weight.view(torch.int16))
    max_rtol = ((y2 - y1).abs() / y1.abs().clamp(min=1e-4)).max().item()
    linear.cpu()
    module.cpu()

    fallback = False
    if ratio >= 1:
        print(f'\nWarning! {name} ratio = {ratio:.2%}')
        fallback = True
    if not lossless:
        print(f'\nWarning! {name} does not decode to the original weight')
        fallback = True
    if not disable_precision_check and max_rtol >= 0.02:
        print(f'\nWarning! {name} output mismatch: max rtol = {max_rtol:.2f}')
        fallback = True
    if fallback:
        print('Fallback to regular nn.Linear')
        return linear
    return module


def convert_all_linear(model: nn.Module, min_out_features=4096, progress=True, algo='huffman') -> None:
    """Replace every ``nn.Linear`` with at least ``min_out_features`` outputs in place."""
    targets = [name for name, m in model.named_modules()
               if isinstance(m, nn.Linear) and m.out_features >= min_out_features]
    for name in tqdm(targets, disable=not progress):
        model.set_submodule(name, convert(model.get_submodule(name), name, algo=algo))


def linear_nibble(input: Tensor, weight: NibbleWeight, bias: Optional[Tensor] = None) -> Tensor:
    """``F.linear`` with a :class:`NibbleWeight` (fused up to 8 rows, else decode + GEMM)."""
    def fused(x):
        split_k, M, N = weight.rem.shape
        x = x.view(-1, split_k, N)
        _check_weight_call(weight.rem, weight.exp, x)
        y = torch.empty((x.size(0), M), dtype=torch.bfloat16, device=x.device)
        gemv_bf16_nibble(weight.rem, weight.exp, x.contiguous(), y, weight.offsets, weight.LUT)
        return y
    return _linear_compressed(input, weight, bias, fused)


def check_layout(weight: "HuffmanWeight") -> None:
    """Raises unless ``weight``'s buffers are in THIS package's task layout.

    A weight saved by the reference package has the same buffer names, dtypes and (for rANS)
    shapes, but its ``offsets`` are per row and its stream has no zero tail: the kernels would
    read it as garbage, past the end of ``exp``.  Checked: the format header (Huffman), unused
    chunk slots of ``offsets`` are 0, offsets are aligned and ascending in task order, the last
    task ends in front of the tail pad, and the tail pad is zero."""
    consts = _lib.constants()
    lib = _lib.load()
    hint = ('; a weight compressed by the reference package must be converted with '
            'bf16_huffman_infer_amd.reference_format.transcode_reference_weight')
    rem, exp, offsets = weight.rem, weight.exp, weight.offsets
    if rem.dim() != 3 or offsets.dim() != 2 or tuple(offsets.shape) != tuple(rem.shape[:2]):
        raise RuntimeError(f'compressed weight: rem {tuple(rem.shape)} / offsets {tuple(offsets.shape)} do not fit' + hint)
    split_k, M, Ks = rem.shape
    if isinstance(weight, HuffmanWeight) and hasattr(weight, 'LUT1'):
        header = weight.code_lengths.flatten()[:2].tolist()
        if weight.LUT1.numel() != 4 << consts['table_bits'] or header != [consts['format_version'], consts['table_bits']]:
            raise RuntimeError('compressed weight: Huffman tables are not in this package\'s format' + hint)
    if M % GROUP_ROWS or Ks % STEP_COLS:
        raise RuntimeError(f'compressed weight: {M}x{split_k * Ks} does not fit the task layout' + hint)
    nc = lib.bhi_chunks_per_group(M, Ks, split_k)
    pad, align = consts['tail_pad_words'], consts['align_words']
    off = offsets.reshape(split_k, M // GROUP_ROWS, GROUP_ROWS).to(torch.int64)
    used = off[:, :, :nc].flatten()
    ok = (exp.numel() >= pad and not bool(off[:, :, nc:].any()) and not bool((used % align).any())
          and bool((used[1:] > used[:-1]).all()) and int(used[0]) == 0 and int(used[-1]) < exp.numel() - pad
          and not bool(exp[exp.numel() - pad:].any()))
    if not ok:
        raise RuntimeError('compressed weight: offsets / exp are not in this package\'s task layout' + hint)


def load_compressed_state_dict(model: nn.Module, state_dict: dict, strict: bool = True):
    """Load the ``state_dict()`` of a converted model into a freshly built, unconverted one.

    The reference leaves this to the user (its converted modules only exist after
    ``convert_all_linear`` has run on real weights).  Here every ``nn.Linear`` of ``model``
    whose compressed buffers are in ``state_dict`` (``<name>.weight.rem`` ...) is replaced
    by a :class:`CompressedLinear` around those tensors -- ``LUT1`` present means Huffman,
    ``LUT`` means rANS or (by its marker word) the nibble code -- and the remaining entries go through ``load_state_dict``.  The
    skeleton's linears may live on the meta device; nothing is decoded or re-encoded.
    """
    huffman_keys = ('rem', 'exp', 'offsets', 'LUT1', 'LUT2', 'LUT3', 'LUT4', 'code_lengths')
    ans_keys = ('rem', 'exp', 'offsets', 'LUT')
    for name, module in list(model.named_modules()):
        if not isinstance(module, nn.Linear) or f'{name}.weight.rem' not in state_dict:
            continue
        keys = huffman_keys if f'{name}.weight.LUT1' in state_dict else ans_keys
        if keys is huffman_keys:
            cls = HuffmanWeight
        else:
            nibble = int(state_dict[f'{name}.weight.LUT'][2]) == NibbleWeight.MAGIC
            cls = NibbleWeight if nibble else ANSWeight
        weight = cls(**{k: state_dict[f'{name}.weight.{k}'] for k in keys})
        check_layout(weight)
        split_k, M, Ks = weight.rem.shape
        if (M, split_k * Ks) != (module.out_features, module.in_features):
            raise RuntimeError(f'{name}: compressed weight is {M}x{split_k * Ks}, '
                               f'the module expects {module.out_features}x{module.in_features}')
        bias = state_dict.get(f'{name}.bias')
        if bias is not None:
            bias = nn.Parameter(bias, requires_grad=False)
        model.set_submodule(name, CompressedLinear(weight=weight, bias=bias))
    return model.load_state_dict(state_dict, strict=strict, assign=True)


def prefers_matrix_cores(rows: int, M: int, K: int) -> bool:
    """Whether ``rows`` <= 8 rows of activations go through the matrix-core kernel rather than the
    GEMV.  The GEMV spends four dot products per row and step and one load of X per row; the
    matrix-core kernel shares X among the wavefronts of a block through LDS and costs the same for
    5..8 rows, but starts slower and keeps fewer wavefronts on a compute unit.  Measured on MI355X
    (us, GEMV / matrix cores):

    ===========  ===========  ===========  ===========  ===========
    M x K        4 rows       5 rows       6 rows       8 rows
    ===========  ===========  ===========  ===========  ===========
    3584x18944   26.4 / 25.9  29.3 / 28.4  31.5 / 28.7  36.8 / 29.3
    14336x4096   21.8 / 20.5  23.6 / 22.5  25.2 / 22.5  28.4 / 22.5
    18944x3584   23.4 / 23.9  25.3 / 26.1  27.0 / 26.1  30.8 / 26.2
    12288x4096   19.0 / 19.4  20.6 / 21.2  23.9 / 21.2  26.4 / 21.2
    11008x4096   18.6 / 19.0  20.3 / 20.7  23.2 / 20.8  25.3 / 20.8
    4096x14336   21.9 / 22.8  24.1 / 24.4  26.0 / 24.8  29.5 / 25.5
    4096x12288   22.1 / 26.1  24.6 / 27.7  25.7 / 27.8  28.6 / 28.0
    4096x11008   18.6 / 20.7  20.5 / 22.7  21.7 / 23.1  24.7 / 23.8
    8192x8192    23.1 / 27.7  25.1 / 30.0  27.1 / 30.2  30.8 / 30.3
    ===========  ===========  ===========  ===========  ===========

    and the layers of 6144x4096 and below are 0.4-4 us faster on the GEMV at every row count; output
    layers the size of a vocabulary -- or a group of layers that large together -- are faster on the
    matrix cores from 3 rows (152064x3584: 138 / 147, 157 / 148, 180 / 148, 225 / 185 us at 2, 3, 4, 8
    rows; 37888x3584: 39.1 / 39.6, 41.9 / 39.7, 44.4 / 39.8, 58.7 / 48.9).  The rANS kernels cross over
    at the same places (18944x3584 at 6 rows 37.7 / 36.0, 3584x18944 at 4 rows 34.7 / 33.9,
    37888x3584 at 3 rows 53.6 / 51.2)."""
    if rows >= 8 and K >= 11008:
        return True
    if rows >= 6 and ((M >= 10240 and K >= 3584) or K >= 14336):
        return True
    if rows >= 4 and (K >= 16384 or (M >= 14336 and K >= 4096)):
        return True
    return rows >= 3 and M >= 32768 and K >= 3584


def _linear_compressed(input: Tensor, weight: HuffmanWeight, bias: Optional[Tensor], fused) -> Tensor:
    assert input.dim() >= 2, input
    shape = input.shape
    input = input.flatten(0, -2)
    if input.size(0) == 0:                       # no rows: nothing to launch
        return input.new_empty((*shape[:-1], weight.rem.shape[1]))
    split_k, M, N = weight.rem.shape
    wide = (input.size(0) <= MAX_FUSED_BATCH and not isinstance(weight, NibbleWeight) and input.dtype == torch.bfloat16
            and (bias is None or bias.dtype == torch.bfloat16) and prefers_matrix_cores(input.size(0), M, split_k * N))
    if input.size(0) <= MAX_FUSED_BATCH and not wide:
        if bias is not None and bias.dtype == torch.bfloat16:
            # the grouped entry point adds the bias in the kernel's last store (same bits, one launch less)
            return linear_grouped(input, [weight], [bias])[0].unflatten(0, shape[:-1])
        output = fused(input)
        if bias is not None:
            output += bias[None, :]
    elif wide or (input.size(0) <= GEMM_MAX_ROWS and not isinstance(weight, NibbleWeight) and input.dtype == torch.bfloat16
                  and (bias is None or bias.dtype == torch.bfloat16)):
        # 9..32 rows (and fewer where the rule above says so): decode inside the matrix-core kernel,
        # no BF16 weight in memory
        x = input.view(-1, split_k, N)
        _check_weight_call(weight.rem, weight.exp, x)
        output = torch.empty((x.size(0), M), dtype=torch.bfloat16, device=x.device)
        gemm_bf16(weight, x.contiguous(), output, None if bias is None else bias.detach().contiguous())
    else:
        output = F.linear(input, weight.get_weight(), bias)
    return output.unflatten(0, shape[:-1])


def linear_huffman(input: Tensor, weight: HuffmanWeight, bias: Optional[Tensor] = None) -> Tensor:
    """``F.linear`` with a :class:`HuffmanWeight`: fused kernel up to 8 rows, else decode +
    dense GEMM (reference ``functional.py:390-411``)."""
    return _linear_compressed(input, weight, bias, lambda x: mv_huffman(
        weight.rem, weight.exp, x, weight.offsets,
        weight.LUT1, weight.LUT2, weight.LUT3, weight.LUT4, weight.code_lengths))


def linear_ans(input: Tensor, weight: ANSWeight, bias: Optional[Tensor] = None) -> Tensor:
    """rANS counterpart of :func:`linear_huffman` (reference ``functional.py:447-466``)."""
    return _linear_compressed(input, weight, bias, lambda x: mv_ans(
        weight.rem, weight.exp, x, weight.offsets, weight.LUT))
