"""Loading weights that were compressed by the reference package.

The reference's modules keep ``rem``/``exp``/``offsets`` in its own layout (64 private
streams per row, ``bf16_huffman_infer/functional.py:129-242``) and its Huffman tables as
four 256-entry byte tables.  The kernels of this package use a different layout, so such
buffers are first decoded back to the BF16 weight (on the GPU, by the reference's own
rules) and then compressed again here.  The result is a module of this package holding
exactly the same weight.
"""
import torch
from torch import Tensor

from . import _lib
from .functional import ANSWeight, HuffmanWeight

__all__ = ["decode_reference_huffman", "decode_reference_ans", "transcode_reference_weight"]


def _prepare(rem: Tensor, exp: Tensor, offsets: Tensor, device):
    if rem.dim() == 2:                      # legacy modules without the split axis (functional.py:33-35)
        rem, offsets = rem[None], offsets[None]
    assert rem.dim() == 3 and rem.dtype == torch.uint8 and exp.dtype == torch.int32 and offsets.dtype == torch.int32
    assert offsets.shape == rem.shape[:2] and rem.size(2) % 128 == 0
    return rem.to(device).contiguous(), exp.to(device).contiguous(), offsets.to(device).contiguous()


def _stream(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def decode_reference_huffman(rem: Tensor, exp: Tensor, offsets: Tensor, LUT1: Tensor, LUT2: Tensor,
                             LUT3: Tensor, LUT4: Tensor, code_lengths: Tensor, device="cuda") -> Tensor:
    """The BF16 weight ``[M, K]`` held by a reference ``HuffmanWeight``'s buffers."""
    device = torch.device(device)
    rem, exp, offsets = _prepare(rem, exp, offsets, device)
    tables = [t.to(device=device, dtype=torch.uint8).contiguous() for t in (LUT1, LUT2, LUT3, LUT4, code_lengths)]
    assert all(t.numel() == 256 for t in tables), "the reference's tables have 256 entries each"
    split_k, M, Ks = rem.shape
    Y = torch.empty(M, split_k * Ks, dtype=torch.bfloat16, device=device)
    with torch.cuda.device(device):
        rc = _lib.load().bhi_reference_huffman_decode(
            rem.data_ptr(), exp.data_ptr(), exp.numel(), Y.data_ptr(), offsets.data_ptr(),
            *[t.data_ptr() for t in tables], split_k, M, Ks, _stream(device))
    _lib.check(rc, "reference_huffman_decode")
    return Y


def decode_reference_ans(rem: Tensor, exp: Tensor, offsets: Tensor, LUT: Tensor, device="cuda") -> Tensor:
    """The BF16 weight ``[M, K]`` held by a reference ``ANSWeight``'s buffers."""
    device = torch.device(device)
    rem, exp, offsets = _prepare(rem, exp, offsets, device)
    LUT = LUT.to(device=device, dtype=torch.int32).contiguous()
    assert LUT.numel() == 256
    split_k, M, Ks = rem.shape
    Y = torch.empty(M, split_k * Ks, dtype=torch.bfloat16, device=device)
    with torch.cuda.device(device):
        rc = _lib.load().bhi_reference_ans_decode(
            rem.data_ptr(), exp.data_ptr(), exp.numel(), Y.data_ptr(), offsets.data_ptr(), LUT.data_ptr(),
            split_k, M, Ks, _stream(device))
    _lib.check(rc, "reference_ans_decode")
    return Y


def transcode_reference_weight(buffers: dict, algo: str = "same"):
    """``buffers``: the named buffers of a reference ``HuffmanWeight`` / ``ANSWeight`` (as in
    its ``state_dict``).  Returns this package's module for the same weight; ``algo`` is
    ``'same'`` (keep the codec family), ``'huffman'``, ``'ans'`` or ``'smallest'``."""
    if "LUT1" in buffers:
        weight = decode_reference_huffman(*[buffers[k] for k in (
            "rem", "exp", "offsets", "LUT1", "LUT2", "LUT3", "LUT4", "code_lengths")])
        family = "huffman"
    else:
        weight = decode_reference_ans(*[buffers[k] for k in ("rem", "exp", "offsets", "LUT")])
        family = "ans"
    algo = family if algo == "same" else algo
    assert algo in ("huffman", "ans", "smallest")
    if algo == "smallest":
        both = [HuffmanWeight.compress(weight), ANSWeight.compress(weight)]
        return min(both, key=lambda w: sum(b.nelement() * b.element_size() for b in w.buffers()))
    return (HuffmanWeight if algo == "huffman" else ANSWeight).compress(weight)
