"""Bit-plane helpers, the split chooser and model-size accounting.

Same functions and meanings as the reference's ``bf16_huffman_infer/utils.py``.
"""
import copy
from typing import Tuple

import torch
from torch import Tensor, nn


def split_bf16(x: Tensor) -> Tuple[Tensor, Tensor]:
    """BF16 tensor -> (rem, exp) uint8 planes: exp = bits 14..7, rem = sign<<7 | mantissa.

    Reference: ``utils.py:7-12``.
    """
    assert x.dtype == torch.bfloat16
    bits = x.contiguous().view(torch.int16).to(torch.int32)
    exp = ((bits >> 7) & 0xFF).to(torch.uint8)
    rem = (((bits >> 8) & 0x80) | (bits & 0x7F)).to(torch.uint8)
    return rem, exp


def get_block_size_n(x: Tensor) -> Tuple[int]:
    """``(split_k,)`` for a weight ``[out_features, in_features]`` (reference ``utils.py:15-31``).

    Prefers blocks of at most 4096 columns with at most 8 splits, then blocks of
    4096..16384 columns with at most 32 splits, then small blocks with at most 32
    splits; in_features that fit none of these raise.
    """
    n = x.size(1)
    if n % 128 == 0:
        units = n // 128
        passes = (
            (range(32, 2, -1), 8),
            (range(32, 129), 32),
            (range(32, 2, -1), 32),
        )
        for block_units, max_splits in passes:
            for u in block_units:
                if units % u == 0 and units // u <= max_splits:
                    return (units // u,)
    raise RuntimeError(f"Could not find suitable block size for shape {x.shape}")


def get_model_size(model: nn.Module) -> int:
    """Bytes held by parameters and buffers (reference ``utils.py:34-42``)."""
    tensors = list(model.parameters()) + list(model.buffers())
    return sum(t.nelement() * t.element_size() for t in tensors)


def print_stats(ori: Tensor, new: nn.Module) -> None:
    ori_size = ori.nelement() * ori.element_size()
    new_size = sum(b.nelement() * b.element_size() for b in new.buffers())
    print(f'ori size = {ori_size / 1024 ** 2:.2f}MiB')
    print(f'new size = {new_size / 1024 ** 2:.2f}MiB')
    print(f'compression ratio = {new_size / ori_size:.2%}')
    print(f'bits = {new_size / ori_size * 16:.2f}')


def shallow_copy_model(model: nn.Module) -> nn.Module:
    """Deep copy of the module tree that shares every parameter and buffer."""
    memo = {id(t): t for t in list(model.parameters()) + list(model.buffers())}
    return copy.deepcopy(model, memo=memo)
