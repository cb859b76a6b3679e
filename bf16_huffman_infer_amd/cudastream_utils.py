"""Fewer serial launches for the projections that share an input.

The reference's ``bf16_huffman_infer/cudastream_utils.py`` puts ``q_proj`` and ``k_proj``
of every attention block on side streams so that q/k/v overlap inside the captured
graph (``:8-47``).  On this hardware a kernel node costs a few microseconds of launch
floor however small it is and a short GEMV cannot fill the chip, so the same names
here tie the sibling projections into one *grouped launch* instead: the first
projection's call runs all of them as one grid (``functional.LinearGroup``).  No extra
streams are created.  ``gate_proj``/``up_proj`` get the same treatment.

Linears that are not compressed (raw BF16 ``nn.Linear``) are left alone.
"""
from torch import nn

from .functional import CompressedLinear, LinearGroup
from .utils import shallow_copy_model

__all__ = ["parallelize_qkv", "parallelize_gate_up", "parallelize_qkv_model", "get_parallelize_qkv_model"]


def _group(parent: nn.Module, names) -> bool:
    members = [getattr(parent, n, None) for n in names]
    if not all(isinstance(m, CompressedLinear) for m in members):
        return False
    if any(m._group is not None for m in members):
        return False
    group = LinearGroup(members)
    if not group.uniform:        # different codecs or splits: nothing to share
        group.dissolve()
    return group.uniform


def parallelize_qkv(self_attn: nn.Module) -> bool:
    """Group ``q_proj, k_proj, v_proj`` of ``self_attn`` (reference ``cudastream_utils.py:8-47``).
    Returns whether a grouped launch will be used."""
    return _group(self_attn, ("q_proj", "k_proj", "v_proj"))


def parallelize_gate_up(mlp: nn.Module) -> bool:
    """Group ``gate_proj, up_proj`` of ``mlp`` (no counterpart in the reference)."""
    return _group(mlp, ("gate_proj", "up_proj"))


def parallelize_qkv_model(model: nn.Module, gate_up: bool = True) -> None:
    """Every module that owns ``q_proj/k_proj/v_proj`` (and, with ``gate_up``, every one
    that owns ``gate_proj/up_proj``) gets its group (reference ``cudastream_utils.py:50-52``
    walks ``model.model.layers[*].self_attn``; walking all modules finds the same ones)."""
    for module in model.modules():
        if hasattr(module, "q_proj") and hasattr(module, "k_proj") and hasattr(module, "v_proj"):
            parallelize_qkv(module)
        if gate_up and hasattr(module, "gate_proj") and hasattr(module, "up_proj"):
            parallelize_gate_up(module)


def get_parallelize_qkv_model(model: nn.Module, gate_up: bool = True) -> nn.Module:
    """A copy of the module tree (sharing all tensors) with grouped projections; ``model``
    itself is not modified (reference ``cudastream_utils.py:55-58``)."""
    new_model = shallow_copy_model(model)
    parallelize_qkv_model(new_model, gate_up=gate_up)
    return new_model
