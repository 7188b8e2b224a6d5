"""Bookkeeping shared by the grouped modules: token-split prefix sums, fp8 dtype
names and the index arithmetic into the per-GEMM scaling metadata.

Same names and meaning as the reference's ``fp8_gmm/utils.py`` (enums :7-23, dtype
maps :26-45, ``cumsum_group_sizes`` :48-62, ``Fp8MetaWrapper`` :65-103); the
``tex.DType`` values of TransformerEngine are replaced by the local :class:`DType`.
"""
from enum import IntEnum

import numpy as np
import torch

PAD_MULTIPLE = 16  # the transposed (wgrad) operands pad each expert's tokens to this (reference utils.py:57)


class DType(IntEnum):
    """Stand-in for the three ``tex.DType`` members the reference uses (utils.py:26-45)."""

    kFloat8E4M3 = 0
    kFloat8E5M2 = 1
    kBFloat16 = 2


class MetaTensorType(IntEnum):
    kScale = 0
    kScaleInv = 1
    kAmax = 2


class Fp8TensorType(IntEnum):
    kInputGroup1 = 0
    kInputGroup2 = 1
    kWeightGroup1 = 2
    kWeightGroup2 = 3
    kGradOutputGroup1 = 4
    kGradOutputGroup2 = 5
    kForwardInputGroup1 = 6
    kForwardInputGroup2 = 7
    kForwardWeightGroup1 = 8
    kForwardWeightGroup2 = 9


_TORCH_TO_DTYPE = {
    torch.float8_e4m3fn: DType.kFloat8E4M3,
    torch.float8_e5m2: DType.kFloat8E5M2,
    torch.bfloat16: DType.kBFloat16,
}
_DTYPE_TO_TORCH = {v: k for k, v in _TORCH_TO_DTYPE.items()}


def to_tex_dtype(dtype):
    try:
        return _TORCH_TO_DTYPE[dtype]
    except KeyError:
        raise ValueError(f"Unsupported dtype: {dtype}") from None


def to_torch_dtype(dtype):
    try:
        return _DTYPE_TO_TORCH[dtype]
    except KeyError:
        raise ValueError(f"Unsupported dtype: {dtype}") from None


def round_up(x, multiple):
    return (x + multiple - 1) // multiple * multiple


def cumsum_group_sizes(group_sizes, need_padding=False, pad_multiple=PAD_MULTIPLE):
    """Prefix sums of the per-expert token counts.

    Returns ``(num_groups, padded, cumsums, padded_cumsums)``: ``cumsums`` has ``E + 1``
    entries starting at 0; with ``need_padding`` every count is rounded up to
    ``pad_multiple`` before summing into ``padded_cumsums`` (else None), and ``padded``
    says whether any count actually grew.  Zero counts are allowed.
    """
    sizes = [int(g) for g in group_sizes]
    cumsums = [0]
    for g in sizes:
        cumsums.append(cumsums[-1] + g)
    if not need_padding:
        return len(sizes), False, cumsums, None
    padded_cumsums = [0]
    for g in sizes:
        padded_cumsums.append(padded_cumsums[-1] + round_up(g, pad_multiple))
    return len(sizes), padded_cumsums[-1] != cumsums[-1], cumsums, padded_cumsums


class Fp8MetaWrapper:
    """Picks per-expert views out of the flat scaling-metadata tensors.

    Layout (reference utils.py:66-67,98-103): the forward tensors hold 3 slots per
    GEMM (input, weight, output), the backward tensors 2 (grad_output, grad_input).
    Expert ``i`` of group ``g`` (0 for ``*Group1``, 1 for ``*Group2``) is GEMM
    ``g * E + i``; weights sit one slot after their GEMM's input.  The
    ``kForward*`` types read the copy of the forward ``scale_inv`` taken right
    after the forward pass, so that a later scale update cannot change what the
    backward GEMMs dequantise with.
    """

    _FORWARD_OFFSET = 3
    _BACKWARD_OFFSET = 2

    def __init__(self, num_groups, fp8_meta):
        self._num_groups = num_groups
        self._fp8_meta = fp8_meta
        self._forward_scale_inv_cloned = None
        self._slot_offsets = {}

    def num_groups(self):
        return self._num_groups

    def set_forward_scale_inv_cloned(self):
        self._forward_scale_inv_cloned = self._fp8_meta["scaling_fwd"].scale_inv.clone()

    def _select(self, fp8_tensor_type, meta_tensor_type):
        """(flat tensor, first index, stride) of the E slots of this tensor type."""
        rule = _SLOT_RULES.get(int(fp8_tensor_type))
        if rule is None:
            raise ValueError(f"{fp8_tensor_type} is not a valid Fp8TensorType")
        forward_copy, backward, stride, second_group, weight = rule
        if forward_copy:
            assert meta_tensor_type == MetaTensorType.kScaleInv
            assert self._forward_scale_inv_cloned is not None, "forward scale_inv has not been cloned yet"
            flat = self._forward_scale_inv_cloned
        else:
            meta = self._fp8_meta["scaling_bwd" if backward else "scaling_fwd"]
            if meta_tensor_type == MetaTensorType.kScale:
                flat = meta.scale
            elif meta_tensor_type == MetaTensorType.kScaleInv:
                flat = meta.scale_inv
            elif meta_tensor_type == MetaTensorType.kAmax:
                flat = meta.amax_history[0]
            else:
                raise ValueError(f"unknown meta tensor type {meta_tensor_type}")
        first = (self._num_groups if second_group else 0) * stride + weight
        return flat, first, stride

    def get_meta_tensors(self, fp8_tensor_type, meta_tensor_type):
        """List of E zero-dim views, one per expert (the reference's return value)."""
        flat, first, stride = self._select(fp8_tensor_type, meta_tensor_type)
        return [flat[first + i * stride] for i in range(self._num_groups)]

    def get_meta_pointers(self, fp8_tensor_type, meta_tensor_type):
        """Device addresses of the same E slots as a uint64 array, without creating E tensor views
        (every backend entry point takes such an array wherever it takes a list of scalars)."""
        flat, first, stride = self._select(fp8_tensor_type, meta_tensor_type)
        offsets = self._slot_offsets.get(stride)
        if offsets is None:
            offsets = self._slot_offsets[stride] = np.arange(self._num_groups, dtype=np.uint64) * np.uint64(stride * 4)
        if flat.dim() != 1 or flat.dtype != torch.float32:
            raise RuntimeError("fp8 meta tensors must be flat fp32 tensors")
        return np.uint64(flat.data_ptr() + first * 4) + offsets


def _slot_rule(t):
    name = t.name
    return (t >= Fp8TensorType.kForwardInputGroup1,                  # reads the copy of the forward scale_inv
            Fp8TensorType.kGradOutputGroup1 <= t < Fp8TensorType.kForwardInputGroup1,   # lives in scaling_bwd
            Fp8MetaWrapper._BACKWARD_OFFSET if "GradOutput" in name else Fp8MetaWrapper._FORWARD_OFFSET,
            "Group1" not in name, 1 if "Weight" in name else 0)


_SLOT_RULES = {int(t): _slot_rule(t) for t in Fp8TensorType}
