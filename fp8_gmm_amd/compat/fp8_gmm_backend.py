"""``fp8_gmm_backend``: the reference's pybind11 extension module (csrc/ops.cu:9-16), served by the HIP library.

The reference's ``fp8_gmm/backend.py:1`` does ``import fp8_gmm_backend as backend`` and calls six functions with
lists of tensors.  This module exposes those six names with the argument lists of the C++ functions they bind
(csrc/fp8_gmm.h:11, csrc/multi_pointwise.h:8-13, csrc/multi_pad_fusion.h:9-21), so that the reference's Python
layer runs unchanged on an MI355X with this file in place of the CUDA extension:

    import sys, fp8_gmm_amd.compat; sys.path.insert(0, fp8_gmm_amd.compat.__path__[0])   # then: import fp8_gmm_backend
    # or: from fp8_gmm_amd.compat import fp8_gmm_backend

Every call validates like the extension's TORCH_CHECKs (raising RuntimeError), builds the descriptor table of the
C ABI (include/fp8gmm.h) and launches ONE kernel on torch's current stream.  Differences a caller can rely on:
any number of tensors per call (the extension stops at 64, csrc/multi_pad_fusion.cu:447,512,594,
csrc/multi_pointwise.cu:161,222) and groups without rows.
"""
import torch

from fp8_gmm_amd import backend as _backend  # absolute: this file is also imported as a top-level module

_FP8 = (torch.float8_e4m3fn, torch.float8_e5m2)


def _check(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def fp8_gmm(a, b, c, batch_sizes):
    """``Fp8GroupedGemm`` (csrc/fp8_gmm.cu:163-205): for every group g, ``c[rows of g] = a[rows of g] . b[g]^T`` with
    fp32 accumulation and NO scaling (alpha = 1, beta = 0, csrc/fp8_gmm.cu:137-138); the reference applies the
    scales afterwards with ``multi_scale_mul`` (fp8_gmm/backend.py:78-82).  ``a`` fp8 ``[tokens, k]``, ``b`` e4m3
    ``[groups, n, k]``, ``c`` bf16 ``[tokens, n]``, ``batch_sizes`` CPU int64 ``[groups]``."""
    _check(a.is_cuda and b.is_cuda and c.is_cuda, "fp8_gmm: a, b and c must be GPU tensors")
    _check(a.dim() == 2 and a.dtype in _FP8, "fp8_gmm: a must be a 2-D fp8 tensor")
    _check(b.dim() == 3 and b.dtype == torch.float8_e4m3fn, "fp8_gmm: b must be a 3-D float8_e4m3fn tensor")
    _check(c.dim() == 2 and c.dtype == torch.bfloat16, "fp8_gmm: c must be a 2-D bfloat16 tensor")
    _check(a.is_contiguous() and b.is_contiguous() and c.is_contiguous(), "fp8_gmm: a, b and c must be contiguous")
    _check(not batch_sizes.is_cuda and batch_sizes.dim() == 1 and batch_sizes.dtype == torch.int64,
           "fp8_gmm: batch_sizes must be a 1-D int64 CPU tensor")
    _check(batch_sizes.numel() == b.size(0), "fp8_gmm: one batch size per group of b")
    _check(a.size(1) == b.size(2), "fp8_gmm: the contraction sizes of a and b differ")
    _check(c.size(0) == a.size(0) and c.size(1) == b.size(1), "fp8_gmm: c must be [tokens, n]")
    _backend.fp8_gmm(a, b, batch_sizes, None, None, c, backward=(a.dtype == torch.float8_e5m2))


def multi_quantize(input_list, output_list, scale_list, amax_list):
    """``MultiQuantize`` (csrc/multi_pointwise.cu:155-214): ``output = fp8(input * scale)``, amax merged."""
    _backend.multi_quantize(list(input_list), list(output_list), list(scale_list), list(amax_list))


def multi_scale_mul(input_list, scale_list_1, scale_list_2):
    """``MultiScaleMul`` (csrc/multi_pointwise.cu:216-259): in place ``input = bf16(input * scale_1 * scale_2)``."""
    _backend.multi_scale_mul(list(input_list), list(scale_list_1), list(scale_list_2))


def multi_pad_transpose(input_list, transpose_list):
    """``MultiPadTranspose`` (csrc/multi_pad_fusion.cu:442-503): fp8 ``[m, n]`` -> fp8 ``[n, M >= m]``, zero padded."""
    _backend.multi_transpose(list(input_list), list(transpose_list))


def multi_pad_cast_transpose(input_list, output_list, transpose_list, scale_list, amax_list):
    """``MultiPadCastTranspose`` (csrc/multi_pad_fusion.cu:505-585)."""
    _backend.multi_cast_transpose(list(input_list), list(output_list), list(transpose_list), list(scale_list),
                                  list(amax_list))


def multi_pad_cast_transpose_dgelu(input_list, gelu_input_list, output_list, transpose_list, scale_list, amax_list):
    """``MultiPadCastTransposeDgelu`` (csrc/multi_pad_fusion.cu:587-670)."""
    _backend.multi_cast_transpose_dgelu(list(input_list), list(gelu_input_list), list(output_list),
                                        list(transpose_list), list(scale_list), list(amax_list))
