"""``GroupedLinear``: E expert linears on token-sorted rows, FP8 forward and backward.

Same surface and data flow as the reference's ``fp8_gmm/grouped_linear.py``
(``_GroupedLinear`` :11-183, ``GroupedLinear`` :186-214):

forward   one multi-tensor cast launch over the E activation slices and the E weights
          (e4m3 under HYBRID), then one grouped GEMM
          ``out[rows_i] = x_fp8[rows_i] . w_fp8[i]^T * (x_scale_inv_i * w_scale_inv_i)``.
backward  one cast launch over the E slices of grad_out (e5m2), a grouped dgrad GEMM
          ``dX[rows_i] = dY_i . W_i`` and a grouped wgrad GEMM ``dW[i] = dY_i^T . X_i``.
          In the reference's layout (``reference_layout=True``) the casts also write
          transposed copies - the weights as ``[E, K, N]``, activations and gradients as
          ``[features, Mpad_i]`` with the expert's rows padded to a multiple with zeros -
          and both gradient GEMMs take those; by default they read the row-major fp8
          tensors in place.

Differences from the reference: experts with zero tokens are allowed (their weight
gradient is zero), wgrad is a single launch instead of a per-expert loop, and the
grouped GEMM is the same HIP kernel whatever ``cutlass`` says (``cutlass=True`` keeps
the two-rounding data flow of the reference's CUTLASS path, see ``backend.fp8_gmm``).
"""
import contextlib
import math

import numpy as np
import torch

from . import _lib
from .backend import (TensorBatch, batched_uploads, fp8_gmm, grouped_gemm, linear_pass, multi_cast_transpose,
                      multi_quantize, wgrad_wants_transposed_gradient)
from .fp8 import Fp8GroupedModuleBase, Fp8WeightCache, get_fp8_te_dtype
from .utils import PAD_MULTIPLE, Fp8MetaWrapper, Fp8TensorType, MetaTensorType, cumsum_group_sizes, to_torch_dtype


# Per-expert token counts are padded to this multiple in the TRANSPOSED operands of the weight-gradient
# GEMMs (zeros along the contraction dimension, so results do not change).  The reference pads to 16,
# what cuBLASLt needs (fp8_gmm/utils.py:57); here the natural unit is the 128 bytes of one K step of the
# MFMA pipeline, which also keeps every row of those operands aligned to a cache line.
MODULE_PAD_MULTIPLE = 128


def row_slices(t, bounds):
    """Per-expert row blocks of a token-major tensor (described by arrays: no per-expert tensor objects)."""
    return TensorBatch.rows_of(t, bounds)


def transposed_views(flat, bounds):
    """Per-expert ``[features, tokens_i]`` blocks of a flat ``[sum(tokens_i), features]`` buffer.

    Expert i owns the contiguous block of rows ``bounds[i]:bounds[i+1]``; the block is
    reinterpreted as the transpose ``[features, bounds[i+1]-bounds[i]]``
    (reference grouped_linear.py:36-52).
    """
    return TensorBatch.transposed_blocks_of(flat, bounds)


def alloc_transposed(features, padded, bounds, padded_bounds, dtype, device):
    """Buffer + per-expert blocks for the transposed copy of a ``[tokens, features]`` operand."""
    b = padded_bounds if padded else bounds
    flat = torch.empty(b[-1], features, dtype=dtype, device=device)
    return flat, transposed_views(flat, b)


def stage_weight_cast(weight, fp8_dtype, transpose_needed, cache_transposes, cache, update, scales, amaxes, plain,
                      with_t):
    """Chooses where the fp8 copies of a ``[E, N, K]`` weight stack live and appends their cast to the pending
    cast lists (``plain``: cast only, ``with_t``: cast + transpose).  Returns ``(weight_fp8, weight_t_fp8)``.

    ``transpose_needed``: this pass uses a transposed copy (only in the reference's layout, where the
    data-gradient GEMM reads ``[E, K, N]``, grouped_linear.py:64-85; by default that GEMM reads the row-major copy
    in place and nothing is transposed).  Without a cache the copies are temporaries of this pass.  With a
    cache (fp8.Fp8WeightCache) they are the module's buffers: a refreshing pass casts into them - with the
    transpose whenever ``cache_transposes`` says later micro-batches may need it - and a reusing pass appends
    nothing."""
    e, n, k = weight.shape
    if cache is None:
        weight_fp8 = torch.empty(weight.shape, dtype=fp8_dtype, device=weight.device)
        weight_t_fp8 = torch.empty(e, k, n, dtype=fp8_dtype, device=weight.device) if transpose_needed else None
        cast_t = transpose_needed
    else:
        weight_fp8, weight_t_fp8 = cache.buffers(weight, fp8_dtype, cache_transposes or transpose_needed)
        if not update:
            cache.require(transpose_needed)
            return weight_fp8, (weight_t_fp8 if transpose_needed else None)
        cast_t = cache_transposes or transpose_needed
        cache.valid, cache.valid_t = True, cast_t
    if cast_t:
        for lst, item in zip(with_t, (TensorBatch.stack_of(weight), TensorBatch.stack_of(weight_fp8),
                                      TensorBatch.stack_of(weight_t_fp8), scales, amaxes)):
            lst.append(item)
    else:
        for lst, item in zip(plain, (TensorBatch.stack_of(weight), TensorBatch.stack_of(weight_fp8), scales,
                                     amaxes)):
            lst.append(item)
    return weight_fp8, (weight_t_fp8 if transpose_needed else None)


class _GroupedLinear(torch.autograd.Function):
    # Each pass queues its launches and uploads all their tables with one copy (backend.batched_uploads).
    @staticmethod
    def forward(ctx, *args):
        with batched_uploads():
            return _GroupedLinear._forward(ctx, *args)

    @staticmethod
    def backward(ctx, grad_out):
        with batched_uploads():
            return _GroupedLinear._backward(ctx, grad_out)

    @staticmethod
    def _forward(ctx, input, weight, group_sizes, fp8_meta, is_grad_enabled, cutlass, weight_cache=None,
                 update_fp8_weights=True):
        """The reference's argument list (grouped_linear.py:13) plus, as TransformerEngine's own linear layers
        have them, the cache of fp8 weights and whether this pass refreshes it."""
        wgrad_needed = is_grad_enabled and weight.requires_grad
        dgrad_needed = is_grad_enabled and input.requires_grad
        # By default the gradient GEMMs read the row-major fp8 tensors in place; the reference's layout
        # (transposed fp8 weights, padded transposed activations and gradients) is cast only on request, or when
        # a feature count is not a multiple of 16 (the in-place GEMMs fetch 16-byte pieces along the features).
        reference_layout = bool(fp8_meta.get("reference_layout", False)) or weight.size(1) % 16 != 0 \
            or weight.size(2) % 16 != 0
        num_groups, padded, cumsums, padded_cumsums = cumsum_group_sizes(
            group_sizes.tolist() if isinstance(group_sizes, torch.Tensor) else group_sizes,
            need_padding=wgrad_needed and reference_layout,
            pad_multiple=fp8_meta.get("pad_multiple", PAD_MULTIPLE),
        )
        if cumsums[-1] != input.size(0):
            raise RuntimeError("group_sizes must sum to the number of input rows")
        meta = Fp8MetaWrapper(num_groups, fp8_meta)
        fwd_dtype = get_fp8_te_dtype(fp8_meta["recipe"], fprop_tensor=True)
        fp8_dtype = to_torch_dtype(fwd_dtype)
        dev = input.device

        if fp8_meta.get("planned_passes", True) and not reference_layout and not cutlass and input.is_cuda \
                and input.is_contiguous() and weight.is_contiguous() \
                and input.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16:
            # The default data flow as one planned pass: every table of the cast launch and of the GEMM comes out of
            # one library call (with 64 experts the array arithmetic below costs more host time than the kernels run).
            sizes = np.diff(np.asarray(cumsums, dtype=np.int64))
            input_fp8 = torch.empty(input.shape, dtype=fp8_dtype, device=dev)
            if weight_cache is None:
                weight_fp8, cast_weights = torch.empty(weight.shape, dtype=fp8_dtype, device=dev), True
            else:
                weight_fp8, _ = weight_cache.buffers(weight, fp8_dtype, False)
                cast_weights = bool(update_fp8_weights)
                if cast_weights:
                    weight_cache.valid, weight_cache.valid_t = True, False
                else:
                    weight_cache.require(False)
            out = torch.empty(input.size(0), weight.size(1), dtype=torch.bfloat16, device=dev)
            fwd = fp8_meta["scaling_fwd"]
            linear_pass(dev, False, experts=num_groups, in_features=weight.size(2), out_features=weight.size(1),
                        fwd_fmt=_lib.E4M3 if fp8_dtype == torch.float8_e4m3fn else _lib.E5M2, cast_weights=cast_weights,
                        tokens=input.size(0), group_sizes=sizes, x=input, x_fp8=input_fp8, w=weight, w_fp8=weight_fp8,
                        y=out, fwd_scale=fwd.scale, fwd_scale_inv=fwd.scale_inv, fwd_amax=fwd.amax_history)
            if is_grad_enabled:
                ctx.save_for_backward(input_fp8 if wgrad_needed else None, weight_fp8 if dgrad_needed else None)
                ctx.reference_layout = False
                ctx.planned = True
                ctx.sizes = sizes
                ctx.group_sizes = group_sizes
                meta.set_forward_scale_inv_cloned()
                ctx.meta = meta
                ctx.num_groups = num_groups
                ctx.padded = padded
                ctx.cumsums = cumsums
                ctx.padded_cumsums = padded_cumsums
                ctx.fp8_meta = fp8_meta
                ctx.weight_shape = weight.shape
                ctx.input_requires_grad = input.requires_grad
                ctx.weight_requires_grad = weight.requires_grad
                ctx.cutlass = cutlass
            return out

        plain = ([], [], [], [])            # inputs, outputs, scales, amaxes for cast only
        with_t = ([], [], [], [], [])       # inputs, outputs, transposes, scales, amaxes

        input_fp8 = torch.empty(input.shape, dtype=fp8_dtype, device=dev)
        input_t_fp8 = None
        x_scales = meta.get_meta_pointers(Fp8TensorType.kInputGroup1, MetaTensorType.kScale)
        x_amaxes = meta.get_meta_pointers(Fp8TensorType.kInputGroup1, MetaTensorType.kAmax)
        if wgrad_needed and reference_layout:
            input_t_fp8, x_t_views = alloc_transposed(input.size(1), padded, cumsums, padded_cumsums,
                                                      fp8_dtype, dev)
            for lst, item in zip(with_t, (row_slices(input, cumsums), row_slices(input_fp8, cumsums), x_t_views,
                                          x_scales, x_amaxes)):
                lst.append(item)
        else:
            for lst, item in zip(plain, (row_slices(input, cumsums), row_slices(input_fp8, cumsums), x_scales,
                                         x_amaxes)):
                lst.append(item)

        w_scales = meta.get_meta_pointers(Fp8TensorType.kWeightGroup1, MetaTensorType.kScale)
        w_amaxes = meta.get_meta_pointers(Fp8TensorType.kWeightGroup1, MetaTensorType.kAmax)
        weight_fp8, weight_t_fp8 = stage_weight_cast(
            weight, fp8_dtype, dgrad_needed and reference_layout, is_grad_enabled and reference_layout,
            weight_cache, update_fp8_weights, w_scales, w_amaxes, plain, with_t)

        if plain[0]:
            multi_quantize(TensorBatch.concat(plain[0]), TensorBatch.concat(plain[1]), np.concatenate(plain[2]),
                           np.concatenate(plain[3]))
        if with_t[0]:
            multi_cast_transpose(TensorBatch.concat(with_t[0]), TensorBatch.concat(with_t[1]),
                                 TensorBatch.concat(with_t[2]), np.concatenate(with_t[3]), np.concatenate(with_t[4]))

        out = fp8_gmm(
            input_fp8, weight_fp8, group_sizes,
            meta.get_meta_pointers(Fp8TensorType.kInputGroup1, MetaTensorType.kScaleInv),
            meta.get_meta_pointers(Fp8TensorType.kWeightGroup1, MetaTensorType.kScaleInv),
            backward=False, cutlass=cutlass,
        )

        if is_grad_enabled:
            if reference_layout:
                ctx.save_for_backward(input_t_fp8, weight_t_fp8)
            else:
                ctx.save_for_backward(input_fp8 if wgrad_needed else None, weight_fp8 if dgrad_needed else None)
            ctx.reference_layout = reference_layout
            ctx.planned = False
            ctx.group_sizes = group_sizes
            meta.set_forward_scale_inv_cloned()
            ctx.meta = meta
            ctx.num_groups = num_groups
            ctx.padded = padded
            ctx.cumsums = cumsums
            ctx.padded_cumsums = padded_cumsums
            ctx.fp8_meta = fp8_meta
            ctx.weight_shape = weight.shape
            ctx.input_requires_grad = input.requires_grad
            ctx.weight_requires_grad = weight.requires_grad
            ctx.cutlass = cutlass
        return out

    @staticmethod
    def _backward(ctx, grad_out):
        input_for_wgrad, weight_for_dgrad = ctx.saved_tensors   # transposed copies in the reference's layout
        meta = ctx.meta
        cumsums, padded_cumsums, padded = ctx.cumsums, ctx.padded_cumsums, ctx.padded
        grad_dtype = to_torch_dtype(get_fp8_te_dtype(ctx.fp8_meta["recipe"], fprop_tensor=False))
        grad_out = grad_out.contiguous()
        dev = grad_out.device

        if ctx.planned and not wgrad_wants_transposed_gradient(cumsums[-1], ctx.num_groups) \
                and grad_out.dtype == torch.bfloat16 and (ctx.input_requires_grad or ctx.weight_requires_grad):
            e, n, k = ctx.weight_shape
            grad_out_fp8 = torch.empty(grad_out.shape, dtype=grad_dtype, device=dev)
            grad_input = torch.empty(grad_out.size(0), k, dtype=torch.bfloat16, device=dev) \
                if ctx.input_requires_grad else None
            grad_weight = torch.empty(ctx.weight_shape, dtype=torch.bfloat16, device=dev) \
                if ctx.weight_requires_grad else None
            bwd = ctx.fp8_meta["scaling_bwd"]
            fwd_fmt = get_fp8_te_dtype(ctx.fp8_meta["recipe"], fprop_tensor=True)
            linear_pass(dev, True, experts=e, in_features=k, out_features=n,
                        fwd_fmt=_lib.E4M3 if to_torch_dtype(fwd_fmt) == torch.float8_e4m3fn else _lib.E5M2,
                        bwd_fmt=_lib.E4M3 if grad_dtype == torch.float8_e4m3fn else _lib.E5M2,
                        dgrad=int(ctx.input_requires_grad), wgrad=int(ctx.weight_requires_grad),
                        tokens=grad_out.size(0), group_sizes=ctx.sizes, dy=grad_out, dy_fp8=grad_out_fp8,
                        x_fp8=input_for_wgrad, w_fp8=weight_for_dgrad, dx=grad_input, dw=grad_weight,
                        fwd_scale_inv=meta._forward_scale_inv_cloned, bwd_scale=bwd.scale,
                        bwd_scale_inv=bwd.scale_inv, bwd_amax=bwd.amax_history)
            return grad_input, grad_weight, None, None, None, None, None, None

        g_scales = meta.get_meta_pointers(Fp8TensorType.kGradOutputGroup1, MetaTensorType.kScale)
        g_amaxes = meta.get_meta_pointers(Fp8TensorType.kGradOutputGroup1, MetaTensorType.kAmax)
        g_scale_invs = meta.get_meta_pointers(Fp8TensorType.kGradOutputGroup1, MetaTensorType.kScaleInv)
        grad_out_fp8 = torch.empty(grad_out.shape, dtype=grad_dtype, device=dev)
        g_t_views = None
        # on request (backend.wgrad_wants_transposed_gradient) the weight gradient runs on a transposed copy of the
        # gradient; the activation is still read where it lies
        grad_copy = ctx.weight_requires_grad and not ctx.reference_layout and \
            wgrad_wants_transposed_gradient(cumsums[-1], ctx.num_groups)
        if grad_copy:
            _, copy_padded, _, copy_bounds = cumsum_group_sizes(
                np.diff(np.asarray(cumsums)).tolist(), need_padding=True,
                pad_multiple=ctx.fp8_meta.get("pad_multiple", PAD_MULTIPLE))
            _, g_t_views = alloc_transposed(grad_out.size(1), copy_padded, cumsums, copy_bounds, grad_dtype, dev)
            multi_cast_transpose(row_slices(grad_out, cumsums), row_slices(grad_out_fp8, cumsums), g_t_views,
                                 g_scales, g_amaxes)
        elif ctx.weight_requires_grad and ctx.reference_layout:
            _, g_t_views = alloc_transposed(grad_out.size(1), padded, cumsums, padded_cumsums, grad_dtype,
                                            dev)
            multi_cast_transpose(row_slices(grad_out, cumsums), row_slices(grad_out_fp8, cumsums), g_t_views,
                                 g_scales, g_amaxes)
        else:
            multi_quantize(row_slices(grad_out, cumsums), row_slices(grad_out_fp8, cumsums), g_scales, g_amaxes)

        # the weight gradient first (the reference runs it second, grouped_linear.py:153-184): its operands are what
        # the casts have just written, and behind the data gradient's pass over all the weights less of them is left in
        # the memory-side cache
        grad_weight = None
        if ctx.weight_requires_grad:
            grad_weight = torch.empty(ctx.weight_shape, dtype=torch.bfloat16, device=dev)
            x_scale_invs = meta.get_meta_pointers(Fp8TensorType.kForwardInputGroup1, MetaTensorType.kScaleInv)
            if ctx.reference_layout:
                x_t_views = transposed_views(input_for_wgrad, padded_cumsums if padded else cumsums)
                grouped_gemm(g_t_views, x_t_views, TensorBatch.stack_of(grad_weight), g_scale_invs, x_scale_invs)
            elif grad_copy:
                grouped_gemm(g_t_views, row_slices(input_for_wgrad, cumsums), TensorBatch.stack_of(grad_weight),
                             g_scale_invs, x_scale_invs, transposed="b")
            else:  # dW[i] = dY_i^T . X_i on the row-major slices, contraction over the expert's rows
                grouped_gemm(row_slices(grad_out_fp8, cumsums), row_slices(input_for_wgrad, cumsums),
                             TensorBatch.stack_of(grad_weight), g_scale_invs, x_scale_invs, transposed=True)

        grad_input = None
        if ctx.input_requires_grad:
            grad_input = fp8_gmm(
                grad_out_fp8, weight_for_dgrad, ctx.group_sizes, g_scale_invs,
                meta.get_meta_pointers(Fp8TensorType.kForwardWeightGroup1, MetaTensorType.kScaleInv),
                backward=True, cutlass=ctx.cutlass, b_transposed=not ctx.reference_layout,
            )
        return grad_input, grad_weight, None, None, None, None, None, None


class GroupedLinear(Fp8GroupedModuleBase):
    """E independent ``in_features -> out_features`` linears (no bias) over token-sorted rows.

    ``forward(input[tokens, in_features], group_sizes[E])`` where ``group_sizes`` is a CPU
    int64 tensor (or list) of rows per expert, in order; returns ``[tokens, out_features]`` bf16.
    ``reference_layout=True`` keeps the reference's buffers: transposed fp8 weights ``[E, K, N]`` for the
    data-gradient GEMM and zero-padded transposed fp8 activations / gradients for the weight-gradient GEMM.  By
    default those GEMMs read the row-major fp8 tensors in place and none of the copies is cast: same results bit
    for bit, less memory traffic, no padding.
    ``planned_passes=False`` builds the tables of every launch in Python through the per-launch entry points of
    ``backend`` (the same tables, several times the host time).
    ``is_first_microbatch``: None casts the weights to fp8 on every pass; True casts them into buffers the
    module keeps; False reuses those buffers (gradient accumulation over micro-batches of one optimizer step).
    """

    def __init__(self, in_features, out_features, num_groups, dtype, device="cuda", cutlass=False,
                 pad_multiple=MODULE_PAD_MULTIPLE, reference_layout=False, planned_passes=True):
        super().__init__()
        self.fp8_meta["pad_multiple"] = pad_multiple
        self.fp8_meta["reference_layout"] = reference_layout
        self.fp8_meta["planned_passes"] = planned_passes
        assert dtype == torch.bfloat16, "bfloat16 parameters only"
        self.in_features = in_features
        self.out_features = out_features
        self.num_groups = num_groups
        self.cutlass = cutlass
        self.weight_tensor = torch.nn.Parameter(
            torch.empty(num_groups, out_features, in_features, dtype=dtype, device=device)
        )
        bound = math.sqrt(1.0 / in_features)
        torch.nn.init.uniform_(self.weight_tensor.data, -bound, bound)
        self._weight_cache = Fp8WeightCache()
        self._weight_caches.append(self._weight_cache)

    def get_fp8_weights_scratchpad(self, is_first_microbatch):
        """``[weight_fp8, weight_t_fp8]``: the buffers that keep the fp8 weights across micro-batches, or Nones
        when ``is_first_microbatch`` is None and every pass casts into temporaries (all the reference
        supports, grouped_linear.py:200-202)."""
        if is_first_microbatch is None:
            return [None, None]
        dtype = to_torch_dtype(get_fp8_te_dtype(self.fp8_meta["recipe"], fprop_tensor=True))
        return list(self._weight_cache.buffers(self.weight_tensor, dtype, self.fp8_meta["reference_layout"]))

    def cast_weights_ahead(self):
        """Start the next forward pass before its group sizes are known: the delayed-scaling update and the cast of
        the weights to fp8 are enqueued now, and the next ``forward(input, group_sizes)`` runs only what is left, with
        the same results.  For callers whose sizes come from the device (a router): the GPU works on the weights
        while the host waits for the sizes and plans the launches.  No counterpart in the reference.  Returns False,
        having done nothing, for a module in the reference's layout."""
        return self._cast_ahead([(self.weight_tensor, Fp8TensorType.kWeightGroup1)])

    def forward(self, input, group_sizes, is_first_microbatch=None):
        ahead = self._take_ahead(is_first_microbatch)
        with (contextlib.nullcontext() if ahead is not None else
              self.prepare_forward(input, is_first_microbatch, self.num_groups)):
            grad = torch.is_grad_enabled()
            args = (input, self.weight_tensor, group_sizes, self.fp8_meta, grad, self.cutlass)
            if ahead is not None:
                args += (ahead[0], False)
            elif is_first_microbatch is not None:
                args += (self._weight_cache, bool(is_first_microbatch))
            if grad:
                return _GroupedLinear.apply(*args)
            return _GroupedLinear.forward(None, *args)
