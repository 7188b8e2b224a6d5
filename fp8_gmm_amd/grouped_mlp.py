"""``GroupedMlp``: E expert MLPs (fc1 -> tanh-GELU -> fc2) on token-sorted rows in FP8.

Same surface and data flow as the reference's ``fp8_gmm/grouped_mlp.py``
(``_GroupedMlp`` :18-325, ``GroupedMlp`` :328-366).  ``GroupedMlp(in=H, out=F)`` owns
``fc1_weight [E, F, H]`` and ``fc2_weight [E, H, F]``.

forward   one cast launch over the E activation slices and 2E weights;
          fc1 grouped GEMM with the GELU-aux epilogue (writes bf16 pre-GELU values and
          the e4m3 GELU output scaled by the InputGroup2 scale, recording its amax);
          fc2 grouped GEMM to bf16.
backward  cast of grad_out to e5m2; fc2 wgrad; fc2 dgrad; fused (dgelu * grad) cast under
          the GradOutputGroup2 scale; fc1 dgrad (optionally all-reduced over a
          tensor-parallel group, overlapped with fc1 wgrad); fc1 wgrad.

In the reference's layout (``reference_layout=True``) every cast also writes the transposed
copy its gradient GEMM takes (weights ``[E, K, N]``; activations, the GELU output and the
gradients zero-padded per expert), as grouped_mlp.py:60-150,196-262 does; by default the
gradient GEMMs read the row-major fp8 tensors in place and no such copy exists.

Experts with zero tokens are allowed; each wgrad is one grouped launch.  In the default layout a whole pass is
planned by one library call (``backend.mlp_pass``); the launch-by-launch code below it builds the same tables and
serves the other layouts and options.
"""
import contextlib
import math

import numpy as np
import torch

from . import _lib
from .backend import (
    TensorBatch,
    batched_uploads,
    flush_uploads,
    fp8_gmm,
    grouped_gemm,
    mlp_pass,
    multi_cast_transpose,
    multi_cast_dgelu,
    multi_cast_transpose_dgelu,
    multi_quantize,
    multi_transpose,
    wgrad_wants_transposed_gradient,
)
from .fp8 import Fp8GroupedModuleBase, Fp8WeightCache, get_fp8_te_dtype
from .grouped_linear import MODULE_PAD_MULTIPLE, alloc_transposed, row_slices, stage_weight_cast, transposed_views
from .utils import PAD_MULTIPLE, Fp8MetaWrapper, Fp8TensorType, MetaTensorType, cumsum_group_sizes, to_torch_dtype

_T = Fp8TensorType
_M = MetaTensorType


class _GroupedMlp(torch.autograd.Function):
    # Each pass queues its launches and uploads all their tables with one copy (backend.batched_uploads).
    @staticmethod
    def forward(ctx, *args):
        with batched_uploads():
            return _GroupedMlp._forward(ctx, *args)

    @staticmethod
    def backward(ctx, grad_out):
        with batched_uploads():
            return _GroupedMlp._backward(ctx, grad_out)

    @staticmethod
    def _forward(ctx, input, fc1_weight, fc2_weight, group_sizes, fp8_meta, is_grad_enabled, has_tp, tp_group,
                 weight_caches=(None, None), update_fp8_weights=True):
        input_requires_grad = input.requires_grad
        weight_requires_grad = fc1_weight.requires_grad
        wgrad_needed = is_grad_enabled and weight_requires_grad
        # fc2's transposed weights feed the fc2 dgrad, which both the input and the fc1 weight gradients need
        dgrad_needed = is_grad_enabled and (input_requires_grad or weight_requires_grad)
        # in-place gradient GEMMs unless the reference's layout is asked for (see GroupedLinear)
        reference_layout = bool(fp8_meta.get("reference_layout", False)) or fc1_weight.size(1) % 16 != 0 \
            or fc1_weight.size(2) % 16 != 0
        num_groups, padded, cumsums, padded_cumsums = cumsum_group_sizes(
            group_sizes.tolist() if isinstance(group_sizes, torch.Tensor) else group_sizes,
            need_padding=wgrad_needed and reference_layout,
            pad_multiple=fp8_meta.get("pad_multiple", PAD_MULTIPLE),
        )
        if cumsums[-1] != input.size(0):
            raise RuntimeError("group_sizes must sum to the number of input rows")
        meta = Fp8MetaWrapper(num_groups, fp8_meta)
        fp8_dtype = to_torch_dtype(get_fp8_te_dtype(fp8_meta["recipe"], fprop_tensor=True))
        dev = input.device
        tokens, ffn = input.size(0), fc1_weight.size(1)

        if fp8_meta.get("planned_passes", True) and not reference_layout and input.is_cuda \
                and input.is_contiguous() and fc1_weight.is_contiguous() and fc2_weight.is_contiguous() \
                and input.dtype == fc1_weight.dtype == fc2_weight.dtype == torch.bfloat16:
            # The default data flow as one planned pass: the tables of the cast launch and of both GEMMs come out of
            # one library call and reach the device in one upload (the same tables, to the byte, that the code below
            # builds array by array - which with 64 experts costs more host time than the kernels run)
            sizes = np.diff(np.asarray(cumsums, dtype=np.int64))
            input_fp8 = torch.empty(input.shape, dtype=fp8_dtype, device=dev)
            weights_fp8 = []
            cast_weights = True
            for weight, cache in zip((fc1_weight, fc2_weight), weight_caches):
                if cache is None:
                    weights_fp8.append(torch.empty(weight.shape, dtype=fp8_dtype, device=dev))
                    continue
                weights_fp8.append(cache.buffers(weight, fp8_dtype, False)[0])
                cast_weights = bool(update_fp8_weights)
                if cast_weights:
                    cache.valid, cache.valid_t = True, False
                else:
                    cache.require(False)
            fc1_weight_fp8, fc2_weight_fp8 = weights_fp8
            pre_gelu_out = torch.empty(tokens, ffn, dtype=torch.bfloat16, device=dev)
            gelu_out_fp8 = torch.empty(tokens, ffn, dtype=fp8_dtype, device=dev)
            out = torch.empty(tokens, input.size(1), dtype=torch.bfloat16, device=dev)
            fwd = fp8_meta["scaling_fwd"]
            mlp_pass(dev, False, experts=num_groups, hidden=input.size(1), ffn=ffn,
                     fwd_fmt=_lib.E4M3 if fp8_dtype == torch.float8_e4m3fn else _lib.E5M2, cast_weights=cast_weights,
                     tokens=tokens, group_sizes=sizes, x=input, x_fp8=input_fp8, w1=fc1_weight, w1_fp8=fc1_weight_fp8,
                     w2=fc2_weight, w2_fp8=fc2_weight_fp8, pre=pre_gelu_out, act_fp8=gelu_out_fp8, y=out,
                     fwd_scale=fwd.scale, fwd_scale_inv=fwd.scale_inv, fwd_amax=fwd.amax_history)
            capture = fp8_meta.get("capture")
            if capture is not None:  # see GroupedMlp.capture_intermediates
                capture.update(pre_gelu_out=pre_gelu_out, gelu_out_fp8=gelu_out_fp8)
            if is_grad_enabled:
                ctx.save_for_backward(input_fp8 if wgrad_needed else None,
                                      fc1_weight_fp8 if (dgrad_needed and input_requires_grad) else None,
                                      fc2_weight_fp8 if dgrad_needed else None, pre_gelu_out,
                                      gelu_out_fp8 if wgrad_needed else None)
                ctx.planned = True
                ctx.sizes = sizes
                _GroupedMlp._remember(ctx, False, group_sizes, meta, num_groups, padded, cumsums, padded_cumsums, fp8_meta,
                                      fc1_weight, fc2_weight, input_requires_grad, weight_requires_grad, has_tp, tp_group)
            return out

        plain = ([], [], [], [])
        with_t = ([], [], [], [], [])

        input_fp8 = torch.empty(input.shape, dtype=fp8_dtype, device=dev)
        input_t_fp8 = None
        x_scales = meta.get_meta_pointers(_T.kInputGroup1, _M.kScale)
        x_amaxes = meta.get_meta_pointers(_T.kInputGroup1, _M.kAmax)
        if wgrad_needed and reference_layout:
            input_t_fp8, x_t_views = alloc_transposed(input.size(1), padded, cumsums, padded_cumsums, fp8_dtype, dev)
            for lst, item in zip(with_t, (row_slices(input, cumsums), row_slices(input_fp8, cumsums), x_t_views,
                                          x_scales, x_amaxes)):
                lst.append(item)
        else:
            for lst, item in zip(plain, (row_slices(input, cumsums), row_slices(input_fp8, cumsums), x_scales,
                                         x_amaxes)):
                lst.append(item)

        need_t, cache_t = dgrad_needed and reference_layout, is_grad_enabled and reference_layout
        fc1_weight_fp8, fc1_weight_t_fp8 = stage_weight_cast(
            fc1_weight, fp8_dtype, need_t, cache_t, weight_caches[0], update_fp8_weights,
            meta.get_meta_pointers(_T.kWeightGroup1, _M.kScale), meta.get_meta_pointers(_T.kWeightGroup1, _M.kAmax),
            plain, with_t)
        fc2_weight_fp8, fc2_weight_t_fp8 = stage_weight_cast(
            fc2_weight, fp8_dtype, need_t, cache_t, weight_caches[1], update_fp8_weights,
            meta.get_meta_pointers(_T.kWeightGroup2, _M.kScale), meta.get_meta_pointers(_T.kWeightGroup2, _M.kAmax),
            plain, with_t)

        if plain[0]:
            # fc2's weights first, the input last: the launch walks its table in order, and what it wrote last is
            # what the memory-side cache still holds when fc1's GEMM starts reading (config 4: that GEMM -14 us)
            plain = tuple(lst[::-1] for lst in plain)
            multi_quantize(TensorBatch.concat(plain[0]), TensorBatch.concat(plain[1]), np.concatenate(plain[2]),
                           np.concatenate(plain[3]))
        if with_t[0]:
            multi_cast_transpose(TensorBatch.concat(with_t[0]), TensorBatch.concat(with_t[1]),
                                 TensorBatch.concat(with_t[2]), np.concatenate(with_t[3]), np.concatenate(with_t[4]))

        pre_gelu_out = torch.empty(tokens, ffn, dtype=torch.bfloat16, device=dev)
        gelu_out_fp8 = torch.empty(tokens, ffn, dtype=fp8_dtype, device=dev)
        # fc1: GELU-aux epilogue, fp8 output scaled for fc2 (slot InputGroup2)
        fp8_gmm(
            input_fp8, fc1_weight_fp8, group_sizes,
            meta.get_meta_pointers(_T.kInputGroup1, _M.kScaleInv),
            meta.get_meta_pointers(_T.kWeightGroup1, _M.kScaleInv),
            c=gelu_out_fp8, pre_gelu_out=pre_gelu_out,
            c_scales=meta.get_meta_pointers(_T.kInputGroup2, _M.kScale),
            c_amaxes=meta.get_meta_pointers(_T.kInputGroup2, _M.kAmax),
            backward=False, cutlass=False,
        )
        capture = fp8_meta.get("capture")
        if capture is not None:  # see GroupedMlp.capture_intermediates
            capture.update(pre_gelu_out=pre_gelu_out, gelu_out_fp8=gelu_out_fp8)
        if not is_grad_enabled:
            pre_gelu_out = None
        out = fp8_gmm(
            gelu_out_fp8, fc2_weight_fp8, group_sizes,
            meta.get_meta_pointers(_T.kInputGroup2, _M.kScaleInv),
            meta.get_meta_pointers(_T.kWeightGroup2, _M.kScaleInv),
            backward=False, cutlass=False,
        )
        if not wgrad_needed:
            gelu_out_fp8 = None

        if is_grad_enabled:
            if reference_layout:
                x_wgrad, w1_dgrad, w2_dgrad = input_t_fp8, fc1_weight_t_fp8, fc2_weight_t_fp8
            else:  # the gradient GEMMs read the row-major copies in place
                x_wgrad = input_fp8 if wgrad_needed else None
                w1_dgrad = fc1_weight_fp8 if (dgrad_needed and input_requires_grad) else None
                w2_dgrad = fc2_weight_fp8 if dgrad_needed else None
            ctx.save_for_backward(x_wgrad, w1_dgrad, w2_dgrad, pre_gelu_out, gelu_out_fp8)
            ctx.planned = False
            _GroupedMlp._remember(ctx, reference_layout, group_sizes, meta, num_groups, padded, cumsums, padded_cumsums,
                                  fp8_meta, fc1_weight, fc2_weight, input_requires_grad, weight_requires_grad, has_tp,
                                  tp_group)
        return out

    @staticmethod
    def _remember(ctx, reference_layout, group_sizes, meta, num_groups, padded, cumsums, padded_cumsums, fp8_meta,
                  fc1_weight, fc2_weight, input_requires_grad, weight_requires_grad, has_tp, tp_group):
        """What the backward pass needs besides the saved tensors."""
        ctx.reference_layout = reference_layout
        ctx.group_sizes = group_sizes
        meta.set_forward_scale_inv_cloned()
        ctx.meta = meta
        ctx.num_groups = num_groups
        ctx.padded = padded
        ctx.cumsums = cumsums
        ctx.padded_cumsums = padded_cumsums
        ctx.fp8_meta = fp8_meta
        ctx.fc1_weight_shape = fc1_weight.shape
        ctx.fc2_weight_shape = fc2_weight.shape
        ctx.input_requires_grad = input_requires_grad
        ctx.weight_requires_grad = weight_requires_grad
        ctx.has_tp = has_tp
        if has_tp:
            assert tp_group is not None
        ctx.tp_group = tp_group

    @staticmethod
    def _backward(ctx, grad_out):
        input_for_wgrad, fc1_weight_dgrad, fc2_weight_dgrad, pre_gelu_out, gelu_out_fp8 = ctx.saved_tensors
        in_place = not ctx.reference_layout
        b_transposed = in_place
        meta = ctx.meta
        cumsums, padded_cumsums, padded = ctx.cumsums, ctx.padded_cumsums, ctx.padded
        t_bounds = padded_cumsums if padded else cumsums
        grad_dtype = to_torch_dtype(get_fp8_te_dtype(ctx.fp8_meta["recipe"], fprop_tensor=False))
        grad_out = grad_out.contiguous()
        dev = grad_out.device
        wgrad = ctx.weight_requires_grad

        if ctx.planned and not ctx.has_tp and grad_out.dtype == torch.bfloat16 \
                and not ctx.fp8_meta.get("fused_dgelu", False) \
                and not wgrad_wants_transposed_gradient(cumsums[-1], ctx.num_groups):
            # the whole pass from one library call (with a tensor-parallel group the collective between the launches
            # wants the first data gradient flushed on its own: that case takes the per-launch path below)
            bwd = ctx.fp8_meta["scaling_bwd"]
            fwd_dtype = to_torch_dtype(get_fp8_te_dtype(ctx.fp8_meta["recipe"], fprop_tensor=True))
            tokens, ffn = pre_gelu_out.shape
            grad_out_fp8 = torch.empty(grad_out.shape, dtype=grad_dtype, device=dev)
            grad_gelu_out = torch.empty(tokens, ffn, dtype=torch.bfloat16, device=dev)
            grad_pre_fp8 = torch.empty(tokens, ffn, dtype=grad_dtype, device=dev)
            grad_input = torch.empty(grad_out.shape, dtype=torch.bfloat16, device=dev) \
                if ctx.input_requires_grad else None
            grad_fc1_weight = torch.empty(ctx.fc1_weight_shape, dtype=torch.bfloat16, device=dev) if wgrad else None
            grad_fc2_weight = torch.empty(ctx.fc2_weight_shape, dtype=torch.bfloat16, device=dev) if wgrad else None
            mlp_pass(dev, True, experts=ctx.num_groups, hidden=grad_out.size(1), ffn=ffn,
                     fwd_fmt=_lib.E4M3 if fwd_dtype == torch.float8_e4m3fn else _lib.E5M2,
                     bwd_fmt=_lib.E4M3 if grad_dtype == torch.float8_e4m3fn else _lib.E5M2,
                     dgrad=int(ctx.input_requires_grad), wgrad=int(wgrad), tokens=tokens, group_sizes=ctx.sizes,
                     x_fp8=input_for_wgrad, w1_fp8=fc1_weight_dgrad, w2_fp8=fc2_weight_dgrad, pre=pre_gelu_out,
                     act_fp8=gelu_out_fp8, dy=grad_out, dy_fp8=grad_out_fp8, dact=grad_gelu_out, dpre_fp8=grad_pre_fp8,
                     dx=grad_input, dw1=grad_fc1_weight, dw2=grad_fc2_weight,
                     fwd_scale_inv=meta._forward_scale_inv_cloned, bwd_scale=bwd.scale, bwd_scale_inv=bwd.scale_inv,
                     bwd_amax=bwd.amax_history)
            capture = ctx.fp8_meta.get("capture")
            if capture is not None:
                capture.update(grad_gelu_out=grad_gelu_out, grad_pre_fp8=grad_pre_fp8)
            return grad_input, grad_fc1_weight, grad_fc2_weight, None, None, None, None, None, None, None

        g1_scales = meta.get_meta_pointers(_T.kGradOutputGroup1, _M.kScale)
        g1_amaxes = meta.get_meta_pointers(_T.kGradOutputGroup1, _M.kAmax)
        g1_scale_invs = meta.get_meta_pointers(_T.kGradOutputGroup1, _M.kScaleInv)
        grad_out_fp8 = torch.empty(grad_out.shape, dtype=grad_dtype, device=dev)

        # In place, the weight-gradient GEMMs read both operands contraction-major.  On request
        # (backend.wgrad_wants_transposed_gradient) the casts below also write a transposed copy of the gradient,
        # zero-padded per expert, and only the activations are read in place.
        grad_copy = wgrad and in_place and wgrad_wants_transposed_gradient(cumsums[-1], ctx.num_groups)
        if grad_copy:
            _, copy_padded, _, copy_bounds = cumsum_group_sizes(
                np.diff(np.asarray(cumsums)).tolist(), need_padding=True,
                pad_multiple=ctx.fp8_meta.get("pad_multiple", PAD_MULTIPLE))
        grad_fc2_weight = None
        if grad_copy:
            _, g_t_views = alloc_transposed(grad_out.size(1), copy_padded, cumsums, copy_bounds, grad_dtype, dev)
            multi_cast_transpose(row_slices(grad_out, cumsums), row_slices(grad_out_fp8, cumsums), g_t_views,
                                 g1_scales, g1_amaxes)
        elif wgrad and not in_place:
            _, g_t_views = alloc_transposed(grad_out.size(1), padded, cumsums, padded_cumsums, grad_dtype, dev)
            _, gelu_t_views = alloc_transposed(gelu_out_fp8.size(1), padded, cumsums, padded_cumsums,
                                               gelu_out_fp8.dtype, dev)
            multi_cast_transpose(row_slices(grad_out, cumsums), row_slices(grad_out_fp8, cumsums), g_t_views,
                                 g1_scales, g1_amaxes)
            multi_transpose(row_slices(gelu_out_fp8, cumsums), gelu_t_views)
        else:
            multi_quantize(row_slices(grad_out, cumsums), row_slices(grad_out_fp8, cumsums), g1_scales, g1_amaxes)
        if wgrad:
            # fc2 wgrad: dW2[i][H, F] = dY_i^T . gelu_i (reference layout: dY_i^T[H, Mpad] . gelu_i^T[F, Mpad]^T)
            grad_fc2_weight = torch.empty(ctx.fc2_weight_shape, dtype=torch.bfloat16, device=dev)
            gelu_scale_invs = meta.get_meta_pointers(_T.kForwardInputGroup2, _M.kScaleInv)
            if grad_copy:
                grouped_gemm(g_t_views, row_slices(gelu_out_fp8, cumsums), TensorBatch.stack_of(grad_fc2_weight),
                             g1_scale_invs, gelu_scale_invs, transposed="b")
            elif in_place:
                grouped_gemm(row_slices(grad_out_fp8, cumsums), row_slices(gelu_out_fp8, cumsums),
                             TensorBatch.stack_of(grad_fc2_weight), g1_scale_invs, gelu_scale_invs, transposed=True)
            else:
                grouped_gemm(g_t_views, gelu_t_views, TensorBatch.stack_of(grad_fc2_weight), g1_scale_invs,
                             gelu_scale_invs)

        grad_pre_fp8 = torch.empty(pre_gelu_out.shape, dtype=grad_dtype, device=dev)
        g2_scales = meta.get_meta_pointers(_T.kGradOutputGroup2, _M.kScale)
        g2_amaxes = meta.get_meta_pointers(_T.kGradOutputGroup2, _M.kAmax)
        fused = bool(ctx.fp8_meta.get("fused_dgelu", False)) and in_place and not grad_copy
        grad_gelu_out = None
        if fused:
            # fc2 dgrad with the GELU's derivative and the cast in its epilogue: d(pre_gelu) in fp8 straight from the
            # fp32 accumulators; no bf16 d(gelu_out), no separate pass over [tokens, F]
            fp8_gmm(grad_out_fp8, fc2_weight_dgrad, ctx.group_sizes, g1_scale_invs,
                    meta.get_meta_pointers(_T.kForwardWeightGroup2, _M.kScaleInv), c=grad_pre_fp8,
                    c_scales=g2_scales, c_amaxes=g2_amaxes, backward=True, b_transposed=True, dgelu_pre=pre_gelu_out)
        else:
            # fc2 dgrad: d(gelu_out)[tokens, F]
            grad_gelu_out = fp8_gmm(
                grad_out_fp8, fc2_weight_dgrad, ctx.group_sizes, g1_scale_invs,
                meta.get_meta_pointers(_T.kForwardWeightGroup2, _M.kScaleInv),
                backward=True, cutlass=False, b_transposed=b_transposed,
            )

        # d(pre_gelu) = d(gelu_out) * dgelu(pre_gelu), cast to fp8; the padded transpose only feeds fc1 wgrad in
        # the reference's layout (the reference always transposes and notes the missing cast-only kernel,
        # grouped_mlp.py:252-253)
        if fused:
            pass
        elif grad_copy or (wgrad and not in_place):
            if grad_copy:
                _, grad_pre_t_views = alloc_transposed(pre_gelu_out.size(1), copy_padded, cumsums, copy_bounds,
                                                       grad_dtype, dev)
            else:
                _, grad_pre_t_views = alloc_transposed(pre_gelu_out.size(1), padded, cumsums, padded_cumsums,
                                                       grad_dtype, dev)
            multi_cast_transpose_dgelu(
                row_slices(grad_gelu_out, cumsums), row_slices(pre_gelu_out, cumsums),
                row_slices(grad_pre_fp8, cumsums), grad_pre_t_views, g2_scales, g2_amaxes,
            )
        else:
            multi_cast_dgelu(row_slices(grad_gelu_out, cumsums), row_slices(pre_gelu_out, cumsums),
                             row_slices(grad_pre_fp8, cumsums), g2_scales, g2_amaxes)
        g2_scale_invs = meta.get_meta_pointers(_T.kGradOutputGroup2, _M.kScaleInv)
        capture = ctx.fp8_meta.get("capture")
        if capture is not None:
            capture.update(grad_gelu_out=grad_gelu_out, grad_pre_fp8=grad_pre_fp8)

        grad_input = None
        handle = None
        if ctx.input_requires_grad:
            grad_input = fp8_gmm(
                grad_pre_fp8, fc1_weight_dgrad, ctx.group_sizes, g2_scale_invs,
                meta.get_meta_pointers(_T.kForwardWeightGroup1, _M.kScaleInv),
                backward=True, cutlass=False, b_transposed=b_transposed,
            )
            if ctx.has_tp:
                flush_uploads()  # the collective must see grad_input
                handle = torch.distributed.all_reduce(
                    grad_input, op=torch.distributed.ReduceOp.SUM, group=ctx.tp_group, async_op=True
                )

        grad_fc1_weight = None
        if wgrad:
            # fc1 wgrad: dW1[i][F, H] = d(pre)_i^T[F, Mpad] . X_i^T[H, Mpad]^T
            grad_fc1_weight = torch.empty(ctx.fc1_weight_shape, dtype=torch.bfloat16, device=dev)
            x_scale_invs = meta.get_meta_pointers(_T.kForwardInputGroup1, _M.kScaleInv)
            if grad_copy:
                grouped_gemm(grad_pre_t_views, row_slices(input_for_wgrad, cumsums),
                             TensorBatch.stack_of(grad_fc1_weight), g2_scale_invs, x_scale_invs, transposed="b")
            elif in_place:
                grouped_gemm(row_slices(grad_pre_fp8, cumsums), row_slices(input_for_wgrad, cumsums),
                             TensorBatch.stack_of(grad_fc1_weight), g2_scale_invs, x_scale_invs, transposed=True)
            else:
                grouped_gemm(grad_pre_t_views, transposed_views(input_for_wgrad, t_bounds),
                             TensorBatch.stack_of(grad_fc1_weight), g2_scale_invs, x_scale_invs)
        if handle is not None:
            handle.wait()
        return grad_input, grad_fc1_weight, grad_fc2_weight, None, None, None, None, None, None, None


class GroupedMlp(Fp8GroupedModuleBase):
    """E expert MLPs ``in_features -> out_features -> in_features`` with tanh-GELU, no biases.

    ``forward(input[tokens, in_features], group_sizes[E], has_tp=False, tp_group=None, is_first_microbatch=None)``;
    ``reference_layout`` and ``is_first_microbatch`` as for GroupedLinear (None: cast the weights every pass; True /
    False: cast into / reuse the module's fp8 weight buffers).
    ``fused_dgelu=True`` (default layout only): the fc2 data-gradient GEMM applies the GELU's derivative and the cast to
    fp8 in its epilogue, from the fp32 accumulators (one rounding, where the separate pass rounds to bf16 first), and
    the pass over ``[tokens, out_features]`` that the reference runs behind that GEMM (grouped_mlp.py:243-287) is gone.
    Off by default: with one wavefront per SIMD the epilogue's arithmetic costs the GEMM more than the pass it
    replaces.
    ``planned_passes=False`` builds the tables of every launch in Python through the per-launch entry points of
    ``backend`` instead of one library call per pass (same tables, same launches, more host time).
    """

    def __init__(self, in_features, out_features, num_groups, dtype, device="cuda",
                 pad_multiple=MODULE_PAD_MULTIPLE, reference_layout=False, fused_dgelu=False, planned_passes=True):
        super().__init__()
        self.fp8_meta["planned_passes"] = planned_passes
        self.fp8_meta["pad_multiple"] = pad_multiple
        self.fp8_meta["reference_layout"] = reference_layout
        self.fp8_meta["fused_dgelu"] = fused_dgelu
        assert dtype == torch.bfloat16, "bfloat16 parameters only"
        self.num_groups = num_groups
        self.fc1_weight = torch.nn.Parameter(
            torch.empty(num_groups, out_features, in_features, dtype=dtype, device=device)
        )
        self.fc2_weight = torch.nn.Parameter(
            torch.empty(num_groups, in_features, out_features, dtype=dtype, device=device)
        )
        b1, b2 = math.sqrt(1.0 / in_features), math.sqrt(1.0 / out_features)
        torch.nn.init.uniform_(self.fc1_weight.data, -b1, b1)
        torch.nn.init.uniform_(self.fc2_weight.data, -b2, b2)
        self._weight_caches.extend([Fp8WeightCache(), Fp8WeightCache()])

    def capture_intermediates(self, store):
        """Keep references to the tensors a pass produces between its kernels in the dict ``store`` (None: stop):
        ``pre_gelu_out`` bf16 and ``gelu_out_fp8`` of the forward pass, ``grad_gelu_out`` bf16 and ``grad_pre_fp8``
        of the backward pass.  For checks that follow the data flow stage by stage; costs nothing when unset."""
        if store is None:
            self.fp8_meta.pop("capture", None)
        else:
            self.fp8_meta["capture"] = store

    def get_fp8_weights_scratchpad(self, is_first_microbatch):
        """``[fc1_weight_fp8, fc1_weight_t_fp8, fc2_weight_fp8, fc2_weight_t_fp8]`` kept across micro-batches, or
        Nones when ``is_first_microbatch`` is None (all the reference supports, grouped_mlp.py:343-345)."""
        if is_first_microbatch is None:
            return [None, None, None, None]
        dtype = to_torch_dtype(get_fp8_te_dtype(self.fp8_meta["recipe"], fprop_tensor=True))
        tw = self.fp8_meta["reference_layout"]
        return list(self._weight_caches[0].buffers(self.fc1_weight, dtype, tw)) + \
            list(self._weight_caches[1].buffers(self.fc2_weight, dtype, tw))

    def cast_weights_ahead(self):
        """As ``GroupedLinear.cast_weights_ahead``: the scaling update and the casts of both weight stacks are enqueued
        now, the next ``forward(input, group_sizes)`` runs the rest."""
        return self._cast_ahead([(self.fc1_weight, _T.kWeightGroup1), (self.fc2_weight, _T.kWeightGroup2)])

    def forward(self, input, group_sizes, has_tp=False, tp_group=None, is_first_microbatch=None):
        ahead = self._take_ahead(is_first_microbatch)
        with (contextlib.nullcontext() if ahead is not None else
              self.prepare_forward(input, is_first_microbatch, self.num_groups * 2)):
            grad = torch.is_grad_enabled()
            args = (input, self.fc1_weight, self.fc2_weight, group_sizes, self.fp8_meta, grad, has_tp, tp_group)
            if ahead is not None:
                args += (ahead, False)
            elif is_first_microbatch is not None:
                args += (tuple(self._weight_caches), bool(is_first_microbatch))
            if grad:
                return _GroupedMlp.apply(*args)
            return _GroupedMlp.forward(None, *args)
