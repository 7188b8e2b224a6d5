"""Token routing around the grouped expert layers: sort by expert, histogram, gather, scatter.

The reference's example MoE layers take these operators from the megablocks package
(``megablocks.ops`` in fp8_gmm/example.py:4,15-32,52,59,88,94,115,119).  megablocks is not part of the
reference tree and no version of it is pinned there; this module provides the operators under the same names,
argument order and meaning, on HIP kernels of this package's library (csrc/router.hip):

    sort(x, end_bit)                                   -> (sorted x, original positions), stable
    histogram(x, num_bins)                             -> entries per value
    inclusive_cumsum(x, dim)
    gather(x, indices, bin_ids, bins, top_k)           -> x[indices // top_k]               (autograd)
    scatter(x, indices, bin_ids, weights, bins, top_k) -> sum_k weights * rows, token order (autograd)

plus ``indices_and_bins`` and ``topk`` of the example itself (example.py:15-32), the former as ONE library call.
Differences, stated where they matter: the weighted sum of ``scatter`` is accumulated in fp32 and rounded to bf16
once (megablocks rounds every weighted row to the output type before adding), and ids outside ``[0, 2**end_bit)``
are clamped into the range instead of being undefined.
"""
import torch

from . import _lib
from .backend import _fail, _stream, _timed

MAX_EXPERTS = 4096  # size of the on-chip expert table of the sort kernels


def _check_ids(x):
    if not x.is_cuda:
        _fail("fp8_gmm_amd: expected GPU tensors (the HIP path has no CPU fallback)")
    if x.dtype != torch.int32 or x.dim() != 1 or not x.is_contiguous():
        _fail("fp8_gmm_amd: expert ids must be a contiguous 1-D int32 tensor")


def route(top_expert, num_experts, want_sort=True, want_inverse=False, want_counts=True):
    """One pass over the expert ids: ``(bin_ids, indices, inverse, tokens_per_expert, bins)``, None where not asked for."""
    _check_ids(top_expert)
    if not 1 <= num_experts <= MAX_EXPERTS:
        _fail(f"fp8_gmm_amd: between 1 and {MAX_EXPERTS} experts are supported, got {num_experts}")
    n, dev = top_expert.numel(), top_expert.device
    L = _lib.load()

    def new(count):
        return torch.empty(count, dtype=torch.int32, device=dev)

    bin_ids = new(n) if want_sort else None
    indices = new(n) if want_sort else None
    inverse = new(n) if want_inverse else None
    counts = new(num_experts) if want_counts else None
    bins = new(num_experts) if want_counts else None
    work = torch.empty(L.fp8gmm_route_workspace_bytes(n, num_experts), dtype=torch.uint8, device=dev)

    def ptr(t):
        return t.data_ptr() if t is not None and t.numel() else None

    with torch.cuda.device(dev):
        rc = L.fp8gmm_route_sort(ptr(top_expert), n, num_experts, ptr(bin_ids), ptr(indices), ptr(inverse),
                                 ptr(counts), ptr(bins), ptr(work), _stream(dev))
    _lib.check(rc)
    return bin_ids, indices, inverse, counts, bins


def sort(x, end_bit=None):
    """Stable ascending sort of non-negative int32 ids below ``2**end_bit`` (all of 0..4095 when None): returns
    ``(sorted ids, positions they came from)`` like ``megablocks.ops.sort``."""
    num = MAX_EXPERTS if end_bit is None else 1 << int(end_bit)
    bin_ids, indices, _, _, _ = route(x, num, want_counts=False)
    return bin_ids, indices


def histogram(x, num_bins):
    """Number of entries of every value in ``[0, num_bins)``, int32 (``megablocks.ops.histogram``)."""
    return route(x, int(num_bins), want_sort=False)[3]


def inclusive_cumsum(x, dim):
    """``megablocks.ops.inclusive_cumsum``: running sum along ``dim`` in the dtype of ``x``."""
    if x.dim() == 0:
        return x.clone()
    return torch.cumsum(x, dim).to(x.dtype)


def indices_and_bins(top_expert, sort_end_bit, n_experts):
    """``(indices, bin_ids, bins, tokens_per_expert)`` as the example's helper of the same name returns them
    (fp8_gmm/example.py:26-32), from one library call instead of three operators."""
    del sort_end_bit  # the counting sort needs the expert count, not a bit count
    top_expert = top_expert.int().contiguous()
    bin_ids, indices, _, tokens_per_expert, bins = route(top_expert, n_experts)
    return indices, bin_ids, bins, tokens_per_expert


MAX_TOP_K = 8


class _TopK(torch.autograd.Function):
    """softmax over the experts + the top_k largest in one launch, and the chain back to the scores in another."""

    @staticmethod
    def forward(ctx, scores, top_k):
        tokens, experts = scores.shape
        probs = torch.empty(tokens, experts, dtype=torch.float32, device=scores.device)
        weights = torch.empty(tokens, top_k, dtype=torch.float32, device=scores.device)
        selected = torch.empty(tokens, top_k, dtype=torch.int64, device=scores.device)
        _lib.check(_lib.load().fp8gmm_route_topk(scores.data_ptr(), int(scores.dtype == torch.bfloat16), tokens,
                                                experts, top_k, probs.data_ptr(), weights.data_ptr(),
                                                selected.data_ptr(), _stream(scores.device)))
        ctx.save_for_backward(probs, selected)
        ctx.dtype = scores.dtype
        ctx.mark_non_differentiable(selected)
        return weights, selected

    @staticmethod
    def backward(ctx, grad_weights, _):
        probs, selected = ctx.saved_tensors
        tokens, experts = probs.shape
        grad_weights = grad_weights.contiguous().float()
        grad = torch.empty(tokens, experts, dtype=ctx.dtype, device=probs.device)
        _lib.check(_lib.load().fp8gmm_route_topk_backward(probs.data_ptr(), selected.data_ptr(), grad_weights.data_ptr(),
                                                         tokens, experts, selected.shape[1], grad.data_ptr(),
                                                         int(ctx.dtype == torch.bfloat16), _stream(probs.device)))
        return grad, None


def topk(scores, top_k, moe_renorm=False):
    """Softmax over experts in fp32, then the ``top_k`` largest (fp8_gmm/example.py:15-23): weights fp32
    ``[tokens, top_k]`` and expert ids int64.  One kernel for 2-D bf16 / fp32 scores on the GPU with ``top_k`` up to 8
    (equal scores: the lower expert first); torch's operators otherwise."""
    if scores.is_cuda and scores.dim() == 2 and scores.dtype in (torch.bfloat16, torch.float32) \
            and 1 <= top_k <= min(MAX_TOP_K, scores.shape[1]):
        with torch.cuda.device(scores.device):
            multiplier, selected_experts = _TopK.apply(scores.contiguous(), top_k)
    else:
        weights = torch.nn.functional.softmax(scores, dim=1, dtype=torch.float)
        multiplier, selected_experts = torch.topk(weights, top_k)
    if moe_renorm:
        multiplier = multiplier / multiplier.sum(dim=-1, keepdim=True)
    return multiplier, selected_experts


def _check_rows(x, what):
    if not x.is_cuda:
        _fail("fp8_gmm_amd: expected GPU tensors (the HIP path has no CPU fallback)")
    if x.dtype != torch.bfloat16 or x.dim() != 2:
        _fail(f"fp8_gmm_amd: {what} must be a 2-D bfloat16 tensor")


def _check_indices(indices, rows):
    _check_ids(indices)
    if indices.numel() != rows:
        _fail(f"fp8_gmm_amd: expected {rows} indices, got {indices.numel()}")


def _invert(indices):
    inverse = torch.empty_like(indices)
    dev = indices.device
    with torch.cuda.device(dev):
        rc = _lib.load().fp8gmm_route_invert(indices.data_ptr(), indices.numel(), inverse.data_ptr(), _stream(dev))
    _lib.check(rc)
    return inverse


def _gather_rows(x, indices, weights, top_k):
    """out[i] = weights[indices[i]] * x[indices[i] // top_k]"""
    rows, hidden = x.shape[0] * top_k, x.shape[1]
    out = torch.empty(rows, hidden, dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device), _timed("moe_gather", lambda: 4 * rows * hidden):
        rc = _lib.load().fp8gmm_moe_gather(x.data_ptr(), indices.data_ptr(),
                                           weights.data_ptr() if weights is not None else None, out.data_ptr(),
                                           rows, hidden, top_k, _stream(x.device))
    _lib.check(rc)
    return out


def _scatter_rows(x, inverse, weights, top_k):
    """out[t] = sum_k weights[t * top_k + k] * x[inverse[t * top_k + k]]"""
    tokens, hidden = x.shape[0] // top_k, x.shape[1]
    out = torch.empty(tokens, hidden, dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device), _timed("moe_scatter", lambda: 2 * (x.shape[0] + tokens) * hidden):
        rc = _lib.load().fp8gmm_moe_scatter(x.data_ptr(), inverse.data_ptr(),
                                            weights.data_ptr() if weights is not None else None, out.data_ptr(),
                                            tokens, hidden, top_k, _stream(x.device))
    _lib.check(rc)
    return out


class _Gather(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, indices, top_k):
        ctx.save_for_backward(indices)
        ctx.top_k = top_k
        return _gather_rows(x, indices, None, top_k)

    @staticmethod
    def backward(ctx, grad):
        (indices,) = ctx.saved_tensors
        return _scatter_rows(grad.contiguous(), _invert(indices), None, ctx.top_k), None, None


class _Scatter(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, indices, weights, top_k):
        ctx.save_for_backward(x if weights is not None and ctx.needs_input_grad[2] else None, indices, weights)
        ctx.top_k = top_k
        return _scatter_rows(x, _invert(indices), weights, top_k)

    @staticmethod
    def backward(ctx, grad):
        x, indices, weights = ctx.saved_tensors
        grad = grad.contiguous()
        if weights is not None and ctx.needs_input_grad[0] and ctx.needs_input_grad[2]:
            # both gradients: one pass that reads every gradient row once
            rows, hidden = x.shape
            grad_x = torch.empty(rows, hidden, dtype=grad.dtype, device=grad.device)
            grad_w = torch.zeros_like(weights)
            with torch.cuda.device(grad.device), _timed("moe_scatter_backward", lambda: 6 * rows * hidden):
                rc = _lib.load().fp8gmm_moe_scatter_backward(x.data_ptr(), grad.data_ptr(), indices.data_ptr(),
                                                             weights.data_ptr(), grad_x.data_ptr(), grad_w.data_ptr(),
                                                             rows, hidden, ctx.top_k, _stream(grad.device))
            _lib.check(rc)
            return grad_x, None, grad_w, None
        grad_x = _gather_rows(grad, indices, weights, ctx.top_k) if ctx.needs_input_grad[0] else None
        grad_w = None
        if weights is not None and ctx.needs_input_grad[2]:
            grad_w = torch.zeros_like(weights)
            with torch.cuda.device(grad.device):
                rc = _lib.load().fp8gmm_moe_scatter_wgrad(x.data_ptr(), grad.data_ptr(), indices.data_ptr(),
                                                          grad_w.data_ptr(), x.shape[0], x.shape[1], ctx.top_k,
                                                          _stream(grad.device))
            _lib.check(rc)
        return grad_x, None, grad_w, None


def gather(x, indices, bin_ids, bins, top_k):
    """Rows of ``x[tokens, hidden]`` into expert order: ``out[i] = x[indices[i] // top_k]``, ``[tokens * top_k,
    hidden]`` (``megablocks.ops.gather``; ``bin_ids`` and ``bins`` are accepted for that signature and unused).
    Differentiable in ``x``."""
    del bin_ids, bins
    _check_rows(x, "gather input")
    _check_indices(indices, x.shape[0] * top_k)
    return _Gather.apply(x.contiguous(), indices, int(top_k))


def scatter(x, indices, bin_ids, weights, bins, top_k):
    """Rows in expert order back to token order, weighted: ``out[t] = sum_k weights[t * top_k + k] * x[pos(t, k)]``
    with ``pos`` the inverse of ``indices``; ``weights`` ``[tokens * top_k]`` in (token, choice) order, or None for
    a plain sum (``megablocks.ops.scatter``).  Differentiable in ``x`` and ``weights``."""
    del bin_ids, bins
    _check_rows(x, "scatter input")
    top_k = int(top_k)
    if x.shape[0] % top_k:
        _fail("fp8_gmm_amd: scatter needs tokens * top_k rows")
    _check_indices(indices, x.shape[0])
    if weights is not None:
        if weights.numel() != x.shape[0]:
            _fail(f"fp8_gmm_amd: expected {x.shape[0]} scatter weights, got {weights.numel()}")
        weights = weights.reshape(-1).float().contiguous()  # differentiable; a no-op for the example's fp32 weights
    return _Scatter.apply(x.contiguous(), indices, weights, top_k)
