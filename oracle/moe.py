"""CPU oracle of the token-routing operators around the expert layers.  TEST INFRASTRUCTURE ONLY.

The reference's example layers take these operators from megablocks (``megablocks.ops`` in
fp8_gmm/example.py:4,15-32,52,59,88,94,115,119), a dependency that is neither vendored in the reference tree nor
pinned to a version there.  What is restated here is the published meaning of the operators, on plain torch /
numpy CPU arithmetic:

    topk               softmax over the experts in fp32 + the top_k largest (the example's own function, torch ops)
    sort(x)            stable ascending sort: (sorted ids, original positions)
    histogram, inclusive_cumsum
    gather             out[i] = x[indices[i] // top_k]
    scatter            out[t] = bf16( sum_{k ascending} fp32(w[t*top_k+k] * x[pos(t,k)]) ),  pos = inverse of indices
    gather_backward    = scatter without weights;  scatter_backward = weighted gather + per-row dot products

Parity status: sort / histogram / cumsum / gather are integer and copy operations fixed by their definition
(pinned in the tests by brute force on small inputs).  scatter's rounding (fp32 accumulation, one rounding to bf16)
is this build's own rule - megablocks rounds each weighted row to the output type before adding - so scatter is
"parity unpinned" against megablocks itself and pinned against its definition only.
"""
import numpy as np
import torch


def sort(x):
    x = np.asarray(x, dtype=np.int64)
    order = np.argsort(x, kind="stable")
    return x[order].astype(np.int32), order.astype(np.int32)


def histogram(x, num_bins):
    return np.bincount(np.asarray(x, dtype=np.int64), minlength=num_bins)[:num_bins].astype(np.int32)


def inclusive_cumsum(x):
    return np.cumsum(np.asarray(x, dtype=np.int64)).astype(np.int32)


def indices_and_bins(top_expert, n_experts):
    """(indices, bin_ids, bins, tokens_per_expert) - fp8_gmm/example.py:26-32"""
    bin_ids, indices = sort(top_expert)
    tokens_per_expert = histogram(top_expert, n_experts)
    return indices, bin_ids, inclusive_cumsum(tokens_per_expert), tokens_per_expert


def topk(scores, top_k):
    """(weights fp32 [tokens, top_k], expert ids int64) - fp8_gmm/example.py:15-23 without moe_renorm: softmax over
    the experts in fp32, then the top_k largest.  The choice is made on the scores (softmax is monotone), the lower
    expert first on equal scores - torch.topk leaves the order of equal elements open."""
    z = np.asarray(scores, dtype=np.float32)
    ex = np.exp(z - z.max(axis=1, keepdims=True), dtype=np.float32)
    p = ex / ex.sum(axis=1, keepdims=True, dtype=np.float32)
    order = np.argsort(-z, axis=1, kind="stable")[:, :top_k]
    return np.take_along_axis(p, order, axis=1), order.astype(np.int64)


def topk_backward(scores, selected, grad_weights):
    """Gradient of topk's weights with respect to the scores, in float64."""
    z = np.asarray(scores, dtype=np.float64)
    ex = np.exp(z - z.max(axis=1, keepdims=True))
    p = ex / ex.sum(axis=1, keepdims=True)
    g = np.zeros_like(p)
    np.put_along_axis(g, np.asarray(selected), np.asarray(grad_weights, dtype=np.float64), axis=1)
    return p * (g - (g * p).sum(axis=1, keepdims=True))


def invert(indices):
    indices = np.asarray(indices, dtype=np.int64)
    inverse = np.empty_like(indices)
    inverse[indices] = np.arange(len(indices))
    return inverse


def gather(x, indices, top_k, weights=None):
    """x bf16 [tokens, hidden] -> bf16 [tokens * top_k, hidden]; with weights: bf16(w[indices[i]] * row)."""
    idx = torch.as_tensor(np.asarray(indices, dtype=np.int64))
    rows = x[idx // top_k]
    if weights is None:
        return rows.clone()
    w = weights.float().reshape(-1)[idx]
    return (rows.float() * w[:, None]).to(torch.bfloat16)


def scatter(x, indices, top_k, weights=None):
    """x bf16 [tokens * top_k, hidden] in sorted order -> bf16 [tokens, hidden]."""
    inv = torch.as_tensor(invert(indices)).reshape(-1, top_k)
    tokens = inv.shape[0]
    acc = torch.zeros(tokens, x.shape[1], dtype=torch.float32)
    w = weights.float().reshape(tokens, top_k) if weights is not None else None
    for k in range(top_k):
        rows = x[inv[:, k]].float()
        acc = acc + (rows * w[:, k: k + 1] if w is not None else rows)   # product rounded to fp32, then added
    return acc.to(torch.bfloat16)


def gather_backward(grad, indices, top_k):
    return scatter(grad, indices, top_k, None)


def scatter_backward(grad, x, indices, top_k, weights):
    """(grad_x, grad_weights) of scatter: grad_x[i] = bf16(w[indices[i]] * grad[indices[i] // top_k]),
    grad_w[indices[i]] = <x[i], grad[indices[i] // top_k]> in fp32 (fp64 accumulation here)."""
    idx = torch.as_tensor(np.asarray(indices, dtype=np.int64))
    grad_x = gather(grad, indices, top_k, weights)
    grad_w = None
    if weights is not None:
        dots = (x.double() * grad[idx // top_k].double()).sum(dim=1)
        grad_w = torch.zeros(x.shape[0], dtype=torch.float32)
        grad_w[idx] = dots.float()
    return grad_x, grad_w
