"""Pins of the routing oracle (oracle/moe.py) against what fixes each operator independently of its formula:
brute force in plain Python on small inputs, permutation / conservation properties, and torch autograd of an
index-op formulation in float64 for the two backward rules."""
import numpy as np
import torch

from oracle import moe


def _ids(n, e, seed):
    return np.random.default_rng(seed).integers(0, e, size=n)


def test_sort_is_the_stable_sort():
    for n, e, seed in [(1, 1, 0), (8, 4, 1), (1000, 7, 2), (5000, 64, 3), (64, 2, 4)]:
        x = _ids(n, e, seed)
        want = sorted(range(n), key=lambda i: x[i])          # Python's sort is stable
        bin_ids, indices = moe.sort(x)
        assert indices.tolist() == want
        assert bin_ids.tolist() == [int(x[i]) for i in want]
        counts = moe.histogram(x, e)
        assert counts.tolist() == [int((x == k).sum()) for k in range(e)]
        bins = moe.inclusive_cumsum(counts)
        # bins[e] is where expert e ends in the sorted list
        for k in range(e):
            assert (bin_ids[: bins[k]] <= k).all() and (bin_ids[bins[k]:] > k).all()
        inv = moe.invert(indices)
        assert (np.asarray(indices)[inv] == np.arange(n)).all()


def test_gather_and_scatter_by_brute_force():
    rng = np.random.default_rng(5)
    tokens, top_k, hidden, e = 13, 3, 5, 4
    x = torch.tensor(rng.standard_normal((tokens, hidden)), dtype=torch.bfloat16)
    experts = _ids(tokens * top_k, e, 6)
    _, indices = moe.sort(experts)
    w = torch.tensor(rng.random(tokens * top_k), dtype=torch.float32)
    g = moe.gather(x, indices, top_k)
    for i in range(tokens * top_k):
        assert torch.equal(g[i], x[indices[i] // top_k])
    y = torch.tensor(rng.standard_normal((tokens * top_k, hidden)), dtype=torch.bfloat16)
    out = moe.scatter(y, indices, top_k, w)
    where = {int(indices[i]): i for i in range(tokens * top_k)}   # flat (token, choice) -> sorted row
    for t in range(tokens):
        for c in range(hidden):
            acc = np.float32(0)
            for k in range(top_k):
                acc = np.float32(acc + np.float32(np.float32(y[where[t * top_k + k], c].item()) * np.float32(w[t * top_k + k].item())))
            assert out[t, c].item() == torch.tensor(float(acc)).to(torch.bfloat16).item()
    # unweighted scatter of a gather gives top_k * x when the sum is exact (small integers)
    xi = torch.tensor(rng.integers(-8, 9, size=(tokens, hidden)), dtype=torch.bfloat16)
    assert torch.equal(moe.scatter(moe.gather(xi, indices, top_k), indices, top_k).float(), xi.float() * top_k)


def test_backward_rules_against_autograd():
    rng = np.random.default_rng(7)
    tokens, top_k, hidden = 9, 2, 6
    experts = _ids(tokens * top_k, 5, 8)
    _, indices = moe.sort(experts)
    idx = torch.as_tensor(indices.astype(np.int64))
    # values on a coarse grid so that bf16 / fp32 products and sums are exact and the comparison can be strict
    y = torch.tensor(rng.integers(-4, 5, size=(tokens * top_k, hidden)) / 4.0, dtype=torch.float64, requires_grad=True)
    w = torch.tensor(rng.integers(1, 5, size=tokens * top_k) / 4.0, dtype=torch.float64, requires_grad=True)
    grad = torch.tensor(rng.integers(-4, 5, size=(tokens, hidden)) / 2.0, dtype=torch.float64)
    out = torch.zeros(tokens, hidden, dtype=torch.float64).index_add(0, idx // top_k, y * w[idx][:, None])
    assert torch.equal(out.detach(), moe.scatter(y.detach().to(torch.bfloat16), indices, top_k, w.detach().float()).double())
    out.backward(grad)
    gx, gw = moe.scatter_backward(grad.to(torch.bfloat16), y.detach().to(torch.bfloat16), indices, top_k,
                                  w.detach().float())
    assert torch.equal(gx.double(), y.grad) and torch.equal(gw.double(), w.grad)
    x = torch.tensor(rng.integers(-4, 5, size=(tokens, hidden)) / 4.0, dtype=torch.float64, requires_grad=True)
    x[idx // top_k].backward(y.detach())
    assert torch.equal(moe.gather_backward(y.detach().to(torch.bfloat16), indices, top_k).double(), x.grad)


def test_topk_is_softmax_then_the_largest():
    """The oracle's topk against the reference's own formulation in torch operators (fp8_gmm/example.py:15-23) on
    scores without ties, its tie rule on a hand-made row, and its gradient against autograd."""
    rng = np.random.default_rng(5)
    z = rng.standard_normal((300, 16)).astype(np.float32)
    w, sel = moe.topk(z, 2)
    tw, tsel = torch.topk(torch.softmax(torch.from_numpy(z), dim=1, dtype=torch.float), 2)
    assert (sel == tsel.numpy()).all()
    np.testing.assert_allclose(w, tw.numpy(), rtol=2e-6, atol=0)
    tie = np.array([[1.0, 3.0, 3.0, 0.5, 3.0]], dtype=np.float32)
    w, sel = moe.topk(tie, 3)
    assert sel.tolist() == [[1, 2, 4]] and w[0, 0] == w[0, 1] == w[0, 2]
    zt = torch.from_numpy(z).double().requires_grad_()
    gw = rng.standard_normal((300, 2))
    (torch.softmax(zt, dim=1).gather(1, torch.from_numpy(sel_of(z))) * torch.from_numpy(gw)).sum().backward()
    np.testing.assert_allclose(moe.topk_backward(z, sel_of(z), gw), zt.grad.numpy(), rtol=1e-9, atol=1e-12)


def sel_of(z):
    return moe.topk(z, 2)[1]
