"""fp8gmm_grouped_gemm_static: the grouped GEMM for callers that cannot allocate, whose tail-balancing scratch is
an array inside the library's device image.  Called through the C ABI and compared bit for bit with
fp8gmm_grouped_gemm on a caller-provided workspace, on two calls in a row, the second with a smaller input (the
array keeps the first call's partial sums: stale contents must not leak into the second result)."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

E4M3 = torch.float8_e4m3fn


def _launch(L, _lib, dev, a, b, sizes, static):
    """One grouped GEMM c[rows of expert i] = a[rows] . b[i]^T through the C ABI; returns (c, plan)."""
    e, (tokens, k), n = len(sizes), a.shape, b.shape[1]
    c = torch.full((tokens, n), float("nan"), dtype=torch.bfloat16, device=dev)
    starts = np.concatenate([[0], np.cumsum(sizes)])[:-1].astype(np.uint64)
    table = np.zeros(e, dtype=_lib.GEMM_PROBLEM)
    table["a"] = a.data_ptr() + starts * np.uint64(k)
    table["b"] = b.data_ptr() + np.arange(e, dtype=np.uint64) * np.uint64(n * k)
    table["c"] = c.data_ptr() + starts * np.uint64(2 * n)
    table["m"], table["n"], table["k"] = sizes, n, k
    table["lda"] = table["ldb"] = k
    table["ldc"] = n
    grid = _lib.gemm_grid(_lib.init(dev.index))
    plan, items, fixups = _lib.plan_grouped_gemm_launch(table, 0, grid, True)
    blob = np.concatenate([table.view(np.uint8).reshape(-1), np.zeros((-table.nbytes) % 128, dtype=np.uint8),
                           items.view(np.uint8).reshape(-1), fixups.view(np.uint8).reshape(-1)])
    off_items = (table.nbytes + 127) // 128 * 128
    dev_blob = torch.from_numpy(blob).to(dev)
    p = dev_blob.data_ptr()
    fix = p + off_items + items.nbytes if plan.n_fixups else None
    stream = torch.cuda.current_stream(dev).cuda_stream
    if static:
        rc = L.fp8gmm_grouped_gemm_static(p, e, p + off_items, fix, plan, 0, 0, 2, 0, stream)
    else:
        ws = torch.empty(max(1, plan.n_slots) * _lib.GEMM_SLOT_BYTES, dtype=torch.uint8, device=dev)
        rc = L.fp8gmm_grouped_gemm(p, e, p + off_items, fix, plan, 0, 0, 2, 0, ws.data_ptr(), ws.numel(), stream)
    _lib.check(rc)
    torch.cuda.synchronize()
    return c, plan


def test_static_scratch_entry_point_equals_the_workspace_entry_point(dev):
    from fp8_gmm_amd import _lib

    L = _lib.load()
    g = torch.Generator(device=dev).manual_seed(2024)
    # few tiles and a long K: both launches share tiles along K, i.e. both use the scratch; the second is smaller
    cases = [([300, 0, 513, 90], 512, 7168), ([256], 256, 4096)]
    for sizes, n, k in cases:
        a = torch.randn(sum(sizes), k, generator=g, device=dev).to(E4M3)
        b = torch.randn(len(sizes), n, k, generator=g, device=dev).to(E4M3)
        want, plan = _launch(L, _lib, dev, a, b, sizes, static=False)
        assert plan.n_fixups > 0 and 0 < plan.n_slots <= _lib.GEMM_STATIC_SLOTS, "the case is meant to use the scratch"
        got, _ = _launch(L, _lib, dev, a, b, sizes, static=True)
        assert torch.isfinite(want.float()).all()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), f"sizes {sizes} n {n} k {k}"
        ref = torch.cat([a[s: s + m].float() @ b[i].float().t() for i, (s, m) in enumerate(
            zip(np.concatenate([[0], np.cumsum(sizes)])[:-1].tolist(), sizes))])
        assert (got.float() - ref).abs().max() <= 1e-2 * ref.abs().max()


def test_static_scratch_entry_point_refuses_what_does_not_fit(dev):
    from fp8_gmm_amd import _lib

    L = _lib.load()
    too_many = _lib.GemmPlan(grid=256, rounds=2, total_tiles=1, n_fixups=1, n_slots=_lib.GEMM_STATIC_SLOTS + 1)
    fake = 0x10000  # never dereferenced: the size check comes first
    assert L.fp8gmm_grouped_gemm_static(fake, 1, fake, fake, too_many, 0, 0, 2, 0, None) == -9
    assert L.fp8gmm_grouped_gemm_static(fake, 1, fake, fake, None, 0, 0, 2, 0, None) == -1
