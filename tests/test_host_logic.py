"""Host-side logic that needs no GPU: token-split bookkeeping, scaling-metadata slot arithmetic,
the delayed-scaling update rule and the recipe / autocast plumbing.

Expected values are worked out from the reference's formulas (fp8_gmm/utils.py:48-62 and :98-103),
not by calling the code under test twice.
"""
import pytest
import torch

from fp8_gmm_amd import fp8
from fp8_gmm_amd.utils import (
    DType,
    Fp8MetaWrapper,
    Fp8TensorType,
    MetaTensorType,
    cumsum_group_sizes,
    to_tex_dtype,
    to_torch_dtype,
)
from oracle import modules as orc


def test_cumsum_group_sizes_config1():
    # worked by hand: [137, 401, 59, 403] padded to multiples of 16 -> [144, 416, 64, 416]
    e, padded, cums, pcums = cumsum_group_sizes([137, 401, 59, 403], need_padding=True)
    assert (e, padded) == (4, True)
    assert cums == [0, 137, 538, 597, 1000]
    assert pcums == [0, 144, 560, 624, 1040]


def test_cumsum_group_sizes_variants():
    assert cumsum_group_sizes([16, 32, 16], need_padding=True) == (3, False, [0, 16, 48, 64], [0, 16, 48, 64])
    assert cumsum_group_sizes([16, 32, 16]) == (3, False, [0, 16, 48, 64], None)
    assert cumsum_group_sizes([5, 0, 17], need_padding=True) == (3, True, [0, 5, 5, 22], [0, 16, 16, 48])
    assert cumsum_group_sizes([5, 0, 129], True, pad_multiple=128) == (3, True, [0, 5, 5, 134], [0, 128, 128, 384])
    assert cumsum_group_sizes(torch.tensor([3, 4]).tolist(), True)[3] == [0, 16, 32]
    assert cumsum_group_sizes([], True) == (0, False, [0], [0])


def test_dtype_maps():
    assert to_tex_dtype(torch.float8_e4m3fn) == DType.kFloat8E4M3
    assert to_tex_dtype(torch.float8_e5m2) == DType.kFloat8E5M2
    assert to_tex_dtype(torch.bfloat16) == DType.kBFloat16
    for d in DType:
        assert to_tex_dtype(to_torch_dtype(d)) == d
    with pytest.raises(ValueError):
        to_tex_dtype(torch.float16)


class _Meta:
    def __init__(self, slots, hist=2):
        self.scale = torch.arange(slots, dtype=torch.float32) + 1000
        self.scale_inv = torch.arange(slots, dtype=torch.float32) + 2000
        self.amax_history = (torch.arange(hist * slots, dtype=torch.float32) + 3000).reshape(hist, slots)


@pytest.mark.parametrize("e", [1, 4])
def test_meta_wrapper_slot_arithmetic(e):
    """slot = (group * E + i) * stride + weight, stride 3 forward / 2 backward (utils.py:98-103)."""
    fwd, bwd = _Meta(3 * 2 * e), _Meta(2 * 2 * e)
    w = Fp8MetaWrapper(e, {"scaling_fwd": fwd, "scaling_bwd": bwd})
    w.set_forward_scale_inv_cloned()
    expect = {
        Fp8TensorType.kInputGroup1: ("fwd", [3 * i for i in range(e)]),
        Fp8TensorType.kInputGroup2: ("fwd", [3 * (e + i) for i in range(e)]),
        Fp8TensorType.kWeightGroup1: ("fwd", [3 * i + 1 for i in range(e)]),
        Fp8TensorType.kWeightGroup2: ("fwd", [3 * (e + i) + 1 for i in range(e)]),
        Fp8TensorType.kGradOutputGroup1: ("bwd", [2 * i for i in range(e)]),
        Fp8TensorType.kGradOutputGroup2: ("bwd", [2 * (e + i) for i in range(e)]),
        Fp8TensorType.kForwardInputGroup1: ("clone", [3 * i for i in range(e)]),
        Fp8TensorType.kForwardInputGroup2: ("clone", [3 * (e + i) for i in range(e)]),
        Fp8TensorType.kForwardWeightGroup1: ("clone", [3 * i + 1 for i in range(e)]),
        Fp8TensorType.kForwardWeightGroup2: ("clone", [3 * (e + i) + 1 for i in range(e)]),
    }
    for ttype, (which, slots) in expect.items():
        if which == "clone":
            got = w.get_meta_tensors(ttype, MetaTensorType.kScaleInv)
            assert [t.item() for t in got] == [2000.0 + s for s in slots]
            with pytest.raises(AssertionError):
                w.get_meta_tensors(ttype, MetaTensorType.kScale)
            continue
        meta = fwd if which == "fwd" else bwd
        assert [t.item() for t in w.get_meta_tensors(ttype, MetaTensorType.kScale)] == [1000.0 + s for s in slots]
        assert [t.item() for t in w.get_meta_tensors(ttype, MetaTensorType.kScaleInv)] == [2000.0 + s for s in slots]
        assert [t.item() for t in w.get_meta_tensors(ttype, MetaTensorType.kAmax)] == [3000.0 + s for s in slots]
        # views, not copies: the kernels write amax in place; and the pointer form addresses the same slots
        views = w.get_meta_tensors(ttype, MetaTensorType.kAmax)
        ptrs = w.get_meta_pointers(ttype, MetaTensorType.kAmax)
        assert [v.data_ptr() for v in views] == [int(p) for p in ptrs]
        assert views[0].data_ptr() == meta.amax_history.data_ptr() + 4 * slots[0]


def test_forward_scale_inv_clone_is_a_snapshot():
    fwd, bwd = _Meta(3), _Meta(2)
    w = Fp8MetaWrapper(1, {"scaling_fwd": fwd, "scaling_bwd": bwd})
    w.set_forward_scale_inv_cloned()
    fwd.scale_inv.fill_(-1.0)
    assert w.get_meta_tensors(Fp8TensorType.kForwardWeightGroup1, MetaTensorType.kScaleInv)[0].item() == 2001.0
    assert w.get_meta_tensors(Fp8TensorType.kWeightGroup1, MetaTensorType.kScaleInv)[0].item() == -1.0


def test_delayed_scaling_update_rule():
    """amax = max over history; scale = fp8_max / amax / 2^margin where amax is finite and > 0;
    history rolls by one row and row 0 is cleared."""
    meta = fp8.Fp8MetaTensors(4, 3, torch.device("cpu"))
    meta.amax_history.copy_(torch.tensor([[2.0, 0.0, float("inf"), 7.0], [4.0, 0.0, 1.0, 1.0], [1.0, 0.0, 1.0, 28.0]]))
    meta.scale.copy_(torch.tensor([9.0, 9.0, 9.0, 9.0]))
    fp8.amax_and_scale_update(meta, 448.0, fp8.DelayedScaling(margin=1, amax_history_len=3))
    assert meta.scale.tolist() == [448.0 / 4.0 / 2.0, 9.0, 9.0, 448.0 / 28.0 / 2.0]
    assert torch.equal(meta.scale_inv, 1.0 / meta.scale)
    assert meta.amax_history.tolist() == [[0.0, 0.0, 0.0, 0.0], [1.0, 0.0, 1.0, 28.0], [2.0, 0.0, float("inf"), 7.0]]
    # most_recent uses row 0 only
    meta2 = fp8.Fp8MetaTensors(1, 2, torch.device("cpu"))
    meta2.amax_history.copy_(torch.tensor([[2.0], [100.0]]))
    fp8.amax_and_scale_update(meta2, 448.0, fp8.DelayedScaling(amax_history_len=2, amax_compute_algo="most_recent"))
    assert meta2.scale.item() == 224.0
    # history of length 1: no roll, just cleared
    meta3 = fp8.Fp8MetaTensors(1, 1, torch.device("cpu"))
    meta3.amax_history.fill_(8.0)
    fp8.amax_and_scale_update(meta3, 57344.0, fp8.DelayedScaling(amax_history_len=1))
    assert meta3.scale.item() == 7168.0 and meta3.amax_history.item() == 0.0


def test_update_rule_equals_the_oracle_restatement():
    """The oracle's Meta.update is pinned by hand-worked numbers (tests/test_oracle_pins.py::test_meta_update_*);
    the product's rule is then held against the oracle over several updates, for every option."""
    g = torch.Generator().manual_seed(3)
    hist = torch.rand(5, 12, generator=g) * torch.tensor([0.0, 1.0, 10.0] * 4)
    hist[2, 5] = float("inf")
    hist[1, 7] = float("nan")
    for algo, margin, keep in (("max", 0, None), ("most_recent", 0, None), ("max", 2, None), ("max", 0, (3, 1))):
        want = orc.Meta(12, 5)
        want.amax_history = hist.clone()
        got = fp8.Fp8MetaTensors(12, 5, torch.device("cpu"))
        got.amax_history.copy_(hist)
        recipe = fp8.DelayedScaling(amax_history_len=5, amax_compute_algo=algo, margin=margin)
        kept = [s for s in range(12) if keep and s % keep[0] == keep[1]]
        for _ in range(7):
            want.update(448.0, margin=margin, algo=algo, keep_scale_inv=kept)
            fp8.amax_and_scale_update(got, 448.0, recipe, keep_scale_inv=keep)
            assert torch.equal(got.scale, want.scale) and torch.equal(got.scale_inv, want.scale_inv), (algo, margin)
            assert torch.equal(got.amax_history.nan_to_num(nan=-1.0), want.amax_history.nan_to_num(nan=-1.0))
            want.amax_history[0] += 1.5
            got.amax_history[0] += 1.5


def test_recipe_and_autocast():
    r = fp8.DelayedScaling()
    assert (r.margin, r.interval, r.fp8_format, r.amax_compute_algo) == (0, 1, fp8.Format.HYBRID, "max")
    assert fp8.get_fp8_te_dtype(r, True) == DType.kFloat8E4M3
    assert fp8.get_fp8_te_dtype(r, False) == DType.kFloat8E5M2
    assert fp8.get_fp8_te_dtype(fp8.DelayedScaling(fp8_format=fp8.Format.E4M3), False) == DType.kFloat8E4M3
    assert fp8.current_recipe() is None
    with fp8.fp8_autocast(enabled=True, fp8_recipe=r):
        assert fp8.current_recipe() is r
        with fp8.fp8_autocast(enabled=False):
            assert fp8.current_recipe() is None
        assert fp8.current_recipe() is r
    assert fp8.current_recipe() is None
    with pytest.raises(ValueError):
        fp8.DelayedScaling(amax_compute_algo="median")
    assert fp8.recipe.DelayedScaling is fp8.DelayedScaling and fp8.recipe.Format is fp8.Format


def test_prepare_forward_allocates_three_and_two_slots_per_gemm():
    m = fp8.Fp8GroupedModuleBase()
    x = torch.zeros(4, 8)
    with fp8.fp8_autocast(fp8_recipe=fp8.DelayedScaling(amax_history_len=7)):
        with m.prepare_forward(x, None, num_gemms=6):
            pass
    assert m.fp8_meta["scaling_fwd"].scale.shape == (18,)
    assert m.fp8_meta["scaling_bwd"].scale.shape == (12,)
    assert m.fp8_meta["scaling_fwd"].amax_history.shape == (7, 18)
    assert m.fp8_meta["scaling_fwd"].scale.eq(1).all() and m.fp8_meta["scaling_bwd"].scale_inv.eq(1).all()
    # scaling state round-trips through extra_state
    m.fp8_meta["scaling_fwd"].scale.fill_(3.0)
    state = m.get_extra_state()
    m2 = fp8.Fp8GroupedModuleBase()
    m2.set_extra_state(state)
    with fp8.fp8_autocast(fp8_recipe=fp8.DelayedScaling(amax_history_len=7)):
        with m2.prepare_forward(x, None, num_gemms=6):
            pass
    assert m2.fp8_meta["scaling_fwd"].scale.eq(3).all()


def test_reusing_cached_weights_keeps_their_scale_inv():
    """is_first_microbatch=False: the update still moves every scale, but the weights' scale_inv (slot 1 of
    each GEMM's three forward slots) stays what the cached fp8 weights were cast with; True / None update all."""
    m = fp8.Fp8GroupedModuleBase()
    x = torch.zeros(4, 8)
    rec = fp8.DelayedScaling(amax_history_len=1)
    weight_slots = torch.tensor([1, 4])
    other_slots = torch.tensor([0, 2, 3, 5])

    def step(first, amax):
        with fp8.fp8_autocast(fp8_recipe=rec), m.prepare_forward(x, first, num_gemms=2):
            pass
        m.fp8_meta["scaling_fwd"].amax_history[0] = amax   # what the kernels of the pass would record
        m.fp8_meta["scaling_bwd"].amax_history[0] = 1.0

    step(True, 2.0)                       # first pass: no update yet, scales 1
    step(False, 4.0)                      # update from amax 2: scale 224, weights keep scale_inv 1
    fwd = m.fp8_meta["scaling_fwd"]
    assert fwd.scale.eq(224.0).all()
    assert fwd.scale_inv[weight_slots].eq(1.0).all() and fwd.scale_inv[other_slots].eq(1 / 224.0).all()
    assert m.fp8_meta["scaling_bwd"].scale_inv.eq(1 / 57344.0).all()   # the gradient direction has no weights
    step(True, 8.0)                       # update from amax 4: everything follows
    assert fwd.scale.eq(112.0).all() and fwd.scale_inv.eq(1 / 112.0).all()
    step(None, 8.0)
    assert fwd.scale.eq(56.0).all() and fwd.scale_inv.eq(1 / 56.0).all()


def test_weight_cache_bookkeeping():
    cache = fp8.Fp8WeightCache()
    w = torch.zeros(3, 4, 5, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="is_first_microbatch=False"):
        cache.require(False)
    a, a_t = cache.buffers(w, torch.float8_e4m3fn)
    assert a.shape == (3, 4, 5) and a_t.shape == (3, 5, 4) and a.dtype == a_t.dtype == torch.float8_e4m3fn
    b, b_t = cache.buffers(w, torch.float8_e4m3fn)
    assert b is a and b_t is a_t                        # kept, not reallocated
    cache.valid = True
    cache.require(False)
    with pytest.raises(RuntimeError, match="transposes"):
        cache.require(True)
    c, _ = cache.buffers(torch.zeros(3, 4, 6, dtype=torch.bfloat16), torch.float8_e4m3fn)
    assert c is not a and not cache.valid               # a new shape drops the old contents
    # a module drops its caches when the scaling state is replaced
    m = fp8.Fp8GroupedModuleBase()
    m._weight_caches.append(cache)
    cache.valid = cache.valid_t = True
    with fp8.fp8_autocast(fp8_recipe=fp8.DelayedScaling(amax_history_len=3)), m.prepare_forward(w, None, 2):
        pass
    assert not cache.valid and not cache.valid_t


def test_tensor_batch_describes_the_same_memory_as_views():
    """TensorBatch (array form of "per-expert views") must address exactly what the tensor views address."""
    from fp8_gmm_amd.backend import TensorBatch

    x = torch.zeros(10, 6, dtype=torch.bfloat16)
    bounds = [0, 3, 3, 7, 10]
    b = TensorBatch.rows_of(x, bounds)
    views = [x[bounds[i]: bounds[i + 1]] for i in range(4)]
    assert [int(p) for p in b.ptr] == [x.data_ptr() + bounds[i] * 6 * 2 for i in range(4)]
    assert b.rows.tolist() == [v.shape[0] for v in views] and b.cols.tolist() == [6] * 4 and b.contiguous
    assert [int(p) for p, v in zip(b.ptr, views) if v.numel()] == [v.data_ptr() for v in views if v.numel()]

    w = torch.zeros(3, 4, 5, dtype=torch.float8_e4m3fn)
    s = TensorBatch.stack_of(w)
    assert [int(p) for p in s.ptr] == [v.data_ptr() for v in w.unbind(0)]
    assert (s.rows.tolist(), s.cols.tolist()) == ([4] * 3, [5] * 3)

    flat = torch.zeros(12, 6, dtype=torch.float8_e4m3fn)
    pb = [0, 4, 4, 8, 12]
    t = TensorBatch.transposed_blocks_of(flat, pb)
    for i in range(4):
        rows = pb[i + 1] - pb[i]
        if rows:
            v = flat[pb[i]: pb[i + 1]].view(6, rows)  # the reference's reinterpretation (grouped_linear.py:36-52)
            assert int(t.ptr[i]) == v.data_ptr() and (int(t.rows[i]), int(t.cols[i])) == tuple(v.shape)
    both = b + TensorBatch.rows_of(x, [0, 10])
    assert len(both) == 5 and both.rows.tolist() == [3, 0, 4, 3, 10]
    with pytest.raises(RuntimeError):
        TensorBatch.concat([b, s])  # dtypes differ
    with pytest.raises(RuntimeError):
        TensorBatch.rows_of(x.t(), [0, 1])  # not contiguous
