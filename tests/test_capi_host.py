"""The C-ABI library on a machine without a GPU: it loads, exports every function the header
declares, its structs have the documented layout, and the host-side planners validate and
schedule correctly.  No kernel is launched here.
"""
import ctypes
import os
import re

import numpy as np
import pytest

from fp8_gmm_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "fp8gmm.h")


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fp8gmm_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_function():
    lib = ctypes.CDLL(_lib.LIB_PATH)
    names = _declared_functions()
    assert len(names) >= 13
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in include/fp8gmm.h but not exported"
    assert sorted(_lib.EXPORTS) == names, "the Python binding and the header list different functions"


def test_struct_layouts_match_the_binding():
    lib = _lib.load()
    assert lib.fp8gmm_sizeof_tensor_desc() == _lib.TENSOR_DESC.itemsize == 128  # one cache line per tensor
    assert lib.fp8gmm_sizeof_gemm_problem() == _lib.GEMM_PROBLEM.itemsize == 96
    assert _lib.TENSOR_DESC.fields["rows"][1] == 48 and _lib.TENSOR_DESC.fields["block_begin"][1] == 60
    assert _lib.GEMM_PROBLEM.fields["m"][1] == 64 and _lib.GEMM_PROBLEM.fields["tile_begin"][1] == 88
    assert lib.fp8gmm_sizeof_gemm_item() == _lib.GEMM_ITEM.itemsize == 64 and _lib.GEMM_FIXUP.itemsize == 32
    assert _lib.GEMM_ITEM.fields["lda"][1] == 24 and _lib.GEMM_ITEM.fields["k"][1] == 32
    assert _lib.GEMM_ITEM.fields["prob"][1] == 52
    assert ctypes.sizeof(_lib.GemmPlan) == 32
    assert lib.fp8gmm_version() == _lib.ABI_VERSION == 3
    assert _lib.gemm_tile_shape() == (256, 256)
    assert lib.fp8gmm_status_string(0) == b"ok"
    assert b"NULL" in lib.fp8gmm_status_string(-1)


def _desc(rows, cols, rows_padded=0, inp=0x1000, out=0x2000, out_t=0x3000, in2=0):
    t = np.zeros(len(rows), dtype=_lib.TENSOR_DESC)
    t["rows"], t["cols"], t["rows_padded"] = rows, cols, rows_padded
    t["in"], t["out"], t["out_t"], t["in2"] = inp, out, out_t, in2
    return t


def test_plan_quantize_counts_16384_element_workgroups():
    t = _desc([1, 1, 1, 0, 1], [16384, 16385, 1, 0, 3 * 16384], 0)
    total = _lib.plan_multi_tensor(t, _lib.OP_QUANTIZE)
    assert total == 1 + 2 + 1 + 0 + 3
    assert t["block_begin"].tolist() == [0, 1, 3, 4, 4]


def test_plan_pad_kernels_count_128x128_tiles_of_the_padded_extent():
    t = _desc([137, 128, 0, 1], [256, 129, 64, 3221], [144, 128, 0, 16])
    total = _lib.plan_multi_tensor(t, _lib.OP_PAD_CAST_TRANSPOSE)
    assert t["block_begin"].tolist() == [0, 4, 6, 6]   # ceil(144/128)*ceil(256/128), 1*2, 0, 1*26
    assert total == 4 + 2 + 0 + 26
    # a transposed output narrower than the input is refused, like TORCH_CHECK(trans_cols >= num_rows)
    bad = _desc([17], [8], [16])
    with pytest.raises(_lib.Fp8GmmError):
        _lib.plan_multi_tensor(bad, _lib.OP_PAD_TRANSPOSE)


def test_plan_multi_tensor_error_codes():
    lib = _lib.load()
    total = ctypes.c_int(0)
    t = _desc([4], [4], [16], inp=0)
    assert lib.fp8gmm_plan_multi_tensor(t.ctypes.data, 1, _lib.OP_PAD_TRANSPOSE, ctypes.byref(total)) == -1
    t = _desc([4], [4], [16], out_t=0)
    assert lib.fp8gmm_plan_multi_tensor(t.ctypes.data, 1, _lib.OP_PAD_CAST_TRANSPOSE, ctypes.byref(total)) == -1
    t = _desc([4], [4], [16])  # dgelu needs the second input
    assert lib.fp8gmm_plan_multi_tensor(t.ctypes.data, 1, _lib.OP_PAD_CAST_TRANSPOSE_DGELU, ctypes.byref(total)) == -1
    t = _desc([-1], [4], [16])
    assert lib.fp8gmm_plan_multi_tensor(t.ctypes.data, 1, _lib.OP_QUANTIZE, ctypes.byref(total)) == -2
    t = _desc([4], [4], [16])
    assert lib.fp8gmm_plan_multi_tensor(t.ctypes.data, 1, 99, ctypes.byref(total)) == -6
    assert lib.fp8gmm_plan_multi_tensor(t.ctypes.data, -1, 0, ctypes.byref(total)) == -6
    assert lib.fp8gmm_plan_multi_tensor(t.ctypes.data, 1, 0, None) == -1
    assert lib.fp8gmm_plan_multi_tensor(None, 0, 0, ctypes.byref(total)) == 0 and total.value == 0


def _prob(m, n, k, a=0x10000, b=0x20000, c=0x30000, lda=None, ldb=None, ldc=None):
    t = np.zeros(len(m), dtype=_lib.GEMM_PROBLEM)
    t["m"], t["n"], t["k"] = m, n, k
    t["a"], t["b"], t["c"] = a, b, c
    t["lda"] = k if lda is None else lda
    t["ldb"] = k if ldb is None else ldb
    t["ldc"] = n if ldc is None else ldc
    return t


def test_plan_grouped_gemm_tiles():
    t = _prob([137, 0, 401, 256, 300], [512, 512, 512, 257, 64], [256, 256, 256, 0, 16])
    total = _lib.plan_grouped_gemm(t)
    assert t["tile_begin"].tolist() == [0, 2, 2, 6, 8]   # 1x2, 0, 2x2, 1x2, 2x1 tiles of 256 x 256
    # K = 128 steps of all earlier tiles: 2 tiles x 2 steps, none, 4 x 2, 2 tiles without K count 1 each
    assert t["cost_begin"].tolist() == [0, 4, 4, 12, 14]
    assert total == 10


def test_plan_grouped_gemm_error_codes():
    lib = _lib.load()
    total = ctypes.c_int(0)

    def rc(t):
        return lib.fp8gmm_plan_grouped_gemm(t.ctypes.data, len(t), ctypes.byref(total))

    assert rc(_prob([16], [16], [24])) == -4            # K not a multiple of 16
    assert rc(_prob([16], [16], [32], a=0x10008)) == -4  # operand not 16-byte aligned
    assert rc(_prob([16], [16], [32], lda=40)) == -4     # pitch not a multiple of 16
    assert rc(_prob([16], [16], [32], lda=16)) == -2     # pitch smaller than k
    assert rc(_prob([16], [16], [32], c=0)) == -1
    assert rc(_prob([16], [16], [32], b=0)) == -1
    assert rc(_prob([-1], [16], [32])) == -2
    assert rc(_prob([70000], [16], [65536])) == 0       # a large operand is fine: descriptors span one tile's rows
    assert rc(_prob([16], [16], [1 << 24], lda=1 << 24, ldb=1 << 24)) == -2   # ... 256 rows must stay below 4 GiB
    assert rc(_prob([16], [16], [0], a=0, b=0)) == 0     # k == 0 never reads the operands
    assert rc(_prob([0], [16], [32], a=0, b=0, c=0)) == 0 and total.value == 0


def test_launch_entry_points_validate_before_touching_the_gpu():
    lib = _lib.load()
    assert lib.fp8gmm_multi_quantize(None, 0, 0, 0, None) == 0          # nothing to do
    assert lib.fp8gmm_multi_quantize(None, 1, 1, 7, None) == -3         # unknown format
    assert lib.fp8gmm_multi_quantize(None, 1, 1, 0, None) == -1         # table missing
    assert lib.fp8gmm_multi_pad_cast_transpose(None, -1, 0, 0, None) == -6
    plan = _lib.GemmPlan(grid=8, rounds=2, total_tiles=1)

    def gemm(n, a_fmt, b_fmt, out_kind, epilogue, plan=plan, workspace=None, workspace_bytes=0, items=None):
        return lib.fp8gmm_grouped_gemm(None, n, items, None, plan, a_fmt, b_fmt, out_kind, epilogue, workspace,
                                       workspace_bytes, None)

    assert gemm(1, 1, 1, 2, 0) == -3  # e5m2 x e5m2
    assert gemm(1, 0, 0, 9, 0) == -3  # unknown output kind
    assert gemm(1, 0, 0, 2, 16) == -6  # unknown epilogue flag
    assert gemm(1, 0, 0, 2, 1 | 8) == -6  # GELU and its derivative exclude each other
    assert gemm(1, 0, 0, 2, 0) == -1  # tables missing
    assert gemm(0, 0, 0, 2, 0) == 0   # nothing to do
    assert gemm(1, 0, 0, 2, 0, plan=_lib.GemmPlan()) == 0   # a plan without tiles
    assert lib.fp8gmm_grouped_gemm(None, 1, None, None, None, 0, 0, 2, 0, None, 0, None) == -1   # no plan
    # a launch that shares tiles along K needs its workspace, large enough and 256-byte aligned
    sk = _lib.GemmPlan(grid=8, rounds=2, total_tiles=1, n_fixups=1, n_slots=2)
    assert gemm(1, 0, 0, 2, 0, plan=sk, items=0x1000) == -1                       # tables first
    fake = 0x10000  # never dereferenced: validation ends before any launch
    assert lib.fp8gmm_grouped_gemm(fake, 1, fake, fake, sk, 0, 0, 2, 0, None, 0, None) == -9
    assert lib.fp8gmm_grouped_gemm(fake, 1, fake, fake, sk, 0, 0, 2, 0, fake, 2 * 262144 - 1, None) == -9
    assert lib.fp8gmm_grouped_gemm(fake, 1, fake, fake, sk, 0, 0, 2, 0, fake + 8, 2 * 262144, None) == -9
    assert b"workspace" in lib.fp8gmm_status_string(-9)


def test_plan_grouped_gemm_layouts():
    """Operands stored contraction-major: which pitch, alignment and size rules apply to which operand."""
    lib = _lib.load()
    total = ctypes.c_int(0)
    B, A = _lib.GEMM_B_KMAJOR, _lib.GEMM_A_KMAJOR

    def rc(t, layout):
        return lib.fp8gmm_plan_grouped_gemm_layout(t.ctypes.data, len(t), layout, ctypes.byref(total))

    # b[k, n]: ldb is the pitch of a k row (>= n), n must be a multiple of 16, a keeps the row-major rules
    assert rc(_prob([100], [256], [512], ldb=256), B) == 0 and total.value == 1
    assert rc(_prob([100], [256], [512], ldb=128), B) == -2      # pitch smaller than n
    assert rc(_prob([100], [256], [512]), 0) == 0                # the same table row-major: ldb = k
    assert rc(_prob([100], [264], [512], ldb=272), B) == -4      # n not a multiple of 16
    assert rc(_prob([100], [256], [520], ldb=256), B) == -4      # a is still fetched in 16-byte pieces of k
    assert rc(_prob([16], [65536], [65536], ldb=65536), B) == -2  # k * ldb >= 2^32
    # rows up to 127 past k are addressed and must fall outside the 32-bit descriptor, not wrap: (k + 128) * ldb
    assert rc(_prob([16], [65536], [65392], lda=65392, ldb=65536), B) == 0
    assert rc(_prob([16], [65536], [65408], lda=65408, ldb=65536), B) == -2
    # a[k, m] and b[k, n]: k is a row count and may be anything; m and n multiples of 16
    assert rc(_prob([512], [256], [137], lda=512, ldb=256), A | B) == 0
    assert rc(_prob([512], [256], [137], lda=500, ldb=256), A | B) == -2
    assert rc(_prob([520], [256], [137], lda=528, ldb=256), A | B) == -4
    assert rc(_prob([512], [256], [0], lda=512, ldb=256, a=0, b=0), A | B) == 0   # an expert without rows
    # a contraction-major a alone is not a layout the path uses; unknown bits are refused
    assert rc(_prob([512], [256], [128], lda=512), A) == -6
    assert rc(_prob([16], [16], [16]), 8) == -6
    # the launch refuses the same combinations, and a contraction-major b that is not e4m3
    plan = _lib.GemmPlan(grid=8, rounds=2, total_tiles=1)
    assert lib.fp8gmm_grouped_gemm(None, 1, None, None, plan, 0, 0, 2, A, None, 0, None) == -6
    assert lib.fp8gmm_grouped_gemm(None, 1, None, None, plan, 0, 1, 2, B, None, 0, None) == -3
    assert lib.fp8gmm_grouped_gemm(None, 1, None, None, plan, 0, 0, 2, A | B | _lib.EPI_GELU, None, 0,
                                   None) == -1   # valid flags, no table
    t = _prob([137, 0, 401], [512, 512, 512], [300, 0, 77], lda=[137 + 7, 16, 416], ldb=512)
    t["lda"] = [144, 16, 416]
    assert rc(t, A | B) == -4     # m = 137 is not a multiple of 16
    t = _prob([144, 0, 416], [512, 512, 512], [300, 0, 77], ldb=512)
    t["lda"] = [144, 16, 416]
    assert rc(t, A | B) == 0 and t["tile_begin"].tolist() == [0, 2, 2] and t["cost_begin"].tolist() == [0, 6, 6]


def test_gemm_grid_is_one_workgroup_per_compute_unit_in_multiples_of_eight():
    assert [_lib.gemm_grid(c) for c in (256, 304, 250, 8, 3, 0)] == [256, 304, 248, 8, 8, 8]


def test_launch_plan_reports_sizes_before_it_writes():
    """Arrays too small: status -8 and the required sizes in the plan; then the same call with room."""
    lib = _lib.load()
    t = _prob([1000, 300], [512, 512], [256, 256])
    plan = _lib.GemmPlan()
    items = np.full(4, 0x55, dtype=np.uint8).view(np.uint8)
    rc = lib.fp8gmm_plan_grouped_gemm_launch(t.ctypes.data, 2, 0, 16, 0, items.ctypes.data, 0, None, 0,
                                             ctypes.byref(plan))
    assert rc == -8 and (items == 0x55).all()
    # 4 x 2 + 2 x 2 = 12 tiles on 16 workgroups: one record each plus the end record
    assert (plan.total_tiles, plan.grid, plan.rounds, plan.n_fixups, plan.n_slots) == (12, 16, 2, 0, 0)
    p2, it, fx = _lib.plan_grouped_gemm_launch(t, 0, 16, False)
    assert (p2.grid, p2.rounds) == (16, 2) and len(it) == 32 and len(fx) == 0
    assert sorted(it["prob"][:16].tolist()) == [-1] * 4 + [0] * 8 + [1] * 4 and (it["prob"][16:] == -1).all()
    # a launch never has more workgroups than tiles (rounded up to a multiple of 8) when nothing is shared along K
    p3, it3, _ = _lib.plan_grouped_gemm_launch(_prob([100], [100], [128]), 0, 256, False)
    assert (p3.grid, p3.rounds, p3.total_tiles) == (8, 2, 1) and (it3["prob"] >= 0).sum() == 1
    # room for part of the list only: the same status and sizes; with exactly the room asked for, the same records
    # as with room to spare
    some = np.zeros(20, dtype=_lib.GEMM_ITEM)
    rc = lib.fp8gmm_plan_grouped_gemm_launch(t.ctypes.data, 2, 0, 16, 0, some.ctypes.data, 20, None, 0,
                                             ctypes.byref(plan))
    assert rc == -8 and (plan.grid, plan.rounds) == (16, 2)
    exact = np.zeros(32, dtype=_lib.GEMM_ITEM)
    rc = lib.fp8gmm_plan_grouped_gemm_launch(t.ctypes.data, 2, 0, 16, 0, exact.ctypes.data, 32, None, 0,
                                             ctypes.byref(plan))
    assert rc == 0 and exact.tobytes() == it.tobytes()
    # the form the launches upload: [problem table | work list | shared tiles]
    p4, blob, off_items, off_fix = _lib.plan_grouped_gemm_blob(t, 0, 16, False)
    assert (p4.grid, p4.rounds) == (16, 2) and off_items % 128 == 0 and off_fix == off_items + it.nbytes
    assert blob[: t.nbytes].tobytes() == t.tobytes() and blob[off_items: off_fix].tobytes() == it.tobytes()
    assert len(blob) == off_fix
    assert lib.fp8gmm_plan_grouped_gemm_launch(t.ctypes.data, 2, 0, 12, 0, None, 0, None, 0, ctypes.byref(plan)) == -6
    assert lib.fp8gmm_plan_grouped_gemm_launch(t.ctypes.data, 2, 0, 16, 0, None, 0, None, 0, None) == -1


def _mlp_pass(sizes, h, f, **over):
    """An fp8gmm_mlp_pass over made-up addresses (the planners are host code and never follow them)."""
    e = len(sizes)
    gs = np.asarray(sizes, dtype=np.int64)
    names = ("x", "x_fp8", "w1", "w1_fp8", "w2", "w2_fp8", "pre", "act_fp8", "y", "dy", "dy_fp8", "dact", "dpre_fp8",
             "dx", "dw1", "dw2", "fwd_scale", "fwd_scale_inv", "fwd_amax", "bwd_scale", "bwd_scale_inv", "bwd_amax")
    addr = {n: (i + 1) << 36 for i, n in enumerate(names)}
    fields = dict(experts=e, hidden=h, ffn=f, fwd_fmt=_lib.E4M3, bwd_fmt=_lib.E5M2, cast_weights=1, dgrad=1, wgrad=1,
                  grid=64, stream_k=1, tile_policy=0, tokens=int(gs.sum()), group_sizes=gs.ctypes.data, **addr)
    fields.update(over)
    return _lib.MlpPass(**fields), addr, gs


def test_mlp_pass_planner_lays_out_the_reference_data_flow():
    """fp8gmm_plan_mlp_forward / _backward against the data flow of the reference's grouped MLP stated launch by
    launch (fp8_gmm/grouped_mlp.py:60-150 forward, :183-318 backward): operand addresses of every expert, shapes,
    pitches and the scaling slots (forward 3 g / 3 g + 1 with fc2's GEMMs from g = E, backward 2 i and 2 E + 2 i)."""
    lib = _lib.load()
    assert lib.fp8gmm_sizeof_mlp_pass() == ctypes.sizeof(_lib.MlpPass) == 240
    sizes, h, f = [300, 0, 77, 513, 1], 256, 512
    e = len(sizes)
    desc, A, gs = _mlp_pass(sizes, h, f)
    row0 = np.concatenate([[0], np.cumsum(gs)[:-1]]).astype(np.uint64)
    idx = np.arange(e, dtype=np.uint64)
    slot = lambda name, first, stride: np.uint64(A[name] + 4 * first) + idx * np.uint64(4 * stride)
    blob = np.zeros(1 << 22, dtype=np.uint8)
    plan = _lib.PassPlan()

    def table(rec, dtype):
        return blob[rec.table_offset: rec.table_offset + rec.n * dtype.itemsize].view(dtype)

    def rows_problem(t, a, b, c, c_bytes, n, k, kmajor, a_si, b_si, aux=None):
        assert (t["a"] == np.uint64(A[a]) + row0 * np.uint64(k)).all()
        assert (t["b"] == np.uint64(A[b]) + idx * np.uint64(n * k)).all()
        assert (t["c"] == np.uint64(A[c]) + row0 * np.uint64(n * c_bytes)).all()
        assert (t["aux"] == (np.uint64(A[aux]) + row0 * np.uint64(2 * n) if aux else 0)).all()
        assert (t["m"] == gs).all() and (t["n"] == n).all() and (t["k"] == k).all()
        assert (t["lda"] == k).all() and (t["ldb"] == (n if kmajor else k)).all() and (t["ldc"] == n).all()
        assert (t["a_scale_inv"] == a_si).all() and (t["b_scale_inv"] == b_si).all()

    def wgrad_problem(t, a, b, c, m, n, a_si, b_si):
        assert (t["a"] == np.uint64(A[a]) + row0 * np.uint64(m)).all()
        assert (t["b"] == np.uint64(A[b]) + row0 * np.uint64(n)).all()
        assert (t["c"] == np.uint64(A[c]) + idx * np.uint64(2 * m * n)).all()
        assert (t["m"] == m).all() and (t["n"] == n).all() and (t["k"] == gs).all()
        assert (t["lda"] == m).all() and (t["ldb"] == n).all() and (t["ldc"] == n).all()
        assert (t["a_scale_inv"] == a_si).all() and (t["b_scale_inv"] == b_si).all()
        assert (t["aux"] == 0).all() and (t["c_scale"] == 0).all()

    def row_casts(t, src, dst, cols, scale, amax, src2=None):
        assert (t["in"] == np.uint64(A[src]) + row0 * np.uint64(2 * cols)).all()
        assert (t["out"] == np.uint64(A[dst]) + row0 * np.uint64(cols)).all()
        assert (t["in2"] == (np.uint64(A[src2]) + row0 * np.uint64(2 * cols) if src2 else 0)).all()
        assert (t["cols"] == gs * cols).all() and (t["rows"] == (gs > 0)).all()
        assert (t["scale"] == scale).all() and (t["amax"] == amax).all()

    _lib.check(lib.fp8gmm_plan_mlp_forward(ctypes.byref(desc), blob.ctypes.data, blob.nbytes, ctypes.byref(plan)))
    assert plan.n_launches == 3 and [plan.launch[i].kind for i in range(3)] == [_lib.PASS_CAST, _lib.PASS_GEMM, _lib.PASS_GEMM]
    t = table(plan.launch[0], _lib.TENSOR_DESC)
    assert len(t) == 3 * e
    for part, (src, dst, first) in enumerate((("w2", "w2_fp8", 3 * e + 1), ("w1", "w1_fp8", 1))):
        w = t[part * e: (part + 1) * e]
        assert (w["in"] == np.uint64(A[src]) + idx * np.uint64(2 * h * f)).all()
        assert (w["out"] == np.uint64(A[dst]) + idx * np.uint64(h * f)).all()
        assert (w["rows"] == 1).all() and (w["cols"] == h * f).all()
        assert (w["scale"] == slot("fwd_scale", first, 3)).all() and (w["amax"] == slot("fwd_amax", first, 3)).all()
    row_casts(t[2 * e:], "x", "x_fp8", h, slot("fwd_scale", 0, 3), slot("fwd_amax", 0, 3))
    fc1 = table(plan.launch[1], _lib.GEMM_PROBLEM)
    rows_problem(fc1, "x_fp8", "w1_fp8", "act_fp8", 1, f, h, False, slot("fwd_scale_inv", 0, 3),
                 slot("fwd_scale_inv", 1, 3), aux="pre")
    assert (fc1["c_scale"] == slot("fwd_scale", 3 * e, 3)).all() and (fc1["c_amax"] == slot("fwd_amax", 3 * e, 3)).all()
    assert (plan.launch[1].out_kind, plan.launch[1].epilogue, plan.launch[1].plan.tile) == (_lib.E4M3, _lib.EPI_GELU, 256)
    fc2 = table(plan.launch[2], _lib.GEMM_PROBLEM)
    rows_problem(fc2, "act_fp8", "w2_fp8", "y", 2, h, f, False, slot("fwd_scale_inv", 3 * e, 3),
                 slot("fwd_scale_inv", 3 * e + 1, 3))
    assert (fc2["c_scale"] == 0).all() and plan.launch[2].out_kind == _lib.OUT_BF16
    # algorithmic bytes of the GELU launch: both operands, the fp8 result and the bf16 pre-activation
    m = gs.astype(np.float64)
    assert plan.launch[1].bytes == float(((m + f) * h + m * f * 3).sum())
    assert plan.launch[1].work == float((2 * m * f * h).sum())

    _lib.check(lib.fp8gmm_plan_mlp_backward(ctypes.byref(desc), blob.ctypes.data, blob.nbytes, ctypes.byref(plan)))
    assert plan.n_launches == 6
    assert [(plan.launch[i].kind, plan.launch[i].op) for i in range(6)] == [
        (_lib.PASS_CAST, _lib.OP_QUANTIZE), (_lib.PASS_GEMM, 0), (_lib.PASS_GEMM, 0),
        (_lib.PASS_CAST, _lib.OP_CAST_DGELU), (_lib.PASS_GEMM, 0), (_lib.PASS_GEMM, 0)]
    g1 = (slot("bwd_scale", 0, 2), slot("bwd_amax", 0, 2), slot("bwd_scale_inv", 0, 2))
    g2 = (slot("bwd_scale", 2 * e, 2), slot("bwd_amax", 2 * e, 2), slot("bwd_scale_inv", 2 * e, 2))
    row_casts(table(plan.launch[0], _lib.TENSOR_DESC), "dy", "dy_fp8", h, g1[0], g1[1])
    wgrad_problem(table(plan.launch[1], _lib.GEMM_PROBLEM), "dy_fp8", "act_fp8", "dw2", h, f, g1[2],
                  slot("fwd_scale_inv", 3 * e, 3))
    rows_problem(table(plan.launch[2], _lib.GEMM_PROBLEM), "dy_fp8", "w2_fp8", "dact", 2, f, h, True, g1[2],
                 slot("fwd_scale_inv", 3 * e + 1, 3))
    row_casts(table(plan.launch[3], _lib.TENSOR_DESC), "dact", "dpre_fp8", f, g2[0], g2[1], src2="pre")
    rows_problem(table(plan.launch[4], _lib.GEMM_PROBLEM), "dpre_fp8", "w1_fp8", "dx", 2, h, f, True, g2[2],
                 slot("fwd_scale_inv", 1, 3))
    wgrad_problem(table(plan.launch[5], _lib.GEMM_PROBLEM), "dpre_fp8", "x_fp8", "dw1", f, h, g2[2],
                  slot("fwd_scale_inv", 0, 3))
    kk = _lib.GEMM_A_KMAJOR | _lib.GEMM_B_KMAJOR
    assert [plan.launch[i].epilogue for i in (1, 2, 4, 5)] == [kk, _lib.GEMM_B_KMAJOR, _lib.GEMM_B_KMAJOR, kk]
    # a cast leaves the merge of its running maxima to the GEMM launch right behind it, which finds the cast's table
    assert [plan.launch[i].merge_n for i in range(6)] == [e, e, 0, e, e, 0]
    assert plan.launch[1].merge_offset == plan.launch[0].table_offset
    assert plan.launch[4].merge_offset == plan.launch[3].table_offset
    assert [(plan.launch[i].a_fmt, plan.launch[i].b_fmt) for i in (1, 2, 4, 5)] == [(_lib.E5M2, _lib.E4M3)] * 4
    assert plan.launch[3].bytes == float((m * f * 5).sum()) and plan.launch[3].out_fmt == _lib.E5M2
    # every table on its own cache line, none overlapping the next
    ends = 0
    for i in range(6):
        rec = plan.launch[i]
        assert rec.table_offset % 128 == 0 and rec.table_offset >= ends
        ends = rec.table_offset + rec.n * (128 if rec.kind == _lib.PASS_CAST else 96)
        if rec.kind == _lib.PASS_GEMM:
            assert rec.items_offset % 128 == 0 and rec.items_offset >= ends
            ends = rec.items_offset + rec.plan.rounds * rec.plan.grid * 64
            assert rec.fixups_offset >= ends
            ends = rec.fixups_offset + rec.plan.n_fixups * 32
    assert ends <= plan.blob_bytes


def test_mlp_pass_planner_options_and_errors():
    lib = _lib.load()
    sizes, h, f = [300, 0, 77], 256, 512
    e = len(sizes)
    blob = np.zeros(1 << 21, dtype=np.uint8)
    plan = _lib.PassPlan()
    fwd, bwd = lib.fp8gmm_plan_mlp_forward, lib.fp8gmm_plan_mlp_backward
    run = lambda fn, d, room=blob.nbytes: fn(ctypes.byref(d), blob.ctypes.data, room, ctypes.byref(plan))
    # cached weights: only the input is cast
    d, _, _ = _mlp_pass(sizes, h, f, cast_weights=0, w1=0, w2=0)
    assert run(fwd, d) == 0 and plan.launch[0].n == e
    # gradients of the input only / of the weights only
    d, _, _ = _mlp_pass(sizes, h, f, wgrad=0, dw1=0, dw2=0, x_fp8=0, act_fp8=0)
    assert run(bwd, d) == 0 and plan.n_launches == 4
    assert [plan.launch[i].kind for i in range(4)] == [_lib.PASS_CAST, _lib.PASS_GEMM, _lib.PASS_CAST, _lib.PASS_GEMM]
    d, _, _ = _mlp_pass(sizes, h, f, dgrad=0, dx=0, w1_fp8=0)
    assert run(bwd, d) == 0 and plan.n_launches == 5
    # no tokens at all: nothing to do but the weight gradients, which are written as zeros
    d, _, _ = _mlp_pass([0, 0], h, f)
    assert run(bwd, d) == 0 and [plan.launch[i].kind for i in range(plan.n_launches)] == [0, _lib.PASS_GEMM, 0, 0, 0, _lib.PASS_GEMM]
    assert run(fwd, d) == 0 and [plan.launch[i].kind for i in range(3)] == [_lib.PASS_CAST, 0, 0]   # the weights
    assert plan.launch[0].merge_n == 0   # ... whose cast merges its own maxima: no GEMM follows
    # too little room: the size the pass needs, and nothing written past the room given
    d, _, _ = _mlp_pass(sizes, h, f)
    blob[:] = 0x55
    assert run(bwd, d, 4096) == -8 and (blob[4096:] == 0x55).all()
    need = plan.blob_bytes
    assert run(bwd, d, need) == 0 and plan.blob_bytes == need
    assert run(bwd, d, need - 128) == -8
    # errors
    for over, status in ((dict(hidden=250), -4), (dict(ffn=0), -6), (dict(tokens=5), -2), (dict(tile_policy=64), -6),
                         (dict(grid=0), -6), (dict(pre=0), -1), (dict(dact=0), -1), (dict(dw2=0), -1)):
        d, _, _ = _mlp_pass(sizes, h, f, **over)
        assert run(bwd, d) == status, over
    for over, status in ((dict(w1=0), -1), (dict(act_fp8=0), -1), (dict(fwd_amax=0), -1)):
        d, _, _ = _mlp_pass(sizes, h, f, **over)
        assert run(fwd, d) == status, over
    d, _, _ = _mlp_pass([-1, 1], h, f)
    assert run(fwd, d) == -2
    assert lib.fp8gmm_plan_mlp_forward(None, blob.ctypes.data, blob.nbytes, ctypes.byref(plan)) == -1
