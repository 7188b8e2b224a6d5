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
    assert lib.fp8gmm_version() == 2
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
