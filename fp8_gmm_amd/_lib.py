"""ctypes binding of ``libfp8gmm_hip.so`` (the C ABI declared in ``include/fp8gmm.h``).

This plays the role of ``import fp8_gmm_backend`` in the reference
(fp8_gmm/backend.py:1, pybind module defined in csrc/ops.cu:9-16).  There is no
fallback: if the shared library is missing or does not export the expected
symbols, importing the backend raises.
"""
import ctypes
import threading
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libfp8gmm_hip.so")

E4M3 = 0
E5M2 = 1
OUT_BF16 = 2
EPI_GELU = 1
EPI_DGELU = 8
GEMM_B_KMAJOR = 2
GEMM_A_KMAJOR = 4
GEMM_TILE_128 = 0x100   # planning flag: 128 x 128 tiles, two workgroups per compute unit
GEMM_TILE_DUAL = 0x200  # planning flag: 128 x 256 tiles for the kernel form with two sets of accumulators

OP_QUANTIZE = 0
OP_SCALE_MUL = 1
OP_PAD_TRANSPOSE = 2
OP_PAD_CAST_TRANSPOSE = 3
OP_PAD_CAST_TRANSPOSE_DGELU = 4
OP_CAST_DGELU = 5

# struct fp8gmm_tensor_desc (128 bytes)
TENSOR_DESC = np.dtype(
    [
        ("in", "<u8"),
        ("in2", "<u8"),
        ("out", "<u8"),
        ("out_t", "<u8"),
        ("scale", "<u8"),
        ("amax", "<u8"),
        ("rows", "<i4"),
        ("cols", "<i4"),
        ("rows_padded", "<i4"),
        ("block_begin", "<i4"),
        ("amax_partial", "<u4"),   # scratch of the kernels (zeroed by the plan)
        ("reserved", "<u4", (15,)),  # pads the descriptor to one 128-byte cache line
    ],
    align=False,
)

# struct fp8gmm_gemm_problem (96 bytes)
GEMM_PROBLEM = np.dtype(
    [
        ("a", "<u8"),
        ("b", "<u8"),
        ("c", "<u8"),
        ("aux", "<u8"),
        ("a_scale_inv", "<u8"),
        ("b_scale_inv", "<u8"),
        ("c_scale", "<u8"),
        ("c_amax", "<u8"),
        ("m", "<i4"),
        ("n", "<i4"),
        ("k", "<i4"),
        ("lda", "<i4"),
        ("ldb", "<i4"),
        ("ldc", "<i4"),
        ("tile_begin", "<i4"),
        ("cost_begin", "<i4"),
    ],
    align=False,
)

# struct fp8gmm_gemm_item (64 bytes): one record of a launch's work list
GEMM_ITEM = np.dtype(
    [
        ("a", "<u8"),
        ("b", "<u8"),
        ("a_bytes", "<u4"),
        ("b_bytes", "<u4"),
        ("lda", "<i4"),
        ("ldb", "<i4"),
        ("k", "<i4"),
        ("k_begin", "<i4"),
        ("nk", "<i4"),
        ("m0", "<i4"),
        ("n0", "<i4"),
        ("prob", "<i4"),
        ("slot", "<i4"),
        ("flags", "<i4"),
    ],
    align=False,
)

# struct fp8gmm_gemm_fixup_desc (32 bytes): one tile that was shared along K
GEMM_FIXUP = np.dtype(
    [("prob", "<i4"), ("m0", "<i4"), ("n0", "<i4"), ("first_slot", "<i4"), ("n_pieces", "<i4"),
     ("reserved", "<i4", (3,))],
    align=False,
)

GEMM_SLOT_BYTES = 262144
GEMM_STATIC_SLOTS = 256


class GemmPlan(ctypes.Structure):
    """struct fp8gmm_gemm_plan"""

    _fields_ = [("grid", ctypes.c_int32), ("rounds", ctypes.c_int32), ("n_fixups", ctypes.c_int32),
                ("n_slots", ctypes.c_int32), ("total_tiles", ctypes.c_int32), ("tile", ctypes.c_int32),
                ("tile_m", ctypes.c_int32), ("reserved", ctypes.c_int32)]


class LinearPass(ctypes.Structure):
    """struct fp8gmm_linear_pass: one pass of a grouped linear layer, as the pass planner takes it"""

    _fields_ = [("experts", ctypes.c_int32), ("in_features", ctypes.c_int32), ("out_features", ctypes.c_int32),
                ("fwd_fmt", ctypes.c_int32), ("bwd_fmt", ctypes.c_int32), ("cast_weights", ctypes.c_int32),
                ("dgrad", ctypes.c_int32), ("wgrad", ctypes.c_int32), ("grid", ctypes.c_int32),
                ("stream_k", ctypes.c_int32), ("tile_policy", ctypes.c_int32), ("reserved", ctypes.c_int32),
                ("tokens", ctypes.c_int64), ("group_sizes", ctypes.c_void_p),
                ("x", ctypes.c_void_p), ("x_fp8", ctypes.c_void_p), ("w", ctypes.c_void_p), ("w_fp8", ctypes.c_void_p),
                ("y", ctypes.c_void_p), ("dy", ctypes.c_void_p), ("dy_fp8", ctypes.c_void_p), ("dx", ctypes.c_void_p),
                ("dw", ctypes.c_void_p), ("fwd_scale", ctypes.c_void_p), ("fwd_scale_inv", ctypes.c_void_p),
                ("fwd_amax", ctypes.c_void_p), ("bwd_scale", ctypes.c_void_p), ("bwd_scale_inv", ctypes.c_void_p),
                ("bwd_amax", ctypes.c_void_p)]


class MlpPass(ctypes.Structure):
    """struct fp8gmm_mlp_pass: one pass of a grouped MLP, as the pass planner takes it"""

    _fields_ = [("experts", ctypes.c_int32), ("hidden", ctypes.c_int32), ("ffn", ctypes.c_int32),
                ("fwd_fmt", ctypes.c_int32), ("bwd_fmt", ctypes.c_int32), ("cast_weights", ctypes.c_int32),
                ("dgrad", ctypes.c_int32), ("wgrad", ctypes.c_int32), ("grid", ctypes.c_int32),
                ("stream_k", ctypes.c_int32), ("tile_policy", ctypes.c_int32), ("reserved", ctypes.c_int32),
                ("tokens", ctypes.c_int64), ("group_sizes", ctypes.c_void_p)] + \
        [(name, ctypes.c_void_p) for name in (
            "x", "x_fp8", "w1", "w1_fp8", "w2", "w2_fp8", "pre", "act_fp8", "y", "dy", "dy_fp8", "dact", "dpre_fp8",
            "dx", "dw1", "dw2", "fwd_scale", "fwd_scale_inv", "fwd_amax", "bwd_scale", "bwd_scale_inv", "bwd_amax")]


class ScalingUpdate(ctypes.Structure):
    """struct fp8gmm_scaling_update"""

    _fields_ = [("amax_history", ctypes.c_void_p), ("scale", ctypes.c_void_p), ("scale_inv", ctypes.c_void_p),
                ("history_len", ctypes.c_int32), ("slots", ctypes.c_int32), ("fp8_max", ctypes.c_float),
                ("margin", ctypes.c_int32), ("most_recent", ctypes.c_int32), ("keep_period", ctypes.c_int32),
                ("keep_phase", ctypes.c_int32), ("reserved", ctypes.c_int32)]


MAX_SCALING_UPDATES = 4


class PassLaunch(ctypes.Structure):
    """struct fp8gmm_pass_launch"""

    _fields_ = [("kind", ctypes.c_int32), ("op", ctypes.c_int32), ("n", ctypes.c_int32),
                ("total_blocks", ctypes.c_int32), ("out_fmt", ctypes.c_int32), ("a_fmt", ctypes.c_int32),
                ("b_fmt", ctypes.c_int32), ("out_kind", ctypes.c_int32), ("epilogue", ctypes.c_int32),
                ("merge_n", ctypes.c_int32), ("table_offset", ctypes.c_int64), ("items_offset", ctypes.c_int64),
                ("fixups_offset", ctypes.c_int64), ("merge_offset", ctypes.c_int64), ("plan", GemmPlan),
                ("work", ctypes.c_double),
                ("bytes", ctypes.c_double)]


class PassPlan(ctypes.Structure):
    """struct fp8gmm_pass_plan"""

    _fields_ = [("n_launches", ctypes.c_int32), ("reserved", ctypes.c_int32), ("blob_bytes", ctypes.c_int64),
                ("launch", PassLaunch * 8)]


PASS_CAST = 1
PASS_GEMM = 2

EXPORTS = (
    "fp8gmm_version",
    "fp8gmm_status_string",
    "fp8gmm_sizeof_tensor_desc",
    "fp8gmm_sizeof_gemm_problem",
    "fp8gmm_sizeof_gemm_item",
    "fp8gmm_init",
    "fp8gmm_gemm_grid",
    "fp8gmm_plan_grouped_gemm_launch",
    "fp8gmm_grouped_gemm_static",
    "fp8gmm_plan_linear_forward",
    "fp8gmm_plan_linear_backward",
    "fp8gmm_plan_mlp_forward",
    "fp8gmm_plan_mlp_backward",
    "fp8gmm_sizeof_mlp_pass",
    "fp8gmm_run_planned",
    "fp8gmm_host_alloc",
    "fp8gmm_host_free",
    "fp8gmm_delayed_scaling_updates",
    "fp8gmm_sizeof_linear_pass",
    "fp8gmm_sizeof_pass_plan",
    "fp8gmm_gemm_tile_shape",
    "fp8gmm_plan_multi_tensor",
    "fp8gmm_plan_grouped_gemm",
    "fp8gmm_plan_grouped_gemm_layout",
    "fp8gmm_multi_quantize",
    "fp8gmm_multi_scale_mul",
    "fp8gmm_multi_pad_transpose",
    "fp8gmm_multi_pad_cast_transpose",
    "fp8gmm_multi_pad_cast_transpose_dgelu",
    "fp8gmm_multi_cast_dgelu",
    "fp8gmm_grouped_gemm",
    "fp8gmm_delayed_scaling_update",
    "fp8gmm_upload",
    "fp8gmm_route_workspace_bytes",
    "fp8gmm_route_sort",
    "fp8gmm_route_invert",
    "fp8gmm_moe_scatter_backward",
    "fp8gmm_route_topk",
    "fp8gmm_route_topk_backward",
    "fp8gmm_moe_gather",
    "fp8gmm_moe_scatter",
    "fp8gmm_moe_scatter_wgrad",
    "fp8gmm_gemm_schedule",
    "fp8gmm_gemm_fixup",
)


class Fp8GmmError(RuntimeError):
    """Raised when a C-ABI call returns a non-zero status (the reference raises RuntimeError via TORCH_CHECK)."""


_lib = None


ABI_VERSION = 3   # FP8GMM_VERSION of include/fp8gmm.h that the structures and argument lists below were written for


def load():
    """Load the shared library once; raise loudly when it is absent, incomplete or of another interface version."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} not found: the HIP extension is not built. "
            "Run `make -C fp8_gmm_amd/csrc -j8` (or `python -c 'import __graft_entry__ as g; g.build()'`)."
        )
    L = ctypes.CDLL(LIB_PATH)
    missing = [s for s in EXPORTS if not hasattr(L, s)]
    if missing:
        raise ImportError(f"{LIB_PATH} does not export {missing}")
    vp, ci = ctypes.c_void_p, ctypes.c_int
    ip = ctypes.POINTER(ctypes.c_int)
    L.fp8gmm_version.restype = ci
    L.fp8gmm_version.argtypes = []
    if L.fp8gmm_version() != ABI_VERSION:
        raise ImportError(f"{LIB_PATH} speaks version {L.fp8gmm_version()} of the interface, this package version "
                          f"{ABI_VERSION}: rebuild it (`make -C fp8_gmm_amd/csrc -j8`)")
    L.fp8gmm_status_string.restype = ctypes.c_char_p
    L.fp8gmm_status_string.argtypes = [ci]
    L.fp8gmm_sizeof_tensor_desc.restype = ctypes.c_size_t
    L.fp8gmm_sizeof_tensor_desc.argtypes = []
    L.fp8gmm_sizeof_gemm_problem.restype = ctypes.c_size_t
    L.fp8gmm_sizeof_gemm_problem.argtypes = []
    L.fp8gmm_gemm_tile_shape.restype = None
    L.fp8gmm_gemm_tile_shape.argtypes = [ip, ip]
    L.fp8gmm_plan_multi_tensor.restype = ci
    L.fp8gmm_plan_multi_tensor.argtypes = [vp, ci, ci, ip]
    L.fp8gmm_plan_grouped_gemm.restype = ci
    L.fp8gmm_plan_grouped_gemm.argtypes = [vp, ci, ip]
    L.fp8gmm_plan_grouped_gemm_layout.restype = ci
    L.fp8gmm_plan_grouped_gemm_layout.argtypes = [vp, ci, ci, ip]
    L.fp8gmm_multi_quantize.restype = ci
    L.fp8gmm_multi_quantize.argtypes = [vp, ci, ci, ci, vp]
    L.fp8gmm_multi_scale_mul.restype = ci
    L.fp8gmm_multi_scale_mul.argtypes = [vp, ci, ci, vp]
    L.fp8gmm_multi_pad_transpose.restype = ci
    L.fp8gmm_multi_pad_transpose.argtypes = [vp, ci, ci, vp]
    L.fp8gmm_multi_pad_cast_transpose.restype = ci
    L.fp8gmm_multi_pad_cast_transpose.argtypes = [vp, ci, ci, ci, vp]
    L.fp8gmm_multi_pad_cast_transpose_dgelu.restype = ci
    L.fp8gmm_multi_pad_cast_transpose_dgelu.argtypes = [vp, ci, ci, ci, vp]
    L.fp8gmm_multi_cast_dgelu.restype = ci
    L.fp8gmm_multi_cast_dgelu.argtypes = [vp, ci, ci, ci, vp]
    L.fp8gmm_sizeof_gemm_item.restype = ctypes.c_size_t
    L.fp8gmm_sizeof_gemm_item.argtypes = []
    L.fp8gmm_init.restype = ci
    L.fp8gmm_init.argtypes = [ci]
    L.fp8gmm_gemm_grid.restype = ci
    L.fp8gmm_gemm_grid.argtypes = [ci]
    pp = ctypes.POINTER(GemmPlan)
    L.fp8gmm_plan_grouped_gemm_launch.restype = ci
    L.fp8gmm_plan_grouped_gemm_launch.argtypes = [vp, ci, ci, ci, ci, vp, ci, vp, ci, pp]
    L.fp8gmm_grouped_gemm.restype = ci
    L.fp8gmm_grouped_gemm.argtypes = [vp, ci, vp, vp, pp, ci, ci, ci, ci, vp, ctypes.c_size_t, vp]
    L.fp8gmm_grouped_gemm_static.restype = ci
    L.fp8gmm_grouped_gemm_static.argtypes = [vp, ci, vp, vp, pp, ci, ci, ci, ci, vp]
    for fn in (L.fp8gmm_plan_linear_forward, L.fp8gmm_plan_linear_backward):
        fn.restype = ci
        fn.argtypes = [ctypes.POINTER(LinearPass), vp, ctypes.c_size_t, ctypes.POINTER(PassPlan)]
    for fn in (L.fp8gmm_plan_mlp_forward, L.fp8gmm_plan_mlp_backward):
        fn.restype = ci
        fn.argtypes = [ctypes.POINTER(MlpPass), vp, ctypes.c_size_t, ctypes.POINTER(PassPlan)]
    L.fp8gmm_sizeof_mlp_pass.restype = ctypes.c_size_t
    L.fp8gmm_sizeof_mlp_pass.argtypes = []
    L.fp8gmm_run_planned.restype = ci
    L.fp8gmm_run_planned.argtypes = [vp, ctypes.POINTER(PassLaunch), vp, ctypes.c_size_t, vp]
    L.fp8gmm_sizeof_linear_pass.restype = ctypes.c_size_t
    L.fp8gmm_sizeof_linear_pass.argtypes = []
    L.fp8gmm_sizeof_pass_plan.restype = ctypes.c_size_t
    L.fp8gmm_sizeof_pass_plan.argtypes = []
    L.fp8gmm_delayed_scaling_update.restype = ci
    L.fp8gmm_delayed_scaling_update.argtypes = [vp, vp, vp, ci, ci, ctypes.c_float, ci, ci, ci, ci, vp]
    L.fp8gmm_delayed_scaling_updates.restype = ci
    L.fp8gmm_delayed_scaling_updates.argtypes = [ctypes.POINTER(ScalingUpdate), ci, vp]
    L.fp8gmm_host_alloc.restype = vp
    L.fp8gmm_host_alloc.argtypes = [ctypes.c_size_t]
    L.fp8gmm_host_free.restype = None
    L.fp8gmm_host_free.argtypes = [vp]
    L.fp8gmm_upload.restype = ci
    L.fp8gmm_upload.argtypes = [vp, vp, ctypes.c_size_t, vp]
    L.fp8gmm_route_workspace_bytes.restype = ctypes.c_size_t
    L.fp8gmm_route_workspace_bytes.argtypes = [ci, ci]
    L.fp8gmm_route_sort.restype = ci
    L.fp8gmm_route_sort.argtypes = [vp, ci, ci, vp, vp, vp, vp, vp, vp, vp]
    L.fp8gmm_route_invert.restype = ci
    L.fp8gmm_route_invert.argtypes = [vp, ci, vp, vp]
    L.fp8gmm_moe_scatter_backward.restype = ci
    L.fp8gmm_moe_scatter_backward.argtypes = [vp, vp, vp, vp, vp, vp, ci, ci, ci, vp]
    L.fp8gmm_route_topk.restype = ci
    L.fp8gmm_route_topk.argtypes = [vp, ci, ci, ci, ci, vp, vp, vp, vp]
    L.fp8gmm_route_topk_backward.restype = ci
    L.fp8gmm_route_topk_backward.argtypes = [vp, vp, vp, ci, ci, ci, vp, ci, vp]
    L.fp8gmm_moe_gather.restype = ci
    L.fp8gmm_moe_gather.argtypes = [vp, vp, vp, vp, ci, ci, ci, vp]
    L.fp8gmm_moe_scatter.restype = ci
    L.fp8gmm_moe_scatter.argtypes = [vp, vp, vp, vp, ci, ci, ci, vp]
    L.fp8gmm_moe_scatter_wgrad.restype = ci
    L.fp8gmm_moe_scatter_wgrad.argtypes = [vp, vp, vp, vp, ci, ci, ci, vp]
    L.fp8gmm_gemm_schedule.restype = ci
    L.fp8gmm_gemm_schedule.argtypes = [vp, ci, ci, ci, ci, ci, vp, ci]
    L.fp8gmm_gemm_fixup.restype = ci
    L.fp8gmm_gemm_fixup.argtypes = [vp, ci, ci, ci, ci, ip, vp, ci]
    if L.fp8gmm_sizeof_tensor_desc() != TENSOR_DESC.itemsize or L.fp8gmm_sizeof_gemm_problem() != GEMM_PROBLEM.itemsize \
            or L.fp8gmm_sizeof_gemm_item() != GEMM_ITEM.itemsize or ctypes.sizeof(GemmPlan) != 32 \
            or L.fp8gmm_sizeof_linear_pass() != ctypes.sizeof(LinearPass) \
            or L.fp8gmm_sizeof_mlp_pass() != ctypes.sizeof(MlpPass) or ctypes.sizeof(ScalingUpdate) != 56 \
            or L.fp8gmm_sizeof_pass_plan() != ctypes.sizeof(PassPlan):
        raise ImportError("struct layout mismatch between fp8_gmm_amd/_lib.py and include/fp8gmm.h")
    _lib = L
    return L


def check(status):
    if status != 0:
        raise Fp8GmmError(f"fp8gmm error {status}: {load().fp8gmm_status_string(status).decode()}")


def plan_multi_tensor(table, op):
    """Validate + schedule a host table (numpy structured array of TENSOR_DESC). Returns total workgroups."""
    total = ctypes.c_int(0)
    check(load().fp8gmm_plan_multi_tensor(table.ctypes.data, len(table), op, ctypes.byref(total)))
    return total.value


def plan_grouped_gemm(table, layout=0):
    total = ctypes.c_int(0)
    check(load().fp8gmm_plan_grouped_gemm_layout(table.ctypes.data, len(table), layout, ctypes.byref(total)))
    return total.value


_plan_scratch = threading.local()   # grow-only output buffers of the launch planner, one set per thread


def _plan_into_scratch(table, layout, grid, stream_k):
    """Plan a launch into this thread's scratch buffers; returns (GemmPlan, items view, fixups view).  The views
    are overwritten by the thread's next call."""
    L = load()
    plan = GemmPlan()
    sc = _plan_scratch
    items = getattr(sc, "items", None)
    if items is None:
        items = sc.items = np.empty(8192, dtype=GEMM_ITEM)
        sc.fixups = np.empty(1024, dtype=GEMM_FIXUP)
    fixups = sc.fixups
    args = (table.ctypes.data, len(table), layout, grid, int(stream_k))   # 0 off, 1 on, > 1 on with that many slots
    rc = L.fp8gmm_plan_grouped_gemm_launch(*args, items.ctypes.data, len(items), fixups.ctypes.data, len(fixups),
                                           ctypes.byref(plan))
    if rc == -8:  # FP8GMM_ERR_BUFFER_TOO_SMALL: the sizes are in the plan
        if plan.rounds * plan.grid > len(items):
            items = sc.items = np.empty(2 * plan.rounds * plan.grid, dtype=GEMM_ITEM)
        if plan.n_fixups > len(fixups):
            fixups = sc.fixups = np.empty(2 * plan.n_fixups, dtype=GEMM_FIXUP)
        rc = L.fp8gmm_plan_grouped_gemm_launch(*args, items.ctypes.data, len(items), fixups.ctypes.data, len(fixups),
                                               ctypes.byref(plan))
    check(rc)
    return plan, items[: plan.rounds * plan.grid], fixups[: plan.n_fixups]


def plan_grouped_gemm_launch(table, layout, grid, stream_k):
    """Validate a host problem table and write the work list of a launch with `grid` workgroups.
    Returns (GemmPlan, items, fixups): numpy arrays of GEMM_ITEM [rounds * grid] and GEMM_FIXUP [n_fixups]."""
    plan, items, fixups = _plan_into_scratch(table, layout, grid, stream_k)
    return plan, items.copy(), fixups.copy()


def plan_grouped_gemm_blob(table, layout, grid, stream_k):
    """The same, as the bytes a launch uploads: [problem table | work list | shared tiles], each part on its own
    cache lines.  Returns (GemmPlan, blob, offset of the work list, offset of the shared-tile records)."""
    plan, items, fixups = _plan_into_scratch(table, layout, grid, stream_k)
    off_items = (table.nbytes + 127) // 128 * 128
    off_fix = off_items + items.nbytes
    blob = np.empty(off_fix + fixups.nbytes, dtype=np.uint8)
    blob[: table.nbytes] = table.view(np.uint8).reshape(-1)
    blob[table.nbytes: off_items] = 0
    blob[off_items: off_fix] = items.view(np.uint8).reshape(-1)
    blob[off_fix:] = fixups.view(np.uint8).reshape(-1)
    return plan, blob, off_items, off_fix


_num_cu = {}


def init(device_index):
    """fp8gmm_init once per device: compute-unit count (cached)."""
    cus = _num_cu.get(device_index)
    if cus is None:
        cus = load().fp8gmm_init(device_index)
        if cus <= 0:
            check(cus if cus < 0 else -7)
        _num_cu[device_index] = cus
    return cus


def gemm_grid(num_cu):
    return load().fp8gmm_gemm_grid(num_cu)


def gemm_schedule(table, total_tiles, grid, stream_k, wg, max_items=4096):
    """Items (tile, problem, m0, n0, k_begin, nk, slot) that workgroup `wg` of a `grid`-workgroup launch processes."""
    buf = np.zeros((max_items, 7), dtype=np.int32)
    n = load().fp8gmm_gemm_schedule(table.ctypes.data, len(table), total_tiles, grid, int(stream_k), wg,
                                    buf.ctypes.data, max_items)
    if n < 0:
        check(n)
    if n > max_items:
        return gemm_schedule(table, total_tiles, grid, stream_k, wg, n)
    return buf[:n]


def gemm_fixup(table, total_tiles, grid, wg, max_slots=64):
    """(tile, [slots in K order]) that fix-up workgroup `wg` completes; tile == -1: nothing to do."""
    tile = ctypes.c_int(-1)
    buf = np.zeros(max_slots, dtype=np.int32)
    n = load().fp8gmm_gemm_fixup(table.ctypes.data, len(table), total_tiles, grid, wg, ctypes.byref(tile),
                                 buf.ctypes.data, max_slots)
    if n < 0:
        check(n)
    return tile.value, buf[:min(n, max_slots)].tolist()


def gemm_tile_shape():
    tm, tn = ctypes.c_int(0), ctypes.c_int(0)
    load().fp8gmm_gemm_tile_shape(ctypes.byref(tm), ctypes.byref(tn))
    return tm.value, tn.value
