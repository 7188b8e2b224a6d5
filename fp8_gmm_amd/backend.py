"""Python entry points of the MI355X FP8 grouped-GEMM backend.

Same names, positional signatures and meaning as the reference's
``fp8_gmm/backend.py`` (``multi_quantize`` :9, ``multi_transpose`` :13,
``multi_cast_transpose`` :17, ``multi_cast_transpose_dgelu`` :21,
``cublas_fp8_gemm`` :26, ``fp8_gmm`` :58), plus ``multi_scale_mul`` (pybind name in
csrc/ops.cu:12) and ``grouped_gemm``, the list form the wgrad path uses.  Every
function validates its arguments like the reference's TORCH_CHECKs, builds a
descriptor table, has the C library plan it, uploads it through pinned memory on
the current stream and enqueues ONE kernel.  Nothing here computes on the CPU and
there is no fallback: without the HIP library the import fails.
"""
import collections
import contextlib
import ctypes
import threading

import numpy as np
import torch

from . import _lib
from ._lib import GEMM_PROBLEM, TENSOR_DESC
import os

_lib.load()  # fail at import time, loudly, when the extension is missing

_FP8_DTYPES = (torch.float8_e4m3fn, torch.float8_e5m2)
_FMT = {torch.float8_e4m3fn: _lib.E4M3, torch.float8_e5m2: _lib.E5M2}
_OUT_KIND = {torch.bfloat16: _lib.OUT_BF16, torch.float8_e4m3fn: _lib.E4M3, torch.float8_e5m2: _lib.E5M2}


def _fail(msg):
    raise RuntimeError(msg)


class _on_device:
    """``torch.cuda.device(device)``, entered only when `device` is not the current one already (every launch sits
    in such a block, and the context manager costs the host several microseconds)."""

    __slots__ = ("guard",)

    def __init__(self, device):
        current = device.index is None or torch.cuda.current_device() == device.index
        self.guard = None if current else torch.cuda.device(device)

    def __enter__(self):
        if self.guard is not None:
            self.guard.__enter__()

    def __exit__(self, *exc):
        return self.guard.__exit__(*exc) if self.guard is not None else False


class kernel_timing:
    """Context manager that brackets every kernel launch of this module with HIP events.

    The events are recorded on the stream the kernels are launched on (torch's current
    stream).  ``records`` holds ``(kernel name, algorithmic work, algorithmic bytes, start event, end event,
    form)``; ``summary()`` synchronises and returns per-kernel launch counts, mean duration in ms, the
    algorithmic work (flops for the GEMM, bytes for the other kernels) and the algorithmic bytes
    (every operand read once, every result written once) per launch; for the grouped GEMM also the same four
    figures per operand form under ``"forms"`` (``gemm_form``).
    """

    _active = None

    def __init__(self):
        self.records = []

    def __enter__(self):
        kernel_timing._active = self
        return self

    def __exit__(self, *exc):
        kernel_timing._active = None
        return False

    def summary(self):
        torch.cuda.synchronize()
        out = {}
        for name, work, nbytes, start, end, form in self.records:
            ms = start.elapsed_time(end)
            d = out.setdefault(name, {"launches": 0, "ms": 0.0, "work": 0.0, "bytes": 0.0})
            cells = [d]
            if form is not None:
                cells.append(d.setdefault("forms", {}).setdefault(form, {"launches": 0, "ms": 0.0, "work": 0.0,
                                                                         "bytes": 0.0}))
            for c in cells:
                c["launches"] += 1
                c["ms"] += ms
                c["work"] += work
                c["bytes"] += nbytes
        for d in out.values():
            for c in [d] + list(d.get("forms", {}).values()):
                for key in ("ms", "work", "bytes"):
                    c[key] /= c["launches"]
        return out


def gemm_form(a_fmt, flags, plan=None):
    """Name of a grouped-GEMM launch by what it reads: the format of operand a (0 = e4m3, 1 = e5m2: a gradient) and
    which operands are stored contraction-major (the launch's FP8GMM_GEMM_*_KMAJOR flags); with the launch's plan,
    also the tile where it is not the 256 x 256 one."""
    fmt = "e5m2" if a_fmt == _lib.E5M2 else "e4m3"
    tile = ""
    if plan is not None and plan.tile_m not in (0, plan.tile):
        tile = f"; {plan.tile_m} x {plan.tile} tiles, two sets of accumulators"
    elif plan is not None and plan.tile not in (0, 256):
        tile = f"; {plan.tile} x {plan.tile} tiles"
    if flags & _lib.GEMM_A_KMAJOR:
        return f"{fmt} a and b contraction-major (weight gradient in place)" + tile
    if flags & _lib.GEMM_B_KMAJOR:
        return f"{fmt} a row-major, b contraction-major" + tile
    return f"{fmt} a and b row-major" + (", GELU epilogue" if flags & _lib.EPI_GELU else "") + tile


class _timed:
    def __init__(self, name, work_fn, bytes_fn=None, form=None):
        self.rec = kernel_timing._active
        if self.rec is not None:
            self.name, self.work = name, float(work_fn())
            self.bytes = float(bytes_fn()) if bytes_fn is not None else self.work
            self.form = form() if callable(form) else form

    def __enter__(self):
        if self.rec is not None:
            self.start = torch.cuda.Event(enable_timing=True)
            self.start.record()

    def __exit__(self, *exc):
        if self.rec is not None:
            end = torch.cuda.Event(enable_timing=True)
            end.record()
            self.rec.records.append((self.name, self.work, self.bytes, self.start, end, self.form))
        return False


_OP_NAMES = {
    _lib.OP_QUANTIZE: "multi_quantize",
    _lib.OP_SCALE_MUL: "multi_scale_mul",
    _lib.OP_PAD_TRANSPOSE: "multi_pad_transpose",
    _lib.OP_PAD_CAST_TRANSPOSE: "multi_pad_cast_transpose",
    _lib.OP_PAD_CAST_TRANSPOSE_DGELU: "multi_pad_cast_transpose_dgelu",
    _lib.OP_CAST_DGELU: "multi_cast_dgelu",
}


def _algorithmic_bytes(op, table):
    """HBM bytes an ideal kernel moves: every input element read once, every output element written once."""
    rows = table["rows"].astype(np.int64)
    cols = table["cols"].astype(np.int64)
    rpad = table["rows_padded"].astype(np.int64)
    if op == _lib.OP_QUANTIZE:
        return int((rows * cols * 3).sum())
    if op == _lib.OP_SCALE_MUL:
        return int((rows * cols * 4).sum())
    if op == _lib.OP_CAST_DGELU:
        return int((rows * cols * 5).sum())
    has_out = (table["out"] != 0).astype(np.int64)
    in_bytes = {_lib.OP_PAD_TRANSPOSE: 1, _lib.OP_PAD_CAST_TRANSPOSE: 2, _lib.OP_PAD_CAST_TRANSPOSE_DGELU: 4}[op]
    return int((cols * (rows * in_bytes + rows * has_out + rpad)).sum())


def _algorithmic_flops(table):
    return int((2 * table["m"].astype(np.int64) * table["n"].astype(np.int64) * table["k"].astype(np.int64)).sum())


def _algorithmic_gemm_bytes(table, c_bytes):
    """Both fp8 operands read once, the result (and the bf16 pre-GELU copy, where there is one) written once."""
    m, n, k = (table[f].astype(np.int64) for f in ("m", "n", "k"))
    aux = (table["aux"] != 0).astype(np.int64) * 2
    return int(((m + n) * k + m * n * (c_bytes + aux)).sum())


def _device_of(tensors):
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            _fail("fp8_gmm_amd: expected GPU tensors (the HIP path has no CPU fallback)")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            _fail("fp8_gmm_amd: all tensors of one call must live on the same device")
    return dev


class _Staging:
    """Page-locked host memory, mapped into the device's address space, in which the tables of the launches are
    written and from which ``fp8gmm_upload`` (a kernel on the launch stream) copies them to device memory.

    Two halves used in turn: pieces are handed out from one half until it is full; before the other half is written
    again, the host waits for the events recorded, on every stream that read from it, when it was left - so a piece
    is never overwritten while a copy kernel may still read it, and the host only ever waits when the GPU is a whole
    half (hundreds of launches) behind.  One per device, shared by all threads."""

    HALF = 16 << 20

    def __init__(self):
        # zeroed, not just allocated: the first write to each page of fresh page-locked memory costs the host a
        # page fault (0.15 ms per MB of tables, for the first 2 x HALF bytes of uploads)
        self.host = torch.zeros(2 * self.HALF, dtype=torch.uint8, pin_memory=True)
        self.bytes = self.host.numpy()
        self.base = self.host.data_ptr()
        self.lock = threading.Lock()
        self.half, self.used = 0, 0
        self.readers = [{}, {}]     # per half: stream handle -> torch stream object that read from it
        self.left = [[], []]        # per half: events recorded when it was left

    def reserve(self, nbytes, stream):
        """Offset of ``nbytes`` (rounded up to 256) of staging memory that ``stream`` will read, or None when the
        request is larger than a half."""
        n = (nbytes + 255) & ~255
        if n > self.HALF:
            return None
        with self.lock:
            if self.used + n > self.HALF:
                for s in self.readers[self.half].values():
                    ev = torch.cuda.Event()
                    ev.record(s)
                    self.left[self.half].append(ev)
                self.readers[self.half] = {}
                self.half ^= 1
                self.used = 0
                for ev in self.left[self.half]:
                    ev.synchronize()
                self.left[self.half] = []
            offset = self.half * self.HALF + self.used
            self.used += n
            self.readers[self.half].setdefault(stream.cuda_stream, stream)
        return offset

    def give_back(self, offset, reserved, used):
        """The piece at ``offset`` needs only ``used`` of its ``reserved`` bytes: the rest is handed out again if
        nothing was reserved after it."""
        reserved, used = (reserved + 255) & ~255, (used + 255) & ~255
        with self.lock:
            if offset + reserved == self.half * self.HALF + self.used:
                self.used -= reserved - used


class _CaptureArena:
    """Page-locked memory for the tables of launches that are being captured into a graph.  A replay runs the
    captured copy kernel again, which reads its source again: the tables must stay where they are, unchanged, for as
    long as the graph may be replayed, so this memory is handed out once and never recycled (a captured step of a
    module takes 0.1 - 1.5 MB of it).  Allocated through the library, which can do so while a stream is capturing."""

    CHUNK = 4 << 20

    def __init__(self):
        self.lock = threading.Lock()
        self.chunks = []        # (address, numpy view): alive until the process ends
        self.used = self.CHUNK  # of the last chunk

    def take(self, nbytes):
        n = (nbytes + 255) & ~255
        with self.lock:
            if self.used + n > self.CHUNK or not self.chunks:
                size = max(self.CHUNK, n)
                address = _lib.load().fp8gmm_host_alloc(size)
                if not address:
                    _fail("fp8_gmm_amd: could not allocate page-locked memory for the tables of a captured launch")
                view = np.ctypeslib.as_array((ctypes.c_uint8 * size).from_address(address))
                self.chunks.append((address, view))
                self.used = 0 if size == self.CHUNK else self.CHUNK
                if size != self.CHUNK:
                    return address, view[:nbytes]
            address, view = self.chunks[-1]
            offset = self.used
            self.used += n
        return address + offset, view[offset: offset + nbytes]


_capture_arena = _CaptureArena()
_staging = {}


def _staging_of(device):
    index = device.index if device.index is not None else torch.cuda.current_device()
    st = _staging.get(index)
    if st is None:
        st = _staging.setdefault(index, _Staging())
    return st


def _to_device(device, room, fill):
    """Device copy (uint8 tensor) of the tables that ``fill(host address, numpy view of the host bytes)`` writes
    into ``room`` bytes of staging memory; ``fill`` returns how many of them it used (None: all; 0: nothing to
    copy, the result is None).  The copy is enqueued on the current stream of ``device``."""
    room = (room + 15) & ~15
    with _on_device(device):
        stream = torch.cuda.current_stream(device)
        if torch.cuda.is_current_stream_capturing():
            # the captured copy kernel reads its source again at every replay: memory of its own, kept for good
            address, host = _capture_arena.take(room)
            used = fill(address, host)
            used = room if used is None else (used + 15) & ~15
            if not used:
                return None
            out = torch.empty(used, dtype=torch.uint8, device=device)
            _lib.check(_lib.load().fp8gmm_upload(out.data_ptr(), address, used, stream.cuda_stream))
            return out
        staged = options.upload == "kernel"
        st = _staging_of(device) if staged else None
        offset = st.reserve(room, stream) if st is not None else None
        if offset is None:   # larger than the staging area, or by choice: a pinned buffer of its own and torch's copy
            pinned = torch.empty(room, dtype=torch.uint8, pin_memory=True)
            used = fill(pinned.data_ptr(), pinned.numpy())
            used = room if used is None else (used + 15) & ~15
            return pinned[:used].to(device, non_blocking=True) if used else None
        used = fill(st.base + offset, st.bytes[offset: offset + room])
        used = room if used is None else (used + 15) & ~15
        if used < room:
            st.give_back(offset, room, used)
        if not used:
            return None
        out = torch.empty(used, dtype=torch.uint8, device=device)
        _lib.check(_lib.load().fp8gmm_upload(out.data_ptr(), st.base + offset, used, stream.cuda_stream))
    return out


def _upload(table, device):
    """Host table (numpy structured array) -> device bytes, asynchronously on the current stream."""
    raw = table.view(np.uint8).reshape(-1)

    def fill(_, host):
        host[: raw.size] = raw
        host[raw.size:] = 0

    return _to_device(device, raw.size, fill)


# A launch needs its table in device memory, and every upload is a small copy kernel in front of it.  Inside
# ``batched_uploads()`` the entry points only plan and queue their launch; at the end of the block all queued
# tables travel in ONE copy and the kernels are launched back to back, in the order they were queued.
_pending = threading.local()


@contextlib.contextmanager
def batched_uploads():
    """Queue the launches issued inside the block and upload all their tables with one copy at its end.

    Only for sequences made of this module's entry points: anything else that consumes their results
    (a torch op, a collective) has to come after the block, because the kernels are not enqueued before
    the block ends.  Nested blocks join the outermost one.  If the block raises, nothing is launched."""
    if getattr(_pending, "items", None) is not None:
        yield
        return
    _pending.items = []
    try:
        yield
        items = _pending.items
    finally:
        _pending.items = None
    _flush(items)


def flush_uploads():
    """Upload and launch what has been queued so far (for a consumer inside the block that is not one of this
    module's entry points, e.g. a collective on a result); queueing goes on afterwards."""
    items = getattr(_pending, "items", None)
    if items:
        _pending.items = []
        _flush(items)


def _submit(table, device, launch, keep):
    """Run ``launch(device address of table)`` now, or queue it when inside ``batched_uploads()``.

    ``keep`` holds every tensor the table points into.  A queued table is only raw addresses: without the
    references the caller's temporaries would be freed before the launch, and the allocator could hand
    their memory to someone else - to the uploaded tables themselves, for one."""
    items = getattr(_pending, "items", None)
    if items is not None:
        items.append((table, device, launch, keep))
        return
    dev_table = _upload(table, device)
    launch(dev_table.data_ptr())


def _flush(items):
    by_device = {}
    for it in items:
        by_device.setdefault(it[1], []).append(it)
    for device, group in by_device.items():
        offsets, total = [], 0
        for table, _, _, _ in group:
            offsets.append(total)
            total += (table.nbytes + 127) // 128 * 128   # every table on its own cache lines
        def fill(_, host, group=group, offsets=offsets):
            for (table, _, _, _), off in zip(group, offsets):
                host[off: off + table.nbytes] = table.view(np.uint8).reshape(-1)

        dev_tables = _to_device(device, total, fill)
        base = dev_tables.data_ptr()
        for (_, _, launch, _), off in zip(group, offsets):
            launch(base + off)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(device):
    """The HIP stream handle of torch's current stream on `device`."""
    if _raw_stream is not None and device.index is not None:
        return _raw_stream(device.index)
    return torch.cuda.current_stream(device).cuda_stream


def _scalar_ptrs(scalars, n, what):
    """Device addresses of n fp32 scalars given as a list of 0-d / 1-element tensors, a 1-D tensor, or None."""
    if scalars is None:
        return np.zeros(n, dtype=np.uint64)
    if isinstance(scalars, np.ndarray):  # device addresses already (Fp8MetaWrapper.get_meta_pointers)
        if scalars.dtype != np.uint64 or scalars.shape != (n,):
            _fail(f"fp8_gmm_amd: expected {n} device addresses for {what}")
        return scalars
    if isinstance(scalars, torch.Tensor):
        if scalars.dtype != torch.float32 or scalars.numel() != n or not scalars.is_contiguous():
            _fail(f"fp8_gmm_amd: {what} must be {n} contiguous fp32 values")
        _device_of([scalars])
        return scalars.data_ptr() + 4 * np.arange(n, dtype=np.uint64)
    if len(scalars) != n:
        _fail(f"fp8_gmm_amd: expected {n} {what}, got {len(scalars)}")
    out = np.zeros(n, dtype=np.uint64)
    for i, s in enumerate(scalars):
        if s is None:
            continue
        if s.dtype != torch.float32 or s.numel() != 1 or not s.is_cuda:
            _fail(f"fp8_gmm_amd: every entry of {what} must be a one-element fp32 GPU tensor")
        out[i] = s.data_ptr()
    return out


def _launch_multi(op, table, out_fmt, device, keep):
    """Plan, upload and launch one multi-tensor kernel over `table`."""
    total = _lib.plan_multi_tensor(table, op)
    if total == 0:
        return
    L = _lib.load()
    n = len(table)

    def launch(dev_ptr):
        with _on_device(device), _timed(_OP_NAMES[op], lambda: _algorithmic_bytes(op, table)):
            s = _stream(device)
            if op == _lib.OP_QUANTIZE:
                rc = L.fp8gmm_multi_quantize(dev_ptr, n, total, out_fmt, s)
            elif op == _lib.OP_SCALE_MUL:
                rc = L.fp8gmm_multi_scale_mul(dev_ptr, n, total, s)
            elif op == _lib.OP_PAD_TRANSPOSE:
                rc = L.fp8gmm_multi_pad_transpose(dev_ptr, n, total, s)
            elif op == _lib.OP_PAD_CAST_TRANSPOSE:
                rc = L.fp8gmm_multi_pad_cast_transpose(dev_ptr, n, total, out_fmt, s)
            elif op == _lib.OP_CAST_DGELU:
                rc = L.fp8gmm_multi_cast_dgelu(dev_ptr, n, total, out_fmt, s)
            else:
                rc = L.fp8gmm_multi_pad_cast_transpose_dgelu(dev_ptr, n, total, out_fmt, s)
        _lib.check(rc)

    _submit(table, device, launch, keep)


def _int64_vector(x, n):
    """x as n int64 values: an array of that shape as it is, a scalar repeated."""
    if isinstance(x, np.ndarray):
        if x.dtype == np.int64 and x.shape == (n,):
            return x
    elif isinstance(x, int):
        return np.full(n, x, dtype=np.int64)
    return np.broadcast_to(np.asarray(x, dtype=np.int64), (n,))


class TensorBatch:
    """n row-major 2-D tensors of one dtype on one device, held as arrays (address, rows, columns, row
    pitch in elements) instead of n tensor objects.

    The reference's entry points take Python lists of per-expert tensor views; with a hundred experts
    creating and inspecting those views costs more host time than the kernels run.  The modules
    therefore describe "rows bounds[i]:bounds[i+1] of this tensor", "slice i of this stack" or "block i
    of this buffer seen transposed" with array arithmetic on one base address.  Every entry point that
    takes a list of tensors also takes a TensorBatch."""

    __slots__ = ("ptr", "rows", "cols", "pitch", "dtype", "device", "_keep")

    def __init__(self, ptr, rows, cols, pitch, dtype, device, keep=()):
        n = len(ptr)
        self.ptr = np.asarray(ptr, dtype=np.uint64)
        self.rows = _int64_vector(rows, n)
        self.cols = _int64_vector(cols, n)
        self.pitch = _int64_vector(pitch, n)
        self.dtype = dtype
        self.device = device
        self._keep = tuple(keep)  # the tensors whose memory is described stay alive with the batch

    def __len__(self):
        return len(self.ptr)

    @property
    def contiguous(self):
        return bool(np.all((self.pitch == self.cols) | (self.rows <= 1) | (self.cols == 0)))

    @staticmethod
    def rows_of(t, bounds):
        """Row blocks bounds[i]:bounds[i+1] of a contiguous 2-D tensor."""
        if t.dim() != 2 or not t.is_contiguous():
            _fail("fp8_gmm_amd: row blocks need a contiguous 2-D tensor")
        b = np.asarray(bounds, dtype=np.int64)
        cols = t.shape[1]
        ptr = np.uint64(t.data_ptr()) + (b[:-1] * (cols * t.element_size())).astype(np.uint64)
        return TensorBatch(ptr, np.diff(b), cols, cols, t.dtype, t.device, (t,))

    @staticmethod
    def stack_of(t):
        """The slices t[i] of a contiguous [n, rows, cols] tensor."""
        if t.dim() != 3 or not t.is_contiguous():
            _fail("fp8_gmm_amd: a stack needs a contiguous 3-D tensor")
        n, r, c = t.shape
        ptr = np.uint64(t.data_ptr()) + np.arange(n, dtype=np.uint64) * np.uint64(r * c * t.element_size())
        return TensorBatch(ptr, r, c, c, t.dtype, t.device, (t,))

    @staticmethod
    def transposed_blocks_of(flat, bounds):
        """Block i = rows bounds[i]:bounds[i+1] of the contiguous buffer flat[sum, features], reinterpreted as
        the [features, bounds[i+1] - bounds[i]] transpose that the pad/transpose kernels write."""
        if flat.dim() != 2 or not flat.is_contiguous():
            _fail("fp8_gmm_amd: transposed blocks need a contiguous 2-D buffer")
        b = np.asarray(bounds, dtype=np.int64)
        feat = flat.shape[1]
        ptr = np.uint64(flat.data_ptr()) + (b[:-1] * (feat * flat.element_size())).astype(np.uint64)
        width = np.diff(b)
        return TensorBatch(ptr, feat, width, width, flat.dtype, flat.device, (flat,))

    @staticmethod
    def concat(batches):
        batches = [b for b in batches if b is not None and len(b)]
        if not batches:
            return None
        first = batches[0]
        for b in batches[1:]:
            if b.dtype != first.dtype:
                _fail("fp8_gmm_amd: all tensors of one argument must share a dtype")
            if b.device != first.device:
                _fail("fp8_gmm_amd: all tensors of one call must live on the same device")
        keep = tuple(t for b in batches for t in b._keep)
        return TensorBatch(np.concatenate([b.ptr for b in batches]), np.concatenate([b.rows for b in batches]),
                           np.concatenate([b.cols for b in batches]), np.concatenate([b.pitch for b in batches]),
                           first.dtype, first.device, keep)

    def __add__(self, other):
        return TensorBatch.concat([self, other])


def _as_batch(tensors, what, flatten=False):
    """A list of tensors (the reference's calling convention) as a TensorBatch.  flatten: any contiguous
    shape, seen as one row of numel elements; otherwise 2-D with a contiguous last dimension."""
    if isinstance(tensors, TensorBatch):
        return tensors
    tensors = list(tensors)
    n = len(tensors)
    dev = _device_of(tensors)
    ptr = np.zeros(n, dtype=np.uint64)
    rows = np.zeros(n, dtype=np.int64)
    cols = np.zeros(n, dtype=np.int64)
    pitch = np.zeros(n, dtype=np.int64)
    dtype = tensors[0].dtype if n else None
    for i, t in enumerate(tensors):
        if t.dtype != dtype:
            _fail(f"fp8_gmm_amd: all {what} of one call must share one dtype")
        ptr[i] = t.data_ptr()
        if flatten:
            if not t.is_contiguous():
                _fail(f"fp8_gmm_amd: {what} must be contiguous")
            numel = t.numel()
            rows[i], cols[i], pitch[i] = (1 if numel else 0), numel, numel
        else:
            if t.dim() != 2:
                _fail(f"fp8_gmm_amd: {what} must be 2-D")
            r, c = t.shape
            if c > 1 and t.stride(1) != 1:
                _fail(f"fp8_gmm_amd: {what} must have a contiguous last dimension")
            rows[i], cols[i] = r, c
            pitch[i] = t.stride(0) if (r > 1 and c > 0 and not t.is_contiguous()) else c
    return TensorBatch(ptr, rows, cols, pitch, dtype, dev, tensors)


def _same_device(*batches):
    dev = None
    for b in batches:
        if b is None:
            continue
        if b.device is None or b.device.type != "cuda":
            _fail("fp8_gmm_amd: expected GPU tensors (the HIP path has no CPU fallback)")
        if dev is None:
            dev = b.device
        elif b.device != dev:
            _fail("fp8_gmm_amd: all tensors of one call must live on the same device")
    return dev


def _fp8_dtype_of(*batches):
    dt = batches[0].dtype
    if dt not in _FP8_DTYPES:
        _fail("fp8_gmm_amd: outputs must be float8_e4m3fn or float8_e5m2")
    for b in batches[1:]:
        if b.dtype != dt:
            _fail("fp8_gmm_amd: all fp8 outputs of one call must share one fp8 dtype")
    return dt


def _check_counts(n, **args):
    for name, a in args.items():
        if len(a) != n:
            _fail(f"fp8_gmm_amd: {name} has {len(a)} entries, expected {n}")


# ------------------------------------------------------------------------------------------------
# multi-tensor element-wise / pad / transpose entry points
# ------------------------------------------------------------------------------------------------
def multi_quantize(inputs, outputs, scales, amaxes):
    """outputs[i] = fp8(inputs[i] * scales[i]); amaxes[i] = max(amaxes[i], max|inputs[i]|)."""
    n = len(inputs)
    if n == 0:
        return
    _check_counts(n, outputs=outputs, scales=scales, amaxes=amaxes)
    x, o = _as_batch(inputs, "multi_quantize inputs", flatten=True), _as_batch(outputs, "outputs", flatten=True)
    dev = _same_device(x, o)
    dt = _fp8_dtype_of(o)
    if x.dtype != torch.bfloat16:
        _fail("fp8_gmm_amd: multi_quantize inputs must be bfloat16")
    if not (x.contiguous and o.contiguous):
        _fail("fp8_gmm_amd: multi_quantize needs contiguous tensors")
    numel = x.rows * x.cols
    if np.any(numel != o.rows * o.cols):
        _fail("fp8_gmm_amd: multi_quantize input / output shapes differ")
    if np.any(numel >= 2**31):
        _fail("fp8_gmm_amd: tensors of 2^31 or more elements are not supported")
    table = np.zeros(n, dtype=TENSOR_DESC)
    table["in"], table["out"] = x.ptr, o.ptr
    table["rows"] = (numel > 0).astype(np.int32)
    table["cols"] = numel
    table["scale"] = _scalar_ptrs(scales, n, "scales")
    table["amax"] = _scalar_ptrs(amaxes, n, "amaxes")
    _launch_multi(_lib.OP_QUANTIZE, table, _FMT[dt], dev, (x, o, scales, amaxes))


def multi_scale_mul(inputs, scales_1, scales_2):
    """In place inputs[i] = bf16(inputs[i] * scales_1[i] * scales_2[i])."""
    n = len(inputs)
    if n == 0:
        return
    _check_counts(n, scales_1=scales_1, scales_2=scales_2)
    x = _as_batch(inputs, "multi_scale_mul inputs", flatten=True)
    dev = _same_device(x)
    if x.dtype != torch.bfloat16:
        _fail("fp8_gmm_amd: multi_scale_mul inputs must be bfloat16")
    if not x.contiguous:
        _fail("fp8_gmm_amd: multi_scale_mul needs contiguous tensors")
    numel = x.rows * x.cols
    table = np.zeros(n, dtype=TENSOR_DESC)
    table["in"] = x.ptr
    table["rows"] = (numel > 0).astype(np.int32)
    table["cols"] = numel
    table["scale"] = _scalar_ptrs(scales_1, n, "scales_1")
    table["in2"] = _scalar_ptrs(scales_2, n, "scales_2")
    _launch_multi(_lib.OP_SCALE_MUL, table, _lib.E4M3, dev, (x, scales_1, scales_2))


def _fill_transpose_shapes(table, x, t):
    if np.any(t.rows != x.cols) or np.any(t.cols < x.rows):
        _fail("fp8_gmm_amd: transposed output must be [cols, M] with M >= rows")
    if not (x.contiguous and t.contiguous):
        _fail("fp8_gmm_amd: transposes need contiguous tensors")
    if np.any(x.rows >= 2**31) or np.any(x.cols >= 2**31) or np.any(t.cols >= 2**31):
        _fail("fp8_gmm_amd: tensor extents of 2^31 or more are not supported")
    table["rows"] = x.rows
    table["cols"] = x.cols
    table["rows_padded"] = t.cols


def multi_transpose(inputs, outputs):
    """outputs[i][n, M] = pad(inputs[i][m, n].T): fp8 -> fp8, columns m..M-1 zero."""
    n = len(inputs)
    if n == 0:
        return
    _check_counts(n, outputs=outputs)
    x, t = _as_batch(inputs, "multi_transpose inputs"), _as_batch(outputs, "multi_transpose outputs")
    dev = _same_device(x, t)
    if x.dtype not in _FP8_DTYPES or x.dtype != t.dtype:
        _fail("fp8_gmm_amd: multi_transpose needs fp8 inputs and outputs of the same dtype")
    table = np.zeros(n, dtype=TENSOR_DESC)
    _fill_transpose_shapes(table, x, t)
    table["in"], table["out_t"] = x.ptr, t.ptr
    _launch_multi(_lib.OP_PAD_TRANSPOSE, table, _lib.E4M3, dev, (x, t))


def multi_cast_transpose(inputs, outputs, trans_outputs, scales, amaxes):
    """outputs[i] = fp8(inputs[i] * scale); trans_outputs[i] = its zero-padded transpose; amax merged."""
    n = len(inputs)
    if n == 0:
        return
    _check_counts(n, outputs=outputs, trans_outputs=trans_outputs, scales=scales, amaxes=amaxes)
    x = _as_batch(inputs, "multi_cast_transpose inputs")
    o = _as_batch(outputs, "multi_cast_transpose outputs")
    t = _as_batch(trans_outputs, "multi_cast_transpose transposed outputs")
    dev = _same_device(x, o, t)
    dt = _fp8_dtype_of(o, t)
    if x.dtype != torch.bfloat16:
        _fail("fp8_gmm_amd: multi_cast_transpose inputs must be bfloat16")
    if np.any(x.rows != o.rows) or np.any(x.cols != o.cols) or not o.contiguous:
        _fail("fp8_gmm_amd: multi_cast_transpose input / output shapes differ or output not contiguous")
    table = np.zeros(n, dtype=TENSOR_DESC)
    _fill_transpose_shapes(table, x, t)
    table["in"], table["out"], table["out_t"] = x.ptr, o.ptr, t.ptr
    table["scale"] = _scalar_ptrs(scales, n, "scales")
    table["amax"] = _scalar_ptrs(amaxes, n, "amaxes")
    _launch_multi(_lib.OP_PAD_CAST_TRANSPOSE, table, _FMT[dt], dev, (x, o, t, scales, amaxes))


def multi_cast_transpose_dgelu(inputs, gelu_inputs, outputs, trans_outputs, scales, amaxes):
    """Like multi_cast_transpose on x = inputs[i] * dgelu(gelu_inputs[i]) (tanh-GELU derivative)."""
    n = len(inputs)
    if n == 0:
        return
    _check_counts(n, gelu_inputs=gelu_inputs, outputs=outputs, trans_outputs=trans_outputs, scales=scales,
                  amaxes=amaxes)
    x = _as_batch(inputs, "multi_cast_transpose_dgelu inputs")
    g = _as_batch(gelu_inputs, "multi_cast_transpose_dgelu gelu inputs")
    o = _as_batch(outputs, "multi_cast_transpose_dgelu outputs")
    t = _as_batch(trans_outputs, "multi_cast_transpose_dgelu transposed outputs")
    dev = _same_device(x, g, o, t)
    dt = _fp8_dtype_of(o, t)
    if x.dtype != torch.bfloat16 or g.dtype != torch.bfloat16:
        _fail("fp8_gmm_amd: multi_cast_transpose_dgelu inputs must be bfloat16")
    same = np.all(x.rows == o.rows) and np.all(x.cols == o.cols) and np.all(x.rows == g.rows) and np.all(x.cols == g.cols)
    if not same or not (o.contiguous and g.contiguous):
        _fail("fp8_gmm_amd: multi_cast_transpose_dgelu shapes differ or tensors not contiguous")
    table = np.zeros(n, dtype=TENSOR_DESC)
    _fill_transpose_shapes(table, x, t)
    table["in"], table["in2"], table["out"], table["out_t"] = x.ptr, g.ptr, o.ptr, t.ptr
    table["scale"] = _scalar_ptrs(scales, n, "scales")
    table["amax"] = _scalar_ptrs(amaxes, n, "amaxes")
    _launch_multi(_lib.OP_PAD_CAST_TRANSPOSE_DGELU, table, _FMT[dt], dev, (x, g, o, t, scales, amaxes))


def multi_cast_dgelu(inputs, gelu_inputs, outputs, scales, amaxes):
    """outputs[i] = fp8(x * scales[i]) with x = inputs[i] * dgelu(gelu_inputs[i]); amaxes[i] = max(amaxes[i], max|x|).

    ``multi_cast_transpose_dgelu`` without the transposed copy, for a backward pass that needs no weight
    gradient.  The reference has no such kernel and notes the gap (fp8_gmm/grouped_mlp.py:252-253); the
    bytes and amax are those of ``multi_cast_transpose_dgelu``'s ``outputs``."""
    n = len(inputs)
    if n == 0:
        return
    _check_counts(n, gelu_inputs=gelu_inputs, outputs=outputs, scales=scales, amaxes=amaxes)
    x = _as_batch(inputs, "multi_cast_dgelu inputs", flatten=True)
    g = _as_batch(gelu_inputs, "multi_cast_dgelu gelu inputs", flatten=True)
    o = _as_batch(outputs, "multi_cast_dgelu outputs", flatten=True)
    dev = _same_device(x, g, o)
    dt = _fp8_dtype_of(o)
    if x.dtype != torch.bfloat16 or g.dtype != torch.bfloat16:
        _fail("fp8_gmm_amd: multi_cast_dgelu inputs must be bfloat16")
    if not (x.contiguous and g.contiguous and o.contiguous):
        _fail("fp8_gmm_amd: multi_cast_dgelu needs contiguous tensors")
    numel = x.rows * x.cols
    if np.any(numel != o.rows * o.cols) or np.any(numel != g.rows * g.cols):
        _fail("fp8_gmm_amd: multi_cast_dgelu input / gelu input / output shapes differ")
    if np.any(numel >= 2**31):
        _fail("fp8_gmm_amd: tensors of 2^31 or more elements are not supported")
    table = np.zeros(n, dtype=TENSOR_DESC)
    table["in"], table["in2"], table["out"] = x.ptr, g.ptr, o.ptr
    table["rows"] = (numel > 0).astype(np.int32)
    table["cols"] = numel
    table["scale"] = _scalar_ptrs(scales, n, "scales")
    table["amax"] = _scalar_ptrs(amaxes, n, "amaxes")
    _launch_multi(_lib.OP_CAST_DGELU, table, _FMT[dt], dev, (x, g, o, scales, amaxes))


# ------------------------------------------------------------------------------------------------
# GEMMs
# ------------------------------------------------------------------------------------------------
def _launch_gemm(table, a_dtype, b_dtype, c_dtype, gelu, device, keep, b_kmajor=False, a_kmajor=False, dgelu=False):
    if a_dtype not in _FP8_DTYPES or b_dtype not in _FP8_DTYPES:
        _fail("fp8_gmm_amd: GEMM operands must be fp8")
    if a_dtype == torch.float8_e5m2 and b_dtype == torch.float8_e5m2:
        _fail("fp8_gmm_amd: e5m2 x e5m2 GEMMs are not supported")
    if c_dtype not in _OUT_KIND:
        _fail("fp8_gmm_amd: GEMM output must be bfloat16 or fp8")
    if b_kmajor and b_dtype != torch.float8_e4m3fn:
        _fail("fp8_gmm_amd: a contraction-major b must be float8_e4m3fn")
    layout = (_lib.GEMM_B_KMAJOR if b_kmajor else 0) | (_lib.GEMM_A_KMAJOR if a_kmajor else 0)
    grid = _lib.gemm_grid(_lib.init(device.index if device.index is not None else torch.cuda.current_device()))
    epi = _lib.EPI_GELU if gelu else _lib.EPI_DGELU if dgelu else 0
    if not epi and _small_tiles(table):
        plan, blob, off_items, off_fix = _lib.plan_grouped_gemm_blob(table, layout | _lib.GEMM_TILE_128, 2 * grid, False)
    elif not epi and c_dtype == torch.bfloat16 and _dual_tiles(table, a_kmajor):
        plan, blob, off_items, off_fix = _lib.plan_grouped_gemm_blob(table, layout | _lib.GEMM_TILE_DUAL, grid, False)
    else:
        plan, blob, off_items, off_fix = _lib.plan_grouped_gemm_blob(table, layout | epi, grid, options.stream_k)
    if plan.total_tiles == 0:
        return
    n = len(table)
    fmts = (_FMT[a_dtype], _FMT[b_dtype], _OUT_KIND[c_dtype], epi | layout)

    def launch(dev_ptr):
        with _on_device(device):
            ws = _gemm_workspace(device, plan.n_slots)
            ws_ptr, ws_bytes = (ws.data_ptr(), ws.numel()) if ws is not None else (None, 0)
            with _timed("grouped_gemm", lambda: _algorithmic_flops(table),
                        lambda: _algorithmic_gemm_bytes(table, 2 if c_dtype == torch.bfloat16 else 1),
                        lambda: gemm_form(fmts[0], fmts[3], plan)):
                fix_ptr = dev_ptr + off_fix if plan.n_fixups else None
                rc = _lib.load().fp8gmm_grouped_gemm(dev_ptr, n, dev_ptr + off_items, fix_ptr, plan, *fmts, ws_ptr,
                                                     ws_bytes, _stream(device))
        _lib.check(rc)

    _submit(blob, device, launch, keep)


# Weight-gradient GEMMs contract over an expert's rows, the contiguous index of neither operand.  Both can be read
# in place (contraction-major), or the gradient can be cast with a transposed, zero-padded copy, as the reference
# does, and only the activation read in place (grouped_gemm(..., transposed="b")).  A contraction-major operand takes
# twice the LDS read instructions; on isolated back-to-back launches of config 2's shapes the copy form is 7 - 15 %
# faster (900 -> 765 us, 855 -> 795 us), inside the step the two weight gradients gain 40 us together and the two casts
# that write the copies lose 64 (config 2: 5.79 ms against 5.76 in place; config 4: 1.76 against 1.69).  So the
# modules read both operands in place; options.wgrad = "copy" selects the other form.  Same bits either way.
#
# Tile size of a grouped GEMM.  The 256 x 256 tile is the fast one per flop.  The 128 x 128 tile (two workgroups per
# compute unit, twice the operand traffic from L2) wins where the large tile leaves the machine idle: launches with
# fewer large tiles than about half the compute units, and launches whose problems are so short or narrow that the
# large tiles are mostly padding (measured 1.1 - 1.7 x there, 0.8 - 0.9 x on launches that fill the machine with
# full tiles).  Whole tiles get the same bits from either size; a tile that the large-tile launch shares along K is
# summed from fp32 partial sums, a deterministic but differently associated sum.  options.tile = "256" / "128"
# forces one size.
#
# Tail balancing of the grouped GEMM (the workgroups of an XCD share their range's last tiles along K) needs
# scratch memory for partial sums and a second, small launch; options.stream_k = False plans every launch without it.
class GemmOptions:
    """Launch policy of the grouped GEMMs of this process: ``tile`` "auto" | "256" | "128" | "dual", ``stream_k`` (share the
    tail tiles of a launch along K), ``wgrad`` "in_place" | "copy", ``upload`` "kernel" (tables reach the device
    through staging memory and a copy kernel of the library) | "copy" (a pinned buffer per upload and torch's
    asynchronous copy; while a stream is being captured into a graph the tables always take the first way, from
    memory that is kept for the replays).  The defaults can be preset with the environment variables FP8GMM_TILE, FP8GMM_STREAMK
    (0 turns sharing off), FP8GMM_WGRAD and FP8GMM_UPLOAD, read once when the module is imported; afterwards assign
    the attributes or use ``gemm_options(...)`` for a block."""

    __slots__ = ("tile", "stream_k", "wgrad", "upload")

    def __init__(self, env=os.environ):
        self.tile = env.get("FP8GMM_TILE", "auto")
        self.stream_k = env.get("FP8GMM_STREAMK", "1") != "0"
        self.wgrad = env.get("FP8GMM_WGRAD", "in_place")
        self.upload = env.get("FP8GMM_UPLOAD", "kernel")


options = GemmOptions()


@contextlib.contextmanager
def gemm_options(**changes):
    """Set attributes of ``options`` for the duration of a block."""
    saved = {k: getattr(options, k) for k in changes}
    for k, v in changes.items():
        setattr(options, k, v)
    try:
        yield options
    finally:
        for k, v in saved.items():
            setattr(options, k, v)


def wgrad_wants_transposed_gradient(total_rows, num_groups):
    return options.wgrad == "copy" and num_groups > 0 and total_rows > 0


# The form with two sets of accumulators (128 x 256 tiles, a finished tile stored between the products of the next
# one) takes the tile boundaries out of a launch and pays with operand traffic: 1.33 x the bytes from L2 per flop and
# three quarters of the bytes in flight per compute unit.  It wins where the boundaries are what a launch waits for
# - contractions of up to 2048 whose operands and result the 256 MB memory-side cache can largely hold, 7 - 17 %
# there - and loses where the launch streams from HBM (by 15 - 25 % on config 4's launches) or keeps the matrix pipes
# busy (by 20 - 35 % at K >= 3072).  The weight-gradient form (both operands contraction-major) loses 4 % even
# then.  options.tile = "dual" forces it wherever it exists (bf16 results, no fused epilogue).
_DUAL_MAX_K = 2048
_DUAL_MAX_BYTES = 320 << 20


def _dual_tiles(table, a_kmajor):
    if options.tile != "auto":
        return options.tile == "dual"
    if a_kmajor or len(table) == 0:
        return False
    m, n, k = (table[f].astype(np.int64) for f in ("m", "n", "k"))
    return int(k.max()) <= _DUAL_MAX_K and int(((m + n) * k + 2 * m * n).sum()) <= _DUAL_MAX_BYTES


def _small_tiles(table):
    if options.tile != "auto":
        return options.tile == "128"
    m, n = table["m"].astype(np.int64), table["n"].astype(np.int64)
    large = int((((m + 255) // 256) * ((n + 255) // 256)).sum())
    if large == 0:
        return False
    small = int((((m + 127) // 128) * ((n + 127) // 128)).sum())
    return large <= 160 or 2 * small <= 5 * large


# The partial sums of tiles shared along K go to a workspace that the library takes from the caller.  One buffer
# per (device, stream), grown on demand: launches on one stream are ordered and can share it.  The cache keeps the
# buffers of the few streams used most recently (a program that creates and destroys streams would otherwise leave a
# buffer behind for each, and a recycled handle would find a stranger's entry - harmless, the contents never
# matter, but unbounded); release_workspaces() drops them all.
_MAX_WORKSPACES = 8
_workspaces = collections.OrderedDict()


def _gemm_workspace(device, n_slots):
    if n_slots == 0:
        return None
    key = (device.index if device.index is not None else torch.cuda.current_device(), _stream(device))
    ws = _workspaces.get(key)
    need = n_slots * _lib.GEMM_SLOT_BYTES
    if ws is None or ws.numel() < need:
        ws = torch.empty(need, dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    _workspaces.move_to_end(key)
    while len(_workspaces) > _MAX_WORKSPACES:
        _workspaces.popitem(last=False)   # queued kernels keep using it: the allocator frees in stream order
    return ws


def release_workspaces():
    """Drop the cached tail-balancing workspaces (they are allocated again on demand)."""
    _workspaces.clear()


def warm_up(device=None):
    """Do everything a first launch on `device` would do besides the launch itself - the library's per-device
    initialisation, the allocation of a tail-balancing workspace of the largest size a launch can need
    (2 x grid slots of 256 KB: 128 MiB on 256 compute units) for the current stream, and of the page-locked staging
    memory of the table uploads - so that none of it falls into a timed or captured region."""
    device = torch.device("cuda") if device is None else torch.device(device)
    if device.index is None:
        device = torch.device("cuda", torch.cuda.current_device())
    grid = _lib.gemm_grid(_lib.init(device.index))
    with _on_device(device):
        _gemm_workspace(device, 2 * grid)
        if options.upload == "kernel":
            _staging_of(device)


# ------------------------------------------------------------------------------------------------
# a whole pass of a grouped linear layer, planned by one library call
# ------------------------------------------------------------------------------------------------
def _run_pass(device, desc, fields, plan_fn, bound_fn):
    """Fill the pass description `desc` from `fields`, plan it with `plan_fn` straight into staging memory (of
    `bound_fn(desc, grid)` bytes at first; the planner says how much it needs when that is too little), upload the
    tables and enqueue the launches."""
    L = _lib.load()
    flush_uploads()   # launches queued before this pass come first
    keep = []
    for name, value in fields.items():
        if isinstance(value, torch.Tensor):
            keep.append(value)
            value = value.data_ptr()
        elif isinstance(value, np.ndarray):
            keep.append(value)
            value = value.ctypes.data
        setattr(desc, name, value)
    index = device.index if device.index is not None else torch.cuda.current_device()
    grid = _lib.gemm_grid(_lib.init(index))
    desc.grid = grid
    desc.stream_k = int(bool(options.stream_k))
    desc.tile_policy = {"auto": 0, "256": 256, "128": 128, "dual": _lib.GEMM_TILE_DUAL}[options.tile]
    bound = bound_fn(desc, grid)
    plan = _lib.PassPlan()
    while True:
        def fill(address, _):
            fill.rc = plan_fn(ctypes.byref(desc), address, bound, ctypes.byref(plan))
            return int(plan.blob_bytes) if fill.rc == 0 else 0

        blob = _to_device(device, bound, fill)
        if fill.rc == -8 and plan.blob_bytes > bound:   # FP8GMM_ERR_BUFFER_TOO_SMALL
            bound = int(plan.blob_bytes)
            continue
        _lib.check(fill.rc)
        break
    if blob is None:
        return plan
    with _on_device(device):
        base, stream = blob.data_ptr(), _stream(device)
        for i in range(plan.n_launches):
            rec = plan.launch[i]
            if rec.kind == 0:
                continue
            gemm = rec.kind == _lib.PASS_GEMM
            ws = _gemm_workspace(device, rec.plan.n_slots) if gemm else None
            ws_ptr, ws_bytes = (ws.data_ptr(), ws.numel()) if ws is not None else (None, 0)
            with _timed("grouped_gemm" if gemm else _OP_NAMES[rec.op], lambda: rec.work, lambda: rec.bytes,
                        (lambda: gemm_form(rec.a_fmt, rec.epilogue, rec.plan)) if gemm else None):
                rc = L.fp8gmm_run_planned(base, ctypes.byref(rec), ws_ptr, ws_bytes, stream)
            _lib.check(rc)
    return plan


def _pass_room(experts, tokens, shapes, casts, grid):
    """Bytes that surely hold the tables of a pass with GEMMs over ``shapes`` (pairs of feature counts; every GEMM
    is token-sliced in one dimension or per expert in both) and ``casts`` cast descriptors: per GEMM a problem table
    and a work list of at most one record per 128 x 128 tile plus a few rounds of end records and the shared-tile
    records."""
    room = 4096 + casts * 128
    for a, b in shapes:
        widest = max(a, b)
        tiles = (tokens // 128 + experts) * ((widest + 127) // 128) + experts * ((a + 127) // 128) * ((b + 127) // 128)
        room += experts * 96 + 256 + (tiles + 8 * grid) * 64 + 32 * 2 * grid
    return room


def linear_pass(device, backward=False, **fields):
    """Plans one pass of a grouped linear layer with ONE library call (fp8gmm_plan_linear_forward / _backward),
    uploads its tables with one copy and enqueues its launches.  ``fields`` are the members of
    ``fp8gmm_linear_pass`` (include/fp8gmm.h): tensors are given as tensors (their addresses are taken here),
    ``group_sizes`` as an int64 numpy array.  The tables are the ones the per-launch entry points of this module
    build for the same tensors; what this call saves is the host time of building them in Python."""
    L = _lib.load()
    return _run_pass(
        device, _lib.LinearPass(), fields, L.fp8gmm_plan_linear_backward if backward else L.fp8gmm_plan_linear_forward,
        lambda d, grid: _pass_room(d.experts, d.tokens, [(d.in_features, d.out_features)] * 3, 2 * d.experts, grid))


def mlp_pass(device, backward=False, **fields):
    """The same for one pass of a grouped MLP in its default data flow (fp8gmm_plan_mlp_forward / _backward, members
    of ``fp8gmm_mlp_pass``): three launches forward, up to six backward, from one library call and one upload."""
    L = _lib.load()
    return _run_pass(
        device, _lib.MlpPass(), fields, L.fp8gmm_plan_mlp_backward if backward else L.fp8gmm_plan_mlp_forward,
        lambda d, grid: _pass_room(d.experts, d.tokens, [(d.hidden, d.ffn)] * 4, 3 * d.experts, grid))


def delayed_scaling_update(amax_history, scale, scale_inv, fp8_max, margin=0, most_recent=False, keep_scale_inv=None):
    """In-place delayed-scaling update of one direction in ONE kernel (the rule of
    ``fp8.amax_and_scale_update``): ``amax_history`` [history, slots], ``scale`` / ``scale_inv`` [slots].
    ``keep_scale_inv=(period, phase)`` leaves ``scale_inv[slot]`` untouched where ``slot % period == phase``."""
    period, phase = keep_scale_inv if keep_scale_inv is not None else (0, 0)
    for t, what in ((amax_history, "amax_history"), (scale, "scale"), (scale_inv, "scale_inv")):
        if t.dtype != torch.float32 or not t.is_contiguous():
            _fail(f"fp8_gmm_amd: {what} must be a contiguous fp32 tensor")
    if amax_history.dim() != 2 or scale.numel() != amax_history.shape[1] or scale_inv.numel() != scale.numel():
        _fail("fp8_gmm_amd: amax_history must be [history, slots] and scale / scale_inv [slots]")
    dev = _device_of([amax_history, scale, scale_inv])
    with _on_device(dev):
        rc = _lib.load().fp8gmm_delayed_scaling_update(
            amax_history.data_ptr(), scale.data_ptr(), scale_inv.data_ptr(), amax_history.shape[0],
            amax_history.shape[1], float(fp8_max), int(margin), int(bool(most_recent)), int(period), int(phase),
            _stream(dev))
    _lib.check(rc)


def delayed_scaling_updates(updates):
    """Several ``delayed_scaling_update`` calls (tuples of its arguments, all tensors on one device) in ONE kernel
    launch: a module's forward and backward scaling state in front of every step."""
    if not updates:
        return
    if len(updates) > _lib.MAX_SCALING_UPDATES:
        _fail(f"fp8_gmm_amd: at most {_lib.MAX_SCALING_UPDATES} scaling updates per launch")
    table = (_lib.ScalingUpdate * len(updates))()
    tensors = []
    for u, args in zip(table, updates):
        amax_history, scale, scale_inv, fp8_max = args[:4]
        margin, most_recent, keep = (tuple(args[4:]) + (0, False, None)[len(args) - 4:])[:3]
        for t, what in ((amax_history, "amax_history"), (scale, "scale"), (scale_inv, "scale_inv")):
            if t.dtype != torch.float32 or not t.is_contiguous():
                _fail(f"fp8_gmm_amd: {what} must be a contiguous fp32 tensor")
        if amax_history.dim() != 2 or scale.numel() != amax_history.shape[1] or scale_inv.numel() != scale.numel():
            _fail("fp8_gmm_amd: amax_history must be [history, slots] and scale / scale_inv [slots]")
        period, phase = keep if keep is not None else (0, 0)
        u.amax_history, u.scale, u.scale_inv = amax_history.data_ptr(), scale.data_ptr(), scale_inv.data_ptr()
        u.history_len, u.slots = amax_history.shape
        u.fp8_max, u.margin, u.most_recent = float(fp8_max), int(margin), int(bool(most_recent))
        u.keep_period, u.keep_phase = int(period), int(phase)
        tensors += [amax_history, scale, scale_inv]
    dev = _device_of(tensors)
    with _on_device(dev):
        rc = _lib.load().fp8gmm_delayed_scaling_updates(table, len(updates), _stream(dev))
    _lib.check(rc)


def grouped_gemm(a_list, b_list, c_list, a_scale_invs, b_scale_invs, pre_gelu_outs=None, c_scales=None,
                 c_amaxes=None, transposed=False):
    """c_list[i][m, n] = epilogue(a_list[i][m, k] . b_list[i][n, k]^T) for all i in ONE launch.

    The list form of ``cublas_fp8_gemm``: the reference issues these as a Python loop of
    cuBLASLt calls (wgrad, grouped_linear.py:173-182; grouped_mlp.py:234-242,313-322).
    k may differ per entry and may be 0 (the output is then the epilogue of zero).
    Lists of tensors or TensorBatches.

    ``transposed=True`` (not in the reference): the operands are given contraction-major, ``a_list[i][k, m]`` and
    ``b_list[i][k, n]``, and ``c = a^T . b``.  That is the weight gradient ``dW = dY^T . X`` on the row-major
    gradient and activation slices of an expert, with no padded transposed copies; k (the expert's row count) may be
    any number, m and n must be multiples of 16.

    ``transposed="b"``: only b is contraction-major, ``a_list[i][m, kpad]`` (a zero-padded transposed copy, kpad >= k a
    multiple of 16) and ``b_list[i][k, n]``, ``c = a[:, :k] . b``: the weight gradient with the reference's transposed
    copy of the gradient and the activation read in place.  A contraction-major operand takes twice the LDS read
    instructions of a row-major one; as isolated launches with long contractions this form is 7 - 15 % faster than
    ``transposed=True``; same bits.
    """
    n = len(a_list)
    if n == 0:
        return
    if isinstance(transposed, (bool, np.bool_)):
        transposed = bool(transposed)
    elif transposed != "b":
        _fail('fp8_gmm_amd: transposed must be False, True or "b"')
    _check_counts(n, b_list=b_list, c_list=c_list)
    a, b, c = _as_batch(a_list, "a"), _as_batch(b_list, "b"), _as_batch(c_list, "c")
    aux = None if pre_gelu_outs is None else _as_batch(pre_gelu_outs, "pre_gelu_outs")
    dev = _same_device(a, b, c, aux)
    fp8_out = c.dtype in _FP8_DTYPES
    if fp8_out and c_scales is None:
        _fail("fp8_gmm_amd: an fp8 GEMM output needs c_scales")
    table = np.zeros(n, dtype=GEMM_PROBLEM)
    table["a"], table["b"], table["c"] = a.ptr, b.ptr, c.ptr
    if transposed == "b":
        if np.any(a.cols < b.rows) or np.any(c.rows != a.rows) or np.any(c.cols != b.cols):
            _fail("fp8_gmm_amd: GEMM shapes do not match: a [m, kpad >= k], b [k, n], c [m, n]")
        table["m"], table["n"], table["k"] = a.rows, b.cols, b.rows
    elif transposed:
        if np.any(a.rows != b.rows) or np.any(c.rows != a.cols) or np.any(c.cols != b.cols):
            _fail("fp8_gmm_amd: GEMM shapes do not match: a [k, m], b [k, n], c [m, n]")
        table["m"], table["n"], table["k"] = a.cols, b.cols, a.rows
    else:
        if np.any(a.cols != b.cols) or np.any(c.rows != a.rows) or np.any(c.cols != b.rows):
            _fail("fp8_gmm_amd: GEMM shapes do not match: a [m, k], b [n, k], c [m, n]")
        table["m"], table["n"], table["k"] = a.rows, b.rows, a.cols
    table["lda"] = np.maximum(a.pitch, a.cols)
    table["ldb"] = np.maximum(b.pitch, b.cols)
    table["ldc"] = np.maximum(c.pitch, c.cols)
    if aux is not None:
        if len(aux) != n or aux.dtype != torch.bfloat16 or np.any(aux.rows != c.rows) or np.any(aux.cols != c.cols) \
                or np.any(np.maximum(aux.pitch, aux.cols) != table["ldc"]):
            _fail("fp8_gmm_amd: pre_gelu_out must be bf16 [m, n] with the row pitch of c")
        table["aux"] = aux.ptr
    table["a_scale_inv"] = _scalar_ptrs(a_scale_invs, n, "a_scale_invs")
    table["b_scale_inv"] = _scalar_ptrs(b_scale_invs, n, "b_scale_invs")
    if fp8_out:
        table["c_scale"] = _scalar_ptrs(c_scales, n, "c_scales")
        table["c_amax"] = _scalar_ptrs(c_amaxes, n, "c_amaxes")
    _launch_gemm(table, a.dtype, b.dtype, c.dtype, aux is not None, dev,
                 (a, b, c, aux, a_scale_invs, b_scale_invs, c_scales, c_amaxes), b_kmajor=bool(transposed),
                 a_kmajor=transposed is True)


def cublas_fp8_gemm(a, b, c, a_scale_inv, b_scale_inv, pre_gelu_out=None, c_scale=None, c_amax=None, backward=False):
    """c[m, n] = (a[m, k] . b[n, k]^T) * a_scale_inv * b_scale_inv, both operands K-contiguous ("TN").

    With ``pre_gelu_out`` the epilogue is GELU-aux: pre_gelu_out = bf16(result), c = gelu(result);
    an fp8 ``c`` is additionally multiplied by ``c_scale`` and its amax recorded.  ``backward``
    selected split accumulation in the reference's cuBLASLt call (backend.py:52); the MFMA
    kernel always accumulates in full fp32, so the flag changes nothing here.
    """
    if c.dtype in _FP8_DTYPES and (c_scale is None or c_amax is None):
        _fail("fp8_gmm_amd: an fp8 output needs c_scale and c_amax")
    grouped_gemm(
        [a], [b], [c], [a_scale_inv], [b_scale_inv],
        pre_gelu_outs=None if pre_gelu_out is None else [pre_gelu_out],
        c_scales=None if c_scale is None else [c_scale],
        c_amaxes=None if c_amax is None else [c_amax],
    )


def _group_sizes_list(group_sizes):
    if isinstance(group_sizes, torch.Tensor):
        if group_sizes.dim() != 1:
            _fail("fp8_gmm_amd: group_sizes must be 1-D")
        return [int(g) for g in group_sizes.tolist()]
    return [int(g) for g in group_sizes]


def fp8_gmm(a, b, group_sizes, a_scale_invs, b_scale_invs, c=None, c_dtype=torch.bfloat16, pre_gelu_out=None,
            c_scales=None, c_amaxes=None, backward=False, cutlass=False, b_transposed=False, dgelu_pre=None):
    """Grouped GEMM over row slices of ``a``: expert i multiplies rows
    ``[sum(group_sizes[:i]), sum(group_sizes[:i+1]))`` of ``a[tokens, k]`` with ``b[i][n, k]^T``.

    One persistent kernel launch for all experts.  ``cutlass=True`` reproduces the data
    flow of the reference's CUTLASS path (backend.py:78-82): an unscaled GEMM to bf16
    followed by ``multi_scale_mul`` (two roundings); the default applies the scales to
    the fp32 accumulator in the GEMM epilogue (one rounding), like its cuBLASLt path.
    Experts with zero rows are allowed.

    ``b_transposed=True`` (not in the reference): ``b`` is ``[experts, k, n]`` and expert i multiplies with
    ``b[i]`` as it stands.  That is a forward weight stack used by the data-gradient GEMM without the transposed
    copy the reference casts for it (grouped_linear.py:69-74,163); same results, bit for bit.

    ``dgelu_pre`` (not in the reference, which notes the missing fusion at grouped_mlp.py:252-253): a bf16
    ``[tokens, n]`` pre-GELU activation; the result is multiplied by ``dgelu_tanh(dgelu_pre)`` in the GEMM's epilogue
    before the one rounding to ``c``'s type.  With an fp8 ``c`` this is the fc2 data-gradient GEMM and the
    cast + dGELU pass behind it in one kernel; the product is formed from the fp32 accumulator, where the separate
    pass starts from the bf16-rounded gradient.
    """
    sizes = _group_sizes_list(group_sizes)
    e = len(sizes)
    if a.dim() != 2 or b.dim() != 3:
        _fail("fp8_gmm_amd: fp8_gmm expects a [tokens, k] and b [experts, n, k]")
    if not (a.is_contiguous() and b.is_contiguous()):
        _fail("fp8_gmm_amd: fp8_gmm expects contiguous a and b")
    tokens, k = a.shape
    if b.shape[0] != e or b.shape[1 if b_transposed else 2] != k:
        _fail("fp8_gmm_amd: b must be [len(group_sizes), n, k] with k == a.shape[1] ([.., k, n] when b_transposed)")
    if any(g < 0 for g in sizes) or sum(sizes) != tokens:
        _fail("fp8_gmm_amd: group_sizes must be non-negative and sum to a.shape[0]")
    nn = b.shape[2 if b_transposed else 1]
    if c is None:
        c = torch.empty(tokens, nn, device=a.device, dtype=c_dtype)
    if tuple(c.shape) != (tokens, nn) or not c.is_contiguous():
        _fail("fp8_gmm_amd: c must be a contiguous [tokens, n] tensor")
    fp8_out = c.dtype in _FP8_DTYPES
    if fp8_out and (c_scales is None or c_amaxes is None):
        _fail("fp8_gmm_amd: an fp8 output needs c_scales and c_amaxes")
    if cutlass and (c.dtype != torch.bfloat16 or pre_gelu_out is not None):
        _fail("fp8_gmm_amd: cutlass=True supports a bf16 output without GELU only")
    if pre_gelu_out is not None and (
        pre_gelu_out.dtype != torch.bfloat16 or tuple(pre_gelu_out.shape) != (tokens, nn)
        or not pre_gelu_out.is_contiguous()
    ):
        _fail("fp8_gmm_amd: pre_gelu_out must be a contiguous bf16 [tokens, n] tensor")
    if dgelu_pre is not None:
        if pre_gelu_out is not None or cutlass:
            _fail("fp8_gmm_amd: dgelu_pre excludes pre_gelu_out and cutlass=True")
        if dgelu_pre.dtype != torch.bfloat16 or tuple(dgelu_pre.shape) != (tokens, nn) or not dgelu_pre.is_contiguous():
            _fail("fp8_gmm_amd: dgelu_pre must be a contiguous bf16 [tokens, n] tensor")
    dev = _device_of([a, b, c, pre_gelu_out, dgelu_pre])

    starts = np.zeros(e + 1, dtype=np.int64)
    np.cumsum(np.asarray(sizes, dtype=np.int64), out=starts[1:])
    row0 = starts[:-1].astype(np.uint64)
    table = np.zeros(e, dtype=GEMM_PROBLEM)
    table["a"] = a.data_ptr() + row0 * np.uint64(k * a.element_size())
    table["b"] = b.data_ptr() + np.arange(e, dtype=np.uint64) * np.uint64(nn * k * b.element_size())
    table["c"] = c.data_ptr() + row0 * np.uint64(nn * c.element_size())
    if pre_gelu_out is not None:
        table["aux"] = pre_gelu_out.data_ptr() + row0 * np.uint64(nn * 2)
    if dgelu_pre is not None:
        table["aux"] = dgelu_pre.data_ptr() + row0 * np.uint64(nn * 2)
    table["m"] = np.asarray(sizes, dtype=np.int32)
    table["n"] = nn
    table["k"] = k
    table["lda"] = k
    table["ldb"] = nn if b_transposed else k
    table["ldc"] = nn
    if not cutlass:
        table["a_scale_inv"] = _scalar_ptrs(a_scale_invs, e, "a_scale_invs")
        table["b_scale_inv"] = _scalar_ptrs(b_scale_invs, e, "b_scale_invs")
    if fp8_out:
        table["c_scale"] = _scalar_ptrs(c_scales, e, "c_scales")
        table["c_amax"] = _scalar_ptrs(c_amaxes, e, "c_amaxes")
    _launch_gemm(table, a.dtype, b.dtype, c.dtype, pre_gelu_out is not None, dev,
                 (a, b, c, pre_gelu_out, dgelu_pre, a_scale_invs, b_scale_invs, c_scales, c_amaxes),
                 b_kmajor=b_transposed, dgelu=dgelu_pre is not None)
    if cutlass:
        multi_scale_mul(TensorBatch.rows_of(c, starts), a_scale_invs, b_scale_invs)
    return c
