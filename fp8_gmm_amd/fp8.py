"""Per-tensor delayed-scaling FP8 metadata for the grouped modules.

The reference inherits this machinery from TransformerEngine
(``TransformerEngineBaseModule.prepare_forward`` / ``fp8_meta``, ``fp8_autocast``,
``recipe.DelayedScaling``, ``get_fp8_te_dtype``; call sites grouped_linear.py:4-5,19,124,186,206,
grouped_mlp.py:4-5,28,178,328,349, utils.py:78-96, example.py:156,159).  TransformerEngine
is not a dependency here; this module provides the same names with the same
meaning, sized for what the grouped modules use:

* ``fp8_meta["scaling_fwd"]`` has 3 slots per GEMM (input, weight, output) and
  ``fp8_meta["scaling_bwd"]`` 2 (grad_output, grad_input); each holds ``scale``,
  ``scale_inv`` (fp32 ``[slots]``) and ``amax_history`` (fp32 ``[history, slots]``),
  with the kernels writing amax into ``amax_history[0]``.
* Update rule (applied at the start of a forward pass, from the second pass on):
      amax      = max(amax_history, dim=0)        ("max")  or amax_history[0] ("most_recent")
      new_scale = (fp8_max / amax) / 2**margin    where amax is finite and > 0, else the old scale
      scale_inv = 1 / new_scale
      amax_history = roll(amax_history, -1, dim=0);  amax_history[0] = 0
  fp8_max is 448 for e4m3 and 57344 for e5m2.  HYBRID means e4m3 for forward tensors
  and e5m2 for gradients.
* FP8 weight caching (``forward(..., is_first_microbatch=True / False)``, TransformerEngine's convention, which
  the reference stubs out at grouped_linear.py:200-202 and grouped_mlp.py:343-345): the first micro-batch of a
  step casts the weights into buffers the module keeps, the later ones reuse them and skip the cast.  On those
  later passes the update leaves the weights' ``scale_inv`` alone (the cached bytes were cast with it) and their
  amax slots receive nothing.  ``None`` (the default, and all the reference supports) casts on every pass.
* Both directions are updated.  (The reference never enters TransformerEngine's
  backward context, so its gradient scales stay at their initial value of 1; updating
  them is a deliberate difference - e5m2 gradients need real scales.)

No test vector of the reference pins TransformerEngine's update rule; the rule
above is this package's own statement of it.
"""
import contextlib
import threading
from dataclasses import dataclass
from enum import Enum

import numpy as np
import torch

from .utils import DType

FP8_MAX = {DType.kFloat8E4M3: 448.0, DType.kFloat8E5M2: 57344.0}


class Format(Enum):
    E4M3 = "e4m3"
    E5M2 = "e5m2"
    HYBRID = "hybrid"


@dataclass
class DelayedScaling:
    """Delayed-scaling recipe (same fields and defaults the reference's example uses, example.py:156)."""

    margin: int = 0
    interval: int = 1
    fp8_format: Format = Format.HYBRID
    amax_history_len: int = 1024
    amax_compute_algo: str = "max"

    def __post_init__(self):
        if self.amax_compute_algo not in ("max", "most_recent"):
            raise ValueError(f"unsupported amax_compute_algo {self.amax_compute_algo!r}")
        if self.amax_history_len < 1:
            raise ValueError("amax_history_len must be >= 1")
        if self.interval < 1:
            raise ValueError("interval must be >= 1")


class recipe:  # noqa: N801 - namespace with the spelling user code already has (`recipe.DelayedScaling`)
    DelayedScaling = DelayedScaling
    Format = Format


def get_fp8_te_dtype(fp8_recipe, fprop_tensor=True):
    """fp8 type of forward (``fprop_tensor``) or gradient tensors under a recipe."""
    if fp8_recipe.fp8_format == Format.E4M3 or (fp8_recipe.fp8_format == Format.HYBRID and fprop_tensor):
        return DType.kFloat8E4M3
    return DType.kFloat8E5M2


class _State(threading.local):
    def __init__(self):
        self.enabled = False
        self.recipe = None


_STATE = _State()


@contextlib.contextmanager
def fp8_autocast(enabled=True, fp8_recipe=None):
    """Selects the recipe used by modules called inside the block."""
    prev = (_STATE.enabled, _STATE.recipe)
    _STATE.enabled = enabled
    _STATE.recipe = (fp8_recipe or DelayedScaling()) if enabled else None
    try:
        yield
    finally:
        _STATE.enabled, _STATE.recipe = prev


def current_recipe():
    return _STATE.recipe if _STATE.enabled else None


class Fp8MetaTensors:
    """scale / scale_inv / amax_history of one direction."""

    def __init__(self, slots, history_len, device):
        self.scale = torch.ones(slots, dtype=torch.float32, device=device)
        self.scale_inv = torch.ones(slots, dtype=torch.float32, device=device)
        self.amax_history = torch.zeros(history_len, slots, dtype=torch.float32, device=device)

    def state(self):
        return {"scale": self.scale, "scale_inv": self.scale_inv, "amax_history": self.amax_history}

    def load_state(self, state):
        self.scale.copy_(state["scale"])
        self.scale_inv.copy_(state["scale_inv"])
        self.amax_history.copy_(state["amax_history"])


def amax_and_scale_update(meta, fp8_max, fp8_recipe, keep_scale_inv=None):
    """Delayed-scaling update of one direction, in place (rule in the module docstring).
    ``keep_scale_inv=(period, phase)``: ``scale_inv`` of the slots with ``slot % period == phase`` is not touched.

    Scaling state that lives on the GPU is updated by one fused kernel
    (``backend.delayed_scaling_update``); the torch statement of the rule below serves CPU tensors
    (host-side tests of the bookkeeping) and is what the kernel is checked against bit for bit."""
    hist = meta.amax_history
    most_recent = fp8_recipe.amax_compute_algo != "max"
    if hist.is_cuda and float(fp8_recipe.margin) == int(fp8_recipe.margin):
        from . import backend

        backend.delayed_scaling_update(hist, meta.scale, meta.scale_inv, fp8_max, int(fp8_recipe.margin), most_recent,
                                       keep_scale_inv)
        return
    amax = hist[0].clone() if most_recent else hist.max(dim=0).values
    sf = (fp8_max / amax) / (2.0 ** fp8_recipe.margin)
    ok = (amax > 0) & torch.isfinite(amax)
    meta.scale.copy_(torch.where(ok, sf, meta.scale))
    new_inv = 1.0 / meta.scale
    if keep_scale_inv is not None:
        kept = torch.arange(meta.scale.numel(), device=meta.scale.device) % keep_scale_inv[0] == keep_scale_inv[1]
        new_inv = torch.where(kept, meta.scale_inv, new_inv)
    meta.scale_inv.copy_(new_inv)
    if hist.shape[0] > 1:
        hist.copy_(torch.roll(hist, -1, 0))
    hist[0].zero_()


class Fp8WeightCache:
    """fp8 copies (row-major and transposed) of one ``[E, N, K]`` weight stack, kept across micro-batches."""

    def __init__(self):
        self.fp8 = None      # [E, N, K]
        self.fp8_t = None    # [E, K, N]
        self.valid = False   # fp8 holds a cast of the weights
        self.valid_t = False  # fp8_t does too

    def buffers(self, weight, dtype, with_transpose=True):
        if self.fp8 is None or self.fp8.shape != weight.shape or self.fp8.dtype != dtype \
                or self.fp8.device != weight.device:
            self.fp8 = torch.empty(weight.shape, dtype=dtype, device=weight.device)
            self.fp8_t = None
            self.valid = self.valid_t = False
        if with_transpose and self.fp8_t is None:
            e, n, k = weight.shape
            self.fp8_t = torch.empty(e, k, n, dtype=dtype, device=weight.device)
            self.valid_t = False
        return self.fp8, self.fp8_t

    def require(self, transposed):
        if not self.valid or (transposed and not self.valid_t):
            raise RuntimeError(
                "is_first_microbatch=False, but no earlier pass with is_first_microbatch=True has cast the "
                "weights" + (" with their transposes (it ran without gradients)" if self.valid else ""))


class Fp8GroupedModuleBase(torch.nn.Module):
    """The slice of ``TransformerEngineBaseModule`` the grouped modules rely on."""

    FWD_SLOTS_PER_GEMM = 3
    BWD_SLOTS_PER_GEMM = 2
    WEIGHT_SLOT = 1  # position of a GEMM's weight among its forward slots (input, weight, output)

    def __init__(self):
        super().__init__()
        self.fp8_meta = {}
        self._fp8_steps = 0
        self._weight_caches = []  # Fp8WeightCache objects of the subclass; dropped whenever the scales are replaced
        self._ahead = None        # fp8 weights that cast_weights_ahead() made for the next forward pass

    def _invalidate_weight_caches(self):
        for cache in self._weight_caches:
            cache.valid = cache.valid_t = False

    def _init_fp8_meta(self, fp8_recipe, num_gemms, device):
        meta = self.fp8_meta
        same = (
            meta.get("num_gemms") == num_gemms
            and meta.get("recipe") == fp8_recipe
            and "scaling_fwd" in meta
            and meta["scaling_fwd"].scale.device == device
        )
        if same:
            return
        meta["recipe"] = fp8_recipe
        meta["num_gemms"] = num_gemms
        meta["scaling_fwd"] = Fp8MetaTensors(num_gemms * self.FWD_SLOTS_PER_GEMM, fp8_recipe.amax_history_len, device)
        meta["scaling_bwd"] = Fp8MetaTensors(num_gemms * self.BWD_SLOTS_PER_GEMM, fp8_recipe.amax_history_len, device)
        meta["fp8_max_fwd"] = FP8_MAX[get_fp8_te_dtype(fp8_recipe, True)]
        meta["fp8_max_bwd"] = FP8_MAX[get_fp8_te_dtype(fp8_recipe, False)]
        self._fp8_steps = 0
        self._invalidate_weight_caches()

    @contextlib.contextmanager
    def prepare_forward(self, inp, is_first_microbatch, num_gemms=1):
        """Makes ``self.fp8_meta`` ready for a forward pass of ``num_gemms`` GEMMs.

        Outside ``fp8_autocast`` the default recipe is used (the modules are FP8-only).
        In training mode every pass after the first starts with the delayed-scaling
        update of both directions, every ``recipe.interval`` passes.  ``is_first_microbatch=False``
        (cached fp8 weights are reused) keeps the weights' ``scale_inv`` out of that update.
        """
        update_weights = is_first_microbatch is None or bool(is_first_microbatch)
        fp8_recipe = current_recipe() or self.fp8_meta.get("recipe") or DelayedScaling()
        self._init_fp8_meta(fp8_recipe, num_gemms, inp.device)
        self._apply_pending_state()
        if self.training and torch.is_grad_enabled():
            if self._fp8_steps > 0 and self._fp8_steps % fp8_recipe.interval == 0:
                fwd, bwd = self.fp8_meta["scaling_fwd"], self.fp8_meta["scaling_bwd"]
                keep = None if update_weights else (self.FWD_SLOTS_PER_GEMM, self.WEIGHT_SLOT)
                with torch.no_grad():
                    if fwd.amax_history.is_cuda and float(fp8_recipe.margin) == int(fp8_recipe.margin):
                        # both directions in one kernel launch (the rule is amax_and_scale_update's)
                        from . import backend

                        margin, recent = int(fp8_recipe.margin), fp8_recipe.amax_compute_algo != "max"
                        backend.delayed_scaling_updates([
                            (fwd.amax_history, fwd.scale, fwd.scale_inv, self.fp8_meta["fp8_max_fwd"], margin, recent, keep),
                            (bwd.amax_history, bwd.scale, bwd.scale_inv, self.fp8_meta["fp8_max_bwd"], margin, recent)])
                    else:
                        amax_and_scale_update(fwd, self.fp8_meta["fp8_max_fwd"], fp8_recipe, keep)
                        amax_and_scale_update(bwd, self.fp8_meta["fp8_max_bwd"], fp8_recipe)
            self._fp8_steps += 1
        yield

    def _cast_ahead(self, weights_and_groups):
        """The part of a forward pass that needs no group sizes, run now: the delayed-scaling update and the cast of
        the weight stacks ``[(weight, Fp8TensorType of its scaling slots), ...]`` into fp8 tensors of their own, one
        launch.  Returns False (and does nothing) where the pass would use the reference's transposed layout."""
        from .backend import TensorBatch, multi_quantize
        from .grouped_linear import stage_weight_cast
        from .utils import Fp8MetaWrapper, MetaTensorType, to_torch_dtype

        first = weights_and_groups[0][0]
        if self.fp8_meta.get("reference_layout") or not first.is_cuda \
                or any(w.size(1) % 16 or w.size(2) % 16 or not w.is_contiguous() for w, _ in weights_and_groups):
            return False
        self._ahead = None
        with self.prepare_forward(first, None, self.num_groups * len(weights_and_groups)):
            meta = Fp8MetaWrapper(self.num_groups, self.fp8_meta)
            fp8_dtype = to_torch_dtype(get_fp8_te_dtype(self.fp8_meta["recipe"], fprop_tensor=True))
            caches = tuple(Fp8WeightCache() for _ in weights_and_groups)
            plain, with_t = ([], [], [], []), ([], [], [], [], [])
            for (weight, group), cache in reversed(list(zip(weights_and_groups, caches))):
                stage_weight_cast(weight, fp8_dtype, False, False, cache, True,
                                  meta.get_meta_pointers(group, MetaTensorType.kScale),
                                  meta.get_meta_pointers(group, MetaTensorType.kAmax), plain, with_t)
            with torch.no_grad():
                multi_quantize(TensorBatch.concat(plain[0]), TensorBatch.concat(plain[1]), np.concatenate(plain[2]),
                               np.concatenate(plain[3]))
        self._ahead = caches
        return True

    def _take_ahead(self, is_first_microbatch):
        ahead, self._ahead = self._ahead, None
        if ahead is not None and is_first_microbatch is not None:
            raise RuntimeError("cast_weights_ahead() has cast this pass's weights: call forward without "
                               "is_first_microbatch")
        return ahead

    # checkpointing of the scaling state (TransformerEngine exposes it the same way)
    def get_extra_state(self):
        if "scaling_fwd" not in self.fp8_meta:
            return None
        return {
            "num_gemms": self.fp8_meta["num_gemms"],
            "steps": self._fp8_steps,
            "scaling_fwd": {k: v.detach().cpu() for k, v in self.fp8_meta["scaling_fwd"].state().items()},
            "scaling_bwd": {k: v.detach().cpu() for k, v in self.fp8_meta["scaling_bwd"].state().items()},
        }

    def set_extra_state(self, state):
        if not state:
            return
        self._pending_extra_state = state

    def _apply_pending_state(self):
        state = getattr(self, "_pending_extra_state", None)
        if state is None or "scaling_fwd" not in self.fp8_meta:
            return
        self._pending_extra_state = None
        fwd, bwd = self.fp8_meta["scaling_fwd"], self.fp8_meta["scaling_bwd"]
        if (
            state["num_gemms"] != self.fp8_meta["num_gemms"]
            or state["scaling_fwd"]["amax_history"].shape != fwd.amax_history.shape
        ):
            raise RuntimeError("saved FP8 scaling state does not match this module's recipe / expert count")
        fwd.load_state(state["scaling_fwd"])
        bwd.load_state(state["scaling_bwd"])
        self._fp8_steps = state["steps"]
        self._invalidate_weight_caches()
