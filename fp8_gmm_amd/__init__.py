"""MI355X-native FP8 grouped GEMM for MoE expert layers.

Drop-in for the Python surface of centwang/fp8_gmm (``fp8_gmm/__init__.py:1-3`` imports the
same three submodules): ``backend`` entry points, ``GroupedLinear`` and ``GroupedMlp``;
``moe_ops`` / ``moe`` add the token routing and the routed layers of the reference's example.
Importing the package loads the HIP shared library and fails if it is not built.
"""
from . import backend  # noqa: F401  (loads libfp8gmm_hip.so)
from . import grouped_linear, grouped_mlp, moe, moe_ops  # noqa: F401
from .fp8 import DelayedScaling, Format, fp8_autocast, recipe  # noqa: F401
from .grouped_linear import GroupedLinear  # noqa: F401
from .grouped_mlp import GroupedMlp  # noqa: F401
