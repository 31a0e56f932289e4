"""torch bindings: Genred, KernelSolve, LazyTensor (Vi, Vj, Pm), generic_* shortcuts and cluster helpers."""
from . import cluster  # noqa: F401
from .generic_ops import generic_argkmin, generic_argmin, generic_logsumexp, generic_sum  # noqa: F401
from .generic_red import Genred  # noqa: F401
from .lazytensor import LazyTensor, Pm, Vi, Vj  # noqa: F401
from .operations import KernelSolve  # noqa: F401
