"""Per-op timer hook of the layer classes.

The reference wraps every layer op in ``CudaTimer(name, layer_id=...)``
(sarathi/metrics/cuda_timer.py:10-54; e.g. layers/layernorm.py:29-32), a context manager that
reports the op's device time to its metrics store under the operation name.  The metrics store is
not part of this library; the layers here keep the labels and enter whatever context manager a host
installs with :func:`set_op_timer_factory` (called as ``factory(name, layer_id)``), so the
reference's timers -- or any other -- can be attached at the same places.  Without a factory, or
for an op without a name, nothing is timed and nothing is synchronised.
"""
import contextlib
from typing import Callable, ContextManager, Optional

_factory: Optional[Callable[[str, Optional[int]], ContextManager]] = None
_NULL = contextlib.nullcontext()


def set_op_timer_factory(factory: Optional[Callable[[str, Optional[int]], ContextManager]]) -> None:
    """Install (or with ``None`` remove) the factory of per-op timers.  Layers built afterwards use it."""
    global _factory
    _factory = factory


def op_timer(name: Optional[str], layer_id: Optional[int] = None) -> ContextManager:
    """The timer a layer enters around its op: the installed factory's, or a no-op."""
    if name is None or _factory is None:
        return _NULL
    return _factory(name, layer_id)
