"""Backend seam: how a set of kernels ("target") announces itself and how an op finds it.

Same protocol as the reference's ``tileops.backend`` package
(src/tileops/backend/__init__.py:1-36, protocol.py:10-53, registry.py:42-156, dispatch.py:12-129,
errors.py:6-23), so a backend written against one registers unchanged against the other:

    register_detector(target, detect)                      # "is this device mine?"  -> bool, never raises
    register_kernel_builder(op, target, build_kernel)      # build_kernel(*TensorSpec, **manifest_params) -> callable

A target is chosen once per op instance: explicit ``target=`` first, then the process default
(``set_default_target``), then detection from the first tensor's device.  ``None`` means "no external
target": the op runs its in-tree HIP kernels.  There is never a silent fall-back from a selected target to
the in-tree kernels.

Backends are discovered through the entry-point group ``tileops_amd.backends`` (value = a module whose
import performs the registration), loaded once, all-or-nothing per backend.
"""

from __future__ import annotations

import threading
import traceback
import warnings
from importlib.metadata import entry_points
from typing import Callable, Final, NamedTuple, Optional, Union

import torch

__all__ = [
    "BUILTIN", "AmbiguousTargetError", "BackendError", "BuildKernel", "KernelResult", "OpNotAvailableError",
    "Target", "TensorSpec", "UnknownTargetError", "default_target", "load_failures", "register_detector",
    "register_kernel_builder", "registered_targets", "set_default_target",
]

ENTRY_POINT_GROUP = "tileops_amd.backends"


# --- errors ------------------------------------------------------------------------------------------
class BackendError(Exception):
    """Base class of everything this layer raises."""


class UnknownTargetError(BackendError):
    """A target was named that nothing registered."""


class AmbiguousTargetError(BackendError):
    """Two or more detectors claimed one device."""


class OpNotAvailableError(BackendError):
    """The selected target cannot serve the op; there is no falling back to another implementation."""


# --- protocol types ------------------------------------------------------------------------------------
class TensorSpec(NamedTuple):
    """A tensor's device, dtype and shape without the tensor; what ``build_kernel`` is described with."""

    device: torch.device
    dtype: torch.dtype
    shape: tuple[int, ...]

    @staticmethod
    def of(tensor: torch.Tensor) -> "TensorSpec":
        return TensorSpec(tensor.device, tensor.dtype, tuple(tensor.shape))


KernelResult = Union[torch.Tensor, tuple[torch.Tensor, ...], None]
BuildKernel = Callable[..., Callable[..., KernelResult]]
DetectFn = Callable[[torch.device], bool]


class _Builtin:
    __slots__ = ()

    def __repr__(self) -> str:
        return "BUILTIN"


#: Request the in-tree implementation whatever is installed.  Compared by identity; not a target name.
BUILTIN: Final = _Builtin()
Target = Union[str, _Builtin, None]


# --- registry ------------------------------------------------------------------------------------------
class _State(NamedTuple):
    detectors: dict
    builders: dict
    failures: list
    default: Target


_lock = threading.RLock()
_detectors: dict[str, DetectFn] = {}
_builders: dict[tuple[str, str], BuildKernel] = {}
_failures: list[str] = []
_default: Target = None
_loaded = False
_discovering = threading.local()


def _name_of(fn: Callable) -> str:
    return f"{getattr(fn, '__module__', '?')}.{getattr(fn, '__qualname__', repr(fn))}"


def register_detector(target: str, detect: DetectFn) -> None:
    """Record how *target* recognises its devices.  One detector per target; a second is a misinstall."""
    with _lock:
        if target in _detectors:
            raise BackendError(
                f"target {target!r} already has detector {_name_of(_detectors[target])}; {_name_of(detect)} cannot replace it."
            )
        _detectors[target] = detect


def register_kernel_builder(op: str, target: str, build_kernel: BuildKernel) -> None:
    """Record how *target* builds a kernel for the op whose manifest key is *op*.  Must be lazy."""
    with _lock:
        if (op, target) in _builders:
            raise BackendError(
                f"{(op, target)} is already registered to {_name_of(_builders[(op, target)])}; "
                f"{_name_of(build_kernel)} cannot take it. A target belongs to one distribution."
            )
        _builders[(op, target)] = build_kernel


def snapshot() -> _State:
    """Copy of the registry, for tests and for all-or-nothing backend loading."""
    with _lock:
        return _State(dict(_detectors), dict(_builders), list(_failures), _default)


def restore(state: _State) -> None:
    global _default
    with _lock:
        _detectors.clear()
        _detectors.update(state.detectors)
        _builders.clear()
        _builders.update(state.builders)
        _failures[:] = state.failures
        _default = state.default


def _known() -> set[str]:
    return set(_detectors) | {t for _, t in _builders}


def _suffix() -> str:
    return f" ({len(_failures)} backend(s) failed to load; see load_failures())" if _failures else ""


def ensure_loaded() -> None:
    """Import every declared backend module once.  A backend that raises is rolled back and recorded."""
    global _loaded
    if _loaded or getattr(_discovering, "on", False):
        return
    with _lock:
        if _loaded:
            return
        _discovering.on = True
        new_failures = []
        try:
            for ep in sorted(entry_points(group=ENTRY_POINT_GROUP), key=lambda e: (e.name, e.value)):
                before = snapshot()
                try:
                    ep.load()
                except Exception as exc:  # noqa: BLE001 - one broken plug-in must not take the rest down
                    restore(before)
                    why = "".join(traceback.format_exception_only(type(exc), exc)).strip()
                    _failures.append(f"{ep.name} ({ep.value}): {why}")
                    new_failures.append(_failures[-1])
                except BaseException:
                    restore(before)
                    raise
            _loaded = True
        finally:
            _discovering.on = False
    for f in new_failures:
        warnings.warn(f"backend failed to load and was skipped: {f} See load_failures().", RuntimeWarning, stacklevel=3)


# --- dispatch ------------------------------------------------------------------------------------------
def detect_target(device: torch.device) -> Optional[str]:
    """The one target whose detector claims *device*, or None when no backend does."""
    ensure_loaded()
    claimed = []
    for target, detect in list(_detectors.items()):
        try:
            if detect(device):
                claimed.append(target)
        except Exception as exc:
            raise BackendError(
                f"detector for target {target!r} ({_name_of(detect)}) raised on device {device}: {exc!r}. "
                f"A detector returns False for devices it does not serve.{_suffix()}"
            ) from exc
    if len(claimed) > 1:
        raise AmbiguousTargetError(f"device {device} is claimed by {sorted(claimed)}; pass target= to choose{_suffix()}")
    return claimed[0] if claimed else None


def select_target(requested: Target, device: Optional[torch.device]) -> Target:
    """requested -> process default -> detection.  Returns a name, BUILTIN, or None (in-tree by default)."""
    ensure_loaded()
    if requested is not None:
        if requested is not BUILTIN and requested not in _known():
            raise UnknownTargetError(
                f"no backend registered target {requested!r}; known targets: {sorted(_known())}{_suffix()}"
            )
        return requested
    if _default is not None:
        return _default
    if device is None:
        return None
    return detect_target(device)


def registered_kernel_builder(op: str, target: str) -> Optional[BuildKernel]:
    ensure_loaded()
    return _builders.get((op, target))


def registered_targets(op: Optional[str] = None) -> list[str]:
    """Targets that registered a builder for *op*; every known target when *op* is None."""
    ensure_loaded()
    if op is None:
        return sorted(_known())
    return sorted(t for name, t in _builders if name == op)


def set_default_target(target: Target) -> None:
    """Route ops constructed without ``target=`` to *target*; None restores detection, BUILTIN forces in-tree."""
    global _default
    ensure_loaded()
    if target is not None and target is not BUILTIN and target not in _known():
        raise UnknownTargetError(f"no backend registered target {target!r}; known targets: {sorted(_known())}{_suffix()}")
    _default = target


def default_target() -> Target:
    return _default


def load_failures() -> tuple[str, ...]:
    """One line per backend that failed to import and was skipped."""
    ensure_loaded()
    return tuple(_failures)
