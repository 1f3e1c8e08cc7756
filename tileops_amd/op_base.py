"""L2 op base: the host-side contract every op of this package follows.

Mirrors the reference's ``Op`` (src/tileops/ops/op_base.py:53-656) in what a caller and a backend can
observe: ``op(*tensors)`` settles the serving target once per instance and delegates to ``forward``;
``get_or_build_kernel`` is the single place where the in-tree implementation and an external target's
``build_kernel`` fork; ``select_kernel_key`` picks among in-tree kernels by asking each class whether it
serves the call; manifest-derived ``_validate_dtypes`` / ``eval_roofline`` / ``__manifest_param_names__``
are installed when a subclass is created.  Construction touches no device.
"""

from __future__ import annotations

import importlib
from typing import Any, Callable, Hashable, Mapping, Optional, Sequence

import torch

from .backend import (
    BUILTIN, BuildKernel, OpNotAvailableError, Target, TensorSpec, ensure_loaded, registered_kernel_builder,
    registered_targets, select_target,
)
from .manifest import try_load_entry

_UNRESOLVED = object()

_DTYPES = {
    "float16": torch.float16, "bfloat16": torch.bfloat16, "float32": torch.float32, "int32": torch.int32,
    "int64": torch.int64, "float8_e4m3fn": torch.float8_e4m3fn,
}


def _make_dtype_validator(entry: dict) -> Optional[Callable]:
    """Build ``_validate_dtypes(self, *tensors)`` from ``signature.inputs`` (+ ``dtype_combos``).

    Follows the rules the reference's codegen implements (src/tileops/ops/_dtype_codegen.py:145-297):
    a union ``"a | b"`` accepts any member, ``same_as(x)`` must equal input x's dtype, an
    ``optional: true`` input may be None, and when ``dtype_combos`` is present the tuple of dtypes of
    the inputs it names must be one of its rows.
    """
    sig = entry.get("signature") or {}
    inputs = sig.get("inputs")
    if not isinstance(inputs, dict) or not inputs:
        return None
    names = list(inputs)
    combos = sig.get("dtype_combos")

    def _validate_dtypes(self, *tensors: Optional[torch.Tensor]) -> None:
        if len(tensors) > len(names):
            raise ValueError(f"{type(self).__name__} takes {len(names)} tensor inputs, got {len(tensors)}")
        given = dict(zip(names, tensors))
        for name in names:
            spec = inputs[name]
            t = given.get(name)
            if t is None:
                if spec.get("optional"):
                    continue
                raise ValueError(f"{name} is required")
            rule = spec["dtype"]
            if rule.startswith("same_as("):
                other = rule[len("same_as("):-1]
                if given.get(other) is not None and t.dtype != given[other].dtype:
                    raise ValueError(f"Expected {name}.dtype {given[other].dtype} (same as {other}), got {t.dtype}")
            else:
                allowed = [_DTYPES[s.strip()] for s in rule.split("|")]
                if t.dtype not in allowed:
                    raise ValueError(f"Expected {name}.dtype in {allowed}, got {t.dtype}")
        if combos:
            keys = list(combos[0])
            got = tuple(given[k].dtype for k in keys)
            legal = {tuple(_DTYPES[row[k]] for k in keys) for row in combos}
            if got not in legal:
                raise ValueError(f"dtype combination {dict(zip(keys, got))} is not supported; supported: {sorted(map(str, legal))}")

    return _validate_dtypes


def _make_eval_roofline(entry: dict) -> Optional[Callable]:
    func_path = (entry.get("roofline") or {}).get("func")
    if not func_path:
        return None
    mod_name, _, fn_name = func_path.rpartition(".")

    def eval_roofline(self) -> tuple[int, int]:
        fn = getattr(importlib.import_module(mod_name), fn_name)
        return fn(self)

    return eval_roofline


class Op:
    """Base class of the package's ops."""

    #: Which set of kernels serves this instance: a target name, ``BUILTIN``, or None (decide from the device).
    target: Target = None
    _builder: object = _UNRESOLVED
    _settled_target: Target = None
    kernel_map: Optional[dict[str, type]] = None
    _overridden_keys: frozenset = frozenset()
    tune: bool = False
    dtype: Optional[torch.dtype] = None
    #: ``torch.library`` operators this op's call traces to under ``torch.compile(op, fullgraph=True)``
    #: (reference: ``Op.compile_op_names``, src/tileops/ops/op_base.py:140-147).
    compile_op_names: tuple = ()

    def __init_subclass__(cls, **kwargs: object) -> None:
        super().__init_subclass__(**kwargs)
        entry = try_load_entry(cls.__name__)
        if entry is None or entry.get("status") == "spec-only":
            return
        if "_validate_dtypes" not in cls.__dict__:
            fn = _make_dtype_validator(entry)
            if fn is not None:
                cls._validate_dtypes = fn
        if "eval_roofline" not in cls.__dict__:
            fn = _make_eval_roofline(entry)
            if fn is not None:
                cls.eval_roofline = fn
        params = (entry.get("signature") or {}).get("params")
        if isinstance(params, dict):
            cls.__manifest_param_names__ = tuple(params)

    # -- to be supplied by concrete ops ---------------------------------------------------------------
    @property
    def default_kernel_map(self) -> dict[str, type]:
        raise NotImplementedError("Op must implement default_kernel_map")

    def _infer_output_shapes(self, **shape_kwargs: tuple[int, ...]) -> dict[str, tuple[int, ...]]:
        raise NotImplementedError("_infer_output_shapes must be implemented by the concrete Op subclass")

    def _validate_dtypes(self, *args: torch.Tensor) -> None:
        raise NotImplementedError("_validate_dtypes must be implemented by the concrete Op subclass")

    def eval_roofline(self) -> tuple[int, int]:
        raise NotImplementedError("eval_roofline must be implemented by the concrete Op subclass")

    def forward(self, *args: object, **kwargs: object) -> Any:
        raise NotImplementedError("forward method is not implemented")

    # -- kernel map -------------------------------------------------------------------------------------
    def dispatch_kernel(self, kernel_map: Optional[dict[str, type]] = None) -> None:
        """Discover backends (before any call) and install the kernel map, overrides winning per key."""
        ensure_loaded()
        defaults = self.default_kernel_map
        override = dict(kernel_map) if kernel_map else {}
        if not defaults:
            self.kernel_map = override
            self._overridden_keys = frozenset(override)
            return
        self.kernel_map = {name: override.get(name, cls) for name, cls in defaults.items()}
        self._overridden_keys = frozenset(override) & frozenset(self.kernel_map)

    def select_kernel_key(self, keys: tuple[str, ...], call: object) -> str:
        """The one key among *keys* whose kernel class serves *call*.

        Each class answers for itself through ``refusal(call)``; a class marked ``general`` runs only where
        no specialised one applies; a caller-supplied replacement is never silently bypassed
        (reference rule: src/tileops/ops/op_base.py:238-301).
        """
        applicable, rejected, refused_overrides = [], [], []
        for key in keys:
            cls = (self.kernel_map or {}).get(key)
            if cls is None:
                continue
            why = cls.refusal(call)
            if why is None:
                applicable.append(key)
                continue
            rejected.append(f"{key} ({cls.__name__}: {why})")
            if key in self._overridden_keys:
                refused_overrides.append(rejected[-1])
        chosen = [k for k in applicable if not self.kernel_map[k].general] or applicable
        if len(chosen) == 1:
            if refused_overrides and chosen[0] not in self._overridden_keys:
                raise ValueError(
                    "the kernel supplied for " + "; ".join(refused_overrides)
                    + f" — selection does not fall back to the shipped '{chosen[0]}' when a replacement is in force. Call: {call}"
                )
            return chosen[0]
        if not chosen:
            lead = "the kernel supplied for " + "; ".join(refused_overrides) + ", and " if refused_overrides else ""
            raise ValueError(
                lead + "no implementation serves this call: "
                + "; ".join(rejected or ["no implementation is installed"]) + f". Call: {call}"
            )
        raise ValueError(
            f"dispatch is ambiguous: {', '.join(chosen)} all serve this call, so none is the answer. "
            f"Implementations of one key must serve disjoint regions, and at most one may be general. Call: {call}"
        )

    # -- target settling ------------------------------------------------------------------------------
    def __call__(self, *args: object, **kwargs: object) -> Any:
        if self._builder is not _UNRESOLVED:
            return self.forward(*args, **kwargs)
        self._resolve_builder(args, kwargs)
        try:
            return self.forward(*args, **kwargs)
        except Exception:
            self._unsettle()  # a call that fails aims nothing
            raise

    def _unsettle(self) -> None:
        self._builder = _UNRESOLVED
        self._settled_target = None
        self._kernel_roles = {}

    @staticmethod
    def _first_tensor_device(args: tuple, kwargs: dict) -> Optional[torch.device]:
        for a in list(args) + list(kwargs.values()):
            if isinstance(a, torch.Tensor):
                return a.device
        return None

    def _resolve_builder(self, args: tuple, kwargs: dict) -> None:
        device = self._first_tensor_device(args, kwargs)
        target = select_target(self.target, device)
        if target is None:
            self._settled_target = None
            if device is not None:
                self._builder = None
            return
        if target is BUILTIN:
            self._settled_target, self._builder = BUILTIN, None
            return
        builder = registered_kernel_builder(type(self).__name__, target)
        if builder is None:
            raise OpNotAvailableError(
                f"target {target!r} registers no kernel builder for {type(self).__name__}; targets that do: "
                f"{registered_targets(type(self).__name__)}. There is no fall back to the in-tree implementation."
            )
        self._settled_target, self._builder = target, builder

    # -- the in-tree / external fork -------------------------------------------------------------------
    def get_or_build_kernel(self, name: str, inputs: Sequence[Optional[torch.Tensor]], *, key: Hashable = None,
                            build: Optional[Callable[[], object]] = None) -> object:
        """The kernel for this call, built once.  In-tree entries are keyed by *key*; an external target's by
        ``(device, (dtype, shape) per input)`` because this layer cannot know what that target specialises on."""
        roles = getattr(self, "_kernel_roles", None)
        if roles is None:
            roles = self._kernel_roles = {}
        entries = roles.setdefault(name, {})
        settled_here = self._builder is _UNRESOLVED
        if settled_here:
            self._resolve_builder(tuple(inputs), {})
        try:
            builder = self._builder
            if builder is None or builder is _UNRESOLVED:
                if build is None:
                    raise OpNotAvailableError(
                        f"{type(self).__name__} has no in-tree implementation for {name!r}; known targets for this op: "
                        f"{registered_targets(type(self).__name__)}"
                    )
                if key not in entries:
                    entries[key] = build()
                return entries[key]
            specs = tuple(None if t is None else TensorSpec.of(t) for t in inputs)
            present = [s for s in specs if s is not None]
            if not present:
                raise OpNotAvailableError(
                    f"target {self._settled_target!r} serves {type(self).__name__}, but its {name!r} call site hands over no tensors"
                )
            signature = (present[0].device,) + tuple(None if s is None else (s.dtype, s.shape) for s in specs)
            if signature not in entries:
                entries[signature] = self._build_external(builder, name, specs)
            return entries[signature]
        except Exception:
            if settled_here:
                self._unsettle()
            raise

    def _build_external(self, builder: BuildKernel, name: str, specs: tuple) -> object:
        kernel = builder(*specs, **self._manifest_params())
        if not callable(kernel):
            raise OpNotAvailableError(
                f"target {self._settled_target!r} built {kernel!r} for {type(self).__name__}.{name}, which is not callable"
            )
        return kernel

    def _manifest_params(self) -> dict[str, object]:
        """Manifest params by name with the values this instance settled on (defaults already resolved)."""
        values = {}
        for param in getattr(self, "__manifest_param_names__", None) or ():
            try:
                values[param] = getattr(self, param)
            except AttributeError:
                raise AttributeError(
                    f"{type(self).__name__} declares manifest param {param!r} but keeps no attribute of that name"
                ) from None
        return values

    def built_kernels(self, role: str) -> Mapping[Hashable, object]:
        return dict((getattr(self, "_kernel_roles", None) or {}).get(role, {}))
