"""Programmatic access to the op manifest (YAML files in this package directory).

Same entry points as the reference loader (src/tileops/manifest/__init__.py:28-92):
``manifest_files()``, ``load_manifest()``, ``try_load_entry(op)``, ``load_workloads(op)``.
"""

from __future__ import annotations

import functools
from pathlib import Path
from typing import Any, Optional

import yaml

_DIR = Path(__file__).resolve().parent


def manifest_files() -> list[Path]:
    return sorted(p for p in _DIR.iterdir() if p.is_file() and p.suffix == ".yaml")


@functools.lru_cache(maxsize=1)
def load_manifest() -> dict[str, Any]:
    """All ops of all files merged; a name defined twice is an error."""
    merged: dict[str, Any] = {}
    seen_in: dict[str, str] = {}
    for path in manifest_files():
        ops = yaml.safe_load(path.read_text(encoding="utf-8")) or {}
        if not isinstance(ops, dict):
            raise ValueError(f"manifest file {path.name} must map op name -> entry, got {type(ops).__name__}")
        for name, entry in ops.items():
            if name in merged:
                raise ValueError(f"duplicate op {name!r} in {path.name} (already defined in {seen_in[name]})")
            merged[name] = entry
            seen_in[name] = path.name
    return merged


def try_load_entry(op_name: str) -> Optional[dict[str, Any]]:
    """The entry for *op_name*, or None on any failure (an unreadable manifest never blocks class creation)."""
    try:
        entry = load_manifest().get(op_name)
    except Exception:  # noqa: BLE001
        return None
    return entry if isinstance(entry, dict) else None


def load_workloads(op_name: str) -> list[dict[str, Any]]:
    ops = load_manifest()
    if op_name not in ops:
        raise KeyError(f"op '{op_name}' not found in ops manifest")
    return ops[op_name]["workloads"]
