"""Backend registration: target ``"mi355x"`` for the paged GQA decode ops.

This module is what a ``tileops.backends`` entry point names
(``[project.entry-points."tileops.backends"] mi355x = "tileops_amd.tileops_plugin"``): importing it registers a
device detector and lazy kernel builders with the reference's registry
(src/tileops/backend/registry.py:42-84) when TileOPs is installed.  ``register(into=...)`` performs the same
registration against any module exposing ``register_detector`` / ``register_kernel_builder`` -- e.g. this
package's own ``tileops_amd.backend``.

``build_kernel`` follows the protocol (src/tileops/backend/__init__.py:21-26, ops/op_base.py:418): one
``TensorSpec`` per manifest input in order (``None`` for an absent optional input), then the manifest params
by keyword, with ``sm_scale`` / ``softcap`` already resolved to numbers.  Nothing is compiled or loaded at
import time; the HIP library is opened on the first build.
"""

from __future__ import annotations

from typing import Any, Callable, Optional

import torch

TARGET = "mi355x"
OP_SINGLE = "GroupedQueryAttentionDecodePagedWithKVCacheFwdOp"
OP_MULTI = "GroupedQueryAttentionMultiTokenDecodePagedWithKVCacheFwdOp"


def detect(device: torch.device) -> bool:
    """True iff *device* is a ROCm gfx950 GPU.  ROCm reports ``device.type == "cuda"``, so the architecture
    name decides."""
    from . import native

    try:
        return native.is_gfx950(device)
    except Exception:  # noqa: BLE001 - a detector answers False, it never raises
        return False


def _build(q: Any, k: Any, v: Any, real_seqlen_kv: Any, block_table: Any, k_scale: Any = None, v_scale: Any = None, *,
           page_size: int, sm_scale: float, softcap: float, is_causal: bool = True) -> Callable[..., torch.Tensor]:
    from .kernels import AttentionCall, GQADecodePagedKernel, GQADecodePagedMfmaKernel, get_arch

    if (k_scale is None) != (v_scale is None):
        raise ValueError("k_scale and v_scale come together")
    if len(q.shape) == 4:
        batch, q_len, heads, dim = q.shape
    else:
        (batch, heads, dim), q_len = q.shape, 1
    seqlen_kv, heads_kv, _ = k.shape
    index = q.device.index if q.device.type == "cuda" else None
    call = AttentionCall(dtype=q.dtype, kv_dtype=k.dtype, batch=batch, heads=heads, heads_kv=heads_kv, seqlen_kv=seqlen_kv,
                         dim=dim, page_size=page_size, sm_scale=sm_scale, softcap=softcap or 0.0, q_len=q_len,
                         is_causal=is_causal, arch=get_arch(index))
    cls = GQADecodePagedMfmaKernel if GQADecodePagedMfmaKernel.refusal(call) is None else GQADecodePagedKernel
    return cls(batch, heads, heads_kv, seqlen_kv, dim, page_size, q.dtype, sm_scale=sm_scale, softcap=softcap or 0.0,
               kv_dtype=k.dtype, q_len=q_len, is_causal=is_causal, device_index=index)


def build_gqa_decode_paged(q, k, v, real_seqlen_kv, block_table, k_scale=None, v_scale=None, *, page_size, sm_scale, softcap):
    """``build_kernel`` for ``GroupedQueryAttentionDecodePagedWithKVCacheFwdOp``."""
    return _build(q, k, v, real_seqlen_kv, block_table, k_scale, v_scale, page_size=page_size, sm_scale=sm_scale, softcap=softcap)


def build_gqa_multi_token_decode_paged(q, k, v, real_seqlen_kv, block_table, k_scale=None, v_scale=None, *, page_size,
                                       is_causal, sm_scale, softcap):
    """``build_kernel`` for ``GroupedQueryAttentionMultiTokenDecodePagedWithKVCacheFwdOp``."""
    return _build(q, k, v, real_seqlen_kv, block_table, k_scale, v_scale, page_size=page_size, sm_scale=sm_scale,
                  softcap=softcap, is_causal=is_causal)


def register(into: Optional[Any] = None, target: str = TARGET) -> None:
    """Register detector and builders with *into* (default: the installed ``tileops.backend``)."""
    if into is None:
        import tileops.backend as into  # noqa: PLC0415 - only when TileOPs is installed
    into.register_detector(target=target, detect=detect)
    into.register_kernel_builder(op=OP_SINGLE, target=target, build_kernel=build_gqa_decode_paged)
    into.register_kernel_builder(op=OP_MULTI, target=target, build_kernel=build_gqa_multi_token_decode_paged)


def _tileops_installed() -> bool:
    import importlib.util

    try:
        return importlib.util.find_spec("tileops.backend") is not None
    except (ImportError, ValueError):
        return False


if _tileops_installed():  # entry-point import: perform the registration
    register()
