"""(flops, bytes) models for paged GQA decode.

``gqa_decode_paged_roofline`` is the manifest's ``roofline.func``.  With only shapes it evaluates the
reference formula (src/tileops/perf/formulas.py:690-711), which prices the K/V *pool* once.  When the op
has seen a call (it records the sum of context lengths and pages in ``forward``) it returns the bytes a
call actually has to move -- every addressed K and V row once per sequence, scales, Q, O and the metadata
read -- which is what an HBM roofline for a shared page pool has to be measured against.
"""

from __future__ import annotations

from typing import Any, Optional

_ITEMSIZE = {"float16": 2, "bfloat16": 2, "float8_e4m3fn": 1, "float32": 4, "int32": 4}


def _itemsize(dtype: Any) -> int:
    if isinstance(dtype, (list, tuple)):
        dtype = dtype[0] if dtype else "float16"
    if hasattr(dtype, "itemsize"):
        return int(dtype.itemsize)
    name = str(dtype).split(".")[-1]
    return _ITEMSIZE.get(name, 2)


def _fields(op: Any, kwargs: dict[str, Any]) -> dict[str, Any]:
    if op is None:
        return kwargs
    return op if isinstance(op, dict) else vars(op)


def reference_formula(batch: int, heads: int, heads_kv: int, seqlen_kv: int, dim: int, page_size: int,
                      elem_bytes: int) -> tuple[int, int]:
    """src/tileops/perf/formulas.py:703-711, S = pool size, K/V counted once for the whole batch."""
    flops = 4 * batch * heads * seqlen_kv * dim
    q_elems = batch * heads * dim
    kv_elems = seqlen_kv * heads_kv * dim
    meta = batch * 4 + batch * max(1, (seqlen_kv + page_size - 1) // page_size) * 4
    return int(flops), int((q_elems + 2 * kv_elems + q_elems) * elem_bytes + meta)


def algorithmic_bytes(*, sum_len: int, sum_pages: int, batch: int, q_len: int, heads: int, heads_kv: int, dim: int,
                      q_bytes: int, kv_bytes: int, fp8_scales: bool) -> dict[str, int]:
    """Bytes one call must move, by term.  ``kv`` + ``scales`` is the "KV-read" figure of the headline metric."""
    kv = sum_len * heads_kv * dim * 2 * kv_bytes
    scales = sum_len * heads_kv * 2 * 4 if fp8_scales else 0
    qo = 2 * batch * q_len * heads * dim * q_bytes
    meta = 4 * batch + 4 * sum_pages
    return {"kv": kv, "scales": scales, "qo": qo, "meta": meta, "total": kv + scales + qo + meta}


def algorithmic_flops(*, sum_len: int, q_len: int, heads: int, dim: int) -> int:
    return 4 * q_len * heads * dim * sum_len


def gqa_decode_paged_roofline(op: Optional[Any] = None, **kwargs: Any) -> tuple[int, int]:
    d = _fields(op, kwargs)
    q_len = 1
    if "q_shape" in d:
        qs = tuple(d["q_shape"])
        if len(qs) == 4:
            batch, q_len, heads, dim = qs
        else:
            batch, heads, dim = qs
        seqlen_kv, heads_kv, _ = d["kv_shape"]
    else:
        batch, heads, heads_kv, seqlen_kv, dim = d["batch"], d["heads"], d["heads_kv"], d["seqlen_kv"], d["dim"]
        q_len = int(d.get("q_len", 1) or 1)
    page_size = int(d["page_size"])
    q_bytes = _itemsize(d.get("dtype") or d.get("dtypes") or "float16")
    seen = d.get("_seen_call")
    if seen is None:
        flops, nbytes = reference_formula(batch, heads, heads_kv, seqlen_kv, dim, page_size, q_bytes)
        return flops * q_len, nbytes
    b = algorithmic_bytes(sum_len=seen["sum_len"], sum_pages=seen["sum_pages"], batch=batch, q_len=q_len, heads=heads,
                          heads_kv=heads_kv, dim=dim, q_bytes=q_bytes, kv_bytes=seen["kv_bytes"], fp8_scales=seen["fp8"])
    return algorithmic_flops(sum_len=seen["sum_len"], q_len=q_len, heads=heads, dim=dim), b["total"]


def gqa_decode_roofline(op: Optional[Any] = None, **kwargs: Any) -> tuple[int, int]:
    """Contiguous-cache GQA decode: the reference formula (src/tileops/perf/formulas.py:668-687) from shapes;
    once the op has seen a call, the tokens it actually addressed instead of the allocated ``seqlen_kv``."""
    d = _fields(op, kwargs)
    if "q_shape" in d:
        batch, heads, dim = d["q_shape"]
        _, seqlen_kv, heads_kv, _ = d["kv_shape"]
    else:
        batch, heads, heads_kv, seqlen_kv, dim = d["batch"], d["heads"], d["heads_kv"], d["seqlen_kv"], d["dim"]
    q_bytes = _itemsize(d.get("dtype") or d.get("dtypes") or "float16")
    seen = d.get("_seen_call")
    if seen is None:
        flops = 4 * batch * heads * seqlen_kv * dim
        q_elems = batch * heads * dim
        kv_elems = batch * seqlen_kv * heads_kv * dim
        return int(flops), int((q_elems + 2 * kv_elems + q_elems) * q_bytes)
    b = algorithmic_bytes(sum_len=seen["sum_len"], sum_pages=0, batch=batch, q_len=1, heads=heads, heads_kv=heads_kv,
                          dim=dim, q_bytes=q_bytes, kv_bytes=seen["kv_bytes"], fp8_scales=seen["fp8"])
    return algorithmic_flops(sum_len=seen["sum_len"], q_len=1, heads=heads, dim=dim), b["total"] - 4 * batch


def _distribute_total(total: int, batch: int, max_len: int) -> list[int]:
    """src/tileops/perf/formulas.py:467-475."""
    lengths, remaining = [0] * batch, total
    for idx in range(batch):
        value = min(max_len, remaining - (batch - idx - 1))
        lengths[idx] = value
        remaining -= value
    return lengths


def gqa_prefill_paged_with_kv_cache_fwd_roofline(op: Optional[Any] = None, **kwargs: Any) -> tuple[int, int]:
    """Paged-cache GQA prefill: the reference's conservative model (src/tileops/perf/formulas.py:532-587) -- visible
    score count from per-request ``q_lens`` / ``cache_lens`` (a deterministic fill when a workload row omits them);
    bytes = Q, old K/V, new K/V read, new K/V appended, O, and the metadata, all at the attention element size."""
    d = _fields(op, kwargs)
    batch, heads, heads_kv, dim = int(d["batch"]), int(d["heads"]), int(d["heads_kv"]), int(d["dim"])
    max_pages, page = int(d["max_pages_per_req"]), int(d["page_size"])
    max_q = int(d.get("max_seqlen_q") or max_pages * page)
    causal = bool(d.get("is_causal", True))
    elem = _itemsize(d.get("dtype") or d.get("dtypes") or "float16")
    q_lens = d.get("q_lens")
    total_q = int(d["total_q"]) if d.get("total_q") is not None else (int(sum(q_lens)) if q_lens is not None else batch * max_q)
    if q_lens is None:
        q_lens = _distribute_total(total_q, batch, max_q)
    cache_lens = d.get("cache_lens")
    if cache_lens is None:
        cap = max_pages * page if d.get("max_position") is None else int(d["max_position"])
        cache_lens = [max(cap - int(n), 0) for n in q_lens]
    visible = old = 0
    for n, m in zip(q_lens, cache_lens):
        n, m = int(n), int(m)
        old += m
        visible += n * m + n * (n + 1) // 2 if causal else n * (m + n)
    q_elems = total_q * heads * dim
    new_kv = 2 * total_q * heads_kv * dim
    nbytes = (q_elems + 2 * old * heads_kv * dim + new_kv + new_kv + q_elems) * elem + (batch + 1) * 4 + batch * 4 + batch * max_pages * 4
    return int(4 * heads * visible * dim), int(nbytes)
