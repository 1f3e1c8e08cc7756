"""``torch.library`` registration of the library's entry points, so that the ops trace under ``torch.compile``.

The reference registers each of its compiled attention kernels as a custom operator with a fake (meta)
implementation (src/tileops/kernels/attention/gqa_decode_paged.py:401-508), which is what lets
``torch.compile(op, fullgraph=True)`` put the call into a graph instead of breaking at it
(contract: tests/compile_contract.py).  A ctypes call is opaque to the tracer, so the same is done here: every
kernel class's ``forward`` goes through one of the operators below.  Each operator

* takes the tensors plus the scalars of the C entry point it wraps,
* allocates the output and the workspace with torch inside its implementation and enqueues the HIP kernels on
  the current stream (nothing else: no host read-back, no synchronisation),
* has a fake implementation that only states the output's shape and dtype (``empty_like(q)``),
* declares the page pools it appends to as mutated (the two prefill operators).

Operator names: ``tileops_amd::gqa_paged_decode``, ``tileops_amd::gqa_decode``, ``tileops_amd::gqa_prefill_paged``,
``tileops_amd::gqa_prefill_paged_rope``.
"""

from __future__ import annotations

from typing import Optional

import torch

from . import native

__all__ = ["OP_NAMES", "gqa_decode", "gqa_paged_decode", "gqa_prefill_paged", "gqa_prefill_paged_rope"]

OP_NAMES = ("tileops_amd::gqa_paged_decode", "tileops_amd::gqa_decode", "tileops_amd::gqa_prefill_paged",
            "tileops_amd::gqa_prefill_paged_rope")

# (workspace bytes, partition count) per shape: a workspace query touches no device and never changes its answer
_decode_plans: dict[tuple, tuple[int, int]] = {}
_contig_plans: dict[tuple, tuple[int, int]] = {}
_prefill_plans: dict[tuple, int] = {}


def _workspace(nbytes: int, device: torch.device) -> Optional[torch.Tensor]:
    return torch.empty(nbytes, dtype=torch.uint8, device=device) if nbytes else None


@torch.library.custom_op("tileops_amd::gqa_paged_decode", mutates_args=())
def gqa_paged_decode(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, real_seqlen_kv: torch.Tensor, block_table: torch.Tensor,
                     k_scale: Optional[torch.Tensor], v_scale: Optional[torch.Tensor], q_len: int, heads: int, heads_kv: int,
                     dim: int, page_size: int, sm_scale: float, softcap: float, causal: bool, num_split: int,
                     kernel: int) -> torch.Tensor:
    """Paged GQA decode (``mi355_gqa_paged_decode``): ``q [B, H, D]`` or ``[B, S_q, H, D]``, pool ``k, v [N_kv, H_kv, D]``."""
    native.require_gfx950(q.device)
    batch = q.shape[0]
    key = (batch, q_len, heads, heads_kv, dim, page_size, block_table.shape[1], q.dtype, k.dtype, num_split, kernel & 0xFF)
    plan = _decode_plans.get(key)
    if plan is None:
        nbytes, nsplit, _ = native.decode_workspace(batch, q_len, heads, heads_kv, dim, page_size, block_table.shape[1], q.dtype,
                                                    k.dtype, num_split, kernel & 0xFF)
        plan = _decode_plans[key] = (nbytes, nsplit)
    out = torch.empty_like(q)
    native.paged_decode(q, k, v, k_scale, v_scale, real_seqlen_kv, block_table, out, _workspace(plan[0], q.device), batch=batch,
                        q_len=q_len, heads=heads, heads_kv=heads_kv, dim=dim, page_size=page_size, sm_scale=sm_scale,
                        softcap=softcap, causal=causal, num_split=plan[1], kernel=kernel)
    return out


@gqa_paged_decode.register_fake
def _(q, k, v, real_seqlen_kv, block_table, k_scale, v_scale, q_len, heads, heads_kv, dim, page_size, sm_scale, softcap, causal,
      num_split, kernel):
    return torch.empty_like(q)


@torch.library.custom_op("tileops_amd::gqa_decode", mutates_args=())
def gqa_decode(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, k_scale: Optional[torch.Tensor], v_scale: Optional[torch.Tensor],
               real_seqlen_kv: int, heads: int, heads_kv: int, dim: int, sm_scale: float, softcap: float, causal: bool,
               num_split: int, kernel: int) -> torch.Tensor:
    """GQA decode over a contiguous cache (``mi355_gqa_decode``): ``q [B, H, D]``, ``k, v [B, N_kv, H_kv, D]``."""
    native.require_gfx950(q.device)
    batch = q.shape[0]
    key = (batch, heads, heads_kv, dim, real_seqlen_kv, q.dtype, k.dtype, num_split, kernel)
    plan = _contig_plans.get(key)
    if plan is None:
        nbytes, nsplit, _ = native.contiguous_decode_workspace(batch, 1, heads, heads_kv, dim, max(real_seqlen_kv, 1), q.dtype, k.dtype,
                                                               num_split, kernel)
        plan = _contig_plans[key] = (nbytes, nsplit)
    out = torch.empty_like(q)
    native.contiguous_decode(q, k, v, k_scale, v_scale, out, _workspace(plan[0], q.device), batch=batch, q_len=1, heads=heads,
                             heads_kv=heads_kv, dim=dim, real_seqlen_kv=real_seqlen_kv, sm_scale=sm_scale, softcap=softcap,
                             causal=causal, num_split=plan[1], kernel=kernel)
    return out


@gqa_decode.register_fake
def _(q, k, v, k_scale, v_scale, real_seqlen_kv, heads, heads_kv, dim, sm_scale, softcap, causal, num_split, kernel):
    return torch.empty_like(q)


@torch.library.custom_op("tileops_amd::gqa_prefill_paged", mutates_args=("k_pages", "v_pages"))
def gqa_prefill_paged(q: torch.Tensor, k_new: torch.Tensor, v_new: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                      k_scale: torch.Tensor, v_scale: torch.Tensor, cu_seqlens_q: torch.Tensor, cache_seqlens: torch.Tensor,
                      block_table: torch.Tensor, max_seqlen_q: int, heads: int, heads_kv: int, dim: int, page_size: int,
                      sm_scale: float, softcap: float, causal: bool, kernel: int) -> torch.Tensor:
    """Packed prefill chunk with paged-cache append (``mi355_gqa_prefill_paged``); writes the chunk into the pages."""
    native.require_gfx950(q.device)
    batch = cache_seqlens.shape[0]
    key = (batch, max_seqlen_q, q.shape[0], heads, heads_kv, dim, page_size, block_table.shape[1], q.dtype, k_pages.dtype, kernel)
    nbytes = _prefill_plans.get(key)
    if nbytes is None:
        nbytes = _prefill_plans[key] = native.prefill_paged_workspace(batch, max_seqlen_q, q.shape[0], heads, heads_kv, dim, page_size,
                                                                      block_table.shape[1], q.dtype, k_pages.dtype, kernel)
    out = torch.empty_like(q)
    native.prefill_paged(q, k_new, v_new, k_pages, v_pages, k_scale, v_scale, cu_seqlens_q, cache_seqlens, block_table, out,
                         _workspace(nbytes, q.device), batch=batch, max_seqlen_q=max_seqlen_q, heads=heads, heads_kv=heads_kv, dim=dim,
                         page_size=page_size, sm_scale=sm_scale, softcap=softcap, causal=causal, kernel=kernel)
    return out


@gqa_prefill_paged.register_fake
def _(q, k_new, v_new, k_pages, v_pages, k_scale, v_scale, cu_seqlens_q, cache_seqlens, block_table, max_seqlen_q, heads, heads_kv,
      dim, page_size, sm_scale, softcap, causal, kernel):
    return torch.empty_like(q)


@torch.library.custom_op("tileops_amd::gqa_prefill_paged_rope", mutates_args=("k_pages", "v_pages"))
def gqa_prefill_paged_rope(q: torch.Tensor, k_new: torch.Tensor, v_new: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                           cos_table: torch.Tensor, sin_table: torch.Tensor, cu_seqlens_q: torch.Tensor, cache_seqlens: torch.Tensor,
                           block_table: torch.Tensor, max_seqlen_q: int, heads: int, heads_kv: int, dim: int, page_size: int,
                           rotary_dim: int, sm_scale: float, softcap: float, causal: bool, kernel: int) -> torch.Tensor:
    """The same with rotary position embedding fused in (``mi355_gqa_prefill_paged_rope``)."""
    native.require_gfx950(q.device)
    batch = cache_seqlens.shape[0]
    key = (batch, max_seqlen_q, q.shape[0], heads, heads_kv, dim, page_size, block_table.shape[1], q.dtype, "rope", kernel)
    nbytes = _prefill_plans.get(key)
    if nbytes is None:
        nbytes = _prefill_plans[key] = native.prefill_paged_rope_workspace(batch, max_seqlen_q, q.shape[0], heads, heads_kv, dim,
                                                                           page_size, block_table.shape[1], q.dtype, kernel)
    out = torch.empty_like(q)
    workspace = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=q.device)
    native.prefill_paged_rope(q, k_new, v_new, k_pages, v_pages, cos_table, sin_table, cu_seqlens_q, cache_seqlens, block_table, out,
                              workspace, batch=batch, max_seqlen_q=max_seqlen_q, heads=heads, heads_kv=heads_kv, dim=dim,
                              page_size=page_size, rotary_dim=rotary_dim, sm_scale=sm_scale, softcap=softcap, causal=causal,
                              kernel=kernel)
    return out


@gqa_prefill_paged_rope.register_fake
def _(q, k_new, v_new, k_pages, v_pages, cos_table, sin_table, cu_seqlens_q, cache_seqlens, block_table, max_seqlen_q, heads,
      heads_kv, dim, page_size, rotary_dim, sm_scale, softcap, causal, kernel):
    return torch.empty_like(q)
