"""Seeded synthetic inputs for the paged GQA decode ops.

``GroupedQueryAttentionDecodePagedWorkload`` reproduces the reference's generator
(workloads/attention/gqa.py:178-226): lengths drawn as multiples of the page size, one identity block table
shared by every sequence.  ``PagedDecodeConfig`` / ``BASELINE_CONFIGS`` describe the five benchmark
configurations (ragged lengths, every sequence on its own pages taken from one random permutation of a shared
pool) and ``gen_paged_inputs`` materialises them on any device from a seed.

Only input *generation* lives here (including the per-token FP8 quantizer that defines the cache format,
workloads/fp8_quant.py:27-33); nothing in this module computes attention.
"""

from __future__ import annotations

import math
from dataclasses import dataclass, replace
from typing import Optional

import torch

FP8 = torch.float8_e4m3fn
FP8_MAX = 448.0


@dataclass(frozen=True)
class PagedDecodeConfig:
    name: str
    batch: int
    heads: int
    heads_kv: int
    dim: int
    page_size: int
    n_pages: int                 # pages in the shared pool
    len_range: tuple[int, int]   # inclusive range of per-sequence context lengths
    q_len: int = 1
    dtype: torch.dtype = torch.bfloat16
    kv_dtype: torch.dtype = torch.bfloat16
    seed: int = 0
    description: str = ""

    @property
    def seqlen_kv(self) -> int:
        return self.n_pages * self.page_size

    @property
    def table_width(self) -> int:
        return math.ceil(self.len_range[1] / self.page_size)

    def scaled(self, *, batch: Optional[int] = None, n_pages: Optional[int] = None,
               len_range: Optional[tuple[int, int]] = None) -> "PagedDecodeConfig":
        """A smaller instance of the same configuration (for parity tests the CPU oracle finishes quickly)."""
        return replace(self, batch=batch or self.batch, n_pages=n_pages or self.n_pages, len_range=len_range or self.len_range)


BASELINE_CONFIGS: dict[str, PagedDecodeConfig] = {
    "c2": PagedDecodeConfig("c2", 64, 32, 8, 128, 64, 16384, (512, 8192), seed=1,
                            description="Llama-3-8B-shape paged GQA decode, bf16 KV"),
    "c3": PagedDecodeConfig("c3", 64, 32, 8, 128, 64, 16384, (512, 8192), kv_dtype=FP8, seed=1,
                            description="Llama-3-8B-shape paged GQA decode, FP8-e4m3fn KV with per-token scales"),
    "c4": PagedDecodeConfig("c4", 8, 64, 8, 128, 64, 16384, (131072, 131072), kv_dtype=FP8, seed=2,
                            description="long-context split-KV stress, 8 x 131072 tokens, FP8 KV"),
    "c5": PagedDecodeConfig("c5", 32, 64, 8, 128, 64, 16384, (1024, 16384), q_len=8, kv_dtype=FP8, seed=3,
                            description="multi-token (speculative verify) decode, 8 query tokens, FP8 KV"),
}


#: Benchmark configuration name -> (op, label of its manifest workload row)
BASELINE_WORKLOAD_ROWS: dict[str, tuple[str, str]] = {
    "c2": ("GroupedQueryAttentionDecodePagedWithKVCacheFwdOp", "llama3-8b-paged-bf16"),
    "c3": ("GroupedQueryAttentionDecodePagedWithKVCacheFwdOp", "llama3-8b-paged-fp8kv"),
    "c4": ("GroupedQueryAttentionDecodePagedWithKVCacheFwdOp", "long-context-128k-fp8kv"),
    "c5": ("GroupedQueryAttentionMultiTokenDecodePagedWithKVCacheFwdOp", "spec-verify-8tok-fp8kv"),
}


def config_from_workload(row: dict, name: str = "", description: str = "") -> PagedDecodeConfig:
    """A manifest workload row with ``seqlen_range`` (ragged lengths over a shared pool, permuted block table) as a
    ``PagedDecodeConfig``: ``q_shape`` ``[B, H, D]`` or ``[B, S_q, H, D]``, ``kv_shape`` ``[N_kv, H_kv, D]``."""
    qs, (n_kv, heads_kv, dim) = list(row["q_shape"]), row["kv_shape"]
    batch, heads = qs[0], qs[-2]
    q_len = qs[1] if len(qs) == 4 else 1
    dtype = getattr(torch, row["dtypes"][0])
    kv_dtype = getattr(torch, row["kv_dtype"]) if row.get("kv_dtype") else dtype
    page = row["page_size"]
    return PagedDecodeConfig(name or row["label"], batch, heads, heads_kv, dim, page, n_kv // page, tuple(row["seqlen_range"]),
                             q_len=q_len, dtype=dtype, kv_dtype=kv_dtype, seed=row.get("seed", 0), description=description)


def quantize_kv_per_token(x: torch.Tensor, chunk_tokens: int = 1 << 16) -> tuple[torch.Tensor, torch.Tensor]:
    """``x [N, H_kv, D]`` -> (e4m3fn ``[N, H_kv, D]``, fp32 scale ``[N, H_kv]``): ``scale = max(absmax, 1e-4)/448``,
    ``q = clamp(x/scale, -448, 448)`` cast with round-to-nearest-even.  Chunked so a whole pool fits."""
    q8 = torch.empty(x.shape, dtype=FP8, device=x.device)
    scale = torch.empty(x.shape[:-1], dtype=torch.float32, device=x.device)
    for s in range(0, x.shape[0], chunk_tokens):
        xf = x[s:s + chunk_tokens].float()
        amax = xf.abs().amax(dim=-1, keepdim=True).clamp(min=1e-4)
        sc = amax / FP8_MAX
        q8[s:s + chunk_tokens] = torch.clamp(xf / sc, min=-FP8_MAX, max=FP8_MAX).to(FP8)
        scale[s:s + chunk_tokens] = sc.squeeze(-1)
    return q8, scale


@dataclass
class PagedInputs:
    q: torch.Tensor
    k: torch.Tensor
    v: torch.Tensor
    real_seqlen_kv: torch.Tensor
    block_table: torch.Tensor
    k_scale: Optional[torch.Tensor] = None
    v_scale: Optional[torch.Tensor] = None

    def as_args(self) -> tuple:
        base = (self.q, self.k, self.v, self.real_seqlen_kv, self.block_table)
        return base if self.k_scale is None else base + (self.k_scale, self.v_scale)

    def to(self, device) -> "PagedInputs":
        mv = lambda t: None if t is None else t.to(device)  # noqa: E731
        return PagedInputs(mv(self.q), mv(self.k), mv(self.v), mv(self.real_seqlen_kv), mv(self.block_table),
                           mv(self.k_scale), mv(self.v_scale))

    @property
    def sum_len(self) -> int:
        return int(self.real_seqlen_kv.sum().item())


def gen_paged_inputs(cfg: PagedDecodeConfig, device: "torch.device | str" = "cpu", *, unused_page: int = 0) -> PagedInputs:
    """Materialise *cfg*.  Lengths, the page permutation and Q come from a CPU generator seeded with
    ``cfg.seed`` (identical on every machine); the K/V pool is drawn by a generator on *device* with the same
    seed, chunk by chunk, so a 4 GiB pool never exists in fp32."""
    device = torch.device(device)
    g = torch.Generator().manual_seed(cfg.seed)
    lo, hi = cfg.len_range
    lens = torch.randint(lo, hi + 1, (cfg.batch,), generator=g, dtype=torch.int64)
    perm = torch.randperm(cfg.n_pages, generator=g)
    pages = (lens + cfg.page_size - 1) // cfg.page_size
    if int(pages.sum()) > cfg.n_pages:
        raise ValueError(f"{cfg.name}: sequences need {int(pages.sum())} pages, pool has {cfg.n_pages}")
    table = torch.full((cfg.batch, cfg.table_width), unused_page, dtype=torch.int32)
    start = 0
    for b in range(cfg.batch):
        n = int(pages[b])
        table[b, :n] = perm[start:start + n].to(torch.int32)
        start += n
    q_shape = (cfg.batch, cfg.heads, cfg.dim) if cfg.q_len == 1 else (cfg.batch, cfg.q_len, cfg.heads, cfg.dim)
    q = torch.randn(q_shape, generator=g).to(cfg.dtype)

    gd = torch.Generator(device=device).manual_seed(cfg.seed)
    n_tok = cfg.seqlen_kv
    fp8 = cfg.kv_dtype == FP8
    k = torch.empty((n_tok, cfg.heads_kv, cfg.dim), dtype=cfg.kv_dtype, device=device)
    v = torch.empty_like(k)
    ks = torch.empty((n_tok, cfg.heads_kv), dtype=torch.float32, device=device) if fp8 else None
    vs = torch.empty_like(ks) if fp8 else None
    chunk = 1 << 16
    for s in range(0, n_tok, chunk):
        e = min(n_tok, s + chunk)
        for dst, dsc in ((k, ks), (v, vs)):
            x = torch.randn((e - s, cfg.heads_kv, cfg.dim), generator=gd, device=device)
            if fp8:
                dst[s:e], dsc[s:e] = quantize_kv_per_token(x)
            else:
                dst[s:e] = x.to(cfg.kv_dtype)
    return PagedInputs(q.to(device), k, v, lens.to(torch.int32).to(device), table.to(device), ks, vs)


def gen_contiguous_inputs(seed: int = 0, batch: int = 1, heads: int = 32, heads_kv: int = 8, seqlen_kv: int = 1024,
                          dim: int = 128, dtype: torch.dtype = torch.float32) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Config 1 (CPU plumbing): contiguous GQA decode inputs ``q [B,H,D]``, ``k,v [B,S,H_kv,D]`` ~ N(0,1)."""
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(batch, heads, dim, generator=g).to(dtype)
    k = torch.randn(batch, seqlen_kv, heads_kv, dim, generator=g).to(dtype)
    v = torch.randn(batch, seqlen_kv, heads_kv, dim, generator=g).to(dtype)
    return q, k, v


def contiguous_as_paged(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, page_size: int) -> PagedInputs:
    """View a contiguous cache ``[B,S,H_kv,D]`` as a page pool with an identity block table (S % page_size == 0)."""
    B, S, H_kv, D = k.shape
    if S % page_size:
        raise ValueError("seqlen must be a multiple of page_size")
    ppb = S // page_size
    table = torch.arange(B * ppb, dtype=torch.int32, device=k.device).reshape(B, ppb)
    lens = torch.full((B,), S, dtype=torch.int32, device=k.device)
    return PagedInputs(q, k.reshape(B * S, H_kv, D), v.reshape(B * S, H_kv, D), lens, table)


class GroupedQueryAttentionDecodePagedWorkload:
    """The reference's workload for the op: constructor and ``gen_inputs`` semantics of
    workloads/attention/gqa.py:178-226 (random page-multiple lengths, identity block table for every row)."""

    def __init__(self, batch: int, heads: int, heads_kv: int, seqlen_kv: int, dim: int, page_size: int,
                 dtype: torch.dtype, sm_scale: Optional[float] = None, softcap: Optional[float] = None) -> None:
        self.batch, self.heads, self.heads_kv, self.seqlen_kv = batch, heads, heads_kv, seqlen_kv
        self.dim, self.page_size, self.dtype = dim, page_size, dtype
        self.sm_scale = dim ** -0.5 if sm_scale is None else sm_scale
        self.softcap = 0.0 if softcap is None else softcap

    def gen_inputs(self, device: "torch.device | str" = "cuda", seed: int = 1235):
        g = torch.Generator().manual_seed(seed)
        num_pages = self.seqlen_kv // self.page_size
        lens = torch.randint(self.page_size, self.seqlen_kv + 1, (self.batch,), generator=g, dtype=torch.int32)
        lens = (lens // self.page_size) * self.page_size
        q = torch.randn(self.batch, self.heads, self.dim, generator=g).to(self.dtype)
        k = torch.randn(self.seqlen_kv, self.heads_kv, self.dim, generator=g).to(self.dtype)
        v = torch.randn(self.seqlen_kv, self.heads_kv, self.dim, generator=g).to(self.dtype)
        table = torch.arange(num_pages, dtype=torch.int32).unsqueeze(0).expand(self.batch, -1).contiguous()
        return tuple(t.to(device).contiguous() for t in (q, k, v, lens, table))
