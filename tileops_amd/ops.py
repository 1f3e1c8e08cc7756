"""L2 ops: paged GQA decode over a KV page pool, bf16/fp16 or FP8-e4m3fn cache, on MI355X.

``GroupedQueryAttentionDecodePagedWithKVCacheFwdOp`` keeps the reference op's contract
(src/tileops/ops/attention/gqa.py:1357-1454): same constructor arguments, defaults and error messages
(``_validate_gqa_dims`` :74-78, ``_validate_positive`` :66-71, scale/softcap defaults :81-90), same
``forward(q, k, v, real_seqlen_kv, block_table)`` order, output = ``q``'s shape and dtype.  On top of it:

* ``k``/``v`` may be ``float8_e4m3fn`` with trailing optional ``k_scale, v_scale [N_kv, H_kv]`` fp32
  (dequant ``fp8.float() * scale``; scale rules follow the paged prefill op, gqa.py:992-999);
* ``forward`` validates device, dtype, rank/shape, contiguity and metadata dtypes (the reference's forward
  validates nothing; its sibling paged prefill op does, gqa.py:897-1046, and that is the template);
* an external target's builder, once settled, is consulted *before* in-tree kernel selection, so a target
  whose devices the in-tree kernels cannot run on is still reachable.

``GroupedQueryAttentionMultiTokenDecodePagedWithKVCacheFwdOp`` is the multi-token (speculative-verify)
sibling: ``q [B, S_q, H, D]``, the cache already holds the S_q new tokens, and the causal mask is
bottom-right aligned (key j visible to query i iff ``j <= i + (len - S_q)``; gqa.py:558-562).
"""

from __future__ import annotations

from typing import Dict, Optional

import torch

from . import native
from .backend import Target
from .kernels import (
    DECODE_KEYS, PAGED_DECODE_KEYS, PAGED_PREFILL_KEYS, AttentionCall, GQADecodeKernel, GQADecodeMfmaKernel,
    GQADecodePagedKernel, GQADecodePagedMfmaKernel, GQAPrefillPagedWithFP8KVCacheFwdKernel,
    GQAPrefillPagedWithKVCacheRopeFwdKernel,
    GQAPrefillPagedWithKVCacheFwdKernel, PrefillCall, get_arch,
)
from .op_base import _UNRESOLVED, Op

__all__ = [
    "GroupedQueryAttentionDecodeWithKVCacheFwdOp",
    "GroupedQueryAttentionDecodePagedWithKVCacheFwdOp",
    "GroupedQueryAttentionMultiTokenDecodePagedWithKVCacheFwdOp",
    "GroupedQueryAttentionPrefillPagedWithKVCacheFwdOp",
]

FP8 = torch.float8_e4m3fn


def _validate_attention_dtype(dtype: torch.dtype) -> None:
    if dtype not in (torch.float16, torch.bfloat16):
        raise ValueError(f"Expected dtype torch.float16 or torch.bfloat16, got {dtype}")


def _validate_positive(**values: int) -> None:
    for name, value in values.items():
        if value <= 0:
            raise ValueError(f"{name} must be positive")


def _validate_gqa_dims(heads: int, heads_kv: int, dim: int) -> None:
    _validate_positive(heads=heads, heads_kv=heads_kv)
    if heads % heads_kv != 0:
        raise ValueError("heads must be divisible by heads_kv")
    _validate_positive(dim=dim)


def _attention_scale(dim: int, sm_scale: Optional[float]) -> float:
    return dim ** -0.5 if sm_scale is None else sm_scale


def _score_softcap(softcap: Optional[float]) -> float:
    if softcap is None:
        return 0.0
    if softcap < 0:
        raise ValueError("softcap must be non-negative")
    return softcap


class _PagedDecodeOp(Op):
    """What the single-token op and its multi-token sibling share."""

    q_len: int = 1
    is_causal: bool = True
    compile_op_names = ("tileops_amd::gqa_paged_decode",)
    #: Set True to also check values that live on the device (scales finite and positive, block-table
    #: entries inside the pool).  Costs a device read-back per call, so it is off on the serving path.
    debug_checks: bool = False
    _seen_call: Optional[dict] = None

    def _init_common(self, batch: int, heads: int, heads_kv: int, seqlen_kv: int, dim: int, page_size: int,
                     sm_scale: Optional[float], softcap: Optional[float], kernel_map: Optional[Dict[str, type]],
                     tune: bool, target: Target) -> None:
        _validate_gqa_dims(heads, heads_kv, dim)
        self.batch, self.heads, self.heads_kv, self.seqlen_kv, self.dim = batch, heads, heads_kv, seqlen_kv, dim
        self.page_size = page_size
        _validate_positive(page_size=page_size)
        self.sm_scale = _attention_scale(dim, sm_scale)
        self.softcap = _score_softcap(softcap)
        self.tune = tune
        self._selected_keys: dict = {}
        if target is not None:
            self.target = target
        self.dispatch_kernel(kernel_map)

    @property
    def default_kernel_map(self) -> Dict[str, type]:
        return {
            "gqa_decode_paged_kernel": GQADecodePagedKernel,
            "gqa_decode_paged_mfma_kernel": GQADecodePagedMfmaKernel,
        }

    def attention_call(self, dtype: torch.dtype, kv_dtype: Optional[torch.dtype] = None,
                       device: Optional[torch.device] = None) -> AttentionCall:
        """State what one call is, for selection to filter against.  Reads the device architecture (not the ctor)."""
        index = device.index if device is not None and device.type == "cuda" else None
        return AttentionCall(
            dtype=dtype, kv_dtype=kv_dtype or dtype, batch=self.batch, heads=self.heads, heads_kv=self.heads_kv,
            seqlen_kv=self.seqlen_kv, dim=self.dim, page_size=self.page_size, sm_scale=self.sm_scale,
            softcap=self.softcap, tune=self.tune, q_len=self.q_len, is_causal=self.is_causal, arch=get_arch(index))

    def _get_kernel(self, inputs: "tuple[torch.Tensor | None, ...]", dtype: torch.dtype,
                    kv_dtype: Optional[torch.dtype] = None):
        _validate_attention_dtype(dtype)
        kv_dtype = kv_dtype or dtype
        if self._builder is not None and self._builder is not _UNRESOLVED:
            # an external target serves this instance: its builder chooses among its own kernels
            return self.get_or_build_kernel("gqa_decode_paged_kernel", inputs)
        device = next((t.device for t in inputs if t is not None), None)
        # selection is a function of the call and of the kernel map: settled once per (dtypes, device, map), like the
        # reference's once-per-dtype kernel choice (ops/attention/gqa.py:1389-1408)
        memo_key = (dtype, kv_dtype, device, tuple(self.kernel_map.items()))
        memo = self._selected_keys
        hit = memo.get(memo_key)
        if hit is None:
            call = self.attention_call(dtype, kv_dtype, device)
            hit = memo[memo_key] = (self.select_kernel_key(PAGED_DECODE_KEYS, call), call)
        key, call = hit

        def build():
            return self.kernel_map[key](
                call.batch, call.heads, call.heads_kv, call.seqlen_kv, call.dim, call.page_size, call.dtype,
                sm_scale=call.sm_scale, softcap=call.softcap, tune=call.tune, kv_dtype=call.kv_dtype,
                q_len=call.q_len, is_causal=call.is_causal,
                device_index=device.index if device is not None and device.type == "cuda" else None)

        return self.get_or_build_kernel(key, inputs, key=(dtype, kv_dtype), build=build)

    # -- validation ------------------------------------------------------------------------------------
    def _q_shape(self) -> tuple[int, ...]:
        return (self.batch, self.heads, self.dim) if self.q_len == 1 and not self._q_is_4d else (
            self.batch, self.q_len, self.heads, self.dim)

    _q_is_4d = False

    def _validate_call(self, q, k, v, real_seqlen_kv, block_table, k_scale, v_scale) -> None:
        named = {"q": q, "k": k, "v": v, "real_seqlen_kv": real_seqlen_kv, "block_table": block_table}
        for name, t in named.items():
            if not isinstance(t, torch.Tensor):
                raise ValueError(f"{name} must be a torch.Tensor, got {type(t).__name__}")
        self._validate_dtypes(q, k, v, real_seqlen_kv, block_table, k_scale, v_scale)
        fp8 = k.dtype == FP8
        if fp8 and (k_scale is None or v_scale is None):
            raise ValueError("k_scale and v_scale are required when the KV cache is float8_e4m3fn")
        if not fp8 and (k_scale is not None or v_scale is not None):
            raise ValueError("k_scale and v_scale must be None unless the KV cache is float8_e4m3fn")
        if fp8:
            named.update(k_scale=k_scale, v_scale=v_scale)
        for name, t in named.items():
            if t.device != q.device:
                raise ValueError(f"Expected {name} on {q.device}, got {t.device}")
        want_q = self._q_shape()
        if tuple(q.shape) != want_q:
            raise ValueError(f"Expected q.shape {want_q}, got {tuple(q.shape)}")
        want_kv = (self.seqlen_kv, self.heads_kv, self.dim)
        for name, t in (("k", k), ("v", v)):
            if tuple(t.shape) != want_kv:
                raise ValueError(f"Expected {name}.shape {want_kv}, got {tuple(t.shape)}")
        if tuple(real_seqlen_kv.shape) != (self.batch,):
            raise ValueError(f"Expected real_seqlen_kv.shape {(self.batch,)}, got {tuple(real_seqlen_kv.shape)}")
        if block_table.dim() != 2 or block_table.shape[0] != self.batch or block_table.shape[1] < 1:
            raise ValueError(f"Expected block_table.shape ({self.batch}, num_pages), got {tuple(block_table.shape)}")
        for name, t in (("q", q), ("k", k), ("v", v), ("real_seqlen_kv", real_seqlen_kv)):
            if not t.is_contiguous():
                raise ValueError(f"{name} must be contiguous")
        if block_table.stride(1) != 1:
            raise ValueError("block_table rows must be contiguous (stride(1) == 1)")
        if fp8:
            for name, t in (("k_scale", k_scale), ("v_scale", v_scale)):
                if tuple(t.shape) != (self.seqlen_kv, self.heads_kv):
                    raise ValueError(f"Expected {name}.shape {(self.seqlen_kv, self.heads_kv)}, got {tuple(t.shape)}")
                if not t.is_contiguous():
                    raise ValueError(f"{name} must be contiguous")
        if self.debug_checks:
            if fp8:
                for name, t in (("k_scale", k_scale), ("v_scale", v_scale)):
                    if not torch.all(torch.isfinite(t) & (t > 0)).item():
                        raise ValueError(f"{name} must contain finite positive values")
            if real_seqlen_kv.min().item() < 0:
                raise ValueError("real_seqlen_kv must be non-negative")
            need = (real_seqlen_kv.max().item() + self.page_size - 1) // self.page_size
            if need > block_table.shape[1]:
                raise ValueError(f"block_table has {block_table.shape[1]} columns but the longest sequence needs {need}")
            if block_table.min().item() < 0 or block_table.max().item() >= self.seqlen_kv // self.page_size:
                raise ValueError("block_table entries must lie in [0, seqlen_kv // page_size)")

    def observe_call(self, real_seqlen_kv: torch.Tensor, kv_dtype: torch.dtype) -> None:
        """Record the context lengths of a call so that ``eval_roofline`` prices the bytes actually addressed.
        Reads device memory once; benchmarks call it outside the timed region."""
        lens = real_seqlen_kv.to("cpu", torch.int64)
        pages = (lens + self.page_size - 1) // self.page_size
        self._seen_call = {
            "sum_len": int(lens.sum()), "sum_pages": int(pages.sum()),
            "kv_bytes": torch.empty((), dtype=kv_dtype).element_size(), "fp8": kv_dtype == FP8,
        }

    def capture(self, q, k, v, real_seqlen_kv, block_table, k_scale=None, v_scale=None):
        """Record one call in a HIP graph and return ``replay() -> out``: every replay re-reads the same tensors in place
        (new cache contents, lengths and block-table entries are picked up; shapes and addresses are fixed) and leaves the
        result in the same output tensor.  A decode step costs one graph launch instead of a host launch per kernel.  The
        call holds no memset node and nothing the host reads back, so replays equal eager calls bit for bit."""
        args = (q, k, v, real_seqlen_kv, block_table) + (() if k_scale is None else (k_scale, v_scale))
        self(*args)  # validation, kernel selection and the library's one-time per-device set-up happen outside the capture
        side = torch.cuda.Stream(device=q.device)
        side.wait_stream(torch.cuda.current_stream(q.device))
        with torch.cuda.stream(side):
            self(*args)
        torch.cuda.current_stream(q.device).wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out = self(*args)

        def replay() -> torch.Tensor:
            graph.replay()
            return out

        replay.graph = graph  # keeps the graph (and its private memory pool) alive with the callable
        return replay

    def _run(self, q, k, v, real_seqlen_kv, block_table, k_scale, v_scale) -> torch.Tensor:
        self._validate_call(q, k, v, real_seqlen_kv, block_table, k_scale, v_scale)
        self.dtype = q.dtype
        inputs = (q, k, v, real_seqlen_kv, block_table, k_scale, v_scale)
        kernel = self._get_kernel(inputs, q.dtype, k.dtype)
        if k_scale is None:
            return kernel(q, k, v, real_seqlen_kv, block_table)
        return kernel(q, k, v, real_seqlen_kv, block_table, k_scale, v_scale)


class GroupedQueryAttentionDecodePagedWithKVCacheFwdOp(_PagedDecodeOp):
    """Paged GQA decode with dynamic KV cache. Layout: Q [batch, heads, dim] (BHD);
    K, V physical cache [seqlen_kv, heads_kv, dim]; real_seqlen_kv [batch]; block_table [batch, num_pages]."""

    def __init__(self, batch: int, heads: int, heads_kv: int, seqlen_kv: int, dim: int, page_size: int,
                 sm_scale: Optional[float] = None, softcap: Optional[float] = None,
                 kernel_map: Optional[Dict[str, type]] = None, tune: bool = False, *, target: Target = None) -> None:
        self._init_common(batch, heads, heads_kv, seqlen_kv, dim, page_size, sm_scale, softcap, kernel_map, tune, target)

    def _infer_output_shapes(self, q_shape, k_shape, v_shape, real_seqlen_kv_shape, block_table_shape,
                             k_scale_shape=None, v_scale_shape=None) -> dict[str, tuple[int, ...]]:
        """Manifest ``shape_rules``: ``o.shape == q.shape``."""
        return {"o": tuple(q_shape)}

    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, real_seqlen_kv: torch.Tensor,
                block_table: torch.Tensor, k_scale: Optional[torch.Tensor] = None,
                v_scale: Optional[torch.Tensor] = None) -> torch.Tensor:
        return self._run(q, k, v, real_seqlen_kv, block_table, k_scale, v_scale)


class GroupedQueryAttentionMultiTokenDecodePagedWithKVCacheFwdOp(_PagedDecodeOp):
    """Multi-token paged GQA decode (speculative verify). Layout: Q [batch, q_len, heads, dim] (BSHD);
    K, V physical cache [seqlen_kv, heads_kv, dim] already holding the q_len new tokens;
    real_seqlen_kv [batch] counts them; block_table [batch, num_pages]."""

    _q_is_4d = True

    def __init__(self, batch: int, q_len: int, heads: int, heads_kv: int, seqlen_kv: int, dim: int, page_size: int,
                 is_causal: bool = True, sm_scale: Optional[float] = None, softcap: Optional[float] = None,
                 kernel_map: Optional[Dict[str, type]] = None, tune: bool = False, *, target: Target = None) -> None:
        _validate_positive(q_len=q_len)
        self.q_len = q_len
        self.is_causal = bool(is_causal)
        self._init_common(batch, heads, heads_kv, seqlen_kv, dim, page_size, sm_scale, softcap, kernel_map, tune, target)

    def _infer_output_shapes(self, q_shape, k_shape, v_shape, real_seqlen_kv_shape, block_table_shape,
                             k_scale_shape=None, v_scale_shape=None) -> dict[str, tuple[int, ...]]:
        return {"o": tuple(q_shape)}

    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, real_seqlen_kv: torch.Tensor,
                block_table: torch.Tensor, k_scale: Optional[torch.Tensor] = None,
                v_scale: Optional[torch.Tensor] = None) -> torch.Tensor:
        return self._run(q, k, v, real_seqlen_kv, block_table, k_scale, v_scale)


class GroupedQueryAttentionDecodeWithKVCacheFwdOp(Op):
    """GQA decode over a contiguous KV cache.  Layout: Q ``[batch, heads, dim]``; K, V ``[batch, N_kv, heads_kv, dim]``
    (BSHD) with ``N_kv <= seqlen_kv`` the context length of every sequence.

    Keeps the reference op's contract (src/tileops/ops/attention/gqa.py:1260-1350): same constructor arguments,
    defaults and error messages, ``forward(q, k, v)`` with the real length taken from ``k.shape[1]``, output =
    ``q``'s shape and dtype.  The reference zero-pads K/V to the compiled ``seqlen_kv`` (:1338-1345); the kernels
    here take the length at run time and read only the tokens that exist, so nothing is copied.  As for the paged
    ops, K/V may be ``float8_e4m3fn`` with trailing ``k_scale, v_scale [batch, N_kv, heads_kv]`` fp32.
    """

    _seen_call: Optional[dict] = None
    compile_op_names = ("tileops_amd::gqa_decode",)

    def __init__(self, batch: int, heads: int, heads_kv: int, seqlen_kv: int, dim: int,
                 sm_scale: Optional[float] = None, softcap: Optional[float] = None,
                 kernel_map: Optional[Dict[str, type]] = None, tune: bool = False, *, target: Target = None) -> None:
        _validate_gqa_dims(heads, heads_kv, dim)
        self.batch, self.heads, self.heads_kv, self.seqlen_kv, self.dim = batch, heads, heads_kv, seqlen_kv, dim
        self.sm_scale = _attention_scale(dim, sm_scale)
        self.softcap = _score_softcap(softcap)
        self.tune = tune
        if target is not None:
            self.target = target
        self.dispatch_kernel(kernel_map)

    @property
    def default_kernel_map(self) -> Dict[str, type]:
        return {"gqa_decode_kernel": GQADecodeKernel, "gqa_decode_mfma_kernel": GQADecodeMfmaKernel}

    def attention_call(self, dtype: torch.dtype, kv_dtype: Optional[torch.dtype] = None,
                       device: Optional[torch.device] = None) -> AttentionCall:
        index = device.index if device is not None and device.type == "cuda" else None
        return AttentionCall(
            dtype=dtype, kv_dtype=kv_dtype or dtype, batch=self.batch, heads=self.heads, heads_kv=self.heads_kv,
            seqlen_kv=self.seqlen_kv, dim=self.dim, page_size=0, sm_scale=self.sm_scale, softcap=self.softcap,
            tune=self.tune, arch=get_arch(index))

    def _get_kernel(self, inputs: "tuple[torch.Tensor | None, ...]", dtype: torch.dtype,
                    kv_dtype: Optional[torch.dtype] = None):
        _validate_attention_dtype(dtype)
        kv_dtype = kv_dtype or dtype
        if self._builder is not None and self._builder is not _UNRESOLVED:
            return self.get_or_build_kernel("gqa_decode_kernel", inputs)
        device = next((t.device for t in inputs if t is not None), None)
        call = self.attention_call(dtype, kv_dtype, device)
        key = self.select_kernel_key(DECODE_KEYS, call)

        def build():
            return self.kernel_map[key](
                call.batch, call.heads, call.heads_kv, call.seqlen_kv, call.dim, call.dtype, sm_scale=call.sm_scale,
                softcap=call.softcap, tune=call.tune, kv_dtype=call.kv_dtype,
                device_index=device.index if device is not None and device.type == "cuda" else None)

        return self.get_or_build_kernel(key, inputs, key=(dtype, kv_dtype), build=build)

    def _infer_output_shapes(self, q_shape, k_shape, v_shape, k_scale_shape=None, v_scale_shape=None) -> dict[str, tuple[int, ...]]:
        """Manifest ``shape_rules``: ``o.shape == q.shape``."""
        return {"o": tuple(q_shape)}

    def _validate_call(self, q, k, v, k_scale, v_scale) -> None:
        named = {"q": q, "k": k, "v": v}
        for name, t in named.items():
            if not isinstance(t, torch.Tensor):
                raise ValueError(f"{name} must be a torch.Tensor, got {type(t).__name__}")
        self._validate_dtypes(q, k, v, k_scale, v_scale)
        fp8 = k.dtype == FP8
        if fp8 and (k_scale is None or v_scale is None):
            raise ValueError("k_scale and v_scale are required when the KV cache is float8_e4m3fn")
        if not fp8 and (k_scale is not None or v_scale is not None):
            raise ValueError("k_scale and v_scale must be None unless the KV cache is float8_e4m3fn")
        if fp8:
            named.update(k_scale=k_scale, v_scale=v_scale)
        for name, t in named.items():
            if t.device != q.device:
                raise ValueError(f"Expected {name} on {q.device}, got {t.device}")
        want_q = (self.batch, self.heads, self.dim)
        if tuple(q.shape) != want_q:
            raise ValueError(f"Expected q.shape {want_q}, got {tuple(q.shape)}")
        if k.dim() != 4 or k.shape[0] != self.batch or tuple(k.shape[2:]) != (self.heads_kv, self.dim):
            raise ValueError(f"Expected k.shape ({self.batch}, N_kv, {self.heads_kv}, {self.dim}), got {tuple(k.shape)}")
        if tuple(v.shape) != tuple(k.shape):
            raise ValueError(f"Expected v.shape {tuple(k.shape)}, got {tuple(v.shape)}")
        if k.shape[1] > self.seqlen_kv:
            raise ValueError(f"k holds {k.shape[1]} tokens per sequence but the op was built for seqlen_kv={self.seqlen_kv}")
        for name, t in named.items():
            if not t.is_contiguous():
                raise ValueError(f"{name} must be contiguous")
        if fp8:
            for name, t in (("k_scale", k_scale), ("v_scale", v_scale)):
                if tuple(t.shape) != tuple(k.shape[:3]):
                    raise ValueError(f"Expected {name}.shape {tuple(k.shape[:3])}, got {tuple(t.shape)}")

    def observe_call(self, real_seqlen_kv: int, kv_dtype: torch.dtype) -> None:
        """Record the context length of a call so that ``eval_roofline`` prices the bytes actually addressed."""
        self._seen_call = {
            "sum_len": int(real_seqlen_kv) * self.batch, "sum_pages": 0,
            "kv_bytes": torch.empty((), dtype=kv_dtype).element_size(), "fp8": kv_dtype == FP8,
        }

    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, k_scale: Optional[torch.Tensor] = None,
                v_scale: Optional[torch.Tensor] = None) -> torch.Tensor:
        self._validate_call(q, k, v, k_scale, v_scale)
        self.dtype = q.dtype
        real_seqlen_kv = k.shape[1]
        kernel = self._get_kernel((q, k, v, k_scale, v_scale), q.dtype, k.dtype)
        if k_scale is None:
            return kernel(q, k, v, real_seqlen_kv)
        return kernel(q, k, v, real_seqlen_kv, k_scale, v_scale)


def _paged_cache_dtype(cache_dtype: Optional[torch.dtype]) -> Optional[torch.dtype]:
    """``None`` follows the attention dtype; otherwise fp16, bf16 or float8_e4m3fn (gqa.py:57-63)."""
    if cache_dtype is None:
        return None
    if cache_dtype != FP8:
        _validate_attention_dtype(cache_dtype)
    return cache_dtype


class GroupedQueryAttentionPrefillPagedWithKVCacheFwdOp(Op):
    """Packed GQA prefill with paged KV cache append. Layout: THD.

    The current chunk is packed by request. ``cache_seqlens`` stores each request's logical KV length before append.
    ``block_table`` maps logical page ids to physical pages in ``k_pages`` / ``v_pages``.

    Keeps the reference op's contract (src/tileops/ops/attention/gqa.py:765-1157): constructor arguments, defaults and
    messages, the eleven ``forward`` arguments in order, the validation of devices, contiguity, shapes, dtypes, scale
    values, ``cu_seqlens_q`` / ``cache_seqlens`` consistency, capacity and block-table range (:897-1046; like the
    reference it reads a few device scalars to do so -- ``validate_inputs=False`` skips exactly those reads).  With ``fuse_rope=True`` (16-bit cache only, as in the reference)
    query and new key rows are rotated at their logical positions before the append; the cos/sin tables are built once
    per (device, dtype) like the reference's (:1048-1065, src/tileops/ops/rope.py:97-120).

    Under ``torch.compile(fullgraph=True)`` the op traces to one operator when built with ``validate_inputs=False``; the
    value checks read device memory on the host, which no graph can hold (the reference's checks do the same).
    """

    compile_op_names = ("tileops_amd::gqa_prefill_paged", "tileops_amd::gqa_prefill_paged_rope")

    def __init__(self, batch: int, heads: int, heads_kv: int, max_pages_per_req: int, page_size: int, dim: int,
                 is_causal: bool = True, cache_dtype: Optional[torch.dtype] = None, sm_scale: Optional[float] = None,
                 softcap: Optional[float] = None, kernel_map: Optional[Dict[str, type]] = None, tune: bool = False,
                 fuse_rope: bool = False, rope_base: float = 10000.0, max_position: Optional[int] = None,
                 rotary_dim: Optional[int] = None, *, target: Target = None, validate_inputs: bool = True) -> None:
        _validate_gqa_dims(heads, heads_kv, dim)
        # validate_inputs=False (not in the reference) keeps the shape / dtype / layout checks and drops those that
        # read device memory (scale values, cu_seqlens_q / cache_seqlens consistency, capacity, block-table range):
        # each is a device-to-host round trip during which the GPU idles.  The kernels clamp page ids into the pool.
        self.validate_inputs = validate_inputs
        if fuse_rope:
            rotary_dim = dim if rotary_dim is None else rotary_dim
            if rotary_dim <= 0 or rotary_dim % 2 != 0 or rotary_dim > dim:
                raise ValueError("rotary_dim must be a positive even number no larger than dim")
            if max_position is None:
                raise ValueError("max_position is required when fuse_rope=True")
            _validate_positive(max_position=max_position)
        elif rotary_dim is not None:
            raise ValueError("rotary_dim requires fuse_rope=True")
        _validate_positive(batch=batch, max_pages_per_req=max_pages_per_req, page_size=page_size)
        if page_size & (page_size - 1) != 0:
            raise ValueError("page_size must be a power of two")
        cache_dtype = _paged_cache_dtype(cache_dtype)
        if fuse_rope and cache_dtype == FP8:
            raise ValueError("fuse_rope is not supported with FP8 paged KV cache yet")
        self.batch, self.heads, self.heads_kv, self.groups = batch, heads, heads_kv, heads // heads_kv
        self.max_pages_per_req, self.page_size = max_pages_per_req, page_size
        self.max_cache_len = max_pages_per_req * page_size
        self.dim, self.is_causal, self.cache_dtype = dim, is_causal, cache_dtype
        self.sm_scale = _attention_scale(dim, sm_scale)
        self.softcap = _score_softcap(softcap)
        self.fuse_rope, self.rope_base, self.max_position, self.rotary_dim = fuse_rope, rope_base, max_position, rotary_dim
        self._rope_cos_cache: Dict[tuple, tuple] = {}
        self.tune = tune
        if target is not None:
            self.target = target
        self.dispatch_kernel(kernel_map)

    @property
    def default_kernel_map(self) -> Dict[str, type]:
        return {
            "gqa_prefill_paged_with_kv_cache_rope_fwd_kernel": GQAPrefillPagedWithKVCacheRopeFwdKernel,
            "gqa_prefill_paged_with_kv_cache_fwd_kernel": GQAPrefillPagedWithKVCacheFwdKernel,
            "gqa_prefill_paged_with_fp8_kv_cache_fwd_kernel": GQAPrefillPagedWithFP8KVCacheFwdKernel,
        }

    def _rope_tables(self, device: torch.device, dtype: torch.dtype) -> "tuple[Optional[torch.Tensor], Optional[torch.Tensor]]":
        """cos/sin ``[max_position, rotary_dim / 2]`` in *dtype*: angle = position * base**(-i / half), computed in fp32
        (src/tileops/ops/rope.py:116-120), cached per (device, dtype) (gqa.py:1048-1065)."""
        if not self.fuse_rope:
            return None, None
        cached = self._rope_cos_cache.get((device, dtype))
        if cached is None:
            half = self.rotary_dim // 2
            freqs = 1.0 / (self.rope_base ** (torch.arange(0, half, device=device, dtype=torch.float32) / half))
            angles = torch.outer(torch.arange(self.max_position, device=device, dtype=torch.float32), freqs)
            cached = (torch.cos(angles).to(dtype).contiguous(), torch.sin(angles).to(dtype).contiguous())
            self._rope_cos_cache[(device, dtype)] = cached
        return cached

    def _resolved_cache_dtype(self, dtype: torch.dtype) -> torch.dtype:
        return dtype if self.cache_dtype is None else self.cache_dtype

    def attention_call(self, dtype: torch.dtype, device: Optional[torch.device] = None) -> PrefillCall:
        index = device.index if device is not None and device.type == "cuda" else None
        return PrefillCall(
            dtype=dtype, batch=self.batch, heads=self.heads, heads_kv=self.heads_kv, dim=self.dim,
            max_pages_per_req=self.max_pages_per_req, page_size=self.page_size, is_causal=self.is_causal,
            sm_scale=self.sm_scale, softcap=self.softcap, cache_dtype=self._resolved_cache_dtype(dtype),
            fuse_rope=self.fuse_rope, max_position=self.max_position, rotary_dim=self.rotary_dim, tune=self.tune,
            arch=get_arch(index))

    def _get_kernel(self, inputs: "tuple[torch.Tensor | None, ...]", key: str, call: PrefillCall):
        device = next((t.device for t in inputs if t is not None), None)

        def build():
            return self.kernel_map[key](
                batch=call.batch, heads=call.heads, heads_kv=call.heads_kv, max_pages_per_req=call.max_pages_per_req,
                page_size=call.page_size, dim=call.dim, is_causal=call.is_causal, dtype=call.dtype, sm_scale=call.sm_scale,
                softcap=call.softcap, max_position=call.max_position, rotary_dim=call.rotary_dim, tune=call.tune,
                device_index=device.index if device is not None and device.type == "cuda" else None)

        return self.get_or_build_kernel(key, inputs, key=call.dtype, build=build)

    def _validate_forward_inputs(self, q, k_new, v_new, k_pages, v_pages, k_scale, v_scale, cu_seqlens_q, cache_seqlens,
                                 block_table, max_seqlen_q) -> None:
        tensors = {"q": q, "k_new": k_new, "v_new": v_new, "k_pages": k_pages, "v_pages": v_pages, "k_scale": k_scale,
                   "v_scale": v_scale, "cu_seqlens_q": cu_seqlens_q, "cache_seqlens": cache_seqlens, "block_table": block_table}
        for name, t in tensors.items():
            if t.device.type != "cuda":
                raise ValueError(f"{name} must be on a cuda device, got {t.device}")
            if not t.is_contiguous():
                raise ValueError(f"{name} must be contiguous")
        q_tail, kv_tail = (self.heads, self.dim), (self.heads_kv, self.dim)
        if q.ndim != 3 or tuple(q.shape[1:]) != q_tail:
            raise ValueError(f"q must have shape [total_q, {self.heads}, {self.dim}], got {q.shape}")
        if k_new.ndim != 3 or tuple(k_new.shape[1:]) != kv_tail:
            raise ValueError(f"k_new must have shape [total_q, {self.heads_kv}, {self.dim}], got {k_new.shape}")
        if v_new.shape != k_new.shape:
            raise ValueError(f"v_new must have the same shape as k_new, got {v_new.shape} and {k_new.shape}")
        if k_new.shape[0] != q.shape[0]:
            raise ValueError(f"k_new.shape[0] ({k_new.shape[0]}) must equal q.shape[0] ({q.shape[0]})")
        if k_pages.ndim != 3 or tuple(k_pages.shape[1:]) != kv_tail:
            raise ValueError(f"k_pages must have shape [physical_tokens, {self.heads_kv}, {self.dim}], got {k_pages.shape}")
        if v_pages.shape != k_pages.shape:
            raise ValueError(f"v_pages must have the same shape as k_pages, got {v_pages.shape} and {k_pages.shape}")
        if k_pages.shape[0] % self.page_size != 0:
            raise ValueError("k_pages physical token dimension must be divisible by page_size")
        if k_scale.shape != (1,) or v_scale.shape != (1,):
            raise ValueError(f"k_scale and v_scale must have shape (1,), got {k_scale.shape} and {v_scale.shape}")
        if cu_seqlens_q.shape != (self.batch + 1,):
            raise ValueError(f"cu_seqlens_q shape must be ({self.batch + 1},), got {tuple(cu_seqlens_q.shape)}")
        if cache_seqlens.shape != (self.batch,):
            raise ValueError(f"cache_seqlens shape must be ({self.batch},), got {tuple(cache_seqlens.shape)}")
        if block_table.shape != (self.batch, self.max_pages_per_req):
            raise ValueError(f"block_table shape must be ({self.batch}, {self.max_pages_per_req}), got {tuple(block_table.shape)}")
        _validate_attention_dtype(q.dtype)
        cache_dtype = self._resolved_cache_dtype(q.dtype)
        if cache_dtype != q.dtype and cache_dtype != FP8:
            raise ValueError(f"cache_dtype must be either same as the q element type or torch.float8_e4m3fn, got {cache_dtype}")
        for name, t in (("k_new", k_new), ("v_new", v_new)):
            if t.dtype != q.dtype:
                raise ValueError(f"Expected {name}.dtype {q.dtype}, got {t.dtype}")
        for name, t in (("k_pages", k_pages), ("v_pages", v_pages)):
            if t.dtype != cache_dtype:
                raise ValueError(f"Expected {name}.dtype {cache_dtype}, got {t.dtype}")
        for name, t in (("k_scale", k_scale), ("v_scale", v_scale)):
            if t.dtype != torch.float32:
                raise ValueError(f"{name} must have dtype torch.float32, got {t.dtype}")
        for name, t in (("cu_seqlens_q", cu_seqlens_q), ("cache_seqlens", cache_seqlens), ("block_table", block_table)):
            if t.dtype != torch.int32:
                raise ValueError(f"{name} must have dtype torch.int32, got {t.dtype}")
        if not self.validate_inputs:
            return
        # The value checks of the reference (gqa.py:997-1040), in its order and with its messages.  The reference reads
        # each fact from the device on its own (five to seven round trips with the GPU idle in between); here the facts
        # are reduced by one small kernel of the library into ten integers that cross to the host once.
        facts = native.prefill_input_facts(cu_seqlens_q, cache_seqlens, block_table, k_scale if cache_dtype == FP8 else None,
                                           v_scale if cache_dtype == FP8 else None)
        for name, ok in zip(("k_scale", "v_scale"), facts[:2]):
            if not ok:
                raise ValueError(f"{name} must contain finite positive values")
        facts = facts[2:]
        cu_first, min_q, total_q, actual_max_q, min_cache, max_total_len, min_page, max_page = (int(x) for x in facts)
        if cu_first != 0:
            raise ValueError("cu_seqlens_q[0] must be 0")
        if min_q < 0:
            raise ValueError("cu_seqlens_q must be non-decreasing")
        if total_q != q.shape[0]:
            raise ValueError(f"cu_seqlens_q[-1] ({total_q}) must equal q.shape[0] ({q.shape[0]})")
        if max_seqlen_q < actual_max_q:
            raise ValueError(f"max_seqlen_q ({max_seqlen_q}) must be >= actual max Q sequence length ({actual_max_q})")
        if min_cache < 0:
            raise ValueError("cache_seqlens must be non-negative")
        if max_total_len > self.max_cache_len:
            raise ValueError("cache_seqlens + q_len exceeds paged KV capacity: "
                             f"max total length {max_total_len}, capacity {self.max_cache_len}")
        if self.fuse_rope and max_total_len > self.max_position:
            raise ValueError("cache_seqlens + q_len exceeds RoPE max_position: "
                             f"max total length {max_total_len}, max_position {self.max_position}")
        num_pages = k_pages.shape[0] // self.page_size
        if min_page < 0:
            raise ValueError("block_table must contain non-negative physical page ids")
        if max_page >= num_pages:
            raise ValueError(f"block_table references page {max_page}, but only {num_pages} pages exist")

    def _infer_output_shapes(self, q_shape, k_new_shape, v_new_shape, k_pages_shape, v_pages_shape, k_scale_shape,
                             v_scale_shape, cu_seqlens_q_shape, cache_seqlens_shape, block_table_shape) -> dict[str, tuple[int, ...]]:
        """Manifest ``shape_rules``: ``o.shape == q.shape``."""
        return {"o": tuple(q_shape)}

    def forward(self, q: torch.Tensor, k_new: torch.Tensor, v_new: torch.Tensor, k_pages: torch.Tensor,
                v_pages: torch.Tensor, k_scale: torch.Tensor, v_scale: torch.Tensor, cu_seqlens_q: torch.Tensor,
                cache_seqlens: torch.Tensor, block_table: torch.Tensor, max_seqlen_q: int) -> torch.Tensor:
        self._validate_forward_inputs(q, k_new, v_new, k_pages, v_pages, k_scale, v_scale, cu_seqlens_q, cache_seqlens,
                                      block_table, max_seqlen_q)
        self.dtype = q.dtype
        inputs = (q, k_new, v_new, k_pages, v_pages, k_scale, v_scale, cu_seqlens_q, cache_seqlens, block_table)
        call = self.attention_call(q.dtype, q.device)
        key = self.select_kernel_key(PAGED_PREFILL_KEYS, call)
        cos_table, sin_table = self._rope_tables(q.device, q.dtype)
        return self._get_kernel(inputs, key, call)(*inputs, max_seqlen_q, cos_table, sin_table)

    @property
    def total_flops(self) -> int:
        raise NotImplementedError("total_flops is not defined for paged varlen ops; "
                                  "compute per-sample from cu_seqlens and cache_seqlens at call time.")

    @property
    def total_memory(self) -> int:
        raise NotImplementedError("total_memory is not defined for paged varlen ops; "
                                  "compute per-sample from cu_seqlens and cache_seqlens at call time.")
