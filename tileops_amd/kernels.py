"""L1 host wrappers of the gfx950 HIP kernels.

``Kernel`` reproduces the lifecycle of the reference's kernel base
(src/tileops/kernels/kernel_base.py:47-365): architecture check at construction, ``config`` /
``default_config`` / ``autotune_configs``, and the selection protocol ``applies`` / ``general`` /
``refusal``.  The two concrete classes take the place of ``GQADecodePagedKernel``
(src/tileops/kernels/attention/gqa_decode_paged.py:513-746) and of the specialised sibling
(``GQADecodePagedBs1Kernel``, src/tileops/kernels/attention/gqa_decode_bs1_paged.py:177-299): the general
VALU kernel serves every call, the MFMA kernel states the narrower region it serves and wins there.

Nothing here computes attention: ``forward`` allocates the output and the workspace with torch and
enqueues the HIP kernels through the C ABI.  No host read-back of device data happens on the call path.
"""

from __future__ import annotations

import functools
import itertools
from dataclasses import dataclass
from typing import Any, Optional

import torch

from . import custom_ops as _custom_ops  # noqa: F401 - registers torch.ops.tileops_amd.*
from . import native

__all__ = [
    "AttentionCall", "DECODE_KEYS", "GQADecodeKernel", "GQADecodeMfmaKernel", "GQADecodePagedKernel",
    "GQADecodePagedMfmaKernel", "GQAPrefillPagedWithFP8KVCacheFwdKernel", "GQAPrefillPagedWithKVCacheFwdKernel",
    "GQAPrefillPagedWithKVCacheRopeFwdKernel", "Kernel",
    "PAGED_DECODE_KEYS", "PAGED_PREFILL_KEYS", "PrefillCall",
    "gqa_decode_paged_block_n", "gqa_decode_paged_block_ns", "get_arch", "mfma_kernel_serves",
]

#: Dispatch keys of the paged decode ops, in no particular order (selection never reads the order).
PAGED_DECODE_KEYS = ("gqa_decode_paged_kernel", "gqa_decode_paged_mfma_kernel")
#: Dispatch keys of the paged prefill op (reference: src/tileops/ops/attention/selection.py:37-42).
PAGED_PREFILL_KEYS = ("gqa_prefill_paged_with_kv_cache_rope_fwd_kernel", "gqa_prefill_paged_with_fp8_kv_cache_fwd_kernel",
                      "gqa_prefill_paged_with_kv_cache_fwd_kernel")
#: Dispatch keys of the contiguous-cache decode op.
DECODE_KEYS = ("gqa_decode_kernel", "gqa_decode_mfma_kernel")

GFX950_ARCH = 95  # torch.cuda.get_device_capability() == (9, 5) on gfx950


@torch._dynamo.assume_constant_result
def _arch_of(device_index: Optional[int]) -> Optional[int]:
    # (a constant to the tracer: asked once while a graph is being built, never a node of it)
    if not torch.cuda.is_available():
        return None
    major, minor = torch.cuda.get_device_capability(device_index)
    return major * 10 + minor


@functools.lru_cache(maxsize=None)
def get_arch(device_index: Optional[int] = None) -> Optional[int]:
    """major*10+minor of a ROCm device, or None when no GPU is visible."""
    return _arch_of(device_index)


def _as_torch_dtype(dtype: Any) -> torch.dtype:
    if isinstance(dtype, torch.dtype):
        return dtype
    return getattr(torch, str(dtype))


@dataclass(frozen=True)
class AttentionCall:
    """Facts of one decode call that kernel selection filters on (``page_size`` 0 = contiguous cache)
    (reference: src/tileops/kernels/attention/call_spec.py:44-76, kernels/call_spec.py:8-42)."""

    dtype: torch.dtype
    batch: int
    heads: int
    heads_kv: int
    seqlen_kv: int
    dim: int
    page_size: int
    sm_scale: float
    softcap: float
    tune: bool = False
    kv_dtype: Optional[torch.dtype] = None
    q_len: int = 1
    is_causal: bool = True
    arch: Optional[int] = None

    @property
    def group(self) -> int:
        return self.heads // self.heads_kv


def mfma_kernel_serves(dim: int, page_size: int, dtype: torch.dtype, kv_dtype: torch.dtype) -> bool:
    """The region the library's MFMA kernel serves (``mfma_supported`` in csrc/paged_decode_mfma.hip; a test holds the
    two together): head dim 64, 128 or 256, pages of 16 tokens or a multiple of 32, a 16-bit cache of the query's type or
    an FP8-e4m3fn cache.  Stated here in plain Python so that kernel selection is traceable by ``torch.compile``."""
    if dtype not in (torch.float16, torch.bfloat16):
        return False
    if kv_dtype != torch.float8_e4m3fn and kv_dtype != dtype:
        return False
    return dim in (64, 128, 256) and (page_size == 16 or (page_size > 0 and page_size % 32 == 0))


def gqa_decode_paged_block_ns(page_size: int) -> tuple[int, ...]:
    """KV tile heights that cover a page exactly, widest first.

    Same rule and same messages as the reference (gqa_decode_paged.py:21-33): 128 or 64 when they divide
    the page, the page itself below 64, otherwise the layout is rejected.
    """
    if page_size <= 0:
        raise ValueError("page_size must be positive")
    fits = tuple(n for n in (128, 64) if n <= page_size and page_size % n == 0)
    if fits:
        return fits
    if page_size < 64:
        return (page_size,)
    raise ValueError(f"page_size={page_size} matches no supported block_N")


def gqa_decode_paged_block_n(page_size: int) -> int:
    return gqa_decode_paged_block_ns(page_size)[0]


class Kernel:
    """Base of the host-side kernel wrappers."""

    supported_archs: Optional[list[int]] = None
    #: True for the implementation that runs where no specialised one applies.
    general: bool = False
    autotune_configs: Optional[list[dict]] = None

    def __init__(self, *, device_index: Optional[int] = None) -> None:
        self.device_index = device_index
        self._check_arch()
        self.config: dict[str, Any] = {}

    @classmethod
    def applies(cls, call: Any) -> bool:
        return True

    @classmethod
    def refusal(cls, call: Any) -> Optional[str]:
        """Why this class cannot serve *call*, or None when it can."""
        archs = cls.supported_archs
        if archs is not None and call.arch not in archs:
            return f"built for architectures {sorted(archs)}, device reports {call.arch}"
        if not cls.applies(call):
            return "does not serve this call"
        return None

    def _check_arch(self) -> None:
        cls = type(self)
        if cls.supported_archs is None:
            return
        arch = get_arch(self.device_index)
        if arch not in cls.supported_archs:
            where = "the current device" if self.device_index is None else f"cuda:{self.device_index}"
            raise ValueError(
                f"{cls.__name__} is built for architectures {sorted(cls.supported_archs)}, but {where} reports {arch}"
            )

    @property
    def default_config(self) -> dict[str, Any]:
        return {}

    def init_config(self, config: Optional[dict[str, Any]] = None, tune: bool = False) -> None:
        if tune and not self.autotune_configs:
            tune = False
        if tune:
            self.autotune()
        elif config is not None:
            self.config = {k: (config[k] if config.get(k) is not None else v) for k, v in self.default_config.items()}
        else:
            self.config = dict(self.default_config)

    def autotune(self) -> None:
        raise NotImplementedError

    def forward(self, *args: Any, **kwargs: Any) -> Any:
        raise NotImplementedError

    def __call__(self, *args: Any, **kwargs: Any) -> Any:
        return self.forward(*args, **kwargs)


class GQADecodePagedKernel(Kernel):
    """General paged GQA decode on gfx950: the VALU HIP kernel plus fp32 split-KV combine.

    Constructor arguments follow the reference class (gqa_decode_paged.py:526-538); ``groups`` is the
    number of KV heads, as there.  ``kv_dtype`` (default: same as ``dtype``), ``q_len`` and ``is_causal``
    are this package's extensions for an FP8 cache and multi-token queries.
    """

    supported_archs = [GFX950_ARCH]
    general = True
    _native_kernel = native.KERNEL_GENERIC

    def __init__(self, batch: int, heads: int, groups: int, seqlen_kv: int, dim: int, page_size: int,
                 dtype: Any = "float16", sm_scale: Optional[float] = None, softcap: float = 0.0,
                 config: Optional[dict] = None, tune: bool = False, *, kv_dtype: Any = None, q_len: int = 1,
                 is_causal: bool = True, device_index: Optional[int] = None) -> None:
        super().__init__(device_index=device_index)
        self.batch, self.heads, self.groups, self.seqlen_kv = batch, heads, groups, seqlen_kv
        self.dim, self.page_size = dim, page_size
        self.dtype = _as_torch_dtype(dtype)
        self.kv_dtype = self.dtype if kv_dtype is None else _as_torch_dtype(kv_dtype)
        self.q_len, self.is_causal = q_len, is_causal
        self.sm_scale = dim ** -0.5 if sm_scale is None else sm_scale
        self.softcap = softcap
        self._supported_block_ns = gqa_decode_paged_block_ns(page_size)
        if config is not None:
            block_n = config.get("block_N")
            if block_n is not None and block_n not in self._supported_block_ns:
                raise ValueError(f"block_N={block_n} is not supported for page_size={page_size}")
        if self.groups <= 0:
            raise ValueError("groups must be positive")
        if self.heads % self.groups != 0:
            raise ValueError("heads must be divisible by groups")
        if self.seqlen_kv <= 0:
            raise ValueError("seqlen_kv must be positive")
        if self.page_size <= 0:
            raise ValueError("page_size must be positive")
        if self.seqlen_kv % self.page_size != 0:
            raise ValueError("seqlen_kv must be divisible by page_size")
        self.init_config(config, tune)

    # -- config ----------------------------------------------------------------------------------------
    @property
    def default_config(self) -> dict[str, Any]:
        # block_N is the page-contained tile the launch assumes; num_split 0 lets the library choose
        return {"block_N": gqa_decode_paged_block_n(self.page_size), "num_split": 0}

    @property
    def autotune_configs(self) -> list[dict]:
        return [{"block_N": n, "num_split": s} for n, s in itertools.product(self._supported_block_ns, (0, 8, 16, 32))]

    def autotune(self) -> None:
        """Time every ``autotune_configs`` entry on synthetic full-length inputs and keep the fastest."""
        device = torch.device("cuda", self.device_index if self.device_index is not None else torch.cuda.current_device())
        n_pages = self.seqlen_kv // self.page_size
        q_shape = (self.batch, self.heads, self.dim) if self.q_len == 1 else (self.batch, self.q_len, self.heads, self.dim)
        q = torch.randn(q_shape, device=device, dtype=self.dtype)
        kv = torch.randn(2, self.seqlen_kv, self.groups, self.dim, device=device, dtype=torch.float32)
        if self.kv_dtype == torch.float8_e4m3fn:
            k, v = kv[0].clamp(-448, 448).to(self.kv_dtype), kv[1].clamp(-448, 448).to(self.kv_dtype)
            ks = torch.full((self.seqlen_kv, self.groups), 0.01, device=device, dtype=torch.float32)
            vs = ks.clone()
        else:
            k, v, ks, vs = kv[0].to(self.kv_dtype), kv[1].to(self.kv_dtype), None, None
        lens = torch.full((self.batch,), self.seqlen_kv, dtype=torch.int32, device=device)
        table = torch.arange(n_pages, dtype=torch.int32, device=device).unsqueeze(0).expand(self.batch, -1).contiguous()
        best, best_ms = None, float("inf")
        for cfg in self.autotune_configs:
            self.config = dict(cfg)
            for _ in range(3):
                self.forward(q, k, v, lens, table, ks, vs)
            start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            for _ in range(10):
                self.forward(q, k, v, lens, table, ks, vs)
            stop.record()
            stop.synchronize()
            ms = start.elapsed_time(stop) / 10
            if ms < best_ms:
                best, best_ms = dict(cfg), ms
        self.config = best

    # -- launch ----------------------------------------------------------------------------------------
    #: Measurement aid: when True, ``forward`` launches the attention kernel alone (no combine), so a benchmark
    #: can time the dominant kernel by itself.  The returned tensor is then incomplete.
    attention_kernel_only: bool = False

    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, real_seqlen_kv: torch.Tensor,
                block_table: torch.Tensor, k_scale: Optional[torch.Tensor] = None,
                v_scale: Optional[torch.Tensor] = None) -> torch.Tensor:
        # one registered operator (custom_ops.py): output and workspace are allocated inside it, so a compiled caller
        # sees a single graph node
        return torch.ops.tileops_amd.gqa_paged_decode(
            q, k, v, real_seqlen_kv, block_table, k_scale, v_scale, self.q_len, self.heads, self.groups, self.dim,
            self.page_size, float(self.sm_scale), float(self.softcap), bool(self.is_causal),
            int(self.config.get("num_split", 0) or 0),
            self._native_kernel | (native.KERNEL_FLAG_SKIP_COMBINE if self.attention_kernel_only else 0))


class GQADecodePagedMfmaKernel(GQADecodePagedKernel):
    """MFMA paged GQA decode on gfx950: direct-to-LDS page gather, QK^T and PV on the matrix cores, the KV
    tile stream partitioned evenly over all compute units.  Serves the region the HIP library reports as
    supported (head dims 64, 128, 256, page size 16 or a multiple of 32, ...); everything else stays on the general kernel."""

    general = False
    _native_kernel = native.KERNEL_MFMA

    @classmethod
    def applies(cls, call: AttentionCall) -> bool:
        return mfma_kernel_serves(call.dim, call.page_size, call.dtype, call.kv_dtype or call.dtype)

    @property
    def default_config(self) -> dict[str, Any]:
        return {"block_N": gqa_decode_paged_block_n(self.page_size), "num_split": 0}

    @property
    def autotune_configs(self) -> list[dict]:
        """``num_split`` is the number of equal ranges the KV tile stream is cut into (0 = one per resident wave, the
        library's own choice).  The candidates are that choice and whole multiples / halves of it: the grid then stays a
        whole number of rounds over the compute units (a count in between leaves a round part-filled and measured
        25-30 % slower on the Llama-3-8B shapes; two rounds of half-length ranges cost 3-7 % there, and pay only where
        the sequences are too few and too uneven for one round to balance)."""
        block_n = gqa_decode_paged_block_n(self.page_size)
        _, auto, _ = native.decode_workspace(self.batch, self.q_len, self.heads, self.groups, self.dim, self.page_size, 1,
                                             self.dtype, self.kv_dtype, 0, native.KERNEL_MFMA)
        counts = [0] + [n for n in (auto // 2, 2 * auto, 4 * auto) if n >= 1]
        return [{"block_N": block_n, "num_split": n} for n in counts]


class GQADecodeKernel(Kernel):
    """General GQA decode over a contiguous ``[batch, N_kv, heads_kv, dim]`` cache on gfx950: the VALU HIP kernel
    with identity addressing plus the fp32 split-KV combine.

    Constructor arguments and the default split policy follow the reference class
    (src/tileops/kernels/attention/gqa_decode.py:426-449, :511-553); ``groups`` is the number of KV heads, as
    there.  ``forward(Q, K, V, real_seqlen_kv)`` reads only the first ``real_seqlen_kv`` tokens of each
    sequence, so the cache needs no padding up to ``seqlen_kv``.  ``kv_dtype`` is this package's FP8 extension.
    """

    supported_archs = [GFX950_ARCH]
    general = True
    _native_kernel = native.KERNEL_GENERIC

    def __init__(self, batch: int, heads: int, groups: int, seqlen_kv: int, dim: int, dtype: Any = "float16",
                 sm_scale: Optional[float] = None, softcap: float = 0.0, config: Optional[dict] = None,
                 tune: bool = False, *, kv_dtype: Any = None, device_index: Optional[int] = None) -> None:
        super().__init__(device_index=device_index)
        self.batch, self.heads, self.groups, self.seqlen_kv, self.dim = batch, heads, groups, seqlen_kv, dim
        self.dtype = _as_torch_dtype(dtype)
        self.kv_dtype = self.dtype if kv_dtype is None else _as_torch_dtype(kv_dtype)
        self.sm_scale = dim ** -0.5 if sm_scale is None else sm_scale
        self.softcap = softcap
        if self.groups <= 0:
            raise ValueError("groups must be positive")
        if self.heads % self.groups != 0:
            raise ValueError("heads must be divisible by groups")
        if self.seqlen_kv <= 0:
            raise ValueError("seqlen_kv must be positive")
        self.init_config(config, tune)

    def _default_num_split(self) -> int:
        """Reference policy (gqa_decode.py:520-532): 32 splits for single-request decode with at most two KV
        heads and a query group of at least eight, 16 otherwise, never more than there are tokens."""
        kv_group_num = self.heads // self.groups
        candidate = 32 if (self.batch == 1 and self.dim == 128 and self.groups <= 2 and kv_group_num >= 8) else 16
        return min(candidate, self.seqlen_kv)

    @property
    def default_config(self) -> dict[str, Any]:
        return {"num_split": self._default_num_split()}

    @property
    def autotune_configs(self) -> list[dict]:
        return [{"num_split": ns} for ns in ([n for n in (2, 4, 8, 16, 32) if n <= self.seqlen_kv] or [1])]

    def autotune(self) -> None:
        device = torch.device("cuda", self.device_index if self.device_index is not None else torch.cuda.current_device())
        q = torch.randn(self.batch, self.heads, self.dim, device=device, dtype=self.dtype)
        kv = torch.randn(2, self.batch, self.seqlen_kv, self.groups, self.dim, device=device, dtype=torch.float32)
        if self.kv_dtype == torch.float8_e4m3fn:
            k, v = kv[0].clamp(-448, 448).to(self.kv_dtype), kv[1].clamp(-448, 448).to(self.kv_dtype)
            ks = torch.full((self.batch, self.seqlen_kv, self.groups), 0.01, device=device, dtype=torch.float32)
            vs = ks.clone()
        else:
            k, v, ks, vs = kv[0].to(self.kv_dtype), kv[1].to(self.kv_dtype), None, None
        best, best_ms = None, float("inf")
        for cfg in self.autotune_configs:
            self.config = dict(cfg)
            for _ in range(3):
                self.forward(q, k, v, self.seqlen_kv, ks, vs)
            start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            for _ in range(10):
                self.forward(q, k, v, self.seqlen_kv, ks, vs)
            stop.record()
            stop.synchronize()
            ms = start.elapsed_time(stop) / 10
            if ms < best_ms:
                best, best_ms = dict(cfg), ms
        self.config = best

    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, real_seqlen_kv: int,
                k_scale: Optional[torch.Tensor] = None, v_scale: Optional[torch.Tensor] = None) -> torch.Tensor:
        if real_seqlen_kv > self.seqlen_kv:
            raise ValueError(f"real_seqlen_kv={real_seqlen_kv} exceeds the seqlen_kv={self.seqlen_kv} this kernel was built for")
        return torch.ops.tileops_amd.gqa_decode(
            q, k, v, k_scale, v_scale, int(real_seqlen_kv), self.heads, self.groups, self.dim, float(self.sm_scale),
            float(self.softcap), True, int(self.config.get("num_split", 0) or 0), self._native_kernel)


class GQADecodeMfmaKernel(GQADecodeKernel):
    """MFMA GQA decode over a contiguous cache: the paged MFMA kernel with identity addressing.  Takes the place of
    the reference's specialised sibling (``GQADecodeBs1Kernel``, src/tileops/kernels/attention/gqa_decode_bs1.py):
    it states the narrower region it serves (head dims 64, 128, 256, ...) and wins there, for any batch."""

    general = False
    _native_kernel = native.KERNEL_MFMA

    @classmethod
    def applies(cls, call: AttentionCall) -> bool:
        return mfma_kernel_serves(call.dim, 32, call.dtype, call.kv_dtype or call.dtype)  # (walked in 32-token tiles)

    @property
    def default_config(self) -> dict[str, Any]:
        return {"num_split": 0}  # the tile stream is cut evenly over the chip; there is nothing to choose

    @property
    def autotune_configs(self) -> list[dict]:
        return [dict(self.default_config)]


@dataclass(frozen=True)
class PrefillCall:
    """Facts of one paged prefill call that kernel selection filters on
    (reference: src/tileops/ops/attention/gqa.py:843-861, the fields of ``attention_call``)."""

    dtype: torch.dtype
    batch: int
    heads: int
    heads_kv: int
    dim: int
    max_pages_per_req: int
    page_size: int
    is_causal: bool
    sm_scale: float
    softcap: float
    cache_dtype: torch.dtype
    fuse_rope: bool = False
    max_position: Optional[int] = None
    rotary_dim: Optional[int] = None
    tune: bool = False
    arch: Optional[int] = None


class GQAPrefillPagedWithKVCacheFwdKernel(Kernel):
    """Packed GQA prefill chunk with paged-cache append, cache element type = attention element type.

    Constructor keywords and ``forward`` argument order follow the reference class
    (src/tileops/kernels/attention/gqa_fwd.py:938-1003 and its base).  One library call appends the chunk to the
    pages and runs attention over old + new tokens with the decode kernels (every query row of a chunk is a
    decode query; chunks of different lengths are packed).  Long chunks re-stream the keys once per 32-64 query
    rows of a kv head: the layout is right for chunked prefill next to decode, not for long prompts.
    """

    supported_archs = [GFX950_ARCH]
    general = True
    _cache_is_fp8 = False

    @classmethod
    def applies(cls, call: PrefillCall) -> bool:
        return not call.fuse_rope and call.cache_dtype == call.dtype

    def __init__(self, *, batch: int, heads: int, heads_kv: int, max_pages_per_req: int, page_size: int, dim: int,
                 is_causal: bool = True, dtype: Any = "float16", sm_scale: Optional[float] = None, softcap: float = 0.0,
                 max_position: Optional[int] = None, rotary_dim: Optional[int] = None, config: Optional[dict] = None,
                 tune: bool = False, device_index: Optional[int] = None) -> None:
        super().__init__(device_index=device_index)
        self.batch, self.heads, self.heads_kv, self.dim = batch, heads, heads_kv, dim
        self.max_pages_per_req, self.page_size, self.is_causal = max_pages_per_req, page_size, is_causal
        self.dtype = _as_torch_dtype(dtype)
        self.sm_scale = dim ** -0.5 if sm_scale is None else sm_scale
        self.softcap = softcap
        self.init_config(config, tune)

    @property
    def default_config(self) -> dict[str, Any]:
        return {"kernel": native.KERNEL_AUTO}

    @property
    def autotune_configs(self) -> list[dict]:
        return [{"kernel": native.KERNEL_AUTO}, {"kernel": native.KERNEL_GENERIC}]

    def forward(self, q: torch.Tensor, k_new: torch.Tensor, v_new: torch.Tensor, k_pages: torch.Tensor,
                v_pages: torch.Tensor, k_scale: Optional[torch.Tensor], v_scale: Optional[torch.Tensor],
                cu_seqlens_q: torch.Tensor, cache_seqlens: torch.Tensor, block_table: torch.Tensor, max_seqlen_q: int,
                cos_table: Optional[torch.Tensor] = None, sin_table: Optional[torch.Tensor] = None) -> torch.Tensor:
        if cos_table is not None or sin_table is not None:
            raise ValueError(f"{type(self).__name__} takes no rotary tables; the fused-RoPE call is served by "
                             "GQAPrefillPagedWithKVCacheRopeFwdKernel")
        kernel = int(self.config.get("kernel", native.KERNEL_AUTO))
        if k_scale is None:  # never read with a 16-bit cache; the entry point wants a pointer all the same
            k_scale = v_scale = torch.ones(1, dtype=torch.float32, device=q.device)
        return torch.ops.tileops_amd.gqa_prefill_paged(
            q, k_new, v_new, k_pages, v_pages, k_scale, v_scale, cu_seqlens_q, cache_seqlens, block_table, int(max_seqlen_q),
            self.heads, self.heads_kv, self.dim, self.page_size, float(self.sm_scale), float(self.softcap), bool(self.is_causal),
            kernel)


class GQAPrefillPagedWithFP8KVCacheFwdKernel(GQAPrefillPagedWithKVCacheFwdKernel):
    """The same call against an FP8-e4m3fn cache with per-tensor scales (reference:
    src/tileops/kernels/attention/gqa_fwd.py:1005-1460): the chunk is quantised into the pages, attention reads the
    old tokens dequantised and the chunk's own tokens unquantised (two passes merged by log-sum-exp)."""

    general = False
    _cache_is_fp8 = True

    @classmethod
    def applies(cls, call: PrefillCall) -> bool:
        return not call.fuse_rope and call.cache_dtype == torch.float8_e4m3fn



class GQAPrefillPagedWithKVCacheRopeFwdKernel(GQAPrefillPagedWithKVCacheFwdKernel):
    """The 16-bit-cache call with rotary position embedding fused in (reference:
    src/tileops/kernels/attention/gqa_fwd.py:2020-2090 and the two TileLang kernels it launches, :1464-1582, :1660-1917):
    query and new key rows are rotated (GPT-NeoX halves, position = cached length + index in the chunk), the rotated keys
    are appended to the pages, attention runs over old + new tokens.  ``forward`` takes the cos/sin tables
    ``[max_position, rotary_dim / 2]`` in the element type as its last two arguments."""

    general = False

    @classmethod
    def applies(cls, call: PrefillCall) -> bool:
        return bool(call.fuse_rope) and call.cache_dtype == call.dtype

    def __init__(self, *, max_position: Optional[int] = None, rotary_dim: Optional[int] = None, **kwargs: Any) -> None:
        super().__init__(max_position=max_position, rotary_dim=rotary_dim, **kwargs)
        if rotary_dim is None or max_position is None:
            raise ValueError("GQAPrefillPagedWithKVCacheRopeFwdKernel requires max_position and rotary_dim")
        if rotary_dim <= 0 or rotary_dim % 2 != 0 or rotary_dim > self.dim:
            raise ValueError("rotary_dim must be positive, even, and <= dim")
        self.max_position, self.rotary_dim = max_position, rotary_dim

    def forward(self, q: torch.Tensor, k_new: torch.Tensor, v_new: torch.Tensor, k_pages: torch.Tensor,
                v_pages: torch.Tensor, k_scale: Optional[torch.Tensor], v_scale: Optional[torch.Tensor],
                cu_seqlens_q: torch.Tensor, cache_seqlens: torch.Tensor, block_table: torch.Tensor, max_seqlen_q: int,
                cos_table: Optional[torch.Tensor] = None, sin_table: Optional[torch.Tensor] = None) -> torch.Tensor:
        if cos_table is None or sin_table is None:
            raise ValueError("the fused-RoPE prefill kernel needs cos_table and sin_table")
        want = (self.max_position, self.rotary_dim // 2)
        for name, t in (("cos_table", cos_table), ("sin_table", sin_table)):
            if tuple(t.shape) != want or t.dtype != q.dtype or not t.is_contiguous() or t.device != q.device:
                raise ValueError(f"{name} must be a contiguous {q.dtype} tensor of shape {want} on {q.device}, got "
                                 f"{t.dtype} {tuple(t.shape)} on {t.device}")
        kernel = int(self.config.get("kernel", native.KERNEL_AUTO))
        return torch.ops.tileops_amd.gqa_prefill_paged_rope(
            q, k_new, v_new, k_pages, v_pages, cos_table, sin_table, cu_seqlens_q, cache_seqlens, block_table, int(max_seqlen_q),
            self.heads, self.heads_kv, self.dim, self.page_size, int(self.rotary_dim), float(self.sm_scale), float(self.softcap),
            bool(self.is_causal), kernel)
