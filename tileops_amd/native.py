"""ctypes binding of ``libmi355_tileops.so`` (the C ABI declared in ``include/mi355_tileops.h``).

torch is used here only for device memory and streams: tensors are handed over as raw ``data_ptr()``
values plus the current HIP stream.  There is no CPU or eager-torch fallback: if the library is missing
or the device is not a gfx950 GPU, calls raise.
"""

from __future__ import annotations

import ctypes
import threading
from pathlib import Path
from typing import Optional

import torch

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libmi355_tileops.so"
ABI_VERSION = 1

DT_BF16, DT_FP16, DT_FP8_E4M3FN = 0, 1, 2
KERNEL_AUTO, KERNEL_GENERIC, KERNEL_MFMA = 0, 1, 2
KERNEL_FLAG_SKIP_COMBINE = 0x100  # this package's benchmark only (csrc/common.h): attention kernel alone, partials left unmerged
KERNEL_NAMES = {KERNEL_AUTO: "auto", KERNEL_GENERIC: "generic", KERNEL_MFMA: "mfma"}

EXPORTED_SYMBOLS = (
    "mi355_abi_version",
    "mi355_last_error",
    "mi355_gqa_paged_decode_workspace",
    "mi355_gqa_paged_decode",
    "mi355_gqa_paged_decode_static",
    "mi355_gqa_decode_workspace",
    "mi355_gqa_decode",
    "mi355_gqa_prefill_paged_workspace",
    "mi355_gqa_prefill_paged",
    "mi355_gqa_prefill_paged_rope_workspace",
    "mi355_gqa_prefill_paged_rope",
    "mi355_gather_probe",
    "mi355_kv_append_fp8",
    "mi355_prefill_input_facts",
)


class NativeLibraryError(RuntimeError):
    """The HIP library is missing, stale, or reported an error."""


_lock = threading.Lock()
_lib: Optional[ctypes.CDLL] = None
_facts_local = threading.local()  # per-thread pinned buffer of prefill_input_facts

_c_int, _c_i64, _c_f32, _c_vp, _c_sz = ctypes.c_int, ctypes.c_int64, ctypes.c_float, ctypes.c_void_p, ctypes.c_size_t


def _declare(lib: ctypes.CDLL) -> None:
    lib.mi355_abi_version.restype = _c_int
    lib.mi355_abi_version.argtypes = []
    lib.mi355_last_error.restype = ctypes.c_char_p
    lib.mi355_last_error.argtypes = []
    lib.mi355_gqa_paged_decode_workspace.restype = _c_int
    lib.mi355_gqa_paged_decode_workspace.argtypes = [
        _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_i64, _c_int, _c_int, _c_int, _c_int,
        ctypes.POINTER(_c_sz), ctypes.POINTER(_c_int), ctypes.POINTER(_c_int),
    ]
    lib.mi355_gqa_paged_decode.restype = _c_int
    lib.mi355_gqa_paged_decode.argtypes = [
        _c_vp, _c_vp, _c_vp, _c_vp, _c_vp, _c_vp, _c_vp, _c_i64, _c_vp, _c_vp, _c_sz,
        _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_i64, _c_int, _c_int,
        _c_f32, _c_f32, _c_int, _c_int, _c_int, _c_vp,
    ]
    lib.mi355_gqa_paged_decode_static.restype = _c_int
    lib.mi355_gqa_paged_decode_static.argtypes = [
        _c_vp, _c_vp, _c_vp, _c_vp, _c_vp, _c_vp, _c_vp, _c_i64, _c_vp,
        _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_i64, _c_int, _c_int,
        _c_f32, _c_f32, _c_int, _c_int, _c_int, _c_vp,
    ]
    lib.mi355_gqa_decode_workspace.restype = _c_int
    lib.mi355_gqa_decode_workspace.argtypes = [
        _c_int, _c_int, _c_int, _c_int, _c_int, _c_i64, _c_int, _c_int, _c_int, _c_int,
        ctypes.POINTER(_c_sz), ctypes.POINTER(_c_int), ctypes.POINTER(_c_int),
    ]
    lib.mi355_gqa_decode.restype = _c_int
    lib.mi355_gqa_decode.argtypes = [
        _c_vp, _c_vp, _c_vp, _c_vp, _c_vp, _c_vp, _c_vp, _c_sz,
        _c_int, _c_int, _c_int, _c_int, _c_int, _c_i64, _c_int, _c_int, _c_int,
        _c_f32, _c_f32, _c_int, _c_int, _c_int, _c_vp,
    ]
    lib.mi355_gqa_prefill_paged_workspace.restype = _c_int
    lib.mi355_gqa_prefill_paged_workspace.argtypes = [
        _c_int, _c_int, _c_i64, _c_int, _c_int, _c_int, _c_int, _c_i64, _c_int, _c_int, _c_int, ctypes.POINTER(_c_sz),
    ]
    lib.mi355_gqa_prefill_paged.restype = _c_int
    lib.mi355_gqa_prefill_paged.argtypes = [
        _c_vp, _c_vp, _c_vp, _c_vp, _c_vp, _c_vp, _c_vp, _c_vp, _c_vp, _c_vp, _c_i64, _c_vp, _c_vp, _c_sz,
        _c_int, _c_int, _c_i64, _c_int, _c_int, _c_int, _c_int, _c_i64, _c_int, _c_int,
        _c_f32, _c_f32, _c_int, _c_int, _c_vp,
    ]
    lib.mi355_gqa_prefill_paged_rope_workspace.restype = _c_int
    lib.mi355_gqa_prefill_paged_rope_workspace.argtypes = [
        _c_int, _c_int, _c_i64, _c_int, _c_int, _c_int, _c_int, _c_i64, _c_int, _c_int, ctypes.POINTER(_c_sz),
    ]
    lib.mi355_gqa_prefill_paged_rope.restype = _c_int
    lib.mi355_gqa_prefill_paged_rope.argtypes = [
        _c_vp, _c_vp, _c_vp, _c_vp, _c_vp, _c_vp, _c_vp, _c_vp, _c_vp, _c_vp, _c_i64, _c_vp, _c_vp, _c_sz,
        _c_int, _c_int, _c_i64, _c_int, _c_int, _c_int, _c_int, _c_i64, _c_int, _c_int, _c_i64,
        _c_f32, _c_f32, _c_int, _c_int, _c_vp,
    ]
    lib.mi355_gather_probe.restype = _c_int
    lib.mi355_gather_probe.argtypes = [_c_vp, _c_vp, _c_vp, _c_i64, _c_vp, _c_int, _c_i64, _c_i64, _c_int, _c_i64, _c_vp]
    lib.mi355_prefill_input_facts.restype = _c_int
    lib.mi355_prefill_input_facts.argtypes = [_c_vp, _c_vp, _c_vp, _c_i64, _c_vp, _c_vp, _c_int, _c_int, _c_vp, _c_vp]
    lib.mi355_kv_append_fp8.restype = _c_int
    lib.mi355_kv_append_fp8.argtypes = [
        _c_vp, _c_vp, _c_vp, _c_vp, _c_vp, _c_i64, _c_int, _c_int, _c_int, _c_int, _c_i64, _c_int, _c_vp,
    ]


def load() -> ctypes.CDLL:
    """Load the in-tree shared library (once).  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not LIB_PATH.exists():
            raise NativeLibraryError(
                f"{LIB_PATH} is missing: build it with `python -m tileops_amd.build` "
                "(there is no CPU fallback for the MI355X kernels)"
            )
        lib = ctypes.CDLL(str(LIB_PATH))
        for sym in EXPORTED_SYMBOLS:
            if not hasattr(lib, sym):
                raise NativeLibraryError(f"{LIB_PATH} does not export {sym}")
        _declare(lib)
        got = lib.mi355_abi_version()
        if got != ABI_VERSION:
            raise NativeLibraryError(f"{LIB_PATH} has ABI version {got}, this package expects {ABI_VERSION}; rebuild")
        _lib = lib
        return lib


def last_error() -> str:
    return load().mi355_last_error().decode("utf-8", "replace")


def _check(rc: int) -> None:
    if rc == 0:
        return
    msg = last_error()
    if rc in (-1,):
        raise ValueError(msg)
    if rc == -2:
        raise NotImplementedError(msg)
    raise NativeLibraryError(f"mi355 error {rc}: {msg}")


def dtype_code(dtype: torch.dtype) -> int:
    if dtype == torch.bfloat16:
        return DT_BF16
    if dtype == torch.float16:
        return DT_FP16
    if dtype == torch.float8_e4m3fn:
        return DT_FP8_E4M3FN
    raise ValueError(f"dtype {dtype} has no MI355X kernel (bfloat16, float16, float8_e4m3fn)")


_GFX950_BY_INDEX: dict[int, bool] = {}  # a device's architecture does not change: asked once per device index


def is_gfx950(device: torch.device) -> bool:
    """True iff *device* is a ROCm GPU whose architecture is gfx950 (MI350X / MI355X)."""
    if device.type != "cuda" or torch.version.hip is None:
        return False
    index = device.index
    known = _GFX950_BY_INDEX.get(index) if index is not None else None
    if known is not None:
        return known
    if not torch.cuda.is_available():
        return False
    name = getattr(torch.cuda.get_device_properties(device), "gcnArchName", "")
    answer = name.split(":")[0] == "gfx950"
    if index is not None:
        _GFX950_BY_INDEX[index] = answer
    return answer


def require_gfx950(device: torch.device) -> None:
    if not is_gfx950(device):
        raise NativeLibraryError(f"device {device} is not a gfx950 (MI355X) GPU; these kernels run nowhere else")


def _stream_ptr(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def decode_workspace(
    batch: int, q_len: int, heads: int, heads_kv: int, dim: int, page_size: int, max_blocks_per_seq: int,
    q_dtype: torch.dtype, kv_dtype: torch.dtype, num_split: int = 0, kernel: int = KERNEL_AUTO,
) -> tuple[int, int, int]:
    """(workspace_bytes, num_split, kernel) for a decode call of this shape.  Touches no device."""
    lib = load()
    nbytes, nsplit, kout = _c_sz(0), _c_int(0), _c_int(0)
    _check(lib.mi355_gqa_paged_decode_workspace(
        batch, q_len, heads, heads_kv, dim, page_size, max_blocks_per_seq, dtype_code(q_dtype), dtype_code(kv_dtype),
        num_split, kernel, ctypes.byref(nbytes), ctypes.byref(nsplit), ctypes.byref(kout)))
    return int(nbytes.value), int(nsplit.value), int(kout.value)


def paged_decode(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, k_scale: Optional[torch.Tensor], v_scale: Optional[torch.Tensor],
    seqlens: torch.Tensor, block_table: torch.Tensor, out: torch.Tensor, workspace: Optional[torch.Tensor], *,
    batch: int, q_len: int, heads: int, heads_kv: int, dim: int, page_size: int,
    sm_scale: float, softcap: float, causal: bool, num_split: int, kernel: int,
) -> None:
    """Enqueue one decode call on the current stream of ``q.device``.  Arguments are assumed validated."""
    lib = load()
    _check(lib.mi355_gqa_paged_decode(
        q.data_ptr(), k.data_ptr(), v.data_ptr(),
        k_scale.data_ptr() if k_scale is not None else None,
        v_scale.data_ptr() if v_scale is not None else None,
        seqlens.data_ptr(), block_table.data_ptr(), block_table.stride(0), out.data_ptr(),
        workspace.data_ptr() if workspace is not None else None,
        workspace.numel() * workspace.element_size() if workspace is not None else 0,
        batch, q_len, heads, heads_kv, dim, page_size, k.shape[0],
        dtype_code(q.dtype), dtype_code(k.dtype), float(sm_scale), float(softcap), int(bool(causal)),
        int(num_split), int(kernel), _stream_ptr(q.device)))


def paged_decode_static(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, k_scale: Optional[torch.Tensor], v_scale: Optional[torch.Tensor],
    seqlens: torch.Tensor, block_table: torch.Tensor, out: torch.Tensor, *,
    batch: int, q_len: int, heads: int, heads_kv: int, dim: int, page_size: int,
    sm_scale: float, softcap: float, causal: bool, num_split: int = 0, kernel: int = KERNEL_AUTO,
) -> None:
    """The same call through the entry point that allocates nothing: the library's static scratch takes the place of the
    workspace (calls needing more than 80 MiB are refused; calls overlapping on one GPU race)."""
    lib = load()
    _check(lib.mi355_gqa_paged_decode_static(
        q.data_ptr(), k.data_ptr(), v.data_ptr(),
        k_scale.data_ptr() if k_scale is not None else None,
        v_scale.data_ptr() if v_scale is not None else None,
        seqlens.data_ptr(), block_table.data_ptr(), block_table.stride(0), out.data_ptr(),
        batch, q_len, heads, heads_kv, dim, page_size, k.shape[0],
        dtype_code(q.dtype), dtype_code(k.dtype), float(sm_scale), float(softcap), int(bool(causal)),
        int(num_split), int(kernel), _stream_ptr(q.device)))


def contiguous_decode_workspace(
    batch: int, q_len: int, heads: int, heads_kv: int, dim: int, max_seqlen_kv: int,
    q_dtype: torch.dtype, kv_dtype: torch.dtype, num_split: int = 0, kernel: int = KERNEL_AUTO,
) -> tuple[int, int, int]:
    """(workspace_bytes, num_split, kernel) for a contiguous-cache decode call.  Touches no device."""
    lib = load()
    nbytes, nsplit, kout = _c_sz(0), _c_int(0), _c_int(0)
    _check(lib.mi355_gqa_decode_workspace(
        batch, q_len, heads, heads_kv, dim, max_seqlen_kv, dtype_code(q_dtype), dtype_code(kv_dtype),
        num_split, kernel, ctypes.byref(nbytes), ctypes.byref(nsplit), ctypes.byref(kout)))
    return int(nbytes.value), int(nsplit.value), int(kout.value)


def contiguous_decode(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, k_scale: Optional[torch.Tensor], v_scale: Optional[torch.Tensor],
    out: torch.Tensor, workspace: Optional[torch.Tensor], *, batch: int, q_len: int, heads: int, heads_kv: int, dim: int,
    real_seqlen_kv: int, sm_scale: float, softcap: float, causal: bool, num_split: int, kernel: int,
) -> None:
    """Enqueue one contiguous-cache decode call (``k``/``v`` ``[batch, N_kv, heads_kv, dim]``) on the current stream."""
    lib = load()
    _check(lib.mi355_gqa_decode(
        q.data_ptr(), k.data_ptr(), v.data_ptr(),
        k_scale.data_ptr() if k_scale is not None else None,
        v_scale.data_ptr() if v_scale is not None else None,
        out.data_ptr(),
        workspace.data_ptr() if workspace is not None else None,
        workspace.numel() * workspace.element_size() if workspace is not None else 0,
        batch, q_len, heads, heads_kv, dim, k.shape[1], int(real_seqlen_kv),
        dtype_code(q.dtype), dtype_code(k.dtype), float(sm_scale), float(softcap), int(bool(causal)),
        int(num_split), int(kernel), _stream_ptr(q.device)))


def prefill_paged_workspace(batch: int, max_seqlen_q: int, total_q: int, heads: int, heads_kv: int, dim: int, page_size: int,
                            max_pages_per_req: int, q_dtype: torch.dtype, cache_dtype: torch.dtype,
                            kernel: int = KERNEL_AUTO) -> int:
    """Workspace bytes of a paged prefill call.  Touches no device."""
    lib = load()
    nbytes = _c_sz(0)
    _check(lib.mi355_gqa_prefill_paged_workspace(
        batch, max_seqlen_q, total_q, heads, heads_kv, dim, page_size, max_pages_per_req, dtype_code(q_dtype),
        dtype_code(cache_dtype), kernel, ctypes.byref(nbytes)))
    return int(nbytes.value)


def prefill_paged(q: torch.Tensor, k_new: torch.Tensor, v_new: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                  k_scale: torch.Tensor, v_scale: torch.Tensor, cu_seqlens_q: torch.Tensor, cache_seqlens: torch.Tensor,
                  block_table: torch.Tensor, out: torch.Tensor, workspace: Optional[torch.Tensor], *, batch: int,
                  max_seqlen_q: int, heads: int, heads_kv: int, dim: int, page_size: int, sm_scale: float, softcap: float,
                  causal: bool, kernel: int = KERNEL_AUTO) -> None:
    """Enqueue one paged prefill call (append + attention) on the current stream of ``q.device``."""
    lib = load()
    _check(lib.mi355_gqa_prefill_paged(
        q.data_ptr(), k_new.data_ptr(), v_new.data_ptr(), k_pages.data_ptr(), v_pages.data_ptr(), k_scale.data_ptr(),
        v_scale.data_ptr(), cu_seqlens_q.data_ptr(), cache_seqlens.data_ptr(), block_table.data_ptr(), block_table.stride(0),
        out.data_ptr(), workspace.data_ptr() if workspace is not None else None,
        workspace.numel() * workspace.element_size() if workspace is not None else 0,
        batch, max_seqlen_q, q.shape[0], heads, heads_kv, dim, page_size, k_pages.shape[0], dtype_code(q.dtype),
        dtype_code(k_pages.dtype), float(sm_scale), float(softcap), int(bool(causal)), int(kernel), _stream_ptr(q.device)))


def prefill_paged_rope_workspace(batch: int, max_seqlen_q: int, total_q: int, heads: int, heads_kv: int, dim: int, page_size: int,
                                 max_pages_per_req: int, q_dtype: torch.dtype, kernel: int = KERNEL_AUTO) -> int:
    """Workspace bytes of a paged prefill call with fused rotary embedding.  Touches no device."""
    lib = load()
    nbytes = _c_sz(0)
    _check(lib.mi355_gqa_prefill_paged_rope_workspace(
        batch, max_seqlen_q, total_q, heads, heads_kv, dim, page_size, max_pages_per_req, dtype_code(q_dtype), kernel,
        ctypes.byref(nbytes)))
    return int(nbytes.value)


def prefill_paged_rope(q: torch.Tensor, k_new: torch.Tensor, v_new: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                       cos_table: torch.Tensor, sin_table: torch.Tensor, cu_seqlens_q: torch.Tensor, cache_seqlens: torch.Tensor,
                       block_table: torch.Tensor, out: torch.Tensor, workspace: torch.Tensor, *, batch: int, max_seqlen_q: int,
                       heads: int, heads_kv: int, dim: int, page_size: int, rotary_dim: int, sm_scale: float, softcap: float,
                       causal: bool, kernel: int = KERNEL_AUTO) -> None:
    """Enqueue one paged prefill call with fused rotary embedding (rotate q and k_new, append, attention)."""
    lib = load()
    _check(lib.mi355_gqa_prefill_paged_rope(
        q.data_ptr(), k_new.data_ptr(), v_new.data_ptr(), k_pages.data_ptr(), v_pages.data_ptr(), cos_table.data_ptr(),
        sin_table.data_ptr(), cu_seqlens_q.data_ptr(), cache_seqlens.data_ptr(), block_table.data_ptr(), block_table.stride(0),
        out.data_ptr(), workspace.data_ptr(), workspace.numel() * workspace.element_size(),
        batch, max_seqlen_q, q.shape[0], heads, heads_kv, dim, page_size, k_pages.shape[0], dtype_code(q.dtype),
        int(rotary_dim), int(cos_table.shape[0]), float(sm_scale), float(softcap), int(bool(causal)), int(kernel),
        _stream_ptr(q.device)))


def gather_probe(cache: torch.Tensor, seqlens: torch.Tensor, block_table: torch.Tensor, page_size: int, max_len: int) -> torch.Tensor:
    """Dense ``[batch, max_len, *cache.shape[1:]]`` copy of the rows a decode call would read
    (rows past each sequence's length are zero).  Device page arithmetic only -- the index-probe."""
    require_gfx950(cache.device)
    lib = load()
    batch = seqlens.shape[0]
    row_bytes = cache[0].numel() * cache.element_size()
    out = torch.zeros((batch, max_len) + tuple(cache.shape[1:]), dtype=cache.dtype, device=cache.device)
    _check(lib.mi355_gather_probe(
        cache.data_ptr(), seqlens.data_ptr(), block_table.data_ptr(), block_table.stride(0), out.data_ptr(),
        batch, max_len, row_bytes, page_size, cache.shape[0], _stream_ptr(cache.device)))
    return out


def kv_append_fp8(x_new: torch.Tensor, cache: torch.Tensor, scale: torch.Tensor, seqlens: torch.Tensor,
                  block_table: torch.Tensor, page_size: int) -> None:
    """Quantize ``x_new [batch, heads_kv, dim]`` per (token, head) and store it at each sequence's last position."""
    require_gfx950(cache.device)
    lib = load()
    batch, heads_kv, dim = x_new.shape
    _check(lib.mi355_kv_append_fp8(
        x_new.data_ptr(), cache.data_ptr(), scale.data_ptr(), seqlens.data_ptr(), block_table.data_ptr(),
        block_table.stride(0), batch, heads_kv, dim, page_size, cache.shape[0], dtype_code(x_new.dtype),
        _stream_ptr(cache.device)))


def prefill_input_facts(cu_seqlens_q: torch.Tensor, cache_seqlens: torch.Tensor, block_table: torch.Tensor,
                        k_scale: Optional[torch.Tensor], v_scale: Optional[torch.Tensor]) -> list[int]:
    """The ten facts behind the paged prefill op's value checks (see ``mi355_prefill_input_facts``): one small kernel,
    one transfer to the host."""
    require_gfx950(block_table.device)
    lib = load()
    # the kernel indexes all three as dense int32 arrays: a direct caller gets an error here, not a wrong fact
    batch = cache_seqlens.shape[0]
    if cu_seqlens_q.numel() != batch + 1 or not cu_seqlens_q.is_contiguous() or not cache_seqlens.is_contiguous():
        raise ValueError(f"cu_seqlens_q must be a contiguous array of {batch + 1} entries and cache_seqlens contiguous, got "
                         f"{tuple(cu_seqlens_q.shape)} and {tuple(cache_seqlens.shape)}")
    if any(t.dtype != torch.int32 for t in (cu_seqlens_q, cache_seqlens, block_table)) or block_table.stride(1) != 1:
        raise ValueError("cu_seqlens_q, cache_seqlens and block_table must be int32, block_table rows contiguous")
    for name, t in (("k_scale", k_scale), ("v_scale", v_scale)):
        if t is not None and (t.dtype != torch.float32 or t.numel() < 1):
            raise ValueError(f"{name} must hold at least one float32 value")
    # The kernel writes the ten values straight into pinned host memory (device-addressable at the same address), and the
    # host waits for the stream: no device buffer, no copy back.  One buffer per thread, so that threads that drive
    # different streams do not share it.
    facts = getattr(_facts_local, "buf", None)
    if facts is None:
        facts = _facts_local.buf = torch.empty(10, dtype=torch.int32, pin_memory=True)
    stream = torch.cuda.current_stream(block_table.device)
    _check(lib.mi355_prefill_input_facts(
        cu_seqlens_q.data_ptr(), cache_seqlens.data_ptr(), block_table.data_ptr(), block_table.stride(0),
        k_scale.data_ptr() if k_scale is not None else None, v_scale.data_ptr() if v_scale is not None else None,
        cache_seqlens.shape[0], block_table.shape[1], facts.data_ptr(), stream.cuda_stream))
    stream.synchronize()
    return facts.tolist()
