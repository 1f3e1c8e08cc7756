"""TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's paged GQA decode semantics.

Nothing under ``tileops_amd/`` may import this module.  Only ``tests/``, ``__graft_entry__.smoke()`` and
``bench.py``'s ``cpu_baseline`` leg use it, and only as the checker.

Every function cites the reference file:line it follows (paths relative to the reference checkout).

Parity status of each function (how it is pinned, without importing the reference):

* ``gather_pages``              pure indexing; pinned bit-exact against ``k.view(P, page, H_kv, D)[table]``
                                and by a per-token loop restating ``_physical_pos``.
* ``ref_paged_gqa_decode``      pinned against ``torch.nn.functional.scaled_dot_product_attention`` (a library
                                routine, the reference benchmark's own baseline), a float64 NumPy brute force,
                                and closed forms (q=0 -> mean of V, len=1 -> V row, dominant key, softcap->inf).
* ``ref_paged_gqa_decode_sdpa_math``  the reference benchmark's torch baseline; pinned against ``ref_paged_gqa_decode``.
* ``ref_gqa_decode_contiguous`` pinned against SDPA and the paged oracle with an identity table.
* ``quantize_kv_per_token``     pinned against the C codec in ``oracle/fp8_e4m3fn.c`` and torch's fp8 cast.
* causal chunk mask             pinned by "query i of a chunk == single-token decode at length len-S_q+i+1".
* ``ref_gqa_prefill_paged``     pinned against SDPA per sequence (explicit boolean mask), against "row i of a chunk ==
                                single-token decode over old tokens + chunk[:i+1]" through the pinned decode oracle,
                                and, for the append, against a per-token loop over ``physical_pos`` and torch's fp8 cast.
* ``rope_tables`` / ``apply_neox_rope`` / ``ref_gqa_prefill_paged_rope``
                                pinned by what the mathematics fixes: position 0 is the identity; each (d, d+half) pair is
                                rotated by exactly ``pos * base**(-i/half)`` (checked against complex multiplication in
                                float64); pair norms are preserved; ``<rope(q, m), rope(k, n)>`` depends on ``m - n`` only;
                                dimensions past ``rotary_dim`` pass through bit for bit; the fused op equals "rotate, then
                                the pinned plain prefill oracle".

The exact floating-point bits of the reference's TileLang-generated CUDA kernels are not reproducible here
(TileLang is absent); the reference itself defines correctness against this torch program within tolerance.
"""

from __future__ import annotations

import math
from typing import Optional

import numpy as np
import torch

FP8_MAX = 448.0


def physical_pos(block_table: torch.Tensor, batch_idx: int, logical_pos: int, page_size: int) -> int:
    """Logical token -> physical token.  tests/ops/attention/test_gqa_prefill_paged.py:25-31."""
    page = int(block_table[batch_idx, logical_pos // page_size])
    return page * page_size + logical_pos % page_size


def gather_pages(
    cache: torch.Tensor, block_table_row: torch.Tensor, length: int, page_size: int
) -> torch.Tensor:
    """Reassemble one sequence's logical ``[length, ...]`` rows from the physical pool ``[N_kv, ...]``.

    tests/ops/attention/test_gqa_decode_paged.py:46-59 (page-by-page copy, then truncate to the real
    length).  Pure indexing: the result is bit-identical to the pool rows it names.
    """
    if length == 0:
        return cache[:0]
    n_pages = math.ceil(length / page_size)
    pages = block_table_row[:n_pages].to(torch.long)
    idx = (pages[:, None] * page_size + torch.arange(page_size)[None, :]).reshape(-1)[:length]
    return cache.index_select(0, idx)


def _scores_to_probs(scores: torch.Tensor, softcap: float) -> torch.Tensor:
    if softcap > 0:
        # tests/ops/attention/test_gqa_decode_paged.py:66-67 ; online_softmax.py:162-171
        scores = softcap * torch.tanh(scores / softcap)
    return scores


def ref_paged_gqa_decode(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    real_seqlen_kv: torch.Tensor,
    block_table: torch.Tensor,
    *,
    page_size: int,
    sm_scale: Optional[float] = None,
    softcap: float = 0.0,
    k_scale: Optional[torch.Tensor] = None,
    v_scale: Optional[torch.Tensor] = None,
    is_causal: bool = True,
    out_dtype: Optional[torch.dtype] = None,
) -> torch.Tensor:
    """fp32 attention over gathered (and dequantized) pages, cast to ``q.dtype``.

    ``q`` is ``[B, H, D]`` (one query token; tests/ops/attention/test_gqa_decode_paged.py:30-72) or
    ``[B, S_q, H, D]`` (a chunk of S_q new tokens whose K/V are already in the cache; the mask is
    bottom-right aligned -- key j visible to query i iff ``j <= i + (len - S_q)`` --
    tests/ops/attention/test_gqa_prefill_paged.py:110-115, src/tileops/ops/attention/gqa.py:558-562).
    ``k, v`` are the physical pools ``[N_kv, H_kv, D]`` in fp16/bf16/fp32 or float8_e4m3fn; with fp8 the
    per-token-per-head fp32 ``k_scale, v_scale [N_kv, H_kv]`` dequantize as ``fp8.float() * scale``
    (tests/ops/attention/test_gqa_fp8.py:216-219).

    Uses a grouped einsum instead of the reference's ``repeat_interleave`` head expansion: same numbers,
    no ``group``-fold copy of K/V.
    """
    multi = q.dim() == 4
    q4 = q if multi else q.unsqueeze(1)
    B, S_q, H, D = q4.shape
    H_kv = k.shape[1]
    G = H // H_kv
    scale = D ** -0.5 if sm_scale is None else sm_scale
    out = torch.empty(B, S_q, H, D, dtype=torch.float32)
    for b in range(B):
        n = int(real_seqlen_kv[b])
        if n == 0:
            out[b] = 0.0  # softmax over nothing: nan_to_num convention, test_gqa_prefill_paged.py:115
            continue
        k_b = gather_pages(k, block_table[b], n, page_size).float()
        v_b = gather_pages(v, block_table[b], n, page_size).float()
        if k_scale is not None:
            k_b = k_b * gather_pages(k_scale, block_table[b], n, page_size).float()[..., None]
        if v_scale is not None:
            v_b = v_b * gather_pages(v_scale, block_table[b], n, page_size).float()[..., None]
        qg = q4[b].float().reshape(S_q, H_kv, G, D)
        scores = torch.einsum("sjgd,njd->jgsn", qg, k_b) * scale  # [H_kv, G, S_q, n]
        scores = _scores_to_probs(scores, softcap)
        if multi and is_causal and S_q > 1:
            q_pos = torch.arange(S_q)[:, None] + (n - S_q)
            kv_pos = torch.arange(n)[None, :]
            scores = scores.masked_fill(~(kv_pos <= q_pos), float("-inf"))
        probs = torch.softmax(scores, dim=-1).nan_to_num()
        o = torch.einsum("jgsn,njd->sjgd", probs, v_b)
        out[b] = o.reshape(S_q, H, D)
    out = out.to(out_dtype or q.dtype)
    return out if multi else out.squeeze(1)


def ref_paged_gqa_decode_sdpa_math(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, real_seqlen_kv: torch.Tensor, block_table: torch.Tensor, *,
    page_size: int, k_scale: Optional[torch.Tensor] = None, v_scale: Optional[torch.Tensor] = None, is_causal: bool = True,
) -> torch.Tensor:
    """The torch baseline the reference *benchmark* times (benchmarks/ops/attention/bench_gqa_decode_paged.py:21-66):
    per sequence, reassemble the pages, expand K/V to the query heads by indexing, and call
    ``F.scaled_dot_product_attention`` under ``sdpa_kernel(MATH)`` -- in fp32 on the dequantized cache here, so that it
    is the same function as ``ref_paged_gqa_decode`` (default scale, no softcap) computed by the library routine.
    Multi-token queries pass the bottom-right causal mask explicitly.  Pinned against ``ref_paged_gqa_decode``."""
    import torch.nn.functional as F
    from torch.nn.attention import SDPBackend, sdpa_kernel

    multi = q.dim() == 4
    q4 = q if multi else q.unsqueeze(1)
    B, S_q, H, D = q4.shape
    H_kv = k.shape[1]
    group_id = torch.arange(H, dtype=torch.long) // (H // H_kv)
    out = torch.zeros(B, S_q, H, D, dtype=torch.float32)
    for b in range(B):
        n = int(real_seqlen_kv[b])
        if n == 0:
            continue
        k_b = gather_pages(k, block_table[b], n, page_size).float()
        v_b = gather_pages(v, block_table[b], n, page_size).float()
        if k_scale is not None:
            k_b = k_b * gather_pages(k_scale, block_table[b], n, page_size).float()[..., None]
        if v_scale is not None:
            v_b = v_b * gather_pages(v_scale, block_table[b], n, page_size).float()[..., None]
        k_bhsd = k_b[:, group_id, :].unsqueeze(0).transpose(1, 2)
        v_bhsd = v_b[:, group_id, :].unsqueeze(0).transpose(1, 2)
        q_bhsd = q4[b].float().transpose(0, 1).unsqueeze(0)  # [1, H, S_q, D]
        mask = None
        if multi and is_causal and S_q > 1:
            mask = torch.arange(n)[None, :] <= (torch.arange(S_q)[:, None] + (n - S_q))
        with sdpa_kernel(backends=[SDPBackend.MATH]):
            o = F.scaled_dot_product_attention(q_bhsd, k_bhsd, v_bhsd, attn_mask=mask)
        out[b] = o[0].transpose(0, 1)
    out = out.to(q.dtype)
    return out if multi else out.squeeze(1)


def ref_gqa_decode_contiguous(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    *,
    sm_scale: Optional[float] = None,
    softcap: float = 0.0,
) -> torch.Tensor:
    """Contiguous-cache GQA decode: ``q [B,H,D]``, ``k,v [B,S,H_kv,D]``.  workloads/attention/gqa.py:165-175."""
    B, H, D = q.shape
    H_kv = k.shape[2]
    G = H // H_kv
    scale = D ** -0.5 if sm_scale is None else sm_scale
    qg = q.float().reshape(B, H_kv, G, D)
    scores = torch.einsum("bjgd,bnjd->bjgn", qg, k.float()) * scale
    scores = _scores_to_probs(scores, softcap)
    probs = torch.softmax(scores, dim=-1)
    o = torch.einsum("bjgn,bnjd->bjgd", probs, v.float())
    return o.reshape(B, H, D).to(q.dtype).contiguous()


def brute_force_f64(
    q: np.ndarray,
    k: np.ndarray,
    v: np.ndarray,
    lens: np.ndarray,
    table: np.ndarray,
    page_size: int,
    sm_scale: float,
    softcap: float = 0.0,
    causal: bool = True,
) -> np.ndarray:
    """Token-by-token float64 evaluation (tiny shapes only).  Same semantics as ``ref_paged_gqa_decode``
    written with scalar page arithmetic so an indexing slip in either shows up as a mismatch."""
    multi = q.ndim == 4
    q4 = q if multi else q[:, None]
    B, S_q, H, D = q4.shape
    H_kv = k.shape[1]
    G = H // H_kv
    out = np.zeros((B, S_q, H, D), dtype=np.float64)
    for b in range(B):
        n = int(lens[b])
        for s in range(S_q):
            limit = n - S_q + s + 1 if (multi and causal) else n
            for h in range(H):
                j = h // G
                sc = np.empty(max(limit, 0), dtype=np.float64)
                rows = np.empty((max(limit, 0), D), dtype=np.float64)
                for t in range(limit):
                    phys = int(table[b, t // page_size]) * page_size + t % page_size
                    x = float(np.dot(q4[b, s, h].astype(np.float64), k[phys, j].astype(np.float64))) * sm_scale
                    if softcap > 0:
                        x = softcap * math.tanh(x / softcap)
                    sc[t] = x
                    rows[t] = v[phys, j]
                if limit <= 0:
                    continue
                p = np.exp(sc - sc.max())
                p /= p.sum()
                out[b, s, h] = p @ rows
    return out if multi else out[:, 0]


def quantize_kv_per_token(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """Per-(token, kv-head) FP8-E4M3FN quantizer: ``x [N, H_kv, D]`` -> ``(q8 [N,H_kv,D] fp8, scale [N,H_kv] f32)``.

    workloads/fp8_quant.py:27-33: ``amax = |x|.amax(-1).clamp(min=1e-4)``; ``scale = amax / 448``;
    ``q = clamp(x / scale, -448, 448).to(float8_e4m3fn)``.  The clamp matters: torch's cast does not
    saturate (values rounding above 448 become NaN).
    """
    xf = x.float()
    amax = xf.abs().amax(dim=-1, keepdim=True).clamp(min=1e-4)
    scale = amax / FP8_MAX
    q8 = torch.clamp(xf / scale, min=-FP8_MAX, max=FP8_MAX).to(torch.float8_e4m3fn)
    return q8, scale.squeeze(-1).contiguous()


def dequantize_kv(q8: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """``fp8.float() * scale``.  tests/ops/attention/test_gqa_fp8.py:216-219."""
    return q8.float() * scale.float()[..., None]


# --- split-KV bookkeeping restated from the reference (known-answer material for the host-side tests) ----


def reference_block_ns(page_size: int) -> tuple[int, ...]:
    """Tile heights the reference's generic paged kernel accepts.
    src/tileops/kernels/attention/gqa_decode_paged.py:21-33."""
    if page_size <= 0:
        raise ValueError("page_size must be positive")
    ns = tuple(n for n in (128, 64) if n <= page_size and page_size % n == 0)
    if ns:
        return ns
    if page_size < 64:
        return (page_size,)
    raise ValueError(f"page_size={page_size} matches no supported block_N")


def combine_partials(partial_o: torch.Tensor, lse2: torch.Tensor) -> torch.Tensor:
    """Merge normalised per-split outputs with their log2-domain LSE.

    src/tileops/kernels/attention/gqa_decode_paged.py:344-374:
    ``lse = log2 sum_s 2^(lse_s - max) + max`` ; ``O = sum_s 2^(lse_s - lse) * O_s``.
    ``partial_o [..., S, D]``, ``lse2 [..., S]`` (``-inf`` marks an empty split).
    """
    m = lse2.max(dim=-1, keepdim=True).values
    m = torch.where(torch.isfinite(m), m, torch.zeros_like(m))
    w = torch.exp2(lse2 - m)
    lse = torch.log2(w.sum(dim=-1, keepdim=True)) + m
    wn = torch.exp2(lse2 - lse).nan_to_num()
    return (partial_o * wn[..., None]).sum(dim=-2)


def reference_roofline(
    batch: int, heads: int, heads_kv: int, seqlen_kv: int, dim: int, page_size: int, elem_bytes: int
) -> tuple[int, int]:
    """(flops, bytes) exactly as src/tileops/perf/formulas.py:690-711 (S = pool size, K/V counted once)."""
    flops = 4 * batch * heads * seqlen_kv * dim
    q_elems = batch * heads * dim
    kv_elems = seqlen_kv * heads_kv * dim
    meta = batch * 4 + batch * max(1, (seqlen_kv + page_size - 1) // page_size) * 4
    return int(flops), int((q_elems + 2 * kv_elems + q_elems) * elem_bytes + meta)


def quantize_per_tensor(x: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """``clamp(x / scale, -448, 448)`` cast to e4m3fn (round to nearest even): the append of the reference's FP8 paged
    prefill kernel, src/tileops/kernels/attention/gqa_fwd.py:1059-1061; expectation of its test,
    tests/ops/attention/test_gqa_prefill_paged.py:402-405."""
    return (x.float() / scale.float().reshape(())).clamp(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn)


def ref_gqa_prefill_paged(
    q: torch.Tensor,
    k_new: torch.Tensor,
    v_new: torch.Tensor,
    k_pages: torch.Tensor,
    v_pages: torch.Tensor,
    k_scale: torch.Tensor,
    v_scale: torch.Tensor,
    cu_seqlens_q: torch.Tensor,
    cache_seqlens: torch.Tensor,
    block_table: torch.Tensor,
    *,
    page_size: int,
    is_causal: bool = True,
    sm_scale: Optional[float] = None,
    softcap: float = 0.0,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Packed prefill chunk over a paged cache: ``(o [total_q,H,D], k_pages_after, v_pages_after)``.

    Restates ``_gqa_prefill_paged_ref`` and the append checks of the reference's test
    (tests/ops/attention/test_gqa_prefill_paged.py:76-117, :301-313, :398-415): per sequence, attention in fp32 over
    ``cat(old tokens, chunk)`` with ``kv_pos <= old_len + i`` when causal; the old tokens of an FP8 cache are
    dequantised as ``(fp8.float() * scale).to(q.dtype)`` (:347-348; kernel: gqa_fwd.py:1063-1065), the chunk's own
    tokens enter unquantised; the chunk is written to logical positions ``old_len + i`` (copied, or quantised per
    tensor for an FP8 cache); nothing else in the pool changes.
    """
    total_q, H, D = q.shape
    H_kv = k_new.shape[1]
    G = H // H_kv
    scale = D ** -0.5 if sm_scale is None else sm_scale
    fp8 = k_pages.dtype == torch.float8_e4m3fn
    k_after, v_after = k_pages.clone(), v_pages.clone()
    out = torch.zeros(total_q, H, D, dtype=q.dtype)
    batch = cache_seqlens.shape[0]
    for b in range(batch):
        q0, q1 = int(cu_seqlens_q[b]), int(cu_seqlens_q[b + 1])
        q_len, old_len = q1 - q0, int(cache_seqlens[b])
        if q_len == 0:
            continue
        idx = torch.tensor([physical_pos(block_table, b, t, page_size) for t in range(old_len)], dtype=torch.long)
        k_old, v_old = k_pages[idx], v_pages[idx]
        if fp8:
            k_old = (k_old.float() * k_scale.float().reshape(())).to(q.dtype)
            v_old = (v_old.float() * v_scale.float().reshape(())).to(q.dtype)
        k_all = torch.cat([k_old.to(q.dtype), k_new[q0:q1]], 0).float()
        v_all = torch.cat([v_old.to(q.dtype), v_new[q0:q1]], 0).float()
        total_len = old_len + q_len
        qg = q[q0:q1].float().reshape(q_len, H_kv, G, D)
        scores = torch.einsum("sjgd,njd->jgsn", qg, k_all) * scale
        if softcap > 0:
            scores = softcap * torch.tanh(scores / softcap)
        if is_causal:
            q_pos = torch.arange(q_len)[:, None] + old_len
            kv_pos = torch.arange(total_len)[None, :]
            scores = scores.masked_fill(~(kv_pos <= q_pos), float("-inf"))
        probs = torch.softmax(scores, dim=-1).nan_to_num()
        o = torch.einsum("jgsn,njd->sjgd", probs, v_all)
        out[q0:q1] = o.reshape(q_len, H, D).to(q.dtype)
        for i in range(q_len):
            pos = physical_pos(block_table, b, old_len + i, page_size)
            if fp8:
                k_after[pos] = quantize_per_tensor(k_new[q0 + i], k_scale)
                v_after[pos] = quantize_per_tensor(v_new[q0 + i], v_scale)
            else:
                k_after[pos] = k_new[q0 + i]
                v_after[pos] = v_new[q0 + i]
    return out, k_after, v_after


def rope_tables(rotary_dim: int, max_position: int, base: float = 10000.0, dtype: torch.dtype = torch.float32) -> tuple[torch.Tensor, torch.Tensor]:
    """cos/sin ``[max_position, rotary_dim // 2]``: ``angle[p, i] = p * base**(-i / half)`` evaluated in fp32, then cast
    to *dtype*.  src/tileops/ops/rope.py:97-120 (``base_freqs``)."""
    half = rotary_dim // 2
    freqs = 1.0 / (base ** (torch.arange(0, half, dtype=torch.float32) / half))
    angles = torch.outer(torch.arange(max_position, dtype=torch.float32), freqs)
    return torch.cos(angles).to(dtype), torch.sin(angles).to(dtype)


def apply_neox_rope(x: torch.Tensor, positions: torch.Tensor, cos_table: torch.Tensor, sin_table: torch.Tensor,
                    rotary_dim: Optional[int] = None) -> torch.Tensor:
    """GPT-NeoX rotary embedding of packed rows ``x [T, heads, D]`` at ``positions [T]``:
    ``y[d] = x[d]*c + r*s`` with ``c, s = table[pos, d % half]``, ``r = -x[d + half]`` for ``d < half``, ``+x[d - half]``
    for ``half <= d < rotary_dim``; dimensions from ``rotary_dim`` on pass through
    (src/tileops/kernels/rope.py:228-246; the fused prefill kernels: kernels/attention/gqa_fwd.py:1521-1535, :1755-1768).
    The reference evaluates the expression on 16-bit operands inside TileLang; here the products are formed in fp32 from
    the same 16-bit operands (tables included) and rounded once to ``x.dtype`` -- at most an ulp or two apart."""
    D = x.shape[-1]
    rotary_dim = D if rotary_dim is None else rotary_dim
    half = rotary_dim // 2
    pos = positions.long()
    work = torch.float64 if x.dtype == torch.float64 else torch.float32
    c = cos_table[pos].to(work)[:, None, :]  # [T, 1, half]
    s = sin_table[pos].to(work)[:, None, :]
    xf = x.to(work)
    lo, hi = xf[..., :half], xf[..., half:rotary_dim]
    y = xf.clone()
    y[..., :half] = lo * c - hi * s
    y[..., half:rotary_dim] = hi * c + lo * s
    return y.to(x.dtype)


def ref_gqa_prefill_paged_rope(
    q: torch.Tensor,
    k_new: torch.Tensor,
    v_new: torch.Tensor,
    k_pages: torch.Tensor,
    v_pages: torch.Tensor,
    cu_seqlens_q: torch.Tensor,
    cache_seqlens: torch.Tensor,
    block_table: torch.Tensor,
    cos_table: torch.Tensor,
    sin_table: torch.Tensor,
    *,
    page_size: int,
    rotary_dim: Optional[int] = None,
    is_causal: bool = True,
    sm_scale: Optional[float] = None,
    softcap: float = 0.0,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """The prefill chunk with fused rotary embedding, as the reference's test builds its expectation
    (tests/ops/attention/test_gqa_prefill_paged.py:485-600): rotate ``q`` and ``k_new`` at positions
    ``cache_seqlens[b] + i`` (the cache already holds rotated keys), then the plain chunk semantics on the rotated
    tensors; the pages receive the rotated keys and the untouched values."""
    positions = torch.cat([torch.arange(int(cache_seqlens[b]), int(cache_seqlens[b]) + int(cu_seqlens_q[b + 1]) - int(cu_seqlens_q[b]))
                           for b in range(cache_seqlens.shape[0])]).to(torch.int32)
    q_rot = apply_neox_rope(q, positions, cos_table, sin_table, rotary_dim)
    k_rot = apply_neox_rope(k_new, positions, cos_table, sin_table, rotary_dim)
    one = torch.ones(1, dtype=torch.float32)
    return ref_gqa_prefill_paged(q_rot, k_rot, v_new, k_pages, v_pages, one, one, cu_seqlens_q, cache_seqlens, block_table,
                                 page_size=page_size, is_causal=is_causal, sm_scale=sm_scale, softcap=softcap)
