"""Paged prefill chunk with cache append: pins of the CPU oracle (no GPU) and GPU parity through the op layer and the C ABI.

The GPU block restates the reference's test file (tests/ops/attention/test_gqa_prefill_paged.py:120-415): the same
eight 16-bit cases and six FP8-cache cases (shapes, interleaved block table, scales 0.02, inputs scaled by 0.5), the
same tolerances (fp16 5e-3/1e-5, bf16 8e-2/1e-2, FP8 cache 8e-2/2e-2), the same three checks -- output, appended rows
(bit-exact for FP8), untouched old rows -- and the scale validation cases (:418-470).  Fused RoPE (:473-) has no
counterpart here.  Beyond the reference: head_dim 128 (MFMA kernel), empty chunks and empty caches, both kernels.
"""

from itertools import accumulate

import pytest
import torch
import torch.nn.functional as F

from oracle.paged_gqa_decode_ref import (
    apply_neox_rope, physical_pos, quantize_per_tensor, ref_gqa_prefill_paged, ref_gqa_prefill_paged_rope, ref_paged_gqa_decode,
    rope_tables,
)
from tests.conftest import require_gfx950
from tileops_amd import native
from tileops_amd.ops import GroupedQueryAttentionPrefillPagedWithKVCacheFwdOp as PrefillOp
from tileops_amd.roofline import gqa_prefill_paged_with_kv_cache_fwd_roofline

DEV = "cuda"
FP8 = torch.float8_e4m3fn
TOL = {torch.float16: (5e-3, 1e-5), torch.bfloat16: (8e-2, 1e-2)}


def _block_table(batch, max_pages_per_req):
    """tests/ops/attention/test_gqa_prefill_paged.py:34-40: even pages first, then odd ones."""
    rows = []
    for b in range(batch):
        pages = list(range(b * max_pages_per_req, (b + 1) * max_pages_per_req))
        rows.append(pages[::2] + pages[1::2])
    return torch.tensor(rows, dtype=torch.int32)


def _case(q_lens, old_lens, heads, heads_kv, dim, dtype, *, fp8=False, page=64, max_pages=8, seed=0):
    g = torch.Generator().manual_seed(seed)
    batch, total_q = len(q_lens), sum(q_lens)
    amp = 0.5 if fp8 else 1.0
    table = _block_table(batch, max_pages)
    cu = torch.tensor([0, *accumulate(q_lens)], dtype=torch.int32)
    cache = torch.tensor(old_lens, dtype=torch.int32)
    q = torch.randn(total_q, heads, dim, generator=g).to(dtype)
    k_new = (torch.randn(total_q, heads_kv, dim, generator=g) * amp).to(dtype)
    v_new = (torch.randn(total_q, heads_kv, dim, generator=g) * amp).to(dtype)
    scale = torch.tensor([0.02 if fp8 else 1.0])
    n = batch * max_pages * page
    k_pages = torch.zeros(n, heads_kv, dim, dtype=FP8 if fp8 else dtype)
    v_pages = torch.zeros_like(k_pages)
    for b, old in enumerate(old_lens):  # only the addressed old tokens hold data, as in the reference's fixture
        ko = (torch.randn(old, heads_kv, dim, generator=g) * amp).to(dtype)
        vo = (torch.randn(old, heads_kv, dim, generator=g) * amp).to(dtype)
        for t in range(old):
            pos = physical_pos(table, b, t, page)
            k_pages[pos] = quantize_per_tensor(ko[t], scale) if fp8 else ko[t]
            v_pages[pos] = quantize_per_tensor(vo[t], scale) if fp8 else vo[t]
    return q, k_new, v_new, k_pages, v_pages, scale, scale.clone(), cu, cache, table


# --- oracle pins (CPU) --------------------------------------------------------------------------------------
def test_oracle_matches_sdpa_with_an_explicit_mask_per_sequence():
    q_lens, old_lens, H, Hkv, D, page = [5, 12, 1], [20, 0, 70], 8, 2, 32, 16
    case = _case(q_lens, old_lens, H, Hkv, D, torch.float32, page=page, max_pages=8, seed=3)
    q, k_new, v_new, k_pages, v_pages, ks, vs, cu, cache, table = case
    for causal in (True, False):
        out, _, _ = ref_gqa_prefill_paged(*case, page_size=page, is_causal=causal)
        for b, (n, old) in enumerate(zip(q_lens, old_lens)):
            q0 = int(cu[b])
            idx = torch.tensor([physical_pos(table, b, t, page) for t in range(old)], dtype=torch.long)
            k_all = torch.cat([k_pages[idx], k_new[q0:q0 + n]]).repeat_interleave(H // Hkv, 1).transpose(0, 1)
            v_all = torch.cat([v_pages[idx], v_new[q0:q0 + n]]).repeat_interleave(H // Hkv, 1).transpose(0, 1)
            mask = (torch.arange(old + n)[None, :] <= torch.arange(n)[:, None] + old) if causal else None
            want = F.scaled_dot_product_attention(q[q0:q0 + n].transpose(0, 1), k_all, v_all, attn_mask=mask).transpose(0, 1)
            torch.testing.assert_close(out[q0:q0 + n], want, atol=2e-5, rtol=1e-5)


def test_oracle_row_i_of_a_chunk_is_a_single_token_decode_over_old_tokens_and_the_chunk_up_to_i():
    """Ties the prefill oracle to the (separately pinned) decode oracle, through the appended pages."""
    q_lens, old_lens, H, Hkv, D, page = [7, 3], [33, 5], 8, 4, 16, 16
    case = _case(q_lens, old_lens, H, Hkv, D, torch.float32, page=page, max_pages=8, seed=4)
    q, _, _, _, _, _, _, cu, cache, table = case
    out, k_after, v_after = ref_gqa_prefill_paged(*case, page_size=page, is_causal=True, softcap=3.0)
    for b, (n, old) in enumerate(zip(q_lens, old_lens)):
        for i in range(n):
            row = int(cu[b]) + i
            lens = torch.tensor([old + i + 1], dtype=torch.int32)
            want = ref_paged_gqa_decode(q[row:row + 1], k_after, v_after, lens, table[b:b + 1], page_size=page, softcap=3.0)
            torch.testing.assert_close(out[row:row + 1], want, atol=2e-5, rtol=1e-5)


def test_oracle_append_touches_exactly_the_chunk_positions_and_quantises_like_a_torch_cast():
    q_lens, old_lens, page = [9, 0, 4], [60, 17, 0], 32
    for fp8 in (False, True):
        case = _case(q_lens, old_lens, 4, 2, 16, torch.float16, fp8=fp8, page=page, max_pages=4, seed=5)
        _, k_new, v_new, k_pages, v_pages, ks, vs, cu, cache, table = case
        _, k_after, v_after = ref_gqa_prefill_paged(*case, page_size=page)
        touched = torch.zeros(k_pages.shape[0], dtype=torch.bool)
        for b, (n, old) in enumerate(zip(q_lens, old_lens)):
            for i in range(n):
                pos = physical_pos(table, b, old + i, page)
                touched[pos] = True
                src = k_new[int(cu[b]) + i]
                want = (src.float() / 0.02).to(FP8) if fp8 else src  # tests/ops/attention/test_gqa_prefill_paged.py:402
                assert torch.equal(k_after[pos].view(torch.uint8), want.view(torch.uint8))
        assert touched.sum() == sum(q_lens)
        assert torch.equal(k_after[~touched].view(torch.uint8), k_pages[~touched].view(torch.uint8))
        assert torch.equal(v_after[~touched].view(torch.uint8), v_pages[~touched].view(torch.uint8))


def test_oracle_rope_is_a_rotation_of_each_pair_by_position_times_frequency():
    """Pins ``rope_tables`` / ``apply_neox_rope`` by what the mathematics fixes (float64 tables, so that only the formula
    is on trial): position 0 is the identity; the pair (x[i], x[i + half]) read as a complex number is multiplied by
    exp(j * pos * base**(-i/half)); pair norms are preserved; dimensions from rotary_dim on pass through bit for bit;
    and <rope(q, m), rope(k, n)> depends on m - n only."""
    g = torch.Generator().manual_seed(5)
    D, rd, base, P = 64, 32, 10000.0, 300
    half = rd // 2
    cos, sin = rope_tables(rd, P, base, torch.float64)
    assert cos.shape == (P, half) and sin.shape == (P, half)
    x = torch.randn(7, 3, D, generator=g, dtype=torch.float64)
    pos = torch.tensor([0, 1, 2, 17, 100, 255, 299], dtype=torch.int32)
    y = apply_neox_rope(x, pos, cos, sin, rd)
    assert torch.equal(y[0], x[0])                                  # position 0
    assert torch.equal(y[..., rd:], x[..., rd:])                    # the tail is untouched
    zx = torch.complex(x[..., :half], x[..., half:rd])
    zy = torch.complex(y[..., :half], y[..., half:rd])
    freqs = base ** (-torch.arange(half, dtype=torch.float64) / half)
    expect = zx * torch.exp(1j * pos.double()[:, None, None] * freqs)
    # the tables come from fp32 angles (as the reference builds them): |angle error| <= ~300 * 2^-24
    torch.testing.assert_close(zy, expect, atol=5e-5, rtol=0)
    torch.testing.assert_close(zy.abs(), zx.abs(), atol=0, rtol=5e-7)   # a rotation, up to cos^2 + sin^2 of fp32 table entries
    # relative-position property (on a full rotary_dim, with one row at two position pairs of equal distance)
    cos2, sin2 = rope_tables(D, P, base, torch.float64)
    qv, kv = torch.randn(1, 1, D, generator=g, dtype=torch.float64), torch.randn(1, 1, D, generator=g, dtype=torch.float64)
    def dot(m, n):
        a = apply_neox_rope(qv, torch.tensor([m]), cos2, sin2)
        b = apply_neox_rope(kv, torch.tensor([n]), cos2, sin2)
        return float((a * b).sum())
    assert abs(dot(40, 10) - dot(130, 100)) < 2e-4 and abs(dot(40, 10) - dot(41, 10)) > 1e-3


def test_oracle_fused_rope_prefill_is_rotate_then_plain_prefill_and_tables_round_like_the_reference():
    q_lens, old_lens, dtype = [5, 3], [7, 70], torch.float16
    q, k_new, v_new, k_pages, v_pages, ks, vs, cu, cache, table = _case(q_lens, old_lens, 4, 2, 64, dtype, seed=9)
    cos, sin = rope_tables(32, 128, 10000.0, dtype)
    assert cos.dtype == dtype and float(cos[0].min()) == 1.0 and float(sin[0].abs().max()) == 0.0
    out, k_after, v_after = ref_gqa_prefill_paged_rope(q, k_new, v_new, k_pages, v_pages, cu, cache, table, cos, sin,
                                                       page_size=64, rotary_dim=32)
    positions = torch.tensor([7, 8, 9, 10, 11, 70, 71, 72], dtype=torch.int32)
    k_rot = apply_neox_rope(k_new, positions, cos, sin, 32)
    for t, (b, i) in enumerate([(0, 0), (0, 1), (0, 2), (0, 3), (0, 4), (1, 0), (1, 1), (1, 2)]):
        pos = physical_pos(table, b, old_lens[b] + i, 64)
        assert torch.equal(k_after[pos], k_rot[t]) and torch.equal(v_after[pos], v_new[t])
    plain, _, _ = ref_gqa_prefill_paged(apply_neox_rope(q, positions, cos, sin, 32), k_rot, v_new, k_pages, v_pages, ks, vs, cu,
                                        cache, table, page_size=64)
    assert torch.equal(out, plain)


def test_roofline_formula_by_hand():
    """src/tileops/perf/formulas.py:567-587 on the reference's llama-8b row: 8 x (512 new, 4096 old), fp16."""
    flops, nbytes = gqa_prefill_paged_with_kv_cache_fwd_roofline(
        batch=8, heads=32, heads_kv=8, dim=128, max_pages_per_req=72, page_size=64, max_seqlen_q=512, total_q=4096,
        q_lens=[512] * 8, cache_lens=[4096] * 8, is_causal=True, dtype="float16")
    visible = 8 * (512 * 4096 + 512 * 513 // 2)
    assert flops == 4 * 32 * visible * 128 == 292091330560
    assert nbytes == (2 * 4096 * 32 * 128 + 2 * 32768 * 8 * 128 + 2 * 2 * 4096 * 8 * 128) * 2 + 9 * 4 + 8 * 4 + 8 * 72 * 4 == 234883396
    # rows without per-request lengths: deterministic fill (:467-475, :559-565)
    f2, _ = gqa_prefill_paged_with_kv_cache_fwd_roofline(batch=2, heads=8, heads_kv=2, dim=64, max_pages_per_req=4, page_size=64,
                                                         max_seqlen_q=100, total_q=150, is_causal=False, dtype="float16")
    assert f2 == 4 * 8 * (100 * 256 + 50 * 256) * 64


def test_op_constructs_without_device_and_validates_like_the_reference():
    op = PrefillOp(batch=2, heads=8, heads_kv=2, max_pages_per_req=8, page_size=64, dim=64, cache_dtype=FP8, softcap=2.0)
    assert op.max_cache_len == 512 and op.groups == 4 and op.softcap == 2.0
    with pytest.raises(ValueError, match="page_size must be a power of two"):
        PrefillOp(batch=1, heads=8, heads_kv=2, max_pages_per_req=8, page_size=48, dim=64)
    with pytest.raises(ValueError, match="max_position is required when fuse_rope=True"):
        PrefillOp(batch=1, heads=8, heads_kv=2, max_pages_per_req=8, page_size=64, dim=64, fuse_rope=True)
    with pytest.raises(ValueError, match="rotary_dim requires fuse_rope=True"):
        PrefillOp(batch=1, heads=8, heads_kv=2, max_pages_per_req=8, page_size=64, dim=64, rotary_dim=32)
    with pytest.raises(ValueError, match="rotary_dim must be"):
        PrefillOp(batch=1, heads=8, heads_kv=2, max_pages_per_req=8, page_size=64, dim=64, fuse_rope=True, max_position=512, rotary_dim=31)
    with pytest.raises(ValueError, match="fuse_rope is not supported with FP8 paged KV cache yet"):
        PrefillOp(batch=1, heads=8, heads_kv=2, max_pages_per_req=8, page_size=64, dim=64, fuse_rope=True, max_position=512, cache_dtype=FP8)
    with pytest.raises(NotImplementedError):
        _ = op.total_flops


# --- GPU parity ---------------------------------------------------------------------------------------------
def _run(op, case, page, dtype, *, fp8=False, causal=True, softcap=0.0, atol=None, rtol=None):
    ref, k_after, v_after = ref_gqa_prefill_paged(*case, page_size=page, is_causal=causal, softcap=softcap)
    dev = [t.to(DEV) for t in case]
    cu = case[7]
    q_lens = (cu[1:] - cu[:-1]).tolist()
    out = op(*dev, max(q_lens))
    torch.cuda.synchronize()
    assert isinstance(out, torch.Tensor) and out.shape == case[0].shape and out.dtype == dtype
    if atol is None:
        atol, rtol = (8e-2, 2e-2) if fp8 else TOL[dtype]
    torch.testing.assert_close(out.cpu().float(), ref.float(), atol=atol, rtol=rtol)
    # appended rows bit for bit, everything else untouched
    assert torch.equal(dev[3].cpu().view(torch.uint8), k_after.view(torch.uint8))
    assert torch.equal(dev[4].cpu().view(torch.uint8), v_after.view(torch.uint8))
    return out


@pytest.mark.gpu
@pytest.mark.parametrize(
    "q_lens, old_lens, heads, heads_kv, dim, is_causal, dtype",
    [pytest.param([64, 96], [80, 128], 8, 2, 64, True, torch.float16, id="gqa_ratio4_mixed_fp16"),
     pytest.param([17, 33], [37, 100], 8, 2, 64, True, torch.float16, id="gqa_unaligned_old_len_fp16"),
     pytest.param([1], [511], 8, 2, 64, True, torch.float16, id="gqa_decode_len_capacity_boundary_fp16"),
     pytest.param([1, 17], [511, 37], 8, 2, 64, True, torch.float16, id="gqa_mixed_capacity_boundary_fp16"),
     pytest.param([64, 64], [64, 128], 8, 8, 64, True, torch.float16, id="mha_fp16"),
     pytest.param([32, 64], [96, 160], 8, 1, 64, True, torch.float16, id="mqa_fp16"),
     pytest.param([64, 96], [80, 128], 8, 2, 64, False, torch.float16, id="gqa_noncausal_fp16"),
     pytest.param([64, 96], [80, 128], 8, 2, 64, True, torch.bfloat16, id="gqa_ratio4_bf16")],
)
def test_gqa_prefill_paged_with_kv_cache_fwd(q_lens, old_lens, heads, heads_kv, dim, is_causal, dtype):
    require_gfx950()
    case = _case(q_lens, old_lens, heads, heads_kv, dim, dtype)
    op = PrefillOp(batch=len(q_lens), heads=heads, heads_kv=heads_kv, max_pages_per_req=8, page_size=64, dim=dim, is_causal=is_causal)
    _run(op, case, 64, dtype, causal=is_causal)


@pytest.mark.gpu
@pytest.mark.parametrize(
    "is_causal, softcap, dtype, page_size",
    [pytest.param(True, None, torch.float16, 64, id="causal-fp16-page64"), pytest.param(False, None, torch.float16, 64, id="noncausal-fp16-page64"),
     pytest.param(True, 2.0, torch.float16, 64, id="causal-softcap-fp16-page64"), pytest.param(True, None, torch.bfloat16, 64, id="causal-bf16-page64"),
     pytest.param(True, None, torch.float16, 16, id="causal-fp16-page16"), pytest.param(True, None, torch.float16, 128, id="causal-fp16-page128")],
)
def test_gqa_prefill_paged_with_fp8_kv_cache_fwd(is_causal, softcap, dtype, page_size):
    require_gfx950()
    case = _case([33, 48], [67, 80], 8, 2, 64, dtype, fp8=True, page=page_size)
    op = PrefillOp(batch=2, heads=8, heads_kv=2, max_pages_per_req=8, page_size=page_size, dim=64, is_causal=is_causal,
                   cache_dtype=FP8, softcap=softcap)
    _run(op, case, page_size, dtype, fp8=True, causal=is_causal, softcap=softcap or 0.0)


@pytest.mark.gpu
@pytest.mark.parametrize("scale_name, bad_value", [("k_scale", 0.0), ("k_scale", -0.01), ("k_scale", float("inf")), ("v_scale", float("nan"))])
def test_gqa_prefill_paged_with_fp8_kv_cache_rejects_invalid_scales(scale_name, bad_value):
    require_gfx950()
    case = [t.to(DEV) for t in _case([1], [0], 8, 2, 64, torch.float16, fp8=True, max_pages=1)]
    case[5 if scale_name == "k_scale" else 6] = torch.tensor([bad_value], device=DEV)
    op = PrefillOp(batch=1, heads=8, heads_kv=2, max_pages_per_req=1, page_size=64, dim=64, cache_dtype=FP8)
    with pytest.raises(ValueError, match=f"{scale_name}.*finite positive"):
        op(*case, 1)


@pytest.mark.gpu
@pytest.mark.parametrize("kernel", [native.KERNEL_GENERIC, native.KERNEL_AUTO], ids=["general", "mfma"])
@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_head_dim_128_empty_chunks_empty_caches_and_both_kernels(kernel, fp8, dtype):
    """Chunks of 0, 1, 33 and 130 rows (more than one row group per kv head), caches of 0, 5 and 700 tokens, tails that
    are not tile multiples; the same call on the general kernel and on the MFMA kernel (head_dim 128)."""
    require_gfx950()
    q_lens, old_lens = [33, 0, 130, 1, 20], [700, 5, 0, 257, 64]
    case = _case(q_lens, old_lens, 16, 4, 128, dtype, fp8=fp8, page=32, max_pages=32, seed=11)
    op = PrefillOp(batch=len(q_lens), heads=16, heads_kv=4, max_pages_per_req=32, page_size=32, dim=128, cache_dtype=FP8 if fp8 else None)
    call = op.attention_call(dtype, torch.device(DEV, 0))
    key = op.select_kernel_key(tuple(op.kernel_map), call)
    assert key == ("gqa_prefill_paged_with_fp8_kv_cache_fwd_kernel" if fp8 else "gqa_prefill_paged_with_kv_cache_fwd_kernel")
    inputs = [t.to(DEV) for t in case]
    op._get_kernel(tuple(inputs), key, call).config["kernel"] = kernel
    tol = (8e-2, 2e-2) if fp8 else ((2e-2, 2e-2) if dtype == torch.bfloat16 else (5e-3, 1e-3))
    _run(op, case, 32, dtype, fp8=fp8, atol=tol[0], rtol=tol[1])


@pytest.mark.gpu
def test_validate_inputs_false_skips_the_device_reads_and_nothing_else():
    """Same result bit for bit; a call whose cu_seqlens_q is inconsistent is then no longer caught on the host (the
    check needs a device read), while shape and dtype mistakes still are."""
    require_gfx950()
    case = _case([33, 48], [67, 80], 8, 2, 64, torch.float16)
    kw = dict(batch=2, heads=8, heads_kv=2, max_pages_per_req=8, page_size=64, dim=64)
    dev = [t.to(DEV) for t in case]
    out_checked = PrefillOp(**kw)(*[t.clone() for t in dev], 48)
    fast = PrefillOp(**kw, validate_inputs=False)
    torch.cuda.synchronize()
    syncs_before = torch.cuda.get_sync_debug_mode()
    torch.cuda.set_sync_debug_mode("error")  # any host read of device memory raises
    try:
        out_fast = fast(*[t.clone() for t in dev], 48)
    finally:
        torch.cuda.set_sync_debug_mode(syncs_before)
    assert torch.equal(out_checked, out_fast)
    with pytest.raises(ValueError, match="block_table shape"):
        fast(*dev[:9], dev[9][:, :4].contiguous(), 48)
    bad_cu = dev[7].clone()
    bad_cu[0] = 1
    with pytest.raises(ValueError, match=r"cu_seqlens_q\[0\] must be 0"):
        PrefillOp(**kw)(*dev[:7], bad_cu, *dev[8:], 48)


@pytest.mark.gpu
@pytest.mark.parametrize("fp8", [False, True])
def test_value_checks_cost_one_host_read(fp8):
    """The reference's value checks (scales, cu_seqlens_q, cache_seqlens, capacity, block-table range) are reduced on
    the device and cross to the host in one transfer: torch's sync debug mode reports one synchronising call."""
    import warnings
    require_gfx950()
    case = [t.to(DEV) for t in _case([33, 48], [67, 80], 8, 2, 64, torch.float16, fp8=fp8)]
    op = PrefillOp(batch=2, heads=8, heads_kv=2, max_pages_per_req=8, page_size=64, dim=64, cache_dtype=FP8 if fp8 else None)
    op(*[t.clone() for t in case], 48)  # builds the kernel object and its tables
    torch.cuda.synchronize()
    before = torch.cuda.get_sync_debug_mode()
    torch.cuda.set_sync_debug_mode("warn")
    try:
        with warnings.catch_warnings(record=True) as seen:
            warnings.simplefilter("always")
            op._validate_forward_inputs(*case, 48)
    finally:
        torch.cuda.set_sync_debug_mode(before)
    syncs = [w for w in seen if "synchroniz" in str(w.message).lower()]
    assert len(syncs) == 1, [str(w.message) for w in seen]


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["plain", "fp8", "rope"])
def test_chunk_tokens_past_the_block_table_row_are_not_appended(mode):
    """With the value checks off, a chunk that overruns its sequence's pages (cache 120 + 20 new tokens on two 64-token
    pages) appends the eight tokens that fit and drops the rest: the pool afterwards differs from the pool before in
    exactly the rows the table addresses, and no other sequence's pages are written."""
    require_gfx950()
    page, max_pages, heads, heads_kv, dim, dtype = 64, 2, 8, 2, 64, torch.float16
    q_lens, old_lens = [20, 5], [120, 10]
    fp8, rope = mode == "fp8", mode == "rope"
    case = _case(q_lens, old_lens, heads, heads_kv, dim, dtype, fp8=fp8, page=page, max_pages=max_pages, seed=21)
    q, k_new, v_new, k_pages, v_pages, ks, vs, cu, cache, table = case
    op = PrefillOp(batch=2, heads=heads, heads_kv=heads_kv, max_pages_per_req=max_pages, page_size=page, dim=dim,
                   cache_dtype=FP8 if fp8 else None, fuse_rope=rope, max_position=256 if rope else None, validate_inputs=False)
    dev = [t.to(DEV) for t in case]
    out = op(*dev, max(q_lens))
    torch.cuda.synchronize()
    assert out.shape == q.shape
    written = torch.zeros(k_pages.shape[0], dtype=torch.bool)
    for b, (n, old) in enumerate(zip(q_lens, old_lens)):
        for i in range(n):
            t = old + i
            if t >= max_pages * page:
                continue
            pos = physical_pos(table, b, t, page)
            written[pos] = True
            if not rope:  # values are copied (or quantised) as they are; rotated keys are checked by the rope tests
                want_v = quantize_per_tensor(v_new[int(cu[b]) + i], vs) if fp8 else v_new[int(cu[b]) + i]
                assert torch.equal(dev[4][pos].cpu().view(torch.uint8), want_v.view(torch.uint8))
    assert int(written.sum()) == 8 + 5
    for after, before in ((dev[3], k_pages), (dev[4], v_pages)):
        assert torch.equal(after.cpu().view(torch.uint8)[~written], before.view(torch.uint8)[~written])
        assert not torch.equal(after.cpu().view(torch.uint8)[written], before.view(torch.uint8)[written])


@pytest.mark.gpu
@pytest.mark.parametrize("stride, width", [(512, 300), (511, 301), (512, 3), (513, 513), (2048, 1031)])
def test_input_facts_entry_point_against_torch(stride, width):
    """mi355_prefill_input_facts on a strided block table with negative entries, a length sum that leaves int32 and a
    bad scale, against the same reductions in torch.  Row strides that allow 16-byte loads and ones that do not, widths
    with and without a tail of fewer than four entries, rows longer than one round of loads."""
    require_gfx950()
    g = torch.Generator().manual_seed(5)
    batch = 37
    q_lens = torch.randint(-3, 900, (batch,), generator=g, dtype=torch.int32)
    cu = torch.full((batch + 1,), 7, dtype=torch.int32)
    cu[1:] += torch.cumsum(q_lens, 0).to(torch.int32)
    cache = torch.randint(-5, 1 << 20, (batch,), generator=g, dtype=torch.int32)
    cache[3] = 2**31 - 5  # with any positive q_len the sum leaves int32: the fact saturates
    q_lens[3] = 11
    cu[4:] += 11 - (cu[4] - cu[3])
    wide = torch.randint(-9, 1 << 22, (batch, stride), generator=g, dtype=torch.int32)
    wide[:, width:] = torch.randint(-(1 << 30), 1 << 30, (batch, stride - width), generator=g, dtype=torch.int32)  # not addressed: must not count
    table_dev = wide.to(DEV)[:, :width]  # rows `stride` entries apart, `width` of them addressed
    assert table_dev.is_contiguous() == (stride == width)
    ks, vs = torch.tensor([0.5], device=DEV), torch.tensor([float("nan")], device=DEV)
    got = native.prefill_input_facts(cu.to(DEV), cache.to(DEV), table_dev, ks, vs)
    ql = (cu[1:] - cu[:-1]).to(torch.int64)
    tot = torch.clamp(cache.to(torch.int64) + ql, -2**31, 2**31 - 1)
    table = wide[:, :width]
    want = [1, 0, int(cu[0]), int(ql.min()), int(cu[-1]), int(ql.max()), int(cache.min()), int(tot.max()), int(table.min()), int(table.max())]
    assert got == want and want[7] == 2**31 - 1
    assert native.prefill_input_facts(cu.to(DEV), cache.to(DEV), table_dev, None, None)[:2] == [1, 1]


@pytest.mark.gpu
def test_prefill_rejects_bad_calls():
    require_gfx950()
    case = [t.to(DEV) for t in _case([4, 4], [10, 10], 8, 2, 64, torch.float16)]
    op = PrefillOp(batch=2, heads=8, heads_kv=2, max_pages_per_req=8, page_size=64, dim=64)
    with pytest.raises(ValueError, match="max_seqlen_q .3. must be >= actual max Q sequence length .4."):
        op(*case, 3)
    bad = list(case)
    bad[8] = torch.tensor([510, 10], dtype=torch.int32, device=DEV)
    with pytest.raises(ValueError, match="exceeds paged KV capacity"):
        op(*bad, 4)
    bad = list(case)
    bad[9] = case[9] + 100
    with pytest.raises(ValueError, match="block_table references page"):
        op(*bad, 4)
    bad = list(case)
    bad[3] = case[3].to(torch.bfloat16)
    with pytest.raises(ValueError, match="Expected k_pages.dtype"):
        op(*bad, 4)
    bad = list(case)
    bad[8] = torch.tensor([-1, 10], dtype=torch.int32, device=DEV)
    with pytest.raises(ValueError, match="cache_seqlens must be non-negative"):
        op(*bad, 4)
    bad = list(case)
    bad[7] = torch.tensor([0, 6, 4], dtype=torch.int32, device=DEV)
    with pytest.raises(ValueError, match="cu_seqlens_q must be non-decreasing"):
        op(*bad, 6)
    bad = list(case)
    bad[7] = torch.tensor([0, 4, 7], dtype=torch.int32, device=DEV)
    with pytest.raises(ValueError, match=r"cu_seqlens_q\[-1\] .7. must equal q.shape\[0\] .8."):
        op(*bad, 4)
    bad = list(case)
    bad[9] = case[9].clone()
    bad[9][1, 3] = -2
    with pytest.raises(ValueError, match="non-negative physical page ids"):
        op(*bad, 4)


@pytest.mark.gpu
@pytest.mark.parametrize("fp8", [False, True])
def test_llama_shape_chunks_of_hundreds_of_rows_against_long_prefixes(fp8):
    """The reference's llama-8b workload shape at reduced batch (attention.yaml:296): 32/8 heads, head_dim 128, page 64,
    chunks of 512 and 300 rows against prefixes of 4096 and 1000 tokens -- dozens of row groups per kv head, prefixes
    spanning many partitions, a chunk that ends mid-page."""
    require_gfx950()
    q_lens, old_lens = [512, 300], [4096, 1000]
    case = _case(q_lens, old_lens, 32, 8, 128, torch.float16, fp8=fp8, page=64, max_pages=72, seed=21)
    op = PrefillOp(batch=2, heads=32, heads_kv=8, max_pages_per_req=72, page_size=64, dim=128, cache_dtype=FP8 if fp8 else None)
    _run(op, case, 64, torch.float16, fp8=fp8)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("is_causal", [True, False])
def test_fp8_cache_long_chunks_make_one_pass_over_rows_dequantised_once_and_wide_tables_keep_two_passes(dtype, is_causal):
    """From 1024 query rows per kv head an FP8-cache call dequantises the cached tokens once into contiguous 16-bit rows
    (as the reference does: ``(fp8.float() * scale).to(dtype)``), copies the chunk behind them and makes one 16-bit pass;
    the workspace query says so.  The same call through a block table as wide as a large pool would need more workspace than
    the library takes for this, keeps the two passes (fp8 pages, then the chunk), and agrees.  Chunks of 300, 256 and 1
    tokens at group 4, an empty cache, a chunk that ends mid-page."""
    require_gfx950()
    q_lens, old_lens, heads, heads_kv, dim, page, max_pages = [300, 256, 1], [1000, 0, 77], 16, 4, 128, 64, 24
    case = _case(q_lens, old_lens, heads, heads_kv, dim, dtype, fp8=True, page=page, max_pages=max_pages, seed=41)
    packed_rows = len(q_lens) * max_pages * page * heads_kv * dim * 2 * 2
    narrow = native.prefill_paged_workspace(len(q_lens), max(q_lens), sum(q_lens), heads, heads_kv, dim, page, max_pages, dtype, FP8,
                                            native.KERNEL_AUTO)
    assert narrow >= packed_rows
    op = PrefillOp(batch=len(q_lens), heads=heads, heads_kv=heads_kv, max_pages_per_req=max_pages, page_size=page, dim=dim,
                   cache_dtype=FP8, is_causal=is_causal)
    out = _run(op, case, page, dtype, fp8=True, causal=is_causal)
    wide_pages = 600_000
    wide = native.prefill_paged_workspace(len(q_lens), max(q_lens), sum(q_lens), heads, heads_kv, dim, page, wide_pages, dtype, FP8,
                                          native.KERNEL_AUTO)
    wider = native.prefill_paged_workspace(len(q_lens), max(q_lens), sum(q_lens), heads, heads_kv, dim, page, wide_pages + 100_000, dtype,
                                           FP8, native.KERNEL_AUTO)
    assert wide == wider  # no packed rows in it: it does not grow with the table
    table = torch.zeros(len(q_lens), wide_pages, dtype=torch.int32)
    table[:, :max_pages] = case[9]
    case_wide = (*case[:9], table)
    op_wide = PrefillOp(batch=len(q_lens), heads=heads, heads_kv=heads_kv, max_pages_per_req=wide_pages, page_size=page, dim=dim,
                        cache_dtype=FP8, is_causal=is_causal)
    out_wide = _run(op_wide, case_wide, page, dtype, fp8=True, causal=is_causal)
    torch.testing.assert_close(out.float(), out_wide.float(), atol=2e-2, rtol=2e-2)


@pytest.mark.gpu
@pytest.mark.parametrize("dim, heads, heads_kv", [(256, 16, 4), (64, 16, 2), (256, 8, 8)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_head_dims_64_and_256_with_chunks_of_hundreds_of_rows(dim, heads, heads_kv, dtype):
    """The reference's qwen3.5 rows use head dim 256 and its softcap rows head dim 64 (attention.yaml:280-289): chunks of
    hundreds of rows against prefixes spanning several partitions, a chunk that ends mid-page, an empty cache."""
    require_gfx950()
    q_lens, old_lens = [257, 96, 40], [1500, 0, 333]
    case = _case(q_lens, old_lens, heads, heads_kv, dim, dtype, page=64, max_pages=30, seed=23)
    op = PrefillOp(batch=3, heads=heads, heads_kv=heads_kv, max_pages_per_req=30, page_size=64, dim=dim)
    _run(op, case, 64, dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("kernel", [native.KERNEL_GENERIC, native.KERNEL_AUTO], ids=["general", "mfma"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("heads, heads_kv", [(16, 4), (8, 8)])
def test_fp8_cache_head_dim_256_like_the_qwen_fp8_row(kernel, dtype, heads, heads_kv):
    """The reference's `qwen35-9b-prefill-paged-fp8-cache-b8-prefix32k-chunk1k-p64` row (attention.yaml:287: FP8 cache, head dim
    256, page 64) at reduced sizes: 256-byte cache rows with per-tensor scales, the second pass over the chunk's own
    16-bit tokens carrying the first pass's state.  A prefix that spans many partitions, an empty cache, an empty chunk,
    a single-token chunk, a chunk that ends mid-page; on the general kernel and on the MFMA kernel."""
    require_gfx950()
    q_lens, old_lens = [257, 96, 0, 1, 40], [3000, 0, 100, 511, 333]
    case = _case(q_lens, old_lens, heads, heads_kv, 256, dtype, fp8=True, page=64, max_pages=52, seed=29)
    op = PrefillOp(batch=len(q_lens), heads=heads, heads_kv=heads_kv, max_pages_per_req=52, page_size=64, dim=256, cache_dtype=FP8)
    call = op.attention_call(dtype, torch.device(DEV, 0))
    key = op.select_kernel_key(tuple(op.kernel_map), call)
    assert key == "gqa_prefill_paged_with_fp8_kv_cache_fwd_kernel"
    inputs = [t.to(DEV) for t in case]
    op._get_kernel(tuple(inputs), key, call).config["kernel"] = kernel
    _run(op, case, 64, dtype, fp8=True)


@pytest.mark.gpu
def test_fused_rope_head_dim_256_partial_rotary_like_the_qwen_rows():
    """attention.yaml:280-281 at reduced size: head dim 256, rotary_dim 64, mixed chunk lengths against long prefixes."""
    require_gfx950()
    _fused_rope_case([256, 40, 130], [1024, 3000, 7], 16, 4, 256, torch.float16, 64, 3200, True, None, atol=5e-3, max_pages=50)



@pytest.mark.gpu
@pytest.mark.parametrize(
    "rotary_dim, is_causal, softcap",
    [pytest.param(None, True, None, id="full-causal"), pytest.param(32, True, None, id="partial-causal"),
     pytest.param(32, False, None, id="partial-noncausal"), pytest.param(32, True, 2.0, id="partial-causal-softcap"),
     pytest.param(30, True, None, id="odd-number-of-pairs")],
)
def test_gqa_prefill_paged_with_kv_cache_fused_rope(rotary_dim, is_causal, softcap):
    """The reference's fused-RoPE case (tests/ops/attention/test_gqa_prefill_paged.py:476-600): raw q / k_new in, the
    cache holds rotated old keys; output against "rotate, then plain prefill", appended keys equal the rotated new
    keys, values are copied, old tokens and the inputs are untouched."""
    require_gfx950()
    q_lens, old_lens, heads, heads_kv, dim, dtype = [48, 33], [67, 100], 8, 2, 64, torch.float16
    max_position = max(o + n for o, n in zip(old_lens, q_lens)) + 1
    _fused_rope_case(q_lens, old_lens, heads, heads_kv, dim, dtype, rotary_dim, max_position, is_causal, softcap, atol=5e-3)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype, atol", [(torch.bfloat16, 3e-2), (torch.float16, 5e-3)])
@pytest.mark.parametrize("kernel", ["auto", "generic"])
def test_fused_rope_head_dim_128_long_positions_empty_chunk_and_empty_cache(dtype, atol, kernel):
    """Head dim 128 (MFMA path), positions in the thousands (where bf16 tables are coarse), a sequence with nothing
    cached, one with an empty chunk, a chunk that crosses a page boundary."""
    require_gfx950()
    q_lens, old_lens = [70, 0, 9, 130], [0, 300, 1999, 62]
    _fused_rope_case(q_lens, old_lens, 16, 4, 128, dtype, 64, 2100, True, None, atol=atol, max_pages=33,
                     config={"kernel": native.KERNEL_GENERIC} if kernel == "generic" else None)


def _fused_rope_case(q_lens, old_lens, heads, heads_kv, dim, dtype, rotary_dim, max_position, is_causal, softcap, *, atol,
                     max_pages=8, config=None):
    g = torch.Generator().manual_seed(41)
    batch, total_q, page = len(q_lens), sum(q_lens), 64
    rd = dim if rotary_dim is None else rotary_dim
    op = PrefillOp(batch=batch, heads=heads, heads_kv=heads_kv, max_pages_per_req=max_pages, page_size=page, dim=dim,
                   is_causal=is_causal, softcap=softcap, fuse_rope=True, max_position=max_position, rotary_dim=rotary_dim)
    # The op builds its tables on the device, like the reference (ops/attention/gqa.py:1048-1065); device and host
    # cos/sin may disagree in the last fp32 bit, hence now and then in the last 16-bit one.  The tables are pinned
    # against the oracle's to that one ulp, and the rotation is then checked with the very tables the kernel reads.
    cos, sin = (t.cpu() for t in op._rope_tables(torch.device(DEV, 0), dtype))
    cos_ref, sin_ref = rope_tables(rd, max_position, 10000.0, dtype)
    one_ulp = torch.finfo(dtype).eps
    torch.testing.assert_close(cos.float(), cos_ref.float(), atol=one_ulp, rtol=0)
    torch.testing.assert_close(sin.float(), sin_ref.float(), atol=one_ulp, rtol=0)
    assert float((cos != cos_ref).float().mean()) < 0.05 and float((sin != sin_ref).float().mean()) < 0.05
    table = _block_table(batch, max_pages)
    cu = torch.tensor([0, *accumulate(q_lens)], dtype=torch.int32)
    cache = torch.tensor(old_lens, dtype=torch.int32)
    q = torch.randn(total_q, heads, dim, generator=g).to(dtype)
    k_new = torch.randn(total_q, heads_kv, dim, generator=g).to(dtype)
    v_new = torch.randn(total_q, heads_kv, dim, generator=g).to(dtype)
    k_pages = torch.zeros(batch * max_pages * page, heads_kv, dim, dtype=dtype)
    v_pages = torch.zeros_like(k_pages)
    for b, old in enumerate(old_lens):
        if old == 0:
            continue
        ko = apply_neox_rope(torch.randn(old, heads_kv, dim, generator=g).to(dtype), torch.arange(old, dtype=torch.int32), cos, sin, rd)
        vo = torch.randn(old, heads_kv, dim, generator=g).to(dtype)
        idx = torch.tensor([physical_pos(table, b, t, page) for t in range(old)])
        k_pages[idx], v_pages[idx] = ko, vo
    ref, k_after, v_after = ref_gqa_prefill_paged_rope(q, k_new, v_new, k_pages, v_pages, cu, cache, table, cos, sin, page_size=page,
                                                       rotary_dim=rd, is_causal=is_causal, softcap=softcap or 0.0)
    if config is not None:
        key = "gqa_prefill_paged_with_kv_cache_rope_fwd_kernel"
        base = op.kernel_map[key]
        op.kernel_map = dict(op.kernel_map)
        op.kernel_map[key] = type("Forced", (base,), {"default_config": property(lambda self: dict(config))})
    dev = [t.to(DEV) for t in (q, k_new, v_new, k_pages, v_pages)]
    one = torch.ones(1, dtype=torch.float32, device=DEV)
    q_before, k_before = dev[0].clone(), dev[1].clone()
    out = op(*dev, one, one.clone(), cu.to(DEV), cache.to(DEV), table.to(DEV), max(q_lens))
    torch.cuda.synchronize()
    assert torch.equal(dev[0], q_before) and torch.equal(dev[1], k_before)          # inputs are not rotated in place
    torch.testing.assert_close(out.float().cpu(), ref.float(), atol=atol, rtol=1e-2)
    # appended keys: the rotated chunk.  Kernel and oracle both evaluate x*c + r*s in fp32 on the same 16-bit operands and
    # round once, but not with the same fp32 roundings (fused multiply-add or not), so they may differ by one 16-bit ulp of
    # the result plus, where the two products cancel, a few fp32 ulps of the operands (|x| < 5 here).  Values are copied;
    # every other row of the pool is as before.
    assert torch.equal(dev[4].cpu(), v_after)
    k_dev = dev[3].cpu()
    torch.testing.assert_close(k_dev.float(), k_after.float(), atol=2e-6, rtol=torch.finfo(dtype).eps)
    touched = torch.zeros(k_pages.shape[0], dtype=torch.bool)
    for b, (n, old) in enumerate(zip(q_lens, old_lens)):
        for i in range(n):
            touched[physical_pos(table, b, old + i, page)] = True
    assert torch.equal(k_dev[~touched], k_pages[~touched])


@pytest.mark.gpu
@pytest.mark.parametrize("rope", [False, True])
def test_prefill_kernels_capture_into_a_graph_and_replay_on_new_values(rope):
    """The library calls behind the prefill kernel classes enqueue only (no allocation, no synchronisation, no host read
    of device data), so a kernel's ``forward`` can be captured in a HIP graph: every replay, with new query and chunk
    values written into the same tensors, must equal the eager call on the same contents -- output and appended pages."""
    require_gfx950()
    from tileops_amd.kernels import GQAPrefillPagedWithKVCacheFwdKernel, GQAPrefillPagedWithKVCacheRopeFwdKernel

    q_lens, old_lens, heads, heads_kv, dim, dtype = [40, 7, 130], [300, 0, 1000], 16, 4, 128, torch.bfloat16
    case = [t.to(DEV) for t in _case(q_lens, old_lens, heads, heads_kv, dim, dtype, page=64, max_pages=20, seed=51)]
    q, k_new, v_new, k_pages, v_pages, ks, vs, cu, cache, table = case
    kw = dict(batch=3, heads=heads, heads_kv=heads_kv, max_pages_per_req=20, page_size=64, dim=dim, is_causal=True, dtype=dtype)
    if rope:
        kernel = GQAPrefillPagedWithKVCacheRopeFwdKernel(max_position=1200, rotary_dim=64, **kw)
        cos, sin = (t.to(DEV) for t in rope_tables(64, 1200, 10000.0, dtype))
        call = lambda: kernel(q, k_new, v_new, k_pages, v_pages, ks, vs, cu, cache, table, max(q_lens), cos, sin)  # noqa: E731
    else:
        kernel = GQAPrefillPagedWithKVCacheFwdKernel(**kw)
        call = lambda: kernel(q, k_new, v_new, k_pages, v_pages, ks, vs, cu, cache, table, max(q_lens))  # noqa: E731
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            call()  # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_g = call()
    previous = None
    for it in range(3):
        if it:
            q.mul_(-0.75)
            k_new.mul_(1.0 + 0.5 * it)
            v_new.add_(0.125 * it)
        graph.replay()
        torch.cuda.synchronize()
        pages_g = (k_pages.clone(), v_pages.clone())
        eager = call()
        torch.cuda.synchronize()
        assert torch.isfinite(eager).all()
        assert torch.equal(out_g, eager), f"replay {it} differs from the eager call"
        assert torch.equal(pages_g[0], k_pages) and torch.equal(pages_g[1], v_pages)
        assert previous is None or not torch.equal(previous, eager)
        previous = eager.clone()


@pytest.mark.gpu
@pytest.mark.parametrize("page, max_pages", [(64, 12), (16, 45)], ids=["page64", "page16-odd-page-count"])
def test_fp8_cache_long_chunks_with_a_corrupt_cache_length_stay_inside_their_slot(page, max_pages):
    """The dequantise-once route of long FP8-cache chunks under ``validate_inputs=False`` and a ``cache_seqlens`` entry of
    ``2**31 - 5``: the packed slot of that sequence is filled from the pages its table row addresses and no further, its
    chunk is appended nowhere, the output is finite, and the sane sequences match the oracle.  With 16-token pages and an odd
    page count the slot is a few rows longer than the table row can address (slots are multiples of 32 rows)."""
    require_gfx950()
    H, Hkv, D, ql = 16, 4, 128, 260  # 1040 query rows per kv head
    q_lens, old_lens = [ql, ql, 256], [300, 100, 0]
    case = list(_case(q_lens, old_lens, H, Hkv, D, torch.float16, fp8=True, page=page, max_pages=max_pages, seed=19))
    q, k_new, v_new, k_pages, v_pages, ks, vs, cu, cache, table = case
    packed = native.prefill_paged_workspace(3, max(q_lens), sum(q_lens), H, Hkv, D, page, max_pages, torch.float16, FP8, native.KERNEL_AUTO)
    assert packed >= 3 * max_pages * page * Hkv * D * 4  # the route under test
    op = PrefillOp(batch=3, heads=H, heads_kv=Hkv, max_pages_per_req=max_pages, page_size=page, dim=D, is_causal=True, cache_dtype=FP8,
                   validate_inputs=False)
    dev = [t.to(DEV) for t in case]
    bad = cache.clone()
    bad[1] = 2**31 - 5
    dev[8] = bad.to(DEV)
    kp_before, vp_before = dev[3].clone(), dev[4].clone()
    out = op(*dev, max(q_lens)).float().cpu()
    torch.cuda.synchronize()
    assert torch.isfinite(out).all()
    row1 = torch.cat([torch.arange(int(p) * page, (int(p) + 1) * page) for p in table[1]])
    assert torch.equal(dev[3].cpu().view(torch.uint8)[row1], kp_before.cpu().view(torch.uint8)[row1])  # nothing appended
    assert torch.equal(dev[4].cpu().view(torch.uint8)[row1], vp_before.cpu().view(torch.uint8)[row1])
    ref_out, _, _ = ref_gqa_prefill_paged(*case, page_size=page, is_causal=True)
    for lo, hi in ((0, ql), (2 * ql, 2 * ql + 256)):
        torch.testing.assert_close(out[lo:hi], ref_out.float()[lo:hi], atol=8e-2, rtol=2e-2)


@pytest.mark.gpu
@pytest.mark.parametrize("kernel", [native.KERNEL_GENERIC, native.KERNEL_AUTO], ids=["general", "mfma"])
@pytest.mark.parametrize("rope", [False, True])
def test_a_cache_length_near_int_max_is_clamped_not_wrapped(kernel, rope):
    """With ``validate_inputs=False`` nothing stops a corrupt ``cache_seqlens`` entry.  ``2**31 - 5`` plus an eight-token chunk
    must not wrap to a negative number (which would read as an empty sequence and return zeros): the length saturates at what
    the block-table row addresses, the chunk -- whose positions lie outside that row -- is appended nowhere, and the sequence's
    rows are a bottom-right-causal decode over the row's whole capacity.  The sane sequences of the batch are not disturbed."""
    require_gfx950()
    H, Hkv, D, page, max_pages, ql = 32, 8, 128, 64, 4, 8
    q_lens, old_lens = [ql, ql, ql], [100, 50, 30]
    case = list(_case(q_lens, old_lens, H, Hkv, D, torch.bfloat16, page=page, max_pages=max_pages, seed=17))
    g = torch.Generator().manual_seed(18)
    case[3] = torch.randn(case[3].shape, generator=g).to(torch.bfloat16)  # every pool row holds data: the clamped sequence
    case[4] = torch.randn(case[4].shape, generator=g).to(torch.bfloat16)  # attends to all 256 tokens of its row
    q, k_new, v_new, k_pages, v_pages, ks, vs, cu, cache, table = case
    kw = dict(fuse_rope=True, max_position=1024, rotary_dim=D) if rope else {}
    op = PrefillOp(batch=3, heads=H, heads_kv=Hkv, max_pages_per_req=max_pages, page_size=page, dim=D, is_causal=True,
                   validate_inputs=False, **kw)
    dev = [t.to(DEV) for t in case]
    call = op.attention_call(torch.bfloat16, torch.device(DEV, 0))
    op._get_kernel(tuple(dev), op.select_kernel_key(tuple(op.kernel_map), call), call).config["kernel"] = kernel
    bad = cache.clone()
    bad[1] = 2**31 - 5
    dev[8] = bad.to(DEV)
    kp_before, vp_before = dev[3].clone(), dev[4].clone()
    out = op(*dev, ql).float().cpu()
    torch.cuda.synchronize()
    assert torch.isfinite(out).all()
    kp_after, vp_after = dev[3].cpu(), dev[4].cpu()
    row1 = torch.cat([torch.arange(int(p) * page, (int(p) + 1) * page) for p in table[1]])
    assert torch.equal(kp_after[row1], kp_before.cpu()[row1]) and torch.equal(vp_after[row1], vp_before.cpu()[row1])  # nothing appended
    # the corrupt sequence: a decode of its eight rows over the 256 tokens its table row addresses
    q1 = q[ql:2 * ql]
    if rope:
        cos, sin = op._rope_tables(torch.device(DEV), torch.bfloat16)
        pos = torch.full((ql,), 1023, dtype=torch.long)  # positions past the tables read the last entry
        q1 = apply_neox_rope(q1, pos, cos.cpu(), sin.cpu(), D)
    want1 = ref_paged_gqa_decode(q1.view(1, ql, H, D), kp_after, vp_after, torch.tensor([max_pages * page], dtype=torch.int32), table[1:2],
                                 page_size=page, is_causal=True).float().view(ql, H, D)
    torch.testing.assert_close(out[ql:2 * ql], want1, atol=8e-2, rtol=1e-2)
    assert out[ql:2 * ql].abs().max() > 1e-3  # (zeros are what a wrapped length used to give)
    # the sane sequences against the oracle run on the uncorrupted lengths
    if rope:
        cos, sin = op._rope_tables(torch.device(DEV), torch.bfloat16)
        ref_out, _, _ = ref_gqa_prefill_paged_rope(q, k_new, v_new, k_pages, v_pages, cu, cache, table, cos.cpu(), sin.cpu(),
                                                   page_size=page, is_causal=True, rotary_dim=D)
    else:
        ref_out, _, _ = ref_gqa_prefill_paged(*case, page_size=page, is_causal=True)
    for b in (0, 2):
        torch.testing.assert_close(out[b * ql:(b + 1) * ql], ref_out.float()[b * ql:(b + 1) * ql], atol=8e-2, rtol=1e-2)
