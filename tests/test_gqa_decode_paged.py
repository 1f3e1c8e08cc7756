"""GPU parity tests of the paged GQA decode ops against the CPU oracle, through the op layer and the C ABI.

The first block restates the reference's own test file case by case
(tests/ops/attention/test_gqa_decode_paged.py:75-272): same shapes, same workload generator semantics, same
comparison (max |diff| < 1e-3 and per-sequence cosine > 0.99 in fp16).  The rest covers what the reference
leaves untested or does not have: bf16 numerics, ragged lengths and tails, permuted tables, NaN poison in
unaddressed tokens, FP8 KV, multi-token causal queries, split invariance and the index-probe gather.
Tolerances: atol = rtol = 2e-2 for bf16, 3e-2 for FP8 KV.
"""

import math

import pytest
import torch
import torch.nn.functional as F

from oracle.paged_gqa_decode_ref import quantize_kv_per_token, ref_paged_gqa_decode
from tests.conftest import require_gfx950
from tileops_amd import native
from tileops_amd.ops import (
    GroupedQueryAttentionDecodePagedWithKVCacheFwdOp as PagedOp,
    GroupedQueryAttentionMultiTokenDecodePagedWithKVCacheFwdOp as MultiOp,
)
from tileops_amd.workloads import GroupedQueryAttentionDecodePagedWorkload

pytestmark = pytest.mark.gpu
DEV = "cuda"
KERNELS = ["gqa_decode_paged_kernel", "gqa_decode_paged_mfma_kernel"]


def _maxdiff_cosine_compare(out, ref, batch, atol=1e-3):
    """tests/ops/attention/test_gqa_decode_paged.py:17-28."""
    out, ref = out.float().cpu(), ref.float()
    max_diff = (out - ref).abs().max().item()
    assert max_diff < atol, f"max diff {max_diff} too large (atol={atol})"
    cos = F.cosine_similarity(out.reshape(batch, -1), ref.reshape(batch, -1), dim=-1, eps=1e-8)
    assert cos.min() > 0.99, f"cosine similarity {cos.min().item()} too low"


def _check_reference_style(op, wl, inputs, atol=1e-3):
    q, k, v, lens, table = inputs
    ref = ref_paged_gqa_decode(q.cpu(), k.cpu(), v.cpu(), lens.cpu(), table.cpu(), page_size=wl.page_size,
                               sm_scale=wl.sm_scale, softcap=wl.softcap)
    out = op(q, k, v, lens, table)
    assert out.shape == q.shape and out.dtype == q.dtype
    _maxdiff_cosine_compare(out, ref, wl.batch, atol)


# --- the reference's cases ----------------------------------------------------------------------------------
@pytest.mark.parametrize(
    "batch, heads, heads_kv, seqlen_kv, dim, page_size",
    [(1, 16, 8, 512, 128, 128), (2, 8, 4, 1024, 64, 256), (1, 32, 8, 256, 128, 64), (1, 8, 4, 1024, 64, 256),
     (2, 16, 8, 512, 128, 128), (1, 16, 4, 2048, 128, 512), (1, 32, 16, 512, 64, 128)],
)
def test_gqa_decode_paged_op(batch, heads, heads_kv, seqlen_kv, dim, page_size):
    require_gfx950()
    wl = GroupedQueryAttentionDecodePagedWorkload(batch, heads, heads_kv, seqlen_kv, dim, page_size, torch.float16)
    op = PagedOp(batch=batch, heads=heads, heads_kv=heads_kv, seqlen_kv=seqlen_kv, dim=dim, page_size=page_size, tune=False)
    _check_reference_style(op, wl, wl.gen_inputs(DEV))


def test_gqa_decode_paged_non_divisible_128_page_split():
    """page_size=192 uses 64-token tiles without skipping page tails; reversed block table, full length."""
    require_gfx950()
    batch, heads, heads_kv, seqlen_kv, dim, page_size = 1, 16, 4, 3072, 128, 192
    wl = GroupedQueryAttentionDecodePagedWorkload(batch, heads, heads_kv, seqlen_kv, dim, page_size, torch.float16)
    q, k, v, lens, table = wl.gen_inputs(DEV)
    lens.fill_(seqlen_kv)
    table.copy_(torch.arange(seqlen_kv // page_size, device=DEV, dtype=torch.int32).flip(0).unsqueeze(0))
    op = PagedOp(batch, heads, heads_kv, seqlen_kv, dim, page_size)
    kernel = op._get_kernel((q,), torch.float16)
    assert page_size % kernel.config["block_N"] == 0
    assert {c["block_N"] for c in kernel.autotune_configs} == {64}
    _check_reference_style(op, wl, (q, k, v, lens, table))


@pytest.mark.parametrize("page_size", [96, 160, 224])
def test_gqa_decode_paged_rejects_unsupported_page_tile(page_size):
    require_gfx950()
    op = PagedOp(1, 16, 4, page_size * 16, 128, page_size)
    with pytest.raises(ValueError, match="matches no supported block_N"):
        op._get_kernel((torch.empty(1, device=DEV),), torch.float16)


@pytest.mark.parametrize("sm_scale, softcap", [pytest.param(0.25, None, id="custom-sm-scale"), pytest.param(None, 2.0, id="softcap")])
def test_gqa_decode_paged_op_softmax_controls(sm_scale, softcap):
    require_gfx950()
    batch, heads, heads_kv, seqlen_kv, dim, page_size = 1, 16, 8, 512, 128, 128
    wl = GroupedQueryAttentionDecodePagedWorkload(batch, heads, heads_kv, seqlen_kv, dim, page_size, torch.float16,
                                                  sm_scale=sm_scale, softcap=softcap)
    op = PagedOp(batch=batch, heads=heads, heads_kv=heads_kv, seqlen_kv=seqlen_kv, dim=dim, page_size=page_size,
                 sm_scale=sm_scale, softcap=softcap)
    _check_reference_style(op, wl, wl.gen_inputs(DEV))


@pytest.mark.parametrize("real_len, reverse_pages", [pytest.param(512, False, id="no-split"), pytest.param(4096, True, id="ctx-reversed-pages")])
def test_gqa_decode_paged_bs1_both_tiers(real_len, reverse_pages):
    """Batch-1 short (one partial) and long (many partials) contexts, with output-distinguishing page translation."""
    require_gfx950()
    batch, heads, heads_kv, seqlen_kv, dim, page_size = 1, 32, 4, 4096, 128, 256
    wl = GroupedQueryAttentionDecodePagedWorkload(batch, heads, heads_kv, seqlen_kv, dim, page_size, torch.float16)
    op = PagedOp(batch, heads, heads_kv, seqlen_kv, dim, page_size)
    q, k, v, lens, table = wl.gen_inputs(DEV, seed=0)
    lens.fill_(real_len)
    if reverse_pages:
        table = table.flip(-1).contiguous()
    _check_reference_style(op, wl, (q, k, v, lens, table))


@pytest.mark.parametrize(
    "batch, dtype, dim, page_size, softcap",
    [pytest.param(2, torch.float16, 128, 256, None, id="batched"), pytest.param(1, torch.bfloat16, 128, 256, None, id="bf16"),
     pytest.param(1, torch.float16, 64, 256, None, id="head-dim"), pytest.param(1, torch.float16, 128, 16, None, id="small-page"),
     pytest.param(1, torch.float16, 128, 192, None, id="generic-page-tile"), pytest.param(1, torch.float16, 128, 256, 2.0, id="softcap")],
)
def test_gqa_decode_paged_dispatch_lands_on_a_kernel_that_serves_the_call(batch, dtype, dim, page_size, softcap):
    """Every shape of the reference's dispatch table is served: by the specialised kernel inside its region,
    by the general one elsewhere (head dims 64 and 128 are inside the MFMA region, page 192 is not)."""
    require_gfx950()
    seqlen_kv = 8064 if page_size == 192 else 8192
    op = PagedOp(batch, 32, 4, seqlen_kv, dim, page_size, softcap=softcap)
    kernel = op._get_kernel((torch.empty(1, device=DEV),), dtype)
    call = op.attention_call(dtype, None, torch.device(DEV, 0))
    expected = "GQADecodePagedMfmaKernel" if op.kernel_map["gqa_decode_paged_mfma_kernel"].applies(call) else "GQADecodePagedKernel"
    assert kernel.__class__.__name__ == expected
    assert expected == "GQADecodePagedMfmaKernel"  # head dims 64, 128, 256; pages of 16 or a multiple of 32 tokens


# --- beyond the reference's coverage ------------------------------------------------------------------------
def _ragged_case(B, H, H_kv, D, page, lens, dtype, q_len=1, fp8=False, seed=0, spare_pages=3, poison=True):
    g = torch.Generator().manual_seed(seed)
    need = [math.ceil(n / page) for n in lens]
    n_pages = sum(need) + spare_pages
    q_shape = (B, H, D) if q_len == 1 else (B, q_len, H, D)
    q = torch.randn(q_shape, generator=g).to(dtype)
    k = torch.randn(n_pages * page, H_kv, D, generator=g)
    v = torch.randn(n_pages * page, H_kv, D, generator=g)
    perm = torch.randperm(n_pages, generator=g)
    table = torch.full((B, max(1, max(need))), int(perm[-1]), dtype=torch.int32)  # unused entries name a spare page
    used = torch.zeros(n_pages * page, dtype=torch.bool)
    at = 0
    for b, n in enumerate(lens):
        table[b, :need[b]] = perm[at:at + need[b]].to(torch.int32)
        for j in range(need[b]):
            p = int(perm[at + j])
            used[p * page: p * page + min(page, n - j * page)] = True
        at += need[b]
    if fp8:
        k, ks = quantize_kv_per_token(k)
        v, vs = quantize_kv_per_token(v)
    else:
        k, v, ks, vs = k.to(dtype), v.to(dtype), None, None
    if poison:  # every token no (table, length) pair addresses holds NaN; fp8 NaN is 0x7F
        if fp8:
            k.view(torch.uint8)[~used] = 0x7F
            v.view(torch.uint8)[~used] = 0x7F
            ks[~used] = float("nan")
            vs[~used] = float("nan")
        else:
            k[~used] = float("nan")
            v[~used] = float("nan")
    return q, k, v, torch.tensor(lens, dtype=torch.int32), table, ks, vs


def _run_and_compare(op, case, page, tol, **ref_kw):
    q, k, v, lens, table, ks, vs = case
    ref = ref_paged_gqa_decode(q, k, v, lens, table, page_size=page, k_scale=ks, v_scale=vs, **ref_kw)
    dev = [None if t is None else t.to(DEV) for t in case]
    out = op(*dev[:5]) if ks is None else op(*dev)
    torch.cuda.synchronize()
    assert torch.isfinite(out).all()
    torch.testing.assert_close(out.float().cpu(), ref.float(), atol=tol, rtol=tol)
    return out


@pytest.mark.parametrize("kernel_key", KERNELS)
@pytest.mark.parametrize("dtype, fp8, tol", [(torch.bfloat16, False, 2e-2), (torch.float16, False, 2e-2), (torch.bfloat16, True, 3e-2)])
def test_ragged_lengths_tails_permuted_tables_and_poison(kernel_key, dtype, fp8, tol):
    """Lengths that are not page or tile multiples, a length-1 and a length-0 sequence, a far longer neighbour
    (empty splits for the short ones), every sequence on its own permuted pages, NaN everywhere else."""
    require_gfx950()
    lens = [1, 0, 63, 64, 65, 777, 4099, 130]
    case = _ragged_case(len(lens), 32, 8, 128, 64, lens, dtype, fp8=fp8, seed=21)
    op = PagedOp(len(lens), 32, 8, case[1].shape[0], 128, 64)
    if not _serves(op, kernel_key, dtype, fp8):
        pytest.skip(f"{kernel_key} does not serve this shape")
    _force(op, kernel_key)
    _run_and_compare(op, case, 64, tol)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("page", [16, 32, 64, 128])
@pytest.mark.parametrize("q_len", [1, 3], ids=["one-row-block", "two-row-blocks"])
@pytest.mark.parametrize("dim", [64, 256])
def test_fp8_cache_at_head_dims_64_and_256_on_the_mfma_kernel(dtype, page, q_len, dim):
    """64-byte rows: two fetch instructions per K tile, four lanes per token row; 256-byte rows: eight instructions, two
    128-deep score steps, sixteen V^T column blocks; each width with its own LDS swizzles.  Ragged lengths with tails, a
    length-1 and an empty sequence, permuted pages, NaN in every token that no table addresses."""
    require_gfx950()
    lens = [q_len, 0, 63, 64, 65, 777, 2051, 130]
    case = _ragged_case(len(lens), 32, 4, dim, page, lens, dtype, q_len=q_len, fp8=True, seed=57)
    if q_len == 1:
        op = PagedOp(len(lens), 32, 4, case[1].shape[0], dim, page)
    else:
        op = MultiOp(len(lens), q_len, 32, 4, case[1].shape[0], dim, page, is_causal=True)
    assert _serves(op, "gqa_decode_paged_mfma_kernel", dtype, True)
    _force(op, "gqa_decode_paged_mfma_kernel")
    _run_and_compare(op, case, page, 3e-2, **({} if q_len == 1 else {"is_causal": True}))


@pytest.mark.parametrize(
    "heads, heads_kv, dim, fp8, lens",
    [
        pytest.param(8, 1, 128, True, [70001], id="one-kv-head-fp8-2048-partitions"),
        pytest.param(32, 4, 128, False, [40000], id="256-partitions"),
        pytest.param(32, 4, 128, False, [333, 0], id="fewer-tiles-than-partitions"),
        pytest.param(16, 2, 64, False, [3000], id="head-dim-64-fewer-tiles-than-partitions"),
        pytest.param(16, 2, 256, True, [9001, 5], id="head-dim-256-fp8-two-sequences"),
        pytest.param(64, 8, 128, True, [33, 20000, 1], id="three-sequences-one-long"),
    ],
)
def test_few_sequences_spread_over_hundreds_of_partitions(heads, heads_kv, dim, fp8, lens):
    """Batch 1-3: every sequence spans far more than 64 partitions of the tile stream on average, which takes the
    sixteen-wave merge (four LSEs per lane, lane groups on different partitions, the tail loop beyond 256 partitions,
    and -- with fewer tiles than partitions -- the walk over the partitions that own a tile)."""
    require_gfx950()
    case = _ragged_case(len(lens), heads, heads_kv, dim, 64, lens, torch.bfloat16, fp8=fp8, seed=71)
    op = PagedOp(len(lens), heads, heads_kv, case[1].shape[0], dim, 64)
    assert _serves(op, "gqa_decode_paged_mfma_kernel", torch.bfloat16, fp8)
    _force(op, "gqa_decode_paged_mfma_kernel")
    n_parts = native.decode_workspace(len(lens), 1, heads, heads_kv, dim, 64, case[4].shape[1], torch.bfloat16,
                                      torch.float8_e4m3fn if fp8 else torch.bfloat16, 0, native.KERNEL_MFMA)[1]
    assert n_parts > 64 * len(lens)
    _run_and_compare(op, case, 64, 3e-2 if fp8 else 2e-2)


@pytest.mark.parametrize(
    "heads, heads_kv, dim, fp8, q_len, lens",
    [
        pytest.param(32, 8, 128, False, 1, [4096] + [64] * 15, id="one-sequence-over-a-hundred-partitions-among-short-ones"),
        pytest.param(32, 8, 128, True, 1, [2048] + [256] * 31, id="fp8-one-sequence-over-dozens-of-partitions"),
        pytest.param(32, 8, 128, True, 1, [700, 0, 5000, 33, 1, 2000, 64, 900] * 4, id="fp8-ragged-with-empty"),
        pytest.param(16, 4, 256, False, 1, [3000, 100, 100, 100, 1500, 100, 100, 100] * 2, id="head-dim-256-two-halves"),
        pytest.param(32, 8, 64, True, 2, [1000 + 37 * i for i in range(32)], id="head-dim-64-fp8-two-query-tokens"),
        pytest.param(32, 8, 128, False, 1, [20] * 16, id="fewer-tiles-than-partitions-falls-back"),
    ],
)
def test_long_and_short_sequences_share_the_partitions(heads, heads_kv, dim, fp8, q_len, lens):
    """Batches whose sequences span at most eight partitions on average (the one-wave-per-row merge), with single
    sequences far outside that average: inside one partition (no merge), over two to eight, over dozens and over more than
    a hundred partitions (second and later rounds of partial loads), empty ones, and a call with fewer tiles than
    partitions.  Then a shorter call on the same, now dirty, workspace shapes."""
    require_gfx950()
    kv = torch.float8_e4m3fn if fp8 else torch.bfloat16
    case = _ragged_case(len(lens), heads, heads_kv, dim, 64, lens, torch.bfloat16, q_len=q_len, fp8=fp8, seed=83)
    n_parts = native.decode_workspace(len(lens), q_len, heads, heads_kv, dim, 64, case[4].shape[1], torch.bfloat16, kv, 0,
                                      native.KERNEL_MFMA)[1]
    assert n_parts <= 8 * len(lens)
    if q_len == 1:
        op = PagedOp(len(lens), heads, heads_kv, case[1].shape[0], dim, 64)
    else:
        op = MultiOp(len(lens), q_len, heads, heads_kv, case[1].shape[0], dim, 64)
    _force(op, "gqa_decode_paged_mfma_kernel")
    tol = 3e-2 if fp8 else 2e-2
    kw = {"is_causal": True} if q_len > 1 else {}
    out = _run_and_compare(op, case, 64, tol, **kw)
    assert out.shape == case[0].shape
    short = [max(n // 3, 0) for n in lens]
    case2 = _ragged_case(len(lens), heads, heads_kv, dim, 64, short, torch.bfloat16, q_len=q_len, fp8=fp8, seed=84)
    if case2[4].shape[1] == case[4].shape[1] and case2[1].shape[0] == case[1].shape[0]:
        _run_and_compare(op, case2, 64, tol, **kw)


def _serves(op, key, dtype, fp8):
    call = op.attention_call(dtype, torch.float8_e4m3fn if fp8 else None, torch.device(DEV, 0))
    return op.kernel_map[key].refusal(call) is None


def _force(op, key):
    """Make selection return *key* (the other key is removed from the map)."""
    op.kernel_map = {key: op.kernel_map[key]}


@pytest.mark.parametrize("kernel_key", KERNELS)
@pytest.mark.parametrize("page", [16, 32, 64, 128, 256])
def test_page_sizes(kernel_key, page):
    require_gfx950()
    lens = [300, 1000, 17]
    case = _ragged_case(3, 32, 8, 128, page, lens, torch.bfloat16, seed=22)
    op = PagedOp(3, 32, 8, case[1].shape[0], 128, page)
    if not _serves(op, kernel_key, torch.bfloat16, False):
        pytest.skip(f"{kernel_key} does not serve page_size {page}")
    _force(op, kernel_key)
    _run_and_compare(op, case, page, 2e-2)


@pytest.mark.parametrize("kernel_key", KERNELS)
@pytest.mark.parametrize("heads, heads_kv", [(8, 8), (16, 8), (64, 8), (128, 8), (4, 1), (24, 3)])
def test_group_sizes(kernel_key, heads, heads_kv):
    require_gfx950()
    lens = [200, 1500]
    case = _ragged_case(2, heads, heads_kv, 128, 64, lens, torch.bfloat16, seed=23)
    op = PagedOp(2, heads, heads_kv, case[1].shape[0], 128, 64)
    if not _serves(op, kernel_key, torch.bfloat16, False):
        pytest.skip(f"{kernel_key} does not serve heads {heads}/{heads_kv}")
    _force(op, kernel_key)
    _run_and_compare(op, case, 64, 2e-2)


@pytest.mark.parametrize("kernel_key", KERNELS)
@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("q_len, is_causal", [(8, True), (3, True), (4, False)])
def test_multi_token_causal_chunk(kernel_key, fp8, q_len, is_causal):
    require_gfx950()
    lens = [1500, 300, q_len, 65]
    case = _ragged_case(4, 64, 8, 128, 64, lens, torch.bfloat16, q_len=q_len, fp8=fp8, seed=24)
    op = MultiOp(4, q_len, 64, 8, case[1].shape[0], 128, 64, is_causal=is_causal)
    if not _serves(op, kernel_key, torch.bfloat16, fp8):
        pytest.skip(f"{kernel_key} does not serve q_len {q_len}")
    _force(op, kernel_key)
    out = _run_and_compare(op, case, 64, 3e-2 if fp8 else 2e-2, is_causal=is_causal)
    if is_causal:
        # query i of the chunk equals a single-token decode at length len - q_len + i + 1
        q, k, v, lens_t, table, ks, vs = [None if t is None else t.to(DEV) for t in case]
        single = PagedOp(4, 64, 8, k.shape[0], 128, 64)
        i = q_len - 2
        lens_i = (lens_t - q_len + i + 1).clamp(min=0).to(torch.int32)
        args = (q[:, i].contiguous(), k, v, lens_i, table) + (() if ks is None else (ks, vs))
        torch.testing.assert_close(out[:, i].float(), single(*args).float(), atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("dim", [64, 128, 256])
def test_many_rows_merged_four_at_a_time(fp8, dim):
    """More than 4096 rows in the call (40 sequences x 8 query tokens x 32 heads): the merge kernel's waves take four rows each
    and have all their partial rows in flight together.  Ragged lengths so that sequences lie in one partition, in a few, or
    are empty; the general kernel (its own merge) is the second opinion beside the oracle."""
    require_gfx950()
    g = torch.Generator().manual_seed(77)
    B, q_len, H, H_kv = 40, 8, 32, 4
    lens = [int(x) for x in torch.randint(q_len, 3000, (B,), generator=g)]
    lens[3], lens[17], lens[39] = 0, q_len, 6000
    case = _ragged_case(B, H, H_kv, dim, 64, lens, torch.bfloat16, q_len=q_len, fp8=fp8, seed=78)
    op = MultiOp(B, q_len, H, H_kv, case[1].shape[0], dim, 64, is_causal=True)
    _force(op, "gqa_decode_paged_mfma_kernel")
    out = _run_and_compare(op, case, 64, 3e-2 if fp8 else 2e-2, is_causal=True)
    other = MultiOp(B, q_len, H, H_kv, case[1].shape[0], dim, 64, is_causal=True)
    _force(other, "gqa_decode_paged_kernel")
    args = [None if t is None else t.to(DEV) for t in case]
    args = tuple(args[:5]) + (() if args[5] is None else (args[5], args[6]))
    torch.testing.assert_close(out.float(), other(*args).float(), atol=3e-2 if fp8 else 2e-2, rtol=3e-2 if fp8 else 2e-2)


@pytest.mark.parametrize("dtype, fp8, tol", [(torch.bfloat16, False, 2e-2), (torch.float16, False, 2e-2), (torch.bfloat16, True, 3e-2),
                                             (torch.float16, True, 3e-2)])
@pytest.mark.parametrize(
    "q_len, heads, heads_kv",
    [
        pytest.param(8, 64, 8, id="rows64-ring-of-2"),
        pytest.param(16, 24, 3, id="rows128-ring-of-4-three-kv-heads"),
        pytest.param(12, 8, 1, id="rows96-odd-row-groups-one-kv-head"),
        pytest.param(24, 16, 2, id="rows192-six-row-groups-ring-of-2"),
        pytest.param(32, 64, 8, id="rows256-ring-of-8-or-4"),
        pytest.param(40, 16, 2, id="rows320-ten-row-groups"),
    ],
)
@pytest.mark.parametrize("dim", [128, 64, 256])
def test_many_query_rows_per_kv_head_share_their_stages(dtype, fp8, tol, q_len, heads, heads_kv, dim):
    """More than 32 query rows per kv head: the row groups of a kv head run as 2, 4 or 8 waves around one LDS ring (or
    fall back to one wave of four row blocks when their number is odd).  Ragged lengths so that partitions start and
    end inside sequences, tails shorter than a tile, a sequence shorter than the chunk, NaN in every unaddressed token;
    head counts that leave the grid with workgroups past the last (partition, kv head)."""
    require_gfx950()
    lens = [2100, q_len, q_len + 33, 700, q_len + 31, q_len + 1]
    case = _ragged_case(len(lens), heads, heads_kv, dim, 64, lens, dtype, q_len=q_len, fp8=fp8, seed=31)
    op = MultiOp(len(lens), q_len, heads, heads_kv, case[1].shape[0], dim, 64, is_causal=True)
    if not _serves(op, "gqa_decode_paged_mfma_kernel", dtype, fp8):
        pytest.skip("the MFMA kernel does not serve this shape")
    _force(op, "gqa_decode_paged_mfma_kernel")
    out = _run_and_compare(op, case, 64, tol, is_causal=True)
    # and against the other implementation, which shares none of the tiling
    other = MultiOp(len(lens), q_len, heads, heads_kv, case[1].shape[0], dim, 64, is_causal=True)
    if _serves(other, "gqa_decode_paged_kernel", dtype, fp8):
        _force(other, "gqa_decode_paged_kernel")
        dev = [None if t is None else t.to(DEV) for t in case]
        ref2 = other(*dev[:5]) if case[5] is None else other(*dev)
        torch.testing.assert_close(out.float(), ref2.float(), atol=tol, rtol=tol)


@pytest.mark.parametrize("num_split", [1, 2, 3, 7])
@pytest.mark.parametrize(
    "q_len, heads, heads_kv, dim, fp8",
    [
        pytest.param(8, 64, 8, 128, True, id="fp8-ring-of-2"),
        pytest.param(16, 32, 4, 128, True, id="fp8-ring-of-4"),
        pytest.param(16, 32, 4, 128, False, id="bf16-ring-of-4"),
        pytest.param(32, 32, 4, 128, False, id="bf16-ring-of-8"),
        pytest.param(8, 64, 8, 64, False, id="bf16-head-dim-64-ring-of-2"),
        pytest.param(32, 32, 4, 256, False, id="bf16-head-dim-256-ring-of-8"),
    ],
)
def test_ring_waves_walk_many_tiles_over_sequence_borders(num_split, q_len, heads, heads_kv, dim, fp8):
    """The tile stream cut into one, two, three or seven ranges only, so that every wave of a shared ring walks dozens
    of tiles: steps of two tiles per barrier (half of a four-stage ring) wherever two tiles of one sequence are left,
    steps of one at the end of sequences with an odd number of tiles, at one-tile sequences and at the end of a range,
    with the ring's refill running across sequence borders.  Against the oracle, NaN in every unaddressed token."""
    require_gfx950()
    lens = [2100, q_len, q_len + 33, 700, 64 + q_len, q_len + 1, 1500, 96, 4000]
    case = _ragged_case(len(lens), heads, heads_kv, dim, 64, lens, torch.bfloat16, q_len=q_len, fp8=fp8, seed=97)
    q, k, v, seqlens, table, ks, vs = case
    ref = ref_paged_gqa_decode(q, k, v, seqlens, table, page_size=64, k_scale=ks, v_scale=vs, is_causal=True)
    dev = [None if t is None else t.to(DEV) for t in case]
    out = torch.ops.tileops_amd.gqa_paged_decode(dev[0], dev[1], dev[2], dev[3], dev[4], dev[5], dev[6], q_len, heads, heads_kv, dim, 64,
                                                 dim ** -0.5, 0.0, True, num_split, native.KERNEL_MFMA)
    torch.cuda.synchronize()
    assert torch.isfinite(out).all()
    tol = 3e-2 if fp8 else 2e-2
    torch.testing.assert_close(out.float().cpu(), ref.float(), atol=tol, rtol=tol)
    # the same call cut into the default number of ranges (a tile or two per wave) differs by fp32 summation order and, in
    # calls with this many query rows, by the partial rows' one rounding to the query's type
    auto = torch.ops.tileops_amd.gqa_paged_decode(dev[0], dev[1], dev[2], dev[3], dev[4], dev[5], dev[6], q_len, heads, heads_kv, dim, 64,
                                                  dim ** -0.5, 0.0, True, 0, native.KERNEL_MFMA)
    torch.testing.assert_close(out.float(), auto.float(), atol=tol, rtol=tol)


@pytest.mark.parametrize("batch, q_len, many_rows", [(3, 8, False), (9, 8, True), (70, 1, False)])
def test_partial_rows_are_fp32_for_few_query_rows_and_rounded_once_to_the_query_type_for_many(batch, q_len, many_rows):
    """A range of the tile stream that ends inside a sequence leaves a partial row for the merge.  Single-token decode, and
    multi-token calls with up to 4096 query rows, keep those rows in fp32: cutting the stream differently moves the result by
    fp32 summation order, far below one fp16 ulp.  Multi-token calls with more rows (verify steps of a batch, prefill chunks)
    store them in the query's type, as the reference stores every partial (gqa_decode_paged.py:216-217,718-722): each partial is rounded once, the merged row
    is a convex combination of them, so the result moves by at most one ulp of the largest value plus its own rounding."""
    require_gfx950()
    heads, heads_kv, dim = 64, 8, 128
    assert (q_len > 1 and heads * q_len * batch > 4096) == many_rows
    assert heads * q_len * batch > 4096 or batch == 3  # (the single-token case is past the row count, and still fp32)
    lens = ([2100, 8, 41, 700, 72, 9, 1500, 96, 4000] + [(97 * i) % 900 + 33 for i in range(61)])[:batch]
    case = _ragged_case(len(lens), heads, heads_kv, dim, 64, lens, torch.float16, q_len=q_len, seed=131)
    q, k, v, seqlens, table, _, _ = case
    dev = [None if t is None else t.to(DEV) for t in case]
    run = lambda ns: torch.ops.tileops_amd.gqa_paged_decode(dev[0], dev[1], dev[2], dev[3], dev[4], dev[5], dev[6], q_len, heads, heads_kv, dim,
                                                           64, dim ** -0.5, 0.0, True, ns, native.KERNEL_MFMA).float()
    whole = run(1)   # one range per kv head: every sequence inside it, no partial rows at all
    cut = run(0)     # the default: a few tiles per wave, most sequences cut many times
    ref = ref_paged_gqa_decode(q, k, v, seqlens, table, page_size=64, is_causal=True)
    torch.testing.assert_close(whole.cpu(), ref.float(), atol=5e-3, rtol=5e-3)
    assert whole.shape == cut.shape == ref.shape
    ulp = torch.finfo(torch.float16).eps  # of values in [1, 2)
    vmax = float(torch.nan_to_num(v.float(), nan=0.0).abs().max())  # (unaddressed tokens hold NaN)
    outmax = float(whole.abs().max())
    diff = (cut - whole).abs().max().item()
    if many_rows:
        assert diff <= ulp * (0.5 * vmax + outmax), diff
    else:
        assert diff <= ulp * outmax, diff  # fp32 values a hair apart (summation order, the probabilities' own rounding), rounded to fp16


@pytest.mark.parametrize("softcap", [0.0, 30.0])
def test_closed_forms_on_device(softcap):
    require_gfx950()
    lens = [100, 1, 700]
    q, k, v, lens_t, table, _, _ = _ragged_case(3, 32, 8, 128, 64, lens, torch.bfloat16, seed=25)
    op = PagedOp(3, 32, 8, k.shape[0], 128, 64, softcap=softcap or None)
    dev = [t.to(DEV) for t in (q, k, v, lens_t, table)]
    out0 = op(torch.zeros_like(dev[0]), *dev[1:]).float().cpu()     # q = 0 -> mean of V over the valid tokens
    for b, n in enumerate(lens):
        pages = table[b, : math.ceil(n / 64)].long()
        rows = v.view(-1, 64, 8, 128)[pages].reshape(-1, 8, 128)[:n].float()
        torch.testing.assert_close(out0[b], rows.mean(0).repeat_interleave(4, dim=0), atol=1e-2, rtol=1e-2)
    out = op(*dev).float().cpu()
    torch.testing.assert_close(out[1], v[int(table[1, 0]) * 64].float().repeat_interleave(4, dim=0), atol=1e-2, rtol=1e-2)  # len 1


def test_generic_kernel_is_invariant_to_the_split_count():
    require_gfx950()
    lens = [4099, 777]
    q, k, v, lens_t, table, _, _ = [None if t is None else t.to(DEV) for t in _ragged_case(2, 32, 8, 128, 64, lens, torch.bfloat16, seed=26)]
    outs = []
    for ns in (1, 2, 5, 64):
        out = torch.empty_like(q)
        nbytes, nsplit, _ = native.decode_workspace(2, 1, 32, 8, 128, 64, table.shape[1], q.dtype, k.dtype, ns, native.KERNEL_GENERIC)
        ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=DEV)
        native.paged_decode(q, k, v, None, None, lens_t, table, out, ws, batch=2, q_len=1, heads=32, heads_kv=8, dim=128,
                            page_size=64, sm_scale=128 ** -0.5, softcap=0.0, causal=True, num_split=nsplit, kernel=native.KERNEL_GENERIC)
        outs.append(out.float())
    for o in outs[1:]:
        torch.testing.assert_close(o, outs[0], atol=8e-3, rtol=8e-3)  # fp32 partials: differences are bf16 output rounding


def test_kernels_agree_with_each_other_and_joint_page_permutation_is_bit_invariant():
    require_gfx950()
    lens = [2000, 513, 64]
    case = _ragged_case(3, 32, 8, 128, 64, lens, torch.bfloat16, seed=27, poison=False)
    q, k, v, lens_t, table, _, _ = [None if t is None else t.to(DEV) for t in case]
    outs = {}
    for key in KERNELS:
        op = PagedOp(3, 32, 8, k.shape[0], 128, 64)
        if not _serves(op, key, torch.bfloat16, False):
            continue
        _force(op, key)
        outs[key] = op(q, k, v, lens_t, table)
        # move every physical page and rename it in the table: the same rows are read, so not a bit may change
        n_pages = k.shape[0] // 64
        sigma = torch.randperm(n_pages, generator=torch.Generator().manual_seed(5)).to(DEV)
        k2, v2 = torch.empty_like(k), torch.empty_like(v)
        k2.view(n_pages, 64, 8, 128)[sigma] = k.view(n_pages, 64, 8, 128)
        v2.view(n_pages, 64, 8, 128)[sigma] = v.view(n_pages, 64, 8, 128)
        table2 = sigma[table.long()].to(torch.int32)
        assert torch.equal(op(q, k2, v2, lens_t, table2), outs[key])
    vals = list(outs.values())
    for o in vals[1:]:
        torch.testing.assert_close(o.float(), vals[0].float(), atol=2e-2, rtol=2e-2)


def test_wide_block_table_like_the_reference_contract_and_strided_rows():
    """The reference hands over block_table [B, N_kv/page] (pool-wide); only the leading ceil(len/page) entries matter."""
    require_gfx950()
    lens = [900, 100]
    q, k, v, lens_t, table, _, _ = _ragged_case(2, 32, 8, 128, 64, lens, torch.bfloat16, seed=28)
    n_pages = k.shape[0] // 64
    wide = torch.full((2, n_pages), n_pages - 1, dtype=torch.int32)
    wide[:, : table.shape[1]] = table
    op = PagedOp(2, 32, 8, k.shape[0], 128, 64)
    ref = ref_paged_gqa_decode(q, k, v, lens_t, table, page_size=64)
    out = op(q.to(DEV), k.to(DEV), v.to(DEV), lens_t.to(DEV), wide.to(DEV))
    torch.testing.assert_close(out.float().cpu(), ref.float(), atol=2e-2, rtol=2e-2)
    padded = torch.zeros(2, n_pages + 5, dtype=torch.int32, device=DEV)
    padded[:, :n_pages] = wide.to(DEV)
    out2 = op(q.to(DEV), k.to(DEV), v.to(DEV), lens_t.to(DEV), padded[:, :n_pages])  # row stride != width
    assert torch.equal(out2, out)


def test_gather_probe_is_bit_identical_to_torch_indexing():
    """Index-probe: K[t, h, d] encodes the physical token t, so any page-arithmetic slip shows as a wrong id."""
    require_gfx950()
    page, H_kv, D = 64, 8, 128
    lens = [1, 64, 65, 1000, 4097]
    need = [math.ceil(n / page) for n in lens]
    n_pages = sum(need) + 7
    g = torch.Generator().manual_seed(31)
    perm = torch.randperm(n_pages, generator=g)
    table = torch.zeros(len(lens), max(need), dtype=torch.int32)
    at = 0
    for b, c in enumerate(need):
        table[b, :c] = perm[at:at + c].to(torch.int32)
        at += c
    tok = torch.arange(n_pages * page, dtype=torch.int32)
    probe = (tok[:, None, None] * 1024 + torch.arange(H_kv, dtype=torch.int32)[None, :, None] * 128
             + torch.arange(D, dtype=torch.int32)[None, None, :]).contiguous()        # int32 rows: every element names itself
    lens_t = torch.tensor(lens, dtype=torch.int32)
    max_len = max(lens)
    for cache in (probe, probe.view(torch.float32)):
        dense = native.gather_probe(cache.to(DEV), lens_t.to(DEV), table.to(DEV), page, max_len).cpu()
        for b, n in enumerate(lens):
            want = cache.view(n_pages, page, H_kv, D)[table[b, : need[b]].long()].reshape(-1, H_kv, D)[:n]
            assert torch.equal(dense[b, :n].view(torch.int32), want.view(torch.int32))
            assert (dense[b, n:].view(torch.int32) == 0).all()
    # byte-wide cache rows (fp8) and the [N_kv, H_kv] scale rows go through the same routine
    k8 = torch.randint(0, 255, (n_pages * page, H_kv, D), dtype=torch.uint8, generator=g)
    dense8 = native.gather_probe(k8.to(DEV), lens_t.to(DEV), table.to(DEV), page, max_len).cpu()
    for b, n in enumerate(lens):
        want = k8.view(n_pages, page, H_kv, D)[table[b, : need[b]].long()].reshape(-1, H_kv, D)[:n]
        assert torch.equal(dense8[b, :n], want)


def test_kv_append_fp8_matches_the_quantizer_bit_for_bit():
    """Append-then-read: the appended row's bytes and scale equal the oracle quantizer's
    (tests/ops/attention/test_gqa_prefill_paged.py:398-415 checks its fused append the same way)."""
    require_gfx950()
    page, H_kv, D, B = 64, 8, 128, 5
    lens = [1, 64, 65, 200, 130]
    case = _ragged_case(B, 32, H_kv, D, page, lens, torch.bfloat16, fp8=True, seed=33, poison=False)
    q, k8, v8, lens_t, table, ks, vs = case
    g = torch.Generator().manual_seed(34)
    x_new = (torch.randn(B, H_kv, D, generator=g) * torch.tensor([1e-6, 0.1, 1.0, 10.0, 300.0])[:, None, None]).to(torch.bfloat16)
    want_q, want_s = quantize_kv_per_token(x_new)
    kd, sd = k8.to(DEV), ks.to(DEV)
    before_k, before_s = kd.clone(), sd.clone()
    native.kv_append_fp8(x_new.to(DEV), kd, sd, lens_t.to(DEV), table.to(DEV), page)
    torch.cuda.synchronize()
    touched = torch.zeros(k8.shape[0], dtype=torch.bool)
    for b, n in enumerate(lens):
        phys = int(table[b, (n - 1) // page]) * page + (n - 1) % page
        touched[phys] = True
        assert torch.equal(kd[phys].cpu().view(torch.uint8), want_q[b].view(torch.uint8))
        assert torch.equal(sd[phys].cpu(), want_s[b])
    assert torch.equal(kd.cpu().view(torch.uint8)[~touched], before_k.cpu().view(torch.uint8)[~touched])
    assert torch.equal(sd.cpu()[~touched], before_s.cpu()[~touched])


def test_kv_append_fp8_writes_nothing_for_positions_the_block_table_row_does_not_address():
    """Lengths of 0 (position -1) and beyond the row's pages: the append skips them instead of reading a page id from
    the next row (or past the table) and writing into another sequence's page."""
    require_gfx950()
    page, H_kv, D, B, width = 64, 8, 128, 4, 3
    lens = [0, width * page + 1, 70, width * page + 500]  # the last row's overrun would leave the table
    case = _ragged_case(B, 32, H_kv, D, page, [1, 1, 130, 1], torch.bfloat16, fp8=True, seed=35, poison=False)  # table of three pages a row
    q, k8, v8, _, table, ks, vs = case
    assert table.shape == (B, width) and table.is_contiguous()
    x_new = torch.randn(B, H_kv, D, generator=torch.Generator().manual_seed(36)).to(torch.bfloat16)
    want_q, want_s = quantize_kv_per_token(x_new)
    kd, sd = k8.to(DEV), ks.to(DEV)
    before_k, before_s = kd.clone(), sd.clone()
    native.kv_append_fp8(x_new.to(DEV), kd, sd, torch.tensor(lens, dtype=torch.int32, device=DEV), table.to(DEV), page)
    torch.cuda.synchronize()
    phys = int(table[2, 69 // page]) * page + 69 % page
    touched = torch.zeros(k8.shape[0], dtype=torch.bool)
    touched[phys] = True
    assert torch.equal(kd[phys].cpu().view(torch.uint8), want_q[2].view(torch.uint8)) and torch.equal(sd[phys].cpu(), want_s[2])
    assert torch.equal(kd.cpu().view(torch.uint8)[~touched], before_k.cpu().view(torch.uint8)[~touched])
    assert torch.equal(sd.cpu()[~touched], before_s.cpu()[~touched])


def test_external_builder_path_runs_the_same_kernels():
    """The plug-in's build_kernel, reached through the seam, gives the same bits as the in-tree path."""
    require_gfx950()
    from tileops_amd import backend, tileops_plugin

    saved = backend.snapshot()
    try:
        backend.restore(backend._State({}, {}, [], None))
        tileops_plugin.register(into=backend)
        case = _ragged_case(2, 32, 8, 128, 64, [700, 90], torch.bfloat16, seed=35)
        dev = [t.to(DEV) for t in case[:5]]
        ext = PagedOp(2, 32, 8, dev[1].shape[0], 128, 64)
        out_ext = ext(*dev)
        assert ext._settled_target == "mi355x"
        builtin = PagedOp(2, 32, 8, dev[1].shape[0], 128, 64, target=backend.BUILTIN)
        assert torch.equal(builtin(*dev), out_ext)
    finally:
        backend.restore(saved)


def test_tune_picks_a_config_and_stays_correct():
    require_gfx950()
    wl = GroupedQueryAttentionDecodePagedWorkload(2, 32, 8, 4096, 128, 64, torch.float16)
    op = PagedOp(2, 32, 8, 4096, 128, 64, tune=True)
    inputs = wl.gen_inputs(DEV)
    _check_reference_style(op, wl, inputs)
    kernel = next(iter(op.built_kernels(next(iter(op._kernel_roles))).values()))
    assert kernel.config in kernel.autotune_configs


@pytest.mark.parametrize("kernel_key", KERNELS)
@pytest.mark.parametrize("fp8", [False, True])
def test_more_than_64_sequences_with_empty_ones_in_between(kernel_key, fp8):
    """Batch 150: the per-wave caches of sequence lengths hold 64 entries and are refilled while a wave walks the
    tile stream; empty sequences sit at the refill boundaries, at the start and at the end."""
    require_gfx950()
    g = torch.Generator().manual_seed(5)
    lens = torch.randint(1, 400, (150,), generator=g).tolist()
    for b in (0, 63, 64, 65, 127, 128, 149):
        lens[b] = 0
    lens[66] = 3000
    case = _ragged_case(len(lens), 16, 4, 128, 32, lens, torch.bfloat16, fp8=fp8, seed=33)
    op = PagedOp(len(lens), 16, 4, case[1].shape[0], 128, 32)
    if not _serves(op, kernel_key, torch.bfloat16, fp8):
        pytest.skip(f"{kernel_key} does not serve this shape")
    _force(op, kernel_key)
    out = _run_and_compare(op, case, 32, 3e-2 if fp8 else 2e-2)
    assert (out[[0, 63, 64, 65, 127, 128, 149]] == 0).all()


@pytest.mark.parametrize("fp8", [False, True])
def test_graph_capture_and_replay_with_changing_cache_contents(fp8):
    """The call captured in a HIP graph and replayed: every replay, with eager work and synchronisation in between
    and new K/V values written into the same pool, must equal the eager result on the same contents."""
    require_gfx950()
    lens = [900, 33, 2048, 5, 1500, 64]
    case = _ragged_case(len(lens), 32, 8, 128, 64, lens, torch.bfloat16, fp8=fp8, seed=9)
    dev = [None if t is None else t.to(DEV) for t in case]
    args = dev[:5] if not fp8 else dev
    op = PagedOp(len(lens), 32, 8, case[1].shape[0], 128, 64)
    eager0 = op(*args)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            op(*args)  # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_g = op(*args)
    for it in range(4):
        if it:  # new contents in place: same pointers, different values
            if fp8:  # flip signs: the NaN poison of unaddressed tokens stays where it is
                args[1].view(torch.uint8).bitwise_xor_(0x80)
                args[6].mul_(1.0 + 0.25 * it)
            else:
                args[1].mul_(-0.5)
                args[2].mul_(1.0 + 0.25 * it)
        graph.replay()
        torch.cuda.synchronize()
        eager = op(*args)
        torch.cuda.synchronize()
        assert torch.isfinite(eager).all()
        assert torch.equal(out_g, eager), f"replay {it} differs from the eager call"
        assert torch.equal(eager, eager0) == (it == 0)


@pytest.mark.parametrize("fp8", [False, True])
def test_op_capture_replays_equal_eager_calls(fp8):
    """``op.capture(...)``: the whole call (attention and merge) recorded once in a HIP graph; every replay, with eager work and
    synchronisation in between and new values, lengths and page ids written into the same tensors, equals the eager call."""
    require_gfx950()
    lens = [900, 33, 2048, 5, 1500, 64]
    case = _ragged_case(len(lens), 32, 8, 128, 64, lens, torch.bfloat16, fp8=fp8, seed=19, poison=False)
    dev = [None if t is None else t.to(DEV) for t in case]
    args = dev[:5] if not fp8 else dev
    op = PagedOp(len(lens), 32, 8, case[1].shape[0], 128, 64)
    replay = op.capture(*args)
    for it in range(4):
        if it == 1:
            args[2].mul_(-0.5) if not fp8 else args[6].mul_(1.5)          # new values in place
        if it == 2:
            args[3].copy_(torch.tensor([100, 33, 1024, 0, 1500, 1], dtype=torch.int32))   # shorter sequences, an empty one
        if it == 3:
            args[4][0, :4] = args[4][0, :4].flip(0)                        # other pages for the first 256 tokens of sequence 0
        out_g = replay()
        torch.cuda.synchronize()
        eager = op(*args)
        torch.cuda.synchronize()
        assert torch.isfinite(eager).all()
        assert torch.equal(out_g, eager), f"replay {it} differs from the eager call"


@pytest.mark.parametrize("kernel_key", KERNELS)
@pytest.mark.parametrize("fp8", [False, True])
def test_lengths_are_clamped_to_what_the_block_table_row_addresses(kernel_key, fp8):
    """A corrupt ``real_seqlen_kv`` -- far beyond the table's width, or negative -- must neither run a kernel past the
    sequence's block-table row nor derail its neighbours: an oversized sequence computes exactly what it computes with
    the length its row can address, a negative one what an empty one does (zeros), every other row is untouched, and
    no unaddressed (NaN-filled) token is read.  Past a row lies the next sequence's row (other, valid pages: reading
    them changes the result); past the last row lies the end of the table."""
    require_gfx950()
    page, width = 64, 4
    lens_ok = [100, 0, width * page, 64, width * page]
    case = _ragged_case(len(lens_ok), 32, 8, 128, page, lens_ok, torch.bfloat16, fp8=fp8, seed=23)
    assert case[4].shape[1] == width
    dev = [None if t is None else t.to(DEV) for t in case]
    op = PagedOp(len(lens_ok), 32, 8, case[1].shape[0], 128, page)
    op.kernel_map = {kernel_key: op.kernel_map[kernel_key]}
    args = dev[:5] if not fp8 else dev
    want = op(*args).clone()
    torch.cuda.synchronize()
    assert torch.isfinite(want).all() and (want[1] == 0).all()
    for bad in ([100, -7, 2 ** 31 - 1, 64, width * page + 1], [100, -(2 ** 31), width * page + 1, 64, 10 ** 9]):
        got = op(args[0], args[1], args[2], torch.tensor(bad, dtype=torch.int32, device=DEV), *args[4:])
        torch.cuda.synchronize()
        assert torch.isfinite(got).all()
        assert torch.equal(got, want)


def _random_configs(n, seed):
    """Seeded draw of small shapes over everything the ops accept: head counts and groups, head_dim, page size, query
    tokens, dtype, FP8 cache, softcap, custom scale (also negative), causal or not, ragged lengths with zeros."""
    g = torch.Generator().manual_seed(seed)
    pick = lambda xs: xs[int(torch.randint(len(xs), (1,), generator=g))]  # noqa: E731
    out = []
    for i in range(n):
        heads_kv = pick([1, 2, 4, 8])
        group = pick([1, 2, 3, 4, 5, 8, 16])
        dim = pick([128, 128, 128, 64, 256])
        page = pick([16, 32, 64, 128, 48] if dim != 128 else [16, 32, 64, 128])
        q_len = pick([1, 1, 1, 2, 3, 5, 8, 11])
        batch = pick([1, 2, 3, 7])
        lens = [int(torch.randint(0, 900, (1,), generator=g)) for _ in range(batch)]
        lens = [max(n_, q_len) if n_ > 0 else 0 for n_ in lens]
        out.append(dict(i=i, heads_kv=heads_kv, heads=heads_kv * group, dim=dim, page=page, q_len=q_len, lens=lens,
                        dtype=pick([torch.bfloat16, torch.float16]), fp8=pick([False, False, True]),
                        softcap=pick([0.0, 0.0, 0.0, 5.0, 30.0]), sm_scale=pick([None, None, None, 0.05, -0.11, 0.3]),
                        causal=pick([True, True, False])))
    return out


@pytest.mark.parametrize("cfg", _random_configs(48, seed=2024), ids=lambda c: f"r{c['i']}")
def test_random_shapes_against_the_oracle_on_every_kernel_that_serves_them(cfg):
    require_gfx950()
    c = cfg
    case = _ragged_case(len(c["lens"]), c["heads"], c["heads_kv"], c["dim"], c["page"], c["lens"], c["dtype"], q_len=c["q_len"],
                        fp8=c["fp8"], seed=100 + c["i"])
    n_kv = case[1].shape[0]
    tol = 3e-2 if c["fp8"] else 2e-2
    ran = 0
    for key in KERNELS:
        if c["q_len"] == 1:
            op = PagedOp(len(c["lens"]), c["heads"], c["heads_kv"], n_kv, c["dim"], c["page"], sm_scale=c["sm_scale"], softcap=c["softcap"] or None)
        else:
            op = MultiOp(len(c["lens"]), c["q_len"], c["heads"], c["heads_kv"], n_kv, c["dim"], c["page"], is_causal=c["causal"],
                         sm_scale=c["sm_scale"], softcap=c["softcap"] or None)
        if not _serves(op, key, c["dtype"], c["fp8"]):
            continue
        _force(op, key)
        kw = dict(sm_scale=c["sm_scale"], softcap=c["softcap"])
        if c["q_len"] > 1:
            kw["is_causal"] = c["causal"]
        _run_and_compare(op, case, c["page"], tol, **kw)
        ran += 1
    assert ran >= 1
