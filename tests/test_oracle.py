"""Pins the CPU oracle (oracle/paged_gqa_decode_ref.py) without the reference being importable.

Each check is chosen so that a plausible slip -- a dropped scale, a wrong page index, a transposed operand,
a top-left instead of bottom-right causal mask, a missing softcap -- fails at least one of them:
library routine (torch SDPA), float64 brute force with scalar page arithmetic, closed forms, invariances,
and the reference's own known answers (tile rule, roofline formula).
"""

import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle.paged_gqa_decode_ref import (
    brute_force_f64, combine_partials, dequantize_kv, gather_pages, physical_pos, quantize_kv_per_token,
    ref_gqa_decode_contiguous, ref_paged_gqa_decode, ref_paged_gqa_decode_sdpa_math, reference_block_ns, reference_roofline,
)
from tileops_amd.workloads import contiguous_as_paged, gen_contiguous_inputs


def _case(B, H, H_kv, D, page, lens, n_pages=None, seed=0, q_len=1, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    need = sum(math.ceil(n / page) for n in lens)
    n_pages = n_pages or need + 2
    q_shape = (B, H, D) if q_len == 1 else (B, q_len, H, D)
    q = torch.randn(q_shape, generator=g).to(dtype)
    k = torch.randn(n_pages * page, H_kv, D, generator=g).to(dtype)
    v = torch.randn(n_pages * page, H_kv, D, generator=g).to(dtype)
    perm = torch.randperm(n_pages, generator=g)
    width = max(1, max(math.ceil(n / page) for n in lens))
    table = torch.zeros(B, width, dtype=torch.int32)
    at = 0
    for b, n in enumerate(lens):
        c = math.ceil(n / page)
        table[b, :c] = perm[at:at + c].to(torch.int32)
        at += c
    return q, k, v, torch.tensor(lens, dtype=torch.int32), table


# --- page gather ----------------------------------------------------------------------------------------
def test_gather_matches_view_indexing_and_scalar_page_arithmetic():
    q, k, v, lens, table = _case(3, 4, 2, 8, 16, [40, 16, 1], seed=3)
    for b in range(3):
        n = int(lens[b])
        got = gather_pages(k, table[b], n, 16)
        # k.view(P, page, H_kv, D)[block_table[b, :n_pages]] -- pure indexing
        want = k.view(-1, 16, 2, 8)[table[b, : math.ceil(n / 16)].long()].reshape(-1, 2, 8)[:n]
        assert torch.equal(got, want)
        for t in (0, n // 2, n - 1):
            assert torch.equal(got[t], k[physical_pos(table, b, t, 16)])


def test_gather_is_invariant_under_joint_page_permutation():
    q, k, v, lens, table = _case(2, 4, 2, 8, 8, [30, 17], seed=5)
    n_pages = k.shape[0] // 8
    sigma = torch.randperm(n_pages, generator=torch.Generator().manual_seed(9))
    k2 = torch.empty_like(k)
    k2.view(n_pages, 8, 2, 8)[sigma] = k.view(n_pages, 8, 2, 8)  # page p moves to sigma[p]
    table2 = sigma[table.long()].to(torch.int32)
    for b in range(2):
        assert torch.equal(gather_pages(k, table[b], int(lens[b]), 8), gather_pages(k2, table2[b], int(lens[b]), 8))


# --- attention math ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("softcap", [0.0, 2.0])
@pytest.mark.parametrize("sm_scale", [None, 0.25])
def test_matches_float64_brute_force(softcap, sm_scale):
    q, k, v, lens, table = _case(2, 6, 2, 16, 4, [13, 5], seed=11)
    scale = 16 ** -0.5 if sm_scale is None else sm_scale
    got = ref_paged_gqa_decode(q, k, v, lens, table, page_size=4, sm_scale=sm_scale, softcap=softcap)
    want = brute_force_f64(q.numpy(), k.numpy(), v.numpy(), lens.numpy(), table.numpy(), 4, scale, softcap)
    np.testing.assert_allclose(got.numpy(), want, rtol=2e-5, atol=2e-6)


def test_matches_torch_sdpa_library_routine():
    # the reference benchmark's own baseline is F.scaled_dot_product_attention on the gathered, head-expanded
    # K/V (benchmarks/ops/attention/bench_gqa_decode_paged.py:62-63)
    q, k, v, lens, table = _case(3, 8, 2, 32, 8, [64, 23, 1], seed=2)
    got = ref_paged_gqa_decode(q, k, v, lens, table, page_size=8)
    for b in range(3):
        n = int(lens[b])
        kb = gather_pages(k, table[b], n, 8).repeat_interleave(4, dim=1).transpose(0, 1)  # [H, n, D]
        vb = gather_pages(v, table[b], n, 8).repeat_interleave(4, dim=1).transpose(0, 1)
        want = F.scaled_dot_product_attention(q[b][:, None, :], kb, vb)[:, 0]
        torch.testing.assert_close(got[b], want, rtol=2e-5, atol=2e-6)


@pytest.mark.parametrize("q_len", [1, 5])
def test_sdpa_math_baseline_is_the_same_function_as_the_oracle(q_len):
    """The reference benchmark's torch baseline (bench_gqa_decode_paged.py:21-66: reassemble pages, expand heads by index,
    SDPA under the MATH backend) against the einsum oracle: ragged lengths, an empty sequence, FP8 with scales, and the
    bottom-right causal mask for several query tokens."""
    lens = [0 if q_len == 1 else q_len, 70, 129, 33]
    q, k, v, lens_t, table = _case(4, 8, 2, 64, 32, lens, seed=5, q_len=q_len)
    a = ref_paged_gqa_decode(q, k, v, lens_t, table, page_size=32)
    b = ref_paged_gqa_decode_sdpa_math(q, k, v, lens_t, table, page_size=32)
    torch.testing.assert_close(a, b, atol=2e-6, rtol=1e-5)
    k8, ks = quantize_kv_per_token(k)
    v8, vs = quantize_kv_per_token(v)
    a = ref_paged_gqa_decode(q.bfloat16(), k8, v8, lens_t, table, page_size=32, k_scale=ks, v_scale=vs)
    b = ref_paged_gqa_decode_sdpa_math(q.bfloat16(), k8, v8, lens_t, table, page_size=32, k_scale=ks, v_scale=vs)
    torch.testing.assert_close(a.float(), b.float(), atol=1e-2, rtol=1e-2)  # both round an fp32 result to bf16


def test_contiguous_reference_config1_and_identity_paging_agree():
    # BASELINE config 1: batch 1, 32/8 heads, D 128, 1024 contiguous tokens, fp32, seed 0
    q, k, v = gen_contiguous_inputs(seed=0)
    want = ref_gqa_decode_contiguous(q, k, v)
    kb = k[0].repeat_interleave(4, dim=1).transpose(0, 1)
    vb = v[0].repeat_interleave(4, dim=1).transpose(0, 1)
    sdpa = F.scaled_dot_product_attention(q[0][:, None, :], kb, vb)[:, 0]
    torch.testing.assert_close(want[0], sdpa, rtol=2e-5, atol=2e-6)
    p = contiguous_as_paged(q, k, v, 64)
    got = ref_paged_gqa_decode(p.q, p.k, p.v, p.real_seqlen_kv, p.block_table, page_size=64)
    torch.testing.assert_close(got, want, rtol=1e-6, atol=1e-7)


def test_closed_form_zero_query_gives_mean_of_values():
    q, k, v, lens, table = _case(2, 4, 2, 8, 4, [10, 3], seed=1)
    out = ref_paged_gqa_decode(torch.zeros_like(q), k, v, lens, table, page_size=4)
    for b in range(2):
        mean_v = gather_pages(v, table[b], int(lens[b]), 4).mean(dim=0)  # [H_kv, D]
        torch.testing.assert_close(out[b], mean_v.repeat_interleave(2, dim=0), rtol=1e-5, atol=1e-6)


def test_closed_form_single_token_returns_that_value_row():
    q, k, v, lens, table = _case(2, 4, 2, 8, 4, [1, 1], seed=4)
    out = ref_paged_gqa_decode(q, k, v, lens, table, page_size=4)
    for b in range(2):
        row = v[int(table[b, 0]) * 4]
        torch.testing.assert_close(out[b], row.repeat_interleave(2, dim=0))


def test_dominant_key_selects_its_value_row_through_the_block_table():
    q, k, v, lens, table = _case(1, 2, 1, 8, 4, [11], seed=6)
    t_star = 9  # lives in logical page 2, slot 1
    phys = physical_pos(table, 0, t_star, 4)
    k = k.clone()
    k[phys, 0] = 50.0 * q[0, 0] / q[0, 0].norm()
    out = ref_paged_gqa_decode(q, k, v, lens, table, page_size=4, sm_scale=1.0)
    torch.testing.assert_close(out[0, 0], v[phys, 0], rtol=1e-4, atol=1e-4)


def test_heads_of_a_group_with_equal_queries_agree_and_softcap_limit():
    q, k, v, lens, table = _case(1, 4, 2, 8, 4, [9], seed=8)
    q[:, 1] = q[:, 0]
    out = ref_paged_gqa_decode(q, k, v, lens, table, page_size=4)
    assert torch.equal(out[0, 0], out[0, 1])           # heads 0,1 share kv head 0
    assert not torch.allclose(out[0, 0], out[0, 2])    # head 2 reads kv head 1
    capped = ref_paged_gqa_decode(q, k, v, lens, table, page_size=4, softcap=1e6)
    torch.testing.assert_close(capped, out, rtol=1e-4, atol=1e-5)  # softcap -> inf is no softcap
    strong = ref_paged_gqa_decode(q, k, v, lens, table, page_size=4, softcap=0.5)
    assert not torch.allclose(strong, out, atol=1e-3)


def test_unaddressed_tokens_do_not_matter():
    q, k, v, lens, table = _case(2, 4, 2, 8, 4, [10, 3], n_pages=9, seed=12)
    base = ref_paged_gqa_decode(q, k, v, lens, table, page_size=4)
    used = torch.zeros(k.shape[0], dtype=torch.bool)
    for b in range(2):
        for t in range(int(lens[b])):
            used[physical_pos(table, b, t, 4)] = True
    k2, v2 = k.clone(), v.clone()
    k2[~used] = float("nan")
    v2[~used] = float("inf")
    assert torch.equal(ref_paged_gqa_decode(q, k2, v2, lens, table, page_size=4), base)


# --- causal chunk -----------------------------------------------------------------------------------------
def test_causal_chunk_is_bottom_right_and_reduces_to_single_token_decodes():
    S_q = 3
    q, k, v, lens, table = _case(2, 4, 2, 8, 4, [10, 5], seed=13, q_len=S_q)
    out = ref_paged_gqa_decode(q, k, v, lens, table, page_size=4, is_causal=True)
    for i in range(S_q):
        lens_i = lens - S_q + i + 1
        single = ref_paged_gqa_decode(q[:, i], k, v, lens_i, table, page_size=4)
        torch.testing.assert_close(out[:, i], single, rtol=1e-6, atol=1e-7)
    full = ref_paged_gqa_decode(q, k, v, lens, table, page_size=4, is_causal=False)
    torch.testing.assert_close(full[:, -1], out[:, -1])
    assert not torch.allclose(full[:, 0], out[:, 0])
    want = brute_force_f64(q.numpy(), k.numpy(), v.numpy(), lens.numpy(), table.numpy(), 4, 8 ** -0.5, 0.0, True)
    np.testing.assert_allclose(out.numpy(), want, rtol=2e-5, atol=2e-6)


def test_rows_with_no_visible_key_are_zero():
    q, k, v, lens, table = _case(1, 2, 1, 8, 4, [2], seed=14, q_len=4)  # len < S_q: queries 0,1 see nothing
    out = ref_paged_gqa_decode(q, k, v, lens, table, page_size=4)
    assert torch.equal(out[0, :2], torch.zeros(2, 2, 8))
    assert torch.isfinite(out).all()
    empty = ref_paged_gqa_decode(q[:, 0], k, v, torch.tensor([0], dtype=torch.int32), table, page_size=4)
    assert torch.equal(empty, torch.zeros(1, 2, 8))


# --- FP8 dequant convention ---------------------------------------------------------------------------------
def test_fp8_kv_equals_attention_on_dequantized_cache():
    q, k, v, lens, table = _case(2, 4, 2, 16, 4, [9, 6], seed=15)
    k8, ks = quantize_kv_per_token(k)
    v8, vs = quantize_kv_per_token(v)
    got = ref_paged_gqa_decode(q, k8, v8, lens, table, page_size=4, k_scale=ks, v_scale=vs)
    want = ref_paged_gqa_decode(q, dequantize_kv(k8, ks), dequantize_kv(v8, vs), lens, table, page_size=4)
    torch.testing.assert_close(got, want, rtol=1e-6, atol=1e-7)
    exact = ref_paged_gqa_decode(q, k, v, lens, table, page_size=4)
    assert (got - exact).abs().max() < 0.15  # quantisation error is visible but bounded


# --- split / combine -----------------------------------------------------------------------------------------
@pytest.mark.parametrize("cuts", [[0, 13], [0, 4, 13], [0, 1, 2, 12, 13], [0, 13, 13]])
def test_combine_of_normalised_partials_reproduces_the_whole(cuts):
    # gqa_decode_paged.py:327-374: partial = softmax-weighted V over a slice, lse2 = log2 sum exp2(logit2)
    g = torch.Generator().manual_seed(16)
    s = torch.randn(3, 13, generator=g) * 3  # logits (natural log domain) for 3 rows
    v = torch.randn(13, 8, generator=g)
    whole = torch.softmax(s, dim=-1) @ v
    parts, lses = [], []
    for a, b in zip(cuts[:-1], cuts[1:]):
        if a == b:
            parts.append(torch.zeros(3, 8))
            lses.append(torch.full((3,), float("-inf")))
            continue
        sl = s[:, a:b]
        parts.append(torch.softmax(sl, dim=-1) @ v[a:b])
        lses.append(torch.logsumexp(sl, dim=-1) * math.log2(math.e))
    got = combine_partials(torch.stack(parts, dim=1), torch.stack(lses, dim=1))
    torch.testing.assert_close(got, whole, rtol=1e-5, atol=1e-6)


# --- known answers the reference's tests hold ---------------------------------------------------------------
def test_tile_rule_known_answers():
    # tests/ops/attention/test_gqa_decode_paged.py:122-151
    assert reference_block_ns(192) == (64,)
    assert reference_block_ns(64) == (64,)
    assert reference_block_ns(128) == (128, 64)
    assert reference_block_ns(256) == (128, 64)
    assert reference_block_ns(16) == (16,)
    for page in (96, 160, 224):
        with pytest.raises(ValueError, match="matches no supported block_N"):
            reference_block_ns(page)
    with pytest.raises(ValueError, match="page_size must be positive"):
        reference_block_ns(0)


def test_reference_roofline_formula_by_hand():
    # src/tileops/perf/formulas.py:703-711 evaluated by hand for manifest rows (fp16 = 2 bytes)
    # serving-8b-p64: q [32,32,128], kv [4096,8,128]
    flops, nbytes = reference_roofline(32, 32, 8, 4096, 128, 64, 2)
    assert flops == 4 * 32 * 32 * 4096 * 128 == 2147483648
    assert nbytes == (2 * 32 * 32 * 128 + 2 * 4096 * 8 * 128) * 2 + 32 * 4 + 32 * 64 * 4 == 17309824
    # serving-405b-p256: q [4,128,128], kv [4096,8,128], page 256
    flops, nbytes = reference_roofline(4, 128, 8, 4096, 128, 256, 2)
    assert flops == 1073741824
    assert nbytes == (2 * 4 * 128 * 128 + 2 * 4096 * 8 * 128) * 2 + 4 * 4 + 4 * 16 * 4 == 17039632
