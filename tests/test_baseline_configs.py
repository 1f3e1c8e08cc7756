"""BASELINE configurations 2-5 at their full sizes on the GPU, plus configuration 1 (CPU plumbing).

At full size the CPU oracle is run on a sample of sequences (their pages are gathered into a compact host pool
with torch indexing, which does not involve the kernels under test); the rest of the batch is covered by
size-independent properties: the two HIP kernels agree with each other, a joint permutation of physical pages and
block table changes no bit, and NaN written into every unaddressed page changes no bit.
"""

import math

import pytest
import torch

from oracle.paged_gqa_decode_ref import ref_gqa_decode_contiguous, ref_paged_gqa_decode
from tests.conftest import require_gfx950
from tileops_amd import ops
from tileops_amd.workloads import BASELINE_CONFIGS, contiguous_as_paged, gen_contiguous_inputs, gen_paged_inputs

FP8 = torch.float8_e4m3fn


def _make_op(cfg, key=None):
    if cfg.q_len == 1:
        op = ops.GroupedQueryAttentionDecodePagedWithKVCacheFwdOp(cfg.batch, cfg.heads, cfg.heads_kv, cfg.seqlen_kv, cfg.dim, cfg.page_size)
    else:
        op = ops.GroupedQueryAttentionMultiTokenDecodePagedWithKVCacheFwdOp(cfg.batch, cfg.q_len, cfg.heads, cfg.heads_kv, cfg.seqlen_kv,
                                                                            cfg.dim, cfg.page_size)
    if key:
        op.kernel_map = {key: op.kernel_map[key]}
    return op


def _host_subproblem(inp, cfg, seq_ids):
    """Compact CPU copy of the sequences *seq_ids*: their pages renumbered 0..n-1 in a small pool."""
    lens = inp.real_seqlen_kv[seq_ids].cpu()
    rows, tables = [], []
    at = 0
    for i, b in enumerate(seq_ids):
        n_pages = math.ceil(int(lens[i]) / cfg.page_size)
        rows.append(inp.block_table[b, :n_pages].long())
        t = torch.zeros(cfg.table_width, dtype=torch.int32)
        t[:n_pages] = torch.arange(at, at + n_pages, dtype=torch.int32)
        tables.append(t)
        at += n_pages
    pages = torch.cat(rows)
    idx = (pages[:, None] * cfg.page_size + torch.arange(cfg.page_size, device=pages.device)[None, :]).reshape(-1)
    take = lambda t: None if t is None else t.index_select(0, idx).cpu()  # noqa: E731
    return inp.q[seq_ids].cpu(), take(inp.k), take(inp.v), lens, torch.stack(tables), take(inp.k_scale), take(inp.v_scale)


def test_config1_cpu_plumbing():
    """Config 1: batch 1, 32/8 heads, D 128, one query token, 1024 contiguous tokens, fp32, seed 0 -- oracle only."""
    q, k, v = gen_contiguous_inputs(seed=0)
    out = ref_gqa_decode_contiguous(q, k, v, sm_scale=128 ** -0.5)
    assert out.shape == (1, 32, 128) and out.dtype == torch.float32 and torch.isfinite(out).all()
    p = contiguous_as_paged(q, k, v, 64)
    torch.testing.assert_close(ref_paged_gqa_decode(p.q, p.k, p.v, p.real_seqlen_kv, p.block_table, page_size=64), out, rtol=1e-6, atol=1e-7)
    # softmax weights sum to one: attention over constant V returns that constant
    ones = ref_gqa_decode_contiguous(q, k, torch.full_like(v, 0.5))
    torch.testing.assert_close(ones, torch.full_like(ones, 0.5))


@pytest.mark.gpu
def test_config1_on_device_matches_cpu_reference():
    require_gfx950()
    q, k, v = gen_contiguous_inputs(seed=0)
    want = ref_gqa_decode_contiguous(q.bfloat16(), k.bfloat16(), v.bfloat16())
    p = contiguous_as_paged(q.bfloat16(), k.bfloat16(), v.bfloat16(), 64).to("cuda")
    op = ops.GroupedQueryAttentionDecodePagedWithKVCacheFwdOp(1, 32, 8, 1024, 128, 64)
    torch.testing.assert_close(op(*p.as_args()).float().cpu(), want.float(), atol=2e-2, rtol=2e-2)


@pytest.mark.gpu
@pytest.mark.parametrize("name, n_check", [("c2", 8), ("c3", 8), ("c4", 8), ("c5", 4)])
def test_full_size_configuration(name, n_check):
    require_gfx950()
    cfg = BASELINE_CONFIGS[name]
    fp8 = cfg.kv_dtype == FP8
    tol = 3e-2 if fp8 else 2e-2
    inp = gen_paged_inputs(cfg, "cuda")
    op = _make_op(cfg)
    out = op(*inp.as_args())
    torch.cuda.synchronize()
    assert out.shape == inp.q.shape and out.dtype == torch.bfloat16 and torch.isfinite(out).all()
    kernel = next(iter(next(iter(op._kernel_roles.values())).values()))
    assert type(kernel).__name__ == "GQADecodePagedMfmaKernel"

    # (1) oracle on a sample: the longest, the shortest and evenly spaced sequences
    lens = inp.real_seqlen_kv.cpu()
    order = torch.argsort(lens)
    picks = sorted({int(order[0]), int(order[-1]), *[int(order[i]) for i in torch.linspace(0, cfg.batch - 1, n_check).long()]})[:max(n_check, 2)]
    # (c4: all eight sequences, one at a time -- a dequantised 131072-token sequence is a gigabyte on the host)
    for group in ([[b] for b in range(cfg.batch)] if name == "c4" else [picks]):
        q, k, v, l, t, ks, vs = _host_subproblem(inp, cfg, group)
        ref = ref_paged_gqa_decode(q, k, v, l, t, page_size=cfg.page_size, k_scale=ks, v_scale=vs)
        torch.testing.assert_close(out[group].float().cpu(), ref.float(), atol=tol, rtol=tol)

    # (2) the general kernel gives the same answer for the whole batch
    out_gen = _make_op(cfg, "gqa_decode_paged_kernel")(*inp.as_args())
    torch.testing.assert_close(out.float(), out_gen.float(), atol=tol, rtol=tol)

    # (3) NaN in every page no sequence owns changes no bit
    used = torch.zeros(cfg.n_pages, dtype=torch.bool, device="cuda")
    pages_per = (inp.real_seqlen_kv.long() + cfg.page_size - 1) // cfg.page_size
    for b in range(cfg.batch):
        used[inp.block_table[b, : int(pages_per[b])].long()] = True
    if (~used).any():
        free_tok = (~used).repeat_interleave(cfg.page_size)
        if fp8:
            inp.k.view(torch.uint8)[free_tok] = 0x7F
            inp.v.view(torch.uint8)[free_tok] = 0x7F
            inp.k_scale[free_tok] = float("nan")
            inp.v_scale[free_tok] = float("nan")
        else:
            inp.k[free_tok] = float("nan")
            inp.v[free_tok] = float("nan")
        assert torch.equal(op(*inp.as_args()), out)

    # (4) reversing each sequence's physical placement (pool mirrored, table renamed) changes no bit
    P = cfg.n_pages
    mirror = lambda x: x.view(P, cfg.page_size, *x.shape[1:]).flip(0).reshape(x.shape)  # noqa: E731
    inp.k, inp.v = mirror(inp.k), mirror(inp.v)
    if fp8:
        inp.k_scale, inp.v_scale = mirror(inp.k_scale), mirror(inp.v_scale)
    inp.block_table = (P - 1 - inp.block_table).to(torch.int32)
    assert torch.equal(op(*inp.as_args()), out)
