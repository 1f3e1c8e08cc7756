"""Index probe through the MFMA attention kernel itself: its page gather pinned bit for bit.

The MFMA kernel does not use the shared ``physical_token()`` routine: it walks the block table with an incremental
cursor (page / in-page offset carried from tile to tile, the table row cached in a register, pool rows advanced by 32
inside a page).  This test reads that arithmetic back out of the attention output.  Every V row holds its own physical
token id (and kv head, and a hash of the column) as small integers that the cache element type represents exactly; one
key per sequence is made dominant by more than 200 in the log2 domain, so every other softmax weight underflows to
exactly 0 and the dominant one is exactly 1.  The output row must then equal ``V[physical(b, pos_b)]`` bit for bit,
where the expected physical row comes from plain torch indexing of ``block_table``
(``k.view(P, page, H_kv, D)[block_table[b, :n]]``, the page reassembly of the reference's ref_program,
tests/ops/attention/test_gqa_decode_paged.py:46-59; its "output-distinguishing page translation" cases :192-232).
The dominant position sweeps page borders, 32-token tile borders, partition borders (tiny calls: every tile is its own
partition; larger ones: partitions of several tiles), the first and the last token, 16-token pages, 16-bit and FP8
caches.  Decoy keys that are even more dominant sit just past each sequence's length and in pages no table names:
reading one of them changes the output.
"""

import math

import pytest
import torch

from tests.conftest import require_gfx950
from tileops_amd.ops import (
    GroupedQueryAttentionDecodePagedWithKVCacheFwdOp as PagedOp,
    GroupedQueryAttentionMultiTokenDecodePagedWithKVCacheFwdOp as MultiOp,
)

pytestmark = pytest.mark.gpu
DEV = "cuda"
FP8 = torch.float8_e4m3fn
MFMA_KEY = "gqa_decode_paged_mfma_kernel"


def _encode_v(n_tok, heads_kv, dim, base):
    """V[t, h, d]: digits of t in the given base at d = 0..3, h at d = 4, a hash of (t, h, d) elsewhere; all in [0, base)."""
    t = torch.arange(n_tok, dtype=torch.int64)[:, None, None]
    h = torch.arange(heads_kv, dtype=torch.int64)[None, :, None]
    d = torch.arange(dim, dtype=torch.int64)[None, None, :]
    v = (t * 31 + h * 17 + d * 7 + (t * d) % 13) % base
    for i in range(4):
        v[:, :, i] = ((t // base ** i) % base)[:, :, 0].expand(n_tok, heads_kv)
    v[:, :, 4] = (h % base)[:, :, 0].expand(n_tok, heads_kv)
    return v.float()


def _probe_case(lens, positions, page, heads, heads_kv, dim, dtype, kv_dtype, seed, q_len=1):
    """Inputs in which token ``positions[b]`` of sequence b is the only key with a non-zero weight."""
    g = torch.Generator().manual_seed(seed)
    batch = len(lens)
    need = [math.ceil(n / page) for n in lens]
    n_pages = sum(need) + 5                                  # five pages that no table names
    perm = torch.randperm(n_pages, generator=g)
    table = torch.full((batch, max(need) + 2), int(perm[-1]), dtype=torch.int32)   # unused entries name an unowned page
    at = 0
    for b, c in enumerate(need):
        table[b, :c] = perm[at:at + c].to(torch.int32)
        at += c
    n_tok = n_pages * page
    fp8 = kv_dtype == FP8
    base = 16 if fp8 else 128                                # integers the cache element type holds exactly
    v = _encode_v(n_tok, heads_kv, dim, base)
    # keys: element 0 decides (the query is non-zero only there), the rest is noise the query never sees
    k = torch.randint(-3, 4, (n_tok, heads_kv, dim), generator=g).float()
    k[:, :, 0] = 32.0                                        # every token nobody addresses is a decoy ...
    expect_rows = []
    for b, n in enumerate(lens):
        pages = table[b, : need[b]].long()
        phys = (pages[:, None] * page + torch.arange(page)[None, :]).reshape(-1)[:n]
        k[phys, :, 0] = 0.0                                  # ... the addressed ones are neutral
        k[phys[positions[b]], :, 0] = 16.0                   # the dominant key of this sequence
        expect_rows.append(int(phys[positions[b]]))
    q = torch.zeros(batch, q_len, heads, dim)
    q[..., 0] = 16.0                                         # score 256 for the dominant key, 0 for the others, 512 for decoys
    q = q.to(dtype)
    if q_len == 1:
        q = q[:, 0]
    ones = torch.ones(n_tok, heads_kv) if fp8 else None
    return (q, k.to(kv_dtype), v.to(kv_dtype), torch.tensor(lens, dtype=torch.int32), table, ones, ones), expect_rows, v


def _run_probe(lens, positions, page, heads, heads_kv, dim, dtype, kv_dtype, seed, q_len=1):
    case, rows, v = _probe_case(lens, positions, page, heads, heads_kv, dim, dtype, kv_dtype, seed, q_len)
    n_kv = case[1].shape[0]
    if q_len == 1:
        op = PagedOp(len(lens), heads, heads_kv, n_kv, dim, page, sm_scale=1.0)
    else:
        op = MultiOp(len(lens), q_len, heads, heads_kv, n_kv, dim, page, sm_scale=1.0, is_causal=True)
    op.kernel_map = {MFMA_KEY: op.kernel_map[MFMA_KEY]}
    args = [t.to(DEV) for t in case if t is not None]
    out = op(*args).cpu()
    group = heads // heads_kv
    for b, row in enumerate(rows):
        want = v[row].to(dtype)                               # [heads_kv, dim]: the encoded ids, exact in the output type
        got = out[b].reshape(q_len, heads_kv, group, dim)
        for s in range(q_len):
            for gi in range(group):
                assert torch.equal(got[s, :, gi].view(torch.int16), want.view(torch.int16)), (
                    f"sequence {b} (len {lens[b]}, dominant token {positions[b]}, query {s}, group member {gi}): expected physical row "
                    f"{row}, output decodes to row {int(sum(int(got[s, 0, gi, i]) * (16 if kv_dtype == FP8 else 128) ** i for i in range(4)))}")


def _sweep_positions(n, page):
    """Borders a cursor can slip on, clipped to the sequence."""
    cand = {0, 1, 15, 16, 17, 31, 32, 33, 63, 64, 65, page - 1, page, page + 1, 2 * page - 1, 2 * page, n // 2, n - 33, n - 32, n - 2, n - 1}
    return sorted(p for p in cand if 0 <= p < n)


@pytest.mark.parametrize("kv_dtype", [torch.bfloat16, torch.float16, FP8], ids=["bf16", "fp16", "fp8"])
@pytest.mark.parametrize("page", [64, 16, 128, 32])
def test_dominant_key_reads_back_its_physical_row_small_calls(kv_dtype, page):
    """Fewer tiles than partitions: every 32-token tile is a partition of its own, so every tile border is also a
    partition border and every sequence of more than one tile goes through the merge."""
    require_gfx950()
    dtype = torch.float16 if kv_dtype == torch.float16 else torch.bfloat16
    lens = [1, 31, 32, 33, 64, 65, 127, 200, 257, 300]
    sweeps = [_sweep_positions(n, page) for n in lens]
    for r in range(max(len(s) for s in sweeps)):
        positions = [s[r % len(s)] for s in sweeps]
        _run_probe(lens, positions, page, 32, 8, 128, dtype, kv_dtype, seed=100 + r)


@pytest.mark.parametrize("kv_dtype", [torch.bfloat16, FP8], ids=["bf16", "fp8"])
@pytest.mark.parametrize("dim, heads, heads_kv", [(128, 32, 8), (64, 16, 4), (256, 16, 4)])
def test_dominant_key_reads_back_its_physical_row_across_multi_tile_partitions(kv_dtype, dim, heads, heads_kv):
    """More tiles than partitions: a partition owns a run of tiles that crosses page and sequence borders, so the
    incremental row cursor (+32 inside a page, table look-up at page and sequence borders) is what is being read back.
    The dominant token sweeps a window of positions around page / tile borders deep inside long sequences."""
    require_gfx950()
    lens = [3000, 4097, 1, 2500, 6000, 777, 5000, 4000, 3500, 2047, 4500, 3100]
    g = torch.Generator().manual_seed(7)
    for r in range(6):
        positions = []
        for n in lens:
            border = int(torch.randint(0, max(n // 32, 1), (1,), generator=g)) * 32   # a tile border somewhere in the sequence
            positions.append(min(max(border + (-1, 0, 1, 31, 32, 63)[r], 0), n - 1))
        _run_probe(lens, positions, 64, heads, heads_kv, dim, torch.bfloat16, kv_dtype, seed=200 + r)


@pytest.mark.parametrize("kv_dtype", [torch.bfloat16, FP8], ids=["bf16", "fp8"])
def test_dominant_key_with_eight_query_tokens_on_shared_stages(kv_dtype):
    """Multi-token queries (64 rows per kv head: two waves around one LDS ring, each fetching half of every stage).  The
    dominant key lies before the chunk, so the causal mask hides it from no query row."""
    require_gfx950()
    lens = [40, 100, 513, 2000, 64, 3000, 1500, 96]
    for r, off in enumerate((0, 31, 32, 63, 64, -1)):
        positions = [min(max((n - 9) // 2 // 32 * 32 + off, 0), n - 9) for n in lens]
        _run_probe(lens, positions, 64, 64, 8, 128, torch.bfloat16, kv_dtype, seed=300 + r, q_len=8)
