"""The decode entry point that allocates nothing (``mi355_gqa_paged_decode_static``) against the workspace entry point.

Called through the C ABI (ctypes, raw pointers): two calls in a row on the library's static scratch, the second with a
smaller input (fewer, shorter sequences), each compared bit for bit with ``mi355_gqa_paged_decode`` on a workspace of the
caller's -- the same kernels run on both, so the results must be identical, and leftovers of the first call in the
scratch must not leak into the second.  Both kernels, 16-bit and FP8 caches, one and four query tokens; a call that
needs more scratch than the library holds is refused with a message.
"""

import pytest
import torch

from tests.conftest import require_gfx950
from tests.test_gqa_decode_paged import _ragged_case
from tileops_amd import native

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _both(case, q_len, kernel):
    q, k, v, lens, table, ks, vs = [None if t is None else t.to(DEV) for t in case]
    batch, heads, dim = q.shape[0], q.shape[-2], q.shape[-1]
    heads_kv, page = k.shape[1], 64
    kw = dict(batch=batch, q_len=q_len, heads=heads, heads_kv=heads_kv, dim=dim, page_size=page, sm_scale=dim ** -0.5, softcap=0.0,
              causal=True)
    nbytes, nsplit, _ = native.decode_workspace(batch, q_len, heads, heads_kv, dim, page, table.shape[1], q.dtype, k.dtype, 0, kernel)
    ws = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=DEV)
    want = torch.full_like(q, float("nan"))
    native.paged_decode(q, k, v, ks, vs, lens, table, want, ws, num_split=nsplit, kernel=kernel, **kw)
    got = torch.full_like(q, float("nan"))
    before = torch.cuda.memory_allocated()
    native.paged_decode_static(q, k, v, ks, vs, lens, table, got, num_split=nsplit, kernel=kernel, **kw)
    assert torch.cuda.memory_allocated() == before           # (torch's allocator at least was not asked for anything)
    torch.cuda.synchronize()
    assert torch.isfinite(got).all()
    assert torch.equal(got, want)


@pytest.mark.parametrize("kernel", [native.KERNEL_MFMA, native.KERNEL_GENERIC], ids=["mfma", "generic"])
@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("q_len", [1, 4])
def test_static_scratch_entry_point_equals_the_workspace_entry_point_twice_in_a_row(kernel, fp8, q_len):
    require_gfx950()
    big = [3000, 33, 2048, 700, 1500, 64, 4096, 1]           # sequences spread over many partitions / splits
    small = [130, 64, 9]                                     # then fewer and shorter ones on the same scratch
    for lens, seed in ((big, 41), (small, 42)):
        _both(_ragged_case(len(lens), 32, 8, 128, 64, lens, torch.bfloat16, q_len=q_len, fp8=fp8, seed=seed), q_len, kernel)


def test_static_scratch_entry_point_refuses_what_does_not_fit():
    """The general kernel's plan grows with batch x splits; 256 sequences x 64 splits need 270 MB.  The call is refused from
    its shape alone, before anything is launched (the tensors below are far smaller than the shape claims)."""
    require_gfx950()
    batch, width = 256, 512
    need = native.decode_workspace(batch, 1, 32, 8, 128, 64, width, torch.bfloat16, torch.bfloat16, 0, native.KERNEL_GENERIC)[0]
    assert need > 80 << 20
    q = torch.zeros(batch, 32, 128, dtype=torch.bfloat16, device=DEV)
    k = torch.zeros(64, 8, 128, dtype=torch.bfloat16, device=DEV)
    lens = torch.zeros(batch, dtype=torch.int32, device=DEV)
    table = torch.zeros(batch, width, dtype=torch.int32, device=DEV)
    with pytest.raises(native.NativeLibraryError, match=f"needs {need} bytes of scratch, the static buffer of mi355_gqa_paged_decode_static holds {80 << 20}"):
        native.paged_decode_static(q, k, k, None, None, lens, table, torch.empty_like(q), batch=batch, q_len=1, heads=32, heads_kv=8, dim=128,
                                   page_size=64, sm_scale=1.0, softcap=0.0, causal=True, kernel=native.KERNEL_GENERIC)
    # every plan of the MFMA kernel fits, the largest included (64 query rows per kv head)
    assert native.decode_workspace(32, 8, 64, 8, 128, 64, 256, torch.bfloat16, torch.float8_e4m3fn, 0, native.KERNEL_MFMA)[0] < 80 << 20


@pytest.mark.parametrize("fp8", [False, True])
def test_static_scratch_entry_point_captured_in_a_graph_and_replayed_on_changed_inputs(fp8):
    """What the entry point is for: a caller under HIP graph capture.  One warm-up call outside the capture (the first call
    on a device asks for the scratch's address and sets the kernels' LDS limit, which is not stream work), then the call is
    captured and replayed three times, each time after the cache contents, the lengths and the block table have been
    changed in place; every replay must equal an eager call of the workspace entry point on the same inputs bit for bit."""
    require_gfx950()
    lens0 = [3000, 33, 2048, 700, 1500, 64, 4096, 1]
    q, k, v, lens, table, ks, vs = [None if t is None else t.to(DEV) for t in
                                    _ragged_case(len(lens0), 32, 8, 128, 64, lens0, torch.bfloat16, q_len=1, fp8=fp8, seed=51, poison=False)]
    batch, heads, dim, heads_kv, page = q.shape[0], q.shape[-2], q.shape[-1], k.shape[1], 64
    kw = dict(batch=batch, q_len=1, heads=heads, heads_kv=heads_kv, dim=dim, page_size=page, sm_scale=dim ** -0.5, softcap=0.0, causal=True)
    nbytes, nsplit, _ = native.decode_workspace(batch, 1, heads, heads_kv, dim, page, table.shape[1], q.dtype, k.dtype, 0, native.KERNEL_MFMA)
    ws = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=DEV)
    got = torch.full_like(q, float("nan"))
    native.paged_decode_static(q, k, v, ks, vs, lens, table, got, num_split=nsplit, kernel=native.KERNEL_MFMA, **kw)  # warm-up
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        native.paged_decode_static(q, k, v, ks, vs, lens, table, got, num_split=nsplit, kernel=native.KERNEL_MFMA, **kw)
    gen = torch.Generator(device="cpu").manual_seed(52)
    for step in range(3):
        # new cache bytes (a rotation of the pool keeps every value a legal element), shorter or longer sequences, other pages
        k.view(torch.uint8).copy_(torch.roll(k.view(torch.uint8), 1 + step, 0))
        v.view(torch.uint8).copy_(torch.roll(v.view(torch.uint8), 2 + step, 0))
        new_lens = torch.tensor([max(1, n // (step + 1)) for n in lens0], dtype=torch.int32)
        lens.copy_(new_lens.to(DEV))
        table.copy_(table[torch.randperm(batch, generator=gen).to(DEV)])
        q.copy_(torch.randn(q.shape, generator=gen).to(q.dtype).to(DEV))
        want = torch.full_like(q, float("nan"))
        native.paged_decode(q, k, v, ks, vs, lens, table, want, ws, num_split=nsplit, kernel=native.KERNEL_MFMA, **kw)
        got.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.isfinite(got).all()
        assert torch.equal(got, want), f"replay {step}"
