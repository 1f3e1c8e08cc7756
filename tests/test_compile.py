"""The ops under ``torch.compile(fullgraph=True)``: one registered operator per call, no graph break.

Mirrors the reference's compile contract (tests/compile_contract.py, tests/test_compile.py): an op class names the
``torch.library`` operators it traces to in ``compile_op_names``; compiling the op cold with ``fullgraph=True`` must
yield a graph whose only calls are those operators; the compiled op's output equals the eager op's.  The CPU tests trace
with a backend that records the graph and never runs it (the kernels need a gfx950 GPU); the GPU tests run it.
"""
import operator

import pytest
import torch

import tileops_amd  # noqa: F401 - registers torch.ops.tileops_amd.*
from tileops_amd import custom_ops, kernels, native, ops
from tileops_amd.workloads import BASELINE_CONFIGS, gen_paged_inputs


def operator_overload(name: str):
    namespace, _, opname = name.partition("::")
    return getattr(getattr(torch.ops, namespace), opname).default


def _names(calls) -> set:
    """Qualified operator names of graph call targets (an overload packet or one of its overloads)."""
    return {getattr(c, "_qualified_op_name", None) or (c.name() if hasattr(c, "name") else f"{c.__module__}.{c.__qualname__}") for c in calls}


def traced_call_targets(op, *inputs, run=None):
    """Compile *op* with ``fullgraph=True`` and return the operators its graph calls (``operator.getitem`` left out)."""
    traced = []

    def capture(gm, example_inputs):
        traced.append([n.target for n in gm.graph.nodes if n.op == "call_function" and n.target is not operator.getitem])
        if run is not None:
            return run  # stands in for the graph on a machine that cannot run the kernels
        return gm.forward

    torch.compile(op, backend=capture, fullgraph=True)(*inputs)
    (calls,) = traced
    return set(calls)


@pytest.fixture
def pretend_gfx950(monkeypatch):
    """Kernel selection asks the device architecture; on a machine without a GPU answer "gfx950" so that tracing reaches
    the operator call (which the recording backend never executes)."""
    kernels.get_arch.cache_clear()
    monkeypatch.setattr(kernels, "get_arch", lambda index=None: kernels.GFX950_ARCH)
    monkeypatch.setattr(ops, "get_arch", lambda index=None: kernels.GFX950_ARCH)
    monkeypatch.setattr(native, "is_gfx950", lambda device: True)
    yield


def test_operators_are_registered_with_fake_implementations():
    for name in custom_ops.OP_NAMES:
        overload = operator_overload(name)
        assert overload._schema.name == name
    schema = str(torch.ops.tileops_amd.gqa_prefill_paged.default._schema)
    assert "Tensor(a3!) k_pages" in schema and "Tensor(a4!) v_pages" in schema  # the appended pools are declared mutated
    assert "!" not in str(torch.ops.tileops_amd.gqa_paged_decode.default._schema)


def test_fake_implementations_state_shape_and_dtype_only():
    from torch._subclasses.fake_tensor import FakeTensorMode

    with FakeTensorMode():
        q = torch.empty(4, 8, 32, 128, dtype=torch.bfloat16, device="cuda")
        k = torch.empty(4096, 8, 128, dtype=torch.float8_e4m3fn, device="cuda")
        ks = torch.empty(4096, 8, dtype=torch.float32, device="cuda")
        lens = torch.empty(4, dtype=torch.int32, device="cuda")
        bt = torch.empty(4, 16, dtype=torch.int32, device="cuda")
        out = torch.ops.tileops_amd.gqa_paged_decode(q, k, k, lens, bt, ks, ks, 8, 32, 8, 128, 64, 0.1, 0.0, True, 0, 0)
        assert out.shape == q.shape and out.dtype == q.dtype and out.device == q.device
        qd = torch.empty(4, 32, 128, dtype=torch.float16, device="cuda")
        kd = torch.empty(4, 512, 8, 128, dtype=torch.float16, device="cuda")
        out = torch.ops.tileops_amd.gqa_decode(qd, kd, kd, None, None, 512, 32, 8, 128, 0.1, 0.0, True, 0, 0)
        assert out.shape == qd.shape and out.dtype == qd.dtype


def _decode_case(q_len, dtype=torch.float16):
    B, H, HKV, D, P, N = 4, 32, 8, 128, 64, 4096
    if q_len == 1:
        op = ops.GroupedQueryAttentionDecodePagedWithKVCacheFwdOp(B, H, HKV, N, D, P)
        q = torch.randn(B, H, D).to(dtype)
    else:
        op = ops.GroupedQueryAttentionMultiTokenDecodePagedWithKVCacheFwdOp(B, q_len, H, HKV, N, D, P)
        q = torch.randn(B, q_len, H, D).to(dtype)
    k, v = torch.randn(N, HKV, D).to(dtype), torch.randn(N, HKV, D).to(dtype)
    lens = torch.full((B,), 100, dtype=torch.int32)
    bt = torch.arange(B * 8, dtype=torch.int32).reshape(B, 8)
    return op, (q, k, v, lens, bt)


@pytest.mark.parametrize("q_len", [1, 8])
def test_paged_decode_ops_trace_cold_to_one_operator(pretend_gfx950, q_len):
    op, inputs = _decode_case(q_len)
    assert type(op).compile_op_names == ("tileops_amd::gqa_paged_decode",)
    calls = traced_call_targets(op, *inputs, run=lambda *a: (torch.zeros_like(inputs[0]),))
    assert _names(calls) == {"tileops_amd::gqa_paged_decode"}


def test_contiguous_decode_op_traces_cold_to_one_operator(pretend_gfx950):
    B, H, HKV, D, N = 2, 32, 8, 128, 512
    op = ops.GroupedQueryAttentionDecodeWithKVCacheFwdOp(B, H, HKV, N, D)
    q = torch.randn(B, H, D).half()
    k, v = torch.randn(B, N, HKV, D).half(), torch.randn(B, N, HKV, D).half()
    calls = traced_call_targets(op, q, k, v, run=lambda *a: (torch.zeros_like(q),))
    assert _names(calls) == {"tileops_amd::gqa_decode"}


def _on_gpu():
    return torch.cuda.is_available() and native.is_gfx950(torch.device("cuda", 0))


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["c2", "c3", "c5"])
def test_compiled_paged_decode_equals_eager(name):
    if not _on_gpu():
        pytest.skip("needs a gfx950 GPU")
    device = torch.device("cuda", 0)
    cfg = BASELINE_CONFIGS[name].scaled(batch=4, n_pages=128, len_range=(100, 1500))
    inp = gen_paged_inputs(cfg, device)
    if cfg.q_len == 1:
        op = ops.GroupedQueryAttentionDecodePagedWithKVCacheFwdOp(cfg.batch, cfg.heads, cfg.heads_kv, cfg.seqlen_kv, cfg.dim, cfg.page_size)
    else:
        op = ops.GroupedQueryAttentionMultiTokenDecodePagedWithKVCacheFwdOp(cfg.batch, cfg.q_len, cfg.heads, cfg.heads_kv, cfg.seqlen_kv,
                                                                            cfg.dim, cfg.page_size)
    args = inp.as_args()
    calls = traced_call_targets(op, *args)  # cold: the first call of this op instance is the compiled one
    assert _names(calls) == {"tileops_amd::gqa_paged_decode"}
    torch._dynamo.reset()
    compiled = torch.compile(op, fullgraph=True, backend="aot_eager")
    got = compiled(*args)
    want = op(*args)
    torch.cuda.synchronize()
    assert torch.equal(got, want)  # same kernels on the same inputs: bit for bit


@pytest.mark.gpu
def test_compiled_prefill_appends_to_the_pages_like_eager():
    if not _on_gpu():
        pytest.skip("needs a gfx950 GPU")
    device = torch.device("cuda", 0)
    torch.manual_seed(7)
    B, H, HKV, D, P, pages_per_req, chunk, old = 2, 16, 4, 128, 64, 8, 48, 200
    op = ops.GroupedQueryAttentionPrefillPagedWithKVCacheFwdOp(B, H, HKV, pages_per_req, P, D, validate_inputs=False)
    total = B * chunk
    q = torch.randn(total, H, D, device=device, dtype=torch.float16)
    k_new = torch.randn(total, HKV, D, device=device, dtype=torch.float16)
    v_new = torch.randn(total, HKV, D, device=device, dtype=torch.float16)
    pool = torch.randn(2, B * pages_per_req * P, HKV, D, device=device, dtype=torch.float16)
    ones = torch.ones(1, device=device, dtype=torch.float32)
    cu = torch.arange(0, total + 1, chunk, device=device, dtype=torch.int32)
    cache_lens = torch.full((B,), old, device=device, dtype=torch.int32)
    bt = torch.randperm(B * pages_per_req, device=device).to(torch.int32).reshape(B, pages_per_req)

    def run(fn):
        k_pages, v_pages = pool[0].clone(), pool[1].clone()
        out = fn(q, k_new, v_new, k_pages, v_pages, ones, ones, cu, cache_lens, bt, chunk)
        torch.cuda.synchronize()
        return out, k_pages, v_pages

    want = run(op)
    compiled = torch.compile(op, fullgraph=True, backend="aot_eager")
    got = run(compiled)
    for g, w in zip(got, want):
        assert torch.equal(g, w)
    assert not torch.equal(want[1], pool[0])  # the chunk did reach the pages


def test_python_statement_of_the_mfma_region_matches_the_library():
    """``mfma_kernel_serves`` (what selection asks, traceable) against the library's own answer, over a grid."""
    fp8 = torch.float8_e4m3fn
    for dim in (32, 64, 96, 128, 192, 256, 512):
        for page in (8, 16, 24, 32, 48, 64, 96, 128, 192, 256):
            for dt, kv in ((torch.float16, torch.float16), (torch.bfloat16, torch.bfloat16), (torch.bfloat16, fp8),
                           (torch.float16, fp8)):
                try:
                    native.decode_workspace(4, 1, 32, 8, dim, page, 4, dt, kv, 0, native.KERNEL_MFMA)
                    lib_says = True
                except (NotImplementedError, ValueError):
                    lib_says = False
                assert kernels.mfma_kernel_serves(dim, page, dt, kv) == lib_says, (dim, page, dt, kv)
