"""GPU parity tests of the contiguous-cache GQA decode op against the CPU oracle, through the op layer and the C ABI.

The first block restates the reference's test file (tests/ops/attention/test_gqa_decode.py:18-170): same shapes,
same generator (N(0,1) Q/K/V), same tolerance (atol = rtol = 1e-2).  The default split policy, constructor
errors and kernel selection are checked as there; the batch-1 tiers of the reference's specialised kernel have
no counterpart here (the MFMA kernel partitions every call the same way), so the run-time context switch test
keeps its lengths and drops the tier assertions.  The rest covers bf16, lengths that are not tile multiples,
a cache shorter than the op's ``seqlen_kv`` (the reference pads, this library reads what exists) and FP8 KV.
"""

import pytest
import torch

from oracle.paged_gqa_decode_ref import quantize_kv_per_token, ref_gqa_decode_contiguous
from tests.conftest import require_gfx950
from tileops_amd.kernels import GQADecodeKernel
from tileops_amd.ops import GroupedQueryAttentionDecodeWithKVCacheFwdOp as DecodeOp

DEV = "cuda"
KERNELS = ["gqa_decode_kernel", "gqa_decode_mfma_kernel"]


def _gen(batch, heads, heads_kv, seqlen_kv, dim, dtype, seed=0):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(batch, heads, dim, generator=g).to(dtype)
    k = torch.randn(batch, seqlen_kv, heads_kv, dim, generator=g).to(dtype)
    v = torch.randn(batch, seqlen_kv, heads_kv, dim, generator=g).to(dtype)
    return q, k, v


def _check(op, q, k, v, *, sm_scale=None, softcap=0.0, atol=1e-2, rtol=1e-2):
    ref = ref_gqa_decode_contiguous(q, k, v, sm_scale=sm_scale, softcap=softcap)
    out = op(q.to(DEV), k.to(DEV), v.to(DEV))
    assert out.shape == q.shape and out.dtype == q.dtype
    torch.testing.assert_close(out.float().cpu(), ref.float(), atol=atol, rtol=rtol)


def _only(key):
    from tileops_amd.kernels import GQADecodeMfmaKernel
    return {key: {"gqa_decode_kernel": GQADecodeKernel, "gqa_decode_mfma_kernel": GQADecodeMfmaKernel}[key]}


# --- the reference's cases ----------------------------------------------------------------------------------
@pytest.mark.gpu
@pytest.mark.parametrize(
    "batch, heads, heads_kv, seq_len_kv, dim, dtype",
    [(1, 32, 8, 8192, 128, torch.float16), (1, 32, 8, 8192, 128, torch.bfloat16), (1, 16, 2, 8192, 128, torch.float16),
     (8, 64, 16, 8192, 128, torch.float16)],
)
def test_gqa_decode(batch, heads, heads_kv, seq_len_kv, dim, dtype):
    require_gfx950()
    op = DecodeOp(batch, heads, heads_kv, seq_len_kv, dim, tune=False)
    _check(op, *_gen(batch, heads, heads_kv, seq_len_kv, dim, dtype))


@pytest.mark.gpu
@pytest.mark.parametrize("sm_scale, softcap", [pytest.param(0.25, None, id="custom-sm-scale"), pytest.param(None, 2.0, id="softcap")])
def test_gqa_decode_softmax_controls(sm_scale, softcap):
    require_gfx950()
    batch, heads, heads_kv, seq_len_kv, dim = 1, 16, 4, 1024, 64
    op = DecodeOp(batch, heads, heads_kv, seq_len_kv, dim, sm_scale=sm_scale, softcap=softcap)
    _check(op, *_gen(batch, heads, heads_kv, seq_len_kv, dim, torch.float16), sm_scale=sm_scale, softcap=softcap or 0.0)


@pytest.mark.gpu
def test_gqa_decode_default_split_policy():
    require_gfx950()
    assert GQADecodeKernel(1, 16, 2, 8192, 128, dtype="float16").config["num_split"] == 32
    assert GQADecodeKernel(1, 16, 2, 8, 128, dtype="float16").config["num_split"] == 8
    assert GQADecodeKernel(1, 40, 8, 8192, 128, dtype="float16").config["num_split"] == 16
    assert GQADecodeKernel(8, 16, 2, 8192, 128, dtype="float16").config["num_split"] == 16


@pytest.mark.gpu
def test_gqa_decode_split_policy_filters_short_kv_autotune_configs():
    require_gfx950()
    kernel = GQADecodeKernel(1, 16, 2, 8, 128, dtype="float16")
    assert {cfg["num_split"] for cfg in kernel.autotune_configs} == {2, 4, 8}
    tiny = GQADecodeKernel(1, 16, 2, 1, 128, dtype="float16")
    assert tiny.config["num_split"] == 1
    assert {cfg["num_split"] for cfg in tiny.autotune_configs} == {1}


@pytest.mark.gpu
@pytest.mark.parametrize("args, match", [((1, 16, 0, 8192, 128), "groups must be positive"),
                                          ((1, 15, 2, 8192, 128), "heads must be divisible by groups"),
                                          ((1, 16, 2, 0, 128), "seqlen_kv must be positive")])
def test_gqa_decode_kernel_rejects(args, match):
    require_gfx950()
    with pytest.raises(ValueError, match=match):
        GQADecodeKernel(*args, dtype="float16")


@pytest.mark.gpu
def test_gqa_decode_dispatch():
    """Head dims 64, 128 and 256 select the MFMA kernel for every dtype and batch."""
    require_gfx950()
    q = torch.empty(1, device=DEV)
    op = DecodeOp(1, 32, 4, 8192, 128)
    assert op._get_kernel((q,), torch.float16).__class__.__name__ == "GQADecodeMfmaKernel"
    assert op._get_kernel((q,), torch.bfloat16).__class__.__name__ == "GQADecodeMfmaKernel"
    assert DecodeOp(4, 32, 4, 4096, 64)._get_kernel((q,), torch.float16).__class__.__name__ == "GQADecodeMfmaKernel"
    assert DecodeOp(4, 32, 4, 4096, 256)._get_kernel((q,), torch.float16).__class__.__name__ == "GQADecodeMfmaKernel"


@pytest.mark.gpu
def test_gqa_decode_runtime_context_switch():
    """One op instance stays correct as the cache grows: crossover, aligned, unaligned and short lengths."""
    require_gfx950()
    op = DecodeOp(1, 32, 4, 8192, 128)
    for real in (6000, 3072, 2048, 1024, 512, 33, 1):
        _check(op, *_gen(1, 32, 4, real, 128, torch.float16, seed=real))


@pytest.mark.gpu
def test_gqa_decode_group4():
    require_gfx950()
    op = DecodeOp(1, 32, 8, 4096, 128)
    _check(op, *_gen(1, 32, 8, 4096, 128, torch.float16))


# --- beyond the reference -----------------------------------------------------------------------------------
@pytest.mark.gpu
@pytest.mark.parametrize("key", KERNELS)
@pytest.mark.parametrize("batch, heads, heads_kv, n_kv, dtype", [(3, 32, 8, 777, torch.bfloat16), (2, 16, 16, 130, torch.float16),
                                                                 (5, 64, 8, 2049, torch.bfloat16)])
def test_gqa_decode_each_kernel(key, batch, heads, heads_kv, n_kv, dtype):
    require_gfx950()
    op = DecodeOp(batch, heads, heads_kv, 4096, 128, kernel_map=_only(key))
    _check(op, *_gen(batch, heads, heads_kv, n_kv, 128, dtype, seed=n_kv), atol=2e-2, rtol=2e-2)


@pytest.mark.gpu
@pytest.mark.parametrize("key", KERNELS)
def test_gqa_decode_fp8_cache(key):
    """FP8-e4m3fn cache with per-(token, head) scales; oracle = dequantise to fp32, then the same attention."""
    require_gfx950()
    batch, heads, heads_kv, n_kv, dim = 4, 32, 8, 1500, 128
    q, k, v = _gen(batch, heads, heads_kv, n_kv, dim, torch.bfloat16, seed=7)
    k8, ks = quantize_kv_per_token(k.reshape(-1, heads_kv, dim).float())
    v8, vs = quantize_kv_per_token(v.reshape(-1, heads_kv, dim).float())
    kd = (k8.float() * ks.unsqueeze(-1)).reshape(batch, n_kv, heads_kv, dim)
    vd = (v8.float() * vs.unsqueeze(-1)).reshape(batch, n_kv, heads_kv, dim)
    ref = ref_gqa_decode_contiguous(q.float(), kd, vd)
    op = DecodeOp(batch, heads, heads_kv, 2048, dim, kernel_map=_only(key))
    out = op(q.to(DEV), k8.reshape(batch, n_kv, heads_kv, dim).to(DEV), v8.reshape(batch, n_kv, heads_kv, dim).to(DEV),
             ks.reshape(batch, n_kv, heads_kv).to(DEV), vs.reshape(batch, n_kv, heads_kv).to(DEV))
    torch.testing.assert_close(out.float().cpu(), ref.float(), atol=3e-2, rtol=3e-2)


@pytest.mark.gpu
def test_gqa_decode_rejects_bad_calls():
    require_gfx950()
    op = DecodeOp(2, 16, 4, 256, 128)
    q, k, v = (t.to(DEV) for t in _gen(2, 16, 4, 256, 128, torch.float16))
    with pytest.raises(ValueError, match="Expected q.shape"):
        op(q[:1], k, v)
    with pytest.raises(ValueError, match="seqlen_kv=256"):
        op(q, torch.cat([k, k], 1), torch.cat([v, v], 1))
    with pytest.raises(ValueError, match="contiguous"):
        op(q, k.transpose(1, 2).contiguous().transpose(1, 2), v)
    with pytest.raises(ValueError, match="k_scale and v_scale must be None"):
        op(q, k, v, torch.ones(2, 256, 4, device=DEV), torch.ones(2, 256, 4, device=DEV))


# --- host-only ----------------------------------------------------------------------------------------------
def test_gqa_decode_op_constructs_without_device():
    op = DecodeOp(4, 32, 8, 4096, 128, softcap=30.0)
    assert set(op.kernel_map) == set(KERNELS)
    assert op.sm_scale == 128 ** -0.5 and op.softcap == 30.0
    flops, nbytes = op.eval_roofline()  # reference formula: src/tileops/perf/formulas.py:683-687
    assert flops == 4 * 4 * 32 * 4096 * 128
    assert nbytes == (2 * 4 * 32 * 128 + 2 * 4 * 4096 * 8 * 128) * 2
    with pytest.raises(ValueError, match="heads must be divisible by heads_kv"):
        DecodeOp(1, 30, 8, 128, 128)
    with pytest.raises(ValueError, match="softcap must be non-negative"):
        DecodeOp(1, 32, 8, 128, 128, softcap=-1.0)
