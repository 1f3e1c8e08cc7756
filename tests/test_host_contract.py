"""Host-side contract of the op layer, the backend seam and the C ABI -- no GPU involved.

Modelled on the reference's CPU tests with fakes (tests/test_op_backend_seam.py, tests/test_backend.py) and on
the known answers in tests/ops/attention/test_gqa_decode_paged.py.
"""

import ctypes
import re
from pathlib import Path

import pytest
import torch

import tileops_amd
from tileops_amd import backend, native
from tileops_amd.backend import BUILTIN, BackendError, OpNotAvailableError, TensorSpec, UnknownTargetError
from tileops_amd.kernels import (
    AttentionCall, GQADecodePagedKernel, GQADecodePagedMfmaKernel, Kernel, PAGED_DECODE_KEYS, gqa_decode_paged_block_n,
    gqa_decode_paged_block_ns,
)
from tileops_amd.manifest import load_manifest, load_workloads
from tileops_amd.ops import (
    GroupedQueryAttentionDecodePagedWithKVCacheFwdOp as PagedOp,
    GroupedQueryAttentionMultiTokenDecodePagedWithKVCacheFwdOp as MultiOp,
)
from tileops_amd.roofline import algorithmic_bytes, gqa_decode_paged_roofline

ROOT = Path(__file__).resolve().parent.parent


def _cpu_inputs(batch=2, heads=4, heads_kv=2, n_tok=32, dim=64, page=16, dtype=torch.float16, kv_dtype=None):
    q = torch.zeros(batch, heads, dim, dtype=dtype)
    k = torch.zeros(n_tok, heads_kv, dim, dtype=dtype).to(kv_dtype or dtype)
    v = k.clone()
    lens = torch.full((batch,), page, dtype=torch.int32)
    table = torch.zeros(batch, n_tok // page, dtype=torch.int32)
    return q, k, v, lens, table


# --- constructor contract (gqa.py:1362-1387) ---------------------------------------------------------------
def test_constructor_defaults_and_validation_messages():
    op = PagedOp(2, 32, 8, 4096, 128, 64)
    assert op.sm_scale == 128 ** -0.5 and op.softcap == 0.0 and op.tune is False
    assert PagedOp(2, 32, 8, 4096, 128, 64, sm_scale=0.25, softcap=2.0).sm_scale == 0.25
    for kwargs, msg in [
        (dict(heads=0), "heads must be positive"), (dict(heads_kv=0), "heads_kv must be positive"),
        (dict(heads=30), "heads must be divisible by heads_kv"), (dict(dim=0), "dim must be positive"),
        (dict(page_size=0), "page_size must be positive"), (dict(softcap=-1.0), "softcap must be non-negative"),
    ]:
        args = dict(batch=2, heads=32, heads_kv=8, seqlen_kv=4096, dim=128, page_size=64)
        args.update(kwargs)
        with pytest.raises(ValueError, match=msg):
            PagedOp(**args)
    # positional order is the reference's: batch, heads, heads_kv, seqlen_kv, dim, page_size, sm_scale, softcap, kernel_map, tune
    op = PagedOp(1, 16, 4, 1024, 128, 64, None, 2.0, None, False)
    assert op.softcap == 2.0


def test_manifest_entry_keeps_the_reference_shape():
    entry = load_manifest()["GroupedQueryAttentionDecodePagedWithKVCacheFwdOp"]
    sig = entry["signature"]
    assert list(sig["inputs"])[:5] == ["q", "k", "v", "real_seqlen_kv", "block_table"]
    assert list(sig["params"]) == ["page_size", "sm_scale", "softcap"]
    assert sig["params"]["sm_scale"]["default"] is None and sig["params"]["softcap"]["default"] is None
    assert all(sig["inputs"][n].get("optional") for n in ("k_scale", "v_scale"))
    assert entry["roofline"]["func"] == "tileops_amd.roofline.gqa_decode_paged_roofline"
    assert set(entry["source"]["kernel_map"]) == set(PAGED_DECODE_KEYS)
    labels = [w["label"] for w in load_workloads("GroupedQueryAttentionDecodePagedWithKVCacheFwdOp")]
    assert labels[:3] == ["serving-8b-p64", "serving-8b-long-p64", "throughput-8b-p64"] and "llama3-8b-paged-fp8kv" in labels
    # kernel_map values are class names that exist; forward's leading parameters are the manifest inputs in order
    import inspect

    import tileops_amd.kernels as K
    for cls_name in entry["source"]["kernel_map"].values():
        assert issubclass(getattr(K, cls_name), Kernel)
    for op_cls in (PagedOp, MultiOp):
        params = list(inspect.signature(op_cls.forward).parameters)[1:]
        assert params == list(load_manifest()[op_cls.__name__]["signature"]["inputs"])
        assert op_cls.__manifest_param_names__ == tuple(load_manifest()[op_cls.__name__]["signature"]["params"])
        init = inspect.signature(op_cls.__init__).parameters
        assert "kernel_map" in init and init["sm_scale"].default is None and init["softcap"].default is None


def test_validate_dtypes_follows_the_manifest():
    op = PagedOp(2, 4, 2, 32, 64, 16)
    q, k, v, lens, table = _cpu_inputs()
    op._validate_dtypes(q, k, v, lens, table, None, None)
    op._validate_dtypes(q, k.to(torch.float8_e4m3fn), v.to(torch.float8_e4m3fn), lens, table, torch.ones(32, 2), torch.ones(32, 2))
    with pytest.raises(ValueError, match="q.dtype"):
        op._validate_dtypes(q.float(), k, v, lens, table)
    with pytest.raises(ValueError, match="same as k"):
        op._validate_dtypes(q, k, v.to(torch.bfloat16), lens, table)
    with pytest.raises(ValueError, match="real_seqlen_kv.dtype"):
        op._validate_dtypes(q, k, v, lens.long(), table)
    with pytest.raises(ValueError, match="combination"):
        op._validate_dtypes(q, k.to(torch.bfloat16), v.to(torch.bfloat16), lens, table)
    with pytest.raises(ValueError, match="k_scale.dtype"):
        op._validate_dtypes(q, k.to(torch.float8_e4m3fn), v.to(torch.float8_e4m3fn), lens, table, torch.ones(32, 2).half(), torch.ones(32, 2))


def test_forward_validates_layout_before_any_kernel_is_built():
    op = PagedOp(2, 4, 2, 32, 64, 16)
    q, k, v, lens, table = _cpu_inputs()
    cases = [
        ((q[:, :2], k, v, lens, table), "q.shape"), ((q, k[:16], v[:16], lens, table), "k.shape"),
        ((q, k, v, lens[:1], table), "real_seqlen_kv.shape"), ((q, k, v, lens, table[:1]), "block_table.shape"),
        ((q.transpose(0, 1).contiguous().transpose(0, 1), k, v, lens, table), "q must be contiguous"),
        ((q, k, v, lens, table, torch.ones(32, 2), torch.ones(32, 2)), "must be None unless"),
        ((q, k.to(torch.float8_e4m3fn), v.to(torch.float8_e4m3fn), lens, table), "are required"),
        ((q, k.to(torch.float8_e4m3fn), v.to(torch.float8_e4m3fn), lens, table, torch.ones(16, 2), torch.ones(32, 2)), "k_scale.shape"),
    ]
    for args, msg in cases:
        with pytest.raises(ValueError, match=msg):
            op(*args)
        assert op._builder is not None and op._settled_target is None  # a failed call settles nothing
    assert op._infer_output_shapes((2, 4, 64), (32, 2, 64), (32, 2, 64), (2,), (2, 2)) == {"o": (2, 4, 64)}
    m = MultiOp(2, 3, 4, 2, 32, 64, 16)
    with pytest.raises(ValueError, match=re.escape("q.shape (2, 3, 4, 64)")):
        m(q, k, v, lens, table)
    with pytest.raises(ValueError, match="q_len must be positive"):
        MultiOp(2, 0, 4, 2, 32, 64, 16)


def test_no_gpu_means_a_loud_failure_not_a_fallback():
    op = PagedOp(2, 4, 2, 32, 64, 16)
    if torch.cuda.is_available():
        pytest.skip("CPU-only expectation")
    with pytest.raises(ValueError, match=r"built for architectures \[95\], device reports None"):
        op(*_cpu_inputs())
    with pytest.raises(ValueError, match="no implementation serves this call"):
        op._get_kernel((), torch.float16)


# --- tile rule and selection (test_gqa_decode_paged.py:122-151, 235-272) -----------------------------------
def test_page_tile_rule_known_answers():
    assert gqa_decode_paged_block_ns(192) == (64,) and gqa_decode_paged_block_n(256) == 128
    assert gqa_decode_paged_block_ns(16) == (16,)
    for page in (96, 160, 224):
        with pytest.raises(ValueError, match="matches no supported block_N"):
            gqa_decode_paged_block_ns(page)


def _call(**kw):
    base = dict(dtype=torch.bfloat16, batch=64, heads=32, heads_kv=8, seqlen_kv=1 << 20, dim=128, page_size=64,
                sm_scale=128 ** -0.5, softcap=0.0, arch=95)
    base.update(kw)
    return AttentionCall(**base)


def test_selection_regions():
    op = PagedOp(64, 32, 8, 1 << 20, 128, 64)
    assert GQADecodePagedKernel.general and not GQADecodePagedMfmaKernel.general
    assert GQADecodePagedKernel.refusal(_call()) is None
    assert "device reports 90" in GQADecodePagedKernel.refusal(_call(arch=90))
    key = op.select_kernel_key(PAGED_DECODE_KEYS, _call())
    mfma_serves = GQADecodePagedMfmaKernel.applies(_call())
    assert key == ("gqa_decode_paged_mfma_kernel" if mfma_serves else "gqa_decode_paged_kernel")
    # shapes outside the specialised region stay on the general kernel
    for kw in (dict(page_size=24), dict(dim=96), dict(dim=32, kv_dtype=torch.float8_e4m3fn)):
        assert not GQADecodePagedMfmaKernel.applies(_call(**kw))
        assert op.select_kernel_key(PAGED_DECODE_KEYS, _call(**kw)) == "gqa_decode_paged_kernel"
    # head dims 64 and 256 are inside it, with either cache
    assert GQADecodePagedMfmaKernel.applies(_call(dim=64)) == mfma_serves
    assert GQADecodePagedMfmaKernel.applies(_call(dim=64, kv_dtype=torch.float8_e4m3fn)) == mfma_serves
    assert GQADecodePagedMfmaKernel.applies(_call(dim=256, kv_dtype=torch.float8_e4m3fn)) == mfma_serves
    assert GQADecodePagedMfmaKernel.applies(_call(dim=256)) == mfma_serves
    with pytest.raises(ValueError, match="no implementation serves this call"):
        op.select_kernel_key(PAGED_DECODE_KEYS, _call(arch=90))


def test_selection_never_bypasses_a_caller_override():
    class Picky(GQADecodePagedKernel):
        general = False

        @classmethod
        def applies(cls, call):
            return call.batch == 1

    op = PagedOp(64, 32, 8, 1 << 20, 128, 64, kernel_map={"gqa_decode_paged_mfma_kernel": Picky})
    assert op.kernel_map["gqa_decode_paged_mfma_kernel"] is Picky and op.kernel_map["gqa_decode_paged_kernel"] is GQADecodePagedKernel
    assert op.select_kernel_key(PAGED_DECODE_KEYS, _call(batch=1)) == "gqa_decode_paged_mfma_kernel"
    with pytest.raises(ValueError, match="does not fall back to the shipped"):
        op.select_kernel_key(PAGED_DECODE_KEYS, _call(batch=2))

    class Greedy(GQADecodePagedKernel):
        general = False

    op2 = PagedOp(1, 32, 8, 1 << 20, 128, 64, kernel_map={"gqa_decode_paged_kernel": Greedy, "gqa_decode_paged_mfma_kernel": Picky})
    with pytest.raises(ValueError, match="dispatch is ambiguous"):
        op2.select_kernel_key(PAGED_DECODE_KEYS, _call(batch=1))


def test_kernel_constructor_validation_needs_the_right_arch_first():
    if torch.cuda.is_available():
        pytest.skip("CPU-only expectation")
    with pytest.raises(ValueError, match=r"built for architectures \[95\]"):
        GQADecodePagedKernel(1, 16, 4, 1536, 128, 96)


# --- backend seam with fakes (tests/test_op_backend_seam.py:23-248) ----------------------------------------
class _Recorder:
    def __init__(self, result=None):
        self.builds, self.calls, self.result = [], [], result

    def __call__(self, *specs, **params):
        self.builds.append((specs, params))
        return self.result if self.result is not None else self._kernel

    def _kernel(self, *tensors):
        self.calls.append(tensors)
        return torch.full_like(tensors[0], 7.0)


def test_external_target_is_built_once_per_signature_with_manifest_params(clean_registry):
    rec = _Recorder()
    backend.register_detector("fake", lambda dev: dev.type == "cpu")
    backend.register_kernel_builder(PagedOp.__name__, "fake", rec)
    op = PagedOp(2, 4, 2, 32, 64, 16, softcap=None)
    args = _cpu_inputs()
    out = op(*args)
    assert torch.equal(out, torch.full_like(args[0], 7.0)) and op._settled_target == "fake"
    op(*args)
    assert len(rec.builds) == 1 and len(rec.calls) == 2          # built once, called twice
    specs, params = rec.builds[0]
    assert len(specs) == 7 and specs[5] is None and specs[6] is None  # absent optional inputs keep their slot
    assert specs[0] == TensorSpec(torch.device("cpu"), torch.float16, (2, 4, 64))
    assert params == {"page_size": 16, "sm_scale": 64 ** -0.5, "softcap": 0.0}  # defaults arrive resolved
    assert len(rec.calls[0]) == 5                                 # kernel(q, k, v, real_seqlen_kv, block_table)
    op(*_cpu_inputs(dtype=torch.bfloat16))
    assert len(rec.builds) == 2                                   # a new dtype signature builds again


def test_external_target_rules(clean_registry):
    args = _cpu_inputs()
    with pytest.raises(UnknownTargetError, match="no backend registered target 'nope'"):
        PagedOp(2, 4, 2, 32, 64, 16, target="nope")(*args)
    backend.register_detector("fake", lambda dev: True)
    op = PagedOp(2, 4, 2, 32, 64, 16)
    with pytest.raises(OpNotAvailableError, match="registers no kernel builder"):
        op(*args)
    assert op._settled_target is None                             # failed settling pins nothing
    backend.register_kernel_builder(PagedOp.__name__, "fake", _Recorder(result="not callable"))
    with pytest.raises(OpNotAvailableError, match="not callable"):
        op(*args)
    with pytest.raises(BackendError, match="already has detector"):
        backend.register_detector("fake", lambda dev: False)
    with pytest.raises(BackendError, match="already registered"):
        backend.register_kernel_builder(PagedOp.__name__, "fake", _Recorder())
    backend.register_detector("other", lambda dev: True)
    with pytest.raises(backend.AmbiguousTargetError):
        PagedOp(2, 4, 2, 32, 64, 16)(*args)
    backend.register_detector("broken", lambda dev: 1 / 0)
    with pytest.raises(BackendError, match="raised on device"):
        backend.detect_target(torch.device("cpu"))


def test_target_selection_order_and_builtin(clean_registry):
    a, b = _Recorder(), _Recorder()
    backend.register_kernel_builder(PagedOp.__name__, "a", a)
    backend.register_kernel_builder(PagedOp.__name__, "b", b)
    backend.register_detector("a", lambda dev: True)
    assert backend.registered_targets(PagedOp.__name__) == ["a", "b"] and backend.registered_targets() == ["a", "b"]
    args = _cpu_inputs()
    PagedOp(2, 4, 2, 32, 64, 16)(*args)                            # detection -> a
    backend.set_default_target("b")
    PagedOp(2, 4, 2, 32, 64, 16)(*args)                            # default beats detection -> b
    PagedOp(2, 4, 2, 32, 64, 16, target="a")(*args)                # explicit beats default -> a
    assert (len(a.builds), len(b.builds)) == (2, 1)
    backend.set_default_target(None)
    assert backend.default_target() is None
    with pytest.raises(UnknownTargetError):
        backend.set_default_target("zzz")
    if not torch.cuda.is_available():
        with pytest.raises(ValueError, match="no implementation serves this call"):
            PagedOp(2, 4, 2, 32, 64, 16, target=BUILTIN)(*args)   # BUILTIN = in-tree HIP kernels, which need the GPU


def test_plugin_registers_detector_and_lazy_builders(clean_registry):
    from tileops_amd import tileops_plugin

    tileops_plugin.register(into=backend)
    assert backend.registered_targets(PagedOp.__name__) == ["mi355x"] == backend.registered_targets(MultiOp.__name__)
    assert tileops_plugin.detect(torch.device("cpu")) is False
    assert backend.detect_target(torch.device("cpu")) is None


# --- roofline ------------------------------------------------------------------------------------------------
def test_roofline_reference_formula_and_true_bytes():
    op = PagedOp(64, 32, 8, 1 << 20, 128, 64)
    op.dtype = torch.bfloat16
    assert op.eval_roofline() == (4 * 64 * 32 * (1 << 20) * 128, (2 * 64 * 32 * 128 + 2 * (1 << 20) * 8 * 128) * 2 + 64 * 4 + 64 * 16384 * 4)
    lens = torch.tensor([512, 8192] * 32, dtype=torch.int32)
    op.observe_call(lens, torch.bfloat16)
    flops, nbytes = op.eval_roofline()
    sum_len = int(lens.sum())
    assert flops == 4 * 32 * 128 * sum_len
    assert nbytes == sum_len * 8 * 128 * 2 * 2 + 2 * 64 * 32 * 128 * 2 + 4 * 64 + 4 * int(((lens + 63) // 64).sum())
    b = algorithmic_bytes(sum_len=278528, sum_pages=4352, batch=64, q_len=1, heads=32, heads_kv=8, dim=128, q_bytes=2, kv_bytes=1, fp8_scales=True)
    assert b["kv"] == 570425344 and b["scales"] == 17825792 and b["total"] == 570425344 + 17825792 + 1048576 + 256 + 17408
    assert gqa_decode_paged_roofline(q_shape=[32, 32, 128], kv_shape=[4096, 8, 128], page_size=64, dtypes=["float16"]) == (2147483648, 17309824)


# --- C ABI: the library loads and exports what the header declares (no compute calls) ----------------------
def test_library_exports_every_declared_symbol():
    header = (ROOT / "include" / "mi355_tileops.h").read_text()
    declared = set(re.findall(r"\b(mi355_[a-z0-9_]+)\s*\(", header))
    assert declared == set(native.EXPORTED_SYMBOLS)
    lib = native.load()
    for sym in declared:
        assert hasattr(lib, sym)
    assert lib.mi355_abi_version() == int(re.search(r"#define MI355_ABI_VERSION (\d+)", header).group(1))


def test_workspace_planning_is_host_only_and_reports_errors():
    nbytes, nsplit, kernel = native.decode_workspace(64, 1, 32, 8, 128, 64, 128, torch.bfloat16, torch.bfloat16, 0, native.KERNEL_GENERIC)
    assert kernel == native.KERNEL_GENERIC and nsplit == 16           # 128 pages * 64 / 512-token splits
    assert nbytes == 64 * 16 * 8 * 4 * 128 * 4 + 64 * 16 * 8 * 4 * 4
    assert native.decode_workspace(1, 1, 16, 8, 128, 128, 4, torch.float16, torch.float16, 0, native.KERNEL_GENERIC)[:2] == (0, 1)
    with pytest.raises(ValueError, match="heads must be divisible by heads_kv"):
        native.decode_workspace(1, 1, 30, 8, 128, 64, 4, torch.bfloat16, torch.bfloat16)
    with pytest.raises(NotImplementedError, match="head dim 96"):
        native.decode_workspace(1, 1, 32, 8, 96, 64, 4, torch.bfloat16, torch.bfloat16)
    with pytest.raises(ValueError, match="must equal q_dtype"):
        native.decode_workspace(1, 1, 32, 8, 128, 64, 4, torch.bfloat16, torch.float16)
    # the MFMA kernel cuts the tile stream so that every compute unit holds eight waves (four at head dim 256)
    fp8 = torch.float8_e4m3fn
    assert [native.decode_workspace(64, 1, 32, 8, d, 64, 128, torch.bfloat16, fp8, 0, native.KERNEL_MFMA)[1:] for d in (64, 128, 256)] == \
        [(256, native.KERNEL_MFMA), (256, native.KERNEL_MFMA), (128, native.KERNEL_MFMA)]
    # prefill: the fused-RoPE call adds room for the rotated queries, an FP8 cache two fp32 result sets to merge
    plain = native.prefill_paged_workspace(8, 512, 4096, 32, 8, 128, 64, 72, torch.bfloat16, torch.bfloat16)
    assert native.prefill_paged_rope_workspace(8, 512, 4096, 32, 8, 128, 64, 72, torch.bfloat16) == plain + 4096 * 32 * 128 * 2
    assert native.prefill_paged_workspace(8, 512, 4096, 32, 8, 128, 64, 72, torch.bfloat16, fp8) >= plain + 2 * 4096 * 32 * 128 * 4
    with pytest.raises(ValueError, match="heads must be divisible by heads_kv"):
        native.prefill_paged_workspace(8, 512, 4096, 30, 8, 128, 64, 72, torch.bfloat16, torch.bfloat16)
    with pytest.raises(ValueError, match="total_q must be non-negative"):
        native.prefill_paged_rope_workspace(8, 512, -1, 32, 8, 128, 64, 72, torch.bfloat16)
    with pytest.raises(NotImplementedError, match="head dim 96"):
        native.prefill_paged_workspace(8, 512, 4096, 32, 8, 96, 64, 72, torch.bfloat16, torch.bfloat16)
    lib = native.load()
    rc = lib.mi355_gqa_paged_decode(None, None, None, None, None, None, None, 1, None, None, 0, 1, 1, 32, 8, 128, 64, 64,
                                    native.DT_BF16, native.DT_BF16, 1.0, 0.0, 1, 0, 0, None)
    assert rc == -1 and b"non-null" in lib.mi355_last_error()
    assert tileops_amd.__version__


@pytest.mark.skipif(torch.cuda.is_available(), reason="needs a host without a GPU: the pointers below are made up")
def test_entry_points_refuse_without_a_gfx950_device_before_launching():
    """A call whose arguments pass validation still launches nothing when no gfx950 device is current: every launching
    entry point returns MI355_EDEVICE with a message (the reference refuses by architecture before it builds a kernel,
    src/tileops/kernels/kernel_base.py:98-112).  Argument errors keep precedence, workspace queries touch no device."""
    lib = native.load()
    header = (ROOT / "include" / "mi355_tileops.h").read_text()
    edevice = int(re.search(r"#define MI355_EDEVICE \((-?\d+)\)", header).group(1))
    fake = 0x10000  # aligned, never dereferenced
    ws_bytes, n_parts, _ = native.decode_workspace(2, 1, 32, 8, 128, 64, 4, torch.bfloat16, torch.bfloat16, 0, native.KERNEL_MFMA)
    rc = lib.mi355_gqa_paged_decode(fake, fake, fake, None, None, fake, fake, 4, fake, fake, ws_bytes, 2, 1, 32, 8, 128, 64, 64 * 8,
                                    native.DT_BF16, native.DT_BF16, 1.0, 0.0, 1, 0, native.KERNEL_MFMA, None)
    assert rc == edevice and b"gfx950" in lib.mi355_last_error()
    rc = lib.mi355_gqa_decode(fake, fake, fake, None, None, fake, fake, 1 << 30, 2, 1, 32, 8, 128, 4096, 1000,
                              native.DT_BF16, native.DT_BF16, 1.0, 0.0, 1, 0, native.KERNEL_GENERIC, None)
    assert rc == edevice
    rc = lib.mi355_gather_probe(fake, fake, fake, 4, fake, 2, 256, 2048, 64, 64 * 8, None)
    assert rc == edevice
    rc = lib.mi355_kv_append_fp8(fake, fake, fake, fake, fake, 4, 2, 8, 128, 64, 64 * 8, native.DT_BF16, None)
    assert rc == edevice
    need = native.prefill_paged_workspace(2, 16, 32, 32, 8, 128, 64, 4, torch.bfloat16, torch.bfloat16)
    rc = lib.mi355_gqa_prefill_paged(fake, fake, fake, fake, fake, fake, fake, fake, fake, fake, 4, fake, fake, need, 2, 16, 32, 32, 8,
                                     128, 64, 64 * 8, native.DT_BF16, native.DT_BF16, 1.0, 0.0, 1, native.KERNEL_AUTO, None)
    assert rc == edevice
    # an argument error is still reported first
    rc = lib.mi355_gqa_paged_decode(fake, fake, fake, None, None, fake, fake, 4, fake, fake, ws_bytes, 2, 1, 30, 8, 128, 64, 64 * 8,
                                    native.DT_BF16, native.DT_BF16, 1.0, 0.0, 1, 0, native.KERNEL_MFMA, None)
    assert rc == -1
    # the Python binding turns the code into the package's library error
    q = torch.zeros(2, 32, 128, dtype=torch.bfloat16)
    with pytest.raises(native.NativeLibraryError):
        native._check(lib.mi355_gather_probe(fake, fake, fake, 4, fake, 2, 256, 2048, 64, 64 * 8, None))
    assert "gfx950" in native.last_error() and q.device.type == "cpu"


def test_benchmark_configurations_are_manifest_rows():
    """bench.py takes its four GPU configurations from the manifest (`load_workloads`), not from shapes of its own: the
    rows must describe exactly the configurations the parity tests run at full size."""
    from tileops_amd.workloads import BASELINE_CONFIGS, BASELINE_WORKLOAD_ROWS, config_from_workload

    assert set(BASELINE_WORKLOAD_ROWS) == set(BASELINE_CONFIGS) == {"c2", "c3", "c4", "c5"}
    for name, (op_name, label) in BASELINE_WORKLOAD_ROWS.items():
        row = next(r for r in load_workloads(op_name) if r["label"] == label)
        want = BASELINE_CONFIGS[name]
        assert config_from_workload(row, name, want.description) == want
    for op_name in ("GroupedQueryAttentionDecodePagedWithKVCacheFwdOp", "GroupedQueryAttentionMultiTokenDecodePagedWithKVCacheFwdOp"):
        entry = load_manifest()[op_name]
        assert entry["source"]["bench"] == "bench.py" and entry["source"].get("bench_manifest_driven") is True
    src = (ROOT / "bench.py").read_text()
    assert "load_workloads(" in src and "eval_roofline()" in src


def test_bench_refuses_more_than_one_gpu_with_a_message():
    """``bench.py --gpus N`` with N above 1 (or a multi-rank launch) exits non-zero before touching a device and says why."""
    import subprocess
    import sys
    from pathlib import Path

    bench = Path(__file__).resolve().parents[1] / "bench.py"
    res = subprocess.run([sys.executable, str(bench), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert res.returncode != 0 and "one GPU" in res.stderr and res.stdout.strip() == ""
    env = dict(__import__("os").environ, WORLD_SIZE="4")
    res = subprocess.run([sys.executable, str(bench)], capture_output=True, text=True, timeout=120, env=env)
    assert res.returncode != 0 and "one GPU" in res.stderr
