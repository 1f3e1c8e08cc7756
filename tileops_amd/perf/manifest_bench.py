"""Manifest-driven benchmark of the ops, reporting in the reference's formats.

Takes the place of the reference's benchmark plumbing for these ops (benchmarks/ops/attention/
bench_gqa_decode_paged.py:150-210 and bench_gqa_decode.py drive the manifest workloads; benchmarks/report.py:117-262
collects records and dumps ``profile_run.log``; benchmarks/conftest.py:52-136 attaches ``<tag>_<metric>``
properties to the JUnit XML).  This runner needs no pytest plugin: it walks the manifest, times every workload
and writes both artefacts itself.

    python -m tileops_amd.perf.manifest_bench [--op NAME] [--label SUBSTR] [--steps N] [--out DIR]

Per workload and implementation (tag) it records ``latency_ms`` (median device time of one call, HIP events, the
L2/MALL flushed between calls -- the methodology of benchmarks/timing.py:546-585), ``tflops`` and
``bandwidth_tbs`` from the op's ``eval_roofline()`` after it has seen the call, and ``hbm_frac`` = bandwidth over
the 8 TB/s peak.  ``device_busy_ms`` (sum of kernel durations) is taken from the torch profiler when it delivers
device events, otherwise left out.  Baselines on the same device (no FlashInfer / AITER build is importable in this
image; the tag slot is there): tag ``torch_sdpa`` = ``F.scaled_dot_product_attention`` for the contiguous op; tag
``torch_gather_sdpa`` = for a paged row, two dense ``index_select`` copies of the pages each sequence addresses followed by
SDPA with a boolean padding mask and ``enable_gqa`` (torch's math path) -- a plain-torch way to do the same job, not a
tuned kernel, so its ratio says what a user gains over eager torch and nothing about kernel quality.  Rows with an FP8
cache, several query tokens or a softcap have no device baseline; the run lists them at its end.
"""

from __future__ import annotations

import argparse
import statistics
import sys
import time
import xml.etree.ElementTree as ET
from datetime import datetime
from pathlib import Path
from typing import Any, Callable, Optional

import torch

from .. import native
from ..manifest import load_manifest
from ..ops import (
    GroupedQueryAttentionDecodePagedWithKVCacheFwdOp, GroupedQueryAttentionDecodeWithKVCacheFwdOp,
    GroupedQueryAttentionMultiTokenDecodePagedWithKVCacheFwdOp, GroupedQueryAttentionPrefillPagedWithKVCacheFwdOp,
)
from ..roofline import _distribute_total, gqa_prefill_paged_with_kv_cache_fwd_roofline
from ..workloads import FP8, GroupedQueryAttentionDecodePagedWorkload, PagedDecodeConfig, gen_paged_inputs, quantize_kv_per_token

HBM_PEAK_TBS = 8.0
_DT = {"float16": torch.float16, "bfloat16": torch.bfloat16, "float8_e4m3fn": FP8}


class BenchmarkReport:
    """Records per op and tag, dumped as the markdown log the reference leaves behind (report.py:117-262)."""

    def __init__(self) -> None:
        self.records: dict[str, list[dict]] = {}

    def record(self, op_name: str, params: dict, result: dict, tag: str = "tileops", config: Optional[dict] = None) -> None:
        entry = {"params": params, "result": result, "tag": tag}
        if config:
            entry["config"] = config
        self.records.setdefault(op_name, []).append(entry)

    @staticmethod
    def _environment() -> list[str]:
        lines = [f"- **Torch version**: {torch.__version__}", f"- **HIP version (torch)**: {torch.version.hip or 'N/A'}"]
        if torch.cuda.is_available():
            props = torch.cuda.get_device_properties(0)
            lines.append(f"- **GPU model**: {props.name} ({getattr(props, 'gcnArchName', '?')}, {props.multi_processor_count} CUs)")
        else:
            lines.append("- **GPU model**: N/A (no device)")
        # The amdgpu kernel module publishes its version in sysfs; no child process is started from a process that
        # holds the GPU.
        try:
            driver = Path("/sys/module/amdgpu/version").read_text().strip() or "N/A"
        except OSError:
            driver = "N/A"
        lines.append(f"- **Driver version**: {driver}")
        return lines

    def dump(self, path: Path) -> None:
        if not self.records:
            return
        lines = ["# TileOPs Benchmark Report", f"Generated: {datetime.now().strftime('%Y-%m-%d %H:%M:%S')}", "",
                 "## Environment", "", *self._environment(), ""]
        default_keys = ["device_busy_ms", "latency_ms", "gap_ms", "n_kernels", "tflops", "bandwidth_tbs"]
        for name, entries in self.records.items():
            lines += [f"## {name}", ""]
            keys = list(default_keys)
            for e in entries:
                keys += [k for k in e["result"] if k not in keys]
            by_tag: dict[str, list[dict]] = {}
            for e in entries:
                by_tag.setdefault(e["tag"], []).append(e)
            for tag, group in by_tag.items():
                lines += [f"### {tag}", ""]
                pkeys = list(group[0]["params"])
                has_cfg = any("config" in e for e in group)
                header = pkeys + keys + (["config"] if has_cfg else [])
                lines.append("| " + " | ".join(header) + " |")
                lines.append("| " + " | ".join(["---"] * len(header)) + " |")
                for e in group:
                    row = [str(e["params"].get(k, "")) for k in pkeys]
                    for k in keys:
                        val = e["result"].get(k)
                        row.append("N/A" if val is None else (f"{val:.4f}" if isinstance(val, (int, float)) and not isinstance(val, bool) else str(val)))
                    if has_cfg:
                        row.append(str(e.get("config") or ""))
                    lines.append("| " + " | ".join(row) + " |")
                lines.append("")
        path.write_text("\n".join(lines) + "\n", encoding="utf-8")


def _prop(value: Any) -> str:
    """benchmarks/conftest.py:36-47: significant digits, not fixed decimals."""
    if isinstance(value, (bool, int)):
        return str(value)
    if isinstance(value, float):
        return str(int(value)) if value.is_integer() else f"{value:.6g}"
    return str(value)


_NOT_A_MEASUREMENT = frozenset({"tag", "op", "op_module"})  # set by the recorder, not measured


def junit_case(suite: ET.Element, name: str, entries: list[dict]) -> ET.Element:
    """One ``<testcase>`` with the properties the reference's pytest hook attaches (benchmarks/conftest.py:52-136).

    ``entries`` are the records of one benchmark case, each ``{"tag", "op", "op_module", <measurements>}``.  The first
    entry whose tag starts with ``tileops`` gives ``op``, ``op_module``, ``tileops_variant`` (for a tag
    ``tileops_<variant>``) and ``tileops_<metric>``; every other entry is written under its own tag as
    ``<tag>_<metric>``, the first of them also as ``baseline_<metric>`` with ``baseline_tag``; ``<tag>_ratio`` (and
    ``baseline_ratio``) = baseline time over ours, on ``device_busy_ms`` when both sides have it, else on ``latency_ms``.
    ``None`` values are left out.
    """
    ours = next((e for e in entries if e["tag"].startswith("tileops")), None)
    baselines = [e for e in entries if not e["tag"].startswith("tileops")]
    lat = (ours or {}).get("latency_ms") or 0.0
    case = ET.SubElement(suite, "testcase", classname=(ours or entries[0]).get("op", ""), name=name, time=f"{lat / 1e3:.6f}")
    props = ET.SubElement(case, "properties")

    def emit(tag: str, entry: dict) -> None:
        for key, val in entry.items():
            if key in _NOT_A_MEASUREMENT or val is None:
                continue
            ET.SubElement(props, "property", name=f"{tag}_{key}", value=_prop(val))

    if ours:
        ET.SubElement(props, "property", name="op", value=ours["op"])
        if "op_module" in ours:
            ET.SubElement(props, "property", name="op_module", value=ours["op_module"])
        tag = ours["tag"]
        if tag != "tileops" and tag.startswith("tileops_"):
            ET.SubElement(props, "property", name="tileops_variant", value=tag[len("tileops_"):])
        emit("tileops", ours)
    for idx, be in enumerate(baselines):
        emit(be["tag"], be)
        if idx == 0:
            ET.SubElement(props, "property", name="baseline_tag", value=be["tag"])
            emit("baseline", be)
        if not ours:
            continue
        key = "device_busy_ms" if (ours.get("device_busy_ms") or 0) > 0 and (be.get("device_busy_ms") or 0) > 0 else "latency_ms"
        tl, bl = ours.get(key) or 0, be.get(key) or 0
        if tl > 0 and bl > 0:
            ET.SubElement(props, "property", name=f"{be['tag']}_ratio", value=f"{bl / tl:.4f}")
            if idx == 0:
                ET.SubElement(props, "property", name="baseline_ratio", value=f"{bl / tl:.4f}")
    return case


def write_junit(suite: ET.Element, path: Path) -> None:
    suite.set("tests", str(len(suite.findall("testcase"))))
    ET.ElementTree(suite).write(path, encoding="utf-8", xml_declaration=True)


class _Flusher:
    """Evicts L2 and the memory-side cache between timed calls: a 512 MiB write followed by a 512 MiB read."""

    def __init__(self, device: torch.device) -> None:
        self.w = torch.empty(512 << 20, dtype=torch.uint8, device=device)
        self.r = torch.ones(128 << 20, dtype=torch.int32, device=device)
        self.i = 0

    def __call__(self) -> None:
        self.i += 1
        self.w.fill_(self.i & 255)
        self.r.max()


#: warm-up budget and iteration clamp of the reference's protocol (benchmarks/timing.py:30-36, :577): as many untimed,
#: flushed iterations as fit 25 ms, at least 10 and at most 200.  After idle the device runs its first tens of
#: milliseconds below its sustained clocks (the 8 x 512-token prefill row reads 465 us in its first twenty calls and
#: 427 us from the fortieth on), so a row timed after three warm-up calls reports the ramp, not the kernel.
_DRY_RUN_MS, _MIN_ITERS, _MAX_ITERS = 25.0, 10, 200


def _time(fn: Callable[[], Any], flush: _Flusher, steps: int) -> float:
    flush()
    fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(3):  # calibration: one flushed iteration costs this much
        flush()
        fn()
    torch.cuda.synchronize()
    per_iter_ms = max((time.perf_counter() - t0) * 1e3 / 3, 1e-3)
    for _ in range(min(max(int(_DRY_RUN_MS / per_iter_ms), _MIN_ITERS), _MAX_ITERS)):
        flush()
        fn()
    ts = []
    for _ in range(steps):
        flush()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        b.synchronize()
        ts.append(a.elapsed_time(b))
    return statistics.median(ts)


def _device_busy(fn: Callable[[], Any]) -> tuple[Optional[float], Optional[int]]:
    """(sum of kernel durations in ms, number of kernels) of one call, from the torch profiler; (None, None) if
    the profiler delivers no device events on this build."""
    try:
        from torch.profiler import ProfilerActivity, profile
        fn()
        torch.cuda.synchronize()
        with profile(activities=[ProfilerActivity.CUDA]) as prof:
            fn()
            torch.cuda.synchronize()
        evs = [e for e in prof.events() if e.device_type == torch.autograd.DeviceType.CUDA]
        if not evs:
            return None, None
        return sum(e.device_time for e in evs) / 1e3, len(evs)
    except Exception:  # noqa: BLE001 - the profiler is optional evidence, never a reason to fail a benchmark
        return None, None


def _result(op: Any, latency_ms: float, busy: tuple[Optional[float], Optional[int]]) -> dict:
    flops, nbytes = op.eval_roofline()
    res = {"latency_ms": latency_ms, "tflops": flops / latency_ms / 1e9, "bandwidth_tbs": nbytes / latency_ms / 1e9}
    res["hbm_frac"] = res["bandwidth_tbs"] / HBM_PEAK_TBS
    if busy[0] is not None:
        res["device_busy_ms"], res["n_kernels"] = busy[0], busy[1]
        res["gap_ms"] = max(latency_ms - busy[0], 0.0)
    return res


def _paged_case(row: dict, dtype: torch.dtype, device: torch.device, multi: bool):
    qs, (n_kv, heads_kv, dim) = row["q_shape"], row["kv_shape"]
    batch, heads = qs[0], qs[-2]
    q_len = qs[1] if multi else 1
    page = row["page_size"]
    kv_dtype = _DT[row.get("kv_dtype", str(dtype).removeprefix("torch."))]
    kw = dict(sm_scale=row.get("sm_scale"), softcap=row.get("softcap"))
    if multi:
        op = GroupedQueryAttentionMultiTokenDecodePagedWithKVCacheFwdOp(batch, q_len, heads, heads_kv, n_kv, dim, page, **kw)
    else:
        op = GroupedQueryAttentionDecodePagedWithKVCacheFwdOp(batch, heads, heads_kv, n_kv, dim, page, **kw)
    if "seqlen_range" in row:  # ragged lengths over a shared pool with a permuted block table
        cfg = PagedDecodeConfig(row["label"], batch, heads, heads_kv, dim, page, n_kv // page, tuple(row["seqlen_range"]),
                                q_len=q_len, dtype=dtype, kv_dtype=kv_dtype, seed=row.get("seed", 0))
        inp = gen_paged_inputs(cfg, device)
        args = (inp.q, inp.k, inp.v, inp.real_seqlen_kv, inp.block_table) + ((inp.k_scale, inp.v_scale) if inp.k_scale is not None else ())
        lens = inp.real_seqlen_kv
    else:  # the reference's generator: page-multiple random lengths, identity table
        wl = GroupedQueryAttentionDecodePagedWorkload(batch, heads, heads_kv, n_kv, dim, page, dtype, **kw)
        args = wl.gen_inputs(device)
        lens = args[3]
    op.observe_call(lens, kv_dtype)
    return op, args, _paged_torch_baseline(op, args, row, page, multi, kv_dtype)


def _paged_torch_baseline(op: Any, args: tuple, row: dict, page: int, multi: bool, kv_dtype: torch.dtype) -> Optional[Callable[[], Any]]:
    """torch on the same device for a paged row: gather the pages each sequence addresses into a dense [B, max_len] cache
    (one ``index_select`` per tensor, on an index tensor built from the block table ahead of the timed call), then
    ``F.scaled_dot_product_attention`` with a padding mask -- the role of the reference benchmark's SDPA baseline
    (benchmarks/ops/attention/bench_gqa_decode_paged.py:21-66) without its per-page host loop.  16-bit caches, one query
    token, no softcap, dense copy of at most 2 GiB; otherwise no baseline."""
    q, k, v, lens, table = args[:5]
    max_len = int(lens.max().item())
    dense_bytes = 2 * q.shape[0] * max_len * k.shape[1] * k.shape[2] * k.element_size()
    if multi or kv_dtype == FP8 or row.get("softcap") or dense_bytes > (2 << 30):
        return None
    import torch.nn.functional as F

    # what depends on the block table and the lengths only is built once, outside the timed call
    t = torch.arange(max_len, device=q.device)
    idx = table.long().gather(1, (t // page).expand(q.shape[0], -1)) * page + t % page  # [B, max_len] physical tokens
    live = t[None, :] < lens[:, None]
    idx = torch.where(live, idx, torch.zeros_like(idx)).reshape(-1)
    mask = live[:, None, None, :]

    def baseline():
        kd = k.index_select(0, idx).view(q.shape[0], max_len, k.shape[1], k.shape[2]).transpose(1, 2)
        vd = v.index_select(0, idx).view(q.shape[0], max_len, v.shape[1], v.shape[2]).transpose(1, 2)
        return F.scaled_dot_product_attention(q.unsqueeze(2), kd, vd, attn_mask=mask, scale=op.sm_scale, enable_gqa=True)

    baseline.tag = "torch_gather_sdpa"
    return baseline


def _contiguous_case(row: dict, dtype: torch.dtype, device: torch.device):
    (batch, heads, dim), (_, n_kv, heads_kv, _) = row["q_shape"], row["kv_shape"]
    kv_dtype = _DT[row.get("kv_dtype", str(dtype).removeprefix("torch."))]
    op = GroupedQueryAttentionDecodeWithKVCacheFwdOp(batch, heads, heads_kv, n_kv, dim, sm_scale=row.get("sm_scale"),
                                                     softcap=row.get("softcap"))
    q = torch.randn(batch, heads, dim, device=device, dtype=dtype)
    k = torch.randn(batch, n_kv, heads_kv, dim, device=device, dtype=dtype)
    v = torch.randn(batch, n_kv, heads_kv, dim, device=device, dtype=dtype)
    baseline = None
    if kv_dtype == FP8:
        k8, ks = quantize_kv_per_token(k.reshape(-1, heads_kv, dim))
        v8, vs = quantize_kv_per_token(v.reshape(-1, heads_kv, dim))
        args = (q, k8.reshape(k.shape), v8.reshape(v.shape), ks.reshape(batch, n_kv, heads_kv), vs.reshape(batch, n_kv, heads_kv))
    else:
        args = (q, k, v)
        if not row.get("softcap"):
            import torch.nn.functional as F
            qb, kb, vb = q.unsqueeze(2), k.transpose(1, 2), v.transpose(1, 2)  # [B,H,1,D], [B,Hkv,N,D]

            def baseline():
                return F.scaled_dot_product_attention(qb, kb, vb, scale=op.sm_scale, enable_gqa=True)
    op.observe_call(n_kv, kv_dtype)
    return op, args, baseline


class _PrefillView:
    """Gives ``eval_roofline`` of a prefill call the per-request lengths of the workload row."""

    def __init__(self, row: dict, dtype: str) -> None:
        self.row, self.dtype = dict(row), dtype

    def eval_roofline(self) -> tuple[int, int]:
        return gqa_prefill_paged_with_kv_cache_fwd_roofline(dtype=self.dtype, **{k: v for k, v in self.row.items() if k not in ("dtypes", "label", "fuse_rope", "max_position", "rotary_dim", "rope_base")})


_VALIDATE_INPUTS = True  # prefill op: the reference's device-reading input checks (host round trips inside the timed call)


def _prefill_case(row: dict, dtype: torch.dtype, device: torch.device):
    batch, heads, heads_kv, dim = row["batch"], row["heads"], row["heads_kv"], row["dim"]
    page, max_pages, max_q = row["page_size"], row["max_pages_per_req"], row["max_seqlen_q"]
    cache_dtype = _DT[row.get("cache_dtype", str(dtype).removeprefix("torch."))]
    q_lens = row.get("q_lens") or _distribute_total(row["total_q"], batch, max_q)
    cache_lens = row.get("cache_lens") or [max(max_pages * page - int(n), 0) for n in q_lens]
    total_q = sum(q_lens)
    op = GroupedQueryAttentionPrefillPagedWithKVCacheFwdOp(
        batch=batch, heads=heads, heads_kv=heads_kv, max_pages_per_req=max_pages, page_size=page, dim=dim,
        is_causal=row.get("is_causal", True), cache_dtype=cache_dtype if cache_dtype == FP8 else None, softcap=row.get("softcap"),
        fuse_rope=bool(row.get("fuse_rope", False)), max_position=row.get("max_position"), rotary_dim=row.get("rotary_dim"),
        validate_inputs=_VALIDATE_INPUTS)
    fp8 = cache_dtype == FP8
    amp = 0.5 if fp8 else 1.0
    q = torch.randn(total_q, heads, dim, device=device, dtype=dtype)
    k_new = (torch.randn(total_q, heads_kv, dim, device=device) * amp).to(dtype)
    v_new = (torch.randn(total_q, heads_kv, dim, device=device) * amp).to(dtype)
    n_phys = row["physical_tokens"]
    scale = torch.tensor([0.02 if fp8 else 1.0], device=device)
    pool = torch.randn(2, n_phys, heads_kv, dim, device=device) * amp
    k_pages = (pool[0] / scale).clamp(-448, 448).to(FP8) if fp8 else pool[0].to(dtype)
    v_pages = (pool[1] / scale).clamp(-448, 448).to(FP8) if fp8 else pool[1].to(dtype)
    del pool
    perm = torch.randperm(n_phys // page, device=device)[:batch * max_pages].to(torch.int32)
    table = perm.reshape(batch, max_pages).contiguous()
    cu = torch.tensor([0, *torch.tensor(q_lens).cumsum(0).tolist()], dtype=torch.int32, device=device)
    cache = torch.tensor(cache_lens, dtype=torch.int32, device=device)
    args = (q, k_new, v_new, k_pages, v_pages, scale, scale.clone(), cu, cache, table, max(q_lens))
    view_row = dict(row, q_lens=q_lens, cache_lens=cache_lens, total_q=total_q)
    op.eval_roofline = _PrefillView(view_row, str(dtype).removeprefix("torch.")).eval_roofline
    return op, args, None


_CASES = {
    "GroupedQueryAttentionDecodePagedWithKVCacheFwdOp": lambda r, d, dev: _paged_case(r, d, dev, False),
    "GroupedQueryAttentionMultiTokenDecodePagedWithKVCacheFwdOp": lambda r, d, dev: _paged_case(r, d, dev, True),
    "GroupedQueryAttentionDecodeWithKVCacheFwdOp": _contiguous_case,
    "GroupedQueryAttentionPrefillPagedWithKVCacheFwdOp": _prefill_case,
}


def main(argv: Optional[list[str]] = None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--op", default=None, help="only this op (class name)")
    ap.add_argument("--label", default=None, help="only workloads whose label contains this")
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--max-kv-gib", type=float, default=8.0, help="skip workloads whose K+V exceed this")
    ap.add_argument("--out", default="manifest_bench_out", help="directory for junit.xml and profile_run.log")
    ap.add_argument("--no-validate", action="store_true",
                    help="prefill op: skip the input checks that read device memory (validate_inputs=False)")
    args = ap.parse_args(argv)
    global _VALIDATE_INPUTS
    _VALIDATE_INPUTS = not args.no_validate
    device = torch.device("cuda", 0)
    native.require_gfx950(device)
    out_dir = Path(args.out)
    out_dir.mkdir(parents=True, exist_ok=True)
    report, flush = BenchmarkReport(), _Flusher(device)
    suite = ET.Element("testsuite", name="tileops_amd.manifest_bench")
    n = 0
    no_baseline: list[str] = []
    for op_name, entry in load_manifest().items():
        if op_name not in _CASES or (args.op and args.op != op_name):
            continue
        for row in entry["workloads"]:
            if args.label and args.label not in row["label"]:
                continue
            for dname in row["dtypes"]:
                dtype = _DT[dname]
                kv_elems = 2
                for s in row.get("kv_shape") or (row["physical_tokens"], row["heads_kv"], row["dim"]):
                    kv_elems *= s
                if kv_elems * 2 / 2**30 > args.max_kv_gib:
                    print(f"skip {op_name} {row['label']} {dname}: K+V of {kv_elems * 2 / 2**30:.1f} GiB", flush=True)
                    continue
                torch.manual_seed(1235)
                op, inputs, baseline = _CASES[op_name](row, dtype, device)
                call = lambda: op(*inputs)  # noqa: E731
                lat = _time(call, flush, args.steps)
                res = _result(op, lat, _device_busy(call))
                kernel = next(iter(op.iter_kernels()), None) if hasattr(op, "iter_kernels") else None
                if "q_shape" in row:
                    params = {"label": row["label"], "q_shape": tuple(row["q_shape"]), "kv_shape": tuple(row["kv_shape"]), "dtype": dname,
                              "kv_dtype": row.get("kv_dtype", dname)}
                else:
                    params = {"label": row["label"], "total_q": row["total_q"], "batch": row["batch"], "heads": row["heads"],
                              "heads_kv": row["heads_kv"], "dim": row["dim"], "dtype": dname, "kv_dtype": row.get("cache_dtype", dname)}
                if "page_size" in row:
                    params["page_size"] = row["page_size"]
                report.record(op_name, params, res, "tileops", getattr(kernel, "config", None))
                entries = [dict(res, tag="tileops", op=op_name, op_module=type(op).__module__)]
                line = f"{op_name[:40]:40s} {row['label']:28s} {dname:9s} {lat * 1e3:9.1f} us  {res['bandwidth_tbs']:.2f} TB/s ({100 * res['hbm_frac']:.1f}%)"
                if baseline is not None:
                    bl = _time(baseline, flush, max(args.steps // 2, 3))
                    flops, nbytes = op.eval_roofline()
                    bres = {"latency_ms": bl, "tflops": flops / bl / 1e9, "bandwidth_tbs": nbytes / bl / 1e9}
                    tag = getattr(baseline, "tag", "torch_sdpa")
                    report.record(op_name, params, bres, tag)
                    entries.append(dict(bres, tag=tag, op=op_name))
                    line += f"   {tag} {bl * 1e3:9.1f} us (x{bl / lat:.2f})"
                else:
                    no_baseline.append(f"{row['label']}-{dname}")
                junit_case(suite, f"{row['label']}-{dname}", entries)
                print(line, flush=True)
                n += 1
                del op, inputs, baseline, call
                torch.cuda.empty_cache()
    write_junit(suite, out_dir / "junit.xml")
    report.dump(out_dir / "profile_run.log")
    if no_baseline:
        print("no device baseline (FP8 cache, several query tokens, softcap or prefill): " + ", ".join(no_baseline))
    print(f"{n} workloads -> {out_dir}/junit.xml, {out_dir}/profile_run.log")
    return 0


if __name__ == "__main__":
    sys.exit(main())
