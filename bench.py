"""Headline benchmark: paged GQA decode on one MI355X.

One "step" = one forward of the op over one batch of synthetic input already resident in HBM.  Prints ONE JSON
line: us/call of the Llama-3-8B-shape bf16 configuration (config 2) with the HBM roofline of its dominant kernel and the
CPU references timed on this box's host cores beside it; ``also`` holds the same blocks for the FP8-KV configuration
(c3), the 8 x 128K-token split-KV configuration (c4) and the eight-query-token configuration (c5).  The four
configurations are workload rows of the op manifest (``load_workloads``); bytes and flops come from the op's
``eval_roofline()`` after it has seen the call.  Exit status 1 if any configuration misses its parity tolerance.

Every configuration is measured in a process of its own (this one only starts them and joins their results): device
memory that has been freed and allocated again inside one process reads 3-5 % slower than a fresh process's first
allocations (measured: the FP8 configurations 99 -> 102 us and 335 -> 352 us after one ``empty_cache()``), and a serving
process allocates its KV pool once, at start-up.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c2|c3|c4|c5] [--also c3,c4,c5] [--no-cpu]
"""

from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0       # MI355X published HBM3E bandwidth
MFMA_PEAK_TFLOPS = 2500.0   # MI355X published dense bf16 matrix rate (the PV product and, for 16-bit caches, QK^T run in bf16)
TRAFFIC_SOURCE = "profiles/hbm_traffic.json"
DRY_RUN_MS = 25.0            # warm-up budget of the reference's timing protocol (benchmarks/timing.py)

DESCRIPTIONS = {
    "c2": "Llama-3-8B-shape paged GQA decode, bf16 KV",
    "c3": "Llama-3-8B-shape paged GQA decode, FP8-e4m3fn KV with per-token scales",
    "c4": "long-context split-KV stress, 8 x 131072 tokens, FP8 KV",
    "c5": "multi-token (speculative verify) decode, 8 query tokens, FP8 KV",
}


def _config(name: str):
    """The configuration as the manifest states it."""
    from tileops_amd.manifest import load_workloads
    from tileops_amd.workloads import BASELINE_WORKLOAD_ROWS, config_from_workload

    op_name, label = BASELINE_WORKLOAD_ROWS[name]
    row = next(r for r in load_workloads(op_name) if r["label"] == label)
    return config_from_workload(row, name, DESCRIPTIONS[name]), op_name, label


def _device_busy_ms(fn, flush, calls: int):
    """Mean over ``calls`` flushed calls of the durations of this library's kernels in one call, from the torch profiler's
    device events: (all kernels, attention kernel, merge kernel) in ms; None when the profiler delivers none."""
    try:
        import torch
        from torch.profiler import ProfilerActivity, profile

        totals, attn, merge = [], [], []
        for i in range(calls):
            flush(i)
            torch.cuda.synchronize()
            with profile(activities=[ProfilerActivity.CUDA]) as prof:
                fn()
                torch.cuda.synchronize()
            evs = [e for e in prof.events() if e.device_type == torch.autograd.DeviceType.CUDA and "mi355" in e.name]
            if not evs:
                return None
            totals.append(sum(e.device_time for e in evs) / 1e3)
            attn.append(sum(e.device_time for e in evs if "combine" not in e.name) / 1e3)
            merge.append(sum(e.device_time for e in evs if "combine" in e.name) / 1e3)
        n = len(totals)
        return sum(totals) / n, sum(attn) / n, sum(merge) / n
    except Exception as exc:  # noqa: BLE001 - optional evidence; the timed figures above do not depend on it
        print(f"device-busy time not measured: {exc!r}", file=sys.stderr)
        return None


def _spread(xs_ms: list[float]) -> dict:
    """min / p10 / median / p90 / max of per-step times, in us."""
    xs = sorted(x * 1e3 for x in xs_ms)
    pick = lambda f: xs[min(len(xs) - 1, max(0, round(f * (len(xs) - 1))))]  # noqa: E731
    return {"min": xs[0], "p10": pick(0.1), "median": statistics.median(xs), "p90": pick(0.9), "max": xs[-1]}


def _timed_steps(fn, flush, steps: int) -> tuple[list[float], float]:
    """``steps`` calls, each after a cache flush and between its own pair of events on the stream the kernels run on."""
    import torch

    starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    stops = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    torch.cuda.synchronize()
    wall0 = time.perf_counter()
    for i in range(steps):
        flush(i)
        starts[i].record()
        fn()
        stops[i].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - wall0
    return [s.elapsed_time(e) for s, e in zip(starts, stops)], wall


def _run_config(name: str, steps: int, warmup: int, with_cpu: bool, kernel_key: str | None) -> dict:
    import torch

    from tileops_amd import ops
    from tileops_amd.roofline import algorithmic_bytes
    from tileops_amd.workloads import gen_paged_inputs

    cfg, op_name, label = _config(name)
    device = torch.device("cuda", 0)
    inp = gen_paged_inputs(cfg, device)
    if cfg.q_len == 1:
        op = ops.GroupedQueryAttentionDecodePagedWithKVCacheFwdOp(cfg.batch, cfg.heads, cfg.heads_kv, cfg.seqlen_kv, cfg.dim, cfg.page_size)
    else:
        op = ops.GroupedQueryAttentionMultiTokenDecodePagedWithKVCacheFwdOp(cfg.batch, cfg.q_len, cfg.heads, cfg.heads_kv, cfg.seqlen_kv,
                                                                            cfg.dim, cfg.page_size)
    assert type(op).__name__ == op_name
    if kernel_key:
        op.kernel_map = {kernel_key: op.kernel_map[kernel_key]}
    args = inp.as_args()
    # Between steps a 512 MiB buffer is overwritten and a second 512 MiB buffer is read: the write evicts L2 and
    # the 256 MB Infinity Cache, the read pushes the dirty lines out again so the timed call starts on a clean,
    # cold cache and every K/V byte comes from HBM.
    flush_wr = torch.empty(512 << 20, dtype=torch.uint8, device=device)
    flush_rd = torch.ones(128 << 20, dtype=torch.int32, device=device)

    def flush(i: int) -> None:
        flush_wr.fill_(i & 0xFF)
        flush_rd.max()

    for i in range(max(warmup, 1)):  # the flush kernels are part of what has to be warm
        flush(i)
        out = op(*args)
    torch.cuda.synchronize()
    # The W calls asked for are followed by the dry-run phase of the reference's own timing protocol
    # (benchmarks/timing.py:527-585): as many flushed calls as fit 25 ms, at least 10 and at most 200, counted from one
    # calibration pass, the calls above included.  After idle the device runs its first tens of milliseconds slower (the
    # FP8 configuration reads 100.5 us/call over twenty calls timed after five, 98.8 after the dry run), so without it a
    # short run reports the ramp rather than the call.  Untimed, like the W calls; the timed region below is exactly K steps.
    t0 = time.perf_counter()
    for i in range(3):
        flush(i)
        op(*args)
    torch.cuda.synchronize()
    per_iter_ms = max((time.perf_counter() - t0) * 1e3 / 3, 1e-3)
    warm_calls = max(warmup, 1) + 3
    for i in range(max(min(max(int(DRY_RUN_MS / per_iter_ms), 10), 200) - warm_calls, 0)):
        flush(i)
        op(*args)
        warm_calls += 1
    torch.cuda.synchronize()
    per_step_ms, wall = _timed_steps(lambda: op(*args), flush, steps)
    ms = sum(per_step_ms) / steps
    ms_median = statistics.median(per_step_ms)
    # What the timer reads with nothing between its two records (same flush before): 4-5 us on this stack.  It is NOT a
    # constant to subtract -- with kernels between the records the pair reads only 1-3 us more than the profiler's sum of
    # the kernels' durations -- but it is the floor under every event-timed call, and most of a very small call's time.
    empty_ms, _ = _timed_steps(lambda: None, flush, max(steps, 30))
    tare_ms = statistics.median(empty_ms)
    # the same K calls back to back (no flush) for reference
    s0, s1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s0.record()
    for _ in range(steps):
        op(*args)
    s1.record()
    torch.cuda.synchronize()
    b2b_ms = s0.elapsed_time(s1) / steps

    # The dominant (attention) kernel alone: launches that skip the merge of partial results.  The roofline figure is the
    # cold one -- ONE launch per event pair, each after a cache flush, as a caller's launch finds the chip.  Beside it, for
    # reference only, KREP launches back to back per event pair (warm address translation and metadata: 3-5 % kinder).
    kernel = next(iter(next(iter(op._kernel_roles.values())).values()))
    kernel.attention_kernel_only = True
    k_cold_ms, _ = _timed_steps(lambda: op(*args), flush, steps)
    kernel_ms = sum(k_cold_ms) / steps
    KREP = 4

    def attention_only() -> None:
        for _ in range(KREP):
            op(*args)

    k_b2b_ms, _ = _timed_steps(attention_only, flush, steps)
    kernel.attention_kernel_only = False
    kernel_b2b_ms = sum(k_b2b_ms) / (steps * KREP)
    out = op(*args)  # complete output again for the parity check below
    torch.cuda.synchronize()

    # a whole call captured once in a HIP graph and replayed (what a serving loop does): no host launch gaps
    graph_ms = graph_median_ms = graph8_ms = None
    if hasattr(op, "capture"):
        replay = op.capture(*args)
        for _ in range(3):
            replay()
        g_ms, _ = _timed_steps(replay, flush, steps)
        graph_ms, graph_median_ms = sum(g_ms) / steps, statistics.median(g_ms)
        torch.cuda.synchronize()
        # A serving loop's graph holds a whole model step, not one call: eight calls in ONE graph, replayed back to back, per
        # call -- to be read against us_per_call_back_to_back (eager, also without flushes).  What a graph costs per LAUNCH
        # (not per node) drops out of this figure and stays in the one-call figure above.
        many = torch.cuda.CUDAGraph()
        with torch.cuda.graph(many):
            for _ in range(8):
                op(*args)
        for _ in range(2):
            many.replay()
        s0.record()
        for _ in range(max(steps // 4, 3)):
            many.replay()
        s1.record()
        torch.cuda.synchronize()
        graph8_ms = s0.elapsed_time(s1) / (max(steps // 4, 3) * 8)
        del many

    # Device-busy time of a whole call: the sum of the durations of the kernels it launches (attention + merge), launch
    # latency and gaps excluded -- the quantity the reference's own timing protocol reports (its benchmarks take the
    # per-iteration device-busy time from the profiler, benchmarks/timing.py:527-585).  Ten flushed calls.
    busy = _device_busy_ms(lambda: op(*args), flush, max(steps, 10))

    op.observe_call(inp.real_seqlen_kv, cfg.kv_dtype)
    flops, total_bytes = op.eval_roofline()
    lens = inp.real_seqlen_kv.cpu().to(torch.int64)
    sum_len = int(lens.sum())
    sum_pages = int(((lens + cfg.page_size - 1) // cfg.page_size).sum())
    fp8 = cfg.kv_dtype == torch.float8_e4m3fn
    b = algorithmic_bytes(sum_len=sum_len, sum_pages=sum_pages, batch=cfg.batch, q_len=cfg.q_len, heads=cfg.heads, heads_kv=cfg.heads_kv,
                          dim=cfg.dim, q_bytes=2, kv_bytes=1 if fp8 else 2, fp8_scales=fp8)
    assert b["total"] == total_bytes
    kv_read = b["kv"] + b["scales"]
    achieved = total_bytes / (kernel_ms * 1e-3) / 1e9
    traffic = None
    try:  # measured with hardware counters in a separate profiler run (not in this run); absent for configurations not profiled
        traffic = json.loads((ROOT / TRAFFIC_SOURCE).read_text()).get(name, {}).get("traffic_bytes")
    except (OSError, ValueError):
        pass

    def gbs(nbytes: int, t_ms: float) -> float:
        return nbytes / (t_ms * 1e-3) / 1e9

    res = {
        "workload": f"{name} = manifest row '{label}': {cfg.description}; batch {cfg.batch}, q_len {cfg.q_len}, {cfg.heads}q/{cfg.heads_kv}kv heads, "
                    f"dim {cfg.dim}, page {cfg.page_size}, len in {list(cfg.len_range)}, {cfg.n_pages}-page pool, seed {cfg.seed}",
        "kernel": type(kernel).__name__,
        "us_per_call": ms * 1e3,
        "us_per_call_median": ms_median * 1e3,
        "us_per_call_back_to_back": b2b_ms * 1e3,
        "sum_len": sum_len,
        "decode_tokens_per_s": cfg.batch * cfg.q_len / (ms * 1e-3),
        "kv_tokens_per_s": sum_len / (ms * 1e-3),
        "algorithmic_bytes": b,
        "flops": flops,
        # the whole call (attention kernel, merge of partial results where one is launched, launch gaps): mean and median of the
        # flushed steps, on the K/V (+ scale) bytes alone -- the figure the 70 % target is stated on -- and on all bytes
        "whole_call": {
            "us_mean": ms * 1e3, "us_median": ms_median * 1e3, "us_spread": _spread(per_step_ms),
            "kv_read_gbs_mean": gbs(kv_read, ms), "kv_read_gbs_median": gbs(kv_read, ms_median),
            "kv_read_frac_of_peak_mean": gbs(kv_read, ms) / HBM_PEAK_GBS, "kv_read_frac_of_peak_median": gbs(kv_read, ms_median) / HBM_PEAK_GBS,
            "all_bytes_frac_of_peak_mean": gbs(total_bytes, ms) / HBM_PEAK_GBS,
            "event_pair_reads_when_empty_us": tare_ms * 1e3,
            "untimed_calls_before_the_timed_steps": warm_calls,
        },
        # the attention kernel alone, cold: one launch per HIP-event pair, each after a cache flush (mean of the steps)
        "attention_kernel_us": kernel_ms * 1e3,
        "attention_kernel_us_spread": _spread(k_cold_ms),
        # the same kernel launched four times back to back per event pair (warm translation and metadata), for reference
        "attention_kernel_us_back_to_back_x4": kernel_b2b_ms * 1e3,
        "frac_back_to_back_x4": total_bytes / (kernel_b2b_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
        # dominant kernel alone: algorithmic bytes of one launch / its own cold duration (HIP events around the one launch)
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                     "timer": "one HIP-event pair around one cold launch", "traffic": traffic, "traffic_source": f"{TRAFFIC_SOURCE} (rocprofv3 FETCH_SIZE/WRITE_SIZE of an earlier profiler run, not counted in this run)"},
        "wall_s_timed_region": wall,
    }
    if busy is not None and busy[1] < 0.5 * kernel_ms:
        busy = None  # (under an outer profiler the inner one's durations are meaningless: leave them out)
    if busy is not None:
        busy_ms, busy_attn_ms, busy_merge_ms = busy
        # The roofline figure: the attention kernel's own begin/end timestamps of cold dispatches, taken in this run through
        # the profiler (the clock rocprofv3's kernel trace reads).  An event pair around the same single launch reads 1-4 us
        # more (the pair's own cost): that figure stays beside it.
        r = res["roofline"]
        r.update({"achieved_hip_events": r["achieved"], "frac_hip_events": r["frac"],
                  "achieved": total_bytes / (busy_attn_ms * 1e-3) / 1e9, "frac": total_bytes / (busy_attn_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                  "timer": "kernel begin/end timestamps of cold dispatches (torch.profiler device events, this run); *_hip_events: one HIP-event pair around one cold launch"})
        res["whole_call"].update({"us_device_busy_mean": busy_ms * 1e3, "kv_read_frac_of_peak_device_busy": gbs(kv_read, busy_ms) / HBM_PEAK_GBS})
        # the profiler's own durations of the two kernels of a flushed call (no event pair involved)
        res["profiler"] = {"attention_kernel_us": busy_attn_ms * 1e3, "merge_kernel_us": busy_merge_ms * 1e3,
                           "attention_kernel_frac": total_bytes / (busy_attn_ms * 1e-3) / 1e9 / HBM_PEAK_GBS if busy_attn_ms else None}
    if graph_ms is not None:
        res["whole_call"].update({
            "us_graph_mean": graph_ms * 1e3, "us_graph_median": graph_median_ms * 1e3,
            "kv_read_frac_of_peak_graph_mean": gbs(kv_read, graph_ms) / HBM_PEAK_GBS,
            "kv_read_frac_of_peak_graph_median": gbs(kv_read, graph_median_ms) / HBM_PEAK_GBS,
            "us_per_call_in_a_graph_of_8_back_to_back": graph8_ms * 1e3,
        })
    if cfg.q_len * (cfg.heads // cfg.heads_kv) >= 16:
        # enough query rows per kv head for the products to be dense matrix work: report the matrix rate beside the bandwidth
        tf = flops / ((busy[1] if busy is not None else kernel_ms) * 1e-3) / 1e12  # (same clock as the roofline figure)
        from tileops_amd.perf import load_profile

        eff = load_profile("mi355x")["matrix"]["bf16"]["effective_tflops"]  # what a pure matrix-instruction stream sustains (probe)
        res["mfma"] = {"flops": flops, "achieved_tflops": tf, "peak_tflops": MFMA_PEAK_TFLOPS, "frac_of_2500": tf / MFMA_PEAK_TFLOPS,
                       "calibrated_peak_tflops": eff, "frac_of_calibrated": tf / eff}
    if with_cpu:
        from oracle.paged_gqa_decode_ref import ref_paged_gqa_decode, ref_paged_gqa_decode_sdpa_math

        host = inp.to("cpu")
        threads = os.cpu_count() or 1
        torch.set_num_threads(threads)
        kw = dict(page_size=cfg.page_size, k_scale=host.k_scale, v_scale=host.v_scale)
        # bounded sample: as many leading sequences as take roughly 6 s, timed 3 times (median)
        t0 = time.perf_counter()
        ref_paged_gqa_decode(host.q[:1], host.k, host.v, host.real_seqlen_kv[:1], host.block_table[:1], **kw)
        one = time.perf_counter() - t0
        n_seq = max(1, min(cfg.batch, int(6.0 / max(one, 1e-3))))
        times = []
        for _ in range(3):
            t0 = time.perf_counter()
            ref = ref_paged_gqa_decode(host.q[:n_seq], host.k, host.v, host.real_seqlen_kv[:n_seq], host.block_table[:n_seq], **kw)
            times.append(time.perf_counter() - t0)
        sample_len = int(lens[:n_seq].sum())
        scale_up = sum_len / sample_len
        cpu_s = statistics.median(times) * scale_up  # scaled to the whole batch by tokens
        t0 = time.perf_counter()
        ref_sdpa = ref_paged_gqa_decode_sdpa_math(host.q[:n_seq], host.k, host.v, host.real_seqlen_kv[:n_seq], host.block_table[:n_seq], **kw)
        sdpa_s = (time.perf_counter() - t0) * scale_up
        tol = 3e-2 if fp8 else 2e-2
        got = out[:n_seq].float().cpu()
        err = (got - ref.float()).abs().max().item()
        ok = torch.allclose(got, ref.float(), atol=tol, rtol=tol) and torch.allclose(got, ref_sdpa.float(), atol=tol, rtol=tol)
        sample = f"the first {n_seq} of {cfg.batch} sequences ({sample_len} of {sum_len} KV tokens), scaled by tokens to the whole batch"
        res["cpu_baseline"] = {"value": cpu_s * 1e6, "unit": "us/call", "cores": torch.get_num_threads(), "kind": "port",
                               "sample": f"torch fp32 oracle (gather pages, dequantise, grouped einsum softmax) on {sample}, median of 3 runs"}
        res["cpu_baseline_sdpa_math"] = {"value": sdpa_s * 1e6, "unit": "us/call", "cores": torch.get_num_threads(), "kind": "port",
                                         "sample": f"F.scaled_dot_product_attention under sdpa_kernel(MATH), fp32, heads expanded by indexing "
                                                   f"(the torch baseline of the reference's own benchmark) on {sample}, one run"}
        res["parity"] = {"max_abs_err": err, "tolerance": tol, "within_tolerance": bool(ok), "sequences_checked": n_seq}
    del inp, args, flush_wr, flush_rd
    torch.cuda.empty_cache()
    return res


def _measure_here(name: str, a) -> dict:
    import torch

    from tileops_amd import native

    native.require_gfx950(torch.device("cuda", 0))
    return _run_config(name, a.steps, a.warmup, not a.no_cpu, a.kernel)


def _measure_in_child(name: str, a) -> dict:
    """One configuration in a process of its own.  This process has not touched the GPU (it imports no torch), so the
    child is an ordinary fresh program; its stderr passes through, its last stdout line is the result."""
    import subprocess

    cmd = [sys.executable, str(Path(__file__).resolve()), "--child", name, "--steps", str(a.steps), "--warmup", str(a.warmup)]
    if a.no_cpu:
        cmd.append("--no-cpu")
    if a.kernel:
        cmd += ["--kernel", a.kernel]
    done = subprocess.run(cmd, stdout=subprocess.PIPE, text=True)
    lines = [ln for ln in done.stdout.splitlines() if ln.startswith("{")]
    if done.returncode != 0 or not lines:
        sys.exit(f"measuring {name} failed (exit status {done.returncode}): {done.stdout[-2000:]}")
    return json.loads(lines[-1])


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--config", default="c2", choices=["c2", "c3", "c4", "c5"])
    ap.add_argument("--also", default="c3,c4,c5", help="comma-separated extra configurations reported under 'also' ('' for none)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU reference legs (and with them the parity check)")
    ap.add_argument("--kernel", default=None, choices=[None, "gqa_decode_paged_kernel", "gqa_decode_paged_mfma_kernel"])
    ap.add_argument("--in-process", action="store_true",
                    help="measure every configuration in this process, one after the other (their pools then land in memory that "
                         "was freed and allocated again: 3-5 %% slower from the second configuration on)")
    ap.add_argument("--child", default=None, choices=["c2", "c3", "c4", "c5"], help=argparse.SUPPRESS)
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run three plain 1 GiB device copies, so a hardware-counter pass has a kernel of known traffic to scale by")
    a = ap.parse_args()
    if a.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py measures one GPU: the path is single-GPU by construction (every (sequence, kv-head) is independent); "
                 "run with --gpus 1")
    names = [a.config] + [n for n in a.also.split(",") if n and n != a.config]
    if a.child:
        # one configuration, in this process; the result goes to the parent as one JSON line
        print(json.dumps(_measure_here(a.child, a)))
        return
    if len(names) == 1 or a.in_process:
        results = [_measure_here(n, a) for n in names]  # (a profiler run names one configuration and lands here)
    else:
        results = [_measure_in_child(n, a) for n in names]
    main_res, also = results[0], results[1:]
    fp8 = a.config != "c2"
    line = {
        "metric": "GQA paged-decode us/call (achieved HBM GB/s and fraction of the 8 TB/s peak under 'roofline')",
        "value": main_res["us_per_call"], "unit": "us/call", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": main_res["us_per_call"] / 1e3, "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp8_e4m3fn KV / bf16 Q, fp32 accumulate" if fp8 else "bf16",
        "data": "synthetic", "config": {"workload": main_res["workload"], "kernel": main_res["kernel"],
                                        "process": "one per configuration" if len(names) > 1 and not a.in_process else "this one"},
        "roofline": main_res["roofline"],
        "warmup_protocol": f"the {a.warmup} calls asked for, then the reference protocol's dry run (flushed calls for {DRY_RUN_MS:.0f} ms, 10 to 200): "
                           f"{main_res['whole_call']['untimed_calls_before_the_timed_steps']} untimed calls in all before the {a.steps} timed steps",
    }
    for key in ("cpu_baseline", "cpu_baseline_sdpa_math", "parity", "mfma"):
        if key in main_res:
            line[key] = main_res[key]
    line["detail"] = {k: v for k, v in main_res.items() if k not in ("roofline", "cpu_baseline", "cpu_baseline_sdpa_math", "parity", "mfma", "workload")}
    line["also"] = also
    if a.copy_calibration and (len(names) == 1 or a.in_process):
        import torch

        src = torch.ones(1 << 28, dtype=torch.int32, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        line["copy_calibration"] = {"bytes_read": src.numel() * 4, "bytes_written": dst.numel() * 4, "launches": 3}
    print(json.dumps(line))
    failed = [r["workload"].split(" ")[0] for r in [main_res, *also] if "parity" in r and not r["parity"]["within_tolerance"]]
    if failed:
        sys.exit(f"parity outside tolerance for {', '.join(failed)}")


if __name__ == "__main__":
    main()
