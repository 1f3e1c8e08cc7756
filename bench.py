"""Headline benchmark: paged GQA decode on one MI355X.

One "step" = one forward of the op over one batch of synthetic input already resident in HBM.  Prints ONE JSON
line: us/call of the Llama-3-8B-shape bf16 configuration (BASELINE config 2) with the HBM roofline of the call,
the CPU oracle timed on this box's host cores beside it, and (in ``also``) the FP8-KV configuration.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c2|c3|c4|c5] [--also c3,...] [--no-cpu]
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

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth


def _run_config(name: str, steps: int, warmup: int, with_cpu: bool, kernel_key: str | None) -> dict:
    import torch

    from tileops_amd import ops
    from tileops_amd.roofline import algorithmic_bytes, algorithmic_flops
    from tileops_amd.workloads import BASELINE_CONFIGS, gen_paged_inputs

    cfg = BASELINE_CONFIGS[name]
    device = torch.device("cuda", 0)
    inp = gen_paged_inputs(cfg, device)
    if cfg.q_len == 1:
        op = ops.GroupedQueryAttentionDecodePagedWithKVCacheFwdOp(cfg.batch, cfg.heads, cfg.heads_kv, cfg.seqlen_kv, cfg.dim, cfg.page_size)
    else:
        op = ops.GroupedQueryAttentionMultiTokenDecodePagedWithKVCacheFwdOp(cfg.batch, cfg.q_len, cfg.heads, cfg.heads_kv, cfg.seqlen_kv,
                                                                            cfg.dim, cfg.page_size)
    if kernel_key:
        op.kernel_map = {kernel_key: op.kernel_map[kernel_key]}
    args = inp.as_args()
    # Between steps a 512 MiB buffer is overwritten and a second 512 MiB buffer is read: the write evicts L2 and
    # the 256 MB Infinity Cache, the read pushes the dirty lines out again so the timed call starts on a clean,
    # cold cache and every K/V byte comes from HBM.
    flush = torch.empty(512 << 20, dtype=torch.uint8, device=device)
    flush_rd = torch.ones(128 << 20, dtype=torch.int32, device=device)
    for _ in range(max(warmup, 1)):
        out = op(*args)
    torch.cuda.synchronize()
    # timed region: exactly `steps` calls, each bracketed by events on the stream the kernels run on
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    stops = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    torch.cuda.synchronize()
    wall0 = time.perf_counter()
    for i in range(steps):
        flush.fill_(i & 0xFF)
        flush_rd.max()
        starts[i].record()
        out = op(*args)
        stops[i].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - wall0
    per_step_ms = [s.elapsed_time(e) for s, e in zip(starts, stops)]
    ms = sum(per_step_ms) / steps
    # the same K calls back to back (no flush) for reference
    s0, s1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s0.record()
    for _ in range(steps):
        op(*args)
    s1.record()
    torch.cuda.synchronize()
    b2b_ms = s0.elapsed_time(s1) / steps

    # The dominant (attention) kernel alone: launches that skip the combine kernel, KREP back to back per event
    # pair so that the few microseconds an event pair costs are spread over KREP launches.  Each launch streams
    # far more than the 256 MB Infinity Cache holds, so a launch finds next to nothing of its predecessor cached.
    KREP = 4
    kernel = next(iter(next(iter(op._kernel_roles.values())).values()))
    kernel.attention_kernel_only = True
    k_starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    k_stops = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    for i in range(steps):
        flush.fill_(i & 0xFF)
        flush_rd.max()
        k_starts[i].record()
        for _ in range(KREP):
            op(*args)
        k_stops[i].record()
    torch.cuda.synchronize()
    kernel.attention_kernel_only = False
    kernel_ms = sum(s.elapsed_time(e) for s, e in zip(k_starts, k_stops)) / (steps * KREP)
    out = op(*args)  # complete output again for the parity check below

    lens = inp.real_seqlen_kv.cpu().to(torch.int64)
    sum_len = int(lens.sum())
    sum_pages = int(((lens + cfg.page_size - 1) // cfg.page_size).sum())
    fp8 = cfg.kv_dtype == torch.float8_e4m3fn
    b = algorithmic_bytes(sum_len=sum_len, sum_pages=sum_pages, batch=cfg.batch, q_len=cfg.q_len, heads=cfg.heads, heads_kv=cfg.heads_kv,
                          dim=cfg.dim, q_bytes=2, kv_bytes=1 if fp8 else 2, fp8_scales=fp8)
    flops = algorithmic_flops(sum_len=sum_len, q_len=cfg.q_len, heads=cfg.heads, dim=cfg.dim)
    achieved = b["total"] / (kernel_ms * 1e-3) / 1e9
    traffic = None
    try:  # measured with hardware counters in a separate profiler run; absent for configurations not profiled
        traffic = json.loads((ROOT / "profiles" / "hbm_traffic.json").read_text()).get(name, {}).get("traffic_bytes")
    except (OSError, ValueError):
        pass
    res = {
        "workload": f"{name}: {cfg.description}; batch {cfg.batch}, q_len {cfg.q_len}, {cfg.heads}q/{cfg.heads_kv}kv heads, dim {cfg.dim}, "
                    f"page {cfg.page_size}, len in {list(cfg.len_range)}, {cfg.n_pages}-page pool, seed {cfg.seed}",
        "kernel": type(kernel).__name__,
        "us_per_call": ms * 1e3,
        "us_per_call_median": statistics.median(per_step_ms) * 1e3,
        "us_per_call_back_to_back": b2b_ms * 1e3,
        "sum_len": sum_len,
        "decode_tokens_per_s": cfg.batch * cfg.q_len / (ms * 1e-3),
        "kv_tokens_per_s": sum_len / (ms * 1e-3),
        "algorithmic_bytes": b,
        "flops": flops,
        "kv_read_gbs": (b["kv"] + b["scales"]) / (ms * 1e-3) / 1e9,
        "attention_kernel_us": kernel_ms * 1e3,
        "whole_call_gbs": b["total"] / (ms * 1e-3) / 1e9,
        "whole_call_frac_of_peak": b["total"] / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
        # dominant kernel: algorithmic bytes of one launch / its own duration (events around the attention kernel alone)
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                     "traffic": traffic},
        "wall_s_timed_region": wall,
    }
    if with_cpu:
        from oracle.paged_gqa_decode_ref import ref_paged_gqa_decode

        host = inp.to("cpu")
        threads = os.cpu_count() or 1
        torch.set_num_threads(threads)
        kw = dict(page_size=cfg.page_size, k_scale=host.k_scale, v_scale=host.v_scale)
        # bounded sample: as many leading sequences as take roughly 10 s, timed 3 times (median)
        t0 = time.perf_counter()
        ref_paged_gqa_decode(host.q[:1], host.k, host.v, host.real_seqlen_kv[:1], host.block_table[:1], **kw)
        one = time.perf_counter() - t0
        n_seq = max(1, min(cfg.batch, int(10.0 / max(one, 1e-3))))
        times = []
        for _ in range(3):
            t0 = time.perf_counter()
            ref = ref_paged_gqa_decode(host.q[:n_seq], host.k, host.v, host.real_seqlen_kv[:n_seq], host.block_table[:n_seq], **kw)
            times.append(time.perf_counter() - t0)
        sample_len = int(lens[:n_seq].sum())
        cpu_s = statistics.median(times) * (sum_len / sample_len)  # scaled to the whole batch by tokens
        tol = 3e-2 if fp8 else 2e-2
        err = (out[:n_seq].float().cpu() - ref.float()).abs().max().item()
        ok = torch.allclose(out[:n_seq].float().cpu(), ref.float(), atol=tol, rtol=tol)
        res["cpu_baseline"] = {"value": cpu_s * 1e6, "unit": "us/call", "cores": torch.get_num_threads(), "kind": "port",
                               "sample": f"torch fp32 oracle on the first {n_seq} of {cfg.batch} sequences ({sample_len} of {sum_len} KV tokens), "
                                         f"median of 3 runs, scaled by tokens to the whole batch"}
        res["parity"] = {"max_abs_err": err, "tolerance": tol, "within_tolerance": bool(ok), "sequences_checked": n_seq}
    del inp, args, flush, flush_rd
    torch.cuda.empty_cache()
    return res


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--config", default="c2", choices=["c2", "c3", "c4", "c5"])
    ap.add_argument("--also", default="c3", help="comma-separated extra configurations reported under 'also' ('' for none)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU oracle leg")
    ap.add_argument("--kernel", default=None, choices=[None, "gqa_decode_paged_kernel", "gqa_decode_paged_mfma_kernel"])
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run three plain 1 GiB device copies, so a hardware-counter pass has a kernel of known traffic to scale by")
    a = ap.parse_args()
    if a.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py measures one GPU: the path is single-GPU by construction (every (sequence, kv-head) is independent); "
                 "run with --gpus 1")
    import torch

    from tileops_amd import native

    native.require_gfx950(torch.device("cuda", 0))
    main_res = _run_config(a.config, a.steps, a.warmup, not a.no_cpu, a.kernel)
    also = [_run_config(n, a.steps, a.warmup, not a.no_cpu, a.kernel) for n in a.also.split(",") if n and n != a.config]
    fp8 = "fp8" in main_res["workload"].lower() and a.config != "c2"
    line = {
        "metric": "GQA paged-decode us/call (achieved HBM GB/s and fraction of the 8 TB/s peak under 'roofline')",
        "value": main_res["us_per_call"], "unit": "us/call", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": main_res["us_per_call"] / 1e3, "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp8_e4m3fn KV / bf16 Q, fp32 accumulate" if fp8 else "bf16",
        "data": "synthetic", "config": {"workload": main_res["workload"], "kernel": main_res["kernel"]},
        "roofline": main_res["roofline"],
    }
    if "cpu_baseline" in main_res:
        line["cpu_baseline"] = main_res["cpu_baseline"]
        line["parity"] = main_res["parity"]
    line["detail"] = {k: v for k, v in main_res.items() if k not in ("roofline", "cpu_baseline", "parity", "workload")}
    line["also"] = also
    if a.copy_calibration:
        src = torch.ones(1 << 28, dtype=torch.int32, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        line["copy_calibration"] = {"bytes_read": src.numel() * 4, "bytes_written": dst.numel() * 4, "launches": 3}
    print(json.dumps(line))


if __name__ == "__main__":
    main()
