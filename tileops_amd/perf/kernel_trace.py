"""Kernel-trace companions of the benchmark: what ``rocprofv3 --kernel-trace`` says about this library's kernels.

Two jobs, both offline readers of a ``rocprofv3 --kernel-trace --output-format csv -d DIR -- <program>`` output directory:

``python -m tileops_amd.perf.kernel_trace summary DIR``
    Per kernel of the library: calls, average / minimum / maximum duration, launch geometry and registers, with every
    dispatch put into one of two classes by the kernel that ran just before it on the device -- *cold* (the predecessor is
    one of the benchmark's cache-flush kernels, a fill or a reduction over 512 MiB: the launch finds caches and address
    translation as a caller's launch finds them) or *warm* (the predecessor is another kernel of this library: back-to-back
    launches, graph replays of several calls).  The roofline figure of ``bench.py`` is the cold one.

``python -m tileops_amd.perf.kernel_trace replay CONFIG`` (to be run *under* the profiler) and
``python -m tileops_amd.perf.kernel_trace replay-summary DIR``
    Eager calls against HIP-graph replays of the same call, phase by phase (eager flushed, one-call graph flushed, eager
    back to back, a graph of eight calls), separated in the trace by marker kernels: kernel durations per phase, so that
    what a graph replay costs can be attributed to the kernels (inside the library) or to what lies between the host's
    launch and the first kernel (the runtime's graph launch).

The profiler serialises dispatches, so a kernel's recorded start follows its predecessor's end without a gap and its
duration includes what the command processor spends dispatching it.
"""

from __future__ import annotations

import csv
import statistics
import sys
from pathlib import Path

#: torch kernels the benchmark's flush launches (a fill over 512 MiB, a max-reduction over 512 MiB)
_FLUSH_MARKS = ("reduce_kernel", "fillBuffer", "FillFunctor")
_PHASES = {1: "eager, flushed", 2: "graph replay of one call, flushed", 3: "eager, back to back", 4: "graph of eight calls, back to back"}
_PHASE_MARKERS = ("cos_kernel_cuda", "sin_kernel_cuda", "tanh_kernel_cuda", "exp_kernel_cuda", "AbsFunctor<float>")  # elementwise kernels on 64 floats


def _rows(out_dir: str) -> list[dict]:
    files = sorted(Path(out_dir).rglob("*kernel_trace.csv"))
    if not files:
        sys.exit(f"no *kernel_trace.csv under {out_dir}")
    rows = [r for f in files for r in csv.DictReader(f.open())]
    rows.sort(key=lambda r: int(r["Start_Timestamp"]))
    return rows


def _short(name: str) -> str:
    name = name.replace("void mi355::(anonymous namespace)::", "").replace("mi355::", "").replace("_tag", "")
    return name.split("(")[0]


def summary(out_dir: str) -> str:
    rows = _rows(out_dir)
    stats: dict[tuple[str, str], list[float]] = {}
    meta: dict[str, dict] = {}
    prev = ""
    for r in rows:
        name = r["Kernel_Name"]
        if "mi355" in name:
            cls = "cold" if any(m in prev for m in _FLUSH_MARKS) else ("warm" if "mi355" in prev else "other")
            stats.setdefault((_short(name), cls), []).append((int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3)
            meta[_short(name)] = r
        prev = name
    lines = ["| kernel | follows | calls | avg us | min us | max us | grid (threads) | workgroup | VGPR | AGPR |",
             "|---|---|---:|---:|---:|---:|---:|---:|---:|---:|"]
    for (name, cls), d in sorted(stats.items()):
        r = meta[name]
        grid = int(r["Grid_Size_X"]) * int(r["Grid_Size_Y"]) * int(r["Grid_Size_Z"])
        follows = {"cold": "a cache flush (cold)", "warm": "a kernel of the library (warm)", "other": "another kernel"}[cls]
        lines.append(f"| `{name}` | {follows} | {len(d)} | {statistics.mean(d):.2f} | {min(d):.2f} | {max(d):.2f} | {grid} | "
                     f"{r['Workgroup_Size_X']} | {r['VGPR_Count']} | {r['Accum_VGPR_Count']} |")
    return "\n".join(lines)


def replay_run(config: str) -> None:
    """The program to put after ``rocprofv3 --kernel-trace ... --``: phases of eager calls and graph replays."""
    import torch

    from .. import ops
    from ..workloads import BASELINE_CONFIGS, gen_paged_inputs

    cfg = BASELINE_CONFIGS[config]
    dev = torch.device("cuda", 0)
    inp = gen_paged_inputs(cfg, dev)
    if cfg.q_len == 1:
        op = ops.GroupedQueryAttentionDecodePagedWithKVCacheFwdOp(cfg.batch, cfg.heads, cfg.heads_kv, cfg.seqlen_kv, cfg.dim, cfg.page_size)
    else:
        op = ops.GroupedQueryAttentionMultiTokenDecodePagedWithKVCacheFwdOp(cfg.batch, cfg.q_len, cfg.heads, cfg.heads_kv, cfg.seqlen_kv,
                                                                            cfg.dim, cfg.page_size)
    args = inp.as_args()
    fill = torch.empty(512 << 20, dtype=torch.uint8, device=dev)
    read = torch.ones(128 << 20, dtype=torch.int32, device=dev)
    mark = torch.zeros(64, device=dev)

    def flush(i: int) -> None:
        fill.fill_(i & 255)
        read.max()

    for i in range(5):
        flush(i)
        op(*args)
    replay = op.capture(*args)
    many = torch.cuda.CUDAGraph()
    with torch.cuda.graph(many):
        for _ in range(8):
            op(*args)
    for i in range(3):
        flush(i)
        replay()
    many.replay()
    torch.cuda.synchronize()
    n = 20
    mark.cos_()  # phase 1
    for i in range(n):
        flush(i)
        op(*args)
    torch.cuda.synchronize()
    mark.sin_()  # phase 2
    for i in range(n):
        flush(i)
        replay()
    torch.cuda.synchronize()
    mark.tanh_()  # phase 3
    for _ in range(16):
        op(*args)
    torch.cuda.synchronize()
    mark.exp_()  # phase 4
    many.replay()
    many.replay()
    torch.cuda.synchronize()
    mark.abs_()
    torch.cuda.synchronize()


def replay_summary(out_dir: str) -> str:
    rows = _rows(out_dir)
    phase, durs = 0, {}
    for r in rows:
        name = r["Kernel_Name"]
        hit = [i for i, m in enumerate(_PHASE_MARKERS) if m in name and int(r["Grid_Size_X"]) <= 1024]
        if hit:
            phase = hit[0] + 1
            continue
        if "mi355" in name and phase in _PHASES:
            kind = "merge" if "combine" in name else "attention"
            durs.setdefault((phase, kind), []).append((int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3)
    lines = ["| phase | kernel | dispatches | avg us | median us |", "|---|---|---:|---:|---:|"]
    for (ph, kind), d in sorted(durs.items()):
        lines.append(f"| {_PHASES[ph]} | {kind} | {len(d)} | {statistics.mean(d):.2f} | {statistics.median(d):.2f} |")
    return "\n".join(lines)


def main(argv: list[str]) -> int:
    if len(argv) == 2 and argv[0] == "summary":
        print(summary(argv[1]))
    elif len(argv) == 2 and argv[0] == "replay":
        replay_run(argv[1])
    elif len(argv) == 2 and argv[0] == "replay-summary":
        print(replay_summary(argv[1]))
    else:
        sys.exit(__doc__)
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
