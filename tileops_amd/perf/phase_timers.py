"""Per-wave phase timers of the MFMA decode kernel: where a wave's time goes, and when each XCD finishes.

Builds an instrumented copy of the library (``-DMI355_PHASE_TIMERS``) next to the product one, runs one of the
baseline configurations with cold caches and prints, over all waves of the attention kernel:

* cycles spent issuing direct-to-LDS loads (includes the stall when the memory system pushes back), waiting for
  data, computing, and in per-sequence work (query loads, partial writes), plus the prologue;
* wall-clock (100 MHz ``s_memrealtime``) start and end of every wave, grouped by ``workgroup % 8`` -- the XCD the
  workgroup is dealt to -- which is how the finish-time imbalance between XCDs shows up.

    python -m tileops_amd.perf.phase_timers [c2,c3,c4,c5] [--reps N]

The instrumented kernel writes eight floats per wave *behind* the workspace the library asks for, so this tool
over-allocates the workspace; the product library never does that.
"""

from __future__ import annotations

import argparse
import sys
from pathlib import Path

import torch

from .. import build as build_mod
from .. import native
from ..workloads import BASELINE_CONFIGS, FP8, gen_paged_inputs

TIMER_LIB = Path(build_mod.LIB_PATH).with_name("libmi355_tileops_phase_timers.so")
NAMES = ("issue", "wait", "compute", "segment", "prologue", "total")


def _row_blocks(rows: int, dim: int) -> int:
    """Row blocks per wave the launcher picks (csrc/paged_decode_mfma.hip: row_blocks_for)."""
    return 1 if (rows <= 16 or dim == 256) else 2


def _ring_waves(rows: int, nrb: int, row_bytes: int) -> int:
    """Waves per shared LDS ring (csrc/paged_decode_mfma.hip: ring_waves_for, max_ring_for)."""
    n = (rows + 16 * nrb - 1) // (16 * nrb)
    if n <= 1:
        return 1
    max_ring = 8 if row_bytes == 256 else (2 if row_bytes == 64 else 4)
    even = (n + 1) // 2 * 2
    if even % 8 == 0 and max_ring >= 8:
        return 8
    return 4 if (even % 4 == 0 and max_ring >= 4) else 2


def run(name: str, hot: bool = False) -> None:
    cfg = BASELINE_CONFIGS[name]
    dev = torch.device("cuda", 0)
    inp = gen_paged_inputs(cfg, dev)
    if hot:  # every logical page is physical page 0: the whole cache read hits in L1/L2, what remains is on-chip time
        inp.block_table.zero_()
    out = torch.empty_like(inp.q)
    nbytes, nparts, _ = native.decode_workspace(cfg.batch, cfg.q_len, cfg.heads, cfg.heads_kv, cfg.dim, cfg.page_size,
                                                inp.block_table.shape[1], inp.q.dtype, inp.k.dtype, 0, native.KERNEL_MFMA)
    fp8 = inp.k.dtype == FP8
    rows = cfg.q_len * (cfg.heads // cfg.heads_kv)
    nrb = _row_blocks(rows, cfg.dim)
    shw = _ring_waves(rows, nrb, cfg.dim * (1 if fp8 else 2))
    n_rg = ((rows + 16 * nrb - 1) // (16 * nrb) + shw - 1) // shw * shw  # whole rings
    waves = nparts * cfg.heads_kv * n_rg
    nw = shw if shw > 1 else (8 if (fp8 or cfg.dim == 64) else (2 if cfg.dim == 256 else 4))  # waves per workgroup
    if shw > 1:
        waves = shw * 8 * (n_rg // shw) * ((nparts * cfg.heads_kv + 7) // 8)  # grid padded to whole rounds of the 8 XCDs
    ws = torch.zeros(nbytes + waves * 32 + 4096, dtype=torch.uint8, device=dev)
    flush_w = torch.empty(512 << 20, dtype=torch.uint8, device=dev)
    flush_r = torch.ones(128 << 20, dtype=torch.int32, device=dev)

    def call() -> None:
        native.paged_decode(inp.q, inp.k, inp.v, inp.k_scale, inp.v_scale, inp.real_seqlen_kv, inp.block_table, out, ws,
                            batch=cfg.batch, q_len=cfg.q_len, heads=cfg.heads, heads_kv=cfg.heads_kv, dim=cfg.dim,
                            page_size=cfg.page_size, sm_scale=cfg.dim ** -0.5, softcap=0.0, causal=True, num_split=nparts,
                            kernel=native.KERNEL_MFMA | native.KERNEL_FLAG_SKIP_COMBINE)

    for _ in range(2):
        flush_w.fill_(1)
        flush_r.max()
        call()
    flush_w.fill_(2)
    flush_r.max()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    call()
    b.record()
    torch.cuda.synchronize()
    # workspace layout: partial rows, LSE, per-sequence records (padded to 256 B), then the timer rows
    slots = 2 * nparts * cfg.heads_kv * rows
    al = lambda x: (x + 255) // 256 * 256  # noqa: E731
    off = al(slots * cfg.dim * 4) + al(slots * 4) + ((cfg.batch + 1) * 4 + 63) // 64 * 64 * 4
    t = ws[off:off + waves * 32].view(torch.float32).view(waves, 8).cpu().double()
    ran = t[:, 5] > 0  # waves of partitions past the last one leave before the timers
    xcd_all = (torch.arange(waves) // nw) % 8
    t, xcd_all, waves = t[ran], xcd_all[ran], int(ran.sum())
    print(f"{name}{' (all pages = page 0)' if hot else ''}: attention kernel {a.elapsed_time(b) * 1e3:.1f} us (HIP events), {waves} waves, {nparts} partitions, {nw} waves per workgroup")
    for i, n in enumerate(NAMES):
        print(f"   {n:9s} cycles: mean {t[:, i].mean():10.0f}  max {t[:, i].max():10.0f}")
    start = (t[:, 6] - t[:, 6].min()) / 100.0
    end = (t[:, 7] - t[:, 6].min()) / 100.0
    q = lambda x, ps: [round(float(torch.quantile(x, p)), 1) for p in ps]  # noqa: E731
    print(f"   wall clock: waves start within {float(start.max()):.1f} us; end at {q(end, [0, .1, .5, .9, 1])} us (min/10%/50%/90%/max), mean {float(end.mean()):.1f}")
    xcd = xcd_all
    print("   mean end per XCD (workgroup % 8): " + "  ".join(f"{k}:{float(end[xcd == k].mean()):.1f}" for k in range(8)))


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("configs", nargs="?", default="c2,c3")
    ap.add_argument("--reps", type=int, default=1)
    ap.add_argument("--hot", action="store_true", help="point every block-table entry at page 0 (no HBM traffic)")
    ap.add_argument("--no-build", action="store_true", help="use an instrumented library built earlier")
    args = ap.parse_args(argv)
    if not args.no_build or not TIMER_LIB.exists():
        build_mod.build(verbose=False, extra_flags=("-DMI355_PHASE_TIMERS",), lib_path=TIMER_LIB)
    native.LIB_PATH = TIMER_LIB  # before the first native call: this process measures, it does not serve
    native.require_gfx950(torch.device("cuda", 0))
    for name in args.configs.split(","):
        for _ in range(args.reps):
            run(name, args.hot)
    return 0


if __name__ == "__main__":
    sys.exit(main())
