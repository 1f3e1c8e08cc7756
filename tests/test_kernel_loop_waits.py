"""Static check of the compiled MFMA attention kernels: no prefetch drain inside the tile loop.

The kernels keep several direct-to-LDS loads of later K/V tiles in flight while they work on the current tile.  An
`s_waitcnt vmcnt(0)` in the blocks of the tile loop that read LDS or issue matrix instructions would wait for all of
them on every tile.  The source never asks for one there (its own waits name the count of loads that may stay in
flight); the compiler adds one when an ordinary global load is left formally outstanding on some path into the loop and
a register it writes is reused in the loop, which is easy to cause by accident in the rare blocks that load sequence
lengths or query rows.  This test compiles the kernel source to assembly (device side only, no GPU needed) and looks.
"""
import re
import shutil
import subprocess
from pathlib import Path

import pytest

from tileops_amd import build

SRC = Path(build.__file__).resolve().parent / "csrc" / "paged_decode_mfma.hip"


def _functions(asm: str):
    for m in re.finditer(r"\n(_ZN5mi355\S*paged_decode_mfma_kernel[^:\s]*):", asm):
        start = m.end()
        yield m.group(1), asm[start:asm.index(".Lfunc_end", start)]


def drains_in_tile_loop(body: str) -> int:
    """Blocks of loops nested two deep or more (the tile loop and what it contains) that read LDS or issue matrix
    instructions and also hold an `s_waitcnt vmcnt(0)`."""
    n = 0
    for block in re.split(r"\n(?=\.LBB\d+_\d+:)", body):
        head = block.split("\n", 1)[0]
        if "Depth=2" not in head and "Depth=3" not in head:
            continue
        for sub in re.split(r"\n; %bb\.\d+:", block):
            if ("v_mfma" in sub or "ds_read" in sub) and re.search(r"s_waitcnt[^\n]*vmcnt\(0\)", sub):
                n += 1
    return n


def test_detector_sees_a_drain_in_a_loop_block():
    body = (".LBB1_2:  ; =>This Inner Loop Header: Depth=2\n\tds_read_b128 v[0:3], v4\n\ts_waitcnt vmcnt(0)\n"
            "\tv_mfma_f32_16x16x32_bf16 v[0:3], v[4:7], v[8:11], v[0:3]\n"
            ".LBB1_3:  ; in Loop: Header=BB1_2 Depth=1\n\ts_waitcnt vmcnt(0)\n\tds_read_b128 v[0:3], v4\n")
    assert drains_in_tile_loop(body) == 1


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="hipcc not on PATH")
def test_no_compiler_inserted_drain_in_the_tile_loop(tmp_path):
    out = tmp_path / "mfma.s"
    cmd = [shutil.which("hipcc"), *build.HIPCC_FLAGS, "--cuda-device-only", "-S", str(SRC), "-o", str(out)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-2000:]
    found = {name: n for name, body in _functions(out.read_text()) if (n := drains_in_tile_loop(body))}
    names = [name for name, _ in _functions(out.read_text())]
    assert len(names) >= 40  # the instantiations are there under the expected symbol names
    assert not found, f"vmcnt(0) inside the tile loop of: {sorted(found)}"
