"""Hardware profile of the target GPU and the probe that calibrates it.

``load_profile("mi355x")`` returns the YAML under ``profiles/`` with ``hbm.effective = theoretical x calibration``
(same convention as the reference's src/tileops/perf/profile.py:58-84 and perf/profiles/h200.yaml:11-13).
``build_probe()`` compiles ``hbm_page_read_probe.hip`` and ``mfma_rate_probe.hip`` to stand-alone binaries next to them.
"""

from __future__ import annotations

import subprocess
from pathlib import Path
from typing import Any

import yaml

_DIR = Path(__file__).resolve().parent
PROBE_SRC = _DIR / "hbm_page_read_probe.hip"
PROBE_BIN = _DIR / "hbm_page_read_probe"


MFMA_PROBE_SRC = _DIR / "mfma_rate_probe.hip"
MFMA_PROBE_BIN = _DIR / "mfma_rate_probe"


def load_profile(gpu: str = "mi355x") -> dict[str, Any]:
    """The profile with the effective rates filled in: ``hbm.effective_gbs`` and, per matrix element type,
    ``matrix.<type>.effective_tflops`` = theoretical x calibration (reference: ``tensor_core.<type>`` of h200.yaml)."""
    prof = yaml.safe_load((_DIR / "profiles" / f"{gpu}.yaml").read_text())
    hbm = prof["hbm"]
    hbm["effective_gbs"] = hbm["theoretical_gbs"] * hbm["calibration"]
    for entry in prof.get("matrix", {}).values():
        if isinstance(entry, dict) and "theoretical_tflops" in entry:
            entry["effective_tflops"] = entry["theoretical_tflops"] * entry["calibration"]
    return prof


def build_probe() -> Path:
    for src, out in ((PROBE_SRC, PROBE_BIN), (MFMA_PROBE_SRC, MFMA_PROBE_BIN)):
        cmd = ["hipcc", "--offload-arch=gfx950", "-O3", str(src), "-o", str(out)]
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src.name}:\n{res.stderr}")
    return PROBE_BIN


if __name__ == "__main__":
    print(build_probe())
