"""Hardware profile of the target GPU and the probe that calibrates it.

``load_profile("mi355x")`` returns the YAML under ``profiles/`` with ``hbm.effective = theoretical x calibration``
(same convention as the reference's src/tileops/perf/profile.py:58-84 and perf/profiles/h200.yaml:11-13).
``build_probe()`` compiles ``hbm_page_read_probe.hip`` to a stand-alone binary next to it.
"""

from __future__ import annotations

import subprocess
from pathlib import Path
from typing import Any

import yaml

_DIR = Path(__file__).resolve().parent
PROBE_SRC = _DIR / "hbm_page_read_probe.hip"
PROBE_BIN = _DIR / "hbm_page_read_probe"


def load_profile(gpu: str = "mi355x") -> dict[str, Any]:
    prof = yaml.safe_load((_DIR / "profiles" / f"{gpu}.yaml").read_text())
    hbm = prof["hbm"]
    hbm["effective_gbs"] = hbm["theoretical_gbs"] * hbm["calibration"]
    return prof


def build_probe() -> Path:
    cmd = ["hipcc", "--offload-arch=gfx950", "-O3", str(PROBE_SRC), "-o", str(PROBE_BIN)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on the probe:\n{res.stderr}")
    return PROBE_BIN


if __name__ == "__main__":
    print(build_probe())
