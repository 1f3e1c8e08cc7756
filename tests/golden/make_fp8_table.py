"""Writes tests/golden/fp8_e4m3fn_table.json: the 256 values of OCP FP8 E4M3FN as torch.float8_e4m3fn decodes
them, as fp32 bit patterns (null for the two NaN codes).  torch is a library present on every box; the reference is
not involved.  The encoder's rounding is pinned elsewhere (tests/test_oracle_fp8.py: a dense grid, the midpoints
between neighbouring codes included, against torch's own cast).  Run once: ``python tests/golden/make_fp8_table.py``."""

import json
import struct
from pathlib import Path

import torch

codes = torch.arange(256, dtype=torch.uint8)
vals = codes.view(torch.float8_e4m3fn).float()
table = [None if v != v else struct.unpack("<I", struct.pack("<f", float(v)))[0] for v in vals.tolist()]
out = {"format": "e4m3fn", "decode_f32_bits": table}
Path(__file__).with_name("fp8_e4m3fn_table.json").write_text(json.dumps(out))
print("wrote", len(table), "codes;", sum(t is None for t in table), "NaN codes")
