"""Pins the FP8-E4M3FN byte codec and the per-token quantizer of the oracle (C and Python restatements)."""

import ctypes
import json
import math
import struct
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import build as oracle_build
from oracle.paged_gqa_decode_ref import dequantize_kv, quantize_kv_per_token
from tileops_amd import workloads

FP8 = torch.float8_e4m3fn


@pytest.fixture(scope="module")
def clib():
    oracle_build.build()
    return oracle_build.load()


def _decode_all(clib):
    return np.array([clib.fp8_e4m3fn_decode(c) for c in range(256)], dtype=np.float32)


def test_decode_table_matches_committed_fixture_and_torch(clib):
    got = _decode_all(clib)
    fixture = json.loads((Path(__file__).parent / "golden" / "fp8_e4m3fn_table.json").read_text())["decode_f32_bits"]
    live = torch.arange(256, dtype=torch.uint8).view(FP8).float().numpy()
    for c in range(256):
        if fixture[c] is None:
            assert math.isnan(got[c]) and math.isnan(live[c]) and c in (0x7F, 0xFF)
        else:
            want = struct.unpack("<f", struct.pack("<I", fixture[c]))[0]
            assert got[c] == want == live[c], c
    # spot values fixed by the format definition: bias 7, 3 mantissa bits, max 448, subnormal step 2^-9
    assert got[0x38] == 1.0 and got[0x7E] == 448.0 and got[0x01] == 2.0 ** -9 and got[0x08] == 2.0 ** -6
    assert got[0xB8] == -1.0 and got[0x00] == 0.0


def test_encode_matches_torch_cast_on_every_rounding_boundary(clib):
    finite = sorted(v for v in _decode_all(clib)[:0x7F].tolist())
    probes = []
    for a, b in zip(finite[:-1], finite[1:]):
        mid = np.float32((np.float64(a) + np.float64(b)) / 2)
        probes += [a, b, mid, np.nextafter(mid, np.float32(-1)), np.nextafter(mid, np.float32(1e9))]
    probes += [448.0, 460.0, np.nextafter(np.float32(464), np.float32(0)), 2.0 ** -10, np.nextafter(np.float32(2.0 ** -10), np.float32(1)), 1e-8, 0.0]
    x = np.array(probes + [-p for p in probes], dtype=np.float32)
    want = torch.from_numpy(x).to(FP8).view(torch.uint8).numpy()
    got = np.array([clib.fp8_e4m3fn_encode(float(v)) for v in x], dtype=np.uint8)
    np.testing.assert_array_equal(got, want)


def test_encode_random_dense_and_overflow_to_nan(clib):
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.normal(0, 100, 20000), rng.normal(0, 0.01, 20000), rng.uniform(-463.9, 463.9, 20000)]).astype(np.float32)
    want = torch.from_numpy(x).to(FP8).view(torch.uint8).numpy()
    got = np.empty_like(want)
    clib.fp8_e4m3fn_encode_n(x.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), got.ctypes.data_as(ctypes.POINTER(ctypes.c_uint8)), x.size)
    np.testing.assert_array_equal(got, want)
    # torch's cast does not saturate: beyond the 464 tie (which rounds to even = 448) the result is NaN,
    # which is why the quantizer clamps first
    assert clib.fp8_e4m3fn_encode(464.0) == 0x7E and torch.tensor(464.0).to(FP8).float().item() == 448.0
    for v in (float(np.nextafter(np.float32(464), np.float32(1e9))), 500.0, 1e9, float("inf")):
        assert clib.fp8_e4m3fn_encode(v) == 0x7F and math.isnan(torch.tensor(v).to(FP8).float().item())


def test_decode_encode_round_trip_is_identity(clib):
    for c in range(256):
        if c in (0x7F, 0xFF):
            continue
        assert clib.fp8_e4m3fn_encode(clib.fp8_e4m3fn_decode(c)) == c or (c == 0x80 and clib.fp8_e4m3fn_encode(-0.0) == 0x80)


def test_quantizer_c_python_and_workload_generator_agree_bit_for_bit(clib):
    g = torch.Generator().manual_seed(3)
    x = torch.randn(257, 3, 64, generator=g) * torch.logspace(-3, 2, 257)[:, None, None]
    x[5] = 0.0          # absmax below the 1e-4 floor
    x[6, 0, 0] = 1e-6
    q_py, s_py = quantize_kv_per_token(x)
    q_wl, s_wl = workloads.quantize_kv_per_token(x, chunk_tokens=100)
    assert torch.equal(q_py.view(torch.uint8), q_wl.view(torch.uint8)) and torch.equal(s_py, s_wl)
    rows = x.reshape(-1, 64).contiguous().numpy()
    qc = np.empty(rows.shape, dtype=np.uint8)
    sc = np.empty(rows.shape[0], dtype=np.float32)
    clib.fp8_quant_per_token(rows.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), qc.ctypes.data_as(ctypes.POINTER(ctypes.c_uint8)),
                             sc.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), rows.shape[0], 64)
    np.testing.assert_array_equal(qc, q_py.view(torch.uint8).reshape(-1, 64).numpy())
    np.testing.assert_array_equal(sc, s_py.reshape(-1).numpy())


def test_quantizer_properties():
    g = torch.Generator().manual_seed(4)
    x = torch.randn(64, 2, 128, generator=g)
    q8, s = quantize_kv_per_token(x)
    # scale = absmax/448 exactly; the absmax element maps to +-448; nothing is NaN; error <= half a step of the top binade
    amax = x.abs().amax(-1)
    assert torch.equal(s, amax / 448.0)
    assert torch.equal(q8.float().abs().amax(-1), torch.full_like(amax, 448.0))
    deq = dequantize_kv(q8, s)
    assert torch.isfinite(deq).all()
    assert ((deq - x).abs() <= amax[..., None] * (16.0 / 448.0) + 1e-7).all()
    zeros, sz = quantize_kv_per_token(torch.zeros(2, 1, 8))
    assert torch.equal(sz, torch.full((2, 1), 1e-4 / 448.0)) and torch.equal(zeros.float(), torch.zeros(2, 1, 8))
