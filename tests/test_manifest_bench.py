"""The benchmark report plumbing: JUnit ``<tag>_<metric>`` properties and the ``profile_run.log`` tables.

The reference tests its harness on synthetic records (benchmarks/tests/test_benchmark_base.py:78-224) and fixes the
property naming in its pytest hook (benchmarks/conftest.py:52-136) and the log layout in benchmarks/report.py:117-262;
the first tests here do the same on the CPU, the last one runs one manifest row end to end on the GPU.
"""

import xml.etree.ElementTree as ET

import pytest
import torch

from tileops_amd.perf import manifest_bench as mb


def _props(case: ET.Element) -> dict:
    return {p.get("name"): p.get("value") for p in case.find("properties")}


def test_property_values_keep_significant_digits():
    # benchmarks/conftest.py:36-47: bools and ints verbatim, integral floats as ints, others with six significant digits
    assert mb._prop(True) == "True" and mb._prop(3) == "3" and mb._prop(2.0) == "2"
    assert mb._prop(0.000123456789) == "0.000123457" and mb._prop(1234.56789) == "1234.57" and mb._prop("x") == "x"


def test_junit_case_names_follow_the_tag_metric_scheme(tmp_path):
    suite = ET.Element("testsuite", name="t")
    ours = {"tag": "tileops", "op": "SomeFwdOp", "op_module": "pkg.ops", "latency_ms": 0.25, "device_busy_ms": 0.2, "tflops": 1.5,
            "bandwidth_tbs": 4.0, "gap_ms": None}
    first = {"tag": "torch_sdpa", "op": "SomeFwdOp", "latency_ms": 1.0, "device_busy_ms": 0.8, "tflops": 0.375}
    second = {"tag": "other-impl", "op": "SomeFwdOp", "latency_ms": 0.5}
    case = mb.junit_case(suite, "row-float16", [ours, first, second])
    p = _props(case)
    assert case.get("classname") == "SomeFwdOp" and case.get("name") == "row-float16" and case.get("time") == "0.000250"
    assert p["op"] == "SomeFwdOp" and p["op_module"] == "pkg.ops" and "tileops_variant" not in p
    assert p["tileops_latency_ms"] == "0.25" and p["tileops_device_busy_ms"] == "0.2" and p["tileops_tflops"] == "1.5"
    assert "tileops_gap_ms" not in p                                   # None is not a measurement
    assert not any(k in p for k in ("tileops_tag", "tileops_op", "tileops_op_module"))
    # every baseline under its own tag; the first also under the unprefixed legacy names
    assert p["torch_sdpa_latency_ms"] == "1" and p["baseline_tag"] == "torch_sdpa" and p["baseline_latency_ms"] == "1"
    assert p["other-impl_latency_ms"] == "0.5" and "baseline_tflops" in p
    # ratios compare device-busy time when both sides have it, wall latency otherwise
    assert p["torch_sdpa_ratio"] == "4.0000" and p["baseline_ratio"] == "4.0000" and p["other-impl_ratio"] == "2.0000"
    # a variant tag is published as such; a case without our entry still lists its baselines
    v = _props(mb.junit_case(suite, "v", [dict(ours, tag="tileops_mfma")]))
    assert v["tileops_variant"] == "mfma" and v["tileops_latency_ms"] == "0.25"
    only_bl = _props(mb.junit_case(suite, "b", [first]))
    assert only_bl["baseline_tag"] == "torch_sdpa" and "op" not in only_bl and "baseline_ratio" not in only_bl
    mb.write_junit(suite, tmp_path / "junit.xml")
    root = ET.parse(tmp_path / "junit.xml").getroot()
    assert root.get("tests") == "3" and len(root.findall("testcase")) == 3


def test_report_log_groups_by_op_and_tag(tmp_path):
    rep = mb.BenchmarkReport()
    rep.dump(tmp_path / "empty.log")
    assert not (tmp_path / "empty.log").exists()                        # nothing recorded, nothing written
    params = {"label": "row-a", "q_shape": (4, 32, 128), "dtype": "float16"}
    rep.record("SomeFwdOp", params, {"latency_ms": 0.25, "tflops": 1.5, "bandwidth_tbs": 4.0, "hbm_frac": 0.5}, "tileops", {"num_split": 0})
    rep.record("SomeFwdOp", dict(params, label="row-b"), {"latency_ms": 0.5, "tflops": 0.75, "bandwidth_tbs": 2.0, "hbm_frac": 0.25})
    rep.record("SomeFwdOp", params, {"latency_ms": 1.0, "tflops": 0.375, "bandwidth_tbs": 1.0}, "torch_sdpa")
    rep.record("OtherOp", {"label": "z"}, {"latency_ms": 2.0, "ok": True})
    rep.dump(tmp_path / "profile_run.log")
    text = (tmp_path / "profile_run.log").read_text()
    lines = text.splitlines()
    assert lines[0] == "# TileOPs Benchmark Report" and "## Environment" in lines
    assert lines.index("## SomeFwdOp") < lines.index("### tileops") < lines.index("### torch_sdpa") < lines.index("## OtherOp")
    # the column the implementations are compared on leads; measurements not in the default list follow; config closes
    header = next(ln for ln in lines if ln.startswith("| label"))
    assert header == "| label | q_shape | dtype | device_busy_ms | latency_ms | gap_ms | n_kernels | tflops | bandwidth_tbs | hbm_frac | config |"
    row_a = next(ln for ln in lines if ln.startswith("| row-a"))
    assert row_a == "| row-a | (4, 32, 128) | float16 | N/A | 0.2500 | N/A | N/A | 1.5000 | 4.0000 | 0.5000 | {'num_split': 0} |"
    assert next(ln for ln in lines if ln.startswith("| row-b")).endswith("| 0.2500 |  |")   # no config recorded for this row
    assert "| z | N/A | 2.0000 | N/A | N/A | N/A | N/A | True |" in text                     # bools are not formatted as numbers


@pytest.mark.gpu
def test_one_manifest_row_end_to_end(tmp_path):
    """One reference workload row through the runner: both artefacts are written and parse back."""
    rc = mb.main(["--op", "GroupedQueryAttentionDecodePagedWithKVCacheFwdOp", "--label", "serving-8b-p64", "--steps", "3",
                  "--out", str(tmp_path)])
    assert rc == 0
    cases = ET.parse(tmp_path / "junit.xml").getroot().findall("testcase")
    assert cases and all(c.get("classname") == "GroupedQueryAttentionDecodePagedWithKVCacheFwdOp" for c in cases)
    for c in cases:
        p = _props(c)
        assert p["op"] == "GroupedQueryAttentionDecodePagedWithKVCacheFwdOp" and p["op_module"] == "tileops_amd.ops"
        assert float(p["tileops_latency_ms"]) > 0 and float(p["tileops_bandwidth_tbs"]) > 0 and 0 < float(p["tileops_hbm_frac"]) < 1
        assert abs(float(c.get("time")) * 1e3 - float(p["tileops_latency_ms"])) < 1e-3
        # the same-device torch baseline of a paged row rides along under its own tag, and as the first baseline
        if "softcap" not in c.get("name"):  # (torch's SDPA has no softcap: that row carries no baseline)
            assert p["baseline_tag"] == "torch_gather_sdpa" and float(p["torch_gather_sdpa_latency_ms"]) > 0 and float(p["baseline_ratio"]) > 1
    log = (tmp_path / "profile_run.log").read_text()
    assert "## GroupedQueryAttentionDecodePagedWithKVCacheFwdOp" in log and "### tileops" in log and "serving-8b-p64" in log
    assert "### torch_gather_sdpa" in log
    assert torch.cuda.is_available()


@pytest.mark.gpu
def test_paged_torch_baseline_computes_what_the_op_computes():
    """The baseline that paged rows are compared with (gather by block table, SDPA with a padding mask) agrees with the op
    on ragged lengths and a permuted table -- a ratio against a wrong baseline would mean nothing."""
    from tileops_amd.manifest import load_workloads

    row = dict(next(r for r in load_workloads("GroupedQueryAttentionDecodePagedWithKVCacheFwdOp") if r["label"] == "serving-8b-p64"))
    row.update(seqlen_range=[100, 4000], seed=4, kv_shape=[65536, 8, 128])
    op, args, baseline = mb._paged_case(row, torch.bfloat16, torch.device("cuda", 0), False)
    assert baseline is not None
    torch.testing.assert_close(op(*args).float(), baseline().squeeze(2).float(), atol=2e-2, rtol=2e-2)
