"""The figures bench.py copies from the profile summaries (counters cannot be read from inside
the benchmark's own process) must be the ones the summaries state."""

import importlib.util
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench():
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_traffic_and_mfma_constants_match_the_profile_summary():
    bench = _bench()
    text = open(os.path.join(ROOT, "profiles", "attend32_c2_qwen3_4b.md")).read()
    key = (2, 1024, 32)
    assert "chunk_tokens 1024, rows_per_item 32" in text  # the summary is for this key
    m = re.search(r"HBM traffic per launch = ([\d.]+) MB", text)
    assert m and round(float(m.group(1)) * 1e6) == bench.MEASURED_TRAFFIC_BYTES[key]
    # fetched + written, from the table of the two counter passes
    row = re.search(r"\| fca_attend32_kernel \| \d+ \| ([\d.]+) MB \| \d+ \| ([\d.]+) MB \|", text)
    assert row and abs(float(row.group(1)) + float(row.group(2)) - float(m.group(1))) < 0.05
    util = bench.MEASURED_MFMA_UTIL[key]
    assert os.path.exists(os.path.join(ROOT, util["source"]))
    whole = re.search(r"MFMA utilisation = .* = ([\d.]+) %", text)
    assert whole and abs(float(whole.group(1)) / 100 - util["attention_launch"]) < 5e-4
    prefix = re.search(r"shared-prefix pass .*\| ([\d.]+) % \|", text)
    assert prefix and abs(float(prefix.group(1)) / 100 - util["prefix_pass"]) < 5e-4
    # every key with a traffic figure names an existing summary through the MFMA table or the default one
    assert set(bench.MEASURED_TRAFFIC_BYTES) == set(bench.MEASURED_MFMA_UTIL)


def test_metric_string_is_the_baselines():
    import json

    bench = _bench()
    base = json.load(open(os.path.join(ROOT, "BASELINE.json")))
    assert bench.METRIC == base["metric"]
