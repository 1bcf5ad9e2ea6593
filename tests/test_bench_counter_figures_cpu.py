"""The counter figures bench.py quotes from profiles/*.md belong to one build: they are given only when the summary's
recorded build id equals the loaded library's."""
import os
import re
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import bench  # noqa: E402
import candle_amd  # noqa: E402

PROFILES = sorted(f for f in os.listdir(os.path.join(ROOT, "profiles")) if f.endswith(".md"))
FIGURES = [("q4k_up_decode_hbm_traffic.md", "traffic_bytes_per_launch", "batch=32"),
           ("q4k_gemm_prefill_4096_kernel_trace.md", "mfma_busy_frac", "prefill_up"),
           ("q8_0_gemm_config4_kernel_trace.md", "traffic_bytes_per_launch", "config4")]


@pytest.mark.parametrize("name", PROFILES)
def test_every_profile_summary_names_the_build_it_was_measured_on(name):
    assert re.fullmatch(r"[0-9a-f]{16}", bench.profile_build_id(name) or ""), name


@pytest.mark.parametrize("name,label,key", FIGURES)
def test_a_figure_is_given_for_its_own_build_only(name, label, key, monkeypatch):
    own = bench.profile_build_id(name)
    monkeypatch.setattr(candle_amd, "build_id", lambda: own)
    value, note = bench.counter_figure(name, label, key)
    assert value is not None and value > 0 and own in note
    monkeypatch.setattr(candle_amd, "build_id", lambda: "0123456789abcdef")
    value, note = bench.counter_figure(name, label, key)
    assert value is None and own in note and "0123456789abcdef" in note and "withheld" in note


def test_a_figure_the_summary_does_not_hold_is_none(monkeypatch):
    name = FIGURES[0][0]
    monkeypatch.setattr(candle_amd, "build_id", lambda: bench.profile_build_id(name))
    value, note = bench.counter_figure(name, "traffic_bytes_per_launch", "batch=7")
    assert value is None and "holds no" in note
