"""bench.py end to end with one timed step per workload: every workload of the table runs, the line parses and carries
the fields its readers take (metric, value, roofline with a measured duration, the workloads' fractions)."""
import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_bench_line():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--steps", "1", "--warmup", "0", "--ramp-ms", "0", "--no-cpu-baseline"],
                       capture_output=True, text=True, timeout=600, cwd=ROOT)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [ln for ln in r.stdout.splitlines() if ln.startswith("{")]
    assert len(lines) == 1, r.stdout[-2000:]
    d = json.loads(lines[0])
    assert d["n_gpus"] == 1 and d["steps"] == 1 and d["higher_is_better"] is True and d["unit"] == "TFLOP/s"
    assert d["value"] > 0 and d["ms_per_step"] > 0 and d["dtype"] == "bf16" and "workload" in d["config"]
    roof = d["roofline"]
    assert roof["bound"] == "mfma" and roof["peak"] == 2500.0 and 0 < roof["frac"] < 1 and abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    others = d["other_workloads"]
    for name in ("c2_sigmoid_causal", "c2_softmax_causal_operator", "c2_softmax_causal_bwd", "c3_retnet_chunked", "c3_retnet_parallel",
                 "c3_retnet_parallel_operator", "c3_retnet_parallel_generated_mask", "c3_retnet_parallel_bwd", "c3_retnet_chunked_bwd",
                 "c4_mamba2_ssd", "c4_mamba2_bwd", "c3_retnet_chunked_operator", "c4_mamba2_ssd_operator", "c5_mla_decode_operator",
                 "c5_mla_decode", "gqa_decode"):
        assert name in others and "error" not in others[name], (name, others.get(name))
        assert others[name]["ms"] > 0
    ref = others["reference_shapes"]
    assert "error" not in ref and len([k for k in ref if k != "note"]) == 11
    for key, entry in ref.items():
        if key != "note":
            assert entry["ms"] > 0 and entry["reference_ms"]
    rb = others["reference_benchmark_shapes"]
    assert "error" not in rb and len(rb) == 9, rb
    assert all(min(v for k, v in e.items() if k.endswith("ms") or k.startswith("ms")) > 0 for e in rb.values())
    hs = others["head_sizes"]
    assert "error" not in hs and len([k for k in hs if k != "note"]) == 18, hs
    assert all(e["fwd_ms"] > 0 and e["bwd_ms"] > 0 for k, e in hs.items() if k != "note")
    # the operator recognised the decay mask the workload builds
    assert "generates it" in others["c3_retnet_parallel_operator"]["flop_convention"]
    for name in ("c5_mla_decode", "gqa_decode"):
        assert 0 < others[name]["frac_of_hbm_peak"] <= others[name]["frac_of_hbm_peak_clean_read"] * 1.5

