"""The last stdout line of bench.py must stay small: whatever reads it keeps only the end of the program's output,
and a line that has outgrown that loses its head (metric, value, roofline).  These tests build the result from
stub timings (no GPU, no library) and check the size and the fields of the line."""
import json

import pytest

import bench


class _StubOp:
    def __init__(self, key, label, nbytes):
        self.key, self.label, self.nbytes = key, label, nbytes
        self.kernel = "some_kernel_name<float, 4, 1, true> (family, variant)"


def _stub_result(traffic_note=None, with_cpu=True):
    step_bytes = 9_940_946_944
    result = bench.headline(20, 5, 1 << 28, step_bytes, 1.65331234, 1.66001234)
    adam = _StubOp("c3_adam", "configs[3] Adam step, 268435456 float32 parameters", 28 << 28)
    stored = {"traffic": 7_516_999_999, "kernel_us": 1169.48}
    result["roofline"] = bench.adam_roofline(adam, 1.2205, stored, traffic_note)
    # every section as full as a real run makes it: long labels, every optional field present
    for section, n_ops in (("ops", 16), ("others", 10), ("midsize", 8), ("variants", 7), ("patterns", 14), ("small", 12),
                           ("adjacent", 16)):
        sect = {}
        for i in range(n_ops):
            op = _StubOp(f"{section}_{i}", f"{section} workload {i}: " + "x" * 120, 268_500_992)
            sect[op.label] = bench.roofline_block(op, 0.04567, stored, host_us=4.37)
        result[section] = sect
    # the workloads the line quotes one fraction for
    for _, section, key in bench.CONFIG_FRACS:
        op = _StubOp(key, f"label of {key} " + "y" * 100, 268_500_992)
        result[section][op.label] = bench.roofline_block(op, 0.04567, stored, host_us=4.37)
    result["c_caller"] = {"calls": 2000, "note": "n" * 300}
    if with_cpu:
        result["cpu_baseline"] = {"value": 46.178, "unit": "GB/s", "cores": 16, "kind": "port",
                                  "sample": "47 full steps (Adam over 268435456 float32 parameters, the twelve configs[2] "
                                            "reductions, the configs[0] bias add) in 10.12 s; C++ restatement of the cortex "
                                            "CPU backend, OpenMP over the index space the reference hands to parallel-for"}
    return result


@pytest.mark.parametrize("traffic_note", [None, "kernel sources changed since profiles/traffic.json was measured "
                                                "(0123abcd -> 89ef4567): traffic not reported"])
def test_final_line_is_small_and_complete(traffic_note):
    result = _stub_result(traffic_note)
    assert len(json.dumps(result)) > 20000  # the detail really is too large for one line
    line = bench.final_line(result)
    text = json.dumps(line)
    assert len(text) < bench.FINAL_LINE_LIMIT <= 4096
    assert "\n" not in text
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in line, key
    assert line["metric"] == "achieved HBM GB/s (% of MI355X peak) for binary-op!, unary-reduce!, Adam step"
    assert line["vs_baseline"] is None and line["n_gpus"] == 1 and line["dtype"] == "f32"
    assert set(line["config"]) >= {"workload", "algorithmic_bytes_per_step"} and "model" not in line["config"]
    roof = line["roofline"]
    for key in ("bound", "achieved", "peak", "unit", "frac", "traffic"):
        assert key in roof, key
    assert roof["bound"] == "hbm" and roof["peak"] == 8000.0
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    assert len(roof["note"]) <= 200
    for key in ("value", "unit", "cores", "kind", "sample"):
        assert key in line["cpu_baseline"], key
    fracs = line["frac_of_peak_by_config"]
    assert len(fracs) == len(bench.CONFIG_FRACS) <= 25
    assert all(isinstance(v, float) for v in fracs.values())
    for section in ("ops", "others", "midsize", "variants", "patterns", "adjacent", "c_caller", "small"):
        assert section not in line


def test_final_line_without_optional_sections():
    result = _stub_result(with_cpu=False)
    for section in ("others", "midsize", "variants", "patterns", "adjacent", "small", "c_caller"):
        del result[section]
    line = bench.final_line(result)
    assert "cpu_baseline" not in line
    assert set(line["frac_of_peak_by_config"]) == {n for n, s, _ in bench.CONFIG_FRACS if s == "ops"}


def test_final_line_refuses_to_grow():
    result = _stub_result()
    result["roofline"]["note"] = "z" * 5000
    with pytest.raises(RuntimeError):
        bench.final_line(result)


def test_headline_value_follows_from_bytes_and_time():
    h = bench.headline(20, 5, 1 << 28, 8_000_000_000, 1.0, 1.0)
    assert h["value"] == 8000.0 and h["config"]["frac_of_peak"] == 1.0 and h["ms_per_step"] == 1.0
