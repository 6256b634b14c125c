"""The one stdout line of bench.py stays small enough for the harness that records it and keeps
the keys that harness reads, whatever ran and whatever failed."""

import json

import bench


def _dense(name, bound="hbm", plan="g1 split-k=8 partial #4 " + "x" * 400):
    roof = {"bound": bound, "achieved": 4970.1, "peak": 8000.0, "unit": "GB/s", "frac": 0.6213, "traffic": 97050000,
            "measured_stream_peak": 6180.0, "frac_of_measured_stream": 0.804}
    return {"op": name, "workload": f"{name} workload " + "w" * 80, "best_us": 21.379, "dominant_kernel_us": 18.24,
            "graph_replay_us": 20.9, "variant": "split-k=8", "plan": plan, "candidates": 48, "validated": 48,
            "hbm": roof, "mfma": roof, "roofline": roof, "algorithmic_bytes": 90669056, "algorithmic_flops": 1442840576,
            "cpu_us": 41234.5, "cpu_sample": "full workload, median of 20 runs"}


def _registry():
    rows = []
    for i in range(9):
        per = {f"wl_{a}_{b}_{c}": 12.34 for a in (1, 8, 64) for b in range(4) for c in range(4)}
        rows.append({"op": f"gqa_paged_prefill_causal_h32_kv{i}_d128_ps1", "dtype": "bf16", "workloads": len(per),
                     "candidates": 12, "validated": 12, "best": "y" * 200, "geomean_us": 17.01, "per_workload_us": per,
                     "reference_h100_us": per, "reference_h100_geomean_us": 18.0, "search_s": 10.0})
    return {"op": "dyn", "workload": "registry operators", "operators": rows}


DEFAULT_OPS = ["c2", "c1", "c3", "c4", "c5", "mm", "mm_nt", "mm8k", "swiglu", "rmsmm", "lora", "mmrs", "mm2d", "rsdiv",
               "attn", "qknorm", "mlapf", "dyn"]


def _results():
    res = {n: _dense(n, "mfma" if n.startswith("mm") else "hbm") for n in DEFAULT_OPS if n != "dyn"}
    res["dyn"] = _registry()
    return res


def test_line_is_small_and_round_trips():
    line = bench.final_line(_results(), DEFAULT_OPS, 20, 5, 16)
    text = json.dumps(line)
    assert len(text) < bench.LINE_LIMIT
    back = json.loads(text)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline", "ops"):
        assert key in back, key
    assert back["steps"] == 20 and back["warmup"] == 5 and back["n_gpus"] == 1
    assert set(back["roofline"]) == {"bound", "achieved", "peak", "unit", "frac", "traffic"}
    assert back["cpu_baseline"]["cores"] == 16 and back["cpu_baseline"]["kind"] == "port"
    assert back["config"]["workload"].startswith("c2 workload")
    assert [r["op"] for r in back["ops"]] == DEFAULT_OPS
    assert set(back["ops"][0]) == {"op", "best_us", "dominant_kernel_us", "frac", "bound"}
    assert len(back["ops"][-1]["geomean_us"]) == 9


def test_default_operator_list_is_what_the_line_was_sized_for():
    import re

    src = open(bench.__file__).read()
    default = re.search(r'"--ops", default="([^"]+)"', src).group(1).split(",")
    assert len(default) <= len(DEFAULT_OPS) + 4
    res = {n: _dense(n) for n in default if n != "dyn"}
    res["dyn"] = _registry()
    assert len(json.dumps(bench.final_line(res, default, 200, 20, 16))) < bench.LINE_LIMIT


def test_failed_operators_and_a_missing_headline_still_give_a_line():
    res = _results()
    res["c3"] = {"op": "c3", "error": "RuntimeError: " + "e" * 300}
    line = bench.final_line(res, DEFAULT_OPS, 20, 5, None)
    assert line["cpu_baseline"] is None and len(json.dumps(line)) < bench.LINE_LIMIT
    assert len(line["ops"][2]["error"]) <= 80
    wanted = ["c3", "mm"]
    line = bench.final_line({"c3": res["c3"], "mm": res["mm"]}, wanted, 20, 5, 8)
    assert line["value"] == res["mm"]["best_us"] and line["roofline"]["bound"] == "mfma"
    only_dyn = bench.final_line({"dyn": res["dyn"]}, ["dyn"], 20, 5, 8)
    assert "ops" in only_dyn and len(json.dumps(only_dyn)) < bench.LINE_LIMIT


def test_oversized_rows_fall_back_to_fractions_only():
    many = [f"op{i}" for i in range(120)]
    res = {n: _dense(n) for n in many}
    line = bench.final_line(res, many, 20, 5, 8)
    assert len(json.dumps(line)) < 2 * bench.LINE_LIMIT and set(line["ops"][0]) == {"op", "frac"}
