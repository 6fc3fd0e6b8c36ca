"""The record bench.py prints last has to fit the driver's bounded view of stdout:
one line, under 4 KB, valid JSON, with the fields the measurement contract names.
Built here from canned numbers through the same function the benchmark uses."""
import json

import bench


def canned(rows_per_cfg=1, long_names=False):
    pad = " on a host whose processor reports a very long marketing name" * (8 if long_names else 0)
    step = [{"op": n, "bytes": 411041792, "us": 63.4, "GBps": 6486.8, "frac": 0.8108, "vs_copy": 0.99}
            for n in ("activate_relu", "activate_sigmoid", "unary_exp", "unary_abs", "unary_sqrt_of_abs",
                      "activate_tanh", "scale_relu_fused")]
    step.append({"op": "plain_copy (yardstick, not part of the step)", "bytes": 411041792, "us": 62.4,
                 "GBps": 6587.0, "frac": 0.82, "vs_copy": 1.0})
    names = (["binary_add_channel_broadcast"], ["reduce_sum_hw", "reduce_avg_hw", "reduce_max_c", "reduce_sum_all"],
             ["broadcast_%s_%s" % (o, t) for t in ("i", "ii", "iii") for o in ("mul", "sub", "div", "max")]
             + ["scalar_%s_iii" % o for o in ("mul", "sub", "div", "max")],
             ["scale", "eltwise_sum", "relu", "reduce_avg_hw", "fused_tail (CPU: the four operators)"])
    configs = []
    for cfg, ops in zip((1, 3, 4, 5), names):
        for op in ops * rows_per_cfg:
            configs.append({"cfg": cfg, "op": op, "bytes": 51380480, "us": 123456.78, "GBps": 5459.7, "frac": 0.682512,
                            "Gelem_s": 682.46, "ceiling": "copy", "ceiling_us": 9.48, "frac_of_ceiling": 1.00812,
                            "cpu_us": 241567.7, "cpu_median_us": 92555.1, "cpu_GBps": 0.555, "speedup_vs_cpu": 9831.4})
    for k in range(58):
        configs.append({"cfg": "next" if k % 2 else "movers", "op": "neighbouring operator %d with a long label" % k,
                        "bytes": 1 << 28, "us": 55.5, "GBps": 4800.0, "frac": 0.6, "Gelem_s": 900.0,
                        "ceiling": "copy", "ceiling_us": 40.0, "frac_of_ceiling": 0.72})
    for k in range(21):
        configs.append({"cfg": "ceiling", "op": "copy of %d MB" % k, "bytes": 1 << 25, "us": 9.0, "GBps": 5700.0,
                        "frac": 0.71})
    return {
        "metric": "achieved HBM GB/s (% of MI355X peak) per op; speedup vs host-CPU Shadow",
        "value": 6468.1, "unit": "GB/s", "n_gpus": 1, "steps": 20, "warmup": 5, "ms_per_step": 0.4448,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "BASELINE configs[1]: fp32 [64,256,56,56] ~N(0,2) seed 201; relu, sigmoid, exp, abs, "
                               "sqrt(abs), tanh as single ops + fused per-channel Scale+ReLU (7 launches per step); "
                               "two resident copies of the input take turns step by step",
                   "elements": 51380224, "bytes_per_step": 2877294592,
                   "device": "AMD Instinct MI355X|gfx950:sramecc+:xnack-|256|2400000" + pad},
        "frac_of_hbm_peak": 0.8085, "elements_per_s": 808507132235.6,
        "roofline": {"bound": "valu", "kernel": "activate_tanh", "achieved": 5669.3, "peak": 8000.0, "unit": "GB/s",
                     "frac": 0.7087, "traffic": 411040000, "traffic_source": "profiles/x.txt", "avg_us": 72.5,
                     "algorithmic_bytes": 411041792, "same_size_copy_us": 63.86, "time_vs_same_size_copy": 1.19,
                     "valu": {"insts_per_element": 61.3, "valu_busy": 1.22}, "valu_source": "profiles/y.txt",
                     "note": "n" * 300},
        "step_ops": step, "step_ops_note": "s" * 200,
        "cpu_baseline": {"value": 2.882, "unit": "GB/s", "cores": 1, "kind": "port", "seconds_per_step": 0.999,
                         "sample": "5 full passes of the same step on the same buffers (51.4M elements, 8 operator "
                                   "runs each, outputs allocated beforehand), best pass 1.00 s; host: AMD EPYC 9575F "
                                   "64-Core Processor, 16 logical CPUs" + pad,
                         "ops": {d["op"]: {"best_us": 22223.1, "median_us": 22300.0} for d in step}},
        "speedup_vs_cpu": 2244.3, "configs": configs, "configs_note": "c" * 400,
        "network": {"model": "m" * 90, "us_per_forward": 122.5, "operators": 6, "launches": 5, "input_copies": 2,
                    "bytes_moved": 667942912, "GBps": 5451.0},
    }


def check(line):
    assert "\n" not in line and len(line) < 4096
    rec = json.loads(line)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in rec, key
    assert rec["config"]["workload"].startswith("BASELINE configs[1]")
    roof = rec["roofline"]
    assert roof["kernel"] == "activate_tanh" and roof["frac"] == 0.7087 and roof["bound"] in ("hbm", "valu", "mfma")
    assert roof["peak"] == 8000.0 and roof["unit"] == "GB/s" and roof["traffic"] == 411040000
    cpu = rec["cpu_baseline"]
    assert cpu["value"] == 2.882 and cpu["cores"] == 1 and cpu["kind"] == "port" and cpu["sample"]
    return rec


def test_final_line_is_short_and_complete():
    rec = check(bench.final_line(canned(), "gpurun_out/bench_table.json"))
    assert rec["table"] == "gpurun_out/bench_table.json"
    assert len(rec["baseline_rows"]) == 26 and len(rec["baseline_rows_columns"]) == len(rec["baseline_rows"][0])
    assert rec["baseline_rows"][0][:2] == [1, "add_chan_bcast"]
    assert len(rec["step_ops"]) == 7
    assert "configs" not in rec and "configs_note" not in rec and "ops" not in rec["cpu_baseline"]


def test_final_line_sheds_tables_before_it_outgrows_the_limit():
    rec = check(bench.final_line(canned(rows_per_cfg=4)))
    assert "baseline_rows" not in rec or len(json.dumps(rec)) < 4096
    check(bench.final_line(canned(long_names=True)))


def test_without_the_cpu_and_config_legs_the_line_still_parses():
    full = canned()
    for k in ("cpu_baseline", "speedup_vs_cpu", "configs", "network"):
        full.pop(k)
    rec = json.loads(bench.final_line(full))
    assert "baseline_rows" not in rec and rec["roofline"]["frac"] == 0.7087


def test_more_than_one_gpu_is_refused(monkeypatch):
    import pytest
    monkeypatch.setattr("sys.argv", ["bench.py", "--gpus", "2"])
    with pytest.raises(SystemExit) as e:
        bench.main()
    assert "one GPU" in str(e.value)
