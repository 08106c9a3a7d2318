"""The benchmark's record is the last line of its stdout, and whoever runs it may keep only the tail
of that stream: the line must stay a few kB of strict JSON whatever the tables beside it grow to."""
import json
import os

import bench


def fake_record(tmp_path, nan=False):
    roofline = dict(bound="hbm", achieved=6345.1, peak=8000.0, unit="GB/s", frac=0.7931, traffic=411337696,
                    traffic_source="x" * 120, kernel="epilogue_fwd_kernel<PXH_LEAKY, true, *>",
                    bytes_per_launch=411378834, mean_launch_ms=0.06483)
    cpu = dict(value=0.693, unit="GB/s", cores=1, kind="port", sample="s" * 100, host_cpus=16)
    model_order = dict(total_ms=float("nan") if nan else 13.846, leanest_total_ms=10.96, forward_ms=4.8,
                       phases={"p%d" % i: i * 0.1 for i in range(200)})
    config0 = dict(gpu_graph_ms=0.068, cpu_ms=42.8, by_kind={"k%d" % i: 1.0 for i in range(50)})
    details = dict(extras=[dict(kernel="k%d" % i, shape="16x256x76^2", ms=0.1, note="n" * 80) for i in range(400)],
                   per_shape=[dict(act="leaky", ms=0.1)] * 21, model_order=model_order, config0=config0,
                   bad=float("inf"))
    path = bench.write_details(details, folder=str(tmp_path))
    line = bench.final_line(50, 20, 6215.8, 1.3898, 8638955520.0, 21, roofline, cpu, model_order, 9.948, 6154.0,
                            6342.0, config0, details_file=path)
    return line, path


def test_final_line_is_small_strict_json_whatever_the_tables_hold(tmp_path):
    line, path = fake_record(tmp_path)
    assert "\n" not in line and len(line) < bench.MAX_LINE_BYTES
    rec = json.loads(line)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in rec, key
    assert rec["roofline"]["frac"] == 0.7931 and rec["cpu_baseline"]["cores"] == 1
    assert rec["noconv_ms_per_batch_yolov3_608"] == 13.846
    assert rec["n_gpus"] == 1 and rec["vs_baseline"] is None and "workload" in rec["config"]
    # value x ms_per_step is the step's bytes
    assert abs(rec["value"] * 1e9 * rec["ms_per_step"] * 1e-3 / rec["config"]["bytes_per_step"] - 1.0) < 1e-3
    # the tables are in the file the line names
    with open(os.path.join(bench.ROOT, path)) as f:
        details = json.load(f)
    assert len(details["extras"]) == 400 and details["bad"] is None


def test_final_line_has_no_nan(tmp_path):
    line, _ = fake_record(tmp_path, nan=True)
    assert "NaN" not in line and json.loads(line)["noconv_ms_per_batch_yolov3_608"] is None
