"""bench.py's one JSON line must survive a reader that keeps only the last 8 KB of the output:
it stays below bench.LINE_LIMIT with every row present, and the schedule figures come last."""
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import bench  # noqa: E402


def _fake_line():
    m_head = {"ms_per_step": 0.483217, "settle_launches": 620, "settle_ms": 303.12, "settle_ended_by": "converged",
              "cold_ms_per_step": 0.9312, "timed_blocks": 200, "block_ms_min": 0.4801, "block_ms_max": 0.4999, "timed_region_s": 0.213}
    other = {name: {"ms_per_step": 0.8123, "tflops": 1234.56, "pct_of_bf16_mfma_peak": 49.38, "launches_per_step": 36, "avg_launch_us": 22.56}
             for name in ("rank", "step")}
    other["rank_flags"] = {"ms_per_step": 0.5612, "tflops": 1234.56, "launches_per_step": 8, "faulted": False}
    cpu = {"value": 0.3513, "unit": "TFLOP/s", "cores": 128, "kind": "port",
           "sample": "backward pairs [1,2048,16,128]: 1 d 1289 ms + 1 f 1250 ms measured, x 16 d + 120 f = 1134.6 s"}
    rows = {}
    for name, spec in bench.ROW_SPECS.items():
        rows[name] = bench.make_row(name, 13.148612, 12345.67, **{k: 12345.678 for k in spec[5]})
        rows[name]["cpu_baseline"] = dict(cpu)
    host = {"logical": 256, "physical": 128, "affinity": 128, "omp_num_threads_env": "128", "torch_num_threads": 128}
    src = "recorded: profiles/flash_fwd_traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by a 1 GiB copy)"
    return bench.assemble_line(20, 5, "all", m_head, other, rows, dict(cpu), host, 565112827, src)


def test_line_fits_the_tail_a_reader_keeps():
    text = json.dumps(_fake_line())
    assert len(text) < bench.LINE_LIMIT, len(text)


def test_schedule_figures_come_last_and_rows_are_complete():
    line = _fake_line()
    keys = list(line)
    assert keys[-3:] == ["other_schedules", "ring_step", "protocol"]
    assert keys.index("rows") < keys.index("other_schedules")
    assert [r["row"] for r in line["rows"]] == list(bench.ROW_SPECS)
    assert set(bench.ROW_NOTES) == set(bench.ROW_SPECS)
    for r in line["rows"]:
        assert {"bound", "achieved", "peak", "unit", "frac", "traffic"} <= set(r["roofline"])
        assert {"value", "unit", "cores", "kind", "sample"} <= set(r["cpu_baseline"])
    # the contract keys of the driver, and the two schedules again inside `roofline`
    for k in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline",
              "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert k in line, k
    assert line["roofline"]["rank_tflops"] == 1234.56 and line["roofline"]["step_tflops"] == 1234.56
    assert line["protocol"]["settle_ended_by"] in ("converged", "cap")
    assert line["ring_step"]["flag_driven_tflops"] == 1234.56


def test_more_than_one_gpu_is_refused():
    import subprocess
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode == 2 and "one GPU" in r.stderr
