"""The benchmark's result line: small enough for a line-oriented reader, with the roofline and the
CPU baseline at its end.  No GPU: the line is assembled from synthetic measurements."""
import argparse
import json
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

import bench  # noqa: E402


def _table(n):
    recs = []
    for i in range(n):
        op = "stream_copy" if i < 13 else f"layernorm_bwd_two_streams_{i}"
        recs.append({"op": op, "config": f"small [8192,768] bf16, row pass timed, sums on a second stream {i}",
                     "algorithmic_bytes": 37823488, "ms_warm": 0.01234, "ms_cold": 0.01399, "ms_cold_per_call_events": 0.0161,
                     "gbps_warm": 3065.1, "gbps_cold": 2703.6, "frac_cold": 0.338, "buffer_sets": 17, "calls_per_batch": 40,
                     "copy_ms_same_bytes": 0.00734, "frac_of_copy": 0.525, "cpu_ms": 3.61,
                     "cpu_path": "ATen CPU ops of the reference's task body, fp32, 16 threads"})
    return recs


def _line(n_rows):
    args = argparse.Namespace(steps=20, warmup=5)
    head = {"ms_per_step": 0.28761, "rows_kernel_ms_avg": 0.2838, "rows_kernel_ms_median": 0.2835, "buffers": 25,
            "loss": 12.31415, "seconds": 0.0057522}
    cpu = {"value": 6.383, "unit": "GB/s", "cores": 16, "kind": "port", "sample": "x" * 300, "ms": 258.0}
    return bench.result_line(args, head, 5726.3, 5803.1, cpu, _table(n_rows))


def test_result_line_is_short_and_complete():
    line = _line(60)
    text = json.dumps(line)
    assert len(text) < 8192, len(text)
    back = json.loads(text)
    assert back["roofline"]["frac"] > 0 and back["cpu_baseline"]["value"] > 0
    assert len(back["per_op"]) == 60 and "per_op_truncated" not in back
    assert set(back["per_op"][0]) == {"op", "cfg", "ms", "frac"}
    # what a reader of the end of the line sees: per_op comes first, the two objects after it
    assert text.index('"per_op"') < text.index('"roofline"') < text.index('"cpu_baseline"')
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config"):
        assert key in back


def test_result_line_sheds_calibration_rows_before_it_grows():
    line = _line(400)
    text = json.dumps(line)
    assert len(text) <= bench.MAX_LINE_BYTES
    assert line["per_op_truncated"] is True
    assert not any(r["op"].startswith("stream_") for r in line["per_op"])
    assert line["roofline"]["frac"] > 0 and line["cpu_baseline"]["value"] > 0
