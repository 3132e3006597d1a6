"""The one line that bench.py prints: its keys, their kinds and how the figures hang together.
The refusal of more than one GPU runs anywhere; the measurement itself (two layers of the headline
shape, a few steps) needs the GPU."""
import io
import json
import sys
from contextlib import redirect_stdout

import pytest

import bench


def run_bench(arguments):
    saved = sys.argv
    sys.argv = ["bench.py"] + arguments
    captured = io.StringIO()
    try:
        with redirect_stdout(captured):
            code = bench.main()
    finally:
        sys.argv = saved
    return code, captured.getvalue()


def test_more_than_one_gpu_is_refused_in_one_line():
    code, printed = run_bench(["--gpus", "2"])
    assert code == 2
    assert len(printed.strip().splitlines()) == 1 and "--gpus 2" in printed


@pytest.mark.gpu
def test_line_of_a_short_run():
    code, printed = run_bench(["--layers", "2", "--steps", "3", "--warmup", "2"])
    assert code == 0
    lines = [line for line in printed.splitlines() if line.startswith("{")]
    assert len(lines) == 1
    record = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "prefill", "roofline", "points"):
        assert key in record, key
    assert record["n_gpus"] == 1 and record["steps"] == 3 and record["warmup"] == 2
    assert record["higher_is_better"] is True and record["dtype"] == "bf16" and record["data"] == "synthetic"
    config = record["config"]
    assert len(config) <= 20 and all(not isinstance(value, (dict, list)) for value in config.values())
    assert config["layers"] == 2 and config["layers_of_configuration"] == bench.SHAPES["0.5b"]["num_hidden_layers"]
    assert config["global_batch"] == 8 and config["seq_len"] == bench.CONTEXT
    # tokens a second is the batch over the step's time
    assert record["value"] == pytest.approx(8 / (record["ms_per_step"] * 1e-3), rel=1e-3)
    prefill = record["prefill"]
    assert set(prefill) == {"value", "tokens", "ms", "frac"} and prefill["tokens"] == bench.PREFILL_TOKENS
    assert prefill["value"] == pytest.approx(prefill["tokens"] / (prefill["ms"] * 1e-3), rel=1e-3)
    assert 0.0 < prefill["frac"] < 1.0
    roofline = record["roofline"]
    assert roofline["bound"] == "hbm" and roofline["unit"] == "GB/s" and roofline["peak"] == 8000.0
    assert roofline["frac"] == pytest.approx(roofline["achieved"] / roofline["peak"], abs=1e-4)
    assert 0.0 < roofline["frac"] < 1.0
    assert set(record["points"]) == {"decode_b1", "decode_b64"}
    assert record["points"]["decode_b1"] < record["value"] < record["points"]["decode_b64"]
