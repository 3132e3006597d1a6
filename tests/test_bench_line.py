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


def test_the_shape_is_written_as_a_config_json(tmp_path):
    """What the kernel-trace summary reads as --config: the shape's keys with the number of layers asked for,
    and the configuration class reads it back."""
    from macllm_infer_amd.config.registry import config_from_dict
    path = tmp_path / "config.json"
    code, printed = run_bench(["--shape", "7b", "--layers", "12", "--write-config", str(path)])
    assert code == 0 and printed == ""
    raw = json.loads(path.read_text())
    assert raw == dict(bench.SHAPES["7b"], num_hidden_layers=12)
    spec = config_from_dict(raw).to_model_spec()
    assert len(spec.layers) == 12 and spec.hidden_size == 3072


@pytest.mark.gpu
def test_line_of_a_short_run():
    code, printed = run_bench(["--layers", "2", "--steps", "20", "--warmup", "2"])
    assert code == 0
    lines = [line for line in printed.splitlines() if line.startswith("{")]
    assert len(lines) == 1
    record = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "prefill", "roofline", "points"):
        assert key in record, key
    assert record["n_gpus"] == 1 and record["steps"] == 20 and record["warmup"] == 2
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
    # the bytes are those the step has to read (every weight once, the cache and state of its requests)
    assert roofline["achieved"] == pytest.approx(record["bytes"]["read_mb"] / record["ms_per_step"], rel=2e-3)
    assert 0 < record["bytes"]["written_mb"] < record["bytes"]["read_mb"]
    times = record["step_ms"]
    assert set(times) == {"mean", "p50", "p95"} and 0 < times["p50"] <= times["p95"]
    # a step is queued before the tokens of the one before are read, so a step's own time runs from one step's
    # tokens to the next's, and the last step's work ends after the last of these times: 1 part in 20 here
    assert 0.85 * record["ms_per_step"] <= times["mean"] <= 1.02 * record["ms_per_step"]
    assert record["prefill_uncaptured_ms"] >= 0.9 * prefill["ms"]
    # the same prompt through the true 32-bit path: slower than bfloat16, against the float32 peak
    wide = record["prefill_f32"]
    assert set(wide) == {"value", "tokens", "ms", "frac"} and wide["tokens"] == bench.PREFILL_TOKENS
    assert wide["ms"] > prefill["ms"] and 0.0 < wide["frac"] < 1.0
    assert {"in", "out", "gate_up", "down"} <= set(record["choices"])
    long_points = {f"decode_b{batch}_ctx{context}" for batch, context in bench.LONG_POINTS}
    assert set(record["points"]) == {"decode_b1", "decode_b64"} | long_points == set(record["points_frac"])
    assert record["points"]["decode_b1"] < record["value"] < record["points"]["decode_b64"]
    # a longer context costs time and raises the fraction of the bandwidth (more bytes beside the same latencies;
    # with the two layers of this run the points among themselves are within noise of each other)
    assert record["points_frac"]["decode_b8_ctx32768"] > record["roofline"]["frac"]
    assert all(0.0 < value < 1.0 for value in record["points_frac"].values())


@pytest.mark.gpu
def test_microbench_line():
    code, printed = run_bench(["--microbench"])
    assert code == 0
    record = json.loads([line for line in printed.splitlines() if line.startswith("{")][0])
    assert 1000.0 < record["read_modify_write_gbs"] < 8000.0 and 1000.0 < record["read_gbs"] < 8000.0
    assert record["read_frac"] == pytest.approx(record["read_gbs"] / 8000.0, abs=1e-3)


def test_costs_of_the_headline_step_are_the_ones_worked_out_by_hand():
    """Falcon-H1-0.5B shape: 974.8 MB of weights; at 2,048 tokens a request reads 37.7 MB of keys and values,
    28.3 MB of state and 0.4 MB of conv tails; a 2,048-token prompt is 2.10 TFLOP."""
    from macllm_infer_amd.config import FalconH1Config
    from macllm_infer_amd.utils import costs
    spec = FalconH1Config.from_dict(bench.SHAPE).to_model_spec()
    step = costs.decode_step_costs(spec, 8, 2048.0)
    weights = sum(step[name].read for name in step if name != "mixers")
    assert weights == pytest.approx(974.8e6, rel=1e-3)
    assert step["mixers"].read / 8 == pytest.approx(37.75e6 + 28.31e6 + 0.39e6, rel=2e-3)
    assert step["mixers"].written / 8 == pytest.approx(28.31e6 + 0.39e6 + 36 * 2 * 2 * 64 * 2, rel=2e-3)
    assert costs.total(costs.prefill_costs(spec, 2048)).flops == pytest.approx(2.10e12, rel=2e-3)
    assert costs.group_of("void fused_gemm_kernel<1, 0, 2, 4, 1>(FusedGemmParams)", costs.DECODE_GROUPS) == "input projections"
    assert costs.group_of("void fused_gemm_kernel<1, 1, 0, 8, 1>(FusedGemmParams)", costs.DECODE_GROUPS) \
        == "output projections + down projections"
    assert costs.group_of("void fused_gemm_kernel<1, 1, 0, 8, 1>(FusedGemmParams)", costs.DECODE_GROUPS, calls=1) == "output head"
    for kernel in ("void fused_gemm_kernel<4, 1, 3, 8, 1>(FusedGemmParams)", "void fused_gemm_kernel<1, 2, 0, 8, 1>(FusedGemmParams)",
                   "void shared_rows_gemm_kernel<4, 1, 0>(FusedGemmParams)"):
        assert costs.group_of(kernel, costs.DECODE_GROUPS, calls=1) == "output projections + down projections"
    assert costs.group_of("void shared_rows_gemm_kernel<3, 2, 1>(FusedGemmParams)", costs.DECODE_GROUPS) == "gate and up projections"
    assert costs.group_of("void shared_rows_gemm_kernel<3, 2, 2>(FusedGemmParams)", costs.DECODE_GROUPS) == "input projections"
    assert costs.group_of("Cijk_Alik_Bljk_BBS_BH", costs.DECODE_GROUPS) is None
    assert costs.merged(step, "output projections + down projections").read == pytest.approx(302.0e6, rel=1e-3)


def test_kernel_trace_summary_of_a_made_up_trace(tmp_path, capsys):
    """``utils.kernel_trace`` on a small made-up trace database: the last step from its first kernel to its last,
    launches, busy time and span, the kernels by total time, the roofline table from a model's sizes, and the
    launches one by one with the idle time before each."""
    import sqlite3
    from macllm_infer_amd.utils import kernel_trace
    database = tmp_path / "trace.db"
    connection = sqlite3.connect(database)
    connection.execute("create table kernels (name text, start integer, end integer)")
    rows = []
    for step in range(2):                                     # two steps; the second one is summarized
        base = 1_000_000 * step
        rows += [("embed_kernel", base, base + 4_000),
                 ("void fused_gemm_kernel<1, 0, 2, 4, 1>(FusedGemmParams)", base + 4_000, base + 12_000),
                 ("void mixer_decode_kernel<64>(MixerParams)", base + 12_000, base + 24_000),
                 ("side_kernel", base + 13_000, base + 15_000),                 # beside the mixer, on another queue
                 ("void fused_gemm_kernel<1, 0, 2, 4, 1>(FusedGemmParams)", base + 30_000, base + 38_000),
                 ("argmax_kernel(float const*, int, int*)", base + 38_000, base + 45_000)]
    connection.executemany("insert into kernels values (?, ?, ?)", rows)
    connection.commit()
    connection.close()
    config = tmp_path / "config.json"
    config.write_text(json.dumps(dict(bench.SHAPES["0.5b"], num_hidden_layers=1)))
    saved = sys.argv
    sys.argv = ["kernel_trace", str(database), "--first", "embed_kernel", "--last", "argmax", "--config", str(config),
                "--batch", "8", "--context", "2060", "--timeline", "0:6"]
    try:
        kernel_trace.main()
    finally:
        sys.argv = saved
    printed = capsys.readouterr().out
    assert "launches 6   busy 41.0 us   span 45.0 us" in printed
    lines = printed.splitlines()
    first = next(line for line in lines if line.startswith("void fused_gemm_kernel"))
    assert first.split()[-4:] == ["2", "16.0", "8.00", "39.0%"]                   # calls, total, average, share
    assert any(line.startswith("input projections") for line in lines) and any("the step (all kernels" in line for line in lines)
    timeline = [line.split() for line in lines if line.strip() and line.split()[0].isdigit()]
    assert [row[0] for row in timeline] == ["0", "1", "2", "3", "4", "5"]
    assert timeline[3][3] == "-11.00" and timeline[4][3] == "6.00"              # beside the mixer; a gap of 6 us before the next
