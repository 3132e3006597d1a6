"""The step function, cache manager and scheduler with the kernels replaced by their plain
PyTorch references (tests/ref_ops.py), on the CPU: what the host code does with pages,
slots, lanes and rows, compared with the plain whole-sequence implementation."""
import pytest
import torch

import plain_impl
import ref_ops
import tiny_configs
from macllm_infer_amd.cache import CacheExhausted
from macllm_infer_amd.engine import Engine, EngineConfig, Lane, Scheduler, StepError
from macllm_infer_amd.sampling import Sampler, SamplingParams


@pytest.fixture
def host_ops(monkeypatch):
    ref_ops.install(monkeypatch)


def engine_for(name, folder, capacity=256, page=8, requests=4):
    tiny_configs.make_model_dir(name, folder)
    cfg, tensors = plain_impl.load_model_dir(str(folder))
    engine = Engine(str(folder), dtype="float32", device="cpu", kv_cache_block_tokens=page,
                    kv_cache_capacity_tokens=capacity, max_active_sequences=requests, check_device=False)
    return engine, cfg, tensors


def tokens_for(cfg, count, seed):
    return torch.randint(0, cfg["vocab_size"], (count,), generator=torch.Generator().manual_seed(seed)).tolist()


@pytest.mark.parametrize("name", ["A", "B"])
def test_whole_chunked_and_mixed_match_the_plain_model(host_ops, tmp_path, name):
    engine, cfg, tensors = engine_for(name, tmp_path, capacity=96, page=8)
    first, second = tokens_for(cfg, 45, 1), tokens_for(cfg, 30, 2)
    want_first = plain_impl.falcon_h1_logits(cfg, tensors, first)
    want_second = plain_impl.falcon_h1_logits(cfg, tensors, second)
    engine.add_request("whole")
    got = engine.step([Lane("whole", first, list(range(45)))])
    assert (got - want_first).abs().max() < 1e-4
    engine.finish("whole")
    engine.add_request("cut")
    outputs, cursor = [], 0
    for size in [7, 2, 5, 3, 11, 2, 1, 1, 13]:
        outputs.append(engine.step([Lane("cut", first[cursor:cursor + size], list(range(size)))]))
        cursor += size
    assert (torch.cat(outputs) - want_first).abs().max() < 1e-4
    engine.finish("cut")
    engine.add_request("c")
    engine.add_request("d")
    one = engine.step([Lane("c", first[:20], [19]), Lane("d", second[:3], [0, 1, 2])])
    two = engine.step([Lane("d", second[3:30], list(range(27))), Lane("c", first[20:21], [0])])
    assert (one[0] - want_first[19]).abs().max() < 1e-4 and (one[1:] - want_second[:3]).abs().max() < 1e-4
    assert (two[:27] - want_second[3:30]).abs().max() < 1e-4 and (two[27] - want_first[20]).abs().max() < 1e-4
    engine.cache.check()


def test_portions_beside_several_decoded_tokens_run_as_two_batches_in_the_callers_order(host_ops, tmp_path, monkeypatch):
    """A step that holds portions of prompts beside four or more single tokens is queued as two batches (the
    portions, then the single tokens); the logits come back in the order of the lanes and of their wanted
    places, whatever that order is, and are the plain model's.  A step that is refused is refused whole."""
    engine, cfg, tensors = engine_for("A", tmp_path, capacity=400, page=8, requests=7)
    assert engine.split_from_lanes == 4
    batches = []
    real = engine._run
    monkeypatch.setattr(engine, "_run", lambda lanes, lowered: (batches.append([lane.request for lane in lanes]), real(lanes, lowered))[1])
    streams = {key: tokens_for(cfg, 40, 30 + index) for index, key in enumerate("abcdefg")}
    wants = {key: plain_impl.falcon_h1_logits(cfg, tensors, tokens) for key, tokens in streams.items()}
    for key in streams:
        engine.add_request(key)
    engine.step([Lane(key, streams[key][:10], []) for key in "abcde"])                  # five requests that decode
    assert batches == [list("abcde")]
    batches.clear()
    # portions of f and g between the single tokens of a..e; f wants two places, g none, d none
    lanes = [Lane("a", streams["a"][10:11], [0]), Lane("f", streams["f"][:12], [3, 11]), Lane("b", streams["b"][10:11], [0]),
             Lane("c", streams["c"][10:11], [0]), Lane("g", streams["g"][:7], []), Lane("d", streams["d"][10:11], []),
             Lane("e", streams["e"][10:11], [0])]
    got = engine.step(lanes)
    assert batches == [["f", "g"], ["a", "b", "c", "d", "e"]]
    expected = [wants["a"][10], wants["f"][3], wants["f"][11], wants["b"][10], wants["c"][10], wants["e"][10]]
    assert got.shape[0] == len(expected)
    for row, want in enumerate(expected):
        assert (got[row] - want).abs().max() < 1e-4, row
    # three single tokens beside a portion stay one batch
    batches.clear()
    got = engine.step([Lane("a", streams["a"][11:12], [0]), Lane("g", streams["g"][7:20], [12]), Lane("b", streams["b"][11:12], [0]),
                       Lane("c", streams["c"][11:12], [0])])
    assert batches == [["a", "g", "b", "c"]]
    for row, want in enumerate([wants["a"][11], wants["g"][19], wants["b"][11], wants["c"][11]]):
        assert (got[row] - want).abs().max() < 1e-4, row
    # a token outside the vocabulary in the portion: nothing runs, nothing changes
    batches.clear()
    before = engine.cache.stats()
    with pytest.raises(StepError):
        engine.step([Lane(key, streams[key][12:13], [0]) for key in "abcd"] + [Lane("f", [cfg["vocab_size"]] * 3, [])])
    assert batches == [] and engine.cache.stats() == before
    engine.cache.check()


def test_refused_steps_change_nothing(host_ops, tmp_path):
    engine, cfg, tensors = engine_for("A", tmp_path, capacity=32, page=8, requests=2)
    engine.add_request("a")
    tokens = tokens_for(cfg, 40, 3)
    engine.step([Lane("a", tokens[:10], [9])])
    before = engine.cache.stats()
    for lanes, error in [
            ([Lane("a", [], [])], StepError), ([Lane("ghost", [1], [])], StepError),
            ([Lane("a", [1], []), Lane("a", [2], [])], StepError), ([Lane("a", [256], [])], StepError),
            ([Lane("a", [-1], [])], StepError), ([Lane("a", [1, 2], [2])], StepError), ([], StepError),
            ([Lane("a", tokens[10:40], [])], CacheExhausted)]:          # 40 tokens > 32 of capacity
        with pytest.raises(error):
            engine.step(lanes)
        assert engine.cache.stats() == before and engine.length("a") == 10
    # and the request goes on as if nothing had happened
    want = plain_impl.falcon_h1_logits(cfg, tensors, tokens[:12])
    got = engine.step([Lane("a", tokens[10:12], [0, 1])])
    assert (got - want[10:12]).abs().max() < 1e-4
    with pytest.raises(StepError, match="context limit"):
        engine.max_context = 12
        engine.step([Lane("a", [1], [])])


def test_pages_and_slots_are_used_again_without_leaking_state(host_ops, tmp_path):
    """A pool for one request at a time: each new request gets the pages and the slot the last
    one gave back, and its logits are those of a fresh sequence."""
    engine, cfg, tensors = engine_for("B", tmp_path, capacity=40, page=8, requests=1)
    for seed in range(3):
        tokens = tokens_for(cfg, 33 + seed, 10 + seed)
        engine.add_request(seed)
        got = engine.step([Lane(seed, tokens[:20], [19])])
        got = torch.cat([got, engine.step([Lane(seed, tokens[20:], [len(tokens) - 21])])])
        want = plain_impl.falcon_h1_logits(cfg, tensors, tokens)
        assert (got - want[[19, len(tokens) - 1]]).abs().max() < 1e-4
        engine.finish(seed)
    assert engine.cache.stats()["groups"][0]["free_pages"] == 5


@pytest.mark.parametrize("name", ["A", "B"])
def test_scheduler_greedy_generation_equals_the_plain_model(host_ops, tmp_path, name):
    engine, cfg, tensors = engine_for(name, tmp_path, capacity=160, page=8, requests=3)
    sampler = Sampler(engine.vocab_size, "cpu", check_device=False)
    scheduler = Scheduler(engine, sampler, EngineConfig(max_active_sequences=3, scheduler_token_budget=16,
                                                        prefill_token_quantum=11))
    prompts = [tokens_for(cfg, length, 20 + length) for length in (5, 17, 33)]
    params = SamplingParams(max_new_tokens=6, temperature=0.0, top_k=0, top_p=1.0, repetition_penalty=1.0)
    for index, prompt in enumerate(prompts):
        scheduler.submit(index, prompt, params)
    finished = scheduler.run()
    for index, prompt in enumerate(prompts):
        assert finished[index].generated == plain_impl.greedy_generate(cfg, tensors, prompt, 6)
    stats = engine.cache.stats()
    assert stats["live_requests"] == 0 and stats["free_slots"] == 3


def test_scheduler_seeded_sampling_equals_the_plain_sampler(host_ops, tmp_path):
    engine, cfg, tensors = engine_for("B", tmp_path, capacity=256, page=8, requests=4)
    sampler = Sampler(engine.vocab_size, "cpu", check_device=False)
    scheduler = Scheduler(engine, sampler, EngineConfig(max_active_sequences=4, scheduler_token_budget=24,
                                                        prefill_token_quantum=11))
    prompts = [tokens_for(cfg, length, 40 + length) for length in (1, 7, 24)]
    params = [SamplingParams(max_new_tokens=5, temperature=0.8, top_k=0, top_p=1.0, repetition_penalty=1.0, seed=3),
              SamplingParams(max_new_tokens=5, temperature=0.9, top_k=12, top_p=0.7, repetition_penalty=1.3, seed=4),
              SamplingParams(max_new_tokens=5, temperature=1.1, top_k=0, top_p=0.9, presence_penalty=0.4,
                             frequency_penalty=0.2, repetition_penalty=1.0, seed=5)]
    for index, prompt in enumerate(prompts):
        scheduler.submit(index, prompt, params[index])
    finished = scheduler.run()
    for index, prompt in enumerate(prompts):
        p = params[index]
        tokens, generated = list(prompt), []
        for draw in range(5):
            logits = plain_impl.falcon_h1_logits(cfg, tensors, tokens)[-1]
            token = plain_impl.sample_token(
                logits, temperature=p.temperature, top_k=p.top_k, top_p=p.top_p,
                repetition_penalty=p.repetition_penalty, presence_penalty=p.presence_penalty,
                frequency_penalty=p.frequency_penalty, history=tokens, generated=generated, seed=p.seed,
                draw_index=draw)
            tokens.append(token)
            generated.append(token)
        assert finished[index].generated == generated


@pytest.mark.parametrize("schedule", __import__("toy_parts").SCHEDULES, ids=__import__("toy_parts").SCHEDULE_IDS)
def test_toy_parts_register_build_and_step_on_the_host(host_ops, schedule):
    """The framework's generality without a GPU: a mixer with state of its own, another
    position encoding, a window, a layer that runs twice and a run that reads another run's
    cache, registered from the tests and stepped through the engine."""
    import toy_parts
    toy_parts.exercise(schedule, "cpu", check_device=False)


def test_a_mixer_declares_a_step_table_of_its_own_on_the_host(host_ops):
    """A toy mixer, registered from the tests, names an index table of its own; the step carries it, written by the
    mixer's function from the step's lanes, and the model says what the plain one says."""
    import toy_parts
    del toy_parts.TABLE_FILLS[:]
    engine = toy_parts.exercise_step_table("cpu", check_device=False, graphs=False)
    assert (2, 14) in toy_parts.TABLE_FILLS and (3, 3) in toy_parts.TABLE_FILLS
    assert engine.graphs is None


def test_a_step_that_fails_once_launched_ends_its_requests_and_leaves_the_others_alone(host_ops, tmp_path, monkeypatch):
    """A kernel refuses in the second layer, after the first has written keys, values and state in place:
    the requests of that step are ended and give back pages and slots (the reference restores a checkpoint
    instead, src/decoder.rs:4146-4190); a request that was not in the step goes on and still matches."""
    from macllm_infer_amd import StepFailed
    from macllm_infer_amd.kernels import ops
    engine, cfg, tensors = engine_for("B", tmp_path, capacity=96, page=8, requests=3)
    bystander, first, second = tokens_for(cfg, 30, 1), tokens_for(cfg, 20, 2), tokens_for(cfg, 9, 3)
    for name in ("bystander", "first", "second"):
        engine.add_request(name)
    engine.step([Lane("bystander", bystander[:17], []), Lane("first", first[:12], [11])])
    free_before = engine.cache.stats()["groups"][0]["free_pages"]
    held = {name: len(engine.cache.table(0, name).live_pages()) for name in ("first", "bystander")}
    real, calls = ops.gate_norm, {"count": 0}

    def refuses_in_the_second_layer(*arguments, **named):
        calls["count"] += 1
        if calls["count"] == 2:
            raise ops.KernelError("gate_norm: size not supported by this kernel")
        return real(*arguments, **named)

    monkeypatch.setattr(ops, "gate_norm", refuses_in_the_second_layer)
    with pytest.raises(StepFailed) as caught:
        engine.step([Lane("first", first[12:], [7]), Lane("second", second, [8])])
    assert caught.value.requests == ["first", "second"] and isinstance(caught.value.__cause__, ops.KernelError)
    assert not engine.has_request("first") and not engine.has_request("second") and engine.has_request("bystander")
    stats = engine.cache.stats()
    assert stats["groups"][0]["free_pages"] == free_before + held["first"] and stats["free_slots"] == 2
    engine.cache.check()
    monkeypatch.setattr(ops, "gate_norm", real)
    want = plain_impl.falcon_h1_logits(cfg, tensors, bystander)
    got = engine.step([Lane("bystander", bystander[17:], list(range(13)))])
    assert (got - want[17:]).abs().max() < 1e-4
    # the names are free again: the same request can start over in the slot and pages it gave back
    engine.add_request("first")
    got = engine.step([Lane("first", first, [19])])
    assert (got - plain_impl.falcon_h1_logits(cfg, tensors, first)[[19]]).abs().max() < 1e-4


def test_the_scheduler_fails_the_requests_of_a_failed_step_and_serves_the_rest(host_ops, tmp_path, monkeypatch):
    from macllm_infer_amd.kernels import ops
    engine, cfg, tensors = engine_for("A", tmp_path, capacity=160, page=8, requests=3)
    sampler = Sampler(engine.vocab_size, "cpu", check_device=False)
    scheduler = Scheduler(engine, sampler, EngineConfig(max_active_sequences=1, scheduler_token_budget=64,
                                                        prefill_token_quantum=64))
    prompts = [tokens_for(cfg, length, 70 + length) for length in (9, 14)]
    params = SamplingParams(max_new_tokens=4, temperature=0.0, top_k=0, top_p=1.0, repetition_penalty=1.0)
    for index, prompt in enumerate(prompts):
        scheduler.submit(index, prompt, params)
    real, calls = ops.swiglu, {"count": 0}

    def refuses_once(*arguments, **named):
        calls["count"] += 1
        if calls["count"] == 4:                  # the second decode step of request 0 (two layers a step)
            raise ops.KernelError("swiglu: bad argument")
        return real(*arguments, **named)

    monkeypatch.setattr(ops, "swiglu", refuses_once)
    finished = scheduler.run()
    assert finished[0].finish_reason.startswith("failed: swiglu") and len(finished[0].generated) == 1
    assert finished[1].finish_reason == "length"
    assert finished[1].generated == plain_impl.greedy_generate(cfg, tensors, prompts[1], 4)
    stats = engine.cache.stats()
    assert stats["live_requests"] == 0 and stats["free_slots"] == 3
    engine.cache.check()


@pytest.mark.parametrize("change, word", [
    ({"mamba_d_conv": 17}, "'mamba_d_conv' = 17"),
    ({"mamba_d_state": 520}, "'mamba_d_state' = 520"),
    ({"head_dim": 258}, "'head_dim' = 258"),
    ({"hidden_size": 16416, "num_attention_heads": 6}, "'hidden_size' = 16416"),
    ({"mamba_d_conv": 20, "head_dim": 300}, "'head_dim' = 300.*'mamba_d_conv' = 20"),
])
def test_sizes_no_kernel_takes_are_refused_before_a_weight_is_read(change, word):
    """The limits are the kernels' own (a test below reads them in the sources); the error names the
    config.json key; ``tensors=None`` shows that no weight was asked for."""
    from macllm_infer_amd.config import ConfigError
    raw = dict(tiny_configs.TINY_B)
    raw.update(change)
    with pytest.raises(ConfigError, match=word):
        Engine(config=raw, tensors=None, dtype="float32", device="cpu", check_device=False)
    for dtype in ("float32", "bfloat16"):
        with pytest.raises(ConfigError, match="more than the kernels take"):
            Engine(config=raw, tensors=None, dtype=dtype, device="cpu", check_device=False)


def test_the_limits_are_the_ones_in_the_kernel_sources():
    import os
    import re
    from macllm_infer_amd.kernels import build, limits

    def define(module, name):
        with open(os.path.join(build.CSRC, f"{module}.hip")) as handle:
            return int(re.search(rf"#define {name} (\d+)", handle.read()).group(1))

    assert limits.ATTENTION_MAX_HEAD_DIM == define("attention", "ATT_MAX_DH")
    assert limits.CONV_MAX_TAPS == define("mamba2", "CONV_MAX_K")
    assert limits.SCAN_MAX_STATE == 64 * define("mamba2", "SCAN_MAX_PER_THREAD")
    with open(os.path.join(build.CSRC, "common.hip")) as handle:
        assert "(size_t)d * sizeof(float) > 64 * 1024" in handle.read()
    assert limits.NORM_MAX_WIDTH * 4 == 64 * 1024
    # and the sizes at the limits are accepted
    raw = dict(tiny_configs.TINY_B, mamba_d_conv=16, mamba_d_state=512, head_dim=256)
    from macllm_infer_amd.config import FalconH1Config
    from macllm_infer_amd.engine.model import DecoderModel
    assert DecoderModel.limits(FalconH1Config.from_dict(raw).to_model_spec()) == []


def test_a_round_ahead_of_its_tokens_ends_requests_like_a_round_that_waits(host_ops, tmp_path):
    """The scheduler that queues a round before it has read the tokens of the round before (tokens fed on the
    device) and the one that reads every token first: the same tokens, finish reasons and callbacks for
    requests that end by a stop token, by the caller's ``on_token``, by a cancellation, by their length, for a
    request with penalties (it waits for its tokens) and under a budget that leaves requests out of rounds.
    A request that ended one round earlier than the host knew has run one token too far: nothing of it shows,
    and every page and slot comes back."""
    engine, cfg, tensors = engine_for("B", tmp_path, capacity=512, page=8, requests=5)
    prompts = [tokens_for(cfg, length, 70 + length) for length in (3, 9, 20, 5, 14, 6)]
    greedy = dict(temperature=0.0, top_k=0, top_p=1.0, repetition_penalty=1.0)
    free = [plain_impl.greedy_generate(cfg, tensors, prompt, 9) for prompt in prompts]
    params = [SamplingParams(max_new_tokens=9, stop_token_ids=(free[0][3],), **greedy),          # a stop token on the way
              SamplingParams(max_new_tokens=9, **greedy),                                       # the caller stops it
              SamplingParams(max_new_tokens=9, **greedy),                                       # cancelled on the way
              SamplingParams(max_new_tokens=4, **greedy),                                       # its length
              SamplingParams(max_new_tokens=7, temperature=0.9, top_k=10, top_p=0.8, repetition_penalty=1.2,
                             presence_penalty=0.3, seed=11),                                    # penalties
              SamplingParams(max_new_tokens=8, temperature=0.8, top_k=0, top_p=1.0, repetition_penalty=1.0, seed=5)]
    outcomes = {}
    for ahead in (False, True):
        sampler = Sampler(engine.vocab_size, "cpu", check_device=False)
        emitted = []

        def on_token(request, token):
            emitted.append((request.request_id, token))
            if request.request_id == 2 and len(request.generated) == 2:
                request.cancel()
            return not (request.request_id == 1 and len(request.generated) == 5)

        scheduler = Scheduler(engine, sampler, EngineConfig(max_active_sequences=5, scheduler_token_budget=12,
                                                            prefill_token_quantum=7), on_token=on_token)
        assert scheduler.ahead
        scheduler.ahead = ahead
        for index, prompt in enumerate(prompts):
            scheduler.submit(index, prompt, params[index])
        finished = scheduler.run()
        outcomes[ahead] = ({index: (request.generated, request.finish_reason) for index, request in finished.items()},
                           sorted(emitted), scheduler.rounds)
        stats = engine.cache.stats()
        assert stats["live_requests"] == 0 and stats["free_slots"] == 5
        assert all(group["free_pages"] == group["total_pages"] for group in stats["groups"])
        engine.cache.check()
    assert outcomes[True][0] == outcomes[False][0] and outcomes[True][1] == outcomes[False][1]
    results = outcomes[True][0]
    assert results[0] == (free[0][:3], "stop") and results[1] == (free[1][:5], "stop")
    assert results[2] == (free[2][:2], "cancelled") and results[3] == (free[3][:4], "length")
    assert results[4][1] == results[5][1] == "length" and len(results[4][0]) == 7 and len(results[5][0]) == 8
