"""In-process GPU tests: each part alone against the plain implementation, greedy and seeded
generation through the entry points, and the framework's generality: a toy mixer with state
of its own, another position encoding, a window, a layer that runs twice and a layer that
reads another layer's cache, all registered from here without a change to the package."""
import math
import subprocess
import sys
import numpy as np
import pytest
import torch

import plain_impl
import tiny_configs
import toy_parts
from traces import ROOT

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def tolerance(dtype, want=None):
    """float32: 1e-4; bfloat16: 3 % of the output's scale (8 bits of mantissa, a few roundings
    in a row).  Both relative to the largest wanted value when that exceeds one."""
    scale = 1.0 if want is None else max(1.0, want.abs().max().item())
    return (1e-4 if dtype == torch.float32 else 3e-2) * scale


def rand(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def tokens_for(vocab, count, seed):
    return torch.randint(0, vocab, (count,), generator=torch.Generator().manual_seed(seed)).tolist()


# ------------------------------------------------------------------ a harness for single parts
class PartHarness:
    """Builds one mixer with a cache of its own and feeds it lanes of normed inputs."""

    def __init__(self, spec, tensors, hidden, dtype, page_size=8, capacity=512, requests=4):
        from macllm_infer_amd.cache import CacheManager
        from macllm_infer_amd.kernels import build
        from macllm_infer_amd.parts import BuildContext, part_class
        cls = part_class(spec)
        build.ensure_modules(cls.kernel_modules)
        self.build = BuildContext(hidden_size=hidden, dtype=dtype, device=torch.device(DEV), max_context=4096)
        self.part = cls(spec, "p", {f"p.{name}": value for name, value in tensors.items()}, self.build)
        self.cache = CacheManager({(0, "p"): cls.cache_needs(spec)}, {}, page_size, capacity, requests, dtype, DEV)

    def run(self, lanes):
        """lanes: [(request, x [t, hidden])] -> outputs per lane."""
        from macllm_infer_amd.engine import Lane, build_step_context
        for request, x in lanes:
            if request not in self.cache.requests:
                self.cache.add_request(request)
        self.cache.reserve([(request, x.shape[0]) for request, x in lanes])
        step = build_step_context([Lane(request, [0] * x.shape[0]) for request, x in lanes], self.cache, DEV,
                                  query_tile=getattr(self.part, "query_tile", 0))
        x = torch.cat([x for _, x in lanes]).to(self.build.dtype).to(DEV)
        out = self.part.forward(x, step, self.cache.entry((0, "p"))).float().cpu()
        pieces, cursor = [], 0
        for request, lane_x in lanes:
            self.cache.commit(request, lane_x.shape[0])
            pieces.append(out[cursor:cursor + lane_x.shape[0]])
            cursor += lane_x.shape[0]
        return pieces


def rounded(tensors, dtype):
    """What the part sees: matrices in ``dtype``; the plain model gets the same values."""
    return {name: value.to(dtype) if value.dim() >= 2 else value for name, value in tensors.items()}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window, use_rope", [(None, True), (11, True), (None, False)])
def test_attention_part_alone(dtype, window, use_rope):
    """Hq*dh != hidden, 3 query heads per kv head, biases, all three multipliers; fed whole,
    in portions and token by token, beside another request."""
    from macllm_infer_amd.config import AttentionSpec, NoPositionSpec, RopeSpec
    hidden, Hq, Hkv, dh = 40, 6, 2, 16
    spec = AttentionSpec(num_heads=Hq, num_kv_heads=Hkv, head_dim=dh, scale=1 / math.sqrt(dh),
                         position=RopeSpec(theta=1e4, rotary_dim=dh) if use_rope else NoPositionSpec(),
                         window=window, qkv_bias=True, out_bias=True, in_multiplier=1.3, key_multiplier=0.7,
                         out_multiplier=0.8)
    tensors = {"q_proj.weight": rand(Hq * dh, hidden, seed=1, scale=0.3), "k_proj.weight": rand(Hkv * dh, hidden, seed=2, scale=0.3),
               "v_proj.weight": rand(Hkv * dh, hidden, seed=3, scale=0.3), "o_proj.weight": rand(hidden, Hq * dh, seed=4, scale=0.2),
               "q_proj.bias": rand(Hq * dh, seed=5, scale=0.1), "k_proj.bias": rand(Hkv * dh, seed=6, scale=0.1),
               "v_proj.bias": rand(Hkv * dh, seed=7, scale=0.1), "o_proj.bias": rand(hidden, seed=8, scale=0.1)}
    tensors = rounded(tensors, dtype)
    x = rand(50, hidden, seed=9).to(dtype).float()
    other = rand(23, hidden, seed=10).to(dtype).float()
    plain = lambda rows: plain_impl.attention_mixer(
        rows, tensors, num_heads=Hq, num_kv_heads=Hkv, head_dim=dh, theta=1e4, in_multiplier=1.3,
        key_multiplier=0.7, out_multiplier=0.8, window=window, use_rope=use_rope)
    want, want_other = plain(x), plain(other)
    harness = PartHarness(spec, tensors, hidden, dtype)
    assert (harness.run([("whole", x)])[0] - want).abs().max() < tolerance(dtype, want)
    got, got_other = [], []
    got.append(harness.run([("cut", x[:19])])[0])
    a, b = harness.run([("cut", x[19:21]), ("other", other[:20])])
    got.append(a), got_other.append(b)
    for position in range(21, 24):
        a, b = harness.run([("other", other[position - 1:position]), ("cut", x[position:position + 1])])
        got.append(b), got_other.append(a)
    got.append(harness.run([("cut", x[24:])])[0])
    assert (torch.cat(got) - want).abs().max() < tolerance(dtype, want)
    assert (torch.cat(got_other) - want_other[:23]).abs().max() < tolerance(dtype, want_other)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("gated_norm, bias, K", [(False, False, 4), (True, True, 3), (True, False, 2)])
def test_mamba2_part_alone(dtype, gated_norm, bias, K):
    from macllm_infer_amd.config import Mamba2Spec
    hidden, H, P, N, G = 40, 6, 8, 24, 2
    multipliers = (0.8, 1.4, 0.6, 1.5, 1.1)
    spec = Mamba2Spec(num_heads=H, head_dim=P, state_size=N, num_groups=G, conv_kernel=K, chunk_size=8,
                      norm_eps=2e-5, conv_bias=bias, proj_bias=bias, gated_norm=gated_norm, in_multiplier=1.2,
                      out_multiplier=0.9, multipliers=multipliers)
    E, C = H * P, H * P + 2 * G * N
    tensors = {"in_proj.weight": rand(E + C + H, hidden, seed=1, scale=0.25), "conv1d.weight": rand(C, K, seed=2, scale=0.5),
               "dt_bias": rand(H, seed=3) - 2.0, "A_log": torch.log(torch.rand(H, generator=torch.Generator().manual_seed(4)) * 3 + 0.2),
               "D": rand(H, seed=5), "out_proj.weight": rand(hidden, E, seed=6, scale=0.2)}
    if bias:
        tensors.update({"conv1d.bias": rand(C, seed=7, scale=0.1), "in_proj.bias": rand(E + C + H, seed=8, scale=0.1),
                        "out_proj.bias": rand(hidden, seed=9, scale=0.1)})
    if gated_norm:
        tensors["norm.weight"] = (rand(G, E // G, seed=10, scale=0.1) + 1.0)
    tensors = rounded(tensors, dtype)
    x = rand(60, hidden, seed=11).to(dtype).float()
    other = rand(9, hidden, seed=12).to(dtype).float()
    plain = lambda rows: plain_impl.mamba2_mixer(
        rows, tensors, num_heads=H, head_dim=P, state_size=N, num_groups=G, conv_kernel=K, eps=2e-5,
        in_multiplier=1.2, out_multiplier=0.9, multipliers=multipliers)
    want, want_other = plain(x), plain(other)
    harness = PartHarness(spec, tensors, hidden, dtype)
    assert (harness.run([("whole", x)])[0] - want).abs().max() < tolerance(dtype, want)
    got = [harness.run([("cut", x[:1])])[0]]                    # one token: shorter than the conv tail
    a, b = harness.run([("other", other), ("cut", x[1:3])])
    got.append(b)
    assert (a - want_other).abs().max() < tolerance(dtype, want_other)
    got.append(harness.run([("cut", x[3:40])])[0])
    for position in range(40, 60):
        got.append(harness.run([("cut", x[position:position + 1])])[0])
    assert (torch.cat(got) - want).abs().max() < tolerance(dtype, want)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_feed_forward_and_norm_parts_alone(dtype):
    from macllm_infer_amd.config import RmsNormSpec, SwiGLUSpec
    from macllm_infer_amd.kernels import build
    from macllm_infer_amd.parts import BuildContext, Residual, RmsNorm, SwiGLU
    build.ensure_modules(("common", "gemm"))
    hidden, inner = 72, 100
    context = BuildContext(hidden_size=hidden, dtype=dtype, device=torch.device(DEV), max_context=64)
    tensors = rounded({"f.gate_proj.weight": rand(inner, hidden, seed=1, scale=0.2), "f.up_proj.weight": rand(inner, hidden, seed=2, scale=0.2),
                       "f.down_proj.weight": rand(hidden, inner, seed=3, scale=0.2), "f.gate_proj.bias": rand(inner, seed=4, scale=0.1),
                       "f.up_proj.bias": rand(inner, seed=5, scale=0.1), "f.down_proj.bias": rand(hidden, seed=6, scale=0.1)}, dtype)
    ffn = SwiGLU(SwiGLUSpec(intermediate_size=inner, bias=True, gate_multiplier=1.25, down_multiplier=0.75), "f", tensors, context)
    x = rand(13, hidden, seed=7).to(dtype)
    want = plain_impl.swiglu_mlp(x.float(), {name[2:]: value for name, value in tensors.items()}, 1.25, 0.75)
    assert (ffn.forward(x.to(DEV)).float().cpu() - want).abs().max() < tolerance(dtype, want)
    weight = rand(hidden, seed=8, scale=0.1) + 1.0
    norm = RmsNorm(RmsNormSpec(eps=3e-6), "n", {"n.weight": weight}, context)
    h, delta = rand(13, hidden, seed=9), rand(13, hidden, seed=10).to(dtype)
    residual = Residual(h.clone().to(DEV))
    residual.pending = [delta.to(DEV)]
    got = norm.forward(residual)
    assert (residual.h.cpu() - (h + delta.float())).abs().max() < 1e-6 and residual.pending == []
    assert (got.float().cpu() - plain_impl.rms_norm(h + delta.float(), weight, 3e-6)).abs().max() < tolerance(dtype)


# ------------------------------------------------------------------ generation through the entry points
@pytest.mark.parametrize("name, dtype", [("A", "float32"), ("B", "float32"), ("B", "bfloat16"), ("C", "bfloat16")])
def test_greedy_generation_through_the_entry_point(tmp_path, name, dtype):
    """The workload of the tiny configurations: prompts of 5/17/33 tokens, 12 greedy steps."""
    from macllm_infer_amd import LLM, EngineConfig, SamplingParams, generate
    folder = tiny_configs.make_model_dir(name, tmp_path, torch.float32 if dtype == "float32" else torch.bfloat16)
    cfg, tensors = plain_impl.load_model_dir(folder)
    prompts = [tokens_for(cfg["vocab_size"], length, 60 + length) for length in (5, 17, 33)]
    llm = LLM(folder, dtype=dtype, kv_cache_block_tokens=16 if name == "A" else 8, kv_cache_capacity_tokens=256,
              engine_config=EngineConfig(max_active_sequences=3, scheduler_token_budget=24, prefill_token_quantum=11))
    params = SamplingParams(max_new_tokens=12, temperature=0.0, top_k=0, top_p=1.0, repetition_penalty=1.0)
    results = llm.generate(prompts, params)
    assert [result.finish_reason for result in results] == ["length"] * 3
    assert generate(llm, prompts, params) == [result.token_ids for result in results]        # and the same again
    for prompt, result in zip(prompts, results):
        tokens = result.token_ids
        assert len(tokens) == 12
        if dtype == "float32":
            assert tokens == plain_impl.greedy_generate(cfg, tensors, prompt, 12)
        else:
            # bfloat16 may part ways with the plain model where two logits are close, and goes its own way from
            # there; every token it chose must be the plain model's best for the sequence so far, or within the
            # 16-bit gate (6 % of the logits' scale) of it
            logits = plain_impl.falcon_h1_logits(cfg, tensors, prompt + tokens)
            for index, token in enumerate(tokens):
                row = logits[len(prompt) - 1 + index]
                assert row[token] >= row.max() - 0.06 * row.abs().max(), (index, token)
    assert llm.engine.cache.stats()["live_requests"] == 0


def test_sampled_generation_a_round_ahead_equals_generation_that_waits(tmp_path):
    """float32 on the GPU, where a token does not depend on what shares its step: twenty requests with seeded
    sampling (penalties for most), stop tokens that are hit, callers' stops and a tight budget, once with every
    round queued ahead of the tokens of the round before and once with every token read first.  The same tokens
    and finish reasons, token for token what the plain sampler draws from the plain model for three of them."""
    from macllm_infer_amd import Engine, EngineConfig, SamplingParams
    from macllm_infer_amd.engine.scheduler import Scheduler
    from macllm_infer_amd.sampling import Sampler
    folder = tiny_configs.make_model_dir("B", tmp_path, torch.float32)
    cfg, tensors = plain_impl.load_model_dir(folder)
    generator = torch.Generator().manual_seed(7)
    prompts = [tokens_for(cfg["vocab_size"], int(torch.randint(1, 40, (1,), generator=generator)), 300 + index)
               for index in range(20)]
    params = [SamplingParams(max_new_tokens=4 + index % 9, temperature=0.0 if index % 5 == 0 else 0.7 + 0.05 * (index % 4),
                             top_k=0 if index % 3 == 0 else 12, top_p=1.0 if index % 2 else 0.85,
                             repetition_penalty=1.0 if index % 4 == 0 else 1.15, presence_penalty=0.2 * (index % 3),
                             frequency_penalty=0.1 * (index % 2), seed=50 + index,
                             stop_token_ids=tuple(range(0, cfg["vocab_size"], 9)) if index % 6 == 1 else ())
              for index in range(20)]
    outcomes = []
    for ahead in (True, False):
        engine = Engine(folder, dtype="float32", kv_cache_block_tokens=8, kv_cache_capacity_tokens=512,
                        max_active_sequences=6)
        scheduler = Scheduler(engine, Sampler(engine.vocab_size, engine.device),
                              EngineConfig(max_active_sequences=6, scheduler_token_budget=20, prefill_token_quantum=9),
                              on_token=lambda request, token: not (request.request_id % 7 == 3 and len(request.generated) == 3))
        assert scheduler.ahead
        scheduler.ahead = ahead
        for index, prompt in enumerate(prompts):
            scheduler.submit(index, prompt, params[index])
        finished = scheduler.run()
        outcomes.append({index: (request.generated, request.finish_reason) for index, request in finished.items()})
        assert engine.cache.stats()["live_requests"] == 0
        engine.cache.check()
    assert outcomes[0] == outcomes[1]
    assert {reason for _, reason in outcomes[0].values()} == {"length", "stop"}
    for index in (2, 5, 11):
        p, tokens, generated = params[index], list(prompts[index]), []
        for draw in range(len(outcomes[0][index][0])):
            logits = plain_impl.falcon_h1_logits(cfg, tensors, tokens)[-1]
            token = plain_impl.sample_token(
                logits, temperature=p.temperature, top_k=p.top_k, top_p=p.top_p, repetition_penalty=p.repetition_penalty,
                presence_penalty=p.presence_penalty, frequency_penalty=p.frequency_penalty, history=tokens,
                generated=generated, seed=p.seed, draw_index=draw)
            tokens.append(token)
            generated.append(token)
        assert generated == outcomes[0][index][0], index


def test_generation_under_a_constraint_on_the_tokens(tmp_path):
    """Requests with a fixed list of allowed tokens, with a list that follows what was generated (the next token
    must be one of three that depend on the last: the scheduler reads the round on its way before it draws),
    without any, and one whose constraint comes to allow nothing (it fails alone).  A round ahead and waiting give
    the same tokens; every token is an allowed one, and the greedy ones are the plain model's best allowed token."""
    from macllm_infer_amd import Engine, EngineConfig, SamplingParams
    from macllm_infer_amd.engine.scheduler import Scheduler
    from macllm_infer_amd.sampling import Sampler
    folder = tiny_configs.make_model_dir("B", tmp_path, torch.float32)
    cfg, tensors = plain_impl.load_model_dir(folder)
    V = cfg["vocab_size"]
    follows = lambda generated: [(generated[-1] * 7 + 3 + k) % V for k in range(3)] if generated else [11, 12, 13]
    dead_end = lambda generated: [5, 6] if len(generated) < 2 else []
    fixed = tuple(range(40, 60))
    params = [SamplingParams(max_new_tokens=9, temperature=0.0, top_k=0, top_p=1.0, repetition_penalty=1.0, allowed_token_ids=fixed),
              SamplingParams(max_new_tokens=8, temperature=0.0, top_k=0, top_p=1.0, repetition_penalty=1.2, allowed_token_ids=follows),
              SamplingParams(max_new_tokens=7, temperature=0.9, top_k=5, top_p=0.9, seed=3, allowed_token_ids=follows),
              SamplingParams(max_new_tokens=6, temperature=0.8, top_k=0, top_p=1.0, seed=4, allowed_token_ids=(7, 300, 9)),
              SamplingParams(max_new_tokens=6, temperature=0.0, top_k=0, top_p=1.0, repetition_penalty=1.0),
              SamplingParams(max_new_tokens=6, temperature=0.0, top_k=0, top_p=1.0, repetition_penalty=1.0, allowed_token_ids=dead_end)]
    prompts = [tokens_for(V, 5 + 3 * index, 600 + index) for index in range(len(params))]
    outcomes = []
    for ahead in (True, False):
        engine = Engine(folder, dtype="float32", kv_cache_block_tokens=8, kv_cache_capacity_tokens=512, max_active_sequences=6)
        scheduler = Scheduler(engine, Sampler(engine.vocab_size, engine.device),
                              EngineConfig(max_active_sequences=6, scheduler_token_budget=24, prefill_token_quantum=7))
        scheduler.ahead = ahead
        for index, prompt in enumerate(prompts):
            scheduler.submit(index, prompt, params[index])
        finished = scheduler.run()
        outcomes.append({index: (request.generated, request.finish_reason) for index, request in finished.items()})
        assert engine.cache.stats()["live_requests"] == 0
        engine.cache.check()
    assert outcomes[0] == outcomes[1]
    got = outcomes[0]
    assert [got[index][1] for index in range(5)] == ["length"] * 5
    assert got[5][1].startswith("failed") and "rejected every token" in got[5][1] and len(got[5][0]) == 2
    assert set(got[5][0]) <= {5, 6} and set(got[0][0]) <= set(fixed) and set(got[3][0]) <= {7, 300, 9}
    for index in (1, 2):
        generated = got[index][0]
        assert all(token in follows(generated[:place]) for place, token in enumerate(generated))
    assert not set(got[4][0]) <= set(fixed)
    for index in (0, 1):                                           # greedy: the plain model's best allowed token
        p, tokens, generated = params[index], list(prompts[index]), []
        for _ in got[index][0]:
            logits = plain_impl.falcon_h1_logits(cfg, tensors, tokens)[-1]
            allowed = list(p.allowed_after(generated))
            token = plain_impl.sample_token(
                logits, temperature=0.0, top_k=0, top_p=1.0, repetition_penalty=p.repetition_penalty, presence_penalty=0.0,
                frequency_penalty=0.0, history=tokens, generated=generated, seed=p.seed, draw_index=0, allowed=allowed)
            tokens.append(token)
            generated.append(token)
        assert generated == got[index][0], index


def test_generation_with_more_live_requests_than_the_skinny_kernels_take_rows(tmp_path):
    """Seventy-two requests live at once through the scheduler (bfloat16, configuration D): prompts of 3 to 40
    tokens in portions of 24 beside the decoded tokens of the others (so steps run as two batches), then rounds of
    up to 72 single tokens (two halves at once, each a graph of its own on a stream of its own).  Every request runs to its length, no
    page or slot is left held, and for five of the requests every token is the plain model's choice or as good
    as it (the plain model's logit of the token within a few per cent of its best: bfloat16 may swap near ties)."""
    from macllm_infer_amd import LLM, EngineConfig, SamplingParams
    folder = tiny_configs.make_model_dir("D", tmp_path, torch.bfloat16)
    cfg, tensors = plain_impl.load_model_dir(folder)
    count = 72
    prompts = [tokens_for(cfg["vocab_size"], 3 + (7 * index) % 38, 500 + index) for index in range(count)]
    llm = LLM(folder, dtype="bfloat16", kv_cache_block_tokens=16, kv_cache_capacity_tokens=64 * count,
              engine_config=EngineConfig(max_active_sequences=count, scheduler_token_budget=24 + count,
                                         prefill_token_quantum=24))
    llm.engine.split_from_lanes = 4             # two batches from four single tokens on, whatever the clock would say
    llm.engine.in_halves = True                 # and more than 64 single tokens as two halves at once
    runs, halves = [], []
    real, real_halves = llm.engine._run, llm.engine._run_in_halves
    llm.engine._run = lambda lanes, lowered, graphs=None: (runs.append((len(lanes), int(lowered.lengths.max()))),
                                                           real(lanes, lowered, graphs))[1]
    llm.engine._run_in_halves = lambda lanes: (halves.append(len(lanes)), real_halves(lanes))[1]
    params = SamplingParams(max_new_tokens=7, temperature=0.0, top_k=0, top_p=1.0, repetition_penalty=1.0, ignore_eos=True)
    results = llm.generate(prompts, params)
    assert [result.finish_reason for result in results] == ["length"] * count
    assert all(len(result.token_ids) == 7 for result in results)
    assert halves and max(halves) > 64 and llm.engine.graphs_beside.counts["decode_replays"] == len(halves)   # rounds of more than 64 single tokens: two halves at once
    assert any(longest > 1 for _, longest in runs) and any(lanes >= 4 and longest == 1 for lanes, longest in runs)
    assert llm.engine.cache.stats()["live_requests"] == 0
    llm.engine.cache.check()
    for index in (0, 17, 40, 63, 71):
        tokens = list(prompts[index])
        for token in results[index].token_ids:
            logits = plain_impl.falcon_h1_logits(cfg, tensors, tokens)[-1]
            assert logits[token].item() >= logits.max().item() - 0.06 * logits.abs().max().item(), (index, len(tokens))
            tokens.append(token)


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_a_step_of_many_single_tokens_runs_as_two_halves_at_once(tmp_path, dtype):
    """More single decoded tokens than the skinny kernels take rows (81 and 100 of them, uneven halves): the step
    runs as two halves at once, each half a captured graph of its own on a stream of its own, the second half fed
    from the device like the first.  Six steps in a row with nothing waiting in between; every row against the
    plain model, in float32 the same bits as the same step through one graph, and nothing held afterwards."""
    import gates
    from macllm_infer_amd import Engine, Lane
    folder = tiny_configs.make_model_dir("D", tmp_path, torch.bfloat16 if dtype == "bfloat16" else torch.float32)
    cfg, tensors = plain_impl.load_model_dir(folder)
    requests = 100
    prompts = {index: tokens_for(cfg["vocab_size"], 4 + index % 9 + 6, 800 + index) for index in range(requests)}
    outcomes = {}
    for in_halves in (True, False):
        engine = Engine(folder, dtype=dtype, kv_cache_block_tokens=16, kv_cache_capacity_tokens=64 * (requests + 1),
                        max_active_sequences=requests + 1)
        engine.in_halves = in_halves
        if in_halves:
            assert len(engine.warm_up([(100, 100), (81, 81)])) == 2          # 50 + 50 and 41 + 40: a graph of 64 lanes in each bank
        for index in prompts:
            engine.add_request(index)
        for first in range(0, requests, 25):
            engine.step([Lane(index, prompts[index][:-6], []) for index in range(first, first + 25)])
        rows = {index: [] for index in prompts}
        for turn in range(6):
            live = range(requests) if turn % 2 == 0 else range(19, requests)                 # 100, then 81
            logits = engine.step([Lane(index, [prompts[index][len(prompts[index]) - 6 + len(rows[index])]], [0])
                                  for index in live])
            for row, index in enumerate(live):
                rows[index].append(logits[row])
        torch.cuda.synchronize()
        if in_halves:
            assert engine.graphs_beside is not None and engine.graphs_beside.counts["decode_replays"] == 6
            assert engine.graphs.counts["decode_replays"] == 6
        else:
            assert engine.graphs_beside is None
        outcomes[in_halves] = {index: torch.stack(values).float().cpu() for index, values in rows.items()}
        for index in prompts:
            engine.finish(index)
        engine.cache.check()
        assert engine.cache.stats()["live_requests"] == 0
    for index in (0, 18, 19, 49, 50, 59, 60, 99):
        tokens = prompts[index]
        want = plain_impl.falcon_h1_logits(cfg, tensors, tokens)[-6:]
        have = outcomes[True][index]
        assert have.shape[0] == (6 if index >= 19 else 3)
        for place in range(have.shape[0]):
            if dtype == "float32":
                assert gates.float32_close(have[place].numpy(), want[place].numpy()), (index, place)
            else:
                assert gates.bfloat16_close(have[place].numpy(), want[place].numpy()), (index, place)
    if dtype == "float32":
        assert all(torch.equal(outcomes[True][index], outcomes[False][index]) for index in prompts)


def test_the_clock_says_whether_many_single_tokens_run_as_two_halves(tmp_path):
    """Nothing is measured until a step of 65 single tokens or more comes; then one graph of 128 padding lanes is
    timed against two of 64 at once, once, and the halves are taken if they win by the margin.  Without a clock
    such a step stays one graph."""
    from macllm_infer_amd import Engine, Lane
    from macllm_infer_amd.engine import engine as engine_module
    folder = tiny_configs.make_model_dir("D", tmp_path, torch.bfloat16)
    cfg, _ = plain_impl.load_model_dir(folder)
    fixed = Engine(folder, dtype="bfloat16", kv_cache_capacity_tokens=70 * 32, max_active_sequences=70, measured_paths=False)
    assert fixed.in_halves is False and fixed.halves_share is None
    engine = Engine(folder, dtype="bfloat16", kv_cache_capacity_tokens=70 * 32, max_active_sequences=70)
    for index in range(70):
        engine.add_request(index)
    for first in range(0, 70, 35):
        engine.step([Lane(index, tokens_for(cfg["vocab_size"], 5, index), []) for index in range(first, first + 35)])
    engine.step([Lane(index, [3], [0]) for index in range(64)])
    assert engine._in_halves is None                                   # 64 single tokens: no question
    got = engine.step([Lane(index, [4], [0]) for index in range(70)])
    assert got.shape[0] == 70
    print("two halves over one graph:", engine.halves_share, "in halves:", engine.in_halves)
    assert engine.halves_share is not None and engine.halves_share > 0
    assert engine.in_halves == (engine.halves_share < engine_module.HALVES_MARGIN)
    assert (engine.graphs_beside is not None) == engine.in_halves
    engine.cache.check()


def test_generation_when_pages_run_out(tmp_path):
    """Seven requests on a cache of six pages, three live at a time: lanes are dropped from steps
    and retried, pages and slots are used again, and a request that cannot grow while the others
    hold their pages fails alone.  Whatever finishes says what the plain model says; whatever
    fails said so up to there; nothing stays behind."""
    from macllm_infer_amd import LLM, EngineConfig, SamplingParams
    folder = tiny_configs.make_model_dir("A", tmp_path)
    cfg, tensors = plain_impl.load_model_dir(folder)
    prompts = [tokens_for(cfg["vocab_size"], length, 90 + length) for length in (20, 37, 9, 30, 41, 16, 200)]
    llm = LLM(folder, dtype="float32", kv_cache_block_tokens=16, kv_cache_capacity_tokens=96,
              engine_config=EngineConfig(max_active_sequences=3, scheduler_token_budget=40, prefill_token_quantum=13))
    params = SamplingParams(max_new_tokens=10, temperature=0.0, top_k=0, top_p=1.0, repetition_penalty=1.0)
    results = llm.generate(prompts, params)
    reasons = [result.finish_reason for result in results]
    assert reasons[-1].startswith("rejected") and "cache capacity" in reasons[-1]      # could never fit
    assert reasons.count("length") >= 3 and set(reasons[:-1]) <= {"length", "resource_exhausted"}
    for prompt, result in zip(prompts[:-1], results[:-1]):
        want = plain_impl.greedy_generate(cfg, tensors, prompt, 10)
        assert result.token_ids == want[:len(result.token_ids)]
        assert len(result.token_ids) == 10 or result.finish_reason == "resource_exhausted"
    stats = llm.engine.cache.stats()
    assert stats["live_requests"] == 0 and stats["free_slots"] == stats["total_slots"]
    assert all(group["free_pages"] == group["total_pages"] for group in stats["groups"])
    llm.engine.cache.check()


def test_seeded_sampling_through_the_entry_point(tmp_path):
    """Config B's workload: five requests of 1/7/24/40/63 tokens, prompts cut into portions of
    11, temperature 0.8 with seeded draws, 20 decode steps, pages of 8."""
    from macllm_infer_amd import LLM, EngineConfig, SamplingParams
    folder = tiny_configs.make_model_dir("B", tmp_path)
    cfg, tensors = plain_impl.load_model_dir(folder)
    prompts = [tokens_for(cfg["vocab_size"], length, 80 + length) for length in (1, 7, 24, 40, 63)]
    llm = LLM(folder, dtype="float32", kv_cache_block_tokens=8, kv_cache_capacity_tokens=512,
              engine_config=EngineConfig(max_active_sequences=5, scheduler_token_budget=64, prefill_token_quantum=11))
    params = SamplingParams(max_new_tokens=20, temperature=0.8, top_k=0, top_p=1.0, repetition_penalty=1.0, seed=5)
    results = llm.generate(prompts, params)
    for index, (prompt, result) in enumerate(zip(prompts, results)):
        tokens = list(prompt)
        for draw in range(20):
            logits = plain_impl.falcon_h1_logits(cfg, tensors, tokens)[-1]
            tokens.append(plain_impl.sample_token(logits, temperature=0.8, seed=5 + index, draw_index=draw))
        assert result.token_ids == tokens[len(prompt):] and result.finish_reason == "length"
        assert result.time_to_first_token is not None and result.total_time > 0


def test_command_line_run(tmp_path):
    folder = tiny_configs.make_model_dir("A", tmp_path)
    cfg, tensors = plain_impl.load_model_dir(folder)
    prompt = tokens_for(cfg["vocab_size"], 9, 70)
    done = subprocess.run([sys.executable, "-m", "macllm_infer_amd", "run", "-m", folder, "--dtype", "f32",
                           "--tokens", ",".join(map(str, prompt)), "--max-new-tokens", "5", "--temperature", "0",
                           "--repetition-penalty", "1.0", "--prefill-token-quantum", "4"],
                          cwd=ROOT, capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stderr
    assert [int(t) for t in done.stdout.split()] == plain_impl.greedy_generate(cfg, tensors, prompt, 5)
    assert "finish=length" in done.stderr and "prefill=" in done.stderr and "model-decode=" in done.stderr
    assert "tok/s" in done.stderr and "TTFT=" in done.stderr


# ------------------------------------------------------------------ generality, shown with toy parts
@pytest.mark.parametrize("schedule", toy_parts.SCHEDULES, ids=toy_parts.SCHEDULE_IDS)
def test_toy_parts_register_build_and_step(schedule):
    """A mixer with state of its own, another position encoding, a windowed layer whose pages
    are given back, a layer that runs twice with two caches and a run that reads another
    run's cache: registered in the tests, built by the engine, stepped whole, in portions
    and mixed, on the GPU with the package's kernels."""
    toy_parts.exercise(schedule, DEV, check_device=True)


@pytest.mark.parametrize("name, dtype", [("A", "float32"), ("B", "float32"), ("B", "bfloat16"), ("C", "bfloat16")])
def test_decode_graphs_match_eager_steps(tmp_path, name, dtype):
    """Decode steps replayed from captured graphs, with eager prompt portions of other requests
    and synchronizations between the replays; every replay is compared with the same step of an
    engine without graphs, for changing batch sizes (buckets 1, 2, 4 with padding lanes)."""
    from macllm_infer_amd import Engine, Lane
    folder = tiny_configs.make_model_dir(name, tmp_path, torch.float32 if dtype == "float32" else torch.bfloat16)
    cfg, _ = plain_impl.load_model_dir(folder)
    make = lambda graphs: Engine(folder, dtype=dtype, kv_cache_block_tokens=8, kv_cache_capacity_tokens=512,
                                 max_active_sequences=4, decode_graphs=graphs)
    with_graphs, eager = make(True), make(False)
    assert with_graphs.graphs is not None and eager.graphs is None
    sequences = {key: tokens_for(cfg["vocab_size"], 90, 30 + index) for index, key in enumerate("abcd")}
    cursor = {key: 0 for key in sequences}

    def both(lanes_spec):
        lanes = [Lane(key, sequences[key][cursor[key]:cursor[key] + count], list(range(count)))
                 for key, count in lanes_spec]
        got, want = with_graphs.step(lanes).float().cpu(), eager.step(lanes).float().cpu()
        for key, count in lanes_spec:
            cursor[key] += count
        scale = max(1.0, want.abs().max().item())
        assert (got - want).abs().max() <= (1e-5 if dtype == "float32" else 3e-2) * scale

    for engine in (with_graphs, eager):
        for key in sequences:
            engine.add_request(key)
    both([("a", 9)])
    for turn in range(40):
        if turn == 3:
            both([("b", 17)])                                   # an eager prompt between replays
        if turn == 10:
            both([("c", 5), ("d", 12)])
        if turn == 20:
            torch.cuda.synchronize()
        live = [key for key in "abcd" if cursor[key] > 0]
        if turn % 7 == 6:
            live = live[:1]                                     # bucket 1
        both([(key, 1) for key in live])
    assert {lanes for lanes, _ in with_graphs.graphs._graphs} == {1, 2, 4}
    assert with_graphs.cache.stats() == eager.cache.stats()


@pytest.mark.parametrize("requests, library", [(24, False), (40, False), (5, True), (24, True), (40, "clock"),
                                               (24, "split"), (40, "split"), (24, "tiles"), (40, "tiles"), (80, False),
                                               (24, "shared"), (40, "shared"), (57, "shared"), (80, "shared"), (128, "shared"),
                                               (5, "shared"), (14, "shared")])
def test_wide_decode_batches_match_the_plain_model(tmp_path, monkeypatch, requests, library):
    """More single-token lanes than the norm-fused kernels take (16): the block's fast path with
    norms of their own, through graphs of buckets 32 and 64, against the plain model.  ``library``:
    the projections go through the BLAS library (with the conv step and SwiGLU as kernels of their
    own), as large weights do where that is measured to be faster; "clock": the measurement itself
    runs on this model's small weights and either outcome must be right; "split": the projections
    that feed the residual stream are split over K into float32 slabs that the next norm adds up; "tiles": a
    workgroup of the skinny kernel owns four tiles of 16 output features, split projections included; "shared":
    the slabs come from the kernel whose waves own feature tiles and share the step's rows through LDS (the only
    one of them that also takes 80 and 128 rows, the output projection of which then comes from it).  80
    requests: more rows than the skinny kernels take; every product through the library, around the mixers'
    decode kernel (not the prompt kernels, which would take them as 80 prompts of one token)."""
    from macllm_infer_amd import Engine, Lane
    from macllm_infer_amd.parts import fused
    if library == "clock":
        monkeypatch.setattr(fused, "LIBRARY_MIN_WEIGHT", 0)
    elif library == "split":
        monkeypatch.setattr(fused, "FORCE_SPLIT", 3)
    elif library == "shared":
        monkeypatch.setattr(fused, "FORCE_SPLIT", 2 if requests == 40 else 3)
        monkeypatch.setattr(fused, "FORCE_SHARED_ROWS", 2 if requests == 24 else 1)
    elif library == "tiles":
        monkeypatch.setattr(fused, "FORCE_TILES", 4)
        monkeypatch.setattr(fused, "FORCE_SPLIT", 2 if requests == 40 else 0)
    elif library:
        monkeypatch.setattr(fused, "FORCE_LIBRARY", True)
    # (the library takes rows whose width is a multiple of 8 elements: configuration D's; C's are not)
    # (and every step size of D runs its norms as kernels, so that the forced ways apply to steps of 5 and 14 rows too)
    wide = library is True or requests > 64 or (library == "shared" and requests < 16)
    folder = tiny_configs.make_model_dir("D" if wide else "C", tmp_path, torch.bfloat16)
    cfg, tensors = plain_impl.load_model_dir(folder)
    engine = Engine(folder, dtype="bfloat16", kv_cache_block_tokens=16, kv_cache_capacity_tokens=64 * (requests + 1),
                    max_active_sequences=requests + 1)
    engine.in_halves = False                     # 80 and 128 single tokens as one graph (not as two halves at once)
    if library is True:
        fusion = engine.model.blocks[0].fusion
        assert fusion.general and all(fusion.library_in) and all(fusion.library_out) and all(fusion.library_down)
    if library == "split":
        fusion = engine.model.blocks[0].fusion
        assert fusion.split_out[:6] == (0, 0, 0, 3, 3, 3) and fusion.split_down[:6] == (0, 0, 0, 3, 3, 3)
    if library == "shared" and wide:
        fusion = engine.model.blocks[0].fusion
        assert fusion.split_out[fused.BEYOND] == 3 and fusion.tiles_out[fused.BEYOND] == -1 and fusion.f_out is not None
        assert fusion.split_down[fused.BEYOND] == 0               # a K of 64
        assert fusion.split_out[:6] == (3,) * 6 and fusion.tiles_out[:6] == fusion.tiles_gate_up[:6] == (-1,) * 6
    elif library == "shared":
        fusion = engine.model.blocks[0].fusion
        slabs, tiles = (2 if requests == 40 else 3), (-2 if requests == 24 else -1)
        assert fusion.split_out[:6] == fusion.split_down[:6] == (0, 0, 0, slabs, slabs, slabs)
        assert fusion.tiles_out[:6] == (1, 1, 1, tiles, tiles, tiles)
        assert fusion.tiles_down[:6] == (1,) * 6                  # a K of 96 is below that kernel's stage of 128 columns
        assert fusion.tiles_gate_up[:6] == (1, 1, 1, tiles, tiles, tiles) and fusion.library_gate_up[:6] == (False,) * 6
        assert fusion.tiles_in[:6] == (1, 1, 1, tiles, tiles, tiles) and fusion.library_in[:6] == (False,) * 6
    if library == "tiles":
        fusion = engine.model.blocks[0].fusion
        assert fusion.tiles_in[:6] == fusion.tiles_gate_up[:6] == fusion.tiles_out[:6] == fusion.tiles_down[:6] == (1, 1, 1, 4, 4, 4)
        assert fusion.library_in[:6] == fusion.library_down[:6] == (False,) * 6
    prompts = {index: tokens_for(cfg["vocab_size"], 3 + index % 7 + 6, 500 + index) for index in range(requests)}
    for index, tokens in prompts.items():
        engine.add_request(index)
    engine.step([Lane(index, tokens[:-6], []) for index, tokens in prompts.items()])
    got = {index: [] for index in prompts}
    for turn in range(6):
        logits = engine.step([Lane(index, [tokens[len(tokens) - 6 + turn]], [0]) for index, tokens in prompts.items()])
        for row, index in enumerate(prompts):
            got[index].append(logits[row].float().cpu())
    assert {lanes for lanes, _ in engine.graphs._graphs} == {8 if requests <= 8 else 16 if requests <= 16 else 32 if requests <= 32 else 64 if requests <= 64 else 128}
    if requests > 64:
        fusion = engine.model.blocks[0].fusion
        assert fusion.general and fusion.library_in[fused.BEYOND] and fusion.library_down[fused.BEYOND]
    for index, tokens in prompts.items():
        want = plain_impl.falcon_h1_logits(cfg, tensors, tokens)[-6:]
        have = torch.stack(got[index])
        scale = want.abs().max().item()
        assert (have - want).abs().max().item() <= 6e-2 * scale
        assert ((have - want).pow(2).mean().sqrt() / want.pow(2).mean().sqrt()).item() <= 3e-2
    if library == "shared":
        # a prompt of 41 tokens as one step goes the same way with the mixers' own kernels between the products:
        # the input projection then leaves plain rows (no conv step in its epilogue)
        tokens = tokens_for(cfg["vocab_size"], 41, 77)
        engine.add_request("portion")
        have = engine.step([Lane("portion", tokens, [0, 20, 40])]).float().cpu()
        want = plain_impl.falcon_h1_logits(cfg, tensors, tokens)[[0, 20, 40]]
        scale = want.abs().max().item()
        assert (have - want).abs().max().item() <= 6e-2 * scale
        assert ((have - want).pow(2).mean().sqrt() / want.pow(2).mean().sqrt()).item() <= 3e-2


@pytest.mark.parametrize("graphs", [False, True], ids=["eager", "graphs"])
def test_lanes_fed_from_the_device_say_what_lanes_fed_by_the_host_say(tmp_path, graphs):
    """Two engines decode the same three requests greedily, one with every token read by the host before the
    next step, one with each step queued before the tokens of the step before were read (``Lane.feed`` from
    the sampler's tokens on the device), beside a prompt portion of a fourth request in some steps: the same
    logits bit for bit and the same tokens, and the tokens the plain model prefers."""
    from macllm_infer_amd import Engine, Lane
    from macllm_infer_amd.sampling import GREEDY, Sampler, SamplerRow
    folder = tiny_configs.make_model_dir("C", tmp_path, torch.bfloat16)
    cfg, tensors = plain_impl.load_model_dir(folder)
    prompts = {name: tokens_for(cfg["vocab_size"], length, 60 + length) for name, length in (("a", 9), ("b", 33), ("c", 70))}
    late = tokens_for(cfg["vocab_size"], 40, 99)
    results = {}
    for fed in (False, True):
        engine = Engine(folder, dtype="bfloat16", kv_cache_block_tokens=16, kv_cache_capacity_tokens=1024,
                        max_active_sequences=4, decode_graphs=graphs)
        sampler = Sampler(engine.vocab_size, engine.device)
        rows = [SamplerRow(GREEDY, (), ()) for _ in prompts]
        for name, tokens in prompts.items():
            engine.add_request(name)
        logits = engine.step([Lane(name, tokens, [len(tokens) - 1]) for name, tokens in prompts.items()])
        handle = sampler.sample_async(logits.clone(), rows)
        seen, emitted = [logits.float().cpu()], []
        engine.add_request("late")
        for turn in range(10):
            if fed:
                lanes = [Lane(name, [0], [0], feed=(handle.device, row)) for row, name in enumerate(prompts)]
            else:
                lanes = [Lane(name, [token], [0]) for name, token in zip(prompts, handle.wait())]
            if turn in (2, 3, 5):                                   # a portion of another prompt beside them
                portion = late[(turn - 2) * 10:(turn - 1) * 10] if turn < 5 else late[20:]
                lanes.insert(1, Lane("late", portion, []))
            logits = engine.step(lanes)
            newer = sampler.sample_async(logits.clone(), rows)
            emitted.append(handle.wait())
            handle = newer
            seen.append(logits.float().cpu())
        emitted.append(handle.wait())
        results[fed] = (torch.cat(seen), emitted)
    assert torch.equal(results[True][0], results[False][0]) and results[True][1] == results[False][1]
    for row, (name, tokens) in enumerate(prompts.items()):
        mine = [step[row] for step in results[True][1]]
        want = plain_impl.falcon_h1_logits(cfg, tensors, tokens + mine[:-1])[len(tokens) - 1:]
        for place, token in enumerate(mine):                          # each token is the plain model's choice, or as good
            best = want[place].max().item()
            assert want[place][token].item() >= best - 0.06 * want[place].abs().max().item(), (name, place)


def test_fixed_paths_take_no_measurement(tmp_path, monkeypatch):
    """``measured_paths=False``: even where every weight would be timed (the limit lowered to 0), the layers take
    the fixed rules, the same in every process, and say so; the engine that measures reports a choice for each
    of the six step sizes.  Both decode 24 lanes like the plain model."""
    import gates
    from macllm_infer_amd import Engine, Lane
    from macllm_infer_amd.parts import fused
    monkeypatch.setattr(fused, "LIBRARY_MIN_WEIGHT", 0)
    monkeypatch.setattr(fused, "_chain_wins", {})
    folder = tiny_configs.make_model_dir("C", tmp_path, torch.bfloat16)
    cfg, tensors = plain_impl.load_model_dir(folder)
    prompts = {index: tokens_for(cfg["vocab_size"], 5 + index % 4, 900 + index) for index in range(24)}
    for measured in (False, True):
        engine = Engine(folder, dtype="bfloat16", kv_cache_block_tokens=16, kv_cache_capacity_tokens=64 * 24,
                        max_active_sequences=24, measured_paths=measured)
        choices = engine.path_choices()
        assert set(choices) == {"in", "out", "gate_up", "down", "tiles_in", "tiles_out", "tiles_gate_up", "tiles_down",
                                "padded_in", "norms", "rows", "beyond_out_down"}
        assert all(len(value.split("/")) == {"padded_in": 5, "beyond_out_down": 2}.get(name, 6)
                   for name, value in choices.items())
        assert bool(fused._chain_wins) == measured          # the layers' chain was timed too, once for the shape
        if not measured:
            assert choices["in"] == choices["out"] == choices["gate_up"] == choices["down"] == "S/S/S/S/S/S"
            assert choices["norms"] == "D/D/D/D/D/D"
            assert choices["tiles_in"] == choices["tiles_down"] == "1/1/1/1/1/1" and choices["padded_in"] == "-/-/-/-/-"
            assert choices["beyond_out_down"] == "L/L"
            assert choices["rows"] == "1111/1111/1111/1414/1414/1414"       # few output features: one tile of rows a workgroup
        for index in prompts:
            engine.add_request(index)
        engine.step([Lane(index, tokens[:-1], []) for index, tokens in prompts.items()])
        logits = engine.step([Lane(index, tokens[-1:], [0]) for index, tokens in prompts.items()]).float().cpu()
        for row, tokens in enumerate(prompts.values()):
            want = plain_impl.falcon_h1_logits(cfg, tensors, tokens)[-1]
            assert gates.bfloat16_close(logits[row].numpy(), want.numpy()), (measured, row)


def test_norms_left_to_the_projections_around_them(tmp_path, monkeypatch):
    """A layer whose projections all run through the skinny kernels leaves its norms to them: the output and
    down projections add to the float32 stream themselves and hand on the rows times the next norm's weight with
    their sums of squares, up to the output head.  With that switched off the norms run in prologues or as
    kernels of their own.  Both ways: steps of 1, 5 and 18 single tokens and a step of 20 and 3 prompt tokens
    beside decoded ones (more than 16 rows: several row tiles), each close to the plain model."""
    import gates
    from macllm_infer_amd import Engine, Lane
    from macllm_infer_amd.parts import fused
    folder = tiny_configs.make_model_dir("C", tmp_path, torch.bfloat16)
    cfg, tensors = plain_impl.load_model_dir(folder)
    prompts = {index: tokens_for(cfg["vocab_size"], 6 + index % 5, 400 + index) for index in range(24)}
    late = {"x": tokens_for(cfg["vocab_size"], 21, 450), "y": tokens_for(cfg["vocab_size"], 4, 451)}
    for deferred in (False, None):
        monkeypatch.setattr(fused, "FORCE_DEFERRED_NORM", deferred)
        engine = Engine(folder, dtype="bfloat16", kv_cache_block_tokens=16, kv_cache_capacity_tokens=64 * 26,
                        max_active_sequences=26)
        assert engine.path_choices()["norms"] == ("-/-/-/-/-/-" if deferred is False else "D/D/D/D/D/D")
        for index in list(prompts) + list(late):
            engine.add_request(index)
        engine.step([Lane(index, tokens[:-1], []) for index, tokens in prompts.items()])
        checked = 0
        for group in (range(0, 1), range(1, 6), range(6, 24)):             # steps of 1, 5 and 18 single tokens
            logits = engine.step([Lane(index, prompts[index][-1:], [0]) for index in group]).float().cpu()
            for row, index in enumerate(group):
                want = plain_impl.falcon_h1_logits(cfg, tensors, prompts[index])[-1]
                assert gates.bfloat16_close(logits[row].numpy(), want.numpy()), (deferred, index)
                checked += 1
        lanes = [Lane("x", late["x"][:20], [19]), Lane("y", late["y"][:3], [0, 2])]
        lanes += [Lane(index, [7 + index], [0]) for index in range(3)]
        logits = engine.step(lanes).float().cpu()
        wants = [plain_impl.falcon_h1_logits(cfg, tensors, late["x"][:20])[19],
                 plain_impl.falcon_h1_logits(cfg, tensors, late["y"][:3])[0],
                 plain_impl.falcon_h1_logits(cfg, tensors, late["y"][:3])[2]]
        wants += [plain_impl.falcon_h1_logits(cfg, tensors, prompts[index] + [7 + index])[-1] for index in range(3)]
        for row, want in enumerate(wants):
            assert gates.bfloat16_close(logits[row].numpy(), want.numpy()), (deferred, "mixed", row)
        assert checked == 24
        engine.cache.check()


@pytest.mark.parametrize("row_tiles", [2, 4])
def test_the_rows_of_a_step_dealt_out_to_several_workgroups(tmp_path, monkeypatch, row_tiles):
    """Where the norms are left to the projections, a step of more than 16 rows may have its tiles of 16 rows
    dealt out to two or four workgroups per tile of features, in all four projections of a layer (the conv step of
    each row's own slot included): steps of 40, 33 and 17 single tokens, each close to the plain model."""
    import gates
    from macllm_infer_amd import Engine, Lane
    from macllm_infer_amd.parts import fused
    monkeypatch.setattr(fused, "FORCE_ROW_TILES", row_tiles)
    folder = tiny_configs.make_model_dir("C", tmp_path, torch.bfloat16)
    cfg, tensors = plain_impl.load_model_dir(folder)
    prompts = {index: tokens_for(cfg["vocab_size"], 5 + index % 6, 700 + index) for index in range(40)}
    engine = Engine(folder, dtype="bfloat16", kv_cache_block_tokens=16, kv_cache_capacity_tokens=64 * 40,
                    max_active_sequences=40)
    choices = engine.path_choices()
    assert choices["norms"] == "D/D/D/D/D/D" and choices["rows"] == "/".join([str(row_tiles) * 4] * 6)
    for index in prompts:
        engine.add_request(index)
    for first in range(0, 40, 8):                                           # the prompts, eight at a time
        engine.step([Lane(index, prompts[index], []) for index in range(first, first + 8)])
    history = {index: list(tokens) for index, tokens in prompts.items()}
    for group in (range(40), range(7, 40), range(3, 20)):
        lanes = []
        for index in group:
            history[index].append((index * 7 + len(history[index])) % cfg["vocab_size"])
            lanes.append(Lane(index, history[index][-1:], [0]))
        logits = engine.step(lanes).float().cpu()
        for row, index in enumerate(group):
            want = plain_impl.falcon_h1_logits(cfg, tensors, history[index])[-1]
            assert gates.bfloat16_close(logits[row].numpy(), want.numpy()), (row_tiles, len(group), index)
    engine.cache.check()


def test_the_clock_says_from_how_many_single_tokens_a_mixed_step_runs_as_two_batches(tmp_path):
    """Nothing is measured until a step could need the answer (portions beside four single tokens or more); then the
    engine times a portion alone, beside single tokens and the single tokens alone, once, on padding lanes, and
    splits from the number the three times give.  Without the clock the fewest allowed stands."""
    from macllm_infer_amd import Engine, Lane
    from macllm_infer_amd.engine import engine as engine_module
    folder = tiny_configs.make_model_dir("C", tmp_path, torch.bfloat16)
    cfg, _ = plain_impl.load_model_dir(folder)
    fixed = Engine(folder, dtype="bfloat16", kv_cache_capacity_tokens=1024, max_active_sequences=8, measured_paths=False)
    assert fixed.split_from_lanes == engine_module.SPLIT_FROM_LANES and fixed.lane_share is None
    engine = Engine(folder, dtype="bfloat16", kv_cache_capacity_tokens=1024, max_active_sequences=8)
    for index in range(6):
        engine.add_request(index)
        engine.step([Lane(index, tokens_for(cfg["vocab_size"], 9, index), [])])
    engine.step([Lane(0, [1, 2, 3], []), Lane(1, [4], [0]), Lane(2, [5], [0])])
    assert engine._split_from_lanes is None                       # two single tokens: no question
    got = engine.step([Lane(0, [1, 2, 3], [2])] + [Lane(index, [7], [0]) for index in range(1, 6)])
    assert got.shape[0] == 6
    print("lane share", engine.lane_share, "split from", engine.split_from_lanes)
    assert engine._split_from_lanes is not None and engine.split_from_lanes >= engine_module.SPLIT_FROM_LANES
    assert engine.lane_share is None or engine.lane_share > 0
    if engine.lane_share is not None:
        assert engine.split_from_lanes == max(engine_module.SPLIT_FROM_LANES, int(1.0 / engine.lane_share + 0.5))
    engine.cache.check()


def test_a_mixer_with_a_step_table_of_its_own_runs_under_captured_graphs():
    """A toy mixer, registered from the tests, declares an index table of its own.  The step carries it at a fixed
    address with the size of the step's capacity; the mixer's function rewrites it before every replay, and graphs
    of single tokens and of prompt portions say what the plain model says, whatever the order of the lanes."""
    del toy_parts.TABLE_FILLS[:]
    engine = toy_parts.exercise_step_table(DEV, check_device=True, graphs=True)
    counts = engine.graphs.counts
    assert counts["bucket_captures"] == 1 and counts["bucket_replays"] >= 4 and counts["decode_replays"] >= 30
    assert (4, 16) in toy_parts.TABLE_FILLS                 # the capacity that the portions were padded to
    assert {fill for fill in toy_parts.TABLE_FILLS if fill[0] == fill[1]} >= {(1, 1), (2, 2), (4, 4)}   # decode buckets
    eager = toy_parts.exercise_step_table(DEV, check_device=True, graphs=False)
    assert eager.graphs is None


def test_a_position_encoding_that_declares_its_rotation_gets_the_fused_decode_step():
    """A toy rotation, registered from the tests: the class that says what it rotates by (``fused_rotation``) decodes
    through the one-launch mixer kernel; the class that keeps it to itself is told so with a warning and decodes
    through its own ``rotate_and_store`` and the general kernels.  Both say the same, and not what the package's own
    rotation says."""
    import gates
    from macllm_infer_amd import Engine, Lane
    from macllm_infer_amd.config import FalconH1Config
    from macllm_infer_amd.parts import FastPathDeclined
    from macllm_infer_amd.weights.random_init import random_tensors
    toy_parts.register_toys()
    base = dict(tiny_configs.TINY_C, rope_theta=50.0)
    tensors = random_tensors(FalconH1Config.from_dict(base), 6, torch.bfloat16, "unit")
    prompts = {index: tokens_for(base["vocab_size"], length, 40 + index) for index, length in enumerate([90, 33, 61])}

    def decode(config, expect_kernel):
        engine = Engine(config=config, tensors=tensors, dtype="bfloat16", kv_cache_block_tokens=16,
                        kv_cache_capacity_tokens=1024, max_active_sequences=4, measured_paths=False)
        fusion = engine.model.blocks[0].fusion
        assert (fusion.kernel is not None) == expect_kernel
        for index, tokens in prompts.items():
            engine.add_request(index)
            engine.step([Lane(index, tokens[:-6], [])])
        rows = [engine.step([Lane(index, [tokens[turn - 6]], [0]) for index, tokens in prompts.items()]).float().cpu()
                for turn in range(6)]
        return torch.cat(rows)

    stretched = lambda kind: toy_parts.ToyStretchedConfig({"architectures": ["ToyStretchedForTests"], "base": base,
                                                          "stretch": 3.0, "position_kind": kind})
    import warnings
    with warnings.catch_warnings():
        warnings.simplefilter("error", FastPathDeclined)
        said = decode(stretched("toy_stretched_rope"), True)
        own = decode(FalconH1Config.from_dict(base), True)
    with pytest.warns(FastPathDeclined, match="StretchedRopeUnsaid declares no rotation"):
        unsaid = decode(stretched("toy_stretched_rope_unsaid"), False)
    for row in range(said.shape[0]):
        assert gates.bfloat16_close(said[row].numpy(), unsaid[row].numpy()), row
    assert not all(gates.bfloat16_close(said[row].numpy(), own[row].numpy()) for row in range(said.shape[0]))


def test_the_output_projection_may_merge_the_runs_of_keys(monkeypatch):
    """Steps of up to 16 single tokens: whether the runs of keys of the attended heads are merged by a kernel of
    their own or in the prologue of the output projection, the logits are the same bit for bit, with contexts
    of one run of keys and of several, through graphs and without."""
    from macllm_infer_amd import Engine, Lane
    from macllm_infer_amd.parts import fused
    from macllm_infer_amd.config import FalconH1Config
    from macllm_infer_amd.weights.random_init import random_tensors
    config = FalconH1Config.from_dict(dict(tiny_configs.TINY_C, max_position_embeddings=4096))
    tensors = random_tensors(config, 5, torch.bfloat16, "unit")
    prompts = {index: tokens_for(config.vocab_size, length, 700 + index) for index, length in enumerate([700, 3, 260, 41, 1030])}
    results = {}
    for later in (False, True):
        monkeypatch.setattr(fused, "FORCE_MERGE_LATER", later)
        for graphs in (False, True):
            engine = Engine(config=config, tensors=tensors, dtype="bfloat16", kv_cache_block_tokens=16,
                            kv_cache_capacity_tokens=4096, max_active_sequences=8, decode_graphs=graphs)
            fusion = engine.model.blocks[0].fusion
            assert fusion.kernel is not None and not fusion.library_out[0] and not fusion.split_out[0]
            for index, tokens in prompts.items():
                engine.add_request(index)
                engine.step([Lane(index, tokens[:-1], [])])
            rows = []
            for turn in range(4):
                lanes = [Lane(index, [tokens[-1] if turn == 0 else 5 + turn], [0]) for index, tokens in prompts.items()]
                rows.append(engine.step(lanes[:1 + turn] if turn < 2 else lanes).float().cpu())
            results[later, graphs] = torch.cat(rows)
    for key, rows in results.items():
        assert torch.equal(rows, results[False, False]), key


def test_graphs_come_in_buckets_of_context_length():
    """A model that allows long contexts: a short request decodes through a graph made for 2,048
    tokens, a longer one through a graph made for 4,096 (wider block tables, more runs of keys),
    beside each other through the wider one; all say what an engine without graphs says."""
    from macllm_infer_amd import Engine, Lane
    from macllm_infer_amd.config import FalconH1Config
    from macllm_infer_amd.weights.random_init import random_tensors
    config = FalconH1Config.from_dict(dict(tiny_configs.TINY_C, max_position_embeddings=16384))
    tensors = random_tensors(config, 4, torch.bfloat16, "unit")
    make = lambda graphs: Engine(config=config, tensors=tensors, dtype="bfloat16", kv_cache_capacity_tokens=8192,
                                 max_active_sequences=2, decode_graphs=graphs)
    with_graphs, eager = make(True), make(False)
    short, long = tokens_for(config.vocab_size, 40, 1), tokens_for(config.vocab_size, 2100, 2)

    def both(lanes):
        got, want = with_graphs.step(lanes).float().cpu(), eager.step(lanes).float().cpu()
        assert got.shape == want.shape
        if got.numel():
            assert (got - want).abs().max() <= 3e-2 * max(1.0, want.abs().max().item())

    for engine in (with_graphs, eager):
        engine.add_request("short")
        engine.add_request("long")
    both([Lane("short", short[:30], [29])])
    for token in short[30:35]:
        both([Lane("short", [token], [0])])
    assert set(with_graphs.graphs._graphs) == {(1, 2048)}
    both([Lane("long", long[:2050], [2049])])
    for token in long[2050:2055]:
        both([Lane("long", [token], [0])])
    assert set(with_graphs.graphs._graphs) == {(1, 2048), (1, 4096)}
    for first, second in zip(short[35:40], long[2055:2060]):
        both([Lane("short", [first], [0]), Lane("long", [second], [0])])
    assert set(with_graphs.graphs._graphs) == {(1, 2048), (1, 4096), (2, 4096)}
    both([Lane("short", [short[39]], [0])])                               # and back through the narrow one
    assert with_graphs.graphs.counts["decode_replays"] == 16


def sharpened(tensors, factor=8.0):
    """Random weights give every key nearly the same score, and a fault in one far page is then one part in
    thousands of an attended row.  With the query and key projections scaled up the scores spread over several
    units and a few keys anywhere in the context carry a row: a wrong page, run of keys or rotation shows."""
    out = dict(tensors)
    for name, tensor in tensors.items():
        if name.endswith("q_proj.weight") or name.endswith("k_proj.weight"):
            out[name] = (tensor.float() * factor).to(tensor.dtype)
    return out


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_contexts_beyond_2048_tokens_match_the_plain_model(dtype):
    """What the benchmark's contexts go through, against the plain model: a prompt of 2,100 tokens in portions of
    512 (the second portion captures the graph of its capacity, the later ones replay it, the last ones through
    the wider bucket of contexts), then eight decode steps of three requests at 2,100, 700 and 40 tokens in one
    batch (several runs of keys for one request beside a single short one).  Every row is wanted and compared.
    The attention scores are sharpened so that far keys count (``sharpened``)."""
    import gates
    from macllm_infer_amd import Engine, Lane
    from macllm_infer_amd.config import FalconH1Config
    from macllm_infer_amd.weights.random_init import random_tensors
    config = FalconH1Config.from_dict(dict(tiny_configs.TINY_C, max_position_embeddings=16384))
    storage = torch.float32 if dtype == "float32" else torch.bfloat16
    tensors = sharpened(random_tensors(config, 4, storage, "unit"))
    plain = {name: tensor.float() for name, tensor in tensors.items()}
    cfg = config.to_dict()
    lengths = {"long": 2100, "mid": 700, "short": 40}
    tokens = {name: tokens_for(config.vocab_size, count + 8, 70 + index) for index, (name, count) in enumerate(lengths.items())}
    engine = Engine(config=config, tensors=tensors, dtype=dtype, kv_cache_capacity_tokens=4096, max_active_sequences=3)
    rows = {name: [] for name in tokens}
    for name in tokens:
        engine.add_request(name)
    for first in range(0, 2100, 512):
        count = min(512, 2100 - first)
        rows["long"].append(engine.step([Lane("long", tokens["long"][first:first + count], list(range(count)))]).cpu())
    if engine.graphs is not None:
        assert engine.graphs.counts["bucket_captures"] >= 1 and engine.graphs.counts["bucket_replays"] >= 3
    mixed = engine.step([Lane("mid", tokens["mid"][:700], list(range(700))),
                         Lane("short", tokens["short"][:40], list(range(40)))]).cpu()
    rows["mid"].append(mixed[:700])
    rows["short"].append(mixed[700:])
    for turn in range(8):
        out = engine.step([Lane(name, [tokens[name][lengths[name] + turn]], [0]) for name in tokens]).cpu()
        for row, name in enumerate(tokens):
            rows[name].append(out[row:row + 1])
    for name in tokens:
        want = plain_impl.falcon_h1_logits(cfg, plain, tokens[name]).numpy()
        got = torch.cat(rows[name]).numpy()
        assert got.shape == want.shape
        if dtype == "float32":
            ok, text = gates.conditioned_close_f32(got, want, cfg, plain, tokens[name])
        else:
            ok, text = gates.conditioned_close(got, want, cfg, plain, tokens[name])
        assert ok, f"{name}: {text}"
        # the far keys do count: the same rows with the first 256 positions' keys and values out of reach
        # (the sequence without its first 256 tokens) are somewhere else
    shifted = plain_impl.falcon_h1_logits(cfg, plain, tokens["long"][256:]).numpy()
    whole = plain_impl.falcon_h1_logits(cfg, plain, tokens["long"]).numpy()
    assert np.abs(shifted[-8:] - whole[-8:]).max() > 0.05 * np.abs(whole).max()
    engine.cache.check()


@pytest.mark.parametrize("name, dtype", [("C", "bfloat16"), ("B", "float32")])
def test_capacity_graphs_with_four_lanes_and_padding_match_the_plain_model(tmp_path, name, dtype):
    """Steps of four lanes (portions of changing sizes beside single tokens) whose tokens do not fill a capacity:
    the graph of eight lanes is captured at the second step and replayed for the rest, with three padding lanes of
    one token and one that holds the remainder; every row against the plain model, not against another path of
    the engine."""
    import gates
    from macllm_infer_amd import Engine, Lane
    storage = torch.float32 if dtype == "float32" else torch.bfloat16
    folder = tiny_configs.make_model_dir(name, tmp_path, storage)
    cfg, tensors = plain_impl.load_model_dir(folder)
    plain = {key: value.float() for key, value in tensors.items()}
    engine = Engine(folder, dtype=dtype, kv_cache_block_tokens=8, kv_cache_capacity_tokens=768, max_active_sequences=4)
    engine.split_from_lanes = 1 << 30                       # one batch a step, whatever it holds
    sequences = {key: tokens_for(cfg["vocab_size"], 150, 40 + index) for index, key in enumerate("abcd")}
    cursor = {key: 0 for key in sequences}
    rows = {key: [] for key in sequences}
    for key in sequences:
        engine.add_request(key)
    shapes = [(20, 1, 15, 2), (1, 19, 3, 13), (9, 9, 9, 9), (2, 1, 30, 1), (17, 16, 2, 2), (1, 1, 1, 34), (5, 21, 1, 11),
              (12, 3, 12, 12)]
    for shape in shapes:                                                     # 33 to 48 tokens each: one capacity
        assert 32 < sum(shape) <= 44
        lanes = [Lane(key, sequences[key][cursor[key]:cursor[key] + count], list(range(count)))
                 for key, count in zip(sequences, shape)]
        out = engine.step(lanes).cpu()
        for key, count in zip(sequences, shape):
            rows[key].append(out[:count])
            out = out[count:]
            cursor[key] += count
    counts = engine.graphs.counts
    assert counts["bucket_captures"] == 1 and counts["bucket_replays"] == len(shapes) - 1 and counts["bucket_eager"] == 1
    assert [key[:2] for key in engine.graphs._bucket_graphs] == [(8, 48)]
    for key, sequence in sequences.items():
        want = plain_impl.falcon_h1_logits(cfg, plain, sequence[:cursor[key]]).numpy()
        got = torch.cat(rows[key]).numpy()
        ok = gates.float32_close(got, want) if dtype == "float32" else gates.bfloat16_close(got, want)
        assert ok, f"{key}: {np.abs(got - want).max():.3e} of {np.abs(want).max():.2f}"
    engine.cache.check()


def test_layers_of_one_mixer_and_a_mixer_from_outside_take_the_fast_paths(monkeypatch):
    """The fast paths of a layer belong to no model: a layer with attention alone decodes through the skinny
    kernels (norm in the prologue, SiLU(g)*u in the epilogue), and so do the projections of a toy mixer with
    state of its own that is registered from the tests and hands out its pieces, between toy norms and before
    a routed toy feed-forward, which run through their own ``forward``.  Nothing in the package is edited."""
    import gates
    from macllm_infer_amd import Engine, Lane
    from macllm_infer_amd.kernels import ops
    from macllm_infer_amd.weights.random_init import random_tensors
    toy_parts.register_toys()
    raw = {"architectures": ["ToyFastForTests"], "hidden": 64, "vocab": 150, "width": 96, "decay": 0.8}
    config = toy_parts.ToyFastConfig(raw)
    tensors = random_tensors(config, 9, torch.bfloat16, "unit")
    engine = Engine(config=config, tensors=tensors, dtype="bfloat16", kv_cache_block_tokens=16,
                    kv_cache_capacity_tokens=512, max_active_sequences=3)
    first, second = engine.model.blocks[0].fusion, engine.model.blocks[1].fusion
    assert first is not None and first.decode_ok and first.norm_fits and first.gate_up is not None and first.kernel is None
    assert second is not None and second.decode_ok and second.mixer_rms is None and second.gate_up is None
    assert second.in_width == 192 and second.mixed_width == 96
    calls = {"skinny": 0, "library": 0}
    real_skinny, real_library = ops.fused_gemm, ops.linear

    def skinny(*arguments, **named):
        calls["skinny"] += 1
        return real_skinny(*arguments, **named)

    def library(*arguments, **named):
        calls["library"] += 1
        return real_library(*arguments, **named)

    calls["to the stream"] = 0
    real_residual = ops.fused_gemm_residual

    def to_the_stream(*arguments, **named):
        calls["to the stream"] += 1
        return real_residual(*arguments, **named)

    monkeypatch.setattr(ops, "fused_gemm", skinny)
    monkeypatch.setattr(ops, "fused_gemm_residual", to_the_stream)
    monkeypatch.setattr(ops, "linear", library)
    sequences = {"a": tokens_for(150, 60, 21), "b": tokens_for(150, 45, 22)}
    rows = {"a": [], "b": []}
    for name in sequences:
        engine.add_request(name)
    out = engine.step([Lane("a", sequences["a"][:40], list(range(40))), Lane("b", sequences["b"][:30], list(range(30)))])
    rows["a"].append(out[:40].cpu()), rows["b"].append(out[40:].cpu())
    assert calls["skinny"] == 0 and calls["library"] > 0          # a prompt portion: the fused matrices, library products
    calls.update(skinny=0, library=0)
    for position in range(15):
        out = engine.step([Lane("a", [sequences["a"][40 + position]], [0]), Lane("b", [sequences["b"][30 + position]], [0])])
        rows["a"].append(out[:1].cpu()), rows["b"].append(out[1:].cpu())
    # a decode step: input and output projections of both layers, gate/up and down of the first, and the head; the
    # first layer's output projection adds to the stream itself and leaves the norm to gate/up (its down projection
    # does not: the toy norm that follows is none it could prepare for)
    assert calls["skinny"] == 15 * 6 and calls["to the stream"] == 15 and calls["library"] == 0
    for name, tokens in sequences.items():
        want = toy_parts.toy_fast_plain_logits(raw, tensors, tokens[:len(torch.cat(rows[name]))]).numpy()
        assert gates.bfloat16_close(torch.cat(rows[name]).numpy(), want), name
    engine.cache.check()


def test_replays_that_follow_one_another_without_a_wait_keep_their_own_arrays(tmp_path):
    """Steps of one captured shape whose logits nobody wants (portions of prompts, decoded tokens of a
    replay that asks for nothing) are queued one behind the other while the GPU is still busy with earlier
    work: each replay must run with the positions, cells and block tables that were packed for it, not with
    those of a step packed later.  The host is made to run ahead by a second of matrix products queued
    first; the engine beside it launches the same steps kernel by kernel."""
    from macllm_infer_amd import Engine, Lane
    folder = tiny_configs.make_model_dir("C", tmp_path, torch.bfloat16)
    cfg, tensors = plain_impl.load_model_dir(folder)
    plain = {key: tensor.float() for key, tensor in tensors.items()}
    make = lambda graphs: Engine(folder, dtype="bfloat16", kv_cache_block_tokens=16, kv_cache_capacity_tokens=2048,
                                 max_active_sequences=6, decode_graphs=graphs)
    with_graphs, eager = make(True), make(False)
    names = "abcde"
    streams = {key: tokens_for(cfg["vocab_size"], 64 * 3 + 12, 40 + index) for index, key in enumerate(names)}
    for engine in (with_graphs, eager):
        for key in names:
            engine.add_request(key)
    # a step of this size (one lane of 64 tokens) comes again and its capacity is captured
    plan = [("a", 0), ("b", 0), ("c", 0)]
    busy = [("a", 64), ("b", 64), ("c", 64), ("d", 0), ("e", 0), ("a", 128), ("d", 64), ("e", 64)]
    for key, first in plan:
        for engine in (with_graphs, eager):
            assert engine.step([Lane(key, streams[key][first:first + 64], [])]).shape[0] == 0
    assert with_graphs.graphs.counts["bucket_captures"] == 1 and with_graphs.graphs.counts["bucket_replays"] == 2
    ballast = torch.randn(4096, 4096, device=DEV, dtype=torch.bfloat16)
    for engine in (with_graphs, eager):
        torch.cuda.synchronize()
        for _ in range(200):                           # some hundred milliseconds of work the steps queue behind
            ballast @ ballast
        for key, first in busy:
            engine.step([Lane(key, streams[key][first:first + 64], [])])
    assert with_graphs.graphs.counts["bucket_replays"] == 2 + len(busy)
    # decoded tokens, every request in a step of its own with nothing wanted, then all at once with their logits
    cursor = {"a": 192, "b": 128, "c": 128, "d": 128, "e": 128}
    for engine in (with_graphs, eager):
        for _ in range(100):
            ballast @ ballast
        for turn in range(4):
            for key in names:
                engine.step([Lane(key, [streams[key][cursor[key] + turn]], [])])
    lanes = [Lane(key, [streams[key][cursor[key] + 4]], [0]) for key in names]
    got, want = with_graphs.step(lanes).float().cpu(), eager.step(lanes).float().cpu()
    assert with_graphs.graphs.counts["decode_replays"] == 21
    assert (got - want).abs().max() <= 3e-2 * max(1.0, want.abs().max().item())
    for key in names:                                  # and against the plain model
        exact = plain_impl.falcon_h1_logits(cfg, plain, streams[key][:cursor[key] + 5])[-1]
        row = got[names.index(key)]
        assert (row - exact).abs().max() <= 6e-2 * exact.abs().max(), key


@pytest.mark.parametrize("name, dtype", [("B", "float32"), ("C", "bfloat16")])
def test_portion_graphs_match_eager_steps(tmp_path, name, dtype):
    """Steps with prompt portions run from graphs captured for a capacity (so many tokens in so many lanes):
    portions of 70 and 40 tokens and of 60 and 40 meet the graph of 112 tokens in 4 lanes from their second
    sighting on, a portion of 10 tokens the one of 16 tokens in 2 lanes, portions beside three decoded tokens
    one more; four decoded tokens beside a portion run as a batch of their own.  Every step, through pages that are given back and
    used again and with decode replays between, is compared with an engine without graphs."""
    from macllm_infer_amd import Engine, Lane
    folder = tiny_configs.make_model_dir(name, tmp_path, torch.float32 if dtype == "float32" else torch.bfloat16)
    cfg, _ = plain_impl.load_model_dir(folder)
    make = lambda graphs: Engine(folder, dtype=dtype, kv_cache_block_tokens=16, kv_cache_capacity_tokens=640,
                                 max_active_sequences=5, decode_graphs=graphs)
    with_graphs, eager = make(True), make(False)

    def both(lanes):
        got, want = with_graphs.step(lanes).float().cpu(), eager.step(lanes).float().cpu()
        scale = max(1.0, want.abs().max().item())
        assert got.shape == want.shape
        assert (got - want).abs().max() <= (1e-5 if dtype == "float32" else 3e-2) * scale

    for round_index in range(4):
        a, b = f"a{round_index}", f"b{round_index}"
        tokens_a = tokens_for(cfg["vocab_size"], 141, 700 + round_index)
        tokens_b = tokens_for(cfg["vocab_size"], 81, 800 + round_index)
        for engine in (with_graphs, eager):
            engine.add_request(a)
            engine.add_request(b)
        first = [Lane(a, tokens_a[:70], [3, 69]), Lane(b, tokens_b[:40], [39])]
        both(first if round_index % 2 == 0 else first[::-1])
        both([Lane(a, tokens_a[70:130], [3, 59]), Lane(b, tokens_b[40:80], [39])])      # other lengths, the same capacity
        both([Lane(a, tokens_a[130:140], [9])])                                           # a capacity of its own (16 tokens)
        both([Lane(a, tokens_a[140:], [0]), Lane(b, tokens_b[80:], [0])])                 # a decode replay between
        for engine in (with_graphs, eager):
            engine.finish(a)
            engine.finish(b)
    assert sorted(key[:2] for key in with_graphs.graphs._bucket_graphs) == [(2, 16), (4, 112)]
    assert with_graphs.graphs.counts["bucket_eager"] == 2 and with_graphs.graphs.counts["bucket_replays"] == 10
    assert with_graphs.cache.stats() == eager.cache.stats()
    # decoded tokens beside a portion: three, then four single-token lanes share one graph (padded to four)
    for engine in (with_graphs, eager):
        for key in "pqrst":
            engine.add_request(key)
    streams = {key: tokens_for(cfg["vocab_size"], 400, 950 + index) for index, key in enumerate("pqrst")}
    cursor = {key: 0 for key in streams}

    def lane(key, count, want):
        tokens = streams[key][cursor[key]:cursor[key] + count]
        cursor[key] += count
        return Lane(key, tokens, want)

    both([lane(key, 5, [4]) for key in "pqrs"])
    replays = with_graphs.graphs.counts["bucket_replays"]
    for turn in range(6):
        lanes = [lane(key, 1, [0]) for key in "pqr"] + [lane("t", 32, [31] if turn == 5 else [])]
        both(lanes if turn % 2 == 0 else lanes[::-1])
    # three decoded tokens beside a portion of 32: 48 tokens in 8 lanes (four cannot be padded), whatever their order
    assert (8, 48) in [key[:2] for key in with_graphs.graphs._bucket_graphs]
    assert with_graphs.graphs.counts["bucket_replays"] == replays + 5
    # four decoded tokens beside a portion are a batch of their own (where the clock, set aside here, says so): the
    # portion goes through the graph of its capacity, the four through a decode graph, and the logits come back in
    # the order of the lanes
    with_graphs.split_from_lanes = eager.split_from_lanes = 4
    replays, decodes = with_graphs.graphs.counts["bucket_replays"], with_graphs.graphs.counts["decode_replays"]
    for turn in range(4):
        lanes = [lane(key, 1, [0]) for key in "pq"] + [lane("t", 20, [0, 19] if turn != 1 else [])]
        lanes += [lane(key, 1, [0]) for key in "rs"]
        both(lanes if turn % 2 == 0 else lanes[::-1])
    assert with_graphs.graphs.counts["decode_replays"] == decodes + 4
    assert with_graphs.graphs.counts["bucket_replays"] == replays + 3


@pytest.mark.parametrize("name, dtype, seed, shared", [("B", "float32", 0, False), ("C", "bfloat16", 1, False),
                                                      ("A", "bfloat16", 2, False), ("C", "bfloat16", 3, True)])
def test_steps_of_any_shape_through_graphs_of_a_capacity_match_eager_steps(tmp_path, monkeypatch, name, dtype, seed, shared):
    """Sixty steps drawn at random (one to five lanes, portions of 2 to 90 tokens beside decoded tokens, wanted
    places anywhere or nowhere, requests that end and begin) through an engine with graphs, some of them
    captured before the first request, beside an engine that launches every step kernel by kernel: the same
    logits and the same cache accounting, whichever way a step went (a capacity's first sighting is launched,
    later ones replay its graph), and a step whose capacity was warmed up replays at once.  ``shared``: the engine
    with graphs takes the kernel that shares the rows wherever a product of a step of 17 to 64 tokens has it
    (in slabs where it feeds the stream), the other engine none of it."""
    import random
    from macllm_infer_amd import Engine, Lane
    from macllm_infer_amd.parts import fused
    folder = tiny_configs.make_model_dir(name, tmp_path, torch.float32 if dtype == "float32" else torch.bfloat16)
    cfg, _ = plain_impl.load_model_dir(folder)
    make = lambda graphs: Engine(folder, dtype=dtype, kv_cache_block_tokens=8, kv_cache_capacity_tokens=3000,
                                 max_active_sequences=6, decode_graphs=graphs)
    if shared:
        monkeypatch.setattr(fused, "FORCE_SPLIT", 2)
        monkeypatch.setattr(fused, "FORCE_SHARED_ROWS", 1)
    with_graphs = make(True)
    if shared:
        assert with_graphs.model.blocks[0].fusion.tiles_out[3:6] == with_graphs.model.blocks[0].fusion.tiles_in[3:6] == (-1,) * 3
        monkeypatch.setattr(fused, "FORCE_SPLIT", None)
        monkeypatch.setattr(fused, "FORCE_SHARED_ROWS", None)
    eager = make(False)
    captured = with_graphs.warm_up([(1, 1), (4, 4), (1, 40), (2, 100), (3, 130), (5, 200)])
    assert len(captured) == 6 and with_graphs.graphs.counts["bucket_replays"] == 0
    first = tokens_for(cfg["vocab_size"], 100, 2999)
    for engine in (with_graphs, eager):
        engine.add_request("warm")
        engine.add_request("warmer")
    lanes = [Lane("warm", first[:63], [62]), Lane("warmer", first[63:], [0])]
    got, want = with_graphs.step(lanes).float().cpu(), eager.step(lanes).float().cpu()
    assert with_graphs.graphs.counts["bucket_replays"] == 1 and with_graphs.graphs.counts["bucket_eager"] == 0
    assert (got - want).abs().max() <= (1e-5 if dtype == "float32" else 3e-2) * max(1.0, want.abs().max().item())
    for engine in (with_graphs, eager):
        engine.finish("warm")
        engine.finish("warmer")
    rng = random.Random(seed)
    live, serial = {}, 0
    for step in range(60):
        while len(live) < 5 and (len(live) < 2 or rng.random() < 0.3):
            live[f"r{serial}"] = [tokens_for(cfg["vocab_size"], rng.randrange(20, 260), 3000 + serial), 0]
            serial += 1
            for engine in (with_graphs, eager):
                engine.add_request(f"r{serial - 1}")
        picked = rng.sample(sorted(live), rng.randrange(1, len(live) + 1))
        lanes = []
        for key in picked:
            tokens, cursor = live[key]
            count = min(len(tokens) - cursor, 1 if rng.random() < 0.4 else rng.randrange(2, 91))
            want = sorted(rng.sample(range(count), rng.randrange(0, min(count, 3) + 1)))
            lanes.append(Lane(key, tokens[cursor:cursor + count], want))
            live[key][1] += count
        got, want = with_graphs.step(lanes).float().cpu(), eager.step(lanes).float().cpu()
        assert got.shape == want.shape
        if want.numel():
            scale = max(1.0, want.abs().max().item())
            assert (got - want).abs().max() <= (1e-5 if dtype == "float32" else 3e-2) * scale, f"step {step}"
        for key in picked:
            if live[key][1] == len(live[key][0]):
                del live[key]
                for engine in (with_graphs, eager):
                    engine.finish(key)
        assert with_graphs.cache.stats() == eager.cache.stats()
    counts = with_graphs.graphs.counts
    assert counts["bucket_eager"] + counts["bucket_replays"] + counts["decode_replays"] == 61
    assert counts["bucket_replays"] >= 12 and counts["bucket_captures"] >= 8
    with_graphs.cache.check()


@pytest.mark.parametrize("name", ["C", "D"])
def test_long_portions_overlap_their_mixers(tmp_path, name):
    """Portions of 256 tokens and more run attention on a second stream beside the state-space
    chain (with the conv inside the chunked scan): a prompt of 300 tokens beside one of 259, launched kernel
    by kernel and, from the second step of that size on, from a captured graph; then the same requests go on
    with a portion and a decoded token.  Every wanted row against the plain model."""
    from macllm_infer_amd import Engine, Lane
    from macllm_infer_amd.parts import block
    folder = tiny_configs.make_model_dir(name, tmp_path, torch.bfloat16)
    cfg, tensors = plain_impl.load_model_dir(folder)
    engine = Engine(folder, dtype="bfloat16", kv_cache_block_tokens=16, kv_cache_capacity_tokens=4096,
                    max_active_sequences=8)
    assert engine.model.blocks[0].fusion is not None and block.OVERLAP_MIN_TOKENS <= 259

    def check(got, want):
        scale = want.abs().max().item()
        assert (got - want).abs().max().item() <= 6e-2 * scale
        assert ((got - want).pow(2).mean().sqrt() / want.pow(2).mean().sqrt()).item() <= 3e-2

    for turn in range(4):
        a, b = f"a{turn}", f"b{turn}"
        tokens_a = tokens_for(cfg["vocab_size"], 340, 1000 + turn)
        tokens_b = tokens_for(cfg["vocab_size"], 270, 1100 + turn)
        engine.add_request(a)
        engine.add_request(b)
        logits = engine.step([Lane(a, tokens_a[:300], [0, 150, 299]), Lane(b, tokens_b[:259], [258])]).float().cpu()
        want_a = plain_impl.falcon_h1_logits(cfg, tensors, tokens_a)
        want_b = plain_impl.falcon_h1_logits(cfg, tensors, tokens_b)
        check(logits[:3], want_a[[0, 150, 299]])
        check(logits[3:], want_b[[258]])
        logits = engine.step([Lane(a, tokens_a[300:], [39]), Lane(b, tokens_b[259:260], [0])]).float().cpu()
        check(logits[:1], want_a[[339]])
        check(logits[1:], want_b[[259]])
        engine.finish(a)
        engine.finish(b)
    assert engine.graphs.counts["bucket_replays"] >= 5


def test_the_second_stream_is_never_the_stream_it_runs_beside(monkeypatch):
    """Streams come from a pool that hands them out in turn; whichever of them a graph is captured on, the
    stream that the first mixer of a long portion runs on is another one (on the same one the two mixers
    would run one after the other), and two streams are all that is ever drawn for it."""
    from macllm_infer_amd.parts import block
    monkeypatch.setattr(block, "_side_streams", {})
    device = torch.device(DEV)
    pool = [torch.cuda.Stream(device=device) for _ in range(70)]           # every stream of the pool, twice over
    for main in pool + [torch.cuda.current_stream(device)]:
        side = block.side_stream(device, main)
        assert side != main and side.device == main.device
    assert len(block._side_streams[device.index]) <= 2


@pytest.mark.parametrize("name", ["A", "B"])
def test_long_float32_portions_overlap_their_mixers_and_keep_their_bits(tmp_path, monkeypatch, name):
    """The float32 path runs a layer part by part; in a captured graph the two mixers of a portion of 256 tokens
    or more run beside each other on two streams there too.  Prompts of 300 and 259 tokens beside each other, the
    same shape of step four times over (launched kernel by kernel first, from the graph of its capacity after):
    every replay gives the bits of an engine without graphs, which never leaves one stream."""
    from macllm_infer_amd import Engine, Lane
    from macllm_infer_amd.parts import block
    folder = tiny_configs.make_model_dir(name, tmp_path, torch.float32)
    cfg, _ = plain_impl.load_model_dir(folder)
    forks = []
    real = block.side_stream
    monkeypatch.setattr(block, "side_stream", lambda device, beside: (forks.append(1), real(device, beside))[1])
    make = lambda graphs: Engine(folder, dtype="float32", kv_cache_block_tokens=16, kv_cache_capacity_tokens=4096,
                                 max_active_sequences=8, decode_graphs=graphs)
    with_graphs, eager = make(True), make(False)
    assert with_graphs.model.blocks[0].fusion is None
    for turn in range(4):
        a, b = f"a{turn}", f"b{turn}"
        tokens_a = tokens_for(cfg["vocab_size"], 340, 2000 + turn)
        tokens_b = tokens_for(cfg["vocab_size"], 270, 2100 + turn)
        rows = []
        for engine in (with_graphs, eager):
            engine.add_request(a)
            engine.add_request(b)
            first = engine.step([Lane(a, tokens_a[:300], [0, 150, 299]), Lane(b, tokens_b[:259], [258])]).cpu()
            second = engine.step([Lane(a, tokens_a[300:], [39]), Lane(b, tokens_b[259:260], [0])]).cpu()
            rows.append(torch.cat([first, second]))
            engine.finish(a)
            engine.finish(b)
        assert torch.equal(rows[0], rows[1]), turn
    assert with_graphs.graphs.counts["bucket_replays"] >= 2
    assert len(forks) >= len(cfg_layers(cfg))                   # every layer of the captured step forked


def cfg_layers(cfg):
    return range(cfg["num_hidden_layers"])


@pytest.mark.parametrize("padding", [False, True])
def test_a_wide_model_runs_through_the_fast_paths(tmp_path, monkeypatch, padding):
    """Hidden size 2 112: the fused layer paths are built although the norm prologue does not fit;
    prompt portions, a mixed step and graph-replayed decode steps against the plain model.
    ``padding``: the input projection of prompt portions multiplies with rows of zeros added up to
    a multiple of 256 features (what a measurement at build decides for large weights)."""
    from macllm_infer_amd import Engine, Lane
    from macllm_infer_amd.parts import fused
    monkeypatch.setattr(fused, "FORCE_PADDING", padding)
    folder = tiny_configs.make_model_dir("D", tmp_path, torch.bfloat16)
    cfg, tensors = plain_impl.load_model_dir(folder)
    engine = Engine(folder, dtype="bfloat16", kv_cache_block_tokens=16, kv_cache_capacity_tokens=512,
                    max_active_sequences=3)
    fusion = engine.model.blocks[0].fusion
    assert fusion is not None and not fusion.norm_fits and fusion.general
    assert (fusion.w_in_wide.shape[0] % 256 == 0) == padding and fusion.w_in.shape[0] == fusion.in_width
    assert fusion.w_in.data_ptr() == fusion.w_in_wide.data_ptr()
    sequences = {key: tokens_for(cfg["vocab_size"], 70 + 9 * index, 900 + index) for index, key in enumerate("abc")}
    got = {key: [] for key in sequences}
    for key in sequences:
        engine.add_request(key)

    def step(spec):
        lanes = [Lane(key, sequences[key][start:start + count], list(range(count))) for key, start, count in spec]
        logits = engine.step(lanes).float().cpu()
        row = 0
        for key, start, count in spec:
            got[key].append(logits[row:row + count])
            row += count

    step([("a", 0, 40), ("b", 0, 33)])
    step([("a", 40, 1), ("b", 33, 30), ("c", 0, 70)])                  # a decoded token beside portions
    cursor = {"a": 41, "b": 63, "c": 70}
    while any(cursor[key] < len(sequences[key]) for key in sequences):
        live = [key for key in sequences if cursor[key] < len(sequences[key])]
        step([(key, cursor[key], 1) for key in live])
        for key in live:
            cursor[key] += 1
    assert engine.graphs is not None and engine.graphs._graphs
    for key, tokens in sequences.items():
        want = plain_impl.falcon_h1_logits(cfg, tensors, tokens)
        have = torch.cat(got[key])
        scale = want.abs().max().item()
        assert (have - want).abs().max().item() <= 6e-2 * scale
        assert ((have - want).pow(2).mean().sqrt() / want.pow(2).mean().sqrt()).item() <= 3e-2


# Seeds 0 to 7 of both draws, and the cases of earlier sweeps (100 and 60 seeds) whose bfloat16 logits left the
# plain gate.  Every one of them is the model's conditioning, not a kernel: the plain model with its
# activations rounded to bfloat16 departs from the exact one as far at the same positions (3038: a width of 40
# over one state-space head of 64 x 64 with the gated norm, off by the whole scale at position 52, where the
# float32 engine is off by 3e-4 instead of 3e-6; 3024: 0.27 of the scale at position 195; 3022, 3040, 3041 and
# the odd draw's 1, 3, 12, 22, 23, 28, 34, 57: 0.06 to 0.18).  ``gates.conditioned_close`` states the gate in
# those terms.
# A further sweep (seeds 7000 to 7059 of the even draw, 8000 to 8039 of the odd one) left the fixed gates at 7019
# in float32 (one position, where the plain model in float32 is itself 7.7e-4 from the plain model in float64:
# ``gates.conditioned_close_f32``) and in bfloat16 at 7019, 7027, 7039, 7047, 7054 and the odd draw's 8002, 8009,
# 8011; those run here in both dtypes, under the gates that state the model's own rounding noise.
RANDOM_CASES = ([(seed, False) for seed in range(8)] + [(seed, True) for seed in range(8)]
                + [(seed, False) for seed in (3022, 3024, 3038, 3040, 3041)]
                + [(seed, True) for seed in (12, 22, 23, 28, 34, 57)]
                + [(seed, False) for seed in (7019, 7027, 7039, 7047, 7054)]
                + [(seed, True) for seed in (8002, 8009, 8011)]
                + [(9109, False), (9305, True)])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed, odd", RANDOM_CASES)
def test_configurations_drawn_at_random_match_the_plain_model(seed, odd, dtype):
    """Every size and option at random (head sizes 16..128 in steps of 16, 1..12 heads, widths and
    vocabularies that are multiples of nothing, multipliers 0.5..2, pages of 4..64 tokens; ``odd``: sizes no
    matrix-core kernel takes): whole, and two requests cut at random beside each other with their last tokens
    one by one."""
    import gates
    from macllm_infer_amd import Engine, Lane
    from macllm_infer_amd.config import FalconH1Config
    from macllm_infer_amd.weights.random_init import random_tensors
    raw, page, rng = tiny_configs.random_config(seed, odd)
    config = FalconH1Config.from_dict(raw)
    cfg = config.to_dict()
    tensors = random_tensors(config, seed, torch.float32 if dtype == "float32" else torch.bfloat16, "unit")
    plain = {name: tensor.float() for name, tensor in tensors.items()}
    generator = torch.Generator().manual_seed(seed)
    tokens = {"a": torch.randint(0, raw["vocab_size"], (rng.choice([70, 131, 200]),), generator=generator).tolist()}
    tokens["b"] = torch.randint(0, raw["vocab_size"], (rng.choice([9, 40, 77]),), generator=generator).tolist()
    wanted = {name: plain_impl.falcon_h1_logits(cfg, plain, tokens[name]).numpy() for name in tokens}

    def close(got, name, what):
        want = wanted[name]
        if dtype == "float32":
            ok, text = gates.conditioned_close_f32(got, want, cfg, plain, tokens[name])
        else:
            ok, text = gates.conditioned_close(got, want, cfg, plain, tokens[name])
        assert ok, f"seed {seed} {what}: {text}"

    engine = Engine(config=config, tensors=tensors, dtype=dtype, kv_cache_block_tokens=page,
                    kv_cache_capacity_tokens=640, max_active_sequences=3)
    engine.add_request("whole")
    close(engine.step([Lane("whole", tokens["a"], list(range(len(tokens["a"]))))]).cpu().numpy(), "a", "whole")
    engine.finish("whole")
    engine.add_request("a")
    engine.add_request("b")
    cursor, rows = {"a": 0, "b": 0}, {"a": [], "b": []}
    while cursor["a"] < len(tokens["a"]) or cursor["b"] < len(tokens["b"]):
        lanes = []
        for name, tail, sizes in (("a", 12, [2, 5, 17, 64, 33]), ("b", 6, [2, 3, 11, 30])):
            left = len(tokens[name]) - cursor[name]
            if left > 0 and (name == "a" or rng.random() < 0.7):
                count = 1 if left <= tail else min(rng.choice(sizes), left - tail)
                lanes.append(Lane(name, tokens[name][cursor[name]:cursor[name] + count], list(range(count))))
        if not lanes:
            continue
        out = engine.step(lanes).cpu().numpy()
        for lane in lanes:
            rows[lane.request].append(out[:len(lane.tokens)])
            out = out[len(lane.tokens):]
            cursor[lane.request] += len(lane.tokens)
    for name in ("a", "b"):
        close(np.concatenate(rows[name]), name, f"cut {name}")
    engine.cache.check()


@pytest.mark.parametrize("shape, layers, vocab", [("0.5b", 2, None), ("7b", 1, 1003)])
def test_layers_of_the_benchmark_shapes_match_the_plain_model(shape, layers, vocab):
    """Layers with the sizes bench.py measures (0.5B shape: width 1024, 8 query heads on 2, 24
    state-space heads of 64 x 128, chunk 128, a vocabulary of 32,784; 7B shape: width 3072, 12 query
    heads of 128 on 2, state-space heads of 128 x 256, a small vocabulary), through the paths those
    sizes take: a prompt in portions long enough for the chunked scan, the matrix-core attention and
    the library's products, replayed from captured graphs, then decoding in a batch of three."""
    import bench
    from macllm_infer_amd import Engine, Lane
    from macllm_infer_amd.config import FalconH1Config
    from macllm_infer_amd.weights.random_init import random_tensors
    from gates import bfloat16_close
    raw = dict(bench.SHAPES[shape], num_hidden_layers=layers)
    config = FalconH1Config.from_dict(dict(raw, vocab_size=vocab or raw["vocab_size"]))
    tensors = random_tensors(config, 7, torch.bfloat16, "unit")
    plain = {name: tensor.float() for name, tensor in tensors.items()}
    prompts = {name: tokens_for(config.vocab_size, length, seed)
               for name, length, seed in (("long", 2 * 300 + 37 + 8, 1), ("short", 45 + 8, 2), ("third", 300 + 8, 3))}
    engine = Engine(config=config, tensors=tensors, dtype="bfloat16", kv_cache_capacity_tokens=1536, max_active_sequences=3)
    rows = {name: [] for name in prompts}
    for name in prompts:
        engine.add_request(name)
    # steps of one size (300 tokens, last place wanted) three times: launched, captured and replayed, replayed
    for name, first in (("long", 0), ("third", 0), ("long", 300)):
        rows[name].append(engine.step([Lane(name, prompts[name][first:first + 300], [299])]).cpu())
    assert engine.graphs.counts["bucket_captures"] == 1 and engine.graphs.counts["bucket_replays"] == 2
    mixed = engine.step([Lane("long", prompts["long"][600:637], [36]), Lane("short", prompts["short"][:45], [0, 44])]).cpu()
    rows["long"].append(mixed[:1])
    rows["short"].append(mixed[1:])
    rows["long"].append(engine.step([Lane("long", prompts["long"][637:638], [0])]).cpu())
    for turn in range(7):
        lanes = [Lane("long", [prompts["long"][638 + turn]], [0]), Lane("short", [prompts["short"][45 + turn]], [0]),
                 Lane("third", [prompts["third"][300 + turn]], [0])]
        out = engine.step(lanes).cpu()
        for row, name in enumerate(("long", "short", "third")):
            rows[name].append(out[row:row + 1])
    places = {"long": [299, 599, 636] + list(range(637, 645)), "short": [0, 44] + list(range(45, 52)),
              "third": [299] + list(range(300, 307))}
    for name, tokens in prompts.items():
        want = plain_impl.falcon_h1_logits(config.to_dict(), plain, tokens[:places[name][-1] + 1])[places[name]].numpy()
        got = torch.cat(rows[name]).numpy()
        assert got.shape == want.shape, name
        assert bfloat16_close(got, want), f"{name}: {np.abs(got - want).max():.3e} of {np.abs(want).max():.2f}"


@pytest.mark.parametrize("name", ["A", "B"])
def test_float32_logits_are_the_same_bits_however_the_tokens_are_cut(tmp_path, name):
    """Every float32 kernel sums in an order that the sizes alone fix, so a position's logits are
    bit for bit the same whole, in portions, token by token and beside another request."""
    from macllm_infer_amd import Engine, Lane
    folder = tiny_configs.make_model_dir(name, tmp_path)
    cfg, _ = plain_impl.load_model_dir(folder)
    tokens, other = tokens_for(cfg["vocab_size"], 47, 31), tokens_for(cfg["vocab_size"], 29, 32)
    engine = Engine(folder, dtype="float32", kv_cache_block_tokens=8, kv_cache_capacity_tokens=256, max_active_sequences=3)
    engine.add_request("whole")
    whole = engine.step([Lane("whole", tokens, list(range(47)))]).cpu()
    engine.finish("whole")
    for cuts in ([5] * 9 + [2], [1] * 47, [30, 16, 1]):
        engine.add_request("cut")
        engine.add_request("other")
        rows, first, fed = [], 0, 0
        for count in cuts:
            lanes = [Lane("cut", tokens[first:first + count], list(range(count)))]
            if fed < len(other):                                   # a neighbour whose lane changes from step to step
                take = min(1 + first % 4, len(other) - fed)
                lanes.insert(0, Lane("other", other[fed:fed + take], [take - 1]))
                fed += take
            rows.append(engine.step(lanes).cpu()[len(lanes) - 1:])
            first += count
        assert torch.equal(torch.cat(rows), whole), f"cuts {cuts[:3]}..."
        engine.finish("cut")
        engine.finish("other")
