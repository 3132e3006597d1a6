"""Decode and prefill throughput of a Falcon-H1 0.5B-shaped model with random weights on one
MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--dtype bf16|f32] [--layers L]
    python bench.py --workload serving [--shape 0.5b|7b|34b]
    python bench.py --microbench

One JSON line: ``value`` = decoded tokens a second at batch 8 with every request at a
2,048-token context (a step = one decode step of the whole batch: model, greedy sampling,
tokens fed back); ``prefill`` = one 2,048-token prompt in one step (replayed from its captured
graph; ``prefill_uncaptured_ms`` = the same step launched kernel by kernel, as a shape is when it
comes for the first time); ``roofline`` = the bytes the decode step has to read (every weight it
uses once, and the cache and state of the live requests; ``bytes`` gives them and what the step
writes) over its time, against 8 TB/s; ``points`` = decode at batch 1 and 64, and at longer contexts (batch 8
at 8,192 and 32,768 tokens, batch 64 at 8,192, from an engine of the same layers that allows such contexts;
``points_frac`` = their fractions of 8 TB/s on the bytes they have to read); ``prefill_f32`` = the same prompt
step through the true 32-bit path (the headline shape only), against the float32 matrix cores' peak;
``step_ms`` = mean,
median and 95th percentile of the timed steps (the reference reports the same three:
src/benchmark/stats.rs:10-16); ``choices`` = what the build-time measurements chose for each
projection of a layer at up to 16 / 32 / 64 rows (L = library, S = skinny kernel, a digit = slabs
over K; then the skinny kernel's tiles of 16 features).

``--microbench`` prints what this GPU's memory delivers to a plain streaming read and a plain
read-modify-write (the ceilings that the decode kernels can be held against).

``--workload serving`` runs whole requests through the scheduler and the sampler instead
(``LLM.generate``): for the 7B shape (and the 0.5B one) 64 requests with prompt lengths uniform in
[128, 4096] and 256 greedy tokens each, prompts cut into portions of 2,048 tokens; for the 34B
shape 8 prompts of 8,192 tokens and 128 greedy tokens each.  Its line reports prompt and generated
tokens a second over the whole run and the spread of the rounds' times.
"""
import argparse
import json
import sys
import time

from macllm_infer_amd.utils.costs import PEAK_FLOPS, PEAK_HBM_BYTES, decode_step_costs, prefill_costs, total

PEAK_HBM_GBS = PEAK_HBM_BYTES / 1e9

# Falcon-H1-0.5B-shaped: the layer sizes of the benchmark configuration
SHAPE = dict(
    architectures=["FalconH1ForCausalLM"], model_type="falcon_h1", hidden_size=1024, num_hidden_layers=36,
    num_attention_heads=8, num_key_value_heads=2, head_dim=64, intermediate_size=2048, vocab_size=32784,
    max_position_embeddings=4096, rms_norm_eps=1e-5, rope_theta=1e11, mamba_n_heads=24, mamba_d_head=64,
    mamba_d_ssm=1536, mamba_d_state=128, mamba_n_groups=1, mamba_d_conv=4, mamba_chunk_size=128,
    mamba_conv_bias=True, mamba_proj_bias=False, mamba_rms_norm=False, attention_bias=False, mlp_bias=False,
    tie_word_embeddings=True)
# further shapes of the family for measurements beside the headline one (--shape)
SHAPES = {
    "0.5b": SHAPE,
    "7b": dict(SHAPE, hidden_size=3072, num_hidden_layers=44, num_attention_heads=12, num_key_value_heads=2,
               head_dim=128, intermediate_size=12288, vocab_size=130049, mamba_n_heads=24, mamba_d_head=128,
               mamba_d_ssm=3072, mamba_d_state=256, mamba_n_groups=1, tie_word_embeddings=False),
    "34b": dict(SHAPE, hidden_size=5120, num_hidden_layers=72, num_attention_heads=20, num_key_value_heads=4,
                head_dim=128, intermediate_size=21504, vocab_size=261120, mamba_n_heads=32, mamba_d_head=128,
                mamba_d_ssm=4096, mamba_d_state=256, mamba_n_groups=2, tie_word_embeddings=False),
}
CONTEXT = 2048
PREFILL_TOKENS = 2048
LONG_POINTS = ((8, 8192), (8, 32768), (64, 8192))      # (batch, context) of the decode points beyond the headline context
# whole-request workloads (--workload serving): requests, prompt lengths (lowest, highest), new tokens
SERVING = {"0.5b": (64, 128, 4096, 256), "7b": (64, 128, 4096, 256), "34b": (8, 8192, 8192, 128)}
SERVING_PORTION = 2048


def serving(args, shape) -> int:
    """Whole requests through the scheduler: admission, portions of prompts beside decoded tokens,
    sampling, finishing."""
    import torch
    from macllm_infer_amd import LLM, Engine, EngineConfig, SamplingParams
    from macllm_infer_amd.config import FalconH1Config
    from macllm_infer_amd.weights.random_init import random_tensors

    requests, shortest, longest, new_tokens = SERVING[args.shape]
    layers = args.layers or shape["num_hidden_layers"]
    raw = dict(shape, num_hidden_layers=layers, max_position_embeddings=longest + new_tokens)
    config = FalconH1Config.from_dict(raw)
    storage = torch.bfloat16 if args.dtype == "bf16" else torch.float32
    tensors = random_tensors(config, 0, storage, "baseline", device="cpu" if args.shape == "0.5b" else "cuda:0")
    generator = torch.Generator().manual_seed(0)
    lengths = torch.randint(shortest, longest + 1, (requests,), generator=generator).tolist()
    prompts = [torch.randint(0, config.vocab_size, (length,), generator=generator).tolist() for length in lengths]
    capacity = sum(-(-(length + new_tokens) // 64) * 64 for length in lengths)
    engine = Engine(config=config, tensors=tensors, dtype="bfloat16" if args.dtype == "bf16" else "float32",
                    kv_cache_block_tokens=args.page_tokens, kv_cache_capacity_tokens=capacity,
                    max_active_sequences=requests, measured_paths=not args.fixed_paths)
    del tensors
    llm = LLM(engine, engine_config=EngineConfig(max_active_sequences=requests, prefill_token_quantum=SERVING_PORTION,
                                                 scheduler_token_budget=SERVING_PORTION + requests))
    params = SamplingParams(max_new_tokens=new_tokens, temperature=0.0, top_k=0, top_p=1.0, repetition_penalty=1.0,
                            ignore_eos=True)
    runs = []
    for repeat in range(2):                      # the first run captures the graphs of the repeating shapes
        round_times = []
        torch.cuda.synchronize()
        started = time.perf_counter()
        results = llm.generate(prompts, params, on_round=round_times.append)
        torch.cuda.synchronize()
        runs.append((time.perf_counter() - started, results, sorted(round_times)))
    seconds, results, round_times = runs[-1]
    generated = sum(result.generated_tokens for result in results)
    assert all(result.finish_reason == "length" for result in results), "a request did not run to its length"
    first = sorted(result.time_to_first_token for result in results)
    pick = lambda values, fraction: values[min(len(values) - 1, int(fraction * len(values)))]
    print(json.dumps({
        "metric": "generated tok/s over whole requests (scheduler, portions of prompts beside decoded tokens)",
        "value": round(generated / seconds, 1), "unit": "tokens/s", "n_gpus": 1, "higher_is_better": True,
        "dtype": args.dtype, "data": "synthetic", "seconds": round(seconds, 3), "first_run_seconds": round(runs[0][0], 3),
        "prompt_tokens": sum(lengths), "generated_tokens": generated,
        "all_tokens_per_second": round((sum(lengths) + generated) / seconds, 1),
        "rounds": len(round_times), "round_ms": {"mean": round(1e3 * sum(round_times) / len(round_times), 3),
                                                 "p50": round(1e3 * pick(round_times, 0.5), 3),
                                                 "p95": round(1e3 * pick(round_times, 0.95), 3)},
        "first_token_s": {"p50": round(pick(first, 0.5), 3), "p95": round(pick(first, 0.95), 3)},
        "config": {"model": f"falcon-h1-{args.shape}-shaped, random weights", "layers": layers,
                   "layers_of_configuration": shape["num_hidden_layers"], "requests": requests,
                   "prompt_tokens_lowest": shortest, "prompt_tokens_highest": longest, "new_tokens": new_tokens,
                   "portion": SERVING_PORTION, "page_tokens": args.page_tokens, "sampling": "greedy"}}))
    return 0


def microbench() -> int:
    """Streaming read and read-modify-write bandwidth of this GPU, with this package's own kernels."""
    import torch
    from macllm_infer_amd.kernels import ops
    ops.require_gpu("cuda:0")
    results = {}
    sink = torch.zeros(4, dtype=torch.int32, device="cuda:0")
    for name, megabytes in (("read", 4096), ("rmw", 2048)):
        data = torch.ones(megabytes * (1 << 20) // 4, dtype=torch.float32, device="cuda:0")
        best = 0.0
        for blocks in (1024, 2048, 4096, 8192, 16384):
            run = (lambda: ops.stream_read(data, sink, blocks)) if name == "read" else (lambda: ops.stream_rmw(data, 1.0, blocks))
            for _ in range(2):
                run()
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            for _ in range(5):
                run()
            end.record()
            end.synchronize()
            seconds = start.elapsed_time(end) * 1e-3 / 5
            moved = data.numel() * 4 * (1 if name == "read" else 2)
            best = max(best, moved / seconds / 1e9)
        results[name] = best
        del data
    print(json.dumps({"metric": "streaming memory bandwidth of this GPU (16 bytes a lane a load, float32)",
                      "read_gbs": round(results["read"], 1), "read_modify_write_gbs": round(results["rmw"], 1),
                      "unit": "GB/s", "published_peak_gbs": PEAK_HBM_GBS,
                      "read_frac": round(results["read"] / PEAK_HBM_GBS, 4),
                      "read_modify_write_frac": round(results["rmw"] / PEAK_HBM_GBS, 4)}))
    return 0


def choices_of(engine) -> dict:
    """What the first layer's fast path chose for steps of up to 4 / 8 / 16 / 32 / 48 / 64 rows, as short strings
    (S: the skinny kernel, L: the library, a number: that many slabs over K; empty when the layer has none)."""
    choices = dict(engine.path_choices())
    if getattr(engine, "halves_share", None) is not None:     # a step of more than 64 single tokens came: two halves at once over one graph
        choices["halves_over_one_graph"] = round(engine.halves_share, 3)
    return choices


def main() -> int:
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=64)
    parser.add_argument("--warmup", type=int, default=8)
    parser.add_argument("--dtype", default="bf16", choices=["bf16", "f32"])
    parser.add_argument("--shape", default="0.5b", choices=sorted(SHAPES),
                        help="layer sizes: the headline Falcon-H1-0.5B shape, or the 7B / 34B shapes")
    parser.add_argument("--layers", type=int, default=None,
                        help="fewer layers than the configuration has (both numbers are reported)")
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--page-tokens", type=int, default=16)
    parser.add_argument("--fixed-paths", action="store_true",
                        help="the layers' fixed rules instead of the build-time clock (as `run --fixed-paths`): the same "
                             "kernels in every process, also under a profiler, whose overhead the clock would measure")
    parser.add_argument("--skip-points", action="store_true", help="only the headline batch")
    parser.add_argument("--skip-long-points", action="store_true", help="no decode points at longer contexts")
    parser.add_argument("--prefill-only", action="store_true",
                        help="only the 2,048-token prefill (for profiles; the line then reports prefill tokens/s)")
    parser.add_argument("--workload", default="steps", choices=["steps", "serving"],
                        help="steps: the headline decode and prefill steps; serving: whole requests through the scheduler")
    parser.add_argument("--microbench", action="store_true",
                        help="only this GPU's streaming read and read-modify-write bandwidth")
    parser.add_argument("--write-config", default=None, metavar="PATH",
                        help="write the config.json of --shape / --layers there and exit (what "
                             "utils.kernel_trace --config reads)")
    args = parser.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this engine")
        return 2
    if args.microbench:
        return microbench()
    if args.write_config:
        shape = SHAPES[args.shape]
        with open(args.write_config, "w") as handle:
            json.dump(dict(shape, num_hidden_layers=args.layers or shape["num_hidden_layers"]), handle)
        return 0
    if args.workload == "serving":
        return serving(args, SHAPES[args.shape])

    import torch
    from macllm_infer_amd import Engine, Lane
    from macllm_infer_amd.config import FalconH1Config
    from macllm_infer_amd.sampling import GREEDY, Sampler, SamplerRow
    from macllm_infer_amd.weights.random_init import random_tensors

    shape = SHAPES[args.shape]
    raw = dict(shape, num_hidden_layers=args.layers or shape["num_hidden_layers"])
    config = FalconH1Config.from_dict(raw)
    storage = torch.bfloat16 if args.dtype == "bf16" else torch.float32
    element = 2 if args.dtype == "bf16" else 4
    # the 0.5B shape is drawn on the CPU like every test model; the large shapes on the GPU (minutes otherwise)
    tensors = random_tensors(config, 0, storage, "baseline", device="cpu" if args.shape == "0.5b" else "cuda:0")
    batches = [args.batch] if args.skip_points else sorted({1, args.batch, 64})
    if args.prefill_only:
        batches = []
    largest = max(batches, default=1)
    total_steps = args.steps + args.warmup
    per_request = -(-(CONTEXT + total_steps + 1) // 64) * 64
    engine = Engine(config=config, tensors=tensors, dtype="bfloat16" if args.dtype == "bf16" else "float32",
                    kv_cache_block_tokens=args.page_tokens,
                    kv_cache_capacity_tokens=per_request * largest + PREFILL_TOKENS + 64,
                    max_active_sequences=largest + 1, measured_paths=not args.fixed_paths)
    sampler = Sampler(engine.vocab_size, engine.device)
    generator = torch.Generator().manual_seed(0)
    vocab = config.vocab_size

    def synchronize():
        torch.cuda.synchronize()

    # ---------------------------------------------------------------- prefill: one 2,048-token prompt
    def prefill_step(engine=engine):
        prompt = torch.randint(0, vocab, (PREFILL_TOKENS,), generator=generator).tolist()
        engine.add_request("prefill")
        synchronize()
        started = time.perf_counter()
        engine.step([Lane("prefill", prompt, [PREFILL_TOKENS - 1])])
        synchronize()
        seconds = time.perf_counter() - started
        engine.finish("prefill")
        return seconds

    graphs, engine.graphs = engine.graphs, None         # launched kernel by kernel: what a capacity costs the first time
    uncaptured_seconds = min([prefill_step() for _ in range(3)][1:])
    engine.graphs = graphs
    prefill_times = [prefill_step() for _ in range(6)]  # the step's graph is captured when its capacity comes again
    prefill_seconds = sorted(prefill_times[3:])[1]      # the median of the last three

    d, L = config.hidden_size, config.num_hidden_layers
    prefill_flops = total(prefill_costs(engine.spec, PREFILL_TOKENS, element)).flops

    # ---------------------------------------------------------------- decode at each batch size
    def decode_point(engine, sampler, batch, context_tokens):
        names = [f"b{batch}_{index}" for index in range(batch)]
        for name in names:
            engine.add_request(name)
            prompt = torch.randint(0, vocab, (context_tokens,), generator=generator).tolist()
            for first in range(0, context_tokens, PREFILL_TOKENS):          # long contexts in portions
                engine.step([Lane(name, prompt[first:first + PREFILL_TOKENS], [])])
        tokens = torch.randint(0, vocab, (batch,), generator=generator).tolist()
        rows = [SamplerRow(GREEDY, (), ()) for _ in names]

        # a step is queued before the host has read the tokens of the step before it (they are fed on the
        # device), as the scheduler does it; the host reads them while the GPU works
        def decode_step(before):
            if before is None:
                lanes = [Lane(name, [token], [0]) for name, token in zip(names, tokens)]
            else:
                lanes = [Lane(name, [0], [0], feed=(before.device, row)) for row, name in enumerate(names)]
            return sampler.sample_async(engine.step(lanes), rows)

        on_their_way = decode_step(None)
        for _ in range(args.warmup):
            newer = decode_step(on_their_way)
            on_their_way.wait()
            on_their_way = newer
        synchronize()
        step_times = []
        started = time.perf_counter()
        for _ in range(args.steps):                   # a step's time: from one step's tokens on the host to the next's
            tick = time.perf_counter()
            newer = decode_step(on_their_way)
            on_their_way.wait()
            on_their_way = newer
            step_times.append(time.perf_counter() - tick)
        synchronize()
        seconds = time.perf_counter() - started
        for name in names:
            engine.finish(name)
        step_seconds = seconds / args.steps
        context = context_tokens + args.warmup + args.steps / 2.0
        moved = total(decode_step_costs(engine.spec, batch, context, element))
        step_times.sort()
        pick = lambda fraction: step_times[min(len(step_times) - 1, int(fraction * len(step_times)))]
        return dict(tokens_per_second=batch / step_seconds, ms=step_seconds * 1e3,
                    gbs=moved.read / step_seconds / 1e9, read_mb=moved.read / 1e6, written_mb=moved.written / 1e6,
                    step_ms={"mean": round(1e3 * sum(step_times) / len(step_times), 4),
                             "p50": round(1e3 * pick(0.5), 4), "p95": round(1e3 * pick(0.95), 4)})

    results = {batch: decode_point(engine, sampler, batch, CONTEXT) for batch in batches}

    # ---------------------------------------------------------------- the same at longer contexts
    long_points = {}
    if not (args.skip_points or args.skip_long_points or args.prefill_only):
        choices = choices_of(engine)
        del engine, sampler, graphs
        torch.cuda.empty_cache()
        most = max(context for _, context in LONG_POINTS)
        long_config = FalconH1Config.from_dict(dict(raw, max_position_embeddings=most + 2 * per_request))
        room = max(batch * (-(-(context + total_steps + 1) // 64) * 64) for batch, context in LONG_POINTS)
        long_engine = Engine(config=long_config, tensors=tensors, dtype="bfloat16" if args.dtype == "bf16" else "float32",
                             kv_cache_block_tokens=args.page_tokens, kv_cache_capacity_tokens=room + 64,
                             max_active_sequences=max(batch for batch, _ in LONG_POINTS) + 1)
        long_sampler = Sampler(long_engine.vocab_size, long_engine.device)
        for batch, context in LONG_POINTS:
            long_points[(batch, context)] = decode_point(long_engine, long_sampler, batch, context)
    else:
        choices = choices_of(engine)
    # the same prefill through the true 32-bit path (the small shape only: the weights once more in float32)
    prefill_f32 = None
    if args.dtype == "bf16" and args.shape == "0.5b" and not (args.skip_points or args.skip_long_points or args.prefill_only):
        wide = {name: tensor.to(torch.float32) for name, tensor in tensors.items()}
        wide_engine = Engine(config=config, tensors=wide, dtype="float32", kv_cache_block_tokens=args.page_tokens,
                             kv_cache_capacity_tokens=PREFILL_TOKENS + 64, max_active_sequences=1)
        del wide
        times = [prefill_step(wide_engine) for _ in range(6)]
        seconds = sorted(times[3:])[1]
        flops = total(prefill_costs(wide_engine.spec, PREFILL_TOKENS, 4)).flops
        prefill_f32 = {"value": round(PREFILL_TOKENS / seconds, 1), "tokens": PREFILL_TOKENS, "ms": round(seconds * 1e3, 3),
                       "frac": round(flops / seconds / PEAK_FLOPS["f32"], 5)}
        del wide_engine
    del tensors

    if args.prefill_only:
        print(json.dumps({"metric": "prefill tok/s at 2,048 tokens", "value": round(PREFILL_TOKENS / prefill_seconds, 1),
                          "unit": "tokens/s", "n_gpus": 1, "ms": round(prefill_seconds * 1e3, 3), "dtype": args.dtype,
                          "frac": round(prefill_flops / prefill_seconds / PEAK_FLOPS[args.dtype], 5),
                          "higher_is_better": True, "data": "synthetic", "config": {"layers": L}}))
        return 0
    headline = results[args.batch]
    record = {
        "metric": "decode tok/s at batch 8 (2,048-token context); prefill tok/s at 2,048 tokens",
        "value": round(headline["tokens_per_second"], 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(headline["ms"], 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": args.dtype, "data": "synthetic",
        "config": {"model": f"falcon-h1-{args.shape}-shaped, random weights", "layers": L,
                   "layers_of_configuration": shape["num_hidden_layers"], "hidden": d,
                   "heads": config.num_attention_heads, "kv_heads": config.num_key_value_heads,
                   "head_dim": config.head_dim, "intermediate": config.intermediate_size,
                   "mamba_heads": config.mamba_n_heads, "mamba_head_dim": config.mamba_d_head,
                   "mamba_state": config.mamba_d_state, "mamba_groups": config.mamba_n_groups,
                   "mamba_conv": config.mamba_d_conv, "mamba_chunk": config.mamba_chunk_size, "vocab": vocab,
                   "tied_embeddings": config.tie_word_embeddings, "global_batch": args.batch, "seq_len": CONTEXT,
                   "page_tokens": args.page_tokens, "parallelism": "single GPU"},
        "prefill": {"value": round(PREFILL_TOKENS / prefill_seconds, 1), "tokens": PREFILL_TOKENS,
                    "ms": round(prefill_seconds * 1e3, 3),
                    "frac": round(prefill_flops / prefill_seconds / PEAK_FLOPS[args.dtype], 5)},
        "roofline": {"bound": "hbm", "achieved": round(headline["gbs"], 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(headline["gbs"] / PEAK_HBM_GBS, 5)},
        "points": dict({f"decode_b{batch}": round(result["tokens_per_second"], 1) for batch, result in results.items()
                        if batch != args.batch},
                       **{f"decode_b{batch}_ctx{context}": round(result["tokens_per_second"], 1)
                          for (batch, context), result in long_points.items()}),
        "points_frac": dict({f"decode_b{batch}": round(result["gbs"] / PEAK_HBM_GBS, 5) for batch, result in results.items()
                             if batch != args.batch},
                            **{f"decode_b{batch}_ctx{context}": round(result["gbs"] / PEAK_HBM_GBS, 5)
                               for (batch, context), result in long_points.items()}),
        "step_ms": headline["step_ms"],
        "bytes": {"read_mb": round(headline["read_mb"], 1), "written_mb": round(headline["written_mb"], 1)},
        "prefill_uncaptured_ms": round(uncaptured_seconds * 1e3, 3),
        "choices": choices,
    }
    if prefill_f32 is not None:
        record["prefill_f32"] = prefill_f32
    print(json.dumps(record))
    return 0


if __name__ == "__main__":
    sys.exit(main())
