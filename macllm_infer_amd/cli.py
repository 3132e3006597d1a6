"""Command line: ``run`` (generate from token ids), ``inspect`` (sizes of a model folder)
and ``random-weights`` (write a model folder from a configuration and a seed).

Option names, meanings and defaults follow the reference's ``macllm run``
(src/main.rs:114-215); where it takes text (``--prompt``) this takes token ids
(``--tokens``), as its serving input ``TokenIds`` does (src/engine.rs:2976-3002).
"""
from __future__ import annotations

import argparse
import json
import sys
from typing import List

import torch


def _token_list(text: str) -> List[int]:
    try:
        return [int(item) for item in text.replace(",", " ").split()]
    except ValueError as error:
        raise argparse.ArgumentTypeError(f"token ids must be integers: {error}")


def _runtime_arguments(parser: argparse.ArgumentParser) -> None:
    parser.add_argument("-m", "--model", required=True, help="folder with config.json and model.safetensors")
    parser.add_argument("--device", default="hip", choices=["hip"], help="backend (one MI355X)")
    parser.add_argument("--dtype", default="bf16", choices=["f32", "bf16", "float32", "bfloat16"],
                        help="activation dtype; f32 runs every product in true 32-bit")
    parser.add_argument("--fixed-paths", action="store_true",
                        help="no timing of alternative kernels when the model is built: the same kernels, and the "
                             "same bits in bfloat16, in every process (slower on large models)")
    parser.add_argument("--kv-cache-block-tokens", type=int, default=16, help="tokens per cache page")
    parser.add_argument("--kv-cache-capacity-tokens", type=int, default=None,
                        help="token capacity of the cache shared by all requests (default: one model context)")


def _run(args) -> int:
    from .engine.generate import LLM
    from .engine.scheduler import EngineConfig
    from .sampling.params import SamplingParams
    prompts: List[List[int]] = list(args.tokens or [])
    if args.tokens_file:
        with open(args.tokens_file) as handle:
            prompts += [_token_list(line) for line in handle if line.strip()]
    if not prompts:
        print("error: give --tokens or --tokens-file", file=sys.stderr)
        return 2
    budget = max(args.scheduler_token_budget, 1)
    quantum = min(args.prefill_token_quantum or budget, budget)
    llm = LLM(args.model, dtype=args.dtype, kv_cache_block_tokens=args.kv_cache_block_tokens,
              kv_cache_capacity_tokens=args.kv_cache_capacity_tokens, measured_paths=not args.fixed_paths,
              engine_config=EngineConfig(max_active_sequences=args.max_active_sequences,
                                         scheduler_token_budget=budget, prefill_token_quantum=quantum))
    params = SamplingParams(max_new_tokens=args.max_new_tokens, temperature=args.temperature, top_k=args.top_k,
                            top_p=args.top_p, repetition_penalty=args.repetition_penalty,
                            presence_penalty=args.presence_penalty, frequency_penalty=args.frequency_penalty,
                            seed=args.seed, ignore_eos=args.ignore_eos)
    results = llm.generate(prompts, params)
    for index, result in enumerate(results):
        print(" ".join(str(token) for token in result.token_ids))
        # the reference's metrics line (src/main.rs:1396-1410), without its prefix-cache figures
        number = lambda value, form: "-" if value is None else format(value, form)
        print(f"[request {index}] prompt={result.prompt_tokens} output={result.generated_tokens} "
              f"finish={result.finish_reason} "
              f"TTFT={number(None if result.time_to_first_token is None else result.time_to_first_token * 1e3, '.1f')}ms "
              f"prefill={number(result.prefill_tokens_per_second, '.1f')} tok/s "
              f"model-decode={number(result.decode_tokens_per_second, '.1f')} tok/s "
              f"e2e-output={number(result.output_tokens_per_second, '.1f')} tok/s total={result.total_time * 1e3:.1f}ms",
              file=sys.stderr)
    return 0


def _inspect(args) -> int:
    from .config.registry import load_config
    from .engine.model import DecoderModel
    config = load_config(args.model)
    spec = config.to_model_spec()
    parameters = 0
    for expect in DecoderModel.expected_tensors(spec):
        count = 1
        for dim in expect.shapes[0]:
            count *= dim
        parameters += count
    report = {"architecture": spec.architecture, "layers": len(spec.layers), "hidden_size": spec.hidden_size,
              "vocab_size": spec.vocab_size, "max_context": spec.max_context, "parameters": parameters,
              "tied_embeddings": spec.tied_embeddings}
    if hasattr(config, "kv_bytes_per_token"):
        report["kv_bytes_per_token_bf16"] = config.kv_bytes_per_token(2)
        report["kv_bytes_per_token_f32"] = config.kv_bytes_per_token(4)
        report["fixed_state_bytes_per_request_bf16"] = config.fixed_state_bytes(2)
        report["fixed_state_bytes_per_request_f32"] = config.fixed_state_bytes(4)
    print(json.dumps(report, indent=1))
    return 0


def _random_weights(args) -> int:
    from .config.registry import config_from_dict
    from .weights.random_init import write_random_model
    with open(args.config) as handle:
        config = config_from_dict(json.load(handle))
    dtype = torch.float32 if args.dtype in ("f32", "float32") else torch.bfloat16
    folder = write_random_model(config, args.seed, args.out, dtype, args.init)
    print(folder)
    return 0


def main(argv=None) -> int:
    parser = argparse.ArgumentParser(prog="macllm_infer_amd", description=__doc__.split("\n\n")[0])
    commands = parser.add_subparsers(dest="command", required=True)

    run = commands.add_parser("run", help="generate from token ids")
    _runtime_arguments(run)
    run.add_argument("--tokens", type=_token_list, action="append",
                     help='prompt token ids, e.g. "1,2,3"; repeat the flag for a batch')
    run.add_argument("--tokens-file", help="one prompt per line, token ids separated by spaces or commas")
    run.add_argument("--max-new-tokens", type=int, default=128)
    run.add_argument("--temperature", type=float, default=0.7, help="0 = greedy argmax")
    run.add_argument("--top-k", type=int, default=20)
    run.add_argument("--top-p", type=float, default=0.8)
    run.add_argument("--repetition-penalty", type=float, default=1.1)
    run.add_argument("--presence-penalty", type=float, default=0.0)
    run.add_argument("--frequency-penalty", type=float, default=0.0)
    run.add_argument("--seed", type=int, default=42)
    run.add_argument("--ignore-eos", action="store_true", help="do not stop at the end-of-sequence token")
    run.add_argument("--prefill-token-quantum", type=int, default=None,
                     help="most prompt tokens of one request per step (default: the whole budget)")
    run.add_argument("--scheduler-token-budget", type=int, default=4096, help="most tokens per step")
    run.add_argument("--max-active-sequences", type=int, default=64)
    run.set_defaults(handler=_run)

    inspect = commands.add_parser("inspect", help="print a model folder's geometry")
    inspect.add_argument("-m", "--model", required=True)
    inspect.set_defaults(handler=_inspect)

    random_weights = commands.add_parser("random-weights", help="write a model folder with random weights")
    random_weights.add_argument("--config", required=True, help="a config.json")
    random_weights.add_argument("--seed", type=int, default=0)
    random_weights.add_argument("--out", required=True)
    random_weights.add_argument("--dtype", default="bf16", choices=["f32", "bf16", "float32", "bfloat16"])
    random_weights.add_argument("--init", default="baseline", choices=["baseline", "unit"])
    random_weights.set_defaults(handler=_random_weights)

    args = parser.parse_args(argv)
    return args.handler(args)


if __name__ == "__main__":
    sys.exit(main())
