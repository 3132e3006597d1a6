"""Trace replay through bin/trace_run, in float32 and in bfloat16, for both tiny models:
each request alone and whole; most of it in one step and the last 32 tokens one by one; in
portions of changing size; mixed with other requests in a pool so small that pages and
slots are used again; long decoding; the first tokens of a sequence.  Every logit row is
compared with the plain whole-sequence implementation."""
import numpy as np
import pytest
import torch

import plain_impl
import tiny_configs
import traces
from gates import FLOAT32_TOLERANCE, bfloat16_close

pytestmark = pytest.mark.gpu


def requests_for(cfg, lengths, seed):
    generator = torch.Generator().manual_seed(seed)
    return {f"r{seed}_{index}": torch.randint(0, cfg["vocab_size"], (length,), generator=generator).tolist()
            for index, length in enumerate(lengths)}


def check(steps, out_dir, cfg, tensors, requests, dtype):
    lengths = {name: len(tokens) for name, tokens in requests.items()}
    got = traces.collect(steps, out_dir, cfg["vocab_size"], lengths)
    for name, tokens in requests.items():
        want = plain_impl.falcon_h1_logits(cfg, tensors, tokens).numpy()
        assert not np.isnan(got[name]).any(), f"{name}: a wanted row was not written"
        if dtype == "float32":
            error = np.abs(got[name] - want).max(axis=1)
            worst = int(error.argmax())
            assert error.max() <= FLOAT32_TOLERANCE, \
                f"{name}: max error {error.max():.3e} at position {worst} of {len(tokens)}"
        else:
            assert bfloat16_close(got[name], want), \
                f"{name}: max error {np.abs(got[name] - want).max():.3e} of scale {np.abs(want).max():.2f}"


@pytest.fixture(scope="module", params=[("A", "float32"), ("B", "float32"), ("A", "bfloat16"), ("B", "bfloat16"),
                                        ("C", "float32"), ("C", "bfloat16")],
                ids=lambda p: f"{p[0]}-{p[1]}")
def model(request, tmp_path_factory):
    name, dtype = request.param
    folder = tmp_path_factory.mktemp(f"model_{name}_{dtype}")
    tiny_configs.make_model_dir(name, folder, torch.float32 if dtype == "float32" else torch.bfloat16)
    cfg, tensors = plain_impl.load_model_dir(str(folder))
    return name, dtype, str(folder), cfg, tensors


def test_whole_tail_decoded_and_portions(model, tmp_path):
    name, dtype, folder, cfg, tensors = model
    requests = requests_for(cfg, [5, 17, 33, 63, 64, 65, 130], seed=1)
    families = {}
    steps = []
    for label, family in (("whole", traces.whole), ("tail", traces.tail_decoded), ("portions", traces.portions)):
        renamed = {f"{label}_{key}": tokens for key, tokens in requests.items()}
        families.update(renamed)
        steps += family(renamed)
    traces.number(steps)
    traces.replay(folder, dtype, steps, max_tokens=256, out_dir=tmp_path)
    check(steps, tmp_path, cfg, tensors, families, dtype)


def test_mixed_requests_in_a_small_pool(model, tmp_path):
    """Nine requests, four live at a time, in a pool that holds the peak and no more: pages and
    slots of finished requests are used again by later ones."""
    name, dtype, folder, cfg, tensors = model
    requests = requests_for(cfg, [50, 97, 64, 33, 120, 71, 16, 128, 45], seed=2)
    steps = traces.number(traces.mixed(requests, seed=7))
    peak = traces.peak_tokens(steps)
    assert peak < sum(len(tokens) for tokens in requests.values())        # pages have to be reused
    assert any(len(step["entries"]) == 4 for step in steps)
    assert any(len({len(entry["tokens"]) for entry in step["entries"]}) > 1 and
               any(len(entry["tokens"]) == 1 for entry in step["entries"]) for step in steps)
    traces.replay(folder, dtype, steps, max_tokens=peak, out_dir=tmp_path)
    check(steps, tmp_path, cfg, tensors, requests, dtype)


def test_long_decoding_and_first_tokens(model, tmp_path):
    """A prompt of three tokens and 300 tokens decoded one by one (many pages, the conv tail
    and the state carried across hundreds of steps), and sequences of one and two tokens."""
    name, dtype, folder, cfg, tensors = model
    requests = requests_for(cfg, [303, 1, 2], seed=3)
    names = list(requests)
    steps = traces.tail_decoded({names[0]: requests[names[0]]}, tail=300)
    steps += traces.whole({names[1]: requests[names[1]]})
    steps += traces.tail_decoded({names[2]: requests[names[2]]}, tail=1)
    traces.number(steps)
    traces.replay(folder, dtype, steps, max_tokens=320, out_dir=tmp_path)
    check(steps, tmp_path, cfg, tensors, requests, dtype)


def test_nothing_wanted_writes_no_file_and_larger_pages(model, tmp_path):
    name, dtype, folder, cfg, tensors = model
    requests = requests_for(cfg, [70], seed=4)
    (key, tokens), = requests.items()
    steps = [{"step": 0, "entries": [{"id": key, "tokens": tokens[:40], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": key, "tokens": tokens[40:], "want": [0, 29]}], "end": [key]}]
    traces.replay(folder, dtype, steps, max_tokens=128, out_dir=tmp_path, extra=["--page-tokens", "64"])
    assert not (tmp_path / "0.f32").exists()
    rows = np.fromfile(tmp_path / "1.f32", dtype="<f4").reshape(2, cfg["vocab_size"])
    want = plain_impl.falcon_h1_logits(cfg, tensors, tokens).numpy()[[40, 69]]
    assert np.abs(rows - want).max() <= FLOAT32_TOLERANCE if dtype == "float32" else bfloat16_close(rows, want)


def test_decoded_tokens_whose_logits_nobody_wants(model, tmp_path):
    """Three requests decode in turn, one request a step, and ask for no logits for forty steps in a row:
    the replay program answers each step without waiting for the GPU, so steps of one shape queue one
    behind the other.  The logits of the tokens after that must be those of the whole sequences."""
    name, dtype, folder, cfg, tensors = model
    requests = requests_for(cfg, [80, 75, 70], seed=6)
    steps = []
    for key, tokens in requests.items():
        steps.append({"entries": [{"id": key, "tokens": tokens[:20], "want": []}], "end": []})
    for turn in range(40):
        for key, tokens in requests.items():
            steps.append({"entries": [{"id": key, "tokens": [tokens[20 + turn]], "want": []}], "end": []})
    wanted = {}
    for key, tokens in requests.items():
        for position in range(60, len(tokens)):
            steps.append({"entries": [{"id": key, "tokens": [tokens[position]], "want": [0]}],
                          "end": [key] if position == len(tokens) - 1 else []})
    traces.number(steps)
    traces.replay(folder, dtype, steps, max_tokens=256, out_dir=tmp_path)
    got = traces.collect(steps, tmp_path, cfg["vocab_size"], {key: len(tokens) for key, tokens in requests.items()})
    for key, tokens in requests.items():
        want = plain_impl.falcon_h1_logits(cfg, tensors, tokens).numpy()[60:]
        rows = got[key][60:]
        assert not np.isnan(rows).any() and np.isnan(got[key][:60]).all()
        if dtype == "float32":
            assert np.abs(rows - want).max() <= FLOAT32_TOLERANCE, key
        else:
            assert bfloat16_close(rows, want), key
