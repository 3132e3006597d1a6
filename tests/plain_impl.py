"""Plain, slow Falcon-H1 in float32: whole sequences, no cache, one function per part.

This file is the oracle of the test-suite.  It shares no code with the package
under test: it parses ``config.json`` as a raw dict, reads ``model.safetensors``
with the ``safetensors`` library, and computes every position of one sequence
from scratch on the CPU.  Every function cites the lines of the reference
(paths relative to the reference checkout) whose formula it writes down.

Conventions taken from the reference:
  * projections are ``y = x @ W.T + b`` with ``W [out, in]``
    (src/model_weights.rs:530-545);
  * one epsilon for every RMSNorm of the model (src/decoder.rs:2138, 2581-2591);
  * the Mamba2 input projection is split in the order z, x, B, C, dt
    (src/decoder.rs:2203-2209, order comment :5944).

Two things the reference leaves to the checkpoint are written out here, as the
engine's own contract: the decay is stored as ``A_log`` and used as
``A = -exp(A_log)`` (the reference reads the already negative ``A``,
src/decoder.rs:2129, 2336), and the muP multipliers are applied at run time
(the reference has them folded into the file, src/gguf_model.rs:607-629).
"""
from __future__ import annotations

import contextlib
import json
import math
import os
from typing import Dict, List, Optional, Sequence

import torch
import torch.nn.functional as F


# --------------------------------------------------------------------------- rounding of activations
# The model below is exact float32 by default.  Inside ``activations_rounded_to(torch.bfloat16)`` every
# activation that a 16-bit engine keeps in 16 bits between two kernels (normed rows, projected rows, rotated
# queries and keys, attended rows, the conv's output, the gated scan output, the feed-forward's activations
# and each branch's output) is rounded to that dtype and widened again; sums, softmax, norm statistics, the
# recurrence and the residual stream stay float32.  The distance of that model from the exact one is what 16-bit
# activations cost on a given set of weights: a measure of the model's conditioning, not of any kernel.
# With ``dither`` (a torch.Generator) every value is first moved by a random fraction of its last kept bit, so
# that several runs give several samples of the rounding noise (an engine that sums in another order, or folds
# a multiplier into a weight, is one more sample of the same noise).
_ROUND_TO: Optional[torch.dtype] = None
_DITHER: Optional[torch.Generator] = None
# The precision everything is computed in.  float32 is the model; inside ``computed_in(torch.float64)`` the same
# functions run in float64 on the same weights and tokens, which tells how far float32 rounding alone moves this
# model's logits (the inverse frequencies of the rotation stay rounded to float32: they are part of the model).
_EXACT: torch.dtype = torch.float32


@contextlib.contextmanager
def computed_in(dtype: torch.dtype):
    global _EXACT
    before = _EXACT
    _EXACT = dtype
    try:
        yield
    finally:
        _EXACT = before


@contextlib.contextmanager
def activations_rounded_to(dtype: Optional[torch.dtype], dither: Optional[torch.Generator] = None):
    global _ROUND_TO, _DITHER
    before = (_ROUND_TO, _DITHER)
    _ROUND_TO, _DITHER = dtype, dither
    try:
        yield
    finally:
        _ROUND_TO, _DITHER = before


def _r(x: torch.Tensor) -> torch.Tensor:
    if _ROUND_TO is None:
        return x
    if _DITHER is not None:
        bits = 8 if _ROUND_TO == torch.bfloat16 else 11 if _ROUND_TO == torch.float16 else 24
        x = x * (1.0 + (torch.rand(x.shape, generator=_DITHER).to(_EXACT) - 0.5) * 2.0 ** -bits)
    return x.to(_ROUND_TO).to(_EXACT)


# --------------------------------------------------------------------------- parts

def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """y = x / sqrt(mean(x^2) + eps) * w, eps inside the root.

    Closed form confirmed by the golden of src/decoder.rs:10331-10334; built at
    src/model_weights.rs:563-565.
    """
    x = x.to(_EXACT)
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps) * weight.to(_EXACT)


def rope_inverse_frequencies(theta: float, rotary_dim: int) -> torch.Tensor:
    """f_j = 1 / theta^(2j / rotary_dim), formed in float64 and rounded to float32
    (src/decoder.rs:136-144)."""
    return torch.tensor(
        [1.0 / (theta ** (index / rotary_dim)) for index in range(0, rotary_dim, 2)],
        dtype=torch.float64,
    ).to(torch.float32)


def rope_half_split(x: torch.Tensor, positions: torch.Tensor, theta: float,
                    rotary_dim: Optional[int] = None) -> torch.Tensor:
    """Rotate the first ``rotary_dim`` dims of every head, pairing j with j + rotary_dim/2.

    x [T, heads, dh]; positions [T].  Angles = position(float32) * f_j in float32
    (src/decoder.rs:186-195); out[j] = x[j] cos - x[j+half] sin,
    out[j+half] = x[j+half] cos + x[j] sin (layout doc src/architecture.rs:44-48);
    dims past rotary_dim pass through (src/decoder.rs:226-251).
    """
    x = x.to(_EXACT)
    dh = x.shape[-1]
    rotary_dim = dh if rotary_dim is None else rotary_dim
    half = rotary_dim // 2
    freq = rope_inverse_frequencies(theta, rotary_dim)
    angle = positions.to(_EXACT)[:, None] * freq.to(_EXACT)[None, :]      # [T, half]
    cos = angle.cos()[:, None, :]
    sin = angle.sin()[:, None, :]
    first, second = x[..., :half], x[..., half:rotary_dim]
    rotated = torch.cat([first * cos - second * sin, second * cos + first * sin], dim=-1)
    return torch.cat([rotated, x[..., rotary_dim:]], dim=-1)


def gqa_causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                         window: Optional[int] = None) -> torch.Tensor:
    """Dense masked attention over one whole sequence.

    q [T, Hq, dh]; k, v [T, Hkv, dh]; query head h reads kv head h // (Hq // Hkv)
    (src/decoder.rs:4641-4647).  s = q.k * scale; a key is masked when its position
    is after the query's, or when query - key >= window (src/decoder.rs:4515-4532);
    softmax in float32 (src/decoder.rs:4665-4667); o = p @ v.  Returns [T, Hq, dh].
    """
    q, k, v = q.to(_EXACT), k.to(_EXACT), v.to(_EXACT)
    T, Hq, dh = q.shape
    Hkv = k.shape[1]
    group = Hq // Hkv
    out = torch.empty(T, Hq, v.shape[-1], dtype=_EXACT)
    position = torch.arange(T)
    masked = position[None, :] > position[:, None]
    if window is not None:
        masked = masked | ((position[:, None] - position[None, :]) >= window)
    for head in range(Hq):
        kv_head = head // group
        scores = (q[:, head, :] @ k[:, kv_head, :].T) * scale
        scores = scores.masked_fill(masked, float("-inf"))
        probabilities = torch.softmax(scores, dim=-1)
        out[:, head, :] = probabilities @ v[:, kv_head, :]
    return out


def causal_depthwise_conv(x: torch.Tensor, weight: torch.Tensor,
                          bias: Optional[torch.Tensor]) -> torch.Tensor:
    """c[t, ch] = b[ch] + sum_k w[ch, k] * x[t - (K-1) + k, ch]; samples before the
    sequence are zero; w[ch, 0] multiplies the oldest sample.

    x [T, C]; weight [C, K].  src/decoder.rs:2211-2252 (window = history ++ x,
    tap k reads window[t + k]); orientation comment :5948-5950.
    """
    x = x.to(_EXACT)
    T, C = x.shape
    K = weight.shape[1]
    window = torch.cat([torch.zeros(K - 1, C, dtype=_EXACT), x], dim=0)
    out = torch.zeros(T, C, dtype=_EXACT)
    for tap in range(K):
        out = out + window[tap:tap + T, :] * weight[:, tap].to(_EXACT)[None, :]
    if bias is not None:
        out = out + bias.to(_EXACT)[None, :]
    return out


def softplus(x: torch.Tensor) -> torch.Tensor:
    """max(x, 0) + log(1 + exp(-|x|)) (src/decoder.rs:2458-2467;
    crates/macllm-kernels/src/mamba2.rs:263-264)."""
    return torch.clamp(x, min=0.0) + torch.log1p(torch.exp(-x.abs()))


def selective_scan(x: torch.Tensor, B: torch.Tensor, C: torch.Tensor, dt_raw: torch.Tensor,
                   dt_bias: torch.Tensor, A: torch.Tensor, D: torch.Tensor,
                   initial_state: Optional[torch.Tensor] = None):
    """Token-serial state-space recurrence.

    x [T, H, P]; B, C [T, G, N]; dt_raw [T, H]; dt_bias, A, D [H]; state [H, P, N].
    delta = softplus(dt + bias); S = exp(delta * A) * S + delta * x (outer) B;
    y = S . C + D * x; head h uses group h // (H // G).
    crates/macllm-kernels/src/mamba2.rs:259-288; src/decoder.rs:2321-2346.
    Returns (y [T, H, P], final state).
    """
    x, B, C, dt_raw = x.to(_EXACT), B.to(_EXACT), C.to(_EXACT), dt_raw.to(_EXACT)
    T, H, P = x.shape
    G, N = B.shape[1], B.shape[2]
    heads_per_group = H // G
    state = torch.zeros(H, P, N, dtype=_EXACT) if initial_state is None else initial_state.clone().to(_EXACT)
    delta = softplus(dt_raw + dt_bias.to(_EXACT)[None, :])              # [T, H]
    y = torch.empty(T, H, P, dtype=_EXACT)
    group_of_head = torch.arange(H) // heads_per_group
    for t in range(T):
        decay = torch.exp(delta[t] * A.to(_EXACT))                       # [H]
        Bt = B[t][group_of_head]                                      # [H, N]
        Ct = C[t][group_of_head]
        state = state * decay[:, None, None] + (delta[t][:, None, None] * x[t][:, :, None]) * Bt[:, None, :]
        y[t] = (state * Ct[:, None, :]).sum(-1) + D.to(_EXACT)[:, None] * x[t]
    return y, state


def gate_and_group_norm(y: torch.Tensor, z: torch.Tensor, norm_weight: Optional[torch.Tensor],
                        groups: int, eps: float) -> torch.Tensor:
    """y * SiLU(z), then (if a weight is given) RMSNorm over each group of E/G channels.

    y, z [T, E].  Gate first, norm after (src/decoder.rs:2350-2367).
    """
    y = y.to(_EXACT) * F.silu(z.to(_EXACT))
    if norm_weight is None:
        return y
    T, E = y.shape
    grouped = y.view(T, groups, E // groups)
    grouped = grouped / torch.sqrt(grouped.pow(2).mean(-1, keepdim=True) + eps)
    return (grouped * norm_weight.to(_EXACT).reshape(groups, E // groups)[None]).reshape(T, E)


def swiglu(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """SiLU(gate) * up (src/decoder.rs:298-305)."""
    return F.silu(gate.to(_EXACT)) * up.to(_EXACT)


def linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor]) -> torch.Tensor:
    """x @ W.T (+ b) (src/model_weights.rs:530-545)."""
    y = x.to(_EXACT) @ weight.to(_EXACT).T
    return y if bias is None else y + bias.to(_EXACT)


# --------------------------------------------------------------------------- mixers

def attention_mixer(n: torch.Tensor, w: Dict[str, torch.Tensor], *, num_heads: int,
                    num_kv_heads: int, head_dim: int, theta: float,
                    in_multiplier: float = 1.0, key_multiplier: float = 1.0,
                    out_multiplier: float = 1.0, window: Optional[int] = None,
                    positions: Optional[torch.Tensor] = None,
                    use_rope: bool = True) -> torch.Tensor:
    """q/k/v projections, RoPE on q and k, causal GQA with scale 1/sqrt(dh), o_proj.

    src/decoder.rs:1099-1161 (projections), :953-962 (RoPE at the lane's start),
    :4580-4670 (scores), :923-931 (output); scale fixed at 1/sqrt(dh),
    src/gguf_model.rs:584.  ``w`` holds q_proj/k_proj/v_proj/o_proj ``.weight``
    (+ optional ``.bias``).
    """
    T = n.shape[0]
    positions = torch.arange(T) if positions is None else positions
    n = n.to(_EXACT) * in_multiplier
    q = _r(linear(n, w["q_proj.weight"], w.get("q_proj.bias"))).view(T, num_heads, head_dim)
    k = linear(n, w["k_proj.weight"], w.get("k_proj.bias")).view(T, num_kv_heads, head_dim)
    k = _r(k * key_multiplier)
    v = _r(linear(n, w["v_proj.weight"], w.get("v_proj.bias"))).view(T, num_kv_heads, head_dim)
    if use_rope:
        q = _r(rope_half_split(q, positions, theta))
        k = _r(rope_half_split(k, positions, theta))
    o = _r(gqa_causal_attention(q, k, v, 1.0 / math.sqrt(head_dim), window))
    return _r(linear(o.reshape(T, num_heads * head_dim), w["o_proj.weight"], w.get("o_proj.bias")) * out_multiplier)


def mamba2_mixer(n: torch.Tensor, w: Dict[str, torch.Tensor], *, num_heads: int, head_dim: int,
                 state_size: int, num_groups: int, conv_kernel: int, eps: float,
                 in_multiplier: float = 1.0, out_multiplier: float = 1.0,
                 multipliers: Sequence[float] = (1.0, 1.0, 1.0, 1.0, 1.0),
                 projected: Optional[torch.Tensor] = None, return_state: bool = False):
    """in_proj -> split z,x,B,C,dt -> causal conv + SiLU over [x,B,C] -> scan -> D skip
    (inside the scan) -> * SiLU(z) -> optional grouped RMSNorm -> out_proj.

    src/decoder.rs:2175 (in_proj), :2203-2209 (split), :2211-2253 (conv, SiLU),
    :2295-2349 (scan), :2350-2367 (gate, norm), :2368-2371 (out_proj).
    ``projected`` bypasses in_proj (the reference's operator test feeds the projected
    rows directly, src/decoder.rs:7190).
    """
    E = num_heads * head_dim
    GN = num_groups * state_size
    if projected is None:
        u = linear(n.to(_EXACT) * in_multiplier, w["in_proj.weight"], w.get("in_proj.bias"))
    else:
        u = projected.to(_EXACT)
    T = u.shape[0]
    z, x, B, C, dt = torch.split(u, [E, E, GN, GN, num_heads], dim=-1)
    z, x, B, C, dt = (_r(z * multipliers[0]), _r(x * multipliers[1]), _r(B * multipliers[2]),
                      _r(C * multipliers[3]), _r(dt * multipliers[4]))
    xbc = torch.cat([x, B, C], dim=-1)
    conv_weight = w["conv1d.weight"]
    if conv_weight.dim() == 3:                      # [C, 1, K] accepted, src/decoder.rs:2089-2095
        conv_weight = conv_weight.squeeze(1)
    conv = _r(F.silu(causal_depthwise_conv(xbc, conv_weight, w.get("conv1d.bias"))))
    xc, Bc, Cc = torch.split(conv, [E, GN, GN], dim=-1)
    A = -torch.exp(w["A_log"].to(_EXACT).reshape(num_heads))
    y, state = selective_scan(
        xc.view(T, num_heads, head_dim), Bc.view(T, num_groups, state_size),
        Cc.view(T, num_groups, state_size), dt, w["dt_bias"].to(_EXACT), A,
        w["D"].to(_EXACT).reshape(num_heads))
    y = _r(gate_and_group_norm(y.reshape(T, E), z, w.get("norm.weight"), num_groups, eps))
    out = _r(linear(y, w["out_proj.weight"], w.get("out_proj.bias")) * out_multiplier)
    if return_state:
        return out, state, xbc[-(conv_kernel - 1):] if conv_kernel > 1 else None
    return out


def swiglu_mlp(f: torch.Tensor, w: Dict[str, torch.Tensor], gate_multiplier: float = 1.0,
               down_multiplier: float = 1.0) -> torch.Tensor:
    """down(SiLU(gate(f)) * up(f)) (src/decoder.rs:276-304)."""
    gate = _r(linear(f, w["gate_proj.weight"], w.get("gate_proj.bias")) * gate_multiplier)
    up = _r(linear(f, w["up_proj.weight"], w.get("up_proj.bias")))
    return _r(linear(_r(swiglu(gate, up)), w["down_proj.weight"], w.get("down_proj.bias")) * down_multiplier)


# --------------------------------------------------------------------------- the model

def _sub(tensors: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    return {name[len(prefix):]: value for name, value in tensors.items() if name.startswith(prefix)}


def falcon_h1_layer(h: torch.Tensor, tensors: Dict[str, torch.Tensor], layer: int, cfg: dict,
                    ablate: Sequence[str] = ()) -> torch.Tensor:
    """n = norm(h); h1 = h + attention(n) + mamba(n); h2 = h1 + mlp(norm(h1)).

    src/decoder.rs:2658-2682 (parallel mixers on the same normed input, summed),
    :2684-2699 (residuals, second norm, feed-forward).
    """
    prefix = f"model.layers.{layer}."
    eps = cfg.get("rms_norm_eps", 1e-5)
    n = _r(rms_norm(h, tensors[prefix + "attn_norm.weight"], eps))
    mixed = torch.zeros_like(h)
    if "attention" not in ablate:
        mixed = mixed + attention_mixer(
            n, _sub(tensors, prefix + "self_attn."),
            num_heads=cfg["num_attention_heads"],
            num_kv_heads=cfg.get("num_key_value_heads", cfg["num_attention_heads"]),
            head_dim=cfg.get("head_dim", cfg["hidden_size"] // cfg["num_attention_heads"]),
            theta=cfg.get("rope_theta", 1e11),
            in_multiplier=cfg.get("attention_in_multiplier", 1.0),
            key_multiplier=cfg.get("key_multiplier", 1.0),
            out_multiplier=cfg.get("attention_out_multiplier", 1.0))
    if "mamba" not in ablate:
        mixed = mixed + mamba2_mixer(
            n, _sub(tensors, prefix + "mamba."),
            num_heads=cfg["mamba_n_heads"],
            head_dim=cfg.get("mamba_d_head", cfg.get("mamba_d_ssm", 0) // cfg["mamba_n_heads"]),
            state_size=cfg["mamba_d_state"], num_groups=cfg.get("mamba_n_groups", 1),
            conv_kernel=cfg.get("mamba_d_conv", 4), eps=eps,
            in_multiplier=cfg.get("ssm_in_multiplier", 1.0),
            out_multiplier=cfg.get("ssm_out_multiplier", 1.0),
            multipliers=cfg.get("ssm_multipliers", [1.0] * 5))
    h1 = h + mixed
    if "mlp" in ablate:
        return h1
    f = _r(rms_norm(h1, tensors[prefix + "ffn_norm.weight"], eps))
    mlp_multipliers = cfg.get("mlp_multipliers", [1.0, 1.0])
    return h1 + swiglu_mlp(f, _sub(tensors, prefix + "mlp."), mlp_multipliers[0], mlp_multipliers[1])


def falcon_h1_logits(cfg: dict, tensors: Dict[str, torch.Tensor], tokens: Sequence[int],
                     ablate: Sequence[str] = ()) -> torch.Tensor:
    """Logits [T, V] (float32) at every position of one whole sequence.

    Embedding * multiplier (src/decoder.rs:3194-3197), layers, final norm, lm_head (tied:
    the embedding matrix, src/decoder.rs:3045-3053) * multiplier (src/decoder.rs:3349-3357).
    """
    token_ids = torch.tensor(list(tokens), dtype=torch.long)
    embedding = tensors["model.embed_tokens.weight"].to(_EXACT)
    h = embedding[token_ids] * cfg.get("embedding_multiplier", 1.0)
    for layer in range(cfg["num_hidden_layers"]):
        h = falcon_h1_layer(h, tensors, layer, cfg, ablate)
    h = _r(rms_norm(h, tensors["model.norm.weight"], cfg.get("rms_norm_eps", 1e-5)))
    head = embedding if cfg.get("tie_word_embeddings", False) else tensors["lm_head.weight"].to(_EXACT)
    return (h @ head.T) * cfg.get("lm_head_multiplier", 1.0)


def load_model_dir(path: str):
    """(config dict, tensors) from a folder with config.json and model.safetensors."""
    from safetensors.torch import load_file
    with open(os.path.join(path, "config.json")) as handle:
        cfg = json.load(handle)
    tensors = load_file(os.path.join(path, "model.safetensors"))
    return cfg, tensors


# --------------------------------------------------------------------------- sampling

_MASK64 = (1 << 64) - 1


def draw_uniform(seed: int, draw_index: int) -> float:
    """The engine's own counter-based generator (the reference's ChaCha8 stream is a
    library detail, src/sampling.rs:57,167): splitmix64 of seed + (index+1)*golden,
    top 24 bits / 2^24."""
    z = (seed + (draw_index + 1) * 0x9E3779B97F4A7C15) & _MASK64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK64
    z = z ^ (z >> 31)
    return (z >> 40) / float(1 << 24)


def sample_token(logits: torch.Tensor, *, temperature: float = 0.0, top_k: int = 0,
                 top_p: float = 1.0, repetition_penalty: float = 1.0,
                 presence_penalty: float = 0.0, frequency_penalty: float = 0.0,
                 history: Sequence[int] = (), generated: Sequence[int] = (),
                 seed: int = 0, draw_index: int = 0, allowed: Optional[Sequence[int]] = None) -> int:
    """One token from one row of logits, in the reference's order of operations.

    Repetition penalty over prompt+generated (x<0 ? x*p : x/p, src/sampling.rs:407-423),
    presence/frequency over generated only (:392-405), then argmax with the lowest
    index on ties (:425-433) or: divide by temperature, keep the top-k (value
    descending, index ascending), softmax (max-subtracted, float32), keep the shortest
    descending prefix whose mass reaches top_p (:337-375), draw u*total and walk the
    kept tokens in index order (:165-169, :378-390).  ``allowed``: a constraint's mask over the penalized
    row, every other token at -inf (:119-130, before argmax or the stochastic path).
    """
    import numpy as np
    values = logits.detach().float().cpu().numpy().astype(np.float32).copy()
    if repetition_penalty > 0 and abs(repetition_penalty - 1.0) >= 1.1920929e-07:
        for token in sorted(set(int(t) for t in history)):
            if 0 <= token < values.size:
                values[token] = values[token] * np.float32(repetition_penalty) if values[token] < 0 \
                    else values[token] / np.float32(repetition_penalty)
    if (presence_penalty != 0.0 or frequency_penalty != 0.0) and len(generated) > 0:
        counts: Dict[int, int] = {}
        for token in generated:
            counts[int(token)] = counts.get(int(token), 0) + 1
        for token, count in counts.items():
            if 0 <= token < values.size:
                values[token] -= np.float32(frequency_penalty) * np.float32(count) + np.float32(presence_penalty)
    if allowed is not None:
        masked = np.full_like(values, -np.inf)
        for token in allowed:
            masked[int(token)] = values[int(token)]
        values = masked
    if temperature <= 0.0:
        return int(np.argmax(values))                      # first index of the maximum
    values = values / np.float32(temperature)
    vocab = values.size
    order = sorted(range(vocab), key=lambda index: (-float(values[index]), index))
    if 0 < top_k < vocab:
        for index in order[top_k:]:
            values[index] = -np.inf
        order = order[:top_k]
    maximum = values.max()
    probabilities = np.exp(values - maximum).astype(np.float32)
    total = np.float32(0.0)
    for index in range(vocab):
        total = np.float32(total + probabilities[index])
    probabilities = (probabilities / total).astype(np.float32)
    order.sort(key=lambda index: (-float(probabilities[index]), index))
    if 0.0 <= top_p < 1.0:
        cumulative = np.float32(0.0)
        keep = 0
        for index in order:
            cumulative = np.float32(cumulative + probabilities[index])
            keep += 1
            if cumulative >= np.float32(top_p):
                break
        for index in order[keep:]:
            probabilities[index] = 0.0
    kept_total = np.float32(0.0)
    for index in range(vocab):
        kept_total = np.float32(kept_total + probabilities[index])
    target = np.float32(draw_uniform(seed, draw_index)) * kept_total
    cumulative = np.float32(0.0)
    for index in range(vocab):
        if probabilities[index] <= 0.0:
            continue
        cumulative = np.float32(cumulative + probabilities[index])
        if target < cumulative:
            return index
    return int(np.argmax(probabilities))


def greedy_generate(cfg: dict, tensors: Dict[str, torch.Tensor], prompt: Sequence[int],
                    max_new_tokens: int) -> List[int]:
    """Greedy continuation by recomputing the whole sequence for every new token."""
    tokens = list(prompt)
    out: List[int] = []
    for _ in range(max_new_tokens):
        logits = falcon_h1_logits(cfg, tensors, tokens)[-1]
        token = sample_token(logits)
        out.append(token)
        tokens.append(token)
    return out
