"""Toy parts for the tests of the framework's generality: a mixer with state of its own, a
position encoding that is no rotation, a feed-forward that routes each token to two of its
experts, a norm that centres its rows, an arrangement of a layer with a norm after the mixer, and a
toy architecture that uses them together with a
windowed attention layer, a layer that runs twice and a run that reads another run's cache.
They are registered from here, without a change to the package, and never become a model."""
from dataclasses import dataclass

import torch

import plain_impl

@dataclass(frozen=True)
class DecayMixerSpec:
    """A toy mixer with state of its own: s_t = a * s_{t-1} + x_t W; y_t = s_t."""
    width: int
    decay: float
    kind: str = "toy_decay"

    def validate(self):
        assert 0 < self.decay < 1


@dataclass(frozen=True)
class AlibiLikeSpec:
    """A toy position encoding with both hooks: it scales q and k by (1 + position * slope) before the cache
    write, and it biases the scores by distance: score(head h, query s, key p) -= bias / (h + 1) * (s - p)."""
    slope: float
    bias: float = 0.0
    heads: int = 4
    kind: str = "toy_scale_position"

    def validate(self, head_dim):
        pass


@dataclass(frozen=True)
class RoutedSpec:
    """A toy feed-forward with routing: a float32 router picks each token's two best experts
    (ties to the lower index), weighs them by the softmax of their two logits, and each expert
    is down(relu(up(x)))."""
    experts: int
    inner: int
    kind: str = "toy_routed"

    def validate(self):
        assert self.experts >= 2 and self.inner > 0


@dataclass(frozen=True)
class CentredNormSpec:
    """A toy norm: y = (x - mean) / sqrt(var + eps) * w + b."""
    eps: float
    kind: str = "toy_centred_norm"

    def validate(self):
        assert self.eps > 0


@dataclass(frozen=True)
class GatedDecaySpec:
    """A toy mixer with state of its own that hands out its pieces: [a | b] = x W_in; s_t = decay * s_{t-1} + a_t;
    y_t = s_t * sigmoid(b_t); out = y W_out."""
    width: int
    decay: float
    kind: str = "toy_gated_decay"

    def validate(self):
        assert 0 < self.decay < 1 and self.width > 0


@dataclass
class ToyFastConfig:
    """A toy architecture of two one-mixer layers for the fast paths of a layer: layer 0 = attention alone
    with the package's own norm and feed-forward; layer 1 = the gated decay mixer alone, between the centring
    toy norms, with the routed toy feed-forward."""
    raw: dict
    architecture_names = ("ToyFastForTests",)

    @classmethod
    def from_dict(cls, raw):
        return cls(raw)

    def to_dict(self):
        return dict(self.raw)

    def to_model_spec(self):
        from macllm_infer_amd.config import (AttentionSpec, LayerSpec, MixerSlot, ModelSpec, RmsNormSpec, RopeSpec,
                                             ScheduleEntry, SwiGLUSpec)
        raw = self.raw
        norm = RmsNormSpec(eps=1e-5)
        attention = AttentionSpec(num_heads=2, num_kv_heads=1, head_dim=64, scale=0.125,
                                  position=RopeSpec(theta=1e4, rotary_dim=64))
        layers = (LayerSpec(prefix="model.layers.0", ffn=SwiGLUSpec(intermediate_size=64), mixer_norm=norm, ffn_norm=norm,
                            mixers=(MixerSlot("self_attn", attention),)),
                  LayerSpec(prefix="model.layers.1", ffn=RoutedSpec(3, 24), mixer_norm=CentredNormSpec(1e-4),
                            ffn_norm=CentredNormSpec(1e-4),
                            mixers=(MixerSlot("decay", GatedDecaySpec(raw["width"], raw["decay"])),)))
        return ModelSpec(architecture="ToyFastForTests", hidden_size=raw["hidden"], vocab_size=raw["vocab"],
                         max_context=512, layers=layers, schedule=(ScheduleEntry(0), ScheduleEntry(1)),
                         final_norm=norm, tied_embeddings=True)


@dataclass
class ToyConfig:
    """A toy architecture: layer 0 = attention (toy position encoding) and the decay mixer in
    parallel, layer 1 = windowed attention with partial RoPE and the routed feed-forward, its norms
    the centring toy norm, arranged with one more norm on the mixer's output (``toy_sandwich``).  ``raw["schedule"]`` lists
    (layer, entry whose cache is read or None) in running order."""
    raw: dict
    architecture_names = ("ToyForTests",)

    @classmethod
    def from_dict(cls, raw):
        return cls(raw)

    def to_dict(self):
        return dict(self.raw)

    def to_model_spec(self):
        from macllm_infer_amd.config import (AttentionSpec, LayerSpec, MixerSlot, ModelSpec, RmsNormSpec, RopeSpec,
                                             ScheduleEntry, SwiGLUSpec)
        raw = self.raw
        hidden = raw["hidden"]
        norm = RmsNormSpec(eps=1e-5)
        full = AttentionSpec(num_heads=4, num_kv_heads=2, head_dim=16, scale=0.25,
                             position=AlibiLikeSpec(slope=raw["slope"], bias=raw.get("bias", 0.0)))
        windowed = AttentionSpec(num_heads=4, num_kv_heads=2, head_dim=16, scale=0.25,
                                 position=RopeSpec(theta=100.0, rotary_dim=8), window=raw["window"])
        ffn = SwiGLUSpec(intermediate_size=48)
        layers = (LayerSpec(prefix="model.layers.0", ffn=ffn, mixer_norm=norm, ffn_norm=norm,
                            mixers=(MixerSlot("self_attn", full), MixerSlot("decay", DecayMixerSpec(hidden, raw["decay"])))),
                  LayerSpec(prefix="model.layers.1", ffn=RoutedSpec(raw["experts"], 24), mixer_norm=CentredNormSpec(1e-4),
                            ffn_norm=CentredNormSpec(1e-4), arrangement="toy_sandwich",
                            mixers=(MixerSlot("self_attn", windowed),)))
        schedule = tuple(ScheduleEntry(layer=layer, kv_from=source) for layer, source in raw["schedule"])
        return ModelSpec(architecture="ToyForTests", hidden_size=hidden, vocab_size=raw["vocab"], max_context=512,
                         layers=layers, schedule=schedule, final_norm=norm, tied_embeddings=True)


@dataclass(frozen=True)
class TableDecaySpec:
    """The decay mixer once more, s_t = decay * s_{t-1} + x_t W; y_t = s_t, without a look at the host: where a
    token's lane begins and which state slot it reads and writes comes from an index table of the mixer's own in
    every step (``step_tables``), so that its forward pass can be captured in a graph."""
    width: int
    decay: float
    kind: str = "toy_table_decay"

    def validate(self):
        assert 0 < self.decay < 1 and self.width > 0


@dataclass
class ToyTableConfig:
    """A toy architecture of one layer: attention beside the decay mixer that reads a step table of its own."""
    raw: dict
    architecture_names = ("ToyTableForTests",)

    @classmethod
    def from_dict(cls, raw):
        return cls(raw)

    def to_dict(self):
        return dict(self.raw)

    def to_model_spec(self):
        from macllm_infer_amd.config import (AttentionSpec, LayerSpec, MixerSlot, ModelSpec, RmsNormSpec, RopeSpec,
                                             ScheduleEntry, SwiGLUSpec)
        raw = self.raw
        norm = RmsNormSpec(eps=1e-5)
        attention = AttentionSpec(num_heads=2, num_kv_heads=1, head_dim=32, scale=32 ** -0.5,
                                  position=RopeSpec(theta=1e3, rotary_dim=32))
        layer = LayerSpec(prefix="model.layers.0", ffn=SwiGLUSpec(intermediate_size=48), mixer_norm=norm, ffn_norm=norm,
                          mixers=(MixerSlot("self_attn", attention),
                                  MixerSlot("decay", TableDecaySpec(raw["hidden"], raw["decay"]))))
        return ModelSpec(architecture="ToyTableForTests", hidden_size=raw["hidden"], vocab_size=raw["vocab"],
                         max_context=512, layers=(layer,), schedule=(ScheduleEntry(0), ScheduleEntry(0)),
                         final_norm=norm, tied_embeddings=True, logit_multiplier=raw["logit_scale"],
                         logit_softcap=raw["logit_cap"])


@dataclass(frozen=True)
class StretchedRopeSpec:
    """A toy position encoding: the half-split rotation with every angle divided by ``stretch``.  ``kind`` picks the
    class that says so to the fused decode kernel (``fused_rotation``) or the one that keeps it to itself."""
    theta: float
    rotary_dim: int
    stretch: float
    kind: str = "toy_stretched_rope"

    def validate(self, head_dim=None):
        assert self.stretch > 0 and self.rotary_dim % 2 == 0


@dataclass
class ToyStretchedConfig:
    """The package's own hybrid architecture with the toy rotation in place of its own in every layer:
    ``raw["base"]`` is that architecture's config.json, ``raw["stretch"]`` and ``raw["position_kind"]`` the toy's."""
    raw: dict
    architecture_names = ("ToyStretchedForTests",)

    @classmethod
    def from_dict(cls, raw):
        return cls(raw)

    def to_dict(self):
        return dict(self.raw)

    def to_model_spec(self):
        from dataclasses import replace
        from macllm_infer_amd.config import FalconH1Config
        spec = FalconH1Config.from_dict(self.raw["base"]).to_model_spec()
        layers = []
        for layer in spec.layers:
            mixers = []
            for slot in layer.mixers:
                position = getattr(slot.spec, "position", None)
                if position is not None:
                    toy = StretchedRopeSpec(position.theta, position.rotary_dim, self.raw["stretch"], self.raw["position_kind"])
                    slot = replace(slot, spec=replace(slot.spec, position=toy))
                mixers.append(slot)
            layers.append(replace(layer, mixers=tuple(mixers)))
        return replace(spec, architecture="ToyStretchedForTests", layers=tuple(layers))


TABLE_FILLS = []          # (lanes, tokens) of every fill of the toy mixer's step table


def register_toys():
    from macllm_infer_amd.cache import StateNeed
    from macllm_infer_amd.config import register_architecture
    from macllm_infer_amd.parts import (FeedForward, Mixer, Part, PositionEncoding, part_class, register_arrangement,
                                        register_part)
    from macllm_infer_amd.weights import Expect

    @register_part("toy_decay")
    class DecayMixer(Mixer):
        kernel_modules = ()

        @classmethod
        def expected_tensors(cls, spec, prefix, hidden_size):
            return [Expect(f"{prefix}.w.weight", ((spec.width, hidden_size),))]

        @classmethod
        def cache_needs(cls, spec):
            return [StateNeed("s", (spec.width,), "float32")]

        def __init__(self, spec, prefix, tensors, build):
            self.spec = spec
            self.weight = tensors[f"{prefix}.w.weight"].float().to(build.device)

        def forward(self, x, step, cache):
            state = cache.states["s"]
            projected = x.float() @ self.weight.T
            out = torch.empty_like(projected)
            cursor = 0
            for lane, length in enumerate(step.lane_lengths):          # a toy: token-serial on the host
                slot = int(step.slot_ids[lane])
                s = state[slot].clone()
                for t in range(cursor, cursor + length):
                    s = self.spec.decay * s + projected[t]
                    out[t] = s
                state[slot] = s
                cursor += length
            return out.to(x.dtype)

    @register_part("toy_table_decay")
    class TableDecay(Mixer):
        kernel_modules = ()
        graph_safe = True
        TABLE = "toy_decay_rows"

        @classmethod
        def expected_tensors(cls, spec, prefix, hidden_size):
            return [Expect(f"{prefix}.w.weight", ((spec.width, hidden_size),))]

        @classmethod
        def cache_needs(cls, spec):
            return [StateNeed("s", (spec.width,), "float32")]

        def __init__(self, spec, prefix, tensors, build):
            self.spec = spec
            self.weight = tensors[f"{prefix}.w.weight"].float().to(build.device)

        def step_tables(self):
            from macllm_infer_amd.engine import StepTable

            def fill(out, packed):
                # a row a token: (first row of its lane, state slot it reads, state slot its state is written to:
                # the lane's own for the lane's last token, the spare one for every other)
                TABLE_FILLS.append((packed.num_lanes, packed.num_tokens))
                rows = out.reshape(-1, 3)
                for lane in range(packed.num_lanes):
                    first, end = int(packed.first_token[lane]), int(packed.first_token[lane + 1])
                    rows[first:end, 0] = first
                    rows[first:end, 1] = packed.slot_ids[lane]
                    rows[first:end, 2] = packed.scratch_slot
                    rows[end - 1, 2] = packed.slot_ids[lane]

            return [StepTable(self.TABLE, lambda lanes, tokens: 3 * tokens, fill)]

        def forward(self, x, step, cache):
            state = cache.states["s"]
            tokens = x.shape[0]
            table = step.tables[self.TABLE].view(-1, 3)[:tokens].long()
            first, read_from, write_to = table[:, 0], table[:, 1], table[:, 2]
            projected = x.float() @ self.weight.T
            rows = torch.arange(tokens, device=x.device)
            distance = rows[:, None] - rows[None, :]
            together = (first[:, None] == first[None, :]) & (distance >= 0)
            powers = torch.where(together, torch.pow(self.spec.decay, distance.clamp(min=0).float()), 0.0)
            carried = state[read_from] * torch.pow(self.spec.decay, (rows - first + 1).float())[:, None]
            out = powers @ projected + carried
            state.index_copy_(0, write_to, out)
            return out.to(x.dtype)

    @register_part("toy_gated_decay")
    class GatedDecay(Mixer):
        kernel_modules = ("gemm",)

        @classmethod
        def expected_tensors(cls, spec, prefix, hidden_size):
            return [Expect(f"{prefix}.in_proj.weight", ((2 * spec.width, hidden_size),)),
                    Expect(f"{prefix}.out_proj.weight", ((hidden_size, spec.width),))]

        @classmethod
        def cache_needs(cls, spec):
            return [StateNeed("s", (spec.width,), "float32")]

        def __init__(self, spec, prefix, tensors, build):
            from macllm_infer_amd.parts import Linear
            self.spec = spec
            self.in_proj = Linear([tensors[f"{prefix}.in_proj.weight"]], [None], build)
            self.out_proj = Linear([tensors[f"{prefix}.out_proj.weight"]], [None], build)

        def projections(self):
            return self.in_proj, self.out_proj, self.spec.width

        def forward(self, x, step, cache):
            mixed = torch.empty((x.shape[0], self.spec.width), dtype=x.dtype, device=x.device)
            self.mix(self.in_proj(x), step, cache, mixed)
            return self.out_proj(mixed)

        def mix(self, projected, step, cache, out):
            width, state = self.spec.width, cache.states["s"]
            a, b = projected[:, :width].float(), projected[:, width:2 * width].float()
            cursor = 0
            for lane, length in enumerate(step.lane_lengths):          # a toy: token-serial on the host
                slot = int(step.slot_ids[lane])
                s = state[slot].clone()
                for t in range(cursor, cursor + length):
                    s = self.spec.decay * s + a[t]
                    out[t] = (s * torch.sigmoid(b[t])).to(out.dtype)
                state[slot] = s
                cursor += length

    @register_part("toy_scale_position")
    class ScalePosition(PositionEncoding):
        def __init__(self, spec, head_dim, build):
            self.slope = spec.slope
            if spec.bias:
                self.score_slopes = torch.tensor([spec.bias / (head + 1) for head in range(spec.heads)],
                                                 dtype=torch.float32, device=build.device)

        def rotate(self, qkv, num_heads, num_kv_heads, head_dim, step):
            factor = (1.0 + step.positions.float() * self.slope)[:, None]
            width = (num_heads + num_kv_heads) * head_dim
            qkv[:, :width] = (qkv[:, :width].float() * factor).to(qkv.dtype)

    @register_part("toy_stretched_rope_unsaid")
    class StretchedRopeUnsaid(PositionEncoding):
        graph_safe = True

        def __init__(self, spec, head_dim, build):
            from macllm_infer_amd.kernels import ops
            self.ops = ops
            self.rotary_dim = spec.rotary_dim
            frequencies = [1.0 / (spec.theta ** (index / spec.rotary_dim)) / spec.stretch
                           for index in range(0, spec.rotary_dim, 2)]
            self.inv_freq = torch.tensor(frequencies, dtype=torch.float64).to(torch.float32).to(build.device)

        def rotate_and_store(self, qkv, num_heads, num_kv_heads, head_dim, step, cache):
            owns = cache.owns_kv
            self.ops.rope_kv_store(qkv, num_heads, num_kv_heads, head_dim, step.positions, self.inv_freq,
                                   self.rotary_dim, step.slot_mappings[cache.group] if owns else None,
                                   cache.k_cache if owns else None, cache.v_cache if owns else None)

    @register_part("toy_stretched_rope")
    class StretchedRope(StretchedRopeUnsaid):
        def fused_rotation(self):
            return self.inv_freq, self.rotary_dim

    @register_part("toy_routed")
    class Routed(FeedForward):
        @classmethod
        def expected_tensors(cls, spec, prefix, hidden_size):
            return [Expect(f"{prefix}.router.weight", ((spec.experts, hidden_size),)),
                    Expect(f"{prefix}.up.weight", ((spec.experts, spec.inner, hidden_size),)),
                    Expect(f"{prefix}.down.weight", ((spec.experts, hidden_size, spec.inner),))]

        def __init__(self, spec, prefix, tensors, build):
            self.router, self.up, self.down = (tensors[f"{prefix}.{name}.weight"].float().to(build.device)
                                               for name in ("router", "up", "down"))

        def forward(self, x):
            return routed_feed_forward(x.float(), self.router, self.up, self.down).to(x.dtype)

    @register_part("toy_centred_norm")
    class CentredNorm(Part):
        @classmethod
        def expected_tensors(cls, spec, prefix, hidden_size):
            return [Expect(f"{prefix}.weight", ((hidden_size,),), init="norm"),
                    Expect(f"{prefix}.bias", ((hidden_size,),), init="bias")]

        def __init__(self, spec, prefix, tensors, build):
            self.eps, self.dtype = spec.eps, build.dtype
            self.weight = tensors[f"{prefix}.weight"].float().to(build.device)
            self.bias = tensors[f"{prefix}.bias"].float().to(build.device)

        def forward(self, residual, rows=None):
            for delta in residual.pending:                  # a norm folds the branch outputs into the stream
                residual.h += delta.float()
            residual.pending = []
            x = residual.h if rows is None else residual.h[rows.long()]
            return centred_norm(x, self.weight, self.bias, self.eps).to(self.dtype)

    @register_arrangement("toy_sandwich")
    class Sandwich:
        """h += post(mixer(pre(h))); h += ffn(norm(h)): one mixer, and a norm of its own
        (``<prefix>.post_norm``, of the kind of the layer's mixer norm) on the mixer's output."""

        @classmethod
        def parts(cls, layer):
            norm = part_class(layer.mixer_norm)
            slot = layer.mixers[0]
            return [(norm, layer.mixer_norm, f"{layer.prefix}.{layer.mixer_norm_name}"),
                    (part_class(slot.spec), slot.spec, f"{layer.prefix}.{slot.name}"),
                    (norm, layer.mixer_norm, f"{layer.prefix}.post_norm"),
                    (part_class(layer.ffn_norm), layer.ffn_norm, f"{layer.prefix}.{layer.ffn_norm_name}"),
                    (part_class(layer.ffn), layer.ffn, f"{layer.prefix}.{layer.ffn_name}")]

        @classmethod
        def expected_tensors(cls, layer, hidden_size):
            return [expect for kind, spec, prefix in cls.parts(layer)
                    for expect in kind.expected_tensors(spec, prefix, hidden_size)]

        @classmethod
        def kernel_modules(cls, layer):
            return [module for kind, _, _ in cls.parts(layer) for module in kind.kernel_modules]

        def __init__(self, layer, tensors, build):
            self.pre, self.mixer, self.post, self.ffn_norm, self.ffn = (
                kind(spec, prefix, tensors, build) for kind, spec, prefix in self.parts(layer))
            self.mixers = [(layer.mixers[0].name, self.mixer)]       # what the model asks caches for
            self.graph_safe = False

        def forward(self, residual, step, caches):
            from macllm_infer_amd.parts.base import Residual
            mixed = self.mixer.forward(self.pre.forward(residual), step, caches[self.mixers[0][0]])
            residual.pending = [self.post.forward(Residual(mixed.float()))]
            residual.pending = [self.ffn.forward(self.ffn_norm.forward(residual))]

    register_architecture(ToyConfig)
    register_architecture(ToyFastConfig)
    register_architecture(ToyTableConfig)
    register_architecture(ToyStretchedConfig)


def centred_norm(x, weight, bias, eps):
    centred = x - x.mean(dim=-1, keepdim=True)
    return centred / torch.sqrt(centred.pow(2).mean(dim=-1, keepdim=True) + eps) * weight + bias


def distance_biased_attention(q, k, v, scale, slopes):
    """Causal attention, head by head, with score(s, p) = q_s . k_p * scale - slope_head * (s - p)."""
    T, heads, _ = q.shape
    group = heads // k.shape[1]
    distance = (torch.arange(T)[:, None] - torch.arange(T)[None, :]).float()
    out = torch.empty_like(q)
    for head in range(heads):
        scores = q[:, head] @ k[:, head // group].T * scale - slopes[head] * distance
        scores = scores.masked_fill(distance < 0, float("-inf"))
        out[:, head] = torch.softmax(scores, dim=-1) @ v[:, head // group]
    return out


def routed_feed_forward(x, router, up, down):
    """Each token through its two best experts; a token's result depends on that token alone."""
    logits = x @ router.T
    best = torch.sort(logits, dim=-1, descending=True, stable=True).indices[:, :2]
    weights = torch.softmax(torch.gather(logits, 1, best), dim=-1)
    out = torch.zeros_like(x)
    for rank in range(2):
        chosen = best[:, rank]
        hidden = torch.relu(torch.einsum("td,tid->ti", x, up[chosen]))
        out += weights[:, rank:rank + 1] * torch.einsum("ti,tdi->td", hidden, down[chosen])
    return out


def toy_plain_logits(raw, tensors, tokens):
    """The toy model, whole sequence, from the plain parts."""
    T = len(tokens)
    positions = torch.arange(T)
    h = tensors["model.embed_tokens.weight"].float()[torch.tensor(tokens)]
    caches = {}
    for index, (layer, source) in enumerate(raw["schedule"]):
        p = f"model.layers.{layer}."
        if layer == 0:
            norm = lambda x, name: plain_impl.rms_norm(x, tensors[p + name + ".weight"], 1e-5)
        else:
            norm = lambda x, name: centred_norm(x, tensors[p + name + ".weight"].float(), tensors[p + name + ".bias"].float(), 1e-4)
        n = norm(h, "attn_norm")
        w = {name[len(p + "self_attn."):]: value for name, value in tensors.items() if name.startswith(p + "self_attn.")}
        q = plain_impl.linear(n, w["q_proj.weight"], None).view(T, 4, 16)
        k = plain_impl.linear(n, w["k_proj.weight"], None).view(T, 2, 16)
        v = plain_impl.linear(n, w["v_proj.weight"], None).view(T, 2, 16)
        if layer == 0:
            factor = (1.0 + positions.float() * raw["slope"])[:, None, None]
            q, k = q * factor, k * factor
            window = None
        else:
            q = plain_impl.rope_half_split(q, positions, 100.0, rotary_dim=8)
            k = plain_impl.rope_half_split(k, positions, 100.0, rotary_dim=8)
            window = raw["window"]
        if source is None:
            caches[index] = (k, v)
        else:
            k, v = caches[source]                       # reads the other run's keys and values
        if layer == 0 and raw.get("bias"):
            attended = distance_biased_attention(q, k, v, 0.25, [raw["bias"] / (head + 1) for head in range(4)])
        else:
            attended = plain_impl.gqa_causal_attention(q, k, v, 0.25, window)
        mixed = plain_impl.linear(attended.reshape(T, 64), w["o_proj.weight"], None)
        if layer == 0:
            projected = n @ tensors[p + "decay.w.weight"].float().T
            s = torch.zeros(raw["hidden"])
            rows = []
            for t in range(T):
                s = raw["decay"] * s + projected[t]
                rows.append(s)
            mixed = mixed + torch.stack(rows)
        else:
            mixed = norm(mixed, "post_norm")             # the sandwich: a norm on the mixer's output
        h = h + mixed
        f = norm(h, "ffn_norm")
        if layer == 0:
            h = h + plain_impl.swiglu_mlp(f, {name[len(p + "mlp."):]: value for name, value in tensors.items()
                                              if name.startswith(p + "mlp.")})
        else:                                           # token by token, expert by expert
            router, up, down = (tensors[p + f"mlp.{name}.weight"].float() for name in ("router", "up", "down"))
            rows = []
            for t in range(T):
                logits = router @ f[t]
                first = int(torch.argmax(logits))
                rest = logits.clone()
                rest[first] = float("-inf")
                second = int(torch.argmax(rest))
                gate = torch.softmax(torch.stack([logits[first], logits[second]]), dim=0)
                rows.append(sum(gate[rank] * (down[expert] @ torch.relu(up[expert] @ f[t]))
                                for rank, expert in enumerate((first, second))))
            h = h + torch.stack(rows)
    h = plain_impl.rms_norm(h, tensors["model.norm.weight"], 1e-5)
    return h @ tensors["model.embed_tokens.weight"].float().T




SCHEDULES = [[(0, None), (1, None)], [(0, None), (0, None), (1, None), (1, 2)]]
SCHEDULE_IDS = ["plain-order", "layer-twice-and-shared-cache"]


def tokens_for(vocab, count, seed):
    return torch.randint(0, vocab, (count,), generator=torch.Generator().manual_seed(seed)).tolist()


def exercise(schedule, device, check_device):
    """Register the toys, build the toy model through the engine and compare whole, cut and
    mixed steps with ``toy_plain_logits``."""
    from macllm_infer_amd import Engine, Lane
    from macllm_infer_amd.weights.random_init import random_tensors
    register_toys()
    raw = {"architectures": ["ToyForTests"], "hidden": 32, "vocab": 90, "slope": 0.01, "bias": 0.3, "decay": 0.9,
           "window": 13, "experts": 5, "schedule": schedule}
    config = ToyConfig(raw)
    tensors = random_tensors(config, 5, torch.float32, "unit")
    assert "model.layers.0.decay.w.weight" in tensors and tensors["model.layers.1.mlp.up.weight"].shape == (5, 24, 32)
    assert "model.layers.1.post_norm.bias" in tensors and "model.layers.0.post_norm.weight" not in tensors
    engine = Engine(config=config, tensors=tensors, dtype="float32", device=device, kv_cache_block_tokens=4,
                    kv_cache_capacity_tokens=160, max_active_sequences=3, check_device=check_device)
    windows = sorted(str(group.need.window) for group in engine.cache.groups)
    assert windows == ["13", "None"]                                           # two groups, pages of their own
    if len(schedule) == 4:
        assert len(engine.cache.groups[0].members) == 2 and not engine.cache.entry((3, "self_attn")).owns_kv
    first, second = tokens_for(90, 70, 1), tokens_for(90, 41, 2)
    want_first, want_second = toy_plain_logits(raw, tensors, first), toy_plain_logits(raw, tensors, second)
    engine.add_request("whole")
    got = engine.step([Lane("whole", first, list(range(70)))]).cpu()
    assert (got - want_first).abs().max() < 1e-4
    engine.finish("whole")
    engine.add_request("a")
    engine.add_request("b")
    rows_a, rows_b = [], []
    rows_a.append(engine.step([Lane("a", first[:30], list(range(30)))]).cpu())
    out = engine.step([Lane("a", first[30:32], [0, 1]), Lane("b", second[:25], list(range(25)))]).cpu()
    rows_a.append(out[:2]), rows_b.append(out[2:])
    for position in range(32, 70):
        lanes = [Lane("a", first[position:position + 1], [0])]
        if position - 7 < 41:
            lanes.insert(0, Lane("b", second[position - 7:position - 6], [0]))
        out = engine.step(lanes).cpu()
        rows_a.append(out[-1:])
        if len(lanes) == 2:
            rows_b.append(out[:1])
    assert (torch.cat(rows_a) - want_first).abs().max() < 1e-4
    assert (torch.cat(rows_b) - want_second[:len(torch.cat(rows_b))]).abs().max() < 1e-4
    window_group = [group for group in engine.cache.groups if group.need.window][0]
    assert len(window_group.tables["a"].live_pages()) <= 5 < len(window_group.tables["a"].pages)   # passed pages went back
    engine.cache.check()


def toy_fast_plain_logits(raw, tensors, tokens):
    """The two one-mixer layers of ``ToyFastConfig``, whole sequence, from the plain parts."""
    T = len(tokens)
    t = {name: value.float() for name, value in tensors.items()}
    h = t["model.embed_tokens.weight"][torch.tensor(tokens)]
    sub = lambda prefix: {name[len(prefix):]: value for name, value in t.items() if name.startswith(prefix)}
    n = plain_impl.rms_norm(h, t["model.layers.0.attn_norm.weight"], 1e-5)
    h = h + plain_impl.attention_mixer(n, sub("model.layers.0.self_attn."), num_heads=2, num_kv_heads=1, head_dim=64,
                                       theta=1e4)
    h = h + plain_impl.swiglu_mlp(plain_impl.rms_norm(h, t["model.layers.0.ffn_norm.weight"], 1e-5),
                                  sub("model.layers.0.mlp."))
    p = "model.layers.1."
    n = centred_norm(h, t[p + "attn_norm.weight"], t[p + "attn_norm.bias"], 1e-4)
    projected = n @ t[p + "decay.in_proj.weight"].T
    width = raw["width"]
    s, rows = torch.zeros(width), []
    for position in range(T):
        s = raw["decay"] * s + projected[position, :width]
        rows.append(s * torch.sigmoid(projected[position, width:]))
    h = h + torch.stack(rows) @ t[p + "decay.out_proj.weight"].T
    f = centred_norm(h, t[p + "ffn_norm.weight"], t[p + "ffn_norm.bias"], 1e-4)
    h = h + routed_feed_forward(f, t[p + "mlp.router.weight"], t[p + "mlp.up.weight"], t[p + "mlp.down.weight"])
    h = plain_impl.rms_norm(h, t["model.norm.weight"], 1e-5)
    return h @ t["model.embed_tokens.weight"].T


def toy_table_plain_logits(raw, tensors, tokens):
    """The layer of ``ToyTableConfig``, run twice, whole sequence, from the plain parts."""
    T = len(tokens)
    t = {name: value.float() for name, value in tensors.items()}
    h = t["model.embed_tokens.weight"][torch.tensor(tokens)]
    sub = lambda prefix: {name[len(prefix):]: value for name, value in t.items() if name.startswith(prefix)}
    p = "model.layers.0."
    for _ in range(2):
        n = plain_impl.rms_norm(h, t[p + "attn_norm.weight"], 1e-5)
        attended = plain_impl.attention_mixer(n, sub(p + "self_attn."), num_heads=2, num_kv_heads=1, head_dim=32,
                                              theta=1e3)
        projected = n @ t[p + "decay.w.weight"].T
        s, rows = torch.zeros(raw["hidden"]), []
        for position in range(T):
            s = raw["decay"] * s + projected[position]
            rows.append(s)
        h = h + attended + torch.stack(rows)
        h = h + plain_impl.swiglu_mlp(plain_impl.rms_norm(h, t[p + "ffn_norm.weight"], 1e-5), sub(p + "mlp."))
    h = plain_impl.rms_norm(h, t["model.norm.weight"], 1e-5)
    logits = h @ t["model.embed_tokens.weight"].T * raw["logit_scale"]
    return raw["logit_cap"] * torch.tanh(logits / raw["logit_cap"])       # src/decoder.rs:3349-3355, 4791-4796


def exercise_step_table(device, check_device, graphs):
    """The toy mixer with a step table of its own: registered, built and stepped (whole, in portions beside decoded
    tokens of others, lanes in changing order), against ``toy_table_plain_logits``.  Returns the engine."""
    from macllm_infer_amd import Engine, Lane
    from macllm_infer_amd.weights.random_init import random_tensors
    register_toys()
    raw = {"architectures": ["ToyTableForTests"], "hidden": 40, "vocab": 77, "decay": 0.8, "logit_scale": 1.75,
           "logit_cap": 2.5}
    config = ToyTableConfig(raw)
    tensors = random_tensors(config, 11, torch.float32, "unit")
    engine = Engine(config=config, tensors=tensors, dtype="float32", device=device, kv_cache_block_tokens=8,
                    kv_cache_capacity_tokens=512, max_active_sequences=4, check_device=check_device,
                    decode_graphs=graphs)
    assert [table.name for table in engine.model.step_tables] == ["toy_decay_rows"]      # two runs of the layer, one table
    prompts = {name: tokens_for(77, length, seed) for seed, (name, length) in enumerate([("a", 61), ("b", 38), ("c", 50)])}
    wants = {name: toy_table_plain_logits(raw, tensors, tokens) for name, tokens in prompts.items()}
    got = {name: [] for name in prompts}
    done = {name: 0 for name in prompts}

    def run(portions):
        lanes = []
        for name, count in portions:
            lanes.append(Lane(name, prompts[name][done[name]:done[name] + count], list(range(count))))
        out = engine.step(lanes).cpu()
        row = 0
        for name, count in portions:
            got[name].append(out[row:row + count])
            done[name] += count
            row += count

    for name in prompts:
        engine.add_request(name)
    # portions of the same capacity several times over (a graph of that capacity is captured at the second), with
    # the lanes in changing order and single tokens beside them; then single tokens alone, lanes coming and going
    run([("a", 13), ("b", 1)])
    run([("b", 1), ("a", 13)])
    run([("c", 11), ("a", 2), ("b", 1)])
    run([("b", 12), ("c", 2)])
    run([("c", 1), ("b", 13)])
    run([("a", 9), ("c", 5)])
    while any(done[name] < len(prompts[name]) for name in prompts):
        order = [name for name in ("c", "a", "b") if done[name] < len(prompts[name])]
        if done["a"] % 2:
            order.reverse()
        run([(name, 1) for name in order])
    for name in prompts:
        assert (torch.cat(got[name]) - wants[name]).abs().max() < 1e-4, name
        assert 2.0 < wants[name].abs().max() < 2.5                # the cap on the logits is felt
    engine.cache.check()
    return engine
