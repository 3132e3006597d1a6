"""The decoder model: embedding, the layers in the order the schedule gives, final norm
and output projection, put together from registered parts according to a ``ModelSpec``.
(reference: src/decoder.rs:2980-3105 load, :3146-3358 packed forward.)
"""
from __future__ import annotations

from typing import Dict, Hashable, List

import torch

from ..config.spec import ModelSpec
from ..kernels import ops
from ..parts.base import BuildContext, Residual, part_class
from ..parts.block import arrangement_class
from ..weights.loader import Expect


# Up to this many wanted rows the output head streams through the skinny kernel (the norm as a kernel of its own
# before it), beyond through the library: a 130,049 x 3,072 head takes 138 / 144 / 159 / 203 us at 1 / 4 / 8 / 16 rows
# against the library's 147 / 152 / 155 / 160, a 32,784 x 1,024 one 22 to 24 against 25 to 26.  (The norm in the skinny
# kernel's prologue, every workgroup normalizing the rows again, took 305 to 370 us on the first and 23 to 39 on the
# second, and 1,333 on a 261,120 x 5,120 head that streams in 450.)
HEAD_SKINNY_ROWS = 8


class DecoderModel:
    @staticmethod
    def expected_tensors(spec: ModelSpec) -> List[Expect]:
        """Every tensor the model binds, by exact name with its shape
        (name tables: src/architecture.rs:1595-1647)."""
        out = [Expect(f"{spec.embedding_name}.weight", ((spec.vocab_size, spec.hidden_size),), init="embedding")]
        for layer in spec.layers:
            out += arrangement_class(layer.arrangement).expected_tensors(layer, spec.hidden_size)
        out += part_class(spec.final_norm).expected_tensors(spec.final_norm, spec.final_norm_name, spec.hidden_size)
        if not spec.tied_embeddings:
            out.append(Expect(f"{spec.lm_head_name}.weight", ((spec.vocab_size, spec.hidden_size),)))
        return out

    @staticmethod
    def tensor_copies(spec: ModelSpec) -> Dict[str, str]:
        """Tensors a checkpoint may hold although the model binds another one in their place, if both are
        equal: a tied model saved with its output head written out beside the embedding."""
        if spec.tied_embeddings:
            return {f"{spec.lm_head_name}.weight": f"{spec.embedding_name}.weight"}
        return {}

    @staticmethod
    def limits(spec: ModelSpec) -> list:
        """Every size of the model that some part's kernels refuse, each once (``kernels.limits.Limit``)."""
        found = list(part_class(spec.final_norm).limits(spec.final_norm, spec.hidden_size))
        for layer in spec.layers:
            arrangement = arrangement_class(layer.arrangement)
            if hasattr(arrangement, "limits"):
                found += arrangement.limits(layer, spec.hidden_size)
        return list(dict.fromkeys(found))

    @staticmethod
    def kernel_modules(spec: ModelSpec) -> List[str]:
        modules = ["common", "gemm"]
        for layer in spec.layers:
            modules += arrangement_class(layer.arrangement).kernel_modules(layer)
        return list(dict.fromkeys(modules))

    @staticmethod
    def cache_layout(spec: ModelSpec):
        """(needs, shared): (entry, mixer name) -> that mixer's cache needs, and which
        (entry, mixer) reads the K/V of which earlier one."""
        needs: Dict[Hashable, list] = {}
        shared: Dict[Hashable, Hashable] = {}
        for index, entry in enumerate(spec.schedule):
            layer = spec.layers[entry.layer]
            for slot in layer.mixers:
                key = (index, slot.name)
                needs[key] = list(part_class(slot.spec).cache_needs(slot.spec))
                if entry.kv_from is not None and any(getattr(need, "token_proportional", False) for need in needs[key]):
                    shared[key] = (entry.kv_from, slot.name)
        return needs, shared

    def __init__(self, spec: ModelSpec, tensors: Dict[str, torch.Tensor], build: BuildContext):
        spec.validate()
        self.spec = spec
        self.build = build
        table = tensors[f"{spec.embedding_name}.weight"]
        if build.dtype == torch.float32:
            table = table.to(torch.float32)
        self.embedding = table.contiguous().to(build.device)
        self.blocks = [arrangement_class(layer.arrangement)(layer, tensors, build) for layer in spec.layers]
        for block in self.blocks:                    # what a layer decides by timing itself among the others
            tune = getattr(block, "tune", None)
            if tune is not None:
                tune(self.blocks)
        self.final_norm = part_class(spec.final_norm)(spec.final_norm, spec.final_norm_name, tensors, build)
        if spec.tied_embeddings:
            self.lm_head = self.embedding
        else:
            head = tensors[f"{spec.lm_head_name}.weight"]
            if build.dtype == torch.float32:
                head = head.to(torch.float32)
            self.lm_head = head.contiguous().to(build.device)
        # the copy of the head that the skinny kernel streams fastest, for steps that want few rows
        fused_head = (build.device.type == "cuda" and build.dtype == torch.bfloat16 and self.lm_head.dtype == torch.bfloat16
                      and spec.hidden_size % 32 == 0 and ops.fused_gemm_supported(False, 1, spec.hidden_size))
        self._head_fragments = ops.fragment_order(self.lm_head) if fused_head else None
        # the final norm's (weight, eps), if it is a root-mean-square norm: the last layer may prepare the stream for it
        prologue = getattr(self.final_norm, "rms_prologue", None)
        self._final_rms = prologue() if prologue is not None else None
        # for every scheduled layer the (weight, eps) of the norm that follows it, where that is a root-mean-square
        # norm: a layer may then hand the stream over prepared for it
        def rms_of(norm):
            prologue = getattr(norm, "rms_prologue", None)
            return prologue() if prologue is not None else None

        firsts = [rms_of(getattr(self.blocks[entry.layer], "first_norm", None)) for entry in spec.schedule]
        self._next_norms = firsts[1:] + [self._final_rms]
        # the step's table of runs of one lane's tokens is cut for the mixer with the largest tile
        mixers = [mixer for block in self.blocks for _, mixer in block.mixers]
        self.query_tile = max((getattr(mixer, "query_tile", 0) for mixer in mixers), default=0)
        # and its tables of chunks for the chunk sizes the mixers name
        self.chunk_sizes = tuple(sorted({getattr(mixer, "chunk_tokens", 0) for mixer in mixers} - {0}))
        # and the tables the mixers declare themselves; one name is one table, whichever layers read it
        declared = {}
        for mixer in mixers:
            for table in (mixer.step_tables() if hasattr(mixer, "step_tables") else ()):
                declared.setdefault(table.name, table)
        self.step_tables = tuple(declared.values())

    @property
    def step_layout(self) -> dict:
        """What the step's index arrays hold beyond the lanes themselves, as the arguments of
        ``build_step_context`` and ``StaticStep``."""
        return dict(query_tile=self.query_tile, chunk_sizes=self.chunk_sizes, tables=self.step_tables)

    @property
    def graph_safe(self) -> bool:
        return all(block.graph_safe for block in self.blocks) and getattr(self.final_norm, "graph_safe", False)

    def forward(self, step, cache) -> torch.Tensor:
        """Run the step's tokens through every scheduled layer and return float32 logits
        [wanted, vocab] at ``step.want_rows`` (empty tensor when nothing is wanted)."""
        spec = self.spec
        h = torch.empty((step.num_tokens, spec.hidden_size), dtype=torch.float32, device=self.build.device)
        ops.embed(step.token_ids, self.embedding, spec.embedding_multiplier, h)
        residual = Residual(h)
        for index, entry in enumerate(spec.schedule):
            block = self.blocks[entry.layer]
            caches = {name: cache.entry((index, name)) for name, _ in block.mixers}
            residual.next_norm = self._next_norms[index]
            block.forward(residual, step, caches)
        wanted = step.want_rows.numel()
        if wanted == 0:
            return torch.empty((0, spec.vocab_size), dtype=torch.float32, device=self.build.device)
        logits = torch.empty((wanted, spec.vocab_size), dtype=torch.float32, device=self.build.device)
        scaled = residual.scaled
        if (self._head_fragments is not None and scaled is not None and self._final_rms is not None
                and scaled.weight is self._final_rms[0] and not residual.pending and self._every_row_wanted(step, wanted)):
            # the last layer left the rows times the norm's weight and their sums of squares: projection, the
            # norm's division and the scaling of the logits in one launch
            ops.fused_gemm(self.lm_head, None, logits, out_scale=spec.logit_multiplier, x=scaled.rows,
                           row_scale=ops.RowScale(scaled.ssq, spec.hidden_size, self._final_rms[1]),
                           fragments=self._head_fragments)
            return self._capped(logits)
        normed = self.final_norm.forward(residual, rows=step.want_rows)
        if self._head_fragments is not None and wanted <= HEAD_SKINNY_ROWS:
            ops.fused_gemm(self.lm_head, None, logits, out_scale=spec.logit_multiplier, x=normed,
                           fragments=self._head_fragments)
            return self._capped(logits)
        raw = ops.linear(normed, self.lm_head, None, keep_float32=True)      # the sums as they are, not rounded to bfloat16
        ops.scale_to_f32(raw, spec.logit_multiplier, logits)
        return self._capped(logits)

    def _capped(self, logits: torch.Tensor) -> torch.Tensor:
        if self.spec.logit_softcap is not None:
            ops.tanh_softcap(logits, self.spec.logit_softcap)
        return logits

    @staticmethod
    def _every_row_wanted(step, wanted: int) -> bool:
        """A step of single tokens that wants the logits of each: the wanted rows are the step's rows."""
        return (step.max_query_len == 1 and wanted == step.num_tokens and wanted <= HEAD_SKINNY_ROWS
                and len(step.lane_lengths) == wanted)
