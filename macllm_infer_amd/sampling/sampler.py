"""Sampling on the GPU over rows of float32 logits.

Order of operations, as the reference's sampler (src/sampling.rs:95-161): repetition
penalty over prompt and generated tokens, presence and frequency penalties over generated
tokens, then the request's constraint if it has one (only the allowed tokens keep their logits), then
argmax (lowest index on ties) or temperature -> top-k -> softmax -> top-p ->
one uniform draw, walked in index order.  One draw per stochastic token; the uniform
comes from a counter-based generator keyed by (seed, number of tokens drawn so far), so a
request's tokens do not depend on what else is in the batch.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import numpy as np
import torch

from ..kernels import build as kernel_build
from ..kernels import ops
from .params import SamplingParams


class SamplerRow:
    """What the sampler needs to know of one request.  ``newest``: (int32 tensor on the device, row) of a token
    already drawn for the request that ``generated`` does not hold yet; it counts for the draw's index and,
    read on the device, for the penalties."""
    __slots__ = ("params", "prompt", "generated", "newest", "allowed")

    def __init__(self, params: SamplingParams, prompt: Sequence[int], generated: Sequence[int],
                 newest: Optional[tuple] = None):
        self.params, self.prompt, self.generated, self.newest = params, prompt, generated, newest
        if newest is not None and params.constrained_by_history:
            raise ValueError("a constraint that reads the generated tokens needs them all on the host")
        self.allowed = params.allowed_after(generated)          # the tokens that may come now, or None for any

    @property
    def pending(self) -> int:
        return 0 if self.newest is None else 1


class PendingTokens:
    """The tokens of one ``sample_async`` call: on the device at once (``device``, int32 [B], what a next
    step may be fed from), on the host after ``wait()``."""

    def __init__(self, device: torch.Tensor, host: torch.Tensor, event):
        self.device, self._host, self._event = device, host, event

    def wait(self) -> List[int]:
        if self._event is not None:
            self._event.synchronize()
        return self._host[:self.device.numel()].tolist()


class Sampler:
    kernel_modules = ("sampling",)

    def __init__(self, vocab_size: int, device, check_device: bool = True):
        self.vocab_size = vocab_size
        self.device = torch.device(device)
        self.padded = 1
        while self.padded < vocab_size:
            self.padded <<= 1
        if check_device:
            ops.require_gpu(device)
            kernel_build.ensure_modules(self.kernel_modules)
        self._keys = None
        self._counts = None
        self._host_tokens: List[torch.Tensor] = []      # pinned, used in turn by the calls in flight
        self._turn = 0

    def _work(self, rows: int):
        if self._keys is None or self._keys.shape[0] < rows:
            self._keys = torch.empty((rows, self.padded), dtype=torch.int64, device=self.device)
        return self._keys

    def _count_areas(self, rows: int):
        if self._counts is None or self._counts[0].numel() < rows * self.vocab_size:
            self._counts = (torch.zeros(rows * self.vocab_size, dtype=torch.int32, device=self.device),
                            torch.zeros(rows * self.vocab_size, dtype=torch.int32, device=self.device))
        return self._counts

    HOST_BUFFERS = 3               # calls whose tokens nobody has waited for yet, at most

    def sample(self, logits: torch.Tensor, rows: Sequence[SamplerRow]) -> List[int]:
        """One token for each row of ``logits`` [B, V] (float32; overwritten)."""
        return self.sample_async(logits, rows).wait()

    def sample_async(self, logits: torch.Tensor, rows: Sequence[SamplerRow]) -> PendingTokens:
        """The same, without waiting: the kernels and the copy of the tokens to the host are queued, and the
        caller waits for them when it needs them (at most HOST_BUFFERS - 1 calls later)."""
        B = len(rows)
        if logits.shape != (B, self.vocab_size):
            raise ValueError(f"logits have shape {tuple(logits.shape)}, expected {(B, self.vocab_size)}")
        device = self.device

        if any(row.params.uses_penalties for row in rows):
            newest = [row for row in rows if row.newest is not None and row.params.uses_penalties]
            if any(row.newest[0] is not newest[0].newest[0] for row in newest):
                raise ValueError("the newest tokens of a call's rows must lie in one tensor")
            tokens: List[int] = []
            offsets = [0]
            for row in rows:
                if row.params.uses_penalties:
                    tokens.extend(row.prompt)
                    tokens.extend(row.generated)
                offsets.append(len(tokens))
            count_all, count_gen = self._count_areas(B)
            # one upload: offsets (B+1) | prompt lengths | the three penalties (float bits) | rows of the newest
            # tokens on the device | the histories
            head = 6 * B + 1
            words = np.empty(head + max(len(tokens), 1), dtype=np.int32)
            words[:B + 1] = offsets
            words[B + 1:2 * B + 1] = [len(row.prompt) for row in rows]
            words[2 * B + 1:3 * B + 1].view(np.float32)[:] = [row.params.repetition_penalty for row in rows]
            words[3 * B + 1:4 * B + 1].view(np.float32)[:] = [row.params.presence_penalty for row in rows]
            words[4 * B + 1:5 * B + 1].view(np.float32)[:] = [row.params.frequency_penalty for row in rows]
            words[5 * B + 1:head] = [row.newest[1] if row.newest is not None and row.params.uses_penalties else -1
                                     for row in rows]
            words[head:] = tokens or [0]
            packed = torch.from_numpy(words).to(device, non_blocking=True)
            ops.apply_penalties(
                logits, packed[head:], packed[:B + 1], packed[B + 1:2 * B + 1],
                packed[2 * B + 1:3 * B + 1].view(torch.float32), packed[3 * B + 1:4 * B + 1].view(torch.float32),
                packed[4 * B + 1:5 * B + 1].view(torch.float32), count_all, count_gen,
                newest[0].newest[0] if newest else None, packed[5 * B + 1:head] if newest else None)
        if any(row.allowed is not None for row in rows):
            # after the penalties, before the choice (src/sampling.rs:119-130): one upload, offsets then ids
            offsets = [0]
            ids: List[int] = []
            for row in rows:
                if row.allowed is not None:
                    if max(row.allowed) >= self.vocab_size:
                        raise ValueError(f"allowed token {max(row.allowed)} is outside the vocabulary of {self.vocab_size}")
                    ids.extend(row.allowed)
                offsets.append(len(ids))
            words = np.asarray(offsets + ids, dtype=np.int32)
            packed = torch.from_numpy(words).to(device, non_blocking=True)
            ops.keep_allowed(logits, packed[B + 1:], packed[:B + 1], self._work(B))
        out = torch.empty(B, dtype=torch.int32, device=device)
        if all(row.params.greedy for row in rows):
            ops.argmax(logits, out)
        else:
            # one upload for the five parameter arrays: seeds (int64) first, then 32-bit words
            words = np.empty(6 * B, dtype=np.int32)
            words[:2 * B].view(np.uint64)[:] = [row.params.seed & ((1 << 64) - 1) for row in rows]
            words[2 * B:3 * B].view(np.float32)[:] = [row.params.temperature for row in rows]
            words[3 * B:4 * B].view(np.float32)[:] = [row.params.top_p for row in rows]
            words[4 * B:5 * B] = [row.params.top_k for row in rows]
            words[5 * B:] = [len(row.generated) + row.pending for row in rows]
            packed = torch.from_numpy(words).to(device, non_blocking=True)
            ops.sample(logits, packed[2 * B:3 * B].view(torch.float32), packed[4 * B:5 * B],
                       packed[3 * B:4 * B].view(torch.float32), packed[:2 * B].view(torch.int64), packed[5 * B:],
                       self._work(B), out, torch.empty(B, dtype=torch.int32, device=device))
        if self.device.type != "cuda":                 # host-side tests: nothing is in flight
            return PendingTokens(out, out, None)
        # the buffers are used strictly in turn: call n writes buffer n % HOST_BUFFERS, so a call's tokens stay
        # readable until HOST_BUFFERS - 1 further calls have been made
        turn = self._turn
        self._turn = (turn + 1) % self.HOST_BUFFERS
        if len(self._host_tokens) <= turn:
            self._host_tokens.append(torch.empty(max(B, 64), dtype=torch.int32, pin_memory=True))
        if self._host_tokens[turn].numel() < B:
            self._host_tokens[turn] = torch.empty(B, dtype=torch.int32, pin_memory=True)
        host = self._host_tokens[turn]
        host[:B].copy_(out, non_blocking=True)
        event = torch.cuda.Event()
        event.record()
        return PendingTokens(out, host, event)
