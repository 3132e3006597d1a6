"""The sizes beyond which no kernel of a part's general path runs, as the parts report them when a
model is built: a configuration outside them is refused before any weight is read, never at the first
step.  The numbers are those of the kernels' sources (``csrc/*.hip``); a test reads them there.

The fast paths (matrix-core attention, the chunked scan, the fused decode kernels) have narrower sizes
of their own; outside those the general kernels below run, so they limit nothing.
"""
from __future__ import annotations

from dataclasses import dataclass

ATTENTION_MAX_HEAD_DIM = 256      # ATT_MAX_DH in attention.hip: a query row in LDS, head_dim / 64 sums a lane
CONV_MAX_TAPS = 16                # CONV_MAX_K in mamba2.hip: the taps of a channel in registers
SCAN_MAX_STATE = 512              # WAVE * SCAN_MAX_PER_THREAD in mamba2.hip: a state row over one wave
NORM_MAX_WIDTH = 16384            # 64 KiB of LDS hold a float32 row in common.hip's norm
GRID_MOST = 65535                 # heads, groups or lanes that index a launch's y or z dimension


@dataclass(frozen=True)
class Limit:
    """``field`` of a part's spec (or "hidden_size") is ``value``, which is more than ``most``."""
    kind: str
    field: str
    value: int
    most: int
    why: str

    def text(self, names=()) -> str:
        """``names``: ("kind.field", the configuration's own key) pairs for the message."""
        key = dict(names).get(f"{self.kind}.{self.field}", f"{self.kind} {self.field}")
        return f"'{key}' = {self.value} is more than the kernels take (at most {self.most}: {self.why})"


def beyond(kind: str, field: str, value: int, most: int, why: str):
    return [Limit(kind, field, int(value), most, why)] if value > most else []
