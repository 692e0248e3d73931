"""Position encodings.  GPT-2 adds a learned table row to the token embedding
(core/src/main/java/io/teknek/deliverance/model/gpt2/Gpt2Model.java:42-48) and does nothing
to queries and keys (its rotary step is skipped: core/.../generator/CausalSelfAttention.java:341)."""
from __future__ import annotations

from .base import PositionEncoding, register_position, to_vector


class LearnedPositions(PositionEncoding):
    def __init__(self, spec, params, dtype, device):
        self.max_positions = spec.max_positions
        self.table = to_vector(params["table"], dtype, device)
        if self.table.shape[0] != self.max_positions:
            raise ValueError(f"position table has {self.table.shape[0]} rows, config says {self.max_positions}")

    def embed_table(self):
        return self.table


class NoPositions(PositionEncoding):
    def __init__(self, spec=None, params=None, dtype=None, device=None):
        pass


register_position("learned", LearnedPositions)
register_position("none", NoPositions)
