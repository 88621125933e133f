"""What a model may do to its token embeddings before the first layer, or to its logits after the head
(ModelSpec.embed_post / logits_post): a class of STREAM_OPS with `forward(x, rows)`, in place on the first rows
of x ([rows, width]: the stream in the engine's dtype, or the float32 logits). The architecture of this
repository uses neither; a multiplied embedding or softly capped logits are a matter of the spec, not of
DecoderModel.
"""
from __future__ import annotations

from ..kernels import ops
from .base import Part
from .registry import STREAM_OPS
from .spec import TensorSpec


@STREAM_OPS.register("scale_softcap")
class ScaleSoftcap(Part):
    """x *= scale, then x = softcap * tanh(x / softcap) where a cap is given. No tensors."""

    def __init__(self, width: int, scale: float = 1.0, softcap: float | None = None):
        if softcap is not None and not softcap > 0:
            raise ValueError(f"softcap must be positive, got {softcap}")
        self.width, self.scale, self.softcap = width, float(scale), softcap

    def forward(self, x, rows: int) -> None:
        ops.scale_softcap(x, rows, self.scale, self.softcap)


@STREAM_OPS.register("pass_start")
class PassStart(Part):
    """What a model that runs a group of its layers several times adds to the stream at the start of a pass
    (RunEntry.before): x += embeddings (where `add_embedding`: the token embeddings as they first entered the stream)
    + table[row], with `table` [rows, width] a tensor of the weight file."""

    def __init__(self, width: int, table: str, rows: int, row: int, add_embedding: bool = False):
        if not 0 <= row < rows:
            raise ValueError(f"pass_start: row {row} of a table of {rows}")
        self.width, self.table, self.rows, self.row = width, table, rows, row
        self.needs_embedding = bool(add_embedding)
        self.vec = None

    def tensors(self):
        return {self.table: TensorSpec((self.rows, self.width))}

    def load(self, get):
        self.vec = get(self.table).float()[self.row].contiguous()

    def forward(self, x, rows: int, embedding=None) -> None:
        if self.needs_embedding and embedding is None:
            raise RuntimeError("pass_start: the model kept no embeddings to add")
        ops.add_rows(x, rows, a=embedding if self.needs_embedding else None, vec=self.vec)
