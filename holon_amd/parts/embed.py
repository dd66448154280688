"""Token embedding and the output head. std/holon_std/ops/units.py:280-348 (`Embedding`, `LMHead`)."""
from __future__ import annotations

import torch

from ..registry import register_part
from ..spec import PartRef
from .base import Build, EmbedPart, Part


@register_part("embed", "table")
class Embedding(EmbedPart):
    """Rows of a table. With `norm` (any registered norm whose `forward` takes `out_dtype`) the rows go through it
    and come out in float32: the start of a residual stream that is kept in 32-bit. With `scale` the rows are
    multiplied by it, in float32, and come out in float32 as well."""

    graph_safe = True

    def __init__(self, build: Build, *, vocab: int, hidden: int, norm: PartRef | None = None,
                 scale: float | None = None) -> None:
        super().__init__(build)
        self.declare("weight", (vocab, hidden))
        self.scale = None if scale is None else float(scale)
        if self.scale is not None and norm is not None:
            raise ValueError("embed table: either a norm or a scale")
        self.norm = None
        if norm is not None:
            self.attach("norm", build.make(norm, dim=hidden))

    def rows(self, ids: torch.Tensor) -> torch.Tensor:
        return self.kernels.embedding(ids, self.weight)

    def forward(self, ids: torch.Tensor, take: tuple[torch.Tensor, torch.Tensor] | None = None,
                want_stats: bool = False):
        """Rows of the table; `take`: where a token is still on the device, see the kernel contract. With
        `want_stats`: (rows, their statistics for a norm that follows, or None)."""
        if self.scale is not None:
            rows = self.kernels.scale_rows(self.kernels.embedding(ids, self.weight, take, False), self.scale)
            return (rows, None) if want_stats else rows
        if self.norm is None:
            return self.kernels.embedding(ids, self.weight, take, want_stats)
        rows = self.norm(self.kernels.embedding(ids, self.weight, take, False), out_dtype=torch.float32)
        return (rows, None) if want_stats else rows

    __call__ = forward


@register_part("head", "linear")
class LMHead(Part):
    """Logits in float32, optionally squashed into (-softcap, softcap). A tied head owns no tensor: it reads the
    embedding's."""

    graph_safe = True

    def __init__(self, build: Build, *, vocab: int, hidden: int, tied: bool, embed: Embedding,
                 softcap: float | None = None) -> None:
        super().__init__(build)
        self.tied = tied
        self.softcap = float(softcap) if softcap else None      # logits <- cap * tanh(logits / cap)
        self._embed = [embed]                     # in a list: the embedding part keeps the one owner of the tensor
        self.tiled: torch.Tensor | None = None
        if not tied:
            self.declare("weight", (vocab, hidden))

    def _weight(self) -> torch.Tensor:
        return self._embed[0].weight if self.tied else self.weight

    def finalize(self) -> None:
        if self.build.decode_copy and self._weight() is not None:
            self.tiled = self.kernels.tile_weight(self._weight())

    def extra_tensors(self) -> list[torch.Tensor]:
        return [self.tiled] if self.tiled is not None else []

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        logits = self.kernels.linear(h, self._weight(), torch.float32, self.tiled)
        return logits if self.softcap is None else self.kernels.softcap(logits, self.softcap)

    __call__ = forward
