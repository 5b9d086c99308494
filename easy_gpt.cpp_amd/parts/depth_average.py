"""What goes on to the next layer as a learned weighted sum over the depth.

With X_0 the embedding's output and X_(i+1) the result of the i-th entry of the run order, the entry after it (or the
final norm) reads sum_(j <= i+1) a[j] * X_j, where a is that entry's own tensor of i + 2 weights.  Every X_j of a step
is kept, in float32 [entries + 1, T, H] (`ctx.shared`), until the step ends; the sum is float32.  The arrangement
hands the layer's last addition to `join`, whose kernel stores X_(i+1) beside the others and writes the weighted sum
in the same pass.
"""
from __future__ import annotations

import torch

from .base import StreamJoin, register_part
from .spec import ParamSpec

_KEY = "depth_average.results"


class DepthAverage(StreamJoin):
    graph_safe = True

    def __init__(self, prefix: str, hidden_size: int, index: int, total: int, name: str = "dwa"):
        """index: which result of the depth this layer's is (1 for the first entry of the run order; 0 is the
        embedding's output); total: how many results a step keeps (the run order's entries + 1)."""
        if not 1 <= int(index) < int(total):
            raise ValueError(f"a depth average at result {index} needs 1 <= index < total ({total})")
        self.prefix, self.hidden_size = prefix, int(hidden_size)
        self.index, self.total, self.name = int(index), int(total), name
        self.weights: torch.Tensor | None = None

    def param_specs(self):
        return [ParamSpec(self.prefix + self.name, (self.index + 1,), role="mean_weights", dtype="float32")]

    def load(self, get, dtype, device):
        self.weights = get(self.prefix + self.name).to(torch.float32).to(device).contiguous()

    def results(self, ctx, h: torch.Tensor) -> torch.Tensor:
        """The step's results so far, float32 [total, T, H].  The first layer's join makes the tensor and puts the stream
        that the layer was given (the embedding's output) in as result 0."""
        kept = ctx.shared.get(_KEY)
        if kept is None:
            if self.index != 1:
                raise RuntimeError("the first entry of the run order must be the first to join the depth's results")
            kept = torch.empty((self.total, *h.shape), dtype=torch.float32, device=h.device)
            kept[0].copy_(h)
            ctx.shared[_KEY] = kept
        return kept


register_part("stream_join", "depth_average", DepthAverage)
