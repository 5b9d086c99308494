"""Token embedding and the output projection.

Embedding: x[t, :] = E[id_t, :] (/root/reference/src/models/embedding.cpp:54-76; an
id outside [0, V) is an error there and here).  Output: logits = xn E^T with the
embedding table when tied (/root/reference/src/models/embedding.cpp:78-81,
src/models/gpt_model.cpp:328); the reference always ties; here `tied=False`
uses a separate `lm_head.weight` [V, H].  Logits come out in float32.
"""
from __future__ import annotations

import torch

from .. import kernels
from .base import Embedding, OutputHead, register_part
from .spec import ParamSpec


class TokenEmbedding(Embedding):
    graph_safe = True

    def __init__(self, prefix: str, hidden_size: int, vocab_size: int, name: str = "weight"):
        self.prefix = prefix
        self.hidden_size = int(hidden_size)
        self.vocab_size = int(vocab_size)
        self.name = name                   # the table is the tensor `prefix + name`
        self.table: torch.Tensor | None = None

    def param_specs(self):
        return [ParamSpec(self.prefix + self.name, (self.vocab_size, self.hidden_size), role="embedding")]

    def load(self, get, dtype, device):
        self.table = self._to(get(self.prefix + self.name), "compute", dtype, device)

    def output_matrix(self) -> torch.Tensor:
        return self.table

    def forward(self, ctx) -> torch.Tensor:
        k = kernels.backend()
        token_ids = ctx.token_ids
        out = torch.empty((token_ids.shape[0], self.hidden_size), device=token_ids.device,
                          dtype=k.residual_dtype(token_ids.shape[0], self.table.dtype))     # the residual stream
        k.embed(token_ids, self.table, out)
        return out


class NormedTokenEmbedding(TokenEmbedding):
    """x[t, :] = N(E[id_t, :]) with an RMS norm that has one gain for all coordinates (the tensor `prefix + norm_name`):
    gather, statistics and the product with the gain in one kernel, in float32, written as the residual stream (of the
    kind that the backend names for the step's size)."""

    def __init__(self, prefix: str, hidden_size: int, vocab_size: int, eps: float, name: str = "weight",
                 norm_name: str = "norm"):
        super().__init__(prefix, hidden_size, vocab_size, name)
        self.eps = float(eps)
        self.norm_name = norm_name
        self.gain: torch.Tensor | None = None

    def param_specs(self):
        return super().param_specs() + [ParamSpec(self.prefix + self.norm_name, (), role="norm_scale", alt_shapes=((1,),))]

    def load(self, get, dtype, device):
        super().load(get, dtype, device)
        gain = get(self.prefix + self.norm_name).reshape(1).to(dtype)
        self.gain = gain.expand(self.hidden_size).to(device).contiguous()

    def forward(self, ctx) -> torch.Tensor:
        k = kernels.backend()
        token_ids = ctx.token_ids
        out = torch.empty((token_ids.shape[0], self.hidden_size), device=token_ids.device,
                          dtype=k.residual_dtype(token_ids.shape[0], self.table.dtype))
        k.embed_rmsnorm(token_ids, self.table, self.gain, self.eps, out)
        return out


class ScaledTokenEmbedding(TokenEmbedding):
    """x[t, :] = E[id_t, :] * scale, written as a float32 residual stream (the parts of a design that norms with a mean
    read the stream in float32)."""

    def __init__(self, prefix: str, hidden_size: int, vocab_size: int, scale: float, name: str = "weight"):
        super().__init__(prefix, hidden_size, vocab_size, name)
        self.scale = float(scale)

    def forward(self, ctx) -> torch.Tensor:
        token_ids = ctx.token_ids
        out = torch.empty((token_ids.shape[0], self.hidden_size), device=token_ids.device, dtype=torch.float32)
        kernels.backend().embed_scaled(token_ids, self.table, self.scale, out)
        return out


class PositionedTokenEmbedding(TokenEmbedding):
    """x[t, :] = E[id_t, :] + P[position_t, :] with a learned vector per position (the tensor `prefix + position_name`,
    [max_positions, H]), added in float32 and written as a float32 residual stream.  A request cannot grow beyond the
    table's rows (the model's `max_position`)."""

    def __init__(self, prefix: str, hidden_size: int, vocab_size: int, max_positions: int, name: str = "weight",
                 position_name: str = "pos"):
        super().__init__(prefix, hidden_size, vocab_size, name)
        self.max_positions = int(max_positions)
        self.position_name = position_name
        self.position_table: torch.Tensor | None = None

    def param_specs(self):
        return super().param_specs() + [ParamSpec(self.prefix + self.position_name, (self.max_positions, self.hidden_size),
                                                  role="embedding")]

    def load(self, get, dtype, device):
        super().load(get, dtype, device)
        self.position_table = self._to(get(self.prefix + self.position_name), "compute", dtype, device)

    def forward(self, ctx) -> torch.Tensor:
        token_ids = ctx.token_ids
        out = torch.empty((token_ids.shape[0], self.hidden_size), device=token_ids.device, dtype=torch.float32)
        kernels.backend().embed_positions(token_ids, ctx.positions, self.table, self.position_table, out)
        return out


class LinearHead(OutputHead):
    graph_safe = True

    def __init__(self, prefix: str, hidden_size: int, vocab_size: int, tied: bool, name: str = "weight",
                 softcap: float | None = None, scale: float | None = None):
        """scale s: logits <- s * logits; softcap c: then logits <- c * tanh(logits / c) (None: not)."""
        self.softcap = float(softcap) if softcap else None
        self.scale = float(scale) if scale is not None and float(scale) != 1.0 else None
        self.prefix = prefix
        self.hidden_size = int(hidden_size)
        self.vocab_size = int(vocab_size)
        self.tied = bool(tied)
        self.name = name                   # the matrix is the tensor `prefix + name`
        self.weight: torch.Tensor | None = None

    def param_specs(self):
        if self.tied:
            return []
        return [ParamSpec(self.prefix + self.name, (self.vocab_size, self.hidden_size))]

    def load(self, get, dtype, device):
        if not self.tied:
            self.weight = self._to(get(self.prefix + self.name), "compute", dtype, device)

    def tie(self, matrix: torch.Tensor) -> None:
        if tuple(matrix.shape) != (self.vocab_size, self.hidden_size):
            raise ValueError(f"a tied output head needs a [{self.vocab_size}, {self.hidden_size}] matrix, "
                             f"got {tuple(matrix.shape)}")
        self.weight = matrix

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        out = torch.empty((x.shape[0], self.vocab_size), dtype=torch.float32, device=x.device)
        kernels.backend().linear(x, self.weight, None, out)
        if self.softcap is not None or self.scale is not None:
            kernels.backend().tanh_cap(out, self.softcap, scale=1.0 if self.scale is None else self.scale)
        return out


register_part("embedding", "token_embedding", TokenEmbedding)
register_part("embedding", "token_embedding_normed", NormedTokenEmbedding)
register_part("embedding", "token_embedding_scaled", ScaledTokenEmbedding)
register_part("embedding", "token_embedding_positions", PositionedTokenEmbedding)
register_part("output_head", "linear_head", LinearHead)
