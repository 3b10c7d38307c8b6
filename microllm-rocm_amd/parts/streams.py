"""The residual stream in several copies (hyper-connections), the norm that reads them, and an embedding that adds a
sinusoidal position vector.

A token has ``S`` rows ``x_0 .. x_(S-1)`` instead of one, all equal to the embedding's output at the start. A sublayer
with connection weights ``take [S]``, ``mix [S, S]`` (indexed from, to) and ``give [S]`` reads ``u = sum_s take[s] x_s``,
computes ``y = sublayer(norm(u))``, and every stream becomes ``x_t <- sum_s mix[s, t] x_s + give[t] y``, all from the
old rows. The model's result is the sum of the streams. As a block with one stream hands its last delta on to the
norm that follows, a block here hands on a ``StreamDelta`` (the sublayer's result with its connection's ``mix`` and
``give``): the write, the next read and the next norm are one kernel.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Mapping, Optional

import torch

from ..ops import kernels
from .base import MATRIX, Norm, Part, Runtime, TensorDecl, VECTOR
from .block import Block, register_arrangement
from .registry import register_part
from .spec import PartSpec


@dataclass
class StreamDelta:
    """A sublayer's result that is still to be written into the streams: ``values`` is float32 ``[tokens, width]`` or
    partial sums ``[parts, tokens, width]``; ``mix`` and ``give`` are the connection's (None: identity and ones)."""
    values: torch.Tensor
    mix: Optional[torch.Tensor] = None
    give: Optional[torch.Tensor] = None


class StreamNorm(Norm):
    """Layer norm with a weight and no bias, ``(u - mean) / sqrt(var + eps) * w`` with the variance as the mean of the
    squared deviations (``rms``: ``u / sqrt(mean(u^2) + eps) * w``), over a stream of one or several copies: ``h`` is
    ``[tokens, width]`` or ``[tokens, streams, width]``, ``delta`` a tensor, partial sums or a ``StreamDelta``, and
    ``take`` the weights of the read (None: the plain sum of the streams)."""
    graph_safe = True

    def __init__(self, spec: PartSpec, runtime: Runtime):
        super().__init__(spec, runtime)
        self.size = int(spec.params["size"])
        self.eps = float(spec.params["eps"])
        self.rms = bool(spec.params.get("rms", False))
        self.weight: Optional[torch.Tensor] = None

    def tensors(self) -> Dict[str, TensorDecl]:
        return {self.name("weight"): TensorDecl((self.size,), VECTOR)}

    def bind(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.weight = tensors[self.name("weight")]

    def forward(self, h, delta=None, write_h=True, rows=None, take=None):
        mix = give = None
        if isinstance(delta, StreamDelta):
            delta, mix, give = delta.values, delta.mix, delta.give
        return kernels.stream_norm(h, self.weight, self.eps, self.runtime.dtype, rms=self.rms, delta=delta, mix=mix,
                                   give=give, take=take, rows=rows,
                                   write_x=write_h and delta is not None and rows is None)


class HyperConnection(Part):
    """The three weights that join one sublayer to the streams."""
    category = "connection"
    graph_safe = True

    def __init__(self, spec: PartSpec, runtime: Runtime):
        super().__init__(spec, runtime)
        self.streams = int(spec.params["streams"])
        self.take: Optional[torch.Tensor] = None
        self.give: Optional[torch.Tensor] = None
        self.mix: Optional[torch.Tensor] = None

    def tensors(self) -> Dict[str, TensorDecl]:
        return {self.name("in"): TensorDecl((self.streams,), VECTOR), self.name("out"): TensorDecl((self.streams,), VECTOR),
                self.name("mix"): TensorDecl((self.streams, self.streams), VECTOR)}

    def bind(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.take, self.give, self.mix = tensors[self.name("in")], tensors[self.name("out")], tensors[self.name("mix")]


class HyperConnectionBlock(Block):
    """Pre-norm sublayers joined to several streams. ``LayerSpec.extra`` names the connections: ``mixer_connection``
    and, with a feed-forward, ``ffn_connection`` (category ``connection``)."""

    def forward(self, h, pending, ctx, cache, next_block=None):
        joint = self.extra["mixer_connection"]
        x = self.mixer_norm.forward(h, delta=pending, write_h=True, take=joint.take)
        pending = StreamDelta(self.mixer.forward(x, ctx, cache), joint.mix, joint.give)
        if self.ffn is not None:
            joint = self.extra["ffn_connection"]
            x = self.ffn_norm.forward(h, delta=pending, write_h=True, take=joint.take)
            pending = StreamDelta(self.ffn.forward(x, ctx), joint.mix, joint.give)
        return pending


class SinusoidTokenEmbedding(Part):
    """``h0[t] = E[id_t] + w(p_t)`` in float32, with ``w(p)[2i] = sin(p * base^(-2i / width))`` and ``w(p)[2i + 1]``
    the cosine of the same angle."""
    category = "embedding"
    graph_safe = True

    def __init__(self, spec: PartSpec, runtime: Runtime):
        super().__init__(spec, runtime)
        self.vocab = int(spec.params["vocab_size"])
        self.width = int(spec.params["hidden_size"])
        self.base = float(spec.params.get("base", 10000.0))
        # base^(-2i / width) for every pair of columns, in float64 as the angles are
        pairs = torch.arange((self.width + 1) // 2, dtype=torch.float64)
        self.rates = (self.base ** (-2.0 * pairs / self.width)).to(runtime.device)
        self.table: Optional[torch.Tensor] = None

    def tensors(self):
        return {self.name("weight"): TensorDecl((self.vocab, self.width), MATRIX)}

    def bind(self, tensors):
        self.table = tensors[self.name("weight")]

    def forward(self, ctx) -> torch.Tensor:
        return kernels.embedding_sinusoid(self.table, ctx.tokens, ctx.positions, self.rates)

    def bytes_read(self, rows: int, context: int) -> int:
        return rows * self.width * self.table.element_size()


register_part("norm", "layer_norm", StreamNorm)
register_part("connection", "hyper_connection", HyperConnection)
register_part("embedding", "sinusoid_token_embedding", SinusoidTokenEmbedding)
register_arrangement("hyper_connections", HyperConnectionBlock)
