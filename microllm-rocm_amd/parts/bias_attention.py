"""Causal softmax attention whose positions enter through the scores: a learned bias by distance bucket, a sink in
the softmax, and a query factor that grows with the position. No rotation.

``q = Wq x``, ``k = Wk x``, ``v = Wv x`` (no biases); query head ``h`` uses kv head ``h // (heads / kv_heads)``; keys
have ``key_dim`` and values ``value_dim`` channels. With ``qk_norm`` queries and keys are divided by their root mean
square over the head (eps inside the root) and multiplied by a weight ``[key_dim]`` that all heads share. Queries
at position ``p`` are multiplied by ``1 + temp_coef * ln(floor((p + 1) / temp_every) + 1)``. The score of key ``j``
for a query at ``i >= j`` is ``(q . k) * scale + table[bucket(i - j), h]`` with, for a table of ``B`` rows and a
longest distance ``D``: ``bucket(n) = n`` below ``B / 2``, else ``min(B - 1, B/2 + floor(ln(n / (B/2)) / ln(D / (B/2))
* (B - B/2)))``. The softmax's denominator also holds ``exp(sink[h])``, which has no key and no value.

Every distance from ``D`` on falls into the last bucket, so the table is unrolled once, at load, into one row per
distance up to ``D`` and the kernels index it with ``min(i - j, D)``.

In bfloat16, with keys and values of one width that is a multiple of 16, the pages are the paged attention's own
(``PagedKVNeed``) and the attention runs on its MFMA kernels, which take the bias, the sink and the result's factor
as extras; everything else (float32, two widths, other sizes) lies in plain pages (``PagedKeyValueNeed``) and runs on
the kernel that takes a wave per token and head.
"""
from __future__ import annotations

import math
from typing import Dict, Mapping, Optional

import torch

from ..ops import kernels
from .attention import QueryTilePlanner
from .base import MATRIX, Mixer, PagedKeyValueNeed, PagedKVNeed, Runtime, TensorDecl, VECTOR
from .linear import Weight, linear
from .registry import register_part
from .spec import PartSpec


def distance_bucket(distance: int, rows: int, longest: int) -> int:
    """The row of a ``rows``-row bias table for ``distance >= 0``: exact below ``rows // 2``, logarithmic up to
    ``longest``, the last row beyond."""
    half = rows // 2
    if distance < half:
        return distance
    return min(rows - 1, half + int(math.floor(math.log(distance / half) / math.log(longest / half) * (rows - half))))


class BucketBiasAttention(Mixer):
    graph_safe = True

    def __init__(self, spec: PartSpec, runtime: Runtime):
        super().__init__(spec, runtime)
        p = spec.params
        self.hidden = int(p["hidden_size"])
        self.heads = int(p["heads"])
        self.kv_heads = int(p["kv_heads"])
        self.key_dim = int(p["key_dim"])
        self.value_dim = int(p["value_dim"])
        self.scale = float(p.get("scale", 1.0 / math.sqrt(self.key_dim)))
        self.qk_norm = bool(p.get("qk_norm", True))
        self.eps = float(p.get("eps", 1e-6))
        self.temp_coef = float(p.get("temp_coef", 0.0))
        self.temp_every = int(p.get("temp_every", 1))
        self.bias_rows = int(p["bias_rows"]) if p.get("bias_rows") else 0      # 0: no bias
        self.bias_max = int(p.get("bias_max", 0))
        self.has_sink = bool(p.get("sink", True))
        if self.heads % self.kv_heads != 0:
            raise ValueError("heads must divide into kv_heads groups")
        if self.bias_rows and self.bias_max <= self.bias_rows // 2:
            raise ValueError("bias_max must lie beyond the distances that have a bucket of their own")
        # the paged attention's pages and MFMA kernels, where they fit (the bias column must fit the prefill kernel's LDS)
        self.tiled = (runtime.dtype == torch.bfloat16 and self.key_dim == self.value_dim and self.key_dim % 16 == 0
                      and self.key_dim <= 256 and self.bias_max + 1 <= kernels.MFMA_BIAS_ROWS)
        self.planner = QueryTilePlanner(False) if self.tiled else None
        self.qkv_weight: Optional[Weight] = None
        self.o_tensor: Optional[torch.Tensor] = None
        self.o_weight: Optional[Weight] = None
        self.q_norm = self.k_norm = self.bias = self.sink = None

    @property
    def inner_width(self) -> int:
        return self.heads * self.value_dim

    def tensors(self) -> Dict[str, TensorDecl]:
        decls = {self.name("q"): TensorDecl((self.heads * self.key_dim, self.hidden), MATRIX),
                 self.name("k"): TensorDecl((self.kv_heads * self.key_dim, self.hidden), MATRIX),
                 self.name("v"): TensorDecl((self.kv_heads * self.value_dim, self.hidden), MATRIX),
                 self.name("o"): TensorDecl((self.hidden, self.heads * self.value_dim), MATRIX)}
        if self.qk_norm:
            decls[self.name("q_norm")] = TensorDecl((self.key_dim,), VECTOR)
            decls[self.name("k_norm")] = TensorDecl((self.key_dim,), VECTOR)
        if self.bias_rows:
            decls[self.name("bias")] = TensorDecl((self.bias_rows, self.heads), VECTOR)
        if self.has_sink:
            decls[self.name("sink")] = TensorDecl((self.heads,), VECTOR)
        return decls

    def bind(self, tensors: Mapping[str, torch.Tensor]) -> None:
        weights = [tensors[self.name(role)] for role in ("q", "k", "v")]
        if len({w.dtype for w in weights}) != 1:
            raise TypeError("the q, k and v weights of one layer must share a dtype to be stacked")
        self.qkv_weight = Weight(torch.cat(weights, dim=0).contiguous(), keep_plain=self.runtime.keep_plain_weights)
        del weights
        self.o_tensor = tensors[self.name("o")]
        if self.qk_norm:
            self.q_norm, self.k_norm = tensors[self.name("q_norm")], tensors[self.name("k_norm")]
        if self.bias_rows:
            table = tensors[self.name("bias")]
            rows = [distance_bucket(distance, self.bias_rows, self.bias_max) for distance in range(self.bias_max + 1)]
            self.bias = table[torch.tensor(rows, dtype=torch.int64, device=table.device)].contiguous()   # [bias_max + 1, heads]
        if self.has_sink:
            self.sink = tensors[self.name("sink")]

    def take_output_projection(self) -> Optional[torch.Tensor]:
        """The output projection ``[hidden, inner_width]`` as loaded, for a mixer that runs this one beside others and
        multiplies all their results with one stacked weight; this part then no longer holds it."""
        tensor, self.o_tensor = self.o_tensor, None
        return tensor

    def step_planner(self):
        return self.planner

    def cache_need(self):
        if self.tiled:
            return PagedKVNeed(self.kv_heads, self.key_dim)
        return PagedKeyValueNeed(self.kv_heads, self.key_dim, self.value_dim)

    def flops(self, tokens: int) -> float:
        pairs = tokens * (tokens + 1) / 2
        columns = (self.heads + self.kv_heads) * self.key_dim + self.kv_heads * self.value_dim
        if self.o_tensor is not None or self.o_weight is not None:      # else the mixer that took the projection counts it
            columns += self.heads * self.value_dim
        return 2.0 * tokens * self.hidden * columns + 2.0 * self.heads * (self.key_dim + self.value_dim) * pairs

    def forward_inner(self, x, ctx, cache, out: Optional[torch.Tensor] = None, out_scale: float = 1.0) -> torch.Tensor:
        """The heads' results side by side, ``[tokens, heads * value_dim]`` times ``out_scale``, before the output
        projection; written into ``out`` if given (columns of a wider buffer)."""
        view = ctx.paged[cache.group]
        qkv = linear(x, self.qkv_weight, out_dtype=torch.float32, partials=True)     # rounded once, after norm and factor
        q = kernels.qk_norm_store(qkv, self.q_norm, self.k_norm, self.eps, ctx.positions, view.slot_mapping, self.temp_coef,
                                  self.temp_every, cache.k, cache.v, self.heads, self.kv_heads, self.key_dim, self.value_dim,
                                  self.runtime.dtype, tiled_page_size=view.page_size if self.tiled else 0)
        if self.tiled:
            if out is None:
                out = torch.empty((x.shape[0], self.heads * self.value_dim), dtype=self.runtime.dtype, device=x.device)
            extras = kernels.AttentionExtras(self.bias, self.sink, out_scale)
            return kernels.paged_attention(q, cache.k, cache.v, view, ctx, self.scale, 0, self.heads, self.kv_heads, self.key_dim,
                                           planner=self.planner, extras=extras, out=out)
        return kernels.bias_attention(q, cache.k, cache.v, view.block_table, ctx.seq_of_token, ctx.positions, self.bias,
                                      self.sink, self.scale, out_scale, self.heads, self.kv_heads, self.key_dim,
                                      self.value_dim, out=out)

    def forward(self, x, ctx, cache):
        if self.o_weight is None:
            if self.o_tensor is None:
                raise RuntimeError("this attention's output projection was taken by the mixer it is a part of")
            self.o_weight = Weight(self.take_output_projection(), keep_plain=self.runtime.keep_plain_weights)
        return linear(self.forward_inner(x, ctx, cache), self.o_weight, out_dtype=torch.float32, partials=True)


register_part("mixer", "bucket_bias_attention", BucketBiasAttention)
