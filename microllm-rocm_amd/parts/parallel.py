"""Several mixers side by side: all read the same input, and the result is the sum of theirs, each times a scale.

Where every member can hand over its output projection and write what it computes before that projection into a
buffer it is given (``take_output_projection``, ``forward_inner(x, ctx, cache, out=, out_scale=)``,
``inner_width``), the members write side by side into one buffer, each already times its scale, and one product with
the stacked output weights gives the sum. Otherwise the members run whole and their results are scaled and stacked
as partial sums, which the next norm adds in order. What the members keep between steps is a ``CompositeNeed``.
"""
from __future__ import annotations

from typing import Dict, List, Mapping, Optional

import torch

from .base import CompositeNeed, Mixer, Runtime, TensorDecl
from .linear import Weight, linear
from .registry import build_part, register_part
from .spec import PartSpec


class ParallelMixer(Mixer):
    def __init__(self, spec: PartSpec, runtime: Runtime):
        super().__init__(spec, runtime)
        members = spec.params["members"]          # a sequence of (PartSpec of a mixer, scale)
        if not members:
            raise ValueError("a parallel mixer needs at least one member")
        self.members: List[Mixer] = [build_part("mixer", member, runtime) for member, _ in members]
        self.scales: List[float] = [float(scale) for _, scale in members]
        self.graph_safe = all(member.graph_safe for member in self.members)
        self.o_weight: Optional[Weight] = None

    def sub_parts(self):
        return tuple(self.members)

    def tensors(self) -> Dict[str, TensorDecl]:
        decls: Dict[str, TensorDecl] = {}
        for member in self.members:
            decls.update(member.tensors())
        return decls

    def bind(self, tensors: Mapping[str, torch.Tensor]) -> None:
        for member in self.members:
            member.bind(tensors)
        if all(hasattr(member, "take_output_projection") and hasattr(member, "forward_inner") for member in self.members):
            outputs = [member.take_output_projection() for member in self.members]
            if len({tensor.dtype for tensor in outputs}) != 1:
                raise TypeError("the output projections of one layer must share a dtype to be stacked")
            self.o_weight = Weight(torch.cat(outputs, dim=1).contiguous(), keep_plain=self.runtime.keep_plain_weights)

    def step_planner(self):
        return None

    def cache_need(self):
        return CompositeNeed(tuple(member.cache_need() for member in self.members))

    def flops(self, tokens: int) -> float:
        total = sum(member.flops(tokens) for member in self.members)
        if self.o_weight is not None:
            total += 2.0 * tokens * self.o_weight.out_features * self.o_weight.in_features
        return total

    def forward(self, x, ctx, cache):
        if self.o_weight is None:
            results = []
            for member, scale, binding in zip(self.members, self.scales, cache.parts):
                result = member.forward(x, ctx, binding).to(torch.float32)
                results.append((result.sum(0) if result.dim() == 3 else result) * scale)
            return torch.stack(results)
        widths = [member.inner_width for member in self.members]
        inner = torch.empty((x.shape[0], sum(widths)), dtype=self.runtime.dtype, device=x.device)
        first = 0
        for member, scale, binding, width in zip(self.members, self.scales, cache.parts, widths):
            member.forward_inner(x, ctx, binding, out=inner[:, first:first + width], out_scale=scale)
            first += width
        return linear(inner, self.o_weight, out_dtype=torch.float32, partials=True)


register_part("mixer", "parallel", ParallelMixer)
