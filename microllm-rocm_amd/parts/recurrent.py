"""A recurrent block around a real-gated linear recurrent unit.

Two branches of ``width`` channels read the input: ``y = gelu_tanh(Wy x + by)`` and ``u = conv(Wx x + bx)``, a causal
convolution per channel over the last ``taps`` inputs (zeros before the request's first token). ``u`` is cut into
``blocks`` equal parts; in each, two gates come from square matrices: ``r = sigmoid(A_b u_b + a_b)``,
``i = sigmoid(B_b u_b + b_b)``. With ``a = exp(-decay_scale * r * softplus(lam))`` per channel,

    S_t = a_t S_(t-1) + sqrt(1 - a_t^2) * i_t * u_t,        out_t = Wo (S_t * y_t),

from ``S = 0``, the first token included. A request keeps ``S`` and the convolution's last ``taps - 1`` inputs, both
float32, in its state slot, so it can be cut into steps anywhere. The two projections that read ``x`` are one stacked
product with a float32 result; the convolution, the gates' products, the decay and the recurrence are float32.
"""
from __future__ import annotations

from typing import Dict, Mapping, Optional

import torch

from ..ops import kernels
from .base import CompositeNeed, MATRIX, Mixer, Runtime, StateNeed, TensorDecl, VECTOR
from .linear import Weight, linear, linear_into_stream, takes_unscaled
from .registry import register_part
from .spec import PartSpec


class GatedLinearRecurrence(Mixer):
    # A step that is run twice would advance the state twice: the engine, which runs a step once before it captures
    # it, saves the step's state slots before that run and puts them back.
    graph_safe = True
    fuses_residual = True
    LONG_PORTION = 32       # from this many tokens of one request in a step on, the recurrence is walked in chunks side by side

    def __init__(self, spec: PartSpec, runtime: Runtime):
        super().__init__(spec, runtime)
        p = spec.params
        self.hidden = int(p["hidden_size"])
        self.width = int(p["width"])
        self.blocks = int(p["blocks"])
        self.taps = int(p["taps"])
        self.decay_scale = float(p["decay_scale"])
        if self.width % self.blocks != 0 or self.taps < 1:
            raise ValueError("the width must divide into the blocks, and the convolution needs a tap")
        self.size = self.width // self.blocks
        self.y_at, self.x_at = 0, self.width
        self.in_weight: Optional[Weight] = None
        self.o_weight: Optional[Weight] = None
        self.gate_weight: Optional[torch.Tensor] = None
        self.y_bias = self.x_bias = self.conv = self.conv_bias = self.r_bias = self.i_bias = self.lam = None

    def tensors(self) -> Dict[str, TensorDecl]:
        square = (self.blocks, self.size, self.size)
        return {self.name("y"): TensorDecl((self.width, self.hidden), MATRIX), self.name("y_bias"): TensorDecl((self.width,), VECTOR),
                self.name("x"): TensorDecl((self.width, self.hidden), MATRIX), self.name("x_bias"): TensorDecl((self.width,), VECTOR),
                self.name("conv"): TensorDecl((self.width, self.taps), VECTOR), self.name("conv_bias"): TensorDecl((self.width,), VECTOR),
                self.name("ra"): TensorDecl(square, MATRIX), self.name("ra_bias"): TensorDecl((self.blocks, self.size), VECTOR),
                self.name("ri"): TensorDecl(square, MATRIX), self.name("ri_bias"): TensorDecl((self.blocks, self.size), VECTOR),
                self.name("lam"): TensorDecl((self.width,), VECTOR), self.name("o"): TensorDecl((self.hidden, self.width), MATRIX)}

    def bind(self, tensors: Mapping[str, torch.Tensor]) -> None:
        y, x = tensors[self.name("y")], tensors[self.name("x")]
        if y.dtype != x.dtype:
            raise TypeError("the two branches' weights must share a dtype to be stacked")
        keep = self.runtime.keep_plain_weights
        self.in_weight = Weight(torch.cat([y, x], dim=0).contiguous(), keep_plain=keep)
        del y, x
        self.o_weight = Weight(tensors[self.name("o")], keep_plain=keep)
        # both gates' matrices per block as [in, out], side by side along out: one product per block gives both
        ra, ri = tensors[self.name("ra")], tensors[self.name("ri")]
        self.gate_weight = torch.cat([ra.transpose(1, 2), ri.transpose(1, 2)], dim=2).contiguous()
        self.y_bias, self.x_bias = tensors[self.name("y_bias")], tensors[self.name("x_bias")]
        self.conv, self.conv_bias = tensors[self.name("conv")], tensors[self.name("conv_bias")]
        self.r_bias = tensors[self.name("ra_bias")].reshape(-1).contiguous()
        self.i_bias = tensors[self.name("ri_bias")].reshape(-1).contiguous()
        self.lam = tensors[self.name("lam")]

    def cache_need(self):
        return CompositeNeed((StateNeed((self.taps - 1, self.width), torch.float32), StateNeed((self.width,), torch.float32)))

    def flops(self, tokens: int) -> float:
        return super().flops(tokens) + 2.0 * tokens * self.width * (2 * self.size + self.taps + 8)

    def takes_unscaled(self, rows: int) -> bool:
        return takes_unscaled(self.in_weight, rows)

    def forward(self, x, ctx, cache, residual=None):
        kept, state = cache.parts[0].state, cache.parts[1].state
        n_tokens = x.shape[0]
        proj = linear(x, self.in_weight, out_dtype=torch.float32)     # applies the rows' factors where x comes without them
        u = kernels.rglru_conv(proj, self.x_at, self.x_bias, self.conv, self.conv_bias, kept, ctx.seq_of_token, ctx.cu_tokens, ctx.slots)
        gates = torch.empty((n_tokens, self.blocks, 2 * self.size), dtype=torch.float32, device=proj.device)
        kernels.head_product(u.view(n_tokens, self.blocks, self.size), self.gate_weight, gates)
        out = kernels.rglru_scan(proj, self.x_at, self.x_bias, self.y_at, self.y_bias, u, gates.view(n_tokens, 2 * self.width),
                                 self.r_bias, self.i_bias, self.lam, self.decay_scale, state, kept, ctx.cu_tokens, ctx.slots,
                                 ctx.n_seqs, self.blocks, self.taps, self.runtime.dtype, chunked=ctx.max_count >= self.LONG_PORTION)
        if residual is not None:
            begun = linear_into_stream(out, self.o_weight, residual)
            if begun is not None:
                return begun
        return linear(out, self.o_weight, out_dtype=torch.float32, partials=True)


register_part("mixer", "rglru", GatedLinearRecurrence)
