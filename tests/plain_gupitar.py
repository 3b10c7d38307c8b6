"""A plain, slow implementation of the Gupitar decoder in numpy float64: one function per mechanism, whole sequences,
no cache, no batching. The tests hold the engine against it. It shares nothing with the package: it reads
config.json as a dict and the tensors by their names in the file.

Notation: a sequence has ``n`` tokens at positions ``0 .. n-1``; ``x`` is ``[n, width]``; a linear weight is stored
``[out, in]`` and applied as ``x @ W.T``.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional, Sequence

import numpy as np

from plain_qwen2 import read_safetensors  # noqa: F401  (a reader of the file format, nothing of a model)


def read_config(folder: str) -> dict:
    with open(os.path.join(folder, "config.json"), "r", encoding="utf-8") as handle:
        return json.load(handle)


# ---- small pieces ---------------------------------------------------------------------------------------------
def unit_rms(x: np.ndarray, eps: float) -> np.ndarray:
    return x / np.sqrt((x ** 2).mean(axis=-1, keepdims=True) + eps)


def norm_around_zero(x: np.ndarray, weight: np.ndarray, eps: float) -> np.ndarray:
    """The layers' norm: the stored weight is the distance of the gain from one."""
    return unit_rms(x, eps) * (1.0 + weight)


def norm_plain(x: np.ndarray, weight: np.ndarray, eps: float) -> np.ndarray:
    """The latents' norm: the stored weight is the gain."""
    return unit_rms(x, eps) * weight


def sigmoid(x: np.ndarray) -> np.ndarray:
    e = np.exp(-np.abs(x))
    return np.where(x >= 0, 1.0 / (1.0 + e), e / (1.0 + e))


def silu(x: np.ndarray) -> np.ndarray:
    return x * sigmoid(x)


def softplus(x: np.ndarray) -> np.ndarray:
    return np.maximum(x, 0.0) + np.log1p(np.exp(-np.abs(x)))


def gelu_tanh(x: np.ndarray) -> np.ndarray:
    return 0.5 * x * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * x ** 3)))


# ---- rotation -------------------------------------------------------------------------------------------------
def rotate_half(x: np.ndarray, positions: Sequence[int], dims: int, base: float) -> np.ndarray:
    """``x``: [n, ..., d]. Of the last axis the first ``dims`` entries turn: entry i with entry i + dims/2 by the
    angle ``p * base^(-2i/dims)``; the rest stays."""
    out = np.array(x, dtype=np.float64, copy=True)
    half = dims // 2
    for row, p in enumerate(positions):
        for i in range(half):
            angle = p * base ** (-2.0 * i / dims)
            c, s = math.cos(angle), math.sin(angle)
            u, v = x[row, ..., i], x[row, ..., i + half]
            out[row, ..., i] = u * c - v * s
            out[row, ..., i + half] = v * c + u * s
    return out


# ---- the attention through latents --------------------------------------------------------------------------------
def latent_keys(h: np.ndarray, t: Dict[str, np.ndarray], prefix: str, m: dict, eps: float):
    """What a layer with a down projection of its own leaves for itself and for the layers that borrow from it:
    the normed latent [n, kv_rank] and the turned shared key part [n, rot_dim]."""
    rank, rot = m["kv_rank"], m["rot_dim"]
    down = h @ t[prefix + "dkv"].T
    latent = norm_plain(down[:, :rank], t[prefix + "dkv.norm"], eps)
    shared = rotate_half(down[:, rank:rank + rot], range(h.shape[0]), m["rot"]["dims"], m["rot"]["base"])
    return latent, shared


def latent_attention(h: np.ndarray, t: Dict[str, np.ndarray], prefix: str, m: dict, eps: float, latent: np.ndarray,
                     shared: np.ndarray) -> np.ndarray:
    n = h.shape[0]
    heads, dim, rot, vdim = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    window = m["mask"]["size"]
    cq = norm_plain(h @ t[prefix + "dq"].T, t[prefix + "dq.norm"], eps)
    q = (cq @ t[prefix + "uq"].T).reshape(n, heads, dim + rot)
    q_flat, q_turn = q[:, :, :dim], rotate_half(q[:, :, dim:], range(n), m["rot"]["dims"], m["rot"]["base"])
    k_flat = (latent @ t[prefix + "uk"].T).reshape(n, heads, dim)
    values = (latent @ t[prefix + "uv"].T).reshape(n, heads, vdim)
    out = np.zeros((n, heads, vdim))
    for i in range(n):
        first = max(0, i - window + 1)
        for head in range(heads):
            scores = (k_flat[first:i + 1, head] @ q_flat[i, head] + shared[first:i + 1] @ q_turn[i, head]) * m["scale"]
            weights = np.exp(scores - scores.max())
            weights /= weights.sum()
            out[i, head] = weights @ values[first:i + 1, head]
    gate = sigmoid(h @ t[prefix + "g"].T)
    return (out.reshape(n, heads * vdim) * gate) @ t[prefix + "o"].T


# ---- the gated linear recurrence ------------------------------------------------------------------------------
def causal_conv(x: np.ndarray, taps: np.ndarray, bias: np.ndarray) -> np.ndarray:
    """``taps``: [channels, k]; the last column multiplies the token itself, zeros stand before the start."""
    n, k = x.shape[0], taps.shape[1]
    out = np.zeros_like(x)
    for i in range(n):
        for j in range(k):
            source = i - (k - 1 - j)
            if source >= 0:
                out[i] += taps[:, j] * x[source]
    return out + bias


def block_gate(u: np.ndarray, weight: np.ndarray, bias: np.ndarray) -> np.ndarray:
    """``weight``: [blocks, size, size] with [out, in] in each block, ``bias`` [blocks, size]."""
    blocks, size = weight.shape[0], weight.shape[1]
    parts = u.reshape(u.shape[0], blocks, size)
    z = np.einsum("nbi,boi->nbo", parts, weight) + bias
    return sigmoid(z).reshape(u.shape[0], blocks * size)


def rglru(h: np.ndarray, t: Dict[str, np.ndarray], prefix: str, m: dict) -> np.ndarray:
    width, blocks = m["width"], m["blocks"]
    y = gelu_tanh(h @ t[prefix + "y"].T + t[prefix + "y.b"])
    u = causal_conv(h @ t[prefix + "x"].T + t[prefix + "x.b"], t[prefix + "conv"], t[prefix + "conv.b"])
    size = width // blocks
    r = block_gate(u, t[prefix + "ra"].reshape(blocks, size, size), t[prefix + "ra.b"].reshape(blocks, size))
    i = block_gate(u, t[prefix + "ri"].reshape(blocks, size, size), t[prefix + "ri.b"].reshape(blocks, size))
    log_a = -8.0 * r * softplus(t[prefix + "lam"])
    a = np.exp(log_a)
    state = np.zeros(width)
    out = np.zeros_like(u)
    for step in range(h.shape[0]):
        state = a[step] * state + np.sqrt(1.0 - a[step] ** 2) * i[step] * u[step]
        out[step] = state
    return (out * y) @ t[prefix + "o"].T


# ---- feed-forwards ----------------------------------------------------------------------------------------------
def gated_ff(h: np.ndarray, t: Dict[str, np.ndarray], prefix: str) -> np.ndarray:
    return (silu(h @ t[prefix + "gate"].T) * (h @ t[prefix + "up"].T)) @ t[prefix + "down"].T


def routed_ff(h: np.ndarray, t: Dict[str, np.ndarray], prefix: str, mlp: dict, margins: Optional[List[np.ndarray]] = None) -> np.ndarray:
    """``margins`` collects, per token, how far the last chosen expert's logit lies above the best one not chosen
    (infinite where every expert is chosen): a token whose margin is tiny may go to another expert in an engine that
    rounds, and a test of such an engine leaves it out."""
    experts, top = mlp["router"]["experts"], mlp["router"]["top"]
    z = h @ t[prefix + "router"].T
    scores = sigmoid(z)
    if margins is not None:
        ordered = -np.sort(-z, axis=1)
        margins.append(ordered[:, top - 1] - ordered[:, top] if top < experts else np.full(h.shape[0], np.inf))
    out = np.zeros_like(h)
    for row in range(h.shape[0]):
        chosen = sorted(range(experts), key=lambda e: (-scores[row, e], e))[:top]
        for e in chosen:
            out[row] += gated_ff(scores[row, e] * h[row:row + 1], t, f"{prefix}e{e}.")[0]
    if mlp.get("shared") is not None:
        out += gated_ff(h, t, prefix + "shared.") * sigmoid(h @ t[prefix + "shared.sg"].T)
    return out


# ---- the model ------------------------------------------------------------------------------------------------
def forward(config: dict, tensors: Dict[str, np.ndarray], tokens: Sequence[int], layers_out: Optional[List[np.ndarray]] = None,
            margins: Optional[List[np.ndarray]] = None) -> np.ndarray:
    """Logits ``[n, vocab]`` of one sequence run whole. ``layers_out`` collects the residual stream after every layer,
    ``margins`` the routers' margins (``routed_ff``)."""
    t = {name: np.asarray(value, dtype=np.float64) for name, value in tensors.items()}
    eps = config["norm"]["eps"]
    x = t["embed"][np.asarray(tokens, dtype=np.int64)]
    kept = {}
    for index, layer in enumerate(config["layers"]):
        prefix = f"l{index}."
        m = layer["mixer"]
        h = norm_around_zero(x, t[prefix + "norm1"], eps)
        if layer["type"] == "latent_attention":
            if m.get("kv_from") is None:
                kept[index] = latent_keys(h, t, prefix + "mix.", m, eps)
            latent, shared = kept[m["kv_from"] if m.get("kv_from") is not None else index]
            x = x + latent_attention(h, t, prefix + "mix.", m, eps, latent, shared)
        elif layer["type"] == "rglru":
            x = x + rglru(h, t, prefix + "mix.", m)
        else:
            raise ValueError(f"unknown layer type {layer['type']!r}")
        mlp = layer.get("mlp")
        if mlp is not None:
            h = norm_around_zero(x, t[prefix + "norm2"], eps)
            x = x + (gated_ff(h, t, prefix + "mlp.") if mlp["kind"] == "dense" else routed_ff(h, t, prefix + "mlp.", mlp, margins))
        if layers_out is not None:
            layers_out.append(x.copy())
    return norm_around_zero(x, t["final.norm"], eps) @ t["head"].T


def folded_attention(q_full: np.ndarray, rows: np.ndarray, kv_rank: int, window: int, scale: float, first: int = 0) -> np.ndarray:
    """The attention as it runs on cached rows: ``q_full`` [n, heads, row] are queries at positions ``first ..``,
    ``rows`` [first + n, row] one cached row a position (latent, then the shared turned key part); a query at p sees
    rows p - window + 1 .. p, and the result is the weighted sum of the rows' first ``kv_rank`` entries."""
    n, heads, _ = q_full.shape
    out = np.zeros((n, heads, kv_rank))
    for i in range(n):
        p = first + i
        low = max(0, p - window + 1) if window > 0 else 0
        for head in range(heads):
            scores = rows[low:p + 1] @ q_full[i, head] * scale
            weights = np.exp(scores - scores.max())
            out[i, head] = (weights / weights.sum()) @ rows[low:p + 1, :kv_rank]
    return out


def choose_experts(z: np.ndarray, top: int, softmax: bool = False, renormalize: bool = False):
    """Per row of router logits: the ``top`` experts with the largest scores (ties: the lower index) and their weights."""
    if softmax:
        e = np.exp(z - z.max(axis=-1, keepdims=True))
        scores = e / e.sum(axis=-1, keepdims=True)
    else:
        scores = sigmoid(z)
    ids = np.zeros((z.shape[0], top), dtype=np.int64)
    weights = np.zeros((z.shape[0], top))
    for row in range(z.shape[0]):
        order = sorted(range(z.shape[1]), key=lambda e: (-z[row, e], e))[:top]
        ids[row], weights[row] = order, scores[row, order]
        if renormalize:
            weights[row] /= weights[row].sum()
    return ids, weights


def generate_greedy(config: dict, tensors: Dict[str, np.ndarray], prompt: Sequence[int], new_tokens: int) -> List[int]:
    """The first maximum of the last position's logits, appended ``new_tokens`` times; the whole sequence is run again
    for every token."""
    tokens = list(prompt)
    for _ in range(new_tokens):
        tokens.append(int(np.argmax(forward(config, tensors, tokens)[-1])))
    return tokens[len(prompt):]
