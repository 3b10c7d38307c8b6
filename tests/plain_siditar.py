"""A plain, slow implementation of the Siditar decoder in numpy float64: one function per mechanism, whole sequences,
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
def position_waves(count: int, width: int, first: int = 0) -> np.ndarray:
    """Row p: entry 2i is sin(p / 10000^(2i / width)), entry 2i + 1 the cosine of the same angle."""
    out = np.zeros((count, width))
    for row in range(count):
        for column in range(width):
            angle = (first + row) * 10000.0 ** (-2.0 * (column // 2) / width)
            out[row, column] = math.cos(angle) if column % 2 else math.sin(angle)
    return out


def layer_norm(x: np.ndarray, weight: np.ndarray, eps: float) -> np.ndarray:
    centred = x - x.mean(axis=-1, keepdims=True)
    return centred / np.sqrt((centred ** 2).mean(axis=-1, keepdims=True) + eps) * weight


def unit_rms(x: np.ndarray, weight: np.ndarray, eps: float) -> np.ndarray:
    return x / np.sqrt((x ** 2).mean(axis=-1, keepdims=True) + eps) * weight


def sigmoid(x: np.ndarray) -> np.ndarray:
    return np.where(x >= 0, 1.0 / (1.0 + np.exp(-np.abs(x))), np.exp(-np.abs(x)) / (1.0 + np.exp(-np.abs(x))))


# ---- streams --------------------------------------------------------------------------------------------------
def streams_read(streams: List[np.ndarray], take: np.ndarray) -> np.ndarray:
    return sum(take[s] * streams[s] for s in range(len(streams)))


def streams_write(streams: List[np.ndarray], mix: np.ndarray, give: np.ndarray, y: np.ndarray) -> List[np.ndarray]:
    count = len(streams)
    return [sum(mix[s, t] * streams[s] for s in range(count)) + give[t] * y for t in range(count)]


# ---- the softmax attention --------------------------------------------------------------------------------------
def bucket_of(distance: int, rows: int, longest: int) -> int:
    half = rows // 2
    if distance < half:
        return distance
    return min(rows - 1, half + int(math.floor(math.log(distance / half) / math.log(longest / half) * (rows - half))))


def query_factor(position: int, coef: float, every: int) -> float:
    return 1.0 + coef * math.log((position + 1) // every + 1)


def bias_sink_attention(q: np.ndarray, k: np.ndarray, v: np.ndarray, scale: float, table: Optional[np.ndarray],
                        longest: int, sink: Optional[np.ndarray]) -> np.ndarray:
    """q [n, H, d], k [n, G, d], v [n, G, dv] -> [n, H, dv]; query i sees keys j <= i."""
    n, heads, _ = q.shape
    group = heads // k.shape[1]
    out = np.zeros((n, heads, v.shape[2]))
    for head in range(heads):
        for i in range(n):
            scores = np.array([q[i, head] @ k[j, head // group] * scale +
                               (table[bucket_of(i - j, table.shape[0], longest), head] if table is not None else 0.0)
                               for j in range(i + 1)])
            top = max(scores.max(), sink[head]) if sink is not None else scores.max()
            weights = np.exp(scores - top)
            total = weights.sum() + (math.exp(sink[head] - top) if sink is not None else 0.0)
            out[i, head] = (weights / total) @ v[: i + 1, head // group]
    return out


def left_mixer(x: np.ndarray, w: Dict[str, np.ndarray], prefix: str, c: dict, eps: float, first: int = 0) -> np.ndarray:
    n = x.shape[0]
    heads, kv_heads, dim, vdim = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    q = unit_rms((x @ w[prefix + "q"].T).reshape(n, heads, dim), w[prefix + "q.norm"], eps)
    k = unit_rms((x @ w[prefix + "k"].T).reshape(n, kv_heads, dim), w[prefix + "k.norm"], eps)
    v = (x @ w[prefix + "v"].T).reshape(n, kv_heads, vdim)
    for i in range(n):
        q[i] *= query_factor(first + i, c["q_temp"]["coef"], c["q_temp"]["every"])
    out = bias_sink_attention(q, k, v, c["scale"], w[prefix + "rel"], c["bias_max"], w[prefix + "sink"])
    return out.reshape(n, heads * vdim) @ w[prefix + "o"].T


# ---- the linear attention ---------------------------------------------------------------------------------------
def decayed_state_walk(q: np.ndarray, k: np.ndarray, v: np.ndarray, decay: np.ndarray,
                       state: Optional[np.ndarray] = None):
    """q, k, decay [n, H, d], v [n, H, dv]; S <- decay[:, None] * S + k v^T; o = S^T q. Returns (o, last state)."""
    n, heads, dim = q.shape
    state = np.zeros((heads, dim, v.shape[2])) if state is None else state.copy()
    out = np.zeros((n, heads, v.shape[2]))
    for t in range(n):
        for head in range(heads):
            state[head] = decay[t, head][:, None] * state[head] + np.outer(k[t, head], v[t, head])
            out[t, head] = state[head].T @ q[t, head]
    return out, state


def right_mixer(x: np.ndarray, w: Dict[str, np.ndarray], prefix: str, c: dict, eps: float) -> np.ndarray:
    n = x.shape[0]
    heads, dim, vdim = c["heads"], c["dim"], c["vdim"]
    q = (x @ w[prefix + "q"].T).reshape(n, heads, dim) * dim ** -0.5
    k = (x @ w[prefix + "k"].T).reshape(n, heads, dim)
    v = (x @ w[prefix + "v"].T).reshape(n, heads, vdim)
    z = (x @ w[prefix + "a1"].T) @ w[prefix + "a2"].T + w[prefix + "a2.b"]
    decay = (sigmoid(z) ** (1.0 / c["tau"])).reshape(n, heads, dim)
    o, _ = decayed_state_walk(q, k, v, decay)
    o = unit_rms(o, w[prefix + "norm"], eps).reshape(n, heads * vdim)
    gate = x @ w[prefix + "g"].T
    return (o * gate * sigmoid(gate)) @ w[prefix + "o"].T


def parallel_mixer(x, w, prefix, c, eps):
    return (c["left_scale"] * left_mixer(x, w, prefix + "left.", c["left"], eps) +
            c["right_scale"] * right_mixer(x, w, prefix + "right.", c["right"], eps))


# ---- the feed-forward -------------------------------------------------------------------------------------------
def clamped_gated_ffn(x, w, prefix, c):
    gate = np.minimum(x @ w[prefix + "gate"].T, c["limit"])
    up = np.clip(x @ w[prefix + "up"].T, -c["limit"], c["limit"])
    return (gate * sigmoid(1.702 * gate) * (up + 1.0)) @ w[prefix + "down"].T


# ---- the model --------------------------------------------------------------------------------------------------
def run_order(config: dict) -> List[int]:
    count = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return list(range(count))
    return (list(range(loop["start"])) + list(range(loop["start"], loop["stop"])) * loop["times"] +
            list(range(loop["stop"], count)))


def forward(config: dict, w: Dict[str, np.ndarray], tokens: Sequence[int], after_runs: Optional[list] = None) -> np.ndarray:
    """Logits ``[n, vocab]`` of a whole sequence; ``after_runs`` collects the stream (summed) after every layer run."""
    w = {name: np.asarray(value, dtype=np.float64) for name, value in w.items()}
    eps = config["norm"]["eps"]
    x = w["embed"][np.asarray(tokens, dtype=np.int64)] + position_waves(len(tokens), config["width"])
    count = config.get("streams")
    streams = [x.copy() for _ in range(count)] if count else None
    for index in run_order(config):
        layer, prefix = config["layers"][index], f"l{index}."
        assert layer["type"] == "parallel"
        sublayers = [("1", lambda u: parallel_mixer(u, w, prefix + "mix.", layer["mixer"], eps))]
        if layer["mlp"] is not None:
            assert layer["mlp"]["kind"] == "dense"
            sublayers.append(("2", lambda u: clamped_gated_ffn(u, w, prefix + "mlp.", layer["mlp"])))
        for number, sublayer in sublayers:
            if streams is not None:
                joint = prefix + "hc" + number
                y = sublayer(layer_norm(streams_read(streams, w[joint + ".in"]), w[prefix + "norm" + number], eps))
                streams = streams_write(streams, w[joint + ".mix"], w[joint + ".out"], y)
            else:
                x = x + sublayer(layer_norm(x, w[prefix + "norm" + number], eps))
        if after_runs is not None:
            after_runs.append(sum(streams) if streams is not None else x.copy())
    if streams is not None:
        x = sum(streams)
    return layer_norm(x, w["final.norm"], eps) @ w["head"].T


def generate_greedy(config: dict, w: Dict[str, np.ndarray], prompt: Sequence[int], new_tokens: int) -> List[int]:
    tokens = list(prompt)
    for _ in range(new_tokens):
        tokens.append(int(np.argmax(forward(config, w, tokens)[-1])))
    return tokens[len(prompt):]
