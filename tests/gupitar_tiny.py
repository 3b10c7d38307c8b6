"""Tiny Gupitar configurations for the tests, each different from the others in every size, and their model folders."""
from __future__ import annotations

import os

import torch

from microllm_rocm_amd.config.gupitar import (DenseMlpConfig, GupitarConfig, GupitarLayerConfig, LatentAttentionConfig, MoeMlpConfig,
                                              RglruConfig)
from microllm_rocm_amd.weights import write_model_folder


def _attention(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, window, base=10000.0, kv_from=None):
    return LatentAttentionConfig(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, q_rank=q_rank, kv_rank=kv_rank, scale=scale,
                                 window=window, rot_base=base, rot_dims=rot_dim, kv_from=kv_from)


def _layer(mixer, mlp):
    return GupitarLayerConfig("latent_attention" if isinstance(mixer, LatentAttentionConfig) else "rglru", mixer, mlp)


# Cached rows of 48 elements (a multiple of 16: in bfloat16 the paged attention's pages and MFMA kernels); a layer that
# borrows them with a wider window than the lender's; two experts a token with a shared expert; one expert a token
# without; a recurrence of one block and one tap without a feed-forward; cached rows of 42 elements (plain pages).
TINY_A = GupitarConfig(
    vocab=211, width=64, norm_eps=1e-5,
    layers=(
        _layer(_attention(4, 16, 8, 12, 24, 40, 0.2, 17), DenseMlpConfig(96)),
        _layer(RglruConfig(width=96, blocks=3, conv=4), MoeMlpConfig(experts=6, top=2, expert_ff=40, shared_ff=56)),
        _layer(_attention(2, 8, 8, 20, 16, 40, 0.3, 33, kv_from=0), MoeMlpConfig(experts=5, top=1, expert_ff=24, shared_ff=None)),
        _layer(RglruConfig(width=64, blocks=1, conv=1), None),
        _layer(_attention(3, 10, 6, 14, 20, 36, 0.25, 9, base=500.0), MoeMlpConfig(experts=4, top=3, expert_ff=32, shared_ff=16)),
    ))
# A recurrence first; a width that is no multiple of 8; one head; a window of one token (a query sees itself alone) and
# one longer than every test prompt; every expert for every token; two taps; a borrower of plain pages.
TINY_B = GupitarConfig(
    vocab=97, width=50, norm_eps=1e-6,
    layers=(
        _layer(RglruConfig(width=70, blocks=5, conv=2), DenseMlpConfig(44)),
        _layer(_attention(1, 12, 4, 9, 10, 18, 0.4, 1), MoeMlpConfig(experts=3, top=3, expert_ff=20, shared_ff=12)),
        _layer(_attention(5, 6, 10, 6, 30, 25, 0.3, 1000, base=77.0), None),
        _layer(_attention(2, 14, 10, 5, 12, 25, 0.5, 64, base=77.0, kv_from=2), DenseMlpConfig(60)),
    ))
# Rows of 256 elements (the widest the MFMA kernels take) and of 32; heads of unequal query, key and value sizes;
# windows that end exactly on a page's edge and one position off it.
TINY_C = GupitarConfig(
    vocab=150, width=96, norm_eps=1e-6,
    layers=(
        _layer(_attention(5, 24, 32, 40, 48, 224, 0.15, 32), MoeMlpConfig(experts=8, top=2, expert_ff=48, shared_ff=32)),
        _layer(_attention(6, 16, 16, 16, 32, 16, 0.25, 15), DenseMlpConfig(128)),
        _layer(RglruConfig(width=128, blocks=2, conv=3), MoeMlpConfig(experts=2, top=1, expert_ff=64, shared_ff=64)),
        _layer(_attention(3, 8, 32, 8, 16, 224, 0.2, 49, kv_from=0), DenseMlpConfig(80)),
    ))

CONFIGS = {"A": TINY_A, "B": TINY_B, "C": TINY_C}
SEEDS = {"A": 21, "B": 22, "C": 23}
STDS = {"std": 0.1, "norm_std": 0.15, "bias_std": 0.4}


def make_gupitar_folder(tmp_path, which: str) -> str:
    folder = os.path.join(str(tmp_path), f"gupitar_{which}")
    write_model_folder(folder, CONFIGS[which], SEEDS[which], dtype=torch.bfloat16, stds=STDS)
    return folder
