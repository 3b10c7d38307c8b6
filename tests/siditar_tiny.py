"""Tiny Siditar configurations for the tests, each different from the others in every size, and their model folders."""
from __future__ import annotations

import os

import torch

from microllm_rocm_amd.config.siditar import (BiasAttentionConfig, DenseMlpConfig, LinearAttentionConfig, LoopConfig,
                                              ParallelMixerConfig, SiditarConfig, SiditarLayerConfig)
from microllm_rocm_amd.weights import write_model_folder


def _layer(left, right, scales, mlp):
    return SiditarLayerConfig("parallel", ParallelMixerConfig(left, right, scales[0], scales[1]), mlp)


# Three streams; grouped kv heads and a single one; key and value widths that differ and are no multiples of 8; a
# layer without a feed-forward; a loop that starts at the first layer and runs three times.
TINY_A = SiditarConfig(
    vocab=211, width=64, norm_eps=1e-5, streams=3, loop=LoopConfig(0, 2, 3),
    layers=(
        _layer(BiasAttentionConfig(heads=4, kv_heads=2, dim=24, vdim=16, scale=0.3, bias_max=40, temp_coef=0.7, temp_every=5, bias_rows=12),
               LinearAttentionConfig(heads=3, dim=16, vdim=8, tau=4.0, decay_rank=5), (0.7, 1.3), DenseMlpConfig(96, 1.0)),
        _layer(BiasAttentionConfig(heads=2, kv_heads=1, dim=20, vdim=40, scale=0.25, bias_max=9, temp_coef=0.2, temp_every=1, bias_rows=6),
               LinearAttentionConfig(heads=1, dim=40, vdim=24, tau=1.5, decay_rank=3), (1.2, 0.5), None),
        _layer(BiasAttentionConfig(heads=3, kv_heads=3, dim=8, vdim=8, scale=0.5, bias_max=100, temp_coef=1.0, temp_every=32, bias_rows=16),
               LinearAttentionConfig(heads=2, dim=8, vdim=72, tau=16.0, decay_rank=1), (1.0, 1.0), DenseMlpConfig(80, 2.5)),
    ))
# One residual stream with a plain sum (no streams named), no loop, other sizes.
TINY_B = SiditarConfig(
    vocab=97, width=40, norm_eps=1e-6, streams=None, loop=None,
    layers=(
        _layer(BiasAttentionConfig(heads=5, kv_heads=1, dim=16, vdim=24, scale=0.2, bias_max=30, temp_coef=0.4, temp_every=7, bias_rows=10),
               LinearAttentionConfig(heads=2, dim=24, vdim=16, tau=8.0, decay_rank=4), (0.9, 0.8), DenseMlpConfig(56, 1.5)),
        _layer(BiasAttentionConfig(heads=2, kv_heads=2, dim=32, vdim=12, scale=0.15, bias_max=64, temp_coef=0.0, temp_every=3, bias_rows=4),
               LinearAttentionConfig(heads=5, dim=8, vdim=8, tau=2.0, decay_rank=8), (1.1, 1.4), DenseMlpConfig(64, 0.75)),
    ))
# One stream that still goes through its connection weights; a width that is no multiple of 4; a loop over the last layer alone, twice; no feed-forward
# in the first layer.
TINY_C = SiditarConfig(
    vocab=130, width=50, norm_eps=1e-5, streams=1, loop=LoopConfig(1, 2, 2),
    layers=(
        _layer(BiasAttentionConfig(heads=2, kv_heads=2, dim=12, vdim=20, scale=0.3, bias_max=17, temp_coef=0.5, temp_every=4, bias_rows=8),
               LinearAttentionConfig(heads=4, dim=12, vdim=12, tau=3.0, decay_rank=2), (1.0, 0.6), None),
        _layer(BiasAttentionConfig(heads=6, kv_heads=3, dim=16, vdim=8, scale=0.25, bias_max=50, temp_coef=0.3, temp_every=16, bias_rows=14),
               LinearAttentionConfig(heads=1, dim=16, vdim=32, tau=6.0, decay_rank=6), (0.8, 1.2), DenseMlpConfig(72, 3.0)),
    ))

# Keys and values of one width that is a multiple of 16: in bfloat16 these layers take the paged attention's own pages
# and MFMA kernels; two streams; grouped kv heads; a bias table whose longest distance is shorter than the tests' prompts.
TINY_D = SiditarConfig(
    vocab=150, width=64, norm_eps=1e-6, streams=2, loop=LoopConfig(0, 1, 2),
    layers=(
        _layer(BiasAttentionConfig(heads=4, kv_heads=2, dim=32, vdim=32, scale=0.2, bias_max=70, temp_coef=0.5, temp_every=8, bias_rows=12),
               LinearAttentionConfig(heads=2, dim=16, vdim=32, tau=8.0, decay_rank=4), (0.8, 1.1), DenseMlpConfig(96, 1.5)),
        _layer(BiasAttentionConfig(heads=2, kv_heads=2, dim=16, vdim=16, scale=0.3, bias_max=20, temp_coef=0.3, temp_every=3, bias_rows=8),
               LinearAttentionConfig(heads=3, dim=8, vdim=16, tau=2.0, decay_rank=2), (1.2, 0.9), DenseMlpConfig(64, 2.0)),
    ))

CONFIGS = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "D": TINY_D}
SEEDS = {"A": 11, "B": 12, "C": 13, "D": 14}
STDS = {"std": 0.08, "norm_std": 0.1, "connection_std": 0.15, "bias_std": 0.7}


def make_siditar_folder(tmp_path, which: str) -> str:
    folder = os.path.join(str(tmp_path), f"siditar_{which}")
    write_model_folder(folder, CONFIGS[which], SEEDS[which], dtype=torch.bfloat16, stds=STDS)
    return folder
