"""Tiny Kalevik configurations for the tests, each different from the others in every size, and their model folders."""
from __future__ import annotations

import os

import torch

from microllm_rocm_amd.config.kalevik import (ChunkAttentionConfig, DenseMlpConfig, KalevikConfig, KalevikLayerConfig, LatentAttentionConfig,
                                              LoopConfig, MoeMlpConfig, ParallelConfig, RetentionConfig)
from microllm_rocm_amd.weights import write_model_folder


def _latent(heads, dim, rot_dim, vdim, kv_rank, scale, base=10000.0):
    return LatentAttentionConfig(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank, scale=scale, rot_base=base,
                                 rot_dims=rot_dim)


def _left(heads, kv_heads, dim, vdim, scale, chunk, rot_dims, base=10000.0, factor=1.0):
    return ChunkAttentionConfig(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale, chunk=chunk, rot_base=base,
                                rot_dims=rot_dims, rot_factor=factor)


def _right(dim, vdim, decay):
    return RetentionConfig(heads=len(decay), dim=dim, vdim=vdim, decay=tuple(decay))


def _layer(mixer, mlp):
    kind = "latent_attention" if isinstance(mixer, LatentAttentionConfig) else "parallel"
    if isinstance(mlp, int):
        mlp = DenseMlpConfig(mlp)
    return KalevikLayerConfig(kind, mixer, mlp)


# A parallel layer first (chunks of 19 positions through the MFMA kernels in bfloat16, a quarter of the head turned, positions
# stretched), experts in four groups of which two are kept; cached latent rows of 48 elements; a parallel layer of equal
# head counts, unequal key and value sizes, whole heads turned, chunks shorter than a page and a retention of one head,
# without a feed-forward; experts without groups and without a shared one; layers 1 and 2 run twice.
TINY_A = KalevikConfig(
    vocab=211, width=64, norm_eps=1e-5, embedding_scale=2.0, loop=LoopConfig(1, 3, 2),
    layers=(
        _layer(ParallelConfig(_left(4, 2, 16, 16, 0.3, 19, 8, factor=2.0), _right(12, 10, [0.9, 0.95, 0.99]), 0.7, 1.1),
               MoeMlpConfig(experts=8, top=2, expert_ff=24, groups=4, keep_groups=2, shared_ff=40)),
        _layer(_latent(4, 16, 8, 12, 40, 0.2), 96),
        _layer(ParallelConfig(_left(6, 6, 10, 6, 0.4, 7, 10), _right(9, 14, [0.5]), 1.3, 0.4), None),
        _layer(_latent(1, 12, 4, 9, 18, 0.4, base=77.0), MoeMlpConfig(experts=5, top=3, expert_ff=20)),
    ))
# A width that is no multiple of 8; no factor on the embedding and no loop; latent rows of 42 elements (plain pages in
# either format) in a layer without a feed-forward; one key/value head for three query heads, chunks of exactly a page,
# positions stretched eightfold; one expert a token out of the one kept group of three; chunks longer than every test
# prompt; decays of one (nothing forgotten) and near zero (little but the token itself).
TINY_B = KalevikConfig(
    vocab=97, width=50, norm_eps=1e-6, embedding_scale=1.0, loop=None,
    layers=(
        _layer(_latent(3, 10, 6, 14, 36, 0.25), None),
        _layer(ParallelConfig(_left(3, 1, 32, 32, 0.2, 16, 32, base=500.0, factor=8.0), _right(40, 7, [0.8, 0.999]), 1.0, 1.0),
               MoeMlpConfig(experts=6, top=1, expert_ff=20, groups=3, keep_groups=1, shared_ff=28)),
        _layer(ParallelConfig(_left(2, 2, 48, 48, 0.15, 1000, 16), _right(8, 8, [1.0, 0.05, 0.7, 0.97]), 0.5, 2.0), 60),
    ))
# The looped range begins with a parallel layer at layer 0, three passes; latent rows of 256 elements (the widest the MFMA
# kernels take); chunks of one position (a query sees itself alone) and of 17 (a page and one); all groups kept; four of
# sixteen experts of 64 channels (in bfloat16 prompts the experts' tiled products).
TINY_C = KalevikConfig(
    vocab=150, width=96, norm_eps=1e-6, embedding_scale=0.5, loop=LoopConfig(0, 2, 3),
    layers=(
        _layer(ParallelConfig(_left(8, 2, 32, 32, 0.18, 17, 16, factor=3.0), _right(16, 24, [0.5, 0.75, 0.875]), 0.75, 1.25),
               MoeMlpConfig(experts=16, top=4, expert_ff=64, groups=4, keep_groups=4, shared_ff=32)),
        _layer(_latent(5, 24, 32, 40, 224, 0.15, base=500.0), 128),
        _layer(ParallelConfig(_left(2, 1, 24, 40, 0.3, 1, 24), _right(128, 12, [0.96]), 1.0, 0.8),
               MoeMlpConfig(experts=12, top=3, expert_ff=16, groups=6, keep_groups=2, shared_ff=None)),
    ))

CONFIGS = {"A": TINY_A, "B": TINY_B, "C": TINY_C}
SEEDS = {"A": 41, "B": 42, "C": 43}
STDS = {"std": 0.1, "norm_std": 0.15}


def without_choice(config: KalevikConfig) -> KalevikConfig:
    """The same model with every token sent through all of its experts, weighted by their scores. Which experts a token
    takes is a step function of the router's logits: an engine that rounds to bfloat16 takes another expert than the
    plain run wherever two logits lie within the rounding of each other (a few tokens in a hundred, whatever the
    weights' scale), and what such a token then caches moves every later position. The bfloat16 engine is therefore held
    against the plain run on these models, where the experts' sum is continuous; the choice itself is held in float32."""
    import dataclasses
    layers = tuple(dataclasses.replace(layer, mlp=dataclasses.replace(layer.mlp, top=layer.mlp.experts, groups=1, keep_groups=1))
                   if isinstance(layer.mlp, MoeMlpConfig) else layer for layer in config.layers)
    return dataclasses.replace(config, layers=layers)


def make_kalevik_folder(tmp_path, which: str, choice: bool = True) -> str:
    folder = os.path.join(str(tmp_path), f"kalevik_{which}" + ("" if choice else "_all"))
    write_model_folder(folder, CONFIGS[which] if choice else without_choice(CONFIGS[which]), SEEDS[which], dtype=torch.bfloat16, stds=STDS)
    return folder
