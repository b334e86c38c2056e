"""Tiny Zabozen configurations for the tests, each different from the others in every size, and their model folders."""
from __future__ import annotations

import os

import torch

from microllm_rocm_amd.config.zabozen import (DeltaConfig, DenseMlpConfig, LatentAttentionConfig, WindowAttentionConfig, ZabozenConfig,
                                              ZabozenLayerConfig)
from microllm_rocm_amd.weights import write_model_folder


def _latent(heads, dim, rot_dim, vdim, kv_rank, scale, base=10000.0):
    return LatentAttentionConfig(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank, scale=scale, rot_base=base,
                                 rot_dims=rot_dim)


def _window(heads, kv_heads, dim, vdim, scale, window, kv_from=None):
    return WindowAttentionConfig(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale, window=window, kv_from=kv_from)


def _layer(mixer, mlp):
    kind = {LatentAttentionConfig: "latent_attention", WindowAttentionConfig: "attention", DeltaConfig: "delta"}[type(mixer)]
    return ZabozenLayerConfig(kind, mixer, DenseMlpConfig(mlp) if mlp else None)


# A window attention of equal key and value sizes that are a multiple of 16 (in bfloat16 the paged attention's pages
# and MFMA kernels) with a borrower whose window is wider than the lender's and one whose window is narrower; a delta
# rule with three value heads a key head, unequal key and value sizes and three taps; cached latent rows of 48 elements;
# a layer without a feed-forward; a factor of 0.5 on the sublayers; a cap on the logits.
TINY_A = ZabozenConfig(
    vocab=211, width=64, norm_eps=1e-5, residual_mult=0.5, logit_softcap=12.0,
    layers=(
        _layer(_window(6, 2, 16, 16, 0.3, 19), 96),
        _layer(DeltaConfig(heads=6, kv_heads=2, dim=12, vdim=10, conv=3), 72),
        _layer(_window(4, 2, 16, 16, 0.25, 37, kv_from=0), None),
        _layer(_latent(4, 16, 8, 12, 40, 0.2), 80),
        _layer(_window(2, 2, 16, 16, 0.4, 7, kv_from=0), 56),
    ))
# A delta rule first, of one head and one tap (no kept inputs) and then one of equal head counts and key heads of 40
# channels (more than a lane's usual share); a width that is no multiple of 8; no cap on the logits and no factor on
# the sublayers; a window of one token (a query sees itself alone) and one longer than every test prompt; key and
# value sizes that differ (plain pages in either format); one key/value head for all query heads; a latent attention
# of one head.
TINY_B = ZabozenConfig(
    vocab=97, width=50, norm_eps=1e-6, residual_mult=1.0, logit_softcap=None,
    layers=(
        _layer(DeltaConfig(heads=1, kv_heads=1, dim=9, vdim=14, conv=1), 44),
        _layer(_window(3, 1, 10, 6, 0.5, 1), 36),
        _layer(_latent(1, 12, 4, 9, 18, 0.4, base=77.0), None),
        _layer(DeltaConfig(heads=3, kv_heads=3, dim=40, vdim=7, conv=2), 60),
        _layer(_window(5, 5, 6, 11, 0.35, 1000), 28),
        _layer(_window(5, 5, 6, 11, 0.2, 3, kv_from=4), None),
    ))
# Two latent attentions of unlike sizes (rows of 256 elements, the widest the MFMA kernels take, and of 42, plain pages);
# windows that end exactly on a page's edge and one position off it; a delta rule of five taps and key heads of 128
# channels; a factor above one; heads of 32 channels through the MFMA kernels with four query heads a key/value head.
TINY_C = ZabozenConfig(
    vocab=150, width=96, norm_eps=1e-6, residual_mult=1.25, logit_softcap=50.0,
    layers=(
        _layer(_latent(5, 24, 32, 40, 224, 0.15, base=500.0), 128),
        _layer(_window(8, 2, 32, 32, 0.18, 32), 64),
        _layer(DeltaConfig(heads=4, kv_heads=1, dim=128, vdim=24, conv=5), 112),
        _layer(_window(8, 2, 32, 32, 0.22, 17, kv_from=1), 48),
        _layer(_latent(3, 10, 6, 14, 36, 0.25), 80),
        _layer(_window(2, 1, 48, 48, 0.12, 65), None),
    ))

CONFIGS = {"A": TINY_A, "B": TINY_B, "C": TINY_C}
SEEDS = {"A": 31, "B": 32, "C": 33}
STDS = {"std": 0.1, "norm_std": 0.15, "bias_std": 0.4, "conv_std": 0.5}


def make_zabozen_folder(tmp_path, which: str) -> str:
    folder = os.path.join(str(tmp_path), f"zabozen_{which}")
    write_model_folder(folder, CONFIGS[which], SEEDS[which], dtype=torch.bfloat16, stds=STDS)
    return folder
