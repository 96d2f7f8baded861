"""Tiny Makuzen configurations of the tests.

A: three layers that differ in every size: a window of 24 with scaled rotation and two of five experts plus a shared
   one; no window, plain rotation and no feed-forward; a window of 9, one of three experts, no shared expert.
B: values that are often equal made different, and values that are often above one made one: one head, three of
   four experts, embedding scale and residual factor 1, a window of one (a token sees only itself) beside one longer
   than any sequence, plain widths unlike value widths, query rank unlike key/value rank.
C: sizes in whole tiles of the matrix cores (latent 64 + 32 rotated, heads of 32), windows of 40 (no multiple of a
   page) and 32 (two pages of 16), sequences of a few hundred tokens.
D: sizes that are multiples of nothing (width 100, latent 36 + 6, five heads of 12 + 6, values 20 wide, vocabulary 97).
"""
import os

import torch

from gesso_amd.config import LatentAttentionConfig, MakuzenConfig, MakuzenLayer, TableMoEConfig, YarnScaling
from gesso_amd.weights import write_model_folder

STD = 0.15


def _mixer(heads, dim, rot, vdim, q_rank, kv_rank, scale, base=1e4, scaling=None, window=None):
    return LatentAttentionConfig(heads=heads, dim=dim, rot_dim=rot, vdim=vdim, q_rank=q_rank, kv_rank=kv_rank,
                                 scale=scale, rot_base=base, scaling=scaling, window=window)


MK_A = MakuzenConfig(vocab=211, width=96, embedding_scale=2.0, norm_eps=1e-5, residual_mult=0.7, max_position=512, layers=(
    MakuzenLayer(_mixer(3, 24, 8, 16, 40, 48, 0.2, 1e4, YarnScaling(4.0, 64.0, 8.0, 2.0), 24), TableMoEConfig(5, 2, 40, 56)),
    MakuzenLayer(_mixer(2, 32, 16, 32, 32, 64, 0.15, 5e5), None),
    MakuzenLayer(_mixer(4, 8, 4, 8, 24, 32, 0.3, 1e3, YarnScaling(2.0, 32.0, 4.0, 1.0), 9), TableMoEConfig(3, 1, 24, None))))

MK_B = MakuzenConfig(vocab=150, width=64, embedding_scale=1.0, norm_eps=1e-6, residual_mult=1.0, max_position=512, layers=(
    MakuzenLayer(_mixer(1, 16, 8, 24, 20, 40, 0.25, 1e4, None, 1), TableMoEConfig(4, 3, 16, 48)),
    MakuzenLayer(_mixer(1, 40, 2, 8, 48, 16, 0.1, 1e5, YarnScaling(8.0, 16.0, 2.0, 1.0), 1000), TableMoEConfig(4, 4, 8, 8))))

MK_C = MakuzenConfig(vocab=320, width=128, embedding_scale=0.5, norm_eps=1e-5, residual_mult=0.5, max_position=1024, layers=(
    MakuzenLayer(_mixer(4, 32, 32, 32, 64, 64, 0.125, 5e5, YarnScaling(2.0, 128.0, 32.0, 1.0), 40), TableMoEConfig(8, 2, 32, 64)),
    MakuzenLayer(_mixer(8, 16, 32, 16, 32, 64, 0.15, 1e4, None, 32), TableMoEConfig(6, 2, 64, 32)),
    MakuzenLayer(_mixer(2, 64, 32, 64, 96, 64, 0.1, 1e4, None, None), TableMoEConfig(4, 1, 32, 32))))

MK_D = MakuzenConfig(vocab=97, width=100, embedding_scale=1.5, norm_eps=1e-4, residual_mult=0.3, max_position=384, layers=(
    MakuzenLayer(_mixer(5, 12, 6, 20, 28, 36, 0.2, 3e4, YarnScaling(3.0, 40.0, 6.0, 1.5), 17), TableMoEConfig(7, 3, 20, 36)),
    MakuzenLayer(_mixer(5, 12, 6, 20, 28, 36, 0.2, 3e4, None, 50), None)))

CONFIGS = {"A": (MK_A, 20), "B": (MK_B, 21), "C": (MK_C, 22), "D": (MK_D, 23)}


def write_tiny(root: str, name: str, dtype=torch.float32) -> str:
    cfg, seed = CONFIGS[name]
    d = os.path.join(root, f"makuzen_{name}_{str(dtype).split('.')[-1]}")
    if not os.path.exists(os.path.join(d, "model.safetensors")):
        write_model_folder(d, cfg, seed, dtype, std=STD)
    return d
