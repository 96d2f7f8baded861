"""Tiny Fazezen configurations of the tests.

A: a lightning layer, a pair without a feed-forward (keys turned in part, stretched frequencies, runs of 24, two query
   heads a key head), a lightning layer with one head.
B: values that are often equal made different and values that are often one made otherwise: a pair first; as many key
   heads as query heads; keys wider than values on the left and narrower on the right; another base on the right than
   on the left; runs of 7 (no multiple of a page) and of 1 (a token sees itself and the sink only); a decay of exactly
   1 and one of 0; scales of the two sides far apart; a left side without any turn and a right side without one.
C: sizes in whole tiles of the matrix cores (heads of 64 and 128), runs of 64 and of 128, sequences of a few hundred.
D: sizes that are multiples of nothing (width 100, vocabulary 97, heads of 12, 10 and 14, runs of 17), and a pair whose
   left side has no runs at all.
"""
import os

import torch

from gesso_amd.config import (ChunkedAttentionConfig, DenseConfig, FazezenConfig, FazezenLayer, LightningConfig,
                              ParallelConfig, RetentionConfig, Rotation, Stretch)
from gesso_amd.weights import write_model_folder

STD = 0.15


def light(heads, dim, vdim, decay, ff):
    return FazezenLayer("lightning", LightningConfig(heads, dim, vdim, tuple(decay)), None if ff is None else DenseConfig(ff))


def pair(left, right, ls, rs, ff):
    return FazezenLayer("parallel", ParallelConfig(left, right, ls, rs), None if ff is None else DenseConfig(ff))


FZ_A = FazezenConfig(vocab=211, width=96, norm_eps=1e-5, max_position=512, layers=(
    light(3, 24, 16, (0.5, 0.9, 0.99), 80),
    pair(ChunkedAttentionConfig(4, 2, 24, 16, 0.2, Rotation(1e4, 16, Stretch(4.0, 1.0, 4.0, 64.0)), 24),
         RetentionConfig(2, 16, 24, (0.9, 0.97), Rotation(1e4, 8)), 1.3, 0.8, None),
    light(1, 40, 48, (0.95,), 40)))

FZ_B = FazezenConfig(vocab=150, width=64, norm_eps=1e-6, max_position=512, layers=(
    pair(ChunkedAttentionConfig(2, 2, 16, 8, 0.3, Rotation(1e5, 16, Stretch(8.0, 2.0, 6.0, 16.0)), 7),
         RetentionConfig(3, 8, 16, (1.0, 0.0, 0.8), Rotation(1e3, 8, Stretch(2.0, 1.0, 3.0, 32.0))), 0.25, 2.0, 48),
    light(2, 8, 24, (0.999, 0.7), None),
    pair(ChunkedAttentionConfig(3, 1, 12, 20, 0.15, None, 1),
         RetentionConfig(1, 24, 8, (0.9,), None), 1.0, 1.0, 24),
    pair(ChunkedAttentionConfig(1, 1, 8, 4, 0.5, Rotation(50.0, 4), 1000),
         RetentionConfig(2, 4, 4, (0.6, 0.95), Rotation(7.0, 4)), 0.7, 1.1, 16)))

FZ_C = FazezenConfig(vocab=320, width=128, norm_eps=1e-5, max_position=1024, layers=(
    light(2, 64, 64, (0.97, 0.995), 256),
    pair(ChunkedAttentionConfig(4, 2, 64, 64, 0.125, Rotation(5e5, 64, Stretch(4.0, 1.0, 4.0, 128.0)), 64),
         RetentionConfig(2, 64, 128, (0.98, 0.999), Rotation(5e5, 64)), 1.2, 0.9, 128),
    light(1, 128, 128, (0.99,), 128),
    pair(ChunkedAttentionConfig(2, 1, 128, 128, 0.09, Rotation(1e4, 128), 128),
         RetentionConfig(4, 32, 64, (0.9, 0.95, 0.99, 0.999), Rotation(1e4, 32)), 0.9, 1.1, 64)))

FZ_D = FazezenConfig(vocab=97, width=100, norm_eps=1e-4, max_position=384, layers=(
    light(5, 12, 20, (0.3, 0.6, 0.9, 0.97, 0.999), 36),
    pair(ChunkedAttentionConfig(6, 3, 10, 14, 0.3, Rotation(3e4, 6, Stretch(3.0, 1.5, 5.0, 40.0)), 17),
         RetentionConfig(5, 6, 10, (0.5, 0.8, 0.9, 0.95, 0.99), Rotation(3e4, 2)), 1.5, 0.5, 52),
    pair(ChunkedAttentionConfig(2, 1, 18, 6, 0.2, Rotation(1e4, 18), None),
         RetentionConfig(2, 10, 18, (0.85, 0.98), Rotation(2e4, 10)), 0.6, 1.4, None)))

CONFIGS = {"A": (FZ_A, 40), "B": (FZ_B, 41), "C": (FZ_C, 42), "D": (FZ_D, 43)}


def write_tiny(root: str, name: str, dtype=torch.float32) -> str:
    cfg, seed = CONFIGS[name]
    d = os.path.join(root, f"fazezen_{name}_{str(dtype).split('.')[-1]}")
    if not os.path.exists(os.path.join(d, "model.safetensors")):
        write_model_folder(d, cfg, seed, dtype, std=STD)
    return d
