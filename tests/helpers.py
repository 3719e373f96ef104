"""Tiny configurations and model folders shared by the tests.

The two configurations differ in every size and option: layers, width, heads and their grouping,
head size, feed-forward width, vocabulary (neither a power of two in B), rope base, llama3 scaling
or none, tied or untied head, the norms' eps, and the dtype their weights are stored in.
"""

from __future__ import annotations

import random

import torch

from tinyserve_llm_amd.config import LlamaConfig, RopeScaling
from tinyserve_llm_amd.weights.random_init import write_random_model

TINY_A = LlamaConfig(
    vocab_size=256, hidden_size=64, intermediate_size=128, num_hidden_layers=2, num_attention_heads=4,
    num_key_value_heads=2, head_dim=16, max_position_embeddings=192, rms_norm_eps=1e-5, rope_theta=10000.0,
    rope_scaling=None, tie_word_embeddings=True, eos_token_id=255)

TINY_B = LlamaConfig(
    vocab_size=384, hidden_size=96, intermediate_size=160, num_hidden_layers=3, num_attention_heads=3,
    num_key_value_heads=1, head_dim=32, max_position_embeddings=320, rms_norm_eps=1e-6, rope_theta=500000.0,
    rope_scaling=RopeScaling(factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                             original_max_position_embeddings=64),
    tie_word_embeddings=False, eos_token_id=383)

CONFIGS = {"A": (TINY_A, 0, torch.float32), "B": (TINY_B, 1, torch.bfloat16)}


def make_folder(tmp_path_factory, name: str) -> str:
    config, seed, stored = CONFIGS[name]
    folder = tmp_path_factory.mktemp(f"tiny_{name}")
    write_random_model(str(folder), config, seed, stored)
    return str(folder)


def prompt(seed: int, length: int, vocab: int) -> list[int]:
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(length)]


def rugezen_configs():
    """Two small Rugezen configurations that differ from each other in every size and option: key/value
    grouping, key and value head sizes (equal or not), how much of a head turns, caps, layer order, a
    looped stretch (three passes over two layers, or none), a layer without feed-forward, eps, the
    residual multiplier, and widths that are no multiples of 64."""
    from tinyserve_llm_amd.config.rugezen import RugezenAttention, RugezenConfig, RugezenLayer, RugezenMinGRU
    att_p = RugezenAttention(heads=4, kv_heads=2, dim=32, vdim=48, rot_dims=16, rot_base=10000.0, scale=0.31, softcap=3.0)
    att_q = RugezenAttention(heads=2, kv_heads=2, dim=16, vdim=16, rot_dims=16, rot_base=700.0, scale=0.25, softcap=30.0)
    att_r = RugezenAttention(heads=6, kv_heads=1, dim=24, vdim=8, rot_dims=4, rot_base=50000.0, scale=0.2, softcap=1.5)
    att_s = RugezenAttention(heads=4, kv_heads=2, dim=64, vdim=64, rot_dims=32, rot_base=1000.0, scale=0.15, softcap=2.5)
    P = RugezenConfig(vocab=200, width=80, norm_eps=1e-6, residual_mult=0.37, loop_start=0, loop_stop=2, loop_times=3,
                      layers=(RugezenLayer("mingru", RugezenMinGRU(width=72), 96), RugezenLayer("attention", att_p, 144),
                              RugezenLayer("attention", att_r, None)))
    Q = RugezenConfig(vocab=131, width=48, norm_eps=1e-4, residual_mult=1.0,
                      layers=(RugezenLayer("attention", att_q, 64), RugezenLayer("mingru", RugezenMinGRU(width=100), None),
                              RugezenLayer("mingru", RugezenMinGRU(width=16), 40), RugezenLayer("attention", att_s, 56)))
    # sizes that are multiples of nothing in particular: no kernel's fast path takes them
    att_t = RugezenAttention(heads=3, kv_heads=1, dim=20, vdim=12, rot_dims=6, rot_base=100.0, scale=0.3, softcap=5.0)
    R = RugezenConfig(vocab=77, width=99, norm_eps=1e-5, residual_mult=0.8, loop_start=1, loop_stop=2, loop_times=2,
                      layers=(RugezenLayer("attention", att_t, 52), RugezenLayer("mingru", RugezenMinGRU(width=35), 44)))
    # a width that the weight-streaming kernels take (steps of few rows then run the fused forms), heads of a
    # matrix-core size
    att_u = RugezenAttention(heads=8, kv_heads=2, dim=64, vdim=64, rot_dims=64, rot_base=20000.0, scale=0.11, softcap=8.0)
    S = RugezenConfig(vocab=300, width=512, norm_eps=1e-6, residual_mult=0.45, loop_start=0, loop_stop=1, loop_times=2,
                      layers=(RugezenLayer("attention", att_u, 640), RugezenLayer("mingru", RugezenMinGRU(width=256), 768)))
    return {"P": (P, 3), "Q": (Q, 4), "R": (R, 5), "S": (S, 6)}
