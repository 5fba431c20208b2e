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
