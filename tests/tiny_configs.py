"""Two tiny configurations of the architecture that differ in every size and option, plus
helpers that write them as model folders into a temporary directory."""
from __future__ import annotations

import os

import torch

# layers, hidden, heads, kv heads, head_dim (n_heads*head_dim == hidden vs !=), intermediate,
# vocab (one a power of two, one not), theta, eps, tied vs untied head, max positions.
TINY_A = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=256, hidden_size=64,
              intermediate_size=128, num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2,
              head_dim=16, rope_theta=10000.0, rms_norm_eps=1e-6, tie_word_embeddings=True,
              max_position_embeddings=512, hidden_act="silu")
TINY_B = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=387, hidden_size=96,
              intermediate_size=160, num_hidden_layers=3, num_attention_heads=6, num_key_value_heads=3,
              head_dim=32, rope_theta=1000000.0, rms_norm_eps=1e-5, tie_word_embeddings=False,
              max_position_embeddings=1024, hidden_act="silu")
# A third one with a single kv head, one query head per group of 5, head_dim 48 (no power of two).
TINY_C = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=130, hidden_size=40,
              intermediate_size=72, num_hidden_layers=1, num_attention_heads=5, num_key_value_heads=1,
              head_dim=48, rope_theta=500.0, rms_norm_eps=1e-3, tie_word_embeddings=False,
              max_position_embeddings=512, hidden_act="silu")

TINY = {"A": TINY_A, "B": TINY_B, "C": TINY_C}
PAGE_SIZE = {"A": 4, "B": 8, "C": 16}


def write_model(folder: str, raw: dict, seed: int, dtype=torch.bfloat16) -> str:
    from inferrs_amd.config import Qwen3Config
    from inferrs_amd.weights import write_random_model
    return write_random_model(folder, Qwen3Config.from_dict(raw), seed, dtype)


def random_tokens(n: int, vocab: int, seed: int):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()
