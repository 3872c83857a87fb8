"""Tiny configurations of the architecture that differ in every size and option, plus helpers
that write them as model folders into a temporary directory."""
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
# A third one with a single kv head, one group of 5 query heads, head_dim 48 (no power of two).
TINY_C = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=130, hidden_size=40,
              intermediate_size=72, num_hidden_layers=1, num_attention_heads=5, num_key_value_heads=1,
              head_dim=48, rope_theta=500.0, rms_norm_eps=1e-3, tie_word_embeddings=False,
              max_position_embeddings=512, hidden_act="silu")
# The serving head size with few of everything else: 8 query heads per kv head, head_dim 128.
TINY_D = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=515, hidden_size=136,
              intermediate_size=200, num_hidden_layers=2, num_attention_heads=8, num_key_value_heads=1,
              head_dim=128, rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=False,
              max_position_embeddings=2048, hidden_act="silu")

# Sizes that fit no vector width or tile: hidden 100 and intermediate 150 are no multiple of 8, the
# vocabulary is a prime, three query heads share one kv head.
TINY_E = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=131, hidden_size=100,
              intermediate_size=150, num_hidden_layers=2, num_attention_heads=3, num_key_value_heads=1,
              head_dim=16, rope_theta=777.0, rms_norm_eps=1e-4, tie_word_embeddings=True,
              max_position_embeddings=512, hidden_act="silu")

# A head size that is no multiple of 16 (24) and another that is no multiple of 8 (20 would not be even in halves
# of 8: 24 / 2 = 12 rotary pairs): the matrix-core kernels refuse it, the plain kernels run it in both precisions.
TINY_F = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=203, hidden_size=56,
              intermediate_size=88, num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2,
              head_dim=24, rope_theta=50000.0, rms_norm_eps=1e-5, tie_word_embeddings=True,
              max_position_embeddings=512, hidden_act="silu")

# Widths in steps of 128 (what the products of 17 to 64 rows take) at the serving head size: steps of that many
# rows run those kernels, and the two products of 1,024 inputs are split along k and added up by the norm after them.
TINY_G = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=300, hidden_size=256,
              intermediate_size=1024, num_hidden_layers=2, num_attention_heads=8, num_key_value_heads=2,
              head_dim=128, rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=False,
              max_position_embeddings=1024, hidden_act="silu")

TINY = {"G": TINY_G, "A": TINY_A, "B": TINY_B, "C": TINY_C, "D": TINY_D, "E": TINY_E, "F": TINY_F}
PAGE_SIZE = {"G": 16, "A": 4, "B": 8, "C": 16, "D": 16, "E": 16, "F": 8}


def write_model(folder: str, raw: dict, seed: int, dtype=torch.bfloat16, sharpen: float = 1.0) -> str:
    """A model folder with random weights.  `sharpen` multiplies the per-head norm weights of
    queries and keys, so that scores spread by sharpen**4 and each query singles out a few keys
    somewhere in its context: a key that is lost, misplaced or read from a wrong page then
    changes the logits by far more than rounding does."""
    import json

    from inferrs_amd.config import Qwen3Config
    from inferrs_amd.parts import generated_tensors
    from inferrs_amd.weights import random_tensors, write_safetensors
    config = Qwen3Config.from_dict(raw)
    tensors = random_tensors(generated_tensors(config.to_spec()), seed, dtype)
    if sharpen != 1.0:
        for name in tensors:
            if name.endswith("q_norm.weight") or name.endswith("k_norm.weight"):
                tensors[name] = (tensors[name].float() * sharpen).to(dtype)
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config.to_dict(), f)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors)
    return folder


def random_tokens(n: int, vocab: int, seed: int):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()
