"""Two tiny Llama configurations that differ in every size and option, and the
folders with random weights the tests run on."""
from __future__ import annotations

import os

import torch

import llm_rs_amd
from llm_rs_amd import LlamaConfig, random_model_tensors, write_model_folder

TINY_A = dict(
    architectures=["LlamaForCausalLM"], num_hidden_layers=2, hidden_size=64, num_attention_heads=4,
    num_key_value_heads=2, head_dim=16, intermediate_size=192, vocab_size=256, rope_theta=10000.0,
    rope_scaling=None, max_position_embeddings=128, rms_norm_eps=1e-5, tie_word_embeddings=True,
    hidden_act="silu", torch_dtype="bfloat16")

TINY_B = dict(
    architectures=["LlamaForCausalLM"], num_hidden_layers=3, hidden_size=96, num_attention_heads=3,
    num_key_value_heads=1, head_dim=32, intermediate_size=320, vocab_size=384, rope_theta=500000.0,
    rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=64),
    max_position_embeddings=512, rms_norm_eps=1e-6, tie_word_embeddings=False, hidden_act="silu",
    torch_dtype="bfloat16")

# One layer with the widths of an 8B model (and a small vocabulary): what the tiny configurations never
# reach, the kernels that wide layers get (matrix-core products of every row count, head size 128).
WIDE = dict(
    architectures=["LlamaForCausalLM"], num_hidden_layers=1, hidden_size=4096, num_attention_heads=32,
    num_key_value_heads=8, head_dim=128, intermediate_size=14336, vocab_size=512, rope_theta=500000.0,
    rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=8192),
    max_position_embeddings=1024, rms_norm_eps=1e-5, tie_word_embeddings=False, hidden_act="silu",
    torch_dtype="bfloat16")

PAGE_SIZE = {"A": 4, "B": 16, "W": 16}
CONFIGS = {"A": TINY_A, "B": TINY_B, "W": WIDE}


def make_folder(tmp_path, which: str, seed: int = 0, dtype=torch.bfloat16) -> str:
    cfg = LlamaConfig.from_dict(CONFIGS[which])
    folder = os.path.join(str(tmp_path), f"tiny_{which}_{seed}")
    write_model_folder(folder, cfg, random_model_tensors(cfg, seed, dtype=dtype))
    return folder
