"""Two tiny Llama configurations that differ in every size and option, and their random weights.

A: 2 layers, width 64, 4 heads over 2 key/value heads of size 16, feed-forward 176, vocabulary 256, theta 1e4 without
   scaling, eps 1e-5, tied head, 128 positions, pages of 4 tokens, seed 0.
B: 3 layers, width 192, 6 heads over 1 key/value head (MQA) of size 32, feed-forward 512, vocabulary 1000, theta 5e5 with
   llama3 scaling (8, 1, 4, 64), eps 1e-6, own head, 256 positions, pages of 8 tokens, seed 1.
"""

from __future__ import annotations

import torch

TINY = {
    "A": dict(
        cfg=dict(architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=256, hidden_size=64, intermediate_size=176,
                 num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, head_dim=16, rms_norm_eps=1e-5,
                 rope_theta=10000.0, max_position_embeddings=128, tie_word_embeddings=True),
        seed=0, page=4, prompts=(5, 17, 33)),
    "B": dict(
        cfg=dict(architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=1000, hidden_size=192, intermediate_size=512,
                 num_hidden_layers=3, num_attention_heads=6, num_key_value_heads=1, head_dim=32, rms_norm_eps=1e-6,
                 rope_theta=500000.0, max_position_embeddings=256, tie_word_embeddings=False,
                 rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                   original_max_position_embeddings=64)),
        seed=1, page=8, prompts=(1, 9, 40, 100, 130)),
}


def write_folder(folder, name: str, dtype=torch.float32):
    from nanospec_amd.config import LlamaConfig
    from nanospec_amd.weights import write_model_folder

    config = LlamaConfig.from_hf(TINY[name]["cfg"])
    return write_model_folder(folder, config, TINY[name]["seed"], dtype)


def random_tokens(n: int, vocab: int, seed: int) -> list[int]:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


# bf16 has an 8-bit significand: one ulp is 2^-7 of the value; logits are judged against their row's largest
# magnitude (reference: tests/conftest.py:20-32).
BF16_ULP = 2.0 ** -7


def ulps_of_row_max(ours: torch.Tensor, ref: torch.Tensor) -> torch.Tensor:
    """Per row: largest |ours - ref| in bf16 ulps of the reference row's largest magnitude."""
    scale = BF16_ULP * ref.float().abs().amax(-1, keepdim=True).clamp_min(1e-30)
    return ((ours.float() - ref.float()).abs() / scale).amax(-1)
