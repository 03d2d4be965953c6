"""Tiny Llama configurations for the tests and a helper that writes their model folders.

A and B differ in every size and option: layers, width, heads and groups, head
size, feed-forward width (no power of two), vocabulary, eps, theta, rope scaling,
tied or separate head, norm weights.  C adds a sliding window on some layers, a
head size that is no power of two and an explicit head_dim.
"""
import torch

from infernum_amd.config import LlamaConfig
from infernum_amd.weights import write_random_model

TINY_A = dict(
    model_type="llama", num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2,
    intermediate_size=176, vocab_size=256, rope_theta=10000.0, rms_norm_eps=1e-5, tie_word_embeddings=True,
    max_position_embeddings=512,
)
TINY_B = dict(
    model_type="llama", num_hidden_layers=3, hidden_size=128, num_attention_heads=4, num_key_value_heads=1,
    intermediate_size=352, vocab_size=384, rope_theta=500000.0, rms_norm_eps=1e-6, tie_word_embeddings=False,
    max_position_embeddings=256,
    rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=64),
)
TINY_C = dict(
    model_type="mistral", num_hidden_layers=3, hidden_size=96, num_attention_heads=6, num_key_value_heads=3,
    head_dim=48, intermediate_size=200, vocab_size=250, rope_theta=20000.0, rms_norm_eps=3e-6,
    tie_word_embeddings=False, max_position_embeddings=1024, sliding_window=24, use_sliding_window=True,
    max_window_layers=2,
)

# D: sizes that no fast kernel takes: a head size that is no multiple of 16, a width and a feed-forward
# width that are no multiples of 4, an odd vocabulary: the plain kernels (or the library product) must serve.
TINY_D = dict(
    model_type="llama", num_hidden_layers=2, hidden_size=100, num_attention_heads=5, num_key_value_heads=5,
    head_dim=20, intermediate_size=150, vocab_size=333, rope_theta=10000.0, rms_norm_eps=1e-5,
    tie_word_embeddings=True, max_position_embeddings=512,
)

SPEC_KW = {
    "A": dict(norm_init=("ones",)),
    "B": dict(norm_init=("uniform", 0.5, 1.5)),
    "C": dict(norm_init=("uniform", 0.5, 1.5), init_std=0.05),
    "D": dict(norm_init=("uniform", 0.5, 1.5), init_std=0.05),
}
RAW = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "D": TINY_D}
SEED = {"A": 0, "B": 1, "C": 2, "D": 3}


def tiny_config(name: str) -> LlamaConfig:
    return LlamaConfig.from_dict(RAW[name], where=f"tiny {name}")


def write_tiny(name: str, out_dir: str, dtype=torch.float32) -> str:
    return write_random_model(tiny_config(name), out_dir, SEED[name], dtype=dtype, **SPEC_KW[name])
