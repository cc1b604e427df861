"""Tiny configurations and helpers shared by the tests.

The first three configurations differ in every size and option: layer count, width, head
counts and grouping (2:1, 3:1 multi-query, 1:1), head size (16, 32, 48), feed-forward
width, vocabulary (a power of two, a multiple of 128, an odd number), rope base and
scaling, tied or untied head, norm eps, biases.
"""

from __future__ import annotations

import random
from pathlib import Path

import torch

TINY_A = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 4, "num_key_value_heads": 2,
    "head_dim": 16, "intermediate_size": 128, "vocab_size": 256, "rope_theta": 10000.0,
    "rope_scaling": None, "tie_word_embeddings": False, "rms_norm_eps": 1e-5,
    "max_position_embeddings": 128, "hidden_act": "silu",
}
TINY_A_PAGE = 16

TINY_B = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 3, "hidden_size": 96, "num_attention_heads": 3, "num_key_value_heads": 1,
    "head_dim": 32, "intermediate_size": 256, "vocab_size": 384, "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                     "high_freq_factor": 4.0, "original_max_position_embeddings": 64},
    "tie_word_embeddings": True, "rms_norm_eps": 1e-6, "max_position_embeddings": 256,
    "hidden_act": "silu",
}
TINY_B_PAGE = 8

TINY_C = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 2, "hidden_size": 80, "num_attention_heads": 5, "num_key_value_heads": 5,
    "head_dim": 48, "intermediate_size": 176, "vocab_size": 331, "rope_theta": 25000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 4.0, "low_freq_factor": 1.0,
                     "high_freq_factor": 2.0, "original_max_position_embeddings": 32},
    "tie_word_embeddings": False, "rms_norm_eps": 3e-6, "max_position_embeddings": 512,
    "attention_bias": True, "mlp_bias": True, "hidden_act": "silu",
}
TINY_C_PAGE = 32

# head size 64, four query heads per kv head, pages of 16: the shape class that the
# matrix-core attention kernels serve in bfloat16 (the other three run the general kernel)
TINY_D = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 2, "hidden_size": 128, "num_attention_heads": 8, "num_key_value_heads": 2,
    "head_dim": 64, "intermediate_size": 192, "vocab_size": 512, "rope_theta": 1000000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 2.0, "low_freq_factor": 1.0,
                     "high_freq_factor": 8.0, "original_max_position_embeddings": 128},
    "tie_word_embeddings": False, "rms_norm_eps": 1e-5, "max_position_embeddings": 1024,
    "hidden_act": "silu",
}
TINY_D_PAGE = 16

# wide enough (multiples of 512) for the products of a few dozen rows that share their rows
# through LDS; not one of the configurations that every test runs
WIDE = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 2, "hidden_size": 512, "num_attention_heads": 8, "num_key_value_heads": 2,
    "head_dim": 64, "intermediate_size": 1024, "vocab_size": 640, "rope_theta": 10000.0,
    "tie_word_embeddings": False, "rms_norm_eps": 1e-6, "max_position_embeddings": 512,
    "hidden_act": "silu", "mlp_bias": True,
}
WIDE_PAGE = 16

CONFIGS = {"A": (TINY_A, TINY_A_PAGE), "B": (TINY_B, TINY_B_PAGE), "C": (TINY_C, TINY_C_PAGE),
           "D": (TINY_D, TINY_D_PAGE)}


def make_model_dir(folder: Path, config: dict, seed: int, dtype=torch.bfloat16, bias_std: float = 0.05) -> Path:
    """A model folder made by the product's random-weights mode.  Biases, which that
    mode zeroes, are overwritten with noise so that a dropped bias shows."""
    from safetensors.torch import load_file, save_file

    from kvcore_amd.weights.loader import write_random_model

    write_random_model(folder, config, seed, dtype=dtype)
    if config.get("attention_bias") or config.get("mlp_bias"):
        path = folder / "model.safetensors"
        tensors = load_file(str(path))
        gen = torch.Generator().manual_seed(seed + 1)
        for name in list(tensors):
            if name.endswith(".bias"):
                tensors[name] = (torch.randn(tensors[name].shape, generator=gen) * bias_std).to(tensors[name].dtype)
        save_file(tensors, str(path))
    return folder


def random_tokens(n: int, vocab: int, seed: int) -> list[int]:
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(n)]


TINY_LOGIT_RMS = 0.2  # root mean square of the tiny models' logits (0.16 to 0.24)


def tolerance(dtype: torch.dtype, logit_rms: float = TINY_LOGIT_RMS, sum_length: int = 0) -> dict:
    """Bounds on |engine - plain| for logits of the tiny models (|logit| is about 0.1 to
    1).  float32: both sides sum the same products in different orders, a few 1e-7
    relative per operation over a few hundred operations.  bfloat16: activations are
    rounded to 8 bits of mantissa (2^-9 relative) at about ten places per layer.
    The absolute part is 4% of the logits' root mean square (a small logit's error comes
    from the large terms that cancel in it): a model with larger logits says so.

    ``sum_length``: the longest sum of products in the model (its widest K), for models far
    wider than the tiny ones.  A float32 sum of K terms taken in order errs, relative to its
    result, in proportion to sqrt(K) (the rounding errors of the partial sums add up like a
    random walk of steps that grow with the partial sums); the tiny models' sums have a few
    hundred terms, so the float32 bound grows by sqrt(K / 1024) beyond 1024 terms (3.7 times
    at the 14336 of Llama-3-8B's feed-forward; the worst error measured there, over 2e7
    logits, is 0.3 of that bound, and a product in any reduced precision would miss it by a
    factor of ten or more).  bfloat16 sums are float32 sums of products whose inputs were
    rounded first: that rounding dominates whatever the length, so its bound stays."""
    scale = max(1.0, logit_rms / TINY_LOGIT_RMS)
    if dtype == torch.float32:
        scale *= max(1.0, (sum_length / 1024) ** 0.5)
        return dict(atol=5e-6 * scale, rtol=2e-5)
    return dict(atol=8e-3 * scale, rtol=2e-2)


ERROR_STATS: dict[str, list[float]] = {}


def note_error(label: str, ratio: float, abs_err: float) -> None:
    """Keeps the worst error seen per label (largest fraction of its bound, largest
    absolute value); the terminal summary prints them."""
    cur = ERROR_STATS.setdefault(label, [0.0, 0.0])
    cur[0] = max(cur[0], ratio)
    cur[1] = max(cur[1], abs_err)
