"""Tiny Qwen2 configurations that differ in every size and option, and helpers that build
their random model folders and the plain implementation's logits for them."""

from __future__ import annotations

import json
import random
from pathlib import Path

import torch

from plain import qwen2_plain as plain

#: A: grouped heads (G=2), tied head, no window, page 16.
CONFIG_A = {
    "architectures": ["Qwen2ForCausalLM"],
    "model_type": "qwen2",
    "hidden_size": 64,
    "num_hidden_layers": 2,
    "num_attention_heads": 4,
    "num_key_value_heads": 2,
    "intermediate_size": 128,
    "vocab_size": 256,
    "rope_theta": 10000.0,
    "rms_norm_eps": 1e-6,
    "tie_word_embeddings": True,
    "use_sliding_window": False,
    "max_position_embeddings": 128,
}
PAGE_A = 16

#: B: one KV head for three query heads, head size 32, sizes that are no power of two,
#: untied head, window 16 from layer 1 on (layer 0 keeps all keys), page 8.
CONFIG_B = {
    "architectures": ["Qwen2ForCausalLM"],
    "model_type": "qwen2",
    "hidden_size": 96,
    "num_hidden_layers": 3,
    "num_attention_heads": 3,
    "num_key_value_heads": 1,
    "intermediate_size": 200,
    "vocab_size": 320,
    "rope_theta": 1000000.0,
    "rms_norm_eps": 1e-5,
    "tie_word_embeddings": False,
    "use_sliding_window": True,
    "sliding_window": 16,
    "max_window_layers": 1,
    "max_position_embeddings": 256,
}
PAGE_B = 8

#: C: as many KV heads as query heads, head size 48 with heads * head size != hidden,
#: an odd vocabulary, linear position scaling, every layer windowed (window 40), page 32.
CONFIG_C = {
    "architectures": ["Qwen2ForCausalLM"],
    "model_type": "qwen2",
    "hidden_size": 80,
    "num_hidden_layers": 2,
    "num_attention_heads": 5,
    "num_key_value_heads": 5,
    "head_dim": 48,
    "intermediate_size": 72,
    "vocab_size": 301,
    "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "linear", "factor": 2.0},
    "rms_norm_eps": 3e-6,
    "tie_word_embeddings": False,
    "use_sliding_window": True,
    "sliding_window": 40,
    "max_window_layers": 0,
    "max_position_embeddings": 512,
}
PAGE_C = 32

#: D: sizes that 16-byte accesses do not divide: a width of 100, a feed-forward of 172 and five
#: heads of 20 on one KV head (every product's K is 4 more than a multiple of 8, the head size is
#: no multiple of 8 or 16), an odd vocabulary, tied head, a window of 24 in the second layer.
CONFIG_D = {
    "architectures": ["Qwen2ForCausalLM"],
    "model_type": "qwen2",
    "hidden_size": 100,
    "num_hidden_layers": 2,
    "num_attention_heads": 5,
    "num_key_value_heads": 1,
    "intermediate_size": 172,
    "vocab_size": 333,
    "rope_theta": 50000.0,
    "rms_norm_eps": 2e-5,
    "tie_word_embeddings": True,
    "use_sliding_window": True,
    "sliding_window": 24,
    "max_window_layers": 1,
    "max_position_embeddings": 192,
}
PAGE_D = 16

TINY = {"A": (CONFIG_A, 0, PAGE_A), "B": (CONFIG_B, 1, PAGE_B), "C": (CONFIG_C, 2, PAGE_C), "D": (CONFIG_D, 3, PAGE_D)}


#: A wider spread of the weights for 32-bit comparisons.  With the usual 0.02 a model this small
#: hardly mixes its inputs (greedy generation repeats one token, attention weights are near
#: uniform); with 0.15 every layer matters to the next token, so a fault in any of them shows.
WIDE_STD = 0.15
#: The spread for bfloat16 comparisons.  Rounding error grows faster than the spread (peaked
#: attention turns a rounded score into a moved weight): against the 32-bit plain
#: implementation the engine is off by up to 0.7% of a position's largest logit at 0.05, 1.6% at
#: 0.1 and 3.9% at 0.15 (hidden size 64 to 96), and the reference's own formulas evaluated in
#: bfloat16 (the plain implementation on bfloat16 tensors) by 1.6-2.8% at 0.1.  At 0.1 a lost
#: page of one layer's cache still moves the logits by 24-100%.  What matters is the gain of a
#: projection, spread x sqrt(hidden size): a model 200 wide at 0.1 is off by 3.4% in the
#: reference's own bfloat16 arithmetic.  So the spread is 0.1 at 64 wide and falls with the width.
BF16_STD = 0.1
BF16_GAIN = BF16_STD * 64 ** 0.5


def std_for(dtype: torch.dtype, hidden_size: int = 64) -> float:
    return WIDE_STD if dtype == torch.float32 else BF16_GAIN / hidden_size ** 0.5


def make_model_dir(folder: Path, config: dict, seed: int, dtype: torch.dtype = torch.float32, std: float = 0.02) -> Path:
    from turboserve_amd.weights.random_init import write_random_model

    return write_random_model(config, folder, seed=seed, dtype=dtype, std=std)


def read_model_dir(folder: Path) -> tuple[dict, dict[str, torch.Tensor]]:
    """``(config.json mapping, tensors as float32)`` read without any engine code."""
    from safetensors.torch import load_file

    config = json.loads((Path(folder) / "config.json").read_text())
    tensors = load_file(str(Path(folder) / "model.safetensors"))
    return config, plain.as_float32(tensors)


def random_tokens(vocab: int, length: int, seed: int) -> list[int]:
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(length)]


def plain_logits(folder: Path, tokens: list[int]) -> torch.Tensor:
    config, tensors = read_model_dir(folder)
    return plain.forward_logits(config, tensors, tokens)
