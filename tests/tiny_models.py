"""The tiny configurations the tests run: two Llama shapes that differ in every size
and option, and helpers that write them as model folders with random weights."""
from __future__ import annotations

import torch

# A: 2 layers, 4 query / 2 kv heads of 16, tied head, plain rope, eps 1e-5.
TINY_A = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "hidden_size": 64, "intermediate_size": 176, "num_hidden_layers": 2,
    "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 16,
    "vocab_size": 256, "max_position_embeddings": 128, "rms_norm_eps": 1e-5,
    "rope_theta": 10000.0, "rope_scaling": None, "tie_word_embeddings": True,
}
A_INIT = dict(seed=0, std=0.02, norm_mean=1.0, norm_std=0.0)

# B: 3 layers, 3 query heads on 1 kv head of 32 (q_dim == hidden), untied head, llama3 rope
# scaling with a small original length so that all three wavelength bands occur, eps 1e-6.
TINY_B = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "hidden_size": 96, "intermediate_size": 256, "num_hidden_layers": 3,
    "num_attention_heads": 3, "num_key_value_heads": 1, "head_dim": 32,
    "vocab_size": 384, "max_position_embeddings": 256, "rms_norm_eps": 1e-6,
    "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 32.0, "low_freq_factor": 1.0,
                     "high_freq_factor": 4.0, "original_max_position_embeddings": 64},
    "tie_word_embeddings": False,
}
B_INIT = dict(seed=1, std=0.05, norm_mean=1.0, norm_std=0.1)

# C: longer contexts, head size 64 and 48 (a multiple of 16 that is no power of two comes with D)
TINY_C = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "hidden_size": 128, "intermediate_size": 320, "num_hidden_layers": 2,
    "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 64,
    "vocab_size": 500, "max_position_embeddings": 2048, "rms_norm_eps": 1e-5,
    "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                     "high_freq_factor": 4.0, "original_max_position_embeddings": 512},
    "tie_word_embeddings": True,
}
C_INIT = dict(seed=2, std=0.04, norm_mean=1.0, norm_std=0.05)

# D: head size 48, 6 query heads in 2 groups, width 144, vocabulary 331 (odd), no scaling
TINY_D = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "hidden_size": 144, "intermediate_size": 208, "num_hidden_layers": 2,
    "num_attention_heads": 6, "num_key_value_heads": 2, "head_dim": 48,
    "vocab_size": 331, "max_position_embeddings": 512, "rms_norm_eps": 1e-5,
    "rope_theta": 10000.0, "tie_word_embeddings": False,
}
D_INIT = dict(seed=3, std=0.05, norm_mean=1.0, norm_std=0.1)


# E: sizes that no fast kernel takes whole: width 72 with 3 heads of 16 (q_dim 48 != width), feed-forward 100
# (no multiple of 8 or 16), vocabulary 257, 4 layers, MQA
TINY_E = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "hidden_size": 72, "intermediate_size": 100, "num_hidden_layers": 4,
    "num_attention_heads": 3, "num_key_value_heads": 1, "head_dim": 16,
    "vocab_size": 257, "max_position_embeddings": 300, "rms_norm_eps": 1e-5,
    "rope_theta": 10000.0, "tie_word_embeddings": True,
}
E_INIT = dict(seed=4, std=0.06, norm_mean=1.0, norm_std=0.1)


# F: head size 128 with four query heads per key/value head (the sizes of the larger Llama models'
# attention), untied head, rope scaling with another factor
TINY_F = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "hidden_size": 192, "intermediate_size": 272, "num_hidden_layers": 2,
    "num_attention_heads": 4, "num_key_value_heads": 1, "head_dim": 128,
    "vocab_size": 409, "max_position_embeddings": 1024, "rms_norm_eps": 1e-6,
    "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 16.0, "low_freq_factor": 1.0,
                     "high_freq_factor": 4.0, "original_max_position_embeddings": 256},
    "tie_word_embeddings": False,
}
F_INIT = dict(seed=6, std=0.04, norm_mean=1.0, norm_std=0.1)


def make_model_dir(tmp_path, cfg: dict, init: dict, dtype=torch.bfloat16) -> str:
    from llmengine.weights import write_random_model
    return write_random_model(cfg, str(tmp_path), init["seed"], dtype, init["std"], init["norm_mean"],
                              init["norm_std"])


def random_tokens(n: int, vocab: int, seed: int) -> list[int]:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()
