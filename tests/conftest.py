import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


# Two tiny configurations of the architecture that differ in every size and option.
TINY_A = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
    "vocab_size": 256, "hidden_size": 64, "num_hidden_layers": 4,
    "layer_types": ["conv", "full_attention", "conv", "full_attention"],
    "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 16,
    "intermediate_size": 192, "block_auto_adjust_ff_dim": False,
    "rope_theta": 10000.0, "conv_L_cache": 3, "conv_bias": False,
    "tie_word_embeddings": True, "norm_eps": 1e-5, "max_position_embeddings": 128,
    "bos_token_id": 1, "eos_token_id": 7, "pad_token_id": 0,
}
TINY_B = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
    "vocab_size": 384, "hidden_size": 128, "num_hidden_layers": 6,
    "layer_types": ["conv", "conv", "full_attention", "conv", "full_attention", "conv"],
    "num_attention_heads": 4, "num_key_value_heads": 1, "head_dim": 32,
    "intermediate_size": 512, "block_auto_adjust_ff_dim": True, "block_multiple_of": 32,
    "block_ffn_dim_multiplier": 1.0,
    "rope_theta": 1000000.0, "conv_L_cache": 4, "conv_bias": True,
    "tie_word_embeddings": False, "norm_eps": 1e-6, "max_position_embeddings": 256,
    "bos_token_id": 0, "eos_token_id": [2, 3], "pad_token_id": 1,
}
# A third one with sizes that are no power of two (width 96, 6 query heads in 3 groups,
# head size 48, vocabulary 331, five taps; 2 key-value heads, so that kv width = hidden).
TINY_C = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
    "vocab_size": 331, "hidden_size": 96, "num_hidden_layers": 3,
    "layer_types": ["full_attention", "conv", "full_attention"],
    "num_attention_heads": 6, "num_key_value_heads": 2, "head_dim": 48,
    "intermediate_size": 200, "block_auto_adjust_ff_dim": False,
    "rope_theta": 50000.0, "conv_L_cache": 5, "conv_bias": False,
    "tie_word_embeddings": True, "norm_eps": 3e-5, "max_position_embeddings": 512,
    "bos_token_id": 0, "eos_token_id": 5, "pad_token_id": 1,
}
# A fourth one with the head size of the matrix-core and split-key attention kernels (64),
# two taps and two attention layers in a row.
TINY_D = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
    "vocab_size": 500, "hidden_size": 160, "num_hidden_layers": 5,
    "layer_types": ["conv", "full_attention", "full_attention", "conv", "full_attention"],
    "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 64,
    "intermediate_size": 320, "block_auto_adjust_ff_dim": False,
    "rope_theta": 100000.0, "conv_L_cache": 2, "conv_bias": True,
    "tie_word_embeddings": False, "norm_eps": 2e-5, "max_position_embeddings": 512,
    "bos_token_id": 0, "eos_token_id": 4, "pad_token_id": 1,
}
# A fifth one whose inner sizes are all multiples of 64 (what the tiled products for steps of
# many rows take): width 128, 2 query heads of 64, feed-forward 192.
TINY_E = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
    "vocab_size": 300, "hidden_size": 128, "num_hidden_layers": 4,
    "layer_types": ["conv", "full_attention", "conv", "full_attention"],
    "num_attention_heads": 2, "num_key_value_heads": 1, "head_dim": 64,
    "intermediate_size": 192, "block_auto_adjust_ff_dim": False,
    "rope_theta": 20000.0, "conv_L_cache": 3, "conv_bias": True,
    "tie_word_embeddings": True, "norm_eps": 1e-5, "max_position_embeddings": 512,
    "bos_token_id": 0, "eos_token_id": 6, "pad_token_id": 1,
}
TINY = {"A": (TINY_A, 0), "B": (TINY_B, 1), "C": (TINY_C, 2), "D": (TINY_D, 3), "E": (TINY_E, 4)}


@pytest.fixture(scope="session")
def model_folders(tmp_path_factory):
    """name, storage dtype -> folder with config.json and model.safetensors (random
    weights, written by the framework's random-weights mode into a temporary folder)."""
    from celeg_amd.weights import write_random_model
    made = {}

    def get(name, dtype=torch.float32, std=0.02):
        key = (name, dtype, std)
        if key not in made:
            cfg, seed = TINY[name]
            out = tmp_path_factory.mktemp(f"tiny{name}_{str(dtype).split('.')[-1]}")
            made[key] = write_random_model(cfg, str(out), seed=seed, dtype=dtype, std=std)
        return made[key]
    return get
