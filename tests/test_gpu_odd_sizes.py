"""The engine against the plain implementation at sizes that the configuration allows but no
model of this family ships with: head sizes of 80, 96, 128 and 256, eight query heads on one
key/value head, as many key/value heads as query heads, one tap and nine taps, a width that
is no multiple of 8, and one whose inner sizes are all multiples of 64 through both kinds of
products for many rows.  Most of each prompt in one step and the last 32 tokens one by one,
and portions of changing size; 32-bit and bfloat16."""
import pytest
import torch

import plain_lfm2 as plain
from helpers import (WEIGHT_STD, EngineDriver, assert_close, peak_tokens, portions_schedule,
                     random_tokens, tail_decode_schedule)

pytestmark = pytest.mark.gpu

BASE = {"architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2", "block_auto_adjust_ff_dim": False,
        "rope_theta": 10000.0, "conv_bias": False, "tie_word_embeddings": True, "norm_eps": 1e-5,
        "max_position_embeddings": 512, "bos_token_id": 0, "eos_token_id": 5, "pad_token_id": 1}


def config(**sizes):
    return dict(BASE, **sizes)


CASES = {
    "head 96": config(vocab_size=200, hidden_size=192, num_hidden_layers=2,
                      layer_types=["full_attention", "conv"], num_attention_heads=2,
                      num_key_value_heads=1, head_dim=96, intermediate_size=128, conv_L_cache=3),
    "head 128, no groups": config(vocab_size=130, hidden_size=256, num_hidden_layers=2,
                                  layer_types=["conv", "full_attention"], num_attention_heads=2,
                                  num_key_value_heads=2, head_dim=128, intermediate_size=96, conv_L_cache=4),
    "head 80": config(vocab_size=97, hidden_size=160, num_hidden_layers=2,
                      layer_types=["full_attention", "full_attention"], num_attention_heads=2,
                      num_key_value_heads=2, head_dim=80, intermediate_size=72, conv_L_cache=3),
    "head 256": config(vocab_size=90, hidden_size=256, num_hidden_layers=1, layer_types=["full_attention"],
                       num_attention_heads=1, num_key_value_heads=1, head_dim=256, intermediate_size=64,
                       conv_L_cache=3),
    "group of 8": config(vocab_size=150, hidden_size=128, num_hidden_layers=3,
                         layer_types=["full_attention", "conv", "full_attention"], num_attention_heads=8,
                         num_key_value_heads=1, head_dim=16, intermediate_size=100, conv_L_cache=2),
    "nine taps": config(vocab_size=64, hidden_size=64, num_hidden_layers=2, layer_types=["conv", "conv"],
                        num_attention_heads=4, num_key_value_heads=2, head_dim=16, intermediate_size=64,
                        conv_L_cache=9, conv_bias=True),
    "one tap": config(vocab_size=64, hidden_size=104, num_hidden_layers=2, layer_types=["conv", "full_attention"],
                      num_attention_heads=3, num_key_value_heads=3, head_dim=32, intermediate_size=40,
                      conv_L_cache=1),
    "width 100": config(vocab_size=77, hidden_size=100, num_hidden_layers=2, layer_types=["conv", "full_attention"],
                        num_attention_heads=5, num_key_value_heads=5, head_dim=16, intermediate_size=52,
                        conv_L_cache=3),
    "multiples of 64": config(vocab_size=512, hidden_size=256, num_hidden_layers=3,
                              layer_types=["conv", "full_attention", "conv"], num_attention_heads=4,
                              num_key_value_heads=1, head_dim=64, intermediate_size=320, conv_L_cache=3,
                              tie_word_embeddings=False),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(CASES))
def test_engine_matches_plain_at_unusual_sizes(tmp_path, name, dtype):
    from celeg_amd.engine import load_model
    from celeg_amd.weights import write_random_model
    cfg = CASES[name]
    storage = torch.float32 if dtype == "float32" else torch.bfloat16
    folder = str(tmp_path / "model")
    write_random_model(cfg, folder, seed=11, dtype=storage, std=WEIGHT_STD)
    reqs = {f"r{i}": random_tokens(cfg["vocab_size"], n, seed=50 + i) for i, n in enumerate([150, 70, 33])}
    plain_cfg, weights = plain.load_model_folder(folder)
    ref = {rid: plain.model_logits(plain_cfg, weights, toks) for rid, toks in reqs.items()}
    backends = ("library", "tiles") if dtype == "bfloat16" and name == "multiples of 64" else ("library",)
    for backend in backends:
        for mode, schedule in (("tail32", tail_decode_schedule), ("portions", portions_schedule)):
            steps = schedule(reqs)
            tokens = peak_tokens(steps)
            lm = load_model(folder, dtype=dtype, page_tokens=16, n_pages=tokens // 16, max_requests=4,
                            max_batched_tokens=max(tokens, 64), gemm_backend=backend)
            got = EngineDriver(lm).run(steps)
            for rid in reqs:
                assert_close(got[rid], ref[rid], dtype, f"{name}/{dtype}/{backend}/{mode}/{rid}")
            lm.cache.check()
