"""The engine against the plain implementation at the real layer sizes: slices of three or four
layers with the widths, head counts, feed-forward sizes and the vocabulary of 65,536 of the
LFM2-350M, LFM2-1.2B and LFM2-2.6B shapes (the last with its own feed-forward of 7,168 columns
and an attention layer followed by three convolution layers, as that model orders them), so that
every product runs through the kernel (and the tiles of it) that the real model takes: the
output head through the wide-product kernels, the feed-forward at 4,608, 8,192 and 7,168 columns.
Requests are short (up to 128 tokens) so that the float64 plain implementation stays fast."""
import pytest
import torch

import plain_lfm2 as plain
from helpers import (WEIGHT_STD, EngineDriver, assert_close, mixed_schedule, peak_tokens,
                     portions_schedule, random_tokens, tail_decode_schedule, whole_schedule)

pytestmark = pytest.mark.gpu

BASE = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2", "vocab_size": 65536,
    "num_hidden_layers": 3, "layer_types": ["conv", "full_attention", "conv"],
    "num_key_value_heads": 8, "head_dim": 64, "block_auto_adjust_ff_dim": True,
    "block_multiple_of": 256, "block_ffn_dim_multiplier": 1.0, "rope_theta": 1000000.0,
    "conv_L_cache": 3, "conv_bias": False, "tie_word_embeddings": True, "norm_eps": 1e-5,
    "max_position_embeddings": 4096, "bos_token_id": 1, "eos_token_id": 7, "pad_token_id": 0,
}
# (hidden, query heads, intermediate_size -> feed-forward width)
WIDTHS = {
    "350m": dict(BASE, hidden_size=1024, num_attention_heads=16, intermediate_size=6656),    # ff 4608
    "1.2b": dict(BASE, hidden_size=2048, num_attention_heads=32, intermediate_size=12288),   # ff 8192
    "2.6b": dict(BASE, hidden_size=2048, num_attention_heads=32, intermediate_size=10752,    # ff 7168
                 num_hidden_layers=4, layer_types=["full_attention", "conv", "conv", "conv"]),
}
FF = {"350m": 4608, "1.2b": 8192, "2.6b": 7168}
LENGTHS = [128, 70, 100, 45, 33]
SCHEDULES = {"whole": whole_schedule, "tail32": tail_decode_schedule,
             "portions": portions_schedule, "mixed": mixed_schedule}
_folders = {}
_plain = {}


def requests():
    return {f"r{i}": random_tokens(65536, n, seed=900 + i) for i, n in enumerate(LENGTHS)}


def folder_of(tmp_path_factory, shape, storage):
    from celeg_amd.weights import write_random_model
    key = (shape, storage)
    if key not in _folders:
        out = tmp_path_factory.mktemp(f"real_{shape.replace('.', '_')}_{str(storage).split('.')[-1]}")
        _folders[key] = write_random_model(WIDTHS[shape], str(out), seed=11, dtype=storage, std=WEIGHT_STD)
    return _folders[key]


def plain_logits(folder, key):
    if key not in _plain:
        cfg, W = plain.load_model_folder(folder)
        assert plain.ff_dim(cfg["intermediate_size"], True, 256) == W["model.layers.0.feed_forward.w1.weight"].shape[0] == FF[key[0]]
        _plain[key] = {rid: plain.model_logits(cfg, W, toks).float() for rid, toks in requests().items()}
    return _plain[key]


@pytest.mark.parametrize("mode", list(SCHEDULES))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", ["350m", "1.2b", "2.6b"])
def test_engine_matches_plain_at_real_layer_sizes(tmp_path_factory, shape, dtype, mode):
    from celeg_amd.engine import load_model
    storage = torch.float32 if dtype == "float32" else torch.bfloat16
    folder = folder_of(tmp_path_factory, shape, storage)
    reqs = requests()
    steps = SCHEDULES[mode](reqs)
    max_tokens = peak_tokens(steps)
    lm = load_model(folder, dtype=dtype, page_tokens=16, n_pages=max_tokens // 16, max_requests=4,
                    max_context=256, max_batched_tokens=max(max_tokens, 64))
    got = EngineDriver(lm).run(steps)
    ref = plain_logits(folder, (shape, storage))
    for rid in reqs:
        assert_close(got[rid], ref[rid], dtype, f"{shape}/{dtype}/{mode}/{rid}")
    assert lm.cache.n_free_slots == 4 and lm.cache.free_pages() == [max_tokens // 16]
