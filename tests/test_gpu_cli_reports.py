"""The command line's reports: --runtime-metrics (time to first token, time between tokens),
--memory-report, --profile (ms per step by phase) and --dump-hidden, in the reference's
``key=value`` lines on stderr."""
import os
import re
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_lfm2 as plain
from helpers import ROOT, WEIGHT_STD, random_tokens

pytestmark = pytest.mark.gpu


def test_reports_of_the_command_line(model_folders, tmp_path):
    folder = model_folders("D", torch.bfloat16, WEIGHT_STD)
    cfg, W = plain.load_model_folder(folder)
    prompt = random_tokens(cfg["vocab_size"], 20, seed=8)
    dump = str(tmp_path / "hidden")
    proc = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bin", "celeg-run"), "--model", folder, "--dtype", "bfloat16",
         "--prompt", ",".join(map(str, prompt)), "--max-new-tokens", "6", "--repetition-penalty", "1.0",
         "--runtime-tokens", "--runtime-metrics", "--memory-report", "--profile", "--dump-hidden", dump],
        capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr
    values = dict(re.findall(r"^([a-z_.]+)=([^\s]+)", proc.stderr, flags=re.M))
    assert int(values["runtime.prefill_tokens"]) == 20 and int(values["runtime.decode_tokens"]) == 5
    assert float(values["runtime.ttft_seconds"]) > 0 and float(values["runtime.itl_mean_seconds"]) > 0
    assert float(values["runtime.itl_max_seconds"]) >= float(values["runtime.itl_mean_seconds"])
    assert int(values["runtime.graph_replays"]) == 0          # steps that are timed or dumped are not replayed
    for key in ("memory.weights", "memory.kv_cache", "memory.conv_state", "memory.activations"):
        assert int(values[key]) > 0
    assert int(values["profile.steps"]) == 6
    for phase in ("embedding", "mixer_short_conv", "mixer_gqa_attention", "ffn_swiglu", "head"):
        assert float(values[f"profile.{phase}_ms_per_step"]) > 0
    # the first step's last layer: the stream of the prompt's 20 rows, against the plain model
    hidden = []
    plain.model_logits(cfg, W, prompt, hidden=hidden)
    last = len(hidden) - 1
    rows = np.fromfile(os.path.join(dump, f"step0_layer{last}.f32"), dtype="<f4").reshape(20, cfg["hidden_size"])
    ref = hidden[last].float().numpy()
    assert float(np.abs(rows - ref).max()) <= 4e-2 * float(np.abs(ref).max())
    assert len(os.listdir(dump)) == 6 * len(hidden)
