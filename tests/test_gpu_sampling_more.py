"""The sampling kernel against the plain sampler at wide and odd vocabularies: ties at the
threshold and everywhere, more equal maxima than any top_k, penalties, greedy rows among
sampled ones, every top_k, many draws, launches one after the other and from a recorded
graph."""
import pytest
import torch

import plain_lfm2 as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    from kernel_ops import HipOps
    return HipOps(DEV)


def sample_with_draw(logits, temperature, top_k, top_p, penalty, seen, u):
    generator = plain.random_unit
    plain.random_unit = lambda state: (state, u)
    try:
        return plain.sample(logits, temperature, top_k, top_p, penalty, seen, 1)[0]
    finally:
        plain.random_unit = generator


def launch(ops, logits_dev, rows, out=None):
    R, V = logits_dev.shape
    f = torch.tensor([[t, p, pen, u] for t, k, p, pen, u, s in rows], dtype=torch.float32)
    seen = torch.zeros(R, V, dtype=torch.uint8)
    i = []
    for r, (t, k, p, pen, u, s) in enumerate(rows):
        if s is not None:
            seen[r, torch.tensor(s, dtype=torch.long)] = 1
        i.append([k, r if s is not None else -1, -1])
    out = torch.empty(R, dtype=torch.int32, device=DEV) if out is None else out
    args = (logits_dev, f.reshape(-1).to(DEV), torch.tensor(i, dtype=torch.int32).reshape(-1).to(DEV), seen.to(DEV), out)
    ops.sample(*args)
    return out, args


def plain_tokens(logits, rows):
    want = []
    for r, (t, k, p, pen, u, s) in enumerate(rows):
        flags = [False] * logits.shape[1]
        for tok in (s or []):
            flags[tok] = True
        want.append(sample_with_draw(logits[r].tolist(), t, k, p, pen, flags, u))
    return want


@pytest.mark.parametrize("vocab", [8192, 12001, 65536, 131072])
def test_wide_vocabularies_equal_the_plain_sampler(ops, vocab):
    g = torch.Generator().manual_seed(vocab)
    R = 9
    logits = torch.randn(R, vocab, generator=g) * 3
    logits[1, 100:140] = logits[1, 7]                     # ties at one value
    logits[2] = torch.round(logits[2])                    # heavy ties everywhere
    logits[3, 5000:5600] = float(logits[3].max()) + 1.0   # more equal maxima in one part than any top_k
    logits[4, ::4096] = 9.0                               # equal large values far apart
    logits[5] = torch.round(logits[5] * 2) / 2
    logits[6, vocab - 3:] = 8.0                           # the best ones at the very end
    seen = [torch.randint(0, vocab, (60,), generator=g).tolist() for _ in range(R)]
    rows = [(0.8, 40, 0.9, 1.3, 0.37, seen[0]), (1.0, 128, 1.0, 1.0, 0.81, None),
            (0.5, 17, 0.5, 1.0, 0.999, None), (1.1, 50, 1.0, 1.7, 0.93, seen[3]),
            (2.0, 128, 0.95, 1.1, 0.05, seen[4]), (1.3, 2, 1.0, 1.0, 0.5, None),
            (0.0, 50, 1.0, 1.5, 0.0, seen[6]), (0.7, 1, 1.0, 1.0, 0.3, None), (0.1, 50, 1.0, 1.05, 0.6, seen[8])]
    want = plain_tokens(logits, rows)
    dev = logits.to(DEV)
    got, _ = launch(ops, dev, rows)
    assert got.tolist() == want
    assert launch(ops, dev, rows)[0].tolist() == want


def test_every_top_k_and_many_draws(ops):
    vocab = 20000
    g = torch.Generator().manual_seed(5)
    logits = torch.randn(16, vocab, generator=g) * 2
    logits[:, 4090:4100] += 6.0
    dev = logits.to(DEV)
    ks = [1, 2, 3, 7, 16, 31, 50, 64, 65, 100, 127, 128, 128, 5, 50, 90]
    for trial in range(6):
        us = torch.rand(16, generator=g).tolist()
        rows = [(0.6 + 0.2 * trial, ks[r], 1.0 if r % 2 else 0.8, 1.0, us[r], None) for r in range(16)]
        assert launch(ops, dev, rows)[0].tolist() == plain_tokens(logits, rows), f"trial {trial}"


def test_sampling_from_a_recorded_graph(ops):
    vocab = 65536
    g = torch.Generator().manual_seed(9)
    logits = torch.randn(4, vocab, generator=g) * 3
    rows = [(0.9, 50, 0.95, 1.0, 0.42, None), (0.0, 1, 1.0, 1.0, 0.0, None), (1.2, 128, 1.0, 1.0, 0.77, None), (0.4, 10, 0.5, 1.0, 0.1, None)]
    want = plain_tokens(logits, rows)
    dev = logits.to(DEV)
    out, args = launch(ops, dev, rows)
    assert out.tolist() == want
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        ops.sample(*args)
        with torch.cuda.graph(graph, stream=stream):
            ops.sample(*args)
    for _ in range(3):
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert out.tolist() == want
        assert launch(ops, dev, rows)[0].tolist() == want      # eager launches between the replays
