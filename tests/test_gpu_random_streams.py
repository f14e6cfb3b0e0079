"""GPU: seeded random configurations and segment streams through the attention module and the Llama-architecture
harness, checked against the oracle by the runners of test_gpu_attention_module.py and test_gpu_llama.py.

The parametrised tests elsewhere pick their shapes by hand; these draw head counts, group sizes (also 3), chunk
sizes (also 1), windows, merge methods and the cut of the stream into segments (first segments of one token,
segments shorter than a chunk, exact multiples, long ones, runs of single tokens) at random."""
import numpy as np
import pytest
import torch

from tests.gpu_util import say
from tests.test_gpu_attention_module import run_module
from tests.test_gpu_llama import run as run_harness

pytestmark = pytest.mark.gpu


def draw_stream(rng, C, n_parts):
    lens = []
    for _ in range(n_parts):
        kind = rng.integers(0, 4)
        if kind == 0:
            lens += [1] * int(rng.integers(1, 2 * C + 3))
        elif kind == 1:
            lens.append(int(rng.integers(1, max(2, C))))
        elif kind == 2:
            lens.append(C * int(rng.integers(1, 4)))
        else:
            lens.append(int(rng.integers(C, 5 * C + 30)))
    return lens


@pytest.mark.parametrize("seed", range(8))
def test_random_streams_through_the_attention_module(seed):
    rng = np.random.default_rng(1000 + seed)
    C = int(rng.choice([1, 2, 4, 8, 16, 32, 64]))
    W = C * int(rng.integers(1, 6))
    if C == 1:
        W = 16 * W  # the per-token class wants a window of at least its update chunk size
    lens = draw_stream(rng, 16 if C == 1 else C, int(rng.integers(2, 7)))
    say("random module stream", seed, C, W, lens)
    run_module(lens, C, W)


@pytest.mark.parametrize("seed", range(8))
def test_random_configurations_of_the_harness(seed):
    from neuralattentionsearch_amd.llama import NAtSLlamaConfig
    rng = np.random.default_rng(2000 + seed)
    Hkv = int(rng.choice([1, 2, 4]))
    Hq = Hkv * int(rng.choice([1, 2, 3, 4, 8]))
    D = int(rng.choice([64, 128]))
    C = int(rng.choice([1, 4, 8, 16, 64]))
    W = C * int(rng.integers(1, 5))
    if C == 1:
        W = 16 * W
    cfg = NAtSLlamaConfig(vocab_size=500, hidden_size=Hq * D, intermediate_size=256, num_hidden_layers=2,
                          num_attention_heads=Hq, num_key_value_heads=Hkv, chunk_size=C, local_seq_max_length=W,
                          chunk_merge_method=str(rng.choice(["mean", "max"])), fused_decode=bool(rng.integers(0, 2)))
    lens = draw_stream(rng, 16 if C == 1 else C, int(rng.integers(3, 6)))
    say("random harness configuration", seed, cfg, lens)
    # (weights scaled so that q, k, v keep the scale of the 512-wide model the fixed cases use)
    run_harness(cfg, torch.float32, lens, tol=5e-5, B=int(rng.integers(1, 3)), seed=seed, std=0.05 * (512.0 / (Hq * D)) ** 0.5,
                need_all_roles=False)
