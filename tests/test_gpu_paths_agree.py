"""GPU invariant at cfg2's full size that involves no oracle: the tokens of an open chunk after a 32768-token
prompt get the same attention output whichever way they are computed,

  A. as the last rows of one prefill over prompt + tail (role-masked prefill kernel alone),
  B. one at a time over the evicted cache (eviction kernel, cache append, decode kernel),
  C. as one multi-token segment over the evicted cache (eviction kernel, segment form of the prefill kernel).

The visibility rules make the three equal (a local chunk is visible until its next global chunk and is dropped
from the cache once that chunk is processed; a sliding-window chunk is visible for W / C chunk completions and
lives in the ring that long; the open chunk is causal), so a wrong survivor, a stale row read by the decode
kernel or a mask error of the prefill kernel shows as a difference."""
import math

import numpy as np
import pytest
import torch

from tests.gpu_util import say

pytestmark = pytest.mark.gpu

TOL = 2e-2


@pytest.mark.parametrize("Hq,Hkv,L,C,W,tail", [(32, 8, 32768, 64, 256, 37), (8, 8, 8192, 8, 32, 5), (12, 4, 4096, 1, 16, 9)])
def test_prefill_decode_and_segment_agree(Hq, Hkv, L, C, W, tail):
    from neuralattentionsearch_amd import ops
    from neuralattentionsearch_amd.cache import NAtSChunkLayerCache
    say("paths agree", Hq, Hkv, L, C, W, tail)
    B, D = 1, 128
    assert L % C == 0
    S = L // C
    rng = np.random.default_rng(L + C)
    roles = rng.choice(3, size=(B, Hkv, S), p=(0.05, 0.15, 0.80)).astype(np.uint8)
    roles[:, :, 0] = 0
    g = torch.Generator(device="cuda").manual_seed(L + C)
    N = L + tail
    # scores with a standard deviation of 4 nats: every row's output is carried by a few keys and is of the size of
    # v, so that a missing or an extra key shows against the tolerance
    q = (torch.randn(B, Hq, N, D, generator=g, device="cuda") * 4.0).bfloat16()
    k = torch.randn(B, Hkv, N, D, generator=g, device="cuda", dtype=torch.bfloat16)
    v = torch.randn(B, Hkv, N, D, generator=g, device="cuda", dtype=torch.bfloat16)
    scale = 1.0 / math.sqrt(D)
    roles_dev = torch.from_numpy(roles).cuda()

    # A: one prefill over everything; the tail's chunks get their own slots (the roles the tail would be given one
    # token or one segment at a time: global while a chunk is open or just complete)
    n_tail_slots = math.ceil(tail / C)
    roles_all = torch.cat([roles_dev, torch.zeros(B, Hkv, n_tail_slots, dtype=torch.uint8, device="cuda")], dim=-1)
    out_a = ops.prefill_attention(q, k, v, roles_all, C, W, scale)[:, :, L:].float()

    def evicted_cache():
        cache = NAtSChunkLayerCache(B, Hkv, W, chunk_size=C, device="cuda")
        cache.update(k[:, :, :L], v[:, :, :L], None, roles=roles_dev)
        cache.post_update(L)
        return cache

    one_global = torch.zeros(B, Hkv, 1, dtype=torch.uint8, device="cuda")

    # B: token by token
    cache = evicted_cache()
    out_b = []
    for i in range(tail):
        t = L + i
        closes = (cache.chunk_fill_size + 1) >= C
        keys, values = cache.update(k[:, :, t:t + 1], v[:, :, t:t + 1], None, roles=one_global if closes else None)
        row_end, tail_start = cache.decode_hint()
        out_b.append(ops.decode_attention(q[:, :, t:t + 1], keys, values, cache.valid_tokens, keys.shape[2], scale,
                                          row_end=row_end, tail_start=tail_start))
        cache.post_update(1)
    out_b = torch.cat(out_b, dim=2).float()

    # C: the tail as one segment
    cache = evicted_cache()
    cache.update(k[:, :, L:], v[:, :, L:], None, roles=torch.zeros(B, Hkv, n_tail_slots, dtype=torch.uint8, device="cuda"))
    out_c = cache.segment_attention(q[:, :, L:], scale).float()

    assert torch.isfinite(out_a).all() and torch.isfinite(out_b).all() and torch.isfinite(out_c).all()
    rms = out_a.pow(2).mean(-1, keepdim=True).sqrt()
    assert rms.min().item() > 0.05, rms.min().item()
    bound = TOL * torch.maximum(rms, out_a.abs()) + 2e-3  # (both sides are rounded to bf16: an element may differ by its ulp)
    err_ab, err_ac = (out_a - out_b).abs(), (out_a - out_c).abs()
    assert not (err_ab > bound).any(), f"prefill rows vs token-by-token decode: {err_ab.max().item()}"
    assert not (err_ac > bound).any(), f"prefill rows vs one segment over the cache: {err_ac.max().item()}"
