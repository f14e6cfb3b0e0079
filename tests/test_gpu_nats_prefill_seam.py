"""GPU: the kernel-level seam `nats_prefill` in its form over an existing cache (global_kv_size=...), driven with the
call pattern of the reference's own smoke (models/transformer/triton/nats_flashattn_fwd.py:851-979): prefill a layer
cache, evict, append a second segment, hand the cache's size tensors, ring bits, n_ctx_data and tail to the kernel
call, and compare its mask in the three column ranges (ring, cached rows, new rows) and its output with
cache.generate_mask + dense masked attention -- here against the oracle's state machine."""
import math

import numpy as np
import pytest
import torch

from oracle import nats_oracle as orc
from tests.gpu_util import say

pytestmark = pytest.mark.gpu


def end_seq_idx_as_the_reference_computes_it(tsi):
    """nats_flashattn_fwd.py:943-945: last slot forced global in a copy, then flip / cummax / flip."""
    flags = tsi[..., 0].clone().contiguous()
    flags[..., -1] = 1.0
    S = flags.shape[-1]
    return S - 1 - torch.flip(torch.cummax(torch.flip(flags, (-1,)), -1)[1], (-1,))


def run_smoke_pattern(B, H, n_rep, D, W, C, lens, dtype, seed, cache_scalars=False):
    from neuralattentionsearch_amd import ops
    from neuralattentionsearch_amd.cache import NAtSChunkLayerCache, NAtSLayerCache
    tol = 2e-2 if dtype == torch.bfloat16 else 1e-5
    rng = np.random.default_rng(seed)
    g = torch.Generator().manual_seed(seed)
    if C == 1:
        cache, st = NAtSLayerCache(B, H, W, device="cuda"), orc.TokenCacheOracle(B=B, H=H, W=W)
    else:
        cache, st = NAtSChunkLayerCache(B, H, W, chunk_size=C, device="cuda"), orc.ChunkCacheOracle(B=B, H=H, W=W, C=C)
    fill = 0
    for si, n in enumerate(lens):
        say("nats_prefill seam", (B, H, n_rep, D, W, C), "segment", si, n, dtype)
        S = n if C == 1 else math.ceil((fill + n) / C)
        roles = rng.choice(3, size=(B, H, S), p=(0.2, 0.3, 0.5)).astype(np.uint8)
        if si == 0:
            roles[:, :, 0] = 0
        if C > 1 and (fill + n) % C:
            roles[:, :, -1] = 0  # the open chunk (index[:, :, -1] = 0 in the smoke)
        tsi = orc.one_hot_roles(roles, dtype=dtype).cuda()
        q = torch.randn(B, H * n_rep, n, D, generator=g).to(dtype)
        k = torch.randn(B, H, n, D, generator=g).to(dtype)
        v = torch.randn(B, H, n, D, generator=g).to(dtype)
        ko, vo = st.update(k, v, roles)
        k2, v2 = cache.update(k.cuda(), v.cuda(), tsi)
        end_idx = end_seq_idx_as_the_reference_computes_it(tsi)
        common = dict(sliding_tokens=tsi[..., 2].contiguous(), nats_chunk_size=C, end_seqs_idx=end_idx,
                      sm_scale=1 / math.sqrt(D), n_rep=n_rep, return_masks=True, local_seq_max_length=W)
        if si == 0:
            want_mask = orc.prefill_mask(roles, n, C, W)
            o, msk = ops.nats_prefill(q.cuda(), k2, v2, **common)
        else:
            want_mask = st.generate_mask(n)
            if cache_scalars:  # the two numbers the reference's argument list does not carry
                common.update(seen_tokens=cache._seen_tokens, n_global_min=cache._n_global_min)
            o, msk = ops.nats_prefill(
                q.cuda(), k2, v2, **common,
                n_tokens_in_first_chunk=cache.chunk_fill_size - n if C > 1 else 0,
                global_kv_size=cache.size_global_kv, local_kv_size=cache.size_local_kv,
                valid_sw_tokens=cache.valid_tokens[..., :W:C].contiguous(), n_ctx_data=cache.n_ctx_data,
                sw_token_tails=cache.sliding_queue_tail)
            msk_h = msk.cpu().numpy()
            n_ctx_chunk = cache.n_ctx_data // C * C
            for name, cols in (("sw", slice(0, W)), ("past", slice(W, n_ctx_chunk)), ("future", slice(n_ctx_chunk, None))):
                assert np.array_equal(msk_h[..., cols], want_mask[..., cols]), (si, "mask range", name)
        assert msk.dtype == torch.bool and tuple(msk.shape) == want_mask.shape
        assert np.array_equal(msk.cpu().numpy(), want_mask), (si, "mask")
        want = orc.masked_attention(q.float(), ko.float(), vo.float(), want_mask)
        err = (o.float().cpu() - want).abs().max().item()
        assert err <= tol, (si, "output", err)
        st.post_update(n)
        cache.post_update(n)
        fill = (fill + n) % C


def test_the_smoke_of_the_reference_per_token_cache():
    """The smoke's own numbers: batch 4, 8 heads, 507 tokens, head_dim 64, window 32, chunk size 1, then 54 tokens."""
    run_smoke_pattern(4, 8, 1, 64, 32, 1, [507, 54], torch.bfloat16, seed=101)


@pytest.mark.parametrize("C,W,lens", [(8, 32, [512, 56, 54, 10, 40]), (64, 256, [1024, 192, 130, 62, 64]),
                                      (32, 64, [320, 54, 42])])
def test_the_smoke_pattern_on_the_chunked_cache(C, W, lens):
    """Chunk sizes above one: a first segment of whole chunks that fills the window, then segments that end inside a
    chunk (n_tokens_in_first_chunk > 0 on the call after them)."""
    run_smoke_pattern(2, 2, 4, 128, W, C, lens, torch.bfloat16, seed=C)
    run_smoke_pattern(1, 2, 2, 64, W, C, lens, torch.float32, seed=C + 1)


def test_per_token_cache_with_more_segments():
    run_smoke_pattern(2, 4, 4, 128, 64, 1, [300, 54, 160, 32], torch.bfloat16, seed=7)


@pytest.mark.parametrize("C,W,lens", [(8, 32, [16, 8, 24, 40]), (4, 64, [20, 22, 30, 64])])
def test_a_first_segment_shorter_than_the_window(C, W, lens):
    """The ring has not wrapped when the later segments arrive: the limits of its slots follow the branch for
    _seen_tokens < W (nats_chunk_layer_cache.py:666-676), which the call can only take when it is told the number of
    tokens the cache has seen.  (Chunked cache only: a per-token cache that has seen fewer tokens than its window may
    hold blocks of sliding-window tokens left in place behind a head's own rows, nats_layer_cache.py:316-327, which
    the kernel's argument list cannot describe; `cache.segment_attention` covers that case.)"""
    run_smoke_pattern(2, 2, 2, 64, W, C, lens, torch.float32, seed=50 + C, cache_scalars=True)
    run_smoke_pattern(1, 2, 4, 128, W, C, lens, torch.bfloat16, seed=60 + C, cache_scalars=True)


def test_an_unfilled_window_is_not_taken_for_a_full_one():
    from neuralattentionsearch_amd import ops
    say("nats_prefill seam: ambiguous ring")
    W, C = 32, 8
    q = torch.zeros(1, 2, 8, 64, device="cuda")
    k = torch.zeros(1, 2, W + 16 + 8, 64, device="cuda")
    idx = torch.zeros(1, 2, 1, dtype=torch.int64, device="cuda")
    sizes = torch.full((1, 2), W + 8, dtype=torch.int64, device="cuda")
    ring = torch.zeros(1, 2, W // C, dtype=torch.bool, device="cuda")
    ring[..., 0] = True
    kw = dict(nats_chunk_size=C, n_rep=1, local_seq_max_length=W, global_kv_size=sizes, local_kv_size=sizes - W,
              valid_sw_tokens=ring, n_ctx_data=W + 16, sw_token_tails=16)
    with pytest.raises(ValueError, match="seen_tokens"):
        ops.nats_prefill(q, k, k, idx, idx.float(), 1.0, **kw)
    o, _ = ops.nats_prefill(q, k, k, idx, idx.float(), 1.0, seen_tokens=16, **kw)
    assert tuple(o.shape) == (1, 2, 8, 64)


def test_arguments_are_checked():
    from neuralattentionsearch_amd import ops
    say("nats_prefill seam: argument checks")
    q = torch.zeros(1, 2, 8, 64, device="cuda")
    k = torch.zeros(1, 2, 40, 64, device="cuda")
    idx = torch.zeros(1, 2, 1, dtype=torch.int64, device="cuda")
    sizes = torch.full((1, 2), 32, dtype=torch.int64, device="cuda")
    with pytest.raises(ValueError):  # the cache arguments come together
        ops.nats_prefill(q, k, k, idx, idx.float(), 1.0, nats_chunk_size=8, n_rep=1, local_seq_max_length=16,
                         global_kv_size=sizes)
    ring = torch.ones(1, 2, 2, dtype=torch.bool, device="cuda")
    with pytest.raises(ValueError):  # k must hold n_ctx_data + L_q rows
        ops.nats_prefill(q, k, k, idx, idx.float(), 1.0, nats_chunk_size=8, n_rep=1, local_seq_max_length=16,
                         global_kv_size=sizes, local_kv_size=sizes, valid_sw_tokens=ring, n_ctx_data=24, sw_token_tails=0)
