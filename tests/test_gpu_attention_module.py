"""GPU: the attention module + NAtSCache end to end (prefill, then decode steps with live eviction)
against the oracle driven with the module's own projections and role logits."""
import math

import numpy as np
import pytest
import torch

from oracle import nats_oracle as orc
from tests.gpu_util import say

pytestmark = pytest.mark.gpu


def rope_tables(B, start, n, D, device):
    inv = 1.0 / (10000.0 ** (torch.arange(0, D, 2, device=device).float() / D))
    t = torch.arange(start, start + n, device=device).float()
    f = torch.outer(t, inv)
    emb = torch.cat([f, f], dim=-1)
    return emb.cos()[None].expand(B, -1, -1), emb.sin()[None].expand(B, -1, -1)


@pytest.mark.parametrize("L,C,W,steps", [(100, 16, 32, 40), (64, 16, 32, 20), (5, 8, 16, 30), (1, 8, 16, 30),
                                         (100, 12, 36, 40), (50, 3, 12, 20)])  # (chunk sizes that are no power of two)
def test_module_prefill_and_decode(L, C, W, steps):
    run_module([L] + [1] * steps, C, W)


@pytest.mark.parametrize("lens,C,W", [([70, 45, 1, 1, 33, 16, 1, 90], 16, 32), ([3, 9, 40, 1, 1, 1, 25], 8, 16),
                                      ([70, 45, 1, 1, 33, 16, 1, 90], 6, 24)])
def test_module_segments_over_a_filled_cache(lens, C, W):
    """Multi-token segments after the first one run the segment kernel over the evicted cache."""
    run_module(lens, C, W)


@pytest.mark.parametrize("lens,W", [([40] + [1] * 30, 16), ([70, 45, 1, 1, 33, 1, 90], 32),
                                    ([1, 1, 1, 12, 1, 1, 30, 1], 16), ([5] + [1] * 14 + [40, 3, 1, 1, 20], 16)])
def test_module_with_per_token_roles(lens, W):
    """chunk_size == 1: a role per token, the per-token cache class with its eviction deferred by 16 tokens."""
    run_module(lens, 1, W)


def run_module(lens, C, W, executor=None, dim=512):
    from neuralattentionsearch_amd.attention import LlamaNAtSChunkAttentionLayer, apply_rotary_pos_emb
    from neuralattentionsearch_amd.cache import NAtSCache
    say("attention module", lens, C, W)
    torch.manual_seed(0)
    B, Hq, Hkv = 2, 8, 2
    D = dim // Hq
    mod = LlamaNAtSChunkAttentionLayer(dim=dim, n_heads=Hq, n_kv_heads=Hkv, layer_id=0, local_seq_max_length=W,
                                       chunk_size=C).cuda().eval()
    with torch.no_grad():
        mod.proj_layer.weight.mul_(8.0)  # spread the role logits
    mod.executor = executor
    logits_seen = []
    mod.proj_layer.register_forward_hook(lambda m, i, o: logits_seen.append(o.detach().float().cpu()))
    cache = NAtSCache(sliding_window_size=W, chunk_size=C)
    # (chunk_size == 1 builds the per-token class with its deferred eviction, as the reference's container does)
    st = orc.TokenCacheOracle(B=B, H=Hkv, W=W) if C == 1 else orc.ChunkCacheOracle(B=B, H=Hkv, W=W, C=C)

    def qkv(x, start):
        n = x.shape[1]
        q = mod.wq(x).view(B, n, Hq, D).transpose(1, 2)
        k = mod.wk(x).view(B, n, Hkv, D).transpose(1, 2)
        v = mod.wv(x).view(B, n, Hkv, D).transpose(1, 2)
        cos, sin = rope_tables(B, start, n, D, x.device)
        q, k = apply_rotary_pos_emb(q, k, cos, sin)
        return q, k, v, (cos, sin)

    fill, seen = 0, 0
    with torch.no_grad():
        for step, n in enumerate(lens):
            x = torch.randn(B, n, dim, device="cuda")
            q, k, v, pos = qkv(x, seen)
            logits_seen.clear()
            out = mod(x, pos, None, start_pos=seen, cache=cache)
            if mod._cache_is_till_updating is not None:  # an executor runs the eviction; the next call waits for it
                mod._cache_is_till_updating.result()
            # oracle side, fed with the module's own logits
            total = fill + n
            if total < C:
                roles = np.zeros((B, Hkv, 1), dtype=np.uint8)
                assert not logits_seen
                fill = total
            else:
                lg = logits_seen[0].unflatten(-1, (Hkv, 3))
                roles = orc.roles_from_logits(lg, 0.1, force_first_global=seen < C, force_last_global=total % C != 0)
                assert roles.shape[-1] == math.ceil(total / C)
                fill = total % C
            ko, vo = st.update(k.cpu(), v.cpu(), roles)
            if seen == 0:
                mask = orc.prefill_mask(roles, n, C, W)
                att = orc.masked_attention(q.cpu(), ko, vo, mask)
            elif n > 1:
                att = orc.masked_attention(q.cpu(), ko, vo, st.generate_mask(n))
            else:
                att = orc.decode_attention(q.cpu(), ko, vo, torch.from_numpy(st.valid), st.n_ctx_data + 1)
            st.post_update(n)
            want = mod.wo(att.cuda().transpose(1, 2).reshape(B, n, -1))
            err = (out - want).abs().max().item()
            assert err < 2e-4, (step, err)
            layer = cache.cache_model[0]
            assert layer.n_ctx_data == st.n_ctx_data, step
            assert np.array_equal(layer.valid_tokens.cpu().numpy(), st.valid), step
            assert np.array_equal(layer.size_global_kv.cpu().numpy(), st.size_global), step
            seen += n


def test_module_with_post_update_on_an_executor():
    """post_update submitted to a thread pool, as the reference's modules do when `executor` is set
    (nats_attention.py:189-192)."""
    from concurrent.futures import ThreadPoolExecutor
    with ThreadPoolExecutor(max_workers=1) as pool:
        run_module([50, 1, 1, 1, 20, 1, 1], 8, 16, executor=pool)


def test_container_surface_the_reference_callers_use():
    """NAtSCache through the calls and attributes the reference's callers rely on (components/cache/dyn_cache.py:66-195;
    attributes read by hf/llama.py:235-252 and experiments/efficiency/eval_efficiency.py:350-352)."""
    from neuralattentionsearch_amd.cache import NAtSCache
    say("container surface")
    B, H, D, C, W, L = 2, 2, 64, 8, 16, 40
    cache = NAtSCache(sliding_window_size=W, chunk_size=C)
    assert cache.get_seq_length(0) == 0 and cache.get_nats_chunk_fill_size(0) == 0
    assert cache.get_nats_cached_x_in_chunk(0) is None
    g = torch.Generator().manual_seed(5)
    k = torch.randn(B, H, L, D, generator=g).bfloat16().cuda()
    v = torch.randn(B, H, L, D, generator=g).bfloat16().cuda()
    roles = np.array([[[0, 2, 1, 0, 2], [0, 1, 1, 2, 2]]] * B, dtype=np.uint8)
    tsi = orc.one_hot_roles(roles, dtype=torch.bfloat16).cuda()
    keys, values = cache.update(k, v, 0, cache_kwargs={"token_states_info": tsi})
    assert keys.shape == k.shape and torch.equal(keys, k) and torch.equal(values, v)  # the first call hands back the raw K, V
    mask = cache.generate_mask(0, L)
    assert mask.dtype == torch.bool and tuple(mask.shape) == (B, H, L, L)
    cache.post_update(layer_idx=0, x_len=L)
    layer = cache.cache_model[0]
    assert cache.get_seq_length(0) == L and layer.get_seq_length() == L
    assert cache.get_nats_chunk_fill_size(0) == 0 == layer.chunk_fill_size
    assert layer._tokens_info is tsi
    # head 0: global chunks 0 and 3, nothing local after the last global; head 1: global chunk 0, local chunks 1 and 2
    assert layer.size_global_kv.tolist() == [[W + 2 * C, W + C]] * B
    assert layer.size_local_kv.tolist() == [[0, 2 * C]] * B
    assert layer.n_ctx_data == W + 3 * C and layer.sliding_queue_tail == (min(L // C, W // C) * C) % W
    assert layer.valid_tokens.dtype == torch.bool and layer.valid_tokens.shape[:2] == (B, H)
    assert layer.cache_k.shape == layer.cache_v.shape == (B, H, layer.valid_tokens.shape[2], D)
    # ring: the last W / C = 2 chunks, valid where sliding window (head 0: chunk 4; head 1: chunks 3 and 4)
    assert layer.valid_tokens[0, 0, :W].tolist() == [False] * C + [True] * C
    assert layer.valid_tokens[0, 1, :W].tolist() == [True] * W
    cache.reset_cache()
    assert cache.cache_model == [] and cache.get_seq_length(0) == 0


@pytest.mark.parametrize("method", ["mean", "max"])
def test_container_chunk_statistics_follow_the_oracle(method):
    """The running and per-chunk statistics of the hidden states (dyn_cache.py:98-171) that the role projection
    reads, over a stream cut into ragged segments, against the oracle's restatement."""
    from neuralattentionsearch_amd.cache import ChunkMergeType, NAtSCache, NAtSChunkLayerCache
    say("container statistics", method)
    B, dim, C, W = 2, 96, 8, 16
    mm = method == "max"
    kind = ChunkMergeType.MAX if mm else ChunkMergeType.MEAN
    cache = NAtSCache(sliding_window_size=W, chunk_size=C)
    cache.cache_model.append(NAtSChunkLayerCache(B, 1, W, 0, C, device="cuda"))
    layer = cache.cache_model[0]
    weight = torch.zeros(3, dim)
    g = torch.Generator().manual_seed(11)
    fill, carry = 0, None
    for n in (5, 2, 20, 1, 1, 9, 64, 3, 5, 1):
        x = torch.randn(B, n, dim, generator=g)
        pooled_o, _, carry_o, pad_o = orc.pooled_role_logits(x, weight, C, pre_fill=fill, carry_in=carry, merge_max=mm)
        layer.chunk_fill_size = fill
        if fill + n < C:
            cache.update_nats_cached_x_in_chunk(x.cuda(), 0, kind)
            assert pooled_o is None
        else:
            pooled, pad = cache.update_nats_cached_x_across_chunk(x.cuda(), fill, 0, kind)
            assert pad == pad_o and pooled.shape == pooled_o.shape
            torch.testing.assert_close(pooled.cpu(), pooled_o, rtol=1e-6, atol=1e-6)
        got = cache.get_nats_cached_x_in_chunk(0)
        assert (got is None) == (carry_o is None)
        if got is not None:
            if mm:  # (the reference keeps the raw rows of a first partial chunk; their maximum is the statistic)
                got = got.max(1, keepdim=True)[0]
            torch.testing.assert_close(got.cpu(), carry_o, rtol=1e-6, atol=1e-6)
        fill, carry = (fill + n) % C, carry_o


def test_module_on_a_side_stream():
    """Every kernel goes to torch's current stream: the same run under a stream of the caller's own."""
    say("attention module on a side stream")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run_module([40, 1, 1, 1, 20, 1, 1, 9], 8, 16)
    side.synchronize()


def test_module_with_an_executor_under_a_side_stream():
    """The eviction runs on the executor's thread, where torch's current stream would be the default one: the module
    hands the caller's stream over, so the eviction kernels follow the attention kernel that still reads the rows."""
    from concurrent.futures import ThreadPoolExecutor
    say("attention module: executor under a side stream")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with ThreadPoolExecutor(max_workers=1) as pool, torch.cuda.stream(side):
        run_module([300, 1, 1, 1, 120, 1, 1, 9, 200], 8, 16, executor=pool)
        run_module([200] + [1] * 20 + [90], 1, 16, executor=pool)
    side.synchronize()


@pytest.mark.parametrize("dim", [128, 256, 2048])
def test_module_with_other_head_dims(dim):
    """Head dims 16, 32 and 256 (the reference's kernel accepts them too): prefill, segments and one-token steps."""
    run_module([90, 1, 1, 40, 1, 1, 1, 17], 8, 16, dim=dim)


@pytest.mark.parametrize("lens,C,W", [([300, 1, 1, 150, 70, 1, 200], 16, 64), ([130, 65, 1, 1, 1, 40, 260], 64, 128),
                                      ([200] + [1] * 20 + [90, 33], 1, 16)])
def test_module_at_head_dim_256_over_a_filled_cache(lens, C, W):
    """Segments over the rows earlier segments left behind (ring, kept globals, locals up to the first global chunk)
    on the head-dim-256 matrix kernels of both sides."""
    run_module(lens, C, W, dim=2048)
