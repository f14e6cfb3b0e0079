"""GPU parity, bit exact: the HIP-backed NAtSChunkLayerCache against the oracle state machine
(which tests/test_oracle_golden.py pins to vectors written by the reference cache)."""
import math

import numpy as np
import pytest
import torch

from oracle.nats_oracle import ChunkCacheOracle, masked_attention, one_hot_roles
from tests.golden_io import Golden
from tests.gpu_util import say

pytestmark = pytest.mark.gpu

GOLD = Golden()


def compare(hip, st, where):
    assert hip.n_ctx_data == st.n_ctx_data, (where, "n_ctx_data", hip.n_ctx_data, st.n_ctx_data)
    scal = [hip._n_global_min, hip.sliding_queue_tail, hip.chunk_fill_size, hip.chunk_fill_size_last, hip._seen_tokens]
    assert scal == [st.gmin, st.tail, st.fill, st.fill_last, st.seen], (where, scal)
    assert np.array_equal(hip.size_global_kv.cpu().numpy(), st.size_global), (where, "size_global")
    assert np.array_equal(hip.size_local_kv.cpu().numpy(), st.size_local), (where, "size_local")
    assert tuple(hip.valid_tokens.shape) == st.valid.shape, (where, "rows", tuple(hip.valid_tokens.shape), st.valid.shape)
    assert np.array_equal(hip.valid_tokens.cpu().numpy(), st.valid), (where, "valid_tokens")
    # every byte of the cache, stale rows and zero tail included
    assert torch.equal(hip.cache_k.cpu().view(torch.int16 if hip.cache_k.element_size() == 2 else torch.int32),
                       st.cache_k.view(torch.int16 if st.cache_k.element_size() == 2 else torch.int32)), (where, "cache_k")
    assert torch.equal(hip.cache_v.cpu().view(torch.int16 if hip.cache_v.element_size() == 2 else torch.int32),
                       st.cache_v.view(torch.int16 if st.cache_v.element_size() == 2 else torch.int32)), (where, "cache_v")
    if hip.token_positions is not None:
        assert np.array_equal(hip.token_positions.cpu().numpy().astype(np.int64), st.pos_k), (where, "index map")


def drive(name, B, H, D, C, W, segs, dtype, seed, check_masks=True, attend_n_rep=0, layout=None):
    """segs: list of (x_len, roles uint8 [B, H, S]).  With attend_n_rep > 0 every multi-token segment over a
    non-empty cache also runs the segment attention kernel against masked attention on the oracle's cache.
    `layout(op index, k on the GPU, v on the GPU)` may return the same values in another memory layout."""
    from neuralattentionsearch_amd.cache import NAtSChunkLayerCache
    hip = NAtSChunkLayerCache(B, H, W, chunk_size=C, device="cuda", track_positions=True)
    st = ChunkCacheOracle(B=B, H=H, W=W, C=C)
    g = torch.Generator().manual_seed(seed)
    t_seen = 0
    for oi, (x_len, roles) in enumerate(segs):
        say("evict", name, "op", oi, "x_len", x_len, "S", roles.shape[-1])
        k = torch.randn(B, H, x_len, D, generator=g).to(dtype)
        v = torch.randn(B, H, x_len, D, generator=g).to(dtype)
        tsi = one_hot_roles(roles, dtype=dtype)
        ko, vo = st.update(k, v, roles)
        kd, vd = k.cuda(), v.cuda()
        if layout is not None:
            kd, vd = layout(oi, kd, vd)
        kh, vh = hip.update(kd, vd, tsi.cuda())
        assert torch.equal(kh.cpu().view(torch.int16 if dtype == torch.bfloat16 else torch.int32),
                           ko.contiguous().view(torch.int16 if dtype == torch.bfloat16 else torch.int32)), (name, oi, "update K")
        if check_masks:
            want_mask = st.generate_mask(x_len)
            got_mask = hip.generate_mask(x_len).cpu().numpy()
            assert got_mask.shape == want_mask.shape, (name, oi, "mask shape", got_mask.shape, want_mask.shape)
            assert np.array_equal(got_mask, want_mask), (name, oi, "mask", np.argwhere(got_mask != want_mask)[:8])
        if attend_n_rep and x_len > 1 and t_seen > 0:
            q = torch.randn(B, H * attend_n_rep, x_len, D, generator=g).to(dtype)
            want = masked_attention(q.float(), ko.float(), vo.float(), st.generate_mask(x_len))
            got = hip.segment_attention(q.cuda()).float().cpu()
            err = (got - want).abs().max().item()
            tol = 2e-2 if dtype == torch.bfloat16 else 1e-5
            assert err <= tol, (name, oi, "segment attention", err)
        st.post_update(x_len)
        hip.post_update(x_len)
        compare(hip, st, (name, oi, x_len))
        t_seen += x_len
    return hip, st


@pytest.mark.parametrize("name", GOLD.scenario_names())
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_replay_reference_scenarios(name, dtype):
    si, sc = GOLD.scenario(name)
    segs = [(op["x_len"], GOLD.op(si, oi)["roles"]) for oi, op in enumerate(sc["ops"])]
    drive(name, sc["B"], sc["H"], 8, sc["C"], sc["W"], segs, dtype, seed=si)


@pytest.mark.parametrize("name", [n for n in GOLD.scenario_names()
                                  if sum(op["x_len"] > 1 for op in GOLD.scenario(n)[1]["ops"]) > 1])
@pytest.mark.parametrize("dtype,D,n_rep", [(torch.float32, 64, 2), (torch.bfloat16, 128, 4)])
def test_segment_attention_on_reference_scenarios(name, dtype, D, n_rep):
    """Multi-token segments over a non-empty cache: mask (bit exact against the oracle, which the golden
    vectors pin) and attention output of the segment kernel."""
    si, sc = GOLD.scenario(name)
    segs = [(op["x_len"], GOLD.op(si, oi)["roles"]) for oi, op in enumerate(sc["ops"])]
    drive(name, sc["B"], sc["H"], D, sc["C"], sc["W"], segs, dtype, seed=si, attend_n_rep=n_rep)


def role_stream(rng, B, H, C, lens, p):
    """Roles as the attention module would hand them over for a list of segment lengths."""
    segs, fill, seen = [], 0, 0
    for x_len in lens:
        total = fill + x_len
        if total < C:
            roles = np.zeros((B, H, 1), dtype=np.uint8)
            fill = total
        else:
            S = math.ceil(total / C)
            roles = rng.choice(3, size=(B, H, S), p=p).astype(np.uint8)
            if seen == 0:
                roles[:, :, 0] = 0
            if total % C:
                roles[:, :, -1] = 0
            fill = total % C
        segs.append((x_len, roles))
        seen += x_len
    return segs


@pytest.mark.parametrize("C,W,D,dtype", [(64, 256, 128, torch.bfloat16), (64, 128, 64, torch.float32),
                                         (32, 256, 128, torch.bfloat16), (8, 16, 64, torch.bfloat16),
                                         (16, 64, 128, torch.float32)])
def test_prefill_then_decode_random(C, W, D, dtype):
    rng = np.random.default_rng(C + W)
    lens = [20 * C + 5] + [1] * (3 * C + 3)
    drive(f"prefill_decode_C{C}", 2, 4, D, C, W, role_stream(rng, 2, 4, C, lens, (0.1, 0.2, 0.7)), dtype, seed=C)


@pytest.mark.parametrize("C,W", [(64, 256), (16, 32)])
def test_multi_segment_and_streaming_random(C, W):
    rng = np.random.default_rng(C)
    lens = [10 * C, 4 * C, C, C, 3 * C + 7, 2 * C - 7, 1, 1, 5 * C] + [C] * 6
    drive(f"multiseg_C{C}", 2, 3, 128, C, W, role_stream(rng, 2, 3, C, lens, (0.15, 0.25, 0.6)), torch.bfloat16, seed=C,
          check_masks=True, attend_n_rep=4)


@pytest.mark.parametrize("C,W", [(64, 256), (8, 32)])
def test_appended_rows_in_changing_layouts(C, W):
    """The cache keeps calls prepared for the layout of the rows it was last handed and for its present buffers
    (ops.CacheAppendCall, ops.EvictInplaceCall).  A stream whose segments arrive as contiguous tensors, as views of
    a [B, L, H, D] projection output, inside wider rows at addresses that are and are not multiples of 16 bytes (same
    strides; the latter take the slice-assignment path) and with elements that are not contiguous, long enough for
    the capacity buffer to grow several times, leaves the oracle's bytes after every step."""
    rng = np.random.default_rng(77 + C)
    lens = [6 * C] + [C] * 5 + [2 * C + 3, C - 3] + [C] * 30 + [1] * (C + 2) + [C] * 4

    def layout(oi, k, v):
        B, H, L, D = k.shape
        kind = (oi // 2) % 4  # (two steps in a row per kind, so that a prepared call is met again)
        if kind == 1:  # [B, L, H, D] storage, as a projection leaves it
            return (k.transpose(1, 2).contiguous().transpose(1, 2), v.transpose(1, 2).contiguous().transpose(1, 2))
        if kind == 2:  # rows inside a wider buffer, every other time 8 bytes off a 16-byte address
            off = 4 if oi % 2 else 0
            z = lambda n, t: torch.zeros(B, H, L, n, dtype=t.dtype, device=t.device)
            wide = lambda t: torch.cat([z(off, t), t, z(16 - off, t)], dim=-1)[..., off:off + D]
            return wide(k), wide(v)
        if kind == 3 and oi % 16 == 6:  # elements two apart
            every_other = lambda t: torch.stack([t, t], dim=-1).reshape(B, H, L, 2 * D)[..., ::2]
            return every_other(k), every_other(v)
        return k, v

    drive(f"layouts_C{C}", 2, 3, 128, C, W, role_stream(rng, 2, 3, C, lens, (0.15, 0.25, 0.6)), torch.bfloat16, seed=5 + C,
          check_masks=False, layout=layout)


@pytest.mark.parametrize("C,W,D,dtype,n_rep", [(64, 256, 128, torch.bfloat16, 4), (8, 32, 64, torch.bfloat16, 2),
                                               (16, 64, 64, torch.float32, 1), (128, 256, 128, torch.bfloat16, 4)])
def test_segments_before_the_window_is_full_and_ragged_segments(C, W, D, dtype, n_rep):
    """Short first segments (cache seen < W, open chunks carried between segments), then long ones."""
    rng = np.random.default_rng(7 * C + W)
    lens = [C // 2 + 1, C // 2, C + 3, 2 * C - 5, 5, W + 2 * C + 1, 3, C - 1, 6 * C + 9, 1, 1, 2 * C]
    drive(f"ragged_C{C}", 2, 2, D, C, W, role_stream(rng, 2, 2, C, lens, (0.2, 0.3, 0.5)), dtype, seed=C + 1,
          attend_n_rep=n_rep)


def test_surviving_index_map_semantics():
    """Kept rows = globals in stream order, then locals newer than the last global; ring = sliding-window
    chunks among the last W tokens (definition of the compacted layout, independent of the oracle)."""
    C, W, B, H, D = 64, 256, 1, 2, 128
    rng = np.random.default_rng(3)
    S = 40
    roles = rng.choice(3, size=(B, H, S), p=(0.1, 0.3, 0.6)).astype(np.uint8)
    roles[:, :, 0] = 0
    hip, st = drive("index_map", B, H, D, C, W, [(S * C, roles)], torch.bfloat16, seed=1)
    pos = hip.token_positions.cpu().numpy()
    valid = hip.valid_tokens.cpu().numpy()
    for h in range(H):
        r = roles[0, h]
        glob = [s for s in range(S) if r[s] == 0]
        last_g = glob[-1]
        keep = glob + [s for s in range(S) if r[s] == 1 and s > last_g]
        want = np.concatenate([np.arange(s * C, (s + 1) * C) for s in sorted(keep)])
        got = pos[0, h, W:][valid[0, h, W:]]
        assert np.array_equal(got, want)
        ring_want = np.concatenate([np.arange(s * C, (s + 1) * C) if r[s] == 2 else np.full(C, -1)
                                    for s in range(S - W // C, S)])
        assert np.array_equal(pos[0, h, :W], ring_want)


def test_cfg4_bulk_eviction_properties():
    """B=16 x 8 kv heads x 65536 tokens x 128, bf16, window 512: too large for the oracle's loops, checked
    through size-independent properties of the compacted layout."""
    from neuralattentionsearch_amd.cache import NAtSChunkLayerCache
    say("evict cfg4 bulk")
    B, H, L, D, C, W = 16, 8, 65536, 128, 64, 512
    S = L // C
    rng = np.random.default_rng(0)
    roles = rng.choice(3, size=(B, H, S), p=(0.10, 0.15, 0.75)).astype(np.uint8)
    roles[:, :, 0] = 0
    g = torch.Generator(device="cuda").manual_seed(0)
    k = torch.randn(B, H, L, D, generator=g, device="cuda", dtype=torch.bfloat16)
    v = torch.randn(B, H, L, D, generator=g, device="cuda", dtype=torch.bfloat16)
    hip = NAtSChunkLayerCache(B, H, W, chunk_size=C, device="cuda", track_positions=True)
    tsi = one_hot_roles(roles, dtype=torch.bfloat16).cuda()
    hip.update(k, v, tsi)
    hip.post_update(L)
    is_g = roles == 0
    n_glob = is_g.sum(-1)
    last_g = S - 1 - np.argmax(is_g[:, :, ::-1], axis=-1)
    later_loc = np.array([[(roles[b, h, last_g[b, h] + 1:] == 1).sum() for h in range(H)] for b in range(B)])
    sg = hip.size_global_kv.cpu().numpy()
    sl = hip.size_local_kv.cpu().numpy()
    assert np.array_equal(sg, W + n_glob * C)
    assert np.array_equal(sl, later_loc * C)
    assert hip.n_ctx_data == int((sg + sl).max())
    assert hip.cache_k.shape[2] == math.ceil(hip.n_ctx_data / C) * C
    pos = hip.token_positions
    valid = hip.valid_tokens
    # every valid row holds exactly the K / V row of the token the index map names
    for b in (0, 7, 15):
        for h in (0, 3, 7):
            idx = torch.nonzero(valid[b, h]).flatten()
            p = pos[b, h, idx].long()
            assert (p >= 0).all()
            assert torch.equal(hip.cache_k[b, h, idx], k[b, h, p])
            assert torch.equal(hip.cache_v[b, h, idx], v[b, h, p])
            body = p[idx >= W]
            assert (body[1:] > body[:-1]).all(), "kept rows must stay in stream order"
            assert int(valid[b, h, W:].sum()) == int(sg[b, h] - W + sl[b, h])
    assert int(valid.sum()) == int((sg - W + sl).sum() + (roles[:, :, S - W // C:] == 2).sum() * C)
    assert not hip.cache_k[:, :, hip.n_ctx_data:].any()


def test_cfg4_streamed_eviction_equals_bulk():
    """The same 16 x 8 x 65536-token stream appended chunk by chunk (1024 x update(64) + post_update(64)) leaves
    the sizes, the surviving tokens and their rows that one bulk post_update(65536) leaves."""
    from neuralattentionsearch_amd.cache import NAtSChunkLayerCache
    say("evict cfg4 streamed against bulk")
    B, H, L, D, C, W = 16, 8, 65536, 128, 64, 512
    S = L // C
    rng = np.random.default_rng(1)
    roles = rng.choice(3, size=(B, H, S), p=(0.10, 0.15, 0.75)).astype(np.uint8)
    roles[:, :, 0] = 0
    g = torch.Generator(device="cuda").manual_seed(1)
    k = torch.randn(B, H, L, D, generator=g, device="cuda", dtype=torch.bfloat16)
    v = torch.randn(B, H, L, D, generator=g, device="cuda", dtype=torch.bfloat16)
    tsi = one_hot_roles(roles, dtype=torch.bfloat16).cuda()
    bulk = NAtSChunkLayerCache(B, H, W, chunk_size=C, device="cuda", track_positions=True)
    bulk.update(k, v, tsi)
    bulk.post_update(L)
    stream = NAtSChunkLayerCache(B, H, W, chunk_size=C, device="cuda", track_positions=True)
    for s in range(S):
        stream.update(k[:, :, s * C:(s + 1) * C], v[:, :, s * C:(s + 1) * C], tsi[:, :, s:s + 1])
        stream.post_update(C)
    assert torch.equal(stream.size_global_kv, bulk.size_global_kv)
    assert torch.equal(stream.size_local_kv, bulk.size_local_kv)
    assert stream.n_ctx_data == bulk.n_ctx_data and stream.sliding_queue_tail == bulk.sliding_queue_tail
    n = bulk.n_ctx_data
    vs, vb = stream.valid_tokens[:, :, :n], bulk.valid_tokens[:, :, :n]
    assert torch.equal(vs, vb)
    ps, pb = stream.token_positions[:, :, :n], bulk.token_positions[:, :, :n]
    assert torch.equal(torch.where(vs, ps, -1), torch.where(vb, pb, -1))
    m = vs.unsqueeze(-1)
    assert torch.equal(stream.cache_k[:, :, :n] * m, bulk.cache_k[:, :, :n] * m)
    assert torch.equal(stream.cache_v[:, :, :n] * m, bulk.cache_v[:, :, :n] * m)



@pytest.mark.parametrize("C,W,per_token", [(64, 256, False), (16, 32, False), (1, 32, True)])
def test_a_reset_cache_evicts_its_next_prefill_on_a_guessed_capacity(C, W, per_token, monkeypatch):
    """A cache object that is reset and fed a new prompt launches the first eviction into a cache sized from the share
    of rows it kept last time, before the plan kernel's numbers have reached the host.  The state must be the oracle's
    byte for byte whether the guess was right, too small (the eviction runs again at the right size), far too large
    (spare rows: zeros, not valid) or moot (every chunk sliding-window: the reference works in place), and the
    tokens appended afterwards must land in rows that look as the reference's zero padding does."""
    from neuralattentionsearch_amd.cache import NAtSChunkLayerCache, NAtSLayerCache
    from oracle.nats_oracle import TokenCacheOracle
    # Uninitialised GPU memory holds 0x7f bytes for the length of this test (valid bytes that are not 0, positions
    # that are not -1, values that are not 0), so that a spare row nobody initialised shows.
    real_empty = torch.empty

    def poisoned_empty(*args, **kwargs):
        t = real_empty(*args, **kwargs)
        if t.is_cuda and t.numel():
            t.view(torch.uint8).fill_(0x7F)
        return t

    monkeypatch.setattr(torch, "empty", poisoned_empty)
    B, H, D, dtype = 2, 3, 64, torch.bfloat16
    hip = (NAtSLayerCache(B, H, W, device="cuda", track_positions=True) if per_token
           else NAtSChunkLayerCache(B, H, W, chunk_size=C, device="cuda", track_positions=True))
    g = torch.Generator().manual_seed(C + W)
    rng = np.random.default_rng(C)
    runs = [(40 * max(C, 16) + 3, (0.2, 0.3, 0.5)),     # no history yet: the host waits for the size
            (40 * max(C, 16) + 3, (0.2, 0.3, 0.5)),     # the same share again: the guess holds
            (30 * max(C, 16), (0.7, 0.2, 0.1)),         # far more rows kept: too small, runs again
            (50 * max(C, 16) + 1, (0.02, 0.08, 0.9)),   # far fewer rows kept: spare rows
            (6 * max(C, 16), (0.0, 0.0, 1.0)),          # sliding-window only: the uncompacted cache, in place
            (20 * max(C, 16) + 5, (0.3, 0.3, 0.4))]
    for ri, (L, p) in enumerate(runs):
        hip.reset_cache()
        st = TokenCacheOracle(B=B, H=H, W=W) if per_token else ChunkCacheOracle(B=B, H=H, W=W, C=C)
        lens = [L] + [1] * (2 * max(C, 16) + 3) + [max(C, 16) + 7]
        segs = [(n, rng.choice(3, size=(B, H, n), p=p).astype(np.uint8)) for n in lens] if per_token \
            else role_stream(rng, B, H, C, lens, p)
        if p[2] == 1.0 and not per_token:
            segs[0][1][:] = 2  # (role_stream marks the sink chunk global; here really every chunk slides)
        for oi, (x_len, roles) in enumerate(segs):
            say("evict on a guessed capacity", (C, W, per_token), "run", ri, "op", oi, "x_len", x_len)
            k = torch.randn(B, H, x_len, D, generator=g).to(dtype)
            v = torch.randn(B, H, x_len, D, generator=g).to(dtype)
            st.update(k, v, roles)
            hip.update(k.cuda(), v.cuda(), one_hot_roles(roles, dtype=dtype).cuda())
            st.post_update(x_len)
            hip.post_update(x_len)
            compare(hip, st, (ri, oi, x_len))


def test_the_container_takes_its_layers_up_again_after_a_reset():
    """NAtSCache.reset_cache empties the container (components/cache/dyn_cache.py:76-78); the next prompt's updates take
    the layer objects up again, so that their first evictions run on a guessed capacity, and the K / V a layer holds
    for a possible relaunch are released once the next layer has been queued.  State == oracle after every prompt."""
    from neuralattentionsearch_amd import ops
    from neuralattentionsearch_amd.cache import NAtSCache
    B, H, D, C, W, n_layers, dtype = 2, 2, 64, 16, 32, 3, torch.bfloat16
    cache = NAtSCache(W, C, track_positions=True)
    g = torch.Generator().manual_seed(5)
    rng = np.random.default_rng(5)
    first_objects, seqs = None, set()
    for prompt, (L, p) in enumerate([(40 * C + 3, (0.2, 0.3, 0.5)), (37 * C, (0.25, 0.25, 0.5)), (30 * C, (0.7, 0.2, 0.1))]):
        cache.reset_cache()
        assert len(cache) == 0 and cache.get_seq_length() == 0
        oracles = [ChunkCacheOracle(B=B, H=H, W=W, C=C) for _ in range(n_layers)]
        for x_len, roles in role_stream(rng, B, H, C, [L, 1, 1, C], p):
            for li in range(n_layers):
                say("container reuse", "prompt", prompt, "layer", li, "x_len", x_len)
                k = torch.randn(B, H, x_len, D, generator=g).to(dtype)
                v = torch.randn(B, H, x_len, D, generator=g).to(dtype)
                oracles[li].update(k, v, roles)
                cache.update(k.cuda(), v.cuda(), li, {"token_states_info": one_hot_roles(roles, dtype=dtype).cuda()})
                oracles[li].post_update(x_len)
                cache.post_update(li, x_len)
                if li > 0:
                    assert cache.cache_model[li - 1]._redo is None  # nothing of the caller's is held any longer
        for li in range(n_layers):
            compare(cache.cache_model[li], oracles[li], (prompt, li))
            seqs.add(cache.cache_model[li]._evict.seq)
        if first_objects is None:
            first_objects = list(cache.cache_model)
        else:
            assert all(a is b for a, b in zip(first_objects, cache.cache_model))
            assert all(c._kept_share is not None for c in cache.cache_model)
    assert len(seqs) == 3 * n_layers  # sequence numbers are drawn process-wide: no two plans share one
    # a dropped cache hands its pinned mirror back to the module's pool, where the next cache finds it
    mirror = cache.cache_model[0]._evict.mirror
    cache.reset_cache()
    cache._spare_layers = []
    del first_objects, cache
    import gc
    gc.collect()
    assert any(m is mirror for m in ops._mirror_pool)
    assert ops.EvictBuffers("cuda").mirror is not None
