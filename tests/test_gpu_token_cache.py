"""GPU parity, bit exact: the HIP-backed per-token cache NAtSLayerCache (chunk_size == 1, eviction deferred until 16
tokens are pending) against the oracle's TokenCacheOracle, which tests/test_oracle_golden.py pins to vectors written
by the reference's own class."""
import numpy as np
import pytest
import torch

from oracle import nats_oracle as orc
from tests.golden_io import TokenGolden
from tests.gpu_util import say
from tests.test_gpu_evict import compare

pytestmark = pytest.mark.gpu

GOLD = TokenGolden()
TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2}


def bits(t):
    return t.contiguous().view(torch.int16 if t.element_size() == 2 else torch.int32)


def drive(name, B, H, D, W, U, segs, dtype, seed, n_rep=0):
    """segs: list of (x_len, roles uint8 [B, H, x_len]).  With n_rep > 0 every call also runs its attention (prefill
    from empty, segment over the cache, or one-token decode with and without the dead-region hint) against masked
    attention over the oracle's cache."""
    from neuralattentionsearch_amd import ops
    from neuralattentionsearch_amd.cache import NAtSLayerCache
    hip = NAtSLayerCache(B, H, W, update_chunk_size=U, device="cuda", track_positions=True)
    st = orc.TokenCacheOracle(B=B, H=H, W=W, U=U)
    g = torch.Generator().manual_seed(seed)
    for oi, (x_len, roles) in enumerate(segs):
        say("token cache", name, "op", oi, "x_len", x_len, dtype)
        k = torch.randn(B, H, x_len, D, generator=g).to(dtype)
        v = torch.randn(B, H, x_len, D, generator=g).to(dtype)
        ko, vo = st.update(k, v, roles)
        kh, vh = hip.update(k.cuda(), v.cuda(), orc.one_hot_roles(roles, dtype=dtype).cuda())
        assert torch.equal(bits(kh.cpu()), bits(ko)), (name, oi, "update K")
        want_mask = st.generate_mask(x_len)
        got_mask = hip.generate_mask(x_len).cpu().numpy()
        assert got_mask.shape == want_mask.shape, (name, oi, "mask shape", got_mask.shape, want_mask.shape)
        assert np.array_equal(got_mask, want_mask), (name, oi, "mask", np.argwhere(got_mask != want_mask)[:8])
        if n_rep:
            q = torch.randn(B, H * n_rep, x_len, D, generator=g).to(dtype)
            if want_mask.shape == (1, 1, 1, 1):  # the very first token: it sees itself
                want_mask = np.ones((B, H, 1, 1), dtype=bool)
            want = orc.masked_attention(q.float(), ko.float(), vo.float(), want_mask)
            if st.seen == 0:
                got = ops.prefill_attention(q.cuda(), kh, vh, torch.from_numpy(roles).cuda(), 1, W)
            elif x_len > 1:
                got = hip.segment_attention(q.cuda())
            else:
                n_rows = kh.shape[2]
                got = ops.decode_attention(q.cuda(), kh, vh, hip.valid_tokens, n_rows)
                row_end, tail_start = hip.decode_hint()
                hinted = ops.decode_attention(q.cuda(), kh, vh, hip.valid_tokens, n_rows, row_end=row_end,
                                              tail_start=tail_start)
                # (the hint changes how the rows are cut into tiles, hence the order of the sums: both forms are
                # held to the tolerance on their own)
                err_h = (hinted.float().cpu() - want).abs().max().item()
                assert err_h <= TOL[dtype], (name, oi, "attention with the dead-region hint", err_h)
            err = (got.float().cpu() - want).abs().max().item()
            assert err <= TOL[dtype], (name, oi, "attention", err)
        st.post_update(x_len)
        hip.post_update(x_len)
        compare(hip, st, (name, oi, x_len))
    return hip, st


def golden_segs(name):
    si, sc = GOLD.scenario(name)
    return sc, [(op["x_len"], GOLD.op(si, oi)["roles"]) for oi, op in enumerate(sc["ops"])]


@pytest.mark.parametrize("name", GOLD.scenario_names())
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_replay_reference_scenarios(name, dtype):
    sc, segs = golden_segs(name)
    drive(name, sc["B"], sc["H"], 8, sc["W"], sc["U"], segs, dtype, seed=len(name))


@pytest.mark.parametrize("name", GOLD.scenario_names())
@pytest.mark.parametrize("dtype,D,n_rep", [(torch.float32, 64, 2), (torch.bfloat16, 128, 4)])
def test_attention_on_reference_scenarios(name, dtype, D, n_rep):
    """Every call of the reference scenarios with its attention: the mask the kernels work from is the class's own,
    including the tokens a deferred eviction leaves visible."""
    sc, segs = golden_segs(name)
    drive(name, sc["B"], sc["H"], D, sc["W"], sc["U"], segs, dtype, seed=len(name) + 1, n_rep=n_rep)


def role_stream(rng, B, H, lens, p):
    segs = []
    for i, x_len in enumerate(lens):
        roles = rng.choice(3, size=(B, H, x_len), p=p).astype(np.uint8)
        if i == 0:
            roles[:, :, 0] = 0
        segs.append((x_len, roles))
    return segs


@pytest.mark.parametrize("W,D,dtype,n_rep,p", [(64, 128, torch.bfloat16, 4, (0.1, 0.2, 0.7)),
                                               (16, 64, torch.float32, 1, (0.3, 0.3, 0.4)),
                                               (256, 128, torch.bfloat16, 4, (0.05, 0.15, 0.8))])
def test_random_streams(W, D, dtype, n_rep, p):
    """Longer seeded streams: a prefill of some hundred tokens, one-token steps across many deferred evictions,
    segments of every length class (shorter than the update chunk, shorter and longer than the window)."""
    rng = np.random.default_rng(W + D)
    lens = [5 * W + 7] + [1] * 40 + [W // 2 + 3, 9, 1, 1, 2 * W + 5, 3] + [1] * 20 + [16, 16, 700]
    drive(f"random_W{W}", 2, 4, D, W, 16, role_stream(rng, 2, 4, lens, p), dtype, seed=W, n_rep=n_rep)


def test_container_builds_the_per_token_class_for_chunk_size_one():
    from neuralattentionsearch_amd.cache import NAtSCache, NAtSChunkLayerCache, NAtSLayerCache
    say("container: chunk_size 1 -> NAtSLayerCache")
    c1, c8 = NAtSCache(32, 1), NAtSCache(32, 8)
    k = torch.zeros(1, 2, 4, 64, device="cuda")
    tsi = orc.one_hot_roles(np.zeros((1, 2, 4), dtype=np.uint8)).cuda()
    c1.update(k, k, 0, {"token_states_info": tsi})
    c8.update(k, k, 0, {"token_states_info": tsi[:, :, :1]})
    assert type(c1.cache_model[0]) is NAtSLayerCache and c1.cache_model[0].update_chunk_size == 16
    assert type(c8.cache_model[0]) is NAtSChunkLayerCache
    assert c1.get_nats_chunk_fill_size(0) == 0  # as the reference's container answers for chunk_size == 1
    with pytest.raises(NotImplementedError):
        NAtSCache(8, 1).update(k, k, 0, {"token_states_info": tsi})  # window below the update chunk size


@pytest.mark.parametrize("W,D,dtype,n_rep,p", [(16, 64, torch.float32, 2, (0.3, 0.3, 0.4)),
                                               (64, 128, torch.bfloat16, 4, (0.1, 0.2, 0.7)),
                                               (2, 128, torch.bfloat16, 1, (0.2, 0.2, 0.6))])
def test_random_streams_without_deferral(W, D, dtype, n_rep, p):
    """update_chunk_size == 1: every call evicts; one-token steps take the reference's one-step branch
    (nats_layer_cache.py:328-367) unless the token is sliding-window on every head."""
    rng = np.random.default_rng(7 * W + D)
    lens = [1] * 5 + [3 * W + 5] + [1] * 50 + [W // 2 + 3, 1, 1, 2 * W + 5, 2] + [1] * 30 + [300]
    segs = role_stream(rng, 2, 4, lens, p)
    for i in (8, 9, 30):  # some steps whose token is sliding-window on every head (:316-327 instead of :328-367)
        segs[i] = (1, np.full((2, 4, 1), 2, np.uint8))
    drive(f"random_U1_W{W}", 2, 4, D, W, 1, segs, dtype, seed=W, n_rep=n_rep)
