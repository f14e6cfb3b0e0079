"""The oracle's cache state machine against vectors written by the reference's own
NAtSChunkLayerCache on CPU (tests/golden/make_golden.py): every byte of cache_k, cache_v,
valid_tokens, the size tensors and the scalars, after every post_update, plus every mask."""
import numpy as np
import pytest
import torch

from oracle.nats_oracle import ChunkCacheOracle, TokenCacheOracle
from tests.golden_io import Golden, TokenGolden

GOLD = Golden()
TOKEN_GOLD = TokenGolden()


@pytest.mark.parametrize("name", GOLD.scenario_names())
def test_cache_state_machine_matches_reference_vectors(name):
    si, sc = GOLD.scenario(name)
    B, H, D, C, W = sc["B"], sc["H"], sc["D"], sc["C"], sc["W"]
    st = ChunkCacheOracle(B=B, H=H, W=W, C=C)
    t_seen = 0
    for oi, op in enumerate(sc["ops"]):
        g = GOLD.op(si, oi)
        x_len = op["x_len"]
        pos = torch.arange(t_seen, t_seen + x_len, dtype=torch.float32).view(1, 1, -1, 1) + 1.0
        k = pos.expand(B, H, x_len, D).contiguous()
        v = torch.from_numpy(g["v"])
        st.update(k, v, g["roles"])
        mask = st.generate_mask(x_len)
        assert mask.shape == g["mask"].shape, (name, oi, mask.shape, g["mask"].shape)
        assert np.array_equal(mask, g["mask"]), (name, oi, "mask")
        st.post_update(x_len)
        t_seen += x_len
        where = (name, oi, x_len)
        assert np.array_equal(st.size_global, g["size_global"]), where
        assert np.array_equal(st.size_local, g["size_local"]), where
        scal = [st.n_ctx_data, st.gmin, st.tail, st.fill, st.fill_last, st.seen]
        assert scal == [int(x) for x in g["scalars"]], (where, scal, g["scalars"])
        assert st.valid.shape == g["valid"].shape, where
        assert np.array_equal(st.valid, g["valid"]), where
        assert np.array_equal(st.cache_k.numpy(), g["cache_k"]), where
        assert np.array_equal(st.cache_v.numpy(), g["cache_v"]), where
        # the position shadow is consistent with the position-coded keys wherever a row is valid
        kk = st.cache_k.numpy()[..., 0]
        vv = st.valid[:, :, :st.n_ctx_data]
        assert np.array_equal(kk[:, :, :st.n_ctx_data][vv] - 1, st.pos_k[:, :, :st.n_ctx_data][vv]), where


@pytest.mark.parametrize("name", TOKEN_GOLD.scenario_names())
def test_token_cache_state_machine_matches_reference_vectors(name):
    """The per-token class (chunk_size == 1: 16-token deferred eviction, ring of rows copied whatever the role,
    `tail` = slot written last) against vectors written by the reference's own NAtSLayerCache on CPU
    (tests/golden/make_golden_token.py)."""
    si, sc = TOKEN_GOLD.scenario(name)
    assert sc["error"] is None and sc["ops"], name
    B, H, D, W, U = sc["B"], sc["H"], sc["D"], sc["W"], sc["U"]
    st = TokenCacheOracle(B=B, H=H, W=W, U=U)
    t_seen = 0
    for oi, op in enumerate(sc["ops"]):
        g = TOKEN_GOLD.op(si, oi)
        x_len = op["x_len"]
        pos = torch.arange(t_seen, t_seen + x_len, dtype=torch.float32).view(1, 1, -1, 1) + 1.0
        k = pos.expand(B, H, x_len, D).contiguous()
        st.update(k, torch.from_numpy(g["v"]), g["roles"])
        mask = st.generate_mask(x_len)
        where = (name, oi, x_len)
        assert mask.shape == g["mask"].shape, (where, mask.shape, g["mask"].shape)
        assert np.array_equal(mask, g["mask"]), (where, "mask", np.argwhere(mask != g["mask"])[:5])
        st.post_update(x_len)
        t_seen += x_len
        assert np.array_equal(st.size_global, g["size_global"]), where
        assert np.array_equal(st.size_local, g["size_local"]), where
        scal = [st.n_ctx_data, st.gmin, st.tail, st.fill, st.fill_last, st.seen]
        assert scal == [int(x) for x in g["scalars"]], (where, scal, g["scalars"])
        assert st.valid.shape == g["valid"].shape, (where, st.valid.shape, g["valid"].shape)
        assert np.array_equal(st.valid, g["valid"]), where
        assert np.array_equal(st.cache_k.numpy(), g["cache_k"]), where
        assert np.array_equal(st.cache_v.numpy(), g["cache_v"]), where
        kk = st.cache_k.numpy()[..., 0]
        vv = st.valid[:, :, :st.n_ctx_data]
        assert np.array_equal(kk[:, :, :st.n_ctx_data][vv] - 1, st.pos_k[:, :, :st.n_ctx_data][vv]), where
