"""Pins the oracle's closed-form pieces against what the mathematics fixes (no GPU)."""
import itertools
import math

import numpy as np
import pytest
import torch

from oracle import nats_oracle as orc


def test_roles_first_maximum_and_bias_on_all_orderings():
    vals = [-1.0, 0.0, 0.05, 0.1, 1.0]
    for a, b, c in itertools.product(vals, repeat=3):
        lg = torch.tensor([[[[a, b, c]]]], dtype=torch.float32)
        got = orc.roles_from_logits(lg, 0.1)[0, 0, 0]
        x = [np.float32(a) + np.float32(0.1), np.float32(b), np.float32(c)]
        want = 0 if x[0] >= x[1] and x[0] >= x[2] else (1 if x[1] >= x[2] else 2)
        assert got == want, (a, b, c)


def test_roles_forced_slots():
    lg = torch.zeros(2, 5, 3, 3)
    lg[..., 2] = 5.0
    r = orc.roles_from_logits(lg, 0.1, force_first_global=True, force_last_global=True)
    assert (r[:, :, 0] == 0).all() and (r[:, :, -1] == 0).all() and (r[:, :, 1:-1] == 2).all()


def test_next_global_index_closed_form_and_brute_force():
    # globals at 2, 5, 6 (and the forced last slot): the neighbouring quantity of the reference docstring
    flags = np.array([[[0, 0, 1, 0, 0, 1, 1]]], dtype=bool)
    assert orc.next_global_index(flags)[0, 0].tolist() == [2, 2, 2, 5, 5, 5, 6]
    rng = np.random.default_rng(0)
    for _ in range(50):
        S = int(rng.integers(1, 40))
        f = rng.random((1, 1, S)) < 0.3
        got = orc.next_global_index(f)[0, 0]
        for n in range(S):
            cand = [g for g in range(n, S) if f[0, 0, g] or g == S - 1]
            assert got[n] == cand[0]


def test_docstring_seven_by_seven_mask():
    """components/masks/utils_simple.py:94-107: flags F F T F T T T (token granularity, no sliding window)."""
    roles = np.array([[[1, 1, 0, 1, 0, 0, 0]]], dtype=np.uint8)
    got = orc.prefill_mask(roles, 7, 1, 4)[0, 0]
    want = np.array([
        [1, 0, 0, 0, 0, 0, 0],
        [1, 1, 0, 0, 0, 0, 0],
        [1, 1, 1, 0, 0, 0, 0],
        [0, 0, 1, 1, 0, 0, 0],
        [0, 0, 1, 1, 1, 0, 0],
        [0, 0, 1, 0, 1, 1, 0],
        [0, 0, 1, 0, 1, 1, 1]], dtype=bool)
    assert np.array_equal(got, want)


def test_special_role_patterns_reduce_to_textbook_masks():
    L, C, W = 48, 4, 8
    S = L // C
    allg = np.zeros((1, 1, S), dtype=np.uint8)
    assert np.array_equal(orc.prefill_mask(allg, L, C, W)[0, 0], np.tril(np.ones((L, L), dtype=bool)))
    allsw = np.full((1, 1, S), 2, dtype=np.uint8)
    m = np.arange(L)[:, None]
    n = np.arange(L)[None, :]
    band = (n <= m) & ((m // C - n // C) <= W // C)
    assert np.array_equal(orc.prefill_mask(allsw, L, C, W)[0, 0], band)
    # all local: no global ever closes a run, so everything stays visible (one open sub-sequence)
    alll = np.ones((1, 1, S), dtype=np.uint8)
    assert np.array_equal(orc.prefill_mask(alll, L, C, W)[0, 0], np.tril(np.ones((L, L), dtype=bool)))


def test_mask_predicate_brute_force():
    rng = np.random.default_rng(1)
    for _ in range(20):
        C = int(rng.choice([1, 2, 4]))
        wc = int(rng.integers(1, 4))
        S = int(rng.integers(2, 12))
        L = S * C - int(rng.integers(0, C))
        roles = rng.choice(3, size=(1, 1, S)).astype(np.uint8)
        got = orc.prefill_mask(roles, L, C, wc * C)[0, 0]
        r = roles[0, 0]
        for m in range(L):
            for n in range(L):
                mc, nc = m // C, n // C
                if n > m:
                    want = False
                elif r[nc] == 0 or nc == S - 1 and r[nc] != 2:
                    want = True
                elif r[nc] == 2:
                    want = mc - nc <= wc
                else:  # local: visible until (and including) the next global slot, the last slot counting
                    nxt = next(g for g in range(nc, S) if r[g] == 0 or g == S - 1)
                    want = mc <= nxt
                assert got[m, n] == want, (C, wc, S, L, m, n)


def test_worked_example_of_the_cache():
    """C=2, W=4, L=12, roles G L S G L S: ring [0 0 t10 t11], rows t0 t1 t6 t7 | t8 t9."""
    st = orc.ChunkCacheOracle(B=1, H=1, W=4, C=2)
    k = torch.arange(12, dtype=torch.float32).view(1, 1, 12, 1) + 1
    roles = np.array([[[0, 1, 2, 0, 1, 2]]], dtype=np.uint8)
    st.update(k, k.clone(), roles)
    st.post_update(12)
    assert st.n_ctx_data == 10 and st.tail == 0
    assert st.size_global[0, 0] == 8 and st.size_local[0, 0] == 2
    assert st.pos_k[0, 0].tolist() == [-1, -1, 10, 11, 0, 1, 6, 7, 8, 9]
    assert st.valid[0, 0].tolist() == [False, False, True, True] + [True] * 6


def test_decode_attention_equals_masked_sdpa():
    g = torch.Generator().manual_seed(0)
    B, Hq, Hkv, N, D = 2, 4, 2, 50, 16
    q = torch.randn(B, Hq, 1, D, generator=g)
    k = torch.randn(B, Hkv, N, D, generator=g)
    v = torch.randn(B, Hkv, N, D, generator=g)
    valid = torch.rand(B, Hkv, N, generator=g) < 0.5
    valid[:, :, -1] = True
    a = orc.decode_attention(q, k, v, valid, N)
    b = orc.masked_attention(q, k, v, valid[:, :, None, :])
    assert (a - b).abs().max().item() < 1e-5


def test_masked_attention_explicit_form_matches_sdpa():
    g = torch.Generator().manual_seed(1)
    q = torch.randn(1, 4, 24, 8, generator=g)
    k = torch.randn(1, 2, 24, 8, generator=g)
    v = torch.randn(1, 2, 24, 8, generator=g)
    roles = np.array([[[0, 1, 2, 0, 1, 2], [0, 2, 2, 1, 0, 1]]], dtype=np.uint8)
    mask = orc.prefill_mask(roles, 24, 4, 8)
    a = orc.masked_attention(q, k, v, mask)
    b = orc.masked_attention(q, k, v, mask, explicit=True)
    assert (a - b).abs().max().item() < 1e-5


# ---- pooled_role_logits ---------------------------------------------------------------------------
def test_pooling_closed_forms():
    """Constant chunks pool to their constant; an open last chunk is averaged over C with zero padding (max
    pooling sees the zeros too); one-hot projection rows pick single pooled columns."""
    C, dim, H = 4, 6, 2
    x = torch.zeros(1, 10, dim)
    x[0, 0:4] = 2.0
    x[0, 4:8] = -3.0
    x[0, 8:10] = 5.0
    w = torch.zeros(H * 3, dim)
    for o in range(H * 3):
        w[o, o] = 1.0
    pooled, logits, carry, pad = orc.pooled_role_logits(x, w, C)
    assert pad == 2 and pooled.shape == (1, 3, dim) and logits.shape == (1, 3, H, 3)
    assert torch.equal(pooled[0, :, 0], torch.tensor([2.0, -3.0, 2.5]))  # 2 * 5 / 4: zeros count in the mean
    assert torch.equal(logits[0, :, 1, 2], pooled[0, :, 5])
    assert torch.equal(carry[0, 0], torch.full((dim,), 2.5))
    pooled_m, _, carry_m, _ = orc.pooled_role_logits(-x, w, C, merge_max=True)
    assert torch.equal(pooled_m[0, :, 0], torch.tensor([-2.0, 3.0, 0.0]))  # the zero padding wins over -5
    assert torch.equal(carry_m[0, 0], torch.full((dim,), -5.0))  # ... but is not carried on


@pytest.mark.parametrize("merge_max", [False, True])
def test_pooling_is_independent_of_how_the_stream_is_cut(merge_max):
    C, dim, H, B = 8, 16, 3, 2
    g = torch.Generator().manual_seed(5)
    x = torch.randn(B, 61, dim, generator=g)
    w = torch.randn(H * 3, dim, generator=g)
    whole, logits_whole, _, _ = orc.pooled_role_logits(x, w, C, merge_max=merge_max)
    n_full = 61 // C
    for cuts in ([61], [3, 2, 9, 1, 1, 30, 15], [8, 8, 8, 37], [5, 56]):
        pre, carry, pos, got = 0, None, 0, []
        for n in cuts:
            pooled, logits, carry_new, pad = orc.pooled_role_logits(x[:, pos:pos + n], w, C, pre_fill=pre, carry_in=carry,
                                                                    merge_max=merge_max)
            total = pre + n
            if pooled is not None:
                done = total // C
                got.append(pooled[:, :done])
                carry = carry_new
            else:
                carry = carry_new
            pre, pos = total % C, pos + n
        got = torch.cat(got, 1)
        assert got.shape[1] == n_full
        assert torch.allclose(got, whole[:, :n_full], atol=1e-6)
