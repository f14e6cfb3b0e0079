"""CPU: host-side logic of the tensor front end that needs no kernel."""
import torch

from neuralattentionsearch_amd import ops


def test_roles_travel_with_their_one_hot_tensor_until_either_is_written():
    """A caller that edits token_states_info in place after sampling (a slot forced global, a head masked) must get
    the roles of the edited tensor (models/transformer/attention/nats_attention.py:96-109 hands only the one-hot
    tensor on)."""
    roles = torch.tensor([[[0, 1, 2, 2]]], dtype=torch.uint8)
    one_hot = torch.nn.functional.one_hot(roles.long(), 3).float()
    ops._attach_roles(one_hot, roles)
    assert ops.roles_from_one_hot(one_hot) is roles
    one_hot[0, 0, 1] = torch.tensor([1.0, 0.0, 0.0])  # slot 1 forced global after the fact
    got = ops.roles_from_one_hot(one_hot)
    assert got is not roles and got.tolist() == [[[0, 0, 2, 2]]]
    ops._attach_roles(one_hot, got)
    got[0, 0, 3] = 1  # the compact form edited instead
    assert ops.roles_from_one_hot(one_hot).tolist() == [[[0, 0, 2, 2]]]


def test_plan_sequence_numbers_are_process_wide():
    a = [ops._next_evict_seq() for _ in range(5)]
    assert all(y == x + 1 for x, y in zip(a, a[1:])) and min(a) >= 1


def test_the_bench_role_logit_biases_give_the_configured_shares():
    """bench.py draws its roles as the argmax of N(0, 1) logits plus committed constants, with the 0.1 on the global
    logit that the role kernel adds (models/transformer/attention/nats_attention.py:96-109).  The constants solve
    P(option i wins) = its configured share; a large sample lands on the shares."""
    import bench
    from oracle import nats_oracle as orc
    for shares in bench.ROLE_LOGIT_BIAS:
        logits = bench.biased_role_logits(1, 1, 400000, 8, shares, device="cpu")
        roles = orc.roles_from_logits(logits, bench.ROLE_GLOBAL_BIAS, False, False)
        got = [(roles == i).mean() for i in range(3)]
        assert all(abs(g - s) < 2e-3 for g, s in zip(got, shares)), (shares, got)
    # and the FLOP count of the prefill leg equals a brute-force count of the visible (query, key) pairs
    import numpy as np
    rng = np.random.default_rng(0)
    roles = rng.choice(3, size=(2, 3, 40), p=(0.2, 0.3, 0.5)).astype(np.uint8)
    roles[:, :, 0] = 0
    C, W, L = 8, 16, 320
    flops, dense = bench.prefill_flops(roles, L, C, W, 64, 4)
    mask = orc.prefill_mask(roles, L, C, W)
    chunk_pairs = mask.reshape(2, 3, 40, C, 40, C).any(axis=(3, 5))
    off = chunk_pairs.sum() - 2 * 3 * 40
    assert flops == 4.0 * 64 * 4 * (off * C * C + 2 * 3 * 40 * (C * (C + 1) // 2))
    assert dense == 4.0 * 64 * 4 * 2 * 3 * (L * (L + 1) // 2)
