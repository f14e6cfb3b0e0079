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
