"""GPU parity, bit exact: role assignment, next-global scan, token masks, tile-skip map."""
import numpy as np
import pytest
import torch

from oracle import nats_oracle as orc
from tests.gpu_util import draw_roles, say, to_dev

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("bias,first,last", [(0.1, True, False), (0.0, False, True), (0.1, False, False)])
def test_roles_from_logits_bit_exact(dtype, bias, first, last):
    from neuralattentionsearch_amd import ops
    say("roles_from_logits", dtype, bias, first, last)
    g = torch.Generator().manual_seed(0)
    logits = torch.randn(3, 77, 5, 3, generator=g).to(dtype)
    # ties and near-ties, where the bias and its rounding decide
    logits[0, :10, :, 1] = logits[0, :10, :, 0]
    logits[1, :10, :, 2] = logits[1, :10, :, 1]
    logits[2, :10, :, 1] = logits[2, :10, :, 0] + 0.1
    want = orc.roles_from_logits(logits, bias, first, last)
    roles, one_hot = ops.roles_from_logits(logits.cuda(), bias, first, last)
    assert np.array_equal(roles.cpu().numpy(), want)
    assert one_hot.dtype == dtype
    assert torch.equal(one_hot.cpu().float(), orc.one_hot_roles(want))
    assert np.array_equal(ops.roles_from_one_hot(one_hot).cpu().numpy(), want)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_roles_match_torch_ops_on_the_device(dtype):
    """The reference's own statement, run by torch on the GPU: logit[..., 0] += 0.1; logit.max(-1)[1]."""
    from neuralattentionsearch_amd import ops
    say("roles vs torch on device", dtype)
    g = torch.Generator().manual_seed(1)
    logits = (torch.randn(4, 512, 8, 3, generator=g) * 0.2).to(dtype)
    logits[0, :, :, 1] = logits[0, :, :, 0] + 0.1
    dev = logits.cuda()
    ref = dev.clone()
    ref[..., 0] += 0.1
    index = ref.max(-1, keepdim=True)[1]
    want = index.squeeze(-1).transpose(1, 2).contiguous().to(torch.uint8)
    roles, _ = ops.roles_from_logits(dev, 0.1, False, False)
    assert torch.equal(roles, want)


@pytest.mark.parametrize("S", [1, 7, 64, 65, 200, 1024])
def test_role_scan_matches_next_global_index(S):
    from neuralattentionsearch_amd import ops
    say("role_scan", S)
    roles = draw_roles(S, 2, 3, S, first_global=False)
    if S > 10:
        roles[0, 0, :] = 1  # no global at all
        roles[0, 1, S // 2:] = 2  # none after the middle
    end_idx, vis_lim = ops.role_scan(to_dev(roles), W=8, C=4)
    want = orc.next_global_index(roles == 0)
    assert np.array_equal(end_idx.cpu().numpy(), want)
    lim = vis_lim.cpu().numpy()
    n = np.arange(S)[None, None]
    expect = np.where(roles == 0, np.iinfo(np.int32).max, np.where(roles == 2, n + 2, want))
    assert np.array_equal(lim, expect)


@pytest.mark.parametrize("L,C,W", [(12, 2, 4), (507, 1, 4), (507, 8, 16), (300, 32, 64), (1000, 64, 256), (640, 128, 256),
                                   (2048, 64, 128)])
def test_prefill_mask_bit_exact(L, C, W):
    from neuralattentionsearch_amd import ops
    say("prefill_mask", L, C, W)
    S = -(-L // C)
    B, H = (1, 2) if L > 600 else (2, 3)
    roles = draw_roles(L + C, B, H, S)
    want = orc.prefill_mask(roles, L, C, W)
    got = ops.prefill_mask(to_dev(roles), L, C, W).cpu().numpy()
    assert got.shape == want.shape
    assert np.array_equal(got, want)


@pytest.mark.parametrize("L,C", [(2000, 1), (6000, 4), (6000, 8)])
def test_prefill_mask_with_long_local_runs(L, C):
    """Hundreds of local slots between two global ones: the search for the next global slot crosses several blocks
    of 64 slots (the search inside the key-limit kernel that a prefill from an empty cache runs)."""
    from neuralattentionsearch_amd import ops
    say("prefill_mask long local runs", L, C)
    rng = np.random.default_rng(L + C)
    S = -(-L // C)
    roles = rng.choice(3, size=(1, 2, S), p=(0.003, 0.9, 0.097)).astype(np.uint8)
    roles[:, :, 0] = 0
    roles[0, 1, S // 3:] = 1  # no global slot after the first third (the last slot counts as one)
    W = 8 * C
    want = orc.prefill_mask(roles, L, C, W)
    got = ops.prefill_mask(to_dev(roles), L, C, W).cpu().numpy()
    assert np.array_equal(got, want)


def test_prefill_mask_worked_example():
    from neuralattentionsearch_amd import ops
    say("prefill_mask worked example")
    roles = np.array([[[0, 1, 2, 0, 1, 2]]], dtype=np.uint8)
    got = ops.prefill_mask(to_dev(roles), 12, 2, 4).cpu().numpy()[0, 0]
    rows = [[1], [1, 1], [1, 1, 1], [1, 1, 1, 1], [1, 0, 1, 1, 1], [1, 0, 0, 1, 1, 1]]
    vis = np.zeros((6, 6), dtype=bool)
    for m, r in enumerate(rows):
        vis[m, :len(r)] = np.array(r, dtype=bool)
    want = np.tril(np.repeat(np.repeat(vis, 2, 0), 2, 1))
    assert np.array_equal(got, want)


@pytest.mark.parametrize("L,C,W", [(2048, 64, 128), (1000, 64, 256), (1024, 16, 64), (2048, 128, 256), (4096, 64, 256)])
def test_tile_map_covers_every_unmasked_tile(L, C, W):
    from neuralattentionsearch_amd import ops
    say("tile_map", L, C, W)
    S = -(-L // C)
    roles = draw_roles(L, 1, 4, S, p=(0.05, 0.15, 0.8))
    mask = orc.prefill_mask(roles, L, C, W)
    T = -(-L // 64)
    pad = T * 64 - L
    mp = np.pad(mask, ((0, 0), (0, 0), (0, pad), (0, pad)))
    need = mp.reshape(1, 4, T, 64, T, 64).any(axis=(3, 5))
    got = ops.prefill_tile_map(to_dev(roles), L, C, W).cpu().numpy()
    assert not (need & ~got).any(), "a tile with unmasked scores is skipped"
    if C >= 64:
        assert np.array_equal(got, need), "at chunk >= tile the map must be exact"
    else:
        assert got.sum() <= 1.5 * need.sum() + 8
