"""GPU parity of the one-token decode attention over a ragged, evicted cache."""
import math

import numpy as np
import pytest
import torch

from oracle import nats_oracle as orc
from tests.gpu_util import say

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2}


def ragged_cache(seed, B, Hkv, D, W, C, n_max_chunks, dtype, frac=(0.1, 1.0), fill=0, poison=True):
    """A cache in the layout the reference leaves between calls: ring with random valid chunks, per-head
    global+local rows, stale rows up to the longest head, an open chunk of `fill` rows; invalid rows hold NaN."""
    rng = np.random.default_rng(seed)
    lens = (rng.uniform(frac[0], frac[1], size=(B, Hkv)) * n_max_chunks).round().astype(np.int64).clip(1) * C
    base = W + int(lens.max())
    n_rows = base + fill + 1  # + the token of this step
    n_alloc = -(-n_rows // C) * C
    g = torch.Generator().manual_seed(seed)
    k = torch.randn(B, Hkv, n_alloc, D, generator=g).to(dtype)
    v = torch.randn(B, Hkv, n_alloc, D, generator=g).to(dtype)
    valid = np.zeros((B, Hkv, n_alloc), dtype=bool)
    ring = rng.random((B, Hkv, W // C)) < 0.8
    valid[:, :, :W] = np.repeat(ring, C, axis=-1)
    for b in range(B):
        for h in range(Hkv):
            valid[b, h, W:W + lens[b, h]] = True
    valid[:, :, base:base + fill + 1] = True
    vt = torch.from_numpy(valid)
    if poison:
        k[~vt] = float("nan")
        v[~vt] = float("nan")
    ragged_cache.row_end = torch.from_numpy(W + lens)  # per head: end of its global + local rows
    ragged_cache.tail_start = base  # first row of the open chunk
    return k, v, vt, n_rows


def run_case(B, Hq, Hkv, D, W, C, n_max_chunks, dtype, seed=0, frac=(0.1, 1.0), fill=0, q_scale=1.0):
    """`q_scale` > 1 makes the scores peaked (their standard deviation in nats is q_scale): a row's output is then
    carried by a few keys and is of the size of v, and the error is held against the row's own magnitude."""
    from neuralattentionsearch_amd import ops
    say("decode", B, Hq, Hkv, D, W, C, n_max_chunks, dtype, seed, frac, fill, q_scale)
    k, v, valid, n_rows = ragged_cache(seed, B, Hkv, D, W, C, n_max_chunks, dtype, frac, fill)
    g = torch.Generator().manual_seed(seed + 100)
    q = (torch.randn(B, Hq, 1, D, generator=g) * q_scale).to(dtype)
    want = orc.decode_attention(q, k, v, valid, n_rows).float()
    rms = want.pow(2).mean(-1, keepdim=True).sqrt()
    bound = TOL[dtype] * (torch.maximum(rms, want.abs()) if q_scale > 1 else 1.0) + (2e-3 if q_scale > 1 else 0.0)
    got = ops.decode_attention(q.cuda(), k.cuda(), v.cuda(), valid.cuda(), n_rows).cpu().float()
    assert torch.isfinite(got).all(), "a row with valid == False was read (NaN poison leaked)"
    assert not ((got - want).abs() > bound).any(), f"max abs err {(got - want).abs().max().item()}"
    # the same call with the dead-region hint the cache object passes
    got2 = ops.decode_attention(q.cuda(), k.cuda(), v.cuda(), valid.cuda(), n_rows, row_end=ragged_cache.row_end.cuda(),
                                tail_start=ragged_cache.tail_start).cpu().float()
    assert torch.isfinite(got2).all()
    assert not ((got2 - want).abs() > bound).any(), f"max abs err with hint {(got2 - want).abs().max().item()}"
    if q_scale > 1:
        assert rms.min().item() > 0.05, rms.min().item()


@pytest.mark.parametrize("n_rep", [1, 2, 3, 4, 5, 6, 7, 8, 12, 16])
@pytest.mark.parametrize("D", [32, 64, 128, 256])
def test_bf16_group_sizes(n_rep, D):
    run_case(2, 2 * n_rep, 2, D, 128, 64, 20, torch.bfloat16, seed=n_rep + D)


@pytest.mark.parametrize("C,W,fill", [(64, 256, 0), (64, 256, 37), (16, 64, 5), (8, 16, 7), (32, 256, 31)])
def test_bf16_chunk_sizes_and_open_chunk(C, W, fill):
    run_case(3, 8, 2, 128, W, C, 30, torch.bfloat16, seed=C + fill, fill=fill)


@pytest.mark.parametrize("share", [1, 37, 128, 176, 255])
@pytest.mark.parametrize("B,Hkv,chunks", [(4, 8, 40), (1, 2, 3), (3, 1, 300)])
def test_bf16_unequal_shares_of_the_two_halves_of_the_grid(share, B, Hkv, chunks, monkeypatch):
    """The balanced schedule may give the first half of its workgroups another share of the tiles than the second
    (NATS_DECODE_SHARE, in 1/256ths; large launches take 176 by themselves): any share, also the extreme ones that
    leave one half with a single tile per workgroup or none, gives the oracle's result."""
    monkeypatch.setenv("NATS_DECODE_SHARE", str(share))
    run_case(B, 4 * Hkv, Hkv, 128, 256, 64, chunks, torch.bfloat16, seed=share + chunks, frac=(0.02, 1.0), fill=9)


def test_bf16_single_sequence_long_cache():
    run_case(1, 32, 8, 128, 256, 64, 300, torch.bfloat16, seed=9, frac=(0.2, 1.0), fill=13)


def test_bf16_more_streams_than_one_launch_schedules():
    """More than 1024 (batch, kv head) streams: the library takes the batch in groups of whole sequences."""
    run_case(300, 8, 4, 64, 16, 8, 6, torch.bfloat16, seed=21, fill=3)   # 1200 streams: 256 + 44 sequences
    run_case(129, 16, 8, 128, 64, 16, 4, torch.bfloat16, seed=22)       # 1032 streams: 128 + 1 sequences


def test_bf16_nothing_but_the_new_token():
    from neuralattentionsearch_amd import ops
    say("decode: only the new token valid")
    B, Hq, Hkv, D, n_rows = 2, 8, 2, 128, 300
    g = torch.Generator().manual_seed(1)
    k = torch.randn(B, Hkv, 320, D, generator=g).bfloat16()
    v = torch.randn(B, Hkv, 320, D, generator=g).bfloat16()
    valid = torch.zeros(B, Hkv, 320, dtype=torch.bool)
    valid[:, :, n_rows - 1] = True
    q = torch.randn(B, Hq, 1, D, generator=g).bfloat16()
    got = ops.decode_attention(q.cuda(), k.cuda(), v.cuda(), valid.cuda(), n_rows).cpu()
    want = v[:, :, n_rows - 1].repeat_interleave(4, 1).unsqueeze(2)
    assert torch.equal(got, want)


@pytest.mark.parametrize("D", [64, 128])
def test_fp32(D):
    run_case(2, 4, 2, D, 128, 64, 12, torch.float32, seed=D, fill=3)


@pytest.mark.parametrize("D", [16, 32, 256])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_other_head_dims(D, dtype):
    run_case(2, 4, 2, D, 32, 8, 20, dtype, seed=D, fill=3)


@pytest.mark.parametrize("B,Hq,Hkv,chunks,fill,q_scale", [(1, 8, 2, 300, 13, 1.0), (4, 16, 4, 150, 0, 4.0),
                                                           (40, 8, 8, 12, 37, 1.0)])
def test_head_dim_256_on_the_matrix_kernel(B, Hq, Hkv, chunks, fill, q_scale):
    """Rows of 512 bytes: a wavefront's two V tiles take 32 KB of LDS, one workgroup per compute unit.  A single long
    sequence, peaked scores, more streams than workgroups."""
    run_case(B, Hq, Hkv, 256, 256, 64, chunks, torch.bfloat16, seed=B + chunks, frac=(0.1, 1.0), fill=fill, q_scale=q_scale)


def test_strided_cache_views():
    """The cache handed over is a view of a larger capacity buffer, as the cache object does."""
    from neuralattentionsearch_amd import ops
    say("decode strided views")
    k, v, valid, n_rows = ragged_cache(4, 2, 2, 128, 128, 64, 10, torch.bfloat16)
    cap = k.shape[2] + 192
    kb = torch.zeros(2, 2, cap, 128, dtype=torch.bfloat16).cuda()
    vb = torch.zeros_like(kb)
    mb = torch.zeros(2, 2, cap, dtype=torch.bool).cuda()
    kb[:, :, :k.shape[2]] = k.cuda()
    vb[:, :, :k.shape[2]] = v.cuda()
    mb[:, :, :k.shape[2]] = valid.cuda()
    q = torch.randn(2, 8, 1, 128, generator=torch.Generator().manual_seed(5)).bfloat16()
    want = orc.decode_attention(q, k, v, valid, n_rows).float()
    got = ops.decode_attention(q.cuda(), kb[:, :, :n_rows], vb[:, :, :n_rows], mb[:, :, :n_rows], n_rows).cpu().float()
    assert (got - want).abs().max().item() <= 2e-2


def test_cfg3_full_size():
    """batch 32, 32 q / 8 kv heads, D=128, context 65536 with 10-30 % of it kept per (sequence, kv head)."""
    run_case(32, 32, 8, 128, 256, 64, int(0.30 * 65536 / 64), torch.bfloat16, seed=0, frac=(1 / 3, 1.0), fill=17, q_scale=4.0)
