"""GPU parity of the prefill kernels against the oracle's mask + torch attention."""
import math

import numpy as np
import pytest
import torch

from oracle import nats_oracle as orc
from tests.gpu_util import draw_roles, say, to_dev

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2}


def run_case(B, Hq, Hkv, L, D, C, W, dtype, seed=0, p=(0.2, 0.3, 0.5), scale_inputs=1.0):
    from neuralattentionsearch_amd import ops
    say("prefill", B, Hq, Hkv, L, D, C, W, dtype, seed)
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(B, Hq, L, D, generator=g) * scale_inputs).to(dtype)
    k = (torch.randn(B, Hkv, L, D, generator=g) * scale_inputs).to(dtype)
    v = (torch.randn(B, Hkv, L, D, generator=g) * scale_inputs).to(dtype)
    S = -(-L // C)
    roles = draw_roles(seed + 1, B, Hkv, S, p=p)
    mask = orc.prefill_mask(roles, L, C, W)
    want = orc.masked_attention(q.float(), k.float(), v.float(), mask)
    got = ops.prefill_attention(q.cuda(), k.cuda(), v.cuda(), to_dev(roles), C, W).cpu().float()
    err = (got - want).abs().max().item()
    assert math.isfinite(err) and err <= TOL[dtype], f"max abs err {err}"
    return err


def test_cfg1_fp32_plumbing_shape():
    # B=1, 8 q/kv heads, L=2048, D=64, fp32, chunk 64, window 128
    run_case(1, 8, 8, 2048, 64, 64, 128, torch.float32)


@pytest.mark.parametrize("L,C,W,D", [(507, 8, 16, 64), (300, 32, 64, 128), (130, 1, 4, 64), (640, 128, 256, 128)])
def test_fp32_ragged_lengths_and_chunk_sizes(L, C, W, D):
    run_case(2, 4, 2, L, D, C, W, torch.float32, seed=L)


@pytest.mark.parametrize("n_rep", [1, 2, 3, 4, 6, 7, 8, 12])
def test_bf16_gqa_group_sizes(n_rep):
    run_case(1, 2 * n_rep, 2, 1024, 128, 64, 256, torch.bfloat16, seed=n_rep)
    run_case(1, 2 * n_rep, 2, 1100, 128, 16, 64, torch.bfloat16, seed=n_rep)  # packed tiles


@pytest.mark.parametrize("L,C,W,D", [(1000, 64, 256, 128), (777, 32, 64, 128), (512, 16, 64, 64), (2048, 64, 128, 64),
                                     (1536, 128, 256, 128), (200, 8, 16, 128), (63, 64, 64, 128), (65, 64, 64, 128),
                                     (900, 1, 64, 128), (333, 2, 8, 64)])  # per-token roles (chunk size 1) included
def test_bf16_shapes(L, C, W, D):
    run_case(2, 8, 2, L, D, C, W, torch.bfloat16, seed=L + C)


@pytest.mark.parametrize("L,C,W,D,dtype", [(700, 3, 12, 128, torch.bfloat16), (900, 6, 24, 64, torch.bfloat16),
                                           (1000, 12, 36, 128, torch.bfloat16), (1300, 24, 48, 128, torch.bfloat16),
                                           (1500, 48, 96, 128, torch.bfloat16), (2000, 96, 192, 128, torch.bfloat16),
                                           (500, 6, 12, 64, torch.float32), (700, 96, 96, 128, torch.float32)])
def test_chunk_sizes_that_are_no_power_of_two(L, C, W, D, dtype):
    """The reference's cache only asks for W % C == 0 (nats_chunk_layer_cache.py:47): chunks that straddle 16-row
    granules and 64-row tiles.  The golden scenarios with chunk sizes 3, 6 and 12 cover the cache side."""
    run_case(2, 8, 2, L, D, C, W, dtype, seed=L + C)


@pytest.mark.parametrize("Hq,Hkv,L,C,W", [(8, 2, 1000, 64, 128), (8, 2, 777, 32, 64), (4, 4, 900, 16, 32), (4, 2, 650, 1, 16),
                                          (8, 2, 2100, 128, 256)])
def test_head_dim_32_on_the_matrix_kernels(Hq, Hkv, L, C, W):
    """Rows of 64 bytes: a tile is four transfers (wavefronts 0-3 issue one each), one score MFMA step per 16 dims."""
    run_case(2, Hq, Hkv, L, 32, C, W, torch.bfloat16, seed=L + 32)


@pytest.mark.parametrize("Hq,Hkv,L,C,W", [(8, 2, 1000, 64, 128), (8, 1, 777, 32, 64), (4, 4, 900, 16, 32), (4, 2, 650, 1, 16),
                                          (6, 2, 2100, 128, 256), (2, 2, 31, 8, 8), (16, 8, 4100, 64, 256), (3, 1, 129, 3, 6)])
def test_head_dim_256_on_the_matrix_kernel(Hq, Hkv, L, C, W):
    """Rows of 512 bytes: four wavefronts per workgroup, one per SIMD, two K and two V tile buffers; groups of 1, 2, 3
    and 8 q heads, chunks shorter than a tile masked row by row, lengths that end inside a block of 32 rows."""
    run_case(2, Hq, Hkv, L, 256, C, W, torch.bfloat16, seed=L + 256)


@pytest.mark.parametrize("D", [16, 32, 256])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_other_head_dims(D, dtype):
    """The other head dims the reference's kernel accepts (models/transformer/triton/nats_flashattn_fwd.py:634): the
    plain kernel in fp32 and at 16, the matrix kernels in bf16 at 32 and 256."""
    run_case(2, 4, 2, 333, D, 8, 16, dtype, seed=D)
    run_case(1, 2, 2, 200, D, 64, 128, dtype, seed=D + 1)


def test_bf16_llama_head_shape_8_streams():
    # 32 q / 8 kv heads as in Llama-3-8B: exercises the XCD-aware workgroup mapping (B * H_kv % 8 == 0)
    run_case(1, 32, 8, 2048, 128, 64, 256, torch.bfloat16, seed=5, p=(0.05, 0.15, 0.8), scale_inputs=1 / math.sqrt(128) ** 0.5)


def test_bf16_all_global_equals_causal_attention():
    from neuralattentionsearch_amd import ops
    say("prefill all-global == causal")
    g = torch.Generator().manual_seed(3)
    B, Hq, Hkv, L, D = 1, 8, 2, 1024, 128
    q = torch.randn(B, Hq, L, D, generator=g).bfloat16()
    k = torch.randn(B, Hkv, L, D, generator=g).bfloat16()
    v = torch.randn(B, Hkv, L, D, generator=g).bfloat16()
    roles = np.zeros((B, Hkv, L // 64), dtype=np.uint8)
    got = ops.prefill_attention(q.cuda(), k.cuda(), v.cuda(), to_dev(roles), 64, 256).cpu().float()
    want = torch.nn.functional.scaled_dot_product_attention(
        q.float(), k.float().repeat_interleave(4, 1), v.float().repeat_interleave(4, 1), is_causal=True)
    assert (got - want).abs().max().item() <= 2e-2


def test_strided_inputs_and_drop_in_signature():
    """q/k/v as transposed views of [B, L, H, D] projections and the reference's nats_prefill signature."""
    from neuralattentionsearch_amd import ops
    say("prefill strided + nats_prefill signature")
    g = torch.Generator().manual_seed(11)
    B, Hq, Hkv, L, D, C, W = 1, 8, 2, 768, 128, 64, 128
    q = torch.randn(B, L, Hq, D, generator=g).bfloat16()
    k = torch.randn(B, L, Hkv, D, generator=g).bfloat16()
    v = torch.randn(B, L, Hkv, D, generator=g).bfloat16()
    roles = draw_roles(12, B, Hkv, L // C)
    tsi = orc.one_hot_roles(roles)
    flags = tsi[..., 0].clone()
    flags[..., -1] = 1.0
    end_idx = torch.from_numpy(orc.next_global_index(flags.numpy() > 0))
    mask = orc.prefill_mask(roles, L, C, W)
    want = orc.masked_attention(q.transpose(1, 2).float(), k.transpose(1, 2).float(), v.transpose(1, 2).float(), mask)
    o, m = ops.nats_prefill(q.cuda().transpose(1, 2), k.cuda().transpose(1, 2), v.cuda().transpose(1, 2),
                            end_idx.cuda(), tsi[..., 2].cuda(), 1 / math.sqrt(D), nats_chunk_size=C, n_rep=Hq // Hkv,
                            local_seq_max_length=W, return_masks=True)
    assert (o.cpu().float() - want).abs().max().item() <= 2e-2
    assert np.array_equal(m.cpu().numpy(), mask)


def check_sampled_rows(B, Hq, Hkv, L, D, C, W, n_samples=96, p=(0.05, 0.15, 0.8)):
    """A run too large for the oracle's dense mask, checked on sampled query rows against a direct per-row
    evaluation of the mask predicate.  Scores are peaked (standard deviation 4 nats), so a row's output is carried by
    a few keys and is of the size of v: a dropped tile, granule or key shows, and the error is held against the
    row's own magnitude."""
    from neuralattentionsearch_amd import ops
    g = torch.Generator().manual_seed(0)
    q = (torch.randn(B, Hq, L, D, generator=g) * 2.0).bfloat16()
    k = (torch.randn(B, Hkv, L, D, generator=g) * 2.0).bfloat16()
    v = torch.randn(B, Hkv, L, D, generator=g).bfloat16()
    S = -(-L // C)
    roles = draw_roles(1, B, Hkv, S, p=p)
    if L % C:
        roles[:, :, -1] = 0
    out = ops.prefill_attention(q.cuda(), k.cuda(), v.cuda(), to_dev(roles), C, W).cpu().float()
    assert torch.isfinite(out).all()
    gidx = orc.next_global_index(roles == 0)
    rng = np.random.default_rng(7)
    worst, smallest = 0.0, float("inf")
    for i in range(n_samples):
        hq = int(rng.integers(Hq))
        m = int(rng.integers(L)) if i % 4 else L - 1 - int(rng.integers(64))
        hkv = hq // (Hq // Hkv)
        mc = m // C
        n = np.arange(m + 1)
        nc = n // C
        r = roles[0, hkv, nc]
        vis = np.where(r == 0, True, np.where(r == 2, (mc - nc) <= W // C, gidx[0, hkv, nc] >= mc))
        vis |= nc == S - 1
        idx = torch.from_numpy(n[vis])
        s = (q[0, hq, m].float() @ k[0, hkv, idx].float().T) / math.sqrt(D)
        want = torch.softmax(s, -1) @ v[0, hkv, idx].float()
        rms = want.pow(2).mean().sqrt().item()
        err = (out[0, hq, m] - want).abs().max().item()
        assert err <= 2e-2 * rms + 2e-3, (hq, m, err, rms)
        worst, smallest = max(worst, err), min(smallest, rms)
    assert smallest > 0.05, smallest  # the rows checked are far from zero


def test_cfg2_full_size_sampled_rows():
    """L = 32768, Llama-3-8B head shape, chunk 64."""
    say("prefill cfg2 full size")
    check_sampled_rows(1, 32, 8, 32768, 128, 64, 256)


@pytest.mark.parametrize("Hq,Hkv,L,C,W", [(32, 8, 32768, 32, 256),   # the chunk size of the reference's Llama adapter
                                          (4, 1, 70016, 16, 64),      # 4376 granules: two windows of the tile list
                                          (8, 2, 40000, 8, 16)])      # chunks shorter than a granule
def test_packed_tiles_full_size_sampled_rows(Hq, Hkv, L, C, W):
    """Chunks shorter than a 64-row tile: the kernel packs tiles from visible 16-row granules."""
    say("prefill packed, sampled rows", Hq, Hkv, L, C, W)
    check_sampled_rows(1, Hq, Hkv, L, 128, C, W, n_samples=64)


@pytest.fixture
def split_lists(monkeypatch):
    def switch(on: bool):
        monkeypatch.setenv("NATS_PREFILL_SPLIT", "1" if on else "0")
    yield switch
    monkeypatch.delenv("NATS_PREFILL_SPLIT", raising=False)


@pytest.mark.parametrize("C,W,lens", [(64, 256, (6000, 64, 200, 1, 700)), (16, 64, (5000, 100, 33, 900)),
                                      (64, 128, (40000, 128))])
def test_short_segments_over_a_long_cache_split_their_tile_lists(split_lists, C, W, lens):
    """Few query tiles over many key rows: several workgroups share one tile list and a merge kernel combines their
    partial results.  Same outputs as one workgroup per list, to rounding."""
    from neuralattentionsearch_amd import ops
    from neuralattentionsearch_amd.cache import NAtSChunkLayerCache
    say("prefill split lists", C, W, lens)
    B, Hq, Hkv, D = 1, 8, 2, 128
    outs = []
    for on in (False, True):
        split_lists(on)
        gg = torch.Generator().manual_seed(11)
        cache = NAtSChunkLayerCache(B, Hkv, W, chunk_size=C, device="cuda")
        res = []
        for si, n in enumerate(lens):
            q = torch.randn(B, Hq, n, D, generator=gg).bfloat16().cuda()
            k = torch.randn(B, Hkv, n, D, generator=gg).bfloat16().cuda()
            v = torch.randn(B, Hkv, n, D, generator=gg).bfloat16().cuda()
            total = cache.chunk_fill_size + n
            first = cache.get_seq_length() == 0
            if total < C:
                roles = np.zeros((B, Hkv, 1), dtype=np.uint8)
            else:
                roles = draw_roles(si, B, Hkv, math.ceil(total / C), p=(0.3, 0.3, 0.4), first_global=first)
                if total % C:
                    roles[:, :, -1] = 0
            tsi = orc.one_hot_roles(roles).bfloat16().cuda()
            kk, vv = cache.update(k, v, tsi)
            if first:
                o = ops.prefill_attention(q, kk, vv, to_dev(roles), C, W)
            elif n > 1:
                o = cache.segment_attention(q)
            else:
                o = ops.decode_attention(q, kk, vv, cache.valid_tokens, kk.shape[2])
            res.append(o.float())
            cache.post_update(n)
        outs.append(res)
    for x, y in zip(*outs):
        assert torch.isfinite(y).all()
        assert (x - y).abs().max().item() <= 2e-2


@pytest.fixture
def packed_tiles(monkeypatch):
    def switch(on: bool):
        monkeypatch.setenv("NATS_PREFILL_PACKED", "1" if on else "0")
    yield switch
    monkeypatch.delenv("NATS_PREFILL_PACKED", raising=False)


@pytest.mark.parametrize("B,Hq,Hkv,L,D,C,W,p", [
    (1, 32, 8, 2048, 128, 32, 256, (0.05, 0.15, 0.8)),
    (2, 8, 2, 1000, 128, 16, 64, (0.2, 0.3, 0.5)),     # ragged last query tile and last granule
    (1, 16, 2, 777, 128, 8, 16, (0.2, 0.3, 0.5)),      # GQA group of 8, chunks of half a granule
    (2, 8, 2, 2048, 64, 32, 128, (0.1, 0.1, 0.8)),     # head_dim 64
    (1, 8, 2, 3000, 128, 1, 64, (0.1, 0.2, 0.7)),      # per-token roles
    (1, 8, 2, 1500, 128, 16, 64, (0.0, 0.0, 1.0)),     # sliding window only
    (1, 8, 2, 1500, 128, 16, 64, (1.0, 0.0, 0.0)),     # dense: every granule is visible
    (2, 4, 4, 1500, 128, 32, 128, (0.1, 0.2, 0.7)),    # one q head per kv head: four query tiles per workgroup
    (1, 8, 4, 2000, 64, 8, 16, (0.1, 0.2, 0.7)),       # groups of 2, head_dim 64
])
def test_packed_tiles_agree_with_whole_tiles(packed_tiles, B, Hq, Hkv, L, D, C, W, p):
    """The same scores reach the softmax in another order: the two kernels agree to rounding."""
    from neuralattentionsearch_amd import ops
    say("prefill packed vs whole tiles", B, Hq, Hkv, L, D, C, W, p)
    g = torch.Generator().manual_seed(L + C)
    q = torch.randn(B, Hq, L, D, generator=g).bfloat16().cuda()
    k = torch.randn(B, Hkv, L, D, generator=g).bfloat16().cuda()
    v = torch.randn(B, Hkv, L, D, generator=g).bfloat16().cuda()
    roles = draw_roles(L, B, Hkv, -(-L // C), p=p)
    if L % C:
        roles[:, :, -1] = 0
    roles = to_dev(roles)
    packed_tiles(False)
    whole = ops.prefill_attention(q, k, v, roles, C, W).float()
    packed_tiles(True)
    packed = ops.prefill_attention(q, k, v, roles, C, W).float()
    assert torch.isfinite(packed).all()
    assert (packed - whole).abs().max().item() <= 2e-2


def test_packed_tiles_on_segments_over_a_filled_cache(packed_tiles):
    """Rows an earlier segment left in the cache (ring, kept globals and locals, stale rows) as granules."""
    from neuralattentionsearch_amd import ops
    from neuralattentionsearch_amd.cache import NAtSChunkLayerCache
    say("prefill packed, segments over a filled cache")
    B, Hq, Hkv, D, C, W = 1, 8, 2, 128, 16, 64
    outs = []
    for on in (False, True):
        packed_tiles(on)
        gg = torch.Generator().manual_seed(3)
        cache = NAtSChunkLayerCache(B, Hkv, W, chunk_size=C, device="cuda")
        res = []
        for n, seed in ((700, 1), (333, 2), (150, 3), (1000, 4)):
            q = torch.randn(B, Hq, n, D, generator=gg).bfloat16().cuda()
            k = torch.randn(B, Hkv, n, D, generator=gg).bfloat16().cuda()
            v = torch.randn(B, Hkv, n, D, generator=gg).bfloat16().cuda()
            S = math.ceil((cache.chunk_fill_size + n) / C)
            roles = draw_roles(seed, B, Hkv, S, p=(0.2, 0.3, 0.5))
            if (cache.chunk_fill_size + n) % C:
                roles[:, :, -1] = 0
            tsi = orc.one_hot_roles(roles).bfloat16().cuda()
            first = cache.get_seq_length() == 0
            kk, vv = cache.update(k, v, tsi)
            res.append((ops.prefill_attention(q, kk, vv, to_dev(roles), C, W) if first else cache.segment_attention(q)).float())
            cache.post_update(n)
        outs.append(res)
    for x, y in zip(*outs):
        assert torch.isfinite(y).all()
        assert (x - y).abs().max().item() <= 2e-2


# ---- chunks shorter than a granule: rows far behind a query come from the lists of long-lived rows ----------------
@pytest.fixture
def far_rows(monkeypatch):
    def switch(on: bool):
        monkeypatch.setenv("NATS_PREFILL_FAR", "1" if on else "0")
    yield switch
    monkeypatch.delenv("NATS_PREFILL_FAR", raising=False)


@pytest.mark.parametrize("Hq,Hkv,L,C,W,p", [
    (32, 8, 32768, 1, 256, (0.05, 0.15, 0.8)),     # the headline shape with a role per token
    (4, 1, 70016, 1, 64, (0.97, 0.02, 0.01)),      # 1060 tiles of long-lived rows: two windows of gathered tiles
    (8, 2, 40000, 4, 32, (0.004, 0.5, 0.496)),     # long runs of local tokens: long-lived rows with finite limits
    (4, 4, 20000, 2, 16, (0.05, 0.15, 0.8)),       # one q head per kv head: four query tiles share the gathered tiles
])
def test_long_lived_rows_full_size_sampled_rows(Hq, Hkv, L, C, W, p):
    say("prefill gathered rows, sampled rows", Hq, Hkv, L, C, W, p)
    check_sampled_rows(1, Hq, Hkv, L, 128, C, W, n_samples=64, p=p)


@pytest.mark.parametrize("B,Hq,Hkv,L,D,C,W,p", [
    (2, 8, 2, 1500, 128, 1, 4, (0.1, 0.3, 0.6)),
    (1, 8, 2, 1100, 64, 2, 8, (0.05, 0.5, 0.45)),
    (1, 4, 2, 900, 128, 8, 16, (0.2, 0.3, 0.5)),    # groups of 2
    (1, 2, 2, 700, 128, 4, 8, (0.3, 0.3, 0.4)),     # groups of 1
    (1, 8, 2, 1300, 128, 1, 16, (0.0, 0.0, 1.0)),   # no long-lived row but the first
    (1, 8, 2, 1300, 128, 1, 16, (1.0, 0.0, 0.0)),   # every row is long-lived
])
def test_long_lived_rows_against_the_oracle(B, Hq, Hkv, L, D, C, W, p):
    """Small windows, so that most of every query's keys come through the gathered tiles."""
    run_case(B, Hq, Hkv, L, D, C, W, torch.bfloat16, seed=L, p=p)


@pytest.mark.parametrize("L", [1, 2, 15, 16, 17, 31, 63, 64, 65, 129])
@pytest.mark.parametrize("C,W", [(1, 1), (1, 4), (2, 4), (8, 8), (3, 6)])
def test_short_sequences_with_short_chunks(L, C, W):
    """Fewer rows than a granule, a tile, and a few more: the lists of long-lived rows of one or two tiles."""
    run_case(1, 4, 1, L, 64, C, W, torch.bfloat16, seed=L * 7 + C, p=(0.3, 0.3, 0.4))


def test_gathered_rows_agree_with_the_granule_walk(far_rows):
    """The same keys reach the softmax in another order, on a first prefill and on segments over a per-token cache
    (cache rows below the open chunk: ring, kept rows, pending tokens)."""
    from neuralattentionsearch_amd import ops
    from neuralattentionsearch_amd.cache import NAtSLayerCache
    say("prefill gathered rows vs granule walk")
    B, Hq, Hkv, D, W = 1, 8, 2, 128, 32
    outs = []
    for on in (False, True):
        far_rows(on)
        gg = torch.Generator().manual_seed(5)
        cache = NAtSLayerCache(B, Hkv, W, device="cuda")
        res = []
        for n, seed in ((3000, 1), (700, 2), (45, 3), (1200, 4)):
            q = torch.randn(B, Hq, n, D, generator=gg).bfloat16().cuda()
            k = torch.randn(B, Hkv, n, D, generator=gg).bfloat16().cuda()
            v = torch.randn(B, Hkv, n, D, generator=gg).bfloat16().cuda()
            first = cache.get_seq_length() == 0
            roles = draw_roles(seed, B, Hkv, n, p=(0.1, 0.2, 0.7), first_global=first)
            tsi = orc.one_hot_roles(roles).bfloat16().cuda()
            kk, vv = cache.update(k, v, tsi)
            res.append((ops.prefill_attention(q, kk, vv, to_dev(roles), 1, W) if first else cache.segment_attention(q)).float())
            cache.post_update(n)
        outs.append(res)
    for x, y in zip(*outs):
        assert torch.isfinite(y).all()
        assert (x - y).abs().max().item() <= 2e-2


# ---- running maxima that keep rising: the rescaling branch of every variant ------------------------------------
def rising_inputs(B, Hq, Hkv, L, D, step_rows, step_nats, seed):
    """q, k, v whose scores grow by `step_nats` every `step_rows` keys (a common direction u: q carries sqrt(D) u,
    key n carries (n // step_rows) * step_nats * u), on top of unit noise.  Every later block of keys beats the
    running maximum of the earlier ones by more than the slack within which the kernels leave it alone, so their
    accumulators are rescaled with 0 < alpha < 1 again and again."""
    g = torch.Generator().manual_seed(seed)
    u = torch.nn.functional.normalize(torch.randn(D, generator=g), dim=0)
    q = torch.randn(B, Hq, L, D, generator=g) * 0.5 + math.sqrt(D) * u
    level = (torch.arange(L) // step_rows).float() * step_nats
    k = torch.randn(B, Hkv, L, D, generator=g) * 0.5 + level[None, None, :, None] * u
    v = torch.randn(B, Hkv, L, D, generator=g)
    return q.bfloat16(), k.bfloat16(), v.bfloat16()


def check_rising(B, Hq, Hkv, L, D, C, W, p, step_rows=48, step_nats=7.0, seed=0):
    from neuralattentionsearch_amd import ops
    q, k, v = rising_inputs(B, Hq, Hkv, L, D, step_rows, step_nats, seed)
    roles = draw_roles(seed + 1, B, Hkv, -(-L // C), p=p)
    if L % C:
        roles[:, :, -1] = 0
    want = orc.masked_attention(q.float(), k.float(), v.float(), orc.prefill_mask(roles, L, C, W))
    got = ops.prefill_attention(q.cuda(), k.cuda(), v.cuda(), to_dev(roles), C, W).cpu().float()
    assert torch.isfinite(got).all()
    rms = want.pow(2).mean(-1, keepdim=True).sqrt()
    bad = ((got - want).abs() > 2e-2 * torch.maximum(rms, want.abs()) + 2e-3)
    assert not bad.any(), (int(bad.sum()), (got - want).abs().max().item())


@pytest.mark.parametrize("Hq,Hkv,L,D,C,W,p", [
    (8, 2, 1500, 128, 64, 256, (1.0, 0.0, 0.0)),   # whole tiles, dense
    (8, 2, 1500, 128, 64, 128, (0.2, 0.3, 0.5)),   # whole tiles, mixed roles
    (8, 2, 1300, 64, 64, 128, (0.3, 0.3, 0.4)),    # head_dim 64
    (8, 2, 1500, 128, 16, 64, (0.3, 0.3, 0.4)),    # packed tiles
    (4, 4, 1200, 128, 64, 128, (0.3, 0.3, 0.4)),   # one q head per kv head (packed form, four query tiles a workgroup)
    (4, 2, 1200, 128, 8, 32, (0.3, 0.3, 0.4)),     # groups of two
    (6, 2, 900, 128, 64, 128, (0.4, 0.3, 0.3)),    # a group of three: the per-wavefront form
    (8, 2, 4500, 128, 64, 256, (1.0, 0.0, 0.0)),   # dense and long: lists of up to 71 tiles
    (8, 2, 1500, 256, 64, 256, (1.0, 0.0, 0.0)),   # head_dim 256 (its own kernel), dense
    (4, 2, 1300, 256, 16, 64, (0.3, 0.3, 0.4)),    # head_dim 256, short chunks, groups of two
])
def test_rising_scores_rescale_the_accumulators(Hq, Hkv, L, D, C, W, p):
    say("prefill rising scores", Hq, Hkv, L, D, C, W, p)
    check_rising(1, Hq, Hkv, L, D, C, W, p)


def test_rising_scores_in_split_lists_and_the_decode_kernel(split_lists):
    """A short segment over a long cache (several workgroups share a tile list, partial results merged) and one-token
    steps over the same rows (split over workgroups, merged): both with scores that rise along the rows."""
    from neuralattentionsearch_amd import ops
    from neuralattentionsearch_amd.cache import NAtSChunkLayerCache
    say("prefill split lists + decode, rising scores")
    split_lists(True)
    B, Hq, Hkv, D, C, W = 1, 8, 2, 128, 64, 256
    n1, n2 = 6016, 64
    q, k, v = rising_inputs(B, Hq, Hkv, n1 + n2 + 1, D, 40, 6.0, seed=5)
    roles1 = np.zeros((B, Hkv, n1 // C), dtype=np.uint8)  # all global: every row stays in the cache
    roles2 = np.zeros((B, Hkv, 1), dtype=np.uint8)
    cache = NAtSChunkLayerCache(B, Hkv, W, chunk_size=C, device="cuda")
    st = orc.ChunkCacheOracle(B=B, H=Hkv, W=W, C=C)
    for roles, lo, hi in ((roles1, 0, n1), (roles2, n1, n1 + n2), (roles2, n1 + n2, n1 + n2 + 1)):
        n = hi - lo
        ko, vo = st.update(k[:, :, lo:hi], v[:, :, lo:hi], roles)
        kk, vv = cache.update(k[:, :, lo:hi].cuda(), v[:, :, lo:hi].cuda(), orc.one_hot_roles(roles).bfloat16().cuda())
        if lo:
            qq = q[:, :, lo:hi]
            if n > 1:
                want = orc.masked_attention(qq.float(), ko.float(), vo.float(), st.generate_mask(n))
                got = cache.segment_attention(qq.cuda())
            else:
                want = orc.decode_attention(qq, ko, vo, torch.from_numpy(st.valid), st.n_ctx_data + 1).float()
                got = ops.decode_attention(qq.cuda(), kk, vv, cache.valid_tokens, kk.shape[2])
            got = got.float().cpu()
            rms = want.pow(2).mean(-1, keepdim=True).sqrt()
            assert not ((got - want).abs() > 2e-2 * torch.maximum(rms, want.abs()) + 2e-3).any(), (n, (got - want).abs().max().item())
        st.post_update(n)
        cache.post_update(n)


@pytest.fixture
def pooled_groups(monkeypatch):
    def switch(eighths: int | None):
        if eighths is None:
            monkeypatch.delenv("NATS_PREFILL_POOL", raising=False)
        else:
            monkeypatch.setenv("NATS_PREFILL_POOL", str(eighths))
    yield switch
    monkeypatch.delenv("NATS_PREFILL_POOL", raising=False)


@pytest.mark.parametrize("B,Hq,Hkv,L,C,W", [(1, 32, 8, 32768, 64, 256),   # cfg2: eight streams, one per XCD
                                            (1, 24, 6, 12000, 64, 128),    # streams that do not fill the XCDs evenly
                                            (1, 8, 8, 20000, 32, 128),     # packed tiles, four query tiles per workgroup
                                            (1, 64, 8, 6000, 64, 128),     # GQA groups of 8: two head groups per kv head
                                            (2, 32, 8, 9000, 64, 256),     # sixteen streams: two per XCD queue
                                            (3, 16, 8, 7000, 16, 64),      # 24 streams, packed tiles, groups of 2
                                            (1, 16, 8, 4096, 64, 256)])    # too few workgroups: nothing is pooled
def test_pooled_query_groups_change_nothing(pooled_groups, B, Hq, Hkv, L, C, W):
    """Large launches deal their lightest query groups from a counter.  Who computes a query group does not change
    what is computed: the output is the same, bit for bit, with the pool switched off, at another pool size, and on a
    second launch (the counter starts from zero every time)."""
    from neuralattentionsearch_amd import ops
    say("prefill pooled query groups", B, Hq, Hkv, L, C, W)
    D = 128
    g = torch.Generator(device="cuda").manual_seed(3)
    q = (torch.randn(B, Hq, L, D, generator=g, device="cuda") * 2.0).bfloat16()
    k = (torch.randn(B, Hkv, L, D, generator=g, device="cuda") * 2.0).bfloat16()
    v = torch.randn(B, Hkv, L, D, generator=g, device="cuda").bfloat16()
    roles = to_dev(draw_roles(5, B, Hkv, -(-L // C), p=(0.05, 0.15, 0.8)))
    outs = []
    for eighths in (0, None, None, 5, 8):
        pooled_groups(eighths)
        outs.append(ops.prefill_attention(q, k, v, roles, C, W))
    assert torch.isfinite(outs[0].float()).all()
    for o in outs[1:]:
        assert torch.equal(o, outs[0])


def test_two_prefills_on_two_streams_equal_the_serial_results():
    """Scratch buffers are kept per stream: launches that run side by side on two streams do not share key limits."""
    from neuralattentionsearch_amd import ops
    say("prefill on two streams at once")
    B, Hq, Hkv, D, C, W = 1, 8, 2, 128, 64, 128
    cases = []
    for i, L in enumerate((6000, 4100)):
        g = torch.Generator().manual_seed(20 + i)
        q = (torch.randn(B, Hq, L, D, generator=g) * 2).bfloat16().cuda()
        k = (torch.randn(B, Hkv, L, D, generator=g) * 2).bfloat16().cuda()
        v = torch.randn(B, Hkv, L, D, generator=g).bfloat16().cuda()
        roles = to_dev(draw_roles(30 + i, B, Hkv, -(-L // C), p=(0.3, 0.3, 0.4)))
        cases.append((q, k, v, roles))
    serial = [ops.prefill_attention(q, k, v, r, C, W) for q, k, v, r in cases]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    for rep in range(3):
        outs = []
        for st, (q, k, v, r) in zip(streams, cases):
            st.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(st):
                for _ in range(4):  # several launches each, so that the two streams overlap
                    o = ops.prefill_attention(q, k, v, r, C, W)
                outs.append(o)
        for st in streams:
            st.synchronize()
        for o, want in zip(outs, serial):
            assert torch.equal(o, want), rep

