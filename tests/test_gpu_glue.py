"""GPU: the decode-step glue kernels (residual add + RMSNorm + running chunk statistic, rotary embedding + cache
append, SiLU gate, matrix-vector products) against the torch ops the reference runs in their place, and the Llama
harness with and without them.

Elementwise arithmetic must agree bit for bit in bf16 (same rounding points); the RMSNorm's mean of squares is
an fp32 reduction in another order, so its rows are compared to one unit in the last place of the dtype."""
import math

import pytest
import torch

from tests.gpu_util import say

pytestmark = pytest.mark.gpu


def torch_rms(x, w, eps):
    h = x.float()
    h = h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + eps)
    return w * h.to(x.dtype)  # models/transformer/components.py:24-26


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("rows,dim", [(1, 4096), (3, 512), (2, 8192), (5, 100)])
def test_add_rms_norm_and_chunk_statistic(dtype, rows, dim):
    from neuralattentionsearch_amd import ops
    say("add_rms_norm", dtype, rows, dim)
    g = torch.Generator().manual_seed(rows * dim)
    x = torch.randn(rows, 1, dim, generator=g).to(dtype).cuda()
    d = torch.randn(rows, 1, dim, generator=g).to(dtype).cuda()
    w = (1 + 0.1 * torch.randn(dim, generator=g)).to(dtype).cuda()
    C = 16
    ulp = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -21
    # plain norm, x untouched
    x0 = x.clone()
    out = ops.add_rms_norm(x0, None, w, 1e-5)
    want = torch_rms(x, w, 1e-5)
    assert torch.equal(x0, x)
    rel = ((out.float() - want.float()).abs() / want.float().abs().clamp_min(1e-3)).max().item()
    assert rel <= ulp, rel
    # residual add (exact) + norm + statistic (exact given the normalised row)
    for mode, carry0 in [(ops.CARRY_MEAN_FIRST, None), (ops.CARRY_MEAN_ADD, torch.randn(rows, 1, dim, generator=g)),
                         (ops.CARRY_MAX_FIRST, None), (ops.CARRY_MAX_MERGE, torch.randn(rows, 1, dim, generator=g))]:
        x1 = x.clone()
        carry = torch.full_like(x, float("nan")) if carry0 is None else carry0.to(dtype).cuda()
        c_in = carry.clone()
        out = ops.add_rms_norm(x1, d, w, 1e-5, carry, mode, C)
        assert torch.equal(x1, x + d)
        want = torch_rms(x + d, w, 1e-5)
        rel = ((out.float() - want.float()).abs() / want.float().abs().clamp_min(1e-3)).max().item()
        assert rel <= ulp, (mode, rel)
        add = (out / C).sum(1, keepdim=True)  # components/cache/dyn_cache.py:101-104
        if mode == ops.CARRY_MEAN_FIRST:
            c_want = add
        elif mode == ops.CARRY_MEAN_ADD:
            c_want = c_in + add
        elif mode == ops.CARRY_MAX_FIRST:
            c_want = out
        else:
            c_want = torch.max(torch.cat([c_in, out], dim=1), dim=1, keepdim=True)[0]
        assert torch.equal(carry, c_want), mode


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_silu_mul(dtype):
    from neuralattentionsearch_amd import ops
    say("silu_mul", dtype)
    g = torch.Generator().manual_seed(5)
    gu = (3 * torch.randn(3, 1, 2 * 1000, generator=g)).to(dtype).cuda()
    got = ops.silu_mul(gu)
    want = torch.nn.functional.silu(gu[..., :1000]) * gu[..., 1000:]
    if dtype == torch.bfloat16:
        # the exponential may differ in its last fp32 bit, which survives the rounding to bf16 only on exact ties
        assert (got != want).float().mean().item() < 1e-3
    ulp = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -21
    assert ((got.float() - want.float()).abs() <= ulp * want.float().abs() + 1e-30).all()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("B,Hq,Hkv,x_len,D", [(2, 8, 2, 1, 64), (1, 32, 8, 1, 128), (2, 4, 4, 5, 32)])
def test_rope_append(dtype, B, Hq, Hkv, x_len, D):
    from neuralattentionsearch_amd import ops
    from neuralattentionsearch_amd.attention import apply_rotary_pos_emb
    from neuralattentionsearch_amd.llama import rotary_tables
    say("rope_append", dtype, B, Hq, Hkv, x_len, D)
    g = torch.Generator().manual_seed(B * Hq + D)
    qkv = torch.randn(B, x_len, (Hq + 2 * Hkv) * D, generator=g).to(dtype).cuda()
    v4 = qkv.view(B, x_len, Hq + 2 * Hkv, D).transpose(1, 2)  # the strided views the harness passes
    q, k, v = v4[:, :Hq], v4[:, Hq:Hq + Hkv], v4[:, Hq + Hkv:]
    pos = torch.arange(37, 37 + x_len, device="cuda")[None].expand(B, -1)
    cos, sin = rotary_tables(pos, D, 500000.0, dtype)
    rows, row0 = 24, 9
    ck = torch.randn(B, Hkv, rows, D, generator=g).to(dtype).cuda()
    cv = torch.randn(B, Hkv, rows, D, generator=g).to(dtype).cuda()
    valid = torch.zeros(B, Hkv, rows, dtype=torch.uint8, device="cuda")
    tp = torch.full((B, Hkv, rows), -1, dtype=torch.int32, device="cuda")
    ck0, cv0 = ck.clone(), cv.clone()
    q_rot = ops.rope_append(q, k, v, cos, sin, ck, cv, valid, tp, row0, 1000)
    q_want, k_want = apply_rotary_pos_emb(q, k, cos, sin)
    assert torch.equal(q_rot, q_want)
    assert torch.equal(ck[:, :, row0:row0 + x_len], k_want)
    assert torch.equal(cv[:, :, row0:row0 + x_len], v)
    keep = torch.ones(rows, dtype=torch.bool)
    keep[row0:row0 + x_len] = False
    assert torch.equal(ck[:, :, keep], ck0[:, :, keep]) and torch.equal(cv[:, :, keep], cv0[:, :, keep])
    assert valid[:, :, ~keep].all() and not valid[:, :, keep].any()
    assert torch.equal(tp[:, :, ~keep], torch.arange(1000, 1000 + x_len, dtype=torch.int32, device="cuda").expand(B, Hkv, -1))
    assert (tp[:, :, keep] == -1).all()
    with pytest.raises(ValueError):
        ops.rope_append(q, k, v, cos, sin, ck, cv, valid, tp, rows - x_len + 1, 0)  # rows past the allocation


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("rows,n_out,k", [(1, 4096, 4096), (1, 1, 64), (2, 7, 520), (3, 8200, 1032), (4, 24, 14336)])
def test_matvec_against_an_fp64_product(dtype, rows, n_out, k):
    """nn.functional.linear for a few rows: fp32 accumulation in another order than the library's, so the result is
    held to the exact product (fp64) within the rounding of the dtype plus the fp32 accumulation error."""
    from neuralattentionsearch_amd import ops
    say("matvec", dtype, rows, n_out, k)
    g = torch.Generator().manual_seed(rows * n_out + k)
    x = torch.randn(rows, 1, k, generator=g).to(dtype).cuda()
    big = (torch.randn(n_out + 3, k + 16, generator=g) / math.sqrt(k)).to(dtype).cuda()
    for w in (big[:n_out, :k].contiguous(), big[2:2 + n_out, 16:16 + k]):  # packed rows, and rows of a wider matrix
        got = ops.matvec(x, w)
        assert got.shape == (rows, 1, n_out) and got.dtype == dtype
        exact = x.double() @ w.double().T
        mag = (x.double().abs() @ w.double().abs().T)
        tol = (2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -23) * exact.abs() + 2.0 ** -20 * mag
        assert ((got.double() - exact).abs() <= tol).all(), ((got.double() - exact).abs() / tol).max().item()
        lib = torch.nn.functional.linear(x, w)
        assert (got.float() - lib.float()).abs().max().item() <= (2.0 ** -6 if dtype == torch.bfloat16 else 1e-5)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("rows,inter,k", [(1, 1000, 512), (3, 14336, 1024), (4, 5, 64)])
def test_matvec_with_the_silu_gate(dtype, rows, inter, k):
    """gate=True equals the SiLU gate kernel applied to the plain product over the stacked matrix, bit for bit: the
    same sums, the same rounding points."""
    from neuralattentionsearch_amd import ops
    say("matvec gate", dtype, rows, inter, k)
    g = torch.Generator().manual_seed(inter + k)
    x = torch.randn(rows, 1, k, generator=g).to(dtype).cuda()
    w = (2 * torch.randn(2 * inter, k, generator=g) / math.sqrt(k)).to(dtype).cuda()
    got = ops.matvec(x, w, gate=True)
    want = ops.silu_mul(ops.matvec(x, w))
    assert got.shape == (rows, 1, inter)
    assert torch.equal(got, want)
    ref = torch.nn.functional.silu(torch.nn.functional.linear(x, w[:inter])) * torch.nn.functional.linear(x, w[inter:])
    scale = max(1.0, ref.float().abs().max().item())
    assert (got.float() - ref.float()).abs().max().item() <= (2.0 ** -6 if dtype == torch.bfloat16 else 1e-5) * scale


def test_matvec_rejects_what_it_does_not_take():
    from neuralattentionsearch_amd import ops
    x = torch.randn(5, 64).bfloat16().cuda()
    w = torch.randn(8, 64).bfloat16().cuda()
    with pytest.raises(ValueError):
        ops.matvec(x, w)  # five rows
    with pytest.raises(ValueError):
        ops.matvec(x[:1, :60].contiguous(), w[:, :60].contiguous())  # k not in 16-byte pieces
    with pytest.raises(ValueError):
        ops.matvec(x[:1].float(), w)  # mixed dtypes
    with pytest.raises(ValueError):
        ops.matvec(x[:1], w[:7], gate=True)  # odd number of rows for gate / up
    assert not ops.matvec_ok(x, w) and ops.matvec_ok(x[:4], w)


@pytest.mark.parametrize("merge", ["mean", "max"])
def test_fused_decode_steps_equal_the_unfused_harness(merge):
    """fp32: both routes run the same arithmetic; only the GEMMs see other shapes, which the seeded logits' gaps absorb."""
    from neuralattentionsearch_amd.llama import NAtSLlamaConfig, NAtSLlamaForCausalLM
    say("llama fused decode", merge)
    kw = dict(vocab_size=777, hidden_size=512, intermediate_size=768, num_hidden_layers=3, num_attention_heads=8,
              num_key_value_heads=4, chunk_size=8, local_seq_max_length=16, chunk_merge_method=merge)
    ids = torch.randint(0, 777, (2, 45), generator=torch.Generator().manual_seed(1)).cuda()
    res = []
    for fused in (False, True):
        model = NAtSLlamaForCausalLM.random_init(NAtSLlamaConfig(fused_decode=fused, **kw), dtype=torch.float32, seed=3,
                                                 std=0.08)
        cache = model.new_cache(track_positions=True)
        logits = model(ids, 0, cache)
        toks, lgs = [], []
        for i in range(40):
            tok = logits.argmax(-1, keepdim=True)
            toks.append(tok)
            logits = model(tok, 45 + i, cache)
            lgs.append(logits)
        res.append((torch.cat(toks, 1), torch.stack(lgs), cache))
    (ta, la, ca), (tb, lb, cb) = res
    assert torch.equal(ta, tb)
    assert (la - lb).abs().max().item() <= 2e-4 * la.abs().max().item()
    for x, y in zip(ca.cache_model, cb.cache_model):
        assert x.n_ctx_data == y.n_ctx_data and x.chunk_fill_size == y.chunk_fill_size
        assert torch.equal(x.valid_tokens, y.valid_tokens)
        assert torch.equal(x.token_positions, y.token_positions)
        assert torch.equal(x.size_global_kv, y.size_global_kv) and torch.equal(x.size_local_kv, y.size_local_kv)
    for x, y in zip(ca.cached_x, cb.cached_x):
        assert (x is None) == (y is None)
        if x is not None:
            assert (x - y).abs().max().item() <= 1e-5


def test_fused_projection_weights_are_views():
    from neuralattentionsearch_amd.llama import NAtSLlamaConfig, NAtSLlamaForCausalLM
    cfg = NAtSLlamaConfig(vocab_size=100, hidden_size=256, intermediate_size=384, num_hidden_layers=1,
                          num_attention_heads=4, num_key_value_heads=2, chunk_size=8, local_seq_max_length=16)
    model = NAtSLlamaForCausalLM.random_init(cfg, dtype=torch.bfloat16)
    a, m = model.layers[0].self_attn, model.layers[0].mlp
    assert a.fused_ok() and m.fused_ok()
    assert torch.equal(a.qkv_weight, torch.cat([a.q_proj.weight, a.k_proj.weight, a.v_proj.weight]))
    with torch.no_grad():
        a.k_proj.weight.fill_(0.5)  # written through the view
    assert (a.qkv_weight[a.q_proj.weight.shape[0]:a.q_proj.weight.shape[0] + a.k_proj.weight.shape[0]] == 0.5).all()
    model = model.float()  # the parameters are re-created: the merged matrix is rebuilt on the next use
    assert not model.layers[0].self_attn.fused_ok()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("B,Hq,Hkv,L,D", [(2, 8, 2, 37, 64), (1, 32, 8, 300, 128), (2, 4, 4, 5, 32)])
def test_rope_qk(dtype, B, Hq, Hkv, L, D):
    """The segment form of the rotary embedding on the strided views of a merged projection: bit for bit what
    apply_rotary_pos_emb computes."""
    from neuralattentionsearch_amd import ops
    from neuralattentionsearch_amd.attention import apply_rotary_pos_emb
    from neuralattentionsearch_amd.llama import rotary_tables
    say("rope_qk", dtype, B, Hq, Hkv, L, D)
    g = torch.Generator().manual_seed(L)
    qkv = torch.randn(B, L, Hq + 2 * Hkv, D, generator=g).to(dtype).cuda().transpose(1, 2)
    q, k = qkv[:, :Hq], qkv[:, Hq:Hq + Hkv]
    pos = torch.arange(11, 11 + L, device="cuda")[None].expand(B, -1)
    cos, sin = rotary_tables(pos, D, 10000.0, dtype)
    assert ops.rope_qk_ok(q, k, cos, sin)
    q_rot, k_rot = ops.rope_qk(q, k, cos, sin)
    q_want, k_want = apply_rotary_pos_emb(q, k, cos, sin)
    assert q_rot.is_contiguous() and k_rot.is_contiguous()
    assert torch.equal(q_rot, q_want) and torch.equal(k_rot, k_want)
