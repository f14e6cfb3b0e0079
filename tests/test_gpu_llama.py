"""GPU: the Llama-architecture harness, layer by layer against the oracle.

Every attention layer of the model is observed through hooks: its input hidden states, its role logits
and the attention output it hands to o_proj.  The oracle side recomputes, per layer, roles -> cache update ->
mask -> attention -> eviction from the same q / k / v and logits and must agree on the attention output, on
the cache bookkeeping after every call and on the roles."""
import math

import numpy as np
import pytest
import torch

from oracle import nats_oracle as orc
from tests.gpu_util import say

pytestmark = pytest.mark.gpu


class LayerProbe:
    def __init__(self, attn):
        self.attn = attn
        self.hidden = self.logits = self.att = None
        attn.register_forward_pre_hook(self._pre)
        attn.proj_layer.register_forward_hook(self._logit)
        attn.o_proj.register_forward_pre_hook(self._att)

    def _pre(self, m, args):
        self.hidden, self.pos_emb, self.start_pos = args[0].detach(), args[1], args[2]
        self.logits = None

    def _logit(self, m, i, o):
        self.logits = o.detach().float().cpu()

    def _att(self, m, args):
        self.att = args[0].detach()


def run(cfg, dtype, lens, tol, B=2, seed=0, std=0.05, need_all_roles=True):
    from neuralattentionsearch_amd.attention import apply_rotary_pos_emb
    from neuralattentionsearch_amd.llama import NAtSLlamaForCausalLM
    model = NAtSLlamaForCausalLM.random_init(cfg, dtype=dtype, seed=seed, std=std)
    with torch.no_grad():
        for layer in model.layers:
            layer.self_attn.proj_layer.weight.mul_(6.0)  # spread the role logits
    probes = [LayerProbe(layer.self_attn) for layer in model.layers]
    cache = model.new_cache()
    C, W = cfg.chunk_size, cfg.local_seq_max_length
    Hq, Hkv, D = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    # (chunk_size == 1 builds the per-token class with its deferred eviction, as the reference's container does)
    states = [orc.TokenCacheOracle(B=B, H=Hkv, W=W) if C == 1 else orc.ChunkCacheOracle(B=B, H=Hkv, W=W, C=C)
              for _ in model.layers]
    fills = [0] * len(model.layers)
    g = torch.Generator().manual_seed(seed)
    seen = 0
    role_counts = np.zeros(3, dtype=np.int64)
    for step, n in enumerate(lens):
        say("llama harness", dtype, "step", step, "tokens", n)
        ids = torch.randint(0, cfg.vocab_size, (B, n), generator=g).cuda()
        logits = model(ids, seen, cache)
        assert logits.shape == (B, cfg.vocab_size) and torch.isfinite(logits).all()
        for li, (pr, st) in enumerate(zip(probes, states)):
            a = pr.attn
            with torch.no_grad():
                q = a.q_proj(pr.hidden).view(B, n, Hq, D).transpose(1, 2)
                k = a.k_proj(pr.hidden).view(B, n, Hkv, D).transpose(1, 2)
                v = a.v_proj(pr.hidden).view(B, n, Hkv, D).transpose(1, 2)
                q, k = apply_rotary_pos_emb(q, k, *pr.pos_emb)
            total = fills[li] + n
            if total < C:
                roles = np.zeros((B, Hkv, 1), dtype=np.uint8)
                assert pr.logits is None
                fills[li] = total
            else:
                lg = pr.logits.unflatten(-1, (Hkv, 3)).to(dtype)
                roles = orc.roles_from_logits(lg, 0.0, force_first_global=seen < C, force_last_global=total % C != 0)
                assert roles.shape[-1] == math.ceil(total / C)
                fills[li] = total % C
                role_counts += np.bincount(roles.ravel(), minlength=3)
            ko, vo = st.update(k.cpu(), v.cpu(), roles)
            if seen == 0:
                att = orc.masked_attention(q.cpu().float(), ko.float(), vo.float(), orc.prefill_mask(roles, n, C, W))
            elif n > 1:
                att = orc.masked_attention(q.cpu().float(), ko.float(), vo.float(), st.generate_mask(n))
            else:
                att = orc.decode_attention(q.cpu(), ko, vo, torch.from_numpy(st.valid), st.n_ctx_data + 1).float()
            st.post_update(n)
            got = pr.att.float().cpu().view(B, n, Hq, D).transpose(1, 2)
            err = (got - att).abs().max().item()
            assert err <= tol, (step, li, err)
            lc = cache.cache_model[li]
            assert lc.n_ctx_data == st.n_ctx_data, (step, li)
            assert np.array_equal(lc.valid_tokens.cpu().numpy(), st.valid), (step, li)
            assert np.array_equal(lc.size_global_kv.cpu().numpy(), st.size_global), (step, li)
            assert np.array_equal(lc.size_local_kv.cpu().numpy(), st.size_local), (step, li)
        seen += n
    if need_all_roles:
        assert (role_counts > 0).all(), role_counts  # the run exercised all three roles
    return model, cache


def test_small_fp32_model_layer_by_layer():
    from neuralattentionsearch_amd.llama import NAtSLlamaConfig
    cfg = NAtSLlamaConfig(vocab_size=1000, hidden_size=512, intermediate_size=1024, num_hidden_layers=3,
                          num_attention_heads=8, num_key_value_heads=2, chunk_size=16, local_seq_max_length=32)
    run(cfg, torch.float32, [100, 37] + [1] * 40 + [50, 1, 1], tol=2e-5)


def test_per_token_roles_layer_by_layer():
    """chunk_size == 1: a role per token (the per-token adapters of the reference), the per-token cache class."""
    from neuralattentionsearch_amd.llama import NAtSLlamaConfig
    cfg = NAtSLlamaConfig(vocab_size=1000, hidden_size=512, intermediate_size=1024, num_hidden_layers=2,
                          num_attention_heads=8, num_key_value_heads=2, chunk_size=1, local_seq_max_length=16)
    run(cfg, torch.float32, [60, 21] + [1] * 24, tol=2e-5)


def test_max_statistic_after_a_short_first_segment():
    """chunk_merge_method "max": a first segment shorter than a chunk leaves its raw rows as the running statistic
    (dyn_cache.py:111-112); the one-token steps and segments after it must take that form in."""
    from neuralattentionsearch_amd.llama import NAtSLlamaConfig
    cfg = NAtSLlamaConfig(vocab_size=1000, hidden_size=512, intermediate_size=1024, num_hidden_layers=2,
                          num_attention_heads=8, num_key_value_heads=2, chunk_size=8, local_seq_max_length=16,
                          chunk_merge_method="max")
    run(cfg, torch.float32, [3, 1, 1, 2] + [1] * 20 + [19, 1, 1, 30, 1], tol=2e-5, seed=2)


def test_llama_head_shape_bf16_layer_by_layer():
    """32 q heads / 8 kv heads / head_dim 128, chunk 64, window 256, two layers."""
    from neuralattentionsearch_amd.llama import NAtSLlamaConfig
    cfg = NAtSLlamaConfig(vocab_size=512, hidden_size=4096, intermediate_size=1024, num_hidden_layers=2,
                          chunk_size=64, local_seq_max_length=256)
    run(cfg, torch.bfloat16, [1500, 200] + [1] * 70, tol=2e-2, B=1, std=4096 ** -0.5)  # q, k, v of unit scale


def test_generate_is_deterministic_and_matches_stepwise_forward():
    from neuralattentionsearch_amd.llama import NAtSLlamaConfig, NAtSLlamaForCausalLM
    say("llama generate")
    cfg = NAtSLlamaConfig(vocab_size=777, hidden_size=512, intermediate_size=512, num_hidden_layers=2,
                          num_attention_heads=8, num_key_value_heads=4, chunk_size=8, local_seq_max_length=16)
    model = NAtSLlamaForCausalLM.random_init(cfg, dtype=torch.float32, seed=3, std=0.08)
    ids = torch.randint(0, 777, (2, 45), generator=torch.Generator().manual_seed(1)).cuda()
    a, cache_a = model.generate(ids, 30)
    b, _ = model.generate(ids, 30)
    assert torch.equal(a, b) and a.shape == (2, 30)
    cache = model.new_cache()
    logits = model(ids, 0, cache)
    toks = []
    for i in range(30):
        tok = logits.argmax(-1, keepdim=True)
        toks.append(tok)
        logits = model(tok, 45 + i, cache)
    assert torch.equal(torch.cat(toks, 1), a)
    # eviction was live: the cache holds fewer rows than tokens seen for at least one layer
    assert cache_a.get_seq_length(0) == 45 + 29
    assert min(l.n_ctx_data for l in cache_a.cache_model) < 45 + 29 + 16


@pytest.mark.parametrize("method,prompt", [("mean", 45), ("max", 45), ("max", 3), ("mean", 3)])
def test_fused_role_step_gives_the_same_generation(method, prompt):
    """The harness with the fused role-step kernel against the same model with torch pooling + projection (fp32:
    the two differ in summation order only, which the seeded logits' gaps absorb)."""
    from neuralattentionsearch_amd.llama import NAtSLlamaConfig, NAtSLlamaForCausalLM
    say("llama fused role step", method, prompt)
    kw = dict(vocab_size=777, hidden_size=512, intermediate_size=512, num_hidden_layers=2, num_attention_heads=8,
              num_key_value_heads=4, chunk_size=8, local_seq_max_length=16, chunk_merge_method=method)
    ids = torch.randint(0, 777, (2, prompt), generator=torch.Generator().manual_seed(1)).cuda()
    outs, kept = [], []
    for fused in (False, True):
        model = NAtSLlamaForCausalLM.random_init(NAtSLlamaConfig(fused_role_step=fused, **kw), dtype=torch.float32, seed=3, std=0.08)
        toks, cache = model.generate(ids, 30)
        outs.append(toks)
        kept.append([l.valid_tokens.sum().item() for l in cache.cache_model])
    assert torch.equal(outs[0], outs[1])
    assert kept[0] == kept[1]


@pytest.mark.parametrize("C,W", [(8, 16), (1, 32)])
def test_a_transformers_llama_with_patched_attention_layers(C, W):
    """The way the reference is used (models/transformer/hf/llama_nats_chunk.py patches the attention layers of a
    Hugging Face Llama, the callers pass a NAtSCache as past_key_values): a transformers LlamaForCausalLM whose
    attention layers forward to this package's attention module, with the container as its cache, gives the logits
    of the package's own model with the same weights, for a prompt, a later multi-token segment and one-token steps."""
    pytest.importorskip("transformers")
    from transformers import LlamaConfig, LlamaForCausalLM
    from transformers.models.llama import modeling_llama
    from neuralattentionsearch_amd.llama import NAtSLlamaConfig, NAtSLlamaForCausalLM
    say("transformers llama with patched attention", C, W)
    dims = dict(vocab_size=300, hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
                num_key_value_heads=2)
    torch.manual_seed(3)
    hf = LlamaForCausalLM(LlamaConfig(max_position_embeddings=2048, rms_norm_eps=1e-6, attention_bias=False,
                                      mlp_bias=False, tie_word_embeddings=False, **dims)).cuda().float().eval()
    cfg = NAtSLlamaConfig(rms_norm_eps=1e-6, rope_theta=10000.0, chunk_size=C, local_seq_max_length=W, **dims)
    ours = NAtSLlamaForCausalLM(cfg).cuda().float().eval()
    state = {k.removeprefix("model."): v for k, v in hf.state_dict().items()}
    res = ours.load_state_dict(state, strict=False)
    assert not res.unexpected_keys and all(k.endswith("proj_layer.weight") for k in res.missing_keys), res
    with torch.no_grad():
        for layer in ours.layers:  # the role projection has no counterpart in the plain model
            layer.self_attn.proj_layer.weight.normal_(0.0, 0.5)

    def nats_forward(self, hidden_states, position_embeddings=None, attention_mask=None, past_key_values=None, **kwargs):
        start = past_key_values.get_seq_length(self.layer_idx)
        return ours.layers[self.layer_idx].self_attn(hidden_states, position_embeddings, start, past_key_values), None

    g = torch.Generator().manual_seed(11)
    lens = [5 * max(C, 8) + 3, 2 * max(C, 8) + 1] + [1] * (2 * max(C, 16) + 2)
    ids = [torch.randint(0, 300, (2, n), generator=g).cuda() for n in lens]
    cache_hf, cache_own = ours.new_cache(), ours.new_cache()
    original = modeling_llama.LlamaAttention.forward
    modeling_llama.LlamaAttention.forward = nats_forward
    try:
        pos = 0
        with torch.no_grad():
            for i, x in enumerate(ids):
                got = hf(input_ids=x, past_key_values=cache_hf, use_cache=True).logits
                want = ours(x, pos, cache_own, all_logits=True).reshape(got.shape)
                err = (got.float() - want.float()).abs().max().item()
                assert err <= 2e-4, (i, x.shape, err)
                pos += x.shape[1]
    finally:
        modeling_llama.LlamaAttention.forward = original
    assert cache_hf.get_seq_length() == pos == cache_own.get_seq_length()
    for a, b in zip(cache_hf.cache_model, cache_own.cache_model):
        assert a.n_ctx_data == b.n_ctx_data and torch.equal(a.valid_tokens, b.valid_tokens)


def test_full_size_llama3_8b_shape_prefill_16384_and_512_steps():
    """The end-to-end workload at its full size (32 layers, d_model 4096, 32 / 8 heads, FFN 14336, vocabulary 128256,
    bf16; 16384 prompt tokens, 512 greedy steps with eviction live), where no oracle run is affordable: properties
    that hold at any size.  Finite logits; the same tokens from a second run; the same tokens with the role step as
    torch ops instead of the fused kernel (roles are the argmax of logits that differ in summation order only; the
    comparison allows the few near-ties of 8 heads x 33 layers x 260 chunks to flip, by bounding how the kept rows
    differ rather than demanding equal tokens); and in every layer the valid rows are exactly the rows the sizes
    describe: ring slots flagged valid + global rows + local rows + the open chunk."""
    from neuralattentionsearch_amd.llama import NAtSLlamaConfig, NAtSLlamaForCausalLM
    say("llama full size: init")
    cfg = NAtSLlamaConfig.llama3_8b(fused_role_step=True)
    model = NAtSLlamaForCausalLM.random_init(cfg, seed=0)
    W, C, H = cfg.local_seq_max_length, cfg.chunk_size, cfg.num_key_value_heads
    prompt, steps = 16384, 512
    ids = torch.randint(0, cfg.vocab_size, (1, prompt), generator=torch.Generator().manual_seed(0)).cuda()

    def check_layers(cache, seen):
        for li, lc in enumerate(cache.cache_model):
            assert lc.get_seq_length() == seen
            n = lc.n_ctx_data
            valid = lc.valid_tokens[:, :, :n]
            rows = lc.size_global_kv - W + lc.size_local_kv  # [B, H]
            want = rows.sum().item() + valid[:, :, :W].sum().item() + lc.chunk_fill_size * H
            assert valid.sum().item() == want, (li, valid.sum().item(), want)
            assert n == int((lc.size_global_kv + lc.size_local_kv).max()) + lc.chunk_fill_size, li
            assert (lc.size_global_kv % C == 0).all() and (lc.size_local_kv % C == 0).all() and (lc.size_local_kv >= 0).all()
            # a head's own rows are valid, the rows between its end and the open chunk are not
            per_head = valid[:, :, W:n - lc.chunk_fill_size].sum(-1)
            assert torch.equal(per_head, rows), li

    say("llama full size: run 1")
    toks_a, cache_a = model.generate(ids, steps)
    assert toks_a.shape == (1, steps)
    logits = model(toks_a[:, -1:], prompt + steps - 1, cache_a)
    assert torch.isfinite(logits).all() and logits.shape == (1, cfg.vocab_size)
    check_layers(cache_a, prompt + steps)
    kept_a = [int(lc.valid_tokens[:, :, :lc.n_ctx_data].sum()) for lc in cache_a.cache_model]
    assert max(kept_a) < H * (prompt + steps), "nothing was evicted"
    del cache_a
    say("llama full size: run 2 (same tokens)")
    toks_b, cache_b = model.generate(ids, steps)
    assert torch.equal(toks_a, toks_b)
    del cache_b
    say("llama full size: role step as torch ops")
    for layer in model.layers:
        layer.self_attn.fused_role_step = False
    toks_c, cache_c = model.generate(ids, steps)
    check_layers(cache_c, prompt + steps - 1)
    kept_c = [int(lc.valid_tokens[:, :, :lc.n_ctx_data].sum()) for lc in cache_c.cache_model]
    agree = (toks_a == toks_c).float().mean().item()
    say("llama full size: token agreement fused / unfused role step", agree, "kept", sum(kept_a), sum(kept_c))
    # layer 0 sees the same hidden states in both runs: its roles agree except at near-ties of bf16 logits
    assert abs(kept_a[0] - kept_c[0]) <= 0.02 * kept_c[0] + 2 * C * H, (kept_a[0], kept_c[0])
