"""A Llama-architecture inference model whose attention layers follow the call order of the reference's
Hugging Face twin, forward_llama_nats_chunk_one_way (src/nats/models/transformer/hf/llama_nats_chunk.py:171-292):

    q / k / v projections -> pooled role logits -> argmax roles -> RoPE -> cache.update -> attention kernel
    -> cache.post_update -> o_proj

The attention itself, the roles and the cache run on the HIP kernels of this package; embeddings, RMSNorm,
the SwiGLU MLP and the projections are plain torch modules (library GEMMs), as they are in the reference.
Differences from BaseNAtSChunkAttentionLayer that this twin has and that are kept: no bias on the global
logit (:206-214 takes the plain maximum) and `position_ids[0, 0] == 0` decides between the prefill kernel
and the cached paths (:194, :238-270).

With `fused_decode` (the default) the same arithmetic takes a shorter route: q / k / v and gate / up are one
projection each over merged weights (the separate `*_proj.weight` parameters are views of them), the residual add
and RMSNorm (and, for the token of an open chunk, the running chunk statistic) are one kernel, the rotary
embedding another (fused with the cache append for a one-token step), the SiLU gate a third; one-token steps run
their projections through the matrix-vector kernel, so that a decoder layer is about a dozen launches.

Weights are random-initialised (there is no checkpoint loader here); `NAtSLlamaConfig.llama3_8b()` gives the
Llama-3-8B shape.
"""
from __future__ import annotations

import math
from dataclasses import dataclass

import torch
from torch import nn

from . import ops
from .attention import apply_rotary_pos_emb
from .cache import ChunkMergeType, NAtSCache


@dataclass
class NAtSLlamaConfig:
    vocab_size: int = 128256
    hidden_size: int = 4096
    intermediate_size: int = 14336
    num_hidden_layers: int = 32
    num_attention_heads: int = 32
    num_key_value_heads: int = 8
    rms_norm_eps: float = 1e-5
    rope_theta: float = 500000.0
    chunk_size: int = 64
    local_seq_max_length: int = 256  # sliding window, in tokens
    chunk_merge_method: str = "mean"
    fused_role_step: bool = False  # pooling + role projection + argmax in one kernel instead of torch ops
    fused_decode: bool = True      # fused norm / rotary / gate kernels and merged projections (one-token steps and segments)

    @property
    def head_dim(self) -> int:
        return self.hidden_size // self.num_attention_heads

    @staticmethod
    def llama3_8b(**kw) -> "NAtSLlamaConfig":
        return NAtSLlamaConfig(**kw)


class RMSNorm(nn.Module):
    def __init__(self, dim: int, eps: float):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(dim))
        self.eps = eps

    def forward(self, x):
        h = x.float()
        h = h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + self.eps)
        return self.weight * h.to(x.dtype)


_plans: dict = {}


def step_linear(x: torch.Tensor, proj, gate: bool = False) -> torch.Tensor:
    """A bias-free projection of a one-token step: the matrix-vector kernel for the few rows it takes, the library
    GEMM otherwise.  `proj` is a weight matrix or an nn.Linear; a module with hooks is called as a module, so that
    whoever registered them still sees its inputs and outputs.  gate=True: `proj` is the stacked gate / up matrix
    and the result is silu(gate) * up."""
    if isinstance(proj, nn.Module):
        if proj._forward_pre_hooks or proj._forward_hooks or proj.bias is not None:
            return proj(x)
        proj = proj.weight
    plan = _plans.get(id(proj))
    if plan is None or plan.weight() is not proj or not plan.current(proj):
        if len(_plans) > 4096:
            _plans.clear()
        plan = _plans[id(proj)] = ops.MatvecPlan(proj, gate)
    if plan.takes(x):
        return plan(x)
    y = nn.functional.linear(x, proj)
    return ops.silu_mul(y) if gate else y


class LlamaMLP(nn.Module):
    def __init__(self, cfg: NAtSLlamaConfig):
        super().__init__()
        self.gate_proj = nn.Linear(cfg.hidden_size, cfg.intermediate_size, bias=False)
        self.up_proj = nn.Linear(cfg.hidden_size, cfg.intermediate_size, bias=False)
        self.down_proj = nn.Linear(cfg.intermediate_size, cfg.hidden_size, bias=False)
        self.gate_up_weight = None

    def fuse(self):
        """gate_proj / up_proj weights become views of one [2 * I, hidden] matrix."""
        w = torch.cat([self.gate_proj.weight.data, self.up_proj.weight.data], dim=0)
        n = self.gate_proj.weight.shape[0]
        self.gate_proj.weight = nn.Parameter(w[:n], requires_grad=False)
        self.up_proj.weight = nn.Parameter(w[n:], requires_grad=False)
        self.gate_up_weight = w

    def fused_ok(self):
        w = self.gate_up_weight
        return w is not None and w.data_ptr() == self.gate_proj.weight.data_ptr() and w.dtype == self.gate_proj.weight.dtype

    def forward(self, x):
        return self.down_proj(nn.functional.silu(self.gate_proj(x)) * self.up_proj(x))

    def forward_fused(self, x):
        if not self.fused_ok():
            self.fuse()
        return step_linear(step_linear(x, self.gate_up_weight, gate=True), self.down_proj)


def rotary_tables(position_ids: torch.Tensor, head_dim: int, theta: float, dtype: torch.dtype):
    """cos / sin [B, L, head_dim], computed in fp32 and cast, the Hugging Face Llama convention."""
    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2, device=position_ids.device, dtype=torch.float32) / head_dim))
    freqs = position_ids[:, :, None].float() * inv[None, None, :]
    emb = torch.cat([freqs, freqs], dim=-1)
    return emb.cos().to(dtype), emb.sin().to(dtype)


class NAtSLlamaAttention(nn.Module):
    """llama_nats_chunk.py:171-292 with the attention, the roles and the cache on the HIP kernels."""

    def __init__(self, cfg: NAtSLlamaConfig, layer_idx: int):
        super().__init__()
        self.layer_idx = layer_idx
        self.hidden_size = cfg.hidden_size
        self.num_heads = cfg.num_attention_heads
        self.num_key_value_heads = cfg.num_key_value_heads
        self.num_key_value_groups = self.num_heads // self.num_key_value_heads
        self.head_dim = cfg.head_dim
        self.chunk_size = cfg.chunk_size
        self.local_seq_max_length = cfg.local_seq_max_length
        if cfg.chunk_merge_method not in ("mean", "max"):
            raise NotImplementedError(cfg.chunk_merge_method)
        self.chunk_merge_method = ChunkMergeType.MEAN if cfg.chunk_merge_method == "mean" else ChunkMergeType.MAX
        self.q_proj = nn.Linear(cfg.hidden_size, self.num_heads * self.head_dim, bias=False)
        self.k_proj = nn.Linear(cfg.hidden_size, self.num_key_value_heads * self.head_dim, bias=False)
        self.v_proj = nn.Linear(cfg.hidden_size, self.num_key_value_heads * self.head_dim, bias=False)
        self.o_proj = nn.Linear(self.num_heads * self.head_dim, cfg.hidden_size, bias=False)
        self.proj_layer = nn.Linear(cfg.hidden_size, self.num_key_value_heads * 3, bias=False)  # :315-318
        # (the fused role step takes chunk sizes that are a power of two; others go through the torch ops)
        self.fused_role_step = cfg.fused_role_step and cfg.chunk_size & (cfg.chunk_size - 1) == 0
        self.qkv_weight = None

    def fuse(self):
        """q_proj / k_proj / v_proj weights become views of one [(H_q + 2 H_kv) * D, hidden] matrix."""
        w = torch.cat([self.q_proj.weight.data, self.k_proj.weight.data, self.v_proj.weight.data], dim=0)
        nq, nk = self.q_proj.weight.shape[0], self.k_proj.weight.shape[0]
        self.q_proj.weight = nn.Parameter(w[:nq], requires_grad=False)
        self.k_proj.weight = nn.Parameter(w[nq:nq + nk], requires_grad=False)
        self.v_proj.weight = nn.Parameter(w[nq + nk:], requires_grad=False)
        self.qkv_weight = w

    def fused_ok(self):
        w = self.qkv_weight
        return w is not None and w.data_ptr() == self.q_proj.weight.data_ptr() and w.dtype == self.q_proj.weight.dtype

    def _decode_one(self, hidden_states, position_embeddings, start_pos: int, past_key_value: NAtSCache,
                    statistic_done: bool):
        """One token over a cache that holds rows: the same steps as `forward`, with one GEMM for q / k / v and the
        rotary embedding fused with the cache append.  `statistic_done`: the caller's norm kernel has already
        merged this token into the running chunk statistic."""
        bsz = hidden_states.shape[0]
        C, idx = self.chunk_size, self.layer_idx
        Hq, Hkv, D = self.num_heads, self.num_key_value_heads, self.head_dim
        if not self.fused_ok():
            self.fuse()
        qkv = step_linear(hidden_states, self.qkv_weight).view(bsz, 1, Hq + 2 * Hkv, D).transpose(1, 2)
        q, k, v = qkv[:, :Hq], qkv[:, Hq:Hq + Hkv], qkv[:, Hq + Hkv:]
        pre_fill = past_key_value.get_nats_chunk_fill_size(idx)
        roles = tsi = None
        if pre_fill + 1 < C:
            if not statistic_done:
                past_key_value.update_nats_cached_x_in_chunk(hidden_states, idx, self.chunk_merge_method)
        elif self.fused_role_step and C == 1 and (dest := past_key_value.cache_model[idx].role_destination(1)) is not None:
            # a per-token cache takes the role straight into its buffer of pending roles; nothing else needs it
            ops.role_step_token(hidden_states, self.proj_layer.weight, self.local_seq_max_length, dest,
                                merge_max=self.chunk_merge_method == ChunkMergeType.MAX, global_bias=0.0,
                                force_first_global=start_pos < C)
            past_key_value._update_cache_x(None, idx)
            roles = dest
        elif self.fused_role_step:
            dest = None
            step = ops.role_step(hidden_states, self.proj_layer.weight, C, self.local_seq_max_length, pre_fill=pre_fill,
                                 carry_in=past_key_value.get_nats_cached_x_in_chunk(idx) if pre_fill else None,
                                 merge_max=self.chunk_merge_method == ChunkMergeType.MAX, global_bias=0.0,
                                 force_first_global=start_pos < C, with_one_hot=dest is None, roles_out=dest)
            past_key_value._update_cache_x(step["carry"], idx)
            roles, tsi = step["roles"], step["token_states_info"]
        else:
            pooled, pad = past_key_value.update_nats_cached_x_across_chunk(hidden_states, pre_fill, idx,
                                                                           self.chunk_merge_method)
            logit = self.proj_layer(pooled).unflatten(-1, (Hkv, 3))
            roles, tsi = ops.roles_from_logits(logit, 0.0, force_first_global=start_pos < C, force_last_global=pad != 0)
        layer = past_key_value.cache_model[idx]
        cos, sin = position_embeddings
        q, keys, values = layer.append_rotated(q, k, v, cos, sin, tsi, roles)
        row_end, tail_start = layer.decode_hint()
        out = ops.decode_attention(q, keys, values, layer.valid_tokens, keys.shape[2], 1.0 / math.sqrt(D),
                                   row_end=row_end, tail_start=tail_start)
        past_key_value.post_update(layer_idx=idx, x_len=1)
        return step_linear(out.transpose(1, 2).reshape(bsz, 1, -1), self.o_proj)

    def forward(self, hidden_states: torch.Tensor, position_embeddings, start_pos: int, past_key_value: NAtSCache,
                fused_decode: bool = False, statistic_done: bool = False, fused_segment: bool = False):
        bsz, q_len, _ = hidden_states.shape
        C, idx = self.chunk_size, self.layer_idx
        if fused_decode:
            return self._decode_one(hidden_states, position_embeddings, start_pos, past_key_value, statistic_done)
        if fused_segment and self.fused_ok():  # one GEMM over the merged matrix; q / k / v are views of its output
            Hq, Hkv, D = self.num_heads, self.num_key_value_heads, self.head_dim
            qkv = nn.functional.linear(hidden_states, self.qkv_weight).view(bsz, q_len, Hq + 2 * Hkv, D).transpose(1, 2)
            q, k, v = qkv[:, :Hq], qkv[:, Hq:Hq + Hkv], qkv[:, Hq + Hkv:]
        else:
            q = self.q_proj(hidden_states).view(bsz, q_len, self.num_heads, self.head_dim).transpose(1, 2)
            k = self.k_proj(hidden_states).view(bsz, q_len, self.num_key_value_heads, self.head_dim).transpose(1, 2)
            v = self.v_proj(hidden_states).view(bsz, q_len, self.num_key_value_heads, self.head_dim).transpose(1, 2)

        pre_fill = past_key_value.get_nats_chunk_fill_size(idx)
        is_pre_filling = start_pos == 0
        if self.fused_role_step:
            step = ops.role_step(hidden_states, self.proj_layer.weight, C, self.local_seq_max_length, pre_fill=pre_fill,
                                 carry_in=past_key_value.get_nats_cached_x_in_chunk(idx) if pre_fill else None,
                                 merge_max=self.chunk_merge_method == ChunkMergeType.MAX, global_bias=0.0,
                                 force_first_global=start_pos < C)
            past_key_value._update_cache_x(step["carry"], idx)
            roles, tsi = step["roles"], step["token_states_info"]
            if roles is None:
                roles = torch.zeros(bsz, self.num_key_value_heads, 1, dtype=torch.uint8, device=hidden_states.device)
                tsi = torch.zeros(bsz, self.num_key_value_heads, 1, 3, dtype=hidden_states.dtype, device=hidden_states.device)
                tsi[..., 0] = 1
        elif pre_fill + q_len < C:
            past_key_value.update_nats_cached_x_in_chunk(hidden_states, idx, self.chunk_merge_method)
            roles = torch.zeros(bsz, self.num_key_value_heads, 1, dtype=torch.uint8, device=hidden_states.device)
            tsi = torch.zeros(bsz, self.num_key_value_heads, 1, 3, dtype=hidden_states.dtype, device=hidden_states.device)
            tsi[..., 0] = 1
        else:
            pooled, pad = past_key_value.update_nats_cached_x_across_chunk(hidden_states, pre_fill, idx,
                                                                           self.chunk_merge_method)
            logit = self.proj_layer(pooled).unflatten(-1, (self.num_key_value_heads, 3))
            roles, tsi = ops.roles_from_logits(logit, 0.0, force_first_global=start_pos < C, force_last_global=pad != 0)

        cos, sin = position_embeddings
        if fused_segment and ops.rope_qk_ok(q, k, cos, sin):
            q, k = ops.rope_qk(q, k, cos, sin)
        else:
            q, k = apply_rotary_pos_emb(q, k, cos, sin)
        keys, values = past_key_value.update(k, v, idx, cache_kwargs={"token_states_info": tsi})
        layer = past_key_value.cache_model[idx]
        scale = 1.0 / math.sqrt(self.head_dim)
        if is_pre_filling:
            # (written as [B, L, H, D], the layout o_proj reads, through the strided view the kernel takes)
            out = torch.empty(bsz, q_len, self.num_heads, self.head_dim, dtype=q.dtype, device=q.device).transpose(1, 2)
            ops.prefill_attention(q, keys, values, roles, C, self.local_seq_max_length, scale, out=out)
        elif q_len > 1:
            out = layer.segment_attention(q, scale)
        else:
            row_end, tail_start = layer.decode_hint()
            out = ops.decode_attention(q, keys, values, layer.valid_tokens, keys.shape[2], scale, row_end=row_end,
                                       tail_start=tail_start)
        past_key_value.post_update(layer_idx=idx, x_len=q_len)
        return self.o_proj(out.transpose(1, 2).reshape(bsz, q_len, -1))


class NAtSLlamaDecoderLayer(nn.Module):
    def __init__(self, cfg: NAtSLlamaConfig, layer_idx: int):
        super().__init__()
        self.self_attn = NAtSLlamaAttention(cfg, layer_idx)
        self.mlp = LlamaMLP(cfg)
        self.input_layernorm = RMSNorm(cfg.hidden_size, cfg.rms_norm_eps)
        self.post_attention_layernorm = RMSNorm(cfg.hidden_size, cfg.rms_norm_eps)

    def forward(self, x, position_embeddings, start_pos: int, cache: NAtSCache):
        x = x + self.self_attn(self.input_layernorm(x), position_embeddings, start_pos, cache)
        return x + self.mlp(self.post_attention_layernorm(x))

    def segment_step(self, x, delta, position_embeddings, start_pos: int, cache: NAtSCache):
        """A multi-token segment with the fused norm, rotary and gate kernels and the merged projections; `x` and
        `delta` as in `decode_step`."""
        h = ops.add_rms_norm(x, delta, self.input_layernorm.weight, self.input_layernorm.eps)
        att = self.self_attn(h, position_embeddings, start_pos, cache, fused_segment=True)
        h = ops.add_rms_norm(x, att, self.post_attention_layernorm.weight, self.post_attention_layernorm.eps)
        return self.mlp.forward_fused(h)

    def decode_step(self, x, delta, position_embeddings, start_pos: int, cache: NAtSCache):
        """One token.  `x` [B, 1, dim] is the residual stream, updated in place; `delta` is the branch output of the
        previous layer that has not been added yet (None for the first layer).  Returns this layer's MLP output,
        to be added by whoever normalises next."""
        attn = self.self_attn
        idx, C = attn.layer_idx, attn.chunk_size
        pre_fill = cache.get_nats_chunk_fill_size(idx)
        carry, mode = None, ops.CARRY_NONE
        if pre_fill + 1 < C:  # the chunk stays open: its running statistic takes this token in (dyn_cache.py:117-124)
            carry = cache.get_nats_cached_x_in_chunk(idx)
            is_max = attn.chunk_merge_method == ChunkMergeType.MAX
            if carry is None:
                carry = torch.empty_like(x)
                mode = ops.CARRY_MAX_FIRST if is_max else ops.CARRY_MEAN_FIRST
            else:
                if carry.shape[1] != 1:  # (max statistic of a first partial chunk: the reference keeps its raw rows)
                    carry = carry.max(1, keepdim=True)[0]
                carry = carry.contiguous()
                mode = ops.CARRY_MAX_MERGE if is_max else ops.CARRY_MEAN_ADD
        h = ops.add_rms_norm(x, delta, self.input_layernorm.weight, self.input_layernorm.eps, carry, mode, C)
        if mode != ops.CARRY_NONE:
            cache._update_cache_x(carry, idx)
        att = attn(h, position_embeddings, start_pos, cache, fused_decode=True, statistic_done=mode != ops.CARRY_NONE)
        h = ops.add_rms_norm(x, att, self.post_attention_layernorm.weight, self.post_attention_layernorm.eps)
        return self.mlp.forward_fused(h)


class NAtSLlamaForCausalLM(nn.Module):
    def __init__(self, cfg: NAtSLlamaConfig):
        super().__init__()
        self.config = cfg
        self.embed_tokens = nn.Embedding(cfg.vocab_size, cfg.hidden_size)
        self.layers = nn.ModuleList([NAtSLlamaDecoderLayer(cfg, i) for i in range(cfg.num_hidden_layers)])
        self.norm = RMSNorm(cfg.hidden_size, cfg.rms_norm_eps)
        self.lm_head = nn.Linear(cfg.hidden_size, cfg.vocab_size, bias=False)

    @staticmethod
    def random_init(cfg: NAtSLlamaConfig, device="cuda", dtype=torch.bfloat16, seed: int = 0, std: float = 0.02):
        """Builds the model on `device` without a host copy of the weights."""
        with torch.device("meta"):
            model = NAtSLlamaForCausalLM(cfg)
        model = model.to_empty(device=device).to(dtype)
        g = torch.Generator(device=device).manual_seed(seed)
        with torch.no_grad():
            for name, p in model.named_parameters():
                if name.endswith("layernorm.weight") or name == "norm.weight":
                    p.fill_(1.0)
                else:
                    p.normal_(0.0, std, generator=g)
        if cfg.fused_decode:
            for layer in model.layers:
                layer.self_attn.fuse()
                layer.mlp.fuse()
        return model.eval()

    def new_cache(self, track_positions: bool = False) -> NAtSCache:
        return NAtSCache(sliding_window_size=self.config.local_seq_max_length, chunk_size=self.config.chunk_size,
                         track_positions=track_positions)

    @torch.no_grad()
    def forward(self, input_ids: torch.Tensor, start_pos: int, cache: NAtSCache, all_logits: bool = False):
        """input_ids [B, L] -> logits of the last position [B, vocab] (or of every position)."""
        bsz, q_len = input_ids.shape
        x = self.embed_tokens(input_ids)
        pos = torch.arange(start_pos, start_pos + q_len, device=input_ids.device)[None].expand(bsz, -1)
        position_embeddings = rotary_tables(pos, self.config.head_dim, self.config.rope_theta, x.dtype)
        fused = self.config.fused_decode and x.shape[-1] <= ops.NORM_MAX_DIM
        if fused and q_len == 1 and start_pos > 0 and len(cache.cache_model) == len(self.layers):
            x = x.contiguous()
            delta = None
            for layer in self.layers:
                delta = layer.decode_step(x, delta, position_embeddings, start_pos, cache)
            return step_linear(ops.add_rms_norm(x, delta, self.norm.weight, self.norm.eps), self.lm_head)[:, 0]
        if fused and q_len > 1:
            x = x.contiguous()
            delta = None
            for layer in self.layers:
                delta = layer.segment_step(x, delta, position_embeddings, start_pos, cache)
            if all_logits:
                return self.lm_head(ops.add_rms_norm(x, delta, self.norm.weight, self.norm.eps))
            last = x[:, -1:].contiguous()
            return step_linear(ops.add_rms_norm(last, delta[:, -1:].contiguous(), self.norm.weight, self.norm.eps),
                               self.lm_head)[:, 0]
        for layer in self.layers:
            x = layer(x, position_embeddings, start_pos, cache)
        x = self.norm(x if all_logits else x[:, -1:])
        logits = self.lm_head(x)
        return logits if all_logits else logits[:, 0]

    @torch.no_grad()
    def generate(self, input_ids: torch.Tensor, max_new_tokens: int, cache: NAtSCache | None = None):
        """Greedy decoding with eviction live.  Returns (new tokens [B, max_new_tokens], cache)."""
        cache = self.new_cache() if cache is None else cache
        start = cache.get_seq_length(0) if len(cache.cache_model) else 0
        logits = self.forward(input_ids, start, cache)
        pos = start + input_ids.shape[1]
        out = []
        for i in range(max_new_tokens):
            tok = logits.argmax(-1, keepdim=True)
            out.append(tok)
            if i + 1 < max_new_tokens:
                logits = self.forward(tok, pos, cache)
                pos += 1
        return torch.cat(out, dim=1) if out else input_ids[:, :0], cache
