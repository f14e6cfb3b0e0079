"""Attention modules of the NAtS inference path on top of the HIP kernels.

Same class names, constructor arguments and method names as the reference's modules
(src/nats/models/transformer/attention/base_attention.py:11-283, nats_attention.py:14-195,
nats_chunk_attention.py:19-157); inference only (the training branch and its Triton backward kernels are
outside this build).  Differences a caller can see:

* keys / values are never repeated to H_q heads: the kernels read the kv heads directly (``repeat_kv_values``
  returns its arguments);
* no [B, H, L, N] mask is built: ``multi_head_attention`` calls the prefill kernel for a multi-token segment
  (over an empty cache, or over the rows earlier segments left) and the decode kernel for one token;
  ``cache.generate_mask`` stays available for inspection.
"""
from __future__ import annotations

import math

import torch
from torch import nn

from . import ops
from .cache import ChunkMergeType, NAtSCache


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    x1, x2 = x[..., : x.shape[-1] // 2], x[..., x.shape[-1] // 2:]
    return torch.cat((-x2, x1), dim=-1)


def apply_rotary_pos_emb(q, k, cos, sin, unsqueeze_dim: int = 1):
    """q * cos + rotate_half(q) * sin, the HF Llama convention the reference imports
    (base_attention.py:8, 147-151); cos / sin are [B, L, D]."""
    cos = cos.unsqueeze(unsqueeze_dim)
    sin = sin.unsqueeze(unsqueeze_dim)
    return (q * cos) + (rotate_half(q) * sin), (k * cos) + (rotate_half(k) * sin)


class AttentionLayer(nn.Module):
    """Projections and head bookkeeping (base_attention.py:13-137)."""

    def __init__(self, dim: int = 4096, n_heads: int = 32, n_kv_heads: int | None = None, layer_id: int = 0,
                 dropout: float = 0.0, use_flash: bool = True, on_ddp: bool = False):
        super().__init__()
        self.n_kv_heads = n_heads if n_kv_heads is None else n_kv_heads
        self.layer_id = layer_id
        self.n_local_heads = n_heads
        self.n_local_kv_heads = self.n_kv_heads
        self.n_rep = self.n_local_heads // self.n_local_kv_heads
        self.head_dim = dim // n_heads
        self.wq = nn.Linear(dim, n_heads * self.head_dim, bias=False)
        self.wk = nn.Linear(dim, self.n_kv_heads * self.head_dim, bias=False)
        self.wv = nn.Linear(dim, self.n_kv_heads * self.head_dim, bias=False)
        self.wo = nn.Linear(n_heads * self.head_dim, dim, bias=False)
        self.use_flash = use_flash
        self._use_flash = use_flash
        self.dropout = dropout

    def add_rotary_emb(self, xq, xk, pos_emb):
        if pos_emb is not None:
            cos, sin = pos_emb
            xq, xk = apply_rotary_pos_emb(xq, xk, cos, sin)
        return xq, xk

    def repeat_kv_values(self, keys, values):
        return keys, values

    def forward(self, x: torch.Tensor, pos_emb, mask, start_pos: int = 0, cache: NAtSCache | None = None, **kwargs):
        """[B, L, dim] -> [B, L, dim] (base_attention.py:259-283)."""
        if self.training:
            raise NotImplementedError("only the inference path is built; call module.eval()")
        bsz, seqlen, _ = x.shape
        xq, xk, xv, mha_kwargs = self.prepare_x_values(x, bsz=bsz, seqlen=seqlen, pos_emb=pos_emb, start_pos=start_pos,
                                                       cache=cache)
        keys, values = self.prepare_kv(xq, xk, xv, start_pos, cache=cache, kwargs=mha_kwargs)
        keys, values = self.repeat_kv_values(keys, values)
        output = self.multi_head_attention(xq, keys, values, mask=mask, cache=cache, kwargs=mha_kwargs)
        output = output.transpose(1, 2).reshape(bsz, seqlen, -1)
        return self.wo(output)


class BaseNAtSAttentionLayer(AttentionLayer):
    """Role logits and the cache hand-over (nats_attention.py:14-134)."""

    def __init__(self, dim: int = 4096, n_heads: int = 32, n_kv_heads: int | None = None, layer_id: int = 0,
                 dropout: float = 0.0, use_flash: bool = True, on_ddp: bool = False, n_msks: int | None = None,
                 sparse_regularized_value: float = 0.0, local_seq_max_length: int = 4, n_options: int = 3,
                 global_token_enhanced_value: float = 0.1):
        super().__init__(dim, n_heads, n_kv_heads, layer_id, dropout, use_flash, on_ddp)
        if n_msks is None:
            n_msks = n_kv_heads or n_heads
        if n_options != 3:
            raise ValueError("the kernels implement the three roles global / local / sliding window")
        if n_msks != self.n_kv_heads:
            raise NotImplementedError("one role stream per kv head is supported (n_msks == n_kv_heads)")
        self.proj_layer = nn.Linear(dim, n_msks * n_options, bias=False)
        self.n_msks = n_msks
        self.n_options = n_options
        self.n_rep_msk = n_heads // n_msks
        self.sm_scale = 1 / math.sqrt(self.head_dim)
        self.sparse_regularized_value = sparse_regularized_value
        self.local_seq_max_length = local_seq_max_length
        self.global_token_enhanced_value = global_token_enhanced_value
        one_hot_values = torch.zeros(n_options)
        one_hot_values[0] = 1.0
        self.one_hot_values = one_hot_values
        self.executor = None
        self._cache_is_till_updating = None

    def prepare_x_values(self, x, bsz: int, seqlen: int, pos_emb, start_pos: int = 0, cache: NAtSCache | None = None):
        xq, xk, xv = self.wq(x), self.wk(x), self.wv(x)
        xq = xq.view(bsz, seqlen, self.n_local_heads, self.head_dim).transpose(1, 2)
        xk = xk.view(bsz, seqlen, self.n_local_kv_heads, self.head_dim).transpose(1, 2)
        xv = xv.view(bsz, seqlen, self.n_local_kv_heads, self.head_dim).transpose(1, 2)
        token_states_info = self._sample_for_token_info_values_inference(x, start_pos=start_pos, cache=cache)
        xq, xk = self.add_rotary_emb(xq, xk, pos_emb)
        return xq, xk, xv, {"token_states_info": token_states_info}

    def role_logits(self, x_pooled: torch.Tensor) -> torch.Tensor:
        """[B, S, dim] -> [B, S, H_kv, 3]"""
        return self.proj_layer(x_pooled).unflatten(-1, (self.n_msks, self.n_options))

    def _sample_for_token_info_values_inference(self, x, start_pos, cache: NAtSCache | None = None,
                                                sink_token_end: int = 1, force_last_global: bool = False):
        """nats_attention.py:96-109 on the roles kernel: bias on option 0, first maximum, sink slot global."""
        logit = self.role_logits(x)
        _, one_hot = ops.roles_from_logits(logit, self.global_token_enhanced_value,
                                           force_first_global=start_pos < sink_token_end,
                                           force_last_global=force_last_global)
        return one_hot

    def prepare_kv(self, xq, xk, xv, start_pos: int = 0, cache: NAtSCache | None = None, kwargs: dict | None = None):
        if self._cache_is_till_updating is not None:  # nats_attention.py:122-123
            self._cache_is_till_updating.result()
            self._cache_is_till_updating = None
        return cache.update(key_states=xk, value_states=xv, layer_idx=self.layer_id, cache_kwargs=kwargs)

    def _post_update(self, cache: NAtSCache, x_len: int):
        """Eviction after the attention (nats_attention.py:189-195).  With an executor the job is handed to its
        thread together with the caller's stream: torch's current stream is a per-thread setting, and the eviction
        kernels must follow the attention kernel on the stream that ran it."""
        if self.executor is None:
            cache.post_update(layer_idx=self.layer_id, x_len=x_len)
            return
        stream = torch.cuda.current_stream()

        def job():
            with torch.cuda.stream(stream):
                cache.post_update(layer_idx=self.layer_id, x_len=x_len)

        self._cache_is_till_updating = self.executor.submit(job)

    def multi_head_attention(self, xq, keys, values, mask=None, cache: NAtSCache | None = None,
                             is_first_module: bool = True, kwargs: dict | None = None):
        """Inference branch of nats_attention.py:136-195 / nats_chunk_attention.py:97-157 on the kernels: the mask
        the reference takes from cache.generate_mask is evaluated inside them, from the cache's own window."""
        assert "token_states_info" in kwargs, "Token States Infor is required for multi head attention!"
        x_len = xq.shape[-2]
        layer = cache.cache_model[self.layer_id]
        if x_len == 1 and layer.get_seq_length() > 0:
            row_end, tail_start = layer.decode_hint()
            output = ops.decode_attention(xq, keys, values, layer.valid_tokens, keys.shape[2], self.sm_scale,
                                          row_end=row_end, tail_start=tail_start)
        elif layer.get_seq_length() == 0:
            roles = ops.roles_from_one_hot(kwargs["token_states_info"])
            output = ops.prefill_attention(xq, keys, values, roles, layer.chunk_size, layer.sliding_window_size,
                                           self.sm_scale)
        else:
            output = layer.segment_attention(xq, self.sm_scale)
        self._post_update(cache, x_len)
        return output



class BaseNAtSChunkAttentionLayer(BaseNAtSAttentionLayer):
    """Chunk-granular roles (nats_chunk_attention.py:19-157)."""

    def __init__(self, dim: int = 4096, n_heads: int = 32, n_kv_heads: int | None = None, layer_id: int = 0,
                 dropout: float = 0.0, use_flash: bool = True, on_ddp: bool = False, n_msks: int | None = None,
                 sparse_regularized_value: float = 0.0, local_seq_max_length: int = 4, n_options: int = 3,
                 chunk_size: int = 8, chunk_merge_method: str = "mean", compress_on_q: bool = False):
        super().__init__(dim, n_heads, n_kv_heads, layer_id, dropout, use_flash, on_ddp, n_msks,
                         sparse_regularized_value, local_seq_max_length, n_options)
        if chunk_merge_method == "mean":
            self.chunk_merge_method = ChunkMergeType.MEAN
        elif chunk_merge_method == "max":
            self.chunk_merge_method = ChunkMergeType.MAX
        else:
            raise ValueError(f"Unknown chunk merge method: {chunk_merge_method}")
        self.chunk_size = chunk_size
        self.compress_on_q = compress_on_q

    def get_pad_size(self, x_len):
        return (-x_len) % self.chunk_size

    def _sample_for_token_info_values_inference(self, x, start_pos, cache: NAtSCache | None = None):
        """nats_chunk_attention.py:64-95: while the open chunk is not complete the hidden states are only
        accumulated and a global placeholder role is handed on; otherwise one role per chunk touched, from the
        pooled hidden states, with the open last chunk forced global."""
        x_len = x.shape[1]
        pre_fill = cache.get_nats_chunk_fill_size(self.layer_id)
        if pre_fill + x_len < self.chunk_size:
            cache.update_nats_cached_x_in_chunk(x, self.layer_id, self.chunk_merge_method)
            return self.one_hot_values.to(x).reshape(1, 1, 1, -1).expand(x.shape[0], self.n_kv_heads, 1, -1)
        x_pooled, pad_size = cache.update_nats_cached_x_across_chunk(x, pre_fill, self.layer_id, self.chunk_merge_method)
        return super()._sample_for_token_info_values_inference(x_pooled, start_pos, sink_token_end=self.chunk_size,
                                                               force_last_global=pad_size != 0)



class GPTNAtSAttentionLayer(BaseNAtSAttentionLayer):
    """Per-token roles (chunk_size == 1), nats_attention.py:198-199."""


class LlamaNAtSAttentionLayer(BaseNAtSAttentionLayer):
    """Per-token roles (chunk_size == 1), nats_attention.py:202-203."""


class GPTNAtSChunkAttentionLayer(BaseNAtSChunkAttentionLayer):
    pass


class LlamaNAtSChunkAttentionLayer(BaseNAtSChunkAttentionLayer):
    pass
