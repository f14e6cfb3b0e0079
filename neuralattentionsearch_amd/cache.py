"""KV-cache objects of the NAtS inference path, backed by the HIP eviction / compaction kernels.

Same class names, constructor arguments, methods and observable attributes as the reference's
``NAtSCache`` (src/nats/components/cache/dyn_cache.py:66-195) and ``NAtSChunkLayerCache``
(src/nats/components/cache/nats_chunk_layer_cache.py:15-906), so the attention modules and the HF
monkey-patches can use them unchanged.  What differs is how the state is kept:

* rows live in a capacity buffer that grows geometrically; ``cache_k`` / ``cache_v`` / ``valid_tokens`` are
  views of the logical rows, whose number equals the reference's ``cache_k.shape[2]`` at every step;
* the first prefill is not copied into ``[W zeros | K | pad]``: the raw K / V handed to ``update`` are kept
  until ``post_update`` gathers the surviving rows straight into a right-sized cache;
* ``post_update`` issues two kernels (plan, apply) instead of the reference's gather / scatter ops with six
  device-to-host synchronisations; the plan kernel leaves its 64-byte result (new n_ctx_data, minimum global size)
  in pinned host memory as well, and the host picks it up when it next needs those numbers (the next update of that
  layer, an attribute read), without a stream synchronisation.
"""
from __future__ import annotations

import math
from enum import Enum
from typing import Any

import torch

from . import ops


class ChunkMergeType(Enum):
    """src/nats/chunk_utils.py:65-67"""
    MEAN = 0
    MAX = 1


def get_pad_size(x_len: int, chunk_size: int) -> int:
    """src/nats/chunk_utils.py:9-10"""
    return (-x_len) % chunk_size


def pool_chunks(x: torch.Tensor, chunk_size: int, pad_size: int, method: ChunkMergeType) -> torch.Tensor:
    """[B, L, dim] -> [B, ceil(L / C), dim]: per-chunk mean (zero padded, divided by C) or max
    (src/nats/chunk_utils.py:13-62)."""
    if pad_size:
        x = torch.nn.functional.pad(x, (0, 0, 0, pad_size))
    x = x.unflatten(-2, (-1, chunk_size))
    return x.mean(-2) if method == ChunkMergeType.MEAN else x.max(-2)[0]


class NAtSChunkLayerCache:
    """One layer's cache with chunk-granular roles.  Row layout of cache_k[b, h] between forward calls:

        [0, W)                        ring of the last W tokens of completed chunks (zero rows unless sliding window)
        [W, size_global)              global chunks, stream order
        [size_global, +size_local)    local chunks newer than the last global chunk
        [.., max over heads)          stale rows of shorter heads (valid_tokens == False)
        [base, base + chunk_fill)     the open chunk, same offset for every head
        [n_ctx_data, ..)              zeros
    """

    def __init__(self, bsz: int, n_msks: int, sliding_window_size: int, layer_id: int = 0, chunk_size: int = 16,
                 device: torch.device | str = "cuda", track_positions: bool = False):
        device = torch.device(device)
        if device.type != "cuda":
            raise ValueError("NAtSChunkLayerCache keeps its state on the GPU; pass a cuda device")
        if sliding_window_size % chunk_size != 0:  # nats_chunk_layer_cache.py:47
            raise ValueError("sliding_window_size must be a multiple of chunk_size")
        self.layer_id = layer_id
        self.bsz = bsz
        self.n_msks = n_msks
        self.chunk_size = chunk_size
        self.sliding_window_size = sliding_window_size
        self.n_chunks_per_sw = sliding_window_size // chunk_size
        self.device = device
        self.track_positions = track_positions
        # (the two size tensors are halves of one, so that a reset is one small copy)
        self._sizes = torch.empty(2, bsz, n_msks, device=device, dtype=torch.long)
        self._sizes_init = torch.zeros(2, bsz, n_msks, device=device, dtype=torch.long)
        self._sizes_init[0] = sliding_window_size
        self._sizes_stale = True  # the tensors do not hold the empty cache's sizes yet (written when someone needs them)
        self._row_end = None  # size_global_kv + size_local_kv, kept between evictions
        self._evict = None    # ops.EvictBuffers, made by the first eviction
        self._await = None    # (sequence number, first) of an eviction whose scalars the host has not picked up yet
        self._redo = None     # what a first eviction launched on a guessed capacity needs if the guess was too small
        self._kept_share = None  # logical rows after the last first eviction / rows of the uncompacted cache
        self._append_call = None  # ops.CacheAppendCall / ops.EvictInplaceCall prepared for the present buffers
        self._inplace_call = None
        self._inplace_params = None
        self._planned = None  # (sequence number, roles, facts) of an eviction whose plan rode with the append of its rows
        self.reset_cache()

    # -- state ----------------------------------------------------------------------------------
    # size_global_kv / size_local_kv [B, H] int64 (nats_chunk_layer_cache.py:60-66).  A reset does not write them: the
    # eviction of a first prefill knows what an empty cache holds and writes the new sizes itself; whoever else wants
    # them first (a read of the attributes, an eviction that is not the first) has them written then.
    def _fresh_sizes(self):
        self._resolve()  # (a first eviction still on its way may turn out to have left the sizes alone)
        if self._sizes_stale:
            self._sizes_stale = False
            torch.add(self._sizes_init, 0, out=self._sizes)  # (a kernel; a tensor copy would go through the runtime's copy path)
        return self._sizes

    @property
    def size_global_kv(self):
        return self._fresh_sizes()[0]

    @property
    def size_local_kv(self):
        return self._fresh_sizes()[1]

    def reset_cache(self):
        self._await = self._redo = None  # (a result still on its way belongs to the state that is dropped here)
        self._sizes_stale = True
        self._row_end = None
        self.sliding_queue_tail = 0
        self.chunk_fill_size = 0
        self.chunk_fill_size_last = 0
        self._n_ctx = self.sliding_window_size
        self._gmin = self.sliding_window_size
        self._seen_tokens = 0
        self._tokens_info = None
        self._roles = None
        self._buf_k = self._buf_v = self._buf_valid = self._buf_pos = None
        self._append_call = self._inplace_call = None  # (they hold the buffers)
        self._planned = None
        self._uninit = False  # the buffers came from torch.empty and only the eviction kernel has written them
        self._clean = None    # if set: buffer rows from this one on hold nothing yet, not even zeros
        self._n_rows = 0
        self._pending = None  # raw (K, V) of a first prefill not yet compacted
        self._last_result = None

    # The scalars an eviction computes on the device (n_ctx_data, the minimum global size, through them the number of
    # logical rows after a first update) reach the host lazily: `post_update` only notes that they are on their way.
    def _resolve(self):
        if self._await is None:
            return
        seq, first = self._await
        self._await = None
        res = self._evict.wait(seq)
        redo, self._redo = self._redo, None
        if redo is not None:
            # a first eviction that was launched into a cache of guessed capacity
            src, roles, params, ws, result, full = redo
            if res.all_sw:
                # the kernel left everything alone: the reference keeps the uncompacted cache here and works in place
                self._buf_k = self._buf_v = self._buf_valid = self._buf_pos = None
                self._n_rows = 0
                self._pending = src
                self._materialize_pending()
                params.n_alloc = self._n_rows
                ops.evict_apply_inplace(self._buf_k, self._buf_v, self._buf_valid, self._buf_pos, roles, self.size_global_kv,
                                        self.size_local_kv, params, ws, result)
            else:
                rows = self._logical_rows(int(res.n_ctx_data))
                self._kept_share = rows / full
                if rows > self._buf_k.shape[2]:  # the guess was too small: once more, at the right size
                    self._launch_first(src, roles, params, ws, result, rows)
                self._sizes_stale = False  # the out-of-place kernel has written them
        self._take_result(res, first)

    def settle(self, wait: bool = True):
        """A first eviction launched on a guessed capacity keeps the caller's K / V until the plan's numbers confirm the
        guess (a guess that was too small is redone from those tensors).  `settle` ends that: with `wait` it takes
        the numbers as soon as the plan kernel has written them, without it only if they are there already.  The
        container calls it for a layer when the next layer has been queued, so that the tensors are held for about
        one layer's work and the relaunch, if there is one, reads them before their owner's next forward pass."""
        if self._redo is not None and (wait or self._evict.reported(self._await[0])):
            self._resolve()

    def _logical_rows(self, n_ctx: int) -> int:
        """Rows the reference's cache tensors have after a first eviction that left n_ctx live rows (:373-380)."""
        return math.ceil(n_ctx / self.chunk_size) * self.chunk_size

    def _full_rows(self, x_len: int) -> int:
        """Rows of [W zeros | K | pad] (:215-236)."""
        return self.sliding_window_size + x_len + get_pad_size(x_len, self.chunk_size)

    def _launch_first(self, src, roles, params, ws, result, rows: int):
        """The out-of-place eviction of a first prefill into a fresh cache of `rows` rows."""
        k_raw, v_raw = src
        self._pending = None
        self._allocate(rows, k_raw, zero=False)  # the apply kernel writes all rows
        params.n_alloc = rows
        if k_raw.stride(-1) != 1 or ops.strides_differ(k_raw, v_raw):
            k_raw, v_raw = k_raw.contiguous(), v_raw.contiguous()
        ops.evict_apply_first(k_raw, v_raw, self._buf_k, self._buf_v, self._buf_valid, self._buf_pos, roles,
                              self._sizes[0], self._sizes[1], params, ws, result)  # (writes the sizes unless every chunk slides)

    def _evict_first(self, src, roles, params, ws, result, first: bool):
        """The eviction of a first prefill that is still raw K / V.  The size of the compacted cache is a result of
        the plan kernel.  A cache that has been through a first eviction before (and was reset) allocates on the
        share of rows it kept then, with some room, launches at once and checks the guess when the plan's numbers
        arrive; otherwise the host waits for them.  Returns False if the eviction has to run in place instead."""
        full = self._full_rows(src[0].shape[2])
        if self._kept_share is not None:
            C = self.chunk_size
            cap = min(full, math.ceil((full * min(1.0, self._kept_share * 1.0625) + 2 * C) / C) * C)
            self._launch_first(src, roles, params, ws, result, cap)
            self._redo = (src, roles, params, ws, result, full)
            self._await = (params.seq, first)
            self.settle(wait=False)
            return True
        res = self._evict.wait(params.seq)
        if res.all_sw:  # the reference keeps the untruncated cache here (:283-288)
            self._materialize_pending()
            return False
        rows = self._logical_rows(int(res.n_ctx_data))
        self._kept_share = rows / full
        self._launch_first(src, roles, params, ws, result, rows)
        self._sizes_stale = False  # the out-of-place kernel has written them
        self._take_result(res, first)
        return True

    def _take_result(self, res, first: bool):
        """nats_chunk_layer_cache.py:283-288, 358, 371-380 on the numbers of the plan kernel."""
        self._last_result = res
        self._n_ctx = int(res.n_ctx_data)
        if res.all_sw:
            return
        self._gmin = int(res.gmin)
        if first:
            self._n_rows = math.ceil(self._n_ctx / self.chunk_size) * self.chunk_size
            self._mark_spare()

    def _lazy(name):  # noqa: N805 -- a host scalar that a pending eviction result may still change
        def get(self):
            self._resolve()
            return getattr(self, name)

        def put(self, value):
            self._resolve()
            setattr(self, name, value)
        return property(get, put)

    n_ctx_data = _lazy("_n_ctx")
    _n_global_min = _lazy("_gmin")
    _rows = _lazy("_n_rows")
    del _lazy

    @property
    def last_evict_result(self):
        """All numbers of the last eviction's plan (nats_evict_result), read from device memory."""
        self._resolve()
        return None if self._last_result is None else self._evict.full_result()

    def get_seq_length(self):
        return self._seen_tokens

    def get_chunk_fill_size(self):
        return self.chunk_fill_size

    @property
    def cache_k(self):
        self._materialize_pending()
        return None if self._buf_k is None else self._buf_k[:, :, :self._rows]

    @property
    def cache_v(self):
        self._materialize_pending()
        return None if self._buf_v is None else self._buf_v[:, :, :self._rows]

    @property
    def valid_tokens(self):
        self._materialize_pending()
        return None if self._buf_valid is None else self._buf_valid[:, :, :self._rows].view(torch.bool)

    @property
    def token_positions(self):
        """int32 [B, H, rows]: stream position of the token each row holds (-1 = none); needs track_positions."""
        self._materialize_pending()
        return None if self._buf_pos is None else self._buf_pos[:, :, :self._rows]

    # -- storage --------------------------------------------------------------------------------
    def _allocate(self, rows: int, like: torch.Tensor, zero: bool = True):
        """`zero=False` when the caller's kernel writes every row of every tensor itself."""
        B, H, D = like.shape[0], like.shape[1], like.shape[3]
        new = torch.zeros if zero else torch.empty
        self._uninit, self._clean = not zero, None
        self._buf_k = new(B, H, rows, D, dtype=like.dtype, device=like.device)
        self._buf_v = new(B, H, rows, D, dtype=like.dtype, device=like.device)
        self._buf_valid = new(B, H, rows, dtype=torch.uint8, device=like.device)
        if not self.track_positions:
            self._buf_pos = None
        elif zero:
            self._buf_pos = torch.full((B, H, rows), -1, dtype=torch.int32, device=like.device)
        else:
            self._buf_pos = torch.empty(B, H, rows, dtype=torch.int32, device=like.device)
        self._rows = rows

    def _mark_spare(self):
        """After a first eviction into buffers that came uninitialised: the out-of-place kernel writes the rows up to the
        logical end of the cache only, the spare rows behind them hold nothing yet."""
        if self._uninit and self._buf_k is not None and self._buf_k.shape[2] > self._n_rows:
            self._clean = self._n_rows
        self._uninit = False

    def _init_rows(self, lo: int, hi: int):
        """Buffer rows [lo, hi) as a fresh cache has them: zeros, not valid, no token."""
        self._buf_k[:, :, lo:hi].zero_()
        self._buf_v[:, :, lo:hi].zero_()
        self._buf_valid[:, :, lo:hi].zero_()
        if self._buf_pos is not None:
            self._buf_pos[:, :, lo:hi].fill_(-1)

    def _grow(self, rows: int):
        cap = self._buf_k.shape[2]
        if self._clean is not None and rows > self._clean:
            # the cache extends into spare rows: the ones it takes now (all of them before the buffers are copied)
            hi = cap if rows >= cap else rows
            self._init_rows(self._clean, hi)
            self._clean = hi if hi < cap else None
        if rows > cap:
            new_cap = max(rows, cap + max(cap // 2, 4 * self.chunk_size))
            new_cap = math.ceil(new_cap / self.chunk_size) * self.chunk_size

            def widen(t, fill):
                shape = list(t.shape)
                shape[2] = new_cap
                n = torch.empty(shape, dtype=t.dtype, device=t.device)
                n[:, :, :cap] = t
                n[:, :, cap:].fill_(fill)
                return n

            self._buf_k = widen(self._buf_k, 0)
            self._buf_v = widen(self._buf_v, 0)
            self._buf_valid = widen(self._buf_valid, 0)
            if self._buf_pos is not None:
                self._buf_pos = widen(self._buf_pos, -1)
        self._rows = max(self._rows, rows)

    def _materialize_pending(self):
        """Writes [W zeros | K | pad] (nats_chunk_layer_cache.py:215-236) if the first prefill is still raw."""
        if self._pending is None:
            return
        k, v = self._pending
        self._pending = None
        W, x_len = self.sliding_window_size, k.shape[2]
        rows = W + x_len + get_pad_size(x_len, self.chunk_size)
        self._allocate(rows, k)
        self._buf_k[:, :, W:W + x_len] = k
        self._buf_v[:, :, W:W + x_len] = v
        self._buf_valid[:, :, W:W + x_len] = 1
        if self._buf_pos is not None:
            self._buf_pos[:, :, W:W + x_len] = torch.arange(x_len, dtype=torch.int32, device=k.device)

    # -- append (nats_chunk_layer_cache.py:171-256) ----------------------------------------------
    def _note_roles(self, token_states_info, roles):
        self._tokens_info = token_states_info
        if roles is not None:
            self._roles = roles.contiguous()
        else:
            self._roles = None if token_states_info is None else ops.roles_from_one_hot(token_states_info).contiguous()

    def update(self, key_states: torch.Tensor, value_states: torch.Tensor, token_states_info: torch.Tensor | None,
               roles: torch.Tensor | None = None):
        """`roles` (uint8 [B, H, S]) may be handed over beside the one-hot tensor by a caller that has them already."""
        if not key_states.is_cuda:
            raise ValueError("NAtSChunkLayerCache.update takes GPU tensors")
        x_len = key_states.shape[2]
        self.chunk_fill_size += x_len
        if token_states_info is None and roles is None:
            assert self.chunk_fill_size < self.chunk_size, \
                "a new token_states_info must be generated once the open chunk is full"
        if x_len == 0:
            return self.cache_k[:, :, :self.n_ctx_data], self.cache_v[:, :, :self.n_ctx_data]
        self._note_roles(token_states_info, roles)
        if self._buf_k is None and self._pending is None:
            self._pending = (key_states, value_states)
            if self.chunk_fill_size < self.chunk_size or x_len == 1:
                # nothing will be evicted by the coming post_update, or (one token that is a whole chunk:
                # chunk_size == 1) it takes the one-token form, which works in place
                self._materialize_pending()
            return key_states, value_states
        self._materialize_pending()
        start = self.n_ctx_data
        end = start + x_len
        self._grow(math.ceil(end / self.chunk_size) * self.chunk_size)
        self._write_rows(key_states, value_states, start, end, plan_ahead=True)
        return self._buf_k[:, :, :end], self._buf_v[:, :, :end]

    def _inplace_prepare(self, x_len: int, seen_after: int):
        """Parameter struct and prepared call of the in-place eviction that follows an update of x_len tokens, from the
        state as it stands between that update and its post_update; also the facts the struct was filled from."""
        C, W = self.chunk_size, self.sliding_window_size
        roles, fill = self._roles, self.chunk_fill_size
        S, D = roles.shape[-1], self._buf_k.shape[3]
        params = self._inplace_params
        if params is None or params.D != D:
            params = self._inplace_params = ops.evict_params(self.bsz, self.n_msks, D, C, W, S, 0, 0, 0, 0, 0, False, 0)
        facts = (S, x_len, fill, int(seen_after == x_len), self.n_ctx_data, self._n_global_min, self.sliding_queue_tail, self._rows)
        (params.S, params.x_len, params.fill, params.first, params.n_ctx_data, params.gmin, params.tail, params.n_alloc) = facts
        call = self._inplace_call
        if call is None or not call.matches(self._buf_k, self._buf_v, self._buf_valid, self._buf_pos, S):
            if self._evict is None:
                self._evict = ops.EvictBuffers(self.device)
            call = self._inplace_call = ops.EvictInplaceCall(self._buf_k, self._buf_v, self._buf_valid, self._buf_pos,
                                                             self.size_global_kv, self.size_local_kv, self._evict,
                                                             self.bsz, self.n_msks, S)
        return params, call, facts

    def _write_rows(self, key_states, value_states, start: int, end: int, plan_ahead: bool = False):
        """Rows [start, end) of the cache, their valid bytes and stream positions: one kernel where the layouts
        allow 16-byte accesses, slice assignments otherwise.  When the update completes a chunk and the roles are few,
        the same launch plans the eviction its post_update will run (`plan_ahead`)."""
        call = self._append_call
        if call is None or not call.matches(key_states, value_states, self._buf_k, self._buf_v, self._buf_valid, self._buf_pos):
            call = self._append_call = ops.CacheAppendCall(key_states, value_states, self._buf_k, self._buf_v,
                                                           self._buf_valid, self._buf_pos)
        self._planned = None
        roles = self._roles
        if (plan_ahead and roles is not None and self.chunk_fill_size >= self.chunk_size and call.ok
                and roles.shape[-1] <= ops.EvictInplaceCall.PLAN_WITH_APPEND_SLOTS
                and self.bsz * self.n_msks <= ops.EvictInplaceCall.PLAN_WITH_APPEND_HEADS):
            x_len = end - start
            params, plan, facts = self._inplace_prepare(x_len, self._seen_tokens + x_len)
            if call(key_states, value_states, start, self._seen_tokens, plan=plan, roles=roles, params=params):
                self._planned = (params.seq, roles, facts)
                return
        if call(key_states, value_states, start, self._seen_tokens):
            return
        self._buf_k[:, :, start:end] = key_states.to(self._buf_k.dtype)
        self._buf_v[:, :, start:end] = value_states.to(self._buf_v.dtype)
        self._buf_valid[:, :, start:end] = 1
        if self._buf_pos is not None:
            self._buf_pos[:, :, start:end] = torch.arange(self._seen_tokens, self._seen_tokens + end - start,
                                                          dtype=torch.int32, device=self.device)

    def append_rotated(self, q: torch.Tensor, key_states: torch.Tensor, value_states: torch.Tensor, cos: torch.Tensor,
                       sin: torch.Tensor, token_states_info: torch.Tensor | None = None,
                       roles: torch.Tensor | None = None):
        """`update` for a cache that already holds rows, with the rotary embedding of q and k applied on the way
        (one kernel: hf/llama_nats_chunk.py:227 + nats_chunk_layer_cache.py:243-256).  q / k / v are the projections
        before the rotary embedding; returns (rotated q, keys, values)."""
        if self._buf_k is None and self._pending is None:
            raise ValueError("append_rotated needs a cache that holds rows; the first segment goes through update")
        x_len = key_states.shape[2]
        self.chunk_fill_size += x_len
        if token_states_info is None and roles is None:
            assert self.chunk_fill_size < self.chunk_size, \
                "roles must be generated once the open chunk is full"
        self._note_roles(token_states_info, roles)
        self._materialize_pending()
        start = self.n_ctx_data
        end = start + x_len
        self._grow(math.ceil(end / self.chunk_size) * self.chunk_size)
        q_rot = ops.rope_append(q, key_states, value_states, cos, sin, self._buf_k, self._buf_v, self._buf_valid,
                                self._buf_pos, start, self._seen_tokens)
        return q_rot, self._buf_k[:, :, :end], self._buf_v[:, :, :end]

    # -- masks (nats_chunk_layer_cache.py:156-163, 444-460, 622-632) ------------------------------
    def generate_mask(self, x_len: int):
        """Debug / parity output; the attention kernels never call it."""
        if x_len == 1:
            if self._seen_tokens == 0:
                return torch.ones(1, 1, 1, 1, dtype=torch.bool, device=self.device)
            return self.valid_tokens[:, :, :self.n_ctx_data + 1].unsqueeze(-2)
        if self._seen_tokens == 0:
            if self._roles is None:
                raise ValueError("generate_mask needs the roles handed to update")
            return ops.prefill_mask(self._roles, x_len, self.chunk_size, self.sliding_window_size)
        return ops.prefill_past_mask(self._buf_valid, self.size_global_kv, self.size_local_kv, self.segment_roles(),
                                     x_len, self.chunk_size, self.sliding_window_size, self.past_state(x_len))

    def past_state(self, x_len: int):
        """The scalars a segment of x_len tokens, appended by the last update and not yet evicted, is masked
        with (nats_chunk_layer_cache.py:462-511)."""
        return ops.past_state(self.n_ctx_data, self.chunk_fill_size - x_len, self._n_global_min, self.sliding_queue_tail,
                              self._seen_tokens, self.chunk_fill_size_last)

    def segment_roles(self):
        """Roles handed to the last update; one global slot while the open chunk is not complete (:589-596)."""
        if self._roles is not None:
            return self._roles
        return torch.zeros(self.bsz, self.n_msks, 1, dtype=torch.uint8, device=self.device)

    def segment_attention(self, q: torch.Tensor, sm_scale: float | None = None):
        """Attention of the multi-token segment the last update appended, over the whole cache: what the
        reference computes as SDPA(q, cache_k, cache_v, generate_mask(x_len)) for a non-empty cache."""
        x_len = q.shape[2]
        return ops.prefill_past_attention(q, self._buf_k, self._buf_v, self._buf_valid, self.size_global_kv,
                                          self.size_local_kv, self.segment_roles(), self.chunk_size,
                                          self.sliding_window_size, self.past_state(x_len), sm_scale)

    def row_end(self) -> torch.Tensor:
        """int64 [B, H_kv]: the first cache row past a head's own global and local rows (size_global_kv +
        size_local_kv), the hint `ops.decode_attention` takes.  Computed once per eviction."""
        if self._row_end is None:
            self._row_end = self.size_global_kv + self.size_local_kv
        return self._row_end

    def decode_hint(self):
        """(row_end, tail_start) for `ops.decode_attention` after the update of a one-token step: rows
        [row_end[b, h], tail_start) hold nothing valid; the open chunk starts at tail_start."""
        return self.row_end(), self.n_ctx_data - (self.chunk_fill_size - 1)

    # -- evict + compact (nats_chunk_layer_cache.py:258-389) -------------------------------------
    def post_update(self, x_len: int):
        C, W = self.chunk_size, self.sliding_window_size
        self._seen_tokens += x_len
        if x_len == 0 or self.chunk_fill_size < C:
            self.chunk_fill_size_last = self.chunk_fill_size
            self.n_ctx_data += x_len
            return
        fill = self.chunk_fill_size
        partial, n_done = fill % C, fill // C
        first = self._seen_tokens == x_len
        self._row_end = None  # the apply kernels below rewrite the sizes
        roles = self._roles
        if roles is None:
            raise ValueError("post_update needs the roles handed to the update that completed a chunk")
        S = roles.shape[-1]
        src = self._pending
        like = src[0] if src is not None else self._buf_k
        D = like.shape[3]
        if self._evict is None:
            self._evict = ops.EvictBuffers(self.device)
        if src is None:
            # a cache that holds rows: plan + in-place apply through the call prepared for these buffers; the plan
            # has run already if it rode with the append of these rows
            params, call, facts = self._inplace_prepare(x_len, self._seen_tokens)
            planned, self._planned = self._planned, None
            if planned is not None and planned[1] is roles and planned[2] == facts:
                params.seq = planned[0]
                call.apply_planned(roles, params)
            else:
                call(roles, params)
            self._await = (params.seq, first)  # picked up when the host next needs n_ctx_data or the minimum global size
        else:
            params = ops.evict_params(self.bsz, self.n_msks, D, C, W, S, x_len, fill, self.n_ctx_data, self._n_global_min,
                                      self.sliding_queue_tail, first, max(self._rows, C))
            # (the first tokens of the cache: the plan does not read the size tensors, which may not have been reset)
            ws, result = ops.evict_plan(roles, self._sizes[0], self._sizes[1], params, self._evict)
            if not self._evict_first(src, roles, params, ws, result, first):
                params.n_alloc = self._rows
                ops.evict_apply_inplace(self._buf_k, self._buf_v, self._buf_valid, self._buf_pos, roles,
                                        self.size_global_kv, self.size_local_kv, params, ws, result)
                self._await = (params.seq, first)
        # host-side bookkeeping (nats_chunk_layer_cache.py:400-413)
        n_ring = min(n_done, self.n_chunks_per_sw)
        start = 0 if first else self.sliding_queue_tail
        self.sliding_queue_tail = (start + n_ring * C) % W
        self.chunk_fill_size = partial
        self.chunk_fill_size_last = partial


class NAtSLayerCache(NAtSChunkLayerCache):
    """One layer's cache with a role per token (chunk_size == 1), the reference's NAtSLayerCache
    (src/nats/components/cache/nats_layer_cache.py:20-808): rows are appended at once, the eviction is deferred
    until `update_chunk_size` tokens are pending and then handles the whole pending block.  Row layout of
    cache_k[b, h] between forward calls:

        [0, W)                        ring of the last W evicted-or-kept tokens, `sliding_queue_tail` = the slot
                                      written last; rows are copied whatever the role, valid only if sliding window
        [W, size_global)              global tokens, stream order
        [size_global, +size_local)    local tokens newer than the last global token
        [.., P)                       stale rows of shorter heads (and the rows of earlier all-sliding-window blocks)
        [P, n_ctx_data)               the pending block

    Storage (capacity buffer, deferred first prefill) and the kernels are those of the chunked class with one-token
    chunks; the state machine is this class's own.  With `update_chunk_size == 1` nothing is deferred and a one-token
    step is the reference's one-step branch (:328-367), which the kernels take from `update_chunk == 1, x_len == 1`."""

    def __init__(self, bsz: int, n_msks: int, sliding_window_size: int, layer_id: int = 0, update_chunk_size: int = 16,
                 device: torch.device | str = "cuda", track_positions: bool = False):
        if sliding_window_size < update_chunk_size:  # nats_layer_cache.py:77-78
            raise NotImplementedError("The sliding window size must be greater or equal to the update chunk size!")
        if update_chunk_size < 1:
            raise ValueError("update_chunk_size must be positive")
        if update_chunk_size == 1 and sliding_window_size < 2:
            # nats_layer_cache.py:344 writes ring slot 1 at the first one-token call, which a window of one does not have
            raise NotImplementedError("update_chunk_size == 1 needs a sliding window of at least two tokens")
        self.update_chunk_size = update_chunk_size
        super().__init__(bsz, n_msks, sliding_window_size, layer_id=layer_id, chunk_size=1, device=device,
                         track_positions=track_positions)

    def reset_cache(self):
        super().reset_cache()
        self._clear_slot = None  # ring slot whose valid byte is to be switched off (see post_update) and has not been yet
        self._in_chunk = None   # uint8 [B, H, U]: roles of the pending tokens (:196-200, :218)
        self._block = None      # roles of the whole pending block as of the last update (_tokens_info, :209-219)
        self._block_fill = 0
        self._mask_roles = None  # the block as of the last multi-token update (:229-231)
        self._live_end = self.sliding_window_size  # n_ctx_data after the last eviction that moved rows

    # A step whose eviction is deferred switches off one ring slot (:300-310).  Nothing reads the valid bytes between
    # that step's attention and the next step's, so the byte is written with the next step's rows (one kernel less per
    # token) -- or at once for whoever looks at the valid bytes before.
    def _flush_clear(self):
        slot, self._clear_slot = self._clear_slot, None
        if slot is not None and self._buf_valid is not None:
            self._buf_valid[:, :, slot] = 0

    @property
    def valid_tokens(self):
        self._materialize_pending()
        self._flush_clear()
        return None if self._buf_valid is None else self._buf_valid[:, :, :self._rows].view(torch.bool)

    # -- append (nats_layer_cache.py:167-286) ------------------------------------------------------
    def _pad_rows(self, n: int) -> int:
        U = self.update_chunk_size
        return math.ceil(n / U) * U

    def _materialize_pending(self):
        """[W zeros | K | pad to the update chunk] (:236-258) if the first prefill is still raw."""
        if self._pending is None:
            return
        k, v = self._pending
        self._pending = None
        W, x_len = self.sliding_window_size, k.shape[2]
        self._allocate(W + self._pad_rows(x_len), k)
        self._buf_k[:, :, W:W + x_len] = k
        self._buf_v[:, :, W:W + x_len] = v
        self._buf_valid[:, :, W:W + x_len] = 1
        if self._buf_pos is not None:
            self._buf_pos[:, :, W:W + x_len] = torch.arange(x_len, dtype=torch.int32, device=k.device)

    def _grow(self, rows: int):
        super()._grow(self._pad_rows(rows))

    def _logical_rows(self, n_ctx: int) -> int:
        return n_ctx  # the first eviction cuts the cache to its live rows (:404-408)

    def _full_rows(self, x_len: int) -> int:
        return self.sliding_window_size + self._pad_rows(x_len)

    def role_destination(self, x_len: int = 1):
        """Where the roles of the next x_len tokens belong among the pending ones: a uint8 [B, H, x_len] view into which
        a role kernel may write them directly (`ops.role_step(..., roles_out=...)`); handed to `update` /
        `append_rotated` as `roles` it costs no copy.  None when the tokens do not fit the pending buffer."""
        U = self.update_chunk_size
        if self._in_chunk is None:
            self._in_chunk = torch.zeros(self.bsz, self.n_msks, U, dtype=torch.uint8, device=self.device)
        at = self.chunk_fill_size
        return self._in_chunk[:, :, at:at + x_len] if at + x_len <= U else None

    def _pending_block(self):
        """uint8 [B, H, fill] contiguous: the roles of the whole pending block (made from the buffer when asked for;
        a full buffer is the block itself)."""
        if self._block is None:
            self._block = self._in_chunk[:, :, :self._block_fill].contiguous()
        return self._block

    def _note_roles(self, token_states_info, roles):
        """Roles of the new tokens join the pending block."""
        U = self.update_chunk_size
        if roles is None:
            roles = ops.roles_from_one_hot(token_states_info)
        x_len = roles.shape[-1]
        self._tokens_info = token_states_info
        if self._in_chunk is None:
            self._in_chunk = torch.zeros(self.bsz, self.n_msks, U, dtype=torch.uint8, device=self.device)
        fill, last = self.chunk_fill_size, self.chunk_fill_size_last
        if fill > U:
            self._block = torch.cat([self._in_chunk[:, :, :last], roles], dim=2).contiguous()
        else:
            in_place = (roles.data_ptr() == self._in_chunk.data_ptr() + last and roles.stride(1) == U
                        and (self.bsz == 1 or roles.stride(0) == self.n_msks * U) and (x_len == 1 or roles.stride(2) == 1))
            if not in_place:  # (a role kernel that was given `role_destination` has written them already)
                self._in_chunk[:, :, last:fill] = roles
            self._block = None
        self._block_fill = fill
        self._roles = None
        if x_len > 1:
            self._mask_roles = self._pending_block()

    def update(self, key_states: torch.Tensor, value_states: torch.Tensor, token_states_info: torch.Tensor | None,
               roles: torch.Tensor | None = None):
        """token_states_info [B, H, x_len, 3] (or `roles` uint8 [B, H, x_len]): one role per new token."""
        if not key_states.is_cuda:
            raise ValueError("NAtSLayerCache.update takes GPU tensors")
        x_len = key_states.shape[2]
        if x_len == 0:
            return self.cache_k[:, :, :self.n_ctx_data], self.cache_v[:, :, :self.n_ctx_data]
        if token_states_info is None and roles is None:
            raise ValueError("the per-token cache needs the role of every new token")
        self.chunk_fill_size += x_len
        self._note_roles(token_states_info, roles)
        if self._buf_k is None and self._pending is None:
            self._pending = (key_states, value_states)
            if self.chunk_fill_size < self.update_chunk_size:
                self._materialize_pending()  # nothing will be evicted by the coming post_update
            return key_states, value_states
        self._materialize_pending()
        self._flush_clear()
        start = self.n_ctx_data
        end = start + x_len
        self._grow(end)
        self._write_rows(key_states, value_states, start, end)
        return self._buf_k[:, :, :end], self._buf_v[:, :, :end]

    def append_rotated(self, q, key_states, value_states, cos, sin, token_states_info=None, roles=None):
        """`update` for a cache that already holds rows, with the rotary embedding of q and k applied on the way."""
        if self._buf_k is None and self._pending is None:
            raise ValueError("append_rotated needs a cache that holds rows; the first segment goes through update")
        if token_states_info is None and roles is None:
            raise ValueError("the per-token cache needs the role of every new token")
        x_len = key_states.shape[2]
        self.chunk_fill_size += x_len
        self._note_roles(token_states_info, roles)
        self._materialize_pending()
        start = self.n_ctx_data
        end = start + x_len
        self._grow(end)
        clear, self._clear_slot = self._clear_slot, None
        q_rot = ops.rope_append(q, key_states, value_states, cos, sin, self._buf_k, self._buf_v, self._buf_valid,
                                self._buf_pos, start, self._seen_tokens, -1 if clear is None else clear)
        return q_rot, self._buf_k[:, :, :end], self._buf_v[:, :, :end]

    # -- masks (nats_layer_cache.py:155-162, 469-554) ------------------------------------------------
    def generate_mask(self, x_len: int):
        """Debug / parity output; the attention kernels never call it."""
        if x_len == 1:
            if self._seen_tokens == 0:
                return torch.ones(1, 1, 1, 1, dtype=torch.bool, device=self.device)
            return self.valid_tokens[:, :, :self.n_ctx_data + 1].unsqueeze(-2)
        if self._mask_roles is None:
            raise ValueError("generate_mask needs the roles handed to update")
        if self._seen_tokens == 0:
            return ops.prefill_mask(self._mask_roles, x_len, 1, self.sliding_window_size)
        self._materialize_pending()
        self._flush_clear()
        return ops.prefill_past_mask(self._buf_valid, self.size_global_kv, self.size_local_kv, self._mask_roles, x_len, 1,
                                     self.sliding_window_size, self.past_state(x_len))

    def past_state(self, x_len: int):
        return ops.past_state(self.n_ctx_data, self.chunk_fill_size - x_len, self._n_global_min, self.sliding_queue_tail,
                              self._seen_tokens, self.chunk_fill_size_last, self.update_chunk_size)

    def segment_roles(self):
        return self._mask_roles

    def decode_hint(self):
        """(row_end, tail_start) for `ops.decode_attention` after the update of a one-token step: rows
        [row_end[b, h], tail_start) hold nothing valid.  Pending blocks start where the last eviction that moved rows
        left n_ctx_data (blocks of sliding-window tokens stay where they were, still valid)."""
        self._resolve()
        return self.row_end(), min(self._live_end, self.n_ctx_data)

    def _take_result(self, res, first: bool):
        """nats_layer_cache.py:316-327, 394, 402-408 on the numbers of the plan kernel (`first`: the call held every
        token seen so far, so the cache is cut to its live rows)."""
        self._last_result = res
        if res.all_sw:
            return  # n_ctx_data stays: the block's rows remain where they are, valid
        self._n_ctx = int(res.n_ctx_data)
        self._live_end = self._n_ctx
        self._gmin = int(res.gmin)
        if first:
            self._n_rows = self._n_ctx
            self._mark_spare()

    # -- evict + compact (nats_layer_cache.py:292-418) ---------------------------------------------
    def post_update(self, x_len: int):
        W, U = self.sliding_window_size, self.update_chunk_size
        self._seen_tokens += x_len
        if x_len == 0:
            return
        fill = self.chunk_fill_size
        block_start = self.n_ctx_data - (fill - x_len)  # first row of the pending block
        self.n_ctx_data += x_len
        if fill < U:
            # the eviction is deferred; the ring slot the next token would take is switched off (:300-310)
            slot = fill if self._seen_tokens < U else (fill + self.sliding_queue_tail + 1) % W
            self._materialize_pending()
            self._flush_clear()
            self._clear_slot = slot  # (written with the next step's rows, or by whoever reads the valid bytes first)
            self.chunk_fill_size_last = fill
            return
        self._flush_clear()
        first_ring = fill == self._seen_tokens   # the block holds every token seen so far (:439)
        first_call = self._seen_tokens == x_len  # (:404)
        roles = self._pending_block()
        if x_len == 1 and self._pending is not None:
            # (update_chunk_size == 1: the first token ever is evicted at once, by the one-step branch :328-367, in place)
            self._materialize_pending()
        src = self._pending
        like = src[0] if src is not None else self._buf_k
        D = like.shape[3]
        if self._evict is None:
            self._evict = ops.EvictBuffers(self.device)
        self._row_end = None
        if src is None:
            # a cache that holds rows: plan + in-place apply through the call prepared for these buffers
            params = self._inplace_params
            if params is None or params.D != D:
                params = self._inplace_params = ops.evict_params(self.bsz, self.n_msks, D, 1, W, fill, 0, 0, 0, 0, 0, False, 0,
                                                                 update_chunk=U)
            params.S, params.x_len, params.fill, params.first = fill, x_len, fill, int(first_ring)
            params.n_ctx_data, params.gmin, params.tail = block_start, self._n_global_min, self.sliding_queue_tail
            params.n_alloc = self._rows
            call = self._inplace_call
            if call is None or not call.matches(self._buf_k, self._buf_v, self._buf_valid, self._buf_pos, fill):
                call = self._inplace_call = ops.EvictInplaceCall(self._buf_k, self._buf_v, self._buf_valid, self._buf_pos,
                                                                 self.size_global_kv, self.size_local_kv, self._evict,
                                                                 self.bsz, self.n_msks, fill)
            call(roles, params)
            self._await = (params.seq, first_call)  # picked up when the host next needs n_ctx_data
        else:
            params = ops.evict_params(self.bsz, self.n_msks, D, 1, W, fill, x_len, fill, block_start, self._n_global_min,
                                      self.sliding_queue_tail, first_ring, max(self._rows, 1), update_chunk=U)
            # (the first tokens of the cache: the plan does not read the size tensors, which may not have been reset)
            ws, result = ops.evict_plan(roles, self._sizes[0], self._sizes[1], params, self._evict)
            if not self._evict_first(src, roles, params, ws, result, first_call):
                params.n_alloc = self._rows
                ops.evict_apply_inplace(self._buf_k, self._buf_v, self._buf_valid, self._buf_pos, roles, self.size_global_kv,
                                        self.size_local_kv, params, ws, result)
                self._await = (params.seq, first_call)
        n_ring = min(fill, W)  # :437-445
        self.sliding_queue_tail = n_ring - 1 if first_ring else (self.sliding_queue_tail + n_ring) % W
        self.chunk_fill_size = 0
        self.chunk_fill_size_last = 0
        self._block = self._roles = None


try:  # the reference's container is a transformers cache (dyn_cache.py:66): HF models take it as past_key_values
    from transformers.cache_utils import DynamicCache as _CacheBase
except Exception:  # transformers absent or unusable: a plain class with the same surface
    _CacheBase = object


class NAtSCache(_CacheBase):
    """Container of per-layer caches (src/nats/components/cache/dyn_cache.py:66-195).  A subclass of
    transformers' DynamicCache where that library is importable; like the reference it does not run the base
    class's __init__ and answers every call its callers make itself."""

    def __init__(self, sliding_window_size: int, chunk_size: int = 1, track_positions: bool = False):
        # chunk_size == 1 (per-token roles) builds NAtSLayerCache layers, any other size NAtSChunkLayerCache layers
        # (dyn_cache.py:180-190)
        self.cache_model: list[NAtSChunkLayerCache | NAtSLayerCache] = []
        self.sliding_window_size = sliding_window_size
        self.chunk_size = chunk_size
        self.cached_x: list[torch.Tensor | None] = []
        self.track_positions = track_positions
        self._spare_layers: list = []

    def reset_cache(self):
        """dyn_cache.py:76-78: the container is empty afterwards.  The layer objects are kept aside and taken up again,
        reset, by the next prompt's updates (same batch size, heads and device): they hold the eviction workspaces, the
        pinned result mirror and the share of rows the last first eviction kept, from which the next first eviction
        sizes its cache without waiting for its plan."""
        old = self.cache_model + getattr(self, "_spare_layers", [])[len(self.cache_model):]
        self._spare_layers = old
        self.cache_model = []
        self.cached_x = []

    def __len__(self):
        return len(self.cache_model)

    def get_max_cache_shape(self, layer_idx: int = 0):
        return -1  # no fixed maximum: rows are evicted, capacity grows on demand

    def get_seq_length(self, layer_idx: int = 0) -> int:
        if len(self.cache_model) <= layer_idx:
            return 0
        return self.cache_model[layer_idx]._seen_tokens

    # What a transformers model asks of its cache while it prepares a forward pass (newer releases of that library
    # build their causal mask from these; the NAtS attention layers ignore that mask and compute their own).  The base
    # class answers them from a `layers` list its __init__ would have made, which does not exist here.
    @property
    def layers(self):
        return self.cache_model

    @property
    def is_sliding(self):
        return [False] * len(self.cache_model)

    @property
    def is_compileable(self) -> bool:
        return False

    @property
    def is_initialized(self) -> bool:
        return len(self.cache_model) > 0

    def get_mask_sizes(self, query_length, layer_idx: int = 0):
        """(kv_length, kv_offset) of the mask the caller is about to build: every token seen so far plus the new ones."""
        n = query_length if isinstance(query_length, int) else int(query_length.shape[0])  # (older releases pass cache_position)
        return self.get_seq_length(layer_idx) + n, 0

    def get_max_length(self, layer_idx: int = 0):
        return -1

    def generate_mask(self, layer_idx: int, x_len: int):
        return self.cache_model[layer_idx].generate_mask(x_len)

    def get_nats_chunk_fill_size(self, layer_idx: int = 0):
        if len(self.cache_model) <= layer_idx or self.chunk_size == 1:  # dyn_cache.py:87-91
            return 0
        return self.cache_model[layer_idx].chunk_fill_size

    def get_nats_cached_x_in_chunk(self, layer_idx: int = 0):
        if len(self.cached_x) <= layer_idx:
            return None
        return self.cached_x[layer_idx]

    @staticmethod
    def merge_new_x_values_in_chunk(x_cache, x_new, chunk_size: int, chunk_merge_method=ChunkMergeType.MEAN):
        """Running chunk statistic of the hidden states (dyn_cache.py:98-115): sum of x / C, or max."""
        if chunk_merge_method == ChunkMergeType.MEAN:
            add = (x_new / chunk_size).sum(1, keepdim=True)
            return add if x_cache is None else x_cache + add
        if x_cache is None:
            return x_new
        return torch.max(torch.cat([x_cache, x_new], dim=1), dim=1, keepdim=True)[0]

    def _update_cache_x(self, x_update, layer_idx: int):
        if len(self.cached_x) <= layer_idx:
            self.cached_x.append(x_update)
        else:
            self.cached_x[layer_idx] = x_update

    def update_nats_cached_x_in_chunk(self, x, layer_idx: int = 0, chunk_merge_method=ChunkMergeType.MEAN):
        """dyn_cache.py:117-124"""
        x_cache = self.get_nats_cached_x_in_chunk(layer_idx)
        self._update_cache_x(self.merge_new_x_values_in_chunk(x_cache, x, self.chunk_size, chunk_merge_method), layer_idx)

    def update_nats_cached_x_across_chunk(self, x, pre_fill_chunk_size: int, layer_idx: int = 0,
                                          chunk_merge_method=ChunkMergeType.MEAN):
        """Pooled hidden states of every chunk the new tokens touch, and the pad of the last one
        (dyn_cache.py:130-171)."""
        C = self.chunk_size
        pre = self.get_nats_chunk_fill_size(layer_idx)
        x_len = x.shape[1]
        if pre != 0:
            head_len = C - pre
            head = self.merge_new_x_values_in_chunk(self.get_nats_cached_x_in_chunk(layer_idx), x[:, :head_len], C,
                                                    chunk_merge_method)
            rest = x_len - head_len
            if rest == 0:
                pad, pooled = 0, head
            else:
                pad = get_pad_size(rest, C)
                pooled = torch.cat([head, pool_chunks(x[:, head_len:], C, pad, chunk_merge_method)], dim=1)
        else:
            pad = get_pad_size(x_len, C)
            pooled = pool_chunks(x, C, pad, chunk_merge_method)
        if pad == 0:
            carry = None
        else:
            tail = x[:, pad - C:]
            carry = (tail / C).sum(1, keepdim=True) if chunk_merge_method == ChunkMergeType.MEAN \
                else tail.max(1, keepdim=True)[0]
        self._update_cache_x(carry, layer_idx)
        return pooled, pad

    def update(self, key_states, value_states, layer_idx: int, cache_kwargs: dict[str, Any] | None = None):
        if len(self.cache_model) <= layer_idx:
            bsz, n_kv_heads = key_states.shape[:2]
            new_cache = self._spare_layer(layer_idx, bsz, n_kv_heads, key_states.device)
            if new_cache is not None:
                new_cache.reset_cache()
            elif self.chunk_size == 1:
                new_cache = NAtSLayerCache(bsz, n_kv_heads, self.sliding_window_size, layer_id=layer_idx,
                                           device=key_states.device, track_positions=self.track_positions)
            else:
                new_cache = NAtSChunkLayerCache(bsz, n_kv_heads, self.sliding_window_size, layer_id=layer_idx,
                                                chunk_size=self.chunk_size, device=key_states.device,
                                                track_positions=self.track_positions)
            self.cache_model.append(new_cache)
        elif layer_idx == 0:
            self.cache_model[-1].settle()  # (the last layer of the previous forward pass)
        return self.cache_model[layer_idx].update(key_states, value_states, **(cache_kwargs or {}))

    def _spare_layer(self, layer_idx: int, bsz: int, n_kv_heads: int, device):
        """The layer object a reset put aside for this index, if it fits the new prompt."""
        spare = getattr(self, "_spare_layers", [])
        if len(self.cache_model) != layer_idx or layer_idx >= len(spare) or spare[layer_idx] is None:
            return None
        c, spare[layer_idx] = spare[layer_idx], None
        kind = NAtSLayerCache if self.chunk_size == 1 else NAtSChunkLayerCache
        fits = (type(c) is kind and c.bsz == bsz and c.n_msks == n_kv_heads and c.device == torch.device(device)
                and c.sliding_window_size == self.sliding_window_size and c.track_positions == self.track_positions
                and (self.chunk_size == 1 or c.chunk_size == self.chunk_size))
        return c if fits else None

    def post_update(self, layer_idx: int, x_len=1, **kwargs):
        self.cache_model[layer_idx].post_update(x_len=x_len)
        if layer_idx > 0:
            self.cache_model[layer_idx - 1].settle()
