"""CPU oracle for the NAtS sparse-attention inference path.  TEST INFRASTRUCTURE ONLY.

This module restates, in plain per-(batch, kv-head) loops over numpy / CPU torch tensors, what the
reference computes on its PyTorch masked-attention path.  Nothing in the shipped package imports it;
it is used by the tests, by the smoke check and by the CPU-baseline leg of the benchmark as the
checker the HIP kernels are compared against.

Every function cites the reference lines it follows (paths relative to the reference checkout).

How each function is pinned (see tests/test_oracle_*.py):

* roles_from_logits ............ brute force over all orderings of 3 logits + closed form
                                 (attention/nats_attention.py:96-109, nats_chunk_attention.py:64-95)
* next_global_index ............ docstring vector `[0,2,2,5,5,5,6]`-style closed form, brute force
                                 (components/masks/utils.py:85-87)
* chunk_visibility / prefill_mask  7x7 docstring mask of components/masks/utils_simple.py:94-107,
                                 all-global == tril, all-sw == band, golden masks written by the
                                 reference cache (tests/golden/chunk_cache_golden.npz)
* masked_attention ............. torch SDPA with a bool mask is the library routine itself
* ChunkCacheOracle.update / generate_mask / post_update
                                 golden vectors written by the reference's NAtSChunkLayerCache on CPU
                                 (tests/golden/make_golden.py), 28 scenarios / 305 calls (chunk sizes 1 to 12), compared on
                                 every byte of cache_k, cache_v, valid_tokens, sizes and scalars
* decode_attention ............. equals masked_attention restricted to the valid rows (gather, then dense
                                 softmax); checked against torch SDPA
* pooled_role_logits ........... closed forms (constant chunks, one-hot projection rows), zero padding of the
                                 open chunk, and the invariant that any split of a stream into calls gives
                                 the statistics of one call (dyn_cache.py:98-171, chunk_utils.py:13-62)

* TokenCacheOracle.update / generate_mask / post_update (the per-token class, chunk_size == 1)
                                 golden vectors written by the reference's NAtSLayerCache on CPU
                                 (tests/golden/make_golden_token.py), 30 scenarios / 1030 calls: every mask and,
                                 after every post_update, every byte of cache_k, cache_v, valid_tokens, the sizes
                                 and the scalars (deferred 16-token eviction, ring insert, all-sliding and
                                 all-local blocks, multi-token segments over pending tokens, first segments
                                 shorter than the window and than the update chunk, update chunks of 4 and 8, and the
                                 one-step branch of update chunk 1, :328-367, in five scenarios)

Functions with parity unpinned: none of the above.  Not restated: update_chunk_size == 1 with a window of one token
(cache/nats_layer_cache.py:344 then writes ring slot 1 of a ring that has only slot 0); TokenCacheOracle refuses it.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field

import numpy as np
import torch

ROLE_GLOBAL = 0
ROLE_LOCAL = 1
ROLE_SW = 2


# ----------------------------------------------------------------------------------------------
# roles
# ----------------------------------------------------------------------------------------------
def roles_from_logits(logits: torch.Tensor, global_bias: float = 0.1, force_first_global: bool = False,
                      force_last_global: bool = False) -> np.ndarray:
    """logits [B, S, H_kv, 3] -> roles uint8 [B, H_kv, S].

    attention/nats_attention.py:96-109: the bias is added to option 0 in the logits' own dtype, the role
    is the first maximal option, slot 0 becomes global when the segment starts inside the sink chunk;
    attention/nats_chunk_attention.py:92-94: an open last chunk is marked global."""
    # `logit[..., 0] += 0.1` on the device the module runs on: torch's GPU kernels add the Python scalar in
    # fp32 and round the sum to the logits' dtype (its CPU kernel would round the scalar to bf16 first).
    lg = logits.clone()
    lg[..., 0] = (lg[..., 0].float() + torch.tensor(global_bias, dtype=torch.float32)).to(lg.dtype)
    x = lg.float().numpy()
    B, S, H, _ = x.shape
    roles = np.zeros((B, H, S), dtype=np.uint8)
    for b in range(B):
        for s in range(S):
            for h in range(H):
                best, arg = x[b, s, h, 0], 0
                for o in (1, 2):
                    if x[b, s, h, o] > best:  # strict: the first maximum wins
                        best, arg = x[b, s, h, o], o
                roles[b, h, s] = arg
    if force_first_global:
        roles[:, :, 0] = ROLE_GLOBAL
    if force_last_global:
        roles[:, :, -1] = ROLE_GLOBAL
    return roles


def pooled_role_logits(x: torch.Tensor, weight: torch.Tensor, chunk_size: int, pre_fill: int = 0,
                       carry_in: torch.Tensor | None = None, merge_max: bool = False):
    """Hidden states of the new tokens -> (pooled [B, S, dim], logits [B, S, H_kv, 3], carry, pad), with the
    torch ops the reference runs, in the dtype of x.

    components/cache/dyn_cache.py:98-115 (running statistic: sum of x / C, or max), :130-171 (chunks touched by
    the new tokens: the open chunk completed with its carried statistic, whole chunks pooled with
    chunk_utils.py:13-62, zero padding of an open last chunk) and proj_layer (nats_chunk_attention.py:87).
    While no chunk completes (pre_fill + L < C) pooled and logits are None and only the carry is returned."""
    B, L, dim = x.shape
    C = chunk_size

    def merge(cache, new):  # dyn_cache.py:98-113
        if merge_max:
            return new.max(1, keepdim=True)[0] if cache is None else torch.max(torch.cat([cache, new], 1), 1, keepdim=True)[0]
        add = (new / C).sum(1, keepdim=True)
        return add if cache is None else cache + add

    def pool(t, pad):  # chunk_utils.py:13-62
        if pad:
            t = torch.nn.functional.pad(t, (0, 0, 0, pad))
        t = t.unflatten(1, (-1, C))
        return t.max(2)[0] if merge_max else t.mean(2)

    if carry_in is not None:
        carry_in = carry_in.reshape(B, 1, dim)
    if pre_fill + L < C:  # dyn_cache.py:117-124
        return None, None, merge(carry_in if pre_fill else None, x), 0
    if pre_fill:
        head_len = C - pre_fill
        head = merge(carry_in, x[:, :head_len])
        rest = L - head_len
        if rest == 0:
            pad, pooled = 0, head
        else:
            pad = (-rest) % C
            pooled = torch.cat([head, pool(x[:, head_len:], pad)], 1)
    else:
        pad = (-L) % C
        pooled = pool(x, pad)
    carry = None
    if pad:
        tail = x[:, pad - C:]
        carry = tail.max(1, keepdim=True)[0] if merge_max else (tail / C).sum(1, keepdim=True)
    logits = torch.nn.functional.linear(pooled, weight).unflatten(-1, (-1, 3))
    return pooled, logits, carry, pad


def one_hot_roles(roles: np.ndarray, dtype=torch.float32) -> torch.Tensor:
    """roles [B, H, S] -> token_states_info [B, H, S, 3] (cache/nats_chunk_layer_cache.py:188-190)."""
    t = torch.zeros(*roles.shape, 3, dtype=dtype)
    t.scatter_(-1, torch.from_numpy(roles.astype(np.int64)).unsqueeze(-1), 1.0)
    return t


def roles_from_one_hot(tsi: torch.Tensor) -> np.ndarray:
    return tsi.float().argmax(-1).numpy().astype(np.uint8)


def next_global_index(is_global: np.ndarray) -> np.ndarray:
    """For every slot n: the first slot g >= n that is global, the last slot counting as global.

    components/masks/utils.py:85-87 (flip / cummax / flip with the last flag forced to 1)."""
    flags = np.asarray(is_global).astype(bool)
    S = flags.shape[-1]
    out = np.empty(flags.shape, dtype=np.int64)
    flat_f = flags.reshape(-1, S)
    flat_o = out.reshape(-1, S)
    for r in range(flat_f.shape[0]):
        nxt = S - 1
        for n in range(S - 1, -1, -1):
            if flat_f[r, n] or n == S - 1:
                nxt = n
            flat_o[r, n] = nxt
    return out


# ----------------------------------------------------------------------------------------------
# masks
# ----------------------------------------------------------------------------------------------
def chunk_visibility(roles: np.ndarray, window_chunks: int) -> np.ndarray:
    """roles [B, H, S] -> bool [B, H, S(query slot m), S(key slot n)], no causal cut.

    components/masks/utils.py:89-94 gives (g(n) >= m) | global-or-last(n);
    cache/nats_chunk_layer_cache.py:603-611 replaces the columns of sliding-window slots by
    (m - n) <= W / C, only if at least one slot anywhere is sliding-window."""
    B, H, S = roles.shape
    g = next_global_index(roles == ROLE_GLOBAL)
    vis = np.zeros((B, H, S, S), dtype=bool)
    any_sw = bool((roles == ROLE_SW).any())
    for b in range(B):
        for h in range(H):
            for n in range(S):
                is_g = roles[b, h, n] == ROLE_GLOBAL or n == S - 1
                for m in range(S):
                    if any_sw and roles[b, h, n] == ROLE_SW:
                        vis[b, h, m, n] = (m - n) <= window_chunks
                    else:
                        vis[b, h, m, n] = (g[b, h, n] >= m) or is_g
    return vis


def expand_chunk_mask(vis: np.ndarray, C: int) -> np.ndarray:
    return np.repeat(np.repeat(vis, C, axis=-1), C, axis=-2)


def prefill_mask(roles: np.ndarray, L: int, C: int, W: int) -> np.ndarray:
    """Token-level bool mask [B, H, L, L] of a prefill from an empty cache.

    cache/nats_chunk_layer_cache.py:589-620 with chunk_fill_size == x_len == L."""
    vis = expand_chunk_mask(chunk_visibility(roles, W // C), C)[..., :L, :L]
    return np.tril(vis)


def repeat_for_gqa(x: torch.Tensor, n_rep: int) -> torch.Tensor:
    """[B, H_kv, ...] -> [B, H_kv * n_rep, ...] (models/transformer/utils.py:23-46)."""
    if n_rep == 1:
        return x
    return x.repeat_interleave(n_rep, dim=1)


def masked_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, mask, sm_scale: float | None = None,
                     explicit: bool = False) -> torch.Tensor:
    """q [B, H_q, Lq, D], k / v [B, H_kv, N, D], mask bool [B, H_kv, Lq, N] -> [B, H_q, Lq, D].

    attention/nats_chunk_attention.py:130-149: repeat k, v and the mask to H_q heads, then SDPA with a bool
    mask (`explicit=False`) or matmul / fp32 softmax cast back to q's dtype / matmul (`explicit=True`)."""
    n_rep = q.shape[1] // k.shape[1]
    mask_t = torch.as_tensor(mask)
    k_r, v_r, m_r = repeat_for_gqa(k, n_rep), repeat_for_gqa(v, n_rep), repeat_for_gqa(mask_t, n_rep)
    D = q.shape[-1]
    scale = (1.0 / math.sqrt(D)) if sm_scale is None else sm_scale
    if not explicit:
        return torch.nn.functional.scaled_dot_product_attention(q, k_r, v_r, attn_mask=m_r, is_causal=False,
                                                                scale=scale)
    scores = torch.matmul(q, k_r.transpose(2, 3)) * scale
    scores = scores.float().masked_fill(~m_r, float("-inf"))
    p = torch.softmax(scores, dim=-1).type_as(q)
    return torch.matmul(p, v_r)


def decode_attention(q: torch.Tensor, cache_k: torch.Tensor, cache_v: torch.Tensor, valid: torch.Tensor,
                     n_rows: int, sm_scale: float | None = None) -> torch.Tensor:
    """One query token per sequence over the evicted cache: softmax over the rows flagged valid.

    cache/nats_chunk_layer_cache.py:622-632 (mask = valid_tokens[:, :, :n_ctx_data + 1]) followed by SDPA;
    restated as gather-valid-rows-then-dense-softmax per (b, kv-head) in fp32."""
    B, Hq, one, D = q.shape
    Hkv = cache_k.shape[1]
    n_rep = Hq // Hkv
    scale = (1.0 / math.sqrt(D)) if sm_scale is None else sm_scale
    out = torch.zeros(B, Hq, 1, D, dtype=torch.float32)
    for b in range(B):
        for h in range(Hkv):
            idx = torch.nonzero(valid[b, h, :n_rows]).flatten()
            kk = cache_k[b, h, idx].float()
            vv = cache_v[b, h, idx].float()
            qq = q[b, h * n_rep:(h + 1) * n_rep, 0].float()
            s = (qq @ kk.T) * scale
            p = torch.softmax(s, dim=-1)
            out[b, h * n_rep:(h + 1) * n_rep, 0] = p @ vv
    return out.to(q.dtype)


# ----------------------------------------------------------------------------------------------
# tile-level accounting used by the benchmark and the tile-map tests
# ----------------------------------------------------------------------------------------------
def visited_tiles(roles: np.ndarray, window_chunks: int) -> np.ndarray:
    """bool [B, H, S, S]: (q-chunk m, k-chunk n) pairs that hold at least one unmasked score."""
    vis = chunk_visibility(roles, window_chunks)
    S = roles.shape[-1]
    return vis & np.tril(np.ones((S, S), dtype=bool))


# ----------------------------------------------------------------------------------------------
# the chunked layer cache as an explicit state machine
# ----------------------------------------------------------------------------------------------
@dataclass
class ChunkCacheOracle:
    """State of one layer (cache/nats_chunk_layer_cache.py:16-77).

    `pos_k` shadows cache_k with the stream position of the token each row holds (-1 = no token); it is
    the surviving-token index map the reference does not keep."""
    B: int
    H: int
    W: int
    C: int
    size_global: np.ndarray = field(init=False)
    size_local: np.ndarray = field(init=False)
    n_ctx_data: int = field(init=False)
    gmin: int = field(init=False)
    tail: int = 0
    fill: int = 0
    fill_last: int = 0
    seen: int = 0
    cache_k: torch.Tensor | None = None
    cache_v: torch.Tensor | None = None
    pos_k: np.ndarray | None = None
    valid: np.ndarray | None = None
    roles: np.ndarray | None = None  # roles handed over by the last update

    def __post_init__(self):
        assert self.W % self.C == 0  # :47
        self.size_global = np.full((self.B, self.H), self.W, dtype=np.int64)
        self.size_local = np.zeros((self.B, self.H), dtype=np.int64)
        self.n_ctx_data = self.W
        self.gmin = self.W

    # -- append ---------------------------------------------------------------------------------
    def update(self, k: torch.Tensor, v: torch.Tensor, roles: np.ndarray | None):
        """:171-256.  Returns the K, V the attention of this call runs over."""
        B, H, x_len, D = k.shape
        self.fill += x_len
        if x_len == 0:
            return self.cache_k[:, :, :self.n_ctx_data], self.cache_v[:, :, :self.n_ctx_data]
        self.roles = None if roles is None else np.array(roles, dtype=np.uint8)
        if self.cache_k is None:
            pad = (-x_len) % self.C
            rows = self.W + x_len + pad
            self.cache_k = torch.zeros(B, H, rows, D, dtype=k.dtype)
            self.cache_v = torch.zeros(B, H, rows, D, dtype=v.dtype)
            self.cache_k[:, :, self.W:self.W + x_len] = k
            self.cache_v[:, :, self.W:self.W + x_len] = v
            self.valid = np.zeros((B, H, rows), dtype=bool)
            self.valid[:, :, self.W:self.W + x_len] = True
            self.pos_k = np.full((B, H, rows), -1, dtype=np.int64)
            self.pos_k[:, :, self.W:self.W + x_len] = np.arange(self.seen, self.seen + x_len)
            return k, v
        start = self.n_ctx_data
        end = start + x_len
        need = math.ceil(end / self.C) * self.C
        have = self.cache_k.shape[2]
        if need > have:
            grow = need - have
            self.cache_k = torch.cat([self.cache_k, torch.zeros(B, H, grow, D, dtype=self.cache_k.dtype)], 2)
            self.cache_v = torch.cat([self.cache_v, torch.zeros(B, H, grow, D, dtype=self.cache_v.dtype)], 2)
            self.valid = np.concatenate([self.valid, np.zeros((B, H, grow), dtype=bool)], 2)
            self.pos_k = np.concatenate([self.pos_k, np.full((B, H, grow), -1, dtype=np.int64)], 2)
        self.cache_k[:, :, start:end] = k.to(self.cache_k.dtype)
        self.cache_v[:, :, start:end] = v.to(self.cache_v.dtype)
        self.valid[:, :, start:end] = True
        self.pos_k[:, :, start:end] = np.arange(self.seen, self.seen + x_len)
        return self.cache_k[:, :, :end], self.cache_v[:, :, :end]

    # -- masks ----------------------------------------------------------------------------------
    def _new_token_mask(self, x_len: int):
        """:589-620.  Rows = the x_len new tokens, columns = the open chunk region [base, base + fill)."""
        fill = self.fill
        if self.roles is None:
            roles = np.zeros((self.B, self.H, 1), dtype=np.uint8)
        else:
            roles = self.roles
        vis = chunk_visibility(roles, self.W // self.C)
        g = next_global_index(roles == ROLE_GLOBAL)
        tok = expand_chunk_mask(vis, self.C)[:, :, fill - x_len:fill, :fill]
        rows = np.arange(fill - x_len, fill)[:, None]
        cols = np.arange(tok.shape[-1])[None, :]
        return tok & (cols <= rows), g

    def generate_mask(self, x_len: int) -> np.ndarray:
        """:156-163, :444-511.  Bool [B, H, x_len, n_ctx_data + x_len] (or [.., x_len, x_len] from empty)."""
        if x_len == 1:
            if self.seen == 0:  # :628-629
                return np.ones((1, 1, 1, 1), dtype=bool)
            return self.valid[:, :, None, :self.n_ctx_data + 1].copy()  # :631
        new_mask, g = self._new_token_mask(x_len)
        if self.seen == 0 or self.valid.shape[-1] == 0:
            return new_mask
        C, W = self.C, self.W
        wc = W // C
        old_fill = self.fill - x_len
        base = self.n_ctx_data - self.fill + x_len  # :466, first row of the open chunk region
        cached = np.repeat(self.valid[:, :, None, :base], x_len, axis=2).copy()
        # ring columns age with the query position (:658-713)
        q_chunk = (np.arange(old_fill, self.fill) + self.fill_last) // C  # :666-667 (fill_last added again)
        seen_chunks = self.seen // C
        if self.seen < W:
            ncol = seen_chunks * C
            j = np.arange(ncol) // C  # ring slot counted from slot 0
            ok = (q_chunk[:, None] + j[None, :]) < wc  # :676
            cached[:, :, :, :ncol] &= ok[None, None]
        else:
            slot = np.arange(W) // C
            newest_row = ((slot + 1) * C + W - 1 - self.tail) % W  # queue offset of each slot's last row
            ok = np.zeros((x_len, W), dtype=bool)
            for i in range(x_len):
                r = old_fill + i  # offset of the query inside the open chunk region
                if r < W:  # :687-707, rows beyond the window see no ring slot
                    ok[i] = newest_row >= r
            cached[:, :, :, :W] &= ok[None, None]
        # cached local chunks are visible up to the first new global slot (:480-494, :510)
        gmin = self.gmin
        ncc = (base - gmin) // C
        q_slot = np.arange(old_fill, self.fill) // C
        for b in range(self.B):
            for h in range(self.H):
                lo = (self.size_global[b, h] - gmin) // C
                hi = (self.size_global[b, h] + self.size_local[b, h] - gmin) // C
                for cc in range(ncc):
                    if cc >= hi:
                        col = np.zeros(x_len, dtype=bool)
                    elif cc < lo:
                        col = np.ones(x_len, dtype=bool)
                    else:
                        col = q_slot <= g[b, h, 0]
                    cached[b, h, :, gmin + cc * C:gmin + (cc + 1) * C] = col[:, None]
        return np.concatenate([cached, new_mask], axis=-1)

    # -- evict + compact ------------------------------------------------------------------------
    def post_update(self, x_len: int):
        """:262-389."""
        C, W, B, H = self.C, self.W, self.B, self.H
        self.seen += x_len
        if x_len == 0 or self.fill < C:  # chunk still open (:264-268)
            self.fill_last = self.fill
            self.n_ctx_data += x_len
            return
        partial = self.fill % C
        n_done = self.fill // C
        off = self.n_ctx_data // C  # cache chunk that holds role slot 0
        roles = self.roles
        S = roles.shape[-1]
        assert S == n_done + (1 if partial else 0), "one role slot per (possibly open) chunk"
        first = self.seen == x_len

        # 1. ring insert (:391-437): the last min(n_done, W/C) completed chunks enter the ring
        n_ring = min(n_done, W // C)
        start = 0 if first else self.tail
        for i in range(n_ring * C):
            slot = n_done - n_ring + i // C
            src = (off + n_done - n_ring) * C + i
            dst = (start + i) % W
            is_sw = roles[:, :, slot] == ROLE_SW  # [B, H]
            for b in range(B):
                for h in range(H):
                    if is_sw[b, h]:
                        self.cache_k[b, h, dst] = self.cache_k[b, h, src]
                        self.cache_v[b, h, dst] = self.cache_v[b, h, src]
                        self.pos_k[b, h, dst] = self.pos_k[b, h, src]
                    else:
                        self.cache_k[b, h, dst] = 0
                        self.cache_v[b, h, dst] = 0
                        self.pos_k[b, h, dst] = -1
                    self.valid[b, h, dst] = is_sw[b, h]
        self.tail = (start + n_ring * C) % W
        self.fill = partial
        self.fill_last = partial

        # 2. every new slot sliding-window: only the live length changes (:283-288)
        if (roles == ROLE_SW).all():
            self.n_ctx_data = int((self.size_global + self.size_local).max()) + self.fill
            return

        if x_len == 1:
            # 3a. one completed chunk, scattered for every head (:289-330)
            snap_k = self.cache_k[:, :, off * C:(off + 1) * C].clone()
            snap_v = self.cache_v[:, :, off * C:(off + 1) * C].clone()
            snap_p = self.pos_k[:, :, off * C:(off + 1) * C].copy()
            for b in range(B):
                for h in range(H):
                    r0 = roles[b, h, 0]
                    r_last = roles[b, h, -1]
                    sg, sl = int(self.size_global[b, h]), int(self.size_local[b, h])
                    dst = sg if r0 == ROLE_GLOBAL else sg + sl
                    self.cache_k[b, h, dst:dst + C] = snap_k[b, h]
                    self.cache_v[b, h, dst:dst + C] = snap_v[b, h]
                    self.pos_k[b, h, dst:dst + C] = snap_p[b, h]
                    dec = (sl // C + 1) if r0 == ROLE_GLOBAL else 0
                    dec += 1 if r_last == ROLE_SW else 0
                    if r0 == ROLE_GLOBAL:
                        self.size_global[b, h] += C
                    self.size_local[b, h] -= dec * C
        elif not (roles == ROLE_LOCAL).all():
            # 3b. general path (:715-868 + cache_update.py:25-76)
            last_excluded = partial != 0
            plans = {}
            max_keep = 0
            max_end = None
            for b in range(B):
                for h in range(H):
                    sg, sl = int(self.size_global[b, h]), int(self.size_local[b, h])
                    r = roles[b, h]
                    n_glob = int((r == ROLE_GLOBAL).sum())
                    glob_slots = [s for s in range(S) if r[s] == ROLE_GLOBAL]
                    if last_excluded:  # :782-786
                        n_glob -= 1
                        glob_slots = [s for s in glob_slots if s != S - 1]
                    last_g = glob_slots[-1] if glob_slots else -1
                    later_local = [s for s in range(S) if s > last_g and r[s] == ROLE_LOCAL]
                    n_other = S - max(last_g, 0) - len(later_local) - (1 if last_excluded else 0)  # :797-800
                    dec_local = (last_g * C + sl if last_g > -1 else 0) + n_other * C
                    keep = sorted(set(glob_slots) | set(later_local))
                    if last_excluded:  # :809-811
                        keep = [s for s in keep if s != S - 1]
                    dst_base = (sg + sl) // C if last_g == -1 else sg // C  # :827-828
                    plans[(b, h)] = (keep, dst_base, n_glob * C, dec_local)
                    max_keep = max(max_keep, len(keep))
                    end = len(keep) + dst_base
                    max_end = end if max_end is None else max(max_end, end)
            moves = []  # (b, h, src_chunk, dst_chunk), all gathered before any is written
            for (b, h), (keep, dst_base, _, _) in plans.items():
                for rank, s in enumerate(keep):
                    moves.append((b, h, s + off, dst_base + rank))
            if last_excluded and max_keep < S - 1:  # :840-857, the open chunk follows the longest head
                for b in range(B):
                    for h in range(H):
                        moves.append((b, h, S - 1 + off, max_end))
            if moves:  # cache_update.py:51-52 returns untouched when nothing is kept
                stash = [(self.cache_k[b, h, s * C:(s + 1) * C].clone(),
                          self.cache_v[b, h, s * C:(s + 1) * C].clone(),
                          self.pos_k[b, h, s * C:(s + 1) * C].copy()) for (b, h, s, _) in moves]
                for (b, h, _, d), (kk, vv, pp) in zip(moves, stash):
                    self.cache_k[b, h, d * C:(d + 1) * C] = kk
                    self.cache_v[b, h, d * C:(d + 1) * C] = vv
                    self.pos_k[b, h, d * C:(d + 1) * C] = pp
            for (b, h), (_, _, inc_g, dec_l) in plans.items():
                self.size_global[b, h] += inc_g
                self.size_local[b, h] -= dec_l

        # 4. bookkeeping shared by both paths (:356-385)
        self.size_local += n_done * C
        assert not (self.size_local < 0).any()
        self.n_ctx_data = int((self.size_global + self.size_local).max()) + self.fill
        self.cache_k[:, :, self.n_ctx_data:] = 0
        self.cache_v[:, :, self.n_ctx_data:] = 0
        self.pos_k[:, :, self.n_ctx_data:] = -1
        old_gmin = self.gmin  # :644 uses the minimum from before this call
        if self.n_ctx_data != old_gmin:
            last_chunk = self.n_ctx_data // C * C
            idx = np.arange(old_gmin, last_chunk)
            end = (self.size_global + self.size_local)[:, :, None]
            self.valid[:, :, old_gmin:last_chunk] = idx[None, None, :] < end
            self.valid[:, :, last_chunk:last_chunk + self.fill] = True
        self.gmin = int(self.size_global.min())
        if first:  # :373-380
            keep_rows = math.ceil(self.n_ctx_data / C) * C
            self.cache_k = self.cache_k[:, :, :keep_rows]
            self.cache_v = self.cache_v[:, :, :keep_rows]
            self.valid = self.valid[:, :, :keep_rows]
            self.pos_k = self.pos_k[:, :, :keep_rows]

    # -- derived observables --------------------------------------------------------------------
    def surviving_positions(self, b: int, h: int) -> np.ndarray:
        """Stream positions of the rows a decode step would attend to, in cache order."""
        n = self.n_ctx_data
        return self.pos_k[b, h, :n][self.valid[b, h, :n]]


# ----------------------------------------------------------------------------------------------
# the per-token layer cache (chunk_size == 1) as an explicit state machine
# ----------------------------------------------------------------------------------------------
@dataclass
class TokenCacheOracle:
    """State of one layer of the reference's per-token cache, NAtSLayerCache
    (cache/nats_layer_cache.py:20-80): a role per token, rows appended at once, eviction deferred until
    `U` (update_chunk_size, 16 as the container builds it) tokens are pending.

    Row layout of cache_k[b, h] between calls:
        [0, W)                      ring of the last W tokens that went through an eviction; `tail` is the slot
                                    written last; a slot is valid iff its token was sliding-window (its row is
                                    copied whatever the role)
        [W, size_global)            global tokens, stream order
        [size_global, +size_local)  local tokens newer than the last global token
        [.., P)                     stale rows of shorter heads (and the still-valid rows of pending blocks whose
                                    tokens were all sliding-window, which the reference leaves where they were)
        [P, P + fill)               the pending block, valid, P + fill = n_ctx_data
    Rows at and beyond n_ctx_data keep whatever they held (nothing is zeroed).
    `pos_k` shadows cache_k with the stream position of the token each row holds (-1 = none)."""
    B: int
    H: int
    W: int
    U: int = 16
    size_global: np.ndarray = field(init=False)
    size_local: np.ndarray = field(init=False)
    n_ctx_data: int = field(init=False)
    gmin: int = field(init=False)
    tail: int = 0
    fill: int = 0
    fill_last: int = 0
    seen: int = 0
    cache_k: torch.Tensor | None = None
    cache_v: torch.Tensor | None = None
    pos_k: np.ndarray | None = None
    valid: np.ndarray | None = None
    block: np.ndarray | None = None       # roles of the pending block, [B, H, fill] (:209-219, _tokens_info)
    mask_roles: np.ndarray | None = None  # the block as of the last multi-token update (:229-231)

    def __post_init__(self):
        if self.W < self.U:  # :77-78
            raise NotImplementedError("The sliding window size must be greater or equal to the update chunk size!")
        if self.U == 1 and self.W < 2:
            # :344 writes ring slot 1 at the first one-token call without reducing it modulo W: with W == 1 that is the
            # token's own row, outside the ring
            raise NotImplementedError("update_chunk_size == 1 is restated for windows of at least two tokens")
        self.size_global = np.full((self.B, self.H), self.W, dtype=np.int64)
        self.size_local = np.zeros((self.B, self.H), dtype=np.int64)
        self.n_ctx_data = self.W
        self.gmin = self.W
        self._in_chunk = np.zeros((self.B, self.H, self.U), dtype=np.uint8)

    # -- append (:167-286) ------------------------------------------------------------------------
    def update(self, k: torch.Tensor, v: torch.Tensor, roles: np.ndarray):
        """roles uint8 [B, H, x_len], one per new token.  Returns the K, V the attention of this call runs over."""
        B, H, x_len, D = k.shape
        if x_len == 0:  # :204-205
            return self.cache_k[:, :, :self.n_ctx_data], self.cache_v[:, :, :self.n_ctx_data]
        roles = np.asarray(roles, dtype=np.uint8)
        assert roles.shape == (B, H, x_len)
        self.fill += x_len
        if self.fill > self.U:  # :209-215
            self.block = np.concatenate([self._in_chunk[:, :, :self.fill_last], roles], axis=2)
        else:  # :217-219
            self._in_chunk[:, :, self.fill_last:self.fill] = roles
            self.block = self._in_chunk[:, :, :self.fill].copy()
        if x_len > 1:  # :229-231
            self.mask_roles = self.block.copy()
        if self.cache_k is None:  # :236-259
            pad = (-x_len) % self.U
            rows = self.W + x_len + pad
            self.cache_k = torch.zeros(B, H, rows, D, dtype=k.dtype)
            self.cache_v = torch.zeros(B, H, rows, D, dtype=v.dtype)
            self.cache_k[:, :, self.W:self.W + x_len] = k
            self.cache_v[:, :, self.W:self.W + x_len] = v
            self.valid = np.zeros((B, H, rows), dtype=bool)
            self.valid[:, :, self.W:self.W + x_len] = True
            self.pos_k = np.full((B, H, rows), -1, dtype=np.int64)
            self.pos_k[:, :, self.W:self.W + x_len] = np.arange(self.seen, self.seen + x_len)
            return k, v
        start = self.n_ctx_data  # :265-286
        end = start + x_len
        need = math.ceil(end / self.U) * self.U
        have = self.cache_k.shape[2]
        if need > have:
            grow = need - have
            self.cache_k = torch.cat([self.cache_k, torch.zeros(B, H, grow, D, dtype=self.cache_k.dtype)], 2)
            self.cache_v = torch.cat([self.cache_v, torch.zeros(B, H, grow, D, dtype=self.cache_v.dtype)], 2)
            self.valid = np.concatenate([self.valid, np.zeros((B, H, grow), dtype=bool)], 2)
            self.pos_k = np.concatenate([self.pos_k, np.full((B, H, grow), -1, dtype=np.int64)], 2)
        self.cache_k[:, :, start:end] = k.to(self.cache_k.dtype)
        self.cache_v[:, :, start:end] = v.to(self.cache_v.dtype)
        self.valid[:, :, start:end] = True
        self.pos_k[:, :, start:end] = np.arange(self.seen, self.seen + x_len)
        return self.cache_k[:, :, :end], self.cache_v[:, :, :end]

    # -- masks ------------------------------------------------------------------------------------
    def _block_mask(self, start: int):
        """:519-542.  Rows = block tokens [start, fill), columns = block tokens [0, fill)."""
        roles = self.mask_roles
        fill = roles.shape[-1]
        g = next_global_index(roles == ROLE_GLOBAL)
        any_sw = bool((roles == ROLE_SW).any())
        m = np.arange(start, fill)[:, None]
        n = np.arange(fill)[None, :]
        out = np.zeros((self.B, self.H, fill - start, fill), dtype=bool)
        for b in range(self.B):
            for h in range(self.H):
                r = roles[b, h]
                is_g = (r == ROLE_GLOBAL) | (np.arange(fill) == fill - 1)
                vis = (g[b, h][None, :] >= m) | is_g[None, :]  # masks/utils.py:92
                if any_sw:
                    vis = np.where((r == ROLE_SW)[None, :], (m - n) <= self.W, vis)  # :527-536
                out[b, h] = vis & (n <= m)  # :538
        return out, g

    def generate_mask(self, x_len: int) -> np.ndarray:
        """:155-162, :469-517.  Bool [B, H, x_len, n_ctx_data + x_len] (or [.., x_len, x_len] from empty)."""
        if x_len == 1:
            if self.seen == 0:  # :550-551
                return np.ones((1, 1, 1, 1), dtype=bool)
            return self.valid[:, :, None, :self.n_ctx_data + 1].copy()  # :553
        start = self.fill - x_len  # :159
        new_mask, g = self._block_mask(start)
        if self.seen == 0 or self.valid.shape[-1] == 0:  # :484-488
            return new_mask
        W = self.W
        P = self.n_ctx_data - self.fill_last  # :490, first row of the pending block
        cached = np.repeat(self.valid[:, :, None, :P], x_len, axis=2).copy()
        i = np.arange(x_len)[:, None]  # the query's index within this call, not within the block
        if self.seen < W:  # :612-619: the columns of the tokens seen so far are overwritten, valid or not
            j = np.arange(self.seen)[None, :]
            cached[:, :, :, :self.seen] = ((i + j) < W)[None, None]
        else:  # :621-647: slot tail + 1 is the oldest and is seen by the first query only
            age = (np.arange(W) + W - 1 - self.tail) % W
            ok = (age[None, :] >= i) & (i < W)
            cached[:, :, :, :W] &= ok[None, None]
        gmin = self.gmin  # :502-516: cached local tokens live until the first global token of the block
        for b in range(self.B):
            for h in range(self.H):
                lo = self.size_global[b, h] - gmin
                hi = self.size_global[b, h] + self.size_local[b, h] - gmin
                col_local = (np.arange(x_len) <= g[b, h, 0])
                for c in range(gmin, P):
                    t = c - gmin
                    if t >= hi:
                        cached[b, h, :, c] = False
                    elif t >= lo:
                        cached[b, h, :, c] = col_local
                    else:
                        cached[b, h, :, c] = True
        return np.concatenate([cached, new_mask], axis=-1)

    # -- evict + compact (:292-418) ---------------------------------------------------------------
    def _ring_insert(self):
        """:424-458.  The last min(fill, W) tokens of the pending block enter the ring, rows copied whatever the
        role, valid only if sliding-window."""
        W, n = self.W, self.n_ctx_data
        x_sw = min(self.fill, W)
        if self.fill == self.seen:
            slots = np.arange(x_sw)
            self.tail = x_sw - 1
        else:
            slots = (np.arange(x_sw) + self.tail + 1) % W
            self.tail = (self.tail + x_sw) % W
        self.valid[:, :, slots] = self.block[:, :, -x_sw:] == ROLE_SW
        self.cache_k[:, :, slots] = self.cache_k[:, :, n - x_sw:n].clone()
        self.cache_v[:, :, slots] = self.cache_v[:, :, n - x_sw:n].clone()
        self.pos_k[:, :, slots] = self.pos_k[:, :, n - x_sw:n].copy()

    def post_update(self, x_len: int):
        B, H, W, U = self.B, self.H, self.W, self.U
        self.seen += x_len
        if x_len == 0:
            return
        self.n_ctx_data += x_len
        if self.fill < U:  # :300-310: the eviction is deferred, one ring slot is switched off
            slot = self.fill if self.seen < U else (self.fill + self.tail + 1) % W
            self.valid[:, :, slot] = False
            self.fill_last = self.fill
            return
        block = self.block
        fill = self.fill
        assert block.shape[-1] == fill
        if (block == ROLE_SW).all():  # :316-327: rows and n_ctx_data stay as they are
            self._ring_insert()
            self.fill = self.fill_last = 0
            return
        if x_len == 1 and U == 1:  # :328-367: the one-step branch, every head scatters its one token
            self._one_step(block[:, :, 0])
        else:
            self._ring_insert()
            self._merge_block(block, fill)
        self.size_local += fill  # :393
        assert not (self.size_local < 0).any()
        self.n_ctx_data = int((self.size_global + self.size_local).max())  # :394
        old_gmin = self.gmin  # :565 uses the minimum from before this call
        if self.n_ctx_data != old_gmin:
            idx = np.arange(old_gmin, self.n_ctx_data)
            end = (self.size_global + self.size_local)[:, :, None]
            self.valid[:, :, old_gmin:self.n_ctx_data] = idx[None, None, :] < end
        self.gmin = int(self.size_global.min())
        if self.seen == x_len:  # :404-408
            n = self.n_ctx_data
            self.cache_k, self.cache_v = self.cache_k[:, :, :n], self.cache_v[:, :, :n]
            self.valid, self.pos_k = self.valid[:, :, :n], self.pos_k[:, :, :n]
        self.fill = self.fill_last = 0

    def _one_step(self, role: np.ndarray):
        """:328-367 (update_chunk_size == 1, one new token, not sliding-window on every head).  The token's row
        (n_ctx_data - 1, where update() put it) is written to ring slot tail + 2 (slot 1 for the first token ever;
        `tail` itself advances by one, :340-345) and to row size_global (a global token, which thereby drops the
        head's local rows) or size_global + size_local (local and sliding-window tokens alike); the slot is valid iff
        the token is sliding-window.  The sizes are left so that the common `size_local += 1` (:393) completes them."""
        W, src = self.W, self.n_ctx_data - 1
        if self.seen == 1:
            slot, self.tail = 1, 0
        else:
            slot = (1 + self.tail + 1) % W
            self.tail = (self.tail + 1) % W
        is_g = role == ROLE_GLOBAL
        is_sw = role == ROLE_SW
        dst = np.where(is_g, self.size_global, self.size_global + self.size_local)  # :335-337
        self.valid[:, :, slot] = is_sw  # :347
        new_k, new_v, new_p = self.cache_k[:, :, src].clone(), self.cache_v[:, :, src].clone(), self.pos_k[:, :, src].copy()
        for b in range(self.B):
            for h in range(self.H):
                for row in (int(dst[b, h]), slot):  # :351-355
                    self.cache_k[b, h, row] = new_k[b, h]
                    self.cache_v[b, h, row] = new_v[b, h]
                    self.pos_k[b, h, row] = new_p[b, h]
        dec_local = np.where(is_g, self.size_local + 1, 0) + is_sw  # :357-361
        self.size_global = self.size_global + is_g  # :365
        self.size_local = self.size_local - dec_local  # :366

    def _merge_block(self, block: np.ndarray, fill: int):
        B, H = self.B, self.H
        if not (block == ROLE_LOCAL).all():  # :651-770 + cache_update.py:25-76 (chunk_size 1)
            P = self.n_ctx_data - fill  # :759
            moves = []
            new_sizes = {}
            for b in range(B):
                for h in range(H):
                    r = block[b, h]
                    sg, sl = int(self.size_global[b, h]), int(self.size_local[b, h])
                    glob = [s for s in range(fill) if r[s] == ROLE_GLOBAL]
                    last_g = glob[-1] if glob else -1
                    later_local = [s for s in range(fill) if s > last_g and r[s] == ROLE_LOCAL]
                    dec_local = (last_g + sl if last_g > -1 else 0) + (fill - max(last_g, 0) - len(later_local))  # :723-729
                    keep = sorted(glob + later_local)
                    base = sg + sl if last_g == -1 else sg  # :748-749
                    for rank, s in enumerate(keep):
                        moves.append((b, h, P + s, base + rank))
                    new_sizes[(b, h)] = (sg + len(glob), sl - dec_local)
            stash = [(self.cache_k[b, h, s].clone(), self.cache_v[b, h, s].clone(), self.pos_k[b, h, s])
                     for (b, h, s, _) in moves]
            for (b, h, _, d), (kk, vv, pp) in zip(moves, stash):
                self.cache_k[b, h, d] = kk
                self.cache_v[b, h, d] = vv
                self.pos_k[b, h, d] = pp
            for (b, h), (sg, sl) in new_sizes.items():
                self.size_global[b, h] = sg
                self.size_local[b, h] = sl


def kept_token_fraction(cache: ChunkCacheOracle) -> float:
    """Mean retained-KV fraction as the reference's benchmark reports it
    (experiments/efficiency/eval_efficiency.py:349-355)."""
    kept = cache.size_global + cache.size_local + cache.fill
    return float(kept.mean()) / max(cache.seen, 1)
