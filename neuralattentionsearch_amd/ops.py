"""Torch-tensor front end of the C ABI: the operator level of the NAtS inference path.

Every function takes CUDA (ROCm) tensors, passes raw pointers / strides / the current stream to
libnats_hip.so and returns tensors.  Nothing here computes on the CPU and nothing falls back to PyTorch
ops: CPU tensors are rejected.
"""
from __future__ import annotations

import collections
import ctypes
import math
import time
import weakref

import torch

from . import _lib
from ._lib import NATS_DTYPE_BF16, NATS_DTYPE_F32, EvictParams, EvictResult, PastState, check, i64_array

EvictBrief = collections.namedtuple("EvictBrief", "n_ctx_data gmin all_sw all_local")  # nats_evict_brief without its seq

ROLE_GLOBAL, ROLE_LOCAL, ROLE_SW = 0, 1, 2
TILE = 64

# scratch buffers by (device, raw stream handle, purpose), least recently used first; at most _WORKSPACE_SLOTS of them
_workspaces: "collections.OrderedDict" = collections.OrderedDict()
_WORKSPACE_SLOTS = 32


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(t: torch.Tensor):
    """The current stream of t's device as the handle the library takes."""
    if _raw_stream is not None:
        idx = t.device.index
        return _raw_stream(idx if idx is not None else torch.cuda.current_device()) or None
    return torch.cuda.current_stream(t.device).cuda_stream or None


def _ptr(t: torch.Tensor | None):
    """Device address for a `void*` parameter (ctypes converts the integer; None is NULL)."""
    return None if t is None else t.data_ptr()


def strides_differ(a: torch.Tensor, b: torch.Tensor, dims: int | None = None) -> bool:
    """Whether two tensors of one shape are laid out differently (a dimension of size 1 may carry any stride)."""
    return any(sa != sb for sa, sb, n in list(zip(a.stride(), b.stride(), a.shape))[:dims] if n != 1)


def _dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.bfloat16:
        return NATS_DTYPE_BF16
    if t.dtype == torch.float32:
        return NATS_DTYPE_F32
    raise ValueError(f"unsupported dtype {t.dtype}: the kernels take bfloat16 or float32")


def _require_cuda(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise ValueError("the NAtS kernels run on the GPU only: got a CPU tensor")


def workspace(device, key: str, nbytes: int) -> torch.Tensor:
    """A scratch buffer per (device, current stream, purpose) that only ever grows.

    Calls of one purpose on one stream share the buffer, which the stream orders; calls on different streams (two
    prefills side by side, a worker thread under the caller's stream) get buffers of their own.  The table keeps the
    _WORKSPACE_SLOTS entries used last: a process that creates streams without end does not keep a buffer for every
    stream it ever had (a dropped buffer goes back to torch's allocator, which orders its reuse after the work
    queued on it)."""
    device = torch.device(device)
    idx = device.index if device.index is not None else torch.cuda.current_device()
    handle = _raw_stream(idx) if _raw_stream is not None else torch.cuda.current_stream(device).cuda_stream
    k = (idx, int(handle or 0), key)
    buf = _workspaces.get(k)
    if buf is None or buf.numel() < nbytes:
        buf = torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)
        _workspaces[k] = buf
        while len(_workspaces) > _WORKSPACE_SLOTS:
            _workspaces.popitem(last=False)
    _workspaces.move_to_end(k)
    return buf


# ------------------------------------------------------------------------------------------------
# roles
# ------------------------------------------------------------------------------------------------
def roles_from_logits(logits: torch.Tensor, global_bias: float = 0.1, force_first_global: bool = False,
                      force_last_global: bool = False, with_one_hot: bool = True):
    """logits [B, S, H_kv, 3] -> (roles uint8 [B, H_kv, S], token_states_info [B, H_kv, S, 3] or None).

    models/transformer/attention/nats_attention.py:96-109."""
    _require_cuda(logits)
    lib = _lib.load()
    if logits.dim() != 4 or logits.shape[-1] != 3:
        raise ValueError(f"logits must be [B, S, H_kv, 3], got {tuple(logits.shape)}")
    logits = logits.contiguous()
    B, S, H, _ = logits.shape
    roles = torch.empty(B, H, S, dtype=torch.uint8, device=logits.device)
    one_hot = torch.empty(B, H, S, 3, dtype=logits.dtype, device=logits.device) if with_one_hot else None
    check(lib.nats_roles_from_logits(_ptr(logits), _dtype_code(logits), B, S, H, float(global_bias),
                                     int(force_first_global), int(force_last_global), _ptr(roles), _ptr(one_hot),
                                     _stream(logits)))
    if one_hot is not None:
        _attach_roles(one_hot, roles)  # whoever receives only the one-hot tensor finds the compact form on it
    return roles, one_hot


def role_step(x: torch.Tensor, weight: torch.Tensor, chunk_size: int, window: int, pre_fill: int = 0,
              carry_in: torch.Tensor | None = None, merge_max: bool = False, global_bias: float = 0.1,
              force_first_global: bool = False, with_one_hot: bool = True, with_logits: bool = False,
              with_scan: bool = False, roles_out: torch.Tensor | None = None) -> dict:
    """Chunk pooling of hidden states + role projection + argmax (+ next-global scan) in one call.

    x [B, L, dim] hidden states of the new tokens, weight [H_kv * 3, dim] (proj_layer.weight), carry_in
    [B, 1, dim] or [B, dim] the running statistic of the open chunk (required when pre_fill > 0).
    Returns a dict with `roles` uint8 [B, H_kv, S] (None while no chunk completes), `token_states_info`,
    `logits` [B, S, H_kv, 3], `carry` [B, 1, dim] (statistic of the open chunk, None if every chunk is
    complete), `end_idx`, `vis_lim`, and `pad`.  `roles_out`: a uint8 [B, H_kv, S] view into which the roles are
    written instead of a new tensor (its last dimension contiguous, its first two laid out as those of a contiguous
    [B, H_kv, U] tensor: a slice of the per-token cache's pending roles); not together with `with_scan`.
    components/cache/dyn_cache.py:117-171, models/transformer/attention/nats_chunk_attention.py:64-95."""
    _require_cuda(x, weight, carry_in)
    lib = _lib.load()
    if x.dim() != 3 or weight.dim() != 2 or weight.shape[1] != x.shape[2] or weight.shape[0] % 3 != 0:
        raise ValueError(f"x must be [B, L, dim] and weight [H_kv * 3, dim], got {tuple(x.shape)}, {tuple(weight.shape)}")
    if weight.dtype != x.dtype or (carry_in is not None and carry_in.dtype != x.dtype):
        raise ValueError("x, weight and carry_in must share one dtype")
    B, L, dim = x.shape
    H = weight.shape[0] // 3
    C = chunk_size
    if x.stride(-1) != 1:
        x = x.contiguous()
    weight = weight.contiguous()
    if carry_in is not None:
        if carry_in.dim() == 3 and carry_in.shape[1] != 1:
            # the reference keeps the raw rows of a first partial chunk as its max statistic (dyn_cache.py:111-112)
            if not merge_max:
                raise ValueError(f"carry_in must be [B, 1, dim] or [B, dim], got {tuple(carry_in.shape)}")
            carry_in = carry_in.max(1)[0]
        carry_in = carry_in.reshape(B, dim).contiguous()
    total = pre_fill + L
    S = 0 if total < C else math.ceil(total / C)
    pad = 0 if S == 0 else S * C - total
    dev, dt = x.device, x.dtype
    roles_hs = 0
    if roles_out is not None and S:
        hs = roles_out.stride(1)
        if (tuple(roles_out.shape) != (B, H, S) or roles_out.dtype != torch.uint8 or not roles_out.is_cuda or with_scan
                or (S > 1 and roles_out.stride(2) != 1) or hs < S or (B > 1 and roles_out.stride(0) != H * hs)):
            raise ValueError("roles_out must be a uint8 [B, H_kv, S] slice of a contiguous [B, H_kv, U] tensor")
        roles, roles_hs = roles_out, hs
    else:
        roles = torch.empty(B, H, S, dtype=torch.uint8, device=dev) if S else None
    one_hot = torch.empty(B, H, S, 3, dtype=dt, device=dev) if S and with_one_hot else None
    logits = torch.empty(B, S, H, 3, dtype=dt, device=dev) if S and with_logits else None
    carry = torch.empty(B, 1, dim, dtype=dt, device=dev) if (S == 0 or pad) else None
    end_idx = torch.empty(B, H, S, dtype=torch.int64, device=dev) if S and with_scan else None
    vis_lim = torch.empty(B, H, S, dtype=torch.int32, device=dev) if S and with_scan else None
    check(lib.nats_role_step(_ptr(x), _ptr(carry_in), _ptr(weight), _dtype_code(x), B, L, dim, H, C, window, pre_fill,
                             int(merge_max), float(global_bias), int(force_first_global), i64_array(x.stride()[:2]),
                             _ptr(roles), roles_hs, _ptr(one_hot), _ptr(logits), _ptr(carry), _ptr(end_idx), _ptr(vis_lim),
                             _stream(x)))
    if one_hot is not None:
        _attach_roles(one_hot, roles)
    return {"roles": roles, "token_states_info": one_hot, "logits": logits, "carry": carry, "end_idx": end_idx,
            "vis_lim": vis_lim, "pad": pad}


def _attach_roles(one_hot: torch.Tensor, roles: torch.Tensor) -> None:
    """The compact roles travel with the one-hot tensor they were written with, together with the version counters of
    both: an in-place edit of either afterwards (a slot forced global, a head masked) makes the pair stale."""
    one_hot.nats_roles = roles
    one_hot.nats_roles_version = (one_hot._version, roles._version)


def role_step_token(x: torch.Tensor, weight: torch.Tensor, window: int, roles_out: torch.Tensor, merge_max: bool = False,
                    global_bias: float = 0.1, force_first_global: bool = False) -> None:
    """`role_step` for one token per sequence with a role per token (chunk size 1): x [B, 1, dim] -> the roles, written
    into `roles_out` (uint8 [B, H_kv, 1], a slice of the per-token cache's pending roles, `role_destination`).  Nothing
    is allocated and nothing returned: the call a decoding loop makes once per layer and token."""
    B, L, dim = x.shape
    H = weight.shape[0] // 3
    hs = roles_out.stride(1)
    if (L != 1 or not x.is_cuda or weight.dtype != x.dtype or weight.shape[1] != dim or x.stride(-1) != 1
            or not weight.is_contiguous() or tuple(roles_out.shape) != (B, H, 1) or roles_out.dtype != torch.uint8
            or (B > 1 and roles_out.stride(0) != H * hs)):
        raise ValueError("role_step_token takes x [B, 1, dim], weight [H_kv * 3, dim] and roles_out uint8 [B, H_kv, 1]")
    check(_lib.load().nats_role_step(x.data_ptr(), None, weight.data_ptr(), _dtype_code(x), B, 1, dim, H, 1, window, 0,
                                     int(merge_max), float(global_bias), int(force_first_global), i64_array(x.stride()[:2]),
                                     roles_out.data_ptr(), hs, None, None, None, None, None, _stream(x)))


def roles_from_one_hot(token_states_info: torch.Tensor) -> torch.Tensor:
    """[B, H_kv, S, 3] one-hot float -> uint8 roles (index of the 1).  A tensor that `roles_from_logits` or
    `role_step` produced carries its roles with it; they are used while neither tensor has been written since."""
    roles = getattr(token_states_info, "nats_roles", None)
    if roles is not None and roles.shape == token_states_info.shape[:-1] and roles.device == token_states_info.device \
            and getattr(token_states_info, "nats_roles_version", None) == (token_states_info._version, roles._version):
        return roles
    return token_states_info.argmax(-1).to(torch.uint8)


def role_scan(roles: torch.Tensor, W: int, C: int):
    """roles [B, H_kv, S] -> (end_idx int64, vis_lim int32), both [B, H_kv, S].

    components/masks/utils.py:85-87."""
    _require_cuda(roles)
    lib = _lib.load()
    roles = roles.contiguous()
    B, H, S = roles.shape
    end_idx = torch.empty(B, H, S, dtype=torch.int64, device=roles.device)
    vis_lim = torch.empty(B, H, S, dtype=torch.int32, device=roles.device)
    check(lib.nats_role_scan(_ptr(roles), B, H, S, W, C, _ptr(end_idx), _ptr(vis_lim), _stream(roles)))
    return end_idx, vis_lim


def prefill_mask(roles: torch.Tensor, L: int, C: int, W: int) -> torch.Tensor:
    """Bool [B, H_kv, L, L]: the mask NAtSChunkLayerCache.generate_mask returns for a prefill from empty."""
    _require_cuda(roles)
    lib = _lib.load()
    roles = roles.contiguous()
    B, H, _ = roles.shape
    mask = torch.empty(B, H, L, L, dtype=torch.uint8, device=roles.device)
    ws = workspace(roles.device, "prefill", lib.nats_prefill_workspace_bytes(B, H, H, L, 0, C))
    check(lib.nats_prefill_mask(_ptr(roles), B, H, L, C, W, _ptr(mask), _ptr(ws), ws.numel(), _stream(roles)))
    return mask.bool()


def prefill_tile_map(roles: torch.Tensor, L: int, C: int, W: int) -> torch.Tensor:
    """Bool [B, H_kv, T, T], T = ceil(L / 64): the 64x64 tiles the prefill kernel loads."""
    _require_cuda(roles)
    lib = _lib.load()
    roles = roles.contiguous()
    B, H, _ = roles.shape
    T = (L + TILE - 1) // TILE
    tiles = torch.empty(B, H, T, T, dtype=torch.uint8, device=roles.device)
    ws = workspace(roles.device, "prefill", lib.nats_prefill_workspace_bytes(B, H, H, L, 0, C))
    check(lib.nats_prefill_tile_map(_ptr(roles), B, H, L, C, W, _ptr(tiles), _ptr(ws), ws.numel(), _stream(roles)))
    return tiles.bool()


# ------------------------------------------------------------------------------------------------
# prefill
# ------------------------------------------------------------------------------------------------
def prefill_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, roles: torch.Tensor, chunk_size: int,
                      window: int, sm_scale: float | None = None, out: torch.Tensor | None = None) -> torch.Tensor:
    """Role-masked causal attention of a prefill from an empty cache.

    q [B, H_q, L, D], k / v [B, H_kv, L, D] (any strides with a contiguous last dimension), roles uint8
    [B, H_kv, ceil(L / chunk_size)].  Returns [B, H_q, L, D] (or fills `out`, which may be strided)."""
    _require_cuda(q, k, v, roles)
    lib = _lib.load()
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        raise ValueError("q, k, v must be [B, H, L, D]")
    B, Hq, L, D = q.shape
    Hkv = k.shape[1]
    if k.shape != (B, Hkv, L, D) or v.shape != (B, Hkv, L, D):
        raise ValueError(f"shape mismatch: q {tuple(q.shape)}, k {tuple(k.shape)}, v {tuple(v.shape)}")
    if not (q.dtype == k.dtype == v.dtype):
        raise ValueError("q, k, v must share one dtype")
    S = math.ceil(L / chunk_size)
    if tuple(roles.shape) != (B, Hkv, S) or roles.dtype != torch.uint8:
        raise ValueError(f"roles must be uint8 [B, H_kv, {S}], got {roles.dtype} {tuple(roles.shape)}")
    q, k, v = (t if t.stride(-1) == 1 else t.contiguous() for t in (q, k, v))
    roles = roles.contiguous()
    if out is None:
        out = torch.empty(B, Hq, L, D, dtype=q.dtype, device=q.device)
    elif out.shape != q.shape or out.dtype != q.dtype or out.stride(-1) != 1:
        raise ValueError("out must match q in shape and dtype and have a contiguous last dimension")
    scale = (1.0 / math.sqrt(D)) if sm_scale is None else float(sm_scale)
    nbytes = lib.nats_prefill_workspace_bytes(B, Hq, Hkv, L, D, chunk_size)
    ws = workspace(q.device, "prefill", nbytes)
    check(lib.nats_prefill_fwd(_ptr(q), _ptr(k), _ptr(v), _ptr(roles), _ptr(out), B, Hq, Hkv, L, D, chunk_size, window,
                               i64_array(q.stride()[:3]), i64_array(k.stride()[:3]), i64_array(v.stride()[:3]),
                               i64_array(out.stride()[:3]), scale, _dtype_code(q), _ptr(ws), ws.numel(), _stream(q)))
    return out


def past_state(n_ctx_data: int, old_fill: int, gmin: int, tail: int, seen: int, fill_last: int,
               update_chunk: int = 0) -> PastState:
    """`update_chunk` = U > 0 describes the per-token cache (one role per token, eviction every U tokens)."""
    return PastState(int(n_ctx_data), int(old_fill), int(gmin), int(tail), int(seen), int(fill_last), int(update_chunk))


def _check_past(valid, size_global, size_local, roles, B, Hkv, x_len, C, state: PastState):
    S = math.ceil((state.old_fill + x_len) / C)
    if tuple(roles.shape) != (B, Hkv, S) or roles.dtype != torch.uint8:
        raise ValueError(f"roles must be uint8 [B, H_kv, {S}], got {roles.dtype} {tuple(roles.shape)}")
    if valid.dtype not in (torch.uint8, torch.bool) or valid.dim() != 3 or valid.shape[:2] != (B, Hkv) \
            or valid.shape[2] < state.n_ctx_data or valid.stride(2) != 1:
        raise ValueError("valid must be bool / uint8 [B, H_kv, >= n_ctx_data] with contiguous rows")
    for t in (size_global, size_local):
        if t.dtype != torch.int64 or tuple(t.shape) != (B, Hkv) or not t.is_contiguous():
            raise ValueError("size_global / size_local must be contiguous int64 [B, H_kv]")
    return S


def prefill_past_mask(valid: torch.Tensor, size_global: torch.Tensor, size_local: torch.Tensor, roles: torch.Tensor,
                      x_len: int, C: int, W: int, state: PastState) -> torch.Tensor:
    """Bool [B, H_kv, x_len, n_ctx_data + x_len]: the mask NAtSChunkLayerCache.generate_mask returns for a
    multi-token segment over a non-empty cache (components/cache/nats_chunk_layer_cache.py:462-511)."""
    _require_cuda(valid, size_global, size_local, roles)
    lib = _lib.load()
    B, Hkv = valid.shape[:2]
    roles = roles.contiguous()
    S = _check_past(valid, size_global, size_local, roles, B, Hkv, x_len, C, state)
    N = state.n_ctx_data + x_len
    mask = torch.empty(B, Hkv, x_len, N, dtype=torch.uint8, device=valid.device)
    ws = workspace(valid.device, "prefill", lib.nats_prefill_past_workspace_bytes(B, Hkv, N, S))
    valid_u8 = valid.view(torch.uint8) if valid.dtype == torch.bool else valid
    check(lib.nats_prefill_past_mask(_ptr(valid_u8), _ptr(size_global), _ptr(size_local), _ptr(roles), B, Hkv, x_len, C, W,
                                     ctypes.byref(state), i64_array(valid.stride()[:2]), _ptr(mask), _ptr(ws), ws.numel(),
                                     _stream(valid)))
    return mask.bool()


def prefill_past_attention(q: torch.Tensor, cache_k: torch.Tensor, cache_v: torch.Tensor, valid: torch.Tensor,
                           size_global: torch.Tensor, size_local: torch.Tensor, roles: torch.Tensor, chunk_size: int,
                           window: int, state: PastState, sm_scale: float | None = None) -> torch.Tensor:
    """Attention of a multi-token segment over a cache that earlier segments filled and evicted.

    q [B, H_q, x_len, D]; cache_k / cache_v [B, H_kv, >= n_ctx_data + x_len, D] with the segment already
    appended at rows [n_ctx_data, n_ctx_data + x_len); valid / size_global / size_local are the cache's
    valid_tokens, size_global_kv, size_local_kv; roles uint8 [B, H_kv, ceil((old_fill + x_len) / chunk_size)].
    Equals SDPA(q, cache_k[:, :, :N], cache_v[:, :, :N], generate_mask(x_len)) of the reference."""
    _require_cuda(q, cache_k, cache_v, valid, size_global, size_local, roles)
    lib = _lib.load()
    B, Hq, x_len, D = q.shape
    Hkv = cache_k.shape[1]
    N = state.n_ctx_data + x_len
    if cache_k.shape != cache_v.shape or cache_k.shape[0] != B or cache_k.shape[3] != D or cache_k.shape[2] < N:
        raise ValueError(f"cache_k / cache_v must be [B, H_kv, >= {N}, D], got {tuple(cache_k.shape)}, {tuple(cache_v.shape)}")
    if not (q.dtype == cache_k.dtype == cache_v.dtype):
        raise ValueError("q and the cache must share one dtype")
    if cache_k.stride(-1) != 1 or cache_v.stride(-1) != 1:
        raise ValueError("cache_k / cache_v need a contiguous last dimension")
    roles = roles.contiguous()
    S = _check_past(valid, size_global, size_local, roles, B, Hkv, x_len, chunk_size, state)
    q = q if q.stride(-1) == 1 else q.contiguous()
    out = torch.empty(B, Hq, x_len, D, dtype=q.dtype, device=q.device)
    scale = (1.0 / math.sqrt(D)) if sm_scale is None else float(sm_scale)
    ws = workspace(q.device, "prefill", lib.nats_prefill_past_workspace_bytes(B, Hkv, N, S) +
                   lib.nats_prefill_sched_workspace_bytes(B, Hq, Hkv, x_len, N))
    valid_u8 = valid.view(torch.uint8) if valid.dtype == torch.bool else valid
    check(lib.nats_prefill_past_fwd(_ptr(q), _ptr(cache_k), _ptr(cache_v), _ptr(valid_u8), _ptr(size_global),
                                    _ptr(size_local), _ptr(roles), _ptr(out), B, Hq, Hkv, x_len, D, chunk_size, window,
                                    ctypes.byref(state), i64_array(q.stride()[:3]), i64_array(cache_k.stride()[:3]),
                                    i64_array(cache_v.stride()[:3]), i64_array(valid.stride()[:2]),
                                    i64_array(out.stride()[:3]), scale, _dtype_code(q), _ptr(ws), ws.numel(), _stream(q)))
    return out


def _roles_from_kernel_arguments(end_seqs_idx: torch.Tensor, sliding_tokens: torch.Tensor) -> torch.Tensor:
    """A slot is global iff end_seqs_idx[n] == n (nats_flashattn_fwd.py:110), sliding window iff its flag is set."""
    slots = torch.arange(end_seqs_idx.shape[-1], device=end_seqs_idx.device)
    is_global = end_seqs_idx == slots
    is_sw = sliding_tokens > 0
    return torch.where(is_global, ROLE_GLOBAL, torch.where(is_sw, ROLE_SW, ROLE_LOCAL)).to(torch.uint8)


PER_TOKEN_UPDATE_CHUNK = 16  # update_chunk_size of the per-token cache as NAtSCache builds it (dyn_cache.py:183-185)


def nats_prefill(q, k, v, end_seqs_idx, sliding_tokens, sm_scale, nats_chunk_size: int = 1, global_kv_size=None,
                 local_kv_size=None, valid_sw_tokens=None, n_ctx_data=None, sw_token_tails=None, n_rep: int = 1,
                 n_tokens_in_first_chunk: int = 0, local_seq_max_length: int = 4, return_masks: bool = False,
                 block_n: int = 32, seen_tokens: int | None = None, n_global_min: int | None = None):
    """Drop-in for nats_prefill of models/transformer/triton/nats_flashattn_fwd.py:617-725 (same argument
    names and meaning, returns (o, mask or None)).

    end_seqs_idx [B, H_kv, S] int64 is the next-global index computed with the last slot forced global;
    sliding_tokens [B, H_kv, S] is option 2 of token_states_info.

    With `global_kv_size` the call is a segment over a cache that earlier segments filled (the HAS_PAST_INFO form,
    nats_flashattn_fwd.py:622-627, 476-571, called as in the reference's own smoke :925-956): k / v are the cache
    views `cache.update` returned, [B, H_kv, n_ctx_data + L_q, D]; global_kv_size / local_kv_size are the cache's
    size tensors; valid_sw_tokens [B, H_kv, W / C] = valid_tokens[..., :W:C]; n_ctx_data and sw_token_tails its
    n_ctx_data and sliding_queue_tail before the eviction of this segment; n_tokens_in_first_chunk the tokens of
    the open chunk cached before the segment.  The result is SDPA(q, k, v, cache.generate_mask(L_q)), the path
    this kernel form is checked against there, for a cache in the state those arguments describe: valid_tokens is
    rebuilt from them (ring bits, a head's own rows, the open chunk), and nats_chunk_size == 1 means the per-token
    cache class (`sliding_queue_tail` = the slot written last).

    Two numbers of the cache are not among the reference's arguments; both may be passed here (the cache classes of
    this package know them): `seen_tokens` = the cache's _seen_tokens before this segment, which decides whether the
    ring has wrapped (:666-676 against :678-690) -- without it the window is taken as full, and a call whose other
    arguments fit a ring that has not filled yet (fewer than W rows behind the ring and its last slot empty in
    every head) is refused rather than answered for the wrong case; `n_global_min` = the cache's _n_global_min,
    computed from global_kv_size (one device-to-host read) when it is not given."""
    if q.shape[1] // k.shape[1] != n_rep:
        raise ValueError(f"n_rep={n_rep} does not match {q.shape[1]} q heads / {k.shape[1]} kv heads")
    roles = _roles_from_kernel_arguments(end_seqs_idx, sliding_tokens)
    C, W = int(nats_chunk_size), int(local_seq_max_length)
    if global_kv_size is None:
        o = prefill_attention(q, k, v, roles, C, W, sm_scale)
        mask = prefill_mask(roles, q.shape[2], C, W) if return_masks else None
        return o, mask
    if local_kv_size is None or valid_sw_tokens is None or n_ctx_data is None or sw_token_tails is None:
        raise ValueError("the form over an existing cache needs local_kv_size, valid_sw_tokens, n_ctx_data and sw_token_tails")
    B, Hkv, x_len = k.shape[0], k.shape[1], q.shape[2]
    n_ctx, tail, old_fill = int(n_ctx_data), int(sw_token_tails), int(n_tokens_in_first_chunk)
    if k.shape[2] != n_ctx + x_len:
        raise ValueError(f"k / v must hold n_ctx_data + L_q = {n_ctx + x_len} rows, got {k.shape[2]}")
    if C > 1 and n_ctx % C != old_fill:
        raise ValueError(f"n_ctx_data={n_ctx} does not end {old_fill} tokens into a chunk of {C}")
    if tuple(valid_sw_tokens.shape) != (B, Hkv, W // C):
        raise ValueError(f"valid_sw_tokens must be [B, H_kv, W / C], got {tuple(valid_sw_tokens.shape)}")
    sg = global_kv_size.to(torch.int64).contiguous()
    sl = local_kv_size.to(torch.int64).contiguous()
    if seen_tokens is None:
        if n_ctx - W - old_fill < W and not bool(valid_sw_tokens[..., -1].any()):
            raise ValueError("nats_prefill: these arguments fit a cache whose window has not filled yet as well as a "
                             "full one; pass seen_tokens (the cache's _seen_tokens before this segment)")
        seen_tokens = W
    gmin = int(sg.min()) if n_global_min is None else int(n_global_min)
    rows = torch.arange(n_ctx, device=q.device)
    valid = rows < (sg + sl).unsqueeze(-1)                                       # a head's own global and local rows
    valid[:, :, :W] = valid_sw_tokens.bool().repeat_interleave(C, dim=-1)       # ring slots
    valid[:, :, n_ctx - old_fill:] = True                                        # the open chunk
    state = past_state(n_ctx, old_fill, gmin, tail, int(seen_tokens), old_fill,
                       PER_TOKEN_UPDATE_CHUNK if C == 1 else 0)
    o = prefill_past_attention(q, k, v, valid, sg, sl, roles, C, W, state, sm_scale)
    mask = prefill_past_mask(valid, sg, sl, roles, x_len, C, W, state) if return_masks else None
    return o, mask


# ------------------------------------------------------------------------------------------------
# decode
# ------------------------------------------------------------------------------------------------
def decode_attention(q: torch.Tensor, cache_k: torch.Tensor, cache_v: torch.Tensor, valid: torch.Tensor, n_rows: int,
                     sm_scale: float | None = None, row_end: torch.Tensor | None = None,
                     tail_start: int | None = None) -> torch.Tensor:
    """One query token per sequence over the evicted cache.

    q [B, H_q, 1, D]; cache_k / cache_v [B, H_kv, >= n_rows, D]; valid bool / uint8 [B, H_kv, >= n_rows].
    Attends to rows i < n_rows with valid[b, h, i]; returns [B, H_q, 1, D].
    Optional hint: `row_end` int64 [B, H_kv] and `tail_start` state that rows [row_end, tail_start) of a head
    hold nothing valid (size_global_kv + size_local_kv and the start of the open chunk); they are skipped."""
    _require_cuda(q, cache_k, cache_v, valid)
    lib = _lib.load()
    if q.dim() != 4 or cache_k.dim() != 4 or valid.dim() != 3:
        raise ValueError("decode_attention takes q [B, H_q, 1, D], cache_k / cache_v [B, H_kv, rows, D], valid [B, H_kv, rows]")
    B, Hq, one, D = q.shape
    if one != 1:
        raise ValueError("decode_attention takes exactly one query token per sequence")
    Hkv = cache_k.shape[1]
    if cache_k.shape[0] != B or cache_k.shape[3] != D or tuple(valid.shape[:2]) != (B, Hkv) or Hkv == 0 or Hq % Hkv:
        raise ValueError(f"shape mismatch: q {tuple(q.shape)}, cache {tuple(cache_k.shape)}, valid {tuple(valid.shape)}")
    if cache_k.shape != cache_v.shape or strides_differ(cache_k, cache_v):
        raise ValueError("cache_k and cache_v must share shape and strides")
    if cache_k.shape[2] < n_rows or valid.shape[2] < n_rows:
        raise ValueError(f"n_rows={n_rows} exceeds the cache ({cache_k.shape[2]} rows) or valid ({valid.shape[2]})")
    if cache_k.stride(-1) != 1 or valid.stride(-1) != 1:
        raise ValueError("cache rows and valid rows must be contiguous")
    if not (q.dtype == cache_k.dtype == cache_v.dtype):
        raise ValueError("q and the cache must share one dtype")
    if valid.dtype == torch.bool:
        valid = valid.view(torch.uint8)
    qc = q.reshape(B, Hq, D).contiguous()
    out = torch.empty(B, Hq, D, dtype=q.dtype, device=q.device)
    scale = (1.0 / math.sqrt(D)) if sm_scale is None else float(sm_scale)
    nbytes = lib.nats_decode_workspace_bytes(B, Hq, Hkv, D, n_rows)
    ws = workspace(q.device, "decode", nbytes)
    if row_end is not None:
        if tail_start is None or tuple(row_end.shape) != (B, Hkv) or row_end.dtype != torch.int64:
            raise ValueError("row_end must be int64 [B, H_kv] and come with tail_start")
        row_end = row_end.contiguous()
    check(lib.nats_decode_fwd(_ptr(qc), _ptr(cache_k), _ptr(cache_v), _ptr(valid), _ptr(row_end),
                              0 if tail_start is None else int(tail_start), _ptr(out), B, Hq, Hkv, D, n_rows,
                              i64_array(cache_k.stride()[:3]), i64_array(valid.stride()[:2]), scale, _dtype_code(q),
                              _ptr(ws), ws.numel(), _stream(q)))
    return out.view(B, Hq, 1, D)


# ------------------------------------------------------------------------------------------------
# eviction + compaction
# ------------------------------------------------------------------------------------------------
def evict_params(B, H_kv, D, C, W, S, x_len, fill, n_ctx_data, gmin, tail, first, n_alloc, update_chunk=0) -> EvictParams:
    return EvictParams(B, H_kv, D, C, W, S, x_len, fill, n_ctx_data, gmin, tail, int(first), n_alloc, 0, int(update_chunk))


# Sequence numbers of eviction plans are drawn from one counter for the whole process, and the 16-byte pinned mirrors
# the plan kernels report into are never handed back to the host allocator (a dropped EvictBuffers returns its mirror
# to this pool): a plan kernel of a cache that has been dropped may still be queued, and whatever it writes late can
# then neither land in memory that has a new owner outside this module nor carry a number a live cache waits for.
_evict_seq = 0
_mirror_pool: list = []


def _next_evict_seq() -> int:
    global _evict_seq
    _evict_seq = _evict_seq % 0x7fffffff + 1
    return _evict_seq


class EvictBuffers:
    """What the eviction calls of one cache keep between calls: the plan workspace, the 64-byte result in device
    memory, which the apply kernels read, and 16 bytes of pinned host memory into which the plan kernel also writes
    the numbers the host needs (n_ctx_data, minimum global size, two flags) with the call's sequence number: the
    host polls for that number instead of synchronising with the stream."""

    POLL_SECONDS = 0.1  # how long `wait` polls before it synchronises with the device instead

    def __init__(self, device):
        self.device = torch.device(device)
        self.ws = None
        self.result = torch.zeros(8, dtype=torch.int64, device=self.device)
        self.mirror = _mirror_pool.pop() if _mirror_pool else torch.zeros(4, dtype=torch.int32).pin_memory()
        self.mirror_np = self.mirror.numpy()
        self.seq = 0

    def __del__(self):
        try:
            _mirror_pool.append(self.mirror)
        except Exception:  # (interpreter shutdown)
            pass

    def workspace(self, nbytes: int) -> torch.Tensor:
        if self.ws is None or self.ws.numel() < nbytes:
            have = 0 if self.ws is None else self.ws.numel()
            # (zeros: the plan kernel's ticket counter at the start of the workspace is zero between launches)
            self.ws = torch.zeros(max(int(nbytes), 2 * have, 4096), dtype=torch.uint8, device=self.device)
        return self.ws

    def next_seq(self) -> int:
        self.seq = _next_evict_seq()
        return self.seq

    def reported(self, seq: int) -> bool:
        """Whether the plan call numbered `seq` has written its result (one read, no waiting)."""
        return int(self.mirror_np[0]) == seq

    def wait(self, seq: int) -> EvictBrief:
        """The short result of the plan call numbered `seq`, as soon as its kernel has written it."""
        m = self.mirror_np
        if m[0] != seq:
            spins, deadline = 0, time.perf_counter() + self.POLL_SECONDS
            while m[0] != seq:
                spins += 1
                if spins & 1023:
                    continue
                time.sleep(0)  # (lets other Python threads run)
                if time.perf_counter() > deadline:  # something is slow: a synchronisation instead
                    torch.cuda.synchronize(self.device)
                    if m[0] != seq:
                        raise RuntimeError(f"eviction plan {seq} never reported its result (mirror holds {int(m[0])})")
        flags = int(m[1])
        return EvictBrief(int(m[2]), int(m[3]), flags & 1, (flags >> 1) & 1)

    def full_result(self) -> EvictResult:
        """All eight numbers of the last plan call, copied from device memory (synchronises with the stream)."""
        return read_result(self.result)


def evict_plan(roles: torch.Tensor, size_global: torch.Tensor, size_local: torch.Tensor, params: EvictParams,
               buffers: EvictBuffers | None = None):
    """Returns (workspace, result): the per-head plan (device) and the 64-byte result struct (device int64[8]).
    With `buffers` the call uses that cache's workspace, numbers itself (params.seq) and mirrors its result into
    pinned host memory, where `buffers.wait(params.seq)` finds its short form without a stream synchronisation."""
    _require_cuda(roles, size_global, size_local)
    lib = _lib.load()
    nbytes = lib.nats_evict_workspace_bytes(params.B, params.H_kv, params.S)
    if buffers is None:
        ws = torch.zeros(max(nbytes, 256), dtype=torch.uint8, device=roles.device)  # (its first 256 bytes must be zero)
        result = torch.empty(8, dtype=torch.int64, device=roles.device)
        mirror = None
    else:
        ws, result, mirror = buffers.workspace(nbytes), buffers.result, buffers.mirror
        params.seq = buffers.next_seq()
    check(lib.nats_evict_plan(_ptr(roles), _ptr(size_global), _ptr(size_local), ctypes.byref(params), _ptr(ws), ws.numel(),
                              _ptr(result), _ptr(mirror), _stream(roles)))
    return ws, result


def read_result(result: torch.Tensor) -> EvictResult:
    """Copies the device result struct to the host (synchronises with the stream)."""
    host = result.cpu().tolist()
    return EvictResult(*host)


def _append_layout_ok(k: torch.Tensor, v: torch.Tensor, cache_k: torch.Tensor, cache_v: torch.Tensor) -> bool:
    """One dtype, 16-byte rows and strides everywhere, the cache itself at 16-byte addresses (the addresses of the
    new rows are the caller's to check)."""
    e = 16 // cache_k.element_size()
    ts = (k, v, cache_k, cache_v)
    return (all(t.is_cuda and t.dtype == cache_k.dtype and t.stride(-1) == 1 for t in ts)
            and (cache_k.data_ptr() | cache_v.data_ptr()) % 16 == 0
            and cache_k.shape[-1] % e == 0 and all(st % e == 0 for t in ts for st, n in zip(t.stride()[:3], t.shape[:3]) if n != 1)
            and not strides_differ(cache_k, cache_v))


def cache_append_ok(k: torch.Tensor, v: torch.Tensor, cache_k: torch.Tensor, cache_v: torch.Tensor) -> bool:
    """Whether `cache_append` takes these tensors: one dtype, 16-byte rows, strides and addresses everywhere."""
    return _append_layout_ok(k, v, cache_k, cache_v) and (k.data_ptr() | v.data_ptr()) % 16 == 0


def cache_append(k: torch.Tensor, v: torch.Tensor, cache_k: torch.Tensor, cache_v: torch.Tensor, valid: torch.Tensor,
                 pos: torch.Tensor | None, row0: int, pos0: int = 0):
    """k / v [B, H_kv, x_len, D] into rows [row0, row0 + x_len) of the cache, with their valid bytes (and stream
    positions): the row write of the cache update in one launch."""
    B, H, x_len, D = k.shape
    e = 16 // cache_k.element_size()
    fix = lambda t: tuple(st if n != 1 else e for st, n in zip(t.stride()[:3], t.shape[:3]))  # (a size-1 dimension may carry any stride)
    check(_lib.load().nats_cache_append(_ptr(k), _ptr(v), _ptr(cache_k), _ptr(cache_v), _ptr(valid), _ptr(pos), B, H, x_len, D,
                                        int(row0), min(cache_k.shape[2], valid.shape[2]), int(pos0), i64_array(fix(k)),
                                        i64_array(fix(v)), i64_array(fix(cache_k)), i64_array(valid.stride()[:2]),
                                        cache_k.element_size(), _stream(k)))


class CacheAppendCall:
    """`cache_append` for one pair of layouts (the new rows' and the cache's), with the checks made and the stride
    arrays and buffer addresses prepared once: a caller that appends step after step into the same buffers pays one
    library call per step.  `matches` says whether a prepared call still fits the tensors at hand."""

    def __init__(self, k, v, cache_k, cache_v, valid, pos):
        self.key = (k.shape, k.stride(), v.stride(), k.dtype, v.dtype, k.device)
        self.bufs = (cache_k, cache_v, valid, pos)
        self.ok = _append_layout_ok(k, v, cache_k, cache_v)  # (the rows' addresses are checked per call)
        if not self.ok:
            return
        e = 16 // cache_k.element_size()
        fix = lambda t: tuple(st if n != 1 else e for st, n in zip(t.stride()[:3], t.shape[:3]))
        B, H, x_len, D = k.shape
        self.fn = _lib.load().nats_cache_append
        self.fn_plan = _lib.load().nats_cache_append_plan
        self.head = (_ptr(cache_k), _ptr(cache_v), _ptr(valid), _ptr(pos), B, H, x_len, D)
        self.n_rows = min(cache_k.shape[2], valid.shape[2])
        self.tail = (i64_array(fix(k)), i64_array(fix(v)), i64_array(fix(cache_k)), i64_array(valid.stride()[:2]),
                     cache_k.element_size())

    def matches(self, k, v, cache_k, cache_v, valid, pos) -> bool:
        b = self.bufs
        return (b[0] is cache_k and b[1] is cache_v and b[2] is valid and b[3] is pos
                and self.key == (k.shape, k.stride(), v.stride(), k.dtype, v.dtype, k.device))

    def __call__(self, k, v, row0: int, pos0: int = 0, plan: "EvictInplaceCall | None" = None, roles=None, params=None) -> bool:
        """Appends and returns True; False if these tensors cannot take the kernel (layout or alignment).  With `plan`
        (and the roles and parameters of the eviction that will follow this update) the same launch also plans that
        eviction, which `plan.apply_planned` then only has to apply."""
        pk, pv = k.data_ptr(), v.data_ptr()
        if not self.ok or (pk | pv) & 15:
            return False
        if plan is None:
            check(self.fn(pk, pv, *self.head, row0, self.n_rows, pos0, *self.tail, _stream(k)))
        else:
            params.seq = plan.buffers.next_seq()
            check(self.fn_plan(pk, pv, *self.head, row0, self.n_rows, pos0, *self.tail, roles.data_ptr(), *plan.sizes,
                               ctypes.byref(params), *plan.plan_tail, _stream(k)))
        return True


class EvictInplaceCall:
    """Plan + in-place apply (`evict_plan`, `evict_apply_inplace`) for one set of cache buffers and role layout, checked
    and prepared once; a call takes the roles of the step and the parameter struct."""

    def __init__(self, cache_k, cache_v, valid, pos, size_global, size_local, buffers: "EvictBuffers", B, H_kv, S):
        _require_cuda(cache_k, cache_v, valid, size_global, size_local)
        if cache_k.shape != cache_v.shape or strides_differ(cache_k, cache_v) or cache_k.dtype != cache_v.dtype:
            raise ValueError("cache_k and cache_v must share dtype and strides")
        v8 = valid.view(torch.uint8) if valid.dtype == torch.bool else valid
        if pos is not None and (pos.dtype != torch.int32 or pos.shape != v8.shape or strides_differ(pos, v8, 2)):
            raise ValueError("pos must be int32 with the strides of valid")
        lib = _lib.load()
        self.bufs = (cache_k, cache_v, valid, pos)
        self.S = S
        self.buffers = buffers
        ws = buffers.workspace(lib.nats_evict_workspace_bytes(B, H_kv, S))
        self.ws = ws
        self.plan, self.apply = lib.nats_evict_plan, lib.nats_evict_apply_inplace
        self.sizes = (_ptr(size_global), _ptr(size_local))
        self.plan_tail = (_ptr(ws), ws.numel(), _ptr(buffers.result), _ptr(buffers.mirror))
        self.apply_head = (_ptr(cache_k), _ptr(cache_v), _ptr(v8), _ptr(pos))
        self.apply_tail = (i64_array(cache_k.stride()[:3]), i64_array(v8.stride()[:2]), cache_k.element_size(), _ptr(ws),
                           _ptr(buffers.result))

    def matches(self, cache_k, cache_v, valid, pos, S) -> bool:
        b = self.bufs
        return (b[0] is cache_k and b[1] is cache_v and b[2] is valid and b[3] is pos and self.S == S
                and self.ws is self.buffers.ws)

    PLAN_WITH_APPEND_SLOTS, PLAN_WITH_APPEND_HEADS = 32, 4096  # what nats_cache_append_plan takes

    def __call__(self, roles: torch.Tensor, params: EvictParams):
        if not roles.is_cuda or roles.dtype != torch.uint8 or not roles.is_contiguous():
            raise ValueError("roles must be a contiguous uint8 GPU tensor")
        params.seq = self.buffers.next_seq()
        pr, ref, st = roles.data_ptr(), ctypes.byref(params), _stream(roles)
        check(self.plan(pr, *self.sizes, ref, *self.plan_tail, st))
        check(self.apply(*self.apply_head, pr, *self.sizes, ref, *self.apply_tail, st))

    def apply_planned(self, roles: torch.Tensor, params: EvictParams):
        """The apply step alone, for an eviction whose plan rode with the append (`CacheAppendCall(..., plan=self)`):
        `params` are the ones that launch was given, sequence number included."""
        check(self.apply(*self.apply_head, roles.data_ptr(), *self.sizes, ctypes.byref(params), *self.apply_tail, _stream(roles)))


def evict_apply_inplace(cache_k, cache_v, valid, pos, roles, size_global, size_local, params: EvictParams, ws, result):
    _require_cuda(cache_k, cache_v, valid, roles)
    lib = _lib.load()
    if cache_k.shape != cache_v.shape or strides_differ(cache_k, cache_v) or cache_k.dtype != cache_v.dtype:
        raise ValueError("cache_k and cache_v must share dtype and strides")
    v8 = valid.view(torch.uint8) if valid.dtype == torch.bool else valid
    if pos is not None and (pos.dtype != torch.int32 or pos.shape != v8.shape or strides_differ(pos, v8, 2)):
        raise ValueError("pos must be int32 with the strides of valid")
    check(lib.nats_evict_apply_inplace(_ptr(cache_k), _ptr(cache_v), _ptr(v8), _ptr(pos), _ptr(roles), _ptr(size_global),
                                       _ptr(size_local), ctypes.byref(params), i64_array(cache_k.stride()[:3]),
                                       i64_array(v8.stride()[:2]), cache_k.element_size(), _ptr(ws), _ptr(result),
                                       _stream(cache_k)))


def evict_apply_first(src_k, src_v, cache_k, cache_v, valid, pos, roles, size_global, size_local, params: EvictParams,
                      ws, result):
    _require_cuda(src_k, src_v, cache_k, cache_v, valid, roles)
    lib = _lib.load()
    if src_k.shape != src_v.shape or strides_differ(src_k, src_v) or strides_differ(cache_k, cache_v):
        raise ValueError("K and V must share strides")
    v8 = valid.view(torch.uint8) if valid.dtype == torch.bool else valid
    if pos is not None and (pos.dtype != torch.int32 or pos.shape != v8.shape or strides_differ(pos, v8, 2)):
        raise ValueError("pos must be int32 with the strides of valid")
    check(lib.nats_evict_apply_first(_ptr(src_k), _ptr(src_v), _ptr(cache_k), _ptr(cache_v), _ptr(v8), _ptr(pos),
                                     _ptr(roles), _ptr(size_global), _ptr(size_local), ctypes.byref(params),
                                     i64_array(src_k.stride()[:3]), i64_array(cache_k.stride()[:3]),
                                     i64_array(v8.stride()[:2]), cache_k.element_size(), _ptr(ws), _ptr(result),
                                     _stream(cache_k)))


# ------------------------------------------------------------------------------------------------
# decode-step glue of the HF-shaped caller
# ------------------------------------------------------------------------------------------------
CARRY_NONE, CARRY_MEAN_FIRST, CARRY_MEAN_ADD, CARRY_MAX_FIRST, CARRY_MAX_MERGE = 0, 1, 2, 3, 4
NORM_MAX_DIM = 8192  # widest row add_rms_norm takes


def add_rms_norm(x: torch.Tensor, delta: torch.Tensor | None, weight: torch.Tensor, eps: float,
                 carry: torch.Tensor | None = None, carry_mode: int = CARRY_NONE, chunk_size: int = 1) -> torch.Tensor:
    """x += delta (in place, if delta is given); returns RMSNorm(x) * weight (models/transformer/components.py:14-26).
    With carry_mode != 0 the running chunk statistic `carry` [rows, dim] of the role step is updated from the
    normalised rows (components/cache/dyn_cache.py:98-124)."""
    _require_cuda(x, delta, weight, carry)
    if not x.is_contiguous() or (delta is not None and (not delta.is_contiguous() or delta.shape != x.shape)):
        raise ValueError("add_rms_norm takes contiguous x and delta of one shape")
    dim = x.shape[-1]
    rows = x.numel() // dim
    if weight.shape != (dim,) or weight.dtype != x.dtype or not weight.is_contiguous():
        raise ValueError("add_rms_norm: weight must be [dim] of x's dtype")
    if carry_mode != CARRY_NONE and (carry is None or carry.numel() != x.numel() or not carry.is_contiguous()
                                     or carry.dtype != x.dtype):
        raise ValueError("add_rms_norm: the chunk statistic must be a contiguous tensor of x's size and dtype")
    out = torch.empty_like(x)
    check(_lib.load().nats_add_rms_norm(_ptr(x), _ptr(delta), _ptr(weight), _ptr(out), _ptr(carry), rows, dim, float(eps),
                                        int(carry_mode), int(chunk_size), _dtype_code(x), _stream(x)))
    return out


def silu_mul(gate_up: torch.Tensor) -> torch.Tensor:
    """[..., 2 * I] -> silu(gate_up[..., :I]) * gate_up[..., I:]."""
    _require_cuda(gate_up)
    if not gate_up.is_contiguous() or gate_up.shape[-1] % 2:
        raise ValueError("silu_mul takes a contiguous [..., 2 * I] tensor")
    inter = gate_up.shape[-1] // 2
    out = torch.empty(*gate_up.shape[:-1], inter, dtype=gate_up.dtype, device=gate_up.device)
    check(_lib.load().nats_silu_mul(_ptr(gate_up), _ptr(out), gate_up.numel() // (2 * inter), inter, _dtype_code(gate_up),
                                    _stream(gate_up)))
    return out


MATVEC_MAX_ROWS = 4


def _matvec_weight_ok(weight: torch.Tensor) -> bool:
    e = 16 // weight.element_size()
    return (weight.is_cuda and weight.dim() == 2 and weight.dtype in (torch.bfloat16, torch.float32)
            and weight.shape[1] % e == 0 and weight.stride(1) == 1 and weight.stride(0) % e == 0
            and weight.data_ptr() % 16 == 0)


def matvec_ok(x: torch.Tensor, weight: torch.Tensor) -> bool:
    """Whether `matvec` takes this pair: at most four rows of x, 16-byte pieces along k."""
    k = x.shape[-1]
    return (_matvec_weight_ok(weight) and x.is_cuda and x.dtype == weight.dtype and weight.shape[1] == k
            and x.is_contiguous() and x.data_ptr() % 16 == 0 and 1 <= x.numel() // k <= MATVEC_MAX_ROWS)


def matvec(x: torch.Tensor, weight: torch.Tensor, gate: bool = False) -> torch.Tensor:
    """nn.functional.linear(x, weight) for up to four rows of x: [..., K] x [N, K] -> [..., N].
    gate=True: weight is [2 * I, K] (gate rows, then up rows) and the result is silu(x W_g^T) * (x W_u^T), [..., I]."""
    _require_cuda(x, weight)
    if not matvec_ok(x, weight):
        raise ValueError("matvec: x [<= 4 rows, K] contiguous and weight [N, K] of the same dtype, K a multiple of 16 bytes")
    return MatvecPlan(weight, gate)(x)  # (x keeps `weight` alive for the call)


class MatvecPlan:
    """A weight matrix checked once for `matvec`, for callers that apply it step after step.  `ok` is False when
    the kernel does not take the matrix; `takes(x)` is the per-call part of `matvec_ok`."""

    __slots__ = ("weight", "ok", "gate", "n", "k", "w_ptr", "w_stride", "dtype", "code", "fn")

    def __init__(self, weight: torch.Tensor, gate: bool = False):
        self.weight = weakref.ref(weight)  # the plan must not keep the matrix alive
        self.gate = 1 if gate else 0
        self.ok = _matvec_weight_ok(weight) and not (gate and weight.shape[0] % 2)
        if gate and weight.shape[0] % 2:
            raise ValueError("matvec: a gate / up matrix has an even number of rows")
        self.n = weight.shape[0] // 2 if gate else weight.shape[0]
        self.k = weight.shape[1]
        self.w_ptr = weight.data_ptr()
        self.w_stride = weight.stride(0)
        self.dtype = weight.dtype
        self.code = _dtype_code(weight) if self.ok else -1
        self.fn = _lib.load().nats_matvec

    def current(self, weight: torch.Tensor) -> bool:
        """Whether the plan still describes `weight` (same storage, dtype and shape)."""
        return (weight.data_ptr() == self.w_ptr and weight.dtype == self.dtype and weight.shape[1] == self.k
                and weight.shape[0] == (2 * self.n if self.gate else self.n) and weight.stride(0) == self.w_stride)

    def takes(self, x: torch.Tensor) -> bool:
        k = self.k
        return (self.ok and x.dtype == self.dtype and x.shape[-1] == k and x.is_cuda and x.is_contiguous()
                and 1 <= x.numel() // k <= MATVEC_MAX_ROWS and x.data_ptr() % 16 == 0)

    def __call__(self, x: torch.Tensor) -> torch.Tensor:
        """x must satisfy `takes(x)`."""
        k, n = self.k, self.n
        y = torch.empty(*x.shape[:-1], n, dtype=x.dtype, device=x.device)
        check(self.fn(self.w_ptr, x.data_ptr(), y.data_ptr(), x.numel() // k, n, k, self.w_stride, k, n, self.gate,
                      self.code, _stream(x)))
        return y


def rope_qk_ok(q: torch.Tensor, k: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> bool:
    """Whether `rope_qk` takes these tensors (16-byte rows everywhere)."""
    e = 16 // q.element_size()
    ts = (q, k, cos, sin)
    return (q.dtype in (torch.bfloat16, torch.float32) and all(t.is_cuda and t.dtype == q.dtype and t.stride(-1) == 1 for t in ts)
            and q.shape[-1] % (2 * e) == 0 and all(t.data_ptr() % 16 == 0 for t in ts)
            and all(st % e == 0 for t in (q, k) for st in t.stride()[:3]) and all(st % e == 0 for st in cos.stride()[:2])
            and sin.stride() == cos.stride())


def rope_qk(q: torch.Tensor, k: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor):
    """apply_rotary_pos_emb for a multi-token segment in one launch: q [B, H_q, L, D], k [B, H_kv, L, D] (any strides,
    last dimension contiguous), cos / sin [B, L, D].  Returns contiguous (q_rot, k_rot)."""
    _require_cuda(q, k, cos, sin)
    B, Hq, L, D = q.shape
    Hkv = k.shape[1]
    if k.shape != (B, Hkv, L, D) or cos.shape != (B, L, D) or sin.shape != cos.shape or not rope_qk_ok(q, k, cos, sin):
        raise ValueError("rope_qk: q [B, H_q, L, D], k [B, H_kv, L, D], cos / sin [B, L, D] of one dtype with 16-byte rows")
    q_out = torch.empty(B, Hq, L, D, dtype=q.dtype, device=q.device)
    k_out = torch.empty(B, Hkv, L, D, dtype=q.dtype, device=q.device)
    check(_lib.load().nats_rope_qk(_ptr(q), _ptr(k), _ptr(cos), _ptr(sin), _ptr(q_out), _ptr(k_out), B, Hq, Hkv, L, D,
                                   i64_array(q.stride()[:3]), i64_array(k.stride()[:3]), i64_array(cos.stride()[:2]),
                                   _dtype_code(q), _stream(q)))
    return q_out, k_out


def rope_append(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
                cache_k: torch.Tensor, cache_v: torch.Tensor, valid: torch.Tensor, pos: torch.Tensor | None, row0: int,
                pos0: int = 0, clear_row: int = -1) -> torch.Tensor:
    """Rotary embedding of q and k, and k / v written to rows [row0, row0 + x_len) of the cache with their valid
    bytes (and stream positions).  q [B, H_q, x_len, D], k / v [B, H_kv, x_len, D] (any strides, last dimension
    contiguous), cos / sin [B, x_len, D].  `clear_row` >= 0: the valid byte of that row (below row0) is set to 0 in
    every head.  Returns the rotated q, contiguous."""
    _require_cuda(q, k, v, cos, sin, cache_k, cache_v, valid, pos)
    B, Hq, x_len, D = q.shape
    Hkv = k.shape[1]
    if k.shape != (B, Hkv, x_len, D) or v.shape != k.shape or cos.shape != (B, x_len, D) or sin.shape != cos.shape:
        raise ValueError("rope_append: q / k / v / cos / sin shapes do not fit")
    ts = (q, k, v, cos, sin, cache_k, cache_v)
    if any(t.dtype != q.dtype for t in ts) or any(t.stride(-1) != 1 for t in ts):
        raise ValueError("rope_append: one dtype and a contiguous last dimension everywhere")
    if cache_v.shape != cache_k.shape or strides_differ(cache_v, cache_k) or cache_k.shape[:2] != (B, Hkv) or cache_k.shape[3] != D:
        raise ValueError("rope_append: cache_k / cache_v must be [B, H_kv, rows, D] with equal strides")
    if strides_differ(sin, cos):
        sin = sin.contiguous()
        cos = cos.contiguous()
    if valid.dtype != torch.uint8 or valid.stride(-1) != 1 or (pos is not None and (pos.shape != valid.shape or strides_differ(pos, valid)
                                                                                   or pos.dtype != torch.int32)):
        raise ValueError("rope_append: valid must be uint8 rows (pos: int32 of the same layout)")
    q_out = torch.empty(B, Hq, x_len, D, dtype=q.dtype, device=q.device)
    n_alloc = min(cache_k.shape[2], valid.shape[2])
    check(_lib.load().nats_rope_append(
        _ptr(q), _ptr(k), _ptr(v), _ptr(cos), _ptr(sin), _ptr(q_out), _ptr(cache_k), _ptr(cache_v), _ptr(valid), _ptr(pos),
        B, Hq, Hkv, x_len, D, int(row0), n_alloc, int(pos0), int(clear_row), i64_array(q.stride()[:3]), i64_array(k.stride()[:3]),
        i64_array(v.stride()[:3]), i64_array(cos.stride()[:2]), i64_array(cache_k.stride()[:3]),
        i64_array(valid.stride()[:2]), _dtype_code(q), _stream(q)))
    return q_out
