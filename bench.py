"""Benchmark of the NAtS sparse-attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--skip-cpu] [--no-llama] [--no-extras] [--only prefill|decode|evict|evict_stream|segments|role_step|matvec|llama]

    (other sizes of a single leg: --prefill-len L, --chunk-size C, --decode-batch B, --decode-context N, --llama-chunk C)

One step = one pass of a kernel family over one batch of synthetic input that is already resident in HBM:

* prefill  role-masked chunked flash attention at the Llama-3-8B head shape, L = 32768 (the headline)
* decode   one query token per sequence over the ragged, evicted KV cache (batch 32, context 65536)
* evict    bulk eviction + compaction of a 16 x 8 x 65536 x 128 cache after its prefill
* llama_e2e  the three together inside a random-weight Llama-3-8B-shape model: a 16384-token prefill, then 512 greedy
           one-token steps with eviction live in all 32 layers (seconds for the prefill, ms per token, peak memory);
           llama_e2e_c1 the same with a role per token (the per-token cache class)
* riding along under their own keys: prefill_c32 / prefill_c1 (the prefill at chunk sizes 32 and 1), decode_b1 (one
           sequence), evict.cold (a layer cache that has never evicted), evict_stream (the eviction workload chunk by
           chunk), segments (the prefill cut into four segments over one cache)

Prints ONE JSON line.  `value` is the prefill time in ms; decode tokens/s, GB/s and the compaction GB/s
ride along in the same line, each with its roofline fraction, next to a CPU baseline (the oracle, timed
on this host's cores on a bounded sample of the same workload).
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# HBM bytes per launch of the dominant kernels at the default workloads come from profiler counter runs
# (rocprofv3 --pmc FETCH_SIZE, then WRITE_SIZE, KiB per dispatch, scaled by what a 1 GiB device copy reads on the same
# counters).  They are kept in bench_traffic.json together with a hash of the kernel sources they were measured on:
# once a source has changed the figure is no longer reported (traffic: null) until the counters are read again and
# recorded with `python bench.py --record-traffic prefill=<FETCH KiB>,<WRITE KiB> ...`.
TRAFFIC_FILE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "bench_traffic.json")
TRAFFIC_SOURCES = {
    "prefill": ["nats_prefill.hip", "nats_roles.hip", "nats_common.h"],
    "decode": ["nats_decode.hip", "nats_common.h"],
    "evict": ["nats_evict.hip", "nats_common.h"],
}


def source_hash(names) -> str:
    import hashlib
    h = hashlib.sha256()
    for n in names:
        with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "neuralattentionsearch_amd", "csrc", n), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def measured_traffic(key: str):
    """(bytes read + written per launch, note) of a dominant kernel; bytes is None when there is no current figure."""
    try:
        with open(TRAFFIC_FILE) as f:
            table = json.load(f)
        e = table["kernels"][key]
    except (OSError, KeyError, ValueError):
        return None, "no counter figures recorded"
    if e["source_hash"] != source_hash(TRAFFIC_SOURCES[key]):
        return None, "kernel sources changed since the counters were read (" + e["profile"] + ")"
    cal = table["calibration"]
    return e["fetch_kib"] * 1024 * cal["fetch_factor"] + e["write_kib"] * 1024 * cal["write_factor"], e["profile"]


def record_traffic(items):
    """--record-traffic key=fetch_kib,write_kib ...: stores the figures with the hash of the present sources."""
    with open(TRAFFIC_FILE) as f:
        table = json.load(f)
    for it in items:
        key, vals = it.split("=")
        fetch, write = (float(x) for x in vals.split(","))
        table["kernels"][key].update(fetch_kib=fetch, write_kib=write, source_hash=source_hash(TRAFFIC_SOURCES[key]))
    with open(TRAFFIC_FILE, "w") as f:
        json.dump(table, f, indent=1)
        f.write("\n")


PEAK_HBM_GBS = 8000.0
PEAK_BF16_TFLOPS = 2500.0
METRIC = "NAtS prefill ms @32k (MFMA util); sparse-KV decode tok/s (HBM GB/s %peak)"


def draw_roles(seed, B, H, S, p):
    """Roles drawn directly (CPU legs, where no role kernel runs)."""
    rng = np.random.default_rng(seed)
    r = rng.choice(3, size=(B, H, S), p=p).astype(np.uint8)
    r[:, :, 0] = 0  # sink chunk
    return r


# Role logits of the GPU legs: N(0, 1) per (chunk, head, option) plus these constants on (global, local, sliding window).
# With the 0.1 the role kernel adds to the global logit (models/transformer/attention/nats_attention.py:96-109) the
# first-maximum argmax then lands on the configured shares: P(option i) = int phi(z - b_i) prod_{j != i} Phi(z - b_j) dz
# solved for b (sliding window fixed at 0).
ROLE_LOGIT_BIAS = {
    (0.05, 0.15, 0.80): (-2.17317727, -1.38648285, 0.0),   # prefill workload
    (0.10, 0.15, 0.75): (-1.67833392, -1.31208150, 0.0),   # eviction workload
}
ROLE_GLOBAL_BIAS = 0.1


def biased_role_logits(seed, B, S, H, shares, device="cuda"):
    """fp32 [B, S, H, 3] logits whose argmax (through ops.roles_from_logits with the first chunk forced global) gives
    roles in the shares (global, local, sliding window)."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(B, S, H, 3, generator=g) + torch.tensor(ROLE_LOGIT_BIAS[shares])
    return x.to(device)


def chunk_limits_np(roles: np.ndarray, wc: int) -> np.ndarray:
    """Last query chunk that sees key chunk n, per (b, h, n): global -> S - 1, sliding window -> n + W / C, local ->
    the next global chunk at or after n (the last chunk counts as one)."""
    B, H, S = roles.shape
    is_g = roles == 0
    flags = is_g.copy()
    flags[..., -1] = True
    idx = np.where(flags, np.arange(S), S)  # next global at or after n: reverse running minimum
    g = np.minimum.accumulate(idx[..., ::-1], axis=-1)[..., ::-1]
    lim = np.where(is_g, S - 1, np.where(roles == 2, np.arange(S) + wc, g))
    return np.minimum(lim, S - 1)


def prefill_flops(roles: np.ndarray, L: int, C: int, W: int, D: int, n_rep: int) -> tuple[float, float]:
    """Algorithmic FLOPs on the visited (query chunk, key chunk) pairs and the dense causal count."""
    S = roles.shape[-1]
    lim = chunk_limits_np(roles, W // C).astype(np.int64)
    off = int((lim - np.arange(S)).sum())  # query chunks after n that see it
    n_streams = roles.shape[0] * roles.shape[1]
    pairs = off * C * C + n_streams * S * (C * (C + 1) // 2)
    dense = n_streams * (L * (L + 1) // 2)
    return 4.0 * D * n_rep * pairs, 4.0 * D * n_rep * dense


def time_gpu(fn, steps: int, warmup: int, settle_ms: float = 0.0):
    """Time of `fn` on the current stream: W untimed calls (`settle_ms` keeps the untimed calls going for that long:
    after the host-side set-up of a leg's inputs the GPU has dropped to its idle clock, and a few milliseconds of
    warm-up do not always bring it back), then exactly K calls between one pair of HIP events
    (and one pair of synchronisations), so that the launches follow each other as they do in use.  Returns
    (host wall time per step, GPU time per step, best single step); the best step comes from a short extra loop
    with an event pair around every call, which costs each call about ten microseconds of markers and is
    therefore not what the mean is taken from."""
    for _ in range(warmup):
        fn()
    t_settle = time.perf_counter() + settle_ms * 1e-3
    while time.perf_counter() < t_settle:
        fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    mean = start.elapsed_time(stop) / steps
    n = min(steps, 10)
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(n)]
    stops = [torch.cuda.Event(enable_timing=True) for _ in range(n)]
    for i in range(n):
        starts[i].record()
        fn()
        stops[i].record()
    torch.cuda.synchronize()
    best = min(s.elapsed_time(e) for s, e in zip(starts, stops))
    return wall, float(mean), float(min(best, mean))


# --------------------------------------------------------------------------------------------------
def bench_prefill(args, ops, chunk_size=None, steps=None, warmup=None, compare=True, settle=True):
    B, Hq, Hkv, L, D, C, W = 1, 32, 8, args.prefill_len, args.head_dim, chunk_size or args.chunk_size, 256
    steps, warmup = steps or args.steps, args.warmup if warmup is None else warmup
    n_rep = Hq // Hkv
    dev = "cuda"
    g = torch.Generator(device=dev).manual_seed(0)
    q = (torch.randn(B, Hq, L, D, generator=g, device=dev) / math.sqrt(D)).bfloat16()
    k = (torch.randn(B, Hkv, L, D, generator=g, device=dev) / math.sqrt(D)).bfloat16()
    v = (torch.randn(B, Hkv, L, D, generator=g, device=dev) / math.sqrt(D)).bfloat16()
    logits = biased_role_logits(0, B, L // C, Hkv, (0.05, 0.15, 0.80), dev)
    roles, _ = ops.roles_from_logits(logits, ROLE_GLOBAL_BIAS, True, False, with_one_hot=False)
    roles_np = roles.cpu().numpy()
    out = torch.empty_like(q)
    flops, dense_flops = prefill_flops(roles_np, L, C, W, D, n_rep)

    def sparse_step():  # the op as the attention module runs it: role logits -> roles -> masked attention
        r, _ = ops.roles_from_logits(logits, ROLE_GLOBAL_BIAS, True, False, with_one_hot=False)
        ops.prefill_attention(q, k, v, r, C, W, out=out)

    # Settling phase: the power management of the GPU takes some tens of milliseconds of matrix-heavy load to reach
    # its steady clock (the first launches after idle run up to 30 % slower than the settled ones), and a serving
    # process sees the settled clock.  A few untimed launches of a dense attention provide that load (the library
    # kernel, so that a kernel trace of this run keeps the sparse workload's launches apart); the timed region itself
    # is W warm-up steps + K timed steps of the sparse workload, and the comparators are timed after it.
    roles_dense = torch.zeros_like(roles)
    if settle:
        try:
            for _ in range(3):
                torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True)
        except Exception:
            for _ in range(6):
                ops.prefill_attention(q, k, v, roles_dense, C, W, out=out)

    wall, ev_mean, ev_min = time_gpu(sparse_step, steps, warmup)
    res = {
        "ms": ev_mean, "ms_min": ev_min, "ms_wall": wall,
        "visited_fraction": flops / dense_flops, "algorithmic_tflop": flops / 1e12,
        "tflops_visited": flops / (ev_mean * 1e-3) / 1e12,
        "tokens_per_s": L / (ev_mean * 1e-3),
    }
    shares = [float((roles_np == i).mean()) for i in range(3)]
    res["shape"] = dict(B=B, Hq=Hq, Hkv=Hkv, L=L, D=D, C=C, W=W,
                        roles="argmax of biased N(0,1) logits inside the timed op: %.1f%% global / %.1f%% local / %.1f%% sliding"
                              % tuple(100 * x for x in shares))
    if compare and not args.no_compare:
        # the same kernel on all-global roles = dense causal attention
        _, dm, _ = time_gpu(lambda: ops.prefill_attention(q, k, v, roles_dense, C, W, out=out), max(2, steps // 4), 1)
        res["own_dense_causal_ms"] = dm
        res["own_dense_causal_tflops"] = dense_flops / (dm * 1e-3) / 1e12
        # a library dense causal flash attention of the same shape on the same GPU
        try:
            def sdpa():
                return torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True)
            _, sm, _ = time_gpu(sdpa, max(2, steps // 4), 1)
            res["torch_sdpa_dense_causal_ms"] = sm
            res["torch_sdpa_dense_causal_tflops"] = dense_flops / (sm * 1e-3) / 1e12
            res["frac_of_dense_flash_throughput"] = res["tflops_visited"] / res["torch_sdpa_dense_causal_tflops"]
        except Exception as e:  # library path unavailable on this build
            res["torch_sdpa_error"] = repr(e)[:200]
    return res


def decode_inputs(B, Hq, Hkv, D, C, W, ctx, seed, dev):
    rng = np.random.default_rng(seed)
    n = (rng.uniform(0.10, 0.30, size=(B, Hkv)) * ctx / C).round().astype(np.int64) * C
    base = W + int(n.max())
    fill = 17
    n_rows = base + fill + 1
    n_alloc = -(-n_rows // C) * C
    g = torch.Generator(device=dev).manual_seed(seed)
    k = torch.randn(B, Hkv, n_alloc, D, generator=g, device=dev).bfloat16()
    v = torch.randn(B, Hkv, n_alloc, D, generator=g, device=dev).bfloat16()
    valid = np.zeros((B, Hkv, n_alloc), dtype=bool)
    valid[:, :, :W] = np.repeat(rng.random((B, Hkv, W // C)) < 0.8, C, axis=-1)
    for b in range(B):
        for h in range(Hkv):
            valid[b, h, W:W + n[b, h]] = True
    valid[:, :, base:n_rows] = True
    q = torch.randn(B, Hq, 1, D, generator=g, device=dev).bfloat16()
    hint = (torch.from_numpy(W + n).to(dev), base)  # what the cache object knows: size_global + size_local, open chunk
    return q, k, v, torch.from_numpy(valid).to(dev), n_rows, hint


def bench_decode(args, ops, batch=None, context=None):
    B, Hq, Hkv, D, C, W, ctx = batch or args.decode_batch, 32, 8, args.head_dim, 64, 256, context or args.decode_context
    q, k, v, valid, n_rows, (row_end, tail_start) = decode_inputs(B, Hq, Hkv, D, C, W, ctx, 0, "cuda")
    n_valid = int(valid[:, :, :n_rows].sum().item())
    bytes_alg = n_valid * D * 2 * 2 + 2 * q.numel() * 2
    wall, ev_mean, ev_min = time_gpu(
        lambda: ops.decode_attention(q, k, v, valid, n_rows, row_end=row_end, tail_start=tail_start),
        args.steps * 5, args.warmup, settle_ms=60.0)
    return {
        "ms": ev_mean, "ms_min": ev_min, "ms_wall": wall,
        "tokens_per_s_per_layer": B / (ev_mean * 1e-3),
        "algorithmic_bytes": bytes_alg, "gbs": bytes_alg / (ev_mean * 1e-3) / 1e9,
        "frac_of_hbm_peak": bytes_alg / (ev_mean * 1e-3) / 1e9 / PEAK_HBM_GBS,
        "kept_fraction": n_valid / (B * Hkv * ctx),
        "shape": dict(B=B, Hq=Hq, Hkv=Hkv, D=D, C=C, W=W, context=ctx, rows=n_rows),
    }


def bench_evict(args, ops):
    """Bulk eviction + compaction after a prefill.  `warm`: a layer cache that has been through a prompt before (what
    NAtSCache.reset_cache leaves for the next prompt): the cache is allocated on the share of rows kept last time and the
    apply kernel is launched without waiting for the plan.  `cold`: a layer cache that has never evicted (the first
    prompt of a process): the host waits for the plan's row count before it allocates."""
    from neuralattentionsearch_amd.cache import NAtSChunkLayerCache
    B, Hkv, L, D, C, W = 16, 8, 65536, 128, 64, 512
    dev = "cuda"
    g = torch.Generator(device=dev).manual_seed(0)
    k = torch.randn(B, Hkv, L, D, generator=g, device=dev).bfloat16()
    v = torch.randn(B, Hkv, L, D, generator=g, device=dev).bfloat16()
    logits = biased_role_logits(0, B, L // C, Hkv, (0.10, 0.15, 0.75), dev)
    roles0, _ = ops.roles_from_logits(logits, ROLE_GLOBAL_BIAS, True, False)
    shares = [float((roles0 == i).float().mean().item()) for i in range(3)]
    cache = NAtSChunkLayerCache(B, Hkv, W, chunk_size=C, device=dev)
    moved = {}

    def evict_into(c):
        roles, tsi = ops.roles_from_logits(logits, ROLE_GLOBAL_BIAS, True, False)  # role logits -> roles + one-hot
        c.update(k, v, tsi, roles=roles)
        c.post_update(L)
        moved["n_rows"] = c.cache_k.shape[2]  # (waits for the result of the plan kernel, as the next caller would)

    def warm_step():
        cache.reset_cache()
        evict_into(cache)

    def cold_step():
        evict_into(NAtSChunkLayerCache(B, Hkv, W, chunk_size=C, device=dev))

    steps = max(3, args.steps // 2)
    wall, ev_mean, ev_min = time_gpu(warm_step, steps, 2, settle_ms=30.0)
    moved["rows"] = int(cache.last_evict_result.moved_rows)
    c_wall, c_mean, c_min = time_gpu(cold_step, steps, 2)
    ring_rows = B * Hkv * W
    bytes_alg = (moved["rows"] + ring_rows) * D * 2 * 2 * 2  # rows x 256 B x (K, V) x (read + write)
    return {
        "ms": ev_mean, "ms_min": ev_min, "ms_wall": wall,
        "rows_moved": moved["rows"], "cache_rows_after": moved["n_rows"],
        "algorithmic_bytes": bytes_alg, "gbs": bytes_alg / (ev_mean * 1e-3) / 1e9,
        "frac_of_hbm_peak": bytes_alg / (ev_mean * 1e-3) / 1e9 / PEAK_HBM_GBS,
        "cold": {"ms": c_mean, "ms_min": c_min, "ms_wall": c_wall, "gbs": bytes_alg / (c_mean * 1e-3) / 1e9,
                 "frac_of_hbm_peak": bytes_alg / (c_mean * 1e-3) / 1e9 / PEAK_HBM_GBS,
                 "note": "a fresh layer cache per step: role kernel, plan kernel, the host waits for its row count "
                         "(pinned memory), allocation, apply kernel"},
        "note": "role kernel + cache reset + update + whole post_update (plan kernel, apply kernel into a cache sized from "
                "the previous prompt's kept share) + the wait for the plan's result",
        "shape": dict(B=B, Hkv=Hkv, L=L, D=D, C=C, W=W,
                      roles="argmax of biased N(0,1) logits inside the timed op: %.1f%% global / %.1f%% local / %.1f%% sliding"
                            % tuple(100 * x for x in shares)),
    }


def bench_evict_stream(args, ops):
    """The streamed form of the eviction workload: the same 16 x 8 x 65536 x 128 cache filled chunk by chunk,
    1024 x (update(64 tokens) + post_update(64)); every post_update runs the in-place plan + apply kernels."""
    from neuralattentionsearch_amd.cache import NAtSChunkLayerCache
    B, Hkv, L, D, C, W = 16, 8, 65536, 128, 64, 512
    dev = "cuda"
    n_chunks = L // C
    g = torch.Generator(device=dev).manual_seed(0)
    k = torch.randn(B, Hkv, C, D, generator=g, device=dev).bfloat16()
    v = torch.randn(B, Hkv, C, D, generator=g, device=dev).bfloat16()
    # (the roles of all 1024 steps come from one call of the role kernel ahead of the timed loop)
    roles_all, tsi_all = ops.roles_from_logits(biased_role_logits(0, B, n_chunks, Hkv, (0.10, 0.15, 0.75), dev),
                                               ROLE_GLOBAL_BIAS, True, False)
    tsis = [tsi_all[:, :, i:i + 1].contiguous() for i in range(n_chunks)]
    roles = [roles_all[:, :, i:i + 1].contiguous() for i in range(n_chunks)]
    cache = NAtSChunkLayerCache(B, Hkv, W, chunk_size=C, device=dev)

    def run():
        cache.reset_cache()
        for i in range(n_chunks):
            cache.update(k, v, tsis[i], roles=roles[i])  # (one-hot and compact roles, as the role kernels hand them over)
            cache.post_update(C)

    run()  # warm-up: sizes the capacity buffers
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    run()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return {"total_s": wall, "us_per_chunk_step": wall / n_chunks * 1e6, "chunks": n_chunks,
            "cache_rows_after": int(cache.cache_k.shape[2]),
            "note": "host-driven loop: update (one kernel appends the 64 tokens and plans their eviction) + post_update (in-place apply kernel); the plan's result reaches the host through pinned memory before the next append",
            "shape": dict(B=B, Hkv=Hkv, L=L, D=D, C=C, W=W)}


def bench_segments(args, ops):
    """The prefill workload cut into four segments of 8192 tokens over one cache: segment 1 is a first prefill, the
    others attend over the evicted cache plus their own tokens (the multi-segment path); every segment is followed
    by its eviction, as in the caller."""
    from neuralattentionsearch_amd.cache import NAtSChunkLayerCache
    B, Hq, Hkv, D, C, W = 1, 32, 8, 128, 64, 256
    n_seg = args.segments
    seg = args.segment_len if args.segment_len else args.prefill_len // n_seg
    L = n_seg * seg
    dev = "cuda"
    g = torch.Generator(device=dev).manual_seed(0)
    q = (torch.randn(B, Hq, L, D, generator=g, device=dev) / math.sqrt(D)).bfloat16()
    k = (torch.randn(B, Hkv, L, D, generator=g, device=dev) / math.sqrt(D)).bfloat16()
    v = (torch.randn(B, Hkv, L, D, generator=g, device=dev) / math.sqrt(D)).bfloat16()
    roles, tsi = ops.roles_from_logits(biased_role_logits(0, B, L // C, Hkv, (0.05, 0.15, 0.80), dev), ROLE_GLOBAL_BIAS,
                                       True, False)
    sc = seg // C
    parts = [(q[:, :, i * seg:(i + 1) * seg], k[:, :, i * seg:(i + 1) * seg], v[:, :, i * seg:(i + 1) * seg],
              roles[:, :, i * sc:(i + 1) * sc].contiguous(), tsi[:, :, i * sc:(i + 1) * sc].contiguous()) for i in range(n_seg)]
    cache = NAtSChunkLayerCache(B, Hkv, W, chunk_size=C, device=dev)
    seen = {"pairs": 0, "rows": []}

    def run(count: bool = False):
        cache.reset_cache()
        for i, (qs, ks, vs, rs, ts) in enumerate(parts):
            kc, vc = cache.update(ks, vs, ts, roles=rs)  # (roles and one-hot as the role kernel hands them over together)
            if i == 0:
                ops.prefill_attention(qs, kc, vc, rs, C, W)
            else:
                if count:
                    seen["rows"].append(int(kc.shape[2]))
                    if seen["pairs"] is not None and seg * kc.shape[2] * Hkv <= 2 ** 32:
                        # visible (query, key) pairs of this segment, from the mask the kernel implements
                        seen["pairs"] += int(cache.generate_mask(seg).sum().item())
                    else:
                        seen["pairs"] = None  # (the mask would not be worth materialising)
                cache.segment_attention(qs)
            cache.post_update(seg)

    run(count=True)
    flops = None
    if seen["pairs"] is not None and seg * seg * Hkv <= 2 ** 32:
        first_pairs = int(ops.prefill_mask(parts[0][3], seg, C, W).sum().item())
        flops = 4.0 * D * (Hq // Hkv) * (seen["pairs"] + first_pairs)
    wall, ev_mean, ev_min = time_gpu(run, max(3, args.steps // 4), 2)
    return {"ms": ev_mean, "ms_min": ev_min, "ms_wall": wall, "segments": n_seg, "segment_tokens": seg,
            "tokens_per_s": L / (ev_mean * 1e-3),
            "key_rows_of_later_segments": seen["rows"] if n_seg <= 8 else [min(seen["rows"]), max(seen["rows"])],
            "algorithmic_tflop": None if flops is None else flops / 1e12,
            "tflops_visible_pairs": None if flops is None else flops / (ev_mean * 1e-3) / 1e12,
            "note": "per step: segments x (cache update, attention, eviction); FLOPs counted on visible (query, key) "
                    "pairs, not on visited tiles",
            "shape": dict(B=B, Hq=Hq, Hkv=Hkv, L=L, D=D, C=C, W=W)}


def bench_role_step(args, ops):
    """The fused role step (chunk pooling of the hidden states, role projection, argmax, next-global scan) at the
    Llama-3-8B width: a 32768-token prefill and the token that closes a chunk during decoding."""
    B, L, dim, Hkv, C, W = 1, args.prefill_len, 4096, 8, 64, 256
    dev = "cuda"
    g = torch.Generator(device=dev).manual_seed(0)
    x = torch.randn(B, L, dim, generator=g, device=dev).bfloat16()
    w = (torch.randn(Hkv * 3, dim, generator=g, device=dev) * 0.02).bfloat16()
    _, pre_ms, pre_min = time_gpu(lambda: ops.role_step(x, w, C, W, force_first_global=True, with_scan=True), args.steps, 3)
    x1 = x[:, :1].contiguous()
    carry = x[:, 1:2].contiguous()
    _, one_ms, one_min = time_gpu(lambda: ops.role_step(x1, w, C, W, pre_fill=C - 1, carry_in=carry), args.steps, 3)
    nbytes = x.numel() * 2
    return {"prefill_ms": pre_ms, "prefill_ms_min": pre_min, "prefill_gbs": nbytes / (pre_ms * 1e-3) / 1e9,
            "prefill_frac_of_hbm_peak": nbytes / (pre_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, "algorithmic_bytes": nbytes,
            "chunk_closing_token_us": one_ms * 1e3, "chunk_closing_token_us_min": one_min * 1e3,
            "shape": dict(B=B, L=L, dim=dim, Hkv=Hkv, C=C, W=W)}


def bench_matvec(args, ops):
    """The one-token projections of the Llama-3-8B shape through the matrix-vector kernel and through the library,
    one row of x; the weights rotate through about 1.5 GB of copies so that no launch finds them in a cache."""
    shapes = [("qkv", 6144, 4096, False), ("o", 4096, 4096, False), ("gate_up+silu", 14336, 4096, True),
              ("down", 4096, 14336, False), ("lm_head", 128256, 4096, False)]
    dev = "cuda"
    out = {}
    for name, n, k, gate in shapes:
        rows_w = 2 * n if gate else n
        copies = max(2, int(1.5e9 // (rows_w * k * 2)))
        ws = [(torch.randn(rows_w, k, device=dev) * 0.02).bfloat16() for _ in range(copies)]
        x = torch.randn(1, 1, k, device=dev).bfloat16()
        turn = [0]

        def ours():
            turn[0] = (turn[0] + 1) % copies
            return ops.matvec(x, ws[turn[0]], gate=gate)

        def library():
            turn[0] = (turn[0] + 1) % copies
            y = torch.nn.functional.linear(x, ws[turn[0]])
            return ops.silu_mul(y) if gate else y

        _, t_ours, _ = time_gpu(ours, args.steps, 10)
        _, t_lib, _ = time_gpu(library, args.steps, 10)
        nbytes = rows_w * k * 2
        out[name] = {"n_out": n, "k": k, "us": t_ours * 1e3, "gbs": nbytes / (t_ours * 1e-3) / 1e9,
                     "frac_of_hbm_peak": nbytes / (t_ours * 1e-3) / 1e9 / PEAK_HBM_GBS, "library_us": t_lib * 1e3}
        del ws
    return out


def bench_llama(args, chunk_sizes=(64,)):
    """End to end at the Llama-3-8B shape with random weights: one prefill, then greedy decode steps with
    eviction live in all 32 layers.  One set of weights serves every chunk size asked for (chunk size 1 = a role per
    token and the per-token cache class); returns {chunk size: figures}."""
    from neuralattentionsearch_amd.llama import NAtSLlamaConfig, NAtSLlamaForCausalLM
    cfg = NAtSLlamaConfig.llama3_8b(fused_role_step=True)
    model = NAtSLlamaForCausalLM.random_init(cfg, seed=0)
    g = torch.Generator().manual_seed(0)
    ids = torch.randint(0, cfg.vocab_size, (1, args.llama_prefill), generator=g).cuda()
    out = {}
    for C in chunk_sizes:
        cfg.chunk_size = C
        for layer in model.layers:
            layer.self_attn.chunk_size = C
        warm = model.new_cache()
        logits = model(ids[:, :2048], 0, warm)  # loads every kernel and the GEMM heuristics once
        for i in range(3):
            logits = model(logits.argmax(-1, keepdim=True), 2048 + i, warm)
        del warm
        torch.cuda.synchronize()
        torch.cuda.reset_peak_memory_stats()
        mem_before = torch.cuda.memory_allocated()
        cache = model.new_cache()
        t0 = time.perf_counter()
        logits = model(ids, 0, cache)
        torch.cuda.synchronize()
        t_prefill = time.perf_counter() - t0
        peak_prefill = torch.cuda.max_memory_allocated()
        pos = args.llama_prefill
        t0 = time.perf_counter()
        for i in range(args.llama_decode):
            logits = model(logits.argmax(-1, keepdim=True), pos, cache)
            pos += 1
        torch.cuda.synchronize()
        t_decode = time.perf_counter() - t0
        kept = [float(l.valid_tokens[:, :, :l.n_ctx_data].sum().item()) / (cfg.num_key_value_heads * pos) for l in cache.cache_model]
        cache_bytes = sum(t.numel() * t.element_size() for l in cache.cache_model for t in (l._buf_k, l._buf_v, l._buf_valid) if t is not None)
        out[C] = {"prefill_s": t_prefill, "prefill_tokens_per_s": args.llama_prefill / t_prefill,
                  "decode_s": t_decode, "decode_tokens_per_s": args.llama_decode / t_decode,
                  "decode_ms_per_token": t_decode / args.llama_decode * 1e3,
                  "kept_fraction_mean": float(np.mean(kept)), "kept_fraction_min": float(np.min(kept)),
                  "kept_fraction_max": float(np.max(kept)),
                  # what the reference's harness prints beside its timings (experiments/efficiency/eval_efficiency.py:236-250)
                  "max_memory_allocated_gb": torch.cuda.max_memory_allocated() / 1e9,
                  "max_memory_allocated_prefill_gb": peak_prefill / 1e9,
                  "weights_and_inputs_gb": mem_before / 1e9, "kv_cache_after_decode_gb": cache_bytes / 1e9,
                  "shape": dict(layers=cfg.num_hidden_layers, d_model=cfg.hidden_size, heads="32/8", head_dim=cfg.head_dim,
                                ffn=cfg.intermediate_size, vocab=cfg.vocab_size, prefill=args.llama_prefill,
                                decode_steps=args.llama_decode, chunk=C, window=cfg.local_seq_max_length),
                  "note": "random weights give near-uniform roles; prefill projections are library GEMMs; one-token steps use the matrix-vector, fused norm and rotary + append kernels"}
        del cache, logits
    return out


# --------------------------------------------------------------------------------------------------
def cpu_baseline(args):
    """The oracle (a port of the reference's PyTorch path) on this host's cores, bounded samples."""
    from oracle import nats_oracle as orc
    cores = os.cpu_count() or 1
    use = min(cores, 16)  # (the CPU share of a one-GPU box, whatever its core count reads; reported as `cores`)
    torch.set_num_threads(use)
    D, C, W = 128, 64, 256
    samples = {}
    # prefill: one kv-head group (4 q heads) at two lengths, mask generation + SDPA with a bool mask
    for L in (4096, 8192, 16384):
        g = torch.Generator().manual_seed(0)
        q = (torch.randn(1, 4, L, D, generator=g) / math.sqrt(D)).bfloat16()
        k = (torch.randn(1, 1, L, D, generator=g) / math.sqrt(D)).bfloat16()
        v = (torch.randn(1, 1, L, D, generator=g) / math.sqrt(D)).bfloat16()
        roles = draw_roles(0, 1, 1, L // C, (0.05, 0.15, 0.80))
        t0 = time.perf_counter()
        mask = orc.prefill_mask(roles, L, C, W)
        orc.masked_attention(q, k, v, mask)
        samples[L] = time.perf_counter() - t0
    # all eight kv-head groups of the workload at half its length, each with its own roles
    l_big = 16384
    roles8 = draw_roles(0, 1, 8, l_big // C, (0.05, 0.15, 0.80))
    g = torch.Generator().manual_seed(0)
    t_all = 0.0
    for h in range(8):
        q = (torch.randn(1, 4, l_big, D, generator=g) / math.sqrt(D)).bfloat16()
        k = (torch.randn(1, 1, l_big, D, generator=g) / math.sqrt(D)).bfloat16()
        v = (torch.randn(1, 1, l_big, D, generator=g) / math.sqrt(D)).bfloat16()
        t0 = time.perf_counter()
        mask = orc.prefill_mask(roles8[:, h:h + 1], l_big, C, W)
        orc.masked_attention(q, k, v, mask)
        t_all += time.perf_counter() - t0
        del mask
    est_ms = t_all * (32768 / l_big) ** 2 * 1e3  # O(L^2)
    out = {
        "value": est_ms, "unit": "ms", "cores": use, "kind": "port",
        "sample": (f"oracle mask+SDPA, bf16, one kv-head group (4 q heads) at L=4096 {samples[4096]:.2f}s, "
                   f"L=8192 {samples[8192]:.2f}s, L=16384 {samples[16384]:.2f}s; all 8 groups at L=16384 {t_all:.2f}s; "
                   f"value = that x (32768/16384)^2 (extrapolated, the [1,32,32768,32768] bool mask does not fit a host)"),
    }
    # configs[0] whole, the one configuration the reference runs on a CPU: B=1, 8 heads, L=2048, D=64, fp32, chunk 64,
    # window 128, roles = hard argmax of N(0, 1) logits; roles + mask + masked attention
    g = torch.Generator().manual_seed(0)
    q1, k1, v1 = (torch.randn(1, 8, 2048, 64, generator=g) for _ in range(3))
    lg = torch.randn(1, 2048 // 64, 8, 3, generator=g)
    reps, t0 = 0, time.perf_counter()
    while reps < 3 or time.perf_counter() - t0 < 1.0:
        r1 = orc.roles_from_logits(lg, 0.1, True, False)
        orc.masked_attention(q1, k1, v1, orc.prefill_mask(r1, 2048, 64, 128))
        reps += 1
    out["cfg1_whole"] = {"value": (time.perf_counter() - t0) / reps * 1e3, "unit": "ms", "cores": use,
                         "sample": f"configs[0] complete (B=1, H=8, L=2048, D=64, fp32, chunk 64, window 128), mean of {reps} runs"}
    # the same on one core, from the L = 8192 sample
    torch.set_num_threads(1)
    L = 8192
    g = torch.Generator().manual_seed(0)
    q = (torch.randn(1, 4, L, D, generator=g) / math.sqrt(D)).bfloat16()
    k = (torch.randn(1, 1, L, D, generator=g) / math.sqrt(D)).bfloat16()
    v = (torch.randn(1, 1, L, D, generator=g) / math.sqrt(D)).bfloat16()
    roles = draw_roles(0, 1, 1, L // C, (0.05, 0.15, 0.80))
    t0 = time.perf_counter()
    orc.masked_attention(q, k, v, orc.prefill_mask(roles, L, C, W))
    t1 = time.perf_counter() - t0
    torch.set_num_threads(use)
    out["one_core"] = {"value": t1 * (32768 / L) ** 2 * 8 * 1e3, "unit": "ms", "cores": 1,
                       "sample": f"the L=8192 sample on one thread ({t1:.2f}s) x (32768/8192)^2 x 8 groups"}
    # decode: a 2-sequence slice of the batch, scaled linearly to batch 32
    Bs = 2
    q, k, v, valid, n_rows, _ = decode_inputs(Bs, 32, 8, D, C, W, 65536, 0, "cpu")
    t0 = time.perf_counter()
    mask = valid[:, :, None, :n_rows]
    orc.masked_attention(q, k[:, :, :n_rows], v[:, :, :n_rows], mask)
    dt = time.perf_counter() - t0
    out["decode"] = {"tokens_per_s_per_layer": Bs / dt, "cores": use,
                     "sample": f"oracle valid-mask + SDPA on {Bs} of 32 sequences ({dt:.2f}s), same per-head lengths"}
    # eviction: one sequence of the batch through the oracle state machine's gather / scatter
    L = 65536
    g = torch.Generator().manual_seed(0)
    k1 = torch.randn(1, 8, L, D, generator=g).bfloat16()
    v1 = torch.randn(1, 8, L, D, generator=g).bfloat16()
    roles = draw_roles(0, 1, 8, L // C, (0.10, 0.15, 0.75))
    st = orc.ChunkCacheOracle(B=1, H=8, W=512, C=C)
    t0 = time.perf_counter()
    st.update(k1, v1, roles)
    st.post_update(L)
    dt = time.perf_counter() - t0
    out["evict"] = {"ms_for_16_sequences": dt * 16 * 1e3, "cores": 1,
                    "sample": f"oracle update+post_update of 1 of 16 sequences ({dt:.2f}s), scaled x16"}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--prefill-len", type=int, default=32768)
    ap.add_argument("--chunk-size", type=int, default=64, help="chunk size of the prefill leg (the headline uses 64)")
    ap.add_argument("--decode-batch", type=int, default=32, help="sequences of the decode leg (the headline uses 32)")
    ap.add_argument("--decode-context", type=int, default=65536, help="context of the decode leg (the headline uses 65536)")
    ap.add_argument("--head-dim", type=int, default=128, choices=[32, 64, 128, 256],
                    help="head dim of `--only prefill` / `--only decode` (the headline uses 128)")
    ap.add_argument("--skip-cpu", action="store_true")
    ap.add_argument("--no-compare", action="store_true", help="skip the dense comparators of the prefill leg")
    ap.add_argument("--segments", type=int, default=4, help="segments of the `--only segments` leg")
    ap.add_argument("--segment-len", type=int, default=0, help="tokens per segment (default: prefill length / segments)")
    ap.add_argument("--only", choices=["prefill", "decode", "evict", "copy", "evict_stream", "segments", "role_step", "matvec", "llama"], default=None)
    ap.add_argument("--record-traffic", nargs="+", metavar="KEY=FETCH_KIB,WRITE_KIB",
                    help="store counter figures of prefill / decode / evict in bench_traffic.json and exit")
    ap.add_argument("--no-llama", action="store_true", help="skip the end-to-end Llama-3-8B-shape leg of the default run")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the smaller legs of the default run (prefill at chunk 32 / 1, decode at batch 1, streamed eviction, segments, the per-token Llama leg)")
    ap.add_argument("--llama-chunk", type=int, default=64, help="chunk size of `--only llama` (1 = a role per token)")
    ap.add_argument("--llama-prefill", type=int, default=16384)
    ap.add_argument("--llama-decode", type=int, default=512)
    args = ap.parse_args()
    if args.record_traffic:
        record_traffic(args.record_traffic)
        return
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures the one-GPU hot path; it does not run on more than one GPU (--gpus 1 only)",
              file=sys.stderr)
        sys.exit(2)
    from neuralattentionsearch_amd import ops  # raises if the HIP library has not been built

    torch.cuda.set_device(0)
    if args.only == "copy":
        # a plain 1 GiB device copy: the known-size dispatch the FETCH_SIZE / WRITE_SIZE counters are scaled by
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda").random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_bytes": 1 << 30}))
        return
    res = {}
    extras = args.only is None and not args.no_extras  # the smaller legs that ride along in the default run
    if args.only in (None, "prefill"):
        res["prefill"] = bench_prefill(args, ops)
    if extras:
        # the chunk size of the reference's shipped Llama adapter (experiments/configs/finetune_distill.yaml:95) and a
        # role per token, same shape, window and role shares
        # (the clock is settled again before each: the set-up of a leg's inputs leaves the GPU idle for a while)
        few = max(10, args.steps // 2)
        res["prefill_c32"] = bench_prefill(args, ops, chunk_size=32, steps=few, warmup=10, compare=False)
        res["prefill_c1"] = bench_prefill(args, ops, chunk_size=1, steps=few, warmup=10, compare=False)
    if args.only in (None, "decode"):
        res["decode"] = bench_decode(args, ops)
    if extras:
        res["decode_b1"] = bench_decode(args, ops, batch=1, context=65536)  # one sequence: the latency-bound end
    if args.only in (None, "evict"):
        res["evict"] = bench_evict(args, ops)
    if args.only == "evict_stream" or extras:
        res["evict_stream"] = bench_evict_stream(args, ops)
    if args.only == "segments" or extras:
        res["segments"] = bench_segments(args, ops)
    if args.only == "role_step":  # not part of the default run
        res["role_step"] = bench_role_step(args, ops)
    if args.only == "matvec":  # not part of the default run
        res["matvec"] = bench_matvec(args, ops)
    torch.cuda.synchronize()
    cpu = None if args.skip_cpu or args.only in ("evict_stream", "segments", "role_step", "matvec", "llama") else cpu_baseline(args)

    pre = res.get("prefill")
    line = {
        "metric": METRIC,
        "value": pre["ms"] if pre else None,
        "unit": "ms",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": pre["ms"] if pre else None,
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"prefill B=1 Hq=32 Hkv=8 D={args.head_dim} L={args.prefill_len} chunk {args.chunk_size} window 256, roles 5/15/80 "
                               "(global/local/sliding); decode and compaction ride along under their own keys"},
    }
    if pre:
        line["roofline"] = {"bound": "mfma", "achieved": pre["tflops_visited"], "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                            "frac": pre["tflops_visited"] / PEAK_BF16_TFLOPS,
                            "kernel": "prefill_mfma_wide_kernel" if args.head_dim == 256
                                      else f"prefill_mfma_kernel<{args.head_dim}, true, {0 if args.chunk_size >= 64 else 1 if args.chunk_size >= 16 else 2}>"}
        line["roofline"]["traffic"], line["roofline"]["traffic_source"] = (
            measured_traffic("prefill") if (args.prefill_len, args.chunk_size, args.head_dim) == (32768, 64, 128)
            else (None, "not the profiled workload"))
    if "decode" in res:
        d = res["decode"]
        line["roofline_decode"] = {"bound": "hbm", "achieved": d["gbs"], "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                   "frac": d["frac_of_hbm_peak"],
                                   "kernel": f"decode_split_mfma_kernel<{args.head_dim},4> + decode_merge_balanced_kernel"}
        line["roofline_decode"]["traffic"], line["roofline_decode"]["traffic_source"] = (
            measured_traffic("decode") if (args.decode_batch, args.decode_context, args.head_dim) == (32, 65536, 128)
            else (None, "not the profiled workload"))
    if "evict" in res:
        e = res["evict"]
        line["roofline_evict"] = {"bound": "hbm", "achieved": e["gbs"], "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                  "frac": e["frac_of_hbm_peak"],
                                  "kernel": "evict_plan_* + evict_apply_first_kernel (whole post_update)"}
        line["roofline_evict"]["traffic"], line["roofline_evict"]["traffic_source"] = measured_traffic("evict")
    line["cpu_baseline"] = cpu
    if args.only in (None, "llama") and not args.no_llama:
        # the end-to-end workload: last, so that the kernel legs above are timed on a GPU that holds nothing else
        torch.cuda.empty_cache()
        if args.only == "llama":
            r = bench_llama(args, (args.llama_chunk,))
            res["llama_e2e" if args.llama_chunk == 64 else f"llama_e2e_c{args.llama_chunk}"] = r[args.llama_chunk]
        else:
            r = bench_llama(args, (64,) if args.no_extras else (64, 1))
            res["llama_e2e"] = r[64]
            if 1 in r:
                res["llama_e2e_c1"] = r[1]
    line.update(res)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
