"""Writes golden vectors for the chunked NAtS layer cache state machine.

Run in the development container only (it imports the reference from /root/reference/src, which
does not exist anywhere else):

    python tests/golden/make_golden.py

What is recorded: for a list of seeded scenarios, the inputs of every ``update`` call (keys, values,
one-hot roles), the bool mask returned by ``generate_mask`` between ``update`` and ``post_update``, and
the full observable state of ``NAtSChunkLayerCache`` after every ``post_update`` (cache_k, cache_v,
valid_tokens, size_global_kv, size_local_kv, n_ctx_data, _n_global_min, sliding_queue_tail,
chunk_fill_size, chunk_fill_size_last, _seen_tokens).

Reference functions exercised (src/nats/components/cache/nats_chunk_layer_cache.py):
update :171-256, _post_update :262-389, move_sliding_window_tokens_to_head :391-437,
_generate_mask :444-511, _generate_local_mask :589-620, _generate_mask_one_step :622-632,
mask_invalid_tokens :634-656, _fit_sliding_queue_masks :658-713, get_updated_cache_info :715-868;
src/nats/components/cache/cache_update.py merge_local_to_global_caches :25-76;
src/nats/components/masks/utils.py generate_hard_seq_masks :81-94.

Keys are position coded (k[b, h, t, :] = 1 + t, t counted over the whole token stream) so that the
surviving-token index map can be read off the compacted cache; values are seeded random floats.
Only data (inputs and outputs) is written; no reference source text is stored.
"""
import json
import math
import os
import sys

import numpy as np
import torch

REF_SRC = "/root/reference/src"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "chunk_cache_golden.npz")

G, LOC, SW = 0, 1, 2


def one_hot(roles: np.ndarray) -> torch.Tensor:
    t = torch.zeros(*roles.shape, 3, dtype=torch.float32)
    t.scatter_(-1, torch.from_numpy(roles.astype(np.int64)).unsqueeze(-1), 1.0)
    return t


def draw_roles(rng, shape, p):
    return rng.choice(3, size=shape, p=p).astype(np.uint8)


def scenarios():
    """Each scenario: dict(name, B, H, D, C, W, segs=[(x_len, role spec)], p=role probabilities).

    A role spec is 'rand', 'all_g', 'all_l', 'all_s' or an explicit nested list [B][H][S]."""
    out = []
    mix = (0.25, 0.35, 0.40)
    # prefill from empty, chunk aligned, then nothing else
    out.append(dict(name="prefill_aligned_c2_w4", B=2, H=3, D=2, C=2, W=4, p=mix, segs=[(24, "rand")]))
    out.append(dict(name="prefill_aligned_c4_w8", B=2, H=2, D=2, C=4, W=8, p=mix, segs=[(64, "rand")]))
    out.append(dict(name="prefill_aligned_c4_w4", B=1, H=4, D=2, C=4, W=4, p=(0.1, 0.2, 0.7), segs=[(96, "rand")]))
    # the worked example: C=2, W=4, L=12, roles G L S G L S
    out.append(dict(name="worked_example", B=1, H=1, D=2, C=2, W=4, p=mix,
                    segs=[(12, [[[G, LOC, SW, G, LOC, SW]]])]))
    # prefill with a partial last chunk (the attention module forces that slot global)
    out.append(dict(name="prefill_partial_c4_w8", B=2, H=3, D=2, C=4, W=8, p=mix, segs=[(43, "rand")]))
    out.append(dict(name="prefill_partial_c2_w4", B=2, H=2, D=2, C=2, W=4, p=mix, segs=[(17, "rand")]))
    # shorter than the window, shorter than one chunk
    out.append(dict(name="prefill_short_lt_w", B=2, H=2, D=2, C=2, W=8, p=mix, segs=[(6, "rand")]))
    out.append(dict(name="prefill_lt_chunk_then_decode", B=1, H=2, D=2, C=4, W=8, p=mix,
                    segs=[(3, "rand")] + [(1, "rand")] * 14))
    # special role patterns
    out.append(dict(name="prefill_all_global", B=1, H=2, D=2, C=2, W=4, p=mix, segs=[(16, "all_g")]))
    out.append(dict(name="prefill_all_local", B=1, H=2, D=2, C=2, W=4, p=mix, segs=[(16, "all_l"), (8, "rand")]))
    out.append(dict(name="prefill_all_sw", B=1, H=2, D=2, C=2, W=4, p=mix, segs=[(16, "all_s"), (8, "rand")]))
    # prefill then one-token decode steps (roles matter only on the step that completes a chunk)
    out.append(dict(name="prefill_decode_c2_w4", B=2, H=3, D=2, C=2, W=4, p=mix,
                    segs=[(16, "rand")] + [(1, "rand")] * 24))
    out.append(dict(name="prefill_decode_c4_w8", B=2, H=2, D=2, C=4, W=8, p=(0.2, 0.2, 0.6),
                    segs=[(32, "rand")] + [(1, "rand")] * 40))
    out.append(dict(name="prefill_partial_decode_c4_w8", B=2, H=2, D=2, C=4, W=8, p=mix,
                    segs=[(30, "rand")] + [(1, "rand")] * 21))
    out.append(dict(name="decode_many_sw_c2_w4", B=1, H=2, D=2, C=2, W=4, p=(0.1, 0.1, 0.8),
                    segs=[(8, "rand")] + [(1, "rand")] * 40))
    # multi-segment prefill, chunk aligned segments, first segment >= W
    out.append(dict(name="multiseg_aligned_c2_w4", B=2, H=3, D=2, C=2, W=4, p=mix,
                    segs=[(16, "rand"), (12, "rand"), (8, "rand"), (2, "rand"), (20, "rand")]))
    out.append(dict(name="multiseg_aligned_c4_w8", B=2, H=2, D=2, C=4, W=8, p=mix,
                    segs=[(32, "rand"), (16, "rand"), (4, "rand"), (40, "rand")]))
    # streaming chunk by chunk
    out.append(dict(name="stream_chunks_c4_w8", B=2, H=2, D=2, C=4, W=8, p=(0.15, 0.25, 0.6),
                    segs=[(4, "rand")] * 24))
    out.append(dict(name="stream_chunks_c2_w8", B=2, H=2, D=2, C=2, W=8, p=mix, segs=[(2, "rand")] * 30))
    # segments that are not chunk aligned (partial chunk pending at the boundary) and a short first segment
    out.append(dict(name="multiseg_unaligned_c4_w8", B=2, H=2, D=2, C=4, W=8, p=mix,
                    segs=[(30, "rand"), (11, "rand"), (7, "rand"), (1, "rand"), (1, "rand"), (13, "rand")]))
    out.append(dict(name="multiseg_first_lt_w_c2_w8", B=1, H=2, D=2, C=2, W=8, p=mix,
                    segs=[(4, "rand"), (6, "rand"), (12, "rand")]))
    # one-token chunks through the chunk class (the container never builds this, the class accepts it)
    out.append(dict(name="chunk1_prefill_decode_w4", B=2, H=2, D=2, C=1, W=4, p=mix, segs=[(19, "rand")] + [(1, "rand")] * 20))
    out.append(dict(name="chunk1_multiseg_w8", B=1, H=3, D=2, C=1, W=8, p=mix,
                    segs=[(24, "rand"), (9, "rand"), (1, "rand"), (1, "rand"), (13, "rand"), (3, "rand")]))
    out.append(dict(name="chunk1_first_lt_w", B=1, H=2, D=2, C=1, W=8, p=(0.15, 0.25, 0.6),
                    segs=[(3, "rand"), (4, "rand")] + [(1, "rand")] * 12 + [(10, "rand")]))
    # chunk sizes that are no power of two (the class only asks for W % C == 0, :47)
    out.append(dict(name="chunk3_prefill_decode_w6", B=2, H=2, D=2, C=3, W=6, p=mix, segs=[(20, "rand")] + [(1, "rand")] * 15))
    out.append(dict(name="chunk6_multiseg_w12", B=2, H=3, D=2, C=6, W=12, p=mix,
                    segs=[(40, "rand"), (13, "rand"), (1, "rand"), (1, "rand"), (22, "rand"), (6, "rand")]))
    out.append(dict(name="chunk12_stream_w24", B=1, H=2, D=2, C=12, W=24, p=(0.15, 0.25, 0.6),
                    segs=[(12, "rand")] * 8 + [(5, "rand"), (30, "rand")]))
    out.append(dict(name="chunk3_first_lt_w12", B=1, H=2, D=2, C=3, W=12, p=mix, segs=[(4, "rand"), (5, "rand"), (20, "rand")]))
    return out


def main():
    sys.path.insert(0, REF_SRC)
    from nats.components.cache.nats_chunk_layer_cache import NAtSChunkLayerCache  # noqa: E402

    arrays = {}
    index = []
    for si, sc in enumerate(scenarios()):
        rng = np.random.default_rng(1000 + si)
        B, H, D, C, W = sc["B"], sc["H"], sc["D"], sc["C"], sc["W"]
        cache = NAtSChunkLayerCache(bsz=B, n_msks=H, sliding_window_size=W, chunk_size=C,
                                    device=torch.device("cpu"))
        t_seen = 0
        fill = 0
        ops = []
        for oi, (x_len, spec) in enumerate(sc["segs"]):
            n_slots = math.ceil((fill + x_len) / C)
            completes = (fill + x_len) >= C
            partial = (fill + x_len) % C
            if not completes:
                # what the attention module hands over while a chunk is still open: a global placeholder
                roles = np.zeros((B, H, 1), dtype=np.uint8)
            else:
                if spec == "rand":
                    roles = draw_roles(rng, (B, H, n_slots), sc["p"])
                elif spec == "all_g":
                    roles = np.full((B, H, n_slots), G, np.uint8)
                elif spec == "all_l":
                    roles = np.full((B, H, n_slots), LOC, np.uint8)
                elif spec == "all_s":
                    roles = np.full((B, H, n_slots), SW, np.uint8)
                else:
                    roles = np.asarray(spec, dtype=np.uint8)
                    assert roles.shape == (B, H, n_slots)
                if isinstance(spec, str) and spec == "rand":
                    if t_seen == 0:
                        roles[:, :, 0] = G  # sink chunk
                    if partial:
                        roles[:, :, -1] = G  # open chunk is marked global by the module
            pos = torch.arange(t_seen, t_seen + x_len, dtype=torch.float32).view(1, 1, -1, 1) + 1.0
            k = pos.expand(B, H, x_len, D).contiguous()
            v = torch.from_numpy(rng.standard_normal((B, H, x_len, D)).astype(np.float32))
            tsi = one_hot(roles)
            pre = f"s{si}__o{oi}__"
            arrays[pre + "roles"] = roles
            arrays[pre + "v"] = v.numpy().copy()
            cache.update(k.clone(), v.clone(), tsi.clone())
            mask = cache.generate_mask(x_len)
            arrays[pre + "mask"] = np.packbits(mask.numpy().astype(np.uint8), axis=-1)
            arrays[pre + "mask_shape"] = np.asarray(mask.shape, dtype=np.int64)
            cache.post_update(x_len)
            arrays[pre + "cache_k"] = cache.cache_k.numpy().copy()
            arrays[pre + "cache_v"] = cache.cache_v.numpy().copy()
            arrays[pre + "valid"] = cache.valid_tokens.numpy().copy()
            arrays[pre + "size_global"] = cache.size_global_kv.numpy().copy()
            arrays[pre + "size_local"] = cache.size_local_kv.numpy().copy()
            arrays[pre + "scalars"] = np.asarray(
                [int(cache.n_ctx_data), int(cache._n_global_min), int(cache.sliding_queue_tail),
                 int(cache.chunk_fill_size), int(cache.chunk_fill_size_last), int(cache._seen_tokens)],
                dtype=np.int64)
            ops.append(dict(x_len=x_len, n_slots=int(roles.shape[-1])))
            t_seen += x_len
            fill = (fill + x_len) % C if completes else fill + x_len
        index.append(dict(name=sc["name"], B=B, H=H, D=D, C=C, W=W, ops=ops))
    arrays["index_json"] = np.frombuffer(json.dumps(index).encode(), dtype=np.uint8)
    np.savez_compressed(OUT, **arrays)
    print(f"wrote {OUT}: {len(index)} scenarios, {sum(len(s['ops']) for s in index)} ops, "
          f"{os.path.getsize(OUT) / 1024:.1f} KiB")


if __name__ == "__main__":
    main()
