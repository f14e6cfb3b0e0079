"""Writes golden vectors for the per-token NAtS layer cache (chunk_size == 1: NAtSLayerCache).

Run in the development container only (it imports the reference from /root/reference/src, which does not exist
anywhere else):

    python tests/golden/make_golden_token.py

What is recorded: for a list of seeded scenarios, the inputs of every ``update`` call (values, roles; keys are
position coded), the bool mask ``generate_mask`` returns between ``update`` and ``post_update``, and the observable
state of ``NAtSLayerCache`` after every ``post_update`` (cache_k, cache_v, valid_tokens, size_global_kv,
size_local_kv, n_ctx_data, _n_global_min, sliding_queue_tail, chunk_fill_size, chunk_fill_size_last, _seen_tokens).

Reference functions exercised (src/nats/components/cache/nats_layer_cache.py): update :167-286, _post_update
:292-418, move_sliding_window_tokens_to_head :424-458, _generate_mask :469-517, _generate_local_mask :519-542,
_generate_mask_one_step :544-554, mask_invalid_tokens :556-574, _fit_sliding_queue_masks :603-649,
get_updated_cache_info :651-770; src/nats/components/cache/cache_update.py merge_local_to_global_caches :25-76;
src/nats/components/masks/utils.py generate_hard_seq_masks :81-94.

Two things are done to make that module importable and runnable on this CPU-only host, neither of which touches the
class's own code:

* nats_layer_cache.py:16 imports ``post_update_one_step`` from ``nats.components.cache.triton.update_one_step``, a
  module the reference checkout does not contain.  The class never calls that name, so an empty placeholder module
  with a function of that name that raises is registered in ``sys.modules`` before the import.
* ``mask_invalid_tokens`` is decorated with ``@torch.compile`` (:556); TORCHDYNAMO_DISABLE=1 makes the decorator
  return the plain Python function, which runs the same torch ops eagerly.

Keys are position coded (k[b, h, t, :] = 1 + t over the whole token stream); values are seeded random integers
stored as floats.  Per scenario and kind of array the calls are stored back to back in one flat array; the index
holds their shapes.
A scenario in which the reference itself raises is recorded with the calls made up to that point and the
exception's type (``error`` in the index).  Only data (inputs and outputs) is written; no reference source text.
"""
import json
import os
import sys
import types

os.environ["TORCHDYNAMO_DISABLE"] = "1"

import numpy as np  # noqa: E402
import torch  # noqa: E402

REF_SRC = "/root/reference/src"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "token_cache_golden.npz")

G, LOC, SW = 0, 1, 2


def one_hot(roles: np.ndarray) -> torch.Tensor:
    t = torch.zeros(*roles.shape, 3, dtype=torch.float32)
    t.scatter_(-1, torch.from_numpy(roles.astype(np.int64)).unsqueeze(-1), 1.0)
    return t


def scenarios():
    """Each scenario: dict(name, B, H, D, W, U, p, segs=[(x_len, role spec)]).  U is the update chunk size (16 is
    what NAtSCache constructs).  A role spec is 'rand', 'all_g', 'all_l', 'all_s' or a probability triple."""
    mix = (0.25, 0.35, 0.40)
    sw_heavy = (0.1, 0.1, 0.8)
    out = []
    one = lambda n, spec="rand": [(1, spec)] * n
    # prefill, then one-token steps across several deferred updates
    out.append(dict(name="prefill40_decode_w16", B=2, H=3, W=16, p=mix, segs=[(40, "rand")] + one(50)))
    out.append(dict(name="prefill64_decode_w32", B=2, H=2, W=32, p=mix, segs=[(64, "rand")] + one(70)))
    out.append(dict(name="prefill33_decode_w16_swheavy", B=1, H=4, W=16, p=sw_heavy, segs=[(33, "rand")] + one(40)))
    # prefill lengths around the update chunk size and the window
    out.append(dict(name="prefill16_w16", B=2, H=2, W=16, p=mix, segs=[(16, "rand")] + one(20)))
    out.append(dict(name="prefill17_w32", B=2, H=2, W=32, p=mix, segs=[(17, "rand")] + one(36)))
    out.append(dict(name="prefill20_w64_lt_window", B=1, H=3, W=64, p=mix, segs=[(20, "rand")] + one(80)))
    out.append(dict(name="prefill100_w64", B=1, H=2, W=64, p=mix, segs=[(100, "rand")] + one(20)))
    # fewer tokens than one update chunk first, the first deferred update happens while decoding
    out.append(dict(name="prefill5_decode_w16", B=2, H=2, W=16, p=mix, segs=[(5, "rand")] + one(45)))
    out.append(dict(name="decode_from_empty_w16", B=1, H=2, W=16, p=mix, segs=one(50)))
    out.append(dict(name="decode_from_empty_w32", B=2, H=2, W=32, p=sw_heavy, segs=one(70)))
    # special role patterns
    out.append(dict(name="all_global", B=1, H=2, W=16, p=mix, segs=[(32, "all_g")] + one(20, "all_g")))
    out.append(dict(name="all_local_then_mix", B=1, H=2, W=16, p=mix, segs=[(32, "all_l")] + one(16, "all_l") + one(20)))
    out.append(dict(name="all_sw_then_mix", B=1, H=2, W=16, p=mix, segs=[(32, "all_s")] + one(16, "all_s") + one(36)))
    out.append(dict(name="mix_then_all_sw_block", B=2, H=2, W=16, p=mix,
                    segs=[(32, "rand")] + one(16, "all_s") + one(16) + one(16, "all_s") + one(16, "all_s") + one(20)))
    out.append(dict(name="no_global_after_first", B=1, H=3, W=16, p=(0.0, 0.5, 0.5), segs=[(48, "rand")] + one(40)))
    # several multi-token segments
    out.append(dict(name="multiseg_w16", B=2, H=3, W=16, p=mix,
                    segs=[(48, "rand"), (20, "rand"), (16, "rand"), (7, "rand"), (3, "rand"), (33, "rand")] + one(20)))
    out.append(dict(name="multiseg_w32", B=2, H=2, W=32, p=mix,
                    segs=[(64, "rand"), (40, "rand"), (5, "rand"), (5, "rand"), (5, "rand"), (5, "rand"), (50, "rand")]))
    out.append(dict(name="multiseg_pending_then_segment", B=1, H=2, W=16, p=mix,
                    segs=[(32, "rand")] + one(5) + [(9, "rand")] + one(3) + [(30, "rand")] + one(7) + [(2, "rand"), (2, "rand")]))
    out.append(dict(name="multiseg_first_lt_window", B=1, H=2, W=64, p=mix,
                    segs=[(24, "rand"), (10, "rand"), (40, "rand"), (70, "rand")] + one(10)))
    out.append(dict(name="multiseg_first_lt_update_chunk", B=2, H=2, W=16, p=mix,
                    segs=[(6, "rand"), (4, "rand"), (9, "rand"), (20, "rand")] + one(10)))
    out.append(dict(name="segments_longer_than_window", B=1, H=2, W=16, p=mix,
                    segs=[(40, "rand"), (40, "rand"), (17, "rand"), (16, "rand")] + one(5)))
    out.append(dict(name="multiseg_after_all_sw", B=1, H=2, W=16, p=mix,
                    segs=[(32, "rand"), (16, "all_s"), (12, "rand"), (20, "rand")] + one(8)))
    # streaming in blocks of exactly one update chunk
    out.append(dict(name="stream_blocks_w16", B=2, H=2, W=16, p=(0.15, 0.25, 0.6), segs=[(16, "rand")] * 12))
    # other update chunk sizes the class accepts (W >= U)
    out.append(dict(name="update_chunk4_w8", B=2, H=2, W=8, U=4, p=mix, segs=[(11, "rand")] + one(13) + [(6, "rand"), (9, "rand")] + one(6)))
    out.append(dict(name="update_chunk8_w8", B=1, H=3, W=8, U=8, p=mix, segs=[(20, "rand")] + one(20) + [(10, "rand")] + one(9)))
    # update chunk 1: nothing is deferred; a one-token step that is not sliding-window on every head takes the one-step
    # branch (:328-367), which NAtSCache never constructs (dyn_cache.py:183-185 leaves the default of 16)
    out.append(dict(name="update_chunk1_w8", B=2, H=3, W=8, U=1, p=mix, segs=[(11, "rand")] + one(30)))
    out.append(dict(name="update_chunk1_decode_from_empty_w4", B=2, H=2, W=4, U=1, p=mix, segs=one(30)))
    out.append(dict(name="update_chunk1_w2_swheavy", B=1, H=3, W=2, U=1, p=sw_heavy, segs=one(24)))
    out.append(dict(name="update_chunk1_special_roles_w8", B=1, H=2, W=8, U=1, p=mix,
                    segs=[(9, "rand")] + one(4, "all_s") + one(6) + one(3, "all_l") + one(3, "all_g") + one(5, "all_s")
                    + one(8)))
    out.append(dict(name="update_chunk1_multiseg_w8", B=2, H=2, W=8, U=1, p=mix,
                    segs=one(3) + [(5, "rand")] + one(4) + [(12, "rand"), (2, "rand")] + one(6) + [(3, "all_s")] + one(5)))
    for sc in out:
        sc.setdefault("D", 2)
        sc.setdefault("U", 16)
    return out


def draw(rng, spec, shape, p):
    if spec == "rand":
        return rng.choice(3, size=shape, p=p).astype(np.uint8)
    if spec == "all_g":
        return np.full(shape, G, np.uint8)
    if spec == "all_l":
        return np.full(shape, LOC, np.uint8)
    if spec == "all_s":
        return np.full(shape, SW, np.uint8)
    return rng.choice(3, size=shape, p=spec).astype(np.uint8)


def main():
    sys.path.insert(0, REF_SRC)
    stub_pkg = types.ModuleType("nats.components.cache.triton")
    stub_pkg.__path__ = []
    stub = types.ModuleType("nats.components.cache.triton.update_one_step")

    def post_update_one_step(*a, **k):
        raise RuntimeError("placeholder for a module the reference checkout does not contain")

    stub.post_update_one_step = post_update_one_step
    sys.modules["nats.components.cache.triton"] = stub_pkg
    sys.modules["nats.components.cache.triton.update_one_step"] = stub
    from nats.components.cache.nats_layer_cache import NAtSLayerCache  # noqa: E402

    arrays = {}
    index = []
    for si, sc in enumerate(scenarios()):
        rng = np.random.default_rng(5000 + si)
        B, H, D, W, U = sc["B"], sc["H"], sc["D"], sc["W"], sc["U"]
        cache = NAtSLayerCache(bsz=B, n_msks=H, sliding_window_size=W, update_chunk_size=U, device=torch.device("cpu"))
        t_seen = 0
        ops = []
        error = None
        packed = {}  # kind -> list of arrays, one per call; stored as one flat array per scenario and kind
        shapes = {}

        def put(kind, a):
            a = np.array(a, copy=True, order="C")  # a snapshot: the live tensors are updated in place later
            packed.setdefault(kind, []).append(a.reshape(-1))
            shapes.setdefault(kind, []).append(list(a.shape))
        for oi, (x_len, spec) in enumerate(sc["segs"]):
            roles = draw(rng, spec, (B, H, x_len), sc["p"])
            if t_seen == 0 and spec == "rand":
                roles[:, :, 0] = G  # the sink token (nats_attention.py:103-104)
            pos = torch.arange(t_seen, t_seen + x_len, dtype=torch.float32).view(1, 1, -1, 1) + 1.0
            k = pos.expand(B, H, x_len, D).contiguous()
            v = torch.from_numpy(rng.integers(-99, 100, size=(B, H, x_len, D)).astype(np.float32))
            try:
                cache.update(k.clone(), v.clone(), one_hot(roles))
                mask = cache.generate_mask(x_len).clone()  # (a one-token mask is a view of valid_tokens)
                cache.post_update(x_len)
            except Exception as e:  # the reference itself fails in this regime: keep what came before
                error = f"{type(e).__name__} at op {oi}"
                break
            put("roles", roles)
            put("v", v.numpy())
            put("mask", np.packbits(mask.numpy().astype(np.uint8), axis=-1))
            put("mask_shape", np.asarray(mask.shape, dtype=np.int64))
            put("cache_k", cache.cache_k.numpy())
            put("cache_v", cache.cache_v.numpy())
            put("valid", cache.valid_tokens.numpy())
            put("size_global", cache.size_global_kv.numpy())
            put("size_local", cache.size_local_kv.numpy())
            put("scalars", np.asarray(
                [int(cache.n_ctx_data), int(cache._n_global_min), int(cache.sliding_queue_tail),
                 int(cache.chunk_fill_size), int(cache.chunk_fill_size_last), int(cache._seen_tokens)], dtype=np.int64))
            ops.append(dict(x_len=x_len))
            t_seen += x_len
        for kind, parts in packed.items():
            arrays[f"s{si}__{kind}"] = np.concatenate(parts)
        index.append(dict(name=sc["name"], B=B, H=H, D=D, W=W, U=U, ops=ops, error=error, shapes=shapes))
        print(f"{sc['name']}: {len(ops)} of {len(sc['segs'])} calls" + (f"  [{error}]" if error else ""))
    arrays["index_json"] = np.frombuffer(json.dumps(index).encode(), dtype=np.uint8)
    np.savez_compressed(OUT, **arrays)
    print(f"wrote {OUT}: {len(index)} scenarios, {sum(len(s['ops']) for s in index)} calls, "
          f"{os.path.getsize(OUT) / 1024:.1f} KiB")


if __name__ == "__main__":
    main()
