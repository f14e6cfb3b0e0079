"""Readers for tests/golden/chunk_cache_golden.npz (written by tests/golden/make_golden.py) and
tests/golden/token_cache_golden.npz (written by tests/golden/make_golden_token.py)."""
import json
import os

import numpy as np

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "chunk_cache_golden.npz")


class Golden:
    def __init__(self):
        self.z = np.load(PATH, allow_pickle=False)
        self.index = json.loads(bytes(self.z["index_json"]).decode())

    def scenario_names(self):
        return [s["name"] for s in self.index]

    def scenario(self, name):
        for si, s in enumerate(self.index):
            if s["name"] == name:
                return si, s
        raise KeyError(name)

    def op(self, si, oi):
        pre = f"s{si}__o{oi}__"
        d = {k[len(pre):]: self.z[k] for k in self.z.files if k.startswith(pre)}
        shape = tuple(int(x) for x in d["mask_shape"])
        bits = np.unpackbits(d["mask"], axis=-1)[..., :shape[-1]].astype(bool)
        d["mask"] = bits.reshape(shape)
        return d


TOKEN_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "token_cache_golden.npz")


class TokenGolden:
    """Vectors of the reference's per-token cache class.  Per scenario and kind of array the calls are stored back
    to back in one flat array; the index holds the shape of every call's array."""

    def __init__(self):
        self.z = np.load(TOKEN_PATH, allow_pickle=False)
        self.index = json.loads(bytes(self.z["index_json"]).decode())
        self._split = {}

    def scenario_names(self):
        return [s["name"] for s in self.index]

    def scenario(self, name):
        for si, s in enumerate(self.index):
            if s["name"] == name:
                return si, s
        raise KeyError(name)

    def _parts(self, si, kind):
        key = (si, kind)
        if key not in self._split:
            flat = self.z[f"s{si}__{kind}"]
            out, at = [], 0
            for shape in self.index[si]["shapes"][kind]:
                n = int(np.prod(shape))
                out.append(flat[at:at + n].reshape(shape))
                at += n
            assert at == flat.size
            self._split[key] = out
        return self._split[key]

    def op(self, si, oi):
        d = {kind: self._parts(si, kind)[oi] for kind in self.index[si]["shapes"]}
        shape = tuple(int(x) for x in d["mask_shape"])
        bits = np.unpackbits(d["mask"], axis=-1)[..., :shape[-1]].astype(bool)
        d["mask"] = bits.reshape(shape)
        return d
