"""Reader for tests/golden/chunk_cache_golden.npz (written by tests/golden/make_golden.py)."""
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
