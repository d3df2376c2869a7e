"""Loader of the committed fixtures in tests/golden/fa_cases.npz."""
import os

import numpy as np

_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fa_cases.npz")


def load_cases():
    blob = np.load(_PATH, allow_pickle=False)
    cases = {}
    for key in blob.files:
        name, field = key.split("/", 1)
        cases.setdefault(name, {})[field] = blob[key]
    for c in cases.values():
        if "drop_mask" in c:
            Sk = c["k"].shape[2]
            c["drop_mask"] = np.unpackbits(c["drop_mask"], axis=-1)[..., :Sk]
    return cases
