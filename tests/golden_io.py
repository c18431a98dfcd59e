"""Loader for tests/golden/kat_*.npz (written by tests/golden/make_golden.py)."""
import glob
import os
from types import SimpleNamespace

import numpy as np
import torch

GOLDEN_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def names():
    return sorted(os.path.basename(p)[4:-4] for p in glob.glob(os.path.join(GOLDEN_DIR, "kat_*.npz")))


def load(name):
    z = np.load(os.path.join(GOLDEN_DIR, f"kat_{name}.npz"), allow_pickle=False)
    S = int(z["S"])
    mask = np.unpackbits(z["mask"], axis=-1)[:, :S].astype(bool)
    bf = lambda a: torch.from_numpy(a.copy()).view(torch.bfloat16)  # noqa: E731
    meta = SimpleNamespace(unmasked_kv_ids=z["unmasked_kv_ids"], unmasked_lens=z["unmasked_lens"],
                           masked_kv_ids=z["masked_kv_ids"], masked_lens=z["masked_lens"])
    return SimpleNamespace(name=name, S=S, B=int(z["B"]), H=int(z["H"]), D=int(z["D"]), BQ=int(z["BQ"]), BK=int(z["BK"]),
                           mask=mask, q=bf(z["q"]), k=bf(z["k"]), v=bf(z["v"]), meta=meta, out=z["out_fp64"])
