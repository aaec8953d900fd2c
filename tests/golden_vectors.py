"""Reader for tests/golden/reference_vectors.npz (outputs of the reference's own compiled
pack / unpack / micro-kernel / gemv / im_2_col code; written by
tests/golden/make_reference_vectors.py).  Inputs are regenerated from their seeds."""
import json
from pathlib import Path

import numpy as np

import oracle

PATH = Path(__file__).resolve().parent / "golden" / "reference_vectors.npz"


def load():
    z = np.load(PATH, allow_pickle=False)
    meta = json.loads(bytes(z["meta"]).decode())
    return meta, z


def blk_dims(values) -> oracle.BlkDims:
    x = oracle.BlkDims()
    for name, v in zip(oracle.BLK_FIELDS, values):
        setattr(x, name, int(v))
    return x
