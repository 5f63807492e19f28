import glob
import os

import numpy as np
import torch

GOLDEN_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
# vectors whose expected outputs were computed by the reference's own CPU operators (tests/golden/make_reference_golden.py)
REFERENCE_DIR = os.path.join(GOLDEN_DIR, "reference_cpu")


def golden_names():
    return sorted(os.path.splitext(os.path.basename(p))[0] for p in glob.glob(os.path.join(GOLDEN_DIR, "*.npz")))


def reference_golden_names():
    return sorted(os.path.splitext(os.path.basename(p))[0] for p in glob.glob(os.path.join(REFERENCE_DIR, "*.npz")))


def load_golden(name, directory=GOLDEN_DIR):
    with np.load(os.path.join(directory, name + ".npz"), allow_pickle=False) as z:
        d = {k: torch.from_numpy(z[k]) for k in z.files if k != "num_heads"}
        d["num_heads"] = int(z["num_heads"])
    return d
