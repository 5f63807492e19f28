"""
Writes the golden vectors in this directory.

The reference holds no data fixtures for this path, and it is not imported here.  The vectors come from the
textbook formulation evaluated by torch in float64 with autograd (oracle.cpu_attention.dense_attention_f64:
masked softmax of q.k + log quad_weight, times v), on neighborhoods built by the brute-force haversine
construction (oracle.geometry.neighborhood_csr_bruteforce) - neither shares code with the C oracle or the
HIP kernels, which are both checked against these files.

    python tests/golden/make_golden.py
"""

import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import cpu_attention as o  # noqa: E402
from oracle import geometry as g  # noqa: E402

CASES = {
    # name: (B, nh, ck, cv, in_shape, out_shape, grid_in, grid_out, theta_cutoff, seed)
    "self_eq_12x24_h2": (2, 2, 4, 4, (12, 24), (12, 24), "equiangular", "equiangular", 0.45, 333),
    "down2_eq_to_lg_h2": (2, 2, 8, 4, (12, 24), (6, 12), "equiangular", "legendre-gauss", 0.6, 334),
    "down3_odd_h1": (1, 1, 3, 5, (9, 12), (5, 4), "equiangular", "equiangular", None, 335),
    "self_lobatto_pole_heavy": (1, 4, 2, 2, (8, 32), (8, 32), "lobatto", "lobatto", 0.9, 336),
}


def main():
    for name, (B, nh, ck, cv, ins, outs, gi, go, tc, seed) in CASES.items():
        col, roff = g.neighborhood_csr_bruteforce(ins, outs, gi, go, tc)
        col, roff = torch.as_tensor(col), torch.as_tensor(roff)
        w = g.attention_quad_weights(ins[0], ins[1], gi)
        gen = torch.Generator().manual_seed(seed)
        k = torch.randn(B, ins[0], ins[1], nh * ck, generator=gen)
        v = torch.randn(B, ins[0], ins[1], nh * cv, generator=gen)
        q = torch.randn(B, outs[0], outs[1], nh * ck, generator=gen) / ck**0.5
        dy = torch.randn(B, outs[0], outs[1], nh * cv, generator=gen)
        kd, vd, qd = [t.double().requires_grad_(True) for t in (k, v, q)]
        y = o.dense_attention_f64(kd, vd, qd, w, col, roff, nh)
        y.backward(dy.double())
        np.savez_compressed(
            os.path.join(HERE, name + ".npz"),
            k=k.numpy(), v=v.numpy(), q=q.numpy(), dy=dy.numpy(), quad_weights=w.numpy(), col_idx=col.numpy(), row_off=roff.numpy(),
            num_heads=np.int64(nh), y=y.detach().numpy(), dk=kd.grad.numpy(), dv=vd.grad.numpy(), dq=qd.grad.numpy(),
        )  # fmt: skip
        print(name, "nnz", col.numel(), "y", tuple(y.shape))


if __name__ == "__main__":
    main()
