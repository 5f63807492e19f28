"""
Writes tests/golden/reference_cpu/*.npz: inputs and the outputs of the reference's OWN CPU operators on them.

The operators are `attention_kernels::forward` / `backward` of the reference (attention_interface.cpp:114-119), compiled
from its CPU sources by `make -C oracle ref` into oracle/_ref/attention_ref.so and run in a child process
(oracle/reference_ops.py).  That build only exists where the reference's sources are present; the vectors are committed
so that the C oracle and the HIP path are held against the reference's results everywhere else too.  Up-sampling cases
carry psi keyed by the input grid, as the reference's module builds it (attention.py:383-401).

    make -C oracle ref && python tests/golden/make_reference_golden.py
"""

import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import geometry as g  # noqa: E402
from oracle import reference_ops as ref  # noqa: E402

CASES = {
    # name: (B, nh, ck, cv, in_shape, out_shape, grid_in, grid_out, theta_cutoff, seed)
    "self_eq_12x24_h2_d8": (1, 2, 8, 8, (12, 24), (12, 24), "equiangular", "equiangular", None, 433),
    "down2_eq_to_lg_ck5_cv7": (1, 3, 5, 7, (13, 32), (7, 16), "equiangular", "legendre-gauss", None, 434),
    "up2_eq_ck8_cv4": (1, 2, 8, 4, (7, 16), (13, 32), "equiangular", "equiangular", None, 435),
    "up3_eq_to_lg": (2, 1, 5, 5, (5, 12), (9, 36), "equiangular", "legendre-gauss", 0.7, 436),
    "self_eq_8x64_d32": (1, 1, 32, 32, (8, 64), (8, 64), "equiangular", "equiangular", 0.5, 437),  # 64 longitudes, 32 channels: the hybrid matrix-core kernels
    "self_lg_12x32_d16": (1, 1, 16, 16, (12, 32), (12, 32), "legendre-gauss", "legendre-gauss", None, 438),  # the fp32 16-longitude family
    "down2_eq_6x64_d40": (1, 1, 40, 40, (6, 64), (3, 32), "equiangular", "equiangular", 0.9, 439),  # a head narrower than its tile, virtual latitudes
}


def main():
    if not ref.available():
        raise SystemExit("oracle/_ref/attention_ref.so is missing: run `make -C oracle ref` where the reference's sources are present")
    out_dir = os.path.join(HERE, "reference_cpu")
    os.makedirs(out_dir, exist_ok=True)
    inputs, jobs = {}, []
    for name, (B, nh, ck, cv, ins, outs, gi, go, tc, seed) in CASES.items():
        up = outs[1] > ins[1]
        col, roff = g.neighborhood_csr(outs, ins, go, gi, tc) if up else g.neighborhood_csr(ins, outs, gi, go, tc)
        w = g.attention_quad_weights(ins[0], ins[1], gi)
        gen = torch.Generator().manual_seed(seed)
        k = torch.randn(B, ins[0], ins[1], nh * ck, generator=gen)
        v = torch.randn(B, ins[0], ins[1], nh * cv, generator=gen)
        q = torch.randn(B, outs[0], outs[1], nh * ck, generator=gen) / ck**0.5
        dy = torch.randn(B, outs[0], outs[1], nh * cv, generator=gen)
        inputs[name] = (k, v, q, dy, w, col, roff, nh)
        jobs.append(ref.forward_job(k, v, q, w, col, roff, nh))
        jobs.append(ref.backward_job(k, v, q, dy, w, col, roff, nh))
    res = ref.run(jobs)
    for i, (name, (k, v, q, dy, w, col, roff, nh)) in enumerate(inputs.items()):
        y, (dk, dv, dq) = res[2 * i]["out"][0], res[2 * i + 1]["out"]
        np.savez_compressed(
            os.path.join(out_dir, name + ".npz"),
            k=k.numpy(), v=v.numpy(), q=q.numpy(), dy=dy.numpy(), quad_weights=w.numpy(), col_idx=col.numpy(), row_off=roff.numpy(),
            num_heads=np.int64(nh), y=y.numpy(), dk=dk.numpy(), dv=dv.numpy(), dq=dq.numpy(),
        )  # fmt: skip
        print(name, "nnz", col.numel(), "y", tuple(y.shape), y.dtype)


if __name__ == "__main__":
    main()
