"""
The oracle against the reference's OWN CPU operators.

`make -C oracle ref` compiles the reference's CPU path (attention_interface.cpp, kernels_cpu/attention_cpu_{fwd,bwd}.cpp,
their _upsample counterparts and attention_cpu_permute.cpp) from its sources into oracle/_ref/attention_ref.so; the
operators run in a child process (oracle/reference_ops.py).  Skipped where that library has not been built.

Gather direction (self-attention and down-sampling): the C restatement (strict and release-flag builds, and the float64
spec) against `attention_kernels::forward` / `backward` on the same seeded inputs.  Up-sampling direction: the dense
float64 formulation that pins the oracle there against the reference's up-sampling CPU kernels.  Tolerance: the
reference computes in fp32, so rtol = atol = 1e-5 against the float64 results and between the two fp32 builds.
"""

import math

import pytest
import torch

from oracle import cpu_attention as o
from oracle import geometry as g
from oracle import reference_ops as ref
from tests.util import CONFIGS, randn_inputs

pytestmark = pytest.mark.skipif(not ref.available(), reason="oracle/_ref/attention_ref.so is not built (make -C oracle ref)")

GATHER = [
    # B, nh, ck, cv, in_shape, out_shape, grid_in, grid_out, theta_cutoff  (shapes of the reference's tests/test_attention.py:66-80 and more)
    (2, 2, 4, 3, (12, 24), (6, 12), "equiangular", "legendre-gauss", 0.6),
    (1, 1, 1, 1, (6, 12), (6, 12), "equiangular", "equiangular", None),
    (2, 3, 2, 4, (9, 12), (5, 4), "equiangular", "equiangular", None),
    (1, 2, 8, 8, (10, 20), (10, 20), "lobatto", "lobatto", 0.5),
    (1, 4, 16, 16, (12, 24), (12, 24), "equiangular", "equiangular", None),
    (1, 1, 33, 17, (7, 16), (7, 16), "legendre-gauss", "legendre-gauss", None),
    (1, 2, 4, 4, (8, 16), (8, 16), "equiangular", "equiangular", 2 * math.pi),  # every point a neighbor
    (1, 1, 16, 16, (32, 64), (32, 64), "equiangular", "equiangular", None),  # the first benchmark configuration
]
UPSAMPLE = [
    (1, 2, 8, 4, (7, 16), (13, 32), "equiangular", "equiangular", None),
    (2, 1, 5, 5, (5, 12), (9, 36), "equiangular", "legendre-gauss", 0.7),
    (1, 3, 4, 6, (6, 8), (12, 16), "legendre-gauss", "equiangular", None),
]


def _inputs(case, up):
    B, nh, ck, cv, ins, outs, gi, go, tc = case
    col, roff = g.neighborhood_csr(outs, ins, go, gi, tc) if up else g.neighborhood_csr(ins, outs, gi, go, tc)  # up-sampling: rows index the input grid
    w = g.attention_quad_weights(ins[0], ins[1], gi)
    k, v, q, dy = randn_inputs(B, ins[0], ins[1], outs[0], outs[1], nh, ck, cv)
    return k, v, q, dy, w, col, roff, nh


@pytest.fixture(scope="module")
def reference_results():
    """All cases through ONE child process: [(y, dk, dv, dq)] in the order GATHER + UPSAMPLE."""
    jobs = []
    for case, up in [(c, False) for c in GATHER] + [(c, True) for c in UPSAMPLE]:
        k, v, q, dy, w, col, roff, nh = _inputs(case, up)
        jobs.append(ref.forward_job(k, v, q, w, col, roff, nh))
        jobs.append(ref.backward_job(k, v, q, dy, w, col, roff, nh))
    res = ref.run(jobs)
    return [(res[2 * i]["out"][0], *res[2 * i + 1]["out"]) for i in range(len(jobs) // 2)]


def _close(name, got, want, tol=1e-5):
    got, want = got.double(), want.detach().double()
    assert got.shape == want.shape, name
    err = (got - want).abs()
    assert bool((err <= tol + tol * want.abs()).all()), f"{name}: max |err| {err.max().item():.3e}"


@pytest.mark.parametrize("idx", range(len(GATHER)))
def test_restatement_matches_the_reference_cpu_operators(reference_results, idx):
    k, v, q, dy, w, col, roff, nh = _inputs(GATHER[idx], False)
    y_r, dk_r, dv_r, dq_r = reference_results[idx]
    assert y_r.dtype == torch.float32 and y_r.shape == (k.shape[0], q.shape[1], q.shape[2], v.shape[3])
    y64 = o.forward_f64(k, v, q, w, col, roff, nh)
    dk64, dv64, dq64 = o.backward_f64(k, v, q, dy, w, col, roff, nh)
    for name, got, want in (("y", y_r, y64), ("dk", dk_r, dk64), ("dv", dv_r, dv64), ("dq", dq_r, dq64)):
        _close(f"reference vs float64 spec, {name}", got, want)
    for fast in (False, True):
        y32 = o.forward_f32(k, v, q, w, col, roff, nh, fast=fast)
        dk32, dv32, dq32 = o.backward_f32(k, v, q, dy, w, col, roff, nh, fast=fast)
        for name, got, want in (("y", y32, y_r), ("dk", dk32, dk_r), ("dv", dv32, dv_r), ("dq", dq32, dq_r)):
            _close(f"fp32 restatement (fast={fast}) vs reference, {name}", got, want)


@pytest.mark.parametrize("idx", range(len(UPSAMPLE)))
def test_dense_float64_formulation_matches_the_reference_upsampling_operators(reference_results, idx):
    k, v, q, dy, w, col, roff, nh = _inputs(UPSAMPLE[idx], True)
    y_r, dk_r, dv_r, dq_r = reference_results[len(GATHER) + idx]
    kd, vd, qd = [t.double().requires_grad_(True) for t in (k, v, q)]
    y64 = o.dense_attention_f64(kd, vd, qd, w, col, roff, nh)
    y64.backward(dy.double())
    for name, got, want in (("y", y_r, y64), ("dk", dk_r, kd.grad), ("dv", dv_r, vd.grad), ("dq", dq_r, qd.grad)):
        _close(f"reference (up-sampling) vs dense float64, {name}", got, want)


def test_reference_cpu_operators_on_sampled_rows_of_the_headline_configuration():
    """cfg3's grid and cutoff, two heads of 32 channels, five output latitudes including a pole row (5,760 neighbors per
    query): the strict fp32 restatement and the float64 spec against the reference's forward and backward."""
    cfg = CONFIGS["cfg3"]
    (Hi, Wi), (Ho, Wo) = cfg["in_shape"], cfg["out_shape"]
    col, roff = g.neighborhood_csr(cfg["in_shape"], cfg["out_shape"], cfg["grid_in"], cfg["grid_out"], cfg["theta_cutoff"])
    rows = [0, 3, 200, 360, 720]
    lens = (roff[1:] - roff[:-1])[rows]
    ro_s = torch.zeros(len(rows) + 1, dtype=torch.int64)
    ro_s[1:] = torch.cumsum(lens, 0)
    col_s = torch.cat([col[roff[r] : roff[r + 1]] for r in rows])
    w = g.attention_quad_weights(Hi, Wi, cfg["grid_in"])
    nh, d = 2, 32
    k, v, q, dy = randn_inputs(1, Hi, Wi, len(rows), Wo, nh, d, d)
    res = ref.run([ref.forward_job(k, v, q, w, col_s, ro_s, nh), ref.backward_job(k, v, q, dy, w, col_s, ro_s, nh)])
    y_r, (dk_r, dv_r, dq_r) = res[0]["out"][0], res[1]["out"]
    y64 = o.forward_f64(k, v, q, w, col_s, ro_s, nh)
    dk64, dv64, dq64 = o.backward_f64(k, v, q, dy, w, col_s, ro_s, nh)
    y32 = o.forward_f32(k, v, q, w, col_s, ro_s, nh)
    dk32, dv32, dq32 = o.backward_f32(k, v, q, dy, w, col_s, ro_s, nh)
    for name, r, f64, f32 in (("y", y_r, y64, y32), ("dk", dk_r, dk64, dk32), ("dv", dv_r, dv64, dv32), ("dq", dq_r, dq64, dq32)):
        _close(f"reference vs float64 spec, {name}", r, f64)
        _close(f"fp32 restatement vs reference, {name}", f32, r)


def test_reference_layout_operators_are_plain_permutations():
    x = torch.randn(2, 5, 3, 4)
    res = ref.run([dict(op="permute_to_nhwc", args=[x]), dict(op="permute_to_nchw", args=[x])])
    assert torch.equal(res[0]["out"][0], x.permute(0, 2, 3, 1).contiguous())
    assert torch.equal(res[1]["out"][0], x.permute(0, 3, 1, 2).contiguous())
