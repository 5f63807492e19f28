"""
The oracle against vectors computed by the reference's OWN CPU operators (tests/golden/reference_cpu/*.npz, written by
tests/golden/make_reference_golden.py from the reference's compiled CPU path).  The reference computes in fp32:
rtol = atol = 1e-5 for the fp32 restatement (strict and release-flag builds) and for the float64 formulations.
"""

import pytest
import torch

from oracle import cpu_attention as o
from tests.golden_util import REFERENCE_DIR, load_golden, reference_golden_names

TOL = dict(rtol=1e-5, atol=1e-5)


def test_fixtures_present():
    names = reference_golden_names()
    assert len(names) >= 7 and any(n.startswith("up") for n in names)


@pytest.mark.parametrize("name", reference_golden_names())
def test_oracle_matches_the_reference_cpu_results(name):
    d = load_golden(name, REFERENCE_DIR)
    k, v, q, dy = d["k"], d["v"], d["q"], d["dy"]
    psi = (d["quad_weights"], d["col_idx"], d["row_off"], d["num_heads"])
    assert d["y"].dtype == torch.float32
    want = {n: d[n].double() for n in ("y", "dk", "dv", "dq")}
    kd, vd, qd = [t.double().requires_grad_(True) for t in (k, v, q)]
    y64 = o.dense_attention_f64(kd, vd, qd, *psi)
    y64.backward(dy.double())
    for key, got in (("y", y64.detach()), ("dk", kd.grad), ("dv", vd.grad), ("dq", qd.grad)):
        assert torch.allclose(got, want[key], **TOL), f"dense float64 formulation, {key}"
    if o.is_upsample(k.shape[2], q.shape[2]):
        return  # the C restatement covers the gather direction (the up-sampling oracle is the dense formulation above)
    for key, got in zip(("y", "dk", "dv", "dq"), (o.forward_f64(k, v, q, *psi), *o.backward_f64(k, v, q, dy, *psi))):
        assert torch.allclose(got, want[key], **TOL), f"float64 spec, {key}"
    for fast in (False, True):
        got32 = (o.forward_f32(k, v, q, *psi, fast=fast), *o.backward_f32(k, v, q, dy, *psi, fast=fast))
        for key, got in zip(("y", "dk", "dv", "dq"), got32):
            assert torch.allclose(got.double(), want[key], **TOL), f"fp32 restatement (fast={fast}), {key}"
