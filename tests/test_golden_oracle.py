"""The C oracle against the committed golden vectors (tests/golden/*.npz, written by tests/golden/make_golden.py)."""

import pytest
import torch

from oracle import cpu_attention as o
from tests.golden_util import golden_names, load_golden


def test_fixtures_present():
    assert len(golden_names()) >= 4


@pytest.mark.parametrize("name", golden_names())
def test_oracle_matches_golden(name):
    d = load_golden(name)
    args = (d["k"], d["v"], d["q"])
    psi = (d["quad_weights"], d["col_idx"], d["row_off"], d["num_heads"])
    assert torch.allclose(o.forward_f64(*args, *psi), d["y"], rtol=1e-12, atol=1e-12)
    for got, key in zip(o.backward_f64(*args, d["dy"], *psi), ("dk", "dv", "dq")):
        assert torch.allclose(got, d[key], rtol=1e-11, atol=1e-12), key
    assert torch.allclose(o.forward_f32(*args, *psi).double(), d["y"], rtol=1e-5, atol=1e-5)
    for got, key in zip(o.backward_f32(*args, d["dy"], *psi), ("dk", "dv", "dq")):
        assert torch.allclose(got.double(), d[key], rtol=1e-5, atol=1e-5), key
