"""HIP path against the committed golden vectors (float64 dense-softmax results, tests/golden/)."""

import pytest
import torch

from tests.golden_util import golden_names, load_golden
from tests.util import assert_close

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("name", golden_names())
def test_hip_matches_golden(name):
    from torch_harmonics_amd import ops

    d = load_golden(name)
    dev = torch.device("cuda", 0)
    k, v, q, dy, w, ci, ro = [d[n].to(dev) for n in ("k", "v", "q", "dy", "quad_weights", "col_idx", "row_off")]
    nh, Wi, Ho, Wo = d["num_heads"], k.shape[2], q.shape[1], q.shape[2]
    y = ops.forward(k, v, q, w, ci, ro, nh, Wi, Ho, Wo)
    dk, dv, dq = ops.backward(k, v, q, dy, w, ci, ro, nh, Wi, Ho, Wo)
    for key, got in (("y", y), ("dk", dk), ("dv", dv), ("dq", dq)):
        assert_close(f"{name}:{key}", got, d[key], rtol=1e-5, atol=1e-5)
