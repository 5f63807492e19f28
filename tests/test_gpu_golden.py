"""HIP path against the committed golden vectors: float64 dense-softmax results (tests/golden/*.npz) and the outputs of the
reference's own CPU operators on the same inputs (tests/golden/reference_cpu/*.npz)."""

import pytest
import torch

from tests.golden_util import REFERENCE_DIR, golden_names, load_golden, reference_golden_names
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


@pytest.mark.parametrize("name", reference_golden_names())
def test_hip_matches_the_reference_cpu_results(name):
    """Same inputs, the reference's fp32 CPU forward and backward as the expected values (both directions, ck != cv, the
    hybrid and the 16-longitude matrix-core kernels, the vector kernels); through the operators of the reference's names."""
    import torch_harmonics_amd  # noqa: F401  (registers attention_kernels::*)

    d = load_golden(name, REFERENCE_DIR)
    dev = torch.device("cuda", 0)
    k, v, q, dy, w, ci, ro = [d[n].to(dev) for n in ("k", "v", "q", "dy", "quad_weights", "col_idx", "row_off")]
    nh, Wi, Ho, Wo = d["num_heads"], k.shape[2], q.shape[1], q.shape[2]
    y = torch.ops.attention_kernels.forward(k, v, q, w, ci, ro, nh, Wi, Ho, Wo)
    dk, dv, dq = torch.ops.attention_kernels.backward(k, v, q, dy, w, ci, ro, nh, Wi, Ho, Wo)
    for key, got in (("y", y), ("dk", dk), ("dv", dv), ("dq", dq)):
        assert_close(f"{name}:{key}", got, d[key], rtol=1e-5, atol=1e-5)
