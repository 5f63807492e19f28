"""
Pins for oracle/cpu_ring.py (CPU only).  The reference has no CPU implementation and no stored vectors for the ring-step
operators, so the restatement is pinned by what the mathematics fixes: folding the chunks of ANY partition of the input
longitudes, in any order, into fresh state must give the dense float64 softmax attention on the rank's output window, and
the backward passes its autograd gradients.  split_csr_rows is pinned on the reference's own test inputs
(tests/test_attention.py:1350-1366) with the values its documented rule gives.
"""

import pytest
import torch

from oracle import cpu_attention as oracle
from oracle import cpu_ring as ring
from tests.ring_util import RING_CASES, chunk_of, fresh_state, local_problem

D = torch.float64


def _dense_reference(p):
    """y on the window and the gradients of a loss that only sees the window, from the dense float64 formulation."""
    k, v, q = [t.double().requires_grad_(True) for t in (p["k"], p["v"], p["q"])]
    y = oracle.dense_attention_f64(k, v, q, p["quad"], p["col"], p["roff"], 1)
    la, na, lo, no = p["lat_lo"], p["nlat_loc"], p["lon_lo"], p["nlon_loc"]
    win = y[:, la : la + na, lo : lo + no]
    (win * p["dy_l"].double()).sum().backward()
    return win.detach(), k.grad, v.grad, q.grad[:, la : la + na, lo : lo + no]


@pytest.mark.parametrize("case", RING_CASES, ids=lambda c: f"{c[0][0]}x{c[0][1]}to{c[1][0]}x{c[1][1]}_win{c[5]}")
@pytest.mark.parametrize("order", ["natural", "rotated"])
@pytest.mark.parametrize("tight_halo", [True, False], ids=["halo", "fullgrid"])
def test_chunks_fold_to_dense_attention(case, order, tight_halo):
    p = local_problem(case, tight_halo=tight_halo)
    B, ck, cv = p["k"].shape[0], p["k"].shape[3], p["v"].shape[3]
    Wi = p["ins"][1]
    nchunk = len(p["chunks"])
    steps = list(range(nchunk)) if order == "natural" else [(1 + i) % nchunk for i in range(nchunk)]
    geo = lambda c: (p["quad"], p["col_l"], p["roff_l"], Wi, p["pscale"], p["chunks"][c][0], p["halo"][0])  # noqa: E731
    st = fresh_state(B, p["nlat_loc"], p["nlon_loc"], ck, cv, D)
    for c in steps:
        ring.forward_step(chunk_of(p, p["k"], c).double(), chunk_of(p, p["v"], c).double(), p["q_l"].double(), st["y_acc"], st["alpha_sum"], st["qdotk_max"], *geo(c))
    y_ref, dk_ref, dv_ref, dq_ref = _dense_reference(p)
    torch.testing.assert_close(st["y_acc"] / st["alpha_sum"][..., None], y_ref, rtol=1e-12, atol=1e-12)

    bw = fresh_state(B, p["nlat_loc"], p["nlon_loc"], ck, cv, D)
    for c in steps:
        ring.backward_pass1(
            chunk_of(p, p["k"], c).double(), chunk_of(p, p["v"], c).double(), p["q_l"].double(), p["dy_l"].double(),
            bw["alpha_sum"], bw["qdotk_max"], bw["integral"], bw["alpha_k"], bw["alpha_kvw"], *geo(c),
        )  # fmt: skip
    torch.testing.assert_close(bw["alpha_sum"], st["alpha_sum"], rtol=1e-12, atol=0)
    torch.testing.assert_close(bw["qdotk_max"], st["qdotk_max"], rtol=0, atol=0)
    S = bw["alpha_sum"][..., None]
    dq = (S * bw["alpha_kvw"] - bw["integral"][..., None] * bw["alpha_k"]) / S**2  # distributed_attention.py:349-353
    torch.testing.assert_close(dq, dq_ref, rtol=1e-11, atol=1e-12)
    integral_norm = bw["integral"] / bw["alpha_sum"]
    dk, dv = torch.zeros_like(p["k"], dtype=D), torch.zeros_like(p["v"], dtype=D)
    h0, h1 = p["halo"]
    for c in steps:
        kc, vc = chunk_of(p, p["k"], c).double(), chunk_of(p, p["v"], c).double()
        dkc, dvc = torch.zeros_like(kc), torch.zeros_like(vc)
        ring.backward_pass2(kc, vc, p["q_l"].double(), p["dy_l"].double(), st["alpha_sum"], st["qdotk_max"], integral_norm, dkc, dvc, *geo(c))
        lo, hi = p["chunks"][c]
        dk[:, h0:h1, lo:hi] += dkc
        dv[:, h0:h1, lo:hi] += dvc
    torch.testing.assert_close(dk, dk_ref, rtol=1e-11, atol=1e-12)
    torch.testing.assert_close(dv, dv_ref, rtol=1e-11, atol=1e-12)


def test_a_chunk_without_neighbors_leaves_the_state_alone():
    p = local_problem(RING_CASES[1])
    B, ck, cv = p["k"].shape[0], p["k"].shape[3], p["v"].shape[3]
    st = fresh_state(B, p["nlat_loc"], p["nlon_loc"], ck, cv, D)
    # a halo that misses every neighbor latitude: nothing may change, qdotk_max stays -inf
    kc = torch.randn(B, 1, 3, ck, dtype=D)
    ring.forward_step(kc, torch.randn(B, 1, 3, cv, dtype=D), p["q_l"].double(), st["y_acc"], st["alpha_sum"], st["qdotk_max"], p["quad"], p["col_l"], p["roff_l"], p["ins"][1], p["pscale"], 0, 100)
    assert float(st["alpha_sum"].abs().max()) == 0.0 and bool(torch.isinf(st["qdotk_max"]).all()) and float(st["y_acc"].abs().max()) == 0.0


def _csr_from_lengths(lengths):
    rl = torch.as_tensor(lengths, dtype=torch.int64)
    row_off = torch.zeros(rl.numel() + 1, dtype=torch.int64)
    row_off[1:] = torch.cumsum(rl, 0)
    return torch.argsort(rl, descending=True, stable=True).to(torch.int32), row_off


# the reference's own inputs (tests/test_attention.py:1350-1366); expected = its documented rule (attention_cuda_utils.cu:
# 269-285): long rows are the leading rows of length >= max(1024, int(0.1 * longest))
SPLIT_CASES = [
    ("all_short_uniform", [16] * 32, (0, 0, 16)),
    ("all_short_varied", [3, 7, 1, 12, 5, 9, 2, 8, 4, 11], (0, 0, 12)),
    ("all_equal", [512] * 20, (0, 0, 512)),
    ("single_row", [777], (0, 0, 777)),
    ("one_long_rest_short", [4096] + [16] * 31, (1, 4096, 16)),
    ("several_long_floor_1024", [2048, 1536, 1100, 1024, 64, 32, 16, 8], (4, 2048, 64)),
    ("thres_branch_above_floor", [40000, 39000, 12000, 5000, 100, 50, 10], (4, 40000, 100)),
    ("exactly_at_floor", [1024, 1024, 1023, 512, 1], (2, 1024, 1023)),
    ("descending_ramp", list(range(200, 0, -1)), (0, 0, 200)),
    ("all_long", [3000, 2500, 2000], (3, 3000, 0)),
]


@pytest.mark.parametrize("name,lengths,expected", SPLIT_CASES, ids=[c[0] for c in SPLIT_CASES])
def test_split_csr_rows(name, lengths, expected):
    from torch_harmonics_amd import ops

    row_idx, row_off = _csr_from_lengths(lengths)
    assert ring.split_csr_rows(row_idx, row_off, len(lengths)) == expected
    assert tuple(ops.split_csr_rows(row_idx, row_off, len(lengths))) == expected


from tests.ring_util import RING_UP_CASES, local_problem_upsample  # noqa: E402


@pytest.mark.parametrize("case", RING_UP_CASES, ids=lambda c: f"{c[0][0]}x{c[0][1]}to{c[1][0]}x{c[1][1]}_win{c[5]}")
@pytest.mark.parametrize("order", ["natural", "rotated"])
def test_upsample_chunks_fold_to_dense_attention(case, order):
    p = local_problem_upsample(case)
    B, ck, cv = p["k"].shape[0], p["k"].shape[3], p["v"].shape[3]
    Hi, Wo = p["ins"][0], p["outs"][1]
    nchunk = len(p["chunks"])
    steps = list(range(nchunk)) if order == "natural" else [(1 + i) % nchunk for i in range(nchunk)]
    geo = lambda c: (p["quad"], p["col_l"], p["roff_l"], Wo, p["pscale_out"], p["chunks"][c][0], p["halo"][0])  # noqa: E731
    blk = lambda t, c: p["halo_block"](t, *p["chunks"][c]).double()  # noqa: E731
    q_l, g_l = p["q_l"].double(), p["dy_l"].double()
    st = fresh_state(B, p["nlat_loc"], p["nlon_loc"], ck, cv, D)
    for c in steps:
        ring.forward_step_upsample(blk(p["k"], c), blk(p["v"], c), q_l, st["y_acc"], st["alpha_sum"], st["qdotk_max"], *geo(c))
    y_ref, dk_ref, dv_ref, dq_ref = _dense_reference(p)
    torch.testing.assert_close(st["y_acc"] / st["alpha_sum"][..., None], y_ref, rtol=1e-12, atol=1e-12)

    bw = fresh_state(B, p["nlat_loc"], p["nlon_loc"], ck, cv, D)
    for c in steps:
        ring.backward_pass1_upsample(blk(p["k"], c), blk(p["v"], c), q_l, g_l, st["qdotk_max"], bw["integral"], bw["alpha_k"], bw["alpha_kvw"], *geo(c))
    S = st["alpha_sum"][..., None]
    dq = (S * bw["alpha_kvw"] - bw["integral"][..., None] * bw["alpha_k"]) / S**2
    torch.testing.assert_close(dq, dq_ref, rtol=1e-11, atol=1e-12)
    integral_norm = bw["integral"] / st["alpha_sum"]
    dk, dv = torch.zeros_like(p["k"], dtype=D), torch.zeros_like(p["v"], dtype=D)
    h0, h1 = p["halo"]
    a, b = max(h0, 0), min(h1, Hi)
    for c in steps:
        kc, vc = blk(p["k"], c), blk(p["v"], c)
        dkc, dvc = torch.full_like(kc, float("nan")), torch.full_like(vc, float("nan"))  # pass 2 writes every element
        ring.backward_pass2_upsample(kc, vc, q_l, g_l, st["alpha_sum"], st["qdotk_max"], integral_norm, dkc, dvc, *geo(c))
        lo, hi = p["chunks"][c]
        dk[:, a:b, lo:hi] += dkc[:, a - h0 : b - h0]
        dv[:, a:b, lo:hi] += dvc[:, a - h0 : b - h0]
    torch.testing.assert_close(dk, dk_ref, rtol=1e-11, atol=1e-12)
    torch.testing.assert_close(dv, dv_ref, rtol=1e-11, atol=1e-12)
