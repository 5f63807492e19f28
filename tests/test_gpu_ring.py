"""
Ring-step operators on the GPU (through the C ABI) against the CPU restatement oracle/cpu_ring.py after EVERY step, and,
after the last chunk, against the dense float64 softmax attention and its autograd gradients on the rank's output window.
The reference exercises these operators single-rank through opcheck only (tests/test_attention.py:894-1062).
"""

import pytest
import torch

from oracle import cpu_attention as oracle
from oracle import cpu_ring as ring
from tests.ring_util import RING_BAND_CASES, RING_CASES, chunk_of, fresh_state, local_problem
from tests.util import assert_close

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = dict(rtol=1e-5, atol=1e-5)


def _geo_dev(p):
    return p["quad"].to(DEV), p["col_l"].to(DEV), p["roff_l"].to(DEV), p["row_idx"].to(DEV)


# channel counts that are multiples of 8 take the 16-byte load paths; 32 / 64 / 128 / 256 / 512 channels = 4 / 8 / 16 / 32 / 64 lanes per cell
VECTOR_CHANNELS = [(32, 32), (64, 128), (8, 16), (256, 40), (512, 8)]


@pytest.mark.parametrize("case", RING_CASES, ids=lambda c: f"{c[0][0]}x{c[0][1]}to{c[1][0]}x{c[1][1]}_win{c[5]}")
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_ring_steps_against_oracle_and_dense_attention(case, dtype, monkeypatch):
    ck, cv = (70, 33) if case is RING_CASES[1] else (5, 3)  # one case with more than 64 channels
    _gather_direction(case, dtype, ck, cv, monkeypatch)


@pytest.mark.parametrize("chan", VECTOR_CHANNELS, ids=lambda c: f"ck{c[0]}cv{c[1]}")
@pytest.mark.parametrize("case", [RING_CASES[1], RING_CASES[3]], ids=["ratio1", "ratio3"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=["f32", "bf16", "f16"])
def test_ring_steps_vector_load_paths(case, dtype, chan, monkeypatch):
    _gather_direction(case, dtype, *chan, monkeypatch)


@pytest.mark.parametrize("d", [16, 32, 40, 64, 128], ids=lambda d: f"d{d}")
@pytest.mark.parametrize("case", RING_BAND_CASES, ids=lambda c: f"{c[0][0]}x{c[0][1]}to{c[1][0]}x{c[1][1]}_win{c[5]}")
def test_ring_forward_step_and_pass1_on_the_band_staged_kernels(case, d, monkeypatch):
    """Grids wide enough for the band-staged forward step and pass 1 (fp32, ck == cv): the same checks as everywhere else - state
    against the oracle after every chunk, y / dq / dk / dv against the dense attention - with the state coming from those kernels."""
    from torch_harmonics_amd import ops

    taken = []
    real = ops._ring_takes_plan
    monkeypatch.setattr(ops, "_ring_takes_plan", lambda *a: taken.append(real(*a)) or taken[-1])
    _gather_direction(case, torch.float32, d, d, monkeypatch)
    assert taken and all(taken)


@pytest.mark.parametrize("d", [16, 40, 64, 128], ids=lambda d: f"d{d}")
@pytest.mark.parametrize("case", [RING_BAND_CASES[0], RING_BAND_CASES[2], RING_BAND_CASES[-1]], ids=lambda c: f"{c[0][0]}x{c[0][1]}to{c[1][0]}x{c[1][1]}_win{c[5]}")
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
def test_band_staged_ring_steps_take_16_bit_storage(case, dtype, d, monkeypatch):
    """k, v, q, dy in bf16 / fp16 on the band-staged kernels (rows widened at staging, fp32 state): state against the oracle fed the
    same stored values at 1e-5 after every chunk, final results against the dense attention at the storage type's tolerance."""
    from torch_harmonics_amd import ops

    taken = []
    real = ops._ring_takes_plan
    monkeypatch.setattr(ops, "_ring_takes_plan", lambda *a: taken.append(real(*a)) or taken[-1])
    _gather_direction(case, dtype, d, d, monkeypatch)
    assert taken and all(taken)


def _gather_direction(case, dtype, ck, cv, monkeypatch):
    from torch_harmonics_amd import ops

    print(f"case {case} {dtype} ck={ck} cv={cv}", flush=True)
    p = local_problem(case, ck=ck, cv=cv)
    for name in ("k", "v", "q", "dy", "q_l", "dy_l"):  # the values the storage dtype can hold, shared by all three evaluations
        p[name] = p[name].to(dtype).float()
    B, Wi = p["k"].shape[0], p["ins"][1]
    tol = TOL if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    stol = dict(rtol=1e-5, atol=1e-5)  # state against the oracle fed the same stored values: storage dtype plays no role
    quad, col_l, roff_l, row_idx = _geo_dev(p)
    split = ops.split_csr_rows(p["row_idx"], p["roff_l"], p["nlat_loc"])
    tail = lambda c: (Wi, p["pscale"], p["chunks"][c][0], p["halo"][0], p["nlat_loc"], p["nlon_loc"], *split)  # noqa: E731
    ogeo = lambda c: (p["quad"], p["col_l"], p["roff_l"], Wi, p["pscale"], p["chunks"][c][0], p["halo"][0])  # noqa: E731
    qd, gd = p["q_l"].to(DEV, dtype), p["dy_l"].to(DEV, dtype)
    q64, g64 = p["q_l"].double(), p["dy_l"].double()
    nchunk = len(p["chunks"])
    steps = [(1 + i) % nchunk for i in range(nchunk)]

    st = fresh_state(B, p["nlat_loc"], p["nlon_loc"], ck, cv, torch.float32, DEV)
    ref = fresh_state(B, p["nlat_loc"], p["nlon_loc"], ck, cv, torch.float64)
    for c in steps:
        kc, vc = chunk_of(p, p["k"], c), chunk_of(p, p["v"], c)
        ops.forward_ring_step(kc.to(DEV, dtype), vc.to(DEV, dtype), qd, st["y_acc"], st["alpha_sum"], st["qdotk_max"], quad, col_l, roff_l, row_idx, *tail(c))
        ring.forward_step(kc.double(), vc.double(), q64, ref["y_acc"], ref["alpha_sum"], ref["qdotk_max"], *ogeo(c))
        torch.cuda.synchronize()
        seen = torch.isfinite(ref["qdotk_max"])
        assert torch.equal(torch.isfinite(st["qdotk_max"]).cpu(), seen)
        assert_close(f"qdotk_max after chunk {c}", st["qdotk_max"].cpu()[seen], ref["qdotk_max"][seen], **stol)
        assert_close(f"alpha_sum after chunk {c}", st["alpha_sum"].cpu(), ref["alpha_sum"], **stol)
        assert_close(f"y_acc after chunk {c}", st["y_acc"].cpu(), ref["y_acc"], **stol)

    k, v, q = [t.double().requires_grad_(True) for t in (p["k"], p["v"], p["q"])]
    y = oracle.dense_attention_f64(k, v, q, p["quad"], p["col"], p["roff"], 1)
    la, na, lo, no = p["lat_lo"], p["nlat_loc"], p["lon_lo"], p["nlon_loc"]
    win = y[:, la : la + na, lo : lo + no]
    (win * g64).sum().backward()
    assert_close("y", (st["y_acc"] / st["alpha_sum"][..., None]).cpu(), win.detach(), **tol)

    bw = fresh_state(B, p["nlat_loc"], p["nlon_loc"], ck, cv, torch.float32, DEV)
    rbw = fresh_state(B, p["nlat_loc"], p["nlon_loc"], ck, cv, torch.float64)
    for c in steps:
        kc, vc = chunk_of(p, p["k"], c), chunk_of(p, p["v"], c)
        ops.backward_ring_step_pass1(
            kc.to(DEV, dtype), vc.to(DEV, dtype), qd, gd, bw["alpha_sum"], bw["qdotk_max"], bw["integral"], bw["alpha_k"], bw["alpha_kvw"],
            quad, col_l, roff_l, row_idx, *tail(c),
        )  # fmt: skip
        ring.backward_pass1(kc.double(), vc.double(), q64, g64, rbw["alpha_sum"], rbw["qdotk_max"], rbw["integral"], rbw["alpha_k"], rbw["alpha_kvw"], *ogeo(c))
        torch.cuda.synchronize()
        assert_close(f"integral after chunk {c}", bw["integral"].cpu(), rbw["integral"], **stol)
        assert_close(f"alpha_k after chunk {c}", bw["alpha_k"].cpu(), rbw["alpha_k"], **stol)
        assert_close(f"alpha_kvw after chunk {c}", bw["alpha_kvw"].cpu(), rbw["alpha_kvw"], **stol)
    # the same sum from two kernels that accumulate it in the same order; the band-staged pair does so bit for bit (the dq
    # formula below, which takes the forward's alpha_sum with pass 1's other sums like the reference, leans on that for wide heads)
    assert_close("pass 1 alpha_sum == forward alpha_sum", bw["alpha_sum"], st["alpha_sum"], rtol=1e-6, atol=0)
    if ops._ring_takes_plan(chunk_of(p, p["k"], 0).to(DEV, dtype), chunk_of(p, p["v"], 0).to(DEV, dtype), qd, Wi, p["pscale"]):
        assert torch.equal(bw["alpha_sum"], st["alpha_sum"]) and torch.equal(bw["qdotk_max"], st["qdotk_max"])
    S = st["alpha_sum"][..., None]
    dq = (S * bw["alpha_kvw"] - bw["integral"][..., None] * bw["alpha_k"]) / S**2
    assert_close("dq", dq.cpu(), q.grad[:, la : la + na, lo : lo + no], **tol)

    integral_norm = (bw["integral"] / st["alpha_sum"]).contiguous()
    h0, h1 = p["halo"]
    # pass 2 both ways: on the transposed neighborhood (what the operator runs) and straight from the CSR with atomics
    for from_csr in (False, True):
        monkeypatch.setattr(ops, "_RING_PASS2_FROM_CSR", from_csr)
        dk, dv = torch.zeros_like(p["k"]), torch.zeros_like(p["v"])
        for c in steps:
            kc, vc = chunk_of(p, p["k"], c), chunk_of(p, p["v"], c)
            # the step ADDS to what the arrays hold: start from a known non-zero content
            dkc, dvc = torch.full(kc.shape, 0.5, device=DEV), torch.full(vc.shape, -0.25, device=DEV)
            ops.backward_ring_step_pass2(
                kc.to(DEV, dtype), vc.to(DEV, dtype), qd, gd, st["alpha_sum"], st["qdotk_max"], integral_norm, dkc, dvc, quad, col_l, roff_l, row_idx, *tail(c)
            )
            clo, chi = p["chunks"][c]
            dk[:, h0:h1, clo:chi] += dkc.cpu() - 0.5
            dv[:, h0:h1, clo:chi] += dvc.cpu() + 0.25
        assert_close(f"dk (from_csr={from_csr})", dk, k.grad, **tol)
        assert_close(f"dv (from_csr={from_csr})", dv, v.grad, **tol)


@pytest.mark.parametrize("band", [False, True], ids=["gather_kernels", "band_staged_kernels"])
def test_ring_ops_pass_opcheck_and_leave_state_alone_without_neighbors(band):
    from torch_harmonics_amd import ops

    p = local_problem(RING_BAND_CASES[1], ck=32, cv=32) if band else local_problem(RING_CASES[2])
    B, ck, cv, Wi = p["k"].shape[0], p["k"].shape[3], p["v"].shape[3], p["ins"][1]
    quad, col_l, roff_l, row_idx = _geo_dev(p)
    split = ops.split_csr_rows(p["row_idx"], p["roff_l"], p["nlat_loc"])
    qd, gd = p["q_l"].to(DEV), p["dy_l"].to(DEV)
    kc, vc = chunk_of(p, p["k"], 1).to(DEV), chunk_of(p, p["v"], 1).to(DEV)
    tail = (Wi, p["pscale"], p["chunks"][1][0], p["halo"][0], p["nlat_loc"], p["nlon_loc"], *split)
    assert ops._ring_takes_plan(kc, vc, qd, Wi, p["pscale"]) == band
    st = fresh_state(B, p["nlat_loc"], p["nlon_loc"], ck, cv, torch.float32, DEV)
    torch.library.opcheck(ops.forward_ring_step, (kc, vc, qd, st["y_acc"], st["alpha_sum"], st["qdotk_max"], quad, col_l, roff_l, row_idx, *tail))
    torch.library.opcheck(
        ops.backward_ring_step_pass1, (kc, vc, qd, gd, st["alpha_sum"], st["qdotk_max"], st["integral"], st["alpha_k"], st["alpha_kvw"], quad, col_l, roff_l, row_idx, *tail)
    )
    st2 = fresh_state(B, p["nlat_loc"], p["nlon_loc"], ck, cv, torch.float32, DEV)
    ops.forward_ring_step(kc, vc, qd, st2["y_acc"], st2["alpha_sum"], st2["qdotk_max"], quad, col_l, roff_l, row_idx, *tail)
    norm = (st2["integral"] * 0).contiguous()
    torch.library.opcheck(
        ops.backward_ring_step_pass2,
        (kc, vc, qd, gd, st2["alpha_sum"].clamp_min(1e-30), st2["qdotk_max"].clamp_min(-1e30), norm, torch.zeros_like(kc), torch.zeros_like(vc), quad, col_l, roff_l, row_idx, *tail),
    )
    # a halo that holds none of the neighbor latitudes: the state must come back bit for bit
    st3 = fresh_state(B, p["nlat_loc"], p["nlon_loc"], ck, cv, torch.float32, DEV)
    far = (Wi, p["pscale"], 0, 1000, p["nlat_loc"], p["nlon_loc"], *split)
    ops.forward_ring_step(kc, vc, qd, st3["y_acc"], st3["alpha_sum"], st3["qdotk_max"], quad, col_l, roff_l, row_idx, *far)
    torch.cuda.synchronize()
    assert float(st3["alpha_sum"].abs().max()) == 0.0 and bool(torch.isinf(st3["qdotk_max"]).all()) and float(st3["y_acc"].abs().max()) == 0.0
    with pytest.raises(RuntimeError):  # chunk outside the input grid
        ops.forward_ring_step(kc, vc, qd, st3["y_acc"], st3["alpha_sum"], st3["qdotk_max"], quad, col_l, roff_l, row_idx, Wi, p["pscale"], Wi - 1, 0, p["nlat_loc"], p["nlon_loc"], *split)


from tests.ring_util import RING_UP_BAND_CASES, RING_UP_CASES, local_problem_upsample  # noqa: E402


@pytest.mark.parametrize("case", RING_UP_CASES, ids=lambda c: f"{c[0][0]}x{c[0][1]}to{c[1][0]}x{c[1][1]}_win{c[5]}")
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_upsample_ring_steps_against_oracle_and_dense_attention(case, dtype):
    ck, cv = (70, 33) if case is RING_UP_CASES[1] else (5, 3)
    _upsample_direction(case, dtype, ck, cv)


@pytest.mark.parametrize("chan", VECTOR_CHANNELS, ids=lambda c: f"ck{c[0]}cv{c[1]}")
@pytest.mark.parametrize("case", [RING_UP_CASES[1], RING_UP_CASES[2]], ids=["ratio2", "ratio3_padded"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=["f32", "bf16", "f16"])
def test_upsample_ring_steps_vector_load_paths(case, dtype, chan):
    _upsample_direction(case, dtype, *chan)


@pytest.mark.parametrize("d", [16, 32, 40, 64], ids=lambda d: f"d{d}")
@pytest.mark.parametrize("case", RING_UP_BAND_CASES, ids=lambda c: f"{c[0][0]}x{c[0][1]}to{c[1][0]}x{c[1][1]}_win{c[5]}")
def test_upsample_ring_steps_on_the_band_staged_kernels(case, d, monkeypatch):
    """Grids wide enough for the band-staged kernels (fp32, ck == cv): the same checks as everywhere else, with all three steps on
    those kernels."""
    from torch_harmonics_amd import ops

    taken = []
    real = ops._ring_takes_plan
    monkeypatch.setattr(ops, "_ring_takes_plan", lambda *a: taken.append(real(*a)) or taken[-1])
    _upsample_direction(case, torch.float32, d, d)
    assert taken and all(taken)


@pytest.mark.parametrize("d", [16, 40, 64], ids=lambda d: f"d{d}")
@pytest.mark.parametrize("case", [RING_UP_BAND_CASES[0], RING_UP_BAND_CASES[-1]], ids=lambda c: f"{c[0][0]}x{c[0][1]}to{c[1][0]}x{c[1][1]}_win{c[5]}")
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
def test_band_staged_upsample_ring_steps_take_16_bit_storage(case, dtype, d, monkeypatch):
    """The up-sampling direction's three steps on the band-staged kernels with 16-bit k, v, q, dy."""
    from torch_harmonics_amd import ops

    taken = []
    real = ops._ring_takes_plan
    monkeypatch.setattr(ops, "_ring_takes_plan", lambda *a: taken.append(real(*a)) or taken[-1])
    _upsample_direction(case, dtype, d, d)
    assert taken and all(taken)


def _upsample_direction(case, dtype, ck, cv):
    from torch_harmonics_amd import ops

    print(f"case {case} {dtype} ck={ck} cv={cv}", flush=True)
    p = local_problem_upsample(case, ck=ck, cv=cv)
    for name in ("k", "v", "q", "dy", "q_l", "dy_l"):
        p[name] = p[name].to(dtype).float()
    B, (Hi, Wi), Wo = p["k"].shape[0], p["ins"], p["outs"][1]
    tol = TOL if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    stol = dict(rtol=1e-5, atol=1e-5)
    quad, col_l, roff_l = p["quad"].to(DEV), p["col_l"].to(DEV), p["roff_l"].to(DEV)
    tail = lambda c: (Wi, Wo, p["pscale_out"], p["chunks"][c][0], p["halo"][0], p["nlat_loc"], p["nlon_loc"])  # noqa: E731
    ogeo = lambda c: (p["quad"], p["col_l"], p["roff_l"], Wo, p["pscale_out"], p["chunks"][c][0], p["halo"][0])  # noqa: E731
    blk = lambda t, c: p["halo_block"](t, *p["chunks"][c])  # noqa: E731
    qd, gd = p["q_l"].to(DEV, dtype), p["dy_l"].to(DEV, dtype)
    q64, g64 = p["q_l"].double(), p["dy_l"].double()
    nchunk = len(p["chunks"])
    steps = [(1 + i) % nchunk for i in range(nchunk)]

    st = fresh_state(B, p["nlat_loc"], p["nlon_loc"], ck, cv, torch.float32, DEV)
    ref = fresh_state(B, p["nlat_loc"], p["nlon_loc"], ck, cv, torch.float64)
    for c in steps:
        kc, vc = blk(p["k"], c), blk(p["v"], c)
        ops.forward_ring_step_upsample(kc.to(DEV, dtype), vc.to(DEV, dtype), qd, st["y_acc"], st["alpha_sum"], st["qdotk_max"], quad, col_l, roff_l, *tail(c))
        ring.forward_step_upsample(kc.double(), vc.double(), q64, ref["y_acc"], ref["alpha_sum"], ref["qdotk_max"], *ogeo(c))
        torch.cuda.synchronize()
        seen = torch.isfinite(ref["qdotk_max"])
        assert torch.equal(torch.isfinite(st["qdotk_max"]).cpu(), seen)
        assert_close(f"qdotk_max after chunk {c}", st["qdotk_max"].cpu()[seen], ref["qdotk_max"][seen], **stol)
        assert_close(f"alpha_sum after chunk {c}", st["alpha_sum"].cpu(), ref["alpha_sum"], **stol)
        assert_close(f"y_acc after chunk {c}", st["y_acc"].cpu(), ref["y_acc"], **stol)

    k, v, q = [t.double().requires_grad_(True) for t in (p["k"], p["v"], p["q"])]
    y = oracle.dense_attention_f64(k, v, q, p["quad"], p["col"], p["roff"], 1)
    la, na, lo, no = p["lat_lo"], p["nlat_loc"], p["lon_lo"], p["nlon_loc"]
    win = y[:, la : la + na, lo : lo + no]
    (win * g64).sum().backward()
    assert_close("y", (st["y_acc"] / st["alpha_sum"][..., None]).cpu(), win.detach(), **tol)

    bw = fresh_state(B, p["nlat_loc"], p["nlon_loc"], ck, cv, torch.float32, DEV)
    rbw = fresh_state(B, p["nlat_loc"], p["nlon_loc"], ck, cv, torch.float64)
    for c in steps:
        kc, vc = blk(p["k"], c), blk(p["v"], c)
        ops.backward_ring_step_upsample_pass1(kc.to(DEV, dtype), vc.to(DEV, dtype), qd, gd, st["qdotk_max"], bw["integral"], bw["alpha_k"], bw["alpha_kvw"], quad, col_l, roff_l, *tail(c))
        ring.backward_pass1_upsample(kc.double(), vc.double(), q64, g64, ref["qdotk_max"], rbw["integral"], rbw["alpha_k"], rbw["alpha_kvw"], *ogeo(c))
        torch.cuda.synchronize()
        assert_close(f"integral after chunk {c}", bw["integral"].cpu(), rbw["integral"], **stol)
        assert_close(f"alpha_k after chunk {c}", bw["alpha_k"].cpu(), rbw["alpha_k"], **stol)
        assert_close(f"alpha_kvw after chunk {c}", bw["alpha_kvw"].cpu(), rbw["alpha_kvw"], **stol)
    S = st["alpha_sum"][..., None]
    dq = (S * bw["alpha_kvw"] - bw["integral"][..., None] * bw["alpha_k"]) / S**2
    assert_close("dq", dq.cpu(), q.grad[:, la : la + na, lo : lo + no], **tol)

    integral_norm = (bw["integral"] / st["alpha_sum"]).contiguous()
    dk, dv = torch.zeros_like(p["k"]), torch.zeros_like(p["v"])
    h0, h1 = p["halo"]
    a, b = max(h0, 0), min(h1, Hi)
    for c in steps:
        kc, vc = blk(p["k"], c), blk(p["v"], c)
        dkc = torch.full(kc.shape, float("nan"), device=DEV)  # pass 2 writes every element
        dvc = torch.full(vc.shape, float("nan"), device=DEV)
        ops.backward_ring_step_upsample_pass2(kc.to(DEV, dtype), vc.to(DEV, dtype), qd, gd, st["alpha_sum"], st["qdotk_max"], integral_norm, dkc, dvc, quad, col_l, roff_l, *tail(c))
        clo, chi = p["chunks"][c]
        assert bool(torch.isfinite(dkc).all()) and bool(torch.isfinite(dvc).all())
        dk[:, a:b, clo:chi] += dkc.cpu()[:, a - h0 : b - h0]
        dv[:, a:b, clo:chi] += dvc.cpu()[:, a - h0 : b - h0]
    assert_close("dk", dk, k.grad, **tol)
    assert_close("dv", dv, v.grad, **tol)


def test_upsample_ring_ops_pass_opcheck():
    from torch_harmonics_amd import ops

    p = local_problem_upsample(RING_UP_CASES[2])
    B, ck, cv, Wi, Wo = p["k"].shape[0], p["k"].shape[3], p["v"].shape[3], p["ins"][1], p["outs"][1]
    quad, col_l, roff_l = p["quad"].to(DEV), p["col_l"].to(DEV), p["roff_l"].to(DEV)
    qd, gd = p["q_l"].to(DEV), p["dy_l"].to(DEV)
    kc, vc = p["halo_block"](p["k"], *p["chunks"][1]).to(DEV), p["halo_block"](p["v"], *p["chunks"][1]).to(DEV)
    tail = (Wi, Wo, p["pscale_out"], p["chunks"][1][0], p["halo"][0], p["nlat_loc"], p["nlon_loc"])
    st = fresh_state(B, p["nlat_loc"], p["nlon_loc"], ck, cv, torch.float32, DEV)
    ops.forward_ring_step_upsample(kc, vc, qd, st["y_acc"], st["alpha_sum"], st["qdotk_max"], quad, col_l, roff_l, *tail)
    mx = st["qdotk_max"].clamp_min(-1e30)
    # the scatter steps add with fp32 atomics in hardware order: opcheck's repeat-and-compare needs a tolerance there
    torch.library.opcheck(ops.forward_ring_step_upsample, (kc, vc, qd, st["y_acc"], st["alpha_sum"], mx.clone(), quad, col_l, roff_l, *tail), rtol=1e-5, atol=1e-5)
    torch.library.opcheck(ops.backward_ring_step_upsample_pass1, (kc, vc, qd, gd, mx, st["integral"], st["alpha_k"], st["alpha_kvw"], quad, col_l, roff_l, *tail), rtol=1e-5, atol=1e-5)
    norm = torch.zeros_like(mx)
    torch.library.opcheck(
        ops.backward_ring_step_upsample_pass2, (kc, vc, qd, gd, st["alpha_sum"].clamp_min(1e-30), mx, norm, torch.zeros_like(kc), torch.zeros_like(vc), quad, col_l, roff_l, *tail)
    )


def test_pass2_on_psi_regrouped_by_the_host_builder_is_bitwise_the_operator():
    """s2attn_ring_regroup_psi (host arrays, what a C caller uses) feeds s2attn_ring_backward_pass2_transposed the same entries
    in the same order as the operator's device-built arrays: identical dk, dv bit for bit."""
    import ctypes

    from torch_harmonics_amd import _lib, ops

    case = RING_CASES[2]
    p = local_problem(case, ck=16, cv=8)
    B, Wi = p["k"].shape[0], p["ins"][1]
    quad, col_l, roff_l, row_idx = _geo_dev(p)
    split = ops.split_csr_rows(p["row_idx"], p["roff_l"], p["nlat_loc"])
    c = 1
    kc, vc = chunk_of(p, p["k"], c).to(DEV), chunk_of(p, p["v"], c).to(DEV)
    qd, gd = p["q_l"].to(DEV), p["dy_l"].to(DEV)
    gen = torch.Generator().manual_seed(5)
    stat = lambda: (torch.rand(B, p["nlat_loc"], p["nlon_loc"], generator=gen) + 0.5).to(DEV)  # noqa: E731
    asum, qmax, inorm = stat(), stat(), stat()
    tail = (Wi, p["pscale"], p["chunks"][c][0], p["halo"][0], p["nlat_loc"], p["nlon_loc"], *split)
    dk0, dv0 = torch.zeros_like(kc), torch.zeros_like(vc)
    ops.backward_ring_step_pass2(kc, vc, qd, gd, asum, qmax, inorm, dk0, dv0, quad, col_l, roff_l, row_idx, *tail)

    lib = _lib.load()
    nlat_halo, nnz = kc.shape[1], p["col_l"].numel()
    t_lat, t_lon = torch.zeros(nnz, dtype=torch.int32), torch.zeros(nnz, dtype=torch.int32)
    t_off, t_order = torch.zeros(nlat_halo + 1, dtype=torch.int64), torch.zeros(nlat_halo, dtype=torch.int32)
    n = lib.s2attn_ring_regroup_psi(p["col_l"].data_ptr(), p["roff_l"].data_ptr(), p["nlat_loc"], Wi, p["halo"][0], nlat_halo,
                                    t_lat.data_ptr(), t_lon.data_ptr(), t_off.data_ptr(), t_order.data_ptr())  # fmt: skip
    assert n >= 0
    d_lat, d_lon, d_off, d_order = [t.to(DEV) for t in (t_lat, t_lon, t_off, t_order)]
    shape = _lib.RingShapeStruct(B, nlat_halo, kc.shape[2], p["nlat_loc"], p["nlon_loc"], 16, 8, Wi, p["pscale"], p["chunks"][c][0], p["halo"][0], _lib.S2ATTN_F32)
    dk1, dv1 = torch.zeros_like(kc), torch.zeros_like(vc)
    rc = lib.s2attn_ring_backward_pass2_transposed(
        kc.data_ptr(), vc.data_ptr(), qd.data_ptr(), gd.data_ptr(), asum.data_ptr(), qmax.data_ptr(), inorm.data_ptr(), dk1.data_ptr(), dv1.data_ptr(),
        quad.data_ptr(), d_lat.data_ptr(), d_lon.data_ptr(), d_off.data_ptr(), d_order.data_ptr(), ctypes.byref(shape),
        ctypes.c_void_p(torch.cuda.current_stream().cuda_stream),
    )  # fmt: skip
    _lib.check(rc, "s2attn_ring_backward_pass2_transposed")
    torch.cuda.synchronize()
    assert float(dk0.abs().max()) > 0
    assert torch.equal(dk0, dk1) and torch.equal(dv0, dv1)


def test_ring_steps_with_an_empty_local_psi_are_no_ops():
    """A rank whose output rows see no input point at all (an empty col_idx): every step returns without touching the state; pass 2
    of the up-sampling direction still writes every element (zeros)."""
    from torch_harmonics_amd import ops

    B, ck, cv, Ho, Wo, Hh, Wk = 2, 8, 8, 3, 6, 4, 5
    z = lambda *s: torch.zeros(*s, device=DEV)  # noqa: E731
    kc, vc, q, dy = torch.randn(B, Hh, Wk, ck, device=DEV), torch.randn(B, Hh, Wk, cv, device=DEV), torch.randn(B, Ho, Wo, ck, device=DEV), torch.randn(B, Ho, Wo, cv, device=DEV)
    quad = torch.ones(16, device=DEV)
    col = torch.zeros(0, dtype=torch.int64, device=DEV)
    roff, row_idx = torch.zeros(Ho + 1, dtype=torch.int64, device=DEV), torch.arange(Ho, dtype=torch.int32, device=DEV)
    st = fresh_state(B, Ho, Wo, ck, cv, torch.float32, DEV)
    tail = (12, 2, 3, 0, Ho, Wo, 0, 0, 0)
    ops.forward_ring_step(kc, vc, q, st["y_acc"], st["alpha_sum"], st["qdotk_max"], quad, col, roff, row_idx, *tail)
    ops.backward_ring_step_pass1(kc, vc, q, dy, st["alpha_sum"], st["qdotk_max"], st["integral"], st["alpha_k"], st["alpha_kvw"], quad, col, roff, row_idx, *tail)
    dk, dv = torch.full_like(kc, 2.0), torch.full_like(vc, 3.0)
    ops.backward_ring_step_pass2(kc, vc, q, dy, st["alpha_sum"] + 1, st["qdotk_max"].clamp_min(0), z(B, Ho, Wo), dk, dv, quad, col, roff, row_idx, *tail)
    torch.cuda.synchronize()
    assert float(st["y_acc"].abs().max()) == 0 and float(st["alpha_sum"].abs().max()) == 0 and bool(torch.isinf(st["qdotk_max"]).all())
    assert float(st["integral"].abs().max()) == 0 and float(st["alpha_k"].abs().max()) == 0
    assert bool((dk == 2.0).all()) and bool((dv == 3.0).all())  # the gather direction ADDS: untouched
    # up-sampling direction: psi keyed by the chunk's input latitudes
    roff_up = torch.zeros(Hh + 1, dtype=torch.int64, device=DEV)
    up_tail = (6, 12, 2, 0, 0, Ho, Wo)
    st = fresh_state(B, Ho, Wo, ck, cv, torch.float32, DEV)
    ops.forward_ring_step_upsample(kc, vc, q, st["y_acc"], st["alpha_sum"], st["qdotk_max"], quad, col, roff_up, *up_tail)
    ops.backward_ring_step_upsample_pass1(kc, vc, q, dy, st["qdotk_max"], st["integral"], st["alpha_k"], st["alpha_kvw"], quad, col, roff_up, *up_tail)
    dk, dv = torch.full_like(kc, float("nan")), torch.full_like(vc, float("nan"))
    ops.backward_ring_step_upsample_pass2(kc, vc, q, dy, st["alpha_sum"] + 1, st["qdotk_max"].clamp_min(0), z(B, Ho, Wo), dk, dv, quad, col, roff_up, *up_tail)
    torch.cuda.synchronize()
    assert float(st["y_acc"].abs().max()) == 0 and float(st["alpha_sum"].abs().max()) == 0 and float(st["integral"].abs().max()) == 0
    assert float(dk.abs().max()) == 0 and float(dv.abs().max()) == 0
