"""
Host-side logic that runs without a GPU: the C ABI's exports and argument checks, the plan builder,
the product geometry, the module's constructor/state and the operators' shape propagation and errors.
"""

import ctypes
import math
import os
import re
from collections import Counter

import pytest
import torch

import torch_harmonics_amd as tha
from oracle import geometry as ogeo
from torch_harmonics_amd import _lib, ops
from torch_harmonics_amd.neighborhood import precompute_neighborhood_s2
from torch_harmonics_amd.plan import build_host_plan
from torch_harmonics_amd.quadrature import precompute_latitudes, precompute_longitudes

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ---- C ABI -----------------------------------------------------------------------------------


def test_library_loads_and_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "s2attn.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(s2attn_[a-z0-9_]+)\s*\(", header))
    assert {"s2attn_forward", "s2attn_backward", "s2attn_plan_build", "s2attn_permute_to_nhwc"} <= declared
    assert declared == set(_lib.SYMBOLS), "ctypes table and header disagree"
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in include/s2attn.h but not exported"
    assert _lib.load().s2attn_abi_version() == _lib.ABI_VERSION
    assert tha.optimized_kernels_is_available()


def test_entry_points_reject_bad_arguments_before_touching_the_gpu():
    lib = _lib.load()
    shape = _lib.ShapeStruct(1, 2, 4, 8, 4, 8, 8, 8, _lib.S2ATTN_F32)
    plan = _lib.PlanStruct()
    rc = lib.s2attn_forward(None, None, None, None, None, ctypes.byref(plan), ctypes.byref(shape), None)
    assert rc == -1 and b"null" in lib.s2attn_last_error()
    bad = _lib.ShapeStruct(1, 2, 4, 9, 4, 6, 8, 8, _lib.S2ATTN_F32)  # 9 % 6 != 0
    assert lib.s2attn_backward_workspace_bytes(ctypes.byref(bad)) == -1
    assert b"multiple" in lib.s2attn_last_error()
    wide = _lib.ShapeStruct(1, 1, 4, 8, 4, 8, 520, 520, _lib.S2ATTN_F32)
    assert lib.s2attn_backward_workspace_bytes(ctypes.byref(wide)) == -2  # unsupported head width
    dt = _lib.ShapeStruct(1, 1, 4, 8, 4, 8, 8, 8, 7)
    assert lib.s2attn_backward_workspace_bytes(ctypes.byref(dt)) == -1
    assert lib.s2attn_backward_workspace_bytes(ctypes.byref(shape)) == 1 * 2 * 4 * 8 * 8
    assert lib.s2attn_permute_to_nhwc(None, None, 1, 2, 3, 4, 3, None) == -1  # element size 3


# ---- plan builder -------------------------------------------------------------------------------


def _pairs_from_csr(col, roff, Wi, Wo):
    """(ho, wo, hi, wi) pairs of a CSR.  Gather direction (Wi = ps Wo): rows are ho, entries (hi, wi) at wo = 0, shifted by
    ps per output column (attention_torch.py:97-104).  Scatter direction (Wo = ps Wi, ps > 1): rows are hi, entries (ho, wo)
    at wi = 0, shifted by ps per input column (attention_torch.py:613-621)."""
    ref = Counter()
    up = Wo % Wi == 0 and Wo != Wi
    for r in range(len(roff) - 1):
        for z in range(int(roff[r]), int(roff[r + 1])):
            if up:
                ho, wo = divmod(int(col[z]), Wo)
                for wi in range(Wi):
                    ref[(ho, (wo + (Wo // Wi) * wi) % Wo, r, wi)] += 1
            else:
                hi, wi = divmod(int(col[z]), Wi)
                for wo in range(Wo):
                    ref[(r, wo, hi, (wi + (Wi // Wo) * wo) % Wi)] += 1
    return ref


def _pairs_from_plan(arrays, Hi, Wi, Ho, Wo):
    """Expands both run groupings back into (ho, wo, hi, wi) pairs the way the kernels index them: runs live on
    virtual latitudes (real latitude * ps + column class, W = min(Wi, Wo) columns each) of the finer grid, where query
    column j sees key columns (ws + t + j) mod W and key column j is seen by query columns (j - ws - t) mod W."""
    goff, gruns, gorder, soff, sruns, sorder = [a.numpy() for a in arrays]
    up = Wo % Wi == 0 and Wo != Wi
    psk, psq, W = (1, Wo // Wi, Wi) if up else (Wi // Wo, 1, Wo)
    gather, scatter = Counter(), Counter()
    for vo in range(Ho * psq):
        for ri in range(goff[vo], goff[vo + 1]):
            vi, ws, ln, hi = (int(x) for x in gruns[ri])
            assert hi == vi // psk and 0 <= ws < W and 1 <= ln <= W
            for j in range(W):
                for t in range(ln):
                    gather[(vo // psq, j * psq + vo % psq, hi, ((ws + t + j) % W) * psk + vi % psk)] += 1
    for vi in range(Hi * psk):
        for ri in range(soff[vi], soff[vi + 1]):
            vo, ws, ln, ho = (int(x) for x in sruns[ri])
            assert ho == vo // psq
            for j in range(W):
                for t in range(ln):
                    scatter[(ho, ((j - ws - t) % W) * psq + vo % psq, vi // psk, j * psk + vi % psk)] += 1
    return gather, scatter, gorder, sorder


@pytest.mark.parametrize(
    "ins,outs,gi,go,tc",
    [
        ((6, 12), (6, 12), "equiangular", "equiangular", None),
        ((2, 4), (2, 4), "equiangular", "equiangular", None),
        ((12, 24), (6, 8), "equiangular", "equiangular", None),
        ((9, 12), (5, 4), "equiangular", "equiangular", None),
        ((12, 24), (6, 12), "legendre-gauss", "legendre-gauss", 0.7),
        ((6, 12), (6, 12), "equiangular", "equiangular", 7.0),
        # scatter direction (up-sampling): psi keyed by input latitude
        ((6, 12), (12, 24), "equiangular", "equiangular", None),
        ((5, 4), (9, 12), "equiangular", "equiangular", None),
        ((6, 8), (12, 24), "legendre-gauss", "equiangular", 0.9),
    ],
)
def test_plan_covers_exactly_the_csr_pairs(ins, outs, gi, go, tc):
    up = outs[1] % ins[1] == 0 and outs[1] != ins[1]
    if up:  # rows index the (coarser) input grid, columns the output grid (attention.py:372-387)
        col, roff, _ = precompute_neighborhood_s2(outs, ins, go, gi, tc if tc is not None else math.pi / (ins[0] - 1))
    else:
        col, roff, _ = precompute_neighborhood_s2(ins, outs, gi, go, tc)
    arrays, nruns, ndense = build_host_plan(col, roff, ins[0], ins[1], outs[0], outs[1])
    ref = _pairs_from_csr(col, roff, ins[1], outs[1])
    gather, scatter, gorder, sorder = _pairs_from_plan(arrays, ins[0], ins[1], outs[0], outs[1])
    assert gather == ref and scatter == ref
    psk, psq = (1, outs[1] // ins[1]) if up else (ins[1] // outs[1], 1)
    assert sorted(gorder.tolist()) == list(range(outs[0] * psq)) and sorted(sorder.tolist()) == list(range(ins[0] * psk))
    if not up:
        lens = (roff[1:] - roff[:-1]).tolist()
        assert all(lens[gorder[i]] >= lens[gorder[i + 1]] for i in range(outs[0] - 1)), "rows must be ordered longest first"
    assert nruns <= col.numel()


def _pairs_from_items(plan, Hi, Wi, Ho, Wo):
    """Expands the hybrid kernels' work lists the way those kernels walk them: an item is one latitude (its runs) or a pair
    of adjacent latitudes whose merged bands carry, per band position, which of the two latitudes it belongs to."""
    up = Wo % Wi == 0 and Wo != Wi
    psk, psq, W = (1, Wo // Wi, Wi) if up else (Wi // Wo, 1, Wo)
    goff, gruns, _, soff, sruns, _ = [a.numpy() for a in plan.arrays()]
    gather, scatter = Counter(), Counter()
    seen = {"GATHER": [], "SCATTER": []}
    for side, out in (("GATHER", gather), ("SCATTER", scatter)):
        items, poff, pruns = [a.numpy() for a in plan.items(side)]
        off, runs = (goff, gruns) if side == "GATHER" else (soff, sruns)
        for lat, pair in items.tolist():
            members = []  # (own latitude, other latitude, aux, ws, len) in the single-run form of this grouping
            if pair < 0:
                seen[side].append(lat)
                members = [(lat, int(r[0]), int(r[1]), int(r[2])) for r in runs[off[lat] : off[lat + 1]]]
            else:
                seen[side] += [lat, lat + 1]
                for other, ws, ln, aux, dA, lenA, dB, lenB in pruns[poff[pair] : poff[pair + 1]].tolist():
                    assert 1 <= ln < 32 and 0 <= ws < W
                    for own, d, l in ((lat, dA, lenA), (lat + 1, dB, lenB)):
                        if l == 0:
                            continue
                        assert 0 <= d and d + l <= ln
                        # a run (ws', l) of the same grouping: gather bands start at ws + d, scatter bands END d before the union's end
                        members.append((own, other, (ws + d) % W if side == "GATHER" else (ws + ln - d - l) % W, l))
            for own, other, ws, ln in members:
                for j in range(W):
                    for t in range(ln):
                        if side == "GATHER":  # own = virtual output latitude, other = virtual input latitude
                            out[(own // psq, j * psq + own % psq, other // psk, ((ws + t + j) % W) * psk + other % psk)] += 1
                        else:  # own = virtual input latitude, other = virtual output latitude
                            out[(other // psq, ((j - ws - t) % W) * psq + other % psq, own // psk, j * psk + own % psk)] += 1
    return gather, scatter, seen


@pytest.mark.parametrize(
    "ins,outs,gi,go,tc",
    [
        ((24, 128), (24, 128), "equiangular", "equiangular", 2.5 * math.pi / 23),
        ((33, 160), (33, 160), "legendre-gauss", "legendre-gauss", 0.2),
        ((48, 256), (24, 128), "equiangular", "legendre-gauss", 0.3),
        ((20, 128), (41, 256), "equiangular", "equiangular", 0.35),  # up-sampling
        ((6, 12), (6, 12), "equiangular", "equiangular", None),  # too narrow for pairs: single latitudes only
    ],
)
def test_plan_work_lists_with_latitude_pairs_cover_exactly_the_csr_pairs(ins, outs, gi, go, tc):
    from torch_harmonics_amd.plan import build_host_blob

    up = outs[1] % ins[1] == 0 and outs[1] != ins[1]
    if up:
        col, roff, _ = precompute_neighborhood_s2(outs, ins, go, gi, tc)
    else:
        col, roff, _ = precompute_neighborhood_s2(ins, outs, gi, go, tc)
    plan = build_host_blob(col, roff, ins[0], ins[1], outs[0], outs[1])
    ref = _pairs_from_csr(col, roff, ins[1], outs[1])
    gather, scatter, seen = _pairs_from_items(plan, ins[0], ins[1], outs[0], outs[1])
    assert gather == ref and scatter == ref
    h, PH = plan.header, _lib.PH
    assert sorted(seen["GATHER"]) == list(range(h[PH["NVOUT"]])) and sorted(seen["SCATTER"]) == list(range(h[PH["NVIN"]]))
    if ins[1] >= 128:
        assert h[PH["GATHER_NPAIRS"]] > 0 and h[PH["SCATTER_NPAIRS"]] > 0, "the case is meant to form pairs"
    else:
        assert h[PH["GATHER_NPAIRS"]] == 0 and h[PH["SCATTER_NPAIRS"]] == 0


def test_plan_blob_is_self_describing():
    from torch_harmonics_amd.plan import build_host_blob, plan_from_blob

    col, roff, _ = precompute_neighborhood_s2((12, 24), (6, 12), "equiangular", "equiangular", 0.6)
    plan = build_host_blob(col, roff, 12, 24, 6, 12)
    h, PH = plan.header, _lib.PH
    assert h[PH["MAGIC"]] == _lib.PLAN_MAGIC and h[PH["TOTAL"]] == plan.blob.numel() and plan.blob.dtype == torch.int32
    assert (h[PH["NLAT_IN"]], h[PH["NLON_IN"]], h[PH["NLAT_OUT"]], h[PH["NLON_OUT"]]) == (12, 24, 6, 12)
    assert plan.blob[:32].tolist() == list(h)
    again = plan_from_blob(plan.blob.clone(), h, 12, 24, 6, 12)
    assert all(torch.equal(a, b) for a, b in zip(again.arrays(), plan.arrays()))
    with pytest.raises(RuntimeError, match="grid extents"):
        plan_from_blob(plan.blob, h, 12, 24, 6, 24)
    with pytest.raises(RuntimeError, match="header"):
        plan_from_blob(plan.blob[:-4], h, 12, 24, 6, 12)
    # the library refuses a plan made for other grids, before anything is launched
    lib = _lib.load()
    shape = _lib.ShapeStruct(1, 1, 12, 24, 6, 24, 8, 8, _lib.S2ATTN_F32)
    rc = lib.s2attn_forward(1, 1, 1, 1, 1, ctypes.byref(plan.struct), ctypes.byref(shape), None)
    assert rc == -1 and b"built for" in lib.s2attn_last_error()


@pytest.mark.parametrize(
    "ins,outs,cut", [((12, 24), (6, 12), 0.6), ((9, 48), (9, 48), 0.5), ((7, 120), (5, 40), 0.7), ((6, 40), (6, 40), 7.0), ((12, 80), (12, 80), 0.2)]
)
def test_plan_neighbor_arcs_hold_every_run(ins, outs, cut):
    """gather_span: per virtual output latitude an arc (first column, columns) of the circle; every column a run of that latitude
    gives query column 0 lies on it, rows without neighbors have an empty arc, and no arc is longer than the circle."""
    from torch_harmonics_amd.plan import build_host_blob

    col, roff, _ = precompute_neighborhood_s2(ins, outs, "equiangular", "equiangular", cut)
    plan = build_host_blob(col, roff, ins[0], ins[1], outs[0], outs[1])
    h, PH = plan.header, _lib.PH
    goff, gruns = plan.arrays()[0].tolist(), plan.arrays()[1].tolist()
    nvout, W = h[PH["NVOUT"]], min(ins[1], outs[1])
    span = plan.blob[h[PH["GATHER_SPAN"]] : h[PH["GATHER_SPAN"]] + 2 * nvout].view(nvout, 2).tolist()
    short = 0
    for r in range(nvout):
        s0, n = span[r]
        assert 0 <= n <= W and 0 <= s0 < W
        assert (n == 0) == (goff[r] == goff[r + 1])
        for g in range(goff[r], goff[r + 1]):
            _, ws, ln, _ = gruns[g]
            assert all(((ws + t - s0) % W) < n for t in range(ln)), (r, span[r], gruns[g])
        short += 0 < n < W
    if cut < 1.0:
        assert short > 0  # the arcs are not all whole circles


def test_plan_handles_arbitrary_unsorted_csr_with_duplicates():
    gen = torch.Generator().manual_seed(5)
    Hi, Wi, Ho, Wo = 5, 12, 4, 6
    rows = [torch.randint(0, Hi * Wi, (n,), generator=gen) for n in (7, 0, 19, 3)]
    col = torch.cat(rows)
    roff = torch.tensor([0, 7, 7, 26, 29])
    arrays, nruns, ndense = build_host_plan(col, roff, Hi, Wi, Ho, Wo)
    gather, scatter, _, _ = _pairs_from_plan(arrays, Hi, Wi, Ho, Wo)
    ref = _pairs_from_csr(col, roff, Wi, Wo)
    assert gather == ref and scatter == ref


def test_plan_merges_wrapping_intervals_into_one_circular_run():
    Wi = 16
    col = torch.tensor([0, 1, 2, 14, 15, 16 + 5, 16 + 6])  # lat 0: {14,15,0,1,2}; lat 1: {5,6}
    roff = torch.tensor([0, 7])
    arrays, nruns, ndense = build_host_plan(col, roff, 2, Wi, 1, Wi)
    assert nruns == 2
    assert arrays[1][:2].tolist() == [[0, 14, 5, 0], [1, 5, 2, 1]]


def test_plan_builder_rejects_malformed_csr():
    good_col = torch.tensor([0, 1, 2])
    with pytest.raises(RuntimeError, match="outside"):
        build_host_plan(torch.tensor([0, 1, 99]), torch.tensor([0, 3]), 2, 4, 1, 4)
    with pytest.raises(RuntimeError, match="row_off"):
        build_host_plan(good_col, torch.tensor([0, 2]), 2, 4, 1, 4)
    with pytest.raises(RuntimeError, match="multiple"):
        build_host_plan(good_col, torch.tensor([0, 3]), 2, 4, 1, 3)
    with pytest.raises(RuntimeError, match="nlat_out"):
        build_host_plan(good_col, torch.tensor([0, 1, 3]), 2, 4, 1, 4)


# ---- geometry -------------------------------------------------------------------------------------


@pytest.mark.parametrize("grid", ["equiangular", "legendre-gauss", "lobatto", "equiangular-trapezoidal"])
@pytest.mark.parametrize("nlat", [2, 5, 32, 33])
def test_product_quadrature_equals_oracle(grid, nlat):
    th, w = precompute_latitudes(nlat, grid)
    tho, wo = ogeo.colatitudes_and_weights(nlat, grid)
    assert torch.equal(th, tho) and torch.equal(w, wo)
    assert torch.equal(precompute_longitudes(24), ogeo.longitudes(24))
    with pytest.raises(ValueError):
        precompute_latitudes(8, "healpix")


@pytest.mark.parametrize(
    "ins,outs,gi,go,tc",
    [
        ((32, 64), (32, 64), "equiangular", "equiangular", None),
        ((12, 24), (3, 6), "equiangular", "equiangular", None),
        ((11, 24), (7, 12), "equiangular", "equiangular", None),
        ((24, 48), (12, 24), "equiangular", "legendre-gauss", 0.3),
        ((16, 32), (16, 32), "lobatto", "lobatto", 0.25),
        ((128, 256), (128, 256), "equiangular", "equiangular", 4 * math.pi / 127),
        ((6, 12), (6, 12), "equiangular", "equiangular", 2 * math.pi),
    ],
)
def test_product_neighborhood_equals_oracle(ins, outs, gi, go, tc):
    col, roff, row = precompute_neighborhood_s2(ins, outs, gi, go, tc)
    col_o, roff_o = ogeo.neighborhood_csr(ins, outs, gi, go, tc)
    assert torch.equal(col, col_o) and torch.equal(roff, roff_o)
    assert col.dtype == torch.int64 and roff.dtype == torch.int64
    assert torch.equal(row, torch.repeat_interleave(torch.arange(outs[0]), roff[1:] - roff[:-1]))


def test_product_neighborhood_equals_oracle_on_random_small_grids():
    """Degenerate and odd cases of the arc construction: one to five latitudes, one to four longitudes, cutoffs from nothing to
    beyond the sphere, every grid kind, longitude ratios 1-4 in both directions; element-equal to the oracle's psi."""
    import random

    rng = random.Random(2024)
    grids = ["equiangular", "legendre-gauss", "lobatto"]
    checked = 0
    for _ in range(150):
        Hi, Ho = rng.choice([2, 3, 4, 5, 7, 8, 12, 16, 23, 32]), rng.choice([2, 3, 4, 5, 7, 8, 12, 16, 23, 32])
        ratio, small = rng.choice([1, 1, 2, 3, 4]), rng.choice([1, 2, 3, 4, 6, 8, 16, 24, 33, 48])
        big = (Hi, small * ratio), (Ho, small)
        gi, go = rng.choice(grids), rng.choice(grids)
        tc = rng.choice([None, 1e-6, 0.01, 0.05, 0.1, 0.3, 0.7, 1.5, 3.0, 3.2, 7.0, math.pi * rng.random()])
        args = (big[0], big[1], gi, go) if rng.random() < 0.5 else (big[1], big[0], go, gi)  # psi is always built with nlon_in a multiple of nlon_out or the reverse
        want_col, want_off = ogeo.neighborhood_csr(*args, tc)
        col, off, row = precompute_neighborhood_s2(*args, tc)
        assert torch.equal(col, want_col) and torch.equal(off, want_off), (args, tc)
        assert torch.equal(row, torch.repeat_interleave(torch.arange(off.numel() - 1), off[1:] - off[:-1]))
        checked += 1
    assert checked == 150


@pytest.mark.parametrize(
    "ins,outs,gi,go,tc,nnz,lens",
    [
        ((721, 1440), (721, 1440), "equiangular", "equiangular", 3 * math.pi / 720, 99625, (29, 41, 5760)),
        ((721, 1440), (360, 720), "equiangular", "legendre-gauss", 2 * math.pi / 359, 77422, (48, 72, 6271)),
        ((361, 720), (361, 720), "legendre-gauss", "legendre-gauss", 8 * math.pi / 360, 237317, (197, 287, 5562)),
    ],
    ids=["cfg3", "cfg4", "cfg5"],
)
def test_product_neighborhood_at_benchmark_resolution(ins, outs, gi, go, tc, nnz, lens):
    """The band-limited builder against the restatement of the reference's full-grid loop, entry by entry, at the three
    large benchmark grids (its latitude band and slack are what could go wrong at 721 rows and not at 128)."""
    col, roff, _ = precompute_neighborhood_s2(ins, outs, gi, go, tc)
    col_o, roff_o = ogeo.neighborhood_csr(ins, outs, gi, go, tc)
    assert torch.equal(roff, roff_o) and torch.equal(col, col_o)
    n = roff[1:] - roff[:-1]
    assert col.numel() == nnz and (int(n.min()), int(n.median()), int(n.max())) == lens  # torch's median: the lower middle element


# ---- module ---------------------------------------------------------------------------------------


def test_module_state_and_defaults():
    m = tha.NeighborhoodAttentionS2(8, (12, 24), (6, 12), num_heads=2, k_channels=4, out_channels=6, use_qknorm=True)
    sd = m.state_dict()
    assert {k: tuple(v.shape) for k, v in sd.items()} == {
        "q_weights": (4, 8, 1, 1),
        "k_weights": (4, 8, 1, 1),
        "v_weights": (6, 8, 1, 1),
        "proj_weights": (6, 6, 1, 1),
        "q_bias": (4,),
        "k_bias": (4,),
        "v_bias": (6,),
        "proj_bias": (6,),
        "q_norm_weights": (2,),
        "k_norm_weights": (2,),
    }
    # the reference's four non-persistent buffers, plus the run-length plan of psi (also non-persistent: not in the state_dict)
    assert {n for n, _ in m.named_buffers()} == {"quad_weights", "psi_row_idx", "psi_col_idx", "psi_roff_idx", "psi_plan"}
    assert m.psi_plan.dtype == torch.int32 and m.psi_plan[:32].tolist() == m._psi_plan_header
    assert m.theta_cutoff == pytest.approx(math.pi / 5) and m.scale == pytest.approx(1 / math.sqrt(2))
    assert m.quad_weights.dtype == torch.float32 and m.quad_weights.shape == (12,)
    assert m.psi_roff_idx.shape == (7,) and not m.upsample
    bound = math.sqrt(6.0 / (8 + 4))
    assert float(m.q_weights.abs().max()) <= bound and float(m.proj_bias.abs().max()) == 0
    m2 = tha.NeighborhoodAttentionS2(8, (12, 24), (6, 12), num_heads=2, k_channels=4, out_channels=6, use_qknorm=True)
    m2.load_state_dict(sd)
    nb = tha.NeighborhoodAttentionS2(4, (6, 12), (6, 12), bias=False)
    assert nb.q_bias is None and "q_bias" not in nb.state_dict()


def test_module_constructor_errors():
    with pytest.raises(ValueError, match="integer multiple"):
        tha.NeighborhoodAttentionS2(4, (6, 10), (6, 4))
    with pytest.raises(ValueError, match="divides k_channels"):
        tha.NeighborhoodAttentionS2(6, (6, 12), (6, 12), num_heads=4)
    with pytest.raises(ValueError, match="divides out_channels"):
        tha.NeighborhoodAttentionS2(4, (6, 12), (6, 12), num_heads=4, out_channels=6)
    with pytest.raises(ValueError, match="positive"):
        tha.NeighborhoodAttentionS2(4, (6, 12), (6, 12), theta_cutoff=0.0)
    with pytest.raises(NotImplementedError):
        tha.NeighborhoodAttentionS2(4, (6, 12), (6, 12), optimized_kernel=False)


def test_module_upsampling_direction_state():
    """Up-sampling keys psi by input latitude and takes its default radius from the coarser (input) grid (attention.py:337-356,372-387)."""
    m = tha.NeighborhoodAttentionS2(4, (6, 12), (12, 24))
    assert m.upsample and m.psi_roff_idx.shape == (7,)
    assert m.theta_cutoff == pytest.approx(math.pi / 5)
    assert int(m.psi_col_idx.max()) < 12 * 24 and m.quad_weights.shape == (6,)
    col, roff = ogeo.neighborhood_csr((12, 24), (6, 12), "equiangular", "equiangular", math.pi / 5)
    assert torch.equal(m.psi_col_idx, col) and torch.equal(m.psi_roff_idx, roff)


def test_module_forward_checks_shapes_and_has_no_cpu_path():
    m = tha.NeighborhoodAttentionS2(4, (12, 24), (6, 12))
    with pytest.raises(RuntimeError, match="4-dimensional"):
        m(torch.randn(4, 6, 12))
    with pytest.raises(RuntimeError, match="query latitudes"):
        m(torch.randn(1, 4, 7, 12), torch.randn(1, 4, 12, 24), torch.randn(1, 4, 12, 24))
    with pytest.raises(RuntimeError, match="key longitudes"):
        m(torch.randn(1, 4, 6, 12), torch.randn(1, 4, 12, 23), torch.randn(1, 4, 12, 24))
    with pytest.raises(RuntimeError, match="single dtype"):
        m(torch.randn(1, 4, 6, 12), torch.randn(1, 4, 12, 24).double(), torch.randn(1, 4, 12, 24))
    with pytest.raises(RuntimeError, match="only run on a ROCm GPU"):
        m(torch.randn(1, 4, 6, 12), torch.randn(1, 4, 12, 24), torch.randn(1, 4, 12, 24))


# ---- operators ------------------------------------------------------------------------------------


def _op_args(device="cpu", dtype=torch.float32, nh=2):
    m = tha.NeighborhoodAttentionS2(8, (12, 24), (6, 12), num_heads=nh)
    k = torch.randn(2, 12, 24, 8, device=device, dtype=dtype)
    v = torch.randn(2, 12, 24, 4, device=device, dtype=dtype)
    q = torch.randn(2, 6, 12, 8, device=device, dtype=dtype)
    psi = [t.to(device) for t in (m.quad_weights, m.psi_col_idx, m.psi_roff_idx)]
    return k, v, q, psi


def test_operator_shape_propagation_on_meta_tensors():
    k, v, q, psi = _op_args("meta", torch.bfloat16)
    y = ops._neighborhood_s2_attention_optimized(k, v, q, *psi, 2, 24, 6, 12)
    assert y.shape == (2, 6, 12, 4) and y.dtype == torch.bfloat16 and y.device.type == "meta"
    y = ops.forward(k, v, q, *psi, 2, 24, 6, 12)
    assert y.shape == (2, 6, 12, 4)
    dk, dv, dq = ops.backward(k, v, q, y, *psi, 2, 24, 6, 12)
    assert dk.shape == k.shape and dv.shape == v.shape and dq.shape == q.shape
    x = torch.empty(2, 3, 4, 5, device="meta")
    assert ops.permute_to_nhwc(x).shape == (2, 4, 5, 3) and ops.permute_to_nchw(x).shape == (2, 5, 3, 4)


def test_operator_argument_errors():
    k, v, q, psi = _op_args()
    with pytest.raises(RuntimeError, match="divisible by num_heads"):
        ops.forward(k, v, q, *psi, 3, 24, 6, 12)
    with pytest.raises(RuntimeError, match="must match q dtype"):
        ops.forward(k.double(), v, q, *psi, 2, 24, 6, 12)
    with pytest.raises(RuntimeError, match="vice versa"):
        ops.forward(k, v, q, *psi, 2, 24, 6, 9)
    with pytest.raises(RuntimeError, match="num_heads must be positive"):
        ops.forward(k, v, q, *psi, 0, 24, 6, 12)
    with pytest.raises(RuntimeError, match="contiguous"):
        ops.forward(k.transpose(1, 2), v, q, *psi, 2, 24, 6, 12)
    with pytest.raises(RuntimeError, match="dy dtype"):
        ops.backward(k, v, q, torch.randn(2, 6, 12, 4).half(), *psi, 2, 24, 6, 12)
    with pytest.raises(RuntimeError, match="only run on a ROCm GPU"):
        ops.forward(k, v, q, *psi, 2, 24, 6, 12)
    with pytest.raises(RuntimeError, match="only run on a ROCm GPU"):
        ops.permute_to_nhwc(torch.randn(1, 2, 3, 4))
    with pytest.raises(RuntimeError, match="integer multiple"):
        ops.forward(k[:, :, :10].contiguous(), v[:, :, :10].contiguous(), q, *psi, 2, 10, 6, 12)


@pytest.mark.parametrize("modulus,key_lo,nkeys", [(12, 0, 6), (12, 2, 3), (12, -2, 10), (24, 0, 3)])
def test_regrouped_psi_is_a_stable_sort_by_latitude(modulus, key_lo, nkeys):
    """plan.get_transposed_csr against a plain loop: the entries of key key_lo + i, in CSR order, as (CSR row, col mod modulus);
    the launch order lists the keys by decreasing number of entries."""
    from torch_harmonics_amd import plan

    gen = torch.Generator().manual_seed(11)
    nrow = 7
    counts = torch.randint(0, 9, (nrow,), generator=gen)
    roff = torch.cat([torch.zeros(1, dtype=torch.int64), counts.cumsum(0)])
    col = torch.randint(0, 6 * 12, (int(roff[-1]),), generator=gen)  # unsorted, with duplicates
    plan.clear_plan_cache()
    t_lat, t_lon, t_off, t_order = plan.get_transposed_csr(col, roff, modulus, key_lo, nkeys)
    assert t_lat.dtype == torch.int32 and t_lon.dtype == torch.int32 and t_off.dtype == torch.int64 and t_order.dtype == torch.int32
    assert t_off.numel() == nkeys + 1
    want = [[] for _ in range(nkeys)]
    for r in range(nrow):
        for z in range(int(roff[r]), int(roff[r + 1])):
            key = int(col[z]) // modulus - key_lo
            if 0 <= key < nkeys:
                want[key].append((r, int(col[z]) % modulus))
    for i in range(nkeys):
        got = [(int(t_lat[z]), int(t_lon[z])) for z in range(int(t_off[i]), int(t_off[i + 1]))]
        assert got == want[i], f"key {key_lo + i}"
    lens = [len(w) for w in want]
    assert sorted(t_order.tolist()) == list(range(nkeys))
    assert [lens[i] for i in t_order.tolist()] == sorted(lens, reverse=True)
    # the library's host builder gives the same arrays
    lib = _lib.load()
    h_lat, h_lon = torch.full((col.numel(),), -7, dtype=torch.int32), torch.full((col.numel(),), -7, dtype=torch.int32)
    h_off, h_order = torch.zeros(nkeys + 1, dtype=torch.int64), torch.zeros(nkeys, dtype=torch.int32)
    n = lib.s2attn_ring_regroup_psi(col.data_ptr(), roff.data_ptr(), nrow, modulus, key_lo, nkeys, h_lat.data_ptr(), h_lon.data_ptr(), h_off.data_ptr(), h_order.data_ptr())
    lo, hi = int(t_off[0]), int(t_off[-1])  # the torch builder keeps every entry and points into the window; the host builder keeps the window only
    assert n == hi - lo and int(h_off[0]) == 0
    assert torch.equal(h_off, t_off - lo)
    assert torch.equal(h_lat[:n], t_lat[lo:hi]) and torch.equal(h_lon[:n], t_lon[lo:hi])
    assert torch.equal(h_order, t_order)
    again = plan.get_transposed_csr(col, roff, modulus, key_lo, nkeys)
    assert again[0] is t_lat  # served from the cache
    col[0] = (int(col[0]) + modulus) % (6 * 12)  # an in-place edit changes the version counter: rebuilt
    assert plan.get_transposed_csr(col, roff, modulus, key_lo, nkeys)[0] is not t_lat
    order = plan.get_row_order(roff)
    assert [int(counts[i]) for i in order.tolist()] == sorted(counts.tolist(), reverse=True)


def test_ring_entry_points_reject_bad_arguments_before_touching_the_gpu():
    lib = _lib.load()
    ok = _lib.RingShapeStruct(2, 4, 6, 4, 8, 16, 16, 16, 2, 0, 0, _lib.S2ATTN_F32)
    rs = lambda **kw: _lib.RingShapeStruct(**{**{f: getattr(ok, f) for f, _ in ok._fields_}, **kw})  # noqa: E731
    null10, null13, null14 = [None] * 10, [None] * 13, [None] * 14
    assert lib.s2attn_ring_forward_step(*null10, ctypes.byref(ok), None) == -1 and b"null" in lib.s2attn_last_error()
    assert lib.s2attn_ring_forward_step(*null10, None, None) == -1 and b"shape" in lib.s2attn_last_error()
    for bad, word in (
        (rs(pscale=0), b"pscale"),
        (rs(pscale=3), b"pscale"),  # 16 % 3 != 0
        (rs(lon_lo_kx=12), b"leaves the input grid"),  # 12 + 6 > 16
        (rs(nlon_out=9), b"exceeds"),  # 2 * 9 > 16
        (rs(dtype=5), b"dtype"),
        (rs(batch=0), b"positive"),
        (rs(ck=0), b"channel"),
    ):
        assert lib.s2attn_ring_backward_pass1(*null13, ctypes.byref(bad), None) == -1 and word in lib.s2attn_last_error(), word
    assert lib.s2attn_ring_backward_pass2(*null13, ctypes.byref(rs(ck=520)), None) == -2  # unsupported width
    assert lib.s2attn_ring_backward_pass2_transposed(*null14, ctypes.byref(ok), None) == -1 and b"null" in lib.s2attn_last_error()
    up = _lib.RingUpShapeStruct(2, 4, 6, 8, 16, 16, 16, 32, 2, 0, -1, _lib.S2ATTN_BF16)
    us = lambda **kw: _lib.RingUpShapeStruct(**{**{f: getattr(up, f) for f, _ in up._fields_}, **kw})  # noqa: E731
    assert lib.s2attn_ring_forward_step_upsample(*null10, ctypes.byref(up), None) == -1 and b"null" in lib.s2attn_last_error()
    for bad, word in ((us(pscale_out=3), b"pscale_out"), (us(nlon_out=33), b"pscale_out"), (us(lon_lo_kx=11), b"leaves the input grid"), (us(dtype=-1), b"dtype")):
        assert lib.s2attn_ring_backward_pass1_upsample(*[None] * 12, ctypes.byref(bad), None) == -1 and word in lib.s2attn_last_error(), word
    assert lib.s2attn_ring_backward_pass2_upsample(*null13, ctypes.byref(up), None) == -1 and b"null" in lib.s2attn_last_error()


def test_bench_refuses_more_than_one_gpu_with_a_message():
    """bench.py measures one GPU; --gpus N > 1 (or a multi-rank environment) exits with a message that says so, before any GPU use."""
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for argv, env in ((["--gpus", "2"], {}), ([], {"WORLD_SIZE": "4"})):
        proc = subprocess.run([sys.executable, os.path.join(root, "bench.py"), *argv], capture_output=True, text=True, env={**os.environ, **env}, timeout=300)
        assert proc.returncode == 2
        assert "one GPU" in proc.stderr and proc.stdout.strip() == ""


def test_mixed_launch_order_is_the_same_latitudes_interleaved_by_work():
    """gather_order_mixed / scatter_order_mixed: permutations of the latitudes in which the long-run list and the short-run list
    each keep their own order and the long-run latitudes are spread over the launch instead of forming its prefix."""
    from oracle import geometry as ogeo

    ins = outs = (48, 96)
    col, roff = ogeo.neighborhood_csr(ins, outs, "equiangular", "equiangular", 3 * torch.pi / 47)
    arrays, nruns, ndense, mixed = build_host_plan(col, roff, ins[0], ins[1], outs[0], outs[1], with_mixed=True)
    plain = build_host_plan(col, roff, ins[0], ins[1], outs[0], outs[1])
    assert all(torch.equal(a, b) for a, b in zip(arrays, plain[0])) and plain[1:] == (nruns, ndense)
    for order, mix, nd in ((arrays[2], mixed[0], ndense[0]), (arrays[5], mixed[1], ndense[1])):
        order, mix = order.tolist(), mix.tolist()
        assert sorted(mix) == list(range(len(order)))
        assert 0 < nd < len(order), "the case must have both kinds of latitudes"
        dense, vec = order[:nd], order[nd:]
        assert [r for r in mix if r in set(dense)] == dense and [r for r in mix if r in set(vec)] == vec
        where_dense = [i for i, r in enumerate(mix) if r in set(dense)]
        assert where_dense[0] <= 1 and where_dense[-1] >= len(mix) // 2  # spread out, not a prefix


def test_plan_cache_keys_accept_inference_tensors():
    """psi buffers created or moved under torch.inference_mode() have no version counter; the cache keys must not read one."""
    from torch_harmonics_amd import plan

    with torch.inference_mode():
        roff = torch.tensor([0, 2, 3], dtype=torch.int64)
        col = torch.tensor([0, 1, 5], dtype=torch.int64)
    assert roff.is_inference() and plan._version(roff) == 0 and plan._version(col) == 0
    normal = torch.zeros(3, dtype=torch.int64)
    v0 = plan._version(normal)
    normal.add_(1)
    assert plan._version(normal) == v0 + 1
    order = plan.get_row_order(roff)  # a cached lookup keyed by an inference tensor
    assert order.tolist() == [0, 1] and plan.get_row_order(roff) is order
    plan.clear_plan_cache()


@pytest.mark.parametrize("n", [100, 16384, 16384 * 3 + 7, 8192 * 64 + 13, 70001])
def test_weight_gradient_split_reduction(n):
    """g^T x with the reduction over n split into slices (taken from n >= 16384) equals the plain product, remainder rows included."""
    from torch_harmonics_amd.attention import _weight_grad

    gen = torch.Generator().manual_seed(n)
    g, x = torch.randn(n, 6, generator=gen, dtype=torch.float64), torch.randn(n, 5, generator=gen, dtype=torch.float64)
    torch.testing.assert_close(_weight_grad(g, x), g.t() @ x, rtol=1e-12, atol=1e-9)


def test_reference_operator_names_and_schemas_are_registered():
    """The C++ binding defines the reference's operators verbatim (attention_interface.cpp:85-86, 114-119) and implements them
    for the CUDA dispatch key (what ROCm tensors dispatch to); Python adds the fake kernels."""
    want = {
        "permute_to_nhwc": "attention_kernels::permute_to_nhwc(Tensor x) -> Tensor",
        "permute_to_nchw": "attention_kernels::permute_to_nchw(Tensor x) -> Tensor",
        "forward": "attention_kernels::forward(Tensor kx, Tensor vx, Tensor qy, Tensor quad_weights, Tensor col_idx, Tensor row_off, int "
        "num_heads, int nlon_in, int nlat_out, int nlon_out) -> Tensor",
        "backward": "attention_kernels::backward(Tensor kx, Tensor vx, Tensor qy, Tensor dy, Tensor quad_weights, Tensor col_idx, Tensor "
        "row_off, int num_heads, int nlon_in, int nlat_out, int nlon_out) -> (Tensor, Tensor, Tensor)",
    }
    for name, schema in want.items():
        op = getattr(torch.ops.attention_kernels, name).default
        assert str(op._schema) == schema
        assert torch.Tag.pt2_compliant_tag in op.tags
        assert torch._C._dispatch_has_kernel_for_dispatch_key(f"attention_kernels::{name}", "CUDA")
        assert torch._C._dispatch_has_kernel_for_dispatch_key(f"attention_kernels::{name}", "Meta")
    assert ops.forward is torch.ops.attention_kernels.forward and ops.backward is torch.ops.attention_kernels.backward
    assert os.path.exists(_lib.TORCH_LIB_PATH)
    # fake kernels: shapes and dtypes without touching a device
    with torch._subclasses.fake_tensor.FakeTensorMode():
        k, v, q = torch.empty(2, 12, 24, 8), torch.empty(2, 12, 24, 4), torch.empty(2, 6, 12, 8)
        w, ci, ro = torch.empty(12), torch.empty(50, dtype=torch.int64), torch.empty(7, dtype=torch.int64)
        y = torch.ops.attention_kernels.forward(k, v, q, w, ci, ro, 2, 24, 6, 12)
        assert y.shape == (2, 6, 12, 4)
        dk, dv, dq = torch.ops.attention_kernels.backward(k, v, q, y, w, ci, ro, 2, 24, 6, 12)
        assert dk.shape == k.shape and dv.shape == v.shape and dq.shape == q.shape


def test_ring_and_autograd_operators_carry_the_reference_names_and_argument_lists():
    """attention_kernels::forward_ring_step ... backward_ring_step_upsample_pass2, split_csr_rows (attention_interface.cpp:136-189)
    and the autograd-carrying _neighborhood_s2_attention_optimized (attention_optimized.py:230) exist under the reference's names
    with its argument names, order and written-to arguments (Python fragments of the namespace; ints are SymInt there)."""
    ring_tail = "Tensor quad_weights, Tensor col_idx, Tensor row_off, Tensor row_idx, int nlon_in, int pscale, int lon_lo_kx, int lat_halo_start, int nlat_out, int nlon_out, int n_long_rows, int max_row_len, int mid_row_len"
    up_tail = "Tensor quad_weights, Tensor col_idx, Tensor row_off, int nlon_in, int nlon_out_global, int pscale_out, int lon_lo_kx, int lat_halo_start, int nlat_out, int nlon_out"
    want = {
        "split_csr_rows": ("Tensor row_idx, Tensor row_off, int nlat_out", "(int, int, int)"),
        "forward_ring_step": ("Tensor kx, Tensor vx, Tensor qy, Tensor! y_acc, Tensor! alpha_sum_buf, Tensor! qdotk_max_buf, " + ring_tail, "()"),
        "backward_ring_step_pass1": (
            "Tensor kx, Tensor vx, Tensor qy, Tensor dy, Tensor! alpha_sum_buf, Tensor! qdotk_max_buf, Tensor! integral_buf, Tensor! alpha_k_buf, Tensor! alpha_kvw_buf, " + ring_tail,
            "()",
        ),
        "backward_ring_step_pass2": (
            "Tensor kx, Tensor vx, Tensor qy, Tensor dy, Tensor alpha_sum_buf, Tensor qdotk_max_buf, Tensor integral_norm_buf, Tensor! dkx, Tensor! dvx, " + ring_tail,
            "()",
        ),
        "forward_ring_step_upsample": ("Tensor kx, Tensor vx, Tensor qy, Tensor! y_acc, Tensor! alpha_sum_buf, Tensor! qdotk_max_buf, " + up_tail, "()"),
        "backward_ring_step_upsample_pass1": (
            "Tensor kx, Tensor vx, Tensor qy, Tensor dy, Tensor qdotk_max_buf, Tensor! integral_buf, Tensor! alpha_k_buf, Tensor! alpha_kvw_buf, " + up_tail,
            "()",
        ),
        "backward_ring_step_upsample_pass2": (
            "Tensor kx, Tensor vx, Tensor qy, Tensor dy, Tensor alpha_sum_buf, Tensor qdotk_max_buf, Tensor integral_norm_buf, Tensor! dkx, Tensor! dvx, " + up_tail,
            "()",
        ),
        "_neighborhood_s2_attention_optimized": (
            "Tensor kw, Tensor vw, Tensor qw, Tensor quad_weights, Tensor col_idx, Tensor row_off, int nh, int nlon_in, int nlat_out, int nlon_out",
            "Tensor",
        ),
    }
    for name, (args, ret) in want.items():
        schema = getattr(torch.ops.attention_kernels, name).default._schema
        got = ", ".join(("Tensor!" if a.alias_info is not None and a.alias_info.is_write else str(a.type).replace("SymInt", "int")) + " " + a.name for a in schema.arguments)
        assert got == args, f"{name}: {got}"
        rets = [str(r.type).replace("SymInt", "int") for r in schema.returns]
        assert (("(" + ", ".join(rets) + ")") if len(rets) != 1 else rets[0]) == ret, name
    assert torch.ops.attention_kernels.split_csr_rows(torch.tensor([1, 0, 2], dtype=torch.int32), torch.tensor([0, 3, 3000, 3001]), 3) == (1, 2997, 3)


def test_point_strides_are_validated_on_the_host():
    """A tensor may be a column block of a wider buffer (point stride > packed row); strides must cover the packed row and be
    multiples of 4 elements."""
    lib = _lib.load()
    ok = _lib.ShapeStruct(1, 8, 721, 1440, 721, 1440, 32, 32, _lib.S2ATTN_F32, 768, 768, 768, 0, 0, 768, 768, 768)
    assert lib.s2attn_backward_saved_workspace_bytes(ctypes.byref(ok)) == 8 * 721 * 1440 * 8
    short = _lib.ShapeStruct(1, 8, 721, 1440, 721, 1440, 32, 32, _lib.S2ATTN_F32, 128)  # ld_k below num_heads * ck = 256
    assert lib.s2attn_backward_saved_workspace_bytes(ctypes.byref(short)) == -1 and b"point stride" in lib.s2attn_last_error()
    odd = _lib.ShapeStruct(1, 8, 721, 1440, 721, 1440, 32, 32, _lib.S2ATTN_F32, 0, 258)
    assert lib.s2attn_backward_saved_workspace_bytes(ctypes.byref(odd)) == -1
    assert ops.takes_column_blocks(torch.float32, 32, 32, 1440, 1440) and not ops.takes_column_blocks(torch.float32, 64, 64, 720, 720)
    assert not ops.takes_column_blocks(torch.bfloat16, 32, 32, 1440, 1440) and not ops.takes_column_blocks(torch.float32, 32, 32, 48, 48)


def test_fused_projection_function_matches_separate_linears():
    """_FusedLinear1x1 on the CPU (pure torch): outputs, input gradient, weight and bias gradients equal three F.linear,
    both when the gradients arrive as column blocks of one buffer and when they do not."""
    from torch_harmonics_amd.attention import _column_blocks_of_one_buffer, _FusedLinear1x1

    gen = torch.Generator().manual_seed(3)
    x = torch.randn(2, 3, 5, 6, generator=gen, dtype=torch.float64, requires_grad=True)
    ws = [torch.randn(n, 6, generator=gen, dtype=torch.float64, requires_grad=True) for n in (4, 4, 8)]
    bs = [torch.randn(n, generator=gen, dtype=torch.float64, requires_grad=True) for n in (4, 4, 8)]
    outs = _FusedLinear1x1.apply(x, ws[0], bs[0], ws[1], bs[1], ws[2], bs[2])
    ref = [torch.nn.functional.linear(x, w, b) for w, b in zip(ws, bs)]
    assert all(torch.allclose(a, b) for a, b in zip(outs, ref)) and outs[0].stride(2) == 16
    gbuf = torch.randn(2, 3, 5, 16, generator=gen, dtype=torch.float64)
    blocks = gbuf.split([4, 4, 8], dim=-1)
    assert _column_blocks_of_one_buffer(blocks, [4, 4, 8]) is not None and _column_blocks_of_one_buffer([b.contiguous() for b in blocks], [4, 4, 8]) is None
    for grads in (blocks, [b.contiguous() for b in blocks]):
        for t in [x] + ws + bs:
            t.grad = None
        torch.autograd.backward(_FusedLinear1x1.apply(x, ws[0], bs[0], ws[1], bs[1], ws[2], bs[2]), grads)
        got = [t.grad.clone() for t in [x] + ws + bs]
        for t in [x] + ws + bs:
            t.grad = None
        torch.autograd.backward([torch.nn.functional.linear(x, w, b) for w, b in zip(ws, bs)], grads)
        assert all(torch.allclose(a, t.grad) for a, t in zip(got, [x] + ws + bs))


def test_projections_fed_from_and_to_nchw_match_plain_linear():
    """_FusedLinear1x1NCHW (several projections of an NCHW input as one GEMM with a transposed operand, NHWC column blocks out) and
    _Linear1x1ToNCHW (NHWC in, NCHW out): outputs and every gradient against F.linear on permuted tensors, on a grid long enough
    for the split weight-gradient reduction."""
    from torch_harmonics_amd.attention import _FusedLinear1x1NCHW, _Linear1x1ToNCHW

    torch.manual_seed(0)
    B, C, H, W = 2, 12, 5, 3501  # 17505 points: three slices of the reduction
    x = torch.randn(B, C, H, W, dtype=torch.float64, requires_grad=True)
    ws = [torch.randn(n, C, dtype=torch.float64, requires_grad=True) for n in (8, 4, 16)]
    bs = [torch.randn(n, dtype=torch.float64, requires_grad=True) for n in (8, 4, 16)]
    outs = _FusedLinear1x1NCHW.apply(x, ws[0], bs[0], ws[1], bs[1], ws[2], bs[2])
    assert outs[0].untyped_storage().data_ptr() == outs[2].untyped_storage().data_ptr()  # column blocks of one buffer
    ref = [torch.nn.functional.linear(x.permute(0, 2, 3, 1), w, b) for w, b in zip(ws, bs)]
    for o, r in zip(outs, ref):
        assert torch.allclose(o, r, atol=1e-10)
    gs = [torch.randn_like(o) for o in outs]
    for a, r in zip(torch.autograd.grad(outs, [x] + ws + bs, gs), torch.autograd.grad(ref, [x] + ws + bs, gs)):
        assert torch.allclose(a, r, atol=1e-8)
    (single,) = _FusedLinear1x1NCHW.apply(x, ws[1], None)
    assert torch.allclose(single, torch.nn.functional.linear(x.permute(0, 2, 3, 1), ws[1]), atol=1e-10)

    y = torch.randn(B, H, W, C, dtype=torch.float64, requires_grad=True)
    w = torch.randn(7, C, dtype=torch.float64, requires_grad=True)
    b = torch.randn(7, dtype=torch.float64, requires_grad=True)
    o = _Linear1x1ToNCHW.apply(y, w, b)
    r = torch.nn.functional.linear(y, w, b).permute(0, 3, 1, 2)
    assert o.is_contiguous() and torch.allclose(o, r, atol=1e-10)
    g = torch.randn_like(o)
    for a, rr in zip(torch.autograd.grad(o, [y, w, b], g), torch.autograd.grad(r, [y, w, b], g)):
        assert torch.allclose(a, rr, atol=1e-8)


def test_plan_blob_is_cached_on_disk(tmp_path, monkeypatch):
    """A module's plan blob is written to $S2ATTN_CACHE_DIR by the first constructor and read back by the next one; a file that
    does not describe the problem is ignored and replaced; "off" disables the cache."""
    import os

    from torch_harmonics_amd import NeighborhoodAttentionS2

    monkeypatch.setenv("S2ATTN_CACHE_DIR", str(tmp_path))
    kw = dict(in_channels=8, in_shape=(12, 24), out_shape=(6, 12), num_heads=2, theta_cutoff=0.5)
    m1 = NeighborhoodAttentionS2(**kw)
    files = sorted(os.listdir(tmp_path))
    assert len(files) == 1 and files[0].startswith("plan_") and files[0].endswith(".npy")
    stamp = os.stat(tmp_path / files[0]).st_mtime_ns
    m2 = NeighborhoodAttentionS2(**kw)
    assert torch.equal(m1.psi_plan, m2.psi_plan) and m1._psi_plan_header == m2._psi_plan_header
    assert os.stat(tmp_path / files[0]).st_mtime_ns == stamp  # read, not rewritten
    m3 = NeighborhoodAttentionS2(**{**kw, "theta_cutoff": 0.7})  # another psi: another file
    assert len(os.listdir(tmp_path)) == 2 and not torch.equal(m3.psi_plan[: m1.psi_plan.numel()], m1.psi_plan)
    (tmp_path / files[0]).write_bytes(b"not a plan")
    m4 = NeighborhoodAttentionS2(**kw)
    assert torch.equal(m4.psi_plan, m1.psi_plan)
    import numpy as np

    assert np.load(tmp_path / files[0]).shape == (m1.psi_plan.numel(),)  # rewritten
    monkeypatch.setenv("S2ATTN_CACHE_DIR", "off")
    for f in os.listdir(tmp_path):
        os.remove(tmp_path / f)
    NeighborhoodAttentionS2(**kw)
    assert os.listdir(tmp_path) == []


def test_module_constructor_time_at_the_headline_grid():
    """721 x 1440 self-attention: psi from its structure plus the plan build stay far below a second (the reference's loop over
    output latitudes takes seconds there)."""
    import time

    from torch_harmonics_amd import NeighborhoodAttentionS2
    from torch_harmonics_amd.neighborhood import _neighborhood_cached, _segments_cached

    _neighborhood_cached.cache_clear()
    _segments_cached.cache_clear()
    t0 = time.perf_counter()
    m = NeighborhoodAttentionS2(16, (721, 1440), (721, 1440), num_heads=1, theta_cutoff=3 * math.pi / 720)
    dt = time.perf_counter() - t0
    print(f"constructor at 721x1440: {dt * 1e3:.0f} ms")
    assert m.psi_col_idx.numel() == 99625 and dt < 1.0
