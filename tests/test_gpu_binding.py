"""
The boundary as a maintainer of the reference would use it: the operators registered by the C++ binding under the reference's
own names (attention_kernels::forward / backward / permute_to_nhwc / permute_to_nchw, attention_interface.cpp:85-119), called
through torch.ops; the plan a module builds in its constructor (no device-to-host copy in any forward, HIP graph capture of a
fresh module); and the one documented difference in how non-finite inputs spread.
"""

import math

import pytest
import torch

from oracle import cpu_attention as oracle
from oracle import geometry as ogeo
from tests.util import SEED, assert_close, randn_inputs

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = dict(rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize(
    "B,nh,d,ins,outs,tc",
    [(2, 2, 8, (12, 24), (6, 12), 0.6), (1, 2, 32, (24, 96), (24, 96), 0.5), (1, 1, 64, (10, 80), (10, 80), 1.2), (2, 1, 16, (6, 12), (12, 24), 0.9)],
    ids=["vector_down", "hybrid_d32", "m32_d64", "upsample"],
)
def test_reference_named_operators_match_the_oracle(B, nh, d, ins, outs, tc):
    import torch_harmonics_amd  # noqa: F401  (loading the package registers the operators)

    up = oracle.is_upsample(ins[1], outs[1])
    col, roff = ogeo.neighborhood_csr(outs, ins, "equiangular", "equiangular", tc) if up else ogeo.neighborhood_csr(ins, outs, "equiangular", "equiangular", tc)
    w = ogeo.attention_quad_weights(ins[0], ins[1], "equiangular")
    k, v, q, dy = randn_inputs(B, ins[0], ins[1], outs[0], outs[1], nh, d, d)
    kd, vd, qd, gd, wd, cd, rd = [t.to(DEV) for t in (k, v, q, dy, w, col, roff)]
    geo = (wd, cd, rd, nh, ins[1], outs[0], outs[1])
    ak = torch.ops.attention_kernels
    y = ak.forward(kd, vd, qd, *geo)
    dk, dv, dq = ak.backward(kd, vd, qd, gd, *geo)
    kr, vr, qr = [t.double().requires_grad_(True) for t in (k, v, q)]
    y64 = oracle.dense_attention_f64(kr, vr, qr, w, col, roff, nh)
    y64.backward(dy.double())
    for name, got, want in (("y", y, y64.detach()), ("dk", dk, kr.grad), ("dv", dv, vr.grad), ("dq", dq, qr.grad)):
        assert_close(name, got, want, **TOL)
    x = torch.randn(2, 5, 7, 3, device=DEV)
    assert torch.equal(ak.permute_to_nhwc(x), x.permute(0, 2, 3, 1)) and torch.equal(ak.permute_to_nchw(x), x.permute(0, 3, 1, 2))
    # schema, fake-kernel and dispatch checks of the raw operators (tests/test_attention.py:829-892 runs them on the autograd op)
    torch.library.opcheck(ak.forward, (kd, vd, qd, *geo))
    torch.library.opcheck(ak.backward, (kd, vd, qd, gd, *geo))
    torch.library.opcheck(ak.permute_to_nhwc, (x,))


def _module_and_inputs(C=64, nh=2, ins=(24, 96), outs=(24, 96)):
    from torch_harmonics_amd import NeighborhoodAttentionS2

    torch.manual_seed(SEED)
    m = NeighborhoodAttentionS2(C, ins, outs, num_heads=nh, theta_cutoff=0.4).to(DEV)
    x = torch.randn(2, C, *outs, device=DEV, requires_grad=True)
    return m, x


def test_fresh_module_runs_without_any_device_to_host_copy():
    """The plan is built in the constructor from the host CSR and moves with the module: neither the first forward nor the
    first backward may synchronise (the reference's per-call row sort also stays on the device, attention_cuda_utils.cu:74-113)."""
    m, x = _module_and_inputs()
    g = torch.randn(2, 64, 24, 96, device=DEV)
    torch.cuda.synchronize()
    torch.cuda.set_sync_debug_mode("error")
    try:
        out = m(x)
        out.backward(g)
    finally:
        torch.cuda.set_sync_debug_mode("default")
    torch.cuda.synchronize()
    assert torch.isfinite(out).all() and torch.isfinite(x.grad).all()
    # and it is the same result as through the plan derived from (col_idx, row_off) by the operator's own cache
    from torch_harmonics_amd import ops

    k = torch.randn(2, 24, 96, 64, device=DEV)
    q = torch.randn(2, 24, 96, 64, device=DEV) / math.sqrt(32)
    geo = (m.quad_weights, m.psi_col_idx, m.psi_roff_idx, 2, 96, 24, 96)
    y1, l1 = ops.forward_lse(k, k, q, *geo)
    y2, l2 = ops.forward_lse(k, k, q, *geo, m.psi_plan, m._psi_plan_header)
    assert torch.equal(y1, y2) and torch.equal(l1, l2)


def test_fresh_module_attention_captures_into_a_hip_graph_without_warm_up():
    """Forward and backward of the attention op with a freshly built module's plan, captured at their first call and replayed
    on new data: every replay equals the eager result (nothing is allocated by the library, nothing synchronises)."""
    from torch_harmonics_amd import ops

    m, _ = _module_and_inputs(ins=(20, 80), outs=(20, 80))
    geo = (m.quad_weights, m.psi_col_idx, m.psi_roff_idx, 2, 80, 20, 80, m.psi_plan, m._psi_plan_header)
    gen = torch.Generator(device=DEV).manual_seed(5)
    k, v, dy = [torch.randn(1, 20, 80, 64, device=DEV, generator=gen) for _ in range(3)]
    q = torch.randn(1, 20, 80, 64, device=DEV, generator=gen) / math.sqrt(32)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            y, lse = ops.forward_lse(k, v, q, *geo)
            dk, dv, dq = ops.backward_saved(k, v, q, dy, y, lse, *geo)
    torch.cuda.current_stream().wait_stream(side)
    for rep in range(3):
        for t in (k, v, dy):
            t.copy_(torch.randn(t.shape, device=DEV, generator=gen))
        q.copy_(torch.randn(q.shape, device=DEV, generator=gen) / math.sqrt(32))
        graph.replay()
        torch.cuda.synchronize()
        ye, le = ops.forward_lse(k, v, q, *geo)
        ge = ops.backward_saved(k, v, q, dy, ye, le, *geo)
        torch.cuda.synchronize()
        assert torch.equal(y, ye) and all(torch.equal(a, b) for a, b in zip((dk, dv, dq), ge)), f"replay {rep} differs from the eager result"


@pytest.mark.parametrize("d,W", [(32, 96), (8, 24)], ids=["matrix_core_tiles", "vector_kernels"])
def test_non_finite_key_reaches_its_neighbors_and_at_most_their_tiles(d, W):
    """A NaN in one key row makes every query whose neighborhood holds that point NaN, as in the reference.  The reference
    touches true neighbors only (attention_cuda_fwd.cu:137-173); the matrix-core families multiply whole tiles, so the NaN
    may also reach queries of the same latitude band whose staged tile holds the point (0 x NaN): never another head or batch
    entry, never a latitude whose band does not include the point's latitude, never a longitude further than a tile and a run
    away.  The vector kernels touch true neighbors only."""
    from torch_harmonics_amd import ops

    H, nh, tc = 24, 2, 0.45
    col, roff = ogeo.neighborhood_csr((H, W), (H, W), "equiangular", "equiangular", tc)
    w = ogeo.attention_quad_weights(H, W, "equiangular")
    k, v, q, _ = randn_inputs(2, H, W, H, W, nh, d, d)
    hi0, wi0 = 12, 10
    mask = oracle.dense_mask(col, roff, H, W, H, W).reshape(H, W, H, W)[:, :, hi0, wi0]  # queries that see the point
    assert mask.any() and not mask.all()
    kd, vd, qd, wd, cd, rd = [t.to(DEV) for t in (k, v, q, w, col, roff)]
    geo = (wd, cd, rd, nh, W, H, W)
    clean = ops.forward(kd, vd, qd, *geo)
    kd[0, hi0, wi0, :d] = float("nan")  # batch 0, head 0
    dirty = ops.forward(kd, vd, qd, *geo)
    torch.cuda.synchronize()
    bad = torch.isnan(dirty[0, :, :, :d]).any(-1).cpu()
    assert bool(bad[mask].all()), "every query that sees the point must be NaN"
    assert torch.equal(dirty[1], clean[1]) and torch.equal(dirty[0, :, :, d:], clean[0, :, :, d:]), "other batch entries and heads are untouched"
    extra = bad & ~mask
    if d == 8:
        assert not extra.any(), "the vector kernels touch true neighbors only"
        return
    rows_with_point = mask.any(dim=1)
    assert not extra[~rows_with_point].any(), "a latitude whose band does not hold the point's latitude is untouched"
    maxlen = int(mask.sum(dim=1).max())
    lon = torch.arange(W)
    dist = torch.minimum((lon - wi0) % W, (wi0 - lon) % W)
    assert not extra[:, dist > 64 + maxlen].any(), "a query further than a tile and a run from the point is untouched"
    assert torch.equal(dirty[0, :, :, :d][~bad.to(DEV)], clean[0, :, :, :d][~bad.to(DEV)])


@pytest.mark.parametrize("share", ["qkv", "kv"])
def test_column_blocks_of_a_fused_projection_are_read_and_written_in_place(share):
    """q | k | v as column blocks of one (B, nlat, nlon, 3C) buffer (or k | v of a 2C one): same y, lse, dq, dk, dv, bit for bit,
    as on contiguous copies, and the gradients come back as the column blocks of ONE new buffer."""
    from torch_harmonics_amd import ops

    B, nh, d, H, W = 2, 2, 32, 12, 96
    C = nh * d
    col, roff = ogeo.neighborhood_csr((H, W), (H, W), "equiangular", "equiangular", 0.6)
    w = ogeo.attention_quad_weights(H, W, "equiangular")
    gen = torch.Generator(device=DEV).manual_seed(11)
    geo = (w.to(DEV), col.to(DEV), roff.to(DEV), nh, W, H, W)
    if share == "qkv":
        buf = torch.randn(B, H, W, 3 * C, device=DEV, generator=gen)
        q, k, v = buf.split([C, C, C], dim=-1)
    else:
        buf = torch.randn(B, H, W, 2 * C, device=DEV, generator=gen)
        k, v = buf.split([C, C], dim=-1)
        q = torch.randn(B, H, W, C, device=DEV, generator=gen)
    q = q / math.sqrt(d) if share == "kv" else q
    dy = torch.randn(B, H, W, C, device=DEV, generator=gen)
    assert not k.is_contiguous()
    y, lse = ops.forward_lse(k, v, q, *geo)
    dk, dv, dq = ops.backward_saved(k, v, q, dy, y, lse, *geo)
    yc, lsec = ops.forward_lse(k.contiguous(), v.contiguous(), q.contiguous(), *geo)
    dkc, dvc, dqc = ops.backward_saved(k.contiguous(), v.contiguous(), q.contiguous(), dy, yc, lsec, *geo)
    torch.cuda.synchronize()
    assert torch.equal(y, yc) and torch.equal(lse, lsec)
    assert torch.equal(dk, dkc) and torch.equal(dv, dvc) and torch.equal(dq, dqc)
    assert dk.untyped_storage().data_ptr() == dv.untyped_storage().data_ptr() and dk.stride(2) == buf.shape[3]
    assert (dq.untyped_storage().data_ptr() == dk.untyped_storage().data_ptr()) == (share == "qkv")
    # shapes whose kernels do not take column blocks refuse them (the module then projects into separate tensors)
    small = torch.randn(1, H, W, 3 * 16, device=DEV, generator=gen)
    qs, ks, vs = small.split([16, 16, 16], dim=-1)
    with pytest.raises(RuntimeError, match="point stride"):
        ops.forward_lse(ks, vs, qs, geo[0], geo[1], geo[2], 1, W, H, W)


def _geo(ins, outs, tc):
    col, roff = ogeo.neighborhood_csr(ins, outs, "equiangular", "equiangular", tc)
    w = ogeo.attention_quad_weights(ins[0], ins[1], "equiangular")
    return w.to(DEV), col.to(DEV), roff.to(DEV)


@pytest.mark.parametrize("d,dtype", [(16, torch.float32), (64, torch.bfloat16), (32, torch.bfloat16), (32, torch.float32)], ids=["d16_fp32", "d64_bf16", "d32_bf16", "d32_fp32"])
def test_slices_of_a_fused_buffer_work_for_every_kernel_family(d, dtype):
    """q, k, v given as column blocks of one (B, H, W, 3C) buffer: only the fp32 32-channel heads on wide grids are read in place;
    every other shape must be copied by the Python operators (and give what contiguous tensors give), not refused by the library."""
    from torch_harmonics_amd import ops

    nh, ins = 2, (12, 96)
    w, col, roff = _geo(ins, ins, 0.5)
    g = torch.Generator().manual_seed(SEED)
    buf = (0.5 * torch.randn(2, *ins, 3 * nh * d, generator=g)).to(dtype).to(DEV)
    dy = torch.randn(2, *ins, nh * d, generator=g).to(dtype).to(DEV)
    geo = (w, col, roff, nh, ins[1], ins[0], ins[1])

    def run(q, k, v):
        q, k, v = [t.detach().requires_grad_(True) for t in (q, k, v)]
        y = ops.neighborhood_s2_attention(k, v, q, *geo)
        y.backward(dy)
        return y.detach(), k.grad, v.grad, q.grad

    q, k, v = buf.chunk(3, dim=-1)
    assert not k.is_contiguous()
    got = run(q, k, v)
    want = run(q.contiguous(), k.contiguous(), v.contiguous())
    for name, g_, w_ in zip(("y", "dk", "dv", "dq"), got, want):
        assert torch.equal(g_, w_), f"{name}: slices of a fused buffer give something else than contiguous copies"
    # an expanded (stride 0) tensor is not a column block either
    ke = k[:, :, :1].expand(-1, -1, ins[1], -1)
    got = run(q, ke, v)
    want = run(q.contiguous(), ke.contiguous(), v.contiguous())
    for name, g_, w_ in zip(("y", "dk", "dv", "dq"), got, want):
        assert torch.equal(g_, w_), f"{name}: expanded key"


def test_backward_operators_pass_opcheck_on_column_blocks():
    """The fake kernels of the backward operators describe the gradients as the binding lays them out: column blocks of one new
    buffer when k | v | q are disjoint column blocks of one buffer."""
    nh, d, ins = 2, 32, (12, 96)
    w, col, roff = _geo(ins, ins, 0.5)
    g = torch.Generator().manual_seed(SEED)
    buf = (0.5 * torch.randn(2, *ins, 3 * nh * d, generator=g)).to(DEV)
    dy = torch.randn(2, *ins, nh * d, generator=g).to(DEV)
    q, k, v = buf.chunk(3, dim=-1)
    geo = (w, col, roff, nh, ins[1], ins[0], ins[1])
    sk = torch.ops.s2attn_kernels
    y, lse = sk.forward_lse(k, v, q, *geo)
    dk, dv, dq = sk.backward_saved(k, v, q, dy, y, lse, *geo)
    assert dk.stride() == k.stride() and dv.stride() == v.stride() and dq.stride() == q.stride()
    assert dk.untyped_storage().data_ptr() == dv.untyped_storage().data_ptr() == dq.untyped_storage().data_ptr()
    torch.library.opcheck(sk.forward_lse, (k, v, q, *geo))
    torch.library.opcheck(sk.backward_saved, (k, v, q, dy, y, lse, *geo))
    torch.library.opcheck(torch.ops.attention_kernels.backward, (k, v, q, dy, *geo))
    # k | v fused, q separate
    qs = q.contiguous()
    torch.library.opcheck(sk.backward_saved, (k, v, qs, dy, y, lse, *geo))


def test_overlapping_column_blocks_get_separate_gradients():
    """k and v given as the SAME slice of a wider buffer: their gradients must not share memory."""
    nh, d, ins = 2, 32, (12, 96)
    w, col, roff = _geo(ins, ins, 0.5)
    g = torch.Generator().manual_seed(SEED)
    buf = (0.5 * torch.randn(2, *ins, 2 * nh * d, generator=g)).to(DEV)
    dy = torch.randn(2, *ins, nh * d, generator=g).to(DEV)
    q, kv = buf.chunk(2, dim=-1)
    geo = (w, col, roff, nh, ins[1], ins[0], ins[1])
    sk = torch.ops.s2attn_kernels
    y, lse = sk.forward_lse(kv, kv, q, *geo)
    dk, dv, dq = sk.backward_saved(kv, kv, q, dy, y, lse, *geo)
    kc = kv.contiguous()
    yc, lsec = sk.forward_lse(kc, kc.clone(), q.contiguous(), *geo)
    dkc, dvc, dqc = sk.backward_saved(kc, kc.clone(), q.contiguous(), dy, yc, lsec, *geo)
    assert torch.equal(y, yc)
    for name, g_, w_ in (("dk", dk, dkc), ("dv", dv, dvc), ("dq", dq, dqc)):
        assert torch.equal(g_, w_), f"{name}: k and v as one slice"
    torch.library.opcheck(sk.backward_saved, (kv, kv, q, dy, y, lse, *geo))


def test_fused_module_compiles_with_matching_gradient_strides():
    """A 64-channel module with 32-channel heads on a 96-longitude grid takes the fused q | k | v path; traced through AOT autograd
    the backward's outputs must have the strides its fake kernel announced."""
    m, x = _module_and_inputs(C=64, nh=2)
    gout = torch.randn(2, 64, 24, 96, device=DEV)

    def run(fn):
        a = x.detach().clone().requires_grad_(True)
        m.zero_grad(set_to_none=True)
        out = fn(a)
        out.backward(gout)
        return [out.detach(), a.grad] + [p.grad.clone() for p in m.parameters()]

    eager = run(m)
    compiled = run(torch.compile(m, backend="aot_eager", fullgraph=True))
    for i, (e, c) in enumerate(zip(eager, compiled)):
        assert_close(f"tensor {i}", c, e, rtol=1e-6, atol=1e-6)
