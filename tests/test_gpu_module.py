"""
Module- and operator-level behaviour on the GPU, modelled on the reference's tests/test_attention.py and
tests/test_attention_layout.py: module output and every gradient against a float64 CPU evaluation of the
same module, autocast dtypes, selective requires_grad, opcheck, layout conversions bitwise.
"""

import math

import pytest
import torch
import torch.nn.functional as F

from oracle import cpu_attention as oracle
from tests.util import SEED, assert_close

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _reference_module_forward(m, xq, xk, xv):
    """The module's forward (attention.py:456-571) in float64 on the CPU, with the dense masked softmax for the attention."""

    def nhwc(x):
        return x.permute(0, 2, 3, 1)

    p = {n: t.detach().double().cpu() for n, t in m.named_parameters()}
    for t in p.values():
        t.requires_grad_(True)
    q = F.linear(nhwc(xq), p["q_weights"].flatten(1), p.get("q_bias"))
    k = F.linear(nhwc(xk), p["k_weights"].flatten(1), p.get("k_bias"))
    v = F.linear(nhwc(xv), p["v_weights"].flatten(1), p.get("v_bias"))
    if "q_norm_weights" in p:
        eps = torch.finfo(torch.float32).eps  # F.rms_norm's default eps is the input dtype's; the module runs in fp32
        B, H, W, C = q.shape
        q = F.rms_norm(q.reshape(B, H, W, m.num_heads, -1), (C // m.num_heads,), weight=1 + p["q_norm_weights"], eps=eps).reshape(B, H, W, C)
        B, H, W, C = k.shape
        k = F.rms_norm(k.reshape(B, H, W, m.num_heads, -1), (C // m.num_heads,), weight=1 + p["k_norm_weights"], eps=eps).reshape(B, H, W, C)
    y = oracle.dense_attention_f64(k, v, q * m.scale, m.quad_weights.cpu(), m.psi_col_idx.cpu(), m.psi_roff_idx.cpu(), m.num_heads)
    out = F.linear(y, p["proj_weights"].flatten(1), p.get("proj_bias"))
    return out.permute(0, 3, 1, 2), p


MODULE_CASES = [
    # B, C, Cout, heads, in_shape, out_shape, grid_in, grid_out, qknorm   (rows of tests/test_attention.py:89-110,126-146)
    (4, 4, 4, 1, (6, 12), (6, 12), "equiangular", "equiangular", False),
    (4, 4, 4, 2, (6, 12), (6, 12), "equiangular", "equiangular", False),
    (4, 4, 8, 4, (6, 12), (6, 12), "equiangular", "equiangular", False),
    (4, 8, 4, 4, (6, 12), (6, 12), "equiangular", "equiangular", False),
    (4, 1, 4, 1, (2, 4), (2, 4), "equiangular", "equiangular", False),
    (4, 4, 4, 4, (6, 12), (6, 12), "legendre-gauss", "legendre-gauss", False),
    (4, 4, 4, 1, (6, 12), (6, 12), "lobatto", "lobatto", False),
    (4, 8, 4, 4, (12, 24), (6, 12), "equiangular", "equiangular", False),
    (4, 4, 4, 1, (12, 24), (6, 8), "equiangular", "equiangular", False),
    (4, 4, 4, 1, (12, 24), (3, 6), "equiangular", "equiangular", False),
    (4, 4, 4, 1, (9, 12), (5, 4), "equiangular", "equiangular", False),
    (4, 4, 4, 2, (6, 12), (6, 12), "equiangular", "equiangular", True),
    (4, 8, 4, 4, (12, 24), (6, 12), "equiangular", "equiangular", True),
    (2, 64, 64, 4, (24, 48), (24, 48), "equiangular", "equiangular", False),
    # heads of 32 channels on at least 64 longitudes: q | k | v projected by one fused GEMM and read in place
    (2, 64, 64, 2, (12, 96), (12, 96), "equiangular", "equiangular", False),
    (1, 32, 64, 1, (16, 128), (16, 128), "legendre-gauss", "legendre-gauss", False),
    (2, 64, 64, 2, (24, 192), (12, 96), "equiangular", "equiangular", False),
    # up-sampling rows (nlon_out a multiple of nlon_in): psi keyed by input latitude, default radius from the input grid
    (4, 4, 4, 1, (6, 12), (12, 24), "equiangular", "equiangular", False),
    (4, 8, 4, 4, (6, 12), (12, 24), "equiangular", "equiangular", False),
    (2, 4, 4, 2, (3, 6), (12, 24), "legendre-gauss", "equiangular", True),
    (2, 4, 8, 1, (5, 4), (9, 12), "equiangular", "equiangular", False),
]


@pytest.mark.parametrize("case", MODULE_CASES, ids=lambda c: f"C{c[1]}to{c[2]}h{c[3]}_{c[4][0]}x{c[4][1]}to{c[5][0]}x{c[5][1]}_{c[6][:3]}{'_qkn' if c[8] else ''}")
def test_module_output_and_all_gradients(case):
    from torch_harmonics_amd import NeighborhoodAttentionS2

    B, C, Cout, nh, ins, outs, gi, go, qkn = case
    torch.manual_seed(SEED)
    m = NeighborhoodAttentionS2(C, ins, outs, grid_in=gi, grid_out=go, num_heads=nh, use_qknorm=qkn, out_channels=Cout).to(DEV)
    if qkn:
        with torch.no_grad():
            m.q_norm_weights.uniform_(-0.3, 0.3)
            m.k_norm_weights.uniform_(-0.3, 0.3)
    self_attn = ins == outs
    xq = torch.randn(B, C, *outs)
    xk = xq if self_attn else torch.randn(B, C, *ins)
    xv = xq if self_attn else torch.randn(B, C, *ins)
    gout = torch.randn(B, Cout, *outs)

    dq_, dk_, dv_ = [t.clone().to(DEV).requires_grad_(True) for t in (xq, xk, xv)]
    out = m(dq_) if self_attn else m(dq_, dk_, dv_)
    out.backward(gout.to(DEV))

    rq, rk, rv = [t.clone().double().requires_grad_(True) for t in (xq, xk, xv)]
    ref, params = _reference_module_forward(m, rq, rq if self_attn else rk, rq if self_attn else rv)
    ref.backward(gout.double())

    tol = dict(rtol=1e-4, atol=2e-5)  # F.linear runs in fp32 on the GPU (rocBLAS) on both sides of the op
    assert_close("output", out, ref, **tol)
    assert_close("d query", dq_.grad, rq.grad, **tol)
    if not self_attn:
        assert_close("d key", dk_.grad, rk.grad, **tol)
        assert_close("d value", dv_.grad, rv.grad, **tol)
    for name, prm in m.named_parameters():
        assert_close("d " + name, prm.grad, params[name].grad, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("fused", [False, True], ids=["separate", "fused_kv"])
@pytest.mark.parametrize("frozen", [(), ("k_weights", "v_bias"), ("input",)], ids=["all", "frozen_params", "frozen_input"])
def test_shared_key_value_input_gradients(frozen, fused):
    """key is value (one tensor feeding two projections): its gradient is the sum of both projections' input gradients, with
    any subset of the parameters or the input itself frozen.  fused: heads of 32 channels on 64+ longitudes, where k | v come
    out of one GEMM as column blocks of one buffer."""
    from torch_harmonics_amd import NeighborhoodAttentionS2

    torch.manual_seed(SEED)
    C, ins, outs = (64, (12, 128), (6, 64)) if fused else (8, (12, 24), (6, 12))
    m = NeighborhoodAttentionS2(C, ins, outs, num_heads=2).to(DEV)
    for name in frozen:
        if name != "input":
            getattr(m, name).requires_grad_(False)
    xq, xkv, gout = torch.randn(2, C, *outs), torch.randn(2, C, *ins), torch.randn(2, C, *outs)
    dq_ = xq.clone().to(DEV).requires_grad_(True)
    dkv = xkv.clone().to(DEV).requires_grad_("input" not in frozen)
    m(dq_, dkv, dkv).backward(gout.to(DEV))
    rq, rkv = xq.double().requires_grad_(True), xkv.double().requires_grad_(True)
    ref, params = _reference_module_forward(m, rq, rkv, rkv)
    ref.backward(gout.double())
    tol = dict(rtol=1e-4, atol=2e-5)
    assert_close("d query", dq_.grad, rq.grad, **tol)
    if "input" in frozen:
        assert dkv.grad is None
    else:
        assert_close("d key+value", dkv.grad, rkv.grad, **tol)
    for name, prm in m.named_parameters():
        if name in frozen:
            assert prm.grad is None
        else:
            assert_close("d " + name, prm.grad, params[name].grad, rtol=1e-4, atol=1e-4)


def test_self_attention_backward_under_autocast():
    """Self-attention under bf16 autocast: the shared-input backward runs on bf16 gradients and hands back fp32 gradients."""
    from torch_harmonics_amd import NeighborhoodAttentionS2

    torch.manual_seed(SEED)
    m = NeighborhoodAttentionS2(16, (12, 24), (12, 24), num_heads=1).to(DEV)
    x = torch.randn(2, 16, 12, 24, device=DEV)
    grads = []
    for cast in (False, True):
        xi = x.clone().requires_grad_(True)
        m.zero_grad()
        with torch.autocast("cuda", dtype=torch.bfloat16, enabled=cast):
            out = m(xi)
        out.float().square().sum().backward()
        assert xi.grad.dtype == torch.float32 and m.k_weights.grad.dtype == torch.float32
        grads.append([xi.grad.clone(), m.q_weights.grad.clone(), m.k_weights.grad.clone(), m.v_weights.grad.clone()])
    for name, a, b in zip(("d input", "d q_weights", "d k_weights", "d v_weights"), grads[1], grads[0]):
        scale = b.abs().max().item()
        assert (a - b).abs().max().item() <= 6e-2 * scale, name


def _small_module(nh=2, dtype=torch.float32):
    from torch_harmonics_amd import NeighborhoodAttentionS2

    torch.manual_seed(SEED)
    return NeighborhoodAttentionS2(8, (12, 24), (6, 12), num_heads=nh).to(DEV)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_autocast_output_dtype_and_mixed_inputs(dtype):
    """Output dtype follows autocast; k, v, q of different dtypes are reconciled (tests/test_attention.py:288-390)."""
    from torch_harmonics_amd import ops

    m = _small_module()
    xq, xkv = torch.randn(2, 8, 6, 12, device=DEV), torch.randn(2, 8, 12, 24, device=DEV)
    with torch.autocast("cuda", dtype=dtype):
        out = m(xq, xkv, xkv)
    assert out.dtype == dtype
    ref = m(xq, xkv, xkv)
    tol = 2e-2 if dtype == torch.float16 else 5e-2
    assert_close("autocast output", out.float(), ref, rtol=tol, atol=tol)
    k = torch.randn(2, 12, 24, 8, device=DEV)
    v = torch.randn(2, 12, 24, 8, device=DEV, dtype=dtype)
    q = torch.randn(2, 6, 12, 8, device=DEV)
    with torch.autocast("cuda", dtype=dtype):
        y = ops._neighborhood_s2_attention_optimized(k, v, q, m.quad_weights, m.psi_col_idx, m.psi_roff_idx, 2, 24, 6, 12)
    assert y.dtype == dtype
    with pytest.raises(RuntimeError, match="must match q dtype"):
        ops._neighborhood_s2_attention_optimized(k, v, q, m.quad_weights, m.psi_col_idx, m.psi_roff_idx, 2, 24, 6, 12)


def test_selective_requires_grad():
    """A frozen input ends with .grad None while the others match the all-grads run (tests/test_attention.py:392-517)."""
    m = _small_module()
    xq, xk, xv = torch.randn(2, 8, 6, 12, device=DEV), torch.randn(2, 8, 12, 24, device=DEV), torch.randn(2, 8, 12, 24, device=DEV)
    full = [t.clone().requires_grad_(True) for t in (xq, xk, xv)]
    m(*full).sum().backward()
    for frozen in range(3):
        ins = [t.clone().requires_grad_(i != frozen) for i, t in enumerate((xq, xk, xv))]
        m.zero_grad()
        m(*ins).sum().backward()
        for i, t in enumerate(ins):
            if i == frozen:
                assert t.grad is None
            else:
                assert_close(f"grad {i} with input {frozen} frozen", t.grad, full[i].grad, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("nh", [1, 4])
def test_opcheck(nh):
    """Schema, fake-tensor and autograd registration checks (tests/test_attention.py:829-892)."""
    from torch_harmonics_amd import ops

    m = _small_module(nh)
    k = torch.randn(2, 12, 24, 8, device=DEV, requires_grad=True)
    v = torch.randn(2, 12, 24, 8, device=DEV, requires_grad=True)
    q = torch.randn(2, 6, 12, 8, device=DEV, requires_grad=True)
    args = (k, v, q, m.quad_weights, m.psi_col_idx, m.psi_roff_idx, nh, 24, 6, 12)
    torch.library.opcheck(ops._neighborhood_s2_attention_optimized, args)
    torch.library.opcheck(ops._neighborhood_s2_attention_saved, args)
    torch.library.opcheck(ops.forward_lse, tuple(a.detach() if isinstance(a, torch.Tensor) else a for a in args))
    torch.library.opcheck(ops.forward, tuple(a.detach() if isinstance(a, torch.Tensor) else a for a in args))
    x = torch.randn(2, 3, 4, 5, device=DEV, requires_grad=True)
    torch.library.opcheck(ops.permute_to_nhwc, (x,))
    torch.library.opcheck(ops.permute_to_nchw, (x,))


def test_wrong_shapes_raise_runtime_error():
    m = _small_module()
    with pytest.raises(RuntimeError):
        m(torch.randn(2, 8, 6, 13, device=DEV), torch.randn(2, 8, 12, 24, device=DEV), torch.randn(2, 8, 12, 24, device=DEV))
    with pytest.raises(RuntimeError):
        m(torch.randn(2, 8, 6, 12, device=DEV), torch.randn(2, 8, 11, 24, device=DEV), torch.randn(2, 8, 12, 24, device=DEV))


# the last two: more than 65535 tiles along H*W, and more than 65535 batch entries (a launch's y and z extents stop there)
LAYOUT_SHAPES = [(2, 3, 5, 7), (1, 1, 4, 4), (2, 4, 1, 1), (1, 256, 33, 70), (3, 65, 64, 65), (2, 8, 1, 9), (1, 1, 1, 1), (0, 4, 3, 2), (1, 2, 2100, 2048), (70000, 2, 3, 1)]


@pytest.mark.parametrize("shape", LAYOUT_SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16, torch.float64])
def test_layout_conversions_are_bitwise_permutes(shape, dtype):
    """tests/test_attention_layout.py:85-140: equals ATen permute bit for bit, round-trips, never aliases its input."""
    from torch_harmonics_amd import to_nchw, to_nhwc

    x = torch.randn(shape, device=DEV).to(dtype)
    y = to_nhwc(x)
    assert y.shape == (shape[0], shape[2], shape[3], shape[1]) and y.is_contiguous()
    assert torch.equal(y, x.permute(0, 2, 3, 1))
    assert y.numel() == 0 or y.data_ptr() != x.data_ptr()
    z = to_nchw(y)
    assert z.is_contiguous() and torch.equal(z, x)
    assert z.numel() == 0 or z.data_ptr() != y.data_ptr()


def test_layout_conversion_backward_and_noncontiguous_grad():
    from torch_harmonics_amd import to_nchw, to_nhwc

    x = torch.randn(2, 5, 6, 7, device=DEV, requires_grad=True)
    g = torch.randn(2, 7, 6, 5, device=DEV).permute(0, 2, 1, 3)  # non-contiguous (2, 6, 7, 5)
    to_nhwc(x).backward(g)
    assert torch.equal(x.grad, g.permute(0, 3, 1, 2))
    x2 = torch.randn(2, 6, 7, 5, device=DEV, requires_grad=True)
    to_nchw(x2).sum().backward()
    assert torch.equal(x2.grad, torch.ones_like(x2))
    with torch.autocast("cuda", dtype=torch.bfloat16):
        assert to_nhwc(x.detach()).dtype == torch.float32  # a pure element move is not an autocast op


def test_plan_cache_follows_tensor_identity_and_version():
    from torch_harmonics_amd import ops
    from torch_harmonics_amd.plan import get_plan

    m = _small_module()
    p1 = get_plan(m.psi_col_idx, m.psi_roff_idx, 12, 24, 6, 12)
    assert get_plan(m.psi_col_idx, m.psi_roff_idx, 12, 24, 6, 12) is p1
    k, v, q = torch.randn(1, 12, 24, 8, device=DEV), torch.randn(1, 12, 24, 8, device=DEV), torch.randn(1, 6, 12, 8, device=DEV)
    y1 = ops.forward(k, v, q, m.quad_weights, m.psi_col_idx, m.psi_roff_idx, 2, 24, 6, 12)
    # overwrite every row with copies of its first entry, in place: same storage, new version counter -> the plan is rebuilt,
    # and a softmax over identical neighbors returns that neighbor's v
    ro = m.psi_roff_idx.cpu()
    first = m.psi_col_idx.cpu()[ro[:-1]]
    m.psi_col_idx.copy_(first.repeat_interleave(ro[1:] - ro[:-1]).to(DEV))
    p2 = get_plan(m.psi_col_idx, m.psi_roff_idx, 12, 24, 6, 12)
    assert p2 is not p1
    y2 = ops.forward(k, v, q, m.quad_weights, m.psi_col_idx, m.psi_roff_idx, 2, 24, 6, 12)
    hi, wi = (first // 24), (first % 24)
    for wo in range(12):
        assert_close("single neighbor", y2[:, :, wo], v[:, hi.to(DEV), ((wi + 2 * wo) % 24).to(DEV)], rtol=1e-6, atol=1e-6)
    assert not torch.allclose(y1, y2)


def test_forward_and_backward_replay_from_a_hip_graph():
    """The library allocates nothing, never synchronises and launches on the stream it is handed, so a forward + backward can be
    captured into a HIP graph once the plan is cached; every replay (eager work and synchronisations in between) must reproduce
    the eager result for the inputs then in the static buffers."""
    from torch_harmonics_amd import ops

    m = _small_module()
    geo = (m.quad_weights, m.psi_col_idx, m.psi_roff_idx, 2, 24, 6, 12)
    gen = torch.Generator(device=DEV).manual_seed(SEED)
    k, v = [torch.randn(2, 12, 24, 8, device=DEV, generator=gen) for _ in range(2)]
    q, dy = [torch.randn(2, 6, 12, 8, device=DEV, generator=gen) for _ in range(2)]

    def step():
        y, lse = ops.forward_lse(k, v, q, *geo)
        return (y,) + tuple(ops.backward_saved(k, v, q, dy, y, lse, *geo))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):  # warm-up: builds and caches the plan (one host round trip), primes the allocator
            step()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step()
    for it in range(3):
        for t in (k, v, q, dy):
            t.copy_(torch.randn(t.shape, device=DEV, generator=gen))
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs]
        want = step()
        torch.cuda.synchronize()
        for name, g_, w_ in zip(("y", "dk", "dv", "dq"), got, want):
            assert torch.equal(g_, w_), f"replay {it}: {name} differs from the eager result"


def test_module_traces_under_torch_compile():
    """The operators carry fake (meta) kernels and autograd formulas registered through torch.library, so the module traces as one
    graph (fullgraph) through AOT autograd; forward and gradients must equal the eager ones (tests/test_attention_layout.py:170-200
    does the same for the layout ops)."""
    m = _small_module()
    xq = torch.randn(2, 8, 6, 12, device=DEV)
    xkv = torch.randn(2, 8, 12, 24, device=DEV)
    gout = torch.randn(2, 8, 6, 12, device=DEV)

    def run(fn):
        a, b = xq.clone().requires_grad_(True), xkv.clone().requires_grad_(True)
        m.zero_grad(set_to_none=True)
        out = fn(a, b, b)
        out.backward(gout)
        return [out.detach(), a.grad, b.grad] + [p.grad.clone() for p in m.parameters()]

    eager = run(m)
    compiled = run(torch.compile(m, backend="aot_eager", fullgraph=True))
    for i, (e, c) in enumerate(zip(eager, compiled)):
        assert_close(f"tensor {i}", c, e, rtol=1e-6, atol=1e-6)
