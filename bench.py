#!/usr/bin/env python
"""
Benchmark of the spherical neighborhood-attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config cfg3] [--no-cpu-baseline]

One step = one forward plus one backward of the attention op (the C ABI behind
torch_harmonics_amd.ops) on the ERA5-shaped configuration: equiangular 721x1440 grid in and
out, batch 1, 256 channels in 8 heads, fp32, theta_cutoff = 3 latitude spacings.  Inputs are
synthetic (low-degree spherical-harmonic fields plus noise, projected by randomly initialised
q/k/v weights) and resident in HBM before the timed region.  Prints ONE JSON line.

Reported alongside the throughput:
  roofline      the slowest kernel of the step, timed with events recorded on the launch stream
                around every launch of it inside the timed region
  cpu_baseline  the reference's own CPU operators (oracle/_ref, its release flags, OpenMP) and the C restatement of them (oracle/)
                on a bounded sample of the same workload, on this machine's host cores
  other_configs op-level forward and backward times of the other four benchmark configurations
  published_shapes  the reference's own published benchmark shapes (module level, forward and backward timed separately as there)
  reference_signature_ms_per_step  the same step through the operators with the reference's exact signatures
"""

import argparse
import ctypes
import json
import math
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E
FP32_MATRIX_PEAK_TFLOPS = 157.3  # dense fp32 MFMA: the unit the long-run (polar) part of the path runs on
BF16_MATRIX_PEAK_TFLOPS = 2500.0  # dense bf16 MFMA
FP32_VALU_PEAK_TFLOPS = 78.6  # 157.3 TFLOP/s vector fp32 is quoted with packed FMA; these kernels are built without packed fp32

CONFIGS = {
    "cfg1": dict(in_shape=(32, 64), out_shape=(32, 64), grid_in="equiangular", grid_out="equiangular", B=1, C=16, nh=1, theta_cutoff=None),
    "cfg2": dict(in_shape=(128, 256), out_shape=(128, 256), grid_in="equiangular", grid_out="equiangular", B=4, C=64, nh=4, theta_cutoff=4 * math.pi / 127),
    "cfg3": dict(in_shape=(721, 1440), out_shape=(721, 1440), grid_in="equiangular", grid_out="equiangular", B=1, C=256, nh=8, theta_cutoff=3 * math.pi / 720),
    "cfg4": dict(in_shape=(721, 1440), out_shape=(360, 720), grid_in="equiangular", grid_out="legendre-gauss", B=2, C=128, nh=4, theta_cutoff=2 * math.pi / 359),
    "cfg5": dict(
        in_shape=(361, 720), out_shape=(361, 720), grid_in="legendre-gauss", grid_out="legendre-gauss", B=4, C=1024, nh=16, theta_cutoff=8 * math.pi / 360, dtype="bf16"
    ),
    # not one of the five named configurations: fp32 with 64-channel heads (the head width of the reference's published
    # benchmark shapes, benchmarks/attention.py:71-112) at a size where throughput, not launch overhead, sets the time
    "d64": dict(in_shape=(361, 720), out_shape=(361, 720), grid_in="equiangular", grid_out="equiangular", B=2, C=512, nh=8, theta_cutoff=0.03),
}


def smooth_field(B, C, nlat, nlon, grid, gen, device, lmax=8, noise=0.25):
    """(B, C, nlat, nlon) fp32: per channel a random combination of real spherical harmonics up to degree lmax
    (coefficients N(0,1)/(l+1)) plus noise*N(0,1), standardised to unit variance per channel."""
    from scipy.special import lpmv

    from torch_harmonics_amd.quadrature import precompute_latitudes

    theta, _ = precompute_latitudes(nlat, grid)
    x = np.cos(theta.numpy())
    lam = 2 * np.pi * np.arange(nlon) / nlon
    basis, damp = [], []
    for l in range(lmax + 1):
        for m in range(l + 1):
            norm = math.sqrt((2 * l + 1) / (4 * math.pi) * math.factorial(l - m) / math.factorial(l + m))
            leg = norm * lpmv(m, l, x)
            basis.append(np.outer(leg, np.cos(m * lam)))
            damp.append(1.0 / (l + 1))
            if m > 0:
                basis.append(np.outer(leg, np.sin(m * lam)))
                damp.append(1.0 / (l + 1))
    basis = torch.tensor(np.stack(basis), dtype=torch.float32, device=device).reshape(len(damp), -1)
    damp = torch.tensor(damp, dtype=torch.float32)
    coef = (torch.randn(B * C, len(damp), generator=gen) * damp).to(device)
    f = (coef @ basis).reshape(B, C, nlat, nlon)
    f = f + noise * torch.randn(B, C, nlat, nlon, generator=gen).to(device)
    f = (f - f.mean(dim=(2, 3), keepdim=True)) / f.std(dim=(2, 3), keepdim=True)
    return f.contiguous()


def make_workload(cfg, device, seed=333):
    """Module with seeded random weights, its NCHW input, and the op-level tensors k, v, q (scaled), dy in NHWC."""
    from torch_harmonics_amd import NeighborhoodAttentionS2, to_nhwc

    torch.manual_seed(seed)
    mod = NeighborhoodAttentionS2(
        cfg["C"], cfg["in_shape"], cfg["out_shape"], grid_in=cfg["grid_in"], grid_out=cfg["grid_out"], num_heads=cfg["nh"], theta_cutoff=cfg["theta_cutoff"]
    ).to(device)
    gen = torch.Generator().manual_seed(seed)
    x_in = smooth_field(cfg["B"], cfg["C"], *cfg["in_shape"], cfg["grid_in"], gen, device)
    same = cfg["in_shape"] == cfg["out_shape"] and cfg["grid_in"] == cfg["grid_out"]
    x_out = x_in if same else smooth_field(cfg["B"], cfg["C"], *cfg["out_shape"], cfg["grid_out"], gen, device)
    with torch.no_grad():
        xi, xo = to_nhwc(x_in), to_nhwc(x_out)
        k = torch.nn.functional.linear(xi, mod.k_weights.view(mod.k_channels, -1), mod.k_bias).contiguous()
        v = torch.nn.functional.linear(xi, mod.v_weights.view(mod.out_channels, -1), mod.v_bias).contiguous()
        q = (torch.nn.functional.linear(xo, mod.q_weights.view(mod.k_channels, -1), mod.q_bias) * mod.scale).contiguous()
        dy = torch.randn(q.shape[:3] + (v.shape[3],), generator=gen).to(device)
    return mod, x_in, x_out, k, v, q, dy


def time_other_config(name, device, steps=3, cpu=False):
    """Op-level forward + backward (ms) of another benchmark configuration on N(0,1)-type inputs in its own storage
    dtype (cfg5: 0.5 * N(0,1) in bf16), psi and quadrature weights from the package's geometry code."""
    from torch_harmonics_amd import ops
    from torch_harmonics_amd.neighborhood import precompute_neighborhood_s2
    from torch_harmonics_amd.quadrature import precompute_latitudes

    cfg = CONFIGS[name]
    (Hi, Wi), (Ho, Wo) = cfg["in_shape"], cfg["out_shape"]
    nh, B, d = cfg["nh"], cfg["B"], cfg["C"] // cfg["nh"]
    dt = torch.bfloat16 if cfg.get("dtype") == "bf16" else torch.float32
    col, roff, _ = precompute_neighborhood_s2(cfg["in_shape"], cfg["out_shape"], cfg["grid_in"], cfg["grid_out"], cfg["theta_cutoff"])
    w = (2.0 * torch.pi * precompute_latitudes(Hi, cfg["grid_in"])[1].float() / Wi).contiguous().to(device)
    col, roff = col.to(device), roff.to(device)
    gen = torch.Generator(device=device).manual_seed(333)
    scale = 0.5 if dt == torch.bfloat16 else 1.0
    k = (scale * torch.randn(B, Hi, Wi, nh * d, device=device, generator=gen)).to(dt)
    v = (scale * torch.randn(B, Hi, Wi, nh * d, device=device, generator=gen)).to(dt)
    q = (scale * torch.randn(B, Ho, Wo, nh * d, device=device, generator=gen) / math.sqrt(d)).to(dt)
    dy = (scale * torch.randn(B, Ho, Wo, nh * d, device=device, generator=gen)).to(dt)
    geo = (w, col, roff, nh, Wi, Ho, Wo)
    pairs = B * nh * Wo * col.numel()

    def run(f):
        f()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            f()
        torch.cuda.synchronize()
        return 1e3 * (time.perf_counter() - t0) / steps

    y, lse = ops.forward_lse(k, v, q, *geo)
    t_fwd = run(lambda: ops.forward_lse(k, v, q, *geo))
    t_bwd = run(lambda: ops.backward_saved(k, v, q, dy, y, lse, *geo))
    res = {"fwd_ms": t_fwd, "bwd_ms": t_bwd, "pairs": pairs, "pairs_per_s": pairs / ((t_fwd + t_bwd) * 1e-3), "dtype": "bf16" if dt == torch.bfloat16 else "f32"}
    if pairs < 2e8:
        # launch-bound sizes: the same forward + backward captured once into a HIP graph and replayed (the library allocates
        # nothing and never synchronises, so it captures as it is)
        def both():
            y2, l2 = ops.forward_lse(k, v, q, *geo)
            return ops.backward_saved(k, v, q, dy, y2, l2, *geo)

        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            both()
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            both()
        res["graph_fwd_bwd_ms"] = run(graph.replay)
    if cpu and dt == torch.float32:
        # the whole configuration on the CPU port of the reference algorithm (its backward scratch is 2*B*nh*Ho*Wo*max_row floats)
        from oracle import cpu_attention as oracle

        hk, hv, hq, hg, hw, hc, hr = [t.cpu() for t in (k, v, q, dy, w, col, roff)]
        res["cpu_port_fwd_ms"] = 1e3 * best_time(timed_calls(lambda: oracle.forward_f32(hk, hv, hq, hw, hc, hr, nh, fast=True), CPU_REPEAT))
        res["cpu_port_bwd_ms"] = 1e3 * best_time(timed_calls(lambda: oracle.backward_f32(hk, hv, hq, hg, hw, hc, hr, nh, fast=True), CPU_REPEAT))
    return res


def time_ring_steps(device, nchunk=4, reps=2):
    """The ring-step operators on one device (all longitude chunks of K/V folded one after the other, ms for the whole fold):
    gather direction on cfg3's tensors (B = 1, 8 heads of 32 channels folded into the batch, its grid and cutoff), up-sampling
    361x720 -> 721x1440 with the same batch; fp32, and the gather direction once more with k, v, q, dy stored in bf16."""
    from torch_harmonics_amd import ops
    from torch_harmonics_amd.neighborhood import precompute_neighborhood_s2
    from torch_harmonics_amd.quadrature import precompute_latitudes

    BB, d = CONFIGS["cfg3"]["B"] * CONFIGS["cfg3"]["nh"], CONFIGS["cfg3"]["C"] // CONFIGS["cfg3"]["nh"]
    gen = torch.Generator(device=device).manual_seed(333)
    res = {}
    cases = (
        ("gather", (721, 1440), (721, 1440), CONFIGS["cfg3"]["theta_cutoff"], torch.float32),
        ("upsample", (361, 720), (721, 1440), 0.03, torch.float32),
        ("gather_bf16", (721, 1440), (721, 1440), CONFIGS["cfg3"]["theta_cutoff"], torch.bfloat16),
    )
    for name, ins, outs, theta, dtype in cases:
        up = name == "upsample"
        (Hi, Wi), (Ho, Wo) = ins, outs
        col, roff, _ = precompute_neighborhood_s2(outs if up else ins, ins if up else outs, "equiangular", "equiangular", theta)
        w = (2.0 * torch.pi * precompute_latitudes(Hi, "equiangular")[1].float() / Wi).contiguous().to(device)
        row_idx = torch.argsort(roff[1:] - roff[:-1], descending=True, stable=True).to(torch.int32)
        split = ops.split_csr_rows(row_idx, roff, Ho)
        pairs = BB * (Wi if up else Wo) * col.numel()
        col, roff, row_idx = col.to(device), roff.to(device), row_idx.to(device)
        k = torch.randn(BB, Hi, Wi, d, device=device, generator=gen).to(dtype)
        v = torch.randn(BB, Hi, Wi, d, device=device, generator=gen).to(dtype)
        q = (torch.randn(BB, Ho, Wo, d, device=device, generator=gen) / math.sqrt(d)).to(dtype)
        dy = torch.randn(BB, Ho, Wo, d, device=device, generator=gen).to(dtype)
        cw = Wi // nchunk
        parts = [(k[:, :, i * cw : (i + 1) * cw].contiguous(), v[:, :, i * cw : (i + 1) * cw].contiguous(), i * cw) for i in range(nchunk)]
        z = lambda *s: torch.zeros(*s, device=device)  # noqa: E731
        y_acc, asum, qmax = z(BB, Ho, Wo, d), z(BB, Ho, Wo), z(BB, Ho, Wo)
        integ, ak, akvw, as2, qm2 = z(BB, Ho, Wo), z(BB, Ho, Wo, d), z(BB, Ho, Wo, d), z(BB, Ho, Wo), z(BB, Ho, Wo)
        tail = (lambda lo: (Wi, Wo, Wo // Wi, lo, 0, Ho, Wo)) if up else (lambda lo: (Wi, Wi // Wo, lo, 0, Ho, Wo, *split))

        def fwd():
            y_acc.zero_(), asum.zero_(), qmax.fill_(float("-inf"))
            for kc, vc, lo in parts:
                if up:
                    ops.forward_ring_step_upsample(kc, vc, q, y_acc, asum, qmax, w, col, roff, *tail(lo))
                else:
                    ops.forward_ring_step(kc, vc, q, y_acc, asum, qmax, w, col, roff, row_idx, *tail(lo))

        def pass1():
            integ.zero_(), ak.zero_(), akvw.zero_(), as2.zero_(), qm2.fill_(float("-inf"))
            for kc, vc, lo in parts:
                if up:
                    ops.backward_ring_step_upsample_pass1(kc, vc, q, dy, qmax, integ, ak, akvw, w, col, roff, *tail(lo))
                else:
                    ops.backward_ring_step_pass1(kc, vc, q, dy, as2, qm2, integ, ak, akvw, w, col, roff, row_idx, *tail(lo))

        grads = [(torch.zeros_like(kc, dtype=torch.float32), torch.zeros_like(vc, dtype=torch.float32)) for kc, vc, _ in parts]

        def pass2():
            for (kc, vc, lo), (dkc, dvc) in zip(parts, grads):
                if up:
                    ops.backward_ring_step_upsample_pass2(kc, vc, q, dy, asum, qmax, inorm, dkc, dvc, w, col, roff, *tail(lo))
                else:
                    ops.backward_ring_step_pass2(kc, vc, q, dy, asum, qmax, inorm, dkc, dvc, w, col, roff, row_idx, *tail(lo))

        def run(f):
            f()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(reps):
                f()
            torch.cuda.synchronize()
            return 1e3 * (time.perf_counter() - t0) / reps

        t_f, t_1 = run(fwd), run(pass1)
        inorm = (integ / asum).contiguous()
        t_2 = run(pass2)
        # the same attention in one piece (psi keyed the same way), for scale
        geo = (w, col, roff, 1, Wi, Ho, Wo)
        y, lse = ops.forward_lse(k, v, q, *geo)
        t_one = run(lambda: ops.forward_lse(k, v, q, *geo))
        err = ((y_acc / asum[..., None]) - y.float()).abs().max().item()
        res[name] = {
            "grid": f"{Hi}x{Wi} -> {Ho}x{Wo}", "storage": str(dtype).replace("torch.", ""), "theta_cutoff": theta, "pairs": pairs, "chunks": nchunk, "forward_ms": t_f, "pass1_ms": t_1, "pass2_ms": t_2,
            "single_device_forward_ms": t_one, "max_abs_diff_to_single_device_y": err,
        }  # fmt: skip
        del k, v, q, dy, parts, grads, y_acc, ak, akvw, y
    return res


# The reference's own published benchmark shapes (benchmarks/reference_results.csv:11-84; benchmarks/attention.py:71-112): B = 1, 64 channels, one head,
# equiangular grids; published there for H100 / GB200 / GB300 only, so the figures beside them are context, not a baseline for this hardware.
PUBLISHED_SHAPES = [
    # (in_shape, out_shape, theta_cutoff, published H100 fp32 fwd ms, bwd ms, csv line)
    ((180, 360), (180, 360), 0.017, 0.550, 1.115, 12),
    ((180, 360), (180, 360), 0.03, 0.801, 1.781, 15),
    ((360, 720), (360, 720), 0.017, 3.150, 7.394, 18),
    ((360, 720), (360, 720), 0.03, 7.764, 19.431, 21),
    ((360, 720), (180, 360), 0.017, 1.689, 3.499, 24),
    ((360, 720), (180, 360), 0.03, 2.705, 6.049, 27),
    ((180, 360), (360, 720), 0.03, 10.987, 19.280, 33),
]


def time_published_shapes(device, warmup=3, iters=20):
    """Module-level forward and backward of the reference's published shapes, timed separately with device events around each
    (3 warm-up + 20 iterations, upstream gradient of ones, as benchmarks/attention.py:71-112 and benchmarks/bench.py:268-323 do),
    plus the op alone (forward_lse / backward_saved on the projected tensors) for the same shapes."""
    from torch_harmonics_amd import NeighborhoodAttentionS2, ops

    res = []
    for ins, outs, tc, h_f, h_b, line in PUBLISHED_SHAPES:
        torch.manual_seed(333)
        m = NeighborhoodAttentionS2(64, ins, outs, num_heads=1, theta_cutoff=tc).to(device)
        same = ins == outs
        xq = torch.randn(1, 64, *outs, device=device, requires_grad=True)
        xk = xq if same else torch.randn(1, 64, *ins, device=device, requires_grad=True)

        def fwd():
            return m(xq) if same else m(xq, xk, xk)

        for _ in range(warmup):
            o = fwd()
            o.backward(torch.ones_like(o))
        torch.cuda.synchronize()
        tf = tb = 0.0
        for _ in range(iters):
            m.zero_grad(set_to_none=True)
            xq.grad = None
            if xk is not xq:
                xk.grad = None
            e = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
            e[0].record()
            o = fwd()
            e[1].record()
            o.backward(torch.ones_like(o))
            e[2].record()
            torch.cuda.synchronize()
            tf += e[0].elapsed_time(e[1])
            tb += e[1].elapsed_time(e[2])
        # the op alone on N(0,1) tensors of the projected shapes
        (Hi, Wi), (Ho, Wo) = ins, outs
        g = torch.Generator(device=device).manual_seed(333)
        k = torch.randn(1, Hi, Wi, 64, device=device, generator=g)
        v = torch.randn(1, Hi, Wi, 64, device=device, generator=g)
        q = torch.randn(1, Ho, Wo, 64, device=device, generator=g) / 8.0
        dy = torch.ones(1, Ho, Wo, 64, device=device)
        geo = (m.quad_weights, m.psi_col_idx, m.psi_roff_idx, 1, Wi, Ho, Wo)
        y, lse = ops.forward_lse(k, v, q, *geo)
        ops.backward_saved(k, v, q, dy, y, lse, *geo)
        torch.cuda.synchronize()
        of = ob = 0.0
        for _ in range(iters):
            e = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
            e[0].record()
            y, lse = ops.forward_lse(k, v, q, *geo)
            e[1].record()
            ops.backward_saved(k, v, q, dy, y, lse, *geo)
            e[2].record()
            torch.cuda.synchronize()
            of += e[0].elapsed_time(e[1])
            ob += e[1].elapsed_time(e[2])
        nnz = m.psi_col_idx.numel()
        pairs = (Wi if m.upsample else Wo) * nnz
        res.append({
            "shape": f"{Hi}x{Wi} -> {Ho}x{Wo}", "theta_cutoff": tc, "nnz": nnz, "pairs": pairs,
            "module_fwd_ms": tf / iters, "module_bwd_ms": tb / iters, "op_fwd_ms": of / iters, "op_bwd_ms": ob / iters,
            "published_h100_fwd_ms": h_f, "published_h100_bwd_ms": h_b, "published_source": f"benchmarks/reference_results.csv:{line}",
        })  # fmt: skip
        del m, xq, xk, k, v, q, dy, y, lse
    return res


CPU_REPEAT = 4  # 1 warm-up + 3 timed calls for the CPU legs that take under about 2 s


def best_time(seconds):
    """Minimum over the timed calls: the first call is a warm-up when there is more than one."""
    return min(seconds[1:]) if len(seconds) > 1 else seconds[0]


def timed_calls(f, repeat):
    out = []
    for _ in range(repeat):
        t0 = time.perf_counter()
        f()
        out.append(time.perf_counter() - t0)
    return out


def cpu_sample(cfg, col, ro):
    """The bounded sample of a workload that the CPU legs time: the first four heads and every 6th output latitude (both pole
    rows included, so the reference backward's per-neighbor scratch is sized by the longest row, as in the full problem)."""
    nh_s = min(4, cfg["nh"])
    Ho, Wo = cfg["out_shape"]
    stride = 6 if Ho >= 120 else 1
    rows = torch.arange(0, Ho, stride)
    if rows[-1] != Ho - 1:
        rows = torch.cat([rows, torch.tensor([Ho - 1])])
    lens = (ro[1:] - ro[:-1])[rows]
    ro_s = torch.zeros(len(rows) + 1, dtype=torch.int64)
    ro_s[1:] = torch.cumsum(lens, 0)
    col_s = torch.cat([col[ro[r] : ro[r + 1]] for r in rows.tolist()])
    pairs = cfg["B"] * nh_s * Wo * int(lens.sum())
    scratch_gb = 2 * cfg["B"] * nh_s * len(rows) * Wo * int(lens.max()) * 4 / 1e9
    full_pairs = cfg["B"] * cfg["nh"] * Wo * int(col.numel())
    return dict(nh=nh_s, rows=rows, stride=stride, col=col_s, ro=ro_s, pairs=pairs, scratch_gb=scratch_gb, full_pairs=full_pairs, full=full_pairs <= 4e9)


def reference_cpu_times(config_name, others):
    """
    The reference's OWN CPU operators (oracle/_ref/attention_ref.so: its CPU sources compiled with its release flags) on the
    sample of `config_name`, on its full forward where that is feasible, and on the configurations of `others` in full.
    They run in a child process, and this function is called before this process touches the GPU (a process that holds a
    GPU context starts no other program).  The child makes its own N(0,1) tensors of the workload's shapes (the algorithm
    has no data-dependent control flow), on psi from the oracle's geometry, which the tests hold element-equal to the
    module's.  Returns None where the library has not been built.
    """
    from oracle import geometry as ogeo
    from oracle import reference_ops as reference

    if not reference.available():
        return None
    cores = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    jobs, keys = [], []

    def add(key, cfg, col, ro, nh, nlat_out, bwd, slow_bwd=False):
        (Hi, Wi), (_, Wo) = cfg["in_shape"], cfg["out_shape"]
        ck = cfg["C"] // cfg["nh"]
        w = ogeo.attention_quad_weights(Hi, Wi, cfg["grid_in"])
        kk = {"randn": [cfg["B"], Hi, Wi, nh * ck], "seed": 1, "scale": 1.0}
        vv = {"randn": [cfg["B"], Hi, Wi, nh * ck], "seed": 2, "scale": 1.0}
        qq = {"randn": [cfg["B"], nlat_out, Wo, nh * ck], "seed": 3, "scale": 1.0 / math.sqrt(ck)}
        gg = {"randn": [cfg["B"], nlat_out, Wo, nh * ck], "seed": 4, "scale": 1.0}
        # calls expected to take under about 2 s are repeated: 1 warm-up + 3 timed, the minimum is reported; the long ones run once
        jobs.append(dict(op="forward", args=[kk, vv, qq, w, col, ro, nh, Wi, nlat_out, Wo], discard=True, repeat=CPU_REPEAT))
        keys.append((key, "fwd_ms"))
        if bwd:
            jobs.append(dict(op="backward", args=[dict(kk), dict(vv), dict(qq), gg, w, col, ro, nh, Wi, nlat_out, Wo], discard=True, repeat=1 if slow_bwd else CPU_REPEAT))
            keys.append((key, "bwd_ms"))

    cfg = CONFIGS[config_name]
    col, ro = ogeo.neighborhood_csr(cfg["in_shape"], cfg["out_shape"], cfg["grid_in"], cfg["grid_out"], cfg["theta_cutoff"])
    smp = cpu_sample(cfg, col, ro)
    add("sample", cfg, smp["col"], smp["ro"], smp["nh"], len(smp["rows"]), True, slow_bwd=smp["pairs"] > 5e7)
    if smp["full"]:
        add("full", cfg, col, ro, cfg["nh"], cfg["out_shape"][0], False)
    for name in others:
        c = CONFIGS[name]
        oc, orr = ogeo.neighborhood_csr(c["in_shape"], c["out_shape"], c["grid_in"], c["grid_out"], c["theta_cutoff"])
        add(name, c, oc, orr, c["nh"], c["out_shape"][0], True)
    res = reference.run(jobs, threads=cores)
    out = {}
    for (key, what), r in zip(keys, res):
        out.setdefault(key, {})[what] = 1e3 * best_time(r["seconds"])
        out[key][what.replace("_ms", "_runs")] = len(r["seconds"])
    return out


def cpu_baseline(cfg, mod, k, v, q, dy, ref_times=None):
    """
    Times the reference's CPU algorithm forward + backward on a sample of the workload (cpu_sample).  Throughput is
    neighbor pairs of the sample per second.  Two builds: the reference's OWN CPU operators (`ref_times`, from
    reference_cpu_times; `kind` "reference") and the C restatement of the same algorithm (oracle/s2attn_oracle.c, the
    same flags, on the workload's own tensors; `port_*`).  Without the reference build the restatement is the baseline
    (`kind` "port").
    """
    from oracle import cpu_attention as oracle

    ck, cv = mod.k_channels // cfg["nh"], mod.out_channels // cfg["nh"]
    Ho, Wo = cfg["out_shape"]
    col, ro = mod.psi_col_idx.cpu(), mod.psi_roff_idx.cpu()
    smp = cpu_sample(cfg, col, ro)
    nh_s, rows, col_s, ro_s, pairs = smp["nh"], smp["rows"], smp["col"], smp["ro"], smp["pairs"]
    ks = k[..., : nh_s * ck].float().cpu().contiguous()
    vs = v[..., : nh_s * cv].float().cpu().contiguous()
    qs = q[:, rows][..., : nh_s * ck].float().cpu().contiguous()
    gs = dy[:, rows][..., : nh_s * cv].float().cpu().contiguous()
    w = mod.quad_weights.float().cpu()
    cores = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    slow_bwd = pairs > 5e7
    t_f = timed_calls(lambda: oracle.forward_f32(ks, vs, qs, w, col_s, ro_s, nh_s, fast=True), CPU_REPEAT)
    t_b = timed_calls(lambda: oracle.backward_f32(ks, vs, qs, gs, w, col_s, ro_s, nh_s, fast=True), 1 if slow_bwd else CPU_REPEAT)
    port = {"fwd_ms": 1e3 * best_time(t_f), "bwd_ms": 1e3 * best_time(t_b)}
    # The forward alone has no scratch and is feasible in full: all heads, all latitudes of the workload (the reference backward
    # would need 2 * B * heads * nlat_out * nlon_out * max_row_len floats, 383 GB at 721x1440 with 8 heads).
    if smp["full"]:
        kf, vf, qf = k.float().cpu().contiguous(), v.float().cpu().contiguous(), q.float().cpu().contiguous()
        port["full_forward_ms"] = 1e3 * best_time(timed_calls(lambda: oracle.forward_f32(kf, vf, qf, w, col, ro, cfg["nh"], fast=True), CPU_REPEAT))

    timed, kind = port, "port"
    if ref_times and "sample" in ref_times:
        timed, kind = dict(ref_times["sample"]), "reference"
        if smp["full"] and "full" in ref_times:
            timed["full_forward_ms"] = ref_times["full"]["fwd_ms"]
    out = {
        "value": pairs / (1e-3 * (timed["fwd_ms"] + timed["bwd_ms"])),
        "unit": "pairs/s",
        "cores": cores,
        "kind": kind,
        "sample": f"{nh_s} of {cfg['nh']} heads x {len(rows)} of {Ho} output latitudes (every {smp['stride']}th, both poles) = {pairs} pairs; "
        f"fwd {timed['fwd_ms']:.0f} ms + bwd {timed['bwd_ms']:.0f} ms; reference bwd scratch {smp['scratch_gb']:.1f} GB"
        + f"; calls under about 2 s: 1 warm-up + {CPU_REPEAT - 1} timed, minimum; the backward of a large sample: one call"
        + ("; the reference's own CPU operators in a child process, on the child's own N(0,1) tensors of these shapes (not the workload's smooth fields)" if kind == "reference" else ""),
        "fwd_ms": timed["fwd_ms"],
        "bwd_ms": timed["bwd_ms"],
    }
    if "full_forward_ms" in timed:
        out["full_forward_ms"] = timed["full_forward_ms"]
        out["full_forward_pairs_per_s"] = smp["full_pairs"] / (1e-3 * timed["full_forward_ms"])
    if kind == "reference":  # the restatement beside it: same algorithm, same flags, the workload's own tensors
        out["port_value"] = pairs / (1e-3 * (port["fwd_ms"] + port["bwd_ms"]))
        out["port_fwd_ms"], out["port_bwd_ms"] = port["fwd_ms"], port["bwd_ms"]
        if "full_forward_ms" in port:
            out["port_full_forward_ms"] = port["full_forward_ms"]
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", default="cfg3", choices=sorted(CONFIGS))
    ap.add_argument("--no-other-configs", action="store_true", help="skip the op-level timings of the other benchmark configurations and of the ring-step operators")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-module", action="store_true", help="skip the module-level (projections + permutes) timing")
    ap.add_argument("--ring-only", action="store_true", help="time the ring-step operators and nothing else (for profiling)")
    ap.add_argument("--no-reference-route", action="store_true", help="skip the timing of the operators with the reference's exact signatures (for profiling: they launch the same kernels)")
    args = ap.parse_args()

    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    # the reference's own CPU build is timed first, in a child process, while this process has not touched the GPU yet
    ref_times = None
    if not args.no_cpu_baseline and not args.ring_only and torch.cuda.device_count() > 0:
        ref_times = reference_cpu_times(args.config, [] if args.no_other_configs else [n for n in ("cfg1", "cfg2") if n != args.config])
    if not torch.cuda.is_available():
        print("bench.py needs a ROCm GPU", file=sys.stderr)
        sys.exit(2)

    from torch_harmonics_amd import _lib, ops
    from torch_harmonics_amd.plan import get_plan

    lib = _lib.load()  # raises if libs2attn.so is missing: there is no fallback to time
    cfg = CONFIGS[args.config]
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    if args.ring_only:
        print(json.dumps({"ring_steps": time_ring_steps(dev)}))
        return
    mod, x_in, x_out, k, v, q, dy = make_workload(cfg, dev)
    (Hi, Wi), (Ho, Wo) = cfg["in_shape"], cfg["out_shape"]
    nh, B = cfg["nh"], cfg["B"]
    nnz = mod.psi_col_idx.numel()
    pairs = B * nh * Wo * nnz
    wq, ci, ro = mod.quad_weights, mod.psi_col_idx, mod.psi_roff_idx
    bf16 = cfg.get("dtype") == "bf16"
    esz = 2 if bf16 else 4
    if bf16:  # 16-bit storage configuration: inputs scaled by 0.5 and stored as bf16, module in bf16
        mod = mod.to(torch.bfloat16)
        mod.quad_weights = wq  # the quadrature weights stay fp32
        x_in, x_out = (0.5 * x_in).to(torch.bfloat16), (0.5 * x_out).to(torch.bfloat16) if x_out is not x_in else None
        x_out = x_in if x_out is None else x_out
        k, v, q, dy = [(0.5 * t).to(torch.bfloat16).contiguous() for t in (k, v, q, dy)]

    def step():
        y, lse = ops.forward_lse(k, v, q, wq, ci, ro, nh, Wi, Ho, Wo)
        return y, ops.backward_saved(k, v, q, dy, y, lse, wq, ci, ro, nh, Wi, Ho, Wo)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_step = 1e3 * (time.perf_counter() - t0) / args.steps

    # the operators with the reference's exact signatures (attention_kernels::forward / backward: nothing handed from the forward to
    # the backward, which recomputes y and the softmax normaliser first), same tensors
    def ref_step():
        yy = ops.forward(k, v, q, wq, ci, ro, nh, Wi, Ho, Wo)
        return yy, ops.backward(k, v, q, dy, wq, ci, ro, nh, Wi, Ho, Wo)

    ms_ref_step = None
    if not args.no_reference_route:
        ref_step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            ref_step()
        torch.cuda.synchronize()
        ms_ref_step = 1e3 * (time.perf_counter() - t0) / args.steps

    # ---- per-kernel durations: events on the launch stream around each launch, same K steps ----
    plan = get_plan(ci, ro, Hi, Wi, Ho, Wo)
    shape = _lib.ShapeStruct(B, nh, Hi, Wi, Ho, Wo, k.shape[3] // nh, v.shape[3] // nh, _lib.S2ATTN_BF16 if bf16 else _lib.S2ATTN_F32)
    y = torch.empty(q.shape[:3] + (v.shape[3],), device=dev, dtype=k.dtype)
    dk, dv, dq = torch.empty_like(k), torch.empty_like(v), torch.empty_like(q)
    ws = torch.empty(lib.s2attn_backward_saved_workspace_bytes(ctypes.byref(shape)) // 4, device=dev)
    lse = torch.empty((B, nh, Ho, Wo), device=dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    pl, sh = ctypes.byref(plan.struct), ctypes.byref(shape)
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(4)] for _ in range(args.steps)]
    for s in range(args.steps):
        ev[s][0].record()
        _lib.check(lib.s2attn_forward_lse(k.data_ptr(), v.data_ptr(), q.data_ptr(), wq.data_ptr(), y.data_ptr(), lse.data_ptr(), pl, sh, stream), "fwd")
        ev[s][1].record()
        _lib.check(
            lib.s2attn_backward_dq_saved(
                k.data_ptr(), v.data_ptr(), q.data_ptr(), dy.data_ptr(), y.data_ptr(), lse.data_ptr(), wq.data_ptr(), dq.data_ptr(), ws.data_ptr(), pl, sh, stream
            ),
            "dq",
        )
        ev[s][2].record()
        _lib.check(
            lib.s2attn_backward_dkdv(k.data_ptr(), v.data_ptr(), q.data_ptr(), dy.data_ptr(), wq.data_ptr(), dk.data_ptr(), dv.data_ptr(), ws.data_ptr(), pl, sh, stream), "dkdv"
        )
        ev[s][3].record()
    torch.cuda.synchronize()
    t_fwd = sum(e[0].elapsed_time(e[1]) for e in ev) / args.steps
    t_dq = sum(e[1].elapsed_time(e[2]) for e in ev) / args.steps
    t_dkdv = sum(e[2].elapsed_time(e[3]) for e in ev) / args.steps

    nk, nv, nq, ny, nstat = k.numel(), v.numel(), q.numel(), y.numel(), lse.numel()
    d = k.shape[3] // nh
    # per launch: compulsory traffic (every tensor the kernel must read or write, once), algorithmic flops
    # (2*d per contraction per pair: forward q.k, p.v; dq pass q.k, dy.v, dq; dk/dv pass q.k, dy.v, dk, dv), time
    if bf16:
        kname = ("fwd_h16_kernel", "dq_h16_kernel", "dkdv_h16_kernel")
    elif d in (16, 64, 128) or (d == 32 and min(Wi, Wo) < 64):
        kname = ("fwd_m32_kernel", "dq_m32_kernel", "dkdv_m32_kernel")
    else:
        kname = ("fwd_mfma_kernel", "dq_saved_mfma_kernel", "dkdv_mfma_kernel")
    alg = {
        f"s2::{kname[0]} (forward)": (esz * (nq + nk + nv + ny) + 4 * nstat, 4 * d * pairs, t_fwd),
        f"s2::{kname[1]} (backward, dq)": (esz * (nq + nk + nv + ny + ny + nq) + 12 * nstat, 6 * d * pairs, t_dq),
        f"s2::{kname[2]} (backward, dk + dv)": (esz * (nq + nk + nv + ny + nk + nv) + 8 * nstat, 8 * d * pairs, t_dkdv),
    }
    matrix_peak = BF16_MATRIX_PEAK_TFLOPS if bf16 else FP32_MATRIX_PEAK_TFLOPS
    dom = max(alg, key=lambda n: alg[n][2])
    dom_bytes, dom_flops, dom_ms = alg[dom]
    # HBM bytes per launch measured with rocprofv3 counters on this workload (see profiles/); only valid for cfg3
    traffic = None
    tpath = os.path.join(ROOT, "profiles", "cfg3_hbm_traffic.json")
    if args.config == "cfg3" and os.path.exists(tpath):
        with open(tpath) as f:
            traffic = json.load(f).get(dom)
    achieved = dom_bytes / (dom_ms * 1e-3) / 1e9
    achieved_tf = dom_flops / (dom_ms * 1e-3) / 1e12
    # the step's own compulsory traffic: the backward counted as one pass (k, v, q, dy, y read once; dk, dv, dq written)
    step_bytes = esz * ((nq + nk + nv + ny) + (nq + nk + nv + ny + ny + nq + nk + nv)) + 8 * nstat
    flops_alg = 14 * d * pairs

    out = {
        "metric": "NeighborhoodAttentionS2 fwd+bwd neighbor-pairs/s",
        "value": pairs / (ms_step * 1e-3),
        "unit": "pairs/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if bf16 else "f32",
        "data": "synthetic",
        "config": {
            "workload": f"{args.config}: {cfg['grid_in']} {Hi}x{Wi} -> {cfg['grid_out']} {Ho}x{Wo}, B={B}, C={cfg['C']}, heads={nh}, {'bf16' if bf16 else 'fp32'}, theta_cutoff={cfg['theta_cutoff']}, nnz={nnz}, pairs={pairs}",
            "level": "op (s2attn forward + backward through the C ABI); module-level time in module_ms_per_step",
        },
        # 44 flop per compulsory byte puts this workload above the fp32 ridge (157.3 TFLOP/s / 8 TB/s = 20): the fp32
        # matrix peak is the roofline that binds; the HBM view of the same kernel follows in roofline_hbm
        "roofline": {
            "bound": "mfma",
            "kernel": dom,
            "achieved": achieved_tf,
            "peak": matrix_peak,
            "unit": "TFLOP/s",
            "frac": achieved_tf / matrix_peak,
            "traffic": traffic,
            "algorithmic_flops": dom_flops,
            "kernel_ms": dom_ms,
        },
        "roofline_hbm": {
            "bound": "hbm",
            "kernel": dom,
            "achieved": achieved,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS,
            "traffic": traffic,
            "algorithmic_bytes": dom_bytes,
            "kernel_ms": dom_ms,
        },
        "kernel_ms": {"fwd": t_fwd, "dq": t_dq, "dkdv": t_dkdv},
        "reference_signature_ms_per_step": ms_ref_step,  # attention_kernels::forward + attention_kernels::backward (forward recomputed in the backward)
        "step_hbm_frac": step_bytes / (ms_step * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "step_matrix_frac": flops_alg / (ms_step * 1e-3) / 1e12 / matrix_peak,
        "step_fp32_valu_frac": flops_alg / (ms_step * 1e-3) / 1e12 / FP32_VALU_PEAK_TFLOPS,
    }

    if not args.no_module:
        xq = x_out.clone().requires_grad_(True)
        same = x_in is x_out
        xk = None if same else x_in.clone().requires_grad_(True)
        gout = torch.randn(B, mod.out_channels, Ho, Wo, device=dev).to(x_out.dtype)

        def mstep():
            o = mod(xq) if same else mod(xq, xk, xk)
            o.backward(gout)
            mod.zero_grad(set_to_none=True)
            xq.grad = None
            if xk is not None:
                xk.grad = None

        for _ in range(2):
            mstep()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        nm = max(3, args.steps // 2)
        for _ in range(nm):
            mstep()
        torch.cuda.synchronize()
        out["module_ms_per_step"] = 1e3 * (time.perf_counter() - t0) / nm

    if not args.no_other_configs:
        # cfg1 and cfg2 are small enough for the reference's CPU algorithm in full: timed beside the GPU when the CPU leg is on
        out["other_configs"] = {
            name: time_other_config(name, dev, cpu=(not args.no_cpu_baseline) and name in ("cfg1", "cfg2")) for name in sorted(CONFIGS) if name != args.config
        }
        for name, t in (ref_times or {}).items():  # cfg1, cfg2 in full on the reference's own CPU operators
            if name in out["other_configs"]:
                out["other_configs"][name]["cpu_reference_fwd_ms"], out["other_configs"][name]["cpu_reference_bwd_ms"] = t["fwd_ms"], t["bwd_ms"]
        out["ring_steps"] = time_ring_steps(dev)
        out["published_shapes"] = time_published_shapes(dev)

    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(cfg, mod, k, v, q, dy, ref_times)

    print(json.dumps(out))


if __name__ == "__main__":
    main()
