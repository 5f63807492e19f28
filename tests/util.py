"""Shared helpers of the test suite: seeded inputs, the benchmark configurations, tolerances."""

import math

import torch

SEED = 333  # the reference's test seed (tests/testutils.py:58-77)

# the five configurations the benchmark definition names; full sizes
CONFIGS = {
    "cfg1": dict(in_shape=(32, 64), out_shape=(32, 64), grid_in="equiangular", grid_out="equiangular", B=1, C=16, nh=1, theta_cutoff=None, dtype=torch.float32),
    "cfg2": dict(in_shape=(128, 256), out_shape=(128, 256), grid_in="equiangular", grid_out="equiangular", B=4, C=64, nh=4, theta_cutoff=4 * math.pi / 127, dtype=torch.float32),
    "cfg3": dict(in_shape=(721, 1440), out_shape=(721, 1440), grid_in="equiangular", grid_out="equiangular", B=1, C=256, nh=8, theta_cutoff=3 * math.pi / 720, dtype=torch.float32),
    "cfg4": dict(in_shape=(721, 1440), out_shape=(360, 720), grid_in="equiangular", grid_out="legendre-gauss", B=2, C=128, nh=4, theta_cutoff=2 * math.pi / 359, dtype=torch.float32),
    "cfg5": dict(in_shape=(361, 720), out_shape=(361, 720), grid_in="legendre-gauss", grid_out="legendre-gauss", B=4, C=1024, nh=16, theta_cutoff=8 * math.pi / 360, dtype=torch.bfloat16),
}


def randn_inputs(B, Hi, Wi, Ho, Wo, nh, ck, cv, seed=SEED, scale=1.0):
    """
    k, v, dy ~ N(0, scale^2) and q ~ N(0, scale^2) / sqrt(ck), generated on the CPU from one seed, NHWC
    heads-packed, fp32.  The op receives the query already multiplied by the softmax scale
    (attention.py:551), which for the module's default is 1 / sqrt(per-head channels); feeding an
    unscaled N(0,1) query makes q.k ~ N(0, ck) and turns the check into a test of exp() conditioning.
    """
    g = torch.Generator().manual_seed(seed)
    k = scale * torch.randn(B, Hi, Wi, nh * ck, generator=g)
    v = scale * torch.randn(B, Hi, Wi, nh * cv, generator=g)
    q = scale * torch.randn(B, Ho, Wo, nh * ck, generator=g) / math.sqrt(ck)
    dy = scale * torch.randn(B, Ho, Wo, nh * cv, generator=g)
    return k, v, q, dy


def assert_close(name, got, want, rtol, atol):
    got = got.detach().double().cpu()
    want = want.detach().double().cpu()
    assert got.shape == want.shape, f"{name}: shape {tuple(got.shape)} vs {tuple(want.shape)}"
    if got.numel() == 0:
        return
    assert torch.isfinite(got).all(), f"{name}: non-finite values"
    err = (got - want).abs()
    bound = atol + rtol * want.abs()
    worst = (err - bound).max().item()
    assert worst <= 0, f"{name}: max |err| {err.max().item():.3e}, exceeds atol {atol} + rtol {rtol} by {worst:.3e}"
