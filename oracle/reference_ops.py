"""
Front end of the reference's OWN CPU operators, built by `make -C oracle ref` into oracle/_ref/attention_ref.so from the
reference's sources (attention_interface.cpp:85-119 declares them; kernels_cpu/attention_cpu_fwd.cpp:48-141,
attention_cpu_bwd.cpp:40-139 and the _upsample files implement them).

TEST INFRASTRUCTURE ONLY: used to validate the restatement in s2attn_oracle.c and as the timed CPU baseline.  Every call
runs in a child process (ref_worker.py), because the library registers the operator namespace the product's binding
registers as well.  Tensors are CPU tensors in the op's layout, as in cpu_attention.py.
"""
import os
import subprocess
import sys
import tempfile

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIBRARY = os.path.join(_HERE, "_ref", "attention_ref.so")


def available() -> bool:
    return os.path.exists(LIBRARY)


REFERENCE_SOURCES = "/root/reference/torch_harmonics/attention/optimized"


def build(force: bool = False) -> None:
    """Compile the reference's CPU operators where the reference's sources are present (no-op otherwise: a library built
    earlier is kept and used)."""
    if not os.path.isdir(REFERENCE_SOURCES):
        return
    if force:
        subprocess.run(["make", "-C", _HERE, "clean-ref"], check=True, capture_output=True)
    subprocess.run(["make", "-C", _HERE, "ref", "-j6"], check=True, capture_output=True)


def run(jobs, threads=None):
    """jobs: list of {"op", "args", "repeat"?, "discard"?}; returns the worker's list of {"out", "seconds"}."""
    if not available():
        raise RuntimeError("oracle/_ref/attention_ref.so is not built (make -C oracle ref needs the reference's sources)")
    with tempfile.TemporaryDirectory() as tmp:
        jin, jout = os.path.join(tmp, "jobs.pt"), os.path.join(tmp, "results.pt")
        torch.save(jobs, jin)
        env = dict(os.environ)
        if threads:
            env["OMP_NUM_THREADS"] = str(threads)
        done = subprocess.run([sys.executable, os.path.join(_HERE, "ref_worker.py"), jin, jout], env=env, capture_output=True, text=True)
        if done.returncode != 0:
            raise RuntimeError(f"reference worker failed ({done.returncode}):\n{done.stderr[-2000:]}")
        return torch.load(jout, weights_only=True)


def _cpu(t, dtype=None):
    return t.detach().to(device="cpu", dtype=dtype or t.dtype).contiguous()


def forward_job(k, v, q, quad_weights, col_idx, row_off, nh, **kw):
    Wi, Ho, Wo = k.shape[2], q.shape[1], q.shape[2]
    return dict(op="forward", args=[_cpu(k), _cpu(v), _cpu(q), _cpu(quad_weights, torch.float32), _cpu(col_idx, torch.int64), _cpu(row_off, torch.int64), int(nh), Wi, Ho, Wo], **kw)


def backward_job(k, v, q, dy, quad_weights, col_idx, row_off, nh, **kw):
    Wi, Ho, Wo = k.shape[2], q.shape[1], q.shape[2]
    return dict(op="backward", args=[_cpu(k), _cpu(v), _cpu(q), _cpu(dy), _cpu(quad_weights, torch.float32), _cpu(col_idx, torch.int64), _cpu(row_off, torch.int64), int(nh), Wi, Ho, Wo], **kw)


def forward(k, v, q, quad_weights, col_idx, row_off, nh):
    return run([forward_job(k, v, q, quad_weights, col_idx, row_off, nh)])[0]["out"][0]


def backward(k, v, q, dy, quad_weights, col_idx, row_off, nh):
    """Returns (dk, dv, dq), the reference's order."""
    return tuple(run([backward_job(k, v, q, dy, quad_weights, col_idx, row_off, nh)])[0]["out"])
