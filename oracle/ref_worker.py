"""
Child process that runs the reference's own CPU operators from oracle/_ref/attention_ref.so.

TEST INFRASTRUCTURE ONLY.  The library is the reference's CPU path (attention_interface.cpp and kernels_cpu/*.cpp of its
torch_harmonics/attention/optimized directory) compiled by oracle/Makefile (target `ref`); it registers the operator
namespace `attention_kernels`, which the product's own binding registers too, so it lives in a process of its own and is
never imported next to the package.

usage: python ref_worker.py <jobs.pt> <results.pt>
  jobs.pt     torch.save of a list of {"op": name, "args": [tensors and ints], "repeat": n (optional),
              "discard": bool (optional: keep the timings, drop the outputs)}; an argument
              {"randn": shape, "seed": n, "scale": x} stands for a seeded N(0, x^2) fp32 tensor made here
  results.pt  torch.save of a list of {"out": [tensors], "seconds": [wall time of every repetition]}
Operators: forward, backward, permute_to_nhwc, permute_to_nchw (schemas: attention_interface.cpp:85-119).
"""
import os
import sys
import time

import torch


def main(argv):
    here = os.path.dirname(os.path.abspath(__file__))
    torch.ops.load_library(os.path.join(here, "_ref", "attention_ref.so"))
    ops = torch.ops.attention_kernels
    jobs = torch.load(argv[1], weights_only=True)
    results = []
    for job in jobs:
        fn = getattr(ops, job["op"])
        for i, a in enumerate(job["args"]):
            if isinstance(a, dict):
                job["args"][i] = float(a.get("scale", 1.0)) * torch.randn(*a["randn"], generator=torch.Generator().manual_seed(int(a["seed"])))
        seconds, out = [], None
        for _ in range(int(job.get("repeat", 1))):
            t0 = time.perf_counter()
            out = fn(*job["args"])
            seconds.append(time.perf_counter() - t0)
        out = list(out) if isinstance(out, (tuple, list)) else [out]
        results.append({"out": [] if job.get("discard") else out, "seconds": seconds})
    torch.save(results, argv[2])


if __name__ == "__main__":
    main(sys.argv)
