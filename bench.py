#!/usr/bin/env python3
"""Benchmark of the SuperGrok v2 full optimizer step on one MI355X.

A "step" is one call of sg2_batched_step (sort -> bidirectional scan -> GRU ->
PEER -> expert MLP -> Adam/WD) over the whole synthetic parameter set, with
parameters, gradients, moments and meta-net weights already resident in HBM.
Prints ONE JSON line; see DESIGN.md for how each field is derived.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "supergrok1.5_amd"), os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)

BYTES_PER_ELEMENT = 72          # algorithmic HBM bytes per element per step (fp32): 40 read + 32 written
HBM_PEAK_GBS = 8000.0
FLOP_PER_ELEMENT = 30e3         # arithmetic actually required per element (both scan directions + elementwise)
VALU_PEAK_TFLOPS = 157.3


def build_workload(name, device):
    import torch
    import workloads as wl
    from helpers import DIMS
    shapes = {"scale50": wl.scale50_shapes, "shared14": wl.shared14_shapes}[name]()
    gh, di, ds = DIMS["gru_hidden"], DIMS["d_inner"], DIMS["d_state"]
    params = [p.reshape(-1).to(device) for p in wl.make_params(shapes, seed=0)]
    z = lambda *s: torch.zeros(*s, device=device)
    state = dict(params=params, eas=[z(p.numel()) for p in params], easqs=[z(p.numel()) for p in params],
                 mus=[z(p.numel()) for p in params], grus=[z(p.numel(), gh) for p in params],
                 mf=[z(di, ds) for _ in params], mb=[z(di, ds) for _ in params],
                 counts=torch.zeros(DIMS["num_experts"], dtype=torch.int32, device=device))
    # two resident gradient sets, alternated between steps (Student-t(3) tail on 0.5% of the entries,
    # per-tensor norm clip to 1.0 applied up front as the optimizer class does before the step)
    grad_sets = []
    for seed in (1, 2):
        g = wl.clip_per_tensor(wl.make_grads(shapes, seed=seed, tail_frac=0.005, tail="student3"))
        grad_sets.append([t.reshape(-1).to(device) for t in g])
    sharps = [torch.zeros_like(p) for p in params]
    weights = [w.to(device) for w in wl.meta_weights(7)]
    return shapes, state, grad_sets, sharps, weights


def cpu_baseline(sample_elems_target=1_000_000):
    """The CPU restatement of the reference's algorithm (sequential scan, the
    path grokking_optimizers/supergrok2.py:430-470 takes on CPU) timed on one
    host core over a bounded sample of the same parameter set."""
    import numpy as np
    import workloads as wl
    from helpers import default_scalars, f32_scalars, fresh_state_np
    from oracle import oracle as orc
    shapes = wl.scale50_shapes()
    pick, tot = [], 0
    for i, s in enumerate(shapes):           # smallest first until the sample is large enough
        n = wl.numel(s)
        if tot + n > sample_elems_target and pick:
            break
        pick.append(i)
        tot += n
    W = [w.numpy() for w in wl.meta_weights(7)]
    params = wl.make_params([shapes[i] for i in pick], seed=0)
    grads = wl.make_grads([shapes[i] for i in pick], seed=1, tail_frac=0.005, tail="student3")
    t0 = time.perf_counter()
    for k, i in enumerate(pick):
        st = fresh_state_np(params[k].numpy())
        g = grads[k].numpy().reshape(-1)
        orc.sg2_step(W, st, g, np.zeros_like(g), f32_scalars(default_scalars(i=i)), precision=32, chunk_len=0)
    dt = time.perf_counter() - t0
    return {"value": tot / dt, "unit": "elements/s", "cores": 1, "kind": "port",
            "sample": "tensors %d..%d of the 50-tensor set (%d elements), 1 step, sequential scan, "
                      "fp32 C++ restatement, %.1f s" % (pick[0], pick[-1], tot, dt)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="scale50", choices=["scale50", "shared14"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: every box here has one GPU and the path uses no collectives; "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    from grokking_optimizers import _cabi
    from sg2_harness import per_tensor_scalars, shared_scalars
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = "cuda:0"
    shapes, st, grad_sets, sharps, weights = build_workload(args.workload, dev)
    total = sum(p.numel() for p in st["params"])
    step = _cabi.Sg2Step(weights, st["params"], st["eas"], st["easqs"], st["mus"], st["grus"], st["mf"], st["mb"],
                         st["counts"])
    shared = shared_scalars()
    t = 0
    for _ in range(args.warmup):
        t += 1
        step(grad_sets[t & 1], sharps, per_tensor_scalars(len(shapes), t), shared)
    torch.cuda.synchronize()
    scal = [per_tensor_scalars(len(shapes), t + k + 1) for k in range(args.steps)]
    _cabi.profile_enable(True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(args.steps):
        t += 1
        step(grad_sets[t & 1], sharps, scal[k], shared)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    stage_ms, calls = _cabi.profile_read()
    _cabi.profile_enable(False)
    assert calls == min(args.steps, 256)
    for lst in (st["params"], st["eas"], st["grus"]):
        assert all(bool(torch.isfinite(x).all()) for x in lst), "non-finite state after the timed steps"

    ms_per_step = 1e3 * elapsed / args.steps
    value = total * args.steps / elapsed
    stage_avg = {k: v / calls for k, v in stage_ms.items()}
    dom = max(stage_avg, key=stage_avg.get)
    kernel_of = {"sort": "k_keys + 4 x (k_hist, k_spine_*, k_scatter)", "scan_summary": "k_scan<false>",
                 "chunk_prefix": "k_chunk_prefix", "scan_output": "k_scan<true>", "elementwise": "k_elem<false>"}
    achieved = BYTES_PER_ELEMENT * total / (stage_avg[dom] * 1e-3) / 1e9
    out = {
        "metric": "param-elements/sec per optimizer step (SuperGrok v2); % HBM roofline",
        "value": value, "unit": "elements/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "SuperGrok v2 full step, %d tensors, %d elements (%s), fp32, bilevel off"
                               % (len(shapes), total, "BASELINE configs[3]" if args.workload == "scale50" else "configs[2] set"),
                   "chunk_len": _cabi.lib().sg2_get_chunk_len()},
        "roofline": {"bound": "hbm", "kernel": kernel_of[dom], "achieved": achieved, "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS, "traffic": None,
                     "kernel_ms": stage_avg[dom]},
        "step_hbm_frac": BYTES_PER_ELEMENT * value / 1e9 / HBM_PEAK_GBS,
        "step_valu_frac": FLOP_PER_ELEMENT * value / 1e12 / VALU_PEAK_TFLOPS,
        "stage_ms": stage_avg,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
