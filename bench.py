#!/usr/bin/env python3
"""Benchmark of the SuperGrok v2 full optimizer step on one MI355X.

A "step" is one call of sg2_batched_step (sort -> bidirectional scan -> GRU ->
PEER -> expert MLP -> Adam/WD) over the whole synthetic parameter set, with
parameters, gradients, moments and meta-net weights already resident in HBM.
Prints ONE JSON line: whole-step throughput, the roofline figures of the dominant kernel (timed by HIP
events on the step's stream), and a single-core CPU baseline on a bounded sample.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "supergrok1.5_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

BYTES_PER_ELEMENT = 72          # algorithmic HBM bytes per element per step (fp32): 40 read + 32 written
HBM_PEAK_GBS = 8000.0
# HBM bytes per launch (read + written) on the 25M-element workload: constants copied from the rocprofv3 --pmc
# FETCH_SIZE / WRITE_SIZE summary under profiles/ (scaled by what the same counters read for a 1 GiB device copy);
# not measured by this script and valid for the default workload only
PMC_TRAFFIC_BYTES_SCALE50 = {"scan_output": 0.513e9 + 2.501e9, "scan_summary": 0.028e9 + 0.049e9,
                             "elementwise": 2.503e9 + 0.801e9}


# Vector-ALU instructions per launch (SQ_INSTS_VALU of the same profile, default workload only) and the rate the part
# sustains on nothing but independent fp32 instructions (bench.py --workload valu-probe, profiles/valu_probe_mi355x.txt):
# what actually bounds these kernels
# (the per-element kernel's count holds 8.6e6 fp32 matrix instructions of 64 clocks each: 16 vector instructions' worth of time apiece)
PMC_VALU_INSTS_SCALE50 = {"scan_output": 1.89e9, "scan_summary": 1.16e8, "elementwise": 6.19e8 + 15 * 8.6e6}
VALU_SUSTAINED_PER_NS_SIMD = 0.59
SIMDS = 1024


LARGE_GEOMETRY = dict(d_model=16, d_state=32, d_inner=32)     # the second scan geometry the kernels are built for


def build_workload(name, device, nonzero_sharpness=False, weights="bench", geometry="default"):
    import torch
    import workloads as wl
    DIMS = dict(wl.DEFAULT_DIMS, **(LARGE_GEOMETRY if geometry == "large" else {}))
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
    # sharpness is 0 until a SAM probe has run (the optimizer's initial state and the configuration the metric is quoted on);
    # --sharpness measures the step with a populated sharpness cache instead (one more random gather per element)
    sharps = [torch.zeros_like(p) for p in params]
    if nonzero_sharpness:
        sharps = [(g.abs() * 0.5).contiguous() for g in grad_sets[1]]
    # "bench": N(0, 0.1) in every tensor (the configuration the metric is quoted on); "module": the optimizer's own
    # initial meta-net (A_log = log(1..16), default Linear weights)
    weights = [w.to(device) for w in (wl.meta_weights(7, DIMS) if weights == "bench" else wl.module_weights(0))]
    return shapes, state, grad_sets, sharps, weights, DIMS


def cpu_baseline(sample_elems_target=4_000_000):
    """The CPU restatement of the reference's algorithm (sequential scan, the
    path grokking_optimizers/supergrok2.py:430-470 takes on CPU) timed on one
    host core over a bounded sample of the same parameter set."""
    import numpy as np
    import workloads as wl
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
    D = wl.DEFAULT_DIMS
    for k, i in enumerate(pick):
        g = grads[k].numpy().reshape(-1)
        n = g.size
        st = dict(param=params[k].numpy().reshape(-1).copy(), exp_avg=np.zeros(n, np.float32), exp_avg_sq=np.zeros(n, np.float32),
                  mu=np.zeros(n, np.float32), gru=np.zeros((n, D["gru_hidden"]), np.float32),
                  mamba_fwd=np.zeros((D["d_inner"], D["d_state"]), np.float32),
                  mamba_bwd=np.zeros((D["d_inner"], D["d_state"]), np.float32))
        sc = dict(wl.per_tensor_scalars(i + 1, 1)[i], **wl.shared_scalars())
        orc.sg2_step(W, st, g, np.zeros_like(g), sc, precision=32, chunk_len=0)
    dt = time.perf_counter() - t0
    return {"value": tot / dt, "unit": "elements/s", "cores": 1, "kind": "port",
            "sample": "tensors %d..%d of the 50-tensor set (%d elements), 1 step, sequential scan, "
                      "fp32 C++ restatement, %.1f s" % (pick[0], pick[-1], tot, dt)}


def build_step(workload, ops, dev, limit=None):
    """One secondary workload as a closure over `ops` (this package's `_ops`, or the reference's own CPU build: the
    function names and argument orders are the same) on tensors living on `dev`.  limit: use only the first tensors
    of the set, up to that many elements (the bounded CPU sample)."""
    import torch
    import workloads as wl

    def take(shapes):
        if limit is None:
            return shapes
        out, tot = [], 0
        for sh in shapes:
            if out and tot + wl.numel(sh) > limit:
                break
            out.append(sh)
            tot += wl.numel(sh)
        return out

    W = dict(dtype="f32", bound="hbm", peak=HBM_PEAK_GBS, unit="elements/s", bytes_per_elem=40)
    if workload == "muon":
        shapes = [(1024, 4096)] * 12 + [(4096, 1024)] * 12
        if limit is not None:
            shapes = [(1024, 4096), (4096, 1024)]
        gen = torch.Generator().manual_seed(0)
        params = [(torch.randn(*s, generator=gen) * 0.02).to(torch.bfloat16).to(dev) for s in shapes]
        grads = [(torch.randn(*s, generator=gen) * 1e-3).to(torch.bfloat16).to(dev) for s in shapes]
        bufs = [torch.zeros(s, device=dev) for s in shapes]
        W.update(step=lambda: ops.muon_fused_step(params, grads, bufs, 0.95, 0.02, 1.0, 5),
                 units=5 * sum(6 * min(s) ** 2 * max(s) for s in shapes), unit="FLOP/s",       # 6 min^2 max per NS iteration
                 # what the kernels execute: the two symmetric products launch only the 256 x 256 tiles on or above the diagonal
                 executed=5 * sum(2 * 256 * 256 * ((-(-min(s) // 256)) * (-(-min(s) // 256) + 1) // 2) * ((-(-max(s) // 256)) * 256 + (-(-min(s) // 256)) * 256)
                                  + 2 * ((-(-min(s) // 256)) * 256) ** 2 * ((-(-max(s) // 256)) * 256) for s in shapes),
                 name="Muon step, %d x [1024,4096] + %d x [4096,1024], 5 Newton-Schulz iterations" % (len(shapes) // 2, len(shapes) // 2),
                 dtype="bf16", bound="mfma", peak=2500.0)
        return W
    small = workload in ("grokfast", "sg15", "bilevel")
    shapes = take(wl.shared14_shapes() if small else wl.scale50_shapes())
    params = [p.reshape(-1).to(dev) for p in wl.make_params(shapes, seed=0)]
    if small:
        grads = [g.reshape(-1).to(dev) for g in wl.make_grads(shapes, seed=1, tail_frac=0.01 if workload == "sg15" else 0.0)]
    else:
        # the other fused steps, on the 50-tensor / 25 M-element set so that HBM traffic, not launch latency, is measured
        grads = [g.reshape(-1).to(dev) for g in wl.make_grads(shapes, seed=1, tail_frac=0.005, tail="student3")]
    z = lambda: [torch.zeros_like(p) for p in params]
    n = sum(p.numel() for p in params)
    P = len(params)
    a, b, c, d = z(), z(), z(), z()
    gen = torch.Generator().manual_seed(3)
    t = [0]
    setname = "%d tensors, %d elements" % (P, n)
    if workload == "grokfast":
        def step():
            t[0] += 1
            ops.grokfast_adamw_fused_step(params, grads, a, b, c, [t[0]] * P, 0.98, 2.0, 1e-3, 0.9, 0.98, 1e-8, 1.0)
        what = "Grokfast fused step (EMA + amplify + AdamW)"
    elif workload == "sg15":
        H = 32
        W1, b1 = (torch.randn(H, 2, generator=gen) * 0.01).to(dev), torch.zeros(H, device=dev)
        W2, b2 = (torch.randn(1, H, generator=gen) * 0.01).to(dev), torch.zeros(1, device=dev)

        def step():
            ops.supergrok15_fused_step(params, grads, a, b, c, d, [0] * P, [0.98] * P, [0.9 * 0.9 ** i for i in range(P)],
                                       W1, b1, W2, b2, 0.1, H, 0.999, 1e-3, 1.0, 1e-8, 2.0, 1.0, 0.5, 1.0)
        what = "SuperGrok v1.5 full step (H=32, exact GELU, device-side clip)"
    elif workload == "bilevel":
        # gradient of sum <smart_grad, cotangent> with respect to every weight of the v2 meta-net, for all tensors
        # of the model at once: sort + scan forward, per-element forward/backward, scan adjoint, all in HIP
        from grokking_optimizers import Mamba3PEERMetaNet, _bilevel
        torch.manual_seed(0)
        mn = Mamba3PEERMetaNet().to(dev)
        sharps = [g.abs() * 0.5 for g in grads]
        grus = [torch.zeros(g.numel(), 4, device=dev) for g in grads]
        mf = [torch.zeros(16, 16, device=dev) for _ in grads]
        mb = [torch.zeros(16, 16, device=dev) for _ in grads]
        cots = [torch.randn(g.numel(), generator=torch.Generator().manual_seed(5)).to(dev) for g in grads]

        def step():
            mn.zero_grad()
            _bilevel.accumulate_meta_gradients(mn, grads, sharps, grus, mf, mb, cots)
        # per element: grad, sharpness, cotangent, GRU state read (28 B); both contexts written by the scan and read
        # by the per-element pass, their gradients written by it and read by the adjoint (4 x 64 B)
        W["bytes_per_elem"] = 284
        what = "SuperGrok v2 bilevel meta-gradient pass (sort + scan, per-element forward/backward, scan adjoint)"
    elif workload == "grokadamw":
        def step():
            t[0] += 1
            ops.grokadamw_fused_step(params, grads, a, b, c, [t[0]] * P, 0.98, 5.0, 0.9, 0.98, 1e-3, 1.0, 1e-8, 1.0)
        W["bytes_per_elem"], what = 36, "GrokAdamW fused step (clip + EMA + amplify + AdamW)"
    elif workload == "neuralgrok":
        H = 128
        Wn = [(torch.randn(H, 1, generator=gen) * 0.5).to(dev), torch.zeros(H, device=dev),
              (torch.randn(1, H, generator=gen) * 0.1).to(dev), torch.zeros(1, device=dev)]

        def step():
            t[0] += 1
            ops.neuralgrok_fused_step(params, grads, a, b, [t[0]] * P, *Wn, 10.0, 4.0, H, 0.9, 0.98, 1e-3, 1.0, 1e-8, 1.0)
        W["bytes_per_elem"], what = 28, "NeuralGrok fused step (clip + 1->128->1 amplifier + AdamW)"
    elif workload == "prodigy":
        inits = [p.clone() for p in params]
        dl = [1e-6]

        def step():
            t[0] += 1
            dl[0] = ops.prodigy_fused_step(params, grads, a, b, c, inits, [t[0]] * P, dl[0], 0.9, 0.999, 1e-3, 0.0, 1e-8)
        W["bytes_per_elem"], what = 52, "Prodigy fused step (d_lr reduction pass + Adam pass, one host read of d_lr)"
    elif workload == "lion":
        def step():
            ops.lion_fused_step(params, grads, a, 1e-4, 0.9, 0.99, 3.0)
        W["bytes_per_elem"], what = 20, "Lion fused step"
    else:
        H = 32
        Ws = [(torch.randn(H, 2, generator=gen) * 0.01).to(dev), torch.zeros(H, device=dev),
              (torch.randn(1, H, generator=gen) * 0.01).to(dev), torch.zeros(1, device=dev)]
        beta1s = [0.9 * 0.9 ** i for i in range(P)]

        def step():
            ops.supergrok11_fused_step(params, grads, a, b, c, d, [0] * P, [0.98] * P, beta1s, *Ws, 0.1, H, 0.999, 1e-3, 1.0,
                                       1e-8, 5.0, 1.0, 5.0, 1.0)
        W["bytes_per_elem"], what = 52, "SuperGrok v1.1 full step (H=32, exact GELU, device-side clip and cosine gates)"
    W.update(step=step, units=n, name="%s, %s" % (what, setname))
    return W


def cpu_reference_baseline(workload):
    """The reference's own CPU code (its csrc/ops.cpp compiled without CUDA into oracle/_ref by oracle/Makefile.ref),
    timed on a bounded sample of the same workload.  None when that build is not there or has no such step."""
    import torch
    ref_dir = os.path.join(ROOT, "oracle", "_ref")
    if workload in ("bilevel", "grokfast") or not os.path.isdir(ref_dir):
        return None       # the reference has no CPU op for these (Grokfast's AdamW half is Python there)
    sys.path.insert(0, ref_dir)
    try:
        import ref_ops
    except ImportError:
        return None
    W = build_step(workload, ref_ops, "cpu", limit=4_000_000)
    W["step"]()                                   # warm-up (allocations, thread pool)
    steps, t0 = 0, time.perf_counter()
    while steps < 200 and (steps < 3 or time.perf_counter() - t0 < 5.0):
        W["step"]()
        steps += 1
    el = (time.perf_counter() - t0) / steps
    return {"value": W["units"] / el, "unit": W["unit"], "cores": torch.get_num_threads(), "kind": "reference",
            "sample": "%s; %d step(s) of the reference's CPU path (ATen ops, %d threads), %.1f s" %
                      (W["name"], steps, torch.get_num_threads(), el * steps)}


def bench_other(args, dev):
    """Secondary measurements: the other fused steps through `_ops`."""
    import torch
    from grokking_optimizers import _ops
    K, Wm = args.steps, args.warmup
    W = build_step(args.workload, _ops, dev)
    step, units = W["step"], W["units"]
    for _ in range(Wm):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(K):
        step()
    torch.cuda.synchronize()
    el = (time.perf_counter() - t0) / K
    out = {"metric": "secondary: " + args.workload, "value": units / el, "unit": W["unit"], "n_gpus": 1, "steps": K, "warmup": Wm,
           "ms_per_step": 1e3 * el, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": W["dtype"],
           "data": "synthetic", "config": {"workload": W["name"]}}
    if W["bound"] == "mfma":
        out["roofline"] = {"bound": "mfma", "achieved": units / el / 1e12, "peak": W["peak"], "unit": "TFLOP/s",
                           "frac": units / el / 1e12 / W["peak"], "traffic": None}
        if "executed" in W:        # `achieved` counts the algorithm's FLOP; these count the FLOP the kernels execute
            out["roofline"]["achieved_executed"] = W["executed"] / el / 1e12
            out["roofline"]["frac_executed"] = W["executed"] / el / 1e12 / W["peak"]
    else:
        bpe = W["bytes_per_elem"]                      # algorithmic bytes per element of the step
        out["roofline"] = {"bound": "hbm", "achieved": bpe * units / el / 1e9, "peak": W["peak"], "unit": "GB/s",
                           "frac": bpe * units / el / 1e9 / W["peak"], "traffic": None, "bytes_per_element": bpe}
    if not args.no_cpu_baseline:
        base = cpu_reference_baseline(args.workload)
        if base is not None:
            out["cpu_baseline"] = base
    return out


def bench_probe(dev):
    """Issue rate of plain fp32 vector instructions (sg_probe_valu): wave64 instructions per nanosecond and SIMD for
    fma / mul / add / DPP-add streams with every SIMD of the chip busy, by resident waves per SIMD; and the shader
    clock the part holds meanwhile (ticks of the in-kernel clock per nanosecond of the launch)."""
    import ctypes as C
    import torch
    from grokking_optimizers import _cabi
    L = _cabi.lib()
    L.sg_probe_workspace_bytes.restype = C.c_size_t
    L.sg_probe_valu.argtypes = [C.c_int] * 4 + [C.POINTER(C.c_float), C.POINTER(C.c_double), C.POINTER(C.c_double),
                                                C.c_void_p, C.c_size_t, C.c_void_p]
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    ws = torch.empty(L.sg_probe_workspace_bytes(cus, 8), dtype=torch.uint8, device=dev)
    rows, best = [], 0.0
    for ncu in (cus,):
        for op, name in enumerate(("fma", "mul", "add", "add_dpp", "mfma_32x32x16_bf16", "mfma_32x32x16_bf16_random_operands",
                                   "mfma_32x32x1_f32", "mfma_32x32x1_f32_then_8_fma", "mfma_4x4x1_f32")):
            for w in ((1, 2) if op >= 4 else (1, 2, 3, 4, 8)):
                ms, ticks, instr = C.c_float(), C.c_double(), C.c_double()
                if L.sg_probe_valu(op, ncu, w, 2000, C.byref(ms), C.byref(ticks), C.byref(instr), ws.data_ptr(), ws.numel(),
                                   torch.cuda.current_stream().cuda_stream) != 0:
                    raise RuntimeError(_cabi.last_error())
                rate = instr.value * w / (ms.value * 1e6)            # per SIMD: w waves share one
                rows.append({"op": name, "cus": ncu, "waves_per_simd": w, "ms": round(ms.value, 4),
                             "instr_per_ns_per_simd": round(rate, 4),
                             "clock_ticks_per_instr_per_simd": round(ticks.value / instr.value / w, 3),
                             "clock_ticks_per_ns": round(ticks.value / (ms.value * 1e6), 3)})
                if op >= 4:      # flop per matrix instruction (the vector fma of the mixed stream are not counted)
                    rows[-1]["chip_tflops"] = round(rate * (32768, 32768, 4096, 4096, 512)[op - 4] * 4 * ncu / 1e3, 1)
                elif ncu == cus:
                    best = max(best, rate)
    return {"metric": "secondary: valu-probe", "value": best, "unit": "wave64 instructions/ns/SIMD (whole chip, best case)",
            "n_gpus": 1, "steps": 1, "warmup": 1, "ms_per_step": None, "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "f32", "data": "synthetic",
            "config": {"workload": "plain fp32 VALU instruction streams, 8 independent accumulators per lane, %d CUs" % cus},
            "rows": rows}


def class_step_ms(shapes, grad_sets, dev, steps, warmup):
    """Wall time of SuperGrok2.step() itself (per-tensor clip on the device, scalar schedules, the 51-argument
    `_ops` call), same tensors and gradients, the module's own initial meta-weights, recycling off."""
    import torch
    from grokking_optimizers import SuperGrok2
    import workloads as wl
    params = [torch.nn.Parameter(p.to(dev)) for p in wl.make_params(shapes, seed=0)]
    opt = SuperGrok2(params, lr=1e-3, recycle_interval=0)
    t = 0

    def one():
        nonlocal t
        t += 1
        for p, g in zip(params, grad_sets[t & 1]):
            p.grad = g.view(p.shape)
        opt.step()
    for _ in range(warmup):
        one()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        one()
    torch.cuda.synchronize()
    return 1e3 * (time.perf_counter() - t0) / steps


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--sharpness", action="store_true", help="v2 workloads: non-zero sharpness cache (as after a SAM probe)")
    ap.add_argument("--workload", default="scale50", choices=["scale50", "shared14", "grokfast", "sg15", "muon", "grokadamw", "neuralgrok", "prodigy", "lion", "sg11", "bilevel", "valu-probe"],
                    help="scale50 (default, the headline configuration) and shared14 time the SuperGrok v2 step; "
                         "grokfast / sg15 / muon time the other fused steps (14-tensor set; 24 bf16 matrices)")
    ap.add_argument("--chunk-len", type=int, default=0, help="scan chunk length (0: library default)")
    ap.add_argument("--window", type=int, default=-1, help="scan summary window (-1: library default, 0: off)")
    ap.add_argument("--weights", default="bench", choices=["bench", "module"],
                    help="v2 workloads: meta-net weights N(0, 0.1) (default, the measured configuration) or the optimizer's own initialisation")
    ap.add_argument("--geometry", default="default", choices=["default", "large"],
                    help="v2 workloads: meta-net of d_model=8, d_state=16, d_inner=16 (the configuration the metric is quoted on) or 16, 32, 32")
    ap.add_argument("--boundary", default="ops", choices=["ops", "cabi"],
                    help="v2 workloads: time the torch-extension call _ops.supergrok2_mamba_peer_batched_step (default) or the bare C-ABI call")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-class-step", action="store_true", help="skip the wall time of SuperGrok2.step() (keeps a kernel trace to the C-ABI steps)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one plain device copy of 1 GiB (a reference point for scaling the FETCH_SIZE / "
                         "WRITE_SIZE counters of a rocprofv3 --pmc run)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: every box here has one GPU and the path uses no collectives; "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    from grokking_optimizers import _cabi
    from workloads import per_tensor_scalars, shared_scalars
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = "cuda:0"
    if args.workload == "valu-probe":
        print(json.dumps(bench_probe(dev)))
        return
    if args.workload not in ("scale50", "shared14"):
        print(json.dumps(bench_other(args, dev)))
        return
    if _cabi.lib().sg2_set_chunk_len(args.chunk_len) or _cabi.lib().sg2_set_scan_window(args.window):
        raise SystemExit(_cabi.last_error())
    if args.geometry == "large" and args.weights != "bench":
        raise SystemExit("--geometry large runs with --weights bench")
    shapes, st, grad_sets, sharps, weights, D = build_workload(args.workload, dev, args.sharpness, args.weights, args.geometry)
    total = sum(p.numel() for p in st["params"])
    if args.boundary == "cabi":
        step = _cabi.Sg2Step(weights, st["params"], st["eas"], st["easqs"], st["mus"], st["grus"], st["mf"], st["mb"],
                             st["counts"], dims=D)
    else:
        # the reference's own entry point: supergrok2_mamba_peer_batched_step of the torch extension, 51 arguments
        from grokking_optimizers import _ops

        def step(grads, sharps_, per_tensor, sh):
            col = lambda k: [float(sc[k]) for sc in per_tensor]
            _ops.supergrok2_mamba_peer_batched_step(
                st["params"], grads, sharps_, st["eas"], st["easqs"], st["mus"], st["grus"], st["mf"], st["mb"], *weights,
                col("alpha"), col("lamb_eff"), col("beta1"), col("bc1"), col("bc2"), sh["rescale"], sh["beta2"], sh["lr"],
                sh["wd_eff"], sh["eps"], D["d_model"], D["d_state"], D["d_inner"], D["gru_hidden"], D["num_heads"],
                D["pk_dim"], D["expert_hidden"], D["num_experts"], st["counts"])
    shared = shared_scalars()
    if args.copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
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
                               % (len(shapes), total, "50 log-uniform tensors" if args.workload == "scale50" else "2-layer transformer set"),
                   "chunk_len": _cabi.chunk_len_for([p.numel() for p in st["params"]]), "summary_window": _cabi.lib().sg2_get_scan_window(),
                   "timed_call": "_ops.supergrok2_mamba_peer_batched_step" if args.boundary == "ops" else "sg2_batched_step (C ABI)",
                   "meta_weights": "N(0, 0.1), seed 7" if args.weights == "bench" else "Mamba3PEERMetaNet() initialisation, seed 0",
                   "meta_net": "d_model=%d d_state=%d d_inner=%d" % (D["d_model"], D["d_state"], D["d_inner"])},
        "roofline": {"bound": "hbm", "kernel": kernel_of[dom], "achieved": achieved, "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                     "traffic": PMC_TRAFFIC_BYTES_SCALE50.get(dom) if (args.workload, args.weights, args.geometry) == ("scale50", "bench", "default") else None,
                     "kernel_ms": stage_avg[dom]},
        "step_hbm_frac": BYTES_PER_ELEMENT * value / 1e9 / HBM_PEAK_GBS,
        "stage_ms": stage_avg,
    }
    if (args.workload, args.weights, args.geometry) == ("scale50", "bench", "default") and dom in PMC_VALU_INSTS_SCALE50:
        rate = PMC_VALU_INSTS_SCALE50[dom] / (stage_avg[dom] * 1e6) / SIMDS       # wave instructions per ns and SIMD
        out["valu"] = {"kernel": kernel_of[dom], "instructions": PMC_VALU_INSTS_SCALE50[dom], "per_ns_simd": rate,
                       "sustained_per_ns_simd": VALU_SUSTAINED_PER_NS_SIMD, "frac": rate / VALU_SUSTAINED_PER_NS_SIMD}
    if not args.no_class_step and args.geometry == "default":
        out["class_step_ms"] = class_step_ms(shapes, grad_sets, dev, args.steps, args.warmup)
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
