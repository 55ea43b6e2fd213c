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
SIMDS = 1024
REPLAY_WAVES_PER_SIMD = 2        # k_replay: eight one-wave workgroups per compute unit (19.8 KB of LDS each)
STAGE_KERNEL_PREFIX = {"scan_output": "k_replay<", "scan_summary": "k_scan<false, false>", "elementwise": "k_elem<"}


def profile_figures():
    """What the rocprofv3 counter runs committed under profiles/ say about the kernels of the default workload, per
    stage: HBM bytes per launch (FETCH_SIZE + WRITE_SIZE, scaled as that file describes), vector-ALU instructions per
    launch, and the instruction rate the part sustains on nothing but independent fp32 instructions.  Read from the
    text summaries at run time, so a figure can never drift from the file it is quoted from; None where a file or a
    row is missing.  These are figures of the profiled build, not measurements of this run: the JSON names the files."""
    out = {"traffic": {}, "valu": {}, "sustained": None, "source": {}}
    pdir = os.path.join(ROOT, "profiles")

    def rows(name):
        try:
            with open(os.path.join(pdir, name)) as f:
                return f.read().splitlines()
        except OSError:
            return []
    for stage, prefix in STAGE_KERNEL_PREFIX.items():
        for line in rows("sg2_step_scale50_pmc_traffic.txt"):
            if line.startswith(prefix):
                cols = line.split()
                out["traffic"][stage] = (float(cols[-2]) + float(cols[-1])) * 1e9        # read_GB + written_GB
        for line in rows("sg2_step_scale50_pmc_sq.txt"):
            if line.startswith(prefix):
                cols = line[40:].split()                                                   # after the (truncated) kernel name
                out["valu"][stage] = float(cols[1])                                        # us/launch, INSTS_VALU, ...
    best, by_waves = 0.0, {}
    for line in rows("valu_probe_mi355x.txt"):
        cols = line.split()
        if len(cols) >= 5 and cols[0] in ("fma", "fmac", "fma_vector_operands", "fma_scalar_operand", "mul", "add", "add_dpp"):
            try:
                best = max(best, float(cols[3]))
                by_waves.setdefault(int(cols[1]), {})[cols[0]] = float(cols[3])
            except ValueError:
                pass
    out["sustained"] = best or None
    out["sustained_by_waves"] = by_waves        # waves per SIMD -> {instruction kind: instructions per ns and SIMD}
    out["source"] = {"traffic": "profiles/sg2_step_scale50_pmc_traffic.txt", "valu": "profiles/sg2_step_scale50_pmc_sq.txt",
                     "sustained": "profiles/valu_probe_mi355x.txt"}
    return out


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
    elif workload in ("bilevel", "bilevel50"):
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
    """Issue rate of plain fp32 vector instructions (sg_probe_valu of tests/probe/libsg_probe.so, a measurement aid built beside the
    tests, not part of the product library): wave64 instructions per nanosecond and SIMD for
    fma / mul / add / DPP-add streams with every SIMD of the chip busy, by resident waves per SIMD; and the shader
    clock the part holds meanwhile (ticks of the in-kernel clock per nanosecond of the launch)."""
    import ctypes as C
    import torch
    path = os.path.join(ROOT, "tests", "probe", "libsg_probe.so")
    if not os.path.exists(path):
        raise SystemExit("the probe library is not built (%s): make -C tests/probe, or __graft_entry__.build()" % path)
    L = C.CDLL(path)
    L.sg_probe_last_error.restype = C.c_char_p
    L.sg_probe_workspace_bytes.restype = C.c_size_t
    L.sg_probe_valu.argtypes = [C.c_int] * 4 + [C.POINTER(C.c_float), C.POINTER(C.c_double), C.POINTER(C.c_double),
                                                C.c_void_p, C.c_size_t, C.c_void_p]
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    ws = torch.empty(L.sg_probe_workspace_bytes(cus, 8), dtype=torch.uint8, device=dev)
    rows, best = [], 0.0
    for ncu in (cus,):
        for op, name in enumerate(("fma", "mul", "add", "add_dpp", "mfma_32x32x16_bf16", "mfma_32x32x16_bf16_random_operands",
                                   "mfma_32x32x1_f32", "mfma_32x32x1_f32_then_8_fma", "mfma_4x4x1_f32", "fmac", "fma_vector_operands",
                                   "fma_scalar_operand")):
            matrix = 4 <= op <= 8
            for w in ((1, 2) if matrix else (1, 2, 3, 4, 8)):
                ms, ticks, instr = C.c_float(), C.c_double(), C.c_double()
                if L.sg_probe_valu(op, ncu, w, 2000, C.byref(ms), C.byref(ticks), C.byref(instr), ws.data_ptr(), ws.numel(),
                                   torch.cuda.current_stream().cuda_stream) != 0:
                    raise RuntimeError(L.sg_probe_last_error().decode())
                rate = instr.value * w / (ms.value * 1e6)            # per SIMD: w waves share one
                rows.append({"op": name, "cus": ncu, "waves_per_simd": w, "ms": round(ms.value, 4),
                             "instr_per_ns_per_simd": round(rate, 4),
                             "clock_ticks_per_instr_per_simd": round(ticks.value / instr.value / w, 3),
                             "clock_ticks_per_ns": round(ticks.value / (ms.value * 1e6), 3)})
                if matrix:       # flop per matrix instruction (the vector fma of the mixed stream are not counted)
                    rows[-1]["chip_tflops"] = round(rate * (32768, 32768, 4096, 4096, 512)[op - 4] * 4 * ncu / 1e3, 1)
                elif ncu == cus:
                    best = max(best, rate)
    return {"metric": "secondary: valu-probe", "value": best, "unit": "wave64 instructions/ns/SIMD (whole chip, best case)",
            "n_gpus": 1, "steps": 1, "warmup": 1, "ms_per_step": None, "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "f32", "data": "synthetic",
            "config": {"workload": "plain fp32 VALU instruction streams, 8 independent accumulators per lane, %d CUs" % cus},
            "rows": rows}


def make_v2_step(st, weights, D, boundary="ops"):
    """step(grads, sharps, per_tensor, shared) over the tensors of `st`: the reference's own entry point of the torch
    extension (51 arguments), or the bare C-ABI call."""
    from grokking_optimizers import _cabi
    if boundary == "cabi":
        return _cabi.Sg2Step(weights, st["params"], st["eas"], st["easqs"], st["mus"], st["grus"], st["mf"], st["mb"], st["counts"], dims=D)
    from grokking_optimizers import _ops

    def step(grads, sharps_, per_tensor, sh):
        col = lambda k: [float(sc[k]) for sc in per_tensor]
        _ops.supergrok2_mamba_peer_batched_step(
            st["params"], grads, sharps_, st["eas"], st["easqs"], st["mus"], st["grus"], st["mf"], st["mb"], *weights,
            col("alpha"), col("lamb_eff"), col("beta1"), col("bc1"), col("bc2"), sh["rescale"], sh["beta2"], sh["lr"],
            sh["wd_eff"], sh["eps"], D["d_model"], D["d_state"], D["d_inner"], D["gru_hidden"], D["num_heads"],
            D["pk_dim"], D["expert_hidden"], D["num_experts"], st["counts"])
    return step


def time_v2(step, P, grad_sets, sharps, steps, warmup, t0_step=0):
    """W untimed calls, then exactly `steps` calls between two device synchronisations; per-stage times from HIP events
    recorded on the step's stream.  Returns (seconds of the timed region, average stage ms, step counter)."""
    import torch
    from grokking_optimizers import _cabi
    from workloads import per_tensor_scalars, shared_scalars
    shared = shared_scalars()
    t = t0_step
    for _ in range(warmup):
        t += 1
        step(grad_sets[t & 1], sharps, per_tensor_scalars(P, t), shared)
    torch.cuda.synchronize()
    scal = [per_tensor_scalars(P, t + k + 1) for k in range(steps)]
    _cabi.profile_enable(True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(steps):
        t += 1
        step(grad_sets[t & 1], sharps, scal[k], shared)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    stage_ms, calls = _cabi.profile_read()
    _cabi.profile_enable(False)
    assert calls == min(steps, 256)
    return elapsed, {k: v / calls for k, v in stage_ms.items()}, t


def finite_state(st):
    import torch
    return all(bool(torch.isfinite(x).all()) for lst in (st["params"], st["eas"], st["grus"]) for x in lst)


def v2_variants(shapes, st, grad_sets, D, dev, steps=8, warmup=2):
    """The headline set again under the inputs the headline figure is friendliest to, so that its dependence on them is
    measured in the same run: a populated sharpness cache; the optimizer's own initial meta-net; gradients large enough
    that no tile of the scan qualifies for a polynomial form (the general recurrence); and routing spread over many
    experts (per-lane gathers of the expert records in the per-element kernel instead of broadcasts)."""
    import torch
    import workloads as wl
    P, total = len(shapes), sum(p.numel() for p in st["params"])
    out = {}

    def run(name, weights, grads, sharps, note, fresh_gru=None):
        for lst in (st["eas"], st["easqs"], st["mus"], st["mf"], st["mb"]):
            for x in lst:
                x.zero_()
        for x, p0 in zip(st["params"], fresh_params):
            x.copy_(p0)
        for i, x in enumerate(st["grus"]):
            x.zero_() if fresh_gru is None else x.copy_(fresh_gru[i])
        st["counts"].zero_()
        el, stage, _ = time_v2(make_v2_step(st, weights, D), P, grads, sharps, steps, warmup)
        assert finite_state(st), name
        counts = st["counts"].cpu()
        out[name] = {"ms_per_step": 1e3 * el / steps, "elements_per_s": total * steps / el, "stage_ms": stage,
                     "experts_used": int((counts > 0).sum()), "steps": steps, "what": note}
    fresh_params = [p.clone() for p in st["params"]]
    zeros = [torch.zeros_like(p) for p in st["params"]]
    bench_w = [w.to(dev) for w in wl.meta_weights(7, D)]
    run("sharpness", bench_w, grad_sets, [(g.abs() * 0.5).contiguous() for g in grad_sets[1]],
        "sharpness cache populated (|g|/2 of the other gradient set): gather into sorted order, sharpness terms in the projections")
    run("module_weights", [w.to(dev) for w in wl.module_weights(0)], grad_sets, zeros,
        "meta-net as Mamba3PEERMetaNet() initialises it (A_log = log(1..16)): slower contraction, fewer blocks on the product forms")
    big = [[(torch.sign(g) * (g.abs() * 100.0 + 0.5)).contiguous() for g in gs] for gs in grad_sets]
    run("general_path", bench_w, big, zeros,
        "every |g| >= 0.5: no tile takes the Taylor / lane-polynomial / product forms, every block runs the general recurrence")
    del big
    # routing: queries driven by a random GRU state through amplified h columns of the query matrices
    spread_w = [w.clone() for w in bench_w]
    spread_w[26][:, :, :D["gru_hidden"]] *= 30.0
    gen = torch.Generator().manual_seed(11)
    gru0 = [torch.randn(p.numel(), D["gru_hidden"], generator=gen).to(dev) for p in st["params"]]
    run("spread_routing", spread_w, grad_sets, zeros,
        "query rows amplified x30 on a random GRU state: elements of a wave pick different experts", fresh_gru=gru0)
    return out


def muon_precision(dev):
    """One wide and one tall matrix of the Muon workload: this library's step (bf16 Newton-Schulz on the Gram matrix of
    the smaller side, fp32 accumulation) against the reference's arithmetic (fp32 iteration on X X^T, csrc/ops.cpp:704-727
    of the reference) restated with torch fp32 products on the device.  Fraction of updated bf16 parameters that differ
    from the fp32-iteration result rounded to bf16 by more than one bf16 spacing, the fraction that round differently at
    all, and the largest deviation in units of the largest entry of the update (one bf16 spacing of a parameter of size
    0.06 is already larger than the largest update entry, so this is about 1.5 whenever some entry rounds the other way)."""
    import torch
    from grokking_optimizers import _ops
    gen = torch.Generator().manual_seed(0)
    res = {}
    prev = torch.backends.cuda.matmul.allow_tf32
    torch.backends.cuda.matmul.allow_tf32 = False
    try:
        for name, shape in (("wide_1024x4096", (1024, 4096)), ("tall_4096x1024", (4096, 1024))):
            p = (torch.randn(*shape, generator=gen) * 0.02).to(torch.bfloat16).to(dev)
            g = (torch.randn(*shape, generator=gen) * 1e-3).to(torch.bfloat16).to(dev)
            buf = torch.zeros(shape, device=dev)
            p_new = p.clone()
            _ops.muon_fused_step([p_new], [g], [buf], 0.95, 0.02, 1.0, 5)
            X = g.float()
            X = X / (X.norm() + 1e-7)
            if shape[0] > shape[1]:
                X = X.T                       # X X^T of the tall form and X^T X of its transpose give the same iteration
            for _ in range(5):
                A = X @ X.T
                AX = A @ X
                X = 3.4445 * X + (-4.7750) * AX + 2.0315 * (A @ AX)
            if shape[0] > shape[1]:
                X = X.T
            want = ((p.float() - 0.2 * 0.02 * X) * (1.0 - 0.02 * 1.0)).to(torch.bfloat16)
            ulp = torch.maximum(want.float().abs(), torch.tensor(1e-30, device=dev)).log2().floor().exp2() * 2.0 ** -7
            diff = (p_new.float() - want.float()).abs()
            res[name] = {"frac_beyond_one_bf16_ulp": float((diff > ulp * 1.0001).float().mean()),
                         "frac_rounded_differently": float((diff > 0).float().mean()),
                         "largest_deviation_over_largest_update_entry": float(diff.max() / (0.2 * 0.02 * X.abs().max()))}
    finally:
        torch.backends.cuda.matmul.allow_tf32 = prev
    return res


def secondary_configs(dev, steps=20, warmup=3):
    """The other measured configurations, each timed in this run: Grokfast and SuperGrok v1.5 on the 14-tensor set, the
    SuperGrok v2 step on the 14-tensor set, Muon on its 24 bf16 matrices (algorithmic and executed MFMA fraction), the
    bilevel meta-gradient pass of v2 on the 14-tensor and on the 25 M-element set and the five other fused steps on the
    25 M-element set."""
    import torch
    from grokking_optimizers import _ops
    out = {}
    for name, workload in (("config1_grokfast", "grokfast"), ("config2_supergrok15", "sg15"), ("config5_muon", "muon"),
                           ("bilevel_pass_shared14", "bilevel"), ("bilevel_pass_scale50", "bilevel50"), ("grokadamw_scale50", "grokadamw"), ("neuralgrok_scale50", "neuralgrok"),
                           ("prodigy_scale50", "prodigy"), ("lion_scale50", "lion"), ("supergrok11_scale50", "sg11")):
        W = build_step(workload, _ops, dev)
        n_steps, n_warm = (5, 1) if workload == "bilevel50" else (steps, warmup)       # 0.15 s a pass
        for _ in range(n_warm):
            W["step"]()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n_steps):
            W["step"]()
        torch.cuda.synchronize()
        el = (time.perf_counter() - t0) / n_steps
        r = {"workload": W["name"], "ms_per_step": 1e3 * el, "value": W["units"] / el, "unit": W["unit"], "dtype": W["dtype"], "steps": n_steps}
        if W["bound"] == "mfma":
            r["roofline"] = {"bound": "mfma", "peak": W["peak"], "unit": "TFLOP/s", "achieved": W["units"] / el / 1e12,
                             "frac": W["units"] / el / 1e12 / W["peak"], "achieved_executed": W["executed"] / el / 1e12,
                             "frac_executed": W["executed"] / el / 1e12 / W["peak"]}
            r["precision"] = muon_precision(dev)
        else:
            bpe = W["bytes_per_elem"]
            r["roofline"] = {"bound": "hbm", "peak": W["peak"], "unit": "GB/s", "achieved": bpe * W["units"] / el / 1e9,
                             "frac": bpe * W["units"] / el / 1e9 / W["peak"], "bytes_per_element": bpe}
        out[name] = r
        del W
    shapes, st, grad_sets, sharps, weights, D = build_workload("shared14", dev)
    total = sum(p.numel() for p in st["params"])
    el, stage, _ = time_v2(make_v2_step(st, weights, D), len(shapes), grad_sets, sharps, steps, warmup)
    out["config3_supergrok2_shared14"] = {
        "workload": "SuperGrok v2 full step, 14 tensors, %d elements" % total, "ms_per_step": 1e3 * el / steps, "value": total * steps / el,
        "unit": "elements/s", "dtype": "f32", "steps": steps, "stage_ms": stage,
        "roofline": {"bound": "hbm", "peak": HBM_PEAK_GBS, "unit": "GB/s", "achieved": BYTES_PER_ELEMENT * total * steps / el / 1e9,
                     "frac": BYTES_PER_ELEMENT * total * steps / el / 1e9 / HBM_PEAK_GBS, "bytes_per_element": BYTES_PER_ELEMENT},
        "graph_replay_ms_per_step": graph_replay_ms(st, weights, D, grad_sets, sharps, steps)}
    return out


def graph_replay_ms(st, weights, D, grad_sets, sharps, steps):
    """The same step recorded once into a HIP graph (the call copies nothing from the host and blocks nowhere) and
    replayed: what the ~30 launches of a step cost when the host does not issue them one by one.  A replay repeats
    the recorded scalars; the state keeps evolving."""
    import torch
    from workloads import per_tensor_scalars, shared_scalars
    step = make_v2_step(st, weights, D, boundary="cabi")
    P = len(st["params"])
    step(grad_sets[0], sharps, per_tensor_scalars(P, 1), shared_scalars())       # eager first
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step(grad_sets[1], sharps, per_tensor_scalars(P, 2), shared_scalars())
    graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        graph.replay()
    torch.cuda.synchronize()
    return 1e3 * (time.perf_counter() - t0) / steps


def aten_loop_baseline(max_elems=16384, budget_s=10.0):
    """The per-timestep ATen restatement of the reference's CPU path (oracle/aten_loop.py) on the smallest tensors of the
    50-tensor set, as many as fit the time budget; elements per second with the thread count."""
    import torch
    import workloads as wl
    from oracle import aten_loop
    shapes = wl.scale50_shapes()
    W = wl.meta_weights(7)
    D = wl.DEFAULT_DIMS
    done, t0 = 0, time.perf_counter()
    used = []
    for i, sh in enumerate(shapes):
        n = wl.numel(sh)
        if n > max_elems or (used and time.perf_counter() - t0 > budget_s):
            break
        g = wl.make_grads([sh], seed=1 + i)[0].reshape(-1)
        st = dict(param=wl.make_params([sh], seed=i)[0].reshape(-1), exp_avg=torch.zeros(n), exp_avg_sq=torch.zeros(n), mu=torch.zeros(n),
                  gru=torch.zeros(n, D["gru_hidden"]), mamba_fwd=torch.zeros(D["d_inner"], D["d_state"]), mamba_bwd=torch.zeros(D["d_inner"], D["d_state"]))
        sc = dict(wl.per_tensor_scalars(i + 1, 1)[i], **wl.shared_scalars())
        sc["lamb_eff"] = sc.get("lamb_eff", 0.0)
        with torch.no_grad():
            aten_loop.step(W, st, g, torch.zeros_like(g), sc, D)
        done += n
        used.append(i)
    dt = time.perf_counter() - t0
    return {"value": done / dt, "unit": "elements/s", "threads": torch.get_num_threads(), "host_cpus": os.cpu_count(),
            "sample": "tensors %d..%d of the 50-tensor set (%d elements, each at most %d), 1 step, per-timestep ATen loop in fp32, %.1f s; "
                      "the 25 M element set would take about %.1f hours at this rate" % (used[0], used[-1], done, max_elems, dt, 25010032 / (done / dt) / 3600)}


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
    ap.add_argument("--workload", default="scale50", choices=["scale50", "shared14", "grokfast", "sg15", "muon", "grokadamw", "neuralgrok", "prodigy", "lion", "sg11", "bilevel", "bilevel50", "valu-probe"],
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
    ap.add_argument("--no-extras", action="store_true", help="default workload: skip the variants / secondary configurations / ATen-loop baseline that ride on the same run")
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
    step = make_v2_step(st, weights, D, args.boundary)
    if args.copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    elapsed, stage_avg, _ = time_v2(step, len(shapes), grad_sets, sharps, args.steps, args.warmup)
    assert finite_state(st), "non-finite state after the timed steps"

    ms_per_step = 1e3 * elapsed / args.steps
    value = total * args.steps / elapsed
    dom = max(stage_avg, key=stage_avg.get)
    kernel_of = {"sort": "k_keys + 4 x (k_hist, k_spine_*, k_scatter)", "scan_summary": "k_scan<false>",
                 "chunk_prefix": "k_chunk_prefix", "scan_output": "k_replay", "elementwise": "k_elem<false>"}
    achieved = BYTES_PER_ELEMENT * total / (stage_avg[dom] * 1e-3) / 1e9
    default_workload = (args.workload, args.weights, args.geometry, args.sharpness) == ("scale50", "bench", "default", False)
    prof = profile_figures() if default_workload else {"traffic": {}, "valu": {}, "sustained": None, "source": {}}
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
                     "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS, "traffic": prof["traffic"].get(dom),
                     "traffic_source": prof["source"].get("traffic") if prof["traffic"].get(dom) is not None else None,
                     "kernel_ms": stage_avg[dom]},
        "step_hbm_frac": BYTES_PER_ELEMENT * value / 1e9 / HBM_PEAK_GBS,
        "stage_ms": stage_avg,
    }
    if prof["valu"].get(dom) is not None and prof["sustained"]:
        # instructions per launch as counted in the profiled run (the file is named) over THIS run's kernel time
        rate = prof["valu"][dom] / (stage_avg[dom] * 1e6) / SIMDS       # wave instructions per ns and SIMD
        out["valu"] = {"kernel": kernel_of[dom], "instructions": prof["valu"][dom], "instructions_source": prof["source"]["valu"],
                       "per_ns_simd": rate, "sustained_per_ns_simd": prof["sustained"], "sustained_source": prof["source"]["sustained"],
                       "frac": rate / prof["sustained"]}
        # the yardstick that fits the kernel: it keeps REPLAY_WAVES_PER_SIMD waves on a SIMD and issues mostly fma
        at = prof.get("sustained_by_waves", {}).get(REPLAY_WAVES_PER_SIMD)
        if dom == "scan_output" and at:
            # fma_vector_operands: every operand in a vector register, as in the recurrence of the replay;
            # fma / fma_scalar_operand: one operand in a scalar register, as where weights are wave-uniform
            out["valu"].update({"waves_per_simd": REPLAY_WAVES_PER_SIMD, "sustained_at_that_occupancy": at})
            for kind in ("fma_vector_operands", "fma_scalar_operand"):
                if at.get(kind):
                    out["valu"]["frac_of_%s_rate_at_that_occupancy" % kind] = rate / at[kind]
    if not args.no_class_step and args.geometry == "default":
        out["class_step_ms"] = class_step_ms(shapes, grad_sets, dev, args.steps, args.warmup)
    if default_workload and not args.no_extras:
        # everything below is timed in this same run, after the headline's timed region
        out["variants"] = v2_variants(shapes, st, grad_sets, D, dev)
        del st, grad_sets, sharps, step
        torch.cuda.empty_cache()
        out["secondary"] = secondary_configs(dev)
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
        if default_workload and not args.no_extras:
            out["cpu_baseline"]["aten_loop"] = aten_loop_baseline()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
