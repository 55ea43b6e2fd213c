"""bench.py's command line, without a GPU: more than one GPU is refused with a message, and the workload builder
drives the reference-shaped operator interface on CPU tensors (a recording stand-in, no arithmetic)."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0 and "one GPU" in (r.stdout + r.stderr)


def test_every_secondary_workload_calls_its_operator():
    sys.path.insert(0, ROOT)
    import bench

    class Recorder:
        def __init__(self):
            self.calls = []

        def __getattr__(self, name):
            def f(*a):
                self.calls.append((name, len(a)))
                return 1e-6
            return f

    want = {"grokfast": ("grokfast_adamw_fused_step", 13), "sg15": ("supergrok15_fused_step", 23), "muon": ("muon_fused_step", 7),
            "grokadamw": ("grokadamw_fused_step", 14), "neuralgrok": ("neuralgrok_fused_step", 18), "prodigy": ("prodigy_fused_step", 13),
            "lion": ("lion_fused_step", 7), "sg11": ("supergrok11_fused_step", 23)}
    for w, (name, nargs) in want.items():
        rec = Recorder()
        W = bench.build_step(w, rec, "cpu", limit=100_000)
        W["step"]()
        assert rec.calls == [(name, nargs)], (w, rec.calls)
        assert W["units"] > 0 and W["bound"] in ("hbm", "mfma")
