"""grokking_optimizers on MI355X: the optimizer classes of peterc04/SuperGrok1.5
(SuperGrok v2, v1.5, v1.1, Grokfast, GrokAdamW, NeuralGrok, Prodigy, Lion,
LookSAM, Muon), with every fused step running
as hand-written HIP (libsg_hip.so) behind the reference's `_ops` extension
surface.  As in the reference (grokking_optimizers/__init__.py:13-20 there),
importing fails unless the compiled extension is present; there is no Python
or CPU fallback.
"""
try:
    from grokking_optimizers import _ops  # noqa: F401
except ImportError as e:  # pragma: no cover
    raise ImportError(
        "grokking_optimizers needs its compiled extension (_ops) and libsg_hip.so; "
        "build them with `python __graft_entry__.py` at the repository root (%s)" % e)

from grokking_optimizers.grokfast import Grokfast
from grokking_optimizers.muon import Muon
from grokking_optimizers.supergrok15 import SuperGrok15, SharpnessMetaNet
from grokking_optimizers.supergrok2 import SuperGrok2
from grokking_optimizers.mamba3_peer_metanet import Mamba3PEERMetaNet, Mamba3ScanBlock, MiniGRU
from grokking_optimizers.supergrok11 import SuperGrok11
from grokking_optimizers.grokadamw import GrokAdamW
from grokking_optimizers.neuralgrok import NeuralGrok
from grokking_optimizers.prodigy import Prodigy
from grokking_optimizers.lion import Lion
from grokking_optimizers.looksam import LookSAM

__version__ = "2.0.0"      # the reference's (grokking_optimizers/__init__.py:11 there)

__all__ = ["Grokfast", "Muon", "SuperGrok15", "SharpnessMetaNet", "SuperGrok2", "Mamba3PEERMetaNet", "Mamba3ScanBlock", "MiniGRU",
           "SuperGrok11", "GrokAdamW", "NeuralGrok", "Prodigy", "Lion", "LookSAM"]
