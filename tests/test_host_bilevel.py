"""Host-side bookkeeping of the bilevel pass (no GPU): the parameter orders the two flat gradient tensors are cut by
add up to the sizes the C ABI declares, and the header's layout comments name the same shapes."""
import re
import os

import torch

from grokking_optimizers import Mamba3PEERMetaNet, _bilevel, _cabi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _header_define(name):
    text = open(os.path.join(ROOT, "include", "sg_abi.h")).read()
    return int(re.search(r"#define\s+%s\s+(\d+)" % name, text).group(1))


def test_gradient_block_sizes_match_the_parameter_lists():
    mn = Mamba3PEERMetaNet()
    scan = _bilevel.scan_parameters(mn)
    elem = _bilevel.elem_parameters(mn)
    assert len(scan) == 20 and sum(p.numel() for p in scan) == _cabi.SG2_SCAN_GRAD_FLOATS == _header_define("SG2_SCAN_GRAD_FLOATS")
    assert sum(p.numel() for p in elem) == _cabi.SG2_ELEM_GRAD_FLOATS == _header_define("SG2_ELEM_GRAD_FLOATS")
    # together they are every parameter of the meta-net, each exactly once
    ids = [id(p) for p in scan + elem]
    assert len(set(ids)) == len(ids) == len(list(mn.parameters()))
    # the scan list is the first 20 tensors of the fused step's weight order, shape for shape
    flat = mn.flat_weights()
    for p, w in zip(scan, flat[:20]):
        assert tuple(p.shape) == tuple(w.shape)
    # the per-element list follows the rest of that order (queries / keys stacked per head, experts flattened)
    assert [tuple(p.shape) for p in elem[:6]] == [tuple(w.shape) for w in flat[20:26]]
    assert sum(p.numel() for p in elem[6:10]) == flat[26].numel() and sum(p.numel() for p in elem[10:14]) == flat[27].numel()
    assert sum(p.numel() for p in elem[14:18]) == flat[28].numel()
    assert [p.numel() for p in elem[18:]] == [w.numel() for w in flat[29:]]


def test_split_flat_hands_out_views():
    params = [torch.zeros(3, 2), torch.zeros(4), torch.zeros(2, 1, 2)]
    flat = torch.arange(14, dtype=torch.float32)
    parts = _bilevel.split_flat(flat, params)
    assert [tuple(p.shape) for p in parts] == [(3, 2), (4,), (2, 1, 2)]
    assert parts[1].data_ptr() == flat[6:].data_ptr() and float(parts[2][1, 0, 1]) == 13.0


def test_bilevel_needs_gpu_tensors():
    mn = Mamba3PEERMetaNet()
    g = [torch.randn(10)]
    try:
        _bilevel.accumulate_meta_gradients(mn, g, [torch.zeros(10)], [torch.zeros(10, 4)], [None], [None], [torch.ones(10)])
    except RuntimeError as e:
        assert "no CPU path" in str(e)
    else:
        raise AssertionError("a CPU call must fail loudly")
