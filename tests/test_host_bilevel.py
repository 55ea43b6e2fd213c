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


def test_sub_module_forwards_match_the_float64_restatement():
    """Mamba3ScanBlock.forward and MiniGRU.forward, the utilities of the reference's module for callers outside the
    optimizer (mamba3_peer_metanet.py:90-160, 178-192): the block against tests/ref_fp64.scan_block, written from the
    same lines with every step spelled out, in float64 with a carried state and with gradients reaching the weights;
    the cell against its formula."""
    import ref_fp64
    from grokking_optimizers.mamba3_peer_metanet import Mamba3ScanBlock, MiniGRU
    torch.manual_seed(3)
    for kw in (dict(), dict(d_model=4, d_state=6, expand=3)):
        blk = Mamba3ScanBlock(**kw).double()
        with torch.no_grad():
            blk.rope_freq.mul_(20.0)                  # visible rotations
        x = torch.randn(37, blk.d_model, dtype=torch.float64)
        h0 = torch.randn(blk.d_inner, blk.d_state, dtype=torch.float64) * 0.3
        out, hN = blk(x, h0)
        w9 = [t.detach() for t in (blk.in_proj.weight, blk.dt_proj.weight, blk.dt_proj.bias, blk.B_proj.weight, blk.C_proj.weight,
                                   blk.A_log, blk.D, blk.rope_freq, blk.out_proj.weight)]
        want, wantN = ref_fp64.scan_block(x, w9, h0)
        assert out.shape == (37, blk.d_model) and hN.shape == h0.shape
        assert torch.allclose(out, want, rtol=1e-10, atol=1e-12) and torch.allclose(hN, wantN, rtol=1e-10, atol=1e-12)
        out.sum().backward()
        assert all(p.grad is not None and bool(torch.isfinite(p.grad).all()) for p in blk.parameters())
        empty, h_same = blk(x[:0], h0)
        assert empty.shape == (0, blk.d_model) and torch.equal(h_same, h0)
        zero_start, _ = blk(x)
        want0, _ = ref_fp64.scan_block(x, w9, torch.zeros_like(h0))
        assert torch.allclose(zero_start, want0, rtol=1e-10, atol=1e-12)
    cell = MiniGRU(6, 3).double()
    x, h = torch.randn(11, 6, dtype=torch.float64), torch.randn(11, 3, dtype=torch.float64)
    xh = torch.cat([x, h], -1)
    z = torch.sigmoid(xh @ cell.W_z.weight.T + cell.W_z.bias)
    r = torch.sigmoid(xh @ cell.W_r.weight.T + cell.W_r.bias)
    cand = torch.tanh(torch.cat([x, r * h], -1) @ cell.W_h.weight.T + cell.W_h.bias)
    assert torch.allclose(cell(x, h), (1 - z) * h + z * cand, rtol=1e-12, atol=1e-14)


def test_reference_names_for_the_device_bilevel_path():
    mn = Mamba3PEERMetaNet()
    assert mn.has_cuda_bilevel is False                # parameters on the CPU: no device kernels can serve it
    assert callable(mn.forward_for_bilevel_cuda)
