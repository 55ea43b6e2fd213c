"""Meta-net dimension sets other than the two the kernels are specialised for, shared by the CPU and GPU tests."""
import workloads as wl

D = wl.DEFAULT_DIMS


def dims(**kw):
    d = dict(D, **kw)
    return d


CASES = {
    # what the reference's training harness passes (grokking_race_v2.py:1583 -> :775): everything default but the expert width
    "expert_hidden_4": dims(expert_hidden=4),
    # a small scan block: runs embedded in the (8, 16, 16) geometry
    "small_block": dims(d_model=4, d_state=8, d_inner=8),
    # nothing at its default: d_inner != d_state, 3 GRU units, 2 heads, 5 x 5 sub-keys with fewer experts than pk_dim^2
    # (the index clamp), expert width 7
    "all_odd": dims(d_model=6, d_state=6, d_inner=12, gru_hidden=3, num_heads=2, pk_dim=5, expert_hidden=7, num_experts=23),
    # between the two geometries: embedded in (16, 32, 32); the widest GRU the reference admits
    "medium_block": dims(d_model=12, d_state=24, d_inner=24, gru_hidden=8, num_heads=3, pk_dim=6, expert_hidden=5, num_experts=36),
    # the largest scan block with other routing sizes than the specialised kernel's
    "large_block_other_routing": dims(d_model=16, d_state=32, d_inner=32, gru_hidden=4, num_heads=4, pk_dim=12, expert_hidden=4, num_experts=144),
    # more experts than the count histogram holds in LDS
    "many_experts": dims(num_heads=2, pk_dim=70, expert_hidden=2, num_experts=4900),
}
