"""Divide-factor policy (ya_fsdp/_collectives.py:221-272): hand-derived table,
the oracle's restatement, the package's mirror, and the upstream twin that
ships in the installed torch (same loop, different signature)."""

import pytest
import torch

from oracle import torch_ops
from yafsdp_amd import LogicalShardGroup, MixedPrecisionPolicy
from yafsdp_amd._collectives import _get_gradient_divide_factors

# (reduce dtype, force_sum, W) -> (pre, post, op); derived by hand from the rules
TABLE = {
    (torch.bfloat16, False, 1): (None, None, "SUM"),
    (torch.bfloat16, False, 8): (None, None, "AVG"),
    (torch.float32, False, 64): (None, None, "AVG"),
    (torch.float32, False, 256): (None, None, "AVG"),
    (torch.bfloat16, True, 1): (None, 1.0, "SUM"),
    (torch.bfloat16, True, 8): (None, 8.0, "SUM"),
    (torch.float32, True, 64): (None, 64.0, "SUM"),
    (torch.float32, True, 256): (None, 256.0, "SUM"),
    (torch.float16, False, 1): (1, 1.0, "SUM"),
    (torch.float16, False, 8): (4, 2.0, "SUM"),
    (torch.float16, True, 64): (8, 8.0, "SUM"),
    (torch.float16, False, 256): (16, 16.0, "SUM"),
    (torch.float16, False, 2): (2, 1.0, "SUM"),
    (torch.float16, False, 6): (4, 1.5, "SUM"),  # the loop doubles once past the last divisor
}


@pytest.mark.parametrize("key", list(TABLE))
def test_table(key):
    dtype, force_sum, w = key
    want = TABLE[key]
    got_oracle = torch_ops.get_gradient_divide_factors(w, dtype, None, force_sum)
    got_pkg = _get_gradient_divide_factors(LogicalShardGroup(w, 0), dtype, None, force_sum)
    assert got_oracle[:3] == want
    assert got_pkg[:3] == want


def test_custom_factor():
    g = LogicalShardGroup(8, 0)
    assert _get_gradient_divide_factors(g, torch.bfloat16, 8.0, False)[:3] == (None, None, "AVG")
    pre, post, op, premul = _get_gradient_divide_factors(g, torch.bfloat16, 5.0, False)
    assert (pre, post, op) == (None, None, "PREMUL_SUM") and premul == 1 / 5.0
    assert _get_gradient_divide_factors(g, torch.float32, 5.0, True)[:3] == (None, 5.0, "SUM")
    assert torch_ops.get_gradient_divide_factors(8, torch.float32, 5.0, True)[:3] == (None, 5.0, "SUM")
    # a YCCL handle forces sum reduction (:228-230)
    assert torch_ops.get_gradient_divide_factors(8, torch.bfloat16, None, False, has_yccl_handle=True)[:3] == (None, 8.0, "SUM")


@pytest.mark.parametrize("w", [1, 2, 3, 6, 8, 12, 64, 100, 256, 1024])
def test_fp16_split_matches_upstream_twin(w):
    """torch/distributed/fsdp/_fully_shard/_fsdp_collectives.py holds the loop
    this policy was forked from; for the overflow-risk branch both must agree."""
    try:
        from torch.distributed.fsdp._fully_shard._fsdp_collectives import _get_gradient_divide_factors as upstream
    except Exception:
        pytest.skip("upstream twin not importable")
    import inspect

    params = list(inspect.signature(upstream).parameters)

    class G:
        def size(self):
            return w

    kwargs = {}
    if "device_type" in params:
        kwargs["device_type"] = "cuda"
    try:
        up = upstream(G(), None, torch.float16, **kwargs)
    except TypeError:
        pytest.skip(f"upstream signature changed: {params}")
    pre, post = up[0], up[1]
    got = torch_ops.get_gradient_divide_factors(w, torch.float16, None, False)
    assert (float(got[0]), float(got[1])) == (float(pre), float(post))


def test_div_if_needed_rule_is_strictly_greater_than_one():
    x = torch.tensor([3.0, -6.0])
    for f in (None, 0.0, 0.5, 1.0):
        y = x.clone()
        torch_ops.div_if_needed(y, f)
        assert torch.equal(y, x)  # upstream uses != 1; the reference skips anything <= 1 (:271)
    y = x.clone()
    torch_ops.div_if_needed(y, 3.0)
    assert torch.equal(y, torch.tensor([1.0, -2.0]))


def test_mixed_precision_policy_validation():
    MixedPrecisionPolicy(reduce_dtype=torch.bfloat16, bit32_acc_for_bit16_reduce_scatter=True)
    with pytest.raises(ValueError, match="bfloat16"):
        MixedPrecisionPolicy(reduce_dtype=torch.float32, bit32_acc_for_bit16_reduce_scatter=True)
    with pytest.raises(ValueError):
        LogicalShardGroup(4, 4)
