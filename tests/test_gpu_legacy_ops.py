"""The flat-buffer ops of the legacy ``YaFSDP`` class (ya_fsdp/ya_fsdp.py,
ya_fsdp/meta_param.py) are the same kernels under other names: each is run
through the C ABI entry point that replaces it and compared bit for bit with
the reference's torch op on CPU."""

import pytest
import torch

from oracle import torch_ops

from helpers import assert_bits_equal, mixed_values
from yafsdp_amd._layout import make_layout

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def nat():
    from yafsdp_amd import _native

    return _native


@pytest.mark.parametrize("yccl_padding", [False, True])
@pytest.mark.parametrize("world_size,rank", [(1, 0), (4, 3), (7, 2)])
def test_flatten_and_shard(nat, world_size, rank, yccl_padding):
    """ya_fsdp/ya_fsdp.py:836-866 = the ragged layout with alignment 8 (YCCL padding) or 1, a gather into the
    flat buffer with zeroed pad lanes, and a copy of the rank's chunk."""
    g = torch.Generator().manual_seed(301)
    shapes = [(33, 7), (5,), (128, 64), (1,), (1001,)]
    params = [mixed_values(g, torch.Size(s).numel(), torch.float32).view(s) for s in shapes]
    padded, want = torch_ops.legacy_flatten_and_shard(params, world_size, rank, yccl_padding)
    lay = make_layout([p.numel() for p in params], world_size, 8 if yccl_padding else 1)
    assert lay.padded_unsharded_numel == padded and lay.padded_sharded_numel == want.numel()
    table = nat.TensorTable([p.numel() for p in params], padded, torch.device(DEV))
    flat = torch.full((padded,), 9.0, device=DEV)
    table.gather_in([p.to(DEV).view(-1) for p in params], flat, None, None, zero_pad=True)
    s = lay.padded_sharded_numel
    shard = torch.empty(s, device=DEV)
    nat.flat_copy(shard, flat[rank * s : (rank + 1) * s])
    assert_bits_equal(shard, want, "legacy shard")
    table.close()


def test_bit16_copy_and_grad_buffer_upcast(nat):
    g = torch.Generator().manual_seed(302)
    master = mixed_values(g, 100_003, torch.float32)
    want = torch.zeros(100_003, dtype=torch.bfloat16)
    torch_ops.legacy_bit16_copy(want, master)
    got = torch.zeros(100_003, dtype=torch.bfloat16, device=DEV)
    nat.flat_copy(got, master.to(DEV))
    assert_bits_equal(got, want, "bit16 copy (ya_fsdp.py:519-520)")
    grad16 = mixed_values(g, 70_001, torch.bfloat16, 1e-3)
    want32 = torch.zeros(70_001)
    torch_ops.legacy_grad_buffer_upcast(want32, grad16)
    got32 = torch.zeros(70_001, device=DEV)
    nat.flat_copy(got32, grad16.to(DEV))
    assert_bits_equal(got32, want32, "grad buffer upcast (ya_fsdp.py:945-954)")


@pytest.mark.parametrize("target_dtype", [torch.bfloat16, torch.float32])
def test_accumulate_into_fp32_grad_shard(nat, target_dtype):
    g = torch.Generator().manual_seed(303)
    shard = mixed_values(g, 50_001, torch.float32, 1e-4)
    target = mixed_values(g, 50_001, target_dtype, 1e-3).flip(0)
    want = shard.clone()
    torch_ops.legacy_accumulate_shard(want, target)
    got = shard.to(DEV)
    nat.post_reduce(got, target.to(DEV), None, True)
    assert_bits_equal(got, want, "fp32_grad_shard.add_ (ya_fsdp.py:991-992)")


@pytest.mark.parametrize("world_size,steps", [(1, 1), (8, 1), (8, 4), (6, 1), (3, 5)])
def test_final_divide(nat, world_size, steps):
    g = torch.Generator().manual_seed(304)
    grad = mixed_values(g, 60_007, torch.float32, 1e-2)
    want = grad.clone()
    torch_ops.legacy_final_divide(want, world_size, steps)
    got = grad.to(DEV)
    nat.flat_div(got, float(world_size * steps))
    assert_bits_equal(got, want, "grad.div_(W * accumulation steps) (ya_fsdp.py:499-501)")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_narrow_backward(nat, dtype):
    """ya_fsdp/meta_param.py:16-27 at an odd offset of the gradient buffer: first copy_, then add_."""
    g = torch.Generator().manual_seed(305)
    buf = mixed_values(g, 10_000, dtype, 1e-3)
    grads = [mixed_values(g, 33 * 77, dtype, 1e-3).view(33, 77) for _ in range(2)]
    want, got = buf.clone(), buf.to(DEV)
    off = 1237
    for i, gr in enumerate(grads):
        torch_ops.legacy_narrow_backward(want, off, gr, accumulate=i > 0)
        view = got.narrow(0, off, gr.numel())
        if i == 0:
            nat.flat_copy(view, gr.to(DEV).view(-1))
        else:
            nat.post_reduce(view, gr.to(DEV).view(-1), None, True)
    assert_bits_equal(got, want, "Narrow.backward")
