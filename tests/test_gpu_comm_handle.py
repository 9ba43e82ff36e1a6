"""The communication-handle seam (the reference's duck-typed ``yccl.Handle``:
ya_fsdp/_param_group.py:40-69, 500-519; ya_fsdp/_collectives.py:50-52, 67-70,
112-123, 163-164, 229-230; ya_fsdp/_state.py:517-529, 663-677).

A handle owns the gathered buffer, the all-gather input and the reduce buffer
of a buffer context and performs the two exchanges itself; the buffer path keeps
the copy-in into the handle's input buffer, the reduce copy-in into its reduce
buffer, and the post-divide + accumulation out of the rank's chunk.  The handle
here is a one-GPU stand-in that plays the other logical ranks from data the test
gives it, so the gathered buffer and the reduced chunk are complete and can be
compared with the reference's op sequence on CPU tensors, bit for bit.
"""

import pytest
import torch
import torch.nn as nn

from oracle import torch_ops
from tests.helpers import assert_bits_equal
from tests.test_gpu_param_group import BF16_MP, ODD_SHAPES, CpuGroup, _grads, _params
from yafsdp_amd import FSDPMeshInfo, MixedPrecisionPolicy

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


class LocalHandle:
    """Stand-in for a communication library on one GPU."""

    def __init__(self, world_size, rank):
        self.w, self.r = world_size, rank
        self.ag_inputs, self.ag_outputs, self.rs_buffers = [], [], []
        self.calls = []
        self.peer_ag_inputs = None   # list of W bf16-view tensors (entry r unused): what the peers would send
        self.peer_rs_sum = None      # tensor like the reduce buffer: the sum of the peers' contributions
        self.profiling_events_processed = 0

    def _new(self, numel):
        return torch.full((numel,), float("nan"), dtype=torch.bfloat16, device=DEV)  # the path zero-fills it

    def add_all_gather_input_buffer(self, numel):
        self.ag_inputs.append(self._new(numel))
        return self.ag_inputs[-1]

    def add_all_gather_output_buffer(self, numel):
        self.ag_outputs.append(self._new(numel))
        return self.ag_outputs[-1]

    def add_reduce_scatter_buffer(self, numel):
        self.rs_buffers.append(self._new(numel))
        return self.rs_buffers[-1]

    def all_gather(self, inp, out):
        assert inp.dtype == out.dtype == torch.bfloat16 and out.numel() == self.w * inp.numel()
        self.calls.append(("all_gather", inp.data_ptr(), out.data_ptr(), inp.numel()))
        n = inp.numel()
        for k in range(self.w):
            src = inp if k == self.r else self.peer_ag_inputs[k]
            out[k * n : (k + 1) * n].copy_(src)

    def reduce_scatter(self, buf):
        assert buf.dtype == torch.bfloat16
        self.calls.append(("reduce_scatter", buf.data_ptr(), buf.numel()))
        n = buf.numel() // self.w
        chunk = buf[self.r * n : (self.r + 1) * n]
        if self.peer_rs_sum is not None:
            chunk.add_(self.peer_rs_sum[self.r * n : (self.r + 1) * n])  # a sum, rounded to the buffer's dtype

    def process_profiling_events(self):
        self.profiling_events_processed += 1


def _group_with_handle(shapes, w, r, align, mp, handle, master_dtype=torch.float32):
    from yafsdp_amd._param_group import YaFSDPParamGroup, init_shared_state

    cpu_params = _params(shapes, master_dtype, 1)
    dev_params = [p.to(DEV).requires_grad_(True) for p in cpu_params]
    group = YaFSDPParamGroup(dev_params, FSDPMeshInfo(w, r), DEV, mp, align)
    init_shared_state([group], DEV, yccl_handle=handle)
    return group, cpu_params


@pytest.mark.parametrize("w,r", [(4, 2), (2, 0)])
def test_handle_owns_buffers_and_runs_both_exchanges(w, r):
    align = 8
    handle = LocalHandle(w, r)
    group, cpu_params = _group_with_handle(ODD_SHAPES, w, r, align, BF16_MP, handle)
    refs = [CpuGroup(cpu_params, w, k, align, BF16_MP) for k in range(w)]
    ref = refs[r]
    # the three buffers are the handle's, zero-filled by the path
    assert group.data_buffer_ctx.buffers[None].data_ptr() == handle.ag_outputs[0].data_ptr()
    assert group.grad_buffer_ctx.buffers[None].data_ptr() == handle.rs_buffers[0].data_ptr()
    assert group._all_gather_input[None].data_ptr() == handle.ag_inputs[0].data_ptr()
    assert group._all_gather_input[None].dtype == torch.bfloat16
    for buf in handle.ag_inputs + handle.ag_outputs + handle.rs_buffers:
        assert not bool(torch.isnan(buf).any())
    # the peers' all-gather inputs, from the reference's cast of their shards
    peer_inputs = []
    for k in range(w):
        torch_ops.copy_in(refs[k].ag_in, refs[k].shard)
        peer_inputs.append(refs[k].ag_in.to(DEV))
    handle.peer_ag_inputs = peer_inputs
    group.pre_forward()
    torch.cuda.synchronize()
    assert [c[0] for c in handle.calls] == ["all_gather"]
    assert handle.calls[0][1:] == (handle.ag_inputs[0].data_ptr(), handle.ag_outputs[0].data_ptr(),
                                   ref.lay.padded_sharded_numel)
    assert_bits_equal(group._all_gather_input[None], ref.ag_in, "copy-in into the handle's buffer")
    full = torch.cat([refs[k].ag_in for k in range(w)])
    assert_bits_equal(group._all_gather_output[None], full, "gathered buffer, all ranks' slots")
    for fp, v in zip(group.fsdp_params, torch_ops.unsharded_views(full, ref.numels, ref.sizes)):
        assert_bits_equal(fp.unsharded_param.detach(), v, "unsharded parameter")
    group.post_forward()

    # ---- reduce: the handle sums in place (a SUM, so the whole division follows it: (None, W, SUM))
    grads = _grads(ODD_SHAPES, torch.bfloat16, 40)
    peer_sum = (torch.randn(ref.lay.padded_unsharded_numel, generator=torch.Generator().manual_seed(41)) * 1e-3).bfloat16()
    peer_sum[ref.lay.total_numel:] = 0  # peers' pad lanes are zero like this rank's
    handle.peer_rs_sum = peer_sum.to(DEV)
    for it in range(2):
        group.pre_backward()
        for fp, g in zip(group.fsdp_params, grads):
            fp.unsharded_param.grad = g.to(DEV)
        group.post_backward()
        group.finalize_backward()
        torch.cuda.synchronize()
        torch_ops.reduce_copy_in(ref.rs_views, grads, False)
        pre, post, op, _ = torch_ops.get_gradient_divide_factors(w, torch.bfloat16, None, False, has_yccl_handle=True)
        assert (pre, post, op) == (None, float(w), "SUM")
        ref.rs.chunk(w)[r].add_(peer_sum.chunk(w)[r])  # yccl_handle.reduce_scatter(buffer), ya_fsdp/_collectives.py:163-164
        ref.reduce(pre, post, "copy" if it == 0 else "add")
        assert_bits_equal(group._padded_sharded_param_grad[None], ref.grad_shard, f"gradient shard, pass {it}")
    assert [c[0] for c in handle.calls] == ["all_gather"] + ["all_gather", "reduce_scatter"] * 2
    assert handle.calls[2][1:] == (handle.rs_buffers[0].data_ptr(), ref.lay.padded_unsharded_numel)


def test_handle_without_a_cast_still_gets_its_input_buffer_filled():
    """No mixed precision: without a handle the all-gather input IS the master shard; a handle's input buffer is
    a buffer of its own and takes a same-dtype copy (ya_fsdp/_collectives.py:50-54, _param_group.py:502-519)."""
    w, r, align = 2, 1, 8
    handle = LocalHandle(w, r)
    mp = MixedPrecisionPolicy()
    group, cpu_params = _group_with_handle(ODD_SHAPES, w, r, align, mp, handle)
    refs = [CpuGroup(cpu_params, w, k, align, mp) for k in range(w)]
    ag_in = group._all_gather_input[None]
    assert ag_in.dtype == torch.float32 and ag_in.data_ptr() == handle.ag_inputs[0].data_ptr()
    assert ag_in.data_ptr() != group._padded_sharded_param_data[None].data_ptr()
    handle.peer_ag_inputs = [refs[k].shard.to(DEV).view(torch.bfloat16) for k in range(w)]
    group.pre_forward()
    torch.cuda.synchronize()
    assert_bits_equal(ag_in, refs[r].shard, "fp32 copy-in into the handle's buffer")
    assert_bits_equal(group._all_gather_output[None], torch.cat([x.shard for x in refs]), "gathered buffer")
    assert handle.calls[0][3] == 2 * refs[r].lay.padded_sharded_numel  # bf16 view of an fp32 buffer
    group.post_forward()


def test_size_one_group_keeps_its_copies_and_skips_the_handle(monkeypatch):
    """ya_fsdp/_collectives.py:56-58, 140-150: a group of size one never calls the handle's exchanges; its buffers are
    still the handle's, and the reduce takes the general route (the handle forces the sum-then-divide factors)."""
    from yafsdp_amd import _native

    one = {"n": 0}
    real = _native.TensorTable.gather_in_post_reduce
    monkeypatch.setattr(_native.TensorTable, "gather_in_post_reduce",
                        lambda self, *a, **k: one.__setitem__("n", one["n"] + 1) or real(self, *a, **k))
    handle = LocalHandle(1, 0)
    group, cpu_params = _group_with_handle(ODD_SHAPES, 1, 0, 8, BF16_MP, handle)
    ref = CpuGroup(cpu_params, 1, 0, 8, BF16_MP)
    group.pre_forward(); group.post_forward(); group.pre_backward()
    ref.unshard()
    grads = _grads(ODD_SHAPES, torch.bfloat16, 50)
    for fp, g in zip(group.fsdp_params, grads):
        fp.unsharded_param.grad = g.to(DEV)
    group.post_backward()
    group.finalize_backward()
    torch.cuda.synchronize()
    torch_ops.reduce_copy_in(ref.rs_views, grads, False)
    ref.reduce(None, None, "copy")
    assert handle.calls == [] and one["n"] == 0
    assert group.grad_buffer_ctx.buffers[None].data_ptr() == handle.rs_buffers[0].data_ptr()
    assert_bits_equal(group._all_gather_output[None], ref.ag_out, "gathered buffer")
    assert_bits_equal(group._padded_sharded_param_grad[None], ref.grad_shard, "gradient shard")


def test_a_handle_that_returns_the_wrong_buffer_is_refused():
    class Bad(LocalHandle):
        def add_all_gather_output_buffer(self, numel):
            return torch.zeros(numel, dtype=torch.float16, device=DEV)

    with pytest.raises(TypeError, match="add_all_gather_output_buffer"):
        _group_with_handle(ODD_SHAPES, 2, 0, 8, BF16_MP, Bad(2, 0))


def test_fully_shard_with_a_handle_trains_like_without():
    """The handle enters through the root state's lazy init (ya_fsdp/_state.py:127-168), per buffer context or one for
    all; after every backward its profiling events are processed (:517-529)."""
    from yafsdp_amd import fully_shard

    def build():
        torch.manual_seed(7)
        m = nn.Sequential(nn.Linear(24, 48), nn.ReLU(), nn.Linear(48, 24), nn.ReLU(), nn.Linear(24, 8)).to(DEV)
        for layer in (m[0], m[2], m[4]):
            fully_shard(layer, mesh=(1, 0), mp_policy=BF16_MP)
        return fully_shard(m, mesh=(1, 0), mp_policy=BF16_MP)

    plain, handled = build(), build()
    handle = LocalHandle(1, 0)
    handled._get_fsdp_state()._lazy_init(yccl_handle=handle)
    assert len(handle.ag_outputs) == 2 and len(handle.rs_buffers) == 1 and len(handle.ag_inputs) == 3
    opts = [torch.optim.SGD(m.parameters(), lr=0.1) for m in (plain, handled)]
    gen = torch.Generator().manual_seed(8)
    for step in range(3):
        x = torch.randn(16, 24, generator=gen).to(DEV).bfloat16()
        for m, opt in zip((plain, handled), opts):
            opt.zero_grad(set_to_none=True)
            m(x).float().pow(2).mean().backward()
            opt.step()
    torch.cuda.synchronize()
    assert handle.profiling_events_processed > 0 and handle.calls == []
    for a, b in zip(plain.parameters(), handled.parameters()):
        assert_bits_equal(a._local_tensor, b._local_tensor.cpu(), "master shard")
