"""Parameter-group level parity on the GPU: layout, views, stream/event
protocol and the full unshard -> backward -> reduce flow against the
reference's torch-op sequence (oracle.torch_ops) on CPU, bit for bit."""

import pytest
import torch

from oracle import torch_ops
from tests.helpers import assert_bits_equal
from yafsdp_amd import FSDPMeshInfo, MixedPrecisionPolicy, make_layout

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")

TINY_SHAPES = [(512, 512)] * 4 + [(1376, 512), (1376, 512), (512, 1376), (512,), (512,)]
ODD_SHAPES = [(7, 13), (1,), (129, 3), (5,), (64, 33), (2, 2, 2), (1000,), (3,)]


def _params(shapes, dtype, seed, norms_are_ones=True):
    g = torch.Generator().manual_seed(seed)
    out = []
    for s in shapes:
        if len(s) == 1 and norms_are_ones and s[0] >= 512:
            out.append(torch.ones(s, dtype=dtype))
        else:
            out.append((torch.randn(s, generator=g) * 0.02).to(dtype))
    return out


def _grads(shapes, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    return [(torch.randn(s, generator=g) * 1e-3).to(dtype) for s in shapes]


def _make_group(shapes, w, r, align, mp, master_dtype=torch.float32, seed=1):
    from yafsdp_amd._param_group import YaFSDPParamGroup, init_shared_state

    cpu_params = _params(shapes, master_dtype, seed)
    dev_params = [p.to(DEV).requires_grad_(True) for p in cpu_params]
    group = YaFSDPParamGroup(dev_params, FSDPMeshInfo(w, r), DEV, mp, align)
    init_shared_state([group], DEV)
    return group, cpu_params


class CpuGroup:
    """The reference's op sequence for one group on CPU tensors (zero-filled
    buffers so that pad lanes are defined)."""

    def __init__(self, cpu_params, w, r, align, mp):
        self.w, self.r = w, r
        self.numels = [p.numel() for p in cpu_params]
        self.sizes = [tuple(p.shape) for p in cpu_params]
        self.lay = make_layout(self.numels, w, align)
        orig = cpu_params[0].dtype
        self.param_dtype = None if mp.param_dtype in (None, orig) else mp.param_dtype
        reduce_dtype = None if mp.reduce_dtype == mp.param_dtype else mp.reduce_dtype
        self.ag_dtype = self.param_dtype or orig
        self.rs_dtype = reduce_dtype or self.param_dtype or orig
        t, t_pad, s = self.lay.total_numel, self.lay.padded_unsharded_numel, self.lay.padded_sharded_numel
        flat = torch.zeros(t_pad, dtype=orig)
        for v, p in zip(flat[:t].split(self.numels), cpu_params):  # ya_fsdp/_param_group.py:324-326
            v.copy_(p.view(-1))
        self.shard = flat.chunk(w)[r].clone()  # :337-339
        self.grad_shard = torch.zeros(s, dtype=orig)  # :276
        self.ag_in = self.shard if self.param_dtype is None else torch.zeros(s, dtype=self.ag_dtype)
        self.ag_out = torch.zeros(t_pad, dtype=self.ag_dtype)
        self.rs = torch.zeros(t_pad, dtype=self.rs_dtype)
        self.rs_views = [v.view(sz) for v, sz in zip(self.rs[:t].split(self.numels), self.sizes)]

    def unshard(self, first_of_iteration=True):
        if first_of_iteration and self.param_dtype is not None:
            torch_ops.copy_in(self.ag_in, self.shard)
        if self.w == 1:
            torch_ops.all_gather_single_rank(self.ag_out, self.ag_in)
        else:
            self.ag_out.chunk(self.w)[self.r].copy_(self.ag_in)  # this rank's slot of the all-gather
        return torch_ops.unsharded_views(self.ag_out, self.numels, self.sizes)

    def accumulate(self, grads, accumulate_flags):
        cp = [i for i, (g, a) in enumerate(zip(grads, accumulate_flags)) if g is not None and not a]
        ad = [i for i, (g, a) in enumerate(zip(grads, accumulate_flags)) if g is not None and a]
        torch_ops.reduce_copy_in([self.rs_views[i] for i in cp], [grads[i] for i in cp], False)
        torch_ops.reduce_copy_in([self.rs_views[i] for i in ad], [grads[i] for i in ad], True)

    def reduce(self, pre, post, mode, has=None, collective=None):
        torch_ops.reduce_scatter_local(
            self.grad_shard, self.rs, self.w, self.r, pre, post, mode, self.lay.sharded_numels(self.r), has,
            collective=collective,
        )


BF16_MP = MixedPrecisionPolicy(param_dtype=torch.bfloat16)


@pytest.mark.parametrize("shapes,w,r,align", [
    (TINY_SHAPES, 1, 0, 512),   # config 1: tiny Llama-style layer, W=1
    (TINY_SHAPES, 2, 1, 512),
    (ODD_SHAPES, 4, 2, 8),      # ragged: shard boundaries inside tensors, pad lanes
    (ODD_SHAPES, 4, 3, 8),
    (ODD_SHAPES, 7, 0, 1),
])
def test_layout_views_and_unshard(shapes, w, r, align):
    group, cpu_params = _make_group(shapes, w, r, align, BF16_MP)
    ref = CpuGroup(cpu_params, w, r, align, BF16_MP)
    assert group.layout.padded_sharded_numel == ref.lay.padded_sharded_numel
    assert_bits_equal(group._padded_sharded_param_data[None], ref.shard, "master shard")
    for fp, n, go in zip(group.fsdp_params, ref.lay.sharded_numels(r), ref.lay.global_offsets(r)):
        assert fp.sharded_numel == n and fp.placement.global_offset == go
    group.pre_forward()
    views = ref.unshard()
    torch.cuda.synchronize()
    assert group.is_unsharded
    assert_bits_equal(group._all_gather_input[None], ref.ag_in, "copy-in")
    assert_bits_equal(group._all_gather_output[None], ref.ag_out, "gathered buffer")
    for fp, v in zip(group.fsdp_params, views):
        assert fp.unsharded_param.shape == v.shape
        # zero-copy: the unsharded parameter aliases the gathered buffer
        base = group._all_gather_output[None]
        assert base.data_ptr() <= fp.unsharded_param.data_ptr() < base.data_ptr() + base.numel() * base.element_size()
        if w == 1:
            assert_bits_equal(fp.unsharded_param.detach(), v, "unsharded view")
    # materialising copy-out of the same buffer
    outs = [torch.empty(s, dtype=torch.bfloat16, device=DEV) for s in shapes]
    group.copy_out_materialize(outs)
    want = [torch.empty(s, dtype=torch.bfloat16) for s in shapes]
    torch_ops.copy_out_materialize(ref.ag_out, ref.numels, want)
    for a, b in zip(outs, want):
        assert_bits_equal(a, b, "materialised copy-out")
    group.post_forward()
    assert group.is_sharded and group.data_buffer_ctx.owner is None


def _run_backward(group, ref, grads_cpu, reduce=True):
    for fp, g in zip(group.fsdp_params, grads_cpu):
        fp.unsharded_param.grad = None if g is None else g.to(DEV)
    flags = [fp.unsharded_accumulated_grad is not None for fp in group.fsdp_params]
    group.reduce_grads = reduce
    group.post_backward()
    ref.accumulate(grads_cpu, flags)


@pytest.mark.parametrize("shapes,w,r,align", [(TINY_SHAPES, 1, 0, 512), (ODD_SHAPES, 4, 2, 8), (ODD_SHAPES, 4, 3, 8)])
@pytest.mark.parametrize("force_sum", [False, True])
def test_backward_reduce_copy_then_accumulate(shapes, w, r, align, force_sum):
    group, cpu_params = _make_group(shapes, w, r, align, BF16_MP)
    group.force_sum_reduction_for_comms = force_sum
    ref = CpuGroup(cpu_params, w, r, align, BF16_MP)
    # bf16 reduce: (None, None, AVG) -> the scaling by 1/W happens inside the collective (a pre-multiplied sum);
    # force_sum -> (None, W, SUM): a post-divide by W of the rank's chunk.
    post = float(w) if w > 1 and force_sum else None
    collective = ("AVG", None) if w > 1 and not force_sum else None
    for it in range(2):
        group.pre_forward(); group.post_forward(); group.pre_backward()
        ref.unshard(first_of_iteration=True)
        grads = _grads(shapes, torch.bfloat16, 10 + it)
        _run_backward(group, ref, grads)
        ref.reduce(None, post, "copy" if it == 0 else "add", collective=collective)
        group.finalize_backward()
        torch.cuda.synchronize()
        if post is None and collective is None:  # otherwise the reference also rewrites its (scratch) chunk in place
            assert_bits_equal(group._reduce_scatter_input[None], ref.rs, "reduce buffer")
        assert_bits_equal(group._padded_sharded_param_grad[None], ref.grad_shard, f"grad shard after backward {it}")
        for fp in group.fsdp_params:
            assert fp.sharded_param.grad is fp.sharded_param_grad
        assert group.grad_buffer_ctx.owner is None and group._training_state.name == "IDLE"


@pytest.mark.parametrize("w,r", [(3, 1), (6, 5), (8, 3)])
@pytest.mark.parametrize("factor", [None, 3.0, 5.0, "w"])
@pytest.mark.parametrize("reduce_dtype", [torch.bfloat16, torch.float32])
def test_collective_scaling_at_group_sizes_above_one(w, r, factor, reduce_dtype):
    """ya_fsdp/_collectives.py:243-249 for a bf16 / fp32 reduce without forced sum: no factor or factor == W ->
    ReduceOp.AVG, any other factor -> _make_nccl_premul_sum(1 / factor).  Both scale every contribution inside the
    collective by the reciprocal ROUNDED TO THE REDUCE DTYPE (a product, not a division: W = 3, 6 and factors 3, 5
    tell the two apart).  First backward copies into the gradient shard, second accumulates, third leaves two
    parameters without gradient (fragment-wise path, which reads the chunk the collective left)."""
    shapes, align = ODD_SHAPES, 8
    mp = MixedPrecisionPolicy(param_dtype=torch.bfloat16, reduce_dtype=reduce_dtype)
    group, cpu_params = _make_group(shapes, w, r, align, mp)
    f = float(w) if factor == "w" else factor
    group.gradient_divide_factor = f
    ref = CpuGroup(cpu_params, w, r, align, mp)
    pre, post, op, premul = torch_ops.get_gradient_divide_factors(w, reduce_dtype, f, False)
    assert (pre, post) == (None, None) and op == ("AVG" if f in (None, float(w)) else "PREMUL_SUM")
    for it in range(3):
        group.pre_forward(); group.post_forward(); group.pre_backward()
        grads = _grads(shapes, torch.bfloat16, 90 + it)
        if it == 2:
            grads[0] = None; grads[6] = None
        _run_backward(group, ref, grads)
        if it < 2:
            ref.reduce(None, None, "copy" if it == 0 else "add", collective=(op, premul))
        else:
            ref.reduce(None, None, "mixed", [None if g is None else True for g in grads], collective=(op, premul))
        group.finalize_backward()
        torch.cuda.synchronize()
        assert_bits_equal(group._padded_sharded_param_grad[None], ref.grad_shard, f"grad shard after backward {it}")
    # the fragment-wise path leaves the collective's result in this rank's chunk, as the reference does (compared on
    # the fragments whose parameters had a gradient: the others hold leftovers of earlier passes, which the
    # reference scales once more in place and the fused launches of the earlier passes never wrote back)
    s = ref.lay.padded_sharded_numel
    mine, theirs = group._reduce_scatter_input[None][r * s : (r + 1) * s], ref.rs[r * s : (r + 1) * s]
    pos = 0
    for n, g_ in zip(ref.lay.sharded_numels(r), grads):
        if g_ is not None:
            assert_bits_equal(mine[pos : pos + n], theirs[pos : pos + n], "chunk fragment")
        pos += n


def test_bit32_acc_flag_leaves_the_one_contribution_result_unchanged():
    """ya_fsdp/_collectives.py:152-162: the flag only selects the accumulator of the collective; with this rank's
    chunk as the only contribution the result is the chunk, as without the flag."""
    mp = MixedPrecisionPolicy(param_dtype=torch.bfloat16, reduce_dtype=torch.bfloat16,
                              bit32_acc_for_bit16_reduce_scatter=True)
    w, r, align = 4, 2, 8
    group, cpu_params = _make_group(ODD_SHAPES, w, r, align, mp)
    ref = CpuGroup(cpu_params, w, r, align, BF16_MP)
    group.pre_forward(); group.post_forward(); group.pre_backward()
    ref.unshard()
    _run_backward(group, ref, _grads(ODD_SHAPES, torch.bfloat16, 77))
    ref.reduce(None, None, "copy", collective=("AVG", None))
    group.finalize_backward()
    torch.cuda.synchronize()
    assert_bits_equal(group._padded_sharded_param_grad[None], ref.grad_shard, "grad shard")


def test_gradient_accumulation_without_sync_uses_add():
    shapes, w, r, align = ODD_SHAPES, 4, 1, 8
    group, cpu_params = _make_group(shapes, w, r, align, BF16_MP)
    ref = CpuGroup(cpu_params, w, r, align, BF16_MP)
    group.pre_forward(); group.post_forward(); group.pre_backward()
    _run_backward(group, ref, _grads(shapes, torch.bfloat16, 20), reduce=False)   # copy, no reduce
    assert group._post_reduce_event is None
    group.pre_backward()
    _run_backward(group, ref, _grads(shapes, torch.bfloat16, 21), reduce=False)   # add, no reduce
    group.pre_backward()
    _run_backward(group, ref, _grads(shapes, torch.bfloat16, 22), reduce=True)    # add, then reduce
    ref.reduce(None, None, "copy", collective=("AVG", None))
    group.finalize_backward()
    torch.cuda.synchronize()
    assert_bits_equal(group._padded_sharded_param_grad[None], ref.grad_shard, "grad shard")


def test_size_one_group_reduces_in_one_launch(monkeypatch):
    """A shard group of size one takes the launch that does reduce copy-in and post-reduce together (no collective
    and no divide sit between them, ya_fsdp/_collectives.py:140-150); a backward that leaves one parameter
    without a gradient goes the general way.  Both against the reference's op sequence."""
    from yafsdp_amd import _native

    calls = {"one": 0, "gather": 0}
    real_one, real_gather = _native.TensorTable.gather_in_post_reduce, _native.TensorTable.gather_in

    def count_one(self, *a, **k):
        served = real_one(self, *a, **k)
        calls["one"] += int(served)
        return served

    def count_gather(self, *a, **k):
        calls["gather"] += 1
        return real_gather(self, *a, **k)

    monkeypatch.setattr(_native.TensorTable, "gather_in_post_reduce", count_one)
    monkeypatch.setattr(_native.TensorTable, "gather_in", count_gather)
    shapes, w, r, align = ODD_SHAPES, 1, 0, 8
    group, cpu_params = _make_group(shapes, w, r, align, BF16_MP)
    ref = CpuGroup(cpu_params, w, r, align, BF16_MP)
    group.pre_forward(); group.post_forward(); group.pre_backward()
    _run_backward(group, ref, _grads(shapes, torch.bfloat16, 30), reduce=False)   # copy into the buffer, no reduce
    assert calls == {"one": 0, "gather": 1}
    group.pre_backward()
    _run_backward(group, ref, _grads(shapes, torch.bfloat16, 31), reduce=True)    # add + copy into the shard
    ref.reduce(None, None, "copy")
    group.finalize_backward()
    assert calls == {"one": 1, "gather": 1}
    assert_bits_equal(group._reduce_scatter_input[None], ref.rs, "reduce buffer after the first reduce")
    assert_bits_equal(group._padded_sharded_param_grad[None], ref.grad_shard, "grad shard after the first reduce")
    group.pre_forward(); group.post_forward(); group.pre_backward()
    _run_backward(group, ref, _grads(shapes, torch.bfloat16, 32), reduce=True)    # copy + add into the shard
    ref.reduce(None, None, "add")
    group.finalize_backward()
    assert calls == {"one": 2, "gather": 1}
    assert_bits_equal(group._reduce_scatter_input[None], ref.rs, "reduce buffer after the second reduce")
    assert_bits_equal(group._padded_sharded_param_grad[None], ref.grad_shard, "grad shard after the second reduce")
    for fp in group.fsdp_params:
        assert fp.sharded_param.grad is fp.sharded_param_grad
    assert group.grad_buffer_ctx.owner is None and group._training_state.name == "IDLE"
    # one parameter without a gradient: its fragment keeps the old value (:191-214), the general route
    group.pre_forward(); group.post_forward(); group.pre_backward()
    grads = _grads(shapes, torch.bfloat16, 33)
    grads[2] = None
    _run_backward(group, ref, grads, reduce=True)
    ref.reduce(None, None, "mixed", [None if g is None else True for g in grads])
    group.finalize_backward()
    assert calls == {"one": 2, "gather": 3}  # reduce copy-in, and the fragment-wise accumulation into the shard
    torch.cuda.synchronize()
    assert_bits_equal(group._padded_sharded_param_grad[None], ref.grad_shard, "grad shard after the partial backward")


@pytest.mark.parametrize("policy,factor,force_sum,want", [
    ("bf16", 3.0, False, (None, 3.0, None)),     # custom factor: the out-of-place division (:141-148)
    ("bf16", 4.0, True, (None, None, 4.0)),      # forced sum reduction: post-divide only
    ("fp16", 8.0, False, (4.0, None, 2.0)),      # fp16 reduce: pre- and post-divide
])
def test_size_one_group_divides_inside_the_one_launch(monkeypatch, policy, factor, force_sum, want):
    from yafsdp_amd import _native

    seen = []
    real = _native.TensorTable.gather_in_post_reduce

    def spy(self, *a, **k):
        served = real(self, *a, **k)
        seen.append((served, k.get("pre_factor"), k.get("custom_divisor"), k.get("post_factor")))
        return served

    monkeypatch.setattr(_native.TensorTable, "gather_in_post_reduce", spy)
    dt = torch.bfloat16 if policy == "bf16" else torch.float16
    mp = MixedPrecisionPolicy(param_dtype=dt)
    shapes, w, r, align = ODD_SHAPES, 1, 0, 8
    group, cpu_params = _make_group(shapes, w, r, align, mp)
    group.gradient_divide_factor = factor
    group.force_sum_reduction_for_comms = force_sum
    ref = CpuGroup(cpu_params, w, r, align, mp)
    pre, custom, post = want
    for it in range(2):
        group.pre_forward(); group.post_forward(); group.pre_backward()
        _run_backward(group, ref, _grads(shapes, dt, 70 + it))
        torch_ops.div_if_needed(ref.rs, pre)
        if custom is not None:
            ref.rs.copy_(ref.rs / custom)
        rs_before_post = ref.rs.clone()
        ref.reduce(None, post, "copy" if it == 0 else "add")
        group.finalize_backward()
        torch.cuda.synchronize()
        assert seen[-1] == (True, pre, custom, post)
        assert_bits_equal(group._reduce_scatter_input[None], rs_before_post, "reduce buffer")
        assert_bits_equal(group._padded_sharded_param_grad[None], ref.grad_shard, f"grad shard after backward {it}")


def test_mixed_params_with_and_without_sharded_grad(monkeypatch):
    from yafsdp_amd import _native

    def per_run_launches(*a, **k):  # the group-level path is one launch over a fragment table
        raise AssertionError("post_reduce_fragments (one launch per run of fragments) must not be used here")

    monkeypatch.setattr(_native, "post_reduce_fragments", per_run_launches)
    shapes, w, r, align = ODD_SHAPES, 2, 0, 8
    group, cpu_params = _make_group(shapes, w, r, align, BF16_MP)
    ref = CpuGroup(cpu_params, w, r, align, BF16_MP)
    group.pre_forward(); group.post_forward(); group.pre_backward()
    g1 = _grads(shapes, torch.bfloat16, 30)
    g1[1] = None; g1[4] = None                      # two params get no gradient in the first backward
    _run_backward(group, ref, g1)
    has = [None if g is None else False for g in g1]
    ref.reduce(None, None, "mixed", has, collective=("AVG", None))        # partial first reduction goes through the fragment path
    group.finalize_backward()
    group.pre_forward(); group.post_forward(); group.pre_backward()
    ref.unshard()
    g2 = _grads(shapes, torch.bfloat16, 31)
    _run_backward(group, ref, g2)
    has2 = [g is not None for g in g1]              # params that already own a sharded grad accumulate
    ref.reduce(None, None, "mixed", has2, collective=("AVG", None))
    group.finalize_backward()
    torch.cuda.synchronize()
    assert_bits_equal(group._padded_sharded_param_grad[None], ref.grad_shard, "grad shard")
    assert group._fragment_table is not None and group._fragment_table.numels == ref.lay.sharded_numels(r)


def test_fp16_reduce_uses_pre_and_post_divide():
    shapes, w, r, align = ODD_SHAPES, 8, 5, 8
    mp = MixedPrecisionPolicy(param_dtype=torch.float16)
    group, cpu_params = _make_group(shapes, w, r, align, mp)
    ref = CpuGroup(cpu_params, w, r, align, mp)
    group.pre_forward(); group.post_forward(); group.pre_backward()
    _run_backward(group, ref, _grads(shapes, torch.float16, 40))
    ref.reduce(4.0, 2.0, "copy")                    # W=8 -> pre 4, post 2 (ya_fsdp/_collectives.py:252-262)
    group.finalize_backward()
    torch.cuda.synchronize()
    # outside this rank's chunk the reduce buffer holds cast + pre-divide only, like the reference's
    s_, rs_dev = ref.lay.padded_sharded_numel, group._reduce_scatter_input[None]
    assert_bits_equal(rs_dev[: r * s_], ref.rs[: r * s_], "reduce buffer before the chunk")
    assert_bits_equal(rs_dev[(r + 1) * s_ :], ref.rs[(r + 1) * s_ :], "reduce buffer after the chunk")
    assert_bits_equal(group._padded_sharded_param_grad[None], ref.grad_shard, "grad shard fp16 reduce")


def test_bf16_masters_fp32_reduce():
    shapes, w, r, align = ODD_SHAPES, 4, 2, 8
    mp = MixedPrecisionPolicy(param_dtype=torch.bfloat16, reduce_dtype=torch.float32)
    group, cpu_params = _make_group(shapes, w, r, align, mp, master_dtype=torch.bfloat16)
    assert group.param_dtype is None and group.reduce_dtype == torch.float32   # clamping, ya_fsdp/_param.py:170-183
    assert group._all_gather_input[None].data_ptr() == group._padded_sharded_param_data[None].data_ptr()
    ref = CpuGroup(cpu_params, w, r, align, mp)
    for it in range(2):
        group.pre_forward(); group.post_forward(); group.pre_backward()
        _run_backward(group, ref, _grads(shapes, torch.bfloat16, 50 + it))
        ref.reduce(None, None, "copy" if it == 0 else "add", collective=("AVG", None))
        group.finalize_backward()
    torch.cuda.synchronize()
    assert group._padded_sharded_param_grad[None].dtype == torch.bfloat16
    assert_bits_equal(group._padded_sharded_param_grad[None], ref.grad_shard, "bf16 grad shard, fp32 reduce")


def test_fp32_no_mixed_precision_reduces_in_sharded():
    shapes, w, r, align = ODD_SHAPES, 1, 0, 8
    mp = MixedPrecisionPolicy()
    group, cpu_params = _make_group(shapes, w, r, align, mp)
    ref = CpuGroup(cpu_params, w, r, align, mp)
    group.gradient_divide_factor = 3.0              # size-1 group with a custom factor: out-of-place divide (:141-148)
    group.pre_forward(); group.post_forward(); group.pre_backward()
    grads = _grads(shapes, torch.float32, 60)
    _run_backward(group, ref, grads)
    ref.grad_shard.copy_(ref.rs / 3.0)
    group.finalize_backward()
    torch.cuda.synchronize()
    assert_bits_equal(group._padded_sharded_param_grad[None], ref.grad_shard, "fp32 reduce in sharded")


def test_buffer_ownership_protocol():
    from yafsdp_amd._param_group import YaFSDPParamGroup, init_shared_state

    def mk(seed):
        ps = [p.to(DEV).requires_grad_(True) for p in _params(ODD_SHAPES, torch.float32, seed)]
        return YaFSDPParamGroup(ps, FSDPMeshInfo(2, 0), DEV, BF16_MP, 8, module_fqn=f"layer{seed}")

    a, b, c = mk(1), mk(2), mk(3)
    init_shared_state([a, b, c], DEV)               # 2 data buffers round-robin: a and c share one
    assert a.data_buffer_ctx is c.data_buffer_ctx and a.data_buffer_ctx is not b.data_buffer_ctx
    assert a.grad_buffer_ctx is b.grad_buffer_ctx is c.grad_buffer_ctx
    assert a.comm_ctx is b.comm_ctx
    a.pre_forward()
    b.pre_forward()                                 # other buffer: fine
    with pytest.raises(RuntimeError, match="data buffer"):
        c.pre_forward()                             # ya_fsdp/_param_group.py:567-572
    a.post_forward()
    assert a.data_buffer_ctx.release_event is not None
    c._all_gather_result = None
    c.pre_forward()                                 # waits on the release event, then owns the buffer
    assert a.data_buffer_ctx.owner is c and a.data_buffer_ctx.release_event is None
    # gradient buffer: one for all groups
    for fp in b.fsdp_params:
        fp.unsharded_param.grad = torch.zeros_like(fp.unsharded_param)
    b.grad_buffer_ctx.owner = a
    with pytest.raises(RuntimeError, match="gradient buffer"):
        b.post_backward()                           # :660-664
    b.grad_buffer_ctx.owner = None
    b.post_backward()
    assert b.grad_buffer_ctx.owner is None and b.grad_buffer_ctx.release_event is b._post_reduce_event
    b.finalize_backward(); c.post_forward()
    torch.cuda.synchronize()


def test_copy_in_runs_once_per_iteration():
    group, cpu_params = _make_group(ODD_SHAPES, 2, 1, 8, BF16_MP)
    group.pre_forward(); group.post_forward()
    torch.cuda.synchronize()
    first = group._all_gather_input[None].clone()
    with torch.no_grad():
        group._padded_sharded_param_data[None].add_(1.0)        # an optimizer step
    group.pre_backward()                                        # same iteration: stale copy is reused (:47-55)
    torch.cuda.synchronize()
    assert_bits_equal(group._all_gather_input[None], first.cpu(), "copy-in skipped inside one iteration")
    group.post_backward(); group.finalize_backward()            # clears the once-per-iteration set (:783)
    group.pre_forward()
    torch.cuda.synchronize()
    assert not torch.equal(group._all_gather_input[None], first)


def test_constructor_errors():
    from yafsdp_amd._param_group import YaFSDPParamGroup

    mi = FSDPMeshInfo(2, 0)
    with pytest.raises(RuntimeError, match="GPU only"):
        YaFSDPParamGroup([torch.zeros(4)], mi, torch.device("cpu"))
    with pytest.raises(NotImplementedError):
        YaFSDPParamGroup([torch.zeros(4, 4, device=DEV).t()], mi, DEV)
    with pytest.raises(AssertionError, match="uniform original parameter dtype"):
        YaFSDPParamGroup([torch.zeros(4, device=DEV), torch.zeros(4, device=DEV, dtype=torch.bfloat16)], mi, DEV)
    with pytest.raises(ValueError):
        YaFSDPParamGroup([torch.zeros((), device=DEV)], mi, DEV)
    with pytest.raises(ValueError):
        MixedPrecisionPolicy(reduce_dtype=torch.float16, bit32_acc_for_bit16_reduce_scatter=True)
