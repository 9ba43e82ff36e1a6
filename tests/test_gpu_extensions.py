"""Tensor-subclass all-gather extensions on the GPU
(``MixedPrecisionPolicy.all_gather_dtype_to_param_cls`` with
``fsdp_pre_all_gather`` / ``fsdp_post_all_gather``; ya_fsdp/_param_group.py:194-227,
ya_fsdp/_param.py:185-195, 203-257, 281-291, ya_fsdp/_collectives.py:47-58).

A group then has one flat shard, all-gather input, gathered buffer and reduce
buffer per all-gather dtype class.  Checked bit for bit against the reference's
op sequence on CPU tensors (oracle.torch_ops per class): the 1-byte all-gather
input that the subclass produces, its placement in the gathered buffer, the
reduce of every class, and three optimizer steps of a wrapped model against a
hand-written loop with the same arithmetic.
"""

import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from oracle import torch_ops
from tests.ext_subclasses import STEP, Int8Master, Int8Weight, dequantize, quantize
from tests.helpers import assert_bits_equal
from yafsdp_amd import FSDPMeshInfo, MixedPrecisionPolicy, make_layout

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")

# (shape, is_extension): sizes chosen so that shard boundaries fall inside tensors of both classes
MIXED = [((33, 7), True), ((64,), False), ((5, 13), True), ((129, 3), False), ((1000,), True), ((3,), True),
         ((17, 2), False)]
INT8_MP = MixedPrecisionPolicy(param_dtype=torch.bfloat16, all_gather_dtype_to_param_cls={torch.int8: Int8Master})


def _say(*a):
    print(*a, flush=True)


def _values(spec, seed):
    g = torch.Generator().manual_seed(seed)
    return [(torch.randn(s, generator=g) * 0.08) for s, _ in spec]


class CpuClass:
    """One all-gather dtype class of a group as the reference runs it, on CPU tensors."""

    def __init__(self, values, w, r, align, ag_dtype):
        self.w, self.r = w, r
        self.numels = [v.numel() for v in values]
        self.sizes = [tuple(v.shape) for v in values]
        self.lay = make_layout(self.numels, w, align)
        t, t_pad, s = self.lay.total_numel, self.lay.padded_unsharded_numel, self.lay.padded_sharded_numel
        flat = torch.zeros(t_pad)
        for view, v in zip(flat[:t].split(self.numels), values):
            view.copy_(v.view(-1))
        self.shard = flat.chunk(w)[r].clone()
        self.grad_shard = torch.zeros(s)
        self.ag_in = torch.zeros(s, dtype=ag_dtype)
        self.ag_out = torch.zeros(t_pad, dtype=ag_dtype)
        self.rs = torch.zeros(t_pad, dtype=torch.bfloat16)
        self.rs_views = [v.view(sz) for v, sz in zip(self.rs[:t].split(self.numels), self.sizes)]

    def fragments(self, flat_s):
        n = self.lay.sharded_numels(self.r)
        return flat_s[: sum(n)].split(n)

    def place(self):
        self.ag_out.chunk(self.w)[self.r].copy_(self.ag_in)


def _make(spec, w, r, align, seed=3):
    from yafsdp_amd._param_group import YaFSDPParamGroup, init_shared_state

    values = _values(spec, seed)
    dev_params = []
    for v, (_, ext) in zip(values, spec):
        d = v.to(DEV)
        dev_params.append(nn.Parameter(Int8Master(d)) if ext else d.requires_grad_(True))
    group = YaFSDPParamGroup(dev_params, FSDPMeshInfo(w, r), DEV, INT8_MP, align)
    init_shared_state([group], DEV)
    plain = CpuClass([v for v, (_, e) in zip(values, spec) if not e], w, r, align, torch.bfloat16)
    ext = CpuClass([v for v, (_, e) in zip(values, spec) if e], w, r, align, torch.int8)
    return group, plain, ext


@pytest.mark.parametrize("w,r,align", [(1, 0, 8), (2, 1, 8), (4, 2, 8), (3, 0, 1), (5, 4, 16)])
def test_classes_unshard_and_reduce(w, r, align):
    _say("extension classes", w, r, align)
    group, plain, ext = _make(MIXED, w, r, align)
    assert list(group._all_gather_dtype_to_fsdp_params) == [None, torch.int8]
    assert group.has_extension_classes
    assert [p._orig_size for p in group._all_gather_dtype_to_fsdp_params[torch.int8]] == [
        torch.Size(s) for s, e in MIXED if e
    ]
    for key, ref in ((None, plain), (torch.int8, ext)):
        assert group.layouts[key] == ref.lay
        assert_bits_equal(group._padded_sharded_param_data[key], ref.shard, f"master shard {key}")
    for fp in group._all_gather_dtype_to_fsdp_params[torch.int8]:
        assert isinstance(fp.sharded_param._local_tensor, Int8Master)
        assert fp.sharded_param._local_tensor._data.data_ptr() == fp._sharded_param_data.data_ptr()
        assert fp._extensions_data is not None and isinstance(fp.unsharded_param, Int8Weight)
        assert fp.unsharded_param._step is None  # built at lazy_init, before any all-gather
    for fp in group._all_gather_dtype_to_fsdp_params[None]:
        assert fp._extensions_data is None and type(fp.sharded_param._local_tensor) is torch.Tensor
    # buffers: one per class in each context, sized for that class
    assert set(group.data_buffer_ctx.buffers) == {None, torch.int8}
    assert group.data_buffer_ctx.buffers[torch.int8].numel() >= ext.lay.padded_unsharded_numel
    assert group._all_gather_output[torch.int8].dtype == torch.int8
    assert group._reduce_scatter_input[torch.int8].dtype == torch.bfloat16

    # ---- unshard: the subclass's own all-gather input per parameter (its quantised fragment), copied into the flat
    # all-gather input of the class and placed in this rank's slot of the gathered buffer
    group.pre_forward()
    torch.cuda.synchronize()
    torch_ops.copy_in(plain.ag_in, plain.shard)
    plain.place()
    for dst, frag in zip(ext.fragments(ext.ag_in), ext.fragments(ext.shard)):
        torch_ops.extension_copy_in(dst, quantize(frag))  # what Int8Master.fsdp_pre_all_gather returns
    ext.place()
    assert torch.equal(group._all_gather_input[torch.int8].cpu(), ext.ag_in)
    assert torch.equal(group._all_gather_output[torch.int8].cpu(), ext.ag_out)
    assert_bits_equal(group._all_gather_input[None], plain.ag_in, "copy-in of the default class")
    assert_bits_equal(group._all_gather_output[None], plain.ag_out, "gathered buffer of the default class")
    base = group._all_gather_output[torch.int8]
    for fp, numel in zip(group._all_gather_dtype_to_fsdp_params[torch.int8], ext.numels):
        up = fp.unsharded_param
        assert isinstance(up, Int8Weight) and up.dtype == torch.bfloat16 and up._step == STEP
        assert base.data_ptr() <= up._q.data_ptr() < base.data_ptr() + base.numel() and up._q.numel() == numel
        if fp._module_info is None and w == 1:
            want = dequantize(quantize(ext.shard[: ext.lay.total_numel]), STEP, torch.bfloat16)
            off = up._q.data_ptr() - base.data_ptr()
            assert_bits_equal(up.dequantize().view(-1), want[off : off + numel], "dequantised weight")
    group.post_forward()

    # ---- backward: bf16 gradients of every parameter, reduced per class
    g = torch.Generator().manual_seed(11)
    grads = [(torch.randn(s, generator=g) * 1e-3).bfloat16() for s, _ in MIXED]
    for step in range(2):  # second pass accumulates into the gradient shards
        group.pre_backward()
        for fp, gr in zip(group.fsdp_params, grads):
            fp.unsharded_param.grad = gr.to(DEV)
        group.post_backward()
        group.finalize_backward()
        torch.cuda.synchronize()
        # bf16 reduce: ReduceOp.AVG, i.e. the collective multiplies every contribution by 1 / W rounded to bf16
        collective = ("AVG", None) if w > 1 else None
        for key, ref in ((None, plain), (torch.int8, ext)):
            mine = [gr for gr, (_, e) in zip(grads, MIXED) if e == (key is not None)]
            torch_ops.reduce_copy_in(ref.rs_views, mine, False)
            torch_ops.reduce_scatter_local(ref.grad_shard, ref.rs, w, r, None, None, "copy" if step == 0 else "add",
                                           collective=collective)
            assert_bits_equal(group._padded_sharded_param_grad[key], ref.grad_shard, f"gradient shard {key} pass {step}")
        for fp in group.fsdp_params:
            assert fp.sharded_param.grad is fp.sharded_param_grad


def test_group_of_extension_parameters_only():
    """No default class at all: the per-class dictionaries have the one key, the one-class accessors say so."""
    spec = [((40, 3), True), ((9,), True)]
    group, _, ext = _make(spec, 2, 0, 8)
    assert list(group._all_gather_dtype_to_fsdp_params) == [torch.int8]
    with pytest.raises(NotImplementedError, match="all-gather dtype class"):
        group.layout
    group.pre_forward()
    torch.cuda.synchronize()
    for dst, frag in zip(ext.fragments(ext.ag_in), ext.fragments(ext.shard)):
        torch_ops.extension_copy_in(dst, quantize(frag))
    assert torch.equal(group._all_gather_input[torch.int8].cpu(), ext.ag_in)
    group.post_forward()


def test_hooks_must_come_in_pairs():
    from yafsdp_amd._param_group import YaFSDPParamGroup

    class OnlyPre(torch.Tensor):
        @staticmethod
        def __new__(cls, data):
            return torch.Tensor._make_wrapper_subclass(cls, data.shape, dtype=data.dtype, device=data.device)

        def __init__(self, data):
            self._data = data

        def __repr__(self):  # the error message names the tensor
            return f"OnlyPre({tuple(self.shape)})"

        def __tensor_flatten__(self):
            return ["_data"], None

        @classmethod
        def __torch_dispatch__(cls, func, types, args=(), kwargs=None):
            un = [a._data if isinstance(a, OnlyPre) else a for a in args]
            out = func(*un, **(kwargs or {}))
            return OnlyPre(out) if isinstance(out, torch.Tensor) and func != torch.ops.aten.copy_.default else out

        def fsdp_pre_all_gather(self, mesh):
            return (self._data,), None

    p = nn.Parameter(OnlyPre(torch.zeros(16, device=DEV)))
    with pytest.raises(AssertionError, match="Both fsdp_pre_all_gather and fsdp_post_all_gather"):
        YaFSDPParamGroup([p], FSDPMeshInfo(1, 0), DEV,
                         MixedPrecisionPolicy(param_dtype=torch.bfloat16,
                                              all_gather_dtype_to_param_cls={torch.float32: OnlyPre}), 8)


class QLinear(nn.Module):
    """Linear layer whose weight is an ``Int8Master`` parameter (int8 all-gather) and whose bias is plain."""

    def __init__(self, n_in, n_out, gen):
        super().__init__()
        self.weight = nn.Parameter(Int8Master((torch.randn(n_out, n_in, generator=gen) * 0.06).to(DEV)))
        self.bias = nn.Parameter((torch.randn(n_out, generator=gen) * 0.02).to(DEV))

    def forward(self, x):
        return F.linear(x, self.weight, self.bias)


def test_training_with_int8_all_gather_matches_a_hand_written_loop():
    """fully_shard with the extension policy, torch.optim.SGD on the sharded parameters: after three steps the
    fp32 masters equal those of a loop that quantises, dequantises and reduces by hand."""
    from yafsdp_amd import fully_shard

    gen = torch.Generator().manual_seed(5)
    layers = [QLinear(24, 40, gen), QLinear(40, 24, gen)]
    model = nn.Sequential(layers[0], nn.ReLU(), layers[1])
    masters = [(l.weight.detach()._data.clone(), l.bias.detach().clone()) for l in layers]
    for l in layers:
        fully_shard(l, mesh=(1, 0), mp_policy=INT8_MP)
    fully_shard(model, mesh=(1, 0), mp_policy=INT8_MP)
    opt = torch.optim.SGD(model.parameters(), lr=0.05)
    xs = [(torch.randn(16, 24, generator=gen)).to(DEV).bfloat16() for _ in range(3)]
    for step, x in enumerate(xs):
        _say("int8 all-gather training step", step)
        opt.zero_grad(set_to_none=True)
        model(x).float().pow(2).mean().backward()
        opt.step()
        # by hand: the same mixed precision
        ws = [dequantize(quantize(w), STEP, torch.bfloat16).requires_grad_() for w, _ in masters]
        bs = [b.bfloat16().requires_grad_() for _, b in masters]
        h = F.linear(x, ws[0], bs[0]).relu()
        F.linear(h, ws[1], bs[1]).float().pow(2).mean().backward()
        for (w, b), wq, bq in zip(masters, ws, bs):
            w.add_(wq.grad.float(), alpha=-0.05)  # bf16 gradient -> bf16 reduce buffer -> fp32 shard -> SGD
            b.add_(bq.grad.float(), alpha=-0.05)
    torch.cuda.synchronize()
    for l, (w, b) in zip(layers, masters):
        wp = l.weight
        assert isinstance(wp._local_tensor, Int8Master)
        assert_bits_equal(wp._local_tensor._data.view(w.shape), w.cpu(), "weight master")
        assert_bits_equal(l.bias._local_tensor.view(b.shape), b.cpu(), "bias master")


def test_checkpoint_and_full_tensor_of_extension_parameters(tmp_path):
    """The sharded parameter of a tensor-subclass class wraps an ``Int8Master`` around its fragment of the flat master
    shard; ``full_tensor()`` and the ``torch.distributed.checkpoint`` hooks deal in the plain master values."""
    import torch.distributed.checkpoint as dcp

    from yafsdp_amd import RaggedShardDTensor, fully_shard
    from yafsdp_amd.checkpoint import RaggedShardLoadPlanner

    def build(seed):
        gen = torch.Generator().manual_seed(seed)
        layer = QLinear(24, 40, gen)
        values = (layer.weight.detach()._data.clone(), layer.bias.detach().clone())
        return fully_shard(layer, mesh=(1, 0), mp_policy=INT8_MP), values

    model, (w, b) = build(21)
    assert isinstance(model.weight, RaggedShardDTensor) and isinstance(model.weight._local_tensor, Int8Master)
    full = model.weight.full_tensor()
    assert type(full) is torch.Tensor and full.shape == w.shape
    assert_bits_equal(full, w.cpu(), "full_tensor of the extension parameter")
    dcp.save(model.state_dict(), checkpoint_id=str(tmp_path / "ckpt"), no_dist=True)
    other, (w2, _) = build(22)
    assert not torch.equal(w2, w)
    dcp.load(other.state_dict(), checkpoint_id=str(tmp_path / "ckpt"), no_dist=True, planner=RaggedShardLoadPlanner())
    torch.cuda.synchronize()
    assert_bits_equal(other.weight._local_tensor._data.view(w.shape), w.cpu(), "loaded weight master")
    assert_bits_equal(other.bias._local_tensor.view(b.shape), b.cpu(), "loaded bias master")
    # and the loaded masters are what the next all-gather quantises
    x = torch.randn(4, 24, generator=torch.Generator().manual_seed(1)).to(DEV).bfloat16()
    want = F.linear(x, dequantize(quantize(w), STEP, torch.bfloat16), b.bfloat16())
    assert_bits_equal(other(x), want.cpu(), "forward after loading")


@pytest.mark.parametrize("world", [(1, 0), (2, 1)])
def test_grad_norm_fused_into_the_post_reduce_of_every_all_gather_dtype_class(world):
    """``enable_fused_grad_norm`` gives every class of a group its own slot of partial sums: after a backward pass the
    clip coefficient needs no read pass over either gradient shard, and equals the one computed by reading them."""
    from oracle import cref
    from yafsdp_amd import _native, fully_shard
    from yafsdp_amd.optim import disable_fused_grad_norm, enable_fused_grad_norm, fsdp_param_groups, grad_clip_coef

    gen = torch.Generator().manual_seed(37)
    layer = fully_shard(QLinear(24, 40, gen), mesh=world, mp_policy=INT8_MP)
    (group,) = fsdp_param_groups(layer)
    x = torch.randn(16, 24, generator=gen).to(DEV).bfloat16()
    (layer(x).float().pow(2).mean() * 30.0).backward()  # the gradient shards exist from here on
    enable_fused_grad_norm(layer)
    keys = [None, torch.int8]
    assert list(group._grad_sumsq_slot) == keys
    layer.zero_grad(set_to_none=True)
    (layer(x).float().pow(2).mean() * 30.0).backward()
    for k in keys:
        assert group._grad_sumsq_token.get(k) == group._padded_sharded_param_grad[k]._version
    calls = {"read": 0}
    real = _native.sumsq_partials

    def counting(*a, **kw):
        calls["read"] += 1
        return real(*a, **kw)

    _native.sumsq_partials = counting
    try:
        norm_fused, coef_fused = grad_clip_coef(layer, 1e-3)
        assert calls["read"] == 0  # every sum came from a post-reduce
        # a gradient rewritten behind the library's back (a torch op bumps the shard's version): that class alone
        # is read again
        group._padded_sharded_param_grad[torch.int8].mul_(1.0)
        norm_mixed, _ = grad_clip_coef(layer, 1e-3)
        assert calls["read"] == 1
        disable_fused_grad_norm(layer)
        assert not group._grad_sumsq_slot and group._grad_sumsq_partials is None
        norm_read, coef_read = grad_clip_coef(layer, 1e-3)
        assert calls["read"] == 3
    finally:
        _native.sumsq_partials = real
    want, want_coef = cref.clip_coef(
        sum(cref.sumsq(group._padded_sharded_param_grad[k].detach().cpu()) for k in keys), 1e-3)
    assert want > 0 and want_coef < 1.0
    for got in (norm_fused, norm_mixed, norm_read):
        assert abs(got.item() - want) <= 2e-7 * want
    assert abs(coef_fused.item() - want_coef) <= 2e-7 * want_coef


def test_flat_optimizer_passes_cover_every_all_gather_dtype_class():
    """``grad_clip_coef`` / ``clip_grad_norm_`` / ``zero_grad`` / ``FlatAdamW`` run over the flat shards of both
    classes of a group (ordinary parameters and the int8 all-gather class); the fused copy-in serves the default
    class only, the subclass quantises its own masters in the next forward.  Against the C oracle per flat shard."""
    from oracle import cref
    from yafsdp_amd import fully_shard
    from yafsdp_amd.optim import FlatAdamW, clip_grad_norm_, fsdp_param_groups, zero_grad

    gen = torch.Generator().manual_seed(31)
    layer = fully_shard(QLinear(24, 40, gen), mesh=(1, 0), mp_policy=INT8_MP)
    (group,) = fsdp_param_groups(layer)
    assert list(group._padded_sharded_param_grad) == [None, torch.int8]
    opt = FlatAdamW(layer.parameters(), lr=1e-2, betas=(0.9, 0.95), weight_decay=0.1)
    x = torch.randn(16, 24, generator=gen).to(DEV).bfloat16()
    (layer(x).float().pow(2).mean() * 30.0).backward()
    keys = [None, torch.int8]
    masters = {k: group._padded_sharded_param_data[k].detach().cpu().clone() for k in keys}
    grads = {k: group._padded_sharded_param_grad[k].detach().cpu().clone() for k in keys}
    assert all(float(grads[k].abs().max()) > 0 for k in keys)
    # clipping over both shards
    max_norm = 1e-2
    norm, coef = cref.clip_coef(sum(cref.sumsq(grads[k]) for k in keys), max_norm)
    got = clip_grad_norm_(layer, max_norm)
    assert abs(got.item() - norm) <= 6e-8 * norm and coef < 1.0
    for k in keys:
        cref.flat_scale(grads[k], coef)
        assert_bits_equal(group._padded_sharded_param_grad[k], grads[k], f"clipped gradient shard {k}")
    # one AdamW step per flat shard; only the default class gets its 16-bit all-gather input written
    opt.step()
    torch.cuda.synchronize()
    for k in keys:
        n = masters[k].numel()
        out16 = torch.zeros(n, dtype=torch.bfloat16) if k is None else None
        cref.adamw_step(masters[k], grads[k], torch.zeros(n), torch.zeros(n), out16, lr=1e-2, beta1=0.9, beta2=0.95,
                        eps=1e-8, weight_decay=0.1, step=1)
        assert_bits_equal(group._padded_sharded_param_data[k], masters[k], f"master shard {k} after the step")
        if k is None:
            assert_bits_equal(group._all_gather_input[None], out16, "fused copy-in of the default class")
    assert group._all_gather_input_set_dtypes == {None}
    for p in layer.parameters():
        st = opt.state[p]
        assert st["exp_avg"].shape == p.shape and float(st["exp_avg"]._local_tensor.abs().max()) > 0
    # the next forward quantises the updated masters itself
    want = F.linear(x, dequantize(quantize(masters[torch.int8][: 40 * 24].view(40, 24)), STEP, torch.bfloat16).to(DEV),
                    masters[None][:40].bfloat16().to(DEV)).cpu()
    assert_bits_equal(layer(x), want, "forward after the step")
    zero_grad(layer)
    for k in keys:
        assert float(group._padded_sharded_param_grad[k].abs().max()) == 0.0


def test_malformed_extensions_are_refused_with_a_message():
    from yafsdp_amd._param_group import YaFSDPParamGroup, init_shared_state

    class PlainNewZeros(Int8Master):
        """``new_zeros`` falls back to a plain tensor: the sharded parameter would lose the hooks."""

        @classmethod
        def __torch_dispatch__(cls, func, types, args=(), kwargs=None):
            if func == torch.ops.aten.new_zeros.default:
                return func(args[0]._data, *args[1:], **(kwargs or {}))
            return super().__torch_dispatch__(func, types, args, kwargs)

    mp = MixedPrecisionPolicy(param_dtype=torch.bfloat16, all_gather_dtype_to_param_cls={torch.int8: PlainNewZeros})
    p = nn.Parameter(PlainNewZeros(torch.zeros(32, device=DEV)))
    with pytest.raises(AssertionError, match="new_zeros returned a plain tensor"):
        YaFSDPParamGroup([p], FSDPMeshInfo(1, 0), DEV, mp, 8)

    class ShortInput(Int8Master):
        """``fsdp_pre_all_gather`` returns fewer elements than the fragment holds."""

        def fsdp_pre_all_gather(self, mesh):
            return (quantize(self._data)[:-1],), (STEP,)

    mp = MixedPrecisionPolicy(param_dtype=torch.bfloat16, all_gather_dtype_to_param_cls={torch.int8: ShortInput})
    group = YaFSDPParamGroup([nn.Parameter(ShortInput(torch.ones(32, device=DEV)))], FSDPMeshInfo(1, 0), DEV, mp, 8)
    init_shared_state([group], DEV)
    with pytest.raises(AssertionError, match="returned 31 elements for a fragment of 32"):
        group.pre_forward()


def test_full_tensors_reassembles_every_class_from_all_logical_ranks():
    """``checkpoint.full_tensors`` over the W logical ranks of one group: every parameter of both classes comes back
    whole, as plain master values, in the group's parameter order; ``load_full_tensors`` puts them back."""
    from yafsdp_amd.checkpoint import full_tensors, load_full_tensors

    w = 3
    ranks = [_make(MIXED, w, r, 8)[0] for r in range(w)]
    for r, g in enumerate(ranks):
        for i, fp in enumerate(g.fsdp_params):
            fp._param_fqn = f"p{i}"
    values = _values(MIXED, 3)
    got = full_tensors(ranks)
    assert list(got) == [f"p{i}" for i in range(len(MIXED))]
    for i, v in enumerate(values):
        assert type(got[f"p{i}"]) is torch.Tensor and got[f"p{i}"].shape == v.shape
        assert_bits_equal(got[f"p{i}"], v, f"full parameter {i}")
    # other values go in through load_full_tensors, rank by rank, and come back
    g = torch.Generator().manual_seed(77)
    new = {f"p{i}": torch.randn(s, generator=g).to(DEV) for i, (s, _) in enumerate(MIXED)}
    load_full_tensors(ranks, new)
    again = full_tensors(ranks)
    for k, v in new.items():
        assert_bits_equal(again[k], v.cpu(), f"reloaded {k}")
