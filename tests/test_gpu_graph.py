"""A step of the buffer path captured into a HIP graph (tables with at most 16
tensors pass everything in kernel arguments, so nothing but kernel launches is
recorded) and replayed several times, with eager work and synchronisations in
between; every replay must equal the eager result on the same inputs."""

import pytest
import torch

from tests.helpers import assert_bits_equal

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def test_captured_step_replays_match_eager():
    from yafsdp_amd import _native, make_layout

    shapes = [(512, 512)] * 2 + [(1376, 512), (512, 1376), (512,), (333,)]
    numels = [torch.Size(s).numel() for s in shapes]
    w, r = 4, 2
    lay = make_layout(numels, w, 8)
    t, t_pad, s = lay.total_numel, lay.padded_unsharded_numel, lay.padded_sharded_numel
    g = torch.Generator(device=DEV).manual_seed(77)

    def rnd(n, std, dt):
        return (torch.randn(n, device=DEV, generator=g) * std).to(dt)

    master, gathered = rnd(s, 0.02, torch.float32), rnd(t_pad, 0.02, torch.bfloat16)
    grads = [rnd(n, 1e-3, torch.bfloat16) for n in numels]
    ag_in = torch.zeros(s, dtype=torch.bfloat16, device=DEV)
    outs = [torch.zeros(n, dtype=torch.bfloat16, device=DEV) for n in numels]
    rs = torch.zeros(t_pad, dtype=torch.bfloat16, device=DEV)
    shard = rnd(s, 1e-4, torch.float32)
    table = _native.TensorTable(numels, t_pad, DEV)

    def step(ag_in_, outs_, rs_, shard_):
        _native.flat_copy(ag_in_, master)
        table.scatter_out(gathered, outs_)
        table.gather_in(grads, rs_, None, float(w), True)
        _native.post_reduce(shard_, rs_[r * s : (r + 1) * s], None, True)

    # warm up on a side stream, then capture
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step(ag_in, outs, rs, shard.clone())
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    shard_graph = shard.clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step(ag_in, outs, rs, shard_graph)
    shard_graph.copy_(shard)  # capture does not execute; start both accumulators from the same state
    shard_eager = shard.clone()
    for it in range(4):
        # new inputs in place (same addresses), then eager reference on separate outputs
        master.add_(0.001 * (it + 1))
        gathered.mul_(1.0 + 0.125 * it)
        for gr in grads:
            gr.mul_(0.5)
        e_ag, e_outs = torch.zeros_like(ag_in), [torch.zeros_like(o) for o in outs]
        e_rs = torch.zeros_like(rs)
        step(e_ag, e_outs, e_rs, shard_eager)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert_bits_equal(ag_in, e_ag.cpu(), f"replay {it}: copy-in")
        for a, b in zip(outs, e_outs):
            assert_bits_equal(a, b.cpu(), f"replay {it}: copy-out")
        assert_bits_equal(rs, e_rs.cpu(), f"replay {it}: reduce copy-in")
        assert_bits_equal(shard_graph, shard_eager.cpu(), f"replay {it}: post-reduce")
    table.close()


def test_bound_large_table_replays_match_eager():
    """With a binding, a table of more than 16 tensors (metadata in device memory) needs no per-call staging
    copy, so its launches can be captured too."""
    import numpy as np

    from yafsdp_amd import _native

    rng = np.random.default_rng(5)
    numels = (np.floor(np.exp2(rng.uniform(0, 15, size=120))).astype(np.int64) | 1).tolist()
    t = sum(numels)
    t_pad = t + 37
    g = torch.Generator(device=DEV).manual_seed(78)
    grads = [(torch.randn(n, device=DEV, generator=g) * 1e-3).bfloat16() for n in numels]
    gathered = (torch.randn(t_pad, device=DEV, generator=g) * 0.02).bfloat16()
    outs = [torch.zeros(n, dtype=torch.bfloat16, device=DEV) for n in numels]
    rs = torch.zeros(t_pad, dtype=torch.float32, device=DEV)
    table = _native.TensorTable(numels, t_pad, DEV)
    gb, sb = table.bind(grads), table.bind(outs)

    def step():
        sb.scatter_out(gathered)
        gb.gather_in(rs, 8.0, True)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for it in range(3):
        gathered.mul_(1.0 + 0.25 * it)
        for gr in grads:
            gr.mul_(0.5)
        e_outs = [torch.zeros_like(o) for o in outs]
        e_rs = torch.zeros_like(rs)
        table.scatter_out(gathered, e_outs)
        table.gather_in(grads, e_rs, None, 8.0, True)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for a, b in zip(outs, e_outs):
            assert_bits_equal(a, b.cpu(), f"replay {it}: copy-out")
        assert_bits_equal(rs, e_rs.cpu(), f"replay {it}: reduce copy-in")
    gb.close(), sb.close(), table.close()


def test_captured_optimizer_side_replays_match_eager():
    """Post-reduce with the fused squared norm, the two-stage sum of its partial sums, the clip coefficient and the
    fused AdamW pass captured into one HIP graph (kernel launches only) and replayed with new gradients each time."""
    from yafsdp_amd import _native

    n = 300_000
    g = torch.Generator(device=DEV).manual_seed(78)

    def rnd(std, dt=torch.float32):
        return (torch.randn(n, device=DEV, generator=g) * std).to(dt)

    chunk = rnd(1e-3, torch.bfloat16)
    state0 = [rnd(0.02), rnd(1e-4), rnd(1e-3), rnd(1e-3) ** 2]           # param, grad shard, exp_avg, exp_avg_sq
    hp = dict(lr=1e-3, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1, step=3)

    def make():
        return dict(
            st=[x.clone() for x in state0], out16=torch.zeros(n, dtype=torch.bfloat16, device=DEV),
            partials=torch.zeros(_native.post_reduce_sumsq_count(n), dtype=torch.float64, device=DEV),
            stage=torch.zeros(8, dtype=torch.float64, device=DEV), nc=torch.zeros(2, device=DEV),
        )

    def step(b):
        p, grad, m, v = b["st"]
        count = _native.post_reduce_sumsq(grad, chunk, 8.0, True, b["partials"])
        count = _native.sumsq_reduce_partials(b["partials"], count, b["stage"])
        _native.clip_coef_from_partials(b["stage"], count, 1e-3, b["nc"])
        _native.adamw_step(p, grad, m, v, b["out16"], grad_scale=b["nc"][1:2], zero_grad=False, **hp)

    eager, captured = make(), make()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step(make())  # warm up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step(captured)
    for it in range(4):
        chunk.mul_(0.5 + 0.25 * it)   # new gradients in place, eager work between the replays
        step(eager)
        graph.replay()
        torch.cuda.synchronize()
        for name, a, b in zip(("param", "grad", "exp_avg", "exp_avg_sq"), captured["st"], eager["st"]):
            assert_bits_equal(a, b, f"{name}, replay {it}")
        assert_bits_equal(captured["out16"], eager["out16"], f"out16, replay {it}")
        assert torch.equal(captured["nc"], eager["nc"]), it
    del graph


def test_captured_byte_copy_replays_match_eager():
    """The byte copy of a 1-byte all-gather dtype (odd addresses, head and tail bytes) is kernel launches only:
    captured once, replayed with new contents at the same addresses, with eager work in between."""
    from yafsdp_amd import _native

    n = 300_007
    g = torch.Generator(device=DEV).manual_seed(5)
    src_buf = torch.randint(0, 256, (n + 16,), device=DEV, dtype=torch.uint8, generator=g)
    dst_buf = torch.zeros(n + 32, dtype=torch.uint8, device=DEV)
    src, dst = src_buf[3 : 3 + n].view(torch.int8), dst_buf[5 : 5 + n].view(torch.int8)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        _native.flat_copy(dst, src)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _native.flat_copy(dst, src)
    for it in range(4):
        src_buf.copy_(torch.randint(0, 256, (n + 16,), device=DEV, dtype=torch.uint8, generator=g))
        dst_buf.fill_(0xEE)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want = torch.full((n + 32,), 0xEE, dtype=torch.uint8)
        want[5 : 5 + n] = src_buf[3 : 3 + n].cpu()
        assert torch.equal(dst_buf.cpu(), want), f"replay {it}"
        # eager work between the replays
        eager = torch.zeros(n, dtype=torch.int8, device=DEV)
        _native.flat_copy(eager, src)
        assert torch.equal(eager.cpu(), src.cpu())
