"""The benchmark configurations at their real sizes, through the C ABI.

Config 2 (Llama-3-8B layer, W=8) and config 5 (2000 ragged tensors, W=256) are
compared element for element with the oracle.  Config 3 (Llama-3-70B layer,
W=64; 856 M elements) is checked through size-independent properties at full
size (round trips, linearity of the divide, pad zero-fill, checksums), against
the oracle element for element on the fused reduce copy-in with its divide by
64, and against the oracle on the last rank's shard, which holds the pad lanes.
Config 4 (the full 8B model) adds the embedding / head group (525 M elements,
one tensor) and the final-norm group (4096 elements) to config 2's layers.
Inputs are generated on the GPU from a fixed seed and copied to the host for
the oracle, so both sides see the same bits.
"""

import numpy as np
import pytest
import torch

from oracle import torch_ops
from tests.helpers import assert_bits_equal
from yafsdp_amd import make_layout

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")

LLAMA8B = [(4096, 4096), (1024, 4096), (1024, 4096), (4096, 4096), (14336, 4096), (14336, 4096), (4096, 14336),
           (4096,), (4096,)]
LLAMA70B = [(8192, 8192), (1024, 8192), (1024, 8192), (8192, 8192), (28672, 8192), (28672, 8192), (8192, 28672),
            (8192,), (8192,)]


def _numel(s):
    n = 1
    for d in s:
        n *= d
    return n


def _randn_dev(n, std, dtype, gen):
    out = torch.empty(n, dtype=dtype, device=DEV)
    step = 1 << 26
    for i in range(0, n, step):
        m = min(step, n - i)
        out[i : i + m] = (torch.randn(m, device=DEV, generator=gen) * std).to(dtype)
    return out


@pytest.fixture(scope="module")
def nat():
    from yafsdp_amd import _native

    return _native


@pytest.fixture(params=["single_set", "rotating_sets", "tails_on_both_table_kernels"])
def store_policy(request, nat):
    """Which stores write through: at these sizes the boundary between the two kinds of stores lies inside the
    buffers (the conftest fixture restores the library's defaults before the next test)."""
    named = {"tails_on_both_table_kernels": (1 << 20, 1 << 20, 32, 56)}
    nat.set_store_policy(named.get(request.param, request.param))
    return request.param


def test_config2_llama8b_layer_w8(nat, store_policy):
    print("config 2", store_policy, flush=True)
    numels = [_numel(s) for s in LLAMA8B]
    w = 8
    lay = make_layout(numels, w, 512)
    t, t_pad, s = lay.total_numel, lay.padded_unsharded_numel, lay.padded_sharded_numel
    assert (t, t_pad, s) == (218_112_000, 218_112_000, 27_264_000)
    gen = torch.Generator(device=DEV).manual_seed(1002)
    gathered = _randn_dev(t_pad, 0.02, torch.bfloat16, gen)
    grads = [_randn_dev(n, 1e-3, torch.bfloat16, gen) for n in numels]
    table = nat.TensorTable(numels, t_pad, DEV)
    # copy-out
    outs = [torch.empty(n, dtype=torch.bfloat16, device=DEV) for n in numels]
    table.scatter_out(gathered, outs)
    gathered_cpu = gathered.cpu()
    want = [torch.empty(n, dtype=torch.bfloat16) for n in numels]
    torch_ops.copy_out_materialize(gathered_cpu, numels, want)
    for i, (a, b) in enumerate(zip(outs, want)):
        assert_bits_equal(a, b, f"copy-out tensor {i}")
    del outs, want
    # reduce copy-in with /8 pre-divide
    rs = torch.zeros(t_pad, dtype=torch.bfloat16, device=DEV)
    table.gather_in(grads, rs, None, 8.0, True)
    grads_cpu = [g.cpu() for g in grads]
    rs_cpu = torch.zeros(t_pad, dtype=torch.bfloat16)
    torch_ops.reduce_copy_in(list(rs_cpu[:t].split(numels)), grads_cpu, False)
    torch_ops.div_if_needed(rs_cpu, 8.0)
    assert_bits_equal(rs, rs_cpu, "reduce copy-in")
    # copy-in and post-reduce for ragged ranks (0: q,k,v,o-head; 3: gate/up boundary; 7: down tail + norms)
    for r in (0, 3, 7):
        print("  rank", r, flush=True)
        master = _randn_dev(s, 0.02, torch.float32, gen)
        ag_in = torch.zeros(s, dtype=torch.bfloat16, device=DEV)
        nat.flat_copy(ag_in, master)
        ag_cpu = torch.zeros(s, dtype=torch.bfloat16)
        torch_ops.copy_in(ag_cpu, master.cpu())
        assert_bits_equal(ag_in, ag_cpu, f"copy-in rank {r}")
        shard = _randn_dev(s, 1e-4, torch.float32, gen)
        shard_cpu = shard.cpu()
        nat.post_reduce(shard, rs[r * s : (r + 1) * s], None, True)
        torch_ops.reduce_scatter_local(shard_cpu, rs_cpu.clone(), w, r, None, None, "add")
        assert_bits_equal(shard, shard_cpu, f"post-reduce rank {r}")
    table.close()


def _checksum(x: torch.Tensor) -> int:
    return int(x.view(torch.int16).to(torch.int64).sum().item()) if x.numel() else 0


def test_config3_llama70b_layer_w64_properties(nat):
    print("config 3", flush=True)
    numels = [_numel(s) for s in LLAMA70B]
    w, r = 64, 63
    lay = make_layout(numels, w, 512)
    t, t_pad, s = lay.total_numel, lay.padded_unsharded_numel, lay.padded_sharded_numel
    assert (t, t_pad, s) == (855_654_400, 855_670_784, 13_369_856) and lay.pad_numel(r) == 16_384
    gen = torch.Generator(device=DEV).manual_seed(1003)
    gathered = _randn_dev(t_pad, 0.02, torch.bfloat16, gen)
    gathered[t:] = 7.0  # pad lanes of the source must never be read
    table = nat.TensorTable(numels, t_pad, DEV)
    outs = [torch.full((n,), 3.0, dtype=torch.bfloat16, device=DEV) for n in numels]
    table.scatter_out(gathered, outs)
    # (a) byte identity with the split of the source, tensor by tensor, on the GPU
    pos = 0
    for i, (o, n) in enumerate(zip(outs, numels)):
        assert torch.equal(o.view(torch.int16), gathered[pos : pos + n].view(torch.int16)), f"copy-out tensor {i}"
        pos += n
    # (b) checksum of checksums
    assert sum(_checksum(o) for o in outs) == _checksum(gathered[:t])
    # (c) scatter -> gather round trip restores [0, T) and zero-fills the pad
    back = torch.full((t_pad,), 5.0, dtype=torch.bfloat16, device=DEV)
    table.gather_in(outs, back, None, None, True)
    assert torch.equal(back[:t].view(torch.int16), gathered[:t].view(torch.int16))
    assert int(back[t:].view(torch.int16).abs().max().item()) == 0
    # (d) fused pre-divide == copy followed by the stand-alone in-place divide (both bit-exact paths)
    fused = torch.zeros(t_pad, dtype=torch.bfloat16, device=DEV)
    table.gather_in(outs, fused, None, 64.0, True)
    nat.flat_div(back, 64.0)
    assert torch.equal(fused.view(torch.int16), back.view(torch.int16))
    # (d') the fused copy + divide by 64 against the reference's ops at full size, element for element:
    # _foreach_copy_ into the views of the reduce buffer (ya_fsdp/_param_group.py:693-700), then div_ of the padded
    # buffer (ya_fsdp/_collectives.py:139) on an 856 M-element bf16 buffer on the host
    outs_cpu = [o.cpu() for o in outs]
    rs_cpu = torch.zeros(t_pad, dtype=torch.bfloat16)
    torch_ops.reduce_copy_in(list(rs_cpu[:t].split(numels)), outs_cpu, False)
    torch_ops.div_if_needed(rs_cpu, 64.0)
    fused_cpu = fused.cpu()
    assert torch.equal(fused_cpu.view(torch.int16), rs_cpu.view(torch.int16)), "fused reduce copy-in /64 vs the oracle"
    del outs_cpu, rs_cpu, fused_cpu
    # (e) accumulate twice == exact doubling (x + x is exact in bf16 unless it overflows)
    acc = torch.zeros(t_pad, dtype=torch.bfloat16, device=DEV)
    table.gather_in(outs, acc, None, None, True)
    table.gather_in(outs, acc, [2] * len(numels), None, True)
    assert torch.equal(acc[:t].view(torch.int16), (gathered[:t].float() * 2).bfloat16().view(torch.int16))
    # (f) the last rank's shard (down tail + both norms + 16384 pad lanes) against the oracle
    del back, acc
    chunk = fused[r * s : (r + 1) * s]
    shard = _randn_dev(s, 1e-4, torch.float32, gen)
    shard_cpu, chunk_cpu = shard.cpu(), chunk.cpu()
    nat.post_reduce(shard, chunk, None, True)
    shard_cpu.add_(chunk_cpu)  # ya_fsdp/_collectives.py:189
    assert_bits_equal(shard, shard_cpu, "post-reduce last rank")
    assert torch.equal(shard[-16_384:].cpu(), shard_cpu[-16_384:])
    master = _randn_dev(s, 0.02, torch.float32, gen)
    ag_in = torch.zeros(s, dtype=torch.bfloat16, device=DEV)
    nat.flat_copy(ag_in, master)
    want = torch.zeros(s, dtype=torch.bfloat16)
    torch_ops.copy_in(want, master.cpu())
    assert_bits_equal(ag_in, want, "copy-in last rank")
    table.close()


def _stress_numels(seed=1005, p=2000):
    g = torch.Generator().manual_seed(seed)
    u = torch.rand(p, generator=g, dtype=torch.float64) * 22 * np.log(2.0)
    numels = (torch.exp(u).floor().to(torch.int64) | 1).tolist()
    is_fp32_master = (torch.rand(p, generator=g) < 0.7).tolist()
    return numels, is_fp32_master


@pytest.mark.parametrize("which", ["fp32-masters/bf16-compute", "bf16-masters/fp32-reduce"])
def test_config5_ragged_stress_w256(nat, which, store_policy):
    print("config 5", which, flush=True)
    all_numels, is_fp32 = _stress_numels()
    if which.startswith("fp32"):
        numels = [n for n, f in zip(all_numels, is_fp32) if f]
        master_dt, grad_dt, rs_dt, shard_dt = torch.float32, torch.bfloat16, torch.bfloat16, torch.float32
    else:
        numels = [n for n, f in zip(all_numels, is_fp32) if not f]
        master_dt, grad_dt, rs_dt, shard_dt = torch.bfloat16, torch.bfloat16, torch.float32, torch.bfloat16
    assert all(n % 2 == 1 and 1 <= n <= 2**22 for n in numels)
    w = 256
    lay = make_layout(numels, w, 512)
    t, t_pad, s = lay.total_numel, lay.padded_unsharded_numel, lay.padded_sharded_numel
    print(f"  P={len(numels)} T={t} T_pad={t_pad} S={s}", flush=True)
    gen = torch.Generator(device=DEV).manual_seed(1005)
    ag_dt = torch.bfloat16
    gathered = _randn_dev(t_pad, 0.02, ag_dt, gen)
    grads = [_randn_dev(n, 1e-3, grad_dt, gen) for n in numels]
    table = nat.TensorTable(numels, t_pad, DEV)
    # copy-out into 2000 separately allocated odd-sized tensors
    outs = [torch.empty(n, dtype=ag_dt, device=DEV) for n in numels]
    table.scatter_out(gathered, outs)
    got_flat = torch.cat(outs)
    assert torch.equal(got_flat.view(torch.int16), gathered[:t].view(torch.int16)), "copy-out"
    del got_flat, outs
    # reduce copy-in: first micro-batch copy (+/256 pre-divide), second micro-batch accumulate
    rs = torch.zeros(t_pad, dtype=rs_dt, device=DEV)
    grads_cpu = [g.cpu() for g in grads]
    rs_cpu = torch.zeros(t_pad, dtype=rs_dt)
    views = list(rs_cpu[:t].split(numels))
    table.gather_in(grads, rs)                                       # copy, no divide
    torch_ops.reduce_copy_in(views, grads_cpu, False)
    assert_bits_equal(rs, rs_cpu, "reduce copy-in (copy)")
    table.gather_in(grads, rs, [2] * len(numels), 256.0, True)       # accumulate, then /256
    torch_ops.reduce_copy_in(views, grads_cpu, True)
    torch_ops.div_if_needed(rs_cpu, 256.0)
    assert_bits_equal(rs, rs_cpu, "reduce copy-in (add, /256)")
    # ranks whose shard starts and ends mid-tensor, plus rank 0 and the last rank (pad lanes)
    offs = set(lay.offsets)
    mid = [r for r in range(1, w - 1) if r * s not in offs and (r + 1) * s not in offs][:2]
    for r in [0, *mid, w - 1]:
        sn = lay.sharded_numels(r)
        n_frag = sum(1 for x in sn if x)
        print(f"  rank {r}: {n_frag} fragments, pad {lay.pad_numel(r)}", flush=True)
        chunk = rs[r * s : (r + 1) * s]
        shard = _randn_dev(s, 1e-4, shard_dt, gen)
        shard_cpu = shard.cpu()
        nat.post_reduce(shard, chunk, None, True)
        shard_cpu.add_(rs_cpu[r * s : (r + 1) * s])
        assert_bits_equal(shard, shard_cpu, f"post-reduce rank {r}")
        # mixed fragments: every other non-empty fragment already owns a gradient
        shard2 = _randn_dev(s, 1e-4, shard_dt, gen)
        shard2_cpu = shard2.cpu()
        has, k = [], 0
        for x in sn:
            if x == 0:
                has.append(None)
            else:
                has.append(k % 2 == 0)
                k += 1
        modes = [0 if h is None else (2 if h else 1) for h in has]
        nat.post_reduce_fragments(shard2, chunk, sn, modes, None)
        torch_ops.reduce_scatter_local(shard2_cpu, rs_cpu.clone(), w, r, None, None, "mixed", sn, has)
        assert_bits_equal(shard2, shard2_cpu, f"post-reduce fragments rank {r}")
        if master_dt != ag_dt:  # copy-in exists only for the fp32-master group
            master = _randn_dev(s, 0.02, master_dt, gen)
            ag_in = torch.zeros(s, dtype=ag_dt, device=DEV)
            nat.flat_copy(ag_in, master)
            want = torch.zeros(s, dtype=ag_dt)
            torch_ops.copy_in(want, master.cpu())
            assert_bits_equal(ag_in, want, f"copy-in rank {r}")
    table.close()


def test_config4_full_8b_groups_besides_the_decoder_layers(nat):
    """Config 4 (the full Llama-3-8B at W=8) adds three groups to the 32 decoder layers of config 2: the token
    embedding and the output head (one [128256, 4096] tensor each: T = 525,336,576, S = 65,667,072) and the final
    norm ([4096]: S = 512).  The large group is checked through size-independent properties at full size and against
    the oracle on one rank's shard, the small one element for element on every rank."""
    print("config 4: embedding / head group", flush=True)
    numels = [128256 * 4096]
    w, r = 8, 5
    lay = make_layout(numels, w, 512)
    t, t_pad, s = lay.total_numel, lay.padded_unsharded_numel, lay.padded_sharded_numel
    assert (t, t_pad, s) == (525_336_576, 525_336_576, 65_667_072)
    gen = torch.Generator(device=DEV).manual_seed(1004)
    gathered = _randn_dev(t_pad, 0.02, torch.bfloat16, gen)
    table = nat.TensorTable(numels, t_pad, DEV)
    out = torch.full((t,), 3.0, dtype=torch.bfloat16, device=DEV)
    table.scatter_out(gathered, [out])
    assert torch.equal(out.view(torch.int16), gathered.view(torch.int16))              # copy-out: byte identity
    fused = torch.full((t_pad,), 5.0, dtype=torch.bfloat16, device=DEV)
    table.gather_in([out], fused, None, 8.0, True)                                    # reduce copy-in with /8
    assert torch.equal(fused.view(torch.int16), (gathered.float() / 8.0).bfloat16().view(torch.int16))
    del out
    chunk = fused[r * s : (r + 1) * s]
    shard = _randn_dev(s, 1e-4, torch.float32, gen)
    shard_cpu, chunk_cpu = shard.cpu(), chunk.cpu()
    nat.post_reduce(shard, chunk, None, True)
    shard_cpu.add_(chunk_cpu)  # ya_fsdp/_collectives.py:189
    assert_bits_equal(shard, shard_cpu, "post-reduce")
    master = _randn_dev(s, 0.02, torch.float32, gen)
    ag_in = torch.zeros(s, dtype=torch.bfloat16, device=DEV)
    nat.flat_copy(ag_in, master)
    want = torch.zeros(s, dtype=torch.bfloat16)
    torch_ops.copy_in(want, master.cpu())
    assert_bits_equal(ag_in, want, "copy-in")
    table.close()
    del gathered, fused, shard, master

    print("config 4: final norm group", flush=True)
    numels = [4096]
    lay = make_layout(numels, w, 512)
    t, t_pad, s = lay.total_numel, lay.padded_unsharded_numel, lay.padded_sharded_numel
    assert (t, t_pad, s) == (4096, 4096, 512)
    g = torch.Generator().manual_seed(1004)
    gathered = (torch.randn(t_pad, generator=g) * 0.02).bfloat16()
    grad = (torch.randn(t, generator=g) * 1e-3).bfloat16()
    table = nat.TensorTable(numels, t_pad, DEV)
    out = torch.empty(t, dtype=torch.bfloat16, device=DEV)
    table.scatter_out(gathered.to(DEV), [out])
    assert_bits_equal(out, gathered[:t], "copy-out")
    rs = torch.zeros(t_pad, dtype=torch.bfloat16, device=DEV)
    table.gather_in([grad.to(DEV)], rs, None, 8.0, True)
    rs_cpu = torch.zeros(t_pad, dtype=torch.bfloat16)
    torch_ops.reduce_copy_in([rs_cpu[:t]], [grad], False)
    torch_ops.div_if_needed(rs_cpu, 8.0)
    assert_bits_equal(rs, rs_cpu, "reduce copy-in")
    for rank in range(w):
        shard0 = torch.randn(s, generator=g) * 1e-4
        shard = shard0.to(DEV)
        nat.post_reduce(shard, rs[rank * s : (rank + 1) * s], None, True)
        want = shard0.clone()
        torch_ops.reduce_scatter_local(want, rs_cpu.clone(), w, rank, None, None, "add")
        assert_bits_equal(shard, want, f"post-reduce rank {rank}")
    table.close()
