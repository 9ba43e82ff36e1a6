"""Six parameter groups that share the 2 + 1 buffers of one shard group run a forward and a backward pass with
prefetch while GEMMs keep the compute stream busy: the copy kernels on the side stream really run next to other
work, and every hand-over of a shared buffer goes through the owner / release-event protocol
(ya_fsdp/_param_group.py:567-576, 660-668, 770-771).  Every gradient shard, all-gather input and gathered slot is
compared bit for bit with the reference's op sequence on the CPU."""

import pytest
import torch

from tests.helpers import assert_bits_equal
from tests.test_gpu_param_group import BF16_MP, CpuGroup, _grads, _params
from yafsdp_amd import FSDPMeshInfo

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")

GROUP_SHAPES = [
    [(3000, 2048), (2048,), (1111, 2048)],
    [(2048, 2048)] * 3 + [(5003, 2048), (2048,)],
    [(4096, 1024), (1024, 4096), (77,)],
    [(2048, 2048)] * 3 + [(5003, 2048), (2048,)],
    [(8191, 1024), (1024,)],
    [(2048,), (2048, 3001)],
]


@pytest.mark.parametrize("w,r", [(4, 2), (1, 0), (3, 1)])
@pytest.mark.parametrize("copy_in_on_side_stream", [False, True])
def test_groups_sharing_buffers_under_concurrent_gemms(w, r, copy_in_on_side_stream):
    from yafsdp_amd._param_group import YaFSDPParamGroup, init_shared_state

    align = 512
    groups, refs = [], []
    for k, shapes in enumerate(GROUP_SHAPES):
        cpu_params = _params(shapes, torch.float32, 100 + k, norms_are_ones=False)
        dev_params = [p.to(DEV).requires_grad_(True) for p in cpu_params]
        groups.append(YaFSDPParamGroup(dev_params, FSDPMeshInfo(w, r), DEV, BF16_MP, align))
        refs.append(CpuGroup(cpu_params, w, r, align, BF16_MP))
    for g in groups:
        # the opt-in stream plan: reduce copy-in on the reduce-scatter stream, right in front of the post-reduce
        g.reduce_copy_in_on_side_stream = copy_in_on_side_stream
    init_shared_state(groups, DEV)  # 2 data buffers handed out round-robin, 1 gradient buffer
    assert len({id(g.data_buffer_ctx) for g in groups}) == 2 and len({id(g.grad_buffer_ctx) for g in groups}) == 1
    n = len(groups)
    a = torch.randn(4096, 4096, device=DEV).bfloat16()
    b = torch.randn(4096, 4096, device=DEV).bfloat16()
    c = torch.empty(4096, 4096, dtype=torch.bfloat16, device=DEV)

    def gemm(k=1):
        for _ in range(k):
            torch.matmul(a, b, out=c)

    collective = ("AVG", None) if w > 1 else None  # bf16 reduce: the collective scales by 1 / W rounded to bf16
    for it in range(2):
        print("iteration", it, "w", w, flush=True)
        snaps = [None] * n
        grads_cpu = [_grads(GROUP_SHAPES[k], torch.bfloat16, 1000 * it + k) for k in range(n)]
        grads_dev = [[x.to(DEV) for x in gs] for gs in grads_cpu]
        torch.cuda.synchronize()
        # ---- forward with prefetch of the next group
        for i, g in enumerate(groups):
            g.pre_forward()
            if i + 1 < n:
                YaFSDPParamGroup._prefetch_unshard(groups[i + 1], "forward")
            gemm(2)
            s_ = g.layout.padded_sharded_numel
            snaps[i] = (g._all_gather_output[None][r * s_ : (r + 1) * s_].clone(), g._all_gather_input[None].clone())
            gemm(1)
            g.post_forward()
        # ---- backward in reverse order; post_backward hands the one gradient buffer from group to group
        for i in reversed(range(n)):
            g = groups[i]
            g.pre_backward()
            gemm(3)
            for fp, x in zip(g.fsdp_params, grads_dev[i]):
                fp.unsharded_param.grad = x
            flags = [fp.unsharded_accumulated_grad is not None for fp in g.fsdp_params]
            g.post_backward()
            refs[i].accumulate(grads_cpu[i], flags)
        for g in groups:
            g.finalize_backward()
        torch.cuda.synchronize()
        for i, (g, ref) in enumerate(zip(groups, refs)):
            ref.unshard(first_of_iteration=True)
            ref.reduce(None, None, "copy" if it == 0 else "add", collective=collective)
            assert_bits_equal(snaps[i][1], ref.ag_in, f"iteration {it} group {i}: all-gather input")
            assert_bits_equal(snaps[i][0], ref.ag_in, f"iteration {it} group {i}: this rank's slot of the gathered buffer")
            assert_bits_equal(g._padded_sharded_param_grad[None], ref.grad_shard, f"iteration {it} group {i}: grad shard")
            assert g.grad_buffer_ctx.owner is None and g.data_buffer_ctx.owner is None
