"""Entry points are re-entrant: two host threads drive the same table and the
flat kernels on their own streams at the same time (as the main thread and the
autograd engine thread do in training); every result must still be exact."""

import threading

import pytest
import torch

from oracle import torch_ops
from tests.helpers import assert_bits_equal

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def test_two_threads_share_a_table():
    from yafsdp_amd import _native

    numels = [4099, 1, 70001, 333, 8192, 5]
    t = sum(numels)
    t_pad = t + 11
    table = _native.TensorTable(numels, t_pad, DEV)
    errors = []

    def worker(seed):
        try:
            torch.cuda.set_device(DEV)
            stream = torch.cuda.Stream()
            g = torch.Generator().manual_seed(seed)
            for it in range(25):
                flat = (torch.randn(t_pad, generator=g) * 0.02).bfloat16()
                grads = [(torch.randn(n, generator=g) * 1e-3).bfloat16() for n in numels]
                want_outs = [torch.empty(n, dtype=torch.bfloat16) for n in numels]
                torch_ops.copy_out_materialize(flat, numels, want_outs)
                want_rs = torch.zeros(t_pad, dtype=torch.bfloat16)
                torch_ops.reduce_copy_in(list(want_rs[:t].split(numels)), grads, False)
                torch_ops.div_if_needed(want_rs, 4.0)
                with torch.cuda.stream(stream):
                    d_flat = flat.to(DEV)
                    d_grads = [x.to(DEV) for x in grads]
                    outs = [torch.empty(n, dtype=torch.bfloat16, device=DEV) for n in numels]
                    rs = torch.zeros(t_pad, dtype=torch.bfloat16, device=DEV)
                    table.scatter_out(d_flat, outs)
                    table.gather_in(d_grads, rs, None, 4.0, True)
                    f32 = torch.empty(t_pad, dtype=torch.float32, device=DEV)
                    _native.flat_copy(f32, rs)
                stream.synchronize()
                for a, b in zip(outs, want_outs):
                    assert_bits_equal(a, b, f"thread {seed} it {it} scatter")
                assert_bits_equal(rs, want_rs, f"thread {seed} it {it} gather")
                assert_bits_equal(f32, want_rs.float(), f"thread {seed} it {it} cast")
        except Exception as e:  # surfaced in the main thread
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(s,)) for s in (1, 2)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    table.close()
    assert not errors, errors[0]
