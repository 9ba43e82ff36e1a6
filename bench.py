#!/usr/bin/env python3
"""Benchmark of the per-rank buffer hot path on one MI355X.

One "step" is one pass of the path over one batch of synthetic input, in the
order a training step runs it for one parameter group:

    copy-in         fp32 master shard [S]          -> bf16 all-gather input [S]
    copy-out        bf16 gathered buffer [T_pad]   -> P separately allocated tensors
    reduce copy-in  P bf16 gradients               -> bf16 reduce buffer [T_pad], fused /pre, pad zero-fill
    post-reduce     rank's bf16 chunk [S]          -> += into the fp32 gradient shard [S]

Default workload: one Llama-3-8B decoder layer at logical world size 8, one
rank's share.  Inputs are resident in HBM before the timed region starts.
Prints ONE JSON line on stdout; progress goes to stderr.
"""

from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E peak

WORKLOADS = {
    # name: (shapes in parameter order q,k,v,o,gate,up,down,norm,norm; W; rank; alignment; seed)
    "llama3-8b-layer-w8": (
        [(4096, 4096), (1024, 4096), (1024, 4096), (4096, 4096), (14336, 4096), (14336, 4096), (4096, 14336),
         (4096,), (4096,)], 8, 3, 512, 1002),
    "llama3-70b-layer-w64": (
        [(8192, 8192), (1024, 8192), (1024, 8192), (8192, 8192), (28672, 8192), (28672, 8192), (8192, 28672),
         (8192,), (8192,)], 64, 63, 512, 1003),
    "tiny-layer-w1": (
        [(512, 512)] * 4 + [(1376, 512), (1376, 512), (512, 1376), (512,), (512,)], 1, 0, 512, 1001),
}


def _ragged_stress_shapes(seed=1005, p=2000, fp32_masters=True):
    """2,000 tensors with odd element counts, log-uniform in [1, 2^22], 70 % drawn as fp32 masters with bf16
    compute and 30 % as bf16 masters with fp32 reduce; a group has one master dtype, so the two classes are two
    groups (two workloads here)."""
    import torch

    g = torch.Generator().manual_seed(seed)
    u = torch.rand(p, generator=g, dtype=torch.float64) * 22 * 0.6931471805599453
    numels = (torch.exp(u).floor().to(torch.int64) | 1).tolist()
    is_fp32_master = (torch.rand(p, generator=g) < 0.7).tolist()
    return [(n,) for n, f in zip(numels, is_fp32_master) if f == fp32_masters]

# HBM bytes per launch of the dominant kernel (gather_in_kernel), from two rocprofv3 --pmc runs
# (FETCH_SIZE, WRITE_SIZE) of the default command (four buffer sets in rotation), each scaled by the reading of a
# plain copy of known size (factors 1.99986 and 1.00000): (213073.8 * 1.99986 + 426081.6 * 1.00000) KiB.
# Summary and commands: profiles/bench_llama3-8b-layer-w8_hbm_traffic.md.  None = not measured.
# "llama3-8b-layer-w8-optim": adamw_kernel, (213045.6 * 1.99946 + 372753.5 * 0.99996) KiB, scaled by the plain
# fp32 copy of the same run; profiles/bench_llama3-8b-layer-w8-optim_hbm_traffic.md.
# "ragged-stress-w256": gather_in_kernel<LargeMeta>, (379903.9 * 1.99992 + 710944.2 * 0.99984) KiB;
# profiles/bench_ragged-stress-w256_hbm_traffic.md.
# "llama3-70b-layer-w64": gather_in_kernel<SmallMeta,...,128,2>, (835642.75 * 1.99997 + 1671299.6 * 1.00000) KiB;
# "ragged-stress-w256-bf16-masters": gather_in_kernel<LargeMeta,BF16,F32>, (178792.9 * 1.99987 + 633008.8) KiB (the
# reads are 13 % above the algorithmic 323.8 MB: 573 bf16 sources at odd offsets, 2 KB per tile);
# "tiny-layer-w1": gather_post_kernel, (9309.25 * 1.99322 + 18534.0) KiB, below the algorithmic bytes of the two
# kernels it replaces because the reduce buffer is not read back;
# all three in profiles/bench_llama3-8b-layer-w8_hbm_traffic.md.
# Megabytes a GEMM stand-in of the full-model workload moves between the L2s and the memory side per launch
# (TCC_EA0_RDREQ x 128 B + TCC_EA0_WRREQ x 64 B of the hipBLASLt kernel alone; profiles/bench_llama3-8b-full-w8_overlap.md),
# and the rate at which a copy kernel of the path moves its bytes when it has the memory side to itself.
GEMM_MEMORY_SIDE_MB = {"4096x4096x4096": 201.8 + 33.6, "llama-mlp-up 4096x4096x14336": 755.4 + 117.4,
                       "llama-mlp-down 4096x14336x4096": 705.1 + 33.6}
COPY_RATE_MB_PER_MS = 6550.0
MEASURED_TRAFFIC_BYTES = {"llama3-8b-layer-w8": 872_652_200, "llama3-8b-layer-w8-optim": 817_885_000,
                          "ragged-stress-w256": 1_505_902_865, "llama3-70b-layer-w64": 3_422_785_664,
                          "ragged-stress-w256-bf16-masters": 1_014_344_628, "tiny-layer-w1": 37_979_573}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def _event_pair():
    """Two timing events whose HIP handles exist (torch creates them on the first record)."""
    import torch

    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    b.record()
    return a, b


def numel_of(shape):
    n = 1
    for d in shape:
        n *= d
    return n


def _cu_masked_streams(torch, dev, k: int):
    """Two streams of the HIP runtime this process already uses: one limited to compute units [0, k), one to
    [k, 256)."""
    import ctypes

    if not 0 < k < 256:
        raise SystemExit("--copy-cus must lie in 1..255")
    path = next(line.split()[-1] for line in open("/proc/self/maps") if "libamdhip64" in line)
    hip = ctypes.CDLL(path)
    hip.hipExtStreamCreateWithCUMask.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_uint32,
                                                 ctypes.POINTER(ctypes.c_uint32)]
    out = []
    for bits in (range(k), range(k, 256)):
        words = [0] * 8
        for b in bits:
            words[b // 32] |= 1 << (b % 32)
        handle = ctypes.c_void_p()
        rc = hip.hipExtStreamCreateWithCUMask(ctypes.byref(handle), 8, (ctypes.c_uint32 * 8)(*words))
        if rc != 0:
            raise RuntimeError(f"hipExtStreamCreateWithCUMask failed with {rc}")
        out.append(torch.cuda.ExternalStream(handle.value, device=dev))
    return out


def analyze_overlap_trace(path: str) -> int:
    """Reads the kernel trace (CSV) that ``rocprofv3 --kernel-trace --output-format csv`` wrote for
    ``--workload llama3-8b-full-w8 --steps 10 --no-parity`` and prints, per GEMM stand-in: the register, LDS and
    workgroup columns of the GEMM kernel, kernel durations alone and inside the overlapped pass, and for how long
    GEMMs, copy kernels and both at once were running during that pass."""
    import csv

    def kind(name):
        if name.startswith("Cijk"):
            return "gemm"
        for key, k in (("scatter_out_kernel", "copy_out"), ("gather_in_kernel", "reduce_copy_in"),
                       ("flat_kernel<yafsdp::F32", "copy_in"), ("flat_kernel<yafsdp::BF16", "post_reduce")):
            if key in name:
                return k
        return None

    rows = [r for r in csv.DictReader(open(path)) if kind(r["Kernel_Name"])]
    ev = sorted((int(r["Start_Timestamp"]), int(r["End_Timestamp"]), kind(r["Kernel_Name"]), int(r["Grid_Size_X"]), r)
                for r in rows)
    gem = [e for e in ev if e[2] == "gemm"]
    if len(gem) != 3 * 945:
        log(f"expected 2835 GEMM launches (3 stand-ins x 3 phases - alone, overlapped, overlapped with the other "
            f"stream plan - x 3 passes x 105), found {len(gem)}: take the trace with --steps 10 --no-parity")

    def union(iv):
        iv = sorted(iv)
        out, (cs, ce) = [], iv[0]
        for a_, b_ in iv[1:]:
            if a_ <= ce:
                ce = max(ce, b_)
            else:
                out.append((cs, ce))
                cs, ce = a_, b_
        out.append((cs, ce))
        return out

    per = len(gem) // 3  # GEMM launches per stand-in: passes alone, overlapped, overlapped with the other plan
    passes = per // 105
    for shape in range(3):
        g = gem[shape * per : (shape + 1) * per]
        alone, both = g[2 * 105 : 3 * 105], g[(passes // 3 + 2) * 105 : (passes // 3 + 3) * 105]
        r0 = g[0][4]
        print(f"GEMM stand-in {shape}: {r0['Kernel_Name'][:60]}... workgroup {r0['Workgroup_Size_X']}, grid "
              f"{int(r0['Grid_Size_X']) // int(r0['Workgroup_Size_X'])} workgroups, VGPR {r0['VGPR_Count']}, accum VGPR "
              f"{r0['Accum_VGPR_Count']}, SGPR {r0['SGPR_Count']}, LDS {r0['LDS_Block_Size']} B, scratch {r0['Scratch_Size']}")
        t0, t1 = both[0][0], both[-1][1]
        cop = [e for e in ev if e[2] != "gemm" and e[1] > t0 and e[0] < t1]
        ug = union([(e[0], e[1]) for e in both])
        uc = union([(max(e[0], t0), min(e[1], t1)) for e in cop])
        i = j = ov = 0
        while i < len(ug) and j < len(uc):
            a_, b_ = max(ug[i][0], uc[j][0]), min(ug[i][1], uc[j][1])
            if a_ < b_:
                ov += b_ - a_
            if ug[i][1] < uc[j][1]:
                i += 1
            else:
                j += 1
        tot = lambda u: sum(b_ - a_ for a_, b_ in u)  # noqa: E731
        avg = lambda xs: sum(xs) / max(len(xs), 1) / 1e3  # noqa: E731
        print(f"  overlapped pass: {(t1 - t0) / 1e6:.2f} ms from first to last GEMM; GEMM kernels running {tot(ug) / 1e6:.2f} ms, "
              f"copy kernels running {tot(uc) / 1e6:.2f} ms, both at once {ov / 1e6:.2f} ms")
        print(f"  GEMM kernel: {avg([e[1] - e[0] for e in alone]):.1f} us alone, {avg([e[1] - e[0] for e in both]):.1f} us in the overlapped pass")
        for k in ("copy_in", "copy_out", "reduce_copy_in", "post_reduce"):
            d1 = [e[1] - e[0] for e in cop if e[2] == k and e[3] > 1_000_000]
            print(f"  {k:15s} (decoder layers) {avg(d1):7.1f} us per launch in the overlapped pass")
    return 0


def analyze_gaps(path: str) -> int:
    """Reads the kernel trace (CSV) of ``--workload llama3-8b-full-w8 --copies-only`` and prints, per phase (the
    phases are fenced by kernels that are not the library's), how long the GPU idles between consecutive kernels of the
    path, by kind of pair: next kernel's begin minus this kernel's end."""
    import csv

    def kind(name):
        for key, k in (("unshard_kernel", "copy-in + copy-out"), ("gather_in_kernel", "reduce copy-in"),
                       ("flat_kernel<yafsdp::BF16", "post-reduce")):
            if key in name:
                return k
        return None

    rows = sorted(csv.DictReader(open(path)), key=lambda r: int(r["Start_Timestamp"]))
    phases, cur = [], []
    for r in rows:
        k = kind(r["Kernel_Name"])
        if k is None:
            if cur:
                phases.append(cur)
            cur = []
        else:
            cur.append((int(r["Start_Timestamp"]), int(r["End_Timestamp"]), k))
    if cur:
        phases.append(cur)
    for p in (p for p in phases if len(p) >= 200):
        busy, span = sum(e - s_ for s_, e, _ in p), p[-1][1] - p[0][0]
        print(f"phase of {len(p)} kernels: {span / 1e6:.3f} ms from first begin to last end, kernels themselves "
              f"{busy / 1e6:.3f} ms")
        gaps = {}
        for a, b in zip(p, p[1:]):
            gaps.setdefault((a[2], b[2]), []).append(b[0] - a[1])
        for (a, b), v in sorted(gaps.items()):
            print(f"    {a:>20s} -> {b:<20s} n={len(v):4d}  median gap {statistics.median(v) / 1e3:7.2f} us")
    return 0


def run_full_model(args, as_record: bool = False):
    """Full Llama-3-8B per-rank pass at logical W=8 on one GPU: embedding, 32 decoder layers, lm_head and
    the final norm as 35 parameter groups.  Forward: copy-in + copy-out of group i+1 run on a side stream while a
    bf16 GEMM stands in for the compute of group i.  Backward (reverse order): two GEMMs per group, then reduce
    copy-in on the compute stream and post-reduce on the side stream, all groups sharing one reduce buffer per
    shape.  One overlapped pass is checked against the oracle (embedding, a decoder layer, the final norm: all-gather
    input, copy-out tensors, gradient shard; every group has gradients of its own, so a pass that let two groups
    meet in the shared reduce buffer would show).  Reports the overlap efficiency for three GEMM stand-ins (the
    4096^3 square and the two MLP GEMMs of a Llama-3-8B layer at 4096 tokens) and per-kernel GB/s (un-overlapped)."""
    import torch

    from yafsdp_amd import _native
    from yafsdp_amd._layout import make_layout

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    w, r, align = 8, 3, 512
    layer_shapes = WORKLOADS["llama3-8b-layer-w8"][0]
    group_shapes = [[(128256, 4096)]] + [layer_shapes] * 32 + [[(128256, 4096)], [(4096,)]]
    names = ["embed"] + [f"layer{i}" for i in range(32)] + ["lm_head", "norm"]
    gen = torch.Generator(device=dev).manual_seed(1004)

    def randn(n, std, dtype):
        out = torch.empty(n, dtype=dtype, device=dev)
        for i in range(0, n, 1 << 26):
            m = min(1 << 26, n - i)
            out[i : i + m] = (torch.randn(m, device=dev, generator=gen) * std).to(dtype)
        return out

    # per-shape shared resources (the 2 shared data buffers, the shared gradient buffer, output tensors, tables);
    # master shard, gradient shard and gradients are each group's own
    shape_res = {}
    groups = []
    for name, shapes in zip(names, group_shapes):
        numels = [numel_of(s) for s in shapes]
        key = tuple(numels)
        lay = make_layout(numels, w, align)
        if key not in shape_res:
            t_pad = lay.padded_unsharded_numel
            shape_res[key] = {
                "lay": lay, "table": _native.TensorTable(numels, t_pad, dev), "numels": numels,
                "gathered": [randn(t_pad, 0.02, torch.bfloat16) for _ in range(2)],
                "outs": [[torch.empty(n, dtype=torch.bfloat16, device=dev) for n in numels] for _ in range(2)],
                "rs": torch.zeros(t_pad, dtype=torch.bfloat16, device=dev),
            }
            # what fully_shard gives the tables of groups that share ONE gradient buffer (unless options were given)
            if all(v is None for v in (args.gather_tail_mb, args.scatter_tail_mb, args.flat_tail_mb,
                                       args.post_reduce_tail_mb)):
                shape_res[key]["table"].set_option(_native.OPT_GATHER_TAIL_MB, 128)
        s_ = lay.padded_sharded_numel
        groups.append({
            "name": name, "res": shape_res[key], "lay": lay,
            "master": randn(s_, 0.02, torch.float32), "ag_in": torch.zeros(s_, dtype=torch.bfloat16, device=dev),
            "shard": randn(s_, 1e-4, torch.float32), "grads": [randn(n, 1e-3, torch.bfloat16) for n in numels],
        })
    log(f"{len(groups)} groups, {torch.cuda.memory_allocated() / 1e9:.1f} GB allocated")
    side = torch.cuda.Stream(device=dev)  # default priority
    main = torch.cuda.current_stream(dev)
    if args.copy_cus:
        # partition the compute units instead: the copies' stream may use the K lowest-numbered ones, the
        # GEMMs' stream the others (the HIP runtime's per-stream CU mask; both at default priority)
        side, main = _cu_masked_streams(torch, dev, args.copy_cus)
        torch.cuda.set_stream(main)

    gemm_state = {}

    def set_gemm(m, k, n_):
        gemm_state["a"] = randn(m * k, 0.02, torch.bfloat16).view(m, k)
        gemm_state["b"] = randn(k * n_, 0.02, torch.bfloat16).view(k, n_)
        gemm_state["c"] = torch.empty(m, n_, dtype=torch.bfloat16, device=dev)

    def gemm():
        torch.matmul(gemm_state["a"], gemm_state["b"], out=gemm_state["c"])

    def unshard(i):  # copy-in + copy-out of group i as one launch (current stream)
        g = groups[i]
        res = g["res"]
        if not res["table"].copy_in_scatter_out(res["gathered"][i % 2], res["outs"][i % 2], g["ag_in"], g["master"]):
            raise RuntimeError("copy_in_scatter_out declined")

    def reduce_in(i):
        g = groups[i]
        g["res"]["table"].gather_in(g["grads"], g["res"]["rs"], None, float(w), True)

    def post(i):
        g = groups[i]
        s_ = g["lay"].padded_sharded_numel
        _native.post_reduce(g["shard"], g["res"]["rs"][r * s_ : (r + 1) * s_], None, True)

    n = len(groups)
    # the events of the hand-offs between the two streams are recorded by the kernels' own dispatches
    # (_native.launch_recording): one event per group and purpose, each only ever recorded on one stream
    ev_ready = [torch.cuda.Event() for _ in range(n)]   # copy-in + copy-out of group i done (side stream)
    ev_done = [torch.cuda.Event() for _ in range(n)]    # reduce copy-in of group i done (compute stream)
    ev_freed = [torch.cuda.Event() for _ in range(n)]   # post-reduce of group i done: its reduce buffer is free

    def recording(event, launch, stream, markers):
        """`launch` on `stream` with `event` recorded at its end: by the kernel's own dispatch, or (markers) the
        ordinary way, by a marker packet behind it."""
        if markers:
            launch()
            event.record(stream)
            return event
        return _native.launch_recording(event, launch, stream)

    def step(copies=True, gemms=True, gather_on_side=False, markers=False, backward_on_one_stream=False):
        # forward
        if copies:
            with torch.cuda.stream(side):
                recording(ev_ready[0], lambda: unshard(0), side, markers)
        for i in range(n):
            if copies and i + 1 < n:
                with torch.cuda.stream(side):  # prefetch the next group while this one computes
                    recording(ev_ready[i + 1], lambda: unshard(i + 1), side, markers)
            if copies:
                main.wait_event(ev_ready[i])
            if gemms:
                gemm()
        # backward, reverse order
        freed = {}
        for i in reversed(range(n)):
            if gemms:
                gemm()
                gemm()
            if copies and backward_on_one_stream:
                # (measurement only: no hand-off between streams in the backward half)
                if i == n - 1:
                    main.wait_stream(side)
                reduce_in(i)
                post(i)
            elif copies and not gather_on_side:
                key = id(groups[i]["res"])
                if key in freed:
                    main.wait_event(freed[key])   # a shared gradient buffer is released by the post-reduce before
                # compute stream, like the reference's foreach calls
                recording(ev_done[i], lambda: reduce_in(i), main, markers)
                with torch.cuda.stream(side):     # reduce-scatter stream: waits for the reduce copy-in
                    side.wait_event(ev_done[i])
                    freed[key] = recording(ev_freed[i], lambda: post(i), side, markers)
            elif copies:
                # not the reference's plan (the library's opt-in, set_reduce_copy_in_on_side_stream): the reduce
                # copy-in leaves the compute stream as well; the side stream waits for the gradients, then runs both
                # kernels back to back, and its own order keeps the shared buffer safe
                with torch.cuda.stream(side):
                    if gemms:
                        side.wait_event(main.record_event())
                    reduce_in(i)
                    post(i)

    def timed(copies, gemms, reps, gather_on_side=False, **how):
        for _ in range(2):
            step(copies, gemms, gather_on_side, **how)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            step(copies, gemms, gather_on_side, **how)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / reps * 1e3

    if args.copies_only:
        # the copies-only pass under four ways of handing work between the two streams, each phase fenced by a small
        # torch fill kernel so that a kernel trace of this run can be cut into phases (--analyze-gaps)
        out = {}
        for name, how in (("reference_plan_marker_events", dict(markers=True)),
                          ("reference_plan_kernel_recorded_events", dict()),
                          ("reduce_copy_in_on_side_stream", dict(gather_on_side=True)),
                          ("backward_half_on_one_stream", dict(backward_on_one_stream=True))):
            torch.cuda.synchronize()
            torch.zeros(12345, device=dev)
            out[name] = round(timed(True, False, max(1, args.steps // 10), **how), 4)
            log(f"  copies only, {name}: {out[name]} ms per pass")
        torch.zeros(12345, device=dev)
        torch.cuda.synchronize()
        print(json.dumps({"workload": "llama3-8b-full-w8", "copies_only_ms_per_pass": out}), flush=True)
        return 0

    def timed_loop(fn, reps):
        """ms per pass of fn(i) over all groups, back to back on the current stream."""
        for i in range(n):
            fn(i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            for i in range(n):
                fn(i)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / reps * 1e3

    # ---- parity of one overlapped pass against the oracle (three groups; both streams busy)
    parity = "skipped"
    set_gemm(4096, 4096, 4096)
    if not args.no_parity:
        from oracle import torch_ops

        checked = [0, 17, n - 1]  # embedding, a decoder layer in the middle, the final norm
        before = {i: groups[i]["shard"].cpu() for i in checked}
        step(True, True)
        torch.cuda.synchronize()

        def same(a, b):
            iv = torch.int32 if a.dtype == torch.float32 else torch.int16
            return torch.equal(a.cpu().view(iv), b.view(iv))

        ok = True
        for i in checked:
            g, res, lay = groups[i], groups[i]["res"], groups[i]["lay"]
            numels = res["numels"]
            t_, tp, s_ = lay.total_numel, lay.padded_unsharded_numel, lay.padded_sharded_numel
            ag = torch.zeros(s_, dtype=torch.bfloat16)
            torch_ops.copy_in(ag, g["master"].cpu())
            outs = [torch.empty(m, dtype=torch.bfloat16) for m in numels]
            torch_ops.copy_out_materialize(res["gathered"][i % 2].cpu(), numels, outs)
            rs = torch.zeros(tp, dtype=torch.bfloat16)
            torch_ops.reduce_copy_in(list(rs[:t_].split(numels)), [x.cpu() for x in g["grads"]], False)
            shard = before[i].clone()
            torch_ops.reduce_scatter_local(shard, rs, w, r, float(w), None, "add")
            good = same(g["ag_in"], ag) and same(g["shard"], shard)
            # the copy-out tensors of a buffer index are rewritten by every group of that shape and index from the
            # same source, so their final content is this group's as well
            good = good and all(same(a_, b_) for a_, b_ in zip(res["outs"][i % 2], outs))
            log(f"  parity of group {g['name']}: {'bit-exact' if good else 'MISMATCH'}")
            ok = ok and good
        parity = "bit-exact" if ok else "MISMATCH"
        if not ok:
            log("bench.py: the overlapped pass differs from the oracle; refusing to report a throughput.")
            return 4
        del before

    reps = max(1, args.steps // 10)
    if as_record:  # a leg of the default line: bounded
        reps = min(reps, 5)
    caps = (4096, 16, 8, 4, 2, 1) if args.sweep_grid_cap else (4096,)
    gemm_shapes = [("4096x4096x4096", (4096, 4096, 4096)), ("llama-mlp-up 4096x4096x14336", (4096, 4096, 14336)),
                   ("llama-mlp-down 4096x14336x4096", (4096, 14336, 4096))]
    per_gemm = {}
    t_copy_first = None
    # the three kinds of copy work on their own: what the forward prefetch has to hide (copy-in + copy-out), what the
    # reference's plan leaves on the compute stream (reduce copy-in), and what follows it on the side stream
    t_unshard, t_gather, t_post = timed_loop(unshard, reps), timed_loop(reduce_in, reps), timed_loop(post, reps)
    log(f"  copies by kind, alone: copy-in + copy-out {t_unshard:.3f} ms, reduce copy-in {t_gather:.3f} ms, "
        f"post-reduce {t_post:.3f} ms per pass over {n} groups")
    # copies alone under both stream plans (no GEMMs): the reference's (reduce copy-in on the compute stream, every
    # hand-off between the two streams an event) and the library's opt-in (reduce copy-in on the side stream too)
    t_copy_ref, t_copy_side = timed(True, False, reps), timed(True, False, reps, gather_on_side=True)
    log(f"  copies alone as the pass runs them: {t_copy_ref:.3f} ms under the reference's stream plan, "
        f"{t_copy_side:.3f} ms with the reduce copy-in on the side stream")
    # the same copies-only pass under the reference's stream plan captured ONCE into a HIP graph and replayed: the
    # hand-offs between the two streams become edges of the graph instead of events and waits in two queues
    t_copy_graph = None
    try:
        cap = torch.cuda.Stream(device=dev)
        cap.wait_stream(main)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(cap):
            saved_main = main
            main = cap  # the captured pass's compute stream is the capturing stream
            try:
                with torch.cuda.graph(graph, stream=cap):
                    side.wait_stream(cap)  # the side stream joins the capture
                    step(True, False)
                    cap.wait_stream(side)
            finally:
                main = saved_main
        for _ in range(2):
            graph.replay()
        torch.cuda.synchronize()
        g0 = time.perf_counter()
        for _ in range(reps):
            graph.replay()
        torch.cuda.synchronize()
        t_copy_graph = (time.perf_counter() - g0) / reps * 1e3
        log(f"  copies alone, the reference's stream plan replayed from one HIP graph: {t_copy_graph:.3f} ms per pass")
        del graph
    except Exception as exc:  # an optional leg must not cost the measurements below
        log(f"  graph replay of the copies-only pass skipped: {type(exc).__name__}: {exc}")
        torch.cuda.synchronize()
    for gname, (m_, k_, n_) in gemm_shapes:
        set_gemm(m_, k_, n_)
        t_gemm = timed(False, True, reps)
        sweep = {}
        for bpc in caps:  # grid cap of the copy kernels in workgroups per compute unit
            _native.set_option(_native.OPT_FLAT_BLOCKS_PER_CU, bpc)
            _native.set_option(_native.OPT_TABLE_BLOCKS_PER_CU, bpc)
            tc = t_copy_ref if bpc == 4096 else timed(True, False, reps)
            tb = timed(True, True, reps)
            sweep[bpc] = {"ms_copies_alone": round(tc, 3), "ms_overlapped": round(tb, 3),
                          "overlap_efficiency": round(max(tc, t_gemm) / tb, 4)}
            log(f"  {gname}: grid cap {bpc:5d} workgroups/CU: copies alone {tc:.3f} ms, gemms alone {t_gemm:.3f} ms, "
                f"overlapped {tb:.3f} ms, efficiency {max(tc, t_gemm) / tb:.3f}")
        best = min(sweep, key=lambda k: sweep[k]["ms_overlapped"])
        _native.set_option(_native.OPT_FLAT_BLOCKS_PER_CU, 4096)
        _native.set_option(_native.OPT_TABLE_BLOCKS_PER_CU, 4096)
        t_copy, t_both = sweep[best]["ms_copies_alone"], sweep[best]["ms_overlapped"]
        # what the stream plan allows at best: in the forward pass copy-out of group i+1 hides behind GEMM i (or
        # the other way round), with the first group's copies exposed; in the backward pass the reduce copy-in is
        # on the compute stream (ya_fsdp/_param_group.py:669-708), in line with the GEMMs, and only the
        # post-reduce is on the side stream
        critical = max(t_gemm / 3.0, t_unshard) + t_unshard / n + t_gemm * 2.0 / 3.0 + t_gather + t_post / n
        # ... and what the memory system allows: a GEMM is not a pure matrix-core kernel, its tiles refetch the
        # operands from the memory side (GEMM_MEMORY_SIDE_MB per launch, from the L2's counters), and a copy kernel
        # saturates the memory side by itself.  While both run they share it, so a stretch of the pass in which
        # copies of duration c (alone) and GEMMs of duration g (alone, moving m megabytes) overlap takes at least
        # max(g, c + m / copy rate); stretches on one stream only take their own time.
        mem_ms_per_gemm = GEMM_MEMORY_SIDE_MB[gname] / COPY_RATE_MB_PER_MS
        g1 = t_gemm / (3.0 * n)  # one GEMM
        fwd = n * max(g1, t_unshard / n + mem_ms_per_gemm) + t_unshard / n
        bwd_ref = n * max(2 * g1, t_post / n + 2 * mem_ms_per_gemm) + t_gather + t_post / n
        bwd_side = n * max(2 * g1, (t_gather + t_post) / n + 2 * mem_ms_per_gemm) + (t_gather + t_post) / n
        model_ref, model_side = fwd + bwd_ref, fwd + bwd_side
        t_alt = timed(True, True, reps, gather_on_side=True)
        log(f"  {gname}: critical path of the reference's stream plan {critical:.3f} ms, shared-memory-side model "
            f"{model_ref:.3f} ms; with the reduce copy-in on the side stream as well: overlapped {t_alt:.3f} ms "
            f"(model {model_side:.3f} ms)")
        per_gemm[gname] = {
            "critical_path_ms": round(critical, 4), "efficiency_vs_critical_path": round(critical / t_both, 4),
            "memory_side_model_ms": round(model_ref, 4), "efficiency_vs_memory_side_model": round(model_ref / t_both, 4),
            "ms_overlapped_reduce_copy_in_on_side_stream": round(t_alt, 4),
            "memory_side_model_ms_reduce_copy_in_on_side_stream": round(model_side, 4),
            "efficiency_vs_memory_side_model_reduce_copy_in_on_side_stream": round(model_side / t_alt, 4),
            "ms_copies_alone": round(t_copy, 4), "ms_gemms_alone": round(t_gemm, 4), "ms_overlapped": round(t_both, 4),
            "overlap_efficiency": round(max(t_copy, t_gemm) / t_both, 4),
            "hidden_fraction": round((t_copy + t_gemm - t_both) / min(t_copy, t_gemm), 4),
            "gemm_TFLOPs_alone": round(2.0 * m_ * k_ * n_ * 3 * n / t_gemm / 1e9, 1),
            "grid_cap_sweep": sweep, "grid_cap_used": best,
        }
        if t_copy_first is None:
            t_copy_first = t_copy
    first = per_gemm[gemm_shapes[0][0]]
    t_copy, t_gemm, t_both = first["ms_copies_alone"], first["ms_gemms_alone"], first["ms_overlapped"]
    eff, hidden = first["overlap_efficiency"], first["hidden_fraction"]
    bytes_step = 0
    for g in groups:
        lay = g["lay"]
        t_, tp, s_ = lay.total_numel, lay.padded_unsharded_numel, lay.padded_sharded_numel
        bytes_step += s_ * 6 + 4 * t_ + (4 * t_ + 2 * (tp - t_)) + s_ * 10
    log(f"copies alone {t_copy:.3f} ms ({bytes_step / t_copy / 1e6:.0f} GB/s), gemms alone {t_gemm:.3f} ms, "
        f"overlapped {t_both:.3f} ms; overlap efficiency {eff:.3f}, hidden fraction {hidden:.3f}")
    # per-kernel GB/s, un-overlapped, on a decoder layer group
    kernels = {}
    li = 5
    lay = groups[li]["lay"]
    t_, tp, s_ = lay.total_numel, lay.padded_unsharded_numel, lay.padded_sharded_numel
    per = [("copy_in_and_copy_out", lambda: unshard(li), s_ * 6 + 4 * t_),
           ("reduce_copy_in", lambda: reduce_in(li), 4 * t_ + 2 * (tp - t_)),
           ("post_reduce", lambda: post(li), s_ * 10)]
    for name, fn, nbytes in per:
        ts = []
        for _ in range(20):
            unshard(0)  # 1.3 GB of other traffic in between
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(); fn(); e1.record(); e1.synchronize()
            ts.append(e0.elapsed_time(e1) * 1e3)
        med = statistics.median(ts)
        kernels[name] = {"us_median": round(med, 2), "GBps": round(nbytes / med / 1e3, 1)}
    out = {
        "metric": "overlap efficiency of the buffer path against a GEMM stand-in, full Llama-3-8B per-rank pass @W=8",
        "value": round(eff, 4), "unit": "max(copies, gemms) / overlapped", "n_gpus": 1, "steps": reps, "warmup": 2,
        "ms_per_step": round(t_both, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic", "parity": parity,
        "config": {"workload": "llama3-8b-full-w8", "groups": n, "logical_world_size": w, "rank": r,
                   "gemm": "bf16 4096x4096x4096, 1 per group forward, 2 per group backward (headline value); "
                           "the two Llama-3-8B MLP GEMMs at 4096 tokens under `gemm_shapes`",
                   "copy_stream_compute_units": args.copy_cus or 256},
        "ms_copies_alone": round(t_copy, 4), "ms_gemms_alone": round(t_gemm, 4), "ms_overlapped": round(t_both, 4),
        "hidden_fraction": round(hidden, 4),
        "ms_copies_by_kind_alone": {"copy_in_and_copy_out": round(t_unshard, 4), "reduce_copy_in": round(t_gather, 4),
                                    "post_reduce": round(t_post, 4)},
        "gemm_shapes": per_gemm, "copy_GBps_alone": round(bytes_step / t_copy / 1e6, 1),
        "ms_copies_alone_reduce_copy_in_on_side_stream": round(t_copy_side, 4),
        "copy_GBps_alone_reduce_copy_in_on_side_stream": round(bytes_step / t_copy_side / 1e6, 1),
        "copy_GBps_by_kind": round(bytes_step / (t_unshard + t_gather + t_post) / 1e6, 1),
        "ms_copies_alone_replayed_from_one_graph": None if t_copy_graph is None else round(t_copy_graph, 4),
        "copy_GBps_alone_replayed_from_one_graph": None if t_copy_graph is None else round(bytes_step / t_copy_graph / 1e6, 1),
        "copy_GBps_overlapped_lower_bound": round(bytes_step / t_both / 1e6, 1), "bytes_per_step": bytes_step,
        "kernels": kernels,
    }
    if as_record:  # a compact record for the `configs` block of the default workload's line
        for g in groups:
            g.clear()
        for res in shape_res.values():
            res["table"].close()
        return {
            "value": out["value"], "unit": out["unit"], "parity": parity, "ms_overlapped": out["ms_overlapped"],
            "ms_copies_alone": out["ms_copies_alone"], "ms_gemms_alone": out["ms_gemms_alone"],
            "copy_GBps_alone": out["copy_GBps_alone"], "groups": n, "logical_world_size": w, "passes_timed": reps,
            "copy_GBps_alone_reduce_copy_in_on_side_stream": out["copy_GBps_alone_reduce_copy_in_on_side_stream"],
            "copy_GBps_alone_replayed_from_one_graph": out["copy_GBps_alone_replayed_from_one_graph"],
            "copy_GBps_by_kind": out["copy_GBps_by_kind"], "ms_copies_by_kind_alone": out["ms_copies_by_kind_alone"],
            "gemm_shapes": {k: {a_: b_ for a_, b_ in v.items()
                                if a_ in ("ms_gemms_alone", "ms_overlapped", "overlap_efficiency",
                                          "efficiency_vs_critical_path", "critical_path_ms", "memory_side_model_ms",
                                          "efficiency_vs_memory_side_model",
                                          "ms_overlapped_reduce_copy_in_on_side_stream",
                                          "efficiency_vs_memory_side_model_reduce_copy_in_on_side_stream")}
                            for k, v in per_gemm.items()},
        }
    print(json.dumps(out), flush=True)
    return 0


def run_timeline(args) -> int:
    """Where the time of the short kernels goes, and what other stream plans would give (headline workload).

    (1) Per-workgroup timeline of copy-in, post-reduce (copy form) and post-reduce (accumulate) on one rank's shard
    of the Llama-3-8B layer: every workgroup records the GPU's 100 MHz wall clock at its start and after its last
    store has been acknowledged; the dispatch itself is timed with HIP events attached to it.  Reported per kernel:
    dispatch time, time from the first workgroup's start to the last one's end, the rest (before the first wave and
    after the last), time until the first workgroup completes, workgroup life, the plateau rate (workgroups ending
    in the middle half of the span) and the time the launch loses against running at that rate from start to end.
    (2) The step of the headline workload on one stream, with the reference's stream plan (copy-in, copy-out and
    post-reduce on a side stream, reduce copy-in on the compute stream, ya_fsdp/_collectives.py:46, 110-111,
    ya_fsdp/_param_group.py:669), as two independent chains on two streams, and the first and the last of these
    with copy-in and copy-out as one launch (what the default workload times)."""
    import torch

    from yafsdp_amd import _native
    from yafsdp_amd._layout import make_layout

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    shapes, w, r, align, seed = WORKLOADS["llama3-8b-layer-w8"]
    numels = [numel_of(s_) for s_ in shapes]
    lay = make_layout(numels, w, align)
    t, t_pad, s = lay.total_numel, lay.padded_unsharded_numel, lay.padded_sharded_numel
    gen = torch.Generator(device=dev).manual_seed(seed)

    def randn(n, std, dtype):
        out = torch.empty(n, dtype=dtype, device=dev)
        for i in range(0, n, 1 << 26):
            m = min(1 << 26, n - i)
            out[i : i + m] = (torch.randn(m, device=dev, generator=gen) * std).to(dtype)
        return out

    master = randn(s, 0.02, torch.float32)
    ag_in = torch.zeros(s, dtype=torch.bfloat16, device=dev)
    gathered = randn(t_pad, 0.02, torch.bfloat16)
    grads = [randn(n, 1e-3, torch.bfloat16) for n in numels]
    outs = [torch.empty(n, dtype=torch.bfloat16, device=dev) for n in numels]
    rs = torch.zeros(t_pad, dtype=torch.bfloat16, device=dev)
    shard, shard_b = randn(s, 1e-4, torch.float32), torch.empty(s, dtype=torch.float32, device=dev)
    chunk = rs[r * s : (r + 1) * s]
    table = _native.TensorTable(numels, t_pad, dev)
    out_binding = table.bind(outs)

    def op_copy_in():
        _native.flat_copy(ag_in, master)

    def op_copy_out():
        out_binding.scatter_out(gathered)

    def op_reduce_copy_in():
        table.gather_in(grads, rs, None, float(w), True)

    def op_post_reduce():
        _native.post_reduce(shard, chunk, None, True)

    op_reduce_copy_in()
    torch.cuda.synchronize()
    tile_elems = 256 * 8  # elements per workgroup of the flat kernels (256 lanes x one 8-element unit)
    timeline = {}
    for name, fn, bytes_per_elem in (("copy_in", op_copy_in, 6), ("post_reduce_copy", lambda: _native.post_reduce(shard_b, chunk, None, False), 6),
                                     ("post_reduce", op_post_reduce, 10)):
        recs = []
        for _ in range(7):
            op_copy_out()           # 1.7 GB of other traffic in front, as in a step
            op_reduce_copy_in()
            ev = _event_pair()
            with _native.FlatLaunchTrace(1 << 16, dev) as tr:
                _native.time_next_launch(*ev)
                fn()
            torch.cuda.synchronize()
            tm = tr.times().double() * 0.01  # microseconds
            first, last = float(tm[:, 0].min()), float(tm[:, 1].max())
            span = last - first
            ends = tm[:, 1] - first
            life = (tm[:, 1] - tm[:, 0]).sort().values
            mid = ((ends >= 0.25 * span) & (ends < 0.75 * span)).sum().item()
            wg_bytes = tile_elems * bytes_per_elem
            plateau = mid * wg_bytes / (0.5 * span) / 1e3  # GB/s
            total_bytes = tm.shape[0] * wg_bytes
            bins = torch.histc(ends.float(), bins=int(span) + 1, min=0.0, max=float(int(span) + 1))
            recs.append({
                "dispatch_us": ev[0].elapsed_time(ev[1]) * 1e3, "first_start_to_last_end_us": span,
                "first_completion_us": float(ends.min()), "last_start_us": float(tm[:, 0].max()) - first,
                "workgroup_life_us_median": float(life[len(life) // 2]), "workgroup_life_us_p90": float(life[len(life) * 9 // 10]),
                "plateau_GBps": plateau, "lost_against_plateau_us": span - total_bytes / plateau / 1e3,
                "GBps_of_workgroups_ending_per_us": [round(float(b) * wg_bytes / 1e3) for b in bins],
                "workgroups": tm.shape[0],
            })
        recs.sort(key=lambda d: d["dispatch_us"])
        med = recs[len(recs) // 2]
        med["outside_first_start_to_last_end_us"] = med["dispatch_us"] - med["first_start_to_last_end_us"]
        med["bytes"] = med["workgroups"] * tile_elems * bytes_per_elem
        med["GBps_dispatch"] = med["bytes"] / med["dispatch_us"] / 1e3
        timeline[name] = {k: (round(v, 2) if isinstance(v, float) else v) for k, v in med.items()}
        log(f"  {name:17s} dispatch {med['dispatch_us']:.2f} us = span {med['first_start_to_last_end_us']:.2f} + "
            f"{med['outside_first_start_to_last_end_us']:.2f} outside; first completion after {med['first_completion_us']:.2f} us, "
            f"plateau {med['plateau_GBps']:.0f} GB/s, {med['lost_against_plateau_us']:.2f} us lost against it")

    # ---- stream plans for the whole step
    main, side = torch.cuda.current_stream(dev), torch.cuda.Stream(device=dev)
    bytes_per_step = s * 6 + 4 * t + (4 * t + 2 * (t_pad - t)) + s * 10

    def one_stream():
        op_copy_in(); op_copy_out(); op_reduce_copy_in(); op_post_reduce()

    def reference_plan():
        with torch.cuda.stream(side):      # all-gather side: copy-in, copy-out
            op_copy_in(); op_copy_out()
        op_reduce_copy_in()                # compute stream
        done = main.record_event()
        with torch.cuda.stream(side):      # reduce-scatter side: after the compute stream
            side.wait_event(done)
            op_post_reduce()

    def two_chains():
        with torch.cuda.stream(side):
            op_copy_in(); op_copy_out()
        op_reduce_copy_in(); op_post_reduce()

    def op_unshard():  # copy-in and copy-out as one grid
        if not table.copy_in_scatter_out(gathered, outs, ag_in, master):
            raise RuntimeError("copy_in_scatter_out declined")

    def one_stream_three_launches():
        op_unshard(); op_reduce_copy_in(); op_post_reduce()

    def two_chains_three_launches():
        with torch.cuda.stream(side):
            op_unshard()
        op_reduce_copy_in(); op_post_reduce()

    plans = {}
    for name, fn in (("one_stream", one_stream), ("reference_stream_plan", reference_plan),
                     ("two_chains_two_streams", two_chains), ("one_stream_three_launches", one_stream_three_launches),
                     ("two_chains_three_launches", two_chains_three_launches)):
        side.wait_stream(main)
        for _ in range(args.warmup):
            fn()
        main.wait_stream(side)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            fn()
        main.wait_stream(side)
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / args.steps
        plans[name] = {"ms_per_step": round(dt * 1e3, 4), "value": round(bytes_per_step / dt / 1e9, 1), "unit": "GB/s",
                       "frac_of_hbm_peak": round(bytes_per_step / dt / 1e9 / HBM_PEAK_GBS, 4)}
        log(f"  {name:24s} {plans[name]['ms_per_step']} ms per step, {plans[name]['value']} GB/s")
    out = {
        "metric": "launch timeline of the short flat kernels and stream plans of the step, Llama-3-8B layer @W=8",
        "value": plans["one_stream_three_launches"]["value"], "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": plans["one_stream_three_launches"]["ms_per_step"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "launch-timeline", "shard_numel": s, "padded_numel": t_pad, "logical_world_size": w},
        "timeline": timeline, "stream_plans": plans,
    }
    print(json.dumps(out), flush=True)
    out_binding.close()
    table.close()
    return 0


def run_trainer(args) -> int:
    """Whole training iterations on one GPU at world size 1: Llama-3-8B decoder layers (real shapes, random init)
    wrapped one by one with ``fully_shard`` (fp32 masters, bf16 compute), forward + backward + gradient norm +
    AdamW.  Three loops over the same model and inputs:

    * ``fully_shard`` + ``FlatAdamW`` (buffer kernels; the post-reduce leaves the gradient norm, the optimizer pass
      applies the clip coefficient and writes the next copy-in);
    * ``fully_shard`` + ``torch.optim.AdamW(fused=True)`` on the sharded parameters;
    * no wrapper: the same mixed precision written by hand with torch ops (``_foreach_copy_`` of the fp32 masters
      into a bf16 copy of the model, gradients copied back into fp32, fused torch AdamW).

    The compute floor (bf16 forward + backward only, no masters, no optimizer) is reported beside them."""
    import copy

    import torch
    import torch.nn as nn
    import torch.nn.functional as F

    from yafsdp_amd import MixedPrecisionPolicy, fully_shard
    from yafsdp_amd.optim import FlatAdamW, clip_grad_norm_, enable_fused_grad_norm, grad_clip_coef

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    dim, ffn, heads, kv_heads, layers, seq = 4096, 14336, 32, 8, args.layers, args.seq_len
    hd = dim // heads
    world = max(1, args.logical_world_size)
    mesh = None if world == 1 else (world, world // 2)

    class RMSNorm(nn.Module):
        def __init__(self):
            super().__init__()
            self.weight = nn.Parameter(torch.ones(dim))

        def forward(self, x):
            return F.rms_norm(x, (dim,), self.weight, 1e-5)

    class Layer(nn.Module):
        def __init__(self):
            super().__init__()
            self.q = nn.Linear(dim, dim, bias=False)
            self.k = nn.Linear(dim, kv_heads * hd, bias=False)
            self.v = nn.Linear(dim, kv_heads * hd, bias=False)
            self.o = nn.Linear(dim, dim, bias=False)
            self.gate = nn.Linear(dim, ffn, bias=False)
            self.up = nn.Linear(dim, ffn, bias=False)
            self.down = nn.Linear(ffn, dim, bias=False)
            self.n1, self.n2 = RMSNorm(), RMSNorm()

        def forward(self, x):
            b, s_, _ = x.shape
            h = self.n1(x)
            q = self.q(h).view(b, s_, heads, hd).transpose(1, 2)
            k = self.k(h).view(b, s_, kv_heads, hd).transpose(1, 2)
            v = self.v(h).view(b, s_, kv_heads, hd).transpose(1, 2)
            a = F.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True)
            x = x + self.o(a.transpose(1, 2).reshape(b, s_, dim))
            h = self.n2(x)
            return x + self.down(F.silu(self.gate(h)) * self.up(h))

    class Stack(nn.Module):
        def __init__(self):
            super().__init__()
            self.layers = nn.ModuleList([Layer() for _ in range(layers)])

        def forward(self, x):
            for layer in self.layers:
                x = layer(x)
            return x

    torch.manual_seed(1006)
    with torch.device(dev):
        model0 = Stack()
    for p in model0.parameters():
        if p.dim() > 1:
            nn.init.normal_(p, std=0.02)
    n_params = sum(p.numel() for p in model0.parameters())
    x = torch.randn(1, seq, dim, device=dev, dtype=torch.bfloat16)
    log(f"{layers} layers, {n_params / 1e6:.0f} M parameters, {seq} tokens per iteration")
    hyper = dict(lr=1e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)

    def loss_of(y):
        return y.float().pow(2).mean()

    spread = {}

    def timed(step, reps, warm, name):
        """Median over the iterations (events at the iteration boundaries, no host synchronisation between
        them); the mean over the same iterations, host clock, is kept beside it."""
        import gc

        for _ in range(warm):
            step()
        gc.collect()
        torch.cuda.synchronize()
        marks = [torch.cuda.Event(enable_timing=True) for _ in range(reps + 1)]
        t0 = time.perf_counter()
        marks[0].record()
        for i in range(reps):
            step()
            marks[i + 1].record()
        torch.cuda.synchronize()
        mean = (time.perf_counter() - t0) / reps * 1e3
        per = [marks[i].elapsed_time(marks[i + 1]) for i in range(reps)]
        spread[name] = {"mean": round(mean, 3), "min": round(min(per), 3), "max": round(max(per), 3)}
        return statistics.median(per)

    reps, warm = max(3, args.steps // 5), max(2, args.warmup // 5)
    results = {}

    # ---- compute floor: bf16 forward + backward only
    lowp = copy.deepcopy(model0).to(torch.bfloat16)

    def floor_step():
        loss_of(lowp(x)).backward()
        for p in lowp.parameters():
            p.grad = None

    results["compute_only_bf16"] = timed(floor_step, reps, warm, "compute_only_bf16")

    # ---- hand-written mixed precision with torch ops (the whole model's masters and optimizer state on this GPU:
    # comparable with the wrapped loops at world size 1 only)
    if world == 1:
        masters = [p.detach().clone().requires_grad_(True) for p in model0.parameters()]
        lowp_params = list(lowp.parameters())
        for m in masters:
            m.grad = torch.zeros_like(m)
        opt_t = torch.optim.AdamW(masters, fused=True, **hyper)

        def torch_step():
            with torch.no_grad():
                torch._foreach_copy_(lowp_params, masters)          # the cast the copy-in does
            loss_of(lowp(x)).backward()
            with torch.no_grad():
                torch._foreach_copy_([m.grad for m in masters], [p.grad for p in lowp_params])  # bf16 -> fp32 gradients
            for p in lowp_params:
                p.grad = None
            torch.nn.utils.clip_grad_norm_(masters, 1.0, foreach=True)
            opt_t.step()

        results["torch_ops_by_hand"] = timed(torch_step, reps, warm, "torch_ops_by_hand")
        del masters, opt_t, lowp_params
    del lowp
    torch.cuda.empty_cache()

    # ---- fully_shard, two optimizers
    mp = MixedPrecisionPolicy(param_dtype=torch.bfloat16)

    def wrapped():
        m = copy.deepcopy(model0)
        for layer in m.layers:
            fully_shard(layer, mesh=mesh, mp_policy=mp)
        return fully_shard(m, mesh=mesh, mp_policy=mp)

    def seed_peer_slots(m):
        """At a logical world size above one nothing delivers the other ranks' slots of the gathered buffers; they
        get weight-like values once (every later unshard rewrites this rank's slot only), so that the GEMMs run on
        ordinary data."""
        for mod in m._fsdp_modules(True):
            group = mod._get_fsdp_state()._fsdp_param_group
            if group is not None:
                for gathered in group._all_gather_output.values():
                    gathered.normal_(0.0, 0.02)

    for name in ("fully_shard_torch_adamw", "fully_shard_flat_adamw"):
        model = wrapped()
        params = list(model.parameters())
        flat = name == "fully_shard_flat_adamw"
        if flat:
            opt = FlatAdamW(params, **hyper)
            enable_fused_grad_norm(model)  # the post-reduce also leaves the squared norm of each gradient shard
        else:
            opt = torch.optim.AdamW(params, fused=True, **hyper)

        def fs_step():
            loss_of(model(x)).backward()
            if flat:
                _, coef = grad_clip_coef(model, 1.0)   # the norm only; the optimizer pass applies the coefficient
                opt.step(grad_scale=coef)
            else:
                clip_grad_norm_(model, 1.0)
                opt.step()
            # gradients stay allocated (the flat gradient shard); the next backward accumulates into them
            # unless they are cleared, as with torch.optim
            opt.zero_grad(set_to_none=True)

        if world > 1:
            fs_step()  # lazy initialisation assigns the buffers
            seed_peer_slots(model)
        results[name] = timed(fs_step, reps, warm, name)
        del model, params, opt
        torch.cuda.empty_cache()

    for k_, v_ in results.items():
        log(f"  {k_:28s} {v_:8.3f} ms / iteration (median; {spread[k_]})  ({seq / v_ * 1e3:9.0f} tokens/s)")
    best = results["fully_shard_flat_adamw"]
    out = {
        "metric": (f"training iteration at world size 1: {layers} Llama-3-8B decoder layers through fully_shard + flat AdamW"
                   if world == 1 else
                   f"one rank's share of a training iteration at logical world size {world} (no exchanges between "
                   f"ranks): {layers} Llama-3-8B decoder layers through fully_shard + flat AdamW"),
        "value": round(seq / best * 1e3, 1), "unit": "tokens/s", "n_gpus": 1, "steps": reps, "warmup": warm,
        "ms_per_step": round(best, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "fully-shard-trainer-w1", "logical_world_size": world, "layers": layers,
                   "parameters": n_params, "tokens_per_step": seq,
                   "master_dtype": "float32", "optimizer": "AdamW + gradient clipping"},
        "ms_per_iteration": {k_: round(v_, 4) for k_, v_ in results.items()},
        "ms_per_iteration_mean_min_max": spread,
        "overhead_over_compute_ms": {k_: round(v_ - results["compute_only_bf16"], 4) for k_, v_ in results.items()
                                     if k_ != "compute_only_bf16"},
    }
    print(json.dumps(out), flush=True)
    return 0


def run_optim(args) -> int:
    """Optimizer-side passes over one rank's flat shard of the layer (what follows the backward pass of a step):
    squared gradient norm, clip coefficient, and the fused AdamW step that scales the gradient by the coefficient
    and writes the bf16 all-gather input of the next iteration."""
    import torch

    from oracle import cref, torch_ops
    from yafsdp_amd import _native
    from yafsdp_amd._layout import make_layout

    base = args.workload[: -len("-optim")]
    shapes, w, r, align, seed = WORKLOADS[base]
    numels = [numel_of(s) for s in shapes]
    lay = make_layout(numels, w, align)
    s = lay.padded_sharded_numel
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    hp = dict(lr=3e-4, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1)
    max_norm = 1.0
    log(f"workload {args.workload}: shard S={s} (W={w}, rank={r}), AdamW {hp}, max_norm={max_norm}")
    g = torch.Generator().manual_seed(seed + 100)
    master = torch.randn(s, generator=g) * 0.02
    grad = torch.randn(s, generator=g) * 1e-3  # norm ~ 5: clipped at max_norm 1
    m0 = torch.randn(s, generator=g) * 1e-3
    v0 = (torch.randn(s, generator=g) * 1e-3) ** 2
    d_p, d_g, d_m, d_v = (x.to(dev) for x in (master, grad, m0, v0))
    d_out = torch.zeros(s, dtype=torch.bfloat16, device=dev)
    d_sumsq = torch.zeros(1, dtype=torch.float64, device=dev)
    d_nc = torch.zeros(2, dtype=torch.float32, device=dev)
    d_partials = torch.empty(_native.SUMSQ_MAX_PARTIALS, dtype=torch.float64, device=dev)
    d_g_keep = d_g.clone()
    steps_done = [0]

    def op_sumsq():
        count = _native.sumsq_partials(d_g_keep, d_partials, 0)
        _native.clip_coef_from_partials(d_partials, count, max_norm, d_nc, d_sumsq)

    def op_adamw():
        steps_done[0] += 1
        _native.adamw_step(d_p, d_g, d_m, d_v, d_out, step=steps_done[0], grad_scale=d_nc[1:2], **hp)

    def op_adamw_zero():  # also zero-fills the gradient shard: needs a fresh gradient before every launch
        steps_done[0] += 1
        _native.adamw_step(d_p, d_g, d_m, d_v, d_out, step=steps_done[0], grad_scale=d_nc[1:2], zero_grad=True, **hp)

    def refresh_grad():
        _native.flat_copy(d_g, d_g_keep)

    def op_fill():
        _native.flat_fill(d_g, 0.0)

    def op_scale():
        _native.flat_scale(d_g_keep, d_half)

    d_half = torch.full((1,), 0.5, device=dev)
    # the post-reduce that precedes these passes in a step, without and with the fused sum of squares (which makes
    # grad_sumsq's read pass unnecessary)
    d_chunk = (torch.randn(s, generator=g) * 1e-3).bfloat16().to(dev)
    d_pr = torch.zeros(s, device=dev)
    d_pr_partials = torch.empty(_native.post_reduce_sumsq_count(s), dtype=torch.float64, device=dev)

    def op_post_reduce():
        _native.post_reduce(d_pr, d_chunk, None, True)

    def op_post_reduce_sumsq():
        count = _native.post_reduce_sumsq(d_pr, d_chunk, None, True, d_pr_partials)
        _native.clip_coef_from_partials(d_pr_partials, count, max_norm, d_nc2)

    d_nc2 = torch.zeros(2, dtype=torch.float32, device=dev)
    # the timed step leaves the gradient in place (a training step rewrites it in its backward pass); the
    # variant that zero-fills it is timed on its own below, with the gradient restored before each launch
    ops = [
        ("grad_sumsq", op_sumsq, s * 4),
        ("adamw_step", op_adamw, s * (16 + 12 + 2)),
    ]
    extra = [("adamw_step_zero_grad", op_adamw_zero, s * (16 + 12 + 2 + 4)), ("zero_fill", op_fill, s * 4),
             ("grad_scale", op_scale, s * 8), ("post_reduce", op_post_reduce, s * 10),
             ("post_reduce_with_norm", op_post_reduce_sumsq, s * 10)]
    bytes_per_step = sum(b for _, _, b in ops)

    parity = "skipped"
    if not args.no_parity:
        op_sumsq()
        op_adamw_zero()
        torch.cuda.synchronize()
        total = cref.sumsq(grad)
        norm, coef = cref.clip_coef(total, max_norm)
        cp, cg, cm, cv = master.clone(), grad.clone(), m0.clone(), v0.clone()
        cout = torch.zeros(s, dtype=torch.bfloat16)
        cref.adamw_step(cp, cg, cm, cv, cout, step=1, grad_scale=coef, zero_grad=True, **hp)
        checks = {
            "sumsq": abs(d_sumsq.item() - total) <= 1e-12 * total,
            "norm": d_nc[0].item() == norm, "coef": d_nc[1].item() == coef,
            "out16": torch.equal(d_out.cpu().view(torch.int16), cout.view(torch.int16)),
        }
        for name, a, b in (("param", d_p, cp), ("grad", d_g, cg), ("exp_avg", d_m, cm), ("exp_avg_sq", d_v, cv)):
            checks[name] = torch.equal(a.cpu().view(torch.int32), b.view(torch.int32))
        ok = all(checks.values())
        if not ok:
            log("parity details:", checks, d_sumsq.item(), total, d_nc.tolist(), norm, coef)
        parity = "bit-exact" if ok else "MISMATCH"
        log("parity vs oracle:", parity, f"(norm {norm:.6f}, coef {coef:.6f})")
        if not ok:
            log("bench.py: GPU results differ from the oracle; refusing to report a throughput.")
            return 4
    d_g.copy_(d_g_keep)

    def step():
        for _, fn, _ in ops:
            fn()

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    sampled = [k for k in range(args.steps) if k % 4 == 0]
    ev = {k: _event_pair() for k in sampled}
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(args.steps):
        ops[0][1]()
        if k in ev:
            _native.time_next_launch(*ev[k])  # events attached to the AdamW dispatch itself
        ops[1][1]()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps
    value = bytes_per_step * args.steps / elapsed / 1e9
    dom_us = [a.elapsed_time(b) * 1e3 for a, b in ev.values()]
    dom_avg_us = sum(dom_us) / len(dom_us)
    dom_bytes = ops[1][2]
    achieved = dom_bytes / dom_avg_us / 1e3

    kernels = {}
    for name, fn, nbytes in ops + extra:
        times = []
        for _ in range(20):
            a, b = _event_pair()
            for n2, f, _ in ops + extra:  # evict: the other ops stream the other buffers through the caches
                if n2 != name:
                    f()
            refresh_grad()
            if name in ("grad_sumsq", "post_reduce_with_norm"):  # two launches: bracket the pair with recorded events
                a.record()
                fn()
                b.record()
            else:
                _native.time_next_launch(a, b)
                fn()
            torch.cuda.synchronize()
            times.append(a.elapsed_time(b) * 1e3)
        med = statistics.median(times)
        kernels[name] = {"bytes": nbytes, "us_median": round(med, 2), "us_min": round(min(times), 2),
                         "GBps": round(nbytes / med / 1e3, 1), "frac_of_peak": round(nbytes / med / 1e3 / HBM_PEAK_GBS, 4)}
        log(f"  {name:12s} {nbytes / 1e6:8.1f} MB  median {med:7.1f} us  {nbytes / med / 1e3:7.1f} GB/s "
            f"({100 * nbytes / med / 1e3 / HBM_PEAK_GBS:.1f}% of peak)")

    cpu_baseline = None
    if args.cpu_seconds > 0:
        # the reference's path for the same work: clip_grad_norm_ + torch.optim.AdamW + the copy-in cast
        param = torch.nn.Parameter(master.clone())
        opt = torch.optim.AdamW([param], lr=hp["lr"], betas=(hp["beta1"], hp["beta2"]), eps=hp["eps"],
                                weight_decay=hp["weight_decay"])
        ag_in = torch.zeros(s, dtype=torch.bfloat16)
        times, spent = [], 0.0
        while spent < args.cpu_seconds and len(times) < 500:
            param.grad = grad.clone()
            c0 = time.perf_counter()
            torch_ops.clip_grad_norm_([param.grad], max_norm)
            opt.step()
            torch_ops.copy_in(ag_in, param.detach())
            dt = time.perf_counter() - c0
            times.append(dt)
            spent += dt
        med = statistics.median(times)
        cpu_baseline = {
            "value": round(bytes_per_step / med / 1e9, 2), "unit": "GB/s", "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": f"{len(times)} passes of clip_grad_norm_ + torch.optim.AdamW.step + copy-in cast "
                      f"on the same shard with torch on CPU tensors, median, {spent:.1f}s total; rated with the fused "
                      f"pass's algorithmic bytes",
        }
        log(f"cpu baseline: {cpu_baseline['value']} GB/s on {cpu_baseline['cores']} threads ({len(times)} passes)")

    torch_gpu = None
    if not args.no_torch_gpu:
        # what the reference runs on this hardware: torch's clipping, fused AdamW and the copy-in cast on the GPU
        gparam = torch.nn.Parameter(master.to(dev))
        gopt = torch.optim.AdamW([gparam], lr=hp["lr"], betas=(hp["beta1"], hp["beta2"]), eps=hp["eps"],
                                 weight_decay=hp["weight_decay"], fused=True)
        g_ag_in = torch.zeros(s, dtype=torch.bfloat16, device=dev)
        gparam.grad = d_g_keep.clone()

        def gpu_torch_step():
            torch.nn.utils.clip_grad_norm_([gparam], max_norm, foreach=True)
            gopt.step()
            torch_ops.copy_in(g_ag_in, gparam.detach())

        for _ in range(3):
            gpu_torch_step()
        torch.cuda.synchronize()
        reps = 20
        c0 = time.perf_counter()
        for _ in range(reps):
            gpu_torch_step()
        torch.cuda.synchronize()
        dt = (time.perf_counter() - c0) / reps
        torch_gpu = {
            "value": round(bytes_per_step / dt / 1e9, 1), "unit": "GB/s", "ms_per_step": round(dt * 1e3, 4),
            "sample": f"{reps} passes of torch.nn.utils.clip_grad_norm_ + torch.optim.AdamW(fused=True).step + copy-in "
                      f"cast on device tensors with torch {torch.__version__}, rated with the fused pass's bytes",
        }
        log(f"torch ops on the GPU: {torch_gpu['value']} GB/s, {torch_gpu['ms_per_step']} ms per step")

    out = {
        "metric": "HBM GB/s + % of peak for the optimizer-side flat-shard passes (grad norm + fused AdamW/copy-in), "
                  "Llama-3-8B layer @W=8" if base == "llama3-8b-layer-w8" else
                  "HBM GB/s + % of peak for the optimizer-side flat-shard passes (grad norm + fused AdamW/copy-in)",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": args.workload, "shard_numel": s, "logical_world_size": w, "rank": r,
                   "bytes_per_step": bytes_per_step, "hyperparameters": hp, "max_norm": max_norm,
                   "ops": "sum of squares of the fp32 grad shard [S] + clip coefficient; AdamW on fp32 p/g/m/v [S] with "
                          "fused grad scale and bf16 all-gather input"},
        "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4), "parity": parity,
        "roofline": {"bound": "hbm", "kernel": "adamw_kernel (fused AdamW step)", "achieved": round(achieved, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": MEASURED_TRAFFIC_BYTES.get(args.workload), "algorithmic_bytes": dom_bytes, "avg_launch_us": round(dom_avg_us, 2),
                     "launches_timed": len(dom_us)},
        "cpu_baseline": cpu_baseline, "torch_gpu_baseline": torch_gpu, "kernels": kernels,
        "fused_norm": {
            "post_reduce_then_grad_sumsq_us": round(kernels["post_reduce"]["us_median"] + kernels["grad_sumsq"]["us_median"], 2),
            "post_reduce_with_norm_us": kernels["post_reduce_with_norm"]["us_median"],
        },
    }
    print(json.dumps(out), flush=True)
    return 0


def run_exchange(args) -> int:
    """The two exchange points of the path as one-GPU kernels over W local buffers: the copy-in cast written to
    this rank's slot of W gathered buffers (direct all-gather, sender side) and the reduce over this rank's chunk
    of W reduce buffers fused with post-divide and accumulation (direct reduce-scatter, receiver side)."""
    import torch

    from oracle import torch_ops
    from yafsdp_amd import _native
    from yafsdp_amd._layout import make_layout

    base = args.workload[: -len("-exchange")]
    shapes, w, r, align, seed = WORKLOADS[base]
    if w > 16:
        log(f"bench.py: the fan kernels take at most 16 buffers; {base} has W={w}")
        return 2
    lay = make_layout([numel_of(s) for s in shapes], w, align)
    s = lay.padded_sharded_numel
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    log(f"workload {args.workload}: shard S={s}, W={w} buffers on one GPU")
    g = torch.Generator().manual_seed(seed + 200)
    master = torch.randn(s, generator=g) * 0.02
    chunks = [(torch.randn(s, generator=g) * 1e-3).bfloat16() for _ in range(w)]
    shard0 = torch.randn(s, generator=g) * 1e-4
    d_master = master.to(dev)
    d_slots = [torch.zeros(s, dtype=torch.bfloat16, device=dev) for _ in range(w)]
    d_chunks = [c.to(dev) for c in chunks]
    d_shard = shard0.to(dev)
    post = float(w)

    def op_fanout():
        _native.flat_copy_fanout(d_slots, d_master)

    def op_fanin():
        _native.post_reduce_fanin(d_shard, d_chunks, post, True)

    ops = [("copy_in_fanout", op_fanout, s * (4 + 2 * w)), ("reduce_fanin", op_fanin, s * (2 * w + 4 + 4))]
    bytes_per_step = sum(b for _, _, b in ops)

    parity = "skipped"
    if not args.no_parity:
        op_fanout()
        op_fanin()
        torch.cuda.synchronize()
        want_slot = torch.zeros(s, dtype=torch.bfloat16)
        torch_ops.copy_in_fanout([want_slot], master)
        want_shard = shard0.clone()
        torch_ops.reduce_scatter_fanin(want_shard, chunks, post, True)
        ok = all(torch.equal(x.cpu().view(torch.int16), want_slot.view(torch.int16)) for x in d_slots)
        ok = ok and torch.equal(d_shard.cpu().view(torch.int32), want_shard.view(torch.int32))
        parity = "bit-exact" if ok else "MISMATCH"
        log("parity vs oracle:", parity)
        if not ok:
            log("bench.py: GPU results differ from the oracle; refusing to report a throughput.")
            return 4

    for _ in range(args.warmup):
        for _, fn, _ in ops:
            fn()
    torch.cuda.synchronize()
    sampled = [k for k in range(args.steps) if k % 4 == 0]
    ev = {k: _event_pair() for k in sampled}
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(args.steps):
        op_fanout()
        if k in ev:
            _native.time_next_launch(*ev[k])
        op_fanin()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps
    value = bytes_per_step * args.steps / elapsed / 1e9
    dom_us = [a.elapsed_time(b) * 1e3 for a, b in ev.values()]
    dom_avg_us = sum(dom_us) / len(dom_us)
    dom_bytes = ops[1][2]
    achieved = dom_bytes / dom_avg_us / 1e3

    kernels = {}
    for name, fn, nbytes in ops:
        times = []
        for _ in range(20):
            a, b = _event_pair()
            for n2, f, _ in ops:
                if n2 != name:
                    f()
            _native.time_next_launch(a, b)
            fn()
            torch.cuda.synchronize()
            times.append(a.elapsed_time(b) * 1e3)
        med = statistics.median(times)
        kernels[name] = {"bytes": nbytes, "us_median": round(med, 2), "us_min": round(min(times), 2),
                         "GBps": round(nbytes / med / 1e3, 1), "frac_of_peak": round(nbytes / med / 1e3 / HBM_PEAK_GBS, 4)}
        log(f"  {name:15s} {nbytes / 1e6:8.1f} MB  median {med:7.1f} us  {nbytes / med / 1e3:7.1f} GB/s "
            f"({100 * nbytes / med / 1e3 / HBM_PEAK_GBS:.1f}% of peak)")

    def torch_step(slots, shard, cks, src):
        torch_ops.copy_in_fanout(slots, src)
        torch_ops.reduce_scatter_fanin(shard, cks, post, True)

    cpu_baseline = None
    if args.cpu_seconds > 0:
        c_slots = [torch.zeros(s, dtype=torch.bfloat16) for _ in range(w)]
        c_shard = shard0.clone()
        times, spent = [], 0.0
        while spent < args.cpu_seconds and len(times) < 500:
            c0 = time.perf_counter()
            torch_step(c_slots, c_shard, chunks, master)
            dt = time.perf_counter() - c0
            times.append(dt)
            spent += dt
        med = statistics.median(times)
        cpu_baseline = {"value": round(bytes_per_step / med / 1e9, 2), "unit": "GB/s", "cores": torch.get_num_threads(),
                        "kind": "port",
                        "sample": f"{len(times)} passes of the same two steps with torch ops on CPU tensors (W copy_ calls; "
                                  f"fp32 sum of W chunks, cast, div_, add_), median, {spent:.1f}s total"}
        log(f"cpu baseline: {cpu_baseline['value']} GB/s on {cpu_baseline['cores']} threads ({len(times)} passes)")
    torch_gpu = None
    if not args.no_torch_gpu:
        g_slots = [torch.zeros(s, dtype=torch.bfloat16, device=dev) for _ in range(w)]
        g_shard = shard0.to(dev)
        for _ in range(3):
            torch_step(g_slots, g_shard, d_chunks, d_master)
        torch.cuda.synchronize()
        reps = 20
        c0 = time.perf_counter()
        for _ in range(reps):
            torch_step(g_slots, g_shard, d_chunks, d_master)
        torch.cuda.synchronize()
        dt = (time.perf_counter() - c0) / reps
        torch_gpu = {"value": round(bytes_per_step / dt / 1e9, 1), "unit": "GB/s", "ms_per_step": round(dt * 1e3, 4),
                     "sample": f"{reps} passes of the same torch ops on device tensors with torch {torch.__version__}, "
                               f"rated with the fused passes' bytes"}
        log(f"torch ops on the GPU: {torch_gpu['value']} GB/s, {torch_gpu['ms_per_step']} ms per step")

    out = {
        "metric": "HBM GB/s + % of peak for the exchange-point kernels (copy-in fan-out, reduce fan-in) over W local buffers",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": args.workload, "shard_numel": s, "buffers": w, "rank": r, "bytes_per_step": bytes_per_step,
                   "ops": "fp32 master shard [S] -> bf16 into W buffers; W bf16 chunks [S] summed in fp32, /W, += fp32 shard"},
        "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4), "parity": parity,
        "roofline": {"bound": "hbm", "kernel": "fanin_kernel (reduce fan-in)", "achieved": round(achieved, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None,
                     "algorithmic_bytes": dom_bytes, "avg_launch_us": round(dom_avg_us, 2), "launches_timed": len(dom_us)},
        "cpu_baseline": cpu_baseline, "torch_gpu_baseline": torch_gpu, "kernels": kernels,
    }
    print(json.dumps(out), flush=True)
    return 0


def run_ceilings(args) -> int:
    """What this chip's HBM gives streaming kernels of the library at the size of the headline buffer (one bf16
    layer buffer, 436 MB): read-only (sum of squares), write-only (fill), 1:1 copy (same-dtype flat copy), and
    torch's device-to-device copy_ for comparison.  Random data (all-zero buffers run faster on this memory)."""
    import torch

    from yafsdp_amd import _native

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    n = 218_112_000
    g = torch.Generator(device=dev).manual_seed(7)
    a = (torch.randn(n // 2, device=dev, generator=g) * 0.02).bfloat16().repeat(2)
    b = torch.empty_like(a)
    big = (torch.randn(n // 2, device=dev, generator=g)).bfloat16().repeat(2)  # evictor: another 436 MB
    big2 = torch.empty_like(big)
    out = torch.zeros(1, dtype=torch.float64, device=dev)
    partials = torch.empty(_native.SUMSQ_MAX_PARTIALS, dtype=torch.float64, device=dev)
    cases = [
        ("read_only_sumsq_bf16", lambda: _native.sumsq_partials(a, partials, 0), n * 2),
        ("write_only_fill_bf16", lambda: _native.flat_fill(b, 1.5), n * 2),
        ("copy_bf16_to_bf16", lambda: _native.flat_copy(b, a), n * 4),
        ("copy_f32_to_f32", lambda: _native.flat_copy(b.view(torch.float32), a.view(torch.float32)), n * 4),
    ]
    kernels = {}
    for name, fn, nbytes in cases:
        times = []
        for _ in range(max(args.steps, 20)):
            _native.flat_copy(big2, big)  # evict
            x, y = _event_pair()
            _native.time_next_launch(x, y)
            fn()
            torch.cuda.synchronize()
            times.append(x.elapsed_time(y) * 1e3)
        med = statistics.median(times)
        kernels[name] = {"bytes": nbytes, "us_median": round(med, 2), "us_min": round(min(times), 2),
                         "GBps": round(nbytes / med / 1e3, 1), "frac_of_peak": round(nbytes / med / 1e3 / HBM_PEAK_GBS, 4)}
        log(f"  {name:24s} {nbytes / 1e6:8.1f} MB  median {med:7.1f} us  {nbytes / med / 1e3:7.1f} GB/s "
            f"({100 * nbytes / med / 1e3 / HBM_PEAK_GBS:.1f}% of peak)")
    times = []
    for _ in range(20):  # torch's own device-to-device copy (a runtime blit kernel), bracketed by events
        _native.flat_copy(big2, big)
        x, y = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        x.record()
        b.copy_(a)
        y.record()
        torch.cuda.synchronize()
        times.append(x.elapsed_time(y) * 1e3)
    med = statistics.median(times)
    kernels["torch_copy_bf16"] = {"bytes": n * 4, "us_median": round(med, 2), "us_min": round(min(times), 2),
                                  "GBps": round(n * 4 / med / 1e3, 1), "frac_of_peak": round(n * 4 / med / 1e3 / HBM_PEAK_GBS, 4)}
    log(f"  {'torch_copy_bf16':24s} {n * 4 / 1e6:8.1f} MB  median {med:7.1f} us  {n * 4 / med / 1e3:7.1f} GB/s")
    # ---- what a 1:1 copy SUSTAINS: 40 copies back to back over four source / destination pairs (3.5 GB of
    # buffers in rotation), timed from the first kernel's begin to the last one's end.  A single dispatch timed by
    # itself flatters write-through stores (the kernel ends while the memory-side cache still holds its output,
    # and the next kernel pays for the write-back) and penalises non-temporal ones (the kernel's end waits for the
    # L2s' dirty lines); a train of copies counts every byte of every policy once.
    pairs = [(torch.empty_like(a), a.clone()) for _ in range(4)]
    for label, tail in (("non_temporal_stores", 0), ("write_through_stores", 1 << 20)):
        saved = _native.get_option(_native.OPT_FLAT_TAIL_MB)
        _native.set_option(_native.OPT_FLAT_TAIL_MB, tail)
        try:
            rates = []
            for _ in range(5):
                for dst_, src_ in pairs:
                    _native.flat_copy(dst_, src_)
                x, y = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                x.record()
                for k in range(40):
                    _native.flat_copy(*pairs[k % 4])
                y.record()
                torch.cuda.synchronize()
                rates.append(40 * n * 4 / (x.elapsed_time(y) * 1e3) / 1e3)
        finally:
            _native.set_option(_native.OPT_FLAT_TAIL_MB, saved)
        med = statistics.median(rates)
        kernels[f"copy_bf16_train_of_40_over_4_buffer_pairs_{label}"] = {
            "bytes": n * 4, "us_median": round(n * 4 / med / 1e3, 2), "GBps": round(med, 1),
            "frac_of_peak": round(med / HBM_PEAK_GBS, 4)}
        log(f"  train of 40 copies, {label}: {med:7.1f} GB/s ({100 * med / HBM_PEAK_GBS:.1f}% of peak)")
    del pairs
    stream_mixes = _stream_mix_ceilings(torch, _native, dev, lambda: _native.flat_copy(big2, big), max(args.steps, 10))
    best = kernels["copy_bf16_to_bf16"]
    out_line = {
        "metric": "HBM GB/s of plain streaming kernels (read-only, write-only, 1:1 copy) at the headline buffer size",
        "value": best["GBps"], "unit": "GB/s", "n_gpus": 1, "steps": max(args.steps, 20), "warmup": 0,
        "ms_per_step": round(best["us_median"] / 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": args.workload, "elements": n},
        "roofline": {"bound": "hbm", "kernel": "flat_kernel (bf16 -> bf16 copy)", "achieved": best["GBps"],
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": best["frac_of_peak"], "traffic": None},
        "cpu_baseline": None, "kernels": kernels, "stream_mixes": stream_mixes,
    }
    print(json.dumps(out_line), flush=True)
    return 0


def _stream_mix_ceilings(torch, _native, dev, evict, reps):
    """What a single pass over SEVERAL arrays at once reaches on this memory system: the measurement-only mover of
    yafsdp_amd/csrc/ceilings.hip (no arithmetic to speak of) with the stream mixes of the optimizer-side kernels, over
    workgroup shapes, with the arrays at their natural addresses and skewed against each other; next to it the
    library's own kernel of each mix on the same arrays.  One rank's shard of the Llama-3-8B layer (27.3 M elements)."""
    import ctypes

    path = os.path.join(ROOT, "yafsdp_amd", "libyafsdp_ceilings.so")
    if not os.path.exists(path):
        log(f"stream-mix ceilings skipped: {path} is not built (python -m yafsdp_amd._build)")
        return None
    lib = ctypes.CDLL(path)
    vp = ctypes.c_void_p
    lib.ceil_stream_mix.restype = ctypes.c_int
    lib.ceil_stream_mix.argtypes = [ctypes.c_int] * 5 + [vp, vp, vp, ctypes.c_int64, vp, vp, vp]
    n = 26_624 * 1024  # 27,262,976 elements: whole tiles for every shape below
    gen = torch.Generator(device=dev).manual_seed(11)
    stream = vp(torch.cuda.current_stream(dev).cuda_stream)

    def arrays(count, skew_bytes):
        """`count` binary32 arrays of n elements cut from one allocation, array k shifted by k * skew_bytes."""
        stride = n * 4 + skew_bytes
        pool = torch.empty((count * stride + 256) // 4, dtype=torch.float32, device=dev)
        pool.copy_(torch.randn(pool.numel(), device=dev, generator=gen) * 0.02)
        return pool, [pool[(k * stride) // 4 : (k * stride) // 4 + n] for k in range(count)]

    def ptrs(tensors):
        return (vp * max(1, len(tensors)))(*[t.data_ptr() for t in tensors]) if tensors else (vp * 1)()

    def timed(fn_with_events):
        times = []
        for _ in range(reps):
            evict()
            a, b = _event_pair()
            fn_with_events(a, b)
            torch.cuda.synchronize()
            times.append(a.elapsed_time(b) * 1e3)
        return statistics.median(times), min(times)

    def mover(nr, nw32, nw16, block, unroll, reads, w32, w16):
        def run(a, b):
            rc = lib.ceil_stream_mix(nr, nw32, nw16, block, unroll, ptrs(reads), ptrs(w32), ptrs(w16), n, stream,
                                     vp(a.cuda_event), vp(b.cuda_event))
            if rc != 0:
                raise RuntimeError(f"ceil_stream_mix({nr},{nw32},{nw16},{block},{unroll}) returned {rc}")
        return run

    def row(us, nbytes):
        med, lo = us
        return {"bytes": nbytes, "us_median": round(med, 2), "us_min": round(lo, 2), "GBps": round(nbytes / med / 1e3, 1),
                "frac_of_peak": round(nbytes / med / 1e3 / HBM_PEAK_GBS, 4)}

    out = {}
    shapes = [(64, 1), (64, 2), (64, 4), (128, 1), (128, 2), (128, 4), (256, 1), (256, 2), (256, 4), (512, 1), (512, 2),
              (1024, 1)]
    # ---- the fused AdamW mix: p, g, m, v read; p, m, v (binary32) and the 2-byte all-gather input written
    adam_bytes = n * 30
    for skew in (0, 4096 + 256, 1 << 20):
        pool, (p_, g_, m_, v_) = arrays(4, skew)
        out16 = torch.empty(n, dtype=torch.bfloat16, device=dev)
        table = {}
        for block, unroll in shapes:
            table[f"{block}x{unroll}"] = row(timed(mover(4, 3, 1, block, unroll, [p_, g_, m_, v_], [p_, m_, v_], [out16])),
                                             adam_bytes)
        best = max(table, key=lambda k: table[k]["GBps"])

        def adam(a, b):
            _native.time_next_launch(a, b)
            _native.adamw_step(p_, g_, m_, v_, out16, lr=1e-3, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1, step=3)

        out[f"adamw_mix_4r_3w32_1w16_skew_{skew}"] = {"mover_by_shape": table, "mover_best_shape": best,
                                                      "mover_best": table[best], "library_adamw_kernel": row(timed(adam), adam_bytes)}
        log(f"  AdamW mix (16 B read, 14 B written per element), arrays skewed by {skew} B: mover best {best} "
            f"{table[best]['GBps']} GB/s ({table[best]['us_median']} us), library kernel "
            f"{out[f'adamw_mix_4r_3w32_1w16_skew_{skew}']['library_adamw_kernel']['GBps']} GB/s")
        del pool, p_, g_, m_, v_, out16
    # ---- one array read and written in place (the scaling pass), and one read / another written
    pool, (x_, y_) = arrays(2, 0)
    coef = torch.tensor([0.5], device=dev)
    table = {f"{b_}x{u_}": row(timed(mover(1, 1, 0, b_, u_, [x_], [x_], [])), n * 8) for b_, u_ in shapes}
    best = max(table, key=lambda k: table[k]["GBps"])

    def scale(a, b):
        _native.time_next_launch(a, b)
        _native.flat_scale(x_, coef)

    out["in_place_1r_1w32"] = {"mover_by_shape": table, "mover_best_shape": best, "mover_best": table[best],
                               "library_scale_kernel": row(timed(scale), n * 8)}
    log(f"  in-place mix (4 B read, 4 B written): mover best {best} {table[best]['GBps']} GB/s, library scale kernel "
        f"{out['in_place_1r_1w32']['library_scale_kernel']['GBps']} GB/s")
    table = {f"{b_}x{u_}": row(timed(mover(1, 0, 0, b_, u_, [x_], [], [])), n * 4) for b_, u_ in shapes}
    best = max(table, key=lambda k: table[k]["GBps"])
    partials = torch.empty(_native.SUMSQ_MAX_PARTIALS, dtype=torch.float64, device=dev)

    def sumsq(a, b):
        _native.time_next_launch(a, b)
        _native.sumsq_partials(x_, partials, 0)

    out["read_only_1r"] = {"mover_by_shape": table, "mover_best_shape": best, "mover_best": table[best],
                           "library_sumsq_kernel": row(timed(sumsq), n * 4)}
    log(f"  read-only, 109 MB: mover best {best} {table[best]['GBps']} GB/s, library sum-of-squares kernel "
        f"{out['read_only_1r']['library_sumsq_kernel']['GBps']} GB/s")
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--regions", type=int, default=3,
                    help="how many times the timed region (warm-up + exactly --steps steps) is run; the median is reported")
    ap.add_argument("--workload", default="llama3-8b-layer-w8",
                    choices=sorted(WORKLOADS) + ["llama3-8b-full-w8", "ragged-stress-w256", "ragged-stress-w256-bf16-masters",
                                                 "llama3-8b-layer-w8-optim",
                                                 "llama3-70b-layer-w64-optim", "llama3-8b-layer-w8-exchange", "hbm-ceilings", "launch-timeline",
                                                 "fully-shard-trainer-w1"])
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="budget of the CPU baseline leg (0 disables it)")
    ap.add_argument("--no-parity", action="store_true", help="skip the in-run bit-exactness check against the oracle")
    ap.add_argument("--buffer-sets", "--rotating-sets", type=int, default=4, metavar="K", dest="buffer_sets",
                    help="sets of buffers that take turns in the timed region (step k runs on set k mod K; each set of "
                         "the default workload is 2 GB).  1: one set rewritten step after step, which finds its own "
                         "output in the memory-side cache")
    ap.add_argument("--stream-plan", action="store_true",
                    help="add the leg that runs the step on the reference's two streams")
    ap.add_argument("--store-policy-ab", action="store_true",
                    help="add the leg that repeats the rotating loop under other store policies")
    ap.add_argument("--graph", action="store_true",
                    help="add the leg that replays the rotating steps from HIP graphs")
    ap.add_argument("--variants", action="store_true",
                    help="add the table of the other forms of the same kernels (accumulating reduce copy-in, "
                         "post-reduce as a copy, same-dtype copies, in-place divide, each launch alone)")
    for old in ("--no-stream-plan", "--no-store-policy-ab", "--no-rotating-sets", "--no-graph"):
        ap.add_argument(old, action="store_true", help=argparse.SUPPRESS)  # these legs are off unless asked for
    ap.add_argument("--no-torch-gpu", action="store_true",
                    help="skip the leg that times the reference's torch ops on the GPU (outside the timed region)")
    ap.add_argument("--sweep-grid-cap", action="store_true",
                    help="llama3-8b-full-w8 only: repeat the overlap measurement with the copy kernels' grids capped "
                         "at 16/8/4/2/1 workgroups per compute unit")
    ap.add_argument("--copy-cus", type=int, default=0, metavar="K",
                    help="llama3-8b-full-w8 only: run the copies on a stream limited to K of the 256 compute units "
                         "and the GEMMs on a stream limited to the others")
    ap.add_argument("--layers", type=int, default=4, help="fully-shard-trainer-w1 only: decoder layers")
    ap.add_argument("--seq-len", type=int, default=4096, help="fully-shard-trainer-w1 only: tokens per iteration")
    ap.add_argument("--logical-world-size", type=int, default=1, metavar="W",
                    help="fully-shard-trainer-w1 only: wrap with mesh=(W, W // 2), i.e. time one rank's share of a "
                         "W-rank run (its shard of every group; the exchanges between ranks are not part of it)")
    ap.add_argument("--calibrate-copy", type=int, default=0, metavar="N",
                    help="also launch N plain bf16->bf16 flat copies of T_pad elements (a kernel of known traffic, "
                         "used to scale rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE readings); outside the timed region")
    ap.add_argument("--no-fused", action="store_true",
                    help="four launches per step, one per op of the path.  Default: copy-in and copy-out share one "
                         "launch, and a shard group of size one also runs reduce copy-in and post-reduce as one launch")
    ap.add_argument("--no-configs", action="store_true",
                    help="default workload only: skip the `configs` block (the other configurations of the path, each "
                         "with its own oracle check, about a minute in total)")
    ap.add_argument("--sustained-seconds", type=float, default=0.0,
                    help="add a sustained leg: back-to-back rotating steps of the workload for at least this long")
    ap.add_argument("--table-large-log2", type=int, default=None, metavar="N",
                    help="tables with more than 2^N padded elements run two waves per workgroup instead of one "
                         "(the library's launch-shape option; default: the library's own threshold)")
    ap.add_argument("--gather-tail-mb", type=int, default=None, metavar="N",
                    help="megabytes at the end of the reduce buffer that the reduce copy-in stores write-through "
                         "(the library's store-policy option; default: the library's own, 64; 0 = none)")
    ap.add_argument("--scatter-tail-mb", type=int, default=None, metavar="N",
                    help="the same for the last megabytes of tensors that copy-out writes (default: the library's "
                         "own, 0 = none)")
    ap.add_argument("--flat-tail-mb", type=int, default=None, metavar="N",
                    help="the same for the flat kernels (copy-in, flat copies and divides; default 0: they store "
                         "everything non-temporal; 1048576 = write-through everywhere)")
    ap.add_argument("--post-reduce-tail-mb", type=int, default=None, metavar="N", help="the same for the post-reduce")
    ap.add_argument("--copies-only", action="store_true",
                    help="llama3-8b-full-w8 only: run just the copies-only pass under four ways of handing work "
                         "between the two streams (for a kernel trace)")
    ap.add_argument("--analyze-gaps", metavar="CSV", default=None,
                    help="no GPU work; summarise the idle time between consecutive kernels in the kernel-trace CSV that "
                         "rocprofv3 wrote for `--workload llama3-8b-full-w8 --copies-only --no-parity`")
    ap.add_argument("--analyze-trace", metavar="CSV", default=None,
                    help="llama3-8b-full-w8 only: no GPU work; summarise the kernel-trace CSV that rocprofv3 wrote for "
                         "`--workload llama3-8b-full-w8 --steps 10 --no-parity` (GEMM resource columns, concurrency)")
    args = ap.parse_args()

    if args.analyze_trace:
        return analyze_overlap_trace(args.analyze_trace)
    if args.analyze_gaps:
        return analyze_gaps(args.analyze_gaps)
    if args.gpus != 1:
        log(f"bench.py: this build runs on ONE GPU (the logical world size is a layout parameter); "
            f"--gpus {args.gpus} is not supported.")
        return 2

    import torch

    if not torch.cuda.is_available():
        log("bench.py: no GPU visible; the buffer path has no CPU implementation to measure.")
        return 3
    from yafsdp_amd import _native

    for value, option in ((args.gather_tail_mb, _native.OPT_GATHER_TAIL_MB),
                          (args.scatter_tail_mb, _native.OPT_SCATTER_TAIL_MB),
                          (args.flat_tail_mb, _native.OPT_FLAT_TAIL_MB),
                          (args.post_reduce_tail_mb, _native.OPT_POST_REDUCE_TAIL_MB)):
        if value is not None:  # the library's store-policy options, for every workload
            _native.set_option(option, value)
    if args.workload == "llama3-8b-full-w8":
        return run_full_model(args)
    if args.workload.endswith("-optim"):
        return run_optim(args)
    if args.workload.endswith("-exchange"):
        return run_exchange(args)
    if args.workload == "hbm-ceilings":
        return run_ceilings(args)
    if args.workload == "launch-timeline":
        return run_timeline(args)
    if args.workload == "fully-shard-trainer-w1":
        return run_trainer(args)
    try:
        out = run_layer(args, args.workload, args.steps, args.warmup, full=True)
        if args.workload == "llama3-8b-layer-w8" and not args.no_configs:
            # the other configurations of the path, each with its own in-run oracle check (outside the headline's
            # timed region; bounded: fewer steps, no per-kernel tables, no baselines)
            out["configs"] = {}
            for wl, steps, warm in (("tiny-layer-w1", 2000, 100), ("llama3-70b-layer-w64", 20, 5),
                                    ("ragged-stress-w256", 30, 5), ("ragged-stress-w256-bf16-masters", 30, 5)):
                t0 = time.perf_counter()
                out["configs"][wl] = run_layer(args, wl, steps, warm, full=False)
                log(f"config {wl}: {out['configs'][wl]['value']} GB/s, {time.perf_counter() - t0:.1f}s wall")
            # the full-model pass next to GEMMs on a second stream (its own oracle check of an overlapped pass)
            t0 = time.perf_counter()
            rec = run_full_model(args, as_record=True)
            if not isinstance(rec, dict):
                raise ParityError("llama3-8b-full-w8: the overlapped pass differs from the oracle")
            out["configs"]["llama3-8b-full-w8"] = rec
            log(f"config llama3-8b-full-w8: overlap efficiency {rec['value']}, {time.perf_counter() - t0:.1f}s wall")
    except ParityError as exc:
        log(f"bench.py: {exc}; refusing to report a throughput.")
        return 4
    print(json.dumps(out), flush=True)
    return 0


class ParityError(RuntimeError):
    pass


def cpu_model() -> str:
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def run_layer(args, workload: str, steps: int, warmup: int, full: bool = True) -> dict:
    """One parameter group's pass (copy-in, copy-out, reduce copy-in, post-reduce) on synthetic inputs of the named
    workload, over ``--buffer-sets`` sets of buffers taking turns (step k runs on set k mod K): parity of every set
    against the oracle, `warmup` untimed and `steps` timed passes.  `full` adds the per-kernel table, the one-set
    loop and the baselines (and the legs asked for by flags); without it only the timed passes and the parity check
    run, and a compact record comes back."""
    import torch

    from yafsdp_amd import _native
    from yafsdp_amd._layout import make_layout

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.table_large_log2 is not None:
        _native.set_option(_native.OPT_TABLE_LARGE_LOG2, args.table_large_log2)
    # master / compute / reduce dtypes of the group: fp32 masters with bf16 compute and reduce, except the stress
    # test's second group (bf16 masters: no copy-in cast, fp32 reduce buffer, bf16 gradient shard)
    master_dt, rs_dt = torch.float32, torch.bfloat16
    if workload == "ragged-stress-w256":
        shapes, w, r, align, seed = _ragged_stress_shapes(), 256, 1, 512, 1005
    elif workload == "ragged-stress-w256-bf16-masters":
        shapes, w, r, align, seed = _ragged_stress_shapes(fp32_masters=False), 256, 1, 512, 1005
        master_dt, rs_dt = torch.bfloat16, torch.float32
    else:
        shapes, w, r, align, seed = WORKLOADS[workload]
    msz, rsz = master_dt.itemsize, rs_dt.itemsize
    has_copy_in = master_dt != torch.bfloat16
    numels = [numel_of(s) for s in shapes]
    lay = make_layout(numels, w, align)
    t, t_pad, s = lay.total_numel, lay.padded_unsharded_numel, lay.padded_sharded_numel
    pre = float(w) if w > 1 else None
    n_sets = max(1, args.buffer_sets)
    log(f"workload {workload}: P={len(numels)} T={t} T_pad={t_pad} S={s} W={w} rank={r} pre-divide={pre}, "
        f"{n_sets} buffer set(s) in rotation")

    # ---- synthetic inputs, generated on the CPU so that the oracle sees the same bits
    g = torch.Generator().manual_seed(seed)
    t0 = time.perf_counter()
    master = (torch.randn(s, generator=g) * 0.02).to(master_dt)  # master shard
    gathered = torch.empty(t_pad, dtype=torch.bfloat16)
    grads = []
    pos = 0
    for n in numels:  # chunked generation keeps the fp32 temporaries small
        gathered[pos : pos + n] = (torch.randn(n, generator=g) * 0.02).bfloat16()
        grads.append((torch.randn(n, generator=g) * 1e-3).bfloat16())
        pos += n
    gathered[t:] = 0
    shard0 = (torch.randn(s, generator=g) * 1e-4).to(master_dt)  # existing gradient shard (master dtype)
    log(f"inputs generated in {time.perf_counter() - t0:.1f}s")

    table = _native.TensorTable(numels, t_pad, dev)

    # ---- K sets of buffers: the first from the host inputs, the others device copies of it at their own addresses.
    # A training run never comes back to a buffer before gigabytes of other traffic have passed (the reference's
    # groups take turns on two gathered buffers and one reduce buffer, ya_fsdp/_state.py:636-652): with ONE set
    # rewritten step after step a kernel finds what the step before left in the 256-MB memory-side cache, which
    # flatters it.  The timed region therefore rotates over K sets (2 GB each for the default workload).
    def first_set():
        d = {"master": master.to(dev), "gathered": gathered.to(dev), "grads": [x.to(dev) for x in grads],
             "ag_in": torch.zeros(s, dtype=torch.bfloat16, device=dev),
             "outs": [torch.empty(n, dtype=torch.bfloat16, device=dev) for n in numels],
             "rs": torch.zeros(t_pad, dtype=rs_dt, device=dev), "shard": shard0.to(dev)}
        return d

    def another_set(d0):
        return {"master": d0["master"].clone(), "gathered": d0["gathered"].clone(),
                "grads": [x.clone() for x in d0["grads"]], "ag_in": torch.zeros_like(d0["ag_in"]),
                "outs": [torch.empty_like(x) for x in d0["outs"]], "rs": torch.zeros_like(d0["rs"]),
                "shard": shard0.to(dev)}

    sets = [first_set()]
    for _ in range(n_sets - 1):
        sets.append(another_set(sets[0]))
    fused_unshard = has_copy_in and not args.no_fused
    fused_reduce = w == 1 and has_copy_in and not args.no_fused
    for d in sets:
        d["chunk"] = d["rs"][r * s : (r + 1) * s]
        # the copy-out destinations persist across steps: their side of the table is bound once.  Gradients are
        # fresh allocations of autograd in a training step, so the reduce copy-in passes its pointers on every call.
        d["out_binding"] = table.bind(d["outs"])

    copy_in_bytes, copy_out_bytes = s * (msz + 2), 2 * t * 2
    gather_bytes, post_bytes = t * (2 + rsz) + (t_pad - t) * rsz, s * (rsz + 2 * msz)

    def ops_of(d):
        """(name, launch, algorithmic bytes) of one step on buffer set d."""
        def unshard():
            if not table.copy_in_scatter_out(d["gathered"], d["outs"], d["ag_in"], d["master"]):
                raise RuntimeError("copy_in_scatter_out declined")

        def reduce_one_launch():
            if not table.gather_in_post_reduce(d["grads"], d["rs"], d["shard"], True):
                raise RuntimeError("gather_in_post_reduce declined")

        ops = []
        if fused_unshard:
            # copy-in and copy-out as one grid (both sit back to back on the all-gather stream in the reference,
            # ya_fsdp/_collectives.py:46-58 and ya_fsdp/_param_group.py:581-594)
            ops.append(("copy_in_and_copy_out", unshard, copy_in_bytes + copy_out_bytes))
        else:
            if has_copy_in:  # otherwise the all-gather input aliases the master shard (ya_fsdp/_param_group.py:502-505)
                ops.append(("copy_in", lambda: _native.flat_copy(d["ag_in"], d["master"]), copy_in_bytes))
            ops.append(("copy_out", lambda: d["out_binding"].scatter_out(d["gathered"]), copy_out_bytes))
        if fused_reduce:
            # a shard group of size one: nothing happens between reduce copy-in and post-reduce
            # (ya_fsdp/_collectives.py:140-150), one launch does both
            ops.append(("reduce_copy_in_and_post_reduce", reduce_one_launch, gather_bytes + post_bytes))
        else:
            ops.append(("reduce_copy_in", lambda: table.gather_in(d["grads"], d["rs"], None, pre, True), gather_bytes))
            ops.append(("post_reduce", lambda: _native.post_reduce(d["shard"], d["chunk"], None, True), post_bytes))
        return ops

    set_ops = [ops_of(d) for d in sets]
    set_fns = [[fn for _, fn, _ in ops] for ops in set_ops]
    op_names = [n for n, _, _ in set_ops[0]]
    op_bytes = [b for _, _, b in set_ops[0]]
    # what the reference's four ops move, however many launches do it
    bytes_per_step = (copy_in_bytes if has_copy_in else 0) + copy_out_bytes + gather_bytes + post_bytes
    dominant = "reduce_copy_in_and_post_reduce" if fused_reduce else "reduce_copy_in"
    dom_index = op_names.index(dominant)

    def step(k=0):
        for fn in set_fns[k % n_sets]:
            fn()

    # ---- parity of one pass on EVERY buffer set (same run, same inputs): the first set against the oracle on the
    # host, the others against the first on the device (they hold copies of the same inputs)
    parity = "skipped"
    cpu_state = None
    cpu_step = None
    if not args.no_parity:
        from oracle import torch_ops

        def cpu_step(st):
            if has_copy_in:
                torch_ops.copy_in(st["ag_in"], master)
            torch_ops.copy_out_materialize(gathered, numels, st["outs"])
            torch_ops.reduce_copy_in(st["rs_views"], grads, False)
            torch_ops.reduce_scatter_local(st["shard"], st["rs"], w, r, pre, None, "add")

        rs_cpu = torch.zeros(t_pad, dtype=rs_dt)
        cpu_state = {
            "ag_in": torch.zeros(s, dtype=torch.bfloat16),
            "outs": [torch.empty(n, dtype=torch.bfloat16) for n in numels],
            "rs": rs_cpu,
            "rs_views": list(rs_cpu[:t].split(numels)),
            "shard": shard0.clone(),
        }
        cpu_step(cpu_state)
        for k in range(n_sets):
            step(k)
        torch.cuda.synchronize()

        def bits(a):
            return a.view(torch.int32 if a.dtype == torch.float32 else torch.int16)

        def same(a, b):
            return torch.equal(bits(a.cpu()), bits(b))

        d0 = sets[0]
        ok = same(d0["ag_in"], cpu_state["ag_in"]) and same(d0["rs"], cpu_state["rs"]) and same(d0["shard"], cpu_state["shard"])  # noqa: E501 (ag_in stays zero on both sides without a copy-in)
        ok = ok and all(same(a, b) for a, b in zip(d0["outs"], cpu_state["outs"]))
        for d in sets[1:]:
            ok = ok and all(torch.equal(bits(d[key]), bits(d0[key])) for key in ("ag_in", "rs", "shard"))
            ok = ok and all(torch.equal(bits(a), bits(b)) for a, b in zip(d["outs"], d0["outs"]))
        parity = "bit-exact" if ok else "MISMATCH"
        log(f"parity vs oracle ({n_sets} buffer sets):", parity)
        if not ok:
            raise ParityError(f"{workload}: GPU results differ from the oracle")

    if args.calibrate_copy > 0:
        d_copy = torch.empty(t_pad, dtype=torch.bfloat16, device=dev)
        for _ in range(args.calibrate_copy):
            _native.flat_copy(d_copy, sets[0]["gathered"])
        torch.cuda.synchronize()
        del d_copy

    # ---- timed region: `warmup` untimed steps, then exactly `steps` steps between two synchronisations, step k on
    # buffer set k mod K.  The region is run --regions times (3 unless told otherwise) and the MEDIAN region is the
    # one reported (all are listed in the line): the step is driven from the host, a region lasts a few
    # milliseconds, and one stall of the host or the machine inside it (seen once in about twenty runs: 25 ms of
    # idle GPU in a 16-ms region, with every sampled kernel at its normal duration) would otherwise decide the figure.
    # The kernel `roofline` reports is the reduce copy-in, the launch with the path's arithmetic fused in (cast,
    # divide, pad fill) and the lowest fraction of the step's launches (every launch is in `kernels`).  On every 4th
    # step of the timed region (of a long region: on 16 steps spread evenly; attaching the pair costs host time that
    # a launch-bound workload would see) its dispatch carries a pair of HIP events (attached to the dispatch itself:
    # kernel begin and end on the stream it runs on, no launch gap inside the pair).
    every = max(4, -(-steps // (16 if full else 4)))  # the compact records of the other configurations: 4 samples
    if n_sets > 1 and every % n_sets == 0:
        every += 1  # the samples then fall on every buffer set in turn
    sampled = [k for k in range(steps) if k % every == 0]

    def timed_region(first=0, rotate=True):
        def fns_of(k):
            return set_fns[(first + k) % n_sets] if rotate else set_fns[first]

        for w_ in range(warmup):
            if w_ == 0:  # the event-carrying dispatch path runs once before anything is timed
                prime = _event_pair()
                for i, fn in enumerate(fns_of(w_)):
                    if i == dom_index:
                        _native.time_next_launch(*prime)
                    fn()
                continue
            for fn in fns_of(w_):
                fn()
        torch.cuda.synchronize()
        ev = {k: _event_pair() for k in sampled}
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for k in range(steps):
            for i, fn in enumerate(fns_of(warmup + k)):
                if i == dom_index and k in ev:
                    _native.time_next_launch(*ev[k])
                fn()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        return elapsed, [a.elapsed_time(b) * 1e3 for a, b in ev.values()]

    regions = sorted((timed_region() for _ in range(max(1, args.regions))), key=lambda r: r[0])
    elapsed, dom_us = regions[(len(regions) - 1) // 2]  # the median region (the lower one of an even number)
    region_ms_per_step = [round(r[0] * 1e3 / steps, 4) for r in regions]
    ms_per_step = elapsed * 1e3 / steps
    value = bytes_per_step * steps / elapsed / 1e9
    dom_avg_us = sum(dom_us) / len(dom_us)
    dom_bytes = op_bytes[dom_index]
    achieved = dom_bytes / dom_avg_us / 1e3

    def close_all():
        for d in sets:
            d["out_binding"].close()
        table.close()

    def rate(ms):
        return {"ms_per_step": round(ms, 4), "value": round(bytes_per_step / ms / 1e6, 1), "unit": "GB/s",
                "frac_of_hbm_peak": round(bytes_per_step / ms / 1e6 / HBM_PEAK_GBS, 4)}

    if not full:
        close_all()
        return {
            "value": round(value, 1), "unit": "GB/s", "ms_per_step": round(ms_per_step, 4), "steps": steps,
            "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4), "parity": parity, "bytes_per_step": bytes_per_step,
            "params": len(numels), "padded_numel": t_pad, "shard_numel": s, "logical_world_size": w,
            "buffer_sets": n_sets,
            "dominant_kernel_us": round(dom_avg_us, 2), "dominant_kernel_GBps": round(achieved, 1),
            "launches_per_step": len(op_names), "dominant_kernel": dominant,
            "timed_regions_ms_per_step": region_ms_per_step,
        }

    # ---- ONE buffer set rewritten step after step (outside the timed region): the loop finds part of its own output
    # in the memory-side cache, so this is NOT a rate a training run sees.  Under the library's defaults, and under
    # the opt-in policy tuned to exactly this loop ("single_set": write-through everywhere in the flat kernels and a
    # 96-MB tail of the reduce buffer).
    one_set = None
    if n_sets > 1:
        one_ms = timed_region(rotate=False)[0] * 1e3 / steps
        in_force = _native.get_store_policy()
        try:
            _native.set_store_policy("single_set")
            tuned_ms = timed_region(rotate=False)[0] * 1e3 / steps
        finally:
            _native.set_store_policy(in_force)
        one_set = {"note": "cache-assisted: one buffer set rewritten step after step finds its own output in the "
                           "256-MB memory-side cache; not the headline",
                   "steps": steps, **rate(one_ms), "store_policy_single_set": rate(tuned_ms)}
        log(f"one buffer set (cache-assisted): {one_set['ms_per_step']} ms per step, {one_set['value']} GB/s; under "
            f"the single_set store policy {tuned_ms:.4f} ms")
        for k in range(max(1, warmup)):  # the legs below start from the rotation's steady state
            step(k)
        torch.cuda.synchronize()

    # ---- sustained leg (--sustained-seconds): back-to-back rotating steps for at least that long
    sustained = None
    if args.sustained_seconds > 0:
        n_sus = max(steps, int(args.sustained_seconds / (ms_per_step * 1e-3)) + 1)
        torch.cuda.synchronize()
        s0 = time.perf_counter()
        for k in range(n_sus):
            for fn in set_fns[k % n_sets]:
                fn()
        torch.cuda.synchronize()
        s_dt = time.perf_counter() - s0
        sustained = {"steps": n_sus, "seconds": round(s_dt, 3), **rate(s_dt * 1e3 / n_sus)}
        log(f"sustained: {n_sus} steps in {s_dt:.2f}s, {sustained['value']} GB/s")

    # ---- store policies in rotation (--store-policy-ab): the same rotating loop under other tail settings
    policy_ab = None
    if args.store_policy_ab:
        policy_ab = {}
        in_force = _native.get_store_policy()
        try:
            for name, pol in (("all_stores_non_temporal", (0, 0, 0, 0)), ("gather_tail_128", (0, 0, 0, 128)),
                              ("single_set", "single_set")):
                _native.set_store_policy(pol)
                policy_ab[name] = rate(timed_region()[0] * 1e3 / steps)
        finally:
            _native.set_store_policy(in_force)
        policy_ab["in_force"] = {"policy": list(in_force), **rate(ms_per_step)}
        log("store policies in rotation: " + ", ".join(f"{k} {v['ms_per_step']} ms" for k, v in policy_ab.items()))

    # ---- the same launches on the streams the reference puts them on (--stream-plan): copy-in and copy-out on the
    # side stream that serves all-gather and reduce-scatter (ya_fsdp/_collectives.py:46,
    # ya_fsdp/_param_group.py:80-88), the reduce copy-in on the compute stream (ya_fsdp/_param_group.py:669-708), the
    # post-reduce on the side stream once the compute stream has got there (ya_fsdp/_collectives.py:110-111).
    reference_streams = None
    if args.stream_plan:
        main_stream, side_stream = torch.cuda.current_stream(dev), torch.cuda.Stream(device=dev)

        def reference_step(k):
            done = None
            for name, fn in zip(op_names, set_fns[k % n_sets]):
                if name.startswith("reduce_copy_in"):
                    fn()
                    done = main_stream.record_event()
                else:
                    with torch.cuda.stream(side_stream):
                        if name == "post_reduce" and done is not None:
                            side_stream.wait_event(done)
                        fn()

        n_ref = max(steps, 200)
        side_stream.wait_stream(main_stream)
        for k in range(warmup):
            reference_step(k)
        main_stream.wait_stream(side_stream)
        torch.cuda.synchronize()
        r0 = time.perf_counter()
        for k in range(n_ref):
            reference_step(k)
        main_stream.wait_stream(side_stream)
        torch.cuda.synchronize()
        r_dt = (time.perf_counter() - r0) / n_ref
        reference_streams = {
            "plan": "copy-in + copy-out and post-reduce on a side stream, reduce copy-in on the compute stream",
            "steps": n_ref, **rate(r_dt * 1e3)}
        log(f"the reference's stream placement: {reference_streams['ms_per_step']} ms per step, "
            f"{reference_streams['value']} GB/s")
        if not args.no_parity and cpu_state is not None:
            # the overlapped launches left the same bits (the gradient shard has accumulated many passes:
            # compare the buffers that every pass rewrites)
            d0 = sets[0]
            ok = same(d0["ag_in"], cpu_state["ag_in"]) and same(d0["rs"], cpu_state["rs"])
            ok = ok and all(same(a, b) for a, b in zip(d0["outs"], cpu_state["outs"]))
            if not ok:
                raise ParityError(f"{workload}: results of the two-stream step differ from the oracle")

    # ---- the rotating steps captured into HIP graphs and replayed (--graph): one graph of K steps (one per buffer
    # set) and one of 4 K steps; both sides of the table are bound, so the captured launches carry no per-call host
    # work and no staging copy.  A graph launch has a fixed cost of its own (a few microseconds of idle GPU at its
    # start and end), which the longer graph spreads over four times as many steps.
    graph_replay = None
    if args.graph:
        grad_bindings = [table.bind(d["grads"]) for d in sets]

        def bound_step(k):
            d, gb = sets[k % n_sets], grad_bindings[k % n_sets]
            if fused_unshard and len(numels) <= 16:  # small tables carry their pointers as kernel arguments
                for f in set_fns[k % n_sets]:
                    f()
                return
            if has_copy_in:
                _native.flat_copy(d["ag_in"], d["master"])
            d["out_binding"].scatter_out(d["gathered"])
            gb.gather_in(d["rs"], pre, True)
            _native.post_reduce(d["shard"], d["chunk"], None, True)

        graph_replay = {}
        for rounds in (1, 4):
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for k in range(n_sets):
                    bound_step(k)
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                for k in range(rounds * n_sets):
                    bound_step(k)
            for _ in range(3):
                graph.replay()
            torch.cuda.synchronize()
            n_rep = max(1, steps // (rounds * n_sets))
            g0 = time.perf_counter()
            for _ in range(n_rep):
                graph.replay()
            torch.cuda.synchronize()
            g_dt = (time.perf_counter() - g0) / (n_rep * rounds * n_sets)
            graph_replay[f"{rounds * n_sets}_steps_per_graph"] = rate(g_dt * 1e3)
            del graph
        for gb in grad_bindings:
            gb.close()
        log("HIP graph replay: " + ", ".join(f"{k}: {v['ms_per_step']} ms per step" for k, v in graph_replay.items()))

    # ---- per-kernel table (outside the timed region): every launch of 4 K rotating steps carries an event pair on
    # its own dispatch, so each kernel is rated as it runs inside the rotation
    samples = {n: [] for n in op_names}
    pairs = []
    for k in range(4 * n_sets):
        for name, fn in zip(op_names, set_fns[k % n_sets]):
            a, b = _event_pair()
            _native.time_next_launch(a, b)
            fn()
            pairs.append((name, a, b))
    torch.cuda.synchronize()
    for name, a, b in pairs:
        samples[name].append(a.elapsed_time(b) * 1e3)
    kernels = {}
    for name, nbytes in zip(op_names, op_bytes):
        med = statistics.median(samples[name])
        kernels[name] = {
            "bytes": nbytes, "us_median": round(med, 2), "us_min": round(min(samples[name]), 2),
            "GBps": round(nbytes / med / 1e3, 1), "frac_of_peak": round(nbytes / med / 1e3 / HBM_PEAK_GBS, 4),
            "launches_timed": len(samples[name]),
        }
        log(f"  {name:30s} {nbytes / 1e6:8.1f} MB  median {med:7.1f} us  {nbytes / med / 1e3:7.1f} GB/s "
            f"({100 * nbytes / med / 1e3 / HBM_PEAK_GBS:.1f}% of peak)")

    # ---- the other forms of the same kernels (--variants; ya_fsdp/_param_group.py:701-708,
    # ya_fsdp/_collectives.py:56-58, 139, 185): gradient accumulation into the reduce buffer, the first reduce of an
    # iteration (copy instead of add), the all-gather of a size-1 group, the pre-divide as a pass of its own, a
    # same-dtype fp32 copy, and a 1-byte all-gather dtype class between odd byte addresses.  Each is timed on its own
    # dispatch right behind one step on another buffer set (2 GB of other traffic).
    variants = None
    if args.variants:
        d0 = sets[0]
        d_shard_b = torch.empty_like(d0["shard"])
        d_gathered_b = torch.empty_like(d0["gathered"])
        d_rs_b = torch.zeros_like(d0["rs"])
        d_f32_src = torch.randn(t_pad // 2, device=dev)
        d_f32_dst = torch.empty_like(d_f32_src)
        add_modes = [_native.MODE_ADD] * len(numels)
        d_bytes_src = d0["gathered"].view(torch.uint8)[1 : 1 + t_pad]
        d_bytes_dst = d_gathered_b.view(torch.uint8)[3 : 3 + t_pad]
        variant_ops = [
            ("reduce_copy_in_accumulate", lambda: table.gather_in(d0["grads"], d_rs_b, add_modes, None, True),
             t * (2 + 2 * rsz) + (t_pad - t) * rsz),
            ("post_reduce_copy", lambda: _native.post_reduce(d_shard_b, d0["chunk"], None, False), s * (rsz + msz)),
            ("all_gather_size1_copy", lambda: _native.flat_copy(d_gathered_b, d0["gathered"]), 2 * t_pad * 2),
            ("divide_in_place", lambda: _native.flat_div(d_rs_b, 2.0), 2 * t_pad * rsz),
            ("same_dtype_fp32_copy", lambda: _native.flat_copy(d_f32_dst, d_f32_src), 2 * (t_pad // 2) * 4),
            ("all_gather_1byte_dtype_odd_addresses", lambda: _native.flat_copy(d_bytes_dst, d_bytes_src), 2 * t_pad),
            ("copy_in_alone", lambda: _native.flat_copy(d0["ag_in"], d0["master"]), copy_in_bytes),
            ("copy_out_alone", lambda: d0["out_binding"].scatter_out(d0["gathered"]), copy_out_bytes),
        ]
        variants = {}
        for name, fn, nbytes in variant_ops:
            fn()
            times = []
            for _ in range(10):
                step(1)  # evict: a whole step on another buffer set
                a, b = _event_pair()
                _native.time_next_launch(a, b)
                fn()
                torch.cuda.synchronize()
                times.append(a.elapsed_time(b) * 1e3)
            med = statistics.median(times)
            variants[name] = {"bytes": nbytes, "us_median": round(med, 2), "us_min": round(min(times), 2),
                              "GBps": round(nbytes / med / 1e3, 1),
                              "frac_of_peak": round(nbytes / med / 1e3 / HBM_PEAK_GBS, 4)}
            log(f"  {name:38s} {nbytes / 1e6:8.1f} MB  median {med:7.1f} us  {nbytes / med / 1e3:7.1f} GB/s")
        del d_shard_b, d_gathered_b, d_rs_b, d_f32_src, d_f32_dst

    # ---- CPU baseline: the oracle (reference torch-op sequence) on the host cores
    cpu_baseline = None
    if args.cpu_seconds > 0 and cpu_state is not None:
        cores = os.cpu_count() or 1
        torch.set_num_threads(cores)  # every host core the box shows
        for _ in range(3):            # warm-up passes (page faults, thread pool start-up), not timed
            cpu_step(cpu_state)
        reps, spent = 0, 0.0
        times = []
        while (spent < args.cpu_seconds or reps < 10) and reps < 2000:
            c0 = time.perf_counter()
            cpu_step(cpu_state)
            dt = time.perf_counter() - c0
            times.append(dt)
            spent += dt
            reps += 1
        med = statistics.median(times)
        cpu_baseline = {
            "value": round(bytes_per_step / med / 1e9, 2), "unit": "GB/s", "cores": cores,
            "kind": "port", "cpu_model": cpu_model(), "torch_threads": torch.get_num_threads(),
            "sample": f"{reps} full passes of the same workload ({workload}) with the reference's torch ops "
                      f"on CPU tensors after 3 warm-up passes, median of {reps}, {spent:.1f}s total",
        }
        log(f"cpu baseline: {cpu_baseline['value']} GB/s on {cpu_baseline['cores']} threads ({reps} passes)")

    # ---- the same torch-op sequence on the GPU (torch's own ROCm kernels): what the reference runs on this
    # hardware today, over the same K buffer sets in rotation.  Outside the timed region; reported next to the CPU
    # baseline, not a target.
    torch_gpu = None
    if cpu_state is not None and not args.no_torch_gpu:
        from oracle import torch_ops  # noqa: F811

        def gpu_torch_step(d):
            if has_copy_in:
                torch_ops.copy_in(d["ag_in"], d["master"])
            torch_ops.copy_out_materialize(d["gathered"], numels, d["outs"])
            torch_ops.reduce_copy_in(d["rs_views"], d["grads"], False)
            torch_ops.reduce_scatter_local(d["shard"], d["rs"], w, r, pre, None, "add")

        for d in sets:
            d["rs_views"] = list(d["rs"][:t].split(numels))
        for k in range(n_sets):
            gpu_torch_step(sets[k])
        torch.cuda.synchronize()
        reps = 5 * n_sets
        c0 = time.perf_counter()
        for k in range(reps):
            gpu_torch_step(sets[k % n_sets])
        torch.cuda.synchronize()
        dt = (time.perf_counter() - c0) / reps
        torch_gpu = {
            "value": round(bytes_per_step / dt / 1e9, 1), "unit": "GB/s", "ms_per_step": round(dt * 1e3, 4),
            "sample": f"{reps} passes of the reference's torch ops (copy_, split + copy_, _foreach_copy_, div_, add_) on "
                      f"device tensors with torch {torch.__version__}, same inputs and buffer sets, rated with the "
                      f"same algorithmic bytes",
        }
        log(f"torch ops on the GPU: {torch_gpu['value']} GB/s, {torch_gpu['ms_per_step']} ms per step")

    out = {
        "metric": "HBM GB/s + % of peak for copy-in/out+grad-reduce, Llama-3-8B layer @W=8",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": round(ms_per_step, 4),
        "timed_regions_ms_per_step": region_ms_per_step,  # every region: `warmup` + exactly `steps` steps; the median is reported
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": workload, "params": len(numels), "total_numel": t, "padded_numel": t_pad,
            "shard_numel": s, "logical_world_size": w, "rank": r, "shard_alignment": align,
            "predivide": pre, "bytes_per_step": bytes_per_step,
            "buffer_sets": n_sets,  # step k of the timed region runs on buffer set k mod buffer_sets
            "master_dtype": str(master_dt).replace("torch.", ""), "reduce_dtype": str(rs_dt).replace("torch.", ""),
            "ops": ("copy-in master->bf16 [S]; " if has_copy_in else "") +
                   "copy-out bf16 flat->tensors [T]; reduce copy-in bf16 grads->flat /W [T_pad]; "
                   "post-reduce chunk += gradient shard (master dtype) [S]",
            "launches_per_step": op_names,
            "store_policy_mb_flat_postreduce_scatter_gather": list(_native.get_store_policy()),
        },
        "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4),
        "parity": parity,
        "roofline": {
            "bound": "hbm",
            "kernel": "gather_in_kernel (reduce copy-in)" if dominant == "reduce_copy_in"
                      else "gather_post_kernel (reduce copy-in + post-reduce of a size-one group)",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
            "traffic": MEASURED_TRAFFIC_BYTES.get(workload),
            "algorithmic_bytes": dom_bytes, "avg_launch_us": round(dom_avg_us, 2), "launches_timed": len(dom_us),
            "sampled_in": f"the timed region ({n_sets} buffer sets in rotation)",
        },
        "cpu_baseline": cpu_baseline,
        "torch_gpu_baseline": torch_gpu,
        "one_buffer_set": one_set,
        "kernels": kernels,
    }
    for key, leg in (("sustained", sustained), ("store_policies_in_rotation", policy_ab),
                     ("reference_stream_placement", reference_streams), ("graph_replay", graph_replay),
                     ("kernel_variants", variants)):
        if leg is not None:
            out[key] = leg
    close_all()
    return out


if __name__ == "__main__":
    sys.exit(main())
