#!/usr/bin/env python3
"""Benchmark of the FP8 quantized-collective hot path on one MI355X.

One step = one pass of the path over one gradient bucket, as one rank of an
8-way quantized all-reduce sees it (torchft/collectives.py:364-412):
    quantize   the rank's tensors          -> packed buffer A
    reduce     the received buffer B (8 peer slots) in place, own slot rewritten
    dequantize the gathered buffer G       -> the rank's tensors
The two collectives are not part of the step: B and G are prepared beforehand on
the same GPU from 8 independently seeded peers.  Inputs are resident in HBM
before the timed region.  The step rotates over several buffer sets so that the
256 MB last-level cache cannot hold the working set of the next step ("cold").

Workload: benchmark configuration 3, the Llama-3-8B decoder-layer gradient
bucket (9 bf16 tensors, 218 112 000 elements, per-row std log-uniform in
[1e-5, 1e-1]), world size 8, reduce op AVG.

Prints one JSON line.  `value` is algorithmic bytes of the three stages divided
by the wall time of a step; `roofline` is the kernel with the largest share of
the step against the 8 TB/s HBM peak, timed with HIP events on the launch stream
inside the timed region; `stages` has the same figure for each kernel from a
second pass with events around every stage; `cpu_baseline` is the CPU checker (oracle/, a port of the reference arithmetic - the reference has no
CPU implementation) on the host cores, on a bounded sample of the same bucket.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# HBM bytes per launch on benchmark configuration 3 as profiled (profiles/cfg3_bf16_ws8_hbm_traffic.md)
PROFILED_TRAFFIC = {"quantize": 655474688, "reduce": 248143667, "dequantize": 660078592}
# mean kernel durations in the step of the same workload by rocprofv3 --kernel-trace, us
# (profiles/cfg3_bf16_ws8_kernel_trace.md): the cross-check of the event times below
PROFILED_KERNEL_US = {"quantize": 109.3, "reduce": 43.2, "dequantize": 108.1}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--sets", type=int, default=3, help="buffer sets the steps rotate over")
    ap.add_argument("--rank", type=int, default=None)
    ap.add_argument("--config", default="3", choices=["2", "3", "4", "5", "flat", "shape", "ceiling", "ceiling4"],
                    help="workload: 3 = Llama-3-8B layer bucket (the headline, default); 2, 4, 5 = the "
                         "other GPU configurations; flat = one 1-D fp32 tensor of 64 Mi elements "
                         "(what a bucketised DiLoCo all-reduce passes); shape = --shape; ceiling = "
                         "streaming kernels without arithmetic for the read : write mixes of the "
                         "stages, at the headline workload's footprint, beside the product kernels; "
                         "ceiling4 = the accesses of reduce on configuration 4 (4 peers, rows of 2052 and "
                         "5636 bytes) without arithmetic, beside the product's reduce on that configuration")
    ap.add_argument("--shape", default="53248x4096",
                    help="with --config shape: ROWSxCOLS[,ROWSxCOLS...], N(0, 0.02) values")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float16", "float32"],
                    help="with --config shape")
    ap.add_argument("--ws", type=int, default=8, help="with --config shape: group size (reduce AVG)")
    ap.add_argument("--api", default="named", choices=["named", "prepared", "collective"],
                    help="named: the three functions the reference names, as torchft/collectives.py calls "
                         "them (default); prepared: torchft_amd.quantization.prepare() once per tensor "
                         "list, then the bucket's quantize (into a buffer kept from step to step) / "
                         "reduce / dequantize: the form for a bucket that is reduced every step; "
                         "collective: torchft_amd.collectives.allreduce_quantized on the workload (configs 2, 3, "
                         "shape), through torch.distributed's RCCL process group with this process as its only "
                         "rank and through a group of 8 ranks simulated by threads on the one GPU: wall time "
                         "per call against the time of its kernels, and where the host's time goes")
    ap.add_argument("--footprint", default="3", choices=["2", "3"],
                    help="with --config ceiling: the configuration whose footprint and product kernels are timed "
                         "(3: 436 MB of bf16 tensors in 9 tensors; 2: one bf16 tensor of 33.5 MB)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 256 MiB device copy a few times, so that a counter "
                         "profile of this command contains a kernel of known HBM traffic")
    ap.add_argument("--cpu-rows", type=float, default=1.0,
                    help="fraction of the bucket's rows the CPU baseline runs on")
    return ap.parse_args()


def cpu_baseline(fraction: float):
    """Times the CPU checker on `fraction` of the rows of every tensor of the bucket."""
    import torch
    from torch.distributed import ReduceOp

    import workloads
    from oracle import oracle

    ws = 8
    nthreads = max(1, min(oracle.max_threads(), os.cpu_count() or 1))
    tensors = workloads.cfg3(0, scale_rows=fraction)
    ab = workloads.algorithmic_bytes(tensors, ws)
    outs = [torch.empty_like(t) for t in tensors]
    qbuf = oracle.fused_quantize_into_fp8(list(tensors), ws, nthreads=nthreads)  # warm-up, page-in
    recv = qbuf.clone()  # a full buffer of 8 slots stands in for the received one
    oracle.fused_dequantize_from_fp8(outs, qbuf, ws, nthreads=nthreads)
    tq = tr = td = 0.0
    passes = 0
    while passes < 2 or (tq + tr + td < 10.0 and passes < 400):
        t0 = time.perf_counter()
        qbuf = oracle.fused_quantize_into_fp8(list(tensors), ws, nthreads=nthreads)
        t1 = time.perf_counter()
        oracle.fused_reduce_fp8(list(tensors), recv, ws, 3, ReduceOp.AVG, nthreads=nthreads)
        t2 = time.perf_counter()
        oracle.fused_dequantize_from_fp8(outs, qbuf, ws, nthreads=nthreads)
        t3 = time.perf_counter()
        tq, tr, td = tq + t1 - t0, tr + t2 - t1, td + t3 - t2
        passes += 1
    tq, tr, td = tq / passes, tr / passes, td / passes
    total = sum(ab.values())
    model = ""
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                model = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    # For context: the same arithmetic written with torch CPU operators
    # (oracle/torch_restatement.py, the checker's cross-check), on 1/16 of the rows.
    from oracle import torch_restatement as trs
    small = workloads.cfg3(0, scale_rows=1.0 / 16)
    small_ab = sum(workloads.algorithmic_bytes(small, ws).values())
    small_shapes = [tuple(t.shape) if t.dim() == 2 else (t.shape[0], 1) for t in small]
    small_outs = [torch.empty_like(t) for t in small]
    trs_s, trs_passes = 0.0, 0
    while trs_passes < 2 or (trs_s < 3.0 and trs_passes < 50):
        t0 = time.perf_counter()
        buf = trs.quantize(list(small), ws)
        trs.reduce(small_shapes, buf.clone(), ws, 3, True)
        trs.dequantize(small_outs, buf, ws)
        dt = time.perf_counter() - t0
        if trs_passes > 0:  # the first pass warms up
            trs_s += dt
        trs_passes += 1
    torch_gbs = small_ab * (trs_passes - 1) / trs_s / 1e9

    return {
        "value": round(total / (tq + tr + td) / 1e9, 3),
        "unit": "GB/s",
        "cores": nthreads,
        "torch_cpu_restatement_gbs": round(torch_gbs, 3),
        "kind": "port",
        "sample": f"Llama-3-8B layer bucket, {fraction:g} of the rows of each tensor at full row "
                  f"length, {passes} passes of quantize + reduce (ws=8, AVG) + dequantize, "
                  f"{(tq + tr + td) * passes:.1f} s of CPU work, mean per pass",
        "stages_gbs": {"quantize": round(ab["quantize"] / tq / 1e9, 3),
                       "reduce": round(ab["reduce"] / tr / 1e9, 3),
                       "dequantize": round(ab["dequantize"] / td / 1e9, 3)},
        "cpu_model": model,
    }


def run_ceilings(args) -> int:
    """Streaming ceilings (torchft_amd/csrc/tftq_ceiling.hip) at the footprint of the headline
    workload, and the three product kernels timed the same way: every kernel alone in a loop
    that rotates over `--sets` buffer sets (cold last-level cache), HIP events around each
    launch on the launch stream."""
    import ctypes

    import torch
    from torch.distributed import ReduceOp

    import workloads
    from torchft_amd import _build, _lib, quantization as q

    torch.cuda.set_device(0)
    dev = "cuda"
    if not os.path.exists(_build.CEILING_LIB_PATH):
        _build.build_library()
    C = ctypes.CDLL(_build.CEILING_LIB_PATH)
    C.tftq_ceiling_bytes.argtypes = [ctypes.c_int, ctypes.c_int64, ctypes.c_int,
                                     ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_int64)]
    C.tftq_ceiling_launch.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64,
                                      ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                      ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    ws, rank, nsets = 8, 3, max(2, args.sets)
    stream = torch.cuda.current_stream()
    sp = ctypes.c_void_p(stream.cuda_stream)
    ev = lambda: torch.cuda.Event(enable_timing=True)  # noqa: E731

    def timed(launch, nbytes):
        pairs = [(ev(), ev()) for _ in range(args.steps)]
        torch.cuda.synchronize()
        for i in range(args.warmup):  # the timed launches are queued behind these: no idle GPU in between
            launch(i)
        for i, (a, b) in enumerate(pairs):
            a.record(stream)
            launch(i)
            b.record(stream)
        torch.cuda.synchronize()
        us = sorted(a.elapsed_time(b) * 1e3 for a, b in pairs)
        mean = sum(us) / len(us)
        return {"us": round(mean, 2), "us_min": round(us[0], 2), "bytes": nbytes,
                "GBs": round(nbytes / mean / 1e3, 1), "frac_of_peak": round(nbytes / mean / 1e3 / HBM_PEAK_GBS, 4)}

    # footprint of benchmark configuration 3: 436 MB of bf16 tensors, 218 MB packed, slots of 27 MB;
    # of configuration 2: 33.5 MB, 16.8 MB, 2.1 MB
    U = 13312 if args.footprint == "3" else 1024  # chunks of 32 KB
    big = U * 32768               # 436 207 616 bytes
    rows, row_bytes = U // 2, 4100  # one slot of 4096-column rows
    slot = 27292672 if args.footprint == "3" else 2099200  # slot size of the configuration (a multiple of 128)
    bufs = [(torch.empty(big, dtype=torch.uint8, device=dev).random_(),
             torch.empty(big, dtype=torch.uint8, device=dev).random_()) for _ in range(nsets)]
    NT, PLAIN = (1,), (0,)
    BOTH = (0, 1)
    # (label, kind, units, eighths, nt_loads choices, nt_stores choices)
    kinds = [("read only", 0, U, 0, BOTH, PLAIN), ("write only", 1, U, 0, PLAIN, BOTH),
             ("2:1 read:write (quantize, 16-bit tensors)", 2, U, 0, BOTH, BOTH),
             ("1:2 read:write (dequantize, 16-bit tensors)", 3, U, 0, BOTH, BOTH),
             ("4:1 read:write (quantize, fp32 tensors)", 4, U, 0, BOTH, BOTH),
             ("1:4 read:write (dequantize, fp32 tensors)", 5, U, 0, BOTH, BOTH),
             ("2:1 read:write, 4 steps per lane", 11, 2 * U, 0, NT, NT),
             ("1:2 read:write, 4 steps per lane", 12, 2 * U, 0, NT, NT),
             ("4:1 read:write, 4 steps per lane", 13, 2 * U, 0, NT, BOTH),
             ("1:4 read:write, 4 steps per lane", 14, 2 * U, 0, BOTH, NT),
             ("8:1 read:write, one contiguous source (reduce, 8 peers)", 6, U // 2, 0, BOTH, BOTH),
             ("reduce's accesses: 8 slots, 4100-byte rows, in place, an eighth of the rows per XCD",
              7, rows, 1, NT, BOTH),
             ("reduce's accesses, rows in workgroup order", 7, rows, 0, NT, BOTH),
             ("reduce's accesses, an eighth per XCD, wavefronts start on 128-byte lines", 8, rows, 1, NT, BOTH),
             ("quantize's accesses: 8 KB rows -> 4100-byte packed rows through LDS, rows in workgroup order",
              10, 8 * rows, 0, NT, NT),
             ("quantize's accesses, packed rows straight from the registers (plain stores)",
              10, 8 * rows, 0, NT, PLAIN),
             ("dequantize's accesses: 4100-byte packed rows -> 8 KB rows, rows in workgroup order",
              9, 8 * rows, 0, NT, NT),
             ("dequantize's accesses, an eighth of the rows per XCD", 9, 8 * rows, 1, NT, NT)]
    ceilings = {}
    for name, kind, units, eighths, ntls, ntss in kinds:
        rb, wb = ctypes.c_int64(), ctypes.c_int64()
        assert C.tftq_ceiling_bytes(kind, units, row_bytes, ctypes.byref(rb), ctypes.byref(wb)) == 0
        for ntl in ntls:
            for nts in ntss:
                def launch(i, kind=kind, units=units, eighths=eighths, ntl=ntl, nts=nts):
                    a, b = bufs[i % nsets]
                    rc = C.tftq_ceiling_launch(kind, a.data_ptr(), b.data_ptr(), units, slot, row_bytes,
                                               rank, eighths, ntl, nts, sp)
                    assert rc == 0, rc
                label = name
                if kind < 7 or kind >= 11:
                    label += (", streaming loads" if ntl else ", plain loads") if rb.value else ""
                    label += (", streaming stores" if nts else ", plain stores") if wb.value else ""
                elif kind in (7, 8):
                    label += ", streaming stores" if nts else ", plain stores"
                r = timed(launch, rb.value + wb.value)
                r["read_bytes"], r["write_bytes"], r["kind"] = rb.value, wb.value, kind
                ceilings[label] = r
    del bufs

    # the product kernels on benchmark configuration 3, each alone in the same kind of loop
    sets = []
    for k in range(nsets):
        t = (workloads.cfg3 if args.footprint == "3" else workloads.cfg2)(1000 * k + rank, device=dev)
        packed = q.fused_quantize_into_fp8(t, ws)
        sets.append({"tensors": t, "recv": packed.clone(), "gathered": packed})
    ab = workloads.algorithmic_bytes(sets[0]["tensors"], ws)
    product = {
        # the result is kept until the set's next turn: the output block rotates like the inputs
        "quantize": timed(lambda i: sets[i % nsets].__setitem__(
            "packed", q.fused_quantize_into_fp8(sets[i % nsets]["tensors"], ws)), ab["quantize"]),
        "reduce": timed(lambda i: q.fused_reduce_fp8(sets[i % nsets]["tensors"], sets[i % nsets]["recv"], ws,
                                                     rank, ReduceOp.AVG), ab["reduce"]),
        "dequantize": timed(lambda i: q.fused_dequantize_from_fp8(sets[i % nsets]["tensors"],
                                                                  sets[i % nsets]["gathered"], ws), ab["dequantize"]),
    }

    def best(kind):  # over the flavours of the mix, 8 and 4 steps per lane
        twins = {2: 11, 3: 12, 4: 13, 5: 14}
        return max((v for v in ceilings.values() if v["kind"] in (kind, twins.get(kind))), key=lambda v: v["GBs"])

    mix = {"quantize": 2, "reduce": 6, "dequantize": 3}
    for stage, kind in mix.items():
        c = best(kind)
        product[stage]["ceiling_GBs"] = c["GBs"]
        product[stage]["of_ceiling"] = round(product[stage]["GBs"] / c["GBs"], 4)
    for stage, kind in (("quantize", 10), ("reduce", 7), ("dequantize", 9)):
        c = best(kind)
        product[stage]["own_accesses_GBs"] = c["GBs"]
        product[stage]["of_own_accesses"] = round(product[stage]["GBs"] / c["GBs"], 4)
    out = {"metric": "streaming ceilings and product kernels, each kernel alone, HBM GB/s on 1 MI355X",
           "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
           "config": {"workload": ("footprint of benchmark configuration 3 (436 MB of 16-bit tensors, 218 MB "
                                   "packed, 8 slots)" if args.footprint == "3" else
                                   "footprint of configuration 2 (one bf16 tensor of 33.5 MB, 16.8 MB packed, 8 slots)")
                                  + f"; {nsets} rotating buffer sets"},
           "ceilings": ceilings, "product": product}
    print(json.dumps(out))
    return 0


class _TimedGroup:
    """A process group seen through a stopwatch: host time of every collective call and of
    every wait() on the work objects they return (torchft_amd.collectives calls wait() twice
    per all-reduce), and device events around each collective."""

    def __init__(self, pg, log):
        self._pg, self._log = pg, log

    def rank(self):
        return self._pg.rank()

    def size(self):
        return self._pg.size()

    def _call(self, name, fn, *a):
        import torch
        log = self._log
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        stream = torch.cuda.current_stream()
        e0.record(stream)
        t0 = time.perf_counter()
        work = fn(*a)
        log[name + " call"] = time.perf_counter() - t0
        outer = self

        class Work:
            def wait(self, *wa):
                t = time.perf_counter()
                r = work.wait(*wa)
                log[name + " wait()"] = log.get(name + " wait()", 0.0) + time.perf_counter() - t
                e1.record(torch.cuda.current_stream())
                outer._log.setdefault("events", {})[name] = (e0, e1)
                return r

            def get_future(self):
                fut = work.get_future()
                t_asked = time.perf_counter()
                fut.add_done_callback(lambda f: log.__setitem__(name + " future done after", time.perf_counter() - t_asked))
                return fut

        return Work()

    def alltoall_base(self, *a):
        return self._call("all-to-all", self._pg.alltoall_base, *a)

    def allgather_into_tensor_coalesced(self, *a):
        return self._call("all-gather", self._pg.allgather_into_tensor_coalesced, *a)


class _TimedBucket:
    """A prepared bucket seen through a stopwatch: host time and device events of the three launches."""

    def __init__(self, bucket, log):
        self._b, self._log = bucket, log
        self.ws = bucket.ws

    def matches(self, tensors):
        t = time.perf_counter()
        ok = self._b.matches(tensors)
        self._log["bucket.matches()"] = time.perf_counter() - t
        return ok

    def _launch(self, name, fn, *a):
        import torch
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        stream = torch.cuda.current_stream()
        e0.record(stream)
        t = time.perf_counter()
        r = fn(*a)
        self._log[name + " launch"] = time.perf_counter() - t
        self._log[name + " at"] = t
        e1.record(stream)
        self._log.setdefault("events", {})[name] = (e0, e1)
        return r

    def quantize(self, *a):
        return self._launch("quantize", self._b.quantize, *a)

    def reduce(self, *a):
        return self._launch("reduce", self._b.reduce, *a)

    def dequantize(self, *a):
        return self._launch("dequantize", self._b.dequantize, *a)


def run_collective(args, make, op, workload_name) -> int:
    """allreduce_quantized (torchft/collectives.py:297-415) end to end on one GPU."""
    import socket
    import threading

    import torch
    import torch.distributed as dist
    from torch.distributed import ReduceOp

    import sim_pg
    import workloads
    from torchft_amd import collectives as col, quantization as q

    dev = "cuda"
    nsets = max(2, args.sets)
    K, W = args.steps, args.warmup

    def measure(pg_of, ws, rank_threads):
        """Per rank: W + K calls one after the other, each waited for to the end (latency),
        then K calls queued back to back (throughput).  Returns rank 0's figures."""
        result = {}

        def rank_fn(r):
            torch.cuda.set_device(0)
            pg = pg_of(r)
            stream = torch.cuda.Stream()
            sets = [make(1000 * k + r) for k in range(nsets)]
            buckets = [q.prepare(t, ws) for t in sets]
            ab = workloads.algorithmic_bytes(sets[0], ws)
            logs = []

            def one_call(i, timed):
                log = {}
                tensors = sets[i % nsets]
                group = _TimedGroup(pg, log) if timed else pg
                bucket = _TimedBucket(buckets[i % nsets], log) if timed else buckets[i % nsets]
                t0 = time.perf_counter()
                work = col.allreduce_quantized(tensors, op, group, stream, prepared=bucket)
                log["returned after"] = time.perf_counter() - t0
                work.wait()
                work.get_future().wait()
                stream.synchronize()
                log["wall"] = time.perf_counter() - t0
                log["t0"] = t0
                return log

            for i in range(W):
                one_call(i, False)
            torch.cuda.synchronize()
            plain = [one_call(i, False)["wall"] for i in range(K)]     # no stopwatch in the way
            logs = [one_call(i, True) for i in range(K)]
            # back to back: K calls queued, then everything waited for
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            works = [col.allreduce_quantized(sets[i % nsets], op, pg, stream, prepared=buckets[i % nsets])
                     for i in range(K)]
            queued = time.perf_counter() - t0
            for w in works:
                w.wait()
                w.get_future().wait()
            stream.synchronize()
            back_to_back = (time.perf_counter() - t0) / K
            if r != 0:
                return
            us = lambda x: round(x * 1e6, 1)  # noqa: E731
            mean = lambda xs: sum(xs) / len(xs)  # noqa: E731
            host = {}
            for key in ("bucket.matches()", "quantize launch", "all-to-all call", "all-to-all wait()", "reduce launch",
                        "all-gather call", "all-gather wait()", "returned after", "all-gather future done after",
                        "dequantize launch"):
                vals = [l[key] for l in logs if key in l]
                if vals:
                    host[key + " us"] = us(mean(vals))
            host["dequantize queued after the call started us"] = us(mean([l["dequantize at"] - l["t0"] for l in logs]))
            gpu = {}
            for name in ("quantize", "all-to-all", "reduce", "all-gather", "dequantize"):
                vals = [l["events"][name][0].elapsed_time(l["events"][name][1]) * 1e-3 for l in logs if name in l.get("events", {})]
                if vals:
                    gpu[name + " us"] = us(mean(vals))
            first_to_last = [l["events"]["quantize"][0].elapsed_time(l["events"]["dequantize"][1]) * 1e-3 for l in logs]
            # the receive buffer (collectives.py:367 allocates it on every call)
            t = time.perf_counter()
            for _ in range(200):
                buf = torch.empty(buckets[0].output_size, dtype=torch.uint8, device=dev)
            alloc = (time.perf_counter() - t) / 200
            del buf
            # the three kernels alone, queued back to back (no idle GPU between the events)
            alone = {}
            b0 = buckets[0]
            packed0 = b0.quantize()
            for name, fn in (("quantize", lambda: b0.quantize(out=packed0)),
                             ("reduce", lambda: b0.reduce(packed0, pg.rank(), op)),
                             ("dequantize", lambda: b0.dequantize(packed0))):
                pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(K)]
                with torch.cuda.stream(stream):
                    for _ in range(W):
                        fn()
                    for a, b in pairs:
                        a.record(stream)
                        fn()
                        b.record(stream)
                stream.synchronize()
                alone[name + " us"] = us(mean([a.elapsed_time(b) * 1e-3 for a, b in pairs]))
            result.update({
                "ranks": ws,
                "wall_us_per_call": us(mean(plain)),
                "wall_us_per_call_with_stopwatch": us(mean([l["wall"] for l in logs])),
                "back_to_back_us_per_call": us(back_to_back),
                "host_us_to_queue_one_call_back_to_back": us(queued / K),
                "kernels_alone_us": alone,
                "kernels_alone_sum_us": round(sum(alone.values()), 1),
                "gpu_us_first_kernel_to_last_with_stopwatch": us(mean(first_to_last)),
                "gpu_us_between_events_with_stopwatch": gpu,
                "host_us_with_stopwatch": host,
                "receive_buffer_allocation_us": us(alloc),
                "algorithmic_bytes": sum(ab.values()),
                "note": "wall_us_per_call: call, work.wait(), future.wait(), stream.synchronize(), one call after the "
                        "other; back_to_back: K calls queued, then all waited for; the stopwatch pass wraps the group "
                        "and the bucket (host timers, device events) and is slower for it; device events around a "
                        "launch on an idle GPU include the launch latency",
            })

        if rank_threads == 1:
            rank_fn(0)
        else:
            errors = []

            def body(r):
                try:
                    rank_fn(r)
                except BaseException as e:  # noqa: BLE001
                    errors.append(e)
                    group.barrier.abort()

            threads = [threading.Thread(target=body, args=(r,)) for r in range(rank_threads)]
            for t in threads:
                t.start()
            for t in threads:
                t.join()
            if errors:
                raise errors[0]
        return result

    out = {}
    if dist.is_nccl_available():
        with socket.socket() as sock:
            sock.bind(("127.0.0.1", 0))
            port = sock.getsockname()[1]
        # RCCL prints a banner on standard output when it creates its communicator: this command's
        # standard output is one line of JSON, so the descriptor points at standard error meanwhile
        sys.stdout.flush()
        saved = os.dup(1)
        os.dup2(2, 1)
        try:
            dist.init_process_group("nccl", init_method=f"tcp://127.0.0.1:{port}", rank=0, world_size=1,
                                    device_id=torch.device("cuda:0"))
            try:
                pg = dist.distributed_c10d._get_default_group()
                out["RCCL process group, this process its only rank"] = measure(lambda r: pg, 1, 1)
            finally:
                dist.destroy_process_group()
        finally:
            sys.stdout.flush()
            os.dup2(saved, 1)
            os.close(saved)
    group = sim_pg.SimGroup(8)
    out["8 ranks simulated by threads on the one GPU (rank 0's figures; the GPU serves all 8)"] = \
        measure(group.rank, 8, 8)
    print(json.dumps({"metric": "allreduce_quantized end to end on 1 MI355X: wall time per call against its kernels",
                      "unit": "us", "n_gpus": 1, "steps": K, "warmup": W,
                      "config": {"workload": workload_name, "api": "collective", "buffer_sets": nsets},
                      "groups": out}))
    return 0


def run_ceiling4(args, sets, ws, rank, op, ab) -> int:
    """The accesses of reduce on configuration 4 and nothing else (k_reduce_pattern_mix of
    torchft_amd/csrc/tftq_ceiling.hip: 4 slots, 103 296 rows of 2052 bytes handled by a wavefront
    each and 11 264 rows of 5636 bytes handled by a workgroup each, in place, work handed to the
    XCDs in chunks of 64 workgroups), a plain 4 : 1 copy of the same bytes, and the product's
    reduce on configuration 4: every kernel alone in a loop that rotates over the buffer sets,
    HIP events around each launch."""
    import ctypes

    import torch

    from torchft_amd import _build, quantization as q

    if not os.path.exists(_build.CEILING_LIB_PATH):
        _build.build_library()
    C = ctypes.CDLL(_build.CEILING_LIB_PATH)
    C.tftq_ceiling_reduce_mix.argtypes = [ctypes.c_void_p, ctypes.c_int64] + [ctypes.c_int] * 4 + [
        ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.c_void_p]
    C.tftq_ceiling_launch.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64,
                                      ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                      ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    stream = torch.cuda.current_stream()
    sp = ctypes.c_void_p(stream.cuda_stream)
    ev = lambda: torch.cuda.Event(enable_timing=True)  # noqa: E731

    def timed(launch, nbytes):
        pairs = [(ev(), ev()) for _ in range(args.steps)]
        torch.cuda.synchronize()
        for i in range(args.warmup):  # the timed launches are queued behind these: no idle GPU in between
            launch(i)
        for i, (a, b) in enumerate(pairs):
            a.record(stream)
            launch(i)
            b.record(stream)
        torch.cuda.synchronize()
        us = sorted(a.elapsed_time(b) * 1e3 for a, b in pairs)
        mean = sum(us) / len(us)
        return {"us": round(mean, 2), "us_min": round(us[0], 2), "us_median": round(us[len(us) // 2], 2), "bytes": nbytes,
                "GBs": round(nbytes / mean / 1e3, 1), "frac_of_peak": round(nbytes / mean / 1e3 / HBM_PEAK_GBS, 4)}

    out = {}
    # the pattern kernels overwrite the own slot with bytes that are no scales and codes: they
    # run on copies of the received buffers
    scratch = [s_["recv"].clone() for s_ in sets]
    rows_a, rb_a, rows_b, rb_b = 103296, 2052, 11264, 5636  # rows per slot of the two row lengths
    slot = sets[0]["recv"].numel() // ws
    assert rows_a * rb_a + rows_b * rb_b <= slot
    nbytes = (ws + 1) * (rows_a * rb_a + rows_b * rb_b)
    for nts in (0, 1):
        def launch(i, nts=nts):
            rc = C.tftq_ceiling_reduce_mix(scratch[i % len(sets)].data_ptr(), slot, ws, rank, rows_a, rb_a,
                                           rows_b * rb_b, rows_b, rb_b, 0, 6, 1, nts, sp)
            assert rc == 0, rc
        out["reduce's accesses, " + ("streaming" if nts else "plain") + " stores"] = timed(launch, nbytes)
    # a plain 4 : 1 copy of about the same bytes: 33 623 chunks of 32 KB read, 8 KB written
    units = nbytes // (5 * 8192)
    for nts in (0, 1):
        def launch(i, nts=nts):
            a, b = scratch[i % len(sets)], sets[i % len(sets)]["gathered"]
            rc = C.tftq_ceiling_launch(4, a.data_ptr(), b.data_ptr(), units, 0, 0, 0, 0, 1, nts, sp)
            assert rc == 0, rc
        out["4:1 copy, streaming loads, " + ("streaming" if nts else "plain") + " stores"] = timed(launch, units * 5 * 8192)
    del scratch
    # (last: by now the threads of the CPU checker that the parity gate ran have gone to sleep, and
    # the host queues its launches ahead of the GPU)
    out["product reduce"] = timed(lambda i: q.fused_reduce_fp8(sets[i % len(sets)]["tensors"], sets[i % len(sets)]["recv"],
                                                              ws, rank, op), ab["reduce"])
    best = max(v["GBs"] for k, v in out.items() if k.startswith("reduce's accesses"))
    out["product reduce"]["of_own_accesses"] = round(out["product reduce"]["GBs"] / best, 4)
    print(json.dumps({"metric": "reduce on configuration 4: the product kernel and kernels that only make its accesses, "
                                "each alone, HBM GB/s on 1 MI355X", "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
                      "warmup": args.warmup,
                      "config": {"workload": f"configuration 4 (ws=4, slot of {slot} bytes); {len(sets)} rotating buffer sets"},
                      "kernels": out}))
    return 0


def main() -> int:
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the quantized-collective kernels run on one GPU's share "
              "and this build has no cross-GPU path; run with --gpus 1", file=sys.stderr)
        return 2
    if args.config == "ceiling":
        import torch
        from torchft_amd import _lib
        if not torch.cuda.is_available() or _lib.load().tftq_check_device(0) != 0:
            print("bench.py needs a gfx950 GPU", file=sys.stderr)
            return 2
        return run_ceilings(args)

    import torch
    from torch.distributed import ReduceOp

    import workloads
    from torchft_amd import _lib, quantization as q

    if not torch.cuda.is_available():
        print("bench.py needs a gfx950 GPU", file=sys.stderr)
        return 2
    torch.cuda.set_device(0)
    rc = _lib.load().tftq_check_device(0)
    if rc != 0:
        print("bench.py: " + _lib.strerror(rc), file=sys.stderr)
        return 2

    dev = "cuda"
    cfg5_shapes = workloads.cfg5_shapes(10000) if args.config == "5" else None
    table = {
        "2": (lambda seed: workloads.cfg2(seed, device=dev), 8, ReduceOp.AVG,
              "config 2: one bf16 tensor [4096, 4096], N(0, 0.02), ws=8, AVG"),
        "3": (lambda seed: workloads.cfg3(seed, device=dev), 8, ReduceOp.AVG,
              "benchmark configuration 3: Llama-3-8B decoder-layer gradient bucket, "
              "9 bf16 tensors, 218112000 elements, ws=8, reduce AVG"),
        "4": (lambda seed: workloads.cfg4(seed, device=dev), 4, ReduceOp.AVG,
              "config 4: DiLoCo pseudo-gradient of a 1.1B model, 201 fp32 tensors, "
              "1100048384 elements, Student-t(3) x 1e-4, ws=4, AVG"),
        "5": (lambda seed: workloads.cfg5(seed, torch.bfloat16, cfg5_shapes, device=dev), 16,
              ReduceOp.SUM, "config 5: 10000 bf16 tensors of 1..4096 elements, ragged rows, ws=16, SUM"),
        "flat": (lambda seed: [torch.randn(64 * 1024 * 1024, device=dev,
                                           generator=torch.Generator(device=dev).manual_seed(seed))],
                 8, ReduceOp.SUM, "one 1-D fp32 tensor of 67108864 elements (rows of one column), ws=8, SUM"),
    }
    if args.config == "shape":
        shapes = [tuple(int(d) for d in part.split("x")) for part in args.shape.split(",")]
        dt = getattr(torch, args.dtype)

        def make_shape(seed):
            g = torch.Generator(device=dev).manual_seed(seed)
            return [(torch.randn(sh, device=dev, generator=g) * 0.02).to(dt) for sh in shapes]

        table["shape"] = (make_shape, args.ws, ReduceOp.AVG,
                          f"tensors {args.shape} {args.dtype}, N(0, 0.02), ws={args.ws}, AVG")
    table["ceiling4"] = table["4"]
    make, ws, op, workload_name = table[args.config]
    if args.api == "collective":
        if args.config not in ("2", "3", "shape"):
            print("bench.py --api collective runs configurations 2, 3 and shape", file=sys.stderr)
            return 2
        return run_collective(args, make, op, workload_name)
    rank = args.rank if args.rank is not None else min(3, ws - 1)
    if args.config in ("4", "ceiling4"):
        args.sets = min(args.sets, 2)

    # ---- buffer sets: tensors, received buffer B, gathered buffer G ----------
    sets = []
    for k in range(args.sets):
        slots = []
        mine = None
        for peer in range(ws):
            t = make(1000 * k + peer)
            qp = q.fused_quantize_into_fp8(t, ws)
            slot = qp.numel() // ws
            slots.append(qp[rank * slot:(rank + 1) * slot].clone())
            if peer == rank:
                mine = t
            del t, qp
        recv = torch.cat(slots)
        del slots
        gathered = q.fused_quantize_into_fp8(mine, ws)  # any valid packed buffer of this layout
        sets.append({"tensors": mine, "recv": recv, "gathered": gathered})
        if args.api == "prepared":
            sets[-1]["bucket"] = q.prepare(mine, ws)
            sets[-1]["out"] = torch.empty_like(gathered)
    torch.cuda.synchronize()
    ab = workloads.algorithmic_bytes(sets[0]["tensors"], ws)

    # ---- parity gate on the data that is being timed -------------------------
    from oracle import oracle
    # a mid-sized tensor of the first set (config 3: the k_proj gradient [1024, 4096])
    cand = sets[0]["tensors"]
    probe = [cand[1] if len(cand) > 1 else cand[0][: min(cand[0].shape[0], 2048)]]
    probe_cpu = [probe[0].cpu()]
    qg = q.fused_quantize_into_fp8(probe, ws)
    qc = oracle.fused_quantize_into_fp8(list(probe_cpu), ws)
    ok = torch.equal(qg.cpu(), qc)
    rg, rcpu = qg.clone(), qc.clone()
    q.fused_reduce_fp8(probe, rg, ws, rank, op)
    oracle.fused_reduce_fp8(list(probe_cpu), rcpu, ws, rank, op)
    ok = ok and torch.equal(rg.cpu(), rcpu)
    dg, dc = [torch.empty_like(probe[0])], [torch.empty_like(probe_cpu[0])]
    q.fused_dequantize_from_fp8(dg, qg, ws)
    oracle.fused_dequantize_from_fp8(dc, qc, ws)
    ok = ok and torch.equal(dg[0].cpu().reshape(-1).view(torch.uint8), dc[0].reshape(-1).view(torch.uint8))
    if not ok:
        print("bench.py: GPU results differ from the CPU checker", file=sys.stderr)
        return 1

    if args.config == "ceiling4":
        return run_ceiling4(args, sets, ws, rank, op, ab)

    ev = lambda: torch.cuda.Event(enable_timing=True)  # noqa: E731
    STAGES = ("quantize", "reduce", "dequantize")

    def step(i, events=None, only=None):
        # the public drop-in functions, exactly as torchft/collectives.py calls them;
        # events[k] / events[k + 1] bracket stage k (all stages, or stage `only`)
        s = sets[i % len(sets)]
        stream = torch.cuda.current_stream()

        def mark(k):
            if events is not None and (only is None or k in (only, only + 1)):
                events[k].record(stream)

        if args.api == "prepared":
            b = s["bucket"]
            mark(0)
            packed = b.quantize(out=s["out"])
            mark(1)
            b.reduce(s["recv"], rank, op)
            mark(2)
            b.dequantize(s["gathered"])
            mark(3)
            return packed
        mark(0)
        # The result stays alive until this buffer set has its next turn, so that the allocator
        # cannot hand the same block to every step: a packed buffer that is rewritten every
        # ~0.3 ms stays in the 256 MB last-level cache and flatters quantize by 20 us, which no
        # training step would see (a whole step lies between two all-reduces of a bucket).
        packed = s["packed"] = q.fused_quantize_into_fp8(s["tensors"], ws)
        mark(1)
        q.fused_reduce_fp8(s["tensors"], s["recv"], ws, rank, op)
        mark(2)
        q.fused_dequantize_from_fp8(s["tensors"], s["gathered"], ws)
        mark(3)
        return packed

    def stage_means(all_events, which):
        return {STAGES[k]: sum(e[k].elapsed_time(e[k + 1]) for e in all_events) / len(all_events)
                for k in which}

    if args.copy_calibration:
        src = torch.empty(64 * 1024 * 1024, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)  # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst

    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()

    # Which stage takes longest: eight untimed steps with events around every stage.
    probe_events = [[ev() for _ in range(4)] for _ in range(8)]
    for i in range(8):
        step(i, probe_events[i])
    torch.cuda.synchronize()
    probe_ms = stage_means(probe_events, range(3))
    dominant = max(probe_ms, key=lambda k: probe_ms[k])
    dom = STAGES.index(dominant)

    # The timed region: K steps, events only around the dominant kernel (every event record
    # costs ~3 us of dispatch gap: 4 records per step made the step 12 us longer).
    # The pair is recorded on every fourth step: a pair costs the step about 5 us.
    stride = 4 if args.steps >= 8 else 1
    all_events = [[ev() for _ in range(4)] for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        if i % stride == 0:
            step(i, all_events[i], only=dom)
        else:
            step(i)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    dominant_ms = stage_means(all_events[::stride], [dom])[dominant]

    # What a pair of event records reads with no kernel between them, on a busy stream: the
    # part of every event-bracketed duration that is not the kernel.
    gap_events = [(ev(), ev()) for _ in range(args.steps)]
    stream = torch.cuda.current_stream()
    for i in range(args.steps):
        step(i)
        gap_events[i][0].record(stream)
        gap_events[i][1].record(stream)
    torch.cuda.synchronize()
    pair_readings = sorted(a.elapsed_time(b) for a, b in gap_events)
    # the median, and never more than a tenth of the kernel it is taken off: one slow reading
    # must not flatter the corrected figure
    event_pair_ms = min(max(pair_readings[len(pair_readings) // 2], 0.0), 0.1 * dominant_ms)

    # Per-stage breakdown: the same K steps once more with events around every stage
    # (not part of the timed region).
    all_events = [[ev() for _ in range(4)] for _ in range(args.steps)]
    for i in range(args.steps):
        step(i, all_events[i])
    torch.cuda.synchronize()
    stage_ms = stage_means(all_events, range(3))

    # Every stage alone: K launches of the one kernel, rotating over the buffer sets, events
    # around each launch (not part of the timed region).  In a quantized all-reduce the kernels
    # never run back to back (collectives lie between them, torchft/collectives.py:364-412); in the
    # step above a kernel also pays for the write-back of what the one before it left in the
    # caches, here it does not.
    def alone(k, i):
        s = sets[i % len(sets)]
        if k == 0:
            s["packed"] = q.fused_quantize_into_fp8(s["tensors"], ws)  # kept: see step()
        elif k == 1:
            q.fused_reduce_fp8(s["tensors"], s["recv"], ws, rank, op)
        else:
            q.fused_dequantize_from_fp8(s["tensors"], s["gathered"], ws)

    alone_ms = {}
    stream = torch.cuda.current_stream()
    for k in range(3):
        for i in range(args.warmup):
            alone(k, i)
        pairs = [(ev(), ev()) for _ in range(args.steps)]
        for i, (a, b) in enumerate(pairs):
            a.record(stream)
            alone(k, i)
            b.record(stream)
        torch.cuda.synchronize()
        alone_ms[STAGES[k]] = sum(a.elapsed_time(b) for a, b in pairs) / len(pairs)

    total_bytes = sum(ab.values())
    value = total_bytes / (ms_per_step * 1e-3) / 1e9

    stages = {}
    for k in stage_ms:
        gbs = ab[k] / (stage_ms[k] * 1e-3) / 1e9
        stages[k] = {"us": round(stage_ms[k] * 1e3, 2), "bytes": ab[k], "GBs": round(gbs, 1),
                     "frac": round(gbs / HBM_PEAK_GBS, 4)}
    stages["note"] = ("separate pass with events around every stage (every figure holds about event_pair_us, see roofline, "
                       "that is not the kernel); the timed region has events around the dominant kernel only")
    stages_alone = {}
    for k in alone_ms:
        gbs = ab[k] / (alone_ms[k] * 1e-3) / 1e9
        stages_alone[k] = {"us": round(alone_ms[k] * 1e3, 2), "GBs": round(gbs, 1), "frac": round(gbs / HBM_PEAK_GBS, 4)}
    stages_alone["note"] = ("each kernel alone in a loop over the buffer sets, events around every launch "
                            "(an event pair adds 2-3 us to the kernel's own duration)")

    # The roofline entry is for the kernel that takes the largest share of the step: HIP events
    # around its launches inside the timed region (they include the gap to the kernel before it).
    # `traffic` is not measured by this run: HBM bytes per launch on the headline workload from
    # rocprofv3 --pmc FETCH_SIZE (x2.000, calibrated on a 256 MiB copy) + WRITE_SIZE (x1.000), as
    # recorded in profiles/cfg3_bf16_ws8_hbm_traffic.md.
    profiled_traffic = PROFILED_TRAFFIC if args.config == "3" else {}
    profiled_us = PROFILED_KERNEL_US if args.config == "3" else {}
    # `us`, `achieved` and `frac` are what the events around the kernel read.  That reading holds
    # what two event records with no kernel between them read on the same busy stream (5 us on
    # MI355X); `us_less_event_pair` and `frac_less_event_pair` take it off, and agree with
    # rocprofv3's kernel-trace duration of the same launches to 1 %.
    achieved = ab[dominant] / (dominant_ms * 1e-3) / 1e9
    kernel_ms = dominant_ms - event_pair_ms
    roofline = {"bound": "hbm", "kernel": "k_" + dominant, "achieved": round(achieved, 1),
                "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                "us": round(dominant_ms * 1e3, 2),
                "event_pair_us": round(event_pair_ms * 1e3, 2),
                "us_less_event_pair": round(kernel_ms * 1e3, 2),
                "frac_less_event_pair": round(ab[dominant] / (kernel_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                "kernel_trace_us": profiled_us.get(dominant),
                "timing": "HIP events around the kernel on every fourth of the timed quantize -> reduce -> "
                          "dequantize steps (us); event_pair_us: the median of what two records with nothing "
                          "between them read on the same stream; kernel_trace_us: the kernel's mean duration in "
                          "the step by rocprofv3 --kernel-trace (profiles/cfg3_bf16_ws8_kernel_trace.md, not this run)",
                "alone": stages_alone[dominant],
                "traffic": profiled_traffic.get(dominant),
                "traffic_source": "profiles/cfg3_bf16_ws8_hbm_traffic.md (rocprofv3 --pmc, not this run)"
                                  if profiled_traffic else None}

    out = {
        "metric": "quantize+reduce+dequant HBM GB/s on 1 MI355X",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": f"{workload_name}, rank {rank}; {len(sets)} rotating buffer sets "
                               "(cold last-level cache)",
                   "api": args.api,
                   "input_dtype": str(sets[0]["tensors"][0].dtype).replace("torch.", ""),
                   "packed_bytes": int(sets[0]["gathered"].numel()),
                   "algorithmic_bytes_per_step": total_bytes},
        "roofline": roofline,
        "stages": stages,
        "stages_alone": stages_alone,
        "parity": "quantize, reduce, dequantize byte-identical to the CPU checker on the probe tensor",
    }
    if not args.no_cpu_baseline and args.config == "3":
        out["cpu_baseline"] = cpu_baseline(args.cpu_rows)
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
