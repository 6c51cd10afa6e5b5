#!/usr/bin/env python3
"""Benchmark of the combine hot path on one MI355X.

A step is one pass of alamd_combine over one batch of synthetic input that is
already resident in HBM: P = 8 logical-rank buffers folded into one output.
Prints ONE JSON line (see the keys below).  The kernel's own duration is
measured with events on the stream the kernel runs on; the CPU baseline is the
reference's MPI-backend host combine (a direct MPI_Allreduce, 4 ranks) timed
on this box's host cores in the same run.
"""
import argparse
import json
import os
import subprocess
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "combine HBM GB/s (% of 8 TB/s peak), P=8 fp32/bf16 sum, 2 GiB buffers"
HBM_PEAK_GBPS = 8000.0

WORKLOADS = {
    # name: (dtype, count per rank, op, dist, seed base, order[, buffer sets[, (elements the inputs, the
    # output start into their allocations)]])
    "c2_f32_sum": ("f32", 1 << 26, "sum", "uniform_pm1", 1000, "rank_asc"),
    "c2_f32_prod": ("f32", 1 << 26, "prod", "uniform_09_11", 1000, "rank_asc"),
    "c2_f32_sum_tree": ("f32", 1 << 26, "sum", "uniform_pm1", 1000, "tree_rsg"),
    "c2_bf16_sum": ("bf16", 1 << 27, "sum", "normal", 2000, "rank_asc"),
    "c4_i32_max": ("i32", 1 << 28, "max", "fullrange", 3000, "rank_asc"),
    "c4_i64_bxor": ("i64", 1 << 28, "bxor", "fullrange", 3000, "rank_asc"),
    "c4_u8_lxor": ("u8", 1 << 28, "lxor", "bool01", 3000, "rank_asc"),
    # size / type probes
    "f32_sum_2p28": ("f32", 1 << 28, "sum", "uniform_pm1", 1000, "rank_asc"),
    "i32_max_2p26": ("i32", 1 << 26, "max", "fullrange", 3000, "rank_asc"),
    "f16_sum": ("f16", 1 << 27, "sum", "normal", 2000, "rank_asc"),
    "i8_sum": ("i8", 1 << 28, "sum", "fullrange", 3000, "rank_asc"),
    "i16_min": ("i16", 1 << 27, "min", "fullrange", 3000, "rank_asc"),
    "f64_sum": ("f64", 1 << 25, "sum", "uniform_pm1", 1000, "rank_asc"),
    # the primary workload over four rotating buffer sets (9 GiB touched per four launches): nothing a
    # launch reads or writes was touched by the three launches before it
    "c2_f32_sum_rotating": ("f32", 1 << 26, "sum", "uniform_pm1", 1000, "rank_asc", 4),
    "c2_bf16_sum_rotating": ("bf16", 1 << 27, "sum", "normal", 2000, "rank_asc", 4),
    # the same with buffers that start off the 1 KiB boundaries the kernels' tiles like: every buffer one
    # element into its allocation; the inputs at the start of theirs and the output five elements in
    "c2_f32_sum_rotating_one_element_in": ("f32", 1 << 26, "sum", "uniform_pm1", 1000, "rank_asc", 4, (1, 1)),
    "c2_f32_sum_rotating_output_five_elements_in": ("f32", 1 << 26, "sum", "uniform_pm1", 1000, "rank_asc", 4, (0, 5)),
    "c2_f32_sum_tree_rotating_one_element_in": ("f32", 1 << 26, "sum", "uniform_pm1", 1000, "tree_rsg", 4, (1, 1)),
}
P = 8

# The committed rocprofv3 summary of the primary workload: HBM bytes per call from --pmc FETCH_SIZE /
# WRITE_SIZE, each scaled by the same counter's reading for the 1 GiB copy kernel.
TRAFFIC_PROFILE = {"c2_f32_sum": "profiles/fold_vec_kernel_f32_sum_P8_c2.md"}
KERNEL_NAME = {"c2_f32_sum": "alamd::fold_vec_kernel<float, 0 /*sum*/, false /*operand roles*/, 2 /*streams requested "
                             "up front*/, false /*no leading elements*/, 0 /*streaming launch*/>"}

# Every configuration of the headline benchmark beside the primary workload: C2 in the tree order, prod and bf16, the same over
# buffers no earlier call has touched, C4 (integer / bitwise / logical), C3 (ring, both modes), C5 (halo
# faces), the stream flags, and the layouts an Allreduce / Reduce_scatter / Allgather reaches the kernels in.
DEFAULT_ALSO = ("c2_sum_rotating_pair,c2_f32_sum_tree,c2_f32_prod,c2_bf16_sum,c4_i32_max,c4_i64_bxor,"
                "c4_u8_lxor,c3_ring_stepwise,c3_ring_fused,c5_halo,flags,c2_f32_allreduce,"
                "c2_f32_allreduce_rotating,c2_f32_reduce_scatter,c2_f32_reduce_scatter_rotating,"
                "c2_f32_allgather,c2_f32_allgather_rotating,c2_f32_reduce_scatterv_in_place")


def measured_traffic(workload):
    """(bytes per call, where the figure comes from) out of the committed profile summary, or (None, why)."""
    import hashlib
    import re
    rel = TRAFFIC_PROFILE.get(workload)
    if not rel:
        return None, "no counter profile committed for this workload"
    try:
        text = open(os.path.join(ROOT, rel)).read()
    except OSError:
        return None, "%s is missing" % rel
    m = re.search(r"=> (\d+) B per launch, (\d+) B per call", text)
    if not m:
        return None, "%s holds no 'B per call' line" % rel
    return int(m.group(2)), "%s (sha1 %s)" % (rel, hashlib.sha1(text.encode()).hexdigest()[:12])


def halo_traffic():
    """((bytes the six-face pack moves, bytes the six-face unpack moves), source) out of the committed counter
    profile of the halo kernel, or (None, why)."""
    import hashlib
    import re
    rel = "profiles/halo_kernel_f64_c5.md"
    try:
        text = open(os.path.join(ROOT, rel)).read()
    except OSError:
        return None, "%s is missing" % rel
    m = re.search(r"Pack:.*?In all (\d+) B", text, re.S)
    n = re.search(r"Unpack:.*?; (\d+) B", text, re.S)
    if not (m and n):
        return None, "%s holds no byte totals" % rel
    return (int(m.group(1)), int(n.group(1))), "%s (sha1 %s)" % (rel, hashlib.sha1(text.encode()).hexdigest()[:12])


def run_pair_workload(al, torch, steps, warmup):
    """C2 as fp32 and as bf16 over the SAME memory: four rotating sets of eight 256 MiB buffers plus an output
    (9 GiB in all, so nothing a call touches was touched by the three calls before it), filled once with
    bf16 normal(0,1) values and read as 2^27 bf16 or as 2^26 fp32 elements, the two taking turns.  Where the
    buffers lie in HBM moves a rate by up to 3 points from one allocation to the next; measured this way the
    difference between the two types is the kernels' alone."""
    import numpy as np
    import oracle
    nbytes = 256 << 20
    raw = []
    for _ in range(4):
        ins = [torch.empty(nbytes // 2, dtype=torch.int16, device="cuda") for _ in range(P)]
        out = torch.empty(nbytes // 2, dtype=torch.int16, device="cuda")
        for r in range(P):
            al.fill(ins[r], "normal", 2000 + r, dtype="bf16")
        raw.append((ins, out))
    views = {"f32": torch.float32, "bf16": torch.int16}
    calls = {dt: [lambda ins=ins, out=out, dt=dt, v=v: al.combine([out.view(v)], [t.view(v) for t in ins], "sum",
                                                                  order="rank_asc", dtype=dt) for ins, out in raw]
             for dt, v in views.items()}
    # parity: both views of the first and last 2^18 bytes of every set against the oracle's fold of the same bytes
    ok, m = True, 1 << 18
    for dt in views:
        np_dt = oracle.NP_CARRIER[dt]
        for k, (ins, out) in enumerate(raw):
            calls[dt][k]()
            torch.cuda.synchronize()
            for lo in (0, nbytes - m):
                host = [t.view(torch.uint8)[lo:lo + m].cpu().numpy().view(np_dt) for t in ins]
                want = oracle.combine(host, dt, "sum", "rank_asc")
                got = out.view(torch.uint8)[lo:lo + m].cpu().numpy().view(np_dt)
                ok = ok and got.tobytes() == want.tobytes()
    alg = (P + 1) * nbytes
    rates = {dt: [] for dt in views}
    turn = {dt: 0 for dt in views}
    for _ in range(5):
        for dt in views:
            def step(dt=dt):
                calls[dt][turn[dt] % 4]()
                turn[dt] += 1
            _, kms = timed(torch, step, steps, max(4, warmup))
            rates[dt].append(alg / (kms * 1e-3) * 1e-9)
    med = {dt: sorted(r)[len(r) // 2] for dt, r in rates.items()}
    diffs = sorted(b - a for a, b in zip(rates["f32"], rates["bf16"]))
    return {"workload": "c2_sum_rotating_pair", "P": P, "bytes_per_buffer": nbytes, "buffer_sets": 4, "op": "sum",
            "order": "rank_asc", "algorithmic_bytes": alg, "rounds": 5,
            "gbps_kernel_f32": med["f32"], "gbps_kernel_bf16": med["bf16"],
            "frac_f32": med["f32"] / HBM_PEAK_GBPS, "frac_bf16": med["bf16"] / HBM_PEAK_GBPS,
            "bf16_minus_f32_gbps_median_of_paired": diffs[len(diffs) // 2], "parity_vs_oracle": bool(ok)}


def run_halo_policy_workload(al, torch, steps, warmup):
    """The pack of both x faces, and of all six faces, of the C5 grid with the grid loads under each cache
    policy the library can be set to (a measurement: see alamd_tune, halo_load_policy)."""
    import ctypes as C
    n, h = 512, 2
    dims, side = (n, n, n), n + 2 * h
    grid = torch.empty(side ** 3, dtype=torch.float64, device="cuda")
    al.fill(grid, "uniform_01", 4000)
    bufs = {f: torch.empty(al.halo_face_elems(dims, h, f), dtype=torch.float64, device="cuda") for f in range(6)}
    L = al.load()
    tab = (C.c_void_p * 6)(*[bufs[f].data_ptr() for f in range(6)])
    cdims = (C.c_size_t * 3)(*dims)
    gp = C.c_void_p(grid.data_ptr())
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)

    def pack(mask):
        assert L.alamd_halo_pack(tab, gp, cdims, h, 8, mask, st) == 0

    pack(0x3f)
    torch.cuda.synchronize()
    ref = {f: bufs[f].clone() for f in range(6)}
    names = ["plain", "nt", "sc1", "sc0 sc1", "sc0 sc1 nt"]
    res = {"workload": "c5_halo_load_policy", "dtype": "f64", "policies": {}}
    try:
        for lp, name in enumerate(names):
            al.tune("halo_load_policy", lp)
            _, kx = timed(torch, lambda: pack(3), steps, warmup)
            _, ka = timed(torch, lambda: pack(0x3f), steps, warmup)
            for f in range(6):
                bufs[f].zero_()
            pack(0x3f)
            torch.cuda.synchronize()
            res["policies"][name] = {"pack_x_pair_us": kx * 1e3, "pack_all_us": ka * 1e3,
                                     "same_bytes_as_plain": all(bool(torch.equal(bufs[f], ref[f])) for f in range(6))}
    finally:
        al.tune("halo_load_policy", 0)
    return res


def run_combine_workload(al, torch, name, steps, warmup, check=True):
    dtype, count, op, dist, seed, order = WORKLOADS[name][:6]
    nsets = WORKLOADS[name][6] if len(WORKLOADS[name]) > 6 else 1
    in_off, out_off = WORKLOADS[name][7] if len(WORKLOADS[name]) > 7 else (0, 0)
    es = al.dtype_size(dtype)
    carrier = al.torch_dtype(dtype)
    sets = []
    for _ in range(nsets):
        ins = [torch.empty(count + in_off, dtype=carrier, device="cuda")[in_off:] for _ in range(P)]
        out = torch.empty(count + out_off, dtype=carrier, device="cuda")[out_off:]
        for r in range(P):
            al.fill(ins[r], dist, seed + r, dtype=dtype)
        sets.append((ins, out))
    torch.cuda.synchronize()
    for i in range(warmup):
        ins, out = sets[i % nsets]
        al.combine([out], ins, op, order=order, dtype=dtype)
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()
    for i in range(steps):
        ins, out = sets[i % nsets]
        al.combine([out], ins, op, order=order, dtype=dtype)
    ev1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    kernel_ms = ev0.elapsed_time(ev1) / steps
    alg_bytes = (P + 1) * count * es
    res = {
        "workload": name, "dtype": dtype, "op": op, "order": order, "P": P, "count": count,
        "buffer_sets": nsets, "elements_into_allocation": {"inputs": in_off, "output": out_off}, "launches_per_step": al.planned_launches(P, count, dtype),
        "algorithmic_bytes": alg_bytes, "ms_per_step": wall * 1e3 / steps, "kernel_ms": kernel_ms,
        "gbps_wall": alg_bytes / (wall / steps) * 1e-9, "gbps_kernel": alg_bytes / (kernel_ms * 1e-3) * 1e-9,
    }
    if check:
        # parity spot-check against the CPU oracle on the first and last 2^18 elements
        import numpy as np
        import oracle
        m = 1 << 18
        np_dt = oracle.NP_CARRIER[dtype]
        ok = True
        for _, out in sets:
            for lo in (0, count - m):
                want = oracle.combine_generated(P, m, dtype, op, order, 0, dist, seed, lo)
                got = out[lo:lo + m].cpu().numpy().view(np_dt)
                ok = ok and got.tobytes() == want.tobytes()
        res["parity_vs_oracle"] = bool(ok)
    del sets, ins, out
    torch.cuda.empty_cache()
    return res


def timed(torch, fn, steps, warmup):
    """Runs fn `warmup` + `steps` times on torch's current stream; returns (wall s/step, kernel ms/step)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()
    for _ in range(steps):
        fn()
    ev1.record()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps, ev0.elapsed_time(ev1) / steps


def run_ring_workload(al, torch, mode, steps, warmup):
    """C3: ring reduce-scatter + allgather over P=8 logical ranks, bf16, 2^27 elements per rank,
    normal(0,1) seed 2000+rank, 4 MiB chunks, in place."""
    import numpy as np
    import oracle
    dtype, count, chunk = "bf16", 1 << 27, 4 << 20
    bufs = [torch.empty(count, dtype=torch.int16, device="cuda") for _ in range(P)]

    def refill():
        for r in range(P):
            al.fill(bufs[r], "normal", 2000 + r, dtype=dtype)

    refill()
    al.ring_allreduce(bufs, "sum", chunk_bytes=chunk, mode=mode, dtype=dtype)
    torch.cuda.synchronize()
    ok, m = True, 1 << 16
    for s in (0, 3, 7):  # segment s is the ring-order fold starting at rank s
        off, ln = al.capi.ring_segment(count, P, s)
        want = oracle.combine_generated(P, m, dtype, "sum", "ring", s, "normal", 2000, off + ln - m)
        for r in (0, 5):
            got = bufs[r][off + ln - m:off + ln].cpu().numpy().view(np.uint16)
            ok = ok and got.tobytes() == want.tobytes()
    refill()
    wall, kms = timed(torch, lambda: al.ring_allreduce(bufs, "sum", chunk_bytes=chunk, mode=mode, dtype=dtype),
                      steps, warmup)
    es = 2
    # stepwise: each of the P-1 reduce-scatter steps reads two segments and writes one per rank, each of the
    # P-1 allgather steps reads one and writes one; fused: every buffer is read once and written once
    alg = 5 * (P - 1) * count * es if mode == "stepwise" else 2 * P * count * es
    return {"workload": "c3_ring_" + mode, "dtype": dtype, "op": "sum", "P": P, "count": count,
            "chunk_bytes": chunk, "algorithmic_bytes": alg, "ms_per_step": wall * 1e3, "kernel_ms": kms,
            "gbps_wall": alg / wall * 1e-9, "gbps_kernel": alg / (kms * 1e-3) * 1e-9,
            "parity_vs_oracle": bool(ok)}


LAYOUTS = [w + r for w in ("c2_f32_allreduce", "c2_f32_allgather", "c2_f32_reduce_scatter") for r in ("", "_rotating")]
LAYOUTS.append("c2_f32_reduce_scatterv_in_place")


def run_layout_workload(al, torch, name, steps, warmup):
    """The two write-heavy layouts at the C2 shape (P = 8 fp32 ranks, seed 1000+rank):
    c2_f32_allreduce - the combine delivered to all eight ranks' receive buffers (8 reads + 8 writes of
    2^26 elements, order tree_rsg: what Al::Allreduce yields above 2 KiB);
    c2_f32_allgather - eight slices of 2^23 elements gathered into eight receive buffers of 2^26
    (each slice read once, written eight times);
    c2_f32_reduce_scatter - eight send buffers of 2^26 elements, block b folded into receive buffer b of
    2^23 elements (order pairwise_desc from the receiving rank: what MPI_Reduce_scatter_block yields above
    512 KiB).
    c2_f32_reduce_scatterv_in_place - eight buffers of 2^26 elements, counts (1, 2^26 - 1, 0, ...), in place:
    rank 1's block of 2^26 - 1 elements is read one element behind where its result is written, the worst
    case of the chained launch (every tile waits for its neighbour's loads).
    With the suffix _rotating the calls go round four sets of buffers, so that nothing a call reads or
    writes was touched by the three calls before it (no help from the 256 MiB memory-side cache)."""
    import oracle
    m = 1 << 18
    rotating = name.endswith("_rotating")
    base = name[:-len("_rotating")] if rotating else name
    fns, ok = [], True
    for s in range(4 if rotating else 1):
        if base == "c2_f32_allreduce":
            count = 1 << 26
            ins = [torch.empty(count, dtype=torch.float32, device="cuda") for _ in range(P)]
            outs = [torch.empty(count, dtype=torch.float32, device="cuda") for _ in range(P)]
            for r in range(P):
                al.fill(ins[r], "uniform_pm1", 1000 + r)
            fn = lambda ins=ins, outs=outs: al.combine(outs, ins, "sum", order="tree_rsg")
            alg = 2 * P * count * 4
            fn()
            torch.cuda.synchronize()
            for j in (0, P - 1):
                for lo in (0, count - m):
                    # (for a sum the reduce-scatter + gather order gives the bits of the doubling tree
                    # wherever the element lies, so a slice can be checked on its own)
                    want = oracle.combine_generated(P, m, "f32", "sum", "tree_dbl", 0, "uniform_pm1", 1000, lo)
                    ok = ok and outs[j][lo:lo + m].cpu().numpy().tobytes() == want.tobytes()
        elif base == "c2_f32_reduce_scatter":
            count = 1 << 23
            sends = [torch.empty(P * count, dtype=torch.float32, device="cuda") for _ in range(P)]
            recvs = [torch.empty(count, dtype=torch.float32, device="cuda") for _ in range(P)]
            for r in range(P):
                al.fill(sends[r], "uniform_pm1", 1000 + r)
            fn = lambda sends=sends, recvs=recvs: al.reduce_scatter(recvs, sends, "sum", order="pairwise_desc",
                                                                    count=count)
            alg = (P + 1) * P * count * 4
            fn()
            torch.cuda.synchronize()
            for b in (0, P - 1):
                for lo in (0, count - m):
                    want = oracle.combine_generated(P, m, "f32", "sum", "pairwise_desc", b, "uniform_pm1", 1000,
                                                    b * count + lo)
                    ok = ok and recvs[b][lo:lo + m].cpu().numpy().tobytes() == want.tobytes()
        elif base == "c2_f32_allgather":
            count = 1 << 23
            sends = [torch.empty(count, dtype=torch.float32, device="cuda") for _ in range(P)]
            recvs = [torch.empty(P * count, dtype=torch.float32, device="cuda") for _ in range(P)]
            for r in range(P):
                al.fill(sends[r], "uniform_pm1", 1000 + r)
            fn = lambda sends=sends, recvs=recvs: al.allgather(recvs, sends, count=count)
            alg = (P + P * P) * count * 4
            fn()
            torch.cuda.synchronize()
            for j in (0, P - 1):
                for q in (0, P - 1):
                    want = oracle.fill(m, "f32", "uniform_pm1", 1000 + q, count - m)
                    got = recvs[j][(q + 1) * count - m:(q + 1) * count].cpu().numpy()
                    ok = ok and got.tobytes() == want.tobytes()
        elif base == "c2_f32_reduce_scatterv_in_place":
            count = 1 << 26
            counts = [1, count - 1] + [0] * (P - 2)
            bufs = [torch.empty(count, dtype=torch.float32, device="cuda") for _ in range(P)]
            for r in range(P):
                al.fill(bufs[r], "uniform_pm1", 1000 + r)
            fn = lambda bufs=bufs, counts=counts: al.reduce_scatterv(bufs, bufs, counts, "sum",
                                                                     order="pairwise_desc", dtype="f32")
            alg = (P + 1) * count * 4
            fn()  # later calls fold what this one left: the same traffic, other values
            torch.cuda.synchronize()
            for lo in (0, count - 1 - m):
                want = oracle.combine_generated(P, m, "f32", "sum", "pairwise_desc", 1, "uniform_pm1", 1000, 1 + lo)
                ok = ok and bufs[1][lo:lo + m].cpu().numpy().tobytes() == want.tobytes()
        else:
            raise SystemExit("unknown workload %s" % name)
        fns.append(fn)
    turn = [0]

    def step():
        fns[turn[0] % len(fns)]()
        turn[0] += 1
    wall, kms = timed(torch, step, steps, warmup)
    return {"workload": name, "dtype": "f32", "op": "sum", "P": P, "count": count,
            "buffer_sets": len(fns), "algorithmic_bytes": alg, "ms_per_step": wall * 1e3, "kernel_ms": kms,
            "gbps_wall": alg / wall * 1e-9, "gbps_kernel": alg / (kms * 1e-3) * 1e-9, "parity_vs_oracle": bool(ok)}


def run_halo_workload(al, torch, steps, warmup):
    """C5: fp64 grid, interior 512^3, halo 2 (allocation 516^3, x fastest), uniform[0,1) seed 4000;
    pack the six faces, loop them back, unpack into the ghost cells."""
    import numpy as np
    import oracle
    n, h = 512, 2
    dims, side = (n, n, n), n + 2 * h
    grid = torch.empty(side ** 3, dtype=torch.float64, device="cuda")
    al.fill(grid, "uniform_01", 4000)
    bufs = {f: torch.empty(al.halo_face_elems(dims, h, f), dtype=torch.float64, device="cuda") for f in range(6)}
    al.halo_pack(bufs, grid, dims, h)
    al.halo_unpack(grid, bufs, dims, h)
    torch.cuda.synchronize()
    # parity on the host for the whole grid (1 GiB): oracle pack / unpack of the same generated grid
    host = oracle.fill(side ** 3, "f64", "uniform_01", 4000)
    ok = True
    for f in range(6):
        want = oracle.halo_pack(host, n, n, n, h, f)
        ok = ok and bufs[f].cpu().numpy().tobytes() == want.tobytes()
    for f in range(6):
        host = oracle.halo_unpack(host, oracle.halo_pack(host, n, n, n, h, f), n, n, n, h, f)
    ok = ok and grid.cpu().numpy().tobytes() == host.tobytes()
    face_bytes = bufs[0].numel() * 8
    res = {"workload": "c5_halo", "dtype": "f64", "grid": [side] * 3, "halo": h, "face_bytes": face_bytes,
           "parity_vs_oracle": bool(ok)}
    # the timed calls go straight to the C ABI with their arguments built once: a launch of a few
    # microseconds must not be timed through ten microseconds of Python
    import ctypes as C
    L = al.load()
    tab = (C.c_void_p * 6)(*[bufs[f].data_ptr() for f in range(6)])
    cdims = (C.c_size_t * 3)(*dims)
    gp = C.c_void_p(grid.data_ptr())
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)

    def pack(mask):
        assert L.alamd_halo_pack(tab, gp, cdims, h, 8, mask, st) == 0

    def unpack(mask):
        assert L.alamd_halo_unpack(gp, tab, cdims, h, 8, mask, st) == 0

    wall, kms = timed(torch, lambda: pack(0x3f), steps, warmup)
    res["pack_all_us"], res["pack_all_gbps"] = kms * 1e3, 2 * 6 * face_bytes / (kms * 1e-3) * 1e-9
    wall2, kms2 = timed(torch, lambda: unpack(0x3f), steps, warmup)
    res["unpack_all_us"], res["unpack_all_gbps"] = kms2 * 1e3, 2 * 6 * face_bytes / (kms2 * 1e-3) * 1e-9
    # what the six-face launches really move (one 128-byte line per 16-byte run of an x face, 1.26 lines
    # per row when both x faces go together; ghost runs written as 32-byte pieces): from the counter
    # profile profiles/halo_kernel_f64_c5.md
    hbm, res["hbm_bytes_source"] = halo_traffic()
    if hbm:
        res["pack_all_hbm_bytes"], res["unpack_all_hbm_bytes"] = hbm
        res["pack_all_hbm_gbps"] = hbm[0] / (kms * 1e-3) * 1e-9
        res["unpack_all_hbm_gbps"] = hbm[1] / (kms2 * 1e-3) * 1e-9
    for f, name in enumerate(("-x", "+x", "-y", "+y", "-z", "+z")):
        _, k1 = timed(torch, lambda: pack(1 << f), steps, warmup)
        _, k2 = timed(torch, lambda: unpack(1 << f), steps, warmup)
        res["face" + name] = {"pack_us": k1 * 1e3, "pack_gbps": 2 * face_bytes / (k1 * 1e-3) * 1e-9,
                              "unpack_us": k2 * 1e3, "unpack_gbps": 2 * face_bytes / (k2 * 1e-3) * 1e-9}
    _, k1 = timed(torch, lambda: pack(3), steps, warmup)
    _, k2 = timed(torch, lambda: unpack(3), steps, warmup)
    res["faces-x+x"] = {"pack_us": k1 * 1e3, "unpack_us": k2 * 1e3}
    alg = 4 * 6 * face_bytes
    res.update({"algorithmic_bytes": alg, "ms_per_step": (wall + wall2) * 1e3, "kernel_ms": kms + kms2,
                "gbps_wall": alg / (wall + wall2) * 1e-9, "gbps_kernel": alg / ((kms + kms2) * 1e-3) * 1e-9})
    return res


def run_flag_workload():
    exe = os.path.join(ROOT, "tests", "cpp", "bench_flags")
    p = subprocess.run([exe, "2000"], capture_output=True, text=True, timeout=300)
    line = [l for l in p.stdout.splitlines() if l.startswith("{")]
    if p.returncode != 0 or not line:
        return {"workload": "flags", "error": (p.stdout + p.stderr)[-300:]}
    res = json.loads(line[-1])
    res["workload"] = "flags"
    return res


def run_copy_calibration(al, torch, steps, warmup):
    """A plain 1-read + 1-write copy of 1 GiB through alamd_copy: the reference
    point that hardware-counter readings of the combine kernel are scaled by."""
    n = 1 << 30
    src = torch.empty(n, dtype=torch.uint8, device="cuda")
    dst = torch.empty(n, dtype=torch.uint8, device="cuda")
    al.fill(src, "fullrange", 1, dtype="u8")
    torch.cuda.synchronize()
    for _ in range(warmup):
        al.copy(dst, src)
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    ev0.record()
    for _ in range(steps):
        al.copy(dst, src)
    ev1.record()
    torch.cuda.synchronize()
    ms = ev0.elapsed_time(ev1) / steps
    ok = bool(torch.equal(src, dst))
    return {"workload": "copy 1 GiB (alamd_copy)", "bytes_read": n, "bytes_written": n, "kernel_ms": ms,
            "gbps_kernel": 2 * n / (ms * 1e-3) * 1e-9, "copy_ok": ok}


def c2_port_sample():
    """The CPU oracle (a port of the host combine) on a quarter of the C2 workload, all host threads."""
    try:
        import oracle
        n = 1 << 24
        ins = [oracle.fill(n, "f32", "uniform_pm1", 1000 + r) for r in range(P)]
        ts = []
        for _ in range(8):
            t0 = time.perf_counter()
            oracle.combine(ins, "f32", "sum", "rank_asc")
            ts.append(time.perf_counter() - t0)
        med = sorted(ts)[len(ts) // 2]
        return {"value": (P + 1) * n * 4 / med * 1e-9, "unit": "GB/s", "cores": oracle.num_threads(),
                "sample": "CPU oracle RANK_ASC fold of the first 2^24 elements of the eight C2 buffers "
                          "(a quarter of the workload), median of 8", "median_ms": med * 1e3}
    except Exception as e:  # the baseline must never take the GPU figures down with it
        return {"error": str(e)[:200]}


def c1_gpu_checksum(al, torch):
    """C1 on the GPU: the combine of the same four generated 2^20-element buffers, in the order
    MPI_Allreduce applies above 2 KiB; returns the oracle's checksum of the result."""
    import oracle
    n, ranks = 1 << 20, 4
    ins = [torch.empty(n, dtype=torch.float32, device="cuda") for _ in range(ranks)]
    out = torch.empty(n, dtype=torch.float32, device="cuda")
    for r in range(ranks):
        al.fill(ins[r], "uniform_pm1", 1000 + r)
    order, start = al.reference_order("allreduce", ranks, n, "f32")
    al.combine([out], ins, "sum", order=order, start=start)
    torch.cuda.synchronize()
    return "%016x" % oracle.checksum(out.cpu().numpy())


def c1_gpu_time(al, torch):
    """The same configuration as an Allreduce on the GPU (the result in all four ranks' buffers):
    microseconds per call, one call at a time (each followed by a synchronisation), 200 in a row, and
    200 replayed from a HIP graph."""
    n, ranks = 1 << 20, 4
    ins = [torch.empty(n, dtype=torch.float32, device="cuda") for _ in range(ranks)]
    outs = [torch.empty(n, dtype=torch.float32, device="cuda") for _ in range(ranks)]
    for r in range(ranks):
        al.fill(ins[r], "uniform_pm1", 1000 + r)
    call = lambda: al.combine(outs, ins, "sum", order="tree_rsg")
    for _ in range(10):
        call()
    torch.cuda.synchronize()
    one = []
    for _ in range(100):
        t0 = time.perf_counter()
        call()
        torch.cuda.synchronize()
        one.append(time.perf_counter() - t0)
    t0 = time.perf_counter()
    for _ in range(200):
        call()
    torch.cuda.synchronize()
    row = (time.perf_counter() - t0) / 200
    # the same call captured in a HIP graph and replayed: no binding or argument checking in between
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for _ in range(20):
            call()
    g.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(10):
        g.replay()
    torch.cuda.synchronize()
    replay = (time.perf_counter() - t0) / 200
    return {"one_call_and_wait_us": sorted(one)[len(one) // 2] * 1e6, "in_a_row_us": row * 1e6,
            "in_a_graph_us": replay * 1e6,
            "note": "in_a_row is bound by the Python binding that makes the calls, in_a_graph by the device"}


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return None


def cpu_baseline(al=None, torch=None):
    """The reference's MPI-backend host combine on this box's host cores."""
    exe = os.path.join(ROOT, "oracle", "mpi_baseline")
    mpiexec = "/opt/conda/bin/mpiexec"
    if os.path.exists(exe) and os.path.exists(mpiexec):
        try:
            p = subprocess.run([mpiexec, "-n", "4", exe, str(1 << 20), "10", "3000"], capture_output=True,
                               text=True, timeout=180)
            line = [l for l in p.stdout.splitlines() if l.startswith("{")]
            if p.returncode == 0 and line:
                r = json.loads(line[-1])
                same = None
                if al is not None and "checksum" in r:
                    # the bits MPI_Allreduce produced on the host against the GPU's for the same inputs
                    same = c1_gpu_checksum(al, torch) == r["checksum"]
                gpu_us = c1_gpu_time(al, torch) if al is not None else None
                return {"value": r["gbps_median"], "unit": "GB/s", "cores": 4, "kind": "port",
                        "sample": "MPI_Allreduce(MPI_SUM, MPI_FLOAT) on a dup'd communicator, the call "
                                  "Al::Allreduce<MPIBackend> forwards to; 4 MPICH ranks on this host, "
                                  "2^20 elements per rank, uniform[-1,1] seed 1000+rank, 10 warm-up + 3000 "
                                  "timed (about 10 s), median of max-over-ranks; GB/s over (P+1)*n*4 bytes",
                        "median_ms": r["median_ms"], "min_ms": r["min_ms"], "gpu_result_identical": same,
                        "gpu_same_configuration": gpu_us,
                        "host_cpus": os.cpu_count(), "cpu_model": cpu_model(), "same_workload_port": c2_port_sample()}
        except Exception:
            pass
    # MPI-free restatement: the oracle's threaded tree combine on the same shape
    import numpy as np
    import oracle
    n, ranks = 1 << 20, 4
    ins = [oracle.fill(n, "f32", "uniform_pm1", 1000 + r) for r in range(ranks)]
    ts = []
    for _ in range(30):
        t0 = time.perf_counter()
        oracle.combine(ins, "f32", "sum", "tree_dbl")
        ts.append(time.perf_counter() - t0)
    med = sorted(ts)[len(ts) // 2]
    return {"value": (ranks + 1) * n * 4 / med * 1e-9, "unit": "GB/s", "cores": oracle.num_threads(),
            "kind": "port", "sample": "MPI-free restatement: CPU oracle TREE_DBL combine, 4 buffers of 2^20 "
                                      "fp32, median of 30", "median_ms": med * 1e3,
            "host_cpus": os.cpu_count(), "cpu_model": cpu_model()}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="c2_f32_sum",
                    choices=sorted(WORKLOADS) + ["c3_ring_stepwise", "c3_ring_fused", "c5_halo", "c5_halo_load_policy",
                                                 "flags", "c2_sum_rotating_pair"] + LAYOUTS)
    ap.add_argument("--also", default=DEFAULT_ALSO,
                    help="comma-separated extra workloads reported under 'also' ('' for none)")
    ap.add_argument("--batch", default="",
                    help="run these workloads one after the other and print {name: record} (what 'also' runs)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--raw", action="store_true", help="print only the workload's own measurement record")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run only the 1 GiB copy kernel (counter calibration) and print its JSON line")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the P logical ranks live in one GPU's HBM); "
              "--gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch
    import aluminum_amd as al
    al.load()
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    rc = al.load().alamd_init()
    if rc:
        print("bench.py: " + al.load().alamd_last_error().decode(), file=sys.stderr)
        sys.exit(1)

    def run_one(name, steps, warmup):
        if name.startswith("c3_ring_"):
            res = run_ring_workload(al, torch, name[len("c3_ring_"):], steps, warmup)
        elif name == "c5_halo":
            res = run_halo_workload(al, torch, steps, warmup)
        elif name == "c5_halo_load_policy":
            res = run_halo_policy_workload(al, torch, steps, warmup)
        elif name == "c2_sum_rotating_pair":
            res = run_pair_workload(al, torch, steps, warmup)
        elif name == "flags":
            res = run_flag_workload()
        elif name in LAYOUTS:
            res = run_layout_workload(al, torch, name, steps, warmup)
        else:
            res = run_combine_workload(al, torch, name, steps, warmup)
        if "gbps_kernel" in res:
            res["frac"] = res["gbps_kernel"] / HBM_PEAK_GBPS  # of the 8 TB/s HBM peak, from the kernel's own time
        return res

    if args.calibrate_copy:
        print(json.dumps(run_copy_calibration(al, torch, args.steps, args.warmup)))
        return
    if args.batch:
        # one process for all of them; each starts from an empty device
        out = {}
        for name in [w for w in args.batch.split(",") if w]:
            try:
                out[name] = run_one(name, args.steps, args.warmup)
            except Exception as e:  # one workload must not take the others down
                out[name] = {"workload": name, "error": str(e)[:300]}
            torch.cuda.synchronize()
            torch.cuda.empty_cache()
        print(json.dumps(out))
        return
    main_res = run_one(args.workload, args.steps, args.warmup)
    if args.raw or args.workload not in WORKLOADS:
        print(json.dumps(main_res))
        return
    # the secondary workloads run in a fresh process, one after the other, each with its buffers
    # allocated on an empty device like the primary one
    also = {}
    names = [w for w in args.also.split(",") if w and w != args.workload]
    if names:
        torch.cuda.empty_cache()
        p = subprocess.run([sys.executable, os.path.abspath(__file__), "--batch", ",".join(names), "--also", "",
                            "--no-cpu-baseline", "--steps", str(max(5, args.steps // 2)),
                            "--warmup", str(max(2, args.warmup // 2))],
                           capture_output=True, text=True, timeout=900)
        line = [l for l in p.stdout.splitlines() if l.startswith("{")]
        also = json.loads(line[-1]) if p.returncode == 0 and line else {"error": p.stderr[-300:]}
    traffic, traffic_source = measured_traffic(args.workload)
    pair = also.get("c2_sum_rotating_pair") if isinstance(also.get("c2_sum_rotating_pair"), dict) else {}

    out = {
        "metric": METRIC, "value": main_res["gbps_wall"], "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": main_res["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": main_res["dtype"], "data": "synthetic",
        "config": {"workload": "C2 single-GPU P-way combine: P=8 logical-rank fp32 buffers of 2^26 elements "
                               "(2 GiB in, 256 MiB out), ReductionOperator::sum, order %s" % main_res["order"]
                   if args.workload == "c2_f32_sum" else args.workload,
                   "P": P, "count_per_rank": main_res["count"], "op": main_res["op"], "order": main_res["order"],
                   "entry_point": "alamd_combine"},
        "pct_of_hbm_peak": 100.0 * main_res["gbps_wall"] / HBM_PEAK_GBPS,
        "parity_vs_oracle": main_res.get("parity_vs_oracle"),
        "roofline": {"bound": "hbm", "achieved": main_res["gbps_kernel"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": main_res["gbps_kernel"] / HBM_PEAK_GBPS,
                     # the same kernel over four rotating buffer sets: nothing a call reads or writes was
                     # touched by the three calls before it, so the 256 MiB memory-side cache cannot help;
                     # fp32 and bf16 read the same memory, taking turns (also.c2_sum_rotating_pair)
                     "frac_untouched": pair.get("frac_f32"),
                     "frac_untouched_bf16": pair.get("frac_bf16"),
                     # HBM bytes (fetched + written) per call and per launch, read from the committed
                     # counter profile, not measured by this run
                     "traffic": traffic,
                     "traffic_per_launch": traffic // main_res["launches_per_step"] if traffic else None,
                     "traffic_source": traffic_source,
                     "kernel": KERNEL_NAME.get(args.workload, "alamd::fold_vec_kernel"),
                     "kernel_ms": main_res["kernel_ms"],
                     # the launches one call is cut into, as the library's planner reports them
                     "launches_per_step": main_res["launches_per_step"],
                     "launch_avg_us": main_res["kernel_ms"] * 1e3 / main_res["launches_per_step"],
                     "algorithmic_bytes_per_launch": main_res["algorithmic_bytes"] // main_res["launches_per_step"],
                     "algorithmic_bytes": main_res["algorithmic_bytes"]},
        "also": also,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(al, torch)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
