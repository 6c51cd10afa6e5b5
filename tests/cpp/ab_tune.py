"""Each launch-planner size against alternatives, on this machine: the default and the alternatives
take turns (default, alt 1, alt 2, default, alt 1, ...) inside one process, on the same buffers, which
go round four sets so that no call touches what the three calls before it touched.

    python tests/cpp/ab_tune.py [--reps 7] [--steps 8] [--only NAME]

Prints, per case, the median rate of every setting over the repetitions, its spread, and the median
of the paired differences to the default (which placement noise between runs does not enter)."""
import argparse
import os
import statistics
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
HUGE = 1 << 44  # "never cut"


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--reps", type=int, default=7)
    ap.add_argument("--steps", type=int, default=8)
    ap.add_argument("--only", default="")
    args = ap.parse_args()
    import torch
    import aluminum_amd as al
    al.load()

    def timed(fns):
        for f in fns:
            f()  # warm-up, one call per buffer set
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for k in range(args.steps):
            fns[k % len(fns)]()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3 / args.steps

    def bufs(n, count, dtype=torch.float32):
        return [torch.empty(count, dtype=dtype, device="cuda") for _ in range(n)]

    def combine(P, mib, nout):
        count = (mib << 20) // 4
        sets = []
        for _ in range(4):
            ins, outs = bufs(P, count), bufs(nout, count)
            for r, t in enumerate(ins):
                al.fill(t, "uniform_pm1", 1000 + r)
            sets.append(lambda ins=ins, outs=outs: al.combine(outs, ins, "sum", order="rank_asc"))
        return sets, (P + nout) * count * 4

    def allgather(P, mib):
        count = (mib << 20) // 4
        sets = []
        for _ in range(4):
            sends, recvs = bufs(P, count), bufs(P, P * count)
            for r, t in enumerate(sends):
                al.fill(t, "uniform_pm1", 1000 + r)
            sets.append(lambda s=sends, r=recvs: al.allgather(r, s, count=count))
        return sets, (P + P * P) * count * 4

    def ring(P, mib):
        count = (mib << 20) // 2
        sets = []
        for _ in range(4):
            b = bufs(P, count, torch.bfloat16)
            for r, t in enumerate(b):
                al.fill(t, "normal", 2000 + r, dtype="bf16")
            sets.append(lambda b=b: al.ring_allreduce(b, "sum", mode="fused", dtype="bf16"))
        return sets, 2 * P * count * 2

    M = 1 << 20
    cases = [
        # (label, workload, size name, alternatives)
        ("fold P=8, 256 MiB per rank, one output", lambda: combine(8, 256, 1), "launch_bytes", [400 * M, 1600 * M, HUGE]),
        ("fold P=2, 256 MiB per rank, one output", lambda: combine(2, 256, 1), "launch_bytes", [400 * M, 1600 * M, HUGE]),
        ("fold P=4, 256 MiB per rank, one output", lambda: combine(4, 256, 1), "launch_bytes", [400 * M, 1600 * M, HUGE]),
        ("allreduce P=8, 64 MiB per rank, eight outputs", lambda: combine(8, 64, 8), "two_step_min_outputs", [99]),
        ("allreduce P=8, 16 MiB per rank, eight outputs", lambda: combine(8, 16, 8), "two_step_min_outputs", [99]),
        ("allreduce P=8, 8 MiB per rank, eight outputs", lambda: combine(8, 8, 8), "two_step_min_total_bytes", [32 * M]),
        ("allreduce P=4, 16 MiB per rank, four outputs", lambda: combine(4, 16, 4), "two_step_min_total_bytes", [32 * M]),
        ("allreduce P=4, 64 MiB per rank, four outputs", lambda: combine(4, 64, 4), "two_step_min_total_bytes", [HUGE]),
        ("allreduce P=16, 8 MiB per rank, sixteen outputs", lambda: combine(16, 8, 16), "two_step_min_total_bytes", [HUGE]),
        ("allreduce P=8, 1 GiB per rank, eight outputs", lambda: combine(8, 1024, 8), "two_step_piece_bytes", [32 * M, 64 * M, 256 * M, 512 * M, HUGE]),
        ("allreduce P=8, 512 MiB per rank, eight outputs", lambda: combine(8, 512, 8), "two_step_piece_bytes", [64 * M, 256 * M, HUGE]),
        ("allreduce P=8, 256 MiB per rank: the spread of a result just written", lambda: combine(8, 256, 8),
         "spread_cache_chunk_tiles", [1024, 256]),
        ("allreduce P=8, 256 MiB per rank: chunks per spread launch", lambda: combine(8, 256, 8),
         "spread_cache_launch_chunks", [2, 64]),
        ("allgather P=8, 32 MiB slices", lambda: allgather(8, 32), "spread_hbm_chunk_tiles", [512, 2048]),
        ("allgather P=8, 128 MiB slices", lambda: allgather(8, 128), "spread_hbm_launch_chunks", [1, 8, HUGE]),
        ("allgather P=8, 32 MiB slices: bytes per launch", lambda: allgather(8, 32), "spread_launch_bytes", [72 * M, 1152 * M]),
        ("fused ring allreduce bf16 P=8, 256 MiB per rank", lambda: ring(8, 256), "ring_piece_bytes", [16 * M, 64 * M, HUGE]),
        ("fused ring allreduce bf16 P=8, 1 GiB per rank", lambda: ring(8, 1024), "ring_piece_bytes", [64 * M, 128 * M, 512 * M, HUGE]),
        ("fused ring allreduce bf16 P=4, 256 MiB per rank", lambda: ring(4, 256), "ring_piece_bytes", [64 * M, HUGE]),
    ]
    for label, make, name, alts in cases:
        if args.only and args.only not in name and args.only not in label:
            continue
        sets, alg = make()
        default = al.tuned(name)
        settings = [0] + alts  # 0 restores the default
        rates = {v: [] for v in settings}
        for _ in range(args.reps):
            for v in settings:
                al.tune(name, v)
                rates[v].append(alg / timed(sets) * 1e-9)
        al.tune(name, 0)
        print("%s  [%s, default %d]" % (label, name, default), flush=True)
        for v in settings:
            r = rates[v]
            shown = "default" if v == 0 else ("never cut" if v == HUGE else str(v))
            diff = statistics.median(a - b for a, b in zip(r, rates[0]))
            print("    %-12s median %6.0f GB/s (%4.1f %% of 8 TB/s), min %6.0f, max %6.0f, paired difference to default %+6.0f GB/s"
                  % (shown, statistics.median(r), statistics.median(r) / 80.0, min(r), max(r), diff), flush=True)
        del sets
        torch.cuda.empty_cache()


if __name__ == "__main__":
    main()
