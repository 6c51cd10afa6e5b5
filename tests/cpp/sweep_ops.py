"""Randomised sweep over test_ops' option space on one GPU, in the manner of the
reference's test driver (test/run_tests.py: collective x datatype x in place x
non-blocking x sizes), with logical ranks in place of MPI processes.

    python tests/cpp/sweep_ops.py [--seed S] [--runs N] [--max-size M] [--threads SHARE]

Every run is one test_ops process; it compares with the CPU oracle bit for bit.
Exit status 1 if any run fails."""
import argparse
import os
import random
import subprocess
import sys
import time

HERE = os.path.dirname(os.path.abspath(__file__))
OPS = ["allreduce", "reduce", "reduce_scatter", "allgather", "reduce_scatterv", "allgatherv"]
DATATYPES = ["char", "schar", "uchar", "short", "ushort", "int", "uint", "long", "ulong", "longlong", "ulonglong",
             "float", "double", "half", "bfloat16"]
FLOATS = ("float", "double", "half", "bfloat16")
INT_REDUCTIONS = ["sum", "prod", "min", "max", "lor", "land", "lxor", "bor", "band", "bxor", "avg"]
FP_REDUCTIONS = ["sum", "prod", "min", "max", "avg"]
ALGORITHMS = {
    "allreduce": ["automatic", "rank_order", "tree_doubling", "tree_halving", "tree_binomial", "ring", "ring_fused"],
    "reduce": ["automatic", "rank_order", "tree_doubling", "tree_halving", "tree_binomial"],
    "reduce_scatter": ["automatic", "rank_order", "tree_doubling", "tree_halving", "tree_binomial", "pairwise",
                       "ring_fused"],
    "reduce_scatterv": ["automatic"], "allgather": ["automatic"], "allgatherv": ["automatic"],
}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--seed", type=int, default=1)
    ap.add_argument("--runs", type=int, default=200)
    ap.add_argument("--max-size", type=int, default=262144)
    ap.add_argument("--threads", type=float, default=0.0,
                    help="share of runs that drive the sweep from 2 to 4 threads at once (test_ops --threads)")
    args = ap.parse_args()
    exe = os.path.join(HERE, "test_ops")
    if not os.path.exists(exe):
        sys.exit("tests/cpp/test_ops is not built (make -C tests/cpp)")
    rng = random.Random(args.seed)
    t0, fails = time.time(), 0
    last = t0
    for k in range(args.runs):
        op, dt = rng.choice(OPS), rng.choice(DATATYPES)
        ranks = rng.choice([1, 2, 3, 4, 5, 7, 8, 12, 16, 24, 32, 33, 40, 48, 63, 64])
        max_size = rng.choice([4096, 65536, args.max_size])
        # what the run holds in memory (and checks on the host) grows with ranks^2 x size for every
        # collective but allreduce and reduce: keep it to a few GB, or one draw takes minutes
        elem = {"char": 1, "schar": 1, "uchar": 1, "short": 2, "ushort": 2, "half": 2, "bfloat16": 2, "int": 4,
                "uint": 4, "float": 4}.get(dt, 8)
        held = ranks * (ranks if op not in ("allreduce", "reduce") else 2) * elem * 2
        while max_size > 4096 and held * max_size > (8 << 30):
            max_size //= 2
        cmd = [exe, "--op", op, "--datatype", dt,
               "--reduction-op", rng.choice(FP_REDUCTIONS if dt in FLOATS else INT_REDUCTIONS),
               "--algorithm", rng.choice(ALGORITHMS[op]), "--ranks", str(ranks), "--root", str(rng.randrange(ranks)),
               "--odd-sizes", "--min-size", str(rng.choice([0, 1, 3, 64])),
               "--max-size", str(max_size)]
        if rng.random() < 0.5:
            cmd.append("--inplace")
        if rng.random() < 0.5:
            cmd.append("--nonblocking")
        if args.threads > 0 and rng.random() < args.threads:
            cmd += ["--threads", str(rng.choice([2, 3, 4]))]
        p = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
        if p.returncode != 0 or "PASSED" not in p.stdout:
            fails += 1
            print("FAIL rc=%d: %s\n%s\n%s" % (p.returncode, " ".join(cmd[1:]), p.stdout[-600:], p.stderr[-300:]),
                  flush=True)
        if k % 25 == 24 or time.time() - last > 30:  # a line at least every half minute
            last = time.time()
            print("%d runs, %d failed, %.0f s" % (k + 1, fails, time.time() - t0), flush=True)
    print("TOTAL %d runs, %d failed" % (args.runs, fails))
    sys.exit(1 if fails else 0)


if __name__ == "__main__":
    main()
