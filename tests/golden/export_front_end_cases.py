"""Writes mpich_front_end_cases.txt from the mpich_P*.json.gz fixtures next to it: one line per case whose
inputs are the generator's (or, distribution 99, the special values planted by the rule of mpich_golden.c's
plant_specials_many: float min / max only, whose result is one of the operands bit for bit), with the
checksum of what MPICH returned.  The C++ front end's tests read it (no JSON or gzip there) to check that
`automatic` gives MPICH's bits for every collective, root and size.  "allreduce" and "reduce" lines hold what
the non-blocking calls returned (`automatic`); for long messages of native types "allreduce_blocking" and
"reduce_blocking" lines hold what MPI_Allreduce and MPI_Reduce returned (`automatic_mpi_blocking`).

    python tests/golden/export_front_end_cases.py
"""
import glob
import gzip
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import oracle  # noqa: E402


def cs_hex(hexstr):
    return "%016x" % oracle.checksum(np.frombuffer(bytes.fromhex(hexstr), dtype=np.uint8))


def main():
    lines = ["# collective P dtype op ... : see export_front_end_cases.py; checksums are alo_checksum of MPICH's output"]
    paths = sorted(glob.glob(os.path.join(HERE, "mpich_P*.json.gz")), key=lambda p: int(os.path.basename(p)[7:-8]))
    for path in paths:
        with gzip.open(path, "rt") as f:
            doc = json.load(f)
        P = doc["P"]
        for c in doc["cases"]:
            planted = c["note"] == "specials"
            if planted and (P == 2 or c["op"] not in ("min", "max") or c["coll"] not in ("allreduce", "reduce")):
                continue
            head = "%s %d %s %s" % (c["coll"], P, c["dtype"], c["op"])
            gen = "%d %d" % (99 if planted else c["dist"], c["seed_base"])
            long_native = c["dtype"] not in ("f16", "bf16") and c["n"] * oracle.dtype_size(c["dtype"]) > 2048
            if c["coll"] == "allreduce":
                lines.append("%s %d %s %s" % (head, c["n"], gen, cs_hex(c.get("out_nonblocking", c["out"][0]))))
                if long_native:
                    lines.append("allreduce_blocking %s %d %s %s" % (head.split(" ", 1)[1], c["n"], gen, cs_hex(c["out"][0])))
            elif c["coll"] == "reduce":
                cs = c["out_checksum"] if "out_checksum" in c else cs_hex(c["out"])
                nb = cs
                if not c["nonblocking_in_place_same"]:
                    nb = c["out_nonblocking_checksum"] if "out_nonblocking_checksum" in c else cs_hex(c["out_nonblocking"])
                lines.append("%s %d %s %d %s" % (head, c["n"], gen, c["root"], nb))
                if long_native:
                    lines.append("reduce_blocking %s %d %s %d %s" % (head.split(" ", 1)[1], c["n"], gen, c["root"], cs))
            elif c["coll"] == "reduce_scatter":
                cs = c["out_checksum"] if "out_checksum" in c else [cs_hex(h) for h in c["out"]]
                lines.append("%s %d %s %s" % (head, c["n"], gen, " ".join(cs)))
            elif c["coll"] == "reduce_scatterv":
                es = oracle.dtype_size(c["dtype"])
                cs = c["out_checksum"] if "out_checksum" in c else [cs_hex(h[:2 * es * k]) for h, k in zip(c["out"], c["counts"])]
                lines.append("%s %s %s %s" % (head, gen, " ".join(str(k) for k in c["counts"]), " ".join(cs)))
    with open(os.path.join(HERE, "mpich_front_end_cases.txt"), "w") as f:
        f.write("\n".join(lines) + "\n")
    print(len(lines) - 1, "cases")


if __name__ == "__main__":
    main()
