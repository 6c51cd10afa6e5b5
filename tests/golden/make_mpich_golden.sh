#!/bin/bash
# Regenerates tests/golden/mpich_P*.json.gz by calling MPI_Allreduce, MPI_Reduce,
# MPI_Reduce_scatter_block and MPI_Reduce_scatter of the image's MPICH (the calls
# the reference's MPI backend forwards to) on seeded inputs.  P = 16 and above
# run oversubscribed on small machines; their inputs are small.  Needs /opt/conda MPICH; run from the
# repository root:  bash tests/golden/make_mpich_golden.sh
set -euo pipefail
here="$(cd "$(dirname "$0")" && pwd)"
root="$(cd "$here/../.." && pwd)"
tmp="$(mktemp -d)"
trap 'rm -rf "$tmp"' EXIT
gcc -O2 -fopenmp -ffp-contract=off -I/opt/conda/include \
    "$here/mpich_golden.c" "$root/oracle/oracle.c" /opt/conda/lib/libmpi.so \
    -Wl,--disable-new-dtags -Wl,-rpath,/lib/x86_64-linux-gnu:/opt/conda/lib \
    -lm -o "$tmp/mpich_golden"
for P in 2 3 4 5 7 8 16 33 48 64; do
  /opt/conda/bin/mpiexec -n "$P" "$tmp/mpich_golden" big > "$tmp/out.json"
  python3 -c "import json,sys; json.load(open(sys.argv[1]))" "$tmp/out.json"
  gzip -9 -n -c "$tmp/out.json" > "$here/mpich_P$P.json.gz"
  echo "P=$P: $(stat -c %s "$here/mpich_P$P.json.gz") bytes"
done
