#!/bin/bash
# Build ./cuda_extension.so from the workspace sources and report how long it took.
# Run from the workspace directory. Exit status is the compile step's.

t0=$(date +%s.%N)

python3 -m utils.compile
rc=$?

t1=$(date +%s.%N)
echo "[TIME] Compilation took $(awk "BEGIN {printf \"%.2f\", $t1 - $t0}")s"

exit $rc
