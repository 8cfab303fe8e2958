#!/bin/bash
# Sweep drivers in the shape of the reference's src/gemm/run.sh (M from 44160 down in steps of 384 at
# N=2048, K=384, ldc=44160 > M), plus the five benchmark configurations of this library.
#   ./run.sh hpl [dtype]      the reference's HPL trailing-update sweep, best config per size (type 1)
#   ./run.sh configs          the five benchmark configurations with the table's pick (type 0)
#   ./run.sh report MODE [args]   machine-readable records (JSON lines on stdout, --json/--csv FILE) with roofline
#                                 fractions, an fp64 check and the rocprofv3 commands per shape: MODE = configs | hpl |
#                                 shapes SPEC...  (python -m gemm_mmbo_amd.report)
cd "$(dirname "$0")"
mode=${1:-configs}
if [ "$mode" = report ]; then
  shift
  cd ../.. && python3 -m gemm_mmbo_amd.report "$@"
  exit $?
elif [ "$mode" = hpl ]; then
  dt=${2:-d}
  for M in {44160..384..-3840}; do
    ./benchmark 1 ${M} 2048 384 ${M} 2048 44160 N T ${dt} 1 -1 1 || exit 1
  done
else
  ./benchmark 0 1024 1024 1024 1024 1024 1024 N N s 1 1 0 || exit 1
  ./benchmark 0 4096 4096 4096 4096 4096 4096 N T s 1 1.5 0.5 || exit 1
  ./benchmark 0 4096 4096 4096 4096 4096 4096 T N s 1 1.5 0.5 || exit 1
  ./benchmark 0 8192 8192 8192 8192 8192 8192 N N h 1 1 0 || exit 1
  ./benchmark 0 8192 8192 8192 8192 8192 8192 N N s 1 1 0 || exit 1
  for dt in s h; do
    ./benchmark 0 1023 777 513 1023 513 1023 N N ${dt} 1 1 0 || exit 1
    ./benchmark 0 4096 128 4096 4096 4096 4096 N N ${dt} 1 1 0 || exit 1
    ./benchmark 0 128 4096 8192 128 8192 128 N N ${dt} 1 1 0 || exit 1
  done
  ./benchmark 0 512 512 512 512 512 512 T N h 64 1 1 || exit 1
  ./benchmark 0 44160 2048 384 44160 2048 44160 N T d 1 -1 1 || exit 1
fi
