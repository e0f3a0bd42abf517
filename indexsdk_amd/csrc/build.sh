#!/bin/bash
# Builds libindexsdk_amd.so for gfx950 (cross-compiles without a GPU).
set -euo pipefail
HERE="$(cd "$(dirname "${BASH_SOURCE[0]}")" && pwd)"
OUT="${HERE}/../libindexsdk_amd.so"
FLAGS=(-O3 --offload-arch=gfx950 -std=c++17 -fPIC -ffp-contract=off -fvisibility=hidden
       -Xclang -target-feature -Xclang -packed-fp32-ops -Wall -Wno-unused-command-line-argument)
OBJ="${HERE}/.obj"
mkdir -p "${OBJ}"
pids=()
for src in coarse.hip coarse_resident.hip score_ring.hip pq.hip scan.hip flat.hip flat_i8.hip stream_select.hip ivfpq_index.hip ops.hip; do
  [ -f "${HERE}/${src}" ] || continue
  ( /opt/rocm/bin/hipcc "${FLAGS[@]}" -c "${HERE}/${src}" -o "${OBJ}/${src%.hip}.o" 2> >(grep -v "packed-fp32-ops' is not a recognized feature" >&2) ) &
  pids+=($!)
done
for src in capi.cpp faiss_io.cpp; do
  ( /opt/rocm/bin/hipcc "${FLAGS[@]}" -x hip -c "${HERE}/${src}" -o "${OBJ}/${src%.cpp}.o" 2> >(grep -v "packed-fp32-ops' is not a recognized feature" >&2) ) &
  pids+=($!)
done
for p in "${pids[@]}"; do wait "$p"; done
/opt/rocm/bin/hipcc --offload-arch=gfx950 -shared -fPIC -o "${OUT}" "${OBJ}"/*.o
echo "built ${OUT}"
