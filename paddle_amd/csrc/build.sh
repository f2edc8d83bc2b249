#!/bin/bash
# Builds paddle_amd/lib/libwol_gfx950.so from the HIP sources beside this file.
set -euo pipefail
HERE="$(cd "$(dirname "${BASH_SOURCE[0]}")" && pwd)"
ROOT="$(cd "$HERE/../.." && pwd)"
OUT="$HERE/../lib"
OBJ="$HERE/build"
mkdir -p "$OUT" "$OBJ"
HIPCC="${HIPCC:-/opt/rocm/bin/hipcc}"
FLAGS=(--offload-arch=gfx950 -O3 -std=c++17 -fPIC -I"$ROOT/include" -I"$HERE"
       -Xclang -target-feature -Xclang -packed-fp32-ops
       -Wno-unused-command-line-argument -Wno-unknown-attributes)
pids=()
for f in wol_quantize wol_prescale wol_diag wol_linear_stream wol_linear_stream_f16 wol_linear_batch wol_linear_gemm wol_linear_grad wol_llm_int8 wol_c_api; do
  # the remarks list registers, scratch and spills of every kernel
  "$HIPCC" "${FLAGS[@]}" -Rpass-analysis=kernel-resource-usage -c "$HERE/$f.hip" -o "$OBJ/$f.o" \
    2> "$OBJ/$f.resources.txt" &
  pids+=($!)
done
for p in "${pids[@]}"; do wait "$p"; done
# No kernel may spill to memory: spill code is memory traffic in the inner
# loops, and in the GEMM its loads would join the in-order stream the tile
# loads are counted in.  (Scalar registers that overflow into lanes of a vector
# register cost no memory traffic and are allowed.)
if grep -E "(VGPRs Spill|ScratchSize \[bytes/lane\]): [1-9]" "$OBJ"/*.resources.txt; then
  echo "build.sh: a kernel spills registers (see $OBJ/*.resources.txt)" >&2
  exit 1
fi
grep -h "error" "$OBJ"/*.resources.txt >&2 || true
"$HIPCC" --offload-arch=gfx950 -shared -fPIC -o "$OUT/libwol_gfx950.so" \
  "$OBJ/wol_quantize.o" "$OBJ/wol_prescale.o" "$OBJ/wol_diag.o" "$OBJ/wol_linear_stream.o" "$OBJ/wol_linear_stream_f16.o" "$OBJ/wol_linear_batch.o" "$OBJ/wol_linear_gemm.o" "$OBJ/wol_linear_grad.o" "$OBJ/wol_llm_int8.o" "$OBJ/wol_c_api.o"
echo "built $OUT/libwol_gfx950.so"
