#!/bin/bash
# Builds tensor_amd/lib/libotter_hip_int8.so for gfx950 (cross-compiles without a GPU).
set -e
cd "$(dirname "$0")"
mkdir -p ../lib
HIPCC=${HIPCC:-/opt/rocm/bin/hipcc}
FLAGS="--offload-arch=gfx950 -O3 -std=c++17 -fPIC -ffp-contract=off -Xclang -target-feature -Xclang -packed-fp32-ops -mllvm -amdgpu-mfma-vgpr-form=1 -Wno-unused-command-line-argument"
SRCS="capi.hip elementwise.hip conv_direct.hip conv_igemm.hip conv_pw.hip conv_block.hip conv3x3.hip conv3x3_chain.hip conv_dw.hip conv_dw_mfma.hip conv_xdw.hip conv_stem.hip glue.hip reshape.hip"
OBJS=""
pids=""
for s in $SRCS; do
  [ -f "$s" ] || continue
  o=../lib/${s%.hip}.o
  OBJS="$OBJS $o"
  ( $HIPCC $FLAGS -c "$s" -o "$o" 2> >(grep -v "packed-fp32-ops" >&2) ) &
  pids="$pids $!"
done
for p in $pids; do wait $p; done
$HIPCC --offload-arch=gfx950 -shared -fPIC $OBJS -o ../lib/libotter_hip_int8.so
echo "built $(cd ../lib && pwd)/libotter_hip_int8.so"
