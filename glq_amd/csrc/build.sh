#!/bin/bash
# Builds glq_amd/libglq_hip.so for gfx950 (cross-compiles without a GPU).
set -e
here="$(cd "$(dirname "$0")" && pwd)"
out="$here/../libglq_hip.so"
/opt/rocm/bin/hipcc --offload-arch=gfx950 -O3 -std=c++17 -fPIC -shared \
    -Xclang -target-feature -Xclang -packed-fp32-ops \
    -Wall -Wno-unused-function \
    "$here/capi.hip" "$here/fht.hip" "$here/trellis.hip" "$here/trellis_mma.hip" "$here/trellis_tile.hip" "$here/e8.hip" "$here/e8_mma.hip" "$here/e8_tile.hip" "$here/e8_embed.hip" "$here/e8_encode.hip" "$here/trellis_encode.hip" "$here/decoder_ops.hip" \
    -o "$out" "$@"
echo "built $out"
