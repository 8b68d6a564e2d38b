#!/bin/sh
# Builds libixhip.so for gfx950 next to the sources (hipcc cross-compiles, no GPU needed).
set -e
cd "$(dirname "$0")"
HIPCC="${HIPCC:-/opt/rocm/bin/hipcc}"
exec "$HIPCC" --offload-arch=gfx950 -O3 -std=c++17 -fPIC -shared \
    -Xclang -target-feature -Xclang -packed-fp32-ops \
    -Wall -Wno-unused-function -Wno-pass-failed \
    ixh_api.hip ixh_generic.hip ixh_fast358.hip ixh_rows358.hip ixh_prefill.hip ixh_decode_staged.hip ixh_gemv_staged.hip ixh_encode.hip ixh_dense358.hip ixh_decode_rows358.hip -o libixhip.so "$@"
