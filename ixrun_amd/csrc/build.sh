#!/bin/sh
# Builds libixhip.so for gfx950 next to the sources (hipcc cross-compiles, no GPU needed).  One object per
# source file, compiled side by side (JOBS, default 8), then linked.
set -e
cd "$(dirname "$0")"
HIPCC="${HIPCC:-/opt/rocm/bin/hipcc}"
SRCS="ixh_api.hip ixh_generic.hip ixh_fast358.hip ixh_rows358.hip ixh_slots358.hip ixh_strips358.hip ixh_tiles358.hip ixh_prefill.hip ixh_prefill358.hip ixh_decode_staged.hip ixh_gemv_staged.hip ixh_encode.hip ixh_dense358.hip ixh_dense5.hip ixh_decode_rows358.hip"
FLAGS="--offload-arch=gfx950 -O3 -std=c++17 -fPIC -Xclang -target-feature -Xclang -packed-fp32-ops -Wall -Wno-unused-function -Wno-pass-failed $*"
# Kernels of these files take the arguments that their first memory requests need as their leading arguments; the
# hardware loads up to 14 argument words into registers before a wave starts (older firmware runs the loads that the
# compiler keeps at the kernel's entry instead), which takes a read of the argument block off the critical path.
PRELOAD_SRCS="${PRELOAD_SRCS-ixh_rows358.hip}"
PRELOAD_FLAGS="-mllvm -amdgpu-kernarg-preload-count=14"
mkdir -p build
OBJS=""
for s in $SRCS; do OBJS="$OBJS build/${s%.hip}.o"; done
printf '%s\n' $SRCS | xargs -P "${JOBS:-8}" -I{} sh -c "rm -f build/\$(basename {} .hip).o; extra=; case ' $PRELOAD_SRCS ' in *' {} '*) extra='$PRELOAD_FLAGS';; esac; $HIPCC $FLAGS \$extra -c {} -o build/\$(basename {} .hip).o 2>&1 | grep -v 'packed-fp32-ops' >&2; test -f build/\$(basename {} .hip).o"
exec "$HIPCC" --offload-arch=gfx950 -shared -fPIC $OBJS -o libixhip.so
