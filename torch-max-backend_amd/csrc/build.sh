#!/bin/sh
# Builds libtmb_hip.so for gfx950 next to this script. Usage: sh build.sh [extra hipcc flags]
set -e
here="$(cd "$(dirname "$0")" && pwd)"
HIPCC="${HIPCC:-/opt/rocm/bin/hipcc}"
FLAGS="--offload-arch=gfx950 -O3 -std=c++17 -fPIC -Xclang -target-feature -Xclang -packed-fp32-ops"
objs=""
for f in softmax layer_norm reduce gemm attention backward misc; do
  "$HIPCC" $FLAGS "$@" -c "$here/$f.hip" -o "$here/$f.o" &
  objs="$objs $here/$f.o"
done
wait
"$HIPCC" --offload-arch=gfx950 -shared -fPIC $objs -o "$here/libtmb_hip.so"
echo "built $here/libtmb_hip.so"
