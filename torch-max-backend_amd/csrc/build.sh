#!/bin/sh
# Builds libtmb_hip.so for gfx950 next to this script. Usage: sh build.sh [extra hipcc flags]
# Every object is rebuilt from its source; a failed compile stops the build before the link, so a
# stale object can never end up in the library.
set -e
here="$(cd "$(dirname "$0")" && pwd)"
HIPCC="${HIPCC:-/opt/rocm/bin/hipcc}"
FLAGS="--offload-arch=gfx950 -O3 -std=c++17 -fPIC -Wno-inline-asm -Xclang -target-feature -Xclang -packed-fp32-ops"
units="softmax layer_norm reduce reduce_cols gemm attention attention_bwd backward misc"
objs=""
pids=""
for f in $units; do
  rm -f "$here/$f.o"
  "$HIPCC" $FLAGS "$@" -c "$here/$f.hip" -o "$here/$f.o" &
  pids="$pids $!"
  objs="$objs $here/$f.o"
done
failed=0
for pid in $pids; do
  wait "$pid" || failed=1
done
if [ "$failed" -ne 0 ]; then
  echo "build.sh: a compile failed; libtmb_hip.so was not relinked" >&2
  exit 1
fi
for f in $units; do
  [ -s "$here/$f.o" ] || { echo "build.sh: $f.o missing" >&2; exit 1; }
done
rm -f "$here/libtmb_hip.so"
"$HIPCC" --offload-arch=gfx950 -shared -fPIC $objs -o "$here/libtmb_hip.so"
echo "built $here/libtmb_hip.so"
