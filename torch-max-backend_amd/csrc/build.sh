#!/bin/sh
# Builds libtmb_hip.so for gfx950 next to this script. Usage: sh build.sh [extra hipcc flags]
# Every object is rebuilt from its source; a failed compile stops the build before the link, so a
# stale object can never end up in the library.
# TMB_VARIANT=name builds a second library beside it, libtmb_hip_name.so, from objects of its own
# (build_name/), e.g. a diagnostic build:  TMB_VARIANT=diag2 sh build.sh -DTMB_GEMM_DIAG=2
# (load it with TORCH_MOJO_BACKEND_HIP_LIBRARY=<path>).
set -e
here="$(cd "$(dirname "$0")" && pwd)"
objdir="$here"
libname="libtmb_hip.so"
if [ -n "$TMB_VARIANT" ]; then
  objdir="$here/build_$TMB_VARIANT"
  libname="libtmb_hip_$TMB_VARIANT.so"
  mkdir -p "$objdir"
fi
HIPCC="${HIPCC:-/opt/rocm/bin/hipcc}"
FLAGS="--offload-arch=gfx950 -O3 -std=c++17 -fPIC -Wno-inline-asm -Xclang -target-feature -Xclang -packed-fp32-ops"
units="softmax layer_norm reduce reduce_cols gemm attention attention_bwd backward misc"
objs=""
pids=""
for f in $units; do
  rm -f "$objdir/$f.o"
  "$HIPCC" $FLAGS "$@" -c "$here/$f.hip" -o "$objdir/$f.o" &
  pids="$pids $!"
  objs="$objs $objdir/$f.o"
done
failed=0
for pid in $pids; do
  wait "$pid" || failed=1
done
if [ "$failed" -ne 0 ]; then
  echo "build.sh: a compile failed; $libname was not relinked" >&2
  exit 1
fi
for f in $units; do
  [ -s "$objdir/$f.o" ] || { echo "build.sh: $f.o missing" >&2; exit 1; }
done
rm -f "$here/$libname"
"$HIPCC" --offload-arch=gfx950 -shared -fPIC $objs -o "$here/$libname"
echo "built $here/$libname"
