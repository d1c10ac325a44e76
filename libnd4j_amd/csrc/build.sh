#!/bin/bash
# Builds libnd4j_amd.so (gfx950) in-tree from the sources in this directory.  Usage: build.sh [--force] [-jN]
# (--force recompiles every object; otherwise make rebuilds what is out of date)
set -e
cd "$(dirname "$0")"
JOBS=-j8
FORCE=
for a in "$@"; do
  case "$a" in
    --force) FORCE=-B ;;
    -j*) JOBS=$a ;;
  esac
done
OUT=../libnd4j_amd.so
OBJ=build
mkdir -p $OBJ
HIPFLAGS="--offload-arch=gfx950 -O3 -std=c++17 -fPIC -ffp-contract=off -fhip-fp32-correctly-rounded-divide-sqrt -fvisibility=hidden -Xclang -target-feature -Xclang -packed-fp32-ops -Wno-unused-command-line-argument"
SRCS="transform.hip pairwise.hip broadcast.hip scalar.hip reduce.hip reduce3.hip special.hip wholearray.hip datamove.hip indexreduce.hip summarystats.hip random.hip native_ops.cpp native_reduce.cpp native_random.cpp native_special.cpp native_whole.cpp native_stubs.cpp runtime.cpp c_api.cpp"
cat > $OBJ/Makefile <<MK
OBJS := \$(addsuffix .o,\$(basename $SRCS))
all: ../$OUT
../$OUT: \$(OBJS)
	hipcc --offload-arch=gfx950 -shared -fPIC -o \$@ \$(OBJS)
# an object is rebuilt when a header it includes has changed (the compiler writes the list beside it: -MMD)
%.o: ../%.hip
	hipcc $HIPFLAGS -MMD -MP -c \$< -o \$@ 2>&1 | grep -v "packed-fp32-ops' is not a recognized feature" || true
	test -f \$@
%.o: ../%.cpp
	hipcc $HIPFLAGS -MMD -MP -x hip -c \$< -o \$@ 2>&1 | grep -v "packed-fp32-ops' is not a recognized feature" || true
	test -f \$@
-include \$(OBJS:.o=.d)
MK
make -C $OBJ $JOBS $FORCE all
