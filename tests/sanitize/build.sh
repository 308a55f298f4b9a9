#!/bin/bash
# Host code of the library (everything but the HIP layer) compiled with AddressSanitizer and
# UndefinedBehaviorSanitizer and linked with format_driver.cc; objects and the program go to tests/sanitize/build.
set -e
HERE=$(cd "$(dirname "$0")" && pwd)
SRC=$HERE/../../alphasparse_amd/csrc
INC=$HERE/../../include
mkdir -p $HERE/build
for f in $SRC/*.cc; do
  b=$(basename $f .cc)
  [ $b = hip_layer ] && continue
  [ $HERE/build/$b.o -nt $f ] || g++ -std=c++17 -O1 -g -fno-omit-frame-pointer -fsanitize=address,undefined -fno-sanitize-recover=undefined -fPIC -I$SRC -I$INC -c $f -o $HERE/build/$b.o &
done
wait
/opt/rocm/bin/hipcc -std=c++17 -O2 -fPIC --offload-arch=gfx950 -Xclang -target-feature -Xclang -packed-fp32-ops -Wno-unused-command-line-argument -I$SRC -I$INC -c $SRC/hip_layer.cc -o $HERE/build/hip_layer.o 2>/dev/null
g++ -std=c++17 -O1 -g -fsanitize=address,undefined -I$INC $HERE/format_driver.cc $HERE/build/*.o -o $HERE/build/format_driver -L/opt/rocm/lib -lhiprtc -lamdhip64 -Wl,-rpath,/opt/rocm/lib
