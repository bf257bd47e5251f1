#!/bin/bash
# Builds oracle/_ref/libtsref.so from the reference's own sources where they lie under
# /root/reference (nothing is copied): the mask / layer-schedule / RoPE / e4m3 code that compiles with
# stock g++.  The attention arithmetic itself (gpt_cpu.cpp, cpu_infer.cpp) needs the CUDA SDK
# headers and is not buildable here.  Output only into oracle/_ref/.
set -e
HERE="$(cd "$(dirname "$0")" && pwd)"
R=/root/reference/code
[ -d "$R" ] || { echo "no reference checkout at $R; keeping any prebuilt oracle/_ref"; exit 0; }
OUT="$HERE/_ref"
mkdir -p "$OUT/obj"
CXX="g++ -std=c++17 -O1 -mavx2 -mfma -mf16c -fPIC -w -I$R"
$CXX -c "$HERE/ref_wrap.cpp" -o "$OUT/obj/ref_wrap.o"
for f in gpt/att/att.cpp gpt/att/rope.cpp gpt/att/sliding_window.cpp gpt/att/nodes_batch.cpp gpt/model_params/model_dim.cpp lib/config/config.cpp; do
  $CXX -I"$R/$(dirname $f)" -c "$R/$f" -o "$OUT/obj/$(basename $f .cpp).o"
done
# util/ has a string.h of its own: keep it off the <...> search path
for f in util/string.cpp util/tools.cpp; do
  $CXX -iquote "$R/util" -c "$R/$f" -o "$OUT/obj/$(basename $f .cpp).o"
done
g++ -shared -o "$OUT/libtsref.so" "$OUT"/obj/*.o
rm -rf "$OUT/obj"
echo "built $OUT/libtsref.so"
