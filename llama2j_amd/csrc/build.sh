#!/bin/sh
# Builds llama2j_amd/libllama2j_hip.so for gfx950.  Packed-fp32 instruction selection is switched off.
set -e
here="$(cd "$(dirname "$0")" && pwd)"
out="$here/../libllama2j_hip.so"
hipcc -O3 -std=c++17 --offload-arch=gfx950 -fPIC -shared \
    -Xclang -target-feature -Xclang -packed-fp32-ops \
    -Wall -Wno-unused-function \
    -o "$out" "$here/l2j_hip.hip" "$here/host_io.cpp" "$here/host_tokenizer.cpp" -lpthread
echo "built $out"
