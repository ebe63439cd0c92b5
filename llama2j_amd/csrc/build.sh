#!/bin/sh
# Builds llama2j_amd/libllama2j_hip.so for gfx950: every translation unit is compiled on its own (in parallel), then linked.
# Packed-fp32 instruction selection is switched off for the device code (-target-feature -packed-fp32-ops).  The flag also
# reaches each file's host pass, whose x86 back end answers "'-packed-fp32-ops' is not a recognized feature for this
# target (ignoring feature)": that one line is dropped from the output, everything else is shown.
here="$(cd "$(dirname "$0")" && pwd)"
out="$here/../libllama2j_hip.so"
obj="$here/build"
mkdir -p "$obj"
FLAGS="-O3 -std=c++17 --offload-arch=gfx950 -fPIC -Xclang -target-feature -Xclang -packed-fp32-ops -Wall -Wno-unused-function $L2J_EXTRA_FLAGS"
pids=""
for f in l2j_context.hip l2j_forward.hip l2j_sampler.hip l2j_batch.hip host_io.cpp host_tokenizer.cpp; do
    ( hipcc $FLAGS -c "$here/$f" -o "$obj/${f%.*}.o" 2> "$obj/${f%.*}.log"; echo $? > "$obj/${f%.*}.rc" ) &
    pids="$pids $!"
done
wait $pids
rc=0
for f in l2j_context l2j_forward l2j_sampler l2j_batch host_io host_tokenizer; do
    grep -v "'-packed-fp32-ops' is not a recognized feature for this target" "$obj/$f.log" >&2
    [ "$(cat "$obj/$f.rc")" = "0" ] || rc=1
done
[ $rc = 0 ] || { echo "build failed" >&2; exit 1; }
hipcc --offload-arch=gfx950 -shared -fPIC -o "$out" "$obj"/l2j_context.o "$obj"/l2j_forward.o "$obj"/l2j_sampler.o "$obj"/l2j_batch.o \
    "$obj"/host_io.o "$obj"/host_tokenizer.o -lpthread || exit 1
echo "built $out"
