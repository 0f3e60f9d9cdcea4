#!/bin/bash
# Host-side AddressSanitizer + UndefinedBehaviorSanitizer pass over the C ABI's argument validation and launch-geometry code
# (no GPU sanitizer, no GPU run): compiles the library's sources with the HOST pass instrumented, links them with
# abi_driver.cpp into one executable under a temporary directory and runs it.   usage: bash tests/sanitize/run.sh [rounds]
set -e
here="$(cd "$(dirname "$0")" && pwd)"
root="$(cd "$here/../.." && pwd)"
# Q8_SAN_DIR: keep the instrumented objects there between runs (a source is recompiled when it or a header is newer)
if [ -n "$Q8_SAN_DIR" ]; then out="$Q8_SAN_DIR"; mkdir -p "$out"; else out="$(mktemp -d)"; trap 'rm -rf "$out"' EXIT; fi
HIPCC=${HIPCC:-/opt/rocm/bin/hipcc}
SAN="-Xarch_host -fsanitize=address -Xarch_host -fsanitize=undefined -Xarch_host -fno-sanitize-recover=undefined -Xarch_host -fno-omit-frame-pointer"
FLAGS="--offload-arch=gfx950 -O1 -g -std=c++17 -fPIC -Xclang -target-feature -Xclang -packed-fp32-ops"
pids=""
newest_header="$(ls -t "$root"/q8_kernels_amd/csrc/*.h "$root"/include/*.h | head -1)"
for f in api rows fused elementwise gemm attn; do
  src="$root/q8_kernels_amd/csrc/$f.hip"
  if [ -f "$out/$f.o" ] && [ "$out/$f.o" -nt "$src" ] && [ "$out/$f.o" -nt "$newest_header" ]; then continue; fi
  $HIPCC $FLAGS $SAN -c "$src" -o "$out/$f.o" 2> "$out/$f.log" &
  pids="$pids $!"
done
for p in $pids; do wait $p; done
clang=/opt/rocm/lib/llvm/bin/clang++
$clang -fsanitize=address -fsanitize=undefined -fno-sanitize-recover=undefined -g -O1 -std=c++17 -c "$here/abi_driver.cpp" -o "$out/abi_driver.o"
$HIPCC --offload-arch=gfx950 -fsanitize=address -fsanitize=undefined "$out"/*.o -o "$out/abi_driver"
ASAN_OPTIONS=detect_leaks=0:abort_on_error=1 UBSAN_OPTIONS=print_stacktrace=1:halt_on_error=1 "$out/abi_driver" "${1:-3000}"
