#!/bin/bash
# Host-side sanitizer pass, CPU only (no GPU is touched): the C oracle and the
# host code of libwarpctct_hip.so (argument checks, workspace carving, the
# timing hook, the status word's bookkeeping) are rebuilt with
# AddressSanitizer + UndefinedBehaviorSanitizer into a scratch directory, and
# the CPU tests that exercise them run against those builds.  Device code is
# compiled as usual (sanitizers for it are not available here).
#
#   bash tests/run_host_sanitizers.sh
set -euo pipefail
ROOT="$(cd "$(dirname "${BASH_SOURCE[0]}")/.." && pwd)"
OUT="$(mktemp -d /tmp/warpctct_sanitize.XXXXXX)"
trap 'rm -rf "$OUT"' EXIT
LLVM=/opt/rocm/llvm/bin
SAN="-fsanitize=address,undefined -fno-omit-frame-pointer -fno-sanitize-recover=undefined"

# one sanitizer runtime for both libraries: clang's (hipcc's host compiler)
"$LLVM/clang" -O1 -g -fPIC -fopenmp -fno-fast-math -Wall -Wextra $SAN -shared-libasan -shared \
    -o "$OUT/libctct_oracle.so" "$ROOT/oracle/ctct_oracle.c" -lm

SRCS="api lattice lattice_lin units dense_grad simple logmm logits profile status"
OBJS=""
for s in $SRCS; do
    /opt/rocm/bin/hipcc -O1 -g -std=c++17 -fPIC --offload-arch=gfx950 \
        -Xclang -target-feature -Xclang -packed-fp32-ops -Wno-unused-command-line-argument \
        -Xarch_host -fsanitize=address -Xarch_host -fsanitize=undefined \
        -Xarch_host -fno-omit-frame-pointer -Xarch_host -fvisibility=hidden \
        -I"$ROOT/include" -I"$ROOT/warp-ctct_amd/csrc" \
        -c "$ROOT/warp-ctct_amd/csrc/$s.hip" -o "$OUT/$s.o" 2> "$OUT/$s.log" || { cat "$OUT/$s.log"; exit 1; }
    OBJS="$OBJS $OUT/$s.o"
done
/opt/rocm/bin/hipcc --offload-arch=gfx950 -shared -fPIC -fsanitize=address,undefined -shared-libasan \
    -Wl,--version-script="$ROOT/warp-ctct_amd/csrc/exports.map" -o "$OUT/libwarpctct_hip.so" $OBJS

RUNTIME="$("$LLVM/clang" -print-file-name=libclang_rt.asan-x86_64.so)"
cd "$ROOT"
# (python itself is not instrumented: leak reports would be its own allocations)
LD_PRELOAD="$RUNTIME" ASAN_OPTIONS=detect_leaks=0:abort_on_error=1 UBSAN_OPTIONS=print_stacktrace=1 \
WARPCTCT_HIP_LIB="$OUT/libwarpctct_hip.so" CTCT_ORACLE_LIB="$OUT/libctct_oracle.so" \
    python -m pytest tests/test_abi_cpu.py tests/test_oracle_pins.py -x -q -m "not gpu"
