#!/bin/sh
# Regenerates the JSON fixtures in this directory from the reference's own C (build container only).
set -e
here=$(cd "$(dirname "$0")" && pwd)
root=$(cd "$here/../.." && pwd)
REF=${REF:-/root/reference}
make -C "$root/oracle" ref REF="$REF"
gcc -O2 -std=c11 -I"$REF/native" -o "$root/oracle/_ref/make_golden" "$here/make_golden.c" \
    -L"$root/oracle/_ref" -lref -Wl,-rpath,"$root/oracle/_ref" -lm
"$root/oracle/_ref/make_golden" "$here"
gcc -O2 -std=c11 -I"$REF/native" -o "$root/oracle/_ref/make_golden_xs_m" "$here/make_golden_xs_m.c" \
    -L"$root/oracle/_ref" -lref -Wl,-rpath,"$root/oracle/_ref" -lm
"$root/oracle/_ref/make_golden_xs_m" "$here"
