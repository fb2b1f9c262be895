#!/bin/bash
# Rebuilds tests/golden/ck_tile_host_golden.bin from ck_tile's host reference functions (headers under /opt/rocm/include).
# Needs hipcc; run from anywhere.  The fixture it writes is committed; tests only read the fixture.
set -e
here="$(cd "$(dirname "$0")" && pwd)"
tmp="$(mktemp -d)"
hipcc -std=c++20 -O1 --offload-arch=gfx950 -ffp-contract=off "$here/ck_tile_host_golden.cpp" -o "$tmp/gen"
"$tmp/gen" "$here/ck_tile_host_golden.bin"
rm -rf "$tmp"
ls -la "$here/ck_tile_host_golden.bin"
