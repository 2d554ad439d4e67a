#!/bin/sh
# Regenerates abi_constants.txt from the reference's own C headers (header-only, no library needed).
# Usage: tests/golden/make_abi_constants.sh [/root/reference]
set -e
here=$(dirname "$0")
ref=${1:-/root/reference}
gcc -std=c11 -I"$ref/src/nvcv/src/include" "$here/abi_constants.c" -o /tmp/abi_constants_ref
/tmp/abi_constants_ref > "$here/abi_constants.txt"
