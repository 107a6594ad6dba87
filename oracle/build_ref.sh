#!/bin/bash
# Compile the reference's own CPU path for the ZB step from its sources where they lie:
#   mom6_zb/zb_host.f90 (host: field synthesis, stencil packing, de-scaling, corner interpolation)
#   mom6_zb/fwd_native_zb.f90 (the shipped ANN_apply; RKVAL=4 selects single precision, as the
#   reference's run_zb_native.sh:7 does with sed)
# Output goes to oracle/_ref/ only (git-ignored).  Contraction is switched off so that fp32
# expressions round once per operation, as in the reference's `-fmad=false` device code.
set -e
here="$(cd "$(dirname "$0")" && pwd)"
REF="${FORTIS_REFERENCE:-/root/reference}"
FLANG="${FLANG:-/opt/rocm/lib/llvm/bin/flang}"
if [ ! -d "$REF/mom6_zb" ]; then echo "build_ref: $REF/mom6_zb not present, skipping"; exit 0; fi
if [ ! -x "$FLANG" ]; then echo "build_ref: no flang at $FLANG, skipping"; exit 0; fi
mkdir -p "$here/_ref"
cd "$here/_ref"
"$FLANG" -O2 -ffp-contract=off -cpp -DRKVAL=4 "$REF/mom6_zb/fwd_native_zb.f90" "$REF/mom6_zb/zb_host.f90" -o zb_native4
rm -f fwd_native_zb_mod.mod
echo "build_ref: built $here/_ref/zb_native4"
