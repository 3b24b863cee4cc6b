#!/bin/sh
# oracle/_ref/libfm_ref.so: a checker compiled from the reference's own sources.
#
# infer.m as a whole is an Objective-C unit that needs Foundation / Metal / Accelerate /
# GCD (finchmoe/infer.m:45-69) and cannot be compiled here.  The CPU functions of the
# path, though, are plain dependency-free C99 inside it: lines 686-702 (bf16 widening)
# and 1575-1881 (fp16 widening, get_scale_min_k4, gguf_dequant_row, gguf_cpu_matvec,
# cpu_dequant_matvec incl. the raw-BF16 branch, cpu_rms_norm, cpu_swiglu, cpu_softmax,
# cpu_topk, cpu_normalize_weights, cpu_vec_madd).  This recipe cuts those two ranges out
# of the file where it lies into a temporary directory, compiles ref_wrap.c around them
# (four libc headers, no stand-ins) and keeps only the shared library.  The cut itself
# is deleted: no reference text is left in the tree or travels anywhere.
#
# The line ranges are checked against the function names they must contain, so a
# reference tree with shifted lines fails here instead of building something else.
set -e
REF=${FINCH_REFERENCE:-/root/reference}/finchmoe/infer.m
HERE=$(cd "$(dirname "$0")" && pwd)
if [ ! -f "$REF" ]; then
    echo "oracle/_ref: $REF not present, skipped (the prebuilt library is used if there is one)"
    exit 0
fi
TMP=$(mktemp -d)
trap 'rm -rf "$TMP"' EXIT
sed -n '686,702p;1575,1881p' "$REF" > "$TMP/ref_cpu_body.inc"
for fn in bf16_to_f32 fp16_to_f32 get_scale_min_k4 gguf_dequant_row gguf_cpu_matvec \
          cpu_dequant_matvec cpu_rms_norm cpu_swiglu cpu_softmax cpu_topk \
          cpu_normalize_weights cpu_vec_madd cpu_argmax; do
    if ! grep -q "^static .*[ *]$fn(" "$TMP/ref_cpu_body.inc"; then
        echo "oracle/_ref: $fn not found in the cut (reference lines moved?)" >&2
        exit 1
    fi
done
mkdir -p "$HERE/_ref"
# -O2 as the reference's own Makefile builds its CPU path; -ffp-contract=off so that the
# library computes what the C text says on every x86-64 host (clang on arm64 contracts
# a*b+c upstream; none of the compared functions has a result that contraction changes,
# except the matvec accumulations, which are compared within a tolerance for that reason)
${CC:-gcc} -O2 -std=gnu99 -fPIC -shared -fvisibility=hidden -ffp-contract=off -Wall \
    -DREF_BODY="\"$TMP/ref_cpu_body.inc\"" -o "$HERE/_ref/libfm_ref.so" "$HERE/ref_wrap.c" -lm
echo "oracle/_ref/libfm_ref.so built from $REF"
