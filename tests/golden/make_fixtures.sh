#!/bin/sh
# Regenerates the trimmed expected-output fixtures from a reference checkout.
REF=${1:-/root/reference}
cd "$(dirname "$0")"
for f in top_down_prec zero_out_local_decl test_where_precision test_log_stmt_format; do
  sed -n '/^ void /,$p' "$REF/test/operations/$f.c.expected" > "$f.proc.c.expected"
done
sed -n '3,$p' "$REF/arrayjit/test/test_zero_out_codegen.expected" > test_zero_out_codegen.proc.c.expected
sed -n '4,$p' "$REF/arrayjit/test/test_local_scope_init.expected" > test_local_scope_init.expected
# IR text goldens (`.ll`), whole files
for f in test/einsum/inline_permuted_view-c_fwd test/einsum/test_cse-cse_d_fwd test/operations/n3_fwd_with_prec-unoptimized \
         test/operations/top_down_prec-unoptimized test/operations/test_where_precision-unoptimized \
         test/operations/zero_out_local_decl-unoptimized; do
  cp "$REF/$f.ll.expected" "$(basename "$f").ll.expected"
done
