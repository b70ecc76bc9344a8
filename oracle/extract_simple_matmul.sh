#!/bin/sh
# Extracts the emitted C kernel that the reference quotes as a comment in
# morello/examples/simple_matmul_x86.rs (the block starting "void kernel(" and ending at the
# closing brace in column 0 of the comment) into $2/simple_matmul_{u32,f32}.c.
# TEST INFRASTRUCTURE ONLY; outputs stay under oracle/_ref (git-ignored).
set -e
REF="$1"; OUT="$2"
SRC="$REF/morello/examples/simple_matmul_x86.rs"
body=$(sed -n '/^    \/\/   void kernel(/,/^    \/\/   }$/p' "$SRC" | sed 's/^    \/\/   //')
{
  echo '#include <stdint.h>'; echo '#include <string.h>'
  echo "$body" | sed 's/void kernel(/void ref_simple_matmul_u32(/'
} > "$OUT/simple_matmul_u32.c"
{
  echo '#include <stdint.h>'; echo '#include <string.h>'
  echo "$body" | sed 's/void kernel(/void ref_simple_matmul_f32(/; s/uint32_t/float/g'
} > "$OUT/simple_matmul_f32.c"
