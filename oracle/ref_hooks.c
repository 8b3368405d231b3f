/*
 * Embedder hook that the reference ukernels leave to their user
 * (runtime/src/iree/builtins/ukernel/common.h:307-308): called when one of
 * their debug assertions fails. Linked into oracle/_ref/libiree_uk_ref.so
 * only. Test infrastructure, not product code.
 */
#include <stdio.h>
#include <stdlib.h>

void iree_uk_assert_fail(const char* file, int line, const char* function,
                         const char* condition) {
  fprintf(stderr, "%s:%d: %s: assertion failed: %s\n", file, line, function,
          condition);
  fflush(stderr);
  abort();
}
