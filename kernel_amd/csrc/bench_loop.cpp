// Tight host loop over moe_a2a_forward for bench.py: n steps launched back to back from C, so
// the GPU queue never runs dry between steps (an interpreter cannot issue three launches in
// the ~25 us a small step takes).  Steps alternate between two argument sets, the two buffer
// sets of the host class.  Nothing here is needed to use the library.
#include <stddef.h>
#include <stdint.h>

#include "moe_a2a.h"

extern "C" {

// Launches n steps: step i uses sets[i & 1].  Returns the first non-zero code, else 0.
int moe_a2a_bench_steps(int n, const moe_a2a_forward_args* set0, const moe_a2a_forward_args* set1) {
  for (int i = 0; i < n; ++i) {
    int rc = moe_a2a_forward_packed((i & 1) ? set1 : set0);
    if (rc) return rc;
  }
  return 0;
}

}  // extern "C"
