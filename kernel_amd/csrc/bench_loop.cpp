// Tight host loop over moe_a2a_forward for bench.py: n steps launched back to back from C, so
// the GPU queue never runs dry between steps (an interpreter cannot issue three launches in
// the ~25 us a small step takes).  Steps alternate between two argument sets, the two buffer
// sets of the host class.  Nothing here is needed to use the library.
#include <stddef.h>
#include <stdint.h>

#include "moe_a2a.h"

extern "C" {

struct moe_a2a_forward_args {
  const void* x;
  const int32_t* indices;
  const float* weights;
  const int32_t* rank_start;
  int src_rank, T, K, E, W, H, max_recv, in_type, out_type, fp8_dispatch, stub_kind, combine_mode, fuse_route,
      fuse_stub;
  int32_t *counts, *offsets, *slot_of_entry, *src_of_slot, *meta, *status;
  void* disp;
  float* disp_scale;
  void* expert_y;
  void* out;
  void* workspace;
  size_t workspace_bytes;
  moe_a2a_stream_t stream;
};

static int run_one(const moe_a2a_forward_args* a) {
  return moe_a2a_forward(a->x, a->indices, a->weights, a->rank_start, a->src_rank, a->T, a->K, a->E, a->W, a->H,
                         a->max_recv, a->in_type, a->out_type, a->fp8_dispatch, a->stub_kind, a->combine_mode, a->fuse_route,
                         a->fuse_stub, a->counts, a->offsets, a->slot_of_entry, a->src_of_slot, a->meta, a->status,
                         a->disp, a->disp_scale, a->expert_y, a->out, a->workspace, a->workspace_bytes, a->stream);
}

// Launches n steps: step i uses sets[i & 1].  Returns the first non-zero code, else 0.
int moe_a2a_bench_steps(int n, const moe_a2a_forward_args* set0, const moe_a2a_forward_args* set1) {
  for (int i = 0; i < n; ++i) {
    int rc = run_one((i & 1) ? set1 : set0);
    if (rc) return rc;
  }
  return 0;
}

}  // extern "C"
