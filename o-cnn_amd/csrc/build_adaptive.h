// Interface between the octree builder and its second stage for octrees that carry
// a signal at every depth (node_feature) or are trimmed where a planar patch fits
// (adaptive): Octree::build, octree/octree/octree.cpp:96-120.
#pragma once

#include "ocnn_common.h"

namespace ocnn {

struct AdaptiveInput {
  char* blob0;          // device: first-stage octree (one cloud, or a batch in merged layout:
                        //         octree index in the top 16 bits of the keys, child links
                        //         counted over the batch), raw Morton keys, finest-level signal
                        //         normals | displacement | features | average points
  int merged;           // 0: single-octree blob out; 1: octree_batch blob out (neighbour tables)
  Info info0;           // its header (host)
  int ch_normal, ch_feature, ch_dis, has_pt, has_label;
  ocnn_build_params params;   // what the caller asked for
};

// Computes the all-depth signals, optionally extrapolates and trims, and serializes the
// final octree into memory obtained from `alloc` (scratch memory comes from `alloc` too;
// the caller keeps every allocation alive until the stream has finished).  One
// device-to-host copy (the trimmed node counts) is waited for.
int adaptive_finish(const AdaptiveInput& in, ocnn_alloc_fn alloc, void* alloc_ctx, void* info_out,
    void** blob_out, hipStream_t stream);

}  // namespace ocnn
