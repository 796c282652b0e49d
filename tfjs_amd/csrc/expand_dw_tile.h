// The channel-sliced pointwise + depthwise kernel (expand_dw_tile.hip): arguments,
// tiling and launch, used by the entry points in expand_dw.hip.
#pragma once

#include <stddef.h>

namespace tfhip {

struct ExpandDwTileArgs {
  const float *x, *w1, *b1, *w2, *b2;
  float *y;
  int batch, in_h, in_w, cin, c;   // x [batch, in_h, in_w, cin]; expanded [batch, in_h, in_w, c]
  int stride, pad_top, pad_left, out_h, out_w;
  float cap;                       // upper clamp of both activations: 6 (relu6) or +inf (relu)
  // tiling (plan_expand_dw_tile)
  int cs, slices;                  // expanded channels per workgroup, workgroups along the channels
  int rows, chunks_h;              // output rows per workgroup, workgroups along the rows
  int erows, ecols;                // expanded tile with halo: rows of the tallest chunk, columns
  unsigned x_bytes;
  int stream_out;                  // the result leaves as non-temporal stores (8 MB or more in all, or an image
                                   // beyond 32-bit offsets), else written through
};

bool expand_dw_tile_takes_k(int cin);
bool plan_expand_dw_tile(ExpandDwTileArgs &g, size_t *lds_bytes);
int launch_expand_dw_tile(const ExpandDwTileArgs &g, size_t lds_bytes);

}  // namespace tfhip
