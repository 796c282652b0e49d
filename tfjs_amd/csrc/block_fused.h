// The whole-block kernel (block_fused.hip): arguments and tiling.
#pragma once

#include <stddef.h>

namespace tfhip {

struct BlockArgs {
  const float *x, *w1t, *b1, *w2, *b2, *w3t, *b3, *res;
  float *y;
  int batch, in_h, in_w, cin, c, n_out;   // x [batch,in_h,in_w,cin]; c mid channels; y [batch,out_h,out_w,n_out]
  int stride, pad_top, pad_left, out_h, out_w;
  float cap;                              // upper clamp of the two activations: 6 (relu6) or +inf (relu)
  // tiling (plan_block)
  int rows, chunks_h;                     // output rows per workgroup, workgroups per image
  int erows, ecols;                       // expanded tile with halo: rows of the tallest chunk, columns
  int slices, nb, mbp, team;              // mid-channel slices of 64; blocks of 16 output channels; blocks of 16
                                          // output pixels; waves that share an expansion pixel block
  unsigned x_bytes, w1t_bytes, w3t_bytes;
};

bool plan_block(BlockArgs &g, size_t *lds_bytes);
int launch_block_kernel(const BlockArgs &g, size_t lds_bytes);

}  // namespace tfhip
