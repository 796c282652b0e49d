// The register-streaming pointwise + depthwise kernel (expand_dw_stream.hip): arguments,
// tiling and launch, used by the entry points in expand_dw.hip.
#pragma once

#include <stddef.h>

namespace tfhip {

// Tap k = (fr * f_w + fs) * xc + ch of a first-stage filter over few input channels: row / column
// relative to a window's top-left input element, and byte offset from it (rows beyond the filter's
// taps: a row no image has).
constexpr int kMaxStemTaps = 36;
struct StemTaps {
  int dh[kMaxStemTaps], dw[kMaxStemTaps];
  unsigned off_bytes[kMaxStemTaps];
};

struct ExpandDwStreamArgs {
  const float *x, *w1, *b1, *w2, *b2;
  float *y;
  int batch, in_h, in_w, cin, c;   // x [batch, in_h, in_w, cin]; expanded [batch, in_h, in_w, c]
  int stride, pad_top, pad_left, out_h, out_w;
  float cap;                       // upper clamp of both activations: 6 (relu6) or +inf (relu)
  // tiling (plan_expand_dw_stream)
  int strip_w, strips;             // output columns per wavefront, wavefronts along a row
  int rows, chunks_h;              // output rows per wavefront, wavefronts along the rows
  int ahead;                       // rows ahead of their use the inputs are fetched (2 or 4)
  int cblocks, ncb;                // blocks of 16 expanded channels, and how many of them a wavefront takes (1 or 2)
  long long waves;                 // batch x chunks_h x strips x ceil(cblocks / ncb)
  unsigned x_bytes;
  int through;                     // an image of the result fits 32-bit offsets: written through a descriptor
  // first stage a convolution over few input channels instead of a 1x1 one (k_steps > 0): x is
  // [batch, xh, xw, xc], the "expanded" tensor [batch, in_h, in_w, c] is its output; k filter taps
  int xh, xw, xc, conv_stride, conv_pad_top, conv_pad_left, k, k_steps;
};

bool expand_dw_stream_takes_k(int cin);
bool plan_expand_dw_stream(ExpandDwStreamArgs &g);
int launch_expand_dw_stream(const ExpandDwStreamArgs &g);
int launch_stem_dw_stream(const ExpandDwStreamArgs &g, const StemTaps &taps);

}  // namespace tfhip
