// Direct DCNv2 forward: one thread per output element, any shape, NCHW input
// read in place.  It covers the shapes the fused MFMA kernel does not
// (channel counts that are not a multiple of its K slab, very large kernels)
// and gives the tests a second, independent device implementation.
#pragma once

#include "mdcn_common.h"

namespace mdcn {

template <typename E>
__global__ __launch_bounds__(256) void direct_kernel(
    Geom g, const E *__restrict__ input, OffMaskView om, const E *__restrict__ weight,
    const E *__restrict__ bias, E *__restrict__ output, long total) {
  const long plane_out = (long)g.Ho * g.Wo;
  const long plane_in = (long)g.H * g.W;
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    const int wo = (int)(idx % g.Wo);
    const int ho = (int)((idx / g.Wo) % g.Ho);
    const int co = (int)((idx / plane_out) % g.Cout);
    const int n = (int)(idx / (plane_out * g.Cout));
    const int grp = co / g.cout_g;
    const long pix = (long)ho * g.Wo + wo;

    float acc = 0.0f;
    for (int cl = 0; cl < g.cin_g; ++cl) {
      const int c = grp * g.cin_g + cl;
      const int dgi = c / g.ch_per_dg;
      const E *im = input + ((long)n * g.Cin + c) * plane_in;
      const E *off = (const E *)om.off + (long)n * om.off_n + pix * om.off_px +
                     (long)(dgi * 2 * g.taps) * om.off_ch;
      const E *msk = (const E *)om.msk + (long)n * om.msk_n + pix * om.msk_px +
                     (long)(dgi * g.taps) * om.msk_ch;
      const E *wrow = weight + ((long)co * g.cin_g + cl) * g.taps;
      for (int i = 0; i < g.kh; ++i) {
        for (int j = 0; j < g.kw; ++j) {
          const int tap = i * g.kw + j;
          const float dy = to_f32(off[(long)(2 * tap) * om.off_ch]);
          const float dx = to_f32(off[(long)(2 * tap + 1) * om.off_ch]);
          const float m = mask_value<E>(msk[(long)tap * om.msk_ch], om.logit);
          const TapSample s =
              make_tap_sample(ho * g.sh - g.ph + i * g.dh,
                              wo * g.sw - g.pw + j * g.dw, dy, dx, m, g.H, g.W);
          if (!s.inside) continue;
          const int y1 = s.y0 + 1, x1 = s.x0 + 1;
          float v = 0.0f;
          if (s.y0 >= 0 && s.x0 >= 0) v += s.w00 * to_f32(im[s.y0 * g.W + s.x0]);
          if (s.y0 >= 0 && x1 <= g.W - 1) v += s.w01 * to_f32(im[s.y0 * g.W + x1]);
          if (y1 <= g.H - 1 && s.x0 >= 0) v += s.w10 * to_f32(im[y1 * g.W + s.x0]);
          if (y1 <= g.H - 1 && x1 <= g.W - 1) v += s.w11 * to_f32(im[y1 * g.W + x1]);
          acc += to_f32(wrow[tap]) * v;
        }
      }
    }
    if (bias) acc += to_f32(bias[co]);
    output[idx] = from_f32<E>(acc);
  }
}

}  // namespace mdcn
