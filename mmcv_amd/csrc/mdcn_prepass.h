// Pre-pass kernels of the fused path: input re-layout and weight repack.
#pragma once

#include "mdcn_common.h"

namespace mdcn {

// NCHW input -> zero-bordered slab-major copy xt[N][Cin/KC][H+2][W+2][KC]
// (KC channels = 64 bytes per pixel and slab).  The one-pixel zero border makes
// every bilinear corner of an in-range position a plain load: a corner outside
// the image reads a stored zero, which is exactly the per-corner rule of the
// reference sampler (mmcv/ops/csrc/pytorch/cpu/modulated_deform_conv.cpp:17-27).
//
// One block moves a 64-channel x 64-column tile of one padded row through LDS:
// reads run along W (contiguous in NCHW), writes along the KC channels of a
// pixel and on to the next pixel (contiguous in xt).
template <typename E, int KC>
__global__ __launch_bounds__(256) void relayout_kernel(
    Geom g, const E *__restrict__ in, E *__restrict__ xt, int n_xtiles,
    int n_ctiles) {
  __shared__ E tile[64][65];
  int b = blockIdx.x;
  const int xtile = b % n_xtiles;
  b /= n_xtiles;
  const int ctile = b % n_ctiles;
  b /= n_ctiles;
  const int yp = b % g.Hp;
  const int n = b / g.Hp;
  const int slabs_total = g.Cin / KC;

  const int tid = threadIdx.x;
  const bool row_inside = (yp >= 1) && (yp <= g.H);
  {
    const int xl = tid & 63;
    const int xp = xtile * 64 + xl;
    const bool col_inside = (xp >= 1) && (xp <= g.W);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int cl = (tid >> 6) + 4 * i;
      const int c = ctile * 64 + cl;
      E v = from_f32<E>(0.0f);
      if (row_inside && col_inside && c < g.Cin)
        v = in[(((long)n * g.Cin + c) * g.H + (yp - 1)) * g.W + (xp - 1)];
      tile[cl][xl] = v;
    }
  }
  __syncthreads();
  {
    // lanes run over the KC channels of a slab, then over pixels
    const int kc = tid % KC;
    constexpr int PX_PER_PASS = 256 / KC;
#pragma unroll
    for (int sl = 0; sl < 64 / KC; ++sl) {
      const int cl = sl * KC + kc;
      const int c = ctile * 64 + cl;
      const int slab = c / KC;
#pragma unroll
      for (int i = 0; i < 64 / PX_PER_PASS; ++i) {
        const int xl = tid / KC + PX_PER_PASS * i;
        const int xp = xtile * 64 + xl;
        if (xp < g.Wp && c < g.Cin)
          xt[((((long)n * slabs_total + slab) * g.Hp + yp) * g.Wp + xp) * KC + kc] = tile[cl][xl];
      }
    }
  }
}

// weight[Cout][Cin/G][kh][kw] -> wp[G][n_ctiles][nk][CT][KC]: for every
// group, Cout tile and K step (channel slab outer, tap inner) one dense
// CT x KC tile, K contiguous, zero rows past Cout/G.  The main kernel copies
// such a tile to LDS with straight 16-byte loads.
template <typename E>
__global__ __launch_bounds__(256) void pack_weight_kernel(
    Geom g, const E *__restrict__ w, E *__restrict__ wp, int CT, int KC,
    int n_ctiles, int slabs, long total) {
  const int nk = slabs * g.taps;
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    long r = idx;
    const int kc = (int)(r % KC);
    r /= KC;
    const int row = (int)(r % CT);
    r /= CT;
    const int ks = (int)(r % nk);
    r /= nk;
    const int ctile = (int)(r % n_ctiles);
    const int grp = (int)(r / n_ctiles);
    const int slab = ks / g.taps, tap = ks % g.taps;
    const int col = ctile * CT + row;  // output channel within the group
    E v = from_f32<E>(0.0f);
    if (col < g.cout_g) {
      const int co = grp * g.cout_g + col;
      const int cl = slab * KC + kc;
      v = w[((long)co * g.cin_g + cl) * g.taps + tap];
    }
    wp[idx] = v;
  }
}

}  // namespace mdcn
