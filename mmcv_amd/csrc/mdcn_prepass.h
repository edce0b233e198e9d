// Pre-pass kernels of the fused path: input re-layout and weight repack.
#pragma once

#include "mdcn_common.h"

namespace mdcn {

// NCHW input -> zero-bordered slab-major copy xt[N][Cin/KC][H+2][W+2][KC], KC =
// 128 bytes of channels per pixel and slab.  The one-pixel zero border makes
// every bilinear corner of an in-range position a plain load: a corner outside
// the image reads a stored zero, which is exactly the per-corner rule of the
// reference sampler (mmcv/ops/csrc/pytorch/cpu/modulated_deform_conv.cpp:17-27).
//
// One block moves one slab of 128 consecutive pixels of one padded row through
// LDS.  Reads run along W in 32-bit words (two 16-bit pixels or one fp32 pixel,
// a wave takes 256 contiguous bytes of one channel row); writes are 16 bytes per
// lane, a wave covering 1 KiB of contiguous output.  The block's pixels are
// padded columns 1+128*xc .. 128+128*xc, i.e. source columns 128*xc .. , so the
// word reads are aligned; column 0 of the border is written by block xc == 0.
template <typename E>
__global__ __launch_bounds__(256) void relayout_kernel(Geom g, const E *__restrict__ in,
                                                       E *__restrict__ xt, int n_xchunks,
                                                       int words_ok) {
  constexpr int KC = 128 / (int)sizeof(E);
  constexpr int EPW = 4 / (int)sizeof(E);   // elements per 32-bit word
  constexpr int ROWW = 33;                  // LDS words per pixel: 128 bytes + 4 of padding
  __shared__ uint32_t tile[128 * ROWW];

  int b = blockIdx.x;
  const int xc = b % n_xchunks;
  b /= n_xchunks;
  const int slabs_total = g.Cin / KC;
  const int slab = b % slabs_total;
  b /= slabs_total;
  const int yp = b % g.Hp;
  const int n = b / g.Hp;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const bool row_inside = (yp >= 1) && (yp <= g.H);

  if (row_inside) {
    // 64 row segments (KC channels x 128/(64*EPW) parts), 16 per wave
#pragma unroll 4
    for (int it = 0; it < 16; ++it) {
      const int seg = wave + 4 * it;
      const int c = seg % KC;
      const int part = seg / KC;                      // fp32: two halves of 64 pixels
      const int lp = (part * 64 + lane) * EPW;        // first local pixel of the word
      const int x = xc * 128 + lp;
      const E *src = in + (((long)n * g.Cin + slab * KC + c) * g.H + (yp - 1)) * g.W + x;
      if (EPW == 2) {
        uint32_t word = 0;
        if (words_ok) {
          if (x < g.W) word = *(const uint32_t *)src;  // W even: x + 1 < W too
        } else {
          uint32_t lo = 0, hi = 0;
          if (x < g.W) lo = *(const uint16_t *)src;
          if (x + 1 < g.W) hi = *((const uint16_t *)src + 1);
          word = lo | (hi << 16);
        }
        uint16_t *t16 = (uint16_t *)tile;
        t16[lp * (ROWW * 2) + c] = (uint16_t)(word & 0xffffu);
        t16[(lp + 1) * (ROWW * 2) + c] = (uint16_t)(word >> 16);
      } else {
        uint32_t word = 0;
        if (x < g.W) word = *(const uint32_t *)src;
        tile[lp * ROWW + c] = word;
      }
    }
  }
  __syncthreads();
  unsigned char *dst_row =
      (unsigned char *)xt + ((((long)n * slabs_total + slab) * g.Hp + yp) * g.Wp) * 128;
#pragma unroll
  for (int it = 0; it < 4; ++it) {
    const int u = tid + 256 * it;
    const int lp = u >> 3, q = u & 7;
    const int xp = xc * 128 + 1 + lp;
    if (xp < g.Wp) {
      uint4 v = make_uint4(0u, 0u, 0u, 0u);
      if (row_inside) {
        const uint32_t *t = tile + lp * ROWW + q * 4;
        v = make_uint4(t[0], t[1], t[2], t[3]);
      }
      *(uint4 *)(dst_row + (long)xp * 128 + q * 16) = v;
    }
  }
  if (xc == 0 && tid < 8) *(uint4 *)(dst_row + tid * 16) = make_uint4(0u, 0u, 0u, 0u);
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
