// The offset/mask producer of ModulatedDeformConv2dPack: the plain convolution
// conv_offset (mmcv/ops/modulated_deform_conv.py:297-305,328) from Cin to
// 3 * deform_groups * kh * kw channels with the geometry of the deformable
// convolution itself.  It reads the same zero-bordered slab-major input copy as
// the main kernel and writes its result pixel-major, [pixel][CO_pad], so that the
// main kernel's table builder finds the 27 values of a pixel in one or two cache
// lines instead of 27.
#pragma once

#include "mdcn_common.h"
#include "mdcn_fused.h"

namespace mdcn {

struct OconvArgs {
  Geom g;
  const void *xt;     // zero-bordered slab-major input copy
  const void *owp;    // packed conv_offset weights, see pack_offset_weight_kernel
  const void *obias;  // (CO) or null
  void *raw;          // [N * Ho * Wo][CO_pad]
  long total_px;      // N * Ho * Wo
  int CO;             // 3 * DG * taps
  int CO_pad;         // CO rounded up to 32
  int slabs_total;    // Cin / KC
  int plane_px;       // Hp * Wp
};

// conv_offset weight (CO, Cin, kh, kw) -> MFMA B fragments: for every
// (slab, tap, ksub, 32-channel block) the 64 lanes' 16-byte operands back to
// back, i.e. one fully coalesced 1 KiB load per fragment.  Lane l holds output
// channel 32 * block + l % 32 and the input channels of 16-byte chunk
// 2 * ksub + l / 32 of the slab.  Rows past CO are zero.
template <typename E>
__global__ __launch_bounds__(256) void pack_offset_weight_kernel(Geom g, const E *__restrict__ ow,
                                                                 E *__restrict__ owp, int CO,
                                                                 int cof, long total) {
  constexpr int KC = 128 / (int)sizeof(E);
  constexpr int EPC = 16 / (int)sizeof(E);  // elements per 16-byte chunk
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    long r = idx;
    const int e = (int)(r % EPC);
    r /= EPC;
    const int lane = (int)(r % 64);
    r /= 64;
    const int blk = (int)(r % cof);
    r /= cof;
    const int ksub = (int)(r % 4);
    r /= 4;
    const int tap = (int)(r % g.taps);
    const int slab = (int)(r / g.taps);
    const int co = blk * 32 + (lane & 31);
    const int ch = slab * KC + (ksub * 2 + (lane >> 5)) * EPC + e;
    E v = from_f32<E>(0.0f);
    if (co < CO) v = ow[((long)co * g.Cin + ch) * g.taps + tap];
    owp[idx] = v;
  }
}

// Implicit GEMM raw[pixel][co] = sum_{c, tap} x[pixel + tap][c] * ow[co][c][tap] + ob[co].
// No LDS: the A operand of the MFMA (32 pixels x 16 bytes of channels) is loaded
// from the input copy as it lies, the B operand from the packed weights; each
// wave owns PXF blocks of 32 consecutive pixels and all COF blocks of 32 output
// channels.  A tap outside the one-pixel zero border (padding > 1) contributes a
// zero fragment.
template <typename E, int COF, int PXF>
__global__ __launch_bounds__(256) void oconv_kernel(OconvArgs a) {
  using TR = ElemTraits<E>;
  const Geom &g = a.g;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int frow = lane & 31;
  const int fhalf = lane >> 5;
  const int plane_out = g.Ho * g.Wo;
  const long p_wave = ((long)blockIdx.x * 4 + wave) * (32 * PXF);
  if (p_wave >= a.total_px) return;

  // this lane's pixel of each block: image base and top-left tap position in the copy
  long img_base[PXF];
  int by[PXF], bx[PXF];
#pragma unroll
  for (int pf = 0; pf < PXF; ++pf) {
    long p = p_wave + pf * 32 + frow;
    if (p >= a.total_px) p = a.total_px - 1;  // loads stay in range, nothing is stored
    const int n = (int)(p / plane_out);
    const int rem = (int)(p - (long)n * plane_out);
    const int ho = rem / g.Wo, wo = rem - ho * g.Wo;
    img_base[pf] = (long)n * a.slabs_total * a.plane_px;
    by[pf] = ho * g.sh - g.ph + 1;  // +1: coordinates of the bordered copy
    bx[pf] = wo * g.sw - g.pw + 1;
  }

  f32x16 acc[PXF][COF];
#pragma unroll
  for (int pf = 0; pf < PXF; ++pf)
#pragma unroll
    for (int cf = 0; cf < COF; ++cf)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[pf][cf][r] = 0.0f;

  const uint4 *xt = (const uint4 *)a.xt;
  const uint4 *owp = (const uint4 *)a.owp + lane;
  for (int slab = 0; slab < a.slabs_total; ++slab) {
    for (int ti = 0; ti < g.kh; ++ti) {
      for (int tj = 0; tj < g.kw; ++tj) {
        const int tap = ti * g.kw + tj;
        long pix[PXF];
        bool ok[PXF];
#pragma unroll
        for (int pf = 0; pf < PXF; ++pf) {
          const int y = by[pf] + ti * g.dh, x = bx[pf] + tj * g.dw;
          ok[pf] = (y >= 0) && (y < g.Hp) && (x >= 0) && (x < g.Wp);
          pix[pf] = ok[pf] ? img_base[pf] + (long)slab * a.plane_px + (long)y * g.Wp + x : 0;
        }
        const uint4 *wfrag = owp + (long)((slab * g.taps + tap) * 4) * COF * 64;
#pragma unroll
        for (int ksub = 0; ksub < 4; ++ksub) {
          uint4 af[PXF], bf[COF];
#pragma unroll
          for (int pf = 0; pf < PXF; ++pf) {
            af[pf] = xt[pix[pf] * 8 + ksub * 2 + fhalf];
            if (!ok[pf]) af[pf] = make_uint4(0u, 0u, 0u, 0u);
          }
#pragma unroll
          for (int cf = 0; cf < COF; ++cf) bf[cf] = wfrag[(ksub * COF + cf) * 64];
#pragma unroll
          for (int pf = 0; pf < PXF; ++pf)
#pragma unroll
            for (int cf = 0; cf < COF; ++cf) TR::mma(acc[pf][cf], af[pf], bf[cf]);
        }
      }
    }
  }

  // Accumulator block (A = pixels, B = channels): register r of lane l holds
  //   pixel = (r/4)*8 + (l/32)*4 + r%4,  channel = l%32.
  // Lanes 0..31 of one store cover the 32 consecutive channels of one pixel.
  E *raw = (E *)a.raw;
#pragma unroll
  for (int cf = 0; cf < COF; ++cf) {
    const int co = cf * 32 + frow;
    float b = 0.0f;
    if (a.obias && co < a.CO) b = to_f32(((const E *)a.obias)[co]);
#pragma unroll
    for (int pf = 0; pf < PXF; ++pf) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const long p = p_wave + pf * 32 + (r >> 2) * 8 + fhalf * 4 + (r & 3);
        if (p < a.total_px) raw[p * a.CO_pad + co] = from_f32<E>(acc[pf][cf][r] + b);
      }
    }
  }
}

// The same convolution for shapes the slab-major copy does not cover: one thread
// per output element, NCHW in, NCHW out.
template <typename E>
__global__ __launch_bounds__(256) void oconv_direct_kernel(Geom g, const E *__restrict__ input,
                                                           const E *__restrict__ ow,
                                                           const E *__restrict__ ob,
                                                           E *__restrict__ raw, int CO, long total) {
  const long plane_out = (long)g.Ho * g.Wo;
  const long plane_in = (long)g.H * g.W;
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    const int wo = (int)(idx % g.Wo);
    const int ho = (int)((idx / g.Wo) % g.Ho);
    const int co = (int)((idx / plane_out) % CO);
    const int n = (int)(idx / (plane_out * CO));
    float acc = 0.0f;
    for (int c = 0; c < g.Cin; ++c) {
      const E *im = input + ((long)n * g.Cin + c) * plane_in;
      const E *wrow = ow + ((long)co * g.Cin + c) * g.taps;
      for (int i = 0; i < g.kh; ++i) {
        const int y = ho * g.sh - g.ph + i * g.dh;
        if (y < 0 || y >= g.H) continue;
        for (int j = 0; j < g.kw; ++j) {
          const int x = wo * g.sw - g.pw + j * g.dw;
          if (x < 0 || x >= g.W) continue;
          acc += to_f32(wrow[i * g.kw + j]) * to_f32(im[(long)y * g.W + x]);
        }
      }
    }
    if (ob) acc += to_f32(ob[co]);
    raw[idx] = from_f32<E>(acc);
  }
}

// [pixel][CO_pad] -> dense (N, CO, Ho, Wo), for callers that want to see the
// conv_offset output.
template <typename E>
__global__ __launch_bounds__(256) void raw_to_nchw_kernel(const E *__restrict__ raw_pm,
                                                          E *__restrict__ raw, int CO, int CO_pad,
                                                          long plane_out, long total) {
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    const long rem = idx % plane_out;
    const int co = (int)((idx / plane_out) % CO);
    const long n = idx / (plane_out * CO);
    raw[idx] = raw_pm[(n * plane_out + rem) * CO_pad + co];
  }
}

}  // namespace mdcn
