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
  // tiled kernel: a workgroup computes TH x 32 output pixels of one image from a
  // PH x PW patch of the input copy
  int TH, tiles_x, tiles_y, PH, PW;
};

// LDS budgets of the tiled kernel (bytes): two workgroups per CU, or one.
constexpr int kOconvLdsSmall = 80 * 1024;
constexpr int kOconvLdsLarge = 156 * 1024;

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

// Implicit GEMM raw[pixel][co] = sum_{c, tap} x[pixel + tap][c] * ow[co][c][tap] + ob[co],
// variant without LDS for geometries whose input patch does not fit the tiled
// kernel below (large dilated kernels with stride): the A operand of the MFMA
// (32 pixels x 16 bytes of channels) is loaded from the input copy as it lies,
// the B operand from the packed weights; each wave owns PXF blocks of 32
// consecutive pixels and all COF blocks of 32 output channels.  A tap outside the
// one-pixel zero border (padding > 1) contributes a zero fragment.  Every lane of
// an A load reads another cache line, which makes this the slow variant.
template <typename E, int COF, int PXF>
__global__ __launch_bounds__(256) void oconv_gather_kernel(OconvArgs a) {
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

// Tiled variant, the usual one.  A workgroup of 4 waves computes TH = 4 * PXF
// output rows x 32 output columns of one image.  Per channel slab it copies the
// input patch those outputs need (PH x PW pixels, 128 bytes each, contiguous
// runs of PW pixels in the copy) to LDS with coalesced 16-byte loads, zero
// filling what lies outside the bordered copy, and every (tap, 16-byte channel
// chunk) then takes its A operand from LDS: lane (pixel column r, half h) of wave
// w reads chunk 2 * ksub + h of patch pixel ((w * PXF + pf) * sh + i * dh,
// r * sw + j * dw).  Chunk c of patch pixel q sits at c ^ (q & 7), which spreads
// the 32 rows of a fragment read over all banks when sw is odd.  The slab's
// packed weights (taps * 4 * COF KiB) follow the patch in LDS, so that no global
// load sits between the MFMAs.  With the small budget two workgroups share a CU
// and the copy of one overlaps the MFMAs of the other.
template <typename E, int COF, int PXF, int LDS_BYTES>
__global__ __launch_bounds__(256, LDS_BYTES <= kOconvLdsSmall ? 2 : 1) void oconv_tiled_kernel(
    OconvArgs a) {
  using TR = ElemTraits<E>;
  __shared__ uint4 patch[LDS_BYTES / 16];
  const Geom &g = a.g;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int frow = lane & 31;
  const int fhalf = lane >> 5;

  int b = blockIdx.x;
  const int tx = b % a.tiles_x;
  b /= a.tiles_x;
  const int ty = b % a.tiles_y;
  const int n = b / a.tiles_y;
  const int ho0 = ty * a.TH, wo0 = tx * 32;
  const int py0 = ho0 * g.sh - g.ph + 1;  // patch origin in the bordered copy (may lie outside)
  const int px0 = wo0 * g.sw - g.pw + 1;
  const int patch_px = a.PH * a.PW;

  f32x16 acc[PXF][COF];
#pragma unroll
  for (int pf = 0; pf < PXF; ++pf)
#pragma unroll
    for (int cf = 0; cf < COF; ++cf)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[pf][cf][r] = 0.0f;

  // patch pixel of this lane's output pixel for tap (0, 0)
  int q0[PXF];
#pragma unroll
  for (int pf = 0; pf < PXF; ++pf) q0[pf] = ((wave * PXF + pf) * g.sh) * a.PW + frow * g.sw;

  uint4 *wlds = patch + patch_px * 8;
  const int wchunks = g.taps * 4 * COF * 64;  // 16-byte chunks of one slab's weights
  const int total_chunks = patch_px * 8 + wchunks;

  // A slab's LDS contents arrive by direct-to-LDS copies, 1 KiB per wave and
  // instruction: lane l of copy j fills chunk i = 256 * j + 64 * wave + l of the
  // LDS array and reads the source chunk that belongs there (the swizzle is
  // applied on the source side).  Per chunk, once per workgroup and the same for
  // every slab: soff >= 0 is an offset into the slab's plane of the copy, soff < 0
  // weight chunk -1 - soff.  A patch pixel outside the copy reads the copy's
  // corner pixel (0, 0), a stored zero.  All copies of a slab are in flight
  // together; nothing the compiler sees waits between them.
  constexpr int NB = (LDS_BYTES / 16 + 255) / 256;
  int soff[NB];
#pragma unroll
  for (int j = 0; j < NB; ++j) {
    const int idx = tid + 256 * j;
    const int q = idx >> 3;
    const int c = (idx & 7) ^ (q & 7);
    const int r = q / a.PW;
    const int y = py0 + r, x = px0 + (q - r * a.PW);
    const bool in_copy = y >= 0 && y < g.Hp && x >= 0 && x < g.Wp;
    if (idx < patch_px * 8) soff[j] = in_copy ? (y * g.Wp + x) * 8 + c : c;
    else if (idx < total_chunks) soff[j] = -1 - (idx - patch_px * 8);
    else soff[j] = 0;
  }
  const uint32_t lds_wave = (uint32_t)(uintptr_t)(lptr_t)(&patch[0]) +
                            (uint32_t)__builtin_amdgcn_readfirstlane(wave) * 1024u;
  auto fetch = [&](int slab) {
    const uint4 *src = (const uint4 *)a.xt + ((long)n * a.slabs_total + slab) * a.plane_px * 8;
    const uint4 *wsrc = (const uint4 *)a.owp + (long)slab * wchunks;
#pragma unroll
    for (int j = 0; j < NB; ++j) {
      if (256 * j < total_chunks) {
        const uint4 *ptr = soff[j] >= 0 ? src + soff[j] : wsrc + (-1 - soff[j]);
        copy16_global_to_lds(ptr, lds_wave + (uint32_t)j * 4096u);
      }
    }
  };

  for (int slab = 0; slab < a.slabs_total; ++slab) {
    __syncthreads();  // the previous slab's fragment reads are done
    fetch(slab);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    for (int ti = 0; ti < g.kh; ++ti) {
      for (int tj = 0; tj < g.kw; ++tj) {
        const int tap = ti * g.kw + tj;
        const int dq = ti * g.dh * a.PW + tj * g.dw;
        const uint4 *wfrag = wlds + tap * 4 * COF * 64 + lane;
#pragma unroll
        for (int ksub = 0; ksub < 4; ++ksub) {
          uint4 af[PXF], bf[COF];
#pragma unroll
          for (int cf = 0; cf < COF; ++cf) bf[cf] = wfrag[(ksub * COF + cf) * 64];
#pragma unroll
          for (int pf = 0; pf < PXF; ++pf) {
            const int q = q0[pf] + dq;
            af[pf] = patch[q * 8 + ((ksub * 2 + fhalf) ^ (q & 7))];
          }
#pragma unroll
          for (int pf = 0; pf < PXF; ++pf)
#pragma unroll
            for (int cf = 0; cf < COF; ++cf) TR::mma(acc[pf][cf], af[pf], bf[cf]);
        }
      }
    }
  }

  // Accumulator block (A = pixels, B = channels): register r of lane l holds
  //   pixel column = (r/4)*8 + (l/32)*4 + r%4,  channel = l%32.
  E *raw = (E *)a.raw;
  const long plane_out = (long)g.Ho * g.Wo;
#pragma unroll
  for (int cf = 0; cf < COF; ++cf) {
    const int co = cf * 32 + frow;
    float bias = 0.0f;
    if (a.obias && co < a.CO) bias = to_f32(((const E *)a.obias)[co]);
#pragma unroll
    for (int pf = 0; pf < PXF; ++pf) {
      const int ho = ho0 + wave * PXF + pf;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int wo = wo0 + (r >> 2) * 8 + fhalf * 4 + (r & 3);
        if (ho < g.Ho && wo < g.Wo) {
          const long p = (long)n * plane_out + (long)ho * g.Wo + wo;
          raw[p * a.CO_pad + co] = from_f32<E>(acc[pf][cf][r] + bias);
        }
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
