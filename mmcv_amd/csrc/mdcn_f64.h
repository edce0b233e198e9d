// Double-precision kernels of the (modulated) deformable convolution, forward and
// backward.  The reference dispatches its kernels over double as well
// (AT_DISPATCH_FLOATING_TYPES_AND_HALF in
// mmcv/ops/csrc/pytorch/cuda/modulated_deform_conv_cuda.cu:16 and
// cpu/modulated_deform_conv.cpp:333) and its own tests run the layer in
// torch.double (tests/test_ops/test_modulated_deform_conv.py:148-160), so the
// drop-in has to accept such tensors.  Nobody trains in fp64: these kernels are
// written for being right and deterministic where that is free, not for speed.
// Positions, bilinear weights and sums are all double, as in the reference's
// scalar_t = double instantiation
// (cpu/modulated_deform_conv.cpp:5-33 sampler, :34-107 gradient weights,
// :109-320 im2col / col2im / col2im_coord).
#pragma once

#include "mdcn_common.h"

namespace mdcn {

// Sampling position of one (pixel, tap) in double: the four corner weights, which
// corners lie in the image and their offsets in the image plane.
struct TapD {
  bool inside;          // position in the open box (-1,H) x (-1,W)
  bool ok00, ok01, ok10, ok11;
  long o00, o01, o10, o11;
  double ly, lx, hy, hx;
};

__device__ __forceinline__ TapD make_tap_d(int base_y, int base_x, double dy, double dx, int H, int W) {
  TapD s;
  const double py = (double)base_y + dy, px = (double)base_x + dx;
  s.inside = (py > -1.0) && (px > -1.0) && (py < (double)H) && (px < (double)W);
  const double fy = floor(py), fx = floor(px);
  const int y0 = s.inside ? (int)fy : 0, x0 = s.inside ? (int)fx : 0, y1 = y0 + 1, x1 = x0 + 1;
  s.ly = py - fy; s.lx = px - fx; s.hy = 1.0 - s.ly; s.hx = 1.0 - s.lx;
  s.ok00 = s.inside && y0 >= 0 && x0 >= 0;
  s.ok01 = s.inside && y0 >= 0 && x1 <= W - 1;
  s.ok10 = s.inside && y1 <= H - 1 && x0 >= 0;
  s.ok11 = s.inside && y1 <= H - 1 && x1 <= W - 1;
  s.o00 = (long)y0 * W + x0; s.o01 = s.o00 + 1; s.o10 = s.o00 + W; s.o11 = s.o10 + 1;
  return s;
}

// One thread per output element.  mask == nullptr: no modulation (DCNv1).
__global__ __launch_bounds__(256) void f64_forward_kernel(Geom g, const double *__restrict__ input,
                                                          const double *__restrict__ offset,
                                                          const double *__restrict__ mask,
                                                          const double *__restrict__ weight,
                                                          const double *__restrict__ bias,
                                                          double *__restrict__ output, long total) {
  const long plane_out = (long)g.Ho * g.Wo, plane_in = (long)g.H * g.W;
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
    const int wo = (int)(idx % g.Wo);
    const int ho = (int)((idx / g.Wo) % g.Ho);
    const int co = (int)((idx / plane_out) % g.Cout);
    const int n = (int)(idx / (plane_out * g.Cout));
    const int grp = co / g.cout_g;
    const long pix = (long)ho * g.Wo + wo;
    double acc = 0.0;
    for (int cl = 0; cl < g.cin_g; ++cl) {
      const int c = grp * g.cin_g + cl;
      const int dgi = c / g.ch_per_dg;
      const double *im = input + ((long)n * g.Cin + c) * plane_in;
      const double *off = offset + ((long)n * g.DG + dgi) * 2 * g.taps * plane_out + pix;
      const double *msk = mask ? mask + ((long)n * g.DG + dgi) * g.taps * plane_out + pix : nullptr;
      const double *wrow = weight + ((long)co * g.cin_g + cl) * g.taps;
      for (int tap = 0; tap < g.taps; ++tap) {
        const int i = tap / g.kw, j = tap - i * g.kw;
        const TapD s = make_tap_d(ho * g.sh - g.ph + i * g.dh, wo * g.sw - g.pw + j * g.dw,
                                  off[(long)(2 * tap) * plane_out], off[(long)(2 * tap + 1) * plane_out], g.H, g.W);
        if (!s.inside) continue;
        const double v00 = s.ok00 ? im[s.o00] : 0.0, v01 = s.ok01 ? im[s.o01] : 0.0;
        const double v10 = s.ok10 ? im[s.o10] : 0.0, v11 = s.ok11 ? im[s.o11] : 0.0;
        const double v = (s.hy * s.hx) * v00 + (s.hy * s.lx) * v01 + (s.ly * s.hx) * v10 + (s.ly * s.lx) * v11;
        const double m = msk ? msk[(long)tap * plane_out] : 1.0;
        acc += wrow[tap] * (v * m);
      }
    }
    if (bias) acc += bias[co];
    output[idx] = acc;
  }
}

// grad_input (atomics into a zeroed tensor), grad_offset, grad_mask: one thread
// per (image, deformable group, tap, output pixel); the column gradient of each of
// the group's channels, d = sum_co weight[co, c, tap] * grad_output[n, co, pixel],
// is formed on the fly.
__global__ __launch_bounds__(256) void f64_bwd_data_kernel(Geom g, const double *__restrict__ input,
                                                           const double *__restrict__ offset,
                                                           const double *__restrict__ mask,
                                                           const double *__restrict__ weight,
                                                           const double *__restrict__ gout,
                                                           double *__restrict__ gin, double *__restrict__ goff,
                                                           double *__restrict__ gmask, long total) {
  const long plane_out = (long)g.Ho * g.Wo, plane_in = (long)g.H * g.W;
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
    const long pix = idx % plane_out;
    long r = idx / plane_out;
    const int tap = (int)(r % g.taps);
    r /= g.taps;
    const int dgi = (int)(r % g.DG);
    const int n = (int)(r / g.DG);
    const int ho = (int)(pix / g.Wo), wo = (int)(pix - (long)ho * g.Wo);
    const int ti = tap / g.kw, tj = tap - ti * g.kw;
    const long ob = ((long)n * g.DG + dgi) * 2 * g.taps;
    const double dy = offset[(ob + 2 * tap) * plane_out + pix];
    const double dx = offset[(ob + 2 * tap + 1) * plane_out + pix];
    const long mb = (((long)n * g.DG + dgi) * g.taps + tap) * plane_out + pix;
    const double m = mask ? mask[mb] : 1.0;
    const TapD s = make_tap_d(ho * g.sh - g.ph + ti * g.dh, wo * g.sw - g.pw + tj * g.dw, dy, dx, g.H, g.W);
    double acc_m = 0.0, acc_y = 0.0, acc_x = 0.0;
    if (s.inside) {
      for (int c = dgi * g.ch_per_dg; c < (dgi + 1) * g.ch_per_dg; ++c) {
        const int grp = c / g.cin_g, cl = c - grp * g.cin_g;
        const double *grow = gout + ((long)n * g.Cout + (long)grp * g.cout_g) * plane_out + pix;
        const double *wcol = weight + ((long)grp * g.cout_g * g.cin_g + cl) * g.taps + tap;
        double d = 0.0;
        for (int co = 0; co < g.cout_g; ++co) d += wcol[(long)co * g.cin_g * g.taps] * grow[(long)co * plane_out];
        const double *im = input + ((long)n * g.Cin + c) * plane_in;
        const double v00 = s.ok00 ? im[s.o00] : 0.0, v01 = s.ok01 ? im[s.o01] : 0.0;
        const double v10 = s.ok10 ? im[s.o10] : 0.0, v11 = s.ok11 ? im[s.o11] : 0.0;
        acc_m += d * ((s.hy * s.hx) * v00 + (s.hy * s.lx) * v01 + (s.ly * s.hx) * v10 + (s.ly * s.lx) * v11);
        acc_y += d * (s.hx * (v10 - v00) + s.lx * (v11 - v01));
        acc_x += d * (s.hy * (v01 - v00) + s.ly * (v11 - v10));
        const double t = d * m;
        double *gi = gin + ((long)n * g.Cin + c) * plane_in;
        if (s.ok00) atomicAdd(gi + s.o00, (s.hy * s.hx) * t);
        if (s.ok01) atomicAdd(gi + s.o01, (s.hy * s.lx) * t);
        if (s.ok10) atomicAdd(gi + s.o10, (s.ly * s.hx) * t);
        if (s.ok11) atomicAdd(gi + s.o11, (s.ly * s.lx) * t);
      }
    }
    goff[(ob + 2 * tap) * plane_out + pix] = acc_y * m;
    goff[(ob + 2 * tap + 1) * plane_out + pix] = acc_x * m;
    if (gmask) gmask[mb] = acc_m;
  }
}

// Sum of the 256 values of a workgroup (result valid in thread 0), fixed order.
__device__ __forceinline__ double block_sum_d(double v, double *part) {
  part[threadIdx.x] = v;
  __syncthreads();
  for (int w = 128; w > 0; w >>= 1) {
    if ((int)threadIdx.x < w) part[threadIdx.x] += part[threadIdx.x + w];
    __syncthreads();
  }
  const double s = part[0];
  __syncthreads();
  return s;
}

// grad_weight: one workgroup per weight element (co, c, tap) sums
// grad_output[n, co, pixel] * column[n, c, tap, pixel] over images and pixels; plain
// store, so the result does not depend on the order workgroups run in.
__global__ __launch_bounds__(256) void f64_bwd_weight_kernel(Geom g, const double *__restrict__ input,
                                                             const double *__restrict__ offset,
                                                             const double *__restrict__ mask,
                                                             const double *__restrict__ gout,
                                                             double *__restrict__ gweight) {
  __shared__ double part[256];
  const long plane_out = (long)g.Ho * g.Wo, plane_in = (long)g.H * g.W;
  for (long widx = blockIdx.x; widx < (long)g.Cout * g.cin_g * g.taps; widx += gridDim.x) {
    const int tap = (int)(widx % g.taps);
    const int cl = (int)((widx / g.taps) % g.cin_g);
    const int co = (int)(widx / ((long)g.taps * g.cin_g));
    const int grp = co / g.cout_g;
    const int c = grp * g.cin_g + cl;
    const int dgi = c / g.ch_per_dg;
    const int ti = tap / g.kw, tj = tap - ti * g.kw;
    double acc = 0.0;
    for (long e = threadIdx.x; e < (long)g.N * plane_out; e += 256) {
      const int n = (int)(e / plane_out);
      const long pix = e - (long)n * plane_out;
      const int ho = (int)(pix / g.Wo), wo = (int)(pix - (long)ho * g.Wo);
      const long ob = ((long)n * g.DG + dgi) * 2 * g.taps;
      const TapD s = make_tap_d(ho * g.sh - g.ph + ti * g.dh, wo * g.sw - g.pw + tj * g.dw,
                                offset[(ob + 2 * tap) * plane_out + pix], offset[(ob + 2 * tap + 1) * plane_out + pix],
                                g.H, g.W);
      if (!s.inside) continue;
      const double *im = input + ((long)n * g.Cin + c) * plane_in;
      const double v00 = s.ok00 ? im[s.o00] : 0.0, v01 = s.ok01 ? im[s.o01] : 0.0;
      const double v10 = s.ok10 ? im[s.o10] : 0.0, v11 = s.ok11 ? im[s.o11] : 0.0;
      const double v = (s.hy * s.hx) * v00 + (s.hy * s.lx) * v01 + (s.ly * s.hx) * v10 + (s.ly * s.lx) * v11;
      const double m = mask ? mask[(((long)n * g.DG + dgi) * g.taps + tap) * plane_out + pix] : 1.0;
      acc += gout[((long)n * g.Cout + co) * plane_out + pix] * (v * m);
    }
    const double sum = block_sum_d(acc, part);
    if (threadIdx.x == 0) gweight[widx] = sum;
  }
}

// grad_bias[co] = sum over images and pixels of grad_output[:, co].
__global__ __launch_bounds__(256) void f64_bwd_bias_kernel(Geom g, const double *__restrict__ gout,
                                                           double *__restrict__ gbias) {
  __shared__ double part[256];
  const long plane_out = (long)g.Ho * g.Wo;
  for (int co = blockIdx.x; co < g.Cout; co += gridDim.x) {
    double acc = 0.0;
    for (long e = threadIdx.x; e < (long)g.N * plane_out; e += 256) {
      const int n = (int)(e / plane_out);
      acc += gout[((long)n * g.Cout + co) * plane_out + (e - (long)n * plane_out)];
    }
    const double sum = block_sum_d(acc, part);
    if (threadIdx.x == 0) gbias[co] = sum;
  }
}

__global__ __launch_bounds__(256) void f64_zero_kernel(double *p, long n) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) p[i] = 0.0;
}

}  // namespace mdcn
