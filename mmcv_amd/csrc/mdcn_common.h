// Shared definitions of the DCNv2 forward kernels (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mdcn {

typedef __bf16 bf16_t;
typedef _Float16 f16_t;

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// Geometry of one launch, identical for every kernel of the path.
struct Geom {
  int N, Cin, H, W;
  int Cout, kh, kw;
  int sh, sw, ph, pw, dh, dw;
  int G, DG;
  int Ho, Wo;
  int cin_g;      // Cin / G
  int cout_g;     // Cout / G
  int ch_per_dg;  // Cin / DG
  int taps;       // kh * kw
  int Hp, Wp;     // H + 2, W + 2: the zero-bordered channels-last copy
};

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(f16_t v) { return (float)v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return (float)v; }

template <typename E>
__device__ __forceinline__ E from_f32(float v) {
  return (E)v;
}

// Sampling position of one (pixel, tap) and its four mask-scaled bilinear
// weights; same arithmetic order as the reference's CPU sampler
// (mmcv/ops/csrc/pytorch/cpu/modulated_deform_conv.cpp:5-33,158-163) in fp32,
// except that the mask is folded into the four weights.
struct TapSample {
  int y0, x0;              // floor of the position, valid only when inside
  float w00, w01, w10, w11;  // weights of (y0,x0) (y0,x0+1) (y0+1,x0) (y0+1,x0+1)
  bool inside;             // position in the open box (-1,H) x (-1,W)
};

__device__ __forceinline__ TapSample make_tap_sample(int base_y, int base_x,
                                                     float dy, float dx,
                                                     float m, int H, int W) {
  TapSample s;
  const float py = (float)base_y + dy;
  const float px = (float)base_x + dx;
  s.inside = (py > -1.0f) && (px > -1.0f) && (py < (float)H) && (px < (float)W);
  const float fy = floorf(py), fx = floorf(px);
  const float ly = py - fy, lx = px - fx;
  const float hy = 1.0f - ly, hx = 1.0f - lx;
  s.y0 = s.inside ? (int)fy : 0;
  s.x0 = s.inside ? (int)fx : 0;
  const float mm = s.inside ? m : 0.0f;
  s.w00 = s.inside ? (hy * hx) * mm : 0.0f;
  s.w01 = s.inside ? (hy * lx) * mm : 0.0f;
  s.w10 = s.inside ? (ly * hx) * mm : 0.0f;
  s.w11 = s.inside ? (ly * lx) * mm : 0.0f;
  return s;
}

// For reading the four corners from a tensor without a zero border (needs
// H, W >= 2): move the 2x2 block into the image and give the corners that fell
// outside weight 0; the corners that stay valid keep their weight, at their new
// place in the block.  Positions outside (-1,H)x(-1,W) already have zero weights
// and y0 = x0 = 0.
__device__ __forceinline__ void clamp_to_image(TapSample &s, int H, int W) {
  // (selects on values, not conditional stores into the struct, which the compiler parks in scratch memory)
  const bool xl = s.x0 < 0;        // only the right column (x0 + 1 == 0) is inside: it becomes the left one
  const bool xr = s.x0 > W - 2;    // only the left column (x0 == W - 1) is inside: it becomes the right one
  const float a00 = xl ? s.w01 : (xr ? 0.0f : s.w00), a01 = xl ? 0.0f : (xr ? s.w00 : s.w01);
  const float a10 = xl ? s.w11 : (xr ? 0.0f : s.w10), a11 = xl ? 0.0f : (xr ? s.w10 : s.w11);
  const int x0 = xl ? 0 : (xr ? W - 2 : s.x0);
  const bool yu = s.y0 < 0, yd = s.y0 > H - 2;   // likewise the rows
  const float b00 = yu ? a10 : (yd ? 0.0f : a00), b01 = yu ? a11 : (yd ? 0.0f : a01);
  const float b10 = yu ? 0.0f : (yd ? a00 : a10), b11 = yu ? 0.0f : (yd ? a01 : a11);
  const int y0 = yu ? 0 : (yd ? H - 2 : s.y0);
  s.w00 = b00; s.w01 = b01; s.w10 = b10; s.w11 = b11;
  s.x0 = x0; s.y0 = y0;
}

// Where the offsets and the mask of one output pixel live, in elements: image n,
// pixel rem = ho * Wo + wo, channel c sits at base + n * _n + rem * _px + c * _ch.
// The reference op takes two dense NCHW tensors (_px = 1, _ch = Ho * Wo); the
// pack-level entry points read both out of the one conv_offset output, whose
// first 2/3 of the channels are the offsets (chunk + cat of
// mmcv/ops/modulated_deform_conv.py:329-330 is the identity on them) and whose
// last third holds the mask before the sigmoid (`logit` = 1, :331).  `logit` = 2
// stands for "no mask": the unmodulated deformable convolution (DCNv1,
// mmcv/ops/csrc/pytorch/cpu/deform_conv.cpp:115-167, the same sampler without
// the factor); msk then aliases off so that the kernels' loads stay valid.
struct OffMaskView {
  const void *off, *msk;
  long off_n, msk_n;
  long off_ch, msk_ch;
  int off_px, msk_px;
  int logit;
};
constexpr int kMaskPlain = 0, kMaskLogit = 1, kMaskNone = 2;

__host__ __device__ inline OffMaskView dense_view(const void *off, const void *msk, const Geom &g) {
  OffMaskView v;
  const long plane = (long)g.Ho * g.Wo;
  v.off = off; v.msk = msk;
  v.off_n = (long)g.DG * 2 * g.taps * plane; v.msk_n = (long)g.DG * g.taps * plane;
  v.off_ch = plane; v.msk_ch = plane;
  v.off_px = 1; v.msk_px = 1;
  v.logit = kMaskPlain;
  if (!msk) {  // unmodulated: read (and ignore) offsets instead
    v.msk = off; v.msk_n = v.off_n; v.logit = kMaskNone;
  }
  return v;
}

// Mask value from the stored element; a logit goes through the sigmoid and is
// rounded to the element type once, as torch.sigmoid on an E tensor does.
template <typename E>
__device__ __forceinline__ float mask_value(E raw, int logit) {
  float m = to_f32(raw);
  if (logit == kMaskLogit) m = to_f32(from_f32<E>(1.0f / (1.0f + expf(-m))));
  if (logit == kMaskNone) m = 1.0f;
  return m;
}

}  // namespace mdcn
