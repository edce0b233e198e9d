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

}  // namespace mdcn
