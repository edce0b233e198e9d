/*
 * TEST INFRASTRUCTURE ONLY -- never linked into, imported by or called from the
 * shipped library.  Only the test-suite, the smoke check and the benchmark's
 * CPU-baseline leg may load this, and only as the checker.
 *
 * Plain-C restatement of the CPU algorithm of mmcv's modulated deformable
 * convolution (DCNv2) forward:
 *   sampler   mmcv/ops/csrc/pytorch/cpu/modulated_deform_conv.cpp:5-33
 *   im2col    mmcv/ops/csrc/pytorch/cpu/modulated_deform_conv.cpp:109-168
 *   host op   mmcv/ops/csrc/pytorch/modulated_deform_conv.cpp:62-138
 * in float (mdcn_oracle_f32_*) and double (mdcn_oracle_f64_*), the two element
 * types the reference's own CPU tests run.
 *
 * How each function is pinned (tests/test_oracle.py):
 *   bilinear, im2col, forward -- the reference's known-answer vectors
 *     (tests/test_ops/test_modulated_deform_conv.py:28-30 and, with mask == 1,
 *     tests/test_ops/test_deform_conv.py:27-35,47), the compiled reference
 *     itself (oracle/_ref) on seeded random cases, equality with a zero-padded
 *     F.conv2d when all offsets are 0, equality with F.grid_sample
 *     (align_corners=True, zeros padding) + einsum in float64, and a float64
 *     brute-force definition in numpy on tiny shapes.
 */
#include <math.h>

#define MDCN_CAT2(a, b) a##b
#define MDCN_CAT(a, b) MDCN_CAT2(a, b)

#define T float
#define FN(name) MDCN_CAT(mdcn_oracle_f32_, name)
#include "mdcn_oracle_impl.h"
#include "mdcn_oracle_bwd_impl.h"
#undef T
#undef FN

#define T double
#define FN(name) MDCN_CAT(mdcn_oracle_f64_, name)
#include "mdcn_oracle_impl.h"
#include "mdcn_oracle_bwd_impl.h"
#undef T
#undef FN

/* Exposed for the sampler's own unit checks (the static helpers are not
 * visible through the shared object). */
float mdcn_oracle_f32_sample(const float *plane, int height, int width, float h,
                             float w) {
  if (!(h > -1 && w > -1 && h < height && w < width)) return 0.0f;
  return mdcn_oracle_f32_bilinear(plane, width, height, width, h, w);
}

double mdcn_oracle_f64_sample(const double *plane, int height, int width,
                              double h, double w) {
  if (!(h > -1 && w > -1 && h < height && w < width)) return 0.0;
  return mdcn_oracle_f64_bilinear(plane, width, height, width, h, w);
}
