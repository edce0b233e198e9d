/*
 * TEST INFRASTRUCTURE ONLY.  Body of the CPU restatement of mmcv's modulated
 * deformable convolution forward, instantiated once per element type by
 * mdcn_oracle.c (which defines T, FN(name) and includes this file).
 *
 * Nothing in the shipped library may include, link or call this.
 */

/* Zero-padded bilinear sample of one channel plane at the real position (h, w).
 * Follows mmcv/ops/csrc/pytorch/cpu/modulated_deform_conv.cpp:5-33: floorf on
 * the coordinate (so a double coordinate is first narrowed to float, as there),
 * each of the four corners contributes 0 when it lies outside the plane, and
 * the four products are summed in the order v1..v4. */
static T FN(bilinear)(const T *plane, int data_width, int height, int width,
                      T h, T w) {
  int h_low = (int)floorf((float)h);
  int w_low = (int)floorf((float)w);
  int h_high = h_low + 1;
  int w_high = w_low + 1;

  T lh = h - (T)h_low;
  T lw = w - (T)w_low;
  T hh = (T)1 - lh, hw = (T)1 - lw;

  T v1 = 0, v2 = 0, v3 = 0, v4 = 0;
  if (h_low >= 0 && w_low >= 0) v1 = plane[h_low * data_width + w_low];
  if (h_low >= 0 && w_high <= width - 1) v2 = plane[h_low * data_width + w_high];
  if (h_high <= height - 1 && w_low >= 0) v3 = plane[h_high * data_width + w_low];
  if (h_high <= height - 1 && w_high <= width - 1)
    v4 = plane[h_high * data_width + w_high];

  T w1 = hh * hw, w2 = hh * lw, w3 = lh * hw, w4 = lh * lw;
  return (w1 * v1 + w2 * v2 + w3 * v3 + w4 * v4);
}

/* Columns of ONE sample: col[(c*kh*kw + i*kw + j), ho*Wo + wo] =
 * mask * bilinear(input[c], position).  Follows
 * mmcv/ops/csrc/pytorch/cpu/modulated_deform_conv.cpp:109-168 with
 * batch_size == 1, which is how the host loop calls it
 * (mmcv/ops/csrc/pytorch/modulated_deform_conv.cpp:108-112).
 *   im     : (C, H, W)          offset : (dg*2*kh*kw, Ho, Wo)
 *   mask   : (dg*kh*kw, Ho, Wo) col    : (C*kh*kw, Ho*Wo)            */
void FN(im2col)(const T *im, const T *offset, const T *mask, int C, int H,
                int W, int kh, int kw, int ph, int pw, int sh, int sw, int dh,
                int dw, int dgroups, int Ho, int Wo, T *col) {
  const int ch_per_dg = C / dgroups;
  const long plane_out = (long)Ho * Wo;
  const long n = (long)C * plane_out;
  for (long index = 0; index < n; ++index) {
    const int wo = (int)(index % Wo);
    const int ho = (int)((index / Wo) % Ho);
    const int c = (int)(index / plane_out);
    const int dg = c / ch_per_dg;
    const int h_in = ho * sh - ph;
    const int w_in = wo * sw - pw;

    T *col_ptr = col + ((long)c * kh * kw) * plane_out + (long)ho * Wo + wo;
    const T *im_ptr = im + (long)c * H * W;
    const T *off_ptr = offset + (long)dg * 2 * kh * kw * plane_out;
    const T *mask_ptr = mask + (long)dg * kh * kw * plane_out;

    for (int i = 0; i < kh; ++i) {
      for (int j = 0; j < kw; ++j) {
        const int tap = i * kw + j;
        const long pix = (long)ho * Wo + wo;
        const T off_h = off_ptr[(long)(2 * tap) * plane_out + pix];
        const T off_w = off_ptr[(long)(2 * tap + 1) * plane_out + pix];
        const T m = mask_ptr[(long)tap * plane_out + pix];
        T val = 0;
        const T h_im = (T)(h_in + i * dh) + off_h;
        const T w_im = (T)(w_in + j * dw) + off_w;
        if (h_im > -1 && w_im > -1 && h_im < H && w_im < W)
          val = FN(bilinear)(im_ptr, W, H, W, h_im, w_im);
        *col_ptr = val * m;
        col_ptr += plane_out;
      }
    }
  }
}

/* out(rows x cols) += a(rows x inner) * b(inner x cols), all row-major, the
 * contraction the reference hands to ATen's addmm_
 * (mmcv/ops/csrc/pytorch/modulated_deform_conv.cpp:119-124).  Plain loops in
 * element type T, summed in increasing k; rows are split over OpenMP threads. */
static void FN(gemm_acc)(const T *a, const T *b, T *out, int rows, int inner,
                         long cols) {
#pragma omp parallel for schedule(static)
  for (int r = 0; r < rows; ++r) {
    T *o = out + (long)r * cols;
    for (int k = 0; k < inner; ++k) {
      const T s = a[(long)r * inner + k];
      const T *bk = b + (long)k * cols;
      for (long p = 0; p < cols; ++p) o[p] += s * bk[p];
    }
  }
}

/* Whole forward.  Follows the host sequence of
 * mmcv/ops/csrc/pytorch/modulated_deform_conv.cpp:62-138: shape checks, zero the
 * output, then per sample: im2col into a (Cin*kh*kw, Ho*Wo) scratch, one GEMM
 * per group accumulating into the zeroed output, and finally the broadcast bias
 * add.  `bias` may be NULL (with_bias == false).  `columns` is caller scratch of
 * Cin*kh*kw*Ho*Wo elements.  Returns 0, or -1 when Cin != weight_cin*groups
 * (the reference raises there). */
int FN(forward)(const T *input, const T *weight, const T *bias,
                const T *offset, const T *mask, T *output, T *columns, int N,
                int Cin, int H, int W, int Cout, int weight_cin, int kh, int kw,
                int sh, int sw, int ph, int pw, int dh, int dw, int groups,
                int dgroups) {
  if (Cin != weight_cin * groups) return -1;
  const int Ho = (H + 2 * ph - (dh * (kh - 1) + 1)) / sh + 1;
  const int Wo = (W + 2 * pw - (dw * (kw - 1) + 1)) / sw + 1;
  const long plane_out = (long)Ho * Wo;
  const int cout_g = Cout / groups;
  const int k_g = weight_cin * kh * kw;

  for (long i = 0; i < (long)N * Cout * plane_out; ++i) output[i] = 0;

  for (int b = 0; b < N; ++b) {
    FN(im2col)(input + (long)b * Cin * H * W,
               offset + (long)b * dgroups * 2 * kh * kw * plane_out,
               mask + (long)b * dgroups * kh * kw * plane_out, Cin, H, W, kh,
               kw, ph, pw, sh, sw, dh, dw, dgroups, Ho, Wo, columns);
    for (int g = 0; g < groups; ++g) {
      FN(gemm_acc)(weight + (long)g * cout_g * k_g,
                   columns + (long)g * k_g * plane_out,
                   output + ((long)b * Cout + (long)g * cout_g) * plane_out,
                   cout_g, k_g, plane_out);
    }
  }

  if (bias) {
    for (int b = 0; b < N; ++b)
      for (int c = 0; c < Cout; ++c) {
        T *o = output + ((long)b * Cout + c) * plane_out;
        for (long p = 0; p < plane_out; ++p) o[p] += bias[c];
      }
  }
  return 0;
}
