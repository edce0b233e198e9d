/*
 * TEST INFRASTRUCTURE ONLY.  CPU restatement of mmcv's modulated deformable
 * convolution BACKWARD, instantiated per element type by mdcn_oracle.c after
 * mdcn_oracle_impl.h (it uses that file's bilinear, im2col and gemm_acc).
 *
 * Nothing in the shipped library may include, link or call this.
 */

/* d(sample at (ph, pw)) / d(pixel (h, w)): the bilinear weight of corner (h, w),
 * 0 for every other pixel and for positions outside (-1, H) x (-1, W).
 * Follows mmcv/ops/csrc/pytorch/cpu/modulated_deform_conv.cpp:34-58. */
static T FN(pixel_weight)(T ph, T pw, int h, int w, int height, int width) {
  if (ph <= -1 || ph >= height || pw <= -1 || pw >= width) return 0;
  const int h_low = (int)floorf((float)ph), w_low = (int)floorf((float)pw);
  const int h_high = h_low + 1, w_high = w_low + 1;
  T weight = 0;
  if (h == h_low && w == w_low) weight = ((T)(h + 1) - ph) * ((T)(w + 1) - pw);
  if (h == h_low && w == w_high) weight = ((T)(h + 1) - ph) * (pw + (T)1 - (T)w);
  if (h == h_high && w == w_low) weight = (ph + (T)1 - (T)h) * ((T)(w + 1) - pw);
  if (h == h_high && w == w_high) weight = (ph + (T)1 - (T)h) * (pw + (T)1 - (T)w);
  return weight;
}

/* d(sample at (ph, pw)) / d(ph) for dir == 0, / d(pw) for dir == 1, with the
 * forward's per-corner validity rule.  Follows :60-107. */
static T FN(coord_weight)(T ph, T pw, int height, int width, const T *im,
                          int data_width, int dir) {
  if (ph <= -1 || ph >= height || pw <= -1 || pw >= width) return 0;
  const int h_low = (int)floorf((float)ph), w_low = (int)floorf((float)pw);
  const int h_high = h_low + 1, w_high = w_low + 1;
  T weight = 0;
  if (dir == 0) {
    if (h_low >= 0 && w_low >= 0)
      weight += (T)-1 * ((T)(w_low + 1) - pw) * im[h_low * data_width + w_low];
    if (h_low >= 0 && w_high <= width - 1)
      weight += (T)-1 * (pw - (T)w_low) * im[h_low * data_width + w_high];
    if (h_high <= height - 1 && w_low >= 0)
      weight += ((T)(w_low + 1) - pw) * im[h_high * data_width + w_low];
    if (h_high <= height - 1 && w_high <= width - 1)
      weight += (pw - (T)w_low) * im[h_high * data_width + w_high];
  } else {
    if (h_low >= 0 && w_low >= 0)
      weight += (T)-1 * ((T)(h_low + 1) - ph) * im[h_low * data_width + w_low];
    if (h_low >= 0 && w_high <= width - 1)
      weight += ((T)(h_low + 1) - ph) * im[h_low * data_width + w_high];
    if (h_high <= height - 1 && w_low >= 0)
      weight += (T)-1 * (ph - (T)h_low) * im[h_high * data_width + w_low];
    if (h_high <= height - 1 && w_high <= width - 1)
      weight += (ph - (T)h_low) * im[h_high * data_width + w_high];
  }
  return weight;
}

/* grad_im (C, H, W) += scatter of dcol (C*kh*kw, Ho*Wo) * mask through the
 * bilinear weights, ONE sample.  Follows :170-230, including its way of finding
 * the touched pixels: truncate the position toward zero and test the 5x5
 * neighbourhood for |distance| < 1 in both directions. */
static void FN(col2im)(const T *dcol, const T *offset, const T *mask, int C, int H,
                       int W, int kh, int kw, int ph, int pw, int sh, int sw,
                       int dh, int dw, int dgroups, int Ho, int Wo, T *grad_im) {
  const int ch_per_dg = C / dgroups;
  const long plane_out = (long)Ho * Wo;
  const long n = (long)C * kh * kw * plane_out;
  for (long index = 0; index < n; ++index) {
    const int wo = (int)(index % Wo);
    const int ho = (int)((index / Wo) % Ho);
    const int j = (int)((index / plane_out) % kw);
    const int i = (int)((index / plane_out / kw) % kh);
    const int c = (int)(index / plane_out / kw / kh);
    const int dg = c / ch_per_dg;
    const int tap = i * kw + j;
    const long pix = (long)ho * Wo + wo;
    const T *off_ptr = offset + (long)dg * 2 * kh * kw * plane_out;
    const T *mask_ptr = mask + (long)dg * kh * kw * plane_out;
    const T off_h = off_ptr[(long)(2 * tap) * plane_out + pix];
    const T off_w = off_ptr[(long)(2 * tap + 1) * plane_out + pix];
    const T m = mask_ptr[(long)tap * plane_out + pix];
    const T pos_h = (T)(ho * sh - ph + i * dh) + off_h;
    const T pos_w = (T)(wo * sw - pw + j * dw) + off_w;
    const T top = dcol[index] * m;
    const int cur_h = (int)pos_h, cur_w = (int)pos_w;
    for (int dy = -2; dy <= 2; ++dy)
      for (int dx = -2; dx <= 2; ++dx) {
        const int y = cur_h + dy, x = cur_w + dx;
        const T ay = pos_h - (T)y, ax = pos_w - (T)x;
        if (y >= 0 && y < H && x >= 0 && x < W && (ay < 0 ? -ay : ay) < 1 &&
            (ax < 0 ? -ax : ax) < 1)
          grad_im[((long)c * H + y) * W + x] +=
              FN(pixel_weight)(pos_h, pos_w, y, x, H, W) * top;
      }
  }
}

/* grad_offset (dg*2*kh*kw, Ho, Wo) and grad_mask (dg*kh*kw, Ho, Wo) of ONE
 * sample from dcol and the input.  Follows :232-320: for every offset channel
 * the sum over the channels of its deformable group of
 * coord_weight * dcol * mask, and for the mask (taken on the even offset
 * channels) the sum of dcol * unmasked sample. */
static void FN(col2im_coord)(const T *dcol, const T *im, const T *offset,
                             const T *mask, int C, int H, int W, int kh, int kw,
                             int ph, int pw, int sh, int sw, int dh, int dw,
                             int dgroups, int Ho, int Wo, T *grad_offset,
                             T *grad_mask) {
  const int ch_per_dg = C / dgroups;
  const int taps = kh * kw;
  const long plane_out = (long)Ho * Wo;
  const long n = (long)dgroups * 2 * taps * plane_out;
  for (long index = 0; index < n; ++index) {
    const int wo = (int)(index % Wo);
    const int ho = (int)((index / Wo) % Ho);
    const int oc = (int)(index / plane_out);  /* offset channel */
    const int dg = oc / (2 * taps);
    const int oc_in = oc - dg * 2 * taps;
    const int tap = oc_in / 2, dir = oc_in % 2;
    const int i = tap / kw, j = tap % kw;
    const long pix = (long)ho * Wo + wo;
    const T *off_ptr = offset + (long)dg * 2 * taps * plane_out;
    const T off_h = off_ptr[(long)(2 * tap) * plane_out + pix];
    const T off_w = off_ptr[(long)(2 * tap + 1) * plane_out + pix];
    const T m = mask[((long)dg * taps + tap) * plane_out + pix];
    T val = 0, mval = 0;
    for (int cl = 0; cl < ch_per_dg; ++cl) {
      const int c = dg * ch_per_dg + cl;
      const T d = dcol[((long)c * taps + tap) * plane_out + pix];
      const T *plane = im + (long)c * H * W;
      T pos_h = (T)(ho * sh - ph + i * dh) + off_h;
      T pos_w = (T)(wo * sw - pw + j * dw) + off_w;
      if (pos_h <= -1 || pos_w <= -1 || pos_h >= H || pos_w >= W)
        pos_h = pos_w = -2;
      else
        mval += d * FN(bilinear)(plane, W, H, W, pos_h, pos_w);
      val += FN(coord_weight)(pos_h, pos_w, H, W, plane, W, dir) * d * m;
    }
    grad_offset[index] = val;
    if (dir == 0) grad_mask[((long)dg * taps + tap) * plane_out + pix] = mval;
  }
}

/* Whole backward.  Follows the host sequence of
 * mmcv/ops/csrc/pytorch/modulated_deform_conv.cpp:140-251 for gradients that
 * start at zero (its Python caller allocates them with zeros_like,
 * mmcv/ops/modulated_deform_conv.py:177-181): per sample, columns = W^T * gout
 * per group, then the offset/mask gradients, the input gradient, the forward
 * columns again and grad_weight += gout * columns^T, grad_bias += row sums.
 * grad_bias may be NULL.  `columns` is caller scratch of Cin*kh*kw*Ho*Wo. */
int FN(backward)(const T *input, const T *weight, const T *offset, const T *mask,
                 const T *grad_output, T *grad_input, T *grad_weight,
                 T *grad_bias, T *grad_offset, T *grad_mask, T *columns, int N,
                 int Cin, int H, int W, int Cout, int weight_cin, int kh, int kw,
                 int sh, int sw, int ph, int pw, int dh, int dw, int groups,
                 int dgroups) {
  if (Cin != weight_cin * groups) return -1;
  const int Ho = (H + 2 * ph - (dh * (kh - 1) + 1)) / sh + 1;
  const int Wo = (W + 2 * pw - (dw * (kw - 1) + 1)) / sw + 1;
  const long plane_out = (long)Ho * Wo;
  const int taps = kh * kw;
  const int cout_g = Cout / groups;
  const int k_g = weight_cin * taps;

  for (long i = 0; i < (long)N * Cin * H * W; ++i) grad_input[i] = 0;
  for (long i = 0; i < (long)Cout * k_g; ++i) grad_weight[i] = 0;
  if (grad_bias)
    for (int i = 0; i < Cout; ++i) grad_bias[i] = 0;

  for (int b = 0; b < N; ++b) {
    const T *gout = grad_output + (long)b * Cout * plane_out;
    const T *off_b = offset + (long)b * dgroups * 2 * taps * plane_out;
    const T *mask_b = mask + (long)b * dgroups * taps * plane_out;
    const T *im_b = input + (long)b * Cin * H * W;
    /* columns[g] = weight[g]^T (k_g x cout_g) * gout[g] (cout_g x P) */
    for (long i = 0; i < (long)Cin * taps * plane_out; ++i) columns[i] = 0;
    for (int g = 0; g < groups; ++g) {
      const T *wg = weight + (long)g * cout_g * k_g;
      const T *gg = gout + (long)g * cout_g * plane_out;
      T *cg = columns + (long)g * k_g * plane_out;
#pragma omp parallel for schedule(static)
      for (int k = 0; k < k_g; ++k) {
        T *o = cg + (long)k * plane_out;
        for (int co = 0; co < cout_g; ++co) {
          const T s = wg[(long)co * k_g + k];
          const T *gr = gg + (long)co * plane_out;
          for (long p = 0; p < plane_out; ++p) o[p] += s * gr[p];
        }
      }
    }
    FN(col2im_coord)(columns, im_b, off_b, mask_b, Cin, H, W, kh, kw, ph, pw, sh,
                     sw, dh, dw, dgroups, Ho, Wo,
                     grad_offset + (long)b * dgroups * 2 * taps * plane_out,
                     grad_mask + (long)b * dgroups * taps * plane_out);
    FN(col2im)(columns, off_b, mask_b, Cin, H, W, kh, kw, ph, pw, sh, sw, dh, dw,
               dgroups, Ho, Wo, grad_input + (long)b * Cin * H * W);
    FN(im2col)(im_b, off_b, mask_b, Cin, H, W, kh, kw, ph, pw, sh, sw, dh, dw,
               dgroups, Ho, Wo, columns);
    /* grad_weight[g] (cout_g x k_g) += gout[g] (cout_g x P) * columns[g]^T */
    for (int g = 0; g < groups; ++g) {
      const T *gg = gout + (long)g * cout_g * plane_out;
      const T *cg = columns + (long)g * k_g * plane_out;
      T *gw = grad_weight + (long)g * cout_g * k_g;
#pragma omp parallel for schedule(static)
      for (int co = 0; co < cout_g; ++co) {
        const T *gr = gg + (long)co * plane_out;
        for (int k = 0; k < k_g; ++k) {
          const T *cr = cg + (long)k * plane_out;
          T s = 0;
          for (long p = 0; p < plane_out; ++p) s += gr[p] * cr[p];
          gw[(long)co * k_g + k] += s;
        }
        if (grad_bias) {
          T s = 0;
          for (long p = 0; p < plane_out; ++p) s += gr[p];
          grad_bias[g * cout_g + co] += s;
        }
      }
    }
  }
  return 0;
}
