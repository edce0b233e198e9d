// Backward of the (modulated) deformable convolution: gradients with respect to
// input, offset, mask, weight and bias
// (mmcv/ops/csrc/pytorch/modulated_deform_conv.cpp:140-251 and the kernels
// cpu/modulated_deform_conv.cpp:34-107,170-320).  The reference materialises the
// column gradient W^T * grad_output per sample and runs three element-wise
// kernels and two library GEMMs over it; here nothing of column size reaches
// memory:
//   bwd_data_kernel    one thread per (image, deformable group, tap, output
//                      pixel), a workgroup sharing (image, group, tap): builds the column gradients of its channels on
//                      the fly and turns them into grad_offset, grad_mask (plain
//                      stores, every element has one owner) and grad_input
//                      (fp32 atomics, four corners per channel),
//   bwd_weight_kernel  grad_weight = grad_output * columns^T as an MFMA GEMM
//                      whose reduction runs over pixels; the columns tile is
//                      sampled into LDS and never stored,
//   bwd_bias_kernel    row sums of grad_output.
// Accumulation is fp32 throughout; 16-bit tensors receive their gradients through
// fp32 staging buffers in the workspace (round_kernel).
#pragma once

#include "mdcn_common.h"
#include "mdcn_fused.h"

namespace mdcn {

template <typename T>
__global__ __launch_bounds__(256) void fill_zero_kernel(T *p, long n) {
  // 16 bytes per thread and step where the buffer starts aligned (workspace regions do), the rest one by one
  const long first = (long)blockIdx.x * blockDim.x + threadIdx.x, stride = (long)gridDim.x * blockDim.x;
  constexpr long PER = 16 / (long)sizeof(T);
  const long nv = ((uintptr_t)p % 16 == 0) ? n / PER : 0;
  for (long i = first; i < nv; i += stride) ((uint4 *)p)[i] = make_uint4(0u, 0u, 0u, 0u);
  for (long i = nv * PER + first; i < n; i += stride) p[i] = (T)0;
}

template <typename E>
__global__ __launch_bounds__(256) void round_kernel(const float *__restrict__ src, E *__restrict__ dst,
                                                    long n) {
  // eight elements per thread and step (two 16-byte loads; the store lands wherever the caller's tensor
  // starts: global memory takes unaligned accesses), the rest one by one
  const long first = (long)blockIdx.x * blockDim.x + threadIdx.x, stride = (long)gridDim.x * blockDim.x;
  struct In4 { float x, y, z, w; };   // (four floats with the alignment of one)
  struct Out8 { E v[8]; };
  const long nv = n / 8;
  for (long i = first; i < nv; i += stride) {
    const In4 a = ((const In4 *)src)[2 * i], b = ((const In4 *)src)[2 * i + 1];
    Out8 o;
    o.v[0] = from_f32<E>(a.x); o.v[1] = from_f32<E>(a.y); o.v[2] = from_f32<E>(a.z); o.v[3] = from_f32<E>(a.w);
    o.v[4] = from_f32<E>(b.x); o.v[5] = from_f32<E>(b.y); o.v[6] = from_f32<E>(b.z); o.v[7] = from_f32<E>(b.w);
    __builtin_memcpy(dst + 8 * i, &o, sizeof(o));
  }
  for (long i = nv * 8 + first; i < n; i += stride) dst[i] = from_f32<E>(src[i]);
}

// Pixels of one image a block of bwd_bias_kernel sums.
constexpr int kBiasRun = 8192;

// grad_bias[co] = sum over images and pixels of grad_output[:, co]: block (co, s)
// sums every `splits`-th run of kBiasRun pixels of channel co and adds its share
// to the fp32 sum with one atomic.
template <typename E>
__global__ __launch_bounds__(256) void bwd_bias_kernel(Geom g, const E *__restrict__ gout,
                                                       float *__restrict__ gbias32, int runs_per_image,
                                                       int splits) {
  __shared__ float part[4];
  const int co = blockIdx.x;
  const long plane = (long)g.Ho * g.Wo;
  const long work = (long)g.N * runs_per_image;
  float s = 0.0f;
  for (long wi = blockIdx.y; wi < work; wi += splits) {
    const int n = (int)(wi / runs_per_image);
    const long p0 = (wi - (long)n * runs_per_image) * kBiasRun;
    const long p1 = min(plane, p0 + kBiasRun);
    const E *row = gout + ((long)n * g.Cout + co) * plane;
    constexpr int EPV = 16 / (int)sizeof(E);  // elements per 16-byte load
    if (plane % EPV == 0 && ((uintptr_t)gout % 16) == 0) {  // (runs start at multiples of kBiasRun)
      const long nv = (p1 - p0) / EPV;
      const uint4 *src = (const uint4 *)(row + p0);
      // four loads in flight per thread: a run is a handful of loads deep, so their latency is the cost
      for (long v0 = 0; v0 < nv; v0 += 4 * 256) {
        uint4 q[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const long v = v0 + u * 256 + threadIdx.x;
          q[u] = v < nv ? src[v] : make_uint4(0u, 0u, 0u, 0u);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const E *e = (const E *)&q[u];
#pragma unroll
          for (int i = 0; i < EPV; ++i) s += to_f32(e[i]);
        }
      }
      for (long p = p0 + nv * EPV + threadIdx.x; p < p1; p += 256) s += to_f32(row[p]);
    } else {
      for (long p = p0 + threadIdx.x; p < p1; p += 256) s += to_f32(row[p]);
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o);
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x == 0) unsafeAtomicAdd(gbias32 + co, (part[0] + part[1]) + (part[2] + part[3]));
}

// Channels whose column gradient a thread of bwd_data_kernel holds at a time.
constexpr int kBwdChunk = 16;
// Output channels of one weight slice staged in LDS at a time.
constexpr int kBwdCoTile = 256;

// One workgroup per (n, dg, tap) and run of 256 output pixels, one thread per
// pixel.  For the channels of the deformable group, kBwdChunk at a time:
//   d[c] = sum_co weight[co, c, tap] * grad_output[n, co, pixel]    (the column gradient)
//   grad_mask   += d[c] * bilinear(x[c], pos)
//   grad_offset += d[c] * mask * d(bilinear)/d(pos)                  (y, then x)
//   grad_input[c, corner] += d[c] * mask * corner weight             (atomics)
// with the forward's sampling rule: nothing for a position outside (-1,H)x(-1,W),
// no contribution from a corner outside the image
// (cpu/modulated_deform_conv.cpp:34-107,170-320).  The weight slice
// [co tile][chunk] of the workgroup's tap goes through LDS as fp32 and is read
// back as broadcasts, so the inner loop costs one grad_output load and four LDS
// reads per 16 multiply-adds.
template <typename E>
__global__ __launch_bounds__(256) void bwd_data_kernel(Geom g, const E *__restrict__ input,
                                                       OffMaskView om, const E *__restrict__ weight,
                                                       const E *__restrict__ gout,
                                                       float *__restrict__ gin32, E *__restrict__ goff,
                                                       E *__restrict__ gmask, int rows) {
  __shared__ float4 wl[kBwdCoTile][kBwdChunk / 4];
  const long plane_out = (long)g.Ho * g.Wo;
  const long plane_in = (long)g.H * g.W;
  const int tid = threadIdx.x;
  const long pix_raw = (long)blockIdx.x * 256 + tid;
  const bool valid = pix_raw < plane_out;
  const long pix = valid ? pix_raw : 0;
  const int ho = (int)(pix / g.Wo), wo = (int)(pix - (long)ho * g.Wo);

  for (int row = blockIdx.y; row < rows; row += gridDim.y) {  // row = (n, dg, tap), workgroup uniform
    const int tap = row % g.taps;
    const int dgi = (row / g.taps) % g.DG;
    const int n = row / (g.taps * g.DG);
    const int ti = tap / g.kw, tj = tap - ti * g.kw;

    const E *off = (const E *)om.off + (long)n * om.off_n + pix * om.off_px +
                   (long)(dgi * 2 * g.taps) * om.off_ch;
    const E *msk = (const E *)om.msk + (long)n * om.msk_n + pix * om.msk_px +
                   (long)(dgi * g.taps) * om.msk_ch;
    const float dy = to_f32(off[(long)(2 * tap) * om.off_ch]);
    const float dx = to_f32(off[(long)(2 * tap + 1) * om.off_ch]);
    const float m = mask_value<E>(msk[(long)tap * om.msk_ch], om.logit);
    const float py = (float)(ho * g.sh - g.ph + ti * g.dh) + dy;
    const float px = (float)(wo * g.sw - g.pw + tj * g.dw) + dx;
    const bool inside =
        valid && (py > -1.0f) && (px > -1.0f) && (py < (float)g.H) && (px < (float)g.W);
    const float fy = floorf(py), fx = floorf(px);
    const int y0 = inside ? (int)fy : 0, x0 = inside ? (int)fx : 0, y1 = y0 + 1, x1 = x0 + 1;
    const float ly = py - fy, lx = px - fx, hy = 1.0f - ly, hx = 1.0f - lx;
    const bool ok00 = inside && y0 >= 0 && x0 >= 0, ok01 = inside && y0 >= 0 && x1 <= g.W - 1;
    const bool ok10 = inside && y1 <= g.H - 1 && x0 >= 0, ok11 = inside && y1 <= g.H - 1 && x1 <= g.W - 1;
    const long o00 = (long)y0 * g.W + x0, o01 = o00 + 1, o10 = o00 + g.W, o11 = o10 + 1;

    float acc_m = 0.0f, acc_y = 0.0f, acc_x = 0.0f;
    const int c_begin = dgi * g.ch_per_dg, c_end = c_begin + g.ch_per_dg;
    for (int c0 = c_begin; c0 < c_end;) {
      // a chunk stays inside one convolution group
      const int grp = c0 / g.cin_g;
      const int cn = min(kBwdChunk, min(c_end, (grp + 1) * g.cin_g) - c0);
      float d[kBwdChunk];
#pragma unroll
      for (int cc = 0; cc < kBwdChunk; ++cc) d[cc] = 0.0f;
      const E *grow = gout + ((long)n * g.Cout + (long)grp * g.cout_g) * plane_out + pix;
      const E *wrow = weight + ((long)grp * g.cout_g * g.cin_g + (c0 - grp * g.cin_g)) * g.taps + tap;
      for (int cot = 0; cot < g.cout_g; cot += kBwdCoTile) {
        const int ncot = min(kBwdCoTile, g.cout_g - cot);
        __syncthreads();  // the previous slice has been read
        {
          float w16[kBwdChunk];
          const E *wc = wrow + (long)(cot + min(tid, ncot - 1)) * g.cin_g * g.taps;
#pragma unroll
          for (int cc = 0; cc < kBwdChunk; ++cc)
            w16[cc] = (cc < cn && tid < ncot) ? to_f32(wc[(long)cc * g.taps]) : 0.0f;
#pragma unroll
          for (int q = 0; q < kBwdChunk / 4; ++q)
            wl[tid][q] = make_float4(w16[4 * q], w16[4 * q + 1], w16[4 * q + 2], w16[4 * q + 3]);
        }
        __syncthreads();
        if (inside) {
          for (int co = 0; co < ncot; ++co) {
            const float gv = to_f32(grow[(long)(cot + co) * plane_out]);
#pragma unroll
            for (int q = 0; q < kBwdChunk / 4; ++q) {
              const float4 w4 = wl[co][q];
              d[4 * q] += w4.x * gv;
              d[4 * q + 1] += w4.y * gv;
              d[4 * q + 2] += w4.z * gv;
              d[4 * q + 3] += w4.w * gv;
            }
          }
        }
      }
      if (inside) {
#pragma unroll
        for (int cc = 0; cc < kBwdChunk; ++cc) {
          if (cc < cn) {
            const int c = c0 + cc;
            const E *im = input + ((long)n * g.Cin + c) * plane_in;
            const float v00 = ok00 ? to_f32(im[o00]) : 0.0f, v01 = ok01 ? to_f32(im[o01]) : 0.0f;
            const float v10 = ok10 ? to_f32(im[o10]) : 0.0f, v11 = ok11 ? to_f32(im[o11]) : 0.0f;
            const float dc = d[cc];
            acc_m += dc * ((hy * hx) * v00 + (hy * lx) * v01 + (ly * hx) * v10 + (ly * lx) * v11);
            acc_y += dc * (hx * (v10 - v00) + lx * (v11 - v01));
            acc_x += dc * (hy * (v01 - v00) + ly * (v11 - v10));
            const float t = dc * m;
            float *gi = gin32 + ((long)n * g.Cin + c) * plane_in;
            if (ok00) unsafeAtomicAdd(gi + o00, (hy * hx) * t);
            if (ok01) unsafeAtomicAdd(gi + o01, (hy * lx) * t);
            if (ok10) unsafeAtomicAdd(gi + o10, (ly * hx) * t);
            if (ok11) unsafeAtomicAdd(gi + o11, (ly * lx) * t);
          }
        }
      }
      c0 += cn;
    }
    if (valid) {
      const long ob = ((long)n * g.DG + dgi) * 2 * g.taps;
      goff[(ob + 2 * tap) * plane_out + pix] = from_f32<E>(acc_y * m);
      goff[(ob + 2 * tap + 1) * plane_out + pix] = from_f32<E>(acc_x * m);
      if (gmask) gmask[(((long)n * g.DG + dgi) * g.taps + tap) * plane_out + pix] = from_f32<E>(acc_m);
    }
  }
}

// Tiled variant of bwd_data_kernel for kernels of up to 9 taps: a workgroup owns a
// 16 x 16 tile of output pixels of one (image, deformable group) and walks all
// taps itself, so that the scatter into grad_input can be summed in LDS first.
// The taps of a tile and of neighbouring pixels hit the same few input pixels
// again and again (256 pixels x 9 taps x 4 corners land in a window of roughly
// (16 + 2R)^2 pixels): per chunk of kBwdChunk channels the workgroup keeps an fp32
// window [kBwdChunk][WH][WW] of grad_input around its tile, adds into it with LDS
// atomics, and flushes the non-zero entries with one global atomic each; corners
// outside the window go to global memory directly.  grad_offset / grad_mask sums
// stay in registers per (pixel, tap) across the channel chunks.
constexpr int kBwdTile = 16;
constexpr int kBwdTapsMax = 9;
constexpr int kBwdWindowBytes = 48 * 1024;

struct BwdDataTiledArgs {
  Geom g;
  const void *input;
  OffMaskView om;
  const void *weight;
  const void *gout;
  float *gin32;
  void *goff;
  void *gmask;  // null when unmodulated
  int tiles_x, tiles_y;
  int WH, WW;   // window size in input pixels
  int R;        // margin of the window around the tile's undeformed footprint
};

// Output channels of one all-taps weight slice in LDS.
constexpr int kBwdTiledCoTile = 16;

template <typename E>
__global__ __launch_bounds__(256, 2) void bwd_data_tiled_kernel(BwdDataTiledArgs a) {
  // weight slice [co][tap][chunk] of the current channel chunk, fp32
  __shared__ float4 wl[kBwdTiledCoTile][kBwdTapsMax][kBwdChunk / 4];
  __shared__ float win[kBwdWindowBytes / 4];
  const Geom &g = a.g;
  const long plane_out = (long)g.Ho * g.Wo;
  const long plane_in = (long)g.H * g.W;
  const int tid = threadIdx.x;
  int b = blockIdx.x;
  const int tx = b % a.tiles_x;
  b /= a.tiles_x;
  const int ty = b % a.tiles_y;
  b /= a.tiles_y;
  const int dgi = b % g.DG;
  const int n = b / g.DG;
  const int ho = ty * kBwdTile + (tid >> 4), wo = tx * kBwdTile + (tid & 15);
  const bool valid = ho < g.Ho && wo < g.Wo;
  const long pix = valid ? (long)ho * g.Wo + wo : 0;
  // window origin in input coordinates
  const int wy0 = ty * kBwdTile * g.sh - g.ph - a.R, wx0 = tx * kBwdTile * g.sw - g.pw - a.R;
  const int win_px = a.WH * a.WW;

  const E *input = (const E *)a.input, *weight = (const E *)a.weight, *gout = (const E *)a.gout;
  const E *off = (const E *)a.om.off + (long)n * a.om.off_n + pix * a.om.off_px +
                 (long)(dgi * 2 * g.taps) * a.om.off_ch;
  const E *msk = (const E *)a.om.msk + (long)n * a.om.msk_n + pix * a.om.msk_px +
                 (long)(dgi * g.taps) * a.om.msk_ch;

  float acc_m[kBwdTapsMax], acc_y[kBwdTapsMax], acc_x[kBwdTapsMax];
#pragma unroll
  for (int t = 0; t < kBwdTapsMax; ++t) acc_m[t] = acc_y[t] = acc_x[t] = 0.0f;

  const int c_begin = dgi * g.ch_per_dg, c_end = c_begin + g.ch_per_dg;
  for (int c0 = c_begin; c0 < c_end;) {
    const int grp = c0 / g.cin_g;  // a chunk stays inside one convolution group
    const int cn = min(kBwdChunk, min(c_end, (grp + 1) * g.cin_g) - c0);
    __syncthreads();  // the previous chunk's flush is done
    for (int i = tid; i < win_px * kBwdChunk; i += 256) win[i] = 0.0f;
    // (the barriers of the slice loop order the zeroing before any add)

    // ---- column gradients of the chunk for every tap: one grad_output load per
    //      (output channel, pixel) feeds taps x chunk multiply-adds ----
    static_assert(kBwdChunk == 16, "one 16-float vector per tap");
    f32x16 d[kBwdTapsMax];  // (vectors, so that the compiler keeps them in registers)
#pragma unroll
    for (int t = 0; t < kBwdTapsMax; ++t)
#pragma unroll
      for (int cc = 0; cc < kBwdChunk; ++cc) d[t][cc] = 0.0f;
    const E *grow = gout + ((long)n * g.Cout + (long)grp * g.cout_g) * plane_out + pix;
    const E *wrow = weight + ((long)grp * g.cout_g * g.cin_g + (c0 - grp * g.cin_g)) * g.taps;
    for (int cot = 0; cot < g.cout_g; cot += kBwdTiledCoTile) {
      const int ncot = min(kBwdTiledCoTile, g.cout_g - cot);
      __syncthreads();  // the previous slice has been read
      // slice element (co, tap, cc) <- weight[cot + co][c0 + cc][tap]; 16 * 9 * 16 = 2304 elements
      for (int i = tid; i < kBwdTiledCoTile * kBwdTapsMax * kBwdChunk; i += 256) {
        const int cc = i % kBwdChunk, t = (i / kBwdChunk) % kBwdTapsMax, co = i / (kBwdChunk * kBwdTapsMax);
        float v = 0.0f;
        if (co < ncot && t < g.taps && cc < cn)
          v = to_f32(wrow[((long)(cot + co) * g.cin_g + cc) * g.taps + t]);
        ((float *)wl)[i] = v;
      }
      __syncthreads();
      if (valid) {
        for (int co = 0; co < ncot; ++co) {
          const float gv = to_f32(grow[(long)(cot + co) * plane_out]);
#pragma unroll
          for (int t = 0; t < kBwdTapsMax; ++t)
#pragma unroll
            for (int q = 0; q < kBwdChunk / 4; ++q) {
              const float4 w4 = wl[co][t][q];
              d[t][4 * q] += w4.x * gv;
              d[t][4 * q + 1] += w4.y * gv;
              d[t][4 * q + 2] += w4.z * gv;
              d[t][4 * q + 3] += w4.w * gv;
            }
        }
      }
    }

    // ---- per tap: offset / mask sums and the scatter ----
#pragma unroll
    for (int tap = 0; tap < kBwdTapsMax; ++tap) {
      if (tap < g.taps) {
        const int ti = tap / g.kw, tj = tap - ti * g.kw;
        const float dy = to_f32(off[(long)(2 * tap) * a.om.off_ch]);
        const float dx = to_f32(off[(long)(2 * tap + 1) * a.om.off_ch]);
        const float m = mask_value<E>(msk[(long)tap * a.om.msk_ch], a.om.logit);
        const float py = (float)(ho * g.sh - g.ph + ti * g.dh) + dy;
        const float px = (float)(wo * g.sw - g.pw + tj * g.dw) + dx;
        const bool inside =
            valid && (py > -1.0f) && (px > -1.0f) && (py < (float)g.H) && (px < (float)g.W);
        if (inside) {
          const float fy = floorf(py), fx = floorf(px);
          const int y0 = (int)fy, x0 = (int)fx, y1 = y0 + 1, x1 = x0 + 1;
          const float ly = py - fy, lx = px - fx, hy = 1.0f - ly, hx = 1.0f - lx;
          const bool ok00 = y0 >= 0 && x0 >= 0, ok01 = y0 >= 0 && x1 <= g.W - 1;
          const bool ok10 = y1 <= g.H - 1 && x0 >= 0, ok11 = y1 <= g.H - 1 && x1 <= g.W - 1;
          const long o00 = (long)y0 * g.W + x0, o01 = o00 + 1, o10 = o00 + g.W, o11 = o10 + 1;
          // the 2x2 block inside the window?  (then all four corners are)
          const int ry = y0 - wy0, rx = x0 - wx0;
          const bool in_win = ry >= 0 && ry + 1 < a.WH && rx >= 0 && rx + 1 < a.WW;
          const int wbase = ry * a.WW + rx;  // window is [channel][WH][WW]: neighbouring pixels, neighbouring banks
          float am = 0.0f, ay = 0.0f, ax = 0.0f;
#pragma unroll
          for (int cc = 0; cc < kBwdChunk; ++cc) {
            if (cc < cn) {
              const int c = c0 + cc;
              const E *im = input + ((long)n * g.Cin + c) * plane_in;
              const float v00 = ok00 ? to_f32(im[o00]) : 0.0f, v01 = ok01 ? to_f32(im[o01]) : 0.0f;
              const float v10 = ok10 ? to_f32(im[o10]) : 0.0f, v11 = ok11 ? to_f32(im[o11]) : 0.0f;
              const float dc = d[tap][cc];
              am += dc * ((hy * hx) * v00 + (hy * lx) * v01 + (ly * hx) * v10 + (ly * lx) * v11);
              ay += dc * (hx * (v10 - v00) + lx * (v11 - v01));
              ax += dc * (hy * (v01 - v00) + ly * (v11 - v10));
              const float t = dc * m;
              if (in_win) {
                float *wp = win + cc * win_px + wbase;
                if (ok00) atomicAdd(wp, (hy * hx) * t);
                if (ok01) atomicAdd(wp + 1, (hy * lx) * t);
                if (ok10) atomicAdd(wp + a.WW, (ly * hx) * t);
                if (ok11) atomicAdd(wp + a.WW + 1, (ly * lx) * t);
              } else {
                float *gi = a.gin32 + ((long)n * g.Cin + c) * plane_in;
                if (ok00) unsafeAtomicAdd(gi + o00, (hy * hx) * t);
                if (ok01) unsafeAtomicAdd(gi + o01, (hy * lx) * t);
                if (ok10) unsafeAtomicAdd(gi + o10, (ly * hx) * t);
                if (ok11) unsafeAtomicAdd(gi + o11, (ly * lx) * t);
              }
            }
          }
          acc_m[tap] += am;
          acc_y[tap] += ay * m;
          acc_x[tap] += ax * m;
        }
      }
    }
    __syncthreads();  // every add into the window has landed
    for (int i = tid; i < win_px * kBwdChunk; i += 256) {
      const float v = win[i];
      if (v != 0.0f) {
        const int cc = i / win_px, q = i - cc * win_px;
        const int y = wy0 + q / a.WW, x = wx0 + q % a.WW;  // in the image: only valid corners were added
        unsafeAtomicAdd(a.gin32 + ((long)n * g.Cin + c0 + cc) * plane_in + (long)y * g.W + x, v);
      }
    }
    c0 += cn;
  }
  if (valid) {
    E *goff = (E *)a.goff, *gmask = (E *)a.gmask;
    const long ob = ((long)n * g.DG + dgi) * 2 * g.taps;
#pragma unroll
    for (int tap = 0; tap < kBwdTapsMax; ++tap) {
      if (tap < g.taps) {
        goff[(ob + 2 * tap) * plane_out + pix] = from_f32<E>(acc_y[tap]);
        goff[(ob + 2 * tap + 1) * plane_out + pix] = from_f32<E>(acc_x[tap]);
        if (gmask) gmask[(((long)n * g.DG + dgi) * g.taps + tap) * plane_out + pix] = from_f32<E>(acc_m[tap]);
      }
    }
  }
}

struct BwdWeightArgs {
  Geom g;
  const void *input;
  OffMaskView om;
  const void *gout;
  float *gw32;       // (Cout, cin_g, kh, kw) fp32, zero before the launch
  int k_tiles;       // ceil(cin_g * taps / 64)
  int co_tiles;      // ceil(cout_g / 256)
  int px_chunks;     // 64-pixel chunks per image
  int splits;        // workgroups sharing the (image, chunk) range of one tile
  int g_vec_ok;      // grad_output rows may be read 16 bytes at a time
};

// grad_weight[co, k] += sum_pixels grad_output[co, pixel] * col[k, pixel], k = (channel, tap)
// of one group.  Workgroup = 256 output channels x 64 k of one group, for a share
// of the (image, 64-pixel chunk) range; wave w owns channels 64w..64w+63 as 2x2
// MFMA blocks.  Per chunk the 256 threads sample the 64 x 64 columns tile into
// LDS (element type E, rows of 64 pixels, 16-byte chunks swizzled by row), then
// A fragments (channel row, 16 bytes of pixels) come straight from grad_output
// and B fragments (k row, 16 bytes of pixels) from LDS.  The partial sums leave
// through fp32 atomics.
template <typename E>
__global__ __launch_bounds__(256) void bwd_weight_kernel(BwdWeightArgs a) {
  using TR = ElemTraits<E>;
  constexpr int ES = (int)sizeof(E);
  constexpr int PXC = 16 / ES;          // pixels per 16-byte chunk
  constexpr int NCH = 64 / PXC;         // chunks per 64-pixel row
  __shared__ uint4 colT[64 * NCH];
  const Geom &g = a.g;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int frow = lane & 31, fhalf = lane >> 5;
  const long plane_out = (long)g.Ho * g.Wo;
  const long plane_in = (long)g.H * g.W;
  const int k_g = g.cin_g * g.taps;

  int b = blockIdx.x;
  const int kt = b % a.k_tiles;
  b /= a.k_tiles;
  const int ct = b % a.co_tiles;
  const int grp = b / a.co_tiles;
  const int split = blockIdx.y;

  // the 16 columns rows this thread samples: k = kbase + tid / 64 + 4 * i
  const int kbase = kt * 64;
  const int spx = tid & 63;  // ... at pixel spx of the chunk
  int s_c[16], s_tap[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int k = kbase + (tid >> 6) + 4 * i;
    s_c[i] = k < k_g ? grp * g.cin_g + k / g.taps : -1;
    s_tap[i] = k < k_g ? k % g.taps : 0;
  }

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  const int co_base = ct * 256 + wave * 64;  // within the group
  const E *gout = (const E *)a.gout;
  const long work = (long)g.N * a.px_chunks;
  for (long wi = split; wi < work; wi += a.splits) {
    const int n = (int)(wi / a.px_chunks);
    const int p0 = (int)(wi - (long)n * a.px_chunks) * 64;
    // ---- columns tile -> LDS ----
    {
      const int p = p0 + spx;
      const bool pv = p < plane_out;
      const int ho = pv ? p / g.Wo : 0, wo = pv ? p - ho * g.Wo : 0;
      E *c16 = (E *)colT;
#pragma unroll 4
      for (int i = 0; i < 16; ++i) {
        const int kk = (tid >> 6) + 4 * i;
        float v = 0.0f;
        if (pv && s_c[i] >= 0) {
          const int c = s_c[i], tap = s_tap[i];
          const int dgi = c / g.ch_per_dg;
          const int ti = tap / g.kw, tj = tap - ti * g.kw;
          const E *off = (const E *)a.om.off + (long)n * a.om.off_n + (long)p * a.om.off_px +
                         (long)(dgi * 2 * g.taps) * a.om.off_ch;
          const E *msk = (const E *)a.om.msk + (long)n * a.om.msk_n + (long)p * a.om.msk_px +
                         (long)(dgi * g.taps) * a.om.msk_ch;
          const TapSample s = make_tap_sample(
              ho * g.sh - g.ph + ti * g.dh, wo * g.sw - g.pw + tj * g.dw,
              to_f32(off[(long)(2 * tap) * a.om.off_ch]), to_f32(off[(long)(2 * tap + 1) * a.om.off_ch]),
              mask_value<E>(msk[(long)tap * a.om.msk_ch], a.om.logit), g.H, g.W);
          if (s.inside) {
            const E *im = (const E *)a.input + ((long)n * g.Cin + c) * plane_in;
            const int y1 = s.y0 + 1, x1 = s.x0 + 1;
            if (s.y0 >= 0 && s.x0 >= 0) v += s.w00 * to_f32(im[s.y0 * g.W + s.x0]);
            if (s.y0 >= 0 && x1 <= g.W - 1) v += s.w01 * to_f32(im[s.y0 * g.W + x1]);
            if (y1 <= g.H - 1 && s.x0 >= 0) v += s.w10 * to_f32(im[y1 * g.W + s.x0]);
            if (y1 <= g.H - 1 && x1 <= g.W - 1) v += s.w11 * to_f32(im[y1 * g.W + x1]);
          }
        }
        const int chunk = (spx / PXC) ^ (kk & (NCH - 1) & 7);
        c16[(kk * NCH + chunk) * PXC + (spx % PXC)] = from_f32<E>(v);
      }
    }
    __syncthreads();
    // ---- MFMA over the 64 pixels ----
#pragma unroll
    for (int step = 0; step < NCH / 2; ++step) {
      const int ch = step * 2 + fhalf;
      uint4 af[2], bf[2];
#pragma unroll
      for (int mb = 0; mb < 2; ++mb) {
        const int co = co_base + mb * 32 + frow;
        const int p = p0 + ch * PXC;
        af[mb] = make_uint4(0u, 0u, 0u, 0u);
        if (co < g.cout_g) {
          const E *row = gout + ((long)n * g.Cout + (long)grp * g.cout_g + co) * plane_out + p;
          if (a.g_vec_ok && p + PXC <= plane_out) {
            af[mb] = *(const uint4 *)row;
          } else {
            alignas(16) E tmp[PXC];
#pragma unroll
            for (int e = 0; e < PXC; ++e) tmp[e] = (p + e < plane_out) ? row[e] : from_f32<E>(0.0f);
            af[mb] = *(const uint4 *)tmp;
          }
        }
      }
#pragma unroll
      for (int nb = 0; nb < 2; ++nb) {
        const int kk = nb * 32 + frow;
        bf[nb] = colT[kk * NCH + (ch ^ (kk & (NCH - 1) & 7))];
      }
#pragma unroll
      for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) TR::mma(acc[mb][nb], af[mb], bf[nb]);
    }
    __syncthreads();
  }

  // A rows = output channels, B rows = k: register r of lane l holds
  //   channel = (r/4)*8 + (l/32)*4 + r%4,  k = l%32   of its block.
#pragma unroll
  for (int mb = 0; mb < 2; ++mb)
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int co = co_base + mb * 32 + (r >> 2) * 8 + fhalf * 4 + (r & 3);
        const int k = kbase + nb * 32 + frow;
        if (co < g.cout_g && k < k_g)
          unsafeAtomicAdd(a.gw32 + ((long)grp * g.cout_g + co) * k_g + k, acc[mb][nb][r]);
      }
}

}  // namespace mdcn
