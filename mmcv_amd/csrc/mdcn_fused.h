// Fused DCNv2 forward for gfx950: implicit GEMM  out[cout, pixel] = W[cout, k] * S[k, pixel]
// where S (the "columns" of the reference's two-pass design,
// mmcv/ops/csrc/pytorch/modulated_deform_conv.cpp:101-124) is produced on the
// fly -- offset/mask-modulated bilinear samples computed by the wavefronts and
// written straight into LDS tiles that feed MFMA -- and never exists in HBM.
//
// Work split.  One workgroup (4 wavefronts, 256 lanes) owns a tile of PT = 128
// consecutive output pixels (flattened n*Ho*Wo + ho*Wo + wo) x CT output
// channels of one group.  K runs over (channel slab of KC channels) x (tap),
// slab outer, tap inner, so that the KC-channel slice of the neighbourhood a
// tile samples stays cache resident across the kh*kw taps.
//
// Per tile, once per deformable group: a table in LDS holds, for every
// (pixel, tap), the pixel index of the top-left bilinear corner inside the
// zero-bordered channels-last input copy and the four mask-scaled bilinear
// weights.  Positions and weights are computed in fp32.
//
// Per K step: each lane gathers, for one pixel, 32 contiguous bytes of channels
// at each of the four corners (global_load_dwordx4 x 8), blends them, and
// writes 32 bytes of the sample tile; the weight tile is copied from its
// pre-packed form.  Loads for step k+1 are issued before the MFMAs of step k;
// LDS tiles are double buffered, one barrier per step.
//
// MFMA mapping: the "A" operand is the weight tile (rows = output channels),
// the "B" operand the sample tile (columns = pixels), so that in the 32x32
// accumulator block lane%32 indexes the pixel and stores of one register are
// contiguous along W in the NCHW output.
#pragma once

#include "mdcn_common.h"

namespace mdcn {

constexpr int kPT = 128;    // pixels per workgroup tile
constexpr int kRowB = 80;   // LDS bytes per tile row: 64 data + 16 pad (keeps 16-byte
                            // reads of 16 consecutive rows on distinct banks)

struct FusedArgs {
  Geom g;
  const void *xt;      // zero-bordered channels-last input copy
  const void *wp;      // packed weights
  const void *offset;
  const void *mask;
  const void *bias;    // may be null
  void *out;
  long total_px;       // N * Ho * Wo
  int n_ptiles, n_ctiles, slabs;
  uint32_t pix_bytes;  // Cin * sizeof(E)
  uint32_t row_bytes;  // Wp * Cin * sizeof(E)
};

template <typename E>
struct ElemTraits;

// ---- 16-bit element types: v_dot2c blend, 32x32x16 MFMA --------------------
template <typename E>
struct Half16Traits {
  static constexpr int KC = 32;    // channels per K step (64 bytes)
  static constexpr int NACC = 16;  // samples per lane per K step
  static constexpr int TW = 2;     // table dwords per (pixel, tap) for the weights

  static __device__ __forceinline__ uint32_t pack2(float lo, float hi);
  static __device__ __forceinline__ float dot2(uint32_t d, uint32_t w, float acc);

  static __device__ __forceinline__ void store_weights(const TapSample &s,
                                                       uint32_t (&tw)[TW]) {
    tw[0] = ElemTraits<E>::pack2(s.w00, s.w01);
    tw[1] = ElemTraits<E>::pack2(s.w10, s.w11);
  }

  // acc[2d], acc[2d+1] += w * (low, high) element of dword d.  The dword is fed
  // to v_dot2c unchanged, paired with (w, 0) resp. (0, w).
  static __device__ __forceinline__ void blend(float (&acc)[NACC],
                                               const uint4 (&v)[4][2],
                                               const uint32_t (&tw)[TW]) {
    const uint32_t wlo[4] = {tw[0] & 0xffffu, tw[0] >> 16, tw[1] & 0xffffu,
                             tw[1] >> 16};
    const uint32_t whi[4] = {tw[0] << 16, tw[0] & 0xffff0000u, tw[1] << 16,
                             tw[1] & 0xffff0000u};
#pragma unroll
    for (int i = 0; i < NACC; ++i) acc[i] = 0.0f;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const uint32_t d[4] = {v[q][h].x, v[q][h].y, v[q][h].z, v[q][h].w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int k = (h * 4 + j) * 2;
          acc[k] = ElemTraits<E>::dot2(d[j], wlo[q], acc[k]);
          acc[k + 1] = ElemTraits<E>::dot2(d[j], whi[q], acc[k + 1]);
        }
      }
    }
  }

  static __device__ __forceinline__ void pack_samples(const float (&acc)[NACC],
                                                      uint4 (&o)[2]) {
    o[0] = make_uint4(ElemTraits<E>::pack2(acc[0], acc[1]),
                      ElemTraits<E>::pack2(acc[2], acc[3]),
                      ElemTraits<E>::pack2(acc[4], acc[5]),
                      ElemTraits<E>::pack2(acc[6], acc[7]));
    o[1] = make_uint4(ElemTraits<E>::pack2(acc[8], acc[9]),
                      ElemTraits<E>::pack2(acc[10], acc[11]),
                      ElemTraits<E>::pack2(acc[12], acc[13]),
                      ElemTraits<E>::pack2(acc[14], acc[15]));
  }
};

template <>
struct ElemTraits<bf16_t> : Half16Traits<bf16_t> {
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    bf16x2 p;
    p.x = (bf16_t)lo;
    p.y = (bf16_t)hi;
    return __builtin_bit_cast(uint32_t, p);
  }
  static __device__ __forceinline__ float dot2(uint32_t d, uint32_t w, float acc) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, d),
                                           __builtin_bit_cast(bf16x2, w), acc,
                                           false);
  }
  // 16 bytes = 8 consecutive K elements of one row per lane.
  static __device__ __forceinline__ void mma(f32x16 &c, const uint4 &a,
                                             const uint4 &b) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                __builtin_bit_cast(bf16x8, b),
                                                c, 0, 0, 0);
  }
};

template <>
struct ElemTraits<f16_t> : Half16Traits<f16_t> {
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    f16x2 p;
    p.x = (f16_t)lo;
    p.y = (f16_t)hi;
    return __builtin_bit_cast(uint32_t, p);
  }
  static __device__ __forceinline__ float dot2(uint32_t d, uint32_t w, float acc) {
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, d),
                                  __builtin_bit_cast(f16x2, w), acc, false);
  }
  static __device__ __forceinline__ void mma(f32x16 &c, const uint4 &a,
                                             const uint4 &b) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                               __builtin_bit_cast(f16x8, b), c,
                                               0, 0, 0);
  }
};

// ---- fp32: scalar FMA blend, 32x32x2 fp32 MFMA ------------------------------
template <>
struct ElemTraits<float> {
  static constexpr int KC = 16;
  static constexpr int NACC = 8;
  static constexpr int TW = 4;

  static __device__ __forceinline__ void store_weights(const TapSample &s,
                                                       uint32_t (&tw)[TW]) {
    tw[0] = __float_as_uint(s.w00);
    tw[1] = __float_as_uint(s.w01);
    tw[2] = __float_as_uint(s.w10);
    tw[3] = __float_as_uint(s.w11);
  }

  static __device__ __forceinline__ void blend(float (&acc)[NACC],
                                               const uint4 (&v)[4][2],
                                               const uint32_t (&tw)[TW]) {
#pragma unroll
    for (int i = 0; i < NACC; ++i) acc[i] = 0.0f;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const float w = __uint_as_float(tw[q]);
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        acc[h * 4 + 0] += w * __uint_as_float(v[q][h].x);
        acc[h * 4 + 1] += w * __uint_as_float(v[q][h].y);
        acc[h * 4 + 2] += w * __uint_as_float(v[q][h].z);
        acc[h * 4 + 3] += w * __uint_as_float(v[q][h].w);
      }
    }
  }

  static __device__ __forceinline__ void pack_samples(const float (&acc)[NACC],
                                                      uint4 (&o)[2]) {
    o[0] = make_uint4(__float_as_uint(acc[0]), __float_as_uint(acc[1]),
                      __float_as_uint(acc[2]), __float_as_uint(acc[3]));
    o[1] = make_uint4(__float_as_uint(acc[4]), __float_as_uint(acc[5]),
                      __float_as_uint(acc[6]), __float_as_uint(acc[7]));
  }

  // 16 bytes = 4 consecutive K elements of one row per lane; element j of both
  // operands goes to the j-th 32x32x2 MFMA.
  static __device__ __forceinline__ void mma(f32x16 &c, const uint4 &a,
                                             const uint4 &b) {
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.x),
                                             __uint_as_float(b.x), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.y),
                                             __uint_as_float(b.y), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.z),
                                             __uint_as_float(b.z), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.w),
                                             __uint_as_float(b.w), c, 0, 0, 0);
  }
};

// LDS bytes of one workgroup of fused_kernel<E, CT>.
template <typename E>
constexpr size_t fused_lds_bytes(int CT, int taps) {
  return (size_t)2 * kPT * kRowB + (size_t)2 * CT * kRowB +
         (size_t)kPT * taps * 4 * (1 + ElemTraits<E>::TW);
}

template <typename E, int CT>
__global__ __launch_bounds__(256, 2) void fused_kernel(FusedArgs a) {
  using TR = ElemTraits<E>;
  constexpr int PT = kPT;
  constexpr int KC = TR::KC;
  constexpr int TW = TR::TW;
  constexpr int MB = CT / 64;  // 32-row accumulator blocks per wave along Cout
  constexpr int NB = 2;        // ... along pixels (64 pixels per wave)
  constexpr int WREG = CT / 64;  // 16-byte weight-tile pieces per lane

  const Geom &g = a.g;
  const int taps = g.taps;

  // XCD-aware tile order: consecutive workgroup ids go to different XCDs, so
  // give each XCD one contiguous run of tiles (shared halo rows stay in its L2).
  const int total_wg = a.n_ptiles * a.n_ctiles * g.G;
  const int chunk = (total_wg + 7) >> 3;
  int L = (int)(blockIdx.x & 7) * chunk + (int)(blockIdx.x >> 3);
  if (L >= total_wg) return;
  const int ctile = L % a.n_ctiles;
  L /= a.n_ctiles;
  const int grp = L % g.G;
  const int ptile = L / g.G;

  extern __shared__ __align__(16) unsigned char smem[];
  unsigned char *Xs = smem;                        // [2][PT][kRowB]
  unsigned char *Ws = Xs + 2 * PT * kRowB;         // [2][CT][kRowB]
  int32_t *tpix = (int32_t *)(Ws + 2 * CT * kRowB);  // [taps][PT]
  uint32_t *tws = (uint32_t *)(tpix + PT * taps);    // [TW][taps][PT]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_c = wave >> 1;  // which half of the Cout tile
  const int wave_p = wave & 1;   // which half of the pixel tile

  const long plane_out = (long)g.Ho * g.Wo;
  const long p0 = (long)ptile * PT;

  // ---- (pixel, tap) table for one deformable group ------------------------
  // Entry e = tap*PT + pixel; this lane always serves pixel tid%128.
  const int tb_pl = tid & (PT - 1);
  const long tb_p = p0 + tb_pl;
  const bool tb_valid = tb_p < a.total_px;
  int tb_n = 0, tb_ho = 0, tb_wo = 0;
  long tb_rem = 0;
  if (tb_valid) {
    tb_n = (int)(tb_p / plane_out);
    tb_rem = tb_p - (long)tb_n * plane_out;
    tb_ho = (int)(tb_rem / g.Wo);
    tb_wo = (int)(tb_rem - (long)tb_ho * g.Wo);
  }
  auto build_table = [&](int dgi) {
    const E *off = (const E *)a.offset +
                   ((long)tb_n * g.DG + dgi) * 2 * taps * plane_out + tb_rem;
    const E *msk = (const E *)a.mask +
                   ((long)tb_n * g.DG + dgi) * taps * plane_out + tb_rem;
    for (int tap = tid >> 7; tap < taps; tap += 2) {
      int32_t pix = 0;
      uint32_t tw[TW];
#pragma unroll
      for (int i = 0; i < TW; ++i) tw[i] = 0u;
      if (tb_valid) {
        const float dy = to_f32(off[(long)(2 * tap) * plane_out]);
        const float dx = to_f32(off[(long)(2 * tap + 1) * plane_out]);
        const float m = to_f32(msk[(long)tap * plane_out]);
        const int i = tap / g.kw, j = tap - i * g.kw;
        const TapSample s =
            make_tap_sample(tb_ho * g.sh - g.ph + i * g.dh,
                            tb_wo * g.sw - g.pw + j * g.dw, dy, dx, m, g.H, g.W);
        // +1: coordinates in the zero-bordered copy.  y0, x0 are in [-1, H-1] x
        // [-1, W-1] when inside, 0 otherwise (weights are 0 then).
        pix = (tb_n * g.Hp + (s.y0 + 1)) * g.Wp + (s.x0 + 1);
        TR::store_weights(s, tw);
      }
      const int e = tap * PT + tb_pl;
      tpix[e] = pix;
#pragma unroll
      for (int i = 0; i < TW; ++i) tws[i * (PT * taps) + e] = tw[i];
    }
  };

  // ---- producer state: this lane gathers pixel g_px, 32 bytes per corner --
  const int g_px = tid >> 1;
  const uint32_t g_half = (uint32_t)(tid & 1) * 32u;
  const unsigned char *xt = (const unsigned char *)a.xt;
  const uint32_t grp_ch_bytes = (uint32_t)(grp * g.cin_g) * (uint32_t)sizeof(E);

  uint4 gv[4][2];       // gathered corner data of the step in flight
  uint32_t gtw[TW];     // its blend weights
  uint4 wreg[WREG];     // its weight-tile pieces

  const int nk = a.slabs * taps;
  const unsigned char *wp_tile =
      (const unsigned char *)a.wp +
      ((size_t)(grp * a.n_ctiles + ctile) * nk) * (size_t)(CT * 64);

  auto issue_loads = [&](int ks) {
    const int slab = ks / taps;
    const int tap = ks - slab * taps;
    const int e = tap * PT + g_px;
    const uint32_t pix = (uint32_t)tpix[e];
#pragma unroll
    for (int i = 0; i < TW; ++i) gtw[i] = tws[i * (PT * taps) + e];
    const uint32_t o = pix * a.pix_bytes + grp_ch_bytes +
                       (uint32_t)(slab * KC) * (uint32_t)sizeof(E) + g_half;
    const uint32_t co[4] = {o, o + a.pix_bytes, o + a.row_bytes,
                            o + a.row_bytes + a.pix_bytes};
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const uint4 *p = (const uint4 *)(xt + co[q]);
      gv[q][0] = p[0];
      gv[q][1] = p[1];
    }
    const uint4 *wt = (const uint4 *)(wp_tile + (size_t)ks * (CT * 64));
#pragma unroll
    for (int i = 0; i < WREG; ++i) wreg[i] = wt[tid + 256 * i];
  };

  auto commit_tiles = [&](int buf) {
    float acc[TR::NACC];
    TR::blend(acc, gv, gtw);
    uint4 o[2];
    TR::pack_samples(acc, o);
    uint4 *xs = (uint4 *)(Xs + (buf * PT + g_px) * kRowB + g_half);
    xs[0] = o[0];
    xs[1] = o[1];
#pragma unroll
    for (int i = 0; i < WREG; ++i) {
      const int q = tid + 256 * i;
      *(uint4 *)(Ws + (buf * CT + (q >> 2)) * kRowB + (q & 3) * 16) = wreg[i];
    }
  };

  f32x16 acc[MB][NB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[mb][nb][r] = 0.0f;

  const int frag_row = lane & 31;
  const int frag_off = (lane >> 5) * 16;

  auto mma_phase = [&](int buf) {
#pragma unroll
    for (int ksub = 0; ksub < 2; ++ksub) {
      uint4 wf[MB], xf[NB];
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
        wf[mb] = *(const uint4 *)(Ws +
                                  (buf * CT + wave_c * (CT / 2) + mb * 32 + frag_row) * kRowB +
                                  ksub * 32 + frag_off);
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
        xf[nb] = *(const uint4 *)(Xs +
                                  (buf * PT + wave_p * 64 + nb * 32 + frag_row) * kRowB +
                                  ksub * 32 + frag_off);
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) TR::mma(acc[mb][nb], wf[mb], xf[nb]);
    }
  };

  // ---- main loop ----------------------------------------------------------
  const int ch0 = grp * g.cin_g;  // first input channel of this group
  int cur_dg = ch0 / g.ch_per_dg;
  build_table(cur_dg);
  __syncthreads();
  issue_loads(0);
  commit_tiles(0);
  __syncthreads();

  for (int ks = 0; ks < nk; ++ks) {
    const int buf = ks & 1;
    const bool has_next = (ks + 1) < nk;
    if (has_next) {
      const int nslab = (ks + 1) / taps;
      const int ndg = (ch0 + nslab * KC) / g.ch_per_dg;
      if (ndg != cur_dg) {  // uniform over the workgroup
        // Every lane read the table for step ks before the barrier that ended
        // the previous iteration, so it can be overwritten now.
        cur_dg = ndg;
        build_table(cur_dg);
        __syncthreads();
      }
      issue_loads(ks + 1);
    }
    mma_phase(buf);
    if (has_next) commit_tiles(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue: bias, round once, NCHW store -----------------------------
  // Accumulator block: register r of lane l holds
  //   row (cout) = (r/4)*8 + (l/32)*4 + r%4,  column (pixel) = l%32.
  E *out = (E *)a.out;
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const long p = p0 + wave_p * 64 + nb * 32 + (lane & 31);
    if (p >= a.total_px) continue;
    const int n = (int)(p / plane_out);
    const long rem = p - (long)n * plane_out;
    E *obase = out + ((long)n * g.Cout + (long)grp * g.cout_g) * plane_out + rem;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int col = ctile * CT + wave_c * (CT / 2) + mb * 32 + (r >> 2) * 8 +
                        (lane >> 5) * 4 + (r & 3);
        if (col < g.cout_g) {
          float v = acc[mb][nb][r];
          if (a.bias) v += to_f32(((const E *)a.bias)[grp * g.cout_g + col]);
          obase[(long)col * plane_out] = from_f32<E>(v);
        }
      }
    }
  }
}

}  // namespace mdcn
