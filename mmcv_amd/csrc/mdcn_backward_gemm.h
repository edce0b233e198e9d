// Backward, data side, for channel counts that fill MFMA tiles: the column
// gradient  d[pixel, (tap, c)] = sum_co grad_output[co, pixel] * weight[co, c, tap]
// (the reference's first GEMM, mmcv/ops/csrc/pytorch/modulated_deform_conv.cpp:199-206)
// is a plain matrix product, so it runs on the matrix cores
// (bwd_colgrad_kernel) and is handed to the scatter kernel through memory in a
// layout made for that kernel: d[image][16-channel chunk][tap][pixel][16].  The
// scatter kernel (bwd_scatter_kernel) then is the reference's three element-wise
// kernels in one pass (cpu/modulated_deform_conv.cpp:34-107,170-320): a thread
// owns an output pixel, reads 4 to 16 channels of d and of the four corners (from
// the zero-bordered pixel-major input copy, 16 or 32 contiguous bytes per corner,
// one tap ahead of their use), forms its share of grad_offset / grad_mask from
// the four sums of d times a corner's values, and adds the grad_input
// contributions into an LDS window around its 8 x 32 pixel tile, which is flushed
// with one global atomic per non-zero entry.  On the way it can
// store the forward's columns, from which grad_weight is a second plain product
// (bwd_wgrad_kernel).
// Both operands of the product are pixel-major / K-contiguous copies written by
// small pre-passes (relayout_vec_kernel<E, false> for grad_output,
// pack_weight_t_kernel for the weights).
#pragma once

#include "mdcn_backward.h"

namespace mdcn {

// Rows of either operand per workgroup tile of the two products: 256 (8
// wavefronts, each 128 x 64) where both operands have that many rows, else 128
// (4 wavefronts, each 64 x 64).  Per K step a 256-tile moves 64 KB for 2 048 MFMA
// clocks, a 128-tile 32 KB for 512: with two K steps in flight the small tile is
// bound by the latency of its copies, the large one is not.
constexpr int kCgTile = 128;
constexpr int kCgTileBig = 256;

// Work index of a workgroup of a 1-D launch of 8 * ceil(total / 8) workgroups, or
// -1 for the few that have none.  Consecutive workgroup ids sit on different
// XCDs (each with its own L2); this hands every XCD one contiguous run of work
// indices, so that neighbours in the work order -- made to share an operand tile
// -- run on the same XCD at about the same time and fetch that tile from HBM
// once instead of once per XCD.
__device__ __forceinline__ long xcd_work_index(long total) {
  const long chunk = (total + 7) >> 3;
  const long xcd = blockIdx.x & 7, i = blockIdx.x >> 3;
  const long L = xcd * chunk + i;
  return (i < chunk && L < total) ? L : -1;
}

// weight[Cout][cin_g][taps] -> wT[G][M_pad][cout_g], row m = tap * cin_g + c,
// zero rows from taps * cin_g up to M_pad (a multiple of kCgTile).
template <typename E>
__global__ __launch_bounds__(256) void pack_weight_t_kernel(Geom g, const E *__restrict__ w,
                                                            E *__restrict__ wT, int M_pad, long total) {
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    long r = idx;
    const int co = (int)(r % g.cout_g);
    r /= g.cout_g;
    const int m = (int)(r % M_pad);
    const int grp = (int)(r / M_pad);
    E v = from_f32<E>(0.0f);
    if (m < g.taps * g.cin_g) {
      const int tap = m / g.cin_g, c = m - tap * g.cin_g;
      v = w[((long)(grp * g.cout_g + co) * g.cin_g + c) * g.taps + tap];
    }
    wT[idx] = v;
  }
}

struct ColGradArgs {
  const void *wT;  // [G][M_pad][cout_g]
  const void *gT;  // [N][Cout / KC][P][KC], KC = 128 bytes of channels
  void *D;         // [images of the pass][Cin / 16][taps][P][16]
  int P;           // output pixels per image
  int px_tiles, m_tiles;
  int M, M_pad;    // taps * cin_g and its padded size
  int cin_g, cout_g, taps, G, Cin, Cout;
  int kslabs;      // cout_g / KC
  int n0;          // first image of the pass
  long total;      // workgroups with work: images of the pass x G x px_tiles x m_tiles
  uint32_t *dmax;  // bit pattern of the largest |d| stored so far (a float >= 0), or null
};

// Workgroup = TILE rows of wT (one group) x TILE pixels of one image, reduction
// over the group's output channels in slabs of 128 bytes; TILE / 32 waves as
// 2 x TILE / 64, each TILE / 64 x 2 MFMA blocks of 32 x 32.  Both operand tiles of a slab go to LDS with
// 16-byte direct-to-LDS copies (rows of 128 bytes, the 16-byte chunks of a row
// swizzled by the row number on the source side, so that fragment reads are
// conflict free), double buffered.  A rows = (tap, channel), B rows = pixels:
// a lane ends up with 4 x 4 consecutive channels of one pixel, which is what the
// d layout wants (8- or 16-byte stores).
template <typename E, int TILE>
__global__ __launch_bounds__(TILE * 2, TILE == 128 ? 2 : 1) void bwd_colgrad_kernel(ColGradArgs a) {
  using TR = ElemTraits<E>;
  constexpr int ES = (int)sizeof(E);
  constexpr int KC = 128 / ES;
  constexpr int MB = TILE / 64;            // 32-row blocks of A per wave
  constexpr uint32_t kBuf = TILE * 128u;   // bytes of one operand tile
  __shared__ uint4 As[2][TILE * 8];
  __shared__ uint4 Bs[2][TILE * 8];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int frow = lane & 31, fhalf = lane >> 5;
  const int wm = wave & 1, wn = wave >> 1;
  // (the row tiles of one pixel tile are neighbours: they share the grad_output tile)
  long b = xcd_work_index(a.total);
  if (b < 0) return;
  const int mt = (int)(b % a.m_tiles);
  b /= a.m_tiles;
  const int pt = (int)(b % a.px_tiles);
  b /= a.px_tiles;
  const int grp = (int)(b % a.G);
  const int nl = (int)(b / a.G);
  const int n = a.n0 + nl;

  // this lane's share of the copies: 4 of the 16 one-KiB blocks (8 rows) of each tile
  const unsigned char *a_src[4], *b_src[4];
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int row = (wave * 4 + c) * 8 + (lane >> 3);
    const int ch = (lane & 7) ^ (row & 7);
    a_src[c] = (const unsigned char *)a.wT +
               ((long)grp * a.M_pad + (long)mt * TILE + row) * a.cout_g * ES + ch * 16;
    // rows past the image repeat its last pixel; they are never stored
    const int px = min(pt * TILE + row, a.P - 1);
    b_src[c] = (const unsigned char *)a.gT +
               (((long)n * (a.Cout / KC) + (long)grp * a.kslabs) * a.P + px) * 128 + ch * 16;
  }
  const long b_step = (long)a.P * 128;
  const uint32_t lds_a = (uint32_t)(uintptr_t)(lptr_t)(&As[0][0]) +
                         (uint32_t)__builtin_amdgcn_readfirstlane(wave) * 4096u;
  const uint32_t lds_b = (uint32_t)(uintptr_t)(lptr_t)(&Bs[0][0]) +
                         (uint32_t)__builtin_amdgcn_readfirstlane(wave) * 4096u;
  auto issue = [&](int ks, int buf) {
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      copy16_global_to_lds(a_src[c] + (long)ks * 128, lds_a + (uint32_t)buf * kBuf + (uint32_t)c * 1024u);
      copy16_global_to_lds(b_src[c] + (long)ks * b_step, lds_b + (uint32_t)buf * kBuf + (uint32_t)c * 1024u);
    }
  };

  f32x16 acc[MB][2];
#pragma unroll
  for (int i = 0; i < MB; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  issue(0, 0);
  for (int ks = 0; ks < a.kslabs; ++ks) {
    const int buf = ks & 1;
    if (ks + 1 < a.kslabs) {
      issue(ks + 1, buf ^ 1);  // (its buffer was last read before the barrier that ended step ks - 1)
      asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    } else {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    __syncthreads();
#pragma unroll
    for (int ksub = 0; ksub < 4; ++ksub) {
      uint4 af[MB], bf[2];
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const int row = wm * (TILE / 2) + mb * 32 + frow;
        af[mb] = As[buf][row * 8 + ((ksub * 2 + fhalf) ^ (row & 7))];
      }
#pragma unroll
      for (int nb = 0; nb < 2; ++nb) {
        const int row = wn * 64 + nb * 32 + frow;
        bf[nb] = Bs[buf][row * 8 + ((ksub * 2 + fhalf) ^ (row & 7))];
      }
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) TR::mma(acc[mb][nb], af[mb], bf[nb]);
    }
    __syncthreads();
  }

  // register r of lane l: A row (r/4)*8 + (l/32)*4 + r%4 of the block, B row l%32
  E *D = (E *)a.D;
  const int chunks = a.Cin / 16;
  if (a.dmax) {  // (every accumulator counts: rows and pixels past the end repeat real ones or are zero)
    float mx = 0.0f;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int nb = 0; nb < 2; ++nb)
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, fabsf(acc[mb][nb][r]));
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
    // (non-negative floats order like their bits; the plain read first keeps all but the few
    // waves that raise the maximum from queueing on one address)
    if (lane == 0 && __float_as_uint(mx) > __builtin_nontemporal_load(a.dmax)) atomicMax(a.dmax, __float_as_uint(mx));
  }
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int m0 = mt * TILE + wm * (TILE / 2) + mb * 32;  // a block = one tap, 32 consecutive channels
    if (m0 >= a.M) continue;
    const int tap = m0 / a.cin_g;
    const int cb = grp * a.cin_g + (m0 - tap * a.cin_g);
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
      const int px = pt * TILE + wn * 64 + nb * 32 + frow;
      if (px >= a.P) continue;
      // The two halves of the wave exchange their 4-channel groups so that a lane holds 8 consecutive
      // channels: one 16-byte store per lane and 16 channels, 32 pixels x 32 bytes contiguous per instruction
      // (the lower half takes the first 8 channels of a 16-channel chunk, the upper half the second 8).
      if constexpr (sizeof(E) == 2) {
#pragma unroll
        for (int jp = 0; jp < 2; ++jp) {
          const f32x16 &c16 = acc[mb][nb];
          const int ja = 2 * jp, jb = 2 * jp + 1;
          const uint32_t a0 = TR::pack2(c16[4 * ja], c16[4 * ja + 1]), a1 = TR::pack2(c16[4 * ja + 2], c16[4 * ja + 3]);
          const uint32_t b0 = TR::pack2(c16[4 * jb], c16[4 * jb + 1]), b1 = TR::pack2(c16[4 * jb + 2], c16[4 * jb + 3]);
          const auto s0 = __builtin_amdgcn_permlane32_swap(a0, b0, false, false);
          const auto s1 = __builtin_amdgcn_permlane32_swap(a1, b1, false, false);
          const int c = cb + jp * 16 + fhalf * 8;
          E *dst = D + ((((long)nl * chunks + (c >> 4)) * a.taps + tap) * a.P + px) * 16 + (c & 15);
          *(uint4 *)dst = make_uint4(s0[0], s1[0], s0[1], s1[1]);
        }
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int c = cb + j * 8 + fhalf * 4;
          E *dst = D + ((((long)nl * chunks + (c >> 4)) * a.taps + tap) * a.P + px) * 16 + (c & 15);
          TR::store4((unsigned char *)dst, acc[mb][nb][4 * j], acc[mb][nb][4 * j + 1],
                     acc[mb][nb][4 * j + 2], acc[mb][nb][4 * j + 3]);
        }
      }
    }
  }
}

// Bytes of the scatter kernel's window (two workgroups per CU).  It holds CH
// channels of a WH x WW pixel neighbourhood of the tile; kScWindowPx pixels fit
// with the larger channel count of a type (16-bit tensors: 16 channels of 32-bit
// fixed point; fp32 tensors: 8 channels of doubles), twice as many -- stride 2,
// dilation -- with the smaller one.  (A 48 KB window with 8 channels and three
// workgroups per CU was slower: the passes over the window double.)
constexpr int kScWindowBytes = 60 * 1024;
constexpr int kScWindowPx = kScWindowBytes / 64;
// Contributions one window entry can receive at most: every (pixel, tap) of the
// tile touches an entry at most once per channel.
constexpr int kScMaxAdds = 256 * 9;

// largest |x| of a tensor, as the bit pattern of a non-negative float
template <typename E>
__global__ __launch_bounds__(256) void absmax_kernel(const E *__restrict__ x, long n, uint32_t *out) {
  float mx = 0.0f;
  constexpr int EPV = 16 / (int)sizeof(E);  // elements per 16-byte load
  const long nv = (((uintptr_t)x % 16) == 0) ? n / EPV : 0;
  for (long v = (long)blockIdx.x * blockDim.x + threadIdx.x; v < nv; v += (long)gridDim.x * blockDim.x) {
    const uint4 q = ((const uint4 *)x)[v];
    const E *e = (const E *)&q;
#pragma unroll
    for (int i = 0; i < EPV; ++i) mx = fmaxf(mx, fabsf(to_f32(e[i])));
  }
  for (long i = nv * EPV + (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x)
    mx = fmaxf(mx, fabsf(to_f32(x[i])));
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
  __shared__ float wmax[4];
  if ((threadIdx.x & 63) == 0) wmax[threadIdx.x >> 6] = mx;
  __syncthreads();
  if (threadIdx.x == 0)  // one atomic per workgroup: they all queue on one address
    atomicMax(out, __float_as_uint(fmaxf(fmaxf(wmax[0], wmax[1]), fmaxf(wmax[2], wmax[3]))));
}

// CH consecutive channels (8 to 32 bytes) as floats.
template <typename E, int CH>
struct VecCh {
  static constexpr int NW = CH * (int)sizeof(E) / 4;  // 32-bit words
  uint32_t raw[NW];
  __device__ __forceinline__ void load(const E *p) {
    if constexpr (NW % 4 == 0) {
#pragma unroll
      for (int i = 0; i < NW / 4; ++i) {
        const uint4 v = ((const uint4 *)p)[i];
        raw[4 * i] = v.x;
        raw[4 * i + 1] = v.y;
        raw[4 * i + 2] = v.z;
        raw[4 * i + 3] = v.w;
      }
    } else {
      static_assert(NW == 2, "8 bytes");
      const uint2 v = *(const uint2 *)p;
      raw[0] = v.x;
      raw[1] = v.y;
    }
  }
  // channels 2 i and 2 i + 1
  __device__ __forceinline__ void pair(int i, float &lo, float &hi) const {
    if constexpr (sizeof(E) == 4) {
      lo = __uint_as_float(raw[2 * i]);
      hi = __uint_as_float(raw[2 * i + 1]);
    } else {
      ElemTraits<E>::unpack2(raw[i], lo, hi);
    }
  }
  // acc + this's channels 2 i and 2 i + 1 times o's
  __device__ __forceinline__ float dot_pair(const VecCh &o, int i, float acc) const {
    if constexpr (sizeof(E) == 4) {
      acc = fmaf(__uint_as_float(raw[2 * i]), __uint_as_float(o.raw[2 * i]), acc);
      return fmaf(__uint_as_float(raw[2 * i + 1]), __uint_as_float(o.raw[2 * i + 1]), acc);
    } else {
      return ElemTraits<E>::dot2(raw[i], o.raw[i], acc);
    }
  }
  __device__ __forceinline__ void unpack(float (&out)[CH]) const {
    if constexpr (sizeof(E) == 4) {
#pragma unroll
      for (int i = 0; i < CH; ++i) out[i] = __uint_as_float(raw[i]);
    } else {
#pragma unroll
      for (int i = 0; i < NW; ++i) ElemTraits<E>::unpack2(raw[i], out[2 * i], out[2 * i + 1]);
    }
  }
};

// Output-pixel tile of the scatter kernel: 8 rows x 32 columns, one thread per
// pixel (rows of 32 keep the loads of d and the stores of the columns in 64-byte
// or longer runs, and the window around it stays under 48 KiB for a margin of 3).
constexpr int kScTH = 8;
constexpr int kScTW = 32;

struct BwdScatterArgs {
  Geom g;
  const void *xt;  // zero-bordered input copy in 32-byte records [N][Cin / RC][H + 2][W + 2][RC], RC = 32 bytes of channels
  OffMaskView om;
  const void *D;   // column gradient of the pass, layout of ColGradArgs::D; null: columns only
  float *gin32;
  void *goff;
  void *gmask;     // null when unmodulated
  void *col;       // columns of the pass [image][group][tap][channel of the group][P_pad], or null
  long P_pad;      // row pitch of col in elements
  int tiles_x, tiles_y;
  int WH, WW;      // window size in input pixels
  int R;           // margin of the window around the tile's undeformed footprint
  int n0;          // first image of the pass
  // A deformable group's channels are shared among `parts` workgroups per tile
  // (blockIdx.y), so that the launch has several times more workgroups than the
  // chip has room for and its last round is short; with parts > 1 each writes its
  // share of the offset / mask sums as floats to poff / pmask ([part][layout of
  // grad_offset / grad_mask]), which combine_parts_kernel adds up.
  int parts;
  float *poff, *pmask;
  long off_total, mask_total;  // elements of grad_offset / grad_mask
  // fixed-point window (16-bit tensors): largest |d| and largest |mask| (null: 1)
  const uint32_t *dmax, *mmax;
};

// out[i] = sum over parts of part[p][i], rounded once.  Four elements per thread
// and step where the parts start at multiples of 16 bytes (total a multiple of 4).
template <typename E>
__global__ __launch_bounds__(256) void combine_parts_kernel(const float *__restrict__ part, E *__restrict__ out,
                                                            long total, int parts) {
  const long first = (long)blockIdx.x * blockDim.x + threadIdx.x, stride = (long)gridDim.x * blockDim.x;
  const long nv = (total % 4 == 0 && (uintptr_t)part % 16 == 0) ? total / 4 : 0;
  struct Out4 { E v[4]; };
  for (long i = first; i < nv; i += stride) {
    float4 s = ((const float4 *)part)[i];
    for (int p = 1; p < parts; ++p) {
      const float4 t = ((const float4 *)(part + (long)p * total))[i];
      s.x += t.x; s.y += t.y; s.z += t.z; s.w += t.w;
    }
    Out4 o;
    o.v[0] = from_f32<E>(s.x); o.v[1] = from_f32<E>(s.y); o.v[2] = from_f32<E>(s.z); o.v[3] = from_f32<E>(s.w);
    __builtin_memcpy(out + 4 * i, &o, sizeof(o));
  }
  for (long i = nv * 4 + first; i < total; i += stride) {
    float s = 0.0f;
    for (int p = 0; p < parts; ++p) s += part[(long)p * total + i];
    out[i] = from_f32<E>(s);
  }
}

// The window is not fp32: LDS single-precision atomic adds are slow on this
// hardware (measured per wavefront instruction per CU: ds_add_f32 170 clocks,
// ds_add_f64 26, ds_add_u32 11, whatever the addresses).  fp32 tensors use a
// double-precision window (WT = double).  16-bit tensors use 32-bit fixed point
// (WT = int32_t): with B = max|d| * max|mask| bounding every contribution and at
// most kScMaxAdds contributions per entry, the scale 2^k <= 2^30 / (B * kScMaxAdds)
// cannot overflow, and one contribution is rounded to B * 2^-19 at worst -- two
// thousand times finer than the bf16/fp16 rounding of the result.  Integer sums
// are exact, so the window part of grad_input does not depend on the order of
// the adds.  Two channels share one 64-bit entry (ds_add_u64 costs 14 clocks
// where two ds_add_u32 cost 22): the even channel's value sign-extended plus the
// odd channel's shifted up by 32 bits; the low half's borrows and carries into
// the high half cancel when the entry is taken apart again (low = the entry's low
// word as a signed number, high = (entry - low) >> 32), since neither sum leaves
// 32 bits.
// DATA: the gradient part (a.D, window, offset / mask sums).  COL: the kernel
// stores the forward's columns (mask * bilinear sample, rounded to E as the
// reference's columns tensor is) to a.col for the weight-gradient product.  At
// least one of the two.
template <typename E, int CH, typename WT, bool DATA, bool COL>
__global__ __launch_bounds__(256, 2) void bwd_scatter_kernel(BwdScatterArgs a) {
  constexpr int RC = 32 / (int)sizeof(E);   // channels per record of the input copy
  static_assert(DATA || COL, "nothing to do");
  static_assert(CH <= RC && RC % CH == 0, "a pass reads a record or a whole fraction of one");
  static_assert(CH % 2 == 0, "fixed-point window entries hold two channels");
  constexpr bool kFixed = sizeof(WT) == 4;
  static_assert(kScTH * kScTW == 256, "one thread per pixel of the tile");
  static_assert(kScTH * kScTW * kBwdTapsMax <= kScMaxAdds, "bound on the adds per window entry");
  __shared__ __align__(16) WT win[DATA ? kScWindowBytes / sizeof(WT) : 4];
  float fx_scale = 1.0f, fx_inv = 1.0f;
  if (kFixed && DATA) {
    const float bound = __uint_as_float(*a.dmax) * (a.mmax ? __uint_as_float(*a.mmax) : 1.0f) * (float)kScMaxAdds;
    // largest power of two not above 2^30 / bound (any scale will do when everything is zero)
    const int e = (bound > 0.0f && bound < 3.0e38f) ? 29 - ilogbf(bound) : 0;
    fx_scale = ldexpf(1.0f, max(-120, min(120, e)));
    fx_inv = 1.0f / fx_scale;
  }
  const Geom &g = a.g;
  const long plane_out = (long)g.Ho * g.Wo;
  const long plane_in = (long)g.H * g.W;
  const long slab_px = (long)g.Hp * g.Wp;
  const int tid = threadIdx.x;
  int b = blockIdx.x;
  const int tx = b % a.tiles_x;
  b /= a.tiles_x;
  const int ty = b % a.tiles_y;
  b /= a.tiles_y;
  const int dgi = b % g.DG;
  const int nl = b / g.DG;
  const int n = a.n0 + nl;
  const int ho = ty * kScTH + tid / kScTW, wo = tx * kScTW + tid % kScTW;
  const bool valid = ho < g.Ho && wo < g.Wo;
  const long pix = valid ? (long)ho * g.Wo + wo : 0;
  const int wy0 = ty * kScTH * g.sh - g.ph - a.R, wx0 = tx * kScTW * g.sw - g.pw - a.R;
  const int win_px = a.WH * a.WW;

  const E *off = (const E *)a.om.off + (long)n * a.om.off_n + pix * a.om.off_px +
                 (long)(dgi * 2 * g.taps) * a.om.off_ch;
  const E *msk = (const E *)a.om.msk + (long)n * a.om.msk_n + pix * a.om.msk_px +
                 (long)(dgi * g.taps) * a.om.msk_ch;

  float acc_m[kBwdTapsMax], acc_y[kBwdTapsMax], acc_x[kBwdTapsMax];
#pragma unroll
  for (int t = 0; t < kBwdTapsMax; ++t) acc_m[t] = acc_y[t] = acc_x[t] = 0.0f;
  // this pixel's offsets and mask, fetched once: every channel pass needs them before it can
  // address its corners
  E t_dy[kBwdTapsMax], t_dx[kBwdTapsMax], t_m[kBwdTapsMax];
#pragma unroll
  for (int t = 0; t < kBwdTapsMax; ++t) {
    const int tc = min(t, g.taps - 1);
    t_dy[t] = off[(long)(2 * tc) * a.om.off_ch];
    t_dx[t] = off[(long)(2 * tc + 1) * a.om.off_ch];
    t_m[t] = msk[(long)tc * a.om.msk_ch];
  }

  const int part = blockIdx.y;
  const int ch_per_part = g.ch_per_dg / a.parts;
  const int c_begin = dgi * g.ch_per_dg + part * ch_per_part, c_end = c_begin + ch_per_part;

  // Window pixels this thread flushes (tid, tid + 256, ...) as offsets into an image plane, the same
  // in every pass; -1 for one outside the image or past the window (it only ever receives zeros).
  constexpr int NE = kFixed ? CH / 2 : CH;  // window entries per pixel
  constexpr int kSlots = DATA ? (kScWindowBytes / (NE * 8) + 255) / 256 : 1;
  int flush_at[kSlots];
  if constexpr (DATA) {
#pragma unroll
    for (int j = 0; j < kSlots; ++j) {
      const int q = tid + 256 * j;
      const int y = wy0 + q / a.WW, x = wx0 + q % a.WW;
      flush_at[j] = (q < win_px && y >= 0 && y < g.H && x >= 0 && x < g.W) ? y * g.W + x : -1;
    }
    // (the flush leaves the window zeroed for the next pass)
    for (int i = tid; i < kScWindowBytes / 16; i += 256) ((uint4 *)win)[i] = make_uint4(0u, 0u, 0u, 0u);
  }

  // One tap's sampling position and what was loaded there.  No branch around a tap's body: a
  // position outside the sampling range (or a lane past the image) samples the border's corner
  // pixel with weights, mask and d of zero, so it stores a column of zeros and adds zeros.
  // Per-corner conditions become weights of zero too: a wavefront pays for an LDS atomic
  // whether or not a lane sits it out, and a branch per corner and channel was most of the
  // instructions this kernel issued.
  struct Sample {
    int y0, x0;
    float ly, lx, m;
    bool inside;
    VecCh<E, CH> r00, r01, r10, r11, rd;
  };
  auto fetch = [&](int c0, int tap, E e_dy, E e_dx, E e_m, Sample &s) {
    const int ti = tap / g.kw, tj = tap - ti * g.kw;
    float dy = to_f32(e_dy);
    float dx = to_f32(e_dx);
    // (opaque to the optimiser: it would otherwise move the position arithmetic of all taps
    // out of the channel loop and spill what that keeps alive)
    asm volatile("" : "+v"(dy), "+v"(dx));
    const float py = (float)(ho * g.sh - g.ph + ti * g.dh) + dy;
    const float px = (float)(wo * g.sw - g.pw + tj * g.dw) + dx;
    s.inside = valid && (py > -1.0f) && (px > -1.0f) && (py < (float)g.H) && (px < (float)g.W);
    const float fy = floorf(py), fx = floorf(px);
    s.y0 = s.inside ? (int)fy : -1;
    s.x0 = s.inside ? (int)fx : -1;
    s.ly = s.inside ? py - fy : 0.0f;
    s.lx = s.inside ? px - fx : 0.0f;
    s.m = s.inside ? mask_value<E>(e_m, a.om.logit) : 0.0f;
    // corners outside the image read the copy's zero border
    const E *xp = (const E *)a.xt + (((long)n * (g.Cin / RC) + c0 / RC) * slab_px) * RC + (c0 % RC) +
                  ((long)(s.y0 + 1) * g.Wp + (s.x0 + 1)) * RC;
    s.r00.load(xp);
    s.r01.load(xp + RC);
    s.r10.load(xp + (long)g.Wp * RC);
    s.r11.load(xp + (long)(g.Wp + 1) * RC);
    if constexpr (DATA)
      s.rd.load((const E *)a.D + (((long)nl * (g.Cin / 16) + (c0 >> 4)) * g.taps + tap) * plane_out * 16 + pix * 16 +
                (c0 & 15));
  };
  // A tap's loads are issued one tap ahead, in front of the previous tap's stores and atomics
  // (a wait for loads also waits for every older store, and the compiler cannot move a load
  // above a store that might alias it); the last tap of a pass fetches the first of the next.
  Sample cur;
  fetch(c_begin, 0, t_dy[0], t_dx[0], t_m[0], cur);

  for (int c0 = c_begin; c0 < c_end; c0 += CH) {
    if constexpr (DATA) __syncthreads();  // the window is zero: first fill or the previous pass's flush
    // row of the columns matrix of channel c0 at tap 0 (a chunk stays inside one group)
    const int grp = c0 / g.cin_g;
    E *cbase = (E *)a.col + (((long)nl * g.Cin + (long)grp * g.cin_g) * g.taps + (c0 - grp * g.cin_g)) * a.P_pad + pix;
    const int c_next = min(c0 + CH, c_end - CH);  // (the last pass fetches its own first tap again: unused)
#pragma unroll
    for (int tap = 0; tap < kBwdTapsMax; ++tap) {
      if (tap < g.taps) {
        Sample nxt;
        {
          const bool more = tap + 1 < g.taps;  // workgroup uniform
          const int tn = tap + 1 < kBwdTapsMax ? tap + 1 : 0;  // (a constant once the loop is unrolled)
          fetch(more ? c0 : c_next, more ? tn : 0, more ? t_dy[tn] : t_dy[0], more ? t_dx[tn] : t_dx[0],
                more ? t_m[tn] : t_m[0], nxt);
        }
        const bool inside = cur.inside;
        const int y0 = cur.y0, x0 = cur.x0, y1 = y0 + 1, x1 = x0 + 1;
        const float ly = cur.ly, lx = cur.lx, hy = 1.0f - ly, hx = 1.0f - lx, m = cur.m;
        const bool ok00 = y0 >= 0 && x0 >= 0, ok01 = y0 >= 0 && x1 <= g.W - 1;
        const bool ok10 = y1 <= g.H - 1 && x0 >= 0, ok11 = y1 <= g.H - 1 && x1 <= g.W - 1;
        const float w00 = hy * hx, w01 = hy * lx, w10 = ly * hx, w11 = ly * lx;
        VecCh<E, CH> &rd = cur.rd;
        if constexpr (DATA) {
          const uint32_t keep = inside ? ~0u : 0u;  // (whatever d holds where nothing is sampled)
#pragma unroll
          for (int i = 0; i < VecCh<E, CH>::NW; ++i) rd.raw[i] &= keep;
        }
        const int ry = y0 - wy0, rx = x0 - wx0;
        const bool in_win = ry >= 0 && ry + 1 < a.WH && rx >= 0 && rx + 1 < a.WW;
        const bool to_win = inside && in_win;
        // window is [channel][WH][WW]: neighbouring pixels, neighbouring banks; a lane with nothing
        // for the window adds its zeros at an entry of its own
        const int wbase = to_win ? ry * a.WW + rx : (tid & 63);
        const float s00 = (to_win && ok00) ? w00 : 0.0f, s01 = (to_win && ok01) ? w01 : 0.0f;
        const float s10 = (to_win && ok10) ? w10 : 0.0f, s11 = (to_win && ok11) ? w11 : 0.0f;
        const float mts = m * fx_scale;
        // sums over the pass's channels of d times each corner's value: the offset and mask
        // gradients are combinations of these four
        float S00 = 0.0f, S01 = 0.0f, S10 = 0.0f, S11 = 0.0f;
        E cv[CH];
        // two channels at a time, straight from the loaded words
#pragma unroll
        for (int cp = 0; cp < CH / 2; ++cp) {
          if constexpr (DATA) {
            S00 = cur.r00.dot_pair(rd, cp, S00);
            S01 = cur.r01.dot_pair(rd, cp, S01);
            S10 = cur.r10.dot_pair(rd, cp, S10);
            S11 = cur.r11.dot_pair(rd, cp, S11);
          }
          if constexpr (COL) {
            float v00[2], v01[2], v10[2], v11[2];
            cur.r00.pair(cp, v00[0], v00[1]);
            cur.r01.pair(cp, v01[0], v01[1]);
            cur.r10.pair(cp, v10[0], v10[1]);
            cur.r11.pair(cp, v11[0], v11[1]);
#pragma unroll
            for (int h = 0; h < 2; ++h)
              cv[2 * cp + h] = from_f32<E>(m * (w00 * v00[h] + w01 * v01[h] + w10 * v10[h] + w11 * v11[h]));
          }
          if constexpr (DATA) {
            float d[2];
            rd.pair(cp, d[0], d[1]);
            if constexpr (kFixed) {
              // round(w * ts) to nearest even in one multiply-add: the sum's mantissa holds the
              // integer (|w * ts| < 2^19 by the choice of the scale).  An entry is the even
              // channel's value sign-extended plus the odd one's shifted up 32 bits.
              const float tl = d[0] * mts, th = d[1] * mts;
              auto entry = [](float w, float tl, float th) {
                const int lo = __float_as_int(fmaf(w, tl, 12582912.0f)) - 0x4B400000;
                const uint32_t hi = (uint32_t)__float_as_int(fmaf(w, th, 12582912.0f)) - 0x4B400000u + (uint32_t)(lo >> 31);
                return (unsigned long long)(uint32_t)lo | ((unsigned long long)hi << 32);
              };
              unsigned long long *wp = (unsigned long long *)win + cp * win_px + wbase;
              atomicAdd(wp, entry(s00, tl, th));
              atomicAdd(wp + 1, entry(s01, tl, th));
              atomicAdd(wp + a.WW, entry(s10, tl, th));
              atomicAdd(wp + a.WW + 1, entry(s11, tl, th));
            } else {
#pragma unroll
              for (int h = 0; h < 2; ++h) {
                const float t = d[h] * m;
                WT *wp = win + (2 * cp + h) * win_px + wbase;
                atomicAdd(wp, (WT)(s00 * t));
                atomicAdd(wp + 1, (WT)(s01 * t));
                atomicAdd(wp + a.WW, (WT)(s10 * t));
                atomicAdd(wp + a.WW + 1, (WT)(s11 * t));
              }
            }
          }
        }
        if constexpr (COL) {
          if (valid) {
            E *crow = cbase + (long)tap * g.cin_g * a.P_pad;
#pragma unroll
            for (int cc = 0; cc < CH; ++cc) crow[(long)cc * a.P_pad] = cv[cc];
          }
        }
        if constexpr (DATA) {
          acc_m[tap] += w00 * S00 + w01 * S01 + w10 * S10 + w11 * S11;
          acc_y[tap] += m * (hx * (S10 - S00) + lx * (S11 - S01));
          acc_x[tap] += m * (hy * (S01 - S00) + ly * (S11 - S10));
          if (inside && !in_win) {  // rare: corners beyond the window go to memory directly
            const long o00 = (long)y0 * g.W + x0, o01 = o00 + 1, o10 = o00 + g.W, o11 = o10 + 1;
            float d[CH];
            rd.unpack(d);
#pragma unroll
            for (int cc = 0; cc < CH; ++cc) {
              const float t = d[cc] * m;
              float *gi = a.gin32 + ((long)n * g.Cin + c0 + cc) * plane_in;
              if (ok00) unsafeAtomicAdd(gi + o00, w00 * t);
              if (ok01) unsafeAtomicAdd(gi + o01, w01 * t);
              if (ok10) unsafeAtomicAdd(gi + o10, w10 * t);
              if (ok11) unsafeAtomicAdd(gi + o11, w11 * t);
            }
          }
        }
        cur = nxt;
      }
    }
    if constexpr (DATA) {
      __syncthreads();  // every add into the window has landed
      float *gplane = a.gin32 + ((long)n * g.Cin + c0) * plane_in;
#pragma unroll
      for (int j = 0; j < kSlots; ++j) {
        if (flush_at[j] >= 0) {
          const int q = tid + 256 * j;
          float *gi = gplane + flush_at[j];
          if constexpr (kFixed) {
            long long *w64 = (long long *)win + q;
#pragma unroll
            for (int cp = 0; cp < NE; ++cp) {
              const long long e = w64[cp * win_px];
              if (e != 0) {
                w64[cp * win_px] = 0;
                const int lo = (int)(unsigned)(unsigned long long)e;
                const int hi = (int)((e - (long long)lo) >> 32);
                if (lo != 0) unsafeAtomicAdd(gi + (long)(2 * cp) * plane_in, (float)lo * fx_inv);
                if (hi != 0) unsafeAtomicAdd(gi + (long)(2 * cp + 1) * plane_in, (float)hi * fx_inv);
              }
            }
          } else {
#pragma unroll
            for (int cc = 0; cc < NE; ++cc) {
              const WT v = win[cc * win_px + q];
              if (v != (WT)0) {
                win[cc * win_px + q] = (WT)0;
                unsafeAtomicAdd(gi + (long)cc * plane_in, (float)v);
              }
            }
          }
        }
      }
    }
  }
  if constexpr (DATA) {
    if (valid) {
      const long ob = ((long)n * g.DG + dgi) * 2 * g.taps;
      const long mb = ((long)n * g.DG + dgi) * g.taps;
      if (a.parts == 1) {
        E *goff = (E *)a.goff, *gmask = (E *)a.gmask;
#pragma unroll
        for (int tap = 0; tap < kBwdTapsMax; ++tap) {
          if (tap < g.taps) {
            goff[(ob + 2 * tap) * plane_out + pix] = from_f32<E>(acc_y[tap]);
            goff[(ob + 2 * tap + 1) * plane_out + pix] = from_f32<E>(acc_x[tap]);
            if (gmask) gmask[(mb + tap) * plane_out + pix] = from_f32<E>(acc_m[tap]);
          }
        }
      } else {
        float *poff = a.poff + (long)part * a.off_total;
        float *pmask = a.gmask ? a.pmask + (long)part * a.mask_total : nullptr;
#pragma unroll
        for (int tap = 0; tap < kBwdTapsMax; ++tap) {
          if (tap < g.taps) {
            poff[(ob + 2 * tap) * plane_out + pix] = acc_y[tap];
            poff[(ob + 2 * tap + 1) * plane_out + pix] = acc_x[tap];
            if (pmask) pmask[(mb + tap) * plane_out + pix] = acc_m[tap];
          }
        }
      }
    }
  }
}

// Zeroes the padding columns [P, P_pad) of every row of the columns matrix.
template <typename E>
__global__ __launch_bounds__(256) void zero_col_pad_kernel(E *col, long rows, int P, long P_pad) {
  const int padn = (int)(P_pad - P);
  const long total = rows * padn;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
    const long r = i / padn;
    col[r * P_pad + P + (i - r * padn)] = from_f32<E>(0.0f);
  }
}

// dst[row][0 .. P_pad) = src[row][0 .. P), zeros behind: grad_output with rows that start 16-byte
// aligned, for images whose pixel count is not a multiple of the copy granule.
template <typename E>
__global__ __launch_bounds__(256) void pad_rows_kernel(const E *__restrict__ src, E *__restrict__ dst, long rows,
                                                       int P, long P_pad) {
  const long total = rows * P_pad;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
    const long r = i / P_pad;
    const long p = i - r * P_pad;
    dst[i] = p < P ? src[r * P + p] : from_f32<E>(0.0f);
  }
}

struct WGradArgs {
  const void *gout;  // [N][Cout][a_pitch]: grad_output in place (a_pitch = P) or its padded copy (P_pad)
  long a_pitch;
  const void *col;   // [images of the pass][G][taps][cin_g][P_pad]
  float *part;       // partial sums [split][G][cout_g][M], every element written
  int P;
  long P_pad;
  int ksteps;        // P_pad / (pixels per 128 bytes)
  int nb, n0;        // images of the pass, first image
  int M;             // taps * cin_g
  int cin_g, cout_g, taps, G, Cin, Cout;
  int co_tiles, m_tiles;
  int splits;        // workgroups sharing the (image, K step) range of one tile
  long total;        // workgroups with work: G x co_tiles x m_tiles x splits
};

// grad_weight[co, (c, tap)] += sum over the pass's images and pixels of
// grad_output[co, pixel] * col[(tap, c), pixel]: a plain product with the pixels
// as reduction dimension (the reference's second GEMM,
// mmcv/ops/csrc/pytorch/modulated_deform_conv.cpp:227-237).  Workgroup = 128
// output channels x 128 column rows of one group over a share of the (image,
// 128-byte pixel run) steps; both operand tiles go to LDS with direct copies as
// in bwd_colgrad_kernel (grad_output is read in place: its rows are pixel
// contiguous).  Runs of pixels past the end of an image read the row's last
// 16 bytes again; the zero padding of col cancels them.  Rows past the group's
// channels repeat its last row and are dropped at the end.  Each share of the K
// range stores its partial tile (plain stores, rows of M contiguous);
// wgrad_reduce_kernel adds the shares up in a fixed order, so grad_weight does
// not vary from run to run.
template <typename E, int TILE>
__global__ __launch_bounds__(TILE * 2, TILE == 128 ? 2 : 1) void bwd_wgrad_kernel(WGradArgs a) {
  using TR = ElemTraits<E>;
  constexpr int ES = (int)sizeof(E);
  constexpr int PXC = 16 / ES;  // pixels per 16-byte chunk
  constexpr int MB = TILE / 64;
  constexpr uint32_t kBuf = TILE * 128u;
  __shared__ uint4 As[2][TILE * 8];
  __shared__ uint4 Bs[2][TILE * 8];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int frow = lane & 31, fhalf = lane >> 5;
  const int wm = wave & 1, wn = wave >> 1;
  // (all tiles of one share of the K range are neighbours: those of a row of
  // tiles share the grad_output tile, those of a column the columns tile)
  long b = xcd_work_index(a.total);
  if (b < 0) return;
  const int ct = (int)(b % a.co_tiles);
  b /= a.co_tiles;
  const int mt = (int)(b % a.m_tiles);
  b /= a.m_tiles;
  const int grp = (int)(b % a.G);
  const int split = (int)(b / a.G);

  // this lane's rows and 16-byte chunk of the copies
  long a_row[4], b_row[4];
  int chunk[4];
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int row = (wave * 4 + c) * 8 + (lane >> 3);
    chunk[c] = (lane & 7) ^ (row & 7);
    const int co = min(ct * TILE + row, a.cout_g - 1);
    const int m = min(mt * TILE + row, a.M - 1);
    a_row[c] = ((long)grp * a.cout_g + co) * a.a_pitch;      // + n * Cout * a_pitch
    b_row[c] = ((long)grp * a.M + m) * a.P_pad;              // + nl * taps * Cin * P_pad
  }
  const uint32_t lds_a = (uint32_t)(uintptr_t)(lptr_t)(&As[0][0]) +
                         (uint32_t)__builtin_amdgcn_readfirstlane(wave) * 4096u;
  const uint32_t lds_b = (uint32_t)(uintptr_t)(lptr_t)(&Bs[0][0]) +
                         (uint32_t)__builtin_amdgcn_readfirstlane(wave) * 4096u;
  const E *gout = (const E *)a.gout, *col = (const E *)a.col;
  const int last_chunk_px = (int)a.a_pitch - PXC;  // (the pitch is a multiple of PXC)
  auto issue = [&](long wi, int buf) {
    const int nl = (int)(wi / a.ksteps);
    const int p0 = (int)(wi - (long)nl * a.ksteps) * (8 * PXC);
    const E *ga = gout + (long)(a.n0 + nl) * a.Cout * a.a_pitch;
    const E *cb = col + (long)nl * a.taps * a.Cin * a.P_pad;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int px = p0 + chunk[c] * PXC;
      copy16_global_to_lds(ga + a_row[c] + min(px, last_chunk_px), lds_a + (uint32_t)buf * kBuf + (uint32_t)c * 1024u);
      copy16_global_to_lds(cb + b_row[c] + px, lds_b + (uint32_t)buf * kBuf + (uint32_t)c * 1024u);
    }
  };

  f32x16 acc[MB][2];
#pragma unroll
  for (int i = 0; i < MB; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  // this workgroup's contiguous share of the (image, K step) range
  const long work = (long)a.nb * a.ksteps;
  const long per = (work + a.splits - 1) / a.splits;
  const long w_begin = (long)split * per, w_end = min(work, w_begin + per);
  if (w_begin < w_end) {
    issue(w_begin, 0);
    int buf = 0;
    for (long wi = w_begin; wi < w_end; ++wi, buf ^= 1) {
      if (wi + 1 < w_end) {
        issue(wi + 1, buf ^ 1);
        asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
      } else {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      }
      __syncthreads();
#pragma unroll
      for (int ksub = 0; ksub < 4; ++ksub) {
        uint4 af[MB], bf[2];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
          const int row = wm * (TILE / 2) + mb * 32 + frow;
          af[mb] = As[buf][row * 8 + ((ksub * 2 + fhalf) ^ (row & 7))];
        }
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
          const int row = wn * 64 + nb * 32 + frow;
          bf[nb] = Bs[buf][row * 8 + ((ksub * 2 + fhalf) ^ (row & 7))];
        }
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
          for (int nb = 0; nb < 2; ++nb) TR::mma(acc[mb][nb], af[mb], bf[nb]);
      }
      __syncthreads();
    }
  }

  // register r of lane l: A row (output channel) (r/4)*8 + (l/32)*4 + r%4 of the block, B row (column row) l%32
  float *part = a.part + ((long)split * a.G + grp) * a.cout_g * a.M;
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
      const int m = mt * TILE + wn * 64 + nb * 32 + frow;
      if (m >= a.M) continue;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int co = ct * TILE + wm * (TILE / 2) + mb * 32 + (r >> 2) * 8 + fhalf * 4 + (r & 3);
        if (co < a.cout_g) part[(long)co * a.M + m] = acc[mb][nb][r];
      }
    }
}

// gw32[(grp, co), (c, tap)] += sum over the shares of part[share][grp][co][m = tap * cin_g + c].
__global__ __launch_bounds__(256) void wgrad_reduce_kernel(const float *__restrict__ part, float *__restrict__ gw32,
                                                           int splits, int cin_g, int taps, long n_w) {
  const int M = cin_g * taps;
  // four consecutive elements per thread (M is a multiple of 32 here: they share a row and a tap), the shares
  // in a fixed order with four loads in flight
  for (long i = 4 * ((long)blockIdx.x * blockDim.x + threadIdx.x); i < n_w; i += 4 * (long)gridDim.x * blockDim.x) {
    const long row = i / M;  // (grp, co)
    const int m = (int)(i - row * M);
    float4 sum = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    int sp = 0;
    for (; sp + 4 <= splits; sp += 4) {
      float4 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) v[u] = *(const float4 *)(part + (long)(sp + u) * n_w + i);
#pragma unroll
      for (int u = 0; u < 4; ++u) sum.x += v[u].x, sum.y += v[u].y, sum.z += v[u].z, sum.w += v[u].w;
    }
    for (; sp < splits; ++sp) {
      const float4 v = *(const float4 *)(part + (long)sp * n_w + i);
      sum.x += v.x, sum.y += v.y, sum.z += v.z, sum.w += v.w;
    }
    const int tap = m / cin_g, cl = m - tap * cin_g;
    float *dst = gw32 + row * M + (long)cl * taps + tap;
    dst[0] += sum.x;
    dst[taps] += sum.y;
    dst[2 * taps] += sum.z;
    dst[3 * taps] += sum.w;
  }
}

}  // namespace mdcn
