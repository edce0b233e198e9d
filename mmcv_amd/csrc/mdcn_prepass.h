// Pre-pass kernels of the fused path: input re-layout and weight repack.
#pragma once

#include "mdcn_common.h"

namespace mdcn {

// NCHW input -> zero-bordered slab-major copy xt[N][Cin/KC][H+2][W+2][KC], KC =
// 128 bytes of channels per pixel and slab.  The one-pixel zero border makes
// every bilinear corner of an in-range position a plain load: a corner outside
// the image reads a stored zero, which is exactly the per-corner rule of the
// reference sampler (mmcv/ops/csrc/pytorch/cpu/modulated_deform_conv.cpp:17-27).
// Image rows run on into each other in the flattened plane, so every block but
// the last of a plane is full whatever W is.  The pixel that ends an image row
// also zeroes the two border pixels that follow it in the copy (right border of
// its row, left border of the next); the first block of a plane zeroes the top
// border row and the pixel after it, the last one the bottom row.
// BORDER = false writes the plain pixel-major copy [N][Cin/KC][H*W][KC] instead
// (the backward's pixel-major grad_output).
//
// No LDS: channel rows are read 16 bytes at a time, at
// whatever alignment the plane size and the tensor give them (global memory takes
// unaligned accesses; only the last, partial run of a plane whose size is not a
// multiple of the run is read element by element, so that nothing past the
// tensor is touched).  A thread owns EPV = 16 / sizeof(E) consecutive pixels x EPV
// consecutive channels: EPV loads of 16 bytes (one channel each), a transpose in
// registers (16-bit elements: one v_perm_b32 per output word; fp32: none, the
// words only change names) and EPV stores of 16 bytes (one pixel each).  Eight
// neighbouring lanes hold the eight channel groups of a pixel run, so a load
// instruction reads 128 contiguous bytes per channel and a store instruction
// writes whole 128-byte pixels.  One block = 32 pixel runs x 8 channel groups:
// one slab of 32 * EPV pixels.
// REC = 32 writes the copy in records of 32 bytes instead of 128: [N][Cin/RC][H+2][W+2][RC] with RC = 32 bytes
// of channels, i.e. each 128-byte slab as four planes -- for a reader that takes 32 bytes of a pixel at a
// time and whose neighbouring lanes read neighbouring pixels (the backward's scatter kernel): four pixels
// share a cache line there, where the 128-byte records give every lane a line of its own.
template <typename E, bool BORDER, int REC = 128>
__device__ __forceinline__ void relayout_vec_block(const Geom &g, const E *__restrict__ in, E *__restrict__ xt,
                                                   int n_pchunks, int b) {
  static_assert(REC == 128 || REC == 32, "whole slabs or quarters of them");
  constexpr int EPV = 16 / (int)sizeof(E);
  constexpr int KC = 128 / (int)sizeof(E);
  constexpr int PXB = 32 * EPV;  // pixels per block
  const int pc = b % n_pchunks;
  b /= n_pchunks;
  const int slabs_total = g.Cin / KC;
  const int slab = b % slabs_total;
  const int n = b / slabs_total;
  const int tid = threadIdx.x;
  const int cg = tid & 7, pg = tid >> 3;
  const int plane = g.H * g.W;
  const int p0 = pc * PXB + pg * EPV;
  const long plane_px = BORDER ? (long)g.Hp * g.Wp : (long)plane;   // pixels of a plane of the copy
  unsigned char *dst_slab = (unsigned char *)xt + (((long)n * slabs_total + slab) * plane_px) * 128;
  // where this thread's 16 bytes of pixel 0 go
  unsigned char *dst_cg = REC == 128 ? dst_slab + cg * 16 : dst_slab + (long)(cg >> 1) * plane_px * 32 + (cg & 1) * 16;
  const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
  uint4 o[EPV];    // o[i] = this thread's EPV channels of pixel p0 + i
#pragma unroll
  for (int i = 0; i < EPV; ++i) o[i] = zero;
  const int np = max(0, min(EPV, plane - p0));  // pixels of the run that exist
  if (p0 < plane) {
    const E *src = in + ((long)n * g.Cin + slab * KC + cg * EPV) * plane + p0;
    uint4 r[EPV];
    if (np == EPV) {  // (16 bytes at the alignment of an element: one load instruction all the same)
#pragma unroll
      for (int j = 0; j < EPV; ++j) __builtin_memcpy(&r[j], src + (long)j * plane, 16);
    } else {
#pragma unroll
      for (int j = 0; j < EPV; ++j) {
        E e[EPV];
#pragma unroll
        for (int i = 0; i < EPV; ++i) e[i] = i < np ? src[(long)j * plane + i] : from_f32<E>(0.0f);
        __builtin_memcpy(&r[j], e, 16);
      }
    }
    if constexpr (sizeof(E) == 2) {
      // r[j] = 8 pixels of channel j; o[i] = 8 channels of pixel i
      const uint32_t *rw = (const uint32_t *)r;
      uint32_t *ow = (uint32_t *)o;
#pragma unroll
      for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          const uint32_t lo = rw[(2 * a) * 4 + w], hi = rw[(2 * a + 1) * 4 + w];
          ow[(2 * w) * 4 + a] = __builtin_amdgcn_perm(hi, lo, 0x05040100u);      // low halves: pixel 2w
          ow[(2 * w + 1) * 4 + a] = __builtin_amdgcn_perm(hi, lo, 0x07060302u);  // high halves: pixel 2w + 1
        }
    } else {
      const uint32_t *rw = (const uint32_t *)r;
      uint32_t *ow = (uint32_t *)o;
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) ow[i * 4 + j] = rw[j * 4 + i];
    }
  }
  if constexpr (REC == 128) {
    int y = p0 / g.W;
    int x = p0 - y * g.W;
#pragma unroll
    for (int i = 0; i < EPV; ++i) {
      if (i >= np) break;
      unsigned char *d = dst_cg + (BORDER ? (long)(y + 1) * g.Wp + (x + 1) : (long)(p0 + i)) * REC;
      *(uint4 *)d = o[i];
      if (BORDER && x == g.W - 1) {
        *(uint4 *)(d + REC) = zero;
        *(uint4 *)(d + 2 * REC) = zero;
      }
      if (++x == g.W) {
        x = 0;
        ++y;
      }
    }
  } else {
    // 32-byte records: a store instruction of the wave would write its eight runs' pixel i, 256 bytes apart
    // each.  The runs of four neighbouring lanes groups (lane bits 4 and 5) first trade pixels with each
    // other (register bits 0 and 1 against those lane bits), after which register i holds, across these
    // lanes, four consecutive pixels: 128 contiguous bytes per plane and instruction.
#pragma unroll
    for (int i = 0; i < EPV; ++i) {
      if ((i & 2) == 0) {
        uint32_t *lo = (uint32_t *)&o[i], *hi = (uint32_t *)&o[i | 2];
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          const auto sw = __builtin_amdgcn_permlane32_swap(lo[w], hi[w], false, false);
          lo[w] = sw[0];
          hi[w] = sw[1];
        }
      }
    }
#pragma unroll
    for (int i = 0; i < EPV; ++i) {
      if ((i & 1) == 0) {
        uint32_t *lo = (uint32_t *)&o[i], *hi = (uint32_t *)&o[i | 1];
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          const auto sw = __builtin_amdgcn_permlane16_swap(lo[w], hi[w], false, false);
          lo[w] = sw[0];
          hi[w] = sw[1];
        }
      }
    }
    // register i now holds pixel src_i of the run of lane group src_pg
    const int b5 = (pg >> 2) & 1, b4 = (pg >> 1) & 1;
#pragma unroll
    for (int i = 0; i < EPV; ++i) {
      const int src_pg = (pg & ~6) | (((i >> 1) & 1) << 2) | ((i & 1) << 1);
      const int src_i = (i & ~3) | (b5 << 1) | b4;
      const int q = pc * PXB + src_pg * EPV + src_i;
      if (q < plane) {
        const int y = q / g.W, x = q - y * g.W;
        unsigned char *d = dst_cg + (BORDER ? (long)(y + 1) * g.Wp + (x + 1) : (long)q) * REC;
        *(uint4 *)d = o[i];
        if (BORDER && x == g.W - 1) {
          *(uint4 *)(d + REC) = zero;
          *(uint4 *)(d + 2 * REC) = zero;
        }
      }
    }
  }
  if (!BORDER) return;
  constexpr int NPL = 128 / REC;       // planes of the copy per slab
  constexpr int QPP = REC / 16;        // 16-byte pieces per pixel of a plane
  if (pc == 0) {  // top border row and the left border pixel of the first image row
    const int per = (g.Wp + 1) * QPP;
    for (int i = tid; i < per * NPL; i += 256)
      *(uint4 *)(dst_slab + (long)(i / per) * plane_px * REC + (long)(i % per) * 16) = zero;
  }
  if (pc == n_pchunks - 1) {  // bottom border row
    const int per = g.Wp * QPP;
    for (int i = tid; i < per * NPL; i += 256)
      *(uint4 *)(dst_slab + (long)(i / per) * plane_px * REC + ((long)(g.Hp - 1) * g.Wp) * REC + (long)(i % per) * 16) = zero;
  }
}

template <typename E, bool BORDER = true, int REC = 128>
__global__ __launch_bounds__(256) void relayout_vec_kernel(Geom g, const E *__restrict__ in, E *__restrict__ xt,
                                                           int n_pchunks) {
  relayout_vec_block<E, BORDER, REC>(g, in, xt, n_pchunks, (int)blockIdx.x);
}

// weight[Cout][Cin/G][kh][kw] -> wp[G][n_ctiles][nk][CT][KC]: for every
// group, Cout tile and K step (channel slab outer, tap inner) one dense
// CT x KC tile, K contiguous, zero rows past Cout/G.  The main kernel copies
// such a tile to LDS with straight 16-byte loads.  Element idx, idx + stride, ...
// Also clears the `zero_n` words at `zero_ptr` (the main kernel's cut-tile counters).
template <typename E>
__device__ __forceinline__ void pack_weight_elems(const Geom &g, const E *__restrict__ w, E *__restrict__ wp, int CT,
                                                  int KC, int n_ctiles, int slabs, long total, long first,
                                                  long stride, uint32_t *__restrict__ zero_ptr, int zero_n) {
  for (long i = first; i < zero_n; i += stride) zero_ptr[i] = 0u;
  // one 16-byte run of a row (EPV consecutive input channels of one output channel and tap) per step: the
  // index arithmetic is paid once per run and the store is whole
  constexpr int EPV = 16 / (int)sizeof(E);
  const int nk = slabs * g.taps;
  const int runs = KC / EPV;
  for (long idx = first; idx < total / EPV; idx += stride) {
    long r = idx;
    const int kc = (int)(r % runs) * EPV;
    r /= runs;
    const int row = (int)(r % CT);
    r /= CT;
    const int ks = (int)(r % nk);
    r /= nk;
    const int ctile = (int)(r % n_ctiles);
    const int grp = (int)(r / n_ctiles);
    const int slab = ks / g.taps, tap = ks % g.taps;
    const int col = ctile * CT + row;  // output channel within the group
    E v[EPV];
    if (col < g.cout_g) {
      const int co = grp * g.cout_g + col;
      const E *src = w + ((long)co * g.cin_g + slab * KC + kc) * g.taps + tap;
#pragma unroll
      for (int i = 0; i < EPV; ++i) v[i] = src[(long)i * g.taps];
    } else {
#pragma unroll
      for (int i = 0; i < EPV; ++i) v[i] = from_f32<E>(0.0f);
    }
    uint4 o;
    __builtin_memcpy(&o, v, 16);
    *(uint4 *)(wp + idx * EPV) = o;
  }
}

template <typename E>
__global__ __launch_bounds__(256) void pack_weight_kernel(
    Geom g, const E *__restrict__ w, E *__restrict__ wp, int CT, int KC,
    int n_ctiles, int slabs, long total, uint32_t *__restrict__ zero_ptr, int zero_n) {
  pack_weight_elems<E>(g, w, wp, CT, KC, n_ctiles, slabs, total, (long)blockIdx.x * blockDim.x + threadIdx.x,
                       (long)gridDim.x * blockDim.x, zero_ptr, zero_n);
}

// Both pre-passes of a forward call in one launch: the first `pack_blocks`
// workgroups repack the weights (geometry gw: that of the whole call), the others
// re-lay the input of one batch chunk (geometry g) as relayout_vec_kernel does.
// The two are independent, and the small weight repack hides under the copy.
template <typename E>
__global__ __launch_bounds__(256) void prepass_kernel(Geom g, const E *__restrict__ in, E *__restrict__ xt,
                                                      int n_pchunks, Geom gw, const E *__restrict__ w,
                                                      E *__restrict__ wp, int CT, int KC, int n_ctiles, int slabs,
                                                      long wtotal, int pack_blocks,
                                                      uint32_t *__restrict__ zero_ptr, int zero_n) {
  if ((int)blockIdx.x < pack_blocks) {
    pack_weight_elems<E>(gw, w, wp, CT, KC, n_ctiles, slabs, wtotal, (long)blockIdx.x * 256 + threadIdx.x,
                         (long)pack_blocks * 256, zero_ptr, zero_n);
    return;
  }
  relayout_vec_block<E, true>(g, in, xt, n_pchunks, (int)blockIdx.x - pack_blocks);
}

}  // namespace mdcn
