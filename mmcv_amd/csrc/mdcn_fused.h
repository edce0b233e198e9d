// Fused DCNv2 forward for gfx950: implicit GEMM  out[pixel, cout] = S[pixel, k] * W[k, cout]
// where S (the "columns" of the reference's two-pass design,
// mmcv/ops/csrc/pytorch/modulated_deform_conv.cpp:101-124) is produced on the
// fly -- offset/mask-modulated bilinear samples computed by wavefronts and
// written straight into LDS tiles that feed MFMA -- and never exists in HBM.
//
// Work split.  A persistent workgroup of 8 wavefronts owns, one after another,
// tiles of PT = 128 consecutive output pixels (flattened n*Ho*Wo + ho*Wo + wo)
// x CT output channels of one group.  K runs over (slab of KC channels) x
// (tap), slab outer, tap inner.  A slab is 128 bytes of channels (64 bf16/fp16,
// 32 fp32), and the input copy is stored slab-major
// ([N][Cin/KC][H+2][W+2][KC]): one bilinear corner of one slab is exactly one
// aligned 128-byte cache line, so every byte a gather pulls from L2 is used.
//
// The wavefronts are specialised:
//   waves 4..7  PRODUCERS.  Once per tile (and deformable group) they fill a
//     table in LDS with, for every (pixel, tap), the index of the top-left
//     bilinear corner in the zero-bordered input copy and the four mask-scaled
//     bilinear weights (positions and weights in fp32).  Per K step, each lane
//     gathers for two pixels 2 x 16 bytes of channels at each of the four corners
//     (16 x global_load_dwordx4, issued kGatherAhead steps ahead, held in
//     registers), blends them (16-bit types: horizontal corners paired with
//     v_perm_b32, one v_dot2 per two products; fp32: FMA) and writes 4 x 16
//     bytes of the sample tile.
//   waves 0..3  CONSUMERS.  2 x 2 over the tile (64 pixels x CT/2 channels
//     each): read sample and weight fragments from LDS, run MFMA
//     (32x32x16 bf16/f16, 32x32x2 fp32) into fp32 accumulators; at the end of
//     the tile add the bias, round once, transpose through LDS and store
//     16 bytes per lane along W of the NCHW output.  They also issue the
//     direct-to-LDS copy of the weight tile kWeightAhead steps ahead.
// One workgroup barrier per K step keeps the two roles in step; the sample
// tile is double buffered, the weight tiles sit in a ring of kWeightSlots.
// Where the epilogue's staging fits one ring slot (16-bit types, CT = 256) the
// producers start the next tile (table, gathers, first sample tile) while the
// consumers store the current one.
//
// LDS tiles have 128-byte rows (one pixel resp. one output channel, KC elements
// of K); the 16-byte chunks of a row are permuted (swz) so that both the
// 16-byte fragment reads (32 consecutive rows, one chunk) and the writes
// (4 lanes per row) spread over all banks.
#pragma once

#include "mdcn_common.h"

namespace mdcn {

constexpr int kPT = 128;           // pixels per tile
constexpr int kRowB = 128;         // bytes of K per tile row and K step
constexpr int kRowChunks = kRowB / 16;
constexpr int kGatherAhead = 2;    // K steps a gather is in flight
constexpr int kWeightAhead = 1;    // K steps a weight-tile copy is in flight
constexpr int kWeightSlots = kWeightAhead + 2;
constexpr int kProducerWaves = 4;                        // waves 4 .. 4 + kProducerWaves - 1
constexpr int kThreads = 256 + 64 * kProducerWaves;
constexpr int kPxPerLane = 8 / kProducerWaves;           // pixels of the tile a producer lane serves
constexpr int kTapGroups = kProducerWaves / 2;           // producer lanes per pixel in the table build
constexpr int kCutMax = 4;         // parts a tile of the schedule's last round is cut into at most

struct FusedArgs {
  Geom g;
  const void *xt;      // zero-bordered slab-major input copy, or the caller's channels-last input itself
  const void *wp;      // packed weights
  OffMaskView om;      // offsets and mask of the images of this launch
  const void *bias;    // may be null
  void *out;
  long total_px;       // N * Ho * Wo
  int n_ptiles, n_ctiles, slabs;   // slabs = (Cin/G) / KC
  int slabs_total;     // Cin / KC
  int plane_px;        // Hp * Wp
  int out_vec_ok;      // (Ho*Wo) % (16/sizeof(E)) == 0 and the output pointer is 16-byte aligned
  uint32_t row_bytes;  // bytes between vertically adjacent pixels: Wp * kRowB (copy) or W * Cin * sizeof(E)
  uint32_t px_bytes;   // bytes between horizontally adjacent pixels: kRowB (copy) or Cin * sizeof(E)
  uint32_t slab_bytes; // bytes between channel slabs of one pixel: plane_px * kRowB (copy) or kRowB
  uint32_t img_bytes;  // bytes between images
  // fused2_kernel only: tiles of the last, partial round of the schedule are cut along K into up to
  // cut_max parts (0 or 1: never) that meet in cut_part, gridDim.x buffers of kPT x 256 floats,
  // counted in cut_cnt, gridDim.x words that are zero when the kernel starts
  int cut_max;
  void *cut_part;
  void *cut_cnt;
  // fused2_kernel only: first pixel of its tiles (a multiple of 256; the pixels in front of it belong to
  // fused3_kernel, which is launched beside it); n_ptiles counts the tiles from there on
  int px0;
};

typedef __attribute__((address_space(3))) void *lptr_t;

// Byte offset, inside one image of the input copy, of the upper left corner of
// a sample's 2 x 2 block (slab 0).
// Zero-bordered copy: +1 in both coordinates (y0, x0 >= -1 when the position is
// inside).  A position outside (-1,H) x (-1,W) adds nothing in the reference
// (mmcv/ops/csrc/pytorch/cpu/modulated_deform_conv.cpp:160-164): its block is
// put on padded pixels (0, Wp-1), (1, 0), (1, Wp-1), (2, 0) -- four border
// pixels that follow one another in memory the way a block's corners do -- so
// that the four loads return stored zeros whatever the image holds.
// Channels-last input read in place: the block is moved into the image and the
// weights of the corners that were outside become zero (clamp_to_image; call
// before the weights are taken from `s`).
template <bool UNBORDERED>
__device__ __forceinline__ uint32_t corner_offset(TapSample &s, const Geom &g, const FusedArgs &a) {
  if (UNBORDERED) {
    clamp_to_image(s, g.H, g.W);
    return (uint32_t)s.y0 * a.row_bytes + (uint32_t)s.x0 * a.px_bytes;
  }
  return s.inside ? (uint32_t)(s.y0 + 1) * a.row_bytes + (uint32_t)(s.x0 + 1) * (uint32_t)kRowB
                  : (uint32_t)(g.Wp - 1) * (uint32_t)kRowB;
}

template <typename E>
struct ElemTraits;

// ---- 16-bit element types ---------------------------------------------------
// A 32-bit word of gathered data holds two channels.  The two horizontal
// neighbours of a row are paired channel by channel with v_perm_b32 and one
// v_dot2 applies both of their weights: (v(x0), v(x0+1)) . (w_left, w_right).
// The perms run on the integer pipe, which keeps working while the other wave
// of the SIMD streams MFMAs; floating-point VALU work does not (measured: it is
// starved completely), so halving the number of dot instructions matters more
// than the instruction count says.  The table keeps the weight pairs
// (w00, w01) and (w10, w11), rounded to the element type.
template <typename E>
struct Half16Traits {
  static constexpr int KC = 64;  // channels per K step (128 bytes)

  static __device__ __forceinline__ void table_weights(const TapSample &s, uint32_t (&tw)[4]) {
    tw[0] = ElemTraits<E>::pack2(s.w00, s.w01);
    tw[1] = ElemTraits<E>::pack2(s.w10, s.w11);
    tw[2] = 0u;
    tw[3] = 0u;
  }

  // four consecutive pixels of one output channel, rounded, to the staging row
  static __device__ __forceinline__ void store4(unsigned char *dst, float a, float b, float c,
                                                float d) {
    *(uint2 *)dst = make_uint2(ElemTraits<E>::pack2(a, b), ElemTraits<E>::pack2(c, d));
  }

  // 16 bytes (8 channels) of one pixel from the same 16 bytes at its 4 corners
  // (v0, v1: upper row left/right; v2, v3: lower row)
  static __device__ __forceinline__ uint4 blend(const uint4 &v0, const uint4 &v1, const uint4 &v2,
                                                const uint4 &v3, const uint4 &w) {
    const uint32_t t0[4] = {v0.x, v0.y, v0.z, v0.w}, t1[4] = {v1.x, v1.y, v1.z, v1.w};
    const uint32_t b0[4] = {v2.x, v2.y, v2.z, v2.w}, b1[4] = {v3.x, v3.y, v3.z, v3.w};
    uint32_t o[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      // low channel of word j: bytes 0,1 of both neighbours; high channel: bytes 2,3
      const uint32_t top_lo = __builtin_amdgcn_perm(t1[j], t0[j], 0x05040100u);
      const uint32_t top_hi = __builtin_amdgcn_perm(t1[j], t0[j], 0x07060302u);
      const uint32_t bot_lo = __builtin_amdgcn_perm(b1[j], b0[j], 0x05040100u);
      const uint32_t bot_hi = __builtin_amdgcn_perm(b1[j], b0[j], 0x07060302u);
      const float lo = ElemTraits<E>::dot2(bot_lo, w.y, ElemTraits<E>::dot2(top_lo, w.x, 0.0f));
      const float hi = ElemTraits<E>::dot2(bot_hi, w.y, ElemTraits<E>::dot2(top_hi, w.x, 0.0f));
      o[j] = ElemTraits<E>::pack2(lo, hi);
    }
    return make_uint4(o[0], o[1], o[2], o[3]);
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
  // the two channels of a 32-bit word as floats
  static __device__ __forceinline__ void unpack2(uint32_t w, float &lo, float &hi) {
    lo = __uint_as_float(w << 16);
    hi = __uint_as_float(w & 0xffff0000u);
  }
  // (the builtin, not inline assembly: the compiler must see the DOT instruction
  // to insert the wait states its result needs before another VALU reads it)
  static __device__ __forceinline__ float dot2(uint32_t d, uint32_t w, float c) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, d),
                                           __builtin_bit_cast(bf16x2, w), c, false);
  }
  // 16 bytes = 8 consecutive K elements of one row per lane.
  static __device__ __forceinline__ void mma(f32x16 &c, const uint4 &a, const uint4 &b) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
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
  static __device__ __forceinline__ void unpack2(uint32_t w, float &lo, float &hi) {
    const f16x2 p = __builtin_bit_cast(f16x2, w);
    lo = (float)p.x;
    hi = (float)p.y;
  }
  static __device__ __forceinline__ float dot2(uint32_t d, uint32_t w, float c) {
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, d), __builtin_bit_cast(f16x2, w), c, false);
  }
  static __device__ __forceinline__ void mma(f32x16 &c, const uint4 &a, const uint4 &b) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                               __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  // fp16 has packed arithmetic (bf16 on this chip has not): the table keeps every
  // corner weight twice in one word, and a word of two channels takes one
  // v_pk_mul_f16 and three v_pk_fma_f16 -- four instructions where the dot-product
  // form needs nine.  The blend then rounds to fp16 after every corner instead of
  // once (three more roundings of 2^-11 relative, far inside the fp16 bar).
  static __device__ __forceinline__ void table_weights(const TapSample &s, uint32_t (&tw)[4]) {
    tw[0] = pack2(s.w00, s.w00);
    tw[1] = pack2(s.w01, s.w01);
    tw[2] = pack2(s.w10, s.w10);
    tw[3] = pack2(s.w11, s.w11);
  }
  static __device__ __forceinline__ uint4 blend(const uint4 &v0, const uint4 &v1, const uint4 &v2,
                                                const uint4 &v3, const uint4 &w) {
    const uint32_t c0[4] = {v0.x, v0.y, v0.z, v0.w}, c1[4] = {v1.x, v1.y, v1.z, v1.w};
    const uint32_t c2[4] = {v2.x, v2.y, v2.z, v2.w}, c3[4] = {v3.x, v3.y, v3.z, v3.w};
    const f16x2 w0 = __builtin_bit_cast(f16x2, w.x), w1 = __builtin_bit_cast(f16x2, w.y);
    const f16x2 w2 = __builtin_bit_cast(f16x2, w.z), w3 = __builtin_bit_cast(f16x2, w.w);
    uint32_t o[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      f16x2 acc = __builtin_bit_cast(f16x2, c0[j]) * w0;
      acc = __builtin_elementwise_fma(__builtin_bit_cast(f16x2, c1[j]), w1, acc);
      acc = __builtin_elementwise_fma(__builtin_bit_cast(f16x2, c2[j]), w2, acc);
      acc = __builtin_elementwise_fma(__builtin_bit_cast(f16x2, c3[j]), w3, acc);
      o[j] = __builtin_bit_cast(uint32_t, acc);
    }
    return make_uint4(o[0], o[1], o[2], o[3]);
  }
};

// ---- fp32 --------------------------------------------------------------------
template <>
struct ElemTraits<float> {
  static constexpr int KC = 32;

  static __device__ __forceinline__ void table_weights(const TapSample &s, uint32_t (&tw)[4]) {
    tw[0] = __float_as_uint(s.w00);
    tw[1] = __float_as_uint(s.w01);
    tw[2] = __float_as_uint(s.w10);
    tw[3] = __float_as_uint(s.w11);
  }

  static __device__ __forceinline__ void store4(unsigned char *dst, float a, float b, float c,
                                                float d) {
    *(uint4 *)dst = make_uint4(__float_as_uint(a), __float_as_uint(b), __float_as_uint(c),
                               __float_as_uint(d));
  }

  static __device__ __forceinline__ uint4 blend(const uint4 &v0, const uint4 &v1, const uint4 &v2,
                                                const uint4 &v3, const uint4 &w) {
    const float ww[4] = {__uint_as_float(w.x), __uint_as_float(w.y), __uint_as_float(w.z),
                         __uint_as_float(w.w)};
    const uint4 v[4] = {v0, v1, v2, v3};
    float acc[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const float d[4] = {__uint_as_float(v[q].x), __uint_as_float(v[q].y),
                          __uint_as_float(v[q].z), __uint_as_float(v[q].w)};
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[j] = (q == 0) ? ww[q] * d[j] : acc[j] + ww[q] * d[j];
    }
    return make_uint4(__float_as_uint(acc[0]), __float_as_uint(acc[1]), __float_as_uint(acc[2]),
                      __float_as_uint(acc[3]));
  }

  // 16 bytes = 4 consecutive K elements of one row per lane; element j of both
  // operands goes to the j-th 32x32x2 MFMA.
  static __device__ __forceinline__ void mma(f32x16 &c, const uint4 &a, const uint4 &b) {
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.x), __uint_as_float(b.x), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.y), __uint_as_float(b.y), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.z), __uint_as_float(b.z), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.w), __uint_as_float(b.w), c, 0, 0, 0);
  }
};

// Bytes per row of the epilogue staging area: 64 pixels + 16 bytes of padding.
// Each consumer wave stages 32 such rows; waves 0,1 use the sample tiles,
// waves 2,3 the weight ring (both are idle once the K loop has ended).
template <typename E>
constexpr int stage_row_bytes() {
  return 64 * (int)sizeof(E) + 16;
}
static_assert(2 * 32 * (64 * 4 + 16) <= 2 * kPT * kRowB, "two staging areas fit the sample tiles");
static_assert(2 * 32 * (64 * 4 + 16) <= kWeightSlots * 64 * kRowB,
              "two staging areas fit the smallest weight ring");

// LDS of one workgroup: two sample tiles, the ring of weight tiles, the
// (pixel, tap) table (corner index + four weights per entry).
constexpr size_t fused_lds_bytes(int CT, int tmax) {
  return (size_t)2 * kPT * kRowB + (size_t)kWeightSlots * CT * kRowB + (size_t)kPT * tmax * 20 + 16;
}

// Table capacities the kernel is instantiated for (taps = kh * kw).
constexpr int kTapsSmall = 9;
constexpr int kTapsLarge = 25;

// Workgroup barrier without the memory-model fence of __syncthreads(): that
// fence would also wait for every outstanding vector-memory operation, i.e.
// drain the prefetch at every K step.  Waits for this wave's own LDS operations
// and for all but `VM` of its vector-memory operations.
#define MDCN_BARRIER(VM) \
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(VM) : "memory")
#define MDCN_BARRIER_LDS() asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory")

// 16 bytes per lane from global memory straight into LDS: lane i's data lands at
// lds_base + 16*i (lds_base, in M0, is the same for the whole wave).  Written as
// inline assembly on purpose: the compiler treats the builtin as a flat access
// that may touch both memories and then answers every later register or LDS
// dependency with vmcnt(0)/lgkmcnt(0), which would drain the gather prefetch at
// every K step.  Unseen by the compiler, the copies only make its own vmcnt
// waits stricter than necessary (they count as extra younger operations); their
// completion is waited for explicitly (MDCN_BARRIER).
__device__ __forceinline__ void copy16_global_to_lds(const void *src, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
               :
               : "s"(lds_base), "v"(src)
               : "memory");
}

// A pointer every lane of the wave holds the same value of, moved to scalar
// registers (for an "s" operand of an asm statement: the compiler does not always
// see that a value is uniform, and then hands such an operand vector registers).
__device__ __forceinline__ const unsigned char *uniform_ptr(const unsigned char *p) {
  const uint64_t v = (uint64_t)(uintptr_t)p;
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));
  return (const unsigned char *)(uintptr_t)(((uint64_t)hi << 32) | lo);
}

// Work of one workgroup under the XCD-aware persistent schedule: XCD x owns a
// contiguous run of tiles and hands them out round robin to its `stride`
// workgroups.  The run rarely is a multiple of `stride`: its last round has
// rest < stride tiles, and without further ado `rest` workgroups would compute a
// whole tile while the others wait.  Instead each of those tiles is cut along K
// into parts = stride / rest ranges (whole multiples of `round` steps, at most
// cut_max of them, each at least `min_rounds` rounds long), one per workgroup:
// a "unit" is a tile together with a range of K steps; a workgroup walks whole
// tiles first (units 0 .. T_full - 1) and at most one part last.  The parts of
// a tile meet in memory.
struct UnitSchedule {
  int xcd, wg, stride, chunk;
  int T_full, T;
  bool has_part;
  int parts, part_tile, part_idx, part_kb, part_pad;

  __device__ __forceinline__ void init(int total_tiles, int nk_pad, int round, int min_rounds, int cut_max) {
    xcd = (int)(blockIdx.x & 7);
    wg = (int)(blockIdx.x >> 3);
    stride = (int)(gridDim.x >> 3);
    chunk = (total_tiles + 7) >> 3;
    const int tile_end = min((xcd + 1) * chunk, total_tiles);
    const int chunk_x = max(tile_end - xcd * chunk, 0);
    const int full_rounds = chunk_x / stride;
    const int rest = chunk_x - full_rounds * stride;
    const int rounds = nk_pad / round;
    parts = 1;
    if (cut_max > 1 && rest > 0) parts = max(1, min(min(stride / rest, cut_max), rounds / min_rounds));
    const bool cut = parts > 1;
    T_full = full_rounds + ((!cut && wg < rest) ? 1 : 0);
    has_part = cut && wg < rest * parts;
    T = T_full + (has_part ? 1 : 0);
    part_tile = xcd * chunk + full_rounds * stride + wg / parts;
    part_idx = wg - (wg / parts) * parts;
    part_kb = (part_idx * rounds / parts) * round;
    part_pad = ((part_idx + 1) * rounds / parts) * round - part_kb;
  }
  __device__ __forceinline__ bool is_part(int u) const { return has_part && u == T_full; }
  __device__ __forceinline__ int tile_of(int u) const { return is_part(u) ? part_tile : xcd * chunk + wg + u * stride; }
  // the counter of this workgroup's cut tile and the first of the tile's buffers (one per workgroup of the grid)
  __device__ __forceinline__ int counter_slot() const { return xcd * stride + wg / parts; }
  __device__ __forceinline__ int buffer_slot0() const { return xcd * stride + (wg / parts) * parts; }
};

// Walks the K steps of a tile in issue order (channel slab outer, tap inner) and
// reports when a step starts a new deformable group.  Producers and consumers
// run identical cursors, so both know when the table is rebuilt.
struct StepCursor {
  int step, slab, tap, dgrem;
  bool new_dg;
  // `step` counts from the unit's first step kb (0 for a whole tile)
  __device__ __forceinline__ void init(int slab0, int spd, int kb, int taps) {
    step = 0;
    slab = kb / taps;
    tap = kb - slab * taps;
    dgrem = (slab0 + slab) % spd;
    new_dg = false;
  }
  // Move to the next step; past the last step the cursor stays on it.
  __device__ __forceinline__ void advance(int nk, int taps, int spd) {
    if (step >= nk - 1) return;
    ++step;
    if (++tap == taps) {
      tap = 0;
      ++slab;
      if (++dgrem == spd) {
        dgrem = 0;
        new_dg = true;
      }
    }
  }
};

// Position of 16-byte chunk c of row r inside a tile: chunk c sits at c ^ swz(r).
// swz runs through all 8 values over 16 consecutive rows (two rows share one and
// sit in opposite halves of the 256-byte bank period), so the fragment reads
// (16 consecutive rows, one chunk) are conflict free; rows 2 apart differ in
// bit 2, so the writes (4 consecutive rows x chunks 0..3 or 4..7) are too.
__device__ __forceinline__ int swz(int r) { return (((r >> 1) & 1) << 2) | ((r >> 2) & 3); }
__device__ __forceinline__ int tile_chunk(int r, int c) { return r * kRowChunks + (c ^ swz(r)); }

// MULTI_DG: more than one deformable group, i.e. the table is rebuilt inside the
// K loop.  Kept out of the single-group instantiation because a conditional
// block with loads inside the step loop makes the compiler drain the gather
// prefetch (vmcnt(0)) at every step.
// UNBORDERED: a.xt is the caller's dense channels-last (N, H, W, Cin) input, read
// in place: no copy, no zero border.  The table then clamps each 2x2 corner block
// into the image and moves the weights of the corners that fell outside to zero
// (clamp_to_image), which keeps the reference's per-corner rule.
template <typename E, int CT, int TMAX, bool MULTI_DG, bool UNBORDERED>
__global__ __launch_bounds__(kThreads, 2) void fused_kernel(FusedArgs a) {
  using TR = ElemTraits<E>;
  constexpr int PT = kPT;
  constexpr int KC = TR::KC;
  constexpr int ES = (int)sizeof(E);
  constexpr int MB = CT / 64;        // 32-channel accumulator blocks per consumer wave
  constexpr int NB = 2;              // 32-pixel blocks per consumer wave
  constexpr int WDMA = CT / 32;      // 1 KiB direct-to-LDS copies per consumer wave and K step
  constexpr int TPT = (TMAX + kTapGroups - 1) / kTapGroups;  // table entries per producer lane
  static_assert(kWeightAhead * WDMA < 64, "vmcnt holds 6 bits");
  // Epilogue overlap: when the consumers' four staging areas fit the ring slot
  // that no copy targets before the first K step of a tile, the epilogue leaves
  // the sample tiles alone, and the producers build the next tile's table and
  // first samples while the consumers store the current one.
  constexpr bool OVL = 4 * 32 * stage_row_bytes<E>() <= CT * kRowB && kWeightAhead + 1 < kWeightSlots;

  __shared__ uint4 Xs[2][PT * kRowChunks];                // sample tiles
  __shared__ uint4 Ws[kWeightSlots][CT * kRowChunks];     // weight tiles
  __shared__ uint32_t tpix[PT * TMAX];                    // (pixel, tap) table, [tap][PT]: corner byte offset
  __shared__ uint4 tws[PT * TMAX];                        // ... and the four weights
  __shared__ uint32_t part_arrived;                       // parts of a cut tile that were there before this one

  const Geom &g = a.g;
  const int taps = g.taps;
  const int nk_tile = a.slabs * taps;
  const int nk_tile_pad = (nk_tile + kGatherAhead - 1) / kGatherAhead * kGatherAhead;
  const int plane_out = g.Ho * g.Wo;
  const int total_px = (int)a.total_px;
  const int spd = g.ch_per_dg / KC;  // slabs per deformable group

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const bool producer = wave >= 4;

  // XCD-aware persistent schedule: consecutive workgroup ids sit on different
  // XCDs; each XCD walks one contiguous run of tiles so that the halo rows
  // neighbouring tiles share stay in its L2.  Tiles of the run's last round are
  // cut along K (UnitSchedule): parts of at least 8 steps.
  UnitSchedule us;
  us.init(a.n_ptiles * a.n_ctiles * g.G, nk_tile_pad, kGatherAhead, 8 / kGatherAhead, a.cut_max);
  bool first_tile = true;

  for (int u = 0; u < us.T; ++u, first_tile = false) {
    const bool is_part = us.is_part(u);
    // K range of the unit: steps kb .. kb + nk - 1 of the tile, padded to nk_pad
    const int kb = is_part ? us.part_kb : 0;
    const int nk_pad = is_part ? us.part_pad : nk_tile_pad;
    const int nk = min(nk_tile - kb, nk_pad);
    const bool more_units = u + 1 < us.T;
    int L = us.tile_of(u);
    const int ctile = L % a.n_ctiles;
    L /= a.n_ctiles;
    const int grp = L % g.G;
    const int ptile = L / g.G;
    const int p0 = ptile * PT;
    const int ch0 = grp * g.cin_g;  // first input channel of the group
    const int slab0 = ch0 / KC;

    StepCursor cur;  // the next step whose gather is issued
    cur.init(slab0, spd, kb, taps);

    if (producer) {
      // =================== PRODUCER ===================
      // fp32 tiles of <= 128 channels: the consumers' MFMAs are short of work there and the step
      // waits for the producers, so the arbiter is told to prefer them (cfg 3: 0.527 -> 0.486 ms).
      // With 256-channel fp32 tiles the same setting costs 1-3 %, with 16-bit tensors it is a wash.
      if constexpr (sizeof(E) == 4 && CT <= 128) __builtin_amdgcn_s_setprio(2);
      const int ptid = tid - 256;
      const int q = ptid & 3;          // this lane handles 16-byte chunks q and q + 4 of a row
      const int pxl = ptid >> 2;       // ... of pixels pxl and pxl + 64 of the tile
      const unsigned char *xt = (const unsigned char *)a.xt;
      // horizontal neighbour: an instruction offset for the copy, a register otherwise
      const uint32_t pxb = UNBORDERED ? a.px_bytes : (uint32_t)kRowB;

      // -- (pixel, tap) table of one deformable group; lane serves pixel ptid%128
      const int tb_pl = ptid & (PT - 1);
      const int tb_p = p0 + tb_pl;
      const bool tb_valid = tb_p < total_px;
      int tb_n = 0, tb_ho = 0, tb_wo = 0, tb_rem = 0;
      if (tb_valid) {
        tb_n = tb_p / plane_out;
        tb_rem = tb_p - tb_n * plane_out;
        tb_ho = tb_rem / g.Wo;
        tb_wo = tb_rem - tb_ho * g.Wo;
      }
      auto build_table = [&](int dgi) {
        // (an invalid pixel reads the entries of pixel 0 of image 0 and stores zeros)
        const E *off = (const E *)a.om.off + (long)tb_n * a.om.off_n + (long)tb_rem * a.om.off_px +
                       (long)(dgi * 2 * taps) * a.om.off_ch;
        const E *msk = (const E *)a.om.msk + (long)tb_n * a.om.msk_n + (long)tb_rem * a.om.msk_px +
                       (long)(dgi * taps) * a.om.msk_ch;
        // all loads first (unconditional, clamped), then the arithmetic
        E rdy[TPT], rdx[TPT], rm[TPT];
#pragma unroll
        for (int i = 0; i < TPT; ++i) {
          const int tap = min((ptid >> 7) + kTapGroups * i, taps - 1);
          rdy[i] = off[(long)(2 * tap) * a.om.off_ch];
          rdx[i] = off[(long)(2 * tap + 1) * a.om.off_ch];
          rm[i] = msk[(long)tap * a.om.msk_ch];
        }
#pragma unroll
        for (int i = 0; i < TPT; ++i) {
          const int tap = (ptid >> 7) + kTapGroups * i;
          if (tap < taps) {
            const int ti = tap / g.kw, tj = tap - ti * g.kw;
            TapSample sm =
                make_tap_sample(tb_ho * g.sh - g.ph + ti * g.dh, tb_wo * g.sw - g.pw + tj * g.dw,
                                to_f32(rdy[i]), to_f32(rdx[i]), mask_value<E>(rm[i], a.om.logit), g.H, g.W);
            // byte offset of the upper left corner, slab 0 of image tb_n
            uint32_t pix = (uint32_t)tb_n * a.img_bytes + corner_offset<UNBORDERED>(sm, g, a);
            uint32_t tw[4];
            TR::table_weights(sm, tw);
            if (!tb_valid) {
              pix = 0;
              tw[0] = tw[1] = tw[2] = tw[3] = 0u;
            }
            tpix[tap * PT + tb_pl] = pix;
            tws[tap * PT + tb_pl] = make_uint4(tw[0], tw[1], tw[2], tw[3]);
          }
        }
      };

      // -- gather state: kGatherAhead register sets, set m % kGatherAhead holds step m;
      //    [pixel][corner][half of the lane's 32 bytes]
      uint4 gv[kGatherAhead][kPxPerLane][4][2];
      uint4 gw[kGatherAhead][kPxPerLane];

      // Gather of the cursor's step (rebuilding the table first when the step
      // opens a new deformable group), then move the cursor on.
      auto issue_gather = [&](uint4 (&v)[kPxPerLane][4][2], uint4 (&w)[kPxPerLane]) {
        if (MULTI_DG && cur.new_dg) {
          // Every producer issued the previous group's last step before the
          // barrier that ended the previous K step, with its weights in registers.
          cur.new_dg = false;
          build_table((ch0 + cur.slab * KC) / g.ch_per_dg);
          MDCN_BARRIER_LDS();  // R: new table visible (the consumers join)
        }
        const uint32_t sbase = (uint32_t)(slab0 + cur.slab) * a.slab_bytes + (uint32_t)q * 16u;
#pragma unroll
        for (int h = 0; h < kPxPerLane; ++h) {
          const int e = cur.tap * PT + pxl + (PT / kPxPerLane) * h;
          const uint32_t o = tpix[e] + sbase;
          w[h] = tws[e];
          const unsigned char *top = xt + o;
          const unsigned char *bot = top + a.row_bytes;
          v[h][0][0] = *(const uint4 *)(top);
          v[h][0][1] = *(const uint4 *)(top + 64);
          v[h][1][0] = *(const uint4 *)(top + pxb);
          v[h][1][1] = *(const uint4 *)(top + pxb + 64);
          v[h][2][0] = *(const uint4 *)(bot);
          v[h][2][1] = *(const uint4 *)(bot + 64);
          v[h][3][0] = *(const uint4 *)(bot + pxb);
          v[h][3][1] = *(const uint4 *)(bot + pxb + 64);
        }
        cur.advance(nk, taps, spd);
      };

      // Blend the set (step s) into sample tile `buf` and refill it with the
      // gather of the cursor's step, 16 bytes x 4 corners at a time: the loads go
      // out between the blends, so the memory pipeline works while the VALU does.
      auto commit_and_refill = [&](int buf, uint4 (&v)[kPxPerLane][4][2], uint4 (&w)[kPxPerLane]) {
        if (MULTI_DG && cur.new_dg) {
          cur.new_dg = false;
          build_table((ch0 + cur.slab * KC) / g.ch_per_dg);
          MDCN_BARRIER_LDS();  // R
        }
        const uint32_t sbase = (uint32_t)(slab0 + cur.slab) * a.slab_bytes + (uint32_t)q * 16u;
        uint32_t o[kPxPerLane];
        uint4 wn[kPxPerLane];
#pragma unroll
        for (int h = 0; h < kPxPerLane; ++h) {
          const int e = cur.tap * PT + pxl + (PT / kPxPerLane) * h;
          o[h] = tpix[e] + sbase;
          wn[h] = tws[e];
        }
#pragma unroll
        for (int h = 0; h < kPxPerLane; ++h) {
          const int row = pxl + (PT / kPxPerLane) * h;
#pragma unroll
          for (int half = 0; half < 2; ++half) {
            Xs[buf][tile_chunk(row, q + 4 * half)] =
                TR::blend(v[h][0][half], v[h][1][half], v[h][2][half], v[h][3][half], w[h]);
            const unsigned char *top = xt + o[h] + half * 64;
            const unsigned char *bot = top + a.row_bytes;
            v[h][0][half] = *(const uint4 *)(top);
            v[h][1][half] = *(const uint4 *)(top + pxb);
            v[h][2][half] = *(const uint4 *)(bot);
            v[h][3][half] = *(const uint4 *)(bot + pxb);
            __builtin_amdgcn_sched_barrier(0);
          }
          w[h] = wn[h];
        }
        cur.advance(nk, taps, spd);
      };

      build_table((ch0 + cur.slab * KC) / g.ch_per_dg);
      MDCN_BARRIER_LDS();  // B0: table visible

#pragma unroll
      for (int j = 0; j < kGatherAhead; ++j) issue_gather(gv[j], gw[j]);
      commit_and_refill(0, gv[0], gw[0]);
      MDCN_BARRIER_LDS();  // B1: X[0] (and the consumers' W[0]) visible

      // The step loop runs in whole rounds of kGatherAhead steps (register sets are
      // addressed statically and the body stays branch-free, so the compiler's
      // vmcnt bookkeeping sees one fixed issue pattern); steps past nk repeat the
      // last one and nobody reads what they produce.
      for (int ks0 = 0; ks0 < nk_pad; ks0 += kGatherAhead) {
#pragma unroll
        for (int j = 0; j < kGatherAhead; ++j) {
          const int ks = ks0 + j;
          const int set = (j + 1) % kGatherAhead;  // holds step ks + 1, refilled with ks + 1 + kGatherAhead
          commit_and_refill((ks + 1) & 1, gv[set], gw[set]);
          MDCN_BARRIER_LDS();  // end of step ks: X[ks+1] visible
        }
      }
      // The gathers issued past the last step are never read.  Retire them with a
      // wait the compiler can see: it tracks these loads' destination registers,
      // carries that state round the tile loop into the consumer branch (it cannot
      // know that a wave keeps its role) and would otherwise guard the consumers'
      // registers with vmcnt waits that also wait for their in-flight weight copies.
      __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0), other counters untouched
      MDCN_BARRIER_LDS();   // E0: the K loop is over for everybody
      if (is_part) {        // the consumers' two barriers around the arrival count of a cut tile
        MDCN_BARRIER_LDS();
        MDCN_BARRIER_LDS();
      }
      if (!OVL) MDCN_BARRIER_LDS();   // E1: epilogue done, tiles and table may be rewritten
    } else {
      // =================== CONSUMER ===================
      const int wave_p = wave & 1;   // which 64 pixels
      const int wave_c = wave >> 1;  // which CT/2 output channels
      f32x16 acc[NB][MB];
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[nb][mb][r] = 0.0f;

      const int frow = lane & 31;
      const int fhalf = lane >> 5;
      // bias of this lane's output channels, fetched now so that the epilogue
      // never waits on a load (a wait there would also wait for its own stores)
      float bv[MB];
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const int mycol = ctile * CT + wave_c * (CT / 2) + mb * 32 + frow;
        bv[mb] = 0.0f;
        if (a.bias && mycol < g.cout_g) bv[mb] = to_f32(((const E *)a.bias)[grp * g.cout_g + mycol]);
      }
      // mirror of the producers' issue sequence, for the table-rebuild barriers
      auto mirror_issue = [&]() {
        if (MULTI_DG && cur.new_dg) {
          cur.new_dg = false;
          MDCN_BARRIER_LDS();  // R
        }
        cur.advance(nk, taps, spd);
      };
      // Weight tile of step ks -> next ring slot, straight into LDS: lane i of
      // copy c writes chunk c*64+i of the slot and reads the source chunk that
      // the swizzle assigns to it.  The consumers issue these copies (they have
      // the idle time); they are this wave's only vector-memory operations in
      // the K loop, WDMA per step, so "at most kWeightAhead*WDMA outstanding"
      // means the next step's tile has landed.
      const unsigned char *wp_tile = (const unsigned char *)a.wp +
                                     ((size_t)(grp * a.n_ctiles + ctile) * nk_tile + kb) * (size_t)(CT * kRowB);
      uint32_t wlane[WDMA];  // byte offset of this lane's source chunk inside a tile
#pragma unroll
      for (int c = 0; c < WDMA; ++c) {
        const int d = (wave * WDMA + c) * 64 + lane;
        const int row = d >> 3;
        wlane[c] = (uint32_t)(row * kRowB + (((d & 7) ^ swz(row)) * 16));
      }
      int islot = 0;  // ring slot of the next weight tile to issue
      auto issue_weights = [&](int ks) {
        const int kk = min(ks, nk - 1);  // past the end: repeat the last tile (never read)
        const unsigned char *src = wp_tile + (size_t)kk * (CT * kRowB);
#pragma unroll
        for (int c = 0; c < WDMA; ++c) {
          const int blk = wave * WDMA + c;  // 1 KiB block of the tile
          copy16_global_to_lds(src + wlane[c], (uint32_t)(uintptr_t)(lptr_t)(&Ws[islot][blk * 64]));
        }
        islot = (islot == kWeightSlots - 1) ? 0 : islot + 1;
      };

      // (the previous tile's output stores are older than these copies, so the
      // vmcnt waits below also cover them)
#pragma unroll
      for (int j = 0; j <= kWeightAhead; ++j) issue_weights(j);
      if (!OVL || first_tile) MDCN_BARRIER_LDS();  // B0 (with OVL: passed before the previous tile's epilogue)
#pragma unroll
      for (int v = 0; v <= kGatherAhead; ++v) mirror_issue();
      MDCN_BARRIER(kWeightAhead * WDMA);  // B1: W[0] landed

      int wslot = 0;
      for (int ks = 0; ks < nk_pad; ++ks) {
        const uint4 *X = Xs[ks & 1];
        const uint4 *W = Ws[wslot];
        wslot = (wslot == kWeightSlots - 1) ? 0 : wslot + 1;
        issue_weights(ks + 1 + kWeightAhead);
        if (ks < nk) {
#pragma unroll
          for (int ksub = 0; ksub < 4; ++ksub) {
            const int ch = ksub * 2 + fhalf;
            uint4 xf[NB], wf[MB];
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) xf[nb] = X[tile_chunk(wave_p * 64 + nb * 32 + frow, ch)];
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
              wf[mb] = W[tile_chunk(wave_c * (CT / 2) + mb * 32 + frow, ch)];
#pragma unroll
            for (int nb = 0; nb < NB; ++nb)
#pragma unroll
              for (int mb = 0; mb < MB; ++mb) TR::mma(acc[nb][mb], xf[nb], wf[mb]);
          }
        }
        mirror_issue();
        MDCN_BARRIER(kWeightAhead * WDMA);  // end of step ks: W[ks+1] landed
      }
      MDCN_BARRIER(0);  // E0: copies issued past the end have landed; tiles become staging
      // B0 of the next tile, taken early: the producers need nothing from the
      // consumers for its table, gathers and first sample tile
      if (OVL && more_units) MDCN_BARRIER_LDS();

      // ---- a part of a tile: the parts meet in memory.  Every part stores its
      // accumulators (fp32, register order) and counts itself in; the part that
      // arrives last adds them up -- two parts: its own registers plus the other's
      // values, the same in either order; more: all from memory in index order, so
      // the sum does not depend on who was last -- and goes on to the epilogue; the
      // others are done.  Nobody waits for anybody; the last part leaves the counter
      // at zero for the next launch.  Stores and loads are device coherent (sc1):
      // they go past the caches private to a CU or an XCD.  A part is a workgroup's
      // last unit, and the producers take part in the two barriers.
      bool store_tile = true;
      if (is_part) {
        constexpr int NQ = NB * MB * 4;           // 16-byte quads of accumulators per lane
        constexpr int CQ = 8;                     // quads read back at a time (NQ is a multiple of 8)
        const int tslot = us.counter_slot();
        const unsigned char *pbase =
            (const unsigned char *)a.cut_part + (size_t)us.buffer_slot0() * (size_t)(PT * 256 * 4);
        const unsigned char *mine = uniform_ptr(pbase + (size_t)us.part_idx * (size_t)(PT * 256 * 4));
        // quad j of the 256 consumer lanes is one 4 KiB run.  (The offset is opaque to the optimiser,
        // which would otherwise form the addresses below ahead of the unit loop and keep them live.)
        uint32_t voff = (uint32_t)tid * 16u;
        asm volatile("" : "+v"(voff));
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
          for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int qd = 0; qd < 4; ++qd) {
              const f32x16 &c = acc[nb][mb];
              const f32x4 v = {c[4 * qd], c[4 * qd + 1], c[4 * qd + 2], c[4 * qd + 3]};
              const uint32_t vo = voff + (uint32_t)(((nb * MB + mb) * 4 + qd) * 4096);
              // (s_nop: a vector-memory instruction must not read a scalar register within five issue
              // slots of a vector instruction writing it -- a reload of spilled scalars, say -- and the
              // compiler does not look into assembly text to keep that distance)
              asm volatile("s_nop 4\n\tglobal_store_dwordx4 %0, %1, %2 sc1" : : "v"(vo), "v"(v), "s"(mine) : "memory");
            }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        MDCN_BARRIER_LDS();
        if (tid == 0)
          part_arrived = __hip_atomic_fetch_add((uint32_t *)a.cut_cnt + tslot, 1u, __ATOMIC_RELAXED,
                                                __HIP_MEMORY_SCOPE_AGENT);
        MDCN_BARRIER_LDS();
        store_tile = part_arrived == (uint32_t)(us.parts - 1);
        if (store_tile) {
          const bool two = us.parts == 2;
          const unsigned char *src0 = two ? pbase + (size_t)(1 - us.part_idx) * (size_t)(PT * 256 * 4) : pbase;
          for (int i = two ? 1 : 0; i < us.parts; ++i) {
            const unsigned char *src = uniform_ptr(src0);
#pragma unroll
            for (int q0 = 0; q0 < NQ; q0 += CQ) {
              f32x4 tmp[CQ];
#pragma unroll
              for (int j = 0; j < CQ; ++j) {
                const uint32_t vo = voff + (uint32_t)((q0 + j) * 4096);
                asm volatile("s_nop 4\n\tglobal_load_dwordx4 %0, %1, %2 sc1" : "=v"(tmp[j]) : "v"(vo), "s"(src));
              }
#pragma unroll
              for (int j = 0; j < CQ; ++j) asm volatile("s_waitcnt vmcnt(0)" : "+v"(tmp[j]));
#pragma unroll
              for (int j = 0; j < CQ; ++j) {
                const int qi = q0 + j, blk = qi >> 2, qd = qi & 3;
#pragma unroll
                for (int e = 0; e < 4; ++e)
                  acc[blk / MB][blk % MB][4 * qd + e] =
                      i == 0 ? tmp[j][e] : acc[blk / MB][blk % MB][4 * qd + e] + tmp[j][e];
              }
            }
            src0 += PT * 256 * 4;
          }
          if (tid == 0)
            __hip_atomic_store((uint32_t *)a.cut_cnt + tslot, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }

      // ---- epilogue: bias, round once, transpose through LDS, NCHW store ----
      // Accumulator block (A = samples, B = weights): register r of lane l holds
      //   pixel = (r/4)*8 + (l/32)*4 + r%4,  channel = l%32.
      constexpr int RB = stage_row_bytes<E>();
      constexpr int CHUNK_PX = 16 / ES;           // pixels per 16-byte chunk
      constexpr int CHUNKS = 64 / CHUNK_PX;       // chunks per staged row
      unsigned char *stage =
          OVL ? (unsigned char *)&Ws[kWeightSlots - 1][0] + (size_t)wave * 32 * RB
              : (wave < 2 ? (unsigned char *)&Xs[0][0] : (unsigned char *)&Ws[0][0]) + (size_t)(wave & 1) * 32 * RB;
      E *out = (E *)a.out;
      const int pw0 = p0 + wave_p * 64;           // first pixel of this wave
      const bool vec_ok = a.out_vec_ok != 0;      // 16-byte chunks never straddle images, aligned
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        if (!store_tile) break;  // a part that was not the last to arrive has nothing to store
        const int col0 = ctile * CT + wave_c * (CT / 2) + mb * 32;  // channel within the group
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
          for (int r4 = 0; r4 < 4; ++r4) {
            const int px = nb * 32 + r4 * 8 + fhalf * 4;
            TR::store4(stage + frow * RB + px * ES, acc[nb][mb][r4 * 4 + 0] + bv[mb],
                       acc[nb][mb][r4 * 4 + 1] + bv[mb], acc[nb][mb][r4 * 4 + 2] + bv[mb],
                       acc[nb][mb][r4 * 4 + 3] + bv[mb]);
          }
        }
        // the same wave wrote and now reads: only its own LDS operations matter
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll 1
        for (int it = 0; it < 32 * CHUNKS / 64; ++it) {
          const int idx = it * 64 + lane;
          const int row = idx / CHUNKS;        // channel of the block
          const int chunk_i = idx % CHUNKS;
          const int col = col0 + row;
          const int p = pw0 + chunk_i * CHUNK_PX;
          if (col < g.cout_g && p < total_px) {
            const uint4 val = *(const uint4 *)(stage + row * RB + chunk_i * 16);
            const long cbase = (long)grp * g.cout_g + col;
            if (vec_ok && p + CHUNK_PX <= total_px) {
              const int n = p / plane_out;
              const int rem = p - n * plane_out;
              *(uint4 *)(out + ((long)n * g.Cout + cbase) * plane_out + rem) = val;
            } else {
              const E *ve = (const E *)&val;
#pragma unroll 1
              for (int i = 0; i < CHUNK_PX; ++i) {
                const int pi = p + i;
                if (pi < total_px) {
                  const int ni = pi / plane_out;
                  const int ri = pi - ni * plane_out;
                  out[((long)ni * g.Cout + cbase) * plane_out + ri] = ve[i];
                }
              }
            }
          }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      }
      if (!OVL) MDCN_BARRIER_LDS();  // E1
    }
  }
}

}  // namespace mdcn
