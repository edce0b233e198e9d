// Fused DCNv2 forward for gfx950, 256-channel output tiles: the same implicit
// GEMM, tile shapes, LDS layouts and input copy as mdcn_fused.h, with another
// division of labour.
//
// Eight wavefronts, all alike.  Per K step (128 bytes of channels of one tap)
// every wave
//   * "produces" 16 of the tile's 128 pixels: waits for the gather it issued two
//     steps earlier (4 corners x 2 x 16 bytes per lane, held in registers),
//     blends the corners into 2 x 16 bytes of the sample tile, writes them to
//     LDS and refills the registers with the gather of the step after next;
//   * issues its share (4 x 1 KiB) of the direct-to-LDS copy of the weight tile
//     of the next step;
//   * "consumes": 16 MFMAs (32x32x16) on its 64 pixel x 64 channel part of the
//     tile, fragments read from LDS.
// One workgroup barrier per step.  The two waves that share a SIMD run the two
// halves in opposite order (waves 0-3: MFMA, produce, barrier; waves 4-7: MFMA,
// barrier, produce -- the same instruction stream with the barrier at another
// place), so that the matrix pipe of a SIMD works for one wave while its
// vector ALU blends for the other.
//
// The blend itself runs on the matrix pipe for 16-bit types: one
// v_mfma_f32_4x4x4 (16 blocks of 4x4x4) takes the four lanes that serve one
// pixel as one block, the lane's 4 channels as a column of B and
// (corner weight) x identity as A, so four instructions -- one per corner --
// accumulate the bilinear sum of 4 channels in fp32 without unpacking the
// 16-bit values on the vector ALU (which would otherwise be the busiest unit of
// the kernel).  fp32 tensors blend with FMAs.
//
// All vector-memory traffic of the K loop is issued from inline assembly and
// waited for with explicit counts: a wave has 2 x 8 gather loads and the weight
// copies of up to three steps in flight, and the compiler's own bookkeeping
// would drain them at every use.  Per wave and K step the order of issue is
// fixed: kWD weight copies, then 8 gather loads (two groups of four, each group
// issued right after the blend that frees its registers), which makes the
// number of younger operations at every wait a constant.
#pragma once

#include "mdcn_fused.h"

namespace mdcn {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));

constexpr int kF2Threads = 512;
constexpr int kF2CT = 256;             // output channels per tile
constexpr int kF2Slots = 3;            // ring of weight tiles
constexpr int kF2GL = 8;               // gather loads per wave and K step
constexpr int kF2WD = kF2CT / 64;      // 1 KiB weight copies per wave and K step
constexpr int kF2Sets = 3;             // gather register sets: a gather is in flight for kF2Sets steps
constexpr int kF2Unroll = 6;           // steps per round of the K loop: sets, sample tiles and ring slots are static
// vector-memory operations younger than the last load of a gather group (half a
// set) when that group is blended: the rest of its set, the copies and loads of
// the steps issued since, the copies of the current step, the refills issued so far
constexpr int kF2VmBlend = (kF2GL - 4) + (kF2Sets - 1) * (kF2WD + kF2GL) + kF2WD;
// ... younger than the weight copies that must have landed at a step's barrier
constexpr int kF2VmBar = 2 * kF2GL + kF2WD;
static_assert(kF2VmBlend < 64 && kF2VmBar < 64, "vmcnt holds 6 bits");
static_assert(kF2Unroll % kF2Sets == 0 && kF2Unroll % 2 == 0 && kF2Unroll % kF2Slots == 0, "static indices");

constexpr size_t fused2_lds_bytes(int tmax) {
  return (size_t)2 * kPT * kRowB + (size_t)kF2Slots * kF2CT * kRowB + (size_t)kPT * tmax * 20;
}

// 16 bytes per lane from `base` (two SGPRs) + 32-bit byte offset + immediate
#ifndef MDCN_F2_ABLATE
#define MDCN_F2_ABLATE 0
#endif
#ifndef MDCN_F2_PROFILE
#define MDCN_F2_PROFILE 0
#endif
#if MDCN_F2_PROFILE
#define MDCN_PROF(slot) do { const long long t_ = clock64(); prof_acc[slot] += t_ - prof_t; prof_t = t_; } while (0)
#else
#define MDCN_PROF(slot) do { } while (0)
#endif
#if MDCN_F2_ABLATE & 1
#define MDCN_GLOAD(dst, voff, base, imm) asm volatile("" : "=v"(dst) : "v"(voff), "s"(base), "n"(imm))
#else
#define MDCN_GLOAD(dst, voff, base, imm) \
  asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "=v"(dst) : "v"(voff), "s"(base), "n"(imm))
#endif
#define MDCN_DSREAD(dst, addr, imm) \
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(imm))
// wait until at most N vector-memory (LDS) operations of this wave are outstanding;
// the four registers become usable only afterwards
#define MDCN_VMWAIT4(N, a, b, c, d) \
  asm volatile("s_waitcnt vmcnt(%4)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d) : "n"(N))
#define MDCN_LGKMWAIT4(N, a, b, c, d) \
  asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d) : "n"(N))
typedef __attribute__((address_space(3))) u32x4 *lds_u32x4_ptr;
static_assert(kF2WD == 4, "issue_weights spells out four copies");

// Blend of one 16-byte chunk (8 or 4 channels) from the same chunk at the four
// corners.  prep() turns a table entry into what run() needs, once per step.
template <typename E>
struct Blend2;

template <typename E>
struct Blend2Half {
  struct Wt { u32x2 a[4]; };
  // sh, m0, m1 depend on the lane's place q among the four lanes of its pixel:
  // the corner weight sits at K position q of the lane's row of A, zeros elsewhere
  static __device__ __forceinline__ Wt prep(const uint4 &tw, uint32_t sh, uint32_t m0, uint32_t m1) {
    const uint32_t c[4] = {tw.x & 0xffffu, tw.x >> 16, tw.y & 0xffffu, tw.y >> 16};
    Wt w;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t v = c[i] << sh;
      w.a[i].x = v & m0;
      w.a[i].y = v & m1;
    }
    return w;
  }
  static __device__ __forceinline__ u32x4 run(const u32x4 (&v)[4], const Wt &w) {
    f32x4 d0 = {0.f, 0.f, 0.f, 0.f}, d1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const u32x2 b0 = {v[c].x, v[c].y}, b1 = {v[c].z, v[c].w};
      d0 = Blend2<E>::mma4(w.a[c], b0, d0);
      d1 = Blend2<E>::mma4(w.a[c], b1, d1);
    }
    u32x4 o;
    o.x = ElemTraits<E>::pack2(d0[0], d0[1]);
    o.y = ElemTraits<E>::pack2(d0[2], d0[3]);
    o.z = ElemTraits<E>::pack2(d1[0], d1[1]);
    o.w = ElemTraits<E>::pack2(d1[2], d1[3]);
    return o;
  }
  static __device__ __forceinline__ void table_weights(const TapSample &s, uint32_t (&tw)[4]) {
    Half16Traits<E>::table_weights(s, tw);  // (w00, w01), (w10, w11) rounded to E
  }
};

#ifndef MDCN_F2_BLEND_MFMA
#define MDCN_F2_BLEND_MFMA 0
#endif
#if MDCN_F2_BLEND_MFMA
template <>
struct Blend2<bf16_t> : Blend2Half<bf16_t> {
  static __device__ __forceinline__ f32x4 mma4(const u32x2 &a, const u32x2 &b, const f32x4 &c) {
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    return __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(s16x4, a), __builtin_bit_cast(s16x4, b), c, 0, 0, 0);
  }
};

template <>
struct Blend2<f16_t> : Blend2Half<f16_t> {
  static __device__ __forceinline__ f32x4 mma4(const u32x2 &a, const u32x2 &b, const f32x4 &c) {
    return __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(f16x4, a), __builtin_bit_cast(f16x4, b), c, 0, 0, 0);
  }
};
#else
// bf16 on the vector ALU: a 32-bit word holds two channels; shifting / masking
// turns each into an fp32 value exactly, the four corners are summed with fp32
// FMAs (fp32 weights) and the pair is rounded to bf16 once.
template <>
struct Blend2<bf16_t> {
  struct Wt { float w[4]; };
  static __device__ __forceinline__ Wt prep(const uint4 &tw, uint32_t, uint32_t, uint32_t) {
    Wt w;
    w.w[0] = __uint_as_float(tw.x); w.w[1] = __uint_as_float(tw.y);
    w.w[2] = __uint_as_float(tw.z); w.w[3] = __uint_as_float(tw.w);
    return w;
  }
  static __device__ __forceinline__ u32x4 run(const u32x4 (&v)[4], const Wt &w) {
    u32x4 o;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float lo = w.w[0] * __uint_as_float(v[0][j] << 16);
      float hi = w.w[0] * __uint_as_float(v[0][j] & 0xffff0000u);
#pragma unroll
      for (int c = 1; c < 4; ++c) {
        lo = __builtin_fmaf(w.w[c], __uint_as_float(v[c][j] << 16), lo);
        hi = __builtin_fmaf(w.w[c], __uint_as_float(v[c][j] & 0xffff0000u), hi);
      }
      o[j] = ElemTraits<bf16_t>::pack2(lo, hi);
    }
    return o;
  }
  static __device__ __forceinline__ void table_weights(const TapSample &s, uint32_t (&tw)[4]) {
    ElemTraits<float>::table_weights(s, tw);
  }
};

// fp16 has packed arithmetic: see ElemTraits<f16_t>::blend
template <>
struct Blend2<f16_t> {
  struct Wt { uint4 w; };
  static __device__ __forceinline__ Wt prep(const uint4 &tw, uint32_t, uint32_t, uint32_t) {
    Wt w;
    w.w = tw;
    return w;
  }
  static __device__ __forceinline__ u32x4 run(const u32x4 (&v)[4], const Wt &w) {
    const uint4 r = ElemTraits<f16_t>::blend(__builtin_bit_cast(uint4, v[0]), __builtin_bit_cast(uint4, v[1]),
                                             __builtin_bit_cast(uint4, v[2]), __builtin_bit_cast(uint4, v[3]), w.w);
    return __builtin_bit_cast(u32x4, r);
  }
  static __device__ __forceinline__ void table_weights(const TapSample &s, uint32_t (&tw)[4]) {
    ElemTraits<f16_t>::table_weights(s, tw);
  }
};
#endif

template <>
struct Blend2<float> {
  struct Wt { float w[4]; };
  static __device__ __forceinline__ Wt prep(const uint4 &tw, uint32_t, uint32_t, uint32_t) {
    Wt w;
    w.w[0] = __uint_as_float(tw.x); w.w[1] = __uint_as_float(tw.y);
    w.w[2] = __uint_as_float(tw.z); w.w[3] = __uint_as_float(tw.w);
    return w;
  }
  static __device__ __forceinline__ u32x4 run(const u32x4 (&v)[4], const Wt &w) {
    u32x4 o;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float acc = w.w[0] * __uint_as_float(v[0][j]);
      acc = acc + w.w[1] * __uint_as_float(v[1][j]);
      acc = acc + w.w[2] * __uint_as_float(v[2][j]);
      acc = acc + w.w[3] * __uint_as_float(v[3][j]);
      o[j] = __float_as_uint(acc);
    }
    return o;
  }
  static __device__ __forceinline__ void table_weights(const TapSample &s, uint32_t (&tw)[4]) {
    ElemTraits<float>::table_weights(s, tw);
  }
};

template <typename E, int TMAX, bool UNBORDERED>
__global__ __launch_bounds__(kF2Threads) void fused2_kernel(FusedArgs a) {
  using TR = ElemTraits<E>;
  using BL = Blend2<E>;
  constexpr int PT = kPT;
  constexpr int CT = kF2CT;
  constexpr int KC = TR::KC;
  constexpr int ES = (int)sizeof(E);
  constexpr int NS = kF2Sets;
  constexpr int TPT = (TMAX + 3) / 4;          // table entries per lane and build
  constexpr int NB = 2, MB = 2;                // 32 x 32 accumulator blocks per wave: pixels x channels
  constexpr uint32_t kXTile = PT * kRowB, kWTile = CT * kRowB;

  __shared__ uint4 Xs[2][PT * kRowChunks];               // sample tiles
  __shared__ uint4 Ws[kF2Slots][CT * kRowChunks];        // weight tiles
  __shared__ uint32_t tpix[PT * TMAX];                   // (pixel, tap) table, [tap][PT]: corner byte offset
  __shared__ uint4 tws[PT * TMAX];                       // ... and the blend weights

  const Geom &g = a.g;
  const int taps = g.taps;
  const int nk = a.slabs * taps;
  const int nk_pad = (nk + kF2Unroll - 1) / kF2Unroll * kF2Unroll;
  const int plane_out = g.Ho * g.Wo;
  const int total_px = (int)a.total_px;
  const int spd = g.ch_per_dg / KC;  // slabs per deformable group

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // waves 4..7 run the produce half of a step after its barrier (see above)
  const bool late = wave >= 4;
  const int ahead = late ? 2 : 1;

  const uint32_t lds_x = (uint32_t)(uintptr_t)(lptr_t)(&Xs[0][0]);
  const uint32_t lds_w = (uint32_t)(uintptr_t)(lptr_t)(&Ws[0][0]);

  // ---- produce role: lane serves 16-byte chunks q and q + 4 of pixel pl
  const int q = lane & 3;
  const int pl = wave * 16 + (lane >> 2);
  const uint32_t bsh = (uint32_t)(q & 1) * 16u;
  const uint32_t bm0 = q < 2 ? 0xffffffffu : 0u, bm1 = ~bm0;
  const uint32_t xw0 = lds_x + (uint32_t)tile_chunk(pl, q) * 16u;       // where its two chunks go in X[0]
  const uint32_t xw1 = lds_x + (uint32_t)tile_chunk(pl, q + 4) * 16u;
  const unsigned char *xt = (const unsigned char *)a.xt;
  const uint32_t pxb = UNBORDERED ? a.px_bytes : (uint32_t)kRowB;

  // ---- consume role: 64 pixels x 64 channels
  const int wave_p = wave & 1, wave_c = wave >> 1;
  const int frow = lane & 31, fhalf = lane >> 5;
  const uint32_t xa0 = (uint32_t)tile_chunk(wave_p * 64 + frow, fhalf) * 16u;   // K sub-step s: ^ (s << 5)
  const uint32_t wa0 = (uint32_t)tile_chunk(wave_c * 64 + frow, fhalf) * 16u;

  // weight copies: a wave copies kF2WD consecutive 1 KiB blocks (8 rows each) of
  // the tile; lane i of a copy writes chunk i of the block and reads the source
  // chunk the swizzle assigns to it.  The swizzle looks at bits 1..3 of the row:
  // bits 1, 2 come from the lane, bit 3 is the block's parity, which flips bit 1
  // of the chunk number, i.e. bit 5 of the byte offset, for the odd blocks.
  const uint32_t wlane = (uint32_t)(wave * kF2WD) * 1024u +
                         (uint32_t)((lane >> 3) * kRowB + (((lane & 7) ^ swz(lane >> 3)) * 16));

  // XCD-aware persistent schedule (as in fused_kernel)
  const int total_tiles = a.n_ptiles * a.n_ctiles * g.G;
  const int xcd = (int)(blockIdx.x & 7);
  const int wg_in_xcd = (int)(blockIdx.x >> 3);
  const int wgs_per_xcd = (int)(gridDim.x >> 3);
  const int chunk = (total_tiles + 7) >> 3;
  const int tile_end = min((xcd + 1) * chunk, total_tiles);

  // ---- state of the tile whose gathers are being issued
  int ctile = 0, grp = 0, p0 = 0, ch0 = 0, slab0 = 0;
  int tb_n = 0, tb_ho = 0, tb_wo = 0, tb_rem = 0;
  bool tb_valid = false;
  const int tb_pl = tid & (PT - 1);
  const unsigned char *wp_tile = nullptr;
  StepCursor cur;   // the next step whose gather is issued
  StepCursor bcur;  // the next step to blend
  auto set_tile = [&](int tile) {
    int L = tile;
    ctile = L % a.n_ctiles;
    L /= a.n_ctiles;
    grp = L % g.G;
    p0 = (L / g.G) * PT;
    ch0 = grp * g.cin_g;
    slab0 = ch0 / KC;
    // table: lane serves pixel tid % 128, taps tid / 128 + 4 i
    const int tb_p = p0 + tb_pl;
    tb_valid = tb_p < total_px;
    tb_n = tb_ho = tb_wo = tb_rem = 0;
    if (tb_valid) {
      tb_n = tb_p / plane_out;
      tb_rem = tb_p - tb_n * plane_out;
      tb_ho = tb_rem / g.Wo;
      tb_wo = tb_rem - tb_ho * g.Wo;
    }
    wp_tile = (const unsigned char *)a.wp + ((size_t)(grp * a.n_ctiles + ctile) * nk) * (size_t)kWTile;
    cur.init(slab0, spd);
    bcur.init(slab0, spd);
  };
  auto build_table = [&](int dgi) {
    // (opaque to the optimiser: the per-tap address arithmetic below would otherwise
    // be computed once per kernel and kept in -- spilled -- registers across the K loop)
    int tapq = tid >> 7;
    asm volatile("" : "+v"(tapq));
    const E *off = (const E *)a.om.off + (long)tb_n * a.om.off_n + (long)tb_rem * a.om.off_px +
                   (long)(dgi * 2 * taps) * a.om.off_ch;
    const E *msk = (const E *)a.om.msk + (long)tb_n * a.om.msk_n + (long)tb_rem * a.om.msk_px +
                   (long)(dgi * taps) * a.om.msk_ch;
    E rdy[TPT], rdx[TPT], rm[TPT];
#pragma unroll
    for (int i = 0; i < TPT; ++i) {
      const int tap = min(tapq + 4 * i, taps - 1);
      rdy[i] = off[(long)(2 * tap) * a.om.off_ch];
      rdx[i] = off[(long)(2 * tap + 1) * a.om.off_ch];
      rm[i] = msk[(long)tap * a.om.msk_ch];
    }
#pragma unroll
    for (int i = 0; i < TPT; ++i) {
      const int tap = tapq + 4 * i;
      if (tap < taps) {
        const int ti = tap / g.kw, tj = tap - ti * g.kw;
        TapSample sm = make_tap_sample(tb_ho * g.sh - g.ph + ti * g.dh, tb_wo * g.sw - g.pw + tj * g.dw,
                                       to_f32(rdy[i]), to_f32(rdx[i]), mask_value<E>(rm[i], a.om.logit), g.H, g.W);
        const uint32_t pix = tb_valid ? (uint32_t)tb_n * a.img_bytes + corner_offset<UNBORDERED>(sm, g, a) : 0u;
        uint32_t tw[4];
        BL::table_weights(sm, tw);
        if (!tb_valid) tw[0] = tw[1] = tw[2] = tw[3] = 0u;
        tpix[tap * PT + tb_pl] = pix;
        tws[tap * PT + tb_pl] = make_uint4(tw[0], tw[1], tw[2], tw[3]);
      }
    }
  };

  // gather registers: sets x two halves of the 128-byte row x four corners
  u32x4 gs[NS][2][4];

  // addresses of the gather cursor's step, then move the cursor on
  uint32_t o_tl, o_tr, o_bl, o_br;
  auto next_addresses = [&]() {
    const int e = cur.tap * PT + pl;
    o_tl = tpix[e] + (uint32_t)(slab0 + cur.slab) * a.slab_bytes + (uint32_t)q * 16u;
    o_tr = o_tl + pxb;
    o_bl = o_tl + a.row_bytes;
    o_br = o_bl + pxb;
    cur.advance(nk, taps, spd);
  };
#define MDCN_F2_GATHER_HALF(S, H)                     \
  do {                                                \
    MDCN_GLOAD(S[H][0], o_tl, xt, 0 + 64 * (H));      \
    MDCN_GLOAD(S[H][1], o_tr, xt, 0 + 64 * (H));      \
    MDCN_GLOAD(S[H][2], o_bl, xt, 0 + 64 * (H));      \
    MDCN_GLOAD(S[H][3], o_br, xt, 0 + 64 * (H));      \
  } while (0)
#define MDCN_F2_GATHER(SI)                            \
  do {                                                \
    next_addresses();                                 \
    MDCN_F2_GATHER_HALF(gs[SI], 0);                   \
    MDCN_F2_GATHER_HALF(gs[SI], 1);                   \
  } while (0)

  int islot = 0;  // ring slot of the next weight tile to issue
  auto issue_weights = [&](int ks) {
    const int kk = min(ks, nk - 1);  // past the end: repeat the last tile (never read)
    const uint32_t voff = (uint32_t)kk * kWTile + wlane;
    const uint32_t voff_odd = voff ^ 32u;
    const uint32_t dst = lds_w + (uint32_t)islot * kWTile + (uint32_t)(wave * kF2WD) * 1024u;
    if (!(MDCN_F2_ABLATE & 2)) {
      // (the instruction's offset moves the LDS side along with the global one)
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\t"
                   "global_load_lds_dwordx4 %1, %3\n\t"
                   "global_load_lds_dwordx4 %2, %3 offset:1024\n\t"
                   "global_load_lds_dwordx4 %1, %3 offset:2048\n\t"
                   "global_load_lds_dwordx4 %2, %3 offset:3072"
                   :
                   : "s"(dst), "v"(voff), "v"(voff_odd), "s"(wp_tile)
                   : "memory");
    }
    islot = (islot == kF2Slots - 1) ? 0 : islot + 1;
  };

  // One produce block: the weight copies of step j + 1, the blend of step j
  // (gather set SI) into sample tile j % 2, the gather of step j + NS into the set.
#define MDCN_F2_BLOCK(J, SI)                                                            \
  do {                                                                                  \
    const int j_ = (J);                                                                 \
    if (j_ < nk) {                                                                      \
      issue_weights(j_ + 1);                                                            \
      next_addresses();                                                                 \
      const typename BL::Wt w_ = BL::prep(tws[bcur.tap * PT + pl], bsh, bm0, bm1);      \
      bcur.advance(nk, taps, spd);                                                      \
      const uint32_t xo_ = (j_ & 1) ? kXTile : 0u;                                      \
      MDCN_VMWAIT4(kF2VmBlend, gs[SI][0][0], gs[SI][0][1], gs[SI][0][2], gs[SI][0][3]); \
      {                                                                                 \
        const u32x4 o_ = (MDCN_F2_ABLATE & 4) ? (gs[SI][0][0] ^ gs[SI][0][1] ^ gs[SI][0][2] ^ gs[SI][0][3]) \
                                              : BL::run(gs[SI][0], w_);                 \
        *(lds_u32x4_ptr)(xw0 + xo_) = o_;                                               \
      }                                                                                 \
      MDCN_F2_GATHER_HALF(gs[SI], 0);                                                   \
      MDCN_VMWAIT4(kF2VmBlend, gs[SI][1][0], gs[SI][1][1], gs[SI][1][2], gs[SI][1][3]); \
      {                                                                                 \
        const u32x4 o_ = (MDCN_F2_ABLATE & 4) ? (gs[SI][1][0] ^ gs[SI][1][1] ^ gs[SI][1][2] ^ gs[SI][1][3]) \
                                              : BL::run(gs[SI][1], w_);                 \
        *(lds_u32x4_ptr)(xw1 + xo_) = o_;                                               \
      }                                                                                 \
      MDCN_F2_GATHER_HALF(gs[SI], 1);                                                   \
    }                                                                                   \
  } while (0)

  f32x16 acc[NB][MB];
  int rslot = 0;  // ring slot of the weight tile the next MFMA step reads
  auto mfma_step = [&](int k) {
    const uint32_t xb = lds_x + ((k & 1) ? kXTile : 0u) + xa0;
    const uint32_t wb = lds_w + (uint32_t)rslot * kWTile + wa0;
    rslot = (rslot == kF2Slots - 1) ? 0 : rslot + 1;
    if (k >= nk) return;
    u32x4 xf[4][NB], wf[4][MB];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const uint32_t xk = xb ^ (uint32_t)(s << 5), wk = wb ^ (uint32_t)(s << 5);
      MDCN_DSREAD(xf[s][0], xk, 0); MDCN_DSREAD(xf[s][1], xk, 4096);
      MDCN_DSREAD(wf[s][0], wk, 0); MDCN_DSREAD(wf[s][1], wk, 4096);
    }
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      if (s < 3) MDCN_LGKMWAIT4(4, xf[s][0], xf[s][1], wf[s][0], wf[s][1]);
      else MDCN_LGKMWAIT4(0, xf[s][0], xf[s][1], wf[s][0], wf[s][1]);
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
          if (!(MDCN_F2_ABLATE & 8)) TR::mma(acc[nb][mb], __builtin_bit_cast(uint4, xf[s][nb]), __builtin_bit_cast(uint4, wf[s][mb]));
          else acc[nb][mb][s] += __uint_as_float(xf[s][nb].x ^ wf[s][mb].y);
      if (s + 2 < 4) {
        const uint32_t xk = xb ^ (uint32_t)((s + 2) << 5), wk = wb ^ (uint32_t)((s + 2) << 5);
        MDCN_DSREAD(xf[s + 2][0], xk, 0); MDCN_DSREAD(xf[s + 2][1], xk, 4096);
        MDCN_DSREAD(wf[s + 2][0], wk, 0); MDCN_DSREAD(wf[s + 2][1], wk, 4096);
      }
    }
  };

  // Table and first gathers of a tile.  A wave keeps step j in set j % NS; the
  // late waves, which run one block ahead, in set (j + NS - 1) % NS, so that both
  // kinds use the same set at the same place of the K loop.  The issue order
  // gather, copies, gather, copies, ... is the K loop's, which keeps the counts
  // of the waits valid from the first block on (the second group of copies
  // repeats what block 0 issues again: same data, same slot).
  auto tile_prologue = [&](int tile) {
    set_tile(tile);
    __builtin_amdgcn_sched_barrier(0);
    build_table(ch0 / g.ch_per_dg);
    MDCN_BARRIER_LDS();  // T0: table visible
    __builtin_amdgcn_sched_barrier(0);
    islot = 0;
    rslot = 0;
    if (!late) {
      MDCN_F2_GATHER(0);
      issue_weights(0);
      MDCN_F2_GATHER(1);
      issue_weights(1);
      islot = 1;
      MDCN_F2_GATHER(2);
    } else {
      MDCN_F2_GATHER(2);
      issue_weights(0);
      MDCN_F2_GATHER(0);
      issue_weights(1);
      islot = 1;
      MDCN_F2_GATHER(1);
    }
  };
  static_assert(kF2Sets == 3, "the prologue spells out three sets");

#if MDCN_F2_PROFILE
  long long prof_acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  long long prof_t = clock64();
#endif
  int tile = xcd * chunk + wg_in_xcd;
  if (tile < tile_end) tile_prologue(tile);
  MDCN_PROF(2);

  while (tile < tile_end) {
    // the tile whose products are accumulated now (the state above moves on to
    // the next tile before this one's results are stored)
    const int c_ctile = ctile, c_grp = grp, c_p0 = p0;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[nb][mb][r] = 0.0f;

    if (!late) {
      MDCN_F2_BLOCK(0, 0);
    } else {
      MDCN_F2_BLOCK(0, 2);
      MDCN_F2_BLOCK(1, 0);
    }
    MDCN_PROF(2);
    MDCN_BARRIER(kF2VmBar);  // X[0] and W[0] complete
    __builtin_amdgcn_sched_barrier(0);
    MDCN_PROF(1);

    // ---- K loop: kF2Unroll steps per round; step k runs block k + 1 (late waves: k + 2) on set (k + 1) % NS
#define MDCN_F2_STEP(K, SI)                                   \
  do {                                                        \
    mfma_step(K);                                             \
    __builtin_amdgcn_sched_barrier(0);                        \
    MDCN_PROF(3);                                             \
    if (late) MDCN_BARRIER(kF2VmBar);                         \
    __builtin_amdgcn_sched_barrier(0);                        \
    MDCN_PROF(5);                                             \
    MDCN_F2_BLOCK((K) + ahead, SI);                           \
    __builtin_amdgcn_sched_barrier(0);                        \
    MDCN_PROF(4);                                             \
    if (!late) MDCN_BARRIER(kF2VmBar);                        \
    __builtin_amdgcn_sched_barrier(0);                        \
    MDCN_PROF(5);                                             \
  } while (0)
    for (int k = 0; k < nk_pad; k += kF2Unroll) {
      MDCN_F2_STEP(k + 0, 1);
      MDCN_F2_STEP(k + 1, 2);
      MDCN_F2_STEP(k + 2, 0);
      MDCN_F2_STEP(k + 3, 1);
      MDCN_F2_STEP(k + 4, 2);
      MDCN_F2_STEP(k + 5, 0);
    }
    // every copy and gather issued past the last step has landed, every wave is
    // through with the table, the sample tiles and the ring
    MDCN_VMWAIT4(0, gs[0][0][0], gs[0][1][0], gs[1][0][0], gs[2][1][0]);
    MDCN_BARRIER(0);  // E0
    __builtin_amdgcn_sched_barrier(0);
    MDCN_PROF(5);

    // bias of this lane's output channels
    float bv[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      const int mycol = c_ctile * CT + wave_c * 64 + mb * 32 + frow;
      bv[mb] = 0.0f;
      if (a.bias && mycol < g.cout_g) bv[mb] = to_f32(((const E *)a.bias)[c_grp * g.cout_g + mycol]);
    }

    // ---- epilogue: bias, one rounding, NCHW store straight from the accumulators.
    // Accumulator block (A = samples, B = weights): register r of lane l holds
    //   pixel = (r/4)*8 + (l/32)*4 + r%4,  channel = l%32.
    // 16-bit types: the two halves of the wave exchange packed pixel pairs
    // (v_permlane32_swap), after which a lane holds 8 consecutive pixels = 16 bytes.
    {
      E *out = (E *)a.out;
      const bool vec_ok = a.out_vec_ok != 0;
      const int pw0 = c_p0 + wave_p * 64;
      auto store_run = [&](int col, int p, const uint4 &val) {  // 16 bytes: pixels p .. of channel col
        constexpr int RUN = 16 / ES;
        if (col >= g.cout_g || p >= total_px) return;
        const long cbase = (long)c_grp * g.cout_g + col;
        if (vec_ok && p + RUN <= total_px) {
          const int n = p / plane_out;
          const int rem = p - n * plane_out;
          *(uint4 *)(out + ((long)n * g.Cout + cbase) * plane_out + rem) = val;
        } else {
          const E *ve = (const E *)&val;
#pragma unroll 1
          for (int i = 0; i < RUN; ++i) {
            const int pi = p + i;
            if (pi < total_px) {
              const int ni = pi / plane_out;
              const int ri = pi - ni * plane_out;
              out[((long)ni * g.Cout + cbase) * plane_out + ri] = ve[i];
            }
          }
        }
      };
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const int col = c_ctile * CT + wave_c * 64 + mb * 32 + frow;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          const f32x16 &c = acc[nb][mb];
          if constexpr (ES == 2) {
#pragma unroll
            for (int g2 = 0; g2 < 2; ++g2) {
              const int ga = 2 * g2, gb = 2 * g2 + 1;
              const uint32_t a0 = TR::pack2(c[4 * ga + 0] + bv[mb], c[4 * ga + 1] + bv[mb]);
              const uint32_t a1 = TR::pack2(c[4 * ga + 2] + bv[mb], c[4 * ga + 3] + bv[mb]);
              const uint32_t b0 = TR::pack2(c[4 * gb + 0] + bv[mb], c[4 * gb + 1] + bv[mb]);
              const uint32_t b1 = TR::pack2(c[4 * gb + 2] + bv[mb], c[4 * gb + 3] + bv[mb]);
              // lower half keeps group ga and receives the upper half's part of it; upper half likewise with gb
              const auto s0 = __builtin_amdgcn_permlane32_swap(a0, b0, false, false);
              const auto s1 = __builtin_amdgcn_permlane32_swap(a1, b1, false, false);
              const int p = pw0 + nb * 32 + 8 * (fhalf ? gb : ga);
              store_run(col, p, make_uint4(s0[0], s1[0], s0[1], s1[1]));
            }
          } else {
#pragma unroll
            for (int gq = 0; gq < 4; ++gq) {
              const int p = pw0 + nb * 32 + 8 * gq + 4 * fhalf;
              store_run(col, p, make_uint4(__float_as_uint(c[4 * gq + 0] + bv[mb]), __float_as_uint(c[4 * gq + 1] + bv[mb]),
                                           __float_as_uint(c[4 * gq + 2] + bv[mb]), __float_as_uint(c[4 * gq + 3] + bv[mb])));
            }
          }
        }
      }
    }
    MDCN_PROF(6);
    __builtin_amdgcn_sched_barrier(0);  // (keeps the next tile's address arithmetic out of the epilogue's registers)
    // ---- the next tile's table and first gathers
    tile += wgs_per_xcd;
    if (tile < tile_end) tile_prologue(tile);
    __builtin_amdgcn_sched_barrier(0);
    MDCN_PROF(0);

  }
#undef MDCN_F2_STEP
#undef MDCN_F2_BLOCK
#undef MDCN_F2_GATHER
#undef MDCN_F2_GATHER_HALF
#if MDCN_F2_PROFILE
  // slots: 0 next tile's table and first gathers, 1 barrier before the K loop, 2 first blocks, 3 MFMA steps,
  //        4 produce blocks, 5 step barriers, 6 epilogue
  if (a.prof && lane == 0 && (blockIdx.x == 0 || blockIdx.x == 101))
    for (int i = 0; i < 8; ++i) ((long long *)a.prof)[((blockIdx.x ? 1 : 0) * 8 + wave) * 8 + i] = prof_acc[i];
#endif
}

}  // namespace mdcn
