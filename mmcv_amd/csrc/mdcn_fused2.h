// Fused DCNv2 forward for gfx950, 16-bit tensors, 256-channel output tiles, one
// deformable group: the same implicit GEMM, tile shapes, LDS tile layouts and
// input copy as mdcn_fused.h, with another division of labour.
//
// Eight wavefronts, all alike.  Per K step (128 bytes of channels of one tap)
// every wave
//   * "produces" 16 of the tile's 128 pixels: waits for the gather it issued
//     two steps earlier (4 corners x 16 bytes of each of two pixels per lane,
//     held in registers: eight lanes read a pixel's whole 128-byte row),
//     blends the corners into 2 x 16 bytes of the sample tile, writes them to
//     LDS and refills the registers with the gather of two steps ahead;
//   * issues its share (4 x 1 KiB) of the direct-to-LDS copy of the weight tile
//     of the next step;
//   * "consumes": 16 MFMAs (32x32x16) on its 64 pixel x 64 channel part of the
//     tile, fragments read from LDS.
// One workgroup barrier per step.  The two waves that share a SIMD run the two
// halves in opposite order (waves 0-3: MFMA, produce, barrier; waves 4-7: MFMA,
// barrier, produce -- the same instruction stream with the barrier at another
// place), so that one wave of a SIMD computes while the other waits for memory.
//
// The produce side streams across the tiles of a workgroup: its three cursors
// (gather, blend, weight copy) walk one sequence of steps -- tile after tile,
// each tile's step count padded to a multiple of six so that register sets,
// sample tiles and ring slots are addressed statically -- and step over a tile
// boundary three, zero and one step ahead of the consume side, so the memory
// pipeline never drains between tiles.  The (pixel, tap) table exists twice;
// the next tile's is built during the second round of the current tile's K
// loop.  At the end of a tile a wave stores its accumulators straight from
// registers (the two halves of the wave exchange packed pixel pairs with
// v_permlane32_swap, after which a lane holds 16 bytes of one channel's row).
//
// All vector-memory traffic of the K loop is issued from inline assembly and
// waited for with explicit counts: a wave has 2 x 8 gather loads and the weight
// copies of up to three steps in flight, and the compiler's own bookkeeping
// would drain them at every use.  Per wave and K step the order of issue is
// fixed: kWD weight copies, then 8 gather loads (two groups of four, each group
// issued right after the blend that frees its registers), which makes the
// number of younger operations at every wait a constant.
//
#pragma once

#include "mdcn_fused.h"

namespace mdcn {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));

constexpr int kF2Threads = 512;
constexpr int kF2CT = 256;             // output channels per tile at most (the template parameter CT: 256 or 128)
constexpr int kF2Slots = 3;            // ring of weight tiles
constexpr int kF2GL = 8;               // gather loads per wave and K step
// Gather register sets: a gather is in flight for kF2Sets steps.  Two are enough -- the loaded latency of a
// gather is well under one step, and three sets measure the same on every shape tried (+-0.5 %) --
// and leave the 256-channel kernel at 224 instead of 256 vector registers.
#ifndef MDCN_F2_SETS
#define MDCN_F2_SETS 2
#endif
constexpr int kF2Sets = MDCN_F2_SETS;
constexpr int kF2Unroll = 6;           // steps per round of the K loop: sets, sample tiles and ring slots are static
static_assert(kF2Unroll % kF2Sets == 0 && kF2Unroll % 2 == 0 && kF2Unroll % kF2Slots == 0, "static indices");

constexpr int kF2Taps = kTapsSmall;    // table capacity (kh * kw)
constexpr int kF2MinSteps = 18;        // padded steps per tile the streaming needs (the next table is built in the second pass of the K loop)
constexpr size_t fused2_lds_bytes(int CT) {
  return (size_t)2 * kPT * kRowB + (size_t)kF2Slots * CT * kRowB + (size_t)2 * kPT * kF2Taps * 12 + 16;
}

// 16 bytes per lane from `base` (two SGPRs) + 32-bit byte offset + immediate
#define MDCN_GLOAD(dst, voff, base, imm) \
  asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "=v"(dst) : "v"(voff), "s"(base), "n"(imm))
#define MDCN_DSREAD(dst, addr, imm) \
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(imm))
// wait until at most N vector-memory (LDS) operations of this wave are outstanding;
// the four registers become usable only afterwards (the comment names them for the
// build's scan of the assembly, asm_check.py)
#define MDCN_VMWAIT4(N, a, b, c, d) \
  asm volatile("s_waitcnt vmcnt(%4) ; %0 %1 %2 %3" : "+v"(a), "+v"(b), "+v"(c), "+v"(d) : "n"(N))
#define MDCN_LGKMWAIT4(N, a, b, c, d) \
  asm volatile("s_waitcnt lgkmcnt(%4) ; %0 %1 %2 %3" : "+v"(a), "+v"(b), "+v"(c), "+v"(d) : "n"(N))
#define MDCN_LGKMWAIT3(N, a, b, c) \
  asm volatile("s_waitcnt lgkmcnt(%3) ; %0 %1 %2" : "+v"(a), "+v"(b), "+v"(c) : "n"(N))
typedef __attribute__((address_space(3))) u32x4 *lds_u32x4_ptr;
// Marks code that only waves of one role execute (a comment in the assembly, no instruction): the
// build's scan of the assembly drops paths that would pass markers of two roles (asm_check.py).
#define MDCN_ROLE(name) asm volatile("; mdcn-role " name)

// Blend of one 16-byte chunk (8 channels) from the same chunk at the four
// corners.  The table keeps the four mask-scaled bilinear weights as two words of
// E pairs, (w00, w01) and (w10, w11); prep() turns them into what run() needs,
// once per step.
template <typename E>
struct Blend2;

// bf16 on the matrix pipe: one v_mfma_f32_4x4x4 (16 blocks of 4x4x4) takes the four
// lanes that serve one pixel as one block, a lane's 4 channels (two words) as a
// column of B and (corner weight) x identity as A -- lane q of the block holds row
// q: the weight at K position q, zeros elsewhere -- so four instructions, one per
// corner, accumulate the bilinear sum of 4 channels in fp32 without unpacking the
// 16-bit values on the vector ALU.
template <>
struct Blend2<bf16_t> {
  struct Wt { u32x2 a[4]; };
  static __device__ __forceinline__ Wt prep(const uint2 &tw, int q) {
    const uint32_t sh = (uint32_t)(q & 1) * 16u;
    const uint32_t m0 = q < 2 ? 0xffffffffu : 0u, m1 = ~m0;
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
  static __device__ __forceinline__ f32x4 mma4(const u32x2 &a, const u32x2 &b, const f32x4 &c) {
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    return __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(s16x4, a), __builtin_bit_cast(s16x4, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ u32x4 run(const u32x4 (&v)[4], const Wt &w) {
    f32x4 d0 = {0.f, 0.f, 0.f, 0.f}, d1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const u32x2 b0 = {v[c].x, v[c].y}, b1 = {v[c].z, v[c].w};
      d0 = mma4(w.a[c], b0, d0);
      d1 = mma4(w.a[c], b1, d1);
    }
    u32x4 o;
    o.x = ElemTraits<bf16_t>::pack2(d0[0], d0[1]);
    o.y = ElemTraits<bf16_t>::pack2(d0[2], d0[3]);
    o.z = ElemTraits<bf16_t>::pack2(d1[0], d1[1]);
    o.w = ElemTraits<bf16_t>::pack2(d1[2], d1[3]);
    return o;
  }
};

// fp16 has packed arithmetic: every corner weight in both halves of a word, one
// v_pk_mul_f16 and three v_pk_fma_f16 per two channels (the blend then rounds to
// fp16 after every corner instead of once).
template <>
struct Blend2<f16_t> {
  struct Wt { uint4 w; };
  static __device__ __forceinline__ Wt prep(const uint2 &tw, int) {
    Wt w;
    w.w.x = (tw.x & 0xffffu) | (tw.x << 16);
    w.w.y = (tw.x >> 16) | (tw.x & 0xffff0000u);
    w.w.z = (tw.y & 0xffffu) | (tw.y << 16);
    w.w.w = (tw.y >> 16) | (tw.y & 0xffff0000u);
    return w;
  }
  static __device__ __forceinline__ u32x4 run(const u32x4 (&v)[4], const Wt &w) {
    const uint4 r = ElemTraits<f16_t>::blend(__builtin_bit_cast(uint4, v[0]), __builtin_bit_cast(uint4, v[1]),
                                             __builtin_bit_cast(uint4, v[2]), __builtin_bit_cast(uint4, v[3]), w.w);
    return __builtin_bit_cast(u32x4, r);
  }
};

template <typename E, int CT, bool UNBORDERED>
__global__ __launch_bounds__(kF2Threads) void fused2_kernel(FusedArgs a) {
  using TR = ElemTraits<E>;
  using BL = Blend2<E>;
  static_assert(sizeof(E) == 2, "16-bit element types");
  static_assert(CT == 256 || CT == 128, "a wave owns 64 pixels x CT / 4 channels");
  constexpr int PT = kPT;
  constexpr int KC = TR::KC;
  constexpr int TMAX = kF2Taps;
  constexpr int TBL = PT * TMAX;               // entries of one table
  constexpr int TPT = (TMAX + 3) / 4;          // table entries per lane and build
  constexpr int NB = 2, MB = CT / 128;         // 32 x 32 accumulator blocks per wave: pixels x channels
  constexpr int WCH = CT / 4;                  // output channels per wave
  constexpr int kF2WD = CT / 64;               // 1 KiB weight copies per wave and K step
  // vector-memory operations younger than the last load of a gather group (half a
  // set) when that group is blended: the rest of its set, the copies and loads of
  // the steps issued since, the copies of the current step, the refills issued so far
  constexpr int kF2VmBlend = (kF2GL - 4) + (kF2Sets - 1) * (kF2WD + kF2GL) + kF2WD;
  // ... younger than the weight copies that must have landed at a step's barrier
  constexpr int kF2VmBar = 2 * kF2GL + kF2WD;
  static_assert(kF2VmBlend < 64 && kF2VmBar < 64, "vmcnt holds 6 bits");
  constexpr uint32_t kXTile = PT * kRowB, kWTile = CT * kRowB;

  __shared__ uint4 Xs[2][PT * kRowChunks];               // sample tiles
  __shared__ uint4 Ws[kF2Slots][CT * kRowChunks];        // weight tiles
  __shared__ uint32_t tpix[2][TBL];                      // (pixel, tap) tables, [tap][PT]: corner byte offset
  __shared__ uint2 tws[2][TBL];                          // ... and the blend weights
  __shared__ uint32_t part_arrived;                      // parts of a cut tile that were there before this one

  const Geom &g = a.g;
  const int taps = g.taps;
  const int nk = a.slabs * taps;
  const int nk_pad = (nk + kF2Unroll - 1) / kF2Unroll * kF2Unroll;
  const int plane_out = g.Ho * g.Wo;
  const int total_px = (int)a.total_px;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // waves 4..7 run the produce half of a step after its barrier (see above)
  const bool late = wave >= 4;

  const uint32_t lds_x = (uint32_t)(uintptr_t)(lptr_t)(&Xs[0][0]);
  const uint32_t lds_w = (uint32_t)(uintptr_t)(lptr_t)(&Ws[0][0]);

  // ---- produce role: lane serves 16-byte chunk ck of pixels pl and pl + 8, so that
  // one load instruction of the wave reads whole 128-byte rows of 8 pixels (half as
  // many cache lines per instruction as half rows of 16 pixels, which the vector
  // cache serves measurably faster)
  const int q = lane & 3;            // row of the lane in its block of four (the matrix-pipe blend)
  const int ck = lane & 7;
  const int pl = wave * 16 + (lane >> 3);
  const uint32_t xw0 = lds_x + (uint32_t)tile_chunk(pl, ck) * 16u;       // where the two chunks go in X[0]
  const uint32_t xw1 = lds_x + (uint32_t)tile_chunk(pl + 8, ck) * 16u;
  const unsigned char *xt = (const unsigned char *)a.xt;
  const uint32_t pxb = UNBORDERED ? a.px_bytes : (uint32_t)kRowB;

  // ---- consume role: 64 pixels x 64 channels
  const int wave_p = wave & 1, wave_c = wave >> 1;
  const int frow = lane & 31, fhalf = lane >> 5;
  const uint32_t xa0 = (uint32_t)tile_chunk(wave_p * 64 + frow, fhalf) * 16u;   // K sub-step s: ^ (s << 5)
  const uint32_t wa0 = (uint32_t)tile_chunk(wave_c * WCH + frow, fhalf) * 16u;

  // weight copies: a wave copies kF2WD consecutive 1 KiB blocks (8 rows each) of
  // the tile; lane i of a copy writes chunk i of the block and reads the source
  // chunk the swizzle assigns to it.  The swizzle looks at bits 1..3 of the row:
  // bits 1, 2 come from the lane, bit 3 is the block's parity, which flips bit 1
  // of the chunk number, i.e. bit 5 of the byte offset, for the odd blocks.
  const uint32_t wlane = (uint32_t)(wave * kF2WD) * 1024u +
                         (uint32_t)((lane >> 3) * kRowB + (((lane & 7) ^ swz(lane >> 3)) * 16));

  // XCD-aware persistent schedule (as in fused_kernel): XCD x owns a contiguous run
  // of tiles and hands them out round robin to its `stride` workgroups.  The run
  // rarely is a multiple of `stride`: the last round has r < stride tiles, and
  // without further ado r workgroups would compute a whole tile while the others
  // wait.  Instead each of those r tiles is cut along K into f = stride / r parts
  // (whole rounds of kF2Unroll steps, at most a.cut_max parts), one part per
  // workgroup: a "unit" is a tile together with a range of K steps, every
  // workgroup walks whole tiles first and at most one part last.  The parts of a
  // tile meet in memory (see the epilogue).
  const int total_tiles = a.n_ptiles * a.n_ctiles * g.G;
  const int xcd = (int)(blockIdx.x & 7);
  const int stride = (int)(gridDim.x >> 3);
  const int chunk = (total_tiles + 7) >> 3;
  const int wg = (int)(blockIdx.x >> 3);
  const int first = xcd * chunk + wg;
  const int tile_end = min((xcd + 1) * chunk, total_tiles);
  const int chunk_x = max(tile_end - xcd * chunk, 0);
  const int full_rounds = chunk_x / stride;
  const int rest = chunk_x - full_rounds * stride;       // tiles of the last, partial round
  int parts = 1;
  if (a.cut_max > 1 && rest > 0) parts = min(min(stride / rest, a.cut_max), nk_pad / kF2Unroll);
  const bool cut = parts > 1;
  const int T_full = full_rounds + ((!cut && wg < rest) ? 1 : 0);
  const bool has_part = cut && wg < rest * parts;
  const int T = T_full + (has_part ? 1 : 0);
  if (T == 0) return;
  // this workgroup's part: tile, index among the tile's parts, K range
  const int part_tile = xcd * chunk + full_rounds * stride + wg / parts;
  const int part_idx = wg - (wg / parts) * parts;
  const int part_kb = (part_idx * (nk_pad / kF2Unroll) / parts) * kF2Unroll;
  const int part_pad = ((part_idx + 1) * (nk_pad / kF2Unroll) / parts) * kF2Unroll - part_kb;
  const int part_n = min(nk - part_kb, part_pad);
  // unit t: first step, number of steps, padded number of steps (macros rather than closures: closures that
  // capture closures keep their captures in memory)
#define MDCN_F2_IS_PART(t) (has_part && (t) == T_full)
#define MDCN_F2_UNIT_KB(t) (MDCN_F2_IS_PART(t) ? part_kb : 0)
#define MDCN_F2_UNIT_N(t) (MDCN_F2_IS_PART(t) ? part_n : nk)
#define MDCN_F2_UNIT_PAD(t) (MDCN_F2_IS_PART(t) ? part_pad : nk_pad)

  auto decode = [&](int t, int &ctile, int &grp, int &p0) __attribute__((always_inline)) {
    int L = MDCN_F2_IS_PART(t) ? part_tile : first + t * stride;
    ctile = L % a.n_ctiles;
    L /= a.n_ctiles;
    grp = L % g.G;
    p0 = a.px0 + (L / g.G) * PT;
  };
  auto weights_of = [&](int t) __attribute__((always_inline)) {
    int ctile, grp, p0;
    decode(t, ctile, grp, p0);
    return (const unsigned char *)a.wp + ((size_t)(grp * a.n_ctiles + ctile) * nk + MDCN_F2_UNIT_KB(t)) * (size_t)kWTile;
  };
  auto slab0_of = [&](int t) __attribute__((always_inline)) {
    int ctile, grp, p0;
    decode(t, ctile, grp, p0);
    return grp * g.cin_g / KC;
  };

  // ---- (pixel, tap) table of tile t into buffer t % 2: lane serves pixel tid % 128, taps tid / 128 + 4 i
  auto build_table = [&](int t) {
    // (opaque to the optimiser: the per-tap address arithmetic below would otherwise
    // be computed once per kernel and kept in -- spilled -- registers across the K loop)
    int tapq = tid >> 7;
    asm volatile("" : "+v"(tapq));
    int ctile, grp, p0;
    decode(t, ctile, grp, p0);
    const int tb_pl = tid & (PT - 1);
    const int tb_p = p0 + tb_pl;
    const bool tb_valid = tb_p < total_px;
    int tb_n = 0, tb_ho = 0, tb_wo = 0, tb_rem = 0;
    if (tb_valid) {
      tb_n = tb_p / plane_out;
      tb_rem = tb_p - tb_n * plane_out;
      tb_ho = tb_rem / g.Wo;
      tb_wo = tb_rem - tb_ho * g.Wo;
    }
    const E *off = (const E *)a.om.off + (long)tb_n * a.om.off_n + (long)tb_rem * a.om.off_px;
    const E *msk = (const E *)a.om.msk + (long)tb_n * a.om.msk_n + (long)tb_rem * a.om.msk_px;
    E rdy[TPT], rdx[TPT], rm[TPT];
#pragma unroll
    for (int i = 0; i < TPT; ++i) {
      const int tap = min(tapq + 4 * i, taps - 1);
      rdy[i] = off[(long)(2 * tap) * a.om.off_ch];
      rdx[i] = off[(long)(2 * tap + 1) * a.om.off_ch];
      rm[i] = msk[(long)tap * a.om.msk_ch];
    }
    uint32_t *tp = tpix[t & 1];
    uint2 *tw2 = tws[t & 1];
#pragma unroll
    for (int i = 0; i < TPT; ++i) {
      const int tap = tapq + 4 * i;
      if (tap < taps) {
        const int ti = tap / g.kw, tj = tap - ti * g.kw;
        TapSample sm = make_tap_sample(tb_ho * g.sh - g.ph + ti * g.dh, tb_wo * g.sw - g.pw + tj * g.dw,
                                       to_f32(rdy[i]), to_f32(rdx[i]), mask_value<E>(rm[i], a.om.logit), g.H, g.W);
        const uint32_t pix = tb_valid ? (uint32_t)tb_n * a.img_bytes + corner_offset<UNBORDERED>(sm, g, a) : 0u;
        uint2 w2 = make_uint2(TR::pack2(sm.w00, sm.w01), TR::pack2(sm.w10, sm.w11));
        if (!tb_valid) w2 = make_uint2(0u, 0u);
        tp[tap * PT + tb_pl] = pix;
        tw2[tap * PT + tb_pl] = w2;
      }
    }
    // Retire the loads above with a wait the compiler can see.  Those of taps past
    // the last one are never read; the compiler would otherwise keep their
    // registers marked as pending and guard every later write to them -- the
    // assembly loads of the K loop -- with a full wait.
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0), other counters untouched
  };

  // ---- the three cursors of the produce side.  Each walks steps 0 .. nk_pad - 1
  // of tile 0, 1, ...; steps nk .. nk_pad - 1 repeat the last real step (loads
  // nobody uses, which keep the wait counts constant).  Past the last tile the
  // gather and weight cursors stay where they are.
  // (a unit that is a part starts in the middle of the K range)
  int g_t = 0, g_s = 0, g_slab = MDCN_F2_UNIT_KB(0) / taps, g_tap = MDCN_F2_UNIT_KB(0) - g_slab * taps, g_slab0 = slab0_of(0);  // gather
  int g_n = MDCN_F2_UNIT_N(0), g_pad = MDCN_F2_UNIT_PAD(0);
  int b_t = 0, b_s = 0, b_tap = g_tap, b_n = g_n, b_pad = g_pad;       // blend
  int w_t = 0, w_s = 0, w_n = g_n, w_pad = g_pad;                      // weight copies
  const unsigned char *w_ptr = weights_of(0);

  // gather registers: sets x two halves of the 128-byte row x four corners
  u32x4 gs[kF2Sets][2][4];

  uint32_t o_px[2];  // top-left corner of the lane's two pixels
  auto next_addresses = [&]() {
    const uint32_t *tp_ = &tpix[g_t & 1][g_tap * PT + pl];
    const uint32_t add_ = (uint32_t)(g_slab0 + g_slab) * a.slab_bytes + (uint32_t)ck * 16u;
    o_px[0] = tp_[0] + add_;
    o_px[1] = tp_[8] + add_;
    ++g_s;
    if (g_s < g_n) {
      if (++g_tap == taps) {
        g_tap = 0;
        ++g_slab;
      }
    } else if (g_s == g_pad) {
      if (g_t + 1 < T) {
        ++g_t;
        g_s = 0;
        g_slab = MDCN_F2_UNIT_KB(g_t) / taps;
        g_tap = MDCN_F2_UNIT_KB(g_t) - g_slab * taps;
        g_n = MDCN_F2_UNIT_N(g_t);
        g_pad = MDCN_F2_UNIT_PAD(g_t);
        g_slab0 = slab0_of(g_t);
      } else {
        g_s = g_pad - 1;
      }
    }
  };
#define MDCN_F2_GATHER_HALF(S, H)                     \
  do {                                                \
    const uint32_t tl_ = o_px[H];                     \
    const uint32_t tr_ = tl_ + pxb;                   \
    const uint32_t bl_ = tl_ + a.row_bytes;           \
    const uint32_t br_ = bl_ + pxb;                   \
    MDCN_GLOAD(S[H][0], tl_, xt, 0);                  \
    MDCN_GLOAD(S[H][1], tr_, xt, 0);                  \
    MDCN_GLOAD(S[H][2], bl_, xt, 0);                  \
    MDCN_GLOAD(S[H][3], br_, xt, 0);                  \
  } while (0)
#define MDCN_F2_GATHER(SI)                            \
  do {                                                \
    next_addresses();                                 \
    MDCN_F2_GATHER_HALF(gs[SI], 0);                   \
    MDCN_F2_GATHER_HALF(gs[SI], 1);                   \
  } while (0)

  int islot = 0;  // ring slot of the next weight tile to issue
  auto issue_weights = [&](bool advance) {
    const int kk = min(w_s, w_n - 1);
    const uint32_t voff = (uint32_t)kk * kWTile + wlane;
    const uint32_t voff_odd = voff ^ 32u;
    const uint32_t dst = lds_w + (uint32_t)islot * kWTile + (uint32_t)(wave * kF2WD) * 1024u;
    {
      // (the instruction's offset moves the LDS side along with the global one; the five idle slots
      // cover a reload of the spilled base pointer right in front of the statement)
      if constexpr (kF2WD == 4)
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 4\n\t"
                     "global_load_lds_dwordx4 %1, %3\n\t"
                     "global_load_lds_dwordx4 %2, %3 offset:1024\n\t"
                     "global_load_lds_dwordx4 %1, %3 offset:2048\n\t"
                     "global_load_lds_dwordx4 %2, %3 offset:3072"
                     :
                     : "s"(dst), "v"(voff), "v"(voff_odd), "s"(w_ptr)
                     : "memory");
      else
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 4\n\t"
                     "global_load_lds_dwordx4 %1, %3\n\t"
                     "global_load_lds_dwordx4 %2, %3 offset:1024"
                     :
                     : "s"(dst), "v"(voff), "v"(voff_odd), "s"(w_ptr)
                     : "memory");
    }
    if (!advance) return;
    islot = (islot == kF2Slots - 1) ? 0 : islot + 1;
    if (++w_s == w_pad) {
      if (w_t + 1 < T) {
        ++w_t;
        w_s = 0;
        w_n = MDCN_F2_UNIT_N(w_t);
        w_pad = MDCN_F2_UNIT_PAD(w_t);
        w_ptr = weights_of(w_t);
      } else {
        w_s = w_pad - 1;
      }
    }
  };
  static_assert(kF2WD == 4 || kF2WD == 2, "issue_weights spells out the copies");

  // The blend weights of the blend cursor's step for the lane's two pixels are read from the
  // table ahead of the block that needs them -- right behind the last MFMA of the MFMA phase in
  // front of it, which for the late waves is a barrier away -- so that the block does not start
  // with an LDS round trip (256-channel tiles: 1.5 % off the kernel; with 128-channel tiles, whose
  // MFMA phase is half as long, it costs as much and is left out).
  constexpr bool kF2TwAhead = CT == 256;
  u32x2 tw_pf[2];
  const uint32_t lds_tw = (uint32_t)(uintptr_t)(lptr_t)(&tws[0][0]) + (uint32_t)pl * 8u;
  auto prefetch_tw = [&]() {
    if constexpr (!kF2TwAhead) return;
    const uint32_t a_ = lds_tw + (uint32_t)(((b_t & 1) ? TBL : 0) + b_tap * PT) * 8u;
    asm volatile("ds_read_b64 %0, %1" : "=v"(tw_pf[0]) : "v"(a_));
    asm volatile("ds_read_b64 %0, %1 offset:64" : "=v"(tw_pf[1]) : "v"(a_));
  };

  // One produce block: the weight copies of the step after the blend cursor's,
  // the blend of the cursor's step (gather set SI) into its sample tile, the
  // gather of kF2Sets steps ahead into the set.
#define MDCN_F2_BLOCK(SI)                                                               \
  do {                                                                                  \
    if constexpr (kF2TwAhead)                                                           \
      asm volatile("s_waitcnt lgkmcnt(0) ; %0 %1" : "+v"(tw_pf[0]), "+v"(tw_pf[1]));    \
    if (b_t < T) {                                                                      \
      issue_weights(true);                                                              \
      next_addresses();                                                                 \
      uint2 tw0_, tw1_;                                                                 \
      if constexpr (kF2TwAhead) {                                                       \
        tw0_ = make_uint2(tw_pf[0].x, tw_pf[0].y);                                      \
        tw1_ = make_uint2(tw_pf[1].x, tw_pf[1].y);                                      \
      } else {                                                                          \
        const uint2 *tw_ = &tws[b_t & 1][b_tap * PT + pl];                              \
        tw0_ = tw_[0];                                                                  \
        tw1_ = tw_[8];                                                                  \
      }                                                                                 \
      const uint32_t xo_ = (b_s & 1) ? kXTile : 0u;                                     \
      {                                                                                 \
        const typename BL::Wt w_ = BL::prep(tw0_, q);                                   \
        MDCN_VMWAIT4(kF2VmBlend, gs[SI][0][0], gs[SI][0][1], gs[SI][0][2], gs[SI][0][3]); \
        const u32x4 o_ = BL::run(gs[SI][0], w_);                                        \
        *(lds_u32x4_ptr)(uintptr_t)(xw0 + xo_) = o_;                                    \
      }                                                                                 \
      MDCN_F2_GATHER_HALF(gs[SI], 0);                                                   \
      {                                                                                 \
        const typename BL::Wt w_ = BL::prep(tw1_, q);                                   \
        MDCN_VMWAIT4(kF2VmBlend, gs[SI][1][0], gs[SI][1][1], gs[SI][1][2], gs[SI][1][3]); \
        const u32x4 o_ = BL::run(gs[SI][1], w_);                                        \
        *(lds_u32x4_ptr)(uintptr_t)(xw1 + xo_) = o_;                                    \
      }                                                                                 \
      MDCN_F2_GATHER_HALF(gs[SI], 1);                                                   \
      ++b_s;                                                                            \
      if (b_s < b_n) {                                                                  \
        if (++b_tap == taps) b_tap = 0;                                                 \
      } else if (b_s == b_pad) {                                                        \
        ++b_t;                                                                          \
        b_s = 0;                                                                        \
        b_tap = MDCN_F2_UNIT_KB(b_t) % taps;                                                    \
        b_n = MDCN_F2_UNIT_N(b_t);                                                              \
        b_pad = MDCN_F2_UNIT_PAD(b_t);                                                          \
      }                                                                                 \
    }                                                                                   \
  } while (0)

  f32x16 acc[NB][MB];
  int rslot = 0;  // ring slot of the weight tile the next MFMA step reads
  int c_n = 0;  // steps of the unit the consume side is in
  auto mfma_step = [&](int k) {
    const uint32_t xb = lds_x + ((k & 1) ? kXTile : 0u) + xa0;
    const uint32_t wb = lds_w + (uint32_t)rslot * kWTile + wa0;
    rslot = (rslot == kF2Slots - 1) ? 0 : rslot + 1;
    if (k >= c_n) return;
    // The two waves of a SIMD are in opposite phases most of the time.  The MFMA phase is a
    // stream of long instructions that keeps the matrix pipe busy whenever it gets an issue
    // slot; the produce block is a chain of short dependent steps (table read, wait, blend,
    // sample write, gather issue) whose delay moves the step barrier.  So the arbiter is told
    // to prefer the wave that produces: priority 0 here, 2 from the end of this phase on
    // (measured: 3 % off the kernel; the opposite preference costs 1 %).
    __builtin_amdgcn_s_setprio(0);
    u32x4 xf[4][NB], wf[4][MB];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const uint32_t xk = xb ^ (uint32_t)(s << 5), wk = wb ^ (uint32_t)(s << 5);
      MDCN_DSREAD(xf[s][0], xk, 0); MDCN_DSREAD(xf[s][1], xk, 4096);
      MDCN_DSREAD(wf[s][0], wk, 0);
      if constexpr (MB == 2) MDCN_DSREAD(wf[s][1], wk, 4096);
    }
    constexpr int kRd = 2 + MB;  // fragment reads per K sub-step
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      if constexpr (MB == 2) {
        if (s < 3) MDCN_LGKMWAIT4(kRd, xf[s][0], xf[s][1], wf[s][0], wf[s][1]);
        else MDCN_LGKMWAIT4(0, xf[s][0], xf[s][1], wf[s][0], wf[s][1]);
      } else {
        if (s < 3) MDCN_LGKMWAIT3(kRd, xf[s][0], xf[s][1], wf[s][0]);
        else MDCN_LGKMWAIT3(0, xf[s][0], xf[s][1], wf[s][0]);
      }
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
          TR::mma(acc[nb][mb], __builtin_bit_cast(uint4, xf[s][nb]), __builtin_bit_cast(uint4, wf[s][mb]));
      if (s + 2 < 4) {
        const uint32_t xk = xb ^ (uint32_t)((s + 2) << 5), wk = wb ^ (uint32_t)((s + 2) << 5);
        MDCN_DSREAD(xf[s + 2][0], xk, 0); MDCN_DSREAD(xf[s + 2][1], xk, 4096);
        MDCN_DSREAD(wf[s + 2][0], wk, 0);
        if constexpr (MB == 2) MDCN_DSREAD(wf[s + 2][1], wk, 4096);
      }
    }
    __builtin_amdgcn_s_setprio(2);
  };


  // ---- start of the stream: first table, first gathers.  A wave keeps step j of
  // the stream in set j % kF2Sets; the late waves, which run one block ahead, in set
  // (j - 1) % kF2Sets, so that both kinds use the same set at the same place of the K
  // loop.  The issue order gather, copies, gather (..., copies, gather with three
  // sets) is the K loop's, which keeps the counts of the waits valid from the first
  // block on (with three sets the second group of copies is issued again by the
  // first block: same data, same slot).
  // bias of this lane's output channels, fetched together with a tile's table (the
  // wait that ends the table's loads covers it, so the epilogue never waits on memory)
  float bv[MB], bv_next[MB];
  auto load_bias = [&](int t, float (&b)[MB]) {
    int ctile, grp, p0;
    decode(t, ctile, grp, p0);
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      const int col = ctile * CT + wave_c * WCH + mb * 32 + frow;
      b[mb] = (a.bias && col < g.cout_g) ? to_f32(((const E *)a.bias)[(long)grp * g.cout_g + col]) : 0.0f;
    }
  };
  load_bias(0, bv);
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) bv_next[mb] = 0.0f;
  build_table(0);
  MDCN_BARRIER_LDS();  // table visible
  __builtin_amdgcn_sched_barrier(0);
  if constexpr (kF2Sets == 3) {
    if (!late) {
      MDCN_ROLE("early");
      MDCN_F2_GATHER(0);
      issue_weights(true);
      MDCN_F2_GATHER(1);
      issue_weights(false);
      MDCN_F2_GATHER(2 % kF2Sets);
      prefetch_tw();
      MDCN_F2_BLOCK(0);
    } else {
      MDCN_ROLE("late");
      MDCN_F2_GATHER(2 % kF2Sets);
      issue_weights(true);
      MDCN_F2_GATHER(0);
      issue_weights(false);
      MDCN_F2_GATHER(1);
      prefetch_tw();
      MDCN_F2_BLOCK(2 % kF2Sets);
      prefetch_tw();
      MDCN_F2_BLOCK(0);
    }
  } else {
    // two sets: step j in set j % 2 (late waves: (j + 1) % 2)
    if (!late) {
      MDCN_ROLE("early");
      MDCN_F2_GATHER(0);
      issue_weights(true);
      MDCN_F2_GATHER(1);
      prefetch_tw();
      MDCN_F2_BLOCK(0);
    } else {
      MDCN_ROLE("late");
      MDCN_F2_GATHER(1);
      issue_weights(true);
      MDCN_F2_GATHER(0);
      prefetch_tw();
      MDCN_F2_BLOCK(1);
      prefetch_tw();
      MDCN_F2_BLOCK(0);
    }
  }
  static_assert(kF2Sets == 3 || kF2Sets == 2, "the prologue spells out the sets");
  MDCN_BARRIER(kF2VmBar);  // X[0] and W[0] complete
  __builtin_amdgcn_sched_barrier(0);

  // ---- K loop of a tile: kF2Unroll steps per round; step k runs the produce
  // block one (late waves: two) steps ahead on set (k + 1) % kF2Sets
#define MDCN_F2_STEP(K, SI)                                   \
  do {                                                        \
    mfma_step(K);                                             \
    prefetch_tw();                                            \
    __builtin_amdgcn_sched_barrier(0);                        \
    if (late) {                                               \
      MDCN_ROLE("late");                                      \
      MDCN_BARRIER(kF2VmBar);                                 \
    }                                                         \
    __builtin_amdgcn_sched_barrier(0);                        \
    MDCN_F2_BLOCK(SI);                                        \
    __builtin_amdgcn_sched_barrier(0);                        \
    if (!late) {                                              \
      MDCN_ROLE("early");                                     \
      MDCN_BARRIER(kF2VmBar);                                 \
    }                                                         \
    __builtin_amdgcn_sched_barrier(0);                        \
  } while (0)

  for (int t = 0; t < T; ++t) {
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[nb][mb][r] = 0.0f;

    c_n = MDCN_F2_UNIT_N(t);
    const int c_pad = MDCN_F2_UNIT_PAD(t);
    for (int k = 0; k < c_pad; k += kF2Unroll) {
      if (k == kF2Unroll && t + 1 < T) {
        // the next tile's table: its buffer was last read in the previous tile, its
        // first reader is the gather cursor near the end of this one
        load_bias(t + 1, bv_next);
        build_table(t + 1);
        __builtin_amdgcn_sched_barrier(0);
      }
      MDCN_F2_STEP(k + 0, 1 % kF2Sets);
      MDCN_F2_STEP(k + 1, 2 % kF2Sets);
      MDCN_F2_STEP(k + 2, 3 % kF2Sets);
      MDCN_F2_STEP(k + 3, 4 % kF2Sets);
      MDCN_F2_STEP(k + 4, 5 % kF2Sets);
      MDCN_F2_STEP(k + 5, 6 % kF2Sets);
    }

    // ---- a part of a tile: the parts meet in memory.  Every part stores its
    // accumulators (fp32, register order) and counts itself in; the part that
    // arrives last adds all of them up in index order -- so the sum does not
    // depend on who was last -- and goes on to the epilogue; the others are done.
    // Nobody waits for anybody.  The last part also resets the counter, which is
    // thereby zero again for the next launch.  The partial sums are written and
    // read with device-coherent stores and loads (sc1), which go past the caches
    // that are private to a CU or an XCD, so no cache has to be written back or
    // invalidated as a whole; a wave's stores have completed (wait on the
    // vector-memory counter) before its workgroup counts itself in.
    bool store_tile = true;
    if (MDCN_F2_IS_PART(t)) {
      // First of all nothing is in flight any more: the gathers the cursors issued past the last step
      // have landed, and every gather register counts as read here, so none of them is handed to another
      // value while a load may still write it.
#pragma unroll
      for (int si = 0; si < kF2Sets; ++si)
#pragma unroll
        for (int h = 0; h < 2; ++h) MDCN_VMWAIT4(0, gs[si][h][0], gs[si][h][1], gs[si][h][2], gs[si][h][3]);
      const int tslot = xcd * stride + wg / parts;                       // the tile's counter
      const unsigned char *pbase =
          (const unsigned char *)a.cut_part + (size_t)(xcd * stride + (wg / parts) * parts) * (size_t)(PT * CT * 4);
      const unsigned char *mine = uniform_ptr(pbase + (size_t)part_idx * (size_t)(PT * CT * 4));
      // a lane's 64 values travel as 16 quads of 16 bytes; quad j of the wave's lanes is one 1 KiB run.
      // (The offset is opaque to the optimiser, which would otherwise form the addresses below once,
      // ahead of the tile loop, and keep them -- spilled -- across the K loop.)
      constexpr int NQ = NB * MB * 4;   // quads per lane
      uint32_t voff = (uint32_t)((wave * NQ * 64 + lane) * 16);
      asm volatile("" : "+v"(voff));
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
          for (int qd = 0; qd < 4; ++qd) {
            const f32x16 &c = acc[nb][mb];
            const f32x4 v = {c[4 * qd], c[4 * qd + 1], c[4 * qd + 2], c[4 * qd + 3]};
            const uint32_t vo = voff + (uint32_t)(((nb * MB + mb) * 4 + qd) * 1024);
            // (s_nop: the compiler may have written the base's scalar registers with a vector instruction --
            // a reload of spilled scalars -- right in front of this statement, and a vector-memory
            // instruction must not read such a register within the next five issue slots; the compiler
            // keeps that distance for its own instructions but does not look into assembly text)
            asm volatile("s_nop 4\n\tglobal_store_dwordx4 %0, %1, %2 sc1" : : "v"(vo), "v"(v), "s"(mine) : "memory");
          }
      // this wave's stores -- and whatever gathers and weight copies it still had in flight -- are done
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      if (tid == 0)
        part_arrived = __hip_atomic_fetch_add((uint32_t *)a.cut_cnt + tslot, 1u, __ATOMIC_RELAXED,
                                              __HIP_MEMORY_SCOPE_AGENT);
      __syncthreads();
      store_tile = part_arrived == (uint32_t)(parts - 1);
      if (store_tile) {
        // the gather registers are free now (nothing is in flight): sets 0 and 1 take the 16 quads of a part
        // (two parts: a + b is the same in either order, so the last one adds the other's values to
        // the ones it still holds; more parts: everything from memory, in index order)
        const bool two = parts == 2;
        const unsigned char *src0 = two ? pbase + (size_t)(1 - part_idx) * (size_t)(PT * CT * 4) : pbase;
        for (int i = two ? 1 : 0; i < parts; ++i) {
          const unsigned char *src = uniform_ptr(src0);
#pragma unroll
          for (int j = 0; j < NQ; ++j) {
            const uint32_t vo = voff + (uint32_t)(j * 1024);
            asm volatile("s_nop 4\n\tglobal_load_dwordx4 %0, %1, %2 sc1"
                         : "=v"(gs[j >> 3][(j >> 2) & 1][j & 3])
                         : "v"(vo), "s"(src));
          }
          MDCN_VMWAIT4(0, gs[0][0][0], gs[0][0][1], gs[0][0][2], gs[0][0][3]);
          MDCN_VMWAIT4(0, gs[0][1][0], gs[0][1][1], gs[0][1][2], gs[0][1][3]);
          if constexpr (NQ > 8) {
            MDCN_VMWAIT4(0, gs[1][0][0], gs[1][0][1], gs[1][0][2], gs[1][0][3]);
            MDCN_VMWAIT4(0, gs[1][1][0], gs[1][1][1], gs[1][1][2], gs[1][1][3]);
          }
#pragma unroll
          for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
              for (int qd = 0; qd < 4; ++qd) {
                const int j = (nb * MB + mb) * 4 + qd;
                const f32x4 v = __builtin_bit_cast(f32x4, gs[j >> 3][(j >> 2) & 1][j & 3]);
#pragma unroll
                for (int e = 0; e < 4; ++e)
                  acc[nb][mb][4 * qd + e] = i == 0 ? v[e] : acc[nb][mb][4 * qd + e] + v[e];
              }
          src0 += PT * CT * 4;
        }
        if (tid == 0)
          __hip_atomic_store((uint32_t *)a.cut_cnt + tslot, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }

    // ---- epilogue: bias, one rounding, NCHW store straight from the accumulators.
    // Accumulator block (A = samples, B = weights): register r of lane l holds
    //   pixel = (r/4)*8 + (l/32)*4 + r%4,  channel = l%32.
    // The two halves of the wave exchange packed pixel pairs, after which a lane
    // holds 8 consecutive pixels = 16 bytes of one channel.
    if (store_tile) {
      int ctile, grp, p0;
      decode(t, ctile, grp, p0);
      E *out = (E *)a.out;
      // A run of 8 pixels of one channel is one 16-byte store wherever it lies in one image; planes that are
      // not whole 16-byte runs (25 x 42 pixels, say) make such a store start at any even or odd pixel, which
      // global memory takes (unaligned access mode).  Only runs across the end of an image go pixel by pixel.
      const int pw0 = p0 + wave_p * 64;
      // image and pixel-in-image of the wave's first pixel; the runs below step on from there
      const int n0 = pw0 / plane_out;
      const int rem0 = pw0 - n0 * plane_out;
      auto store_run = [&](long cbase, int dp, const u32x4 &val) {  // pixels pw0 + dp .. + 7 of channel cbase
        const int p = pw0 + dp;
        if (p >= total_px) return;
        int n = n0, rem = rem0 + dp;
        while (rem >= plane_out) {
          rem -= plane_out;
          ++n;
        }
        E *dst = out + ((long)n * g.Cout + cbase) * plane_out + rem;
        if (p + 8 <= total_px && rem + 8 <= plane_out) {
          __builtin_memcpy(dst, &val, 16);
        } else {
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            const uint32_t word = val[i >> 1];
            const uint16_t bits = (uint16_t)((i & 1) ? (word >> 16) : (word & 0xffffu));
            if (p + i < total_px) {
              int ni = n, ri = rem + i;
              while (ri >= plane_out) {
                ri -= plane_out;
                ++ni;
              }
              *(uint16_t *)(out + ((long)ni * g.Cout + cbase) * plane_out + ri) = bits;
            }
          }
        }
      };
      // the common case: the wave's 64 pixels lie in one image and every run is one 16-byte store
      const bool plain = pw0 + 64 <= total_px && rem0 + 64 <= plane_out;
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const int col = ctile * CT + wave_c * WCH + mb * 32 + frow;
        const bool col_ok = col < g.cout_g;
        const long cbase = (long)grp * g.cout_g + col;
        const float bvm = bv[mb];
        E *row = out + ((long)n0 * g.Cout + cbase) * plane_out + rem0 + 8 * fhalf;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          const f32x16 &c = acc[nb][mb];
#pragma unroll
          for (int g2 = 0; g2 < 2; ++g2) {
            const int ga = 2 * g2, gb = 2 * g2 + 1;
            const uint32_t a0 = TR::pack2(c[4 * ga + 0] + bvm, c[4 * ga + 1] + bvm);
            const uint32_t a1 = TR::pack2(c[4 * ga + 2] + bvm, c[4 * ga + 3] + bvm);
            const uint32_t b0 = TR::pack2(c[4 * gb + 0] + bvm, c[4 * gb + 1] + bvm);
            const uint32_t b1 = TR::pack2(c[4 * gb + 2] + bvm, c[4 * gb + 3] + bvm);
            // lower half keeps group ga and receives the upper half's part of it; upper half likewise with gb
            const auto s0 = __builtin_amdgcn_permlane32_swap(a0, b0, false, false);
            const auto s1 = __builtin_amdgcn_permlane32_swap(a1, b1, false, false);
            u32x4 val;
            val.x = s0[0]; val.y = s1[0]; val.z = s0[1]; val.w = s1[1];
            if (plain) {
              if (col_ok) __builtin_memcpy(row + nb * 32 + 16 * g2, &val, 16);
            } else if (col_ok) {
              store_run(cbase, nb * 32 + 8 * (fhalf ? gb : ga), val);
            }
          }
        }
      }
    }
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) bv[mb] = bv_next[mb];
    __builtin_amdgcn_sched_barrier(0);
  }
  // copies issued past the last step must have landed before the workgroup gives up its LDS
  MDCN_VMWAIT4(0, gs[0][0][0], gs[0][1][0], gs[1][0][0], gs[kF2Sets - 1][1][0]);
#undef MDCN_F2_STEP
#undef MDCN_F2_IS_PART
#undef MDCN_F2_UNIT_KB
#undef MDCN_F2_UNIT_N
#undef MDCN_F2_UNIT_PAD
#undef MDCN_F2_BLOCK
#undef MDCN_F2_GATHER
#undef MDCN_F2_GATHER_HALF
}

}  // namespace mdcn
