// Fused DCNv2 forward for gfx950, 16-bit tensors, tiles of 256 pixels x CT (256 or
// 128) output channels, one deformable group, 3 to 9 taps, bordered input copy
// or a channels-last tensor read in place:
// the implicit GEMM of mdcn_fused.h / mdcn_fused2.h with a tile twice as tall.
//
// Why another tile.  Per K step (128 bytes of channels of one tap) a tile of PT
// pixels x CT channels pulls 4 * PT corner rows and CT weight rows of 128 bytes
// through the compute unit's vector-memory path for PT * CT * 64 multiply-adds,
// and that path (64 bytes per clock) is what the 128-pixel kernels are bound by.
// 256 x 256 moves 160 KiB per 2 048 MFMA clocks where 128 x 256 moves 96 KiB per
// 1 024: one sixth fewer bytes per FLOP, half the weight-tile copies, a quarter
// fewer fragment reads, half the barriers.
//
// Eight wavefronts.  A wave owns 64 pixels x CT / 2 channels of the tile (128
// accumulator registers per lane for CT = 256).  Per K step every wave
//   * "produces" 32 of the tile's pixels: waits for the gather it issued one step
//     earlier (4 corners x 16 bytes of four pixels per lane: one load instruction
//     of the wave reads the whole 128-byte rows of 8 pixels), blends the corners
//     pixel by pixel into the sample tile in LDS and reissues each pixel's four
//     loads for the next step right behind its blend -- one register set, every
//     load a whole step in flight;
//   * "consumes": 8 * CT / 64 MFMAs (32x32x16), fragments read from LDS three
//     pairs of MFMAs ahead.
// The two waves of a SIMD do the halves in opposite order between two barriers:
// waves 0-3 ("early") run their MFMAs first and produce afterwards, waves 4-7
// ("late") produce first.  The late waves also issue the whole direct-to-LDS copy
// of the next step's weight tile, right behind the barrier: the ring holds two
// tiles (LDS: 2 x 32 KiB samples + 2 x 32 KiB weights + the 27 KiB table + the
// bias), so a slot is free only once every wave has passed the barrier that ends
// its step, and the early waves' MFMA phase, which comes first, is kept free of
// vector-memory instructions.  One barrier per step.
//
// The produce side streams across the tiles of a workgroup: its cursors (gather,
// blend, weight copy) walk one sequence of steps, tile after tile, two, one and
// one step ahead of the MFMAs, so the memory pipeline never drains between
// tiles.  The (pixel, tap) table exists once.  K runs slab outer, tap inner, so a
// tap's row of the table is read for the last time in the tile's last slab; from
// there on the early waves -- whose produce half is the lighter one -- rewrite
// it, one row per step, for the next tile: each of them serves its own 32 pixels
// and those of the late wave four above it, loads offsets and mask one step
// ahead and writes the row one barrier after its last reader.  A tile's output
// is stored right behind its last MFMAs; the bias comes from a copy in LDS, so
// that the K loop holds no load the compiler knows of (it would guard such a
// load's registers with waits that drain the gathers).
// A tile's K range is never cut here: the host gives this kernel whole tiles
// only (and decides how many), the rest of the pixels go to the 128-pixel kernel
// of mdcn_fused2.h.
//
// All vector-memory loads of the K loop are issued from inline assembly and
// waited for with explicit counts (see mdcn_fused2.h for why); per wave and step
// the order of issue is fixed -- late waves: WD weight copies; early waves: three
// loads for the table; then, both kinds, four groups of four gather loads -- so
// the number of younger loads at every wait is a constant.  (The stores of a
// tile's output are younger still where they occur; they only make a wait
// stricter.)
#pragma once

#include "mdcn_fused2.h"

namespace mdcn {

constexpr int kF3PT = 256;             // pixels per tile
constexpr int kF3Threads = 512;
constexpr int kF3Taps = kTapsSmall;    // table capacity (kh * kw)
constexpr int kF3MinSteps = 4;         // K steps per tile the pipeline needs (and an even number of them)
constexpr int kF3MinTaps = 3;          // a row of the table is rewritten at least two steps before its next reader
constexpr int kF3MaxBias = 2048;       // output channels whose bias the kernel keeps in LDS
constexpr size_t fused3_lds_bytes(int CT) {
  return (size_t)2 * kF3PT * kRowB + (size_t)2 * CT * kRowB + (size_t)kF3PT * kF3Taps * 12 + (size_t)kF3MaxBias * 2;
}

// four corners of one pixel: 16 bytes per lane each, from `base` / `base_row`
// (scalar pointers to the copy and to its next pixel row) + 32-bit byte offset;
// the right-hand corners are the next 128 bytes.  (s_nop: the compiler may have
// reloaded the scalar operands with a vector instruction right in front of the
// statement, and a vector-memory instruction must not read such a register within
// the next five issue slots.)
#define MDCN_F3_GLOAD4(d, voff, base, base_row)                                  \
  asm volatile("s_nop 4\n\t"                                                     \
               "global_load_dwordx4 %0, %4, %5\n\t"                              \
               "global_load_dwordx4 %1, %4, %5 offset:128\n\t"                   \
               "global_load_dwordx4 %2, %4, %6\n\t"                              \
               "global_load_dwordx4 %3, %4, %6 offset:128"                       \
               : "=&v"(d[0]), "=&v"(d[1]), "=&v"(d[2]), "=&v"(d[3])              \
               : "v"(voff), "s"(base), "s"(base_row))
// ... from a channels-last tensor read in place: the right-hand corners are a whole pixel (all channels)
// further on, at `base_r` / `base_row_r`
#define MDCN_F3_GLOAD4_NHWC(d, voff, base, base_r, base_row, base_row_r)         \
  asm volatile("s_nop 4\n\t"                                                     \
               "global_load_dwordx4 %0, %4, %5\n\t"                              \
               "global_load_dwordx4 %1, %4, %6\n\t"                              \
               "global_load_dwordx4 %2, %4, %7\n\t"                              \
               "global_load_dwordx4 %3, %4, %8"                                  \
               : "=&v"(d[0]), "=&v"(d[1]), "=&v"(d[2]), "=&v"(d[3])              \
               : "v"(voff), "s"(base), "s"(base_r), "s"(base_row), "s"(base_row_r))

// Barrier of a step for the waves that copy weight tiles: all but N of the wave's loads have landed -- the
// youngest direct-to-LDS copies among them, which the comment tells the build's scan of the assembly
// (asm_check.py) -- and its own LDS operations are done.
#define MDCN_F3_BARRIER_COPIES(N) \
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0) ; lds-copies\n\ts_barrier" ::"n"(N) : "memory")

template <int N>
__device__ __forceinline__ void f3_vmwait4(u32x4 &a, u32x4 &b, u32x4 &c, u32x4 &d) {
  asm volatile("s_waitcnt vmcnt(%4) ; %0 %1 %2 %3" : "+v"(a), "+v"(b), "+v"(c), "+v"(d) : "n"(N));
}
template <int N>
__device__ __forceinline__ void f3_lgkmwait4(u32x4 &a, u32x4 &b, u32x4 &c, u32x4 &d) {
  asm volatile("s_waitcnt lgkmcnt(%4) ; %0 %1 %2 %3" : "+v"(a), "+v"(b), "+v"(c), "+v"(d) : "n"(N));
}
template <int N>
__device__ __forceinline__ void f3_lgkmwait3(u32x4 &a, u32x4 &b, u32x4 &c) {
  asm volatile("s_waitcnt lgkmcnt(%3) ; %0 %1 %2" : "+v"(a), "+v"(b), "+v"(c) : "n"(N));
}
template <int N>
__device__ __forceinline__ void f3_lgkmwait1(u32x4 &a) {
  asm volatile("s_waitcnt lgkmcnt(%1) ; %0" : "+v"(a) : "n"(N));
}

// The whole kernel as one kind of wave runs it: the two kinds share no code path
// between the first branch and the end (a register that an asm-issued load is still
// writing must never meet another copy of itself at a join, where the compiler would
// be free to move it).
template <typename E, int CT, bool LATE, bool UNBORDERED>
__device__ __forceinline__ void fused3_role(const FusedArgs &a, const uint32_t lds_x, const uint32_t lds_w,
                                            uint32_t *tpix, uint2 *tws, E *bias_s, const int wave) {
  using TR = ElemTraits<E>;
  using BL = Blend2<E>;
  static_assert(sizeof(E) == 2, "16-bit element types");
  static_assert(CT == 256 || CT == 128, "a wave owns 64 pixels x CT / 2 channels");
  constexpr int PT = kF3PT;
  constexpr int KC = TR::KC;
  constexpr int TMAX = kF3Taps;
  constexpr int TPT = (TMAX + 1) / 2;          // table entries per lane of the first tile's build
  constexpr int NB = 2, MB = CT / 64;          // 32 x 32 accumulator blocks per wave: pixels x channels
  constexpr int WCH = CT / 2;                  // output channels per wave
  constexpr int WD = CT / 32;                  // 1 KiB weight copies per late wave and K step
  constexpr int NG = 4 * MB;                   // MFMA groups (2 MFMAs each) per K step
  constexpr int TL = LATE ? 0 : 3;             // table loads per early wave and K step
  // loads younger than those of a pixel when it is blended: the pixels behind it of the same step and the
  // ones before it of the next (12), and what the wave issues in between (weight copies / table loads)
  constexpr int kVmBlend = 12 + (LATE ? WD : TL);
  // ... younger than the weight copies (late waves) at the barrier that ends their step, and than the
  // table loads (early waves) where the step after theirs uses them: the sixteen gathers
  constexpr int kVmStep = 16;
  constexpr uint32_t kXTile = PT * kRowB, kWTile = CT * kRowB;
  static_assert(fused3_lds_bytes(CT) <= 160 * 1024, "LDS of one compute unit");

  const Geom &g = a.g;
  const int taps = g.taps;
  const int slabs = a.slabs;
  const int nk = slabs * taps;                 // even and >= kF3MinSteps (the host checks)
  const int plane_out = g.Ho * g.Wo;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  // The code that runs once per tile (epilogue) takes the thread index through this: what it derives from
  // it is then computed there, not once per kernel and kept in -- spilled -- registers across the K loop.
  auto tile_tid = [&]() __attribute__((always_inline)) {
    int v = tid;
    asm volatile("" : "+v"(v));
    return v;
  };
  // (likewise the divisors of that code: the reciprocals its divisions go through are computed on the
  // vector ALU, and hoisted out of the loop they would each hold a vector register for good)
  auto tile_s = [](int v) __attribute__((always_inline)) {
    asm volatile("" : "+s"(v));
    return v;
  };

  // ---- produce role: lane serves 16-byte chunk ck of pixels pl + 8 i, i = 0..3
  const int q = lane & 3;            // row of the lane in its block of four (the matrix-pipe blend)
  const int ck = lane & 7;
  const int pl = wave * 32 + (lane >> 3);
  // where the four chunks go in X[0] (rows 8 apart differ in bit 1 of the swizzle, rows 16 apart in none)
  const uint32_t xwa = lds_x + (uint32_t)tile_chunk(pl, ck) * 16u;
  const uint32_t xwb = lds_x + (uint32_t)tile_chunk(pl + 8, ck) * 16u;
  const unsigned char *xt = uniform_ptr((const unsigned char *)a.xt);
  const unsigned char *xt_row = uniform_ptr((const unsigned char *)a.xt + a.row_bytes);
  // (channels-last input read in place: the pixel to the right is a.px_bytes away, not 128 bytes)
  const unsigned char *xt_r = uniform_ptr((const unsigned char *)a.xt + a.px_bytes);
  const unsigned char *xt_row_r = uniform_ptr((const unsigned char *)a.xt + a.row_bytes + a.px_bytes);
  // the four loads of one pixel
#define MDCN_F3_GATHER(d, voff)                                                  \
  do {                                                                           \
    if constexpr (UNBORDERED)                                                    \
      MDCN_F3_GLOAD4_NHWC(d, voff, xt, xt_r, xt_row, xt_row_r);                  \
    else                                                                         \
      MDCN_F3_GLOAD4(d, voff, xt, xt_row);                                       \
  } while (0)

  // ---- consume role: 64 pixels x WCH channels
  const int wave_p = wave & 3, wave_c = wave >> 2;
  const int frow = lane & 31, fhalf = lane >> 5;
  const uint32_t xa0 = (uint32_t)tile_chunk(wave_p * 64 + frow, fhalf) * 16u;   // K sub-step s: ^ (s << 5)
  const uint32_t wa0 = (uint32_t)tile_chunk(wave_c * WCH + frow, fhalf) * 16u;

  // weight copies (late waves): wave 4 + j copies the WD consecutive 1 KiB blocks (8
  // rows each) from block j * WD on; lane i of a copy writes chunk i of the block and
  // reads the source chunk the swizzle assigns to it (bits 1, 2 of the row come from
  // the lane, bit 3 is the block's parity, which flips bit 1 of the chunk number, i.e.
  // bit 5 of the byte offset, for the odd blocks).
  const uint32_t wblock0 = (uint32_t)((wave & 3) * WD) * 1024u;
  const uint32_t wlane = wblock0 + (uint32_t)((lane >> 3) * kRowB + (((lane & 7) ^ swz(lane >> 3)) * 16));

  // XCD-aware persistent schedule: XCD x owns a contiguous run of tiles and hands
  // them out round robin to its workgroups.
  const int total_tiles = a.n_ptiles * a.n_ctiles * g.G;
  const int xcd = (int)(blockIdx.x & 7);
  const int stride = (int)(gridDim.x >> 3);
  const int chunk = (total_tiles + 7) >> 3;
  const int first = xcd * chunk + (int)(blockIdx.x >> 3);
  const int tile_end = min((xcd + 1) * chunk, total_tiles);
  if (first >= tile_end) return;  // (a whole workgroup: the barriers below are never short of waves)
  const int T = (tile_end - first + stride - 1) / stride;

  auto decode = [&](int t, int &ctile, int &grp, int &p0) __attribute__((always_inline)) {
    int L = first + t * stride;
    const int nct = tile_s(a.n_ctiles), ng = tile_s(g.G);
    ctile = L % nct;
    L /= nct;
    grp = L % ng;
    p0 = (L / ng) * PT;
    // (uniform, and kept in scalar registers: the divisions run on the vector ALU)
    ctile = __builtin_amdgcn_readfirstlane(ctile);
    grp = __builtin_amdgcn_readfirstlane(grp);
    p0 = __builtin_amdgcn_readfirstlane(p0);
  };
  auto slab0_of = [&](int t) __attribute__((always_inline)) {
    int ctile, grp, p0;
    decode(t, ctile, grp, p0);
    return __builtin_amdgcn_readfirstlane(grp * g.cin_g / KC);
  };
  auto weights_of = [&](int t) __attribute__((always_inline)) {
    int ctile, grp, p0;
    decode(t, ctile, grp, p0);
    return uniform_ptr((const unsigned char *)a.wp + (size_t)(grp * a.n_ctiles + ctile) * nk * (size_t)kWTile);
  };

  // One entry of the (pixel, tap) table: pixel p (of the whole launch; every pixel of this kernel's tiles
  // exists), tap, its two offsets and its mask value as stored.
  auto table_entry = [&](int p, int tap, E dy, E dx, E m, int tb_pl) __attribute__((always_inline)) {
    const int po = tile_s(plane_out), wo = tile_s(g.Wo), kw = tile_s(g.kw);
    const int tb_n = p / po;
    const int tb_rem = p - tb_n * po;
    const int tb_ho = tb_rem / wo;
    const int tb_wo = tb_rem - tb_ho * wo;
    const int ti = tap / kw, tj = tap - ti * kw;
    TapSample sm = make_tap_sample(tb_ho * g.sh - g.ph + ti * g.dh, tb_wo * g.sw - g.pw + tj * g.dw, to_f32(dy),
                                   to_f32(dx), mask_value<E>(m, a.om.logit), g.H, g.W);
    tpix[tap * PT + tb_pl] = (uint32_t)tb_n * a.img_bytes + corner_offset<UNBORDERED>(sm, g, a);
    tws[tap * PT + tb_pl] = make_uint2(TR::pack2(sm.w00, sm.w01), TR::pack2(sm.w10, sm.w11));
  };
  // where the offsets and the mask of pixel p live (tap 0)
  auto offsets_of = [&](int p, const E *&off, const E *&msk) __attribute__((always_inline)) {
    const int po = tile_s(plane_out);
    const int tb_n = p / po;
    const int tb_rem = p - tb_n * po;
    off = (const E *)a.om.off + (long)tb_n * a.om.off_n + (long)tb_rem * a.om.off_px;
    msk = (const E *)a.om.msk + (long)tb_n * a.om.msk_n + (long)tb_rem * a.om.msk_px;
  };

  // ---- cursors of the stream (all uniform).  Steps are counted through the tiles of the workgroup; in
  // the interval between two barriers in which the MFMAs of step (c_t, c_s) run, the blend cursor is one
  // step ahead of it, the gather cursor two, the weight-copy cursor one.  Past the last step of the last
  // tile the gather and weight cursors stay on it (loads nobody uses, which keep the wait counts constant).
  int c_t = 0, c_s = 0;                                     // MFMAs: tile, step
  int b_tap = 0;                                            // blend: tap (the table's row; the tile follows from the rewriting)
  int g_t = 0, g_tap = 0, g_slab = 0, g_slab0 = slab0_of(0);  // gather
  int w_t = 0, w_s = 0;                                     // weight copies
  const unsigned char *w_ptr = weights_of(0);               // ... packed weights of tile w_t, step 0

  // gather registers: four pixels x four corners
  u32x4 gs[4][4];
  // slab part of the gather addresses of the step the gather cursor is on; moves the cursor on
  auto next_slab_offset = [&]() {
    const uint32_t add_ = (uint32_t)(g_slab0 + g_slab) * a.slab_bytes + (uint32_t)ck * 16u;
    if (++g_tap == taps) {
      g_tap = 0;
      if (++g_slab == slabs) {
        if (g_t + 1 < T) {
          ++g_t;
          g_slab = 0;
          g_slab0 = slab0_of(g_t);
        } else {
          g_tap = taps - 1;
          g_slab = slabs - 1;
        }
      }
    }
    return add_;
  };

  // weight tile of the step the weight cursor is on into ring slot `slot` (late waves); moves the cursor on
  auto issue_weights = [&](int slot) {
    const uint32_t voff = (uint32_t)w_s * kWTile + wlane;
    const uint32_t voff_odd = voff ^ 32u;
    const uint32_t dst = lds_w + (uint32_t)slot * kWTile + wblock0;
    {
      // (the instruction's offset moves the LDS side along with the global one)
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 4\n\t"
                   "global_load_lds_dwordx4 %1, %3\n\t"
                   "global_load_lds_dwordx4 %2, %3 offset:1024\n\t"
                   "global_load_lds_dwordx4 %1, %3 offset:2048\n\t"
                   "global_load_lds_dwordx4 %2, %3 offset:3072"
                   :
                   : "s"(dst), "v"(voff), "v"(voff_odd), "s"(w_ptr)
                   : "memory");
      if constexpr (WD == 8) {
        const uint32_t voff2 = voff + 4096u, voff2_odd = voff_odd + 4096u;
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 4\n\t"
                     "global_load_lds_dwordx4 %1, %3\n\t"
                     "global_load_lds_dwordx4 %2, %3 offset:1024\n\t"
                     "global_load_lds_dwordx4 %1, %3 offset:2048\n\t"
                     "global_load_lds_dwordx4 %2, %3 offset:3072"
                     :
                     : "s"(dst + 4096u), "v"(voff2), "v"(voff2_odd), "s"(w_ptr)
                     : "memory");
      }
    }
    if (++w_s == nk) {
      if (w_t + 1 < T) {
        ++w_t;
        w_s = 0;
        w_ptr = weights_of(w_t);
      } else {
        w_s = nk - 1;
      }
    }
  };
  static_assert(WD == 8 || WD == 4, "issue_weights spells out the copies");

  // ---- the table's next edition (early waves).  In the interval of step (t, s) with s in the tile's last
  // slab, row s - (nk - taps) is written for tile t + 1: its last readers were the blends of the interval
  // before, a barrier ago.  Lane l of wave w serves pixel w * 32 + l % 32 + 128 * (l / 32): its own wave's
  // and those of the late wave four above.  The row's offsets and mask are loaded in the interval before;
  // with row 0 the lane works out where its pixel of the new tile lies (image, row, column) and keeps that
  // for the tile's rows.
  uint32_t tl_dy = 0, tl_dx = 0, tl_m = 0;   // what the interval before loaded (16 bits each)
  int tb_n = 0, tb_ho = 0, tb_wo = 0;        // the lane's pixel of the tile whose table is being written
  const int tb_pl = (wave & 3) * 32 + (lane & 31) + ((lane >> 5) << 7);
  // row that the interval of step (t, s) writes (for tile t + 1); < 0: none
  auto table_row = [&](int t, int s) __attribute__((always_inline)) { return t + 1 < T ? s - (nk - taps) : -1; };
  auto table_issue = [&](int t, int s) {  // loads for what the interval of step (t, s) will write
    const int row = table_row(t, s);
    const E *pdy = (const E *)a.om.off, *pdx = pdy, *pm = (const E *)a.om.msk;  // (nothing due: any valid address)
    if (row >= 0) {
      if (row == 0) {
        int ctile, grp, p0;
        decode(t + 1, ctile, grp, p0);
        const int po = tile_s(plane_out), wo = tile_s(g.Wo);
        const int p = p0 + tb_pl;
        tb_n = p / po;
        const int rem = p - tb_n * po;
        tb_ho = rem / wo;
        tb_wo = rem - tb_ho * wo;
      }
      const long rem = (long)(tb_ho * g.Wo + tb_wo);
      const E *off = (const E *)a.om.off + (long)tb_n * a.om.off_n + rem * a.om.off_px;
      pdy = off + (long)(2 * row) * a.om.off_ch;
      pdx = pdy + a.om.off_ch;
      pm = (const E *)a.om.msk + (long)tb_n * a.om.msk_n + rem * a.om.msk_px + (long)row * a.om.msk_ch;
    }
    asm volatile("global_load_ushort %0, %3, off\n\t"
                 "global_load_ushort %1, %4, off\n\t"
                 "global_load_ushort %2, %5, off"
                 : "=&v"(tl_dy), "=&v"(tl_dx), "=&v"(tl_m)
                 : "v"(pdy), "v"(pdx), "v"(pm));
  };
  auto table_write = [&](int t, int s) {  // with what table_issue(t, s) loaded, kVmStep loads ago
    asm volatile("s_waitcnt vmcnt(%3) ; %0 %1 %2" : "+v"(tl_dy), "+v"(tl_dx), "+v"(tl_m) : "n"(kVmStep));
    const int row = table_row(t, s);
    if (row >= 0) {
      const uint16_t by = (uint16_t)tl_dy, bx = (uint16_t)tl_dx, bm = (uint16_t)tl_m;
      const int kw = tile_s(g.kw);
      const int ti = __builtin_amdgcn_readfirstlane(row / kw), tj = row - ti * kw;
      TapSample sm = make_tap_sample(tb_ho * g.sh - g.ph + ti * g.dh, tb_wo * g.sw - g.pw + tj * g.dw,
                                     to_f32(__builtin_bit_cast(E, by)), to_f32(__builtin_bit_cast(E, bx)),
                                     mask_value<E>(__builtin_bit_cast(E, bm), a.om.logit), g.H, g.W);
      tpix[row * PT + tb_pl] = (uint32_t)tb_n * a.img_bytes + corner_offset<UNBORDERED>(sm, g, a);
      tws[row * PT + tb_pl] = make_uint2(TR::pack2(sm.w00, sm.w01), TR::pack2(sm.w10, sm.w11));
    }
  };

  // Blend of the lane's pixel I of the step the blend cursor is on into sample tile
  // XB, after a wait that leaves VM younger loads in flight; the pixel's loads for the
  // step behind it are issued right away.  The table entries of pixel I + 1 (blend
  // weights; corner offset of the step to gather) are read one pixel ahead.
#define MDCN_F3_PIXEL(I, VM, XB)                                                                 \
  do {                                                                                           \
    const uint2 twc_ = tw_;                                                                      \
    const uint32_t npc_ = np_ + add_;                                                            \
    if constexpr ((I) < 3) {                                                                     \
      tw_ = twp_[8 * ((I) + 1)];                                                                 \
      np_ = tp_[8 * ((I) + 1)];                                                                  \
    }                                                                                            \
    const typename BL::Wt w_ = BL::prep(twc_, q);                                                \
    f3_vmwait4<VM>(gs[I][0], gs[I][1], gs[I][2], gs[I][3]);                                      \
    const u32x4 o_ = BL::run(gs[I], w_);                                                         \
    *(lds_u32x4_ptr)(uintptr_t)((((I) & 1) ? xwb : xwa) + (uint32_t)(((I) >> 1) * 16 * kRowB) + (XB) * kXTile) = o_; \
    MDCN_F3_GATHER(gs[I], npc_);                                                                 \
  } while (0)
  // One produce block: blend the blend cursor's step, gather the gather cursor's.
#define MDCN_F3_BLOCK(XB)                                                                        \
  do {                                                                                           \
    const uint2 *twp_ = &tws[b_tap * PT + pl];                                                   \
    const uint32_t *tp_ = &tpix[g_tap * PT + pl];                                                \
    uint2 tw_ = twp_[0];                                                                         \
    uint32_t np_ = tp_[0];                                                                       \
    const uint32_t add_ = next_slab_offset();                                                    \
    if (++b_tap == taps) b_tap = 0;                                                              \
    MDCN_F3_PIXEL(0, kVmBlend, XB);                                                              \
    MDCN_F3_PIXEL(1, kVmBlend, XB);                                                              \
    MDCN_F3_PIXEL(2, kVmBlend, XB);                                                              \
    MDCN_F3_PIXEL(3, kVmBlend, XB);                                                              \
  } while (0)

  f32x16 acc[NB][MB];

  // ---- MFMA phase of one step: sample tile and ring slot XB.  The step is a chain
  // of 4 * MB groups -- K sub-step s = G / MB, channel block mb = G % MB -- of two
  // MFMAs (both pixel blocks against one channel block); the fragments of a group
  // (the channel block; with a new sub-step also the two pixel blocks) are read
  // three groups ahead.
  u32x4 xf[4][NB], wf[4][MB];
#define MDCN_F3_NREADS(G) ((G) < NG ? (((G) % MB) == 0 ? 3 : 1) : 0)
#define MDCN_F3_READS(G)                                                                         \
  do {                                                                                           \
    if constexpr ((G) < NG) {                                                                    \
      constexpr int s_ = (G) / MB, m_ = (G) % MB;                                                \
      const uint32_t wk_ = wb_ ^ (uint32_t)(s_ << 5);                                            \
      if constexpr (m_ == 0) {                                                                   \
        const uint32_t xk_ = xb_ ^ (uint32_t)(s_ << 5);                                          \
        MDCN_DSREAD(xf[s_][0], xk_, 0);                                                          \
        MDCN_DSREAD(xf[s_][1], xk_, 4096);                                                       \
      }                                                                                          \
      MDCN_DSREAD(wf[s_][m_], wk_, m_ * 4096);                                                   \
    }                                                                                            \
  } while (0)
#define MDCN_F3_GROUP(G)                                                                         \
  do {                                                                                           \
    if constexpr ((G) < NG) {                                                                    \
      constexpr int s_ = (G) / MB, m_ = (G) % MB;                                                \
      constexpr int after_ = MDCN_F3_NREADS((G) + 1) + MDCN_F3_NREADS((G) + 2) + MDCN_F3_NREADS((G) + 3); \
      if constexpr (m_ == 0)                                                                     \
        f3_lgkmwait3<after_>(xf[s_][0], xf[s_][1], wf[s_][0]);                                   \
      else                                                                                       \
        f3_lgkmwait1<after_>(wf[s_][m_]);                                                        \
      _Pragma("unroll") for (int nb_ = 0; nb_ < NB; ++nb_)                                       \
        TR::mma(acc[nb_][m_], __builtin_bit_cast(uint4, xf[s_][nb_]), __builtin_bit_cast(uint4, wf[s_][m_])); \
      MDCN_F3_READS((G) + 4);                                                                    \
    }                                                                                            \
  } while (0)
  // (priority: the arbiter prefers the wave of a SIMD that produces -- a chain of short
  // dependent steps whose delay moves the barrier -- over the one that streams MFMAs)
#define MDCN_F3_MFMA(XB)                                                                         \
  do {                                                                                           \
    uint32_t xb_ = lds_x + (XB) * kXTile + xa0;                                                  \
    uint32_t wb_ = lds_w + (XB) * kWTile + wa0;                                                  \
    /* (opaque: the four sub-step addresses of both tiles would otherwise live in registers across the loop) */ \
    asm volatile("" : "+v"(xb_), "+v"(wb_));                                                     \
    __builtin_amdgcn_s_setprio(0);                                                               \
    MDCN_F3_READS(0); MDCN_F3_READS(1); MDCN_F3_READS(2); MDCN_F3_READS(3);                      \
    MDCN_F3_GROUP(0); MDCN_F3_GROUP(1); MDCN_F3_GROUP(2); MDCN_F3_GROUP(3);                      \
    MDCN_F3_GROUP(4); MDCN_F3_GROUP(5); MDCN_F3_GROUP(6); MDCN_F3_GROUP(7);                      \
    MDCN_F3_GROUP(8); MDCN_F3_GROUP(9); MDCN_F3_GROUP(10); MDCN_F3_GROUP(11);                    \
    MDCN_F3_GROUP(12); MDCN_F3_GROUP(13); MDCN_F3_GROUP(14); MDCN_F3_GROUP(15);                  \
    __builtin_amdgcn_s_setprio(2);                                                               \
  } while (0)

  // ---- a tile's output: bias, one rounding, NCHW store straight from the accumulators.
  // Accumulator block (A = samples, B = weights): register r of lane l holds
  //   pixel = (r/4)*8 + (l/32)*4 + r%4,  channel = l%32.
  // The two halves of the wave exchange packed pixel pairs, after which a lane
  // holds 8 consecutive pixels = 16 bytes of one channel.  The host gives this
  // kernel whole tiles only, output planes of whole, aligned 16-byte runs that are
  // at least 64 pixels long -- so every run is one 16-byte store and the wave's 64
  // pixels cross at most one image boundary, between two runs -- and groups of whole
  // channel tiles (Cout / G a multiple of CT), so no lane is ever without a channel.
  auto store_tile = [&](int t) __attribute__((always_inline)) {
    int ctile, grp, p0;
    decode(t, ctile, grp, p0);
    E *out = (E *)a.out;
    const int tt = tile_tid();
    const int frow_ = tt & 31, fhalf_ = (tt >> 5) & 1;
    const int pw0 = p0 + wave_p * 64;
    const int po = tile_s(plane_out);
    const int n0 = __builtin_amdgcn_readfirstlane(pw0 / po);
    const int rem0 = pw0 - n0 * po + 8 * fhalf_;      // of the lane's first run
    const long next_image = (long)(g.Cout - 1) * po;  // what a run in the following image adds to the address
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      const int col = ctile * CT + wave_c * WCH + mb * 32 + frow_;
      const long cbase = (long)grp * g.cout_g + col;
      const float bvm = to_f32(bias_s[cbase]);
      E *row = out + ((long)n0 * g.Cout + cbase) * po + rem0;
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
          const int dp = nb * 32 + 16 * g2;
          E *dst = row + dp + ((rem0 + dp >= po) ? next_image : 0L);
          *(u32x4 *)dst = val;
        }
      }
    }
  };
  // behind the MFMAs of a step: the tile's output and fresh accumulators when it was the tile's last;
  // the MFMA cursor moves on
#define MDCN_F3_STEP_DONE(MAY_END)                                       \
  do {                                                                   \
    if (MAY_END && c_s == nk - 1) {                                      \
      store_tile(c_t);                                                   \
      _Pragma("unroll") for (int nb = 0; nb < NB; ++nb)                  \
        _Pragma("unroll") for (int mb = 0; mb < MB; ++mb)                \
          _Pragma("unroll") for (int r = 0; r < 16; ++r) acc[nb][mb][r] = 0.0f; \
      ++c_t;                                                             \
      c_s = 0;                                                           \
    } else {                                                             \
      ++c_s;                                                             \
    }                                                                    \
  } while (0)

  // One step of the stream between two barriers (XB = parity of the step; a tile has an even number of
  // steps, so its last one has XB = 1): MFMAs on sample tile and ring slot XB, blend of the next step into
  // the other sample tile, gather of the step after that; the late waves first copy the next step's weight
  // tile into the other slot, the early waves tend the table.
#define MDCN_F3_STEP(XB)                                                 \
  do {                                                                   \
    if constexpr (LATE) {                                                \
      issue_weights(1 - (XB));                                           \
      MDCN_F3_BLOCK(1 - (XB));                                           \
      __builtin_amdgcn_sched_barrier(0);                                 \
      MDCN_F3_MFMA(XB);                                                  \
      __builtin_amdgcn_sched_barrier(0);                                 \
      MDCN_F3_STEP_DONE((XB) == 1);                                      \
      MDCN_F3_BARRIER_COPIES(kVmStep);                                   \
    } else {                                                             \
      MDCN_F3_MFMA(XB);                                                  \
      __builtin_amdgcn_sched_barrier(0);                                 \
      const int it_ = c_t, is_ = c_s;                                    \
      MDCN_F3_STEP_DONE((XB) == 1);                                      \
      table_write(it_, is_);                                             \
      table_issue(c_t, c_s);                                             \
      MDCN_F3_BLOCK(1 - (XB));                                           \
      MDCN_BARRIER_LDS();                                                \
    }                                                                    \
    __builtin_amdgcn_sched_barrier(0);                                   \
  } while (0)

  // ---- start of the stream: the bias and the first tile's table (every lane: pixel tid % 256, taps
  // tid / 256 + 2 i), the gather of step 0 and its weight tile, its blend, the gather of step 1
  for (int i = tid; i < g.Cout; i += kF3Threads)
    bias_s[i] = a.bias ? ((const E *)a.bias)[i] : from_f32<E>(0.0f);
  {
    int ctile, grp, p0;
    decode(0, ctile, grp, p0);
    const int tapq = tid >> 8, px = tid & (PT - 1);
    const E *off, *msk;
    offsets_of(p0 + px, off, msk);
    E rdy[TPT], rdx[TPT], rm[TPT];
#pragma unroll
    for (int i = 0; i < TPT; ++i) {
      const int tap = min(tapq + 2 * i, taps - 1);
      rdy[i] = off[(long)(2 * tap) * a.om.off_ch];
      rdx[i] = off[(long)(2 * tap + 1) * a.om.off_ch];
      rm[i] = msk[(long)tap * a.om.msk_ch];
    }
#pragma unroll
    for (int i = 0; i < TPT; ++i) {
      const int tap = tapq + 2 * i;
      if (tap < taps) table_entry(p0 + px, tap, rdy[i], rdx[i], rm[i], px);
    }
    // (retire the loads with a wait the compiler can see: those of taps past the last one are never read,
    // and it would otherwise keep their registers marked as pending and guard the K loop's assembly loads
    // into them with full waits)
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0), other counters untouched
  }
  MDCN_BARRIER_LDS();  // table and bias visible
  __builtin_amdgcn_sched_barrier(0);
  {
    const uint32_t *tp_ = &tpix[g_tap * PT + pl];
    const uint32_t add_ = next_slab_offset();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t o_ = tp_[8 * i] + add_;
      MDCN_F3_GATHER(gs[i], o_);
    }
  }
  if constexpr (LATE) issue_weights(0);
#pragma unroll
  for (int i = 0; i < 4; ++i) f3_vmwait4<0>(gs[i][0], gs[i][1], gs[i][2], gs[i][3]);
  {
    const uint2 *twp_ = &tws[b_tap * PT + pl];
    if (++b_tap == taps) b_tap = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const typename BL::Wt w_ = BL::prep(twp_[8 * i], q);
      const u32x4 o_ = BL::run(gs[i], w_);
      *(lds_u32x4_ptr)(uintptr_t)(((i & 1) ? xwb : xwa) + (uint32_t)((i >> 1) * 16 * kRowB)) = o_;
    }
  }
  if constexpr (!LATE) table_issue(0, 0);
  {
    const uint32_t *tp_ = &tpix[g_tap * PT + pl];
    const uint32_t add_ = next_slab_offset();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t o_ = tp_[8 * i] + add_;
      MDCN_F3_GATHER(gs[i], o_);
    }
  }
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[nb][mb][r] = 0.0f;
  MDCN_BARRIER_LDS();  // X[0] complete (W[0] landed before the blend)
  __builtin_amdgcn_sched_barrier(0);

  // ---- the stream: T tiles of nk steps, two steps per round
  const int rounds = T * (nk >> 1);
  for (int r = 0; r < rounds; ++r) {
    MDCN_F3_STEP(0);
    MDCN_F3_STEP(1);
  }
  // what the cursors issued past the last step has landed before the registers (and the workgroup's LDS)
  // are given up
#pragma unroll
  for (int i = 0; i < 4; ++i) f3_vmwait4<0>(gs[i][0], gs[i][1], gs[i][2], gs[i][3]);
  asm volatile("s_waitcnt vmcnt(0) ; %0 %1 %2" : "+v"(tl_dy), "+v"(tl_dx), "+v"(tl_m));
#undef MDCN_F3_STEP
#undef MDCN_F3_STEP_DONE
#undef MDCN_F3_MFMA
#undef MDCN_F3_GROUP
#undef MDCN_F3_READS
#undef MDCN_F3_NREADS
#undef MDCN_F3_BLOCK
#undef MDCN_F3_PIXEL
#undef MDCN_F3_GATHER
}

template <typename E, int CT, bool UNBORDERED>
__global__ __launch_bounds__(kF3Threads) void fused3_kernel(FusedArgs a) {
  __shared__ uint4 Xs[2][kF3PT * kRowChunks];      // sample tiles
  __shared__ uint4 Ws[2][CT * kRowChunks];         // weight tiles
  __shared__ uint32_t tpix[kF3PT * kF3Taps];       // (pixel, tap) table, [tap][pixel]: corner byte offset
  __shared__ uint2 tws[kF3PT * kF3Taps];           // ... and the blend weights
  __shared__ E bias_s[kF3MaxBias];                 // the bias of every output channel (zeros without one)
  // (for the build's scan of the assembly: every count-based wait of this kernel is to be checked against
  // the loads issued behind the registers it names)
  asm volatile("; mdcn-counted-waits");
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const uint32_t lds_x = (uint32_t)(uintptr_t)(lptr_t)(&Xs[0][0]);
  const uint32_t lds_w = (uint32_t)(uintptr_t)(lptr_t)(&Ws[0][0]);
  if (wave >= 4) {
    MDCN_ROLE("late");
    fused3_role<E, CT, true, UNBORDERED>(a, lds_x, lds_w, tpix, tws, bias_s, wave);
  } else {
    MDCN_ROLE("early");
    fused3_role<E, CT, false, UNBORDERED>(a, lds_x, lds_w, tpix, tws, bias_s, wave);
  }
}

}  // namespace mdcn
