// C ABI of libmdcn_hip.so (see include/mdcn.h): parameter checks, path choice,
// workspace carving and kernel launches.  No allocation, no synchronisation
// (mdcn_forward_timed excepted, which exists to measure).
#include "../../include/mdcn.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cstdio>
#include <mutex>
#include <type_traits>

#include "mdcn_common.h"
#include "mdcn_direct.h"
#include "mdcn_f64.h"
#include "mdcn_backward.h"
#include "mdcn_backward_gemm.h"
#include "mdcn_fused.h"
#include "mdcn_fused2.h"
#include "mdcn_fused3.h"
#include "mdcn_oconv.h"
#include "mdcn_prepass.h"

namespace {

using namespace mdcn;

constexpr size_t kAlign = 256;
constexpr size_t kMaxLds = 160 * 1024;
// Device byte offsets into the channels-last copy are 32-bit.
constexpr uint64_t kMaxXtBytes = 0xF0000000ull;
// Column gradient (and columns) held in memory per pass of the backward's matrix-core paths.
constexpr uint64_t kBwdColGradCap = (uint64_t)3 << 29;  // 1.5 GiB each
// Per-pass limits in force (mdcn_set_pass_limits lowers them; process wide).  Atomic, so that a
// call that runs while another thread changes them reads one of the two values; a workspace that was
// sized under one value and used under another is still the caller's to avoid.
std::atomic<uint64_t> g_fwd_pass_bytes{kMaxXtBytes};
std::atomic<uint64_t> g_bwd_pass_bytes{kBwdColGradCap};

inline size_t align_up(size_t v) { return (v + kAlign - 1) / kAlign * kAlign; }

// Scratch of mdcn_forward_noalloc(): the input copy and the packed weights of one
// call, held by every device the library runs on until the process ends.  Host
// code never uses the array's name as an address: scratch_of_current_device()
// asks the runtime where the current device keeps its copy.
static __device__ __align__(256) unsigned char scratch[MDCN_NOALLOC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices] = {nullptr};

int scratch_of_current_device(void **out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return MDCN_ERR_LAUNCH;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void *ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) return MDCN_ERR_LAUNCH;
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return MDCN_OK;
}

inline size_t elem_size(int dtype) { return dtype == MDCN_F64 ? 8 : dtype == MDCN_F32 ? 4 : 2; }

int check_params(const mdcn_params *p, Geom *g, bool need_ptrs, bool need_offsets = true) {
  if (!p) return MDCN_ERR_NULL;
  if (p->dtype != MDCN_F32 && p->dtype != MDCN_F16 && p->dtype != MDCN_BF16 && p->dtype != MDCN_F64)
    return MDCN_ERR_DTYPE;
  if (p->N <= 0 || p->Cin <= 0 || p->H <= 0 || p->W <= 0 || p->Cout <= 0 ||
      p->kh <= 0 || p->kw <= 0 || p->sh <= 0 || p->sw <= 0 || p->ph < 0 ||
      p->pw < 0 || p->dh <= 0 || p->dw <= 0 || p->groups <= 0 || p->dgroups <= 0)
    return MDCN_ERR_SHAPE;
  if (p->Cin % p->groups || p->Cout % p->groups || p->Cin % p->dgroups)
    return MDCN_ERR_SHAPE;
  const long Ho = ((long)p->H + 2L * p->ph - ((long)p->dh * (p->kh - 1) + 1)) / p->sh + 1;
  const long Wo = ((long)p->W + 2L * p->pw - ((long)p->dw * (p->kw - 1) + 1)) / p->sw + 1;
  if ((long)p->H + 2L * p->ph < (long)p->dh * (p->kh - 1) + 1 ||
      (long)p->W + 2L * p->pw < (long)p->dw * (p->kw - 1) + 1 || Ho <= 0 || Wo <= 0)
    return MDCN_ERR_SHAPE;
  if (need_ptrs && (!p->input || !p->weight || !p->output)) return MDCN_ERR_NULL;
  if (need_ptrs && need_offsets && !p->offset) return MDCN_ERR_NULL;  // mask NULL: unmodulated
  g->N = p->N; g->Cin = p->Cin; g->H = p->H; g->W = p->W;
  g->Cout = p->Cout; g->kh = p->kh; g->kw = p->kw;
  g->sh = p->sh; g->sw = p->sw; g->ph = p->ph; g->pw = p->pw;
  g->dh = p->dh; g->dw = p->dw; g->G = p->groups; g->DG = p->dgroups;
  g->Ho = (int)Ho; g->Wo = (int)Wo;
  g->cin_g = p->Cin / p->groups;
  g->cout_g = p->Cout / p->groups;
  g->ch_per_dg = p->Cin / p->dgroups;
  g->taps = p->kh * p->kw;
  g->Hp = p->H + 2; g->Wp = p->W + 2;
  return MDCN_OK;
}

// channels per K step: 128 bytes
inline int slab_channels(int dtype) { return dtype == MDCN_F32 ? 32 : 64; }

inline int table_capacity(int taps) { return taps <= kTapsSmall ? kTapsSmall : kTapsLarge; }

// Output-channel tile of the fused kernel for a group of cout_g channels; the
// 256-wide tile leaves LDS room for the 9-tap table only.
inline int pick_ct(int cout_g, int taps) {
  if (cout_g > 128 && taps <= kTapsSmall) return 256;
  return cout_g > 64 ? 128 : 64;
}

bool fused_ok(const mdcn_params *p, const Geom &g) {
  if (p->dtype == MDCN_F64) return false;  // double precision: the one-thread-per-output kernels only
  const int KC = slab_channels(p->dtype);
  if (p->input_nhwc && (g.H < 2 || g.W < 2 || ((uintptr_t)p->input % 16) != 0)) return false;
  if (g.cin_g % KC || g.ch_per_dg % KC) return false;
  if (g.taps > kTapsLarge) return false;
  if (fused_lds_bytes(pick_ct(g.cout_g, g.taps), table_capacity(g.taps)) > kMaxLds) return false;
  // one padded image must fit the 32-bit offsets
  const uint64_t img = (uint64_t)g.Hp * g.Wp * g.Cin * elem_size(p->dtype);
  if (img > kMaxXtBytes) return false;
  if ((uint64_t)g.N * g.Ho * g.Wo > 0x7fffffffull) return false;
  return true;
}

int num_cus() {
  static int cached[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    cached[dev] = n;
  }
  return cached[dev];
}

// Length of the persistent schedule of `tiles` tiles of nk K steps in tile times, as UnitSchedule lays it
// out: whole rounds, then the last round's tiles whole or cut into parts.
double schedule_rounds(long tiles, int nk, bool may_cut) {
  const int stride = std::max(1, num_cus() / 8);
  const long chunk = (tiles + 7) / 8;  // the fullest XCD
  const long full = chunk / stride, rest = chunk % stride;
  if (rest == 0) return (double)full;
  const int rounds = (nk + kGatherAhead - 1) / kGatherAhead;
  long parts = 1;
  if (may_cut) parts = std::max<long>(1, std::min<long>(std::min<long>(stride / rest, kCutMax), rounds / (8 / kGatherAhead)));
  return (double)full + 1.0 / (double)parts;
}

struct Plan {
  bool fused;
  int CT, KC, n_ctiles, slabs;
  int n_chunk;       // images per launch of the fused path
  size_t xt_bytes;   // channels-last copy of one chunk
  size_t wp_bytes;   // packed weights
  size_t cut_bytes;  // eight-wave kernel: buffers and counters of the tiles it cuts along K (may be left out)
  int cut_wgs;     // ... one buffer and one counter per workgroup of its grid
  // pack-level call only
  int CO, CO_pad;    // conv_offset channels: 3 (2 when unmodulated) * DG * taps, rounded up to 32
  int mask_kind;     // kMaskLogit, or kMaskNone when unmodulated
  size_t owp_bytes;  // packed conv_offset weights (fused path, conv_offset run here)
  size_t raw_bytes;  // conv_offset output kept in the workspace
};

// What a pack-level call adds to the plain one.
struct PackExtra {
  const void *offset_weight, *offset_bias;
  void *raw;
};

inline bool forced_fused(int path) {
  return path == MDCN_PATH_FUSED || path == MDCN_PATH_FUSED_SPLIT || path == MDCN_PATH_FUSED_WIDE ||
         path == MDCN_PATH_FUSED_NARROW;
}

// 16-bit tensors, 256- or 128-channel tiles, one deformable group, enough K steps: the eight-wave
// kernels (mdcn_fused2.h; mdcn_fused3.h beside it where wide_ok() says so)
bool uses_fused2(const mdcn_params *p, const Geom &g, const Plan &pl) {
  if ((pl.CT != 256 && pl.CT != 128) || g.taps > kTapsSmall || elem_size(p->dtype) != 2 || g.DG != 1 ||
      p->path == MDCN_PATH_FUSED_SPLIT)
    return false;
  const int nk_pad = (pl.slabs * g.taps + kF2Unroll - 1) / kF2Unroll * kF2Unroll;
  return nk_pad >= kF2MinSteps;
}

// ... and the kernel with 256-pixel tiles for whole tiles of such a call: an even
// number of K steps, output planes of whole 16-byte runs (the caller checks the pointer's alignment), groups of
// whole channel tiles
bool wide_ok(const mdcn_params *p, const Geom &g, const Plan &pl) {
  if (!pl.fused || !uses_fused2(p, g, pl) || p->path == MDCN_PATH_FUSED_NARROW)
    return false;
  const int nk = pl.slabs * g.taps;
  const long plane_out = (long)g.Ho * g.Wo;
  return nk >= kF3MinSteps && nk % 2 == 0 && g.taps >= kF3MinTaps && plane_out % 8 == 0 && plane_out >= 64 &&
         g.cout_g % pl.CT == 0 && g.Cout <= kF3MaxBias;
}

// Rounds of the 128-pixel kernel's schedule for `tiles` tiles of nk K steps, in tile times (its last round's
// tiles are cut along K when that is allowed).
double narrow_rounds(long tiles, int nk, bool may_cut) {
  if (tiles <= 0) return 0.0;
  const int stride = std::max(1, num_cus() / 8);
  const long chunk = (tiles + 7) / 8;
  const long full = chunk / stride, rest = chunk % stride;
  if (rest == 0) return (double)full;
  const long steps6 = (nk + kF2Unroll - 1) / kF2Unroll;
  long parts = 1;
  if (may_cut) parts = std::max<long>(1, std::min<long>(std::min<long>(stride / rest, kCutMax), steps6));
  return (double)full + 1.0 / (double)parts;
}

// How many of a launch's pixel tiles of 256 go to the wide kernel: all of them (`all`), or whole rounds of
// its one-workgroup-per-CU grid when that and the 128-pixel kernel on the rest come out shorter than the
// 128-pixel kernel alone.  wide_cost: time of a 256-pixel tile in units of a 128-pixel one (measured).
// 256 channels, stride 1 (N=16, 100x152): 79.7 us per round of 256-pixel tiles against 46.6 us.
// 128 channels, stride 1 (N=16, 100x168): 29.4 us against 19.4 us.
// Stride 2 (128 channels, 200x336 input): the wide kernel's main stage takes as long as the narrow one's;
// neighbouring pixels share no input rows there and the time goes with the rows the L2 delivers.
inline double wide_tile_cost(int CT, bool unit_stride) { return !unit_stride ? 2.0 : CT == 256 ? 1.71 : 1.52; }
constexpr double kSecondKernelCost = 0.45;  // what launching the 128-pixel kernel behind it costs (ramps, table, tail)
long wide_tiles(long total_px, int n_ctiles_groups, int nk, bool may_cut, bool all, double wide_cost) {
  const long full = total_px / kF3PT;
  if (all || full == 0) return full;
  const long grid = std::max(8, num_cus() / 8 * 8);
  auto cost = [&](long n3) {
    const long wg_tiles = (n3 * n_ctiles_groups + grid - 1) / grid;  // tiles of the busiest workgroup
    const long px2 = total_px - n3 * kF3PT;
    const long tiles2 = (px2 + kPT - 1) / kPT * n_ctiles_groups;
    return wg_tiles * wide_cost + narrow_rounds(tiles2, nk, may_cut) + ((n3 && tiles2) ? kSecondKernelCost : 0.0);
  };
  const long rounds = full * n_ctiles_groups / grid;
  const long whole = rounds * grid / n_ctiles_groups;  // pixel tiles of the whole rounds
  long best = 0;
  double best_cost = cost(0);
  for (long n3 : {whole, full})
    if (n3 > 0 && cost(n3) < best_cost) best = n3, best_cost = cost(n3);
  return best;
}

// ... for a launch of total_px pixels of the call *p
long wide_tiles_of_call(const mdcn_params *p, const Geom &g, const Plan &pl, long total_px, bool out_vec_ok) {
  if (!wide_ok(p, g, pl) || !out_vec_ok) return 0;
  return wide_tiles(total_px, pl.n_ctiles * g.G, pl.slabs * g.taps, pl.cut_bytes != 0, p->path == MDCN_PATH_FUSED_WIDE,
                    wide_tile_cost(pl.CT, g.sh == 1 && g.sw == 1));
}

int make_plan(const mdcn_params *p, const Geom &g, Plan *pl) {
  const bool ok = fused_ok(p, g);
  if (forced_fused(p->path) && !ok) return MDCN_ERR_PATH;
  if (p->input_nhwc && (!ok || p->path == MDCN_PATH_DIRECT)) return MDCN_ERR_PATH;  // in-place reads: fused kernel only
  pl->fused = ok && p->path != MDCN_PATH_DIRECT;
  pl->CT = pl->KC = pl->n_ctiles = pl->slabs = pl->n_chunk = 0;
  pl->xt_bytes = pl->wp_bytes = pl->owp_bytes = pl->raw_bytes = pl->cut_bytes = 0;
  pl->cut_wgs = 0;
  pl->CO = 3 * g.DG * g.taps;
  pl->CO_pad = (pl->CO + 31) / 32 * 32;
  pl->mask_kind = kMaskLogit;
  if (!pl->fused) return MDCN_OK;
  const size_t es = elem_size(p->dtype);
  pl->KC = slab_channels(p->dtype);
  pl->CT = pick_ct(g.cout_g, g.taps);
  pl->slabs = g.cin_g / pl->KC;
  const uint64_t img = (uint64_t)g.Hp * g.Wp * g.Cin * es;
  pl->n_chunk = (int)std::min<uint64_t>((uint64_t)g.N, std::max<uint64_t>(1, g_fwd_pass_bytes.load() / img));
  if (p->dtype == MDCN_F32 && pl->CT == 256) {
    // fp32 tiles are bound by the matrix pipe (a K step of a 128 x 256 tile is some 7 000 clocks of
    // 32x32x2 MFMAs against 3 000 of sampling), so a tile's time goes with its width and what counts is
    // how evenly the tiles fill the workgroups: take the 128-wide tile when its schedule is shorter
    const long px_tiles = ((long)pl->n_chunk * g.Ho * g.Wo + kPT - 1) / kPT;
    const int nk = pl->slabs * g.taps;
    auto cost = [&](int ct) {
      const long tiles = px_tiles * ((g.cout_g + ct - 1) / ct) * g.G;
      return schedule_rounds(tiles, nk, !p->no_k_split) * std::max(7000.0 * ct / 256, 3000.0);
    };
    if (cost(128) < 0.95 * cost(256)) pl->CT = 128;
  }
  pl->n_ctiles = (g.cout_g + pl->CT - 1) / pl->CT;
  pl->xt_bytes = p->input_nhwc ? 0 : align_up((size_t)img * pl->n_chunk);
  pl->wp_bytes = align_up((size_t)g.G * pl->n_ctiles * pl->slabs * g.taps * pl->CT * pl->KC * es);
  // Tiles of the 128-pixel kernels' last round are cut along K where workgroups would otherwise idle: one
  // 128 x 256 fp32 tile and a counter per workgroup of the persistent grid -- asked for only when a launch
  // of this call has such a round (the 256-pixel kernel never cuts; what it leaves to the 128-pixel one may)
  if (!p->no_k_split) {
    const int stride = std::max(1, num_cus() / 8);
    auto may_cut = [&](long tiles) {  // an XCD's run of tiles ends in a round that fills at most half of its workgroups
      if (tiles <= 0) return false;
      const long chunk = (tiles + 7) / 8;
      for (long run : {chunk, tiles - 7 * chunk}) {
        const long rest = run > 0 ? run % stride : 0;
        if (rest > 0 && stride / rest >= 2) return true;
      }
      return false;
    };
    const long plane_out = (long)g.Ho * g.Wo;
    bool cuts = false;
    for (int n0 = 0; n0 < g.N && !cuts; n0 += pl->n_chunk) {
      const long total_px = (long)std::min(pl->n_chunk, g.N - n0) * plane_out;
      long px = total_px;
      if (wide_ok(p, g, *pl)) {
        // (the split itself looks at whether cutting is allowed: take the answer for "allowed")
        pl->cut_bytes = 1;
        px -= wide_tiles_of_call(p, g, *pl, total_px, plane_out % 8 == 0) * kF3PT;
        pl->cut_bytes = 0;
      }
      cuts = may_cut((px + kPT - 1) / kPT * pl->n_ctiles * g.G);
    }
    if (cuts) {
      pl->cut_wgs = num_cus() / 8 * 8;
      pl->cut_bytes = align_up((size_t)pl->cut_wgs * kPT * kF2CT * 4) + align_up((size_t)pl->cut_wgs * 4);
    }
  }
  if (p->path == MDCN_PATH_FUSED_WIDE && !wide_ok(p, g, *pl)) return MDCN_ERR_PATH;
  return MDCN_OK;
}

// Workspace of a pack-level call: [xt][wp][owp][raw] on the fused path, [raw] on
// the direct one (nothing when the caller's own raw buffer serves).
int make_pack_plan(const mdcn_pack_params *pp, const Geom &g, Plan *pl) {
  const mdcn_params *p = &pp->conv;
  if (p->input_nhwc) return MDCN_ERR_PATH;
  const int rc = make_plan(p, g, pl);
  if (rc != MDCN_OK) return rc;
  if (pp->unmodulated) {
    pl->CO = 2 * g.DG * g.taps;
    pl->CO_pad = (pl->CO + 31) / 32 * 32;
    pl->mask_kind = kMaskNone;
  }
  const size_t es = elem_size(p->dtype);
  const size_t plane = (size_t)g.Ho * g.Wo;
  if (pp->offset_weight) {
    if (pl->fused) {
      if (pl->CO_pad > 128) {  // accumulator blocks of the conv_offset kernel
        if (forced_fused(p->path)) return MDCN_ERR_PATH;
        pl->fused = false;
        pl->xt_bytes = pl->wp_bytes = pl->cut_bytes = 0;
        pl->cut_wgs = 0;
      } else {
        pl->owp_bytes = align_up((size_t)(g.Cin / pl->KC) * g.taps * 4 * (pl->CO_pad / 32) * 64 * 16);
        pl->raw_bytes = align_up((size_t)pl->n_chunk * plane * pl->CO_pad * es);
      }
    }
    if (!pl->fused && !pp->raw) pl->raw_bytes = align_up((size_t)g.N * pl->CO * plane * es);
  }
  return MDCN_OK;
}

// conv_offset of one batch chunk: the tiled kernel when its input patch and one
// slab of weights fit an LDS budget, else the gather variant.
template <typename E, int COF>
hipError_t launch_oconv(OconvArgs oa, hipStream_t st) {
  const Geom &g = oa.g;
  const int PW = 31 * g.sw + (g.kw - 1) * g.dw + 1;
  const long wbytes = (long)g.taps * 4 * COF * 1024;
  auto lds_bytes = [&](int th) {
    return (long)((th - 1) * g.sh + (g.kh - 1) * g.dh + 1) * PW * kRowB + wbytes;
  };
  oa.tiles_x = (g.Wo + 31) / 32;
  oa.PW = PW;
  auto tiled = [&](int th, auto kernel) {
    oa.TH = th;
    oa.tiles_y = (g.Ho + th - 1) / th;
    oa.PH = (th - 1) * g.sh + (g.kh - 1) * g.dh + 1;
    const long tiles = (long)g.N * oa.tiles_y * oa.tiles_x;
    hipLaunchKernelGGL(kernel, dim3((unsigned)tiles), dim3(256), 0, st, oa);
    return hipGetLastError();
  };
  // 8 rows per workgroup when that still fills the chip, else 4
  if constexpr (COF <= 2) {
    const long tiles8 = (long)g.N * ((g.Ho + 7) / 8) * oa.tiles_x;
    if (lds_bytes(8) <= kOconvLdsSmall && tiles8 >= 2L * num_cus())
      return tiled(8, oconv_tiled_kernel<E, COF, 2, kOconvLdsSmall>);
  }
  if (lds_bytes(4) <= kOconvLdsSmall) return tiled(4, oconv_tiled_kernel<E, COF, 1, kOconvLdsSmall>);
  if (lds_bytes(4) <= kOconvLdsLarge) return tiled(4, oconv_tiled_kernel<E, COF, 1, kOconvLdsLarge>);
  constexpr int PXF = COF == 1 ? 4 : (COF == 2 ? 2 : 1);
  const long px_per_block = 4L * 32 * PXF;
  const long blocks = (oa.total_px + px_per_block - 1) / px_per_block;
  hipLaunchKernelGGL((oconv_gather_kernel<E, COF, PXF>), dim3((unsigned)blocks), dim3(256), 0, st, oa);
  return hipGetLastError();
}

template <typename E, int CT, int TMAX, bool MULTI_DG>
hipError_t launch_fused_ct(const FusedArgs &fa, bool unbordered, hipStream_t st) {
  // persistent workgroups: one per CU, a multiple of the 8 XCDs
  // (with tiles cut along K, workgroups beyond the tile count take parts of tiles: the whole chip)
  const int total_wg = fa.n_ptiles * fa.n_ctiles * fa.g.G;
  const int per_xcd = fa.cut_max > 1 ? std::max(1, num_cus() / 8)
                                       : std::max(1, std::min((total_wg + 7) / 8, num_cus() / 8));
  if (unbordered)
    hipLaunchKernelGGL((fused_kernel<E, CT, TMAX, MULTI_DG, true>), dim3(per_xcd * 8), dim3(kThreads),
                       0, st, fa);
  else
    hipLaunchKernelGGL((fused_kernel<E, CT, TMAX, MULTI_DG, false>), dim3(per_xcd * 8), dim3(kThreads),
                       0, st, fa);
  return hipGetLastError();
}

// 16-bit tensors, 256- and 128-channel tiles: the eight-wave kernel of mdcn_fused2.h
template <typename E, int CT>
hipError_t launch_fused2(const FusedArgs &fa, bool unbordered, hipStream_t st) {
  const int total_wg = fa.n_ptiles * fa.n_ctiles * fa.g.G;
  const int per_xcd = fa.cut_max > 1 ? std::max(1, num_cus() / 8)
                                       : std::max(1, std::min((total_wg + 7) / 8, num_cus() / 8));
  if (unbordered)
    hipLaunchKernelGGL((fused2_kernel<E, CT, true>), dim3(per_xcd * 8), dim3(kF2Threads), 0, st, fa);
  else
    hipLaunchKernelGGL((fused2_kernel<E, CT, false>), dim3(per_xcd * 8), dim3(kF2Threads), 0, st, fa);
  return hipGetLastError();
}

// 16-bit tensors, 256- or 128-channel tiles, whole tiles of 256 pixels: mdcn_fused3.h
template <typename E>
hipError_t launch_fused3(const FusedArgs &fa, int CT, bool nhwc, hipStream_t st) {
  const int total_wg = fa.n_ptiles * fa.n_ctiles * fa.g.G;
  const int per_xcd = std::max(1, std::min((total_wg + 7) / 8, num_cus() / 8));
  const dim3 grid(per_xcd * 8), block(kF3Threads);
  if (CT == 256) {
    if (nhwc)
      hipLaunchKernelGGL((fused3_kernel<E, 256, true>), grid, block, 0, st, fa);
    else
      hipLaunchKernelGGL((fused3_kernel<E, 256, false>), grid, block, 0, st, fa);
  } else {
    if (nhwc)
      hipLaunchKernelGGL((fused3_kernel<E, 128, true>), grid, block, 0, st, fa);
    else
      hipLaunchKernelGGL((fused3_kernel<E, 128, false>), grid, block, 0, st, fa);
  }
  return hipGetLastError();
}

template <typename E, int CT>
hipError_t launch_fused_tm(const FusedArgs &fa, bool ub, bool eight_wave, hipStream_t st) {
  const bool small = fa.g.taps <= kTapsSmall;
  if constexpr (sizeof(E) == 2 && (CT == 256 || CT == 128)) {
    if (eight_wave) return launch_fused2<E, CT>(fa, ub, st);
  }
  if constexpr (CT == 256) {  // (pick_ct never pairs the 256-wide tile with the large table)
    return fa.g.DG > 1 ? launch_fused_ct<E, CT, kTapsSmall, true>(fa, ub, st)
                       : launch_fused_ct<E, CT, kTapsSmall, false>(fa, ub, st);
  } else {
    if (fa.g.DG > 1)
      return small ? launch_fused_ct<E, CT, kTapsSmall, true>(fa, ub, st)
                   : launch_fused_ct<E, CT, kTapsLarge, true>(fa, ub, st);
    return small ? launch_fused_ct<E, CT, kTapsSmall, false>(fa, ub, st)
                 : launch_fused_ct<E, CT, kTapsLarge, false>(fa, ub, st);
  }
}

template <typename E>
hipError_t launch_fused(const FusedArgs &fa, int CT, bool ub, bool eight_wave, hipStream_t st) {
  switch (CT) {
    case 64: return launch_fused_tm<E, 64>(fa, ub, eight_wave, st);
    case 128: return launch_fused_tm<E, 128>(fa, ub, eight_wave, st);
    default: return launch_fused_tm<E, 256>(fa, ub, eight_wave, st);
  }
}

template <typename E>
int run_typed(const mdcn_params *p, const Geom &g, const Plan &pl, hipStream_t st,
              float *ms, const PackExtra *px) {
  hipEvent_t ev[2] = {nullptr, nullptr};
  auto tic = [&]() { if (ms) (void)hipEventRecord(ev[0], st); };
  auto toc = [&](int slot) {
    if (!ms) return;
    (void)hipEventRecord(ev[1], st);
    (void)hipEventSynchronize(ev[1]);
    float t = 0.f;
    (void)hipEventElapsedTime(&t, ev[0], ev[1]);
    ms[slot] += t;
  };
  if (ms) {
    ms[0] = ms[1] = ms[2] = ms[3] = 0.f;
    if (px) ms[4] = 0.f;
    if (hipEventCreate(&ev[0]) != hipSuccess || hipEventCreate(&ev[1]) != hipSuccess)
      return MDCN_ERR_LAUNCH;
  }
  int rc = MDCN_OK;
  const size_t es = sizeof(E);
  const long plane_out = (long)g.Ho * g.Wo;

  // the conv_offset output of a pack-level call as dense (N, CO, Ho, Wo)
  auto nchw_raw_view = [&](const E *raw) {
    OffMaskView v;
    v.off = raw;
    v.msk = raw + (long)2 * g.DG * g.taps * plane_out;
    v.off_n = v.msk_n = (long)pl.CO * plane_out;
    v.off_ch = v.msk_ch = plane_out;
    v.off_px = v.msk_px = 1;
    v.logit = pl.mask_kind;
    if (pl.mask_kind == kMaskNone) v.msk = raw;
    return v;
  };

  if (!pl.fused) {
    OffMaskView om = dense_view(p->offset, p->mask, g);
    if (px) {
      E *raw = (E *)px->raw;
      if (px->offset_weight) {
        if (!raw) raw = (E *)p->workspace;
        const long total = (long)g.N * pl.CO * plane_out;
        const int grid = (int)std::min<long>((total + 255) / 256, 1L << 20);
        tic();
        hipLaunchKernelGGL(oconv_direct_kernel<E>, dim3(grid), dim3(256), 0, st, g,
                           (const E *)p->input, (const E *)px->offset_weight,
                           (const E *)px->offset_bias, raw, pl.CO, total);
        if (hipGetLastError() != hipSuccess) rc = MDCN_ERR_LAUNCH;
        toc(4);
      }
      om = nchw_raw_view(raw);
    }
    const long total = (long)g.N * g.Cout * plane_out;
    const int grid = (int)std::min<long>((total + 255) / 256, 1L << 20);
    tic();
    hipLaunchKernelGGL(direct_kernel<E>, dim3(grid), dim3(256), 0, st, g,
                       (const E *)p->input, om, (const E *)p->weight,
                       (const E *)p->bias, (E *)p->output, total);
    if (hipGetLastError() != hipSuccess) rc = MDCN_ERR_LAUNCH;
    toc(2);
  } else {
    unsigned char *ws = (unsigned char *)p->workspace;
    E *xt = (E *)ws;
    E *wp = (E *)(ws + pl.xt_bytes);
    E *owp = (E *)(ws + pl.xt_bytes + pl.wp_bytes);
    E *raw_pm = (E *)(ws + pl.xt_bytes + pl.wp_bytes + pl.owp_bytes);
    const bool own_oconv = px && px->offset_weight;
    const int cof = pl.CO_pad / 32;
    float *cut_part = (float *)(ws + pl.xt_bytes + pl.wp_bytes + pl.owp_bytes + pl.raw_bytes);
    uint32_t *cut_cnt = (uint32_t *)((unsigned char *)cut_part + align_up((size_t)pl.cut_wgs * kPT * kF2CT * 4));
    if (!pl.cut_bytes) cut_part = nullptr, cut_cnt = nullptr;

    // weights: once per call -- inside the launch that re-lays the first batch chunk; on their own when
    // there is no such launch (channels-last input read in place)
    constexpr int EPV = 16 / (int)sizeof(E);
    const bool vec_relayout = !p->input_nhwc;
    const long wtotal = (long)g.G * pl.n_ctiles * pl.slabs * g.taps * pl.CT * pl.KC;
    bool packed = false;
    {
      tic();
      if (!vec_relayout) {
        const int grid = (int)std::min<long>((wtotal + 255) / 256, 1L << 16);
        hipLaunchKernelGGL(pack_weight_kernel<E>, dim3(grid), dim3(256), 0, st, g,
                           (const E *)p->weight, wp, pl.CT, pl.KC, pl.n_ctiles,
                           pl.slabs, wtotal, cut_cnt, pl.cut_wgs);
        if (hipGetLastError() != hipSuccess) rc = MDCN_ERR_LAUNCH;
        packed = true;
      }
      if (own_oconv) {
        const long ototal = (long)(g.Cin / pl.KC) * g.taps * 4 * cof * 64 * (16 / (long)es);
        const int ogrid = (int)std::min<long>((ototal + 255) / 256, 1L << 16);
        hipLaunchKernelGGL(pack_offset_weight_kernel<E>, dim3(ogrid), dim3(256), 0, st, g,
                           (const E *)px->offset_weight, owp, pl.CO, cof, ototal);
        if (hipGetLastError() != hipSuccess) rc = MDCN_ERR_LAUNCH;
      }
      toc(1);
    }
    for (int n0 = 0; n0 < g.N && rc == MDCN_OK; n0 += pl.n_chunk) {
      Geom gc = g;
      gc.N = std::min(pl.n_chunk, g.N - n0);
      const E *in = (const E *)p->input + (size_t)n0 * g.Cin * g.H * g.W;
      const bool nhwc = p->input_nhwc != 0;
      if (!nhwc && vec_relayout) {
        const int n_pchunks = (gc.H * gc.W + 32 * EPV - 1) / (32 * EPV);
        const long blocks = (long)gc.N * (gc.Cin / pl.KC) * n_pchunks;
        tic();
        if (!packed) {
          const int pack_blocks = (int)std::max<long>(1, std::min<long>(wtotal / (256 * 8), 512));
          hipLaunchKernelGGL(prepass_kernel<E>, dim3((unsigned)(blocks + pack_blocks)), dim3(256), 0, st, gc, in, xt,
                             n_pchunks, g, (const E *)p->weight, wp, pl.CT, pl.KC, pl.n_ctiles, pl.slabs, wtotal,
                             pack_blocks, cut_cnt, pl.cut_wgs);
          packed = true;
        } else {
          hipLaunchKernelGGL((relayout_vec_kernel<E, true>), dim3((unsigned)blocks), dim3(256), 0, st, gc, in, xt,
                             n_pchunks);
        }
        if (hipGetLastError() != hipSuccess) rc = MDCN_ERR_LAUNCH;
        toc(0);
      }
      FusedArgs fa;
      fa.g = gc;
      fa.xt = nhwc ? (const void *)in : (const void *)xt;
      fa.wp = wp;
      if (nhwc) {
        fa.px_bytes = (uint32_t)(g.Cin * es);
        fa.row_bytes = (uint32_t)g.W * fa.px_bytes;
        fa.slab_bytes = (uint32_t)kRowB;
        fa.img_bytes = (uint32_t)g.H * fa.row_bytes;
      } else {
        fa.px_bytes = (uint32_t)kRowB;
        fa.row_bytes = (uint32_t)g.Wp * (uint32_t)kRowB;
        fa.slab_bytes = (uint32_t)(g.Hp * g.Wp) * (uint32_t)kRowB;
        fa.img_bytes = (uint32_t)(g.Cin / pl.KC) * fa.slab_bytes;
      }
      if (own_oconv) {
        OconvArgs oa;
        oa.g = gc;
        oa.xt = xt;
        oa.owp = owp;
        oa.obias = px->offset_bias;
        oa.raw = raw_pm;
        oa.total_px = (long)gc.N * plane_out;
        oa.CO = pl.CO;
        oa.CO_pad = pl.CO_pad;
        oa.slabs_total = g.Cin / pl.KC;
        oa.plane_px = g.Hp * g.Wp;
        tic();
        hipError_t e = cof == 1 ? launch_oconv<E, 1>(oa, st)
                     : cof == 2 ? launch_oconv<E, 2>(oa, st)
                     : cof == 3 ? launch_oconv<E, 3>(oa, st)
                                : launch_oconv<E, 4>(oa, st);
        if (e != hipSuccess) rc = MDCN_ERR_LAUNCH;
        if (px->raw) {
          const long total = (long)gc.N * pl.CO * plane_out;
          const int grid = (int)std::min<long>((total + 255) / 256, 1L << 20);
          hipLaunchKernelGGL(raw_to_nchw_kernel<E>, dim3(grid), dim3(256), 0, st, raw_pm,
                             (E *)px->raw + (size_t)n0 * pl.CO * plane_out, pl.CO, pl.CO_pad,
                             plane_out, total);
          if (hipGetLastError() != hipSuccess) rc = MDCN_ERR_LAUNCH;
        }
        toc(4);
        // pixel-major: the values of one pixel are CO_pad consecutive elements
        fa.om.off = raw_pm;
        fa.om.msk = raw_pm + 2 * g.DG * g.taps;
        fa.om.off_n = fa.om.msk_n = plane_out * pl.CO_pad;
        fa.om.off_ch = fa.om.msk_ch = 1;
        fa.om.off_px = fa.om.msk_px = pl.CO_pad;
        fa.om.logit = pl.mask_kind;
        if (pl.mask_kind == kMaskNone) fa.om.msk = raw_pm;
      } else if (px) {
        fa.om = nchw_raw_view((const E *)px->raw + (size_t)n0 * pl.CO * plane_out);
      } else {
        fa.om = dense_view((const E *)p->offset + (size_t)n0 * g.DG * 2 * g.taps * plane_out,
                           p->mask ? (const E *)p->mask + (size_t)n0 * g.DG * g.taps * plane_out : nullptr, g);
      }
      fa.cut_max = pl.cut_bytes ? kCutMax : 0;
      fa.cut_part = cut_part;
      fa.cut_cnt = cut_cnt;
      fa.bias = p->bias;
      fa.out = (E *)p->output + (size_t)n0 * g.Cout * plane_out;
      fa.total_px = (long)gc.N * plane_out;
      fa.n_ptiles = (int)((fa.total_px + kPT - 1) / kPT);
      fa.n_ctiles = pl.n_ctiles;
      fa.slabs = pl.slabs;
      fa.slabs_total = g.Cin / pl.KC;
      fa.plane_px = g.Hp * g.Wp;
      fa.out_vec_ok = (plane_out % (long)(16 / es) == 0) && (((uintptr_t)fa.out % 16) == 0);
      fa.px0 = 0;
      tic();
      const bool eight_wave = uses_fused2(p, g, pl);
      bool rest = true;
      if constexpr (sizeof(E) == 2) {
        {
          // whole tiles of 256 pixels to the wide kernel, what is left to the 128-pixel one
          const long n3 = wide_tiles_of_call(p, g, pl, fa.total_px, fa.out_vec_ok != 0);
          if (n3 > 0) {
            FusedArgs fw = fa;
            fw.n_ptiles = (int)n3;
            if (launch_fused3<E>(fw, pl.CT, nhwc, st) != hipSuccess) rc = MDCN_ERR_LAUNCH;
            fa.px0 = (int)(n3 * kF3PT);
            fa.n_ptiles = (int)((fa.total_px - fa.px0 + kPT - 1) / kPT);
            rest = fa.n_ptiles > 0;
          }
        }
      }
      if (rest && launch_fused<E>(fa, pl.CT, nhwc, eight_wave, st) != hipSuccess) rc = MDCN_ERR_LAUNCH;
      toc(2);
    }
  }
  if (ms) {
    ms[3] = ms[0] + ms[1] + ms[2] + (px ? ms[4] : 0.f);
    (void)hipEventDestroy(ev[0]);
    (void)hipEventDestroy(ev[1]);
  }
  return rc;
}

// Double precision: one kernel, no workspace.
int run_f64(const mdcn_params *p, const Geom &g, hipStream_t st, float *ms) {
  hipEvent_t ev[2] = {nullptr, nullptr};
  if (ms) {
    ms[0] = ms[1] = ms[2] = ms[3] = 0.f;
    if (hipEventCreate(&ev[0]) != hipSuccess || hipEventCreate(&ev[1]) != hipSuccess) return MDCN_ERR_LAUNCH;
    (void)hipEventRecord(ev[0], st);
  }
  const long total = (long)g.N * g.Cout * g.Ho * g.Wo;
  const int grid = (int)std::min<long>((total + 255) / 256, 1L << 20);
  hipLaunchKernelGGL(f64_forward_kernel, dim3(grid), dim3(256), 0, st, g, (const double *)p->input,
                     (const double *)p->offset, (const double *)p->mask, (const double *)p->weight,
                     (const double *)p->bias, (double *)p->output, total);
  const int rc = hipGetLastError() == hipSuccess ? MDCN_OK : MDCN_ERR_LAUNCH;
  if (ms) {
    (void)hipEventRecord(ev[1], st);
    (void)hipEventSynchronize(ev[1]);
    (void)hipEventElapsedTime(&ms[2], ev[0], ev[1]);
    ms[3] = ms[2];
    (void)hipEventDestroy(ev[0]);
    (void)hipEventDestroy(ev[1]);
  }
  return rc;
}

int run(const mdcn_params *p, void *stream, float *ms, const mdcn_pack_params *pp = nullptr) {
  Geom g;
  int rc = check_params(p, &g, true, pp == nullptr);
  if (rc != MDCN_OK) return rc;
  Plan pl;
  PackExtra px_store, *px = nullptr;
  if (pp) {
    if (!pp->offset_weight && !pp->raw) return MDCN_ERR_NULL;
    rc = make_pack_plan(pp, g, &pl);
    px_store.offset_weight = pp->offset_weight;
    px_store.offset_bias = pp->offset_bias;
    px_store.raw = pp->raw;
    px = &px_store;
  } else {
    rc = make_plan(p, g, &pl);
  }
  if (rc != MDCN_OK) return rc;
  if (p->dtype == MDCN_F64) {
    if (pp) return MDCN_ERR_DTYPE;  // the pack-level call has no double-precision form
    return run_f64(p, g, (hipStream_t)stream, ms);
  }
  // (the split-tile buffers come last and are optional: a workspace without them runs unsplit)
  const size_t need = pl.xt_bytes + pl.wp_bytes + pl.owp_bytes + pl.raw_bytes;
  if (need > 0 && (!p->workspace || p->workspace_bytes < need ||
                   ((uintptr_t)p->workspace % kAlign) != 0))
    return MDCN_ERR_WORKSPACE;
  if (p->workspace_bytes < need + pl.cut_bytes) pl.cut_bytes = 0, pl.cut_wgs = 0;
  hipStream_t st = (hipStream_t)stream;
  switch (p->dtype) {
    case MDCN_F32: return run_typed<float>(p, g, pl, st, ms, px);
    case MDCN_F16: return run_typed<f16_t>(p, g, pl, st, ms, px);
    default: return run_typed<bf16_t>(p, g, pl, st, ms, px);
  }
}

// Largest margin R (up to 8) for which the LDS window of a th x tw output-pixel
// tile fits max_px pixels; -1 if even R = 0 does not.
int window_margin(const Geom &g, int th, int tw, long max_px, int *WH, int *WW) {
  const long base_h = (long)(th - 1) * g.sh + (long)(g.kh - 1) * g.dh + 2;
  const long base_w = (long)(tw - 1) * g.sw + (long)(g.kw - 1) * g.dw + 2;
  int R = -1;
  while (R < 8 && (base_h + 2 * (R + 1)) * (base_w + 2 * (R + 1)) <= max_px) ++R;
  *WH = (int)base_h + 2 * std::max(R, 0);
  *WW = (int)base_w + 2 * std::max(R, 0);
  return R;
}

struct BwdPlan {
  size_t gin_bytes, gw_bytes;  // fp32 staging (0 for fp32 tensors)
  // grad_input / grad_offset / grad_mask by bwd_data_tiled_kernel (else, without
  // `gemm`, one workgroup per tap):
  bool tiled;
  int R, WH, WW;   // its window margin and size
  // matrix-core paths (bwd_colgrad_kernel + bwd_scatter_kernel, bwd_wgrad_kernel):
  bool gemm;       // data gradients
  bool wgemm;      // grad_weight from stored columns
  int sR, sWH, sWW;  // window of the scatter kernel
  int sCH;         // channels per pass over that window
  int n_chunk;     // images per pass
  int cg_tile;     // tile of the column-gradient product (kCgTile or kCgTileBig)
  int M_pad;       // rows of the transposed weight matrix per group
  long P_pad;      // row pitch of the columns matrix
  int parts;       // workgroups of the scatter kernel per tile (shares of the channels)
  size_t xt_bytes, gt_bytes, wt_bytes, d_bytes, col_bytes, part_bytes;
  int w_tile, w_splits;  // weight-gradient product: tile, shares of the K range
  size_t wpart_bytes;    // ... and their partial sums
  size_t gpad_bytes;     // grad_output with padded rows, when its own rows cannot be copied 16 bytes at a time
  size_t gb_bytes;  // fp32 sum of grad_bias (16-bit tensors)
  size_t mx_bytes;  // the two maxima that scale the fixed-point window (16-bit tensors)
  size_t total() const {
    return gin_bytes + gw_bytes + gb_bytes + mx_bytes + xt_bytes + gt_bytes + wt_bytes + d_bytes + col_bytes + part_bytes +
           wpart_bytes + gpad_bytes;
  }
};

void make_bwd_plan(const mdcn_bwd_params *bp, const Geom &g, BwdPlan *pl) {
  const bool f64 = bp->conv.dtype == MDCN_F64;
  const bool staged = bp->conv.dtype != MDCN_F32 && !f64;
  const size_t es = elem_size(bp->conv.dtype);
  pl->gin_bytes = (staged && bp->grad_input) ? align_up((size_t)g.N * g.Cin * g.H * g.W * 4) : 0;
  pl->gw_bytes = (staged && bp->grad_weight) ? align_up((size_t)g.Cout * g.cin_g * g.taps * 4) : 0;
  pl->gb_bytes = (staged && bp->grad_bias) ? align_up((size_t)g.Cout * 4) : 0;
  pl->mx_bytes = 0;
  pl->tiled = pl->gemm = pl->wgemm = false;
  pl->xt_bytes = pl->gt_bytes = pl->wt_bytes = pl->d_bytes = pl->col_bytes = pl->part_bytes = pl->wpart_bytes = 0;
  pl->w_tile = kCgTile;
  pl->w_splits = 1;
  pl->gpad_bytes = 0;
  pl->parts = 1;
  pl->n_chunk = g.N;
  pl->M_pad = 0;
  pl->cg_tile = kCgTile;
  pl->P_pad = 0;
  pl->R = pl->sR = -1;
  pl->WH = pl->WW = pl->sWH = pl->sWW = 0;
  const int path = forced_fused(bp->conv.path) ? MDCN_PATH_FUSED : bp->conv.path;
  if (path == MDCN_PATH_DIRECT || g.taps > kBwdTapsMax || f64) return;
  const bool forced = path == MDCN_PATH_FUSED;
  const size_t plane_out = (size_t)g.Ho * g.Wo;

  // matrix-core paths: channels in whole 128-byte slabs, 32-channel blocks per tap
  const int KC = (int)(128 / es);
  const size_t d_img = (size_t)g.taps * g.Cin * plane_out * es;
  // channels per pass: 16 / 8 of 32-bit fixed point (16-bit tensors), 8 / 4 doubles (fp32)
  const int ch_big = es == 2 ? 16 : 8;
  pl->sCH = ch_big;
  pl->sR = window_margin(g, kScTH, kScTW, kScWindowPx, &pl->sWH, &pl->sWW);
  if (pl->sR < 2 || g.ch_per_dg % ch_big) {  // fewer channels at a time buy a wider window
    int wh, ww;
    const int r = window_margin(g, kScTH, kScTW, 2 * kScWindowPx, &wh, &ww);
    if (r > pl->sR || g.ch_per_dg % ch_big) {
      pl->sCH = ch_big / 2;
      pl->sR = r;
      pl->sWH = wh;
      pl->sWW = ww;
    }
  }
  const long s_tiles = (long)g.N * g.DG * ((g.Ho + kScTH - 1) / kScTH) * ((g.Wo + kScTW - 1) / kScTW);
  const bool mfma_ok = g.Cin % KC == 0 && g.cout_g % KC == 0 && g.cin_g % 32 == 0 &&
                       g.ch_per_dg % pl->sCH == 0 && pl->sR >= 1 && (s_tiles >= 64 || forced) &&
                       d_img <= kBwdColGradCap && plane_out <= ((size_t)1 << 30) &&
                       (size_t)g.H * g.W <= ((size_t)1 << 30);  // (plane offsets held in 32 bits)
  if (mfma_ok) {
    pl->gemm = bp->grad_input != nullptr;
    pl->wgemm = bp->grad_weight != nullptr;
  }
  if (pl->gemm || pl->wgemm) {
    pl->n_chunk = (int)std::min<uint64_t>((uint64_t)g.N, std::max<uint64_t>(1, g_bwd_pass_bytes.load() / d_img));
    pl->xt_bytes = align_up((size_t)g.N * (g.Cin / KC) * g.Hp * g.Wp * 128);
  }
  if (pl->gemm) {
    pl->cg_tile = (g.taps * g.cin_g >= kCgTileBig && plane_out >= (size_t)kCgTileBig) ? kCgTileBig : kCgTile;
    pl->M_pad = (g.taps * g.cin_g + pl->cg_tile - 1) / pl->cg_tile * pl->cg_tile;
    pl->gt_bytes = align_up((size_t)g.N * (g.Cout / KC) * plane_out * 128);
    pl->wt_bytes = align_up((size_t)g.G * pl->M_pad * g.cout_g * es);
    pl->d_bytes = align_up(d_img * pl->n_chunk);
    // enough workgroups for eight rounds or so of the chip's 2 x CUs slots
    while (pl->parts < 8 && s_tiles * pl->parts < 4096 && g.ch_per_dg % (2 * pl->parts * pl->sCH) == 0)
      pl->parts *= 2;
    if (staged) pl->mx_bytes = kAlign;
    if (pl->parts > 1) pl->part_bytes = align_up((size_t)pl->parts * g.N * g.DG * 3 * g.taps * plane_out * 4);
  }
  if (pl->wgemm) {
    const long kpx = 128 / (long)es;  // pixels per K step
    pl->P_pad = ((long)plane_out + kpx - 1) / kpx * kpx;
    pl->col_bytes = align_up((size_t)pl->n_chunk * g.taps * g.Cin * pl->P_pad * es);
    const int M = g.taps * g.cin_g;
    pl->w_tile = (g.cout_g >= 192 && M >= kCgTileBig) ? kCgTileBig : kCgTile;
    const long tiles = (long)g.G * ((g.cout_g + pl->w_tile - 1) / pl->w_tile) * ((M + pl->w_tile - 1) / pl->w_tile);
    // one round of workgroups (256-tiles: one per CU, 128-tiles: two), shares of at least 8 K steps
    const long slots = pl->w_tile == kCgTileBig ? 256 : 512;
    const long work = (long)pl->n_chunk * (pl->P_pad / kpx);
    pl->w_splits = (int)std::max<long>(1, std::min<long>(std::min<long>(work / 8, 64), slots / tiles));
    pl->wpart_bytes = align_up((size_t)pl->w_splits * g.Cout * M * 4);
    // grad_output rows go to LDS 16 bytes at a time: in place when they start aligned
    if (plane_out % (16 / es) != 0 || ((uintptr_t)bp->grad_output % 16) != 0)
      pl->gpad_bytes = align_up((size_t)g.N * g.Cout * pl->P_pad * es);
  }
  if (bp->grad_input && !pl->gemm) {
    // (small problems keep the per-tap kernel: it has taps x more workgroups)
    pl->R = window_margin(g, kBwdTile, kBwdTile, kBwdWindowBytes / (4 * kBwdChunk), &pl->WH, &pl->WW);
    const long n_tiles = (long)g.N * g.DG * ((g.Ho + kBwdTile - 1) / kBwdTile) * ((g.Wo + kBwdTile - 1) / kBwdTile);
    pl->tiled = pl->R >= 1 && (n_tiles >= 512 || forced);
  }
}

template <typename E>
int run_backward_typed(const mdcn_bwd_params *bp, const Geom &g, const BwdPlan &pl, hipStream_t st) {
  const mdcn_params *p = &bp->conv;
  constexpr int KC = 128 / (int)sizeof(E);
  const long plane_out = (long)g.Ho * g.Wo;
  const OffMaskView om = dense_view(p->offset, p->mask, g);
  unsigned char *ws = (unsigned char *)p->workspace;
  auto blocks_for = [](long n) { return (int)std::max<long>(1, std::min<long>((n + 255) / 256, 1L << 20)); };
  int rc = MDCN_OK;
  auto check = [&]() { if (hipGetLastError() != hipSuccess) rc = MDCN_ERR_LAUNCH; };

  const long n_in = (long)g.N * g.Cin * g.H * g.W;
  const long n_w = (long)g.Cout * g.cin_g * g.taps;
  float *gin32 = pl.gin_bytes ? (float *)ws : (float *)bp->grad_input;
  float *gw32 = pl.gw_bytes ? (float *)(ws + pl.gin_bytes) : (float *)bp->grad_weight;
  float *gb32 = pl.gb_bytes ? (float *)(ws + pl.gin_bytes + pl.gw_bytes) : (float *)bp->grad_bias;
  uint32_t *maxima = (uint32_t *)(ws + pl.gin_bytes + pl.gw_bytes + pl.gb_bytes);  // [0] |d|, [1] |mask|
  unsigned char *xt = ws + pl.gin_bytes + pl.gw_bytes + pl.gb_bytes + pl.mx_bytes;
  unsigned char *gT = xt + pl.xt_bytes;
  unsigned char *wT = gT + pl.gt_bytes;
  unsigned char *D = wT + pl.wt_bytes;
  unsigned char *col = D + pl.d_bytes;
  const long off_total = (long)g.N * g.DG * 2 * g.taps * plane_out, mask_total = off_total / 2;
  float *poff = (float *)(col + pl.col_bytes);
  float *pmask = poff + (long)pl.parts * off_total;
  float *wpart = (float *)(col + pl.col_bytes + pl.part_bytes);
  const bool wgemm = pl.wgemm;
  unsigned char *gpad = (unsigned char *)wpart + pl.wpart_bytes;
  const bool gemm = pl.gemm;

  if (bp->grad_input) {
    hipLaunchKernelGGL(fill_zero_kernel<float>, dim3(blocks_for(n_in / 4 + 1)), dim3(256), 0, st, gin32, n_in);  // (16 bytes per thread)
    check();
  }
  if (bp->grad_weight) {
    hipLaunchKernelGGL(fill_zero_kernel<float>, dim3(blocks_for(n_w / 4 + 1)), dim3(256), 0, st, gw32, n_w);
    check();
  }

  if (gemm || wgemm) {
    {  // zero-bordered copy of the input in 32-byte records (what the scatter kernel reads per corner)
      constexpr int EPV = 16 / (int)sizeof(E);
      const int n_pchunks = (g.H * g.W + 32 * EPV - 1) / (32 * EPV);
      hipLaunchKernelGGL((relayout_vec_kernel<E, true, 32>), dim3((unsigned)((long)g.N * (g.Cin / KC) * n_pchunks)),
                         dim3(256), 0, st, g, (const E *)p->input, (E *)xt, n_pchunks);
      check();
    }
    if (gemm) {  // pixel-major grad_output, transposed weights
      Geom gg = g;
      gg.Cin = g.Cout;
      gg.H = g.Ho;
      gg.W = g.Wo;
      constexpr int EPV = 16 / (int)sizeof(E);
      const int o_pchunks = (int)((plane_out + 32 * EPV - 1) / (32 * EPV));
      hipLaunchKernelGGL((relayout_vec_kernel<E, false>), dim3((unsigned)((long)g.N * (g.Cout / KC) * o_pchunks)),
                         dim3(256), 0, st, gg, (const E *)bp->grad_output, (E *)gT, o_pchunks);
      check();
      if (pl.mx_bytes) {
        hipLaunchKernelGGL(fill_zero_kernel<uint32_t>, dim3(1), dim3(256), 0, st, maxima, 2L);
        check();
        if (p->mask) {
          const long n_mask = (long)g.N * g.DG * g.taps * plane_out;
          hipLaunchKernelGGL(absmax_kernel<E>, dim3(std::min(blocks_for(n_mask / 8), 256)), dim3(256), 0, st,
                             (const E *)p->mask, n_mask, maxima + 1);
          check();
        }
      }
      const long wtotal = (long)g.G * pl.M_pad * g.cout_g;
      hipLaunchKernelGGL(pack_weight_t_kernel<E>, dim3(blocks_for(wtotal)), dim3(256), 0, st, g,
                         (const E *)p->weight, (E *)wT, pl.M_pad, wtotal);
      check();
    }
    if (wgemm && pl.gpad_bytes) {
      const long rows = (long)g.N * g.Cout;
      hipLaunchKernelGGL(pad_rows_kernel<E>, dim3(blocks_for(rows * pl.P_pad)), dim3(256), 0, st,
                         (const E *)bp->grad_output, (E *)gpad, rows, (int)plane_out, pl.P_pad);
      check();
    }
    if (wgemm && pl.P_pad > plane_out) {
      const long rows = (long)pl.n_chunk * g.taps * g.Cin;
      hipLaunchKernelGGL(zero_col_pad_kernel<E>, dim3(blocks_for(rows * (pl.P_pad - plane_out))), dim3(256), 0, st,
                         (E *)col, rows, (int)plane_out, pl.P_pad);
      check();
    }
    for (int n0 = 0; n0 < g.N; n0 += pl.n_chunk) {
      const int nb = std::min(pl.n_chunk, g.N - n0);
      if (gemm) {
        ColGradArgs ca;
        ca.wT = wT;
        ca.gT = gT;
        ca.D = D;
        ca.P = (int)plane_out;
        ca.px_tiles = (int)((plane_out + pl.cg_tile - 1) / pl.cg_tile);
        ca.m_tiles = pl.M_pad / pl.cg_tile;
        ca.M = g.taps * g.cin_g;
        ca.M_pad = pl.M_pad;
        ca.cin_g = g.cin_g;
        ca.cout_g = g.cout_g;
        ca.taps = g.taps;
        ca.G = g.G;
        ca.Cin = g.Cin;
        ca.Cout = g.Cout;
        ca.kslabs = g.cout_g / KC;
        ca.n0 = n0;
        ca.dmax = pl.mx_bytes ? maxima : nullptr;
        ca.total = (long)nb * g.G * ca.px_tiles * ca.m_tiles;
        if (pl.cg_tile == kCgTileBig)
          hipLaunchKernelGGL((bwd_colgrad_kernel<E, kCgTileBig>), dim3((unsigned)((ca.total + 7) / 8 * 8)),
                             dim3(2 * kCgTileBig), 0, st, ca);
        else
          hipLaunchKernelGGL((bwd_colgrad_kernel<E, kCgTile>), dim3((unsigned)((ca.total + 7) / 8 * 8)),
                             dim3(2 * kCgTile), 0, st, ca);
        check();
      }
      BwdScatterArgs sa;
      sa.g = g;
      sa.xt = xt;
      sa.om = om;
      sa.D = gemm ? D : nullptr;
      sa.gin32 = gin32;
      sa.goff = bp->grad_offset;
      sa.gmask = bp->grad_mask;
      sa.col = wgemm ? col : nullptr;
      sa.P_pad = pl.P_pad;
      sa.tiles_x = (g.Wo + kScTW - 1) / kScTW;
      sa.tiles_y = (g.Ho + kScTH - 1) / kScTH;
      sa.R = pl.sR;
      sa.WH = pl.sWH;
      sa.WW = pl.sWW;
      sa.n0 = n0;
      sa.parts = gemm ? pl.parts : 1;
      sa.poff = poff;
      sa.pmask = pmask;
      sa.off_total = off_total;
      sa.mask_total = mask_total;
      sa.dmax = maxima;
      sa.mmax = p->mask ? maxima + 1 : nullptr;
      const long sblocks = (long)nb * g.DG * sa.tiles_y * sa.tiles_x;
      {
        // 16-bit tensors: 32-bit fixed-point window (needs the maxima the data path computes;
        // a columns-only call adds nothing to the window); fp32 tensors: doubles
        constexpr bool k16 = sizeof(E) == 2;
        using WT = typename std::conditional<k16, int32_t, double>::type;
        constexpr int CHB = k16 ? 16 : 8;
        const dim3 sgrid((unsigned)sblocks, (unsigned)sa.parts);
        auto launch = [&](auto chv) {
          constexpr int CHS = decltype(chv)::value;
          if (gemm && wgemm)
            hipLaunchKernelGGL((bwd_scatter_kernel<E, CHS, WT, true, true>), sgrid, dim3(256), 0, st, sa);
          else if (gemm)
            hipLaunchKernelGGL((bwd_scatter_kernel<E, CHS, WT, true, false>), sgrid, dim3(256), 0, st, sa);
          else
            hipLaunchKernelGGL((bwd_scatter_kernel<E, CHS, WT, false, true>), sgrid, dim3(256), 0, st, sa);
        };
        if (pl.sCH == CHB)
          launch(std::integral_constant<int, CHB>());
        else
          launch(std::integral_constant<int, CHB / 2>());
      }
      check();
      if (wgemm) {
        WGradArgs wa;
        wa.gout = pl.gpad_bytes ? (const void *)gpad : bp->grad_output;
        wa.a_pitch = pl.gpad_bytes ? pl.P_pad : plane_out;
        wa.col = col;
        wa.part = wpart;
        wa.P = (int)plane_out;
        wa.P_pad = pl.P_pad;
        wa.ksteps = (int)(pl.P_pad / KC);
        wa.nb = nb;
        wa.n0 = n0;
        wa.M = g.taps * g.cin_g;
        wa.cin_g = g.cin_g;
        wa.cout_g = g.cout_g;
        wa.taps = g.taps;
        wa.G = g.G;
        wa.Cin = g.Cin;
        wa.Cout = g.Cout;
        const int wtile = pl.w_tile;
        wa.co_tiles = (g.cout_g + wtile - 1) / wtile;
        wa.m_tiles = (wa.M + wtile - 1) / wtile;
        const long tiles = (long)g.G * wa.co_tiles * wa.m_tiles;
        wa.splits = pl.w_splits;
        wa.total = tiles * wa.splits;
        if (wtile == kCgTileBig)
          hipLaunchKernelGGL((bwd_wgrad_kernel<E, kCgTileBig>), dim3((unsigned)((wa.total + 7) / 8 * 8)),
                             dim3(2 * kCgTileBig), 0, st, wa);
        else
          hipLaunchKernelGGL((bwd_wgrad_kernel<E, kCgTile>), dim3((unsigned)((wa.total + 7) / 8 * 8)),
                             dim3(2 * kCgTile), 0, st, wa);
        check();
        hipLaunchKernelGGL(wgrad_reduce_kernel, dim3(blocks_for(n_w / 4 + 1)), dim3(256), 0, st, wpart, gw32, wa.splits,
                           g.cin_g, g.taps, n_w);
        check();
      }
    }
  }

  if (bp->grad_input) {
    if (gemm) {
      if (pl.parts > 1) {
        hipLaunchKernelGGL(combine_parts_kernel<E>, dim3(blocks_for(off_total / 4 + 1)), dim3(256), 0, st, poff,
                           (E *)bp->grad_offset, off_total, pl.parts);
        check();
        if (bp->grad_mask) {
          hipLaunchKernelGGL(combine_parts_kernel<E>, dim3(blocks_for(mask_total / 4 + 1)), dim3(256), 0, st, pmask,
                             (E *)bp->grad_mask, mask_total, pl.parts);
          check();
        }
      }
    } else if (pl.tiled) {
      BwdDataTiledArgs da;
      da.g = g;
      da.input = p->input;
      da.om = om;
      da.weight = p->weight;
      da.gout = bp->grad_output;
      da.gin32 = gin32;
      da.goff = bp->grad_offset;
      da.gmask = bp->grad_mask;
      da.tiles_x = (g.Wo + kBwdTile - 1) / kBwdTile;
      da.tiles_y = (g.Ho + kBwdTile - 1) / kBwdTile;
      da.R = pl.R;
      da.WH = pl.WH;
      da.WW = pl.WW;
      const long blocks = (long)g.N * g.DG * da.tiles_y * da.tiles_x;
      hipLaunchKernelGGL(bwd_data_tiled_kernel<E>, dim3((unsigned)blocks), dim3(256), 0, st, da);
      check();
    } else {
      const int rows = g.N * g.DG * g.taps;  // (image, deformable group, tap)
      const dim3 grid((unsigned)((plane_out + 255) / 256), (unsigned)std::min(rows, 65535));
      hipLaunchKernelGGL(bwd_data_kernel<E>, grid, dim3(256), 0, st, g, (const E *)p->input, om,
                         (const E *)p->weight, (const E *)bp->grad_output, gin32,
                         (E *)bp->grad_offset, (E *)bp->grad_mask, rows);
      check();
    }
    if (pl.gin_bytes) {
      hipLaunchKernelGGL(round_kernel<E>, dim3(blocks_for(n_in / 8 + 1)), dim3(256), 0, st, gin32,  // (8 elements per thread)
                         (E *)bp->grad_input, n_in);
      check();
    }
  }
  if (bp->grad_weight) {
    if (!wgemm) {
      BwdWeightArgs wa;
      wa.g = g;
      wa.input = p->input;
      wa.om = om;
      wa.gout = bp->grad_output;
      wa.gw32 = gw32;
      wa.k_tiles = (g.cin_g * g.taps + 63) / 64;
      wa.co_tiles = (g.cout_g + 255) / 256;
      wa.px_chunks = (int)((plane_out + 63) / 64);
      const long tiles = (long)wa.k_tiles * wa.co_tiles * g.G;
      const long work = (long)g.N * wa.px_chunks;
      wa.splits = (int)std::max<long>(1, std::min<long>(work, (4L * num_cus() + tiles - 1) / tiles));
      wa.g_vec_ok = (plane_out % (16 / (long)sizeof(E)) == 0) && (((uintptr_t)bp->grad_output % 16) == 0);
      hipLaunchKernelGGL(bwd_weight_kernel<E>, dim3((unsigned)tiles, (unsigned)wa.splits), dim3(256), 0,
                         st, wa);
      check();
    }
    if (pl.gw_bytes) {
      hipLaunchKernelGGL(round_kernel<E>, dim3(blocks_for(n_w / 8 + 1)), dim3(256), 0, st, gw32,
                         (E *)bp->grad_weight, n_w);
      check();
    }
  }
  if (bp->grad_bias) {
    hipLaunchKernelGGL(fill_zero_kernel<float>, dim3(blocks_for(g.Cout)), dim3(256), 0, st, gb32, (long)g.Cout);
    check();
    const int runs = (int)((plane_out + kBiasRun - 1) / kBiasRun);
    const int splits = (int)std::min<long>((long)g.N * runs, 64);
    hipLaunchKernelGGL(bwd_bias_kernel<E>, dim3(g.Cout, splits), dim3(256), 0, st, g,
                       (const E *)bp->grad_output, gb32, runs, splits);
    check();
    if (pl.gb_bytes) {
      hipLaunchKernelGGL(round_kernel<E>, dim3(blocks_for(g.Cout)), dim3(256), 0, st, gb32,
                         (E *)bp->grad_bias, (long)g.Cout);
      check();
    }
  }
  return rc;
}

// Double precision: grad_input by atomics into the zeroed tensor, everything else
// has one owner; no workspace.
int run_backward_f64(const mdcn_bwd_params *bp, const Geom &g, hipStream_t st) {
  const mdcn_params *p = &bp->conv;
  const long plane_out = (long)g.Ho * g.Wo;
  auto blocks_for = [](long n) { return (int)std::max<long>(1, std::min<long>((n + 255) / 256, 1L << 20)); };
  int rc = MDCN_OK;
  auto check = [&]() { if (hipGetLastError() != hipSuccess) rc = MDCN_ERR_LAUNCH; };
  if (bp->grad_input) {
    const long n_in = (long)g.N * g.Cin * g.H * g.W;
    hipLaunchKernelGGL(f64_zero_kernel, dim3(blocks_for(n_in)), dim3(256), 0, st, (double *)bp->grad_input, n_in);
    check();
    const long total = (long)g.N * g.DG * g.taps * plane_out;
    hipLaunchKernelGGL(f64_bwd_data_kernel, dim3(blocks_for(total)), dim3(256), 0, st, g, (const double *)p->input,
                       (const double *)p->offset, (const double *)p->mask, (const double *)p->weight,
                       (const double *)bp->grad_output, (double *)bp->grad_input, (double *)bp->grad_offset,
                       (double *)bp->grad_mask, total);
    check();
  }
  if (bp->grad_weight) {
    const long n_w = (long)g.Cout * g.cin_g * g.taps;
    hipLaunchKernelGGL(f64_bwd_weight_kernel, dim3((unsigned)std::min<long>(n_w, 1L << 20)), dim3(256), 0, st, g,
                       (const double *)p->input, (const double *)p->offset, (const double *)p->mask,
                       (const double *)bp->grad_output, (double *)bp->grad_weight);
    check();
  }
  if (bp->grad_bias) {
    hipLaunchKernelGGL(f64_bwd_bias_kernel, dim3((unsigned)std::min(g.Cout, 65535)), dim3(256), 0, st, g,
                       (const double *)bp->grad_output, (double *)bp->grad_bias);
    check();
  }
  return rc;
}

int check_bwd(const mdcn_bwd_params *bp, Geom *g, bool need_ptrs) {
  if (!bp) return MDCN_ERR_NULL;
  const mdcn_params *p = &bp->conv;
  int rc = check_params(p, g, false);
  if (rc != MDCN_OK) return rc;
  if (p->input_nhwc) return MDCN_ERR_PATH;
  if (!need_ptrs) return MDCN_OK;
  if (!p->input || !p->offset || !p->weight || !bp->grad_output) return MDCN_ERR_NULL;
  // grad_input and the offset/mask gradients come out of one kernel
  const bool data = bp->grad_input != nullptr;
  if (data != (bp->grad_offset != nullptr)) return MDCN_ERR_NULL;
  if (p->mask ? (data != (bp->grad_mask != nullptr)) : (bp->grad_mask != nullptr)) return MDCN_ERR_NULL;
  if ((uint64_t)g->N * g->DG * g->taps > 0x7fffffffull) return MDCN_ERR_TOO_LARGE;
  if (p->dtype == MDCN_F64 && forced_fused(p->path)) return MDCN_ERR_PATH;
  if (forced_fused(p->path)) {  // asked for the tiled kernels: the shape must allow them
    BwdPlan pl;
    make_bwd_plan(bp, *g, &pl);
    if ((data && !pl.tiled && !pl.gemm) || (!data && bp->grad_weight && !pl.wgemm)) return MDCN_ERR_PATH;
  }
  return MDCN_OK;
}

}  // namespace

extern "C" {

int mdcn_abi_version(void) { return MDCN_ABI_VERSION; }

void mdcn_set_pass_limits(uint64_t forward_bytes, uint64_t backward_bytes) {
  g_fwd_pass_bytes.store(forward_bytes ? std::min<uint64_t>(forward_bytes, kMaxXtBytes) : kMaxXtBytes);
  g_bwd_pass_bytes.store(backward_bytes ? std::min<uint64_t>(backward_bytes, kBwdColGradCap) : kBwdColGradCap);
}

const char *mdcn_status_string(int status) {
  switch (status) {
    case MDCN_OK: return "ok";
    case MDCN_ERR_NULL: return "a required pointer is NULL";
    case MDCN_ERR_SHAPE: return "invalid shape (non-positive size or channels not divisible by groups)";
    case MDCN_ERR_DTYPE: return "unsupported dtype";
    case MDCN_ERR_WORKSPACE: return "workspace missing, misaligned or too small";
    case MDCN_ERR_PATH: return "shape not covered by the fused path";
    case MDCN_ERR_TOO_LARGE: return "tensor too large for 32-bit device offsets";
    case MDCN_ERR_LAUNCH: return "HIP launch error";
    case MDCN_ERR_SCRATCH_LIMIT: return "call needs more scratch than the library's built-in buffer holds";
    default: return "unknown status";
  }
}

int mdcn_output_size(const mdcn_params *p, int32_t *Ho, int32_t *Wo) {
  Geom g;
  const int rc = check_params(p, &g, false);
  if (rc != MDCN_OK) return rc;
  if (Ho) *Ho = g.Ho;
  if (Wo) *Wo = g.Wo;
  return MDCN_OK;
}

int mdcn_fused_eligible(const mdcn_params *p) {
  Geom g;
  if (check_params(p, &g, false) != MDCN_OK) return 0;
  return fused_ok(p, g) ? 1 : 0;
}

const char *mdcn_forward_kernels(const mdcn_params *p) {
  Geom g;
  if (check_params(p, &g, false) != MDCN_OK) return "";
  Plan pl;
  if (make_plan(p, g, &pl) != MDCN_OK) return "";
  if (p->dtype == MDCN_F64) return "f64_forward_kernel";
  if (!pl.fused) return "direct_kernel";
  if (!uses_fused2(p, g, pl)) return "fused_kernel";
  const size_t es = elem_size(p->dtype);
  const long plane_out = (long)g.Ho * g.Wo;
  const bool out_vec_ok = (plane_out % (long)(16 / es) == 0) && (((uintptr_t)p->output % 16) == 0);
  const long total_px = (long)std::min(pl.n_chunk, g.N) * plane_out;
  const long n3 = wide_tiles_of_call(p, g, pl, total_px, out_vec_ok);
  if (n3 == 0) return "fused2_kernel";
  return total_px - n3 * kF3PT > 0 ? "fused3_kernel+fused2_kernel" : "fused3_kernel";
}

size_t mdcn_workspace_bytes(const mdcn_params *p) {
  Geom g;
  if (check_params(p, &g, false) != MDCN_OK) return 0;
  Plan pl;
  if (make_plan(p, g, &pl) != MDCN_OK) return 0;
  return pl.fused ? pl.xt_bytes + pl.wp_bytes + pl.cut_bytes : 0;
}

int mdcn_forward(const mdcn_params *p, void *hip_stream) {
  return run(p, hip_stream, nullptr);
}

int mdcn_forward_noalloc(const mdcn_params *p, void *hip_stream) {
  Geom g;
  int rc = check_params(p, &g, true);
  if (rc != MDCN_OK) return rc;
  Plan pl;
  rc = make_plan(p, g, &pl);
  if (rc != MDCN_OK) return rc;
  if (pl.xt_bytes + pl.wp_bytes > (size_t)MDCN_NOALLOC_SCRATCH_BYTES) return MDCN_ERR_SCRATCH_LIMIT;
  void *ptr = nullptr;
  rc = scratch_of_current_device(&ptr);
  if (rc != MDCN_OK) return rc;
  mdcn_params q = *p;
  q.workspace = ptr;
  q.workspace_bytes = (size_t)MDCN_NOALLOC_SCRATCH_BYTES;
  return run(&q, hip_stream, nullptr);
}

int mdcn_forward_timed(const mdcn_params *p, void *hip_stream, float ms[4]) {
  if (!ms) return MDCN_ERR_NULL;
  return run(p, hip_stream, ms);
}

size_t mdcn_pack_workspace_bytes(const mdcn_pack_params *pp) {
  Geom g;
  if (!pp || check_params(&pp->conv, &g, false) != MDCN_OK) return 0;
  Plan pl;
  if (make_pack_plan(pp, g, &pl) != MDCN_OK) return 0;
  return pl.xt_bytes + pl.wp_bytes + pl.owp_bytes + pl.raw_bytes + pl.cut_bytes;
}

int mdcn_pack_forward(const mdcn_pack_params *pp, void *hip_stream) {
  if (!pp) return MDCN_ERR_NULL;
  return run(&pp->conv, hip_stream, nullptr, pp);
}

size_t mdcn_backward_workspace_bytes(const mdcn_bwd_params *bp) {
  Geom g;
  if (check_bwd(bp, &g, false) != MDCN_OK) return 0;
  BwdPlan pl;
  make_bwd_plan(bp, g, &pl);
  return pl.total();
}

int mdcn_backward(const mdcn_bwd_params *bp, void *hip_stream) {
  Geom g;
  const int rc = check_bwd(bp, &g, true);
  if (rc != MDCN_OK) return rc;
  BwdPlan pl;
  make_bwd_plan(bp, g, &pl);
  const size_t need = pl.total();
  const mdcn_params *p = &bp->conv;
  if (need > 0 && (!p->workspace || p->workspace_bytes < need || ((uintptr_t)p->workspace % kAlign) != 0))
    return MDCN_ERR_WORKSPACE;
  hipStream_t st = (hipStream_t)hip_stream;
  switch (p->dtype) {
    case MDCN_F64: return run_backward_f64(bp, g, st);
    case MDCN_F32: return run_backward_typed<float>(bp, g, pl, st);
    case MDCN_F16: return run_backward_typed<f16_t>(bp, g, pl, st);
    default: return run_backward_typed<bf16_t>(bp, g, pl, st);
  }
}

int mdcn_pack_forward_timed(const mdcn_pack_params *pp, void *hip_stream, float ms[5]) {
  if (!pp || !ms) return MDCN_ERR_NULL;
  return run(&pp->conv, hip_stream, ms, pp);
}

}  // extern "C"
