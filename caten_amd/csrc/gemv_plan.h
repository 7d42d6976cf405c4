// How a single-row Linear launch is laid out: which kernel variant, how many workgroups of how many threads, how
// much LDS, which of the kernel's modes.  Pure host arithmetic (no HIP): launch_gemv (linear.hip) executes the plan,
// and the bounds harness under tests/ walks the same plan thread by thread on the CPU.
#pragma once
#include <stddef.h>

#include <vector>

#include "../../include/caten_hip.h"

namespace cthip {

// the (lanes per row, 16-byte chunks per lane) shapes instantiated per weight type (gemv_*.hip)
#define GEMV_SHAPES_Q8(V) V(CTHIP_Q8_0, 16, 1) V(CTHIP_Q8_0, 16, 2) V(CTHIP_Q8_0, 16, 3) V(CTHIP_Q8_0, 16, 4) V(CTHIP_Q8_0, 32, 3) \
  V(CTHIP_Q8_0, 32, 4) V(CTHIP_Q8_0, 64, 3) V(CTHIP_Q8_0, 64, 4) V(CTHIP_Q8_0, 64, 6) V(CTHIP_Q8_0, 64, 8)
#define GEMV_SHAPES_Q4(V) V(CTHIP_Q4_0, 16, 1) V(CTHIP_Q4_0, 16, 2) V(CTHIP_Q4_0, 32, 2) V(CTHIP_Q4_0, 64, 1) V(CTHIP_Q4_0, 64, 2) \
  V(CTHIP_Q4_0, 64, 3) V(CTHIP_Q4_0, 64, 4)
#define GEMV_SHAPES_F32(V) V(CTHIP_F32, 16, 4) V(CTHIP_F32, 64, 1) V(CTHIP_F32, 64, 2) V(CTHIP_F32, 64, 3) V(CTHIP_F32, 64, 4) \
  V(CTHIP_F32, 64, 6) V(CTHIP_F32, 64, 8) V(CTHIP_F32, 64, 12) V(CTHIP_F32, 64, 16) V(CTHIP_F32, 64, 24)
#define GEMV_SHAPES_F16(V) V(CTHIP_F16, 16, 2) V(CTHIP_F16, 64, 1) V(CTHIP_F16, 64, 2) V(CTHIP_F16, 64, 3) V(CTHIP_F16, 64, 4) \
  V(CTHIP_F16, 64, 6) V(CTHIP_F16, 64, 8) V(CTHIP_F16, 64, 12)

// looping launches keep about 12 sixteen-byte loads per lane in flight; the widest 4-bit variants (96+ input floats per
// lane in registers) keep two tiles, which leaves room for a second wavefront per SIMD
#define PD_OF_T(T, KC) (KC >= 12 ? 1 : (KC >= 6 || ((T) == CTHIP_Q4_0 && KC >= 3)) ? 2 : 4)

// tiles a wavefront of the looping kernel keeps in flight
inline int gemv_ring_depth(int type, int KC) { return PD_OF_T(type, KC); }
struct GemvShape {
  int type, G, KC;
};
inline const std::vector<GemvShape> &gemv_shapes() {
  static const std::vector<GemvShape> all = {
#define GEMV_SHAPE_ENTRY(T, G, KC) {T, G, KC},
      GEMV_SHAPES_Q8(GEMV_SHAPE_ENTRY) GEMV_SHAPES_Q4(GEMV_SHAPE_ENTRY) GEMV_SHAPES_F32(GEMV_SHAPE_ENTRY) GEMV_SHAPES_F16(GEMV_SHAPE_ENTRY)
#undef GEMV_SHAPE_ENTRY
  };
  return all;
}

inline int gemv_xpc(int type) {  // input elements one 16-byte chunk multiplies
  switch (type) {
    case CTHIP_Q8_0: return 16;
    case CTHIP_Q4_0: return 32;
    case CTHIP_F16: return 8;
    default: return 4;
  }
}

// index into gemv_shapes() of the variant that covers `cols` with the least idle lanes, or -1
inline int gemv_pick_shape(int type, int cols) {
  const int xpc = gemv_xpc(type);
  if (cols % xpc) return -1;
  const int nchunks = cols / xpc;
  int best = -1, best_waste = 1 << 30;
  const std::vector<GemvShape> &all = gemv_shapes();
  for (int i = 0; i < (int)all.size(); i++) {
    const GemvShape &v = all[i];
    if (v.type != type || v.G * v.KC < nchunks) continue;
    const int waste = v.G * v.KC - nchunks;
    if (waste < best_waste || (waste == best_waste && best >= 0 && v.G < all[best].G)) {
      best = i;
      best_waste = waste;
    }
  }
  return best;
}

// Rows wider than any register-resident variant (FFN down-projections of 7B-class models and up) are multiplied as
// column slices of equal width, one launch each: slice 0 carries the epilogue, every later one adds its products to
// what is there.  Returns the number of slices (0 = the width needs none, or cannot be cut on block boundaries into
// widths that variants cover) and their width (the last slice has what is left).
inline int gemv_slices(int type, long long cols, int *width) {
  const int xpc = gemv_xpc(type);
  const int unit = (type == CTHIP_Q8_0 || type == CTHIP_Q4_0) ? 32 : xpc;  // a slice starts on a block scale
  if (cols <= 0 || cols > 0x7fffffff || cols % unit) return 0;
  int maxc = 0;
  for (const GemvShape &sh : gemv_shapes())
    if (sh.type == type && sh.G * sh.KC * xpc > maxc) maxc = sh.G * sh.KC * xpc;
  if (!maxc || cols <= maxc) return 0;
  for (int n = (int)((cols + maxc - 1) / maxc); n <= 64; n++) {
    const int wdt = (int)(((cols + n - 1) / n + unit - 1) / unit * unit);
    const long long last = cols - (long long)wdt * (n - 1);
    if (wdt <= maxc && last > 0 && gemv_pick_shape(type, wdt) >= 0 && gemv_pick_shape(type, (int)last) >= 0) {
      *width = wdt;
      return n;
    }
  }
  return 0;
}

struct GemvPlanIn {
  int type, rows, cols, m;
  int pro;            // CTHIP_PRO_*
  bool fold;          // a LayerNorm folded through the product (fold_s given)
  bool bias, bias0, residual, argmax;
  int compute_units;
  int occupancy;      // resident 256-thread workgroups of the looping kernel per compute unit (from the runtime)
};

enum GemvKernelKind { GEMV_K_SMALL, GEMV_K_LOOP, GEMV_K_LOOP_EPI, GEMV_K_LOOP_DIRECT };

struct GemvPlan {
  int shape = -1;      // index into gemv_shapes(); -1 = no register-resident variant (generic fallback)
  unsigned grid_x = 0, grid_y = 0, block = 0;
  size_t lds = 0;
  bool stage = false;  // the workgroup stages the input vector in LDS once
  bool unfold = false; // the launch drops the fold terms and normalises the staged vector itself
  GemvKernelKind kernel = GEMV_K_SMALL;
  int nwaves = 0;
  const char *error = nullptr;
};

inline GemvPlan gemv_plan(const GemvPlanIn &in) {
  GemvPlan p;
  p.shape = gemv_pick_shape(in.type, in.cols);
  p.grid_y = (unsigned)in.m;
  if (p.shape < 0) return p;
  const GemvShape &v = gemv_shapes()[p.shape];
  const int rpw = 64 / v.G;
  const int nrq = (in.rows + rpw - 1) / rpw;
  bool fold = in.fold, bias = in.bias, residual = in.residual;
  const bool folded = (in.pro == CTHIP_PRO_RMSNORM) || (in.pro == CTHIP_PRO_LAYERNORM && fold);
  const bool quantised = in.type == CTHIP_Q8_0 || in.type == CTHIP_Q4_0;
  // The input vector goes through LDS once per workgroup when it must be normalised or gated first, or when it is
  // large next to a weight tile (a 4-bit tile multiplies 8 input bytes per weight byte): then four wavefronts share
  // one copy and every wavefront takes several tiles.  Quantised launches with a folded norm stage at every size.
  p.stage = (in.pro != CTHIP_PRO_NONE && !folded) || (in.type == CTHIP_Q4_0 && in.cols >= 1024) || (folded && (in.cols >= 2048 || quantised));
  p.lds = p.stage ? sizeof(float) * (size_t)in.cols : 0;
  if (p.lds > 64 * 1024) {
    p.error = "input features exceed the LDS staging buffer";
    return p;
  }
  bool small, direct = false;
  if (!p.stage && nrq <= 2048) {
    // small matrices are pure latency: one tile per wavefront, one wavefront per workgroup, spread over as many
    // compute units as there are tiles
    small = true;
    p.block = 64;
    p.grid_x = (unsigned)nrq;
  } else if (p.stage && nrq <= in.compute_units * 3) {
    // one tile per wavefront, as many wavefronts per workgroup (at most three) as leave about one workgroup per
    // compute unit: fewer workgroups repeat the staging less, but idle units stream nothing
    small = true;
    int wpb = (nrq + in.compute_units - 1) / in.compute_units;
    wpb = wpb < 1 ? 1 : wpb > 3 ? 3 : wpb;
    p.block = 64u * (unsigned)wpb;
    p.grid_x = (unsigned)((nrq + wpb - 1) / wpb);
  } else {
    // larger matrices: at least one wavefront per SIMD, more (up to what the register budget keeps resident) once
    // every wavefront has four tiles
    small = false;
    const int occ = in.occupancy > 0 ? in.occupancy : 1;
    p.block = 256;
    const int base = in.compute_units * 4;
    // unstaged: a wavefront per tile up to three resident wavefronts per SIMD
    int wanted = p.stage ? (nrq + 3) / 4 : nrq;
    if (wanted < base) wanted = base;
    const int cap = base * (p.stage || occ < 3 ? occ : 3);
    if (wanted > cap) wanted = cap;
    // staged launches pay the input staging once per workgroup: whole workgroups per compute unit, two when there
    // is work for more than one
    if (p.stage && wanted > base && occ >= 2) wanted = 2 * base;
    const int iters = (nrq + wanted - 1) / wanted;
    // every resident wavefront slot is used even if some wavefronts then loop once more than others
    const int waves = wanted < nrq ? wanted : nrq;
    p.grid_x = (unsigned)((waves + 3) / 4);
    // the ring requests all its slots unconditionally: a wavefront with a single tile takes the kernel without one
    if (iters == 1) small = true;
    // a looping launch normalises the staged vector itself rather than carrying the fold terms: two more operands
    // per row in the weight ring hold the stream up more than the second barrier of the staging costs
    if (!small && p.stage && in.pro == CTHIP_PRO_LAYERNORM && fold && !in.bias0 && !residual && in.cols <= 4096) {
      p.unfold = true;
      fold = false;
      bias = false;
    }
    direct = !small && p.stage && in.pro == CTHIP_PRO_LAYERNORM && !fold && !bias && !residual && in.cols <= 4096;
  }
  p.nwaves = (int)(p.grid_x * (p.block / 64));
  const bool epi = bias || residual || fold;
  p.kernel = small ? GEMV_K_SMALL : epi ? GEMV_K_LOOP_EPI : direct ? GEMV_K_LOOP_DIRECT : GEMV_K_LOOP;
  // what the kernels assume of their launch
  if (p.kernel != GEMV_K_SMALL && p.block != 256) p.error = "a looping launch must have 256 threads per workgroup";
  if (p.block > 512) p.error = "more than eight wavefronts per workgroup";
  return p;
}

// The wide-row kernel (gemv_wide.hip): the input vector lives in LDS instead of in registers, so a row may be as
// wide as LDS holds and the registers a lane needs do not grow with the width.  A round = 64 chunks (one per lane);
// a tile = nc rounds of a pair of neighbouring rows, requested together; a row = tpr tiles.  lds counts floats: the staged vector, one
// sum per chunk for 4-bit weights, 16 for the reduction of a norm's statistics.
struct GemvWidePlan {
  bool ok = false;
  int nc = 0, tpr = 0, rw = 1;  // rw: rows a wavefront streams together (1 or 2)
  unsigned grid = 0, block = 512;
  size_t lds_floats = 0;
};
constexpr size_t kGemvWideMaxLdsBytes = 150 * 1024;
inline GemvWidePlan gemv_wide_plan(int type, long long rows, long long cols, int compute_units) {
  GemvWidePlan p;
  if (type != CTHIP_Q8_0 && type != CTHIP_Q4_0 && type != CTHIP_F16 && type != CTHIP_F32) return p;
  const int xpc = gemv_xpc(type);
  const bool quant = type == CTHIP_Q8_0 || type == CTHIP_Q4_0;
  if (rows <= 0 || rows > 0x7fffffff || cols < 64 || cols % (quant ? 32 : xpc) || cols > 0x7fffffff) return p;
  const int nchunks = (int)(cols / xpc);
  p.lds_floats = (size_t)cols + (type == CTHIP_Q4_0 ? (size_t)nchunks : 0) + 16;
  if (p.lds_floats * 4 > kGemvWideMaxLdsBytes) return p;
  const int rounds = (nchunks + 63) / 64;
  // (six 16-byte requests of weights per lane and tile: 3, 2 or 1 rounds of two rows)
  // (4-bit chunks are 32 inputs wide: with more than one round's inputs between LDS and the arithmetic the kernel
  // does not fit the 128 registers that let four wavefronts share a SIMD)
  p.nc = type == CTHIP_Q4_0 ? 1 : rounds % 3 == 0 ? 3 : rounds % 2 == 0 ? 2 : 1;
  p.tpr = rounds / p.nc;
  // two workgroups per compute unit where LDS holds two copies of the vector; never more wavefronts than rows
  const long long per_cu = p.lds_floats * 4 * 2 <= kGemvWideMaxLdsBytes ? 2 : 1;
  long long grid = (long long)compute_units * per_cu;
  // rows go in pairs where the pairs still fill every wavefront slot of the launch
  p.rw = (rows + 1) / 2 >= grid * 8 ? 2 : 1;
  const long long need = ((rows + p.rw - 1) / p.rw + 7) / 8;
  if (grid > need) grid = need;
  p.grid = (unsigned)(grid < 1 ? 1 : grid);
  p.ok = true;
  return p;
}

// How the split-K reduction + norm pass (rowops.hip) lays a row out: `wide` = four wavefronts per row instead of
// one; `vpl` = the float4-per-lane count of the kernel instantiation chosen (one of 1,2,3,4,6,8 narrow / 1,2,4,8
// wide); `nz` = the share bucket.  ok is false when no instantiation covers the row.
struct ReduceNormPlan {
  bool ok, wide;
  int vpl, nz;
};
inline ReduceNormPlan reduce_norm_plan(int n, int nparts, long long rows) {
  ReduceNormPlan p = {false, false, 0, 0};
  if (n < 4 || n % 4 || n > 8192 || nparts < 1 || nparts > 16) return p;
  p.nz = nparts <= 2 ? 2 : nparts <= 4 ? 4 : nparts <= 8 ? 8 : 16;
  const int v1 = (n / 4 + 63) / 64, v4 = (n / 4 + 255) / 256;
  // the shares of a row are all requested at once: VPL x NZ float4 per lane have to stay in registers
  const bool narrow_fits = v1 * p.nz <= 32 && v1 <= 8, wide_fits = v4 * p.nz <= 32 && v4 <= 8;
  if (!narrow_fits && !wide_fits) return p;
  // four wavefronts per row where one cannot hold the row's shares, and for a prompt's few rows of some width: the
  // pass is a single memory round trip, and four times the threads ask for it four times as wide
  p.wide = !narrow_fits || (wide_fits && rows <= 2048 && n >= 512);
  if (p.wide) p.vpl = v4 <= 1 ? 1 : v4 <= 2 ? 2 : v4 <= 4 ? 4 : 8;
  else p.vpl = v1 <= 4 ? v1 : v1 <= 6 ? 6 : 8;
  p.ok = true;
  return p;
}

}  // namespace cthip
