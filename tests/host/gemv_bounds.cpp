// CPU bounds harness for the single-row Linear launches.  For every weight type x matrix shape x prologue /
// epilogue combination x occupancy the launcher can see, it takes the launch plan the library itself computes
// (caten_amd/csrc/gemv_plan.h, the code launch_gemv runs) and walks every workgroup, wavefront and lane of that
// plan through a transcription of the kernels' index arithmetic (k_gemv / gemv_ring / coop_prologue / coop_fold of
// caten_amd/csrc/gemv_kernels.h), asserting for each access that the pointer it dereferences exists and that the
// bytes lie inside the operand: quant plane, scale plane, input vector(s), gamma / beta, bias / residual / fold
// terms, output, argmax partials, the LDS staging buffer and the `red` array.  Prints the number of launches and
// accesses checked and every violation; exit status 1 if there is any.
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <string>

#include "../../caten_amd/csrc/gemv_plan.h"

using namespace cthip;

static long long g_checked = 0, g_violations = 0, g_launches = 0;
static std::string g_case;

struct Region {
  const char *name;
  bool present;
  long long bytes;
};
static void touch(const Region &r, long long off, long long n, const char *what) {
  g_checked++;
  if (!r.present) {
    if (g_violations++ < 40) printf("VIOLATION %s: %s dereferences %s, which is null\n", g_case.c_str(), what, r.name);
    return;
  }
  if (off < 0 || off + n > r.bytes || (off % n) != 0) {
    if (g_violations++ < 40) printf("VIOLATION %s: %s touches %s[%lld..%lld) of %lld bytes\n", g_case.c_str(), what, r.name, off, off + n, r.bytes);
  }
}

struct Case {
  int type, rows, cols, m, pro;
  bool fold, bias, bias0, residual, argmax, pair;
  int cus, occ;
  int full_cols, col0;  // the launch covers columns [col0, col0 + cols) of a matrix full_cols wide (0 = the whole matrix)
};

static void walk(const Case &c) {
  GemvPlanIn in = {};
  in.type = c.type; in.rows = c.rows; in.cols = c.cols; in.m = c.m; in.pro = c.pro; in.fold = c.fold; in.bias = c.bias;
  in.bias0 = c.bias0; in.residual = c.residual; in.argmax = c.argmax; in.compute_units = c.cus; in.occupancy = c.occ;
  GemvPlan p = gemv_plan(in);
  char buf[256];
  snprintf(buf, sizeof(buf), "type %d (%d,%d) m %d pro %d fold %d bias %d bias0 %d resid %d argmax %d pair %d cus %d occ %d", c.type, c.rows, c.cols,
           c.m, c.pro, c.fold, c.bias, c.bias0, c.residual, c.argmax, c.pair, c.cus, c.occ);
  g_case = buf;
  if (p.shape < 0 || p.error) return;  // generic fallback / refused: not these kernels
  g_launches++;
  const GemvShape &v = gemv_shapes()[p.shape];
  const int G = v.G, KC = v.KC, XPC = gemv_xpc(c.type), RPW = 64 / G;
  const int PD = p.kernel == GEMV_K_SMALL ? 1 : PD_OF_T(c.type, KC);
  const bool QUANT = c.type == CTHIP_Q8_0 || c.type == CTHIP_Q4_0;
  bool fold = c.fold, bias = c.bias;
  if (p.unfold) fold = false, bias = false;
  const bool swiglu = c.pro == CTHIP_PRO_SWIGLU, layernorm = c.pro == CTHIP_PRO_LAYERNORM;
  const bool folded = c.pro == CTHIP_PRO_RMSNORM || (layernorm && fold);
  const bool coop = p.stage;
  // a column slice: the launcher's pointer offsets, row pitches and gate / up distance (launch_gemv in linear.hip)
  const int full = c.full_cols ? c.full_cols : c.cols;
  const long long q0 = 16ll * (c.col0 / XPC), d0 = 2ll * (c.col0 >> 5), x0 = 4ll * c.col0, upo = full;
  const int in_cols = swiglu ? 2 * full : full;
  const long long x_stride = in_cols, out_rows = c.pair ? c.rows / 2 : c.rows, y_stride = out_rows;
  const long long row_bytes = c.type == CTHIP_Q8_0 ? full : c.type == CTHIP_Q4_0 ? full / 2 : c.type == CTHIP_F16 ? 2ll * full : 4ll * full;
  Region Q = {"quant plane", true, row_bytes * c.rows}, D = {"scale plane", QUANT, 2ll * (full / 32) * c.rows};
  Region X = {"x", true, 4 * x_stride * c.m}, NG = {"norm_g", c.pro == CTHIP_PRO_LAYERNORM || c.pro == CTHIP_PRO_RMSNORM, 4ll * c.cols};
  Region NB = {"norm_b", layernorm, 4ll * c.cols}, B = {"bias", bias, 4ll * c.rows}, R = {"residual", c.residual, 4 * y_stride * c.m};
  Region FS = {"fold_s", fold, 4ll * c.rows}, Y = {"y", true, 4 * y_stride * c.m}, AM = {"argmax partials", c.argmax, 4ll * 16384};
  Region LDS = {"LDS staging buffer", p.lds > 0, (long long)p.lds}, RED = {"red", true, 4 * 24};
  const int nchunks = c.cols / XPC, nrq = (c.rows + RPW - 1) / RPW, n4 = c.cols >> 2;
  const int nthr = (int)p.block, wpb = nthr >> 6, total_waves = (int)p.grid_x * wpb;
  const int scales_per_row = full >> 5;
  const long long row_chunks = full / XPC;
  const bool ring = PD > 1;
  if (ring && nthr != 256) { g_violations++; printf("VIOLATION %s: the looping kernel is compiled for 256 threads, launched with %d\n", g_case.c_str(), nthr); }
  const bool epi_kernel = p.kernel == GEMV_K_LOOP_EPI, direct_kernel = p.kernel == GEMV_K_LOOP_DIRECT;
  for (int m = 0; m < c.m; m++)
    for (unsigned bx = 0; bx < p.grid_x; bx++)
      for (int tid = 0; tid < nthr; tid++) {
        const int lane = tid & 63, g = lane / G, l = lane % G, wave = (int)bx * wpb + (tid >> 6);
        const long long xoff = 4 * x_stride * m + x0;
        auto tile = [&](int rq, const char *what) {
          int row = rq * RPW + g;
          row = row < c.rows ? row : c.rows - 1;
          for (int j = 0; j < KC; j++) {
            const int cc = l + G * j;
            if (cc >= nchunks) continue;  // reads the zero block
            touch(Q, q0 + ((long long)row * row_chunks + cc) * 16, 16, what);
            if (QUANT) touch(D, d0 + 2 * ((long long)row * scales_per_row + (c.type == CTHIP_Q8_0 ? (cc >> 1) : cc)), 2, what);
          }
          return row;
        };
        auto epi_operands = [&](int row, bool in_ring) {
          if (in_ring) {  // gemv_ring: one request by the first three lanes; `any` must exist
            if (!bias && !c.residual && !fold) { g_violations++; printf("VIOLATION %s: the ring's epilogue request has no operand\n", g_case.c_str()); return; }
            if (bias) touch(B, 4ll * row, 4, "epilogue request");
            if (c.residual) touch(R, 4 * (y_stride * m + row), 4, "epilogue request");
            if (fold) touch(FS, 4ll * row, 4, "epilogue request");
          } else {
            if (bias) touch(B, 4ll * row, 4, "bias");
            if (c.residual) touch(R, 4 * (y_stride * m + row), 4, "residual");
            if (fold) touch(FS, 4ll * row, 4, "fold term");
          }
        };
        auto store = [&](int rq) {
          const int row = rq * RPW + g;
          if (row >= c.rows) return;
          if (c.pair) { if (l == 0 && (g & 1) == 0) touch(Y, 4 * (y_stride * m + (row >> 1)), 4, "paired store"); }
          else if (l == 0) touch(Y, 4 * (y_stride * m + row), 4, "store");
        };
        auto x_slice = [&](bool from_lds) {
          for (int j = 0; j < KC; j++) {
            const int cc = l + G * j;
            if (cc >= nchunks) continue;
            for (int t = 0; t < XPC / 4; t++) {
              if (from_lds) touch(LDS, 4ll * (cc * XPC + 4 * t), 16, "staged slice");
              else touch(X, xoff + 4ll * (cc * XPC + 4 * t), 16, "input slice");
            }
          }
        };
        auto gamma_slice = [&]() {
          for (int j = 0; j < KC; j++) {
            const int cc = l + G * j;
            if (cc >= nchunks) continue;
            for (int t = 0; t < XPC / 4; t++) touch(NG, 4ll * (cc * XPC + 4 * t), 16, "gamma slice");
          }
        };
        auto coop_prologue = [&](bool normalise) {
          if (!swiglu && !normalise) { for (int i = tid; i < n4; i += nthr) touch(X, xoff + 16ll * i, 16, "copy"), touch(LDS, 16ll * i, 16, "copy"); return; }
          if (swiglu) { for (int i = tid; i < n4; i += nthr) touch(X, xoff + 16ll * i, 16, "gate"), touch(X, xoff + 4ll * upo + 16ll * i, 16, "up"), touch(LDS, 16ll * i, 16, "swiglu"); return; }
          for (int i = tid; i < n4; i += nthr) {
            touch(X, xoff + 16ll * i, 16, "norm input");
            touch(NG, 16ll * i, 16, "norm gamma");
            if (layernorm) touch(NB, 16ll * i, 16, "norm beta");
            touch(LDS, 16ll * i, 16, "normalised");
          }
          touch(RED, 4 * (tid >> 6), 4, "red");
          if (wpb > 8) { g_violations++; printf("VIOLATION %s: %d wavefronts overflow red\n", g_case.c_str(), wpb); }
        };
        if (!ring) {
          // ---- k_gemv, one tile in flight ----
          const int rq0 = wave < nrq ? wave : nrq - 1;
          epi_operands(tile(rq0, "first tile"), false);
          if (folded && layernorm) touch(X, xoff, 4, "pivot");
          if (coop) {
            if (folded) {
              for (int i = tid; i < n4; i += nthr) touch(X, xoff + 16ll * i, 16, "fold input"), touch(NG, 16ll * i, 16, "fold gamma"), touch(LDS, 16ll * i, 16, "fold stage");
              touch(RED, 4 * (tid >> 6), 4, "red"), touch(RED, 4 * (8 + (tid >> 6)), 4, "red");
            } else coop_prologue(c.pro != CTHIP_PRO_NONE);
          }
          x_slice(coop);
          if (folded && !coop) gamma_slice();
          for (int base = wave; base < nrq; base += total_waves) {
            store(base);
            if (base + total_waves < nrq) epi_operands(tile(base + total_waves, "next tile"), false);
          }
        } else {
          // ---- gemv_ring ----
          const bool direct = direct_kernel && coop && layernorm && !fold && n4 <= 4 * 256;
          const bool early = coop && (folded || swiglu || c.pro == CTHIP_PRO_NONE || direct);
          if (early) {
            for (int k = 0; k < 4; k++) {
              int i = tid + k * 256;
              i = i < n4 ? i : n4 - 1;
              touch(X, xoff + 16ll * i, 16, "early input");
              if (swiglu) touch(X, xoff + 4ll * upo + 16ll * i, 16, "early up");
              else if ((layernorm || folded) && NG.present) touch(NG, 16ll * i, 16, "early gamma");
              if (direct_kernel && direct) touch(NB, 16ll * i, 16, "early beta");
            }
          } else if (!coop) {
            x_slice(false);
            if (!QUANT && folded) gamma_slice();
          }
          const int own = wave < nrq ? wave : nrq - 1;
          auto request = [&](int rq) { const int row = tile(rq, "ring tile"); if (epi_kernel) epi_operands(row, true); };
          request(wave < nrq ? wave : own);
          if (coop && !early) coop_prologue(true);
          if (early) {
            for (int i = tid; i < n4; i += 256) {
              if (i >= tid + 4 * 256) { touch(X, xoff + 16ll * i, 16, "late input"); if (swiglu) touch(X, xoff + 4ll * upo + 16ll * i, 16, "late up"); else if (NG.present) touch(NG, 16ll * i, 16, "late gamma"); }
              touch(LDS, 16ll * i, 16, "stage");
            }
            touch(RED, 4 * (tid >> 6), 4, "red"), touch(RED, 4 * (8 + (tid >> 6)), 4, "red"), touch(RED, 4 * (16 + (tid >> 6)), 4, "red");
          }
          if (coop) x_slice(true);
          for (int pp = 1; pp < PD; pp++) { const int rq = wave + pp * total_waves; request(rq < nrq ? rq : own); }
          if (folded && !coop && QUANT) gamma_slice();
          const int stride = PD * total_waves;
          int base = wave;
          for (; base + stride < nrq; base += stride)
            for (int pp = 0; pp < PD; pp++) { const int rq = base + pp * total_waves; store(rq); const int nxt = rq + stride; request(nxt < nrq ? nxt : rq); }
          for (int pp = 0; pp < PD; pp++) { const int rq = base + pp * total_waves; if (rq < nrq) store(rq); }
        }
        if (c.argmax && lane == 0) touch(AM, 4ll * wave, 4, "argmax partial");
      }
}

// The wide-row kernel (caten_amd/csrc/gemv_wide.hip: input vector in LDS, rows streamed as tiles of nc rounds): the
// plan is the library's (gemv_wide_plan), the walk a transcription of k_gemv_wide's requests, LDS traffic and stores.
static void walk_wide(int type, int rows, int cols, int m_rows, int pro, bool bias, bool residual, bool gamma, int cus) {
  const GemvWidePlan p = gemv_wide_plan(type, rows, cols, cus);
  char buf[200];
  snprintf(buf, sizeof(buf), "wide type %d (%d,%d) m %d pro %d bias %d resid %d gamma %d cus %d", type, rows, cols, m_rows, pro, bias, residual, gamma, cus);
  g_case = buf;
  if (!p.ok) return;
  g_launches++;
  const bool Q4 = type == CTHIP_Q4_0, swiglu = pro == CTHIP_PRO_SWIGLU, rms = pro == CTHIP_PRO_RMSNORM;
  const int XPC = gemv_xpc(type), F4 = XPC / 4, NC = p.nc, RW = p.rw, PD = 12 / (NC * RW), tpr = p.tpr;
  const int nchunks = cols / XPC, n4 = cols >> 2, spr = cols >> 5;
  const long long x_stride = swiglu ? 2ll * cols : cols, y_stride = rows;
  const bool QUANT = Q4 || type == CTHIP_Q8_0;
  const long long row_bytes = Q4 ? cols / 2 : type == CTHIP_Q8_0 ? cols : type == CTHIP_F16 ? 2ll * cols : 4ll * cols;
  Region Q = {"quant plane", true, row_bytes * rows}, D = {"scale plane", QUANT, 2ll * spr * rows};
  Region X = {"x", true, 4 * x_stride * m_rows}, NG = {"norm_g", rms && gamma, 4ll * cols}, B = {"bias", bias, 4ll * rows};
  Region R = {"residual", residual, 4 * y_stride * m_rows}, Y = {"y", true, 4 * y_stride * m_rows};
  Region LDS = {"LDS", true, 4ll * (long long)p.lds_floats};
  const long long csum0 = 4ll * cols, red0 = csum0 + (Q4 ? 4ll * nchunks : 0);
  if (p.lds_floats * 4 > kGemvWideMaxLdsBytes || p.block != 512 || NC * tpr * 64 < nchunks || 12 % (NC * RW) || (RW != 1 && RW != 2)) {
    g_violations++;
    printf("VIOLATION %s: plan nc %d tpr %d lds %zu block %u\n", g_case.c_str(), NC, tpr, p.lds_floats, p.block);
    return;
  }
  auto slot = [&](int i) { return (i & ~(F4 - 1)) | ((i ^ (i / F4)) & (F4 - 1)); };
  const int total_waves = (int)p.grid * 8;
  for (int m = 0; m < m_rows; m++)
    for (unsigned bx = 0; bx < p.grid; bx++)
      for (int tid = 0; tid < 512; tid++) {
        const int lane = tid & 63, wv = tid >> 6, wave = (int)bx * 8 + wv;
        const long long xoff = 4 * x_stride * m;
        const int npairs = (rows + RW - 1) / RW;
        const int pairs_w = wave < npairs ? (npairs - wave + total_waves - 1) / total_waves : 0, nt = pairs_w * tpr;
        int rq_pair = wave < npairs ? wave : npairs - 1, rq_grp = 0, rq_left = nt;
        auto request = [&]() {
          const int row0 = RW * rq_pair, row1 = row0 + RW - 1 < rows ? row0 + RW - 1 : rows - 1;
          for (int k = 0; k < NC; k++) {
            const int c = (rq_grp * NC + k) * 64 + lane;
            if (c >= nchunks) continue;  // reads the zero block
            for (int row : {row0, row1}) {
              touch(Q, ((long long)row * nchunks + c) * 16, 16, "wide tile");
              if (QUANT) touch(D, 2 * ((long long)row * spr + (Q4 ? c : c >> 1)), 2, "wide scale");
            }
          }
          const int er = (lane & 2) ? row1 : row0;
          const bool want_r = lane & 1;
          if (want_r ? residual : bias) touch(want_r ? R : B, want_r ? 4 * (y_stride * m + er) : 4ll * er, 4, "wide epilogue request");
          else if (bias) touch(B, 4ll * er, 4, "wide epilogue request");
          else if (residual) touch(R, 4 * (y_stride * m + er), 4, "wide epilogue request");
          if (rq_left > 1) { rq_left--; if (++rq_grp == tpr) { rq_grp = 0; rq_pair += total_waves; } }
        };
        request();
        for (int i = tid; i < n4; i += 512) {
          touch(X, xoff + 16ll * i, 16, "wide input");
          if (swiglu) touch(X, xoff + 4ll * cols + 16ll * i, 16, "wide up");
          else if (rms && gamma) touch(NG, 16ll * i, 16, "wide gamma");
          touch(LDS, 16ll * slot(i), 16, "wide stage");
        }
        if (rms) touch(LDS, red0 + 4 * wv, 4, "wide red");
        if (Q4)
          for (int c = tid; c < nchunks; c += 512) {
            for (int t = 0; t < F4; t++) touch(LDS, 16ll * (F4 * c + (t ^ (c & (F4 - 1)))), 16, "wide chunk sum read");
            touch(LDS, csum0 + 4ll * c, 4, "wide chunk sum");
          }
        for (int pp = 1; pp < PD; pp++) request();
        int cs_pair = wave, cs_grp = 0;
        auto consume = [&]() {
          for (int k = 0; k < NC; k++) {
            const int c = (cs_grp * NC + k) * 64 + lane, cl = c < nchunks ? c : nchunks - 1;
            for (int t = 0; t < F4; t++) touch(LDS, 16ll * (F4 * cl + (t ^ (cl & (F4 - 1)))), 16, "wide x read");
            if (Q4) touch(LDS, csum0 + 4ll * cl, 4, "wide chunk sum read");
          }
          if (++cs_grp == tpr) {
            const int row0 = RW * cs_pair;
            if (row0 >= rows) { g_violations++; printf("VIOLATION %s: stores row %d\n", g_case.c_str(), row0); }
            if (lane == 0) touch(Y, 4 * (y_stride * m + row0), 4, "wide store");
            if (RW > 1 && lane == 1 && row0 + 1 < rows) touch(Y, 4 * (y_stride * m + row0 + 1), 4, "wide store");
            cs_grp = 0;
            cs_pair += total_waves;
          }
        };
        int t = 0;
        for (; t + PD <= nt; t += PD)
          for (int pp = 0; pp < PD; pp++) { consume(); request(); }
        for (int pp = 0; pp < PD; pp++)
          if (t + pp < nt) consume();
      }
}

// the split-K reduction + norm pass: whatever (row length, shares, rows) the launcher accepts, the instantiation it
// picks covers the whole row (lanes x float4 per lane x 4 floats) and keeps its shares within the register budget
static void check_reduce_norm_plans() {
  for (int n = 4; n <= 8192; n += 4)
    for (int nparts = 1; nparts <= 16; nparts++)
      for (long long rows : {1ll, 512ll, 2048ll, 2049ll, 4096ll, 100000ll}) {
        const ReduceNormPlan p = reduce_norm_plan(n, nparts, rows);
        if (!p.ok) continue;
        g_checked++;
        const int lanes = p.wide ? 256 : 64;
        const bool inst = p.wide ? (p.vpl == 1 || p.vpl == 2 || p.vpl == 4 || p.vpl == 8) : (p.vpl >= 1 && p.vpl <= 8 && p.vpl != 5 && p.vpl != 7);
        if (lanes * p.vpl * 4 < n || !inst || p.vpl * p.nz > 64 || p.nz < nparts)
          if (g_violations++ < 40) printf("VIOLATION reduce + norm: n %d shares %d rows %lld -> wide %d vpl %d nz %d\n", n, nparts, rows, p.wide, p.vpl, p.nz);
      }
}

// "shape TYPE ROWS COLS [TYPE ROWS COLS ...]": only these Linears (TYPE = the library's code: 0 fp32, 1 fp16, 2 Q4_0,
// 8 Q8_0), with every prologue and the flag sets a decoder launches -- for a model size outside the table below
static int walk_given_shapes(int argc, char **argv) {
  for (int i = 2; i + 2 < argc; i += 3) {
    const int type = atoi(argv[i]), rows = atoi(argv[i + 1]), cols = atoi(argv[i + 2]);
    const int xpc = gemv_xpc(type);
    if (rows <= 0 || cols <= 0 || xpc <= 0 || cols % xpc || ((type == CTHIP_Q8_0 || type == CTHIP_Q4_0) && cols % 32)) {
      printf("gemv bounds: shape %d %d %d is not a Linear of the library\n", type, rows, cols);
      return 2;
    }
    for (int pro : {(int)CTHIP_PRO_NONE, (int)CTHIP_PRO_SWIGLU, (int)CTHIP_PRO_RMSNORM})
      for (int flags = 0; flags < 4; flags++)
        for (int mm : {1, 3}) {
          if (mm == 3 && flags != 3) continue;
          walk_wide(type, rows, cols, mm, pro, flags & 1, flags & 2, flags & 1, 256);
        }
    walk_wide(type, rows, cols, 1, CTHIP_PRO_NONE, true, true, false, 64);
    int width = 0;
    const int nsl = gemv_pick_shape(type, cols) < 0 ? gemv_slices(type, cols, &width) : 0;
    if (nsl > 0) {  // what launch_gemv queues for a row wider than any variant: no norm, no activation, no argmax
      for (int pro : {(int)CTHIP_PRO_NONE, (int)CTHIP_PRO_SWIGLU})
        for (int flags : {0, 2, 8, 10})
          for (int mm : {1, 3})
            for (int sl = 0; sl < nsl; sl++) {
              Case c = {};
              c.type = type; c.rows = rows; c.m = mm; c.pro = pro; c.cus = 256; c.occ = 2;
              c.full_cols = cols; c.col0 = sl * width; c.cols = sl + 1 < nsl ? width : cols - c.col0;
              c.bias = sl == 0 && (flags & 2);
              c.residual = sl > 0 || (flags & 8);
              walk(c);
            }
      continue;
    }
    for (int pro = 0; pro <= 3; pro++)
      for (int flags : {0, 2, 8, 10, 11, 15, 17, 24}) {
        Case c = {};
        c.type = type; c.rows = rows; c.cols = cols; c.m = 1; c.pro = pro;
        c.fold = (flags & 1) && pro == CTHIP_PRO_LAYERNORM;
        if ((flags & 1) && pro != CTHIP_PRO_LAYERNORM) continue;
        if ((flags & 4) && !c.fold) continue;
        c.bias = (flags & 2) || c.fold;
        c.bias0 = c.fold && (flags & 4);
        c.residual = flags & 8;
        c.argmax = flags & 16;
        c.cus = 256; c.occ = 2;
        walk(c);
      }
    if (rows % 2 == 0) {
      Case c = {};
      c.type = type; c.rows = rows; c.cols = cols; c.m = 1; c.pro = CTHIP_PRO_RMSNORM; c.pair = true; c.cus = 256; c.occ = 2;
      const int sh = gemv_pick_shape(type, cols);
      if (sh >= 0 && gemv_shapes()[sh].G <= 32) walk(c);
    }
  }
  printf("gemv bounds: %lld launches, %lld accesses checked, %lld violations\n", g_launches, g_checked, g_violations);
  return g_violations ? 1 : 0;
}

int main(int argc, char **argv) {
  if (argc > 1 && !strcmp(argv[1], "shape")) return walk_given_shapes(argc, argv);
  check_reduce_norm_plans();
  // default: a few seconds (every shape, the flag combinations thinned out on the large ones); "full": everything
  const bool full = argc > 1 && !strcmp(argv[1], "full");
  const int types[] = {CTHIP_Q8_0, CTHIP_Q4_0, CTHIP_F32, CTHIP_F16};
  // widths: each variant's exact width, one chunk less, the smallest, and the model widths
  const int rowsv[] = {1, 2, 3, 5, 17, 64, 767, 768, 2304, 3072, 5003, 32000, 50257};
  for (int type : types) {
    const int xpc = gemv_xpc(type);
    std::vector<int> colsv = {xpc, 2 * xpc, 768, 1024, 1280, 1600, 2048, 3072, 4096, 5632, 8192};
    for (const GemvShape &s : gemv_shapes())
      if (s.type == type) colsv.push_back(s.G * s.KC * xpc), colsv.push_back((s.G * s.KC - 1) * xpc);
    for (int cols : colsv) {
      if (cols <= 0 || cols % xpc || ((type == CTHIP_Q8_0 || type == CTHIP_Q4_0) && cols % 32)) continue;
      for (int rows : rowsv) {
        if ((long long)rows * cols > 50257ll * 1024) continue;
        for (int pro = 0; pro <= 3; pro++)
          for (int flags = 0; flags < 32; flags++) {
            Case c = {};
            c.type = type; c.rows = rows; c.cols = cols; c.m = (rows < 100 ? 3 : 1); c.pro = pro;
            c.fold = (flags & 1) && pro == CTHIP_PRO_LAYERNORM;
            c.bias = (flags & 2) || c.fold;  // a folded launch always carries W.beta + bias
            c.bias0 = c.fold && (flags & 4);
            c.residual = flags & 8;
            c.argmax = (flags & 16) && c.m == 1;
            if ((flags & 16) && c.m != 1) continue;
            if ((flags & 4) && !c.fold) continue;
            if ((flags & 1) && pro != CTHIP_PRO_LAYERNORM) continue;
            // very large walks: one occupancy only
            const long long cost = (long long)rows * cols;
            const bool big = cost > 8000000;
            // (flags: 1 fold, 2 bias, 4 the Linear's own bias beside the fold, 8 residual, 16 argmax; 17 = what lm_head launches)
            if (!full && cost > 20000 && flags != 0 && flags != 2 && flags != 11 && flags != 15 && flags != 17 && flags != 24) continue;
            if (!full && cost > 1000000 && (pro == 3 || (flags != 0 && flags != 11 && flags != 17))) continue;
            if (!full && cost > 20000000 && !(pro == 1 && flags == 17) && !(pro == 0 && flags == 0)) continue;
            for (int occ = 1; occ <= (big ? 2 : 4); occ++) {
              if (big && (flags & ~25)) continue;
              if (!full && cost > 20000 && occ != 2) continue;
              c.cus = 256; c.occ = occ;
              walk(c);
            }
            if (!big && (full || cost <= 20000)) { c.cus = 64; c.occ = 2; walk(c); }
          }
        // gate / up pairs: two rows per wavefront, even row count, no residual
        if (rows % 2 == 0) {
          Case c = {};
          c.type = type; c.rows = rows; c.cols = cols; c.m = 1; c.pro = CTHIP_PRO_RMSNORM; c.pair = true; c.cus = 256; c.occ = 2;
          const int sh = gemv_pick_shape(type, cols);
          if (sh >= 0 && gemv_shapes()[sh].G <= 32) walk(c);
        }
      }
    }
  }
  // the wide-row kernel on widths around its tile sizes, and rows fewer / more than wavefronts
  for (int type : {CTHIP_Q8_0, CTHIP_Q4_0, CTHIP_F16, CTHIP_F32})
    for (int cols : {64, 96, 2048, 2080, 4096, 5504, 6144, 8192, 8224, 11008})
      for (int rows : {1, 7, 513, 4100})
        for (int pro : {(int)CTHIP_PRO_NONE, (int)CTHIP_PRO_SWIGLU, (int)CTHIP_PRO_RMSNORM})
          walk_wide(type, rows, cols, rows < 100 ? 3 : 1, pro, rows & 1, cols & 64, true, 256);
  printf("gemv bounds: %lld launches, %lld accesses checked, %lld violations\n", g_launches, g_checked, g_violations);
  return g_violations ? 1 : 0;
}
