// Memory-bound fused items over the last axis (softmax, LayerNorm, RMSNorm and
// LayerNorm->softmax), elementwise activations, embedding gather, argmax, RoPE
// and the KV-cached attention of batch-1 decode.
//
// Row ops: one wavefront owns one row and keeps it in registers (VPL float4 per
// lane, 128-bit coalesced loads/stores), so every row is read once and written
// once; the reductions are 64-lane shuffles, no LDS.  Rows longer than
// 64*4*8 = 2048 floats fall back to one 256-thread block per row that re-reads
// the row through L2.
#include <type_traits>
#include "common.h"
#include "gemv_plan.h"

namespace cthip {

enum { ROW_SOFTMAX = 0, ROW_LAYERNORM = 1, ROW_RMSNORM = 2, ROW_LN_SOFTMAX = 3 };

struct RowArgs {
  float *y;
  const float *x;
  const float *g;
  const float *b;
  float eps;
  int64_t rows;
  int n;
};

template <int MODE, int VPL>
__global__ __launch_bounds__(256) void k_rowop(RowArgs a) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (row >= a.rows) return;
  const int n = a.n;
  const int n4 = n >> 2;  // n % 4 == 0 on this path
  const float4 *__restrict__ xp = (const float4 *)(a.x + row * n);
  float4 *__restrict__ yp = (float4 *)(a.y + row * n);
  float v[VPL][4];
  bool ok[VPL];
  // every request of the row (and of gamma / beta) goes out before anything is used, none behind a branch: lanes
  // past the end repeat the last chunk and drop it.  A load inside `if (ok)` is waited for at the end of that block,
  // which turns a row into one memory round trip per chunk.
  constexpr bool NORM = MODE == ROW_LAYERNORM || MODE == ROW_RMSNORM || MODE == ROW_LN_SOFTMAX;
  float4 t[VPL], gm[NORM ? VPL : 1], bt[NORM ? VPL : 1];
#pragma unroll
  for (int j = 0; j < VPL; j++) {
    const int c = lane + 64 * j;
    ok[j] = c < n4;
    t[j] = xp[ok[j] ? c : n4 - 1];
  }
  if (NORM) {
    const float4 *g4 = a.g ? (const float4 *)a.g : xp, *b4 = a.b ? (const float4 *)a.b : xp;  // xp: unused stand-in
#pragma unroll
    for (int j = 0; j < VPL; j++) {
      const int c = lane + 64 * j;
      gm[NORM ? j : 0] = g4[ok[j] ? c : n4 - 1];
      bt[NORM ? j : 0] = b4[ok[j] ? c : n4 - 1];
    }
  }
#pragma unroll
  for (int j = 0; j < VPL; j++) {
    v[j][0] = ok[j] ? t[j].x : 0.0f;
    v[j][1] = ok[j] ? t[j].y : 0.0f;
    v[j][2] = ok[j] ? t[j].z : 0.0f;
    v[j][3] = ok[j] ? t[j].w : 0.0f;
  }
  if (MODE == ROW_LAYERNORM || MODE == ROW_RMSNORM || MODE == ROW_LN_SOFTMAX) {
    const float inv_n = 1.0f / (float)n;
    float mean = 0.0f;
    if (MODE != ROW_RMSNORM) {
      float s = 0.0f;
#pragma unroll
      for (int j = 0; j < VPL; j++)
#pragma unroll
        for (int e = 0; e < 4; e++) s += v[j][e];
      mean = wave_sum(s) * inv_n;
    }
    float q = 0.0f;
#pragma unroll
    for (int j = 0; j < VPL; j++)
#pragma unroll
      for (int e = 0; e < 4; e++) {
        float d = ok[j] ? v[j][e] - mean : 0.0f;
        v[j][e] = d;
        q = fmaf(d, d, q);
      }
    const float rstd = 1.0f / sqrtf(wave_sum(q) * inv_n + a.eps);
#pragma unroll
    for (int j = 0; j < VPL; j++) {
      if (ok[j]) {
        const float4 g = a.g ? gm[NORM ? j : 0] : make_float4(1.f, 1.f, 1.f, 1.f);
        const float4 b = a.b ? bt[NORM ? j : 0] : make_float4(0.f, 0.f, 0.f, 0.f);
        v[j][0] = v[j][0] * rstd * g.x + b.x;
        v[j][1] = v[j][1] * rstd * g.y + b.y;
        v[j][2] = v[j][2] * rstd * g.z + b.z;
        v[j][3] = v[j][3] * rstd * g.w + b.w;
      }
    }
  }
  if (MODE == ROW_SOFTMAX || MODE == ROW_LN_SOFTMAX) {
    float m = -INFINITY;
#pragma unroll
    for (int j = 0; j < VPL; j++)
#pragma unroll
      for (int e = 0; e < 4; e++)
        if (ok[j]) m = fmaxf(m, v[j][e]);
    m = wave_max(m);
    float s = 0.0f;
#pragma unroll
    for (int j = 0; j < VPL; j++)
#pragma unroll
      for (int e = 0; e < 4; e++) {
        float ex = ok[j] ? ct_exp(v[j][e] - m) : 0.0f;
        v[j][e] = ex;
        s += ex;
      }
    const float inv = 1.0f / wave_sum(s);
#pragma unroll
    for (int j = 0; j < VPL; j++)
#pragma unroll
      for (int e = 0; e < 4; e++) v[j][e] *= inv;
  }
#pragma unroll
  for (int j = 0; j < VPL; j++)
    if (ok[j]) yp[lane + 64 * j] = make_float4(v[j][0], v[j][1], v[j][2], v[j][3]);
}

// Split-K reduction, residual update and the following norm in one pass over the rows (prompt batches): a row-split
// Linear whose reduction axis was shared among `nparts` workgroups per tile leaves raw partial tiles; the next thing
// that happens to its output is the residual add and a LayerNorm / RMSNorm.  One wavefront per row:
//   x = sum_z parts[z][row] (ascending z, as k_splitk_reduce adds them) + bias + resid   -> xout[row]
//   y[row] = norm(x)                                                                    (arithmetic of k_rowop)
struct ReduceNormArgs {
  float *y, *xout;
  const float *parts;
  int nparts;
  int64_t part_stride;  // floats between two partial matrices
  const float *bias, *resid, *g, *b;
  float eps;
  int64_t rows;
  int n;
};

template <int MODE, int VPL, int NZ>
__global__ __launch_bounds__(256) void k_reduce_norm(ReduceNormArgs a) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (row >= a.rows) return;
  const int n = a.n, n4 = n >> 2;
  float4 t[VPL][NZ], bs[VPL], rs[VPL], gm[VPL], bt[VPL];
  bool ok[VPL];
  // every request first, none behind a branch: shares past nparts repeat share 0 and are dropped
#pragma unroll
  for (int j = 0; j < VPL; j++) {
    const int c = lane + 64 * j;
    ok[j] = c < n4;
    const int cc = ok[j] ? c : n4 - 1;
#pragma unroll
    for (int z = 0; z < NZ; z++) t[j][z] = ((const float4 *)(a.parts + (int64_t)(z < a.nparts ? z : 0) * a.part_stride + row * n))[cc];
    bs[j] = ((const float4 *)(a.bias ? a.bias : a.parts))[cc];
    rs[j] = ((const float4 *)((a.resid ? a.resid : a.parts) + row * n))[cc];
    gm[j] = ((const float4 *)(a.g ? a.g : a.parts))[cc];
    bt[j] = ((const float4 *)(a.b ? a.b : a.parts))[cc];
  }
  float v[VPL][4];
#pragma unroll
  for (int j = 0; j < VPL; j++) {
    float x[4] = {t[j][0].x, t[j][0].y, t[j][0].z, t[j][0].w};
#pragma unroll
    for (int z = 1; z < NZ; z++)
      if (z < a.nparts) x[0] += t[j][z].x, x[1] += t[j][z].y, x[2] += t[j][z].z, x[3] += t[j][z].w;
    if (a.bias) x[0] += bs[j].x, x[1] += bs[j].y, x[2] += bs[j].z, x[3] += bs[j].w;
    if (a.resid) x[0] += rs[j].x, x[1] += rs[j].y, x[2] += rs[j].z, x[3] += rs[j].w;
    if (ok[j]) ((float4 *)(a.xout + row * n))[lane + 64 * j] = make_float4(x[0], x[1], x[2], x[3]);
#pragma unroll
    for (int e = 0; e < 4; e++) v[j][e] = ok[j] ? x[e] : 0.0f;
  }
  const float inv_n = 1.0f / (float)n;
  float mean = 0.0f;
  if (MODE != ROW_RMSNORM) {
    float s = 0.0f;
#pragma unroll
    for (int j = 0; j < VPL; j++)
#pragma unroll
      for (int e = 0; e < 4; e++) s += v[j][e];
    mean = wave_sum(s) * inv_n;
  }
  float q = 0.0f;
#pragma unroll
  for (int j = 0; j < VPL; j++)
#pragma unroll
    for (int e = 0; e < 4; e++) {
      float d = ok[j] ? v[j][e] - mean : 0.0f;
      v[j][e] = d;
      q = fmaf(d, d, q);
    }
  const float rstd = 1.0f / sqrtf(wave_sum(q) * inv_n + a.eps);
#pragma unroll
  for (int j = 0; j < VPL; j++) {
    if (ok[j]) {
      const float4 g = a.g ? gm[j] : make_float4(1.f, 1.f, 1.f, 1.f);
      const float4 b = a.b ? bt[j] : make_float4(0.f, 0.f, 0.f, 0.f);
      ((float4 *)(a.y + row * n))[lane + 64 * j] = make_float4(v[j][0] * rstd * g.x + b.x, v[j][1] * rstd * g.y + b.y,
                                                             v[j][2] * rstd * g.z + b.z, v[j][3] * rstd * g.w + b.w);
    }
  }
}

// true if the fused pass can take this shape (otherwise the caller reduces and normalises in two launches)
// The same with four wavefronts per row (rows too wide, or with too many shares, for one wavefront's registers):
// thread t of the row's 256 owns float4 t + 256 j, the row statistics meet in LDS.
template <int MODE, int VPL, int NZ>
__global__ __launch_bounds__(256) void k_reduce_norm_wide(ReduceNormArgs a) {
  __shared__ float red[2][4];
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int64_t row = blockIdx.x;
  const int n = a.n, n4 = n >> 2;
  float4 t[VPL][NZ], bs[VPL], rs[VPL], gm[VPL], bt[VPL];
  bool ok[VPL];
  // every request first, none behind a branch: shares past nparts repeat share 0 and are dropped
#pragma unroll
  for (int j = 0; j < VPL; j++) {
    const int c = tid + 256 * j;
    ok[j] = c < n4;
    const int cc = ok[j] ? c : n4 - 1;
#pragma unroll
    for (int z = 0; z < NZ; z++) t[j][z] = ((const float4 *)(a.parts + (int64_t)(z < a.nparts ? z : 0) * a.part_stride + row * n))[cc];
    bs[j] = ((const float4 *)(a.bias ? a.bias : a.parts))[cc];
    rs[j] = ((const float4 *)((a.resid ? a.resid : a.parts) + row * n))[cc];
    gm[j] = ((const float4 *)(a.g ? a.g : a.parts))[cc];
    bt[j] = ((const float4 *)(a.b ? a.b : a.parts))[cc];
  }
  float v[VPL][4];
#pragma unroll
  for (int j = 0; j < VPL; j++) {
    float x[4] = {t[j][0].x, t[j][0].y, t[j][0].z, t[j][0].w};
#pragma unroll
    for (int z = 1; z < NZ; z++)
      if (z < a.nparts) x[0] += t[j][z].x, x[1] += t[j][z].y, x[2] += t[j][z].z, x[3] += t[j][z].w;
    if (a.bias) x[0] += bs[j].x, x[1] += bs[j].y, x[2] += bs[j].z, x[3] += bs[j].w;
    if (a.resid) x[0] += rs[j].x, x[1] += rs[j].y, x[2] += rs[j].z, x[3] += rs[j].w;
    if (ok[j]) ((float4 *)(a.xout + row * n))[tid + 256 * j] = make_float4(x[0], x[1], x[2], x[3]);
#pragma unroll
    for (int e = 0; e < 4; e++) v[j][e] = ok[j] ? x[e] : 0.0f;
  }
  const float inv_n = 1.0f / (float)n;
  float mean = 0.0f;
  if (MODE != ROW_RMSNORM) {
    float s = 0.0f;
#pragma unroll
    for (int j = 0; j < VPL; j++)
#pragma unroll
      for (int e = 0; e < 4; e++) s += v[j][e];
    s = wave_sum(s);
    if (lane == 0) red[0][wv] = s;
    __syncthreads();
    mean = ((red[0][0] + red[0][1]) + (red[0][2] + red[0][3])) * inv_n;
  }
  float q = 0.0f;
#pragma unroll
  for (int j = 0; j < VPL; j++)
#pragma unroll
    for (int e = 0; e < 4; e++) {
      float d = ok[j] ? v[j][e] - mean : 0.0f;
      v[j][e] = d;
      q = fmaf(d, d, q);
    }
  q = wave_sum(q);
  if (lane == 0) red[1][wv] = q;
  __syncthreads();
  const float rstd = 1.0f / sqrtf(((red[1][0] + red[1][1]) + (red[1][2] + red[1][3])) * inv_n + a.eps);
#pragma unroll
  for (int j = 0; j < VPL; j++) {
    if (ok[j]) {
      const float4 g = a.g ? gm[j] : make_float4(1.f, 1.f, 1.f, 1.f);
      const float4 b = a.b ? bt[j] : make_float4(0.f, 0.f, 0.f, 0.f);
      ((float4 *)(a.y + row * n))[tid + 256 * j] = make_float4(v[j][0] * rstd * g.x + b.x, v[j][1] * rstd * g.y + b.y,
                                                             v[j][2] * rstd * g.z + b.z, v[j][3] * rstd * g.w + b.w);
    }
  }
}

bool reduce_norm_supported(int n, int nparts) { return reduce_norm_plan(n, nparts, 1).ok || reduce_norm_plan(n, nparts, 1 << 20).ok; }

int launch_reduce_norm(float *y, float *xout, const float *parts, int nparts, int64_t part_stride, const float *bias,
                       const float *resid, const float *g, const float *b, float eps, int64_t rows, int n, bool rms) {
  if (rows == 0 || n == 0) return 0;
  if (!reduce_norm_supported(n, nparts)) return fail(CTHIP_E_BAD_ARG, "reduce + norm: rows of %d with %d shares", n, nparts);
  ReduceNormArgs a = {y, xout, parts, nparts, part_stride, bias, resid, g, b, eps, rows, n};
  hipStream_t st = state().stream;
  const ReduceNormPlan pl = reduce_norm_plan(n, nparts, rows);
  if (pl.wide) {
    const int vplw = pl.vpl;
    dim3 gridw((unsigned)rows), blockw(256);
#define RW3(MODE, V, Z) hipLaunchKernelGGL((k_reduce_norm_wide<MODE, V, Z>), gridw, blockw, 0, st, a)
#define RW2(MODE, V)                       \
    if (nparts <= 2) RW3(MODE, V, 2);      \
    else if (nparts <= 4) RW3(MODE, V, 4); \
    else if (nparts <= 8) RW3(MODE, V, 8); \
    else RW3(MODE, V, 16)
#define RW1(MODE)                            \
    if (vplw <= 1) { RW2(MODE, 1); }         \
    else if (vplw <= 2) { RW2(MODE, 2); }    \
    else if (vplw <= 4) { RW2(MODE, 4); }    \
    else { RW2(MODE, 8); }
    if (rms) { RW1(ROW_RMSNORM) } else { RW1(ROW_LAYERNORM) }
#undef RW1
#undef RW2
#undef RW3
    CTHIP_LAUNCH_CHECK();
    return 0;
  }
  const int vpl = pl.vpl;
  // a row per wavefront; few rows (a prompt) go one to a workgroup so that they spread over the compute units
  const int wpb = rows <= 4096 ? 1 : 4;
  dim3 grid((unsigned)((rows + wpb - 1) / wpb)), block(64 * wpb);
#define RN3(MODE, V, Z) hipLaunchKernelGGL((k_reduce_norm<MODE, V, Z>), grid, block, 0, st, a)
#define RN2(MODE, V)               \
  if (nparts <= 2) RN3(MODE, V, 2); \
  else if (nparts <= 4) RN3(MODE, V, 4); \
  else if (nparts <= 8) RN3(MODE, V, 8); \
  else RN3(MODE, V, 16)
#define RN1(MODE)                  \
  if (vpl <= 1) { RN2(MODE, 1); }  \
  else if (vpl <= 2) { RN2(MODE, 2); } \
  else if (vpl <= 3) { RN2(MODE, 3); } \
  else if (vpl <= 4) { RN2(MODE, 4); } \
  else if (vpl <= 6) { RN2(MODE, 6); } \
  else { RN2(MODE, 8); }
  if (rms) { RN1(ROW_RMSNORM) } else { RN1(ROW_LAYERNORM) }
#undef RN1
#undef RN2
#undef RN3
  CTHIP_LAUNCH_CHECK();
  return 0;
}

// any n: one block per row, three passes through L2
template <int MODE>
__global__ __launch_bounds__(256) void k_rowop_generic(RowArgs a) {
  __shared__ float red[4];
  const int tid = threadIdx.x;
  const int n = a.n;
  const float *__restrict__ xr = a.x + (int64_t)blockIdx.x * n;
  float *__restrict__ yr = a.y + (int64_t)blockIdx.x * n;
  auto block_sum = [&](float v) {
    v = wave_sum(v);
    __syncthreads();
    if ((tid & 63) == 0) red[tid >> 6] = v;
    __syncthreads();
    return red[0] + red[1] + red[2] + red[3];
  };
  auto block_max = [&](float v) {
    v = wave_max(v);
    __syncthreads();
    if ((tid & 63) == 0) red[tid >> 6] = v;
    __syncthreads();
    return fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  };
  float mean = 0.0f, rstd = 1.0f;
  const bool norm = MODE != ROW_SOFTMAX;
  if (norm) {
    if (MODE != ROW_RMSNORM) {
      float s = 0.0f;
      for (int i = tid; i < n; i += 256) s += xr[i];
      mean = block_sum(s) / (float)n;
    }
    float q = 0.0f;
    for (int i = tid; i < n; i += 256) {
      float d = xr[i] - mean;
      q = fmaf(d, d, q);
    }
    rstd = 1.0f / sqrtf(block_sum(q) / (float)n + a.eps);
  }
  auto val = [&](int i) {
    float t = xr[i];
    if (norm) {
      t = (t - mean) * rstd;
      if (a.g) t *= a.g[i];
      if (a.b) t += a.b[i];
    }
    return t;
  };
  if (MODE == ROW_LAYERNORM || MODE == ROW_RMSNORM) {
    for (int i = tid; i < n; i += 256) yr[i] = val(i);
    return;
  }
  float m = -INFINITY;
  for (int i = tid; i < n; i += 256) m = fmaxf(m, val(i));
  m = block_max(m);
  float s = 0.0f;
  for (int i = tid; i < n; i += 256) s += ct_exp(val(i) - m);
  const float inv = 1.0f / block_sum(s);
  for (int i = tid; i < n; i += 256) yr[i] = ct_exp(val(i) - m) * inv;
}

template <int MODE>
static int launch_rowop(RowArgs a) {
  if (a.rows == 0 || a.n == 0) return 0;
  hipStream_t st = state().stream;
  if (a.n % 4 == 0 && a.n <= 2048 && ((uintptr_t)a.x % 16 == 0) && ((uintptr_t)a.y % 16 == 0) &&
      (!a.g || (uintptr_t)a.g % 16 == 0) && (!a.b || (uintptr_t)a.b % 16 == 0)) {
    const int n4 = a.n / 4;
    const int vpl = (n4 + 63) / 64;
    if ((a.rows + 3) / 4 > 0x7fffffff) return fail(CTHIP_E_BAD_ARG, "row op: too many rows");
    dim3 grid((unsigned)((a.rows + 3) / 4)), block(256);
    switch (vpl) {
      case 1: hipLaunchKernelGGL((k_rowop<MODE, 1>), grid, block, 0, st, a); break;
      case 2: hipLaunchKernelGGL((k_rowop<MODE, 2>), grid, block, 0, st, a); break;
      case 3: hipLaunchKernelGGL((k_rowop<MODE, 3>), grid, block, 0, st, a); break;
      case 4: hipLaunchKernelGGL((k_rowop<MODE, 4>), grid, block, 0, st, a); break;
      case 5: case 6: hipLaunchKernelGGL((k_rowop<MODE, 6>), grid, block, 0, st, a); break;
      default: hipLaunchKernelGGL((k_rowop<MODE, 8>), grid, block, 0, st, a); break;
    }
  } else {
    if (a.rows > 0x7fffffff) return fail(CTHIP_E_BAD_ARG, "row op: too many rows");
    hipLaunchKernelGGL((k_rowop_generic<MODE>), dim3((unsigned)a.rows), dim3(256), 0, st, a);
  }
  CTHIP_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------ elementwise
// A block owns UNARY_PER_BLOCK consecutive elements; a thread takes UNARY_VEC-wide pieces 256 pieces apart, all of
// its loads issued before the first store.  (A capped grid with a grid-stride loop, one float4 in flight per thread,
// ran at 75 us on 50 M elements; this at what the renderer's element-wise kernels reach.)
template <int VEC>
__global__ __launch_bounds__(256) void k_unary(int kind, float *__restrict__ y, const float *__restrict__ x, int64_t n) {
  constexpr int PER = 256 * 4 * VEC;  // elements per block
  const int64_t base = (int64_t)blockIdx.x * PER;
  if (base + PER <= n) {
    if (VEC == 4) {
      float4 v[4];
#pragma unroll
      for (int e = 0; e < 4; e++) v[e] = ((const float4 *)(x + base))[256 * e + threadIdx.x];
#pragma unroll
      for (int e = 0; e < 4; e++) {
        v[e].x = apply_act(kind, v[e].x);
        v[e].y = apply_act(kind, v[e].y);
        v[e].z = apply_act(kind, v[e].z);
        v[e].w = apply_act(kind, v[e].w);
        ((float4 *)(y + base))[256 * e + threadIdx.x] = v[e];
      }
    } else {
      float v[4];
#pragma unroll
      for (int e = 0; e < 4; e++) v[e] = x[base + 256 * e + threadIdx.x];
#pragma unroll
      for (int e = 0; e < 4; e++) y[base + 256 * e + threadIdx.x] = apply_act(kind, v[e]);
    }
  } else {
    for (int64_t k = base + threadIdx.x; k < n; k += 256) y[k] = apply_act(kind, x[k]);
  }
}

// out[t,:] = W[idx[t],:]  (+ W2[pos0 + t,:] when W2 is given: wte + wpe of Transformer, layers.lisp:80-82)
__global__ __launch_bounds__(256) void k_embedding(float *__restrict__ out, const float *__restrict__ W,
                                                   const float *__restrict__ idx_f, const int *__restrict__ idx_i,
                                                   int vocab, int dim, const float *__restrict__ W2,
                                                   const int *__restrict__ pos, int max_pos) {
  const int t = blockIdx.x;
  int id = idx_f ? (int)idx_f[t] : idx_i[t];
  const bool hit = id >= 0 && id < vocab && (!idx_f || (float)id == idx_f[t]);
  int p = 0;
  bool phit = false;
  if (W2) {
    p = pos[0] + t;
    phit = p >= 0 && p < max_pos;
  }
  for (int d = threadIdx.x; d < dim; d += blockDim.x) {
    // an index no vocabulary row equals selects nothing in the reference's one-hot sum: 0
    float v = hit ? W[(int64_t)id * dim + d] : 0.0f;
    if (W2) v += phit ? W2[(int64_t)p * dim + d] : 0.0f;
    out[(int64_t)t * dim + d] = v;
  }
}

// out[t,:] = W[first + step * t,:] (+ addend[t,:]): an Embedding whose indices are an arithmetic progression, as the
// position table of Transformer is read (wpe(start-pos + arange(seq-len)), external/llm/layers.lisp:81-82).  A row
// the table does not have selects nothing in the one-hot sum: 0.
__global__ __launch_bounds__(256) void k_embedding_rows(float *__restrict__ out, const float *__restrict__ W, long long first,
                                                        long long step, int vocab, int dim, const float *__restrict__ addend) {
  const int t = blockIdx.x;
  const long long row = first + step * t;
  const bool hit = row >= 0 && row < vocab;
  for (int d = threadIdx.x; d < dim; d += blockDim.x) {
    float v = hit ? W[row * dim + d] : 0.0f;
    if (addend) v += addend[(int64_t)t * dim + d];
    out[(int64_t)t * dim + d] = v;
  }
}

// lowest index of the maximum of each row; one 1024-thread block per row.
// tok_out/pos (optional) feed the device-resident decode loop: the token is also
// stored as int32 and the position counter advanced.
__global__ __launch_bounds__(1024) void k_argmax(int64_t *__restrict__ out, const float *__restrict__ x, int n,
                                                 int *__restrict__ tok_out, int *__restrict__ pos,
                                                 int64_t *__restrict__ history, int *__restrict__ hist_n) {
  __shared__ float sm[16];
  __shared__ int si[16];
  const float *__restrict__ xr = x + (int64_t)blockIdx.x * n;
  float best = -INFINITY;
  int bi = 0x7fffffff;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    float v = xr[i];
    if (v > best || (v == best && i < bi)) {
      best = v;
      bi = i;
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    float ob = __shfl_xor(best, o, 64);
    int oi = __shfl_xor(bi, o, 64);
    if (ob > best || (ob == best && oi < bi)) {
      best = ob;
      bi = oi;
    }
  }
  const int w = threadIdx.x >> 6, nw = blockDim.x >> 6;
  if ((threadIdx.x & 63) == 0) {
    sm[w] = best;
    si[w] = bi;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int k = 1; k < nw; k++)
      if (sm[k] > best || (sm[k] == best && si[k] < bi)) {
        best = sm[k];
        bi = si[k];
      }
    if (bi == 0x7fffffff) bi = 0;  // all-NaN / empty row
    out[blockIdx.x] = bi;
    if (tok_out) *tok_out = bi;
    if (history) {
      history[*hist_n] = bi;
      *hist_n = *hist_n + 1;
    }
    if (pos) *pos = *pos + 1;
  }
}

// A few long rows (the logits of a decode step: one row of 50 257): one block per row reads its row alone, a
// memory round trip per 1024 elements.  Here kArgmaxParts blocks per row each reduce a contiguous part ...
constexpr int kArgmaxParts = 64;
__global__ __launch_bounds__(256) void k_argmax_parts(float *__restrict__ pv, int *__restrict__ pi, const float *__restrict__ x, int n) {
  __shared__ float sm[4];
  __shared__ int si[4];
  const int row = blockIdx.x, part = blockIdx.y;
  const int per = (n + kArgmaxParts - 1) / kArgmaxParts;
  const int lo = part * per, hi = min(n, lo + per);
  const float *__restrict__ xr = x + (int64_t)row * n;
  float best = -INFINITY;
  int bi = 0x7fffffff;
  for (int i = lo + threadIdx.x; i < hi; i += 256) {
    const float v = xr[i];
    if (v > best || (v == best && i < bi)) {
      best = v;
      bi = i;
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ob = __shfl_xor(best, o, 64);
    const int oi = __shfl_xor(bi, o, 64);
    if (ob > best || (ob == best && oi < bi)) {
      best = ob;
      bi = oi;
    }
  }
  if ((threadIdx.x & 63) == 0) {
    sm[threadIdx.x >> 6] = best;
    si[threadIdx.x >> 6] = bi;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int k = 1; k < 4; k++)
      if (sm[k] > best || (sm[k] == best && si[k] < bi)) {
        best = sm[k];
        bi = si[k];
      }
    pv[row * kArgmaxParts + part] = best;
    pi[row * kArgmaxParts + part] = bi;
  }
}
// ... and one wavefront per row settles the parts (lowest index among equal maxima, as k_argmax).
__global__ __launch_bounds__(64) void k_argmax_settle(int64_t *__restrict__ out, const float *__restrict__ pv, const int *__restrict__ pi,
                                                      int *__restrict__ tok_out, int *__restrict__ pos,
                                                      int64_t *__restrict__ history, int *__restrict__ hist_n) {
  const int row = blockIdx.x;
  float best = pv[row * kArgmaxParts + threadIdx.x];
  int bi = pi[row * kArgmaxParts + threadIdx.x];
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ob = __shfl_xor(best, o, 64);
    const int oi = __shfl_xor(bi, o, 64);
    if (ob > best || (ob == best && oi < bi)) {
      best = ob;
      bi = oi;
    }
  }
  if (threadIdx.x == 0) {
    if (bi == 0x7fffffff) bi = 0;  // all-NaN / empty row
    out[row] = bi;
    if (tok_out) *tok_out = bi;
    if (history) {
      history[*hist_n] = bi;
      *hist_n = *hist_n + 1;
    }
    if (pos) *pos = *pos + 1;
  }
}

// RoPE on (B,S,H,Dh), one thread per (pair)
__global__ __launch_bounds__(256) void k_rope(float *__restrict__ out, const float *__restrict__ x, int64_t npairs,
                                              int S, int H, int Dh, float log2_base, int start_pos,
                                              const int *__restrict__ pos) {
  int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= npairs) return;
  const int half = Dh >> 1;
  const int i = (int)(p % half);
  const int64_t r = p / half;  // (b*S + s)*H + h
  const int s = (int)((r / H) % S);
  const int at = s + start_pos + (pos ? pos[0] : 0);
  // theta_i = exp(-(2i/Dh) * ln base), spelled through exp2/log2 with a float rounding at each
  // tensor the reference materialises (positional-encoding.lisp:26-35)
  const float expo = (float)(2 * i) / (float)Dh;
  const float logb = log2_base * 0.6931472f;
  const float theta = exp2f(-(expo * logb) * 1.442695f);
  const float ang = (float)at * theta;
  float sn, cs;
  sincosf(ang, &sn, &cs);
  const float x0 = x[2 * p], x1 = x[2 * p + 1];
  rope_pair(x0, x1, sn, cs, out[2 * p], out[2 * p + 1]);
}

// Llama-shaped decode: rotate the new key row (Hkv,Dh) at position pos[0] into the K cache and
// copy the new value row beside it.  kv holds k then v, KD floats each.
__global__ __launch_bounds__(256) void k_rope_append(float *__restrict__ kc, float *__restrict__ vc,
                                                     const float *__restrict__ kv, int Hkv, int Dh, float log2_base,
                                                     const int *__restrict__ pos) {
  const int KD = Hkv * Dh;
  const int p = blockIdx.x * blockDim.x + threadIdx.x;  // pair index
  if (p >= KD / 2) return;
  const int at = pos[0];
  const int i = p % (Dh / 2);
  const float expo = (float)(2 * i) / (float)Dh;
  const float logb = log2_base * 0.6931472f;
  const float theta = exp2f(-(expo * logb) * 1.442695f);
  const float ang = (float)at * theta;
  float sn, cs;
  sincosf(ang, &sn, &cs);
  const float x0 = kv[2 * p], x1 = kv[2 * p + 1];
  float *ko = kc + (int64_t)at * KD;
  float *vo = vc + (int64_t)at * KD;
  rope_pair(x0, x1, sn, cs, ko[2 * p], ko[2 * p + 1]);
  vo[2 * p] = kv[KD + 2 * p];
  vo[2 * p + 1] = kv[KD + 2 * p + 1];
}

// Prefill: one fused-qkv row per block -> q (contiguous, rotated for RoPE models), k (rotated) and v
// into the cache rows start_pos + i.
__global__ __launch_bounds__(256) void k_qkv_split(float *__restrict__ q, float *__restrict__ kc,
                                                   float *__restrict__ vc, const float *__restrict__ qkv, int start_pos,
                                                   int H, int Hkv, int Dh, float log2_base, int rope) {
  const int i = blockIdx.x;
  const int D = H * Dh, KD = Hkv * Dh;
  const float *row = qkv + (int64_t)i * (D + 2 * KD);
  const int at = start_pos + i;
  float *ko = kc + (int64_t)at * KD, *vo = vc + (int64_t)at * KD, *qo = q + (int64_t)i * D;
  for (int p = threadIdx.x; p < (D + KD) / 2; p += blockDim.x) {  // pairs of q then k
    const bool isq = p < D / 2;
    const int pp = isq ? p : p - D / 2;
    const float x0 = isq ? row[2 * pp] : row[D + 2 * pp], x1 = isq ? row[2 * pp + 1] : row[D + 2 * pp + 1];
    float o0 = x0, o1 = x1;
    if (rope) {
      const int ii = pp % (Dh / 2);
      const float expo = (float)(2 * ii) / (float)Dh;
      const float theta = exp2f(-(expo * (log2_base * 0.6931472f)) * 1.442695f);
      float sn, cs;
      sincosf((float)at * theta, &sn, &cs);
      rope_pair(x0, x1, sn, cs, o0, o1);
    }
    float *dst = isq ? qo : ko;
    dst[2 * pp] = o0;
    dst[2 * pp + 1] = o1;
  }
  for (int j = threadIdx.x; j < KD; j += blockDim.x) vo[j] = row[D + KD + j];
}

// ------------------------------------------------------------------ attention over the KV cache
// One 1024-thread block per (query head h, query row i); keys 0..T-1 with T = pos+i+1 (the causal
// mask of layers.lisp:83 is implicit).  K/V cache layout (max_len, Hkv, Dh).
//
// A key row is read by DH/4 adjacent lanes as one float4 each (coalesced 4*DH bytes), so a wavefront
// covers 64/(DH/4) keys per pass and holds KPT passes of K and V in registers, all requested before
// any arithmetic.  Every wavefront runs its own online softmax over its keys (shuffles only); the 16
// per-wavefront partials (max, sum, DH outputs) meet once in LDS, so a block needs one barrier.
//
// APPEND (decode of RoPE models, one row): the step's new key / value row is still in `newkv` (k then v,
// Hkv*DH floats each, unrotated).  Every block rotates its query and its kv head's new key in registers
// (positional-encoding.lisp:3-64 at position pos), uses them for key T-1, and the first query head of each
// kv group stores the rotated key and the value into cache row T-1 -- the rotation and the `!assign` into
// the cache (layers.lisp:13-33) need no launches of their own.
//
// SPLIT (one query row, long contexts): gridDim.z workgroups share a head's keys.  With one workgroup per head a
// 32-head model reads its cache through 32 compute units (Llama-7B shape at position 1940: 107 us per layer for
// 64 MB of rows); here the keys are cut into ranges of whole tiles, a workgroup leaves (max, sum, unnormalised
// output) of its range in `sp_part`, takes a ticket from the head's counter, and the one that draws the last ticket
// adds the ranges up.  The grid is fixed when the step is captured while the position is device data, so how many
// ranges are in use is decided here: workgroups past the last range leave at once, and a context of one tile is
// one range whose workgroup writes the output itself, without a ticket.
template <int DH, bool APPEND, bool SPLIT>
__global__ __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(4, 4)))
void k_attn_cached(float *__restrict__ out, const float *__restrict__ q,
                                                      float *__restrict__ kc, float *__restrict__ vc,
                                                      int start_pos, const int *__restrict__ pos, int H, int Hkv,
                                                      const float *__restrict__ newkv, float log2_base,
                                                      float *__restrict__ sp_part, int *__restrict__ sp_count) {
  constexpr int LPK = DH / 4;      // lanes per key
  constexpr int KPW = 64 / LPK;    // keys per wavefront per pass
  constexpr int KPT = 4;           // passes held in registers
  constexpr int NW = 16;
  constexpr int TILE = NW * KPW * KPT;
  __shared__ float part[NW][DH];
  __shared__ float pm[NW], pl[NW];
  __shared__ int ticket;
  const int h = attn_head_of_block(blockIdx.x, H, Hkv), i = blockIdx.y;
  const int T = start_pos + (pos ? pos[0] : 0) + i + 1;
  // this workgroup's keys [k0, k1): everything, or one of `nranges` ranges of whole tiles
  int k0 = 0, k1 = T, nranges = 1;
  if (SPLIT) {
    const int nz = (int)gridDim.z, tiles = (T + TILE - 1) / TILE;
    const int per = ((tiles + nz - 1) / nz) * TILE;  // keys per range
    nranges = (T + per - 1) / per;
    k0 = (int)blockIdx.z * per;
    if (k0 >= T) return;  // (uniform) no range for this workgroup
    k1 = min(T, k0 + per);
  }
  const int hk = h / (H / Hkv);
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int g = lane / LPK, c = lane % LPK;
  const unsigned kvs4 = (unsigned)(Hkv * DH / 4);
  float4 q4 = *(const float4 *)(q + ((int64_t)i * H + h) * DH + 4 * c);
  const float4 *__restrict__ kp = (const float4 *)(kc + (int64_t)hk * DH) + c;
  const float4 *__restrict__ vp = (const float4 *)(vc + (int64_t)hk * DH) + c;
  const float scale = 1.0f / sqrtf((float)DH);
  float4 kn = make_float4(0.f, 0.f, 0.f, 0.f), vn = kn;
  if (APPEND) {
    kn = *(const float4 *)(newkv + hk * DH + 4 * c);
    vn = *(const float4 *)(newkv + Hkv * DH + hk * DH + 4 * c);
  }
  // One tile = NP key passes per wavefront, all requested together: wavefront wv owns keys t0 + (wv*NP + u)*KPW + g.
  // Up to TILE keys that is KPT passes; a longer context takes tiles of twice as many passes, so that positions up
  // to twice as far still cost one memory round trip instead of two.
  auto request = [&](auto np_tag, int t0, float4 *kr, float4 *vr) {
    constexpr int NP = decltype(np_tag)::value;
#pragma unroll
    for (int u = 0; u < NP; u++) {
      const int j = t0 + (wv * NP + u) * KPW + g;
      // clamp: masked below, never out of the cache; APPEND: row T-1 comes from the registers
      const unsigned jj = (unsigned)min(j, APPEND ? max(T - 2, 0) : T - 1);
      kr[u] = kp[jj * kvs4];
      vr[u] = vp[jj * kvs4];
    }
  };
  // rotation of the query and of the new key, and the new row's store.  The angles need the position alone and many
  // registers for a moment: they are worked out before the rows are asked for, the rotation itself afterwards.
  auto rotate_and_append = [&]() {
    if (APPEND) {
      const int KD = Hkv * DH;
      const Rope4 ra = rope4_angles(c, DH, log2_base, T - 1);
      q4 = rope4_apply(q4, ra);
      kn = rope4_apply(kn, ra);
      if (h % (H / Hkv) == 0 && tid < LPK && (!SPLIT || blockIdx.z == 0)) {
        ((float4 *)(kc + (int64_t)(T - 1) * KD + hk * DH))[c] = kn;
        ((float4 *)(vc + (int64_t)(T - 1) * KD + hk * DH))[c] = vn;
      }
    }
  };
  float m = -INFINITY, l = 0.0f;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  auto consume = [&](auto np_tag, int t0, float4 *kr, float4 *vr) {
    constexpr int NP = decltype(np_tag)::value;
    if (APPEND) {
#pragma unroll
      for (int u = 0; u < NP; u++) {
        if (t0 + (wv * NP + u) * KPW + g >= T - 1) {
          kr[u] = kn;
          vr[u] = vn;
        }
      }
    }
    float sc[NP];
    float tmax = -INFINITY;
#pragma unroll
    for (int u = 0; u < NP; u++) {
      float d = q4.x * kr[u].x;
      d = fmaf(q4.y, kr[u].y, d);
      d = fmaf(q4.z, kr[u].z, d);
      d = fmaf(q4.w, kr[u].w, d);
      if (LPK == 16) {  // the key's lanes are one row of the data-parallel primitives: no trip through the LDS crossbar
        d = row16_sum(d);
      } else {
#pragma unroll
        for (int o = LPK / 2; o > 0; o >>= 1) d += __shfl_xor(d, o, 64);
      }
      const bool ok = (t0 + (wv * NP + u) * KPW + g) < k1;
      sc[u] = ok ? d * scale : -INFINITY;
      tmax = fmaxf(tmax, sc[u]);
    }
    if (LPK == 16) {
      tmax = groups16_max(tmax);
    } else {
#pragma unroll
      for (int o = LPK; o < 64; o <<= 1) tmax = fmaxf(tmax, __shfl_xor(tmax, o, 64));
    }
    const float m_new = fmaxf(m, tmax);   // finite: this wavefront has at least one key here
    const float corr = ct_exp(m - m_new);  // 0 on its first tile (m = -inf)
    float ps = 0.0f;
#pragma unroll
    for (int k2 = 0; k2 < 4; k2++) acc[k2] *= corr;
#pragma unroll
    for (int u = 0; u < NP; u++) {
      const float p = ct_exp(sc[u] - m_new);  // exp2(-inf) = 0 for masked keys
      ps += p;
      acc[0] = fmaf(p, vr[u].x, acc[0]);
      acc[1] = fmaf(p, vr[u].y, acc[1]);
      acc[2] = fmaf(p, vr[u].z, acc[2]);
      acc[3] = fmaf(p, vr[u].w, acc[3]);
    }
    if (LPK == 16) {  // every lane of a key holds the same p
      ps = groups16_sum(ps);
    } else {
#pragma unroll
      for (int o = LPK; o < 64; o <<= 1) ps += __shfl_xor(ps, o, 64);
    }
    l = l * corr + ps;
    m = m_new;
  };
  // The first tile's rows are asked for as soon as the position is known, BEFORE the query is waited for and rotated:
  // their round trip to memory runs beside the query's, the new row's and the angles' arithmetic.
  if (k1 - k0 <= TILE) {
    const bool has_keys = k0 + wv * KPT * KPW < k1;  // (uniform per wavefront)
    float4 kr[KPT], vr[KPT];
    if (has_keys) request(std::integral_constant<int, KPT>(), k0, kr, vr);
    rotate_and_append();
    if (has_keys) consume(std::integral_constant<int, KPT>(), k0, kr, vr);
  } else {
    const bool has_keys = k0 + wv * 2 * KPT * KPW < k1;
    float4 kr[2 * KPT], vr[2 * KPT];
    if (has_keys) request(std::integral_constant<int, 2 * KPT>(), k0, kr, vr);
    rotate_and_append();
    // (two spellings of one loop: the register allocator keeps each variant of the kernel inside its 128 registers
    // with one of them only)
    if (APPEND) {
      for (int t0 = k0; t0 < k1; t0 += 2 * TILE) {
        if (t0 + wv * 2 * KPT * KPW >= k1) break;  // nothing left for this wavefront (uniform)
        if (t0 != k0) request(std::integral_constant<int, 2 * KPT>(), t0, kr, vr);
        consume(std::integral_constant<int, 2 * KPT>(), t0, kr, vr);
      }
    } else if (has_keys) {
      for (int t0 = k0;;) {
        consume(std::integral_constant<int, 2 * KPT>(), t0, kr, vr);
        t0 += 2 * TILE;
        if (t0 + wv * 2 * KPT * KPW >= k1) break;
        request(std::integral_constant<int, 2 * KPT>(), t0, kr, vr);
      }
    }
  }
  // combine the key groups inside the wavefront, then the wavefronts through LDS
#pragma unroll
  for (int o = LPK; o < 64; o <<= 1) {
#pragma unroll
    for (int k2 = 0; k2 < 4; k2++) acc[k2] += __shfl_xor(acc[k2], o, 64);
  }
  if (lane < LPK) {
#pragma unroll
    for (int k2 = 0; k2 < 4; k2++) part[wv][4 * lane + k2] = acc[k2];
  }
  if (lane == 0) {
    pm[wv] = m;
    pl[wv] = l;
  }
  __syncthreads();
  if (tid < DH) {
    float M = pm[0];
#pragma unroll
    for (int w = 1; w < NW; w++) M = fmaxf(M, pm[w]);
    float o = 0.0f, L = 0.0f;
#pragma unroll
    for (int w = 0; w < NW; w++) {
      const float e = ct_exp(pm[w] - M);  // wavefronts without keys hold m = -inf: weight 0
      o = fmaf(e, part[w][tid], o);
      L = fmaf(e, pl[w], L);
    }
    if (!SPLIT || nranges == 1) {
      out[((int64_t)i * H + h) * DH + tid] = o / L;
    } else {
      // device-scope stores: written through to memory, no cache to flush (a fence here would write back and
      // invalidate the whole L2 of the XCD under every other workgroup's key reads: measured 2x slower than no split)
      float *mine = sp_part + ((int64_t)h * gridDim.z + blockIdx.z) * (DH + 2);
      __hip_atomic_store(mine + tid, o, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (tid == 0) {
        __hip_atomic_store(mine + DH, M, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(mine + DH + 1, L, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  }
  if (SPLIT && nranges > 1) {
    // a thread's stores have reached memory when the memory counter is back at zero; after the barrier that holds
    // for the whole workgroup, and only then is its ticket drawn.  The workgroup with the last ticket reads every
    // range's triple with device-scope loads (which do not look into a cache that could hold an older launch's).
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) ticket = __hip_atomic_fetch_add(sp_count + h, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (ticket != nranges - 1) return;  // (uniform)
    if (tid < DH) {
      out[((int64_t)i * H + h) * DH + tid] = attn_split_merge(sp_part + (int64_t)h * gridDim.z * (DH + 2), nranges, DH, tid);
    }
    if (tid == 0) __hip_atomic_store(sp_count + h, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // the next launch counts again
  }
}

// sum over aligned groups of LPK lanes (8, 16 or 32), every lane gets the sum
template <int LPK>
__device__ __forceinline__ float lpk_sum(float v) {
  v += dpp_f<0xB1>(v);   // quad_perm [1,0,3,2]
  v += dpp_f<0x4E>(v);   // quad_perm [2,3,0,1]
  v += dpp_f<0x141>(v);  // row_half_mirror: 8 lanes
  if (LPK >= 16) v += dpp_f<0x140>(v);  // row_mirror: 16 lanes
  if (LPK >= 32) v += __shfl_xor(v, 16, 64);
  return v;
}

// Prompt rows (s > 1): one 256-thread block per (head, group of R consecutive query rows).  The group
// shares every K / V tile it loads, so the cache is read once per R rows instead of once per row; the
// causal mask (layers.lisp:83) is applied per row.  Same lane layout and per-wavefront online softmax
// as k_attn_cached, with R running (max, sum, output) triples.
template <int DH, int R>
__global__ __launch_bounds__(256) void k_attn_rows(float *__restrict__ out, const float *__restrict__ q,
                                                   const float *__restrict__ kc, const float *__restrict__ vc, int S,
                                                   int start_pos, const int *__restrict__ pos, int H, int Hkv) {
  constexpr int LPK = DH / 4, KPW = 64 / LPK, KPT = 8, NW = 4, TILE = NW * KPW * KPT;
  __shared__ float part[NW][R][DH];
  __shared__ float pm[NW][R], pl[NW][R];
  // the last groups see the most keys: they are dispatched first so the short ones fill the tail
  const int h = blockIdx.x, i0 = (gridDim.y - 1 - blockIdx.y) * R;
  const int base = start_pos + (pos ? pos[0] : 0);
  const int nrows = min(R, S - i0);
  const int Tmax = base + i0 + nrows;  // keys the last row of the group sees
  const int hk = h / (H / Hkv);
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int g = lane / LPK, c = lane % LPK;
  const unsigned kvs4 = (unsigned)(Hkv * DH / 4);
  const float4 *__restrict__ kp = (const float4 *)(kc + (int64_t)hk * DH) + c;
  const float4 *__restrict__ vp = (const float4 *)(vc + (int64_t)hk * DH) + c;
  const float scale = 1.0f / sqrtf((float)DH);
  float4 q4[R];
  float m[R], l[R], acc[R][4];
#pragma unroll
  for (int r = 0; r < R; r++) {
    const int row = min(i0 + r, S - 1);  // rows past the end repeat the last one and are not stored
    q4[r] = *(const float4 *)(q + ((int64_t)row * H + h) * DH + 4 * c);
    m[r] = -INFINITY;
    l[r] = 0.0f;
    acc[r][0] = acc[r][1] = acc[r][2] = acc[r][3] = 0.0f;
  }
  for (int t0 = 0; t0 < Tmax; t0 += TILE) {
    if (t0 + wv * KPT * KPW >= Tmax) break;  // nothing left for this wavefront (uniform)
    float4 kr[KPT], vr[KPT];
#pragma unroll
    for (int u = 0; u < KPT; u++) {
      const int j = t0 + (wv * KPT + u) * KPW + g;
      const unsigned jj = (unsigned)min(j, Tmax - 1);
      kr[u] = kp[jj * kvs4];
      vr[u] = vp[jj * kvs4];
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
      const int Tr = base + min(i0 + r, S - 1) + 1;  // keys row r sees
      float sc[KPT];
      float tmax = -INFINITY;
#pragma unroll
      for (int u = 0; u < KPT; u++) {
        float d = q4[r].x * kr[u].x;
        d = fmaf(q4[r].y, kr[u].y, d);
        d = fmaf(q4[r].z, kr[u].z, d);
        d = fmaf(q4[r].w, kr[u].w, d);
        d = lpk_sum<LPK>(d);
        const bool ok = (t0 + (wv * KPT + u) * KPW + g) < Tr;
        sc[u] = ok ? d * scale : -INFINITY;
        tmax = fmaxf(tmax, sc[u]);
      }
#pragma unroll
      for (int o = LPK; o < 64; o <<= 1) tmax = fmaxf(tmax, __shfl_xor(tmax, o, 64));
      const float m_new = fmaxf(m[r], tmax);
      const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;  // every key of this tile masked for row r so far
      const float corr = ct_exp(m[r] - m_use);
      float ps = 0.0f;
#pragma unroll
      for (int k2 = 0; k2 < 4; k2++) acc[r][k2] *= corr;
#pragma unroll
      for (int u = 0; u < KPT; u++) {
        const float p = ct_exp(sc[u] - m_use);
        ps += p;
        acc[r][0] = fmaf(p, vr[u].x, acc[r][0]);
        acc[r][1] = fmaf(p, vr[u].y, acc[r][1]);
        acc[r][2] = fmaf(p, vr[u].z, acc[r][2]);
        acc[r][3] = fmaf(p, vr[u].w, acc[r][3]);
      }
#pragma unroll
      for (int o = LPK; o < 64; o <<= 1) ps += __shfl_xor(ps, o, 64);
      l[r] = l[r] * corr + ps;
      m[r] = m_new;
    }
  }
#pragma unroll
  for (int r = 0; r < R; r++) {
#pragma unroll
    for (int o = LPK; o < 64; o <<= 1) {
#pragma unroll
      for (int k2 = 0; k2 < 4; k2++) acc[r][k2] += __shfl_xor(acc[r][k2], o, 64);
    }
    if (lane < LPK) {
#pragma unroll
      for (int k2 = 0; k2 < 4; k2++) part[wv][r][4 * lane + k2] = acc[r][k2];
    }
    if (lane == 0) {
      pm[wv][r] = m[r];
      pl[wv][r] = l[r];
    }
  }
  __syncthreads();
  for (int e = tid; e < nrows * DH; e += 256) {
    const int r = e / DH, d = e % DH;
    float M = pm[0][r];
#pragma unroll
    for (int w = 1; w < NW; w++) M = fmaxf(M, pm[w][r]);  // finite: key 0 is visible to every row
    float o = 0.0f, L = 0.0f;
#pragma unroll
    for (int w = 0; w < NW; w++) {
      const float wgt = ct_exp(pm[w][r] - M);
      o = fmaf(wgt, part[w][r][d], o);
      L = fmaf(wgt, pl[w][r], L);
    }
    out[((int64_t)(i0 + r) * H + h) * DH + d] = o / L;
  }
}

// Prompt rows on the matrix cores (s >= 32): one block per (head, 32 consecutive query rows); its
// NW wavefronts take the 32-key tiles of the visible cache round-robin, each with its own online softmax
// for all 32 rows, and meet once in LDS.  fp32 MFMA operands (v_mfma_f32_32x32x2_f32): the products are the
// reference's fp32 products, only the summation order differs.
//   S^T = K Q^T : lane l feeds K[key l%32][d = (l/32) DH/2 + s] (from a d-major LDS copy of the key tile) and
//                 Q[query l%32][the same d] (registers), so a lane ends up with 16 keys of ONE query;
//   softmax     : per lane over its 16 registers + one exchange with lane l^32;
//   O^T += V^T P^T : lane l feeds V[key of register s][d = l%32 (+32 per block)] straight from the cache
//                 (128 contiguous bytes per half-wavefront) and P = its own register s: the output stays
//                 one query per lane, so the running rescale is a per-lane scalar.
typedef float v16f_t __attribute__((ext_vector_type(16)));

template <int DH, int NW>
__global__ __launch_bounds__(64 * NW) void k_attn_mfma(float *__restrict__ out, const float *__restrict__ q,
                                                   const float *__restrict__ kc, const float *__restrict__ vc, int S,
                                                   int start_pos, int H, int Hkv) {
  constexpr int NS = DH / 2;   // k-steps of K Q^T
  constexpr int DB = DH / 32;  // 32-wide blocks of the head dimension
  // per wavefront: its key tile, d-major; once its tiles are done, its unnormalised outputs for the combine
  __shared__ union {
    float Kt[DH][33];
    float Co[DB * 16][64];
  } W[NW];
  __shared__ float Cm[NW][64], Cl[NW][64];
  const int h = blockIdx.x, i0 = (gridDim.y - 1 - blockIdx.y) * 32;  // the longest groups are dispatched first
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int half = lane >> 5, col = lane & 31;
  const int hk = h / (H / Hkv), KD = Hkv * DH;
  const int qrow = min(i0 + col, S - 1);  // rows past the end repeat the last one and are not stored
  const int Tq = start_pos + qrow + 1;    // keys this lane's query sees
  const int Tmax = start_pos + min(i0 + 32, S);
  const int ntiles = (Tmax + 31) / 32;
  const float scale = 1.0f / sqrtf((float)DH);
  // the key tile of a pass is requested one pass ahead, its values at the start of the pass: both are in
  // registers by the time the matrix cores need them
  float4 kreg[DH / 8];
  auto load_k = [&](int t) {
#pragma unroll
    for (int u = 0; u < DH / 8; u++) {
      const int f = lane + 64 * u, key = f / (DH / 4), d4 = f % (DH / 4);
      const int kr = min(t * 32 + key, Tmax - 1);  // rows clamped to the last visible one: masked below
      kreg[u] = *(const float4 *)(kc + (int64_t)kr * KD + hk * DH + 4 * d4);
    }
  };
  if (wv < ntiles) load_k(wv);
  // The block's 32 query rows go through LDS (the memory of the key tiles, before they are written): whole
  // rows in 16-byte pieces, one request per cache line and block.  (Every wavefront fetching its own operand
  // registers straight from memory asked for each line 128 times: 4 us of a 512-token launch.)
  constexpr int QP = DH + 4;  // row pitch: 16-byte reads of 8 consecutive rows spread over all banks
  static_assert(32 * QP * 4 <= sizeof(W), "the query rows fit the key tile memory");
  float(*Qs)[QP] = reinterpret_cast<float(*)[QP]>(&W[0]);
  for (int f = tid; f < 8 * DH; f += 64 * NW) {
    const int row = f / (DH / 4), c4 = f % (DH / 4);
    *(float4 *)&Qs[row][4 * c4] = *(const float4 *)(q + ((int64_t)min(i0 + row, S - 1) * H + h) * DH + 4 * c4);
  }
  __syncthreads();
  float qreg[NS];  // k-step s of this lane: d = half * NS + s
#pragma unroll
  for (int j = 0; j < NS / 4; j++) {
    const float4 t = *(const float4 *)&Qs[col][half * NS + 4 * j];
    qreg[4 * j + 0] = t.x, qreg[4 * j + 1] = t.y, qreg[4 * j + 2] = t.z, qreg[4 * j + 3] = t.w;
  }
  __syncthreads();  // the key tiles may overwrite the rows now
  float m = -INFINITY, l = 0.0f;
  v16f_t o[DB];
#pragma unroll
  for (int b = 0; b < DB; b++)
#pragma unroll
    for (int r = 0; r < 16; r++) o[b][r] = 0.0f;

  for (int t = wv; t < ntiles; t += NW) {
    const int kb = t * 32;
    // the key tile, transposed into LDS
#pragma unroll
    for (int u = 0; u < DH / 8; u++) {
      const int f = lane + 64 * u, key = f / (DH / 4), d4 = f % (DH / 4);
      W[wv].Kt[4 * d4 + 0][key] = kreg[u].x;
      W[wv].Kt[4 * d4 + 1][key] = kreg[u].y;
      W[wv].Kt[4 * d4 + 2][key] = kreg[u].z;
      W[wv].Kt[4 * d4 + 3][key] = kreg[u].w;
    }
    float vreg[DB][16];
#pragma unroll
    for (int s = 0; s < 16; s++) {
      const int kr = min(kb + 8 * (s >> 2) + 4 * half + (s & 3), Tmax - 1);
      const float *vrow = vc + (int64_t)kr * KD + hk * DH + col;
#pragma unroll
      for (int b = 0; b < DB; b++) vreg[b][s] = vrow[32 * b];
    }
    if (t + NW < ntiles) load_k(t + NW);
    __builtin_amdgcn_wave_barrier();
    v16f_t sacc;
#pragma unroll
    for (int r = 0; r < 16; r++) sacc[r] = 0.0f;
#pragma unroll
    for (int s = 0; s < NS; s++) sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(W[wv].Kt[half * NS + s][col], qreg[s], sacc, 0, 0, 0);
    __builtin_amdgcn_wave_barrier();
    // sacc[r] = score of key kb + 8*(r/4) + 4*half + r%4 against query `col`
    float tmax = -INFINITY;
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int key = kb + 8 * (r >> 2) + 4 * half + (r & 3);
      const float sc = (key < Tq) ? sacc[r] * scale : -INFINITY;
      sacc[r] = sc;
      tmax = fmaxf(tmax, sc);
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
    const float m_new = fmaxf(m, tmax);
    const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;  // no key of this tile visible to this query yet
    const float corr = ct_exp(m - m_use);
    float ps = 0.0f;
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const float p = ct_exp(sacc[r] - m_use);
      sacc[r] = p;
      ps += p;
    }
    ps += __shfl_xor(ps, 32, 64);
    l = l * corr + ps;
    m = m_new;
#pragma unroll
    for (int b = 0; b < DB; b++)
#pragma unroll
      for (int r = 0; r < 16; r++) o[b][r] *= corr;
#pragma unroll
    for (int s = 0; s < 16; s++)
#pragma unroll
      for (int b = 0; b < DB; b++) o[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(vreg[b][s], sacc[s], o[b], 0, 0, 0);
  }
  // o[b][r] = unnormalised output element d = 32b + 8*(r/4) + 4*half + r%4 of query `col`
  Cm[wv][lane] = m;
  Cl[wv][lane] = l;
#pragma unroll
  for (int b = 0; b < DB; b++)
#pragma unroll
    for (int r = 0; r < 16; r++) W[wv].Co[b * 16 + r][lane] = o[b][r];
  __syncthreads();
  float M = Cm[0][lane];
#pragma unroll
  for (int w = 1; w < NW; w++) M = fmaxf(M, Cm[w][lane]);  // finite: the wavefront holding key 0 saw it
  float e[NW], L = 0.0f;
#pragma unroll
  for (int w = 0; w < NW; w++) {
    e[w] = (Cm[w][lane] == -INFINITY) ? 0.0f : ct_exp(Cm[w][lane] - M);
    L = fmaf(e[w], Cl[w][lane], L);
  }
  const float inv = 1.0f / L;
  if (i0 + col < S) {
    float *orow = out + ((int64_t)(i0 + col) * H + h) * DH;
    // wavefront wv finishes registers wv * RPW .. of every lane
    constexpr int RPW = DB * 16 / NW;
#pragma unroll
    for (int k = 0; k < RPW; k++) {
      const int R = wv * RPW + k, b = R >> 4, r = R & 15;
      float v = 0.0f;
#pragma unroll
      for (int w = 0; w < NW; w++) v = fmaf(e[w], W[w].Co[R][lane], v);
      orow[32 * b + 8 * (r >> 2) + 4 * half + (r & 3)] = v * inv;
    }
  }
}

// The same prompt attention with bf16 matrix instructions (v_mfma_f32_32x32x16_bf16, 16 times the rate of the
// fp32-operand one): every operand is written as hi + lo bf16 terms and each product as hi*hi + hi*lo + lo*hi, so
// what is dropped is below 2^-16 of a product -- the "two terms" grade of the GEMMs (gemm_precision 2).  With
// fp32 operands the matrix instructions alone are 4096 cycles of a 32-key tile; here they are 768 and the tile is
// bound by the conversions.
//   S^T = K Q^T : lane l feeds K[key l%32][d = 16 s + 8 (l/32) .. +7] (16 bytes of the row-major bf16 copy of
//                 the key tile in LDS) and Q[query l%32][the same d] (registers): 16 keys of ONE query per lane,
//                 key of register r = 8 (r/4) + 4 (l/32) + r%4 as in the fp32 kernel;
//   O^T += V^T P^T : registers 8 t .. 8 t + 7 of a lane are exactly the 8 keys it has to supply for the t-th
//                 16-key slice, so P is packed from its own registers and V[those keys][d = l%32 (+32 per block)]
//                 comes straight from the cache as before.
typedef __bf16 v8bf_t __attribute__((ext_vector_type(8)));
typedef __bf16 v2bf_t __attribute__((ext_vector_type(2)));
typedef float v2f_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ unsigned pk_bf16(float x0, float x1) {  // one v_cvt_pk_bf16_f32, x0 in the low half
  const v2f_t v = {x0, x1};
  return __builtin_bit_cast(unsigned, __builtin_convertvector(v, v2bf_t));
}
// 8 floats -> their bf16 leading terms and the bf16 of what those miss, packed for one matrix operand each
__device__ __forceinline__ void split8(const float *x, v8bf_t &hi, v8bf_t &lo) {
  unsigned h[4], l[4];
#pragma unroll
  for (int k = 0; k < 4; k++) {
    h[k] = pk_bf16(x[2 * k], x[2 * k + 1]);
    l[k] = pk_bf16(x[2 * k] - __uint_as_float(h[k] << 16), x[2 * k + 1] - __uint_as_float(h[k] & 0xffff0000u));
  }
  hi = __builtin_bit_cast(v8bf_t, make_uint4(h[0], h[1], h[2], h[3]));
  lo = __builtin_bit_cast(v8bf_t, make_uint4(l[0], l[1], l[2], l[3]));
}

template <int DH, int NW>
__global__ __launch_bounds__(64 * NW) void k_attn_mfma_bf(float *__restrict__ out, const float *__restrict__ q,
                                                      const float *__restrict__ kc, const float *__restrict__ vc, int S,
                                                      int start_pos, int H, int Hkv) {
  constexpr int NSL = DH / 16;  // 16-wide slices of the head dimension in K Q^T
  constexpr int DB = DH / 32;   // 32-wide blocks of the head dimension
  constexpr int KP = DH + 8;    // row pitch of the bf16 key tile: 16-byte reads of 8 consecutive rows hit all banks
  // per wavefront: its key tile (hi and lo planes, row-major); once its tiles are done, its unnormalised outputs
  __shared__ union {
    unsigned short K[2][32][KP];
    float Co[DB * 16][64];
  } W[NW];
  __shared__ float Cm[NW][64], Cl[NW][64];
  const int h = blockIdx.x, i0 = (gridDim.y - 1 - blockIdx.y) * 32;  // the longest groups are dispatched first
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int half = lane >> 5, col = lane & 31;
  const int hk = h / (H / Hkv), KD = Hkv * DH;
  const int qrow = min(i0 + col, S - 1);  // rows past the end repeat the last one and are not stored
  const int Tq = start_pos + qrow + 1;    // keys this lane's query sees
  const int Tmax = start_pos + min(i0 + 32, S);
  const int ntiles = (Tmax + 31) / 32;
  const float scale = 1.0f / sqrtf((float)DH);
  // the key tile of a pass is requested one pass ahead, its values at the start of the pass
  float4 kreg[DH / 8];
  auto load_k = [&](int t) {
#pragma unroll
    for (int u = 0; u < DH / 8; u++) {
      const int f = lane + 64 * u, key = f / (DH / 4), d4 = f % (DH / 4);
      const int kr = min(t * 32 + key, Tmax - 1);  // rows clamped to the last visible one: masked below
      kreg[u] = *(const float4 *)(kc + (int64_t)kr * KD + hk * DH + 4 * d4);
    }
  };
  if (wv < ntiles) load_k(wv);
  // the block's 32 query rows through LDS (the memory of the key tiles, before they are written), see k_attn_mfma
  constexpr int QP = DH + 4;
  static_assert(32 * QP * 4 <= sizeof(W), "the query rows fit the key tile memory");
  float(*Qs)[QP] = reinterpret_cast<float(*)[QP]>(&W[0]);
  for (int f = tid; f < 8 * DH; f += 64 * NW) {
    const int row = f / (DH / 4), c4 = f % (DH / 4);
    *(float4 *)&Qs[row][4 * c4] = *(const float4 *)(q + ((int64_t)min(i0 + row, S - 1) * H + h) * DH + 4 * c4);
  }
  __syncthreads();
  v8bf_t qh[NSL], ql[NSL];  // slice s of this lane: d = 16 s + 8 half .. +7
#pragma unroll
  for (int s = 0; s < NSL; s++) {
    const float4 t0 = *(const float4 *)&Qs[col][16 * s + 8 * half], t1 = *(const float4 *)&Qs[col][16 * s + 8 * half + 4];
    const float x[8] = {t0.x, t0.y, t0.z, t0.w, t1.x, t1.y, t1.z, t1.w};
    split8(x, qh[s], ql[s]);
  }
  __syncthreads();  // the key tiles may overwrite the rows now
  float m = -INFINITY, l = 0.0f;
  v16f_t o[DB];
#pragma unroll
  for (int b = 0; b < DB; b++)
#pragma unroll
    for (int r = 0; r < 16; r++) o[b][r] = 0.0f;

  for (int t = wv; t < ntiles; t += NW) {
    const int kb = t * 32;
    // the key tile, split, into LDS
#pragma unroll
    for (int u = 0; u < DH / 8; u++) {
      const int f = lane + 64 * u, key = f / (DH / 4), d4 = f % (DH / 4);
      const unsigned h0 = pk_bf16(kreg[u].x, kreg[u].y), h1 = pk_bf16(kreg[u].z, kreg[u].w);
      const unsigned l0 = pk_bf16(kreg[u].x - __uint_as_float(h0 << 16), kreg[u].y - __uint_as_float(h0 & 0xffff0000u));
      const unsigned l1 = pk_bf16(kreg[u].z - __uint_as_float(h1 << 16), kreg[u].w - __uint_as_float(h1 & 0xffff0000u));
      *(uint2 *)&W[wv].K[0][key][4 * d4] = make_uint2(h0, h1);
      *(uint2 *)&W[wv].K[1][key][4 * d4] = make_uint2(l0, l1);
    }
    float vreg[DB][16];
#pragma unroll
    for (int s = 0; s < 16; s++) {
      const int kr = min(kb + 8 * (s >> 2) + 4 * half + (s & 3), Tmax - 1);
      const float *vrow = vc + (int64_t)kr * KD + hk * DH + col;
#pragma unroll
      for (int b = 0; b < DB; b++) vreg[b][s] = vrow[32 * b];
    }
    if (t + NW < ntiles) load_k(t + NW);
    __builtin_amdgcn_wave_barrier();
    v16f_t sacc;
#pragma unroll
    for (int r = 0; r < 16; r++) sacc[r] = 0.0f;
#pragma unroll
    for (int s = 0; s < NSL; s++) {
      const v8bf_t kh = __builtin_bit_cast(v8bf_t, *(const uint4 *)&W[wv].K[0][col][16 * s + 8 * half]);
      const v8bf_t kl = __builtin_bit_cast(v8bf_t, *(const uint4 *)&W[wv].K[1][col][16 * s + 8 * half]);
      sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kl, qh[s], sacc, 0, 0, 0);  // smallest products first
      sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kh, ql[s], sacc, 0, 0, 0);
      sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kh, qh[s], sacc, 0, 0, 0);
    }
    __builtin_amdgcn_wave_barrier();
    // sacc[r] = score of key kb + 8*(r/4) + 4*half + r%4 against query `col`
    float tmax = -INFINITY;
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int key = kb + 8 * (r >> 2) + 4 * half + (r & 3);
      const float sc = (key < Tq) ? sacc[r] * scale : -INFINITY;
      sacc[r] = sc;
      tmax = fmaxf(tmax, sc);
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
    const float m_new = fmaxf(m, tmax);
    const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;  // no key of this tile visible to this query yet
    const float corr = ct_exp(m - m_use);
    float ps = 0.0f, pr[16];
#pragma unroll
    for (int r = 0; r < 16; r++) {
      pr[r] = ct_exp(sacc[r] - m_use);
      ps += pr[r];
    }
    ps += __shfl_xor(ps, 32, 64);
    l = l * corr + ps;
    m = m_new;
#pragma unroll
    for (int b = 0; b < DB; b++)
#pragma unroll
      for (int r = 0; r < 16; r++) o[b][r] *= corr;
#pragma unroll
    for (int t2 = 0; t2 < 2; t2++) {  // the two 16-key slices of the tile
      v8bf_t ph, pl;
      split8(pr + 8 * t2, ph, pl);
#pragma unroll
      for (int b = 0; b < DB; b++) {
        v8bf_t vh, vl;
        split8(&vreg[b][8 * t2], vh, vl);
        o[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vl, ph, o[b], 0, 0, 0);
        o[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vh, pl, o[b], 0, 0, 0);
        o[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vh, ph, o[b], 0, 0, 0);
      }
    }
  }
  // o[b][r] = unnormalised output element d = 32b + 8*(r/4) + 4*half + r%4 of query `col`
  __builtin_amdgcn_wave_barrier();
  Cm[wv][lane] = m;
  Cl[wv][lane] = l;
#pragma unroll
  for (int b = 0; b < DB; b++)
#pragma unroll
    for (int r = 0; r < 16; r++) W[wv].Co[b * 16 + r][lane] = o[b][r];
  __syncthreads();
  float M = Cm[0][lane];
#pragma unroll
  for (int w = 1; w < NW; w++) M = fmaxf(M, Cm[w][lane]);  // finite: the wavefront holding key 0 saw it
  float e[NW], L = 0.0f;
#pragma unroll
  for (int w = 0; w < NW; w++) {
    e[w] = (Cm[w][lane] == -INFINITY) ? 0.0f : ct_exp(Cm[w][lane] - M);
    L = fmaf(e[w], Cl[w][lane], L);
  }
  const float inv = 1.0f / L;
  if (i0 + col < S) {
    float *orow = out + ((int64_t)(i0 + col) * H + h) * DH;
    constexpr int RPW = DB * 16 / NW;  // wavefront wv finishes registers wv * RPW .. of every lane
#pragma unroll
    for (int k = 0; k < RPW; k++) {
      const int R = wv * RPW + k, b = R >> 4, r = R & 15;
      float v = 0.0f;
#pragma unroll
      for (int w = 0; w < NW; w++) v = fmaf(e[w], W[w].Co[R][lane], v);
      orow[32 * b + 8 * (r >> 2) + 4 * half + (r & 3)] = v * inv;
    }
  }
}

int launch_attn(float *out, const float *q, const float *kc, const float *vc, int S, int start_pos, const int *pos,
                int max_T, int H, int Hkv, int Dh, const AttnSplit *split) {
  if (S == 0) return 0;
  (void)max_T;
  hipStream_t st = state().stream;
  if (S >= 32 && pos == nullptr) {  // prompt rows on the matrix cores
    // eight wavefronts per block where their LDS tiles fit (head_dim <= 64), four otherwise
    dim3 grid(H, (S + 31) / 32);
    if (state().gemm_precision == 0) {  // fp32 operands asked for: the products are fp32 products
      switch (Dh) {
        case 32: hipLaunchKernelGGL((k_attn_mfma<32, 8>), grid, dim3(512), 0, st, out, q, kc, vc, S, start_pos, H, Hkv); break;
        case 64: hipLaunchKernelGGL((k_attn_mfma<64, 8>), grid, dim3(512), 0, st, out, q, kc, vc, S, start_pos, H, Hkv); break;
        case 128: hipLaunchKernelGGL((k_attn_mfma<128, 4>), grid, dim3(256), 0, st, out, q, kc, vc, S, start_pos, H, Hkv); break;
        default: return fail(CTHIP_E_UNSUPPORTED, "attention: head_dim %d (supported: 32, 64, 128)", Dh);
      }
    } else {  // two bf16 terms per operand, whatever the GEMMs use
      switch (Dh) {
        case 32: hipLaunchKernelGGL((k_attn_mfma_bf<32, 8>), grid, dim3(512), 0, st, out, q, kc, vc, S, start_pos, H, Hkv); break;
        case 64: hipLaunchKernelGGL((k_attn_mfma_bf<64, 8>), grid, dim3(512), 0, st, out, q, kc, vc, S, start_pos, H, Hkv); break;
        case 128: hipLaunchKernelGGL((k_attn_mfma_bf<128, 4>), grid, dim3(256), 0, st, out, q, kc, vc, S, start_pos, H, Hkv); break;
        default: return fail(CTHIP_E_UNSUPPORTED, "attention: head_dim %d (supported: 32, 64, 128)", Dh);
      }
    }
    CTHIP_LAUNCH_CHECK();
    return 0;
  }
  constexpr int R = 8;
  if (S >= 2 * R) {  // short prompts: groups of R rows share their K / V loads
    dim3 grid(H, (S + R - 1) / R), block(256);
    switch (Dh) {
      case 32: hipLaunchKernelGGL((k_attn_rows<32, R>), grid, block, 0, st, out, q, kc, vc, S, start_pos, pos, H, Hkv); break;
      case 64: hipLaunchKernelGGL((k_attn_rows<64, R>), grid, block, 0, st, out, q, kc, vc, S, start_pos, pos, H, Hkv); break;
      case 128: hipLaunchKernelGGL((k_attn_rows<128, R>), grid, block, 0, st, out, q, kc, vc, S, start_pos, pos, H, Hkv); break;
      default: return fail(CTHIP_E_UNSUPPORTED, "attention: head_dim %d (supported: 32, 64, 128)", Dh);
    }
    CTHIP_LAUNCH_CHECK();
    return 0;
  }
  float *kcw = const_cast<float *>(kc), *vcw = const_cast<float *>(vc);
  const float *nokv = nullptr;
  float *nop = nullptr;
  int *noc = nullptr;
  if (split && split->ranges > kAttnSplitMaxRanges) return fail(CTHIP_E_BAD_ARG, "attention: %d key ranges per head (at most %d)", split->ranges, kAttnSplitMaxRanges);
  if (S == 1 && split && split->ranges > 1) {  // one row over a context that may be long: the keys shared by several workgroups
    dim3 grid(H, 1, split->ranges), block(1024);
    switch (Dh) {
      case 32: hipLaunchKernelGGL((k_attn_cached<32, false, true>), grid, block, 0, st, out, q, kcw, vcw, start_pos, pos, H, Hkv, nokv, 0.0f, split->part, split->count); break;
      case 64: hipLaunchKernelGGL((k_attn_cached<64, false, true>), grid, block, 0, st, out, q, kcw, vcw, start_pos, pos, H, Hkv, nokv, 0.0f, split->part, split->count); break;
      case 128: hipLaunchKernelGGL((k_attn_cached<128, false, true>), grid, block, 0, st, out, q, kcw, vcw, start_pos, pos, H, Hkv, nokv, 0.0f, split->part, split->count); break;
      default: return fail(CTHIP_E_UNSUPPORTED, "attention: head_dim %d (supported: 32, 64, 128)", Dh);
    }
    CTHIP_LAUNCH_CHECK();
    return 0;
  }
  dim3 grid(H, S), block(1024);
  switch (Dh) {
    case 32: hipLaunchKernelGGL((k_attn_cached<32, false, false>), grid, block, 0, st, out, q, kcw, vcw, start_pos, pos, H, Hkv, nokv, 0.0f, nop, noc); break;
    case 64: hipLaunchKernelGGL((k_attn_cached<64, false, false>), grid, block, 0, st, out, q, kcw, vcw, start_pos, pos, H, Hkv, nokv, 0.0f, nop, noc); break;
    case 128: hipLaunchKernelGGL((k_attn_cached<128, false, false>), grid, block, 0, st, out, q, kcw, vcw, start_pos, pos, H, Hkv, nokv, 0.0f, nop, noc); break;
    default: return fail(CTHIP_E_UNSUPPORTED, "attention: head_dim %d (supported: 32, 64, 128)", Dh);
  }
  CTHIP_LAUNCH_CHECK();
  return 0;
}

// one decode row of a RoPE model: rotates q and the new key, appends k / v at `pos`, attends (see k_attn_cached)
int launch_attn_rope_append(float *out, const float *q, float *kc, float *vc, const float *newkv, const int *pos, int H,
                            int Hkv, int Dh, float base, const AttnSplit *split) {
  hipStream_t st = state().stream;
  const float lb = log2f(base);
  if (split && split->ranges > kAttnSplitMaxRanges) return fail(CTHIP_E_BAD_ARG, "attention: %d key ranges per head (at most %d)", split->ranges, kAttnSplitMaxRanges);
  if (split && split->ranges > 1) {
    dim3 grid(H, 1, split->ranges), block(1024);
    switch (Dh) {
      case 32: hipLaunchKernelGGL((k_attn_cached<32, true, true>), grid, block, 0, st, out, q, kc, vc, 0, pos, H, Hkv, newkv, lb, split->part, split->count); break;
      case 64: hipLaunchKernelGGL((k_attn_cached<64, true, true>), grid, block, 0, st, out, q, kc, vc, 0, pos, H, Hkv, newkv, lb, split->part, split->count); break;
      case 128: hipLaunchKernelGGL((k_attn_cached<128, true, true>), grid, block, 0, st, out, q, kc, vc, 0, pos, H, Hkv, newkv, lb, split->part, split->count); break;
      default: return fail(CTHIP_E_UNSUPPORTED, "attention: head_dim %d (supported: 32, 64, 128)", Dh);
    }
    CTHIP_LAUNCH_CHECK();
    return 0;
  }
  dim3 grid(H, 1), block(1024);
  float *nop = nullptr;
  int *noc = nullptr;
  switch (Dh) {
    case 32: hipLaunchKernelGGL((k_attn_cached<32, true, false>), grid, block, 0, st, out, q, kc, vc, 0, pos, H, Hkv, newkv, lb, nop, noc); break;
    case 64: hipLaunchKernelGGL((k_attn_cached<64, true, false>), grid, block, 0, st, out, q, kc, vc, 0, pos, H, Hkv, newkv, lb, nop, noc); break;
    case 128: hipLaunchKernelGGL((k_attn_cached<128, true, false>), grid, block, 0, st, out, q, kc, vc, 0, pos, H, Hkv, newkv, lb, nop, noc); break;
    default: return fail(CTHIP_E_UNSUPPORTED, "attention: head_dim %d (supported: 32, 64, 128)", Dh);
  }
  CTHIP_LAUNCH_CHECK();
  return 0;
}

int launch_embedding(float *out, const float *W, const float *idx_f, const int *idx_i, int ntok, int vocab, int dim,
                     const float *W2, const int *pos, int max_pos) {
  if (ntok == 0) return 0;
  hipLaunchKernelGGL(k_embedding, dim3(ntok), dim3(256), 0, state().stream, out, W, idx_f, idx_i, vocab, dim, W2, pos,
                     max_pos);
  CTHIP_LAUNCH_CHECK();
  return 0;
}

int launch_embedding_rows(float *out, const float *W, long long first, long long step, int ntok, int vocab, int dim, const float *addend) {
  if (ntok == 0) return 0;
  hipLaunchKernelGGL(k_embedding_rows, dim3(ntok), dim3(256), 0, state().stream, out, W, first, step, vocab, dim, addend);
  CTHIP_LAUNCH_CHECK();
  return 0;
}

int launch_argmax(int64_t *out, const float *x, int64_t rows, int n, int *tok_out, int *pos, int64_t *history,
                  int *hist_n) {
  if (rows == 0) return 0;
  static_assert(kArgmaxParts == 64, "k_argmax_settle reads one part per lane");
  if (rows <= 16 && n >= 8192) {  // few long rows: parts of a row in parallel, then one wavefront per row
    float *pv = nullptr;
    int rc = alloc_scratch((void **)&pv, (size_t)rows * kArgmaxParts * 8);
    if (rc) return rc;
    int *pi = (int *)(pv + rows * kArgmaxParts);
    hipLaunchKernelGGL(k_argmax_parts, dim3((unsigned)rows, kArgmaxParts), dim3(256), 0, state().stream, pv, pi, x, n);
    hipError_t e = hipGetLastError();
    if (e == hipSuccess) {
      hipLaunchKernelGGL(k_argmax_settle, dim3((unsigned)rows), dim3(64), 0, state().stream, out, pv, pi, tok_out, pos, history, hist_n);
      e = hipGetLastError();
    }
    rc = cthip_free(pv);  // stream-ordered: handed out again only to later work on this stream
    if (e != hipSuccess) return fail((int)e, "argmax: launch -> %s", hipGetErrorString(e));
    return rc;
  }
  hipLaunchKernelGGL(k_argmax, dim3((unsigned)rows), dim3(1024), 0, state().stream, out, x, n, tok_out, pos, history,
                     hist_n);
  CTHIP_LAUNCH_CHECK();
  return 0;
}

int launch_rope(float *out, const float *x, int B, int S, int H, int Dh, float base, int start_pos, const int *pos) {
  const int64_t npairs = (int64_t)B * S * H * (Dh / 2);
  if (npairs == 0) return 0;
  hipLaunchKernelGGL(k_rope, dim3((unsigned)((npairs + 255) / 256)), dim3(256), 0, state().stream, out, x, npairs, S, H,
                     Dh, log2f(base), start_pos, pos);
  CTHIP_LAUNCH_CHECK();
  return 0;
}

int launch_qkv_split(float *q, float *kc, float *vc, const float *qkv, int S, int start_pos, int H, int Hkv, int Dh,
                     float rope_base) {
  if (S == 0) return 0;
  hipLaunchKernelGGL(k_qkv_split, dim3(S), dim3(256), 0, state().stream, q, kc, vc, qkv, start_pos, H, Hkv, Dh,
                     rope_base > 0.0f ? log2f(rope_base) : 0.0f, rope_base > 0.0f ? 1 : 0);
  CTHIP_LAUNCH_CHECK();
  return 0;
}

int launch_rope_append(float *kc, float *vc, const float *kv, int Hkv, int Dh, float base, const int *pos) {
  const int pairs = Hkv * Dh / 2;
  hipLaunchKernelGGL(k_rope_append, dim3((pairs + 255) / 256), dim3(256), 0, state().stream, kc, vc, kv, Hkv, Dh,
                     log2f(base), pos);
  CTHIP_LAUNCH_CHECK();
  return 0;
}

}  // namespace cthip

using namespace cthip;

extern "C" {

int cthip_softmax(float *y, const float *x, int64_t rows, int n) {
  CTHIP_REQUIRE_INIT();
  CTHIP_ARG(rows >= 0 && n >= 0 && (rows * n == 0 || (y && x)));
  RowArgs a = {y, x, nullptr, nullptr, 0.0f, rows, n};
  return launch_rowop<ROW_SOFTMAX>(a);
}

int cthip_layernorm(float *y, const float *x, const float *gamma, const float *beta, float eps, int64_t rows, int n) {
  CTHIP_REQUIRE_INIT();
  CTHIP_ARG(rows >= 0 && n >= 0 && (rows * n == 0 || (y && x)));
  RowArgs a = {y, x, gamma, beta, eps, rows, n};
  return launch_rowop<ROW_LAYERNORM>(a);
}

int cthip_rmsnorm(float *y, const float *x, const float *w, float eps, int64_t rows, int n) {
  CTHIP_REQUIRE_INIT();
  CTHIP_ARG(rows >= 0 && n >= 0 && (rows * n == 0 || (y && x)));
  RowArgs a = {y, x, w, nullptr, eps, rows, n};
  return launch_rowop<ROW_RMSNORM>(a);
}

int cthip_layernorm_softmax(float *y, const float *x, const float *gamma, const float *beta, float eps, int64_t rows,
                            int n) {
  CTHIP_REQUIRE_INIT();
  CTHIP_ARG(rows >= 0 && n >= 0 && (rows * n == 0 || (y && x)));
  RowArgs a = {y, x, gamma, beta, eps, rows, n};
  return launch_rowop<ROW_LN_SOFTMAX>(a);
}

int cthip_unary(int kind, float *y, const float *x, int64_t n) {
  CTHIP_REQUIRE_INIT();
  CTHIP_ARG(n >= 0 && (n == 0 || (y && x)));
  CTHIP_ARG(kind >= CTHIP_ACT_NONE && kind <= CTHIP_ACT_TANH);
  if (n == 0) return 0;
  const bool vec = ((uintptr_t)x % 16 == 0) && ((uintptr_t)y % 16 == 0);
  const int64_t per = vec ? 4096 : 1024, blocks = (n + per - 1) / per;
  if (blocks > 0x7fffffff) return fail(CTHIP_E_BAD_ARG, "cthip_unary: %lld elements exceed the grid", (long long)n);
  if (vec) hipLaunchKernelGGL(k_unary<4>, dim3((unsigned)blocks), dim3(256), 0, state().stream, kind, y, x, n);
  else hipLaunchKernelGGL(k_unary<1>, dim3((unsigned)blocks), dim3(256), 0, state().stream, kind, y, x, n);
  CTHIP_LAUNCH_CHECK();
  return 0;
}

int cthip_embedding(float *out, const float *W, const float *idx, int ntok, int vocab, int dim) {
  CTHIP_REQUIRE_INIT();
  CTHIP_ARG(ntok >= 0 && vocab > 0 && dim > 0 && (ntok == 0 || (out && W && idx)));
  return launch_embedding(out, W, idx, nullptr, ntok, vocab, dim, nullptr, nullptr, 0);
}

int cthip_argmax(int64_t *out, const float *x, int64_t rows, int n) {
  CTHIP_REQUIRE_INIT();
  CTHIP_ARG(rows >= 0 && n > 0 && (rows == 0 || (out && x)));
  if (rows > 0x7fffffff) return fail(CTHIP_E_BAD_ARG, "cthip_argmax: too many rows");
  return launch_argmax(out, x, rows, n, nullptr, nullptr, nullptr, nullptr);
}

int cthip_rope(float *out, const float *x, int B, int S, int H, int Dh, float base, int start_pos) {
  CTHIP_REQUIRE_INIT();
  CTHIP_ARG(B >= 0 && S >= 0 && H >= 0 && Dh >= 0 && Dh % 2 == 0 && base > 0.0f);
  CTHIP_ARG((int64_t)B * S * H * Dh == 0 || (out && x));
  return launch_rope(out, x, B, S, H, Dh, base, start_pos, nullptr);
}

int cthip_sdpa_cached(float *out, const float *q, const float *k_cache, const float *v_cache, int S, int start_pos,
                      int H, int Hkv, int Dh) {
  CTHIP_REQUIRE_INIT();
  CTHIP_ARG(S >= 0 && start_pos >= 0 && H > 0 && Hkv > 0 && H % Hkv == 0);
  CTHIP_ARG(S == 0 || (out && q && k_cache && v_cache));
  return launch_attn(out, q, k_cache, v_cache, S, start_pos, nullptr, start_pos + S, H, Hkv, Dh, nullptr);
}

}  // extern "C"
