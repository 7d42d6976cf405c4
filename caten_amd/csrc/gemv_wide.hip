// Single-row Linear for rows of any width LDS can hold (every weight format), streamed with the input vector in LDS.
//
// The register-resident kernels (gemv_kernels.h) give every lane its share of the input vector for the whole
// launch: 128 floats per lane at 8192 columns of 4-bit weights, which is 304 registers and one wavefront per SIMD
// (measured 3.65 TB/s on a 264 MB matrix), and nothing at all past 8192 columns.  Here a workgroup of eight
// wavefronts stages the vector once -- with its prologue: SwiGLU, or an RMSNorm folded through the product
// (gamma * x staged, the row's sum multiplied by rstd at the end) -- and every wavefront streams whole rows: lane l
// takes chunks l, l + 64, ... of the row, a tile is NC such rounds of RW rows requested together, PD = 12 / (NC RW)
// tiles are in flight per wavefront across row boundaries (twelve 16-byte requests per lane), all requests
// unconditional (rows past the end repeat the last row and are not stored; chunks past the end of a row read a zero
// block).  A chunk's 16 / 32 input floats are read from
// LDS when its weights have arrived; float4 t of chunk c is stored at position t ^ (c mod 4 or 8) of the chunk, so
// that the 16-byte reads of neighbouring lanes, 64 or 128 bytes apart, spread over the banks.  4-bit weights need
// the sum of a chunk's inputs (q - 8 = q minus a constant): one float per chunk, computed once after the staging.
// Where there are rows enough to fill the device twice over, a wavefront streams two neighbouring rows at a time
// against one read of the inputs: the LDS traffic per weight byte is what bounds the kernel then (eight input bytes
// per 4-bit weight byte), and two rows halve it (Llama-70B shape: 11.1 -> 10.4 ms per step); with fewer rows the
// pairs would leave wavefront slots empty (GPT-2 XL's 1600 x 6400 projection, the 13B shape's 5120 x 13824).
#include <map>

#include "common.h"
#include "gemv_kernels.h"
#include "gemv_plan.h"

namespace cthip {

template <int F4>
__device__ __forceinline__ int wide_slot(int i) {  // float4 index -> where it is kept
  return (i & ~(F4 - 1)) | ((i ^ (i / F4)) & (F4 - 1));
}

template <int TYPE, int NC, int RW, bool NT, int PDX = 0>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(4, 4)))
void k_gemv_wide(GemvArgs a, int tpr) {
  // (PDX: a shorter ring for launches in which no wavefront has as many tiles as the full one holds)
  constexpr int XPC = Fmt<TYPE>::XPC, F4 = XPC / 4, PD = PDX ? PDX : 12 / (NC * RW);
  constexpr bool Q4 = TYPE == CTHIP_Q4_0, QUANT = TYPE == CTHIP_Q4_0 || TYPE == CTHIP_Q8_0;
  extern __shared__ float wide_lds[];
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int nchunks = a.cols / XPC, n4 = a.cols >> 2;
  float *xs = wide_lds, *csum = wide_lds + a.cols, *red = csum + (Q4 ? nchunks : 0);
  const int m = blockIdx.y;
  const float *__restrict__ x = a.x + (int64_t)m * a.x_stride;
  const uint4 *__restrict__ qp = (const uint4 *)a.q;
  const int scales_per_row = a.cols >> 5;
  const int wave = blockIdx.x * 8 + wv, total_waves = gridDim.x * 8;
  const int posv = a.pos ? a.pos[0] : 0;
  const bool swiglu = a.pro == CTHIP_PRO_SWIGLU, rms = a.pro == CTHIP_PRO_RMSNORM;
  // row groups wave, wave + total_waves, ... (group i = rows RW i .. RW i + RW - 1, RW = 1 or 2): nt tiles in all
  const int npairs = (a.rows + RW - 1) / RW;
  const int pairs_w = wave < npairs ? (npairs - wave + total_waves - 1) / total_waves : 0;
  const int nt = pairs_w * tpr;

  // ---- the weight ring ----
  uint4 wt[PD][RW][NC];
  unsigned st[PD][RW][NC];
  float epi_t[PD];
  int rq_pair = wave < npairs ? wave : npairs - 1, rq_grp = 0, rq_left = nt;  // the next tile to request
  auto request = [&](int p) {
    const int row0 = RW * rq_pair, row1 = min(row0 + RW - 1, a.rows - 1);  // (an odd last row is read twice, stored once)
#pragma unroll
    for (int k = 0; k < NC; k++) {
      const int c = (rq_grp * NC + k) * 64 + lane;
      const bool ok = c < nchunks;
      const int sidx = Q4 ? c : c >> 1;
      wt[p][0][k] = load_chunk<NT>(ok ? qp + (int64_t)row0 * nchunks + c : (const uint4 *)g_gemv_zeros);
      if (RW > 1) wt[p][RW - 1][k] = load_chunk<NT>(ok ? qp + (int64_t)row1 * nchunks + c : (const uint4 *)g_gemv_zeros);
      if (QUANT) {
        st[p][0][k] = *(ok ? a.d + (int64_t)row0 * scales_per_row + sidx : (const unsigned short *)g_gemv_zeros);
        if (RW > 1) st[p][RW - 1][k] = *(ok ? a.d + (int64_t)row1 * scales_per_row + sidx : (const unsigned short *)g_gemv_zeros);
      }
    }
    // the rows' bias and residual travel with their tiles: lanes 0, 1 ask for row0's, lanes 2, 3 for row1's
    const int er = (lane & 2) ? row1 : row0;
    const float *pb = a.bias ? a.bias + er : nullptr;
    const float *pr = a.residual ? a.residual + (int64_t)m * a.y_stride + er : nullptr;
    const float *any = pb ? pb : pr ? pr : (const float *)g_gemv_zeros;
    epi_t[p] = *((lane & 1) ? (pr ? pr : any) : (pb ? pb : any));
    // advance; past the last tile the last one is requested again (and never consumed)
    if (rq_left > 1) {
      rq_left--;
      if (++rq_grp == tpr) {
        rq_grp = 0;
        rq_pair += total_waves;
      }
    }
  };
  request(0);  // goes out before the staging: its answer arrives while the vector is being prepared

  // ---- the input vector ----
  const float4 *x4 = (const float4 *)x;
  const float4 *u4 = swiglu ? (const float4 *)(x + a.cols) : (rms && a.norm_g) ? (const float4 *)a.norm_g : x4;
  float s2 = 0.0f;
  // SB pieces of the vector (and of its partner: SwiGLU's other half, the norm's gamma) are asked for together: a
  // piece per loop iteration would cost a memory round trip each
  constexpr int SB = 6;
  for (int i0 = tid; i0 < n4; i0 += 512 * SB) {
    float4 vb[SB], ub[SB];
#pragma unroll
    for (int b = 0; b < SB; b++) {
      const int i = min(i0 + 512 * b, n4 - 1);
      vb[b] = x4[i];
      ub[b] = u4[i];
    }
#pragma unroll
    for (int b = 0; b < SB; b++) {
      const int i = i0 + 512 * b;
      if (i < n4) {
        const float4 v = vb[b], u = ub[b];
        float4 o = v;
        if (swiglu) o = make_float4(ct_silu(v.x) * u.x, ct_silu(v.y) * u.y, ct_silu(v.z) * u.z, ct_silu(v.w) * u.w);
        if (rms) {
          s2 = fmaf(v.x, v.x, fmaf(v.y, v.y, fmaf(v.z, v.z, fmaf(v.w, v.w, s2))));
          if (a.norm_g) o = make_float4(v.x * u.x, v.y * u.y, v.z * u.z, v.w * u.w);
        }
        ((float4 *)xs)[wide_slot<F4>(i)] = o;
      }
    }
  }
  if (rms) {
    s2 = wave_sum(s2);
    if (lane == 0) red[wv] = s2;
  }
  __syncthreads();
  float rstd = 1.0f;
  if (rms) {
    float t = 0.0f;
#pragma unroll
    for (int w = 0; w < 8; w++) t += red[w];
    rstd = 1.0f / sqrtf(t / (float)a.cols + a.eps);
  }
  if (Q4) {
    for (int c = tid; c < nchunks; c += 512) {
      float s = 0.0f;
#pragma unroll
      for (int t = 0; t < F4; t++) {
        const float4 v = ((const float4 *)xs)[F4 * c + (t ^ (c & (F4 - 1)))];
        s += (v.x + v.y) + (v.z + v.w);
      }
      csum[c] = s;
    }
    __syncthreads();
  }
#pragma unroll
  for (int p = 1; p < PD; p++) request(p);

  // ---- stream ----
  float acc0 = 0.0f, acc1 = 0.0f, row_epi = 0.0f;
  int cs_pair = wave, cs_grp = 0;  // the tile being consumed
  auto consume = [&](int p) {
    if (cs_grp == 0) row_epi = epi_t[p];
#pragma unroll
    for (int k = 0; k < NC; k++) {
      const int c = (cs_grp * NC + k) * 64 + lane;
      const int cl = c < nchunks ? c : nchunks - 1;  // (a chunk past the end has zero weights and a zero scale)
      float xl[XPC];
#pragma unroll
      for (int t = 0; t < F4; t++) {
        const float4 v = ((const float4 *)xs)[F4 * cl + (t ^ (cl & (F4 - 1)))];
        xl[4 * t] = v.x, xl[4 * t + 1] = v.y, xl[4 * t + 2] = v.z, xl[4 * t + 3] = v.w;
      }
      const float cs = Q4 ? csum[cl] : 0.0f;
      acc0 += chunk_dot<TYPE>(wt[p][0][k], QUANT ? half_bits_to_float((unsigned short)st[p][0][k]) : 1.0f, xl, cs);
      if (RW > 1) acc1 += chunk_dot<TYPE>(wt[p][RW - 1][k], QUANT ? half_bits_to_float((unsigned short)st[p][RW - 1][k]) : 1.0f, xl, cs);
    }
    if (++cs_grp == tpr) {  // (uniform) the pair of rows is complete
      const float s0 = wave_sum(acc0) * rstd, s1 = RW > 1 ? wave_sum(acc1) * rstd : 0.0f;
      const int row0 = RW * cs_pair;
      const float b0 = a.bias ? __shfl(row_epi, 0, 64) : 0.0f, r0 = a.residual ? __shfl(row_epi, 1, 64) : 0.0f;
      const float b1 = a.bias ? __shfl(row_epi, 2, 64) : 0.0f, r1 = a.residual ? __shfl(row_epi, 3, 64) : 0.0f;
      if (RW > 1 && a.pair_swiglu) {  // the pair is a (gate, up) row pair: SwiGLU here, one output per pair
        if (lane == 0) a.y[(int64_t)m * a.y_stride + (row0 >> 1)] = ct_silu(s0 + b0) * (s1 + b1);
      } else {
        if (lane == 0) gemv_store(a, m, row0, s0, posv, b0, r0);
        if (RW > 1 && lane == 1 && row0 + 1 < a.rows) gemv_store(a, m, row0 + 1, s1, posv, b1, r1);
      }
      acc0 = acc1 = 0.0f;
      cs_grp = 0;
      cs_pair += total_waves;
    }
  };
  int t = 0;
  for (; t + PD <= nt; t += PD) {
#pragma unroll
    for (int p = 0; p < PD; p++) {
      consume(p);
      request(p);
    }
  }
#pragma unroll
  for (int p = 0; p < PD; p++)
    if (t + p < nt) consume(p);  // (uniform)
}

// true when the launch is one this kernel runs: quantised rows that LDS holds, no LayerNorm, no fused argmax, no
// paired epilogue
bool gemv_wide_supported(const WMat *w, const GemvArgs &a) {
  if (a.pro == CTHIP_PRO_LAYERNORM || a.fold_s || a.am_val) return false;
  const GemvWidePlan p = gemv_wide_plan(w->type, w->rows, w->cols, state().compute_units);
  // the paired SwiGLU epilogue: a wavefront must hold a (gate, up) row pair, outputs plain
  if (a.pair_swiglu && (p.rw != 2 || (w->rows & 1) || a.residual || a.act != CTHIP_ACT_NONE || (a.split1 > 0 && a.split1 != (int)w->rows))) return false;
  return p.ok;
}

int launch_gemv_wide(const WMat *w, GemvArgs a, int m) {
  State &s = state();
  const GemvWidePlan p = gemv_wide_plan(w->type, w->rows, w->cols, s.compute_units);
  if (!p.ok) return fail(CTHIP_E_UNSUPPORTED, "gemv: no wide-row launch for a (%lld, %lld) matrix of type %d", (long long)w->rows, (long long)w->cols, w->type);
  a.q = w->q;
  a.d = (const unsigned short *)w->d;
  a.rows = (int)w->rows;
  a.cols = (int)w->cols;
  a.ld_chunks = a.ld_scales = a.up_off = 0;
  if (a.split1 <= 0) a.split1 = a.split2 = a.rows;
  const bool nt = s.gemv_stream < 0 ? w->stream : s.gemv_stream != 0;
  typedef void (*wide_fn)(GemvArgs, int);
  wide_fn fn = nullptr;
#define PICK(T, NC_)                                                                                                  \
  if (w->type == T && p.nc == NC_)                                                                                    \
    fn = p.rw == 2 ? (nt ? k_gemv_wide<T, NC_, 2, true> : k_gemv_wide<T, NC_, 2, false>)                              \
                   : (nt ? k_gemv_wide<T, NC_, 1, true> : k_gemv_wide<T, NC_, 1, false>);
  PICK(CTHIP_Q4_0, 1)
  PICK(CTHIP_Q8_0, 1) PICK(CTHIP_Q8_0, 2) PICK(CTHIP_Q8_0, 3)
  PICK(CTHIP_F16, 1) PICK(CTHIP_F16, 2) PICK(CTHIP_F16, 3)
  PICK(CTHIP_F32, 1) PICK(CTHIP_F32, 2) PICK(CTHIP_F32, 3)
#undef PICK
  // 8-bit rows, one per wavefront and tile, no wavefront with more than six (eight) tiles: a ring of six (eight), so
  // that no slot asks for the last tile again (GPT-2 XL's 1600 x 6400 projection: 1.507 -> 1.469 ms per step; the
  // 4-bit rows of the 7B shape were 2 % slower with the shorter ring and keep the full one)
  if (p.rw == 1 && p.nc == 1 && w->type == CTHIP_Q8_0) {
    const long long waves = (long long)p.grid * 8, rows_w = (w->rows + waves - 1) / waves, tiles_w = rows_w * p.tpr;
    if (tiles_w <= 6) fn = nt ? k_gemv_wide<CTHIP_Q8_0, 1, 1, true, 6> : k_gemv_wide<CTHIP_Q8_0, 1, 1, false, 6>;
    else if (tiles_w <= 8) fn = nt ? k_gemv_wide<CTHIP_Q8_0, 1, 1, true, 8> : k_gemv_wide<CTHIP_Q8_0, 1, 1, false, 8>;
  }
  if (!fn) return fail(CTHIP_E_STATE, "gemv: no wide-row kernel for %d rounds per tile", p.nc);
  const size_t lds = p.lds_floats * sizeof(float);
  if (lds > 64 * 1024) {
    // (set once per kernel: the largest request so far)
    static std::map<const void *, size_t> granted;
    size_t &g = granted[(const void *)fn];
    if (lds > g) {
      CTHIP_CHECK(hipFuncSetAttribute((const void *)fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kGemvWideMaxLdsBytes));
      g = kGemvWideMaxLdsBytes;
    }
  }
  hipLaunchKernelGGL(fn, dim3(p.grid, (unsigned)m), dim3(p.block), lds, s.stream, a, p.tpr);
  CTHIP_LAUNCH_CHECK();
  return 0;
}

}  // namespace cthip
