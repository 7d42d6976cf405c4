// GGUF block codecs, the packed weight matrix, and the dequant-in-register
// GEMV that carries batch-1 decode (Linear, source/nn/linear.lisp:3-17, with
// the LayerNorm/RMSNorm/SwiGLU prologue and bias/activation/residual epilogue
// that Caten's scheduler fuses around a matmul, test-scheduler.lisp:140-163).
//
// HBM layout of a packed matrix (rows x cols):
//   quant plane  Q8_0: int8  [rows][cols]      Q4_0: u8 [rows][cols/2]
//                F32 : float [rows][cols]      F16 : half [rows][cols]
//   scale plane  fp16 [rows][cols/32]          (quantised types only)
// Q4_0 keeps ggml's nibble order inside each 16-byte block (low nibbles are
// elements 0..15, high nibbles 16..31).  Total bytes equal the GGUF bytes, but
// every lane can issue aligned 128-bit loads, which the 34/18-byte GGUF blocks
// do not allow.
//
// GEMV work distribution: a row is owned by an aligned group of G lanes
// (G = 16, 32 or 64; 64/G rows per wavefront), lane l of the group streams the
// 16-byte chunks l, l+G, l+2G, ... (KC of them) of the row.  The slice of the
// input vector that multiplies those chunks is loaded ONCE per wavefront into
// registers (after applying the fused prologue) and reused for every row the
// wavefront visits, so the steady state touches nothing but weights.  Partial
// sums are combined with DPP/shuffle steps inside the group and the group's
// first lane applies the epilogue.
#include <stdlib.h>
#include <string.h>

#include <vector>

#include "common.h"
#include "gemv_kernels.h"
#include "gemv_plan.h"

namespace cthip {

// ------------------------------------------------------------------ codecs
__global__ void k_dequant_q8_0_raw(const uint8_t *__restrict__ raw, int64_t n, float *__restrict__ out) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  int64_t b = i >> 5;
  int j = (int)(i & 31);
  const uint8_t *p = raw + 34 * b;
  float scale = half_bits_to_float((unsigned short)(p[0] | (p[1] << 8)));
  out[i] = (float)(int8_t)p[2 + j] * scale;
}

__global__ void k_dequant_q4_0_raw(const uint8_t *__restrict__ raw, int64_t n, float *__restrict__ out) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  int64_t b = i >> 5;
  int j = (int)(i & 31);
  const uint8_t *p = raw + 18 * b;
  float d = half_bits_to_float((unsigned short)(p[0] | (p[1] << 8)));
  int byte = p[2 + (j & 15)];
  int nib = (j < 16) ? (byte & 0x0f) : (byte >> 4);
  out[i] = (float)(nib - 8) * d;
}

__global__ void k_dequant_f16_raw(const uint8_t *__restrict__ raw, int64_t n, float *__restrict__ out) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  out[i] = half_bits_to_float((unsigned short)(raw[2 * i] | (raw[2 * i + 1] << 8)));
}

__global__ void k_dequant_f32_raw(const uint8_t *__restrict__ raw, int64_t n, float *__restrict__ out) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  uint32_t u = (uint32_t)raw[4 * i] | ((uint32_t)raw[4 * i + 1] << 8) | ((uint32_t)raw[4 * i + 2] << 16) |
               ((uint32_t)raw[4 * i + 3] << 24);
  out[i] = __uint_as_float(u);
}

// GGUF blocks -> planes. One thread per block.
__global__ void k_repack_q8_0(const uint8_t *__restrict__ raw, int64_t nblocks, uint32_t *__restrict__ q,
                              unsigned short *__restrict__ d) {
  int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= nblocks) return;
  const uint8_t *p = raw + 34 * b;
  d[b] = (unsigned short)(p[0] | (p[1] << 8));
#pragma unroll
  for (int t = 0; t < 8; t++) {
    const uint8_t *s = p + 2 + 4 * t;
    q[8 * b + t] = (uint32_t)s[0] | ((uint32_t)s[1] << 8) | ((uint32_t)s[2] << 16) | ((uint32_t)s[3] << 24);
  }
}

__global__ void k_repack_q4_0(const uint8_t *__restrict__ raw, int64_t nblocks, uint32_t *__restrict__ q,
                              unsigned short *__restrict__ d) {
  int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= nblocks) return;
  const uint8_t *p = raw + 18 * b;
  d[b] = (unsigned short)(p[0] | (p[1] << 8));
#pragma unroll
  for (int t = 0; t < 4; t++) {
    const uint8_t *s = p + 2 + 4 * t;
    q[4 * b + t] = (uint32_t)s[0] | ((uint32_t)s[1] << 8) | ((uint32_t)s[2] << 16) | ((uint32_t)s[3] << 24);
  }
}

// planes -> fp32, one thread per element
__global__ void k_wmat_dequant(int type, const void *__restrict__ qp, const unsigned short *__restrict__ dp,
                               int64_t n, float *__restrict__ out) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  if (type == CTHIP_Q8_0) {
    out[i] = (float)((const int8_t *)qp)[i] * half_bits_to_float(dp[i >> 5]);
  } else if (type == CTHIP_Q4_0) {
    int64_t b = i >> 5;
    int j = (int)(i & 31);
    int byte = ((const uint8_t *)qp)[16 * b + (j & 15)];
    int nib = (j < 16) ? (byte & 0x0f) : (byte >> 4);
    out[i] = (float)(nib - 8) * half_bits_to_float(dp[b]);
  } else if (type == CTHIP_F16) {
    out[i] = half_bits_to_float(((const unsigned short *)qp)[i]);
  } else {
    out[i] = ((const float *)qp)[i];
  }
}

// one block: the greedy token goes where the next step's embedding reads it, is appended to the
// history, and the position advances
__global__ __launch_bounds__(256) void k_argmax_finish(GemvArgs a, int nparts) {
  __shared__ float sv[4];
  __shared__ int si[4];
  __shared__ int next_tok, next_pos;
  // the loop state is requested up front so its latency overlaps the reduction
  int hist_n = 0, pos = 0, eos = -1, stopped = 0, cur_tok = 0;
  if (threadIdx.x == 0) {
    if (a.am_hist) hist_n = *a.am_hist_n;
    if (a.am_pos) pos = *a.am_pos;
    if (a.am_ctrl) {
      eos = a.am_ctrl[0];
      stopped = a.am_ctrl[1];
      cur_tok = a.am_tok ? *a.am_tok : 0;
    }
  }
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  // eight partials per thread are requested together (clamped addresses, no request behind a branch), so the
  // 1 800 partials of a GPT-2 lm_head cost one memory round trip instead of seven dependent ones
  for (int base = 0; base < nparts; base += 8 * 256) {
    float pv[8];
    int pi[8];
#pragma unroll
    for (int k = 0; k < 8; k++) {
      const int i = base + threadIdx.x + 256 * k;
      const int ic = i < nparts ? i : nparts - 1;
      pv[k] = a.am_val[ic];
      pi[k] = a.am_idx[ic];
    }
#pragma unroll
    for (int k = 0; k < 8; k++)
      if (base + threadIdx.x + 256 * k < nparts) argmax_merge(bv, bi, pv[k], pi[k]);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) argmax_merge(bv, bi, __shfl_xor(bv, o, 64), __shfl_xor(bi, o, 64));
  if ((threadIdx.x & 63) == 0) {
    sv[threadIdx.x >> 6] = bv;
    si[threadIdx.x >> 6] = bi;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int k = 1; k < 4; k++) argmax_merge(bv, bi, sv[k], si[k]);
    if (bi == 0x7fffffff) bi = 0;  // no comparable value (all NaN)
    if (stopped) {
      // the sequence has ended: this step (queued before the host could know) leaves the loop state as it is
      next_tok = cur_tok;
      next_pos = pos;
    } else {
      *a.am_token64 = bi;
      if (a.am_tok) *a.am_tok = bi;
      if (a.am_hist) {
        a.am_hist[hist_n] = bi;
        *a.am_hist_n = hist_n + 1;
      }
      if (a.am_pos) *a.am_pos = pos + 1;
      if (a.am_ctrl && bi == eos) a.am_ctrl[1] = 1;
      next_tok = bi;
      next_pos = pos + 1;
    }
  }
  if (a.nx_out) {  // same values as the embedding launch of the next forward would write
    __syncthreads();
    const int id = next_tok, p = next_pos;
    const bool hit = id >= 0 && id < a.nx_vocab, phit = p >= 0 && p < a.nx_max_pos;
    if ((a.nx_dim & 3) == 0) {  // rows are 16-byte aligned: four floats per request
      const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
      for (int d = threadIdx.x; d < (a.nx_dim >> 2); d += 256) {
        const float4 e = hit ? ((const float4 *)(a.nx_wte + (int64_t)id * a.nx_dim))[d] : zero;
        const float4 w = (a.nx_wpe && phit) ? ((const float4 *)(a.nx_wpe + (int64_t)p * a.nx_dim))[d] : zero;
        ((float4 *)a.nx_out)[d] = a.nx_wpe ? make_float4(e.x + w.x, e.y + w.y, e.z + w.z, e.w + w.w) : e;
      }
    } else {
      for (int d = threadIdx.x; d < a.nx_dim; d += 256) {
        float v = hit ? a.nx_wte[(int64_t)id * a.nx_dim + d] : 0.0f;
        if (a.nx_wpe) v += phit ? a.nx_wpe[(int64_t)p * a.nx_dim + d] : 0.0f;
        a.nx_out[d] = v;
      }
    }
  }
}

// Fallback for shapes no (G,KC) instantiation covers: one wavefront per row, the
// input vector re-read through the cache hierarchy. `x` must already carry the prologue.
template <int TYPE>
__global__ __launch_bounds__(256) void k_gemv_generic(GemvArgs a) {
  constexpr int XPC = Fmt<TYPE>::XPC;
  constexpr bool QUANT = (TYPE == CTHIP_Q8_0 || TYPE == CTHIP_Q4_0);
  const int lane = threadIdx.x & 63;
  const int wave = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int total_waves = gridDim.x * (blockDim.x >> 6);
  const int nchunks = a.cols / XPC;
  const int m = blockIdx.y;
  const float *__restrict__ x = a.x + (int64_t)m * a.x_stride;
  const uint4 *__restrict__ qp = (const uint4 *)a.q;
  const int posv = a.pos ? a.pos[0] : 0;
  float best_v = -INFINITY;
  int best_i = 0x7fffffff;
  for (int row = wave; row < a.rows; row += total_waves) {
    float acc = 0.0f;
    for (int c = lane; c < nchunks; c += 64) {
      uint4 w = qp[(int64_t)row * nchunks + c];
      float xl[XPC];
      float xsum = 0.0f;
#pragma unroll
      for (int e = 0; e < XPC; e++) {
        xl[e] = x[(int64_t)c * XPC + e];
        xsum += xl[e];
      }
      float scale = 1.0f;
      if (QUANT) {
        const int sidx = (TYPE == CTHIP_Q8_0) ? (c >> 1) : c;
        scale = half_bits_to_float(a.d[(int64_t)row * (a.cols >> 5) + sidx]);
      }
      acc += chunk_dot<TYPE>(w, scale, xl, xsum);
    }
    acc = wave_sum(acc);
    if (lane == 0) {
      const float v = gemv_store(a, m, row, acc, posv, a.bias ? a.bias[row] : 0.0f,
                                 a.residual ? a.residual[(int64_t)m * a.y_stride + row] : 0.0f);
      argmax_merge(best_v, best_i, v, row);
    }
  }
  if (a.am_val) gemv_argmax_tail(a, wave, lane, best_v, best_i);
}

// fp32 / fp16 rows whose width is no multiple of a 16-byte chunk: rows start at any element, so the lanes of a
// wavefront stride the row element by element.  `x` must already carry the prologue.
template <int TYPE>
__global__ __launch_bounds__(256) void k_gemv_elements(GemvArgs a) {
  const int lane = threadIdx.x & 63;
  const int wave = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int total_waves = gridDim.x * (blockDim.x >> 6);
  const int m = blockIdx.y;
  const float *__restrict__ x = a.x + (int64_t)m * a.x_stride;
  const int posv = a.pos ? a.pos[0] : 0;
  float best_v = -INFINITY;
  int best_i = 0x7fffffff;
  for (int row = wave; row < a.rows; row += total_waves) {
    float acc = 0.0f;
    for (int c = lane; c < a.cols; c += 64) {
      const int64_t e = (int64_t)row * a.cols + c;
      const float w = TYPE == CTHIP_F16 ? half_bits_to_float(((const unsigned short *)a.q)[e]) : ((const float *)a.q)[e];
      acc = fmaf(w, x[c], acc);
    }
    acc = wave_sum(acc);
    if (lane == 0) {
      const float v = gemv_store(a, m, row, acc, posv, a.bias ? a.bias[row] : 0.0f,
                                 a.residual ? a.residual[(int64_t)m * a.y_stride + row] : 0.0f);
      argmax_merge(best_v, best_i, v, row);
    }
  }
  if (a.am_val) gemv_argmax_tail(a, wave, lane, best_v, best_i);
}

// prologue as a kernel of its own, for the generic fallback: one block per input vector
__global__ __launch_bounds__(256) void k_prologue(float *__restrict__ out, const float *__restrict__ x, int cols,
                                                  int pro, const float *__restrict__ g,
                                                  const float *__restrict__ b, float eps, int64_t x_stride) {
  __shared__ float red[4];
  const float *xi = x + (int64_t)blockIdx.x * x_stride;
  float *o = out + (int64_t)blockIdx.x * cols;
  const int tid = threadIdx.x;
  auto block_sum = [&](float v) {
    v = wave_sum(v);
    __syncthreads();
    if ((tid & 63) == 0) red[tid >> 6] = v;
    __syncthreads();
    return red[0] + red[1] + red[2] + red[3];
  };
  if (pro == CTHIP_PRO_SWIGLU) {
    for (int i = tid; i < cols; i += 256) o[i] = ct_silu(xi[i]) * xi[cols + i];
    return;
  }
  float mean = 0.0f;
  if (pro == CTHIP_PRO_LAYERNORM) {
    float s = 0.0f;
    for (int i = tid; i < cols; i += 256) s += xi[i];
    mean = block_sum(s) / (float)cols;
  }
  float v = 0.0f;
  for (int i = tid; i < cols; i += 256) {
    float dlt = xi[i] - mean;
    v = fmaf(dlt, dlt, v);
  }
  const float rstd = 1.0f / sqrtf(block_sum(v) / (float)cols + eps);
  for (int i = tid; i < cols; i += 256) {
    float t = (xi[i] - mean) * rstd;
    if (g) t *= g[i];
    if (b) t += b[i];
    o[i] = t;
  }
}

// ------------------------------------------------------------------ dispatch
// every variant of every weight type, in one table (assembled once from the per-type translation units)
static const std::vector<GemvVariant> &all_variants() {
  static const std::vector<GemvVariant> all = [] {
    std::vector<GemvVariant> v;
    v.insert(v.end(), kGemvQ8, kGemvQ8 + kGemvQ8Count);
    v.insert(v.end(), kGemvQ4, kGemvQ4 + kGemvQ4Count);
    v.insert(v.end(), kGemvF32, kGemvF32 + kGemvF32Count);
    v.insert(v.end(), kGemvF16, kGemvF16 + kGemvF16Count);
    return v;
  }();
  return all;
}

static int xpc_of(int type) { return gemv_xpc(type); }

// the kernels of the variant the plan names (the tables of the per-type translation units are in gemv_shapes() order)
static const GemvVariant *variant_of(int shape) {
  if (shape < 0) return nullptr;
  const std::vector<GemvVariant> &all = all_variants();
  const GemvShape &sh = gemv_shapes()[shape];
  const GemvVariant &v = all[(size_t)shape];
  return (v.type == sh.type && v.G == sh.G && v.KC == sh.KC) ? &v : nullptr;
}
static const GemvVariant *pick_variant(int type, int cols) { return variant_of(gemv_pick_shape(type, cols)); }

// silu(gate) * up of m rows laid out (gate[cols], up[cols]): element-wise, so a row is spread over as many workgroups
// as it has blocks of 1024 elements (one workgroup per row took 35 us for the 28672 features of a 70B-shape FFN)
__global__ __launch_bounds__(256) void k_swiglu_rows(float *__restrict__ out, const float *__restrict__ x, int cols,
                                                     int64_t x_stride) {
  const float *xi = x + (int64_t)blockIdx.y * x_stride;
  float *o = out + (int64_t)blockIdx.y * cols;
  const int i0 = blockIdx.x * 1024 + threadIdx.x;
#pragma unroll
  for (int k = 0; k < 4; k++) {
    const int i = i0 + 256 * k;
    if (i < cols) o[i] = ct_silu(xi[i]) * xi[cols + i];
  }
}

int launch_prologue(float *out, const float *x, int cols, int pro, const float *g, const float *b, float eps,
                    int64_t x_stride, int m) {
  if (m == 0) return 0;
  if (pro == CTHIP_PRO_SWIGLU)
    hipLaunchKernelGGL(k_swiglu_rows, dim3((unsigned)((cols + 1023) / 1024), (unsigned)m), dim3(256), 0, state().stream, out, x, cols, x_stride);
  else
    hipLaunchKernelGGL(k_prologue, dim3(m), dim3(256), 0, state().stream, out, x, cols, pro, g, b, eps, x_stride);
  CTHIP_LAUNCH_CHECK();
  return 0;
}

bool gemv_is_direct(const WMat *w) {
  int width = 0;
  return pick_variant(w->type, (int)w->cols) != nullptr || gemv_slices(w->type, (long long)w->cols, &width) > 0 ||
         gemv_wide_plan(w->type, w->rows, w->cols, state().compute_units).ok;
}
// true when a single-row launch over a (rows, cols) matrix of gate / up rows in turn can apply SwiGLU in its epilogue:
// the launch it will be holds a row pair per wavefront (the routing of launch_gemv, repeated)
// The wide-row kernel takes the rows no variant covers, and those whose variant holds so much of the input vector
// per lane (128 floats: 4-bit rows past 6144 columns, 8-bit rows past 4096) that it needs more than 256 registers
// and runs one wavefront per SIMD (Llama-70B shape, 8192-wide 4-bit rows: 12.3 -> 11.8 ms per step; narrower
// rows are faster from registers: 7B / 13B shapes 1.83 / 2.96 ms against 2.02 / 3.29 with every launch here).
// (a wavefront there takes whole rows: with few rows it leaves compute units idle -- GPT-2 large's 1280 x 5120
// projection is slower there, GPT-2 XL's 1600 x 6400, whose variant needs 366 registers, faster)
static bool gemv_prefers_wide(const GemvVariant *v, int type, int64_t rows) {
  const bool heavy = v && ((type == CTHIP_Q4_0 && v->KC >= 4 && rows >= 1024) ||
                           (type == CTHIP_Q8_0 && (v->KC >= 8 ? rows >= 1024 : v->KC >= 6 && rows >= 4096)));
  const int opt = state().gemv_wide;
  return opt && (!v || heavy || opt >= 2);
}
bool gemv_pair_swiglu_ok(int type, int64_t rows, int64_t cols) {
  if (rows <= 0 || (rows & 1) || cols <= 0 || cols > 0x7fffffff) return false;
  const GemvVariant *v = pick_variant(type, (int)cols);
  const State &s = state();
  if (gemv_prefers_wide(v, type, rows)) {
    const GemvWidePlan p = gemv_wide_plan(type, rows, cols, s.compute_units);
    if (p.ok) return p.rw == 2;
  }
  if (!v) return false;
  if (v->G <= 32) return true;  // two rows and more per wavefront: the pair sits in neighbouring lane groups
  // one row per wavefront: the pair sits in neighbouring slots of the ring, which a looping launch with an even ring
  // has (enough rows for every wavefront to loop at any occupancy)
  return (gemv_ring_depth(type, v->KC) & 1) == 0 && rows >= 32ll * s.compute_units;
}
int gemv_rows_per_wave(int type, int64_t cols) {
  const GemvVariant *v = cols <= 0x7fffffff ? pick_variant(type, (int)cols) : nullptr;
  return v ? 64 / v->G : 0;
}

__global__ __launch_bounds__(256) void k_swiglu_pairs(float *__restrict__ out, const float *__restrict__ in, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
    const float2 v = ((const float2 *)in)[i];
    out[i] = ct_silu(v.x) * v.y;
  }
}
int launch_swiglu_pairs(float *out, const float *in, int64_t n) {
  if (n <= 0) return 0;
  int64_t blocks = (n + 255) / 256;
  if (blocks > 8192) blocks = 8192;
  hipLaunchKernelGGL(k_swiglu_pairs, dim3((unsigned)blocks), dim3(256), 0, state().stream, out, in, n);
  CTHIP_LAUNCH_CHECK();
  return 0;
}

// one launch of a register-resident variant over a.cols columns (a whole matrix, or a column slice of one)
static int launch_variant(const GemvVariant *v, const WMat *w, GemvArgs a, int m) {
  State &s = state();
  {
    const int vi = (int)(v - all_variants().data());
    static std::vector<int> occ_cache(all_variants().size(), 0);
    GemvPlanIn in = {};
    in.type = w->type;
    in.rows = a.rows;
    in.cols = a.cols;
    in.m = m;
    in.pro = a.pro;
    in.fold = a.fold_s != nullptr;
    in.bias = a.bias != nullptr;
    in.bias0 = a.bias0 != nullptr;
    in.residual = a.residual != nullptr;
    in.argmax = a.am_val != nullptr;
    in.compute_units = s.compute_units;
    in.occupancy = 1;
    GemvPlan p = gemv_plan(in);
    if (!p.error && p.kernel != GEMV_K_SMALL) {  // a looping launch: how many of its workgroups a compute unit holds
      if (occ_cache[vi] == 0) {
        int nb = 0;
        CTHIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb, v->fn[0], 256, 16 * 1024));
        occ_cache[vi] = nb > 0 ? nb : 1;
      }
      in.occupancy = occ_cache[vi];
      p = gemv_plan(in);
    }
    if (p.error) return fail(CTHIP_E_UNSUPPORTED, "gemv: (%d, %d): %s", a.rows, a.cols, p.error);
    // the paired SwiGLU epilogue with one row per wavefront: the pair sits in two neighbouring slots of the ring
    const bool pair1 = a.pair_swiglu && v->G > 32;
    if (pair1 && (p.kernel != GEMV_K_LOOP || !v->fn_pair[0]))
      return fail(CTHIP_E_UNSUPPORTED, "gemv: the paired SwiGLU epilogue over (%d, %d) needs a looping launch with an even ring and no per-row operands", a.rows, a.cols);
    a.stage_x = p.stage ? 1 : 0;
    if (p.unfold) {
      a.fold_s = nullptr;
      a.bias = nullptr;
    }
    if (a.am_val && p.nwaves > kGemvMaxWaves)
      return fail(CTHIP_E_UNSUPPORTED, "gemv: %d wavefronts exceed the argmax scratch", p.nwaves);
    const int nt = s.gemv_stream < 0 ? (w->stream ? 1 : 0) : s.gemv_stream;
    // the looping kernel with per-row operands in its ring dereferences one of them unconditionally
    if (p.kernel == GEMV_K_LOOP_EPI && !a.bias && !a.residual && !a.fold_s)
      return fail(CTHIP_E_STATE, "gemv: a launch with epilogue operands in its ring has none");
    const gemv_fn fn = pair1 ? v->fn_pair[nt] : p.kernel == GEMV_K_SMALL ? v->fn_small[nt] : p.kernel == GEMV_K_LOOP_EPI ? v->fn_epi[nt]
                     : p.kernel == GEMV_K_LOOP_DIRECT ? v->fn_direct[nt] : v->fn[nt];
    hipLaunchKernelGGL(fn, dim3(p.grid_x, p.grid_y), dim3(p.block), p.lds, s.stream, a);
    CTHIP_LAUNCH_CHECK();
    if (a.am_val) {
      hipLaunchKernelGGL(k_argmax_finish, dim3(1), dim3(256), 0, s.stream, a, p.nwaves);
      CTHIP_LAUNCH_CHECK();
    }
    return 0;
  }
}

// Queues one fused Linear on the stream. Used by cthip_linear and by the decoder.
int launch_gemv(const WMat *w, GemvArgs a, int m) {
  State &s = state();
  a.q = w->q;
  a.d = (const unsigned short *)w->d;
  a.rows = (int)w->rows;
  a.cols = (int)w->cols;
  a.ld_chunks = a.ld_scales = a.up_off = 0;
  if (a.split1 <= 0) a.split1 = a.split2 = a.rows;
  if (a.am_val && m != 1) return fail(CTHIP_E_BAD_ARG, "gemv: the fused argmax needs m == 1");
  const GemvVariant *v = pick_variant(w->type, a.cols);
  if (gemv_prefers_wide(v, w->type, a.rows) && gemv_wide_supported(w, a)) return launch_gemv_wide(w, a, m);
  if (a.pair_swiglu && (!v || (a.rows & 1) || a.am_val || a.residual || a.split1 != a.rows))
    return fail(CTHIP_E_UNSUPPORTED, "gemv: the paired SwiGLU epilogue needs a register-resident launch and plain outputs");
  if (v) return launch_variant(v, w, a, m);
  // wider than any variant: column slices, when nothing in the launch needs the whole row at once (a norm of the
  // input, an activation of the sum, an argmax) and the output is one plain vector per input row
  int width = 0;
  const int nsl = (a.pro == CTHIP_PRO_NONE || a.pro == CTHIP_PRO_SWIGLU) && a.act == CTHIP_ACT_NONE && !a.am_val &&
                          !a.fold_s && a.split1 == a.rows && a.y
                      ? gemv_slices(w->type, a.cols, &width)
                      : 0;
  if (nsl > 0) {
    const int xpc = xpc_of(w->type), cols = a.cols;
    for (int sl = 0; sl < nsl; sl++) {
      const int c0 = sl * width;
      GemvArgs b = a;
      b.cols = sl + 1 < nsl ? width : cols - c0;
      b.q = (const char *)w->q + (int64_t)(c0 / xpc) * 16;
      b.d = w->d ? (const unsigned short *)w->d + (c0 >> 5) : nullptr;
      b.x = a.x + c0;
      b.ld_chunks = cols / xpc;
      b.ld_scales = cols >> 5;
      b.up_off = a.pro == CTHIP_PRO_SWIGLU ? cols : 0;
      if (sl > 0) {  // adds to what the slices before it left (each output element is read and written by one lane)
        b.bias = b.bias0 = nullptr;
        b.residual = a.y;
      }
      const GemvVariant *vs = pick_variant(w->type, b.cols);
      if (!vs) return fail(CTHIP_E_STATE, "gemv: no variant for a slice of %d columns", b.cols);
      const int rc = launch_variant(vs, w, b, m);
      if (rc) return rc;
    }
    return 0;
  }
  // generic path: prologue into a temporary, then wave-per-row
  float *tmp = nullptr;
  if (a.pro != CTHIP_PRO_NONE) {
    int rc = alloc_scratch((void **)&tmp, sizeof(float) * (size_t)a.cols * m);  // fully written below
    if (rc) return rc;
    rc = launch_prologue(tmp, a.x, a.cols, a.pro, a.norm_g, a.norm_b, a.eps, a.x_stride, m);
    if (rc) {
      cthip_free(tmp);
      return rc;
    }
    a.x = tmp;
    a.x_stride = a.cols;
    a.pro = CTHIP_PRO_NONE;
  }
  int blocks = (a.rows + 3) / 4;
  int cap = s.compute_units * 8;
  if (cap * 4 > kGemvMaxWaves) cap = kGemvMaxWaves / 4;
  dim3 grid(blocks < cap ? blocks : cap, m), block(256);
  // rows that are whole 16-byte chunks are read chunk by chunk; any other width (fp32 / fp16 only: quantised rows
  // are multiples of 32) element by element
  const bool chunks = a.cols % xpc_of(w->type) == 0;
  switch (w->type) {
    case CTHIP_Q8_0: hipLaunchKernelGGL(k_gemv_generic<CTHIP_Q8_0>, grid, block, 0, s.stream, a); break;
    case CTHIP_Q4_0: hipLaunchKernelGGL(k_gemv_generic<CTHIP_Q4_0>, grid, block, 0, s.stream, a); break;
    case CTHIP_F16:
      if (chunks) hipLaunchKernelGGL(k_gemv_generic<CTHIP_F16>, grid, block, 0, s.stream, a);
      else hipLaunchKernelGGL(k_gemv_elements<CTHIP_F16>, grid, block, 0, s.stream, a);
      break;
    default:
      if (chunks) hipLaunchKernelGGL(k_gemv_generic<CTHIP_F32>, grid, block, 0, s.stream, a);
      else hipLaunchKernelGGL(k_gemv_elements<CTHIP_F32>, grid, block, 0, s.stream, a);
      break;
  }
  CTHIP_LAUNCH_CHECK();
  if (a.am_val) {
    hipLaunchKernelGGL(k_argmax_finish, dim3(1), dim3(256), 0, s.stream, a, (int)(grid.x * 4));
    CTHIP_LAUNCH_CHECK();
  }
  if (tmp) return cthip_free(tmp);
  return 0;
}

int wmat_create_impl(WMat **out, int type, const void *raw, int64_t rows, int64_t cols) {
  State &s = state();
  WMat *w = new WMat();
  w->type = type;
  w->rows = rows;
  w->cols = cols;
  w->q = w->d = nullptr;
  const int64_t n = rows * cols;
  int rc = 0;
  if (type == CTHIP_Q8_0 || type == CTHIP_Q4_0) {
    const int64_t nblocks = n / 32;
    w->q_bytes = (type == CTHIP_Q8_0) ? n : n / 2;
    w->d_bytes = nblocks * 2;
    if ((rc = cthip_alloc(&w->q, (size_t)w->q_bytes)) || (rc = cthip_alloc(&w->d, (size_t)w->d_bytes))) {
      cthip_free(w->q);
      delete w;
      return rc;
    }
    unsigned blocks = (unsigned)((nblocks + 255) / 256);
    if (type == CTHIP_Q8_0)
      hipLaunchKernelGGL(k_repack_q8_0, dim3(blocks), dim3(256), 0, s.stream, (const uint8_t *)raw, nblocks,
                         (uint32_t *)w->q, (unsigned short *)w->d);
    else
      hipLaunchKernelGGL(k_repack_q4_0, dim3(blocks), dim3(256), 0, s.stream, (const uint8_t *)raw, nblocks,
                         (uint32_t *)w->q, (unsigned short *)w->d);
    CTHIP_LAUNCH_CHECK();
  } else {
    w->q_bytes = n * (type == CTHIP_F32 ? 4 : 2);
    w->d_bytes = 0;
    if ((rc = cthip_alloc(&w->q, (size_t)w->q_bytes))) {
      delete w;
      return rc;
    }
    CTHIP_CHECK(hipMemcpyAsync(w->q, raw, (size_t)w->q_bytes, hipMemcpyDeviceToDevice, s.stream));
  }
  w->stream = w->q_bytes + w->d_bytes > kInfinityCacheBytes;  // cannot stay cached between two uses by itself
  *out = w;
  return 0;
}

}  // namespace cthip

using namespace cthip;

extern "C" {

int cthip_dequant(int ggml_type, const void *raw, int64_t n, float *out) {
  CTHIP_REQUIRE_INIT();
  if (n == 0) return 0;
  CTHIP_ARG(raw != nullptr && out != nullptr && n > 0);
  if (!device_readable(raw) || !device_readable(out))
    return fail(CTHIP_E_BAD_ARG, "cthip_dequant: raw and out must be device pointers (upload the bytes with cthip_h2d first)");
  dim3 grid((unsigned)((n + 255) / 256)), block(256);
  hipStream_t st = state().stream;
  switch (ggml_type) {
    case CTHIP_Q8_0: hipLaunchKernelGGL(k_dequant_q8_0_raw, grid, block, 0, st, (const uint8_t *)raw, n, out); break;
    case CTHIP_Q4_0:
      if (n % 32) return fail(CTHIP_E_BAD_ARG, "cthip_dequant: Q4_0 needs n %% 32 == 0, got %lld", (long long)n);
      hipLaunchKernelGGL(k_dequant_q4_0_raw, grid, block, 0, st, (const uint8_t *)raw, n, out);
      break;
    case CTHIP_F16: hipLaunchKernelGGL(k_dequant_f16_raw, grid, block, 0, st, (const uint8_t *)raw, n, out); break;
    case CTHIP_F32: hipLaunchKernelGGL(k_dequant_f32_raw, grid, block, 0, st, (const uint8_t *)raw, n, out); break;
    default:
      // tensor-info.lisp:36-41 signals "Not ready" for every other ggml type
      return fail(CTHIP_E_UNSUPPORTED, "cthip_dequant: ggml type %d is not supported", ggml_type);
  }
  CTHIP_LAUNCH_CHECK();
  return 0;
}

int cthip_wmat_create(void **wmat, int ggml_type, const void *raw, int64_t rows, int64_t cols) {
  CTHIP_REQUIRE_INIT();
  CTHIP_ARG(wmat != nullptr && raw != nullptr && rows > 0 && cols > 0);
  if (ggml_type != CTHIP_Q8_0 && ggml_type != CTHIP_Q4_0 && ggml_type != CTHIP_F32 && ggml_type != CTHIP_F16)
    return fail(CTHIP_E_UNSUPPORTED, "cthip_wmat_create: ggml type %d is not supported", ggml_type);
  if ((ggml_type == CTHIP_Q8_0 || ggml_type == CTHIP_Q4_0) && cols % 32)
    return fail(CTHIP_E_BAD_ARG, "cthip_wmat_create: quantised rows need cols %% 32 == 0, got %lld", (long long)cols);
  if (rows > 0x7fffffff || cols > 0x7fffffff) return fail(CTHIP_E_BAD_ARG, "cthip_wmat_create: dimension too large");
  if (!device_readable(raw))
    return fail(CTHIP_E_BAD_ARG, "cthip_wmat_create: raw must be a device pointer (upload the bytes with cthip_h2d first)");
  WMat *w = nullptr;
  int rc = wmat_create_impl(&w, ggml_type, raw, rows, cols);
  if (rc) return rc;
  *wmat = w;
  return 0;
}

int cthip_wmat_destroy(void *wmat) {
  if (!wmat) return 0;
  WMat *w = (WMat *)wmat;
  cthip_free(w->q);
  cthip_free(w->d);
  if (w->fold_s) cthip_free(w->fold_s);
  if (w->fold_c) cthip_free(w->fold_c);
  delete w;
  return 0;
}

int cthip_wmat_fold_layernorm(void *wmat, const float *gamma, const float *beta, const float *bias) {
  CTHIP_REQUIRE_INIT();
  CTHIP_ARG(wmat != nullptr && gamma != nullptr && beta != nullptr);
  WMat *w = (WMat *)wmat;
  if (!pick_variant(w->type, (int)w->cols)) return fail(CTHIP_E_UNSUPPORTED, "cthip_wmat_fold_layernorm: no single-row kernel covers %lld columns", (long long)w->cols);
  int rc;
  if (!w->fold_s && (rc = cthip_alloc((void **)&w->fold_s, sizeof(float) * (size_t)w->rows))) return rc;
  if (!w->fold_c && (rc = cthip_alloc((void **)&w->fold_c, sizeof(float) * (size_t)w->rows))) return rc;
  w->fold_g = w->fold_b = w->fold_bias = nullptr;  // not valid until both products are queued
  GemvArgs s = {};  // S = W . gamma
  s.x = gamma;
  s.y = w->fold_s;
  s.x_stride = w->cols;
  s.y_stride = w->rows;
  if ((rc = launch_gemv(w, s, 1))) return rc;
  GemvArgs c = {};  // C = W . beta + bias
  c.x = beta;
  c.bias = bias;
  c.y = w->fold_c;
  c.x_stride = w->cols;
  c.y_stride = w->rows;
  if ((rc = launch_gemv(w, c, 1))) return rc;
  w->fold_g = gamma;
  w->fold_b = beta;
  w->fold_bias = bias;
  return 0;
}

int64_t cthip_wmat_nbytes(const void *wmat) {
  const WMat *w = (const WMat *)wmat;
  return w ? w->q_bytes + w->d_bytes : 0;
}

int cthip_wmat_dequant(const void *wmat, float *out) {
  CTHIP_REQUIRE_INIT();
  CTHIP_ARG(wmat != nullptr && out != nullptr);
  const WMat *w = (const WMat *)wmat;
  const int64_t n = w->rows * w->cols;
  hipLaunchKernelGGL(k_wmat_dequant, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, state().stream, w->type, w->q,
                     (const unsigned short *)w->d, n, out);
  CTHIP_LAUNCH_CHECK();
  return 0;
}

int cthip_linear(float *y, const void *wmat, const float *x, int m, const float *bias, const float *residual,
                 int act, int prologue, const float *norm_g, const float *norm_b, float eps) {
  CTHIP_REQUIRE_INIT();
  CTHIP_ARG(y != nullptr && wmat != nullptr && x != nullptr && m >= 0);
  CTHIP_ARG(prologue >= CTHIP_PRO_NONE && prologue <= CTHIP_PRO_SWIGLU);
  CTHIP_ARG(act >= CTHIP_ACT_NONE && act <= CTHIP_ACT_TANH);
  if (m == 0) return 0;
  if (m > 65535) return fail(CTHIP_E_BAD_ARG, "cthip_linear: m = %d exceeds 65535", m);
  const WMat *w = (const WMat *)wmat;
  if (m >= 8) {
    // several input rows: the MFMA tile path reads the weights once instead of once per row
    const float *xin = x;
    float *tmp = nullptr;
    int rc;
    if (prologue != CTHIP_PRO_NONE) {
      if ((rc = alloc_scratch((void **)&tmp, sizeof(float) * (size_t)w->cols * m))) return rc;  // fully written below
      rc = launch_prologue(tmp, x, (int)w->cols, prologue, norm_g, norm_b, eps,
                           (int64_t)(prologue == CTHIP_PRO_SWIGLU ? 2 * w->cols : w->cols), m);
      if (rc) {
        cthip_free(tmp);
        return rc;
      }
      xin = tmp;
    }
    rc = launch_linear_gemm(y, w, xin, m, bias, residual, act, state().gemm_precision);
    if (tmp) cthip_free(tmp);
    return rc;
  }
  GemvArgs a = {};
  a.y = y;
  a.x = x;
  a.bias = bias;
  a.residual = residual;
  a.act = act;
  a.pro = prologue;
  a.norm_g = norm_g;
  a.norm_b = norm_b;
  a.eps = eps;
  a.x_stride = (prologue == CTHIP_PRO_SWIGLU) ? 2 * w->cols : w->cols;
  a.y_stride = w->rows;
  if (prologue == CTHIP_PRO_LAYERNORM && w->fold_g && w->fold_g == norm_g && w->fold_b == norm_b && w->fold_bias == bias) {
    a.fold_s = w->fold_s;  // the norm goes through the product: see k_gemv
    a.bias = w->fold_c;
    a.bias0 = bias;
  }
  return launch_gemv(w, a, m);
}

int cthip_set_option(const char *name, int value) {
  if (!name) return fail(CTHIP_E_BAD_ARG, "cthip_set_option: null name");
  if (!strcmp(name, "gemm_precision")) {
    if (value < GEMM_FP32 || value > GEMM_BF16X6) return fail(CTHIP_E_BAD_ARG, "cthip_set_option: gemm_precision is 0..3");
    state().gemm_precision = value;
    return 0;
  }
  if (!strcmp(name, "gemv_stream_weights")) {
    if (value < -1 || value > 1) return fail(CTHIP_E_BAD_ARG, "cthip_set_option: gemv_stream_weights is -1, 0 or 1");
    state().gemv_stream = value;
    return 0;
  }
  if (!strcmp(name, "attn_split")) {
    if (value < 0 || value > kAttnSplitMaxRanges) return fail(CTHIP_E_BAD_ARG, "cthip_set_option: attn_split is 0, 1 or a number of key ranges per head up to %d", kAttnSplitMaxRanges);
    state().attn_split = value;
    return 0;
  }
  if (!strcmp(name, "attn_long_from")) {
    if (value < 0) return fail(CTHIP_E_BAD_ARG, "cthip_set_option: attn_long_from is a position (0 = never)");
    state().attn_long_from = value;
    return 0;
  }
  if (!strcmp(name, "gemv_wide")) {
    if (value < 0 || value > 2) return fail(CTHIP_E_BAD_ARG, "cthip_set_option: gemv_wide is 0, 1 or 2");
    state().gemv_wide = value;
    return 0;
  }
  if (!strcmp(name, "decoder_graph") || !strcmp(name, "prefill_gemm") || !strcmp(name, "decode_fused") ||
      !strcmp(name, "render_routes")) {
    if (value != 0 && value != 1) return fail(CTHIP_E_BAD_ARG, "cthip_set_option: %s is 0 or 1", name);
    if (!strcmp(name, "decoder_graph")) state().decoder_graph = value;
    else if (!strcmp(name, "prefill_gemm")) state().prefill_gemm = value;
    else if (!strcmp(name, "render_routes")) state().render_routes = value;
    else state().decode_fused = value;
    return 0;
  }
  if (!strcmp(name, "decode_flow")) {
    if (value < 0 || value > 2) return fail(CTHIP_E_BAD_ARG, "cthip_set_option: decode_flow is 0, 1 or 2 (1 with a timeline of the last step)");
    state().decode_flow = value;
    return 0;
  }
  if (!strcmp(name, "kv_cache")) {
    if (value < 0 || value > 2) return fail(CTHIP_E_BAD_ARG, "cthip_set_option: kv_cache is 0 (fp32 rows), 1 (Q8_0 rows) or 2 (fp32 rows in pages)");
    state().kv_cache = value;
    return 0;
  }
  if (!strcmp(name, "decode_skip")) {
    if (value < 0 || value > 31) return fail(CTHIP_E_BAD_ARG, "cthip_set_option: decode_skip is a mask of 5 bits");
    state().decode_skip = value;
    return 0;
  }
  if (!strcmp(name, "gemm_bf16")) {  // 1 = operands rounded to bf16, 0 = back to the default
    state().gemm_precision = value ? GEMM_BF16 : GEMM_BF16X3;
    return 0;
  }
  return fail(CTHIP_E_BAD_ARG, "cthip_set_option: unknown option '%s'", name);
}

}  // extern "C"
