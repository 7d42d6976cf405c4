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

#include "common.h"

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

// ------------------------------------------------------------------ GEMV
template <int TYPE>
struct Fmt;
template <>
struct Fmt<CTHIP_Q8_0> {
  static constexpr int XPC = 16;  // input elements multiplied by one 16-byte chunk
};
template <>
struct Fmt<CTHIP_Q4_0> {
  static constexpr int XPC = 32;
};
template <>
struct Fmt<CTHIP_F32> {
  static constexpr int XPC = 4;
};
template <>
struct Fmt<CTHIP_F16> {
  static constexpr int XPC = 8;
};

template <int TYPE>
__device__ __forceinline__ float chunk_dot(const uint4 w, float scale, const float *__restrict__ x, float xsum);

template <>
__device__ __forceinline__ float chunk_dot<CTHIP_Q8_0>(const uint4 w, float scale, const float *__restrict__ x, float) {
  const uint32_t dw[4] = {w.x, w.y, w.z, w.w};
  float s = 0.0f;
#pragma unroll
  for (int t = 0; t < 4; t++) {
    int v = (int)dw[t];
    s = fmaf((float)(int)(int8_t)(v), x[4 * t + 0], s);
    s = fmaf((float)(int)(int8_t)(v >> 8), x[4 * t + 1], s);
    s = fmaf((float)(int)(int8_t)(v >> 16), x[4 * t + 2], s);
    s = fmaf((float)(v >> 24), x[4 * t + 3], s);
  }
  return s * scale;
}

template <>
__device__ __forceinline__ float chunk_dot<CTHIP_Q4_0>(const uint4 w, float scale, const float *__restrict__ x, float xsum) {
  const uint32_t dw[4] = {w.x, w.y, w.z, w.w};
  float s = 0.0f;
#pragma unroll
  for (int t = 0; t < 4; t++) {
    uint32_t lo = dw[t] & 0x0f0f0f0fu;
    uint32_t hi = (dw[t] >> 4) & 0x0f0f0f0fu;
    s = fmaf((float)(lo & 0xff), x[4 * t + 0], s);
    s = fmaf((float)((lo >> 8) & 0xff), x[4 * t + 1], s);
    s = fmaf((float)((lo >> 16) & 0xff), x[4 * t + 2], s);
    s = fmaf((float)(lo >> 24), x[4 * t + 3], s);
    s = fmaf((float)(hi & 0xff), x[16 + 4 * t + 0], s);
    s = fmaf((float)((hi >> 8) & 0xff), x[16 + 4 * t + 1], s);
    s = fmaf((float)((hi >> 16) & 0xff), x[16 + 4 * t + 2], s);
    s = fmaf((float)(hi >> 24), x[16 + 4 * t + 3], s);
  }
  // sum (n-8) x = sum n x - 8 sum x
  return (s - 8.0f * xsum) * scale;
}

template <>
__device__ __forceinline__ float chunk_dot<CTHIP_F32>(const uint4 w, float, const float *__restrict__ x, float) {
  float s = __uint_as_float(w.x) * x[0];
  s = fmaf(__uint_as_float(w.y), x[1], s);
  s = fmaf(__uint_as_float(w.z), x[2], s);
  s = fmaf(__uint_as_float(w.w), x[3], s);
  return s;
}

template <>
__device__ __forceinline__ float chunk_dot<CTHIP_F16>(const uint4 w, float, const float *__restrict__ x, float) {
  const uint32_t dw[4] = {w.x, w.y, w.z, w.w};
  float s = 0.0f;
#pragma unroll
  for (int t = 0; t < 4; t++) {
    s = fmaf(half_bits_to_float((unsigned short)(dw[t] & 0xffff)), x[2 * t], s);
    s = fmaf(half_bits_to_float((unsigned short)(dw[t] >> 16)), x[2 * t + 1], s);
  }
  return s;
}

// lowest-index argmax merge: (v, i) <- better of (v, i) and (ov, oi)
__device__ __forceinline__ void argmax_merge(float &v, int &i, float ov, int oi) {
  if (ov > v || (ov == v && oi < i)) {
    v = ov;
    i = oi;
  }
}

// Epilogue shared by the GEMV kernels: bias, activation, residual, routing of fused-qkv rows.
__device__ __forceinline__ float gemv_store(const GemvArgs &a, int m, int row, float acc, int posv, float bias,
                                            float resid) {
  float v = acc + bias;
  v = apply_act(a.act, v);
  v += resid;
  float *dst;
  if (row < a.split1) {
    dst = a.y + (int64_t)m * a.y_stride + row;
  } else {
    const int64_t off = (int64_t)(posv + m) * a.pos_stride;
    dst = (row < a.split2) ? a.y1 + off + (row - a.split1) : a.y2 + off + (row - a.split2);
  }
  *dst = v;
  return v;
}

// ArgMaxNode fused behind the last Linear (lm_head): every wavefront publishes the best
// (value, lowest row) of the rows it produced; k_argmax_finish combines them.  (A single ticket
// counter instead of a second launch would serialise thousands of same-address atomics.)
__device__ __forceinline__ void gemv_argmax_tail(const GemvArgs &a, int wave, int lane, float bv, int bi) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) argmax_merge(bv, bi, __shfl_xor(bv, o, 64), __shfl_xor(bi, o, 64));
  if (lane == 0) {
    a.am_val[wave] = bv;
    a.am_idx[wave] = bi;
  }
}

// one block: the greedy token goes where the next step's embedding reads it, is appended to the
// history, and the position advances
__global__ __launch_bounds__(256) void k_argmax_finish(GemvArgs a, int nparts) {
  __shared__ float sv[4];
  __shared__ int si[4];
  __shared__ int next_tok, next_pos;
  // the loop state is requested up front so its latency overlaps the reduction
  int hist_n = 0, pos = 0;
  if (threadIdx.x == 0) {
    if (a.am_hist) hist_n = *a.am_hist_n;
    if (a.am_pos) pos = *a.am_pos;
  }
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  for (int i = threadIdx.x; i < nparts; i += 256) argmax_merge(bv, bi, a.am_val[i], a.am_idx[i]);
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
    *a.am_token64 = bi;
    if (a.am_tok) *a.am_tok = bi;
    if (a.am_hist) {
      a.am_hist[hist_n] = bi;
      *a.am_hist_n = hist_n + 1;
    }
    if (a.am_pos) *a.am_pos = pos + 1;
    next_tok = bi;
    next_pos = pos + 1;
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

// Block-cooperative prologue: the workgroup normalises (or gates) the input vector ONCE into LDS --
// every thread owns cols/blockDim elements, the two reductions go wavefront-shuffle then LDS --
// instead of every wavefront redoing it in registers.  xs must hold a.cols floats.
__device__ __forceinline__ void coop_prologue(const GemvArgs &a, const float *__restrict__ x, float *xs, float *red,
                                              bool normalise) {
  const int tid = threadIdx.x, nthr = blockDim.x, nw = nthr >> 6;
  const int n4 = a.cols >> 2;
  if (a.pro != CTHIP_PRO_SWIGLU && !normalise) {  // plain copy: the norm (if any) is folded through the product
    for (int i = tid; i < n4; i += nthr) ((float4 *)xs)[i] = ((const float4 *)x)[i];
    __syncthreads();
    return;
  }
  if (a.pro == CTHIP_PRO_SWIGLU) {
    for (int i = tid; i < n4; i += nthr) {
      float4 v = ((const float4 *)x)[i];
      float4 u = ((const float4 *)(x + a.cols))[i];
      ((float4 *)xs)[i] = make_float4(ct_silu(v.x) * u.x, ct_silu(v.y) * u.y, ct_silu(v.z) * u.z, ct_silu(v.w) * u.w);
    }
    __syncthreads();
    return;
  }
  // LayerNorm / RMSNorm; a thread keeps up to 4 float4 in registers, longer vectors re-read x
  constexpr int KEEP = 4;
  float4 xv[KEEP], gv[KEEP], bv[KEEP];
#pragma unroll
  for (int k = 0; k < KEEP; k++) {
    const int i = tid + k * nthr;
    const bool ok = i < n4;
    xv[k] = ok ? ((const float4 *)x)[i] : make_float4(0.f, 0.f, 0.f, 0.f);
    gv[k] = (ok && a.norm_g) ? ((const float4 *)a.norm_g)[i] : make_float4(1.f, 1.f, 1.f, 1.f);
    bv[k] = (ok && a.norm_b) ? ((const float4 *)a.norm_b)[i] : make_float4(0.f, 0.f, 0.f, 0.f);
  }
  const bool fits = n4 <= KEEP * nthr;
  const float inv_n = 1.0f / (float)a.cols;
  auto block_sum = [&](float v) {
    v = wave_sum(v);
    __syncthreads();
    if ((tid & 63) == 0) red[tid >> 6] = v;
    __syncthreads();
    float t = 0.0f;
    for (int w = 0; w < nw; w++) t += red[w];
    return t;
  };
  float mean = 0.0f;
  if (a.pro == CTHIP_PRO_LAYERNORM) {
    float s = 0.0f;
#pragma unroll
    for (int k = 0; k < KEEP; k++) s += (xv[k].x + xv[k].y) + (xv[k].z + xv[k].w);
    if (!fits)
      for (int i = tid + KEEP * nthr; i < n4; i += nthr) {
        float4 v = ((const float4 *)x)[i];
        s += (v.x + v.y) + (v.z + v.w);
      }
    mean = block_sum(s) * inv_n;
  }
  float q = 0.0f;
#pragma unroll
  for (int k = 0; k < KEEP; k++) {
    if (tid + k * nthr < n4) {
      xv[k].x -= mean; xv[k].y -= mean; xv[k].z -= mean; xv[k].w -= mean;
      q = fmaf(xv[k].x, xv[k].x, q); q = fmaf(xv[k].y, xv[k].y, q);
      q = fmaf(xv[k].z, xv[k].z, q); q = fmaf(xv[k].w, xv[k].w, q);
    }
  }
  if (!fits)
    for (int i = tid + KEEP * nthr; i < n4; i += nthr) {
      float4 v = ((const float4 *)x)[i];
      v.x -= mean; v.y -= mean; v.z -= mean; v.w -= mean;
      q = fmaf(v.x, v.x, q); q = fmaf(v.y, v.y, q); q = fmaf(v.z, v.z, q); q = fmaf(v.w, v.w, q);
    }
  const float rstd = 1.0f / sqrtf(block_sum(q) * inv_n + a.eps);
#pragma unroll
  for (int k = 0; k < KEEP; k++) {
    const int i = tid + k * nthr;
    if (i < n4)
      ((float4 *)xs)[i] = make_float4(xv[k].x * rstd * gv[k].x + bv[k].x, xv[k].y * rstd * gv[k].y + bv[k].y,
                                      xv[k].z * rstd * gv[k].z + bv[k].z, xv[k].w * rstd * gv[k].w + bv[k].w);
  }
  if (!fits)
    for (int i = tid + KEEP * nthr; i < n4; i += nthr) {
      float4 v = ((const float4 *)x)[i];
      float4 gg = a.norm_g ? ((const float4 *)a.norm_g)[i] : make_float4(1.f, 1.f, 1.f, 1.f);
      float4 bb = a.norm_b ? ((const float4 *)a.norm_b)[i] : make_float4(0.f, 0.f, 0.f, 0.f);
      ((float4 *)xs)[i] = make_float4((v.x - mean) * rstd * gg.x + bb.x, (v.y - mean) * rstd * gg.y + bb.y,
                                      (v.z - mean) * rstd * gg.z + bb.z, (v.w - mean) * rstd * gg.w + bb.w);
    }
  __syncthreads();
}

// Folded norm with a staged input: the workgroup writes gamma * x into LDS once and reduces the
// shifted sums  s1 = sum(x - pivot), s2 = sum((x - pivot)^2)  over the whole vector, so no wavefront
// loads gamma or repeats the statistics.  xs must hold a.cols floats; blockDim.x <= 256.
__device__ __forceinline__ void coop_fold(const GemvArgs &a, const float *__restrict__ x, float *xs, float *red,
                                          float pivot, float &s1_out, float &s2_out) {
  const int tid = threadIdx.x, nthr = blockDim.x, nw = nthr >> 6;
  const int n4 = a.cols >> 2;
  float s1 = 0.0f, s2 = 0.0f;
  for (int i = tid; i < n4; i += nthr) {
    const float4 v = ((const float4 *)x)[i];
    const float4 g = a.norm_g ? ((const float4 *)a.norm_g)[i] : make_float4(1.f, 1.f, 1.f, 1.f);
    const float d0 = v.x - pivot, d1 = v.y - pivot, d2 = v.z - pivot, d3 = v.w - pivot;
    s1 += (d0 + d1) + (d2 + d3);
    s2 = fmaf(d0, d0, s2);
    s2 = fmaf(d1, d1, s2);
    s2 = fmaf(d2, d2, s2);
    s2 = fmaf(d3, d3, s2);
    ((float4 *)xs)[i] = make_float4(v.x * g.x, v.y * g.y, v.z * g.z, v.w * g.w);
  }
  auto block_sum = [&](float v) {
    v = wave_sum(v);
    __syncthreads();
    if ((tid & 63) == 0) red[tid >> 6] = v;
    __syncthreads();
    float t = 0.0f;
    for (int w = 0; w < nw; w++) t += red[w];
    return t;
  };
  s1_out = block_sum(s1);
  s2_out = block_sum(s2);  // its barriers also publish xs
}

// Sixteen bytes that stay zero: lanes with nothing to fetch point their requests here, so that every
// lane issues the same loads and no request sits behind a branch (the compiler can then wait for
// exactly the tile it needs instead of for everything in flight).  Not const: a select between a
// kernel-argument pointer and a constant would be addressed through the flat aperture.
__device__ __align__(16) unsigned g_gemv_zeros[4];

template <bool NT>
__device__ __forceinline__ uint4 load_chunk(const uint4 *src) {
  if (NT)
    return make_uint4(__builtin_nontemporal_load(&src->x), __builtin_nontemporal_load(&src->y),
                      __builtin_nontemporal_load(&src->z), __builtin_nontemporal_load(&src->w));
  return *src;
}

// The looping launches (PD > 1 tiles in flight per wavefront).  The kernel is a stream: its time is the
// first-byte latency plus bytes / bandwidth only if a new tile is requested whenever one has been
// consumed, so (i) every request is unconditional -- rows past the end repeat the last row and are never
// stored, chunks past the end of a row read the zero block -- and the loop body is the same on every
// pass (a separate last pass requests nothing), which lets the wait before tile p count exactly the
// PD - 1 tiles requested after it; (ii) the input side (vector, gamma or the gate's partner) is
// requested BEFORE the weight ring: loads return in order, so a vector requested behind four tiles
// would hold back the first product until all four had arrived.
template <int TYPE, int G, int KC, int PD, bool NT, bool EPI, bool DIRECT>
__device__ __forceinline__ void gemv_ring(const GemvArgs &a, float *xs_lds, float *red) {
  constexpr int XPC = Fmt<TYPE>::XPC;
  constexpr int RPW = 64 / G;
  constexpr bool QUANT = (TYPE == CTHIP_Q8_0 || TYPE == CTHIP_Q4_0);
  constexpr int SG = 4;  // float4 per thread of the staged vector that are requested ahead of the weights
  constexpr int nthr = 256;  // what the looping launches use (reading blockDim would cost a memory round trip up front)
  constexpr int waves_per_block = nthr >> 6;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int g = lane / G, l = lane % G;
  const int wave = blockIdx.x * waves_per_block + (tid >> 6);
  const int total_waves = gridDim.x * waves_per_block;
  const int nchunks = a.cols / XPC;
  const int m = blockIdx.y;
  const float *__restrict__ x = a.x + (int64_t)m * a.x_stride;
  const uint4 *__restrict__ qp = (const uint4 *)a.q;
  const int64_t row_chunks = nchunks;
  const int scales_per_row = a.cols >> 5;
  const int nrq = (a.rows + RPW - 1) / RPW;
  const float *zf = (const float *)g_gemv_zeros;
  const uint4 *z16 = (const uint4 *)g_gemv_zeros;
  const unsigned short *zh = (const unsigned short *)g_gemv_zeros;
  const bool folded = (a.pro == CTHIP_PRO_RMSNORM) || (a.pro == CTHIP_PRO_LAYERNORM && a.fold_s != nullptr);
  const bool swiglu = a.pro == CTHIP_PRO_SWIGLU;
  const bool coop = a.stage_x != 0;
  const int posv = a.pos ? a.pos[0] : 0;
  const bool layernorm = a.pro == CTHIP_PRO_LAYERNORM;
  const int n4 = a.cols >> 2;
  // a LayerNorm that is not folded is applied while staging, when a thread's share of the vector stays in registers
  const bool direct = DIRECT && coop && layernorm && !a.fold_s && n4 <= SG * nthr;
  // staged inputs whose first SG * blockDim float4 are requested ahead of the weights
  const bool early = coop && (folded || swiglu || a.pro == CTHIP_PRO_NONE || direct);

  // ---- (1) the input side ----
  float4 sv[SG], su[SG], sb[SG];
  float xr[KC][XPC];
  float gr[QUANT ? 1 : KC][QUANT ? 1 : XPC];  // gamma of an unstaged folded norm (fp32 / fp16 weights)
  const float4 *x4 = (const float4 *)x;
  // the second operand of the staging: the gate's partner, gamma, or (unused) the vector again
  const float4 *u4 = swiglu ? (const float4 *)(x + a.cols) : (layernorm || folded) && a.norm_g ? (const float4 *)a.norm_g : x4;
  const float4 *b4 = (direct && a.norm_b) ? (const float4 *)a.norm_b : x4;  // beta of a LayerNorm applied here
  if (early) {
#pragma unroll
    for (int k = 0; k < SG; k++) {
      int i = tid + k * nthr;
      i = i < n4 ? i : n4 - 1;
      sv[k] = x4[i];
      su[k] = u4[i];
      if constexpr (DIRECT) sb[k] = b4[i];  // unconditional (the vector again when unused): a request behind a branch would make every later wait a wait for everything
    }
  } else if (!coop) {
#pragma unroll
    for (int j = 0; j < KC; j++) {
      const int c = l + G * j;
      const bool ok = c < nchunks;
#pragma unroll
      for (int t = 0; t < XPC / 4; t++) {
        const float4 v = *(ok ? (const float4 *)(x + (int64_t)c * XPC + 4 * t) : (const float4 *)g_gemv_zeros);
        xr[j][4 * t + 0] = v.x;
        xr[j][4 * t + 1] = v.y;
        xr[j][4 * t + 2] = v.z;
        xr[j][4 * t + 3] = v.w;
        if (!QUANT) {
          const float4 gv = *((ok && folded && a.norm_g) ? (const float4 *)(a.norm_g + (int64_t)c * XPC + 4 * t)
                                                         : (const float4 *)g_gemv_zeros);
          gr[QUANT ? 0 : j][QUANT ? 0 : 4 * t + 0] = gv.x;
          gr[QUANT ? 0 : j][QUANT ? 0 : 4 * t + 1] = gv.y;
          gr[QUANT ? 0 : j][QUANT ? 0 : 4 * t + 2] = gv.z;
          gr[QUANT ? 0 : j][QUANT ? 0 : 4 * t + 3] = gv.w;
        }
      }
    }
  }

  // ---- (2) the weight ring ----
  auto request = [&](int rq, uint4 *w, unsigned short *s, float &epi) {
    int row = rq * RPW + g;
    row = row < a.rows ? row : a.rows - 1;
#pragma unroll
    for (int j = 0; j < KC; j++) {
      const int c = l + G * j;
      const bool ok = c < nchunks;
      w[j] = load_chunk<NT>(ok ? qp + (int64_t)row * row_chunks + c : z16);
      if (QUANT) {
        const int sidx = (TYPE == CTHIP_Q8_0) ? (c >> 1) : c;
        s[j] = *(ok ? a.d + (int64_t)row * scales_per_row + sidx : zh);
      }
    }
    // the epilogue operands of the row travel with its weights, in ONE request: the first three lanes of the
    // row's group fetch bias, residual and fold term, and the group's first lane collects them with two lane
    // shifts when it stores.  Lanes with nothing to fetch repeat a neighbour's address: a common dummy line
    // would be re-fetched by every tile of every wavefront and its L2 channel would hold all of them up.
    if (EPI) {
      const float *pb = a.bias ? a.bias + row : nullptr;
      const float *pr = a.residual ? a.residual + (int64_t)m * a.y_stride + row : nullptr;
      const float *pf = a.fold_s ? a.fold_s + row : nullptr;
      const float *any = pb ? pb : pr ? pr : pf;  // one of them exists, or the launcher takes the kernel without EPI
      epi = *(l == 0 ? (pb ? pb : any) : l == 1 ? (pr ? pr : any) : l == 2 ? (pf ? pf : any) : any);
    }
  };
  uint4 wt[PD][KC];
  unsigned short st[PD][KC];
  float epi_t[PD];
#pragma unroll
  for (int p = 0; p < PD; p++) epi_t[p] = 0.0f;
  const int own = wave < nrq ? wave : nrq - 1;  // what a slot without a tile requests: lines this wavefront fetches anyway
  // Only the first tile goes out before the staged input is picked up: requests are issued in program order and
  // a compute unit accepts them no faster than earlier ones are answered, so the whole ring in front of the
  // staging code would hold that code back until most of the ring had arrived.
  constexpr int PRE = 1;
#pragma unroll
  for (int p = 0; p < PRE; p++) {
    const int rq = wave + p * total_waves;
    request(rq < nrq ? rq : own, wt[p], st[p], epi_t[p]);
  }

  // a norm that is not folded is applied by the whole workgroup (its own loads wait for the tile above as well)
  if (coop && !early) coop_prologue(a, x, xs_lds, red, true);

  // ---- (3) the input side arrives ----
  // Statistics of a folded norm over a staged vector.  No value is shared up front (a common shift, say the
  // first element, would be one more round trip in front of everything): every thread sums its own elements
  // shifted by its own first one, and the (count, mean, squared deviation) triples are merged exactly,
  // thread -> wavefront by lane shuffles, wavefront -> workgroup through LDS.
  float mu = 0.0f, rstd = 1.0f;
  if (early) {
    float s1 = 0.0f, s2 = 0.0f, cnt = 0.0f;
    const float pivot = layernorm ? sv[0].x : 0.0f;  // this thread's first element (threads without one sum nothing)
    auto put = [&](int i, const float4 v, const float4 u) {
      if (swiglu) {
        ((float4 *)xs_lds)[i] = make_float4(ct_silu(v.x) * u.x, ct_silu(v.y) * u.y, ct_silu(v.z) * u.z, ct_silu(v.w) * u.w);
      } else if (folded || direct) {
        const float4 gm = a.norm_g ? u : make_float4(1.f, 1.f, 1.f, 1.f);
        const float d0 = v.x - pivot, d1 = v.y - pivot, d2 = v.z - pivot, d3 = v.w - pivot;
        s1 += (d0 + d1) + (d2 + d3);
        s2 = fmaf(d0, d0, s2);
        s2 = fmaf(d1, d1, s2);
        s2 = fmaf(d2, d2, s2);
        s2 = fmaf(d3, d3, s2);
        cnt += 4.0f;
        // (a norm applied here writes its values once the statistics are known)
        if (!direct) ((float4 *)xs_lds)[i] = make_float4(v.x * gm.x, v.y * gm.y, v.z * gm.z, v.w * gm.w);
      } else {
        ((float4 *)xs_lds)[i] = v;
      }
    };
#pragma unroll
    for (int k = 0; k < SG; k++) {
      const int i = tid + k * nthr;
      if (i < n4) put(i, sv[k], su[k]);
    }
    // longer vectors: the rest is requested behind the first tiles
    for (int i = tid + SG * nthr; i < n4; i += nthr) put(i, x4[i], u4[i]);
    if ((folded || direct) && layernorm) {
      const float inv = cnt > 0.0f ? 1.0f / cnt : 0.0f;
      const float mean_t = cnt > 0.0f ? pivot + s1 * inv : 0.0f;
      const float n_w = wave_sum(cnt);
      const float mean_w = wave_sum(cnt * mean_t) / fmaxf(n_w, 1.0f);
      const float dm = mean_t - mean_w;
      const float m2_w = wave_sum(s2 - s1 * s1 * inv + cnt * dm * dm);
      if (lane == 0) {
        red[tid >> 6] = n_w;
        red[8 + (tid >> 6)] = mean_w;
        red[16 + (tid >> 6)] = m2_w;
      }
    } else if (folded) {  // RMSNorm: the plain sum of squares
      s2 = wave_sum(s2);
      if (lane == 0) red[tid >> 6] = s2;
    }
    __syncthreads();  // publishes the staged vector and the per-wavefront statistics
    if (folded || direct) {
      const float inv_n = 1.0f / (float)a.cols;
      float m2 = 0.0f;
      if (layernorm) {
        float sum = 0.0f;
        for (int w = 0; w < waves_per_block; w++) sum += red[w] * red[8 + w];
        mu = sum * inv_n;
        for (int w = 0; w < waves_per_block; w++) {
          const float dw = red[8 + w] - mu;
          m2 += red[16 + w] + red[w] * dw * dw;
        }
      } else {
        for (int w = 0; w < waves_per_block; w++) m2 += red[w];
      }
      rstd = 1.0f / sqrtf(fmaxf(m2 * inv_n, 0.0f) + a.eps);
    }
    if (direct) {
      // y = ((x - mean) * rstd) * gamma + beta, as the unfused LayerNorm item computes it; nothing is left for the epilogue
#pragma unroll
      for (int k = 0; k < SG; k++) {
        const int i = tid + k * nthr;
        if (i < n4) {
          const float4 v = sv[k];
          const float4 gm = a.norm_g ? su[k] : make_float4(1.f, 1.f, 1.f, 1.f);
          const float4 bt = a.norm_b ? sb[k] : make_float4(0.f, 0.f, 0.f, 0.f);
          ((float4 *)xs_lds)[i] = make_float4((v.x - mu) * rstd * gm.x + bt.x, (v.y - mu) * rstd * gm.y + bt.y,
                                              (v.z - mu) * rstd * gm.z + bt.z, (v.w - mu) * rstd * gm.w + bt.w);
        }
      }
      mu = 0.0f;
      rstd = 1.0f;
      __syncthreads();
    }
  }
  if (coop) {
#pragma unroll
    for (int j = 0; j < KC; j++) {
      const int c = l + G * j;
      const bool ok = c < nchunks;
#pragma unroll
      for (int t = 0; t < XPC / 4; t++) {
        const float4 v = ok ? *(const float4 *)(xs_lds + (int64_t)c * XPC + 4 * t) : make_float4(0.f, 0.f, 0.f, 0.f);
        xr[j][4 * t + 0] = v.x;
        xr[j][4 * t + 1] = v.y;
        xr[j][4 * t + 2] = v.z;
        xr[j][4 * t + 3] = v.w;
      }
    }
  }
#pragma unroll
  for (int p = PRE; p < PD; p++) {
    const int rq = wave + p * total_waves;
    request(rq < nrq ? rq : own, wt[p], st[p], epi_t[p]);
  }
  if (folded && !coop) {
    // every group of G lanes holds the whole vector in registers: mean, then squared deviations, then gamma
    const float inv_n = 1.0f / (float)a.cols;
    if (layernorm) {
      float s1 = 0.0f;
#pragma unroll
      for (int j = 0; j < KC; j++)
#pragma unroll
        for (int e = 0; e < XPC; e++) s1 += xr[j][e];  // lanes past the end hold zeros
      mu = group_sum<G>(s1) * inv_n;
    }
    float s2 = 0.0f;
    {
#pragma unroll
      for (int j = 0; j < KC; j++) {
        const int c = l + G * j;
        const bool ok = c < nchunks;
#pragma unroll
        for (int t = 0; t < XPC / 4; t++) {
          float gg[4] = {1.f, 1.f, 1.f, 1.f};
          if (QUANT) {  // (the launcher stages quantised folded launches; kept for completeness)
            if (ok && a.norm_g) {
              const float4 gv = *(const float4 *)(a.norm_g + (int64_t)c * XPC + 4 * t);
              gg[0] = gv.x, gg[1] = gv.y, gg[2] = gv.z, gg[3] = gv.w;
            }
          } else if (a.norm_g) {
#pragma unroll
            for (int e = 0; e < 4; e++) gg[e] = gr[QUANT ? 0 : j][QUANT ? 0 : 4 * t + e];
          }
#pragma unroll
          for (int e = 0; e < 4; e++) {
            const float d = ok ? xr[j][4 * t + e] - mu : 0.0f;
            s2 = fmaf(d, d, s2);
            xr[j][4 * t + e] *= gg[e];
          }
        }
      }
    }
    rstd = 1.0f / sqrtf(group_sum<G>(s2) * inv_n + a.eps);
  }
  float xs[KC];
#pragma unroll
  for (int j = 0; j < KC; j++) {
    float s = 0.0f;
    if (TYPE == CTHIP_Q4_0) {
#pragma unroll
      for (int e = 0; e < XPC; e++) s += xr[j][e];
    }
    xs[j] = s;
  }

  // ---- (4) stream the rows: slot p of the ring holds tile base + p * total_waves ----
  float best_v = -INFINITY;
  int best_i = 0x7fffffff;
  auto consume = [&](int p, int rq) {
    float acc = 0.0f;
#pragma unroll
    for (int j = 0; j < KC; j++) {
      const float scale = QUANT ? half_bits_to_float(st[p][j]) : 1.0f;
      acc += chunk_dot<TYPE>(wt[p][j], scale, xr[j], xs[j]);
    }
    acc = group_sum<G>(acc);
    // valid in the group's first lane, which is the one that stores
    const float bias = (EPI && a.bias) ? epi_t[p] : 0.0f;
    const float resid = (EPI && a.residual) ? dpp_f<0x101>(epi_t[p]) : 0.0f;  // row_shl:1
    const float fs = (EPI && a.fold_s) ? dpp_f<0x102>(epi_t[p]) : 0.0f;       // row_shl:2
    if (folded) acc = rstd * (acc - mu * fs);
    const int row = rq * RPW + g;
    if (RPW >= 2 && a.pair_swiglu) {
      // SwiGLU across the (gate, up) row pair held by neighbouring lane groups
      const float mine = acc + bias;
      const float other = __shfl_xor(mine, G & 63, 64);
      if (l == 0 && (g & 1) == 0 && row < a.rows) a.y[(int64_t)m * a.y_stride + (row >> 1)] = ct_silu(mine) * other;
    } else if (l == 0 && row < a.rows) {
      const float v = gemv_store(a, m, row, acc, posv, bias, resid);
      argmax_merge(best_v, best_i, v, row);
    }
  };
  const int stride = PD * total_waves;
  int base = wave;
  for (; base + stride < nrq; base += stride) {  // every slot holds a tile; slot 0 has a successor
#pragma unroll
    for (int p = 0; p < PD; p++) {
      const int rq = base + p * total_waves;
      consume(p, rq);
      const int nxt = rq + stride;
      request(nxt < nrq ? nxt : rq, wt[p], st[p], epi_t[p]);
    }
  }
#pragma unroll
  for (int p = 0; p < PD; p++) {
    const int rq = base + p * total_waves;
    if (rq < nrq) consume(p, rq);  // wavefront-uniform
  }
  if (a.am_val) gemv_argmax_tail(a, wave, lane, best_v, best_i);
}

// PD = weight tiles a wavefront keeps in flight: 1 for the small, latency-bound launches (one tile
// per wavefront), 4 for the large ones, whose throughput is bytes-in-flight / memory latency.
// NT: the weights are requested with the non-temporal hint.  A model whose weights exceed the 256 MB Infinity
// Cache streams all of them from HBM every step whatever the hint; without it the stream also evicts the
// vectors, fold terms and KV rows that the step does reuse.
template <int TYPE, int G, int KC, int PD, bool NT, bool EPI = false, bool DIRECT = false>
__global__ __launch_bounds__(256) void k_gemv(GemvArgs a) {
  constexpr int XPC = Fmt<TYPE>::XPC;
  constexpr int RPW = 64 / G;  // rows per wavefront per iteration
  constexpr bool QUANT = (TYPE == CTHIP_Q8_0 || TYPE == CTHIP_Q4_0);
  extern __shared__ float xs_lds[];  // a.cols floats when a prologue is fused
  __shared__ float red[24];
  const int lane = threadIdx.x & 63;
  const int g = lane / G, l = lane % G;
  const int waves_per_block = blockDim.x >> 6;
  const int wave = blockIdx.x * waves_per_block + (threadIdx.x >> 6);
  const int total_waves = gridDim.x * waves_per_block;
  const int nchunks = a.cols / XPC;
  const int m = blockIdx.y;
  const float *__restrict__ x = a.x + (int64_t)m * a.x_stride;
  const uint4 *__restrict__ qp = (const uint4 *)a.q;
  const int64_t row_chunks = nchunks;  // 16-byte chunks per row in the quant plane
  const int scales_per_row = a.cols >> 5;
  const int nrq = (a.rows + RPW - 1) / RPW;

  // LayerNorm / RMSNorm folded through the product instead of applied to the input first:
  //   sum_k W[r,k] * (((x_k - mu) * rstd) * g_k + b_k) = rstd * (sum_k W[r,k] (g_k x_k) - mu * S_r) + C_r
  // with S_r = sum_k W[r,k] g_k and C_r = sum_k W[r,k] b_k (+ bias) precomputed per matrix.  The
  // statistics mu, rstd are then needed only by the epilogue, so their reductions overlap the weight
  // stream instead of preceding it.  RMSNorm has no mu / beta term and needs no precomputation.
  const bool folded = (a.pro == CTHIP_PRO_RMSNORM) || (a.pro == CTHIP_PRO_LAYERNORM && a.fold_s != nullptr);
  const bool coop = a.stage_x != 0;  // input staged (and normalised, unless folded) once per workgroup
  auto load = [&](int rq, uint4 *w, unsigned short *s, float &bias, float &resid, float &fs) {
    const int row = rq * RPW + g;
    const bool rok = row < a.rows;
    // the epilogue operands of the row travel with its weights
    bias = (rok && a.bias) ? a.bias[row] : 0.0f;
    resid = (rok && a.residual) ? a.residual[(int64_t)m * a.y_stride + row] : 0.0f;
    fs = (rok && a.fold_s) ? a.fold_s[row] : 0.0f;
#pragma unroll
    for (int j = 0; j < KC; j++) {
      const int c = l + G * j;
      const bool ok = rok && c < nchunks;
      if (NT) {
        uint4 t = make_uint4(0u, 0u, 0u, 0u);
        if (ok) {
          const uint4 *src = &qp[(int64_t)row * row_chunks + c];
          t = make_uint4(__builtin_nontemporal_load(&src->x), __builtin_nontemporal_load(&src->y),
                         __builtin_nontemporal_load(&src->z), __builtin_nontemporal_load(&src->w));
        }
        w[j] = t;
      } else {
        w[j] = ok ? qp[(int64_t)row * row_chunks + c] : make_uint4(0u, 0u, 0u, 0u);
      }
      if (QUANT) {
        const int sidx = (TYPE == CTHIP_Q8_0) ? (c >> 1) : c;
        s[j] = ok ? a.d[(int64_t)row * scales_per_row + sidx] : (unsigned short)0;
      }
    }
  };

  if constexpr (PD > 1) {
    gemv_ring<TYPE, G, KC, PD, NT, EPI, DIRECT>(a, xs_lds, red);
    return;
  }
  // Everything this wavefront needs from memory is requested before any arithmetic so the
  // latencies overlap: position, the first weight tiles, then the input vector.
  const int posv = a.pos ? a.pos[0] : 0;
  uint4 wt[PD][KC];
  unsigned short st[PD][KC];
  float bias_t[PD], resid_t[PD], fs_t[PD];
#pragma unroll
  for (int p = 0; p < PD; p++) {
    bias_t[p] = resid_t[p] = fs_t[p] = 0.0f;
    const int rq = wave + p * total_waves;
    if (rq < nrq) load(rq, wt[p], st[p], bias_t[p], resid_t[p], fs_t[p]);
  }

  float xr[KC][XPC];
  float xs[KC];
  float bs1 = 0.0f, bs2 = 0.0f;  // block-wide statistics when the folded norm is staged
  const float pivot = (folded && a.pro == CTHIP_PRO_LAYERNORM) ? x[0] : 0.0f;
  if (coop) {
    if (folded) coop_fold(a, x, xs_lds, red, pivot, bs1, bs2);
    else coop_prologue(a, x, xs_lds, red, a.pro != CTHIP_PRO_NONE);
  }
  const float *__restrict__ xsrc = coop ? xs_lds : x;
#pragma unroll
  for (int j = 0; j < KC; j++) {
    const int c = l + G * j;
    const bool ok = c < nchunks;
#pragma unroll
    for (int t = 0; t < XPC / 4; t++) {
      float4 v = ok ? *(const float4 *)(xsrc + (int64_t)c * XPC + 4 * t) : make_float4(0.f, 0.f, 0.f, 0.f);
      xr[j][4 * t + 0] = v.x;
      xr[j][4 * t + 1] = v.y;
      xr[j][4 * t + 2] = v.z;
      xr[j][4 * t + 3] = v.w;
    }
  }
  float mu = 0.0f, rstd = 1.0f;
  if (folded) {
    // every group of G lanes holds the whole vector: shifted one-pass mean / variance (the shift by
    // x[0] keeps E[d^2] - E[d]^2 well conditioned), then scale the slice by gamma -- unless the
    // workgroup has already done both while staging
    float s1 = 0.0f, s2 = 0.0f;
    if (!coop) {
#pragma unroll
    for (int j = 0; j < KC; j++) {
      const int c = l + G * j;
      const bool ok = c < nchunks;
#pragma unroll
      for (int t = 0; t < XPC / 4; t++) {
        const float4 gv = (ok && a.norm_g) ? *(const float4 *)(a.norm_g + (int64_t)c * XPC + 4 * t)
                                           : make_float4(1.f, 1.f, 1.f, 1.f);
        const float gg[4] = {gv.x, gv.y, gv.z, gv.w};
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const float d = ok ? xr[j][4 * t + e] - pivot : 0.0f;
          s1 += d;
          s2 = fmaf(d, d, s2);
          xr[j][4 * t + e] *= gg[e];
        }
      }
    }
    }
    const float inv_n = 1.0f / (float)a.cols;
    const float m1 = (coop ? bs1 : group_sum<G>(s1)) * inv_n;
    const float m2 = (coop ? bs2 : group_sum<G>(s2)) * inv_n;
    if (a.pro == CTHIP_PRO_LAYERNORM) {
      mu = pivot + m1;
      rstd = 1.0f / sqrtf(fmaxf(m2 - m1 * m1, 0.0f) + a.eps);
    } else {
      rstd = 1.0f / sqrtf(m2 + a.eps);
    }
  }
#pragma unroll
  for (int j = 0; j < KC; j++) {
    float s = 0.0f;
    if (TYPE == CTHIP_Q4_0) {
#pragma unroll
      for (int e = 0; e < XPC; e++) s += xr[j][e];
    }
    xs[j] = s;
  }

  // ---- stream the rows: slot p of the ring holds tile base + p*total_waves ----
  float best_v = -INFINITY;
  int best_i = 0x7fffffff;
  for (int base = wave; base < nrq; base += PD * total_waves) {
#pragma unroll
    for (int p = 0; p < PD; p++) {
      const int rq = base + p * total_waves;
      if (rq < nrq) {  // wavefront-uniform
        float acc = 0.0f;
#pragma unroll
        for (int j = 0; j < KC; j++) {
          const float scale = QUANT ? half_bits_to_float(st[p][j]) : 1.0f;
          acc += chunk_dot<TYPE>(wt[p][j], scale, xr[j], xs[j]);
        }
        acc = group_sum<G>(acc);
        if (folded) acc = rstd * (acc - mu * fs_t[p]);
        const int row = rq * RPW + g;
        if (RPW >= 2 && a.pair_swiglu) {
          // SwiGLU across the (gate, up) row pair held by neighbouring lane groups
          const float mine = acc + bias_t[p];
          const float other = __shfl_xor(mine, G & 63, 64);
          if (l == 0 && (g & 1) == 0 && row < a.rows) a.y[(int64_t)m * a.y_stride + (row >> 1)] = ct_silu(mine) * other;
        } else if (l == 0 && row < a.rows) {
          const float v = gemv_store(a, m, row, acc, posv, bias_t[p], resid_t[p]);
          argmax_merge(best_v, best_i, v, row);
        }
        const int nxt = rq + PD * total_waves;
        if (nxt < nrq) load(nxt, wt[p], st[p], bias_t[p], resid_t[p], fs_t[p]);
      }
    }
  }
  if (a.am_val) gemv_argmax_tail(a, wave, lane, best_v, best_i);
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
typedef void (*gemv_fn)(GemvArgs);
struct GemvVariant {
  int type, G, KC;
  gemv_fn fn[2];       // looping launches: [0] cached weights, [1] streamed (non-temporal) weights
  gemv_fn fn_epi[2];   // the same with per-row epilogue operands (bias, residual, fold term) travelling in the ring
  gemv_fn fn_direct[2];  // looping, no epilogue operands, a LayerNorm applied to the staged input
  gemv_fn fn_small[2]; // one tile per wavefront: latency-bound launches
};
// large launches keep about 12 sixteen-byte loads per lane in flight
#define PD_OF(KC) (KC >= 12 ? 1 : KC >= 6 ? 2 : 4)
#define V(T, G, KC)                                                                           \
  {T, G, KC, {k_gemv<T, G, KC, PD_OF(KC), false>, k_gemv<T, G, KC, PD_OF(KC), true>},         \
   {k_gemv<T, G, KC, PD_OF(KC), false, PD_OF(KC) != 1>, k_gemv<T, G, KC, PD_OF(KC), true, PD_OF(KC) != 1>}, \
   {k_gemv<T, G, KC, PD_OF(KC), false, false, PD_OF(KC) != 1>, k_gemv<T, G, KC, PD_OF(KC), true, false, PD_OF(KC) != 1>}, \
   {k_gemv<T, G, KC, 1, false>, k_gemv<T, G, KC, 1, true>}}
static const GemvVariant kVariants[] = {
    V(CTHIP_Q8_0, 16, 1), V(CTHIP_Q8_0, 16, 2), V(CTHIP_Q8_0, 16, 3), V(CTHIP_Q8_0, 16, 4),
    V(CTHIP_Q8_0, 32, 3), V(CTHIP_Q8_0, 32, 4), V(CTHIP_Q8_0, 64, 3), V(CTHIP_Q8_0, 64, 4),
    V(CTHIP_Q8_0, 64, 6), V(CTHIP_Q8_0, 64, 8),
    V(CTHIP_Q4_0, 16, 1), V(CTHIP_Q4_0, 16, 2), V(CTHIP_Q4_0, 32, 2), V(CTHIP_Q4_0, 64, 1),
    V(CTHIP_Q4_0, 64, 2), V(CTHIP_Q4_0, 64, 3), V(CTHIP_Q4_0, 64, 4),
    V(CTHIP_F32, 16, 4), V(CTHIP_F32, 64, 1), V(CTHIP_F32, 64, 2), V(CTHIP_F32, 64, 3), V(CTHIP_F32, 64, 4),
    V(CTHIP_F32, 64, 6), V(CTHIP_F32, 64, 8), V(CTHIP_F32, 64, 12), V(CTHIP_F32, 64, 16), V(CTHIP_F32, 64, 24),
    V(CTHIP_F16, 16, 2), V(CTHIP_F16, 64, 1), V(CTHIP_F16, 64, 2), V(CTHIP_F16, 64, 3), V(CTHIP_F16, 64, 4),
    V(CTHIP_F16, 64, 6), V(CTHIP_F16, 64, 8), V(CTHIP_F16, 64, 12),
};
#undef V
#undef PD_OF

static int xpc_of(int type) {
  switch (type) {
    case CTHIP_Q8_0: return 16;
    case CTHIP_Q4_0: return 32;
    case CTHIP_F16: return 8;
    default: return 4;
  }
}

static const GemvVariant *pick_variant(int type, int cols) {
  const int xpc = xpc_of(type);
  if (cols % xpc) return nullptr;
  const int nchunks = cols / xpc;
  const GemvVariant *best = nullptr;
  int best_waste = 1 << 30;
  for (const GemvVariant &v : kVariants) {
    if (v.type != type || v.G * v.KC < nchunks) continue;
    int waste = v.G * v.KC - nchunks;
    if (waste < best_waste || (waste == best_waste && best && v.G < best->G)) {
      best = &v;
      best_waste = waste;
    }
  }
  return best;
}

int launch_prologue(float *out, const float *x, int cols, int pro, const float *g, const float *b, float eps,
                    int64_t x_stride, int m) {
  if (m == 0) return 0;
  hipLaunchKernelGGL(k_prologue, dim3(m), dim3(256), 0, state().stream, out, x, cols, pro, g, b, eps, x_stride);
  CTHIP_LAUNCH_CHECK();
  return 0;
}

bool gemv_is_direct(const WMat *w) { return pick_variant(w->type, (int)w->cols) != nullptr; }
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

// Queues one fused Linear on the stream. Used by cthip_linear and by the decoder.
int launch_gemv(const WMat *w, GemvArgs a, int m) {
  State &s = state();
  a.q = w->q;
  a.d = (const unsigned short *)w->d;
  a.rows = (int)w->rows;
  a.cols = (int)w->cols;
  if (a.split1 <= 0) a.split1 = a.split2 = a.rows;
  if (a.am_val && m != 1) return fail(CTHIP_E_BAD_ARG, "gemv: the fused argmax needs m == 1");
  const GemvVariant *v = pick_variant(w->type, a.cols);
  if (a.pair_swiglu && (!v || v->G > 32 || (a.rows & 1) || a.am_val || a.residual || a.split1 != a.rows))
    return fail(CTHIP_E_UNSUPPORTED, "gemv: the paired SwiGLU epilogue needs two rows per wavefront and plain outputs");
  if (v) {
    const int rpw = 64 / v->G;
    const int nrq = (a.rows + rpw - 1) / rpw;
    dim3 grid, block;
    const bool folded = (a.pro == CTHIP_PRO_RMSNORM) || (a.pro == CTHIP_PRO_LAYERNORM && a.fold_s != nullptr);
    const bool quantised = w->type == CTHIP_Q8_0 || w->type == CTHIP_Q4_0;
    // The input vector goes through LDS once per workgroup when it must be normalised or gated first,
    // or when it is large next to a weight tile (a 4-bit tile multiplies 8 input bytes per weight byte):
    // then four wavefronts share one copy and every wavefront takes several tiles.  Quantised launches with a
    // folded norm stage at every size: a lane's slice is 48-64 floats, and gamma * x plus the statistics once
    // per workgroup beat once per wavefront (GPT-2 decode: Q8_0 284.6 -> 280.3 us / step, Q4_0 339 -> 308;
    // fp32 / fp16 weights, 12-24 floats per lane, measured the other way round: 354 -> 369, 328 -> 347).
    const bool stage = (a.pro != CTHIP_PRO_NONE && !folded) || (w->type == CTHIP_Q4_0 && a.cols >= 1024) ||
                       (folded && (a.cols >= 2048 || quantised));
    const size_t lds = stage ? sizeof(float) * (size_t)a.cols : 0;
    if (lds > 64 * 1024) return fail(CTHIP_E_UNSUPPORTED, "gemv: %d input features exceed the LDS staging buffer", a.cols);
    a.stage_x = stage ? 1 : 0;
    bool small, direct = false;
    if (!stage && nrq <= 2048) {
      // small matrices are pure latency: one tile per wavefront, one wavefront per workgroup, spread
      // over as many compute units as there are tiles
      small = true;
      block = dim3(64);
      grid = dim3(nrq, m);
    } else if (stage && nrq <= s.compute_units * 3) {
      // one tile per wavefront, as many wavefronts per workgroup (at most three) as leave about one workgroup
      // per compute unit: fewer workgroups repeat the staging less, but idle units stream nothing
      // (GPT-2 c_attn / c_fc, 576 / 768 tiles: 3 per workgroup 279.9 us / step, 4: 283.1, 2: 286.8, 1: 289.1).
      // Beyond three tiles per compute unit the looping launch below is ahead (TinyLlama wo, 1024 tiles:
      // 0.780 -> 0.772 ms / step; with the limit at two, GPT-2 loses 1 %)
      small = true;
      int wpb = (nrq + s.compute_units - 1) / s.compute_units;
      wpb = wpb < 1 ? 1 : wpb > 3 ? 3 : wpb;
      block = dim3(64 * wpb);
      grid = dim3((nrq + wpb - 1) / wpb, m);
    } else {
      // larger matrices: at least one wavefront per SIMD, more (up to what the register budget keeps
      // resident) once every wavefront has four tiles; all loop over the same number of tiles (an
      // uneven last pass would idle most of the chip)
      small = false;
      static int occ_cache[sizeof(kVariants) / sizeof(kVariants[0])];
      const int vi = (int)(v - kVariants);
      if (occ_cache[vi] == 0) {
        int nb = 0;
        CTHIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb, v->fn[0], 256, 16 * 1024));
        occ_cache[vi] = nb > 0 ? nb : 1;
      }
      block = dim3(256);
      const int base = s.compute_units * 4;
      // unstaged: a wavefront per tile up to three resident wavefronts per SIMD (fp32 GPT-2 decode with every large
      // launch at 1024 / 2048 / 3072 / 4096 wavefronts: 369 / 343 / 334 / 343 us per step)
      int wanted = stage ? (nrq + 3) / 4 : nrq;
      if (wanted < base) wanted = base;
      const int cap = base * (stage || occ_cache[vi] < 3 ? occ_cache[vi] : 3);
      if (wanted > cap) wanted = cap;
      // staged launches pay the input staging once per workgroup: whole workgroups per compute unit, two
      // when there is work for more than one (measured best; a third does not fit beside the first two)
      if (stage && wanted > base && occ_cache[vi] >= 2) wanted = 2 * base;
      static const char *ovr = getenv("CTHIP_GEMV_WAVES");  // tuning aid: overrides the wavefront count
      if (ovr && atoi(ovr) > 0) wanted = atoi(ovr);
      const int iters = (nrq + wanted - 1) / wanted;
      const int waves = (nrq + iters - 1) / iters;
      grid = dim3((waves + 3) / 4, m);
      // the ring requests all its slots unconditionally: a wavefront with a single tile takes the kernel without one
      if (iters == 1) small = true;
      // A looping launch normalises the staged vector itself rather than carrying the fold terms: two more
      // operands per row in the weight ring hold the stream up more than the second barrier of the staging costs
      // (GPT-2 lm_head: 11.0 us folded, 10.0 us with neither)
      if (!small && stage && a.pro == CTHIP_PRO_LAYERNORM && a.fold_s && !a.bias0 && !a.residual && a.cols <= 4096) {
        a.fold_s = nullptr;
        a.bias = nullptr;
      }
      direct = !small && stage && a.pro == CTHIP_PRO_LAYERNORM && !a.fold_s && !a.bias && !a.residual && a.cols <= 4096;
    }
    const int nwaves = (int)(grid.x * (block.x / 64));
    if (a.am_val && nwaves > kGemvMaxWaves)
      return fail(CTHIP_E_UNSUPPORTED, "gemv: %d wavefronts exceed the argmax scratch", nwaves);
    const int nt = s.gemv_stream < 0 ? (w->stream ? 1 : 0) : s.gemv_stream;
    const bool epi = a.bias || a.residual || a.fold_s;
    hipLaunchKernelGGL(small ? v->fn_small[nt] : epi ? v->fn_epi[nt] : direct ? v->fn_direct[nt] : v->fn[nt], grid, block, lds,
                       s.stream, a);
    CTHIP_LAUNCH_CHECK();
    if (a.am_val) {
      hipLaunchKernelGGL(k_argmax_finish, dim3(1), dim3(256), 0, s.stream, a, nwaves);
      CTHIP_LAUNCH_CHECK();
    }
    return 0;
  }
  // generic path: prologue into a temporary, then wave-per-row
  float *tmp = nullptr;
  if (a.pro != CTHIP_PRO_NONE) {
    int rc = alloc_scratch((void **)&tmp, sizeof(float) * (size_t)a.cols * m);  // fully written below
    if (rc) return rc;
    hipLaunchKernelGGL(k_prologue, dim3(m), dim3(256), 0, s.stream, tmp, a.x, a.cols, a.pro, a.norm_g, a.norm_b, a.eps,
                       a.x_stride);
    CTHIP_LAUNCH_CHECK();
    a.x = tmp;
    a.x_stride = a.cols;
    a.pro = CTHIP_PRO_NONE;
  }
  int blocks = (a.rows + 3) / 4;
  int cap = s.compute_units * 8;
  if (cap * 4 > kGemvMaxWaves) cap = kGemvMaxWaves / 4;
  dim3 grid(blocks < cap ? blocks : cap, m), block(256);
  switch (w->type) {
    case CTHIP_Q8_0: hipLaunchKernelGGL(k_gemv_generic<CTHIP_Q8_0>, grid, block, 0, s.stream, a); break;
    case CTHIP_Q4_0: hipLaunchKernelGGL(k_gemv_generic<CTHIP_Q4_0>, grid, block, 0, s.stream, a); break;
    case CTHIP_F16: hipLaunchKernelGGL(k_gemv_generic<CTHIP_F16>, grid, block, 0, s.stream, a); break;
    default: hipLaunchKernelGGL(k_gemv_generic<CTHIP_F32>, grid, block, 0, s.stream, a); break;
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
  if (!gemv_is_direct(w)) return fail(CTHIP_E_UNSUPPORTED, "cthip_wmat_fold_layernorm: no single-row kernel covers %lld columns", (long long)w->cols);
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
      hipLaunchKernelGGL(k_prologue, dim3(m), dim3(256), 0, state().stream, tmp, x, (int)w->cols, prologue, norm_g, norm_b,
                         eps, (int64_t)(prologue == CTHIP_PRO_SWIGLU ? 2 * w->cols : w->cols));
      CTHIP_LAUNCH_CHECK();
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
  if (!strcmp(name, "gemm_bf16")) {  // 1 = operands rounded to bf16, 0 = back to the default
    state().gemm_precision = value ? GEMM_BF16 : GEMM_BF16X3;
    return 0;
  }
  return fail(CTHIP_E_BAD_ARG, "cthip_set_option: unknown option '%s'", name);
}

}  // extern "C"
