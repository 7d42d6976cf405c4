// The dequant-in-register GEMV kernels (templates) and their variant table type.  Included by linear.hip (launch
// logic) and by one translation unit per weight type (gemv_*.hip), which instantiate that type's variants: the 35
// variants x 8 kernels compile in parallel instead of in one three-minute unit.
#pragma once
#include "common.h"
#include "gemv_plan.h"

namespace cthip {

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
    const uint32_t lo = dw[t] & 0x0f0f0f0fu;
    const uint32_t hi = (dw[t] >> 4) & 0x0f0f0f0fu;
    s = fmaf(ubyte0_f32(lo), x[4 * t + 0], s);
    s = fmaf(ubyte1_f32(lo), x[4 * t + 1], s);
    s = fmaf(ubyte2_f32(lo), x[4 * t + 2], s);
    s = fmaf(ubyte3_f32(lo), x[4 * t + 3], s);
    s = fmaf(ubyte0_f32(hi), x[16 + 4 * t + 0], s);
    s = fmaf(ubyte1_f32(hi), x[16 + 4 * t + 1], s);
    s = fmaf(ubyte2_f32(hi), x[16 + 4 * t + 2], s);
    s = fmaf(ubyte3_f32(hi), x[16 + 4 * t + 3], s);
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
      float4 u = ((const float4 *)(x + (a.up_off ? a.up_off : a.cols)))[i];
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
// loads gamma or repeats the statistics.  xs must hold a.cols floats, red 16; blockDim.x <= 256.
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
  // both sums cross the workgroup behind ONE barrier, which also publishes xs (red holds 8 + 8 partials)
  s1 = wave_sum(s1);
  s2 = wave_sum(s2);
  if ((tid & 63) == 0) {
    red[tid >> 6] = s1;
    red[8 + (tid >> 6)] = s2;
  }
  __syncthreads();
  float t1 = 0.0f, t2 = 0.0f;
  for (int w = 0; w < nw; w++) {
    t1 += red[w];
    t2 += red[8 + w];
  }
  s1_out = t1;
  s2_out = t2;
}

// Sixteen bytes that stay zero: lanes with nothing to fetch point their requests here, so that every
// lane issues the same loads and no request sits behind a branch (the compiler can then wait for
// exactly the tile it needs instead of for everything in flight).  Not const: a select between a
// kernel-argument pointer and a constant would be addressed through the flat aperture.
static __device__ __align__(16) unsigned g_gemv_zeros[4];  // one per translation unit

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
template <int TYPE, int G, int KC, int PD, bool NT, bool EPI, bool DIRECT, bool PAIR1>
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
  const int64_t row_chunks = a.ld_chunks ? a.ld_chunks : nchunks;
  const int scales_per_row = a.ld_scales ? a.ld_scales : a.cols >> 5;
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
  const float4 *u4 = swiglu ? (const float4 *)(x + (a.up_off ? a.up_off : a.cols)) : (layernorm || folded) && a.norm_g ? (const float4 *)a.norm_g : x4;
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
  auto request = [&](int rq, uint4 *w, unsigned *s, float &epi) {
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
  // (one 32-bit register per scale: 16-bit elements would be packed in pairs right behind their loads, and that
  // use would make the wavefront wait for the tile before it has requested anything else)
  unsigned st[PD][KC];
  float epi_t[PD];
#pragma unroll
  for (int p = 0; p < PD; p++) epi_t[p] = 0.0f;
  // Which tile ring slot p holds first.  Plain: wave + p * total_waves.  With one row per wavefront and the paired
  // SwiGLU epilogue a wavefront takes (gate, up) row pairs: slots 2k and 2k + 1 hold rows 2 (wave + k * total_waves)
  // and the one after it; a slot's next tile is PD * total_waves further on either way.
  // (PAIR1 is its own instantiation: the others keep the plain order as constants)
  constexpr bool pair1 = PAIR1;
  static_assert(!PAIR1 || (RPW == 1 && PD >= 2 && PD % 2 == 0 && !EPI && !DIRECT), "row pairs in ring slots: one row per wavefront, an even ring");
  const int first = pair1 ? 2 * wave : wave;
  auto slot_off = [&](int p) { return pair1 ? (p >> 1) * 2 * total_waves + (p & 1) : p * total_waves; };
  const int own = first < nrq ? first : nrq - 1;  // what a slot without a tile requests: lines this wavefront fetches anyway
  // Only the first tile goes out before the staged input is picked up: requests are issued in program order and
  // a compute unit accepts them no faster than earlier ones are answered, so the whole ring in front of the
  // staging code would hold that code back until most of the ring had arrived.
  constexpr int PRE = 1;
#pragma unroll
  for (int p = 0; p < PRE; p++) {
    const int rq = first + slot_off(p);
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
    const int rq = first + slot_off(p);
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
  float held_gate = 0.0f;
  auto consume = [&](int p, int rq) {
    float acc = 0.0f;
#pragma unroll
    for (int j = 0; j < KC; j++) {
      const float scale = QUANT ? half_bits_to_float((unsigned short)st[p][j]) : 1.0f;
      acc += chunk_dot<TYPE>(wt[p][j], scale, xr[j], xs[j]);
    }
    acc = group_sum<G>(acc);
    // valid in the group's first lane, which is the one that stores
    const float bias = (EPI && a.bias) ? epi_t[p] : 0.0f;
    const float resid = (EPI && a.residual) ? dpp_f<0x101>(epi_t[p]) : 0.0f;  // row_shl:1
    const float fs = (EPI && a.fold_s) ? dpp_f<0x102>(epi_t[p]) : 0.0f;       // row_shl:2
    if (folded) acc = rstd * (acc - mu * fs);
    const int row = rq * RPW + g;
    if (PAIR1) {
      // SwiGLU across the (gate, up) row pair held by two neighbouring ring slots of this wavefront
      if (p & 1) {
        if (l == 0 && row < a.rows) a.y[(int64_t)m * a.y_stride + (row >> 1)] = ct_silu(held_gate) * (acc + bias);
      } else {
        held_gate = acc + bias;
      }
    } else if (RPW >= 2 && a.pair_swiglu) {
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
  int base = first;
  for (; base + stride < nrq; base += stride) {  // every slot holds a tile; slot 0 has a successor
#pragma unroll
    for (int p = 0; p < PD; p++) {
      const int rq = base + slot_off(p);
      consume(p, rq);
      const int nxt = rq + stride;
      request(nxt < nrq ? nxt : rq, wt[p], st[p], epi_t[p]);
    }
  }
#pragma unroll
  for (int p = 0; p < PD; p++) {
    const int rq = base + slot_off(p);
    if (rq < nrq) consume(p, rq);  // wavefront-uniform
  }
  if (a.am_val) gemv_argmax_tail(a, wave, lane, best_v, best_i);
}

// PD = weight tiles a wavefront keeps in flight: 1 for the small, latency-bound launches (one tile
// per wavefront), 4 for the large ones, whose throughput is bytes-in-flight / memory latency.
// NT: the weights are requested with the non-temporal hint.  A model whose weights exceed the 256 MB Infinity
// Cache streams all of them from HBM every step whatever the hint; without it the stream also evicts the
// vectors, fold terms and KV rows that the step does reuse.
template <int TYPE, int G, int KC, int PD, bool NT, bool EPI = false, bool DIRECT = false, bool PAIR1 = false>
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
  const int64_t row_chunks = a.ld_chunks ? a.ld_chunks : nchunks;  // 16-byte chunks per row in the quant plane
  const int scales_per_row = a.ld_scales ? a.ld_scales : a.cols >> 5;
  const int nrq = (a.rows + RPW - 1) / RPW;

  // LayerNorm / RMSNorm folded through the product instead of applied to the input first:
  //   sum_k W[r,k] * (((x_k - mu) * rstd) * g_k + b_k) = rstd * (sum_k W[r,k] (g_k x_k) - mu * S_r) + C_r
  // with S_r = sum_k W[r,k] g_k and C_r = sum_k W[r,k] b_k (+ bias) precomputed per matrix.  The
  // statistics mu, rstd are then needed only by the epilogue, so their reductions overlap the weight
  // stream instead of preceding it.  RMSNorm has no mu / beta term and needs no precomputation.
  const bool folded = (a.pro == CTHIP_PRO_RMSNORM) || (a.pro == CTHIP_PRO_LAYERNORM && a.fold_s != nullptr);
  const bool coop = a.stage_x != 0;  // input staged (and normalised, unless folded) once per workgroup
  // Every request is unconditional (a row past the end repeats the last row and is never stored, a chunk past the
  // end of a row reads the zero block, an absent epilogue operand reads the zero block): a load behind a branch
  // leaves a copy of its result at the end of that branch, and the wavefront would wait there for the whole tile
  // before it has even requested its input vector -- two memory round trips in a launch that is nothing but latency.
  auto load = [&](int rq, uint4 *w, unsigned *s, float &bias, float &resid, float &fs) {
    int row = rq * RPW + g;
    row = row < a.rows ? row : a.rows - 1;
    const float *zf = (const float *)g_gemv_zeros;
    bias = *(a.bias ? a.bias + row : zf);
    resid = *(a.residual ? a.residual + (int64_t)m * a.y_stride + row : zf);
    fs = *(a.fold_s ? a.fold_s + row : zf);
#pragma unroll
    for (int j = 0; j < KC; j++) {
      const int c = l + G * j;
      const bool ok = c < nchunks;
      w[j] = load_chunk<NT>(ok ? qp + (int64_t)row * row_chunks + c : (const uint4 *)g_gemv_zeros);
      if (QUANT) {
        const int sidx = (TYPE == CTHIP_Q8_0) ? (c >> 1) : c;
        s[j] = *(ok ? a.d + (int64_t)row * scales_per_row + sidx : (const unsigned short *)g_gemv_zeros);
      }
    }
  };

  if constexpr (PD > 1) {
    gemv_ring<TYPE, G, KC, PD, NT, EPI, DIRECT, PAIR1>(a, xs_lds, red);
    return;
  }
  // Everything this wavefront needs from memory is requested before any arithmetic so the
  // latencies overlap: position, the first weight tiles, then the input vector.
  const int posv = a.pos ? a.pos[0] : 0;
  uint4 wt[PD][KC];
  // (one 32-bit register per scale: 16-bit elements would be packed in pairs right behind their loads, and that
  // use would make the wavefront wait for the tile before it has requested anything else)
  unsigned st[PD][KC];
  float bias_t[PD], resid_t[PD], fs_t[PD];
#pragma unroll
  for (int p = 0; p < PD; p++) {
    const int rq = wave + p * total_waves;
    load(rq < nrq ? rq : nrq - 1, wt[p], st[p], bias_t[p], resid_t[p], fs_t[p]);
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
          const float scale = QUANT ? half_bits_to_float((unsigned short)st[p][j]) : 1.0f;
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

// ------------------------------------------------------------------ dispatch
typedef void (*gemv_fn)(GemvArgs);
struct GemvVariant {
  int type, G, KC;
  gemv_fn fn[2];       // looping launches: [0] cached weights, [1] streamed (non-temporal) weights
  gemv_fn fn_epi[2];   // the same with per-row epilogue operands (bias, residual, fold term) travelling in the ring
  gemv_fn fn_direct[2];  // looping, no epilogue operands, a LayerNorm applied to the staged input
  gemv_fn fn_small[2]; // one tile per wavefront: latency-bound launches
  gemv_fn fn_pair[2];  // looping, one row per wavefront, (gate, up) row pairs in neighbouring ring slots with SwiGLU as the epilogue; null where the shape has none
};
template <int T, int G, int KC, bool NT>
constexpr gemv_fn gemv_pair_fn() {
  if constexpr (G == 64 && PD_OF_T(T, KC) >= 2 && PD_OF_T(T, KC) % 2 == 0) return k_gemv<T, G, KC, PD_OF_T(T, KC), NT, false, false, true>;
  else return nullptr;
}
#define V(T, G, KC)                                                                           \
  {T, G, KC, {k_gemv<T, G, KC, PD_OF_T(T, KC), false>, k_gemv<T, G, KC, PD_OF_T(T, KC), true>},         \
   {k_gemv<T, G, KC, PD_OF_T(T, KC), false, PD_OF_T(T, KC) != 1>, k_gemv<T, G, KC, PD_OF_T(T, KC), true, PD_OF_T(T, KC) != 1>}, \
   {k_gemv<T, G, KC, PD_OF_T(T, KC), false, false, PD_OF_T(T, KC) != 1>, k_gemv<T, G, KC, PD_OF_T(T, KC), true, false, PD_OF_T(T, KC) != 1>}, \
   {k_gemv<T, G, KC, 1, false>, k_gemv<T, G, KC, 1, true>},                                              \
   {gemv_pair_fn<T, G, KC, false>(), gemv_pair_fn<T, G, KC, true>()}},
// defined in gemv_q8.hip, gemv_q4.hip, gemv_f32.hip, gemv_f16.hip
extern const GemvVariant kGemvQ8[], kGemvQ4[], kGemvF32[], kGemvF16[];
extern const int kGemvQ8Count, kGemvQ4Count, kGemvF32Count, kGemvF16Count;

}  // namespace cthip
