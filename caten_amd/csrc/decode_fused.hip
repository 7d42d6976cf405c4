// Three launches per layer for one decode row of a GPT-2 shaped Transformer (external/llm/layers.lisp:35-71)
// with Q8_0, Q4_0, fp32 or fp16 weights (template argument TYPE), instead of five.  A decode step is bound by the number of DEPENDENT launches, not by
// bytes, so two pairs of consecutive Linears are merged around the vector that sits between them:
//
//   k_dec_qkv        x -> LayerNorm1 -> c_attn (+bias): q to a buffer, k / v rows into the cache at `pos`
//   k_dec_attn_proj  four workgroups per head: attention over cache rows 0..pos, then a quarter of the rows of
//                    that head's 64 columns of attn.c_proj applied to its 64 outputs -> one partial vector per head
//   k_dec_mlp        one workgroup per 16 hidden units (32 with Q4_0 weights, whose blocks are 32 wide): LayerNorm2
//                    -> those rows of c_fc (+bias, GELU) -> their columns of mlp.c_proj -> partial vector, added
//                    into one accumulator per XCD
//
// A Linear whose INPUT is split over workgroups produces one partial output vector per workgroup; the
// consumer of the vector adds the partials while it stages its input, so the residual stream travels as
// "base vector + bias + partials" and is materialised by whoever reads it next:
//   * attention: H partial vectors of fp32, plain stores (Patt);
//   * MLP: F/16 workgroups would be too many partials to re-read, so each workgroup adds its vector into the
//     accumulator of the XCD it runs on (Pmlp[xcd][D]).  Atomics that carry no device-scope bits execute in
//     the L2 of the issuing XCD, which all its compute units share, and an accumulator is only ever touched
//     from its own XCD, so no traffic crosses the fabric; the lines are written back at the end of the
//     kernel like any other store.  The accumulators are 64-bit fixed point (2^-32): integer addition is
//     associative, so the sum does not depend on the order the workgroups arrive in.
// Weights of the two "column" Linears are re-laid at load so that a workgroup's share is contiguous.
#include <stdlib.h>

#include <type_traits>

#include "common.h"
#include "gemv_kernels.h"
#define CTHIP_DECODE_DEVICE_HELPERS
#include "decode_fused.h"

namespace cthip {

// The registers a launch's input vector  x = base + bias + sum(partials)  is requested into (one float4 per thread,
// D <= 1024).  MODE 0: base only; 1: + bias + NP fp32 partial vectors; 2: + bias + NP fixed-point accumulators.
template <int MODE, int NP>
struct DecStageRegs {
  float4 v, g, b;
  float4 p[MODE == 1 ? NP : 1];
  longlong2 lo[MODE == 2 ? NP : 1], hi[MODE == 2 ? NP : 1];
  int i;
  bool active;
};

// Requests only, every one unconditional.  A launch issues these FIRST, then its weight requests, then fences the
// scheduler: answers come back in request order, so the vector is staged while the weights are still arriving,
// and no use of an answer (the compiler likes to start adding partials early, to save registers) ends up in
// front of a later request, where it would hold that request back by a memory round trip.
template <int MODE, int NP>
__device__ __forceinline__ void dec_stage_request(const DecStage &s, DecStageRegs<MODE, NP> &r) {
  const int tid = threadIdx.x;
  const int n4 = s.D >> 2;
  r.active = tid < n4;
  const int i = r.active ? tid : n4 - 1;
  r.i = i;
  r.v = ((const float4 *)s.base)[i];
  r.g = ((const float4 *)s.gamma)[i];
  if (MODE != 0) r.b = ((const float4 *)s.bias)[i];
  if (MODE == 1) {
#pragma unroll
    for (int k = 0; k < NP; k++) r.p[k] = ((const float4 *)(s.fparts + (int64_t)k * s.D))[i];
  }
  if (MODE == 2) {
#pragma unroll
    for (int k = 0; k < NP; k++) {
      const longlong2 *src = (const longlong2 *)(s.iparts + (int64_t)k * s.D) + 2 * i;
      r.lo[k] = src[0];
      r.hi[k] = src[1];
    }
  }
}

// Adds the answers up, writes gamma * x to LDS and returns the LayerNorm statistics of x; block 0 also stores x to
// s.xout.  red holds 24 floats.  blockDim.x == 256.
template <bool SWZ, int MODE, int NP>
__device__ __forceinline__ void dec_stage_finish(const DecStage &s, DecStageRegs<MODE, NP> &r, float *xs, float *red,
                                                 float &mu, float &rstd) {
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const bool active = r.active;
  const int i = r.i;
  float4 v = r.v;
  const float4 g = r.g;
  if (MODE == 1) {
    v = f4add(v, r.b);
#pragma unroll
    for (int k = 0; k < NP; k++) v = f4add(v, r.p[k]);
  }
  if (MODE == 2) {
    long long t0 = 0, t1 = 0, t2 = 0, t3 = 0;
#pragma unroll
    for (int k = 0; k < NP; k++) {
      t0 += r.lo[k].x;
      t1 += r.lo[k].y;
      t2 += r.hi[k].x;
      t3 += r.hi[k].y;
    }
    v = f4add(v, r.b);
    v = f4add(v, make_float4(from_fix(t0), from_fix(t1), from_fix(t2),
                             from_fix(t3)));
  }
  // (count, mean, squared deviation) per thread, merged exactly: thread -> wavefront by lane reductions,
  // wavefront -> workgroup through LDS behind the one barrier that also publishes the staged vector
  const float cnt = active ? 4.0f : 0.0f;
  const float mean_t = 0.25f * ((v.x + v.y) + (v.z + v.w));
  const float d0 = v.x - mean_t, d1 = v.y - mean_t, d2 = v.z - mean_t, d3 = v.w - mean_t;
  const float m2_t = active ? fmaf(d0, d0, fmaf(d1, d1, fmaf(d2, d2, d3 * d3))) : 0.0f;
  const float n_w = wave_sum(cnt);
  const float mean_w = wave_sum(cnt * mean_t) / fmaxf(n_w, 1.0f);
  const float dm = mean_t - mean_w;
  const float m2_w = wave_sum(m2_t + cnt * dm * dm);
  if (active) {
    ((float4 *)xs)[dec_slot<SWZ>(i)] = make_float4(v.x * g.x, v.y * g.y, v.z * g.z, v.w * g.w);
    if (blockIdx.x == 0 && s.xout) ((float4 *)s.xout)[i] = v;
  }
  if (lane == 0) {
    red[wv] = n_w;
    red[8 + wv] = mean_w;
    red[16 + wv] = m2_w;
  }
  __syncthreads();
  const float inv_n = 1.0f / (float)s.D;
  float sum = 0.0f;
#pragma unroll
  for (int w = 0; w < 4; w++) sum += red[w] * red[8 + w];
  mu = sum * inv_n;
  float m2 = 0.0f;
#pragma unroll
  for (int w = 0; w < 4; w++) {
    const float dw = red[8 + w] - mu;
    m2 += red[16 + w] + red[w] * dw * dw;
  }
  rstd = 1.0f / sqrtf(fmaxf(m2 * inv_n, 0.0f) + s.eps);
}

// ---- launch 1: LayerNorm1 folded through c_attn; 16 rows per workgroup (32 with 8 lanes a row) ----
template <int TYPE, int KC, int MODE, int NP>
__global__ __launch_bounds__(256) void k_dec_qkv(DecQkvArgs a) {
  typedef DecFmt<TYPE> F;
  __shared__ __align__(16) float xs[256 * KC];
  __shared__ float red[24];
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int g = lane / F::LPR, l = lane % F::LPR;
  const int D = a.st.D;
  int row = blockIdx.x * (4 * F::RPW) + wv * F::RPW + g;
  const bool row_ok = row < a.rows;
  row = row_ok ? row : a.rows - 1;
  DecStageRegs<MODE, NP> sr;
  dec_stage_request(a.st, sr);
  const int posv = a.pos[0];
  __builtin_amdgcn_sched_barrier(0);
  constexpr int NCL = KC * 256 / F::XPC / F::LPR;
  uint4 w[NCL];
  unsigned sc[NCL];
  dec_row_request<TYPE, KC>(a.wq, a.wd, row, l, w, sc);
  const float fs = a.fold_s[row], fc = a.fold_c[row];
  __builtin_amdgcn_sched_barrier(0);
  float mu, rstd;
  dec_stage_finish<F::SWZ>(a.st, sr, xs, red, mu, rstd);
  const float acc = dec_row_dot<TYPE, KC>(w, sc, xs, l);
  if (l == 0 && row_ok) {
    // rstd * (W.(gamma x) - mu * W.gamma) + (W.beta + bias)  =  W.LayerNorm(x) + bias
    const float v = rstd * (acc - mu * fs) + fc;
    if (row < D) a.q[row] = v;
    else if (row < 2 * D) a.kc[(int64_t)posv * a.kv_stride + (row - D)] = v;
    else a.vc[(int64_t)posv * a.kv_stride + (row - 2 * D)] = v;
  }
}

// ---- launch 2: attention of one query row per head, then that head's columns of attn.c_proj ----
// Attention as in k_attn_cached (rowops.hip): a key row is read by DH/4 lanes as one float4 each, a wavefront
// holds four passes of K and V in registers, per-wavefront online softmax, one meeting in LDS.  The head's
// slab of the projection (D rows x DH columns, contiguous after the re-layout) does not depend on anything
// computed here and is requested first, so it arrives while the keys are being processed.
template <int TYPE, int DH, int JR, bool ATT_IN>
__global__ __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(4, 4)))
void k_dec_attn_proj(DecAttnArgs a) {
  constexpr int LPK = DH / 4, KPW = 64 / LPK, KPT = 4, NW = 16, TILE = NW * KPW * KPT;
  constexpr int XPC = DecFmt<TYPE>::XPC;
  constexpr int CPR = DH / XPC;         // 16-byte chunks of a projection row inside the slab
  constexpr int RPP = 1024 / CPR;       // projection rows per pass of the workgroup
  __shared__ float part[NW][DH];
  __shared__ float pm[NW], pl[NW];
  __shared__ __align__(16) float oh[DH];
  const int h = blockIdx.x, H = gridDim.x, D = H * DH;
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int g = lane / LPK, c = lane % LPK;
  // The projection slab of this head.  gridDim.y workgroups per head repeat the head's attention and share the
  // slab's rows: what one compute unit has to fetch bounds the launch, and the slab is most of it.
  const int rr = D / (int)gridDim.y, rbase = (int)blockIdx.y * rr;  // this workgroup's rows of the slab
  const int pc = tid % CPR, pr0 = tid / CPR;
  uint4 pw[JR];
  unsigned ps[JR];
#pragma unroll
  for (int j = 0; j < JR; j++) {
    int r = pr0 + RPP * j;
    r = rbase + (r < rr ? r : rr - 1);
    pw[j] = ((const uint4 *)a.pq)[((int64_t)h * D + r) * CPR + pc];
    ps[j] = DecFmt<TYPE>::QUANT ? a.pd[((int64_t)h * D + r) * (DH / 32) + ((pc * XPC) >> 5)] : 0;
  }
  // the accumulators of the MLP launch are cleared here: their last reader (this layer's k_dec_qkv) has finished
  auto clear_accumulators = [&]() {
    uint4 *z = (uint4 *)a.zero;
    const uint4 zz = make_uint4(0u, 0u, 0u, 0u);
    const int64_t nthr = (int64_t)H * gridDim.y * 1024;
    for (int64_t k = ((int64_t)blockIdx.y * H + h) * 1024 + tid; k < a.zero_n16; k += nthr) z[k] = zz;
  };
  if constexpr (ATT_IN) {
    clear_accumulators();
    // the head's attention was computed by a launch of its own (long contexts: its keys shared by several workgroups)
    if (tid < DH) oh[tid] = a.att_in[h * DH + tid];
    __syncthreads();
  } else {
    const int T = a.pos[0] + 1;
    const unsigned kvs4 = (unsigned)(D / 4);
    const float4 q4 = *(const float4 *)(a.q + h * DH + 4 * c);
    const float4 *__restrict__ kp = (const float4 *)(a.kc + h * DH) + c;
    const float4 *__restrict__ vp = (const float4 *)(a.vc + h * DH) + c;
    const float scale = 1.0f / sqrtf((float)DH);
    clear_accumulators();
    float m = -INFINITY, lsum = 0.0f;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    // One tile = NP key passes per wavefront, all requested together: wavefront wv owns keys t0 + (wv*NP + u)*KPW + g.
    // Up to 16*KPW*KPT keys that is KPT passes; a longer context takes tiles of twice as many passes, so that
    // positions up to twice as far still cost ONE memory round trip instead of two.
    auto tile = [&](auto np_tag, int t0) {
      constexpr int NP = decltype(np_tag)::value;
      float4 kr[NP], vr[NP];
  #pragma unroll
      for (int u = 0; u < NP; u++) {
        const int j = t0 + (wv * NP + u) * KPW + g;
        const unsigned jj = (unsigned)min(j, T - 1);  // clamped: masked below, never outside the cache
        kr[u] = kp[jj * kvs4];
        vr[u] = vp[jj * kvs4];
      }
      float sc[NP];
      float tmax = -INFINITY;
  #pragma unroll
      for (int u = 0; u < NP; u++) {
        float d = q4.x * kr[u].x;
        d = fmaf(q4.y, kr[u].y, d);
        d = fmaf(q4.z, kr[u].z, d);
        d = fmaf(q4.w, kr[u].w, d);
        // over the key's 16 lanes: data-parallel-primitive adds, no trip through the LDS crossbar
        if (LPK == 16) {
          d = row16_sum(d);
        } else {
  #pragma unroll
          for (int o = LPK / 2; o > 0; o >>= 1) d += __shfl_xor(d, o, 64);
        }
        const bool ok = (t0 + (wv * NP + u) * KPW + g) < T;
        sc[u] = ok ? d * scale : -INFINITY;
        tmax = fmaxf(tmax, sc[u]);
      }
      if (LPK == 16) {
        tmax = groups16_max(tmax);
      } else {
  #pragma unroll
        for (int o = LPK; o < 64; o <<= 1) tmax = fmaxf(tmax, __shfl_xor(tmax, o, 64));
      }
      const float m_new = fmaxf(m, tmax);
      const float corr = ct_exp(m - m_new);
      float psum = 0.0f;
  #pragma unroll
      for (int k2 = 0; k2 < 4; k2++) acc[k2] *= corr;
  #pragma unroll
      for (int u = 0; u < NP; u++) {
        const float p = ct_exp(sc[u] - m_new);
        psum += p;
        acc[0] = fmaf(p, vr[u].x, acc[0]);
        acc[1] = fmaf(p, vr[u].y, acc[1]);
        acc[2] = fmaf(p, vr[u].z, acc[2]);
        acc[3] = fmaf(p, vr[u].w, acc[3]);
      }
      if (LPK == 16) {
        psum = groups16_sum(psum);
      } else {
  #pragma unroll
        for (int o = LPK; o < 64; o <<= 1) psum += __shfl_xor(psum, o, 64);
      }
      lsum = lsum * corr + psum;
      m = m_new;
    };
    if (T <= TILE) {
      if (wv * KPT * KPW < T) tile(std::integral_constant<int, KPT>(), 0);  // (uniform per wavefront)
    } else {
      for (int t0 = 0; t0 < T; t0 += 2 * TILE) {
        if (t0 + wv * 2 * KPT * KPW >= T) break;  // nothing left for this wavefront (uniform)
        tile(std::integral_constant<int, 2 * KPT>(), t0);
      }
    }
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
      pl[wv] = lsum;
    }
    __syncthreads();
    if (tid < DH) {
      float M = pm[0];
  #pragma unroll
      for (int w = 1; w < NW; w++) M = fmaxf(M, pm[w]);
      float o = 0.0f, L = 0.0f;
  #pragma unroll
      for (int w = 0; w < NW; w++) {
        const float e = ct_exp(pm[w] - M);
        o = fmaf(e, part[w][tid], o);
        L = fmaf(e, pl[w], L);
      }
      oh[tid] = o / L;
    }
    __syncthreads();
  }
  // partial projection: row r of the slab times the head's outputs; CPR lanes share a row
  float xr[XPC];
  lds_floats<XPC>(oh + pc * XPC, xr);
  float xsum = 0.0f;
  if (TYPE == CTHIP_Q4_0) {
#pragma unroll
    for (int t = 0; t < XPC; t++) xsum += xr[t];
  }
#pragma unroll
  for (int j = 0; j < JR; j++) {
    float s = chunk_dot<TYPE>(pw[j], DecFmt<TYPE>::QUANT ? half_bits_to_float((unsigned short)ps[j]) : 1.0f, xr, xsum);
    if (CPR >= 2) s += dpp_f<0xB1>(s);    // quad_perm [1,0,3,2]
    if (CPR >= 4) s += dpp_f<0x4E>(s);    // quad_perm [2,3,0,1]
    if (CPR >= 8) s += dpp_f<0x141>(s);   // row_half_mirror
    if (CPR >= 16) s += dpp_f<0x140>(s);  // row_mirror
    const int r = pr0 + RPP * j;
    if (pc == 0 && r < rr) a.part[(int64_t)h * D + rbase + r] = s;
  }
}

// ---- launch 2 over a cache of Q8_0 rows ----
// The attention of k_attn_cached_q8 (kvq.hip) with sixteen wavefronts: a key row of a head is 64 int8 = 4 lanes x 16
// bytes, a wavefront covers 16 keys a pass, the products run on the integers and a block's scale is applied to its
// partial sum.  The step's new row is quantised here as k_kvq_append quantises it (per block of 32: d = absmax / 127
// kept as fp16, q = x / d rounded half away from zero) by the one wavefront that owns key T - 1, after it has
// requested its other keys; it uses the row in that form and, in the head's first workgroup, stores it into the
// planes -- the session's two append launches and its attention launch in one.
template <int TYPE, int JR>
__global__ __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(4, 4)))
void k_dec_attn_proj_q8(DecAttnQ8Args a) {
  constexpr int DH = 64, LPK = DH / 16, KPW = 64 / LPK, KPT = 2, NW = 16, TILE = NW * KPW * KPT;
  constexpr int XPC = DecFmt<TYPE>::XPC;
  constexpr int CPR = DH / XPC, RPP = 1024 / CPR;
  __shared__ float part[NW][DH];
  __shared__ float pm[NW], pl[NW];
  __shared__ __align__(16) float oh[DH];
  const int h = blockIdx.x, H = gridDim.x, D = H * DH, nb = D / 32;
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int g = lane / LPK, c = lane % LPK;
  const int rr = D / (int)gridDim.y, rbase = (int)blockIdx.y * rr;
  const int pc = tid % CPR, pr0 = tid / CPR;
  uint4 pw[JR];
  unsigned ps[JR];
#pragma unroll
  for (int j = 0; j < JR; j++) {
    int r = pr0 + RPP * j;
    r = rbase + (r < rr ? r : rr - 1);
    pw[j] = ((const uint4 *)a.pq)[((int64_t)h * D + r) * CPR + pc];
    ps[j] = DecFmt<TYPE>::QUANT ? a.pd[((int64_t)h * D + r) * (DH / 32) + ((pc * XPC) >> 5)] : 0;
  }
  const int T = a.pos[0] + 1;
  const int col = h * DH + 16 * c;  // first of this lane's 16 elements inside a cache row
  float qr[16];
#pragma unroll
  for (int e = 0; e < 4; e++) {
    const float4 v = *(const float4 *)(a.q + col + 4 * e);
    qr[4 * e] = v.x, qr[4 * e + 1] = v.y, qr[4 * e + 2] = v.z, qr[4 * e + 3] = v.w;
  }
  // this lane's 16 elements of a new row, quantised; lanes c and c ^ 1 share a block of 32
  auto quantise = [&](const float *src, uint4 &qv, unsigned &dv) {
    float x[16];
#pragma unroll
    for (int e = 0; e < 4; e++) {
      const float4 v = *(const float4 *)(src + col + 4 * e);
      x[4 * e] = v.x, x[4 * e + 1] = v.y, x[4 * e + 2] = v.z, x[4 * e + 3] = v.w;
    }
    float amax = 0.0f;
#pragma unroll
    for (int e = 0; e < 16; e++) amax = fmaxf(amax, fabsf(x[e]));
    amax = fmaxf(amax, dpp_f<0xB1>(amax));  // quad_perm [1,0,3,2]: the block's other half
    const float dd = amax / 127.0f;
    const float inv = dd != 0.0f ? 1.0f / dd : 0.0f;
    unsigned w[4] = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int e = 0; e < 16; e++) {
      const float t = x[e] * inv;
      const int r = (int)(t + copysignf(0.5f, t));  // = copysign(floor(|t| + 0.5), t): the conversion truncates
      w[e >> 2] |= ((unsigned)r & 255u) << (8 * (e & 3));
    }
    qv = make_uint4(w[0], w[1], w[2], w[3]);
    dv = __builtin_bit_cast(unsigned short, (_Float16)dd);
  };
  {  // the accumulators of the MLP launch are cleared here: their last reader (this layer's k_dec_qkv) has finished
    uint4 *z = (uint4 *)a.zero;
    const uint4 zz = make_uint4(0u, 0u, 0u, 0u);
    const int64_t nthr = (int64_t)H * gridDim.y * 1024;
    for (int64_t k = ((int64_t)blockIdx.y * H + h) * 1024 + tid; k < a.zero_n16; k += nthr) z[k] = zz;
  }
  const float scale = 1.0f / sqrtf((float)DH);
  float m = -INFINITY, l = 0.0f;
  float acc[16];
#pragma unroll
  for (int e = 0; e < 16; e++) acc[e] = 0.0f;
  auto widen = [](const uint4 w, float *f) {
    const uint32_t dw[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int t = 0; t < 4; t++) {
      const int v = (int)dw[t];
      f[4 * t + 0] = (float)(int)(int8_t)v;
      f[4 * t + 1] = (float)(int)(int8_t)(v >> 8);
      f[4 * t + 2] = (float)(int)(int8_t)(v >> 16);
      f[4 * t + 3] = (float)(v >> 24);
    }
  };
  // One tile = NP key passes per wavefront, all requested together: wavefront wv owns keys t0 + (wv*NP + u)*KPW + g.
  // (tiles of four passes for long contexts, as the fp32 launch has them, do not fit 128 registers here)
  auto tile = [&](auto np_tag, int t0) {
    constexpr int NP = decltype(np_tag)::value;
    uint4 kr[NP], vr[NP];
    unsigned ks[NP], vs[NP];
    const int j0 = t0 + wv * NP * KPW;
#pragma unroll
    for (int u = 0; u < NP; u++) {
      const int j = j0 + u * KPW + g;
      const int jj = min(j, max(T - 2, 0));  // clamped: masked below; row T - 1 is not in the planes yet
      kr[u] = *(const uint4 *)(a.kq + (int64_t)jj * D + col);
      vr[u] = *(const uint4 *)(a.vq + (int64_t)jj * D + col);
      ks[u] = a.kd[(int64_t)jj * nb + (col >> 5)];
      vs[u] = a.vd[(int64_t)jj * nb + (col >> 5)];
    }
    if (T - 1 >= j0 && T - 1 < j0 + NP * KPW) {  // (uniform) this wavefront owns the new row
      uint4 knq, vnq;
      unsigned knd, vnd;
      quantise(a.newkv, knq, knd);
      quantise(a.newkv + D, vnq, vnd);
#pragma unroll
      for (int u = 0; u < NP; u++) {
        if (j0 + u * KPW + g == T - 1) {
          kr[u] = knq, vr[u] = vnq, ks[u] = knd, vs[u] = vnd;
          if (blockIdx.y == 0) {  // the `!assign` into the cache row at pos
            *(uint4 *)(a.kq + (int64_t)(T - 1) * D + col) = knq;
            *(uint4 *)(a.vq + (int64_t)(T - 1) * D + col) = vnq;
            if ((c & 1) == 0) {
              a.kd[(int64_t)(T - 1) * nb + (col >> 5)] = (unsigned short)knd;
              a.vd[(int64_t)(T - 1) * nb + (col >> 5)] = (unsigned short)vnd;
            }
          }
        }
      }
    }
    float sc[NP];
    float tmax = -INFINITY;
#pragma unroll
    for (int u = 0; u < NP; u++) {
      float kf[16];
      widen(kr[u], kf);
      float dsum = 0.0f;
#pragma unroll
      for (int e = 0; e < 16; e++) dsum = fmaf(qr[e], kf[e], dsum);
      dsum *= half_bits_to_float((unsigned short)ks[u]);
      dsum += dpp_f<0xB1>(dsum);  // over the key's four lanes
      dsum += dpp_f<0x4E>(dsum);
      const bool ok = (j0 + u * KPW + g) < T;
      sc[u] = ok ? dsum * scale : -INFINITY;
      tmax = fmaxf(tmax, sc[u]);
    }
    tmax = wave_max(tmax);
    const float m_new = fmaxf(m, tmax);   // finite: this wavefront has at least one key here
    const float corr = ct_exp(m - m_new);  // 0 on its first tile (m = -inf)
    float psum = 0.0f;
#pragma unroll
    for (int e = 0; e < 16; e++) acc[e] *= corr;
#pragma unroll
    for (int u = 0; u < NP; u++) {
      const float p = ct_exp(sc[u] - m_new);  // exp2(-inf) = 0 for masked keys
      psum += p;
      float vf[16];
      widen(vr[u], vf);
      const float pv = p * half_bits_to_float((unsigned short)vs[u]);
#pragma unroll
      for (int e = 0; e < 16; e++) acc[e] = fmaf(pv, vf[e], acc[e]);
    }
    psum = wave_sum(psum) * 0.25f;  // every one of a key's four lanes holds the same p
    l = l * corr + psum;
    m = m_new;
  };
  int nact;  // wavefronts that hold keys
  if (T <= TILE) {
    nact = (T + KPT * KPW - 1) / (KPT * KPW);
    if (wv < nact) tile(std::integral_constant<int, KPT>(), 0);  // (uniform per wavefront)
  } else {
    nact = NW;
    for (int t0 = 0; t0 < T; t0 += TILE) {
      if (t0 + wv * KPT * KPW >= T) break;  // nothing left for this wavefront (uniform)
      tile(std::integral_constant<int, KPT>(), t0);
    }
  }
  if (wv < nact) {
    // the sum over the wavefront's 16 key groups, halving what is exchanged each time: a lane ends with one of its 16
    // columns, number 8 b0 + 4 b1 + 2 b2 + b3 (b = bits of g)
    float r8[8], r4[4], r2[2], r1;
    const bool b0 = g & 1, b1 = g & 2, b2 = g & 4, b3 = g & 8;
#pragma unroll
    for (int i = 0; i < 8; i++) r8[i] = (b0 ? acc[i + 8] : acc[i]) + __shfl_xor(b0 ? acc[i] : acc[i + 8], 4, 64);
#pragma unroll
    for (int i = 0; i < 4; i++) r4[i] = (b1 ? r8[i + 4] : r8[i]) + __shfl_xor(b1 ? r8[i] : r8[i + 4], 8, 64);
#pragma unroll
    for (int i = 0; i < 2; i++) r2[i] = (b2 ? r4[i + 2] : r4[i]) + __shfl_xor(b2 ? r4[i] : r4[i + 2], 16, 64);
    r1 = (b3 ? r2[1] : r2[0]) + __shfl_xor(b3 ? r2[0] : r2[1], 32, 64);
    part[wv][16 * c + 8 * (int)b0 + 4 * (int)b1 + 2 * (int)b2 + (int)b3] = r1;
    if (lane == 0) {
      pm[wv] = m;
      pl[wv] = l;
    }
  }
  __syncthreads();
  if (tid < DH) {
    float M = pm[0];
    for (int w = 1; w < nact; w++) M = fmaxf(M, pm[w]);
    float o = 0.0f, L = 0.0f;
    for (int w = 0; w < nact; w++) {
      const float e = ct_exp(pm[w] - M);
      o = fmaf(e, part[w][tid], o);
      L = fmaf(e, pl[w], L);
    }
    oh[tid] = o / L;
  }
  __syncthreads();
  // partial projection, as in k_dec_attn_proj
  float xr[XPC];
  lds_floats<XPC>(oh + pc * XPC, xr);
  float xsum = 0.0f;
  if (TYPE == CTHIP_Q4_0) {
#pragma unroll
    for (int t = 0; t < XPC; t++) xsum += xr[t];
  }
#pragma unroll
  for (int j = 0; j < JR; j++) {
    float s = chunk_dot<TYPE>(pw[j], DecFmt<TYPE>::QUANT ? half_bits_to_float((unsigned short)ps[j]) : 1.0f, xr, xsum);
    if (CPR >= 2) s += dpp_f<0xB1>(s);    // quad_perm [1,0,3,2]
    if (CPR >= 4) s += dpp_f<0x4E>(s);    // quad_perm [2,3,0,1]
    if (CPR >= 8) s += dpp_f<0x141>(s);   // row_half_mirror
    if (CPR >= 16) s += dpp_f<0x140>(s);  // row_mirror
    const int r = pr0 + RPP * j;
    if (pc == 0 && r < rr) a.part[(int64_t)h * D + rbase + r] = s;
  }
}

// ---- launch 3: LayerNorm2 folded through RPB rows of c_fc, GELU, their RPB columns of mlp.c_proj ----
// RPB = 16 hidden units per workgroup, 32 where a row takes 8 lanes (Q4_0: the slab is then one block per row)
template <int TYPE, int KC, int NP>
__global__ __launch_bounds__(256) void k_dec_mlp(DecMlpArgs a) {
  typedef DecFmt<TYPE> F;
  constexpr int RPB = 4 * F::RPW;
  __shared__ __align__(16) float xs[256 * KC];
  __shared__ float red[24];
  __shared__ __align__(16) float hs[RPB];
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int g = lane / F::LPR, l = lane % F::LPR;
  const int D = a.st.D;
  const int slab = blockIdx.x;
  const int row = slab * RPB + wv * F::RPW + g;  // < F: the launcher requires F % RPB == 0
  DecStageRegs<1, NP> sr;
  dec_stage_request(a.st, sr);
  __builtin_amdgcn_sched_barrier(0);
  constexpr int XPC = F::XPC, NCL = KC * 256 / XPC / F::LPR, SCH = RPB / XPC;
  uint4 w[NCL];
  unsigned sc[NCL];
  dec_row_request<TYPE, KC>(a.wq, a.wd, row, l, w, sc);
  const float fs = a.fold_s[row], fc = a.fold_c[row];
  // this slab's RPB columns (SCH chunks) of the second Linear: row r = tid + 256 j (D = 256 * KC)
  uint4 pw[KC][SCH];
  unsigned ps[KC];
#pragma unroll
  for (int j = 0; j < KC; j++) {
    const int r = tid + 256 * j;
#pragma unroll
    for (int k = 0; k < SCH; k++) pw[j][k] = ((const uint4 *)a.pq)[((int64_t)slab * D + r) * SCH + k];
    // one scale per 32 columns: two slabs of 16 share it, a slab of 32 has its own
    ps[j] = F::QUANT ? a.pd[(int64_t)(RPB == 16 ? slab >> 1 : slab) * D + r] : 0;
  }
  __builtin_amdgcn_sched_barrier(0);
  float mu, rstd;
  dec_stage_finish<F::SWZ>(a.st, sr, xs, red, mu, rstd);
  const float acc = dec_row_dot<TYPE, KC>(w, sc, xs, l);
  if (l == 0) hs[wv * F::RPW + g] = ct_gelu(rstd * (acc - mu * fs) + fc);
  __syncthreads();
  float hr[RPB], hsum = 0.0f;
#pragma unroll
  for (int t = 0; t < RPB / 4; t++) {
    const float4 v = *(const float4 *)(hs + 4 * t);
    hr[4 * t + 0] = v.x;
    hr[4 * t + 1] = v.y;
    hr[4 * t + 2] = v.z;
    hr[4 * t + 3] = v.w;
    if (TYPE == CTHIP_Q4_0) hsum += (v.x + v.y) + (v.z + v.w);
  }
  long long *accum = a.accum + (int64_t)xcd_id() * D;
#pragma unroll
  for (int j = 0; j < KC; j++) {
    float s = 0.0f;
#pragma unroll
    for (int k = 0; k < SCH; k++)
      s += chunk_dot<TYPE>(pw[j][k], F::QUANT ? half_bits_to_float((unsigned short)ps[j]) : 1.0f, hr + XPC * k, hsum);
    // no device-scope bits: the addition happens in this XCD's L2.  (One device-wide accumulator instead of
    // one per XCD costs the 192 workgroups more in contention than the seven arrays cost the reader.)
    __hip_atomic_fetch_add(accum + tid + 256 * j, to_fix(s), __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_WORKGROUP);
  }
}

// the residual stream as one vector: x = base + bias + accumulators (in front of lm_head)
__global__ __launch_bounds__(256) void k_dec_sum(DecStage s, float *out) {
  const int n4 = s.D >> 2;
  for (int i = threadIdx.x; i < n4; i += 256) {
    float4 v = ((const float4 *)s.base)[i];
    if (s.bias) v = f4add(v, ((const float4 *)s.bias)[i]);
    long long t[4] = {0, 0, 0, 0};
#pragma unroll
    for (int k = 0; k < kDecXcds; k++) {
      const longlong2 *src = (const longlong2 *)(s.iparts + (int64_t)k * s.D) + 2 * i;
      const longlong2 lo = src[0], hi = src[1];
      t[0] += lo.x;
      t[1] += lo.y;
      t[2] += hi.x;
      t[3] += hi.y;
    }
    v = f4add(v, make_float4(from_fix(t[0]), from_fix(t[1]), from_fix(t[2]),
                             from_fix(t[3])));
    ((float4 *)out)[i] = v;
  }
}

// ---- re-layout at load ----
// A "column" Linear keeps a copy in which a workgroup's share is contiguous.  In 16-byte chunks: in[r][cpr] ->
// out[g][r][cpg] (group g = head or 16-column slab, cpr = groups * cpg); Q8_0 scales (one per 32 columns):
// ds[r][spr] -> out[g / gps][r][spg] with gps groups sharing a scale (heads: gps = 1, spg = Dh / 32; slabs of 16
// columns: gps = 2, spg = 1).
__global__ void k_relay_chunks(const uint4 *__restrict__ q, uint4 *__restrict__ pq, int rows, int cpr, int cpg) {
  const int64_t n = (int64_t)rows * cpr;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int cc = (int)(i % cpg);
  const int64_t gr = i / cpg;
  const int r = (int)(gr % rows), g = (int)(gr / rows);
  pq[i] = q[(int64_t)r * cpr + (int64_t)g * cpg + cc];
}
__global__ void k_relay_scales(const unsigned short *__restrict__ d, unsigned short *__restrict__ pd, int rows, int spr, int spg) {
  const int64_t n = (int64_t)rows * spr;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int bb = (int)(i % spg);
  const int64_t gr = i / spg;
  const int r = (int)(gr % rows), g = (int)(gr / rows);
  pd[i] = d[(int64_t)r * spr + (int64_t)g * spg + bb];
}

__global__ void k_xcd_probe(int *out) {
  if (threadIdx.x == 0) {
    const int id = (int)__builtin_amdgcn_s_getreg((3 << 11) | (0 << 6) | 20);
    atomicMax(out, id);
  }
}

// The accumulators of the column Linears are updated by DIFFERENT workgroups of an XCD with atomics that carry no
// device-scope bits.  That the additions of all compute units of an XCD meet (in its L2) is a property of the part,
// not a promise of the memory model, so it is checked before a session relies on it: every thread adds a known
// fixed-point value to a cell of its XCD's row that way (acc) and the same value with a device-scope atomic (ref);
// the two arrays must be identical after the kernel.  64 cells per XCD, thousands of workgroups on all compute units.
__global__ __launch_bounds__(256) void k_xcd_atomics_probe(long long *acc, long long *ref) {
  const int x = xcd_id();
  const int cell = x * 64 + (threadIdx.x & 63);
  const long long v = to_fix(0.125f * (float)(1 + (blockIdx.x % 7)) + 0.001f * (float)(threadIdx.x >> 6));
  __hip_atomic_fetch_add(acc + cell, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  __hip_atomic_fetch_add(ref + cell, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ------------------------------------------------------------------ host side
static int type_xpc(int type) { return type == CTHIP_Q8_0 ? 16 : type == CTHIP_Q4_0 ? 32 : type == CTHIP_F16 ? 8 : type == CTHIP_F32 ? 4 : 0; }
// rows of a 256-thread workgroup: 16 lanes a row, 8 where a chunk is a block of 32
static int type_rpb(int type) { return type == CTHIP_Q4_0 ? 32 : 16; }

bool dec_fused_supported(int type_attn, int type_proj, int type_fc, int type_fc2, int D, int H, int F) {
  if (type_attn != type_proj || type_attn != type_fc || type_attn != type_fc2) return false;
  if (type_attn != CTHIP_Q8_0 && type_attn != CTHIP_Q4_0 && type_attn != CTHIP_F32 && type_attn != CTHIP_F16) return false;
  if (D % 256 || D < 256 || D > 1024) return false;
  if (H <= 0 || D % H || D / H != 64) return false;
  if (H != 4 && H != 8 && H != 12 && H != 16) return false;
  if (F % 32 || F <= 0) return false;
  return true;
}

// max_id: the largest XCD id seen; *max_id = -1 when the per-XCD atomics did not add up (see k_xcd_atomics_probe)
int dec_xcd_probe(int *max_id) {
  static int cached = -2;  // the answer is a property of the device: asked once per process
  if (cached != -2) {
    *max_id = cached;
    return 0;
  }
  int *dev = nullptr;
  const size_t cells = (size_t)kDecXcds * 64;
  int rc = cthip_alloc((void **)&dev, 256 + 2 * cells * sizeof(long long));  // zero-filled
  if (rc) return rc;
  long long *acc = (long long *)((char *)dev + 256), *ref = acc + cells;
  hipLaunchKernelGGL(k_xcd_probe, dim3(4096), dim3(64), 0, state().stream, dev);
  hipError_t e = hipGetLastError();
  if (e == hipSuccess) {
    hipLaunchKernelGGL(k_xcd_atomics_probe, dim3(4096), dim3(256), 0, state().stream, acc, ref);
    e = hipGetLastError();
  }
  long long host[2 * kDecXcds * 64];
  if (e == hipSuccess) rc = cthip_d2h(max_id, dev, sizeof(int));
  if (e == hipSuccess && !rc) rc = cthip_d2h(host, acc, sizeof(host));
  cthip_free(dev);
  if (e != hipSuccess) return fail((int)e, "decoder: XCD probe -> %s", hipGetErrorString(e));
  if (rc) return rc;
  long long total = 0;
  for (size_t k = 0; k < cells; k++) {
    if (host[k] != host[cells + k]) *max_id = -1;
    total += host[cells + k] != 0;
  }
  if (total == 0) *max_id = -1;  // nothing was added at all
  cached = *max_id;
  return 0;
}

// group_cols columns per group; scales (Q8_0): groups_per_scale groups share the 32-column block of a scale
static int relay(const WMat *w, int group_cols, void **pq, void **pd) {
  const int xpc = type_xpc(w->type);
  if (!xpc || w->cols % group_cols || group_cols % xpc)
    return fail(CTHIP_E_BAD_ARG, "decoder: cannot re-lay a %lld x %lld matrix of type %d by groups of %d columns",
                (long long)w->rows, (long long)w->cols, w->type, group_cols);
  const int rows = (int)w->rows, cpr = (int)(w->cols / xpc), cpg = group_cols / xpc;
  int rc;
  *pd = nullptr;
  if ((rc = cthip_alloc(pq, (size_t)rows * cpr * 16))) return rc;
  const int64_t n = (int64_t)rows * cpr;
  hipLaunchKernelGGL(k_relay_chunks, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, state().stream, (const uint4 *)w->q,
                     (uint4 *)*pq, rows, cpr, cpg);
  CTHIP_LAUNCH_CHECK();
  if (w->type == CTHIP_Q8_0 || w->type == CTHIP_Q4_0) {
    const int spr = (int)(w->cols / 32), spg = group_cols >= 32 ? group_cols / 32 : 1;
    if ((rc = cthip_alloc(pd, (size_t)rows * spr * 2))) return rc;
    const int64_t ns = (int64_t)rows * spr;
    hipLaunchKernelGGL(k_relay_scales, dim3((unsigned)((ns + 255) / 256)), dim3(256), 0, state().stream,
                       (const unsigned short *)w->d, (unsigned short *)*pd, rows, spr, spg);
    CTHIP_LAUNCH_CHECK();
  }
  return 0;
}

int dec_relay_heads(const WMat *w, int DH, void **pq, void **pd) { return relay(w, DH, pq, pd); }
int dec_relay_slabs(const WMat *w, void **pq, void **pd) { return relay(w, type_rpb(w->type), pq, pd); }

#define DEC_TYPES(GO_T)                 \
  switch (type) {                       \
    case CTHIP_Q8_0: GO_T(CTHIP_Q8_0); break; \
    case CTHIP_Q4_0: GO_T(CTHIP_Q4_0); break; \
    case CTHIP_F32: GO_T(CTHIP_F32); break;   \
    case CTHIP_F16: GO_T(CTHIP_F16); break;   \
    default: return fail(CTHIP_E_BAD_ARG, "decoder: the three-launch layer has no kernels for weight type %d", type); \
  }

int launch_dec_qkv(const DecQkvArgs &a, int type, bool from_accum) {
  const int D = a.st.D, KC = D / 256;
  if (D % 256 || KC < 1 || KC > 4 || a.rows != 3 * D) return fail(CTHIP_E_BAD_ARG, "decoder: fused qkv launch with D = %d, rows = %d", D, a.rows);
  const int rpb = type_rpb(type);
  dim3 grid((a.rows + rpb - 1) / rpb), block(256);
  hipStream_t st = state().stream;
#define GO(T, KC_)                                                                                  \
  case KC_:                                                                                         \
    if (from_accum) hipLaunchKernelGGL((k_dec_qkv<T, KC_, 2, kDecXcds>), grid, block, 0, st, a);    \
    else hipLaunchKernelGGL((k_dec_qkv<T, KC_, 0, 1>), grid, block, 0, st, a);                      \
    break
#define GO_T(T) \
  switch (KC) { \
    GO(T, 1);   \
    GO(T, 2);   \
    GO(T, 3);   \
    GO(T, 4);   \
  }
  DEC_TYPES(GO_T)
#undef GO_T
#undef GO
  CTHIP_LAUNCH_CHECK();
  return 0;
}

int launch_dec_attn_proj(const DecAttnArgs &a, int type, int H, int D, int replicas) {
  const int xpc = type_xpc(type);
  if (D != H * 64 || D > 1024 || replicas < 1 || D % replicas || !xpc)
    return fail(CTHIP_E_BAD_ARG, "decoder: fused attention launch with D = %d, H = %d, %d workgroups per head", D, H, replicas);
  dim3 grid(H, replicas), block(1024);
  hipStream_t st = state().stream;
  // passes over the slab rows: (D / replicas) rows of 64 / xpc chunks over 1024 threads
  const int rpp = 1024 / (64 / xpc), jr = (D / replicas + rpp - 1) / rpp;
  if (jr > 4) return fail(CTHIP_E_BAD_ARG, "decoder: fused attention launch needs %d passes over its slab", jr);
#define GO_T(T)                                                                                     \
  if (a.att_in) {                                                                                   \
    switch (jr) {                                                                                   \
      case 1: hipLaunchKernelGGL((k_dec_attn_proj<T, 64, 1, true>), grid, block, 0, st, a); break;  \
      case 2: hipLaunchKernelGGL((k_dec_attn_proj<T, 64, 2, true>), grid, block, 0, st, a); break;  \
      case 3: hipLaunchKernelGGL((k_dec_attn_proj<T, 64, 3, true>), grid, block, 0, st, a); break;  \
      default: hipLaunchKernelGGL((k_dec_attn_proj<T, 64, 4, true>), grid, block, 0, st, a); break; \
    }                                                                                               \
  } else {                                                                                          \
    switch (jr) {                                                                                   \
      case 1: hipLaunchKernelGGL((k_dec_attn_proj<T, 64, 1, false>), grid, block, 0, st, a); break;  \
      case 2: hipLaunchKernelGGL((k_dec_attn_proj<T, 64, 2, false>), grid, block, 0, st, a); break;  \
      case 3: hipLaunchKernelGGL((k_dec_attn_proj<T, 64, 3, false>), grid, block, 0, st, a); break;  \
      default: hipLaunchKernelGGL((k_dec_attn_proj<T, 64, 4, false>), grid, block, 0, st, a); break; \
    }                                                                                               \
  }
  DEC_TYPES(GO_T)
#undef GO_T
  CTHIP_LAUNCH_CHECK();
  return 0;
}

int launch_dec_attn_proj_q8(const DecAttnQ8Args &a, int type, int H, int D, int replicas) {
  const int xpc = type_xpc(type);
  if (D != H * 64 || D > 1024 || replicas < 1 || D % replicas || !xpc)
    return fail(CTHIP_E_BAD_ARG, "decoder: fused attention launch with D = %d, H = %d, %d workgroups per head", D, H, replicas);
  dim3 grid(H, replicas), block(1024);
  hipStream_t st = state().stream;
  const int rpp = 1024 / (64 / xpc), jr = (D / replicas + rpp - 1) / rpp;
  if (jr > 4) return fail(CTHIP_E_BAD_ARG, "decoder: fused attention launch needs %d passes over its slab", jr);
#define GO_T(T)                                                                                 \
  switch (jr) {                                                                                 \
    case 1: hipLaunchKernelGGL((k_dec_attn_proj_q8<T, 1>), grid, block, 0, st, a); break;       \
    case 2: hipLaunchKernelGGL((k_dec_attn_proj_q8<T, 2>), grid, block, 0, st, a); break;       \
    case 3: hipLaunchKernelGGL((k_dec_attn_proj_q8<T, 3>), grid, block, 0, st, a); break;       \
    default: hipLaunchKernelGGL((k_dec_attn_proj_q8<T, 4>), grid, block, 0, st, a); break;      \
  }
  DEC_TYPES(GO_T)
#undef GO_T
  CTHIP_LAUNCH_CHECK();
  return 0;
}

int launch_dec_mlp(const DecMlpArgs &a, int type, int F, int H) {
  const int D = a.st.D, KC = D / 256;
  if (D % 256 || KC < 1 || KC > 4 || F % 32) return fail(CTHIP_E_BAD_ARG, "decoder: fused MLP launch with D = %d, F = %d", D, F);
  const int rpb = type_rpb(type);
  if (H != 4 && H != 8 && H != 12 && H != 16) return fail(CTHIP_E_BAD_ARG, "decoder: fused MLP launch with %d heads", H);
  dim3 grid(F / rpb), block(256);
  hipStream_t st = state().stream;
#define GO2(T, KC_, NP_) hipLaunchKernelGGL((k_dec_mlp<T, KC_, NP_>), grid, block, 0, st, a)
#define GO(T, KC_)                     \
  case KC_:                            \
    if (H == 4) GO2(T, KC_, 4);        \
    else if (H == 8) GO2(T, KC_, 8);   \
    else if (H == 12) GO2(T, KC_, 12); \
    else GO2(T, KC_, 16);              \
    break
#define GO_T(T) \
  switch (KC) { \
    GO(T, 1);   \
    GO(T, 2);   \
    GO(T, 3);   \
    GO(T, 4);   \
  }
  DEC_TYPES(GO_T)
#undef GO_T
#undef GO
#undef GO2
  CTHIP_LAUNCH_CHECK();
  return 0;
}

int launch_dec_sum(const DecStage &s, float *out) {
  hipLaunchKernelGGL(k_dec_sum, dim3(1), dim3(256), 0, state().stream, s, out);
  CTHIP_LAUNCH_CHECK();
  return 0;
}

}  // namespace cthip
