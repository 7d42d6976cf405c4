// Three launches per layer for one decode row of an RMSNorm / RoPE / grouped-query / SwiGLU Transformer with
// Q4_0 weights (the Llama family; layers of the shape of external/llm/layers.lisp:35-71 with the pieces of
// nn/positional-encoding.lisp and nn/normalization.lisp swapped in), the counterpart of decode_fused.hip:
//
//   k_gqa_qkv        x -> RMSNorm -> wq|wk|wv: q and the new key rotated (RoPE) in the epilogue, q to a buffer,
//                    k / v rows into the cache at `pos`
//   k_gqa_attn_proj  `replicas` workgroups per query head: attention over cache rows 0..pos of the head's
//                    key/value group, then a share of the rows of the head's 64 columns of wo, added into the
//                    accumulator of the XCD the workgroup runs on
//   k_gqa_mlp        one workgroup per 32 hidden units: RMSNorm -> their gate and up rows -> SwiGLU -> their 32
//                    columns (one Q4_0 block per row) of the down projection, added into a second accumulator set
//
// With 32 query heads and 176 column slabs there are too many partial vectors to hand over one by one, so both
// "column" Linears add 64-bit fixed-point values (2^-32) into one accumulator per XCD (see decode_fused.hip for
// why those atomics stay inside an XCD's L2 and why the sum does not depend on arrival order).  The set the
// attention launch adds into is cleared by the next layer's qkv launch, the set the MLP launch adds into by the
// attention launch: in both cases the last reader has finished and the next writer has not started.
//
// A row of D = 2048 * KC columns is 64 * KC blocks of 32 (KC = 1 is what is built): lane l of a wavefront owns blocks l + 64 j of every
// row the wavefront handles, so the 32 input floats of a block are read from LDS once and multiply several rows.
// The staged vector is stored with the 16-byte slot index xor-ed by the block index: lanes read whole blocks
// (128 bytes apart), which would otherwise all fall on the same LDS banks.
#include <stdlib.h>

#include <type_traits>

#include "common.h"
#include "gemv_kernels.h"
#include "decode_fused.h"

namespace cthip {

__device__ __forceinline__ int swz(int i4) {  // float4 slot of the i4-th float4 of the staged vector
  const int blk = i4 >> 3;
  return (blk << 3) | ((i4 ^ blk) & 7);
}

// The registers a launch's input vector is requested into: x = base (+ the kDecXcds fixed-point accumulators when
// ACC).  NV float4 per thread: D == 1024 * NV, blockDim.x == 256.
template <int NV, bool ACC>
struct GqaStageRegs {
  float4 v[NV], g[NV];
  longlong2 lo[ACC ? NV : 1][kDecXcds], hi[ACC ? NV : 1][kDecXcds];
};

// Requests only.  A launch issues these FIRST, then its weight requests, then fences the scheduler: answers come
// back in request order, so the vector can be staged while the weights are still arriving, and nothing that
// uses an answer (the compiler would otherwise start adding accumulators early, to save registers) is moved in
// front of a later request.
template <int NT, int NV, bool ACC>
__device__ __forceinline__ void gqa_stage_request(const GqaStage &s, GqaStageRegs<NV, ACC> &r) {
  const int tid = threadIdx.x;
#pragma unroll
  for (int k = 0; k < NV; k++) {
    r.v[k] = ((const float4 *)s.base)[tid + NT * k];
    r.g[k] = ((const float4 *)s.gamma)[tid + NT * k];
  }
  if (ACC) {
#pragma unroll
    for (int k = 0; k < NV; k++)
#pragma unroll
      for (int x = 0; x < kDecXcds; x++) {
        const longlong2 *src = (const longlong2 *)(s.iparts + (int64_t)x * s.D) + 2 * (tid + NT * k);
        r.lo[k][x] = src[0];
        r.hi[k][x] = src[1];
      }
  }
}

// gamma * x to LDS (swizzled), 1 / rms(x) returned; block 0 stores x to s.xout.  red holds NT / 64 floats.
template <int NT, int NV, bool ACC>
__device__ __forceinline__ float gqa_stage_finish(const GqaStage &s, GqaStageRegs<NV, ACC> &r, float *xs, float *red) {
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  if (ACC) {
#pragma unroll
    for (int k = 0; k < NV; k++) {
      long long t0 = 0, t1 = 0, t2 = 0, t3 = 0;
#pragma unroll
      for (int x = 0; x < kDecXcds; x++) {
        t0 += r.lo[k][x].x;
        t1 += r.lo[k][x].y;
        t2 += r.hi[k][x].x;
        t3 += r.hi[k][x].y;
      }
      r.v[k] = f4add(r.v[k], make_float4(from_fix(t0), from_fix(t1),
                                         from_fix(t2), from_fix(t3)));
    }
  }
  float ss = 0.0f;
#pragma unroll
  for (int k = 0; k < NV; k++) {
    const float4 v = r.v[k], g = r.g[k];
    ss = fmaf(v.x, v.x, fmaf(v.y, v.y, fmaf(v.z, v.z, fmaf(v.w, v.w, ss))));
    ((float4 *)xs)[swz(tid + NT * k)] = make_float4(v.x * g.x, v.y * g.y, v.z * g.z, v.w * g.w);
    if (blockIdx.x == 0 && s.xout) ((float4 *)s.xout)[tid + NT * k] = v;
  }
  ss = wave_sum(ss);
  if (lane == 0) red[wv] = ss;
  __syncthreads();
  float tot = (red[0] + red[1]) + (red[2] + red[3]);
  if (NT == 512) tot += (red[4] + red[5]) + (red[6] + red[7]);
  return 1.0f / sqrtf(tot / (float)s.D + s.eps);
}

// the 32 floats of block `blk` of a swizzled vector; returns their sum (Q4_0 stores n + 8)
__device__ __forceinline__ float read_block(const float *xs, int blk, float *xr) {
  float part[8];
#pragma unroll
  for (int k = 0; k < 8; k++) {
    const float4 v = ((const float4 *)xs)[(blk << 3) | ((k ^ blk) & 7)];
    xr[4 * k + 0] = v.x;
    xr[4 * k + 1] = v.y;
    xr[4 * k + 2] = v.z;
    xr[4 * k + 3] = v.w;
    part[k] = (v.x + v.y) + (v.z + v.w);
  }
  return ((part[0] + part[1]) + (part[2] + part[3])) + ((part[4] + part[5]) + (part[6] + part[7]));
}

// ---- launch 1: RMSNorm folded through wq|wk|wv; a wavefront produces four consecutive rows ----
// NT threads per workgroup: with 512 every SIMD holds two wavefronts, and a wavefront issues a vector instruction
// every 8 cycles at best whatever its instruction-level parallelism -- the 2.4 instructions per 4-bit weight and
// the accumulator sums of one wavefront per SIMD are what a 256-thread launch spends its time on.
template <int KC, bool ACC, int NT>
__global__ __launch_bounds__(NT) void k_gqa_qkv(GqaQkvArgs a) {
  constexpr int RW = 16 / (NT / 64);  // rows per wavefront
  __shared__ __align__(16) float xs[2048 * KC];
  __shared__ float red[NT / 64];
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int D = a.st.D;
  const int r0 = blockIdx.x * 16 + wv * RW;  // < rows: the launcher requires rows % 16 == 0
  GqaStageRegs<512 * KC / NT, ACC> sr;
  gqa_stage_request<NT>(a.st, sr);
  const int posv = a.pos[0];
  __builtin_amdgcn_sched_barrier(0);
  uint4 w[RW][KC];
  unsigned sc[RW][KC];
#pragma unroll
  for (int u = 0; u < RW; u++)
#pragma unroll
    for (int j = 0; j < KC; j++) {
      const int64_t idx = (int64_t)(r0 + u) * (64 * KC) + lane + 64 * j;
      w[u][j] = ((const uint4 *)a.wq)[idx];
      sc[u][j] = a.wd[idx];
    }
  __builtin_amdgcn_sched_barrier(0);
  if (a.zero) {  // the attention launch's accumulators: read last by the previous layer's MLP launch
    uint4 *z = (uint4 *)a.zero;
    const uint4 zz = make_uint4(0u, 0u, 0u, 0u);
    for (int64_t k = (int64_t)blockIdx.x * NT + tid; k < a.zero_n16; k += (int64_t)gridDim.x * NT) z[k] = zz;
  }
  const float rstd = gqa_stage_finish<NT>(a.st, sr, xs, red);
  float acc[RW];
#pragma unroll
  for (int u = 0; u < RW; u++) acc[u] = 0.0f;
#pragma unroll
  for (int j = 0; j < KC; j++) {
    float xr[32];
    const float xsum = read_block(xs, lane + 64 * j, xr);
#pragma unroll
    for (int u = 0; u < RW; u++) acc[u] += chunk_dot<CTHIP_Q4_0>(w[u][j], half_bits_to_float((unsigned short)sc[u][j]), xr, xsum);
  }
#pragma unroll
  for (int u = 0; u < RW; u++) acc[u] = wave_sum(acc[u]) * rstd;
  if (lane == 0) {
    // the wavefront's RW rows as (part of) a group of four consecutive rows = two rotation pairs
    const int g0 = r0 & ~3;
    const bool second = RW == 2 && (r0 & 2);
    float4 o = RW == 4 ? make_float4(acc[0], acc[1], acc[RW - 2], acc[RW - 1])
                       : (second ? make_float4(0.f, 0.f, acc[0], acc[1]) : make_float4(acc[0], acc[1], 0.f, 0.f));
    float *dst;
    if (g0 < D) {
      o = rope4(o, (g0 % a.DH) >> 2, a.DH, a.log2_base, posv);
      dst = a.q + g0;
    } else if (g0 < D + a.KD) {
      o = rope4(o, ((g0 - D) % a.DH) >> 2, a.DH, a.log2_base, posv);
      dst = a.kc + (int64_t)posv * a.KD + (g0 - D);
    } else {
      dst = a.vc + (int64_t)posv * a.KD + (g0 - D - a.KD);
    }
    if (RW == 4) *(float4 *)dst = o;
    else if (second) *(float2 *)(dst + 2) = make_float2(o.z, o.w);
    else *(float2 *)dst = make_float2(o.x, o.y);
  }
}

// ---- launch 2: attention of one query row per head, then that head's 64 columns of wo ----
// Attention as in k_dec_attn_proj; the key / value rows are those of the head's group.  The head's slab of wo
// (D rows x two Q4_0 blocks) is requested first.  gridDim.y workgroups per head repeat the attention and share
// the slab's rows.
template <int JR, bool ATT_IN>
__global__ __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(4, 4)))
void k_gqa_attn_proj(GqaAttnArgs a) {
  constexpr int DH = 64, LPK = DH / 4, KPW = 64 / LPK, KPT = 4, NW = 16, TILE = NW * KPW * KPT;
  __shared__ float part[NW][DH];
  __shared__ float pm[NW], pl[NW];
  __shared__ __align__(16) float oh[DH];
  const int H = gridDim.x, D = a.D, KD = a.KD;
  const int h = attn_head_of_block(blockIdx.x, H, KD / DH);  // the query heads of a key / value head on one XCD
  const int hk = h / (H / (KD / DH));
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int g = lane / LPK, c = lane % LPK;
  const int rr = D / (int)gridDim.y, rbase = (int)blockIdx.y * rr;
  const int pc = tid & 1, pr0 = tid >> 1;
  uint4 pw[JR];
  unsigned ps[JR];
#pragma unroll
  for (int j = 0; j < JR; j++) {
    int r = pr0 + 512 * j;
    r = rbase + (r < rr ? r : rr - 1);
    const int64_t idx = ((int64_t)h * D + r) * 2 + pc;
    pw[j] = ((const uint4 *)a.pq)[idx];
    ps[j] = a.pd[idx];
  }
  {  // the MLP launch's accumulators: read last by this layer's qkv launch
    uint4 *z = (uint4 *)a.zero;
    const uint4 zz = make_uint4(0u, 0u, 0u, 0u);
    const int64_t nthr = (int64_t)H * gridDim.y * 1024;
    for (int64_t k = ((int64_t)blockIdx.y * H + h) * 1024 + tid; k < a.zero_n16; k += nthr) z[k] = zz;
  }
  if constexpr (ATT_IN) {
    // the head's attention was computed by a launch of its own (long contexts: its keys shared by several workgroups)
    if (tid < DH) oh[tid] = a.att_in[h * DH + tid];
    __syncthreads();
  } else {
    const int T = a.pos[0] + 1;
    const unsigned kvs4 = (unsigned)(KD / 4);
    const float4 q4 = *(const float4 *)(a.q + h * DH + 4 * c);
    const float4 *__restrict__ kp = (const float4 *)(a.kc + hk * DH) + c;
    const float4 *__restrict__ vp = (const float4 *)(a.vc + hk * DH) + c;
    const float scale = 1.0f / sqrtf((float)DH);
    float m = -INFINITY, lsum = 0.0f;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    // one tile = NP key passes per wavefront, all requested together (see k_dec_attn_proj): KPT passes up to
    // 16*KPW*KPT keys, twice as many beyond, so that twice the context still costs one memory round trip
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
        d = row16_sum(d);
        const bool ok = (t0 + (wv * NP + u) * KPW + g) < T;
        sc[u] = ok ? d * scale : -INFINITY;
        tmax = fmaxf(tmax, sc[u]);
      }
      tmax = groups16_max(tmax);  // LPK == 16: one value per group of 16 lanes
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
      psum = groups16_sum(psum);
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
  float xr[32], xsum = 0.0f;
  {
    float p8[8];
#pragma unroll
    for (int t = 0; t < 8; t++) {
      const float4 v = *(const float4 *)(oh + pc * 32 + 4 * t);
      xr[4 * t + 0] = v.x;
      xr[4 * t + 1] = v.y;
      xr[4 * t + 2] = v.z;
      xr[4 * t + 3] = v.w;
      p8[t] = (v.x + v.y) + (v.z + v.w);
    }
    xsum = ((p8[0] + p8[1]) + (p8[2] + p8[3])) + ((p8[4] + p8[5]) + (p8[6] + p8[7]));
  }
  long long *accum = a.accum + (int64_t)xcd_id() * D;
#pragma unroll
  for (int j = 0; j < JR; j++) {
    float s = chunk_dot<CTHIP_Q4_0>(pw[j], half_bits_to_float((unsigned short)ps[j]), xr, xsum);
    s += dpp_f<0xB1>(s);  // the row's other block
    const int r = pr0 + 512 * j;
    if (pc == 0 && r < rr)
      __hip_atomic_fetch_add(accum + rbase + r, to_fix(s), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  }
}

// ---- launch 3: RMSNorm folded through 32 gate and 32 up rows, SwiGLU, one Q4_0 block per row of `down` ----
template <int KC, int NT>
__global__ __launch_bounds__(NT) void k_gqa_mlp(GqaMlpArgs a) {
  constexpr int RW = 32 / (NT / 64);    // gate rows (and up rows) per wavefront
  constexpr int PJ = 2048 * KC / NT;    // rows of the down projection per thread
  __shared__ __align__(16) float xs[2048 * KC];
  __shared__ float red[NT / 64];
  __shared__ __align__(16) float hs[32];
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int D = a.st.D;
  const int slab = blockIdx.x;
  GqaStageRegs<512 * KC / NT, true> sr;
  gqa_stage_request<NT>(a.st, sr);
  __builtin_amdgcn_sched_barrier(0);
  uint4 wg[RW][KC], wu[RW][KC];
  unsigned sg[RW][KC], su[RW][KC];
#pragma unroll
  for (int u = 0; u < RW; u++) {
    const int64_t gr = (int64_t)(slab * 32 + wv * RW + u) * a.gate_stride, ur = gr + a.up_off;
#pragma unroll
    for (int j = 0; j < KC; j++) {
      const int64_t gi = gr * (64 * KC) + lane + 64 * j, ui = ur * (64 * KC) + lane + 64 * j;
      wg[u][j] = ((const uint4 *)a.wq)[gi];
      wu[u][j] = ((const uint4 *)a.wq)[ui];
      sg[u][j] = a.wd[gi];
      su[u][j] = a.wd[ui];
    }
  }
  // this slab's block of every row of the down projection: row r = tid + NT j (D = 2048 * KC)
  uint4 pw[PJ];
  unsigned ps[PJ];
#pragma unroll
  for (int j = 0; j < PJ; j++) {
    const int64_t idx = (int64_t)slab * D + tid + NT * j;
    pw[j] = ((const uint4 *)a.pq)[idx];
    ps[j] = a.pd[idx];
  }
  __builtin_amdgcn_sched_barrier(0);
  const float rstd = gqa_stage_finish<NT>(a.st, sr, xs, red);
  float ag[RW], au[RW];
#pragma unroll
  for (int u = 0; u < RW; u++) ag[u] = au[u] = 0.0f;
#pragma unroll
  for (int j = 0; j < KC; j++) {
    float xr[32];
    const float xsum = read_block(xs, lane + 64 * j, xr);
#pragma unroll
    for (int u = 0; u < RW; u++) {
      ag[u] += chunk_dot<CTHIP_Q4_0>(wg[u][j], half_bits_to_float((unsigned short)sg[u][j]), xr, xsum);
      au[u] += chunk_dot<CTHIP_Q4_0>(wu[u][j], half_bits_to_float((unsigned short)su[u][j]), xr, xsum);
    }
  }
#pragma unroll
  for (int u = 0; u < RW; u++) {
    ag[u] = wave_sum(ag[u]);
    au[u] = wave_sum(au[u]);
  }
  if (lane == 0) {
#pragma unroll
    for (int u = 0; u < RW; u++) hs[wv * RW + u] = ct_silu(rstd * ag[u]) * (rstd * au[u]);
  }
  __syncthreads();
  float hr[32], hsum;
  {
    float p8[8];
#pragma unroll
    for (int t = 0; t < 8; t++) {
      const float4 v = *(const float4 *)(hs + 4 * t);
      hr[4 * t + 0] = v.x;
      hr[4 * t + 1] = v.y;
      hr[4 * t + 2] = v.z;
      hr[4 * t + 3] = v.w;
      p8[t] = (v.x + v.y) + (v.z + v.w);
    }
    hsum = ((p8[0] + p8[1]) + (p8[2] + p8[3])) + ((p8[4] + p8[5]) + (p8[6] + p8[7]));
  }
  long long *accum = a.accum + (int64_t)xcd_id() * D;
#pragma unroll
  for (int j = 0; j < PJ; j++) {
    const float s = chunk_dot<CTHIP_Q4_0>(pw[j], half_bits_to_float((unsigned short)ps[j]), hr, hsum);
    __hip_atomic_fetch_add(accum + tid + NT * j, to_fix(s), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  }
}

// ---- re-layout at load: column group g of every row made contiguous ----
// in: q[r][cpr] 16-byte blocks, d[r][cpr] scales;  out: pq[g][r][cpg], pd[g][r][cpg]   (cpr = groups * cpg)
__global__ void k_gqa_relay(const uint4 *__restrict__ q, const unsigned short *__restrict__ d, uint4 *__restrict__ pq,
                            unsigned short *__restrict__ pd, int rows, int cpr, int cpg) {
  const int64_t n = (int64_t)rows * cpr;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int cc = (int)(i % cpg);
  const int64_t gr = i / cpg;
  const int r = (int)(gr % rows), g = (int)(gr / rows);
  const int64_t src = (int64_t)r * cpr + (int64_t)g * cpg + cc;
  pq[i] = q[src];
  pd[i] = d[src];
}

// ------------------------------------------------------------------ host side
bool gqa_fused_supported(int type_attn, int type_proj, int type_fc, int type_fc2, int D, int H, int HKV, int F) {
  if (type_attn != CTHIP_Q4_0 || type_proj != CTHIP_Q4_0 || type_fc != CTHIP_Q4_0 || type_fc2 != CTHIP_Q4_0) return false;
  if (D != 2048) return false;  // one Q4_0 block per lane and row
  if (H <= 0 || D % H || D / H != 64) return false;
  if (HKV <= 0 || H % HKV) return false;
  if (F <= 0 || F % 32) return false;
  return true;
}

static int relay(const WMat *w, int cpg, void **pq, void **pd) {
  if (w->type != CTHIP_Q4_0 || w->cols % 32 || cpg < 1 || (w->cols / 32) % cpg)
    return fail(CTHIP_E_BAD_ARG, "decoder: cannot re-lay a %lld x %lld matrix of type %d by groups of %d blocks",
                (long long)w->rows, (long long)w->cols, w->type, cpg);
  const int64_t n = w->rows * (w->cols / 32);
  int rc;
  if ((rc = cthip_alloc(pq, (size_t)n * 16))) return rc;
  if ((rc = cthip_alloc(pd, (size_t)n * 2))) return rc;
  hipLaunchKernelGGL(k_gqa_relay, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, state().stream, (const uint4 *)w->q,
                     (const unsigned short *)w->d, (uint4 *)*pq, (unsigned short *)*pd, (int)w->rows, (int)(w->cols / 32), cpg);
  CTHIP_LAUNCH_CHECK();
  return 0;
}

int gqa_relay_groups(const WMat *w, int group_cols, void **pq, void **pd) { return relay(w, group_cols / 32, pq, pd); }
int gqa_relay_slabs(const WMat *w, void **pq, void **pd) { return relay(w, 1, pq, pd); }

int launch_gqa_qkv(const GqaQkvArgs &a, bool from_accum) {
  const int D = a.st.D;
  if (D != 2048 || a.rows % 16 || a.rows != D + 2 * a.KD || a.DH != 64 || a.KD % 64)
    return fail(CTHIP_E_BAD_ARG, "decoder: fused grouped-query qkv launch with D = %d, rows = %d, KD = %d", D, a.rows, a.KD);
  dim3 grid(a.rows / 16), block(512);
  hipStream_t st = state().stream;
  if (from_accum) hipLaunchKernelGGL((k_gqa_qkv<1, true, 512>), grid, block, 0, st, a);
  else hipLaunchKernelGGL((k_gqa_qkv<1, false, 512>), grid, block, 0, st, a);
  CTHIP_LAUNCH_CHECK();
  return 0;
}

int launch_gqa_attn_proj(const GqaAttnArgs &a, int H, int HKV, int replicas) {
  const int D = a.D;
  if (D != H * 64 || a.KD != HKV * 64 || HKV < 1 || H % HKV || replicas < 1 || D % replicas || D / replicas > 2048)
    return fail(CTHIP_E_BAD_ARG, "decoder: fused grouped-query attention launch with D = %d, H = %d, HKV = %d, %d workgroups per head",
                D, H, HKV, replicas);
  dim3 grid(H, replicas), block(1024);
  hipStream_t st = state().stream;
  const int jr = (D / replicas + 511) / 512;
  if (a.att_in) {
    switch (jr) {
      case 1: hipLaunchKernelGGL((k_gqa_attn_proj<1, true>), grid, block, 0, st, a); break;
      case 2: hipLaunchKernelGGL((k_gqa_attn_proj<2, true>), grid, block, 0, st, a); break;
      default: hipLaunchKernelGGL((k_gqa_attn_proj<4, true>), grid, block, 0, st, a); break;
    }
  } else {
    switch (jr) {
      case 1: hipLaunchKernelGGL((k_gqa_attn_proj<1, false>), grid, block, 0, st, a); break;
      case 2: hipLaunchKernelGGL((k_gqa_attn_proj<2, false>), grid, block, 0, st, a); break;
      default: hipLaunchKernelGGL((k_gqa_attn_proj<4, false>), grid, block, 0, st, a); break;
    }
  }
  CTHIP_LAUNCH_CHECK();
  return 0;
}

int launch_gqa_mlp(const GqaMlpArgs &a, int F, int HKV) {
  (void)HKV;
  const int D = a.st.D;
  if (D != 2048 || F % 32) return fail(CTHIP_E_BAD_ARG, "decoder: fused SwiGLU launch with D = %d, F = %d", D, F);
  dim3 grid(F / 32), block(512);
  hipStream_t st = state().stream;
  hipLaunchKernelGGL((k_gqa_mlp<1, 512>), grid, block, 0, st, a);
  CTHIP_LAUNCH_CHECK();
  return 0;
}

}  // namespace cthip
