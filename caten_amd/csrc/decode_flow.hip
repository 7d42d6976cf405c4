// All layers of one decode row of a GPT-2 shaped Transformer (external/llm/layers.lisp:35-71), Q8_0 weights, as ONE
// launch: a dataflow of role-specialised workgroups instead of three dependent launches per layer.
//
// OPT-IN (option "decode_flow"), and slower than the three launches it replaces: 13.8 us per GPT-2-small layer
// against 12.2.  It stays as the measurement of what a decode layer costs once NO launch boundary is left.  Its
// in-kernel timeline (option value 2) shows that handing a vector from one set of workgroups to another through
// memory costs 0.5-0.9 us when every polled line has one reader and 1.1-2.2 us when a hundred workgroups read it
// (copies of the vector for groups of a dozen readers do not change that), and that a compute unit converts and
// multiplies ~32 int8 weights per cycle, so a layer's 7 M weights have to be spread over ~240 compute units (five
// roles, five hand-overs) before no role computes for more than 1.5 us: 5 x (hand-over + compute) = 13.8 us.
//
// A dependent launch costs 1.9 us of graph node plus a first memory round trip (~1.2 us) before its weights and its
// input have arrived; a decode step of 12 layers pays that 36 times.  Here every workgroup owns one role for the
// whole step, stays resident on a compute unit of its own, and hands its output to the next role through device
// memory in which EVERY 8-BYTE ELEMENT CARRIES ITS VALUE AND A TAG (the step's epoch, the layer and the phase): a
// consumer polls the data itself with device-scope loads until the tag is the one it waits for.  No counters, no
// fences, no barrier between workgroups.  A role is idle while the other roles of a layer run, so it requests
// everything that does not depend on its input -- its weights for the next layer, attention's cached K / V rows --
// BEFORE it starts to wait and keeps them in registers (512 threads a workgroup: 256 registers a thread, the register
// file of the compute unit is the prefetch buffer), and no weight latency is left on the critical path.
//
//   Q  (3D/32 workgroups) x -> LayerNorm1 folded -> 32 rows of c_attn each: q, k, v as tagged elements; k / v also
//                         into the cache rows at `pos` for later steps
//   A  (one per head)     the head's q and new k / v row (tagged), cache rows 0..pos-1 (plain loads, requested
//                         ahead); attention -> the head's 64 outputs (tagged)
//   P  (D/32)             32 rows of attn.c_proj each over all heads' outputs: x' = x + bias + W o (tagged)
//   M  (F/32)             x' -> LayerNorm2 folded -> 32 rows of c_fc -> GELU -> their 32 columns of mlp.c_proj -> one
//                         partial vector per workgroup (tagged)
//   R  (32)               D/32 columns each: x'' = x' + bias + the F/32 partial vectors, added in a fixed order ->
//                         the next layer's input (tagged); after the last layer the residual vector for lm_head
//
// Every buffer belongs to one (layer, phase), so nothing is overwritten within a step; tags of earlier steps never
// match (the epoch differs).  Every wait is bounded: a workgroup that runs out of polls raises the session's error
// flag and leaves, the others then run out as well, and the host reports the step as failed -- no hang.  All
// workgroups must be resident at once: the launcher refuses a grid larger than the number of compute units.
#include "common.h"
#include "gemv_kernels.h"
#define CTHIP_DECODE_DEVICE_HELPERS
#include "decode_fused.h"

namespace cthip {

typedef unsigned long long u64;

constexpr int NT = 512;             // threads of a workgroup: two wavefronts per SIMD, 256 registers each
constexpr int kFlowSpin = 1 << 18;  // polls before a waiter gives up (a poll is ~1 us)
constexpr int kFlowNR = 32;
// Copies of the broadcast vectors: every poll of an element is a request to the memory channel that owns its line, and
// a hundred workgroups polling the same 48 lines queue there (and the producer's stores behind them).  Workgroup j of a
// consumer role polls copy j % copies.
constexpr int kRepX = 8, kRepO = 4, kRepXP = 8;
enum { PH_X = 0, PH_QKV = 1, PH_O = 2, PH_XP = 3, PH_PM = 4 };

__device__ __forceinline__ unsigned flow_tag(unsigned epoch, int layer, int phase) { return (epoch << 8) | (unsigned)(layer * 8 + phase); }
__device__ __forceinline__ void ll_store(u64 *p, float v, unsigned tag) {
  __hip_atomic_store(p, (u64)__float_as_uint(v) | ((u64)tag << 32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ u64 ll_load(const u64 *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

// Polls the N elements addr(0) .. addr(N-1) until all of them carry `tag`.  false = gave up (the error flag is raised).
template <int N, class Addr>
__device__ __forceinline__ bool ll_wait(Addr addr, unsigned tag, float *v, int *err) {
  int spins = 0;
  for (;;) {
    u64 w[N];
#pragma unroll
    for (int k = 0; k < N; k++) w[k] = ll_load(addr(k));
    bool ok = true;
#pragma unroll
    for (int k = 0; k < N; k++) ok = ok && (unsigned)(w[k] >> 32) == tag;
    if (ok) {
#pragma unroll
      for (int k = 0; k < N; k++) v[k] = __uint_as_float((unsigned)w[k]);
      return true;
    }
    if (++spins > kFlowSpin || ((spins & 1023) == 0 && __hip_atomic_load(err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))) {
      __hip_atomic_store(err, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      return false;
    }
    __builtin_amdgcn_s_sleep(1);
  }
}

// timeline of a traced step: stamp k of this workgroup at this layer (constant-rate clock, the same on every XCD)
__device__ __forceinline__ void flow_stamp(const FlowArgs &a, int layer, int k) {
  if (a.trace && threadIdx.x == 0) a.trace[((int64_t)blockIdx.x * a.n_layers + layer) * 4 + k] = (long long)wall_clock64();
}

// The residual vector is spread over the workgroup as NE elements per thread: tid and, for D > 512, tid + 512.
template <int KC>
struct FlowVec {
  static constexpr int D = 256 * KC, NE = (D + NT - 1) / NT;
  __device__ static __forceinline__ bool has(int k) { return (int)threadIdx.x + NT * k < D; }
  // an element of the vector for every (thread, k): threads past the end repeat the last one
  __device__ static __forceinline__ int elem(int k) { return has(k) ? (int)threadIdx.x + NT * k : D - 1; }
};

// LayerNorm of the vector: raw x into xr, gamma * x into xs, ONE barrier; every wavefront then works out mean and
// variance for itself from xr (4 * KC values per lane, the same additions in every wavefront, so all of them hold
// the same mu / rstd bit for bit).
template <int KC>
__device__ __forceinline__ void flow_norm_stage(const float *xv, const float *g, float eps, float *xs, float *xr, float &mu, float &rstd) {
  typedef FlowVec<KC> V;
#pragma unroll
  for (int k = 0; k < V::NE; k++)
    if (V::has(k)) {
      xr[threadIdx.x + NT * k] = xv[k];
      xs[threadIdx.x + NT * k] = xv[k] * g[k];
    }
  __syncthreads();
  const int lane = threadIdx.x & 63;
  float4 v[KC];
  float s = 0.0f;
#pragma unroll
  for (int j = 0; j < KC; j++) {
    v[j] = *(const float4 *)(xr + 4 * (lane + 64 * j));
    s += (v[j].x + v[j].y) + (v[j].z + v[j].w);
  }
  mu = wave_sum(s) * (1.0f / (float)V::D);
  float m2 = 0.0f;
#pragma unroll
  for (int j = 0; j < KC; j++) {
    const float a0 = v[j].x - mu, a1 = v[j].y - mu, a2 = v[j].z - mu, a3 = v[j].w - mu;
    m2 += (a0 * a0 + a1 * a1) + (a2 * a2 + a3 * a3);
  }
  rstd = 1.0f / sqrtf(wave_sum(m2) * (1.0f / (float)V::D) + eps);
}

// ------------------------------------------------------------------ role Q
// workgroup j: rows 32 j .. 32 j + 31 of c_attn (16 lanes a row)
template <int KC>
__device__ __forceinline__ void flow_role_q(const FlowArgs &a, int j, float *xs, float *xr) {
  typedef FlowVec<KC> V;
  constexpr int D = V::D, NE = V::NE;
  const int tid0 = threadIdx.x;
  const int posv = a.tokpos[1];
  const unsigned epoch = (unsigned)a.state[0];
  for (int layer = 0; layer < a.n_layers; layer++) {
    const FlowLayer &Ly = a.layers[layer];
    // (indices are derived anew in every layer: what is hoisted out of the loop stays in registers for the whole step)
    int tid = tid0;
    asm volatile("" : "+v"(tid));
    const int rin = tid >> 4, l = tid & 15;
    const int row = j * (NT / 16) + rin;
    uint4 w[KC];
    unsigned sc[KC];
    dec_row_request<CTHIP_Q8_0, KC>(Ly.attn_q, Ly.attn_d, row, l, w, sc);
    const float fs = Ly.attn_s[row], fc = Ly.attn_c[row];
    float gam[NE], xv[NE];
#pragma unroll
    for (int k = 0; k < NE; k++) gam[k] = Ly.ln1_g[V::elem(k)];
    bool ok = true;
    flow_stamp(a, layer, 0);
    if (layer == 0) {
#pragma unroll
      for (int k = 0; k < NE; k++) xv[k] = a.x0[V::elem(k)];
    } else {
      const u64 *base = a.X + ((int64_t)(j % kRepX) * a.n_layers + layer) * D;
      ok = ll_wait<NE>([&](int k) { return base + V::elem(k); }, flow_tag(epoch, layer, PH_X), xv, a.state + 1);
    }
    if (__syncthreads_or(!ok)) return;
    flow_stamp(a, layer, 1);
    float mu, rstd;
    flow_norm_stage<KC>(xv, gam, a.eps, xs, xr, mu, rstd);
    flow_stamp(a, layer, 2);
    const float acc = dec_row_dot<CTHIP_Q8_0, KC>(w, sc, xs, l);
    if (l == 0) {
      const float v = rstd * (acc - mu * fs) + fc;
      ll_store(a.QKV + (int64_t)layer * 3 * D + row, v, flow_tag(epoch, layer, PH_QKV));
      if (row >= 2 * D) Ly.vc[(int64_t)posv * D + (row - 2 * D)] = v;
      else if (row >= D) Ly.kc[(int64_t)posv * D + (row - D)] = v;
    }
    flow_stamp(a, layer, 3);
    __syncthreads();  // xs / xr are rewritten by the next layer
  }
}

// ------------------------------------------------------------------ role A
// head h.  A key row is read by 16 lanes as one float4 each (four keys per wavefront and step), online softmax per
// wavefront over a tile of 256 keys held in registers, one meeting in LDS.
template <int KC>
__device__ __forceinline__ void flow_role_a(const FlowArgs &a, int h, float *smem) {
  constexpr int D = 256 * KC;
  constexpr int DH = 64, LPK = 16, KPW = 4, KPT = 8, NW = NT / 64, TILE = NW * KPW * KPT;
  float(*part)[DH] = (float(*)[DH])smem;  // [NW][DH]
  float *pm = smem + NW * DH, *pl = pm + NW, *qkvs = pl + NW;  // qkvs: 3 * DH
  const int tid0 = threadIdx.x;
  const int T = a.tokpos[1] + 1;
  const unsigned epoch = (unsigned)a.state[0];
  const unsigned kvs4 = (unsigned)(D / 4);
  const float scale = 0.125f;  // 1 / sqrt(64)
  for (int layer = 0; layer < a.n_layers; layer++) {
    const FlowLayer &Ly = a.layers[layer];
    int tid = tid0;
    asm volatile("" : "+v"(tid));
    const int lane = tid & 63, wv = tid >> 6;
    const int g = lane / LPK, c = lane % LPK;
    // the cached rows: requested before the head's q exists
    const float4 *__restrict__ kp = (const float4 *)(Ly.kc + h * DH) + c;
    const float4 *__restrict__ vp = (const float4 *)(Ly.vc + h * DH) + c;
    float4 kr[KPT], vr[KPT];
#pragma unroll
    for (int u = 0; u < KPT; u++) {
      const int jk = (u * NW + wv) * KPW + g;
      const unsigned jj = (unsigned)min(jk, max(T - 2, 0));  // clamped: masked below; row T-1 comes from the Q role
      kr[u] = kp[jj * kvs4];
      vr[u] = vp[jj * kvs4];
    }
    bool ok = true;
    flow_stamp(a, layer, 0);
    if (tid < 3 * DH) {
      const u64 *p = a.QKV + (int64_t)layer * 3 * D + (tid / DH) * D + h * DH + (tid % DH);
      float v;
      ok = ll_wait<1>([&](int) { return p; }, flow_tag(epoch, layer, PH_QKV), &v, a.state + 1);
      qkvs[tid] = v;
    }
    if (__syncthreads_or(!ok)) return;
    flow_stamp(a, layer, 1);
    const float4 q4 = *(const float4 *)(qkvs + 4 * c);
    const float4 kn = *(const float4 *)(qkvs + DH + 4 * c), vn = *(const float4 *)(qkvs + 2 * DH + 4 * c);
    float m = -INFINITY, lsum = 0.0f;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    // keys are dealt round-robin: step u of a tile gives wavefront wv the four keys (u * NW + wv) * 4 + g, so a short
    // context occupies every wavefront and the steps past its end are skipped by all of them
    for (int t0 = 0; t0 < T; t0 += TILE) {
      if (t0 + wv * KPW >= T) break;        // this wavefront has no key in this tile or any later one (uniform)
      if (t0 > 0) {                          // contexts beyond one tile: the next passes, requested here
#pragma unroll
        for (int u = 0; u < KPT; u++) {
          const int jk = t0 + (u * NW + wv) * KPW + g;
          const unsigned jj = (unsigned)min(jk, max(T - 2, 0));
          kr[u] = kp[jj * kvs4];
          vr[u] = vp[jj * kvs4];
        }
      }
      float sk[KPT];
      float tmax = -INFINITY;
#pragma unroll
      for (int u = 0; u < KPT; u++) {
        sk[u] = -INFINITY;
        if (t0 + u * NW * KPW < T) {         // the step has keys for some wavefront (uniform over the workgroup)
          const int jk = t0 + (u * NW + wv) * KPW + g;
          const float4 kk = jk >= T - 1 ? kn : kr[u];
          float d = q4.x * kk.x;
          d = fmaf(q4.y, kk.y, d);
          d = fmaf(q4.z, kk.z, d);
          d = fmaf(q4.w, kk.w, d);
          d = row16_sum(d);  // LPK == 16: the key's lanes are one row of the data-parallel primitives
          sk[u] = jk < T ? d * scale : -INFINITY;
          tmax = fmaxf(tmax, sk[u]);
        }
      }
      tmax = groups16_max(tmax);
      const float m_new = fmaxf(m, tmax);   // finite: key t0 + 4 wv of step 0 exists
      const float corr = ct_exp(m - m_new);  // 0 on its first tile (m = -inf)
      float psum = 0.0f;
#pragma unroll
      for (int k2 = 0; k2 < 4; k2++) acc[k2] *= corr;
#pragma unroll
      for (int u = 0; u < KPT; u++) {
        if (t0 + u * NW * KPW < T) {
          const int jk = t0 + (u * NW + wv) * KPW + g;
          const float4 vv = jk >= T - 1 ? vn : vr[u];
          const float p = ct_exp(sk[u] - m_new);  // exp2(-inf) = 0 for masked keys
          psum += p;
          acc[0] = fmaf(p, vv.x, acc[0]);
          acc[1] = fmaf(p, vv.y, acc[1]);
          acc[2] = fmaf(p, vv.z, acc[2]);
          acc[3] = fmaf(p, vv.w, acc[3]);
        }
      }
      psum = groups16_sum(psum);
      lsum = lsum * corr + psum;
      m = m_new;
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
    flow_stamp(a, layer, 2);
    if (tid < DH) {
      float M = pm[0];
#pragma unroll
      for (int w2 = 1; w2 < NW; w2++) M = fmaxf(M, pm[w2]);
      float o = 0.0f, L = 0.0f;
#pragma unroll
      for (int w2 = 0; w2 < NW; w2++) {
        const float ee = ct_exp(pm[w2] - M);  // wavefronts without keys hold m = -inf: weight 0
        o = fmaf(ee, part[w2][tid], o);
        L = fmaf(ee, pl[w2], L);
      }
      const float ov = o / L;
#pragma unroll
      for (int rep = 0; rep < kRepO; rep++)
        ll_store(a.O + ((int64_t)rep * a.n_layers + layer) * D + h * DH + tid, ov, flow_tag(epoch, layer, PH_O));
    }
    flow_stamp(a, layer, 3);
    __syncthreads();  // the LDS arrays are rewritten by the next layer
  }
}

// ------------------------------------------------------------------ role P
// workgroup i: rows 32 i .. 32 i + 31 of attn.c_proj over the heads' outputs; x' = x + bias + W o
template <int KC>
__device__ __forceinline__ void flow_role_p(const FlowArgs &a, int i, float *xs) {
  typedef FlowVec<KC> V;
  constexpr int D = V::D, NE = V::NE;
  const int tid0 = threadIdx.x;
  const unsigned epoch = (unsigned)a.state[0];
  for (int layer = 0; layer < a.n_layers; layer++) {
    const FlowLayer &Ly = a.layers[layer];
    int tid = tid0;
    asm volatile("" : "+v"(tid));
    const int rin = tid >> 4, l = tid & 15;
    const int row = i * (NT / 16) + rin;
    uint4 w[KC];
    unsigned sc[KC];
    dec_row_request<CTHIP_Q8_0, KC>(Ly.proj_q, Ly.proj_d, row, l, w, sc);
    const float pb = Ly.proj_b[row];
    // the residual input of this row: complete long before the heads' outputs are
    float xrow;
    bool ok = true;
    flow_stamp(a, layer, 0);
    if (layer == 0) {
      xrow = a.x0[row];
    } else {
      const u64 *px = a.X + ((int64_t)(i % kRepX) * a.n_layers + layer) * D + row;
      ok = ll_wait<1>([&](int) { return px; }, flow_tag(epoch, layer, PH_X), &xrow, a.state + 1);
    }
    float ov[NE];
    {
      const u64 *base = a.O + ((int64_t)(i % kRepO) * a.n_layers + layer) * D;
      ok = ll_wait<NE>([&](int k) { return base + V::elem(k); }, flow_tag(epoch, layer, PH_O), ov, a.state + 1) && ok;
    }
    if (__syncthreads_or(!ok)) return;
    flow_stamp(a, layer, 1);
#pragma unroll
    for (int k = 0; k < NE; k++)
      if (V::has(k)) xs[tid + NT * k] = ov[k];
    __syncthreads();
    flow_stamp(a, layer, 2);
    const float acc = dec_row_dot<CTHIP_Q8_0, KC>(w, sc, xs, l);
    if (l == 0) {
      const float xpv = xrow + pb + acc;
#pragma unroll
      for (int rep = 0; rep < kRepXP; rep++)
        ll_store(a.XP + ((int64_t)rep * a.n_layers + layer) * D + row, xpv, flow_tag(epoch, layer, PH_XP));
    }
    flow_stamp(a, layer, 3);
    __syncthreads();  // xs is rewritten by the next layer
  }
}

// ------------------------------------------------------------------ role M
// workgroup w: hidden units 32 w .. 32 w + 31: their rows of c_fc, GELU, their 32 columns of mlp.c_proj
template <int KC>
__device__ __forceinline__ void flow_role_m(const FlowArgs &a, int w, float *xs, float *xr, float *hs) {
  typedef FlowVec<KC> V;
  constexpr int D = V::D, NE = V::NE;
  constexpr int SJ = D * 2 / NT;              // passes over the slab of mlp.c_proj: D rows x 2 chunks
  const int tid0 = threadIdx.x;
  const unsigned epoch = (unsigned)a.state[0];
  for (int layer = 0; layer < a.n_layers; layer++) {
    const FlowLayer &Ly = a.layers[layer];
    int tid = tid0;
    asm volatile("" : "+v"(tid));
    const int rin = tid >> 4, l = tid & 15;
    const int row = w * (NT / 16) + rin;
    uint4 wq[KC];
    unsigned sc[KC];
    dec_row_request<CTHIP_Q8_0, KC>(Ly.fc_q, Ly.fc_d, row, l, wq, sc);
    const float fs = Ly.fc_s[row], fc = Ly.fc_c[row];
    // thread t takes chunks t + 512 j of the slab: row q / 2, columns 16 * (q % 2) ..; one scale per row
    uint4 pw[SJ];
    unsigned ps[SJ];
#pragma unroll
    for (int jj = 0; jj < SJ; jj++) {
      const int q = tid + NT * jj;
      pw[jj] = ((const uint4 *)Ly.fc2_sq)[(int64_t)w * D * 2 + q];
      ps[jj] = Ly.fc2_sd[(int64_t)w * D + (q >> 1)];
    }
    float g[NE], xv[NE];
#pragma unroll
    for (int k = 0; k < NE; k++) g[k] = Ly.ln2_g[V::elem(k)];
    bool ok = true;
    flow_stamp(a, layer, 0);
    {
      const u64 *base = a.XP + ((int64_t)(w % kRepXP) * a.n_layers + layer) * D;
      ok = ll_wait<NE>([&](int k) { return base + V::elem(k); }, flow_tag(epoch, layer, PH_XP), xv, a.state + 1);
    }
    if (__syncthreads_or(!ok)) return;
    flow_stamp(a, layer, 1);
    float mu, rstd;
    flow_norm_stage<KC>(xv, g, a.eps, xs, xr, mu, rstd);
    const float acc = dec_row_dot<CTHIP_Q8_0, KC>(wq, sc, xs, l);
    if (l == 0) hs[rin] = ct_gelu(rstd * (acc - mu * fs) + fc);
    __syncthreads();
    flow_stamp(a, layer, 2);
#pragma unroll
    for (int jj = 0; jj < SJ; jj++) {
      const int q = tid + NT * jj;
      float hr[16];
      lds_floats<16>(hs + 16 * (q & 1), hr);
      float s = chunk_dot<CTHIP_Q8_0>(pw[jj], half_bits_to_float((unsigned short)ps[jj]), hr, 0.0f);
      s += dpp_f<0xB1>(s);  // quad_perm [1,0,3,2]: the row's other chunk
      if ((q & 1) == 0) ll_store(a.PM + ((int64_t)layer * a.NM + w) * D + (q >> 1), s, flow_tag(epoch, layer, PH_PM));
    }
    flow_stamp(a, layer, 3);
    __syncthreads();  // xs / hs are rewritten by the next layer
  }
}

// ------------------------------------------------------------------ role R
constexpr int kFlowRK = 6;  // partial vectors per thread of the R role, at most
__device__ __forceinline__ void flow_role_r(const FlowArgs &a, int i, float *smem) {
  const int tid = threadIdx.x, D = a.D;
  const int cpw = D / kFlowNR;                // columns per workgroup (8 * KC)
  const int G = NT / cpw;                     // groups of threads that share the partial vectors (>= 16)
  const int c = tid % cpw, p0 = tid / cpw;
  const bool live = p0 < G;
  const int col = i * cpw + c;
  const unsigned epoch = (unsigned)a.state[0];
  for (int layer = 0; layer < a.n_layers; layer++) {
    const FlowLayer &Ly = a.layers[layer];
    const float fb = Ly.fc2_b[col];
    // partial vectors p0, p0 + G, ...: at most kFlowRK per thread
    float t[kFlowRK];
    bool ok = true;
    flow_stamp(a, layer, 0);
    const int NM = a.NM;
    {
      const u64 *base = a.PM + (int64_t)layer * NM * D + col;
      const int fallback = live && p0 < NM ? p0 : 0;  // a partial vector that exists, for the slots past the end
      ok = ll_wait<kFlowRK>(
          [&](int k) {
            const int pp = p0 + k * G;
            return base + (int64_t)(live && pp < NM ? pp : fallback) * D;
          },
          flow_tag(epoch, layer, PH_PM), t, a.state + 1);
    }
    float xp = 0.0f;
    if (p0 == 0) {
      const u64 *px = a.XP + ((int64_t)(i % kRepXP) * a.n_layers + layer) * D + col;
      ok = ll_wait<1>([&](int) { return px; }, flow_tag(epoch, layer, PH_XP), &xp, a.state + 1) && ok;
    }
    if (__syncthreads_or(!ok)) return;
    flow_stamp(a, layer, 1);
    float s = 0.0f;
#pragma unroll
    for (int k = 0; k < kFlowRK; k++)
      if (live && p0 + k * G < NM) s += t[k];
    if (live) smem[p0 * cpw + c] = s;
    __syncthreads();
    if (p0 == 0) {
      float x2 = xp + fb;
      for (int gq = 0; gq < G; gq++) x2 += smem[gq * cpw + c];  // a fixed order: the sum does not depend on timing
      if (layer + 1 < a.n_layers) {
#pragma unroll
        for (int rep = 0; rep < kRepX; rep++)
          ll_store(a.X + ((int64_t)rep * a.n_layers + layer + 1) * D + col, x2, flow_tag(epoch, layer + 1, PH_X));
      } else {
        a.x_out[col] = x2;
      }
    }
    flow_stamp(a, layer, 3);
    __syncthreads();
  }
  if (i == 0 && tid == 0) a.state[0] = (int)(epoch + 1);  // the next step's tags
}

template <int KC, int H>
__global__ __launch_bounds__(NT) void k_dec_flow(FlowArgs a) {
  __shared__ __align__(16) float smem[2048 + 64];
  constexpr int D = 256 * KC, NQ = 3 * D / (NT / 16), NP = D / (NT / 16);
  int b = blockIdx.x;
  if (b < NQ) return flow_role_q<KC>(a, b, smem, smem + 1024);
  b -= NQ;
  if (b < H) return flow_role_a<KC>(a, b, smem);
  b -= H;
  if (b < NP) return flow_role_p<KC>(a, b, smem);
  b -= NP;
  if (b < a.NM) return flow_role_m<KC>(a, b, smem, smem + 1024, smem + 2048);
  flow_role_r(a, b - a.NM, smem);
}

// ------------------------------------------------------------------ host side
void dec_flow_copies(int *x, int *o, int *xp) {
  *x = kRepX;
  *o = kRepO;
  *xp = kRepXP;
}

int dec_flow_grid(int D, int H, int F) { return 3 * D / 32 + H + D / 32 + F / 32 + kFlowNR; }

bool dec_flow_supported(int type_attn, int type_proj, int type_fc, int type_fc2, int D, int H, int F, int n_layers) {
  if (type_attn != CTHIP_Q8_0 || type_proj != CTHIP_Q8_0 || type_fc != CTHIP_Q8_0 || type_fc2 != CTHIP_Q8_0) return false;
  // the widths the kernel is instantiated (and tested) for: d = 256 with 4 heads, d = 768 with 12
  if (!((D == 256 && H == 4) || (D == 768 && H == 12))) return false;
  // the R role adds up F / 32 partial vectors, at most kFlowRK per thread
  if (F % 32 || F / 32 < 1 || F / 32 > kFlowRK * (NT / (D / kFlowNR))) return false;
  // (two layers at least: the workgroup that advances the epoch after the last layer must not get there before every
  // other workgroup has read it, which the hand-overs of an earlier layer guarantee)
  if (n_layers < 2 || n_layers > 31) return false;
  // every workgroup needs a compute unit of its own for the whole step
  return dec_flow_grid(D, H, F) <= state().compute_units;
}

int launch_dec_flow(const FlowArgs &a) {
  if (a.NM != a.F / 32 || a.D % 256 || a.D / a.H != 64) return fail(CTHIP_E_BAD_ARG, "decode flow: inconsistent shape");
  const int grid = dec_flow_grid(a.D, a.H, a.F);
  if (grid > state().compute_units)
    return fail(CTHIP_E_UNSUPPORTED, "decode flow: %d workgroups need %d compute units, the device has %d", grid, grid, state().compute_units);
  hipStream_t st = state().stream;
  const int KC = a.D / 256;
#define FLOW(KC_, H_) hipLaunchKernelGGL((k_dec_flow<KC_, H_>), dim3(grid), dim3(NT), 0, st, a)
  if (KC == 1 && a.H == 4) FLOW(1, 4);
  else if (KC == 3 && a.H == 12) FLOW(3, 12);
  else return fail(CTHIP_E_UNSUPPORTED, "decode flow: d = %d with %d heads", a.D, a.H);
#undef FLOW
  CTHIP_LAUNCH_CHECK();
  return 0;
}

}  // namespace cthip
