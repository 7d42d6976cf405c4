// KV cache kept as Q8_0 rows (option "kv_cache" 1).  The reference's cache is dense fp32, `(B, max_len, H, Dh)`
// created by `linspace ... 0 0` (external/llm/layers.lisp:19-33); at 288 GB per GPU the weights of the models on this
// path are small and what a long-context session holds is its cache, so a session can ask for cache rows in GGUF's
// Q8_0 form instead (external/gguf/dequantize.lisp:40-53: blocks of 32 int8 and one fp16 scale, here as a quant plane
// int8[max_len][KD] and a scale plane fp16[max_len][KD/32]): 1.0625 bytes per element instead of 4.  The new row is
// quantised once, when it is appended (ggml's reference row quantiser: d = absmax / 127, q = round-half-away(x / d));
// attention multiplies the query with the integers and applies a block's scale once per 16-element partial sum.
#include "common.h"

namespace cthip {

// ---- append: fp32 rows -> cache rows [row0 + pos, row0 + pos + s) ----
// one wavefront per 32-element block: lane j < 32 owns element j
__global__ __launch_bounds__(256) void k_kvq_append(signed char *__restrict__ q, unsigned short *__restrict__ d,
                                                    const float *__restrict__ src, int64_t src_stride, int s, int row0,
                                                    const int *__restrict__ pos, int KD) {
  const int nb = KD / 32;
  const int64_t blk = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (blk >= (int64_t)s * nb) return;  // (whole wavefronts leave together)
  const int i = (int)(blk / nb), b = (int)(blk % nb);
  const int row = row0 + (pos ? pos[0] : 0) + i;
  const int j = lane & 31;
  const float x = src[(int64_t)i * src_stride + b * 32 + j];
  float amax = fabsf(x);
#pragma unroll
  for (int o = 16; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));
  const float dd = amax / 127.0f;
  const float inv = dd != 0.0f ? 1.0f / dd : 0.0f;
  const float t = x * inv;
  const float r = copysignf(floorf(fabsf(t) + 0.5f), t);
  if (lane < 32) q[(int64_t)row * KD + b * 32 + j] = (signed char)(int)r;
  if (lane == 0) d[(int64_t)row * nb + b] = __builtin_bit_cast(unsigned short, (_Float16)dd);
}

// ---- rows [0, t) back to fp32 (prompt batches attend over fp32 rows) ----
__global__ __launch_bounds__(256) void k_kvq_dequant(float *__restrict__ dst, const signed char *__restrict__ q,
                                                     const unsigned short *__restrict__ d, int64_t n, int KD) {
  const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (e >= n) return;
  const int64_t row = e / KD;
  const int c = (int)(e % KD);
  dst[e] = (float)q[e] * half_bits_to_float(d[row * (KD / 32) + (c >> 5)]);
}

// ---- one query row per head over cache rows 0..T-1 (T = start_pos + pos + 1), GQA ----
// A key row of a head is DH int8 = DH/16 lanes x 16 bytes; a wavefront covers 64 / (DH/16) keys per pass and holds
// KPT passes of K and V, all requested before any arithmetic (clamped indices, nothing behind a branch); online
// softmax per wavefront, one meeting in LDS -- the layout of the fp32 kernel (k_attn_cached) with 16 elements per lane.
template <int DH>
__global__ __launch_bounds__(256) void k_attn_cached_q8(float *__restrict__ out, const float *__restrict__ qv,
                                                        const signed char *__restrict__ kq, const unsigned short *__restrict__ kd,
                                                        const signed char *__restrict__ vq, const unsigned short *__restrict__ vd,
                                                        int start_pos, const int *__restrict__ pos, int H, int Hkv) {
  constexpr int LPK = DH / 16, KPW = 64 / LPK, KPT = 4, NW = 4, TILE = NW * KPW * KPT;
  __shared__ float part[NW][DH];
  __shared__ float pm[NW], pl[NW];
  const int h = blockIdx.x;
  const int T = start_pos + (pos ? pos[0] : 0) + 1;
  const int hk = h / (H / Hkv);
  const int KD = Hkv * DH, nb = KD / 32;
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int g = lane / LPK, c = lane % LPK;
  float qr[16];
#pragma unroll
  for (int e = 0; e < 4; e++) {
    const float4 v = *(const float4 *)(qv + (int64_t)h * DH + 16 * c + 4 * e);
    qr[4 * e] = v.x, qr[4 * e + 1] = v.y, qr[4 * e + 2] = v.z, qr[4 * e + 3] = v.w;
  }
  const float scale = 1.0f / sqrtf((float)DH);
  const int col = hk * DH + 16 * c;  // first of this lane's 16 elements inside a cache row
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
  for (int t0 = 0; t0 < T; t0 += TILE) {
    if (t0 + wv * KPT * KPW >= T) break;  // nothing left for this wavefront (uniform)
    uint4 kr[KPT], vr[KPT];
    unsigned ks[KPT], vs[KPT];
#pragma unroll
    for (int u = 0; u < KPT; u++) {
      const int j = min(t0 + (wv * KPT + u) * KPW + g, T - 1);  // clamped: masked below, never outside the cache
      kr[u] = *(const uint4 *)(kq + (int64_t)j * KD + col);
      vr[u] = *(const uint4 *)(vq + (int64_t)j * KD + col);
      ks[u] = kd[(int64_t)j * nb + (col >> 5)];
      vs[u] = vd[(int64_t)j * nb + (col >> 5)];
    }
    float sc[KPT];
    float tmax = -INFINITY;
#pragma unroll
    for (int u = 0; u < KPT; u++) {
      float kf[16];
      widen(kr[u], kf);
      float dsum = 0.0f;
#pragma unroll
      for (int e = 0; e < 16; e++) dsum = fmaf(qr[e], kf[e], dsum);
      dsum *= half_bits_to_float((unsigned short)ks[u]);
#pragma unroll
      for (int o = LPK / 2; o > 0; o >>= 1) dsum += __shfl_xor(dsum, o, 64);
      const bool ok = (t0 + (wv * KPT + u) * KPW + g) < T;
      sc[u] = ok ? dsum * scale : -INFINITY;
      tmax = fmaxf(tmax, sc[u]);
    }
#pragma unroll
    for (int o = LPK; o < 64; o <<= 1) tmax = fmaxf(tmax, __shfl_xor(tmax, o, 64));
    const float m_new = fmaxf(m, tmax);   // finite: this wavefront has at least one key here
    const float corr = ct_exp(m - m_new);  // 0 on its first tile (m = -inf)
    float ps = 0.0f;
#pragma unroll
    for (int e = 0; e < 16; e++) acc[e] *= corr;
#pragma unroll
    for (int u = 0; u < KPT; u++) {
      const float p = ct_exp(sc[u] - m_new);  // exp2(-inf) = 0 for masked keys
      ps += p;
      float vf[16];
      widen(vr[u], vf);
      const float pv = p * half_bits_to_float((unsigned short)vs[u]);
#pragma unroll
      for (int e = 0; e < 16; e++) acc[e] = fmaf(pv, vf[e], acc[e]);
    }
#pragma unroll
    for (int o = LPK; o < 64; o <<= 1) ps += __shfl_xor(ps, o, 64);  // every lane of a key holds the same p
    l = l * corr + ps;
    m = m_new;
  }
#pragma unroll
  for (int o = LPK; o < 64; o <<= 1) {
#pragma unroll
    for (int e = 0; e < 16; e++) acc[e] += __shfl_xor(acc[e], o, 64);
  }
  if (lane < LPK) {
#pragma unroll
    for (int e = 0; e < 16; e++) part[wv][16 * lane + e] = acc[e];
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
    out[(int64_t)h * DH + tid] = o / L;
  }
}

// ---- one decode step over Q8_0 rows in ONE launch ----
// What a step of a session with such a cache used to queue per layer besides its Linears: rotate q, rotate the new
// key, quantise and append the key row, the same for the value row, attend.  Here the workgroup does all of it in
// registers: the head's rotation angles are computed once (one pair per thread, shared through LDS; the pair
// rotation has the rounding of k_rope), the lane rotates its 16 query elements and its 16 elements of the new key,
// quantises the new key and value as k_kvq_append does (the planes get the same bits), uses them as key T - 1 and,
// in the first query head of each key / value head, stores them into the planes.  A head's keys are shared by
// gridDim.z workgroups as in k_attn_cached's SPLIT form (ranges of whole tiles, device-scope stores of the
// (max, sum, output) triples, a ticket per range, the last one adds them up in range order).
template <int DH>
__global__ __launch_bounds__(256) void k_attn_q8_step(float *__restrict__ out, const float *__restrict__ qv, const float *__restrict__ newkv,
                                                      signed char *__restrict__ kq, unsigned short *__restrict__ kd,
                                                      signed char *__restrict__ vq, unsigned short *__restrict__ vd,
                                                      const int *__restrict__ pos, int H, int Hkv, float log2_base, int rope,
                                                      float *__restrict__ sp_part, int *__restrict__ sp_count) {
  constexpr int LPK = DH / 16, KPW = 64 / LPK, KPT = 4, NW = 4, TILE = NW * KPW * KPT;
  __shared__ float part[NW][DH];
  __shared__ float pm[NW], pl[NW];
  __shared__ float ang_s[DH / 2], ang_c[DH / 2];
  __shared__ int ticket;
  const int h = attn_head_of_block(blockIdx.x, H, Hkv);
  const int T = pos[0] + 1;
  int k0 = 0, k1 = T, nranges = 1;
  {
    const int nz = (int)gridDim.z, tiles = (T + TILE - 1) / TILE;
    const int per = ((tiles + nz - 1) / nz) * TILE;  // keys per range
    nranges = (T + per - 1) / per;
    k0 = (int)blockIdx.z * per;
    if (k0 >= T) return;  // (uniform) no range for this workgroup
    k1 = min(T, k0 + per);
  }
  const int group = H / Hkv, hk = h / group;
  const int KD = Hkv * DH, nb = KD / 32;
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int g = lane / LPK, c = lane % LPK;
  const int col = hk * DH + 16 * c;  // first of this lane's 16 elements inside a cache row
  // A tile's rows and scales.  The first tile is asked for as soon as the position is known, before the angles, the
  // query and the new row are worked on: its round trip to memory runs beside that arithmetic.
  uint4 kr[KPT], vr[KPT];
  unsigned ks[KPT], vs[KPT];
  auto request = [&](int t0) {
#pragma unroll
    for (int u = 0; u < KPT; u++) {
      const int j = t0 + (wv * KPT + u) * KPW + g;
      const int jj = min(j, max(T - 2, 0));  // clamped: masked below; row T - 1 is not in the planes yet
      kr[u] = *(const uint4 *)(kq + (int64_t)jj * KD + col);
      vr[u] = *(const uint4 *)(vq + (int64_t)jj * KD + col);
      ks[u] = kd[(int64_t)jj * nb + (col >> 5)];
      vs[u] = vd[(int64_t)jj * nb + (col >> 5)];
    }
  };
  if (k0 + wv * KPT * KPW < k1) request(k0);  // (uniform per wavefront)
  if (rope) {
    if (tid < DH / 2) {  // theta_i = base^(-2i / DH), as k_rope spells it
      const float expo = (float)(2 * tid) / (float)DH;
      const float theta = exp2f(-(expo * (log2_base * 0.6931472f)) * 1.442695f);
      float sn, cs;
      sincosf((float)(T - 1) * theta, &sn, &cs);
      ang_s[tid] = sn;
      ang_c[tid] = cs;
    }
    __syncthreads();
  }
  auto load16 = [&](const float *src, float *x) {
#pragma unroll
    for (int e = 0; e < 4; e++) {
      const float4 v = *(const float4 *)(src + 4 * e);
      x[4 * e] = v.x, x[4 * e + 1] = v.y, x[4 * e + 2] = v.z, x[4 * e + 3] = v.w;
    }
  };
  auto rotate16 = [&](float *x) {  // pairs 8c .. 8c + 7 of the head
#pragma unroll
    for (int t = 0; t < 8; t++) {
      float o0, o1;
      rope_pair(x[2 * t], x[2 * t + 1], ang_s[8 * c + t], ang_c[8 * c + t], o0, o1);
      x[2 * t] = o0, x[2 * t + 1] = o1;
    }
  };
  float qr[16];
  load16(qv + (int64_t)h * DH + 16 * c, qr);
  if (rope) rotate16(qr);
  // the new row of this key / value head: needed by the range that ends at T, and by the one that stores it
  uint4 knq = make_uint4(0u, 0u, 0u, 0u), vnq = knq;
  unsigned knd = 0, vnd = 0;
  const bool has_new = k1 == T, stores = blockIdx.z == 0 && h % group == 0;
  if (has_new || stores) {  // (uniform)
    auto quantise = [&](const float *x, uint4 &qv4, unsigned &dv) {  // lanes c and c ^ 1 share a block of 32
      float amax = 0.0f;
#pragma unroll
      for (int e = 0; e < 16; e++) amax = fmaxf(amax, fabsf(x[e]));
      amax = fmaxf(amax, dpp_f<0xB1>(amax));  // quad_perm [1,0,3,2]
      const float dd = amax / 127.0f;
      const float inv = dd != 0.0f ? 1.0f / dd : 0.0f;
      unsigned w[4] = {0u, 0u, 0u, 0u};
#pragma unroll
      for (int e = 0; e < 16; e++) {
        const float t = x[e] * inv;
        const int r = (int)(t + copysignf(0.5f, t));  // = copysign(floor(|t| + 0.5), t): the conversion truncates
        w[e >> 2] |= ((unsigned)r & 255u) << (8 * (e & 3));
      }
      qv4 = make_uint4(w[0], w[1], w[2], w[3]);
      dv = __builtin_bit_cast(unsigned short, (_Float16)dd);
    };
    float x[16];
    load16(newkv + col, x);
    if (rope) rotate16(x);
    quantise(x, knq, knd);
    load16(newkv + KD + col, x);
    quantise(x, vnq, vnd);
    if (stores && tid < LPK) {  // the `!assign` into the cache row at pos
      *(uint4 *)(kq + (int64_t)(T - 1) * KD + col) = knq;
      *(uint4 *)(vq + (int64_t)(T - 1) * KD + col) = vnq;
      if ((c & 1) == 0) {
        kd[(int64_t)(T - 1) * nb + (col >> 5)] = (unsigned short)knd;
        vd[(int64_t)(T - 1) * nb + (col >> 5)] = (unsigned short)vnd;
      }
    }
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
  for (int t0 = k0; t0 < k1; t0 += TILE) {
    if (t0 + wv * KPT * KPW >= k1) break;  // nothing left for this wavefront (uniform)
    if (t0 != k0) request(t0);
#pragma unroll
    for (int u = 0; u < KPT; u++) {
      if (t0 + (wv * KPT + u) * KPW + g >= T - 1) kr[u] = knq, vr[u] = vnq, ks[u] = knd, vs[u] = vnd;
    }
    float sc[KPT];
    float tmax = -INFINITY;
#pragma unroll
    for (int u = 0; u < KPT; u++) {
      float kf[16];
      widen(kr[u], kf);
      float dsum = 0.0f;
#pragma unroll
      for (int e = 0; e < 16; e++) dsum = fmaf(qr[e], kf[e], dsum);
      dsum *= half_bits_to_float((unsigned short)ks[u]);
#pragma unroll
      for (int o = LPK / 2; o > 0; o >>= 1) dsum += __shfl_xor(dsum, o, 64);
      const bool ok = (t0 + (wv * KPT + u) * KPW + g) < k1;
      sc[u] = ok ? dsum * scale : -INFINITY;
      tmax = fmaxf(tmax, sc[u]);
    }
#pragma unroll
    for (int o = LPK; o < 64; o <<= 1) tmax = fmaxf(tmax, __shfl_xor(tmax, o, 64));
    const float m_new = fmaxf(m, tmax);   // finite: this wavefront has at least one key here
    const float corr = ct_exp(m - m_new);  // 0 on its first tile (m = -inf)
    float ps = 0.0f;
#pragma unroll
    for (int e = 0; e < 16; e++) acc[e] *= corr;
#pragma unroll
    for (int u = 0; u < KPT; u++) {
      const float p = ct_exp(sc[u] - m_new);  // exp2(-inf) = 0 for masked keys
      ps += p;
      float vf[16];
      widen(vr[u], vf);
      const float pv = p * half_bits_to_float((unsigned short)vs[u]);
#pragma unroll
      for (int e = 0; e < 16; e++) acc[e] = fmaf(pv, vf[e], acc[e]);
    }
#pragma unroll
    for (int o = LPK; o < 64; o <<= 1) ps += __shfl_xor(ps, o, 64);  // every lane of a key holds the same p
    l = l * corr + ps;
    m = m_new;
  }
#pragma unroll
  for (int o = LPK; o < 64; o <<= 1) {
#pragma unroll
    for (int e = 0; e < 16; e++) acc[e] += __shfl_xor(acc[e], o, 64);
  }
  if (lane < LPK) {
#pragma unroll
    for (int e = 0; e < 16; e++) part[wv][16 * lane + e] = acc[e];
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
    if (nranges == 1) {
      out[(int64_t)h * DH + tid] = o / L;
    } else {
      float *mine = sp_part + ((int64_t)h * gridDim.z + blockIdx.z) * (DH + 2);
      __hip_atomic_store(mine + tid, o, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (tid == 0) {
        __hip_atomic_store(mine + DH, M, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(mine + DH + 1, L, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  }
  if (nranges > 1) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this thread's device-scope stores have reached memory
    __syncthreads();
    if (tid == 0) ticket = __hip_atomic_fetch_add(sp_count + h, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (ticket != nranges - 1) return;  // (uniform)
    if (tid < DH) {
      out[(int64_t)h * DH + tid] = attn_split_merge(sp_part + (int64_t)h * gridDim.z * (DH + 2), nranges, DH, tid);
    }
    if (tid == 0) __hip_atomic_store(sp_count + h, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // the next launch counts again
  }
}

int launch_kvq_append(void *q, void *d, const float *src, int64_t src_stride, int s, int row0, const int *pos, int KD) {
  if (s <= 0) return 0;
  if (KD % 32) return fail(CTHIP_E_BAD_ARG, "quantised KV cache: rows of %d elements are not whole blocks of 32", KD);
  const int64_t blocks = (int64_t)s * (KD / 32);
  hipLaunchKernelGGL(k_kvq_append, dim3((unsigned)((blocks + 3) / 4)), dim3(256), 0, state().stream, (signed char *)q,
                     (unsigned short *)d, src, src_stride, s, row0, pos, KD);
  CTHIP_LAUNCH_CHECK();
  return 0;
}

int launch_kvq_dequant(float *dst, const void *q, const void *d, int rows, int KD) {
  const int64_t n = (int64_t)rows * KD;
  if (n <= 0) return 0;
  hipLaunchKernelGGL(k_kvq_dequant, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, state().stream, dst, (const signed char *)q,
                     (const unsigned short *)d, n, KD);
  CTHIP_LAUNCH_CHECK();
  return 0;
}

int launch_attn_q8(float *out, const float *q, const void *kq, const void *kd, const void *vq, const void *vd, int start_pos,
                   const int *pos, int H, int Hkv, int Dh) {
  dim3 grid((unsigned)H), block(256);
  hipStream_t st = state().stream;
#define ATT(DH_)                                                                                                          \
  hipLaunchKernelGGL((k_attn_cached_q8<DH_>), grid, block, 0, st, out, q, (const signed char *)kq, (const unsigned short *)kd, \
                     (const signed char *)vq, (const unsigned short *)vd, start_pos, pos, H, Hkv)
  switch (Dh) {
    case 32: ATT(32); break;
    case 64: ATT(64); break;
    case 128: ATT(128); break;
    default: return fail(CTHIP_E_UNSUPPORTED, "quantised KV cache: head_dim %d (supported: 32, 64, 128)", Dh);
  }
#undef ATT
  CTHIP_LAUNCH_CHECK();
  return 0;
}

int launch_attn_q8_step(float *out, const float *q, const float *newkv, void *kq, void *kd, void *vq, void *vd, const int *pos,
                        int H, int Hkv, int Dh, float rope_base, const AttnSplit *split) {
  if (Hkv <= 0 || H % Hkv) return fail(CTHIP_E_BAD_ARG, "quantised KV cache: %d query heads over %d key / value heads", H, Hkv);
  if (split && split->ranges > kAttnSplitMaxRanges) return fail(CTHIP_E_BAD_ARG, "quantised KV cache: %d key ranges per head (at most %d)", split->ranges, kAttnSplitMaxRanges);
  const bool shared = split && split->ranges > 1;
  dim3 grid((unsigned)H, 1, shared ? (unsigned)split->ranges : 1u), block(256);
  hipStream_t st = state().stream;
  const int rope = rope_base > 0.0f ? 1 : 0;
  const float lb = rope ? log2f(rope_base) : 0.0f;
#define ATT(DH_)                                                                                                                 \
  hipLaunchKernelGGL((k_attn_q8_step<DH_>), grid, block, 0, st, out, q, newkv, (signed char *)kq, (unsigned short *)kd, (signed char *)vq, \
                     (unsigned short *)vd, pos, H, Hkv, lb, rope, shared ? split->part : nullptr, shared ? split->count : nullptr)
  switch (Dh) {
    case 32: ATT(32); break;
    case 64: ATT(64); break;
    case 128: ATT(128); break;
    default: return fail(CTHIP_E_UNSUPPORTED, "quantised KV cache: head_dim %d (supported: 32, 64, 128)", Dh);
  }
#undef ATT
  CTHIP_LAUNCH_CHECK();
  return 0;
}

}  // namespace cthip

using namespace cthip;

extern "C" {

int cthip_kv_append_q8(void *q_plane, void *d_plane, const float *rows, int s, int row0, int kv_dim) {
  CTHIP_REQUIRE_INIT();
  CTHIP_ARG(s >= 0 && row0 >= 0 && kv_dim > 0 && kv_dim % 32 == 0);
  CTHIP_ARG(s == 0 || (q_plane && d_plane && rows));
  return launch_kvq_append(q_plane, d_plane, rows, kv_dim, s, row0, nullptr, kv_dim);
}

int cthip_sdpa_cached_q8(float *out, const float *q, const void *k_q, const void *k_d, const void *v_q, const void *v_d, int T,
                         int H, int Hkv, int Dh) {
  CTHIP_REQUIRE_INIT();
  CTHIP_ARG(T >= 1 && H > 0 && Hkv > 0 && H % Hkv == 0);
  CTHIP_ARG(out && q && k_q && k_d && v_q && v_d);
  return launch_attn_q8(out, q, k_q, k_d, v_q, v_d, T - 1, nullptr, H, Hkv, Dh);
}

}  // extern "C"

