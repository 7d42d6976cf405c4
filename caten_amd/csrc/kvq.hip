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

