// KV cache kept in pages (option "kv_cache" 2).  The reference allocates its cache densely and once, `(B, max_len, H,
// Dh)` zeros (external/llm/layers.lisp:19-33), so a session holds max_len rows per layer whether it ever reaches them
// or not.  Here a session can instead hold pages of kKvPageRows rows that are opened when the position first
// reaches them: per layer a table of page pointers in device memory (`pages[row / 64] + (row % 64) * KD`), which the
// host extends before it queues the steps that need the rows.  The table's address never changes, so captured graphs
// stay valid while the cache grows.  Rows are fp32, as in the reference: results are those of the dense cache bit for
// bit wherever the arithmetic is the same (the attention below adds in the order of k_attn_cached).
#include <type_traits>

#include "common.h"

namespace cthip {

__device__ __forceinline__ const float *kvp_row(const float *const *pages, int row, int KD) {
  return pages[row / kKvPageRows] + (int64_t)(row % kKvPageRows) * KD;
}

// ---- append: fp32 rows -> cache rows [row0 + pos, row0 + pos + s) of the key pages and of the value pages ----
__global__ __launch_bounds__(256) void k_kvp_append(float *const *__restrict__ kpages, float *const *__restrict__ vpages,
                                                    const float *__restrict__ ksrc, const float *__restrict__ vsrc,
                                                    int64_t src_stride, int s, int row0, const int *__restrict__ pos, int KD) {
  const int n4 = KD / 4;
  const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (e >= (int64_t)s * n4) return;
  const int i = (int)(e / n4), c = (int)(e % n4);
  const int row = row0 + (pos ? pos[0] : 0) + i;
  float *kd = kpages[row / kKvPageRows] + (int64_t)(row % kKvPageRows) * KD;
  float *vd = vpages[row / kKvPageRows] + (int64_t)(row % kKvPageRows) * KD;
  ((float4 *)kd)[c] = ((const float4 *)(ksrc + (int64_t)i * src_stride))[c];
  ((float4 *)vd)[c] = ((const float4 *)(vsrc + (int64_t)i * src_stride))[c];
}

// ---- rows [0, t) as one dense array (prompt batches attend over dense rows; rows of pages not opened yet are zero) ----
__global__ __launch_bounds__(256) void k_kvp_gather(float *__restrict__ dst, const float *const *__restrict__ pages, int64_t n4, int KD) {
  const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (e >= n4) return;
  const int kd4 = KD / 4;
  const int row = (int)(e / kd4), c = (int)(e % kd4);
  const float *page = pages[row / kKvPageRows];
  ((float4 *)dst)[e] = page ? ((const float4 *)(page + (int64_t)(row % kKvPageRows) * KD))[c] : make_float4(0.f, 0.f, 0.f, 0.f);
}

// ---- one query row per head over cache rows 0..T-1 (T = start_pos + pos + 1), GQA ----
// The lane layout of k_attn_cached (rowops.hip): a key row of a head is read by DH/4 adjacent lanes as one float4
// each, a wavefront holds KPT passes of K and V (all page pointers requested first, then all rows: two memory
// round trips a tile instead of one), online softmax per wavefront, one meeting in LDS.
//
// STEP (a session's decode step): the launch also does what k_attn_cached does in its APPEND and SPLIT forms -- the
// step's new key / value row (newkv: k then v, unrotated) is rotated in registers where the model rotates, used as
// key T - 1 and copied into its page by the first query head of each key / value head, and the keys of a head are
// shared by gridDim.z workgroups (ranges of whole tiles, device-scope stores of the (max, sum, output) triples, a
// ticket per range, the last one adds them up in range order).  The page of row T - 1 was opened by the host before
// the step was queued.
template <int DH, bool STEP>
__global__ __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(4, 4)))
void k_attn_cached_paged(float *__restrict__ out, const float *__restrict__ q, const float *const *__restrict__ kpages,
                         const float *const *__restrict__ vpages, int start_pos, const int *__restrict__ pos, int H, int Hkv,
                         const float *__restrict__ newkv, float log2_base, int rope, float *__restrict__ sp_part,
                         int *__restrict__ sp_count) {
  constexpr int LPK = DH / 4, KPW = 64 / LPK, KPT = 4, NW = 16, TILE = NW * KPW * KPT;
  __shared__ float part[NW][DH];
  __shared__ float pm[NW], pl[NW];
  __shared__ int ticket;
  const int h = attn_head_of_block(blockIdx.x, H, Hkv);
  const int T = start_pos + (pos ? pos[0] : 0) + 1;
  int k0 = 0, k1 = T, nranges = 1;
  if (STEP) {
    const int nz = (int)gridDim.z, tiles = (T + TILE - 1) / TILE;
    const int per = ((tiles + nz - 1) / nz) * TILE;  // keys per range
    nranges = (T + per - 1) / per;
    k0 = (int)blockIdx.z * per;
    if (k0 >= T) return;  // (uniform) no range for this workgroup
    k1 = min(T, k0 + per);
  }
  const int hk = h / (H / Hkv);
  const int KD = Hkv * DH;
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int g = lane / LPK, c = lane % LPK;
  float4 q4 = *(const float4 *)(q + (int64_t)h * DH + 4 * c);
  float4 kn = make_float4(0.f, 0.f, 0.f, 0.f), vn = kn;
  if (STEP) {
    kn = *(const float4 *)(newkv + hk * DH + 4 * c);
    vn = *(const float4 *)(newkv + KD + hk * DH + 4 * c);
  }
  // a tile's rows: the page pointers first, then the rows they address
  auto request = [&](auto np_tag, int t0, float4 *kr, float4 *vr) {
    constexpr int NP = decltype(np_tag)::value;
    const float *kpg[NP], *vpg[NP];
    unsigned off[NP];
#pragma unroll
    for (int u = 0; u < NP; u++) {
      const int j = t0 + (wv * NP + u) * KPW + g;
      const int jj = min(j, STEP ? max(T - 2, 0) : T - 1);  // clamped: masked below, never a row that has no page yet; STEP: row T - 1 comes from the registers
      kpg[u] = kpages[jj / kKvPageRows];
      vpg[u] = vpages[jj / kKvPageRows];
      off[u] = (unsigned)(jj % kKvPageRows) * (unsigned)KD + (unsigned)(hk * DH + 4 * c);
    }
#pragma unroll
    for (int u = 0; u < NP; u++) {
      kr[u] = *(const float4 *)(kpg[u] + off[u]);
      vr[u] = *(const float4 *)(vpg[u] + off[u]);
    }
  };
  // rotation of the query and of the new key, and the new row's store (the `!assign` into the cache row at pos)
  auto rotate_and_append = [&]() {
    if (STEP) {
      if (rope) {
        const Rope4 ra = rope4_angles(c, DH, log2_base, T - 1);
        q4 = rope4_apply(q4, ra);
        kn = rope4_apply(kn, ra);
      }
      if (h % (H / Hkv) == 0 && tid < LPK && blockIdx.z == 0) {
        float *kd = const_cast<float *>(kvp_row(kpages, T - 1, KD)), *vd = const_cast<float *>(kvp_row(vpages, T - 1, KD));
        ((float4 *)(kd + hk * DH))[c] = kn;
        ((float4 *)(vd + hk * DH))[c] = vn;
      }
    }
  };
  const float scale = 1.0f / sqrtf((float)DH);
  float m = -INFINITY, l = 0.0f;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  auto consume = [&](auto np_tag, int t0, float4 *kr, float4 *vr) {
    constexpr int NP = decltype(np_tag)::value;
    if (STEP) {
#pragma unroll
      for (int u = 0; u < NP; u++) {
        if (t0 + (wv * NP + u) * KPW + g >= T - 1) kr[u] = kn, vr[u] = vn;
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
      if (LPK == 16) {
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
  // The first tile's rows are asked for as soon as the position is known, before the query is waited for and rotated
  // (as in k_attn_cached).
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
    if (STEP) {
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
    if (!STEP || nranges == 1) {
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
  if (STEP && nranges > 1) {
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

int launch_kvp_append(float *const *kpages, float *const *vpages, const float *ksrc, const float *vsrc, int64_t src_stride, int s,
                      int row0, const int *pos, int KD) {
  if (s == 0) return 0;
  if (KD % 4) return fail(CTHIP_E_BAD_ARG, "paged KV cache: rows of %d floats are not a multiple of four", KD);
  const int64_t n = (int64_t)s * (KD / 4);
  hipLaunchKernelGGL(k_kvp_append, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, state().stream, kpages, vpages, ksrc, vsrc,
                     src_stride, s, row0, pos, KD);
  CTHIP_LAUNCH_CHECK();
  return 0;
}

int launch_kvp_gather(float *dst, const float *const *pages, int rows, int KD) {
  if (rows == 0) return 0;
  const int64_t n4 = (int64_t)rows * (KD / 4);
  hipLaunchKernelGGL(k_kvp_gather, dim3((unsigned)((n4 + 255) / 256)), dim3(256), 0, state().stream, dst, pages, n4, KD);
  CTHIP_LAUNCH_CHECK();
  return 0;
}

int launch_attn_paged(float *out, const float *q, const float *const *kpages, const float *const *vpages, int start_pos,
                      const int *pos, int H, int Hkv, int Dh) {
  dim3 grid(H), block(1024);
  hipStream_t st = state().stream;
  const float *nokv = nullptr;
  float *nop = nullptr;
  int *noc = nullptr;
#define ATT(DH_) hipLaunchKernelGGL((k_attn_cached_paged<DH_, false>), grid, block, 0, st, out, q, kpages, vpages, start_pos, pos, H, Hkv, nokv, 0.0f, 0, nop, noc)
  switch (Dh) {
    case 32: ATT(32); break;
    case 64: ATT(64); break;
    case 128: ATT(128); break;
    default: return fail(CTHIP_E_UNSUPPORTED, "attention: head_dim %d (supported: 32, 64, 128)", Dh);
  }
#undef ATT
  CTHIP_LAUNCH_CHECK();
  return 0;
}

// one decode step over a paged cache: rotation (rope_base > 0) and append of the new row (newkv: k then v, fp32,
// unrotated) and the attention in one launch; `split` as for launch_attn
int launch_attn_paged_step(float *out, const float *q, const float *newkv, float *const *kpages, float *const *vpages, const int *pos,
                           int H, int Hkv, int Dh, float rope_base, const AttnSplit *split) {
  if (Hkv <= 0 || H % Hkv) return fail(CTHIP_E_BAD_ARG, "paged KV cache: %d query heads over %d key / value heads", H, Hkv);
  if (split && split->ranges > kAttnSplitMaxRanges) return fail(CTHIP_E_BAD_ARG, "paged KV cache: %d key ranges per head (at most %d)", split->ranges, kAttnSplitMaxRanges);
  const bool shared = split && split->ranges > 1;
  dim3 grid((unsigned)H, 1, shared ? (unsigned)split->ranges : 1u), block(1024);
  hipStream_t st = state().stream;
  const int rope = rope_base > 0.0f ? 1 : 0;
  const float lb = rope ? log2f(rope_base) : 0.0f;
#define ATT(DH_)                                                                                                               \
  hipLaunchKernelGGL((k_attn_cached_paged<DH_, true>), grid, block, 0, st, out, q, (const float *const *)kpages,                  \
                     (const float *const *)vpages, 0, pos, H, Hkv, newkv, lb, rope, shared ? split->part : nullptr,               \
                     shared ? split->count : nullptr)
  switch (Dh) {
    case 32: ATT(32); break;
    case 64: ATT(64); break;
    case 128: ATT(128); break;
    default: return fail(CTHIP_E_UNSUPPORTED, "attention: head_dim %d (supported: 32, 64, 128)", Dh);
  }
#undef ATT
  CTHIP_LAUNCH_CHECK();
  return 0;
}

}  // namespace cthip

using namespace cthip;

extern "C" {

int cthip_kv_page_rows(void) { return kKvPageRows; }

int cthip_kv_append_paged(void *const *k_pages, void *const *v_pages, const float *k_rows, const float *v_rows, int s, int row0,
                          int kv_dim) {
  CTHIP_REQUIRE_INIT();
  CTHIP_ARG(s >= 0 && row0 >= 0 && kv_dim > 0 && kv_dim % 4 == 0);
  CTHIP_ARG(s == 0 || (k_pages && v_pages && k_rows && v_rows));
  return launch_kvp_append((float *const *)k_pages, (float *const *)v_pages, k_rows, v_rows, kv_dim, s, row0, nullptr, kv_dim);
}

int cthip_sdpa_cached_paged(float *out, const float *q, const void *const *k_pages, const void *const *v_pages, int T, int H, int Hkv,
                            int Dh) {
  CTHIP_REQUIRE_INIT();
  CTHIP_ARG(T >= 1 && H > 0 && Hkv > 0 && H % Hkv == 0);
  CTHIP_ARG(out && q && k_pages && v_pages);
  return launch_attn_paged(out, q, (const float *const *)k_pages, (const float *const *)v_pages, T - 1, nullptr, H, Hkv, Dh);
}

}  // extern "C"
