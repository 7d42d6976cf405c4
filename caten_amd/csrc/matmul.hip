// MFMA GEMM for the matmul-shaped fusions: `!relu(!matmul A B)` (source/api/high-level-ops.lisp:76-99,
// fused per source/test-suite/test-scheduler.lisp:140-163) and Linear over m > 1 rows (prefill,
// source/nn/linear.lisp:3-17) with the weights still packed (dequantised while they are staged).
//
// A workgroup owns a 64x64 tile of C; four of its wavefronts (2x2) accumulate a 32x32 sub-tile each in 16
// accumulator registers, with v_mfma_f32_32x32x2_f32 (k_gemm_f32pc / k_gemm_f32, fp32 operands) or
// v_mfma_f32_32x32x16_bf16 (k_gemm_split, operands split into bf16 terms, fp32 accumulation), while eight more
// stage the operands (k_gemm_f32, packed weights with fp32 operands, is the one kernel whose four wavefronts do
// both).  Operands go through LDS buffers with three K-steps of global loads in flight; 1024x1024 outputs give
// 256 workgroups = one per compute unit.  Quantised weights take k_gemm_qpc: 64x128 tiles, four multiplying and
// eight staging wavefronts.  Finished tiles leave through LDS as whole rows (store_tile).
#include <hip/hip_bf16.h>

#include "common.h"

namespace cthip {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef short v4s __attribute__((ext_vector_type(4)));

enum { B_ROWMAJOR = 0, B_WMAT = 1 };  // B given as (K,N) fp32, or as a packed weight matrix (N rows x K cols)

struct GemmArgs {
  float *C;
  const float *A;        // (M,K) row-major
  const float *B;        // (K,N) row-major (B_ROWMAJOR)
  const void *wq;        // packed planes (B_WMAT)
  const unsigned short *wd;
  int wtype;
  const float *bias;     // per output column, may be null
  const float *residual; // (M,N), may be null
  int M, N, K;
  int act;
  // split-K: workgroup (tile, z) covers k in [z * kper, (z + 1) * kper) and writes
  // its raw partial tile to ws[z][M][N]; k_splitk_reduce adds the partials in z order and applies the epilogue
  int ksplit, kper;
  float *ws;
  // tile -> workgroup mapping: the tm x tn tile grid is cut into rx x ry = 8 regions of
  // rm x rn tiles, one per XCD (workgroup i is dispatched to XCD i % 8), so that every L2 holds only
  // its region's rows of A and columns of B
  int tm, tn, rx, rm, rn;
  int pairs;        // 1: columns (2j, 2j + 1) are (gate, up) and C (M, N / 2) gets silu(gate) * up
  int routed;       // 1: whole tiles go to route.dst[...] instead of C (see GemmRoute)
  GemmRoute route;
};

// ---------------------------------------------------------------------------------------------
// bf16 MFMA GEMM with fp32 accumulation, operands optionally split in two bf16 terms.
//
// v_mfma_f32_32x32x16_bf16 runs at 16x the rate of the fp32-operand MFMA.  NS = 1 rounds both operands
// to bf16 (rtol/atol 1e-2 class).  NS = 3 writes every operand as hi + lo with hi = bf16(x) and
// lo = bf16(x - hi) and accumulates hi*hi + lo*hi + hi*lo: what is dropped is below 2^-16 of a product.
// NS = 6 uses three terms per operand (24 significant bits: the fp32 value itself) and the six
// products above 2^-24: fp32-grade results at a sixth of the bf16 rate, which is still 2.6 times the
// fp32-operand MFMA peak.
//
// A workgroup (2x2 multiplying wavefronts + eight staging ones) owns a 64x64 tile of C and walks K in steps of 64.  The
// fp32 (or packed) operands of a step are converted ONCE per workgroup on their way into LDS, which
// holds them k-contiguous per row in bf16, 16-byte chunks swizzled by row so that neither the operand
// reads nor the staging writes collide on banks.  Two LDS buffers and three register sets keep the
// global loads three K-steps ahead of the MFMAs with one barrier per step.
enum { W_ROWMAJOR = 0, W_F32 = 1, W_F16 = 2, W_Q4 = 3, W_Q8 = 4 };  // W_Q4 / W_Q8: k_gemm_qpc only
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
typedef float v2f __attribute__((ext_vector_type(2)));

// round to nearest even, x0 in the low half: as a vector conversion this is ONE v_cvt_pk_bf16_f32 (two scalar
// conversions are two of them, each with an idle half, plus a shift and an or)
__device__ __forceinline__ unsigned pack_bf16(float x0, float x1) {
  const v2f v = {x0, x1};
  return __builtin_bit_cast(unsigned, __builtin_convertvector(v, v2bf));
}
// 4 consecutive k -> NP planes of 4 bf16: plane 0 = bf16(x), plane p = bf16(what planes 0..p-1 miss)
template <int NP>
__device__ __forceinline__ void split4(float r0, float r1, float r2, float r3, uint2 *pl) {
#pragma unroll
  for (int p = 0; p < NP; p++) {
    pl[p].x = pack_bf16(r0, r1);
    pl[p].y = pack_bf16(r2, r3);
    if (p + 1 < NP) {  // exact: the difference of a float and its own leading bits
      r0 -= __uint_as_float(pl[p].x << 16);
      r1 -= __uint_as_float(pl[p].x & 0xffff0000u);
      r2 -= __uint_as_float(pl[p].y << 16);
      r3 -= __uint_as_float(pl[p].y & 0xffff0000u);
    }
  }
}

// Zeros in device memory: what a request outside an operand reads.  (A load followed by a select would make
// the request's own thread wait for it at once; a branch around it splits the run of requests.)
__device__ __align__(16) unsigned g_zeros[8];  // zero-initialised, never written (not const: a load that may come from
                                                // either here or an operand must stay a global-memory load)

// Four consecutive floats at p without a branch or a dependent instruction: of the four, those past `nvalid`
// (0..4) are read from g_zeros.  AL: the four are 16-byte aligned and all inside or all outside.  A K-step's
// requests stay one straight run of loads, so that the waits before their use count the younger requests
// instead of draining them.
template <bool AL>
__device__ __forceinline__ float4 load4(const float *p, int nvalid) {
  const float *z = (const float *)g_zeros;
  if (AL) return *(const float4 *)(nvalid > 0 ? p : z);
  return make_float4(*(nvalid > 0 ? p : z), *(nvalid > 1 ? p + 1 : z), *(nvalid > 2 ? p + 2 : z), *(nvalid > 3 ? p + 3 : z));
}
__device__ __forceinline__ int clamp04(int v) { return v < 0 ? 0 : v > 4 ? 4 : v; }

struct ARegs {  // one K-step of A held by a thread: rows ar + 16 i
  float4 v0, v1, v2, v3;
};

// (a native vector type: copies of HIP's uint4 struct between address spaces can become memcpy calls, and register
// sets written that way stay in scratch memory)
typedef unsigned v4u __attribute__((ext_vector_type(4)));
template <int BMODE>
struct BRegs {  // one K-step of B held by a thread between its request and its conversion
  static constexpr int NV = (BMODE == W_ROWMAJOR || BMODE == W_F32) ? 4 : (BMODE == W_F16 ? 2 : 1);
  v4u v[NV];
};

// LDS rows are 64 bf16 = eight 16-byte chunks; chunk c of row r is stored at position c ^ swz(r), which
// spreads the 128-bit operand reads of 8 consecutive rows, the 64-bit writes of the transposing B
// staging and the row-wise A writes over all banks.
__device__ __forceinline__ int swz(int row) { return (row ^ (row >> 3)) & 7; }

// Row-wise stores of a finished BM x BN tile that the multiplying wavefronts have put into LDS (Cs, row pitch
// BN + 4 floats): all NT threads of the workgroup take 16-byte pieces of whole rows, so a store instruction covers
// 512 contiguous bytes per 32 lanes and bias / residual are read the same way.  (Stores straight from the
// accumulator layout are 16 or 32 scalar stores per lane and keep a workgroup busy for microseconds.)
// Split-K shares go to their slice of a.ws untouched.  Call after a barrier that follows the writes to Cs.
template <int BM, int BN, int NT>
__device__ __forceinline__ void store_tile(const GemmArgs &a, const float *Cs, int m0, int n0, int tid) {
  constexpr int LDC = BN + 4, F4 = BN / 4;
  const int M = a.M, N = a.N;
  const bool plain = a.ksplit > 1;
  float *dst = plain ? a.ws + (int64_t)blockIdx.y * M * N : a.C;
  int ldd = N, cbase = 0;  // row pitch of the destination and the column its first element stands for
  if (a.routed) {
    const int part = n0 >= a.route.c0[2] ? 2 : n0 >= a.route.c0[1] ? 1 : 0;  // uniform over the workgroup
    dst = a.route.dst[part], ldd = a.route.ld[part], cbase = a.route.c0[part];
  }
  const bool vec = (N & 3) == 0 && (ldd & 3) == 0;
#pragma unroll
  for (int j = 0; j < (BM * F4 + NT - 1) / NT; j++) {
    const int f = tid + NT * j, lr = f / F4, c4 = f % F4;
    const int row = m0 + lr, col = n0 + 4 * c4;
    if (f >= BM * F4 || row >= M || col >= N) continue;
    const float4 v4 = *(const float4 *)(Cs + lr * LDC + 4 * c4);
    float v[4] = {v4.x, v4.y, v4.z, v4.w};
    float *o = dst + (int64_t)row * ldd + (col - cbase);
    if (a.pairs) {  // N is a multiple of 4 and K is not split (the launcher sees to both)
      if (a.bias) {
        const float4 bb = *(const float4 *)(a.bias + col);
        v[0] += bb.x, v[1] += bb.y, v[2] += bb.z, v[3] += bb.w;
      }
      *(float2 *)(a.C + (int64_t)row * (N >> 1) + (col >> 1)) =
          make_float2(apply_act(CTHIP_ACT_SILU, v[0]) * v[1], apply_act(CTHIP_ACT_SILU, v[2]) * v[3]);
      continue;
    }
    if (vec) {
      if (!plain) {
        if (a.bias) {
          const float4 bb = *(const float4 *)(a.bias + col);
          v[0] += bb.x, v[1] += bb.y, v[2] += bb.z, v[3] += bb.w;
        }
#pragma unroll
        for (int t = 0; t < 4; t++) v[t] = apply_act(a.act, v[t]);
        if (a.residual) {
          const float4 rr = *(const float4 *)(a.residual + (int64_t)row * N + col);
          v[0] += rr.x, v[1] += rr.y, v[2] += rr.z, v[3] += rr.w;
        }
      }
      *(float4 *)o = make_float4(v[0], v[1], v[2], v[3]);
    } else {
      for (int t = 0; t < 4 && col + t < N; t++) {
        float x = v[t];
        if (!plain) {
          x = apply_act(a.act, x + (a.bias ? a.bias[col + t] : 0.0f));
          if (a.residual) x += a.residual[(int64_t)row * N + col + t];
        }
        o[t] = x;
      }
    }
  }
}

template <int BMODE, int NS, bool AL>
__global__ __launch_bounds__(768) void k_gemm_split(GemmArgs a) {
  constexpr int BM = 64, BN = 64, BK = 64, LDK = BK, NP = (NS == 1) ? 1 : (NS == 3) ? 2 : 3;
  constexpr int NSET = 3;  // register sets = K-steps of global loads in flight
  constexpr int kOpBytes = 2 * NP * BM * LDK * 2, kCBytes = BM * (BN + 4) * 4;
  // both operand buffers; after the last step the same memory holds the output tile (store_tile)
  __shared__ __align__(16) unsigned char smem[2 * kOpBytes > kCBytes ? 2 * kOpBytes : kCBytes];
  typedef unsigned short(*OpT)[NP][BM][LDK];
  OpT As = (OpT)smem, Bs = (OpT)(smem + kOpBytes);
  float *Cs = (float *)smem;
  // Twelve wavefronts in three roles, one of each per SIMD: 0..3 multiply the current step out of one LDS
  // buffer, 4..7 stage the next step's A into the other (and request the step three further on), 8..11 do the same
  // for B.  Each role runs its own loop (same number of barriers on every path), so a stager's waits count the
  // younger requests of ITS loop and the conversions run under the other wavefronts' matrix instructions.
  const int ltid = threadIdx.x, lane = ltid & 63;
  const int role = __builtin_amdgcn_readfirstlane(ltid) >> 8;  // uniform over a wavefront, and known to be
  const int tid = ltid & 255;                                  // index within the role
  const int wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
  const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
  if (local >= a.rm * a.rn) return;
  const int mi = (xcd % a.rx) * a.rm + local % a.rm, ni = (xcd / a.rx) * a.rn + local / a.rm;
  if (mi >= a.tm || ni >= a.tn) return;  // the regions overhang a grid they do not divide
  const int m0 = mi * BM, n0 = ni * BN;
  const int M = a.M, N = a.N, ldk = a.K;
  const int kbeg = blockIdx.y * a.kper;      // this workgroup's share of the reduction axis
  const int K = min(a.K, kbeg + a.kper);
  v16f acc;
#pragma unroll
  for (int r = 0; r < 16; r++) acc[r] = 0.0f;

  // A: thread -> rows ar + 16 i (i < 4), k = 4 akq .. +3
  const int ar = tid >> 4, akq = tid & 15;
  // B row-major (K,N): thread -> the 4x4 block k = 4 bkq + j, n = 4 bnq .. +3
  const int bkq = tid >> 4, bnq = tid & 15;
  // B packed (N rows of K): thread -> weight row wr, k = 16 wkc .. +15
  const int wr = tid >> 2, wkc = tid & 3;

  // requests without branches (see load4): outside the operands they read zeros
  auto fetch_a = [&](int k0, ARegs &ra) __attribute__((always_inline)) {  // k0 counts from kbeg
    auto ld = [&](int i) __attribute__((always_inline)) {
      const int row = m0 + ar + 16 * i, k = kbeg + k0 + 4 * akq;
      return load4<AL>(a.A + (int64_t)row * ldk + k, row < M ? clamp04(K - k) : 0);
    };
    ra.v0 = ld(0);
    ra.v1 = ld(1);
    ra.v2 = ld(2);
    ra.v3 = ld(3);
  };
  auto fetch_b = [&](int k0, BRegs<BMODE> &rb) __attribute__((always_inline)) {
    if (BMODE == W_ROWMAJOR) {
      auto ld = [&](int j) __attribute__((always_inline)) {
        const int k = kbeg + k0 + 4 * bkq + j, n = n0 + 4 * bnq;
        const float4 v = load4<AL>(a.B + (int64_t)k * N + n, k < K ? clamp04(N - n) : 0);
        return v4u{__float_as_uint(v.x), __float_as_uint(v.y), __float_as_uint(v.z), __float_as_uint(v.w)};
      };
      // constant indices only: the sets must stay in registers
      rb.v[0] = ld(0);
      rb.v[BRegs<BMODE>::NV > 1 ? 1 : 0] = ld(1);
      rb.v[BRegs<BMODE>::NV > 2 ? 2 : 0] = ld(2);
      rb.v[BRegs<BMODE>::NV > 3 ? 3 : 0] = ld(3);
    } else {
      // packed rows: K is a multiple of 16 here, so a 16-wide k chunk is inside the row or past its end
      const int n = n0 + wr, k = kbeg + k0 + 16 * wkc;
      const bool ok = n < N && k < K;
      const int64_t e = (int64_t)n * ldk + k;  // element index of the chunk
      if (BMODE == W_F32) {
        const v4u *src = ok ? (const v4u *)((const float *)a.wq + e) : (const v4u *)g_zeros;
        const int st = ok ? 1 : 0;  // the zeros are 32 bytes long
        rb.v[0] = src[0];
        rb.v[BRegs<BMODE>::NV > 1 ? 1 : 0] = src[st];
        rb.v[BRegs<BMODE>::NV > 2 ? 2 : 0] = src[2 * st];
        rb.v[BRegs<BMODE>::NV > 3 ? 3 : 0] = src[3 * st];
      } else if (BMODE == W_F16) {
        const v4u *src = ok ? (const v4u *)((const unsigned short *)a.wq + e) : (const v4u *)g_zeros;
        rb.v[0] = src[0];
        rb.v[BRegs<BMODE>::NV > 1 ? 1 : 0] = src[1];
      }
    }
  };
  auto stage_a = [&](const ARegs &ra, int buf) __attribute__((always_inline)) {
    auto put = [&](int i, const float4 v) __attribute__((always_inline)) {
      uint2 pl[NP];
      split4<NP>(v.x, v.y, v.z, v.w, pl);
#pragma unroll
      for (int p = 0; p < NP; p++)
        *(uint2 *)&As[buf][p][ar + 16 * i][8 * ((akq >> 1) ^ swz(ar + 16 * i)) + 4 * (akq & 1)] = pl[p];
    };
    put(0, ra.v0);
    put(1, ra.v1);
    put(2, ra.v2);
    put(3, ra.v3);
  };
  auto stage_b = [&](const BRegs<BMODE> &rb, int buf) __attribute__((always_inline)) {
    if (BMODE == W_ROWMAJOR) {
      // column 4 bnq + i gets its 4 consecutive k: a 4x4 transpose in registers
      auto put = [&](int i, unsigned x0, unsigned x1, unsigned x2, unsigned x3) __attribute__((always_inline)) {
        uint2 pl[NP];
        split4<NP>(__uint_as_float(x0), __uint_as_float(x1), __uint_as_float(x2), __uint_as_float(x3), pl);
#pragma unroll
        for (int p = 0; p < NP; p++)
          *(uint2 *)&Bs[buf][p][4 * bnq + i][8 * ((bkq >> 1) ^ swz(4 * bnq + i)) + 4 * (bkq & 1)] = pl[p];
      };
      const v4u q0 = rb.v[0], q1 = rb.v[BRegs<BMODE>::NV > 1 ? 1 : 0], q2 = rb.v[BRegs<BMODE>::NV > 2 ? 2 : 0], q3 = rb.v[BRegs<BMODE>::NV > 3 ? 3 : 0];
      put(0, q0.x, q1.x, q2.x, q3.x);
      put(1, q0.y, q1.y, q2.y, q3.y);
      put(2, q0.z, q1.z, q2.z, q3.z);
      put(3, q0.w, q1.w, q2.w, q3.w);
    } else {
      float x[16];
      if (BMODE == W_F32) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
          const v4u q = rb.v[j];
          x[4 * j + 0] = __uint_as_float(q.x);
          x[4 * j + 1] = __uint_as_float(q.y);
          x[4 * j + 2] = __uint_as_float(q.z);
          x[4 * j + 3] = __uint_as_float(q.w);
        }
      } else if (BMODE == W_F16) {
#pragma unroll
        for (int j = 0; j < 2; j++) {
          const v4u q = rb.v[BRegs<BMODE>::NV > 1 ? j : 0];
          const unsigned dw[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
          for (int t = 0; t < 4; t++) {
            x[8 * j + 2 * t] = half_bits_to_float((unsigned short)(dw[t] & 0xffff));
            x[8 * j + 2 * t + 1] = half_bits_to_float((unsigned short)(dw[t] >> 16));
          }
        }
      }
#pragma unroll
      for (int j = 0; j < 2; j++) {
        uint2 p0[NP], p1[NP];
        split4<NP>(x[8 * j], x[8 * j + 1], x[8 * j + 2], x[8 * j + 3], p0);
        split4<NP>(x[8 * j + 4], x[8 * j + 5], x[8 * j + 6], x[8 * j + 7], p1);
#pragma unroll
        for (int p = 0; p < NP; p++)
          *(uint4 *)&Bs[buf][p][wr][8 * ((2 * wkc + j) ^ swz(wr))] = make_uint4(p0[p].x, p0[p].y, p1[p].x, p1[p].y);
      }
    }
  };
  // all operand reads of a step are issued before its first matrix instruction: the matrix cores start when the
  // first operands arrive and the rest come in behind them (read-then-use pairs each wait out an LDS round trip)
  auto mma = [&](int buf) __attribute__((always_inline)) {
    // 32x32x16: lane l holds A[i = l%32][k = 8*(l/32) .. +7] and B[k = 8*(l/32) .. +7][j = l%32]
    const int rowa = 32 * wm + (lane & 31), rowb = 32 * wn + (lane & 31);
    v8bf av[BK / 16][NP], bv[BK / 16][NP];
#pragma unroll
    for (int s = 0; s < BK / 16; s++) {
      const int ch = 2 * s + (lane >> 5);
#pragma unroll
      for (int p = 0; p < NP; p++) {
        av[s][p] = __builtin_bit_cast(v8bf, *(const uint4 *)&As[buf][p][rowa][8 * (ch ^ swz(rowa))]);
        bv[s][p] = __builtin_bit_cast(v8bf, *(const uint4 *)&Bs[buf][p][rowb][8 * (ch ^ swz(rowb))]);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int s = 0; s < BK / 16; s++) {
      // every pair of planes whose product is above 2^-8(NP) of the leading one, smallest first
#pragma unroll
      for (int t = NP - 1; t >= 0; t--) {
#pragma unroll
        for (int p = 0; p <= t; p++) acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[s][p], bv[s][t - p], acc, 0, 0, 0);
      }
    }
  };
  const int nsteps = K > kbeg ? (K - kbeg + BK - 1) / BK : 0;
  // step i: LDS buffer i%2 holds it; register set (i+1) % NSET holds step i+1, requested NSET steps ago.
  // No conditions inside a staging step (past the last one the requests read zeros and stage them) and no exit
  // inside the loops: the waits before a set is staged then count on a known number of younger requests.
  static_assert(NSET == 3, "the loops below are unrolled by hand over the register sets");
  if (nsteps > 0) {  // K = 0 comes without operands
    if (role == 0) {
      __syncthreads();
      for (int i = 0; i < nsteps; i++) {
        mma(i & 1);
        __syncthreads();
      }
    } else if (role == 1) {
      ARegs ra0, ra1, ra2;  // separate objects with named members: every set stays in registers
      fetch_a(0, ra0);
      fetch_a(BK, ra1);
      fetch_a(2 * BK, ra2);
      stage_a(ra0, 0);
      fetch_a(3 * BK, ra0);
      __syncthreads();
      auto step = [&](int i, ARegs &ran) __attribute__((always_inline)) {
        stage_a(ran, (i + 1) & 1);
        fetch_a((i + 1 + NSET) * BK, ran);
        __syncthreads();
      };
      int i = 0;
      for (; i + NSET <= nsteps; i += NSET) {
        step(i, ra1);
        step(i + 1, ra2);
        step(i + 2, ra0);
      }
      if (i < nsteps) step(i, ra1);
      if (i + 1 < nsteps) step(i + 1, ra2);
    } else {
      BRegs<BMODE> rb0, rb1, rb2;
      fetch_b(0, rb0);
      fetch_b(BK, rb1);
      fetch_b(2 * BK, rb2);
      stage_b(rb0, 0);
      fetch_b(3 * BK, rb0);
      __syncthreads();
      auto step = [&](int i, BRegs<BMODE> &rbn) __attribute__((always_inline)) {
        stage_b(rbn, (i + 1) & 1);
        fetch_b((i + 1 + NSET) * BK, rbn);
        __syncthreads();
      };
      int i = 0;
      for (; i + NSET <= nsteps; i += NSET) {
        step(i, rb1);
        step(i + 1, rb2);
        step(i + 2, rb0);
      }
      if (i < nsteps) step(i, rb1);
      if (i + 1 < nsteps) step(i + 1, rb2);
    }
  }
  // ---- epilogue: acc[r] is C[row = 8*(r/4) + 4*(l/32) + r%4][col = l%32] of the 32x32 sub-tile ----
  // (the last step ended with a barrier: nobody reads the operand buffers any more)
  if (role == 0) {
#pragma unroll
    for (int r = 0; r < 16; r++)
      Cs[(32 * wm + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3)) * (BN + 4) + 32 * wn + (lane & 31)] = acc[r];
  }
  __syncthreads();
  store_tile<BM, BN, 768>(a, Cs, m0, n0, ltid);
}

// ---------------------------------------------------------------------------------------------
// Linear over m rows with Q8_0 / Q4_0 weights: the dequantisation is fused into the accumulation.
//
// A quantised weight is q * d with q a small integer (int8, or nibble - 8) and d the fp16 scale of its
// block of 32.  Every such q is exact in bf16, so the matrix cores multiply the activations (split in
// NPA bf16 terms: 1 = rounded, 2 = 2^-17 per product, 3 = all 24 bits) by the INTEGER plane -- one
// MFMA per activation term and k-slice, exact products, fp32 sums over the 32 weights of a block --
// and the block's scale is applied once to that partial sum:  acc += d[n][block] * (sum_k a[m][k] q[n][k]).
// Against dequantising to fp32 and splitting both operands this needs a third fewer MFMAs, an eighth
// of the conversion work on the weight side, and is more accurate (no rounding of q * d).
//
// K is walked in steps of 64 = two quant blocks, with the LDS layout / swizzle / prefetch depth / XCD regions /
// split-K of k_gemm_split.
template <int NA>
struct ARegsQ {  // one K-step of A held by a staging thread: NA 16-byte pieces
  float4 v[NA];
};

// two small integers (as floats, exact) -> packed bf16 pair, x0 in the low half
__device__ __forceinline__ unsigned pack_int_bf16(float x0, float x1) {
  return __builtin_amdgcn_perm(__float_as_uint(x1), __float_as_uint(x0), 0x07060302u);  // high halves of both
}

// ---------------------------------------------------------------------------------------------
// The two halves of a K-step are done by different wavefronts of a 512-thread workgroup.
//
// When every wavefront stages (conversions on the vector ALU, LDS writes), then multiplies (LDS reads, matrix
// cores, block scales on the vector ALU), then meets the others at a barrier, nothing overlaps with one or two
// wavefronts per SIMD: a step of 64 took 0.7-1.1 us and the matrix cores were busy an eighth of the time.
// Here wavefronts 4..7 only stage the NEXT step (and request the one three further on) while wavefronts 0..3
// only multiply the CURRENT one out of the other LDS buffer, so every SIMD holds one of each and the waits of
// one half are filled by the other.  (Measured with in-kernel timestamps on 512 x 3072 x 768: matrix
// instructions and vector instructions of a SIMD do not issue side by side, so a step costs the sum of both
// halves' instructions, about 0.95 us; what the split removes is the exposed latency between the phases.)
// The tile is 64 x 128 (a multiplying wavefront owns 32 x 64 = two accumulator blocks against one A operand),
// which keeps both halves about equally long and gives the prefill shapes no more workgroups than compute units.
// Weight bytes become floats with one sign-extending conversion each (sbyteN_f32) and pairs of them bf16 with
// one byte permute.
template <int NB>
struct BRegsQ2 {
  uint4 v[NB];       // 16 weights each: units ptid + PT j of the tile's 128 rows x 4 pieces
  unsigned short d;  // fp16 scale bits: row ptid >> 1, block ptid & 1 of the step
};

// FULL: every tile and every K-step of the launch lies inside the operands and their byte offsets fit 32 bits
// (the launcher checks).  The requests of a step are then a scalar base, advanced per step on the scalar unit,
// plus per-thread offsets computed once -- no address arithmetic, bounds tests or selects on the vector unit,
// which the staging wavefronts share with the scale multiplications of the multiplying ones.
template <int WT, int NPA, int NPW, bool FULL>
__global__ __launch_bounds__(256 + 64 * NPW) void k_gemm_qpc(GemmArgs a) {
  constexpr int PT = 64 * NPW, NT = 256 + PT;  // staging threads, all threads
  constexpr int NA = 1024 / PT, NB = 512 / PT;  // 16-byte pieces of A / of the weights per staging thread and step
  constexpr int BM = 64, BN = 128, BK = 64, LDK = BK, LDC = BN + 4;
  constexpr int kABytes = 2 * NPA * BM * LDK * 2, kBBytes = 2 * BN * LDK * 2, kCBytes = BM * LDC * 4;
  // the operand buffers; after the last step the same memory holds the output tile for the row-wise stores
  __shared__ __align__(16) unsigned char smem[(kABytes + kBBytes > kCBytes) ? kABytes + kBBytes : kCBytes];
  __shared__ float Ss[2][BN][2];
  typedef unsigned short(*AsT)[NPA][BM][LDK];
  typedef unsigned short(*BsT)[BN][LDK];
  AsT As = (AsT)smem;
  BsT Bs = (BsT)(smem + kABytes);
  float(*Cs)[LDC] = (float(*)[LDC])smem;
  const int tid = threadIdx.x, lane = tid & 63;
  const bool producer = __builtin_amdgcn_readfirstlane(tid) >= 256;  // uniform over a wavefront, and known to be
  const int ptid = producer ? tid - 256 : tid;  // staging role: index among the staging threads
  const int wave = (tid >> 6) & 3;       // multiplying role: 2 x 2 wavefronts of 32 x 64
  const int wm = wave >> 1, wn = wave & 1;
  const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
  if (local >= a.rm * a.rn) return;
  const int mi = (xcd % a.rx) * a.rm + local % a.rm, ni = (xcd / a.rx) * a.rn + local / a.rm;
  if (mi >= a.tm || ni >= a.tn) return;
  const int m0 = mi * BM, n0 = ni * BN;
  const int M = a.M, N = a.N, ldk = a.K;
  const int kbeg = blockIdx.y * a.kper;
  const int K = min(a.K, kbeg + a.kper);
  v16f acc[2];
#pragma unroll
  for (int b = 0; b < 2; b++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[b][r] = 0.0f;

  const int ar = ptid >> 4, akq = ptid & 15;  // A: rows ar + (PT / 16) i, k = 4 akq .. +3
  const int wr = ptid >> 2, wkc = ptid & 3;   // B: weight rows wr + (PT / 4) j, k = 16 wkc .. +15
  const int sr = (ptid & 255) >> 1, sb = ptid & 1;  // scales: row sr, quant block sb of the step (first 256 stagers)
  const bool scaler = ptid < 256;
  const int blocks_per_row = ldk >> 5;
  const int nsteps = K > kbeg ? (K - kbeg + BK - 1) / BK : 0;
  unsigned aoff[NA], boff[NB], soff;  // FULL: byte offsets of this thread's pieces from the step's bases
#pragma unroll
  for (int i = 0; i < NA; i++) aoff[i] = 4u * ((unsigned)(m0 + ar + (PT / 16) * i) * (unsigned)ldk + 4u * akq);
#pragma unroll
  for (int j = 0; j < NB; j++) {
    const unsigned e = (unsigned)(n0 + wr + (PT / 4) * j) * (unsigned)ldk;
    boff[j] = WT == W_Q8 ? e + 16u * wkc : ((e >> 5) << 4) + ((wkc >> 1) << 4);
  }
  soff = 2u * ((unsigned)(n0 + sr) * (unsigned)blocks_per_row + sb);

  typedef ARegsQ<NA> ARg;
  typedef BRegsQ2<NB> BRg;
  auto fetch = [&](int k0, ARg &ra, BRg &rb) {  // k0 counts from kbeg; requests without branches
    if constexpr (FULL) {
      const int kk = kbeg + min(k0, (nsteps - 1) * BK);  // steps past the end ask for the last one again
      const char *ab = (const char *)(a.A + kk);
      const char *bb = (const char *)a.wq + (WT == W_Q8 ? kk : ((kk >> 5) << 4));
      const char *sbase = (const char *)a.wd + ((kk >> 5) << 1);
#pragma unroll
      for (int i = 0; i < NA; i++) ra.v[i] = *(const float4 *)(ab + aoff[i]);
#pragma unroll
      for (int j = 0; j < NB; j++) rb.v[j] = *(const uint4 *)(bb + boff[j]);
      rb.d = *(const unsigned short *)(sbase + soff);
      return;
    }
#pragma unroll
    for (int i = 0; i < NA; i++) {
      const int row = m0 + ar + (PT / 16) * i, k = kbeg + k0 + 4 * akq;
      ra.v[i] = load4<true>(a.A + (int64_t)row * ldk + k, row < M ? clamp04(K - k) : 0);
    }
    const int k = kbeg + k0 + 16 * wkc;
#pragma unroll
    for (int j = 0; j < NB; j++) {
      const int n = n0 + wr + (PT / 4) * j;
      const int64_t e = (int64_t)n * ldk + k;
      const uint8_t *q = (const uint8_t *)a.wq + (WT == W_Q8 ? e : ((e >> 5) << 4));
      rb.v[j] = *((n < N && k < K) ? (const uint4 *)q : (const uint4 *)g_zeros);
    }
    const int ns = n0 + sr, ks = kbeg + k0 + 32 * sb;
    rb.d = *((ns < N && ks < K) ? a.wd + (int64_t)ns * blocks_per_row + (ks >> 5) : (const unsigned short *)g_zeros);
  };
  auto stage = [&](const ARg &ra, const BRg &rb, int buf) {
#pragma unroll
    for (int i = 0; i < NA; i++) {
      const float x[4] = {ra.v[i].x, ra.v[i].y, ra.v[i].z, ra.v[i].w};
      uint2 pl[NPA];
      split4<NPA>(x[0], x[1], x[2], x[3], pl);
      const int row = ar + (PT / 16) * i;
#pragma unroll
      for (int p = 0; p < NPA; p++) *(uint2 *)&As[buf][p][row][8 * ((akq >> 1) ^ swz(row)) + 4 * (akq & 1)] = pl[p];
    }
#pragma unroll
    for (int jr = 0; jr < NB; jr++) {
      float q[16];
      const unsigned dw[4] = {rb.v[jr].x, rb.v[jr].y, rb.v[jr].z, rb.v[jr].w};
      if (WT == W_Q8) {
#pragma unroll
        for (int t = 0; t < 4; t++) {
          q[4 * t + 0] = sbyte0_f32(dw[t]);
          q[4 * t + 1] = sbyte1_f32(dw[t]);
          q[4 * t + 2] = sbyte2_f32(dw[t]);
          q[4 * t + 3] = sbyte3_f32(dw[t]);
        }
      } else {
        // chunks 0, 2 of the step are the low nibbles of their block, 1, 3 the high
#pragma unroll
        for (int t = 0; t < 4; t++) {
          const unsigned nb = ((wkc & 1) ? dw[t] >> 4 : dw[t]) & 0x0f0f0f0fu;
          q[4 * t + 0] = ubyte0_f32(nb) - 8.0f;
          q[4 * t + 1] = ubyte1_f32(nb) - 8.0f;
          q[4 * t + 2] = ubyte2_f32(nb) - 8.0f;
          q[4 * t + 3] = ubyte3_f32(nb) - 8.0f;
        }
      }
      const int row = wr + (PT / 4) * jr;
#pragma unroll
      for (int j = 0; j < 2; j++)
        *(uint4 *)&Bs[buf][row][8 * ((2 * wkc + j) ^ swz(row))] =
            make_uint4(pack_int_bf16(q[8 * j + 0], q[8 * j + 1]), pack_int_bf16(q[8 * j + 2], q[8 * j + 3]),
                       pack_int_bf16(q[8 * j + 4], q[8 * j + 5]), pack_int_bf16(q[8 * j + 6], q[8 * j + 7]));
    }
    if (scaler) Ss[buf][sr][sb] = half_bits_to_float(rb.d);  // uniform over a wavefront
  };
  // The operand reads of a whole step are issued before its first matrix instruction (left to itself the
  // compiler puts each read right before its use, and every pair of matrix instructions then waits out an LDS
  // round trip): the matrix cores start when the first operands arrive and the rest come in behind them.
  auto mma = [&](int buf) {
    const int rowa = 32 * wm + (lane & 31);
    v8bf av[2][2][NPA], bv[2][2][2];  // [quant block][k-slice][term / accumulator block]
    float d[2][2];
#pragma unroll
    for (int kb = 0; kb < 2; kb++)
#pragma unroll
      for (int s2 = 0; s2 < 2; s2++) {
        const int ch = 4 * kb + 2 * s2 + (lane >> 5);
#pragma unroll
        for (int p = 0; p < NPA; p++) av[kb][s2][p] = __builtin_bit_cast(v8bf, *(const uint4 *)&As[buf][p][rowa][8 * (ch ^ swz(rowa))]);
#pragma unroll
        for (int b = 0; b < 2; b++) {
          const int rowb = 64 * wn + 32 * b + (lane & 31);
          bv[kb][s2][b] = __builtin_bit_cast(v8bf, *(const uint4 *)&Bs[buf][rowb][8 * (ch ^ swz(rowb))]);
        }
      }
#pragma unroll
    for (int b = 0; b < 2; b++) {
      const float2 dd = *(const float2 *)&Ss[buf][64 * wn + 32 * b + (lane & 31)][0];  // this lane's output column
      d[0][b] = dd.x, d[1][b] = dd.y;
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int kb = 0; kb < 2; kb++) {  // the two quant blocks of the step
      v16f tmp[2];
#pragma unroll
      for (int b = 0; b < 2; b++)
#pragma unroll
        for (int r = 0; r < 16; r++) tmp[b][r] = 0.0f;
#pragma unroll
      for (int s2 = 0; s2 < 2; s2++)
#pragma unroll
        for (int b = 0; b < 2; b++)
#pragma unroll
          for (int p = NPA - 1; p >= 0; p--) tmp[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[kb][s2][p], bv[kb][s2][b], tmp[b], 0, 0, 0);
#pragma unroll
      for (int b = 0; b < 2; b++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[b][r] = fmaf(d[kb][b], tmp[b][r], acc[b][r]);
    }
  };

  ARg ra0, ra1, ra2;
  BRg rb0, rb1, rb2;
  // One barrier per step.  Each role runs its own loop, so the staging loop has no branch around its requests:
  // with the role tested inside a shared loop the compiler has to assume the path on which a step's requests
  // were skipped, waits for ALL but the last requests before every use, and the three-steps-ahead prefetch
  // degenerates into one step ahead (each step then costs a memory round trip).  Every wavefront passes the
  // same number of barriers on either path.
  if (nsteps > 0) {
    if (producer) {
      fetch(0, ra0, rb0);
      fetch(BK, ra1, rb1);
      fetch(2 * BK, ra2, rb2);
      stage(ra0, rb0, 0);
      fetch(3 * BK, ra0, rb0);
      __syncthreads();
      auto step = [&](int i, ARg &ran, BRg &rbn) {
        stage(ran, rbn, (i + 1) & 1);
        fetch((i + 4) * BK, ran, rbn);
        __syncthreads();
      };
      int i = 0;
      for (; i + 3 <= nsteps; i += 3) {
        step(i, ra1, rb1);
        step(i + 1, ra2, rb2);
        step(i + 2, ra0, rb0);
      }
      if (i < nsteps) step(i, ra1, rb1);
      if (i + 1 < nsteps) step(i + 1, ra2, rb2);
    } else {
      __syncthreads();
      for (int i = 0; i < nsteps; i++) {
        mma(i & 1);
        __syncthreads();
      }
    }
  }
  // ---- epilogue: acc[b][r] is C[row = 8*(r/4) + 4*(l/32) + r%4][col = l%32] of the wavefront's block b.  The
  // tile goes through LDS (the operand buffers are free after the last barrier) so that all 512 threads store
  // whole rows: 16-byte stores, bias and residual read the same way.
  if (!producer) {
#pragma unroll
    for (int b = 0; b < 2; b++)
#pragma unroll
      for (int r = 0; r < 16; r++)
        Cs[32 * wm + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3)][64 * wn + 32 * b + (lane & 31)] = acc[b][r];
  }
  __syncthreads();
  store_tile<BM, BN, NT>(a, &Cs[0][0], m0, n0, tid);
}

// ---------------------------------------------------------------------------------------------
// fp32-operand MFMA GEMM (v_mfma_f32_32x32x2_f32): the products are fp32 products, only the summation
// order differs from a scalar loop.  This kernel takes PACKED WEIGHTS (N rows x K, any of the five formats,
// dequantised to fp32 while staging); a (K,N) fp32 matrix takes k_gemm_f32pc below.  64x64 tile per 256-thread
// workgroup, 2x2 wavefronts, two LDS buffers, three register sets of global loads in flight, one barrier per
// step, XCD regions, split-K, K-steps of 32, the operands kept as fp32 in LDS, k-major ([k][m], [k][n]):
// lane l of a wavefront reads A[row l%32][k = 2s + l/32] and B[k = 2s + l/32][col l%32], i.e. 32
// consecutive floats per half-wavefront.  A and the weights arrive k-contiguous and are transposed by
// the staging writes.
struct FRegsA {
  float4 v0, v1;  // units tid and tid + 256 of the 64 x 8 float4 of a K-step
};
struct FRegsB {
  uint4 r0, r1;      // packed weights: the raw bytes of 8 consecutive k of one row; row-major B: two float4 (rows k, k + 2)
  unsigned short d;  // block scale (quantised weights)
};

template <bool AL>
__global__ __launch_bounds__(256) void k_gemm_f32(GemmArgs a) {
  // odd row pitches: the staging writes are transposing scalar writes (k varies fastest over the lanes, so
  // k * pitch has to spread over the banks)
  constexpr int BM = 64, BN = 64, BK = 32, LDA = BM + 1, LDB = BN + 1;
  constexpr int kABytes = 2 * BK * LDA * 4, kBBytes = 2 * BK * LDB * 4, kCBytes = BM * (BN + 4) * 4;
  __shared__ __align__(16) unsigned char smem[kABytes + kBBytes > kCBytes ? kABytes + kBBytes : kCBytes];
  float(*As)[BK][LDA] = (float(*)[BK][LDA])smem;
  float(*Bs)[BK][LDB] = (float(*)[BK][LDB])(smem + kABytes);
  float *Cs = (float *)smem;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
  if (local >= a.rm * a.rn) return;
  const int mi = (xcd % a.rx) * a.rm + local % a.rm, ni = (xcd / a.rx) * a.rn + local / a.rm;
  if (mi >= a.tm || ni >= a.tn) return;
  const int m0 = mi * BM, n0 = ni * BN;
  const int M = a.M, N = a.N, ldk = a.K;
  const int kbeg = blockIdx.y * a.kper;
  const int K = min(a.K, kbeg + a.kper);
  v16f acc;
#pragma unroll
  for (int r = 0; r < 16; r++) acc[r] = 0.0f;

  auto load_a = [&](int u, int k0) {  // unit u: row u / 8, k = 4 (u % 8) .. +3
    const int row = m0 + (u >> 3), k = kbeg + k0 + 4 * (u & 7);
    return load4<AL>(a.A + (int64_t)row * ldk + k, row < M ? clamp04(K - k) : 0);
  };
  auto fetch = [&](int k0, FRegsA &ra, FRegsB &rb) {
    ra.v0 = load_a(tid, k0);
    ra.v1 = load_a(tid + 256, k0);
    rb.r0 = rb.r1 = make_uint4(0u, 0u, 0u, 0u);
    rb.d = 0;
    {
      // packed weights: weight row tid / 4, k = 8 (tid % 4) .. +7 of the step.  AL: rows are a multiple of 8
      // wide (quantised rows always are), so the 8 are inside the row or past its end
      const int n = n0 + (tid >> 2), k = kbeg + k0 + 8 * (tid & 3);
      const bool in = n < N && k < K;
      const int64_t e = (int64_t)n * ldk + k;
      const void *z = g_zeros;
      if (!AL) {
        // fp32 / fp16 rows of any width: element loads, zeros past the end of the row
        unsigned x[8];
#pragma unroll
        for (int t = 0; t < 8; t++) {
          const bool ok = in && k + t < K;
          x[t] = a.wtype == CTHIP_F32 ? *(ok ? (const unsigned *)a.wq + e + t : (const unsigned *)z)
                                      : *(ok ? (const unsigned short *)a.wq + e + t : (const unsigned short *)z);
        }
        if (a.wtype == CTHIP_F32) {
          rb.r0 = make_uint4(x[0], x[1], x[2], x[3]);
          rb.r1 = make_uint4(x[4], x[5], x[6], x[7]);
        } else {
          rb.r0 = make_uint4(x[0] | (x[1] << 16), x[2] | (x[3] << 16), x[4] | (x[5] << 16), x[6] | (x[7] << 16));
        }
      } else if (a.wtype == CTHIP_F32) {
        const uint4 *src = in ? (const uint4 *)((const float *)a.wq + e) : (const uint4 *)z;
        rb.r0 = src[0];
        rb.r1 = src[1];
      } else if (a.wtype == CTHIP_F16) {
        rb.r0 = *(in ? (const uint4 *)((const unsigned short *)a.wq + e) : (const uint4 *)z);
      } else {
        // Q8_0: 8 int8.  Q4_0: elements j < 16 of a block are the low nibbles of its bytes j, j >= 16 the high
        // nibbles of bytes j - 16 -- 8 bytes from (k % 16) on either way
        const uint8_t *q = (const uint8_t *)a.wq + (a.wtype == CTHIP_Q8_0 ? e : ((e >> 5) << 4) + (k & 15));
        const uint2 v = *(in ? (const uint2 *)q : (const uint2 *)z);
        rb.r0.x = v.x;
        rb.r0.y = v.y;
        rb.d = *(in ? a.wd + (e >> 5) : (const unsigned short *)z);
      }
    }
  };
  auto put_a = [&](int u, const float4 v, int buf) {
    const int row = u >> 3, k = 4 * (u & 7);
    As[buf][k + 0][row] = v.x;
    As[buf][k + 1][row] = v.y;
    As[buf][k + 2][row] = v.z;
    As[buf][k + 3][row] = v.w;
  };
  auto stage = [&](const FRegsA &ra, const FRegsB &rb, int buf) {
    put_a(tid, ra.v0, buf);
    put_a(tid + 256, ra.v1, buf);
    {
      float w0, w1, w2, w3, w4, w5, w6, w7;
      if (a.wtype == CTHIP_F32) {
        w0 = __uint_as_float(rb.r0.x), w1 = __uint_as_float(rb.r0.y), w2 = __uint_as_float(rb.r0.z), w3 = __uint_as_float(rb.r0.w);
        w4 = __uint_as_float(rb.r1.x), w5 = __uint_as_float(rb.r1.y), w6 = __uint_as_float(rb.r1.z), w7 = __uint_as_float(rb.r1.w);
      } else if (a.wtype == CTHIP_F16) {
        w0 = half_bits_to_float((unsigned short)(rb.r0.x & 0xffff)), w1 = half_bits_to_float((unsigned short)(rb.r0.x >> 16));
        w2 = half_bits_to_float((unsigned short)(rb.r0.y & 0xffff)), w3 = half_bits_to_float((unsigned short)(rb.r0.y >> 16));
        w4 = half_bits_to_float((unsigned short)(rb.r0.z & 0xffff)), w5 = half_bits_to_float((unsigned short)(rb.r0.z >> 16));
        w6 = half_bits_to_float((unsigned short)(rb.r0.w & 0xffff)), w7 = half_bits_to_float((unsigned short)(rb.r0.w >> 16));
      } else if (a.wtype == CTHIP_Q8_0) {
        const float d = half_bits_to_float(rb.d);
        const int v0 = (int)rb.r0.x, v1 = (int)rb.r0.y;
        w0 = (float)(int)(int8_t)(v0)*d, w1 = (float)(int)(int8_t)(v0 >> 8) * d;
        w2 = (float)(int)(int8_t)(v0 >> 16) * d, w3 = (float)(v0 >> 24) * d;
        w4 = (float)(int)(int8_t)(v1)*d, w5 = (float)(int)(int8_t)(v1 >> 8) * d;
        w6 = (float)(int)(int8_t)(v1 >> 16) * d, w7 = (float)(v1 >> 24) * d;
      } else {
        const float d = half_bits_to_float(rb.d);
        // k = 8 (tid % 4) within the block: from 16 on the elements are the high nibbles
        const unsigned sh = ((tid & 3) >= 2) ? 4u : 0u;
        const unsigned v0 = rb.r0.x >> sh, v1 = rb.r0.y >> sh;
        w0 = (float)((int)(v0 & 0xf) - 8) * d, w1 = (float)((int)((v0 >> 8) & 0xf) - 8) * d;
        w2 = (float)((int)((v0 >> 16) & 0xf) - 8) * d, w3 = (float)((int)((v0 >> 24) & 0xf) - 8) * d;
        w4 = (float)((int)(v1 & 0xf) - 8) * d, w5 = (float)((int)((v1 >> 8) & 0xf) - 8) * d;
        w6 = (float)((int)((v1 >> 16) & 0xf) - 8) * d, w7 = (float)((int)((v1 >> 24) & 0xf) - 8) * d;
      }
      const int n = tid >> 2, k = 8 * (tid & 3);
      Bs[buf][k + 0][n] = w0, Bs[buf][k + 1][n] = w1, Bs[buf][k + 2][n] = w2, Bs[buf][k + 3][n] = w3;
      Bs[buf][k + 4][n] = w4, Bs[buf][k + 5][n] = w5, Bs[buf][k + 6][n] = w6, Bs[buf][k + 7][n] = w7;
    }
  };
  // operands of matrix instructions 2j, 2j + 1 of a step (lane l: k = 4j + l/32 and 4j + 2 + l/32)
  auto rd = [&](int buf, int j, float (&av)[2], float (&bv)[2]) {
#pragma unroll
    for (int t = 0; t < 2; t++) {
      const int kk = 4 * j + 2 * t + (lane >> 5);
      av[t] = As[buf][kk][32 * wm + (lane & 31)];
      bv[t] = Bs[buf][kk][32 * wn + (lane & 31)];
    }
  };

  FRegsA ra0, ra1, ra2;
  FRegsB rb0, rb1, rb2;
  const int nsteps = K > kbeg ? (K - kbeg + BK - 1) / BK : 0;
  // no conditions inside a step: past the last step the requests read zeros and stage them
  // A wavefront issues in order and a matrix instruction holds the pipe for 64 cycles.  The step is laid out by
  // hand between scheduling fences: the operand reads run one pair of matrix instructions ahead of their use,
  // the next step's staging and the requests four steps ahead sit between pairs.
  auto step = [&](int i, FRegsA &ran, FRegsB &rbn) {
    const int buf = i & 1;
    float av[2][2], bv[2][2];
    rd(buf, 0, av[0], bv[0]);
#pragma unroll
    for (int j = 0; j < BK / 4; j++) {
      if (j + 1 < BK / 4) rd(buf, j + 1, av[(j + 1) & 1], bv[(j + 1) & 1]);
      if (j == 1) stage(ran, rbn, buf ^ 1);
      if (j == 4) fetch((i + 4) * BK, ran, rbn);
      __builtin_amdgcn_sched_barrier(0);
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av[j & 1][0], bv[j & 1][0], acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av[j & 1][1], bv[j & 1][1], acc, 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();
  };
  if (nsteps > 0) {  // K = 0 comes without operands
    fetch(0, ra0, rb0);
    fetch(BK, ra1, rb1);
    fetch(2 * BK, ra2, rb2);
    stage(ra0, rb0, 0);
    fetch(3 * BK, ra0, rb0);
    __syncthreads();
    int i = 0;
    for (; i + 3 <= nsteps; i += 3) {  // no exit inside: the waits at the top count on a known number of requests
      step(i, ra1, rb1);
      step(i + 1, ra2, rb2);
      step(i + 2, ra0, rb0);
    }
    if (i < nsteps) step(i, ra1, rb1);
    if (i + 1 < nsteps) step(i + 1, ra2, rb2);
  }
  // ---- epilogue: acc[r] is C[row = 8*(r/4) + 4*(l/32) + r%4][col = l%32] of the 32x32 sub-tile ----
  // (the last step ended with a barrier: nobody reads the operand buffers any more)
#pragma unroll
  for (int r = 0; r < 16; r++)
    Cs[(32 * wm + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3)) * (BN + 4) + 32 * wn + (lane & 31)] = acc[r];
  __syncthreads();
  store_tile<BM, BN, 256>(a, Cs, m0, n0, tid);
}

// ---------------------------------------------------------------------------------------------
// The same product with the roles of a step split over wavefronts, as in k_gemm_split: 768 threads, wavefronts
// 0..3 only multiply, 4..7 only stage A, 8..11 only stage B (one loop per role, one barrier per step).
//
// One wavefront per SIMD issues an instruction every 8 cycles or so: with every wavefront staging, requesting and
// multiplying, a step's hundred-odd other instructions did not fit behind its 16 matrix instructions (64 cycles
// each) and a step took 1950 cycles instead of 1024.  Here a multiplying wavefront issues nothing but its matrix
// instructions and the operand reads of the NEXT step (a second register set; the operands of an fp32 matrix
// instruction are one register each), which needs three LDS buffers: in step i the staging wavefronts fill
// buffer (i + 2) % 3 while the multiplying ones read buffer (i + 1) % 3 and compute from registers.
//
// LDS layout: plane p = 2 (k / 4) + (k % 2) holds, for every row, the PAIR (k, k + 2) -- what a lane (row l % 32,
// half l / 32) feeds to the two matrix instructions 2j, 2j + 1 of a step is the 8 bytes [plane 2j + l / 32][row],
// and a staging thread that holds 4 consecutive k of a row writes two such pairs.
//
// FULL (the launcher checks): every tile and every K-step of the launch lies inside the operands and their byte
// offsets fit 32 bits.  A step's requests are then a scalar base, advanced on the scalar unit, plus per-thread
// offsets computed once -- no address arithmetic, bounds tests or selects on the vector unit, which the staging
// wavefronts share with the multiplying one of their SIMD.  B is (K,N) row-major here; packed weights (N,K) keep
// k_gemm_f32, which measured faster on the prompt shapes.
template <bool AL, bool FULL>
__global__ __launch_bounds__(768) void k_gemm_f32pc(GemmArgs a) {
  constexpr int BM = 64, BN = 64, BK = 32, NP = BK / 2;
  // plane pitches in floats: a multiple of 4 where the staging writes are 16 bytes (B), else 8-byte aligned
  constexpr int PA = 2 * BM + 2, PB = 2 * BN + 4;
  constexpr int kABuf = NP * PA * 4, kBBuf = NP * PB * 4;  // bytes per buffer
  constexpr int kABytes = 3 * kABuf, kBBytes = 3 * kBBuf, kCBytes = BM * (BN + 4) * 4;
  __shared__ __align__(16) unsigned char smem[kABytes + kBBytes > kCBytes ? kABytes + kBBytes : kCBytes];
  float *Cs = (float *)smem;
  const int tid = threadIdx.x, lane = tid & 63;
  const int role = __builtin_amdgcn_readfirstlane(tid) >> 8;  // 0 multiply, 1 stage A, 2 stage B: uniform over a wavefront
  const int t = tid & 255;                                    // index within the role
  const int wave = t >> 6, wm = wave >> 1, wn = wave & 1;
  const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
  if (local >= a.rm * a.rn) return;
  const int mi = (xcd % a.rx) * a.rm + local % a.rm, ni = (xcd / a.rx) * a.rn + local / a.rm;
  if (mi >= a.tm || ni >= a.tn) return;
  const int m0 = mi * BM, n0 = ni * BN;
  const int M = a.M, N = a.N, ldk = a.K;
  const int kbeg = blockIdx.y * a.kper;
  const int K = min(a.K, kbeg + a.kper);
  const int nsteps = K > kbeg ? (K - kbeg + BK - 1) / BK : 0;
  v16f acc;
#pragma unroll
  for (int r = 0; r < 16; r++) acc[r] = 0.0f;

  if (nsteps > 0) {  // K = 0 comes without operands
    if (role == 0) {
      // ---- multiply: registers of step i were read during step i - 1
      const unsigned abase = 4u * (unsigned)((lane >> 5) * PA + 2 * (32 * wm + (lane & 31)));
      const unsigned bbase = (unsigned)kABytes + 4u * (unsigned)((lane >> 5) * PB + 2 * (32 * wn + (lane & 31)));
      auto rd = [&](int buf, float2(&av)[8], float2(&bv)[8]) __attribute__((always_inline)) {
        const unsigned char *pa = smem + abase + (unsigned)buf * kABuf, *pb = smem + bbase + (unsigned)buf * kBBuf;
#pragma unroll
        for (int j = 0; j < 8; j++) {
          av[j] = *(const float2 *)(pa + j * (2 * PA * 4));
          bv[j] = *(const float2 *)(pb + j * (2 * PB * 4));
        }
      };
      // the next step's reads are spread between this step's pairs of matrix instructions
      auto step = [&](int nbuf, const float2(&av)[8], const float2(&bv)[8], float2(&an)[8], float2(&bn)[8]) __attribute__((always_inline)) {
        const unsigned char *pa = smem + abase + (unsigned)nbuf * kABuf, *pb = smem + bbase + (unsigned)nbuf * kBBuf;
#pragma unroll
        for (int j = 0; j < 8; j++) {
          an[j] = *(const float2 *)(pa + j * (2 * PA * 4));
          bn[j] = *(const float2 *)(pb + j * (2 * PB * 4));
          __builtin_amdgcn_sched_barrier(0);
          acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av[j].x, bv[j].x, acc, 0, 0, 0);
          acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av[j].y, bv[j].y, acc, 0, 0, 0);
          __builtin_amdgcn_sched_barrier(0);
        }
        __syncthreads();
      };
      float2 a0[8], b0[8], a1[8], b1[8];
      __syncthreads();  // steps 0 and 1 are staged
      rd(0, a0, b0);
      int nb = 1;  // buffer of the step after the current one
      int i = 0;
      for (; i + 2 <= nsteps; i += 2) {
        step(nb, a0, b0, a1, b1);
        nb = nb == 2 ? 0 : nb + 1;
        step(nb, a1, b1, a0, b0);
        nb = nb == 2 ? 0 : nb + 1;
      }
      if (i < nsteps) step(nb, a0, b0, a1, b1);
    } else if (role == 1) {
      // ---- stage A: units t and t + 256 of the 64 rows x 8 groups of 4 consecutive k
      unsigned aoff[2];
#pragma unroll
      for (int h = 0; h < 2; h++) aoff[h] = 4u * ((unsigned)(m0 + ((t + 256 * h) >> 3)) * (unsigned)ldk + 4u * (unsigned)(t & 7));
      auto fetch = [&](int k0, FRegsA &ra) __attribute__((always_inline)) {
        if constexpr (FULL) {
          const char *ab = (const char *)(a.A + kbeg + min(k0, (nsteps - 1) * BK));  // steps past the end ask for the last one again
          ra.v0 = *(const float4 *)(ab + aoff[0]);
          ra.v1 = *(const float4 *)(ab + aoff[1]);
          return;
        }
#pragma unroll
        for (int h = 0; h < 2; h++) {
          const int u = t + 256 * h, row = m0 + (u >> 3), k = kbeg + k0 + 4 * (u & 7);
          const float4 v = load4<AL>(a.A + (int64_t)row * ldk + k, row < M ? clamp04(K - k) : 0);
          if (h == 0) ra.v0 = v;
          else ra.v1 = v;
        }
      };
      auto stage = [&](const FRegsA &ra, int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int h = 0; h < 2; h++) {
          const int u = t + 256 * h, row = u >> 3, g = u & 7;
          const float4 v = h == 0 ? ra.v0 : ra.v1;
          float *p = (float *)(smem + buf * kABuf) + 2 * g * PA + 2 * row;
          *(float2 *)p = make_float2(v.x, v.z);         // k = 4g, 4g + 2
          *(float2 *)(p + PA) = make_float2(v.y, v.w);  // k = 4g + 1, 4g + 3
        }
      };
      FRegsA r0, r1, r2;
      fetch(0, r0);
      fetch(BK, r1);
      fetch(2 * BK, r2);
      stage(r0, 0);
      fetch(3 * BK, r0);
      stage(r1, 1);
      fetch(4 * BK, r1);
      __syncthreads();
      // step i stages step i + 2 (register set and buffer (i + 2) % 3) and requests step i + 5
      auto step = [&](int i, FRegsA &rs, int buf) __attribute__((always_inline)) {
        stage(rs, buf);
        fetch((i + 5) * BK, rs);
        __syncthreads();
      };
      int i = 0;
      for (; i + 3 <= nsteps; i += 3) {
        step(i, r2, 2);
        step(i + 1, r0, 0);
        step(i + 2, r1, 1);
      }
      if (i < nsteps) step(i, r2, 2);
      if (i + 1 < nsteps) step(i + 1, r0, 0);
    } else {
      // ---- stage B
      const unsigned boff = 4u * ((unsigned)(4 * (t >> 5) + ((t >> 4) & 1)) * (unsigned)N + (unsigned)(n0 + 4 * (t & 15)));
      auto fetch = [&](int k0, FRegsB &rb) __attribute__((always_inline)) {
        rb.d = 0;
        if constexpr (FULL) {
          const char *bb = (const char *)(a.B + (int64_t)(kbeg + min(k0, (nsteps - 1) * BK)) * N);
          rb.r0 = *(const uint4 *)(bb + boff);
          rb.r1 = *(const uint4 *)(bb + boff + 8u * (unsigned)N);  // two rows further on
          return;
        }
        // thread (g, h, nq): rows k = 4g + h and 4g + 2 + h of the step, columns 4 nq .. + 3
        const int g = t >> 5, h = (t >> 4) & 1, n = n0 + 4 * (t & 15);
        const int k1 = kbeg + k0 + 4 * g + h, k2 = k1 + 2;
        const float4 v1 = load4<AL>(a.B + (int64_t)k1 * N + n, k1 < K ? clamp04(N - n) : 0);
        const float4 v2 = load4<AL>(a.B + (int64_t)k2 * N + n, k2 < K ? clamp04(N - n) : 0);
        rb.r0 = make_uint4(__float_as_uint(v1.x), __float_as_uint(v1.y), __float_as_uint(v1.z), __float_as_uint(v1.w));
        rb.r1 = make_uint4(__float_as_uint(v2.x), __float_as_uint(v2.y), __float_as_uint(v2.z), __float_as_uint(v2.w));
      };
      auto stage = [&](const FRegsB &rb, int buf) __attribute__((always_inline)) {
        float *p = (float *)(smem + kABytes + buf * kBBuf) + (t >> 4) * PB + 2 * 4 * (t & 15);  // plane 2g + h = t / 16
        *(uint4 *)p = make_uint4(rb.r0.x, rb.r1.x, rb.r0.y, rb.r1.y);
        *(uint4 *)(p + 4) = make_uint4(rb.r0.z, rb.r1.z, rb.r0.w, rb.r1.w);
      };
      FRegsB r0, r1, r2;
      fetch(0, r0);
      fetch(BK, r1);
      fetch(2 * BK, r2);
      stage(r0, 0);
      fetch(3 * BK, r0);
      stage(r1, 1);
      fetch(4 * BK, r1);
      __syncthreads();
      auto step = [&](int i, FRegsB &rs, int buf) __attribute__((always_inline)) {
        stage(rs, buf);
        fetch((i + 5) * BK, rs);
        __syncthreads();
      };
      int i = 0;
      for (; i + 3 <= nsteps; i += 3) {
        step(i, r2, 2);
        step(i + 1, r0, 0);
        step(i + 2, r1, 1);
      }
      if (i < nsteps) step(i, r2, 2);
      if (i + 1 < nsteps) step(i + 1, r0, 0);
    }
  }
  // ---- epilogue: acc[r] is C[row = 8*(r/4) + 4*(l/32) + r%4][col = l%32] of the 32x32 sub-tile ----
  // (the last step ended with a barrier that every role passed: nobody reads or writes the operand buffers any more)
  if (role == 0) {
#pragma unroll
    for (int r = 0; r < 16; r++)
      Cs[(32 * wm + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3)) * (BN + 4) + 32 * wn + (lane & 31)] = acc[r];
  }
  __syncthreads();
  store_tile<BM, BN, 768>(a, Cs, m0, n0, tid);
}

// C = act(sum_z ws[z] + bias) + residual, z in ascending order (the result does not depend on timing)
__global__ __launch_bounds__(256) void k_splitk_reduce(GemmArgs a) {
  const int64_t n = (int64_t)a.M * a.N;
  // Up to eight partials, bias and residual are requested together, none behind a branch (absent ones re-read
  // the first partial and are dropped): a `for (z...) v += ws[z]` loop is one dependent round trip per share.
  // The shares are still added in ascending order, so the result does not depend on the launch.
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
    const float bv = *(a.bias ? a.bias + i % a.N : a.ws + i);
    const float rv = *(a.residual ? a.residual + i : a.ws + i);
    float v = 0.0f;
    for (int zb = 0; zb < a.ksplit; zb += 8) {
      float t[8];
#pragma unroll
      for (int u = 0; u < 8; u++) t[u] = a.ws[(int64_t)(zb + u < a.ksplit ? zb + u : 0) * n + i];
#pragma unroll
      for (int u = 0; u < 8; u++)
        if (zb + u < a.ksplit) v = (zb + u == 0) ? t[u] : v + t[u];
    }
    if (a.bias) v += bv;
    v = apply_act(a.act, v);
    if (a.residual) v += rv;
    a.C[i] = v;
  }
}

// precision: GEMM_FP32 = fp32 MFMA operands (k_gemm_f32), GEMM_BF16 = operands rounded to bf16,
// GEMM_BF16X3 / GEMM_BF16X6 = operands split in two / three bf16 terms.  Q8_0 / Q4_0 weights take k_gemm_qpc
// (integer plane exact in bf16, block scales applied to the partial sums) with 1 / 2 / 3 activation terms.
// Split-K partial tiles of the entry point that allocates nothing (cthip_matmul_noalloc): one array per device,
// held until the process ends.  In host code the name below is only a stand-in; the device address is taken
// once per device with hipGetSymbolAddress (matmul_scratch_init, called by cthip_init) and kept in g_scratch_ptr.
constexpr size_t kScratchBytes = 4ull << 20;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
constexpr int kMaxDevices = 64;
static float *g_scratch_ptr[kMaxDevices] = {};

int matmul_scratch_init(int device) {
  if (device < 0 || device >= kMaxDevices) return fail(CTHIP_E_BAD_ARG, "cthip_init: device %d is beyond the %d this library keeps scratch for", device, kMaxDevices);
  if (g_scratch_ptr[device]) return 0;
  void *p = nullptr;
  CTHIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
  g_scratch_ptr[device] = (float *)p;
  return 0;
}

// static_ws: null = split-K partials come from the caching allocator; otherwise they go to this buffer of
// static_ws_bytes bytes and nothing is allocated or freed
int launch_gemm(GemmArgs a, int bmode, int precision, float *static_ws, size_t static_ws_bytes, GemmDeferred *defer) {
  if (a.M == 0 || a.N == 0) return 0;
  hipStream_t st = state().stream;
  const int cus = state().compute_units;
  // the bf16 kernels read packed rows in 16-element chunks: fp32 / fp16 weight rows of another width go to
  // the fp32 kernel, which is at least as accurate as any of the modes
  if (bmode == B_WMAT && (a.K & 15)) precision = GEMM_FP32;
  const bool quant = precision != GEMM_FP32 && bmode == B_WMAT && (a.wtype == CTHIP_Q8_0 || a.wtype == CTHIP_Q4_0);
  // 64 output rows per workgroup.  (128-row tiles -- two accumulator blocks per wavefront, half the weight-side
  // staging -- measured slower on every prefill shape: one workgroup per compute unit and 32 KB of A per step.)
  const int bm = 64;
  const int bn = quant ? 128 : 64;  // k_gemm_qpc owns 64 x 128
  const int64_t tiles = (int64_t)((a.M + bm - 1) / bm) * ((a.N + bn - 1) / bn);
  if (tiles > 0x7fffffff / 16) return fail(CTHIP_E_BAD_ARG, "gemm: too many tiles");
  dim3 grid((unsigned)tiles), block(256);
  a.ksplit = 1;
  a.kper = a.K > 0 ? a.K : 1;
  a.ws = nullptr;
  {
    // one region of tiles per XCD: the split with the fewest tiles per XCD, then the least operand bytes per L2
    a.tm = (a.M + bm - 1) / bm;
    a.tn = (a.N + bn - 1) / bn;
    const double sza = 4.0 * bm / 64, szb = bmode == B_ROWMAJOR ? 4.0 : a.wtype == CTHIP_Q8_0 ? 1.0625 : a.wtype == CTHIP_Q4_0 ? 0.5625 : a.wtype == CTHIP_F16 ? 2.0 : 4.0;
    double best = -1.0;
    for (int rx = 1; rx <= 8; rx *= 2) {
      const int ry = 8 / rx, rm = (a.tm + rx - 1) / rx, rn = (a.tn + ry - 1) / ry;
      const double score = (double)rm * rn * 1e6 + rm * sza + rn * szb;
      if (best < 0 || score < best) {
        best = score;
        a.rx = rx;
        a.rm = rm;
        a.rn = rn;
      }
    }
    grid.x = 8u * (unsigned)a.rm * (unsigned)a.rn;
    // too few tiles to occupy the chip and a long reduction axis: split K over several workgroups per tile
    const int nsteps = (a.K + 63) / 64;  // K-steps of 64 (two of the fp32 kernel's)
    // workgroups aimed at: two per compute unit where the tiles fill less than half the chip (GPT-2 / Llama
    // prefill 1.47 / 3.29 -> 1.44 / 3.18 ms against 1.5; three per unit: 1.55 / 3.18), else 1.5 (a 1024^3
    // product, one tile per unit, loses 10-30 % when it is split in two)
    // (the 512-thread workgroups of k_gemm_qpc sit one to a compute unit: aim at one each)
    int ks = quant ? (int)(cus / tiles) : (int)((tiles * 2 <= cus ? cus * 2 : cus * 3 / 2) / tiles);
    if (ks > nsteps / 3) ks = nsteps / 3;
    if (ks > 16) ks = 16;
    if (a.routed || a.pairs) ks = 1;  // routed / paired tiles are stored by the workgroup that computed them
    if (ks > 1) {
      const int steps_per = (nsteps + ks - 1) / ks;
      a.kper = steps_per * 64;
      a.ksplit = (nsteps + steps_per - 1) / steps_per;
      if (a.ksplit > 1) {
        const size_t need = sizeof(float) * (size_t)a.ksplit * a.M * a.N;
        if (static_ws) {
          if (need > static_ws_bytes)
            return fail(CTHIP_E_UNSUPPORTED, "cthip_matmul_noalloc: (%d,%d,%d) splits its reduction %d ways and needs %zu bytes of partial "
                        "tiles; the static scratch holds %zu (use cthip_matmul)", a.M, a.N, a.K, a.ksplit, need, static_ws_bytes);
          a.ws = static_ws;  // every element of every share is written before the reduction reads it
        } else {
          int rc = alloc_scratch((void **)&a.ws, need);
          if (rc) return rc;
        }
        grid.y = a.ksplit;
      } else {
        a.kper = a.K;
      }
    }
  }
  if (precision == GEMM_FP32) {
    // aligned: every 4 (8 for packed weights) consecutive operand elements a thread asks for are one aligned vector
    const bool al = bmode == B_ROWMAJOR ? (a.K % 4 == 0 && a.N % 4 == 0) : (a.K % 8 == 0);
    if (bmode == B_ROWMAJOR) {
      const bool full = al && a.M % 64 == 0 && a.N % 64 == 0 && a.K % 32 == 0 && a.kper % 32 == 0 && (int64_t)a.M * a.K * 4 < (1ll << 32) &&
                        ((int64_t)64 * a.N + a.N) * 4 < (1ll << 32);
      if (full) hipLaunchKernelGGL((k_gemm_f32pc<true, true>), grid, dim3(768), 0, st, a);
      else if (al) hipLaunchKernelGGL((k_gemm_f32pc<true, false>), grid, dim3(768), 0, st, a);
      else hipLaunchKernelGGL((k_gemm_f32pc<false, false>), grid, dim3(768), 0, st, a);
    } else {
      if (al) hipLaunchKernelGGL((k_gemm_f32<true>), grid, block, 0, st, a);
      else hipLaunchKernelGGL((k_gemm_f32<false>), grid, block, 0, st, a);
    }
  } else if (quant) {
    const int npa = precision == GEMM_BF16X6 ? 3 : precision == GEMM_BF16X3 ? 2 : 1;
    // whole tiles, whole steps, 32-bit byte offsets: the kernel's addressing without bounds tests
    const bool full = a.M % 64 == 0 && a.N % 128 == 0 && a.K % 64 == 0 && a.kper % 64 == 0 &&
                      (int64_t)a.M * a.K * 4 < (1ll << 32) && (int64_t)a.N * a.K < (1ll << 32);
#define QG(WT, NPA, MB)                                                                    \
  if (full) hipLaunchKernelGGL((k_gemm_qpc<WT, NPA, 8, true>), grid, dim3(768), 0, st, a); \
  else hipLaunchKernelGGL((k_gemm_qpc<WT, NPA, 8, false>), grid, dim3(768), 0, st, a)
#define QSEL(WT)                  \
  if (npa == 3) QG(WT, 3, 1);     \
  else if (npa == 2) QG(WT, 2, 1); \
  else QG(WT, 1, 1);
    if (a.wtype == CTHIP_Q8_0) {
      QSEL(W_Q8)
    } else {
      QSEL(W_Q4)
    }
#undef QSEL
#undef QG
  } else {
    int wm = W_ROWMAJOR;
    if (bmode == B_WMAT) wm = a.wtype == CTHIP_F16 ? W_F16 : W_F32;
#define SPLIT3(MODE, AL)                                                                                      \
  if (precision == GEMM_BF16X6) hipLaunchKernelGGL((k_gemm_split<MODE, 6, AL>), grid, dim3(768), 0, st, a);      \
  else if (precision == GEMM_BF16X3) hipLaunchKernelGGL((k_gemm_split<MODE, 3, AL>), grid, dim3(768), 0, st, a); \
  else hipLaunchKernelGGL((k_gemm_split<MODE, 1, AL>), grid, dim3(768), 0, st, a)
#define SPLIT(MODE)      \
  case MODE:             \
    if (al) {            \
      SPLIT3(MODE, true); \
    } else {             \
      SPLIT3(MODE, false); \
    }                    \
    break
    // aligned: every 4 consecutive floats a thread asks for are one 16-byte vector, inside or outside as a whole
    const bool al = a.K % 4 == 0 && (bmode != B_ROWMAJOR || a.N % 4 == 0);
    switch (wm) {
      SPLIT(W_ROWMAJOR);
      SPLIT(W_F32);
      SPLIT(W_F16);
    }
#undef SPLIT3
#undef SPLIT
  }
  hipError_t le = hipGetLastError();
  if (le != hipSuccess) {
    if (a.ws && !static_ws) cthip_free(a.ws);
    return fail((int)le, "gemm: launch -> %s", hipGetErrorString(le));
  }
  if (a.ksplit > 1 && defer && !static_ws && a.act == CTHIP_ACT_NONE) {  // the caller reduces (and owns the tiles)
    defer->ws = a.ws;
    defer->ksplit = a.ksplit;
    return 0;
  }
  if (a.ksplit > 1) {
    int64_t blocks = ((int64_t)a.M * a.N + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(k_splitk_reduce, dim3((unsigned)blocks), dim3(256), 0, st, a);
    le = hipGetLastError();
    int rc = static_ws ? 0 : cthip_free(a.ws);  // stream-ordered: the block is reused only by later work on the same stream
    if (le != hipSuccess) return fail((int)le, "gemm: launch -> %s", hipGetErrorString(le));
    return rc;
  }
  return 0;
}

// Linear over m rows with packed weights: y (m, rows) = act(x (m, cols) @ W^T + bias) + residual
int launch_splitk_reduce(float *C, float *ws, int ksplit, int m, int n, const float *bias, const float *residual) {
  GemmArgs a = {};
  a.C = C;
  a.ws = ws;
  a.ksplit = ksplit;
  a.M = m;
  a.N = n;
  a.bias = bias;
  a.residual = residual;
  a.act = CTHIP_ACT_NONE;
  int64_t blocks = ((int64_t)m * n + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(k_splitk_reduce, dim3((unsigned)blocks), dim3(256), 0, state().stream, a);
  CTHIP_LAUNCH_CHECK();
  return 0;
}

int launch_linear_gemm(float *y, const WMat *w, const float *x, int m, const float *bias, const float *residual,
                       int act, int precision, GemmDeferred *defer, const GemmRoute *route) {
  GemmArgs a = {};
  a.C = y;
  a.A = x;
  a.wq = w->q;
  a.wd = (const unsigned short *)w->d;
  a.wtype = w->type;
  a.bias = bias;
  a.residual = residual;
  a.M = m;
  a.N = (int)w->rows;
  a.K = (int)w->cols;
  a.act = act;
  if (act == kActSwigluPairs) {
    if (a.N % 4 || residual || route) return fail(CTHIP_E_BAD_ARG, "launch_linear_gemm: paired SwiGLU epilogue with %d rows, a residual or a route", a.N);
    a.act = CTHIP_ACT_NONE;
    a.pairs = 1;
  }
  if (route) {
    for (int i = 0; i < 3; i++)
      if (route->c0[i] != INT_MAX && (route->c0[i] % 128 != 0 || !route->dst[i] || route->ld[i] <= 0))
        return fail(CTHIP_E_BAD_ARG, "launch_linear_gemm: route part %d starts at column %d (whole 128-column tiles are routed)", i, route->c0[i]);
    if (route->c0[0] != 0 || residual) return fail(CTHIP_E_BAD_ARG, "launch_linear_gemm: a route starts at column 0 and takes no residual");
    a.routed = 1;
    a.route = *route;
  }
  return launch_gemm(a, B_WMAT, precision, nullptr, 0, defer);
}

// A matmul-shaped Schedule-Item routed here by the renderer: C (M,N) = act(A (M,K) . B + bias) + residual, B either (K,N)
// row-major or (N,K) rows read through a transposed view (Linear, source/nn/linear.lisp:3-17); fp32-grade operands.
int matmul_routed(float *C, const float *A, const float *B, int M, int N, int K, int act, const float *bias, const float *residual,
                  bool b_is_nk) {
  if (b_is_nk && M < 8) {  // a few rows of a Linear: the single-row kernels stream the weights once per row
    WMat w = {};
    w.type = CTHIP_F32;
    w.rows = N;
    w.cols = K;
    w.q = const_cast<float *>(B);
    w.q_bytes = (int64_t)N * K * 4;
    GemvArgs g = {};
    g.y = C;
    g.x = A;
    g.bias = bias;
    g.residual = residual;
    g.act = act;
    g.x_stride = K;
    g.y_stride = N;
    return launch_gemv(&w, g, M);
  }
  GemmArgs a = {};
  a.C = C;
  a.A = A;
  a.bias = bias;
  a.residual = residual;
  a.M = M;
  a.N = N;
  a.K = K;
  a.act = act;
  if (b_is_nk) {
    a.wq = B;
    a.wtype = CTHIP_F32;
    return launch_gemm(a, B_WMAT, GEMM_BF16X6, nullptr, 0, nullptr);
  }
  a.B = B;
  return launch_gemm(a, B_ROWMAJOR, GEMM_BF16X6, nullptr, 0, nullptr);
}

}  // namespace cthip

using namespace cthip;

static int matmul_entry(float *C, const float *A, const float *B, int M, int N, int K, int act, int precision, bool noalloc) {
  CTHIP_REQUIRE_INIT();
  CTHIP_ARG(M >= 0 && N >= 0 && K >= 0);
  CTHIP_ARG((int64_t)M * N == 0 || (C != nullptr && (K == 0 || (A != nullptr && B != nullptr))));
  CTHIP_ARG(act >= CTHIP_ACT_NONE && act <= CTHIP_ACT_TANH);
  CTHIP_ARG(precision >= GEMM_FP32 && precision <= GEMM_BF16X6);
  GemmArgs a = {};
  a.C = C;
  a.A = A;
  a.B = B;
  a.M = M;
  a.N = N;
  a.K = K;
  a.act = act;
  if (!noalloc) return launch_gemm(a, B_ROWMAJOR, precision, nullptr, 0, nullptr);
  float *ws = g_scratch_ptr[state().device];
  if (!ws) return fail(CTHIP_E_STATE, "cthip_matmul_noalloc: no scratch address for device %d", state().device);
  return launch_gemm(a, B_ROWMAJOR, precision, ws, kScratchBytes, nullptr);
}

extern "C" int cthip_matmul(float *C, const float *A, const float *B, int M, int N, int K, int act, int precision) {
  return matmul_entry(C, A, B, M, N, K, act, precision, false);
}

extern "C" int cthip_matmul_noalloc(float *C, const float *A, const float *B, int M, int N, int K, int act, int precision) {
  return matmul_entry(C, A, B, M, N, K, act, precision, true);
}
