// MFMA GEMM for the matmul-shaped fusions: `!relu(!matmul A B)` (source/api/high-level-ops.lisp:76-99,
// fused per source/test-suite/test-scheduler.lisp:140-163) and Linear over m > 1 rows (prefill,
// source/nn/linear.lisp:3-17) with the weights still packed (dequantised while they are staged).
//
// One 256-thread workgroup (4 wavefronts, 2x2) owns a 64x64 tile of C; each wavefront accumulates a
// 32x32 sub-tile in 16 accumulator registers with v_mfma_f32_32x32x2_f32 (fp32 operands) or
// v_mfma_f32_32x32x8_bf16 (operands rounded to bf16, fp32 accumulation).  A and B are staged through
// LDS in K-steps of 32, k-major so that the MFMA operand reads are conflict-free (lane l reads row
// k = l/32 + ..., column l%32).  1024x1024 outputs give 256 workgroups = one per compute unit.
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
};

__device__ __forceinline__ unsigned short f32_to_bf16_bits(float f) {
  // round to nearest even
  unsigned u = __float_as_uint(f);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (unsigned short)(u >> 16);
}

// element (n, k) of a packed weight matrix as fp32
__device__ __forceinline__ void wmat_load8(const GemmArgs &a, int n, int k, float *out) {
  // 8 consecutive k (k % 8 == 0) of row n
  const int64_t K = a.K;
  if (a.wtype == CTHIP_Q8_0) {
    const uint2 q = *(const uint2 *)((const int8_t *)a.wq + n * K + k);
    const float d = half_bits_to_float(a.wd[n * (K >> 5) + (k >> 5)]);
    const unsigned dw[2] = {q.x, q.y};
#pragma unroll
    for (int t = 0; t < 2; t++) {
      const int v = (int)dw[t];
      out[4 * t + 0] = (float)(int)(int8_t)(v)*d;
      out[4 * t + 1] = (float)(int)(int8_t)(v >> 8) * d;
      out[4 * t + 2] = (float)(int)(int8_t)(v >> 16) * d;
      out[4 * t + 3] = (float)(v >> 24) * d;
    }
  } else if (a.wtype == CTHIP_Q4_0) {
    // block b = k/32; elements j<16 are low nibbles of byte j, j>=16 high nibbles of byte j-16
    const int64_t b = n * (K >> 5) + (k >> 5);
    const int j0 = k & 31;
    const uint2 q = *(const uint2 *)((const uint8_t *)a.wq + 16 * b + (j0 & 15));
    const float d = half_bits_to_float(a.wd[b]);
    const unsigned dw[2] = {q.x, q.y};
    const int sh = (j0 < 16) ? 0 : 4;
#pragma unroll
    for (int t = 0; t < 8; t++) out[t] = (float)((int)((dw[t >> 2] >> (8 * (t & 3) + sh)) & 0xf) - 8) * d;
  } else if (a.wtype == CTHIP_F16) {
    const uint4 h = *(const uint4 *)((const unsigned short *)a.wq + n * K + k);
    const unsigned dw[4] = {h.x, h.y, h.z, h.w};
#pragma unroll
    for (int t = 0; t < 4; t++) {
      out[2 * t] = half_bits_to_float((unsigned short)(dw[t] & 0xffff));
      out[2 * t + 1] = half_bits_to_float((unsigned short)(dw[t] >> 16));
    }
  } else {
    const float4 f0 = *(const float4 *)((const float *)a.wq + n * K + k);
    const float4 f1 = *(const float4 *)((const float *)a.wq + n * K + k + 4);
    out[0] = f0.x; out[1] = f0.y; out[2] = f0.z; out[3] = f0.w;
    out[4] = f1.x; out[5] = f1.y; out[6] = f1.z; out[7] = f1.w;
  }
}

template <int BMODE, bool BF16>
__global__ __launch_bounds__(256) void k_gemm(GemmArgs a) {
  constexpr int BM = 64, BN = 64, BK = 32, PAD = 4;
  // fp32: As[k][m], Bs[k][n] (k-major).  bf16: As[m][k], Bs[n][k] as 16-bit (k contiguous: a lane's
  // MFMA operand is 4 consecutive k)
  __shared__ float As_f[BF16 ? 1 : BK][BF16 ? 1 : BM + PAD];
  __shared__ float Bs_f[BF16 ? 1 : BK][BF16 ? 1 : BN + PAD];
  __shared__ unsigned short As_h[BF16 ? BM : 1][BF16 ? BK + PAD : 1];
  __shared__ unsigned short Bs_h[BF16 ? BN : 1][BF16 ? BK + PAD : 1];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  // consecutive workgroups walk down a column of tiles: they share the B panel through L2
  const int tiles_m = (a.M + BM - 1) / BM;
  const int m0 = (blockIdx.x % tiles_m) * BM, n0 = (blockIdx.x / tiles_m) * BN;
  const bool vecA = (a.K % 4 == 0), vecB = (a.N % 4 == 0);
  v16f acc;
#pragma unroll
  for (int r = 0; r < 16; r++) acc[r] = 0.0f;

  // thread -> staging coordinates
  const int ar = tid >> 2, akc = (tid & 3) * 8;            // A: row ar, 8 consecutive k
  const int bk = tid >> 3, bnc = (tid & 7) * 8;            // B row-major: row k = bk, 8 consecutive n
  const int wr = tid >> 2, wkc = (tid & 3) * 8;            // B packed: weight row wr, 8 consecutive k

  auto fetch_a = [&](int k0, float *v) {
#pragma unroll
    for (int j = 0; j < 8; j++) v[j] = 0.0f;
    const int gm = m0 + ar;
    if (gm < a.M) {
      const float *src = a.A + (int64_t)gm * a.K + k0 + akc;
      if (vecA && k0 + akc + 8 <= a.K) {
        const float4 f0 = *(const float4 *)src, f1 = *(const float4 *)(src + 4);
        v[0] = f0.x; v[1] = f0.y; v[2] = f0.z; v[3] = f0.w; v[4] = f1.x; v[5] = f1.y; v[6] = f1.z; v[7] = f1.w;
      } else {
#pragma unroll
        for (int j = 0; j < 8; j++)
          if (k0 + akc + j < a.K) v[j] = src[j];
      }
    }
  };
  auto fetch_b = [&](int k0, float *v) {
#pragma unroll
    for (int j = 0; j < 8; j++) v[j] = 0.0f;
    if (BMODE == B_ROWMAJOR) {
      if (k0 + bk < a.K) {
        const float *src = a.B + (int64_t)(k0 + bk) * a.N + n0 + bnc;
        if (vecB && n0 + bnc + 8 <= a.N) {
          const float4 f0 = *(const float4 *)src, f1 = *(const float4 *)(src + 4);
          v[0] = f0.x; v[1] = f0.y; v[2] = f0.z; v[3] = f0.w; v[4] = f1.x; v[5] = f1.y; v[6] = f1.z; v[7] = f1.w;
        } else {
#pragma unroll
          for (int j = 0; j < 8; j++)
            if (n0 + bnc + j < a.N) v[j] = src[j];
        }
      }
    } else {
      // packed weights (K % 32 == 0 for every packed type here): dequantised on the way in
      if (n0 + wr < a.N && k0 + wkc < a.K) wmat_load8(a, n0 + wr, k0 + wkc, v);
    }
  };
  auto stage = [&](const float *va, const float *vb) {
    if (BF16) {
#pragma unroll
      for (int j = 0; j < 8; j++) As_h[BF16 ? ar : 0][BF16 ? akc + j : 0] = f32_to_bf16_bits(va[j]);
    } else {
#pragma unroll
      for (int j = 0; j < 8; j++) As_f[BF16 ? 0 : akc + j][BF16 ? 0 : ar] = va[j];
    }
    if (BMODE == B_ROWMAJOR) {
      if (BF16) {
#pragma unroll
        for (int j = 0; j < 8; j++) Bs_h[BF16 ? bnc + j : 0][BF16 ? bk : 0] = f32_to_bf16_bits(vb[j]);
      } else {
#pragma unroll
        for (int j = 0; j < 8; j++) Bs_f[BF16 ? 0 : bk][BF16 ? 0 : bnc + j] = vb[j];
      }
    } else {
      if (BF16) {
#pragma unroll
        for (int j = 0; j < 8; j++) Bs_h[BF16 ? wr : 0][BF16 ? wkc + j : 0] = f32_to_bf16_bits(vb[j]);
      } else {
#pragma unroll
        for (int j = 0; j < 8; j++) Bs_f[BF16 ? 0 : wkc + j][BF16 ? 0 : wr] = vb[j];
      }
    }
  };

  // software pipeline: the next K-step's global loads are in flight while the MFMAs of this one run
  float va[8], vb[8];
  fetch_a(0, va);
  fetch_b(0, vb);
  for (int k0 = 0; k0 < a.K; k0 += BK) {
    stage(va, vb);
    __syncthreads();
    if (k0 + BK < a.K) {
      fetch_a(k0 + BK, va);
      fetch_b(k0 + BK, vb);
    }
    if (BF16) {
      // 32x32x8: lane l holds A[i = l%32][k = 4*(l/32) .. +3] and B[k = 4*(l/32) .. +3][j = l%32]
#pragma unroll
      for (int s = 0; s < BK / 8; s++) {
        const int kk = 8 * s + 4 * (lane >> 5);
        const v4s av = *(const v4s *)&As_h[BF16 ? 32 * wm + (lane & 31) : 0][BF16 ? kk : 0];
        const v4s bv = *(const v4s *)&Bs_h[BF16 ? 32 * wn + (lane & 31) : 0][BF16 ? kk : 0];
        acc = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(av, bv, acc, 0, 0, 0);
      }
    } else {
      // 32x32x2: lane l holds A[i = l%32][k = l/32] and B[k = l/32][j = l%32]
#pragma unroll
      for (int s = 0; s < BK / 2; s++) {
        const int kk = 2 * s + (lane >> 5);
        const float av = As_f[BF16 ? 0 : kk][BF16 ? 0 : 32 * wm + (lane & 31)];
        const float bv = Bs_f[BF16 ? 0 : kk][BF16 ? 0 : 32 * wn + (lane & 31)];
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc, 0, 0, 0);
      }
    }
    __syncthreads();
  }
  // ---- epilogue: acc[r] is C[row = 8*(r/4) + 4*(l/32) + r%4][col = l%32] of the 32x32 sub-tile ----
  const int col = n0 + 32 * wn + (lane & 31);
  if (col < a.N) {
    const float bias = a.bias ? a.bias[col] : 0.0f;
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int row = m0 + 32 * wm + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
      if (row < a.M) {
        float v = apply_act(a.act, acc[r] + bias);
        if (a.residual) v += a.residual[(int64_t)row * a.N + col];
        a.C[(int64_t)row * a.N + col] = v;
      }
    }
  }
}

int launch_gemm(GemmArgs a, int bmode, bool bf16) {
  if (a.M == 0 || a.N == 0) return 0;
  const int64_t tiles = (int64_t)((a.M + 63) / 64) * ((a.N + 63) / 64);
  if (tiles > 0x7fffffff) return fail(CTHIP_E_BAD_ARG, "gemm: too many tiles");
  dim3 grid((unsigned)tiles), block(256);
  hipStream_t st = state().stream;
  if (bmode == B_ROWMAJOR) {
    if (bf16) hipLaunchKernelGGL((k_gemm<B_ROWMAJOR, true>), grid, block, 0, st, a);
    else hipLaunchKernelGGL((k_gemm<B_ROWMAJOR, false>), grid, block, 0, st, a);
  } else {
    if (bf16) hipLaunchKernelGGL((k_gemm<B_WMAT, true>), grid, block, 0, st, a);
    else hipLaunchKernelGGL((k_gemm<B_WMAT, false>), grid, block, 0, st, a);
  }
  CTHIP_LAUNCH_CHECK();
  return 0;
}

// Linear over m rows with packed weights: y (m, rows) = act(x (m, cols) @ W^T + bias) + residual
int launch_linear_gemm(float *y, const WMat *w, const float *x, int m, const float *bias, const float *residual,
                       int act, bool bf16) {
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
  return launch_gemm(a, B_WMAT, bf16);
}

}  // namespace cthip

using namespace cthip;

extern "C" int cthip_matmul(float *C, const float *A, const float *B, int M, int N, int K, int act, int precision) {
  CTHIP_REQUIRE_INIT();
  CTHIP_ARG(M >= 0 && N >= 0 && K >= 0);
  CTHIP_ARG((int64_t)M * N == 0 || (C != nullptr && (K == 0 || (A != nullptr && B != nullptr))));
  CTHIP_ARG(act >= CTHIP_ACT_NONE && act <= CTHIP_ACT_TANH);
  CTHIP_ARG(precision == 0 || precision == 1);
  GemmArgs a = {};
  a.C = C;
  a.A = A;
  a.B = B;
  a.M = M;
  a.N = N;
  a.K = K;
  a.act = act;
  return launch_gemm(a, B_ROWMAJOR, precision == 1);
}
