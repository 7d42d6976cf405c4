// Batched, strided small matmuls: the attention items of a decoder graph as Caten schedules them
// (external/llm/layers.lisp:3-5) -- scores = q . K^T * scale + mask over the cache view, out = P . V -- and the
// batched nest of source/test-suite/test-scheduler.lisp:126-138.  Operands are addressed the way the Schedule-Item
// addresses them, base + sum of stride * index over up to three batch loops, the row i, the column j and the
// reduction index k, so the cache `(max_len, heads, head_dim)` is read in place through its `[0, n+s)` view and q
// straight out of the fused qkv rows.  Few rows (a decode step has one): a launch is bandwidth- and latency-bound,
// so the work is laid out for coalesced 128-bit reads of the operand that is streamed (B):
//   KC  B's reduction index is contiguous (K^T read through a transposed view): 16 lanes x float4 cover 64
//       reduction elements of one output column, four columns per wavefront and pass, 16-lane DPP reduction;
//   NC  B's column index is contiguous (P . V): a lane owns four adjacent columns, the 16 lane groups of a
//       workgroup split the reduction and meet once in LDS.
// Epilogue per element, in this order: alpha * acc, + pre[..] (up to two addends: bias, mask), activation, + post[..].
#include "common.h"

namespace cthip {

template <bool KC>
__global__ __launch_bounds__(256) void k_bmm(BmmArgs a) {
  const int tid = threadIdx.x;
  // batch coordinates of this workgroup
  int bz = blockIdx.z;
  const int b2 = bz % a.nb[2];
  bz /= a.nb[2];
  const int b1 = bz % a.nb[1];
  const int b0 = bz / a.nb[1];
  const int i = blockIdx.y;
  auto off = [&](const BmmOperand &o) { return o.base + (int64_t)b0 * o.sb[0] + (int64_t)b1 * o.sb[1] + (int64_t)b2 * o.sb[2]; };
  const float *__restrict__ A = a.A + off(a.a) + (int64_t)i * a.a.si;
  const float *__restrict__ B = a.B + off(a.b);
  auto epilogue = [&](int j, float acc) {
    float v = a.alpha * acc;
    if (a.pre0) v += a.pre0[off(a.p0) + (int64_t)i * a.p0.si + (int64_t)j * a.p0.sj];
    if (a.pre1) v += a.pre1[off(a.p1) + (int64_t)i * a.p1.si + (int64_t)j * a.p1.sj];
    v = apply_act(a.act, v);
    if (a.post) v += a.post[off(a.r) + (int64_t)i * a.r.si + (int64_t)j * a.r.sj];
    a.C[off(a.c) + (int64_t)i * a.c.si + (int64_t)j * a.c.sj] = v;
  };
  if (KC) {
    // column j = 16 * blockIdx.x + tid / 16; lane c = tid % 16 takes reduction elements 4c + 64 * step ..+3
    const int c = tid & 15;
    int j = blockIdx.x * 16 + (tid >> 4);
    const bool live = j < a.N;
    j = live ? j : a.N - 1;  // requests stay unconditional: a column past the end repeats the last one
    const float *__restrict__ Bj = B + (int64_t)j * a.b.sj;
    float acc = 0.0f;
    for (int k0 = 4 * c; k0 < a.K; k0 += 64) {
      const float4 x = *(const float4 *)(A + k0);
      const float4 w = *(const float4 *)(Bj + k0);
      acc = fmaf(x.x, w.x, acc);
      acc = fmaf(x.y, w.y, acc);
      acc = fmaf(x.z, w.z, acc);
      acc = fmaf(x.w, w.w, acc);
    }
    acc = row16_sum(acc);
    if (live && c == 0) epilogue(j, acc);
  } else {
    // columns 4 * (16 * blockIdx.x + tid % 16) ..+3; reduction elements tid / 16, + 16, ...
    __shared__ float4 red[16][16];
    const int c = tid & 15, g = tid >> 4;
    int j4 = blockIdx.x * 64 + 4 * c;
    const bool live = j4 < a.N;
    j4 = live ? j4 : 0;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int k = g; k < a.K; k += 16) {
      const float x = A[(int64_t)k * a.a.sk];
      const float4 w = *(const float4 *)(B + (int64_t)k * a.b.sk + j4);
      acc.x = fmaf(x, w.x, acc.x);
      acc.y = fmaf(x, w.y, acc.y);
      acc.z = fmaf(x, w.z, acc.z);
      acc.w = fmaf(x, w.w, acc.w);
    }
    red[g][c] = acc;
    __syncthreads();
    if (g == 0 && live) {
      float4 s = red[0][c];
      for (int q = 1; q < 16; q++) {
        const float4 t = red[q][c];
        s.x += t.x;
        s.y += t.y;
        s.z += t.z;
        s.w += t.w;
      }
      epilogue(j4, s.x);
      epilogue(j4 + 1, s.y);
      epilogue(j4 + 2, s.z);
      epilogue(j4 + 3, s.w);
    }
  }
}

// Which of the two layouts fits, if any: 0 = none, 1 = KC, 2 = NC.  Pure arithmetic on the operand description
// (pointers included, for alignment), so the caller can decide before anything is launched.
int bmm_variant(const BmmArgs &a) {
  if (a.M < 1 || a.N < 1 || a.K < 1) return 0;
  for (int q = 0; q < 3; q++)
    if (a.nb[q] < 1) return 0;
  if ((int64_t)a.nb[0] * a.nb[1] * a.nb[2] > 65535 || a.M > 65535) return 0;
  auto al4 = [](const BmmOperand &o, const float *p) {
    return ((uintptr_t)(p + o.base) % 16) == 0 && o.sb[0] % 4 == 0 && o.sb[1] % 4 == 0 && o.sb[2] % 4 == 0 && o.si % 4 == 0;
  };
  if (a.a.sk == 1 && a.b.sk == 1 && a.K % 4 == 0 && al4(a.a, a.A) && al4(a.b, a.B) && a.b.sj % 4 == 0) return 1;
  if (a.b.sj == 1 && a.N % 4 == 0 && al4(a.b, a.B) && a.b.sk % 4 == 0) return 2;
  return 0;
}

int launch_bmm(const BmmArgs &a) {
  const int v = bmm_variant(a);
  if (!v) return fail(CTHIP_E_UNSUPPORTED, "batched matmul: operand layout fits neither variant");
  const unsigned nbatch = (unsigned)(a.nb[0] * a.nb[1] * a.nb[2]);
  hipStream_t st = state().stream;
  if (v == 1) hipLaunchKernelGGL((k_bmm<true>), dim3((unsigned)((a.N + 15) / 16), (unsigned)a.M, nbatch), dim3(256), 0, st, a);
  else hipLaunchKernelGGL((k_bmm<false>), dim3((unsigned)((a.N + 63) / 64), (unsigned)a.M, nbatch), dim3(256), 0, st, a);
  CTHIP_LAUNCH_CHECK();
  return 0;
}

}  // namespace cthip
