// Internal helpers shared by the translation units of libcaten_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <limits.h>
#include <stdint.h>
#include <stdio.h>
#include <string>

#include "../../include/caten_hip.h"

namespace cthip {

constexpr int GEMM_BF16X3_DEFAULT = 2;

// ---- process-wide state (one device, one in-order stream) ----
struct State {
  bool inited = false;
  int device = -1;
  hipStream_t stream = nullptr;
  int compute_units = 0;
  hipEvent_t ev0 = nullptr, ev1 = nullptr;
  int gemm_precision = GEMM_BF16X3_DEFAULT;  // option "gemm_precision" (GEMM_*) of m > 1 Linear launches
  int gemv_stream = -1;  // option "gemv_stream_weights": -1 = per matrix (WMat::stream), 0 / 1 = never / always
  // option "gemv_wide": which single-row launches take the wide-row kernel (input vector in LDS): 0 = none, 1 = rows
  // no register-resident variant covers or only one that runs a single wavefront per SIMD, 2 = every launch it supports
  int gemv_wide = 1;
  // option "attn_split": sessions created afterwards share the keys of a head among several workgroups in the decode
  // attention of the one-launch-per-Linear step (long contexts): 1 = compute units / heads of them (at most 16),
  // 2 .. 16 = that many, 0 = one workgroup per head
  int attn_split = 1;
  // option "attn_long_from": the position from which sessions with a three-launch layer give the attention a launch
  // of its own (keys shared by several workgroups, then the projection): four launches per layer; 0 = never
  int attn_long_from = 896;
  // decoder sessions read these when they first run
  int decoder_graph = 1;  // option "decoder_graph": 0 = the step's launches are issued one by one (kernel tracing)
  int prefill_gemm = 1;   // option "prefill_gemm": 0 = prompts are fed row by row through the decode step
  int decode_fused = 1;   // option "decode_fused": 0 = five launches per layer instead of three
  int decode_flow = 0;    // option "decode_flow": 1 = GPT-2 / Q8_0 sessions run all layers of a step as one launch (decode_flow.hip)
  int render_routes = 1;  // option "render_routes": 0 = every program runs its rendered kernel, none a hand-written one
  // option "decode_skip": launches of the three-launch decode step that are left out, for knock-out timing (bits: 1 qkv,
  // 2 attention + projection, 4 MLP, 8 the sum in front of lm_head, 16 lm_head + argmax); tokens are meaningless then
  int decode_skip = 0;
  // option "kv_cache": how sessions created afterwards keep their KV cache: 1 = as Q8_0 rows (kvq.hip), 2 = fp32 rows in
  // pages opened as the position reaches them (kvp.hip)
  int kv_cache = 0;
};
State &state();
// cthip_alloc without the zero fill, for temporaries that are fully written before they are read
int alloc_scratch(void **out, size_t bytes);
bool device_readable(const void *p);
void set_error(const char *fmt, ...);
int fail(int code, const char *fmt, ...);

#define CTHIP_REQUIRE_INIT()                                                         \
  do {                                                                               \
    if (!cthip::state().inited) return cthip::fail(CTHIP_E_NOT_INIT, "%s: cthip_init has not been called", __func__); \
  } while (0)

#define CTHIP_CHECK(expr)                                                            \
  do {                                                                               \
    hipError_t _e = (expr);                                                          \
    if (_e != hipSuccess)                                                            \
      return cthip::fail((int)_e, "%s: %s -> %s", __func__, #expr, hipGetErrorString(_e)); \
  } while (0)

#define CTHIP_ARG(cond)                                                              \
  do {                                                                               \
    if (!(cond)) return cthip::fail(CTHIP_E_BAD_ARG, "%s: bad argument: %s", __func__, #cond); \
  } while (0)

// checks the launch that was just queued
#define CTHIP_LAUNCH_CHECK() CTHIP_CHECK(hipGetLastError())

// ---- packed weight matrix ----
struct WMat {
  int type;         // CTHIP_F32 / F16 / Q4_0 / Q8_0
  int64_t rows, cols;
  void *q;          // quant plane: Q8_0 int8[rows][cols]; Q4_0 u8[rows][cols/2]; F32 float; F16 half
  void *d;          // scale plane: fp16[rows][cols/32] (quantised types), else NULL
  int64_t q_bytes, d_bytes;
  // the single-row kernels request this matrix with the non-temporal hint: set for a matrix that cannot stay in
  // the Infinity Cache between two uses (too large by itself, or one of a model's that together are too large)
  bool stream;
  // a LayerNorm folded through the product (cthip_wmat_fold_layernorm): fold_s = W.gamma, fold_c = W.beta + bias,
  // valid for exactly these gamma / beta / bias vectors
  const float *fold_g = nullptr, *fold_b = nullptr, *fold_bias = nullptr;
  float *fold_s = nullptr, *fold_c = nullptr;
};
// gfx950: 256 MB of Infinity Cache in front of HBM
static const int64_t kInfinityCacheBytes = 256ll << 20;

// ---- batched, strided small matmul (bmm.hip) ----
// element offset of an operand = base + sum_q batch_q * sb[q] + i * si + j * sj + k * sk (strides in elements;
// an index the operand does not depend on has stride 0)
struct BmmOperand {
  int64_t base, sb[3], si, sj, sk;
};
struct BmmArgs {
  float *C;
  const float *A, *B;
  const float *pre0, *pre1, *post;  // optional addends: before the activation (bias, mask) / after it (residual)
  BmmOperand c, a, b, p0, p1, r;
  int nb[3];                        // batch extents (1 where unused)
  int M, N, K;
  float alpha;
  int act;
};
int bmm_variant(const BmmArgs &a);  // 0 = neither layout fits
int launch_bmm(const BmmArgs &a);

// ---- KV cache as Q8_0 rows (kvq.hip): quant plane int8[max_len][KD], scale plane fp16[max_len][KD/32] ----
// the KV cache in pages (kvp.hip): rows per page; row r of a layer lives at pages[r / kKvPageRows] + (r % kKvPageRows) * KD
constexpr int kKvPageRows = 64;
int launch_kvp_append(float *const *kpages, float *const *vpages, const float *ksrc, const float *vsrc, int64_t src_stride, int s,
                      int row0, const int *pos, int KD);
int launch_kvp_gather(float *dst, const float *const *pages, int rows, int KD);
int launch_attn_paged(float *out, const float *q, const float *const *kpages, const float *const *vpages, int start_pos,
                      const int *pos, int H, int Hkv, int Dh);
struct AttnSplit;
int launch_attn_paged_step(float *out, const float *q, const float *newkv, float *const *kpages, float *const *vpages, const int *pos,
                           int H, int Hkv, int Dh, float rope_base, const AttnSplit *split);
int launch_kvq_append(void *q, void *d, const float *src, int64_t src_stride, int s, int row0, const int *pos, int KD);
int launch_kvq_dequant(float *dst, const void *q, const void *d, int rows, int KD);
int launch_attn_q8(float *out, const float *q, const void *kq, const void *kd, const void *vq, const void *vd, int start_pos,
                   const int *pos, int H, int Hkv, int Dh);
// one decode step over Q8_0 rows: rotation (rope_base > 0), quantisation and append of the new row (newkv: k then v,
// fp32, unrotated) and the attention in one launch; `split` as for launch_attn
struct AttnSplit;
int launch_attn_q8_step(float *out, const float *q, const float *newkv, void *kq, void *kd, void *vq, void *vd, const int *pos,
                        int H, int Hkv, int Dh, float rope_base, const AttnSplit *split);

// Arguments of one fused Linear launch:
//   y = act(prologue(x) . W^T + bias) + residual
// Output rows >= split1 / split2 are routed to y1 / y2 (fused-qkv rows going straight
// into the K / V cache), offset by (pos[0] + m) * pos_stride floats.
struct GemvArgs {
  float *y;
  float *y1;
  float *y2;
  const int *pos;
  int pos_stride;
  int split1, split2;
  const void *q;
  const unsigned short *d;
  const float *x;
  const float *bias;
  const float *residual;
  const float *norm_g;
  const float *norm_b;
  // LayerNorm folded through the product (see k_gemv): fold_s[r] = sum_k W[r,k]*gamma[k]; the caller
  // passes sum_k W[r,k]*beta[k] + b[r] as `bias`.  Null = normalise the input first.
  const float *fold_s;
  // with fold_s: the Linear's own bias (may be null), so that a launch that prefers to normalise the staged
  // input itself can undo the folding (fold_s = null, bias = bias0)
  const float *bias0;
  // rows 2r / 2r+1 are a (gate, up) pair: the launch writes silu(gate_r) * up_r to y[r] (rows/2 outputs)
  // instead of the two products.  Needs a variant with at least two rows per wavefront.
  int pair_swiglu;
  int stage_x;  // set by the launcher: the workgroup stages the input vector in LDS once
  float eps;
  int rows, cols;
  int act, pro;
  // A launch over a slice of the columns of a wider matrix (set by the launcher; 0 = the matrix is `cols` wide):
  // 16-byte chunks and block scales between the starts of two rows, and where the `up` half of a SwiGLU input
  // starts behind x (q, d and x then point at the slice's first column)
  int ld_chunks, ld_scales, up_off;
  int64_t x_stride, y_stride;  // between the m input / output vectors (blockIdx.y)
  // fused greedy argmax over the output rows (m == 1 only); all null when unused.
  // am_val/am_idx hold one partial (best value, lowest row) per wavefront of the launch.
  float *am_val;
  int *am_idx;
  long long *am_token64;
  int *am_tok;
  int *am_pos;
  long long *am_hist;
  int *am_hist_n;
  // stop condition of a device-resident loop: am_ctrl[0] = a token id that ends the sequence (-1 = none),
  // am_ctrl[1] = set to 1 by the step that produced it; from then on the steps still queued change nothing
  // (token, position and history stay as they are).  Null = no stop condition.
  int *am_ctrl;
  // the block that settles the token also gathers the next step's input, nx_out[d] = nx_wte[token][d] +
  // nx_wpe[position + 1][d] (the Embedding items of the next forward), so that a device-resident loop needs no
  // embedding launch between steps.  nx_out null = off; nx_wpe null = no position table.
  float *nx_out;
  const float *nx_wte, *nx_wpe;
  int nx_dim, nx_vocab, nx_max_pos;
};
// most wavefronts any GEMV launch uses (sizes the am_val / am_idx scratch)
constexpr int kGemvMaxWaves = 16384;
int launch_gemv(const WMat *w, GemvArgs a, int m);
// the same Linear by the wide-row kernel (gemv_wide.hip: input vector in LDS); a.q / a.d / a.rows / a.cols are set here
bool gemv_wide_supported(const WMat *w, const GemvArgs &a);
int launch_gemv_wide(const WMat *w, GemvArgs a, int m);
int wmat_create_impl(WMat **out, int type, const void *raw, int64_t rows, int64_t cols);
// true when a register-resident GEMV variant covers the matrix (no temporary is allocated at launch)
bool gemv_is_direct(const WMat *w);
// rows a wavefront of the register-resident variant for (type, cols) produces per pass; 0 = no such variant
int gemv_rows_per_wave(int type, int64_t cols);
// true when the single-row launch over a (rows, cols) matrix whose rows are gate / up rows in turn holds a row pair
// per wavefront, so that SwiGLU can be its epilogue
bool gemv_pair_swiglu_ok(int type, int64_t rows, int64_t cols);
// out[i] = silu(in[2i]) * in[2i+1], i < n (gate / up columns interleaved)
int launch_swiglu_pairs(float *out, const float *in, int64_t n);
// One query row over a long context: `ranges` workgroups per head share the keys (k_attn_cached, SPLIT).  part holds
// H x ranges x (head_dim + 2) floats, count H zeroed ints (each launch leaves them zeroed again).
struct AttnSplit {
  int ranges;
  float *part;
  int *count;
};
constexpr int kAttnSplitMaxRanges = 16;
#ifdef __HIPCC__
// Which head a workgroup of a decode attention launch takes.  Workgroups are dealt to the eight XCDs in turn (XCD =
// linear workgroup id mod 8, blockIdx.x running fastest).  With H a multiple of 8, head (b mod 8) * (H / 8) + b / 8
// puts consecutive heads -- the query heads that share a key / value head -- on ONE XCD: the group's cache rows enter
// one L2 instead of eight (70B shape at position 1940: 11.60 -> 10.96 ms per step).  Heads that share nothing keep
// the plain order, which spreads an XCD's reads over a cache row (7B shape: 3 % faster than the grouped order).
__device__ __forceinline__ int attn_head_of_block(int b, int H, int Hkv) {
  return ((H & 7) || H == Hkv) ? b : (b & 7) * (H >> 3) + (b >> 3);
}
#endif
int launch_attn(float *out, const float *q, const float *kc, const float *vc, int S, int start_pos, const int *pos,
                int max_T, int H, int Hkv, int Dh, const AttnSplit *split = nullptr);
int launch_embedding(float *out, const float *W, const float *idx_f, const int *idx_i, int ntok, int vocab, int dim,
                     const float *W2, const int *pos, int max_pos);
int launch_argmax(int64_t *out, const float *x, int64_t rows, int n, int *tok_out, int *pos, int64_t *history,
                  int *hist_n);
// Linear over m rows on the MFMA path (weights dequantised while staged).  precision: fp32 MFMA operands,
// operands rounded to bf16, or operands split in two / three bf16 terms (2^-16 / fp32-grade).
enum { GEMM_FP32 = 0, GEMM_BF16 = 1, GEMM_BF16X3 = 2, GEMM_BF16X6 = 3 };
// A split-K launch whose reduction the caller takes over (launch_reduce_norm): the raw partial tiles ws[z][m][n]
struct GemmDeferred {
  float *ws = nullptr;  // null: the launch did not split K, y is complete
  int ksplit = 0;
};
// defer: non-null = when the launch splits K, leave the partial tiles (bias / residual NOT applied) and hand them
// over instead of reducing them; the caller releases defer->ws with cthip_free after queuing its reduction
// Output columns routed to up to three destinations (a fused q/k/v projection whose thirds go to the query rows
// and to the cache rows of the two caches): columns [c0[i], c0[i + 1]) land in dst[i] with row pitch ld[i],
// first column at offset 0.  c0[0] = 0; every c0 is a multiple of 128 (whole tiles are routed); an unused
// third part has c0 = INT_MAX.
struct GemmRoute {
  float *dst[3];
  int c0[3];
  int ld[3];
};
// act == kActSwigluPairs: the weight rows are (gate_j, up_j) pairs and y (m, rows / 2) gets silu(gate_j) * up_j
// (SwiGLU, external/llm/layers.lisp:53-64, in the epilogue of the gate|up launch); K is not split then.
constexpr int kActSwigluPairs = 64;
// route: non-null = y is ignored, the columns go where the route says; K is not split then.
int launch_linear_gemm(float *y, const WMat *w, const float *x, int m, const float *bias, const float *residual,
                       int act, int precision, GemmDeferred *defer = nullptr, const GemmRoute *route = nullptr);
bool reduce_norm_supported(int n, int nparts);
// C (m, n) = sum_z ws[z] + bias + residual for partial tiles handed over through GemmDeferred
int launch_splitk_reduce(float *C, float *ws, int ksplit, int m, int n, const float *bias, const float *residual);
int launch_reduce_norm(float *y, float *xout, const float *parts, int nparts, int64_t part_stride, const float *bias,
                       const float *resid, const float *g, const float *b, float eps, int64_t rows, int n, bool rms);
// takes the device address of the static split-K scratch of cthip_matmul_noalloc (once per device, that device current)
int matmul_scratch_init(int device);
// gate|up rows (m, 2*cols) -> silu(gate)*up (m, cols), or a norm, as a launch of its own
int launch_prologue(float *out, const float *x, int cols, int pro, const float *g, const float *b, float eps,
                    int64_t x_stride, int m);
// prefill: split fused qkv rows (S, D+2KD) into q (S,D) and cache rows start_pos.., rotating q and k when rope_base > 0
int launch_qkv_split(float *q, float *kc, float *vc, const float *qkv, int S, int start_pos, int H, int Hkv, int Dh,
                     float rope_base);
int launch_attn_rope_append(float *out, const float *q, float *kc, float *vc, const float *newkv, const int *pos, int H,
                            int Hkv, int Dh, float base, const AttnSplit *split = nullptr);
int launch_rope_append(float *kc, float *vc, const float *kv, int Hkv, int Dh, float base, const int *pos);
int launch_rope(float *out, const float *x, int B, int S, int H, int Dh, float base, int start_pos, const int *pos);

}  // namespace cthip

// ---- device helpers ----
#if defined(__HIPCC__)
namespace cthip {

// Cross-lane reductions.  Steps inside a row of 16 lanes are DPP modifiers on the add itself
// (quad_perm xor 1, xor 2, row_half_mirror, row_mirror: a few cycles each, no LDS traffic); the four
// row totals of a wavefront are then combined through readlane.  A chain of ds_bpermute shuffles
// costs an LDS round trip per step, which dominates a short kernel's critical path.
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
// every lane gets the sum over its row of 16 lanes
__device__ __forceinline__ float row16_sum(float v) {
  v += dpp_f<0xB1>(v);   // quad_perm [1,0,3,2]
  v += dpp_f<0x4E>(v);   // quad_perm [2,3,0,1]
  v += dpp_f<0x141>(v);  // row_half_mirror
  v += dpp_f<0x140>(v);  // row_mirror
  return v;
}
__device__ __forceinline__ float row16_max(float v) {
  v = fmaxf(v, dpp_f<0xB1>(v));
  v = fmaxf(v, dpp_f<0x4E>(v));
  v = fmaxf(v, dpp_f<0x141>(v));
  v = fmaxf(v, dpp_f<0x140>(v));
  return v;
}
__device__ __forceinline__ float lane_bcast(float v, int lane) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}
__device__ __forceinline__ float wave_sum(float v) {
  v = row16_sum(v);
  return (lane_bcast(v, 0) + lane_bcast(v, 16)) + (lane_bcast(v, 32) + lane_bcast(v, 48));
}
__device__ __forceinline__ float wave_max(float v) {
  v = row16_max(v);
  return fmaxf(fmaxf(lane_bcast(v, 0), lane_bcast(v, 16)), fmaxf(lane_bcast(v, 32), lane_bcast(v, 48)));
}
// The four aligned groups of 16 lanes of a wavefront hold one value each (the same in every lane of a group): their
// maximum / sum, in every lane.  Four lane reads on the scalar unit; a butterfly of __shfl_xor is two trips through
// the LDS crossbar.  (All 64 lanes must be active.)
__device__ __forceinline__ float groups16_max(float v) {
  return fmaxf(fmaxf(lane_bcast(v, 0), lane_bcast(v, 16)), fmaxf(lane_bcast(v, 32), lane_bcast(v, 48)));
}
__device__ __forceinline__ float groups16_sum(float v) {
  return (lane_bcast(v, 0) + lane_bcast(v, 16)) + (lane_bcast(v, 32) + lane_bcast(v, 48));
}
// sum over aligned groups of G lanes (G = 16, 32, 64); every lane gets the group's sum
template <int G>
__device__ __forceinline__ float group_sum(float v) {
  if (G == 64) return wave_sum(v);
  v = row16_sum(v);
  if (G == 32) v += __shfl_xor(v, 16, 64);
  return v;
}

__device__ __forceinline__ float half_bits_to_float(unsigned short h) {
  return (float)__builtin_bit_cast(_Float16, h);
}

// Caten's decompositions (api/function.lisp:437-440, nn/activations.lisp:3-7,202-215,
// api/high-level-ops.lisp:112-117): exp(x) = exp2(x * 1/ln2); sigmoid = recip(1 + exp2(-x/ln2));
// tanh(y) = 2*sigmoid(2y) - 1.
__device__ __forceinline__ float ct_exp(float x) { return exp2f(x * 1.442695f); }
// The workgroup that drew a head's last ticket adds the ranges' triples up, in range order: `all` holds nranges
// records of dh unnormalised outputs, the running maximum and the running sum.  The loads are device-scope (they do
// not look into a cache that could hold an older launch's values) and ALL of them are requested before the first is
// used, so the merge costs one memory round trip whatever the number of ranges (one load after the other it cost a
// round trip per range).  Returns output column `col`.
__device__ __forceinline__ float attn_split_merge(const float *all, int nranges, int dh, int col) {
  float mv[kAttnSplitMaxRanges], lv[kAttnSplitMaxRanges], ov[kAttnSplitMaxRanges];
#pragma unroll
  for (int r = 0; r < kAttnSplitMaxRanges; r++) {
    const float *t = all + (int64_t)(r < nranges ? r : nranges - 1) * (dh + 2);
    mv[r] = __hip_atomic_load(t + dh, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    lv[r] = __hip_atomic_load(t + dh + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    ov[r] = __hip_atomic_load(t + col, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  float M = -INFINITY;
#pragma unroll
  for (int r = 0; r < kAttnSplitMaxRanges; r++)
    if (r < nranges) M = fmaxf(M, mv[r]);
  float o = 0.0f, L = 0.0f;
#pragma unroll
  for (int r = 0; r < kAttnSplitMaxRanges; r++) {
    if (r < nranges) {
      const float e = ct_exp(mv[r] - M);
      o = fmaf(e, ov[r], o);
      L = fmaf(e, lv[r], L);
    }
  }
  return o / L;
}
__device__ __forceinline__ float ct_sigmoid(float x) { return 1.0f / (1.0f + exp2f(x * -1.442695f)); }
__device__ __forceinline__ float ct_tanh(float y) { return 2.0f * ct_sigmoid(2.0f * y) - 1.0f; }
// GELU(tanh): 0.5 x (1 + tanh(u)) = x sigmoid(2u), u = sqrt(2/pi) (x + 0.044715 x^3) -- the same function without the
// cancellation in 1 + tanh(u) for negative x, as one exponential and one reciprocal (each within an ulp: the GEMM
// epilogue of c_fc spends a fifth of its launch on this function when it divides and handles subnormal exponentials)
__device__ __forceinline__ float ct_gelu(float x) {
  const float u2 = -2.3022082f * (x * fmaf(0.044715f * x, x, 1.0f));  // -2 u log2(e)
  return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(u2));
}
__device__ __forceinline__ float ct_silu(float x) { return x * ct_sigmoid(x); }
__device__ __forceinline__ float apply_act(int act, float v) {
  switch (act) {
    case CTHIP_ACT_RELU: return fmaxf(v, 0.0f);
    case CTHIP_ACT_GELU: return ct_gelu(v);
    case CTHIP_ACT_SILU: return ct_silu(v);
    case CTHIP_ACT_SIGMOID: return ct_sigmoid(v);
    case CTHIP_ACT_TANH: return ct_tanh(v);
    default: return v;
  }
}

// byte N of a dword as a float in one instruction.  Written out because the compiler, seeing the nibble mask,
// narrows every extract to a 4-bit field extract followed by a byte-0 conversion: two instructions per weight.
#define CTHIP_UBYTE(N)                                                  \
  __device__ __forceinline__ float ubyte##N##_f32(uint32_t v) {         \
    float f;                                                            \
    asm("v_cvt_f32_ubyte" #N " %0, %1" : "=v"(f) : "v"(v));             \
    return f;                                                           \
  }
CTHIP_UBYTE(0)
CTHIP_UBYTE(1)
CTHIP_UBYTE(2)
CTHIP_UBYTE(3)
#undef CTHIP_UBYTE
// the same for a signed byte: the conversion sign-extends the selected byte itself (otherwise a field extract first)
#define CTHIP_SBYTE(N)                                                                                          \
  __device__ __forceinline__ float sbyte##N##_f32(uint32_t v) {                                                 \
    float f;                                                                                                    \
    asm("v_cvt_f32_i32_sdwa %0, sext(%1) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_" #N : "=v"(f) : "v"(v)); \
    return f;                                                                                                   \
  }
CTHIP_SBYTE(0)
CTHIP_SBYTE(1)
CTHIP_SBYTE(2)
CTHIP_SBYTE(3)
#undef CTHIP_SBYTE

// RoPE of four consecutive elements of a head (positional-encoding.lisp:3-64) at position `at`: lane c holds elements
// 4c..4c+3 = pairs 2c and 2c+1 of the head; same arithmetic as k_rope.  The angles' sines and cosines depend on
// (c, at) only, so a launch that rotates a query and a key at the same place computes them once.
// the rotation of one pair with its roundings pinned, so that every kernel that rotates gives the same bits
__device__ __forceinline__ void rope_pair(float x0, float x1, float sn, float cs, float &o0, float &o1) {
  o0 = __fmaf_rn(x0, cs, -__fmul_rn(x1, sn));
  o1 = __fmaf_rn(x0, sn, __fmul_rn(x1, cs));
}
struct Rope4 {
  float sn[2], cs[2];
};
__device__ __forceinline__ Rope4 rope4_angles(int c, int DH, float log2_base, int at) {
  Rope4 r;
#pragma unroll
  for (int t = 0; t < 2; t++) {
    const int i = 2 * c + t;
    const float expo = (float)(2 * i) / (float)DH;
    const float logb = log2_base * 0.6931472f;
    const float theta = exp2f(-(expo * logb) * 1.442695f);
    const float ang = (float)at * theta;
    sincosf(ang, &r.sn[t], &r.cs[t]);
  }
  return r;
}
__device__ __forceinline__ float4 rope4_apply(float4 x, const Rope4 &r) {
  float4 o;
  rope_pair(x.x, x.y, r.sn[0], r.cs[0], o.x, o.y);
  rope_pair(x.z, x.w, r.sn[1], r.cs[1], o.z, o.w);
  return o;
}
__device__ __forceinline__ float4 rope4(float4 x, int c, int DH, float log2_base, int at) {
  return rope4_apply(x, rope4_angles(c, DH, log2_base, at));
}

}  // namespace cthip
#endif
