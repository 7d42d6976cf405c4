// Argument blocks and launchers of the three-launch decode layer (decode_fused.hip).
#pragma once
#include "common.h"

namespace cthip {

constexpr int kDecXcds = 8;  // accelerator dies of gfx950; one MLP accumulator each

constexpr float kFixScale = 4294967296.0f;             // 2^32
constexpr float kFixInv = 2.3283064365386963e-10f;     // 2^-32

// Fixed-point (2^-32) <-> float in a handful of instructions each (the 64-bit conversions of the language are a
// dozen): the integer part and the fraction are converted separately.  to_fix truncates the fraction below 2^-32
// (the same on every run, which is what the accumulators are for); from_fix is within an ulp of the rounded value.
// Magnitudes below 2^31.
__device__ __forceinline__ long long to_fix(float s) {
  const float fl = floorf(s);
  const unsigned lo = (unsigned)((s - fl) * kFixScale);  // s - floor(s) is exact, in [0, 1)
  return (long long)(((unsigned long long)(unsigned)(int)fl << 32) | lo);
}
__device__ __forceinline__ float from_fix(long long t) {
  return fmaf((float)(unsigned)t, kFixInv, (float)(int)(t >> 32));
}

__device__ __forceinline__ int xcd_id() {
  // XCC_ID hardware register (id 20), bits 3:0: the XCD this wavefront runs on
  return (int)__builtin_amdgcn_s_getreg((3 << 11) | (0 << 6) | 20) & (kDecXcds - 1);
}

__device__ __forceinline__ float4 f4add(float4 a, float4 b) { return make_float4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w); }

// how a launch assembles its input vector: x = base + bias + partial vectors
struct DecStage {
  const float *base;        // D floats
  const float *bias;        // D floats (unused when the launch takes the base alone)
  const float *fparts;      // fp32 partial vectors, D floats each (one per head)
  const long long *iparts;  // kDecXcds fixed-point (2^-32) accumulators, D each
  const float *gamma;       // LayerNorm gamma of the Linear that follows
  float *xout;              // block 0 stores the assembled vector here (may be null)
  float eps;
  int D;
};

struct DecQkvArgs {
  DecStage st;
  const void *wq;            // c_attn weights [3D][D] (int8 / fp16 / fp32)
  const unsigned short *wd;  // Q8_0: scale plane, fp16 [3D][D/32]
  const float *fold_s, *fold_c;  // W.gamma and W.beta + bias
  float *q, *kc, *vc;        // q (D), K / V cache (max_seq, D)
  const int *pos;
  int rows;                  // 3D
  int kv_stride;             // floats between cache rows: D; 0 = kc / vc are one row (the new row goes to a buffer)
};

struct DecAttnArgs {
  const float *q, *kc, *vc;
  const int *pos;
  const void *pq;            // attn.c_proj by head: [H][D][Dh]
  const unsigned short *pd;  // Q8_0: fp16 [H][D][Dh/32]
  float *part;               // out: fp32 [H][D], head h's share of the projection
  void *zero;                // cleared here: the MLP accumulators
  int64_t zero_n16;          // ... in 16-byte units
  const float *att_in;       // null, or the heads' attention outputs [H][Dh] from a launch of its own: projection only
};

// the same launch over a cache kept as Q8_0 rows (kvq.hip): the step's new key / value row arrives as fp32 (k then v,
// D floats each), is quantised here, joins the keys as the last row and is stored into the planes
struct DecAttnQ8Args {
  const float *q, *newkv;
  signed char *kq, *vq;        // quant planes int8 [max_seq][D]
  unsigned short *kd, *vd;     // scale planes fp16 [max_seq][D / 32]
  const int *pos;
  const void *pq;
  const unsigned short *pd;
  float *part;
  void *zero;
  int64_t zero_n16;
};

struct DecMlpArgs {
  DecStage st;
  const void *wq;            // c_fc weights [F][D]
  const unsigned short *wd;  // Q8_0: fp16 [F][D/32]
  const float *fold_s, *fold_c;
  const void *pq;            // mlp.c_proj by 16-column slab: [F/16][D][16]
  const unsigned short *pd;  // Q8_0: fp16 [F/32][D]
  long long *accum;          // [kDecXcds][D]
};

#ifdef CTHIP_DECODE_DEVICE_HELPERS
// Weight formats of the fused launches: a 16-byte chunk holds XPC weights (Q8_0: 16 int8, Q4_0: 32 nibbles = one
// block, fp16: 8, fp32: 4); the quantised formats have a scale plane (one fp16 per 32 weights).  LPR lanes share a
// row: 16, or 8 where a chunk is a whole block of 32 (a row of D = 256 KC columns is then 8 KC chunks).  Rows whose
// chunks are 128 bytes of the staged vector apart are read from LDS with the 16-byte slot index xor-ed by the
// block index (SWZ), or every lane of a row group would hit the same banks.
template <int TYPE>
struct DecFmt {
  static constexpr int XPC = Fmt<TYPE>::XPC;
  static constexpr bool QUANT = TYPE == CTHIP_Q8_0 || TYPE == CTHIP_Q4_0;
  static constexpr int LPR = XPC >= 32 ? 8 : 16;
  static constexpr bool SWZ = XPC >= 32;
  static constexpr int RPW = 64 / LPR;  // rows per wavefront
};

// float4 slot of the i4-th float4 of a staged vector
template <bool SWZ>
__device__ __forceinline__ int dec_slot(int i4) {
  if (!SWZ) return i4;
  const int blk = i4 >> 3;
  return (blk << 3) | ((i4 ^ blk) & 7);
}

// XPC consecutive floats of a vector in LDS
template <int XPC>
__device__ __forceinline__ void lds_floats(const float *p, float *xr) {
#pragma unroll
  for (int t = 0; t < XPC / 4; t++) {
    const float4 v = *(const float4 *)(p + 4 * t);
    xr[4 * t + 0] = v.x;
    xr[4 * t + 1] = v.y;
    xr[4 * t + 2] = v.z;
    xr[4 * t + 3] = v.w;
  }
}

// chunk c of a staged vector (swizzled where the format says so); returns the sum of its floats where the format
// needs it (Q4_0 stores n + 8), else 0
template <int TYPE>
__device__ __forceinline__ float dec_chunk_floats(const float *xs, int c, float *xr) {
  constexpr int XPC = DecFmt<TYPE>::XPC;
  if (!DecFmt<TYPE>::SWZ) {
    lds_floats<XPC>(xs + c * XPC, xr);
    return 0.0f;
  }
  float part[8];
#pragma unroll
  for (int k = 0; k < 8; k++) {
    const float4 v = ((const float4 *)xs)[(c << 3) | ((k ^ c) & 7)];
    xr[4 * k + 0] = v.x;
    xr[4 * k + 1] = v.y;
    xr[4 * k + 2] = v.z;
    xr[4 * k + 3] = v.w;
    part[k] = (v.x + v.y) + (v.z + v.w);
  }
  return ((part[0] + part[1]) + (part[2] + part[3])) + ((part[4] + part[5]) + (part[6] + part[7]));
}

// sum over the LPR lanes of a row
template <int LPR>
__device__ __forceinline__ float dec_row_sum(float v) {
  v += dpp_f<0xB1>(v);   // quad_perm [1,0,3,2]
  v += dpp_f<0x4E>(v);   // quad_perm [2,3,0,1]
  v += dpp_f<0x141>(v);  // row_half_mirror
  if (LPR == 16) v += dpp_f<0x140>(v);  // row_mirror
  return v;
}

// One row of D = 256 * KC weights against the staged vector: LPR lanes per row, lane l owns chunks l + LPR j.  Two
// running sums: a chain of dependent FMAs issues at half rate when the SIMD holds one wavefront.
template <int TYPE, int KC>
__device__ __forceinline__ float dec_row_dot(const uint4 *w, const unsigned *sc, const float *xs, int l) {
  constexpr int XPC = DecFmt<TYPE>::XPC, LPR = DecFmt<TYPE>::LPR, NCL = KC * 256 / XPC / LPR;
  float acc[2] = {0.0f, 0.0f};
#pragma unroll
  for (int j = 0; j < NCL; j++) {
    const int c = l + LPR * j;
    float xr[XPC];
    const float xsum = dec_chunk_floats<TYPE>(xs, c, xr);
    acc[j & 1] += chunk_dot<TYPE>(w[j], DecFmt<TYPE>::QUANT ? half_bits_to_float((unsigned short)sc[j]) : 1.0f, xr, xsum);
  }
  return dec_row_sum<LPR>(acc[0] + acc[1]);
}

// requests of one row's chunks (and block scales) for dec_row_dot
template <int TYPE, int KC>
__device__ __forceinline__ void dec_row_request(const void *wq, const unsigned short *wd, int64_t row, int l, uint4 *w, unsigned *sc) {
  constexpr int XPC = DecFmt<TYPE>::XPC, LPR = DecFmt<TYPE>::LPR, NCL = KC * 256 / XPC / LPR;
  const uint4 *qp = (const uint4 *)wq + row * (LPR * NCL);
#pragma unroll
  for (int j = 0; j < NCL; j++) {
    const int c = l + LPR * j;
    w[j] = qp[c];
    if (DecFmt<TYPE>::QUANT) sc[j] = wd[row * (8 * KC) + ((c * XPC) >> 5)];
    else sc[j] = 0;
  }
}

#endif  // CTHIP_DECODE_DEVICE_HELPERS

bool dec_fused_supported(int type_attn, int type_proj, int type_fc, int type_fc2, int D, int H, int F);
int dec_xcd_probe(int *max_id);
int dec_relay_heads(const WMat *w, int DH, void **pq, void **pd);
int dec_relay_slabs(const WMat *w, void **pq, void **pd);  // slabs of 16 columns (a whole block of 32 for Q4_0)
int launch_dec_qkv(const DecQkvArgs &a, int type, bool from_accum);
int launch_dec_attn_proj(const DecAttnArgs &a, int type, int H, int D, int replicas);
int launch_dec_attn_proj_q8(const DecAttnQ8Args &a, int type, int H, int D, int replicas);
int launch_dec_mlp(const DecMlpArgs &a, int type, int F, int H);
int launch_dec_sum(const DecStage &s, float *out);

}  // namespace cthip

// ---- all layers of a step as one launch of role-specialised workgroups (decode_flow.hip) ----
namespace cthip {

struct FlowLayer {
  const void *attn_q;             // c_attn quant plane int8 [3D][D]
  const unsigned short *attn_d;   // ... scale plane fp16 [3D][D/32]
  const float *attn_s, *attn_c;   // LayerNorm1 folded through c_attn: W.gamma, W.beta + bias
  const void *proj_q;             // attn.c_proj int8 [D][D]
  const unsigned short *proj_d;   // fp16 [D][D/32]
  const float *proj_b;
  const void *fc_q;               // c_fc int8 [F][D]
  const unsigned short *fc_d;     // fp16 [F][D/32]
  const float *fc_s, *fc_c;       // LayerNorm2 folded through c_fc
  const void *fc2_sq;             // mlp.c_proj by 32-column slab: int8 [F/32][D][32]
  const unsigned short *fc2_sd;   // fp16 [F/32][D]
  const float *fc2_b;
  const float *ln1_g, *ln2_g;
  float *kc, *vc;                 // K / V cache (max_seq, D)
};

struct FlowArgs {
  const FlowLayer *layers;        // device array, n_layers entries
  int n_layers, D, H, F, NM;      // NM = F / 32
  float eps;
  // tagged elements (value in the low, tag in the high 32 bits), one buffer per (layer, phase)
  // (X, O and XP are broadcast to many workgroups and kept in several copies: [copies][n_layers][D])
  unsigned long long *X;          // [n_layers][D]       a layer's input (layer 0 reads x0 instead)
  unsigned long long *QKV;        // [n_layers][3D]
  unsigned long long *O;          // [n_layers][D]       the heads' attention outputs
  unsigned long long *XP;         // [n_layers][D]       x' = x + attention
  unsigned long long *PM;         // [n_layers][NM][D]   the MLP workgroups' shares of mlp.c_proj
  const float *x0;                // the step's input row (fp32, written by an earlier launch)
  float *x_out;                   // the residual vector after the last layer, for lm_head
  const int *tokpos;              // [1] = position
  int *state;                     // [0] = epoch of the next step's tags, [1] = a waiter gave up
  long long *trace;               // null, or [workgroups][n_layers][4] clock stamps of the last step (option decode_flow 2)
};

bool dec_flow_supported(int type_attn, int type_proj, int type_fc, int type_fc2, int D, int H, int F, int n_layers);
int dec_flow_grid(int D, int H, int F);
void dec_flow_copies(int *x, int *o, int *xp);  // copies kept of the buffers X, O, XP
int launch_dec_flow(const FlowArgs &a);

}  // namespace cthip

// ---- the same three launches for RMSNorm / RoPE / grouped-query / SwiGLU layers with Q4_0 weights (decode_gqa.hip) ----
namespace cthip {

struct GqaStage {
  const float *base;        // D floats
  const long long *iparts;  // kDecXcds fixed-point accumulators, D each (unused when the launch takes the base alone)
  const float *gamma;       // RMSNorm weight of the Linear that follows
  float *xout;              // block 0 stores the assembled vector here
  float eps;
  int D;
};

struct GqaQkvArgs {
  GqaStage st;
  const void *wq;            // wq|wk|wv quant plane, Q4_0 [D + 2 KD][D / 2] bytes
  const unsigned short *wd;  // fp16 [D + 2 KD][D / 32]
  float *q, *kc, *vc;        // q (D, rotated), K / V cache (max_seq, KD): the new key is stored rotated
  const int *pos;
  int rows, KD, DH;
  float log2_base;           // log2 of the RoPE base
  void *zero;                // cleared here: the attention launch's accumulators (may be null)
  int64_t zero_n16;          // ... in 16-byte units
};

struct GqaAttnArgs {
  const float *q, *kc, *vc;
  const int *pos;
  const void *pq;            // wo by query head: Q4_0 [H][D][Dh / 2] bytes
  const unsigned short *pd;  // fp16 [H][D][Dh / 32]
  long long *accum;          // [kDecXcds][D]
  void *zero;                // cleared here: the MLP launch's accumulators
  int64_t zero_n16;
  int D, KD;
  const float *att_in;       // null, or the heads' attention outputs [H][Dh] from a launch of its own: projection only
};

struct GqaMlpArgs {
  GqaStage st;
  const void *wq;            // gate / up quant plane, Q4_0 [2F][D / 2] bytes
  const unsigned short *wd;  // fp16 [2F][D / 32]
  int gate_stride, up_off;   // hidden unit j: gate row j * gate_stride, up row j * gate_stride + up_off
  const void *pq;            // down by 32-column slab: Q4_0 [F / 32][D][16] bytes
  const unsigned short *pd;  // fp16 [F / 32][D]
  long long *accum;          // [kDecXcds][D]
};

bool gqa_fused_supported(int type_attn, int type_proj, int type_fc, int type_fc2, int D, int H, int HKV, int F);
int gqa_relay_groups(const WMat *w, int group_cols, void **pq, void **pd);
int gqa_relay_slabs(const WMat *w, void **pq, void **pd);
int launch_gqa_qkv(const GqaQkvArgs &a, bool from_accum);
int launch_gqa_attn_proj(const GqaAttnArgs &a, int H, int HKV, int replicas);
int launch_gqa_mlp(const GqaMlpArgs &a, int F, int HKV);

}  // namespace cthip
