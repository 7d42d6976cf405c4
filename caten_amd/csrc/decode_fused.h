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
};

struct DecAttnArgs {
  const float *q, *kc, *vc;
  const int *pos;
  const void *pq;            // attn.c_proj by head: [H][D][Dh]
  const unsigned short *pd;  // Q8_0: fp16 [H][D][Dh/32]
  float *part;               // out: fp32 [H][D], head h's share of the projection
  void *zero;                // cleared here: the MLP accumulators
  int64_t zero_n16;          // ... in 16-byte units
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

bool dec_fused_supported(int type_attn, int type_proj, int type_fc, int type_fc2, int D, int H, int F);
int dec_xcd_probe(int *max_id);
int dec_relay_heads(const WMat *w, int DH, void **pq, void **pd);
int dec_relay_slabs(const WMat *w, void **pq, void **pd);
int launch_dec_qkv(const DecQkvArgs &a, int type, bool from_accum);
int launch_dec_attn_proj(const DecAttnArgs &a, int type, int H, int D, int replicas);
int launch_dec_mlp(const DecMlpArgs &a, int type, int F, int H);
int launch_dec_sum(const DecStage &s, float *out);

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
