/*
 * caten_oracle.c -- TEST INFRASTRUCTURE ONLY.  Nothing shipped may call this.
 *
 * A single-threaded plain-C restatement of what Caten's BACKEND=CLANG path
 * computes for the GPT-2 / Llama shaped decode path: one C function per fused
 * schedule item, written the way Caten's CStyle renderer spells its kernels
 * (source/byoc/clang.lisp:21-125, source/codegen/renderer.lisp:314-411):
 *   - nested `for` loops, one scalar `float acc = 0.0` per reduction,
 *     sequential accumulation in index order;
 *   - float literals WITHOUT an `f` suffix, i.e. doubles, printed with the
 *     shortest digits that identify the single-float constant (1.442695,
 *     0.7978846, ...), and libm `sin exp2 log2 sqrt` on doubles;
 *   - RECIP spelled `1.0/(x)` with no outer parentheses, so `(a*1.0/(b))`
 *     evaluates as the double quotient a/b rounded once on store;
 *   - `max(a,b)` as the ((a)>(b)?(a):(b)) macro.
 * Values are rounded to float wherever the reference stores them (array
 * elements and scalar accumulators).
 *
 * What pins it (tests/test_oracle_*.py): PyTorch library routines on the same
 * inputs at the tolerances the reference's own test-suite uses, the literal
 * golden vectors held in the reference's tests (embedding, argmax, triu/tril,
 * all-ones gemm), exhaustive fp16 x int8 products against NumPy's IEEE half
 * conversion, and an independent fp64 PyTorch decoder for the whole forward.
 *
 * PARITY UNPINNED by the reference (it has no implementation to compare to):
 *   orc_dequant_q4_0 / orc_quantize_q4_0 (tensor-info.lisp:36-41 errors "Not
 *   ready"; layout restated from ggml's public block_q4_0 definition), the
 *   Llama-shaped decoder (no GQA/SwiGLU model in the reference) and the RoPE
 *   position offset (positional-encoding.lisp:3-64 has positions 0..seq-1
 *   only).  They are pinned by closed forms / PyTorch restatements instead.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define _negative_infinity (-INFINITY)
#define max(a, b) ((a) > (b) ? (a) : (b))

/* ------------------------------------------------------------------ */
/* IEEE half <-> single.  Reference: decode-float16 is                 */
/* ieee-floats:make-float-converters with 5 exponent / 10 significand  */
/* bits, denormals supported (source/common/dtype.lisp:160-164), read   */
/* little-endian (external/gguf/helpers.lisp:12-15).                   */
/* ------------------------------------------------------------------ */
float orc_f16_to_f32(uint16_t h) {
  int sign = (h >> 15) & 1;
  int e = (h >> 10) & 0x1f;
  int m = h & 0x3ff;
  float v;
  if (e == 0) {
    v = ldexpf((float)m, -24); /* zero and denormals: m * 2^-24 */
  } else if (e == 31) {
    v = m ? NAN : INFINITY;
  } else {
    v = ldexpf((float)(m | 0x400), e - 25); /* (1024+m) * 2^(e-15-10) */
  }
  return sign ? -v : v;
}

/* round-to-nearest-even single -> half; used only by the quantisers */
uint16_t orc_f32_to_f16(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t ax = x & 0x7fffffffu;
  if (ax >= 0x7f800000u) { /* inf / nan */
    return (uint16_t)(sign | 0x7c00u | ((ax > 0x7f800000u) ? 0x200u : 0));
  }
  if (ax >= 0x477ff000u) { /* rounds to >= 65520 -> inf */
    return (uint16_t)(sign | 0x7c00u);
  }
  if (ax < 0x33000001u) { /* < 2^-25 (or == 2^-25 which ties to even 0) */
    return (uint16_t)sign;
  }
  int e = (int)(ax >> 23) - 127;
  uint32_t man = (ax & 0x7fffffu) | 0x800000u; /* 24-bit significand */
  int shift; /* bits to drop */
  uint32_t base;
  if (e < -14) { /* half denormal: value = man * 2^(e-23); unit = 2^-24 */
    shift = -e - 1; /* 13 + (-14 - e) */
    base = 0;
  } else {
    shift = 13;
    base = (uint32_t)(e + 15) << 10;
    man &= 0x7fffffu;
  }
  uint32_t q = man >> shift;
  uint32_t rem = man & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1);
  if (rem > half || (rem == half && (q & 1u))) q++;
  return (uint16_t)(sign | (base + q)); /* carry into exponent is correct */
}

void orc_dequant_f16(const uint8_t *src, int64_t n, float *out) {
  /* external/gguf/dequantize.lisp:27-38 */
  for (int64_t i = 0; i < n; i++) {
    uint16_t h = (uint16_t)(src[2 * i] | (src[2 * i + 1] << 8));
    out[i] = orc_f16_to_f32(h);
  }
}

void orc_dequant_f32(const uint8_t *src, int64_t n, float *out) {
  /* external/gguf/dequantize.lisp:14-25 : little-endian IEEE single */
  for (int64_t i = 0; i < n; i++) {
    uint32_t u = (uint32_t)src[4 * i] | ((uint32_t)src[4 * i + 1] << 8) |
                 ((uint32_t)src[4 * i + 2] << 16) | ((uint32_t)src[4 * i + 3] << 24);
    memcpy(&out[i], &u, 4);
  }
}

void orc_dequant_q8_0(const uint8_t *blocks, int64_t n, float *out) {
  /* external/gguf/dequantize.lisp:40-53 : per block of 32, an fp16 scale then
   * up to 32 signed bytes; out = qval * scale in single float.  The last
   * block may be short. */
  int64_t nblocks = (n + 31) / 32;
  int64_t idx = 0;
  const uint8_t *p = blocks;
  for (int64_t b = 0; b < nblocks; b++) {
    float scale = orc_f16_to_f32((uint16_t)(p[0] | (p[1] << 8)));
    p += 2;
    int64_t in_block = (n - idx) < 32 ? (n - idx) : 32;
    for (int64_t i = 0; i < in_block; i++) {
      int8_t q = (int8_t)*p++;
      out[idx++] = (float)q * scale;
    }
  }
}

void orc_dequant_q4_0(const uint8_t *blocks, int64_t n, float *out) {
  /* Not in the reference (tensor-info.lisp:7 knows type id 2 only).
   * ggml block_q4_0: fp16 d, then 16 bytes; element j<16 is the low nibble of
   * byte j minus 8, element j+16 the high nibble minus 8; times d.
   * n must be a multiple of 32. */
  int64_t nblocks = n / 32;
  for (int64_t b = 0; b < nblocks; b++) {
    const uint8_t *p = blocks + 18 * b;
    float d = orc_f16_to_f32((uint16_t)(p[0] | (p[1] << 8)));
    for (int j = 0; j < 16; j++) {
      int lo = (p[2 + j] & 0x0f) - 8;
      int hi = (p[2 + j] >> 4) - 8;
      out[32 * b + j] = (float)lo * d;
      out[32 * b + j + 16] = (float)hi * d;
    }
  }
}

/* Quantisers: the build's own choice (the reference only reads quantised
 * files); they follow ggml's reference row quantisers so that files written
 * by ggml tools and synthetic weights made here share one convention. */
void orc_quantize_q8_0(const float *w, int64_t n, uint8_t *blocks) {
  int64_t nblocks = n / 32;
  for (int64_t b = 0; b < nblocks; b++) {
    float amax = 0.0f;
    for (int j = 0; j < 32; j++) {
      float a = fabsf(w[32 * b + j]);
      if (a > amax) amax = a;
    }
    float d = amax / 127.0f;
    float id = d ? 1.0f / d : 0.0f;
    uint16_t h = orc_f32_to_f16(d);
    uint8_t *p = blocks + 34 * b;
    p[0] = (uint8_t)(h & 0xff);
    p[1] = (uint8_t)(h >> 8);
    for (int j = 0; j < 32; j++) {
      p[2 + j] = (uint8_t)(int8_t)roundf(w[32 * b + j] * id);
    }
  }
}

void orc_quantize_q4_0(const float *w, int64_t n, uint8_t *blocks) {
  int64_t nblocks = n / 32;
  for (int64_t b = 0; b < nblocks; b++) {
    float amax = 0.0f, mx = 0.0f;
    for (int j = 0; j < 32; j++) {
      float v = w[32 * b + j];
      if (amax < fabsf(v)) {
        amax = fabsf(v);
        mx = v;
      }
    }
    float d = mx / -8.0f;
    float id = d ? 1.0f / d : 0.0f;
    uint16_t h = orc_f32_to_f16(d);
    uint8_t *p = blocks + 18 * b;
    p[0] = (uint8_t)(h & 0xff);
    p[1] = (uint8_t)(h >> 8);
    for (int j = 0; j < 16; j++) {
      float x0 = w[32 * b + j] * id;
      float x1 = w[32 * b + 16 + j] * id;
      int xi0 = (int)(int8_t)(x0 + 8.5f);
      int xi1 = (int)(int8_t)(x1 + 8.5f);
      if (xi0 > 15) xi0 = 15;
      if (xi1 > 15) xi1 = 15;
      p[2 + j] = (uint8_t)(xi0 | (xi1 << 4));
    }
  }
}

/* ------------------------------------------------------------------ */
/* Fused items                                                         */
/* ------------------------------------------------------------------ */

/* !matmul (source/api/high-level-ops.lisp:76-99): C[i,k] = sum_j A[i,j]*B[j,k]
 * rendered as in test-scheduler.lisp:126-135 / scripts/gemm/gemm.c:47-252;
 * relu!=0 appends the fused ReLU epilogue max(acc, 0.0)
 * (nn/activations.lisp:34-44, fusion per test-scheduler.lisp:140-163). */
void orc_matmul(const float *A, const float *B, float *C, int M, int N, int K, int relu) {
  for (int i = 0; i < M; i++) {
    for (int k = 0; k < N; k++) {
      float acc = 0.0;
      for (int j = 0; j < K; j++) {
        acc = (acc + (A[K * i + j] * B[k + N * j]));
      }
      C[N * i + k] = relu ? max(acc, 0.0) : acc;
    }
  }
}

/* Linear (source/nn/linear.lisp:3-17): y = x @ W^T (+ b), W is (N,K) row
 * major read through a transposing view. */
void orc_linear(const float *x, const float *W, const float *b, float *y, int M, int K, int N) {
  for (int i = 0; i < M; i++) {
    for (int o = 0; o < N; o++) {
      float acc = 0.0;
      const float *w = W + (int64_t)K * o;
      for (int k = 0; k < K; k++) {
        acc = (acc + (x[(int64_t)K * i + k] * w[k]));
      }
      y[(int64_t)N * i + o] = b ? (acc + b[o]) : acc;
    }
  }
}

void orc_relu(const float *x, float *y, int64_t n) {
  for (int64_t i = 0; i < n; i++) y[i] = max(x[i], 0.0);
}

/* Sigmoid (nn/activations.lisp:3-7): recip(1 + exp2(x * (-1/ln2))) */
static inline double sigmoid_d(double z) { return 1.0 / ((1.0 + exp2((z * -1.442695)))); }
/* TanhNode (api/high-level-ops.lisp:112-117): 2*sigmoid(2x) - 1 */
static inline double tanh_d(double y) { return ((2.0 * sigmoid_d((2.0 * y))) + -1.0); }

void orc_sigmoid(const float *x, float *y, int64_t n) {
  for (int64_t i = 0; i < n; i++) y[i] = sigmoid_d(x[i]);
}
void orc_tanh(const float *x, float *y, int64_t n) {
  for (int64_t i = 0; i < n; i++) y[i] = tanh_d(x[i]);
}
/* GeLU :tanh (nn/activations.lisp:202-215) */
static inline float gelu_f(float x) {
  return ((0.5 * x) * (1.0 + tanh_d((0.7978846 * (x + (0.044715 * ((x * x) * x)))))));
}
void orc_gelu_tanh(const float *x, float *y, int64_t n) {
  for (int64_t i = 0; i < n; i++) y[i] = gelu_f(x[i]);
}
/* SiLU (nn/activations.lisp:180-189): x * sigmoid(x) */
static inline float silu_f(float x) { return (x * sigmoid_d(x)); }
void orc_silu(const float *x, float *y, int64_t n) {
  for (int64_t i = 0; i < n; i++) y[i] = silu_f(x[i]);
}

/* Softmax over the last axis (nn/activations.lisp:59-62,107-119): m = x-max;
 * e = exp2(m * 1/ln2) (api/function.lisp:437-440); e * recip(sum e). */
void orc_softmax(const float *x, float *y, int64_t rows, int n) {
  for (int64_t r = 0; r < rows; r++) {
    const float *xr = x + r * n;
    float *yr = y + r * n;
    float m = _negative_infinity;
    for (int k = 0; k < n; k++) m = max(m, xr[k]);
    float s = 0.0;
    for (int k = 0; k < n; k++) {
      float e = exp2(((xr[k] + -(m)) * 1.442695));
      yr[k] = e;
      s = (s + e);
    }
    for (int k = 0; k < n; k++) yr[k] = (yr[k] * 1.0 / (s));
  }
}

/* LayerNorm over the last axis (nn/normalization.lisp:39-58); mean is
 * sum * recip(cast N) (api/high-level-ops.lisp:46-56); variance is biased. */
void orc_layernorm(const float *x, const float *gamma, const float *beta, double eps, float *y,
                   int64_t rows, int n) {
  for (int64_t r = 0; r < rows; r++) {
    const float *xr = x + r * n;
    float *yr = y + r * n;
    float s = 0.0;
    for (int k = 0; k < n; k++) s = (s + xr[k]);
    float u = (s * 1.0 / ((float)n));
    float v = 0.0;
    for (int k = 0; k < n; k++) {
      float d = (xr[k] + -(u));
      v = (v + (d * d));
    }
    float var = (v * 1.0 / ((float)n));
    for (int k = 0; k < n; k++) {
      float d = (xr[k] + -(u));
      float t = (d * 1.0 / (sqrt((var + eps))));
      if (gamma) t = (t * gamma[k]);
      if (beta) t = (t + beta[k]);
      yr[k] = t;
    }
  }
}

/* RMSNorm (nn/normalization.lisp:70-85): x * recip(sqrt(eps + mean(x*x))) * w */
void orc_rmsnorm(const float *x, const float *w, double eps, float *y, int64_t rows, int n) {
  for (int64_t r = 0; r < rows; r++) {
    const float *xr = x + r * n;
    float *yr = y + r * n;
    float s = 0.0;
    for (int k = 0; k < n; k++) s = (s + (xr[k] * xr[k]));
    float ms = (s * 1.0 / ((float)n));
    for (int k = 0; k < n; k++) {
      float t = (xr[k] * 1.0 / (sqrt((eps + ms))));
      if (w) t = (t * w[k]);
      yr[k] = t;
    }
  }
}

/* RoPE (nn/positional-encoding.lisp:3-64): x is (B,S,H,Dh), interleaved pairs
 * (x[2i], x[2i+1]); theta_i = exp(-((2i)/Dh) * ln(base)) with exp/log spelled
 * through exp2/log2; cos(a) = sin(a + pi/2) (high-level-ops.lisp:119-122).
 * The reference rotates positions 0..S-1; `start_pos` (not in the reference)
 * shifts them so a KV-cached decode step can rotate position n. */
void orc_rope(const float *x, float *out, int B, int S, int H, int Dh, double base, int start_pos) {
  int dim = Dh / 2;
  for (int b = 0; b < B; b++)
    for (int s = 0; s < S; s++)
      for (int h = 0; h < H; h++)
        for (int i = 0; i < dim; i++) {
          float expo = (((float)i * 2.0) * 1.0 / ((float)Dh));
          float logb = (log2((float)base) * 0.6931472);
          float theta = exp2((-((expo * logb)) * 1.442695));
          float ang = ((float)(s + start_pos) * theta);
          float c = sin((ang + 1.5707964));
          float sn = sin(ang);
          int64_t o = (((int64_t)b * S + s) * H + h) * Dh + 2 * i;
          float x0 = x[o], x1 = x[o + 1];
          out[o] = ((x0 * c) + -((x1 * sn)));
          out[o + 1] = ((x0 * sn) + (x1 * c));
        }
}

/* Embedding (nn/embedding.lisp:3-25): a one-hot masked sum over the whole
 * vocabulary, indices compared as floats: out[t,d] = sum_v (v==idx[t] ? W[v,d] : 0) */
void orc_embedding_onehot(const float *W, const float *idx, float *out, int ntok, int V, int D) {
  for (int t = 0; t < ntok; t++) {
    for (int d = 0; d < D; d++) {
      float acc = 0.0;
      for (int v = 0; v < V; v++) {
        acc = (acc + (((float)v == idx[t]) ? W[(int64_t)D * v + d] : 0.0));
      }
      out[(int64_t)D * t + d] = acc;
    }
  }
}

/* ArgMaxNode (api/high-level-ops.lisp:314-343): idx' = (N-1) - i in floats;
 * map = where(x == max(x), idx', 0); result = cast_int64(N - max(map) - 1),
 * i.e. the LOWEST index among ties. */
int64_t orc_argmax(const float *x, int n) {
  float m = _negative_infinity;
  for (int i = 0; i < n; i++) m = max(m, x[i]);
  float best = _negative_infinity;
  for (int i = 0; i < n; i++) {
    float idx = (((float)n + -1.0) + ((float)i * -1.0));
    float mp = (x[i] == m) ? idx : 0.0;
    best = max(best, mp);
  }
  return (int64_t)((((float)n + -(best)) + -1.0));
}

/* TriuNode applied to full(-inf) (api/high-level-ops.lisp:278-307,
 * external/llm/layers.lisp:83): mask[i,j] = (i <= j-k) ? -inf : 0 */
void orc_triu_neginf(float *mask, int rows, int cols, int k) {
  for (int i = 0; i < rows; i++)
    for (int j = 0; j < cols; j++) mask[(int64_t)cols * i + j] = (i <= j - k) ? _negative_infinity : 0.0;
}
void orc_triu(const float *x, float *y, int rows, int cols, int k) {
  for (int i = 0; i < rows; i++)
    for (int j = 0; j < cols; j++) y[(int64_t)cols * i + j] = (i <= j - k) ? x[(int64_t)cols * i + j] : 0.0;
}
void orc_tril(const float *x, float *y, int rows, int cols, int k) {
  for (int i = 0; i < rows; i++)
    for (int j = 0; j < cols; j++) y[(int64_t)cols * i + j] = (i >= j - k) ? x[(int64_t)cols * i + j] : 0.0;
}

/* scaled-dot-product-attention (external/llm/layers.lisp:3-5) on one
 * (S,H,Dh) query block against a (T,Hkv,Dh) key/value block laid out as the
 * KV cache is ((B,maxlen,H,Dh), layers.lisp:19-33).  Query head h reads
 * key/value head h / (H/Hkv) (GQA; Hkv == H in the reference).
 * scores = q.k * 1.0/(sqrt(Dh)) + mask ; softmax ; @ v.   out is (S,H,Dh),
 * i.e. already permuted back (layers.lisp:46-49).  scratch: S*T floats. */
void orc_sdpa(const float *q, const float *k, const float *v, const float *mask, float *out, int S,
              int T, int H, int Hkv, int Dh, float *scratch) {
  int rep = H / Hkv;
  float sq = sqrtf((float)Dh);
  for (int h = 0; h < H; h++) {
    int hk = h / rep;
    for (int i = 0; i < S; i++) {
      for (int j = 0; j < T; j++) {
        float acc = 0.0;
        for (int d = 0; d < Dh; d++) {
          acc = (acc + (q[((int64_t)i * H + h) * Dh + d] * k[((int64_t)j * Hkv + hk) * Dh + d]));
        }
        float sc = (acc * 1.0 / (sq));
        if (mask) sc = (sc + mask[(int64_t)T * i + j]);
        scratch[(int64_t)T * i + j] = sc;
      }
    }
    orc_softmax(scratch, scratch, S, T);
    for (int i = 0; i < S; i++) {
      for (int d = 0; d < Dh; d++) {
        float acc = 0.0;
        for (int j = 0; j < T; j++) {
          acc = (acc + (scratch[(int64_t)T * i + j] * v[((int64_t)j * Hkv + hk) * Dh + d]));
        }
        out[((int64_t)i * H + h) * Dh + d] = acc;
      }
    }
  }
}

/* ------------------------------------------------------------------ */
/* Decoders                                                            */
/* ------------------------------------------------------------------ */

/* Transformer of external/llm/layers.lisp:35-90 (GPT-2 shaped). All weights
 * fp32 (the reference dequantises at load, dequantize.lisp:3-5). */
typedef struct {
  int n_layers, dim, n_heads, vocab, max_seq, ffn;
  double eps;
  const float *wte, *wpe;           /* (vocab,dim) (max_seq,dim) */
  const float *lnf_g, *lnf_b;       /* (dim) */
  const float *lm_head;             /* (vocab,dim), no bias */
  const float **ln1_g, **ln1_b;     /* per layer */
  const float **attn_w, **attn_b;   /* (3dim,dim) (3dim) */
  const float **proj_w, **proj_b;   /* (dim,dim) (dim) */
  const float **ln2_g, **ln2_b;
  const float **fc_w, **fc_b;       /* (ffn,dim) (ffn) */
  const float **fc2_w, **fc2_b;     /* (dim,ffn) (dim) */
  float **k_cache, **v_cache;       /* per layer (max_seq, n_heads, head_dim), zero-initialised */
} orc_gpt2_t;

/* One `forward` of the compiled graph (apps/gpt2/gpt2.lisp:97-113): `tokens`
 * are s token ids AS FLOATS (gpt2.lisp:95), n is the start position.  Writes
 * the last position's logits to logits_last (vocab floats, may be NULL) and
 * returns the greedy token (layers.lisp:90).  `onehot` selects the
 * reference's one-hot embedding (slow, faithful) or a row copy (same values).
 * `all_logits` computes lm_head for all s rows as the reference graph does. */
int64_t orc_gpt2_forward(const orc_gpt2_t *m, const float *tokens, int s, int n, float *logits_last,
                         int onehot, int all_logits) {
  int D = m->dim, H = m->n_heads, Dh = D / H, F = m->ffn, V = m->vocab, T = n + s;
  float *x = malloc(sizeof(float) * s * D);
  float *pe = malloc(sizeof(float) * s * D);
  float *xn = malloc(sizeof(float) * s * D);
  float *qkv = malloc(sizeof(float) * s * 3 * D);
  float *q = malloc(sizeof(float) * s * D);
  float *att = malloc(sizeof(float) * s * D);
  float *tmp = malloc(sizeof(float) * s * D);
  float *h1 = malloc(sizeof(float) * s * F);
  float *mask = malloc(sizeof(float) * s * T);
  float *scr = malloc(sizeof(float) * s * T);
  float *pos = malloc(sizeof(float) * s);
  for (int i = 0; i < s; i++) pos[i] = (float)(n + i);
  if (onehot) {
    orc_embedding_onehot(m->wte, tokens, x, s, V, D);
    orc_embedding_onehot(m->wpe, pos, pe, s, m->max_seq, D);
  } else {
    for (int i = 0; i < s; i++) {
      memcpy(x + (int64_t)i * D, m->wte + (int64_t)D * (int64_t)tokens[i], sizeof(float) * D);
      memcpy(pe + (int64_t)i * D, m->wpe + (int64_t)D * (n + i), sizeof(float) * D);
    }
  }
  for (int64_t i = 0; i < (int64_t)s * D; i++) x[i] = (x[i] + pe[i]);
  orc_triu_neginf(mask, s, T, 1 + n);
  for (int l = 0; l < m->n_layers; l++) {
    orc_layernorm(x, m->ln1_g[l], m->ln1_b[l], m->eps, xn, s, D);
    orc_linear(xn, m->attn_w[l], m->attn_b[l], qkv, s, D, 3 * D);
    for (int i = 0; i < s; i++) { /* chunk + !assign into cache rows [n, n+s) */
      memcpy(q + (int64_t)i * D, qkv + (int64_t)i * 3 * D, sizeof(float) * D);
      memcpy(m->k_cache[l] + (int64_t)(n + i) * D, qkv + (int64_t)i * 3 * D + D, sizeof(float) * D);
      memcpy(m->v_cache[l] + (int64_t)(n + i) * D, qkv + (int64_t)i * 3 * D + 2 * D, sizeof(float) * D);
    }
    orc_sdpa(q, m->k_cache[l], m->v_cache[l], mask, att, s, T, H, H, Dh, scr);
    orc_linear(att, m->proj_w[l], m->proj_b[l], tmp, s, D, D);
    for (int64_t i = 0; i < (int64_t)s * D; i++) x[i] = (x[i] + tmp[i]);
    orc_layernorm(x, m->ln2_g[l], m->ln2_b[l], m->eps, xn, s, D);
    orc_linear(xn, m->fc_w[l], m->fc_b[l], h1, s, D, F);
    orc_gelu_tanh(h1, h1, (int64_t)s * F);
    orc_linear(h1, m->fc2_w[l], m->fc2_b[l], tmp, s, F, D);
    for (int64_t i = 0; i < (int64_t)s * D; i++) x[i] = (x[i] + tmp[i]);
  }
  orc_layernorm(x, m->lnf_g, m->lnf_b, m->eps, xn, s, D);
  float *logits;
  if (all_logits) {
    logits = malloc(sizeof(float) * (int64_t)s * V);
    orc_linear(xn, m->lm_head, NULL, logits, s, D, V);
  } else {
    logits = malloc(sizeof(float) * V);
    orc_linear(xn + (int64_t)(s - 1) * D, m->lm_head, NULL, logits, 1, D, V);
  }
  const float *last = all_logits ? logits + (int64_t)(s - 1) * V : logits;
  if (logits_last) memcpy(logits_last, last, sizeof(float) * V);
  int64_t tok = orc_argmax(last, V);
  free(x); free(pe); free(xn); free(qkv); free(q); free(att); free(tmp); free(h1);
  free(mask); free(scr); free(pos); free(logits);
  return tok;
}

/* Llama-shaped decoder: NOT in the reference (Readme.md:150-151 lists it as
 * todo).  Built from the reference's RMSNorm, RoPE, SiLU, Linear, SDPA and
 * Embedding formulas with GQA head sharing and a position-offset RoPE. */
typedef struct {
  int n_layers, dim, n_heads, n_kv_heads, vocab, max_seq, ffn;
  double eps, rope_base;
  const float *tok_emb;             /* (vocab,dim) */
  const float *norm_w;              /* (dim) */
  const float *lm_head;             /* (vocab,dim) */
  const float **attn_norm, **ffn_norm;
  const float **wq, **wk, **wv, **wo; /* (dim,dim) (kvdim,dim) (kvdim,dim) (dim,dim) */
  const float **w_gate, **w_up, **w_down; /* (ffn,dim) (ffn,dim) (dim,ffn) */
  float **k_cache, **v_cache;       /* (max_seq, n_kv_heads, head_dim) */
} orc_llama_t;

int64_t orc_llama_forward(const orc_llama_t *m, const float *tokens, int s, int n, float *logits_last) {
  int D = m->dim, H = m->n_heads, Hkv = m->n_kv_heads, Dh = D / H, KD = Hkv * Dh, F = m->ffn,
      V = m->vocab, T = n + s;
  float *x = malloc(sizeof(float) * s * D);
  float *xn = malloc(sizeof(float) * s * D);
  float *q = malloc(sizeof(float) * s * D);
  float *kk = malloc(sizeof(float) * s * KD);
  float *vv = malloc(sizeof(float) * s * KD);
  float *att = malloc(sizeof(float) * s * D);
  float *tmp = malloc(sizeof(float) * s * D);
  float *g = malloc(sizeof(float) * s * F);
  float *u = malloc(sizeof(float) * s * F);
  float *mask = malloc(sizeof(float) * s * T);
  float *scr = malloc(sizeof(float) * s * T);
  for (int i = 0; i < s; i++)
    memcpy(x + (int64_t)i * D, m->tok_emb + (int64_t)D * (int64_t)tokens[i], sizeof(float) * D);
  orc_triu_neginf(mask, s, T, 1 + n);
  for (int l = 0; l < m->n_layers; l++) {
    orc_rmsnorm(x, m->attn_norm[l], m->eps, xn, s, D);
    orc_linear(xn, m->wq[l], NULL, q, s, D, D);
    orc_linear(xn, m->wk[l], NULL, kk, s, D, KD);
    orc_linear(xn, m->wv[l], NULL, vv, s, D, KD);
    orc_rope(q, q, 1, s, H, Dh, m->rope_base, n);
    orc_rope(kk, kk, 1, s, Hkv, Dh, m->rope_base, n);
    memcpy(m->k_cache[l] + (int64_t)n * KD, kk, sizeof(float) * s * KD);
    memcpy(m->v_cache[l] + (int64_t)n * KD, vv, sizeof(float) * s * KD);
    orc_sdpa(q, m->k_cache[l], m->v_cache[l], mask, att, s, T, H, Hkv, Dh, scr);
    orc_linear(att, m->wo[l], NULL, tmp, s, D, D);
    for (int64_t i = 0; i < (int64_t)s * D; i++) x[i] = (x[i] + tmp[i]);
    orc_rmsnorm(x, m->ffn_norm[l], m->eps, xn, s, D);
    orc_linear(xn, m->w_gate[l], NULL, g, s, D, F);
    orc_linear(xn, m->w_up[l], NULL, u, s, D, F);
    for (int64_t i = 0; i < (int64_t)s * F; i++) g[i] = (silu_f(g[i]) * u[i]);
    orc_linear(g, m->w_down[l], NULL, tmp, s, F, D);
    for (int64_t i = 0; i < (int64_t)s * D; i++) x[i] = (x[i] + tmp[i]);
  }
  orc_rmsnorm(x, m->norm_w, m->eps, xn, s, D);
  float *logits = malloc(sizeof(float) * V);
  orc_linear(xn + (int64_t)(s - 1) * D, m->lm_head, NULL, logits, 1, D, V);
  if (logits_last) memcpy(logits_last, logits, sizeof(float) * V);
  int64_t tok = orc_argmax(logits, V);
  free(x); free(xn); free(q); free(kk); free(vv); free(att); free(tmp); free(g); free(u);
  free(mask); free(scr); free(logits);
  return tok;
}
