/*
 * caten_hip.h -- C ABI of libcaten_hip.so, the MI355X (gfx950) execution
 * backend that plugs into Caten's BYOC backend interface as `:HIP`.
 *
 * Everything here is plain C: opaque pointers, sizes, integer status returns.
 * A host in any language binds it the way Caten's CLANG backend binds the
 * shared library gcc produces (source/byoc/clang.lisp:127-157,163-205): one
 * foreign-funcall per entry point, no callbacks into the host.
 *
 * Status: 0 = ok; >0 = a hipError_t / hiprtcResult from the runtime;
 * <0 = an argument or state error detected by this library.  After any
 * non-zero return cthip_last_error() describes the failure (the Lisp side
 * signals `error` with that text so it surfaces as a runtime-error,
 * source/runtime/runtime.lisp:84-104).
 *
 * Threading: one in-order HIP stream per process, as Caten's VM is single
 * threaded (source/runtime/runtime.lisp:134-145).  Every launch and copy below
 * is asynchronous on that stream except cthip_d2h, cthip_sync and the entry
 * points documented as synchronous.
 */
#ifndef CATEN_HIP_H
#define CATEN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- error codes detected here ---- */
#define CTHIP_OK 0
#define CTHIP_E_NOT_INIT (-1)
#define CTHIP_E_BAD_ARG (-2)
#define CTHIP_E_UNSUPPORTED (-3)
#define CTHIP_E_COMPILE (-4)
#define CTHIP_E_STATE (-5)

/* ggml tensor type ids (external/gguf/tensor-info.lisp:3-31) */
#define CTHIP_F32 0
#define CTHIP_F16 1
#define CTHIP_Q4_0 2
#define CTHIP_Q8_0 8

/* ================================================================== */
/* Runtime: device, buffers, modules, launches                         */
/* ================================================================== */

/* HipRuntime's initialize-instance :after (cf. MetalRuntime,
 * source/byoc/metal.lisp:106-112): selects the device, creates the stream.
 * Idempotent for the same device. */
int cthip_init(int device);
/* Frees every cached block and destroys the stream (free-runtime,
 * source/runtime/runtime.lisp:76-81). */
int cthip_shutdown(void);
const char *cthip_last_error(void);
/* name_cap bytes of device name, compute units, wavefront size, LDS bytes per
 * workgroup, total device memory.  Any out pointer may be NULL. */
int cthip_device_info(char *name, int name_cap, int *compute_units, int *wave_size,
                      size_t *lds_bytes, size_t *mem_bytes);

/* open-buffer (source/runtime/buffer.lisp:78-79): device storage of `bytes`
 * bytes, contents zeroed.  Backed by a caching allocator because every buffer
 * whose shape mentions the symbolic `s`/`n` is re-opened on each decode step
 * (source/runtime/runtime.lisp:248-259). bytes == 0 yields a valid 256-byte block. */
int cthip_alloc(void **out, size_t bytes);
/* close-buffer (buffer.lisp:81): returns the block to the cache. NULL is a no-op. */
int cthip_free(void *p);
/* Releases all cached (unused) blocks back to the driver. */
int cthip_cache_trim(void);
int cthip_cache_stats(size_t *live_bytes, size_t *cached_bytes, size_t *driver_allocs);

/* transfer-from-array (buffer.lisp:83): host -> device.  The source is staged
 * so the caller's array may be unpinned as soon as the call returns
 * (cffi:with-pointer-to-vector-data only pins for the call, clang.lisp:177-178). */
int cthip_h2d(void *dst, const void *src, size_t bytes);
/* transfer-into-array (buffer.lisp:85): device -> host; synchronises the stream. */
int cthip_d2h(void *dst, const void *src, size_t bytes);
/* copy-buffer-value (buffer.lisp:87) */
int cthip_d2d(void *dst, const void *src, size_t bytes);
int cthip_memset(void *dst, int byte, size_t bytes);
int cthip_sync(void);
/* The hipStream_t all work is queued on (for event timing by a harness). */
void *cthip_stream(void);

/* %compile-kernel (source/codegen/renderer.lisp:30-34; CLANG: clang.lisp:207-226;
 * METAL: metal.lisp:326-345): compile one HIP source holding every rendered
 * kernel of a graph with hipRTC for `arch` (NULL = "gfx950").  On success
 * `*code` / `*code_size` hold the code object; on failure returns CTHIP_E_COMPILE
 * and *log (if non-NULL) holds the compiler output.  Release both with
 * cthip_release(). Needs no GPU. */
int cthip_compile(const char *hip_source, const char *arch, void **code, size_t *code_size, char **log);
void cthip_release(void *p);
/* Metal-Program's newLibraryWithData / newFunctionWithName (metal.lisp:263-277) */
int cthip_module_load(void **module, const void *code);
int cthip_module_unload(void *module);
int cthip_get_function(void **fn, void *module, const char *name);
/* Metal-Program invoke (metal.lisp:288-322): args[i] points at the i-th kernel
 * argument value (a device pointer or a by-value scalar), in Caten's order
 * outputs -> dynamic shapes -> inputs (source/codegen/rewriting-rules.lisp:207-231). */
int cthip_launch(void *fn, const unsigned grid[3], const unsigned block[3], unsigned lds_bytes,
                 void **args, int nargs);

/* ---- Hip-Renderer: %render-kernel / invoke behind the C ABI ----
 * The renderer protocol (source/codegen/renderer.lisp:30-34) is a Lisp class; its work for this backend -- HIP
 * source with gfx950-aware work distribution for a Schedule-Item, and the choice of a hand-written kernel where
 * the item is a matmul / Linear / one-hot Embedding / ArgMax / softmax / LayerNorm / RMSNorm row shape -- is done
 * here, so the Lisp Hip-Renderer only prints the blueprint as an s-expression (grammar: header of
 * caten_amd/csrc/render.hip).
 *   %render-kernel  = cthip_program_create + cthip_program_source   (CLANG: clang.lisp:21-110; METAL: metal.lisp:178-250)
 *   %compile-kernel = cthip_render_header + every program's source -> cthip_compile -> cthip_module_load ->
 *                     cthip_program_bind per item                   (clang.lisp:207-226, metal.lisp:326-345)
 *   invoke          = cthip_program_launch: args[i] points at the i-th argument value (a device pointer or a
 *                     by-value scalar) in Caten's order outputs -> dynamic shapes -> inputs
 *                     (rewriting-rules.lisp:207-231; metal.lisp:288-322).  The grid comes from the item's
 *                     data-parallel loops and the shape arguments.  A program with a route checks the actual
 *                     layout at every launch and falls back to its rendered kernel when it does not fit.
 * cthip_program_route: "rendered", or the shape recognised at creation ("matmul", "embedding", "argmax",
 * "softmax", "layernorm", "rmsnorm"); cthip_program_last_route: what the last launch ran ("rendered",
 * "cthip_matmul", "cthip_linear", "cthip_bmm", "cthip_embedding", "cthip_argmax", "cthip_softmax",
 * "cthip_layernorm", "cthip_rmsnorm").  Strings stay valid until the program is destroyed.
 * The matmul shape is the nest of (caten (!matmul a b)) behind up to three batch loops
 * (source/test-suite/test-scheduler.lisp:117-138), its result stored as act(alpha * acc + pre...) + post... --
 * recognised by the VALUE of the store statement, whatever its spelling: bias, GELU / ReLU / SiLU, residual add
 * (test-scheduler.lisp:140-163; external/llm/layers.lisp:53-71), attention's scale and mask (layers.lisp:3-5).
 * One dense row-major product runs the MFMA GEMM (fewer than eight rows of a Linear: the single-row kernels);
 * batched, strided or offset operands -- q out of the fused qkv rows, k / v in place out of the cache view --
 * the batched kernel ("cthip_bmm"); operands that fit neither, the rendered kernel.  The embedding shape covers
 * indices that are an expression of the position (wpe(start-pos + arange), layers.lisp:81) and an added array.
 * Option "render_routes" 0 makes every program run its rendered kernel. */
const char *cthip_render_header(void);
int cthip_program_create(void **program, const char *blueprint);
int cthip_program_destroy(void *program);
const char *cthip_program_source(const void *program);
const char *cthip_program_name(const void *program);
const char *cthip_program_route(const void *program);
const char *cthip_program_last_route(const void *program);
int cthip_program_bind(void *program, void *module);
int cthip_program_launch(void *program, void **args, int nargs);

/* ---- the walk of a compiled node list behind one call per forward ----
 * runtime-forward / runtime-step (source/runtime/runtime.lisp:106-145) over the three node kinds a compiled model
 * consists of: `:Allocate` (runtime.lisp:228-259: a pool per node, the same shape gets the same storage back with
 * its contents, another shape a new zero-filled one), the scalar nodes that compute dynamic shapes
 * (`:Add :Mul :Neg :Idiv :Mod :Max`, runtime.lisp:396-449; integer division and modulo round toward minus
 * infinity) and `:JIT_KERNEL` (source/codegen/runner.lisp:20-32: launch, then writes[k] = args[out-positions[k]]).
 * For hosts whose own walk costs more per node than a launch: the list is handed over once, variables as slot
 * numbers, callers as programs; a forward binds the inputs and calls cthip_vm_run.  Node kinds beyond these
 * (views, custom ops) stay with the host's walk.
 *   operands: kinds[k] 0 = the integer ivals[k], 1 = the float fvals[k], 2 = slot ivals[k]
 *   dtypes[k] of a kernel argument: CTHIP_VM_PTR = the slot's device pointer, else the by-value scalar type the
 *     number is cast to (coerce-dtyped-buffer, source/codegen/helpers.lisp:118-125)
 * Parameters and inputs bound with cthip_vm_set_buffer (`:Allocate :from`, runtime.lisp:228-243) are never freed
 * here; buffers the walk opened are freed by cthip_vm_destroy.  cthip_vm_get: kind 0 = unset, 1 = integer,
 * 2 = float, 3 = device buffer.  A failing node stops the walk; the message names its index. */
#define CTHIP_VM_PTR 0
#define CTHIP_VM_BOOL 1
#define CTHIP_VM_F64 2
#define CTHIP_VM_F32 3
#define CTHIP_VM_U64 4
#define CTHIP_VM_I64 5
#define CTHIP_VM_U32 6
#define CTHIP_VM_I32 7
#define CTHIP_VM_U16 8
#define CTHIP_VM_I16 9
#define CTHIP_VM_U8 10
#define CTHIP_VM_I8 11
int cthip_vm_create(void **vm, int n_slots);
int cthip_vm_destroy(void *vm);
/* op: 0 Add, 1 Mul, 2 Neg, 3 Idiv, 4 Mod, 5 Max; the result is an integer when every operand is */
int cthip_vm_add_scalar(void *vm, int op, int out, int n_in, const int *kinds, const long long *ivals, const double *fvals);
int cthip_vm_add_allocate(void *vm, int out, int elem_bytes, int nrank, const int *kinds, const long long *ivals);
int cthip_vm_add_kernel(void *vm, void *program, int nargs, const int *kinds, const long long *ivals, const double *fvals,
                        const int *dtypes, int n_out, const int *out_positions, const int *out_slots);
int cthip_vm_set_int(void *vm, int slot, long long value);
int cthip_vm_set_float(void *vm, int slot, double value);
int cthip_vm_set_buffer(void *vm, int slot, void *device_ptr);
int cthip_vm_run(void *vm);
int cthip_vm_get(const void *vm, int slot, int *kind, long long *ivalue, double *fvalue, void **device_ptr);
long long cthip_vm_launches(const void *vm);  /* kernels launched so far */

/* Event timing on the library's stream (PROFILE=1 in the reference times each
 * JIT kernel on the host clock, source/codegen/runner.lisp:7-31). */
int cthip_timer_start(void);
int cthip_timer_stop(float *milliseconds); /* synchronous */

/* ================================================================== */
/* GGUF block codecs                                                   */
/* ================================================================== */

/* dequantize (external/gguf/dequantize.lisp:14-53) on the device: `raw` is the
 * tensor's bytes exactly as they sit in a GGUF file (device pointer), `n` the
 * element count (Q8_0: the last block may be short; Q4_0, which the reference
 * lacks, needs n % 32 == 0).  out[i] is bit-exact single float. */
int cthip_dequant(int ggml_type, const void *raw, int64_t n, float *out);

/* A weight matrix (rows x cols, Linear's (out,in) layout, source/nn/linear.lisp:9)
 * kept PACKED in HBM for dequant-in-register products.  `raw` = GGUF bytes on
 * the device, row-major, cols % 32 == 0 for quantised types.  The bytes are
 * re-laid into a quant plane and a scale plane (same total size) so that every
 * lane issues aligned 128-bit loads.  The raw buffer may be freed afterwards. */
int cthip_wmat_create(void **wmat, int ggml_type, const void *raw, int64_t rows, int64_t cols);
int cthip_wmat_destroy(void *wmat);
/* Bytes the matrix occupies in HBM (the algorithmic bytes of one GEMV over it). */
int64_t cthip_wmat_nbytes(const void *wmat);
/* Expands the packed planes to fp32 (rows*cols); bit-exact with cthip_dequant of the raw bytes. */
int cthip_wmat_dequant(const void *wmat, float *out);
/* Prepares a LayerNorm (source/nn/normalization.lisp:39-58) in front of this Linear (source/nn/linear.lisp:3-17)
 * to be carried through the product:  W.(((x-mu)*rstd)*gamma + beta) + bias = rstd*(W.(gamma*x) - mu*S) + C  with
 * S = W.gamma and C = W.beta + bias computed here, once (two products over the matrix, queued on the stream).
 * Afterwards cthip_linear(m < 8, CTHIP_PRO_LAYERNORM) called with these SAME gamma / beta / bias pointers needs mu
 * and rstd only in its epilogue, so the statistics overlap the weight stream; this is how a decoder session runs
 * its c_attn, c_fc and lm_head.  The terms are a snapshot: call again after changing gamma, beta or bias
 * (`bias` may be NULL).  Other argument combinations keep normalising the input first. */
int cthip_wmat_fold_layernorm(void *wmat, const float *gamma, const float *beta, const float *bias);

/* ================================================================== */
/* Hand-written fused items (what Caten's Schedule-Items compute)      */
/* ================================================================== */

/* prologue applied to the input vector(s) of cthip_linear */
#define CTHIP_PRO_NONE 0
#define CTHIP_PRO_LAYERNORM 1 /* LayerNorm, nn/normalization.lisp:39-58 */
#define CTHIP_PRO_RMSNORM 2   /* RMSNorm,   nn/normalization.lisp:70-85 */
#define CTHIP_PRO_SWIGLU 3    /* x is (m, 2*cols): silu(x[:cols]) * x[cols:], nn/activations.lisp:180-189 */
/* epilogue activation */
#define CTHIP_ACT_NONE 0
#define CTHIP_ACT_RELU 1 /* nn/activations.lisp:34-44 */
#define CTHIP_ACT_GELU 2 /* GeLU :tanh, nn/activations.lisp:202-215 */
#define CTHIP_ACT_SILU 3

/* Linear (source/nn/linear.lisp:3-17) with the elementwise neighbours Caten's
 * scheduler fuses around it (test-scheduler.lisp:140-163):
 *   y[m,:] = act( prologue(x[m,:]) @ W^T + bias ) + residual[m,:]
 * x (m, cols) [(m, 2*cols) for SWIGLU], y/residual (m, rows), fp32, contiguous.
 * norm_g/norm_b/bias/residual may be NULL.  m == 1 is the dequant-in-register
 * GEMV of batch-1 decode; m >= 8 uses the MFMA tile path (weights dequantised while staged). */
int cthip_linear(float *y, const void *wmat, const float *x, int m, const float *bias,
                 const float *residual, int act, int prologue, const float *norm_g,
                 const float *norm_b, float eps);

/* Library options.
 * "gemm_precision": operand format of the MFMA launches behind cthip_linear with m >= 8 input rows and
 *   the decoder's prefill: 2 (default) = every operand split into two bf16 terms, three bf16 MFMAs
 *   per product, fp32 accumulation (2^-16 of a product is lost); 3 = three terms, six MFMAs per
 *   product: all 24 bits of an fp32 operand; 0 = fp32 MFMA operands; 1 = operands rounded to bf16
 *   (rtol/atol 1e-2).
 * "gemm_bf16": 1 = shorthand for gemm_precision 1, 0 = back to the default.
 * "gemv_stream_weights": whether the single-row Linear kernels request the weights with the non-temporal
 *   hint: -1 (default) = per matrix -- a matrix larger than the 256 MB Infinity Cache, and every matrix of a
 *   decoder session whose weights together exceed three quarters of it; 0 = never; 1 = always.  Results do
 *   not depend on it.  A decoder session picks its kernels when it first runs.
 * "gemv_wide": which single-row Linear launches take the wide-row kernel (input vector staged in LDS instead of
 *   held in registers; rows of up to 36 000 columns in any weight format, no LayerNorm prologue, no fused argmax): 0 = none
 *   (rows wider than the register-resident kernels cover go as column slices, one launch each), 1 (default) = the
 *   rows no register-resident kernel covers and those whose register-resident kernel runs one wavefront per SIMD
 *   (4-bit rows past 6144 columns, 8-bit rows past 4096), 2 = every launch it supports.  Results differ between the two kernel
 *   families only in summation order.
 * "attn_split": 1 (default) = decoder sessions created afterwards that run one launch per Linear and have
 *   max_seq >= 512 share the keys of a head among (compute units / heads) workgroups, at most 16, in their decode
 *   attention (long contexts); 2 .. 16 = that many workgroups per head; 0 = one workgroup per head.  Same tokens;
 *   logits differ in summation order only.
 * "attn_long_from": a position (default 896; 0 = never).  Decoder sessions created afterwards whose layers run as
 *   three launches switch, from this position on (half as far again over Q8_0 cache rows), to four launches per layer: the attention as a
 *   launch of its own with a head's keys shared by several workgroups ("attn_split"), then the projection.  Same
 *   tokens; logits differ in summation order only.
 * "kv_cache": how decoder sessions created afterwards keep their KV cache: 0 (default) = fp32 rows, the
 *   reference's dense cache (external/llm/layers.lisp:19-33); 1 = GGUF-Q8_0 rows (blocks of 32 int8 and one fp16
 *   scale per cache row, quantised once when the row is appended): 3.76x fewer cache bytes held and read per
 *   step.  Such a session runs one launch per Linear + one attention launch (GPT-2 shapes: three launches per layer); logits stay within rtol 2e-2 / atol 2e-2 of the fp32
 *   cache's on the tested models (the band of 8-bit keys and values, not of the fp32 arithmetic around them).
 *   2 = fp32 rows in pages of cthip_kv_page_rows() rows per layer, opened when the position first reaches them
 *   (a session then holds the rows it has used instead of max_seq rows); such a session runs one launch per
 *   Linear; tokens and logits are those of the dense cache.
 * "decode_skip": knock-out timing of the three-launch decode step -- a mask of launches a session created
 *   afterwards leaves out (1 qkv, 2 attention + projection, 4 MLP, 8 the sum in front of lm_head,
 *   16 lm_head + argmax).  Tokens and logits of such a session are meaningless; 0 (default) = none.
 * "decode_flow": 1 = GPT-2 shaped Q8_0 sessions (d 256 / 4 heads or d 768 / 12 heads, fp32 cache) created
 *   afterwards run all layers of a decode step as ONE launch of role-specialised workgroups that hand their
 *   results over through tagged device memory (csrc/decode_flow.hip) -- an experiment kept for its measurements:
 *   same tokens, logits inside the fp32 band, and SLOWER than the three launches per layer it replaces.
 *   2 = the same, and every workgroup keeps clock stamps of its last step (cthip_decoder_peek "flow_trace").
 *   It needs every one of its workgroups resident at once; a step whose bounded waits run out fails with
 *   CTHIP_E_STATE instead of hanging.  0 (default) = off. */
int cthip_set_option(const char *name, int value);

/* !relu(!matmul A B) (api/high-level-ops.lisp:76-99; fused per test-scheduler.lisp:140-163):
 * C (M,N) = act(A (M,K) @ B (K,N)), row-major fp32.  precision 0 = fp32 MFMA operands,
 * 3 = operands split into three bf16 terms (both rtol 1e-3/atol 1e-4), 2 = two bf16 terms
 * (2^-16 of a product is lost), 1 = bf16 MFMA operands (rtol/atol 1e-2); fp32 accumulation
 * in every mode. */
int cthip_matmul(float *C, const float *A, const float *B, int M, int N, int K, int act, int precision);
/* cthip_matmul for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): same arguments, same kernels, same results, but the partial tiles of
 * a split reduction go to a 4 MiB array that is part of the library's code object instead of a block of the
 * caching allocator, and no allocation or release happens during the call.  A shape whose split needs more
 * (split count x M x N x 4 bytes) returns CTHIP_E_UNSUPPORTED.  All calls on one GPU share that array: calls
 * that overlap on one GPU (two host threads, two streams) race.  It has no counterpart in the reference. */
int cthip_matmul_noalloc(float *C, const float *A, const float *B, int M, int N, int K, int act, int precision);

/* Row ops over the last axis, fp32, rows x n contiguous. */
int cthip_softmax(float *y, const float *x, int64_t rows, int n);   /* nn/activations.lisp:59-62,107-119 */
int cthip_layernorm(float *y, const float *x, const float *gamma, const float *beta, float eps,
                    int64_t rows, int n);                            /* nn/normalization.lisp:39-58 */
int cthip_rmsnorm(float *y, const float *x, const float *w, float eps, int64_t rows, int n); /* :70-85 */
/* LayerNorm immediately followed by softmax over the same axis, one pass over HBM. */
int cthip_layernorm_softmax(float *y, const float *x, const float *gamma, const float *beta, float eps,
                            int64_t rows, int n);
/* Elementwise: kind is a CTHIP_ACT_* (plus 4 = sigmoid, 5 = tanh). */
#define CTHIP_ACT_SIGMOID 4
#define CTHIP_ACT_TANH 5
int cthip_unary(int kind, float *y, const float *x, int64_t n);
/* Embedding (nn/embedding.lisp:3-25): out[t,:] = W[idx[t],:], idx given as
 * floats as the reference feeds them (apps/gpt2/gpt2.lisp:95).  The reference
 * sums a one-hot mask over the vocabulary; the result is the same row. */
int cthip_embedding(float *out, const float *W, const float *idx, int ntok, int vocab, int dim);
/* ArgMaxNode over the last axis (api/high-level-ops.lisp:314-343): lowest index among ties. */
int cthip_argmax(int64_t *out, const float *x, int64_t rows, int n);
/* RoPE (nn/positional-encoding.lisp:3-64) on (B,S,H,Dh), interleaved pairs;
 * start_pos shifts the positions (0 reproduces the reference). */
int cthip_rope(float *out, const float *x, int B, int S, int H, int Dh, float base, int start_pos);
/* scaled-dot-product-attention (external/llm/layers.lisp:3-5) of S query rows
 * (S,H,Dh) at positions start_pos..start_pos+S-1 against a KV cache laid out
 * (max_len, Hkv, Dh) (layers.lisp:19-33) holding T = start_pos+S rows, with the
 * causal mask of layers.lisp:83 applied.  out (S,H,Dh).  From 32 rows on the products run on the matrix cores:
 * with two bf16 terms per operand (2^-16 of a product dropped), or with fp32 operands when option
 * "gemm_precision" is 0. */
int cthip_sdpa_cached(float *out, const float *q, const float *k_cache, const float *v_cache,
                      int S, int start_pos, int H, int Hkv, int Dh);
/* The same cache as GGUF-Q8_0 rows (the reference's cache is dense fp32, layers.lisp:19-33; its Q8_0 block is
 * external/gguf/dequantize.lisp:40-53): a quant plane int8[max_len][kv_dim] and a scale plane fp16[max_len][kv_dim/32].
 * cthip_kv_append_q8 quantises `s` fp32 rows (s, kv_dim) into cache rows row0 .. row0+s-1 (per block of 32:
 * d = absmax / 127 stored as fp16, q = x / d rounded half away from zero -- ggml's reference row quantiser).
 * cthip_sdpa_cached_q8 attends ONE query row (H, Dh) over cache rows 0 .. T-1 (the decode step; every key is
 * visible to the last position), out (H, Dh): the products run on the integers, a block's scale is applied to
 * its partial sum. */
int cthip_kv_append_q8(void *q_plane, void *d_plane, const float *rows, int s, int row0, int kv_dim);
int cthip_sdpa_cached_q8(float *out, const float *q, const void *k_q, const void *k_d, const void *v_q, const void *v_d, int T,
                         int H, int Hkv, int Dh);
/* The same cache in pages (the reference allocates (B, max_len, H, Dh) once, layers.lisp:25-26): row r lives at
 * pages[r / cthip_kv_page_rows()] + (r % cthip_kv_page_rows()) * kv_dim, `pages` a device array of device pointers
 * that the owner extends as positions are reached.  cthip_kv_append_paged copies `s` fp32 key rows and value rows
 * (s, kv_dim) into rows row0 .. row0+s-1 of the key pages and the value pages; cthip_sdpa_cached_paged attends ONE
 * query row (H, Dh) over rows 0 .. T-1, out (H, Dh), with the arithmetic of cthip_sdpa_cached. */
int cthip_kv_page_rows(void);
int cthip_kv_append_paged(void *const *k_pages, void *const *v_pages, const float *k_rows, const float *v_rows, int s, int row0,
                          int kv_dim);
int cthip_sdpa_cached_paged(float *out, const float *q, const void *const *k_pages, const void *const *v_pages, int T, int H, int Hkv,
                            int Dh);

/* ================================================================== */
/* Decoder session: Transformer (external/llm/layers.lisp:73-90) and   */
/* the gpt2-generate loop (apps/gpt2/gpt2.lisp:97-113)                 */
/* ================================================================== */

#define CTHIP_ARCH_GPT2 0  /* LayerNorm, learned positions, fused qkv + biases, GELU MLP */
#define CTHIP_ARCH_LLAMA 1 /* RMSNorm, RoPE, GQA, SwiGLU, no biases (not in the reference) */

typedef struct {
  int arch;
  int n_layers, dim, n_heads, n_kv_heads, ffn, vocab, max_seq;
  float eps;
  float rope_base;
} cthip_decoder_config;

int cthip_decoder_create(void **dec, const cthip_decoder_config *cfg);
int cthip_decoder_destroy(void *dec);
/* load-state-dict (source/api/module.lisp:290-320): hands one tensor to the
 * session under its reference state-dict key ("wte.weight", "h.3.attn.c_attn.weight",
 * "h.3.ln_1.affine", "ln_f.bias", "lm_head.weight", ... apps/gpt2/gpt2.lisp:52-70).
 * `host_raw` are the tensor's GGUF bytes in HOST memory (weights arrive as host
 * buffers whatever the backend, external/gguf/tensor-info.lisp:104-120); they
 * are uploaded once and, for 2-D Linear weights, kept packed. */
int cthip_decoder_load(void *dec, const char *key, int ggml_type, const void *host_raw,
                       int64_t rows, int64_t cols);
/* Number of tensors still missing before the session can run. */
int cthip_decoder_missing(const void *dec);
/* One `forward` of the compiled graph (apps/gpt2/gpt2.lisp:104): s token ids AS
 * FLOATS starting at position n.  Writes the greedy token of the last position
 * to *token; logits_out (host, vocab floats) may be NULL.  Synchronous. */
int cthip_decoder_forward(void *dec, const float *tokens, int s, int n, int64_t *token,
                          float *logits_out);
/* gpt2-generate's loop kept on the device: after a forward has left position
 * and last token on the device, runs `steps` further single-token forwards
 * without host round trips and writes their greedy tokens to tokens_out (host).
 * Synchronous at the end only. */
int cthip_decoder_generate(void *dec, int steps, int64_t *tokens_out);
/* The same loop with a stop condition checked ON THE DEVICE (the reference's loop has none, apps/gpt2/gpt2.lisp:102:
 * it always runs max-length forwards): the step that produces `eos_token` ends the sequence -- the steps already
 * queued behind it leave token, position and history untouched, and the host, which looks at the flag between
 * graph launches without waiting for it, stops queuing.  tokens_out receives the tokens up to and including
 * eos_token (or max_steps of them), *n_generated their number; the position advances by that number. */
int cthip_decoder_generate_until(void *dec, int max_steps, int64_t eos_token, int64_t *tokens_out, int *n_generated);
/* Current position (tokens in the KV cache). */
int cthip_decoder_position(const void *dec);
/* Bytes of HBM one decode step must read at position t (weights + norms/biases + KV rows at their stored
 * size: 4 bytes per element, 1.0625 with option "kv_cache" 1). */
int64_t cthip_decoder_step_bytes(const void *dec, int t);
/* Launches per layer of one decode step of this session at short contexts: 3 (attention + projection and the whole MLP merged,
 * per-XCD accumulators -- taken only when the device passed the load-time checks that XCD ids are 0..7 and that
 * atomics of different workgroups of an XCD meet in its L2), 5 (one launch per Linear + attention; over Q8_0 cache
 * rows and over a paged cache the attention launch also rotates, quantises / copies and appends the new row).
 * A session of 3 runs 4 from position "attn_long_from" on.  -1 on error. */
int cthip_decoder_layer_launches(void *dec);
/* Device pointers into the session, for parity tests: "k_cache.<l>", "v_cache.<l>" (fp32 rows; with a Q8_0
 * cache their dequantised values, in a buffer the next peek overwrites), "logits", "x"; with a Q8_0 cache also
 * the planes themselves, "k_cache_q8.<l>" / "v_cache_q8.<l>" (int8[max_seq][kv_dim]) and "k_cache_d.<l>" /
 * "v_cache_d.<l>" (fp16[max_seq][kv_dim / 32]), n_floats counting their bytes in units of four. */
int cthip_decoder_peek(void *dec, const char *what, void **ptr, int64_t *n_floats);

/* ================================================================== */
/* GGUF files (external/gguf/gguf-file.lisp, metadata.lisp,            */
/* tensor-info.lisp).  Host side only: needs no device.                */
/* ================================================================== */

/* load-gguf (gguf-file.lisp:93-104): maps the file, parses header (magic "GGUF", version 2 or 3),
 * metadata key/values and tensor infos; absolute tensor offsets follow general.alignment
 * (default 32; tensor-info.lisp:88-98). */
int cthip_gguf_open(void **gguf, const char *path);
int cthip_gguf_close(void *gguf);
int cthip_gguf_version(const void *gguf);
int64_t cthip_gguf_tensor_count(const void *gguf);
int64_t cthip_gguf_metadata_count(const void *gguf);
int64_t cthip_gguf_alignment(const void *gguf);
/* Tensor-Info (tensor-info.lisp:43-60).  dims are as stored, innermost first: the row-major shape is
 * their reverse (tensor-info.lisp:104-120).  nbytes is 0 for ggml types without a decoder here. */
int cthip_gguf_tensor_info(const void *gguf, int64_t i, const char **name, int *ggml_type, int *n_dims,
                           int64_t dims[4], int64_t *abs_offset, int64_t *nbytes);
int64_t cthip_gguf_find_tensor(const void *gguf, const char *name); /* -1 if absent */
const void *cthip_gguf_tensor_data(const void *gguf, int64_t i);    /* host pointer into the mapping */
/* gguf-metadata-get (gguf-file.lisp:26-27) */
int64_t cthip_gguf_find_metadata(const void *gguf, const char *key); /* -1 if absent */
int cthip_gguf_metadata_info(const void *gguf, int64_t i, const char **key, int *type, int *elem_type, int64_t *count);
int cthip_gguf_metadata_number(const void *gguf, int64_t i, double *out);
/* a string value, or element j of an array of strings; not NUL-terminated */
int cthip_gguf_metadata_string(const void *gguf, int64_t i, int64_t j, const char **data, int64_t *len);
/* make-gpt2's load path (apps/gpt2/gpt2.lisp:82-93): gguf->state-dict + remap-key + load-state-dict
 * for a decoder session; tensors go from the mapping to the device still packed. */
int cthip_decoder_load_gguf(void *dec, const void *gguf, int arch, int *n_loaded);

/* ---- BPE tokenizer (host code): caten/llm's BPETokenizer (external/llm/bpe.lisp) ----
 * cthip_bpe_create mirrors make-bpe-tokenizer (bpe.lisp:14-38): `tokens` = the vocabulary, pieces separated by
 * single spaces, the first piece dropped, the rest numbered from 0; `merges` = one "a b" pair per line, the first
 * line dropped, ranked by line.  encode (bpe.lisp:85-100): GPT-2 pre-tokenisation, byte alphabet, merges by rank;
 * a symbol the vocabulary lacks becomes id 0.  With ids == NULL it only counts.  decode (bpe.lisp:102-114): the
 * inverse; with out == NULL it only measures.  Text is UTF-8 and is not NUL-terminated on output. */
int cthip_bpe_create(void **bpe, const char *tokens, size_t tokens_len, const char *merges, size_t merges_len);
int cthip_bpe_destroy(void *bpe);
int cthip_bpe_vocab_size(const void *bpe);
int cthip_bpe_encode(void *bpe, const char *text, size_t len, int *ids, size_t cap, size_t *n_ids);
int cthip_bpe_decode(const void *bpe, const int *ids, size_t n, char *out, size_t cap, size_t *len);

#ifdef __cplusplus
}
#endif
#endif /* CATEN_HIP_H */
