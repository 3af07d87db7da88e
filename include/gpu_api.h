/*
 * C ABI of the MI355X (gfx950) quantized-linear kernels: libgpu_kernels.so.
 *
 * The first block of entry points has the reference's names, argument order and C types, so the reference's Rust
 * declarations (src/ffi.rs) bind to this library unchanged; each prototype cites the declaration it replaces.
 * All pointers are device pointers unless stated; `stream` is a hipStream_t passed as void* (null = default stream).
 * Every call is asynchronous on `stream` and never throws.  State kept between calls, all of it until the process ends:
 * cached device attributes; per device, the lookup tables of the prologue activations (see gpu_act_tables_init); per
 * stream (the first eight that need it), 24 MiB for the int32 planes of gpu_int8_gemm's split-K shapes; the kernel
 * family forced by the test hook gpu_int8_gemm_force_config; the static scratch of gpu_int8_gemm_static.
 *
 * Return convention (src/ffi.rs:336-344, csrc/common.cuh:128): 0 = ok; > 0 = a hipError_t from the launch
 * (hipGetErrorString names it); < 0 = the launcher refused the arguments, with the reference's codes:
 *   quantizers  -1 shape (K granularity), -2 row too long (K > 32768), -3 prologue id, -4 dtype
 *   int8 GEMM   -200 (plain) / -201 (residual): unknown out_dt, null rscale/resid, K == 0 for the residual form,
 *               or a shape the kernels cannot run (K % 8 != 0; gpu_int8_gemm_static also refuses K % 16 != 0)
 *   w6 decode   -1 (K % 32 or G % 16)
 */
#ifndef GPU_API_H
#define GPU_API_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* dtype codes: csrc/common.cuh:15, src/ffi.rs:11-13 */
enum { DT_F32 = 0, DT_F16 = 1, DT_BF16 = 2 };

/* prologue ids: csrc/kernels.cu:13-15, src/ffi.rs:15-29 */
enum {
    PRO_PLAIN = 0, PRO_RMS = 1, PRO_GATE = 2, PRO_SWIGLU = 3, PRO_LAYERNORM = 4, PRO_SILU = 5, PRO_GELU = 6,
    PRO_ADALN = 7, PRO_SITU = 8, PRO_LN_MOD = 9, PRO_LN_AFFINE = 10, PRO_GELU_TANH = 11, PRO_LN_AFFINE_SILU = 12,
    PRO_SITU_FAST = 13
};

/* Row prologue -> optional ConvRot rotation -> dynamic per-row absmax int8 quantization.
 * Replaces gpu_quant_rows, src/ffi.rs:74-75 / csrc/kernels.cu:271-298.
 * x: T[M, x_stride] (T = bf16 or f32 by `dtype`; rows 16-byte aligned); q: int8 [M, K]; scales: f32 [M].
 * rotate: 0 = none; 1 or 256 = the reference's 256-wide normalized Hadamard; 64 and 128 select a 64- or 128-wide
 * group (an extension: the reference treats the argument as a flag).  K must be a multiple of 256 (of 64 when
 * rotate is 0 or 64, of 128 when rotate is 128).
 * Prologues (x, g, up_offset, norm_w, eps, mod_scale, mod_shift as in QuantParams, csrc/kernels.cu:21-37): all ids of
 * csrc/kernels.cu:280-292, applied inside the quantizer kernel with the reference's rounding points.  Row sums are
 * accumulated in fp64 and rounded once, exp / erf / tanh / 1/sqrt are correctly rounded (the reference has fp32 sums in the
 * order of its thread layout and CUDA's 1-2 ulp routines).  PRO_SITU_FAST, which the reference defines through NVIDIA's
 * approximate tanh/exp/divide (about 2^-11 relative error), runs PRO_SITU's accurate expression. */
int gpu_quant_rows(int dtype, int prologue, const void* x, int64_t x_stride, const void* g, int64_t g_stride,
                   int64_t up_offset, const float* norm_w, float eps, const void* mod_scale, const void* mod_shift,
                   int8_t* q, float* scales, int M, int K, int rotate, void* stream);

/* gpu_quant_rows with a LayerNorm bias.  Replaces gpu_quant_rows_b, src/ffi.rs:246-247 / csrc/kernels.cu:301-313. */
int gpu_quant_rows_b(int dtype, int prologue, const void* x, int64_t x_stride, const float* norm_w,
                     const float* norm_b, float eps, const void* mod_scale, const void* mod_shift, int8_t* q,
                     float* scales, int M, int K, int rotate, void* stream);

/* Same prologues + 256-wide rotation, fp32 in and out, no quantization.
 * Replaces gpu_rotate_rows_f32, src/ffi.rs:35-36 / csrc/kernels.cu:316-327. */
int gpu_rotate_rows_f32(int prologue, const float* x, int64_t x_stride, int64_t up_offset, const float* norm_w,
                        float eps, float* out, int M, int K, void* stream);

/* The row prologues alone: writes the activation row in T for a non-quantized GEMM.
 * Replaces gpu_prologue_rows, src/ffi.rs / csrc/kernels.cu:420-446: dtype bf16 or f32 (-4), prologue PLAIN, RMS, GATE,
 * SWIGLU, LAYERNORM, SILU, GELU, ADALN or SITU (-3).  out: T[M, out_stride]. */
int gpu_prologue_rows(int dtype, int prologue, const void* x, int64_t x_stride, const void* g, int64_t g_stride,
                      int64_t up_offset, const float* norm_w, float eps, const void* mod_scale, const void* mod_shift,
                      void* out, int64_t out_stride, int M, int K, void* stream);

/* The LayerNorm variants with a bias, and the plain activations, in bf16, f16 or f32.
 * Replaces gpu_prologue_rows_b, csrc/kernels.cu:449-474: prologue PLAIN, LAYERNORM, LN_MOD, LN_AFFINE,
 * LN_AFFINE_SILU, SILU, GELU or GELU_TANH (-3). */
int gpu_prologue_rows_b(int dtype, int prologue, const void* x, int64_t x_stride, const float* norm_w,
                        const float* norm_b, float eps, const void* mod_scale, const void* mod_shift, void* out,
                        int64_t out_stride, int M, int K, void* stream);

/* fp16 rows -> optional 64/256 rotation -> int8 rows + scales (the SD/SDXL UNet quantizer).
 * Replaces gpu_sd_quant_rows, src/ffi.rs:252 / csrc/sd.cu:599-606.  rotate in {0, 64, 256}, K % 16 == 0. */
int gpu_sd_quant_rows(const void* x, int64_t x_stride, int8_t* q, float* scales, int M, int K, int rotate,
                      void* stream);

/* The SD UNet's fused quantizers: the half row another kernel would have written, then gpu_sd_quant_rows of it.
 * Replace gpu_sd_ln_quant_rows, gpu_sd_geglu_quant_rows, gpu_sd_unpad_quant_rows, gpu_sd_group_norm_quant_rows,
 * csrc/sd.cu:691-724.  rotate and K as gpu_sd_quant_rows.  The source runs inside the quantizer kernel.
 *   ln:     LayerNorm of x [M, x_stride] with fp32 weight and bias.
 *   geglu:  in [M, 2I] (value, then gate) -> value * gelu(gate), K = I.
 *   unpad:  src [M, H, dp] -> the first d of every dp, K = H * d.
 *   gn:     GroupNorm (no SiLU) of x [N, P, C] per image; rows are pixels, K = C.  sums: 16 * N * G + 16 bytes of device
 *           scratch, which receives (mean, rstd) as two floats at byte 16 * (n * G + g), as the reference leaves them. */
int gpu_sd_ln_quant_rows(const void* x, int64_t x_stride, const float* w, const float* b, float eps, int8_t* q,
                         float* scales, int M, int K, int rotate, void* stream);
int gpu_sd_geglu_quant_rows(const void* in, int8_t* q, float* scales, int M, int I, int rotate, void* stream);
int gpu_sd_unpad_quant_rows(const void* src, int8_t* q, float* scales, int M, int H, int d, int dp, int rotate,
                            void* stream);
int gpu_sd_group_norm_quant_rows(const void* x, const float* w, const float* b, void* sums, int N, int64_t P, int C, int G,
                                 float eps, int8_t* q, float* scales, int rotate, void* stream);

/* Weight-side kernels of the int8 ConvRot format (weights are stored rotated; H256 is its own inverse).
 *   gpu_dequant_i8       out f32 [N,K] = q * s[row].  Replaces csrc/kernels.cu:329-343 (K % 4, else -1).
 *   gpu_embed_dequant    rows of an int8 ConvRot embedding table -> f32 rows holding bf16 values, H256(q * s).
 *                        Replaces csrc/kernels.cu:620-639 (rotate == 0: -1).  K % 256.
 *   gpu_convrot_dequant  the weight in its original basis, f32 (DT_F32) or bf16 (any other code).  csrc/kernels.cu:1345-1407.
 *   gpu_convrot_requant  x [N,K] f32 or bf16 in its original basis -> rotated q [N,K] + row scales; seed 0 rounds to
 *                        nearest, any other seed rounds stochastically with the reference's hash of (element index + seed).
 *                        csrc/kernels.cu:1361-1420.  K % 256, K <= 32768. */
int gpu_dequant_i8(const int8_t* q, const float* s, float* out, int64_t N, int64_t K, void* stream);
int gpu_embed_dequant(const int8_t* q, const float* s, float* out, int M, int K, int rotate, void* stream);
int gpu_convrot_dequant(int dtype, const void* q, const void* s, void* out, int64_t N, int K, void* stream);
int gpu_convrot_requant(int dtype, const void* x, void* q, void* s, int64_t N, int K, uint64_t seed, void* stream);

/* bf16 weight [N,K] in its original basis -> the reference's W6 format: ConvRot256, two alternating-least-squares rounds
 * for the step of every 32 columns, packed [N, 3K/4] (nibble plane then 2-bit plane, code = q + 32), s_rel fp8-e4m3
 * [N, K/32], s_channel f32 [N]; every value is rounded stochastically between its two bracketing grid levels, keyed by
 * element index and seed.  Replaces gpu_w6_requant, src/ffi.rs:132 / csrc/vendor/w6a8_requant.cu:242-252.
 * K % 256 (-1), K <= 39 680 (-2: the rotated row is held in LDS). */
int gpu_w6_requant(const void* weight, void* packed, void* s_rel, void* s_channel, int64_t N, int K, uint64_t seed,
                   void* stream);

/* INT8 attention, head dims 64, 128 and 256: o = softmax(q . k^T * scale) . v with q and k rotated and quantized per
 * scale group (eight groups per block of 32 query rows, 16 at head dim 256; four per key tile), an optional K anchor
 * subtracted first, v quantized per channel, probabilities as u8 per key tile (64 keys; 128 beyond lk = 1024 unless the
 * head dim is 64) and integer P.V partials folded in fp32.  The rotation is the reference's choice by shape: up to 256
 * keys H4 on runs of four channels only; beyond, H64 at head dim 64, sign diagonal + H128 at 128, H128 on each half at
 * 256.  q/k/v/o: [b, seq, heads, head_dim] through element strides (batch, row, head), bf16 (gpu_int8_attn,
 * gpu_int8_attn_d) or f16 (gpu_int8_attn_f16); h % hk == 0 (grouped-query heads); ws: 256-byte aligned device scratch of
 * gpu_int8_attn_workspace[_d] bytes, layout private to the library.
 * Replaces gpu_int8_attn_workspace_d / gpu_int8_attn_workspace (csrc/attn_int8.cu:62-82), gpu_int8_attn_d (:101-108),
 * gpu_int8_attn_f16 (:111-118), gpu_int8_attn (:225-231); src/ffi.rs binds them under the same names.
 * Returns 0, -400 (argument the library refuses: message on stderr; gpu_int8_attn_workspace_d returns 0 bytes for a
 * head dim other than 64, 128, 256) or -401 (launch failure), the reference's codes.
 * gpu_int8_attn_sink (csrc/attn_int8.cu:193-202): attention over lk keys plus `sink` more whose keys and values are
 * zero, which count in the softmax denominator only; the K anchor is off so that a zero key's score stays zero; bf16.
 * A non-null qw normalizes q first as gpu_int8_attn_norm_rope does (weight qw, eps, no rotation), k taken as it is.
 * gpu_int8_attn_norm_rope (csrc/attn_int8.cu:163-174, bound at src/ffi.rs:66-68, called from src/dit.rs:575): per-head
 * RMSNorm with weight qw [128] (null = ones) and rotary embedding applied to q inside its quantizer, and to k as well
 * when kw is not null (a null kw leaves k as it is, whatever rope says); q and k in memory are not written.  rope:
 * f32 [max(lq, lk)][64][2] = (cos, sin) per position and pair, or null; rope_mode 1 rotates channel pairs (2p, 2p+1),
 * 2 the pairs (j, j + 64), 0 none; other values -400.  bf16 only.  The values the quantizer sees are those
 * gpu_qk_norm_rope (csrc/kernels.cu:482-540) would have stored, with 1/sqrt correctly rounded where CUDA's rsqrtf
 * approximates.
 * gpu_int8_attn_key_bias / gpu_int8_attn_key_bias_workspace (csrc/attn_int8.cu:184-223, bound at src/ffi.rs:196-199,
 * called from src/dit.rs:519,573): bias f32 [lk], the same for every batch item, head and query, added to each key's
 * logits (an additive attention mask; a bias that is not finite masks its key, a query row with every key masked gives
 * zeros for lk <= 1024).  Its workspace is the plain one plus the prepared bias row, the reference's size.  bf16.  The
 * two routes of the reference are kept: for lk <= 1024 (64-key tiles) the denominator sums the unrounded probabilities,
 * for longer sequences (128-key tiles) the rounded ones, and a tile whose keys share one finite bias folds it into the
 * exponent's constant. */
int64_t gpu_int8_attn_workspace_d(int b, int h, int hk, int lq, int lk, int head_dim);
int64_t gpu_int8_attn_workspace(int b, int h, int hk, int lq, int lk);
int gpu_int8_attn_d(const void* q, const void* k, const void* v, void* o, void* ws, int b, int lq, int lk, int h, int hk,
                    int head_dim, int64_t q_bs, int64_t q_rs, int64_t q_hs, int64_t k_bs, int64_t k_rs, int64_t k_hs,
                    int64_t v_bs, int64_t v_rs, int64_t v_hs, int64_t o_bs, int64_t o_rs, int64_t o_hs, float scale,
                    void* stream);
int gpu_int8_attn_f16(const void* q, const void* k, const void* v, void* o, void* ws, int b, int lq, int lk, int h, int hk,
                      int head_dim, int64_t q_bs, int64_t q_rs, int64_t q_hs, int64_t k_bs, int64_t k_rs, int64_t k_hs,
                      int64_t v_bs, int64_t v_rs, int64_t v_hs, int64_t o_bs, int64_t o_rs, int64_t o_hs, float scale,
                      void* stream);
int gpu_int8_attn(const void* q, const void* k, const void* v, void* o, void* ws, int b, int lq, int lk, int h, int hk,
                  int64_t q_bs, int64_t q_rs, int64_t q_hs, int64_t k_bs, int64_t k_rs, int64_t k_hs, int64_t v_bs,
                  int64_t v_rs, int64_t v_hs, int64_t o_bs, int64_t o_rs, int64_t o_hs, float scale, void* stream);

int gpu_int8_attn_sink(const void* q, const void* k, const void* v, void* o, void* ws, int b, int lq, int lk, int h, int hk,
                       int64_t q_bs, int64_t q_rs, int64_t q_hs, int64_t k_bs, int64_t k_rs, int64_t k_hs, int64_t v_bs,
                       int64_t v_rs, int64_t v_hs, int64_t o_bs, int64_t o_rs, int64_t o_hs, float scale, float sink,
                       const float* qw, float eps, void* stream);
int gpu_int8_attn_norm_rope(const void* q, const void* k, const void* v, void* o, void* ws, int b, int lq, int lk, int h,
                            int hk, int64_t q_bs, int64_t q_rs, int64_t q_hs, int64_t k_bs, int64_t k_rs, int64_t k_hs,
                            int64_t v_bs, int64_t v_rs, int64_t v_hs, int64_t o_bs, int64_t o_rs, int64_t o_hs, float scale,
                            const float* qw, const float* kw, float eps, const float* rope, int rope_mode, void* stream);

int64_t gpu_int8_attn_key_bias_workspace(int b, int h, int hk, int lq, int lk);
int gpu_int8_attn_key_bias(const void* q, const void* k, const void* v, void* o, void* ws, int b, int lq, int lk, int h,
                           int hk, int64_t q_bs, int64_t q_rs, int64_t q_hs, int64_t k_bs, int64_t k_rs, int64_t k_hs,
                           int64_t v_bs, int64_t v_rs, int64_t v_hs, int64_t o_bs, int64_t o_rs, int64_t o_hs, float scale,
                           const float* bias, void* stream);

/* Test hook, no reference counterpart: y[i] = the gfx950 float -> u8 pack conversion of x[i] (byte 0), which the attention
 * kernel's probabilities rely on being round-to-nearest-even with saturation to 0..255. */
int gpu_internal_cvt_pk_u8_probe(const float* x, uint32_t* y, int n, void* stream);

/* Measurement hook, no reference counterpart: gpu_w6a8_group_gemm (bf16 output, no bias) with parts of its kernel left
 * out, to show what each costs next to the MFMAs: ablate bit 0 the fp32 fold, bit 1 the unpack, bit 2 the LDS-DMA after
 * the prologue (0..7).  With bit 3 set (8, 9, 12, 13 only) the kernel is the form that fetches weights already expanded
 * to int8, and Wp must then point at int8 [N, K] (N*K bytes), not at the packed words.  Shapes are checked as in
 * gpu_w6a8_group_gemm; any other value of ablate returns -200.  D receives meaningless values unless ablate is 0 or 8. */
int gpu_internal_w6a8_group_gemm_ablate(int ablate, const int8_t* A, const void* Wp, const float* xs, const float* sw, void* D,
                                        int64_t M, int64_t N, int64_t K, void* stream);

/* Test hook, no reference counterpart: which form of gpu_w6a8_group_gemm runs.  0 = the weights are expanded to int8
 * inside the kernel, per workgroup; 1 = they are expanded once into a stream-ordered scratch (N*K bytes) and the kernel
 * fetches them like A; -1 = by M (the second form from 4096 rows on).  Both forms give the same bits. */
int gpu_internal_w6a8_group_gemm_mode(int mode);

/* Test hook, no reference counterpart: sums of squares of rows of 128 floats in the order the fused norm of
 * gpu_int8_attn_norm_rope takes them; out[2r] from the quantizers' eight-lane form, out[2r+1] from the anchor search's
 * one-thread form; split != 0 is rope_mode 2's lane layout.  rows % 8 == 0. */
int gpu_internal_attn_sumsq_probe(const float* x, float* out, int rows, int split, void* stream);

/* Test hook, no reference counterpart: byte offsets of the pieces of the attention workspace and its tiling,
 * out[0..9] = qi, ki, qs, ks, vt, vs, anchors, vsum, key tile length, key tiles. */
int gpu_internal_attn_layout(int b, int h, int hk, int lq, int lk, int64_t* out);
int gpu_internal_attn_layout_d(int b, int h, int hk, int lq, int lk, int head_dim, int64_t* out);

/* D[M,N] = Out((A[M,K] . W[N,K]^T) * xs[m] * ws[n] + bias[n]).
 * Replaces gpu_int8_gemm, src/ffi.rs:38 / csrc/gemm.cu:124-129.
 * A, W int8 row-major (K contiguous); xs f32 [M]; ws f32 [N]; bias Out[N] or null; D Out[M,N]; out_dt a DT_* code.
 * K % 16 == 0 is the fast path; K % 16 == 8 (the reference's alignment-8 tile configurations,
 * csrc/vendor/cutlass_gemm_int8.cu:191,237-247) runs on zero-padded copies of A and W in a stream-ordered allocation
 * (A and W 8-byte aligned); any other K is refused.
 * M <= 256 with long K and few output columns splits K; the int32 planes of the slices go to a 24 MiB buffer that the
 * first such call on a stream allocates (hipMalloc) and the library keeps for that stream.  That first call should be
 * made outside graph capture; under capture, on a ninth stream or on hipStreamPerThread the call uses hipMallocAsync /
 * hipFreeAsync on `stream` instead, as does a shape whose planes exceed the buffer (more than 256 rows). */
int gpu_int8_gemm(const int8_t* A, const int8_t* W, const float* xs, const float* ws, const void* bias, void* D,
                  int64_t M, int64_t N, int64_t K, int out_dt, void* stream);

/* D = Out(float(Out(acc*xs*ws + bias)) * rscale[n] + resid[m,n]); D may alias resid.
 * Replaces gpu_int8_gemm_residual, src/ffi.rs:39-40 / csrc/gemm.cu:132-140. */
int gpu_int8_gemm_residual(const int8_t* A, const int8_t* W, const float* xs, const float* ws, const void* bias,
                           const void* rscale, const void* resid, void* D, int64_t M, int64_t N, int64_t K,
                           int out_dt, void* stream);

/* Packed 6-bit weights (two planes per row: K/2 nibble bytes, then K/4 top-bit bytes) with fp8-e4m3 scales
 * s_rel[N, K/G] -> int8 [N, K].  Replaces gpu_w6_decode, src/ffi.rs:121 / csrc/h3.cu:40-46. */
int gpu_w6_decode(const void* q, const void* s_rel, void* out, int64_t N, int K, int G, void* stream);

/* ---------------------------------------------------------------------------------------------------------------
 * Additions with no counterpart in the reference.
 * ------------------------------------------------------------------------------------------------------------- */

/* Builds, for the current device, the lookup tables that the prologues GATE / SWIGLU / SILU / GELU / GELU_TANH / SITU and
 * the SD GEGLU source use on 16-bit rows (all 65536 inputs of each activation, about 1.2 MB, held until the process
 * ends).  Optional: the first call with such a prologue builds them itself, with two device allocations, a fill kernel
 * on a stream of its own and a wait for it -- unless its stream is being captured, in which case that call evaluates
 * the activations per element (same bits, slower) and a later call builds the tables.  Call this once at
 * start-up to keep every quantizer call asynchronous and capturable.  Returns 0, or -1 if the tables could not be
 * built (calls then evaluate per element, and a later call tries again). */
int gpu_act_tables_init(void);

/* The int32 accumulators of gpu_int8_gemm, before the epilogue: acc[M,N] = A . W^T.  For bit-exact checks. */
int gpu_int8_gemm_acc(const int8_t* A, const int8_t* W, int32_t* acc, int64_t M, int64_t N, int64_t K, void* stream);

/* gpu_int8_gemm for callers that cannot allocate device memory (code under HIP graph capture, serving loops and
 * harnesses that forbid hipMalloc): same arguments, same results bit for bit, but the int32 planes of a split-K run
 * (M <= 256 with a narrow N) live in a fixed 24 MiB device array inside the library instead of a buffer allocated
 * for the stream, and the call makes no hipMalloc / hipFree of any kind, first call included.  No counterpart in the reference.
 * Every call on one GPU shares that GPU's array: calls that overlap in time on one GPU (two streams, two threads) race
 * on it and must be serialized by the caller.  Nothing in the array needs clearing between calls (every plane element
 * is written before it is read).  The first call on a device looks up the array's address and sets kernel attributes:
 * make it once before capturing a graph that contains this call.  The array occupies its 24 MiB on every device the
 * process uses, from the moment the library is loaded.  A shape whose planes would not fit returns -210 with a message on
 * stderr (every shape the automatic choice splits fits; with gpu_int8_gemm_force_config(6), M > 256 can exceed it);
 * gpu_int8_gemm_static_limit() returns the array's size in bytes.  K % 16 == 8, which gpu_int8_gemm serves from
 * padded copies that it allocates, is refused here (-200).  Other return codes as gpu_int8_gemm. */
int gpu_int8_gemm_static(const int8_t* A, const int8_t* W, const float* xs, const float* ws, const void* bias, void* D,
                         int64_t M, int64_t N, int64_t K, int out_dt, void* stream);
int64_t gpu_int8_gemm_static_limit(void);

/* One W6A8 linear in a single call: gpu_w6_decode into a stream-ordered scratch buffer, then gpu_int8_gemm with
 * ws = s_channel (the call pattern of src/h3.rs:1208-1216,1251).  Returns -1 for K % 32 or G % 16, otherwise as
 * gpu_int8_gemm. */
int gpu_w6a8_gemm(const int8_t* A, const void* wq, const void* s_rel, int G, const float* xs, const float* s_channel,
                  const void* bias, void* D, int64_t M, int64_t N, int64_t K, int out_dt, void* stream);

/* W6A8 linear with fp32 scales per group of 128 along K, for this library's own packed format (no counterpart in the
 * reference, whose W6 weights are two-plane with e4m3 group factors: gpu_w6_decode / gpu_w6a8_gemm above).  Up to 4095
 * rows of A the weights are expanded to int8 inside the GEMM kernel, ahead of the MFMA; from 4096 rows on they are
 * expanded once into a stream-ordered scratch of N*K bytes (hipMallocAsync / hipFreeAsync on the call's stream) that
 * the same kernel then fetches like A.  Same bits either way.
 *   Wp  uint8 [N, 3K/4]: codes u = q + 32 with q in [-32, 31]; every three bytes are the little-endian 24-bit word
 *       u0 | u1 << 6 | u2 << 12 | u3 << 18 of four consecutive k.
 *   sw  f32 [N, K/128]: one scale per output channel and group of 128 along K.
 *   D[m,n] = Out(fma(accf, xs[m], bias[n])), where accf starts at 0 and takes accf = fma(float(p_g), sw[n,g], accf) for
 *       g = 0, 1, ..., with p_g the exact int32 dot product of A[m, 128g .. 128g+127] and the codes q[n, same].
 *   partials: null, or int32 [M, N, K/128] that receives every p_g (a check hook; slow).
 * A rows, Wp rows and D are 16-byte aligned (K % 128 == 0 gives that for rows of contiguous tensors).
 * Returns -1 for K % 128 != 0; -200 for an unknown out_dt, K == 0, or sizes beyond 32-bit byte offsets. */
int gpu_w6a8_group_gemm(const int8_t* A, const void* Wp, const float* xs, const float* sw, const void* bias, void* D,
                        int32_t* partials, int64_t M, int64_t N, int64_t K, int out_dt, void* stream);

/* Test and tuning hook: force the GEMM kernel family.  1, 2 = 128x128 and 64x64 register-staged tiles; 6 =
 * weight-streaming kernel (256x96 tiles, two groups of waves taking turns on the K tiles, split K when N is small) for
 * M <= 256; 7 = four-wave persistent ring kernel on
 * 128x192 tiles (shapes with few tiles); 9 = two-group kernel (256x256 and 128x256 tiles, one launch), the choice for
 * large shapes; -1 = automatic.  A shape a family cannot run falls back to 1. */
int gpu_int8_gemm_force_config(int cfg);

/* Writes, for each of the 64 lanes and 16 accumulator registers of one v_mfma_i32_32x32x32_i8, the (row of src0,
 * row of src1) pair that the register holds, as out[lane*16 + r] = i*32 + j.  A start-up self check of the operand
 * layout the GEMM kernels assume; out is int32 [1024]. */
int gpu_mfma_layout_probe(int32_t* out, void* stream);

/* Measurement hook: one workgroup of four waves per CU runs iters * 64 v_mfma_i32_32x32x32_i8 per wave (or, with bit 1 of
 * random_bits set, iters * 128 v_mfma_i32_16x16x64_i8: the same operations) on operands held in registers (all zero,
 * or pseudo-random bits when bit 0 of random_bits is set) and nothing else.  cycles[i] receives the
 * shader-clock count of workgroup i (one entry per CU, device int64); ops per launch = CUs * 4 * iters * 64 * 65536.
 * Timed from outside with events, this gives the matrix pipes' ceiling under the chip's power management and, from the
 * cycle counts, the shader clock it settles at.  sink: one device int32 (never written in practice). */
int gpu_mfma_ceiling_probe(int iters, int random_bits, int64_t* cycles, int32_t* sink, void* stream);

/* Library build tag (a static string). */
const char* gpu_kernels_build_info(void);

#ifdef __cplusplus
}
#endif
#endif /* GPU_API_H */
