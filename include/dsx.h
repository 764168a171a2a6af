/*
 * dsx.h — C ABI of libdsx.so: hand-written gfx950 (MI355X / CDNA4) kernels for the
 * DiT denoising-step hot path of DiffSynth-Engine.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer owned by the caller unless stated otherwise;
 *     the library never allocates, frees or keeps device memory;
 *   - every launch goes to the hipStream_t passed as `stream` (NULL = default stream)
 *     and returns without synchronising;
 *   - the return value is DSX_OK (0) or a negative DSX_E* code; nothing throws or exits;
 *   - "bf16" is the 16-bit brain float, "e4m3" the 8-bit OCP float8_e4m3fn
 *     (bias 7, max 448, no inf, 0x7f/0xff = NaN);
 *   - strides and leading dimensions are counted in ELEMENTS of the tensor they describe.
 *
 * Each entry point names the interface of the reference (DiffSynth-Engine v0.1.1,
 * paths relative to its root) whose arithmetic it replaces.
 */
#ifndef DSX_H
#define DSX_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DSX_ABI_VERSION 7

enum {
  DSX_OK = 0,
  DSX_EBADSHAPE = -1, /* a size/stride the kernels do not support          */
  DSX_EALIGN = -2,    /* a pointer or leading dimension not 16-byte aligned */
  DSX_EARCH = -3,     /* current device is not gfx950                       */
  DSX_ELAUNCH = -4,   /* hipLaunchKernel reported an error                  */
  DSX_ENULL = -5,     /* a required pointer is NULL                         */
  DSX_EWORKSPACE = -6 /* the call needs scratch memory that was not given (or more of it) */
};

/* Version of this ABI (DSX_ABI_VERSION of the library that was built). */
int dsx_abi_version(void);

/* Static, NUL-terminated description of a DSX_* code. */
const char* dsx_strerror(int code);

/* 0 when the current HIP device is gfx950, DSX_EARCH otherwise. */
int dsx_check_device(void);

/*
 * Activation quantisation: bf16 -> e4m3, one row ("token") at a time.
 * Replaces `input.to(torch.float8_e4m3fn)` in diffsynth_engine/utils/fp8_linear.py:35.
 *
 *   scale_out == NULL : bare cast, q[m,k] = e4m3_rne(x[m,k]); exactly torch's cast
 *                       (round-to-nearest-even, subnormals kept, |v| > 464 -> NaN).
 *   scale_out != NULL : dynamic per-token scale, a = max(absmax(x[m,:]), 1e-12), s[m] = a / 448,
 *                       q[m,k] = e4m3_rne(float(x[m,k]) * (448 / a)); both divisions and the
 *                       product are single correctly rounded fp32 operations.
 * x: (M,K) bf16, row stride ldx; q: (M,K) e4m3, row stride ldq; K % 8 == 0.
 */
int dsx_quant_fp8_rowwise(const void* x, int64_t ldx, void* q, int64_t ldq, float* scale_out,
                          int64_t M, int64_t K, void* stream);

/*
 * Weight quantisation helper: fp32 absmax of a bf16 (or fp32 when is_fp32 != 0) buffer of n
 * elements into *absmax_out (device fp32, must be zero-initialised by the caller).
 * Used by enable_fp8_linear (diffsynth_engine/utils/fp8_linear.py:7-17) for the per-tensor scale.
 */
int dsx_absmax(const void* x, int64_t n, int is_fp32, float* absmax_out, void* stream);

/*
 * Per-tensor scaled cast.  absmax == NULL: bare cast q[i] = e4m3_rne(x[i]) (scale_out untouched).
 * Otherwise a = max(*absmax, 1e-12), *scale_out = a / 448, q[i] = e4m3_rne(float(x[i]) * (448 / a));
 * each division and the product is a single correctly rounded fp32 operation.
 * Replaces `module.weight.data.to(torch.float8_e4m3fn)` (fp8_linear.py:15).
 */
int dsx_cast_fp8_scaled(const void* x, int is_fp32, const float* absmax, float* scale_out, void* q,
                        int64_t n, void* stream);

/*
 * FP8 scaled GEMM with fused bias:
 *   out[m,n] = bf16( (sum_k a[m,k] * w[n,k]) * a_scale[m] * (*w_scale) + bias[n] ), fp32 accumulate.
 * Replaces `torch._scaled_mm(input, weight.T, scale_a, scale_b, bias, out_dtype)` in
 * diffsynth_engine/utils/fp8_linear.py:41-48,52-59.
 *   a: (M,K) e4m3 row-major (lda); w: (N,K) e4m3 row-major (ldw), i.e. nn.Linear.weight as stored;
 *   a_scale: M fp32 or NULL (= 1); w_scale: device fp32 scalar or NULL (= 1); bias: N bf16 or NULL;
 *   out: (M,N) bf16 (ldo).  K % 16 == 0, lda/ldw % 16 == 0, ldo % 8 == 0 when N % 8 == 0;
 *   M, N, K <= 2^30, lda and ldw < 2^24 (operand offsets inside a tile are 32-bit), ceil(M/64)*ceil(N/64) <= 2^30.
 */
int dsx_fp8_gemm(const void* a, int64_t lda, const void* w, int64_t ldw, const float* a_scale,
                 const float* w_scale, const void* bias, void* out, int64_t ldo, int64_t M,
                 int64_t N, int64_t K, void* stream);

/*
 * dsx_fp8_gemm with the gated residual of the DiT blocks fused into its epilogue:
 *   proj = bf16( acc * a_scale[m] * w_scale + bias[n] );   out[m,n] = bf16( resid[m,n] + bf16(gate[b,n] * proj) )
 * (gate == NULL: out = bf16(resid + proj)); b = m / rows_per_batch, gate row stride gate_sb.
 * Replaces the `x + gate * linear(...)` pairs at models/flux/flux_dit.py:227,229,232,234,318-319 and
 * models/wan/wan_dit.py:189,190,192 without the separate read-modify-write pass.
 * `out` may be `resid` itself.
 */
int dsx_fp8_gemm_gated_residual(const void* a, int64_t lda, const void* w, int64_t ldw,
                                const float* a_scale, const float* w_scale, const void* bias,
                                const void* resid, int64_t ldr, const void* gate, int64_t gate_sb,
                                int64_t rows_per_batch, void* out, int64_t ldo, int64_t M, int64_t N,
                                int64_t K, void* stream);

/*
 * Up to DSX_GEMM_GROUP_MAX independent FP8 GEMMs submitted together.  Each problem is exactly
 * dsx_fp8_gemm (resid == NULL) or dsx_fp8_gemm_gated_residual (resid != NULL) with the same argument
 * meaning and the same checks; neighbouring problems that both qualify for the 256x256-tile kernel
 * and are of the same kind (plain, residual, q/k epilogue) share ONE launch, so a small problem runs on compute units a
 * large one leaves idle.  The reference issues the image-stream and text-stream linears of a joint
 * block as separate F.linear calls (diffsynth_engine/models/flux/flux_dit.py:165-171,190-194,
 * 227-235); this is those pairs.  All problems are validated before anything is launched.
 */
#define DSX_GEMM_GROUP_MAX 4
typedef struct dsx_gemm_problem {
  const void* a; int64_t lda;          /* (M,K) e4m3 */
  const void* w; int64_t ldw;          /* (N,K) e4m3 */
  const float* a_scale;                /* M fp32 or NULL */
  const float* w_scale;                /* device fp32 scalar or NULL */
  const void* bias;                    /* N bf16 or NULL */
  const void* resid; int64_t ldr;      /* (M,N) bf16 or NULL */
  const void* gate; int64_t gate_sb;   /* (batch,N) bf16 or NULL; needs resid */
  int64_t rows_per_batch;              /* >= 1 when resid is given */
  void* out; int64_t ldo;              /* (M,N) bf16 */
  int64_t M, N, K;
  /* Optional (qk_heads > 0; resid must be NULL): the problem is a packed qkv projection whose columns
   * [0, 128*qk_heads) are q heads and [128*qk_heads, 256*qk_heads) k heads (further columns: v, ... untouched),
   * and the per-head RMSNorm (q_norm_w / k_norm_w, bf16 (128,), either may be NULL) and the RoPE rotation
   * (rope: fp32 (cos, sin) table as in dsx_attn_params, NULL = none) are applied to those heads in the epilogue,
   * after bias and the bf16 rounding of the projection and before the store: bit-identical to dsx_rmsnorm_rope_qk
   * run in place on the stored projection.  Row m is token m % rows_per_batch of batch entry m / rows_per_batch and
   * takes table row rope_pos0 + m % rows_per_batch (+ rope_sb per batch entry); rope_rows rows per entry exist.
   * Replaces norm_q / norm_k and apply_rope at models/flux/flux_dit.py:165-171,179-180,297-301 (RMSNorm:
   * models/basic/transformer_helper.py:73-78) without a pass of its own.  Needs the shape the 256x256-tile kernel
   * takes (M > 8, K % 128 == 0, N % 8 == 0, 16-byte aligned out), DSX_EBADSHAPE otherwise. */
  const void* q_norm_w; const void* k_norm_w;
  const float* rope; int64_t rope_sb, rope_pos0, rope_rows;
  float norm_eps;
  int32_t qk_heads;
  /* Optional extension of the reduction axis (K_ext > 0): the product runs over the K columns of (a, w) followed by
   * the K_ext columns of (a_ext, w_ext), as if the operands were the concatenations [a | a_ext] (M, K + K_ext) and
   * [w | w_ext] (N, K + K_ext), without either concatenation existing; one accumulation, one pair of scales, every
   * epilogue as usual.  This is how an unfused low-rank update rides the main product (dsx_lora_down writes a_ext;
   * LoRALinear.forward, models/basic/lora.py:29-32,137-141).  K_ext % 128 == 0, K >= 256, and the shape the
   * 256x256-tile kernel takes (as for qk_heads), DSX_EBADSHAPE otherwise. */
  const void* a_ext; int64_t lda_ext;  /* (M,K_ext) e4m3 */
  const void* w_ext; int64_t ldw_ext;  /* (N,K_ext) e4m3 */
  int64_t K_ext;
} dsx_gemm_problem;
int dsx_fp8_gemm_grouped(const dsx_gemm_problem* problems, int count, void* stream);

/*
 * Down projection of unfused low-rank updates, written as the extension operand of the main product
 * (dsx_gemm_problem.a_ext): out[m, c ranks + r] = e4m3_saturating(row_scale[r] * sum_k a[m,k] d[r,k]) for
 * r < ranks and c < copies, zero codes from column copies * ranks up to E.  a (M,K) e4m3 codes of the activation (its
 * per-token scale is applied later, by the main product, to the whole extended sum), d (R,K) e4m3: the down factors
 * of every update on the layer stacked row-wise and zero-padded from row `ranks` to R, row_scale (R) fp32: per
 * stacked row the product of its factor's quantisation scale and of whatever the caller folded into the matching
 * columns of w_ext (1 / copies included: writing a row's values `copies` times, against as many repeats of w_ext's
 * columns, keeps each of them that much further from e4m3's end).
 * R % 32 == 0, R <= 128, ranks % 4 == 0, ranks <= R, 1 <= copies <= 32, E >= copies * ranks, E % 16 == 0,
 * K % 128 == 0, lda and ldd below 2^24 (DSX_EBADSHAPE otherwise); a, d, out and their leading dimensions 16-byte
 * aligned (DSX_EALIGN).
 * Replaces `lora.down(x)` of LoRA.forward (diffsynth_engine/models/basic/lora.py:29-32) for every update of a layer
 * in one HBM-bound pass over a.
 */
int dsx_lora_down(const void* a, int64_t lda, const void* d, int64_t ldd, const float* row_scale, void* out,
                  int64_t ldo, int64_t M, int64_t K, int64_t R, int64_t ranks, int64_t copies, int64_t E,
                  void* stream);

/*
 * Small-M (M <= 8) form of dsx_fp8_gemm with one weight scale PER OUTPUT ROW (w_row_scale[n]), so that
 * several Linear layers that consume the same activation can be stacked into one (N_total, K) weight
 * and evaluated by one HBM-bound pass.  Used for the AdaLN projections, which all consume
 * silu(conditioning) (models/basic/transformer_helper.py:14,33; models/flux/flux_dit.py:332).
 */
int dsx_fp8_gemv_rowscale(const void* a, int64_t lda, const void* w, int64_t ldw, const float* a_scale,
                          const float* w_row_scale, const void* bias, void* out, int64_t ldo, int64_t M,
                          int64_t N, int64_t K, void* stream);

/*
 * Flash attention, head dim 128, bf16 in/out, fp32 online softmax, non-causal, no mask.
 * Replaces `_attn_func(q, k, v)` = F.scaled_dot_product_attention in
 * diffsynth_engine/models/flux/flux_dit.py:21,182,267,303 and `attention()` in
 * diffsynth_engine/models/wan/wan_dit.py:18-22; with `rope`/`*_norm_w` set it also replaces
 * RMSNorm (models/basic/transformer_helper.py:73-78) and apply_rope (flux_dit.py:154-159)
 * on q and k, and the text-first concat (flux_dit.py:176-178) through the two segments.
 *
 * The query sequence is the concatenation of up to two segments (segment 0 first), each read
 * from its own base pointer with its own strides; likewise keys/values and the output.
 * Element (b,h,s,d) of segment g of q lives at q[g][b*q_sb[g] + h*q_sh[g] + s*q_ss[g] + d].
 */
typedef struct dsx_attn_params {
  const void* q[2];   /* bf16; q[1] may be NULL when sq[1] == 0 */
  const void* k[2];
  const void* v[2];
  void* o[2];         /* bf16 */
  int64_t sq[2];      /* query rows per segment  */
  int64_t skv[2];     /* key/value rows per segment */
  int64_t q_sb[2], q_sh[2], q_ss[2];
  int64_t k_sb[2], k_sh[2], k_ss[2];
  int64_t v_sb[2], v_sh[2], v_ss[2];
  int64_t o_sb[2], o_sh[2], o_ss[2];
  int32_t batch, heads, head_dim; /* head_dim must be 128 */
  float softmax_scale;            /* e.g. 1/sqrt(128) */
  /* Optional fused pre-processing of q and k (NULL = off):
   *   rope      : fp32 table (rope_sb*b + pos*128 + 2*i + {0,1}) = (cos, sin) of pair i at
   *               joint position pos (segment 0 rows first); applied to q and k on pairs (2i,2i+1),
   *               result rounded to bf16.  The table holds rope_rows rows per batch entry; rope_rows must
   *               be at least sq[0]+sq[1] (= skv[0]+skv[1]: the option is for self / joint attention), and
   *               rope_sb is 0 (one table for every batch entry) or at least rope_rows*128.
   *   q_norm_w/k_norm_w[g] : bf16 (128,) RMSNorm weight of segment g; y = bf16(bf16(x*rsqrt(ms+eps))*w). */
  const float* rope;
  int64_t rope_sb;
  int64_t rope_rows;
  const void* q_norm_w[2];
  const void* k_norm_w[2];
  float norm_eps;
  /* Optional promise by the caller: |softmax_scale * q.k| <= score_bound for every query/key pair after
   * the pre-processing above (0 = no promise).  With score_bound*log2(e) <= 64 the kernel keeps the
   * softmax reference at 0 and skips the running maximum; the result is the same softmax.  E.g. after
   * RMSNorm over head_dim with weights wq, wk: head_dim * max|wq| * max|wk| * softmax_scale.  A promise
   * that does not hold can overflow exp2. */
  float score_bound;
  /* Scratch owned by the caller (NULL = none, 16-byte aligned); dsx_attn_workspace_bytes gives the size that
   * serves both uses:
   *  - fused pre-processing of k (rope, k_norm_w): k is normalised/rotated ONCE into the first
   *    2*batch*heads*Skv*128 bytes by a row kernel and the attention kernel reads it from there (every query
   *    block of a head reads all of that head's k, so the work is not repeated per block); q is treated as the
   *    attention kernel loads it, each row once, and needs no scratch.  A call that asks for rope or k_norm_w
   *    without that much scratch returns DSX_EWORKSPACE;
   *  - load balance (optional): when the (batch, head, 256-query block) units do not fill the last round of
   *    workgroups, the key ranges of that round's units are cut into equal pieces over all compute units
   *    and a second kernel merges the partial softmax results held in the scratch.
   * Calls that share a scratch must not overlap. */
  void* workspace;
  int64_t workspace_bytes;
  /* Optional score bound read ON THE DEVICE when the kernels run (NULL = none): two floats,
   * [0] >= |q row|^2 and [1] >= |k row|^2 (squared 2-norms over head_dim) for every (batch, head, row) the call
   * reads, e.g. the maxima dsx_rmsnorm_rows leaves in its head_norm2_max.  |q.k| <= sqrt([0]*[1]) bounds every
   * score; when softmax_scale*log2(e)*sqrt([0]*[1]) (plus 1 % for roundings) is at most 64 the kernel that keeps
   * the softmax reference at 0 does the work, otherwise (Inf and NaN included) the one with the running maximum
   * does: both are launched and the one not chosen returns at once, so the host never waits for the values and
   * the call can sit in a captured graph.  Same softmax either way.  Not combined with the fused pre-processing
   * (rope, *_norm_w change the rows the bound describes): DSX_EBADSHAPE.  Ignored when score_bound already
   * holds a promise.  Unlike score_bound this one cannot be wrong as long as the two floats are true maxima. */
  const float* qk_norm2_max;
} dsx_attn_params;

int dsx_attn_fwd(const dsx_attn_params* p, void* stream);

/* Scratch bytes with which dsx_attn_fwd(p) runs and uses every option described at `workspace` (0: none is
 * needed or would be used).  Reads the shapes and the fused-option pointers of *p only; launches nothing.  No counterpart in
 * the reference, whose attention backends allocate their own temporaries. */
int64_t dsx_attn_workspace_bytes(const dsx_attn_params* p);

/*
 * dsx_attn_fwd for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): same arguments, same kernels, same results, but the scratch is a
 * static device array of DSX_ATTN_STATIC_SCRATCH_BYTES inside the library instead of `workspace`, which must be
 * NULL.  It has no counterpart in the reference, whose attention backends allocate their temporaries themselves.
 * Calls whose dsx_attn_workspace_bytes exceeds the array return DSX_EWORKSPACE before anything is launched; the
 * limit (64 MiB) covers the k copy of a fused RMSNorm/RoPE call at batch * heads * Skv <= 262144 rows (Flux at
 * 1024 x 1024: 24 heads x 4608 tokens = 27 MiB) and the partial results of a key-range split of a few dozen units.  Each GPU the library runs on holds its own copy of the array until the process
 * ends.  Every call on a GPU shares that GPU's array: calls that overlap on one GPU (different streams, or
 * threads) race; calls on one stream are ordered and safe.  Nothing in the array has to start at zero: every
 * byte a call reads was written earlier in that same call.  The entry point calls no hipMalloc, hipFree or other
 * allocating routine.
 */
#define DSX_ATTN_STATIC_SCRATCH_BYTES (64ll << 20)
int dsx_attn_fwd_static(const dsx_attn_params* p, void* stream);

/* DSX_ATTN_STATIC_SCRATCH_BYTES of the library that was built. */
int64_t dsx_attn_static_scratch_bytes(void);

/*
 * Standalone RMSNorm + RoPE of q and k (same arithmetic and rounding points as the fused
 * option of dsx_attn_fwd), written to a strided (B,H,S,128) bf16 view; `out` may be `x` itself
 * (in place).  One tensor per call.  Row s of every head takes table row rope_pos0 + s (+ rope_sb floats per batch
 * entry): the table must hold rope_pos0 + seq rows of 128 floats per entry; the call cannot check that.
 * Replaces RMSNorm.forward (transformer_helper.py:73-78) followed by apply_rope (flux_dit.py:154-159).
 */
int dsx_rmsnorm_rope(const void* x, int64_t x_sb, int64_t x_sh, int64_t x_ss, const void* norm_w,
                     float eps, const float* rope, int64_t rope_sb, int64_t rope_pos0, void* out,
                     int64_t o_sb, int64_t o_sh, int64_t o_ss, int32_t batch, int32_t heads,
                     int64_t seq, void* stream);

/*
 * The same RMSNorm + RoPE applied in place to the q heads and the k heads of a packed qkv
 * projection in ONE pass: token row at x + b*x_sb + s*x_ss, head h of that token at + h*128,
 * heads [0, heads_q) normalised with q_norm_w, heads [heads_q, heads_q + heads_k) with k_norm_w
 * (either weight may be NULL = no norm), all rotated by the RoPE row rope_pos0 + s (rope NULL = no
 * rotation; the table must hold rope_pos0 + seq rows per batch entry, which the call cannot check).  This is the
 * layout FluxJointAttention.forward / process_attention give q and k before chunking (flux_dit.py:165-171,297-301:
 * view (B,S,3H,D), norm_q/norm_k, apply_rope).
 */
int dsx_rmsnorm_rope_qk(void* x, int64_t x_sb, int64_t x_ss, int32_t heads_q, int32_t heads_k,
                        const void* q_norm_w, const void* k_norm_w, float eps, const float* rope,
                        int64_t rope_sb, int64_t rope_pos0, int32_t batch, int64_t seq, void* stream);

/*
 * RMSNorm over whole rows followed by an optional per-head RoPE (head dim 128):
 *   y = bf16( bf16(x * rsqrt(mean(x^2) + eps)) * w ), then pairs (2i,2i+1) of every 128-wide head are rotated by
 *   the (cos, sin) of table row (row % rows_per_batch) [+ rope_sb per batch entry] and rounded to bf16.
 * Replaces Wan's RMSNorm.forward over the full model dim (models/wan/wan_dit.py:61-78,98-99,142-143) and
 * rope_apply (wan_dit.py:54-58; the reference multiplies in complex128, this kernel in fp32).
 * x, out: (rows, D) bf16; w: (D,) bf16; rope: fp32 (pos, 64, 2) or NULL, rows_per_batch table rows per batch
 * entry (not checkable here).  D % 8 == 0 (128 with rope), D <= 16384.
 * head_norm2_max (device, one float, or NULL; needs D % 128 == 0): raised (atomic maximum, never lowered) to the
 * largest squared 2-norm of a 128-wide head of an output row; the caller sets it to 0 before the first call
 * that contributes.  It is what dsx_attn_params.qk_norm2_max reads (no counterpart in the reference).
 */
int dsx_rmsnorm_rows(const void* x, int64_t ldx, const void* w, float eps, const float* rope, int64_t rope_sb,
                     int64_t rows_per_batch, void* out, int64_t ldo, int64_t rows, int64_t D, float* head_norm2_max,
                     void* stream);

/*
 * AdaLN modulate: y = LayerNorm(x; eps, no affine) * (1 + scale) + shift, one row per token.
 * Replaces `self.norm(x) * (1 + scale) + shift` in models/basic/transformer_helper.py:17,21,35,
 * models/flux/flux_dit.py:228,233,334 and `modulate(norm(x), shift, scale)` in
 * models/wan/wan_dit.py:25-26,188,191,236.
 *   x: (B*S, D) bf16 (ldx); scale, shift: bf16 (D,) per batch entry, batch stride mod_sb
 *   (row r uses batch r / rows_per_batch); ln_w/ln_b: optional bf16 affine (Wan norm3) or NULL.
 *   y_bf16 (ldy) and/or (q_fp8 (ldq) + q_scale[rows]) are written; either may be NULL.  q without q_scale is the
 *   reference's bare cast (utils/fp8_linear.py:35): unit scale, values beyond e4m3's range become NaN (this holds
 *   for dsx_gelu_tanh, dsx_gelu_erf and dsx_concat_gelu_tanh too).
 *   Rounding follows the bf16 op sequence: bf16(LN) -> bf16(1+scale) -> bf16(mul) -> bf16(add).
 *   D % 8 == 0, D <= 16384.
 */
int dsx_adaln_modulate(const void* x, int64_t ldx, const void* scale, const void* shift,
                       int64_t mod_sb, int64_t rows_per_batch, const void* ln_w, const void* ln_b,
                       float eps, void* y, int64_t ldy, void* q, int64_t ldq, float* q_scale,
                       int64_t rows, int64_t D, void* stream);

/*
 * Gated residual: out = x + gate * y  (gate == NULL: out = x + y), bf16, gate (D,) per batch entry.
 * Replaces flux_dit.py:227,229,232,234,318-319 and wan_dit.py:189,190,192.
 * Rounding: bf16(x + bf16(gate * y)).
 */
int dsx_gated_residual(const void* x, int64_t ldx, const void* y, int64_t ldy, const void* gate,
                       int64_t gate_sb, int64_t rows_per_batch, void* out, int64_t ldo,
                       int64_t rows, int64_t D, void* stream);

/*
 * tanh-GELU: y = bf16(gelu_tanh(float(x))).  Replaces nn.GELU(approximate="tanh")
 * (flux_dit.py:209,215,315; wan_dit.py:180).  x may be a column slice of a wider buffer (ldx).
 * y_bf16 and/or (q_fp8 + q_scale) are written as in dsx_adaln_modulate.  D % 8 == 0, D <= 16384.
 */
int dsx_gelu_tanh(const void* x, int64_t ldx, void* y, int64_t ldy, void* q, int64_t ldq,
                  float* q_scale, int64_t rows, int64_t D, void* stream);

/*
 * erf-GELU, same arguments: y = bf16(x * 0.5 * (1 + erf(x / sqrt(2)))) in fp32.  Replaces the nn.GELU() of the
 * image-to-video CLIP embedder (models/wan/wan_dit.py:195-211, MLP.proj[2]).
 */
int dsx_gelu_erf(const void* x, int64_t ldx, void* y, int64_t ldy, void* q, int64_t ldq,
                 float* q_scale, int64_t rows, int64_t D, void* stream);

/*
 * Concatenating tanh-GELU: output row = [ prefix (Dp, copied) | gelu_tanh(x) (D) ], emitted as bf16
 * (ldy) and/or per-token-scaled e4m3 (ldq, q_scale) like dsx_gelu_tanh.  Replaces
 * `torch.cat([attn_output, F.gelu(mlp_hidden_states, approximate="tanh")], dim=2)` of the
 * single-stream block (models/flux/flux_dit.py:315-317).  Dp % 8 == 0, D % 8 == 0, Dp + D <= 16384.
 */
int dsx_concat_gelu_tanh(const void* prefix, int64_t ldp, int64_t Dp, const void* x, int64_t ldx, void* y,
                         int64_t ldy, void* q, int64_t ldq, float* q_scale, int64_t rows, int64_t D,
                         void* stream);

/*
 * Flow-match Euler update: out = cast(float(latents) + float(v) * dt), element-wise, bf16 or fp32
 * (is_fp32 selects the storage type of all three buffers).
 * Replaces FlowMatchEulerSampler.step (algorithm/sampler/flow_match/flow_match_euler.py:11-19).
 */
int dsx_flow_match_euler_step(const void* latents, const void* v, float dt, void* out, int64_t n,
                              int is_fp32, void* stream);

/*
 * Diagnostic, no counterpart in the reference: the on-box microbenchmark behind the roofline denominators.
 * Launches `workgroups` workgroups of four wavefronts that each run `iters` rounds of MFMAs on independent
 * accumulators (kind 0: v_mfma_f32_32x32x16_bf16, kind 1: v_mfma_f32_32x32x64 on e4m3 operands, four per round;
 * kinds 2 and 3: the 16x16x32 bf16 and 16x16x128 e4m3 shapes, same operand registers, eight per round; kind + 4:
 * the first operand changes from one MFMA to the next as well, as it does in a real kernel) on register operands
 * taken from
 * operand_bits (16 x 256 dwords, device memory; all zero or random, which changes power draw and with it the clock),
 * with no memory traffic inside the loop.  *flops_out (host memory, may be NULL) receives the flops of the launch; the
 * caller times it.  sink: one device float (never written for finite inputs).
 * iters <= DSX_PROBE_MAX_ITERS and workgroups <= DSX_PROBE_MAX_WORKGROUPS, DSX_EBADSHAPE beyond: one launch at the
 * caps is seconds of device time, and a longer one cannot be told from a hang by whoever shares the device.
 */
#define DSX_PROBE_MAX_ITERS (1ll << 22)
#define DSX_PROBE_MAX_WORKGROUPS (1 << 14)
int dsx_mfma_ceiling_probe(int kind, const void* operand_bits, int64_t iters, int32_t workgroups, void* sink,
                           int64_t* flops_out, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* DSX_H */
