/*
 * q8_hip.h - C ABI of libq8_hip.so: the 8-bit inference hot path of q8_kernels
 * (per-token quantizers, fast Hadamard transform, RMSNorm, RoPE, int8/fp8 GEMM
 * with fused dequant+bias+GELU, fp8 flash-attention forward) as hand-written
 * HIP kernels for gfx950 (MI355X).
 *
 * Conventions (all entry points):
 *   - every pointer is a DEVICE pointer owned by the caller; nothing is
 *     allocated, freed or retained by the library;
 *   - work is enqueued on `stream` (a hipStream_t passed as void*, NULL = the
 *     default stream) and the call returns without synchronising;
 *   - the return value is Q8_OK (0) or a negative Q8_ERR_* code; on error no
 *     kernel has been launched; q8_last_error() returns a thread-local text;
 *   - no global mutable state: calls are re-entrant and thread-safe per stream. (The error text, the last-kernel
 *     record and the two *_set_config overrides for tests and tuning are per-thread.)
 *
 * Each entry point cites the interface of the reference implementation
 * (KONAKONA666/q8_kernels, paths relative to its root) that it replaces.
 */
#ifndef Q8_HIP_H
#define Q8_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* q8_stream_t; /* hipStream_t */

/* element types */
enum {
    Q8_I8 = 0,   /* signed 8-bit integer codes                   */
    Q8_E4M3 = 1, /* OCP fp8 e4m3fn (bias 7, no inf, 0x7f = NaN)  */
    Q8_BF16 = 2,
    Q8_F16 = 3,
    Q8_F32 = 4
};

/* status codes */
enum {
    Q8_OK = 0,
    Q8_ERR_NULL = -1,      /* required pointer is NULL                      */
    Q8_ERR_DTYPE = -2,     /* unsupported element type for this entry point */
    Q8_ERR_SHAPE = -3,     /* unsupported or inconsistent sizes             */
    Q8_ERR_ALIGN = -4,     /* pointer or stride not aligned as required     */
    Q8_ERR_LAUNCH = -5,    /* the HIP runtime refused the launch            */
    Q8_ERR_FLAGS = -6      /* unknown flag bits                             */
};

/* q8_quant_rows flags */
enum {
    Q8_QUANT_RNE = 1,        /* int8 codes: round half to even instead of the reference's
                                round-half-away-from-zero                                  */
    Q8_QUANT_SCALE_DIV = 2   /* stored scale = absmax/QMAX instead of the reference's
                                1/(QMAX/absmax); the codes are unchanged                   */
};

/* q8_attn_fwd V layouts and flags */
enum {
    Q8_V_DS = 0, /* V given as [B,H,D,Nv] (the reference's pre-transposed contract), Nv >= N, Nv % 16 == 0 */
    Q8_V_SD = 1  /* V given as [B,H,N,D]                                                                    */
};
enum {
    Q8_ATTN_SUM_ROUNDED_P = 1, /* the row sum l runs over the e4m3-rounded probabilities (what multiplies V) instead of
                                  the unrounded fp32 ones, so every output is a convex combination of the v_j. The
                                  general kernel takes that sum on the matrix pipe (6 % faster on long sequences, as
                                  accurate against exact attention). Unit scales only; not with the 4 waves x 64
                                  queries tuning shape. The reference sums the unrounded probabilities.            */
    Q8_ATTN_P_UNIT_RANGE = 2,  /* form the probabilities as exp(s - max) <= 1 before their e4m3 cast, like the
                                  reference; by default they are scaled by 2^8 (the factor cancels in o / l),
                                  which keeps weights below 2^-10 of the maximum from being flushed to zero  */
    Q8_ATTN_O_TOKEN_MAJOR = 4, /* write o as [B, M, H, D] (the layout the output projection reads, which the
                                  reference reaches by transpose(1, 2).reshape, modules/attention.py:105)
                                  instead of [B, H, M, D]                                                     */
    Q8_ATTN_LAZY_MAX = 8       /* the maximum that the probabilities of a row are formed against is raised to the
                                  running maximum only when that has grown by more than a factor 8 beyond it
                                  (p = 2^5 exp(s - m) <= 2^8): about 5 % faster on long sequences, same error bound,
                                  but the largest weight of a row is no longer exact (mean error up to two thirds
                                  larger on sharply peaked rows). Not with P_UNIT_RANGE. No counterpart in the
                                  reference, which rescales against the running maximum in every tile.          */
};

/* q8_attn_prep_qk / _qk_pair / _qkv / _kv flags */
enum {
    Q8_PREP_FHT = 1,           /* D-point Hadamard transform * scale per head                                      */
    Q8_PREP_PAIR_TABLES = 2,   /* cos, sin hold one entry per rotated pair, [rows, H*D/2], instead of one per
                                  element: tables built by repeating every frequency twice
                                  (q8_kernels/models/LTXVideo.py:95-148) carry each value twice                    */
    Q8_PREP_SHARED_TABLES = 4  /* cos, sin hold the S positions of one batch element, [S, ...], and serve all B
                                  batch elements, instead of one row per token [B*S, ...]                          */
};

const char* q8_strerror(int status);
const char* q8_last_error(void);

/* CU count, peak engine clock (MHz), HBM bytes, and the gcn arch name (>= 32 bytes buffer, nullable). */
int q8_device_info(int* cu_count, int* clock_mhz, int64_t* hbm_bytes, char* arch_name);

/*
 * Token-wise (per-row) absmax quantizer.
 * Replaces quantizer._C.tokenwise_quant  (csrc/quantizer/tokenwise_quant.cpp:74-111,
 * kernel csrc/quantizer/tokenwise_quant_cuda.cu:91-149).
 *   a = max_j |x[r,j]|;  r = QMAX / a;  codes[r,j] = cast(x[r,j] * r);  scales[r] = 1 / r
 *   QMAX = 127 (Q8_I8, rounding half away from zero, see flags) or 448 (Q8_E4M3, RNE).
 *   A row of zeros yields codes 0 and scale 0.
 * x: [rows, dim] of x_dtype in {BF16,F16,F32,E4M3}, row stride x_row_stride elements,
 * unit column stride; codes: [rows, dim] contiguous; scales: [rows] fp32.
 * dim % 8 == 0, dim <= 32768; x rows and codes rows 16-byte aligned.
 */
int q8_quant_rows(const void* x, int x_dtype, void* codes, int code_dtype, float* scales,
                  int64_t rows, int dim, int64_t x_row_stride, int flags, q8_stream_t stream);

/*
 * Fast Walsh-Hadamard transform along the last dimension.
 * Replaces ops._C.fast_hadamard_transform  (csrc/fast_hadamard/fast_hadamard_transform.cpp:70-121,
 * kernel csrc/fast_hadamard/fast_hadamard_transform_cuda.cu:43-111).
 *   y[r,:] = (H_N [x[r,:], 0...0])[:dim] * scale,  N = 2^ceil(log2 dim), H_N Sylvester;
 *   butterflies in fp32 with ascending stride; cast to y_dtype (E4M3: RNE, |v| > 464 -> NaN).
 * x_dtype, y_dtype in {BF16, E4M3}; dim % 8 == 0, dim <= 32768; rows contiguous
 * (row stride = dim); x and y 16-byte aligned.
 */
int q8_fht(const void* x, int x_dtype, void* y, int y_dtype, int64_t rows, int dim, float scale,
           q8_stream_t stream);

/*
 * RMSNorm forward.
 * Replaces ops._C.rms_norm  (csrc/ops/rms_norm.cpp:103-154, kernel csrc/ops/rms_norm_cuda.cu:101-171).
 *   rstd[r] = rsqrt(mean_j x[r,j]^2 + eps);  y[r,j] = (x[r,j] * rstd[r]) * w[j]   (w NULL = no affine)
 *   The reference has no eps: pass eps = 0 for identical results.
 * x_dtype, y_dtype in {BF16, E4M3}; w fp32 [dim] or NULL; rstd fp32 [rows] or NULL.
 * dim % 8 == 0, dim <= 32768; rows contiguous.
 */
int q8_rmsnorm(const void* x, int x_dtype, const float* w, void* y, int y_dtype, float* rstd,
               int64_t rows, int dim, float eps, q8_stream_t stream);

/*
 * Rotary embedding with full-shape tables.
 * Replaces ops._C.rope  (csrc/ops/rope.cpp:96-146, kernel csrc/ops/rope_cuda.cu:68-106).
 *   y[r,2i]   = x[r,2i]  *cos[r,2i]   - x[r,2i+1]*sin[r,2i]
 *   y[r,2i+1] = x[r,2i+1]*cos[r,2i+1] + x[r,2i]  *sin[r,2i+1]
 * x_dtype, y_dtype in {BF16, E4M3}; cos, sin fp32 [rows, dim]; dim % 8 == 0; rows contiguous.
 */
int q8_rope(const void* x, int x_dtype, const float* cos_t, const float* sin_t, void* y, int y_dtype,
            int64_t rows, int dim, q8_stream_t stream);

/*
 * out = x * (y + scale_add) + z, the AdaLN modulation.
 * Replaces ops._C.fma_8bit  (csrc/ops/fma.cpp:63-112, kernel csrc/ops/fma_cuda.cu:61-98).
 * x, out [rows, dim]; y and z are broadcast over groups of consecutive rows: row r reads row r / y_rows_every of y
 * (the reference: one row of y per batch entry or per token, fma.cpp:85-86). The product and the sum round once
 * (a fused multiply-add, which is what the reference's expression compiles to).
 * x_dtype, out_dtype in {E4M3 (the reference), BF16}; y_dtype, z_dtype in {F32, BF16, E4M3} (the reference has the
 * pairs F32/F32, F32/E4M3, BF16/BF16); dim % 8 == 0 (the reference: 2048 or 8192 only, fma_cuda.cu:117-122).
 */
int q8_fma(const void* x, int x_dtype, const void* y, int y_dtype, const void* z, int z_dtype, void* out,
           int out_dtype, int64_t rows, int dim, int64_t y_rows_every, int64_t z_rows_every, float scale_add,
           q8_stream_t stream);

/*
 * The modulation rows of an AdaLN block: rows[p, r, :] = bf16(table[p, :] + timestep[r, p*dim .. (p+1)*dim)).
 * Replaces the torch expression `scale_shift_table[None, None] + timestep.reshape(B, T, P, dim)` and its unbind
 * (q8_kernels/blocks/ltx_transformer_block.py:30-36) followed by the casts of its six slices: table fp32 [params, dim],
 * timestep fp32 [tokens, params * dim] (tokens = B * T), rows bf16 [params, tokens, dim] - each parameter's rows
 * contiguous, the layout q8_norm_mod_fht_quant_rows and q8_gemm_gated_residual read. The sum is formed in fp32 and
 * rounded once. dim % 8 == 0, 1 <= params <= 64; all pointers 16-byte aligned.
 */
int q8_adaln_rows(const float* table, const float* timestep, void* rows, int params, int64_t tokens, int dim,
                  q8_stream_t stream);

/*
 * tanh-GELU and the operators of the backward pass (the LoRA fine-tuning path of the reference).
 *   q8_gelu             replaces ops._C.gelu_forward      (csrc/ops/gelu_act.cpp, kernel gelu_forward_cuda.cu:12-16,73-100)
 *   q8_gelu_backward    replaces ops._C.gelu_backward     (kernel gelu_backward_cuda.cu:67-105): out = grad * dGELU(x)
 *   q8_rope_backward    replaces ops._C.rope_backward     (csrc/ops/rope.cpp:150-200, kernel rope_backward_cuda.cu:68-118):
 *                       out[2i] = g[2i] cos[2i] + g[2i+1] sin[2i+1]; out[2i+1] = -g[2i] sin[2i] + g[2i+1] cos[2i+1]
 *   q8_rmsnorm_backward replaces ops._C.rms_norm_backward (kernel rms_norm_backward_cuda.cu:101-206):
 *                       out = rstd / dim * (dim * g * w - y / w * sum_j g_j y_j), y the forward output, w NULL = 1
 * All element dtypes in {BF16, E4M3} independently (the reference ties grad's dtype to out's); n, dim % 8 == 0.
 */
int q8_gelu(const void* x, int x_dtype, void* out, int out_dtype, int64_t n, q8_stream_t stream);
int q8_gelu_backward(const void* x, int x_dtype, const void* grad, int grad_dtype, void* out, int out_dtype,
                     int64_t n, q8_stream_t stream);
int q8_rope_backward(const void* grad, int grad_dtype, const float* cos_t, const float* sin_t, void* out,
                     int out_dtype, int64_t rows, int dim, q8_stream_t stream);
int q8_rmsnorm_backward(const void* y, int y_dtype, const float* rstd, const void* grad, int grad_dtype,
                        const float* w, void* out, int out_dtype, int64_t rows, int dim, q8_stream_t stream);

/*
 * Fused row kernels: launch sequences of the reference with the 16-bit tensor between two kernels kept in
 * registers. Each intermediate value is rounded to `mid_dtype` exactly where the unfused sequence stores it
 * (mid_dtype = Q8_BF16 gives the same bits as the separate calls; Q8_F32 skips that rounding; Q8_E4M3, for an
 * E4M3 input, is the e4m3 intermediate that hadamard_transform's default output type produces).
 *
 * q8_fht_quant_rows: codes, scales = quant(FHT(x) * fht_scale). The prologue of the int8 linear layer,
 *   hadamard_transform followed by quantize (q8_kernels/functional/linear.py:30-31), = q8_fht then q8_quant_rows.
 * q8_rmsnorm_quant_rows: codes, scales = quant(rmsnorm(x, w)); rstd (nullable) as q8_rmsnorm. The norm in front
 *   of an 8-bit projection (q8_kernels/modules/attention.py:67-77) = q8_rmsnorm then q8_quant_rows.
 * x_dtype in {BF16, E4M3}; code_dtype in {I8, E4M3}; flags as q8_quant_rows; rows contiguous; dim as the row kernels.
 */
int q8_fht_quant_rows(const void* x, int x_dtype, void* codes, int code_dtype, float* scales, int64_t rows,
                      int dim, float fht_scale, int mid_dtype, int flags, q8_stream_t stream);
int q8_rmsnorm_quant_rows(const void* x, int x_dtype, const float* w, void* codes, int code_dtype, float* scales,
                          float* rstd, int64_t rows, int dim, float eps, int mid_dtype, int flags,
                          q8_stream_t stream);
/*
 * The whole prologue of a projection behind an AdaLN-modulated norm, bf16 x [rows, dim] -> codes, scales:
 *   [apply_norm: rmsnorm(x) * norm_w (norm_w NULL = 1), no epsilon] -> [x * (mod_scale + scale_add) + mod_shift, one
 *   fused multiply-add as q8_fma; mod_scale / mod_shift [rows / rows_per_mod, dim] in mod_dtype (BF16 or F32), both
 *   NULL = none] -> [apply_fht: FHT * fht_scale] -> quantizer. Every step rounds to bfloat16 where the separate calls
 *   (q8_rmsnorm, q8_fma, q8_fht, q8_quant_rows: q8_kernels/blocks/ltx_transformer_block.py:38-40,
 *   q8_kernels/functional/linear.py:30-31) store a bfloat16 tensor, so the codes and scales are the same bits.
 */
int q8_norm_mod_fht_quant_rows(const void* x, const float* norm_w, int apply_norm, const void* mod_scale,
                               const void* mod_shift, int mod_dtype, int64_t rows_per_mod, float scale_add,
                               int apply_fht, float fht_scale, void* codes, int code_dtype, float* scales,
                               int64_t rows, int dim, int flags, q8_stream_t stream);

/*
 * Attention prologues: from token-major 16-bit projections [B, S, H*D] (row stride in elements, so a slice of a
 * fused QKV projection can be passed without a copy) to the e4m3 operands of q8_attn_fwd.
 * Replaces the torch glue of flash_attn_func (q8_kernels/functional/flash_attention.py:38-55: transpose, pad,
 * cast, hadamard_transform) and the RoPE in front of it (q8_kernels/modules/attention.py:84-87).
 *
 * q8_attn_prep_qk: per token: [RMSNorm over the H*D row with fp32 weights norm_w [H*D], no epsilon (the qk-norm of
 *   q8_kernels/modules/attention.py:67-77), NULL = none] -> per head: [RoPE with tables cos, sin fp32 [B*S, H*D],
 *   both NULL = none; Q8_PREP_PAIR_TABLES / Q8_PREP_SHARED_TABLES in flags: the same values stored once, [B*S or S,
 *   H*D or H*D/2], same results] ->
 *   [D-point FHT * scale with Q8_PREP_FHT in flags] -> e4m3 codes [B, H, S, D]. scales == NULL: direct c10 cast (the
 *   reference's cast); otherwise one absmax scale per (token, head) to scales [B, H, S].
 *   D in {64, 128}; H * D in {64, 128, 256} or a multiple of 512 up to 4096.
 * q8_attn_prep_qk_pair: the same for Q and K of a self-attention in one pass (same S, same tables, read once).
 * q8_attn_prep_qkv: q8_attn_prep_qk_pair, and the V projection xv of the same tokens is cast in the same pass to
 *   e4m3 codes [B, H, S, D] (token-major per head: the Q8_V_SD operand of q8_attn_fwd, no transposed copy);
 *   scales_v [B, H, S] together with scales_q / scales_k, or all three NULL for the direct c10 cast.
 * q8_attn_prep_kv: q8_attn_prep_qk on the K projection xk, and the V projection xv of the same tokens is cast in the
 *   same pass to token-major e4m3 codes like in q8_attn_prep_qkv: the keys and values of a cross-attention (whose
 *   queries are other tokens) in one launch.
 * q8_attn_prep_v: e4m3 codes [B, H, D, S_pad] (Q8_V_DS), columns S..S_pad-1 zero, S_pad % 16 == 0;
 *   scales as above. D == 64.
 */
int q8_attn_prep_qk(const void* x, int64_t x_row_stride, const float* norm_w, const float* cos_t, const float* sin_t,
                    void* codes, float* scales, int B, int S, int H, int D, int flags, float scale, int mid_dtype,
                    q8_stream_t stream);
int q8_attn_prep_qk_pair(const void* xq, int64_t xq_row_stride, const void* xk, int64_t xk_row_stride,
                         const float* norm_wq, const float* norm_wk, const float* cos_t, const float* sin_t,
                         void* codes_q, float* scales_q, void* codes_k, float* scales_k, int B, int S, int H, int D,
                         int flags, float scale, int mid_dtype, q8_stream_t stream);
int q8_attn_prep_qkv(const void* xq, int64_t xq_row_stride, const void* xk, int64_t xk_row_stride, const void* xv,
                     int64_t xv_row_stride, const float* norm_wq, const float* norm_wk, const float* cos_t,
                     const float* sin_t, void* codes_q, float* scales_q, void* codes_k, float* scales_k, void* codes_v,
                     float* scales_v, int B, int S, int H, int D, int flags, float scale, int mid_dtype,
                     q8_stream_t stream);
int q8_attn_prep_kv(const void* xk, int64_t xk_row_stride, const void* xv, int64_t xv_row_stride, const float* norm_wk,
                    const float* cos_t, const float* sin_t, void* codes_k, float* scales_k, void* codes_v, float* scales_v,
                    int B, int S, int H, int D, int flags, float scale, int mid_dtype, q8_stream_t stream);
int q8_attn_prep_v(const void* x, int64_t x_row_stride, void* codes, float* scales, int B, int S, int H, int D,
                   int S_pad, q8_stream_t stream);

/*
 * 8-bit GEMM with fused dequantisation, bias and tanh-GELU.
 * Replaces gemm._C.q8_mm / q8_mm_bias / fp8_mm / fp8_mm_bias
 * (csrc/gemm/q8_gemm_api.cpp:40-291; kernels csrc/gemm/{q8,fp8}_matmul{,_bias}.cu).
 *   acc[z,m,n] = sum_k A[za,m,k] * B[zb,n,k]            (int32 exact for I8, fp32 for E4M3)
 *   v = float(acc) * (sa[za*M+m] * sb[zb*N+n]) (+ bias[n]);  if fuse_gelu: v = gelu_tanh(v)
 *   C[z,m,n] = bf16(v)  or  e4m3(v) saturating to +-448
 * A: [batch_a, M, K], B: [batch_b, N, K] contiguous, both K-major; batch_a == batch_b or either == 1
 * (the operand with batch 1 is broadcast); C: [max(batch_a,batch_b), M, N] contiguous.
 * in_dtype in {I8, E4M3}; out_dtype in {BF16, E4M3}; bias fp32 [N] or NULL.
 * K % 16 == 0 and A, B 16-byte aligned; M, N arbitrary (> 0); N % 8 == 0 for BF16 output rows to stay
 * 16-byte aligned, N % 16 == 0 for E4M3 output.
 * M == 0 or N == 0 (no tokens, no output elements) returns Q8_OK without touching any pointer, also in
 * q8_gemm_residual and q8_gemm_i32; negative sizes and K <= 0 are errors.
 */
int q8_gemm(const void* A, const void* B, const float* bias, const float* sa, const float* sb, void* C,
            int batch_a, int batch_b, int M, int N, int K, int in_dtype, int out_dtype, int fuse_gelu,
            q8_stream_t stream);

/*
 * q8_gemm with bf16 output and a residual connection: C = bf16(bf16(epi(...)) + residual), residual bf16 [batch, M, N].
 * Fuses the element-wise addition the reference's blocks run after a projection
 * (q8_kernels/blocks/ltx_transformer_block.py:41-51) into the epilogue; the two roundings are those of the separate
 * addition. Runs on the persistent kernel only: N % 8 == 0, K % 128 == 0, K > 256 (Q8_ERR_SHAPE otherwise).
 */
int q8_gemm_residual(const void* A, const void* B, const float* bias, const float* sa, const float* sb,
                     const void* residual, void* C, int batch_a, int batch_b, int M, int N, int K, int in_dtype,
                     int fuse_gelu, q8_stream_t stream);

/*
 * q8_gemm_residual (one batch) with a gate: C = bf16(fma(bf16(epi(...)), gate[m / rows_per_gate, n], residual[m, n])),
 * gate bf16 [ceil(M / rows_per_gate), N]: the gated residual of the AdaLN block,
 * `attn_output * gate_msa + hidden_states` and `ff_output * gate_mlp + hidden_states`
 * (q8_kernels/blocks/ltx_transformer_block.py:44,57), in the epilogue of the projection that produces the first factor.
 * The bits are those of q8_gemm (bf16 output) followed by q8_fma with bf16 operands. rows_per_gate (tokens per batch
 * element) must be a multiple of 768, so that a 192- or 256-row tile has one gate row; other conditions as q8_gemm_residual.
 */
int q8_gemm_gated_residual(const void* A, const void* B, const float* bias, const float* sa, const float* sb,
                           const void* residual, const void* gate, int64_t rows_per_gate, void* C, int M, int N, int K,
                           int in_dtype, int fuse_gelu, q8_stream_t stream);

/*
 * q8_gemm for a fused QKV projection whose V part feeds the attention kernel directly: columns n < v_col0 (Q and K) are
 * written as bf16 to C [M, v_col0]; columns n >= v_col0 (V, heads of 64) are rounded to bf16 like the others, cast to e4m3
 * (the c10 cast of q8_kernels/functional/flash_attention.py:38-45) and written token-major per head to v_codes
 * [M / tokens, (N - v_col0) / 64, tokens, 64], the Q8_V_SD operand of q8_attn_fwd: the V output of q8_attn_prep_qkv without
 * the bf16 round trip through memory (the fourth fusion the reference's launch boundaries allow around the attention,
 * q8_kernels/modules/attention.py:67-105). M rows = batch elements of `tokens` tokens each. Runs on the persistent kernel
 * only: N % 8 == 0, K % 128 == 0, K > 256; v_col0 a multiple of 256, N - v_col0 a multiple of 64 (Q8_ERR_SHAPE otherwise).
 * v_col0 == 0 is a V projection of its own (a separate to_v layer): every column goes to v_codes, C may be NULL.
 * v_fht_scale != 0: the bf16-rounded results of every head of 64 go through the 64-point Hadamard transform times
 * v_fht_scale before the cast, hadamard_transform(x, scale, out_type=e4m3) of q8_kernels/functional/flash_attention.py:47-51:
 * with v_col0 == 0 the Q (or K) operand of an attention with apply_qk_hadamard straight from its projection, the bits of
 * q8_gemm followed by q8_attn_prep_qk without tables. 0 = the plain cast. Finite and not negative.
 */
int q8_gemm_qkv(const void* A, const void* B, const float* bias, const float* sa, const float* sb, void* C, void* v_codes,
                int M, int N, int K, int v_col0, int tokens, float v_fht_scale, int in_dtype, q8_stream_t stream);

/*
 * Kernel override for q8_gemm / q8_gemm_i32: 0 = choose by problem size (default), 1 = pipelined 256x256 tiles with
 * one tile per workgroup, 2 = 128x128 tiles, 3 = 64x64 tiles, 4 = persistent pipelined 256x256 tiles (bf16 or e4m3 output, N % 8 == 0,
 * K % 128 == 0, K > 256; other calls fall back to 1); 43 / 44 / 40 pin the persistent kernel's tile to 192 / 256 rows /
 * back to automatic. It holds for the calling thread only; meant for tests and tuning, it has no counterpart in the
 * reference (whose tile is fixed at 128x128x64, csrc/gemm/fp8_matmul_bias.cu:426-429).
 */
int q8_gemm_set_config(int cfg);

/*
 * Which kernel the most recent q8_gemm / q8_gemm_residual / q8_gemm_i32 call of the calling thread launched
 * (0 before the first call): one of the Q8_GEMM_KERNEL_* values, Q8_GEMM_KERNEL_RESIDUAL or-ed in when the residual
 * was added in the epilogue. For tests, so that a test of a pinned kernel can tell that the call did not fall back
 * to another one; no counterpart in the reference.
 */
enum {
    Q8_GEMM_KERNEL_PIPE256 = 1,    /* pipelined 256x256 tiles, one tile per workgroup */
    Q8_GEMM_KERNEL_TILE128 = 2,    /* 128x128 tiles                                    */
    Q8_GEMM_KERNEL_TILE64 = 3,     /* 64x64 tiles (small problems)                     */
    Q8_GEMM_KERNEL_PERSIST256 = 4, /* persistent, 256-row tiles                        */
    Q8_GEMM_KERNEL_PERSIST192 = 5, /* persistent, 192-row tiles                        */
    Q8_GEMM_KERNEL_RESIDUAL = 16
};
int q8_gemm_last_kernel(void);

/*
 * Raw int32 accumulators of the int8 GEMM, C[m,n] = sum_k A[m,k]*B[n,k], for bit-exact checks.
 * Same mainloop as q8_gemm with in_dtype = Q8_I8 (csrc/gemm/q8_matmul.cu:109-, accumulators
 * before the float conversion at q8_matmul_bias.cu:315-320).
 */
int q8_gemm_i32(const int8_t* A, const int8_t* B, int32_t* C, int M, int N, int K, q8_stream_t stream);

/*
 * FP8 FlashAttention-2 forward, head dim 64, non-causal, optional per-batch valid KV length.
 * Replaces flash_attention._C.flash_attention
 * (csrc/flash_attention/flash_attention.cpp:18-48; kernels flash_attention_cuda.cu:254-534 and
 * flash_attention_cuda_mask.cu:254-535).
 *   s[i,j] = (q_i . k_j) * softmax_scale * (sq[i]*sk[j] if given);  keys j >= kv_len[b] (or >= N) masked
 *   p[i,j] = 2^8 exp(s[i,j] - max_j s[i,j])  (without the 2^8 under P_UNIT_RANGE);
 *   l_i = sum_j p[i,j]  (fp32, unrounded unless SUM_ROUNDED_P)
 *   o_i = (sum_j e4m3_sat(p[i,j]) * v_j) / l_i;   rows with l_i == 0 or NaN divide by 1
 *   with sv: o_i = svmax * (sum_j e4m3_sat(p[i,j] * sv[j] / svmax) * v_j) / l_i,  svmax = max_{j valid} sv[j]
 *   O = bf16(o) or e4m3_sat(o)
 * q: [B,H,M,64] e4m3; k: [B,H,N,64] e4m3; v: e4m3 in v_layout; o: [B,H,M,64] of out_dtype.
 * kv_len: int32 [B] or NULL; sq: fp32 [B,H,M], sk, sv: fp32 [B,H,N] per-token dequantisation scales
 * or NULL (all three given or none). D must be 64. softmax_scale is the plain (natural-log) scale.
 * B == 0 or M == 0 (no queries) returns Q8_OK without touching any pointer; N has to be positive.
 * q, k, v and o 16-byte aligned (Q8_ERR_ALIGN otherwise). N <= 128 runs a kernel that holds K and V of a (batch, head)
 * in LDS and rounds P against the final row maximum; longer sequences round it against the running maximum.
 */
int q8_attn_fwd(const void* q, const void* k, const void* v, void* o, const int32_t* kv_len,
                const float* sq, const float* sk, const float* sv,
                int B, int H, int M, int N, int D, int v_layout, int64_t v_row_stride,
                float softmax_scale, int out_dtype, int flags, q8_stream_t stream);

/*
 * Workgroup-shape override for q8_attn_fwd: 0 = the default (N <= 128: the short-sequence kernel, K and V of a (batch, head)
 * resident in LDS and P rounded against the final row maximum; longer sequences: the general kernel with 8 waves x 32 queries
 * for unit scales, 4 waves x 32 queries for per-token scales). 1 .. 4 select the general kernel for every N, in the shape
 * 1 = 4 waves x 64 queries (Q8_V_DS only), 2 = 4 waves x 32 queries, 3 = the default shape of the mode, 4 = 8 waves x 32
 * queries. All shapes of the general kernel give the same bits. It holds for the calling thread only; meant for tests and
 * tuning, no counterpart in the reference (whose workgroup is fixed at 4 warps x 16 queries,
 * csrc/flash_attention/flash_attention_cuda.cu:279-287).
 */
int q8_attn_set_config(int cfg);

#ifdef __cplusplus
}
#endif
#endif /* Q8_HIP_H */
