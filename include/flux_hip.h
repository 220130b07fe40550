/*
 * flux_hip.h — C ABI of libfluxhip.so: the Flux transformer-block kernel set for MI355X (gfx950).
 *
 * Every entry point replaces one host launcher (and the Triton kernel behind it) of the reference
 * package `triton_kernels`; the citation on each declaration names the reference interface it
 * stands in for (paths relative to the reference repository root).
 *
 * Conventions
 *   - All data pointers are device pointers. The library never allocates, frees or keeps them,
 *     and no kernel uses device memory beyond the buffers its caller passes.
 *   - Strides are in ELEMENTS, not bytes. The innermost dimension is always contiguous.
 *   - `stream` is a hipStream_t passed as void*; work is enqueued on it and never synchronised.
 *   - Return value: 0 = launched; negative = argument rejected before any launch (FLUX_E_*);
 *     positive = hipError_t reported by the launch. flux_last_error() gives the text for the
 *     calling thread's most recent non-zero return.
 *   - dtype codes: FLUX_BF16 (bfloat16 storage, fp32 arithmetic) and FLUX_F32.
 */
#ifndef FLUX_HIP_H
#define FLUX_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FLUX_ABI_VERSION 4

enum flux_dtype { FLUX_BF16 = 0, FLUX_F32 = 1 };

enum flux_status {
    FLUX_OK = 0,
    FLUX_E_NULL = -1,      /* a required pointer is null */
    FLUX_E_SHAPE = -2,     /* a size is negative, zero where it may not be, or inconsistent */
    FLUX_E_DTYPE = -3,     /* dtype code unknown or not supported by this entry point */
    FLUX_E_ALIGN = -4,     /* pointer or stride breaks the 16-byte vector-access rule */
    FLUX_E_TOO_WIDE = -5,  /* row longer than 65536 elements */
    FLUX_E_UNSUPPORTED = -6
};

enum flux_activation { FLUX_ACT_NONE = 0, FLUX_ACT_GELU_TANH = 1, FLUX_ACT_SILU = 2 };

/* Largest row a row-wise kernel accepts; mirrors MAX_FUSED_SIZE in kernels/utils.py:6-11. */
#define FLUX_MAX_ROW 65536

int flux_abi_version(void);
const char* flux_last_error(void);

/* ---------------------------------------------------------------------------------------------
 * RMSNorm forward.   y[r,:] = x[r,:] * rsqrt(mean(x[r,:]^2) + eps) * scale
 * Replaces _rms_norm.forward / _rms_norm_fwd  (kernels/normalization.py:142-169, 81-106).
 * x is viewed as [d0,d1,d2,n] with element strides (s0,s1,s2,1); y is contiguous [d0*d1*d2, n].
 * rstd (nullable) receives the fp32 reciprocal RMS per row, in y's row order.
 * For FLUX_BF16 the intermediate x*rstd is rounded to bf16 before the multiply by scale, the
 * order of functional/normalization.py:21-25. scale_dtype may be FLUX_F32 while x is FLUX_BF16.
 * Any row count is handled (the reference drops rows % 8).
 * ------------------------------------------------------------------------------------------- */
int flux_rms_norm(const void* x, const void* scale, void* y, float* rstd,
                  int64_t d0, int64_t d1, int64_t d2, int32_t n,
                  int64_t s0, int64_t s1, int64_t s2,
                  int32_t x_dtype, int32_t scale_dtype, float eps, void* stream);

/* RMSNorm backward. Replaces _rms_norm.backward / _rms_norm_bwd (kernels/normalization.py:110-139,
 * 171-190). x, dy, dx contiguous [rows, n]; rstd from the forward; dscale[n] is fp32 and is
 * accumulated with atomics, so the caller zero-fills it first. */
int flux_rms_norm_bwd(const void* dy, const void* x, const void* scale, const float* rstd,
                      void* dx, float* dscale, int64_t rows, int32_t n,
                      int32_t x_dtype, int32_t scale_dtype, void* stream);

/* ---------------------------------------------------------------------------------------------
 * LayerNorm (no affine) + adaLN modulation.   y = (1 + scale[b]) * LN(x[b,l,:]) + shift[b]
 * Replaces layer_norm_modulation / _layer_norm_modulation_fwd (kernels/normalization.py:47-77,
 * 9-44). x, y contiguous [batch, seq, n]; scale/shift are [batch, n] with row stride
 * mod_batch_stride (so chunks of a wider modulation vector can be passed without a copy).
 * ------------------------------------------------------------------------------------------- */
int flux_layer_norm_modulation(const void* x, const void* scale, const void* shift, void* y,
                               int64_t batch, int64_t seq, int32_t n, int64_t mod_batch_stride,
                               int32_t dtype, float eps, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Q/K/V preparation: the fused gather behind RoPE apply and QKV split/concat.
 *
 * For t in {q,k,v} the output t_out is contiguous [B,H,Lt+Li,D]. Row (b,h,s) is taken from the
 * "txt" source when s < Lt and from the "img" source (at s-Lt) otherwise; a source is a
 * [B,H,L*,D] view given by its base pointer and element strides (sb,sh,sl). For q and k the row
 * is optionally RMS-normalised over D with the given scale vectors (txt and img sources may have
 * different scales) and optionally rotated by the 2x2 matrices pe[s, D/2, 2, 2] (fp32, shared by
 * every head; per batch element when pe_batch_stride != 0). v is copied bit-exactly. Any of the three tensors can be left
 * out by passing null output AND null sources for it; Lt may be 0 (then txt pointers are ignored).
 *
 * Replaces, depending on the flags:
 *   apply_rope / _rope_fwd                    (kernels/positional_embedding.py:55-82, 10-52)
 *   torch.cat((txt_*, img_*), dim=2)          (modules/blocks.py:158-160)
 *   triton_qkv_concat                         (ops/qkv_concat.py:5-60)
 *   QKNorm + apply_rope + the .contiguous() copies between them in SingleStreamBlock.forward
 *                                             (modules/blocks.py:115-119, modules/normalization.py:23-26)
 * ------------------------------------------------------------------------------------------- */
typedef struct flux_src4 {
    const void* ptr;   /* null = absent */
    int64_t sb, sh, sl; /* element strides of batch, head, position; last dim contiguous */
} flux_src4;

typedef struct flux_qkv_prep_args {
    flux_src4 q_txt, k_txt, v_txt;
    flux_src4 q_img, k_img, v_img;
    void* q_out; void* k_out; void* v_out;   /* contiguous [B,H,Lt+Li,D] */
    const void* q_scale_txt; const void* k_scale_txt;   /* [D], null = no RMS norm */
    const void* q_scale_img; const void* k_scale_img;
    const float* pe;                                     /* [Lt+Li, D/2, 2, 2], null = no rotation */
    int64_t pe_batch_stride;                             /* floats between the tables of two batch
                                                            elements; 0 = one table for all */
    int64_t B, H, Lt, Li;
    int32_t D;
    int32_t dtype;        /* of q,k,v and outputs */
    int32_t scale_dtype;  /* of the four scale vectors */
    float eps;
} flux_qkv_prep_args;

int flux_qkv_prep(const flux_qkv_prep_args* args, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Linear: Y = act(A * W^T + bias), bf16 operands, fp32 accumulation on MFMA.
 * Replaces linear / _linear_fwd / gelu (kernels/linear.py:104-151, 31-101, 22-28) and the raw
 * triton_linear (ops/linear.py:5-71).
 * A is [M,K] with row stride lda, W is [N,K] (nn.Linear layout) with row stride ldw.
 * in_act == FLUX_ACT_SILU applies x * sigmoid(x) (fp32, rounded to bf16, as flux_silu does) to A on
 * the way in: lin(silu(vec)) of Modulation (modules/blocks.py:62-67) as one launch. Only for
 * M <= 8 (the row-vector path); larger M returns FLUX_E_UNSUPPORTED.
 *
 * Epilogue, applied in this order on the fp32 accumulator:
 *   + bias[n] (nullable)
 *   tanh-GELU for columns n >= act_begin when act == FLUX_ACT_GELU_TANH, evaluated in fp32 on the
 *       un-rounded sum (kernels/linear.py:92-95 rounds to bf16 first; one rounding keeps the result
 *       within half a bf16 ulp of the fp32 value)
 *   -> rounded to bf16
 *   if gate != null:  y = resid[m,n] + gate[(m / rows_per_batch), n] * y   (each step rounded to
 *       bf16), the gated residual of modules/blocks.py:123
 * Output columns [0, split_n) go to Y (row stride ldy); columns [split_n, N) go to Y2 at column
 * (n - split_n + y2_col0) with row stride ldy2. split_n == N (or Y2 == null) means one output.
 * ------------------------------------------------------------------------------------------- */
/* Optional: QK RMSNorm + RoPE applied to the leading columns of a qkv projection on their way out.
 * Replaces, for q and k, the chain of modules/blocks.py:115-119: the "B L (K H D) -> K B H L D"
 * rearrange, QKNorm (modules/normalization.py:17-26 over kernels/normalization.py:142-169) and
 * apply_rope (kernels/positional_embedding.py:55-82).
 * Output columns [0, heads*128) are the q heads, [heads*128, 2*heads*128) the k heads, 128 columns
 * each. For those columns y = A W^T + bias is rounded to bf16, normalised over the head
 * (x * rsqrt(mean x^2 + eps) rounded, times scale rounded), rotated with the 2x2 matrices of its
 * position (pe[pos][c/2] = [[f00,f01],[f10,f11]] for the column pair c, c+1) and stored at
 * q_out / k_out [b, head, pos0 + l, :], where row m of the product is (b, l) = (m / seq_len,
 * m % seq_len). They are not written to Y. Any row count M = B * seq_len is taken: tiles that run
 * past the last row, or that hold the last rows of one batch element and the first of the next,
 * take a checked form of the epilogue. Requirements (else FLUX_E_UNSUPPORTED): seq_len >= 256,
 * N a multiple of 256, 16-byte aligned pointers, no gate, act_begin and split_n at or past
 * 2*heads*128, K a multiple of 8. */
typedef struct flux_linear_qk_fusion {
    void* q_out; void* k_out;                  /* [B, heads, out_len, 128] bf16, contiguous */
    const void* q_scale; const void* k_scale;  /* [128] bf16 */
    const float* pe;                           /* [out_len, 64, 2, 2] fp32 */
    int64_t pe_batch_stride;                   /* floats between the tables of two batch elements; 0 = one table */
    int64_t heads, seq_len, out_len, pos0;
    float eps;
} flux_linear_qk_fusion;

typedef struct flux_linear_args {
    const void* A; const void* W; const void* bias;
    void* Y; void* Y2;
    const void* resid; const void* gate;
    int64_t M, N, K;
    int64_t lda, ldw, ldy, ldy2;
    int64_t split_n, y2_col0;
    int64_t ldresid, gate_batch_stride, rows_per_batch;
    int32_t act; int32_t in_act; int64_t act_begin;
    const flux_linear_qk_fusion* qk;           /* null = off */
    int64_t flags;                             /* FLUX_LINEAR_* bits, 0 = none */
} flux_linear_args;

/* flags: the launch will run beside work of another stream (the txt chain beside the img chain of
 * the double-stream block). The library then keeps the tile shape whose last round leaves CUs free
 * for that work instead of the one that fills every round of the 256 CUs exactly, and gives a
 * small problem few, larger workgroups instead of one or two on every CU; both other choices are
 * the faster ones only when the launch has the GPU to itself. The result is the same bits either
 * way. */
#define FLUX_LINEAR_SHARED_GPU 1

int flux_linear_bf16(const flux_linear_args* args, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Non-causal attention forward: O = softmax(Q K^T * sm_scale) V, bf16 in/out, fp32 online softmax.
 * Replaces scaled_dot_product_attention / _attn_fwd (kernels/attention.py:173-221, 70-170).
 * q,k,v,o are [B,H,L,D] views with element strides (sb,sh,sl,1) each; D in {16,32,64,128,256}
 * (the set kernels/attention.py:184 accepts); any L (ragged tails are masked, which the reference
 * does not do); any finite sm_scale, negative and zero included. lse (nullable) receives
 * m + log2(l) per row as fp32 [B,H,L], the quantity kernels/attention.py:166-169 stores.
 * For D = 64 and 128 the kernels fold sm_scale * log2(e) into Q and round the result to bf16 once
 * where kernels/attention.py:29-30 scales the fp32 scores. Every term of a score then carries a
 * relative error of at most 2^-8, so row i's base-2 scores, and with them lse, move by at most
 * 2^-8 * sm_scale * log2(e) * max_j sum_d |q_id k_jd|: a few 1e-3 for unit-variance inputs (o within
 * 4e-3 of the fp32 result at L = 4608), growing in proportion to |q| |k| (q thirty times larger:
 * lse up to 0.37 away, nearly one-hot outputs up to 0.33 at |v| ~ 4, 4e-3 on average). D = 16, 32
 * and 256 run a plain, unpipelined kernel that scales the fp32 scores.
 * ------------------------------------------------------------------------------------------- */
typedef struct flux_attn_args {
    flux_src4 q, k, v;
    void* o; int64_t o_sb, o_sh, o_sl;
    float* lse;
    int64_t B, H, L;
    int32_t D;
    float sm_scale;
} flux_attn_args;

int flux_attention_fwd_bf16(const flux_attn_args* args, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Small element-wise kernels (the reference's inductor-derived `ops`, plus nn.GELU on a view).
 * ------------------------------------------------------------------------------------------- */

/* y = x * sigmoid(x), fp32 math. Replaces triton_silu (ops/silu.py:5-13). */
int flux_silu(const void* x, void* y, int64_t numel, int32_t dtype, void* stream);

/* y[r,:] = gelu_tanh(x[r,:]) for a [rows, n] view with row strides ldx / ldy.
 * Replaces nn.GELU(approximate="tanh") on the strided mlp half (modules/blocks.py:107,122). */
int flux_gelu_tanh(const void* x, void* y, int64_t rows, int64_t n, int64_t ldx, int64_t ldy,
                   int32_t dtype, void* stream);

/* out[b,l,:] = (1 + mod[b, (chunk+1)*hid + :]) * x[b,l,:] + mod[b, chunk*hid + :]
 * with chunk = 0 (mod1) or 3 (mod2); mod is the [B, mod_row_stride] Modulation output.
 * Replaces triton_modulation_scale_shift (ops/modulation.py:5-27). */
int flux_modulation_scale_shift(const void* x, const void* mod, void* out,
                                int64_t batch, int64_t seq, int64_t hid, int64_t mod_row_stride,
                                int32_t is_mod1, int32_t dtype, void* stream);

/* out[b,l,:] = x[b,l,:] + gate[b,:] * y[b,l,:], gate row stride gate_batch_stride.
 * With gate = mod + 2*hid this is triton_modulation_gate_proj (ops/modulation.py:29-44); it is
 * also the gated residual x + mod.gate * output of modules/blocks.py:123,166-171.
 * round_product != 0 rounds gate*y to the storage dtype before the add (what two torch ops do). */
int flux_gate_residual(const void* x, const void* gate, const void* y, void* out,
                       int64_t batch, int64_t seq, int64_t hid, int64_t gate_batch_stride,
                       int32_t round_product, int32_t dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FLUX_HIP_H */
