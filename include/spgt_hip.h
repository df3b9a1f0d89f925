/* C ABI of libspgt_hip.so: the gfx950 (MI355X) kernels behind SpGT's operator API.
 *
 * Conventions
 *   - every pointer is a device pointer to fp32 data unless stated otherwise;
 *     complex64 tensors are passed as float pairs (re, im);
 *   - the caller owns all memory: outputs and workspaces are passed in, the
 *     library allocates nothing and keeps no state between calls;
 *   - kernels are enqueued on `stream` (0 = the null stream) of the current
 *     device and the call returns without synchronising;
 *   - the return value is SPGT_OK or a negative SPGT_ERR_* code, in which case
 *     nothing was launched and spgt_last_error() describes the problem;
 *   - `*_workspace_bytes` functions return the scratch size the matching call
 *     needs for the same shape arguments (0 for invalid shapes).
 *
 * Each entry point names the interface of the reference (Bloonow/SpGT) that a
 * binding would replace with it.
 */
#ifndef SPGT_HIP_H
#define SPGT_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ihipStream_t* spgt_stream_t; /* == hipStream_t */

enum {
    SPGT_OK = 0,
    SPGT_ERR_INVALID_ARGUMENT = -1,
    SPGT_ERR_WORKSPACE = -2,
    SPGT_ERR_LAUNCH = -3
};

/* Operand orders of the reference's batched GEMMs (extension/utils/gemm_utils.cu:3-12):
 * letter k of the name is the storage order (R row-major, C column-major) of A, B, C. */
enum {
    SPGT_ORDER_RRR = 0, SPGT_ORDER_RRC = 1, SPGT_ORDER_RCR = 2, SPGT_ORDER_RCC = 3,
    SPGT_ORDER_CRR = 4, SPGT_ORDER_CRC = 5, SPGT_ORDER_CCR = 6, SPGT_ORDER_CCC = 7
};

/* Library version as major*10000 + minor*100 + patch. */
int spgt_version(void);

/* Message of the last failed call on the calling thread ("" if none). */
const char* spgt_last_error(void);

/* ---- Galerkin attention ------------------------------------------------ */

/* Replaces multihead_projection_with_position_rrc_forward
 * (extension/bind/galerkin_attention.cu:9-24; same argument order, output passed in).
 *   input [batch, seqlen, dim_hidden], weight [dim_hidden, dim_hidden] used as stored
 *   (x @ W), bias [dim_hidden], position [batch, seqlen, dim_position] or NULL,
 *   out [batch, num_head, dim_position + dim_head, seqlen].
  * dim_head must be 32, dim_hidden 128, 256, 384 or 512 (the reference accepts multiples of 128,
 * network/sp_layer.py:17), dim_position 0 or 2. */
int spgt_multihead_projection_with_position_rrc_forward(
    const float* input, const float* weight, const float* bias, const float* position, float* out,
    int seqlen, int dim_hidden, int num_head, int dim_head, int dim_position, int batch,
    spgt_stream_t stream);

/* Replaces multihead_projection_layernorm_with_position_rrc_forward
 * (extension/bind/galerkin_attention.cu:50-68): the projection above followed, per token
 * and head, by LayerNorm over the 32 head features with affine ln_weight/ln_bias
 * [num_head, 32]; also writes invsigma [batch, num_head, seqlen] = 1/sqrt(var + eps). */
int spgt_multihead_projection_layernorm_with_position_rrc_forward(
    const float* input, const float* weight, const float* bias, const float* ln_weight,
    const float* ln_bias, float norm_eps, const float* position, float* out, float* invsigma,
    int seqlen, int dim_hidden, int num_head, int dim_head, int dim_position, int batch,
    spgt_stream_t stream);

/* Replaces multihead_galerkin_attention_cccr_forward
 * (extension/bind/galerkin_attention.cu:104-124).
 *   Q, K, V : [batch, num_head, d_posk, seqlen]  (feature-major, seqlen contiguous)
 *   out     : [batch, num_head, seqlen, d_posk]
 *   out[b,h,s,j] = sum_i Q[b,h,i,s] * ( sum_t K[b,h,i,t] V[b,h,j,t] / seqlen )
 * d_posk must be 32 or 34.  The seqlen reduction is split over workgroups and
 * finished by a fixed-order second stage, so results are run-to-run identical. */
size_t spgt_galerkin_attention_cccr_workspace_bytes(int batch, int num_head, int d_posk, int seqlen);
int spgt_galerkin_attention_cccr_forward(const float* Q, const float* K, const float* V, float* out,
                                         void* workspace, size_t workspace_bytes, int batch,
                                         int num_head, int d_posk, int seqlen, spgt_stream_t stream);

/* Replaces batched_skinny_gemm (extension/bind/galerkin_attention.cu:175-198) and the
 * launcher under it, sgemm_32x32_4x8_SplitK::sgemm_cuda
 * (extension/native/sgemm_32x32_splitk.cu:662-705):
 *   C[b] = alpha * A[b] * B[b],  A: M x K, B: K x N, C: M x N, small M, N and long K,
 * with batch strides a_stride, b_stride, c_stride (in floats) and any of the eight
 * operand orders.  Two-stage deterministic split-K. */
size_t spgt_batched_skinny_gemm_workspace_bytes(int M, int N, int K, int batch_count);
int spgt_batched_skinny_gemm(const float* A, const float* B, float* C, float alpha, int M, int N,
                             int K, int64_t a_stride, int64_t b_stride, int64_t c_stride, int order,
                             int batch_count, void* workspace, size_t workspace_bytes,
                             spgt_stream_t stream);

/* Replaces sgemm_32x32_4x4::sgemm_cuda (extension/native/sgemm_32x32.cu:683-710), the batched GEMM for a
 * short contraction axis and long M or N that the reference uses for Q (K^T V) and in the attention backward
 * (extension/bind/galerkin_attention.cu:118-122, 142-171):
 *   C[b] = alpha * A[b] * B[b],  A: M x K, B: K x N, C: M x N, any of the eight operand orders,
 * one launch, every 32 x 32 tile of C computed by one workgroup over the whole of K, no workspace. */
int spgt_batched_small_k_gemm(const float* A, const float* B, float* C, float alpha, int M, int N, int K,
                              int64_t a_stride, int64_t b_stride, int64_t c_stride, int order,
                              int batch_count, spgt_stream_t stream);

/* One-call fused attention core on token-major operands.  No single reference
 * function corresponds to it: it computes what Sp_GalerkinAttention.forward
 * (network/sp_layer.py:64-72) obtains from the LayerNorm epilogue of
 * multihead_projection_layernorm_with_position_rrc_forward followed by
 * multihead_galerkin_attention_cccr_forward, i.e. GalerkinAttention's
 * layer_norm + concat + matmuls (network/layer.py:130-152), starting from the
 * plain projections x@W+b.
 *   Q, K, V  : [B, S, H*32] with row stride ld_in floats (>= H*32, multiple of 4)
 *   position : [B, S, 2] (dp == 2) or NULL (dp == 0)
 *   ln_*     : [H, 32] LayerNorm affine of K and of V; eps as in F.layer_norm
 *   out      : [B, S, H*(dp+32)]  (per head: dp position channels, then 32 features)
 *   ktv      : [B, H, dp+32, dp+32] row-major, receives K'^T V' / S */
size_t spgt_galerkin_attention_fused_workspace_bytes(int B, int S, int H, int dp);
int spgt_galerkin_attention_fused_forward(const float* Q, const float* K, const float* V,
                                          int64_t ld_in, const float* position,
                                          const float* ln_weight_K, const float* ln_bias_K,
                                          const float* ln_weight_V, const float* ln_bias_V,
                                          float norm_eps, float* out, float* ktv, void* workspace,
                                          size_t workspace_bytes, int B, int S, int H, int dp,
                                          spgt_stream_t stream);

/* Backward of spgt_galerkin_attention_fused_forward on the same token-major operands: the reference's
 * multihead_galerkin_attention_cccr_backward (extension/bind/galerkin_attention.cu:126-173) together with the
 * LayerNorm backward of its two projection+LayerNorm operators (extension/native/multihead_dim32.cu:148-271),
 * from the plain projections x@W+b as the forward takes them.
 *   grad_out : [B, S, H*(dp+32)] gradient of the forward's `out`
 *   Q, K, V, position, ln_*, norm_eps : the forward's inputs; ktv : the forward's K'^T V' / S
 *   grad_Q, grad_K, grad_V : [B, S, H*32] with row stride ld_out floats: gradients of the plain projections
 *                            (the LayerNorm backward of K and V is applied; position gets no gradient)
 *   grad_ln  : [4, H*32]: gradients of ln_weight_K, ln_bias_K, ln_weight_V, ln_bias_V
 * Two passes over the sequence (Q~^T G / S as partial tiles summed in a fixed order; then one stream over
 * K, V and grad_out that writes the three gradients), LayerNorm statistics recomputed in registers. */
size_t spgt_galerkin_attention_fused_backward_workspace_bytes(int B, int S, int H, int dp);
int spgt_galerkin_attention_fused_backward(const float* grad_out, const float* Q, const float* K, const float* V,
                                           int64_t ld_in, const float* position, const float* ln_weight_K,
                                           const float* ln_bias_K, const float* ln_weight_V,
                                           const float* ln_bias_V, float norm_eps, const float* ktv,
                                           float* grad_Q, float* grad_K, float* grad_V, int64_t ld_out,
                                           float* grad_ln, void* workspace, size_t workspace_bytes, int B, int S,
                                           int H, int dp, spgt_stream_t stream);

/* spgt_galerkin_attention_fused_forward for callers that cannot allocate device memory or hand in
 * a workspace (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).
 * It has no counterpart in the reference.  The partial tiles of the K/V pass go to a device array
 * of spgt_galerkin_attention_fused_static_max_bytes() bytes (16 MiB) that is part of the library's
 * code object: every GPU the library runs on holds one copy until the process ends.  The call
 * allocates and frees nothing; a shape whose spgt_galerkin_attention_fused_workspace_bytes exceeds
 * the array is rejected with SPGT_ERR_WORKSPACE (B=8, S=44521, H=4 needs 4.2 MB).  All calls on
 * one GPU share that GPU's array: calls that overlap in time on one GPU (two streams, two threads)
 * race and must be serialised by the caller.  The first call on a GPU does that GPU's one-time
 * set-up on the host (hipGetSymbolAddress of the array, which may load the code object, and the
 * K/V pass's dynamic-LDS attribute; both checked, SPGT_ERR_LAUNCH on failure): make one call on
 * each GPU before capturing a graph or entering a section that must not allocate.  Arguments and
 * results otherwise as spgt_galerkin_attention_fused_forward (Q and out are required). */
size_t spgt_galerkin_attention_fused_static_max_bytes(void);
int spgt_galerkin_attention_fused_forward_static(const float* Q, const float* K, const float* V,
                                                 int64_t ld_in, const float* position,
                                                 const float* ln_weight_K, const float* ln_bias_K,
                                                 const float* ln_weight_V, const float* ln_bias_V,
                                                 float norm_eps, float* out, float* ktv, int B, int S,
                                                 int H, int dp, spgt_stream_t stream);

/* ---- backward of the attention operators ------------------------------------ */

/* Replaces multihead_galerkin_attention_cccr_backward (extension/bind/galerkin_attention.cu:126-173).
 *   grad_out [batch, num_head, seqlen, d_posk]; Q, K, V, grad_Q, grad_K, grad_V [batch, num_head, d_posk, seqlen]. */
size_t spgt_galerkin_attention_cccr_backward_workspace_bytes(int batch, int num_head, int d_posk, int seqlen);
int spgt_galerkin_attention_cccr_backward(const float* grad_out, const float* Q, const float* K,
                                          const float* V, float* grad_Q, float* grad_K, float* grad_V,
                                          void* workspace, size_t workspace_bytes, int batch, int num_head,
                                          int d_posk, int seqlen, spgt_stream_t stream);

/* Replaces datamove::batched_transpose_gather (extension/native/datamove.cu:121-163), the first step of
 * both projection backwards (extension/bind/galerkin_attention.cu:34-39):
 *   src [batch, num_head, dim_position + dim_head, seqlen], rows dim_position.. of every head
 *   -> dst [batch, seqlen, num_head * dim_head]. */
int spgt_heads_feature_to_token_major(const float* src, float* dst, int batch, int num_head,
                                      int dim_position, int dim_head, int seqlen, spgt_stream_t stream);

/* Replaces mh32::lnorm_grad_ccc_cuda (extension/native/multihead_dim32.cu:148-271, 601-618), on token-major
 * data and from the pre-LayerNorm projection instead of (y - beta) / gamma:
 *   pre_ln, grad_ln, grad_pre_ln [tokens, num_head*32]; ln_weight, grad_ln_weight, grad_ln_bias [num_head, 32]. */
size_t spgt_layernorm_heads_backward_workspace_bytes(int64_t tokens, int num_head);
int spgt_layernorm_heads_backward(const float* pre_ln, const float* grad_ln, const float* ln_weight,
                                  float norm_eps, float* grad_pre_ln, float* grad_ln_weight,
                                  float* grad_ln_bias, void* workspace, size_t workspace_bytes,
                                  int64_t tokens, int num_head, spgt_stream_t stream);

/* ---- FNO2d data movement and spectral contraction --------------------------- */

/* Replaces batched_transpose (extension/bind/datamove.cu:8-23):
 * src [batch_count, M, N] -> dst [batch_count, N, M], 32-bit words moved bit-exactly. */
int spgt_batched_transpose(const float* src, float* dst, int batch_count, int M, int N,
                           spgt_stream_t stream);

/* Replaces transpose_gather_dual (extension/bind/datamove.cu:25-44).  src is complex64
 * [dim, H_all, W_all]; out_k [H_low, W_low, dim] receives the window whose top-left
 * corner is (H_base_k, W_base_k), transposed.  64-bit words moved bit-exactly. */
int spgt_transpose_gather_dual(const float* src, float* out1, float* out2, int dim, int H_all,
                               int W_all, int H_low, int W_low, int H_base_1, int W_base_1,
                               int H_base_2, int W_base_2, spgt_stream_t stream);

/* Replaces transpose_scatter_dual (extension/bind/datamove.cu:46-64), including its
 * torch::zeros: out [dim, H_all, W_all] complex64 is written completely, zero outside
 * the two windows; where the windows overlap the second source wins. */
int spgt_transpose_scatter_dual(const float* src1, const float* src2, float* out, int dim, int H_all,
                                int W_all, int H_low, int W_low, int H_base_1, int W_base_1,
                                int H_base_2, int W_base_2, spgt_stream_t stream);

/* The spectral part of Sp_SpectralConv2D.forward between rfft2 and irfft2 in one call
 * (network/sp_layer.py:139-148: transpose_gather_dual, two complex `@`, and
 * transpose_scatter_dual; the arithmetic is complex_matmul_2D of network/layer.py:249-261):
 *   Out_ft[n, o, hb_k+h, wb_k+w] = sum_i X_ft[n, i, hb_k+h, wb_k+w] * weight_k[h, w, i, o]
 * X_ft [N, Cin, H_all, W_all] complex64, weight_k [H_low, W_low, Cin, Cout] complex64
 * (the accelerated module's parameter layout, sp_layer.py:119-121),
 * Out_ft [N, Cout, H_all, W_all] complex64, written completely (zero outside the windows). */
int spgt_spectral_mode_contract(const float* X_ft, const float* weight_1, const float* weight_2,
                                float* Out_ft, int N, int Cin, int Cout, int H_all, int W_all,
                                int H_low, int W_low, int H_base_1, int W_base_1, int H_base_2,
                                int W_base_2, spgt_stream_t stream);

/* The same contraction on compact operands that hold only the retained modes (for a spectral layer
 * that obtains them by truncated DFTs instead of full FFTs; no reference counterpart):
 *   O[n, k*H_low + h, o, w] = sum_i Z[n, k*H_low + h, i, w] * weight_k[h, w, i, o],  k = 0, 1
 * Z [N, 2*H_low, Cin, W_low], O [N, 2*H_low, Cout, W_low] complex64. */
int spgt_spectral_modes_compact(const float* Z, const float* weight_1, const float* weight_2, float* O,
                                int N, int Cin, int Cout, int H_low, int W_low, spgt_stream_t stream);

/* Replaces F.interpolate(x, size, mode='bilinear', align_corners=True) as used by
 * DownScaler2D / UpScaler2D (network/model.py:30, 36, 59, 63):
 * src [planes, H_in, W_in] -> dst [planes, H_out, W_out]. */
int spgt_bilinear_align_corners(const float* src, float* dst, int planes, int H_in, int W_in,
                                int H_out, int W_out, spgt_stream_t stream);

/* The same resampling fused with the NCHW -> NHWC permute that follows it in UpScaler2D.forward
 * (network/model.py:63-64): src [N, C, H_in, W_in] -> dst [N, H_out, W_out, C]. */
int spgt_bilinear_align_corners_nhwc(const float* src, float* dst, int N, int C, int H_in, int W_in,
                                     int H_out, int W_out, spgt_stream_t stream);

/* 1 when the truncated-DFT row kernels serve this shape (channels a multiple of 32; modes <= 16 with
 * r <= 1024, or modes <= 32 with r <= 512), else 0. */
int spgt_truncated_dft_rows_supported(int r, int channels, int modes);

/* The w-direction of rfft2 restricted to the modes Sp_SpectralConv2D keeps
 * (network/sp_layer.py:136-141: rfft2, then only columns kw < modes are read):
 *   Y[row, c, j] = sum_w x[row, w, c] * table[w, j],   j = (kw, re|im) < 2*modes
 * x [rows, r, channels] (rows = N*r grid rows of the channels-last tensor); table[w, j] =
 * (cos, -sin)(2 pi kw w / r) / sqrt(r), handed over zero-padded to [2*ceil(r/2), 32], or
 * [2*ceil(r/2), 64] when 2*modes > 32 (the layout the kernel keeps in LDS, 16-byte aligned).  Y is [rows, channels, 2*modes], or with planar != 0
 * [N, 2*modes, r, channels] (row = n*r + h), the layout spgt_spectral_modes_middle works on. */
int spgt_truncated_dft_rows_forward(const float* x, const float* table, float* Y, int64_t rows, int r,
                                    int channels, int modes, int planar, spgt_stream_t stream);

/* The w-direction of irfft2 for a spectrum that is zero beyond column `modes`
 * (network/sp_layer.py:149-151):
 *   y[row, w, o] = sum_j table[w, j] * U[row, o, j]
 * U [rows, channels, 2*modes] (or planar [N, 2*modes, r, channels]); table = the forward table
 * with columns scaled by 1 for kw = 0 and the Nyquist column, else 2, handed over zero-padded to
 * [32*ceil(r/32), 2*modes + 1] (16-byte aligned); y [rows, r, channels]. */
int spgt_truncated_dft_rows_inverse(const float* U, const float* table, float* y, int64_t rows, int r,
                                    int channels, int modes, int planar, spgt_stream_t stream);

/* 1 when spgt_spectral_inverse_linear serves this shape ((in, out) features 32 -> 32, 64 -> 64, 64 -> 32,
 * 128 -> 32 or 128 -> 64; 2*modes <= min(64, r), r <= 1024). */
int spgt_spectral_inverse_linear_supported(int r, int in_features, int out_features, int modes);

/* The end of Sp_SpectralConv2D.forward (network/sp_layer.py:132, 149-155) in one pass:
 *   out[row, w, o] = activation(sum_c x[row, w, c] * weight_kn[c, o] + bias[o] + sum_j table[w, j] * U[row, o, j])
 * = the residual Linear, the w-direction of irfft2 for the retained modes (spgt_truncated_dft_rows_inverse),
 * their sum and the activation, without the inverse transform's result going to memory.
 * U planar [N, 2*modes, r, out_features] as spgt_spectral_modes_middle writes it; x [rows = N*r, r, in_features];
 * out [rows, r, out_features]; weight_kn [in_features, out_features] (the transpose of nn.Linear.weight); bias
 * [out_features] or null;
 * table_operand [ceil(r/32), steps, 64], steps = 16 for modes <= 16, else 32: entry (t, kk, l) =
 * table[32 t + l % 32, 2 kk + l / 32] of the inverse table above, zero where the row is >= r or the column
 * >= 2*modes. */
int spgt_spectral_inverse_linear(const float* U, const float* table_operand, const float* x, const float* weight_kn,
                                 const float* bias, int activation, float* out, int64_t rows, int r,
                                 int in_features, int out_features, int modes, spgt_stream_t stream);

/* 1 when spgt_spectral_modes_middle serves this shape (Cin <= 128, Cout <= 64, 2*modes <= min(64, r),
 * r <= 4096). */
int spgt_spectral_modes_middle_supported(int r, int Cin, int Cout, int modes);

/* Bytes of device scratch spgt_spectral_modes_middle needs (the contracted modes O). */
size_t spgt_spectral_modes_middle_workspace_bytes(int N, int Cout, int modes);

/* Everything between the two w-direction products of Sp_SpectralConv2D's inference path
 * (network/sp_layer.py:136-151 restricted to the kept modes; contraction as complex_matmul_2D,
 * network/layer.py:249-261), two launches with O in the caller's workspace:
 *   Z[n, kh, c, kw] = sum_h table_h[kh, h] Y[n, h, c, kw]              kh: the 2*modes kept rows
 *   O[n, kh, o, kw] = sum_c Z[n, kh, c, kw] W[kh, kw, c, o]            W = weight_1 (kh < modes) | weight_2
 *   U[n, h, o, kw]  = sum_kh table_h_inverse[h, kh] O[n, kh, o, kw]
 * Y [N, 2*modes, r, Cin] and U [N, 2*modes, r, Cout] are the planar layouts of the row kernels
 * (plane 2*kw real, 2*kw+1 imaginary); table_h [2*modes, r] and table_h_inverse [r, 2*modes] are
 * complex64; weight_1, weight_2 [modes, modes, Cin, Cout, 2] as network/sp_layer.py:119-121. */
int spgt_spectral_modes_middle(const float* Y, const float* table_h, const float* table_h_inverse,
                               const float* weight_1, const float* weight_2, float* U, void* workspace,
                               size_t workspace_bytes, int N, int r, int Cin, int Cout, int modes,
                               spgt_stream_t stream);

/* Tensor layouts for spgt_bilinear_resample. */
enum { SPGT_LAYOUT_NCHW = 0, SPGT_LAYOUT_NHWC = 1 };

/* Activations (spgt_linear_forward, spgt_ffn_scalar_forward, spgt_bilinear_resample) and
 * residual placement for spgt_linear_forward. */
enum { SPGT_ACT_NONE = 0, SPGT_ACT_RELU = 1, SPGT_ACT_SILU = 2 };
enum { SPGT_RES_NONE = 0, SPGT_RES_BEFORE_ACT = 1, SPGT_RES_AFTER_ACT = 2 };

/* The resampling of DownScaler2D / UpScaler2D (network/model.py:30-38, 59-64) together with the
 * permutes and activations around it: F.interpolate(mode='bilinear', align_corners=True) from
 * src [N, C, H_in, W_in] or [N, H_in, W_in, C] to dst [N, C, H_out, W_out] or [N, H_out, W_out, C]
 * (NCHW->NCHW, NCHW->NHWC and NHWC->NCHW), with pre_activation applied pre_activation_count
 * (0..2) times to every source sample (the activation of ConvResBlock2D, network/layer.py:7-24,
 * and the scaler's own) and post_activation applied to the result.  pre_bias [C] (may be null) is
 * added to every source sample first: the bias of a convolution that was run without it. */
int spgt_bilinear_resample(const float* src, const float* pre_bias, float* dst, int N, int C, int H_in,
                           int W_in, int H_out, int W_out, int src_layout, int dst_layout,
                           int pre_activation, int pre_activation_count, int post_activation,
                           spgt_stream_t stream);

/* Backward of the resampling: the adjoint of F.interpolate(mode='bilinear', align_corners=True) from
 * [H_in, W_in] to [H_out, W_out], grad_in[i] = sum over the outputs o that read source i of weight(o, i) *
 * grad_out[o], gathered per source position in a fixed order (no atomic additions).  The reference leaves this
 * step to autograd of F.interpolate in DownScaler2D / UpScaler2D (network/model.py:30-38, 59-64).  Both tensors
 * have the same layout: SPGT_LAYOUT_NCHW (grad_out [N, C, H_out, W_out], grad_in [N, C, H_in, W_in]) or
 * SPGT_LAYOUT_NHWC (grad_out [N, H_out, W_out, C], grad_in [N, H_in, W_in, C]; C a multiple of 4, 16-byte
 * aligned).  Every element of grad_in is written. */
int spgt_bilinear_adjoint(const float* grad_out, float* grad_in, int N, int C, int H_in, int W_in, int H_out,
                          int W_out, int layout, spgt_stream_t stream);

/* UpScaler2D's last F.interpolate (network/model.py:63-64) on a channels-last source together with the grid
 * columns' share of the decoder's input layer Linear(cat([X, grid])) (network/sp_model.py:60, 118):
 *   dst[n, y, x, c] = bilinear(src)[n, y, x, c] + sum_e extra[n, y, x, e] * w_extra[e, c]
 * with align_corners=True.  The Linear over the hidden features commutes with the resampling, so a caller can
 * run it on the low-resolution tensor and hand its result in as src.  src [N, H_in, W_in, C],
 * dst [N, H_out, W_out, C], extra [N, H_out, W_out, n_extra] and w_extra [n_extra, C] (n_extra 0..4; both may
 * be null when it is 0).  C must be a multiple of 4; src, dst and w_extra 16-byte aligned. */
int spgt_bilinear_nhwc_affine(const float* src, float* dst, int N, int C, int H_in, int W_in, int H_out,
                              int W_out, const float* extra, const float* w_extra, int n_extra,
                              spgt_stream_t stream);

/* DownScaler2D's cat([X1, X2, X3], dim=1) -> F.interpolate -> permute -> activation (network/model.py:35-38)
 * without the concatenated tensor: srcs[s] is an NCHW tensor [N, channels[s], H_in, W_in] (n_src 1..4), dst
 * [N, H_out, W_out, sum channels] channels-last.  Where pre_flags[s] is non-zero, source s is a convolution
 * output that still lacks its bias pre_biases[s] (may be null) and its activation: pre_activation is applied
 * pre_activation_count (0..2) times to its samples first (ConvResBlock2D, network/layer.py:7-24).
 * post_activation is applied to every result.  pre_biases and pre_flags may be null (no source needs them).
 * The channel counts must add up to a multiple of 4; dst 16-byte aligned. */
int spgt_bilinear_resample_concat(const float* const* srcs, const float* const* pre_biases, const int* channels,
                                  const int* pre_flags, int n_src, float* dst, int N, int H_in, int W_in,
                                  int H_out, int W_out, int pre_activation, int pre_activation_count,
                                  int post_activation, spgt_stream_t stream);

/* UpScaler2D's F.interpolate -> conv3x3(padding 1) -> bias -> activation(s) (network/model.py:59-62,
 * network/layer.py:7-24) with the channel mixing done before the interpolation: both are linear, so
 *   conv(interp(X))[y, x, :] = sum over taps t = 3 ky + kx of interp(X . W_t)[y + ky - 1, x + kx - 1, :],
 * taps outside the interpolated image contributing nothing (zero padding).  The caller computes
 * Z [N, H_in, W_in, 9, C] = X . [W_0 | ... | W_8] with one GEMM on the low-resolution tokens
 * (W_t[ci, co] = weight[co, ci, ky, kx]); this call gathers and blends (align_corners=True), adds bias [C]
 * (may be null) and applies `activation` activation_count (0..2) times.  dst [N, H_out, W_out, C]
 * channels-last.  C must be a multiple of 4; Z, bias and dst 16-byte aligned. */
int spgt_upsample_conv3x3_gather(const float* Z, const float* bias, float* dst, int N, int C, int H_in, int W_in,
                                 int H_out, int W_out, int activation, int activation_count,
                                 spgt_stream_t stream);

/* Backward of spgt_upsample_conv3x3_gather without bias and activation: the gradient of the per-tap products,
 * dZ [N, H_in, W_in, 9, C] from grad [N, H_out, W_out, C] (the adjoint of shift + align_corners interpolation per tap,
 * gathered per low-resolution pixel in a fixed order).  With it UpScaler2D's interpolate -> conv3x3
 * (network/model.py:59-62) trains as a Linear on the low-resolution tokens plus this pair of kernels; the reference
 * leaves the step to autograd of F.interpolate and the convolution library.  C a multiple of 4, 16-byte aligned. */
int spgt_upsample_conv3x3_gather_adjoint(const float* grad, float* dZ, int N, int C, int H_in, int W_in, int H_out,
                                         int W_out, spgt_stream_t stream);

/* 1 when spgt_conv3x3_resample serves this number of input channels (1..4), else 0. */
int spgt_conv3x3_resample_supported(int Cin);

/* DownScaler2D's first stage (network/model.py:30-33: conv0 = ConvResBlock2D(in_dim, out_dim, 3, 1),
 * bilinear interpolation to resolution_size[1], activation) for a few input channels, one pass:
 *   out[n, c] = post_activation(interpolate(pre_activation(conv3x3(x, weight, padding 1)[n, c] + bias[c])))
 * x [N, H_in, W_in, Cin] channels-last (the model's input layout), weight [Cout, Cin, 3, 3], bias
 * [Cout] or null, out [N, Cout, H_out, W_out]; align_corners=True as in the reference. */
int spgt_conv3x3_resample(const float* x, const float* weight, const float* bias, float* out, int N, int Cin,
                          int Cout, int H_in, int W_in, int H_out, int W_out, int pre_activation,
                          int post_activation, spgt_stream_t stream);

/* The three down-scaler kernels with ConvResBlock2D's dropout inside them (conv -> dropout -> activation,
 * network/layer.py:7-24; F.dropout's default training=True keeps it on in inference too): the sum of convolution and
 * bias is dropped before the first activation, with one decision per convolution output (n, c, y, x), the same for
 * every resampled pixel that reads it.  seed: two 32-bit words in device memory (8-byte aligned), read by the
 * kernel (see spgt_encoder_tail_forward_dropout); droprate in [0, 1), 0 = the call without dropout (seed may be
 * null).  spgt_bilinear_resample_concat_dropout drops the samples of the sources flagged in pre_flags.  The masks
 * are this library's own: the reference's distribution, not torch's random stream. */
int spgt_bias_activation_nchw_dropout(float* x, const float* bias, int N, int C, int64_t HW, int activation,
                                      int activation_count, const uint32_t* seed, float droprate,
                                      spgt_stream_t stream);
int spgt_conv3x3_resample_dropout(const float* x, const float* weight, const float* bias, float* out, int N, int Cin,
                                  int Cout, int H_in, int W_in, int H_out, int W_out, int pre_activation,
                                  int post_activation, const uint32_t* seed, float droprate, spgt_stream_t stream);
int spgt_bilinear_resample_concat_dropout(const float* const* srcs, const float* const* pre_biases, const int* channels,
                                          const int* pre_flags, int n_src, float* dst, int N, int H_in, int W_in,
                                          int H_out, int W_out, int pre_activation, int pre_activation_count,
                                          int post_activation, const uint32_t* seed, float droprate,
                                          spgt_stream_t stream);

/* Backward of spgt_conv3x3_resample (its _dropout form with a seed) without post activation, for an input that
 * needs no gradient (DownScaler2D's first stage on the model's input field, network/model.py:30-33): the gradients
 * of the convolution's weight and bias from grad = dL/dP, P [N, Cout, H_out, W_out] = bilinear(pre(dropout(conv3x3(x)
 * + bias))).  The full-resolution chain is formed again from x, weight, bias and the forward's seed; nothing of it
 * was stored.  out [Cout][R], R = 4 * ceil((1 + 9 * Cin) / 4): per output channel the bias gradient, then the
 * weight gradient [Cin][3][3], then padding.  The reference leaves this step to autograd (library convolution,
 * dropout, activation and F.interpolate backward).  workspace: spgt_conv3x3_resample_backward_workspace_bytes
 * (0 = unsupported shape), 16-byte aligned. */
size_t spgt_conv3x3_resample_backward_workspace_bytes(int N, int Cin, int Cout, int H_in, int W_in);
int spgt_conv3x3_resample_backward(const float* x, const float* weight, const float* bias, const float* grad,
                                   float* out, void* workspace, size_t workspace_bytes, int N, int Cin, int Cout,
                                   int H_in, int W_in, int H_out, int W_out, int pre_activation, const uint32_t* seed,
                                   float droprate, spgt_stream_t stream);

/* The tail of ConvResBlock2D (network/layer.py:7-24) after a bias-free convolution, and the
 * scaler's own activation where it follows directly (network/model.py:61-62), in place:
 * x[n, c, :] = activation^activation_count(x[n, c, :] + bias[c]) on x [N, C, HW]; bias may be null,
 * activation_count is 0..2. */
int spgt_bias_activation_nchw(float* x, const float* bias, int N, int C, int64_t HW, int activation,
                              int activation_count, spgt_stream_t stream);

/* The end of the model's forward (Sp_GalerkinTransformer2D.forward, network/sp_model.py:109-111) in one pass:
 * out = x * scale + shift (the target normalizer's inverse_transform with scale = std + eps, shift = mean;
 * multiply and add rounded separately, like the two tensor operations), and with zero_boundary the outermost
 * rows and columns of the [H, W] grid set to zero (the Dirichlet branch pads the interior with zeros).
 * x, out [N, H, W, C]; scale and shift point to one value each, or with per_point to H*W*C values. */
int spgt_denormalize_boundary(const float* x, const float* scale, const float* shift, int per_point, float* out,
                              int N, int H, int W, int C, int zero_boundary, spgt_stream_t stream);

/* 1 when spgt_linear_forward has a kernel for this shape (in_features 64, 128, 136 or 256;
 * out_features a multiple of 32), else 0. */
int spgt_linear_supported(int in_features, int out_features);

/* Replaces an nn.Linear call together with the elementwise kernels that follow it in the
 * modules either side of the attention: FeedForward (network/layer.py:155-174: Linear ->
 * activation -> Linear), the attention's fc_layer and the encoder's residual adds
 * (network/sp_layer.py:75, 97-103), Sp_SpectralConv2D's residual_layer + activation
 * (network/sp_layer.py:132, 155) and the decoder's Linear layers (network/sp_model.py:60, 63).
 *   y = x[tokens, in_features] @ weight_kn[in_features, out_features] + bias
 *   out = act(y + residual) | act(y) + residual | act(y)      (residual_mode 1 | 2 | 0)
 * weight_kn is the transpose of nn.Linear.weight, contiguous.  x, residual and out are
 * row-major with row strides ldx, ldr, ldo (in floats, multiples of 4, 16-byte aligned
 * bases); bias may be null; residual may alias out, x may not.
 * x_extra [tokens, extra_features] (row stride ldx_extra) with weight_extra_kn [extra_features,
 * out_features] adds up to four more input columns, y += x_extra @ weight_extra_kn: the grid
 * coordinates that Sp_DecoderRegressor concatenates to its input (network/sp_model.py:59-60).
 * The output columns may be split into planes of out_plane_cols columns (a multiple of 32
 * that divides out_features; 0 = one plane): column n of token t is written to
 * out[(n / out_plane_cols) * out_plane_stride + t * ldo + n % out_plane_cols], which lets one
 * call with the packed [W_Q | W_K | W_V] produce three contiguous projections. */
int spgt_linear_forward(const float* x, int64_t ldx, const float* weight_kn, const float* bias,
                        const float* residual, int64_t ldr, int residual_mode, int activation,
                        const float* x_extra, int64_t ldx_extra, const float* weight_extra_kn,
                        int extra_features, float* out, int64_t ldo, int out_plane_cols,
                        int64_t out_plane_stride, int64_t tokens, int in_features, int out_features,
                        spgt_stream_t stream);

/* 1 when spgt_ffn_scalar_forward has a kernel for this shape (in_features 32, 64 or 128,
 * hidden_features 128 or 256), else 0. */
int spgt_ffn_scalar_supported(int in_features, int hidden_features);

/* Replaces FeedForward (network/layer.py:155-174) when its out_dim is 1, the regression
 * head of Sp_DecoderRegressor (network/sp_model.py:51, 63), in one kernel:
 *   out[t] = sum_n act(x[t, :] . weight1_kn[:, n] + bias1[n]) * weight2[n] + bias2[0]
 * weight1_kn [in_features, hidden_features] is the transpose of layer1.weight, weight2
 * [hidden_features] is layer2.weight's single row; bias1 and bias2 (one element, on the
 * device) may be null.  x is row-major with row stride ldx (floats, a multiple of 4). */
int spgt_ffn_scalar_forward(const float* x, int64_t ldx, const float* weight1_kn, const float* bias1,
                            const float* weight2, const float* bias2, int activation, float* out,
                            int64_t tokens, int in_features, int hidden_features, spgt_stream_t stream);

/* 1 when spgt_encoder_tail_forward has a kernel for this shape (attn_features 128 or 136,
 * dim_hidden 128, ffn_hidden 256), else 0. */
int spgt_encoder_tail_supported(int attn_features, int dim_hidden, int ffn_hidden);

/* Everything an encoder layer does after the attention core (Sp_EncoderLayer.forward,
 * network/sp_layer.py:97-103, with the attention's fc_layer, network/sp_layer.py:75, and
 * FeedForward, network/layer.py:155-174), in one launch:
 *   y1  = x + attn_out @ fc_weight_kn + fc_bias
 *   out = y1 + act(y1 @ ffn1_weight_kn + ffn1_bias) @ ffn2_weight_kn + ffn2_bias
 * attn_out [tokens, attn_features] (row stride ld_attn) is the attention core's output, x and out
 * [tokens, dim_hidden] are the residual stream before and after; the *_kn weights are the
 * transposes of the nn.Linear weights ([in, out], contiguous).  Intermediates stay in LDS. */
int spgt_encoder_tail_forward(const float* attn_out, int64_t ld_attn, const float* x,
                              const float* fc_weight_kn, const float* fc_bias,
                              const float* ffn1_weight_kn, const float* ffn1_bias,
                              const float* ffn2_weight_kn, const float* ffn2_bias, int activation,
                              float* out, int64_t tokens, int attn_features, int dim_hidden,
                              int ffn_hidden, spgt_stream_t stream);

/* The attention core with its last product folded into the layer's output projection
 * (Sp_GalerkinAttention.forward, network/sp_layer.py:64-75: out = fc_layer(Q~ (K~^T V~ / S))).  The product is
 * associative, (Q~ M_h) Wfc_h = Q~ (M_h Wfc_h), so the pass over Q and the [tokens, H*(dp+32)] attention
 * output disappear; three calls replace spgt_galerkin_attention_fused_forward + spgt_encoder_tail_forward:
 *   spgt_galerkin_attention_ktv_forward   K/V pass and tile reduction only: ktv [B, H, dp+32, dp+32] = M
 *                                         (arguments as in spgt_galerkin_attention_fused_forward, same workspace)
 *   spgt_fold_ktv_into_fc                 folded [B, H*32, out_features]: row h*32 + i = (M_h Wfc_h)[dp + i], and
 *                                         folded_pos [B, dp, out_features]: row p = sum_h (M_h Wfc_h)[p]
 *                                         (fc_weight_kn [H*(dp+32), out_features], the transposed fc_layer weight)
 *   spgt_encoder_tail_folded_forward      y1 = x + q @ folded[b] + position @ folded_pos[b] + fc_bias, then the
 *                                         feed-forward net as in spgt_encoder_tail_forward; q [B*S, 128] (row
 *                                         stride ld_q) is the projected Q, position [B*S, 2] (dp == 2) or null */
int spgt_galerkin_attention_ktv_forward(const float* K, const float* V, int64_t ld_in, const float* position,
                                        const float* ln_weight_K, const float* ln_bias_K,
                                        const float* ln_weight_V, const float* ln_bias_V, float norm_eps,
                                        float* ktv, void* workspace, size_t workspace_bytes, int B, int S, int H,
                                        int dp, spgt_stream_t stream);
int spgt_fold_ktv_into_fc(const float* ktv, const float* fc_weight_kn, float* folded, float* folded_pos, int B,
                          int H, int dp, int out_features, spgt_stream_t stream);
int spgt_encoder_tail_folded_forward(const float* q, int64_t ld_q, const float* position, const float* x,
                                     const float* folded_fc, const float* folded_pos, const float* fc_bias,
                                     const float* ffn1_weight_kn, const float* ffn1_bias,
                                     const float* ffn2_weight_kn, const float* ffn2_bias, int activation,
                                     float* out, int B, int64_t S, int dp, int dim_hidden, int ffn_hidden,
                                     spgt_stream_t stream);

/* The same two launches with the reference's dropouts applied inside them: Sp_GalerkinAttention drops the output
 * of fc_layer (network/sp_layer.py:76) and FeedForward its own output (network/layer.py:173), both with
 * F.dropout's default training=True, i.e. also in inference, before the residual is added.
 *   y1 = x + dropout(fc output, fc_droprate)      out = y1 + dropout(ffn output, ffn_droprate)
 * The keep decision of an element is a hash of (seed, site, token, column); kept values are scaled by
 * 1 / (1 - rate).  seed points to two 32-bit words in device memory (8-byte aligned): read by the kernel, so a
 * captured graph that refills them with a generator kernel draws new masks on every replay.  Rates in [0, 1);
 * with both 0 the calls are spgt_encoder_tail_forward / spgt_encoder_tail_folded_forward and seed may be null.
 * The masks are this library's own: they follow the reference's distribution, not torch's random stream. */
int spgt_encoder_tail_forward_dropout(const float* attn_out, int64_t ld_attn, const float* x,
                                      const float* fc_weight_kn, const float* fc_bias,
                                      const float* ffn1_weight_kn, const float* ffn1_bias,
                                      const float* ffn2_weight_kn, const float* ffn2_bias, int activation,
                                      float* out, int64_t tokens, int attn_features, int dim_hidden, int ffn_hidden,
                                      const uint32_t* seed, float fc_droprate, float ffn_droprate,
                                      spgt_stream_t stream);
int spgt_encoder_tail_folded_forward_dropout(const float* q, int64_t ld_q, const float* position, const float* x,
                                             const float* folded_fc, const float* folded_pos, const float* fc_bias,
                                             const float* ffn1_weight_kn, const float* ffn1_bias,
                                             const float* ffn2_weight_kn, const float* ffn2_bias, int activation,
                                             float* out, int B, int64_t S, int dp, int dim_hidden, int ffn_hidden,
                                             const uint32_t* seed, float fc_droprate, float ffn_droprate,
                                             spgt_stream_t stream);

/* One strided copy: dst[i0*dst_stride[0] + i1*dst_stride[1] + i2*dst_stride[2]] =
 * src[i0*src_stride[0] + i1*src_stride[1] + i2*src_stride[2]] for i_k < size[k]; 32-bit words, strides in words. */
typedef struct {
    const float* src;
    float* dst;
    int32_t size[3];
    int32_t src_stride[3];
    int32_t dst_stride[3];
} spgt_copy_desc;

/* Runs `count` strided copies (descs: host array) in ceil(count / 64) launches.  No counterpart in the
 * reference, whose kernels read nn.Parameter layouts directly: the kernels here take some operands in
 * derived layouts (nn.Linear weights transposed to [in, out], [W_Q | W_K | W_V] packed, a 3x3 convolution's
 * weight as nine [Cin, Cout] taps), and the modules refresh all of them from the parameters with this call
 * at the start of a forward, so that a parameter changed in place by any means is never served stale. */
int spgt_strided_copy_batch(const spgt_copy_desc* descs, int count, spgt_stream_t stream);

/* Weight and bias gradients of y = x W + b from dL/dy on token-major operands: what the reference's
 * projection backward computes with a library GEMM on the transposed input and a library reduction
 * (extension/bind/galerkin_attention.cu:41-46).
 *   x    : [tokens, in_features], row stride ldx floats (batch entry b at x + b * x_batch_stride; 0 = shared)
 *   grad : [tokens, out_features], row stride ldg floats (batch entry b at grad + b * grad_batch_stride)
 *   out  : per batch entry in_features * out_features + out_features floats, packed one after the other:
 *          dW [in_features, out_features] row-major (dW[k][n] = sum_t x[t][k] grad[t][n]) followed by
 *          db [out_features] (sum over the tokens)
 * The sum over the tokens is split over at most 256 chunks whose partial results go to the workspace and
 * are added in a fixed order: results are identical from run to run.  out_features must be a multiple of 4. */
size_t spgt_linear_weight_grad_workspace_bytes(int64_t tokens, int in_features, int out_features, int batch);
int spgt_linear_weight_grad(const float* x, int64_t ldx, int64_t x_batch_stride, const float* grad, int64_t ldg,
                            int64_t grad_batch_stride, float* out, void* workspace, size_t workspace_bytes,
                            int64_t tokens, int in_features, int out_features, int batch, spgt_stream_t stream);

/* out = residual + dropout(y, droprate) on [rows, cols] row-major (cols a multiple of 4; residual may be null; out
 * may be y): the reference's F.dropout followed by the residual add (network/sp_layer.py:76, 100-103;
 * network/layer.py:173) in one pass.  Keep decisions: a hash of (seed, site, row, column), kept values scaled by
 * 1 / (1 - droprate); seed = two 32-bit words in device memory.  The same call on dL/dout with the forward's seed
 * and site and no residual is the dropout's backward.  The masks are this library's own. */
int spgt_dropout_add(const float* y, const float* residual, float* out, int64_t rows, int cols,
                     const uint32_t* seed, float droprate, int site, spgt_stream_t stream);

/* Instrumented variant of spgt_galerkin_attention_fused_forward for benchmarks (no reference
 * counterpart): enqueues the call `iterations` times back to back (no synchronisation between
 * them, as a caller's loop would), iteration i reading the input set i % n_sets and writing the
 * output of the same index (Q_sets, K_sets, V_sets, out_sets: host arrays of n_sets device
 * pointers, so that consecutive iterations need not find their operands in the last-level
 * cache), with HIP events recorded on `stream` around each of the
 * three launches.  After one synchronisation at the end it writes, to host memory,
 *   stage_ms[3 i + 0]  K/V pass of iteration i (LayerNorm + partial K'^T V' tiles)
 *   stage_ms[3 i + 1]  fixed-order reduction of the partial tiles
 *   stage_ms[3 i + 2]  Q pass (out = Q' M)
 * in milliseconds, each from the event before the launch to the event after it. */
int spgt_galerkin_attention_fused_profile(const float* const* Q_sets, const float* const* K_sets,
                                          const float* const* V_sets, float* const* out_sets, int n_sets,
                                          int64_t ld_in, const float* position, const float* ln_weight_K,
                                          const float* ln_bias_K, const float* ln_weight_V,
                                          const float* ln_bias_V, float norm_eps, float* ktv, void* workspace,
                                          size_t workspace_bytes, int B, int S, int H, int dp,
                                          spgt_stream_t stream, int iterations, float* stage_ms);

#ifdef __cplusplus
}
#endif

#endif /* SPGT_HIP_H */
