/*
 * vibevoice_hip.h — C ABI of libvibevoice_hip.so, the MI355X (gfx950) backend
 * for vibevoice.c's accelerator seam.
 *
 * Every symbol below that carries a "replaces" citation has the name,
 * argument list and status-code behaviour of the declaration of the same name
 * in the reference's include/vibevoice/device.h, so the C engine above that
 * header links against this library unchanged. Symbols marked "addition" do
 * not exist in the reference: they are the fused forms of adjacent reference
 * calls and follow the same conventions.
 *
 * Conventions (device.h:16-20):
 *   - `void* stream` is a hipStream_t; NULL is the legacy default stream;
 *   - tensors are FP16, row-major, contiguous; pointers are device pointers;
 *   - every op enqueues on `stream` and returns at once with VV_OK or a
 *     negative vv_status_t; no op allocates, synchronises, throws or aborts,
 *     and none keeps state between calls, so concurrent calls on different
 *     streams from different host threads are safe and every op is
 *     graph-capturable;
 *   - a size of zero rows/elements is VV_OK with nothing launched.
 */
#ifndef VIBEVOICE_HIP_H
#define VIBEVOICE_HIP_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Status codes: the values of include/vibevoice/types.h:18-58 that this
 * backend returns. When the reference's types.h is already included its enum
 * is used instead. */
#ifndef VV_TYPES_H
typedef enum vv_status {
    VV_OK               = 0,
    VV_ERR_INVALID_ARG  = -1,
    VV_ERR_NULL_PTR     = -2,
    VV_ERR_UNSUPPORTED  = -7,
    VV_ERR_CUDA         = -100,   /* a runtime (HIP) call failed            */
    VV_ERR_CUDA_OOM     = -101,   /* device allocation: out of memory       */
    VV_ERR_CUDA_LAUNCH  = -102    /* a kernel launch was rejected           */
} vv_status_t;
#endif

/* ── Transformer layer ops: the hot path ───────────────────────────────── */

/* output[r,:] = table[ids[r],:], FP16 bits copied. ids are not range-checked
 * (as in the reference); row offsets are 64-bit.
 * replaces device.h:486-488 (src/cuda/embedding.cu:59-74). */
vv_status_t vv_embedding_dev(const void* table, const int32_t* ids, void* output,
                             int seq_len, int hidden_size, void* stream);

/* output = x * (1/sqrt(mean(x^2)+eps)) * weight per row, FP32 arithmetic,
 * one FP16 rounding. input != output.
 * replaces device.h:490-492 (src/cuda/rmsnorm.cu:82-100). */
vv_status_t vv_rmsnorm_dev(const void* input, const void* weight, void* output,
                           int seq_len, int hidden_size, float eps, void* stream);

/* Rotate-half RoPE in place over [seq_len, n_heads, head_dim]; the first row
 * is at position `*d_position` when d_position is non-NULL (read on the
 * device, so a captured launch can be replayed), else at position_offset.
 * head_dim must be even and at most 256, else VV_ERR_UNSUPPORTED.
 * replaces device.h:500-502 (src/cuda/rope.cu:89-103). */
vv_status_t vv_rope_dev(void* x, int seq_len, int n_heads, int head_dim,
                        int position_offset, const int* d_position, float theta,
                        void* stream);

/* output = silu(gate) * up elementwise; output may alias gate (or up).
 * replaces device.h:504-506 (src/cuda/swiglu.cu:79-103). */
vv_status_t vv_swiglu_dev(const void* gate, const void* up, void* output,
                          int n_elements, void* stream);

/* The same with gate and up as the two halves of one [rows, 2*inter] buffer.
 * replaces device.h:508-510 (declared there; no CUDA definition exists, Metal:
 * src/metal/mtl_transformer.c:88-97). */
vv_status_t vv_swiglu_fused_dev(const void* gate_up, void* output, int rows,
                                int inter, void* stream);

/* x = half_rn(float(x) + float(y)), in place.
 * replaces device.h:512 (src/cuda/conv_vae.cu:37-47). */
vv_status_t vv_residual_add_dev(void* x, const void* y, int total, void* stream);

/* output[m,n] = half_rn(float(output[m,n]) + float(bias[n])), in place.
 * replaces device.h:513-514 (src/cuda/conv_vae.cu:72-84). */
vv_status_t vv_bias_add_dev(void* output, const void* bias, int M, int N,
                            void* stream);

/* replaces device.h:717-720 (src/cuda/conv_vae.cu:100-116). */
vv_status_t vv_fp32_to_fp16_dev(const void* in_fp32, void* out_fp16, int n,
                                void* stream);
vv_status_t vv_fp16_to_fp32_dev(const void* in_fp16, void* out_fp32, int n,
                                void* stream);

/* ── Per-token int8 activations (the W8A8 / W4A8 front end) ─────────────── */

/* Per row: sx[m] = max|v| / 127, xq = clamp(round-half-even(v * 127 / max|v|),
 * +-127), where v is the FP16 value the unfused op would have written, so a
 * fused row is bit-identical to "op, then vv_act_quant_dev" and to the CPU
 * quantiser on those values. `layout` is the order of the int8 values inside
 * each run of 32 columns (0 natural, 1 nibble, 2 W4-GEMV, 3 W4-MMA: the
 * reference's include/vibevoice/q8.h); `xsum` (may be NULL) receives the sum of
 * xq over each run, [M][K/32]. K % 32 != 0, K > 22528 or pointers that are not
 * 16-byte (inputs) / 8-byte (xq) aligned: VV_ERR_UNSUPPORTED, nothing launched;
 * M <= 0, K <= 0 or a bad layout: VV_ERR_INVALID_ARG.
 * replace device.h:320-334 (src/cuda/act_quant.cu:226-275). */
vv_status_t vv_act_quant_dev(const void* x, int M, int K, int layout, int8_t* xq,
                             float* sx, int32_t* xsum, void* stream);
/* RMSNorm fused with the quantiser; K < 256: VV_ERR_UNSUPPORTED. */
vv_status_t vv_rmsnorm_q8_dev(const void* x, const void* weight, int M, int K,
                              float eps, int layout, int8_t* xq, float* sx,
                              int32_t* xsum, void* stream);
/* SwiGLU fused with the quantiser. */
vv_status_t vv_swiglu_q8_dev(const void* gate, const void* up, int M, int K,
                             int layout, int8_t* xq, float* sx, int32_t* xsum,
                             void* stream);
/* acc[k] = max(acc[k], max_m |x[m,k]|), x FP16 [M,K], acc FP32 [K] updated in
 * place (SmoothQuant calibration). replaces device.h:343-344
 * (src/cuda/act_quant.cu:277-313). */
vv_status_t vv_col_absmax_dev(const void* x, int M, int K, float* acc, void* stream);

/* ── W8A8 / W4A8 linear layers ──────────────────────────────────────────── */

/* Which kernel family runs an int8 linear layer (device.h:347-352). Here GEMV
 * is the v_dot4 kernel (M <= 8 only), MMA and SIMT both the MFMA kernels (tiles,
 * or weights straight into MFMA operands up to 64 rows). AUTO: GEMV for one or
 * two rows, MFMA beyond. Integer sums are exact, so the choice never shows in
 * the result. */
#define VV_I8_PATH_AUTO 0
#define VV_I8_PATH_GEMV 1
#define VV_I8_PATH_MMA  2
#define VV_I8_PATH_SIMT 3

/* y[M,N] = sx[m] * sw[n] * (xq[M,K] . w[N,K]^T) + bias[n] + residual[m,n]:
 * xq int8 with per-row scales sx (what vv_act_quant_dev writes in layout 0),
 * w int8 [N][K] with per-output-channel scales sw. bias FP16 [N] or NULL;
 * residual FP16 [M,N] or NULL, may alias y; y FP16, or FP32 when y_f32. The
 * int32 sums are exact, and the FP32 value is ((float)t * sx[m]) * sw[n], then
 * + bias, then + residual, nothing fused: bit-identical to the CPU kernel
 * (src/cpu/cpu_int8.c:480-483) for every M, N, K and path. K % 16 != 0 or
 * xq / w not 16-byte aligned: VV_ERR_UNSUPPORTED (the reference asks K % 32).
 * replaces device.h:363-366 (src/cuda/gemm_i8.cu:584-596). */
vv_status_t vv_w8a8_linear_dev(const int8_t* xq, const float* sx, const int8_t* w,
                               const float* sw, const void* bias, const void* residual,
                               void* y, int y_f32, int M, int N, int K, int path,
                               void* stream);

/* y[m,n] = sx[m] * sum_g s[n,g] * sum_{k in g} (q[n,k] - z[n,g]) xq[m,k] + bias[n]
 * + residual[m,n]: 4-bit weight codes with an FP16 scale and an integer zero
 * point per group of group_size columns. `packed` [N][K/2] is the accelerator
 * layout of the INT4 weights (vv_int4g_to_gpu_layout, src/quant/awq_repack.c:
 * 261-310), `sz` half2 {scale, zero} [N][K/group_size]. x_layout names the
 * order of xq inside every run of 32 columns: VV_Q8_W4_GEMV (2) for the GEMV
 * (M <= 8, K <= 20480), VV_Q8_W4_MMA (3) for the matrix-core tiles (any M);
 * AUTO takes the family the layout belongs to, and a family asked for with the
 * other layout declines (VV_ERR_UNSUPPORTED), as in the reference. Within a
 * family AUTO may pick a third kernel that streams the weights (at most 64
 * rows, group_size 64, 128 or 256; either order); a path asked for by name is
 * the GEMV or the LDS-tiled kernel itself. xsum (the
 * quantiser's int32 [M][K/32] sums, may be NULL) saves the GEMV some integer
 * work and is not read otherwise; the result does not depend on it. Group
 * sums are exact int32 and the groups are added in order in FP32, nothing
 * fused, then * sx[m], + bias, + residual: the CPU kernel's scalar form
 * (src/cpu/cpu_int8.c:212-233, 537-541), the same bits on every path.
 * K % 32, group_size % 32, K % group_size != 0: VV_ERR_UNSUPPORTED.
 * replaces device.h:385-389 (src/cuda/gemm_i8.cu:598-614). */
vv_status_t vv_w4a8_linear_dev(const int8_t* xq, int x_layout, const float* sx,
                               const int32_t* xsum, const void* packed, const void* sz,
                               int group_size, const void* bias, const void* residual, void* y,
                               int y_f32, int M, int N, int K, int path, void* stream);

/* One projection of a shared-input int8 launch (device.h:391-398). */
typedef struct vv_i8_proj {
    const void* w;     /* W8: int8 [N][K]; W4: accelerator-layout codes [N][K/2] */
    const void* sw;    /* W8: FP32 [N] */
    const void* sz;    /* W4: half2 {scale, zero} [N][K/group_size] */
    const void* bias;  /* FP16 [N] or NULL */
    void*       y;     /* FP16 [M][N] */
    int         N;
} vv_i8_proj_t;

/* Several projections of one int8 input (q/k/v, gate/up), each computed exactly
 * as vv_w8a8_linear_dev (w4 == 0; x_layout must be 0) or vv_w4a8_linear_dev
 * (w4 != 0, path AUTO) would. replaces device.h:411-414
 * (src/cuda/gemm_i8.cu:616-645). */
vv_status_t vv_i8_linear_multi_dev(const int8_t* xq, int x_layout, const float* sx,
                                   const int32_t* xsum, int w4, const vv_i8_proj_t* projs,
                                   int n, int group_size, int M, int K, void* stream);

/* ── W4A16 linear layers ───────────────────────────────────────────────── */

/* INT4 group-affine weights in the accelerator layout (vv_int4g_to_gpu_layout,
 * src/quant/awq_repack.c:261-310): packed [N][K/2], sz half2 {scale, zero}
 * [N][K/group_size], group_size one of 32, 64, 128, 256, K % 32 == 0 (the
 * reference asks K % 64 for its tensor-core path and N % 8; neither is needed
 * here). Every kernel dequantises with w = (q - z) * s rounded once to FP16
 * (device.h:233) and accumulates in FP32; the bias is added in FP32 before the
 * one rounding of the output. Other shapes or unaligned pointers:
 * VV_ERR_UNSUPPORTED. */

/* y[N] = W . x (+ bias) for one token; no allocation, no per-token host
 * arguments. replaces device.h:247-249 (src/cuda/w4a16.cu:848-856). */
vv_status_t vv_w4a16_gemv_dev(const void* x, const void* packed, const void* sz,
                              const void* bias, void* y, int N, int K, int group_size,
                              void* stream);
/* One projection of a fused GEMV (device.h:252-258). */
typedef struct vv_w4a16_proj {
    const void* packed;
    const void* sz;
    const void* bias;   /* FP16 [N] or NULL */
    void*       y;      /* FP16 [N] */
    int         N;
} vv_w4a16_proj_t;
/* Up to three GEMVs of the same x in ONE launch (q/k/v, gate/up); each row
 * exactly as vv_w4a16_gemv_dev over the combined row count would compute it.
 * replaces device.h:266-268 (src/cuda/w4a16.cu:858-879). */
vv_status_t vv_w4a16_gemv_multi_dev(const void* x, const vv_w4a16_proj_t* projs, int n_proj,
                                    int K, int group_size, void* stream);
/* out[m][j] = x[m][perm[j]] (FP16, K % 8 == 0, perm 16-byte aligned): the
 * column order of an act-order checkpoint. replaces device.h:275-277. */
vv_status_t vv_w4a16_gather_dev(const void* x, const int32_t* perm, void* out, int M, int K,
                                void* stream);
/* C[M,N] = A[M,K] . W^T (+ bias). M <= 4: the GEMV kernel; to 64 rows: codes
 * straight into 16x16x32 MFMA operands, K split over a workgroup's waves;
 * larger M (or wide layers beyond 16 rows): LDS-tiled FP16 MFMA with the
 * codes dequantised on their way into LDS; from 1024 rows,
 * when `scratch` holds N * K * 2 bytes: the weight dequantised there once, then
 * vv_gemm_fp16_dev started from the bias. `scratch` may be NULL (no split-K
 * partials are ever needed). replaces device.h:288-291
 * (src/cuda/w4a16.cu:894-932). */
vv_status_t vv_w4a16_gemm_dev(const void* A, const void* packed, const void* sz,
                              const void* bias, void* C, void* scratch, size_t scratch_bytes,
                              int M, int N, int K, int group_size, void* stream);
/* Accelerator-layout INT4 -> dense FP16 [N,K]. replaces device.h:294-296. */
vv_status_t vv_w4a16_dequant_dev(const void* packed, const void* sz, void* out_fp16, int N,
                                 int K, int group_size, void* stream);

/* ── The older weight-only formats on FP16 activations ─────────────────── */

/* NF4 (bitsandbytes): codes [N*K/2], the high nibble of a byte the even
 * element; FP16 absmax per 64 flat elements [N*K/64]; w = book[code] * absmax
 * rounded once to FP16 wherever a kernel needs the FP16 weight. */
/* y[N] = W x (+ bias), one row. K % 32 == 0 (the reference asks K % 256 == 0).
 * The code book is met in FP16 and the block's absmax applied to the FP32
 * partial sum. replaces device.h:168-170 (nf4_gemv.cu:44-90). */
vv_status_t vv_nf4_gemv_dev(const void* x, const uint8_t* packed, const void* scales,
                            const void* bias, void* y, int N, int K, void* stream);
/* M <= 8 (K % 32 == 0): the one-row kernel over up to eight rows, no scratch.
 * 9..64 rows: the small-M MFMA kernel where vv_skinny_linear_dev serves the
 * shape, else the tile kernel with the weight dequantised on its way in; no
 * scratch either way. Otherwise the weight is dequantised into temp_weight_fp16
 * [N][K] (NULL there: VV_ERR_NULL_PTR) and vv_gemm_fp16_dev runs; the last two
 * give the same bits. block_size must be 64. replaces device.h:174-178
 * (gemm.cu:468-500). */
vv_status_t vv_nf4_gemm_dev(const void* input_fp16, const uint8_t* weight_packed,
                            const void* weight_scales_fp16, void* output_fp16,
                            void* temp_weight_fp16, int M, int N, int K, int block_size,
                            void* stream);
/* n_elements % 8 == 0, block_size 64. replaces device.h:181-183
 * (dequant_nf4.cu:40-66, 117-147). */
vv_status_t vv_dequant_nf4_dev(const uint8_t* packed, const void* scales_fp16, void* output_fp16,
                               int n_elements, int block_size, void* stream);

/* INT4 group-affine in the row-major form (vv_awq_repack): codes [N][K/2], high
 * nibble = even column; FP16 scales and mins [N][K/G], G in {32, 64, 128, 256};
 * w = q * scale + min. `packed` and `mins` are typed as the reference types
 * them; they are byte and FP16 arrays. */
/* One row; K % 32 == 0. replaces device.h:193-196 (awq_gemv.cu:33-72). */
vv_status_t vv_awq_gemv_dev(const void* x, const uint32_t* packed, const uint32_t* mins,
                            const void* scales, const void* bias, void* y, int N, int K,
                            int group_size, void* stream);
/* M <= 8 and K % 32 == 0: the one-row kernel; 9..64 rows: the small-M MFMA
 * kernel or the tile kernel with the weight dequantised on its way in (no
 * scratch); else dequantise into
 * temp_weight_fp16 + vv_gemm_fp16_dev (the same bits). replaces device.h:199-202
 * (awq_gemv.cu:213-238). */
vv_status_t vv_awq_gemm_dev(const void* input_fp16, const uint32_t* packed, const uint32_t* mins,
                            const void* scales, void* output_fp16, void* temp_weight_fp16,
                            int M, int N, int K, int group_size, void* stream);
/* replaces device.h:205-207 (awq_gemv.cu:125-153). */
vv_status_t vv_dequant_awq_dev(const uint32_t* packed, const uint32_t* mins, const void* scales,
                               void* output_fp16, int N, int K, int group_size, void* stream);

/* Per-channel INT8: q [N][K], FP32 scale per row, w = q * scale; K % 16 == 0. */
/* One row: sum q x in FP32 (the codes as exact FP16 integers), scale and bias
 * once per output. replaces device.h:216-218 (int8_gemv.cu:72-101). */
vv_status_t vv_int8_gemv_dev(const void* x, const int8_t* q, const float* scales,
                             const void* bias, void* y, int N, int K, void* stream);
/* M <= 8 the one-row kernel, 9..64 the small-M MFMA kernel where it serves, else
 * the tile kernel with the weight dequantised on its way in (no scratch either
 * way), above that dequantise + vv_gemm_fp16_dev; all of the last three give
 * the same bits. No bias. replaces device.h:223-226 (int8_gemv.cu:194-223). */
vv_status_t vv_int8_gemm_dev(const void* input_fp16, const int8_t* q, const float* scales,
                             void* output_fp16, void* temp_weight_fp16, int M, int N, int K,
                             void* stream);
/* replaces device.h:229-231 (int8_gemv.cu:139-160, 179-192). */
vv_status_t vv_dequant_int8_dev(const int8_t* q, const float* scales, void* output_fp16, int N,
                                int K, void* stream);

/* ── Batched, streaming Conv-VAE encoder ops ────────────────────────────── */

/* Activations are FP16, channel-first and packed along time: the items of one
 * launch sit side by side in one [C][ld] buffer. Only convolutions look back
 * in time; they take the item boundaries and each item's streaming context
 * from a descriptor passed by value. No result depends on where an item sits
 * in the packed axis or on how a stream was cut into chunks: every output adds
 * its products in one fixed order. device.h:722-755. */
#define VV_VAE_MAX_ITEMS 32
typedef struct vv_vae_conv_item {
    int64_t     in_off;    /* first input column in the packed input */
    int64_t     out_off;   /* first output column in the packed output */
    const void* in_ptr;    /* the item's own input, overriding in_off */
    const void* tail_in;   /* [in_ch][cap] left context; NULL = zeros */
    void*       tail_out;  /* [in_ch][cap] receives the next context */
    void*       out_ptr;   /* transposed output: rows [frame][out_ld] */
    int         in_len;    /* input columns this chunk */
    int         out_len;   /* output columns this chunk */
    int         have;      /* context columns in front of the input */
    int         keep;      /* context columns to leave for the next chunk */
    int         out_ld;    /* transposed output row stride, elements */
    int         skip;      /* leading output frames not written */
} vv_vae_conv_item_t;
typedef struct vv_vae_conv_desc {
    int                n;
    int                cap;   /* context stride per channel, columns */
    vv_vae_conv_item_t it[VV_VAE_MAX_ITEMS];
} vv_vae_conv_desc_t;

/* Causal conv (groups = 1) over every item: y[oc][t] = sum over (in channel,
 * tap) in that order of w[oc][ic][kk] * in[ic][t * stride + kk], an FP32 fused
 * multiply-add chain from zero, plus the bias, rounded once to FP16. Position p
 * of an item's input is column p of [context ++ input]; past the end is zero.
 * `transposed`: rows [frame][out_ch] at each item's out_ptr instead of packed.
 * replaces device.h:762-765 (vae_kernels.cu:50-89, 736-755). */
vv_status_t vv_vae_conv_dev(const vv_vae_conv_desc_t* d, const void* x, int64_t ld_in,
                            const void* w, const void* b, void* y, int64_t ld_out,
                            int in_ch, int out_ch, int k, int stride, bool transposed,
                            void* stream);
/* The last `keep` columns of [context ++ input] of every item into its
 * tail_out. replaces device.h:768-769 (vae_kernels.cu:95-116, 756-765). */
vv_status_t vv_vae_tail_dev(const vv_vae_conv_desc_t* d, const void* x, int64_t ld_in,
                            int in_ch, void* stream);
/* 1 / rms over the channels of every packed column into rinv[0..T), and of
 * every context column of the items in d (may be NULL) into
 * rinv[T + item * cap + j]. replaces device.h:775-777 (vae_kernels.cu:286-318,
 * 766-781). */
vv_status_t vv_vae_rms_dev(const void* x, int64_t ld, int64_t T, int C, float eps, float* rinv,
                           const vv_vae_conv_desc_t* d, void* stream);
/* xout = xin + gamma * (depthwise conv(rmsnorm(xin)) + bias), with an FP16
 * rounding wherever separate kernels would have stored one. k <= 16.
 * replaces device.h:783-787 (vae_kernels.cu:320-392, 782-800). */
vv_status_t vv_vae_mixer_dev(const vv_vae_conv_desc_t* d, const void* xin, void* xout,
                             int64_t ld, const float* rinv, int64_t T_total,
                             const void* norm_w, const void* conv_w, const void* conv_b,
                             const void* gamma, int C, int k, void* stream);
#define VV_VAE_EPI_BIAS_GELU  0  /* C = gelu(half(half(A B) + bias)) */
#define VV_VAE_EPI_BIAS_RESID 1  /* C = half(C + half(half(A B) + bias) * gamma), in place */
#define VV_VAE_EPI_BIAS       2  /* C = half(A B + bias), one rounding */
/* col[ic * k + kk][q] = what tap kk of input channel ic sees for packed output
 * column p0 + q. replaces device.h:802-805 (vae_kernels.cu:118-147, 934-946). */
vv_status_t vv_vae_im2col_dev(const vv_vae_conv_desc_t* d, const void* x, int64_t ld_in,
                              int in_ch, int k, int stride, int64_t p0, int pc, void* col,
                              int64_t ldcol, void* stream);
/* y = w [out_ch][K] x col + b in FP32 fused multiply-adds in K order from
 * zero: bit-identical to vv_vae_conv_dev. y NULL writes the transposed rows of
 * the items in d. `tile` (0, 16, 32, 64) is accepted and changes no bit.
 * replaces device.h:819-822 (vae_kernels.cu:149-284, 906-933). */
vv_status_t vv_vae_conv_gemm_dev(const vv_vae_conv_desc_t* d, const void* w, const void* col,
                                 int64_t ldcol, const void* b, void* y, int64_t ld_out,
                                 int out_ch, int K, int64_t p0, int pc, int tile,
                                 void* stream);
/* C[M,P] (stride ldc) from A[M,K] x B[K,P] (stride ldb) on the matrix cores,
 * FP32 accumulation in K order; rinv and norm_w (both or neither) normalise B
 * on its way in: half(B[k][p] * rinv[p] * norm_w[k]). `tile`: 64 or 128 (the
 * workgroup's output tile edge) or 0 to choose by the grid; it changes no bit. replaces device.h:835-839 (vae_kernels.cu:394-607, 868-905). */
vv_status_t vv_vae_gemm_nn_dev(int epilogue, const void* A, const void* B, int64_t ldb, void* C,
                               int64_t ldc, int M, int K, int P, const void* bias,
                               const void* gamma, const float* rinv, const void* norm_w,
                               int tile, void* stream);
#define VV_VAE_ROWS_PLAIN        0  /* C[r][c], stride ldc */
#define VV_VAE_ROWS_STORE        1  /* segment rows, as computed */
#define VV_VAE_ROWS_STORE_TRUNC  2  /* segment rows, FP16 by truncation, subnormals flushed */
#define VV_VAE_ROWS_ACC_TRUNC    3  /* segment rows += value, truncated */
typedef struct vv_vae_row_seg {
    int   row0;   /* first packed row of this segment */
    int   ld;     /* destination row stride, elements */
    void* dst;
} vv_vae_row_seg_t;
typedef struct vv_vae_rows {
    int              mode;
    int              n;
    vv_vae_row_seg_t seg[VV_VAE_MAX_ITEMS];
} vv_vae_rows_t;
/* C[M,N] = half(half(A[M,K] (stride lda) x B[N,K]^T) + bias), rows scattered per
 * `rows` (NULL = plain). replaces device.h:863-866 (vae_kernels.cu:609-712,
 * 947-970). */
vv_status_t vv_vae_gemm_tn_dev(const void* A, int64_t lda, const void* B, void* C, int64_t ldc,
                               int M, int N, int K, const void* bias,
                               const vv_vae_rows_t* rows, void* stream);
/* FP32 -> FP16 with a 64-bit count. replaces device.h:869-870. */
vv_status_t vv_vae_f32_to_f16_dev(const float* in, void* out, int64_t n, void* stream);

/* C[M,P] = alpha * A[M,K] x B[K,P] + beta * C, all row-major FP16, FP32
 * accumulation on the matrix cores; beta == 0 never reads C.
 * replaces device.h:477-479 (gemm.cu:441-460). */
vv_status_t vv_gemm_fp16_nn_dev(const void* A, const void* B, void* C, int M, int K, int P,
                                float alpha, float beta, void* stream);
/* No handle to release. replaces device.h:482. */
void vv_gemm_cleanup(void);

/* ── BitNet integer layers (include/vibevoice/bitnet.h numerics) ───────── */

/* Per-token int8: s = (float)(127 / max(max|x|, 1e-5)) in double, q = the
 * integer fma(x, s, 1.5 * 2^23) carries (the product is never rounded on its
 * own), clamped to [-128, 127]. x FP16 (x_f16 != 0) or FP32 [M][K]; scale [M];
 * sum [M] = row sums of q, or NULL. Bit-identical to vv_act_quant_i8_cpu.
 * replaces device.h:898-900 (bitnet.cu:44-93). */
vv_status_t vv_act_quant_i8_dev(const void* x, int x_f16, int M, int K, int8_t* q,
                                float* scale, int32_t* sum, void* stream);
/* Ternary (I2_S codes [N][K/4], K % 128 == 0) x int8: acc = sum_k (c - 1) q
 * exactly, and y = ((float)acc / x_scale[m]) * w_scale (+ bias[n]), each step
 * rounded on its own; y FP16 (y_f16) or FP32; acc and y may each be NULL. All
 * row counts run one MFMA kernel. replaces device.h:916-920 (bitnet.cu:138-178,
 * 470-497). */
vv_status_t vv_ternary_gemm_dev(const int8_t* q, const int32_t* xsum, const float* x_scale,
                                const uint8_t* codes, float w_scale, const float* bias,
                                int32_t* acc, void* y, int y_f16, int M, int N, int K,
                                void* stream);
/* int8 x int8: acc = sum_k w a exactly, and y = (float)acc * (w_scale /
 * *a_scale) (+ bias[n]) with max |y| folded into *absmax (device float that
 * must start at 0). Any K; K % 16 != 0 or operands off 16 bytes take a scalar
 * kernel. replaces device.h:928-931 (bitnet.cu:180-222, 499-530). */
vv_status_t vv_i8_gemm_dev(const int8_t* a, const float* a_scale, const int8_t* w, float w_scale,
                           const float* bias, int32_t* acc, float* y, float* absmax, int M,
                           int N, int K, void* stream);
/* q = rne(clamp(y * (127 / *absmax), relu ? 0 : -127, 127)); *out_scale = 127 /
 * *absmax (0 when *absmax is 0). replaces device.h:938-940 (bitnet.cu:369-382). */
vv_status_t vv_i8s_requant_dev(const float* y, int64_t n, const float* absmax, int relu,
                               int8_t* q, float* out_scale, void* stream);
/* Scratch for vv_i8_head_argmax_dev. replaces device.h:943 (bitnet.cu:545-548). */
size_t vv_i8_head_argmax_scratch_bytes(int V);
/* logit_n = ((float)(w_n . q) * w_scale[n]) / *scale; the largest wins, ties to
 * the lowest index. K % 4 == 0. replaces device.h:952-955 (bitnet.cu:384-455,
 * 549-563). */
vv_status_t vv_i8_head_argmax_dev(const int8_t* q, const float* scale, const int8_t* w,
                                  const float* w_scale, int V, int K, int32_t* token,
                                  float* value, void* scratch, void* stream);

/* ── Dense linear layers ───────────────────────────────────────────────── */

/* C[M,N] = alpha * A[M,K] * B[N,K]^T + beta * C; A, B, C FP16 row-major, FP32
 * accumulation on the matrix cores. beta == 0 never reads C. M == 1 streams
 * the weight rows once (one wave per output column); 2 <= M <= 64 feeds them
 * from global memory straight into the MFMA operands with K split over a
 * workgroup's waves; larger M runs 128x128 or 256x256 workgroup tiles (64x64
 * when there are too few of those), all of which add K in the same order and
 * so give the same bits for an element. K % 8 != 0 or A/B off 16 bytes take a
 * scalar kernel. M <= 0 or N <= 0: VV_OK, nothing launched.
 * replaces device.h:423-425 (src/cuda/gemm.cu). */
vv_status_t vv_gemm_fp16_dev(const void* A, const void* B, void* C, int M, int N,
                             int K, float alpha, float beta, void* stream);
/* One projection of a small-M launch: device.h:453-459. */
typedef struct vv_skinny_proj {
    const void* w;        /* format 0: FP16 [N][K]; 1: int8 [N][K]; 2: NF4 codes [N][K/2] */
    const void* scales;   /* 1: FP32 [N]; 2: FP16 absmax [N*K/64]; 0: unused */
    const void* bias;     /* FP16 [N] or NULL */
    void*       y;        /* FP16 [M][N] output */
    int         N;
} vv_skinny_proj_t;
/* y_i = alpha * A[M,K] . W_i^T (+ bias_i) for up to three projections of the
 * same A (q/k/v, gate/up) in one launch, M in 9..64; dense FP16 (format 0),
 * per-channel INT8 (1) or NF4 (2) weights, the quantised ones dequantised in
 * registers to the bits vv_dequant_int8_dev / vv_dequant_nf4_dev write. The
 * result equals dequantising, vv_gemm_fp16_dev (or vv_gemm_fp16_tile_dev) and
 * vv_bias_add_dev bit for bit. Other formats, other M, K % 8 != 0, or a projection wide
 * enough that vv_gemm_fp16_dev would tile it (N >= 12800 above 16 rows):
 * VV_ERR_UNSUPPORTED, nothing launched; the caller runs that path itself
 * (src/inference/decoder.c:375-378, 499-505). replaces device.h:472-475. */
vv_status_t vv_skinny_linear_dev(const void* A, int format,
                                 const vv_skinny_proj_t* projs, int n_proj,
                                 int M, int K, float alpha, void* stream);
/* The LDS-tiled kernel alone (128x128 tile), whatever M — except for 9..64
 * rows, where it runs what vv_gemm_fp16_dev runs: the reference holds its
 * small-M entry point to this one bit for bit (device.h:464-468), and the
 * weight-streaming kernel that serves those rows here adds K in its own order.
 * replaces device.h:432-434. */
vv_status_t vv_gemm_fp16_tile_dev(const void* A, const void* B, void* C, int M,
                                  int N, int K, float alpha, float beta,
                                  void* stream);

/* ── Attention over an FP16 KV cache ───────────────────────────────────── */

/* One layer of a KV cache as the attention kernels see it: k, v are
 * [row][n_kv_heads][head_dim] FP16, row = position, or with a (device)
 * page_table position t lives at row page_table[t / 64] * 64 + t % 64.
 * Same layout as device.h:527-536. */
typedef struct vv_kv_view {
    const void* k;
    const void* v;
    const void* k_meta;       /* TurboQuant formats: FP16 RMS per stored vector [rows][n_kv_heads] */
    const void* v_meta;
    const int*  page_table;   /* device memory, or NULL */
    int         format;       /* vv_kv_format_t 0..6: FP16, FP8 E4M3 / E5M2, TurboQuant 4 / 3 / 2 / 1.5 bits */
    int         n_kv_heads;
    int         head_dim;
} vv_kv_view_t;

/* The backend a context should name (never VV_ATTN_AUTO = 0). All backend
 * names run the same kernels here; a packed format at a head_dim other than
 * 128 answers VV_ATTN_FA1 (1) and the attention calls then decline.
 * replaces device.h:545-546 (src/cuda/attention_fi.cu:554-583). */
int vv_attn_resolve(int requested, int kv_format, bool paged, int n_q_heads,
                    int n_kv_heads, int head_dim);
/* n_q_heads * 2048 * (head_dim + 4) floats: room for the decode slices' partial
 * states (256 per head) and for the partial states of a short prefill split
 * over the keys (rows x key runs <= 2048 per head); one buffer per context.
 * replaces device.h:554 (attention_fi.cu:585-589). */
size_t vv_attn_scratch_bytes(int n_q_heads, int n_kv_heads, int head_dim);
/* The number of slices the decode splits `cache_len` positions into: 16 up to
 * 1024 positions, then 32, 64, 128, 256, doubling as the length passes 1024,
 * 2048, 4096, 8192. A captured decode step is valid while this stays equal.
 * replaces device.h:562-563. */
int vv_attn_decode_shape(int backend, int n_q_heads, int n_kv_heads, int cache_len);
/* q_len query rows at absolute positions q_offset.. against the first kv_len
 * positions of the cache; Q, O [q_len][n_q_heads][head_dim] FP16; causal:
 * query p sees positions <= p. head_dim 128 with 16-byte aligned pointers
 * runs on the matrix cores, any other head_dim <= 256 a wave per row.
 * scratch (vv_attn_scratch_bytes() of device memory, 16-byte aligned, or NULL):
 * with it, few rows against many keys on an FP16 cache (fewer workgroups than
 * fill the chip, at least sixteen 64-key tiles) are split over the keys into
 * up to 16 runs whose partial states a second launch folds - the same values
 * to the rounding of the runs' partial sums; without it every call is one launch.
 * A format other than FP16, head_dim > 256 or n_q_heads % n_kv_heads != 0:
 * VV_ERR_UNSUPPORTED. replaces device.h:575-578 (attention_fi.cu:600-632). */
vv_status_t vv_attn_prefill(int backend, const void* q, const vv_kv_view_t* kv,
                            void* out, int n_q_heads, int q_len, int q_offset,
                            int kv_len, bool causal, void* scratch, void* stream);
/* One query row per head against the whole cache. cache_len sizes the launch;
 * d_cache_len (device int, or NULL) holds the exact length and need only be in
 * the same vv_attn_decode_shape() bucket. scratch: vv_attn_scratch_bytes()
 * of device memory owned by the caller.
 * replaces device.h:586-589 (attention_fi.cu:634-660). */
vv_status_t vv_attn_decode(int backend, const void* q, const vv_kv_view_t* kv,
                           void* out, int n_q_heads, int cache_len,
                           const int* d_cache_len, void* scratch, void* stream);
/* vv_attn_decode without the scratch argument, for callers that cannot
 * allocate device memory (code under graph capture, tight serving loops,
 * harnesses that forbid hipMalloc): the slices' partial states live in a
 * file-scope device array of the library, 8.25 MiB per GPU, held until the
 * process ends. It calls no hipMalloc, hipFree or other allocating routine.
 * Same arguments, results (bit for bit) and status codes as vv_attn_decode;
 * additionally VV_ERR_INVALID_ARG when the split path would need more than
 * VV_ATTN_DECODE_STATIC_MAX_Q_HEADS query heads of partial states, and
 * VV_ERR_CUDA when the array's address cannot be resolved or the stream belongs
 * to another device than the current one (each GPU has its own array, and the
 * current device's is the one the call can name). All calls on one
 * GPU share that GPU's array: calls that overlap on one GPU (two streams, two
 * threads) race, so serialise them or use vv_attn_decode with a buffer per
 * context. The array's address is resolved at the first call on each device:
 * make that call outside a graph capture. No counterpart in the reference. */
#define VV_ATTN_DECODE_STATIC_MAX_Q_HEADS 64
vv_status_t vv_attn_decode_static(int backend, const void* q, const vv_kv_view_t* kv,
                                  void* out, int n_q_heads, int cache_len,
                                  const int* d_cache_len, void* stream);
/* The older entry points for raw FP16 caches: the cache as two pointers
 * instead of a view, otherwise vv_attn_scratch_bytes (the decode's 256 slices per
 * head alone: these prefill forms take no scratch), vv_attn_decode_shape,
 * vv_attn_decode and vv_attn_prefill. replace device.h:621-655. */
size_t vv_gqa_decode_scratch_bytes(int n_q_heads, int head_dim);
int vv_gqa_decode_shape(int cache_len);
vv_status_t vv_gqa_attention_decode_dev(const void* q, const void* k_cache,
                                        const void* v_cache, void* output,
                                        int n_q_heads, int n_kv_heads, int head_dim,
                                        int cache_len, const int* d_cache_len,
                                        void* scratch, void* stream);
vv_status_t vv_gqa_attention_prefill_cached_dev(const void* q, const void* k_cache,
                                                const void* v_cache, void* output,
                                                int n_q_heads, int n_kv_heads,
                                                int head_dim, int q_len, int q_offset,
                                                int kv_len, bool causal, void* stream);
vv_status_t vv_gqa_attention_prefill_dev(const void* q, const void* k, const void* v,
                                         void* output, int n_q_heads, int n_kv_heads,
                                         int head_dim, int seq_len, bool causal,
                                         void* stream);
/* Write K/V rows [n_positions][n_kv_heads][head_dim] into a cache layer at
 * positions pos.. (or *d_pos..), through page_table when it is set. FP16: a
 * copy. FP8 (E4M3 / E5M2, head_dim 128): each value encoded in integer
 * arithmetic exactly as src/cuda/kv_codec.cuh:66-128 (round to nearest even,
 * saturating, NaN -> 0); when k_ref is set the head's reference key is
 * subtracted from K first (softmax does not see a shift common to all keys),
 * and with build_ref it is first computed as this run's mean key. TurboQuant
 * (4 / 3 / 2 / 1.5 bits, head_dim 128): the vector, minus the reference key,
 * goes through the randomised Hadamard transform, its RMS goes to k_meta /
 * v_meta [rows][n_kv_heads] as FP16, and each value (pair) takes the code of
 * the nearest Lloyd-Max level (code word) of value / RMS
 * (src/cuda/kv_quant.cu:86-119). replaces device.h:597-602
 * (src/cuda/kv_quant.cu:507-552). */
vv_status_t vv_kv_store_dev(const void* k_fp16, const void* v_fp16, void* k_store,
                            void* v_store, void* k_meta, void* v_meta, void* k_ref,
                            bool build_ref, int n_kv_heads, int head_dim, int pos,
                            const int* d_pos, int n_positions, int kv_format,
                            const int* page_table, void* stream);
/* The same without a page table, quantised formats only (FP16:
 * VV_ERR_UNSUPPORTED). replaces device.h:689-694 (kv_quant.cu:554-567). */
vv_status_t vv_kv_quant_store_dev(const void* k_fp16, const void* v_fp16, void* k_store,
                                  void* v_store, void* k_meta, void* v_meta, void* k_ref,
                                  bool build_ref, int n_kv_heads, int head_dim, int pos,
                                  const int* d_pos, int n_positions, int kv_format, void* stream);
/* A packed store [n_pos][n_kv_heads][bytes per vector] back to FP16 in the
 * ORIGINAL space: unpacked, for TurboQuant un-rotated, plus `ref`
 * [n_kv_heads][128] when given, rounded once. For inspection and offload, not
 * the hot path. replaces device.h:697-699 (kv_quant.cu:311-338, 586-603). */
vv_status_t vv_kv_dequant_dev(const void* store, const void* meta, const void* ref,
                              void* out_fp16, int n_kv_heads, int head_dim, int n_pos,
                              int kv_format, void* stream);
/* Attention over a quantised cache given as pointers: vv_attn_decode /
 * vv_attn_prefill with the format in the view. The codes are widened to FP16
 * on their way into the tile, so the result is, bit for bit, that of an FP16
 * cache holding the unpacked vectors (FP8: what vv_kv_dequant_dev returns;
 * TurboQuant: RMS times level, still rotated). A TurboQuant cache holds
 * rotated vectors: rotate Q before and un-rotate the output after.
 * replace device.h:662-675 (kv_quant.cu:605-673). */
vv_status_t vv_gqa_attention_decode_q_dev(const void* q, const void* k_store, const void* v_store,
                                          const void* k_meta, const void* v_meta, void* output,
                                          int n_q_heads, int n_kv_heads, int head_dim,
                                          int cache_len, const int* d_cache_len, int kv_format,
                                          void* scratch, void* stream);
vv_status_t vv_gqa_attention_prefill_q_dev(const void* q, const void* k_store, const void* v_store,
                                           const void* k_meta, const void* v_meta, void* output,
                                           int n_q_heads, int n_kv_heads, int head_dim, int q_len,
                                           int q_offset, int kv_len, bool causal, int kv_format,
                                           void* stream);
/* In-place randomised Hadamard transform of [rows][n_heads][128] FP16 (the
 * orthogonal map TurboQuant stores K and V under: dot(Hq, Hk) == dot(q, k)) and
 * its inverse. replace kv_quant.h:96-101 (kv_quant.cu:171-199, 569-584). */
vv_status_t vv_kv_rotate_dev(void* x_fp16, int n_heads, int head_dim, int rows, void* stream);
vv_status_t vv_kv_unrotate_dev(void* x_fp16, int n_heads, int head_dim, int rows, void* stream);
/* page_table[first + i] = pages[i], i < n, ordered on the stream; `pages` is
 * host memory, consumed before the call returns. replaces device.h:610-611. */
vv_status_t vv_kv_page_map_dev(int* page_table, int first, int n, const int* pages,
                               void* stream);

/* ── LM head ───────────────────────────────────────────────────────────── */

/* logits[V] = W[V,K] x[K]; x, W FP16, FP32 accumulation, FP32 logits. Bound by
 * the table bytes: one wave per vocabulary row streams it once.
 * replaces device.h:706-707 (src/cuda/lm_head.cu:139-152). */
vv_status_t vv_lm_head_gemv_dev(const void* x, const void* W, void* logits, int V,
                                int K, void* stream);
/* Greedy argmax over FP32 logits on the device, two launches; scratch_v
 * (FP32) and scratch_i (int32) hold 256 partial winners each; out_token int32,
 * out_value FP32 or NULL. The lowest index among equal maxima wins (the CPU
 * sampler's in-order scan, src/cpu/cpu_kernels.c:1613-1623); a NaN never wins.
 * replaces device.h:710-712 (lm_head.cu:163-183). */
vv_status_t vv_argmax_dev(const void* logits, int V, void* scratch_v, void* scratch_i,
                          void* out_token, void* out_value, void* stream);

/* ── Fused forms (additions) ───────────────────────────────────────────── */

/* addition: vv_residual_add_dev(residual, x) followed by
 * vv_rmsnorm_dev(residual, weight, normed) in one pass over the rows — the
 * adjacent calls at src/inference/decoder.c:950-960 and :988 -> :810. The
 * updated residual (bit-identical to the two-call sequence) is written back in
 * place and the norm reads that rounded FP16 value, as the two calls would.
 * 8*T*H bytes of traffic instead of 10*T*H. */
vv_status_t vv_add_rmsnorm_dev(void* residual, const void* x, const void* weight,
                               void* normed, int seq_len, int hidden_size,
                               float eps, void* stream);

/* addition: vv_rope_dev on Q [seq_len, n_q_heads, head_dim] and on
 * K [seq_len, n_kv_heads, head_dim] in one launch (decoder.c:850-855), the
 * cosine/sine of a position computed once and shared by all heads of both.
 * Either of q, k may be NULL (its head count is then ignored). */
vv_status_t vv_rope_qk_dev(void* q, void* k, int seq_len, int n_q_heads,
                           int n_kv_heads, int head_dim, int position_offset,
                           const int* d_position, float theta, void* stream);

/* addition: vv_bias_add_dev on Q and K followed by vv_rope_qk_dev — the
 * projection epilogue of decoder.c:825-855 (bias, then rotation) in one pass.
 * The biased value is rounded to FP16 before it is rotated, as the two calls
 * would. q_bias [n_q_heads*head_dim], k_bias [n_kv_heads*head_dim]; either
 * may be NULL (no bias for that tensor). */
vv_status_t vv_bias_rope_qk_dev(void* q, void* k, const void* q_bias,
                                const void* k_bias, int seq_len, int n_q_heads,
                                int n_kv_heads, int head_dim, int position_offset,
                                const int* d_position, float theta, void* stream);

/* addition: the cosines and sines of seq_len consecutive positions, computed once for
 * every layer that rotates at those positions (src/inference/decoder.c:850-855 runs
 * the same rotation in each of the 28 layers): table[row][i] = {cos, sin} of
 * (float)(first + row) * theta^(-2i/head_dim), i < head_dim/2, as FP32 pairs
 * (8 * seq_len * head_dim/2 bytes; a table that is not 16-byte aligned is
 * VV_ERR_UNSUPPORTED, the status its readers return for one), first = *d_position
 * when d_position is given, else position_offset. The angle and the full-range
 * sincosf are those of vv_rope_dev, so a rotation that reads the table gives its
 * bits. vv_gemm_bias_rope_dev and vv_gemm_qkv_rope_dev read rows of 64 pairs: they
 * need a table built with head_dim == 128. */
vv_status_t vv_rope_table_dev(void* table, int seq_len, int head_dim, int position_offset,
                              const int* d_position, float theta, void* stream);

/* addition: a rotary projection in ONE launch, the q or k leg of decoder.c:825-855
 * (vv_gemm_fp16_dev, vv_bias_add_dev, vv_rope_dev) with the bias and the rotation
 * done in the GEMM's store: C[M, n_heads*head_dim] = rope(fp16(A[M,K] W[N,K]^T) +
 * bias), row m rotated by row m of a vv_rope_table_dev table. Each step rounds to
 * FP16 where the separate calls store, so the result equals vv_gemm_fp16_dev then
 * vv_bias_rope_qk_dev bit for bit, and the projection is written once instead of
 * written, read and written again. bias may be NULL. head_dim must be 128 and C,
 * bias and the table 16-byte aligned (else VV_ERR_UNSUPPORTED, nothing launched);
 * up to 64 rows, K % 8 != 0 or unaligned A / W run the two steps one after the other. */
vv_status_t vv_gemm_bias_rope_dev(const void* A, const void* W, const void* bias, void* C,
                                  int M, int n_heads, int head_dim, int K,
                                  const void* rope_table, void* stream);

/* addition: the q, k and v projections of a prefill chunk in ONE launch - the whole of
 * decoder.c:815-867 on the dense FP16 path (quant_linear_group :478-505 = three
 * vv_gemm_fp16_dev + vv_bias_add_dev, vv_rope_dev twice :849-855, the KV append
 * :864-867): q[M, n_q_heads*128] = rope(fp16(x Wq^T) + bq), k likewise with Wk / bk,
 * v[M, n_kv_heads*128] = fp16(x Wv^T) + bv, row m rotated by row m of a
 * vv_rope_table_dev table (built with head_dim 128 for the chunk's positions). With
 * k_cache / v_cache (FP16 [positions][n_kv_heads][128], contiguous or behind a table
 * of 64-position pages) the k and v rows also land at positions first .. first+M-1,
 * first = *d_pos when d_pos is given, else pos; k and v may then be NULL. Every step
 * rounds to FP16 where the separate calls store: the result equals
 * vv_gemm_bias_rope_dev (q), vv_gemm_bias_rope_dev (k), vv_gemm_fp16_dev +
 * vv_bias_add_dev (v) and vv_kv_store_dev bit for bit. One grid of equal tiles serves
 * 7 query heads per KV head with head_dim 128 (28 + 4 heads: a tile is one q or k head
 * plus 16 columns of v), more than 64 rows, K % 64 == 0; other shapes run the separate
 * calls through k and v (VV_ERR_UNSUPPORTED if those are NULL) - 2 .. 64 rows, a streaming
 * chunk, as three launches: the three projections with their biases in one launch of the
 * small-M kernel, one rotation of q and k, the append. Biases may be NULL.
 * q, k, v, the caches, the biases and the table must be 16-byte aligned
 * (VV_ERR_UNSUPPORTED otherwise, nothing launched). */
vv_status_t vv_gemm_qkv_rope_dev(const void* x, const void* wq, const void* wk, const void* wv,
                                 const void* bq, const void* bk, const void* bv, void* q,
                                 void* k, void* v, int M, int n_q_heads, int n_kv_heads,
                                 int head_dim, int K, const void* rope_table, void* k_cache,
                                 void* v_cache, const int* page_table, int pos,
                                 const int* d_pos, void* stream);

/* addition: one activation row through up to three projections in ONE launch
 * (the decode step's q/k/v): y_i[N_i] = x[K] . W_i^T (+ bias_i). Equals
 * vv_gemm_fp16_dev(M = 1) followed by vv_bias_add_dev per projection bit for
 * bit (src/inference/decoder.c:458-464 called three times). All N_i must fall
 * in the same width class (below 8192, 8192..16383, or from 16384);
 * otherwise, or when K % 8 != 0: VV_ERR_UNSUPPORTED, nothing launched. */
vv_status_t vv_gemv_multi_dev(const void* x, const vv_skinny_proj_t* projs, int n_proj,
                              int K, void* stream);

/* addition: a prefill's MLP front half in one GEMM, out[M, N] = silu(fp16(A Wg^T)) *
 * fp16(A Wu^T) for A[M, K], Wg and Wu [N, K] (decoder.c:966-977: two
 * vv_gemm_fp16_dev and vv_swiglu_dev). Gate and up are rounded to FP16 where the
 * two GEMMs store and go through the SwiGLU kernel's own function in the GEMM's
 * store, so the result equals the three calls bit for bit and gate and up are
 * never written. Fused for M > 64, K % 64 == 0 and 16-byte aligned A, Wg, Wu, and
 * for 17 .. 64 rows (a streaming chunk) against an N of 12800 or more;
 * one row runs vv_gemv_swiglu_dev; every other shape runs the three calls through
 * the caller's `gate` and `up`
 * buffers ([M, N] each; NULL: VV_ERR_UNSUPPORTED for those shapes, nothing
 * launched). The fused path does not touch `gate` and `up`; `out` may be `gate`
 * (as vv_swiglu_dev's output may be its gate input). */
vv_status_t vv_gemm_swiglu_dev(const void* A, const void* w_gate, const void* w_up, void* gate,
                               void* up, void* out, int M, int N, int K, void* stream);

/* addition: the decode step's MLP front half in one launch,
 * y[N] = silu(x . Wg^T) * (x . Wu^T): equals two vv_gemm_fp16_dev(M = 1) and
 * vv_swiglu_dev bit for bit (decoder.c:966-977) without writing gate and up. */
vv_status_t vv_gemv_swiglu_dev(const void* x, const void* w_gate, const void* w_up,
                               void* y, int N, int K, void* stream);

/* addition: vv_embedding_dev(table, ids, hidden) followed by
 * vv_rmsnorm_dev(hidden, weight, normed): the first-layer chain
 * src/inference/pipeline.c:2309 -> decoder.c:810. hidden is bit-exact. */
vv_status_t vv_embedding_rmsnorm_dev(const void* table, const int32_t* ids,
                                     const void* weight, void* hidden, void* normed,
                                     int seq_len, int hidden_size, float eps,
                                     void* stream);

/* ── Device, memory, streams, events, graphs: the runtime half ─────────── */

/* replaces device.h:39-45 (src/cuda/cuda_utils.cu:20-99). Copies with a NULL
 * stream are synchronous; with a stream they are ordered on it. */
vv_status_t vv_dev_alloc(void** ptr, size_t size);
vv_status_t vv_dev_alloc_pinned(void** ptr, size_t size);
vv_status_t vv_dev_free(void* ptr);
vv_status_t vv_dev_free_pinned(void* ptr);
vv_status_t vv_dev_memcpy_h2d(void* dst, const void* src, size_t size, void* stream);
vv_status_t vv_dev_memcpy_d2h(void* dst, const void* src, size_t size, void* stream);
vv_status_t vv_dev_memcpy_d2d(void* dst, const void* src, size_t size, void* stream);

/* Copy `size` bytes to dst_base + (*d_index) * size, the index read on the
 * device. replaces device.h:54-55 (cuda_utils.cu:131-154). */
vv_status_t vv_dev_memcpy_d2d_at(void* dst_base, const void* src, size_t size,
                                 const int* d_index, void* stream);

/* replaces device.h:56 and :65-66 (cuda_utils.cu:418-422, :213-218). The
 * stream-ordered form is a fill kernel, so it may be captured into a graph. */
vv_status_t vv_dev_memset(void* ptr, int value, size_t size);
vv_status_t vv_dev_memset_async(void* ptr, int value, size_t size, void* stream);

/* replaces device.h:67-75 (cuda_utils.cu:229-271). Both kinds of stream are
 * created at the default priority on this backend. */
vv_status_t vv_dev_stream_create(void** stream);
vv_status_t vv_dev_stream_create_background(void** stream);
vv_status_t vv_dev_stream_destroy(void* stream);
vv_status_t vv_dev_stream_sync(void* stream);

/* replaces device.h:76-101 (cuda_utils.cu:276-292, :327-349, :409-412).
 * sm_count reports compute units. */
vv_status_t vv_dev_set_device(int device_id);
vv_status_t vv_dev_get_device_info(int device_id, size_t* total_mem,
                                   size_t* free_mem, int* sm_count);
int         vv_dev_device_count(void);
vv_status_t vv_dev_get_device_name(int device_id, char* buf, size_t buf_size);
bool        vv_dev_host_shares_memory(int device_id);

/* replaces device.h:111-121 (cuda_utils.cu:301-325). */
vv_status_t vv_dev_memcpy_peer(void* dst, int dst_device, const void* src,
                               int src_device, size_t size, void* stream);
vv_status_t vv_dev_enable_peer(int device, int peer);

/* replaces device.h:125-130, :872 (cuda_utils.cu:362-424). Registering
 * existing host memory is declined with VV_ERR_UNSUPPORTED (the caller at
 * decoder.c:289 then keeps its pageable copy path); unregister is VV_OK. */
vv_status_t vv_dev_event_create(void** ev);
vv_status_t vv_dev_event_destroy(void* ev);
vv_status_t vv_dev_event_record(void* ev, void* stream);
vv_status_t vv_dev_event_sync(void* ev);
vv_status_t vv_dev_stream_wait_event(void* stream, void* ev);
vv_status_t vv_dev_host_register(void* p, size_t n);
vv_status_t vv_dev_host_unregister(void* p);

/* replaces device.h:133. Returns "HIP". */
const char* vv_dev_backend_name(void);

/* replaces device.h:152-160 (cuda_utils.cu:158-204). */
vv_status_t vv_dev_graph_begin(void* stream);
vv_status_t vv_dev_graph_end(void* stream, void** graph_exec);
vv_status_t vv_dev_graph_launch(void* graph_exec, void* stream);
void        vv_dev_graph_destroy(void* graph_exec);

/* *dst = *src + delta on the stream. replaces device.h:163
 * (cuda_utils.cu:126-130). */
vv_status_t vv_pos_add_dev(int* dst, const int* src, int delta, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* VIBEVOICE_HIP_H */
