/*
 * vv_oracle.h — CPU restatement of vibevoice.c's src/cpu layer kernels.
 *
 * TEST INFRASTRUCTURE ONLY. This library is the checker for the HIP backend:
 * tests, the smoke check and the benchmark's cpu_baseline leg link it; the
 * shipped library (libvibevoice_hip.so) never does and has no CPU fallback.
 *
 * Two families of functions:
 *   vvo_*_f32   the reference's CPU kernels, restated operation by operation
 *               (FP32 activations, FP16 weights/table), one function per
 *               reference function, each citing the lines it follows;
 *   vvo_*_f16   the same arithmetic applied to the device contract of
 *               include/vibevoice/device.h (FP16 tensors in and out): inputs
 *               are widened exactly, the f32 kernel runs, and the result is
 *               returned both as FP32 ("ref", what the tolerance is measured
 *               against) and rounded to FP16 with round-to-nearest-even
 *               ("rne", what a device kernel that made no other error stores).
 *
 * Parity status (what pins each function is listed in tests/test_oracle_*.py):
 *   the functions that restate src/cpu (layer kernels, int8 quantisers and
 *   linear layers, weight-only dequantisers, BitNet) are pinned by the compiled
 *   reference (oracle/_ref, bit-for-bit) where that builds, by committed golden
 *   vectors made from it, and by closed forms / invariants that do not retype
 *   their formula. The functions that restate accelerator-only code (the
 *   quantised KV codec, the Conv-VAE ops) have no CPU counterpart to compile
 *   and are pinned by what the mathematics fixes: exhaustive code tables,
 *   Hadamard / Lloyd-Max / signal-to-noise conditions, FP64 convolutions,
 *   invariance under chunking, im2col + GEMM == direct convolution. One table
 *   is PARITY UNPINNED: the +-1 pattern of the TurboQuant rotation (see there).
 */
#ifndef VV_ORACLE_H
#define VV_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* FP16 <-> FP32. Follows include/vibevoice/types.h:107-129 (half -> float,
 * exact, subnormals/inf/NaN included) and types.h:171-196 (float -> half,
 * round-to-nearest-even; NaN -> quiet NaN with the sign kept). */
float    vvo_half_to_float(uint16_t h);
uint16_t vvo_float_to_half_rne(float f);
void     vvo_widen_f16(const uint16_t* in, float* out, size_t n);
void     vvo_narrow_f32_rne(const float* in, uint16_t* out, size_t n);

/* src/cpu/cpu_kernels.c:1432-1451 */
int vvo_rmsnorm_f32(const float* input, const uint16_t* weight_f16,
                    float* output, int rows, int n, float eps);
/* src/cpu/cpu_kernels.c:1453-1478 */
int vvo_rope_f32(float* x, int rows, int n_heads, int head_dim,
                 int position_offset, float theta);
/* src/cpu/cpu_kernels.c:1536-1548 */
int vvo_swiglu_f32(const float* gate, const float* up, float* output, int n);
/* src/cpu/cpu_kernels.c:1550-1558 */
int vvo_residual_add_f32(float* x, const float* y, int n);
/* src/cpu/cpu_kernels.c:1560-1568 with f16_row :587-596 */
int vvo_embedding_f32(const uint16_t* table_f16, const int32_t* ids,
                      float* output, int rows, int hidden);

/* ── device-contract forms (FP16 in, FP32 ref + FP16 rne out) ──────────── */

/* vv_rmsnorm_dev contract (device.h:490-492). out_ref/out_rne may be NULL. */
int vvo_rmsnorm_f16(const uint16_t* x, const uint16_t* w, float* out_ref,
                    uint16_t* out_rne, int rows, int n, float eps);

/* vv_residual_add_dev contract (device.h:512): x = half_rn(float(x)+float(y)),
 * the rounding src/cuda/conv_vae.cu:29-31 applies. Bit-exact target. */
int vvo_residual_add_f16(uint16_t* x, const uint16_t* y, size_t n);

/* Fused residual-add + RMSNorm = vv_residual_add_dev followed by
 * vv_rmsnorm_dev on the rounded sum (decoder.c:950-960). residual is updated
 * in place (bit-exact target); normed as for vvo_rmsnorm_f16. */
int vvo_add_rmsnorm_f16(uint16_t* residual, const uint16_t* x,
                        const uint16_t* w, float* normed_ref,
                        uint16_t* normed_rne, int rows, int n, float eps);

/* vv_rope_dev contract (device.h:500-502); x is not modified. */
int vvo_rope_f16(const uint16_t* x, float* out_ref, uint16_t* out_rne,
                 int rows, int n_heads, int head_dim, int position_offset,
                 float theta);

/* vv_swiglu_dev contract (device.h:504-506). */
int vvo_swiglu_f16(const uint16_t* gate, const uint16_t* up, float* out_ref,
                   uint16_t* out_rne, size_t n);

/* vv_swiglu_fused_dev contract (device.h:508-510): gate_up is [rows, 2*inter],
 * gate in columns [0,inter), up in [inter, 2*inter). */
int vvo_swiglu_fused_f16(const uint16_t* gate_up, float* out_ref,
                         uint16_t* out_rne, int rows, int inter);

/* vv_embedding_dev contract (device.h:486-488): FP16 bits copied. */
int vvo_embedding_f16(const uint16_t* table, const int32_t* ids,
                      uint16_t* out, int rows, int hidden);

/* vv_bias_add_dev contract (device.h:513-514; src/cuda/conv_vae.cu:54-67):
 * out[m,n] = half_rn(float(out[m,n]) + float(bias[n])). Bit-exact target. */
int vvo_bias_add_f16(uint16_t* out, const uint16_t* bias, int M, int N);

/* ── per-token int8 activation quantiser (the W8A8 / W4A8 path's front end) ─ */

/* Where column j (0..31) of a 32-column run is stored, per layout
 * (include/vibevoice/q8.h:19-66): 0 natural, 1 nibble (16 even columns, then
 * 16 odd), 2 W4 GEMV, 3 W4 MMA. */
int vvo_q8_pos(int layout, int j);

/* src/cpu/cpu_int8.c:158-196 (vv_quant_act_q8_cpu): per row, amax = max|x|,
 * sx = amax/127, xq = clamp(rint(x * (127/amax)), +-127) stored at the
 * layout's position inside each run of 32; xsum (optional) = the sum of xq over
 * each run. K must be a multiple of 32. Bit-exact target for the device. */
int vvo_quant_act_q8(const float* x, int M, int K, int layout, int8_t* xq,
                     float* sx, int32_t* xsum);

/* ── the layer's two contractions (checkers for the layer runner) ─────── */

/* out[m,n] = sum_k x[m,k] * w[n,k] + bias[n]; x FP32 [M,K], w FP16 [N,K],
 * bias FP16 [N] or NULL. The reference's CPU kernel (src/cpu/cpu_kernels.c:
 * 1325-1360) sums in a SIMD-dependent order; this is the double-accumulated
 * form its own test holds it to at 1e-5 (tests/test_cpu_kernels.c:128-147). */
int vvo_gemm_f16w(const float* x, const uint16_t* w, const uint16_t* bias,
                  float* out, int M, int N, int K);

/* src/cpu/cpu_kernels.c:1480-1525: causal GQA attention, one pass with an
 * online softmax. q, out [rows, n_q_heads, head_dim]; k, v [kv_len,
 * n_kv_heads, head_dim]; query r sits at absolute position q_offset + r and
 * sees keys 0 .. min(q_offset + r + 1, kv_len) - 1 when causal. */
int vvo_attention_prefill_f32(const float* q, const float* k, const float* v,
                              float* out, int n_q_heads, int n_kv_heads,
                              int head_dim, int rows, int q_offset, int kv_len,
                              int causal);

/* The W8A8 linear layer. src/cpu/cpu_int8.c:455-487 (vv_w8a8_gemm_cpu): exact
 * int32 dot of the int8 rows, then v = (float)t * sx[m] * sw[n] (+ bias[n]),
 * products left to right, nothing fused; the device contract
 * (src/cuda/i8_common.cuh:40-48) then adds a residual [M,N] and writes FP32 or
 * FP16 (RNE). bias16 / res16 are FP16 bit patterns or NULL; out_f32 / out_f16
 * either may be NULL. */
int vvo_w8a8_linear(const int8_t* xq, const float* sx, const int8_t* w, const float* sw,
                    const uint16_t* bias16, const uint16_t* res16, float* out_f32,
                    uint16_t* out_f16, int M, int N, int K);

/* The W4A8 linear layer. src/cpu/cpu_int8.c:212-233 (w4_dot_scalar) inside
 * 489-545 (vv_w4a8_gemm_cpu): per group of G columns an exact int32
 * sum_k q x - z * sum_k x, then acc += s_g * (float)that, groups in order,
 * nothing fused; v = acc * sx[m] (+ bias[n]); the device contract then adds a
 * residual and writes FP32 or FP16 (RNE) as for W8A8. `packed` is the
 * row-major INT4G form ([N][K/2], high nibble = even column), `xq` in column
 * order (the CPU kernel reads VV_Q8_NIBBLE order; an exact integer sum does
 * not depend on the order). The reference's vectorised variants add the
 * groups in another order, so its own FP32 results differ between instruction
 * sets in the last bits: against the compiled reference this function is
 * pinned exactly for unit scales and to 1e-6 otherwise. */
int vvo_w4a8_linear(const int8_t* xq, const float* sx, const uint8_t* packed,
                    const uint16_t* scales16, const uint8_t* zeros, int G,
                    const uint16_t* bias16, const uint16_t* res16, float* out_f32,
                    uint16_t* out_f16, int M, int N, int K);

/* INT4 group-affine weights to dense FP16 [N,K]: w = (q - z) * s rounded once to
 * FP16, the formula include/vibevoice/device.h:233 and src/cuda/w4a16.cu:24-27
 * state for every W4A16 kernel. `packed` is the row-major INT4G form. The
 * W4A16 linear layer is then vvo_gemm_f16w over these weights. */
int vvo_int4g_dequant_f16(const uint8_t* packed, const uint16_t* scales16, const uint8_t* zeros,
                          int N, int K, int G, uint16_t* out16);

/* src/quant/awq_repack.c:261-310 (vv_int4g_to_gpu_layout): row-major INT4G
 * codes to the layout the accelerator kernels read, in place: inside every
 * 16-byte chunk (32 columns), nibble slot s of 32-bit word t holds column
 * 2 (t + 4 (s % 4)) + s / 4; out_sz[n][g] = half2 {scale, (half)zero}. */
int vvo_int4g_to_gpu_layout(uint8_t* packed, const uint16_t* scales16, const uint8_t* zeros,
                            int N, int K, int G, uint16_t* out_sz);

/* The FP8 KV-cache codec, src/cuda/kv_codec.cuh:66-128 (the reference has no
 * CPU form of it; this restates the accelerator's integer arithmetic, and the
 * tests pin it to what the formats themselves fix: every code decodes to its
 * closed-form value, and every FP16 input encodes to a nearest representable
 * value). e5m2 == 0: E4M3 (largest finite 448), else E5M2 (57344); zero and NaN
 * encode as a signed zero, out-of-range magnitudes saturate. */
int vvo_fp8_encode(const float* x, int n, int e5m2, uint8_t* out);
int vvo_fp8_decode(const uint8_t* codes, int n, int e5m2, float* out);
/* src/cuda/kv_quant.cu:157-169 (kv_build_ref_kernel): per head and channel the
 * FP32 mean of the run's keys, positions added in order, rounded to FP16. */
int vvo_kv_build_ref(const uint16_t* k16, int n_pos, int n_kv_heads, int head_dim, uint16_t* ref16);
/* src/cuda/kv_quant.cu:57-84 (kv_store_kernel, FP8 formats): FP16 -> FP32, minus
 * the head's reference key when there is one, then the codec. */
int vvo_kv_store_fp8(const uint16_t* src16, const uint16_t* ref16, int n_pos, int n_kv_heads,
                     int head_dim, int e5m2, uint8_t* store);

/* The older weight-only formats, run on FP16 activations. Each writes the
 * weight as FP16 bits (what a GEMM multiplies after dequantisation) and/or as
 * the FP32 value before that rounding (what the one-row kernels multiply):
 *   vvo_nf4_dequant   dequant_nf4.cu:40-66 — code book[nibble] x FP16 absmax per
 *                     64 flat elements, high nibble = even element
 *   vvo_awq_dequant   awq_gemv.cu:125-153 — q x scale + min per group of G
 *   vvo_int8_dequant  int8_gemv.cu:139-160 — q x FP32 scale of the row */
int vvo_nf4_dequant(const uint8_t* packed, const uint16_t* scales16, size_t n_elements, uint16_t* out16,
                    float* out32);
int vvo_awq_dequant(const uint8_t* packed, const uint16_t* scales16, const uint16_t* mins16, int N, int K,
                    int G, uint16_t* out16, float* out32);
int vvo_int8_dequant(const int8_t* q, const float* scales, int N, int K, uint16_t* out16, float* out32);

/* The TurboQuant KV-cache codec (formats 3..6 of include/vibevoice/kv_quant.h:
 * 4, 3, 2 and 1.5 bits per value, plus an FP16 RMS per vector). Like the FP8
 * codec the reference holds it only as accelerator code (src/cuda/kv_codec.cuh:
 * 38-62, 130-165, 180-285; kv_quant.cu:86-119, 171-199); this restates it with
 * the accelerator's order of FP32 additions. Pinned by what the method fixes:
 * the transform is the 128-point Hadamard matrix times a +-1 diagonal, scaled
 * to be orthogonal; the level tables are the Lloyd-Max fixed points of a unit
 * Gaussian and reach the signal-to-noise ratios the reference quotes for them;
 * a code is the nearest level (code word). The particular +-1 pattern (a hash
 * of the channel index) is restated only: parity unpinned for that one table,
 * which no result depends on as long as store and reader agree.
 *   vvo_kv_rotate   in-place transform (or its inverse) of n_vectors x 128 FP16
 *   vvo_kv_store_tq FP16 [n_pos][n_kv_heads][128] (minus ref16 [n_kv_heads][128]
 *                   when given) -> codes [..][bytes_per_vec] and meta16 [..]
 *   vvo_kv_unpack   any quantised format (FP8 too) as FP16 in the space it was
 *                   stored in (TurboQuant: rotated): what attention reads
 *   vvo_kv_dequant  any quantised format back to FP16 in the ORIGINAL space:
 *                   unpacked, un-rotated (TurboQuant), plus ref16 when given,
 *                   one rounding (kv_quant.cu:311-338) */
int vvo_kv_bytes_per_vec(int fmt);
int vvo_kv_rotate(uint16_t* x16, int n_vectors, int inverse);
int vvo_kv_store_tq(const uint16_t* src16, const uint16_t* ref16, int n_pos, int n_kv_heads, int fmt,
                    uint8_t* store, uint16_t* meta16);
int vvo_kv_unpack(const uint8_t* store, const uint16_t* meta16, int n_vectors, int fmt, uint16_t* out16);
int vvo_kv_dequant(const uint8_t* store, const uint16_t* meta16, const uint16_t* ref16, int n_pos,
                   int n_kv_heads, int fmt, uint16_t* out16);

/* BitNet's integer layers (include/vibevoice/bitnet.h, src/cpu/bitnet_cpu.c),
 * written the slow way: integer sums exact, every FP32 operation rounded on
 * its own in the order the reference states.
 *   vvo_ternary_pack    {-1,0,1} [N][K] -> the I2_S bytes (bitnet_cpu.c:222-235)
 *   vvo_bn_act_quant    per-token int8 with the fused-multiply-add rounding of
 *                       ggml's quantiser (bitnet_cpu.c:352-358, 396-441)
 *   vvo_ternary_linear  acc and y = acc / x_scale * w_scale + bias (:741-790)
 *   vvo_i8_linear       acc, y = acc * (w_scale / a_scale) + bias, max|y| (:1048-1131)
 *   vvo_i8s_requant     one-scale requantisation (:1133-1151)
 *   vvo_i8_head_argmax  int8 tied-head argmax, ties to the lowest index (:1153-1213) */
int vvo_ternary_pack(const int8_t* t, int64_t N, int64_t K, uint8_t* codes);
int vvo_bn_act_quant(const float* x, int M, int K, int8_t* q, float* scale, int32_t* sum);
int vvo_ternary_linear(const int8_t* q, const float* x_scale, const uint8_t* codes, float w_scale,
                       const float* bias, int M, int N, int K, int32_t* acc_out, float* y);
int vvo_i8_linear(const int8_t* a, float a_scale, const int8_t* w, float w_scale, const float* bias,
                  int M, int N, int K, int32_t* acc_out, float* y, float* absmax);
int vvo_i8s_requant(const float* y, int64_t n, float absmax, int relu, int8_t* q, float* out_scale);
int vvo_i8_head_argmax(const int8_t* q, float scale, const int8_t* w, const float* w_scale, int V, int K,
                       int32_t* token, float* value);

/* The batched, streaming Conv-VAE encoder ops (src/cuda/vae_kernels.cu; the
 * reference's CPU encoder works in FP32 with other roundings, so these restate
 * the accelerator's arithmetic). Host pointers throughout; FP16 as uint16 bits.
 * The descriptor is include/vibevoice/device.h:733-755, field for field.
 *   vvo_vae_conv      vae_kernels.cu:50-89   FP32 fused multiply-add chain over
 *                     (in channel, tap) from zero, + bias, one FP16 rounding
 *   vvo_vae_tail      :95-116    the last `keep` columns of [context ++ input]
 *   vvo_vae_im2col    :118-147
 *   vvo_vae_conv_gemm :149-284   the same chain over K of the im2col columns
 *   vvo_vae_rms       :286-318   1 / sqrt(sum of squares (FMA chain) / C + eps)
 *   vvo_vae_mixer     :320-392   half((x * rinv) * w) -> depthwise FMA chain ->
 *                     half -> half(x + y * gamma)
 *   vvo_vae_gemm_nn   :394-607   A[M,K] x B[K,P] (double accumulation here), B
 *                     optionally normalised on its way in, three epilogues
 *   vvo_vae_gemm_tn   :609-712   A x B^T + bias, rows scattered, truncating modes
 *   vvo_trunc_half    :614-625 */
#define VVO_VAE_MAX_ITEMS 32
typedef struct vvo_vae_conv_item {
    int64_t in_off, out_off;
    const void* in_ptr;
    const void* tail_in;
    void* tail_out;
    void* out_ptr;
    int in_len, out_len, have, keep, out_ld, skip;
} vvo_vae_conv_item_t;
typedef struct vvo_vae_conv_desc {
    int n, cap;
    vvo_vae_conv_item_t it[VVO_VAE_MAX_ITEMS];
} vvo_vae_conv_desc_t;
typedef struct vvo_vae_row_seg { int row0, ld; void* dst; } vvo_vae_row_seg_t;
typedef struct vvo_vae_rows { int mode, n; vvo_vae_row_seg_t seg[VVO_VAE_MAX_ITEMS]; } vvo_vae_rows_t;
int vvo_vae_conv(const vvo_vae_conv_desc_t* d, const uint16_t* x, int64_t ld_in, const uint16_t* w,
                 const uint16_t* b, uint16_t* y, int64_t ld_out, int in_ch, int out_ch, int k, int stride,
                 int transposed);
int vvo_vae_tail(const vvo_vae_conv_desc_t* d, const uint16_t* x, int64_t ld_in, int in_ch);
int vvo_vae_im2col(const vvo_vae_conv_desc_t* d, const uint16_t* x, int64_t ld_in, int in_ch, int k, int stride,
                   int64_t p0, int pc, uint16_t* col, int64_t ldcol);
int vvo_vae_conv_gemm(const uint16_t* w, const uint16_t* col, int64_t ldcol, const uint16_t* b, uint16_t* y,
                      int64_t ld_out, int out_ch, int K, int pc);
int vvo_vae_rms(const uint16_t* x, int64_t ld, int64_t T, int C, float eps, float* rinv,
                const vvo_vae_conv_desc_t* d);
int vvo_vae_mixer(const vvo_vae_conv_desc_t* d, const uint16_t* xin, uint16_t* xout, int64_t ld, const float* rinv,
                  int64_t T_total, const uint16_t* nw, const uint16_t* cw, const uint16_t* cb,
                  const uint16_t* gamma, int C, int k);
int vvo_vae_gemm_nn(int epilogue, const uint16_t* A, const uint16_t* B, int64_t ldb, uint16_t* C, int64_t ldc,
                    int M, int K, int P, const uint16_t* bias, const uint16_t* gamma, const float* rinv,
                    const uint16_t* nw);
int vvo_vae_gemm_tn(const uint16_t* A, int64_t lda, const uint16_t* B, uint16_t* C, int64_t ldc, int M, int N,
                    int K, const uint16_t* bias, const vvo_vae_rows_t* rows);
uint16_t vvo_trunc_half(float f);

/* src/cpu/cpu_kernels.c:1613-1623 (vv_sample_greedy_cpu): the first maximum of
 * an in-order scan; a NaN never replaces the running best. */
int vvo_argmax_first(const float* logits, int n, int32_t* token, float* value);

/* ── seeded inputs (the same bytes go to the oracle and to the GPU) ────── */

/* N(mean, std) rounded to FP16 (RNE). Counter-based: element i depends only
 * on (seed, i), so any slice can be regenerated. */
void vvo_fill_normal_f16(uint16_t* out, size_t n, uint64_t seed,
                         double mean, double std);
void vvo_fill_normal_f32(float* out, size_t n, uint64_t seed,
                         double mean, double std);
/* uniform int32 on [0, bound) */
void vvo_fill_ids(int32_t* out, size_t n, uint64_t seed, int32_t bound);

/* OpenMP threads the *_f32 kernels will use (1 if built without OpenMP). */
int vvo_threads(void);
void vvo_set_threads(int n);

#ifdef __cplusplus
}
#endif
#endif /* VV_ORACLE_H */
