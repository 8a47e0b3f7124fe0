/*
 * unsupported.c — the rest of the accelerator seam, declined.
 *
 * vibevoice.c's device.h declares ~100 symbols and a binary links exactly one
 * backend, so a backend that accelerates only part of the op set still has to
 * DEFINE every symbol. The contract for an op a backend does not implement is
 * "return VV_ERR_UNSUPPORTED having launched nothing", which the callers that
 * have a fallback take (include/vibevoice/device.h:468-470; precedent:
 * src/metal/metal_stubs.c:1-30, src/device/device_none.c:129-483).
 *
 * This file is that remainder for libvibevoice_hip: every device.h symbol the
 * HIP library does not define (the NN dense GEMM and the Conv-VAE kernels). It builds into its
 * own small library, libvibevoice_hip_unsupported.so, which a full engine link
 * adds next to libvibevoice_hip.so; the layer-op library's own export list
 * stays exactly what include/vibevoice_hip.h declares.
 *
 * The definitions take no named parameters on purpose: none of them reads an
 * argument, and under the x86-64 System V calling convention the caller owns
 * argument setup and cleanup, so one unprototyped definition serves whatever
 * argument list device.h gives the symbol. Size queries return 0 and shape /
 * backend queries return 0, as device_none.c does (its vv_attn_resolve answer,
 * VV_ATTN_FA1, is the enum's zero).
 */
#include <stddef.h>

#define VV_ERR_UNSUPPORTED (-7) /* include/vibevoice/types.h:27 */

#define VV_DECLINE(name) int name() { return VV_ERR_UNSUPPORTED; }
#define VV_ZERO_INT(name) int name() { return 0; }
#define VV_ZERO_SIZE(name) size_t name() { return 0; }

/* dense FP16 GEMM: the NN form (device.h:477-479); the NT forms are implemented */
VV_DECLINE(vv_gemm_fp16_nn_dev)
void vv_gemm_cleanup() {}



/* Conv-VAE speech encoder (device.h:762-870) */
VV_DECLINE(vv_vae_conv_dev)      VV_DECLINE(vv_vae_tail_dev)      VV_DECLINE(vv_vae_rms_dev)
VV_DECLINE(vv_vae_mixer_dev)     VV_DECLINE(vv_vae_im2col_dev)    VV_DECLINE(vv_vae_conv_gemm_dev)
VV_DECLINE(vv_vae_gemm_nn_dev)   VV_DECLINE(vv_vae_gemm_tn_dev)   VV_DECLINE(vv_vae_f32_to_f16_dev)
