/*
 * ffk - MI355X (gfx950) kernels for the FastFold Evoformer hot path.  C ABI.
 *
 * libffk.so is libtorch-free: every entry point takes raw device pointers, explicit
 * shapes / strides, a dtype tag and a HIP stream (passed as void*), launches on that
 * stream and returns an int status (FFK_OK = 0).  The library allocates nothing and
 * keeps no state; the caller owns every buffer, scratch included.  After a non-zero
 * return ffk_last_error_string() describes the failure (thread-local).
 *
 * Each entry point names the reference interface it stands in for (paths are relative
 * to the reference repository root).
 */
#ifndef FFK_H
#define FFK_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* status codes */
enum {
    FFK_OK = 0,
    FFK_ERR_DTYPE = 1,     /* dtype tag not supported by this entry point          */
    FFK_ERR_SHAPE = 2,     /* a dimension is <= 0, too large, or violates a divisibility rule */
    FFK_ERR_NULL = 3,      /* a required pointer is NULL                           */
    FFK_ERR_ALIGN = 4,     /* a pointer / leading dimension is not 16-byte aligned */
    FFK_ERR_LAUNCH = 5,    /* hipGetLastError() reported a failure after launch    */
    FFK_ERR_UNSUPPORTED = 6
};

/* element types of activation / weight buffers */
enum { FFK_F32 = 0, FFK_BF16 = 1, FFK_F16 = 2 };

int ffk_version(void);
const char* ffk_last_error_string(void);

/* ------------------------------------------------------------------------------------
 * Fused softmax:  out = softmax(where(mask == 0, -1e9, x + bias), dim = -1)
 *   x, out : [B1, B2, H, Nq, Nk]   (out may alias x: the reference's CUDA path is in place)
 *   mask   : [B1, B2, Nk] of the same dtype holding 0/1, or NULL
 *   bias   : [B1, 1, H, Nq, Nk] of the same dtype, or NULL (requires mask != NULL is NOT
 *            demanded; any combination is accepted)
 * fp32 arithmetic inside; dtype f32 / bf16 / f16.
 * Replaces: fastfold_softmax_cuda.{forward, fused_mask_softmax_forward,
 *   fused_mask_bias_softmax_forward}
 *   (fastfold/model/fastnn/kernel/cuda_native/csrc/softmax_cuda.cpp:3-27,
 *    softmax_cuda_kernel.cu:163-250,425-522,708-810) and the Triton wrapper
 *   (kernel/triton/softmax.py:153-186).
 */
int ffk_softmax_fwd(void* out, const void* x, const void* mask, const void* bias,
                    int64_t B1, int64_t B2, int64_t H, int64_t Nq, int64_t Nk,
                    int dtype, void* stream);

/* Softmax backward: dx = (dy - sum(y * dy)) * y over rows of length cols.
 * Replaces: fastfold_softmax_cuda.{backward, fused_mask_softmax_backward,
 *   fused_mask_bias_softmax_backward} (softmax_cuda_kernel.cu:252-334,524-614,812-839);
 * masked entries have y == 0 and therefore dx == 0 without consulting the mask. */
int ffk_softmax_bwd(void* dx, const void* dy, const void* y, int64_t rows, int64_t cols,
                    int dtype, void* stream);

/* ------------------------------------------------------------------------------------
 * LayerNorm over the last dimension, affine:  out = (x - mean) * rsqrt(var + eps) * gamma + beta
 *   x, out : [rows, cols] contiguous;  gamma, beta : [cols] of the same dtype
 *   mean, rstd : optional fp32 [rows] outputs (NULL to skip)
 * Replaces: fastfold_layer_norm_cuda.forward_affine
 *   (kernel/cuda_native/csrc/layer_norm_cuda.cpp:70-95, layer_norm_cuda_kernel.cu:61-152)
 *   and kernel/triton/layer_norm.py:146-176.
 */
int ffk_layernorm_fwd(void* out, float* mean, float* rstd, const void* x, const void* gamma,
                      const void* beta, int64_t rows, int64_t cols, float eps, int dtype,
                      void* stream);

/* LayerNorm backward (dx, dgamma, dbeta).  dgamma/dbeta are fp32 [cols] and must be
 * zero-filled by the caller (the kernel accumulates with atomics).
 * Replaces: fastfold_layer_norm_cuda.backward_affine (layer_norm_cuda.cpp:97-125,
 *   layer_norm_cuda_kernel.cu:224-500). */
int ffk_layernorm_bwd(void* dx, float* dgamma, float* dbeta, const void* dy, const void* x,
                      const float* mean, const float* rstd, const void* gamma,
                      int64_t rows, int64_t cols, int dtype, void* stream);

/* ------------------------------------------------------------------------------------
 * Elementwise fusions (eval-mode dropout: the mask tensor multiplies as given).
 * Tensors are viewed as [B, I, J, C]; `dm` is the dropout mask with strides (in elements)
 * dm_sb, dm_si, dm_sj for the first three axes (0 = broadcast) and unit stride on C;
 * dm may be NULL (= all ones).
 *   ffk_bias_sigmoid_mul      : out = sigmoid(y + bias[C]) * z
 *   ffk_bias_dropout_add      : out = residual + (x + bias[C]) * dm
 *   ffk_bias_ele_dropout_res  : out = z_raw + dm * (g * (ab + bias[C]))
 * Replaces: bias_sigmod_ele, bias_dropout_add, bias_ele_dropout_residual
 *   (fastfold/model/fastnn/kernel/jit/fused_ops.py:5-22).
 */
int ffk_bias_sigmoid_mul(void* out, const void* y, const void* bias, const void* z,
                         int64_t rows, int64_t C, int dtype, void* stream);
int ffk_bias_dropout_add(void* out, const void* x, const void* bias, const void* dm,
                         const void* residual, int64_t B, int64_t I, int64_t J, int64_t C,
                         int64_t dm_sb, int64_t dm_si, int64_t dm_sj, int dtype, void* stream);
int ffk_bias_ele_dropout_res(void* out, const void* ab, const void* bias, const void* g,
                             const void* dm, const void* z_raw, int64_t B, int64_t I, int64_t J,
                             int64_t C, int64_t dm_sb, int64_t dm_si, int64_t dm_sj, int dtype,
                             void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FFK_H */
