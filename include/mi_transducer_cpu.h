/* mi_transducer_cpu.h -- C ABI of the host (CPU) RNNT loss, libmi_transducer_cpu.so.
 *
 * Replaces what the reference runs when RNNTLossNumba is given CPU tensors
 * (nemo/collections/asr/parts/numba/rnnt_loss/):
 *   rnnt_pytorch.py:420-435   the module's log_softmax and clamp hook in front of the loss
 *   rnnt.py:39-135            rnnt_loss_cpu
 *   utils/cpu_utils/cpu_rnnt.py:164-422   CPURNNT (alphas, betas, sparse log-prob gradient, costs)
 * TDT and the multi-blank loss have no CPU path in the reference (rnnt_pytorch.py:137-140, :226-229) and none here.
 *
 * Conventions: plain C, HOST pointers, float32 logits.  Returns 0 on success, 1 on an invalid value (RNNTStatus,
 * utils/global_constants.py:66-68).  acts are raw LOGITS [B,T,U,V] row-major (the library normalises them, which
 * is the module's log_softmax); labels int64 [B,U-1]; lengths int64 [B], clamped into the tensor as on the GPU.
 * num_threads: utterances run in parallel under OpenMP; <= 0 means all available threads (the reference's
 * num_threads argument, rnnt.py:83-86).
 */
#ifndef MI_TRANSDUCER_CPU_H_
#define MI_TRANSDUCER_CPU_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI_TRANSDUCER_CPU_SUCCESS 0
#define MI_TRANSDUCER_CPU_INVALID_VALUE 1

int mi_transducer_cpu_abi_version(void);

/* Scratch bytes for a [B,T,U] lattice: replaces get_workspace_size(..., gpu=False)
 * (utils/rnnt_helper.py:119-142).  The workspace must be 8-byte aligned; what forward leaves in it is what
 * backward reads. */
int mi_rnnt_cpu_workspace_bytes(int B, int T, int U, size_t* out_bytes);

/* costs[b] = -ll_forward[b] * (1 + fastemit_lambda) in float32 (CPURNNT.cost_and_grad_kernel / score_forward,
 * cpu_rnnt.py:214-276, :388-422). */
int mi_rnnt_cpu_forward(const float* acts, const int64_t* labels, const int64_t* act_lens, const int64_t* label_lens,
                        float* costs, int B, int T, int U, int V, int blank, float fastemit_lambda, void* workspace,
                        size_t workspace_bytes, int num_threads);

/* grads[B,T,U,V] = gradient of costs[b] w.r.t. the logits: the reference's sparse gradient w.r.t. the log-probs
 * (compute_betas_and_grads, cpu_rnnt.py:278-345) taken through the log_softmax backward, multiplied by
 * (grad_scale ? grad_scale[b * grad_scale_stride] : 1) * grad_mul -- the 1/B of reduction='mean' and the autograd
 * grad_output (rnnt_pytorch.py:77-92) -- and then clamped to [-clamp, clamp] when clamp > 0 (the hook of
 * cpu_rnnt.py:141-161 sees the finished gradient).  Padded cells get zeros.
 * wrt_log_probs != 0: the sparse gradient w.r.t. the LOG-PROBS itself, as rnnt_loss_cpu leaves it in its `grads`
 * argument (two entries per cell, zeros elsewhere; scaled, never clamped) -- for callers of that function, who
 * pass log-probs as acts (normalising them again changes nothing) and own the log_softmax. */
int mi_rnnt_cpu_backward(const float* acts, const int64_t* labels, const int64_t* act_lens, const int64_t* label_lens,
                         float* grads, const float* grad_scale, int grad_scale_stride, float grad_mul, int B, int T,
                         int U, int V, int blank, float fastemit_lambda, float clamp, int wrt_log_probs,
                         const void* workspace, size_t workspace_bytes, int num_threads);

#ifdef __cplusplus
}
#endif
#endif /* MI_TRANSDUCER_CPU_H_ */
