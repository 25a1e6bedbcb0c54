/* mi_transducer.h -- C ABI of the MI355X (gfx950) transducer-loss library.
 *
 * One shared library, libmi_transducer.so, replaces everything the reference
 * runs below its function-level seam (nemo/collections/asr/parts/numba/rnnt_loss/):
 *   rnnt.py:138-236  rnnt_loss_gpu      -> mi_rnnt_loss  (or mi_rnnt_forward + mi_rnnt_backward)
 *   rnnt.py:239-363  tdt_loss_gpu       -> mi_tdt_loss   (or mi_tdt_forward  + mi_tdt_backward)
 *   rnnt.py:366-483  multiblank_rnnt_loss_gpu -> mi_multiblank_loss (or _forward + _backward)
 *   utils/rnnt_helper.py:119-142 get_workspace_size -> mi_transducer_workspace_bytes
 *
 * Conventions
 *   - plain C: device pointers, sizes, a hipStream_t passed as void*; no torch types.
 *   - every function returns 0 on success, 1 on an invalid value (mirrors RNNTStatus,
 *     utils/global_constants.py:66-68), 2 if a HIP launch failed (3: see mi_rnnt_loss_static).  Nothing throws.
 *   - all work is enqueued on `stream`; no call blocks the host, allocates or frees.
 *   - all device memory is caller-owned.  `workspace` is scratch of at least
 *     mi_transducer_workspace_bytes() bytes, 256-byte aligned; its contents after a
 *     forward call are what the matching backward call reads, so keep it until then.
 *     Concurrent calls must use different workspaces.
 *   - acts:   [B,T,U,V(+D)] row-major contiguous raw LOGITS (the library normalises),
 *             dtype code 0 = float32, 1 = bfloat16, 2 = float16; accumulation is fp32/fp64.
 *   - labels: int64 [B,U-1]; act_lens, label_lens: int64 [B]; all on the device.
 *     Lengths are clamped to [1,T] / [0,U-1] and label ids to [0,V-1] inside the
 *     kernels so that a bad value can never address outside the tensors.
 *   - limits: U <= 1024 (as the reference: one thread per label position,
 *     utils/cuda_utils/gpu_rnnt.py:164), D <= 16, durations strictly ascending,
 *     non-negative and holding 1 at position 0 or 1
 *     (utils/cuda_utils/gpu_rnnt_kernel.py:1137-1148).
 */
#ifndef MI_TRANSDUCER_H_
#define MI_TRANSDUCER_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI_TRANSDUCER_SUCCESS 0
#define MI_TRANSDUCER_INVALID_VALUE 1
#define MI_TRANSDUCER_LAUNCH_FAILURE 2
#define MI_TRANSDUCER_TOO_LARGE 3 /* mi_rnnt_loss_static only: the shape needs more than the built-in workspace */

#define MI_DTYPE_F32 0
#define MI_DTYPE_BF16 1
#define MI_DTYPE_F16 2

/* `riders` of the combined forward + backward entry points (mi_*_loss): whether the lattice launch of the call
 * carries the extra workgroups that zero-fill gradient padding while the recursion runs (see prefill_grads of
 * mi_rnnt_forward).  AUTO: only for gradients of 32 MiB and more (below that a step is bound by its launches).  The
 * results are the same bits either way; any other value is invalid.  A per-call argument: the library keeps no
 * setting that changes what a call computes or launches. */
#define MI_RIDERS_AUTO (-1)
#define MI_RIDERS_OFF 0
#define MI_RIDERS_ON 1

#define MI_TRANSDUCER_MAX_U 1024
#define MI_TRANSDUCER_MAX_DURATIONS 16
#define MI_TRANSDUCER_MAX_BIG_BLANKS 8      /* multi-blank: big blanks beside the standard blank */
#define MI_TRANSDUCER_MAX_BLANK_DURATION 64 /* multi-blank: longest big-blank duration */

/* Library/ABI version; bumped whenever a signature below changes. */
int mi_transducer_abi_version(void);

/* Scratch bytes needed for a [B,T,U] lattice with D duration outputs (D = 0 for RNNT).
 * Replaces get_workspace_size (utils/rnnt_helper.py:119-142); any dimension <= 0 is
 * an invalid value, as there. */
int mi_transducer_workspace_bytes(int B, int T, int U, int D, size_t* out_bytes);

/* RNNT forward: log-softmax denominators of the valid cells (replaces reduce_max +
 * reduce_exp, utils/cuda_utils/reduce.py:121-248), forward variables and
 * costs[b] = -ll[b] * float32(1 + fastemit_lambda) (compute_alphas_kernel,
 * utils/cuda_utils/gpu_rnnt_kernel.py:73-172; compute_costs_data,
 * utils/rnnt_helper.py:106-116).  with_betas != 0 also runs the backward variables
 * (compute_betas_kernel, gpu_rnnt_kernel.py:175-269), which mi_rnnt_backward needs;
 * with_betas == 0 is the reference's score_forward (gpu_rnnt.py:250-265).
 * prefill_grads (nullable; the forward calls of all three losses take it): the buffer, of the shape and dtype of
 * acts, that this call's backward call will write the gradient into.  The lattice recursion keeps a few dozen
 * compute units busy and leaves HBM idle; given the buffer, the lattice launch carries extra workgroups that
 * zero-fill the gradient of padded cells meanwhile (part of what zeros_like + `grads *= 0` do up front in the
 * reference, rnnt_pytorch.py:58, gpu_rnnt.py:156), stop when the lattice ends, and record in the workspace how far
 * they got.  The backward call is then given padding_zeroed = 2.  Ignored when with_betas == 0, and for the shapes
 * whose gradient kernel cannot consult that record (rows beyond 8192 16-byte vectors, more than 128 utterances).
 * Whether a problem is large enough for this to pay is the caller's decision (see MI_RIDERS_AUTO). */
int mi_rnnt_forward(const void* acts, int act_dtype, const int64_t* labels, const int64_t* act_lens,
                    const int64_t* label_lens, float* costs, int B, int T, int U, int V, int blank,
                    float fastemit_lambda, int with_betas, void* prefill_grads, void* workspace,
                    size_t workspace_bytes, void* stream);

/* RNNT backward: writes every element of grads[B,T,U,V] (same dtype as acts): the
 * gradient of costs[b] w.r.t. the logits for valid cells, FastEmit and clamp folded
 * in (compute_grad_kernel, gpu_rnnt_kernel.py:272-407), zeros for padded cells
 * (replaces zeros_like + `grads *= 0`, rnnt_pytorch.py:58, gpu_rnnt.py:156).
 * Utterance b's gradient is multiplied, after the clamp, by
 *     (grad_scale ? grad_scale[b * grad_scale_stride] : 1) * grad_mul
 * which folds the autograd backward `grads.mul_(grad_output)` (rnnt_pytorch.py:88-92; a
 * broadcast grad_output is stride 0) and the 'mean' reduction's 1/B (rnnt_pytorch.py:77-81)
 * into the same pass.  grad_scale: device float32, nullable; grad_scale_stride >= 0 in elements.
 * Must follow mi_rnnt_forward(with_betas != 0) on the same workspace and inputs.
 * padding_zeroed (the backward calls of all three losses take it): 0 = this call writes every padded cell;
 * 1 = the padded cells of grads were already zero-filled by mi_transducer_zero_padding (the caller made this
 * call wait for it) and are skipped; 2 = the forward call on this workspace was given these grads as
 * prefill_grads, and the padded cells it reports as zero-filled are skipped.  Any other value is invalid. */
int mi_rnnt_backward(const void* acts, int act_dtype, const int64_t* labels, const int64_t* act_lens,
                     const int64_t* label_lens, void* grads, const float* grad_scale, int grad_scale_stride,
                     float grad_mul, int padding_zeroed, int B, int T, int U, int V, int blank,
                     float fastemit_lambda, float clamp, void* workspace, size_t workspace_bytes, void* stream);

/* rnnt_loss_gpu in one call (rnnt.py:138-236 -> GPURNNT.cost_and_grad / score_forward,
 * gpu_rnnt.py:125-265): grads == NULL means forward only. */
int mi_rnnt_loss(const void* acts, int act_dtype, const int64_t* labels, const int64_t* act_lens,
                 const int64_t* label_lens, float* costs, void* grads, const float* grad_scale,
                 int grad_scale_stride, float grad_mul, int B, int T, int U, int V, int blank, float fastemit_lambda,
                 float clamp, int riders, void* workspace, size_t workspace_bytes, void* stream);

/* mi_rnnt_loss without a workspace argument, for callers that cannot allocate one: code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference (whose wrapper
 * allocates a workspace per call, rnnt.py:182-189).  The lattice state lives in a device array built into the
 * library, MI_TRANSDUCER_STATIC_WORKSPACE_BYTES (64 MiB) per GPU that the library runs on, held until the process
 * ends; a shape whose workspace (mi_transducer_workspace_bytes(B, T, U, 0)) is larger returns
 * MI_TRANSDUCER_TOO_LARGE and launches nothing.  B=16, T=375, U=121 needs 50 MB.  The call itself allocates and
 * frees nothing and does not block.  All calls on one GPU share that one array: two calls that overlap in time
 * on the same GPU (different streams, or threads) race; calls on one stream are fine, and nothing has to be
 * cleared between calls.  mi_transducer_init() looks the array's address up for the current device (the first
 * mi_rnnt_loss_static on a device does it otherwise): call it once per device before capturing a graph.
 * Results are those of mi_rnnt_loss, bit for bit. */
#define MI_TRANSDUCER_STATIC_WORKSPACE_BYTES (64u << 20)
int mi_transducer_init(void);
int mi_rnnt_loss_static(const void* acts, int act_dtype, const int64_t* labels, const int64_t* act_lens,
                        const int64_t* label_lens, float* costs, void* grads, const float* grad_scale,
                        int grad_scale_stride, float grad_mul, int B, int T, int U, int V, int blank,
                        float fastemit_lambda, float clamp, int riders, void* stream);

/* TDT.  acts is the COMBINED tensor [B,T,U,V+D]: V token logits (blank included)
 * followed by D duration logits, exactly what TDTLossNumba.forward receives
 * (rnnt_pytorch.py:554-583); the split, the .contiguous() copies and the duration
 * log_softmax it performs are done inside the kernels.  durations_host: D ints in
 * HOST memory.  Kernels replaced: compute_tdt_alphas_kernel / _betas_kernel /
 * _grad_kernel (gpu_rnnt_kernel.py:888-1439) with sigma as there.  The gradient is
 * w.r.t. the combined LOGITS: the duration block already carries the log-softmax
 * Jacobian that torch autograd applies for the reference.
 * use_plain_rnnt != 0 is the reference's omega branch (gpu_rnnt.py:606-682): the
 * caller samples r < omega on the host; token logits then go through the plain RNNT
 * kernels and the duration block of the gradient is zero. */
int mi_tdt_forward(const void* acts, int act_dtype, const int64_t* labels, const int64_t* act_lens,
                   const int64_t* label_lens, float* costs, int B, int T, int U, int V, int D,
                   const int32_t* durations_host, int blank, float fastemit_lambda, float sigma, int use_plain_rnnt,
                   int with_betas, void* prefill_grads, void* workspace, size_t workspace_bytes, void* stream);

int mi_tdt_backward(const void* acts, int act_dtype, const int64_t* labels, const int64_t* act_lens,
                    const int64_t* label_lens, void* grads, const float* grad_scale, int grad_scale_stride,
                    float grad_mul, int padding_zeroed, int B, int T, int U, int V, int D,
                    const int32_t* durations_host, int blank, float fastemit_lambda, float clamp, float sigma,
                    int use_plain_rnnt, void* workspace, size_t workspace_bytes, void* stream);

int mi_tdt_loss(const void* acts, int act_dtype, const int64_t* labels, const int64_t* act_lens,
                const int64_t* label_lens, float* costs, void* grads, const float* grad_scale, int grad_scale_stride,
                float grad_mul, int B, int T, int U, int V, int D, const int32_t* durations_host, int blank,
                float fastemit_lambda, float clamp, float sigma, int use_plain_rnnt, int riders, void* workspace,
                size_t workspace_bytes, void* stream);

/* TDT with the reference's function-level operands (tdt_loss_gpu, rnnt.py:239-255; GPUTDT.cost_and_grad /
 * score_forward, utils/cuda_utils/gpu_rnnt.py:563-807): label_acts [B,T,U,V] raw token logits and duration_acts
 * [B,T,U,D] duration LOG-PROBS (the caller has applied log_softmax, rnnt_pytorch.py:568) in two tensors of the
 * same dtype.  label_grads [B,T,U,V] receives the gradient w.r.t. the token logits (as mi_tdt_backward's token
 * block) and duration_grads [B,T,U,D] the gradient w.r.t. the duration log-probs, i.e. minus the posterior of the
 * arcs of each duration (gpu_rnnt_kernel.py:1328-1341; no clamp, no FastEmit on these); padded cells get zeros in
 * both.  use_plain_rnnt != 0 (the omega branch): plain RNNT on the token logits, duration_grads all zero.
 * The workspace is mi_transducer_workspace_bytes(B, T, U, D).  In mi_tdt_split_loss both gradient pointers are
 * given or both are NULL (forward only).  prefill_label_grads / padding_zeroed: as for RNNT, on label_grads (the
 * duration gradient is written by a kernel of its own, padded cells included). */
int mi_tdt_split_forward(const void* label_acts, const void* duration_acts, int act_dtype, const int64_t* labels,
                         const int64_t* act_lens, const int64_t* label_lens, float* costs, int B, int T, int U, int V,
                         int D, const int32_t* durations_host, int blank, float fastemit_lambda, float sigma,
                         int use_plain_rnnt, int with_betas, void* prefill_label_grads, void* workspace,
                         size_t workspace_bytes, void* stream);
int mi_tdt_split_backward(const void* label_acts, int act_dtype, const int64_t* labels, const int64_t* act_lens,
                          const int64_t* label_lens, void* label_grads, void* duration_grads,
                          const float* grad_scale, int grad_scale_stride, float grad_mul, int padding_zeroed, int B,
                          int T, int U, int V, int D, const int32_t* durations_host, int blank, float fastemit_lambda,
                          float clamp, float sigma, int use_plain_rnnt, void* workspace, size_t workspace_bytes,
                          void* stream);
int mi_tdt_split_loss(const void* label_acts, const void* duration_acts, int act_dtype, const int64_t* labels,
                      const int64_t* act_lens, const int64_t* label_lens, float* costs, void* label_grads,
                      void* duration_grads, const float* grad_scale, int grad_scale_stride, float grad_mul, int B,
                      int T, int U, int V, int D, const int32_t* durations_host, int blank, float fastemit_lambda,
                      float clamp, float sigma, int use_plain_rnnt, int riders, void* workspace,
                      size_t workspace_bytes, void* stream);

/* ---- multi-blank transducer ---------------------------------------------------------
 * Replaces rnnt.py:366-483 (multiblank_rnnt_loss_gpu) and what it drives:
 * gpu_rnnt.py:296-509 (MultiblankGPURNNT), gpu_rnnt_kernel.py:410-885 (alphas, betas, gradient).
 * acts: [B,T,U,V] raw logits where V counts the tokens, the num_big_blanks big blanks and the
 * standard blank; big blank i (duration big_blank_durations_host[i] >= 1 frames, host int32
 * array) sits at index blank-1-i; one softmax covers all V entries and every arc pays -sigma.
 * workspace: mi_transducer_workspace_bytes(B, T, U, num_big_blanks).  num_big_blanks <=
 * MI_TRANSDUCER_MAX_BIG_BLANKS, durations <= MI_TRANSDUCER_MAX_BLANK_DURATION, and the LDS ring
 * (longest duration + 1) * (2 + capacity) * 64*ceil(U/64) * 8 bytes must fit 160 KB (capacity =
 * num_big_blanks rounded up to 1, 2, 4 or 8), else invalid value.  Other arguments as for RNNT. */
int mi_multiblank_forward(const void* acts, int act_dtype, const int64_t* labels, const int64_t* act_lens,
                          const int64_t* label_lens, float* costs, int B, int T, int U, int V, int num_big_blanks,
                          const int32_t* big_blank_durations_host, int blank, float fastemit_lambda, float sigma,
                          int with_betas, void* prefill_grads, void* workspace, size_t workspace_bytes, void* stream);

int mi_multiblank_backward(const void* acts, int act_dtype, const int64_t* labels, const int64_t* act_lens,
                           const int64_t* label_lens, void* grads, const float* grad_scale, int grad_scale_stride,
                           float grad_mul, int padding_zeroed, int B, int T, int U, int V, int num_big_blanks,
                           const int32_t* big_blank_durations_host, int blank, float fastemit_lambda, float clamp,
                           float sigma, void* workspace, size_t workspace_bytes, void* stream);

int mi_multiblank_loss(const void* acts, int act_dtype, const int64_t* labels, const int64_t* act_lens,
                       const int64_t* label_lens, float* costs, void* grads, const float* grad_scale,
                       int grad_scale_stride, float grad_mul, int B, int T, int U, int V, int num_big_blanks,
                       const int32_t* big_blank_durations_host, int blank, float fastemit_lambda, float clamp,
                       float sigma, int riders, void* workspace, size_t workspace_bytes, void* stream);

/* The two stages of a forward call on their own (mi_rnnt_forward = denominators + rnnt lattice,
 * mi_tdt_forward = denominators + tdt lattice), for callers that want to order other work between
 * them and for stage-level tests.  They mirror the reference's separately launched kernels:
 * reduce_max/reduce_exp (utils/cuda_utils/reduce.py:299-362) and compute_alphas/betas_kernel
 * (utils/cuda_utils/gpu_rnnt_kernel.py:73-269, :888-1241).  D = 0 for RNNT; the lattice calls need
 * the D the denominators were run with (it fixes the workspace layout). */
int mi_transducer_denominators(const void* acts, int act_dtype, const int64_t* labels, const int64_t* act_lens,
                               const int64_t* label_lens, int B, int T, int U, int V, int D, int blank,
                               void* workspace, size_t workspace_bytes, void* stream);
int mi_rnnt_lattice(const int64_t* act_lens, const int64_t* label_lens, float* costs, int B, int T, int U, int D,
                    float fastemit_lambda, int with_betas, void* workspace, size_t workspace_bytes, void* stream);
int mi_tdt_lattice(const int64_t* act_lens, const int64_t* label_lens, float* costs, int B, int T, int U, int D,
                   const int32_t* durations_host, float fastemit_lambda, float sigma, int with_betas, void* workspace,
                   size_t workspace_bytes, void* stream);

/* Zero-fills the gradient entries of every padded cell (t >= act_lens[b] or u > label_lens[b]) of
 * grads[B,T,U,VD] and touches nothing else.  The reference zero-fills the whole gradient tensor up
 * front (zeros_like, rnnt_pytorch.py:58; `grads *= 0`, gpu_rnnt.py:156); this is the part of that
 * work which survives, split out because it depends on the lengths only: enqueued on a second
 * stream after the denominators it fills the time HBM idles during the lattice recursion; the
 * backward call is then told padding_zeroed = 1 and may even run beside it (the two write disjoint
 * bytes).  Ordering between the streams, and the final join, are the caller's job. */
int mi_transducer_zero_padding(void* grads, int act_dtype, const int64_t* act_lens, const int64_t* label_lens, int B,
                               int T, int U, int VD, void* stream);

/* ---- compact log-prob op ---------------------------------------------------------------
 * Replaces rnnt_logprobs_triton (nemo/collections/asr/parts/k2/rnnt_logprobs_triton.py:20-228), the
 * producer of the graph-transducer losses' inputs (parts/k2/graph_transducer.py:517).
 *
 * forward:  target_scores[b,t,u] = log_softmax(logits[b,t,u,:])[targets[b,u]]   (u <  target_lens[b])
 *           blank_scores [b,t,u] = log_softmax(logits[b,t,u,:])[blank]          (u <= target_lens[b])
 *           for t < source_lens[b]; every other entry of the two float32 [B,T,U] arrays is set to 0
 *           (the reference leaves them at the zeros it allocated, :148-149).  U = max target length + 1.
 *           The workspace (mi_transducer_workspace_bytes(B, T, U, 0)) keeps the denominators.
 * backward: grad_logits[b,t,u,v] = -softmax_v * (gb + gt) + [v = blank] gb + [v = target] gt with
 *           gb = grad_blank_scores[b,t,u], gt = grad_target_scores[b,t,u] (0 where there is no target);
 *           when target == blank only gt is added, as the reference does (:118-122).  Cells outside
 *           an utterance get 0.  have_forward_state != 0: `workspace` is the one the forward call
 *           filled for the same inputs; 0: the denominators are recomputed first (what the
 *           reference always does, :90-104), at the price of one more read of the logits.
 * Lengths and targets are int64 device arrays ([B], [B,U-1]); logits/grad_logits share act_dtype. */
int mi_rnnt_logprobs_forward(const void* logits, int act_dtype, const int64_t* targets, const int64_t* source_lens,
                             const int64_t* target_lens, float* target_scores, float* blank_scores, int B, int T, int U,
                             int V, int blank, void* workspace, size_t workspace_bytes, void* stream);
int mi_rnnt_logprobs_backward(const void* logits, int act_dtype, const int64_t* targets, const int64_t* source_lens,
                              const int64_t* target_lens, const float* grad_target_scores,
                              const float* grad_blank_scores, void* grad_logits, int have_forward_state, int B, int T,
                              int U, int V, int blank, void* workspace, size_t workspace_bytes, void* stream);

/* ---- joint projection fused into the forward pass --------------------------------------
 * Replaces RNNTJoint.joint_after_projection followed by the loss forward
 * (nemo/collections/asr/modules/rnnt.py:1707-1724 and :1573-1578) for the default joint network
 * (activation, optional Dropout, Linear(H -> V); :1759-1777): the [B,T,U,V] tensor is never written.
 * `activation`: 0 ReLU, 1 tanh, 2 sigmoid (the three the reference accepts, :1762-1770); the activation's output is
 * rounded to bf16 as torch's is, and the backward takes its slope at that rounded output.
 *   f [B,T,H], g [B,U,H]: bf16, the projected encoder / prediction-network outputs (16-byte aligned);
 *   weight [V,H], bias [V] (nullable): float32 or bf16 (weight_dtype), the final Linear layer;
 *   logits = act(f[b,t] + g[b,u]) . weight^T + bias with bf16 operands and float32 accumulation
 *   (what the reference computes under bf16 autocast, minus its rounding of the logits to bf16).
 * costs[b] as mi_rnnt_forward; the workspace (mi_joint_workspace_bytes) ends up holding the same
 * lattice state.  H must be one of 256, 320, 384, 512, 640; V any.
 * Dropout of the hidden activations (the joint network's Dropout(p) between activation and Linear, :1772-1776):
 * dropout_p in [0, 1), 0 = none.  The keep mask is a pure function of (dropout_seed, cell, hidden unit): the
 * backward calls below must be given the same two values and then see the same mask; kept activations are scaled
 * by 1 / (1 - p).  mi_joint_dropout_mask writes that mask ([B*T*U][H] bytes, 1 = kept) for tests.
 * TDT (mi_joint_tdt_*): the Linear layer has V + D outputs, the token logits followed by the D duration logits
 * (rnnt_pytorch.py:563-568; D <= 8), weight [V+D,H], bias [V+D]; the token softmax covers the first V, the duration
 * logits are normalised among themselves, and the lattice is the TDT one (durations_host, sigma as mi_tdt_forward).
 * Multi-blank (mi_joint_multiblank_*): V counts the num_big_blanks <= 8 big blanks, which sit at rows blank-1-i of
 * the one softmax (as in mi_multiblank_forward); the lattice is the multi-blank one.
 * Every mi_joint_* call on a workspace takes the same D and num_big_blanks (both 0 for RNNT, at most one of them
 * non-zero): they are part of the workspace layout. */
int mi_joint_workspace_bytes(int B, int T, int U, int H, int V, int D, int num_big_blanks, size_t* out_bytes);
/* A forward call that a backward call is to follow keeps two things, a row per lattice cell in the kernel's tile
 * order -- utterance by utterance, cell t*U_b + u, each utterance padded to a multiple of 128 rows:
 *   saved_logits [saved_tiles*128][padded_vocabulary(V + D)] fp16: the logits (10 mantissa bits: the probabilities
 *     the backward forms from them are as exact as the bf16 gradient entries they are rounded to);
 *   saved_acts   [saved_tiles*128][H+16] bf16: the hidden activations (after activation and dropout) followed by
 *     1, 1 and zeros, so that column H of dlogits^T . saved_acts is the gradient of the bias; zero rows past an
 *     utterance's end.
 * Both NULL: nothing is kept (inference).  saved_tiles must be at least mi_joint_tile_bound(B, T, U), the number of
 * tiles of lattices without padding -- a bound known without reading the lengths back from the device; the tiles
 * actually used (device int32 *tile_count, nullable) come first. */
int mi_joint_tile_bound(int B, int T, int U); /* 0: no such lattice, or more tiles than the kernels index */
int mi_joint_rnnt_forward(const void* f, const void* g, const void* weight, const void* bias, int weight_dtype,
                          const int64_t* labels, const int64_t* act_lens, const int64_t* label_lens, float* costs,
                          int* tile_count, float dropout_p, unsigned long long dropout_seed, int activation, int B, int T, int U, int H,
                          int V, int blank, float fastemit_lambda, int with_betas, void* saved_logits,
                          void* saved_acts, long long saved_tiles, void* workspace, size_t workspace_bytes, void* stream);
int mi_joint_tdt_forward(const void* f, const void* g, const void* weight, const void* bias, int weight_dtype,
                         const int64_t* labels, const int64_t* act_lens, const int64_t* label_lens, float* costs,
                         int* tile_count, float dropout_p, unsigned long long dropout_seed, int activation, int B, int T, int U, int H,
                         int V, int D, const int32_t* durations_host, int blank, float fastemit_lambda, float sigma,
                         int with_betas, void* saved_logits, void* saved_acts, long long saved_tiles, void* workspace,
                         size_t workspace_bytes, void* stream);
int mi_joint_multiblank_forward(const void* f, const void* g, const void* weight, const void* bias, int weight_dtype,
                                const int64_t* labels, const int64_t* act_lens, const int64_t* label_lens, float* costs,
                                int* tile_count, float dropout_p, unsigned long long dropout_seed, int activation, int B, int T, int U,
                                int H, int V, int num_big_blanks, const int32_t* big_blank_durations_host, int blank,
                                float fastemit_lambda, float sigma, int with_betas, void* saved_logits,
                                void* saved_acts, long long saved_tiles, void* workspace, size_t workspace_bytes,
                                void* stream);
int mi_joint_dropout_mask(unsigned char* mask, float dropout_p, unsigned long long dropout_seed, int B, int T, int U,
                          int H, void* stream);

/* Backward of the fused joint (replaces autograd through the joint's Linear and the loss, modules/rnnt.py:1707-1724
 * and gpu_rnnt_kernel.py:340-403).  The gradient of the logits (grad_scale folded in as in mi_rnnt_backward; rows past
 * an utterance's end and columns beyond the vocabulary zero) is formed from the saved logits inside two kernels and
 * never written out:
 *   d_hidden [tiles*128][H] bf16 = dlogits . weight (rows as saved_logits; nullable: not wanted),
 *   dw_part [slices][padded_vocabulary][H] float32, db_part [slices][padded_vocabulary] float32: partial sums of
 *     d weight = dlogits^T . saved_acts and d bias = column sums of dlogits, one per slice of the rows; the caller adds
 *     the slices up (both nullable together: not wanted).  A good `slices` is 256 / (padded_vocabulary / 128).
 * `tiles`: the rows/128 that the buffers hold (the bound given to the forward call).  The workspace is the forward
 * call's, unchanged (forward with with_betas != 0); saved_logits and saved_acts are only read.  Nothing is read back to
 * the host and nothing is allocated.
 * TDT: columns V .. V+D-1 of dlogits are the gradient of the duration logits (gpu_rnnt_kernel.py:1244-1439 followed
 * by the log_softmax backward); no clamp on those, as in the reference. */
int mi_joint_padded_vocabulary(int V);
int mi_joint_rnnt_backward(const int64_t* labels, const int64_t* act_lens, const int64_t* label_lens,
                           void* saved_logits, const void* saved_acts, void* d_hidden, float* dw_part, float* db_part,
                           int slices, long long tiles, const float* grad_scale, int grad_scale_stride, float grad_mul,
                           int B, int T, int U, int H, int V, int blank, float fastemit_lambda, float clamp,
                           void* workspace, size_t workspace_bytes, void* stream);
int mi_joint_tdt_backward(const int64_t* labels, const int64_t* act_lens, const int64_t* label_lens,
                          void* saved_logits, const void* saved_acts, void* d_hidden, float* dw_part, float* db_part,
                          int slices, long long tiles, const float* grad_scale, int grad_scale_stride, float grad_mul,
                          int B, int T, int U, int H, int V, int D, const int32_t* durations_host, int blank,
                          float fastemit_lambda, float clamp, float sigma, void* workspace, size_t workspace_bytes,
                          void* stream);
int mi_joint_multiblank_backward(const int64_t* labels, const int64_t* act_lens, const int64_t* label_lens,
                                 void* saved_logits, const void* saved_acts, void* d_hidden, float* dw_part,
                                 float* db_part, int slices, long long tiles, const float* grad_scale,
                                 int grad_scale_stride, float grad_mul, int B, int T, int U, int H, int V,
                                 int num_big_blanks, const int32_t* big_blank_durations_host, int blank,
                                 float fastemit_lambda, float clamp, float sigma, void* workspace,
                                 size_t workspace_bytes, void* stream);

/* Backward of the fused joint, last step: d_hidden [rows][H] bf16 (= dlogits . weight, rows as above) times the
 * activation's derivative, summed over u into d_f [B,T,H] and over t into d_g [B,U,H] (float32; either may be NULL; frames
 * and label positions outside an utterance get zeros).  The derivative is recomputed from f and g (the forward
 * call's bf16 inputs), `tiles` is the same count as in mi_joint_rnnt_backward, the workspace the forward
 * call's.
 * With dg_part (float32 [chunks][B][U][H], 1 <= chunks <= T; U <= 256; d_g NULL, d_f not) both sums are formed in ONE
 * pass over d_hidden instead of one pass each: d_f as above, and for each of `chunks` runs of frames the run's share of
 * d g, which the caller adds up (d g = the sum of dg_part over its first axis; a fixed order of addition keeps the
 * result the same from call to call). */
int mi_joint_reduce_hidden(const void* d_hidden, const void* f, const void* g, const int64_t* act_lens,
                           const int64_t* label_lens, float* d_f, float* d_g, float* dg_part, int chunks, int tiles,
                           float dropout_p, unsigned long long dropout_seed, int activation, int B, int T, int U, int H,
                           int V, int D, int num_big_blanks, void* workspace, size_t workspace_bytes, void* stream);

/* Where the forward call left the packed weights inside its workspace: *rows x *pitch bf16, row n = weight[n, :]
 * followed by the bias columns (rows beyond V + D are zero in the first H columns), so that the d_hidden product
 * can read them in place. */
int mi_joint_packed_weights(const void* workspace, size_t workspace_bytes, int B, int T, int U, int H, int V, int D,
                            int num_big_blanks, const void** packed, int* rows, int* pitch);

/* Stage-level read-out for kernel parity tests (the reference tests launch each
 * kernel on its own, tests/collections/asr/numba/rnnt_loss/utils/test_gpu_rnnt_kernel.py):
 * copies what the last forward call left in `workspace` into plain [B,T,U] float32
 * arrays (cells outside an utterance's lattice are set to 0) and [B] log-likelihoods.
 * Any output pointer may be NULL.  betas / ll_backward are only meaningful after a
 * forward call with with_betas != 0. */
int mi_transducer_export_lattice(const void* workspace, size_t workspace_bytes, const int64_t* act_lens,
                                 const int64_t* label_lens, int B, int T, int U, int D, float* denom, float* alphas,
                                 float* betas, float* ll_forward, float* ll_backward, void* stream);

/* out[0] = max(act_lens), out[1] = max(label_lens) (device int64[2]).  The host reads them
 * back for the shape check of certify_inputs (rnnt_pytorch.py:628-634: T == max(act_lens),
 * U == max(label_lens) + 1), which the reference does with two torch.max calls. */
int mi_transducer_length_maxima(const int64_t* act_lens, const int64_t* label_lens, int B, int64_t* out,
                                void* stream);

/* ---- diagnostics ------------------------------------------------------------------------
 * Everything from here to the end of this header (mi_transducer_profile_*, mi_transducer_describe_plan,
 * mi_transducer_copy_probe, mi_transducer_prefill_record) binds NO interface of the reference: these are aids for
 * benchmarks, profiles and tests
 * of this library, and a drop-in user of the loss never calls them.
 *
 * Per-kernel timing of the launches a harness itself makes: after
 * mi_transducer_profile_enable(n, mask), each of the next n launches of every pipeline kernel
 * whose bit (1 << MI_PROFILE_*) is set in mask is bracketed by a pair of HIP events on its
 * stream (enable creates the events: the one place this library allocates).  An event pair
 * costs a few microseconds of queue time, so a harness that also times whole steps should
 * select only the kernel it needs.  mi_transducer_profile_read waits for the recorded
 * launches of one kernel class, returns their summed duration and count, and resets that
 * class.  The recording state is the library's only process-wide mutable state; it is guarded by a mutex, so the
 * calls are safe from any thread, but launches from several threads are then counted into the same classes.  Leave
 * it disabled outside benchmarks (disabled, a launch only reads one flag). */
#define MI_PROFILE_DENOM 0   /* denom_rows_kernel / denom_block_kernel / denom_gather_kernel / joint_lse_kernel */
#define MI_PROFILE_LATTICE 1 /* rnnt_lattice_kernel / tdt_lattice_pair_kernel / tdt_lattice_kernel */
#define MI_PROFILE_CELL 2    /* rnnt_cell_kernel / tdt_cell_kernel */
#define MI_PROFILE_GRAD 3    /* grad_rows_kernel / grad_block_kernel / grad_stream_kernel / joint_dhidden_kernel */
#define MI_PROFILE_ZERO 4    /* zero_padding_kernel */
#define MI_PROFILE_DWEIGHT 5 /* joint_dweight_kernel */
#define MI_PROFILE_KERNELS 6
int mi_transducer_profile_enable(int max_launches, unsigned kernel_mask);
int mi_transducer_profile_read(int kernel_id, float* total_ms, int* launches);
int mi_transducer_profile_disable(void);

/* Which kernels a call with this shape would launch, as text:
 * "denominators=...; lattice=...; cells=...; gradient=..." ("cells=-" when the gradient pass derives
 * its coefficients itself).  D = 0 for RNNT; for TDT pass the largest duration; for the multi-blank
 * loss D = 0, num_big_blanks > 0 (V counting the big blanks) and max_duration the longest big blank.  Assumes a gradient
 * buffer at the 16-byte phase of the logits.  Launches nothing.  For benchmarks, profiles and tests
 * that want to name (or pin) the kernel family a shape maps to. */
int mi_transducer_describe_plan(int act_dtype, int B, int T, int U, int V, int D, int max_duration,
                                int use_plain_rnnt, int num_big_blanks, char* out, size_t out_bytes);

/* Plain device-to-device copy of `bytes` (multiple of 16, 16-byte aligned pointers) with a
 * one-vector-per-thread kernel (the fastest streaming pattern measured): the known-size yardstick for hardware traffic
 * counters and for the copy bandwidth the GPU reaches in practice. */
int mi_transducer_copy_probe(const void* src, void* dst, size_t bytes, void* stream);

/* Where a workspace of this shape keeps the record of what the riders of the last forward call with prefill_grads
 * zero-filled: `*words` int32 starting at byte `*offset_bytes`.  Rows of row_bytes bytes go `*rows_per_item` to an
 * item (the last item of a frame may be shorter), items are numbered in memory order over (b, t, item of the frame),
 * and item i has had its padded rows filled iff  i / *words < record[i % *words].  Host arithmetic only.  For
 * benchmarks that report how many bytes moved from the gradient pass into the lattice launch, and for tests. */
int mi_transducer_prefill_record(int B, int T, int U, int D, size_t row_bytes, size_t* offset_bytes, int* words,
                                 int* rows_per_item);

#ifdef __cplusplus
}
#endif
#endif /* MI_TRANSDUCER_H_ */
