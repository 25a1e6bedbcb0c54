// MI355X (gfx950, wave64) transducer-loss kernels and their C ABI (include/mi_transducer.h).
//
// Pipeline of a forward + backward call (one stream, no host synchronisation, nothing allocated):
//   pass 1   denom_rows_kernel | denom_block_kernel | denom_gather_kernel      (mi_streaming.inc)
//            streams the valid rows of acts once (16-byte aligned loads, log-sum-exp per row) and leaves per
//            cell the denominator and, as one record of consecutive floats, the blank / label (/ duration /
//            big-blank) log-probabilities, the records in a SKEWED layout [b][t+u][u][record], so that an
//            anti-diagonal of the lattice is contiguous and a cell's record leaves in one store.
//   lattice  rnnt_lattice_kernel | tdt_lattice_pair_kernel | tdt_lattice_kernel  (mi_lattice.inc)
//            | multiblank_lattice_kernel | multiblank_lattice_pull_kernel        (mi_multiblank.inc)
//            alpha and beta over the anti-diagonals, accumulated in fp64 (only the log1p(exp(.)) term in fp32);
//            the alpha side writes costs.
//   cells    tdt_cell_kernel | multiblank_cell_kernel (RNNT: none, the gradient pass derives them itself)
//            one thread per lattice cell: the few numbers a gradient row needs, grad_scale folded in.
//   pass 2   grad_rows_kernel | grad_block_kernel | grad_stream_kernel          (mi_streaming.inc)
//            streams acts a second time and writes every gradient element once, zeros for padded cells included.
// The compact log-prob op (mi_logprobs.inc) reuses pass 1 and pass 2; the fused joint + loss (mi_joint.inc) replaces
// pass 1 and the producer of the logits by an MFMA kernel.  Host-side checks and launchers: mi_host.inc.
//
// Reference semantics restated here: nemo/collections/asr/parts/numba/rnnt_loss/
//   utils/cuda_utils/reduce.py:121-248, utils/cuda_utils/gpu_rnnt_kernel.py:73-885 and
//   :888-1439, utils/rnnt_helper.py:42-53,106-142, utils/cuda_utils/gpu_rnnt.py:125-231,296-509,563-743.

#include <hip/hip_runtime.h>
#include <math.h>
#include <stdio.h>
#include <stdint.h>
#include <stdlib.h>

#include <atomic>
#include <mutex>
#include <type_traits>
#include <vector>

#include "mi_transducer.h"

// Tunables of the two bandwidth passes (compile-time; the defaults are the measured best).
#ifndef MI_XCD_MAP
#define MI_XCD_MAP 1  // 1: each XCD streams one contiguous eighth of the (b,t) rows
#endif
#ifndef MI_NT_K1
#define MI_NT_K1 1    // non-temporal loads in the denominator pass
#endif
#ifndef MI_NT_K4
#define MI_NT_K4 1    // non-temporal loads in the gradient pass
#endif

namespace {

#include "mi_plan.h"
#include "mi_device.inc"
#include "mi_prefill.inc"
#include "mi_lattice.inc"
#include "mi_logprobs.inc"
#include "mi_multiblank.inc"
#include "mi_streaming.inc"
#include "mi_host.inc"

}  // namespace

// The fused joint + loss kernels and their entry points (outside the namespace: it declares its own extern "C" block).
#include "mi_joint.inc"

// ----------------------------------------------------------------------------------------
// C ABI
// ----------------------------------------------------------------------------------------
extern "C" {

int mi_transducer_abi_version(void) { return 20; }

int mi_transducer_workspace_bytes(int B, int T, int U, int D, size_t* out_bytes) {
  Layout L;
  if (!out_bytes || !make_layout(B, T, U, D, &L)) return MI_TRANSDUCER_INVALID_VALUE;
  *out_bytes = L.total;
  return MI_TRANSDUCER_SUCCESS;
}

int mi_rnnt_forward(const void* acts, int act_dtype, const int64_t* labels, const int64_t* act_lens,
                    const int64_t* label_lens, float* costs, int B, int T, int U, int V, int blank,
                    float fastemit_lambda, int with_betas, void* prefill_grads, void* workspace,
                    size_t workspace_bytes, void* stream) {
  Common c;
  if (!costs) return MI_TRANSDUCER_INVALID_VALUE;
  int st = check_common(acts, act_dtype, labels, act_lens, label_lens, B, T, U, V, 0, blank, workspace,
                        workspace_bytes, stream, &c);
  if (st) return st;
  if ((st = run_denom(c))) return st;
  return run_rnnt_lattice(c, costs, fastemit_lambda, with_betas, with_betas ? prefill_grads : nullptr);
}

int mi_rnnt_backward(const void* acts, int act_dtype, const int64_t* labels, const int64_t* act_lens,
                     const int64_t* label_lens, void* grads, const float* grad_scale, int grad_scale_stride,
                     float grad_mul, int padding_zeroed, int B, int T, int U, int V, int blank,
                     float fastemit_lambda, float clamp, void* workspace, size_t workspace_bytes, void* stream) {
  Common c;
  if (!grads || clamp < 0.f || grad_scale_stride < 0 || padding_zeroed < 0 || padding_zeroed > 2)
    return MI_TRANSDUCER_INVALID_VALUE;
  int st = check_common(acts, act_dtype, labels, act_lens, label_lens, B, T, U, V, 0, blank, workspace,
                        workspace_bytes, stream, &c);
  if (st) return st;
  const ScaleArg sc = {grad_scale, grad_scale_stride, grad_mul};
  const bool fused = rnnt_rows_fused(c, grads);
  if (!fused && (st = run_rnnt_cells(c, sc, fastemit_lambda, clamp))) return st;
  return run_grad_stream(c, grads, padding_flags(padding_zeroed), fused, sc, fastemit_lambda, clamp);
}

int mi_rnnt_loss(const void* acts, int act_dtype, const int64_t* labels, const int64_t* act_lens,
                 const int64_t* label_lens, float* costs, void* grads, const float* grad_scale,
                 int grad_scale_stride, float grad_mul, int B, int T, int U, int V, int blank, float fastemit_lambda,
                 float clamp, int riders, void* workspace, size_t workspace_bytes, void* stream) {
  if (!riders_arg_ok(riders)) return MI_TRANSDUCER_INVALID_VALUE;
  // (with riders the lattice launch zero-fills padded cells of grads while it runs; the gradient pass skips those)
  void* prefill = grads && riders_wanted(riders, B, T, U, V, act_dtype) ? grads : nullptr;
  int st = mi_rnnt_forward(acts, act_dtype, labels, act_lens, label_lens, costs, B, T, U, V, blank, fastemit_lambda,
                           grads != nullptr, prefill, workspace, workspace_bytes, stream);
  if (st || !grads) return st;
  return mi_rnnt_backward(acts, act_dtype, labels, act_lens, label_lens, grads, grad_scale, grad_scale_stride,
                          grad_mul, prefill ? 2 : 0, B, T, U, V, blank, fastemit_lambda, clamp, workspace,
                          workspace_bytes, stream);
}

// ----------------------------------------------------------------------------------------
// The one entry point that brings its own workspace: a device array that lives in the code object.
// ----------------------------------------------------------------------------------------
}  // extern "C"

static __device__ __align__(256) unsigned char scratch[MI_TRANSDUCER_STATIC_WORKSPACE_BYTES];

namespace {
constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices];  // per device: where that device holds its copy of `scratch`
std::mutex g_scratch_mutex;

// The address of `scratch` on the current device.  In host code the array's name is only a handle for the
// runtime, never a device address: the address comes from hipGetSymbolAddress, once per device.
int static_workspace(void** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return MI_TRANSDUCER_LAUNCH_FAILURE;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return MI_TRANSDUCER_LAUNCH_FAILURE;
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return MI_TRANSDUCER_SUCCESS;
}
}  // namespace

extern "C" {

int mi_transducer_init(void) {
  void* p;
  return static_workspace(&p);
}

int mi_rnnt_loss_static(const void* acts, int act_dtype, const int64_t* labels, const int64_t* act_lens,
                        const int64_t* label_lens, float* costs, void* grads, const float* grad_scale,
                        int grad_scale_stride, float grad_mul, int B, int T, int U, int V, int blank,
                        float fastemit_lambda, float clamp, int riders, void* stream) {
  Layout L;
  if (!make_layout(B, T, U, 0, &L)) return MI_TRANSDUCER_INVALID_VALUE;
  if (L.total > (size_t)MI_TRANSDUCER_STATIC_WORKSPACE_BYTES) return MI_TRANSDUCER_TOO_LARGE;
  void* ws = nullptr;
  const int st = static_workspace(&ws);
  if (st) return st;
  // nothing in the workspace has to start at zero: every kernel writes what later kernels of the call read, and
  // what is left there by an earlier call is never read
  return mi_rnnt_loss(acts, act_dtype, labels, act_lens, label_lens, costs, grads, grad_scale, grad_scale_stride,
                      grad_mul, B, T, U, V, blank, fastemit_lambda, clamp, riders, ws, L.total, stream);
}

int mi_tdt_forward(const void* acts, int act_dtype, const int64_t* labels, const int64_t* act_lens,
                   const int64_t* label_lens, float* costs, int B, int T, int U, int V, int D,
                   const int32_t* durations_host, int blank, float fastemit_lambda, float sigma, int use_plain_rnnt,
                   int with_betas, void* prefill_grads, void* workspace, size_t workspace_bytes, void* stream) {
  Common c;
  TdtParams prm;
  if (!costs) return MI_TRANSDUCER_INVALID_VALUE;
  if (!with_betas) prefill_grads = nullptr;
  int st = make_tdt_params(D, durations_host, sigma, &prm);
  if (st) return st;
  st = check_common(acts, act_dtype, labels, act_lens, label_lens, B, T, U, V, D, blank, workspace, workspace_bytes,
                    stream, &c);
  if (st) return st;
  if ((st = run_denom(c))) return st;
  // omega branch (gpu_rnnt.py:607-622): the plain RNNT recursion over the token logits
  if (use_plain_rnnt) return run_rnnt_lattice(c, costs, fastemit_lambda, with_betas, prefill_grads);
  return run_tdt_lattice(c, costs, fastemit_lambda, with_betas, prm, prefill_grads);
}

int mi_tdt_backward(const void* acts, int act_dtype, const int64_t* labels, const int64_t* act_lens,
                    const int64_t* label_lens, void* grads, const float* grad_scale, int grad_scale_stride,
                    float grad_mul, int padding_zeroed, int B, int T, int U, int V, int D,
                    const int32_t* durations_host, int blank, float fastemit_lambda, float clamp, float sigma,
                    int use_plain_rnnt, void* workspace, size_t workspace_bytes, void* stream) {
  Common c;
  TdtParams prm;
  if (!grads || clamp < 0.f || grad_scale_stride < 0 || padding_zeroed < 0 || padding_zeroed > 2)
    return MI_TRANSDUCER_INVALID_VALUE;
  const int pad_flag = padding_flags(padding_zeroed);
  int st = make_tdt_params(D, durations_host, sigma, &prm);
  if (st) return st;
  st = check_common(acts, act_dtype, labels, act_lens, label_lens, B, T, U, V, D, blank, workspace, workspace_bytes,
                    stream, &c);
  if (st) return st;
  const ScaleArg sc = {grad_scale, grad_scale_stride, grad_mul};
  if (use_plain_rnnt) {  // gpu_rnnt.py:646-682: token gradient from the RNNT kernel, duration gradient stays zero
    const bool fused = rnnt_rows_fused(c, grads);
    if (!fused && (st = run_rnnt_cells(c, sc, fastemit_lambda, clamp))) return st;
    return run_grad_stream(c, grads, kFlagZeroDurations | pad_flag, fused, sc, fastemit_lambda, clamp);
  }
  if ((st = run_tdt_cells(c, sc, fastemit_lambda, clamp, prm))) return st;
  return run_grad_stream(c, grads, pad_flag, false, sc, fastemit_lambda, clamp);
}

int mi_tdt_loss(const void* acts, int act_dtype, const int64_t* labels, const int64_t* act_lens,
                const int64_t* label_lens, float* costs, void* grads, const float* grad_scale, int grad_scale_stride,
                float grad_mul, int B, int T, int U, int V, int D, const int32_t* durations_host, int blank,
                float fastemit_lambda, float clamp, float sigma, int use_plain_rnnt, int riders, void* workspace,
                size_t workspace_bytes, void* stream) {
  if (!riders_arg_ok(riders)) return MI_TRANSDUCER_INVALID_VALUE;
  void* prefill = grads && riders_wanted(riders, B, T, U, V + D, act_dtype) ? grads : nullptr;
  int st = mi_tdt_forward(acts, act_dtype, labels, act_lens, label_lens, costs, B, T, U, V, D, durations_host, blank,
                          fastemit_lambda, sigma, use_plain_rnnt, grads != nullptr, prefill, workspace, workspace_bytes,
                          stream);
  if (st || !grads) return st;
  return mi_tdt_backward(acts, act_dtype, labels, act_lens, label_lens, grads, grad_scale, grad_scale_stride, grad_mul,
                         prefill ? 2 : 0, B, T, U, V, D, durations_host, blank, fastemit_lambda, clamp, sigma,
                         use_plain_rnnt, workspace, workspace_bytes, stream);
}

int mi_tdt_split_forward(const void* label_acts, const void* duration_acts, int act_dtype, const int64_t* labels,
                         const int64_t* act_lens, const int64_t* label_lens, float* costs, int B, int T, int U, int V,
                         int D, const int32_t* durations_host, int blank, float fastemit_lambda, float sigma,
                         int use_plain_rnnt, int with_betas, void* prefill_label_grads, void* workspace,
                         size_t workspace_bytes, void* stream) {
  Common c;
  TdtParams prm;
  if (!costs || !duration_acts) return MI_TRANSDUCER_INVALID_VALUE;
  if (!with_betas) prefill_label_grads = nullptr;
  int st = make_tdt_params(D, durations_host, sigma, &prm);
  if (st) return st;
  st = check_common(label_acts, act_dtype, labels, act_lens, label_lens, B, T, U, V, 0, blank, workspace,
                    workspace_bytes, stream, &c, 0, D);
  if (st) return st;
  if ((st = run_denom(c))) return st;
  if (use_plain_rnnt) return run_rnnt_lattice(c, costs, fastemit_lambda, with_betas, prefill_label_grads);
  if ((st = run_tdt_duration_planes(c, duration_acts, D))) return st;
  return run_tdt_lattice(c, costs, fastemit_lambda, with_betas, prm, prefill_label_grads);
}

int mi_tdt_split_backward(const void* label_acts, int act_dtype, const int64_t* labels, const int64_t* act_lens,
                          const int64_t* label_lens, void* label_grads, void* duration_grads,
                          const float* grad_scale, int grad_scale_stride, float grad_mul, int padding_zeroed, int B,
                          int T, int U, int V, int D, const int32_t* durations_host, int blank, float fastemit_lambda,
                          float clamp, float sigma, int use_plain_rnnt, void* workspace, size_t workspace_bytes,
                          void* stream) {
  Common c;
  TdtParams prm;
  if (!label_grads || !duration_grads || clamp < 0.f || grad_scale_stride < 0 || padding_zeroed < 0 ||
      padding_zeroed > 2)
    return MI_TRANSDUCER_INVALID_VALUE;
  const int pad_flag = padding_flags(padding_zeroed);
  int st = make_tdt_params(D, durations_host, sigma, &prm);
  if (st) return st;
  st = check_common(label_acts, act_dtype, labels, act_lens, label_lens, B, T, U, V, 0, blank, workspace,
                    workspace_bytes, stream, &c, 0, D);
  if (st) return st;
  const ScaleArg sc = {grad_scale, grad_scale_stride, grad_mul};
  if (use_plain_rnnt) {  // gpu_rnnt.py:646-682: token gradient from the RNNT kernel, duration gradient stays zero
    const bool fused = rnnt_rows_fused(c, label_grads);
    if (!fused && (st = run_rnnt_cells(c, sc, fastemit_lambda, clamp))) return st;
    if ((st = run_grad_stream(c, label_grads, pad_flag, fused, sc, fastemit_lambda, clamp))) return st;
    return run_tdt_duration_grads(c, duration_grads, D, 1);
  }
  if ((st = run_tdt_cells(c, sc, fastemit_lambda, clamp, prm, 1))) return st;
  if ((st = run_grad_stream(c, label_grads, pad_flag, false, sc, fastemit_lambda, clamp))) return st;
  return run_tdt_duration_grads(c, duration_grads, D, 0);
}

int mi_tdt_split_loss(const void* label_acts, const void* duration_acts, int act_dtype, const int64_t* labels,
                      const int64_t* act_lens, const int64_t* label_lens, float* costs, void* label_grads,
                      void* duration_grads, const float* grad_scale, int grad_scale_stride, float grad_mul, int B,
                      int T, int U, int V, int D, const int32_t* durations_host, int blank, float fastemit_lambda,
                      float clamp, float sigma, int use_plain_rnnt, int riders, void* workspace,
                      size_t workspace_bytes, void* stream) {
  if ((label_grads == nullptr) != (duration_grads == nullptr) || !riders_arg_ok(riders))
    return MI_TRANSDUCER_INVALID_VALUE;
  void* prefill = label_grads && riders_wanted(riders, B, T, U, V, act_dtype) ? label_grads : nullptr;
  int st = mi_tdt_split_forward(label_acts, duration_acts, act_dtype, labels, act_lens, label_lens, costs, B, T, U, V, D,
                                durations_host, blank, fastemit_lambda, sigma, use_plain_rnnt, label_grads != nullptr,
                                prefill, workspace, workspace_bytes, stream);
  if (st || !label_grads) return st;
  return mi_tdt_split_backward(label_acts, act_dtype, labels, act_lens, label_lens, label_grads, duration_grads,
                               grad_scale, grad_scale_stride, grad_mul, prefill ? 2 : 0, B, T, U, V, D, durations_host,
                               blank, fastemit_lambda, clamp, sigma, use_plain_rnnt, workspace, workspace_bytes, stream);
}

int mi_multiblank_forward(const void* acts, int act_dtype, const int64_t* labels, const int64_t* act_lens,
                          const int64_t* label_lens, float* costs, int B, int T, int U, int V, int num_big_blanks,
                          const int32_t* big_blank_durations_host, int blank, float fastemit_lambda, float sigma,
                          int with_betas, void* prefill_grads, void* workspace, size_t workspace_bytes, void* stream) {
  Common c;
  MbParams prm;
  if (!costs) return MI_TRANSDUCER_INVALID_VALUE;
  if (!with_betas) prefill_grads = nullptr;
  int st = make_mb_params(num_big_blanks, big_blank_durations_host, sigma, &prm);
  if (st) return st;
  st = check_common(acts, act_dtype, labels, act_lens, label_lens, B, T, U, V, 0, blank, workspace, workspace_bytes,
                    stream, &c, num_big_blanks);
  if (st) return st;
  if ((st = run_denom(c))) return st;
  return run_multiblank_lattice(c, costs, fastemit_lambda, with_betas, prm, prefill_grads);
}

int mi_multiblank_backward(const void* acts, int act_dtype, const int64_t* labels, const int64_t* act_lens,
                           const int64_t* label_lens, void* grads, const float* grad_scale, int grad_scale_stride,
                           float grad_mul, int padding_zeroed, int B, int T, int U, int V, int num_big_blanks,
                           const int32_t* big_blank_durations_host, int blank, float fastemit_lambda, float clamp,
                           float sigma, void* workspace, size_t workspace_bytes, void* stream) {
  Common c;
  MbParams prm;
  if (!grads || clamp < 0.f || grad_scale_stride < 0 || padding_zeroed < 0 || padding_zeroed > 2)
    return MI_TRANSDUCER_INVALID_VALUE;
  int st = make_mb_params(num_big_blanks, big_blank_durations_host, sigma, &prm);
  if (st) return st;
  st = check_common(acts, act_dtype, labels, act_lens, label_lens, B, T, U, V, 0, blank, workspace, workspace_bytes,
                    stream, &c, num_big_blanks);
  if (st) return st;
  const ScaleArg sc = {grad_scale, grad_scale_stride, grad_mul};
  if ((st = run_multiblank_cells(c, sc, fastemit_lambda, clamp, prm))) return st;
  // the workgroup-per-row gradient kernel writes the big blanks' entries itself; behind the other kernels a small
  // kernel overwrites them
  const bool folded = grad_block_plan(c, grads).RT != 0;
  const int flags = padding_flags(padding_zeroed) | (folded ? prm.NB << kFlagBigBlanksShift : 0);
  if ((st = run_grad_stream(c, grads, flags, false, sc, fastemit_lambda, clamp))) return st;
  return folded ? MI_TRANSDUCER_SUCCESS : run_multiblank_fixup(c, grads, prm);
}

int mi_multiblank_loss(const void* acts, int act_dtype, const int64_t* labels, const int64_t* act_lens,
                       const int64_t* label_lens, float* costs, void* grads, const float* grad_scale,
                       int grad_scale_stride, float grad_mul, int B, int T, int U, int V, int num_big_blanks,
                       const int32_t* big_blank_durations_host, int blank, float fastemit_lambda, float clamp,
                       float sigma, int riders, void* workspace, size_t workspace_bytes, void* stream) {
  if (!riders_arg_ok(riders)) return MI_TRANSDUCER_INVALID_VALUE;
  void* prefill = grads && riders_wanted(riders, B, T, U, V, act_dtype) ? grads : nullptr;
  int st = mi_multiblank_forward(acts, act_dtype, labels, act_lens, label_lens, costs, B, T, U, V, num_big_blanks,
                                 big_blank_durations_host, blank, fastemit_lambda, sigma, grads != nullptr, prefill,
                                 workspace, workspace_bytes, stream);
  if (st || !grads) return st;
  return mi_multiblank_backward(acts, act_dtype, labels, act_lens, label_lens, grads, grad_scale, grad_scale_stride,
                                grad_mul, prefill ? 2 : 0, B, T, U, V, num_big_blanks, big_blank_durations_host, blank, fastemit_lambda,
                                clamp, sigma, workspace, workspace_bytes, stream);
}

int mi_rnnt_logprobs_forward(const void* logits, int act_dtype, const int64_t* targets, const int64_t* source_lens,
                             const int64_t* target_lens, float* target_scores, float* blank_scores, int B, int T, int U,
                             int V, int blank, void* workspace, size_t workspace_bytes, void* stream) {
  Common c;
  if (!target_scores || !blank_scores) return MI_TRANSDUCER_INVALID_VALUE;
  int st = check_common(logits, act_dtype, targets, source_lens, target_lens, B, T, U, V, 0, blank, workspace,
                        workspace_bytes, stream, &c);
  if (st) return st;
  if ((st = run_denom(c))) return st;
  return run_logprobs_export(c, target_scores, blank_scores);
}

int mi_rnnt_logprobs_backward(const void* logits, int act_dtype, const int64_t* targets, const int64_t* source_lens,
                              const int64_t* target_lens, const float* grad_target_scores,
                              const float* grad_blank_scores, void* grad_logits, int have_forward_state, int B, int T,
                              int U, int V, int blank, void* workspace, size_t workspace_bytes, void* stream) {
  Common c;
  if (!grad_target_scores || !grad_blank_scores || !grad_logits) return MI_TRANSDUCER_INVALID_VALUE;
  int st = check_common(logits, act_dtype, targets, source_lens, target_lens, B, T, U, V, 0, blank, workspace,
                        workspace_bytes, stream, &c);
  if (st) return st;
  if (!have_forward_state && (st = run_denom(c))) return st;
  if ((st = run_logprobs_cells(c, grad_target_scores, grad_blank_scores))) return st;
  const ScaleArg sc = {nullptr, 0, 1.f};
  return run_grad_stream(c, grad_logits, 0, false, sc, 0.f, 0.f);
}

int mi_transducer_export_lattice(const void* workspace, size_t workspace_bytes, const int64_t* act_lens,
                                 const int64_t* label_lens, int B, int T, int U, int D, float* denom, float* alphas,
                                 float* betas, float* ll_forward, float* ll_backward, void* stream) {
  Layout L;
  if (!workspace || !act_lens || !label_lens || !make_layout(B, T, U, D, &L) || workspace_bytes < L.total)
    return MI_TRANSDUCER_INVALID_VALUE;
  const char* ws = (const char*)workspace;
  const long long cells = (long long)B * T * U;
  const unsigned grid = (unsigned)((cells + 255) / 256);
  hipLaunchKernelGGL(export_lattice_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream,
                     (const float*)(ws + L.off_denom), (const double*)(ws + L.off_alphas),
                     (const double*)(ws + L.off_betas), (const double*)(ws + L.off_ll),
                     (const float*)(ws + L.off_arcs), act_lens, label_lens, denom, alphas, betas,
                     ll_forward, ll_backward, B, T, U, L.ND, L.Us, L.A, cells);
  return launch_status();
}

int mi_transducer_prefill_record(int B, int T, int U, int D, size_t row_bytes, size_t* offset_bytes, int* words,
                                 int* rows_per_item) {
  Layout L;
  if (!offset_bytes || !words || !rows_per_item || row_bytes == 0 || !make_layout(B, T, U, D, &L))
    return MI_TRANSDUCER_INVALID_VALUE;
  *offset_bytes = L.off_fill + (size_t)kFillProgress * sizeof(int);
  *words = kFillMaxRiders;
  *rows_per_item = 1 << prefill_log_rows(row_bytes);
  return MI_TRANSDUCER_SUCCESS;
}

int mi_transducer_length_maxima(const int64_t* act_lens, const int64_t* label_lens, int B, int64_t* out,
                                void* stream) {
  if (!act_lens || !label_lens || !out || B <= 0) return MI_TRANSDUCER_INVALID_VALUE;
  hipLaunchKernelGGL(length_maxima_kernel, dim3(1), dim3(256), 0, (hipStream_t)stream, act_lens, label_lens, B, out);
  return launch_status();
}

int mi_transducer_denominators(const void* acts, int act_dtype, const int64_t* labels, const int64_t* act_lens,
                               const int64_t* label_lens, int B, int T, int U, int V, int D, int blank,
                               void* workspace, size_t workspace_bytes, void* stream) {
  Common c;
  int st = check_common(acts, act_dtype, labels, act_lens, label_lens, B, T, U, V, D, blank, workspace,
                        workspace_bytes, stream, &c);
  if (st) return st;
  return run_denom(c);
}

int mi_rnnt_lattice(const int64_t* act_lens, const int64_t* label_lens, float* costs, int B, int T, int U, int D,
                    float fastemit_lambda, int with_betas, void* workspace, size_t workspace_bytes, void* stream) {
  Common c;
  if (!costs || !act_lens || !label_lens || !workspace) return MI_TRANSDUCER_INVALID_VALUE;
  if (!make_layout(B, T, U, D, &c.L) || workspace_bytes < c.L.total || ((uintptr_t)workspace & 255))
    return MI_TRANSDUCER_INVALID_VALUE;
  c.act_lens = act_lens; c.label_lens = label_lens;
  c.B = B; c.T = T; c.U = U; c.D = D;
  c.ws = (char*)workspace; c.ws_bytes = workspace_bytes; c.stream = (hipStream_t)stream;
  return run_rnnt_lattice(c, costs, fastemit_lambda, with_betas);
}

int mi_tdt_lattice(const int64_t* act_lens, const int64_t* label_lens, float* costs, int B, int T, int U, int D,
                   const int32_t* durations_host, float fastemit_lambda, float sigma, int with_betas, void* workspace,
                   size_t workspace_bytes, void* stream) {
  Common c;
  TdtParams prm;
  if (!costs || !act_lens || !label_lens || !workspace) return MI_TRANSDUCER_INVALID_VALUE;
  int st = make_tdt_params(D, durations_host, sigma, &prm);
  if (st) return st;
  if (!make_layout(B, T, U, D, &c.L) || workspace_bytes < c.L.total || ((uintptr_t)workspace & 255))
    return MI_TRANSDUCER_INVALID_VALUE;
  c.act_lens = act_lens; c.label_lens = label_lens;
  c.B = B; c.T = T; c.U = U; c.D = D;
  c.ws = (char*)workspace; c.ws_bytes = workspace_bytes; c.stream = (hipStream_t)stream;
  return run_tdt_lattice(c, costs, fastemit_lambda, with_betas, prm);
}

int mi_transducer_zero_padding(void* grads, int act_dtype, const int64_t* act_lens, const int64_t* label_lens, int B,
                               int T, int U, int VD, void* stream) {
  if (!grads || !act_lens || !label_lens || B <= 0 || T <= 0 || U <= 0 || VD <= 0) return MI_TRANSDUCER_INVALID_VALUE;
  if (act_dtype != MI_DTYPE_F32 && act_dtype != MI_DTYPE_BF16 && act_dtype != MI_DTYPE_F16)
    return MI_TRANSDUCER_INVALID_VALUE;
  if ((long long)B * T > 65535LL * 8) return MI_TRANSDUCER_INVALID_VALUE;
  const int nchunks = (U + kChunkRows - 1) / kChunkRows;
  const int nblocks = nchunks * B * T;
  const unsigned turn = 8u * MI_XCD_SPAN;
  const dim3 grid(((unsigned)nblocks + turn - 1) / turn * turn, 1, 1);
  ProfScope prof(MI_PROFILE_ZERO, (hipStream_t)stream);
#define LAUNCH_ZERO(DT)                                                                                          \
  hipLaunchKernelGGL(zero_padding_kernel<DT>, grid, dim3(kRowThreads), 0, (hipStream_t)stream, grads, act_lens,   \
                     label_lens, T, U, VD, nchunks, nblocks, make_griddiv(nchunks, T))
  if (act_dtype == MI_DTYPE_F32) LAUNCH_ZERO(MI_DTYPE_F32);
  else if (act_dtype == MI_DTYPE_BF16) LAUNCH_ZERO(MI_DTYPE_BF16);
  else LAUNCH_ZERO(MI_DTYPE_F16);
#undef LAUNCH_ZERO
  return launch_status();
}

int mi_transducer_profile_enable(int max_launches, unsigned kernel_mask) {
  if (max_launches <= 0 || max_launches > 65536 || kernel_mask == 0) return MI_TRANSDUCER_INVALID_VALUE;
  std::lock_guard<std::mutex> lock(g_prof_mutex);
  g_prof_armed = false;
  g_prof.on = false;
  for (int k = 0; k < MI_PROFILE_KERNELS; ++k) {
    while ((int)g_prof.start[k].size() < max_launches) {
      hipEvent_t a, b;
      if (hipEventCreate(&a) != hipSuccess || hipEventCreate(&b) != hipSuccess) return MI_TRANSDUCER_LAUNCH_FAILURE;
      g_prof.start[k].push_back(a);
      g_prof.stop[k].push_back(b);
    }
    g_prof.count[k] = 0;
  }
  g_prof.cap = max_launches;
  g_prof.mask = kernel_mask;
  g_prof.on = true;
  g_prof_armed = true;
  return MI_TRANSDUCER_SUCCESS;
}

int mi_transducer_profile_read(int kernel_id, float* total_ms, int* launches) {
  if (kernel_id < 0 || kernel_id >= MI_PROFILE_KERNELS || !total_ms || !launches) return MI_TRANSDUCER_INVALID_VALUE;
  std::lock_guard<std::mutex> lock(g_prof_mutex);
  float total = 0.f;
  const int n = g_prof.count[kernel_id];
  for (int i = 0; i < n; ++i) {
    float ms = 0.f;
    if (hipEventSynchronize(g_prof.stop[kernel_id][i]) != hipSuccess ||
        hipEventElapsedTime(&ms, g_prof.start[kernel_id][i], g_prof.stop[kernel_id][i]) != hipSuccess)
      return MI_TRANSDUCER_LAUNCH_FAILURE;
    total += ms;
  }
  *total_ms = total;
  *launches = n;
  g_prof.count[kernel_id] = 0;
  return MI_TRANSDUCER_SUCCESS;
}

int mi_transducer_profile_disable(void) {
  std::lock_guard<std::mutex> lock(g_prof_mutex);
  g_prof_armed = false;
  g_prof.on = false;
  return MI_TRANSDUCER_SUCCESS;
}

int mi_transducer_describe_plan(int act_dtype, int B, int T, int U, int V, int D, int max_duration,
                                int use_plain_rnnt, int num_big_blanks, char* out, size_t out_bytes) {
  Common c;
  if (!out || out_bytes == 0 || V <= 0 || num_big_blanks < 0 || num_big_blanks > MI_TRANSDUCER_MAX_BIG_BLANKS ||
      (num_big_blanks > 0 && D != 0) || !make_layout(B, T, U, num_big_blanks ? num_big_blanks : D, &c.L))
    return MI_TRANSDUCER_INVALID_VALUE;
  if (act_dtype != MI_DTYPE_F32 && act_dtype != MI_DTYPE_BF16 && act_dtype != MI_DTYPE_F16)
    return MI_TRANSDUCER_INVALID_VALUE;
  c.acts = nullptr; c.dt = act_dtype; c.B = B; c.T = T; c.U = U; c.V = V; c.D = D; c.nbig = 0;
  const char* dt = act_dtype == MI_DTYPE_F32 ? "f32" : (act_dtype == MI_DTYPE_BF16 ? "bf16" : "f16");
  char denom[96], lattice[96], cells[48], grad[112];
  const BlockPlan dp = denom_block_plan(c);
  if (dp.RT) snprintf(denom, sizeof denom, "denom_block_kernel<%s, RT=%d, NVT=%d>", dt, dp.RT, dp.NVT);
  else if (denom_rows_R(c)) snprintf(denom, sizeof denom, "denom_rows_kernel<%s, R=%d, RPW=%d>", dt, denom_rows_R(c), denom_rows_per_wave(denom_rows_R(c)));
  else snprintf(denom, sizeof denom, "denom_gather_kernel<%s>", dt);
  const bool tdt = D > 0 && !use_plain_rnnt;
  const bool mb = num_big_blanks > 0;
  if (mb) {
    const int nbc = num_big_blanks <= 1 ? 1 : (num_big_blanks <= 2 ? 2 : (num_big_blanks <= 4 ? 4 : 8));
    const size_t lds = (size_t)(max_duration + 1) * (2 + nbc) * c.L.Us * sizeof(double);
    if (lds > 160 * 1024) snprintf(lattice, sizeof lattice, "multiblank_lattice_pull_kernel");
    else snprintf(lattice, sizeof lattice, "multiblank_lattice_kernel<NBC=%d>", nbc);
  } else if (D == 0 || use_plain_rnnt) {
    snprintf(lattice, sizeof lattice, "rnnt_lattice_kernel<K=%d>", c.L.K);
  } else {
    const int R = max_duration + 2;
    const size_t lds_block = (size_t)R * 2 * D * c.L.Us * sizeof(double);
    if (D <= 8 && c.L.Us <= 256 && lds_block <= 160 * 1024) snprintf(lattice, sizeof lattice, "tdt_lattice_pair_kernel<D=%d>", D);
    else snprintf(lattice, sizeof lattice, "tdt_lattice_kernel<K=%d>", c.L.K);
  }
  // a gradient buffer at the 16-byte phase of the logits is assumed (what every allocator returns)
  const BlockPlan gp = grad_block_plan(c, nullptr);
  const bool fused = !tdt && !mb && rnnt_rows_fused(c, nullptr);
  snprintf(cells, sizeof cells, "%s", fused ? "-" : (mb ? "multiblank_cell_kernel" : (tdt ? "tdt_cell_kernel" : "rnnt_cell_kernel")));
  if (gp.RT) snprintf(grad, sizeof grad, "grad_block_kernel<%s, RT=%d, NVT=%d, %s>", dt, gp.RT, gp.NVT, fused ? "fused" : "coef");
  else if (rows_R(c)) snprintf(grad, sizeof grad, "grad_rows_kernel<%s, R=%d, %s>", dt, rows_R(c), fused ? "fused" : "coef");
  else snprintf(grad, sizeof grad, "grad_stream_kernel<%s>", dt);
  const int n = snprintf(out, out_bytes, "denominators=%s; lattice=%s; cells=%s; gradient=%s%s", denom, lattice, cells,
                         grad, (mb && !gp.RT) ? " + multiblank_fixup_kernel" : "");
  return (n < 0 || (size_t)n >= out_bytes) ? MI_TRANSDUCER_INVALID_VALUE : MI_TRANSDUCER_SUCCESS;
}

int mi_transducer_copy_probe(const void* src, void* dst, size_t bytes, void* stream) {
  if (!src || !dst || bytes == 0 || (bytes & 15) || ((uintptr_t)src & 15) || ((uintptr_t)dst & 15))
    return MI_TRANSDUCER_INVALID_VALUE;
  const size_t nvec = bytes / 16;
  const size_t turn = 8u * MI_XCD_SPAN;
  const size_t blocks = ((nvec + 255) / 256 + turn - 1) / turn * turn;
  if (blocks > 0x7fffffffu) return MI_TRANSDUCER_INVALID_VALUE;
  hipLaunchKernelGGL(copy_probe_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (const uint4*)src,
                     (uint4*)dst, nvec);
  return launch_status();
}

}  // extern "C"
