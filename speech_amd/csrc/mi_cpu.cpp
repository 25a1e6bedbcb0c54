// Host (CPU) implementation of the RNNT loss behind include/mi_transducer_cpu.h.
//
// The reference computes RNNTLossNumba on CPU tensors too (rnnt_pytorch.py:420-435 -> rnnt.py:39-135 ->
// utils/cpu_utils/cpu_rnnt.py:164-422): the module log-softmaxes the logits with torch, CPURNNT walks alpha and beta
// per utterance over a compact [T_b, U_b, 2] table of blank / label log-probs and leaves a sparse gradient w.r.t.
// the log-probs (two entries per cell), torch autograd turns that into the gradient w.r.t. the logits, and a hook
// clamps the result (cpu_rnnt.py:141-161).  This file does the same arithmetic without the intermediate tensors:
//   forward   per row: max and log-sum-exp (the log_softmax denominator); per utterance: alpha, beta, costs
//   backward  per row: g_v = (softmax_v * (P_blank + P_label) - [v = blank] P_blank - [v = label] P_label) * scale,
//             then the clamp; P_* are the arc posteriors exp(alpha + lp + beta' - ll) (label arc times 1 + lambda),
//             i.e. the log-softmax backward applied to the reference's sparse gradient (cpu_rnnt.py:327-343).
// Faithful to the reference's CPU path where it differs from its GPU path:
//   * posteriors are normalised by the BACKWARD log-likelihood beta(0,0) (cpu_rnnt.py:325);
//   * FastEmit scales the label-arc posterior only; there is no extra p_v * lambda * P_label term (the GPU kernel
//     has one, gpu_rnnt_kernel.py:356-372);
//   * when a label equals the blank id the label entry overwrites the blank entry of the sparse gradient
//     (assignment, not accumulation, cpu_rnnt.py:329-337);
//   * the clamp acts on the finished gradient, after the 1/B of reduction='mean' and after grad_output
//     (the hook sits in front of log_softmax in the autograd graph).
// Lattice values are kept in double (the reference keeps float32); utterances run in parallel under OpenMP.

#include "mi_transducer_cpu.h"

#include <math.h>
#include <stddef.h>
#include <stdint.h>

#include <algorithm>
#include <limits>
#include <vector>

#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

struct Shape {
  int B, T, U, V, blank;
  size_t cells() const { return (size_t)B * T * U; }
};

struct Workspace {
  float* denom;    // [B,T,U]  -logsumexp of the row (valid cells)
  double* alphas;  // [B,T,U]
  double* betas;   // [B,T,U]
  double* ll;      // [B][2]   forward, backward
};

size_t workspace_bytes(size_t cells, int B) {
  return cells * (sizeof(float) + 2 * sizeof(double)) + (size_t)B * 2 * sizeof(double) + 64;
}

Workspace carve(void* base, size_t cells, int B) {
  // doubles first: the base is 8-byte aligned (checked by the caller)
  Workspace w;
  char* p = (char*)base;
  w.alphas = (double*)p;  p += cells * sizeof(double);
  w.betas = (double*)p;   p += cells * sizeof(double);
  w.ll = (double*)p;      p += (size_t)B * 2 * sizeof(double);
  w.denom = (float*)p;
  return w;
}

inline int clamp_len(int64_t v, int lo, int hi) { return (int)std::min<int64_t>(std::max<int64_t>(v, lo), hi); }

// log(exp(a) + exp(b)); an infinite operand yields the other one (cpu_rnnt.py:40-53)
inline double lse2(double a, double b) {
  if (std::isinf(a)) return b;
  if (std::isinf(b)) return a;
  return a > b ? a + log1p(exp(b - a)) : b + log1p(exp(a - b));
}

bool check(const Shape& s, const void* acts, const int64_t* labels, const int64_t* act_lens, const int64_t* label_lens,
           const void* ws, size_t ws_bytes) {
  if (!acts || !act_lens || !label_lens || !ws) return false;
  if (s.B <= 0 || s.T <= 0 || s.U <= 0 || s.V <= 0 || s.blank < 0 || s.blank >= s.V) return false;
  if (s.U > 1 && !labels) return false;
  if (((uintptr_t)ws & 7) || ws_bytes < workspace_bytes(s.cells(), s.B)) return false;
  return true;
}

int threads_for(int num_threads, int B) {
#ifdef _OPENMP
  const int avail = omp_get_max_threads();
  int n = num_threads > 0 ? std::min(num_threads, avail) : avail;
  return std::max(1, std::min(n, B));
#else
  (void)num_threads; (void)B;
  return 1;
#endif
}

// one utterance: denominators of its valid rows, then alpha and beta over [Tb, Ub]
void forward_utterance(const Shape& s, const float* acts, const int64_t* labels, int b, int Tb, int Ub,
                       const Workspace& w, float lambda, float* cost) {
  const size_t cell0 = (size_t)b * s.T * s.U;
  const int V = s.V, U = s.U;
  float* dn = w.denom + cell0;
  for (int t = 0; t < Tb; ++t) {
    for (int u = 0; u < Ub; ++u) {
      const float* x = acts + (cell0 + (size_t)t * U + u) * V;
      float m = x[0];
      for (int v = 1; v < V; ++v) m = std::max(m, x[v]);
      double acc = 0.0;
      for (int v = 0; v < V; ++v) acc += (double)expf(x[v] - m);
      dn[(size_t)t * U + u] = -m - (float)log(acc);
    }
  }
  auto lp = [&](int t, int u, int v) {
    const size_t c = (size_t)t * U + u;
    return (double)(acts[(cell0 + c) * V + v] + dn[c]);
  };
  auto lab = [&](int u) { return clamp_len(labels[(size_t)b * (U - 1) + u], 0, V - 1); };
  double* a = w.alphas + cell0;
  double* bt = w.betas + cell0;
  // alpha (cpu_rnnt.py:246-276)
  a[0] = 0.0;
  for (int t = 0; t < Tb; ++t) {
    for (int u = 0; u < Ub; ++u) {
      if (t == 0 && u == 0) continue;
      const double no_emit = t > 0 ? a[(size_t)(t - 1) * U + u] + lp(t - 1, u, s.blank)
                                   : -std::numeric_limits<double>::infinity();
      const double emit = u > 0 ? a[(size_t)t * U + u - 1] + lp(t, u - 1, lab(u - 1))
                                : -std::numeric_limits<double>::infinity();
      a[(size_t)t * U + u] = lse2(emit, no_emit);
    }
  }
  const double ll_forward = a[(size_t)(Tb - 1) * U + Ub - 1] + lp(Tb - 1, Ub - 1, s.blank);
  // beta (cpu_rnnt.py:303-323)
  bt[(size_t)(Tb - 1) * U + Ub - 1] = lp(Tb - 1, Ub - 1, s.blank);
  for (int t = Tb - 1; t >= 0; --t) {
    for (int u = Ub - 1; u >= 0; --u) {
      if (t == Tb - 1 && u == Ub - 1) continue;
      const double no_emit = t < Tb - 1 ? bt[(size_t)(t + 1) * U + u] + lp(t, u, s.blank)
                                        : -std::numeric_limits<double>::infinity();
      const double emit = u < Ub - 1 ? bt[(size_t)t * U + u + 1] + lp(t, u, lab(u))
                                     : -std::numeric_limits<double>::infinity();
      bt[(size_t)t * U + u] = lse2(emit, no_emit);
    }
  }
  w.ll[2 * b] = ll_forward;
  w.ll[2 * b + 1] = bt[0];
  // cpu_rnnt.py:236-244: the cost is -llForward * (1 + lambda), in float32
  const float llf = (float)ll_forward;
  *cost = -(llf + llf * lambda);
}

void backward_utterance(const Shape& s, const float* acts, const int64_t* labels, int b, int Tb, int Ub,
                        const Workspace& w, float lambda, float clamp, float scale, bool wrt_log_probs, float* grads) {
  const size_t cell0 = (size_t)b * s.T * s.U;
  const int V = s.V, U = s.U, T = s.T;
  const float* dn = w.denom + cell0;
  const double* a = w.alphas + cell0;
  const double* bt = w.betas + cell0;
  const double ll = w.ll[2 * b + 1];  // the backward one (cpu_rnnt.py:325)
  const double fast = log1p((double)lambda);
  for (int t = 0; t < T; ++t) {
    for (int u = 0; u < U; ++u) {
      const size_t c = (size_t)t * U + u;
      float* g = grads + (cell0 + c) * V;
      if (t >= Tb || u >= Ub) {
        std::fill(g, g + V, 0.f);
        continue;
      }
      const float* x = acts + (cell0 + c) * V;
      const double lpb = (double)(x[s.blank] + dn[c]);
      // sparse gradient w.r.t. the log-probs: at most one entry at the blank and one at the label
      double g_blank = 0.0, g_label = 0.0;
      int label = -1;
      if (t < Tb - 1) g_blank = -exp(lpb + a[c] + bt[c + U] - ll);
      else if (u == Ub - 1) g_blank = -exp(lpb + a[c] - ll);
      if (u < Ub - 1) {
        label = clamp_len(labels[(size_t)b * (U - 1) + u], 0, V - 1);
        g_label = -exp(fast + (double)(x[label] + dn[c]) + a[c] + bt[c + 1] - ll);
        if (label == s.blank) g_blank = 0.0;  // the label entry overwrites the blank entry
      }
      if (wrt_log_probs) {  // the reference's own output: the sparse row, nothing else (cpu_rnnt.py:327-343)
        std::fill(g, g + V, 0.f);
        if (g_blank != 0.0) g[s.blank] = (float)g_blank * scale;
        if (label >= 0) g[label] = (float)g_label * scale;
        continue;
      }
      const float total = (float)(g_blank + g_label);  // sum of the sparse row
      const float d = dn[c];
      for (int v = 0; v < V; ++v) g[v] = -expf(x[v] + d) * total;
      g[s.blank] += (float)g_blank;
      if (label >= 0) g[label] += (float)g_label;
      if (scale != 1.f)
        for (int v = 0; v < V; ++v) g[v] *= scale;
      if (clamp > 0.f)
        for (int v = 0; v < V; ++v) g[v] = std::min(std::max(g[v], -clamp), clamp);
    }
  }
}

}  // namespace

extern "C" {

int mi_transducer_cpu_abi_version(void) { return 1; }

int mi_rnnt_cpu_workspace_bytes(int B, int T, int U, size_t* out_bytes) {
  if (!out_bytes || B <= 0 || T <= 0 || U <= 0) return MI_TRANSDUCER_CPU_INVALID_VALUE;
  *out_bytes = workspace_bytes((size_t)B * T * U, B);
  return MI_TRANSDUCER_CPU_SUCCESS;
}

int mi_rnnt_cpu_forward(const float* acts, const int64_t* labels, const int64_t* act_lens, const int64_t* label_lens,
                        float* costs, int B, int T, int U, int V, int blank, float fastemit_lambda, void* workspace,
                        size_t workspace_bytes_, int num_threads) {
  const Shape s{B, T, U, V, blank};
  if (!costs || !check(s, acts, labels, act_lens, label_lens, workspace, workspace_bytes_))
    return MI_TRANSDUCER_CPU_INVALID_VALUE;
  const Workspace w = carve(workspace, s.cells(), B);
  const int nthreads = threads_for(num_threads, B);
  (void)nthreads;
#pragma omp parallel for schedule(dynamic, 1) num_threads(nthreads)
  for (int b = 0; b < B; ++b) {
    const int Tb = clamp_len(act_lens[b], 1, T), Ub = clamp_len(label_lens[b] + 1, 1, U);
    forward_utterance(s, acts, labels, b, Tb, Ub, w, fastemit_lambda, costs + b);
  }
  return MI_TRANSDUCER_CPU_SUCCESS;
}

int mi_rnnt_cpu_backward(const float* acts, const int64_t* labels, const int64_t* act_lens, const int64_t* label_lens,
                         float* grads, const float* grad_scale, int grad_scale_stride, float grad_mul, int B, int T,
                         int U, int V, int blank, float fastemit_lambda, float clamp, int wrt_log_probs,
                         const void* workspace, size_t workspace_bytes_, int num_threads) {
  const Shape s{B, T, U, V, blank};
  if (!grads || clamp < 0.f || grad_scale_stride < 0 ||
      !check(s, acts, labels, act_lens, label_lens, workspace, workspace_bytes_))
    return MI_TRANSDUCER_CPU_INVALID_VALUE;
  const Workspace w = carve(const_cast<void*>(workspace), s.cells(), B);
  const int nthreads = threads_for(num_threads, B);
  (void)nthreads;
#pragma omp parallel for schedule(dynamic, 1) num_threads(nthreads)
  for (int b = 0; b < B; ++b) {
    const int Tb = clamp_len(act_lens[b], 1, T), Ub = clamp_len(label_lens[b] + 1, 1, U);
    const float scale = (grad_scale ? grad_scale[(size_t)b * grad_scale_stride] : 1.f) * grad_mul;
    backward_utterance(s, acts, labels, b, Tb, Ub, w, fastemit_lambda, clamp, scale, wrt_log_probs != 0, grads);
  }
  return MI_TRANSDUCER_CPU_SUCCESS;
}

}  // extern "C"
