// MI355X (gfx950, wave64) transducer-loss kernels and their C ABI.
//
// Pipeline (one stream, no host synchronisation):
//   forward : denom_gather_kernel  -> rnnt_lattice_kernel | tdt_lattice_kernel
//   backward: rnnt_cell_kernel | tdt_cell_kernel -> grad_stream_kernel
//
// denom_gather_kernel  streams the valid rows of acts once (16-byte aligned loads, one
//                      wave per row, online log-sum-exp, wave butterfly reduction) and
//                      leaves per cell: the denominator and the blank / label (/ duration)
//                      log-probabilities in a SKEWED layout [b][t+u][plane][u] so that an
//                      anti-diagonal of the lattice is contiguous.
// *_lattice_kernel     one wave per (utterance, direction); walks the anti-diagonals with
//                      the wave's K cells per lane in registers (RNNT: neighbour exchange by
//                      one wave shuffle, no barrier, no LDS) or an LDS ring of max_duration+2
//                      diagonals (TDT).  Lattice values are accumulated in fp64; only the
//                      log1p(exp(.)) term is evaluated in fp32.
// *_cell_kernel        one thread per lattice cell: turns alpha/beta into the four numbers a
//                      row of the gradient needs (occupancy weight, blank and label
//                      corrections, clamp bound) with grad_scale folded in.
// grad_stream_kernel   streams acts a second time and writes every gradient element once,
//                      zeros for padded cells included.
//
// Reference semantics restated here: nemo/collections/asr/parts/numba/rnnt_loss/
//   utils/cuda_utils/reduce.py:121-248, utils/cuda_utils/gpu_rnnt_kernel.py:73-407 and
//   :888-1439, utils/rnnt_helper.py:42-53,106-142, utils/cuda_utils/gpu_rnnt.py:125-231,563-743.

#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>

#include "mi_transducer.h"

namespace {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kNegInf = -INFINITY;
constexpr double kTdtNeg = -10000.0;  // gpu_rnnt_kernel.py:38
constexpr int kRowsPerBlock = 4;      // one wave per row, 256-thread blocks
constexpr int kCoefBase = 8;          // floats per cell before the duration-gradient block

// ----------------------------------------------------------------------------------------
// Workspace layout
// ----------------------------------------------------------------------------------------
struct Layout {
  int K;    // lattice cells per lane (1,2,4,8,16)
  int Us;   // pitch of a skewed lattice row = 64*K >= U
  int ND;   // number of anti-diagonals of the padded lattice = T+U-1
  int A;    // arc planes per diagonal row: blank, label, D duration log-probs
  int CS;   // floats per cell in the coefficient buffer
  size_t off_denom, off_arcs, off_alphas, off_betas, off_ll, off_coef, total;
};

inline size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

bool make_layout(int B, int T, int U, int D, Layout* L) {
  if (B <= 0 || T <= 0 || U <= 0 || D < 0 || U > MI_TRANSDUCER_MAX_U || D > MI_TRANSDUCER_MAX_DURATIONS) return false;
  int K = 1;
  while (64 * K < U) K *= 2;
  L->K = K;
  L->Us = 64 * K;
  L->ND = T + U - 1;
  L->A = 2 + D;
  L->CS = kCoefBase + ((D + 3) & ~3);
  const size_t cells = (size_t)B * T * U;
  const size_t skew = (size_t)B * L->ND * L->Us;
  size_t off = 0;
  L->off_denom = off;  off = align256(off + cells * sizeof(float));
  L->off_arcs = off;   off = align256(off + skew * L->A * sizeof(float));
  L->off_alphas = off; off = align256(off + skew * sizeof(double));
  L->off_betas = off;  off = align256(off + skew * sizeof(double));
  L->off_ll = off;     off = align256(off + (size_t)B * 2 * sizeof(double));
  L->off_coef = off;   off = align256(off + cells * L->CS * sizeof(float));
  L->total = off;
  return true;
}

// ----------------------------------------------------------------------------------------
// Device helpers
// ----------------------------------------------------------------------------------------
__device__ __forceinline__ int clampi(long long v, int lo, int hi) {
  return v < lo ? lo : (v > hi ? hi : (int)v);
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Workgroup ids are dealt round-robin to the 8 XCDs; give each XCD one contiguous
// eighth of the rows so that rows sharing a cache line meet in the same L2.
__device__ __forceinline__ long long remap_block(long long chunk) {
  const unsigned bid = blockIdx.x;
  return (long long)(bid & 7u) * chunk + (long long)(bid >> 3);
}

// Element access for the three logit dtypes.  A "vector" is 16 bytes.
template <int DT> struct Elem;
template <> struct Elem<MI_DTYPE_F32> {
  static constexpr int VEC = 4;
  static constexpr int BYTES = 4;
  static __device__ __forceinline__ void unpack(const uint4& r, float* f) {
    f[0] = __uint_as_float(r.x); f[1] = __uint_as_float(r.y);
    f[2] = __uint_as_float(r.z); f[3] = __uint_as_float(r.w);
  }
  static __device__ __forceinline__ uint4 pack(const float* f) {
    return make_uint4(__float_as_uint(f[0]), __float_as_uint(f[1]), __float_as_uint(f[2]), __float_as_uint(f[3]));
  }
  static __device__ __forceinline__ float load1(const void* base, size_t idx) { return ((const float*)base)[idx]; }
  static __device__ __forceinline__ void store1(void* base, size_t idx, float v) { ((float*)base)[idx] = v; }
};
__device__ __forceinline__ unsigned f32_to_bf16_bits(float f) {
  unsigned u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;  // quiet NaN
  return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;                  // round to nearest even
}
template <> struct Elem<MI_DTYPE_BF16> {
  static constexpr int VEC = 8;
  static constexpr int BYTES = 2;
  static __device__ __forceinline__ void unpack(const uint4& r, float* f) {
    const unsigned w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = __uint_as_float(w[i] << 16);
      f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ uint4 pack(const float* f) {
    unsigned w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = f32_to_bf16_bits(f[2 * i]) | (f32_to_bf16_bits(f[2 * i + 1]) << 16);
    return make_uint4(w[0], w[1], w[2], w[3]);
  }
  static __device__ __forceinline__ float load1(const void* base, size_t idx) {
    return __uint_as_float((unsigned)((const unsigned short*)base)[idx] << 16);
  }
  static __device__ __forceinline__ void store1(void* base, size_t idx, float v) {
    ((unsigned short*)base)[idx] = (unsigned short)f32_to_bf16_bits(v);
  }
};
template <> struct Elem<MI_DTYPE_F16> {
  static constexpr int VEC = 8;
  static constexpr int BYTES = 2;
  static __device__ __forceinline__ void unpack(const uint4& r, float* f) {
    const unsigned w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = (float)__builtin_bit_cast(_Float16, (unsigned short)(w[i] & 0xffffu));
      f[2 * i + 1] = (float)__builtin_bit_cast(_Float16, (unsigned short)(w[i] >> 16));
    }
  }
  static __device__ __forceinline__ uint4 pack(const float* f) {
    unsigned w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
      w[i] = (unsigned)__builtin_bit_cast(unsigned short, (_Float16)f[2 * i]) |
             ((unsigned)__builtin_bit_cast(unsigned short, (_Float16)f[2 * i + 1]) << 16);
    return make_uint4(w[0], w[1], w[2], w[3]);
  }
  static __device__ __forceinline__ float load1(const void* base, size_t idx) {
    return (float)((const _Float16*)base)[idx];
  }
  static __device__ __forceinline__ void store1(void* base, size_t idx, float v) {
    ((_Float16*)base)[idx] = (_Float16)v;
  }
};

// A row of logits seen through 16-byte aligned vectors: vector j of the row's window holds
// row elements j*VEC - mis .. j*VEC - mis + VEC - 1.  The window starts at the aligned
// address at or below the row start, so every load is aligned; elements that fall outside
// the row are masked by the caller.  A 16-byte granule that holds one valid byte lies in
// the same page as that byte, so the few bytes read around a row never leave mapped memory.
template <int DT> struct RowWindow {
  const uint4* vp;
  int mis;
  __device__ __forceinline__ RowWindow(const void* base, size_t first_elem) {
    const uintptr_t a0 = (uintptr_t)base + first_elem * Elem<DT>::BYTES;
    const uintptr_t al = a0 & ~(uintptr_t)15;
    vp = (const uint4*)al;
    mis = (int)((a0 - al) / Elem<DT>::BYTES);
  }
};

// ----------------------------------------------------------------------------------------
// Pass 1: denominators + gather (replaces reduce.py:121-248 and the per-step gathers of
// logp() in gpu_rnnt_kernel.py:42-64).  One wave per (b,t,u) row; padded rows exit.
// ----------------------------------------------------------------------------------------
template <int DT>
__global__ __launch_bounds__(256) void denom_gather_kernel(
    const void* __restrict__ acts, const int64_t* __restrict__ labels, const int64_t* __restrict__ act_lens,
    const int64_t* __restrict__ label_lens, float* __restrict__ denom, float* __restrict__ arcs, int T, int U, int V,
    int D, int blank, int ND, int Us, int A, long long rows, long long chunk) {
  constexpr int VEC = Elem<DT>::VEC;
  constexpr int R = 4;  // vectors in flight per lane
  const int lane = threadIdx.x & 63;
  const long long r =
      __builtin_amdgcn_readfirstlane((int)(remap_block(chunk) * kRowsPerBlock + (threadIdx.x >> 6)));
  if (r >= rows) return;
  const int u = (int)(r % U);
  const long long bt = r / U;
  const int t = (int)(bt % T);
  const int b = (int)(bt / T);
  const int Tb = clampi(act_lens[b], 1, T);
  const int Ub = clampi(label_lens[b] + 1, 1, U);
  if (t >= Tb || u >= Ub) return;

  const int VD = V + D;
  const RowWindow<DT> w(acts, (size_t)r * VD);
  const int nvec = (w.mis + V + VEC - 1) / VEC;  // only the token logits enter the denominator

  float m = kNegInf, s = 0.f;
  for (int j0 = lane; j0 < nvec; j0 += 64 * R) {
    uint4 raw[R];
#pragma unroll
    for (int k = 0; k < R; ++k) {
      const int j = j0 + 64 * k;
      if (j < nvec) raw[k] = w.vp[j];
    }
    float x[R][VEC];
    float cm = kNegInf;
#pragma unroll
    for (int k = 0; k < R; ++k) {
      const int j = j0 + 64 * k;
      Elem<DT>::unpack(raw[k], x[k]);
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const int v = j * VEC + i - w.mis;
        if (j >= nvec || v < 0 || v >= V) x[k][i] = kNegInf;
        cm = fmaxf(cm, x[k][i]);
      }
    }
    const float mnew = fmaxf(m, cm);
    if (mnew > kNegInf) {
      float acc = 0.f;
      const float off = -mnew * kLog2e;
#pragma unroll
      for (int k = 0; k < R; ++k)
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc += fast_exp2(fmaf(x[k][i], kLog2e, off));
      s = s * fast_exp2((m - mnew) * kLog2e) + acc;
      m = mnew;
    }
  }
  const float M = wave_max(m);
  const float part = (m > kNegInf) ? s * fast_exp2((m - M) * kLog2e) : 0.f;
  const float S = wave_sum(part);
  const float dn = -M - logf(S);

  const int lab = (u < Ub - 1) ? clampi(labels[(size_t)b * (U - 1) + u], 0, V - 1) : -1;
  const float xb = Elem<DT>::load1(acts, (size_t)r * VD + blank);
  const float xl = lab >= 0 ? Elem<DT>::load1(acts, (size_t)r * VD + lab) : 0.f;
  const size_t base = ((size_t)(b * ND + t + u) * A) * Us + u;
  if (lane == 0) {
    denom[r] = dn;
    arcs[base] = xb + dn;
    arcs[base + Us] = lab >= 0 ? xl + dn : 0.f;
  }
  if (D > 0) {  // duration log-softmax (rnnt_pytorch.py:568), one lane per duration
    const float xd = lane < D ? Elem<DT>::load1(acts, (size_t)r * VD + V + lane) : kNegInf;
    const float dm = wave_max(xd);
    const float ds = wave_sum(lane < D ? expf(xd - dm) : 0.f);
    const float dden = -dm - logf(ds);
    if (lane < D) arcs[base + (size_t)(2 + lane) * Us] = xd + dden;
  }
}

// ----------------------------------------------------------------------------------------
// Lattice helpers
// ----------------------------------------------------------------------------------------
// log(exp(a)+exp(b)) with the sum carried in fp64 and the correction term in fp32
// (rnnt_helper.py:42-53: the other operand is returned when one is -inf).
__device__ __forceinline__ double lse_h(double a, double b) {
  const double m = fmax(a, b);
  const double n = fmin(a, b);
  if (n == -INFINITY) return m;
  const float d = (float)(n - m);
  return m + (double)__logf(1.0f + __expf(d));
}

template <int K> struct FloatK;
template <> struct FloatK<1> { typedef float type; };
template <> struct FloatK<2> { typedef float type __attribute__((ext_vector_type(2))); };
template <> struct FloatK<4> { typedef float type __attribute__((ext_vector_type(4))); };

template <int K> __device__ __forceinline__ void load_k(const float* p, float* out) {
  if constexpr (K == 1) {
    out[0] = p[0];
  } else if constexpr (K == 2 || K == 4) {
    typedef typename FloatK<K>::type V;
    const V v = *(const V*)p;
#pragma unroll
    for (int k = 0; k < K; ++k) out[k] = v[k];
  } else {
#pragma unroll
    for (int q = 0; q < K / 4; ++q) {
      typedef typename FloatK<4>::type V;
      const V v = *(const V*)(p + 4 * q);
#pragma unroll
      for (int k = 0; k < 4; ++k) out[4 * q + k] = v[k];
    }
  }
}

template <int K> struct Prefetch { static constexpr int P = K <= 2 ? 8 : (K == 4 ? 4 : (K == 8 ? 2 : 1)); };

// RNNT lattice: one wave per (utterance, direction).  Lane l owns columns u = l*K .. l*K+K-1
// and, at step n, the cells (n-u, u) of anti-diagonal n.
//   alpha (gpu_rnnt_kernel.py:73-172): every cell pushes e = alpha + lp_label to its right
//   neighbour and s = alpha + lp_blank to the cell below; the next diagonal is lse(e_in, s_in).
//   beta  (gpu_rnnt_kernel.py:175-269): pulled from the diagonal above.
// The arc log-probs of diagonals n .. n+P-1 are prefetched into registers while the previous
// P diagonals are being computed; they do not depend on the recursion.
template <int K>
__global__ __launch_bounds__(64) void rnnt_lattice_kernel(const float* __restrict__ arcs, double* __restrict__ alphas,
                                                          double* __restrict__ betas, double* __restrict__ ll,
                                                          float* __restrict__ costs,
                                                          const int64_t* __restrict__ act_lens,
                                                          const int64_t* __restrict__ label_lens, int T, int U, int ND,
                                                          int A, float cost_scale, int with_betas) {
  constexpr int P = Prefetch<K>::P;
  constexpr int Us = 64 * K;
  const int b = with_betas ? (int)(blockIdx.x >> 1) : (int)blockIdx.x;
  const int dir = with_betas ? (int)(blockIdx.x & 1) : 0;
  const int lane = threadIdx.x;
  const int u0 = lane * K;
  const int Tb = clampi(act_lens[b], 1, T);
  const int Ub = clampi(label_lens[b] + 1, 1, U);
  const int nd = Tb + Ub - 1;
  const float* arcs_b = arcs + (size_t)b * ND * A * Us + u0;
  const double NINF = -INFINITY;

  float blk[P][K], lab[P][K];
  auto load_rows = [&](int nfirst, int step, float(&Bk)[P][K], float(&Lb)[P][K]) {
#pragma unroll
    for (int p = 0; p < P; ++p) {
      const int n = nfirst + step * p;
      if (n >= 0 && n < nd) {
        const float* rp = arcs_b + (size_t)n * A * Us;
        load_k<K>(rp, Bk[p]);
        load_k<K>(rp + Us, Lb[p]);
      }
    }
  };

  if (dir == 0) {
    double* out = alphas + (size_t)b * ND * Us + u0;
    double e[K], s[K];
#pragma unroll
    for (int k = 0; k < K; ++k) e[k] = s[k] = NINF;
    load_rows(0, 1, blk, lab);
    for (int n0 = 0; n0 < nd; n0 += P) {
      float nb[P][K], nl[P][K];
      load_rows(n0 + P, 1, nb, nl);
#pragma unroll
      for (int p = 0; p < P; ++p) {
        const int n = n0 + p;
        if (n < nd) {
          double left = __shfl_up(e[K - 1], 1, 64);
          if (lane == 0) left = NINF;
          double a[K];
#pragma unroll
          for (int k = 0; k < K; ++k) {
            const int u = u0 + k, t = n - u;
            const bool valid = (u < Ub) && (t >= 0) && (t < Tb);
            double v = lse_h(k == 0 ? left : e[k - 1], s[k]);
            if (n == 0 && u == 0) v = 0.0;
            a[k] = valid ? v : NINF;
          }
#pragma unroll
          for (int k = 0; k < K; ++k) {
            const int u = u0 + k, t = n - u;
            const bool valid = (u < Ub) && (t >= 0) && (t < Tb);
            e[k] = valid ? a[k] + (double)lab[p][k] : NINF;
            s[k] = valid ? a[k] + (double)blk[p][k] : NINF;
            if (valid) out[(size_t)n * Us + k] = a[k];
            if (n == nd - 1 && u == Ub - 1 && valid) {  // llForward and the cost (rnnt_helper.py:106-116)
              ll[2 * b] = s[k];
              costs[b] = -(float)s[k] * cost_scale;
            }
          }
        }
      }
#pragma unroll
      for (int p = 0; p < P; ++p)
#pragma unroll
        for (int k = 0; k < K; ++k) {
          blk[p][k] = nb[p][k];
          lab[p][k] = nl[p][k];
        }
    }
  } else {
    double* out = betas + (size_t)b * ND * Us + u0;
    double bt[K];
#pragma unroll
    for (int k = 0; k < K; ++k) bt[k] = NINF;
    load_rows(nd - 1, -1, blk, lab);
    for (int n0 = nd - 1; n0 >= 0; n0 -= P) {
      float nb[P][K], nl[P][K];
      load_rows(n0 - P, -1, nb, nl);
#pragma unroll
      for (int p = 0; p < P; ++p) {
        const int n = n0 - p;
        if (n >= 0) {
          double right = __shfl_down(bt[0], 1, 64);
          if (lane == 63) right = NINF;
          double nv[K];
#pragma unroll
          for (int k = 0; k < K; ++k) {
            const int u = u0 + k, t = n - u;
            const bool valid = (u < Ub) && (t >= 0) && (t < Tb);
            const double rgt = (k == K - 1) ? right : bt[k + 1];
            const double em = (u + 1 < Ub) ? rgt + (double)lab[p][k] : NINF;
            double ne;
            if (t == Tb - 1)
              ne = (u == Ub - 1) ? (double)blk[p][k] : NINF;
            else
              ne = bt[k] + (double)blk[p][k];
            nv[k] = valid ? lse_h(em, ne) : NINF;
          }
#pragma unroll
          for (int k = 0; k < K; ++k) {
            const int u = u0 + k, t = n - u;
            const bool valid = (u < Ub) && (t >= 0) && (t < Tb);
            bt[k] = nv[k];
            if (valid) out[(size_t)n * Us + k] = nv[k];
            if (n == 0 && u == 0) ll[2 * b + 1] = nv[k];
          }
        }
      }
#pragma unroll
      for (int p = 0; p < P; ++p)
#pragma unroll
        for (int k = 0; k < K; ++k) {
          blk[p][k] = nb[p][k];
          lab[p][k] = nl[p][k];
        }
    }
  }
}

// TDT lattice (gpu_rnnt_kernel.py:888-1241): one wave per (utterance, direction), an LDS
// ring of R = max_duration + 2 anti-diagonals.
//   alpha: a finished cell pushes alpha + arc into the ring slots of the diagonals its arcs
//          land on (each slot has a single writer per step: durations are distinct); a cell's
//          alpha is lse(emit slot, no-emit slot), both seeded with the reference's finite
//          -10000 sentinel.
//   beta : pulled from the ring of later diagonals.
struct TdtParams {
  int D;
  int dur[MI_TRANSDUCER_MAX_DURATIONS];
  int one_idx;  // index of duration 1 (position 0 or 1)
  int R;        // ring depth
  float sigma;
};

template <int K>
__global__ __launch_bounds__(64) void tdt_lattice_kernel(const float* __restrict__ arcs, double* __restrict__ alphas,
                                                         double* __restrict__ betas, double* __restrict__ ll,
                                                         float* __restrict__ costs,
                                                         const int64_t* __restrict__ act_lens,
                                                         const int64_t* __restrict__ label_lens, int T, int U, int ND,
                                                         int A, float cost_scale, int with_betas, TdtParams prm) {
  constexpr int Us = 64 * K;
  extern __shared__ double ring[];  // alpha: [2][R][Us] (emit, no-emit); beta: [R][Us]
  const int b = with_betas ? (int)(blockIdx.x >> 1) : (int)blockIdx.x;
  const int dir = with_betas ? (int)(blockIdx.x & 1) : 0;
  const int lane = threadIdx.x;
  const int u0 = lane * K;
  const int Tb = clampi(act_lens[b], 1, T);
  const int Ub = clampi(label_lens[b] + 1, 1, U);
  const int nd = Tb + Ub - 1;
  const int D = prm.D, R = prm.R;
  const double sigma = (double)prm.sigma;
  const float* arcs_b = arcs + (size_t)b * ND * A * Us;

  if (dir == 0) {
    double* em_ring = ring;
    double* ne_ring = ring + (size_t)R * Us;
    for (int i = lane; i < 2 * R * Us; i += 64) ring[i] = kTdtNeg;
    __syncthreads();
    double* out = alphas + (size_t)b * ND * Us;
    double ll_acc = kTdtNeg;
    for (int n = 0; n < nd; ++n) {
      const int slot = (n % R) * Us;
      const float* rp = arcs_b + (size_t)n * A * Us;
#pragma unroll
      for (int k = 0; k < K; ++k) {
        const int u = u0 + k, t = n - u;
        const bool valid = (u < Ub) && (t >= 0) && (t < Tb);
        const double em = em_ring[slot + u], ne = ne_ring[slot + u];
        em_ring[slot + u] = kTdtNeg;
        ne_ring[slot + u] = kTdtNeg;
        if (valid) {
          double a;
          if (t == 0 && u == 0) a = 0.0;
          else if (u == 0) a = ne;
          else if (t == 0) a = em;
          else a = lse_h(em, ne);
          out[(size_t)n * Us + u] = a;
          const double wb = a + (double)rp[u];
          const double wl = a + (double)rp[Us + u];
          for (int i = 0; i < D; ++i) {
            const int d = prm.dur[i];
            const double dl = (double)rp[(size_t)(2 + i) * Us + u];
            if (d > 0) {
              const double c = (wb - sigma) + dl;
              if (t + d < Tb) {
                double* q = ne_ring + ((n + d) % R) * Us + u;
                *q = lse_h(*q, c);
              } else if (t + d == Tb && u == Ub - 1) {
                ll_acc = lse_h(ll_acc, c);
              }
            }
            if (u + 1 < Ub && t + d < Tb) {
              double* q = em_ring + ((n + d + 1) % R) * Us + u + 1;
              *q = lse_h(*q, (wl - sigma) + dl);
            }
          }
          if (n == nd - 1) {  // (Tb-1, Ub-1): the last contribution to llForward is in
            ll[2 * b] = ll_acc;
            costs[b] = -(float)ll_acc * cost_scale;
          }
        }
      }
      __syncthreads();
    }
  } else {
    for (int i = lane; i < R * Us; i += 64) ring[i] = kTdtNeg;
    __syncthreads();
    double* out = betas + (size_t)b * ND * Us;
    for (int n = nd - 1; n >= 0; --n) {
      const float* rp = arcs_b + (size_t)n * A * Us;
      double nv[K];
#pragma unroll
      for (int k = 0; k < K; ++k) {
        const int u = u0 + k, t = n - u;
        const bool valid = (u < Ub) && (t >= 0) && (t < Tb);
        nv[k] = kTdtNeg;
        if (valid) {
          const double lpb = (double)rp[u], lpl = (double)rp[Us + u];
          double no_emit = kTdtNeg, emit = kTdtNeg;
          for (int i = 0; i < D; ++i) {
            const int d = prm.dur[i];
            const double dl = (double)rp[(size_t)(2 + i) * Us + u];
            if (d > 0) {
              if (t + d < Tb)
                no_emit = lse_h(no_emit, ((ring[((n + d) % R) * Us + u] + lpb) + dl) - sigma);
              else if (t + d == Tb && u == Ub - 1)
                no_emit = lse_h(no_emit, (lpb + dl) - sigma);
            }
            if (u + 1 < Ub && t + d < Tb)
              emit = lse_h(emit, ((ring[((n + d + 1) % R) * Us + u + 1] + lpl) + dl) - sigma);
          }
          double v;
          if (u == Ub - 1) v = no_emit;
          else if (t == Tb - 1) v = emit;
          else v = lse_h(emit, no_emit);
          nv[k] = v;
          out[(size_t)n * Us + u] = v;
          if (n == 0) ll[2 * b + 1] = v;
        }
      }
      __syncthreads();
#pragma unroll
      for (int k = 0; k < K; ++k) ring[(n % R) * Us + u0 + k] = nv[k];
      __syncthreads();
    }
  }
}

// ----------------------------------------------------------------------------------------
// Per-cell gradient coefficients.  For a valid cell the gradient row is
//   g_v = clamp( p_v * W  - [v = blank] PB - [v = label] PL ) * scale,   p_v = exp(x_v + denom)
// with W = exp(alpha+beta-ll) + lambda * post_label, PB = blank-arc posterior,
// PL = (1+lambda) * label-arc posterior: algebraically the five terms of
// gpu_rnnt_kernel.py:340-403 (RNNT) and :1353-1437 (TDT).
// coef[cell] = { denom*log2(e), W*scale, clamp*|scale| (inf = off), G_blank, G_label,
//                label id (-1 none, -2 padded cell), -, -, dlogit_0 .. dlogit_{D-1} }
// where G_blank / G_label are the finished gradient entries of the two special logits.
// ----------------------------------------------------------------------------------------
__device__ __forceinline__ float clamp_sym(float g, float bound) { return fminf(fmaxf(g, -bound), bound); }

__device__ __forceinline__ void write_coef(float* c, float dn, float W, float PB, float PL, float lpb, float lpl,
                                           int lab, int blank, float clamp, float scale) {
  float gb = expf(lpb) * W - PB;
  float gl = lab >= 0 ? expf(lpl) * W - PL : 0.f;
  if (lab == blank) gb = gl = expf(lpb) * W - PB - PL;
  if (clamp > 0.f) {
    gb = clamp_sym(gb, clamp);
    gl = clamp_sym(gl, clamp);
  }
  c[0] = dn * kLog2e;
  c[1] = W * scale;
  c[2] = clamp > 0.f ? clamp * fabsf(scale) : INFINITY;
  c[3] = gb * scale;
  c[4] = gl * scale;
  c[5] = __int_as_float(lab);
}

__global__ __launch_bounds__(256) void rnnt_cell_kernel(
    const float* __restrict__ denom, const float* __restrict__ arcs, const double* __restrict__ alphas,
    const double* __restrict__ betas, const double* __restrict__ ll, const int64_t* __restrict__ labels,
    const int64_t* __restrict__ act_lens, const int64_t* __restrict__ label_lens, const float* __restrict__ grad_scale,
    float* __restrict__ coef, int T, int U, int V, int blank, int ND, int Us, int A, int CS, float lambda, float clamp,
    long long cells) {
  const long long c = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= cells) return;
  const int u = (int)(c % U);
  const long long bt = c / U;
  const int t = (int)(bt % T);
  const int b = (int)(bt / T);
  const int Tb = clampi(act_lens[b], 1, T);
  const int Ub = clampi(label_lens[b] + 1, 1, U);
  float* out = coef + (size_t)c * CS;
  if (t >= Tb || u >= Ub) {
    out[5] = __int_as_float(-2);
    return;
  }
  const size_t row = (size_t)(b * ND + t + u);
  const size_t sk = row * Us + u;
  const double a = alphas[sk], bb = betas[sk], L = ll[2 * b];
  const float lpb = arcs[row * A * Us + u];
  const float lpl = arcs[row * A * Us + Us + u];
  const int lab = (u < Ub - 1) ? clampi(labels[(size_t)b * (U - 1) + u], 0, V - 1) : -1;
  const float gamma = expf((float)(a + bb - L));
  float pb = 0.f, pl = 0.f;
  if (t < Tb - 1)
    pb = expf((float)(a + betas[sk + Us] - L + (double)lpb));  // beta(t+1,u): next diagonal, same column
  else if (u == Ub - 1)
    pb = expf((float)(a - L + (double)lpb));
  if (lab >= 0) pl = expf((float)(a + betas[sk + Us + 1] - L + (double)lpl));  // beta(t,u+1)
  const float scale = grad_scale ? grad_scale[b] : 1.f;
  write_coef(out, denom[c], gamma + lambda * pl, pb, (1.f + lambda) * pl, lpb, lpl, lab, blank, clamp, scale);
}

__global__ __launch_bounds__(256) void tdt_cell_kernel(
    const float* __restrict__ denom, const float* __restrict__ arcs, const double* __restrict__ alphas,
    const double* __restrict__ betas, const double* __restrict__ ll, const int64_t* __restrict__ labels,
    const int64_t* __restrict__ act_lens, const int64_t* __restrict__ label_lens, const float* __restrict__ grad_scale,
    float* __restrict__ coef, int T, int U, int V, int blank, int ND, int Us, int A, int CS, float lambda, float clamp,
    long long cells, TdtParams prm) {
  const long long c = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= cells) return;
  const int u = (int)(c % U);
  const long long bt = c / U;
  const int t = (int)(bt % T);
  const int b = (int)(bt / T);
  const int Tb = clampi(act_lens[b], 1, T);
  const int Ub = clampi(label_lens[b] + 1, 1, U);
  float* out = coef + (size_t)c * CS;
  if (t >= Tb || u >= Ub) {
    out[5] = __int_as_float(-2);
    return;
  }
  const int D = prm.D;
  const double sigma = (double)prm.sigma;
  const size_t row = (size_t)(b * ND + t + u);
  const size_t sk = row * Us + u;
  const double a = alphas[sk], bb = betas[sk], L = ll[2 * b];
  const float* rp = arcs + row * A * Us + u;
  const float lpb = rp[0], lpl = rp[Us];
  const int lab = (u < Ub - 1) ? clampi(labels[(size_t)b * (U - 1) + u], 0, V - 1) : -1;
  const float scale = grad_scale ? grad_scale[b] : 1.f;
  const float gamma = expf((float)(a + bb - L));
  float pb = 0.f, pl = 0.f;
  float arc_post[MI_TRANSDUCER_MAX_DURATIONS], q[MI_TRANSDUCER_MAX_DURATIONS];
#pragma unroll 1
  for (int i = 0; i < D; ++i) {
    const int d = prm.dur[i];
    const double dl = (double)rp[(size_t)(2 + i) * Us];
    float ai = 0.f, bi = 0.f;
    if (t + d < Tb && lab >= 0) ai = expf((float)(a + betas[sk + (size_t)(d + 1) * Us + 1] + (double)lpl - sigma - L + dl));
    if (d > 0) {
      if (t + d < Tb)
        bi = expf((float)(a + betas[sk + (size_t)d * Us] + (double)lpb - sigma - L + dl));
      else if (t + d == Tb && u == Ub - 1)
        bi = expf((float)(a + (double)lpb - sigma - L + dl));
    }
    pl += ai;
    pb += bi;
    arc_post[i] = ai + bi;
    q[i] = expf((float)dl);
  }
  // duration LOGIT gradient: dg_i - softmax_i * sum_j dg_j with dg_i = -(a_i + b_i)
  // (gpu_rnnt_kernel.py:1328-1341 followed by the log_softmax backward of rnnt_pytorch.py:568)
  const float tot = pl + pb;
#pragma unroll 1
  for (int i = 0; i < D; ++i) out[kCoefBase + i] = (q[i] * tot - arc_post[i]) * scale;
  write_coef(out, denom[c], gamma + lambda * pl, pb, (1.f + lambda) * pl, lpb, lpl, lab, blank, clamp, scale);
}

// ----------------------------------------------------------------------------------------
// Pass 2: the gradient stream.  One wave per row; reads V logits (valid rows only), writes
// V + D gradient elements (every row).  Same kernel for RNNT (D = 0) and TDT.
// zero_durations: the omega branch of TDT -- duration gradients are zero.
// ----------------------------------------------------------------------------------------
template <int DT>
__global__ __launch_bounds__(256) void grad_stream_kernel(const void* __restrict__ acts, void* __restrict__ grads,
                                                          const float* __restrict__ coef, int V, int D, int blank,
                                                          int CS, int zero_durations, long long rows,
                                                          long long chunk) {
  constexpr int VEC = Elem<DT>::VEC;
  constexpr int R = 4;
  const int lane = threadIdx.x & 63;
  const long long r =
      __builtin_amdgcn_readfirstlane((int)(remap_block(chunk) * kRowsPerBlock + (threadIdx.x >> 6)));
  if (r >= rows) return;
  const int VD = V + D;
  const float* c = coef + (size_t)r * CS;
  const int lab = __float_as_int(c[5]);
  const RowWindow<DT> win(acts, (size_t)r * VD);
  // acts and grads have the same shape and dtype; their bases may differ in alignment
  const uintptr_t g0 = (uintptr_t)grads + (size_t)r * VD * Elem<DT>::BYTES;
  const bool same_phase = ((g0 & 15) / Elem<DT>::BYTES) == (uintptr_t)win.mis;
  uint4* gvp = (uint4*)(g0 & ~(uintptr_t)15);
  const int mis = win.mis;
  const int nvec = (mis + VD + VEC - 1) / VEC;

  if (lab == -2) {  // padded cell: zeros
    const uint4 z = make_uint4(0, 0, 0, 0);
    for (int j = lane; j < nvec; j += 64) {
      const int first = j * VEC - mis;
      if (same_phase && first >= 0 && first + VEC <= VD) {
        gvp[j] = z;
      } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
          const int v = first + i;
          if (v >= 0 && v < VD) Elem<DT>::store1(grads, (size_t)r * VD + v, 0.f);
        }
      }
    }
    return;
  }

  const float dl2 = c[0], W = c[1], cb = c[2], gB = c[3], gL = c[4];
  const bool clamp_on = cb < INFINITY;
  for (int j0 = lane; j0 < nvec; j0 += 64 * R) {
    uint4 raw[R];
#pragma unroll
    for (int k = 0; k < R; ++k) {
      const int j = j0 + 64 * k;
      if (j < nvec) raw[k] = win.vp[j];
    }
#pragma unroll
    for (int k = 0; k < R; ++k) {
      const int j = j0 + 64 * k;
      if (j < nvec) {
        float x[VEC], g[VEC];
        Elem<DT>::unpack(raw[k], x);
        const int first = j * VEC - mis;
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
          float gi = fast_exp2(fmaf(x[i], kLog2e, dl2)) * W;
          if (clamp_on) gi = clamp_sym(gi, cb);
          g[i] = gi;
        }
        if (blank >= first && blank < first + VEC) {
#pragma unroll
          for (int i = 0; i < VEC; ++i)
            if (first + i == blank) g[i] = gB;
        }
        if (lab >= first && lab < first + VEC) {
#pragma unroll
          for (int i = 0; i < VEC; ++i)
            if (first + i == lab) g[i] = gL;
        }
        if (same_phase && first >= 0 && first + VEC <= V) {
          gvp[j] = Elem<DT>::pack(g);
        } else {
#pragma unroll
          for (int i = 0; i < VEC; ++i) {
            const int v = first + i;
            if (v >= 0 && v < V) {
              Elem<DT>::store1(grads, (size_t)r * VD + v, g[i]);
            } else if (v >= V && v < VD) {
              Elem<DT>::store1(grads, (size_t)r * VD + v, zero_durations ? 0.f : c[kCoefBase + v - V]);
            }
          }
        }
      }
    }
  }
}

// ----------------------------------------------------------------------------------------
// Read-out of the skewed lattice into plain [B,T,U] float arrays (stage-level tests).
// ----------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void export_lattice_kernel(
    const float* __restrict__ ws_denom, const double* __restrict__ ws_alphas, const double* __restrict__ ws_betas,
    const double* __restrict__ ws_ll, const int64_t* __restrict__ act_lens, const int64_t* __restrict__ label_lens,
    float* denom, float* alphas, float* betas, float* llf, float* llb, int B, int T, int U, int ND, int Us,
    long long cells) {
  const long long c = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (c < B) {
    if (llf) llf[c] = (float)ws_ll[2 * c];
    if (llb) llb[c] = (float)ws_ll[2 * c + 1];
  }
  if (c >= cells) return;
  const int u = (int)(c % U);
  const long long bt = c / U;
  const int t = (int)(bt % T);
  const int b = (int)(bt / T);
  const int Tb = clampi(act_lens[b], 1, T);
  const int Ub = clampi(label_lens[b] + 1, 1, U);
  const bool valid = t < Tb && u < Ub;
  const size_t sk = (size_t)(b * ND + t + u) * Us + u;
  if (denom) denom[c] = valid ? ws_denom[c] : 0.f;
  if (alphas) alphas[c] = valid ? (float)ws_alphas[sk] : 0.f;
  if (betas) betas[c] = valid ? (float)ws_betas[sk] : 0.f;
}

// max(act_lens), max(label_lens) -> out[0], out[1]; one block.  Lets the host check the
// tensor shape against the lengths (rnnt_pytorch.py:628-634) with one small read-back.
__global__ __launch_bounds__(256) void length_maxima_kernel(const int64_t* __restrict__ act_lens,
                                                            const int64_t* __restrict__ label_lens, int B,
                                                            int64_t* __restrict__ out) {
  __shared__ long long sm[2][4];
  long long ma = INT64_MIN, ml = INT64_MIN;
  for (int i = threadIdx.x; i < B; i += 256) {
    ma = act_lens[i] > ma ? act_lens[i] : ma;
    ml = label_lens[i] > ml ? label_lens[i] : ml;
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const long long oa = __shfl_xor(ma, o, 64), ol = __shfl_xor(ml, o, 64);
    ma = oa > ma ? oa : ma;
    ml = ol > ml ? ol : ml;
  }
  if ((threadIdx.x & 63) == 0) {
    sm[0][threadIdx.x >> 6] = ma;
    sm[1][threadIdx.x >> 6] = ml;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; ++w) {
      ma = sm[0][w] > ma ? sm[0][w] : ma;
      ml = sm[1][w] > ml ? sm[1][w] : ml;
    }
    out[0] = ma;
    out[1] = ml;
  }
}

// ----------------------------------------------------------------------------------------
// Host side
// ----------------------------------------------------------------------------------------
struct Common {
  const void* acts;
  int dt;
  const int64_t *labels, *act_lens, *label_lens;
  int B, T, U, V, D, blank;
  char* ws;
  hipStream_t stream;
  Layout L;
};

int check_common(const void* acts, int dt, const int64_t* labels, const int64_t* act_lens, const int64_t* label_lens,
                 int B, int T, int U, int V, int D, int blank, void* ws, size_t ws_bytes, void* stream, Common* c) {
  if (!acts || !act_lens || !label_lens || !ws) return MI_TRANSDUCER_INVALID_VALUE;
  if (U > 1 && !labels) return MI_TRANSDUCER_INVALID_VALUE;
  if (dt != MI_DTYPE_F32 && dt != MI_DTYPE_BF16 && dt != MI_DTYPE_F16) return MI_TRANSDUCER_INVALID_VALUE;
  if (V <= 0 || blank < 0 || blank >= V) return MI_TRANSDUCER_INVALID_VALUE;
  if (!make_layout(B, T, U, D, &c->L)) return MI_TRANSDUCER_INVALID_VALUE;
  if (ws_bytes < c->L.total || ((uintptr_t)ws & 255)) return MI_TRANSDUCER_INVALID_VALUE;
  if ((long long)B * T * U > 0x7fffffffLL) return MI_TRANSDUCER_INVALID_VALUE;  // row index is kept in 31 bits
  c->acts = acts; c->dt = dt; c->labels = labels; c->act_lens = act_lens; c->label_lens = label_lens;
  c->B = B; c->T = T; c->U = U; c->V = V; c->D = D; c->blank = blank;
  c->ws = (char*)ws; c->stream = (hipStream_t)stream;
  return MI_TRANSDUCER_SUCCESS;
}

int make_tdt_params(int D, const int32_t* durations, float sigma, TdtParams* p) {
  if (D <= 0 || D > MI_TRANSDUCER_MAX_DURATIONS || !durations) return MI_TRANSDUCER_INVALID_VALUE;
  p->D = D;
  p->sigma = sigma;
  for (int i = 0; i < MI_TRANSDUCER_MAX_DURATIONS; ++i) p->dur[i] = 0;
  for (int i = 0; i < D; ++i) {
    if (durations[i] < 0 || (i > 0 && durations[i] <= durations[i - 1])) return MI_TRANSDUCER_INVALID_VALUE;
    p->dur[i] = durations[i];
  }
  if (durations[0] == 1) p->one_idx = 0;
  else if (D > 1 && durations[1] == 1) p->one_idx = 1;
  else return MI_TRANSDUCER_INVALID_VALUE;
  p->R = durations[D - 1] + 2;
  return MI_TRANSDUCER_SUCCESS;
}

inline int launch_status() { return hipGetLastError() == hipSuccess ? MI_TRANSDUCER_SUCCESS : MI_TRANSDUCER_LAUNCH_FAILURE; }

void stream_grid(long long rows, unsigned* grid, long long* chunk) {
  const long long nblk = (rows + kRowsPerBlock - 1) / kRowsPerBlock;
  *chunk = (nblk + 7) / 8;
  *grid = (unsigned)(*chunk * 8);
}

int run_denom(const Common& c) {
  const Layout& L = c.L;
  const long long rows = (long long)c.B * c.T * c.U;
  unsigned grid; long long chunk;
  stream_grid(rows, &grid, &chunk);
  float* denom = (float*)(c.ws + L.off_denom);
  float* arcs = (float*)(c.ws + L.off_arcs);
#define LAUNCH_DENOM(DT)                                                                                            \
  hipLaunchKernelGGL(denom_gather_kernel<DT>, dim3(grid), dim3(256), 0, c.stream, c.acts, c.labels, c.act_lens,      \
                     c.label_lens, denom, arcs, c.T, c.U, c.V, c.D, c.blank, L.ND, L.Us, L.A, rows, chunk)
  if (c.dt == MI_DTYPE_F32) LAUNCH_DENOM(MI_DTYPE_F32);
  else if (c.dt == MI_DTYPE_BF16) LAUNCH_DENOM(MI_DTYPE_BF16);
  else LAUNCH_DENOM(MI_DTYPE_F16);
#undef LAUNCH_DENOM
  return launch_status();
}

// rnnt_helper.py:116: the cost is scaled by float32(1 + lambda)
inline float cost_scale_of(float lambda) { return (float)(1.0 + (double)lambda); }

int run_rnnt_lattice(const Common& c, float* costs, float lambda, int with_betas) {
  const Layout& L = c.L;
  const float* arcs = (const float*)(c.ws + L.off_arcs);
  double* alphas = (double*)(c.ws + L.off_alphas);
  double* betas = (double*)(c.ws + L.off_betas);
  double* ll = (double*)(c.ws + L.off_ll);
  const unsigned grid = (unsigned)(with_betas ? 2 * c.B : c.B);
#define LAUNCH_LAT(KK)                                                                                               \
  hipLaunchKernelGGL(rnnt_lattice_kernel<KK>, dim3(grid), dim3(64), 0, c.stream, arcs, alphas, betas, ll, costs,      \
                     c.act_lens, c.label_lens, c.T, c.U, L.ND, L.A, cost_scale_of(lambda), with_betas)
  switch (L.K) {
    case 1: LAUNCH_LAT(1); break;
    case 2: LAUNCH_LAT(2); break;
    case 4: LAUNCH_LAT(4); break;
    case 8: LAUNCH_LAT(8); break;
    default: LAUNCH_LAT(16); break;
  }
#undef LAUNCH_LAT
  return launch_status();
}

int run_tdt_lattice(const Common& c, float* costs, float lambda, int with_betas, const TdtParams& prm) {
  const Layout& L = c.L;
  const float* arcs = (const float*)(c.ws + L.off_arcs);
  double* alphas = (double*)(c.ws + L.off_alphas);
  double* betas = (double*)(c.ws + L.off_betas);
  double* ll = (double*)(c.ws + L.off_ll);
  const unsigned grid = (unsigned)(with_betas ? 2 * c.B : c.B);
  const size_t lds = (size_t)2 * prm.R * L.Us * sizeof(double);
  if (lds > 160 * 1024) return MI_TRANSDUCER_INVALID_VALUE;
#define LAUNCH_TLAT(KK)                                                                                              \
  do {                                                                                                               \
    if (lds > 48 * 1024 &&                                                                                           \
        hipFuncSetAttribute((const void*)tdt_lattice_kernel<KK>, hipFuncAttributeMaxDynamicSharedMemorySize,         \
                            (int)lds) != hipSuccess)                                                                 \
      return MI_TRANSDUCER_LAUNCH_FAILURE;                                                                           \
    hipLaunchKernelGGL(tdt_lattice_kernel<KK>, dim3(grid), dim3(64), lds, c.stream, arcs, alphas, betas, ll, costs,  \
                       c.act_lens, c.label_lens, c.T, c.U, L.ND, L.A, cost_scale_of(lambda), with_betas, prm);       \
  } while (0)
  switch (L.K) {
    case 1: LAUNCH_TLAT(1); break;
    case 2: LAUNCH_TLAT(2); break;
    case 4: LAUNCH_TLAT(4); break;
    case 8: LAUNCH_TLAT(8); break;
    default: LAUNCH_TLAT(16); break;
  }
#undef LAUNCH_TLAT
  return launch_status();
}

int run_grad_stream(const Common& c, void* grads, int zero_durations) {
  const Layout& L = c.L;
  const long long rows = (long long)c.B * c.T * c.U;
  unsigned grid; long long chunk;
  stream_grid(rows, &grid, &chunk);
  const float* coef = (const float*)(c.ws + L.off_coef);
#define LAUNCH_GRAD(DT)                                                                                              \
  hipLaunchKernelGGL(grad_stream_kernel<DT>, dim3(grid), dim3(256), 0, c.stream, c.acts, grads, coef, c.V, c.D,       \
                     c.blank, L.CS, zero_durations, rows, chunk)
  if (c.dt == MI_DTYPE_F32) LAUNCH_GRAD(MI_DTYPE_F32);
  else if (c.dt == MI_DTYPE_BF16) LAUNCH_GRAD(MI_DTYPE_BF16);
  else LAUNCH_GRAD(MI_DTYPE_F16);
#undef LAUNCH_GRAD
  return launch_status();
}

int run_rnnt_cells(const Common& c, const float* grad_scale, float lambda, float clamp) {
  const Layout& L = c.L;
  const long long cells = (long long)c.B * c.T * c.U;
  const unsigned grid = (unsigned)((cells + 255) / 256);
  hipLaunchKernelGGL(rnnt_cell_kernel, dim3(grid), dim3(256), 0, c.stream, (const float*)(c.ws + L.off_denom),
                     (const float*)(c.ws + L.off_arcs), (const double*)(c.ws + L.off_alphas),
                     (const double*)(c.ws + L.off_betas), (const double*)(c.ws + L.off_ll), c.labels, c.act_lens,
                     c.label_lens, grad_scale, (float*)(c.ws + L.off_coef), c.T, c.U, c.V, c.blank, L.ND, L.Us, L.A,
                     L.CS, lambda, clamp, cells);
  return launch_status();
}

int run_tdt_cells(const Common& c, const float* grad_scale, float lambda, float clamp, const TdtParams& prm) {
  const Layout& L = c.L;
  const long long cells = (long long)c.B * c.T * c.U;
  const unsigned grid = (unsigned)((cells + 255) / 256);
  hipLaunchKernelGGL(tdt_cell_kernel, dim3(grid), dim3(256), 0, c.stream, (const float*)(c.ws + L.off_denom),
                     (const float*)(c.ws + L.off_arcs), (const double*)(c.ws + L.off_alphas),
                     (const double*)(c.ws + L.off_betas), (const double*)(c.ws + L.off_ll), c.labels, c.act_lens,
                     c.label_lens, grad_scale, (float*)(c.ws + L.off_coef), c.T, c.U, c.V, c.blank, L.ND, L.Us, L.A,
                     L.CS, lambda, clamp, cells, prm);
  return launch_status();
}

}  // namespace

// ----------------------------------------------------------------------------------------
// C ABI
// ----------------------------------------------------------------------------------------
extern "C" {

int mi_transducer_abi_version(void) { return 1; }

int mi_transducer_workspace_bytes(int B, int T, int U, int D, size_t* out_bytes) {
  Layout L;
  if (!out_bytes || !make_layout(B, T, U, D, &L)) return MI_TRANSDUCER_INVALID_VALUE;
  *out_bytes = L.total;
  return MI_TRANSDUCER_SUCCESS;
}

int mi_rnnt_forward(const void* acts, int act_dtype, const int64_t* labels, const int64_t* act_lens,
                    const int64_t* label_lens, float* costs, int B, int T, int U, int V, int blank,
                    float fastemit_lambda, int with_betas, void* workspace, size_t workspace_bytes, void* stream) {
  Common c;
  if (!costs) return MI_TRANSDUCER_INVALID_VALUE;
  int st = check_common(acts, act_dtype, labels, act_lens, label_lens, B, T, U, V, 0, blank, workspace,
                        workspace_bytes, stream, &c);
  if (st) return st;
  if ((st = run_denom(c))) return st;
  return run_rnnt_lattice(c, costs, fastemit_lambda, with_betas);
}

int mi_rnnt_backward(const void* acts, int act_dtype, const int64_t* labels, const int64_t* act_lens,
                     const int64_t* label_lens, void* grads, const float* grad_scale, int B, int T, int U, int V,
                     int blank, float fastemit_lambda, float clamp, void* workspace, size_t workspace_bytes,
                     void* stream) {
  Common c;
  if (!grads || clamp < 0.f) return MI_TRANSDUCER_INVALID_VALUE;
  int st = check_common(acts, act_dtype, labels, act_lens, label_lens, B, T, U, V, 0, blank, workspace,
                        workspace_bytes, stream, &c);
  if (st) return st;
  if ((st = run_rnnt_cells(c, grad_scale, fastemit_lambda, clamp))) return st;
  return run_grad_stream(c, grads, 0);
}

int mi_rnnt_loss(const void* acts, int act_dtype, const int64_t* labels, const int64_t* act_lens,
                 const int64_t* label_lens, float* costs, void* grads, const float* grad_scale, int B, int T, int U,
                 int V, int blank, float fastemit_lambda, float clamp, void* workspace, size_t workspace_bytes,
                 void* stream) {
  int st = mi_rnnt_forward(acts, act_dtype, labels, act_lens, label_lens, costs, B, T, U, V, blank, fastemit_lambda,
                           grads != nullptr, workspace, workspace_bytes, stream);
  if (st || !grads) return st;
  return mi_rnnt_backward(acts, act_dtype, labels, act_lens, label_lens, grads, grad_scale, B, T, U, V, blank,
                          fastemit_lambda, clamp, workspace, workspace_bytes, stream);
}

int mi_tdt_forward(const void* acts, int act_dtype, const int64_t* labels, const int64_t* act_lens,
                   const int64_t* label_lens, float* costs, int B, int T, int U, int V, int D,
                   const int32_t* durations_host, int blank, float fastemit_lambda, float sigma, int use_plain_rnnt,
                   int with_betas, void* workspace, size_t workspace_bytes, void* stream) {
  Common c;
  TdtParams prm;
  if (!costs) return MI_TRANSDUCER_INVALID_VALUE;
  int st = make_tdt_params(D, durations_host, sigma, &prm);
  if (st) return st;
  st = check_common(acts, act_dtype, labels, act_lens, label_lens, B, T, U, V, D, blank, workspace, workspace_bytes,
                    stream, &c);
  if (st) return st;
  if ((st = run_denom(c))) return st;
  // omega branch (gpu_rnnt.py:607-622): the plain RNNT recursion over the token logits
  if (use_plain_rnnt) return run_rnnt_lattice(c, costs, fastemit_lambda, with_betas);
  return run_tdt_lattice(c, costs, fastemit_lambda, with_betas, prm);
}

int mi_tdt_backward(const void* acts, int act_dtype, const int64_t* labels, const int64_t* act_lens,
                    const int64_t* label_lens, void* grads, const float* grad_scale, int B, int T, int U, int V, int D,
                    const int32_t* durations_host, int blank, float fastemit_lambda, float clamp, float sigma,
                    int use_plain_rnnt, void* workspace, size_t workspace_bytes, void* stream) {
  Common c;
  TdtParams prm;
  if (!grads || clamp < 0.f) return MI_TRANSDUCER_INVALID_VALUE;
  int st = make_tdt_params(D, durations_host, sigma, &prm);
  if (st) return st;
  st = check_common(acts, act_dtype, labels, act_lens, label_lens, B, T, U, V, D, blank, workspace, workspace_bytes,
                    stream, &c);
  if (st) return st;
  if (use_plain_rnnt) {  // gpu_rnnt.py:646-682: token gradient from the RNNT kernel, duration gradient stays zero
    if ((st = run_rnnt_cells(c, grad_scale, fastemit_lambda, clamp))) return st;
    return run_grad_stream(c, grads, 1);
  }
  if ((st = run_tdt_cells(c, grad_scale, fastemit_lambda, clamp, prm))) return st;
  return run_grad_stream(c, grads, 0);
}

int mi_tdt_loss(const void* acts, int act_dtype, const int64_t* labels, const int64_t* act_lens,
                const int64_t* label_lens, float* costs, void* grads, const float* grad_scale, int B, int T, int U,
                int V, int D, const int32_t* durations_host, int blank, float fastemit_lambda, float clamp, float sigma,
                int use_plain_rnnt, void* workspace, size_t workspace_bytes, void* stream) {
  int st = mi_tdt_forward(acts, act_dtype, labels, act_lens, label_lens, costs, B, T, U, V, D, durations_host, blank,
                          fastemit_lambda, sigma, use_plain_rnnt, grads != nullptr, workspace, workspace_bytes, stream);
  if (st || !grads) return st;
  return mi_tdt_backward(acts, act_dtype, labels, act_lens, label_lens, grads, grad_scale, B, T, U, V, D,
                         durations_host, blank, fastemit_lambda, clamp, sigma, use_plain_rnnt, workspace,
                         workspace_bytes, stream);
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
                     (const double*)(ws + L.off_betas), (const double*)(ws + L.off_ll), act_lens, label_lens, denom,
                     alphas, betas, ll_forward, ll_backward, B, T, U, L.ND, L.Us, cells);
  return launch_status();
}

int mi_transducer_length_maxima(const int64_t* act_lens, const int64_t* label_lens, int B, int64_t* out,
                                void* stream) {
  if (!act_lens || !label_lens || !out || B <= 0) return MI_TRANSDUCER_INVALID_VALUE;
  hipLaunchKernelGGL(length_maxima_kernel, dim3(1), dim3(256), 0, (hipStream_t)stream, act_lens, label_lens, B, out);
  return launch_status();
}

}  // extern "C"
