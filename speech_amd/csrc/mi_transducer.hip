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
#include <stdio.h>
#include <stdint.h>

#include <vector>

#include "mi_transducer.h"

// Tunables of the two bandwidth passes (compile-time; the defaults are the measured best).
#ifndef MI_XCD_MAP
#define MI_XCD_MAP 1  // 1: each XCD streams one contiguous eighth of the (b,t) rows
#endif
#ifndef MI_NT_K1
#define MI_NT_K1 0    // non-temporal loads in the long-row denominator pass
#endif
#ifndef MI_NT_K4
#define MI_NT_K4 0    // non-temporal loads in the long-row gradient pass
#endif

namespace {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kNegInf = -INFINITY;
constexpr double kTdtNeg = -10000.0;  // gpu_rnnt_kernel.py:38
constexpr int kRowsPerBlock = 4;      // one wave per row, 256-thread blocks
constexpr int kCoefBase = 8;
// flags of the gradient pass
constexpr int kFlagZeroDurations = 1;  // omega branch of TDT: the duration block of the gradient is zero
constexpr int kFlagPaddingDone = 2;    // padded cells were already zero-filled (mi_transducer_zero_padding)
          // floats per cell before the duration-gradient block

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
// the exponential of the two streaming passes (one hardware v_exp_f32 per logit)
__device__ __forceinline__ float stream_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float clamp_sym(float g, float bound) { return fminf(fmaxf(g, -bound), bound); }

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
    const char* p = (const char*)base + first_elem * Elem<DT>::BYTES;
    const int misbytes = (int)((uintptr_t)p & 15);
    vp = (const uint4*)(p - misbytes);
    mis = misbytes / Elem<DT>::BYTES;
  }
};

// ----------------------------------------------------------------------------------------
// Row streaming helpers shared by the two bandwidth passes.
//
// A row of VD elements starting at an arbitrary element offset is split into
//   head : the elements before the first 16-byte boundary inside the row   (< VEC of them)
//   body : nb whole aligned vectors, vector jb0 + i of the row's window     (the bulk)
//   tail : what is left of the token logits after the last whole vector     (< VEC)
// The body is moved with aligned 16-byte accesses, R vectors per lane in flight; head and
// tail (and the D duration entries of a TDT row) are moved one element per lane.
// ----------------------------------------------------------------------------------------
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

// streaming load: the logits are read exactly once per pass, keep them out of the caches' way
template <bool NT> __device__ __forceinline__ uint4 load_stream(const uint4* p) {
  if constexpr (NT) {
    const u32x4 v = __builtin_nontemporal_load((const u32x4*)p);
    return make_uint4(v.x, v.y, v.z, v.w);
  } else {
    return *p;
  }
}

// n / d for n < 2^31 by one multiply and one shift (the round-up multiplier of Granlund and
// Montgomery, "Division by invariant integers using multiplication"): the hardware has no integer
// divide, and the two divisions that split a workgroup id into (b, t, chunk) would otherwise cost
// some sixty instructions at the head of every wave.
struct FastDiv {
  unsigned mul, shift;
};
inline FastDiv make_fastdiv(unsigned d) {
  unsigned l = 0;
  while ((1ull << l) < d) ++l;
  FastDiv f;
  f.mul = (unsigned)((((unsigned long long)1 << 32) * (((unsigned long long)1 << l) - d)) / d + 1);
  f.shift = l;
  return f;
}
__device__ __forceinline__ unsigned fast_div(unsigned n, FastDiv f) { return (__umulhi(n, f.mul) + n) >> f.shift; }
struct GridDiv {
  FastDiv chunks, T;
};
inline GridDiv make_griddiv(int nchunks, int T) {
  GridDiv g;
  g.chunks = make_fastdiv((unsigned)nchunks);
  g.T = make_fastdiv((unsigned)T);
  return g;
}

// Workgroups are dealt round-robin to the 8 XCDs in launch order.  The logical block id is
// permuted so that each XCD takes MI_XCD_SPAN consecutive logical blocks (a contiguous piece
// of the tensor) per turn: contiguous enough for the XCD's own L2 and TLB to see a linear
// walk, fine enough that utterances of different lengths spread evenly over the XCDs.
// MI_XCD_SPAN = 1 is the plain launch order.  The grid is a multiple of 8 * MI_XCD_SPAN.
#ifndef MI_K1_REVERSE
#define MI_K1_REVERSE 1
#endif
#ifndef MI_K4_REVERSE
#define MI_K4_REVERSE 0
#endif
#ifndef MI_XCD_SPAN
#define MI_XCD_SPAN 1024
#endif
__device__ __forceinline__ unsigned logical_block() {
  const unsigned xcd = blockIdx.x & 7u, turn = blockIdx.x >> 3;
  return (turn / MI_XCD_SPAN) * (8u * MI_XCD_SPAN) + xcd * MI_XCD_SPAN + (turn % MI_XCD_SPAN);
}

#ifndef MI_NT_STORE
#define MI_NT_STORE 0
#endif
__device__ __forceinline__ void store_stream(uint4* p, const uint4& v) {
#if MI_NT_STORE
  u32x4 x;
  x.x = v.x; x.y = v.y; x.z = v.z; x.w = v.w;
  __builtin_nontemporal_store(x, (u32x4*)p);
#else
  *p = v;
#endif
}

// Which (b, t, u) row a wave works on.  Grid = (8 * ceil(U/4), ceil(B*T/8)): workgroups are
// dealt round-robin to the 8 XCDs in linear-id order, so blockIdx.x & 7 names the XCD; each
// XCD gets a contiguous eighth of the (b,t) rows and walks it in memory order.  Rows are not
// cache-line aligned, so neighbours share lines: keeping them in one L2 lets a gradient line
// be completed before it is written back.
struct RowId {
  int b, t, u;
  bool in_range;
};
__device__ __forceinline__ RowId row_of_wave(int T, int U, int BT, int bt_chunk) {
  RowId id;
#if MI_XCD_MAP
  const unsigned xcd = blockIdx.x & 7u, ub = blockIdx.x >> 3;
  const unsigned bt = xcd * (unsigned)bt_chunk + blockIdx.y;
#else
  const unsigned ub = blockIdx.x, bt = blockIdx.y;
  (void)bt_chunk;
#endif
  id.u = __builtin_amdgcn_readfirstlane((int)(ub * kRowsPerBlock + (threadIdx.x >> 6)));
  id.b = (int)(bt / (unsigned)T);
  id.t = (int)(bt - (unsigned)id.b * (unsigned)T);
  id.in_range = bt < (unsigned)BT && id.u < U;
#if MI_XCD_MAP
  id.in_range = id.in_range && blockIdx.y < (unsigned)bt_chunk;
#endif
  return id;
}

template <int DT> struct RowSplit {
  int hc;   // head elements: row elements [0, hc)
  int jb0;  // first whole vector of the window
  int nb;   // whole vectors: row elements [hc, hc + nb*VEC)
  int tc;   // tail elements: row elements [hc + nb*VEC, V)
  __device__ __forceinline__ RowSplit(int mis, int V) {
    constexpr int VEC = Elem<DT>::VEC;
    hc = mis ? VEC - mis : 0;
    if (hc > V) hc = V;
    jb0 = mis ? 1 : 0;
    nb = (V - hc) / VEC;
    tc = V - hc - nb * VEC;
  }
  __device__ __forceinline__ int tail0() const { return hc + nb * Elem<DT>::VEC; }
  // window index of whole vector j, clamped into the row so that any lane may load it
  __device__ __forceinline__ int body_vector(int j) const { return nb > 0 ? jb0 + (j < nb ? j : nb - 1) : 0; }
  // head and tail token elements are handled one per lane: lanes [0,hc) take the head, lanes
  // [VEC, VEC+tc) the tail; -1 for every other lane
  __device__ __forceinline__ int extra_token(int lane) const {
    constexpr int VEC = Elem<DT>::VEC;
    if (lane < hc) return lane;
    if (lane >= VEC && lane < VEC + tc) return tail0() + lane - VEC;
    return -1;
  }
};

// A load through the scalar unit: for a wave-uniform address of data that no store of the running
// kernel touches (inputs, and what earlier kernels of the stream left in the workspace).  Scalar
// loads do not queue behind the wave's vector traffic.
template <class T> __device__ __forceinline__ T sload(const T* p) {
  typedef const T __attribute__((address_space(4))) * const_ptr;
  return *(const_ptr)(unsigned long long)p;
}
// wave-uniform values as the compiler should see them: held in scalar registers
__device__ __forceinline__ int uni(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ float uni(float v) { return __int_as_float(uni(__float_as_int(v))); }
__device__ __forceinline__ double uni(double v) {
  return __hiloint2double(uni(__double2hiint(v)), uni(__double2loint(v)));
}
__device__ __forceinline__ long long uni(long long v) {
  const unsigned lo = (unsigned)uni((int)(unsigned)v), hi = (unsigned)uni((int)((unsigned long long)v >> 32));
  return (long long)(((unsigned long long)hi << 32) | lo);
}
// the two lengths of utterance b, clamped into the tensor, fetched in one round trip
struct UttLens {
  int Tb, Ub;
};
__device__ __forceinline__ UttLens load_lens(const int64_t* act_lens, const int64_t* label_lens, int b, int T, int U) {
  long long len_t = uni((long long)sload(act_lens + b)), len_u = uni((long long)sload(label_lens + b));
  asm("" : "+s"(len_t), "+s"(len_u));
  // a length outside [0, limit] (never seen from a checked caller) is taken as the limit
  UttLens r;
  r.Tb = max((unsigned long long)len_t > (unsigned)T ? T : (int)len_t, 1);
  r.Ub = max((unsigned long long)len_u >= (unsigned)U ? U : (int)len_u + 1, 1);
  return r;
}

// running (max, sum of exp) of one lane, base-2 scaled: sum_i 2^(x_i*log2e - m*log2e)
struct LaneLse {
  float m, s;
  __device__ __forceinline__ LaneLse() : m(-1.0e30f), s(0.f) {}
  template <int N> __device__ __forceinline__ void add(const float* x) {
    float cm = x[0];
#pragma unroll
    for (int i = 1; i < N; ++i) cm = fmaxf(cm, x[i]);
    const float mnew = fmaxf(m, cm);  // never below -1e30: no inf - inf, and -mnew*log2e stays finite
    const float off = -mnew * kLog2e;
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < N; ++i) acc += fast_exp2(fmaf(x[i], kLog2e, off));
    s = fmaf(s, fast_exp2((m - mnew) * kLog2e), acc);
    m = mnew;
  }
};

// ----------------------------------------------------------------------------------------
// Pass 1: denominators + gather (replaces reduce.py:121-248 and the per-step gathers of
// logp() in gpu_rnnt_kernel.py:42-64).  Grid (ceil(U/4), T, B), one wave per (b,t,u) row;
// waves of padded rows exit at once.
// ----------------------------------------------------------------------------------------
template <int DT>
__global__ __launch_bounds__(256) void denom_gather_kernel(
    const void* __restrict__ acts, const int64_t* __restrict__ labels, const int64_t* __restrict__ act_lens,
    const int64_t* __restrict__ label_lens, float* __restrict__ denom, float* __restrict__ arcs, int T, int U, int V,
    int D, int nbig, int blank, int ND, int Us, int A, int BT, int bt_chunk) {
  constexpr int VEC = Elem<DT>::VEC;
  constexpr int R = 4;  // vectors in flight per lane
  constexpr bool NT = MI_NT_K1 != 0;
  const int lane = threadIdx.x & 63;
  const RowId id = row_of_wave(T, U, BT, bt_chunk);
  if (!id.in_range) return;
  const int b = id.b, t = id.t, u = id.u;
  const int Tb = clampi(act_lens[b], 1, T);
  const int Ub = clampi(label_lens[b] + 1, 1, U);
  if (t >= Tb || u >= Ub) return;

  const int VD = V + D;
  const size_t r = ((size_t)b * T + t) * U + u;
  const size_t e0 = r * VD;
  // the two gathered logits do not depend on the reduction: ask for them first
  const int lab = (u < Ub - 1) ? clampi(labels[(size_t)b * (U - 1) + u], 0, V - 1) : -1;
  const float xb = Elem<DT>::load1(acts, e0 + blank);
  const float xl = Elem<DT>::load1(acts, e0 + (lab >= 0 ? lab : blank));
  const float xd = (lane < D) ? Elem<DT>::load1(acts, e0 + V + lane)
                              : (lane < nbig ? Elem<DT>::load1(acts, e0 + blank - 1 - lane) : kNegInf);

  const RowWindow<DT> w(acts, e0);
  const RowSplit<DT> sp(w.mis, V);
  // head and tail: one element per lane (lanes [0,hc) and [VEC, VEC+tc))
  float xe = kNegInf;
  if (lane < sp.hc) xe = Elem<DT>::load1(acts, e0 + lane);
  else if (lane >= VEC && lane < VEC + sp.tc) xe = Elem<DT>::load1(acts, e0 + sp.tail0() + lane - VEC);

  LaneLse acc;
  const uint4* vp = w.vp + sp.jb0 + lane;
  int rounds = sp.nb >> 6;
  for (; rounds >= R; rounds -= R, vp += 64 * R) {
    uint4 raw[R];
#pragma unroll
    for (int k = 0; k < R; ++k) raw[k] = load_stream<NT>(vp + 64 * k);
    float x[R * VEC];
#pragma unroll
    for (int k = 0; k < R; ++k) Elem<DT>::unpack(raw[k], x + k * VEC);
    acc.add<R * VEC>(x);
  }
  for (; rounds > 0; --rounds, vp += 64) {
    float x[VEC];
    Elem<DT>::unpack(load_stream<NT>(vp), x);
    acc.add<VEC>(x);
  }
  if (sp.nb & 63) {  // last, partial round of whole vectors
    float x[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) x[i] = kNegInf;
    if (lane < (sp.nb & 63)) Elem<DT>::unpack(load_stream<NT>(vp), x);
    acc.add<VEC>(x);
  }
  acc.add<1>(&xe);

  const float M = wave_max(acc.m);
  const float S = wave_sum(acc.s * fast_exp2((acc.m - M) * kLog2e));
  const float dn = -M - logf(S);

  const size_t base = ((size_t)(b * ND + t + u) * A) * Us + u;
  if (lane == 0) {
    denom[r] = dn;
    arcs[base] = xb + dn;
    arcs[base + Us] = lab >= 0 ? xl + dn : 0.f;
  }
  if (D > 0) {  // duration log-softmax (rnnt_pytorch.py:568), one lane per duration
    const float dm = wave_max(xd);
    const float ds = wave_sum(lane < D ? expf(xd - dm) : 0.f);
    const float dden = -dm - logf(ds);
    if (lane < D) arcs[base + (size_t)(2 + lane) * Us] = xd + dden;
  }
  if (lane < nbig) arcs[base + (size_t)(2 + lane) * Us] = xd + dn;  // big-blank log-probs (multi-blank)
}

// ----------------------------------------------------------------------------------------
// Lattice helpers
// ----------------------------------------------------------------------------------------
// log(exp(a)+exp(b)) with the sum carried in fp64 and the correction term in fp32
// (rnnt_helper.py:42-53: the other operand is returned when one is -inf).  Branch-free:
// with one operand -inf the correction is log(1 + 2^-inf) = 0; only (-inf, -inf) needs the select.
__device__ __forceinline__ double lse_h(double a, double b) {
  const double m = fmax(a, b);
  const double n = fmin(a, b);
  const float d = (float)(n - m);
  const double r = m + (double)(__builtin_amdgcn_logf(1.0f + fast_exp2(d * kLog2e)) * 0.6931471805599453f);
  return (n == -INFINITY) ? m : r;
}

// The RNNT recursion keeps "log 0" as a large finite number instead of -inf: sums stay finite
// (arc values are forced finite too), so the two-operand log-sum-exp needs no special cases.
constexpr double kLogZero = -1.0e300;
__device__ __forceinline__ double lse_fin(double a, double b) {
  const double m = fmax(a, b);
  const float d = -fabsf((float)(a - b));  // -inf when one operand is log 0: the correction vanishes
  return m + (double)(__builtin_amdgcn_logf(1.0f + fast_exp2(d * kLog2e)) * 0.6931471805599453f);
}

// value of the lane below / above (wave shift by one lane through DPP, no LDS round trip);
// lane 0 / lane 63 receives `fill`
__device__ __forceinline__ double from_lane_below(double v, double fill) {
  const int lo = __builtin_amdgcn_update_dpp(__double2loint(fill), __double2loint(v), 0x138, 0xf, 0xf, false);
  const int hi = __builtin_amdgcn_update_dpp(__double2hiint(fill), __double2hiint(v), 0x138, 0xf, 0xf, false);
  return __hiloint2double(hi, lo);
}
__device__ __forceinline__ double from_lane_above(double v, double fill) {
  const int lo = __builtin_amdgcn_update_dpp(__double2loint(fill), __double2loint(v), 0x130, 0xf, 0xf, false);
  const int hi = __builtin_amdgcn_update_dpp(__double2hiint(fill), __double2hiint(v), 0x130, 0xf, 0xf, false);
  return __hiloint2double(hi, lo);
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

template <int K> __device__ __forceinline__ void store_k(double* p, const double* v) {
  typedef double d2 __attribute__((ext_vector_type(2)));
  if constexpr (K == 1) {
    p[0] = v[0];
  } else {
#pragma unroll
    for (int q = 0; q < K / 2; ++q) {
      d2 x;
      x[0] = v[2 * q];
      x[1] = v[2 * q + 1];
      *(d2*)(p + 2 * q) = x;
    }
  }
}

// Arc log-probs of cells outside the utterance's lattice were never written: whatever bits
// are there must not turn a -inf lattice value into NaN, so they are forced finite.
// (one median-of-three instruction; a NaN comes out as the lower bound)
__device__ __forceinline__ float finite_arc(float x) { return __builtin_amdgcn_fmed3f(x, -3.0e38f, 3.0e38f); }

// RNNT lattice: one wave per (utterance, direction).  Lane l owns columns u = l*K .. l*K+K-1
// and, at step n, the cells (n-u, u) of anti-diagonal n.
//   alpha (gpu_rnnt_kernel.py:73-172): every cell pushes e = alpha + lp_label to its right
//   neighbour and s = alpha + lp_blank to the cell below; the next diagonal is lse(e_in, s_in).
//   beta  (gpu_rnnt_kernel.py:175-269): pulled from the diagonal above.
// No boundary tests in the loop: everything starts at log 0 (kLogZero), the only finite source is
// alpha(0,0) = 0 (resp. the corner beta(Tb-1,Ub-1) = lp_blank), and values only flow right/down
// (resp. left/up), so cells outside the lattice either stay at log 0 (where they could feed a
// valid cell) or hold junk that no valid cell ever reads.  Every lane stores its K values of
// every diagonal: the skewed rows are 64*K wide.
// The arc log-probs of P diagonals are fetched into registers while the previous P
// diagonals are being computed; they do not depend on the recursion.
template <int K>
__global__ __launch_bounds__(64) void rnnt_lattice_kernel(const float* __restrict__ arcs, double* __restrict__ alphas,
                                                          double* __restrict__ betas, double* __restrict__ ll,
                                                          float* __restrict__ costs,
                                                          const int64_t* __restrict__ act_lens,
                                                          const int64_t* __restrict__ label_lens, int T, int U, int ND,
                                                          int A, float cost_scale, int with_betas) {
  constexpr int P = Prefetch<K>::P;
  constexpr int Us = 64 * K;
  // the recursion is one long dependent chain: let this wave win the issue arbitration against
  // whatever bandwidth-bound waves share its SIMD
  __builtin_amdgcn_s_setprio(3);
  const int b = with_betas ? (int)(blockIdx.x >> 1) : (int)blockIdx.x;
  const int dir = with_betas ? (int)(blockIdx.x & 1) : 0;
  const int lane = threadIdx.x;
  const int u0 = lane * K;
  const int Tb = clampi(act_lens[b], 1, T);
  const int Ub = clampi(label_lens[b] + 1, 1, U);
  const int nd = Tb + Ub - 1;
  const size_t row_pitch = (size_t)A * Us;
  const float* arcs_b = arcs + (size_t)b * ND * row_pitch + u0;
  const double NINF = kLogZero;

  // rows [n, n + step*P) of the blank and label planes, this lane's K columns (rows clamped into
  // the utterance so that the loads never depend on a branch)
  auto load_rows = [&](int nfirst, int step, float(&Bk)[P][K], float(&Lb)[P][K]) {
#pragma unroll
    for (int p = 0; p < P; ++p) {
      int n = nfirst + step * p;
      n = n < 0 ? 0 : (n >= nd ? nd - 1 : n);
      const float* rp = arcs_b + (size_t)n * row_pitch;
      load_k<K>(rp, Bk[p]);
      load_k<K>(rp + Us, Lb[p]);
    }
  };

  if (dir == 0) {
    double* out = alphas + (size_t)b * ND * Us + u0;
    double e[K], s[K];
#pragma unroll
    for (int k = 0; k < K; ++k) e[k] = s[k] = NINF;
    if (lane == 0) s[0] = 0.0;  // makes alpha(0,0) = lse(log 0, 0) = 0
    auto step_fn = [&](int n, const float* bk, const float* lb) {
      const double left = from_lane_below(e[K - 1], NINF);
      double a[K];
#pragma unroll
      for (int k = 0; k < K; ++k) a[k] = lse_fin(k == 0 ? left : e[k - 1], s[k]);
      store_k<K>(out + (size_t)n * Us, a);
#pragma unroll
      for (int k = 0; k < K; ++k) {
        e[k] = a[k] + (double)finite_arc(lb[k]);
        s[k] = a[k] + (double)finite_arc(bk[k]);
      }
    };
    float bufa_b[P][K], bufa_l[P][K], bufb_b[P][K], bufb_l[P][K];
    int n0 = 0;
    load_rows(0, 1, bufa_b, bufa_l);
    for (; n0 + 2 * P <= nd; n0 += 2 * P) {
      load_rows(n0 + P, 1, bufb_b, bufb_l);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int p = 0; p < P; ++p) step_fn(n0 + p, bufa_b[p], bufa_l[p]);
      load_rows(n0 + 2 * P, 1, bufa_b, bufa_l);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int p = 0; p < P; ++p) step_fn(n0 + P + p, bufb_b[p], bufb_l[p]);
    }
    for (; n0 < nd; ++n0) {  // fewer than 2P diagonals left
      float bk[K], lb[K];
      const float* rp = arcs_b + (size_t)n0 * row_pitch;
      load_k<K>(rp, bk);
      load_k<K>(rp + Us, lb);
      step_fn(n0, bk, lb);
    }
    // after the last diagonal the owner of column Ub-1 holds s = alpha(Tb-1,Ub-1) + lp_blank = llForward
#pragma unroll
    for (int k = 0; k < K; ++k)
      if (u0 + k == Ub - 1) {
        ll[2 * b] = s[k];
        costs[b] = -(float)s[k] * cost_scale;  // rnnt_helper.py:106-116
      }
  } else {
    double* out = betas + (size_t)b * ND * Us + u0;
    double bt[K];
    // diagonal nd-1 holds the corner cell only: beta(Tb-1,Ub-1) = lp_blank(Tb-1,Ub-1)
    {
      float bk[K];
      load_k<K>(arcs_b + (size_t)(nd - 1) * row_pitch, bk);
#pragma unroll
      for (int k = 0; k < K; ++k) bt[k] = (u0 + k == Ub - 1) ? (double)bk[k] : NINF;
      store_k<K>(out + (size_t)(nd - 1) * Us, bt);
    }
    auto step_fn = [&](int n, const float* bk, const float* lb) {
      const double right = from_lane_above(bt[0], NINF);
      double nv[K];
#pragma unroll
      for (int k = 0; k < K; ++k) {
        const double rgt = (k == K - 1) ? right : bt[k + 1];
        nv[k] = lse_fin(rgt + (double)finite_arc(lb[k]), bt[k] + (double)finite_arc(bk[k]));
      }
      store_k<K>(out + (size_t)n * Us, nv);
#pragma unroll
      for (int k = 0; k < K; ++k) bt[k] = nv[k];
    };
    float bufa_b[P][K], bufa_l[P][K], bufb_b[P][K], bufb_l[P][K];
    int n0 = nd - 2;
    load_rows(n0, -1, bufa_b, bufa_l);
    for (; n0 - 2 * P + 1 >= 0; n0 -= 2 * P) {
      load_rows(n0 - P, -1, bufb_b, bufb_l);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int p = 0; p < P; ++p) step_fn(n0 - p, bufa_b[p], bufa_l[p]);
      load_rows(n0 - 2 * P, -1, bufa_b, bufa_l);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int p = 0; p < P; ++p) step_fn(n0 - P - p, bufb_b[p], bufb_l[p]);
    }
    for (; n0 >= 0; --n0) {
      float bk[K], lb[K];
      const float* rp = arcs_b + (size_t)n0 * row_pitch;
      load_k<K>(rp, bk);
      load_k<K>(rp + Us, lb);
      step_fn(n0, bk, lb);
    }
    if (lane == 0) ll[2 * b + 1] = bt[0];  // beta(0,0)
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
    // scores of the blank arcs that end the utterance, one per duration (summed after the loop in the reference's order)
    double end_term[MI_TRANSDUCER_MAX_DURATIONS];
    for (int i = 0; i < MI_TRANSDUCER_MAX_DURATIONS; ++i) end_term[i] = -INFINITY;
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
                end_term[i] = c;
              }
            }
            if (u + 1 < Ub && t + d < Tb) {
              double* q = em_ring + ((n + d + 1) % R) * Us + u + 1;
              *q = lse_h(*q, (wl - sigma) + dl);
            }
          }
          if (n == nd - 1) {  // (Tb-1, Ub-1): the last contribution to llForward is in
            // :1046-1071: the duration-1 term is assigned over the -10000 the sum starts from, longer ones are added
            double ll_acc = kTdtNeg;
            for (int i = 0; i < D; ++i) {
              if (prm.dur[i] == 1) ll_acc = end_term[i];
              else if (prm.dur[i] > 1 && end_term[i] != -INFINITY) ll_acc = lse_h(ll_acc, end_term[i]);
            }
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

// TDT lattice, workgroup version (gpu_rnnt_kernel.py:888-1241): one workgroup per (utterance,
// direction), TWO threads per column u, one anti-diagonal per step, one barrier per step.
//   alpha: a finished cell leaves its 2D outgoing arc scores (alpha + arc weight, blank arcs
//          and label arcs per duration) in an LDS ring of R = max_duration + 2 diagonals; a
//          cell's alpha is one log-sum-exp over the <= 2D scores that land on it plus the
//          reference's finite -10000 seeds.
//   beta : the ring holds beta of the last R diagonals.
// Thread (u, 0) sums the D blank arcs of a cell, thread (u, 1) the D label arcs, and the two partial
// (max, sum) pairs meet through one DPP exchange: the recursion is bound by the instructions one
// wave has to issue per step, and this halves them (at twice the waves, which sit on other SIMDs).
// The steps are written with selects only: a wave-uniform test (on a duration, on the position of
// duration 1) would become a taken branch, and with one wave per SIMD every taken branch is paid in
// full (measured: 392 us with such branches, 323 us without, 293 us with two threads per column).
template <int D>
__global__ __launch_bounds__(512) void tdt_lattice_pair_kernel(
    const float* __restrict__ arcs, double* __restrict__ alphas, double* __restrict__ betas, double* __restrict__ ll,
    float* __restrict__ costs, const int64_t* __restrict__ act_lens, const int64_t* __restrict__ label_lens, int T,
    int U, int ND, int Us, float cost_scale, int with_betas, TdtParams prm) {
  constexpr int A = 2 + D;
  constexpr int P = 4;
  extern __shared__ double ring[];
  const int b = with_betas ? (int)(blockIdx.x >> 1) : (int)blockIdx.x;
  const int dir = with_betas ? (int)(blockIdx.x & 1) : 0;
  const int u = threadIdx.x >> 1;     // blockDim.x == 2 * Us
  const bool lab = threadIdx.x & 1;   // this thread's half: label arcs (else blank arcs)
  const int Tb = clampi(act_lens[b], 1, T);
  const int Ub = clampi(label_lens[b] + 1, 1, U);
  const int nd = Tb + Ub - 1;
  const int R = prm.R;
  const double sigma = (double)prm.sigma;
  const double NEG = kTdtNeg;
  // thr: from which t (alpha) an arc of duration i exists for this half; a blank must advance, so its
  // duration 0 never passes
  int dur[D], thr[D];
#pragma unroll
  for (int i = 0; i < D; ++i) {
    dur[i] = prm.dur[i];
    thr[i] = (lab || prm.dur[i] > 0) ? prm.dur[i] : (1 << 28);
  }
  const bool stay = prm.dur[0] == 0;  // a label may stay on its frame
  const bool one_first = prm.one_idx == 0;
  const size_t row_pitch = (size_t)A * Us;
  const float* arcs_b = arcs + (size_t)b * ND * row_pitch + u;
  const int own_plane = lab ? 1 : 0;  // the token arc of this half: label or blank

  // [0]: this half's token log-prob, [1+i]: duration log-probs
  auto load_rows = [&](int nfirst, int step, float(&W)[P][1 + D]) {
#pragma unroll
    for (int p = 0; p < P; ++p) {
      int n = nfirst + step * p;
      n = n < 0 ? 0 : (n >= nd ? nd - 1 : n);
      const float* rp = arcs_b + (size_t)n * row_pitch;
      W[p][0] = rp[(size_t)own_plane * Us];
#pragma unroll
      for (int i = 0; i < D; ++i) W[p][1 + i] = rp[(size_t)(2 + i) * Us];
    }
  };
  // the other half's value (lanes 2k and 2k+1 swap)
  auto partner_f = [&](float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xf, 0xf, true));
  };
  auto partner_d = [&](double v) {
    return __hiloint2double(__builtin_amdgcn_update_dpp(0, __double2hiint(v), 0xB1, 0xf, 0xf, true),
                            __builtin_amdgcn_update_dpp(0, __double2loint(v), 0xB1, 0xf, 0xf, true));
  };
  // log-sum-exp over both halves: each half holds D entries (-inf = absent) and `seed` copies (0 or 1) of the sentinel
  auto lse_pair = [&](const double* x, int seed) {
    double m = seed > 0 ? NEG : -1.0e300;
#pragma unroll
    for (int i = 0; i < D; ++i) m = fmax(m, x[i]);
    float s = seed > 0 ? fast_exp2((float)(NEG - m) * kLog2e) : 0.f;  // (not seed * exp: 0 * inf for an empty half)
#pragma unroll
    for (int i = 0; i < D; ++i) s += fast_exp2((float)(x[i] - m) * kLog2e);
    const double mo = partner_d(m);
    const float so = partner_f(s);
    const double M = fmax(m, mo);
    const float S = s * fast_exp2((float)(m - M) * kLog2e) + so * fast_exp2((float)(mo - M) * kLog2e);
    return M + (double)(__builtin_amdgcn_logf(S) * 0.6931471805599453f);
  };

  if (dir == 0) {
    const int slot_stride = 2 * D * Us, ring_len = R * slot_stride;
    for (int i = threadIdx.x; i < ring_len; i += 2 * Us) ring[i] = NEG;
    __syncthreads();
    double* out = alphas + (size_t)b * ND * Us + u;
    // ring offsets of the diagonals this half reads: n - d_i (blank arcs, same column) or n - 1 - d_i
    // (label arcs, column u-1); both advance by one slot per step
    int off[D];
#pragma unroll
    for (int i = 0; i < D; ++i) off[i] = (lab ? (R - 1 - dur[i]) : ((R - dur[i]) % R)) * slot_stride;
    int cur_off = 0;
    const int col = lab ? (u > 0 ? u - 1 : 0) : u;
    const int plane0 = lab ? D * Us : 0;
    const bool half_on = !lab || u > 0;  // column 0 has no label arc coming in
    const int seed = half_on ? 1 : 0;    // the emit and the no-emit accumulator are each seeded once
    // arc i lands on this cell from diagonal n on where t = n - u >= its duration: one compare against the
    // (wave-uniform) diagonal number per arc
    int nmin[D];
#pragma unroll
    for (int i = 0; i < D; ++i) nmin[i] = half_on ? u + thr[i] : (1 << 29);
    auto step_fn = [&](int n, const float* w) {
      const int t = n - u;
      double x[D];
#pragma unroll
      for (int i = 0; i < D; ++i) {
        double v = ring[off[i] + plane0 + i * Us + col];
        asm("" : "+v"(v));  // read here, not under the test below
        x[i] = n >= nmin[i] ? v : -INFINITY;
      }
      const double interior = lse_pair(x, seed);
      // row 0: only a duration-0 label arc gets there (:941-955); its score sits in the label half
      const double x0_other = partner_d(x[0]);
      const double label0 = lab ? x[0] : x0_other;
      const double row0 = u == 0 ? 0.0 : (stay ? label0 : NEG);
      const double a = t == 0 ? row0 : interior;
      if (!lab) out[(size_t)n * Us] = a;
      const double wt = (a + (double)w[0]) - sigma;
      double* slot = ring + cur_off + plane0 + u;
#pragma unroll
      for (int i = 0; i < D; ++i) {
        slot[i * Us] = wt + (double)w[1 + i];
      }
#pragma unroll
      for (int i = 0; i < D; ++i) off[i] = off[i] + slot_stride == ring_len ? 0 : off[i] + slot_stride;
      cur_off = cur_off + slot_stride == ring_len ? 0 : cur_off + slot_stride;
      __syncthreads();
    };
    float wa[P][1 + D], wb[P][1 + D];
    int n0 = 0;
    load_rows(0, 1, wa);
    for (; n0 + 2 * P <= nd; n0 += 2 * P) {
      load_rows(n0 + P, 1, wb);
#pragma unroll
      for (int p = 0; p < P; ++p) step_fn(n0 + p, wa[p]);
      load_rows(n0 + 2 * P, 1, wa);
#pragma unroll
      for (int p = 0; p < P; ++p) step_fn(n0 + P + p, wb[p]);
    }
    for (; n0 < nd; ++n0) {
      float w[P][1 + D];
      load_rows(n0, 0, w);
      step_fn(n0, w[0]);
    }
    if (!lab && u == Ub - 1) {
      // the blank arcs that end the utterance (:1040-1071) leave from cells (Tb - d_i, Ub-1) of this thread's own
      // column: their alphas are re-read (this thread stored them) and the arc scores formed as in the loop.
      // In the reference's order (:1046-1071): the duration-1 term is ASSIGNED (the -10000 the sum starts from is
      // gone by then: duration 1 sits at position 0 or 1, and a duration 0 before it is skipped), the longer
      // durations are added while they fit the utterance.  The difference to a sum seeded with -10000 shows only
      // when no alignment exists and the terms themselves are down at the sentinel.
      double ll_acc = NEG;
#pragma unroll
      for (int i = 0; i < D; ++i) {
        const int t0 = Tb - dur[i];
        if (dur[i] > 0 && t0 >= 0) {
          const float* rp = arcs_b + (size_t)(t0 + u) * row_pitch;
          const double a = out[(size_t)(t0 + u) * Us];
          const double term = ((a + (double)rp[0]) - sigma) + (double)rp[(size_t)(2 + i) * Us];
          ll_acc = dur[i] == 1 ? term : lse_h(ll_acc, term);
        }
      }
      ll[2 * b] = ll_acc;
      costs[b] = -(float)ll_acc * cost_scale;
    }
  } else {
    const int ring_len = R * Us;
    for (int i = threadIdx.x; i < ring_len; i += 2 * Us) ring[i] = NEG;
    __syncthreads();
    // a blank that ends the utterance (t + d == Tb in the last column, :1137-1148, :1160-1176) is an arc into a
    // virtual cell beta(Tb, Ub-1) = 0 on diagonal nd: with that cell in the ring it needs no case of its own
    if (threadIdx.x == 0) ring[(nd % R) * Us + Ub - 1] = 0.0;
    __syncthreads();
    double* out = betas + (size_t)b * ND * Us + u;
    double last = NEG;
    // arc i leaves this cell while t + d_i < Tb (<= Tb for the blank arcs of the last column), i.e. on diagonals
    // n < nmax[i]: one compare against the (wave-uniform) diagonal number per arc.  A blank of duration 0 never
    // passes (thr = 2^28), a label arc needs a next column.
    int nmax[D];
#pragma unroll
    for (int i = 0; i < D; ++i)
      nmax[i] = (!lab || u + 1 < Ub) ? Tb + u - thr[i] + ((!lab && u == Ub - 1) ? 1 : 0) : -(1 << 29);
    // ring offsets of the diagonals this half reads: n + d_i (blank arcs, same column) or n + d_i + 1
    // (label arcs, column u+1); both go back by one slot per step
    int off[D];
#pragma unroll
    for (int i = 0; i < D; ++i) off[i] = (((nd - 1) % R + dur[i] + (lab ? 1 : 0)) % R) * Us;
    int cur_off = ((nd - 1) % R) * Us;
    const int col = lab ? (u + 1 < Us ? u + 1 : u) : u;
    auto step_fn = [&](int n, const float* w) {
      const int t = n - u;
      const double tok = (double)w[0];
      double x[D];
#pragma unroll
      for (int i = 0; i < D; ++i) {
        double v = ring[off[i] + col];
        asm("" : "+v"(v));
        const double arc = (tok + (double)w[1 + i]) - sigma;
        x[i] = n < nmax[i] ? v + arc : -INFINITY;
      }
      // one seed for the no-emit (blank) accumulator, one for the emit accumulator unless it is the last column
      const double interior = lse_pair(x, (!lab || u != Ub - 1) ? 1 : 0);
      // the corner ends the utterance with one blank of duration 1 (:1137-1148); the rest of the last row
      // takes duration-0 labels only.  Each half sends the partner the one value it may need.
      const double send = lab ? x[0] : (one_first ? x[0] : x[D > 1 ? 1 : 0]);
      const double recv = partner_d(send);
      const double corner = lab ? recv : send, label0 = lab ? send : recv;
      const double last_row = u == Ub - 1 ? corner : (stay ? label0 : NEG);
      const double v = t == Tb - 1 ? last_row : interior;
      if (!lab) {
        out[(size_t)n * Us] = v;
        ring[cur_off + u] = v;
      }
      last = v;
#pragma unroll
      for (int i = 0; i < D; ++i) off[i] = off[i] == 0 ? ring_len - Us : off[i] - Us;
      cur_off = cur_off == 0 ? ring_len - Us : cur_off - Us;
      __syncthreads();
    };
    float wa[P][1 + D], wb[P][1 + D];
    int n0 = nd - 1;
    load_rows(n0, -1, wa);
    for (; n0 - 2 * P + 1 >= 0; n0 -= 2 * P) {
      load_rows(n0 - P, -1, wb);
#pragma unroll
      for (int p = 0; p < P; ++p) step_fn(n0 - p, wa[p]);
      load_rows(n0 - 2 * P, -1, wa);
#pragma unroll
      for (int p = 0; p < P; ++p) step_fn(n0 - P - p, wb[p]);
    }
    for (; n0 >= 0; --n0) {
      float w[P][1 + D];
      load_rows(n0, 0, w);
      step_fn(n0, w[0]);
    }
    if (threadIdx.x == 0) ll[2 * b + 1] = last;  // beta(0,0)
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
// what the gradient pass needs to derive a row's coefficients itself (RNNT, fused path)
struct LatticeView {
  const float* denom;
  const float* arcs;
  const double* alphas;
  const double* betas;
  const double* ll;
  const int64_t* labels;
  const float* grad_scale;
  int grad_scale_stride;
  float grad_mul;
  int ND, Us, A;
  float lambda, clamp;
};

struct RowCoef {
  float dl2;  // denom * log2(e)
  float W;    // occupancy weight * scale
  float cb;   // clamp bound * |scale| (inf = no clamp)
  float gB;   // finished gradient entry of the blank logit
  float gL;   // finished gradient entry of the label logit
  int lab;    // label id, -1 if the cell has no label arc
};

__device__ __forceinline__ RowCoef make_coef(float dn, float W, float PB, float PL, float lpb, float lpl, int lab,
                                             int blank, float clamp, float scale) {
  float gb = __expf(lpb) * W - PB;
  float gl = lab >= 0 ? __expf(lpl) * W - PL : 0.f;
  if (lab == blank) gb = gl = __expf(lpb) * W - PB - PL;
  if (clamp > 0.f) {
    gb = clamp_sym(gb, clamp);
    gl = clamp_sym(gl, clamp);
  }
  RowCoef c;
  c.dl2 = dn * kLog2e;
  c.W = W * scale;
  c.cb = clamp > 0.f ? clamp * fabsf(scale) : INFINITY;
  c.gB = gb * scale;
  c.gL = gl * scale;
  c.lab = lab;
  return c;
}

__device__ __forceinline__ void write_coef(float* out, const RowCoef& c) {
  out[0] = c.dl2;
  out[1] = c.W;
  out[2] = c.cb;
  out[3] = c.gB;
  out[4] = c.gL;
  out[5] = __int_as_float(c.lab);
}

// the RNNT coefficients of cell (b,t,u) from the lattice state (gpu_rnnt_kernel.py:340-403)
__device__ __forceinline__ RowCoef rnnt_coef(const float* __restrict__ denom, const float* __restrict__ arcs,
                                             const double* __restrict__ alphas, const double* __restrict__ betas,
                                             const double* __restrict__ ll, const int64_t* __restrict__ labels,
                                             float scale, int b, int t, int u, int Tb, int Ub, int T, int U, int V,
                                             int blank, int ND, int Us, int A, float lambda, float clamp) {
  const size_t row = (size_t)(b * ND + t + u);
  const size_t sk = row * Us + u;
  const double a = alphas[sk], bb = betas[sk], L = ll[2 * b];
  const float lpb = arcs[row * A * Us + u];
  const float lpl = arcs[row * A * Us + Us + u];
  const int lab = (u < Ub - 1) ? clampi(labels[(size_t)b * (U - 1) + u], 0, V - 1) : -1;
  // the clamped indices keep the loads unconditional; their values are dropped by the selects below
  const double b_down = betas[sk + (t < Tb - 1 ? Us : 0)];         // beta(t+1,u): next diagonal, same column
  const double b_right = betas[sk + (lab >= 0 ? Us + 1 : 0)];      // beta(t,u+1)
  const float gamma = __expf((float)(a + bb - L));
  float pb = 0.f, pl = 0.f;
  if (t < Tb - 1) pb = __expf((float)(a + b_down - L + (double)lpb));
  else if (u == Ub - 1) pb = __expf((float)(a - L + (double)lpb));
  if (lab >= 0) pl = __expf((float)(a + b_right - L + (double)lpl));
  const float dn = denom[((size_t)b * T + t) * U + u];
  return make_coef(dn, gamma + lambda * pl, pb, (1.f + lambda) * pl, lpb, lpl, lab, blank, clamp, scale);
}

// The same coefficients for a wave that works on one row (every input is wave-uniform).  The ten
// values are fetched by scalar loads that are all issued before the first of them is awaited: a
// load placed under the condition that uses it would cost one memory round trip per condition.
struct CoefRaw {
  double a, bb, b_down, b_right, L;
  float lpb, lpl, dn, gs;
  long long lab;
};
__device__ __forceinline__ CoefRaw load_coef_raw_from(const float* __restrict__ denom, const float* __restrict__ arcs,
                                                      const double* __restrict__ alphas,
                                                      const double* __restrict__ betas, const double* __restrict__ ll,
                                                      const int64_t* __restrict__ labels,
                                                      const float* __restrict__ grad_scale, int grad_scale_stride,
                                                      int ND, int Us, int A, int b, int t, int u, int Tb, int Ub,
                                                      int T, int U) {
  const size_t row = (size_t)(b * ND + t + u);
  const size_t sk = row * Us + u;
  const bool has_down = t < Tb - 1, has_lab = u < Ub - 1;
  // a row without a label arc (and U == 1, where there is no label array at all) reads a dummy word
  const int64_t* lp = has_lab ? labels + ((size_t)b * (U - 1) + u) : (const int64_t*)ll;
  const float* gp = grad_scale ? grad_scale + (size_t)b * grad_scale_stride : (const float*)ll;
  CoefRaw r;
  r.a = uni(sload(alphas + sk));
  r.bb = uni(sload(betas + sk));
  r.b_down = uni(sload(betas + sk + (has_down ? Us : 0)));      // beta(t+1,u): next diagonal, same column
  r.b_right = uni(sload(betas + sk + (has_lab ? Us + 1 : 0)));  // beta(t,u+1)
  r.L = uni(sload(ll + 2 * b));
  r.lpb = uni(sload(arcs + row * A * Us + u));
  r.lpl = uni(sload(arcs + row * A * Us + Us + u));
  r.dn = uni(sload(denom + ((size_t)b * T + t) * U + u));
  r.lab = uni((long long)sload(lp));
  r.gs = uni(sload(gp));
  // every value is now on its way; the registers are claimed here, before any of them is used
  // (an asm without side effects: one that has them would turn every later load into a vector load)
  asm("" : "+s"(r.a), "+s"(r.bb), "+s"(r.b_down), "+s"(r.b_right), "+s"(r.L), "+s"(r.lpb), "+s"(r.lpl), "+s"(r.dn),
      "+s"(r.gs), "+s"(r.lab));
  return r;
}
__device__ __forceinline__ CoefRaw load_coef_raw(const LatticeView& lv, int b, int t, int u, int Tb, int Ub, int T,
                                                 int U) {
  return load_coef_raw_from(lv.denom, lv.arcs, lv.alphas, lv.betas, lv.ll, lv.labels, lv.grad_scale,
                            lv.grad_scale_stride, lv.ND, lv.Us, lv.A, b, t, u, Tb, Ub, T, U);
}
__device__ __forceinline__ RowCoef finish_coef(const CoefRaw& r, const LatticeView& lv, int t, int u, int Tb, int Ub,
                                               int V, int blank) {
  const int lab = (u < Ub - 1) ? clampi(r.lab, 0, V - 1) : -1;
  const float scale = (lv.grad_scale ? r.gs : 1.f) * lv.grad_mul;
  const float gamma = __expf((float)(r.a + r.bb - r.L));
  float pb = 0.f, pl = 0.f;
  if (t < Tb - 1) pb = __expf((float)(r.a + r.b_down - r.L + (double)r.lpb));
  else if (u == Ub - 1) pb = __expf((float)(r.a - r.L + (double)r.lpb));
  if (lab >= 0) pl = __expf((float)(r.a + r.b_right - r.L + (double)r.lpl));
  return make_coef(r.dn, gamma + lv.lambda * pl, pb, (1.f + lv.lambda) * pl, r.lpb, r.lpl, lab, blank, lv.clamp,
                   scale);
}

__global__ __launch_bounds__(1024) void rnnt_cell_kernel(
    const float* __restrict__ denom, const float* __restrict__ arcs, const double* __restrict__ alphas,
    const double* __restrict__ betas, const double* __restrict__ ll, const int64_t* __restrict__ labels,
    const int64_t* __restrict__ act_lens, const int64_t* __restrict__ label_lens, const float* __restrict__ grad_scale,
    int grad_scale_stride, float grad_mul, float* __restrict__ coef, int T, int U, int V, int blank, int ND, int Us,
    int A, int CS, float lambda, float clamp, long long cells) {
  // one workgroup per skewed row (b, n = t + u), one thread per column: the lattice reads of a wave
  // are then consecutive addresses (a thread per cell in [B,T,U] order strides by a whole row + 1)
  const int u = threadIdx.x, b = (int)(blockIdx.x / (unsigned)ND), n = (int)(blockIdx.x - (unsigned)b * (unsigned)ND);
  const int t = n - u;
  if (u >= U || t < 0 || t >= T) return;
  const long long c = ((long long)b * T + t) * U + u;
  (void)cells;
  const int Tb = clampi(act_lens[b], 1, T);
  const int Ub = clampi(label_lens[b] + 1, 1, U);
  float* out = coef + (size_t)c * CS;
  if (t >= Tb || u >= Ub) {
    out[5] = __int_as_float(-2);
    return;
  }
  const float scale = (grad_scale ? grad_scale[(size_t)b * grad_scale_stride] : 1.f) * grad_mul;
  write_coef(out, rnnt_coef(denom, arcs, alphas, betas, ll, labels, scale, b, t, u, Tb, Ub, T, U, V, blank, ND, Us, A,
                            lambda, clamp));
}

// ----------------------------------------------------------------------------------------
// Compact log-prob op (parts/k2/rnnt_logprobs_triton.py:20-228): target and blank log-probs of every
// lattice cell as plain [B,T,U] float32 arrays, and the gradient of the logits given the gradients of
// those two arrays.  The forward is the denominator pass plus this read-out of its arc planes; the
// backward turns the two upstream gradients into the per-cell coefficient records of the streaming
// gradient pass:  g_v = -p_v * (gb + gt) + [v = blank] gb + [v = target] gt  (:118-122; with
// target == blank the target term alone is added, as there).  One workgroup per skewed row, one
// thread per column.
// ----------------------------------------------------------------------------------------
__global__ __launch_bounds__(1024) void logprobs_export_kernel(const float* __restrict__ arcs,
                                                              const int64_t* __restrict__ act_lens,
                                                              const int64_t* __restrict__ label_lens,
                                                              float* __restrict__ target_scores,
                                                              float* __restrict__ blank_scores, int T, int U, int ND,
                                                              int Us, int A) {
  const int u = threadIdx.x, b = (int)(blockIdx.x / (unsigned)ND), n = (int)(blockIdx.x - (unsigned)b * (unsigned)ND);
  const int t = n - u;
  if (u >= U || t < 0 || t >= T) return;
  const size_t c = ((size_t)b * T + t) * U + u;
  const int Tb = clampi(act_lens[b], 1, T);
  const int Ub = clampi(label_lens[b] + 1, 1, U);
  const bool valid = t < Tb && u < Ub;
  const size_t base = (size_t)(b * ND + n) * A * Us + u;
  const float lpb = arcs[base], lpl = arcs[base + Us];
  blank_scores[c] = valid ? lpb : 0.f;                  // cells outside the utterance stay 0 (:148-149)
  target_scores[c] = (valid && u < Ub - 1) ? lpl : 0.f;  // and so does the column without a target
}

__global__ __launch_bounds__(1024) void logprobs_cell_kernel(
    const float* __restrict__ denom, const float* __restrict__ arcs, const int64_t* __restrict__ labels,
    const int64_t* __restrict__ act_lens, const int64_t* __restrict__ label_lens,
    const float* __restrict__ grad_target_scores, const float* __restrict__ grad_blank_scores,
    float* __restrict__ coef, int T, int U, int V, int blank, int ND, int Us, int A, int CS) {
  const int u = threadIdx.x, b = (int)(blockIdx.x / (unsigned)ND), n = (int)(blockIdx.x - (unsigned)b * (unsigned)ND);
  const int t = n - u;
  if (u >= U || t < 0 || t >= T) return;
  const size_t c = ((size_t)b * T + t) * U + u;
  const int Tb = clampi(act_lens[b], 1, T);
  const int Ub = clampi(label_lens[b] + 1, 1, U);
  float* out = coef + c * CS;
  if (t >= Tb || u >= Ub) {
    out[5] = __int_as_float(-2);
    return;
  }
  const size_t base = (size_t)(b * ND + n) * A * Us + u;
  const bool has_target = u < Ub - 1;
  const int lab = has_target ? clampi(labels[(size_t)b * (U - 1) + u], 0, V - 1) : -1;
  const float gb = grad_blank_scores[c];
  const float gt = has_target ? grad_target_scores[c] : 0.f;
  const float sum = gb + gt;
  RowCoef rc;
  rc.dl2 = denom[c] * kLog2e;
  rc.W = -sum;
  rc.cb = INFINITY;
  rc.gB = gb - __expf(arcs[base]) * sum;
  rc.gL = has_target ? gt - __expf(arcs[base + Us]) * sum : 0.f;
  if (lab == blank) rc.gB = rc.gL;
  rc.lab = lab;
  write_coef(out, rc);
}

__global__ __launch_bounds__(1024) void tdt_cell_kernel(
    const float* __restrict__ denom, const float* __restrict__ arcs, const double* __restrict__ alphas,
    const double* __restrict__ betas, const double* __restrict__ ll, const int64_t* __restrict__ labels,
    const int64_t* __restrict__ act_lens, const int64_t* __restrict__ label_lens, const float* __restrict__ grad_scale,
    int grad_scale_stride, float grad_mul, float* __restrict__ coef, int T, int U, int V, int blank, int ND, int Us,
    int A, int CS, float lambda, float clamp, long long cells, TdtParams prm) {
  // one workgroup per skewed row (b, n = t + u), one thread per column: the lattice reads of a wave
  // are then consecutive addresses (a thread per cell in [B,T,U] order strides by a whole row + 1)
  const int u = threadIdx.x, b = (int)(blockIdx.x / (unsigned)ND), n = (int)(blockIdx.x - (unsigned)b * (unsigned)ND);
  const int t = n - u;
  if (u >= U || t < 0 || t >= T) return;
  const long long c = ((long long)b * T + t) * U + u;
  (void)cells;
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
  const float scale = (grad_scale ? grad_scale[(size_t)b * grad_scale_stride] : 1.f) * grad_mul;
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
  write_coef(out, make_coef(denom[c], gamma + lambda * pl, pb, (1.f + lambda) * pl, lpb, lpl, lab, blank, clamp, scale));
}

// ----------------------------------------------------------------------------------------
// Multi-blank transducer (arXiv:2211.03541; gpu_rnnt_kernel.py:410-724).  The softmax covers the
// tokens, NB big blanks (big blank i: index blank-1-i, duration dur[i]) and the standard blank
// (duration 1); every arc pays -sigma.  Same organisation as the TDT workgroup kernel: one
// workgroup per (utterance, direction), one thread per column, one barrier per anti-diagonal.
//   alpha: a finished cell leaves alpha + arc - sigma for each of its outgoing arcs in an LDS
//          ring of max_duration + 1 diagonals (plane 0: label arc, read by column u+1 one step
//          later; plane 1+j: blank arc j, read by the same column dur_j steps later).
//   beta : the ring holds beta of the last max_duration + 1 diagonals.
// Cells outside the lattice hold "log 0" or junk that no valid cell reads, as in the RNNT kernel.
// NBC is the compiled capacity for big blanks; prm.NB <= NBC are in use.
// ----------------------------------------------------------------------------------------
// Workgroup barrier that waits for this wave's LDS traffic only.  __syncthreads() also drains the
// vector-memory counters: at every step of a recursion it would wait for the lattice store to be
// acknowledged and for the prefetched arc rows to arrive.
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0); vmcnt and expcnt left alone
  __builtin_amdgcn_s_barrier();
}

struct MbParams {
  int NB;
  int dur[MI_TRANSDUCER_MAX_BIG_BLANKS];
  int R;  // ring depth: longest blank + 1
  float sigma;
};

// MAXT: the largest workgroup the instantiation is launched with (256 leaves the compiler the whole
// register file; the 1024-thread variant for U > 256 has to make do with 128 registers per thread)
template <int NBC, int MAXT>
__global__ __launch_bounds__(MAXT) void multiblank_lattice_kernel(
    const float* __restrict__ arcs, double* __restrict__ alphas, double* __restrict__ betas, double* __restrict__ ll,
    float* __restrict__ costs, const int64_t* __restrict__ act_lens, const int64_t* __restrict__ label_lens, int T,
    int U, int ND, int Us, int A, float cost_scale, int with_betas, MbParams prm) {
  constexpr int P = 4;
  constexpr int NJ = NBC + 1;  // blank arcs: the standard one, then the big ones
  extern __shared__ double ring[];
  const int b = with_betas ? (int)(blockIdx.x >> 1) : (int)blockIdx.x;
  const int dir = with_betas ? (int)(blockIdx.x & 1) : 0;
  const int u = threadIdx.x;  // blockDim.x == Us
  const int Tb = clampi(act_lens[b], 1, T);
  const int Ub = clampi(label_lens[b] + 1, 1, U);
  const int nd = Tb + Ub - 1;
  const int R = prm.R, NB = prm.NB;
  const double sigma = (double)prm.sigma;
  const double NINF = kLogZero;
  int dur[NJ];
  dur[0] = 1;
#pragma unroll
  for (int j = 1; j < NJ; ++j) dur[j] = j - 1 < NB ? prm.dur[j - 1] : (1 << 28);  // unused slots never fire
  // The step holds no test of NB (a wave-uniform test becomes a taken branch, and a lone wave per SIMD
  // pays for every one of them): unused slots read an existing arc plane and their scores are pushed
  // down to log 0 by this penalty.
  double unused[NJ];
  int plane[NJ];
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    unused[j] = j - 1 < NB ? 0.0 : kLogZero;
    plane[j] = j == 0 ? 0 : (j - 1 < NB ? 1 + j : 0);
  }
  const size_t row_pitch = (size_t)A * Us;
  const float* arcs_b = arcs + (size_t)b * ND * row_pitch + u;

  // arc log-probs of P diagonals for this column: [0] standard blank, [1] label, [2+i] big blank i
  auto load_rows = [&](int nfirst, int step, float(&W)[P][2 + NBC]) {
#pragma unroll
    for (int p = 0; p < P; ++p) {
      int n = nfirst + step * p;
      n = n < 0 ? 0 : (n >= nd ? nd - 1 : n);
      const float* rp = arcs_b + (size_t)n * row_pitch;
      W[p][0] = finite_arc(rp[0]);
      W[p][1] = finite_arc(rp[Us]);
#pragma unroll
      for (int i = 0; i < NBC; ++i) W[p][2 + i] = finite_arc(rp[(size_t)plane[1 + i] * Us]);
    }
  };
  // log-sum-exp of x[0..N); "log 0" entries vanish, all "log 0" stays "log 0"
  auto lse_all = [&](const double* x) {
    constexpr int N = 1 + NJ;
    double m = x[0];
#pragma unroll
    for (int i = 1; i < N; ++i) m = fmax(m, x[i]);
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < N; ++i) s += fast_exp2((float)(x[i] - m) * kLog2e);
    return m + (double)(__builtin_amdgcn_logf(s) * 0.6931471805599453f);
  };

  if (dir == 0) {
    const int slot_stride = (1 + NJ) * Us, ring_len = R * slot_stride;
    for (int i = u; i < ring_len; i += Us) ring[i] = NINF;
    __syncthreads();
    double* out = alphas + (size_t)b * ND * Us + u;
    // ring offsets of the diagonals n-1 (label arc, standard blank) and n-dur_j (big blanks)
    int off_in[NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j) off_in[j] = j - 1 < NB ? ((R - dur[j] % R) % R) * slot_stride : 0;
    int cur_off = 0;
    const int um1 = u > 0 ? u - 1 : 0;
    auto step_fn = [&](int n, const float* w) {
      double x[1 + NJ];
      x[0] = u > 0 ? ring[off_in[0] + um1] : NINF;  // label arc out of (t, u-1)
#pragma unroll
      for (int j = 0; j < NJ; ++j) x[1 + j] = ring[off_in[j] + (1 + j) * Us + u];  // blank arc j out of (t-dur_j, u)
      double a = lse_all(x);
      if (n == 0 && u == 0) a = 0.0;
      out[(size_t)n * Us] = a;
      double* slot = ring + cur_off + u;
      slot[0] = (a + (double)w[1]) - sigma;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const double ob = (a + (double)w[j == 0 ? 0 : 1 + j]) - sigma;
        slot[(1 + j) * Us] = ob + unused[j];
      }
#pragma unroll
      for (int j = 0; j < NJ; ++j) off_in[j] = off_in[j] + slot_stride == ring_len ? 0 : off_in[j] + slot_stride;
      cur_off = cur_off + slot_stride == ring_len ? 0 : cur_off + slot_stride;
      lds_barrier();
    };
    float wa[P][2 + NBC], wb[P][2 + NBC];
    int n0 = 0;
    load_rows(0, 1, wa);
    for (; n0 + 2 * P <= nd; n0 += 2 * P) {
      load_rows(n0 + P, 1, wb);
#pragma unroll
      for (int p = 0; p < P; ++p) step_fn(n0 + p, wa[p]);
      load_rows(n0 + 2 * P, 1, wa);
#pragma unroll
      for (int p = 0; p < P; ++p) step_fn(n0 + P + p, wb[p]);
    }
    for (; n0 < nd; ++n0) {
      float w[P][2 + NBC];
      load_rows(n0, 0, w);
      step_fn(n0, w[0]);
    }
    if (u == Ub - 1) {
      // the blank arcs that end the utterance leave from cells (Tb - dur_j, Ub-1) of this thread's own column
      // (gpu_rnnt_kernel.py:548-568): their alphas are re-read (this thread stored them) and the arc scores
      // formed as in the loop -- the standard blank first, then the big blanks in their order
      double acc = NINF;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int t0 = Tb - dur[j];
        if (t0 >= 0) {  // (unused slots have a duration beyond any utterance)
          const float* rp = arcs_b + (size_t)(t0 + u) * row_pitch;
          const double a = out[(size_t)(t0 + u) * Us];
          const double ob = (a + (double)finite_arc(rp[(size_t)plane[j] * Us])) - sigma;
          acc = j == 0 ? ob : lse_h(acc, ob);
        }
      }
      ll[2 * b] = acc;
      costs[b] = -(float)acc * cost_scale;
    }
  } else {
    const int ring_len = R * Us;
    for (int i = u; i < ring_len; i += Us) ring[i] = NINF;
    __syncthreads();
    // a big blank that ends the utterance from column Ub-1 (t + dur == Tb, gpu_rnnt_kernel.py:660-670; the standard
    // blank does so through the corner cell) is an arc into a virtual cell beta(Tb, Ub-1) = 0 on diagonal nd: with
    // that cell in the ring it needs no case of its own
    if (u == 0) ring[(nd % R) * Us + Ub - 1] = 0.0;
    __syncthreads();
    double* out = betas + (size_t)b * ND * Us + u;
    double last = NINF;
    // blank arc j leaves this cell while t + dur_j < Tb (<= Tb for a big blank in the last column), the label arc
    // while t < Tb: diagonals n < nmax, one compare against the (wave-uniform) diagonal number per arc
    int nmax[NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j) nmax[j] = Tb + u - dur[j] + ((j > 0 && u == Ub - 1) ? 1 : 0);
    const int nmax_label = u < Ub - 1 ? Tb + u : -(1 << 29);
    // ring offsets of the diagonals n+dur_j; the label arc reads diagonal n+1 like the standard blank
    int off_in[NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j) off_in[j] = j - 1 < NB ? (((nd - 1) % R + dur[j] % R) % R) * Us : 0;
    int cur_off = ((nd - 1) % R) * Us;
    const int up1 = u + 1 < Us ? u + 1 : u;
    auto step_fn = [&](int n, const float* w) {
      const int t = n - u;
      double x[1 + NJ];
      x[0] = n < nmax_label ? (ring[off_in[0] + up1] + (double)w[1]) - sigma : NINF;  // label arc to (t, u+1)
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const double arc = (double)w[j == 0 ? 0 : 1 + j] - sigma;
        const double via = ring[off_in[j] + u] + arc;
        x[1 + j] = n < nmax[j] ? via : NINF;  // selects, not branches
      }
      double v = lse_all(x);
      if (t == Tb - 1 && u == Ub - 1) v = (double)w[0] - sigma;  // the corner: one standard blank
      out[(size_t)n * Us] = v;
      ring[cur_off + u] = v;
      last = v;
#pragma unroll
      for (int j = 0; j < NJ; ++j) off_in[j] = off_in[j] == 0 ? ring_len - Us : off_in[j] - Us;
      cur_off = cur_off == 0 ? ring_len - Us : cur_off - Us;
      lds_barrier();
    };
    float wa[P][2 + NBC], wb[P][2 + NBC];
    int n0 = nd - 1;
    load_rows(n0, -1, wa);
    for (; n0 - 2 * P + 1 >= 0; n0 -= 2 * P) {
      load_rows(n0 - P, -1, wb);
#pragma unroll
      for (int p = 0; p < P; ++p) step_fn(n0 - p, wa[p]);
      load_rows(n0 - 2 * P, -1, wa);
#pragma unroll
      for (int p = 0; p < P; ++p) step_fn(n0 - P - p, wb[p]);
    }
    for (; n0 >= 0; --n0) {
      float w[P][2 + NBC];
      load_rows(n0, 0, w);
      step_fn(n0, w[0]);
    }
    if (u == 0) ll[2 * b + 1] = last;  // beta(0,0)
  }
}

// Multi-blank lattice for shapes whose ring of arc scores does not fit LDS (a long label axis with long or many big
// blanks): the same recursion, one thread per column and one barrier per anti-diagonal, but every value is pulled
// from the alphas / betas this workgroup has already stored in global memory, read back from L2 with device-scope
// loads.  A step costs an L2 round trip instead of an LDS one -- the price of having a path at all for these shapes.
// The arithmetic (arc score = (alpha + arc) - sigma, one log-sum-exp over label arc, standard blank, big blanks in
// their order) is that of multiblank_lattice_kernel, so the two give the same values.
__global__ __launch_bounds__(1024) void multiblank_lattice_pull_kernel(
    const float* __restrict__ arcs, double* alphas, double* betas, double* __restrict__ ll, float* __restrict__ costs,
    const int64_t* __restrict__ act_lens, const int64_t* __restrict__ label_lens, int T, int U, int ND, int Us, int A,
    float cost_scale, int with_betas, MbParams prm) {
  const int b = with_betas ? (int)(blockIdx.x >> 1) : (int)blockIdx.x;
  const int dir = with_betas ? (int)(blockIdx.x & 1) : 0;
  const int u = threadIdx.x;  // blockDim.x == Us
  const int Tb = clampi(act_lens[b], 1, T);
  const int Ub = clampi(label_lens[b] + 1, 1, U);
  const int nd = Tb + Ub - 1;
  const int NB = prm.NB;
  const double sigma = (double)prm.sigma;
  const double NINF = kLogZero;
  const size_t row_pitch = (size_t)A * Us;
  const float* arcs_b = arcs + (size_t)b * ND * row_pitch;
  auto arc = [&](int n, int plane, int col) { return (double)finite_arc(arcs_b[(size_t)n * row_pitch + (size_t)plane * Us + col]); };
  auto ld = [&](const double* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); };
  auto st = [&](double* p, double v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); };
  // log-sum-exp of x[0..n) in index order; "log 0" entries vanish
  auto lse_n = [&](const double* x, int n) {
    double m = x[0];
    for (int i = 1; i < n; ++i) m = fmax(m, x[i]);
    float s = 0.f;
    for (int i = 0; i < n; ++i) s += fast_exp2((float)(x[i] - m) * kLog2e);
    return m + (double)(__builtin_amdgcn_logf(s) * 0.6931471805599453f);
  };
  double x[2 + MI_TRANSDUCER_MAX_BIG_BLANKS];
  if (dir == 0) {
    double* out = alphas + (size_t)b * ND * Us;
    for (int n = 0; n < nd; ++n) {
      const int t = n - u;
      if (t >= 0 && t < Tb && u < Ub) {
        x[0] = u > 0 ? (ld(out + (size_t)(n - 1) * Us + u - 1) + arc(n - 1, 1, u - 1)) - sigma : NINF;
        x[1] = t >= 1 ? (ld(out + (size_t)(n - 1) * Us + u) + arc(n - 1, 0, u)) - sigma : NINF;
        for (int i = 0; i < NB; ++i) {
          const int d = prm.dur[i];
          x[2 + i] = t >= d ? (ld(out + (size_t)(n - d) * Us + u) + arc(n - d, 2 + i, u)) - sigma : NINF;
        }
        double a = lse_n(x, 2 + NB);
        if (n == 0) a = 0.0;  // (t, u) = (0, 0)
        st(out + (size_t)n * Us + u, a);
      }
      __syncthreads();
    }
    if (u == Ub - 1) {
      // the blank arcs that end the utterance (gpu_rnnt_kernel.py:548-568): the standard blank, then the big blanks
      double acc = (ld(out + (size_t)(Tb - 1 + u) * Us + u) + arc(Tb - 1 + u, 0, u)) - sigma;
      for (int i = 0; i < NB; ++i) {
        const int t0 = Tb - prm.dur[i];
        if (t0 >= 0) acc = lse_h(acc, (ld(out + (size_t)(t0 + u) * Us + u) + arc(t0 + u, 2 + i, u)) - sigma);
      }
      ll[2 * b] = acc;
      costs[b] = -(float)acc * cost_scale;
    }
  } else {
    double* out = betas + (size_t)b * ND * Us;
    for (int n = nd - 1; n >= 0; --n) {
      const int t = n - u;
      if (t >= 0 && t < Tb && u < Ub) {
        double v;
        if (t == Tb - 1 && u == Ub - 1) {
          v = arc(n, 0, u) - sigma;  // the corner: one standard blank
        } else {
          x[0] = u < Ub - 1 ? (ld(out + (size_t)(n + 1) * Us + u + 1) + arc(n, 1, u)) - sigma : NINF;
          x[1] = t + 1 < Tb ? ld(out + (size_t)(n + 1) * Us + u) + (arc(n, 0, u) - sigma) : NINF;
          for (int i = 0; i < NB; ++i) {
            const int d = prm.dur[i];
            const double a = arc(n, 2 + i, u) - sigma;
            // a big blank may end the utterance from the last column (gpu_rnnt_kernel.py:660-670)
            x[2 + i] = t + d < Tb ? ld(out + (size_t)(n + d) * Us + u) + a : ((t + d == Tb && u == Ub - 1) ? 0.0 + a : NINF);
          }
          v = lse_n(x, 2 + NB);
        }
        st(out + (size_t)n * Us + u, v);
      }
      __syncthreads();
    }
    if (u == 0) ll[2 * b + 1] = ld(out);  // beta(0,0)
  }
}

// Per-cell coefficients of the multi-blank gradient (gpu_rnnt_kernel.py:727-885): the record of the
// RNNT/TDT cell kernels, plus in out[kCoefBase + i] the FINISHED gradient entry of big blank i
// (clamped and scaled), which multiblank_fixup_kernel stores over what the gradient pass put there.
__global__ __launch_bounds__(1024) void multiblank_cell_kernel(
    const float* __restrict__ denom, const float* __restrict__ arcs,
    const double* __restrict__ alphas, const double* __restrict__ betas, const double* __restrict__ ll,
    const int64_t* __restrict__ labels, const int64_t* __restrict__ act_lens, const int64_t* __restrict__ label_lens,
    const float* __restrict__ grad_scale, int grad_scale_stride, float grad_mul, float* __restrict__ coef, int T, int U,
    int V, int blank, int ND, int Us, int A, int CS, float lambda, float clamp, long long cells, MbParams prm) {
  // one workgroup per skewed row (b, n = t + u), one thread per column: the lattice reads of a wave
  // are then consecutive addresses (a thread per cell in [B,T,U] order strides by a whole row + 1)
  const int u = threadIdx.x, b = (int)(blockIdx.x / (unsigned)ND), n = (int)(blockIdx.x - (unsigned)b * (unsigned)ND);
  const int t = n - u;
  if (u >= U || t < 0 || t >= T) return;
  const long long c = ((long long)b * T + t) * U + u;
  (void)cells;
  const int Tb = clampi(act_lens[b], 1, T);
  const int Ub = clampi(label_lens[b] + 1, 1, U);
  float* out = coef + (size_t)c * CS;
  if (t >= Tb || u >= Ub) {
    out[5] = __int_as_float(-2);
    return;
  }
  const double sigma = (double)prm.sigma;
  const size_t row = (size_t)(b * ND + t + u);
  const size_t sk = row * Us + u;
  const double a = alphas[sk], bb = betas[sk], L = ll[2 * b];
  const float* rp = arcs + row * A * Us + u;
  const float lpb = rp[0], lpl = rp[Us];
  const int lab = (u < Ub - 1) ? clampi(labels[(size_t)b * (U - 1) + u], 0, V - 1) : -1;
  const float scale = (grad_scale ? grad_scale[(size_t)b * grad_scale_stride] : 1.f) * grad_mul;
  const float gamma = expf((float)(a + bb - L));
  float pb = 0.f, pl = 0.f;
  if (t < Tb - 1) pb = expf((float)(a + betas[sk + Us] + (double)lpb - sigma - L));
  else if (u == Ub - 1) pb = expf((float)(a + (double)lpb - sigma - L));
  if (lab >= 0) pl = expf((float)(a + betas[sk + Us + 1] + (double)lpl - sigma - L));
  const float W = gamma + lambda * pl, PL = (1.f + lambda) * pl;
#pragma unroll 1
  for (int i = 0; i < prm.NB; ++i) {
    const int d = prm.dur[i];
    const float lpi = rp[(size_t)(2 + i) * Us];
    float pi = 0.f;
    if (t + d < Tb) pi = expf((float)(a + betas[sk + (size_t)d * Us] + (double)lpi - sigma - L));
    else if (t + d == Tb && u == Ub - 1) pi = expf((float)(a + (double)lpi - sigma - L));
    float g = expf(lpi) * W - pi;
    if (lab == blank - 1 - i) g -= PL;
    if (clamp > 0.f) g = clamp_sym(g, clamp);
    out[kCoefBase + i] = g * scale;
  }
  write_coef(out, make_coef(denom[c], W, pb, PL, lpb, lpl, lab, blank, clamp, scale));
}

// stores the finished big-blank entries of every valid cell (after the gradient pass)
template <int DT>
__global__ __launch_bounds__(256) void multiblank_fixup_kernel(void* __restrict__ grads, const float* __restrict__ coef,
                                                               int V, int blank, int NB, int CS, long long cells) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long c = i / NB;
  if (c >= cells) return;
  const int k = (int)(i - c * NB);
  const float* rec = coef + (size_t)c * CS;
  if (__float_as_int(rec[5]) == -2) return;  // padded cell
  Elem<DT>::store1(grads, (size_t)c * V + (blank - 1 - k), rec[kCoefBase + k]);
}


// ----------------------------------------------------------------------------------------
// Pass 2: the gradient stream.  Grid (ceil(U/4), T, B), one wave per row; reads the V token
// logits of valid rows, writes V + D gradient elements of every row.  Same kernel for RNNT
// (D = 0) and TDT.  flags: kFlagZeroDurations, kFlagPaddingDone.
// ----------------------------------------------------------------------------------------
template <int DT>
__global__ __launch_bounds__(256) void grad_stream_kernel(const void* __restrict__ acts, void* __restrict__ grads,
                                                          const float* __restrict__ coef,
                                                          const int64_t* __restrict__ act_lens,
                                                          const int64_t* __restrict__ label_lens, int T, int U, int V,
                                                          int D, int blank, int CS, int flags, int BT,
                                                          int bt_chunk) {
  constexpr int VEC = Elem<DT>::VEC;
  constexpr int R = 4;
  constexpr bool NT = MI_NT_K4 != 0;
  const int lane = threadIdx.x & 63;
  const RowId id = row_of_wave(T, U, BT, bt_chunk);
  if (!id.in_range) return;
  const int b = id.b, t = id.t, u = id.u;
  const int Tb = clampi(act_lens[b], 1, T);
  const int Ub = clampi(label_lens[b] + 1, 1, U);
  const int VD = V + D;
  const size_t r = ((size_t)b * T + t) * U + u;
  const size_t e0 = r * VD;

  const RowWindow<DT> win(acts, e0);
  const uintptr_t g0 = (uintptr_t)grads + e0 * Elem<DT>::BYTES;
  uint4* gvp = (uint4*)(g0 & ~(uintptr_t)15);
  // acts and grads have the same shape and dtype; their bases may still differ in alignment
  const bool same_phase = (int)((g0 & 15) / Elem<DT>::BYTES) == win.mis;

  if (t >= Tb || u >= Ub) {  // padded cell: zeros over all V + D entries
    if (flags & kFlagPaddingDone) return;
    const RowSplit<DT> sp(win.mis, VD);
    const uint4 z = make_uint4(0, 0, 0, 0);
    if (same_phase) {
      for (int i = lane; i < sp.nb; i += 64) gvp[sp.jb0 + i] = z;
      if (lane < sp.hc) Elem<DT>::store1(grads, e0 + lane, 0.f);
      else if (lane >= VEC && lane < VEC + sp.tc) Elem<DT>::store1(grads, e0 + sp.tail0() + lane - VEC, 0.f);
    } else {
      for (int v = lane; v < VD; v += 64) Elem<DT>::store1(grads, e0 + v, 0.f);
    }
    return;
  }

  const float* c = coef + r * CS;
  const float4 c0 = *(const float4*)c;          // denom*log2e, W*scale, clamp bound, G_blank
  const float2 c1 = *(const float2*)(c + 4);    // G_label, label id
  const float dl2 = c0.x, W = c0.y, cb = c0.z, gB = c0.w, gL = c1.x;
  const int lab = __float_as_int(c1.y);
  const bool clamp_on = cb < INFINITY;
  const RowSplit<DT> sp(win.mis, V);

  auto token_grad = [&](float x, int v) {
    float g = fast_exp2(fmaf(x, kLog2e, dl2)) * W;
    if (clamp_on) g = clamp_sym(g, cb);
    if (v == blank) g = gB;
    if (v == lab) g = gL;
    return g;
  };

  // head, tail and duration entries: one element per lane
  {
    int v = -1;
    if (lane < sp.hc) v = lane;
    else if (lane >= VEC && lane < VEC + sp.tc) v = sp.tail0() + lane - VEC;
    else if (lane >= 2 * VEC && lane < 2 * VEC + D) v = V + lane - 2 * VEC;
    if (v >= 0) {
      float g;
      if (v < V) g = token_grad(Elem<DT>::load1(acts, e0 + v), v);
      else g = (flags & kFlagZeroDurations) ? 0.f : c[kCoefBase + v - V];
      Elem<DT>::store1(grads, e0 + v, g);
    }
  }

  if (!same_phase) {  // never the case for two fresh torch tensors; correct but slow
    for (int v = sp.hc + lane; v < sp.tail0(); v += 64)
      Elem<DT>::store1(grads, e0 + v, token_grad(Elem<DT>::load1(acts, e0 + v), v));
    return;
  }

  // whole vectors; the two special logits are patched in the one vector that holds them
  const int jblank = (blank + win.mis) / VEC, jlab = lab >= 0 ? (lab + win.mis) / VEC : -1;
  auto do_vector = [&](const uint4& raw, int j) {
    float x[VEC], g[VEC];
    Elem<DT>::unpack(raw, x);
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      float gi = fast_exp2(fmaf(x[i], kLog2e, dl2)) * W;
      if (clamp_on) gi = clamp_sym(gi, cb);
      g[i] = gi;
    }
    if (j == jblank || j == jlab) {
      const int first = j * VEC - win.mis;
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        if (first + i == blank) g[i] = gB;
        if (first + i == lab) g[i] = gL;
      }
    }
    gvp[j] = Elem<DT>::pack(g);
  };

  int j = sp.jb0 + lane;
  int rounds = sp.nb >> 6;
  for (; rounds >= R; rounds -= R, j += 64 * R) {
    uint4 raw[R];
#pragma unroll
    for (int k = 0; k < R; ++k) raw[k] = load_stream<NT>(win.vp + j + 64 * k);
#pragma unroll
    for (int k = 0; k < R; ++k) do_vector(raw[k], j + 64 * k);
  }
  for (; rounds > 0; --rounds, j += 64) do_vector(load_stream<NT>(win.vp + j), j);
  if (lane < (sp.nb & 63)) do_vector(load_stream<NT>(win.vp + j), j);
}

// ----------------------------------------------------------------------------------------
// Wave reductions through DPP (no LDS round trips): two quad permutes and two mirrors leave
// every 16-lane row holding its own result in all lanes; the four row results are then read
// into scalar registers and combined, so the value returned is wave-uniform.
// ----------------------------------------------------------------------------------------
template <int CTRL> __device__ __forceinline__ float dpp_f(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float lane_value(float v, int lane) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}
__device__ __forceinline__ float wave_max_u(float v) {
  v = fmaxf(v, dpp_f<0xB1>(v));   // quad_perm [1,0,3,2]
  v = fmaxf(v, dpp_f<0x4E>(v));   // quad_perm [2,3,0,1]
  v = fmaxf(v, dpp_f<0x141>(v));  // row_half_mirror
  v = fmaxf(v, dpp_f<0x140>(v));  // row_mirror
  return fmaxf(fmaxf(lane_value(v, 0), lane_value(v, 16)), fmaxf(lane_value(v, 32), lane_value(v, 48)));
}
__device__ __forceinline__ float wave_sum_u(float v) {
  v += dpp_f<0xB1>(v);
  v += dpp_f<0x4E>(v);
  v += dpp_f<0x141>(v);
  v += dpp_f<0x140>(v);
  return (lane_value(v, 0) + lane_value(v, 16)) + (lane_value(v, 32) + lane_value(v, 48));
}

// ----------------------------------------------------------------------------------------
// The bandwidth passes for rows that fit in R vectors per lane (V <= 64*R*VEC, the usual
// subword vocabularies).  A workgroup owns kChunkRows consecutive rows of one (b,t) -- one
// contiguous piece of memory -- and each of its 4 waves walks rows wave, wave+4, ...; while a
// row is being reduced the loads of the wave's next row are already in flight.
// ----------------------------------------------------------------------------------------
#ifndef MI_ROWS_PER_WAVE
#define MI_ROWS_PER_WAVE 1
#endif
constexpr int kRowsPerWave = MI_ROWS_PER_WAVE;
#ifndef MI_ROW_WAVES
#define MI_ROW_WAVES 4
#endif
constexpr int kRowWaves = MI_ROW_WAVES;  // waves (= rows in flight) per workgroup of the row kernels
constexpr int kRowThreads = 64 * kRowWaves;
constexpr int kChunkRows = kRowWaves * kRowsPerWave;

// zero-fills elements [e_begin, e_end) of `base` with the whole workgroup: 16-byte stores on
// the aligned middle, element stores on the ragged ends
template <int DT> __device__ __forceinline__ void zero_elems(void* base, size_t e_begin, size_t e_end) {
  constexpr int BYTES = Elem<DT>::BYTES;
  if (e_begin >= e_end) return;
  char* p0 = (char*)base + e_begin * BYTES;
  char* p1 = (char*)base + e_end * BYTES;
  const size_t len = (size_t)(p1 - p0);
  size_t head = (16 - ((uintptr_t)p0 & 15)) & 15;
  if (head > len) head = len;
  const size_t tail = (len - head) & 15;
  const size_t nvec = (len - head - tail) >> 4;
  const int tid = threadIdx.x;
  if (tid < (int)(head / BYTES)) Elem<DT>::store1(p0, tid, 0.f);
  else if (tid >= 32 && tid - 32 < (int)(tail / BYTES)) Elem<DT>::store1(p1 - tail, tid - 32, 0.f);
  uint4* q = (uint4*)(p0 + head);
  const uint4 z = make_uint4(0, 0, 0, 0);
  for (size_t i = tid; i < nvec; i += kRowThreads) store_stream(q + i, z);
}

template <int DT, int R>
__global__ __launch_bounds__(kRowThreads) void denom_rows_kernel(
    const void* __restrict__ acts, const int64_t* __restrict__ labels, const int64_t* __restrict__ act_lens,
    const int64_t* __restrict__ label_lens, float* __restrict__ denom, float* __restrict__ arcs, int T, int U, int V,
    int D, int nbig, int blank, int ND, int Us, int A, int nchunks, int nblocks, GridDiv gdiv) {
  constexpr int VEC = Elem<DT>::VEC;
  // all kernel arguments are fetched in one go, not one batch per use (the loads this kernel wants
  // on the scalar unit are written as such, so the asm's side effect costs nothing)
  asm volatile("" ::"s"((uintptr_t)acts), "s"((uintptr_t)labels), "s"((uintptr_t)act_lens), "s"((uintptr_t)label_lens),
               "s"((uintptr_t)denom), "s"((uintptr_t)arcs), "s"(T), "s"(U), "s"(V), "s"(D), "s"(nbig), "s"(blank), "s"(ND), "s"(Us),
               "s"(A), "s"(nchunks), "s"(nblocks), "s"(gdiv.chunks.mul), "s"(gdiv.chunks.shift), "s"(gdiv.T.mul),
               "s"(gdiv.T.shift));
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  // 1-D grid over (b,t,chunk), chunk fastest = memory order
  unsigned wg = logical_block();
  if (wg >= (unsigned)nblocks) return;
#if MI_K1_REVERSE
  wg = (unsigned)nblocks - 1u - wg;
#endif
  const unsigned bt = fast_div(wg, gdiv.chunks), chunk = wg - bt * (unsigned)nchunks;
  const int b = (int)fast_div(bt, gdiv.T), t = (int)(bt - (unsigned)b * (unsigned)T);
  const int u_begin = (int)chunk * kChunkRows + wave;
  // the wave's label ids travel with the lengths (a clamped index, dropped below if the row has no
  // label arc; with U == 1 there is no label array and a length is read instead)
  long long lab_raw[kRowsPerWave];
#pragma unroll
  for (int i = 0; i < kRowsPerWave; ++i) {
    const int uu = min(u_begin + kRowWaves * i, U - 2);
    lab_raw[i] = uni((long long)sload(U > 1 ? labels + ((size_t)b * (U - 1) + max(uu, 0)) : act_lens + b));
  }
  const UttLens len = load_lens(act_lens, label_lens, b, T, U);
#pragma unroll
  for (int i = 0; i < kRowsPerWave; ++i) asm("" : "+s"(lab_raw[i]));
  const int Tb = len.Tb, Ub = len.Ub;
  if (t >= Tb) return;
  const int u_end = min(Ub, (int)(chunk + 1) * kChunkRows);
  if (u_begin >= u_end) return;
  const int VD = V + D;
  const unsigned cell0 = ((unsigned)b * (unsigned)T + (unsigned)t) * (unsigned)U;  // B*T*U < 2^31 (host check)

  // the wave's label ids, fetched once so that no row waits on an id before asking for its logit
  int labs[kRowsPerWave];
#pragma unroll
  for (int i = 0; i < kRowsPerWave; ++i) {
    const int uu = u_begin + kRowWaves * i;
    labs[i] = (uu < Ub - 1) ? clampi(lab_raw[i], 0, V - 1) : -1;
  }

  struct Row {
    uint4 raw[R];
    float xe, xb, xl, xd;
    int mis;
  };
  auto fetch = [&](int uu, int lab, Row& d) {
    const size_t e0 = (size_t)(cell0 + (unsigned)uu) * (unsigned)VD;
    const RowWindow<DT> w(acts, e0);
    const RowSplit<DT> sp(w.mis, V);
    d.mis = w.mis;
    // every load is unconditional (out-of-range lanes re-read an in-row address and are masked
    // later): loads under a branch would force the wait counters to drain at every join
#pragma unroll
    for (int k = 0; k < R; ++k) d.raw[k] = load_stream<MI_NT_K1 != 0>(w.vp + sp.body_vector(lane + 64 * k));
    const int ve = sp.extra_token(lane);
    d.xe = Elem<DT>::load1(acts, e0 + (ve >= 0 ? ve : blank));
    d.xb = Elem<DT>::load1(acts, e0 + blank);
    d.xl = Elem<DT>::load1(acts, e0 + (lab >= 0 ? lab : blank));
    d.xd = Elem<DT>::load1(acts, e0 + (lane < D ? V + lane : (lane < nbig ? blank - 1 - lane : blank)));
  };
  auto reduce = [&](int uu, int lab, const Row& d) {
    const RowSplit<DT> sp(d.mis, V);
    const int full = sp.nb >> 6, rem = sp.nb & 63;
    float x[R][VEC];
#pragma unroll
    for (int k = 0; k < R; ++k) {
      Elem<DT>::unpack(d.raw[k], x[k]);
      if (k >= full) {  // wave-uniform: the last, partly filled slot and the unused ones
        const bool ok = (k == full) && (lane < rem);
#pragma unroll
        for (int i = 0; i < VEC; ++i) x[k][i] = ok ? x[k][i] : kNegInf;
      }
    }
    const float xe = sp.extra_token(lane) >= 0 ? d.xe : kNegInf;
    float cm = xe;
#pragma unroll
    for (int k = 0; k < R; ++k)
#pragma unroll
      for (int i = 0; i < VEC; ++i) cm = fmaxf(cm, x[k][i]);
    const float M = wave_max_u(cm);
    const float off = -M * kLog2e;
    float acc = stream_exp2(fmaf(xe, kLog2e, off));
#pragma unroll
    for (int k = 0; k < R; ++k)
#pragma unroll
      for (int i = 0; i < VEC; ++i) acc += stream_exp2(fmaf(x[k][i], kLog2e, off));
    const float S = wave_sum_u(acc);
    const float dn = -M - __builtin_amdgcn_logf(S) * 0.6931471805599453f;

    const size_t base = ((size_t)(b * ND + t + uu) * A) * Us + uu;
    if (lane == 0) {
      denom[cell0 + uu] = dn;
      arcs[base] = d.xb + dn;
      arcs[base + Us] = lab >= 0 ? d.xl + dn : 0.f;
    }
    if (D > 0) {  // duration log-softmax (rnnt_pytorch.py:568), one lane per duration
      const float xd = lane < D ? d.xd : kNegInf;
      const float dm = wave_max_u(xd);
      const float ds = wave_sum_u(lane < D ? expf(xd - dm) : 0.f);
      const float dden = -dm - logf(ds);
      if (lane < D) arcs[base + (size_t)(2 + lane) * Us] = xd + dden;
    }
    if (lane < nbig) arcs[base + (size_t)(2 + lane) * Us] = d.xd + dn;  // big-blank log-probs (multi-blank)
  };

  Row cur, nxt;
  fetch(u_begin, labs[0], cur);
#pragma unroll
  for (int i = 0; i < kRowsPerWave; ++i) {
    const int uu = u_begin + kRowWaves * i;
    if (uu >= u_end) break;
    if (i + 1 < kRowsPerWave) {
      // always fetch (the last row of the wave re-reads itself): an unconditional load keeps the
      // wait counters exact, so reducing row i never waits for the loads of row i+1
      const bool more = uu + kRowWaves < u_end;
      fetch(more ? uu + kRowWaves : uu, more ? labs[i + 1] : labs[i], nxt);
    }
    reduce(uu, labs[i], cur);
    cur = nxt;
  }
}

// FUSED (RNNT): the row's coefficients are derived here from the lattice state, one wave-uniform
// evaluation per row, instead of being read from the coefficient buffer a cell kernel filled.
template <int DT, int R, bool FUSED>
__global__ __launch_bounds__(kRowThreads) void grad_rows_kernel(const void* __restrict__ acts, void* __restrict__ grads,
                                                        const float* __restrict__ coef, LatticeView lv,
                                                        const int64_t* __restrict__ act_lens,
                                                        const int64_t* __restrict__ label_lens, int T, int U, int V,
                                                        int D, int blank, int CS, int flags, int nchunks,
                                                        int nblocks, GridDiv gdiv) {
  constexpr int VEC = Elem<DT>::VEC;
  // all kernel arguments are fetched in one go, not one batch per use (the loads this kernel wants
  // on the scalar unit are written as such, so the asm's side effect costs nothing)
  asm volatile("" ::"s"((uintptr_t)acts), "s"((uintptr_t)grads), "s"((uintptr_t)coef), "s"((uintptr_t)act_lens),
               "s"((uintptr_t)label_lens), "s"((uintptr_t)lv.denom), "s"((uintptr_t)lv.arcs), "s"((uintptr_t)lv.alphas),
               "s"((uintptr_t)lv.betas), "s"((uintptr_t)lv.ll), "s"((uintptr_t)lv.labels), "s"((uintptr_t)lv.grad_scale),
               "s"(lv.grad_scale_stride), "s"(lv.grad_mul), "s"(lv.ND), "s"(lv.Us), "s"(lv.A), "s"(lv.lambda),
               "s"(lv.clamp), "s"(T), "s"(U), "s"(V), "s"(D), "s"(blank), "s"(CS), "s"(flags), "s"(nchunks),
               "s"(nblocks), "s"(gdiv.chunks.mul), "s"(gdiv.chunks.shift), "s"(gdiv.T.mul), "s"(gdiv.T.shift));
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  // 1-D grid over (b,t,chunk), chunk fastest = memory order
  unsigned wg = logical_block();
  if (wg >= (unsigned)nblocks) return;
#if MI_K4_REVERSE
  wg = (unsigned)nblocks - 1u - wg;
#endif
  const unsigned bt = fast_div(wg, gdiv.chunks), chunk = wg - bt * (unsigned)nchunks;
  const int b = (int)fast_div(bt, gdiv.T), t = (int)(bt - (unsigned)b * (unsigned)T);
  const UttLens len = load_lens(act_lens, label_lens, b, T, U);
  const int Tb = len.Tb, Ub = len.Ub;
  const int VD = V + D;
  const unsigned cell0 = ((unsigned)b * (unsigned)T + (unsigned)t) * (unsigned)U;  // B*T*U < 2^31 (host check)
  const int c0 = (int)chunk * kChunkRows;
  const int c1 = min(U, c0 + kChunkRows);
  // rows [c0, z0) of this chunk carry a gradient, rows [z0, c1) are padding: one contiguous range of zeros
  const int z0 = (t >= Tb) ? c0 : max(c0, min(Ub, c1));
  if (!(flags & kFlagPaddingDone)) zero_elems<DT>(grads, (size_t)(cell0 + z0) * VD, (size_t)(cell0 + c1) * VD);
  const int u_begin = c0 + wave;
  if (u_begin >= z0) return;

  struct Row {
    uint4 raw[R];
    RowCoef c;
    float xe, gd;
    int mis;
  };
  // head, tail and duration entries of a row: one element per lane
  auto extra_index = [&](const RowSplit<DT>& sp) {
    int v = sp.extra_token(lane);
    if (lane >= 2 * VEC && lane < 2 * VEC + D) v = V + lane - 2 * VEC;
    return v;
  };
  auto fetch = [&](int uu, Row& d) {
    const size_t e0 = (size_t)(cell0 + (unsigned)uu) * (unsigned)VD;
    const RowWindow<DT> w(acts, e0);
    const RowSplit<DT> sp(w.mis, V);
    d.mis = w.mis;
    // unconditional loads, as in the denominator pass
#pragma unroll
    for (int k = 0; k < R; ++k) d.raw[k] = load_stream<MI_NT_K4 != 0>(w.vp + sp.body_vector(lane + 64 * k));
    const int v = extra_index(sp);
    d.xe = Elem<DT>::load1(acts, e0 + ((v >= 0 && v < V) ? v : blank));
    if constexpr (FUSED) {
      const CoefRaw cr = load_coef_raw(lv, b, t, uu, Tb, Ub, T, U);
      d.c = finish_coef(cr, lv, t, uu, Tb, Ub, V, blank);
      d.gd = 0.f;
    } else {
      const float* c = coef + (size_t)(cell0 + uu) * CS;
      const float4 ca = *(const float4*)c;        // denom*log2e, W*scale, clamp bound, G_blank
      const float2 cb = *(const float2*)(c + 4);  // G_label, label id
      d.c.dl2 = ca.x; d.c.W = ca.y; d.c.cb = ca.z; d.c.gB = ca.w; d.c.gL = cb.x;
      d.c.lab = __float_as_int(cb.y);
      d.gd = c[v >= V ? kCoefBase + v - V : 0];
    }
  };
  auto emit = [&](int uu, const Row& d) {
    const size_t e0 = (size_t)(cell0 + (unsigned)uu) * (unsigned)VD;
    const RowSplit<DT> sp(d.mis, V);
    const float dl2 = d.c.dl2, W = d.c.W, cb = d.c.cb, gB = d.c.gB, gL = d.c.gL;
    const int lab = d.c.lab;
    const bool clamp_on = cb < INFINITY;
    char* grow = (char*)grads + e0 * Elem<DT>::BYTES;  // same 16-byte phase as the acts row
    uint4* gvp = (uint4*)(grow - d.mis * Elem<DT>::BYTES) + sp.jb0 + lane;
    const int jblank = (blank + d.mis) / VEC - sp.jb0, jlab = lab >= 0 ? (lab + d.mis) / VEC - sp.jb0 : -1;
#pragma unroll
    for (int k = 0; k < R; ++k) {
      const int j = lane + 64 * k;  // whole vector j of the row
      if (j < sp.nb) {
        float x[VEC], g[VEC];
        Elem<DT>::unpack(d.raw[k], x);
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
          float gi = stream_exp2(fmaf(x[i], kLog2e, dl2)) * W;
          if (clamp_on) gi = clamp_sym(gi, cb);
          g[i] = gi;
        }
        if (j == jblank || j == jlab) {  // the two special logits are patched in the vector that holds them
          const int first = sp.hc + j * VEC;
#pragma unroll
          for (int i = 0; i < VEC; ++i) {
            if (first + i == blank) g[i] = gB;
            if (first + i == lab) g[i] = gL;
          }
        }
        store_stream(gvp + 64 * k, Elem<DT>::pack(g));
      }
    }
    const int v = extra_index(sp);
    if (v >= 0) {
      float g = (flags & kFlagZeroDurations) ? 0.f : d.gd;
      if (v < V) {
        g = stream_exp2(fmaf(d.xe, kLog2e, dl2)) * W;
        if (clamp_on) g = clamp_sym(g, cb);
        if (v == blank) g = gB;
        if (v == lab) g = gL;
      }
      Elem<DT>::store1(grads, e0 + v, g);
    }
  };

  Row cur, nxt;
  fetch(u_begin, cur);
#pragma unroll
  for (int i = 0; i < kRowsPerWave; ++i) {
    const int uu = u_begin + kRowWaves * i;
    if (uu >= z0) break;
    if (i + 1 < kRowsPerWave) fetch(uu + kRowWaves < z0 ? uu + kRowWaves : uu, nxt);
    emit(uu, cur);
    cur = nxt;
  }
}

// Zero-fill of the padded cells only (every row with t >= T_b or u >= U_b): a function of the
// lengths alone, so it can run on another stream while the lattice recursion runs and HBM
// would otherwise idle.  Same chunk order as the gradient pass.
template <int DT>
__global__ __launch_bounds__(kRowThreads) void zero_padding_kernel(void* __restrict__ grads,
                                                                   const int64_t* __restrict__ act_lens,
                                                                   const int64_t* __restrict__ label_lens, int T,
                                                                   int U, int VD, int nchunks, int nblocks, GridDiv gdiv) {
  const unsigned wg = logical_block();
  if (wg >= (unsigned)nblocks) return;
  const unsigned bt = fast_div(wg, gdiv.chunks), chunk = wg - bt * (unsigned)nchunks;
  const int b = (int)fast_div(bt, gdiv.T), t = (int)(bt - (unsigned)b * (unsigned)T);
  const int Tb = clampi(act_lens[b], 1, T);
  const int Ub = clampi(label_lens[b] + 1, 1, U);
  const unsigned cell0 = ((unsigned)b * (unsigned)T + (unsigned)t) * (unsigned)U;  // B*T*U < 2^31 (host check)
  const int c0 = (int)chunk * kChunkRows;
  const int c1 = min(U, c0 + kChunkRows);
  const int z0 = (t >= Tb) ? c0 : max(c0, min(Ub, c1));
  zero_elems<DT>(grads, (size_t)(cell0 + z0) * VD, (size_t)(cell0 + c1) * VD);
}

// ----------------------------------------------------------------------------------------
// The bandwidth passes for rows too long to sit in one wave's registers: a workgroup of RT
// threads owns one row, every thread moves NVT aligned 16-byte vectors (RT apart), and the
// waves' partial (max, sum) pairs meet in LDS.  Wave 0 of a row also moves the row's ragged
// head and tail (and the duration entries of a TDT row), one element per lane.
// ----------------------------------------------------------------------------------------
template <int RT> struct BlockRows {
  static constexpr int THREADS = RT < 256 ? 256 : RT;
  static constexpr int ROWS = THREADS / RT;  // rows per workgroup
  static constexpr int WPR = RT / 64;        // waves per row
};

template <int DT, int RT, int NVT>
__global__ __launch_bounds__(BlockRows<RT>::THREADS) void denom_block_kernel(
    const void* __restrict__ acts, const int64_t* __restrict__ labels, const int64_t* __restrict__ act_lens,
    const int64_t* __restrict__ label_lens, float* __restrict__ denom, float* __restrict__ arcs, int T, int U, int V,
    int D, int nbig, int blank, int ND, int Us, int A, int nchunks, int nblocks, GridDiv gdiv) {
  constexpr int VEC = Elem<DT>::VEC;
  constexpr int ROWS = BlockRows<RT>::ROWS, WPR = BlockRows<RT>::WPR, WAVES = BlockRows<RT>::THREADS / 64;
  __shared__ float2 part[WAVES];
  // all kernel arguments are fetched in one go, not one batch per use (the loads this kernel wants
  // on the scalar unit are written as such, so the asm's side effect costs nothing)
  asm volatile("" ::"s"((uintptr_t)acts), "s"((uintptr_t)labels), "s"((uintptr_t)act_lens), "s"((uintptr_t)label_lens),
               "s"((uintptr_t)denom), "s"((uintptr_t)arcs), "s"(T), "s"(U), "s"(V), "s"(D), "s"(nbig), "s"(blank), "s"(ND), "s"(Us),
               "s"(A), "s"(nchunks), "s"(nblocks), "s"(gdiv.chunks.mul), "s"(gdiv.chunks.shift), "s"(gdiv.T.mul),
               "s"(gdiv.T.shift));
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int row_in_wg = wave / WPR, wave_in_row = wave - row_in_wg * WPR;
  const int tr = wave_in_row * 64 + lane;  // thread within the row
  unsigned wg = logical_block();
  if (wg >= (unsigned)nblocks) return;
#if MI_K1_REVERSE
  wg = (unsigned)nblocks - 1u - wg;
#endif
  const unsigned bt = fast_div(wg, gdiv.chunks), chunk = wg - bt * (unsigned)nchunks;
  const int b = (int)fast_div(bt, gdiv.T), t = (int)(bt - (unsigned)b * (unsigned)T);
  const int u = (int)chunk * ROWS + row_in_wg;
  // the row's label id travels with the lengths (a clamped index, dropped below if the row has no
  // label arc; with U == 1 there is no label array and a length is read instead)
  long long lab_raw = uni((long long)sload(U > 1 ? labels + ((size_t)b * (U - 1) + max(min(u, U - 2), 0)) : act_lens + b));
  const UttLens len = load_lens(act_lens, label_lens, b, T, U);
  asm("" : "+s"(lab_raw));
  const int Tb = len.Tb, Ub = len.Ub;
  if (t >= Tb || (int)chunk * ROWS >= Ub) return;  // the whole workgroup leaves: no barrier is left waiting
  const bool live = u < Ub;  // wave-uniform
  const int VD = V + D;
  const unsigned cell0 = ((unsigned)b * (unsigned)T + (unsigned)t) * (unsigned)U;  // B*T*U < 2^31 (host check)
  const size_t e0 = (size_t)(cell0 + (unsigned)(live ? u : 0)) * (unsigned)VD;

  float m_w = -1.0e30f, s_w = 0.f;  // this wave's share of the row: max and sum of 2^((x - max) log2 e)
  float xb = 0.f, xl = 0.f, xd = 0.f;
  int lab = -1;
  if (live) {
    const RowWindow<DT> w(acts, e0);
    const RowSplit<DT> sp(w.mis, V);
    uint4 raw[NVT];
#pragma unroll
    for (int k = 0; k < NVT; ++k) raw[k] = load_stream<MI_NT_K1 != 0>(w.vp + sp.body_vector(tr + RT * k));
    float xe = kNegInf;
    if (wave_in_row == 0) {
      lab = (u < Ub - 1) ? clampi(lab_raw, 0, V - 1) : -1;
      const int ve = sp.extra_token(lane);
      const float x1 = Elem<DT>::load1(acts, e0 + (ve >= 0 ? ve : blank));
      xb = Elem<DT>::load1(acts, e0 + blank);
      xl = Elem<DT>::load1(acts, e0 + (lab >= 0 ? lab : blank));
      xd = Elem<DT>::load1(acts, e0 + (lane < D ? V + lane : (lane < nbig ? blank - 1 - lane : blank)));
      xe = ve >= 0 ? x1 : kNegInf;
    }
    float x[NVT][VEC];
#pragma unroll
    for (int k = 0; k < NVT; ++k) {
      Elem<DT>::unpack(raw[k], x[k]);
      const bool ok = tr + RT * k < sp.nb;
#pragma unroll
      for (int i = 0; i < VEC; ++i) x[k][i] = ok ? x[k][i] : kNegInf;
    }
    float cm = xe;
#pragma unroll
    for (int k = 0; k < NVT; ++k)
#pragma unroll
      for (int i = 0; i < VEC; ++i) cm = fmaxf(cm, x[k][i]);
    m_w = fmaxf(wave_max_u(cm), -1.0e30f);  // finite even for a wave that holds no element of the row
    const float off = -m_w * kLog2e;
    float acc = stream_exp2(fmaf(xe, kLog2e, off));
#pragma unroll
    for (int k = 0; k < NVT; ++k)
#pragma unroll
      for (int i = 0; i < VEC; ++i) acc += stream_exp2(fmaf(x[k][i], kLog2e, off));
    s_w = wave_sum_u(acc);
  }
  if (lane == 0) part[wave] = make_float2(m_w, s_w);
  __syncthreads();
  if (!live || wave_in_row != 0) return;
  float M = -1.0e30f;
#pragma unroll
  for (int i = 0; i < WPR; ++i) M = fmaxf(M, part[row_in_wg * WPR + i].x);
  float S = 0.f;
#pragma unroll
  for (int i = 0; i < WPR; ++i) {
    const float2 p = part[row_in_wg * WPR + i];
    S = fmaf(p.y, fast_exp2((p.x - M) * kLog2e), S);
  }
  const float dn = -M - __builtin_amdgcn_logf(S) * 0.6931471805599453f;
  const size_t base = ((size_t)(b * ND + t + u) * A) * Us + u;
  if (lane == 0) {
    denom[cell0 + u] = dn;
    arcs[base] = xb + dn;
    arcs[base + Us] = lab >= 0 ? xl + dn : 0.f;
  }
  if (D > 0) {  // duration log-softmax (rnnt_pytorch.py:568), one lane per duration
    const float xdm = lane < D ? xd : kNegInf;
    const float dm = wave_max_u(xdm);
    const float ds = wave_sum_u(lane < D ? expf(xdm - dm) : 0.f);
    const float dden = -dm - logf(ds);
    if (lane < D) arcs[base + (size_t)(2 + lane) * Us] = xdm + dden;
  }
  if (lane < nbig) arcs[base + (size_t)(2 + lane) * Us] = xd + dn;  // big-blank log-probs (multi-blank)
}

template <int DT, int RT, int NVT, bool FUSED>
__global__ __launch_bounds__(BlockRows<RT>::THREADS) void grad_block_kernel(
    const void* __restrict__ acts, void* __restrict__ grads, const float* __restrict__ coef, LatticeView lv,
    const int64_t* __restrict__ act_lens, const int64_t* __restrict__ label_lens, int T, int U, int V, int D,
    int blank, int CS, int flags, int nchunks, int nblocks, GridDiv gdiv) {
  constexpr int VEC = Elem<DT>::VEC;
  constexpr int ROWS = BlockRows<RT>::ROWS, WPR = BlockRows<RT>::WPR;
  // all kernel arguments are fetched in one go, not one batch per use (the loads this kernel wants
  // on the scalar unit are written as such, so the asm's side effect costs nothing)
  asm volatile("" ::"s"((uintptr_t)acts), "s"((uintptr_t)grads), "s"((uintptr_t)coef), "s"((uintptr_t)act_lens),
               "s"((uintptr_t)label_lens), "s"((uintptr_t)lv.denom), "s"((uintptr_t)lv.arcs), "s"((uintptr_t)lv.alphas),
               "s"((uintptr_t)lv.betas), "s"((uintptr_t)lv.ll), "s"((uintptr_t)lv.labels), "s"((uintptr_t)lv.grad_scale),
               "s"(lv.grad_scale_stride), "s"(lv.grad_mul), "s"(lv.ND), "s"(lv.Us), "s"(lv.A), "s"(lv.lambda),
               "s"(lv.clamp), "s"(T), "s"(U), "s"(V), "s"(D), "s"(blank), "s"(CS), "s"(flags), "s"(nchunks),
               "s"(nblocks), "s"(gdiv.chunks.mul), "s"(gdiv.chunks.shift), "s"(gdiv.T.mul), "s"(gdiv.T.shift));
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int row_in_wg = wave / WPR, wave_in_row = wave - row_in_wg * WPR;
  const int tr = wave_in_row * 64 + lane;
  unsigned wg = logical_block();
  if (wg >= (unsigned)nblocks) return;
#if MI_K4_REVERSE
  wg = (unsigned)nblocks - 1u - wg;
#endif
  const unsigned bt = fast_div(wg, gdiv.chunks), chunk = wg - bt * (unsigned)nchunks;
  const int b = (int)fast_div(bt, gdiv.T), t = (int)(bt - (unsigned)b * (unsigned)T);
  const int u = (int)chunk * ROWS + row_in_wg;
  if (u >= U) return;
  const UttLens len = load_lens(act_lens, label_lens, b, T, U);
  const int Tb = len.Tb, Ub = len.Ub;
  const int VD = V + D;
  const unsigned cell0 = ((unsigned)b * (unsigned)T + (unsigned)t) * (unsigned)U;  // B*T*U < 2^31 (host check)
  const size_t e0 = (size_t)(cell0 + (unsigned)u) * (unsigned)VD;
  const RowWindow<DT> w(acts, e0);
  const RowSplit<DT> sp(w.mis, V);
  char* grow = (char*)grads + e0 * Elem<DT>::BYTES;  // same 16-byte phase as the acts row
  uint4* gvp = (uint4*)(grow - w.mis * Elem<DT>::BYTES) + sp.jb0 + tr;
  // head, tail and duration entries of a row: one element per lane of the row's wave 0
  int v = -1;
  if (wave_in_row == 0) {
    v = sp.extra_token(lane);
    if (lane >= 2 * VEC && lane < 2 * VEC + D) v = V + lane - 2 * VEC;
  }

  if (t >= Tb || u >= Ub) {  // a padded row: zeros
    if (flags & kFlagPaddingDone) return;
    const uint4 z = make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int k = 0; k < NVT; ++k)
      if (tr + RT * k < sp.nb) store_stream(gvp + RT * k, z);
    if (v >= 0) Elem<DT>::store1(grads, e0 + v, 0.f);
    return;
  }

  uint4 raw[NVT];
#pragma unroll
  for (int k = 0; k < NVT; ++k) raw[k] = load_stream<MI_NT_K4 != 0>(w.vp + sp.body_vector(tr + RT * k));
  float xe = 0.f, gd = 0.f;
  if (wave_in_row == 0) xe = Elem<DT>::load1(acts, e0 + ((v >= 0 && v < V) ? v : blank));
  RowCoef c;
  if constexpr (FUSED) {
    const CoefRaw cr = load_coef_raw(lv, b, t, u, Tb, Ub, T, U);
    c = finish_coef(cr, lv, t, u, Tb, Ub, V, blank);
  } else {
    const float* cp = coef + (size_t)(cell0 + u) * CS;
    const float4 ca = *(const float4*)cp;        // denom*log2e, W*scale, clamp bound, G_blank
    const float2 cb = *(const float2*)(cp + 4);  // G_label, label id
    c.dl2 = ca.x; c.W = ca.y; c.cb = ca.z; c.gB = ca.w; c.gL = cb.x;
    c.lab = __float_as_int(cb.y);
    if (wave_in_row == 0) gd = cp[v >= V ? kCoefBase + v - V : 0];
  }
  const float dl2 = c.dl2, W = c.W, cbnd = c.cb, gB = c.gB, gL = c.gL;
  const int lab = c.lab;
  const bool clamp_on = cbnd < INFINITY;
  const int jblank = (blank + w.mis) / VEC - sp.jb0, jlab = lab >= 0 ? (lab + w.mis) / VEC - sp.jb0 : -1;
#pragma unroll
  for (int k = 0; k < NVT; ++k) {
    const int j = tr + RT * k;  // whole vector j of the row
    if (j < sp.nb) {
      float x[VEC], g[VEC];
      Elem<DT>::unpack(raw[k], x);
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        float gi = stream_exp2(fmaf(x[i], kLog2e, dl2)) * W;
        if (clamp_on) gi = clamp_sym(gi, cbnd);
        g[i] = gi;
      }
      if (j == jblank || j == jlab) {  // the two special logits are patched in the vector that holds them
        const int first = sp.hc + j * VEC;
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
          if (first + i == blank) g[i] = gB;
          if (first + i == lab) g[i] = gL;
        }
      }
      store_stream(gvp + RT * k, Elem<DT>::pack(g));
    }
  }
  if (v >= 0) {
    float g = (flags & kFlagZeroDurations) ? 0.f : gd;
    if (v < V) {
      g = stream_exp2(fmaf(xe, kLog2e, dl2)) * W;
      if (clamp_on) g = clamp_sym(g, cbnd);
      if (v == blank) g = gB;
      if (v == lab) g = gL;
    }
    Elem<DT>::store1(grads, e0 + v, g);
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
// Benchmark aid: while enabled, every launch of a pipeline kernel is bracketed by a pair of
// HIP events on the stream it is launched on, so a harness can read per-kernel durations
// of the very launches it timed.  Off by default; the events are created when it is enabled.
struct ProfState {
  bool on = false;
  int cap = 0;
  unsigned mask = ~0u;
  int count[MI_PROFILE_KERNELS] = {};
  std::vector<hipEvent_t> start[MI_PROFILE_KERNELS], stop[MI_PROFILE_KERNELS];
};
ProfState g_prof;

struct ProfScope {
  int id;
  hipStream_t stream;
  bool live;
  ProfScope(int kernel_id, hipStream_t s) : id(kernel_id), stream(s), live(false) {
    if (g_prof.on && ((g_prof.mask >> id) & 1u) && g_prof.count[id] < g_prof.cap) {
      live = true;
      (void)hipEventRecord(g_prof.start[id][g_prof.count[id]], stream);
    }
  }
  ~ProfScope() {
    if (live) {
      (void)hipEventRecord(g_prof.stop[id][g_prof.count[id]], stream);
      ++g_prof.count[id];
    }
  }
};

// Plain 16-byte copy, grid-stride: the yardstick for the HBM counters and for the copy
// bandwidth this GPU actually reaches.
// One 16-byte vector per thread, 4 KB per workgroup, workgroups dealt to the XCDs in spans of
// consecutive pieces: of the streaming patterns measured on this GPU (grid-stride loops, 2 to 8
// vectors per thread, runs of pieces per workgroup) the one that copies fastest.
__global__ __launch_bounds__(256) void copy_probe_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst,
                                                         size_t nvec) {
  const size_t i = (size_t)logical_block() * 256 + threadIdx.x;
  if (i < nvec) dst[i] = src[i];
}

struct Common {
  const void* acts;
  int dt;
  const int64_t *labels, *act_lens, *label_lens;
  int B, T, U, V, D, blank;
  int nbig;  // multi-blank: number of big blanks (their logits sit at blank-1-i); D is 0 then
  char* ws;
  hipStream_t stream;
  Layout L;
};

int check_common(const void* acts, int dt, const int64_t* labels, const int64_t* act_lens, const int64_t* label_lens,
                 int B, int T, int U, int V, int D, int blank, void* ws, size_t ws_bytes, void* stream, Common* c,
                 int nbig = 0) {
  if (!acts || !act_lens || !label_lens || !ws) return MI_TRANSDUCER_INVALID_VALUE;
  if (U > 1 && !labels) return MI_TRANSDUCER_INVALID_VALUE;
  if (dt != MI_DTYPE_F32 && dt != MI_DTYPE_BF16 && dt != MI_DTYPE_F16) return MI_TRANSDUCER_INVALID_VALUE;
  if (V <= 0 || blank < 0 || blank >= V) return MI_TRANSDUCER_INVALID_VALUE;
  // multi-blank: the big blanks take the extra arc planes and coefficient slots that durations take for TDT
  if (nbig < 0 || nbig > MI_TRANSDUCER_MAX_BIG_BLANKS || (nbig > 0 && (D != 0 || blank - nbig < 0)))
    return MI_TRANSDUCER_INVALID_VALUE;
  if (!make_layout(B, T, U, nbig ? nbig : D, &c->L)) return MI_TRANSDUCER_INVALID_VALUE;
  if (ws_bytes < c->L.total || ((uintptr_t)ws & 255)) return MI_TRANSDUCER_INVALID_VALUE;
  if ((long long)B * T > 65535LL * 8) return MI_TRANSDUCER_INVALID_VALUE;  // grid-size limit of the long-row kernels
  c->acts = acts; c->dt = dt; c->labels = labels; c->act_lens = act_lens; c->label_lens = label_lens;
  c->B = B; c->T = T; c->U = U; c->V = V; c->D = D; c->blank = blank; c->nbig = nbig;
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

struct RowGrid {
  dim3 grid;
  int BT, bt_chunk;
};
inline RowGrid row_grid(const Common& c) {
  RowGrid g;
  const unsigned ublocks = (unsigned)((c.U + kRowsPerBlock - 1) / kRowsPerBlock);
  g.BT = c.B * c.T;
#if MI_XCD_MAP
  g.bt_chunk = (g.BT + 7) / 8;
  g.grid = dim3(8 * ublocks, (unsigned)g.bt_chunk, 1);
#else
  g.bt_chunk = g.BT;
  g.grid = dim3(ublocks, (unsigned)g.BT, 1);
#endif
  return g;
}

// smallest R in {1,2,4,8} with floor(V / VEC) <= 64*R, or 0 if the rows are too long for the
// register-resident kernels
#ifndef MI_USE_ROWS
#define MI_USE_ROWS 1
#endif
inline int rows_R(const Common& c) {
  if (!MI_USE_ROWS) return 0;
  const int vec = c.dt == MI_DTYPE_F32 ? 4 : 8;
  const int nb = c.V / vec;
  for (int r = 1; r <= 8; r *= 2)
    if (nb <= 64 * r) return r;
  return 0;
}
// the row kernels store gradient vectors at the 16-byte phase of the logits row
inline int grad_rows_R(const Common& c, const void* grads) {
  const bool same_phase = (((uintptr_t)c.acts ^ (uintptr_t)grads) & 15) == 0;
  return same_phase ? rows_R(c) : 0;
}
// Workgroup-per-row kernels: RT threads per row, NVT vectors per thread.  RT == 0: not applicable.
// The denominator pass uses them for rows too long for the register-resident wave-per-row
// kernels (more than 512 whole vectors).  The gradient pass uses them from 65 vectors up, with
// two vectors per thread where the row allows it: of the splits tried (1, 2 and 4 vectors per
// thread) that one streams fastest.
#ifndef MI_USE_BLOCK_ROWS
#define MI_USE_BLOCK_ROWS 1
#endif
struct BlockPlan {
  int RT, NVT;
  int rows() const { return (RT < 256 ? 256 : RT) / RT; }
  int threads() const { return RT < 256 ? 256 : RT; }
};
inline int whole_vectors(const Common& c) { return c.V / (c.dt == MI_DTYPE_F32 ? 4 : 8); }
inline bool block_rows_ok(const Common& c) {
  return MI_USE_BLOCK_ROWS && 2 * (c.dt == MI_DTYPE_F32 ? 4 : 8) + c.D <= 64;
}
inline BlockPlan denom_block_plan(const Common& c) {
  const int nb = whole_vectors(c);
  if (!block_rows_ok(c) || nb <= 512) return BlockPlan{0, 0};
  for (int nvt = 1; nvt <= 8; nvt *= 2)
    if (nb <= 1024 * nvt) return BlockPlan{1024, nvt};
  return BlockPlan{0, 0};
}
inline BlockPlan grad_block_plan(const Common& c, const void* grads) {
  const bool same_phase = (((uintptr_t)c.acts ^ (uintptr_t)grads) & 15) == 0;
  const int nb = whole_vectors(c);
  if (!same_phase || !block_rows_ok(c) || nb <= 64) return BlockPlan{0, 0};
  for (int rt = 64; rt <= 1024; rt *= 2)
    if (nb <= 2 * rt) return BlockPlan{rt, 2};
  for (int nvt = 4; nvt <= 8; nvt *= 2)
    if (nb <= 1024 * nvt) return BlockPlan{1024, nvt};
  return BlockPlan{0, 0};
}
inline int plan_chunks(const Common& c, const BlockPlan& p) { return (c.U + p.rows() - 1) / p.rows(); }
inline int plan_blocks(const Common& c, const BlockPlan& p) { return plan_chunks(c, p) * c.B * c.T; }
inline dim3 plan_grid(const Common& c, const BlockPlan& p) {
  const unsigned turn = 8u * MI_XCD_SPAN;
  return dim3(((unsigned)plan_blocks(c, p) + turn - 1) / turn * turn, 1, 1);
}
#define MI_FOR_DENOM_PLAN(P, CALL)          \
  do {                                      \
    if ((P).NVT == 1) CALL(1024, 1);        \
    else if ((P).NVT == 2) CALL(1024, 2);   \
    else if ((P).NVT == 4) CALL(1024, 4);   \
    else CALL(1024, 8);                     \
  } while (0)
#define MI_FOR_GRAD_PLAN(P, CALL)           \
  do {                                      \
    if ((P).NVT == 8) CALL(1024, 8);        \
    else if ((P).NVT == 4) CALL(1024, 4);   \
    else if ((P).RT == 64) CALL(64, 2);     \
    else if ((P).RT == 128) CALL(128, 2);   \
    else if ((P).RT == 256) CALL(256, 2);   \
    else if ((P).RT == 512) CALL(512, 2);   \
    else CALL(1024, 2);                     \
  } while (0)

inline int chunks_of(const Common& c) { return (c.U + kChunkRows - 1) / kChunkRows; }
inline int chunk_blocks(const Common& c) { return chunks_of(c) * c.B * c.T; }
// rounded up to whole turns of the XCD permutation
inline dim3 chunk_grid(const Common& c) {
  const unsigned turn = 8u * MI_XCD_SPAN;
  return dim3(((unsigned)chunk_blocks(c) + turn - 1) / turn * turn, 1, 1);
}

int run_denom(const Common& c) {
  const Layout& L = c.L;
  float* denom = (float*)(c.ws + L.off_denom);
  float* arcs = (float*)(c.ws + L.off_arcs);
  const RowGrid g = row_grid(c);
  const int R = rows_R(c);
  ProfScope prof(MI_PROFILE_DENOM, c.stream);
#define LAUNCH_DENOM_ROWS(DT, RR)                                                                                   \
  hipLaunchKernelGGL((denom_rows_kernel<DT, RR>), chunk_grid(c), dim3(kRowThreads), 0, c.stream, c.acts, c.labels,           \
                     c.act_lens, c.label_lens, denom, arcs, c.T, c.U, c.V, c.D, c.nbig, c.blank, L.ND, L.Us, L.A, chunks_of(c), chunk_blocks(c), make_griddiv(chunks_of(c), c.T))
#define LAUNCH_DENOM(DT)                                                                                            \
  do {                                                                                                              \
    switch (R) {                                                                                                    \
      case 1: LAUNCH_DENOM_ROWS(DT, 1); break;                                                                      \
      case 2: LAUNCH_DENOM_ROWS(DT, 2); break;                                                                      \
      case 4: LAUNCH_DENOM_ROWS(DT, 4); break;                                                                      \
      case 8: LAUNCH_DENOM_ROWS(DT, 8); break;                                                                      \
      default:                                                                                                      \
        hipLaunchKernelGGL(denom_gather_kernel<DT>, g.grid, dim3(256), 0, c.stream, c.acts, c.labels, c.act_lens,   \
                           c.label_lens, denom, arcs, c.T, c.U, c.V, c.D, c.nbig, c.blank, L.ND, L.Us, L.A, g.BT,           \
                           g.bt_chunk);                                                                             \
    }                                                                                                               \
  } while (0)
  const BlockPlan bp = denom_block_plan(c);
#define LAUNCH_DENOM_BLOCK(DT, RT_, NVT_)                                                                           \
  hipLaunchKernelGGL((denom_block_kernel<DT, RT_, NVT_>), plan_grid(c, bp), dim3(bp.threads()), 0, c.stream, c.acts, \
                     c.labels, c.act_lens, c.label_lens, denom, arcs, c.T, c.U, c.V, c.D, c.nbig, c.blank, L.ND, L.Us, L.A,  \
                     plan_chunks(c, bp), plan_blocks(c, bp), make_griddiv(plan_chunks(c, bp), c.T))
#define DENOM_BLOCK_F32(RT_, NVT_) LAUNCH_DENOM_BLOCK(MI_DTYPE_F32, RT_, NVT_)
#define DENOM_BLOCK_BF16(RT_, NVT_) LAUNCH_DENOM_BLOCK(MI_DTYPE_BF16, RT_, NVT_)
#define DENOM_BLOCK_F16(RT_, NVT_) LAUNCH_DENOM_BLOCK(MI_DTYPE_F16, RT_, NVT_)
  if (bp.RT) {
    if (c.dt == MI_DTYPE_F32) MI_FOR_DENOM_PLAN(bp, DENOM_BLOCK_F32);
    else if (c.dt == MI_DTYPE_BF16) MI_FOR_DENOM_PLAN(bp, DENOM_BLOCK_BF16);
    else MI_FOR_DENOM_PLAN(bp, DENOM_BLOCK_F16);
  } else if (c.dt == MI_DTYPE_F32) LAUNCH_DENOM(MI_DTYPE_F32);
  else if (c.dt == MI_DTYPE_BF16) LAUNCH_DENOM(MI_DTYPE_BF16);
  else LAUNCH_DENOM(MI_DTYPE_F16);
#undef DENOM_BLOCK_F32
#undef DENOM_BLOCK_BF16
#undef DENOM_BLOCK_F16
#undef LAUNCH_DENOM_BLOCK
#undef LAUNCH_DENOM
#undef LAUNCH_DENOM_ROWS
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
  ProfScope prof(MI_PROFILE_LATTICE, c.stream);
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
  ProfScope prof(MI_PROFILE_LATTICE, c.stream);
  // workgroup version: one thread per column, all of a cell's arcs in one log-sum-exp
  const size_t lds_block = (size_t)prm.R * 2 * prm.D * L.Us * sizeof(double);
  if (prm.D <= 8 && L.Us <= 256 && lds_block <= 160 * 1024) {
#define LAUNCH_TBLK(DD)                                                                                              \
  if (lds_block > 48 * 1024 &&                                                                                       \
      hipFuncSetAttribute((const void*)tdt_lattice_pair_kernel<DD>, hipFuncAttributeMaxDynamicSharedMemorySize,      \
                          (int)lds_block) != hipSuccess)                                                             \
    return MI_TRANSDUCER_LAUNCH_FAILURE;                                                                             \
  hipLaunchKernelGGL(tdt_lattice_pair_kernel<DD>, dim3(grid), dim3(2 * L.Us), lds_block, c.stream, arcs, alphas, betas,  \
                     ll, costs, c.act_lens, c.label_lens, c.T, c.U, L.ND, L.Us, cost_scale_of(lambda), with_betas,   \
                     prm)
    switch (prm.D) {
      case 1: LAUNCH_TBLK(1); break;
      case 2: LAUNCH_TBLK(2); break;
      case 3: LAUNCH_TBLK(3); break;
      case 4: LAUNCH_TBLK(4); break;
      case 5: LAUNCH_TBLK(5); break;
      case 6: LAUNCH_TBLK(6); break;
      case 7: LAUNCH_TBLK(7); break;
      default: LAUNCH_TBLK(8); break;
    }
#undef LAUNCH_TBLK
    return launch_status();
  }
  // general fallback (many durations or a very wide label axis): one wave per lattice
  const size_t lds = (size_t)2 * prm.R * L.Us * sizeof(double);
  if (lds > 160 * 1024) return MI_TRANSDUCER_INVALID_VALUE;  // e.g. U = 1024 with a longest duration above 8
#define LAUNCH_TLAT(KK)                                                                                              \
  if (lds > 48 * 1024 &&                                                                                             \
      hipFuncSetAttribute((const void*)tdt_lattice_kernel<KK>, hipFuncAttributeMaxDynamicSharedMemorySize,           \
                          (int)lds) != hipSuccess)                                                                   \
    return MI_TRANSDUCER_LAUNCH_FAILURE;                                                                             \
  hipLaunchKernelGGL(tdt_lattice_kernel<KK>, dim3(grid), dim3(64), lds, c.stream, arcs, alphas, betas, ll, costs,    \
                     c.act_lens, c.label_lens, c.T, c.U, L.ND, L.A, cost_scale_of(lambda), with_betas, prm)
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

struct ScaleArg {
  const float* ptr;
  int stride;
  float mul;
};

// fused != 0: RNNT rows derive their coefficients from the lattice state inside the pass
// (needs no cell kernel); only the register-resident row kernels can do that
int run_grad_stream(const Common& c, void* grads, int flags, bool fused, const ScaleArg& sc, float lambda,
                    float clamp) {
  const Layout& L = c.L;
  const float* coef = (const float*)(c.ws + L.off_coef);
  const RowGrid g = row_grid(c);
  LatticeView lv;
  lv.denom = (const float*)(c.ws + L.off_denom);
  lv.arcs = (const float*)(c.ws + L.off_arcs);
  lv.alphas = (const double*)(c.ws + L.off_alphas);
  lv.betas = (const double*)(c.ws + L.off_betas);
  lv.ll = (const double*)(c.ws + L.off_ll);
  lv.labels = c.labels;
  lv.grad_scale = sc.ptr;
  lv.grad_scale_stride = sc.stride;
  lv.grad_mul = sc.mul;
  lv.ND = L.ND; lv.Us = L.Us; lv.A = L.A;
  lv.lambda = lambda; lv.clamp = clamp;
  const int R = grad_rows_R(c, grads);
  ProfScope prof(MI_PROFILE_GRAD, c.stream);
#define LAUNCH_GRAD_ROWS(DT, RR)                                                                                    \
  do {                                                                                                              \
    if (fused)                                                                                                      \
      hipLaunchKernelGGL((grad_rows_kernel<DT, RR, true>), chunk_grid(c), dim3(kRowThreads), 0, c.stream, c.acts, grads,     \
                         coef, lv, c.act_lens, c.label_lens, c.T, c.U, c.V, c.D, c.blank, L.CS, flags,               \
                         chunks_of(c), chunk_blocks(c), make_griddiv(chunks_of(c), c.T));                                                            \
    else                                                                                                            \
      hipLaunchKernelGGL((grad_rows_kernel<DT, RR, false>), chunk_grid(c), dim3(kRowThreads), 0, c.stream, c.acts, grads,    \
                         coef, lv, c.act_lens, c.label_lens, c.T, c.U, c.V, c.D, c.blank, L.CS, flags,               \
                         chunks_of(c), chunk_blocks(c), make_griddiv(chunks_of(c), c.T));                                                            \
  } while (0)
#define LAUNCH_GRAD(DT)                                                                                             \
  do {                                                                                                              \
    switch (R) {                                                                                                    \
      case 1: LAUNCH_GRAD_ROWS(DT, 1); break;                                                                       \
      case 2: LAUNCH_GRAD_ROWS(DT, 2); break;                                                                       \
      case 4: LAUNCH_GRAD_ROWS(DT, 4); break;                                                                       \
      case 8: LAUNCH_GRAD_ROWS(DT, 8); break;                                                                       \
      default:                                                                                                      \
        hipLaunchKernelGGL(grad_stream_kernel<DT>, g.grid, dim3(256), 0, c.stream, c.acts, grads, coef, c.act_lens, \
                           c.label_lens, c.T, c.U, c.V, c.D, c.blank, L.CS, flags, g.BT, g.bt_chunk);               \
    }                                                                                                               \
  } while (0)
  const BlockPlan bp = grad_block_plan(c, grads);
#define LAUNCH_GRAD_BLOCK(DT, RT_, NVT_)                                                                            \
  do {                                                                                                              \
    if (fused)                                                                                                      \
      hipLaunchKernelGGL((grad_block_kernel<DT, RT_, NVT_, true>), plan_grid(c, bp), dim3(bp.threads()), 0, c.stream, \
                         c.acts, grads, coef, lv, c.act_lens, c.label_lens, c.T, c.U, c.V, c.D, c.blank, L.CS, flags, \
                         plan_chunks(c, bp), plan_blocks(c, bp), make_griddiv(plan_chunks(c, bp), c.T));                                                   \
    else                                                                                                            \
      hipLaunchKernelGGL((grad_block_kernel<DT, RT_, NVT_, false>), plan_grid(c, bp), dim3(bp.threads()), 0,        \
                         c.stream, c.acts, grads, coef, lv, c.act_lens, c.label_lens, c.T, c.U, c.V, c.D, c.blank,  \
                         L.CS, flags, plan_chunks(c, bp), plan_blocks(c, bp), make_griddiv(plan_chunks(c, bp), c.T));                                      \
  } while (0)
#define GRAD_BLOCK_F32(RT_, NVT_) LAUNCH_GRAD_BLOCK(MI_DTYPE_F32, RT_, NVT_)
#define GRAD_BLOCK_BF16(RT_, NVT_) LAUNCH_GRAD_BLOCK(MI_DTYPE_BF16, RT_, NVT_)
#define GRAD_BLOCK_F16(RT_, NVT_) LAUNCH_GRAD_BLOCK(MI_DTYPE_F16, RT_, NVT_)
  if (bp.RT) {
    if (c.dt == MI_DTYPE_F32) MI_FOR_GRAD_PLAN(bp, GRAD_BLOCK_F32);
    else if (c.dt == MI_DTYPE_BF16) MI_FOR_GRAD_PLAN(bp, GRAD_BLOCK_BF16);
    else MI_FOR_GRAD_PLAN(bp, GRAD_BLOCK_F16);
  } else if (c.dt == MI_DTYPE_F32) LAUNCH_GRAD(MI_DTYPE_F32);
  else if (c.dt == MI_DTYPE_BF16) LAUNCH_GRAD(MI_DTYPE_BF16);
  else LAUNCH_GRAD(MI_DTYPE_F16);
#undef GRAD_BLOCK_F32
#undef GRAD_BLOCK_BF16
#undef GRAD_BLOCK_F16
#undef LAUNCH_GRAD_BLOCK
#undef LAUNCH_GRAD
#undef LAUNCH_GRAD_ROWS
  return launch_status();
}

int run_rnnt_cells(const Common& c, const ScaleArg& sc, float lambda, float clamp) {
  const Layout& L = c.L;
  const long long cells = (long long)c.B * c.T * c.U;
  ProfScope prof(MI_PROFILE_CELL, c.stream);
  hipLaunchKernelGGL(rnnt_cell_kernel, dim3((unsigned)(L.ND * c.B)), dim3(L.Us), 0, c.stream, (const float*)(c.ws + L.off_denom),
                     (const float*)(c.ws + L.off_arcs), (const double*)(c.ws + L.off_alphas),
                     (const double*)(c.ws + L.off_betas), (const double*)(c.ws + L.off_ll), c.labels, c.act_lens,
                     c.label_lens, sc.ptr, sc.stride, sc.mul, (float*)(c.ws + L.off_coef), c.T, c.U, c.V, c.blank, L.ND,
                     L.Us, L.A, L.CS, lambda, clamp, cells);
  return launch_status();
}

int run_logprobs_export(const Common& c, float* target_scores, float* blank_scores) {
  const Layout& L = c.L;
  ProfScope prof(MI_PROFILE_CELL, c.stream);
  hipLaunchKernelGGL(logprobs_export_kernel, dim3((unsigned)(L.ND * c.B)), dim3(L.Us), 0, c.stream,
                     (const float*)(c.ws + L.off_arcs), c.act_lens, c.label_lens, target_scores, blank_scores, c.T,
                     c.U, L.ND, L.Us, L.A);
  return launch_status();
}

int run_logprobs_cells(const Common& c, const float* grad_target_scores, const float* grad_blank_scores) {
  const Layout& L = c.L;
  ProfScope prof(MI_PROFILE_CELL, c.stream);
  hipLaunchKernelGGL(logprobs_cell_kernel, dim3((unsigned)(L.ND * c.B)), dim3(L.Us), 0, c.stream,
                     (const float*)(c.ws + L.off_denom), (const float*)(c.ws + L.off_arcs), c.labels, c.act_lens,
                     c.label_lens, grad_target_scores, grad_blank_scores, (float*)(c.ws + L.off_coef), c.T, c.U, c.V,
                     c.blank, L.ND, L.Us, L.A, L.CS);
  return launch_status();
}

int run_tdt_cells(const Common& c, const ScaleArg& sc, float lambda, float clamp, const TdtParams& prm) {
  const Layout& L = c.L;
  const long long cells = (long long)c.B * c.T * c.U;
  ProfScope prof(MI_PROFILE_CELL, c.stream);
  hipLaunchKernelGGL(tdt_cell_kernel, dim3((unsigned)(L.ND * c.B)), dim3(L.Us), 0, c.stream, (const float*)(c.ws + L.off_denom),
                     (const float*)(c.ws + L.off_arcs), (const double*)(c.ws + L.off_alphas),
                     (const double*)(c.ws + L.off_betas), (const double*)(c.ws + L.off_ll), c.labels, c.act_lens,
                     c.label_lens, sc.ptr, sc.stride, sc.mul, (float*)(c.ws + L.off_coef), c.T, c.U, c.V, c.blank, L.ND,
                     L.Us, L.A, L.CS, lambda, clamp, cells, prm);
  return launch_status();
}

}  // namespace

// ----------------------------------------------------------------------------------------
// C ABI
int make_mb_params(int NB, const int32_t* durations, float sigma, MbParams* p) {
  if (NB < 0 || NB > MI_TRANSDUCER_MAX_BIG_BLANKS || (NB > 0 && !durations)) return MI_TRANSDUCER_INVALID_VALUE;
  p->NB = NB;
  p->sigma = sigma;
  int longest = 1;
  for (int i = 0; i < MI_TRANSDUCER_MAX_BIG_BLANKS; ++i) p->dur[i] = 0;
  for (int i = 0; i < NB; ++i) {
    if (durations[i] < 1 || durations[i] > MI_TRANSDUCER_MAX_BLANK_DURATION) return MI_TRANSDUCER_INVALID_VALUE;
    p->dur[i] = durations[i];
    longest = durations[i] > longest ? durations[i] : longest;
  }
  p->R = longest + 1;
  return MI_TRANSDUCER_SUCCESS;
}

int run_multiblank_lattice(const Common& c, float* costs, float lambda, int with_betas, const MbParams& prm) {
  const Layout& L = c.L;
  const float* arcs = (const float*)(c.ws + L.off_arcs);
  double* alphas = (double*)(c.ws + L.off_alphas);
  double* betas = (double*)(c.ws + L.off_betas);
  double* ll = (double*)(c.ws + L.off_ll);
  const unsigned grid = (unsigned)(with_betas ? 2 * c.B : c.B);
  const int nbc = prm.NB <= 1 ? 1 : (prm.NB <= 2 ? 2 : (prm.NB <= 4 ? 4 : 8));
  const size_t lds = (size_t)prm.R * (2 + nbc) * L.Us * sizeof(double);  // the alpha ring is the larger one
  ProfScope prof(MI_PROFILE_LATTICE, c.stream);
  if (lds > 160 * 1024) {  // the ring does not fit LDS: pull from global memory instead
    hipLaunchKernelGGL(multiblank_lattice_pull_kernel, dim3(grid), dim3(L.Us), 0, c.stream, arcs, alphas, betas, ll,
                       costs, c.act_lens, c.label_lens, c.T, c.U, L.ND, L.Us, L.A, cost_scale_of(lambda), with_betas,
                       prm);
    return launch_status();
  }
#define LAUNCH_MB_T(NN, TT)                                                                                         \
  do {                                                                                                              \
    if (lds > 48 * 1024 && hipFuncSetAttribute((const void*)multiblank_lattice_kernel<NN, TT>,                      \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) \
      return MI_TRANSDUCER_LAUNCH_FAILURE;                                                                          \
    hipLaunchKernelGGL((multiblank_lattice_kernel<NN, TT>), dim3(grid), dim3(L.Us), lds, c.stream, arcs, alphas,    \
                       betas, ll, costs, c.act_lens, c.label_lens, c.T, c.U, L.ND, L.Us, L.A,                       \
                       cost_scale_of(lambda), with_betas, prm);                                                     \
  } while (0)
#define LAUNCH_MB(NN)                     \
  do {                                    \
    if (L.Us <= 256) LAUNCH_MB_T(NN, 256); \
    else LAUNCH_MB_T(NN, 1024);           \
  } while (0)
  switch (nbc) {
    case 1: LAUNCH_MB(1); break;
    case 2: LAUNCH_MB(2); break;
    case 4: LAUNCH_MB(4); break;
    default: LAUNCH_MB(8); break;
  }
#undef LAUNCH_MB_T
#undef LAUNCH_MB
  return launch_status();
}

int run_multiblank_cells(const Common& c, const ScaleArg& sc, float lambda, float clamp, const MbParams& prm) {
  const Layout& L = c.L;
  const long long cells = (long long)c.B * c.T * c.U;
  ProfScope prof(MI_PROFILE_CELL, c.stream);
  hipLaunchKernelGGL(multiblank_cell_kernel, dim3((unsigned)(L.ND * c.B)), dim3(L.Us), 0, c.stream, (const float*)(c.ws + L.off_denom),
                     (const float*)(c.ws + L.off_arcs), (const double*)(c.ws + L.off_alphas),
                     (const double*)(c.ws + L.off_betas), (const double*)(c.ws + L.off_ll), c.labels, c.act_lens,
                     c.label_lens, sc.ptr, sc.stride, sc.mul, (float*)(c.ws + L.off_coef), c.T, c.U, c.V, c.blank, L.ND,
                     L.Us, L.A, L.CS, lambda, clamp, cells, prm);
  return launch_status();
}

int run_multiblank_fixup(const Common& c, void* grads, const MbParams& prm) {
  if (prm.NB == 0) return MI_TRANSDUCER_SUCCESS;
  const Layout& L = c.L;
  const long long cells = (long long)c.B * c.T * c.U;
  const unsigned grid = (unsigned)((cells * prm.NB + 255) / 256);
  const float* coef = (const float*)(c.ws + L.off_coef);
#define LAUNCH_FIX(DT)                                                                                             \
  hipLaunchKernelGGL(multiblank_fixup_kernel<DT>, dim3(grid), dim3(256), 0, c.stream, grads, coef, c.V, c.blank,    \
                     prm.NB, L.CS, cells)
  if (c.dt == MI_DTYPE_F32) LAUNCH_FIX(MI_DTYPE_F32);
  else if (c.dt == MI_DTYPE_BF16) LAUNCH_FIX(MI_DTYPE_BF16);
  else LAUNCH_FIX(MI_DTYPE_F16);
#undef LAUNCH_FIX
  return launch_status();
}

// ----------------------------------------------------------------------------------------
#include "mi_joint.inc"

extern "C" {

int mi_transducer_abi_version(void) { return 11; }

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
                     const int64_t* label_lens, void* grads, const float* grad_scale, int grad_scale_stride,
                     float grad_mul, int padding_zeroed, int B, int T, int U, int V, int blank,
                     float fastemit_lambda, float clamp, void* workspace, size_t workspace_bytes, void* stream) {
  Common c;
  if (!grads || clamp < 0.f || grad_scale_stride < 0) return MI_TRANSDUCER_INVALID_VALUE;
  int st = check_common(acts, act_dtype, labels, act_lens, label_lens, B, T, U, V, 0, blank, workspace,
                        workspace_bytes, stream, &c);
  if (st) return st;
  const ScaleArg sc = {grad_scale, grad_scale_stride, grad_mul};
  const bool fused = grad_rows_R(c, grads) != 0 || grad_block_plan(c, grads).RT != 0;
  if (!fused && (st = run_rnnt_cells(c, sc, fastemit_lambda, clamp))) return st;
  return run_grad_stream(c, grads, padding_zeroed ? kFlagPaddingDone : 0, fused, sc, fastemit_lambda, clamp);
}

int mi_rnnt_loss(const void* acts, int act_dtype, const int64_t* labels, const int64_t* act_lens,
                 const int64_t* label_lens, float* costs, void* grads, const float* grad_scale,
                 int grad_scale_stride, float grad_mul, int B, int T, int U, int V, int blank, float fastemit_lambda,
                 float clamp, void* workspace, size_t workspace_bytes, void* stream) {
  int st = mi_rnnt_forward(acts, act_dtype, labels, act_lens, label_lens, costs, B, T, U, V, blank, fastemit_lambda,
                           grads != nullptr, workspace, workspace_bytes, stream);
  if (st || !grads) return st;
  return mi_rnnt_backward(acts, act_dtype, labels, act_lens, label_lens, grads, grad_scale, grad_scale_stride,
                          grad_mul, 0, B, T, U, V, blank, fastemit_lambda, clamp, workspace, workspace_bytes, stream);
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
                    const int64_t* label_lens, void* grads, const float* grad_scale, int grad_scale_stride,
                    float grad_mul, int padding_zeroed, int B, int T, int U, int V, int D,
                    const int32_t* durations_host, int blank, float fastemit_lambda, float clamp, float sigma,
                    int use_plain_rnnt, void* workspace, size_t workspace_bytes, void* stream) {
  Common c;
  TdtParams prm;
  if (!grads || clamp < 0.f || grad_scale_stride < 0) return MI_TRANSDUCER_INVALID_VALUE;
  const int pad_flag = padding_zeroed ? kFlagPaddingDone : 0;
  int st = make_tdt_params(D, durations_host, sigma, &prm);
  if (st) return st;
  st = check_common(acts, act_dtype, labels, act_lens, label_lens, B, T, U, V, D, blank, workspace, workspace_bytes,
                    stream, &c);
  if (st) return st;
  const ScaleArg sc = {grad_scale, grad_scale_stride, grad_mul};
  if (use_plain_rnnt) {  // gpu_rnnt.py:646-682: token gradient from the RNNT kernel, duration gradient stays zero
    const bool fused = grad_rows_R(c, grads) != 0 || grad_block_plan(c, grads).RT != 0;
    if (!fused && (st = run_rnnt_cells(c, sc, fastemit_lambda, clamp))) return st;
    return run_grad_stream(c, grads, kFlagZeroDurations | pad_flag, fused, sc, fastemit_lambda, clamp);
  }
  if ((st = run_tdt_cells(c, sc, fastemit_lambda, clamp, prm))) return st;
  return run_grad_stream(c, grads, pad_flag, false, sc, fastemit_lambda, clamp);
}

int mi_tdt_loss(const void* acts, int act_dtype, const int64_t* labels, const int64_t* act_lens,
                const int64_t* label_lens, float* costs, void* grads, const float* grad_scale, int grad_scale_stride,
                float grad_mul, int B, int T, int U, int V, int D, const int32_t* durations_host, int blank,
                float fastemit_lambda, float clamp, float sigma, int use_plain_rnnt, void* workspace,
                size_t workspace_bytes, void* stream) {
  int st = mi_tdt_forward(acts, act_dtype, labels, act_lens, label_lens, costs, B, T, U, V, D, durations_host, blank,
                          fastemit_lambda, sigma, use_plain_rnnt, grads != nullptr, workspace, workspace_bytes, stream);
  if (st || !grads) return st;
  return mi_tdt_backward(acts, act_dtype, labels, act_lens, label_lens, grads, grad_scale, grad_scale_stride, grad_mul,
                         0, B, T, U, V, D, durations_host, blank, fastemit_lambda, clamp, sigma, use_plain_rnnt,
                         workspace, workspace_bytes, stream);
}

int mi_multiblank_forward(const void* acts, int act_dtype, const int64_t* labels, const int64_t* act_lens,
                          const int64_t* label_lens, float* costs, int B, int T, int U, int V, int num_big_blanks,
                          const int32_t* big_blank_durations_host, int blank, float fastemit_lambda, float sigma,
                          int with_betas, void* workspace, size_t workspace_bytes, void* stream) {
  Common c;
  MbParams prm;
  if (!costs) return MI_TRANSDUCER_INVALID_VALUE;
  int st = make_mb_params(num_big_blanks, big_blank_durations_host, sigma, &prm);
  if (st) return st;
  st = check_common(acts, act_dtype, labels, act_lens, label_lens, B, T, U, V, 0, blank, workspace, workspace_bytes,
                    stream, &c, num_big_blanks);
  if (st) return st;
  if ((st = run_denom(c))) return st;
  return run_multiblank_lattice(c, costs, fastemit_lambda, with_betas, prm);
}

int mi_multiblank_backward(const void* acts, int act_dtype, const int64_t* labels, const int64_t* act_lens,
                           const int64_t* label_lens, void* grads, const float* grad_scale, int grad_scale_stride,
                           float grad_mul, int B, int T, int U, int V, int num_big_blanks,
                           const int32_t* big_blank_durations_host, int blank, float fastemit_lambda, float clamp,
                           float sigma, void* workspace, size_t workspace_bytes, void* stream) {
  Common c;
  MbParams prm;
  if (!grads || clamp < 0.f || grad_scale_stride < 0) return MI_TRANSDUCER_INVALID_VALUE;
  int st = make_mb_params(num_big_blanks, big_blank_durations_host, sigma, &prm);
  if (st) return st;
  st = check_common(acts, act_dtype, labels, act_lens, label_lens, B, T, U, V, 0, blank, workspace, workspace_bytes,
                    stream, &c, num_big_blanks);
  if (st) return st;
  const ScaleArg sc = {grad_scale, grad_scale_stride, grad_mul};
  if ((st = run_multiblank_cells(c, sc, fastemit_lambda, clamp, prm))) return st;
  if ((st = run_grad_stream(c, grads, 0, false, sc, fastemit_lambda, clamp))) return st;
  return run_multiblank_fixup(c, grads, prm);
}

int mi_multiblank_loss(const void* acts, int act_dtype, const int64_t* labels, const int64_t* act_lens,
                       const int64_t* label_lens, float* costs, void* grads, const float* grad_scale,
                       int grad_scale_stride, float grad_mul, int B, int T, int U, int V, int num_big_blanks,
                       const int32_t* big_blank_durations_host, int blank, float fastemit_lambda, float clamp,
                       float sigma, void* workspace, size_t workspace_bytes, void* stream) {
  int st = mi_multiblank_forward(acts, act_dtype, labels, act_lens, label_lens, costs, B, T, U, V, num_big_blanks,
                                 big_blank_durations_host, blank, fastemit_lambda, sigma, grads != nullptr, workspace,
                                 workspace_bytes, stream);
  if (st || !grads) return st;
  return mi_multiblank_backward(acts, act_dtype, labels, act_lens, label_lens, grads, grad_scale, grad_scale_stride,
                                grad_mul, B, T, U, V, num_big_blanks, big_blank_durations_host, blank, fastemit_lambda,
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
  c.ws = (char*)workspace; c.stream = (hipStream_t)stream;
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
  c.ws = (char*)workspace; c.stream = (hipStream_t)stream;
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
  return MI_TRANSDUCER_SUCCESS;
}

int mi_transducer_profile_read(int kernel_id, float* total_ms, int* launches) {
  if (kernel_id < 0 || kernel_id >= MI_PROFILE_KERNELS || !total_ms || !launches) return MI_TRANSDUCER_INVALID_VALUE;
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
  else if (rows_R(c)) snprintf(denom, sizeof denom, "denom_rows_kernel<%s, R=%d>", dt, rows_R(c));
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
  const bool fused = !tdt && !mb && (gp.RT != 0 || rows_R(c) != 0);
  snprintf(cells, sizeof cells, "%s", fused ? "-" : (mb ? "multiblank_cell_kernel" : (tdt ? "tdt_cell_kernel" : "rnnt_cell_kernel")));
  if (gp.RT) snprintf(grad, sizeof grad, "grad_block_kernel<%s, RT=%d, NVT=%d, %s>", dt, gp.RT, gp.NVT, fused ? "fused" : "coef");
  else if (rows_R(c)) snprintf(grad, sizeof grad, "grad_rows_kernel<%s, R=%d, %s>", dt, rows_R(c), fused ? "fused" : "coef");
  else snprintf(grad, sizeof grad, "grad_stream_kernel<%s>", dt);
  const int n = snprintf(out, out_bytes, "denominators=%s; lattice=%s; cells=%s; gradient=%s%s", denom, lattice, cells,
                         grad, mb ? " + multiblank_fixup_kernel" : "");
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
