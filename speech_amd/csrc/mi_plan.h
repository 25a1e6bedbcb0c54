// mi_plan.h -- the host-side planning of the transducer-loss library: workspace layout, division constants,
// duration parameter blocks and the choice of kernel shape per problem shape.  Plain C++ with no HIP types, so that a
// CPU-only sanitizer build can exercise it (tests/native/fuzz_host.cpp); mi_transducer.hip includes it inside its
// anonymous namespace, ahead of the device code that uses these types.
#ifndef MI_PLAN_H_
#define MI_PLAN_H_

#include <stddef.h>
#include <stdint.h>

#include "mi_transducer.h"

constexpr int kCoefBase = 8;  // floats per cell in the coefficient buffer before the duration-gradient block
// The prefill segment of the workspace, in ints.  While a lattice kernel runs, HBM idles; "riders" (extra workgroups
// of the same launch) zero-fill the padded cells of the gradient meanwhile, as far as they get.
//   [0, kFillMaxLattice)                  per lattice workgroup: (epoch << 13) | (id of the compute unit it runs on + 1)
//   [kFillMaxLattice, 2*kFillMaxLattice)  per lattice workgroup: the epoch, once it has finished
//   [2*kFillMaxLattice, + kFillMaxRiders) per virtual rider: how many of its items have been filled
// An item is 2^prefill_log_rows rows of one frame (b, t), items are numbered in memory order, and item i is the
// (i / kFillMaxRiders)-th item of virtual rider i % kFillMaxRiders: it is done iff  i / kFillMaxRiders <
// progress[i % kFillMaxRiders].  A launch has a power of two of real riders, each standing for the virtual riders
// congruent to it.  Pass 1 clears the whole segment, and the first two blocks are stamped with an epoch that changes
// with every call, so what an earlier call left there is not mistaken for this call's -- also not in a captured
// graph, where the epoch is frozen -- and a record that no rider of this call wrote says that nothing is filled.
constexpr int kFillMaxLattice = 256;
constexpr int kFillMaxRiders = 4096;
constexpr int kFillProgress = 2 * kFillMaxLattice;
constexpr int kFillInts = kFillProgress + kFillMaxRiders;
constexpr int kFillLogRowsShift = 8;  // the gradient kernels find log2(rows per item) in these bits of `flags`
// Rows per item: eight (no workgroup of the gradient pass spans more rows, and none straddles a multiple of eight),
// fewer for long rows, so that a rider looks at the lattice's state every 64 KB or so
inline int prefill_log_rows(size_t row_bytes) {
  int log_rows = 3;
  while (log_rows > 0 && (row_bytes << log_rows) > 64 * 1024) --log_rows;
  return log_rows;
}

// ----------------------------------------------------------------------------------------
// Workspace layout
// ----------------------------------------------------------------------------------------
// A cell's arc log-probs are one record of consecutive floats -- blank, label, then the `extras` duration (TDT) or
// big-blank (multi-blank) log-probs -- so that the pass that forms them writes them with one store: 2 floats, or,
// when there are extras, a multiple of 4 (whole 16-byte pieces) whose LAST float is the cell's log-softmax
// denominator (the cell kernels of those losses read it there, and the pass saves the store into `denom`).
constexpr int arc_record_floats(int extras) { return extras <= 0 ? 2 : (3 + extras + 3) / 4 * 4; }

struct Layout {
  int K;    // lattice cells per lane (1,2,4,8,16)
  int Us;   // pitch of a skewed lattice row = 64*K >= U
  int ND;   // number of anti-diagonals of the padded lattice = T+U-1
  int A;    // floats of a cell's record of arc log-probs (arc_record_floats); a skewed row holds Us records
  int CS;   // floats per cell in the coefficient buffer
  size_t off_denom, off_arcs, off_alphas, off_betas, off_ll, off_coef, off_fill, total;
};

inline size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

inline bool make_layout(int B, int T, int U, int D, Layout* L) {
  if (B <= 0 || T <= 0 || U <= 0 || D < 0 || U > MI_TRANSDUCER_MAX_U || D > MI_TRANSDUCER_MAX_DURATIONS) return false;
  int K = 1;
  while (64 * K < U) K *= 2;
  L->K = K;
  L->Us = 64 * K;
  L->ND = T + U - 1;
  L->A = arc_record_floats(D);
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
  L->off_fill = off;   off = align256(off + (size_t)kFillInts * sizeof(int));
  L->total = off;
  return true;
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
// the two divisions that split a workgroup id into (b, t, chunk), in three words (the shifts share one): this block
// is among the kernel arguments that arrive in registers with the wave, where every word counts
struct GridDiv {
  unsigned mul_chunks, mul_T, shifts;  // shifts = shift of the division by nchunks | shift of the division by T << 8
};
inline FastDiv griddiv_chunks(const GridDiv& g) { return FastDiv{g.mul_chunks, g.shifts & 255u}; }
inline FastDiv griddiv_frames(const GridDiv& g) { return FastDiv{g.mul_T, g.shifts >> 8}; }
inline GridDiv make_griddiv(int nchunks, int T) {
  const FastDiv c = make_fastdiv((unsigned)nchunks), t = make_fastdiv((unsigned)T);
  return GridDiv{c.mul, t.mul, c.shift | (t.shift << 8)};
}


// Consecutive workgroups that one XCD takes per turn (logical_block, mi_device.inc).  Measured on the fwd+bwd step
// with riders (us; B=16, T=375, U=121, V=1025 fp32 / the same as TDT / as multi-blank / B=32, T=750, U=201 bf16 /
// V=16385): 512 -> 1110 / 1181 / 1110 / 3845 / 4996; 1024 -> 1116 / 1186 / 1125 / 3880 / 4990; at the first shape
// 32, 128, 256, 384, 640, 768, 2048, 4096 -> 1123, 1120, 1117, 1115, 1117, 1115, 1133, 1152 (long turns leave XCDs
// idle where an utterance's padding begins; short ones lose the linear walk).
#ifndef MI_XCD_SPAN
#define MI_XCD_SPAN 512
#endif
// The gradient pass over 16-bit rows wants shorter turns (its workgroups hold four rows of 2 KB where the fp32 ones
// hold two of 4 KB): B=32, T=750, U=201, V=1025 bf16: 32 / 64 / 128 / 256 / 512 -> 2556 / 2536 / 2547 / 2575 / 2601 us
// (step 3.76 against 3.83 ms); B=16, T=375, U=121 bf16: 361 / 360 / 359 / 363 / 378 us; the fp32 shapes all lose below
// 512 (T=750, U=201 fp32: 5413 / 5476 / 5328 us at 128 / 256 / 512).  Pass 1 does not care (1038 ... 1043 us).
// MI_XCD_SPAN is a multiple of it (grids are padded to a multiple of 8 * MI_XCD_SPAN).
#ifndef MI_XCD_SPAN_16
#define MI_XCD_SPAN_16 128
#endif
static_assert(MI_XCD_SPAN % MI_XCD_SPAN_16 == 0, "one grid padding must serve both turn lengths");

struct TdtParams {
  int D;
  int dur[MI_TRANSDUCER_MAX_DURATIONS];
  int one_idx;  // index of duration 1 (position 0 or 1)
  int R;        // ring depth
  float sigma;
};


struct MbParams {
  int NB;
  int dur[MI_TRANSDUCER_MAX_BIG_BLANKS];
  int R;  // ring depth: longest blank + 1
  float sigma;
};


inline int make_tdt_params(int D, const int32_t* durations, float sigma, TdtParams* p) {
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


inline int make_mb_params(int NB, const int32_t* durations, float sigma, MbParams* p) {
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


// ----------------------------------------------------------------------------------------
// Kernel shape per problem shape.  The shape of a call as far as these choices go: logit dtype, tokens per row,
// extra row entries (TDT durations), lattice dimensions, and whether logits and gradients share their 16-byte phase.
// ----------------------------------------------------------------------------------------
struct PlanShape {
  int dt, B, T, U, V, D;
  bool same_phase;
  int vec() const { return dt == MI_DTYPE_F32 ? 4 : 8; }  // elements per 16-byte vector
  int whole_vectors() const { return V / vec(); }
};

#ifndef MI_USE_ROWS
#define MI_USE_ROWS 1
#endif
#ifndef MI_USE_BLOCK_ROWS
#define MI_USE_BLOCK_ROWS 1
#endif
#ifndef MI_ROW_WAVES
#define MI_ROW_WAVES 4
#endif
constexpr int kRowWaves = MI_ROW_WAVES;  // waves (= rows in flight) per workgroup of the row kernels

// smallest R in {1,2,4,8} with floor(V / VEC) <= 64*R, or 0 if the rows are too long for the
// register-resident kernels
inline int rows_R(const PlanShape& s) {
  if (!MI_USE_ROWS) return 0;
  const int nb = s.whole_vectors();
  for (int r = 1; r <= 8; r *= 2)
    if (nb <= 64 * r) return r;
  return 0;
}
// The denominator pass may take R = 3, 5, 6 as well: a vocabulary just past a power of two -- 1024 tokens, the
// blank and three big blanks are 257 vectors -- then costs 5 vector loads per lane, not 8.
inline int denom_rows_R(const PlanShape& s) {
  if (!MI_USE_ROWS) return 0;
  const int nb = s.whole_vectors();
  for (int r = 1; r <= 8; ++r)
    if (r != 7 && nb <= 64 * r) return r;
  return 0;
}
// the row kernels store gradient vectors at the 16-byte phase of the logits row
inline int grad_rows_R(const PlanShape& s) { return s.same_phase ? rows_R(s) : 0; }

// Workgroup-per-row kernels: RT threads per row, NVT vectors per thread.  RT == 0: not applicable.
// The denominator pass uses them for rows too long for the register-resident wave-per-row
// kernels (more than 512 whole vectors).  The gradient pass uses them from 65 vectors up, with
// two vectors per thread where the row allows it: of the splits tried (1, 2 and 4 vectors per
// thread) that one streams fastest.
struct BlockPlan {
  int RT, NVT;
  int rows() const { return (RT < 256 ? 256 : RT) / RT; }
  int threads() const { return RT < 256 ? 256 : RT; }
};
inline bool block_rows_ok(const PlanShape& s) { return MI_USE_BLOCK_ROWS && 2 * s.vec() + s.D <= 64; }
inline BlockPlan denom_block_plan(const PlanShape& s) {
  const int nb = s.whole_vectors();
  if (!block_rows_ok(s) || nb <= 512) return BlockPlan{0, 0};
  for (int nvt = 1; nvt <= 8; nvt *= 2)
    if (nb <= 1024 * nvt) return BlockPlan{1024, nvt};
  return BlockPlan{0, 0};
}
inline BlockPlan grad_block_plan(const PlanShape& s) {
  const int nb = s.whole_vectors();
  if (!s.same_phase || !block_rows_ok(s) || nb <= 64) return BlockPlan{0, 0};
  for (int rt = 64; rt <= 1024; rt *= 2) {
    if (nb <= 2 * rt) return BlockPlan{rt, 2};
    // a row just past 2*rt vectors (1024 tokens + blank + big blanks = 257): a third, partly filled vector per
    // thread beats twice the threads with half of them idle -- measured up to about 2.5*rt (V = 1028 ... 2600);
    // towards 3*rt the wider workgroup wins again
    if (nb <= 2 * rt + rt / 2) return BlockPlan{rt, 3};
  }
  for (int nvt = 4; nvt <= 8; nvt *= 2)
    if (nb <= 1024 * nvt) return BlockPlan{1024, nvt};
  return BlockPlan{0, 0};
}
// 1-D grids are rounded up to a whole number of turns of the XCD permutation
inline unsigned padded_grid(long long blocks) {
  const long long turn = 8LL * MI_XCD_SPAN;
  return (unsigned)((blocks + turn - 1) / turn * turn);
}
inline int plan_chunks(const PlanShape& s, const BlockPlan& p) { return (s.U + p.rows() - 1) / p.rows(); }
inline long long plan_blocks(const PlanShape& s, const BlockPlan& p) { return (long long)plan_chunks(s, p) * s.B * s.T; }
// the row kernels: a workgroup takes kRowWaves * rpw consecutive rows of one (b,t)
inline int row_chunks(const PlanShape& s, int rpw) { return (s.U + kRowWaves * rpw - 1) / (kRowWaves * rpw); }
inline long long row_blocks(const PlanShape& s, int rpw) { return (long long)row_chunks(s, rpw) * s.B * s.T; }

#endif  // MI_PLAN_H_
