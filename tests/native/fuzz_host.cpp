// CPU-only sanitizer fuzz of the host code (built with -fsanitize=address,undefined by `make -C oracle asan`).
//   1. speech_amd/csrc/mi_plan.h: workspace layout, division constants, duration parameter blocks and kernel-shape
//      choices over random problem shapes, with the invariants the launchers rely on;
//   2. speech_amd/csrc/mi_cpu.cpp (the product's host RNNT loss) against oracle/transducer_cpu.c (the restated
//      reference CPU path) on random ragged batches, both compiled into this one instrumented binary, so every
//      index either of them forms is checked by the sanitizer.
// Usage: fuzz_host [iterations] [seed]; exit status 0 = no finding.
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <random>
#include <vector>

#include "../../speech_amd/csrc/mi_plan.h"
#include "../../speech_amd/csrc/mi_cpu.cpp"
extern "C" {
int oracle_rnnt_cpu_path_f64(const double* acts, const int64_t* labels, const int64_t* act_lens,
                             const int64_t* label_lens, int B, int T, int U, int V, int blank, double lambda,
                             double clamp, double* costs, double* grads, double* logp, double* work, int num_threads);
int oracle_rnnt_loss_f32(const float* acts, const int64_t* labels, const int64_t* act_lens, const int64_t* label_lens,
                         int B, int T, int U, int V, int blank, float lambda, float clamp, float* costs, float* grads,
                         float* denom, float* alphas, float* betas, float* llf, float* llb, int num_threads);
int oracle_tdt_loss_f32(const float* acts, const int64_t* labels, const int64_t* act_lens, const int64_t* label_lens,
                        int B, int T, int U, int V, int D, const int* durations, int blank, float sigma, float lambda,
                        float clamp, float* costs, float* grads, float* dgrads_lp, float* denom, float* dlp,
                        float* alphas, float* betas, float* llf, float* llb, int num_threads);
int oracle_multiblank_loss_f32(const float* acts, const int64_t* labels, const int64_t* act_lens,
                               const int64_t* label_lens, int B, int T, int U, int V, int NB, const int* durations,
                               int blank, float sigma, float lambda, float clamp, float* costs, float* grads,
                               float* denom, float* alphas, float* betas, float* llf, float* llb, int num_threads);
}

static int failures = 0;
#define EXPECT(cond, ...)                                  \
  do {                                                     \
    if (!(cond)) {                                         \
      ++failures;                                          \
      printf("FAIL %s:%d %s: ", __FILE__, __LINE__, #cond); \
      printf(__VA_ARGS__);                                 \
      printf("\n");                                        \
    }                                                      \
  } while (0)

static void fuzz_plan(std::mt19937& rng, int iterations) {
  auto uni = [&](int lo, int hi) { return std::uniform_int_distribution<int>(lo, hi)(rng); };
  for (int it = 0; it < iterations; ++it) {
    const int B = uni(-1, 70), T = uni(-1, 900), U = uni(-1, 1100), D = uni(-1, 18);
    Layout L;
    const bool ok = make_layout(B, T, U, D, &L);
    const bool want = B > 0 && T > 0 && U > 0 && D >= 0 && U <= MI_TRANSDUCER_MAX_U && D <= MI_TRANSDUCER_MAX_DURATIONS;
    EXPECT(ok == want, "B %d T %d U %d D %d", B, T, U, D);
    if (ok) {
      const size_t offs[] = {L.off_denom, L.off_arcs, L.off_alphas, L.off_betas, L.off_ll,
                             L.off_coef,  L.off_fill, L.total};
      for (int i = 0; i + 1 < 8; ++i) EXPECT(offs[i] < offs[i + 1] && (offs[i] & 255) == 0, "segment %d", i);
      EXPECT(L.Us >= U && L.Us == 64 * L.K && L.ND == T + U - 1 && L.A >= 2 + D && L.A == arc_record_floats(D) && (D == 0 ? L.A == 2 : L.A % 4 == 0 && L.A >= 3 + D && L.A < 3 + D + 4) && L.CS >= kCoefBase + D, "layout");
      const size_t cells = (size_t)B * T * U, skew = (size_t)B * L.ND * L.Us;
      EXPECT(L.off_arcs - L.off_denom >= cells * 4 && L.off_alphas - L.off_arcs >= skew * L.A * 4 &&
                 L.off_betas - L.off_alphas >= skew * 8 && L.off_ll - L.off_betas >= skew * 8 &&
                 L.off_coef - L.off_ll >= (size_t)B * 16 && L.off_fill - L.off_coef >= cells * L.CS * 4 &&
                 L.total - L.off_fill >= (size_t)kFillInts * 4,
             "segment sizes B %d T %d U %d D %d", B, T, U, D);
    }
    // rows per prefill item: a power of two up to eight, down to one for rows beyond 32 KB, never beyond 64 KB an item
    {
      const size_t row_bytes = (size_t)uni(1, 1 << uni(1, 18));
      const int lr = prefill_log_rows(row_bytes);
      EXPECT(lr >= 0 && lr <= 3 && (lr == 0 || (row_bytes << lr) <= 64 * 1024) &&
                 (lr == 3 || (row_bytes << (lr + 1)) > 64 * 1024),
             "prefill_log_rows(%zu) = %d", row_bytes, lr);
    }
    // division by multiply-shift: exact for every n < 2^31
    const unsigned d = (unsigned)uni(1, 1 << (uni(1, 30)));
    const FastDiv f = make_fastdiv(d);
    for (int k = 0; k < 16; ++k) {
      const unsigned n = (unsigned)uni(0, 0x7fffffff);
      const unsigned q = (unsigned)((((unsigned long long)n * f.mul) >> 32) + n) >> f.shift;
      EXPECT(q == n / d, "n %u d %u", n, d);
    }
    // duration blocks
    int32_t dur[MI_TRANSDUCER_MAX_DURATIONS + 2];
    const int nd = uni(0, MI_TRANSDUCER_MAX_DURATIONS + 1);
    int v = uni(0, 2);
    for (int i = 0; i < nd; ++i) { dur[i] = v; v += uni(0, 3); }
    TdtParams tp;
    const int st = make_tdt_params(nd, nd ? dur : nullptr, 0.05f, &tp);
    bool asc = nd >= 1 && nd <= MI_TRANSDUCER_MAX_DURATIONS;
    for (int i = 1; i < nd && asc; ++i) asc = dur[i] > dur[i - 1];
    const bool has_one = asc && (dur[0] == 1 || (nd > 1 && dur[1] == 1));
    EXPECT((st == MI_TRANSDUCER_SUCCESS) == (asc && has_one), "durations n %d first %d", nd, nd ? dur[0] : -1);
    if (st == MI_TRANSDUCER_SUCCESS) EXPECT(tp.R == dur[nd - 1] + 2 && tp.dur[tp.one_idx] == 1, "tdt params");
    MbParams mp;
    const int nbb = uni(0, MI_TRANSDUCER_MAX_BIG_BLANKS + 1);
    int32_t bd[MI_TRANSDUCER_MAX_BIG_BLANKS + 2];
    bool bd_ok = nbb <= MI_TRANSDUCER_MAX_BIG_BLANKS;
    int longest = 1;
    for (int i = 0; i < nbb; ++i) {
      bd[i] = uni(0, MI_TRANSDUCER_MAX_BLANK_DURATION + 2);
      if (i < MI_TRANSDUCER_MAX_BIG_BLANKS && (bd[i] < 1 || bd[i] > MI_TRANSDUCER_MAX_BLANK_DURATION)) bd_ok = false;
      if (bd[i] > longest) longest = bd[i];
    }
    const int ms = make_mb_params(nbb, bd, 0.f, &mp);
    EXPECT((ms == MI_TRANSDUCER_SUCCESS) == bd_ok, "big blanks n %d", nbb);
    if (ms == MI_TRANSDUCER_SUCCESS) EXPECT(mp.R == longest + 1, "ring depth");
    // kernel shapes: whatever is chosen must cover the row and fit a workgroup
    PlanShape s;
    s.dt = uni(0, 2); s.B = uni(1, 64); s.T = uni(1, 800); s.U = uni(1, 1024); s.V = uni(1, 70000); s.D = uni(0, 16);
    s.same_phase = uni(0, 3) != 0;
    const int nb = s.whole_vectors();
    const int r1 = denom_rows_R(s), r4 = grad_rows_R(s);
    if (r1) EXPECT(nb <= 64 * r1 && r1 <= 8 && r1 != 7, "denominator rows R %d nb %d", r1, nb);
    if (r4) EXPECT(nb <= 64 * r4 && s.same_phase, "gradient rows R %d nb %d", r4, nb);
    const BlockPlan dp = denom_block_plan(s), gp = grad_block_plan(s);
    if (dp.RT) EXPECT(dp.RT == 1024 && nb > 512 && nb <= dp.RT * dp.NVT && dp.NVT <= 8, "denominator block plan");
    if (gp.RT) {
      EXPECT(s.same_phase && nb > 64 && nb <= gp.RT * gp.NVT && gp.threads() <= 1024 && gp.rows() * gp.RT == gp.threads(),
             "gradient block plan RT %d NVT %d nb %d", gp.RT, gp.NVT, nb);
      EXPECT(2 * s.vec() + s.D <= 64, "head, tail and duration entries must fit one wave");
      EXPECT((long long)plan_chunks(s, gp) * gp.rows() >= s.U, "chunks cover U");
    }
    EXPECT(padded_grid(row_blocks(s, 1)) % (8u * MI_XCD_SPAN) == 0 && padded_grid(row_blocks(s, 1)) >= row_blocks(s, 1),
           "grid rounding");
  }
}

static void fuzz_cpu_loss(std::mt19937& rng, int iterations) {
  auto uni = [&](int lo, int hi) { return std::uniform_int_distribution<int>(lo, hi)(rng); };
  std::normal_distribution<float> normal(0.f, 2.f);
  for (int it = 0; it < iterations; ++it) {
    const int B = uni(1, 4), T = uni(1, 12), U = uni(1, 7), V = uni(1, 20), blank = uni(0, V - 1);
    const float lambda = uni(0, 1) ? 0.01f : 0.f, clamp = uni(0, 2) ? 0.f : 0.1f;
    const size_t n = (size_t)B * T * U * V;
    std::vector<float> x(n), g(n, NAN), costs(B, NAN);
    std::vector<double> xd(n), gd(n, 0.0), cd(B), logp(n), work((size_t)B * T * U * 4);
    for (size_t i = 0; i < n; ++i) xd[i] = x[i] = normal(rng);
    std::vector<int64_t> labels((size_t)B * (U > 1 ? U - 1 : 1)), al(B), ll(B);
    for (auto& v : labels) v = uni(0, V - 1);
    for (int b = 0; b < B; ++b) { al[b] = uni(1, T); ll[b] = uni(0, U - 1); }
    size_t ws_bytes = 0;
    EXPECT(mi_rnnt_cpu_workspace_bytes(B, T, U, &ws_bytes) == 0, "workspace size");
    std::vector<double> ws(ws_bytes / 8 + 1);
    const int64_t* lab = U > 1 ? labels.data() : nullptr;
    int st = mi_rnnt_cpu_forward(x.data(), lab, al.data(), ll.data(), costs.data(), B, T, U, V, blank, lambda, ws.data(),
                                 ws_bytes, uni(0, 3));
    EXPECT(st == 0, "forward status %d", st);
    st = mi_rnnt_cpu_backward(x.data(), lab, al.data(), ll.data(), g.data(), nullptr, 0, 1.f, B, T, U, V, blank, lambda,
                              clamp, 0, ws.data(), ws_bytes, uni(0, 3));
    EXPECT(st == 0, "backward status %d", st);
    st = oracle_rnnt_cpu_path_f64(xd.data(), labels.data(), al.data(), ll.data(), B, T, U, V, blank, lambda, clamp,
                                  cd.data(), gd.data(), logp.data(), work.data(), 1);
    EXPECT(st == 0, "oracle status %d", st);
    for (int b = 0; b < B; ++b)
      EXPECT(fabs(costs[b] - cd[b]) <= 1e-5 * fabs(cd[b]) + 1e-6, "cost %g vs %g (B %d T %d U %d V %d)", costs[b], cd[b], B, T, U, V);
    double worst = 0;
    for (size_t i = 0; i < n; ++i) worst = fmax(worst, fabs((double)g[i] - gd[i]));
    EXPECT(worst < 1e-5, "gradient differs by %g (B %d T %d U %d V %d blank %d)", worst, B, T, U, V, blank);
    // bad arguments are refused before anything is touched
    EXPECT(mi_rnnt_cpu_forward(x.data(), lab, al.data(), ll.data(), costs.data(), B, T, U, V, V, lambda, ws.data(), ws_bytes, 1) == 1, "blank >= V");
    EXPECT(mi_rnnt_cpu_forward(x.data(), lab, al.data(), ll.data(), costs.data(), B, T, U, V, blank, lambda, ws.data(), ws_bytes - 64, 1) == 1, "short workspace");
  }
}

// the other oracle entry points on random ragged shapes: no second implementation to compare with on the host, the
// sanitizer watches their indexing and the results must be finite where an alignment exists
static void fuzz_oracle(std::mt19937& rng, int iterations) {
  auto uni = [&](int lo, int hi) { return std::uniform_int_distribution<int>(lo, hi)(rng); };
  std::normal_distribution<float> normal(0.f, 1.5f);
  for (int it = 0; it < iterations; ++it) {
    const int B = uni(1, 3), T = uni(1, 10), U = uni(1, 6), NB = uni(0, 3), D = uni(1, 4);
    const int Vt = uni(1, 12);
    std::vector<int64_t> labels((size_t)B * (U > 1 ? U - 1 : 1)), al(B), ll(B);
    for (auto& v : labels) v = uni(0, Vt - 1);
    for (int b = 0; b < B; ++b) { al[b] = uni(1, T); ll[b] = uni(0, U - 1); }
    const size_t cells = (size_t)B * T * U;
    std::vector<float> denom(cells), alphas(cells), betas(cells), llf(B), llb(B), costs(B);
    {  // RNNT, GPU-path semantics
      const int V = Vt + 1;
      std::vector<float> x(cells * V), g(cells * V, 0.f);
      for (auto& v : x) v = normal(rng);
      EXPECT(oracle_rnnt_loss_f32(x.data(), labels.data(), al.data(), ll.data(), B, T, U, V, V - 1, 0.01f, 0.f, costs.data(),
                                  g.data(), denom.data(), alphas.data(), betas.data(), llf.data(), llb.data(), 2) == 0, "rnnt");
      for (int b = 0; b < B; ++b) EXPECT(std::isfinite(costs[b]) && fabsf(llf[b] - llb[b]) < 1e-3f * fabsf(llf[b]) + 1e-4f, "rnnt ll");
    }
    {  // TDT with durations 0 .. D-1 (or 1 .. D): combined logits
      const int V = Vt + 1, first = D > 1 ? uni(0, 1) : 1;
      std::vector<int> dur(D);
      for (int i = 0; i < D; ++i) dur[i] = first + i;
      std::vector<float> x(cells * (V + D)), g(cells * (V + D), 0.f), dg(cells * D, 0.f), dlp(cells * D);
      for (auto& v : x) v = normal(rng);
      EXPECT(oracle_tdt_loss_f32(x.data(), labels.data(), al.data(), ll.data(), B, T, U, V, D, dur.data(), V - 1, 0.05f, 0.f,
                                 0.f, costs.data(), g.data(), dg.data(), denom.data(), dlp.data(), alphas.data(), betas.data(),
                                 llf.data(), llb.data(), 2) == 0, "tdt");
      for (int b = 0; b < B; ++b) EXPECT(!std::isnan(costs[b]), "tdt cost");
    }
    {  // multi-blank: tokens, NB big blanks, the standard blank
      const int V = Vt + NB + 1;
      std::vector<int> dur(NB ? NB : 1);
      for (int i = 0; i < NB; ++i) dur[i] = uni(2, 5);
      std::vector<float> x(cells * V), g(cells * V, 0.f);
      for (auto& v : x) v = normal(rng);
      EXPECT(oracle_multiblank_loss_f32(x.data(), labels.data(), al.data(), ll.data(), B, T, U, V, NB, dur.data(), V - 1,
                                        0.05f, 0.01f, 0.f, costs.data(), g.data(), denom.data(), alphas.data(), betas.data(),
                                        llf.data(), llb.data(), 2) == 0, "multiblank");
      for (int b = 0; b < B; ++b) EXPECT(std::isfinite(costs[b]), "multiblank cost");
    }
  }
}

int main(int argc, char** argv) {
  const int iterations = argc > 1 ? atoi(argv[1]) : 2000;
  std::mt19937 rng(argc > 2 ? (unsigned)atoi(argv[2]) : 1u);
  fuzz_plan(rng, iterations * 10);
  fuzz_cpu_loss(rng, iterations);
  fuzz_oracle(rng, iterations / 4);
  printf("fuzz_host: %d plan shapes, %d loss batches, %d failure(s)\n", iterations * 10, iterations, failures);
  return failures ? 1 : 0;
}
