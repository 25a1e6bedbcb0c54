/* CPU oracle for the RNNT / TDT transducer loss -- TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C restatement of the reference's algorithm, in the reference's own
 * order of floating-point operations, instantiated once in float (what the
 * reference computes in) and once in double (what the mathematics fixes).
 * Only tests, the smoke check and the benchmark's cpu_baseline leg may load
 * the library built from this file; the shipped package never does.
 *
 *   oracle_rnnt_loss_{f32,f64}      GPU-path semantics (logits in, denominator +
 *                                   alpha/beta + dense logits-gradient)
 *   oracle_rnnt_cpu_path_{f32,f64}  the reference's CPU path end to end (log_softmax,
 *                                   sparse log-prob gradient, softmax Jacobian, clamp hook);
 *                                   this is the timed CPU baseline
 *   oracle_tdt_loss_{f32,f64}       TDT, GPU-path semantics (the reference has no CPU TDT)
 *   oracle_multiblank_loss_{f32,f64}  multi-blank transducer, GPU-path semantics (no CPU path
 *                                   in the reference either)
 *
 * Pinning: every entry point is checked against the reference's golden vectors
 * and against oracle/transducer_numpy.py, brute-force path enumeration and torch
 * autograd in tests/test_oracle_*.py.  TDT with FastEmit has no reference vector:
 * it is checked only against the sparse-posterior identity ("derived").  The reference holds no
 * vector for the multi-blank loss: it is pinned by the RNNT vectors (no big blank, sigma 0),
 * path enumeration and autograd; its FastEmit terms are "derived" too.
 *
 * Build: make -C oracle   (gcc -O2 -fopenmp, no fast-math so the operation order stands)
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>

#define REAL float
#define SUF(name) name##_f32
#define R_EXP expf
#define R_LOG logf
#define R_LOG1P log1pf
#define COST_SCALE(l) (1.0f + (float)(l))
#include "transducer_cpu_impl.inc"
#undef REAL
#undef SUF
#undef R_EXP
#undef R_LOG
#undef R_LOG1P
#undef COST_SCALE

#define REAL double
#define SUF(name) name##_f64
#define R_EXP exp
#define R_LOG log
#define R_LOG1P log1p
#define COST_SCALE(l) (1.0 + (double)(l))
#include "transducer_cpu_impl.inc"
#undef REAL
#undef SUF
#undef R_EXP
#undef R_LOG
#undef R_LOG1P
#undef COST_SCALE

int oracle_abi_version(void) { return 1; }
