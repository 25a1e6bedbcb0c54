"""CPU oracle package -- TEST INFRASTRUCTURE ONLY.

Importable from tests/, from __graft_entry__.smoke() and from bench.py's
cpu_baseline leg; the shipped package (speech_amd) must never import it.

`transducer_numpy` is the slow, loop-level restatement; this module wraps the
C restatement (oracle/transducer_cpu.c) with numpy in / numpy out.
"""

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle_transducer.so")
_lib = None


def build(force=False):
    """Compile the C oracle with the Makefile beside it."""
    if force:
        subprocess.run(["make", "-C", _HERE, "clean"], check=True, capture_output=True)
    subprocess.run(["make", "-C", _HERE], check=True, capture_output=True)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
    return _lib


def _ptr(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _prep(acts, labels, act_lens, label_lens, dtype):
    acts = np.ascontiguousarray(acts, dtype=dtype)
    labels = np.ascontiguousarray(labels, dtype=np.int64)
    act_lens = np.ascontiguousarray(act_lens, dtype=np.int64)
    label_lens = np.ascontiguousarray(label_lens, dtype=np.int64)
    B, T, U = acts.shape[:3]
    if labels.shape != (B, U - 1):
        padded = np.zeros((B, max(U - 1, 0)), dtype=np.int64)
        padded[:, : labels.shape[1]] = labels[:, : U - 1]
        labels = padded
    return acts, labels, act_lens, label_lens


def _real(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float32:
        return "f32", ctypes.c_float
    if dtype == np.float64:
        return "f64", ctypes.c_double
    raise TypeError(dtype)


def rnnt_loss(
    acts, labels, act_lens, label_lens, blank, fastemit_lambda=0.0, clamp=0.0, dtype=np.float64, want_grads=True, num_threads=1
):
    """GPU-path semantics.  Returns (costs, grads or None, extras)."""
    suf, creal = _real(dtype)
    acts, labels, act_lens, label_lens = _prep(acts, labels, act_lens, label_lens, dtype)
    B, T, U, V = acts.shape
    costs = np.zeros(B, dtype=dtype)
    grads = np.zeros_like(acts) if want_grads else None
    denom = np.zeros((B, T, U), dtype=dtype)
    alphas = np.full((B, T, U), -np.inf, dtype=dtype)
    betas = np.full((B, T, U), -np.inf, dtype=dtype)
    llf = np.zeros(B, dtype=dtype)
    llb = np.zeros(B, dtype=dtype)
    fn = getattr(lib(), "oracle_rnnt_loss_" + suf)
    fn.restype = ctypes.c_int
    status = fn(
        _ptr(acts), _ptr(labels), _ptr(act_lens), _ptr(label_lens),
        ctypes.c_int(B), ctypes.c_int(T), ctypes.c_int(U), ctypes.c_int(V), ctypes.c_int(blank),
        creal(fastemit_lambda), creal(clamp),
        _ptr(costs), _ptr(grads), _ptr(denom), _ptr(alphas), _ptr(betas), _ptr(llf), _ptr(llb),
        ctypes.c_int(num_threads),
    )  # fmt: skip
    if status != 0:
        raise RuntimeError("oracle_rnnt_loss: invalid value")
    return costs, grads, dict(denom=denom, alphas=alphas, betas=betas, ll_forward=llf, ll_backward=llb)


def rnnt_cpu_path(acts, labels, act_lens, label_lens, blank, fastemit_lambda=0.0, clamp=0.0, dtype=np.float32, num_threads=1):
    """The reference's CPU path end to end.  Returns (costs, grads)."""
    suf, creal = _real(dtype)
    acts, labels, act_lens, label_lens = _prep(acts, labels, act_lens, label_lens, dtype)
    B, T, U, V = acts.shape
    costs = np.zeros(B, dtype=dtype)
    grads = np.zeros_like(acts)
    logp = np.empty_like(acts)
    work = np.zeros(B * T * U * 4, dtype=dtype)
    fn = getattr(lib(), "oracle_rnnt_cpu_path_" + suf)
    fn.restype = ctypes.c_int
    status = fn(
        _ptr(acts), _ptr(labels), _ptr(act_lens), _ptr(label_lens),
        ctypes.c_int(B), ctypes.c_int(T), ctypes.c_int(U), ctypes.c_int(V), ctypes.c_int(blank),
        creal(fastemit_lambda), creal(clamp),
        _ptr(costs), _ptr(grads), _ptr(logp), _ptr(work), ctypes.c_int(num_threads),
    )  # fmt: skip
    if status != 0:
        raise RuntimeError("oracle_rnnt_cpu_path: invalid value")
    return costs, grads


def tdt_loss(
    acts, labels, act_lens, label_lens, blank, durations, sigma=0.0, fastemit_lambda=0.0, clamp=0.0,
    dtype=np.float64, want_grads=True, num_threads=1,
):  # fmt: skip
    """TDT, GPU-path semantics, combined [B,T,U,V+D] logits in and gradient out."""
    suf, creal = _real(dtype)
    acts, labels, act_lens, label_lens = _prep(acts, labels, act_lens, label_lens, dtype)
    durations = np.ascontiguousarray(durations, dtype=np.int32)
    D = int(durations.shape[0])
    B, T, U, VD = acts.shape
    V = VD - D
    costs = np.zeros(B, dtype=dtype)
    grads = np.zeros_like(acts) if want_grads else None
    dgrads_lp = np.zeros((B, T, U, D), dtype=dtype) if want_grads else None
    denom = np.zeros((B, T, U), dtype=dtype)
    dlp = np.zeros((B, T, U, D), dtype=dtype)
    alphas = np.full((B, T, U), -np.inf, dtype=dtype)
    betas = np.full((B, T, U), -np.inf, dtype=dtype)
    llf = np.zeros(B, dtype=dtype)
    llb = np.zeros(B, dtype=dtype)
    fn = getattr(lib(), "oracle_tdt_loss_" + suf)
    fn.restype = ctypes.c_int
    status = fn(
        _ptr(acts), _ptr(labels), _ptr(act_lens), _ptr(label_lens),
        ctypes.c_int(B), ctypes.c_int(T), ctypes.c_int(U), ctypes.c_int(V), ctypes.c_int(D), _ptr(durations),
        ctypes.c_int(blank), creal(sigma), creal(fastemit_lambda), creal(clamp),
        _ptr(costs), _ptr(grads), _ptr(dgrads_lp), _ptr(denom), _ptr(dlp), _ptr(alphas), _ptr(betas),
        _ptr(llf), _ptr(llb), ctypes.c_int(num_threads),
    )  # fmt: skip
    if status != 0:
        raise RuntimeError("oracle_tdt_loss: invalid value")
    extras = dict(
        denom=denom, dlp=dlp, alphas=alphas, betas=betas, ll_forward=llf, ll_backward=llb, duration_grads=dgrads_lp
    )
    return costs, grads, extras


def multiblank_loss(
    acts, labels, act_lens, label_lens, blank, big_blank_durations, sigma=0.0, fastemit_lambda=0.0, clamp=0.0,
    dtype=np.float64, want_grads=True, num_threads=1,
):  # fmt: skip
    """Multi-blank transducer, GPU-path semantics.  Returns (costs, grads or None, extras)."""
    suf, creal = _real(dtype)
    acts, labels, act_lens, label_lens = _prep(acts, labels, act_lens, label_lens, dtype)
    durations = np.ascontiguousarray(big_blank_durations, dtype=np.int32)
    NB = int(durations.shape[0])
    B, T, U, V = acts.shape
    costs = np.zeros(B, dtype=dtype)
    grads = np.zeros_like(acts) if want_grads else None
    denom = np.zeros((B, T, U), dtype=dtype)
    alphas = np.full((B, T, U), -np.inf, dtype=dtype)
    betas = np.full((B, T, U), -np.inf, dtype=dtype)
    llf = np.zeros(B, dtype=dtype)
    llb = np.zeros(B, dtype=dtype)
    fn = getattr(lib(), "oracle_multiblank_loss_" + suf)
    fn.restype = ctypes.c_int
    status = fn(
        _ptr(acts), _ptr(labels), _ptr(act_lens), _ptr(label_lens),
        ctypes.c_int(B), ctypes.c_int(T), ctypes.c_int(U), ctypes.c_int(V), ctypes.c_int(NB),
        _ptr(durations) if NB else None, ctypes.c_int(blank), creal(sigma), creal(fastemit_lambda), creal(clamp),
        _ptr(costs), _ptr(grads), _ptr(denom), _ptr(alphas), _ptr(betas), _ptr(llf), _ptr(llb),
        ctypes.c_int(num_threads),
    )  # fmt: skip
    if status != 0:
        raise RuntimeError("oracle_multiblank_loss: invalid value")
    return costs, grads, dict(denom=denom, alphas=alphas, betas=betas, ll_forward=llf, ll_backward=llb)


def rnnt_logprobs(logits, targets, blank, source_lens=None, target_lens=None):
    """Compact log-prob op, forward (numpy restatement; see transducer_numpy.rnnt_logprobs)."""
    from oracle import transducer_numpy

    return transducer_numpy.rnnt_logprobs(logits, targets, blank, source_lens, target_lens)


def rnnt_logprobs_grad(logits, targets, blank, grad_target_scores, grad_blank_scores, source_lens=None, target_lens=None):
    """Compact log-prob op, backward (numpy restatement; see transducer_numpy.rnnt_logprobs_grad)."""
    from oracle import transducer_numpy

    return transducer_numpy.rnnt_logprobs_grad(
        logits, targets, blank, grad_target_scores, grad_blank_scores, source_lens, target_lens
    )


def joint_rnnt_loss(f, g, weight, bias, labels, act_lens, label_lens, blank, fastemit_lambda=0.0, clamp=0.0, grad_costs=None,
                    keep_mask=None, dropout_p=0.0, durations=None, sigma=0.0, big_blank_durations=None,
                    activation="relu"):
    """Joint network + RNNT / TDT / multi-blank loss (numpy restatement; see transducer_numpy.joint_rnnt_loss)."""
    from oracle import transducer_numpy

    return transducer_numpy.joint_rnnt_loss(
        f, g, weight, bias, labels, act_lens, label_lens, blank, fastemit_lambda, clamp, grad_costs, keep_mask, dropout_p,
        durations, sigma, big_blank_durations, activation,
    )
