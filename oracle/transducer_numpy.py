"""CPU oracle for the RNNT / TDT transducer loss -- TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package may import this module.  It is a plain
numpy restatement (per-cell Python loops, float64 by default) of what the
reference computes on its GPU path, written from the recursions and not from
the reference source.  Each function names the reference lines it restates
(paths relative to nemo/collections/asr/parts/numba/rnnt_loss/).

How each function is pinned (tests/test_oracle_*.py):
  denominator       closed form -logsumexp (scipy) .................. pinned
  lse2              reference KAT log_sum_exp(0,1)*8=10.5060935 ...... pinned
  rnnt_*            reference golden vectors small / small_blank_last /
                    medium (cost + full gradient), clamp vector,
                    FastEmit cost scaling, brute-force path enumeration,
                    torch autograd of an alpha-only recursion ........ pinned
  tdt_*             reference fixed vector (cost 4.155739 + 42 grads),
                    brute-force (token,duration) path enumeration,
                    torch autograd, T=1 and U=1 closed forms ......... pinned
  tdt_* FastEmit    no reference vector or test exists for TDT with
                    fastemit_lambda > 0; pinned by what the kernel's terms
                    (gpu_rnnt_kernel.py:1353-1437) mean: the gradient of the
                    label arcs' log-probs x (1+lambda) through the token
                    softmax Jacobian, the duration branch untouched --
                    tests/helpers.py differentiates exactly that with torch
                    autograd, independently of the restated terms, and
                    test_oracle_tdt.py::test_fastemit_by_definition holds the
                    restatement to it at 1e-10 (a dropped sigma, a wrong beta
                    index or FastEmit leaking into the durations fails it)
                    .............................................. pinned
  multiblank_*      the reference holds no vector (its test compares two of
                    its own implementations on random input); with no big
                    blank and sigma = 0 it must give the RNNT golden vectors,
                    brute-force enumeration of every (token, blank-duration)
                    path, torch autograd of an alpha-only recursion,
                    llForward == beta(0,0) ........................... pinned
  multiblank_* FastEmit  likewise no reference vector; pinned by the
                    meaning of gpu_rnnt_kernel.py:727-885 (label-arc gradient
                    x (1+lambda), blank and big-blank arcs untouched), as
                    for TDT (tests/test_oracle_multiblank.py) ......... pinned
  joint_rnnt_loss   torch autograd (float64) through relu, linear and an
                    alpha-only recursion, with the bf16 roundings applied
                    straight-through; the loss part is rnnt_loss above;
                    with durations / big blanks: torch autograd of relu and
                    linear fed with the logits-gradient of an independent
                    alpha-only TDT / multi-blank recursion ............ pinned
  rnnt_logprobs*    torch log_softmax + gather (the reference's own etalon,
                    parts/k2/rnnt_logprobs.py:19-48) and torch autograd
                    through it, in float64 ........................... pinned

The loops are slow on purpose (clarity first): use them at lattice sizes up to
a few thousand cells; oracle/transducer_cpu.c is the fast restatement.
"""

import numpy as np

NEG_INF = -np.inf
# utils/cuda_utils/gpu_rnnt_kernel.py:38 -- the TDT kernels seed their
# accumulators with a finite sentinel, not with -inf.
TDT_NEG = -10000.0


def lse2(a, b):
    """log(exp(a)+exp(b)); utils/rnnt_helper.py:42-53.

    Returns the other operand untouched when one of them is exactly -inf.
    """
    if a == NEG_INF:
        return b
    if b == NEG_INF:
        return a
    if a > b:
        return np.log1p(np.exp(b - a)) + a
    return np.log1p(np.exp(a - b)) + b


def denominator(acts):
    """denom[...] = -max_v x - log sum_v exp(x - max).

    utils/cuda_utils/reduce.py:121-248 driven by
    utils/cuda_utils/gpu_rnnt.py:93-123 (max pass, then sum-exp pass with
    the sign flipped).
    """
    m = acts.max(axis=-1)
    s = np.exp(acts - m[..., None]).sum(axis=-1)
    return -m - np.log(s)


# ----------------------------------------------------------------------------
# RNNT (utils/cuda_utils/gpu_rnnt_kernel.py:73-407)
# ----------------------------------------------------------------------------


def rnnt_alphas(lp, labels, T, U, blank):
    """Forward variables; gpu_rnnt_kernel.py:73-172.

    lp: [>=T, >=U, V] log-probabilities (logits + denominator).
    labels: at least U-1 label ids.  Returns (alphas[T,U], ll_forward).
    """
    dt = lp.dtype.type
    a = np.full((T, U), NEG_INF, dtype=lp.dtype)
    a[0, 0] = dt(0)
    for t in range(T):
        for u in range(U):
            if t == 0 and u == 0:
                continue
            if u == 0:
                a[t, 0] = a[t - 1, 0] + lp[t - 1, 0, blank]
            elif t == 0:
                a[0, u] = a[0, u - 1] + lp[0, u - 1, labels[u - 1]]
            else:
                no_emit = a[t - 1, u] + lp[t - 1, u, blank]
                emit = a[t, u - 1] + lp[t, u - 1, labels[u - 1]]
                a[t, u] = lse2(emit, no_emit)
    ll = a[T - 1, U - 1] + lp[T - 1, U - 1, blank]
    return a, ll


def rnnt_betas(lp, labels, T, U, blank):
    """Backward variables; gpu_rnnt_kernel.py:175-269.  Returns (betas, betas[0,0])."""
    b = np.full((T, U), NEG_INF, dtype=lp.dtype)
    b[T - 1, U - 1] = lp[T - 1, U - 1, blank]
    for t in range(T - 1, -1, -1):
        for u in range(U - 1, -1, -1):
            if t == T - 1 and u == U - 1:
                continue
            if u == U - 1:
                b[t, u] = b[t + 1, u] + lp[t, u, blank]
            elif t == T - 1:
                b[t, u] = b[t, u + 1] + lp[t, u, labels[u]]
            else:
                no_emit = b[t + 1, u] + lp[t, u, blank]
                emit = b[t, u + 1] + lp[t, u, labels[u]]
                b[t, u] = lse2(emit, no_emit)
    return b, b[0, 0]


def rnnt_grads(lp, alphas, betas, ll, labels, T, U, blank, fastemit_lambda, clamp):
    """Gradient of the cost w.r.t. the logits; gpu_rnnt_kernel.py:272-407.

    Same term order as the kernel: the dense exp(alpha+beta+lp-ll) term, the
    FastEmit addition, the three sparse subtractions, then the clamp.
    """
    dt = lp.dtype.type
    V = lp.shape[-1]
    g = np.zeros((T, U, V), dtype=lp.dtype)
    lam = dt(fastemit_lambda)
    for t in range(T):
        for u in range(U):
            row = np.exp(alphas[t, u] + betas[t, u] + lp[t, u, :] - ll)
            if fastemit_lambda > 0.0 and u < U - 1:
                row = row + lam * np.exp(
                    alphas[t, u] + lp[t, u, labels[u]] + betas[t, u + 1] + lp[t, u, :] - ll
                )
            if t == T - 1 and u == U - 1:
                row[blank] -= np.exp(alphas[t, u] + lp[t, u, blank] - ll)
            if t < T - 1:
                row[blank] -= np.exp(alphas[t, u] + lp[t, u, blank] - ll + betas[t + 1, u])
            if u < U - 1:
                v = labels[u]
                row[v] -= np.exp(np.log1p(lam) + alphas[t, u] + lp[t, u, v] - ll + betas[t, u + 1])
            if clamp > 0.0:
                row = np.minimum(np.maximum(row, dt(-clamp)), dt(clamp))
            g[t, u, :] = row
    return g


def rnnt_loss(acts, labels, act_lens, label_lens, blank, fastemit_lambda=0.0, clamp=0.0, dtype=np.float64):
    """Per-utterance costs and logits-gradient for a padded batch.

    Restates GPURNNT.compute_cost_and_score (utils/cuda_utils/gpu_rnnt.py:125-231)
    plus compute_costs_data (utils/rnnt_helper.py:106-116): cost = -ll*(1+lambda),
    padded cells get a zero gradient.  `acts` are raw logits [B,T,U,V].
    Returns (costs[B], grads[B,T,U,V], extras) with extras holding denom,
    alphas, betas (padded with -inf outside the valid lattice), ll_forward, ll_backward.
    """
    acts = np.asarray(acts, dtype=dtype)
    B, Tm, Um, V = acts.shape
    denom = denominator(acts)
    costs = np.zeros(B, dtype=dtype)
    grads = np.zeros_like(acts)
    alphas = np.full((B, Tm, Um), NEG_INF, dtype=dtype)
    betas = np.full((B, Tm, Um), NEG_INF, dtype=dtype)
    llf = np.zeros(B, dtype=dtype)
    llb = np.zeros(B, dtype=dtype)
    for b in range(B):
        T = int(act_lens[b])
        U = int(label_lens[b]) + 1
        lp = acts[b] + denom[b][..., None]
        lab = [int(x) for x in labels[b][: U - 1]]
        a, ll = rnnt_alphas(lp, lab, T, U, blank)
        bt, ll_b = rnnt_betas(lp, lab, T, U, blank)
        grads[b, :T, :U, :] = rnnt_grads(lp, a, bt, ll, lab, T, U, blank, fastemit_lambda, clamp)
        alphas[b, :T, :U] = a
        betas[b, :T, :U] = bt
        llf[b], llb[b] = ll, ll_b
        costs[b] = -ll * dtype(1.0 + fastemit_lambda)
    return costs, grads, dict(denom=denom, alphas=alphas, betas=betas, ll_forward=llf, ll_backward=llb)


# ----------------------------------------------------------------------------
# TDT (utils/cuda_utils/gpu_rnnt_kernel.py:888-1439)
# ----------------------------------------------------------------------------


def tdt_alphas(lp, dlp, labels, T, U, blank, durations, sigma):
    """TDT forward variables; gpu_rnnt_kernel.py:888-1073.

    lp: token log-probs [.,.,V]; dlp: duration log-probs [.,.,D]; durations ascending.
    """
    dt = lp.dtype.type
    sig = dt(sigma)
    NEG = dt(TDT_NEG)
    D = len(durations)
    a = np.full((T, U), NEG_INF, dtype=lp.dtype)
    a[0, 0] = dt(0)
    for t in range(T):
        for u in range(U):
            if t == 0 and u == 0:
                continue
            if u == 0:
                acc = NEG
                for i in range(D):
                    d = durations[i]
                    if d == 0:
                        continue
                    if t >= d:
                        acc = lse2(acc, a[t - d, 0] + lp[t - d, 0, blank] - sig + dlp[t - d, 0, i])
                    else:
                        break
                a[t, 0] = acc
            elif t == 0:
                if durations[0] == 0:
                    a[0, u] = a[0, u - 1] + lp[0, u - 1, labels[u - 1]] - sig + dlp[0, u - 1, 0]
                else:
                    a[0, u] = NEG
            else:
                no_emit = NEG
                for i in range(D):
                    d = durations[i]
                    if d == 0:
                        continue
                    if t >= d:
                        no_emit = lse2(no_emit, a[t - d, u] + lp[t - d, u, blank] - sig + dlp[t - d, u, i])
                    else:
                        break
                emit = NEG
                for i in range(D):
                    d = durations[i]
                    if t >= d:
                        emit = lse2(emit, a[t - d, u - 1] + lp[t - d, u - 1, labels[u - 1]] - sig + dlp[t - d, u - 1, i])
                    else:
                        break
                a[t, u] = lse2(emit, no_emit)
    ll = NEG
    for i in range(D):
        d = durations[i]
        if d == 0:
            continue
        if d == 1:
            # assigned, not accumulated (gpu_rnnt_kernel.py:1054-1061)
            ll = a[T - 1, U - 1] + lp[T - 1, U - 1, blank] - sig + dlp[T - 1, U - 1, i]
            continue
        if T >= d:
            ll = lse2(ll, a[T - d, U - 1] + lp[T - d, U - 1, blank] - sig + dlp[T - d, U - 1, i])
        else:
            break
    return a, ll


def tdt_betas(lp, dlp, labels, T, U, blank, durations, sigma):
    """TDT backward variables; gpu_rnnt_kernel.py:1076-1241."""
    dt = lp.dtype.type
    sig = dt(sigma)
    NEG = dt(TDT_NEG)
    D = len(durations)
    b = np.full((T, U), NEG_INF, dtype=lp.dtype)
    # the duration-1 index is looked for at positions 0 and 1 only (:1137-1148)
    if durations[0] == 1:
        b[T - 1, U - 1] = lp[T - 1, U - 1, blank] - sig + dlp[T - 1, U - 1, 0]
    elif D > 1 and durations[1] == 1:
        b[T - 1, U - 1] = lp[T - 1, U - 1, blank] - sig + dlp[T - 1, U - 1, 1]
    else:
        raise ValueError("TDT durations must hold 1 at position 0 or 1")
    for t in range(T - 1, -1, -1):
        for u in range(U - 1, -1, -1):
            if t == T - 1 and u == U - 1:
                continue
            if u == U - 1:
                acc = NEG
                for i in range(D):
                    d = durations[i]
                    if d == 0:
                        continue
                    if t + d < T:
                        acc = lse2(acc, b[t + d, u] + lp[t, u, blank] + dlp[t, u, i] - sig)
                    elif t + d == T:
                        acc = lse2(acc, lp[t, u, blank] + dlp[t, u, i] - sig)
                b[t, u] = acc
            elif t == T - 1:
                if durations[0] == 0:
                    b[t, u] = b[t, u + 1] + lp[t, u, labels[u]] + dlp[t, u, 0] - sig
                else:
                    b[t, u] = NEG
            else:
                no_emit = NEG
                for i in range(D):
                    d = durations[i]
                    if d == 0:
                        continue
                    if t + d < T:
                        no_emit = lse2(no_emit, b[t + d, u] + lp[t, u, blank] + dlp[t, u, i] - sig)
                emit = NEG
                for i in range(D):
                    d = durations[i]
                    if t + d < T:
                        emit = lse2(emit, b[t + d, u + 1] + lp[t, u, labels[u]] + dlp[t, u, i] - sig)
                b[t, u] = lse2(emit, no_emit)
    return b, b[0, 0]


def tdt_grads(lp, dlp, alphas, betas, ll, labels, T, U, blank, durations, sigma, fastemit_lambda, clamp):
    """TDT gradients; gpu_rnnt_kernel.py:1244-1439.

    Returns (label_grads[T,U,V] w.r.t. token logits, duration_grads[T,U,D]
    w.r.t. duration LOG-PROBS -- the reference leaves the log-softmax Jacobian
    of the duration branch to torch autograd, rnnt_pytorch.py:564-568).
    """
    dt = lp.dtype.type
    sig = dt(sigma)
    lam = dt(fastemit_lambda)
    D = len(durations)
    V = lp.shape[-1]
    lg = np.zeros((T, U, V), dtype=lp.dtype)
    dg = np.zeros((T, U, D), dtype=lp.dtype)
    for t in range(T):
        for u in range(U):
            lpk_blank = lp[t, u, blank] - sig
            for i in range(D):
                d = durations[i]
                g = dt(0)
                if t + d < T and u < U - 1:
                    lpk_label = lp[t, u, labels[u]] - sig
                    g -= np.exp(alphas[t, u] + betas[t + d, u + 1] + lpk_label - ll)
                if t + d < T and d > 0:
                    g -= np.exp(alphas[t, u] + betas[t + d, u] + lpk_blank - ll)
                if t + d == T and u == U - 1 and d > 0:
                    g -= np.exp(alphas[t, u] + lpk_blank - ll)
                dg[t, u, i] = g * np.exp(dlp[t, u, i])

            row = np.exp(alphas[t, u] + betas[t, u] + lp[t, u, :] - ll)
            if fastemit_lambda > 0.0 and u < U - 1:
                fe = np.zeros(V, dtype=lp.dtype)
                for i in range(D):
                    d = durations[i]
                    if t + d < T:
                        fe = fe + lam * np.exp(
                            alphas[t, u]
                            + lp[t, u, labels[u]]
                            + dlp[t, u, i]
                            + betas[t + d, u + 1]
                            + lp[t, u, :]
                            - sig
                            - ll
                        )
                row = row + fe
            if u == U - 1:
                for i in range(D):
                    d = durations[i]
                    if d == 0:
                        continue
                    if t == T - d:
                        row[blank] -= np.exp(alphas[t, u] + lp[t, u, blank] - sig - ll + dlp[t, u, i])
            for i in range(D):
                d = durations[i]
                if d == 0:
                    continue
                if t < T - d:
                    row[blank] -= np.exp(alphas[t, u] + lp[t, u, blank] - sig - ll + betas[t + d, u] + dlp[t, u, i])
            if u < U - 1:
                v = labels[u]
                for i in range(D):
                    d = durations[i]
                    if t + d < T:
                        row[v] -= np.exp(
                            np.log1p(lam) + alphas[t, u] + lp[t, u, v] - sig - ll + betas[t + d, u + 1] + dlp[t, u, i]
                        )
            if clamp > 0.0:
                row = np.minimum(np.maximum(row, dt(-clamp)), dt(clamp))
            lg[t, u, :] = row
    return lg, dg


def tdt_loss(
    acts, labels, act_lens, label_lens, blank, durations, sigma=0.0, fastemit_lambda=0.0, clamp=0.0, dtype=np.float64
):
    """TDT costs and the gradient w.r.t. the COMBINED logits [B,T,U,V+D].

    Restates TDTLossNumba.forward (rnnt_pytorch.py:554-583: split, token part
    passed un-normalised, duration part log-softmaxed) + GPUTDT with omega = 0
    (utils/cuda_utils/gpu_rnnt.py:563-743) + the autograd of that duration
    log-softmax: dlogit_i = dg_i - softmax_i * sum_j dg_j.
    Returns (costs[B], grads[B,T,U,V+D], extras).
    """
    acts = np.asarray(acts, dtype=dtype)
    durations = [int(d) for d in durations]
    D = len(durations)
    B, Tm, Um, VD = acts.shape
    V = VD - D
    tok = acts[..., :V]
    dur = acts[..., V:]
    denom = denominator(tok)
    dlp_all = dur + denominator(dur)[..., None]
    costs = np.zeros(B, dtype=dtype)
    grads = np.zeros_like(acts)
    label_grads = np.zeros((B, Tm, Um, V), dtype=dtype)
    duration_grads = np.zeros((B, Tm, Um, D), dtype=dtype)
    alphas = np.full((B, Tm, Um), NEG_INF, dtype=dtype)
    betas = np.full((B, Tm, Um), NEG_INF, dtype=dtype)
    llf = np.zeros(B, dtype=dtype)
    llb = np.zeros(B, dtype=dtype)
    for b in range(B):
        T = int(act_lens[b])
        U = int(label_lens[b]) + 1
        lp = tok[b] + denom[b][..., None]
        dlp = dlp_all[b]
        lab = [int(x) for x in labels[b][: U - 1]]
        a, ll = tdt_alphas(lp, dlp, lab, T, U, blank, durations, sigma)
        bt, ll_b = tdt_betas(lp, dlp, lab, T, U, blank, durations, sigma)
        lg, dg = tdt_grads(lp, dlp, a, bt, ll, lab, T, U, blank, durations, sigma, fastemit_lambda, clamp)
        label_grads[b, :T, :U] = lg
        duration_grads[b, :T, :U] = dg
        grads[b, :T, :U, :V] = lg
        grads[b, :T, :U, V:] = dg - np.exp(dlp[:T, :U]) * dg.sum(axis=-1, keepdims=True)
        alphas[b, :T, :U] = a
        betas[b, :T, :U] = bt
        llf[b], llb[b] = ll, ll_b
        costs[b] = -ll * dtype(1.0 + fastemit_lambda)
    extras = dict(
        denom=denom,
        dlp=dlp_all,
        alphas=alphas,
        betas=betas,
        ll_forward=llf,
        ll_backward=llb,
        label_grads=label_grads,
        duration_grads=duration_grads,
    )
    return costs, grads, extras


# ----------------------------------------------------------------------------
# Multi-blank transducer (utils/cuda_utils/gpu_rnnt_kernel.py:410-885)
# ----------------------------------------------------------------------------
# The softmax runs over V token logits, then the big blanks, then the standard blank: big blank i
# (duration big_blank_durations[i]) sits at index blank-1-i.  Every arc score is lp - sigma.


def multiblank_alphas(lp, labels, T, U, blank, big_blank_durations, sigma):
    """Forward variables; gpu_rnnt_kernel.py:410-568.  Returns (alphas[T,U], llForward)."""
    dt = lp.dtype.type
    sig = dt(sigma)
    a = np.full((T, U), NEG_INF, dtype=lp.dtype)
    a[0, 0] = dt(0)
    for t in range(T):
        for u in range(U):
            if t == 0 and u == 0:
                continue
            if u == 0:
                acc = a[t - 1, 0] + lp[t - 1, 0, blank] - sig
                for i, d in enumerate(big_blank_durations):
                    if t >= d:
                        acc = lse2(acc, a[t - d, 0] + lp[t - d, 0, blank - 1 - i] - sig)
                a[t, 0] = acc
            elif t == 0:
                a[0, u] = a[0, u - 1] + lp[0, u - 1, labels[u - 1]] - sig
            else:
                no_emit = a[t - 1, u] + lp[t - 1, u, blank] - sig
                emit = a[t, u - 1] + lp[t, u - 1, labels[u - 1]] - sig
                acc = lse2(emit, no_emit)
                for i, d in enumerate(big_blank_durations):
                    if t >= d:
                        acc = lse2(acc, a[t - d, u] + lp[t - d, u, blank - 1 - i] - sig)
                a[t, u] = acc
    ll = a[T - 1, U - 1] + lp[T - 1, U - 1, blank] - sig
    for i, d in enumerate(big_blank_durations):
        if T >= d:
            ll = lse2(ll, a[T - d, U - 1] + lp[T - d, U - 1, blank - 1 - i] - sig)
    return a, ll


def multiblank_betas(lp, labels, T, U, blank, big_blank_durations, sigma):
    """Backward variables; gpu_rnnt_kernel.py:571-724.  Returns (betas[T,U], llBackward)."""
    dt = lp.dtype.type
    sig = dt(sigma)
    bt = np.full((T, U), NEG_INF, dtype=lp.dtype)
    bt[T - 1, U - 1] = lp[T - 1, U - 1, blank] - sig
    for t in range(T - 1, -1, -1):
        for u in range(U - 1, -1, -1):
            if t == T - 1 and u == U - 1:
                continue
            if u == U - 1:
                acc = bt[t + 1, U - 1] + lp[t, U - 1, blank] - sig
                for i, d in enumerate(big_blank_durations):
                    if t + d < T:
                        acc = lse2(acc, bt[t + d, U - 1] + lp[t, U - 1, blank - 1 - i] - sig)
                    elif t + d == T and d != 1:
                        acc = lse2(acc, lp[t, U - 1, blank - 1 - i] - sig)
                bt[t, U - 1] = acc
            elif t == T - 1:
                bt[T - 1, u] = bt[T - 1, u + 1] + lp[T - 1, u, labels[u]] - sig
            else:
                no_emit = bt[t + 1, u] + lp[t, u, blank] - sig
                emit = bt[t, u + 1] + lp[t, u, labels[u]] - sig
                acc = lse2(emit, no_emit)
                for i, d in enumerate(big_blank_durations):
                    if t < T - d:
                        acc = lse2(acc, bt[t + d, u] + lp[t, u, blank - 1 - i] - sig)
                bt[t, u] = acc
    return bt, bt[0, 0]


def multiblank_grads(lp, alphas, betas, ll, labels, T, U, blank, big_blank_durations, sigma, fastemit_lambda, clamp):
    """Gradient w.r.t. the logits for the valid cells; gpu_rnnt_kernel.py:727-885."""
    dt = lp.dtype.type
    sig = dt(sigma)
    lam = dt(fastemit_lambda)
    V = lp.shape[-1]
    g = np.zeros((T, U, V), dtype=lp.dtype)
    for t in range(T):
        for u in range(U):
            row = np.exp(alphas[t, u] + betas[t, u] + lp[t, u, :] - ll)
            if fastemit_lambda > 0.0 and u < U - 1:
                row = row + lam * np.exp(
                    alphas[t, u] + lp[t, u, labels[u]] + betas[t, u + 1] + lp[t, u, :] - sig - ll
                )
            if t == T - 1 and u == U - 1:
                row[blank] -= np.exp(alphas[t, u] + lp[t, u, blank] - sig - ll)
            for i, d in enumerate(big_blank_durations):
                k = blank - 1 - i
                if t == T - d and u == U - 1:
                    row[k] -= np.exp(alphas[t, u] + lp[t, u, k] - sig - ll)
            if t < T - 1:
                row[blank] -= np.exp(alphas[t, u] + lp[t, u, blank] - sig - ll + betas[t + 1, u])
            for i, d in enumerate(big_blank_durations):
                k = blank - 1 - i
                if t < T - d:
                    row[k] -= np.exp(alphas[t, u] + lp[t, u, k] - sig - ll + betas[t + d, u])
            if u < U - 1:
                v = labels[u]
                row[v] -= np.exp(np.log1p(lam) + alphas[t, u] + lp[t, u, v] - sig - ll + betas[t, u + 1])
            if clamp > 0.0:
                row = np.minimum(np.maximum(row, dt(-clamp)), dt(clamp))
            g[t, u, :] = row
    return g


def multiblank_loss(
    acts, labels, act_lens, label_lens, blank, big_blank_durations, sigma=0.0, fastemit_lambda=0.0, clamp=0.0,
    dtype=np.float64,
):  # fmt: skip
    """Per-utterance costs and logits-gradient; MultiblankGPURNNT.compute_cost_and_score
    (utils/cuda_utils/gpu_rnnt.py:343-440) + compute_costs_data (utils/rnnt_helper.py:106-116).
    `acts` are raw logits [B,T,U,V_tokens + num_big_blanks + 1]."""
    acts = np.asarray(acts, dtype=dtype)
    B, Tm, Um, V = acts.shape
    denom = denominator(acts)
    costs = np.zeros(B, dtype=dtype)
    grads = np.zeros_like(acts)
    alphas = np.full((B, Tm, Um), NEG_INF, dtype=dtype)
    betas = np.full((B, Tm, Um), NEG_INF, dtype=dtype)
    llf = np.zeros(B, dtype=dtype)
    llb = np.zeros(B, dtype=dtype)
    durs = [int(d) for d in big_blank_durations]
    for b in range(B):
        T = int(act_lens[b])
        U = int(label_lens[b]) + 1
        lp = acts[b] + denom[b][..., None]
        lab = [int(x) for x in labels[b][: U - 1]]
        a, ll = multiblank_alphas(lp, lab, T, U, blank, durs, sigma)
        bt, ll_b = multiblank_betas(lp, lab, T, U, blank, durs, sigma)
        grads[b, :T, :U, :] = multiblank_grads(lp, a, bt, ll, lab, T, U, blank, durs, sigma, fastemit_lambda, clamp)
        alphas[b, :T, :U] = a
        betas[b, :T, :U] = bt
        llf[b], llb[b] = ll, ll_b
        costs[b] = -ll * dtype(1.0 + fastemit_lambda)
    return costs, grads, dict(denom=denom, alphas=alphas, betas=betas, ll_forward=llf, ll_backward=llb)


# ----------------------------------------------------------------------------------------
# Compact log-prob op (nemo/collections/asr/parts/k2/rnnt_logprobs_triton.py)
# ----------------------------------------------------------------------------------------
def _logprobs_masks(B, T, U, source_lens, target_lens):
    source_lens = np.full(B, T) if source_lens is None else np.asarray(source_lens)
    target_lens = np.full(B, U - 1) if target_lens is None else np.asarray(target_lens)
    t = np.arange(T)[None, :, None]
    u = np.arange(U)[None, None, :]
    in_time = t < source_lens[:, None, None]
    cell = in_time & (u <= target_lens[:, None, None])  # :46-48: rows with t >= len or u > target_len are skipped
    has_target = in_time & (u < target_lens[:, None, None])  # :64
    return cell, has_target


def rnnt_logprobs(logits, targets, blank, source_lens=None, target_lens=None):
    """(target_scores, blank_scores), [B,T,U] each; rnnt_logprobs_triton.py:20-69.

    log-softmax over the last axis, read at the target id of column u and at the blank id; entries of
    skipped rows, and target entries of columns without a target, stay 0 (:148-149).
    """
    x = np.asarray(logits, dtype=np.float64)
    B, T, U, V = x.shape
    targets = np.asarray(targets).reshape(B, U - 1)
    cell, has_target = _logprobs_masks(B, T, U, source_lens, target_lens)
    m = x.max(axis=-1)
    log_norm = m + np.log(np.exp(x - m[..., None]).sum(axis=-1))
    ids = np.concatenate([targets, np.zeros((B, 1), dtype=targets.dtype)], axis=1)  # column U-1: any id, masked below
    picked = np.take_along_axis(x, np.broadcast_to(ids[:, None, :, None], (B, T, U, 1)), axis=-1)[..., 0]
    target_scores = np.where(has_target, picked - log_norm, 0.0)
    blank_scores = np.where(cell, x[..., blank] - log_norm, 0.0)
    return target_scores, blank_scores


def rnnt_logprobs_grad(logits, targets, blank, grad_target_scores, grad_blank_scores, source_lens=None, target_lens=None):
    """Gradient of the logits given those of the two score arrays; rnnt_logprobs_triton.py:72-127.

    g_v = -softmax_v * (gb + gt), plus gb at the blank id, plus gt at the target id -- and where the
    target id IS the blank id the second `where` (:122) replaces the first, so only gt is added there.
    Skipped rows stay 0 (:211).
    """
    x = np.asarray(logits, dtype=np.float64)
    B, T, U, V = x.shape
    targets = np.asarray(targets).reshape(B, U - 1)
    cell, has_target = _logprobs_masks(B, T, U, source_lens, target_lens)
    gb = np.where(cell, np.asarray(grad_blank_scores, dtype=np.float64), 0.0)
    gt = np.where(has_target, np.asarray(grad_target_scores, dtype=np.float64), 0.0)
    m = x.max(axis=-1, keepdims=True)
    e = np.exp(x - m)
    softmax = e / e.sum(axis=-1, keepdims=True)
    grad = -softmax * (gb + gt)[..., None]
    base = grad.copy()
    grad[..., blank] = base[..., blank] + gb
    ids = np.concatenate([targets, np.zeros((B, 1), dtype=targets.dtype)], axis=1)
    idx = np.broadcast_to(ids[:, None, :, None], (B, T, U, 1))
    at_target = np.take_along_axis(base, idx, axis=-1)[..., 0] + gt
    current = np.take_along_axis(grad, idx, axis=-1)[..., 0]
    np.put_along_axis(grad, idx, np.where(has_target, at_target, current)[..., None], axis=-1)
    return np.where(cell[..., None], grad, 0.0)


# ----------------------------------------------------------------------------------------
# Joint network + loss (nemo/collections/asr/modules/rnnt.py:1707-1724, :1759-1777)
# ----------------------------------------------------------------------------------------
def bf16_round(x):
    """x rounded to the nearest bfloat16 (ties to even), returned as float64."""
    a = np.ascontiguousarray(x, dtype=np.float32)
    bits = a.view(np.uint32).astype(np.uint64)
    rounded = ((bits + 0x7FFF + ((bits >> 16) & 1)) & 0xFFFF0000).astype(np.uint32)
    out = rounded.view(np.float32).astype(np.float64)
    return np.where(np.isfinite(a), out, a.astype(np.float64))


def joint_rnnt_loss(f, g, weight, bias, labels, act_lens, label_lens, blank, fastemit_lambda=0.0, clamp=0.0, grad_costs=None,
                    keep_mask=None, dropout_p=0.0, durations=None, sigma=0.0, big_blank_durations=None,
                    activation="relu"):
    """RNNT (with `durations` TDT, with `big_blank_durations` multi-blank) loss of the joint's logits under
    bf16-autocast arithmetic, and its gradients.  `activation`: relu, tanh or sigmoid (modules/rnnt.py:1762-1770);
    where "relu" stands below read act(x) rounded to bf16, with the derivative taken at that rounded output
    (1 - h^2, h (1 - h)) as torch's tanh / sigmoid backward does.

    logits[b,t,u,:] = drop(relu(bf16(f[b,t] + g[b,u]))) @ bf16(weight).T + bias   (modules/rnnt.py:1707-1724,
    joint_net = ReLU, Dropout, Linear :1766-1777; operands rounded to bf16, products and sums exact here --
    float32 accumulation on the GPU; the bias enters as bf16(bias) + bf16(bias - bf16(bias)), i.e. to about
    16 bits).  drop(x) = bf16(x * keep_mask / (1 - dropout_p)) for a given boolean keep_mask [B,T,U,H]
    (torch.nn.functional.dropout's definition; which units are kept is the caller's business), identity without
    one.  The loss and the gradient of the logits are rnnt_loss's -- tdt_loss's when `durations` is given: the
    Linear layer then has V + len(durations) outputs, token logits first (rnnt_pytorch.py:563-568); the gradients
    of f, g, weight, bias follow by the chain rule with every rounding treated as the identity (what autograd does
    under autocast).
    Returns (costs, d_f, d_g, d_weight, d_bias).
    """
    f = bf16_round(f)
    g = bf16_round(g)
    w = bf16_round(weight)
    B, T, H = f.shape
    U, V = g.shape[1], w.shape[0]
    if bias is None:
        b_eff = np.zeros(V)
    else:
        b_hi = bf16_round(bias)
        b_eff = b_hi + bf16_round(np.asarray(bias, dtype=np.float32) - b_hi.astype(np.float32))
    pre = bf16_round(f[:, :, None, :] + g[:, None, :, :])  # [B,T,U,H]
    if activation == "relu":
        hidden = np.maximum(pre, 0.0)
        chain = (pre > 0).astype(np.float64)  # d hidden / d pre
    elif activation == "tanh":
        hidden = bf16_round(np.tanh(pre))
        chain = 1.0 - hidden * hidden
    elif activation == "sigmoid":
        hidden = bf16_round(1.0 / (1.0 + np.exp(-pre)))
        chain = hidden * (1.0 - hidden)
    else:
        raise ValueError(activation)
    if keep_mask is not None:
        scale = np.float32(1.0) / (np.float32(1.0) - np.float32(dropout_p))
        keep = np.asarray(keep_mask, dtype=bool)
        hidden = np.where(keep, bf16_round(hidden.astype(np.float32) * scale), 0.0)
        chain = chain * keep * np.float64(scale)
    logits = hidden @ w.T + b_eff
    if durations:
        costs, d_logits, _ = tdt_loss(logits, labels, act_lens, label_lens, blank, durations, sigma, fastemit_lambda, clamp)
    elif big_blank_durations:
        costs, d_logits, _ = multiblank_loss(logits, labels, act_lens, label_lens, blank, big_blank_durations, sigma,
                                             fastemit_lambda, clamp)
    else:
        costs, d_logits, _ = rnnt_loss(logits, labels, act_lens, label_lens, blank, fastemit_lambda, clamp)
    if grad_costs is not None:
        d_logits = d_logits * np.asarray(grad_costs, dtype=np.float64).reshape(B, 1, 1, 1)
    d_weight = np.einsum('btuv,btuh->vh', d_logits, hidden)
    d_bias = d_logits.sum(axis=(0, 1, 2))
    d_pre = (d_logits @ w) * chain
    return costs, d_pre.sum(axis=2), d_pre.sum(axis=1), d_weight, d_bias
