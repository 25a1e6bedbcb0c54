"""Independent checkers used to pin the oracle (and, through it, the HIP path).

Nothing here shares code with oracle/: the brute-force enumerators walk every
path of a tiny lattice, and the autograd functions differentiate an alpha-only
recursion written with torch ops in float64.
"""

import math

import numpy as np
import torch


def logsumexp_list(xs):
    if not xs:
        return -math.inf
    m = max(xs)
    if m == -math.inf:
        return -math.inf
    return m + math.log(sum(math.exp(x - m) for x in xs))


def rnnt_bruteforce_ll(logits, labels, blank):
    """log P(labels | logits) by enumerating every alignment.  logits: [T,U,V] float64."""
    T, U, _ = logits.shape
    lp = logits - np.log(np.exp(logits).sum(-1, keepdims=True))
    totals = []

    def walk(t, u, acc):
        if t == T - 1 and u == U - 1:
            totals.append(acc + lp[t, u, blank])
            return
        if t < T - 1:
            walk(t + 1, u, acc + lp[t, u, blank])
        if u < U - 1:
            walk(t, u + 1, acc + lp[t, u, labels[u]])

    walk(0, 0, 0.0)
    return logsumexp_list(totals)


def tdt_bruteforce_ll(logits, labels, blank, durations, sigma):
    """TDT log-likelihood by enumerating every (token, duration) path.

    logits: [T,U,V+D] float64; token softmax over the first V, duration softmax
    over the last D; every emitted token pays -sigma.  A blank must advance by a
    non-zero duration; a label may stay (duration 0) but must land on t' < T; the
    path ends when a blank at u = U-1 lands exactly on t' = T.
    """
    D = len(durations)
    T, U, VD = logits.shape
    V = VD - D
    tok = logits[..., :V]
    dur = logits[..., V:]
    lp = tok - np.log(np.exp(tok).sum(-1, keepdims=True))
    dlp = dur - np.log(np.exp(dur).sum(-1, keepdims=True))
    totals = []

    def walk(t, u, acc):
        for i, d in enumerate(durations):
            if d > 0:
                w = acc + lp[t, u, blank] - sigma + dlp[t, u, i]
                if t + d < T:
                    walk(t + d, u, w)
                elif t + d == T and u == U - 1:
                    totals.append(w)
            if u < U - 1 and t + d < T:
                walk(t + d, u + 1, acc + lp[t, u, labels[u]] - sigma + dlp[t, u, i])

    walk(0, 0, 0.0)
    return logsumexp_list(totals)


def _lse(a, b):
    return torch.logsumexp(torch.stack([a, b]), dim=0)


def rnnt_autograd(logits, labels, blank):
    """(-ll, d(-ll)/dlogits) from an alpha-only recursion in torch float64."""
    x = torch.tensor(np.asarray(logits, dtype=np.float64), requires_grad=True)
    T, U, _ = x.shape
    lp = torch.log_softmax(x, dim=-1)
    alpha = [[None] * U for _ in range(T)]
    alpha[0][0] = torch.zeros((), dtype=torch.float64)
    for t in range(T):
        for u in range(U):
            if t == 0 and u == 0:
                continue
            terms = []
            if t > 0:
                terms.append(alpha[t - 1][u] + lp[t - 1, u, blank])
            if u > 0:
                terms.append(alpha[t][u - 1] + lp[t, u - 1, labels[u - 1]])
            alpha[t][u] = terms[0] if len(terms) == 1 else _lse(terms[0], terms[1])
    nll = -(alpha[T - 1][U - 1] + lp[T - 1, U - 1, blank])
    nll.backward()
    return float(nll.detach()), x.grad.numpy()


def rnnt_fastemit_autograd(logits, labels, blank, lam):
    """FastEmit gradient by its definition: the gradient of -ll w.r.t. the
    log-probs with every label-arc entry scaled by (1+lambda), pushed through the
    log-softmax Jacobian; the cost is scaled by (1+lambda).  Blank arcs and label
    arcs read separate leaves so the two contributions can be scaled apart even
    when a label id equals the blank id."""
    x = torch.tensor(np.asarray(logits, dtype=np.float64), requires_grad=True)
    T, U, V = x.shape
    lp = torch.log_softmax(x, dim=-1)
    lp_blank = lp.detach().clone().requires_grad_(True)
    lp_lab = lp.detach().clone().requires_grad_(True)
    alpha = [[None] * U for _ in range(T)]
    alpha[0][0] = torch.zeros((), dtype=torch.float64)
    for t in range(T):
        for u in range(U):
            if t == 0 and u == 0:
                continue
            terms = []
            if t > 0:
                terms.append(alpha[t - 1][u] + lp_blank[t - 1, u, blank])
            if u > 0:
                terms.append(alpha[t][u - 1] + lp_lab[t, u - 1, labels[u - 1]])
            alpha[t][u] = terms[0] if len(terms) == 1 else _lse(terms[0], terms[1])
    nll = -(alpha[T - 1][U - 1] + lp_blank[T - 1, U - 1, blank])
    g_blank, g_lab = torch.autograd.grad(nll, [lp_blank, lp_lab], allow_unused=True)
    g_lab = torch.zeros_like(lp) if g_lab is None else g_lab
    lp.backward(g_blank + (1.0 + lam) * g_lab)
    return float(nll.detach()) * (1.0 + lam), x.grad.numpy()


def tdt_autograd(logits, labels, blank, durations, sigma, lam=0.0):
    """(-ll, gradient w.r.t. the combined logits) for TDT from an alpha-only
    recursion (Eq. 7 of arXiv:2304.06795) in torch float64.  With lam > 0 the
    token log-prob gradient entries of label arcs are scaled by (1+lam) before
    the token log-softmax Jacobian (duration branch untouched), which is what
    the kernel's FastEmit terms amount to."""
    D = len(durations)
    x = torch.tensor(np.asarray(logits, dtype=np.float64), requires_grad=True)
    T, U, VD = x.shape
    V = VD - D
    lp = torch.log_softmax(x[..., :V], dim=-1)
    dlp = torch.log_softmax(x[..., V:], dim=-1)
    lp_leaf = lp.detach().clone().requires_grad_(True)
    dlp_leaf = dlp.detach().clone().requires_grad_(True)
    # label arcs read lp_lab (so they can be scaled separately), blank arcs lp_leaf
    lp_lab = lp.detach().clone().requires_grad_(True)
    alpha = [[None] * U for _ in range(T)]
    alpha[0][0] = torch.zeros((), dtype=torch.float64)
    for t in range(T):
        for u in range(U):
            if t == 0 and u == 0:
                continue
            terms = []
            for i, d in enumerate(durations):
                if d > 0 and t - d >= 0 and alpha[t - d][u] is not None:
                    terms.append(alpha[t - d][u] + lp_leaf[t - d, u, blank] - sigma + dlp_leaf[t - d, u, i])
                if u > 0 and t - d >= 0 and alpha[t - d][u - 1] is not None:
                    terms.append(alpha[t - d][u - 1] + lp_lab[t - d, u - 1, labels[u - 1]] - sigma + dlp_leaf[t - d, u - 1, i])
            alpha[t][u] = torch.logsumexp(torch.stack(terms), dim=0) if terms else None
    finals = []
    for i, d in enumerate(durations):
        if d > 0 and T - d >= 0 and alpha[T - d][U - 1] is not None:
            finals.append(alpha[T - d][U - 1] + lp_leaf[T - d, U - 1, blank] - sigma + dlp_leaf[T - d, U - 1, i])
    nll = -torch.logsumexp(torch.stack(finals), dim=0)
    g_blank, g_lab, g_dur = torch.autograd.grad(nll, [lp_leaf, lp_lab, dlp_leaf], allow_unused=True)
    g_lab = torch.zeros_like(lp) if g_lab is None else g_lab
    g_tok = g_blank + (1.0 + lam) * g_lab
    torch.autograd.backward([lp, dlp], [g_tok, g_dur])
    return float(nll.detach()) * (1.0 + lam), x.grad.numpy()


def multiblank_bruteforce_ll(logits, labels, blank, big_blank_durations, sigma):
    """Multi-blank log-likelihood (arXiv:2211.03541) by enumerating every path.  logits: [T,U,V]
    float64 with one softmax over tokens, big blanks (index blank-1-i, duration d_i) and the standard
    blank (duration 1); every arc pays -sigma.  A label stays on the frame; a blank of duration d
    moves to frame t+d, which must exist unless the path ends there (t+d == T at u == U-1)."""
    T, U, _ = logits.shape
    lp = logits - np.log(np.exp(logits).sum(-1, keepdims=True))
    blanks = [(blank, 1)] + [(blank - 1 - i, d) for i, d in enumerate(big_blank_durations)]
    totals = []

    def walk(t, u, acc):
        for k, d in blanks:
            w = acc + lp[t, u, k] - sigma
            if t + d < T:
                walk(t + d, u, w)
            elif t + d == T and u == U - 1:
                totals.append(w)
        if u < U - 1:
            walk(t, u + 1, acc + lp[t, u, labels[u]] - sigma)

    walk(0, 0, 0.0)
    return logsumexp_list(totals)


def multiblank_autograd(logits, labels, blank, big_blank_durations, sigma, lam=0.0):
    """(-ll, d(-ll)/dlogits) for the multi-blank transducer from an alpha-only recursion in torch
    float64.  With lam > 0 the log-prob gradient entries of label arcs are scaled by (1+lam) before
    the log-softmax Jacobian and the cost by (1+lam): what the kernel's FastEmit terms amount to."""
    x = torch.tensor(np.asarray(logits, dtype=np.float64), requires_grad=True)
    T, U, _ = x.shape
    lp = torch.log_softmax(x, dim=-1)
    lp_blank = lp.detach().clone().requires_grad_(True)
    lp_lab = lp.detach().clone().requires_grad_(True)
    blanks = [(blank, 1)] + [(blank - 1 - i, d) for i, d in enumerate(big_blank_durations)]
    alpha = [[None] * U for _ in range(T)]
    alpha[0][0] = torch.zeros((), dtype=torch.float64)
    for t in range(T):
        for u in range(U):
            if t == 0 and u == 0:
                continue
            terms = []
            for k, d in blanks:
                if t - d >= 0 and alpha[t - d][u] is not None:
                    terms.append(alpha[t - d][u] + lp_blank[t - d, u, k] - sigma)
            if u > 0 and alpha[t][u - 1] is not None:
                terms.append(alpha[t][u - 1] + lp_lab[t, u - 1, labels[u - 1]] - sigma)
            alpha[t][u] = torch.logsumexp(torch.stack(terms), dim=0) if terms else None
    finals = [
        alpha[T - d][U - 1] + lp_blank[T - d, U - 1, k] - sigma
        for k, d in blanks
        if T - d >= 0 and alpha[T - d][U - 1] is not None
    ]
    nll = -torch.logsumexp(torch.stack(finals), dim=0)
    g_blank, g_lab = torch.autograd.grad(nll, [lp_blank, lp_lab], allow_unused=True)
    g_lab = torch.zeros_like(lp) if g_lab is None else g_lab
    lp.backward(g_blank + (1.0 + lam) * g_lab)
    return float(nll.detach()) * (1.0 + lam), x.grad.numpy()


class _RoundedActivation(torch.autograd.Function):
    """tanh / sigmoid whose output is rounded to bf16 and whose backward takes the slope at that rounded output
    (torch's tanh_backward / sigmoid_backward get the OUTPUT tensor, which under autocast is the bf16 one)."""

    @staticmethod
    def forward(ctx, x, kind):
        out = (torch.tanh(x) if kind == "tanh" else torch.sigmoid(x)).float().to(torch.bfloat16).double()
        ctx.save_for_backward(out)
        ctx.kind = kind
        return out

    @staticmethod
    def backward(ctx, grad):
        (out,) = ctx.saved_tensors
        return grad * ((1.0 - out * out) if ctx.kind == "tanh" else out * (1.0 - out)), None


def joint_autograd(f, g, weight, bias, labels, blank, grad_costs, keep_mask=None, dropout_p=0.0, activation="relu",
                   rounded_activation=True):
    """Costs and gradients of sum_b grad_costs[b] * nll_b through act(f+g) @ W.T + bias, all utterances at
    full length, by torch autograd in float64; `f`, `g`, `weight`, `bias` must already be exactly
    representable in bf16, and the rounding of f+g to bf16 is applied straight-through.  tanh / sigmoid outputs are
    rounded to bf16 with the slope taken there (rounded_activation=False: plain float64 tanh / sigmoid, for a
    loose cross-check that owes nothing to that convention)."""
    f = torch.tensor(np.asarray(f, dtype=np.float64), requires_grad=True)
    g = torch.tensor(np.asarray(g, dtype=np.float64), requires_grad=True)
    w = torch.tensor(np.asarray(weight, dtype=np.float64), requires_grad=True)
    b = torch.tensor(np.asarray(bias, dtype=np.float64), requires_grad=True)
    s = f[:, :, None, :] + g[:, None, :, :]
    s = s + (s.detach().float().to(torch.bfloat16).double() - s.detach())
    if activation == "relu":
        hidden = torch.relu(s)
    elif rounded_activation:
        hidden = _RoundedActivation.apply(s, activation)
    else:
        hidden = torch.tanh(s) if activation == "tanh" else torch.sigmoid(s)
    act_out = hidden
    if keep_mask is not None:  # dropout with a given mask; its bf16 output rounding is straight-through as well
        scale = float(np.float32(1.0) / (np.float32(1.0) - np.float32(dropout_p)))
        hidden = hidden * torch.tensor(np.asarray(keep_mask, dtype=np.float64)) * scale
        # the product is formed in float32 before the rounding, as on the GPU
        exact32 = (act_out.detach().float() * np.float32(scale)).to(torch.bfloat16).double()
        rounded = torch.where(torch.tensor(np.asarray(keep_mask, dtype=bool)), exact32, torch.zeros_like(exact32))
        hidden = hidden + (rounded - hidden.detach())
    logits = torch.nn.functional.linear(hidden, w, b)
    B, T, U, _ = logits.shape
    costs = []
    for i in range(B):
        lp = torch.log_softmax(logits[i], dim=-1)
        alpha = [[None] * U for _ in range(T)]
        alpha[0][0] = torch.zeros((), dtype=torch.float64)
        for t in range(T):
            for u in range(U):
                if t == 0 and u == 0:
                    continue
                terms = []
                if t > 0:
                    terms.append(alpha[t - 1][u] + lp[t - 1, u, blank])
                if u > 0:
                    terms.append(alpha[t][u - 1] + lp[t, u - 1, labels[i][u - 1]])
                alpha[t][u] = terms[0] if len(terms) == 1 else _lse(terms[0], terms[1])
        costs.append(-(alpha[T - 1][U - 1] + lp[T - 1, U - 1, blank]))
    costs = torch.stack(costs)
    (costs * torch.tensor(np.asarray(grad_costs, dtype=np.float64))).sum().backward()
    return costs.detach().numpy(), f.grad.numpy(), g.grad.numpy(), w.grad.numpy(), b.grad.numpy()
