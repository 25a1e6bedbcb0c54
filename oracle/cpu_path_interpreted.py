"""TEST / BENCHMARK INFRASTRUCTURE ONLY -- never imported by the shipped package.

The reference's CPU path as a user of the reference experiences it: an interpreted loop over lattice cells doing
arithmetic on 0-d torch tensors (utils/cpu_utils/cpu_rnnt.py:246-345 runs un-jitted; torch.log_softmax in front of
it and torch autograd behind it, rnnt_pytorch.py:420-435).  Written from the description of that algorithm, not from
its text; it exists to be TIMED beside the GPU kernels at the small CPU configuration and must agree with
oracle.rnnt_cpu_path before its time means anything (tests/test_oracle_rnnt.py checks that).
"""

import math

import torch


def _lse(a, b):
    if torch.isinf(a):
        return b
    if torch.isinf(b):
        return a
    hi, lo = (a, b) if a > b else (b, a)
    return hi + math.log1p(math.exp(lo - hi))


def rnnt_cpu_path_interpreted(acts, labels, act_lens, label_lens, blank, fastemit_lambda=0.0):
    """(costs [B], gradient w.r.t. the logits [B,T,U,V]) as float32 numpy arrays; grad_output = ones, no clamp."""
    x = torch.as_tensor(acts, dtype=torch.float32).clone().requires_grad_(True)
    logp = torch.log_softmax(x, -1)
    lp = logp.detach()
    B, T, U, V = x.shape
    sparse = torch.zeros_like(lp)
    costs = torch.zeros(B)
    boost = math.log1p(fastemit_lambda)
    for b in range(B):
        Tb, Ub = int(act_lens[b]), int(label_lens[b]) + 1
        lab = [int(v) for v in labels[b][: Ub - 1]]
        blank_lp = lp[b, :Tb, :Ub, blank]
        label_lp = [[lp[b, t, u, lab[u]] for u in range(Ub - 1)] for t in range(Tb)]
        alpha = torch.zeros(Tb, Ub)
        for t in range(Tb):
            for u in range(Ub):
                if t == 0 and u == 0:
                    continue
                if u == 0:
                    alpha[t, 0] = alpha[t - 1, 0] + blank_lp[t - 1, 0]
                elif t == 0:
                    alpha[0, u] = alpha[0, u - 1] + label_lp[0][u - 1]
                else:
                    alpha[t, u] = _lse(alpha[t, u - 1] + label_lp[t][u - 1], alpha[t - 1, u] + blank_lp[t - 1, u])
        ll_forward = alpha[Tb - 1, Ub - 1] + blank_lp[Tb - 1, Ub - 1]
        beta = torch.zeros(Tb, Ub)
        beta[Tb - 1, Ub - 1] = blank_lp[Tb - 1, Ub - 1]
        for t in range(Tb - 1, -1, -1):
            for u in range(Ub - 1, -1, -1):
                if t == Tb - 1 and u == Ub - 1:
                    continue
                if u == Ub - 1:
                    beta[t, u] = beta[t + 1, u] + blank_lp[t, u]
                elif t == Tb - 1:
                    beta[t, u] = beta[t, u + 1] + label_lp[t][u]
                else:
                    beta[t, u] = _lse(beta[t, u + 1] + label_lp[t][u], beta[t + 1, u] + blank_lp[t, u])
        ll = beta[0, 0]
        for t in range(Tb):
            for u in range(Ub):
                if t < Tb - 1:
                    sparse[b, t, u, blank] = -torch.exp(blank_lp[t, u] + alpha[t, u] + beta[t + 1, u] - ll)
                if u < Ub - 1:
                    sparse[b, t, u, lab[u]] = -torch.exp(boost + label_lp[t][u] + alpha[t, u] + beta[t, u + 1] - ll)
        sparse[b, Tb - 1, Ub - 1, blank] = -torch.exp(blank_lp[Tb - 1, Ub - 1] + alpha[Tb - 1, Ub - 1] - ll)
        costs[b] = -(ll_forward + ll_forward * fastemit_lambda)
    logp.backward(sparse)
    return costs.numpy(), x.grad.numpy()
