"""Seeded synthetic inputs for the five benchmark configurations of the transducer loss (plus one for the
multi-blank loss, which the reference publishes no configuration for).

Tensors are generated on the CPU with torch.Generator().manual_seed(1234 + index) so
that the GPU path, the CPU baseline and the parity checks see identical values.
Lengths are uniform integers with one utterance forced to T and one to U-1, which is
what the shape check of the loss requires.
"""

from dataclasses import dataclass, field
from typing import List, Optional

import torch


@dataclass
class Config:
    name: str
    B: int
    T: int
    U: int  # label axis of the tensor = max label length + 1
    V: int  # token logits, blank included
    dtype: torch.dtype = torch.float32
    std: float = 1.0
    t_min: Optional[int] = None  # None = full lengths
    u_min: Optional[int] = None
    fastemit_lambda: float = 0.0
    clamp: float = -1.0
    durations: List[int] = field(default_factory=list)
    sigma: float = 0.0
    # multi-blank: durations of the big blanks; V then counts tokens + big blanks + the standard blank
    big_blank_durations: List[int] = field(default_factory=list)
    zipf_labels: bool = False

    @property
    def D(self):
        return len(self.durations)

    @property
    def blank(self):
        return self.V - 1

    @property
    def elems(self):
        return self.B * self.T * self.U * (self.V + self.D)


CONFIGS = [
    Config("cfg1_rnnt_B4_T50_U21_V129_f32", 4, 50, 21, 129),
    Config("cfg2_rnnt_B16_T375_U121_V1025_f32", 16, 375, 121, 1025, t_min=200, u_min=40),
    Config("cfg3_rnnt_B32_T750_U201_V1025_bf16", 32, 750, 201, 1025, dtype=torch.bfloat16, std=2.0, t_min=400,
           u_min=80, fastemit_lambda=0.001),
    Config("cfg4_tdt_B16_T375_U121_V1025_D5_f32", 16, 375, 121, 1025, t_min=200, u_min=40,
           durations=[0, 1, 2, 3, 4], sigma=0.05),
    Config("cfg5_rnnt_B8_T250_U101_V16385_f32", 8, 250, 101, 16385, t_min=150, u_min=30, fastemit_lambda=0.001,
           clamp=5.0, zipf_labels=True),
    # the north-star shape with three big blanks appended to the vocabulary
    Config("cfg6_multiblank_B16_T375_U121_V1028_f32", 16, 375, 121, 1028, t_min=200, u_min=40,
           big_blank_durations=[2, 4, 8], sigma=0.05),
]  # fmt: skip


def make_lengths(cfg, gen):
    if cfg.t_min is None:
        act_lens = torch.full((cfg.B,), cfg.T, dtype=torch.int64)
        label_lens = torch.full((cfg.B,), cfg.U - 1, dtype=torch.int64)
        return act_lens, label_lens
    act_lens = torch.randint(cfg.t_min, cfg.T + 1, (cfg.B,), generator=gen, dtype=torch.int64)
    label_lens = torch.randint(cfg.u_min, cfg.U, (cfg.B,), generator=gen, dtype=torch.int64)
    act_lens[0] = cfg.T
    label_lens[cfg.B - 1] = cfg.U - 1
    return act_lens, label_lens


def make_labels(cfg, gen):
    n_tokens = cfg.V - 1 - len(cfg.big_blank_durations)
    if not cfg.zipf_labels:
        return torch.randint(0, n_tokens, (cfg.B, cfg.U - 1), generator=gen, dtype=torch.int64)
    # Zipf(s = 1.1) over [0, n_tokens) by inverse-CDF sampling of a seeded uniform
    ranks = torch.arange(1, n_tokens + 1, dtype=torch.float64)
    cdf = torch.cumsum(ranks.pow(-1.1), 0)
    cdf = cdf / cdf[-1]
    u = torch.rand(cfg.B, cfg.U - 1, generator=gen, dtype=torch.float64)
    return torch.searchsorted(cdf, u).clamp_(max=n_tokens - 1).to(torch.int64)


def make_inputs(index, device="cpu", generate_on_device=False):
    """(cfg, acts, labels, act_lens, label_lens) for configuration `index` (0-based).

    Labels and lengths always come from the CPU generator.  acts are drawn utterance by
    utterance as fp32 ~ N(0, std) and rounded to cfg.dtype; with generate_on_device they are
    drawn by a generator of `device` seeded the same way (much faster for the multi-GB
    configurations; the values then depend on the device's generator, which is fine for
    checks that read the tensor back)."""
    cfg = CONFIGS[index]
    gen = torch.Generator().manual_seed(1234 + index)
    labels = make_labels(cfg, gen)
    act_lens, label_lens = make_lengths(cfg, gen)
    acts = torch.empty(cfg.B, cfg.T, cfg.U, cfg.V + cfg.D, dtype=cfg.dtype, device=device)
    if generate_on_device:
        gen = torch.Generator(device=device).manual_seed(1234 + index)
    for b in range(cfg.B):
        x = torch.randn(cfg.T, cfg.U, cfg.V + cfg.D, generator=gen, dtype=torch.float32, device=gen.device)
        if cfg.std != 1.0:
            x *= cfg.std
        acts[b].copy_(x.to(cfg.dtype))
    return cfg, acts, labels.to(device), act_lens.to(device), label_lens.to(device)


def algorithmic_bytes(cfg, act_lens, label_lens):
    """Bytes the loss must move per fwd+bwd call: valid logits read twice, every gradient element
    written once, plus the per-cell lattice state (24 bytes per valid cell)."""
    s = torch.tensor([], dtype=cfg.dtype).element_size()
    width = cfg.V + cfg.D
    c_valid = int((act_lens.cpu() * (label_lens.cpu() + 1)).sum())
    cells = cfg.B * cfg.T * cfg.U
    return dict(
        total=2 * c_valid * width * s + cells * width * s + 24 * c_valid,
        denom_gather=c_valid * width * s + 12 * c_valid,
        grad_stream=c_valid * width * s + cells * width * s,  # gradient pass that also zero-fills the padding
        grad_valid=2 * c_valid * width * s,  # gradient pass over the valid rows only
        zero_padding=(cells - c_valid) * width * s,
        c_valid=c_valid,
        cells=cells,
    )
