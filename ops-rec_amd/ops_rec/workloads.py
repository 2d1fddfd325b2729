"""Synthetic jagged batches for the named HSTU attention configurations.

Used by the benchmark and by the parity tests so that both run the same seeded inputs.
Lengths always come from a seeded CPU generator; the tensors are drawn with a seeded
``torch.Generator`` on the device asked for (the CPU by default, so that the CPU oracle and the
GPU operator see identical bits; the large configurations are drawn on the GPU directly).

Configurations (lengths are per sequence, drawn uniformly unless stated):

* ``C1``  fp32-able tiny case: batch 4, heads 2, dim 64, L in [16, 128], alpha 1/8, no rab.
* ``C2``  headline: bf16, batch 32, heads 4, dim 128, L in [256, 1024], max 1024, alpha 128^-0.5,
          silu_scale 1/1024, no rab.
* ``C3``  bf16, batch 16, heads 4, dim 128, L in [512, 2048], rab [16, 4, 2048, 2048] ~ N(0, 0.02).
* ``C4``  bf16, batch 16, heads 8, dim 128, L in [1024, 4096], rab, num_target in [1, 64]
          (group size 1), 8 context tokens.
* ``C5``  batch 64, heads 8, dim 128, L ~ clip(Zipf(1.2), 32, 8192), no rab (quantised variant).
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional

import numpy as np
import torch


@dataclass
class Workload:
    name: str
    q: torch.Tensor
    k: torch.Tensor
    v: torch.Tensor
    seq_offset: torch.Tensor
    max_seq_len: int
    silu_scale: float
    alpha: float
    attn_bias: Optional[torch.Tensor] = None
    mask: Optional[torch.Tensor] = None
    mask_type: int = 0
    num_context: Optional[torch.Tensor] = None
    num_target: Optional[torch.Tensor] = None
    target_group_size: int = 0
    seq_offset_k: Optional[torch.Tensor] = None
    max_seq_len_k: Optional[int] = None
    lengths: list = field(default_factory=list)

    def to(self, device) -> "Workload":
        def mv(t):
            return None if t is None else t.to(device)

        return Workload(
            self.name, mv(self.q), mv(self.k), mv(self.v), mv(self.seq_offset), self.max_seq_len, self.silu_scale,
            self.alpha, mv(self.attn_bias), mv(self.mask), self.mask_type, mv(self.num_context),
            mv(self.num_target), self.target_group_size, mv(self.seq_offset_k), self.max_seq_len_k,
            list(self.lengths),
        )  # fmt: skip

    def op_args(self):
        """Positional arguments of ``hstu_jagged.equal`` (or ``.delta`` when K offsets differ)."""
        if self.seq_offset_k is None:
            return (self.q, self.k, self.v, self.mask, self.attn_bias, self.mask_type, self.max_seq_len,
                    self.silu_scale, self.seq_offset, self.num_context, self.num_target, self.target_group_size,
                    self.alpha)  # fmt: skip
        return (self.q, self.k, self.v, self.mask, self.attn_bias, self.mask_type, self.max_seq_len,
                self.max_seq_len_k, self.silu_scale, self.seq_offset, self.seq_offset_k, self.num_context,
                self.num_target, self.target_group_size, self.alpha)  # fmt: skip

    def oracle_kwargs(self):
        return dict(
            mask=self.mask, attn_bias=self.attn_bias, mask_type=self.mask_type, max_seq_len=self.max_seq_len,
            max_seq_len_k=self.max_seq_len_k if self.max_seq_len_k is not None else self.max_seq_len,
            silu_scale=self.silu_scale, seq_offset=self.seq_offset, seq_offset_k=self.seq_offset_k,
            num_context=self.num_context, num_target=self.num_target, target_group_size=self.target_group_size,
            alpha=self.alpha,
        )  # fmt: skip


def _offsets(lengths, dtype=torch.int32) -> torch.Tensor:
    return torch.tensor([0] + list(np.cumsum(lengths)), dtype=dtype)


def make(
    name: str,
    *,
    batch: int,
    heads: int,
    dim: int,
    lo: int,
    hi: int,
    max_seq_len: Optional[int] = None,
    dtype=torch.bfloat16,
    std: float = 0.1,
    rab_std: Optional[float] = None,
    alpha: Optional[float] = None,
    silu_scale: float = 0.0,
    num_context: int = 0,
    max_target: int = 0,
    target_group_size: int = 0,
    heads_k: Optional[int] = None,
    dim_v: Optional[int] = None,
    lengths: Optional[list] = None,
    index_dtype=torch.int32,
    seed: int = 0,
    device="cpu",
) -> Workload:
    """Lengths are always drawn on the CPU (same values whatever ``device`` is); the tensors are
    drawn on ``device`` -- pass a GPU for sizes whose CPU generation would take long (the
    values then differ from the CPU-generated ones, which only matters for oracle comparisons)."""
    g_len = torch.Generator().manual_seed(seed)
    if lengths is None:
        lengths = torch.randint(lo, hi + 1, (batch,), generator=g_len).tolist()
    g = torch.Generator(device=device).manual_seed(seed + 1)
    batch = len(lengths)
    max_seq_len = max_seq_len or max(lengths)
    heads_k = heads_k or heads
    dim_v = dim_v or dim
    total = int(sum(lengths))
    q = (torch.randn(total, heads, dim, generator=g, device=device) * std).to(dtype)
    k = (torch.randn(total, heads_k, dim, generator=g, device=device) * std).to(dtype)
    v = (torch.randn(total, heads_k, dim_v, generator=g, device=device) * std).to(dtype)
    bias = None
    if rab_std is not None:
        bias = torch.empty(batch, heads, max_seq_len, max_seq_len, dtype=dtype, device=device)
        for b in range(batch):  # per sequence, so the fp32 temporary stays small
            bias[b] = (torch.randn(heads, max_seq_len, max_seq_len, generator=g, device=device) * rab_std).to(dtype)
    ctx = torch.full((batch,), num_context, dtype=index_dtype, device=device) if num_context else None
    tgt = None
    if max_target:
        tgt = torch.randint(1, max_target + 1, (batch,), generator=g_len).to(index_dtype).to(device)
    return Workload(
        name=name, q=q, k=k, v=v, seq_offset=_offsets(lengths, index_dtype).to(device), max_seq_len=max_seq_len,
        silu_scale=silu_scale, alpha=(dim**-0.5 if alpha is None else alpha), attn_bias=bias,
        num_context=ctx, num_target=tgt, target_group_size=target_group_size, lengths=list(lengths),
    )  # fmt: skip


E4M3_MAX = 448.0


def quantize_fp8(x: torch.Tensor):
    """``x[T, H, d]`` -> (``float8_e4m3fn`` tensor, ``descale[H]`` float32) with one scale per head,
    ``descale = absmax / 448``: the quantisation configuration C5 is defined with."""
    absmax = x.abs().amax(dim=(0, 2)).clamp_min(1e-12).float()
    descale = absmax / E4M3_MAX
    x8 = (x.float() / descale[None, :, None]).clamp(-E4M3_MAX, E4M3_MAX).to(torch.float8_e4m3fn)
    return x8, descale


def zipf_lengths(batch: int, s: float = 1.2, lo: int = 32, hi: int = 8192, seed: int = 0) -> list:
    rng = np.random.default_rng(seed)
    return np.clip(rng.zipf(s, size=batch), lo, hi).astype(np.int64).tolist()


def config(name: str, dtype=None, seed: int = 0, device="cpu") -> Workload:
    """One of the named configurations ``C1`` .. ``C5``."""
    if name == "C1":
        return make("C1", batch=4, heads=2, dim=64, lo=16, hi=128, dtype=dtype or torch.float32, alpha=1.0 / 8.0,
                    seed=seed, device=device)  # fmt: skip
    if name == "C2":
        return make("C2", batch=32, heads=4, dim=128, lo=256, hi=1024, max_seq_len=1024, dtype=dtype or torch.bfloat16,
                    silu_scale=1.0 / 1024.0, seed=seed, device=device)  # fmt: skip
    if name == "C3":
        return make("C3", batch=16, heads=4, dim=128, lo=512, hi=2048, max_seq_len=2048, dtype=dtype or torch.bfloat16,
                    rab_std=0.02, seed=seed, device=device)  # fmt: skip
    if name == "C4":
        return make("C4", batch=16, heads=8, dim=128, lo=1024, hi=4096, max_seq_len=4096,
                    dtype=dtype or torch.bfloat16, rab_std=0.02, num_context=8, max_target=64, target_group_size=1,
                    seed=seed, device=device)  # fmt: skip
    if name == "C5":
        lengths = zipf_lengths(64, seed=seed)
        return make("C5", batch=64, heads=8, dim=128, lo=0, hi=0, lengths=lengths, max_seq_len=8192,
                    dtype=dtype or torch.bfloat16, seed=seed, device=device)  # fmt: skip
    raise ValueError(f"unknown configuration {name!r}")
