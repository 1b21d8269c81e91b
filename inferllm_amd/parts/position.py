"""Position encodings.  Every packed row carries its absolute position; an
encoding turns it into a change of q and k (rotary) or does nothing."""
from __future__ import annotations

import math
from typing import Dict, Optional, Tuple

import torch

from ..kernels import ops
from .base import PositionEncoding, StepContext, register_part

_TABLES: Dict[Tuple, torch.Tensor] = {}


def scaled_frequencies(theta: float, rotary_dim: int, scaling: Optional[dict]):
    """(frequencies float64 [rotary_dim/2], gain of cos and sin) with the long-context scaling
    that keeps fast-turning pairs and slows the slow ones: `scaling` = {factor, original, fast,
    slow}.  d(n) = rotary_dim * ln(original / (2 pi n)) / (2 ln theta) is the (fractional) pair
    count at which a wave makes n turns over `original` positions; between lo = floor(d(fast)) and
    hi = ceil(d(slow)) the frequency goes linearly from f to f / factor, and cos and sin are
    multiplied by 0.1 ln(factor) + 1."""
    i = torch.arange(rotary_dim // 2, dtype=torch.float64)
    f = torch.pow(torch.tensor(float(theta), dtype=torch.float64), -2.0 * i / rotary_dim)
    if not scaling:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def pairs_at(turns: float) -> float:
        return rotary_dim * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(theta))
    lo = max(math.floor(pairs_at(float(scaling["fast"]))), 0)
    hi = min(math.ceil(pairs_at(float(scaling["slow"]))), rotary_dim - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotary_table(theta: float, rotary_dim: int, max_positions: int, device,
                 scaling: Optional[dict] = None) -> torch.Tensor:
    """cos and sin of p * theta^(-2i/rotary_dim), float32 [max_positions, rotary_dim/2, 2]; with
    `scaling` the frequencies and the gain of `scaled_frequencies`.

    Angles are formed in double precision, as the reference's plain kernel does
    (src/kern/naive/naive.cpp:396-399), and rounded once.  Tables are shared by all
    layers with the same constants.
    """
    key = (float(theta), int(rotary_dim), int(max_positions), str(device),
           tuple(sorted((k, float(v)) for k, v in scaling.items())) if scaling else None)
    t = _TABLES.get(key)
    if t is None:
        inv, gain = scaled_frequencies(theta, rotary_dim, scaling)
        ang = torch.arange(max_positions, dtype=torch.float64)[:, None] * inv[None, :]
        t = (torch.stack([torch.cos(ang), torch.sin(ang)], dim=-1) * gain).to(torch.float32).to(device)
        _TABLES[key] = t.contiguous()
        t = _TABLES[key]
    return t


@register_part("position", "rotary")
class Rotary(PositionEncoding):
    """Rotation of pairs of q and k by position-dependent angles.

    pairing "half": pairs (i, i + head_dim/2) (src/kern/naive/naive.cpp:389-414, the
    LLaMA-2 graph's RotMode::ModelRotHalf); "interleaved": pairs (2i, 2i+1)
    (naive.cpp:415-440).  theta, rotary_dim and max_positions are parameters; `scaling`
    ({factor, original, fast, slow}, see `scaled_frequencies`) stretches the slow pairs for
    contexts longer than `original`.
    """

    graph_safe_prompts = True

    def __init__(self, head_dim: int, rotary_dim: int, theta: float, pairing: str,
                 max_positions: int, scaling: Optional[dict] = None, tensors=None):
        super().__init__(tensors)
        if pairing not in ("half", "interleaved"):
            raise ValueError(f"unknown rotary pairing {pairing!r}")
        if rotary_dim % 2 or rotary_dim > head_dim or rotary_dim <= 0:
            raise ValueError(f"rotary_dim {rotary_dim} must be even and within head_dim {head_dim}")
        self.head_dim, self.rotary_dim = int(head_dim), int(rotary_dim)
        self.theta, self.pairing, self.max_positions = float(theta), pairing, int(max_positions)
        if scaling:
            lacking = [k for k in ("factor", "original", "fast", "slow") if k not in scaling]
            if lacking or not float(scaling["factor"]) > 0 or not float(scaling["original"]) > 0:
                raise ValueError(f"rotary scaling needs positive factor and original, and fast and slow: {scaling!r}")
        self.scaling = dict(scaling) if scaling else None

    def table(self, device) -> torch.Tensor:
        return rotary_table(self.theta, self.rotary_dim, self.max_positions, device, self.scaling)

    def on_qkv(self, qkv, ctx: StepContext, nh, nkv, hd, kcache, vcache, group) -> None:
        ops.rope_store(qkv, self.table(ctx.device), self.rotary_dim,
                       0 if self.pairing == "half" else 1, ctx.row_pos, ctx.row_slot,
                       ctx.cache.slot_len if ctx.prefill else None, kcache, vcache,
                       group.table if group is not None else None,
                       group.page_size if group is not None else 1,
                       group.ring if group is not None else 0, nh, nkv, hd)


    def qkv_tile_mode(self, head_dim: int) -> str:
        # the fused product + rotation + store kernels pair a row with its partner head_dim / 2 on
        fused = self.pairing == "half" and self.rotary_dim == head_dim and head_dim % 16 == 0
        return "qkv" if fused else "plain"

    def project_qkv(self, h, w_qkv, ctx: StepContext, nh, nkv, hd, kcache, vcache, group):
        if (not ctx.prefill and kcache is not None and self.pairing == "half"
                and self.rotary_dim == hd and ops.qkv_rope_store_fits(h, w_qkv, hd)
                and kcache.dtype == torch.bfloat16):
            return ops.qkv_rope_store(h, w_qkv, self.table(ctx.device), ctx.row_pos, ctx.row_slot,
                                      kcache, vcache, group.table, group.page_size, group.ring,
                                      nh, nkv, hd)
        return super().project_qkv(h, w_qkv, ctx, nh, nkv, hd, kcache, vcache, group)


@register_part("position", "none")
class NoPosition(PositionEncoding):
    """No encoding: q and k stay as they are; k and v are still stored."""

    graph_safe_prompts = True

    def on_qkv(self, qkv, ctx: StepContext, nh, nkv, hd, kcache, vcache, group) -> None:
        ops.rope_store(qkv, None, 0, 0, ctx.row_pos, ctx.row_slot,
                       ctx.cache.slot_len if ctx.prefill else None, kcache,
                       vcache, group.table if group is not None else None,
                       group.page_size if group is not None else 1,
                       group.ring if group is not None else 0, nh, nkv, hd)
