"""Attention over one low-rank latent row per token (keys and values are made from it)."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..cache.manager import KVSpec, TokenTensor
from ..kernels import ops
from ..weights.loader import TensorWant
from .attention import _fuse
from .base import Mixer, StepContext, register_part


@register_part("mixer", "latent_attention")
class LatentAttention(Mixer):
    """Attention whose keys and values come from a latent row c = norm(W_dkv h)[:rank]:

        q_h = (W_q h)_h = [q_plain (head_dim) | q_rot (rot_dim)],  k_rot = (W_dkv h)[rank:]
        score_h(i, j) = (q_plain_h(i) . W_uk,h c(j) + rot(q_rot_h(i)) . rot(k_rot(j))) * scale
        out_h(i) = sigmoid((W_g h(i))_h) * sum_j softmax_j(score_h(i, j)) W_uv,h c(j)

    over the keys j <= i (with `window`: the last `window` of them), then W_o on the heads side
    by side.  k_rot is one vector a token, shared by all heads; the rotation is the block's
    position part (pairs (2i, 2i+1) of the first `rotary_dim` dims of the rot part).  The cache
    keeps c and the rotated k_rot of a token as one row of `rank + rot_dim`.

    Whole prompts make every head's keys and values from the step's own latent rows and use the
    prompt attention kernels (heads padded to one common width).  Single tokens, and rows that go
    on from tokens of earlier steps, walk the cached latent rows instead: the query is taken
    through W_uk first and the weighted sum of latent rows through W_uv afterwards, which is the
    same sum in another order.  `gated` False leaves the output gate out.
    """

    graph_safe_prompts = True
    # rows that go on from earlier tokens are each treated as a single token over the cache, which
    # holds the step's own rows by then (a window's ring is kept from wrapping by the step function)
    takes_continuations = True

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, rot_dim: int, value_dim: int,
                 rank: int, softmax_scale: float, eps: float, window: Optional[int] = None,
                 gated: bool = True, tensors=None):
        super().__init__(tensors)
        self.E, self.H = int(hidden_size), int(num_heads)
        self.dn, self.dr, self.dv, self.R = int(head_dim), int(rot_dim), int(value_dim), int(rank)
        if min(self.E, self.H, self.dv, self.R) <= 0 or self.dn < 0 or self.dr < 0 or self.dn + self.dr <= 0:
            raise ValueError("latent attention: sizes must be positive")
        if self.R > 1024:
            raise ValueError(f"latent attention: rank {self.R} is beyond the kernels' limit of 1024")
        if max(self.dn + self.dr, self.dv) > 256:
            raise ValueError("latent attention: a head wider than 256 is beyond the attention kernels")
        self.scale, self.eps = float(softmax_scale), float(eps)
        self.window = int(window) if window else None
        self.gated = bool(gated)
        self.q_cols = self.H * (self.dn + self.dr)
        self.gate_off = self.q_cols + self.R + self.dr
        self.w_in = self.w_up = self.w_uk = self.w_uv = self.w_o = self.norm_w = None
        # set by `load` (which sees the engine's dtype): keep the latent rows a second time,
        # transposed, for the single-token kernel on the matrix cores
        self.transposed = False

    def shapes(self) -> Dict[str, TensorWant]:
        out = {"q": TensorWant((self.q_cols, self.E)),
               "dkv": TensorWant((self.R + self.dr, self.E)),
               "dkv_norm": TensorWant((self.R,), init="ones_normal", keep_stored=True),
               "uk": TensorWant((self.H * self.dn, self.R)),
               "uv": TensorWant((self.H * self.dv, self.R)),
               "o": TensorWant((self.E, self.H * self.dv))}
        if self.gated:
            out["g"] = TensorWant((self.H, self.E))
        return out

    def kv_spec(self) -> KVSpec:
        kept = (TokenTensor("latent", (self.R + self.dr,)),)
        if self.transposed:
            kept += (TokenTensor("latent_t", (self.R, 1)),)     # stored [page][dim][row][1]
        return KVSpec("window" if self.window else "full", kept, self.window)

    def head_width(self, dtype: torch.dtype) -> int:
        """The common width the heads are padded to for the prompt attention kernels."""
        need = max(self.dn + self.dr, self.dv)
        step = 32 if dtype == torch.float32 and need <= 128 else 16
        return -(-need // step) * step

    def load(self, tensors) -> None:
        if self.position is not None:
            if getattr(self.position, "pairing", None) != "interleaved":
                raise ValueError("latent attention rotates pairs (2i, 2i+1): the block's position part must say so")
            if self.position.head_dim != self.dr or self.position.rotary_dim > self.dr:
                raise ValueError("latent attention: the position part must be made for the rot part of a head")
        ins = [self._take(tensors, "q"), self._take(tensors, "dkv")]
        if self.gated:
            ins.append(self._take(tensors, "g"))
        self.w_in = ops.decode_weight(_fuse(ins), "plain", self.decode_copies)
        self.w_uk = self._take(tensors, "uk").contiguous()
        self.w_uv = self._take(tensors, "uv").contiguous()
        self.w_up = _fuse([self.w_uk, self.w_uv])
        self.w_o = ops.decode_weight(self._take(tensors, "o").contiguous(), "plain", self.decode_copies)
        self.norm_w = self._take(tensors, "dkv_norm").contiguous()
        self.transposed = (self.w_uk.dtype == torch.bfloat16 and self.R % 16 == 0 and self.R <= 512
                           and (self.R + self.dr) % 8 == 0)

    def forward(self, h, ctx: StepContext, line, writes_cache, position):
        H, dn, dr, dv, R = self.H, self.dn, self.dr, self.dv, self.R
        kept, group = ctx.cache.token_line(line)
        cache, cache_t = kept["latent"], kept.get("latent_t")
        if cache_t is not None and not ops.latent_decode_mfma_fits(cache, cache_t, R, dr, group.page_size):
            cache_t = None
        window = self.window or 0
        table = position.table(ctx.device) if position is not None else None
        rot = position.rotary_dim if position is not None else 0
        y = ops.linear(h, self.w_in)
        if not self.gated:
            y = torch.cat([y, y.new_full((y.shape[0], H), 30.0)], dim=1)       # sigmoid(30) = 1
        whole = ctx.prefill and not ctx.continues
        if whole:
            c, kr = ops.latent_rope_store(
                y, H, dn, dr, R, rot, table, self.norm_w, self.eps, ctx.row_pos, ctx.row_slot,
                ctx.cache.slot_len, cache if writes_cache else None, group.table, group.page_size,
                group.ring, want_rows=True, cache_t=cache_t if writes_cache else None)
            if writes_cache:
                ctx.exchange[("latent_rows", line)] = (c, kr)
            else:
                c, kr = ctx.exchange[("latent_rows", line)]    # of the run that stored this line
            P = self.head_width(y.dtype)
            packed = ops.latent_pack(y, ops.linear(c, self.w_up), kr, H, dn, dr, dv, P)
            a = ops.attn_prefill(packed, ctx.cu_seqlens, ctx.n_seqs, ctx.max_len, H, H, P,
                                 self.scale, window)
            o = ops.latent_gate(a, y, self.gate_off, H, dv, P)
        else:
            # rows that walk the cache: the store of the row and the queries against latent rows
            # in one launch (a run that only reads the line rotates its queries and stores nothing)
            qa_dtype = torch.bfloat16 if cache_t is not None else torch.float32
            if writes_cache:
                qa = ops.latent_store_absorb(y, H, dn, dr, R, rot, table, self.norm_w, self.eps,
                                             ctx.row_pos, ctx.row_slot, cache, group.table,
                                             group.page_size, group.ring, self.w_uk, qa_dtype, cache_t)
            else:
                ops.latent_rope_store(y, H, dn, dr, R, rot, table, self.norm_w, self.eps, ctx.row_pos,
                                      ctx.row_slot, None, None, group.table, group.page_size,
                                      group.ring, want_rows=False)
                qa = ops.latent_absorb_q(y, self.w_uk, H, dn, dr, R, qa_dtype)
            longest = min(ctx.max_len, window) if window else ctx.max_len
            nsplit = ops.latent_decode_splits(y.shape[0], H, longest, mfma=cache_t is not None)
            if ctx.prefill:
                # every row is a token of its own over the cache: it sees the keys up to its position
                slots, lens, more = ctx.row_slot, ctx.row_pos, 1
            else:
                slots, lens, more = ctx.seq_slot, ctx.seq_len, 0
            o = ops.latent_attn_decode(qa, y, self.w_uv, self.gate_off, cache, group.table,
                                       group.page_size, group.ring, slots, lens, more, H, dr, R, dv,
                                       self.scale, window, nsplit, cache_t)
        return ops.linear(o, self.w_o)
