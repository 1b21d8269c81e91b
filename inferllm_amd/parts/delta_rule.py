"""The gated delta rule: a recurrent mixer with a matrix of state per head."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..cache.manager import StateSpec
from ..kernels import ops
from ..weights.loader import TensorWant
from .base import Mixer, StepContext, register_part


@register_part("mixer", "gated_delta_rule")
class GatedDeltaRule(Mixer):
    """Per head a state S [key_dim, value_dim] (float32) that every token decays, corrects and reads:

        q, k = unit(silu(conv(W_q h))), unit(silu(conv(W_k h)))    per q/k head; q also * key_dim^-1/2
        v    = silu(conv(W_v h))                                     per head
        beta = sigmoid(W_b h),   g = exp(-exp(A_log) * softplus(a + dt_bias))
        S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
        out  = W_o (o / rms(o) * norm * gate)

    conv filters every channel over time with `conv` taps of its own, the last tap on the token
    itself and nothing but zeros ahead of the sequence's first token; unit(x) = x / sqrt(sum x^2 +
    1e-6); rms is taken over a head's value dims with `eps`.  Head h reads q/k head h / (num_heads / num_kv_heads).  `decay` "head": one g a head,
    "channel": one a head and key channel, acting on the rows of S.  Its pre-activation a is W_a h,
    or with `decay_rank` > 0 the low-rank W_a2 (W_a1 h).  `gate` "silu" or "sigmoid" of W_g h, or
    with `gate_rank` > 0 of W_g2 (W_g1 h), per head and value dim.

    Kept per sequence: S, and the last conv - 1 inputs of the convolution.  A step goes on from
    whatever the slot holds (zeros in a fresh one), by one token or by many.  Everything that
    enters the recurrence is float32; the projections take the engine's dtype.
    """

    graph_safe_prompts = True
    takes_continuations = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, key_dim: int,
                 value_dim: int, conv: int, eps: float, decay: str = "head", decay_rank: int = 0,
                 gate: str = "silu", gate_rank: int = 0, tensors=None):
        super().__init__(tensors)
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads are not a multiple of {num_kv_heads} q/k heads")
        if decay not in ("head", "channel") or gate not in ops.DELTA_GATES:
            raise ValueError(f"gated delta rule: decay {decay!r} or gate {gate!r} is unknown")
        if not 1 <= int(conv) <= 8:
            raise ValueError(f"gated delta rule: {conv} taps; the kernels take 1 to 8")
        if key_dim > 256 or value_dim > 256:
            raise ValueError(f"gated delta rule: head sizes {key_dim}, {value_dim} are beyond the kernels' limit of 256")
        self.E, self.H, self.G = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.dk, self.dv, self.taps, self.eps = int(key_dim), int(value_dim), int(conv), float(eps)
        self.per_channel, self.gate = decay == "channel", gate
        self.ra, self.rg = int(decay_rank), int(gate_rank)
        self.DW = self.dk if self.per_channel else 1
        self.C = 2 * self.G * self.dk + self.H * self.dv          # channels of the convolution

    def shapes(self) -> Dict[str, TensorWant]:
        E, H, G, dk, dv = self.E, self.H, self.G, self.dk, self.dv
        keep = dict(keep_stored=True)
        out = {"q": TensorWant((G * dk, E)), "k": TensorWant((G * dk, E)), "v": TensorWant((H * dv, E)),
               "q_conv": TensorWant((G * dk, self.taps), **keep),
               "k_conv": TensorWant((G * dk, self.taps), **keep),
               "v_conv": TensorWant((H * dv, self.taps), **keep),
               "b": TensorWant((H, E)), "A_log": TensorWant((H,), **keep),
               "dt_bias": TensorWant((H * self.DW,), **keep),
               "norm": TensorWant((dv,), init="ones_normal", **keep),
               "o": TensorWant((E, H * dv))}
        if self.ra:
            out.update(a1=TensorWant((self.ra, E)), a2=TensorWant((H * self.DW, self.ra)))
        else:
            out["a"] = TensorWant((H * self.DW, E))
        if self.rg:
            out.update(g1=TensorWant((self.rg, E)), g2=TensorWant((H * dv, self.rg)))
        else:
            out["g"] = TensorWant((H * dv, E))
        return out

    def state_spec(self):
        return {"S": StateSpec((self.H, self.dk, self.dv), torch.float32),
                "tail": StateSpec((max(self.taps - 1, 1), self.C), None)}

    def load(self, tensors) -> None:
        from .attention import _fuse
        take = lambda n: self._take(tensors, n)
        f32 = lambda n: take(n).to(torch.float32).contiguous()
        H, dv, DW = self.H, self.dv, self.DW
        # one product for everything that reads h at full rank: [q | k | v | b | a? | g?]
        rows = [take("q"), take("k"), take("v"), take("b")]
        self.b_off = self.C
        at = self.C + H
        self.a_off = self.z_off = 0
        if not self.ra:
            rows.append(take("a")); self.a_off = at; at += H * DW
        if not self.rg:
            rows.append(take("g")); self.z_off = at; at += H * dv
        self.w_in = ops.decode_weight(_fuse(rows), "plain", self.decode_copies)
        # the low-rank parts: [a1 ; g1] from h, then one block-diagonal product [a2 0 ; 0 g2]
        self.w_low = self.w_up = None
        if self.ra or self.rg:
            low, n_out = [], (H * DW if self.ra else 0) + (H * dv if self.rg else 0)
            up = torch.zeros((n_out, self.ra + self.rg), dtype=take("q").dtype, device=take("q").device)
            if self.ra:
                low.append(take("a1")); up[: H * DW, : self.ra] = take("a2")
            if self.rg:
                low.append(take("g1")); up[n_out - H * dv:, self.ra:] = take("g2")
                self.z_off = n_out - H * dv
            self.w_low = ops.decode_weight(_fuse(low), "plain", self.decode_copies)
            self.w_up = ops.decode_weight(up.contiguous(), "plain", self.decode_copies)
        self.conv_w = torch.cat([f32("q_conv"), f32("k_conv"), f32("v_conv")], dim=0).contiguous()
        self.a_log, self.dt_bias, self.norm_w = f32("A_log"), f32("dt_bias"), take("norm").contiguous()
        self.w_o = ops.decode_weight(take("o").contiguous(), "plain", self.decode_copies)

    def tunables(self):
        return (("plain", self.w_o, {}),)

    def forward(self, h, ctx: StepContext, line, writes_cache, position):
        P = ops.linear(h, self.w_in)
        P2 = ops.linear(ops.linear(h, self.w_low), self.w_up) if self.w_low is not None else None
        state = ctx.cache.state_line(line)
        S, tail = state["S"], state["tail"]
        qn, kn, vv, beta, dec = ops.delta_prepare(
            P, self.b_off, P2 if self.ra else P, self.a_off, self.conv_w, tail, ctx.row_slot,
            self.a_log, self.dt_bias, self.G, self.H, self.dk, self.dv, self.per_channel,
            update_tail=not ctx.prefill)
        if ctx.prefill:
            ops.delta_conv_tail(P, tail, ctx.cu_seqlens, ctx.seq_slot, ctx.n_seqs, self.taps)
        o = ops.delta_scan(qn, kn, vv, beta, dec, S, ctx.cu_seqlens, ctx.seq_slot, ctx.n_seqs,
                           ctx.max_rows if ctx.prefill else 1)
        y = ops.delta_finish(o, self.norm_w, P2 if self.rg else P, self.z_off, self.gate, self.eps,
                             ctx.act_dtype)
        return ops.linear(y, self.w_o)
