"""Kukupel: a decoder whose layers mix tokens with a gated delta rule, alone or beside softmax
attention with capped scores, feed a mixture of clamped experts, and keep several residual
streams that every sublayer reads as one weighted sum and writes back into all at once.

This file holds what is specific to the design: the keys of its config.json, their checks, the
tensor names of its checkpoints and the translation into a `ModelSpec` of generic parts.

    config.json
      architecture: "Kukupel"; vocab; width; norm.eps; streams?
      layers: [{type: "parallel",
                mixer: {left: {heads, kv_heads, dim, vdim, scale, softcap},
                        right: {heads, kv_heads, dim, vdim, conv}, left_scale, right_scale},
                mlp: null | {kind: "moe", expert: {ff, limit}, router: {experts, top}}}
             | {type: "delta", mixer: {heads, kv_heads, dim, vdim, conv}, mlp: ...}, ...]
    tensors
      embed; final.norm; l<i>.norm1, l<i>.norm2; l<i>.hc<q>.{in, out, mix} (with streams)
      attention (l<i>.mix.left.): q, k, v, o
      delta rule (l<i>.mix. or l<i>.mix.right.): q, k, v, {q,k,v}.conv, b, A_log, dt_bias, norm, o
          and a, g (type "delta": a decay a head, a silu gate) or a1, a2, g1, g2 (beside attention:
          a decay a head and key channel and a sigmoid gate, both through a low rank that the
          tensors' shapes give)
      l<i>.mlp.{router, e<j>.{gate, up, down}}

The head is the embedding table.  Without `streams` a layer is the plain pre-norm arrangement,
x <- x + mixer(norm1(x)), x <- x + ff(norm2(x)).  Positions enter nowhere, so the configuration
has no limit of its own for them; `max_positions` (optional key) bounds a sequence's length and
defaults to 65,536.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import List, Optional

from ..config.registry import ConfigError, register_architecture
from ..config.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

DEFAULT_MAX_POSITIONS = 65536
# The low ranks of the decay and gate projections beside attention are no configuration keys:
# the stored tensors' shapes give them.  A configuration may state them (`mixer.right.decay_rank`,
# `gate_rank`); a model folder's are read from its tensors when the engine loads it.
DEFAULT_LOW_RANK = 24


def _get(d: dict, key: str, where: str, kind=None):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError(f"config.json of Kukupel lacks {where}{key}")
    v = d[key]
    if kind == "int":
        if not isinstance(v, int) or isinstance(v, bool) or v <= 0:
            raise ConfigError(f"{where}{key} must be a positive integer, got {v!r}")
    elif kind == "float":
        if isinstance(v, bool) or not isinstance(v, (int, float)) or not float(v) > 0:
            raise ConfigError(f"{where}{key} must be a positive number, got {v!r}")
    return v


def _heads(m: dict, at: str) -> None:
    for k in ("heads", "kv_heads", "dim", "vdim"):
        _get(m, k, at, "int")
    if m["heads"] % m["kv_heads"]:
        raise ConfigError(f"{at}heads {m['heads']} must be a multiple of kv_heads {m['kv_heads']}")


@register_architecture("Kukupel")
@dataclass
class KukupelConfig:
    vocab: int
    width: int
    eps: float
    streams: int = 0                      # 0: one residual stream, plain pre-norm layers
    layers: List[dict] = field(default_factory=list)
    max_positions: int = DEFAULT_MAX_POSITIONS
    unused_tensors: List[str] = field(default_factory=list)    # in the folder, without a part to act on
    mix_without_ff: List[int] = field(default_factory=list)    # layers without feed-forward that still mix

    architecture = "Kukupel"
    cli_type_names = ("kukupel",)

    # ------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, d: dict) -> "KukupelConfig":
        layers = _get(d, "layers", "")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("layers must be a list with at least one layer")
        streams = d.get("streams")
        if streams is not None and (not isinstance(streams, int) or isinstance(streams, bool)
                                    or not 1 <= streams <= 8):
            raise ConfigError(f"streams must be an integer from 1 to 8, got {streams!r}")
        cfg = cls(vocab=_get(d, "vocab", "", "int"), width=_get(d, "width", "", "int"),
                  eps=float(_get(_get(d, "norm", ""), "eps", "norm.", "float")),
                  streams=int(streams or 0), layers=copy.deepcopy(layers),
                  max_positions=int(d.get("max_positions", DEFAULT_MAX_POSITIONS)))
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.max_positions <= 0:
            raise ConfigError("max_positions must be positive")
        for i, layer in enumerate(self.layers):
            at = f"layers[{i}]."
            kind = _get(layer, "type", at)
            m = _get(layer, "mixer", at)
            if kind == "parallel":
                left, right = _get(m, "left", at + "mixer."), _get(m, "right", at + "mixer.")
                _heads(left, at + "mixer.left.")
                _get(left, "scale", at + "mixer.left.", "float")
                cap = left.get("softcap", 0) or 0
                if isinstance(cap, bool) or not isinstance(cap, (int, float)) or cap < 0:
                    raise ConfigError(f"{at}mixer.left.softcap must be a number >= 0, got {cap!r}")
                _heads(right, at + "mixer.right.")
                _get(right, "conv", at + "mixer.right.", "int")
                for k in ("left_scale", "right_scale"):
                    v = _get(m, k, at + "mixer.")
                    if isinstance(v, bool) or not isinstance(v, (int, float)):
                        raise ConfigError(f"{at}mixer.{k} must be a number, got {v!r}")
            elif kind == "delta":
                _heads(m, at + "mixer.")
                _get(m, "conv", at + "mixer.", "int")
            else:
                raise ConfigError(f"{at}type {kind!r} is not a mixer of this design (parallel, delta)")
            mlp = layer.get("mlp")
            if mlp is None:
                continue
            if _get(mlp, "kind", at + "mlp.") != "moe":
                raise ConfigError(f"{at}mlp.kind {mlp['kind']!r} is not a feed-forward of this design (moe)")
            r = _get(mlp, "router", at + "mlp.")
            n, top = _get(r, "experts", at + "mlp.router.", "int"), _get(r, "top", at + "mlp.router.", "int")
            if top > n:
                raise ConfigError(f"{at}mlp.router: {top} of {n} experts cannot be chosen")
            e = _get(mlp, "expert", at + "mlp.")
            _get(e, "ff", at + "mlp.expert.", "int")
            _get(e, "limit", at + "mlp.expert.", "float")

    def to_dict(self) -> dict:
        d = {"architecture": self.architecture, "layers": copy.deepcopy(self.layers),
             "norm": {"eps": self.eps}, "vocab": self.vocab, "width": self.width}
        if self.streams:
            d["streams"] = self.streams
        if self.max_positions != DEFAULT_MAX_POSITIONS:
            d["max_positions"] = self.max_positions
        return d

    def with_tensor_shapes(self, shapes: dict) -> "KukupelConfig":
        """The configuration with the low ranks that a folder's tensors have (`shapes`: tensor name
        -> shape), where the configuration does not state them."""
        cfg = copy.deepcopy(self)
        for i, layer in enumerate(cfg.layers):
            if layer.get("mlp") is None:
                # a layer without a feed-forward whose folder still holds the second sublayer's
                # tensors: its norm and its read and output weights have nothing to act on (they are
                # left in the file), its mix matrix still mixes the streams
                cfg.unused_tensors += [n for n in (f"l{i}.norm2", f"l{i}.hc2.in", f"l{i}.hc2.out") if n in shapes]
                if f"l{i}.hc2.mix" in shapes:
                    (cfg.mix_without_ff if self.streams else cfg.unused_tensors).append(
                        i if self.streams else f"l{i}.hc2.mix")
            if layer.get("type") != "parallel":
                continue
            right = layer["mixer"]["right"]
            for key, name in (("decay_rank", f"l{i}.mix.right.a1"), ("gate_rank", f"l{i}.mix.right.g1")):
                if key not in right and name in shapes:
                    right[key] = int(shapes[name][0])
        return cfg

    # ------------------------------------------------------------ translation
    def _delta(self, p: str, m: dict, beside_attention: bool) -> PartSpec:
        names = {k: p + k for k in ("q", "k", "v", "b", "A_log", "dt_bias", "norm", "o")}
        names.update({f"{k}_conv": f"{p}{k}.conv" for k in ("q", "k", "v")})
        params = {"hidden_size": self.width, "num_heads": m["heads"], "num_kv_heads": m["kv_heads"],
                  "key_dim": m["dim"], "value_dim": m["vdim"], "conv": m["conv"], "eps": self.eps}
        if beside_attention:
            params.update(decay="channel", decay_rank=int(m.get("decay_rank", DEFAULT_LOW_RANK)),
                          gate="sigmoid", gate_rank=int(m.get("gate_rank", DEFAULT_LOW_RANK)))
            names.update({k: p + k for k in ("a1", "a2", "g1", "g2")})
        else:
            params.update(decay="head", gate="silu")
            names.update({k: p + k for k in ("a", "g")})
        return PartSpec("gated_delta_rule", params, names)

    def _mixer(self, i: int, layer: dict) -> PartSpec:
        m, p = layer["mixer"], f"l{i}.mix."
        if layer["type"] == "delta":
            return self._delta(p, m, False)
        left = m["left"]
        attention = PartSpec(
            "capped_attention",
            {"hidden_size": self.width, "num_heads": left["heads"], "num_kv_heads": left["kv_heads"],
             "key_dim": left["dim"], "value_dim": left["vdim"], "softmax_scale": float(left["scale"]),
             "softcap": float(left.get("softcap", 0) or 0)},
            {k: f"{p}left.{k}" for k in ("q", "k", "v", "o")})
        return PartSpec("side_by_side",
                        {"left": attention, "right": self._delta(p + "right.", m["right"], True),
                         "left_scale": float(m["left_scale"]), "right_scale": float(m["right_scale"])})

    def _feed_forward(self, i: int, mlp: Optional[dict]) -> PartSpec:
        if mlp is None:
            return PartSpec("none")
        p, n = f"l{i}.mlp.", int(mlp["router"]["experts"])
        names = {"router": p + "router"}
        for j in range(n):
            for t in ("gate", "up", "down"):
                names[f"e{j}.{t}"] = f"{p}e{j}.{t}"
        return PartSpec("routed_experts",
                        {"hidden_size": self.width, "expert_size": int(mlp["expert"]["ff"]),
                         "num_experts": n, "top": int(mlp["router"]["top"]), "correction": False,
                         "score": "sigmoid", "activation": "clamped_swish",
                         "limit": float(mlp["expert"]["limit"]), "weight_on": "input"},
                        names)

    def to_spec(self) -> ModelSpec:
        E, V, S = self.width, self.vocab, self.streams

        def norm(name: str, read: Optional[str] = None) -> PartSpec:
            if not S:
                return PartSpec("rms_norm", {"size": E, "eps": self.eps}, {"weight": name})
            names = {"weight": name, **({"read": read} if read else {})}
            return PartSpec("stream_rms_norm", {"size": E, "eps": self.eps, "streams": S}, names)

        layers = []
        for i, layer in enumerate(self.layers):
            has_ff = layer.get("mlp") is not None
            block_tensors = {}
            if S:
                for q in (1, 2) if has_ff else (1,):
                    block_tensors.update({f"mix{q}": f"l{i}.hc{q}.mix", f"out{q}": f"l{i}.hc{q}.out"})
                if i in self.mix_without_ff:
                    block_tensors["mix2"] = f"l{i}.hc2.mix"
            layers.append(LayerSpec(
                block="hyper_connections" if S else "pre_norm",
                mixer=self._mixer(i, layer),
                feed_forward=self._feed_forward(i, layer.get("mlp")),
                mixer_norm=norm(f"l{i}.norm1", f"l{i}.hc1.in"),
                feed_forward_norm=(norm(f"l{i}.norm2", f"l{i}.hc2.in") if has_ff or not S else None),
                position=None,
                block_params={"streams": S} if S else {},
                block_tensors=block_tensors))
        return ModelSpec(
            architecture=self.architecture, vocab_size=V, hidden_size=E,
            max_positions=self.max_positions,
            embedding=PartSpec("token_embedding", {"vocab_size": V, "hidden_size": E, "streams": S},
                               {"weight": "embed"}),
            layers=layers,
            schedule=[ScheduleEntry(layer=i, cache_line=i) for i in range(len(layers))],
            final_norm=norm("final.norm"),
            head=PartSpec("lm_head", {"hidden_size": E, "vocab_size": V}, {"weight": "embed"}),
            bos_token_id=None, eos_token_ids=[], ignored_tensor_suffixes=list(self.unused_tensors))
