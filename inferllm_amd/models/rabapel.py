"""Rabapel: a decoder whose layers add a mixer's and a feed-forward's output, both computed from
one RMS norm of the stream, with latent attention as the mixer and dense or routed feed-forwards.

This file holds what is specific to the design: the keys of its config.json, their checks, the
tensor names of its checkpoints and the translation into a `ModelSpec` of generic parts.

    config.json
      architecture: "Rabapel"; vocab; width; norm.eps; embedding.scale
      layers: [{type: "latent_attention",
                mixer: {heads, dim, rot_dim, vdim, kv_rank, scale, mask: {size}?,
                        rot: {base, dims, scaling: {factor, original, fast, slow}?}},
                mlp: null | {kind: "dense", ff}
                          | {kind: "moe", expert: {ff}, router: {experts, identity?, top},
                             shared: {ff}?}}, ...]
    tensors
      embed; final.norm; l<i>.norm1; l<i>.mix.{q, dkv, dkv.norm, uk, uv, g, o};
      l<i>.mlp.{up, down} | l<i>.mlp.{router, correction, e<j>.{gate, up, down},
      shared.{gate, up, down, sg}}

The embedding rows are multiplied by embedding.scale; the head is the embedding table itself.
Positions have no limit of their own in the configuration; `max_positions` (optional key) sizes
the angle tables and defaults to 65,536.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import List, Optional

from ..config.registry import ConfigError, register_architecture
from ..config.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

DEFAULT_MAX_POSITIONS = 65536


def _get(d: dict, key: str, where: str, kind=None):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError(f"config.json of Rabapel lacks {where}{key}")
    v = d[key]
    if kind == "int":
        if not isinstance(v, int) or isinstance(v, bool) or v <= 0:
            raise ConfigError(f"{where}{key} must be a positive integer, got {v!r}")
    elif kind == "float":
        if isinstance(v, bool) or not isinstance(v, (int, float)) or not float(v) > 0:
            raise ConfigError(f"{where}{key} must be a positive number, got {v!r}")
    return v


@register_architecture("Rabapel")
@dataclass
class RabapelConfig:
    vocab: int
    width: int
    eps: float
    embedding_scale: float
    layers: List[dict] = field(default_factory=list)
    max_positions: int = DEFAULT_MAX_POSITIONS

    architecture = "Rabapel"
    cli_type_names = ("rabapel",)

    # ------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, d: dict) -> "RabapelConfig":
        layers = _get(d, "layers", "")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("layers must be a list with at least one layer")
        emb = d.get("embedding") or {}
        cfg = cls(vocab=_get(d, "vocab", "", "int"), width=_get(d, "width", "", "int"),
                  eps=float(_get(_get(d, "norm", ""), "eps", "norm.", "float")),
                  embedding_scale=float(emb.get("scale", 1.0)),
                  layers=copy.deepcopy(layers),
                  max_positions=int(d.get("max_positions", DEFAULT_MAX_POSITIONS)))
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.max_positions <= 0:
            raise ConfigError("max_positions must be positive")
        for i, layer in enumerate(self.layers):
            at = f"layers[{i}]."
            kind = _get(layer, "type", at)
            if kind != "latent_attention":
                raise ConfigError(f"{at}type {kind!r} is not a mixer of this design (latent_attention)")
            m = _get(layer, "mixer", at)
            for k in ("heads", "vdim", "kv_rank"):
                _get(m, k, at + "mixer.", "int")
            for k in ("dim", "rot_dim"):
                v = _get(m, k, at + "mixer.")
                if not isinstance(v, int) or isinstance(v, bool) or v < 0:
                    raise ConfigError(f"{at}mixer.{k} must be a non-negative integer, got {v!r}")
            if m["dim"] + m["rot_dim"] <= 0:
                raise ConfigError(f"{at}mixer: a head needs query dimensions")
            _get(m, "scale", at + "mixer.", "float")
            if m.get("mask"):
                _get(m["mask"], "size", at + "mixer.mask.", "int")
            rot = m.get("rot")
            if rot:
                dims = _get(rot, "dims", at + "mixer.rot.", "int")
                _get(rot, "base", at + "mixer.rot.", "float")
                if dims % 2 or dims > m["rot_dim"]:
                    raise ConfigError(f"{at}mixer.rot.dims {dims} must be even and at most rot_dim {m['rot_dim']}")
                if rot.get("scaling"):
                    for k in ("factor", "original", "fast", "slow"):
                        _get(rot["scaling"], k, at + "mixer.rot.scaling.", "float")
            mlp = layer.get("mlp")
            if mlp is None:
                continue
            kind = _get(mlp, "kind", at + "mlp.")
            if kind == "dense":
                _get(mlp, "ff", at + "mlp.", "int")
            elif kind == "moe":
                r = _get(mlp, "router", at + "mlp.")
                n = _get(r, "experts", at + "mlp.router.")
                ident = r.get("identity", 0) or 0
                if not all(isinstance(v, int) and not isinstance(v, bool) and v >= 0 for v in (n, ident)):
                    raise ConfigError(f"{at}mlp.router: experts and identity must be non-negative integers")
                top = _get(r, "top", at + "mlp.router.", "int")
                if n + ident <= 0 or top > n + ident:
                    raise ConfigError(f"{at}mlp.router: {top} of {n} + {ident} experts cannot be chosen")
                if n:
                    _get(_get(mlp, "expert", at + "mlp."), "ff", at + "mlp.expert.", "int")
                if mlp.get("shared"):
                    _get(mlp["shared"], "ff", at + "mlp.shared.", "int")
            else:
                raise ConfigError(f"{at}mlp.kind {kind!r} is not a feed-forward of this design (dense, moe)")

    def to_dict(self) -> dict:
        d = {"architecture": self.architecture, "embedding": {"scale": self.embedding_scale},
             "layers": copy.deepcopy(self.layers), "norm": {"eps": self.eps}, "vocab": self.vocab,
             "width": self.width}
        if self.max_positions != DEFAULT_MAX_POSITIONS:
            d["max_positions"] = self.max_positions
        return d

    # ------------------------------------------------------------ translation
    def _feed_forward(self, i: int, mlp: Optional[dict]) -> PartSpec:
        p = f"l{i}.mlp."
        if mlp is None:
            return PartSpec("none")
        if mlp["kind"] == "dense":
            return PartSpec("dense_activation",
                            {"hidden_size": self.width, "intermediate_size": mlp["ff"],
                             "activation": "relu_squared"},
                            {"up": p + "up", "down": p + "down"})
        r = mlp["router"]
        n, shared = int(r["experts"]), mlp.get("shared") or None
        names = {"router": p + "router", "correction": p + "correction"}
        for j in range(n):
            for t in ("gate", "up", "down"):
                names[f"e{j}.{t}"] = f"{p}e{j}.{t}"
        if shared:
            for t in ("gate", "up", "down", "sg"):
                names[f"shared.{t}"] = f"{p}shared.{t}"
        return PartSpec("routed_experts",
                        {"hidden_size": self.width, "expert_size": (mlp.get("expert") or {}).get("ff", 0),
                         "num_experts": n, "num_identity": int(r.get("identity", 0) or 0),
                         "top": int(r["top"]), "correction": True,
                         "shared_size": int(shared["ff"]) if shared else 0, "shared_gate": True},
                        names)

    def to_spec(self) -> ModelSpec:
        E, V = self.width, self.vocab
        norm = lambda name: PartSpec("rms_norm", {"size": E, "eps": self.eps}, {"weight": name})
        layers = []
        for i, layer in enumerate(self.layers):
            m, p = layer["mixer"], f"l{i}.mix."
            rot = m.get("rot") or None
            position = None
            if rot and m["rot_dim"] > 0:
                position = PartSpec("rotary", {"head_dim": m["rot_dim"], "rotary_dim": rot["dims"],
                                               "theta": float(rot["base"]), "pairing": "interleaved",
                                               "max_positions": self.max_positions,
                                               "scaling": dict(rot["scaling"]) if rot.get("scaling") else None})
            layers.append(LayerSpec(
                block="parallel",
                mixer=PartSpec(
                    "latent_attention",
                    {"hidden_size": E, "num_heads": m["heads"], "head_dim": m["dim"],
                     "rot_dim": m["rot_dim"], "value_dim": m["vdim"], "rank": m["kv_rank"],
                     "softmax_scale": float(m["scale"]), "eps": self.eps,
                     "window": (m.get("mask") or {}).get("size"), "gated": True},
                    {"q": p + "q", "dkv": p + "dkv", "dkv_norm": p + "dkv.norm", "uk": p + "uk",
                     "uv": p + "uv", "g": p + "g", "o": p + "o"}),
                feed_forward=self._feed_forward(i, layer.get("mlp")),
                mixer_norm=norm(f"l{i}.norm1"),
                feed_forward_norm=None,
                position=position))
        return ModelSpec(
            architecture=self.architecture, vocab_size=V, hidden_size=E,
            max_positions=self.max_positions,
            embedding=PartSpec("token_embedding", {"vocab_size": V, "hidden_size": E,
                                                   "scale": self.embedding_scale}, {"weight": "embed"}),
            layers=layers,
            schedule=[ScheduleEntry(layer=i, cache_line=i) for i in range(len(layers))],
            final_norm=norm("final.norm"),
            head=PartSpec("lm_head", {"hidden_size": E, "vocab_size": V}, {"weight": "embed"}),
            bos_token_id=None, eos_token_ids=[])
