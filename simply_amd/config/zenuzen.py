"""Typed configuration of Zenuzen, read from the model folder's `config.json`.

A decoder whose layers are listed one by one: each entry of "layers" names its mixer ("attention": softmax
attention with a sink, partial rotary, unit-RMS queries and keys, values mixed with the first such layer's, an
output gate; "delta": the gated delta rule with short convolutions), the mixer's sizes, and its feed-forward (or
none).  A layer norms what its parts return, not what they read: x <- x + m * norm(part(x)).

Keys: "architecture", "vocab", "width", "residual_mult", "norm": {"eps"}, "layers": [{"type", "mixer": {...},
"mlp": {"kind", "ff"} | null}].  Attention mixers: heads, kv_heads, dim, vdim, scale, optional rot {dims, base},
optional v_mix.  Delta mixers: heads, kv_heads, dim, vdim, conv.  Tensors: "embed", "l<i>.norm1", "l<i>.norm2",
"l<i>.mix.*", "l<i>.mlp.*", "final.norm", "head"; matrices are [out, in].
"""
from __future__ import annotations

import dataclasses
from typing import Any, Mapping

from ..registry import ARCHITECTURES
from .gemma2 import ConfigError
from .spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

LAYER_TYPES = ("attention", "delta")
MLP_KINDS = ("dense",)


def _get(d: Mapping[str, Any], key: str, where: str, typ=None):
    if not isinstance(d, Mapping) or key not in d or d[key] is None:
        raise ConfigError(f"config.json: {where}: required key {key!r} is missing")
    v = d[key]
    if typ is int and (isinstance(v, bool) or not isinstance(v, int)):
        raise ConfigError(f"config.json: {where}: {key!r} must be an integer, got {v!r}")
    if typ is float:
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"config.json: {where}: {key!r} must be a number, got {v!r}")
        v = float(v)
    return v


@dataclasses.dataclass(frozen=True)
class ZenuzenLayer:
    type: str
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    # attention
    scale: float | None = None
    rot_dims: int = 0
    rot_base: float = 10000.0
    v_mix: bool = False
    # delta
    conv: int = 0
    # feed-forward: None for none
    mlp_kind: str | None = None
    ff: int = 0

    @classmethod
    def from_dict(cls, d: Mapping[str, Any], i: int) -> "ZenuzenLayer":
        where = f"layers[{i}]"
        kind = _get(d, "type", where)
        if kind not in LAYER_TYPES:
            raise ConfigError(f"config.json: {where}: unknown layer type {kind!r}; known: {', '.join(LAYER_TYPES)}")
        m = _get(d, "mixer", where)
        mw = where + ".mixer"
        kw: dict[str, Any] = dict(type=kind, heads=_get(m, "heads", mw, int), kv_heads=_get(m, "kv_heads", mw, int),
                                  dim=_get(m, "dim", mw, int), vdim=_get(m, "vdim", mw, int))
        if kind == "attention":
            kw["scale"] = _get(m, "scale", mw, float)
            rot = m.get("rot")
            if rot is not None:
                kw["rot_dims"] = _get(rot, "dims", mw + ".rot", int)
                kw["rot_base"] = _get(rot, "base", mw + ".rot", float)
            kw["v_mix"] = bool(m.get("v_mix", False))
        else:
            kw["conv"] = _get(m, "conv", mw, int)
        mlp = d.get("mlp")
        if mlp is not None:
            kw["mlp_kind"] = _get(mlp, "kind", where + ".mlp")
            if kw["mlp_kind"] not in MLP_KINDS:
                raise ConfigError(f"config.json: {where}.mlp: unknown kind {kw['mlp_kind']!r}; known: "
                                  + ", ".join(MLP_KINDS))
            kw["ff"] = _get(mlp, "ff", where + ".mlp", int)
        return cls(**kw)

    def to_dict(self) -> dict[str, Any]:
        m: dict[str, Any] = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim}
        if self.type == "attention":
            m["scale"] = self.scale
            if self.rot_dims:
                m["rot"] = {"dims": self.rot_dims, "base": self.rot_base}
            if self.v_mix:
                m["v_mix"] = True
        else:
            m["conv"] = self.conv
        mlp = None if self.mlp_kind is None else {"kind": self.mlp_kind, "ff": self.ff}
        return {"type": self.type, "mixer": m, "mlp": mlp}

    def validate(self, i: int) -> None:
        where = f"config.json: layers[{i}]"
        for name in ("heads", "kv_heads", "dim", "vdim"):
            if getattr(self, name) <= 0:
                raise ConfigError(f"{where}: {name} must be positive, got {getattr(self, name)}")
        if self.heads % self.kv_heads:
            raise ConfigError(f"{where}: heads {self.heads} is not a multiple of kv_heads {self.kv_heads}")
        if self.type == "attention":
            if self.rot_dims % 2 or not 0 <= self.rot_dims <= self.dim:
                raise ConfigError(f"{where}: rot.dims {self.rot_dims} must be even and at most dim {self.dim}")
            if self.rot_dims and self.rot_base <= 0:
                raise ConfigError(f"{where}: rot.base must be positive")
        elif self.conv < 1:
            raise ConfigError(f"{where}: conv must be at least 1, got {self.conv}")
        if self.mlp_kind is not None and self.ff <= 0:
            raise ConfigError(f"{where}: mlp.ff must be positive, got {self.ff}")


@dataclasses.dataclass(frozen=True)
class ZenuzenConfig:
    vocab: int
    width: int
    residual_mult: float
    norm_eps: float
    layers: tuple[ZenuzenLayer, ...]
    #: not part of the design: the longest sequence that the engine plans for when --max_seq_len does not say
    max_position: int = 8192
    eos_token_ids: tuple[int, ...] = ()
    initializer_range: float = 0.02

    architecture = "Zenuzen"

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "ZenuzenConfig":
        layers = _get(d, "layers", "top level")
        if not isinstance(layers, (list, tuple)) or not layers:
            raise ConfigError('config.json: "layers" must be a non-empty list')
        eos = d.get("eos_token_id")
        eos_ids = () if eos is None else tuple(int(e) for e in (eos if isinstance(eos, (list, tuple)) else [eos]))
        cfg = cls(vocab=_get(d, "vocab", "top level", int), width=_get(d, "width", "top level", int),
                  residual_mult=_get(d, "residual_mult", "top level", float),
                  norm_eps=_get(_get(d, "norm", "top level"), "eps", "norm", float),
                  layers=tuple(ZenuzenLayer.from_dict(l, i) for i, l in enumerate(layers)),
                  max_position=int(d.get("max_position", 8192)), eos_token_ids=eos_ids,
                  initializer_range=float(d.get("initializer_range", 0.02)))
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError("config.json: vocab and width must be positive")
        if self.norm_eps < 0:
            raise ConfigError("config.json: norm.eps must not be negative")
        for i, l in enumerate(self.layers):
            l.validate(i)
        mixing = [l for l in self.layers if l.type == "attention" and l.v_mix]
        if any((l.kv_heads, l.vdim) != (mixing[0].kv_heads, mixing[0].vdim) for l in mixing):
            raise ConfigError("config.json: layers that mix values must agree in kv_heads and vdim")

    def to_dict(self) -> dict[str, Any]:
        d: dict[str, Any] = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                             "residual_mult": self.residual_mult, "norm": {"eps": self.norm_eps},
                             "layers": [l.to_dict() for l in self.layers]}
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids)
        if self.max_position != 8192:
            d["max_position"] = self.max_position
        if self.initializer_range != 0.02:
            d["initializer_range"] = self.initializer_range
        return d

    # ------------------------------------------------------------------ model spec
    def model_spec(self) -> ModelSpec:
        D = self.width

        def norm(name: str, mult: float = 1.0) -> PartSpec:
            return PartSpec("rmsnorm", {"dim": D, "eps": self.norm_eps, "scale_plus_one": False, "mult": mult},
                            {"scale": name})

        layers = []
        seen_mixing = False
        for i, l in enumerate(self.layers):
            p = f"l{i}."
            if l.type == "attention":
                value_mix = None
                if l.v_mix:
                    value_mix, seen_mixing = ("mix" if seen_mixing else "source"), True
                tensors = {"q_proj": p + "mix.q", "k_proj": p + "mix.k", "v_proj": p + "mix.v", "gate_proj": p + "mix.g",
                           "o_proj": p + "mix.o", "sink": p + "mix.sink"}
                if value_mix is not None:
                    tensors["vmix"] = p + "mix.vmix"
                mixer = PartSpec("sink_attention", {
                    "hidden_size": D, "num_heads": l.heads, "num_kv_heads": l.kv_heads, "key_dim": l.dim,
                    "value_dim": l.vdim, "scale": l.scale, "sinks": True, "qk_norm_eps": self.norm_eps,
                    "output_gate": True, "value_mix": value_mix, "value_mix_key": "v_first",
                    "position_encoding": PartSpec("partial_rope", {"head_dim": l.dim, "dims": l.rot_dims,
                                                                   "base": l.rot_base}) if l.rot_dims else None,
                }, tensors)
            else:
                mixer = PartSpec("gated_delta", {
                    "hidden_size": D, "num_heads": l.heads, "num_qk_heads": l.kv_heads, "key_dim": l.dim,
                    "value_dim": l.vdim, "conv_taps": l.conv, "norm_eps": self.norm_eps,
                }, {"q_proj": p + "mix.q", "k_proj": p + "mix.k", "v_proj": p + "mix.v", "q_conv": p + "mix.q.conv",
                    "k_conv": p + "mix.k.conv", "v_conv": p + "mix.v.conv", "a_proj": p + "mix.a", "b_proj": p + "mix.b",
                    "a_log": p + "mix.A_log", "dt_bias": p + "mix.dt_bias", "norm": p + "mix.norm",
                    "gate_proj": p + "mix.g", "o_proj": p + "mix.o"})
            norms = {"input": PartSpec("none"), "post_mixer": norm(p + "norm1", self.residual_mult)}
            ffn = None
            if l.mlp_kind == "dense":
                ffn = PartSpec("dense", {"hidden_size": D, "intermediate_size": l.ff, "activation": "squared_relu"},
                               {"up_proj": p + "mlp.up", "down_proj": p + "mlp.down"})
                norms["post_ffn"] = norm(p + "norm2", self.residual_mult)
            layers.append(LayerSpec(block=PartSpec("post_norm"), mixer=mixer, feed_forward=ffn, norms=norms))
        spec = ModelSpec(
            architecture=self.architecture, hidden_size=D, vocab_size=self.vocab,
            embedding=PartSpec("scaled_embedding", {"vocab_size": self.vocab, "dim": D, "scale": 1.0}, {"table": "embed"}),
            layers=tuple(layers), schedule=tuple(ScheduleEntry(i) for i in range(len(layers))),
            final_norm=norm("final.norm"),
            head=PartSpec("linear_head", {"vocab_size": self.vocab, "dim": D, "soft_cap": None}, {"weight": "head"}),
            max_position=self.max_position, eos_token_ids=self.eos_token_ids, initializer_range=self.initializer_range)
        spec.validate()
        return spec


ARCHITECTURES.register("Zenuzen", ZenuzenConfig)
