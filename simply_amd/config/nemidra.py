"""Typed configuration of Nemidra, read from the model folder's `config.json`.

A decoder whose layers are listed one by one; a run of consecutive layers may be looped over several times with the
same weights (every pass with a cache and state of its own, and the embedding's output added to the stream before
every pass but the first).  The embedding sums the token's row, a hashed row for the pair (previous token, token) and
a learned position row.  A layer is a sandwich block, x += norm(mixer(norm(x))), x += norm(ff(norm(x))), with norms
whose weight is stored around zero, followed by a per-layer input from the token itself.  Mixers: "gla" (gated linear
attention with a decay per key channel) and "parallel" (sliding-window softmax attention with biases and without
positions beside a matrix memory with exponential gates, their results in a weighted sum).  Feed-forwards: "dense"
(exact GELU, no gate), "moe" (routed gated experts with silu, optionally a shared one), or none.

Keys: "architecture", "vocab", "width", "norm": {"eps"}, "embedding": {"bigram": {"buckets", "mul_prev", "mul_cur"}},
"max_positions", "layers": [{"type", "mixer": {...}, "mlp": {...} | null}], "loop": {"start", "stop", "times"},
"token_side": {"dim"}, "logit_softcap".  gla mixers: heads, dim, vdim, tau (the decay's rank is the first dimension of
the tensor "l<i>.mix.a1"; a config that is to be written with random weights may say it as "rank").  parallel mixers:
left {heads, kv_heads, dim, vdim, scale, mask: {size}}, right {heads, dim, vdim, gate_cap}, left_scale, right_scale.
mlp: {"kind": "dense", "ff"} or {"kind": "moe", "expert": {"ff"}, "router": {"experts", "top", "scale"}, "shared": {"ff"}}.
Tensors: "embed", "bigram", "pos", "side.embed", "l<i>.norm1|norm1b|norm2|norm2b", "l<i>.mix.*", "l<i>.mlp.*",
"l<i>.side.gate|proj|norm", "final.norm", "head"; matrices are [out, in].
"""
from __future__ import annotations

import copy
import dataclasses
from typing import Any, Mapping

from ..registry import ARCHITECTURES
from .gemma2 import ConfigError
from .spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
from .zenuzen import _get

LAYER_TYPES = ("gla", "parallel")
MLP_KINDS = ("dense", "moe")


def _positive(v, what: str):
    if v <= 0:
        raise ConfigError(f"config.json: {what} must be positive, got {v}")
    return v


@dataclasses.dataclass(frozen=True)
class NemidraConfig:
    #: the dictionary of config.json, as read (`to_dict` gives it back)
    raw: Mapping[str, Any]
    vocab: int
    width: int
    norm_eps: float
    num_layers: int
    #: the longest sequence that the engine plans for when --max_seq_len does not say: the learned positions, if any
    max_position: int = 8192
    eos_token_ids: tuple[int, ...] = ()
    initializer_range: float = 0.02

    architecture = "Nemidra"

    @classmethod
    def from_dict(cls, d: Mapping[str, Any], check: bool = True) -> "NemidraConfig":
        layers = _get(d, "layers", "top level")
        if not isinstance(layers, (list, tuple)) or not layers:
            raise ConfigError('config.json: "layers" must be a non-empty list')
        eos = d.get("eos_token_id")
        eos_ids = () if eos is None else tuple(int(e) for e in (eos if isinstance(eos, (list, tuple)) else [eos]))
        cfg = cls(raw=copy.deepcopy(dict(d)), vocab=_positive(_get(d, "vocab", "top level", int), "vocab"),
                  width=_positive(_get(d, "width", "top level", int), "width"),
                  norm_eps=_get(_get(d, "norm", "top level"), "eps", "norm", float), num_layers=len(layers),
                  max_position=int(d.get("max_positions") or d.get("max_position") or 8192), eos_token_ids=eos_ids,
                  initializer_range=float(d.get("initializer_range", 0.02)))
        if check:
            cfg.model_spec()   # (reads every key: whatever is missing or wrong is said now)
        return cfg

    @classmethod
    def from_dict_open(cls, d: Mapping[str, Any]) -> "NemidraConfig":
        """The configuration of a model folder before `resolve_shapes` has read the sizes that the tensors give."""
        return cls.from_dict(d, check=False)

    def to_dict(self) -> dict[str, Any]:
        return copy.deepcopy(dict(self.raw))

    def resolve_shapes(self, shapes: Mapping[str, tuple]) -> "NemidraConfig":
        """Sizes that config.json leaves to the tensors: the rank of every gla mixer's decay projection."""
        raw = copy.deepcopy(dict(self.raw))
        for i, l in enumerate(raw["layers"]):
            name = f"l{i}.mix.a1"
            if l.get("type") == "gla" and "rank" not in l["mixer"] and name in shapes:
                l["mixer"]["rank"] = int(shapes[name][0])
        return type(self).from_dict(raw)

    # ------------------------------------------------------------------ schedule
    def schedule(self) -> tuple[ScheduleEntry, ...]:
        n, loop = self.num_layers, self.raw.get("loop")
        if not loop:
            return tuple(ScheduleEntry(i) for i in range(n))
        start, stop, times = (_get(loop, k, "loop", int) for k in ("start", "stop", "times"))
        if not (0 <= start < stop <= n) or times < 1:
            raise ConfigError(f"config.json: loop: layers {start}..{stop - 1} of {n}, {times} times")
        entries = [ScheduleEntry(i) for i in range(start)]
        for rep in range(times):
            entries += [ScheduleEntry(i, add_embedding=(rep > 0 and i == start)) for i in range(start, stop)]
        return tuple(entries + [ScheduleEntry(i) for i in range(stop, n)])

    # ------------------------------------------------------------------ parts
    def _mixer(self, i: int, l: Mapping[str, Any]) -> PartSpec:
        D, eps, p, where = self.width, self.norm_eps, f"l{i}.mix.", f"layers[{i}].mixer"
        m = _get(l, "mixer", f"layers[{i}]")
        if l["type"] == "gla":
            rank = m.get("rank")
            if rank is None:
                raise ConfigError(f"config.json: {where}: the decay's rank is given neither by \"rank\" nor by the tensor "
                                  f"{p}a1 of a model folder")
            return PartSpec("gated_linear_attention", {
                "hidden_size": D, "num_heads": _positive(_get(m, "heads", where, int), "heads"),
                "key_dim": _positive(_get(m, "dim", where, int), "dim"),
                "value_dim": _positive(_get(m, "vdim", where, int), "vdim"), "decay_rank": _positive(int(rank), "rank"),
                "tau": _get(m, "tau", where, float), "norm_eps": eps,
            }, {"q_proj": p + "q", "k_proj": p + "k", "v_proj": p + "v", "gate_proj": p + "g", "o_proj": p + "o",
                "decay_in": p + "a1", "decay_out": p + "a2", "decay_bias": p + "a2.b", "norm": p + "norm"})
        left, right = _get(m, "left", where), _get(m, "right", where)
        lw, rw = where + ".left", where + ".right"
        mask = left.get("mask")
        lp, rp = p + "left.", p + "right."
        attention = PartSpec("sink_attention", {
            "hidden_size": D, "num_heads": _get(left, "heads", lw, int), "num_kv_heads": _get(left, "kv_heads", lw, int),
            "key_dim": _get(left, "dim", lw, int), "value_dim": _get(left, "vdim", lw, int),
            "scale": _get(left, "scale", lw, float), "bias": True,
            "window": None if mask is None else _positive(_get(mask, "size", lw + ".mask", int), "mask.size"),
        })
        memory = PartSpec("matrix_memory", {
            "hidden_size": D, "num_heads": _positive(_get(right, "heads", rw, int), "heads"),
            "key_dim": _positive(_get(right, "dim", rw, int), "dim"),
            "value_dim": _positive(_get(right, "vdim", rw, int), "vdim"),
            "gate_cap": _get(right, "gate_cap", rw, float), "norm_eps": eps})
        tensors = {"left.q_proj": lp + "q", "left.k_proj": lp + "k", "left.v_proj": lp + "v", "left.o_proj": lp + "o",
                   "left.q_bias": lp + "q.b", "left.k_bias": lp + "k.b", "left.v_bias": lp + "v.b",
                   "left.o_bias": lp + "o.b",
                   "right.q_proj": rp + "q", "right.k_proj": rp + "k", "right.v_proj": rp + "v",
                   "right.gate_proj": rp + "g", "right.o_proj": rp + "o", "right.norm": rp + "norm",
                   "right.input_gate": rp + "i", "right.forget_gate": rp + "f", "right.input_bias": rp + "i.b",
                   "right.forget_bias": rp + "f.b"}
        return PartSpec("parallel", {"left": attention, "right": memory,
                                     "left_scale": _get(m, "left_scale", where, float),
                                     "right_scale": _get(m, "right_scale", where, float)}, tensors)

    def _mlp(self, i: int, mlp: Mapping[str, Any]) -> PartSpec:
        D, p, where = self.width, f"l{i}.mlp.", f"layers[{i}].mlp"
        kind = _get(mlp, "kind", where)
        if kind not in MLP_KINDS:
            raise ConfigError(f"config.json: {where}: unknown kind {kind!r}; known: {', '.join(MLP_KINDS)}")
        if kind == "dense":
            return PartSpec("dense", {"hidden_size": D, "intermediate_size": _positive(_get(mlp, "ff", where, int), "ff"),
                                      "activation": "gelu_erf"}, {"up_proj": p + "up", "down_proj": p + "down"})
        router, shared = _get(mlp, "router", where), mlp.get("shared")
        E = _positive(_get(router, "experts", where + ".router", int), "experts")
        tensors = {"router": p + "router"}
        for e in range(E):
            tensors.update({f"e{e}.{n}": f"{p}e{e}.{n}" for n in ("gate", "up", "down")})
        if shared is not None:
            tensors.update({"shared.gate_proj": p + "shared.gate", "shared.up_proj": p + "shared.up",
                            "shared.down_proj": p + "shared.down", "shared.score": p + "shared.sg"})
        return PartSpec("routed_experts", {
            "hidden_size": D, "num_experts": E, "top": _get(router, "top", where + ".router", int),
            "expert_size": _positive(_get(_get(mlp, "expert", where), "ff", where + ".expert", int), "expert.ff"),
            "router_scale": _get(router, "scale", where + ".router", float), "activation": "silu",
            "shared_size": None if shared is None else _positive(_get(shared, "ff", where + ".shared", int), "shared.ff"),
        }, tensors)

    def model_spec(self) -> ModelSpec:
        d, D = self.raw, self.width

        def norm(name: str) -> PartSpec:
            return PartSpec("rmsnorm", {"dim": D, "eps": self.norm_eps, "scale_plus_one": True}, {"scale": name})

        side = d.get("token_side")
        side_dim = None if side is None else _positive(_get(side, "dim", "token_side", int), "token_side.dim")
        layers, ignorable = [], []
        for i, l in enumerate(d["layers"]):
            p, where = f"l{i}.", f"layers[{i}]"
            kind = _get(l, "type", where)
            if kind not in LAYER_TYPES:
                raise ConfigError(f"config.json: {where}: unknown layer type {kind!r}; known: {', '.join(LAYER_TYPES)}")
            norms = {"pre_mixer": norm(p + "norm1"), "post_mixer": norm(p + "norm1b")}
            ffn = None
            if l.get("mlp") is not None:
                ffn = self._mlp(i, l["mlp"])
                norms.update(pre_ffn=norm(p + "norm2"), post_ffn=norm(p + "norm2b"))
            else:
                ignorable += [p + "norm2", p + "norm2b"]
            extras = ()
            if side_dim is not None:
                extras = (PartSpec("token_side", {
                    "hidden_size": D, "dim": side_dim, "vocab_size": self.vocab, "table_width": side_dim * self.num_layers,
                    "column": i * side_dim, "eps": self.norm_eps, "activation": "gelu_tanh",
                }, {"table": "side.embed", "gate": p + "side.gate", "proj": p + "side.proj", "norm": p + "side.norm"}),)
            layers.append(LayerSpec(block=PartSpec("sandwich"), mixer=self._mixer(i, l), feed_forward=ffn, norms=norms,
                                    extras=extras))
        bigram = (d.get("embedding") or {}).get("bigram")
        emb_params: dict[str, Any] = {"vocab_size": self.vocab, "dim": D}
        emb_tensors = {"table": "embed"}
        if bigram is not None:
            emb_params.update(pair_buckets=_positive(_get(bigram, "buckets", "embedding.bigram", int), "buckets"),
                              mul_prev=_get(bigram, "mul_prev", "embedding.bigram", int),
                              mul_cur=_get(bigram, "mul_cur", "embedding.bigram", int))
            emb_tensors["pair"] = "bigram"
        if d.get("max_positions") is not None:
            emb_params["max_positions"] = _positive(_get(d, "max_positions", "top level", int), "max_positions")
            emb_tensors["pos"] = "pos"
        cap = d.get("logit_softcap")
        spec = ModelSpec(
            architecture=self.architecture, hidden_size=D, vocab_size=self.vocab,
            embedding=PartSpec("summed_embedding", emb_params, emb_tensors),
            layers=tuple(layers), schedule=self.schedule(), final_norm=norm("final.norm"),
            head=PartSpec("linear_head", {"vocab_size": self.vocab, "dim": D, "soft_cap": float(cap) if cap else None},
                          {"weight": "head"}),
            max_position=self.max_position, eos_token_ids=self.eos_token_ids, initializer_range=self.initializer_range,
            ignorable=tuple(ignorable))
        spec.validate()
        return spec


ARCHITECTURES.register("Nemidra", NemidraConfig)
