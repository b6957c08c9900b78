"""Typed configuration of the Pelalix design: a pre-norm decoder whose config.json lists its layers one by one.

    {"architecture": "Pelalix", "vocab": V, "width": W, "embedding": {"scale": s}, "norm": {"eps": e},
     "layers": [{"type": "attention",
                 "mixer": {"heads", "kv_heads", "dim", "vdim", "scale", "v_mix"},
                 "mlp": {"kind": "dense", "ff": F} | null}, ...]}

Every size and constant is read from there, layer by layer; nothing else is assumed equal between layers except
what has to be (layers that mix their values share the value size of the first of them).  What the design fixes:
Dynamic Tanh norms with a bias, a gain per channel on both branches, a token shift before every mixer, attention
without positions whose heads' scores are mixed before a softmax with a sink, a sigmoid gate per head, RMS norm over
the whole query and key projections, a gated SiLU feed-forward, an untied head.  Tensor names: `embed`, `head`,
`final.norm[.b|.alpha]`, and per layer `l<i>.` + `norm1`, `norm2` (`.b`, `.alpha`), `ls1`, `ls2`, `shift`,
`mix.{q,k,v,o,g,q.norm,k.norm,talk,sink,vmix}`, `mlp.{gate,up,down}`.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .registry import ConfigError, register_architecture
from .spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry, linear_head, token_embedding

ARCHITECTURE = "Pelalix"
MIXER_TYPES = ("attention",)
MLP_KINDS = ("dense",)


def _number(raw, key, where, typ, default=None, required=True):
    if not isinstance(raw, dict):
        raise ConfigError(f"config.json: {where} must be an object")
    if key not in raw or raw[key] is None:
        if required:
            raise ConfigError(f"config.json: {where} lacks {key!r}")
        return default
    v = raw[key]
    if isinstance(v, bool) != (typ is bool):
        raise ConfigError(f"config.json: {where}.{key} must be {typ.__name__}, got {v!r}")
    if typ is float and isinstance(v, int):
        v = float(v)
    if not isinstance(v, typ):
        raise ConfigError(f"config.json: {where}.{key} must be {typ.__name__}, got {v!r}")
    return v


@dataclass
class PelalixMixer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    v_mix: bool = False


@dataclass
class PelalixLayer:
    type: str
    mixer: PelalixMixer
    mlp_kind: Optional[str] = None  # None: the layer has no feed-forward
    ff: int = 0


@dataclass
class PelalixConfig:
    vocab: int
    width: int
    layers: List[PelalixLayer]
    embedding_scale: float = 1.0
    norm_eps: float = 1e-6
    eos_token_ids: List[int] = field(default_factory=list)
    initializer_range: float = 0.02

    architecture = ARCHITECTURE

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "PelalixConfig":
        layers_raw = raw.get("layers")
        if not isinstance(layers_raw, list) or not layers_raw:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        layers = []
        for i, lr in enumerate(layers_raw):
            where = f"layers[{i}]"
            kind = _number(lr, "type", where, str)
            m = lr.get("mixer")
            mw = where + ".mixer"
            heads = _number(m, "heads", mw, int)
            mixer = PelalixMixer(heads=heads, kv_heads=_number(m, "kv_heads", mw, int, heads, required=False),
                                 dim=_number(m, "dim", mw, int), vdim=_number(m, "vdim", mw, int, None, required=False)
                                 or _number(m, "dim", mw, int), scale=_number(m, "scale", mw, float),
                                 v_mix=_number(m, "v_mix", mw, bool, False, required=False))
            mlp = lr.get("mlp")
            if mlp is None:
                layers.append(PelalixLayer(kind, mixer))
            else:
                layers.append(PelalixLayer(kind, mixer, _number(mlp, "kind", where + ".mlp", str),
                                           _number(mlp, "ff", where + ".mlp", int)))
        eos = raw.get("eos_token_id")
        eos = [] if eos is None else (eos if isinstance(eos, list) else [eos])
        if any(isinstance(x, bool) or not isinstance(x, int) for x in eos):
            raise ConfigError("config.json: eos_token_id must be an integer or a list of integers")
        return cls(vocab=_number(raw, "vocab", "the configuration", int), width=_number(raw, "width", "the configuration", int),
                   layers=layers,
                   embedding_scale=_number(raw.get("embedding", {}), "scale", "embedding", float, 1.0, required=False),
                   norm_eps=_number(raw.get("norm", {}), "eps", "norm", float, 1e-6, required=False),
                   eos_token_ids=list(eos),
                   initializer_range=_number(raw, "initializer_range", "the configuration", float, 0.02, required=False))

    def to_dict(self) -> Dict[str, Any]:
        layers = []
        for l in self.layers:
            m = l.mixer
            layers.append({"type": l.type,
                           "mixer": {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim,
                                     "scale": m.scale, "v_mix": m.v_mix},
                           "mlp": None if l.mlp_kind is None else {"kind": l.mlp_kind, "ff": l.ff}})
        d = {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "layers": layers,
             "embedding": {"scale": self.embedding_scale}, "norm": {"eps": self.norm_eps},
             "initializer_range": self.initializer_range}
        if self.eos_token_ids:
            d["eos_token_id"] = self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else self.eos_token_ids
        return d

    def validate(self) -> None:
        def need(ok, msg):
            if not ok:
                raise ConfigError("config.json: " + msg)

        need(self.vocab > 0 and self.width > 0, "vocab and width must be positive")
        need(self.norm_eps > 0, "norm.eps must be positive")
        need(self.initializer_range > 0, "initializer_range must be positive")
        need(all(0 <= t < self.vocab for t in self.eos_token_ids), "eos_token_id names a token outside the vocabulary")
        source = None
        for i, l in enumerate(self.layers):
            m = l.mixer
            need(l.type in MIXER_TYPES, f"layers[{i}].type {l.type!r} is not a mixer of this design (known: "
                 + ", ".join(MIXER_TYPES) + ")")
            need(min(m.heads, m.kv_heads, m.dim, m.vdim) > 0, f"layers[{i}].mixer: sizes must be positive")
            need(m.heads % m.kv_heads == 0, f"layers[{i}].mixer: heads {m.heads} is not a multiple of kv_heads {m.kv_heads}")
            if l.mlp_kind is not None:
                need(l.mlp_kind in MLP_KINDS, f"layers[{i}].mlp.kind {l.mlp_kind!r} is not known (known: "
                     + ", ".join(MLP_KINDS) + ")")
                need(l.ff > 0, f"layers[{i}].mlp.ff must be positive")
            if m.v_mix:
                if source is None:
                    source = i
                else:
                    s = self.layers[source].mixer
                    need((s.kv_heads, s.vdim) == (m.kv_heads, m.vdim),
                         f"layers[{i}] mixes its values with those of layers[{source}], whose key/value heads or "
                         "value size differ")

    def model_spec(self) -> ModelSpec:
        W, std = self.width, self.initializer_range
        norm = lambda name: PartSpec("dynamic_tanh", {"width": W, "bias": True},
                                     rename={"weight": name, "bias": name + ".b", "alpha": name + ".alpha"})
        layers, ignored = [], []
        source_seen = False
        for i, l in enumerate(self.layers):
            p = f"l{i}."
            m = l.mixer
            value_mix = "none"
            if m.v_mix:
                value_mix = "mix" if source_seen else "source"
                source_seen = True
            mixer = PartSpec(
                "talking_attention",
                {"hidden_size": W, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim,
                 "value_dim": m.vdim, "scale": m.scale, "window": 0, "qk_norm": True, "qk_norm_eps": self.norm_eps,
                 "head_mixing": True, "sink": True, "gate": True, "value_mix": value_mix, "init_std": std},
                prefix=p + "mix.",
                rename={"q.weight": "q", "k.weight": "k", "v.weight": "v", "o.weight": "o", "g.weight": "g",
                        "q_norm.weight": "q.norm", "k_norm.weight": "k.norm", "value_mix": "vmix"})
            if not m.v_mix:
                ignored.append(p + "mix.vmix")
            parts = {"mixer": mixer, "mixer_norm": norm(p + "norm1"),
                     "mixer_gain": PartSpec("channel_gain", {"width": W}, rename={"weight": p + "ls1"}),
                     "mixer_shift": PartSpec("previous_token", {"width": W}, rename={"weight": p + "shift"})}
            if l.mlp_kind is not None:
                parts["feed_forward"] = PartSpec(
                    "dense_mlp", {"hidden_size": W, "width": l.ff, "init_std": std}, prefix=p + "mlp.",
                    rename={"gate_proj.weight": "gate", "up_proj.weight": "up", "down_proj.weight": "down"})
                parts["feed_forward_norm"] = norm(p + "norm2")
                parts["feed_forward_gain"] = PartSpec("channel_gain", {"width": W}, rename={"weight": p + "ls2"})
            else:  # a checkpoint may still hold what the absent feed-forward would have had around it
                ignored += [p + "norm2", p + "norm2.b", p + "norm2.alpha", p + "ls2"]
            layers.append(LayerSpec("prenorm_gained", parts))
        spec = ModelSpec(
            architecture=ARCHITECTURE, hidden_size=W, vocab_size=self.vocab, max_positions=0, layers=layers,
            schedule=[ScheduleEntry(i) for i in range(len(layers))],
            embedding=token_embedding("embed", self.vocab, W, std, scale=self.embedding_scale),
            final_norm=norm("final.norm"), head=linear_head("head", self.vocab, W, std), init_std=std,
            ignored_tensor_suffixes=tuple(ignored))
        spec.validate()
        return spec


register_architecture(ARCHITECTURE, PelalixConfig)
