"""Typed configuration of the Dezudra design: a decoder whose config.json lists its layers one by one, each with a
recurrent mixer (the gated delta rule) or differential attention, and a mixture of small experts.

    {"architecture": "Dezudra", "vocab": V, "width": W, "norm": {"eps": e}, "logit_scale": s,
     "layers": [{"type": "delta", "mixer": {"heads", "kv_heads", "dim", "vdim", "conv"},
                 "mlp": {"kind": "moe", "expert": {"ff": F},
                         "router": {"experts": E, "top": k, "groups": {"count": n, "keep": m}}} | null},
                {"type": "attention", "mixer": {"heads", "kv_heads", "dim", "vdim", "conv", "scale", "diff",
                                                "rot": {"dims", "base"}, "mask": {"size", "keep_first"}}, "mlp": ...}]}

Every size and constant is read from there, layer by layer.  What the design fixes: RMS norms with a weight before
and after each branch; short convolutions on q, k, v; in the recurrent mixer silu after them, unit q and k, a decay
and a step size per head, a gated RMS norm per head; in attention two score maps per head, a rotation of the first
`rot.dims` elements of each map (pairs i, i + dims / 2), a window with kept first tokens, softmax, the difference
normalised per head; experts of squared relu chosen among the best groups, weighted by their softmax scores as they
are; an untied head whose logits are scaled.  Tensor names: `embed`, `head`, `final.norm`, and per layer `l<i>.` +
`norm1`, `norm1b`, `norm2`, `norm2b`, `mix.{q,k,v}[.conv|.b]`, `mix.o`, `mix.{b,a,A_log,dt_bias,norm,g}` (delta),
`mix.{lq1,lk1,lq2,lk2}` (attention), `mlp.router`, `mlp.e<j>.{up,down}`.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .pelalix import _number
from .registry import ConfigError, register_architecture
from .spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry, linear_head, token_embedding

ARCHITECTURE = "Dezudra"
MIXER_TYPES = ("delta", "attention")
MLP_KINDS = ("moe",)


@dataclass
class DezudraMixer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    # attention only
    scale: Optional[float] = None
    diff: float = 0.0
    rot_dims: int = 0
    rot_base: float = 10000.0
    mask_size: int = 0        # 0: every earlier token is seen
    keep_first: int = 0


@dataclass
class DezudraMlp:
    kind: str
    ff: int
    experts: int
    top: int
    groups: int = 1
    groups_keep: int = 1


@dataclass
class DezudraLayer:
    type: str
    mixer: DezudraMixer
    mlp: Optional[DezudraMlp] = None  # None: the layer has no feed-forward


@dataclass
class DezudraConfig:
    vocab: int
    width: int
    layers: List[DezudraLayer]
    norm_eps: float = 1e-6
    logit_scale: float = 1.0
    eos_token_ids: List[int] = field(default_factory=list)
    initializer_range: float = 0.02

    architecture = ARCHITECTURE

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "DezudraConfig":
        layers_raw = raw.get("layers")
        if not isinstance(layers_raw, list) or not layers_raw:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        layers = []
        for i, lr in enumerate(layers_raw):
            where = f"layers[{i}]"
            kind = _number(lr, "type", where, str)
            m, mw = lr.get("mixer"), where + ".mixer"
            heads, dim = _number(m, "heads", mw, int), _number(m, "dim", mw, int)
            mixer = DezudraMixer(heads=heads, kv_heads=_number(m, "kv_heads", mw, int, heads, required=False),
                                 dim=dim, vdim=_number(m, "vdim", mw, int, dim, required=False),
                                 conv=_number(m, "conv", mw, int))
            if kind == "attention":
                mixer.scale = _number(m, "scale", mw, float)
                mixer.diff = _number(m, "diff", mw, float)
                rot, mask = m.get("rot"), m.get("mask")
                if rot is not None:
                    mixer.rot_dims = _number(rot, "dims", mw + ".rot", int)
                    mixer.rot_base = _number(rot, "base", mw + ".rot", float)
                if mask is not None:
                    mixer.mask_size = _number(mask, "size", mw + ".mask", int)
                    mixer.keep_first = _number(mask, "keep_first", mw + ".mask", int, 0, required=False)
            mlp_raw, mlp = lr.get("mlp"), None
            if mlp_raw is not None:
                lw = where + ".mlp"
                router = mlp_raw.get("router") if isinstance(mlp_raw, dict) else None
                expert = mlp_raw.get("expert") if isinstance(mlp_raw, dict) else None
                mlp = DezudraMlp(kind=_number(mlp_raw, "kind", lw, str), ff=_number(expert, "ff", lw + ".expert", int),
                                 experts=_number(router, "experts", lw + ".router", int),
                                 top=_number(router, "top", lw + ".router", int))
                groups = router.get("groups")
                if groups is not None:
                    mlp.groups = _number(groups, "count", lw + ".router.groups", int)
                    mlp.groups_keep = _number(groups, "keep", lw + ".router.groups", int)
            layers.append(DezudraLayer(kind, mixer, mlp))
        eos = raw.get("eos_token_id")
        eos = [] if eos is None else (eos if isinstance(eos, list) else [eos])
        if any(isinstance(x, bool) or not isinstance(x, int) for x in eos):
            raise ConfigError("config.json: eos_token_id must be an integer or a list of integers")
        top = "the configuration"
        return cls(vocab=_number(raw, "vocab", top, int), width=_number(raw, "width", top, int), layers=layers,
                   norm_eps=_number(raw.get("norm", {}), "eps", "norm", float, 1e-6, required=False),
                   logit_scale=_number(raw, "logit_scale", top, float, 1.0, required=False), eos_token_ids=list(eos),
                   initializer_range=_number(raw, "initializer_range", top, float, 0.02, required=False))

    def to_dict(self) -> Dict[str, Any]:
        layers = []
        for l in self.layers:
            m = l.mixer
            mixer: Dict[str, Any] = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "conv": m.conv}
            if l.type == "attention":
                mixer.update({"scale": m.scale, "diff": m.diff})
                if m.rot_dims:
                    mixer["rot"] = {"dims": m.rot_dims, "base": m.rot_base}
                if m.mask_size:
                    mixer["mask"] = {"size": m.mask_size, "keep_first": m.keep_first}
            mlp = None
            if l.mlp is not None:
                f = l.mlp
                mlp = {"kind": f.kind, "expert": {"ff": f.ff},
                       "router": {"experts": f.experts, "top": f.top, "groups": {"count": f.groups, "keep": f.groups_keep}}}
            layers.append({"type": l.type, "mixer": mixer, "mlp": mlp})
        d = {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "layers": layers,
             "norm": {"eps": self.norm_eps}, "logit_scale": self.logit_scale,
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
        for i, l in enumerate(self.layers):
            m, w = l.mixer, f"layers[{i}].mixer"
            need(l.type in MIXER_TYPES, f"layers[{i}].type {l.type!r} is not a mixer of this design (known: "
                 + ", ".join(MIXER_TYPES) + ")")
            need(min(m.heads, m.kv_heads, m.dim, m.vdim) > 0, f"{w}: sizes must be positive")
            need(m.heads % m.kv_heads == 0, f"{w}: heads {m.heads} is not a multiple of kv_heads {m.kv_heads}")
            need(1 <= m.conv <= 64, f"{w}.conv must be between 1 and 64 taps")
            need(m.dim <= 256 and m.vdim <= 4096, f"{w}: dim at most 256")
            if l.type == "attention":
                need(m.vdim <= 256, f"{w}: vdim at most 256")
                need(m.scale is not None and m.scale > 0, f"{w}.scale must be positive")
                need(m.rot_dims >= 0 and m.rot_dims % 2 == 0 and m.rot_dims <= m.dim,
                     f"{w}.rot.dims must be even and at most dim")
                need(m.rot_dims == 0 or m.rot_base > 0, f"{w}.rot.base must be positive")
                need(m.mask_size >= 0 and m.keep_first >= 0, f"{w}.mask: size and keep_first must not be negative")
            if l.mlp is not None:
                f, w = l.mlp, f"layers[{i}].mlp"
                need(f.kind in MLP_KINDS, f"{w}.kind {f.kind!r} is not known (known: " + ", ".join(MLP_KINDS) + ")")
                need(f.ff > 0 and f.experts > 0, f"{w}: expert.ff and router.experts must be positive")
                need(1 <= f.groups <= 64 and f.experts % f.groups == 0, f"{w}.router.groups.count must divide the experts (at most 64 groups)")
                need(1 <= f.groups_keep <= f.groups, f"{w}.router.groups.keep must be between 1 and groups.count")
                need(1 <= f.top <= f.groups_keep * (f.experts // f.groups),
                     f"{w}.router.top must be at least 1 and fit into the kept groups")

    def model_spec(self) -> ModelSpec:
        W, std, eps = self.width, self.initializer_range, self.norm_eps
        norm = lambda name: PartSpec("rmsnorm", {"width": W, "eps": eps}, rename={"weight": name})
        layers, ignored = [], []
        for i, l in enumerate(self.layers):
            p = f"l{i}."
            m = l.mixer
            common = {"hidden_size": W, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim,
                      "value_dim": m.vdim, "conv_taps": m.conv, "norm_eps": eps, "init_std": std}
            weights = {f"{n}.weight": n for n in ("q", "k", "v", "o")}
            if l.type == "delta":
                mixer = PartSpec("gated_delta", common, prefix=p + "mix.",
                                 rename={**weights, "g.weight": "g", "a.weight": "a", "b.weight": "b",
                                         "norm.weight": "norm"})
            else:
                position = None
                if m.rot_dims > 0:
                    position = PartSpec("rope", {"theta": m.rot_base, "rotary_dim": m.rot_dims})
                mixer = PartSpec("differential_attention",
                                 {**common, "diff": m.diff, "scale": m.scale, "window": m.mask_size,
                                  "keep_first": m.keep_first, "position": position}, prefix=p + "mix.",
                                 rename={**weights, "q.bias": "q.b", "k.bias": "k.b", "v.bias": "v.b"})
            parts = {"mixer": mixer, "mixer_norm": norm(p + "norm1"), "mixer_post_norm": norm(p + "norm1b")}
            if l.mlp is not None:
                f = l.mlp
                rename = {"gate.weight": "router"}
                for e in range(f.experts):
                    rename[f"experts.{e}.up_proj.weight"] = f"e{e}.up"
                    rename[f"experts.{e}.down_proj.weight"] = f"e{e}.down"
                parts["feed_forward"] = PartSpec(
                    "moe", {"hidden_size": W, "num_experts": f.experts, "top_k": f.top, "expert_width": f.ff,
                            "gated": False, "activation": "relu2", "renormalize": False, "groups": f.groups,
                            "groups_keep": f.groups_keep, "init_std": std}, prefix=p + "mlp.", rename=rename)
                parts["feed_forward_norm"] = norm(p + "norm2")
                parts["feed_forward_post_norm"] = norm(p + "norm2b")
            else:  # a checkpoint may still hold the norms that the absent feed-forward would have had around it
                ignored += [p + "norm2", p + "norm2b"]
            layers.append(LayerSpec("sandwich_norm", parts))
        spec = ModelSpec(
            architecture=ARCHITECTURE, hidden_size=W, vocab_size=self.vocab, max_positions=0, layers=layers,
            schedule=[ScheduleEntry(i) for i in range(len(layers))],
            embedding=token_embedding("embed", self.vocab, W, std), final_norm=norm("final.norm"),
            head=linear_head("head", self.vocab, W, std, scale=self.logit_scale), init_std=std,
            ignored_tensor_suffixes=tuple(ignored))
        spec.validate()
        return spec


register_architecture(ARCHITECTURE, DezudraConfig)
