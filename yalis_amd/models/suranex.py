"""Suranex: a small decoder whose layers are listed one by one in config.json, each with a mixer
of its own kind and an optional feed-forward.

What the design fixes (everything else is read from config.json or a tensor's shape):
  * blocks norm the OUTPUT of each branch, x += norm(branch(x)), with RMS norms whose weight is
    stored around zero (multiplied as 1 + w); the final norm is of the same kind;
  * mixer "attention": grouped query heads; an RMS norm per head on queries and keys (plain
    weights shared by the heads); rotary positions in half-split pairs on the first ``rot.dims``
    elements with YaRN scaling; values divided by their root mean square, cached rotated by their
    own position over all of ``vdim`` with unscaled frequencies of the same base, and each head's
    output turned back by the query's position; scores times ``scale``, squashed by ``softcap``;
    a sliding window of ``mask.size`` keys below which the first ``mask.keep_first`` keys stay
    visible; a sigmoid gate per head computed from the mixer's input;
  * mixer "rglru": Griffin's recurrent block, decay constant 8;
  * feed-forward "moe": experts chosen by a table over token ids, each weighing 1 / top, plus an
    optional shared expert; experts are gated feed-forwards with the pair
    min(g, limit) * sigmoid(1.702 min(g, limit)) * (clamp(u, -limit, limit) + 1).

config.json: {"architecture": "Suranex", "vocab", "width", "norm": {"eps"}, "layers": [{"type",
"mixer": {...}, "mlp": {...} | null}]}; tensors "embed", "l<i>.norm1", "l<i>.norm2",
"l<i>.mix.*", "l<i>.mlp.*", "final.norm", "head".
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from ..config.reader import ConfigError, KeyReader
from ..config.registry import register_architecture
from ..config.specs import LayerSpec, ModelSpec, PartSpec, RunEntry

ARCHITECTURE_NAME = "Suranex"
RGLRU_RATE = 8.0  # log a = -8 r softplus(lam)
SWISH_SLOPE = 1.702  # the sigmoid's slope in the experts' gated pair
# config.json gives no longest sequence (the rotation has none); engines size their tables from
# their own max_model_len, which this bounds
MAX_POSITIONS = 1 << 20


@dataclass(frozen=True)
class SuranexLayer:
    kind: str  # "attention" | "rglru"
    mixer: Dict[str, Any]
    mlp: Optional[Dict[str, Any]]


@dataclass(frozen=True)
class SuranexConfig:
    vocab: int
    width: int
    eps: float
    layers: Tuple[SuranexLayer, ...]
    raw: Dict[str, Any]

    @staticmethod
    def _attention(m: Dict[str, Any], where: str) -> Dict[str, Any]:
        r = KeyReader(m, where=where)
        out = {
            "heads": r.integer("heads", minimum=1), "kv_heads": r.integer("kv_heads", minimum=1),
            "dim": r.integer("dim", minimum=1), "vdim": r.integer("vdim", minimum=2),
            "scale": r.number("scale", positive=True), "softcap": r.number("softcap", default=None, positive=True),
        }
        if out["heads"] % out["kv_heads"]:
            raise ConfigError(f"{where}: heads={out['heads']} is not a multiple of kv_heads={out['kv_heads']}")
        if out["vdim"] % 2:
            raise ConfigError(f"{where}: vdim={out['vdim']} must be even (values rotate in pairs)")
        mask = r.mapping("mask", default=None)
        out["window"], out["keep_first"] = None, 0
        if mask is not None:
            mr = KeyReader(mask, where=where + " mask")
            out["window"] = mr.integer("size", default=None, minimum=1)
            out["keep_first"] = mr.integer("keep_first", default=0, minimum=0)
            mr.finish()
        rot = KeyReader(r.mapping("rot"), where=where + " rot")
        out["rot_base"] = rot.number("base", positive=True)
        out["rot_dims"] = rot.integer("dims", minimum=2)
        if out["rot_dims"] % 2 or out["rot_dims"] > out["dim"]:
            raise ConfigError(f"{where}: rot.dims={out['rot_dims']} must be even and at most dim={out['dim']}")
        out["rot_scaling"] = None
        sc = rot.mapping("scaling", default=None)
        if sc is not None:
            sr = KeyReader(sc, where=where + " rot.scaling")
            out["rot_scaling"] = {
                "kind": "yarn", "factor": sr.number("factor", positive=True), "original": sr.number("original", positive=True),
                "fast": sr.number("fast", positive=True), "slow": sr.number("slow", positive=True),
            }
            sr.finish()
        rot.finish()
        r.finish()
        return out

    @staticmethod
    def _rglru(m: Dict[str, Any], where: str) -> Dict[str, Any]:
        r = KeyReader(m, where=where)
        out = {"width": r.integer("width", minimum=1), "blocks": r.integer("blocks", minimum=1), "conv": r.integer("conv", minimum=1)}
        if out["width"] % out["blocks"]:
            raise ConfigError(f"{where}: width={out['width']} does not divide into {out['blocks']} blocks")
        r.finish()
        return out

    @staticmethod
    def _mlp(f: Dict[str, Any], where: str) -> Dict[str, Any]:
        r = KeyReader(f, where=where)
        r.require_value("kind", ["moe"], default="moe")
        router = KeyReader(r.mapping("router"), where=where + " router")
        expert = KeyReader(r.mapping("expert"), where=where + " expert")
        out = {
            "experts": router.integer("experts", minimum=1), "top": router.integer("top", minimum=1),
            "ff": expert.integer("ff", minimum=1), "limit": expert.number("limit", positive=True), "shared": None,
        }
        if out["top"] > out["experts"]:
            raise ConfigError(f"{where}: top={out['top']} of {out['experts']} experts")
        shared = r.mapping("shared", default=None)
        if shared is not None:
            sr = KeyReader(shared, where=where + " shared")
            out["shared"] = {"ff": sr.integer("ff", minimum=1), "limit": sr.number("limit", positive=True)}
            sr.finish()
        router.finish()
        expert.finish()
        r.finish()
        return out

    @classmethod
    def from_dict(cls, raw: Dict[str, Any], strict: bool = False) -> "SuranexConfig":
        r = KeyReader(raw)
        vocab = r.integer("vocab", minimum=1)
        width = r.integer("width", minimum=1)
        eps = KeyReader(r.mapping("norm"), where="config.json norm").number("eps", positive=True)
        listed = r.raw_value("layers", None)
        if not isinstance(listed, list) or not listed:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        layers = []
        for i, entry in enumerate(listed):
            where = f"config.json layers[{i}]"
            if not isinstance(entry, dict):
                raise ConfigError(f"{where} must be an object")
            er = KeyReader(entry, where=where)
            kind = er.string("type")
            mixer = er.mapping("mixer")
            if kind == "attention":
                m = cls._attention(mixer, where + " mixer")
            elif kind == "rglru":
                m = cls._rglru(mixer, where + " mixer")
            else:
                raise ConfigError(f"{where}: mixer type {kind!r} is not one of this design's ('attention', 'rglru')")
            mlp = er.mapping("mlp", default=None)
            layers.append(SuranexLayer(kind, m, None if mlp is None else cls._mlp(mlp, where + " mlp")))
            er.finish()
        r.taken.add("architecture")
        r.finish(strict=strict)
        return cls(vocab, width, eps, tuple(layers), dict(raw))

    def to_dict(self) -> Dict[str, Any]:
        return dict(self.raw)


def build_suranex_spec(cfg: SuranexConfig) -> ModelSpec:
    def norm(name: str) -> PartSpec:
        return PartSpec("rmsnorm", {"name": name, "size": cfg.width, "eps": cfg.eps, "unit_offset": True})

    layers = []
    for i, layer in enumerate(cfg.layers):
        p, m = f"l{i}", layer.mixer
        if layer.kind == "attention":
            mixer = PartSpec("attention", {
                "prefix": f"{p}.mix", "hidden_size": cfg.width, "num_heads": m["heads"], "num_kv_heads": m["kv_heads"],
                "head_dim": m["dim"], "value_dim": m["vdim"], "scale": m["scale"], "softcap": m["softcap"],
                "window": m["window"], "keep_first": m["keep_first"],
                "names": {"q": "q", "k": "k", "v": "v", "o": "o"},
                "position": PartSpec("rotary", {"rotary_dim": m["rot_dims"], "theta": m["rot_base"], "pairing": "half",
                                                "scaling": m["rot_scaling"]}),
                "qk_norm": {"q": "q.norm", "k": "k.norm", "eps": cfg.eps},
                "value_norm_eps": cfg.eps,
                "value_position": PartSpec("rotary", {"rotary_dim": m["vdim"], "theta": m["rot_base"], "pairing": "half",
                                                      "scaling": None}),
                "gate": "g",
            })
        else:
            mixer = PartSpec("rglru", {"prefix": f"{p}.mix", "hidden_size": cfg.width, "width": m["width"], "blocks": m["blocks"],
                                       "conv_taps": m["conv"], "rate": RGLRU_RATE})
        ffn = ffn_norm = None
        if layer.mlp is not None:
            f = layer.mlp
            ffn = PartSpec("table_moe", {
                "prefix": f"{p}.mlp", "hidden_size": cfg.width, "vocab_size": cfg.vocab, "experts": f["experts"], "top": f["top"],
                "intermediate_size": f["ff"], "activation": ("clamped_swish", f["limit"], SWISH_SLOPE),
                "shared": None if f["shared"] is None else {
                    "intermediate_size": f["shared"]["ff"], "activation": ("clamped_swish", f["shared"]["limit"], SWISH_SLOPE)},
            })
            ffn_norm = norm(f"{p}.norm2")
        layers.append(LayerSpec.of(p, "branch_norm", mixer=mixer, mixer_norm=norm(f"{p}.norm1"), feed_forward=ffn,
                                   feed_forward_norm=ffn_norm))
    spec = ModelSpec(
        architecture=ARCHITECTURE_NAME,
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        max_positions=MAX_POSITIONS,
        embedding=PartSpec("token_embedding", {"name": "embed", "vocab_size": cfg.vocab, "hidden_size": cfg.width}),
        layers=tuple(layers),
        run_order=tuple(RunEntry(layer=i) for i in range(len(layers))),
        final_norm=norm("final.norm"),
        head=PartSpec("lm_head", {"name": "head", "tied_to": None, "vocab_size": cfg.vocab, "hidden_size": cfg.width}),
    )
    spec.validate()
    return spec


register_architecture(ARCHITECTURE_NAME, SuranexConfig, build_suranex_spec)
