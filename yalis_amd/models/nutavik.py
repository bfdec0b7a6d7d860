"""Nutavik: a small decoder whose config.json lists its layers one by one, each with one of three
mixers and an optional dense feed-forward, between layer norms on both sides of every branch.

What the design fixes (everything else is read from config.json or a tensor's shape):
  * a layer is  x += m * post_1(mixer(pre_1(x)));  x += m * post_2(ff(pre_2(x)))  with m =
    ``residual_mult`` and all four norms layer norms with weight and bias (tensor ``<name>.b``);
    the final norm is of the same kind; the output head is the embedding table, its logits
    multiplied by ``logit_scale``;
  * mixer "latent_attention": queries through a normed latent (``q_rank``), keys and values
    through a normed latent of ``kv_rank`` elements that is all the cache holds beside one rotated
    key part of ``rot_dim`` elements shared by the heads; rotary positions in interleaved pairs
    with YaRN scaling on that part only; causal softmax attention; a sigmoid gate per head; a
    layer may read an earlier layer's cache (``kv_from``) with up-projections of its own;
  * mixer "delta": the gated delta rule on a matrix state per head, behind short causal
    convolutions with silu on q, k and v, unit-length q and k (1e-6 under the root), a sigmoid
    write strength and one decay per head, exp(-exp(A_log) softplus(a + dt_bias));
  * mixer "gla": gated linear attention with a decay per key channel, sigmoid(z)^(1/tau), z from a
    low-rank pair of projections with a bias;
  * both recurrent mixers norm each head's read-out (RMS, one weight shared by the heads) and gate
    it with silu of a projection of the mixer's input;
  * feed-forward "dense": down(relu(up h)^2).

config.json: {"architecture": "Nutavik", "vocab", "width", "residual_mult", "logit_scale", "norm":
{"eps"}, "layers": [{"type", "mixer": {...}, "mlp": {"kind": "dense", "ff"} | null}]}; tensors "embed",
"l<i>.norm1|norm2|norm1b|norm2b" (+ ".b"), "l<i>.mix.*", "l<i>.mlp.up|down", "final.norm" (+ ".b").
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from ..config.reader import ConfigError, KeyReader
from ..config.registry import register_architecture
from ..config.specs import LayerSpec, ModelSpec, PartSpec, RunEntry

ARCHITECTURE_NAME = "Nutavik"
UNIT_EPS = 1e-6  # under the root when the delta rule's q and k are made unit vectors
# config.json gives no longest sequence; engines size their tables from their own max_model_len
MAX_POSITIONS = 1 << 20
MIXERS = ("latent_attention", "delta", "gla")


@dataclass(frozen=True)
class NutavikLayer:
    kind: str
    mixer: Dict[str, Any]
    mlp: Optional[Dict[str, Any]]


@dataclass(frozen=True)
class NutavikConfig:
    vocab: int
    width: int
    eps: float
    residual_mult: float
    logit_scale: float
    layers: Tuple[NutavikLayer, ...]
    raw: Dict[str, Any]

    @staticmethod
    def _rotation(m: Dict[str, Any], where: str) -> Dict[str, Any]:
        rot = KeyReader(m, where=where)
        out = {"base": rot.number("base", positive=True), "dims": rot.integer("dims", minimum=2), "scaling": None}
        sc = rot.mapping("scaling", default=None)
        if sc is not None:
            sr = KeyReader(sc, where=where + ".scaling")
            out["scaling"] = {"kind": "yarn", "factor": sr.number("factor", positive=True), "original": sr.number("original", positive=True),
                              "fast": sr.number("fast", positive=True), "slow": sr.number("slow", positive=True)}
            sr.finish()
        rot.finish()
        return out

    @classmethod
    def _latent_attention(cls, m: Dict[str, Any], where: str) -> Dict[str, Any]:
        r = KeyReader(m, where=where)
        out = {"heads": r.integer("heads", minimum=1), "dim": r.integer("dim", minimum=1), "rot_dim": r.integer("rot_dim", minimum=2),
               "vdim": r.integer("vdim", minimum=1), "kv_rank": r.integer("kv_rank", minimum=1), "q_rank": r.integer("q_rank", minimum=1),
               "scale": r.number("scale", positive=True), "kv_from": r.integer("kv_from", default=None, minimum=0),
               "rot": cls._rotation(r.mapping("rot"), where + " rot")}
        if out["rot"]["dims"] != out["rot_dim"] or out["rot_dim"] % 2:
            raise ConfigError(f"{where}: the rotated part has rot_dim={out['rot_dim']} elements, all of which rotate in pairs "
                              f"(rot.dims={out['rot']['dims']})")
        r.finish()
        return out

    @staticmethod
    def _delta(m: Dict[str, Any], where: str) -> Dict[str, Any]:
        r = KeyReader(m, where=where)
        out = {"heads": r.integer("heads", minimum=1), "kv_heads": r.integer("kv_heads", minimum=1), "dim": r.integer("dim", minimum=1),
               "vdim": r.integer("vdim", minimum=1), "conv": r.integer("conv", minimum=1)}
        if out["heads"] % out["kv_heads"]:
            raise ConfigError(f"{where}: heads={out['heads']} is not a multiple of kv_heads={out['kv_heads']}")
        r.finish()
        return out

    @staticmethod
    def _gla(m: Dict[str, Any], where: str) -> Dict[str, Any]:
        r = KeyReader(m, where=where)
        out = {"heads": r.integer("heads", minimum=1), "dim": r.integer("dim", minimum=1), "vdim": r.integer("vdim", minimum=1),
               "tau": r.number("tau", positive=True),
               # the rank of the decay's pair of projections: read from the tensors' shapes unless given
               "low_rank": r.integer("low_rank", default=None, minimum=1)}
        r.finish()
        return out

    @classmethod
    def from_dict(cls, raw: Dict[str, Any], strict: bool = False) -> "NutavikConfig":
        r = KeyReader(raw)
        vocab, width = r.integer("vocab", minimum=1), r.integer("width", minimum=1)
        eps = KeyReader(r.mapping("norm"), where="config.json norm").number("eps", positive=True)
        mult = r.number("residual_mult", default=1.0)
        logit_scale = r.number("logit_scale", default=1.0)
        listed = r.raw_value("layers", None)
        if not isinstance(listed, list) or not listed:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        readers = {"latent_attention": cls._latent_attention, "delta": cls._delta, "gla": cls._gla}
        layers = []
        for i, entry in enumerate(listed):
            where = f"config.json layers[{i}]"
            if not isinstance(entry, dict):
                raise ConfigError(f"{where} must be an object")
            er = KeyReader(entry, where=where)
            kind = er.string("type")
            if kind not in readers:
                raise ConfigError(f"{where}: mixer type {kind!r} is not one of this design's {MIXERS}")
            m = readers[kind](er.mapping("mixer"), where + " mixer")
            mlp = er.mapping("mlp", default=None)
            if mlp is not None:
                fr = KeyReader(mlp, where=where + " mlp")
                fr.require_value("kind", ["dense"], default="dense")
                mlp = {"ff": fr.integer("ff", minimum=1)}
                fr.finish()
            er.finish()
            layers.append(NutavikLayer(kind, m, mlp))
        for i, layer in enumerate(layers):
            j = layer.mixer.get("kv_from") if layer.kind == "latent_attention" else None
            if j is None:
                continue
            where = f"config.json layers[{i}] mixer"
            if not j < i or layers[j].kind != "latent_attention" or layers[j].mixer["kv_from"] is not None:
                raise ConfigError(f"{where}: kv_from={j} must name an earlier latent_attention layer that keeps a cache of its own")
            for key in ("kv_rank", "rot_dim", "rot"):
                if layers[j].mixer[key] != layer.mixer[key]:
                    raise ConfigError(f"{where}: '{key}' differs from layer {j}'s, whose cache this layer reads")
        r.taken.add("architecture")
        r.finish(strict=strict)
        return cls(vocab, width, eps, mult, logit_scale, tuple(layers), dict(raw))

    def to_dict(self) -> Dict[str, Any]:
        return dict(self.raw)


def build_nutavik_spec(cfg: NutavikConfig) -> ModelSpec:
    def norm(name: str) -> PartSpec:
        return PartSpec("layernorm", {"name": name, "bias": name + ".b", "size": cfg.width, "eps": cfg.eps})

    layers = []
    for i, layer in enumerate(cfg.layers):
        p, m = f"l{i}", layer.mixer
        common = {"prefix": f"{p}.mix", "hidden_size": cfg.width}
        if layer.kind == "latent_attention":
            mixer = PartSpec("latent_attention", dict(
                common, num_heads=m["heads"], head_dim=m["dim"], rot_dim=m["rot_dim"], value_dim=m["vdim"], kv_rank=m["kv_rank"],
                q_rank=m["q_rank"], scale=m["scale"], latent_eps=cfg.eps, gate="g",
                position=PartSpec("rotary", {"rotary_dim": m["rot"]["dims"], "theta": m["rot"]["base"], "pairing": "interleaved",
                                             "scaling": m["rot"]["scaling"]})))
        elif layer.kind == "delta":
            mixer = PartSpec("delta_rule", dict(
                common, num_heads=m["heads"], num_kv_heads=m["kv_heads"], head_dim=m["dim"], value_dim=m["vdim"], conv_taps=m["conv"],
                unit_eps=UNIT_EPS, out_norm_eps=cfg.eps))
        else:
            mixer = PartSpec("gated_linear_attention", dict(
                common, num_heads=m["heads"], head_dim=m["dim"], value_dim=m["vdim"], tau=m["tau"], low_rank=m["low_rank"],
                out_norm_eps=cfg.eps))
        ffn = ffn_norm = ffn_out = None
        if layer.mlp is not None:
            ffn = PartSpec("dense_mlp", {"prefix": f"{p}.mlp", "hidden_size": cfg.width, "intermediate_size": layer.mlp["ff"],
                                         "activation": "relu2", "names": {"up": "up", "down": "down"}})
            ffn_norm, ffn_out = norm(f"{p}.norm2"), norm(f"{p}.norm2b")
        layers.append(LayerSpec.of(p, "sandwich", mixer_norm=norm(f"{p}.norm1"), mixer=mixer, mixer_out_norm=norm(f"{p}.norm1b"),
                                   feed_forward_norm=ffn_norm, feed_forward=ffn, feed_forward_out_norm=ffn_out)
                      .with_params(branch_scale=cfg.residual_mult))
    # a layer with kv_from reads the cache of the run entry of the layer it names
    order = tuple(RunEntry(layer=i, cache_from=layer.mixer.get("kv_from") if layer.kind == "latent_attention" else None)
                  for i, layer in enumerate(cfg.layers))
    spec = ModelSpec(
        architecture=ARCHITECTURE_NAME,
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        max_positions=MAX_POSITIONS,
        embedding=PartSpec("token_embedding", {"name": "embed", "vocab_size": cfg.vocab, "hidden_size": cfg.width}),
        layers=tuple(layers),
        run_order=order,
        final_norm=norm("final.norm"),
        head=PartSpec("lm_head", {"name": "head", "tied_to": "embed", "vocab_size": cfg.vocab, "hidden_size": cfg.width,
                                  "scale": cfg.logit_scale}),
    )
    spec.validate()
    return spec


register_architecture(ARCHITECTURE_NAME, NutavikConfig, build_nutavik_spec)
