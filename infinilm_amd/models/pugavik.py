"""Pugavik: a decoder-only model whose layers each run one mixer (a windowed softmax attention with normed queries
and keys, unit values, scores mixed over the heads and a learned term in the denominator; an attention over latent
rows; a gated linear attention) beside a feed-forward on the same layer-normed input, and in which a stretch of
layers may run several times in a row with the same weights.  This file holds everything that is specific to the
design: config.json's keys, their validation, the tensor names and the description of the model as parts.  No part and
no kernel knows of it.

config.json:  architecture "Pugavik"; vocab, width; embedding.scale; norm.eps;
  layers: a list of {type, mixer: {...}, mlp: {kind: "dense", ff} | null}
    type "attention":         mixer {heads, kv_heads, dim, vdim, scale, mask: {size}, rot: {dims, base}}
    type "latent_attention":  mixer {heads, dim, rot_dim, vdim, kv_rank, scale, rot: {base}}
    type "gla":               mixer {heads, dim, vdim, tau}  (the decay's low rank is the row count of <layer>.mix.a1;
                              a configuration without a checkpoint names it as `decay_rank`)
  loop: {start, stop, times} or absent: layers start .. stop-1 run `times` times in a row, each pass with a cache of its
    own; before every pass but the first the embedding's output is added to the stream again, and before every pass
    row t of the tensor loop.step [times, width].
Tensors: embed, head, final.norm, final.norm.b, loop.step; l<i>.norm1, l<i>.norm1.b; l<i>.mix.* and l<i>.mlp.{up,down}
(matrices stored [out, in], no ".weight" ending, biases end in ".b").
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from ..config.errors import ConfigError
from ..config.registry import register_architecture
from ..config.spec import HeadSpec, LayerRun, LayerSpec, ModelSpec, PartSpec, RunStart
from .kekevik import _need

MAX_POSITIONS = 1 << 30    # the design sets no limit: no table grows with the positions


@dataclass
class PugavikLayer:
    kind: str                       # attention | latent_attention | gla
    mixer: Dict[str, Any]           # the checked sizes and constants of its mixer
    ff: Optional[int]               # the feed-forward's inner size, None: the layer has none


@dataclass
class PugavikConfig:
    vocab: int
    width: int
    embedding_scale: float
    eps: float
    layers: List[PugavikLayer]
    loop: Optional[Dict[str, int]] = None      # {start, stop, times}
    dtype: Optional[str] = "bfloat16"
    eos_token_ids: List[int] = field(default_factory=list)
    raw: Dict[str, Any] = field(default_factory=dict, repr=False)

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "PugavikConfig":
        vocab, width = _need(raw, "vocab", "config", int), _need(raw, "width", "config", int)
        scale = _need(raw.get("embedding"), "scale", "config 'embedding'")
        eps = _need(raw.get("norm"), "eps", "config 'norm'")
        if eps < 0:
            raise ConfigError(f"norm.eps must not be negative, got {eps}")
        entries = _need(raw, "layers", "config", list)
        if not entries:
            raise ConfigError("config 'layers' is empty")
        layers = []
        for i, e in enumerate(entries):
            where = f"layers[{i}]"
            kind = _need(e, "type", where, str)
            m = _need(e, "mixer", where, dict)
            mw = where + ".mixer"
            if kind == "attention":
                mixer = {k: _need(m, k, mw, int) for k in ("heads", "kv_heads", "dim", "vdim")}
                if mixer["heads"] % mixer["kv_heads"]:
                    raise ConfigError(f"{mw}: {mixer['heads']} heads are no multiple of {mixer['kv_heads']} kv_heads")
                mixer["scale"] = _need(m, "scale", mw)
                mixer["window"] = _need(m.get("mask"), "size", mw + ".mask", int)
                rot = m.get("rot") or {}
                dims = int(rot.get("dims", 0) or 0)
                if dims < 0 or dims % 2 or dims > mixer["dim"]:
                    raise ConfigError(f"rot.dims in {mw} must be even and at most dim, got {dims}")
                mixer["rot"] = {"dims": dims, "base": _need(rot, "base", mw + ".rot") if dims else 1.0}
            elif kind == "latent_attention":
                mixer = {k: _need(m, k, mw, int) for k in ("heads", "dim", "vdim", "kv_rank")}
                rd = m.get("rot_dim", 0)
                if isinstance(rd, bool) or not isinstance(rd, int) or rd < 0 or rd % 2:
                    raise ConfigError(f"rot_dim in {mw} must be an even number, got {rd!r}")
                mixer["rot_dim"] = rd
                mixer["scale"] = _need(m, "scale", mw)
                mixer["base"] = _need(m.get("rot"), "base", mw + ".rot") if rd else 1.0
            elif kind == "gla":
                mixer = {k: _need(m, k, mw, int) for k in ("heads", "dim", "vdim")}
                mixer["tau"] = _need(m, "tau", mw)
                if mixer["tau"] <= 0:
                    raise ConfigError(f"tau in {mw} must be positive, got {mixer['tau']}")
                if m.get("decay_rank") is None:
                    raise ConfigError(f"{mw}: the decay's low rank is neither given as 'decay_rank' nor by a checkpoint's "
                                      f"tensor l{i}.mix.a1")
                mixer["decay_rank"] = _need(m, "decay_rank", mw, int)
            else:
                raise ConfigError(f"{where}: unknown layer type {kind!r} (attention, latent_attention, gla)")
            mlp = e.get("mlp")
            ff = None
            if mlp is not None:
                if mlp.get("kind", "dense") != "dense":
                    raise ConfigError(f"{where}.mlp: unknown kind {mlp.get('kind')!r} (dense)")
                ff = _need(mlp, "ff", where + ".mlp", int)
            layers.append(PugavikLayer(kind, mixer, ff))
        loop = raw.get("loop")
        if loop is not None:
            lw = "config 'loop'"
            times = _need(loop, "times", lw, int)
            start, stop = loop.get("start"), loop.get("stop")
            for k, v in (("start", start), ("stop", stop)):
                if isinstance(v, bool) or not isinstance(v, int):
                    raise ConfigError(f"Key '{k}' in {lw} must be an integer, got {v!r}")
            if not 0 <= start < stop <= len(layers):
                raise ConfigError(f"{lw}: layers {start} .. {stop - 1} are not a stretch of the {len(layers)} layers")
            loop = {"start": start, "stop": stop, "times": times}
        return cls(vocab=vocab, width=width, embedding_scale=scale, eps=eps, layers=layers, loop=loop, raw=dict(raw))


def sizes_from_checkpoint(raw: Dict[str, Any], shapes: Dict[str, tuple]) -> Dict[str, Any]:
    """config.json completed with the one size that only a tensor gives: the low rank of a gated layer's decay."""
    layers = raw.get("layers")
    if not isinstance(layers, list):
        return raw
    out = []
    for i, e in enumerate(layers):
        shape = shapes.get(f"l{i}.mix.a1")
        if isinstance(e, dict) and e.get("type") == "gla" and isinstance(e.get("mixer"), dict) and shape is not None \
                and len(shape) == 2 and e["mixer"].get("decay_rank") is None:
            e = dict(e, mixer=dict(e["mixer"], decay_rank=int(shape[0])))
        out.append(e)
    return dict(raw, layers=out)


def _mixer_spec(layer: PugavikLayer, W: int, eps: float) -> PartSpec:
    m = layer.mixer
    if layer.kind == "attention":
        position = PartSpec("normed_pair_rotary", {"dim": m["dim"], "value_dim": m["vdim"], "rotary_dim": m["rot"]["dims"],
                                                   "theta": m["rot"]["base"], "eps": eps, "qk_norm": True, "v_norm": True,
                                                   "names": ("q.norm", "k.norm")})
        return PartSpec("gqa_attention", {"hidden_size": W, "num_heads": m["heads"], "num_kv_heads": m["kv_heads"],
                                          "head_dim": m["dim"], "value_dim": m["vdim"], "qkv_bias": True, "out_bias": False,
                                          "scale": m["scale"], "window": m["window"], "position": position,
                                          "names": ("q", "k", "v", "o"), "suffix": "", "bias_suffix": "b", "head_mix": True,
                                          "sink": True, "mix_names": ("talk", "sink"), "position_prefix": ""})
    if layer.kind == "latent_attention":
        return PartSpec("latent_attention", {"hidden_size": W, "heads": m["heads"], "head_dim": m["dim"], "rotary_dim": m["rot_dim"],
                                             "value_dim": m["vdim"], "kv_rank": m["kv_rank"], "scale": m["scale"],
                                             "theta": m["base"], "eps": eps})
    return PartSpec("gated_linear_attention", {"hidden_size": W, "heads": m["heads"], "key_dim": m["dim"], "value_dim": m["vdim"],
                                               "decay_rank": m["decay_rank"], "tau": m["tau"], "eps": eps, "bias_suffix": "b"})


def build_spec(cfg: PugavikConfig) -> ModelSpec:
    """embed * scale -> runs (h = layer norm; x += mixer(h) + feed-forward(h)) -> layer norm -> head."""
    W = cfg.width
    norm = PartSpec("layernorm", {"size": W, "eps": cfg.eps, "bias": True, "param_name": "", "bias_name": "b"})
    layers = []
    for i, layer in enumerate(cfg.layers):
        parts = {"norm1": norm, "mixer": _mixer_spec(layer, W, cfg.eps)}
        names = {"norm1": "norm1", "mixer": "mix"}
        if layer.ff is not None:
            parts["ffn"] = PartSpec("activation_mlp", {"hidden_size": W, "intermediate_size": layer.ff, "activation": "gelu_tanh",
                                                       "bias": False, "names": ("up", "down"), "suffix": ""})
            names["ffn"] = "mlp"
        layers.append(LayerSpec(prefix=f"l{i}", arrangement="parallel_residual", parts=parts, names=names))
    # the order of runs: every run of a layer has a cache entry of its own
    n = len(layers)
    a, b, times = (cfg.loop["start"], cfg.loop["stop"], cfg.loop["times"]) if cfg.loop else (0, 0, 0)
    order: List[LayerRun] = []

    def add(i, start=None):
        order.append(LayerRun(layer=i, cache=len(order), writes_cache=True, start=start))

    for i in range(a):
        add(i)
    for t in range(times):
        for i in range(a, b):
            add(i, RunStart(embedding=1.0 if t > 0 else 0.0, vector_row=t) if i == a else None)
    for i in range(b, n):
        add(i)
    spec = ModelSpec(architecture="Pugavik", vocab_size=cfg.vocab, hidden_size=W, max_positions=MAX_POSITIONS,
                     embed_name="embed", embed_scale=cfg.embedding_scale, layers=layers, order=order, final_norm=norm,
                     final_norm_name="final.norm", head=HeadSpec(name="head", scale=1.0, tie_to_embedding_when_missing=False,
                                                                 params={"param_name": ""}),
                     eos_token_ids=list(cfg.eos_token_ids), embed_params={"param_name": ""},
                     run_vectors=("loop.step", times) if cfg.loop else None)
    spec.validate()
    return spec


register_architecture(["Pugavik", "pugavik"], PugavikConfig.from_dict, build_spec, sizes_from_checkpoint)
