"""Kekevik: a decoder-only model whose layers each pick one of three mixers (a retention with rotated queries and
keys, a lightning attention, or a capped softmax attention beside a selective state space), with a norm before and
after every sublayer, a squared-relu feed-forward, and logits read from the embedding table.  This file holds
everything that is specific to the design: config.json's keys, their validation, the tensor names and the
description of the model as parts.  No part and no kernel knows of it.

config.json:  architecture "Kekevik"; vocab, width; embedding.scale; norm.eps; layers: a list of
  {type, mixer: {...}, mlp: {kind: "dense", ff} | null}
    type "retention":  mixer {heads, dim, vdim, decay: [heads], rot: {dims, base}}
    type "lightning":  mixer {heads, dim, vdim, decay: [heads]}
    type "parallel":   mixer {left: {heads, kv_heads, dim, vdim, scale, softcap, q_temp: {coef, every}},
                              right: {heads, vdim, state, groups, conv, norm_groups}, left_scale, right_scale}
Tensors: embed; l<i>.norm1, .norm1b, .norm2, .norm2b; l<i>.mix.* and l<i>.mlp.{up,down} (matrices stored [out, in],
no ".weight" ending); final.norm.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from ..config.errors import ConfigError
from ..config.registry import register_architecture
from ..config.spec import HeadSpec, LayerRun, LayerSpec, ModelSpec, PartSpec

MAX_POSITIONS = 1 << 30    # the design sets no limit: no table grows with the positions


def _need(d: Dict[str, Any], key: str, where: str, typ=(int, float)):
    if not isinstance(d, dict) or key not in d or d[key] is None:
        raise ConfigError(f"Key '{key}' not found in {where}.")
    v = d[key]
    if typ is int:
        if isinstance(v, bool) or not isinstance(v, (int, float)) or int(v) != v or int(v) <= 0:
            raise ConfigError(f"Key '{key}' in {where} must be a positive integer, got {v!r}")
        return int(v)
    if typ == (int, float):
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"Key '{key}' in {where} must be a number, got {v!r}")
        return float(v)
    if not isinstance(v, typ):
        raise ConfigError(f"Key '{key}' in {where} must be {typ.__name__}, got {v!r}")
    return v


def _decays(m: dict, heads: int, where: str) -> List[float]:
    d = _need(m, "decay", where, list)
    if len(d) != heads or any(isinstance(a, bool) or not isinstance(a, (int, float)) for a in d):
        raise ConfigError(f"'decay' in {where} must list one number for each of the {heads} heads")
    return [float(a) for a in d]


@dataclass
class KekevikLayer:
    kind: str                       # retention | lightning | parallel
    mixer: Dict[str, Any]           # the checked sizes and constants of its mixer
    ff: Optional[int]               # the feed-forward's inner size, None: the layer has none


@dataclass
class KekevikConfig:
    vocab: int
    width: int
    embedding_scale: float
    eps: float
    layers: List[KekevikLayer]
    dtype: Optional[str] = "bfloat16"
    eos_token_ids: List[int] = field(default_factory=list)
    raw: Dict[str, Any] = field(default_factory=dict, repr=False)

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "KekevikConfig":
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
            if kind in ("retention", "lightning"):
                heads = _need(m, "heads", mw, int)
                mixer = {"heads": heads, "dim": _need(m, "dim", mw, int), "vdim": _need(m, "vdim", mw, int),
                         "decay": _decays(m, heads, mw)}
                if kind == "retention":
                    rot = m.get("rot") or {}
                    dims = int(rot.get("dims", 0) or 0)
                    if dims < 0 or dims % 2 or dims > mixer["dim"]:
                        raise ConfigError(f"rot.dims in {mw} must be even and at most dim, got {dims}")
                    mixer["rot"] = {"dims": dims, "base": _need(rot, "base", mw + ".rot") if dims else 1.0}
            elif kind == "parallel":
                l, r = _need(m, "left", mw, dict), _need(m, "right", mw, dict)
                lw, rw = mw + ".left", mw + ".right"
                left = {"heads": _need(l, "heads", lw, int), "kv_heads": _need(l, "kv_heads", lw, int),
                        "dim": _need(l, "dim", lw, int), "vdim": _need(l, "vdim", lw, int), "scale": _need(l, "scale", lw),
                        "softcap": float(l.get("softcap") or 0.0)}
                if left["heads"] % left["kv_heads"]:
                    raise ConfigError(f"{lw}: {left['heads']} heads are no multiple of {left['kv_heads']} kv_heads")
                qt = l.get("q_temp")
                left["q_temp"] = {"coef": _need(qt, "coef", lw + ".q_temp"), "every": _need(qt, "every", lw + ".q_temp", int)} \
                    if qt else {"coef": 0.0, "every": 0}
                right = {k: _need(r, k, rw, int) for k in ("heads", "vdim", "state", "groups", "conv", "norm_groups")}
                if right["heads"] % right["groups"]:
                    raise ConfigError(f"{rw}: {right['heads']} heads are no multiple of {right['groups']} groups")
                if (right["heads"] * right["vdim"]) % right["norm_groups"]:
                    raise ConfigError(f"{rw}: heads * vdim is no multiple of norm_groups {right['norm_groups']}")
                mixer = {"left": left, "right": right, "left_scale": _need(m, "left_scale", mw),
                         "right_scale": _need(m, "right_scale", mw)}
            else:
                raise ConfigError(f"{where}: unknown layer type {kind!r} (retention, lightning, parallel)")
            mlp = e.get("mlp")
            ff = None
            if mlp is not None:
                if mlp.get("kind", "dense") != "dense":
                    raise ConfigError(f"{where}.mlp: unknown kind {mlp.get('kind')!r} (dense)")
                ff = _need(mlp, "ff", where + ".mlp", int)
            layers.append(KekevikLayer(kind, mixer, ff))
        return cls(vocab=vocab, width=width, embedding_scale=scale, eps=eps, layers=layers, raw=dict(raw))


def _mixer_spec(layer: KekevikLayer, W: int, eps: float) -> PartSpec:
    m = layer.mixer
    if layer.kind == "retention":
        return PartSpec("retention", {"hidden_size": W, "heads": m["heads"], "key_dim": m["dim"], "value_dim": m["vdim"],
                                      "decay": m["decay"], "eps": eps, "rotary": m["rot"]})
    if layer.kind == "lightning":
        return PartSpec("lightning_attention", {"hidden_size": W, "heads": m["heads"], "key_dim": m["dim"],
                                                "value_dim": m["vdim"], "decay": m["decay"], "eps": eps})
    l, r = m["left"], m["right"]
    position = PartSpec("unit_norm_temperature", {"dim": l["dim"], "normed": True, "eps": eps, "coef": l["q_temp"]["coef"],
                                                  "every": l["q_temp"]["every"]})
    left = PartSpec("gqa_attention", {"hidden_size": W, "num_heads": l["heads"], "num_kv_heads": l["kv_heads"],
                                      "head_dim": l["dim"], "value_dim": l["vdim"], "qkv_bias": False, "out_bias": False,
                                      "scale": l["scale"], "softcap": l["softcap"], "window": 0, "position": position,
                                      "names": ("q", "k", "v", "o"), "suffix": "", "whole_output": True})
    right = PartSpec("selective_state_space", {"hidden_size": W, "heads": r["heads"], "head_dim": r["vdim"],
                                               "state_size": r["state"], "groups": r["groups"], "conv_taps": r["conv"],
                                               "norm_groups": r["norm_groups"], "eps": eps})
    return PartSpec("parallel", {"branches": (left, right), "scales": (m["left_scale"], m["right_scale"]),
                                 "names": ("left", "right")})


def build_spec(cfg: KekevikConfig) -> ModelSpec:
    """embed * scale -> layers (norm, mixer, norm, +; norm, feed-forward, norm, +) -> norm -> logits from the table."""
    W = cfg.width
    norm = PartSpec("rmsnorm", {"size": W, "eps": cfg.eps, "param_name": ""})
    layers = []
    for i, layer in enumerate(cfg.layers):
        parts = {"norm1": norm, "mixer": _mixer_spec(layer, W, cfg.eps), "norm1b": norm}
        names = {"norm1": "norm1", "mixer": "mix", "norm1b": "norm1b"}
        if layer.ff is not None:
            parts.update(norm2=norm, norm2b=norm,
                         ffn=PartSpec("activation_mlp", {"hidden_size": W, "intermediate_size": layer.ff, "activation": "relu2",
                                                         "bias": False, "names": ("up", "down"), "suffix": ""}))
            names.update(norm2="norm2", ffn="mlp", norm2b="norm2b")
        layers.append(LayerSpec(prefix=f"l{i}", arrangement="sandwich_norm", parts=parts, names=names))
    order = [LayerRun(layer=i, cache=i, writes_cache=True) for i in range(len(layers))]
    spec = ModelSpec(architecture="Kekevik", vocab_size=cfg.vocab, hidden_size=W, max_positions=MAX_POSITIONS,
                     embed_name="embed", embed_scale=cfg.embedding_scale, layers=layers, order=order, final_norm=norm,
                     final_norm_name="final.norm", head=HeadSpec(name="", scale=1.0, always_tied=True),
                     eos_token_ids=list(cfg.eos_token_ids), embed_params={"param_name": ""})
    spec.validate()
    return spec


register_architecture(["Kekevik", "kekevik"], KekevikConfig.from_dict, build_spec)
