"""A plain, slow implementation of the Pugavik design: whole sequences at once where a mechanism allows it, token by
token where it carries a state, one function per mechanism, in torch on the CPU (float64 unless told otherwise).  It
shares no code with the engine and is what the tests compare the engine with.

Notation: h is a sublayer's input row, p a token's position in its sequence (from 0), W x a stored [out, in] matrix
applied to a column.  `cfg` is config.json as a dict, `w` the tensors by name.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

_ROUND = [None]   # a dtype to which every projection's operands and result are rounded (see `forward`), or None


def proj(h: torch.Tensor, w: torch.Tensor, b: Optional[torch.Tensor] = None) -> torch.Tensor:
    """W h (+ b) for every row of h."""
    if _ROUND[0] is None:
        y = h @ w.T
        return y if b is None else y + b
    y = h.to(_ROUND[0]).to(h.dtype) @ w.T
    if b is not None:
        y = y + b
    return y.to(_ROUND[0]).to(h.dtype)


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def layer_norm(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float) -> torch.Tensor:
    mu = x.mean(-1, keepdim=True)
    dev = x - mu
    var = (dev * dev).mean(-1, keepdim=True)
    return dev / torch.sqrt(var + eps) * weight + bias


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(x: torch.Tensor) -> torch.Tensor:
    return x / (1.0 + torch.exp(-x))


def rotate_pairs(x: torch.Tensor, pos: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """x [T, heads, dim], pos [T]: entries (2i, 2i + 1), i < dims/2, of every head turn by pos * base^(-2i/dims);
    entries from `dims` on pass."""
    if dims == 0:
        return x
    i = torch.arange(dims // 2, dtype=x.dtype)
    freq = torch.pow(torch.tensor(float(base), dtype=x.dtype), -2.0 * i / dims)
    ang = pos.to(x.dtype)[:, None] * freq[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    even, odd = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = even * c - odd * s
    out[..., 1:dims:2] = odd * c + even * s
    return out


def dense_ff(h: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str) -> torch.Tensor:
    return proj(gelu_tanh(proj(h, w[prefix + ".up"])), w[prefix + ".down"])


def window_attention(h: torch.Tensor, m: dict, w: Dict[str, torch.Tensor], pre: str, eps: float) -> torch.Tensor:
    """Softmax attention over the last `mask.size` positions with: biased projections, a weighted RMS norm on every
    query and key head, pairwise rotation, values of unit root mean square, scores mixed over the heads by a matrix,
    and one more term exp(sink) in every head's denominator."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = proj(h, w[pre + ".q"], w[pre + ".q.b"]).view(T, H, dk)
    k = proj(h, w[pre + ".k"], w[pre + ".k.b"]).view(T, G, dk)
    v = proj(h, w[pre + ".v"], w[pre + ".v.b"]).view(T, G, dv)
    q = rms_unit(q, eps) * w[pre + ".q.norm"]
    k = rms_unit(k, eps) * w[pre + ".k.norm"]
    q = rotate_pairs(q, pos, m["rot"]["dims"], m["rot"]["base"])
    k = rotate_pairs(k, pos, m["rot"]["dims"], m["rot"]["base"])
    v = rms_unit(v, eps)
    kv_of = [g // (H // G) for g in range(H)]
    raw = torch.stack([q[:, g, :] @ k[:, kv_of[g], :].T for g in range(H)]) * m["scale"]       # [H, T(query), T(key)]
    mixed = torch.einsum("hg,gij->hij", w[pre + ".talk"].to(raw.dtype), raw)
    i, j = pos[:, None], pos[None, :]
    seen = (j <= i) & (i - j < m["mask"]["size"])
    mixed = mixed.masked_fill(~seen[None], -math.inf)
    top = torch.maximum(mixed.max(-1, keepdim=True).values, w[pre + ".sink"].to(raw.dtype)[:, None, None])
    e = torch.exp(mixed - top)
    denom = e.sum(-1, keepdim=True) + torch.exp(w[pre + ".sink"].to(raw.dtype)[:, None, None] - top)
    prob = e / denom
    out = torch.stack([prob[g] @ v[:, kv_of[g], :] for g in range(H)], dim=1)                  # [T, H, dv]
    if _ROUND[0] is not None:
        out = out.to(_ROUND[0]).to(h.dtype)
    return proj(out.reshape(T, H * dv), w[pre + ".o"])


def latent_attention(h: torch.Tensor, m: dict, w: Dict[str, torch.Tensor], pre: str, eps: float) -> torch.Tensor:
    """Causal softmax attention whose keys and values are made from a small latent row a token: keys = [W_uk c,
    one rotated part shared by the heads], values = W_uv c."""
    T = h.shape[0]
    H, dn, dr, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    q = proj(h, w[pre + ".q"]).view(T, H, dn + dr)
    q_plain, q_turn = q[..., :dn], rotate_pairs(q[..., dn:], pos, dr, m["rot"]["base"])
    down = proj(h, w[pre + ".dkv"])
    c = rms_unit(down[:, :rank], eps) * w[pre + ".dkv.norm"]
    if _ROUND[0] is not None:
        c = c.to(_ROUND[0]).to(h.dtype)
    k_turn = rotate_pairs(down[:, None, rank:], pos, dr, m["rot"]["base"])[:, 0]              # [T, dr]
    k_plain = proj(c, w[pre + ".uk"]).view(T, H, dn)
    v = proj(c, w[pre + ".uv"]).view(T, H, dv)
    score = (torch.einsum("ihd,jhd->hij", q_plain, k_plain) + torch.einsum("ihd,jd->hij", q_turn, k_turn)) * m["scale"]
    score = score.masked_fill(~(pos[None, :] <= pos[:, None])[None], -math.inf)
    prob = torch.softmax(score, dim=-1)
    out = torch.einsum("hij,jhd->ihd", prob, v)
    if _ROUND[0] is not None:
        out = out.to(_ROUND[0]).to(h.dtype)
    return proj(out.reshape(T, H * dv), w[pre + ".o"])


def channel_decay_scan(q, k, v, alpha):
    """q, k, alpha [T, heads, dk], v [T, heads, dv]: S_t = diag(alpha_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t."""
    T, H, dk = q.shape
    S = torch.zeros((H, dk, v.shape[-1]), dtype=q.dtype)
    out = torch.empty((T, H, v.shape[-1]), dtype=q.dtype)
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hkv,hk->hv", S, q[t])
    return out


def gated_linear_attention(h: torch.Tensor, m: dict, w: Dict[str, torch.Tensor], pre: str, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    q = proj(h, w[pre + ".q"]).view(T, H, dk) * dk ** -0.5
    k = proj(h, w[pre + ".k"]).view(T, H, dk)
    v = proj(h, w[pre + ".v"]).view(T, H, dv)
    z = proj(proj(h, w[pre + ".a1"]), w[pre + ".a2"], w[pre + ".a2.b"]).view(T, H, dk)
    alpha = torch.sigmoid(z) ** (1.0 / m["tau"])
    o = rms_unit(channel_decay_scan(q, k, v, alpha), eps) * w[pre + ".norm"]
    y = o.reshape(T, H * dv) * silu(proj(h, w[pre + ".g"]))
    return proj(y, w[pre + ".o"])


MIXERS = {"attention": window_attention, "latent_attention": latent_attention, "gla": gated_linear_attention}


def run_order(cfg: dict) -> List[tuple]:
    """[(layer, pass or None if the run opens no pass)]: layers start .. stop-1 `times` times in a row, the rest once."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    a, b, times = loop["start"], loop["stop"], loop["times"]
    order = [(i, None) for i in range(a)]
    for t in range(times):
        order += [(i, t if i == a else None) for i in range(a, b)]
    return order + [(i, None) for i in range(b, n)]


def forward(cfg: dict, w: Dict[str, torch.Tensor], tokens, dtype=torch.float64, round_to=None, layers_out: Optional[list] = None):
    """Logits [T, vocab] of one sequence.  `round_to`: projections take operands and give results rounded to that
    dtype (what a bfloat16 engine does at its matrix products), everything else stays in `dtype`."""
    _ROUND[0] = round_to
    try:
        w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in w.items()}
        eps = cfg["norm"]["eps"]
        x0 = w["embed"][torch.as_tensor(tokens, dtype=torch.long)] * cfg["embedding"]["scale"]
        x = x0.clone()
        for i, opens in run_order(cfg):
            if opens is not None:
                if opens > 0:
                    x = x + x0
                x = x + w["loop.step"][opens]
            layer, pre = cfg["layers"][i], f"l{i}"
            h = layer_norm(x, w[pre + ".norm1"], w[pre + ".norm1.b"], eps)
            y = MIXERS[layer["type"]](h, layer["mixer"], w, pre + ".mix", eps)
            if layer.get("mlp") is not None:
                y = y + dense_ff(h, w, pre + ".mlp")
            x = x + y
            if layers_out is not None:
                layers_out.append(x.clone())
        x = layer_norm(x, w["final.norm"], w["final.norm.b"], eps)
        return x @ w["head"].T
    finally:
        _ROUND[0] = None


def tensor_shapes(cfg: dict) -> Dict[str, tuple]:
    """Every tensor of a model of this configuration, by name."""
    W, V = cfg["width"], cfg["vocab"]
    out = {"embed": (V, W), "final.norm": (W,), "final.norm.b": (W,), "head": (V, W)}
    if cfg.get("loop"):
        out["loop.step"] = (cfg["loop"]["times"], W)
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}", layer["mixer"]
        out[p + ".norm1"] = out[p + ".norm1.b"] = (W,)
        if layer["type"] == "attention":
            H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            out.update({p + ".mix.q": (H * dk, W), p + ".mix.q.b": (H * dk,), p + ".mix.k": (G * dk, W), p + ".mix.k.b": (G * dk,),
                        p + ".mix.v": (G * dv, W), p + ".mix.v.b": (G * dv,), p + ".mix.q.norm": (dk,), p + ".mix.k.norm": (dk,),
                        p + ".mix.talk": (H, H), p + ".mix.sink": (H,), p + ".mix.o": (W, H * dv)})
        elif layer["type"] == "latent_attention":
            H, dn, dr, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            out.update({p + ".mix.q": (H * (dn + dr), W), p + ".mix.dkv": (r + dr, W), p + ".mix.dkv.norm": (r,),
                        p + ".mix.uk": (H * dn, r), p + ".mix.uv": (H * dv, r), p + ".mix.o": (W, H * dv)})
        else:
            H, dk, dv, low = m["heads"], m["dim"], m["vdim"], m["decay_rank"]
            out.update({p + ".mix.q": (H * dk, W), p + ".mix.k": (H * dk, W), p + ".mix.v": (H * dv, W), p + ".mix.g": (H * dv, W),
                        p + ".mix.o": (W, H * dv), p + ".mix.norm": (dv,), p + ".mix.a1": (low, W), p + ".mix.a2": (H * dk, low),
                        p + ".mix.a2.b": (H * dk,)})
        if layer.get("mlp") is not None:
            out[p + ".mlp.up"], out[p + ".mlp.down"] = (layer["mlp"]["ff"], W), (W, layer["mlp"]["ff"])
    return out


def greedy(cfg: dict, w: Dict[str, torch.Tensor], prompt, n: int) -> List[int]:
    """The n tokens greedy decoding appends to `prompt` (the whole sequence is run again for every token)."""
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(torch.argmax(forward(cfg, w, toks)[-1])))
    return toks[len(prompt):]


def random_weights(cfg: dict, seed: int) -> Dict[str, torch.Tensor]:
    """float32 tensors: matrices N(0, 1/in), norm weights near one, small biases, a head-mixing matrix near the identity
    with sizeable off-diagonal entries, sinks of order one."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in sorted(tensor_shapes(cfg).items()):
        last = name.rsplit(".", 1)[-1]
        if name.endswith(".talk"):
            t = torch.eye(shape[0]) + 0.3 * torch.randn(shape, generator=g)
        elif name.endswith(".sink"):
            t = torch.randn(shape, generator=g)
        elif name.endswith(".a2.b"):
            t = 2.0 + torch.randn(shape, generator=g)                 # decays mostly near one, some fast
        elif last == "b":
            t = 0.1 * torch.randn(shape, generator=g)
        elif len(shape) == 1:
            t = 1.0 + 0.1 * torch.randn(shape, generator=g)
        elif name in ("embed", "loop.step"):
            t = torch.randn(shape, generator=g)
        else:
            t = torch.randn(shape, generator=g) / math.sqrt(shape[1])
        out[name] = t
    return out


def _attention(heads, kv_heads, dim, vdim, window, rot_dims, base=10000.0, scale=None):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": window},
            "rot": {"dims": rot_dims, "base": base}, "scale": scale if scale is not None else dim ** -0.5}


def _latent(heads, dim, rot_dim, vdim, kv_rank, base=10000.0, scale=None):
    return {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "rot": {"base": base, "dims": rot_dim},
            "scale": scale if scale is not None else (dim + rot_dim) ** -0.5}


def _gla(heads, dim, vdim, tau, decay_rank):
    return {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau, "decay_rank": decay_rank}


def _layer(kind, mixer, ff):
    return {"type": kind, "mixer": mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def config_a():
    """No loop; a gated layer first; equal key and value sizes, as many key/value heads as heads, a part of each head turned;
    a layer without a feed-forward."""
    return {"architecture": "Pugavik", "vocab": 97, "width": 64, "embedding": {"scale": 1.5}, "norm": {"eps": 1e-6}, "layers": [
        _layer("gla", _gla(2, 16, 24, 4.0, 4), 96),
        _layer("attention", _attention(4, 4, 16, 16, 7, 8, base=100.0), None),
        _layer("latent_attention", _latent(2, 8, 4, 12, 20), 80)]}


def config_b():
    """Layers 1 and 2 run three times; head sizes that are no multiples of 16 or 8; whole heads turned; one key/value head for
    two query heads; tau 1."""
    return {"architecture": "Pugavik", "vocab": 131, "width": 96, "embedding": {"scale": 0.7}, "norm": {"eps": 1e-5}, "layers": [
        _layer("latent_attention", _latent(3, 16, 8, 16, 40, base=500.0), 128),
        _layer("attention", _attention(6, 3, 12, 20, 33, 12, base=50000.0, scale=0.3), 64),
        _layer("gla", _gla(3, 20, 8, 1.0, 6), 100),
        _layer("attention", _attention(2, 1, 24, 8, 5, 0), 48)],
        "loop": {"start": 1, "stop": 3, "times": 3}}


def config_c():
    """Sizes that take the matrix-core kernels (latent rows of 128 with the turned part, heads of 64); the first layer alone
    runs twice; one key/value head for all heads in one layer; a window longer than most prompts."""
    return {"architecture": "Pugavik", "vocab": 300, "width": 256, "embedding": {"scale": 1.0}, "norm": {"eps": 1e-5}, "layers": [
        _layer("latent_attention", _latent(4, 32, 32, 64, 96), 512),
        _layer("attention", _attention(8, 2, 64, 32, 100, 32), 384),
        _layer("gla", _gla(4, 64, 64, 16.0, 16), 256),
        _layer("attention", _attention(4, 1, 32, 48, 200, 16, base=1e6), None),
        _layer("latent_attention", _latent(2, 64, 16, 32, 160), 256)],
        "loop": {"start": 0, "stop": 1, "times": 2}}


CONFIGS = {"A": config_a, "B": config_b, "C": config_c}
