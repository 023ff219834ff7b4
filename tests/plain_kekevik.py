"""A plain, slow implementation of the Kekevik design: token by token, one function per mechanism, in torch on
the CPU (float64 unless told otherwise).  It shares no code with the engine and is what the tests compare the
engine with.

Notation: h is a sublayer's input row, p a token's position in its sequence (from 0), W x a stored [out, in]
matrix applied to a column.  Every recurrence starts from a zero state.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch


_ROUND = [None]   # a dtype to which every projection's result is rounded (see `forward`), or None


def proj(h: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """W h for every row of h; h and the result pass through the rounding that `forward` was asked for."""
    if _ROUND[0] is None:
        return h @ w.T
    return (h.to(_ROUND[0]).to(h.dtype) @ w.T).to(_ROUND[0]).to(h.dtype)


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(x):
    return x / (1.0 + torch.exp(-x))


def softplus(x):
    return torch.where(x > 30.0, x, torch.log1p(torch.exp(torch.clamp(x, max=30.0))))


def rotate_half(x: torch.Tensor, p: int, dims: int, base: float) -> torch.Tensor:
    """x [heads, dim]: the first `dims` entries of each head turn, entry i paired with entry i + dims/2, by the
    angle p * base^(-2i/dims); the rest pass."""
    if dims == 0:
        return x
    half = dims // 2
    i = torch.arange(half, dtype=x.dtype)
    ang = p * torch.pow(torch.tensor(base, dtype=x.dtype), -2.0 * i / dims)
    c, s = torch.cos(ang), torch.sin(ang)
    u, v = x[:, :half], x[:, half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[:, dims:]], dim=-1)


def decayed_outer_scan(q, k, v, decay):
    """q, k [T, heads, dk], v [T, heads, dv], decay [T, heads] (or [heads]): S_t = decay_t S_(t-1) + k_t v_t^T,
    o_t = S_t^T q_t.  Returns o [T, heads, dv]."""
    T, H, dk = q.shape
    dv = v.shape[-1]
    S = torch.zeros((H, dk, dv), dtype=q.dtype)
    out = torch.empty((T, H, dv), dtype=q.dtype)
    for t in range(T):
        a = decay if decay.dim() == 1 else decay[t]
        S = a[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hkv,hk->hv", S, q[t])
    return out


def retention(h, W: Dict[str, torch.Tensor], m: dict, eps: float):
    """h [T, width] -> [T, width].  Rotated q and k, k / sqrt(dim), a fixed decay a head, each head's output
    divided by its root mean square, gate silu(W_g h)."""
    T = h.shape[0]
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    q = proj(h, W["q"]).view(T, H, dk)
    k = proj(h, W["k"]).view(T, H, dk)
    v = proj(h, W["v"]).view(T, H, dv)
    rot = m.get("rot") or {"dims": 0, "base": 1.0}
    dims, base = int(rot.get("dims", 0) or 0), float(rot.get("base", 1.0))
    q = torch.stack([rotate_half(q[t], t, dims, base) for t in range(T)])
    k = torch.stack([rotate_half(k[t], t, dims, base) for t in range(T)]) * dk ** -0.5
    o = decayed_outer_scan(q, k, v, torch.tensor(m["decay"], dtype=h.dtype))
    o = rms_unit(o, eps).reshape(T, H * dv) * silu(proj(h, W["g"]))
    return proj(o, W["o"])


def lightning(h, W, m, eps):
    """silu on q, k and v, the same recurrence, one norm over all heads with a weight, gate sigmoid(W_g h)."""
    T = h.shape[0]
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    q = silu(proj(h, W["q"])).view(T, H, dk)
    k = silu(proj(h, W["k"])).view(T, H, dk)
    v = silu(proj(h, W["v"])).view(T, H, dv)
    o = decayed_outer_scan(q, k, v, torch.tensor(m["decay"], dtype=h.dtype)).reshape(T, H * dv)
    o = rms_unit(o, eps) * W["norm"] * torch.sigmoid(proj(h, W["g"]))
    return proj(o, W["o"])


def capped_attention(h, W, m, eps):
    """Softmax attention without rotation: q and k of unit root mean square a head, q times a temperature that
    grows with the logarithm of the position, scores capped by a tanh, every earlier key visible."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms_unit(proj(h, W["q"]).view(T, H, dk), eps)
    k = rms_unit(proj(h, W["k"]).view(T, G, dk), eps)
    v = proj(h, W["v"]).view(T, G, dv)
    qt = m.get("q_temp")
    if qt:
        p = torch.arange(T, dtype=h.dtype)
        q = q * (1.0 + qt["coef"] * torch.log(torch.floor((p + 1) / qt["every"]) + 1.0))[:, None, None]
    out = torch.empty((T, H, dv), dtype=h.dtype)
    cap = float(m.get("softcap") or 0.0)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * m["scale"]
        if cap > 0:
            s = cap * torch.tanh(s / cap)
        s = s.masked_fill(torch.triu(torch.ones(T, T, dtype=torch.bool), 1), float("-inf"))
        out[:, hd] = torch.softmax(s, dim=-1) @ v[:, g]
    return proj(out.reshape(T, H * dv), W["o"])


def state_space(h, W, m, eps):
    """The selective state-space mixer: input cut into z | x | B | C | dt, a causal convolution with silu over
    x, B, C, dt = softplus(dt + bias), S_t = exp(-exp(A_log) dt) S_(t-1) + dt B_t x_t^T, y_t = S_t^T C_t + D x_t,
    y silu(z), a norm in equal parts with a weight."""
    T = h.shape[0]
    H, dv, N, G, taps = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
    inner = H * dv
    u = proj(h, W["in"])
    z, xbc, dt = u[:, :inner], u[:, inner:2 * inner + 2 * G * N], u[:, 2 * inner + 2 * G * N:]
    pad = torch.cat([torch.zeros((taps - 1, xbc.shape[1]), dtype=h.dtype), xbc])
    conv = torch.stack([(pad[t:t + taps] * W["conv"].T).sum(0) for t in range(T)]) + W["conv.b"]
    xbc = silu(conv)
    x = xbc[:, :inner].view(T, H, dv)
    B = xbc[:, inner:inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N:].view(T, G, N)
    dt = softplus(dt + W["dt_bias"])
    decay = torch.exp(-torch.exp(W["A_log"]) * dt)
    grp = torch.arange(H) // (H // G)
    y = decayed_outer_scan(C[:, grp], B[:, grp] * dt[:, :, None], x, decay) + W["D"][None, :, None] * x
    y = y.reshape(T, inner) * silu(z)
    parts = m["norm_groups"]
    y = rms_unit(y.view(T, parts, inner // parts), eps).reshape(T, inner) * W["norm"]
    return proj(y, W["o"])


def parallel(h, W, m, eps):
    left = capped_attention(h, {k[5:]: v for k, v in W.items() if k.startswith("left.")}, m["left"], eps)
    right = state_space(h, {k[6:]: v for k, v in W.items() if k.startswith("right.")}, m["right"], eps)
    return m["left_scale"] * left + m["right_scale"] * right


def squared_relu_mlp(h, W):
    return proj(torch.relu(proj(h, W["up"])) ** 2, W["down"])


MIXERS = {"retention": retention, "lightning": lightning, "parallel": parallel}


def forward(config: dict, weights: Dict[str, torch.Tensor], tokens: List[int], dtype=torch.float64,
            layers_out: Optional[list] = None, round_products=None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence.  `layers_out` receives the residual stream after every layer.
    `round_products` (a dtype): every projection's input and result inside the layers is rounded to it (the operands and
    the result of a 16-bit matrix product), everything else stays in `dtype`: the error that a 16-bit engine cannot
    avoid, by which the tests measure the engine's own."""
    _ROUND[0] = round_products
    try:
        return _forward(config, weights, tokens, dtype, layers_out)
    finally:
        _ROUND[0] = None


def _forward(config, weights, tokens, dtype, layers_out):
    W = {k: v.to(dtype) for k, v in weights.items()}
    eps = float(config["norm"]["eps"])
    x = W["embed"][torch.tensor(tokens, dtype=torch.long)] * float(config["embedding"]["scale"])
    for i, layer in enumerate(config["layers"]):
        pre = f"l{i}."
        sub = lambda s: {k[len(pre) + len(s) + 1:]: v for k, v in W.items() if k.startswith(pre + s + ".")}
        y = MIXERS[layer["type"]](rms_unit(x, eps) * W[pre + "norm1"], sub("mix"), layer["mixer"], eps)
        x = x + rms_unit(y, eps) * W[pre + "norm1b"]
        if layer.get("mlp") is not None:
            y = squared_relu_mlp(rms_unit(x, eps) * W[pre + "norm2"], sub("mlp"))
            x = x + rms_unit(y, eps) * W[pre + "norm2b"]
        if layers_out is not None:
            layers_out.append(x.clone())
    return (rms_unit(x, eps) * W["final.norm"]) @ W["embed"].T


# ---- configurations and weights for the tests ---------------------------------------------------------------------------
def tensor_shapes(config: dict) -> Dict[str, tuple]:
    """Every tensor of a model of this configuration, by name, with its shape (matrices are [out, in])."""
    W = config["width"]
    out = {"embed": (config["vocab"], W), "final.norm": (W,)}
    for i, layer in enumerate(config["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = out[p + "norm1b"] = (W,)
        if layer["type"] in ("retention", "lightning"):
            H, dk, dv = m["heads"], m["dim"], m["vdim"]
            out.update({p + "mix.q": (H * dk, W), p + "mix.k": (H * dk, W), p + "mix.v": (H * dv, W), p + "mix.g": (H * dv, W),
                        p + "mix.o": (W, H * dv)})
            if layer["type"] == "lightning":
                out[p + "mix.norm"] = (H * dv,)
        else:
            l, r = m["left"], m["right"]
            out.update({p + "mix.left.q": (l["heads"] * l["dim"], W), p + "mix.left.k": (l["kv_heads"] * l["dim"], W),
                        p + "mix.left.v": (l["kv_heads"] * l["vdim"], W), p + "mix.left.o": (W, l["heads"] * l["vdim"])})
            inner, gn = r["heads"] * r["vdim"], r["groups"] * r["state"]
            out.update({p + "mix.right.in": (2 * inner + 2 * gn + r["heads"], W), p + "mix.right.conv": (inner + 2 * gn, r["conv"]),
                        p + "mix.right.conv.b": (inner + 2 * gn,), p + "mix.right.dt_bias": (r["heads"],),
                        p + "mix.right.A_log": (r["heads"],), p + "mix.right.D": (r["heads"],),
                        p + "mix.right.norm": (inner,), p + "mix.right.o": (W, inner)})
        if layer.get("mlp") is not None:
            out[p + "norm2"] = out[p + "norm2b"] = (W,)
            out[p + "mlp.up"] = (layer["mlp"]["ff"], W)
            out[p + "mlp.down"] = (W, layer["mlp"]["ff"])
    return out


def random_weights(config: dict, seed: int) -> Dict[str, torch.Tensor]:
    """float32 weights whose values are exact in bfloat16, sized so that every branch matters: matrices N(0, 1/in),
    norm weights near 1, slow and fast state-space decays, convolution taps of order one."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in sorted(tensor_shapes(config).items()):
        r = torch.randn(shape, generator=g)
        if name == "embed":
            t = r
        elif name.endswith("A_log"):
            t = -3.0 * torch.rand(shape, generator=g) - 0.5          # decays between exp(-0.6 dt) and exp(-0.03 dt)
        elif name.endswith("dt_bias"):
            t = r
        elif name.endswith(".D"):
            t = 1.0 + 0.3 * r
        elif name.endswith("conv"):
            t = 0.6 * r
        elif name.endswith("conv.b"):
            t = 0.2 * r
        elif len(shape) == 1:
            t = 1.0 + 0.2 * r
        else:
            t = r * (1.5 / math.sqrt(shape[1]))
        out[name] = t.to(torch.bfloat16).to(torch.float32)
    return out


def _layer(kind, mixer, ff):
    return {"type": kind, "mixer": mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def _parallel(heads, kv, dim, vdim, scale, cap, qtemp, rh, rv, state, groups, conv, ngroups, ls, rs):
    left = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale, "softcap": cap}
    if qtemp:
        left["q_temp"] = {"coef": qtemp[0], "every": qtemp[1]}
    return {"left": left, "right": {"heads": rh, "vdim": rv, "state": state, "groups": groups, "conv": conv, "norm_groups": ngroups},
            "left_scale": ls, "right_scale": rs}


def config_a() -> dict:
    """Every layer type once; sizes that differ from each other everywhere; a layer without a feed-forward; sharp
    attention (a large score scale under the cap) so that a lost or misplaced key moves the logits."""
    return {"architecture": "Kekevik", "vocab": 97, "width": 64, "embedding": {"scale": 3.0}, "norm": {"eps": 1e-5}, "layers": [
        _layer("retention", {"heads": 2, "dim": 16, "vdim": 24, "decay": [0.9, 0.9990234375], "rot": {"dims": 8, "base": 100.0}}, 48),
        _layer("lightning", {"heads": 3, "dim": 8, "vdim": 16, "decay": [0.5, 0.96875, 0.99951171875]}, None),
        _layer("parallel", _parallel(4, 2, 16, 32, 2.0, 20.0, (0.3, 16), 4, 8, 16, 2, 3, 2, 0.7, 1.3), 80)]}


def config_b() -> dict:
    """The side-by-side layer first; no cap and no temperature; value heads smaller than the key heads; one key/value
    head; full rotation; convolutions of two and five taps; the last layer without a feed-forward."""
    return {"architecture": "Kekevik", "vocab": 61, "width": 128, "embedding": {"scale": 0.5}, "norm": {"eps": 1e-6}, "layers": [
        _layer("parallel", _parallel(4, 4, 24, 8, 0.75, 0.0, None, 4, 16, 8, 1, 2, 1, 1.0, 0.25), 96),
        _layer("retention", {"heads": 1, "dim": 32, "vdim": 32, "decay": [0.984375], "rot": {"dims": 32, "base": 10000.0}}, 64),
        _layer("parallel", _parallel(6, 1, 24, 24, 0.5, 8.0, (0.4, 5), 6, 8, 12, 3, 5, 3, 1.2, 0.9), 40),
        _layer("lightning", {"heads": 4, "dim": 16, "vdim": 8, "decay": [0.75, 0.9, 0.96875, 0.998046875]}, None)]}


def config_c() -> dict:
    """Sizes that the matrix-core kernels take (heads of 64 and 128, widths in multiples of 64)."""
    return {"architecture": "Kekevik", "vocab": 320, "width": 192, "embedding": {"scale": 8.0}, "norm": {"eps": 1e-6}, "layers": [
        _layer("lightning", {"heads": 2, "dim": 128, "vdim": 64, "decay": [0.9375, 0.9990234375]}, 384),
        _layer("parallel", _parallel(8, 2, 64, 64, 0.5, 30.0, (0.2, 32), 4, 32, 64, 1, 4, 1, 0.8, 0.9), 384),
        _layer("retention", {"heads": 2, "dim": 64, "vdim": 128, "decay": [0.96875, 0.99951171875], "rot": {"dims": 32, "base": 1e6}}, 256),
        _layer("parallel", _parallel(4, 4, 128, 128, 0.25, 50.0, None, 2, 64, 128, 2, 4, 4, 1.0, 1.0), None)]}


CONFIGS = {"A": config_a, "B": config_b, "C": config_c}


def greedy(config: dict, weights, prompt: List[int], n: int) -> List[int]:
    """n tokens, each the first largest logit after the whole sequence so far."""
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(torch.argmax(forward(config, weights, toks)[-1])))
    return toks[len(prompt):]
