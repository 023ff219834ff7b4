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
    q = (h @ W["q"].T).view(T, H, dk)
    k = (h @ W["k"].T).view(T, H, dk)
    v = (h @ W["v"].T).view(T, H, dv)
    rot = m.get("rot") or {"dims": 0, "base": 1.0}
    q = torch.stack([rotate_half(q[t], t, rot["dims"], rot["base"]) for t in range(T)])
    k = torch.stack([rotate_half(k[t], t, rot["dims"], rot["base"]) for t in range(T)]) * dk ** -0.5
    o = decayed_outer_scan(q, k, v, torch.tensor(m["decay"], dtype=h.dtype))
    o = rms_unit(o, eps).reshape(T, H * dv) * silu(h @ W["g"].T)
    return o @ W["o"].T


def lightning(h, W, m, eps):
    """silu on q, k and v, the same recurrence, one norm over all heads with a weight, gate sigmoid(W_g h)."""
    T = h.shape[0]
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ W["q"].T).view(T, H, dk)
    k = silu(h @ W["k"].T).view(T, H, dk)
    v = silu(h @ W["v"].T).view(T, H, dv)
    o = decayed_outer_scan(q, k, v, torch.tensor(m["decay"], dtype=h.dtype)).reshape(T, H * dv)
    o = rms_unit(o, eps) * W["norm"] * torch.sigmoid(h @ W["g"].T)
    return o @ W["o"].T


def capped_attention(h, W, m, eps):
    """Softmax attention without rotation: q and k of unit root mean square a head, q times a temperature that
    grows with the logarithm of the position, scores capped by a tanh, every earlier key visible."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms_unit((h @ W["q"].T).view(T, H, dk), eps)
    k = rms_unit((h @ W["k"].T).view(T, G, dk), eps)
    v = (h @ W["v"].T).view(T, G, dv)
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
    return out.reshape(T, H * dv) @ W["o"].T


def state_space(h, W, m, eps):
    """The selective state-space mixer: input cut into z | x | B | C | dt, a causal convolution with silu over
    x, B, C, dt = softplus(dt + bias), S_t = exp(-exp(A_log) dt) S_(t-1) + dt B_t x_t^T, y_t = S_t^T C_t + D x_t,
    y silu(z), a norm in equal parts with a weight."""
    T = h.shape[0]
    H, dv, N, G, taps = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
    inner = H * dv
    u = h @ W["in"].T
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
    return y @ W["o"].T


def parallel(h, W, m, eps):
    left = capped_attention(h, {k[5:]: v for k, v in W.items() if k.startswith("left.")}, m["left"], eps)
    right = state_space(h, {k[6:]: v for k, v in W.items() if k.startswith("right.")}, m["right"], eps)
    return m["left_scale"] * left + m["right_scale"] * right


def squared_relu_mlp(h, W):
    return torch.relu(h @ W["up"].T) ** 2 @ W["down"].T


MIXERS = {"retention": retention, "lightning": lightning, "parallel": parallel}


def forward(config: dict, weights: Dict[str, torch.Tensor], tokens: List[int], dtype=torch.float64,
            layers_out: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence.  `layers_out` receives the residual stream after every layer."""
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
