"""config.json contents of the model shapes the benchmarks run with random weights: the MiniCPM4-8B,
MiniCPM4-0.5B and MiniCPM-2B-family layer sizes.  LongRoPE factors are drawn from a fixed seed
(uniform in [1, 4]); nothing else is random."""
from __future__ import annotations


def _factors(n: int, seed: int):
    import torch
    g = torch.Generator().manual_seed(seed)
    short = (1.0 + 3.0 * torch.rand(n, generator=g)).tolist()
    long = (1.0 + 3.0 * torch.rand(n, generator=g)).tolist()
    return short, long


def shape_config(name: str, layers: int = 0) -> dict:
    """`name`: "8b", "0.5b", "2b" (MiniCPM4 family) or "kekevik-<width>" (the Kekevik design at that width, 8 layers unless
    told otherwise); `layers` > 0 overrides the number of layers."""
    if name.startswith("kekevik-"):
        width = int(name.split("-")[1])
        return kekevik_shape(width, width // 128, 128, 2, layers or 8, 32768, 6 * width)
    base = {"architectures": ["MiniCPMForCausalLM"], "model_type": "minicpm", "torch_dtype": "bfloat16", "rope_theta": 10000.0,
            "scale_emb": 12, "scale_depth": 1.4, "dim_model_base": 256}
    if name == "8b":
        short, long = _factors(64, 1234)
        cfg = dict(base, num_hidden_layers=32, hidden_size=4096, num_attention_heads=32, num_key_value_heads=2, head_dim=128,
                   intermediate_size=16384, vocab_size=73448, max_position_embeddings=32768, rms_norm_eps=1e-6,
                   tie_word_embeddings=False,
                   rope_scaling={"type": "longrope", "short_factor": short, "long_factor": long,
                                 "original_max_position_embeddings": 32768})
    elif name == "0.5b":
        short, long = _factors(32, 1235)
        cfg = dict(base, num_hidden_layers=24, hidden_size=1024, num_attention_heads=16, num_key_value_heads=2, head_dim=64,
                   intermediate_size=4096, vocab_size=73448, max_position_embeddings=32768, rms_norm_eps=1e-6,
                   tie_word_embeddings=True,
                   rope_scaling={"type": "longrope", "short_factor": short, "long_factor": long,
                                 "original_max_position_embeddings": 32768})
    elif name == "2b":
        cfg = dict(base, num_hidden_layers=40, hidden_size=2304, num_attention_heads=36, num_key_value_heads=36, head_dim=64,
                   intermediate_size=5760, vocab_size=122753, max_position_embeddings=4096, rms_norm_eps=1e-5,
                   tie_word_embeddings=True)
    else:
        raise KeyError(f"unknown shape {name!r}; there are 8b, 0.5b and 2b")
    if layers > 0:
        cfg["num_hidden_layers"] = int(layers)
    return cfg


def kekevik_shape(width: int, heads: int, head_dim: int, kv_heads: int, layers: int, vocab: int, ff: int) -> dict:
    """A Kekevik configuration with the layer sizes of a transformer of this width: the four layer kinds in turn
    (retention, lightning, two side-by-side layers), `heads` heads of `head_dim` everywhere, a state space of
    heads * head_dim channels with 128 state entries a head, `ff` inner units of the feed-forward."""
    decay = [1.0 - 2.0 ** -(5 + (7 * h) // max(heads, 1)) for h in range(heads)]
    lin = {"heads": heads, "dim": head_dim, "vdim": head_dim, "decay": decay}
    par = {"left": {"heads": heads, "kv_heads": kv_heads, "dim": head_dim, "vdim": head_dim, "scale": head_dim ** -0.5,
                    "softcap": 50.0, "q_temp": {"coef": 0.1, "every": 1024}},
           "right": {"heads": heads, "vdim": head_dim, "state": 128, "groups": 1, "conv": 4, "norm_groups": 1},
           "left_scale": 1.0, "right_scale": 1.0}
    kinds = [("retention", dict(lin, rot={"dims": head_dim, "base": 10000.0})), ("lightning", lin), ("parallel", par), ("parallel", par)]
    return {"architecture": "Kekevik", "vocab": vocab, "width": width, "embedding": {"scale": 12.0}, "norm": {"eps": 1e-6},
            "layers": [{"type": kinds[i % 4][0], "mixer": kinds[i % 4][1], "mlp": {"kind": "dense", "ff": ff}} for i in range(layers)]}
