"""Pugavik without a GPU: config.json's keys and their checks, the order of layer runs with what each run adds to the
stream, tensor names against the plain implementation's own list, the one size that only a checkpoint's tensor gives,
heads filled up in the weights, the cache entries of a looped model, and the plain implementation's own consistency (a
prefix's logits do not depend on what follows; a window's edge; the sink takes weight from every key)."""
import copy
import json
import os

import pytest
import torch

import plain_pugavik as P
from infinilm_amd.cache import CacheManager
from infinilm_amd.cache.needs import FixedState, PagedKV
from infinilm_amd.config import ConfigError, load_model_config
from infinilm_amd.config.spec import RunStart
from infinilm_amd.engine.model import CausalLM


@pytest.mark.parametrize("name", sorted(P.CONFIGS))
def test_description_names_every_tensor(name):
    cfg = P.CONFIGS[name]()
    arch, typed = load_model_config(cfg)
    assert arch.name == "Pugavik"
    spec = arch.build_spec(typed)
    model = CausalLM(spec, torch.float32, "meta")
    assert {k: tuple(p.shape) for k, p in model.named_parameters().items()} == P.tensor_shapes(cfg)
    assert not model.head_is_tied
    # the runs follow the plain implementation's order, each with a cache entry of its own
    want = P.run_order(cfg)
    assert [r.layer for r in spec.order] == [i for i, _ in want]
    assert [r.cache for r in spec.order] == list(range(len(want)))
    for run, (_, opens) in zip(spec.order, want):
        assert run.start == (None if opens is None else RunStart(embedding=1.0 if opens > 0 else 0.0, vector_row=opens))
    for run, need in zip(spec.order, model.cache_needs):
        layer = cfg["layers"][run.layer]
        m = layer["mixer"]
        if layer["type"] == "gla":
            assert need == FixedState((m["heads"], m["vdim"], m["dim"]), torch.float32)
        elif layer["type"] == "attention":
            d = m["dim"] if m["dim"] == m["vdim"] else -(-max(m["dim"], m["vdim"]) // 16) * 16
            assert need == PagedKV(m["kv_heads"], d, m["mask"]["size"])
        else:
            n = m["kv_rank"] + m["rot_dim"]
            assert need == PagedKV(1, -(-n // 32) * 32 if n <= 128 else -(-n // 16) * 16, 0)


def test_a_looped_model_keeps_a_cache_for_every_pass():
    cfg = P.config_b()
    arch, typed = load_model_config(cfg)
    model = CausalLM(arch.build_spec(typed), torch.float32, "meta")
    cache = CacheManager(model.cache_needs, page_size=8, num_pages=6, max_requests=2, dtype=torch.float32, device="meta")
    assert len(model.cache_needs) == 1 + 3 * 2 + 1
    assert sorted(g.window for g in cache.groups) == [0, 5, 33]
    assert len(cache.state) == 3 and len(cache.k) == 5
    cache.admit("a")
    cache.reserve("a", 40)
    cache.commit("a", 40)
    by_window = {g.window: t for g, t in zip(cache.groups, cache.requests["a"].tables)}
    assert [p >= 0 for p in by_window[0]] == [True] * 5
    assert [p >= 0 for p in by_window[5]] == [False] * 4 + [True]       # positions 36.. are all the next token sees
    assert [p >= 0 for p in by_window[33]] == [False] + [True] * 4      # positions 8.. (40 - 33 + 1 = 8)
    cache.release("a")
    cache.check()


def test_the_decay_rank_comes_from_the_checkpoint(tmp_path):
    from safetensors.torch import save_file
    cfg = P.config_a()
    W = P.random_weights(cfg, 2)
    bare = copy.deepcopy(cfg)
    bare["layers"][0]["mixer"].pop("decay_rank")
    with pytest.raises(ConfigError, match="decay_rank"):
        load_model_config(bare)
    with open(tmp_path / "config.json", "w") as fh:
        json.dump(bare, fh)
    save_file({k: v.contiguous() for k, v in W.items()}, str(tmp_path / "model.safetensors"))
    arch, typed = load_model_config(str(tmp_path))
    assert typed.layers[0].mixer["decay_rank"] == 4
    from infinilm_amd.weights.loader import checkpoint_shapes
    assert checkpoint_shapes(str(tmp_path)) == {k: tuple(v.shape) for k, v in W.items()}


def test_heads_of_unequal_sizes_are_filled_up_in_the_weights():
    from infinilm_amd.weights.loader import load_state_dict
    cfg = P.config_b()
    arch, typed = load_model_config(cfg)
    model = CausalLM(arch.build_spec(typed), torch.float32, "cpu")
    W = P.random_weights(cfg, 1)
    load_state_dict(model, W)
    att = model.blocks[1].mixer
    assert (att.nh, att.nkv, att.d, att.dn, att.dv, att.window) == (6, 3, 32, 12, 20, 33)
    w = att.qkv.weight.view(6 + 3 + 3, 32, 96)
    assert torch.equal(w[:6, :12].reshape(72, 96), W["l1.mix.q"]) and float(w[:9, 12:].abs().max()) == 0.0
    assert torch.equal(w[9:, :20].reshape(60, 96), W["l1.mix.v"]) and float(w[9:, 20:].abs().max()) == 0.0
    b = att.qkv.bias.view(12, 32)
    assert torch.equal(b[6:9, :12].reshape(36), W["l1.mix.k.b"]) and float(b[:9, 12:].abs().max()) == 0.0
    o = att.o_proj.weight.view(96, 6, 32)
    assert torch.equal(o[:, :, :20].reshape(96, 120), W["l1.mix.o"]) and float(o[:, :, 20:].abs().max()) == 0.0
    assert att.head_mix.dtype == torch.float32 and torch.equal(att.head_mix, W["l1.mix.talk"])
    assert torch.equal(att.sink, W["l1.mix.sink"]) and torch.equal(att.position.k_weight, W["l1.mix.k.norm"])
    assert torch.equal(model.run_vectors, W["loop.step"]) and model.run_vectors.shape == (3, 96)
    gla = model.blocks[2].mixer
    assert torch.equal(gla.a2.bias, W["l2.mix.a2.b"]) and torch.equal(gla._norm_weight(), W["l2.mix.norm"].repeat(3))


@pytest.mark.parametrize("change,message", [
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["layers"][0].update(type="retention"), "unknown layer type"),
    (lambda c: c["layers"][1]["mixer"].update(kv_heads=4), "kv_heads"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=13), "rot.dims"),
    (lambda c: c["layers"][1]["mixer"].pop("mask"), "size"),
    (lambda c: c["layers"][1]["mixer"].pop("scale"), "scale"),
    (lambda c: c["layers"][0]["mixer"].update(rot_dim=7), "rot_dim"),
    (lambda c: c["layers"][0]["mixer"].pop("kv_rank"), "kv_rank"),
    (lambda c: c["layers"][2]["mixer"].update(tau=0.0), "tau"),
    (lambda c: c["layers"][2]["mlp"].update(kind="routed"), "unknown kind"),
    (lambda c: c["loop"].update(stop=9), "stretch"),
    (lambda c: c["loop"].pop("times"), "times"),
    (lambda c: c["norm"].pop("eps"), "eps"),
    (lambda c: c["embedding"].pop("scale"), "scale"),
])
def test_config_errors_name_the_key(change, message):
    cfg = copy.deepcopy(P.config_b())
    change(cfg)
    with pytest.raises(ConfigError, match=message):
        load_model_config(cfg)


def test_random_weights_writer_knows_the_design(tmp_path):
    from infinilm_amd.weights.random_init import write_random_model
    cfg = P.config_a()
    write_random_model(cfg, 3, str(tmp_path), dtype="bfloat16")
    from infinilm_amd.weights.loader import checkpoint_shapes
    assert checkpoint_shapes(str(tmp_path)) == P.tensor_shapes(cfg)
    assert os.path.isfile(tmp_path / "config.json")


# ---- the plain implementation's own consistency -----------------------------------------------------------------------------
@pytest.mark.parametrize("name", sorted(P.CONFIGS))
def test_plain_prefix_logits_do_not_depend_on_what_follows(name):
    cfg = P.CONFIGS[name]()
    W = P.random_weights(cfg, 5)
    g = torch.Generator().manual_seed(1)
    toks = torch.randint(0, cfg["vocab"], (50,), generator=g).tolist()
    whole = P.forward(cfg, W, toks)
    for n in (1, 2, 9, 33):
        assert torch.allclose(P.forward(cfg, W, toks[:n]), whole[:n], atol=1e-9)


def test_plain_window_edge_and_sink():
    m = P._attention(2, 1, 8, 8, 4, 0)
    cfg = {"architecture": "Pugavik", "vocab": 20, "width": 16, "embedding": {"scale": 1.0}, "norm": {"eps": 1e-6},
           "layers": [P._layer("attention", m, None)]}
    W = P.random_weights(cfg, 1)
    toks = [3, 4, 5, 6, 7, 8, 9]
    base = P.forward(cfg, W, toks)[-1]
    inside = P.forward(cfg, W, toks[:3] + [11] + toks[4:])[-1]      # position 3 = 6 - 4 + 1: the window's last place
    outside = P.forward(cfg, W, toks[:2] + [11] + toks[3:])[-1]     # position 2: one too far
    assert not torch.allclose(inside, base, atol=1e-6) and torch.allclose(outside, base, atol=1e-12)
    # a very large sink takes all the weight: the mixer adds nothing, whatever the tokens before
    W2 = dict(W, **{"l0.mix.sink": torch.full((2,), 80.0)})
    a = P.forward(cfg, W2, toks)[-1]
    b = P.forward(cfg, W2, [1, 2, 1, 2, 1, 2, 9])[-1]
    assert torch.allclose(a, b, atol=1e-9)


def test_plain_rotation_keeps_lengths_and_relative_angles():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(6, 3, 10, generator=g, dtype=torch.float64)
    pos = torch.arange(6) + 100
    y = P.rotate_pairs(x, pos, 6, 1000.0)
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1)) and torch.equal(y[..., 6:], x[..., 6:])
    q = torch.randn(1, 1, 6, generator=g, dtype=torch.float64)
    k = torch.randn(1, 1, 6, generator=g, dtype=torch.float64)
    dots = [float((P.rotate_pairs(q, torch.tensor([p + 5]), 6, 1000.0) * P.rotate_pairs(k, torch.tensor([p]), 6, 1000.0)).sum()) for p in (0, 17, 400)]
    assert abs(dots[0] - dots[1]) < 1e-9 and abs(dots[0] - dots[2]) < 1e-9
