"""Kekevik without a GPU: config.json's keys and their checks, the model's description and tensor names against the
plain implementation's own list, cache entries that need several things at once, and the plain implementation's
own consistency (a prefix's logits do not depend on what follows; a rounding-free rotation keeps lengths)."""
import copy

import pytest
import torch

import plain_kekevik as K
from infinilm_amd.cache import CacheManager
from infinilm_amd.cache.needs import FixedState, PagedKV
from infinilm_amd.config import ConfigError, load_model_config
from infinilm_amd.engine.model import CausalLM


@pytest.mark.parametrize("name", sorted(K.CONFIGS))
def test_description_names_every_tensor(name):
    cfg = K.CONFIGS[name]()
    arch, typed = load_model_config(cfg)
    assert arch.name == "Kekevik"
    model = CausalLM(arch.build_spec(typed), torch.float32, "meta")
    assert {k: tuple(p.shape) for k, p in model.named_parameters().items()} == K.tensor_shapes(cfg)
    assert model.head_is_tied and model.head is model.embed
    assert len(model.cache_needs) == len(cfg["layers"])
    for need, layer in zip(model.cache_needs, cfg["layers"]):
        if layer["type"] == "parallel":
            kinds = [type(n) for n in need]
            assert kinds == [PagedKV, FixedState, FixedState]
            r = layer["mixer"]["right"]
            assert need[1].shape == (r["conv"] - 1, r["heads"] * r["vdim"] + 2 * r["groups"] * r["state"])
            assert need[2].shape == (r["heads"], r["vdim"], r["state"])
        else:
            m = layer["mixer"]
            assert need == FixedState((m["heads"], m["vdim"], m["dim"]), torch.float32)


def test_heads_of_unequal_sizes_are_filled_up_in_the_weights():
    """Query/key heads of 16 and value heads of 32 run as heads of 32: the checkpoint's tensors land in the first rows of
    every head (columns for the output projection), the rest are zeros."""
    cfg = K.config_a()
    arch, typed = load_model_config(cfg)
    model = CausalLM(arch.build_spec(typed), torch.float32, "cpu")
    W = K.random_weights(cfg, 1)
    from infinilm_amd.weights.loader import load_state_dict
    load_state_dict(model, W)
    att = model.blocks[2].mixer.branches[0]
    assert (att.d, att.dn, att.dv) == (32, 16, 32)
    w = att.qkv.weight.view(4 + 2 + 2, 32, 64)
    assert torch.equal(w[:4, :16].reshape(64, 64), W["l2.mix.left.q"]) and float(w[:6, 16:].abs().max()) == 0.0
    assert torch.equal(w[6:].reshape(64, 64), W["l2.mix.left.v"])
    assert torch.equal(att.o_proj.weight, W["l2.mix.left.o"])
    # value heads smaller than the key heads: columns of the output projection are filled up
    cfg = K.config_b()
    arch, typed = load_model_config(cfg)
    model = CausalLM(arch.build_spec(typed), torch.float32, "cpu")
    W = K.random_weights(cfg, 1)
    load_state_dict(model, W)
    att = model.blocks[0].mixer.branches[0]
    assert (att.d, att.dn, att.dv) == (32, 24, 8)
    o = att.o_proj.weight.view(128, 4, 32)
    assert torch.equal(o[:, :, :8].reshape(128, 32), W["l0.mix.left.o"]) and float(o[:, :, 8:].abs().max()) == 0.0


@pytest.mark.parametrize("change,message", [
    (lambda c: c.pop("vocab"), "vocab"),
    (lambda c: c["layers"][0].update(type="window"), "unknown layer type"),
    (lambda c: c["layers"][0]["mixer"].update(decay=[0.5]), "decay"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7), "rot.dims"),
    (lambda c: c["layers"][2]["mixer"]["left"].update(kv_heads=3), "kv_heads"),
    (lambda c: c["layers"][2]["mixer"]["right"].update(groups=3), "groups"),
    (lambda c: c["layers"][2]["mixer"]["right"].pop("conv"), "conv"),
    (lambda c: c["layers"][2]["mlp"].update(kind="routed"), "unknown kind"),
    (lambda c: c["norm"].pop("eps"), "eps"),
])
def test_config_errors_name_the_key(change, message):
    cfg = copy.deepcopy(K.config_a())
    change(cfg)
    with pytest.raises(ConfigError, match=message):
        load_model_config(cfg)


def test_cache_entries_that_need_several_things():
    needs = [FixedState((2, 3)), (PagedKV(2, 16), FixedState((1, 4)), FixedState((2, 2, 2))), PagedKV(1, 8, window=32)]
    cache = CacheManager(needs, page_size=16, num_pages=6, max_requests=3, dtype=torch.float32, device="cpu")
    assert set(cache.state) == {0, (1, 1), (1, 2)} and set(cache.k) == {(1, 0), 2}
    assert len(cache.groups) == 2 and cache.bytes_per_token() == 2 * (2 * 16 + 8) * 4
    assert not cache.prefix_caching

    class B:   # what a view reads of a step's batch
        block_tables, slots = ["bt0", "bt1"], ["s0", "s1"]
        state_in, state_out = "in", "out"
    v = cache.view(1, B, True)
    assert v[0].k is cache.k[(1, 0)] and v[0].block_tables == "bt0" and v[1].pool is cache.state[(1, 1)] and v[2].pool is cache.state[(1, 2)]
    assert cache.view(2, B, False).slots is None and cache.view(0, B, True).state_in == "in"
    cache.admit("a")
    cache.reserve("a", 40)
    cache.commit("a", 40)
    assert [len(t) for t in cache.requests["a"].tables] == [3, 3]
    cache.release("a")
    cache.check()


def test_plain_prefix_does_not_depend_on_what_follows():
    cfg = K.config_a()
    W = K.random_weights(cfg, 3)
    toks = list(range(1, 60))
    whole = K.forward(cfg, W, toks)
    assert torch.allclose(K.forward(cfg, W, toks[:23]), whole[:23], atol=1e-9)


def test_plain_rotation_keeps_lengths_and_leaves_the_rest():
    x = torch.randn(3, 12, dtype=torch.float64)
    y = K.rotate_half(x, 17, 8, 100.0)
    assert torch.allclose(y[:, 8:], x[:, 8:]) and torch.allclose((y[:, :8] ** 2).sum(-1), (x[:, :8] ** 2).sum(-1))
    assert torch.allclose(K.rotate_half(x, 0, 8, 100.0), x)
