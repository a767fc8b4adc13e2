"""The Bosalix design without a GPU: its config.json reader and plan, the cache's books where first positions are kept
beside a window, the stretched rotation's table, and the plain implementation's own consistency."""
import copy

import numpy as np
import pytest

import plain_bosalix as plain
from bosalix_cases import CASES, as_float64, attention, config, latent, moe, random_case, random_weights, stretch, tensor_shapes, tokens
from turboquant_cpp_amd.cache.paged import PagedCache
from turboquant_cpp_amd.config.base import ConfigError
from turboquant_cpp_amd.config.registry import config_from_dict
from turboquant_cpp_amd.engine.model import model_from_config
from turboquant_cpp_amd.parts.base import CacheNeed, StateNeed
from turboquant_cpp_amd.parts.rope import Llama3RotaryEncoding, RotaryEncoding


@pytest.mark.parametrize("case", sorted(CASES))
def test_plan_reads_the_tensors_the_design_names(case):
    cfg = CASES[case]
    model = model_from_config(cfg, "float32")
    table = {n: tuple(s) for n, (s, _r) in model.tensor_table().items()}
    assert table == {n: tuple(s) for n, s in tensor_shapes(cfg).items()}
    arch, typed = config_from_dict(cfg)
    again = arch.config_from_json(arch.config_to_json(typed))
    assert again == typed
    needs = model.cache_needs()
    assert all(isinstance(s, StateNeed) and s.shape == (cfg["width"],) for _c, s, _o in needs)
    for (c, _s, _o), layer in zip(needs, cfg["layers"]):
        mask = layer["mixer"].get("mask") or {}
        assert c.window == mask.get("size")
        assert c.keep_first == (mask.get("keep_first", 0) if mask.get("size") else 0)


def test_random_cases_are_valid():
    for seed in range(30):
        model_from_config(random_case(seed), "float32")


def test_what_the_reader_refuses():
    good = CASES["mixed_values"]

    def broken(change):
        c = copy.deepcopy(good)
        change(c)
        return c

    for change in (lambda c: c["layers"][0].update(type="lightning"),
                   lambda c: c["layers"][0]["mlp"].update(kind="dense"),
                   lambda c: c["layers"][0]["mixer"].update(kv_heads=3),
                   lambda c: c["layers"][1]["mixer"]["rot"].update(dims=6),
                   lambda c: c["layers"][1]["mixer"].update(mask={"size": 4, "keep_first": 2}),
                   lambda c: c["layers"][2]["mixer"].update(vdim=16),
                   lambda c: c["layers"][0]["mlp"]["router"].update(top=6),
                   lambda c: c["layers"][2]["mixer"]["rot"]["scaling"].update(high=1.0),
                   lambda c: c["layers"][1]["mixer"]["rot"].update(scaling=stretch()),
                   lambda c: c.pop("norm")):
        with pytest.raises(ConfigError):
            config_from_dict(broken(change))
    # what may be absent
    c = broken(lambda c: (c.pop("residual_mult"), c.pop("embedding"), c["layers"][0]["mixer"].pop("mask")))
    _arch, typed = config_from_dict(c)
    assert typed.residual_mult == 1.0 and typed.embedding_scale == 1.0 and typed.layers[0].mixer.window is None


def test_stretched_table():
    for rot in ({"dims": 32, "base": 20000.0, "scaling": stretch(8.0, 1024, 1.0, 4.0)}, {"dims": 8, "base": 50.0, "scaling": stretch(2.0, 16, 1.0, 2.0)},
                {"dims": 16, "base": 10000.0, "scaling": stretch(4.0, 64)}):
        s = rot["scaling"]
        part = Llama3RotaryEncoding(64, rot["dims"], rot["base"], s["factor"], s["original"], s["low"], s["high"])
        want = plain.frequencies(rot)
        assert np.allclose(part.frequencies(), want, rtol=1e-6, atol=0)
        plain_f = plain.frequencies({"dims": rot["dims"], "base": rot["base"]})
        assert (want <= plain_f + 1e-15).all() and (want[-1] < plain_f[-1] or rot["dims"] <= 8)
    assert np.allclose(RotaryEncoding(8, 8, 100.0, double_table=True).frequencies(), plain.frequencies({"dims": 8, "base": 100.0}), rtol=1e-7)


def test_cache_keeps_the_first_positions_beside_the_window():
    needs = [(CacheNeed(1, 16, window=100, keep_first=70), StateNeed((8,)), None), (CacheNeed(2, 16, window=None), None, None)]
    cache = PagedCache(needs, max_tokens=64 * 40, dtype=None, device=None, page_size=64, max_slots=2, window_step=128)
    windowed = next(g for g in cache.groups if g.key.window == 100)
    assert windowed.kept_pages == 2 and windowed.pool.n_pages == 2 * (4 + 2 + 2)
    slot = cache.open()
    for n in (130, 1, 1, 120, 128, 1):
        cache.reserve(slot, n)
        cache.commit(slot)
    length = cache.length(slot)
    row = windowed.host_table[slot]
    held = [p for p in range(len(row)) if row[p] >= 0]
    assert held == [0, 1] + list(range((length - 100 + 1) // 64, (length - 1) // 64 + 1))
    assert windowed.needed_pages(length) == held
    other = next(g for g in cache.groups if g.key.window is None)
    assert (other.host_table[slot][:(length - 1) // 64 + 1] >= 0).all()
    cache.close(slot)
    assert all(v == 0 for v in cache.pages_held().values())


def test_plain_implementation_is_causal_and_windows_cut_where_they_should():
    cfg = CASES["mixed_values"]
    w = as_float64(random_weights(cfg, 3))
    toks = tokens(cfg, 90, 1)
    whole = plain.forward(cfg, w, toks)
    assert np.allclose(plain.forward(cfg, w, toks[:50]), whole[:50], atol=1e-10)
    see = plain.visible(8, 3, 2)
    assert see[7].tolist() == [True, True, False, False, False, True, True, True]
    assert plain.visible(4, None).tolist() == np.tril(np.ones((4, 4), dtype=bool)).tolist()
    h = np.arange(12.0).reshape(4, 3)
    assert np.allclose(plain.token_shift(h, np.array([0.0, 1.0, 0.5])), [[0, 0, 1], [3, 1, 3.5], [6, 4, 6.5], [9, 7, 9.5]])
    # an identity expert gives the token back, times its weight
    f = {"router": {"experts": 1, "identity": 2, "top": 3}, "expert": {"ff": 4}}
    rng = np.random.default_rng(0)
    ww = {"x.router": rng.standard_normal((3, 5)), "x.correction": np.zeros(3), "x.e0.up": np.zeros((4, 5)), "x.e0.down": np.zeros((5, 4))}
    hh = rng.standard_normal((2, 5))
    z = hh @ ww["x.router"].T
    s = np.exp(z) / np.exp(z).sum(1, keepdims=True)
    assert np.allclose(plain.experts(hh, f, ww, "x."), hh * s[:, 1:].sum(1, keepdims=True))
