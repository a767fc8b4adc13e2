"""The Beronex design without a GPU: its config.json reader, its plan over the library's parts, what its layers ask of the
cache, and the plain implementation's own mechanisms against closed forms."""
import copy
import math

import numpy as np
import pytest

import plain_beronex as plain
from beronex_cases import CASES, attention, config, dense, latent, lightning, moe, random_case, tensors, tokens, yarn
from turboquant_cpp_amd.config.base import ConfigError
from turboquant_cpp_amd.config.registry import config_from_dict
from turboquant_cpp_amd.engine.model import model_from_config
from turboquant_cpp_amd.parts.rope import YarnRotaryEncoding


@pytest.mark.parametrize("case", sorted(CASES))
def test_config_round_trip_and_tensor_table(case):
    cfg = CASES[case]
    arch, typed = config_from_dict(cfg)
    assert arch.name == "Beronex" and arch.config_to_json(typed) == cfg
    table = model_from_config(cfg, "float32").tensor_table()
    w = tensors(cfg, 0)
    assert set(table) == set(w)
    for name, (shape, _role) in table.items():
        assert tuple(shape) == w[name].shape, name


def test_random_cases_are_read():
    for seed in range(30):
        cfg = random_case(seed)
        arch, typed = config_from_dict(cfg)
        assert arch.config_to_json(typed) == cfg
        assert set(model_from_config(cfg, "bfloat16").tensor_table()) == set(tensors(cfg, seed))


def test_what_the_reader_refuses():
    good = CASES["odd"]
    def broken(change):
        cfg = copy.deepcopy(good)
        change(cfg)
        with pytest.raises(ConfigError):
            config_from_dict(cfg)
    broken(lambda c: c["layers"][0].update(type="delta"))
    broken(lambda c: c["layers"][0]["mixer"].update(decay=[0.5]))
    broken(lambda c: c["layers"][0]["mixer"].update(decay=[0.5, 0.5, 1.5]))
    broken(lambda c: c["layers"][3]["mixer"].update(kv_from=1))          # a latent layer keeps no keys
    broken(lambda c: c["layers"][3]["mixer"].update(kv_from=5))          # nor does a layer that reads another's, later
    broken(lambda c: c["layers"][3]["mixer"].update(dim=24))             # other sizes than the layer it reads
    broken(lambda c: c["layers"][2]["mixer"].update(kv_heads=4))
    broken(lambda c: c["layers"][2]["mixer"]["rot"].update(dims=13))
    broken(lambda c: c["layers"][1]["mixer"]["rot"].update(dims=6))      # the rotated part is rot_dim
    broken(lambda c: c["layers"][2]["mlp"]["router"].update(top=6))
    broken(lambda c: c["layers"][2]["mlp"]["expert"].update(limit=0.0))
    broken(lambda c: c["layers"][0]["mlp"].update(kind="glu"))
    broken(lambda c: c.pop("width"))
    broken(lambda c: c["norm"].pop("eps"))


def test_a_cache_keeps_what_its_widest_reader_sees():
    """Layer 2 of "odd" has a window of 70 and is read by layers with windows of 9 and of 100: its cache keeps 100."""
    needs = model_from_config(CASES["odd"], "float32").cache_needs()
    assert needs[2][0].window == 100 and needs[2][2] is None
    assert needs[3][0].window == 9 and needs[3][2] == 2 and needs[5][0].window == 100 and needs[5][2] == 2
    assert needs[6][0].window is None and needs[7][0].window == 33 and needs[7][2] == 6
    assert needs[0][0] is None and needs[0][1].shape == (3 * 20 * 12,)
    assert needs[1][0].num_kv_heads == 1 and needs[1][0].head_dim == 48            # 40 + 4, in sixteens
    cfg = config(32, 40, [(attention(2, 1, 8, 8, window=5), None), (attention(2, 1, 8, 8, kv_from=0), None)])
    assert model_from_config(cfg, "float32").cache_needs()[0][0].window is None   # a reader without a window


def test_stretched_frequencies():
    for dims, base, s in ((64, 50000.0, yarn(4.0, 512, 32.0, 1.0)), (16, 5e5, yarn(8.0, 2048, 32.0, 1.0)), (12, 500.0, yarn(2.0, 16, 4.0, 1.0)),
                          (24, 1e4, yarn(16.0, 40, 10.0, 0.5)), (2, 100.0, yarn(32.0, 4096, 8.0, 2.0))):
        part = YarnRotaryEncoding(dims, dims, base, s["factor"], s["original"], s["fast"], s["slow"], "interleaved")
        f, m = plain.rotation_table({"dims": dims, "base": base, "scaling": s})
        assert np.abs(part.frequencies() - f).max() <= 1e-7 * f.max() and abs(part.amplitude - m) < 1e-12
        plain_f, one = plain.rotation_table({"dims": dims, "base": base})
        assert one == 1.0 and np.all(f <= plain_f * (1 + 1e-12)) and np.all(f >= plain_f / s["factor"] * (1 - 1e-12))
        assert m == pytest.approx(0.1 * math.log(s["factor"]) + 1.0)


def test_the_plain_recurrence_is_the_sum_it_stands_for():
    """o_t = sum_{s <= t} decay^(t - s) (q_t . k_s) v_s, and a sequence cut in two with the state handed on is the whole."""
    cfg = CASES["lightning_only"]
    w = tensors(cfg, 1)
    m = cfg["layers"][0]["mixer"]
    rng = np.random.default_rng(0)
    h = rng.normal(size=(19, cfg["width"]))
    H, D, V = m["heads"], m["dim"], m["vdim"]
    q = plain.silu(h @ w["l0.mix.q"].T).reshape(-1, H, D)
    k = plain.silu(h @ w["l0.mix.k"].T).reshape(-1, H, D)
    v = plain.silu(h @ w["l0.mix.v"].T).reshape(-1, H, V)
    o = np.zeros((19, H, V))
    for t in range(19):
        for s in range(t + 1):
            for head in range(H):
                o[t, head] += m["decay"][head] ** (t - s) * (q[t, head] @ k[s, head]) * v[s, head]
    want = (plain.rms_norm(o.reshape(19, -1), w["l0.mix.norm"], 1e-5) * plain.sigmoid(h @ w["l0.mix.g"].T)) @ w["l0.mix.o"].T
    whole = plain.lightning(h, m, w, "l0.mix.", 1e-5)
    assert np.abs(whole - want).max() < 1e-10
    first, state = plain.lightning(h[:7], m, w, "l0.mix.", 1e-5, return_state=True)
    rest = plain.lightning(h[7:], m, w, "l0.mix.", 1e-5, state=state)
    assert np.abs(np.concatenate([first, rest]) - whole).max() < 1e-12


def test_windows_and_limits_of_the_plain_implementation():
    s = np.zeros((6, 6))
    p = plain.masked_softmax(s, 3)
    assert np.allclose(p[5], [0, 0, 0, 1 / 3, 1 / 3, 1 / 3]) and np.allclose(p[1], [0.5, 0.5, 0, 0, 0, 0]) and p[0, 0] == 1.0
    assert np.allclose(plain.masked_softmax(s, None)[5], 1 / 6) and np.allclose(np.diag(plain.masked_softmax(s, 1)), 1.0)
    w = {"gate": np.array([[5.0], [-5.0], [0.5]]), "up": np.array([[9.0], [-9.0], [0.25]]), "down": np.eye(3)}
    y = plain.expert(np.array([[1.0]]), {"e." + k: v for k, v in w.items()}, "e.", 2.0)[0]
    sw = lambda g: g / (1 + math.exp(-1.702 * g))
    assert np.allclose(y, [sw(2.0) * 3.0, sw(-5.0) * -1.0, sw(0.5) * 1.25])
    f = {"router": {"experts": 4, "top": 2}}
    ids, weights, z = plain.route(np.array([[1.0, 0.0]]), f, {"r.router": np.array([[1.0, 0], [3.0, 0], [2.0, 0], [0.0, 0]]),
                                                          "r.router.b": np.array([0.0, 0.0, 0.0, 3.5])}, "r.")
    assert ids.tolist() == [[3, 1]] and np.allclose(weights, [[1 / (1 + math.exp(-0.5)), 1 / (1 + math.exp(0.5))]])


def test_positions_shift_scores_only_through_their_difference():
    """Rotation of queries and keys: the score of two positions depends on their distance only, in both layouts."""
    rot = {"dims": 8, "base": 100.0, "scaling": yarn(4.0, 16, 4.0, 1.0)}
    rng = np.random.default_rng(3)
    x, y = rng.normal(size=(1, 1, 12)), rng.normal(size=(1, 1, 12))
    for layout in ("pairs", "halves"):
        a = (plain.rotate(x, np.array([5.0]), rot, layout) * plain.rotate(y, np.array([2.0]), rot, layout)).sum()
        b = (plain.rotate(x, np.array([105.0]), rot, layout) * plain.rotate(y, np.array([102.0]), rot, layout)).sum()
        assert abs(a - b) < 1e-9
        assert np.allclose(plain.rotate(x, np.array([7.0]), rot, layout)[..., 8:], x[..., 8:])
