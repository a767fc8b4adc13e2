"""The Bosalix design in the engine against the plain implementation in ``plain_bosalix.py``: every mechanism alone, whole
prompts, the stream behind every layer, decoding through the cache and the state, prompts in portions down to two tokens,
unequal batches, slots and pages that are used again, keys far away, at the borders of pages, just inside and outside a
window and among the first positions that a window keeps in sight, the first tokens of a sequence, long decoding, sizes
of many kinds, the kernels one by one, greedy generation through the library's entry point, the command line, and the
trace runner as a program."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_bosalix as plain
from bosalix_cases import (CASES, as_float64, attention, config, latent, moe, random_case, random_weights, stretch, tokens,
                           write_model_dir)

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
F32_BOUND = 1e-4        # of the logits' root mean square, per position, mean taken off


@pytest.fixture(scope="module")
def made(tmp_path_factory):
    """(case, seed) -> (folder, config, float64 weights), each written once."""
    cache = {}

    def get(case: str, seed: int = 0):
        if (case, seed) not in cache:
            cfg = CASES[case]
            w = random_weights(cfg, seed, torch.bfloat16)
            cache[(case, seed)] = (write_model_dir(str(tmp_path_factory.mktemp(f"bosalix_{case}")), cfg, w), cfg, as_float64(w))
        return cache[(case, seed)]
    return get


def folder_of(path, cfg, w64):
    return write_model_dir(str(path), cfg, {n: torch.from_numpy(np.asarray(a)).to(torch.bfloat16) for n, a in w64.items()})


def engine_of(folder: str, dtype: str = "float32", max_tokens: int = 4096, **kw):
    from turboquant_cpp_amd.engine.model import load_model
    from turboquant_cpp_amd.engine.step import Engine
    return Engine(load_model(folder, act=dtype), max_tokens=max_tokens, page_size=64, **kw)


def errors(got, want: np.ndarray) -> np.ndarray:
    """Per position: root mean square of the difference with its mean taken off, over that of the wanted logits."""
    got = got.detach().double().cpu().numpy() if isinstance(got, torch.Tensor) else np.asarray(got, dtype=np.float64)
    d = got - want
    d = d - d.mean(axis=1, keepdims=True)
    scale = np.sqrt(np.mean((want - want.mean(axis=1, keepdims=True)) ** 2))
    return np.sqrt(np.mean(d * d, axis=1)) / scale


def check(got, want, dtype="float32", what=""):
    e = errors(got, want)
    if dtype == "float32":
        assert e.max() < F32_BOUND, f"{what}: position {int(e.argmax())} differs by {e.max():.2e}"
    elif dtype == "bfloat16":       # rounding of bfloat16 products and activations through all layers of a narrow model
        assert e.max() < 0.25 and np.quantile(e, 0.9) < 0.08 and np.median(e) < 0.04, \
            f"{what}: median {np.median(e):.3f}, 90 % {np.quantile(e, 0.9):.3f}, worst {e.max():.3f} at {int(e.argmax())}"
    else:       # "same path": the engine against itself on another schedule, in bfloat16
        # (a position in a hundred may stand out: where two choice scores of a router lie closer than the rounding of what
        # feeds them, another schedule's products may choose the other expert; the float32 runs of the same tests hold every
        # position to 1e-4)
        assert np.quantile(e, 0.9) < 0.03 and (e > 0.3).sum() <= max(1, len(e) // 100) and e.max() < 0.6, \
            f"{what}: 90 % {np.quantile(e, 0.9):.3f}, position {int(e.argmax())} differs by {e.max():.2e}"


def all_places(n):
    return list(range(n))


def wanted(eng, cfg, w, toks, dtype):
    """In float32 the plain implementation; in bfloat16 the engine's own logits for the whole sequence in one step, alone
    (which test_whole_prompt_bfloat16 holds against the plain implementation)."""
    if dtype == "float32":
        return plain.forward(cfg, w, toks), dtype
    slot = eng.open(1)
    out = eng.step(slot, [toks], [all_places(len(toks))]).double().cpu().numpy()
    eng.close(slot)
    return out, "same path"


def prompt_then_decode(eng, toks, cut):
    slot = eng.open(1)
    rows = [eng.step(slot, [toks[:cut]], [all_places(cut)])] + [eng.step(slot, [[t]]) for t in toks[cut:]]
    eng.close(slot)
    return torch.cat(rows)


# ---------------------------------------------------------------- whole prompts, every configuration
@pytest.mark.parametrize("case", sorted(CASES))
def test_whole_prompt(made, case):
    d, cfg, w = made(case)
    eng = engine_of(d)
    for seed, n in ((1, 1), (2, 150), (3, 67), (4, 2)):
        toks = tokens(cfg, n, seed)
        slot = eng.open(1)
        got = eng.step(slot, [toks], [all_places(n)])
        eng.close(slot)
        check(got, plain.forward(cfg, w, toks), what=f"{case}, {n} tokens")


@pytest.mark.parametrize("case", ["mixed_values", "wide", "experts_behind_attention"])
def test_whole_prompt_bfloat16(made, case):
    d, cfg, w = made(case)
    eng = engine_of(d, "bfloat16")
    toks = tokens(cfg, 200, 4)
    slot = eng.open(1)
    got = eng.step(slot, [toks], [all_places(len(toks))])
    check(got, plain.forward(cfg, w, toks), "bfloat16", case)


@pytest.mark.parametrize("seed", range(10))
def test_sizes_of_many_kinds(tmp_path, seed):
    """Configurations drawn at random: a prompt in two portions and a few decoded tokens, two requests side by side, in
    true 32-bit against the plain implementation at every position, and in bfloat16."""
    cfg = random_case(seed)
    wt = random_weights(cfg, seed, torch.bfloat16)
    w = as_float64(wt)
    d = write_model_dir(str(tmp_path), cfg, wt)
    a, b = tokens(cfg, 140, seed), tokens(cfg, 31, 100 + seed)
    wa, wb = plain.forward(cfg, w, a), plain.forward(cfg, w, b)
    for dtype in ("float32", "bfloat16"):
        eng = engine_of(d, dtype)
        sa, sb = eng.open(2)
        out = eng.step([sa, sb], [a[:70], b[:3]], [all_places(70), all_places(3)])
        rows_a, rows_b = [out[:70]], [out[70:]]
        out = eng.step([sa, sb], [a[70:130], b[3:]], [all_places(60), all_places(len(b) - 3)])
        rows_a.append(out[:60])
        rows_b.append(out[60:])
        eng.close([sb])
        rows_a += [eng.step([sa], [[t]]) for t in a[130:]]
        ga, gb = torch.cat(rows_a), torch.cat(rows_b)
        assert bool(torch.isfinite(ga).all()) and bool(torch.isfinite(gb).all())
        if dtype == "float32":
            check(ga, wa, what=f"seed {seed}: {json.dumps(cfg['layers'])}")
            check(gb, wb, what=f"seed {seed}, second request")
        else:
            assert np.median(errors(ga, wa)) < 0.06, f"seed {seed}: median {np.median(errors(ga, wa)):.3f}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_prompt_of_a_thousand_tokens(made, dtype):
    """Long enough for the plain products of the bfloat16 path to go to the vendor's library, over many pages, with the
    kept first positions far behind the window."""
    d, cfg, w = made("wide")
    eng = engine_of(d, dtype)
    toks = tokens(cfg, 1000, 9)
    slot = eng.open(1)
    got = eng.step(slot, [toks], [all_places(1000)])
    check(got, plain.forward(cfg, w, toks), dtype, "a thousand tokens")


@pytest.mark.parametrize("case", ["mixed_values", "plain_sizes", "wide"])
def test_layers_one_by_one(made, case):
    d, cfg, w = made(case)
    eng = engine_of(d)
    toks = tokens(cfg, 90, 5)
    want = []
    plain.forward(cfg, w, toks, want)
    got = []
    eng.layer_hook = lambda entry, hidden, batch: got.append(hidden.double().cpu().numpy())
    slot = eng.open(1)
    eng.step(slot, [toks])
    eng.layer_hook = None
    assert len(got) == len(want)
    for i, (g, x) in enumerate(zip(got, want)):
        assert np.abs(g - x).max() < 2e-5 * max(1.0, np.abs(x).max()), f"{case}: the stream behind layer {i}"


# ---------------------------------------------------------------- decoding, portions, batches
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("case", sorted(CASES))
def test_prompt_then_token_by_token(made, case, dtype):
    d, cfg, w = made(case)
    eng = engine_of(d, dtype)
    toks = tokens(cfg, 190, 6)
    want, how = wanted(eng, cfg, w, toks, dtype)
    check(prompt_then_decode(eng, toks, 70), want, how, f"{case}: prompt of 70, then token by token")


def test_token_by_token_from_the_first(made):
    d, cfg, w = made("mixed_values")
    eng = engine_of(d)
    toks = tokens(cfg, 140, 7)
    check(prompt_then_decode(eng, toks, 1), plain.forward(cfg, w, toks), what="token by token from the first")


@pytest.mark.parametrize("case", ["mixed_values", "wide", "plain_sizes"])
def test_portions(made, case):
    d, cfg, w = made(case)
    eng = engine_of(d)
    toks = tokens(cfg, 230, 8)
    want = plain.forward(cfg, w, toks)
    for sizes in ([2] * 115, [64, 64, 64, 38], [63, 2, 65, 100], [1, 2, 3, 5, 8, 13, 21, 34, 55, 88], [129, 101]):
        slot, rows, at = eng.open(1), [], 0
        for c in sizes:
            rows.append(eng.step(slot, [toks[at:at + c]], [all_places(c)]))
            at += c
        eng.close(slot)
        check(torch.cat(rows), want[:at], what=f"{case}: portions of {sizes[:4]}...")


def test_portions_bfloat16(made):
    d, cfg, w = made("wide")
    eng = engine_of(d, "bfloat16")
    toks = tokens(cfg, 200, 8)
    want, how = wanted(eng, cfg, w, toks, "bfloat16")
    for sizes in ([2] * 100, [64, 64, 72], [17, 130, 53]):
        slot, rows, at = eng.open(1), [], 0
        for c in sizes:
            rows.append(eng.step(slot, [toks[at:at + c]], [all_places(c)]))
            at += c
        eng.close(slot)
        check(torch.cat(rows), want[:at], how, f"portions of {sizes[:3]}...")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("case", ["mixed_values", "wide"])
def test_unequal_batch(made, case, dtype):
    """Four requests of unequal lengths start together and are decoded together; the short ones end early.  Each against
    itself alone."""
    d, cfg, w = made(case)
    eng = engine_of(d, dtype)
    lens, decoded = [5, 131, 64, 30], [3, 80, 40, 12]
    seqs = [tokens(cfg, n + k, 50 + i) for i, (n, k) in enumerate(zip(lens, decoded))]
    wants = [wanted(eng, cfg, w, s, dtype) for s in seqs]
    slots = eng.open(4)
    out = eng.step(slots, [s[:n] for s, n in zip(seqs, lens)], [all_places(n) for n in lens])
    rows = [[r] for r in torch.split(out, lens)]
    for step in range(max(decoded)):
        live = [i for i in range(4) if step < decoded[i]]
        out = eng.step([slots[i] for i in live], [[seqs[i][lens[i] + step]] for i in live])
        for j, i in enumerate(live):
            rows[i].append(out[j:j + 1])
        for i in range(4):
            if step + 1 == decoded[i]:
                eng.close([slots[i]])
    for i in range(4):
        check(torch.cat(rows[i]), wants[i][0], wants[i][1], f"{case}: request {i} of the batch")


def test_slots_and_pages_used_again(made):
    """A cache with room for little: sequences come and go, each finds the pages and the slot of one before it, with that
    one's keys in the pages and its last row in the slot's state."""
    d, cfg, w = made("mixed_values")
    eng = engine_of(d, max_tokens=384, max_slots=2)
    for turn in range(3):
        a, b = tokens(cfg, 120 + turn, 20 + turn), tokens(cfg, 70, 30 + turn)
        sa, sb = eng.open(2)
        out = eng.step([sa, sb], [a[:100], b[:5]], [all_places(100), all_places(5)])
        rows_a, rows_b = [out[:100]], [out[100:]]
        eng.close([sa])
        rows_b.append(eng.step([sb], [b[5:]], [all_places(len(b) - 5)]))
        sc = eng.open(1)[0]
        assert sc == sa
        c = tokens(cfg, 66, 40 + turn)
        rows_c = [eng.step([sc], [c[:60]], [all_places(60)])] + [eng.step([sc], [[t]]) for t in c[60:]]
        eng.close([sb, sc])
        check(torch.cat(rows_a), plain.forward(cfg, w, a)[:100], what="first")
        check(torch.cat(rows_b), plain.forward(cfg, w, b), what="second")
        check(torch.cat(rows_c), plain.forward(cfg, w, c), what="in the first one's slot")
    assert all(v == 0 for v in eng.cache.pages_held().values())


def test_a_prompt_longer_than_a_window_s_pool_runs_in_cuts(made):
    """Where the pools of the groups with windows are sized for a window and a step of 128 positions, a prompt of 700 tokens
    runs as six steps behind one call: the row that every layer keeps of the token before, the source layer's values of the
    same step and the kept first positions all carry over from cut to cut."""
    d, cfg, w = made("wide")
    eng = engine_of(d, max_slots=1, window_step=128)
    assert eng.cache.step_limit == 128
    toks = tokens(cfg, 700, 13)
    want = plain.forward(cfg, w, toks)
    slot = eng.open(1)
    got = eng.step(slot, [toks[:640]], [all_places(640)])
    rows = [got] + [eng.step(slot, [toks[640:]], [all_places(60)])]
    eng.close(slot)
    check(torch.cat(rows), want, what="700 tokens in cuts of 128")


def test_long_decoding_gives_pages_back_but_the_first(made):
    d, cfg, w = made("wide")
    eng = engine_of(d)
    toks = tokens(cfg, 430, 11)
    slot = eng.open(1)
    rows = [eng.step(slot, [toks[:10]], [all_places(10)])] + [eng.step(slot, [[t]]) for t in toks[10:]]
    held = eng.cache.pages_held()
    for i, g in enumerate(eng.cache.groups):
        if g.key.window is not None:       # the window's pages and the kept first ones, not the 7 that 430 positions touch
            assert held[i] == len(g.needed_pages(430)) < 7
    eng.close(slot)
    check(torch.cat(rows), plain.forward(cfg, w, toks), what="430 tokens, 420 of them decoded")


# ---------------------------------------------------------------- one key that decides: far back, at borders, at a window's edge
def plant_token(w, scale=1.0):
    """Channel 0 of the embedding is nonzero for token 1 only, channel 1 the same for every token; the first layer's
    mixer reads the stream as it is (no blend with the row before)."""
    w["embed"][:, 0] = 0.0
    w["embed"][1, 0] = 4.0 / scale
    w["embed"][:, 1] = 2.0 / scale
    w["l0.shift"][:] = 0.0


def planted_attention(seed: int, window, keep_first=None, kv_heads: int = 1):
    """An attention layer whose every query looks along the last channel of a head (which no rotation touches), where only
    token 1 has a key: behind the head norms both are nearly sqrt(dim) along it, the score 16 against less than 1; with a
    bias of -6 on the scores the planted key weighs 1 and every other key 0.003."""
    D = 16
    cfg = config(32, 40, [(attention(2, kv_heads, D, 16, rot=8, scale=1.0, window=window, keep_first=keep_first,
                                     scaling=stretch(4.0, 32, 1.0, 2.0)), None)], embedding_scale=2.0)
    w = as_float64(random_weights(cfg, seed, torch.bfloat16))
    plant_token(w, 2.0)
    w["l0.mix.pb"][:] = -6.0
    w["l0.mix.q.norm"][:] = 1.0
    w["l0.mix.k.norm"][:] = 1.0
    for g in range(kv_heads):
        w["l0.mix.k"][g * D + D - 1, :] = 0.0
        w["l0.mix.k"][g * D + D - 1, 0] = 50.0
        w["l0.mix.k.b"][g * D + D - 1] = 0.0
    for head in range(2):
        w["l0.mix.q"][head * D + D - 1, :] = 0.0
        w["l0.mix.q"][head * D + D - 1, 1] = 50.0
        w["l0.mix.q.b"][head * D + D - 1] = 0.0
    return cfg, w


def planted_latent(seed: int, window=None):
    """A latent-attention layer: the first number of the latent is nonzero for token 1 only, every head's key along its first
    plain channel is that number, and every query looks along that channel."""
    D, Rr, R, Q = 8, 4, 24, 12
    cfg = config(32, 40, [(latent(2, D, Rr, 16, R, Q, scale=0.25, window=window), None)])
    w = as_float64(random_weights(cfg, seed, torch.bfloat16))
    plant_token(w)
    w["l0.mix.dkv"][0, :] = 0.0
    w["l0.mix.dkv"][0, 0] = 8.0
    w["l0.mix.dkv.norm"][0] = 1.0
    w["l0.mix.dq"][0, :] = 0.0
    w["l0.mix.dq"][0, 1] = 8.0
    w["l0.mix.dq.norm"][0] = 1.0
    for head in range(2):
        w["l0.mix.uk"][head * D, :] = 0.0
        w["l0.mix.uk"][head * D, 0] = 2.0
        w["l0.mix.uq"][head * (D + Rr), :] = 0.0
        w["l0.mix.uq"][head * (D + Rr), 0] = 3.0
    return cfg, w


BASE = [2 + (i * 7) % 38 for i in range(400)]


@pytest.mark.parametrize("kind", ["attention", "latent"])
def test_a_key_far_back_and_at_the_borders_of_pages(tmp_path, kind):
    """The one token that every later query looks for stands at the first position, at a page's last and first places, or
    300 tokens back; the rows behind it are read in a prompt and in decoding.  The plain implementation's own outputs with
    and without it differ by much, so a key that is lost or taken from a wrong place shows."""
    cfg, w = planted_attention(1, None) if kind == "attention" else planted_latent(2)
    eng = engine_of(folder_of(tmp_path, cfg, w))
    base = BASE[:340]
    without = plain.forward(cfg, w, base)
    for place in (0, 63, 64, 65, 127, 128, 255, 300):
        toks = list(base)
        toks[place] = 1
        want = plain.forward(cfg, w, toks)
        assert errors(want[place + 1:], without[place + 1:]).min() > 0.05, place
        for cut in (310, 62, 129):
            check(prompt_then_decode(eng, toks, cut), want, what=f"{kind}: the token at {place}, prompt of {cut}")


@pytest.mark.parametrize("kind,window,kv_heads", [("attention", 70, 1), ("attention", 64, 2), ("attention", 65, 1), ("attention", 5, 1),
                                                  ("attention", 1, 2), ("attention", 130, 1), ("latent", 66, 1), ("latent", 64, 1),
                                                  ("latent", 3, 1), ("latent", 129, 1)])
def test_a_key_just_inside_and_just_outside_a_window(tmp_path, kind, window, kv_heads):
    """A query at position i sees the planted key at p exactly if i - p < window: the plain rows with and without it differ
    by much up to p + window - 1 and not at all from p + window on, in a prompt, in portions and in decoding, with the key
    at the borders of pages."""
    cfg, w = planted_attention(4, window, kv_heads=kv_heads) if kind == "attention" else planted_latent(5, window)
    eng = engine_of(folder_of(tmp_path, cfg, w))
    n = 100 + window + 14
    base = BASE[:n]
    without = plain.forward(cfg, w, base)
    for place in (0, 3, 63, 64, 100):
        toks = list(base)
        toks[place] = 1
        want = plain.forward(cfg, w, toks)
        edge = place + window
        if window > 1:
            assert errors(want[place + 1:edge], without[place + 1:edge]).min() > 0.05, place
        assert errors(want[edge:], without[edge:]).max() < 1e-12, place
        for cut in (n - 2, edge - 1, edge, max(1, edge - 40), place + 1):       # the edge in the prompt, first decoded, decoded
            cut = max(1, min(cut, n - 1))
            check(prompt_then_decode(eng, toks, cut), want, what=f"window {window}: the token at {place}, prompt of {cut}")
        slot, rows, at = eng.open(1), [], 0                                       # and in portions that end around the edge
        for c in [place + 1, window - 2, 1, 1, 2, 7] if window > 3 else [place + 1, 2, 2, 7]:
            rows.append(eng.step(slot, [toks[at:at + c]], [all_places(c)]))
            at += c
        eng.close(slot)
        check(torch.cat(rows), want[:at], what=f"window {window}: the token at {place}, portions")


@pytest.mark.parametrize("window,keep", [(20, 6), (64, 1), (5, 64), (70, 66), (3, 130)])
def test_first_positions_that_a_window_keeps_in_sight(tmp_path, window, keep):
    """The planted key among the first ``keep`` positions is seen by every later token, hundreds of positions behind the
    window; at the next position it is seen through the window only.  In a prompt, in portions and in decoding, with pages
    that the window has given back in between."""
    cfg, w = planted_attention(6, window, keep_first=keep)
    eng = engine_of(folder_of(tmp_path, cfg, w))
    n = keep + window + 260
    base = (BASE + BASE)[:n]
    without = plain.forward(cfg, w, base)
    for place in sorted({0, keep - 1, keep, keep + 1, min(keep - 1, 63), min(keep - 1, 64)}):
        toks = list(base)
        toks[place] = 1
        want = plain.forward(cfg, w, toks)
        if place < keep:
            assert errors(want[place + 1:], without[place + 1:]).min() > 0.05, place
        else:
            assert errors(want[place + window:], without[place + window:]).max() < 1e-12, place
        for cut in (n - 3, place + 1, min(n - 1, place + window), min(n - 1, keep + window + 70)):
            check(prompt_then_decode(eng, toks, max(1, cut)), want, what=f"window {window}, {keep} kept: the token at {place}, prompt of {cut}")
        slot, rows, at = eng.open(1), [], 0
        for c in [place + 1, 2, window, 64, 65, 2, 60]:
            rows.append(eng.step(slot, [toks[at:at + c]], [all_places(c)]))
            at += c
        eng.close(slot)
        check(torch.cat(rows), want[:at], what=f"window {window}, {keep} kept: the token at {place}, portions")


def test_values_that_a_model_may_happen_to_make_equal_or_one(tmp_path):
    """Multipliers of 1, scales of 1, windows as wide as the kept positions, one expert, every router output chosen,
    rotation of nothing and of a whole head, a mix of 0 and of 1."""
    cfg = config(32, 50, [(attention(2, 2, 8, 8, scale=1.0, rot=8, window=4, keep_first=4, v_mix=True), moe(1, 2, 8, identity=1)),
                          (attention(2, 2, 16, 8, scale=1.0, rot=0, v_mix=True), moe(2, 1, 8, identity=0)),
                          (attention(4, 2, 8, 8, window=200, keep_first=0, v_mix=True), None),
                          (latent(1, 8, 8, 8, 8, 8, scale=1.0, window=2), moe(3, 3, 16))], eps=1e-5)
    wt = random_weights(cfg, 12, torch.bfloat16)
    wt["l1.mix.vmix"] = torch.tensor(0.0, dtype=torch.bfloat16)
    wt["l2.mix.vmix"] = torch.tensor(1.0, dtype=torch.bfloat16)
    w = as_float64(wt)
    eng = engine_of(write_model_dir(str(tmp_path), cfg, wt))
    toks = tokens(cfg, 150, 2)
    want = plain.forward(cfg, w, toks)
    check(prompt_then_decode(eng, toks, 80), want, what="ones and equals")
    check(prompt_then_decode(eng, toks, 3), want, what="ones and equals, decoded")


# ---------------------------------------------------------------- kernels one by one
def f32(a):
    return torch.tensor(np.asarray(a), dtype=torch.float32, device="cuda")


def test_token_shift_kernel_keeps_the_last_row_per_slot():
    from turboquant_cpp_amd.csrc import ops
    rng = np.random.default_rng(0)
    H = 40
    wgt = rng.uniform(0, 1, H)
    state = np.zeros((6, H))
    state[4] = rng.standard_normal(H)          # slot 4 goes on from an earlier step, slot 1 is new
    x = rng.standard_normal((7, H))
    runs = {"cu_seqlens": torch.tensor([0, 3, 7], dtype=torch.int32, device="cuda"),
            "slots": torch.tensor([4, 1], dtype=torch.int32, device="cuda")}
    for act in ("float32", "bfloat16"):
        st = f32(state)
        got = ops.token_shift(f32(x), f32(wgt), st, runs, act).double().cpu().numpy()
        before = np.concatenate([state[4:5], x[0:2], state[1:2], x[3:6]])
        want = x + (before - x) * wgt
        assert np.abs(got - want).max() < (1e-6 if act == "float32" else 0.03)
        assert np.allclose(st[4].cpu().numpy(), x[2], atol=1e-7) and np.allclose(st[1].cpu().numpy(), x[6], atol=1e-7)
        assert float(st[0].abs().sum() + st[2].abs().sum()) == 0.0


def test_token_shift_behind_the_sum_of_a_decode_step():
    """One token per sequence: the blend in the launch that sums a normed part into the stream gives the bits of the two
    launches apart, and leaves the same rows in the slots."""
    from turboquant_cpp_amd.csrc import ops
    rng = np.random.default_rng(4)
    for H in (40, 256):
        T = 5
        slots = torch.tensor([7, 2, 0, 5, 3], dtype=torch.int32, device="cuda")
        runs = {"cu_seqlens": torch.arange(T + 1, dtype=torch.int32, device="cuda"), "slots": slots}
        x, d, st = rng.standard_normal((T, H)), rng.standard_normal((2, T, H)), rng.standard_normal((8, H))
        wn, ws = f32(1 + 0.1 * rng.standard_normal(H)), f32(rng.uniform(0, 1, H))
        for act in ("float32", "bfloat16"):
            xa, xb, sa, sb = f32(x), f32(x), f32(st), f32(st)
            ha, _ = ops.add_rmsnorm(xa, ops.NormedDelta(f32(d), wn, 1e-5), None, 0.0, act, stream=True, shift=(ws, sa, slots))
            ops.add_rmsnorm(xb, ops.NormedDelta(f32(d), wn, 1e-5), None, 0.0, act)
            hb = ops.token_shift(xb, ws, sb, runs, act)
            assert torch.equal(xa, xb) and torch.equal(sa, sb) and torch.equal(ha, hb)
            assert torch.equal(sa[slots.long()], xa) and ha.data_ptr() != xa.data_ptr()


def test_unit_values_and_their_mix():
    from turboquant_cpp_amd.csrc import ops
    rng = np.random.default_rng(1)
    T, G, D, V, D1 = 9, 3, 32, 20, 48
    rows = rng.standard_normal((T, 100 + G * D))
    first = rng.standard_normal((T, G * D1))
    for eps, lam in ((1e-5, None), (1e-5, 0.3), (0.0, 0.75)):
        t = f32(rows)
        v = t[:, 100:]
        ops.value_norm_mix(v, G, D, V, eps, "float32", first=None if lam is None else f32(first), first_head_dim=D1,
                           mix=None if lam is None else f32([lam]))
        got = t.double().cpu().numpy()
        want = rows.copy()
        for g in range(G):
            a = rows[:, 100 + g * D:100 + g * D + V]
            a = a / np.sqrt((a * a).mean(1, keepdims=True) + eps) if eps else a
            if lam is not None:
                a = (1 - lam) * a + lam * first[:, g * D1:g * D1 + V]
            want[:, 100 + g * D:100 + g * D + V] = a
        assert np.abs(got - want).max() < 2e-6


def test_head_norms_unit_values_rotation_and_cache_write_in_one_launch():
    """``attn_prep_kv_write`` against ``head_rmsnorm``, ``value_norm_mix`` and ``rope_kv_write`` one after the other: the same
    queries, the same pages, the same values left behind in the rows; a prompt's run and single decoded tokens."""
    from turboquant_cpp_amd.csrc import ops
    rng = np.random.default_rng(5)
    nh, nkv, hd, kd, vd, page, extra = 6, 2, 48, 40, 24, 64, 0
    width = (nh + 2 * nkv) * hd
    inv_freq = f32(1.0 / 100.0 ** (np.arange(8) / 8.0))
    for act in ("float32", "bfloat16"):
        adt = torch.float32 if act == "float32" else torch.bfloat16
        wq, wk = (torch.tensor(np.concatenate([1 + 0.2 * rng.standard_normal(kd), np.zeros(hd - kd)]), dtype=adt, device="cuda") for _ in range(2))
        mix = torch.tensor([0.3], dtype=adt, device="cuda")
        for pairing in (0, 1):
            for n_new, start, with_first in ((70, 0, False), (70, 30, True), (3, 200, True), (1, 64, False)):
                T = n_new
                rows = rng.standard_normal((T, width + extra))
                rows[:, :width].reshape(T, nh + 2 * nkv, hd)[:, :nh + nkv, kd:] = 0.0      # heads laid out wider hold zeros
                rows[:, :width].reshape(T, nh + 2 * nkv, hd)[:, nh + nkv:, vd:] = 0.0
                first = f32(rng.standard_normal((T, nkv * 32))) if with_first else None
                positions = torch.arange(start, start + T, dtype=torch.int32, device="cuda")
                seq = torch.full((T,), 1, dtype=torch.int32, device="cuda")
                n_pages = -(-(start + T) // page)
                table = torch.full((2, n_pages), -1, dtype=torch.int32, device="cuda")
                table[1] = torch.tensor(rng.permutation(n_pages), dtype=torch.int32)
                stride = 2 * nkv * page * hd                        # two layers to a page; this one is the second
                offset = nkv * page * hd
                decode = T == 1
                runs = {"cu_seqlens": torch.tensor([0, T], dtype=torch.int32, device="cuda"), "slots": torch.tensor([1], dtype=torch.int32, device="cuda"),
                        "start": torch.tensor([start], dtype=torch.int32, device="cuda"), "max_new": T, "max_end": start + T, "decode": decode}
                results = []
                for fused in (False, True):
                    t = f32(rows)
                    qkv = t[:, :width]
                    kp = torch.zeros((n_pages * stride,), dtype=adt, device="cuda")
                    vp = torch.zeros_like(kp)
                    args = (positions, seq, table, inv_freq, pairing, 16, kp, vp, offset, page, stride, nh, nkv, hd, act)
                    if fused:
                        q = ops.attn_prep_kv_write(qkv, *args, runs=runs, q_weight=wq, k_weight=wk, qk_eps=1e-5, norm_dim=kd,
                                                   value_eps=1e-5, value_dim=vd, first=first, first_head_dim=32,
                                                   mix=mix if with_first else None)
                    else:
                        ops.head_rmsnorm(qkv, wq, wk, 1e-5, nh, nkv, hd, act, norm_dim=kd)
                        ops.value_norm_mix(qkv[:, (nh + nkv) * hd:], nkv, hd, vd, 1e-5, act, first=first, first_head_dim=32,
                                           mix=mix if with_first else None)
                        q = ops.rope_kv_write(qkv, *args, runs=runs)
                    results.append((q.float(), kp.float(), vp.float(), t[:, (nh + nkv) * hd:].clone()))
                tol = 2e-6 if act == "float32" else 1e-2
                for name, x, y in zip(("queries", "key pages", "value pages", "values left in the rows"), *results):
                    assert (x - y).abs().max() <= tol * max(1.0, float(y.abs().max())), (act, pairing, n_new, start, name)
                assert float(results[1][1].abs().max()) > 0 and float(results[1][2].abs().max()) > 0


def test_choice_by_corrected_scores_with_identity_experts():
    from turboquant_cpp_amd.csrc import ops
    rng = np.random.default_rng(2)
    for T, E, I, top, unit in ((1, 5, 3, 4, 16), (13, 8, 4, 4, 16), (700, 6, 2, 3, 64), (3000, 3, 0, 2, 64), (40, 2, 6, 8, 32)):
        H = 24
        x, r, corr = rng.standard_normal((T, H)), rng.standard_normal((E + I, H)), 0.3 * rng.standard_normal(E + I)
        ids, wts, own, order, slot, tile_e, n_tiles = ops.route(f32(x), f32(r), None, top, False, unit, "float32",
                                                                correction=f32(corr), identity=I)
        z = f32(x).double().cpu().numpy() @ f32(r).double().cpu().numpy().T
        s = np.exp(z - z.max(1, keepdims=True))
        s /= s.sum(1, keepdims=True)
        choice = s + f32(corr).double().cpu().numpy()
        ids, wts, slot, order = ids.cpu().numpy(), wts.cpu().numpy(), slot.cpu().numpy(), order.cpu().numpy()
        tile_e, n = tile_e.cpu().numpy(), int(n_tiles[0])
        for t in range(T):
            best = np.argsort(-choice[t], kind="stable")[:top]
            margin = np.sort(choice[t])[::-1]
            if top < E + I and margin[top - 1] - margin[top] < 1e-5:
                continue
            assert sorted(ids[t]) == sorted(best), (T, t)
            assert np.allclose(wts[t], s[t, ids[t]], rtol=1e-5)
            if I:
                assert abs(float(own[t]) - s[t, [e for e in ids[t] if e >= E]].sum()) < 1e-6
            for j, e in enumerate(ids[t]):
                if e >= E:
                    assert slot[t, j] == -1
                else:
                    assert order[slot[t, j]] == t and tile_e[slot[t, j] // unit] == e and slot[t, j] // unit < n
        assert (tile_e[:n] < E).all()


def test_sigmoid_weights_and_kept_positions_in_every_attention_kernel():
    """The three attention kernels (matrix cores in both types, and the plain one) on one paged cache: sigmoid weights with a
    bias per head, windows, kept first positions; prompts that go on from cached tokens and single decoded tokens."""
    from turboquant_cpp_amd.csrc import ops
    rng = np.random.default_rng(3)
    nh, nkv, hd, page = 4, 2, 32, 64
    for dtype, tol in (("float32", 2e-5), ("bfloat16", 0.03)):
        adt = torch.float32 if dtype == "float32" else torch.bfloat16
        for window, keep, n_old, n_new in ((40, 6, 300, 70), (64, 70, 200, 1), (None, 0, 100, 30), (130, 1, 500, 1), (5, 128, 190, 66),
                                           (130, 70, 4300, 1), (200, 5, 4200, 40), (70, 200, 4100, 1)):
            n = n_old + n_new
            k = rng.standard_normal((n, nkv, hd))
            v = rng.standard_normal((n, nkv, hd))
            q = rng.standard_normal((n_new, nh, hd))
            pb = rng.standard_normal(nh) - 1.0
            k_t, v_t, q_t = (torch.tensor(a, dtype=adt, device="cuda") for a in (k, v, q))
            k, v, q = (a.double().cpu().numpy() for a in (k_t, v_t, q_t))
            n_pages = -(-n // page)
            perm = rng.permutation(n_pages + 3)[:n_pages]
            stride = nkv * page * hd
            kp = torch.zeros(((n_pages + 3) * stride,), dtype=adt, device="cuda")
            vp = torch.zeros_like(kp)
            for lp in range(n_pages):
                rows = slice(lp * page, min(n, (lp + 1) * page))
                cnt = rows.stop - rows.start
                kp.view(-1, nkv, page, hd)[perm[lp], :, :cnt] = k_t[rows].transpose(0, 1)
                vp.view(-1, nkv, hd, page)[perm[lp], :, :, :cnt] = v_t[rows].permute(1, 2, 0)
            table = torch.full((3, n_pages), -1, dtype=torch.int32, device="cuda")
            table[2] = torch.tensor(perm, dtype=torch.int32)
            positions = torch.arange(n_old, n, dtype=torch.int32, device="cuda")
            seq = torch.full((n_new,), 2, dtype=torch.int32, device="cuda")
            runs = {"cu_seqlens": torch.tensor([0, n_new], dtype=torch.int32, device="cuda"),
                    "slots": torch.tensor([2], dtype=torch.int32, device="cuda"),
                    "start": torch.tensor([n_old], dtype=torch.int32, device="cuda"), "max_new": n_new, "max_end": n, "decode": n_new == 1}
            want = np.zeros((n_new, nh, hd))
            for i in range(n_new):
                p = n_old + i
                j = np.arange(p + 1)
                see = (j >= p - window + 1) | (j < keep) if window else np.ones(p + 1, dtype=bool)
                for h in range(nh):
                    s = k[:p + 1, h // (nh // nkv)] @ q[i, h] * 0.2 + pb[h]
                    want[i, h] = (np.where(see, 1 / (1 + np.exp(-s)), 0.0)[:, None] * v[:p + 1, h // (nh // nkv)]).sum(0)
            for with_runs in (True, False):
                got = ops.attention(q_t.reshape(n_new, nh * hd), kp, vp, 0, positions, seq, table, page, stride, nh, nkv, hd, window, 0.2,
                                    dtype, runs=runs if with_runs else None, sigmoid_bias=f32(pb), keep_first=keep)
                got = got.double().cpu().numpy().reshape(n_new, nh, hd)
                assert np.abs(got - want).max() < tol * max(1.0, np.abs(want).max()), (dtype, window, keep, n_old, n_new, with_runs)


# ---------------------------------------------------------------- the library's own entry points
def test_greedy_generation_through_the_entry_point(made):
    from turboquant_cpp_amd import Model
    d, cfg, w = made("mixed_values")
    prompts = [tokens(cfg, 9, 1), tokens(cfg, 70, 2), tokens(cfg, 3, 3)]
    with Model(d, dtype="float32", temperature=0.0, rep_penalty=1.0, max_tokens=12, max_batch=4, stop_tokens=()) as m:
        got = m.generate(prompts, loop_detection=False)
    for p, g in zip(prompts, got):
        assert len(g) == 12
        rows = plain.forward(cfg, w, p + g)
        for j, tok in enumerate(g):          # every chosen token is the plain model's best (or within rounding of it)
            row = rows[len(p) - 1 + j]
            assert row[tok] >= row.max() - 1e-4 * np.abs(row).max(), (p[:3], j)


def test_a_conversation_over_state_and_kept_positions(made, tmp_path):
    """``Model.chat``: a turn that goes on runs only the new tokens; a history that parts from the cached tokens starts over
    (the row that a layer keeps of the token before has no earlier value); a saved conversation, with the pages of its
    windows and of its kept first positions and its rows of state, goes on in another model object with the same tokens."""
    from turboquant_cpp_amd import Model
    d, cfg, w = made("wide")
    opts = dict(dtype="float32", temperature=0.0, rep_penalty=1.0, max_tokens=5, context_length=512)
    h1, extra, other, more = (tokens(cfg, n, 70 + n) for n in (150, 9, 150, 5))
    with Model(d, **opts) as m, Model(d, **opts) as fresh:
        brought = []
        step = m.engine.step
        m.engine.step = lambda slots, toks, *a, **k: (brought.append(len(toks[0])), step(slots, toks, *a, **k))[1]
        out1 = m.chat(h1)
        assert out1 == fresh.generate([h1])[0] and brought[0] == 150
        del brought[:]
        h2 = h1 + out1 + extra
        out2 = m.chat(h2)
        assert brought[0] == 1 + len(extra) and out2 == fresh.generate([h2])[0]
        saved = str(tmp_path / "talk.kv")
        m.save_context(saved)
        del brought[:]
        h3 = h1[:40] + other
        assert m.chat(h3) == fresh.generate([h3])[0] and brought[0] == len(h3)
        with Model(d, **opts) as later:
            later.load_context(saved)
            h4 = h2 + out2 + more
            assert later.chat(h4) == fresh.generate([h4])[0]


def test_command_line(made):
    """``bin/quant``: what it says of the folder, and greedy tokens that are the entry point's."""
    from turboquant_cpp_amd import Model
    d, cfg, w = made("experts_behind_attention")
    quant = os.path.join(ROOT, "bin", "quant")
    info = subprocess.run([quant, d, "--info"], capture_output=True, text=True, timeout=300)
    assert info.returncode == 0 and "Bosalix" in info.stdout, info.stderr[-1000:]
    run = subprocess.run([quant, d, "-p", "5,17,3;8,2", "-n", "6", "-T", "0", "--rep-penalty", "1.0", "--dtype", "float32",
                          "--json", "-M"], capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, run.stderr[-2000:]
    with Model(d, dtype="float32", temperature=0.0, rep_penalty=1.0, max_tokens=6) as m:
        want = m.generate([[5, 17, 3], [8, 2]])
    got = [r["tokens"] for r in json.loads(run.stdout.strip().splitlines()[-1])]
    assert got == want


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_runner_as_a_program(made, tmp_path, dtype):
    """Two requests start together, are decoded together, one ends early; the logits the program writes are the engine's."""
    d, cfg, w = made("mixed_values")
    a, b = tokens(cfg, 80, 1), tokens(cfg, 9, 2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:70], "want": [0, 69]}, {"id": "b", "tokens": b[:5], "want": [4]}], "end": []}]
    for i in range(4):
        steps.append({"step": 1 + i, "entries": [{"id": "a", "tokens": [a[70 + i]], "want": [0]}, {"id": "b", "tokens": [b[5 + i]], "want": [0] if i % 2 else []}],
                      "end": ["b"] if i == 3 else []})
    for i in range(4, 10):
        steps.append({"step": 1 + i, "entries": [{"id": "a", "tokens": [a[70 + i]], "want": [0]}], "end": []})
    out_dir = str(tmp_path / "out")
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", d, "--dtype", dtype, "--out", out_dir,
                          "--max-tokens", "200"], input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, run.stderr[-2000:]
    assert [l for l in run.stdout.splitlines() if l.startswith("done")] == [f"done {s['step']}" for s in steps]
    wa, wb = plain.forward(cfg, w, a), plain.forward(cfg, w, b)
    V = cfg["vocab"]
    first = np.fromfile(os.path.join(out_dir, "0.f32"), dtype="<f4").reshape(-1, V)
    kind = dtype if dtype == "float32" else "bfloat16"
    check(first, np.stack([wa[0], wa[69], wb[4]]), kind, "first step")
    for i in range(10):
        got = np.fromfile(os.path.join(out_dir, f"{1 + i}.f32"), dtype="<f4").reshape(-1, V)
        want = [wa[70 + i]] + ([wb[5 + i]] if i < 4 and i % 2 else [])
        check(got, np.stack(want), kind, f"step {1 + i}")
