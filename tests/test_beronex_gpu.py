"""The Beronex design in the engine against the plain implementation in ``plain_beronex.py``: every mechanism alone, whole
prompts, the stream behind every layer, decoding through the cache and the state, prompts in portions, unequal batches,
slots and pages that are used again, keys far away, at the borders of pages and just inside and outside a window (also the
wider window of a layer that reads another layer's keys), the first tokens of a sequence, long decoding, a state that still
holds the first token hundreds of tokens later, sizes of many kinds, the kernels one by one, greedy generation through the
library's entry point, the command line, and the trace runner as a program."""
import json
import os
import subprocess

import numpy as np
import pytest
import torch

import plain_beronex as plain
from beronex_cases import CASES, attention, config, dense, latent, lightning, moe, random_case, tensors, tokens, write_folder, yarn

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
F32_BOUND = 1e-4        # of the logits' root mean square, per position, mean taken off


@pytest.fixture(scope="module")
def made(tmp_path_factory):
    """(case, seed, peaky) -> (folder, config, weights), each written once."""
    cache = {}

    def get(case: str, seed: int = 0, peaky: float = 1.0):
        key = (case, seed, peaky)
        if key not in cache:
            cfg = CASES[case]
            w = tensors(cfg, seed, peaky)
            cache[key] = (write_folder(str(tmp_path_factory.mktemp(f"beronex_{case}")), cfg, w), cfg, w)
        return cache[key]
    return get


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
        assert e.max() < 0.2 and np.quantile(e, 0.9) < 0.06 and np.median(e) < 0.03, \
            f"{what}: median {np.median(e):.3f}, 90 % {np.quantile(e, 0.9):.3f}, worst {e.max():.3f} at {int(e.argmax())}"
    else:       # "same path": the engine against itself on another schedule, in bfloat16
        assert np.quantile(e, 0.9) < 0.02 and e.max() < 0.3, \
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


@pytest.mark.parametrize("case", ["regular", "odd", "ragged", "wide"])
def test_whole_prompt_bfloat16(made, case):
    d, cfg, w = made(case)
    eng = engine_of(d, "bfloat16")
    toks = tokens(cfg, 200, 4)
    slot = eng.open(1)
    got = eng.step(slot, [toks], [all_places(len(toks))])
    check(got, plain.forward(cfg, w, toks), "bfloat16", case)


@pytest.mark.parametrize("seed", range(12))
def test_sizes_of_many_kinds(tmp_path, seed):
    """Configurations drawn at random: a prompt in two portions and a few decoded tokens, two requests side by side, in
    true 32-bit against the plain implementation at every position, and in bfloat16."""
    cfg = random_case(seed)
    w = tensors(cfg, seed)
    d = write_folder(str(tmp_path), cfg, w)
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
            assert np.median(errors(ga, wa)) < 0.05, f"seed {seed}: median {np.median(errors(ga, wa)):.3f}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_prompt_of_a_thousand_tokens(made, dtype):
    """Long enough for the plain products of the bfloat16 path to go to the vendor's library, over many pages and several
    windows, then decoded on."""
    d, cfg, w = made("regular", seed=7)
    eng = engine_of(d, dtype)
    toks = tokens(cfg, 1010, 13)
    check(prompt_then_decode(eng, toks, 1000), plain.forward(cfg, w, toks), dtype, "1,000 tokens")


@pytest.mark.parametrize("case", ["odd", "ragged"])
def test_layers_one_by_one(made, case):
    """The residual stream behind every layer, layers on another's keys and values included."""
    d, cfg, w = made(case)
    eng = engine_of(d)
    seen = []
    eng.layer_hook = lambda entry, hidden, batch: seen.append(hidden.double().cpu().numpy())
    toks = tokens(cfg, 120, 5)
    eng.step(eng.open(1), [toks], [[]])
    _, streams = plain.forward(cfg, w, toks, return_layers=True)
    assert len(seen) == len(cfg["layers"])
    for i, (a, b) in enumerate(zip(seen, streams)):
        assert np.abs(a - b).max() < 2e-4 * max(1.0, np.abs(b).max()), f"layer {i}"


# ---------------------------------------------------------------- decoding, portions, batches
@pytest.mark.parametrize("case,dtype", [("odd", "float32"), ("ragged", "float32"), ("regular", "float32"),
                                        ("regular", "bfloat16"), ("odd", "bfloat16"), ("ragged", "bfloat16"),
                                        ("wide", "float32"), ("wide", "bfloat16"), ("attention_only", "float32"),
                                        ("lightning_only", "float32"), ("latent_only", "float32"),
                                        ("experts_behind_lightning", "float32"), ("dense_behind_attention", "float32")])
def test_prompt_then_token_by_token(made, case, dtype):
    """Most of a sequence in one step, the rest one token a step (the later steps replayed as graphs), across the edges of
    pages and of windows."""
    d, cfg, w = made(case)
    eng = engine_of(d, dtype)
    toks = tokens(cfg, 150, 6)
    want, how = wanted(eng, cfg, w, toks, dtype)
    check(prompt_then_decode(eng, toks, 58), want, how, case)


def test_token_by_token_from_the_first(made):
    """No prompt step at all: the first tokens of a sequence through the decode kernels, an empty state, a softmax over
    one key, windows that are not yet full."""
    for case in ("odd", "ragged", "regular"):
        d, cfg, w = made(case)
        eng = engine_of(d)
        toks = tokens(cfg, 110, 16)
        check(prompt_then_decode(eng, toks, 1), plain.forward(cfg, w, toks), what=case)


@pytest.mark.parametrize("case", ["odd", "ragged", "regular"])
def test_portions(made, case):
    """The logits do not depend on how a prompt was cut: portions of two tokens and more, of one, of a page and over."""
    d, cfg, w = made(case)
    eng = engine_of(d)
    toks = tokens(cfg, 190, 7)
    want = plain.forward(cfg, w, toks)
    for cuts in ([2, 3, 1, 5, 2, 64, 7, 2, 33, 71], [17, 2, 2, 100, 69], [95, 95], [64, 64, 62], [2] * 95):
        assert sum(cuts) == len(toks)
        slot, rows, at = eng.open(1), [], 0
        for c in cuts:
            rows.append(eng.step(slot, [toks[at:at + c]], [all_places(c)]))
            at += c
        eng.close(slot)
        check(torch.cat(rows), want, what=f"{case}, cuts {cuts[:12]}")


def test_portions_bfloat16(made):
    d, cfg, w = made("regular")
    eng = engine_of(d, "bfloat16")
    toks = tokens(cfg, 190, 7)
    want, how = wanted(eng, cfg, w, toks, "bfloat16")
    slot, rows, at = eng.open(1), [], 0
    for c in [2, 3, 1, 5, 2, 64, 7, 2, 33, 71]:
        rows.append(eng.step(slot, [toks[at:at + c]], [all_places(c)]))
        at += c
    check(torch.cat(rows), want, how, "portions")


@pytest.mark.parametrize("case,dtype", [("odd", "float32"), ("regular", "float32"), ("regular", "bfloat16"),
                                        ("ragged", "float32"), ("wide", "bfloat16"), ("odd", "bfloat16")])
def test_unequal_batch(made, case, dtype):
    """Requests of unequal lengths in one step and decoded together, the shorter ones ending earlier, against each alone."""
    d, cfg, w = made(case)
    eng = engine_of(d, dtype)
    lengths, prompts = [1, 37, 131, 64, 90], [1, 20, 100, 64, 61]
    seqs = [tokens(cfg, n, 10 + i) for i, n in enumerate(lengths)]
    alone = [wanted(eng, cfg, w, s, dtype) for s in seqs]
    slots = eng.open(len(seqs))
    got = [[] for _ in seqs]
    out = eng.step(slots, [s[:p] for s, p in zip(seqs, prompts)], [all_places(p) for p in prompts])
    at = 0
    for i, p in enumerate(prompts):
        got[i].append(out[at:at + p])
        at += p
    done = list(prompts)
    while True:
        live = [i for i, s in enumerate(seqs) if done[i] < len(s)]
        if not live:
            break
        out = eng.step([slots[i] for i in live], [[seqs[i][done[i]]] for i in live])
        for r, i in enumerate(live):
            got[i].append(out[r:r + 1])
            done[i] += 1
            if done[i] == len(seqs[i]):
                eng.close([slots[i]])
    eng.close([slots[0]])
    for i, s in enumerate(seqs):
        check(torch.cat(got[i]), alone[i][0], alone[i][1], f"{case}, request {i}")


def test_slots_and_pages_used_again(made):
    """A cache with room for little: sequences come and go, each finds the pages and the slot of one before it, with that
    one's keys and latents in the pages and its state (a decay of 1 forgets nothing) in the slot's row."""
    d, cfg, w = made("odd")
    eng = engine_of(d, max_tokens=256, max_slots=2)
    for round_ in range(3):
        a, b = tokens(cfg, 120 + round_, 20 + round_), tokens(cfg, 70, 30 + round_)
        sa, sb = eng.open(2)
        out = eng.step([sa, sb], [a[:100], b[:5]], [all_places(100), all_places(5)])
        rows_a, rows_b = [out[:100]], [out[100:]]
        eng.close([sa])
        rows_b.append(eng.step([sb], [b[5:]], [all_places(len(b) - 5)]))
        sc = eng.open(1)[0]
        assert sc == sa
        c = tokens(cfg, 66, 40 + round_)
        rows_c = [eng.step([sc], [c[:60]], [all_places(60)])] + [eng.step([sc], [[t]]) for t in c[60:]]
        eng.close([sb, sc])
        check(torch.cat(rows_a), plain.forward(cfg, w, a)[:100], what="first")
        check(torch.cat(rows_b), plain.forward(cfg, w, b), what="second")
        check(torch.cat(rows_c), plain.forward(cfg, w, c), what="in the first one's slot")
    assert all(v == 0 for v in eng.cache.pages_held().values())


# ---------------------------------------------------------------- one key that decides: far back, at borders, at a window's edge
def plant_token(w):
    """Channel 0 of the embedding is nonzero for token 1 only, channel 1 the same for every token; the norm before the
    first mixer passes both as they are."""
    w["embed"][:, 0] = 0.0
    w["embed"][1, 0] = 4.0
    w["embed"][:, 1] = 2.0
    w["l0.norm1"][:2] = 1.0


def planted_attention(seed: int, window, reader_window="none", kv_heads: int = 1):
    """An attention layer whose every query looks along the last channel of a head (which no rotation touches), where only
    token 1 has a key: behind the head norms both are nearly sqrt(dim) along it, the score 16 against less than 1.  With
    ``reader_window`` a second layer without keys of its own asks the first one's cache the same way, through a window of
    its own."""
    D = 16
    first = attention(2, kv_heads, D, 16, rot=8, scale=1.0, window=window, scaling=yarn(4.0, 32, 8.0, 1.0))
    layers = [(first, None)]
    if reader_window != "none":
        layers.append((attention(2, kv_heads, D, 16, rot=8, scale=1.0, window=reader_window, scaling=yarn(4.0, 32, 8.0, 1.0), kv_from=0), None))
    cfg = config(32, 40, layers)
    w = tensors(cfg, seed)
    plant_token(w)
    for g in range(kv_heads):
        w["l0.mix.k"][g * D + D - 1, :] = 0.0
        w["l0.mix.k"][g * D + D - 1, 0] = 50.0
    for i in range(len(layers)):
        for head in range(2):
            w[f"l{i}.mix.q"][head * D + D - 1, :] = 0.0
            w[f"l{i}.mix.q"][head * D + D - 1, 1] = 50.0
    if len(layers) == 2:          # the first layer adds nothing to the two channels, and the second reads them as they are
        w["l0.norm1b"][:2] = 0.0
        w["l1.norm1"][:2] = 1.0
        w["l0.mix.q"][:] *= 0.0     # the first layer's own rows are flat: only the second layer's window shows
    return cfg, w


def planted_latent(seed: int):
    """A latent-attention layer: the first number of the latent is nonzero for token 1 only, every head's key along its first
    plain channel is that number, and every query looks along that channel."""
    D, Rr, R, Q = 8, 4, 24, 12
    cfg = config(32, 40, [(latent(2, D, Rr, 16, R, Q, scale=0.25, scaling=yarn(2.0, 16, 4.0, 1.0)), None)])
    w = tensors(cfg, seed)
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


@pytest.mark.parametrize("kind", ["attention", "latent"])
def test_a_key_far_back_and_at_the_borders_of_pages(tmp_path, kind):
    """The one token that every later query looks for stands at the first position, at a page's last and first places, or
    300 tokens back; the rows behind it are read in a prompt and in decoding.  The plain implementation's own outputs with
    and without it differ by much, so a key that is lost or taken from a wrong place shows."""
    cfg, w = planted_attention(1, None) if kind == "attention" else planted_latent(2)
    eng = engine_of(write_folder(str(tmp_path), cfg, w))
    n = 340
    base = [2 + (i * 7) % 38 for i in range(n)]
    without = plain.forward(cfg, w, base)
    for place in (0, 63, 64, 65, 127, 128, 255, 300):
        toks = list(base)
        toks[place] = 1
        want = plain.forward(cfg, w, toks)
        assert errors(want[place + 1:], without[place + 1:]).min() > 0.05, place
        for cut in (310, 62, 129):
            check(prompt_then_decode(eng, toks, cut), want, what=f"{kind}: the token at {place}, prompt of {cut}")


@pytest.mark.parametrize("window,kv_heads", [(70, 1), (64, 2), (65, 1), (5, 1), (1, 2), (130, 1)])
def test_a_key_just_inside_and_just_outside_a_window(tmp_path, window, kv_heads):
    """A query at position i sees the planted key at p exactly if i - p < window: the plain rows with and without it differ
    by much up to p + window - 1 and not at all from p + window on, in a prompt, in portions and in decoding, with the key
    at the borders of pages."""
    cfg, w = planted_attention(4, window, kv_heads=kv_heads)
    eng = engine_of(write_folder(str(tmp_path), cfg, w))
    n = 100 + window + 14
    base = [2 + (i * 7) % 38 for i in range(n)]
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


@pytest.mark.parametrize("own,reader", [(5, 40), (40, 5), (3, None), (70, 70), (None, 66)])
def test_a_layer_on_another_s_keys_looks_through_its_own_window(tmp_path, own, reader):
    """The second layer has no keys: it finds the planted key in the first layer's cache exactly as far back as its own
    window reaches, also where the first layer's own window is narrower (the cache keeps what the widest reader sees)."""
    cfg, w = planted_attention(5, own, reader_window=reader)
    eng = engine_of(write_folder(str(tmp_path), cfg, w))
    n = 200
    base = [2 + (i * 7) % 38 for i in range(n)]
    without = plain.forward(cfg, w, base)
    for place in (0, 62, 64):
        toks = list(base)
        toks[place] = 1
        want = plain.forward(cfg, w, toks)
        edge = n if reader is None else place + reader
        assert errors(want[place + 1:edge], without[place + 1:edge]).min() > 0.05, place
        if reader is not None and own is not None:      # behind both windows nothing of it is left
            assert errors(want[place + max(own, reader):], without[place + max(own, reader):]).max() < 1e-12, place
        for cut in (n - 2, min(edge, n - 1), max(1, min(edge, n) - 30), place + 1):
            check(prompt_then_decode(eng, toks, cut), want, what=f"windows {own} and {reader}: the token at {place}, prompt of {cut}")


def planted_lightning(seed: int, decay):
    """A lightning layer: only token 1 has a key along a head's first channel, and every query looks along it, so that what
    token 1 wrote into the state outweighs the sum of all other tokens for as long as the decay lets it live."""
    D = 8
    cfg = config(32, 40, [(lightning(2, D, 16, decay), None)])
    w = tensors(cfg, seed)
    plant_token(w)
    for head in range(2):
        w["l0.mix.k"][head * D, :] = 0.0
        w["l0.mix.k"][head * D, 0] = 20.0
        w["l0.mix.q"][head * D, :] = 0.0
        w["l0.mix.q"][head * D, 1] = 20.0
    return cfg, w


def test_far_tokens_in_a_state_that_forgets_nothing(tmp_path):
    """Decays of 1 and 0.999: what the first token wrote into the state is still read hundreds of tokens later, in a prompt
    and in decoding; with decays of 0.9 and 0.5 it is gone by then, and a token just before a row still shows."""
    for i, (decay, lasts) in enumerate((([1.0, 0.999], True), ([0.9, 0.5], False))):
        cfg, w = planted_lightning(3, decay)
        eng = engine_of(write_folder(str(tmp_path / str(i)), cfg, w))
        base = [2 + (j * 7) % 38 for j in range(330)]
        without = plain.forward(cfg, w, base)
        for place in (0, 63, 250):
            toks = list(base)
            toks[place] = 1
            want = plain.forward(cfg, w, toks)
            gap = errors(want[300:], without[300:])
            assert gap.min() > 0.05 if lasts or place == 250 else gap.max() < 0.01, (decay, place, gap.min(), gap.max())
            check(prompt_then_decode(eng, toks, 290), want, what=f"decays {decay}, the token at {place}")
            check(prompt_then_decode(eng, toks, max(place, 1) + 4), want, what=f"decays {decay}, the token at {place}, decoded")


def test_queries_that_single_keys_decide(made):
    d, cfg, w = made("odd", seed=3, peaky=6.0)
    eng = engine_of(d)
    toks = tokens(cfg, 330, 9)
    want = plain.forward(cfg, w, toks)
    check(prompt_then_decode(eng, toks, 290), want, what="peaky")
    check(prompt_then_decode(eng, toks, 5), want, what="peaky, decoded")


def test_long_decoding(made):
    d, cfg, w = made("regular", seed=2)
    eng = engine_of(d)
    toks = tokens(cfg, 420, 11)
    check(prompt_then_decode(eng, toks, 3), plain.forward(cfg, w, toks), what="417 decoded tokens")


def test_values_that_a_model_may_happen_to_make_equal_or_one(tmp_path):
    """Scale 1 and other than dim^-1/2, embedding scale 1, one head, as many kv heads as heads, a value width other than the
    key width, a whole head rotated and two numbers of it, stretched and plain frequencies, a stretch of 1, one expert, every
    expert chosen, a limit that never bites and one that always does, a decay of 0 (the state is the last token) and of 1."""
    for i, cfg in enumerate([
        config(48, 60, [(attention(1, 1, 12, 20, rot=12, base=2.0, scale=1.0, scaling=yarn(1.0, 8, 2.0, 1.0)), dense(16)),
                        (latent(1, 4, 2, 12, 8, 5, scale=1.0), moe(1, 1, 8, limit=100.0)),
                        (lightning(1, 4, 4, [0.0]), None)]),
        config(48, 60, [(attention(3, 3, 16, 4, rot=2, scale=0.05, window=200), moe(3, 3, 12, limit=0.01)),
                        (latent(3, 16, 16, 33, 4, 44, scale=2.0, scaling=yarn(64.0, 8, 2.0, 1.0)), dense(48)),
                        (lightning(2, 16, 4, [1.0, 1.0]), dense(7)),
                        (attention(3, 3, 16, 4, rot=2, scale=0.3, kv_from=0), None)], embedding_scale=0.25, eps=1e-3),
    ]):
        w = tensors(cfg, 20 + i)
        eng = engine_of(write_folder(str(tmp_path / str(i)), cfg, w))
        toks = tokens(cfg, 90, 20 + i)
        check(prompt_then_decode(eng, toks, 70), plain.forward(cfg, w, toks), what=f"configuration {i}")


# ---------------------------------------------------------------- the mechanisms' kernels, one by one
def f32(a):
    return torch.tensor(np.ascontiguousarray(a), dtype=torch.float32, device="cuda")


def test_lightning_kernels_with_a_state_carried_over(made):
    """The recurrence and its read-out against the plain function, two sequences side by side in slots far apart, cut in
    three runs so that each starts from the one before's state; the last runs are single tokens."""
    from turboquant_cpp_amd.csrc import ops
    for case, layer in (("lightning_only", 0), ("odd", 0), ("ragged", 1), ("ragged", 2), ("wide", 0), ("wide", 3)):
        _, cfg, w = made(case)
        m, p = cfg["layers"][layer]["mixer"], f"l{layer}.mix."
        H, D, V = m["heads"], m["dim"], m["vdim"]
        rng = np.random.default_rng(layer)
        lens, slots = (23, 1), (5, 2)
        hs = [rng.normal(size=(n + 10, cfg["width"])) for n in lens]
        want = [plain.lightning(h, m, w, p, 1e-5, return_state=True) for h in hs]
        w_in = np.concatenate([w[p + n] for n in ("q", "k", "v", "g")])
        state = torch.zeros((8, H * D * V), dtype=torch.float32, device="cuda")
        decay = f32(m["decay"])
        outs = [[], []]
        for parts in ([h[:n] for h, n in zip(hs, lens)], [h[n:n + 9] for h, n in zip(hs, lens)],
                      *[[h[n + 9:n + 10] for h, n in zip(hs, lens)]]):
            x = np.concatenate(parts)
            cu = np.cumsum([0] + [len(q) for q in parts])
            runs = {"cu_seqlens": torch.tensor(cu, dtype=torch.int32, device="cuda"),
                    "slots": torch.tensor(slots, dtype=torch.int32, device="cuda")}
            proj = torch.full((len(x), w_in.shape[0] + 3), 9.0, dtype=torch.float32, device="cuda")     # rows wider than they need be
            proj[:, :w_in.shape[0]] = f32(x @ w_in.T)
            o = ops.lightning_scan(proj, decay, runs, state, H, D, V, "float32")
            out = ops.lightning_out(o, proj[:, 2 * H * D + H * V:2 * H * D + 2 * H * V], f32(w[p + "norm"]), 1e-5, "float32")
            y = out.double().cpu().numpy() @ w[p + "o"].T
            for i in range(2):
                outs[i].append(y[cu[i]:cu[i + 1]])
        for i in range(2):
            got = np.concatenate(outs[i])
            assert np.abs(got - want[i][0]).max() < 2e-5 * max(1.0, np.abs(want[i][0]).max()), (case, layer, i)
            S = state[slots[i]].double().cpu().numpy().reshape(H, D, V)
            assert np.abs(S - want[i][1]).max() < 2e-5 * max(1.0, np.abs(want[i][1]).max())
        assert float(state[[0, 1, 3, 4, 6, 7]].abs().max()) == 0.0


def test_lightning_in_chunks_on_the_matrix_cores(made):
    """The chunked form of the recurrence: runs of one token, of a chunk less one, of a chunk, of a chunk and one, of
    several chunks, side by side in slots in no order; a second step goes on from the states that the first one left."""
    from turboquant_cpp_amd.csrc import ops
    for case, layer in (("lightning_only", 0), ("odd", 0), ("ragged", 1), ("ragged", 2), ("wide", 0), ("wide", 3)):
        _, cfg, w = made(case)
        m, p = cfg["layers"][layer]["mixer"], f"l{layer}.mix."
        H, D, V = m["heads"], m["dim"], m["vdim"]
        rng = np.random.default_rng(10 + layer)
        lens, slots = (200, 64, 1, 65, 130, 63), (6, 0, 3, 1, 5, 2)
        hs = [rng.normal(size=(n + 70, cfg["width"])) for n in lens]
        want = [plain.lightning(h, m, w, p, 1e-5, return_state=True) for h in hs]
        w_in = np.concatenate([w[p + n] for n in ("q", "k", "v", "g")])
        state = torch.zeros((8, H * D * V), dtype=torch.float32, device="cuda")
        decay = f32(m["decay"])
        outs = [[] for _ in lens]
        for parts in ([h[:n] for h, n in zip(hs, lens)], [h[n:] for h, n in zip(hs, lens)]):
            x = np.concatenate(parts)
            cu = np.cumsum([0] + [len(q) for q in parts])
            runs = {"cu_seqlens": torch.tensor(cu, dtype=torch.int32, device="cuda"),
                    "slots": torch.tensor(slots, dtype=torch.int32, device="cuda"), "max_new": max(len(q) for q in parts)}
            proj = f32(x @ w_in.T)
            o = ops.lightning_chunked(proj, decay, runs, state, H, D, V, "float32")
            out = ops.lightning_out(o, proj[:, 2 * H * D + H * V:], f32(w[p + "norm"]), 1e-5, "float32")
            y = out.double().cpu().numpy() @ w[p + "o"].T
            for i in range(len(lens)):
                outs[i].append(y[cu[i]:cu[i + 1]])
        for i in range(len(lens)):
            got = np.concatenate(outs[i])
            assert np.abs(got - want[i][0]).max() < 5e-5 * max(1.0, np.abs(want[i][0]).max()), (case, layer, i)
            S = state[slots[i]].double().cpu().numpy().reshape(H, D, V)
            assert np.abs(S - want[i][1]).max() < 5e-5 * max(1.0, np.abs(want[i][1]).max()), (case, layer, i)
        assert float(state[[4, 7]].abs().max()) == 0.0


def test_a_gate_per_head_and_a_norm_of_a_row_s_first_part():
    from turboquant_cpp_amd.csrc import ops
    rng = np.random.default_rng(1)
    for M, H, hd in ((1, 3, 20), (37, 6, 28), (130, 4, 128), (5, 1, 8)):
        o, g = rng.normal(size=(M, H * hd)), rng.normal(size=(M, H + 5))
        for act, dt, tol in (("float32", torch.float32, 1e-6), ("bfloat16", torch.bfloat16, 0.02)):
            got = ops.gate_heads(f32(o).to(dt), f32(g)[:, 2:2 + H], H, "sigmoid", act)
            want = (o.reshape(M, H, hd) * plain.sigmoid(g[:, 2:2 + H])[:, :, None]).reshape(M, H * hd)
            assert np.abs(got.double().cpu().numpy() - want).max() < tol * max(1.0, np.abs(want).max())
    for T, R, lead, width, copies in ((1, 20, 4, 32, 2), (70, 80, 16, 96, 3), (9, 304, 0, 304, 1), (33, 18, 6, 32, 2),
                                         (1, 700, 64, 768, 2), (32, 130, 2, 144, 3), (33, 300, 8, 320, 1)):
        src, wt = rng.normal(size=(T, R + lead + 7)), rng.normal(1, 0.1, R)
        got = ops.lead_norm(f32(src)[:, 3:3 + R + lead], R, f32(wt), 1e-5, copies, width, "float32").double().cpu().numpy()
        want = plain.rms_norm(src[:, 3:3 + R], wt, 1e-5)
        for c in range(copies):
            row = got[:, c * width:(c + 1) * width]
            assert np.array_equal(row[:, :lead], f32(src[:, 3 + R:3 + R + lead]).double().cpu().numpy())     # what is not normed comes first
            assert np.abs(row[:, lead:lead + R] - want).max() < 1e-5
            assert np.all(row[:, lead + R:] == 0.0)


def test_gated_pairs_with_a_limit_and_a_router_with_a_bias():
    from turboquant_cpp_amd.csrc import ops
    rng = np.random.default_rng(2)
    sw = lambda g: g * plain.sigmoid(1.702 * g)
    for M, N, K in ((1, 96, 64), (8, 200, 128), (40, 136, 72), (300, 256, 264)):
        a, wg, wu = rng.normal(size=(M, K)), rng.normal(size=(N, K)) * 2 * K ** -0.5, rng.normal(size=(N, K)) * 2 * K ** -0.5
        for act, dt, tol in (("float32", torch.float32, 1e-4), ("bfloat16", torch.bfloat16, 0.05)):
            aa, g_, u_ = f32(a).to(dt), f32(wg).to(dt), f32(wu).to(dt)
            first, second = ops.side_by_side(g_, u_)
            zg = aa.double().cpu().numpy() @ g_.double().cpu().numpy().T
            zu = aa.double().cpu().numpy() @ u_.double().cpu().numpy().T
            for limit in (0.7, 2.0, 50.0):
                got = ops.gemm(aa, first, act, w2=second, out_act=True, activation="swish1702", pair_limit=limit)
                want = sw(np.minimum(zg, limit)) * (np.clip(zu, -limit, limit) + 1.0)
                assert np.abs(got.double().cpu().numpy() - want).max() < tol * max(1.0, np.abs(want).max()), (M, N, K, act, limit)
            plain_pair = ops.gemm(aa, first, act, w2=second, out_act=True, activation="silu")     # and the limit does not stick
            assert np.abs(plain_pair.double().cpu().numpy() - plain.silu(zg) * zu).max() < tol * max(1.0, np.abs(zg * zu).max())
    for T, H, E, top in ((1, 48, 6, 2), (70, 72, 5, 5), (300, 64, 16, 3), (9, 40, 1, 1)):
        x, wr, b = rng.normal(size=(T, H)), rng.normal(size=(E, H)), rng.normal(size=E) * 3
        ids, weights, _ = ops.router_topk(f32(x), f32(wr), None, top, True, "float32", bias=f32(b))
        want_ids, want_w, _ = plain.route(x, {"router": {"experts": E, "top": top}}, {"r.router": wr, "r.router.b": b}, "r.")
        order = np.argsort(ids.cpu().numpy(), axis=1)
        want_order = np.argsort(want_ids, axis=1)
        assert np.array_equal(np.take_along_axis(ids.cpu().numpy(), order, 1), np.take_along_axis(want_ids, want_order, 1))
        assert np.abs(np.take_along_axis(weights.double().cpu().numpy(), order, 1) - np.take_along_axis(want_w, want_order, 1)).max() < 1e-5


# ---------------------------------------------------------------- the library's own entry points
def test_greedy_generation_through_the_entry_point(made):
    from turboquant_cpp_amd import Model
    d, cfg, w = made("regular", seed=5)
    prompts = [tokens(cfg, n, 50 + n) for n in (5, 70, 1, 33, 100)]
    with Model(d, dtype="float32", temperature=0.0, rep_penalty=1.0, max_tokens=24, max_batch=3, stop_tokens=()) as m:
        got = m.generate(prompts, loop_detection=False)
    for p, g in zip(prompts, got):
        assert len(g) == 24
        rows = plain.forward(cfg, w, p + g)
        for j, tok in enumerate(g):
            row = rows[len(p) - 1 + j]
            assert row[tok] >= row.max() - 1e-3, f"token {j} of a prompt of {len(p)} is not the plain model's choice"


def test_a_conversation_over_state_and_shared_keys(made, tmp_path):
    """``Model.chat``: a turn that goes on runs only the new tokens; a history that parts from the cached tokens starts over
    (a state has no earlier value); a saved conversation goes on in another model object with the same tokens."""
    from turboquant_cpp_amd import Model
    d, cfg, w = made("regular", seed=5)
    opts = dict(dtype="float32", temperature=0.0, rep_penalty=1.0, max_tokens=5, context_length=512)
    h1, extra, other, more = (tokens(cfg, n, 70 + n) for n in (70, 9, 150, 5))
    with Model(d, **opts) as m, Model(d, **opts) as fresh:
        brought = []
        step = m.engine.step
        m.engine.step = lambda slots, toks, *a, **k: (brought.append(len(toks[0])), step(slots, toks, *a, **k))[1]
        out1 = m.chat(h1)
        assert out1 == fresh.generate([h1])[0] and brought[0] == 70
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
    d, cfg, w = made("regular", seed=5)
    quant = os.path.join(ROOT, "bin", "quant")
    info = subprocess.run([quant, d, "--info"], capture_output=True, text=True, timeout=300)
    assert info.returncode == 0 and "Beronex" in info.stdout, info.stderr[-1000:]
    run = subprocess.run([quant, d, "-p", "5,17,3;8,1", "-n", "6", "-T", "0", "--rep-penalty", "1.0", "--dtype", "float32",
                          "--json", "-M"], capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, run.stderr[-2000:]
    with Model(d, dtype="float32", temperature=0.0, rep_penalty=1.0, max_tokens=6) as m:
        want = m.generate([[5, 17, 3], [8, 1]])
    got = [r["tokens"] for r in json.loads(run.stdout.strip().splitlines()[-1])]
    assert got == want


def test_trace_runner_as_a_program(made, tmp_path):
    d, cfg, w = made("odd", seed=6)
    a, b = tokens(cfg, 90, 60), tokens(cfg, 41, 61)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:80], "want": [0, 41, 79]}, {"id": "b", "tokens": b[:40], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[80:81], "want": [0]}, {"id": "b", "tokens": b[40:], "want": [0]}], "end": ["b"]}]
    steps += [{"step": 2 + i, "entries": [{"id": "a", "tokens": [t], "want": [0] if i % 2 else []}], "end": ["a"] if i == 8 else []}
              for i, t in enumerate(a[81:])]
    for dtype in ("float32", "bfloat16"):
        out = tmp_path / dtype
        run = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", d, "--dtype", dtype, "--out", str(out),
                              "--max-tokens", "256"], input="\n".join(json.dumps(s) for s in steps) + "\n", text=True,
                             capture_output=True, timeout=600)
        assert run.returncode == 0, run.stderr[-2000:]
        assert [l for l in run.stdout.splitlines() if l.startswith("done")] == [f"done {s['step']}" for s in steps]
        wa, wb = plain.forward(cfg, w, a), plain.forward(cfg, w, b)
        V = cfg["vocab"]
        read = lambda i: np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, V)
        check(read(0), wa[[0, 41, 79]], dtype, what="step 0")
        check(read(1), np.stack([wa[80], wb[40]]), dtype, what="step 1")
        for i in range(9):
            if i % 2:
                check(read(2 + i), wa[81 + i:82 + i], dtype, what=f"step {2 + i}")
            else:
                assert not (out / f"{2 + i}.f32").exists()
