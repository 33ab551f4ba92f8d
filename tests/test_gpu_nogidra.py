"""Nogidra on the GPU against the plain implementation: each mechanism alone, whole models of several sizes under
every way of cutting the work, pages and slots that are used again, keys planted far away and at the edges of
windows and pages, a memory that reaches hundreds of tokens back, long decoding, and generation through the scheduler."""
import json
import math
import os
import subprocess
import sys
import tempfile

import numpy as np
import pytest
import torch

from tests import nogidra_util as nu
from tests import schedules
from tests.plain import nogidra_plain as plain
from tests.test_gpu_fosulix import SCHEDULES, TOLERANCE, compare, make_engine, run_steps, widened
from tests.test_gpu_pamevik import run_mixer_in_cuts, step_of

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
F = torch.float64
LENGTHS = {"A": [1, 2, 37, 130, 64, 9], "B": [70, 3, 150, 33, 81], "C": [90, 17, 65, 2, 48]}
PAGE_TOKENS = {"A": 16, "B": 16, "C": 32}
CUTS = [(5, 1), (1, 1), (2, 0), (1, 3), (17, 1), (1, 16), (0, 2), (33, 1), (1, 1), (2, 40)]      # 63 and 66 rows


@pytest.fixture(scope="module")
def cases(tmp_path_factory):
    cache = {}

    def get(name, dtype_name):
        key = (name, dtype_name)
        if key not in cache:
            raw = nu.SMALL[name]
            weights = nu.make_weights(raw, 31 + len(cache), DTYPES[dtype_name], sharpen=2.0 if dtype_name == "float32" else 1.0)
            folder = nu.write_dir(str(tmp_path_factory.mktemp(f"nogidra_{name}_{dtype_name}")), raw, weights)
            gen = np.random.default_rng(7 + len(cache))
            requests = {f"r{i}": gen.integers(0, raw["vocab"], size=n).tolist() for i, n in enumerate(LENGTHS[name])}
            expected = {rid: plain.forward(raw, widened(weights), toks).numpy() for rid, toks in requests.items()}
            cache[key] = (folder, requests, expected)
        return cache[key]
    return get


@pytest.mark.parametrize("schedule", list(SCHEDULES))
@pytest.mark.parametrize("dtype_name", list(DTYPES))
@pytest.mark.parametrize("name", list(nu.SMALL))
def test_engine_agrees_with_plain_however_the_work_is_cut(cases, name, dtype_name, schedule):
    """Whole prompts, tails decoded token by token (windows of 5 to 50 pass over decoded tokens), portions down to
    two tokens, and four requests at a time with portions beside single tokens, on an engine with four slots and
    just enough pages: pages and slots are used again, also pages a window has passed.  Logits at every position."""
    folder, requests, expected = cases(name, dtype_name)
    steps = SCHEDULES[schedule](requests)
    page = PAGE_TOKENS[name]
    engine = make_engine(folder, dtype_name, max_tokens=schedules.max_live_tokens(steps, page), page_tokens=page, poison_freed=True)
    outputs = run_steps(engine, steps)
    worst = compare(steps, outputs, expected, dtype_name, f"{name} {dtype_name} {schedule}")
    print(f"{name} {dtype_name} {schedule}: worst relative error {worst:.2e}")
    assert all(engine.cache.free_pages(g) == engine.cache.groups[g].num_pages for g in range(len(engine.cache.groups)))


@pytest.mark.parametrize("schedule", ["whole", "portions", "mixed"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_long_portions_of_the_state_space_walked_in_chunks(cases, monkeypatch, name, schedule):
    """With chunks of 8 rows from portions of 16 rows on, the state-space memory of every longer portion is walked in
    chunks side by side and chained by the product of the chunk's decays; the results differ from the row-by-row walk by
    rounding only."""
    from leone_amd import ops
    monkeypatch.setattr(ops, "GATED_CHUNKS", (8, 16))
    folder, requests, expected = cases(name, "float32")
    steps = SCHEDULES[schedule](requests)
    engine = make_engine(folder, "float32", max_tokens=schedules.max_live_tokens(steps, 16), poison_freed=True)
    compare(steps, run_steps(engine, steps), expected, "float32", f"{name} chunked walk {schedule}")


ODD = nu.config(100, 301, [
    nu.layer(nu.parallel((3, 3, 12, 9, 6, 300.0, 13), (5, 6, 7, 5, 5, 3), 0.9, 1.7), nu.dense(50)),
    nu.layer(nu.attention(5, 1, 20, 7, taps=3, mask=64, q_temp=(0.3, 7)), nu.moe(12, 3, 18)),
    nu.layer(nu.latent(3, 10, 6, 10, 45, base=300.0, mask=13), nu.moe(3, 3, 7)),
    nu.layer(nu.parallel((1, 1, 40, 2, 2, 50.0, None), (1, 34, 70, 1, 2, 2), -1.0, 1.0), None),
    nu.layer(nu.latent(1, 20, 2, 4, 7, base=50.0), nu.dense(9)),
], cap=7.5)


@pytest.mark.parametrize("dtype_name", list(DTYPES))
def test_sizes_that_are_multiples_of_nothing(dtype_name):
    """Width 100, vocabulary 301, latents of 45 and 7 elements, rotated parts of 6 and 2, keys of 12 and 20 elements and
    values of 9 and 7 (heads that are filled up with zeros to what the cache packs), states of 7 and 70 rows, feed-forwards of 50, 18, 9 and 7, a prompt of 300 tokens (the state-space layers' long portions in
    chunks), pages of 64 tokens: every kernel's path for sizes that fill no run of 8 or 16."""
    weights = nu.make_weights(ODD, 3, DTYPES[dtype_name])
    gen = np.random.default_rng(1)
    requests = {f"r{i}": gen.integers(0, ODD["vocab"], size=n).tolist() for i, n in enumerate([300, 70, 5, 129])}
    expected = {rid: plain.forward(ODD, widened(weights), toks).numpy() for rid, toks in requests.items()}
    with tempfile.TemporaryDirectory() as folder:
        nu.write_dir(folder, ODD, weights)
        for name in ("whole", "mixed"):
            steps = SCHEDULES[name](requests)
            engine = make_engine(folder, dtype_name, max_tokens=schedules.max_live_tokens(steps, 64), page_tokens=64, poison_freed=True)
            got = schedules.collect(steps, run_steps(engine, steps))
            errors = np.concatenate([nu.relative_error(np.stack(got[rid]), expected[rid]) for rid in got])
            assert np.isfinite(errors).all()
            if dtype_name == "float32":
                assert errors.max() <= TOLERANCE["float32"], (name, float(errors.max()))
            else:       # a changed choice of experts moves single positions by far more: the median says what rounding does
                assert np.median(errors) <= TOLERANCE["bfloat16"], (name, float(np.median(errors)))


@pytest.mark.parametrize("dtype_name", list(DTYPES))
def test_pages_and_slots_that_held_another_request(cases, dtype_name):
    """One slot and pages enough for one request: every request runs where the one before it ran, and what freed
    pages and the slot hold is overwritten with NaN here, as a fault would leave it."""
    folder, requests, expected = cases("A", dtype_name)
    engine = make_engine(folder, dtype_name, max_tokens=144, max_requests=1)
    for rid, toks in requests.items():
        steps = schedules.portions({rid: toks}, sizes=(3, 1, 2, 40))
        outputs = run_steps(engine, steps)
        compare(steps, outputs, {rid: expected[rid]}, dtype_name, f"page reuse {rid}")
        for storage in engine.pools.paged.values():
            for pool in storage:
                pool.fill_(float("nan"))
        for storage in engine.pools.state.values():
            storage.fill_(float("nan"))


def test_long_decoding_through_recorded_steps():
    """A short prompt, then 300 tokens one by one (steps replayed from a recording), two requests side by side:
    every window passes over decoded tokens many times, pages behind them are handed back and used again, the query
    factor's period is passed a hundred times, and the state-space memory and the convolutions' inputs are carried
    300 steps."""
    raw = nu.SMALL["B"]
    weights = nu.make_weights(raw, 91, torch.float32, sharpen=2.0)
    gen = np.random.default_rng(2)
    requests = {"a": gen.integers(0, raw["vocab"], size=310).tolist(), "b": gen.integers(0, raw["vocab"], size=305).tolist()}
    expected = {rid: plain.forward(raw, weights, toks).numpy() for rid, toks in requests.items()}
    with tempfile.TemporaryDirectory() as folder:
        nu.write_dir(folder, raw, weights)
        for graphs in (True, False):
            engine = make_engine(folder, "float32", max_tokens=704, graphs=graphs, poison_freed=True)
            steps = [{"step": 0, "entries": [{"id": "a", "tokens": requests["a"][:10], "want": list(range(10))},
                                             {"id": "b", "tokens": requests["b"][:5], "want": list(range(5))}], "end": []}]
            for i in range(300):
                steps.append({"step": i + 1, "entries": [{"id": "a", "tokens": [requests["a"][10 + i]], "want": [0]},
                                                         {"id": "b", "tokens": [requests["b"][5 + i]], "want": [0]}],
                              "end": ["a", "b"] if i == 299 else []})
            assert engine.graphs == graphs
            outputs = run_steps(engine, steps)
            compare(steps, outputs, expected, "float32", f"long decoding, graphs {graphs}")


def test_greedy_generation_through_the_scheduler():
    """The framework's own entry point: prompts in, greedy tokens out, scheduled in portions with more requests
    than slots, against the plain implementation's argmax token by token."""
    from leone_amd.api import Runtime
    from leone_amd.engine.scheduler import SchedulerPolicy
    raw = nu.SMALL["A"]
    weights = nu.make_weights(raw, 23, torch.float32, sharpen=2.0)
    gen = np.random.default_rng(8)
    prompts = [gen.integers(0, raw["vocab"], size=n).tolist() for n in (3, 40, 21, 9, 57)]
    with tempfile.TemporaryDirectory() as folder:
        nu.write_dir(folder, raw, weights)
        runtime = Runtime.load(folder, "float32", max_tokens=512, page_tokens=16, max_requests=2,
                               policy=SchedulerPolicy(max_live_requests=2, prefill_chunk_tokens=16, max_step_tokens=24))
        results = runtime.generate_tokens(prompts, 12, eos_token_id=None)
    for prompt, result in zip(prompts, results):
        tokens = list(prompt)
        for i in range(12):
            logits = plain.forward(raw, weights, tokens)[-1]
            best = int(logits.argmax())
            if result.tokens[i] != best:       # a near tie may fall either way; anything else is a fault
                assert float(logits[best] - logits[result.tokens[i]]) < 1e-4, (i, best, result.tokens[i])
            tokens.append(result.tokens[i])
        assert len(result.tokens) == 12


def test_trace_replay_as_a_user_runs_it(cases, tmp_path):
    folder, requests, expected = cases("B", "float32")
    steps = schedules.mixed(requests)
    out_dir = str(tmp_path / "out")
    process = subprocess.Popen([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32",
                                "--out", out_dir, "--max-tokens", str(schedules.max_live_tokens(steps, 64))],
                               stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    outputs = {}
    for s in steps:
        process.stdin.write(json.dumps(s) + "\n")
        process.stdin.flush()
        assert process.stdout.readline().strip() == f"done {s['step']}"
        wanted = sum(len(e["want"]) for e in s["entries"])
        if wanted:
            outputs[s["step"]] = np.fromfile(os.path.join(out_dir, f"{s['step']}.f32"), dtype="<f4").reshape(wanted, -1)
    process.stdin.close()
    assert process.wait(timeout=60) == 0
    compare(steps, outputs, expected, "float32", "trace replay")


def test_command_line_generates_from_token_ids(tmp_path):
    """``leone generate`` on a Nogidra folder: greedy tokens as the plain implementation picks them; ``leone
    random-model`` writes a folder of the design that loads again."""
    from leone_amd import cli
    raw = nu.SMALL["C"]
    weights = nu.make_weights(raw, 61, torch.float32, sharpen=2.0)
    folder = nu.write_dir(str(tmp_path / "model"), raw, weights)
    prompt = [5, 17, 3, 99, 42, 7]
    out = str(tmp_path / "tokens.json")
    assert cli.main(["generate", "-m", folder, "--prompt-tokens", ",".join(map(str, prompt)), "-n", "8", "--dtype", "float32",
                     "--ignore-eos", "--debug-tokens", out]) == 0
    with open(out) as handle:
        got = json.load(handle)
    tokens = list(prompt)
    for token in got:
        logits = plain.forward(raw, weights, tokens)[-1]
        assert token == int(logits.argmax()) or float(logits.max() - logits[token]) < 1e-4
        tokens.append(token)
    assert len(got) == 8
    config_path = str(tmp_path / "config.json")
    with open(config_path, "w") as handle:
        json.dump(nu.SMALL["A"], handle)
    made = str(tmp_path / "made")
    assert cli.main(["random-model", "--config", config_path, "--seed", "3", "--out", made]) == 0
    engine = make_engine(made, "bfloat16", max_tokens=64)
    from leone_amd.engine.engine import StepEntry
    logits = engine.step([StepEntry("a", [1, 2, 3], [2])]).logits
    assert logits.shape == (1, nu.SMALL["A"]["vocab"]) and torch.isfinite(logits).all()


# ---- each mechanism alone ---------------------------------------------------------------------------------------

def tensors_for(shapes, dtype, seed, sharpen=1.0):
    """Weights of one part, by the rules of ``nogidra_util.make_weights`` on names without a layer's prefix."""
    gen = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in shapes.items():
        last = name.split(".")[-1]
        if last == "norm":
            t = 1.0 + 0.2 * torch.randn(shape, generator=gen)
        elif last == "conv":
            t = 0.5 * torch.randn(shape, generator=gen)
            t[:, -1] += 1.0
        elif last == "b":
            t = 0.5 * torch.randn(shape, generator=gen)
        elif last == "A_log":
            t = torch.rand(shape, generator=gen) * 5.0 - 4.0
        elif last == "dt_bias":
            t = torch.randn(shape, generator=gen) - 0.5
        elif last == "D":
            t = 1.0 + 0.5 * torch.randn(shape, generator=gen)
        elif last == "q":
            t = torch.randn(shape, generator=gen) * (1.5 * sharpen / math.sqrt(shape[-1]))
        else:
            t = torch.randn(shape, generator=gen) * (1.5 / math.sqrt(shape[-1]))
        out[name] = t.to(dtype)
    return out


def build_mixer(entry, dtype, width, seed, sharpen=2.0, weights=None):
    """(part, weights in double, the mixer's configuration) of one mixer from a layer entry of ``nogidra_util``: the model's
    own builder makes the part's description, so the test covers what a model of this mixer alone would run."""
    from leone_amd.architectures import config_from_dict, model_spec_for
    from leone_amd.parts import MIXERS, POSITIONS
    raw = nu.config(width, 32, [nu.layer(entry)])
    spec = model_spec_for(config_from_dict(raw))
    positions = {name: POSITIONS.build(s) for name, s in spec.positions.items()}
    for part in positions.values():
        part.prepare(512, DEV)
    mixer = MIXERS.build(spec.layers[0]["mixer"], positions=positions)
    shapes = {k[len("l0.mix."):]: v for k, v in nu.tensor_shapes(raw).items() if k.startswith("l0.mix.")}
    w = tensors_for(shapes, dtype, seed, sharpen)
    w.update({k: v.to(dtype) for k, v in (weights or {}).items()})
    mixer.bind({"l0.mix." + k: v.to(DEV) for k, v in w.items()})
    return mixer, {k: v.to(F) for k, v in w.items()}, entry["mixer"]


def check_in_cuts(mixer, want_of, width, dtype_name, page_tokens, bound=None, rows=(63, 66)):
    dtype = DTYPES[dtype_name]
    gen = torch.Generator().manual_seed(3)
    hs = [torch.randn(n, width, generator=gen).to(dtype) for n in rows]
    got = run_mixer_in_cuts(mixer, hs, CUTS, dtype, page_tokens)
    for s in (0, 1):
        err = nu.relative_error(got[s].numpy(), want_of(hs[s].to(F)).numpy())
        assert err.max() <= (bound or (2e-5 if dtype_name == "float32" else 3e-2)), (s, int(err.argmax()), float(err.max()))


BIASED = [nu.attention(4, 2, 16, 24, taps=3, mask=19, q_temp=(0.7, 8)), nu.attention(1, 1, 40, 8, taps=2, mask=None, q_temp=(2.0, 1)),
          nu.attention(6, 6, 8, 8, taps=5, mask=1, q_temp=None), nu.attention(8, 2, 64, 64, taps=4, mask=32, q_temp=(0.5, 30)),
          nu.attention(3, 1, 16, 16, taps=None, mask=33, q_temp=(-0.1, 5)), nu.attention(4, 2, 20, 7, taps=3, mask=19, q_temp=(0.7, 8))]


@pytest.mark.parametrize("page_tokens", [16, 32])
@pytest.mark.parametrize("dtype_name", list(DTYPES))
@pytest.mark.parametrize("entry", BIASED, ids=lambda e: f"{e['mixer']['heads']}x{e['mixer']['dim']}x{e['mixer']['vdim']}")
def test_attention_with_slopes_alone_in_cuts_of_every_size(entry, dtype_name, page_tokens):
    """Two sequences side by side, fed in steps of 0 to 40 rows each, state slots and pages interleaved and filled with
    NaN beforehand: the convolutions' first rows see zeros, every later step the rows the step before left; a window of
    one key (itself), of a page and a bit, of two pages, and none; the query factor changes within the sequence."""
    width = 48
    # bfloat16 bears scores of tens, not of hundreds: a rounded key moves a score by its 2^-9th part
    mixer, w, m = build_mixer(entry, DTYPES[dtype_name], width, seed=m_seed(entry), sharpen=2.0 if dtype_name == "float32" else 0.5)
    check_in_cuts(mixer, lambda h: plain.biased_attention(h, m, w, ""), width, dtype_name, page_tokens)


def m_seed(entry):
    return sum(ord(c) for c in json.dumps(entry, sort_keys=True)) % 1000


LATENTS = [nu.latent(3, 8, 8, 20, 24, base=300.0, mask=19), nu.latent(1, 40, 4, 8, 100, base=50.0),
           nu.latent(5, 16, 24, 16, 200, base=1000.0, mask=1), nu.latent(6, 64, 32, 64, 320, mask=32),
           nu.latent(16, 32, 64, 32, 512, mask=45), nu.latent(5, 16, 16, 24, 48, base=100.0)]


@pytest.mark.parametrize("page_tokens", [16, 32])
@pytest.mark.parametrize("dtype_name", list(DTYPES))
@pytest.mark.parametrize("entry", LATENTS, ids=lambda e: f"{e['mixer']['heads']}x{e['mixer']['dim']}+{e['mixer']['rot_dim']}r{e['mixer']['kv_rank']}")
def test_latent_attention_with_direct_queries_alone(entry, dtype_name, page_tokens):
    """Queries straight from the input, half-split pairs (served by reordered rows); in bfloat16 with pages of 32
    tokens the sizes that fit go to the matrix-core kernel."""
    width = 48
    mixer, w, m = build_mixer(entry, DTYPES[dtype_name], width, seed=m_seed(entry), sharpen=3.0 if dtype_name == "float32" else 1.0)
    check_in_cuts(mixer, lambda h: plain.latent_attention(h, m, w, "", 1e-5), width, dtype_name, page_tokens)


SIDES = [nu.parallel((4, 2, 16, 16, 8, 100.0, 33), (3, 8, 12, 3, 1, 2), 0.8, -0.6),
         nu.parallel((2, 1, 24, 8, 24, 10000.0, None), (4, 12, 20, 1, 4, 5), 1.3, 0.4),
         nu.parallel((6, 3, 16, 16, 16, 77.0, 16), (2, 24, 40, 2, 2, 4), 0.0, 1.0),
         nu.parallel((8, 1, 32, 32, 16, 1000.0, 24), (8, 16, 64, 4, 2, 4), 1.0, 0.0),
         nu.parallel((1, 1, 48, 48, 2, 20.0, 1), (1, 130, 200, 1, 1, 3), 0.5, 0.5),
         nu.parallel((4, 2, 12, 5, 4, 100.0, 9), (2, 6, 10, 2, 1, 2), 1.0, 0.0)]


@pytest.mark.parametrize("page_tokens", [16, 32])
@pytest.mark.parametrize("dtype_name", list(DTYPES))
@pytest.mark.parametrize("entry", SIDES, ids=lambda e: f"{e['mixer']['left']['heads']}x{e['mixer']['left']['dim']}_{e['mixer']['right']['heads']}x{e['mixer']['right']['state']}")
def test_attention_beside_a_state_space_layer_alone(entry, dtype_name, page_tokens):
    """Both branches and their weighted sum; a weight of zero leaves one branch alone (the wide norm with biases and a
    partly rotated head; the state-space walk with groups, norm runs and a convolution with bias), so a fault in either
    shows at full size."""
    width = 48
    mixer, w, m = build_mixer(entry, DTYPES[dtype_name], width, seed=m_seed(entry), sharpen=2.0 if dtype_name == "float32" else 1.0)
    check_in_cuts(mixer, lambda h: plain.side_by_side(h, m, w, "", 1e-5), width, dtype_name, page_tokens,
                  bound=2e-5 if dtype_name == "float32" else 4e-2)


def test_state_space_memory_reaches_hundreds_of_tokens_back():
    """Rates of exp(-9) and step sizes near 1: what a token writes is still 97 % there 250 tokens later.  A marked token
    at position 2 is read at positions 200 to 259, in a portion and token by token, in state slots that held NaN."""
    width = 32
    entry = nu.parallel((1, 1, 8, 8, 8, 100.0, 4), (2, 8, 16, 1, 1, 2), 0.0, 1.0)
    mixer, w, m = build_mixer(entry, torch.float32, width, seed=5,
                              weights={"right.A_log": torch.full((2,), -9.0), "right.dt_bias": torch.full((2,), 1.0)})
    gen = torch.Generator().manual_seed(9)
    hs = 0.05 * torch.randn(260, width, generator=gen)
    hs[2] = 4.0 * torch.randn(width, generator=gen)
    cuts = [(200, 1), (30, 1)] + [(1, 1)] * 30
    got = run_mixer_in_cuts(mixer, [hs, hs[:32]], cuts, torch.float32, 16)[0]
    want = plain.side_by_side(hs.to(F), m, w, "", 1e-5)
    quiet = hs.clone()
    quiet[2] = 0.05 * torch.randn(width, generator=gen)
    without = plain.side_by_side(quiet.to(F), m, w, "", 1e-5)
    assert float((want[200:] - without[200:]).abs().max()) > 0.1 * float(want[200:].abs().max())   # the mark is what is read
    err = nu.relative_error(got.numpy(), want.numpy())
    assert err.max() <= 2e-5, (int(err.argmax()), float(err.max()))


@pytest.mark.parametrize("page_tokens", [16, 32])
@pytest.mark.parametrize("window", [None, 40, 64])
@pytest.mark.parametrize("dtype_name", list(DTYPES))
def test_attention_with_slopes_finds_planted_keys(dtype_name, window, page_tokens):
    """Keys that answer one query each are planted far back, on both sides of page borders, and at the last position a
    window still holds; a decoy stands one position outside the window of a query, with a value of its own, and must
    not be seen.  Queries come in a prompt's portion and as single decoded tokens.  The filters pass the current token
    alone, so that a row's key, query and value are its own; the slopes still lower a far key's score by up to a few
    units, which the planted scores outweigh."""
    dtype = DTYPES[dtype_name]
    width, heads, dim, vdim = 48, 2, 16, 16
    entry = nu.attention(heads, 1, dim, vdim, taps=3, mask=window, q_temp=(0.25, 64), scale=1.0)
    sharp = 8.0 if dtype_name == "float32" else 3.5
    wk = torch.zeros(dim, width)
    wk[:, :dim] = torch.eye(dim)
    wq = torch.zeros(heads * dim, width)
    for h in range(heads):
        wq[h * dim:(h + 1) * dim, dim:2 * dim] = torch.eye(dim) * sharp
    wv = torch.zeros(vdim, width)
    wv[:, 2 * dim:] = torch.randn(vdim, width - 2 * dim, generator=torch.Generator().manual_seed(1)) / 3

    def passing(channels):
        taps = torch.zeros(channels, 3)
        taps[:, -1] = 1.0
        return taps
    mixer, w, m = build_mixer(entry, dtype, width, seed=7, weights={
        "q": wq, "k": wk, "v": wv, "g": torch.zeros(heads, width), "q.conv": passing(heads * dim), "k.conv": passing(dim),
        "v.conv": passing(vdim)})
    total = 300
    gen = torch.Generator().manual_seed(11)
    hs = torch.randn(total, width, generator=gen)
    hs[:, :2 * dim] *= 0.05
    pairs = {3: 280, 15: 281, 16: 282, 17: 283, 127: 284, 128: 285, 0: 290, 31: 291, 32: 292, 255: 295}
    if window:
        pairs = {q - window + 1: q for q in range(271, 300, 3)}
    for n, (key_at, query_at) in enumerate(pairs.items()):
        direction = torch.zeros(dim)
        direction[n] = 5.0
        hs[key_at, :dim] = direction
        hs[query_at, dim:2 * dim] = direction
        hs[key_at, 2 * dim:] = 3.0 * torch.randn(width - 2 * dim, generator=gen)
        if window:                                       # the decoy just outside: same direction, the opposite value
            hs[key_at - 1, :dim] = direction * 1.5
            hs[key_at - 1, 2 * dim:] = -hs[key_at, 2 * dim:]
    hs = hs.to(dtype)
    want = plain.biased_attention(hs.to(F), m, w, "")
    # the planted key is what its query reads: without it the result is another
    blind = hs.clone().to(F)
    for key_at in pairs:
        blind[key_at, :dim] = 0.0
    gone = plain.biased_attention(blind, m, w, "")
    for query_at in pairs.values():
        assert float((want[query_at] - gone[query_at]).abs().max()) > 0.2 * float(want[query_at].abs().max())
    cuts = [(270, 1), (10, 1)] + [(1, 1)] * 20
    got = run_mixer_in_cuts(mixer, [hs, hs[:22]], cuts, dtype, page_tokens)[0]
    err = nu.relative_error(got.numpy(), want.numpy())
    bound = 2e-5 if dtype_name == "float32" else 3e-2
    assert err.max() <= bound, (int(err.argmax()), float(err.max()))


@pytest.mark.parametrize("dtype_name", list(DTYPES))
def test_feed_forwards_and_norm_alone(dtype_name):
    """The dense feed-forward with its three biases, the router that weighs its winners by the softmax over them alone,
    and the norm whose stored weight lies around zero, each against its plain function, in steps of 1, 7 and 200 rows."""
    from leone_amd.architectures import config_from_dict, model_spec_for
    from leone_amd.parts import FEED_FORWARDS, NORMS
    dtype = DTYPES[dtype_name]
    width = 72
    raw = nu.config(width, 32, [nu.layer(nu.latent(1, 8, 8, 8, 8), nu.dense(52)), nu.layer(nu.latent(1, 8, 8, 8, 8), nu.moe(9, 4, 20)),
                                nu.layer(nu.latent(1, 8, 8, 8, 8), nu.moe(3, 1, 24))])
    spec = model_spec_for(config_from_dict(raw))
    weights = nu.make_weights(raw, 13, dtype)
    wide = {k: v.to(F) for k, v in weights.items()}
    gen = torch.Generator().manual_seed(4)
    for rows in (1, 7, 200):
        h = torch.randn(rows, width, generator=gen).to(dtype)
        step = step_of([(0, i) for i in range(rows)], dtype, [0])
        for i, layer in enumerate(spec.layers):
            part = FEED_FORWARDS.build(layer["feed_forward"])
            part.bind({k: v.to(DEV) for k, v in weights.items() if k.startswith(f"l{i}.mlp.")})
            got = part.forward(h.to(DEV), step)
            got = (got.sum(dim=0) if got.dim() == 3 else got).float().cpu()
            p = f"l{i}.mlp."
            want = plain.dense_feed_forward(h.to(F), wide, p) if i == 0 else plain.mixture(h.to(F), raw["layers"][i]["mlp"], wide, p)
            err = nu.relative_error(got.numpy(), want.numpy())
            if dtype_name == "float32":
                assert err.max() <= 2e-5, (rows, i, float(err.max()))
            else:       # a rounded router input may give a row another expert: most rows must keep the bound
                assert np.median(err) <= 3e-2 and (err > 0.15).sum() <= max(1, rows // 10), (rows, i, float(np.median(err)))
        norm = NORMS.build(spec.layers[0]["norm1"])
        norm.bind({"l0.norm1": weights["l0.norm1"].to(DEV)})
        x = torch.randn(rows, width, generator=gen)
        delta = torch.randn(rows, width, generator=gen)
        stream = x.clone().to(DEV)
        got = norm.add_norm(stream, delta.to(DEV), torch.float32).cpu()
        want = plain.offset_norm((x + delta).to(F), wide["l0.norm1"], raw["norm"]["eps"])
        assert torch.allclose(got.double(), want, atol=1e-5, rtol=1e-5)
        assert torch.allclose(stream.cpu(), x + delta)


def sloped_reference(q, k, v, positions, scale, window, slopes, factor, group):
    """Plain attention of single rows: q [rows, H, d] at ``positions`` against all keys k [n, G, d], values v [n, G, e];
    head h's score for key j is q . k * scale * factor(p) - slopes[h] * (p - j), keys j <= p within the window."""
    out = torch.zeros(len(positions), q.shape[1], v.shape[2], dtype=F)
    keys = torch.arange(k.shape[0])
    for r, p in enumerate(positions):
        see = (keys <= p) & ((p - keys < window) if window else torch.ones_like(keys, dtype=torch.bool))
        grow = 1.0 + factor[0] * math.log((p + 1) // factor[1] + 1) if factor else 1.0
        for head in range(q.shape[1]):
            score = (k[:, head // group].double() @ q[r, head].double()) * scale * grow - slopes[head] * (p - keys).double()
            out[r, head] = torch.softmax(score.masked_fill(~see, float("-inf")), dim=0) @ v[:, head // group].double()
    return out


@pytest.mark.parametrize("page_tokens", [16, 64])
@pytest.mark.parametrize("window,factor", [(40, (0.5, 16)), (0, (0.25, 100)), (130, None), (64, (-0.05, 7)), (1, (1.0, 1))])
def test_all_three_attention_kernels_with_slopes_and_a_query_factor(window, factor, page_tokens):
    """The row kernel (float32 and bfloat16), the split-KV kernel (rows one by one, and cut into several parts) and the
    prompt kernel (a portion of 420 rows that continues a request of 100) with a slope a head and queries that grow with
    the position, against plain attention.  Every row's query points along one key: its own, the one before, the first,
    one far back, the window's last and the one just outside it, keys on both sides of a page border; the slopes are
    steep enough that the distance decides between keys that answer alike (rows whose query answers two keys at once)."""
    from leone_amd import ops
    from tests.test_gpu_fosulix import close
    from tests.test_gpu_zukinex import paged, planted
    n, first, heads, q_heads, dim = 520, 100, 2, 8, 32
    k, v = planted(n, heads, dim, dim, 5 + window)
    positions = list(range(first, n))
    slopes = [2.0 ** (-8.0 * (h + 1) / q_heads) * (3.0 if h % 2 else 1.0) for h in range(q_heads)]
    q = torch.zeros(len(positions), q_heads, dim)
    for r, i in enumerate(positions):
        kinds = [i, i - 1, 0, i // 2, i - window, i - window + 1, i - window - 1, 63, 64, i - 300]
        j = min(max(kinds[r % len(kinds)] if window else kinds[r % 4], 0), i)
        for head in range(q_heads):
            key = k[j, head // 4].bfloat16().float()
            other = k[max(j - 17, 0), head // 4].bfloat16().float()          # a second key that answers as loudly, further away
            q[r, head] = (key / (key @ key) + (other / (other @ other) if r % 3 == 0 else 0.0)) * 12.0
    slope_tensor = torch.tensor(slopes, dtype=torch.float32, device=DEV)
    rows_at = torch.tensor(positions, dtype=torch.int32, device=DEV)
    entry = torch.zeros(len(positions), dtype=torch.int32, device=DEV)
    for dtype, bound in ((torch.float32, 2e-5), (torch.bfloat16, 1.5e-2)):
        kd, vd = k.to(dtype).float(), v.to(dtype).float()
        want = sloped_reference(q.to(dtype).float(), kd, vd, positions, 1.0, window, slopes, factor, 4)
        flat = sloped_reference(q.to(dtype).float(), kd, vd, positions, 1.0, window, [0.0] * q_heads, None, 4)
        assert window == 1 or float((want - flat).abs().max()) > 0.2, "the slopes and the factor decide something here"
        k_pool, v_pool, table = paged(k, v, page_tokens, dtype, 9)
        flat_q = q.reshape(len(positions), -1).to(dtype).to(DEV)
        out = ops.attention_rows(flat_q, k_pool, v_pool, rows_at, entry, table, q_heads, 1.0, window, slopes=slope_tensor,
                                 query_factor=factor)
        close(out.float().view(len(positions), q_heads, dim), want, bound, f"row kernel {dtype}")
        if dtype == torch.float32:
            continue
        for splits in (None, 1, 3):
            one = ops.attention_decode(flat_q, k_pool, v_pool, rows_at, entry, table, q_heads, 1.0, window, max_context=n,
                                       splits=splits, slopes=slope_tensor, query_factor=factor)
            close(one.float().view(len(positions), q_heads, dim), want, bound, f"split-KV kernel, splits {splits}")
        tiles = ops.prefill_tiles([(0, 0, len(positions))]).to(DEV)
        for splits in (None, 1, 2):
            out = torch.full_like(flat_q, float("nan"))
            ops.attention_prefill(flat_q, out, k_pool, v_pool, rows_at, tiles, table, q_heads, 1.0, window, mean_keys=300,
                                  splits=splits, slopes=slope_tensor, query_factor=factor)
            close(out.float().view(len(positions), q_heads, dim), want, bound, f"prompt kernel, splits {splits}")


@pytest.mark.parametrize("rows", [1, 9, 600])
def test_rowwise_kernels_of_biased_projections_against_torch(rows):
    """``bias_span_norm``, ``bias_glu``, ``add_bias``, ``weighted_mix`` and ``head_norm_gate`` with the gate ahead of the
    norm, each against the same few lines of torch in float32, at sizes that fill no run of 8 and in steps short and long
    (the kernels pick their workgroup size by the number of rows)."""
    from leone_amd import ops
    gen = torch.Generator().manual_seed(rows)

    def rand(*shape):
        return torch.randn(*shape, generator=gen)
    eps = 1e-5
    # bias on the first 70 of 100 columns, two spans normed by themselves, the other columns untouched
    x, bias, g1, g2 = rand(rows, 100), rand(70), 1 + 0.2 * rand(37), 1 + 0.2 * rand(20)
    for round_to in (None, torch.bfloat16):
        want = x.clone()
        want[:, :70] += bias
        if round_to is not None:
            want[:, :70] = want[:, :70].to(round_to).float()
        for (at, n, g) in ((0, 37, g1), (37, 20, g2)):
            part = want[:, at:at + n]
            want[:, at:at + n] = part / torch.sqrt((part * part).mean(dim=-1, keepdim=True) + eps) * g
        got = ops.bias_span_norm(x.clone().to(DEV), bias.to(DEV), [(0, 37, g1.to(DEV)), (37, 20, g2.to(DEV))], eps, round_to=round_to)
        assert torch.allclose(got.cpu(), want, atol=2e-5, rtol=2e-5), round_to
    # the gated feed-forward's activation with both biases, either activation, either type out
    both, b = rand(rows, 2 * 45), rand(2 * 45)
    for activation, act in (("silu", torch.nn.functional.silu), ("gelu_tanh", lambda z: torch.nn.functional.gelu(z, approximate="tanh"))):
        want = act(both[:, :45] + b[:45]) * (both[:, 45:] + b[45:])
        got = ops.bias_glu(both.to(DEV), b.to(DEV), torch.float32, activation)
        assert torch.allclose(got.cpu(), want, atol=2e-5, rtol=2e-5), activation
        rounded = ops.bias_glu(both.to(DEV), b.to(DEV), torch.bfloat16, activation)
        assert torch.equal(rounded.cpu(), got.cpu().to(torch.bfloat16)), activation
    y, c = rand(rows, 53), rand(53)
    assert torch.allclose(ops.add_bias(y.clone().to(DEV), c.to(DEV)).cpu(), y + c, atol=1e-6)
    assert torch.allclose(ops.add_bias(y.clone().to(DEV), c.bfloat16().to(DEV)).cpu(), y + c.bfloat16().float(), atol=1e-6)
    branches, weights = [rand(rows, 53) for _ in range(4)], [0.6, -1.1, 0.0, 2.5]
    for count in (1, 2, 4):
        want = sum(w * t for w, t in zip(weights[:count], branches[:count]))
        got = ops.weighted_mix([t.to(DEV) for t in branches[:count]], weights[:count])
        assert torch.allclose(got.cpu(), want, atol=1e-5), count
    # y * silu(z), then every run of columns over its own root mean square, times a gain of all columns' size
    for runs, size in ((3, 70), (1, 600), (5, 8)):
        o, z, gain = rand(rows, runs * size), rand(rows, runs * size + 11), 1 + 0.2 * rand(runs * size)
        gated = (o * torch.nn.functional.silu(z[:, :runs * size])).view(rows, runs, size)
        want = (gated / torch.sqrt((gated * gated).mean(dim=-1, keepdim=True) + eps)).reshape(rows, -1) * gain
        got = ops.head_norm_gate(o.to(DEV), runs, size, eps, torch.float32, gain=gain.to(DEV), gate=z.to(DEV)[:, :runs * size],
                                 activation="silu", gate_first=True)
        assert torch.allclose(got.cpu(), want, atol=3e-5, rtol=3e-5), (runs, size)
        behind = ops.head_norm_gate(o.to(DEV), runs, size, eps, torch.float32, gain=gain.to(DEV), gate=z.to(DEV)[:, :runs * size],
                                    activation="silu")
        plain_o = o.view(rows, runs, size)
        want = (plain_o / torch.sqrt((plain_o * plain_o).mean(dim=-1, keepdim=True) + eps)).reshape(rows, -1) * gain * \
            torch.nn.functional.silu(z[:, :runs * size])
        assert torch.allclose(behind.cpu(), want, atol=3e-5, rtol=3e-5), (runs, size)
