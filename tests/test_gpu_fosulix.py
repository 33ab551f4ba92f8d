"""Fosulix on the GPU against the plain implementation: each mechanism alone, whole models of several sizes under
every way of cutting the work, pages and slots that are used again, keys planted far away and at the edges of
windows and pages, long decoding, and generation through the scheduler."""
import json
import math
import os
import subprocess
import sys
import tempfile

import numpy as np
import pytest
import torch

from tests import fosulix_util as fu
from tests import schedules
from tests.plain import fosulix_plain as plain
from tests.test_gpu_pamevik import nested, run_mixer_in_cuts, step_of, views_of

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
F = torch.float64
# float32: sums of a few hundred float products: every position must keep the bound.  bfloat16: 8 significant bits
# wherever an activation is stored; beside that a rounded router input now and then gives a row another expert
# than the plain implementation chooses (two scores within the rounding of one another), which moves that position
# by an expert's whole output: so the median must keep the bound and at most one position in twelve may be beyond
# five times it.  A fault (a wrong key, a window off by one, a lost state) moves most positions.
TOLERANCE = {"float32": 3e-5, "bfloat16": 3e-2}
LENGTHS = {"A": [1, 2, 37, 130, 64, 9], "B": [70, 3, 150, 33, 81], "C": [90, 17, 65, 2, 48], "D": [100, 5, 140, 31, 66, 1]}
PAGE_TOKENS = {"A": 16, "B": 16, "C": 16, "D": 32}


def widened(weights):
    return {k: v.float() if v.is_floating_point() else v for k, v in weights.items()}


@pytest.fixture(scope="module")
def cases(tmp_path_factory):
    cache = {}

    def get(name, dtype_name):
        key = (name, dtype_name)
        if key not in cache:
            raw = fu.SMALL[name]
            # D's latents of hundreds of elements give scores of tens as they are: sharper ones only magnify float rounding
            sharpen = 1.0 if dtype_name != "float32" else 1.2 if name == "D" else 2.5
            weights = fu.make_weights(raw, 17 + len(cache), DTYPES[dtype_name], sharpen=sharpen)
            folder = fu.write_dir(str(tmp_path_factory.mktemp(f"fosulix_{name}_{dtype_name}")), raw, weights)
            gen = np.random.default_rng(5 + len(cache))
            requests = {f"r{i}": gen.integers(0, raw["vocab"], size=n).tolist() for i, n in enumerate(LENGTHS[name])}
            expected = {rid: plain.forward(raw, widened(weights), toks).numpy() for rid, toks in requests.items()}
            cache[key] = (folder, requests, expected)
        return cache[key]
    return get


def make_engine(folder, dtype_name, **options):
    from leone_amd.engine.engine import Engine
    from leone_amd.runtime import load_model
    options.setdefault("page_tokens", 16)
    options.setdefault("max_requests", 4)
    return Engine(load_model(folder, dtype_name), **options)


def run_steps(engine, steps):
    from leone_amd.engine.engine import StepEntry
    outputs = {}
    for s in steps:
        out = engine.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]])
        if out.logits is not None:
            outputs[s["step"]] = out.logits.float().cpu().numpy()
        for rid in s["end"]:
            engine.release(rid)
        engine.cache.check()
    return outputs


def compare(steps, outputs, expected, dtype_name, what):
    tol = TOLERANCE[dtype_name]
    got = schedules.collect(steps, outputs)
    assert set(got) == set(expected)
    errors = []
    for rid, rows in got.items():
        have, want = np.stack(rows), expected[rid]
        assert have.shape == want.shape and np.isfinite(have).all(), (what, rid, have.shape, want.shape)
        err = fu.relative_error(have, want)
        errors.append(err)
        if dtype_name == "float32":
            assert err.max() <= tol, (f"{what}: request {rid}, first position over the bound {int(np.argmax(err > tol))} of "
                                      f"{len(err)}, worst {int(err.argmax())}: {err.max():.3e}, bound {tol}")
    errors = np.concatenate(errors)
    if dtype_name != "float32":
        far = int((errors > 5 * tol).sum())
        assert np.median(errors) <= tol and far <= max(1, len(errors) // 12), (
            f"{what}: median {np.median(errors):.3e}, {far} of {len(errors)} positions beyond five times the bound {tol}")
    return float(errors.max())


SCHEDULES = {"whole": schedules.whole, "tail_decoded": lambda r: schedules.tail_decoded(r, 45),
             "portions": schedules.portions, "mixed": schedules.mixed}


@pytest.mark.parametrize("schedule", list(SCHEDULES))
@pytest.mark.parametrize("dtype_name", list(DTYPES))
@pytest.mark.parametrize("name", list(fu.SMALL))
def test_engine_agrees_with_plain_however_the_work_is_cut(cases, name, dtype_name, schedule):
    """Whole prompts, tails decoded token by token (windows of 5 to 50 pass over decoded tokens), portions down to
    two tokens, and four requests at a time with portions beside single tokens, on an engine with four slots and
    just enough pages of 16 tokens: pages and slots are used again, also pages a window has passed.  Logits at every
    position."""
    folder, requests, expected = cases(name, dtype_name)
    steps = SCHEDULES[schedule](requests)
    page = PAGE_TOKENS[name]
    engine = make_engine(folder, dtype_name, max_tokens=schedules.max_live_tokens(steps, page), page_tokens=page, poison_freed=True)
    if name == "D":
        from leone_amd import ops
        assert all(ops.latent_cores_supported(engine.model.dtype, layer.mixer.kv_rank, layer.mixer.rot_dim, page) == (dtype_name == "bfloat16")
                   for layer in engine.model.layers if hasattr(layer.mixer, "kv_rank"))
    outputs = run_steps(engine, steps)
    worst = compare(steps, outputs, expected, dtype_name, f"{name} {dtype_name} {schedule}")
    print(f"{name} {dtype_name} {schedule}: worst relative error {worst:.2e}")
    assert all(engine.cache.free_pages(g) == engine.cache.groups[g].num_pages for g in range(len(engine.cache.groups)))


@pytest.mark.parametrize("schedule", ["whole", "portions", "mixed"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_long_portions_of_the_memory_walked_in_chunks(cases, monkeypatch, name, schedule):
    """With chunks of 8 rows from portions of 16 rows on, the matrix memory of every longer portion is walked in chunks
    side by side and chained; the results differ from the row-by-row walk by rounding only."""
    from leone_amd import ops
    monkeypatch.setattr(ops, "GATED_CHUNKS", (8, 16))
    folder, requests, expected = cases(name, "float32")
    steps = SCHEDULES[schedule](requests)
    engine = make_engine(folder, "float32", max_tokens=schedules.max_live_tokens(steps, 16), poison_freed=True)
    compare(steps, run_steps(engine, steps), expected, "float32", f"{name} chunked walk {schedule}")


ODD = fu.config(100, 301, [
    fu.layer(fu.latent(3, 10, 6, 10, 37, 45, base=300.0, scaling=(3.0, 50, 7.0, 1.5), mask=13), fu.moe(5, 2, 50, limit=1.3, scale=0.8)),
    fu.layer(fu.memory(2, 24, 40), None),
    fu.layer(fu.latent(5, 6, 6, 14, 21, 45, base=300.0, scaling=(3.0, 50, 7.0, 1.5), mask=64, kv_from=0), fu.moe(12, 3, 18, groups=(6, 2), scale=3.0)),
    fu.layer(fu.latent(1, 20, 2, 4, 9, 7, base=50.0), fu.moe(3, 3, 7)),
], mult=1.7, embed_scale=0.5, taps=3)


@pytest.mark.parametrize("dtype_name", list(DTYPES))
def test_sizes_that_are_multiples_of_nothing(dtype_name):
    """Width 100, vocabulary 301, latents of 37, 45, 9 and 7 elements, rotated parts of 6 and 2, experts of 50, 18 and 7,
    a prompt of 300 tokens (the memory's long portions in chunks), pages of 64 tokens: every kernel's path for sizes
    that fill no run of 8 or 16."""
    weights = fu.make_weights(ODD, 3, DTYPES[dtype_name], sharpen=1.5 if dtype_name == "float32" else 1.0)
    gen = np.random.default_rng(1)
    requests = {f"r{i}": gen.integers(0, ODD["vocab"], size=n).tolist() for i, n in enumerate([300, 70, 5, 129])}
    expected = {rid: plain.forward(ODD, widened(weights), toks).numpy() for rid, toks in requests.items()}
    with tempfile.TemporaryDirectory() as folder:
        fu.write_dir(folder, ODD, weights)
        for name in ("whole", "mixed"):
            steps = SCHEDULES[name](requests)
            engine = make_engine(folder, dtype_name, max_tokens=schedules.max_live_tokens(steps, 64), page_tokens=64, poison_freed=True)
            got = schedules.collect(steps, run_steps(engine, steps))
            errors = np.concatenate([fu.relative_error(np.stack(got[rid]), expected[rid]) for rid in got])
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
    every window passes over decoded tokens many times, pages behind them are handed back and used again, and the
    matrix memory is carried 300 steps."""
    raw = fu.SMALL["B"]
    weights = fu.make_weights(raw, 91, torch.float32, sharpen=2.0)
    gen = np.random.default_rng(2)
    requests = {"a": gen.integers(0, raw["vocab"], size=310).tolist(), "b": gen.integers(0, raw["vocab"], size=305).tolist()}
    expected = {rid: plain.forward(raw, weights, toks).numpy() for rid, toks in requests.items()}
    with tempfile.TemporaryDirectory() as folder:
        fu.write_dir(folder, raw, weights)
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
    raw = fu.SMALL["A"]
    weights = fu.make_weights(raw, 23, torch.float32, sharpen=2.0)
    gen = np.random.default_rng(8)
    prompts = [gen.integers(0, raw["vocab"], size=n).tolist() for n in (3, 40, 21, 9, 57)]
    with tempfile.TemporaryDirectory() as folder:
        fu.write_dir(folder, raw, weights)
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
    """``leone generate`` on a Fosulix folder: greedy tokens as the plain implementation picks them; ``leone
    random-model`` writes a folder of the design that loads again."""
    from leone_amd import cli
    raw = fu.SMALL["C"]
    weights = fu.make_weights(raw, 61, torch.float32, sharpen=2.0)
    folder = fu.write_dir(str(tmp_path / "model"), raw, weights)
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
        json.dump(fu.SMALL["A"], handle)
    made = str(tmp_path / "made")
    assert cli.main(["random-model", "--config", config_path, "--seed", "3", "--out", made]) == 0
    engine = make_engine(made, "bfloat16", max_tokens=64)
    from leone_amd.engine.engine import StepEntry
    logits = engine.step([StepEntry("a", [1, 2, 3], [2])]).logits
    assert logits.shape == (1, fu.SMALL["A"]["vocab"]) and torch.isfinite(logits).all()


# ---- each mechanism alone ---------------------------------------------------------------------------------------

def close(have, want, tol, what):
    have, want = have.double().cpu(), want.double().cpu()
    scale = float(want.abs().max()) + 1e-30
    worst = float((have - want).abs().max()) / scale
    assert worst <= tol, f"{what}: off by {worst:.3e} of the largest value, bound {tol}"


CUTS = [(5, 1), (1, 1), (2, 0), (1, 3), (17, 1), (1, 16), (0, 2), (33, 1), (1, 1), (2, 40)]      # 63 and 66 rows


def latent_case(dtype, m, width=48, seed=0, sharpen=3.0):
    """(part, weights in double) of one latent-attention mixer with sizes ``m`` (the configuration's keys)."""
    from leone_amd.parts import MIXERS, POSITIONS, PartSpec
    gen = torch.Generator().manual_seed(seed)

    def mat(rows, cols, scale=1.5):
        return (torch.randn(rows, cols, generator=gen) * scale / math.sqrt(cols)).to(dtype)

    heads, dim, rot, vdim, qr, kr = (m[k] for k in ("heads", "dim", "rot_dim", "vdim", "q_rank", "kv_rank"))
    w = {"dq": mat(qr, width), "dq.norm": ((1 + 0.2 * torch.randn(qr, generator=gen)) * sharpen).to(dtype),
         "uq": mat(heads * (dim + rot), qr), "dkv": mat(kr + rot, width), "dkv.norm": (1 + 0.2 * torch.randn(kr, generator=gen)).to(dtype),
         "uk": mat(heads * dim, kr), "uv": mat(heads * vdim, kr), "o": mat(width, heads * vdim)}
    r = m["rot"]
    if r.get("scaling"):
        rope = POSITIONS.build(PartSpec("rope_scaled_adjacent", {"rotary_dim": r["dims"], "theta": r["base"], **r["scaling"]}))
    else:
        rope = POSITIONS.build(PartSpec("rope_adjacent", {"rotary_dim": r["dims"], "theta": r["base"]}))
    rope.prepare(512, DEV)
    spec = PartSpec("latent_attention", dict(hidden=width, heads=heads, dim=dim, rot_dim=rot, vdim=vdim, q_rank=qr, kv_rank=kr,
                                             scale=m["scale"], eps=1e-5, window=(m.get("mask") or {}).get("size"), position="rope",
                                             dq="dq", dq_norm="dq.norm", uq="uq", dkv="dkv", dkv_norm="dkv.norm", uk="uk",
                                             uv="uv", o="o"))
    part = MIXERS.build(spec, positions={"rope": rope})
    part.bind({k: v.to(DEV) for k, v in w.items()})
    return part, {k: v.to(F) for k, v in w.items()}, width


def plain_latent(h, m, w):
    positions = list(range(h.shape[0]))
    cached = plain.latent_keys(h, m, w, "", 1e-5, positions)
    return plain.latent_attention(h, m, w, "", 1e-5, positions, cached)


LATENTS = [
    {"heads": 3, "dim": 8, "rot_dim": 8, "vdim": 20, "q_rank": 12, "kv_rank": 24, "scale": 0.3,
     "rot": {"dims": 8, "base": 300.0, "scaling": {"factor": 8.0, "original": 32, "fast": 16.0, "slow": 1.0}}, "mask": {"size": 19}},
    {"heads": 1, "dim": 40, "rot_dim": 4, "vdim": 8, "q_rank": 30, "kv_rank": 100, "scale": 0.2, "rot": {"dims": 4, "base": 50.0}},
    {"heads": 5, "dim": 16, "rot_dim": 24, "vdim": 16, "q_rank": 64, "kv_rank": 200, "scale": 0.15,
     "rot": {"dims": 16, "base": 1000.0, "scaling": {"factor": 2.0, "original": 16, "fast": 4.0, "slow": 2.0}}, "mask": {"size": 1}},
    {"heads": 6, "dim": 64, "rot_dim": 32, "vdim": 64, "q_rank": 96, "kv_rank": 320, "scale": 0.1,
     "rot": {"dims": 32, "base": 10000.0}, "mask": {"size": 32}},
    {"heads": 16, "dim": 32, "rot_dim": 64, "vdim": 32, "q_rank": 64, "kv_rank": 512, "scale": 0.1,
     "rot": {"dims": 64, "base": 10000.0}, "mask": {"size": 45}},
    {"heads": 5, "dim": 16, "rot_dim": 16, "vdim": 24, "q_rank": 32, "kv_rank": 48, "scale": 0.2, "rot": {"dims": 16, "base": 100.0}},
]


@pytest.mark.parametrize("page_tokens", [16, 32])
@pytest.mark.parametrize("dtype_name", list(DTYPES))
@pytest.mark.parametrize("m", LATENTS, ids=lambda m: f"{m['heads']}x{m['dim']}+{m['rot_dim']}r{m['kv_rank']}")
def test_latent_attention_alone_in_cuts_of_every_size(m, dtype_name, page_tokens):
    """Two sequences side by side, fed in steps of 0 to 40 rows each, state slots and pages interleaved and filled
    with NaN beforehand: one head and several, latents of 24 to 512 elements, a window of one key (itself), of a
    page and a bit, of two pages, and none.  In bfloat16 with pages of 32 tokens the sizes that fit go to the
    matrix-core kernel."""
    dtype = DTYPES[dtype_name]
    part, w, width = latent_case(dtype, m, seed=m["kv_rank"])
    gen = torch.Generator().manual_seed(3)
    hs = [torch.randn(63, width, generator=gen).to(dtype), torch.randn(66, width, generator=gen).to(dtype)]
    got = run_mixer_in_cuts(part, hs, CUTS, dtype, page_tokens)
    for s in (0, 1):
        want = plain_latent(hs[s].to(F), m, w)
        err = fu.relative_error(got[s].numpy(), want.numpy())
        assert err.max() <= (2e-5 if dtype_name == "float32" else 3e-2), (s, int(err.argmax()), float(err.max()))


@pytest.mark.parametrize("page_tokens", [16, 32])
@pytest.mark.parametrize("window", [None, 40, 64])
@pytest.mark.parametrize("dtype_name", list(DTYPES))
def test_latent_attention_finds_planted_keys(dtype_name, window, page_tokens, monkeypatch):
    """Keys that answer one query each are planted far back, on both sides of page borders (pages of 16), and at the
    last position a window still holds; a decoy stands one position outside the window of a query, with a value of its
    own, and must not be seen.  Queries come in a prompt's portion and as single decoded tokens.  The plain part of the
    query meets the latent through W_uk; the weights here make that the identity on the first elements."""
    from leone_amd import ops
    monkeypatch.setattr(ops, "LATENT_SPLIT_TILES", 1)    # single rows far into a sequence: three workgroups share their keys
    assert ops.latent_splits(2, 290) == 3 and ops.latent_splits(2, 40) == 1 and ops.latent_splits(16 * 300, 290) == 1
    dtype = DTYPES[dtype_name]
    width, heads, dim, rot, vdim, qr, kr = 48, 2, 12, 32, 16, 24, 32      # a latent of 32 + 32: with pages of 32 the matrix cores
    m = {"heads": heads, "dim": dim, "rot_dim": rot, "vdim": vdim, "q_rank": qr, "kv_rank": kr, "scale": 1.0,
         "rot": {"dims": rot, "base": 10.0}}
    if window:
        m["mask"] = {"size": window}
    part, w, _ = latent_case(dtype, m, width=width, seed=7, sharpen=1.0)
    # a row's inputs 0..11 make its key (through the latent and W_uk, the identity there), inputs 12..23 its query (so
    # that a query is no key for itself), the others its value; nothing is rotated
    ident = torch.zeros(qr, width)
    ident[:dim, dim:2 * dim] = torch.eye(dim)
    uq = torch.zeros(heads * (dim + rot), qr)
    uk = torch.zeros(heads * dim, kr)
    for h in range(heads):
        # scores as sharp as the type bears: a rounded key moves a score by its 2^-9th part
        uq[h * (dim + rot):h * (dim + rot) + dim, :dim] = torch.eye(dim) * (6.0 if dtype_name == "float32" else 2.5)
        uk[h * dim:(h + 1) * dim, :dim] = torch.eye(dim)
    dkv = torch.zeros(kr + rot, width)                   # no rotated key part: positions play no role in the scores
    dkv[:dim, :dim] = torch.eye(dim)
    dkv[dim:kr, 2 * dim:] = torch.randn(kr - dim, width - 2 * dim, generator=torch.Generator().manual_seed(1)) / 3
    new = {"dq": ident, "uq": uq, "uk": uk, "dkv": dkv, "dq.norm": torch.ones(qr), "dkv.norm": torch.ones(kr)}
    for k, v in new.items():
        w[k] = v.to(dtype).to(F)
    part.bind({k: v.to(dtype).to(DEV) for k, v in w.items()})
    total = 300
    gen = torch.Generator().manual_seed(11)
    hs = torch.randn(total, width, generator=gen)
    hs[:, :2 * dim] *= 0.05                              # the inputs that keys and queries are made from stay quiet
    # key -> query; with a window every key is the oldest position its query still sees
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
    want = plain_latent(hs.to(F), m, w)
    cuts = [(270, 1), (10, 1)] + [(1, 1)] * 20
    got = run_mixer_in_cuts(part, [hs, hs[:22]], cuts, dtype, page_tokens)[0]
    err = fu.relative_error(got.numpy(), want.numpy())
    tol = 2e-5 if dtype_name == "float32" else 3e-2
    asked = list(pairs.values())
    assert err[asked].max() <= tol, (asked[int(err[asked].argmax())], float(err[asked].max()))
    # a row that sees a key and its decoy with like weights adds two opposite values: there rounded scores show more
    assert err.max() <= (tol if dtype_name == "float32" else 3 * tol) and np.median(err) <= tol, (int(err.argmax()), float(err.max()))
    # the planted keys matter, and so would the decoys: moving the window by one changes the queries' rows by far more
    for shift in ((-1, 1) if window else (0,)):
        other = dict(m)
        if window:
            other["mask"] = {"size": window + shift}
            moved = fu.relative_error(plain_latent(hs.to(F), other, w).numpy(), want.numpy())
        else:
            bare = hs.clone().to(F)
            for key_at in pairs:
                bare[key_at, :dim] = 0
            moved = fu.relative_error(plain_latent(bare, m, w).numpy(), want.numpy())
        assert all(moved[q] > 10 * tol for q in pairs.values()), [float(moved[q]) for q in pairs.values()]


MEMORIES = [{"heads": 3, "dim": 12, "vdim": 20}, {"heads": 1, "dim": 40, "vdim": 7}, {"heads": 2, "dim": 128, "vdim": 64},
            {"heads": 5, "dim": 33, "vdim": 130}, {"heads": 2, "dim": 256, "vdim": 16}]


@pytest.mark.parametrize("dtype_name", list(DTYPES))
@pytest.mark.parametrize("m", MEMORIES, ids=lambda m: f"{m['heads']}x{m['dim']}x{m['vdim']}")
def test_gated_memory_alone_in_cuts_of_every_size(m, dtype_name):
    """The matrix memory with its forget gate, fed in steps of 0 to 40 rows, slots filled with NaN beforehand; some
    lower bounds are so close to 1 that what the first rows wrote still weighs at the end."""
    from leone_amd.parts import MIXERS, PartSpec
    dtype = DTYPES[dtype_name]
    width = 48
    gen = torch.Generator().manual_seed(m["dim"])
    qk, vv = m["heads"] * m["dim"], m["heads"] * m["vdim"]

    def mat(rows, cols, scale=1.5):
        return (torch.randn(rows, cols, generator=gen) * scale / math.sqrt(cols)).to(dtype)

    lower = torch.rand(qk, generator=gen) ** 0.3
    lower[::5] = 0.999
    w = {"q": mat(qk, width), "f": mat(qk, width, 3.0), "f.b": torch.randn(qk, generator=gen).to(dtype), "lower": lower.to(dtype),
         "v": mat(vv, width), "norm": (1 + 0.2 * torch.randn(m["vdim"], generator=gen)).to(dtype), "o": mat(width, vv)}
    part = MIXERS.build(PartSpec("hgrn2", dict(hidden=width, eps=1e-5, **m, q="q", f="f", f_bias="f.b", lower="lower", v="v",
                                               norm="norm", o="o")))
    part.bind({k: v.to(DEV) for k, v in w.items()})
    hs = [torch.randn(63, width, generator=gen).to(dtype), torch.randn(66, width, generator=gen).to(dtype)]
    got = run_mixer_in_cuts(part, hs, CUTS, dtype)
    wp = {k: v.to(F) for k, v in w.items()}
    for s in (0, 1):
        want = plain.gated_memory(hs[s].to(F), m, wp, "", 1e-5)
        err = fu.relative_error(got[s].numpy(), want.numpy())
        assert err.max() <= (2e-5 if dtype_name == "float32" else 3e-2), (s, int(err.argmax()), float(err.max()))


ROUTERS = [{"experts": 10, "top": 3, "scale": 1.25, "groups": {"count": 5, "keep": 3}},
           {"experts": 5, "top": 1, "scale": 1.0},
           {"experts": 9, "top": 4, "scale": 0.5, "groups": {"count": 9, "keep": 5}},
           {"experts": 72, "top": 6, "scale": 2.5, "groups": {"count": 8, "keep": 3}},
           {"experts": 150, "top": 8, "scale": 1.0, "groups": {"count": 10, "keep": 4}},
           {"experts": 200, "top": 5, "scale": 3.0, "groups": {"count": 100, "keep": 30}},
           {"experts": 4, "top": 4, "scale": 1.0, "groups": {"count": 1, "keep": 1}}]


@pytest.mark.parametrize("r", ROUTERS, ids=lambda r: f"{r['experts']}")
def test_router_with_sigmoid_scores_and_groups_scored_by_their_two_best(r):
    """The same experts as the plain router chooses, in any order, with its weights (scores times the scale, not
    renormalised), in both launches (rows alone, and few rows together with the tiles)."""
    from leone_amd import ops
    gen = torch.Generator().manual_seed(r["experts"])
    rows, width = 50, 32
    h = torch.randn(rows, width, generator=gen)
    router = torch.randn(r["experts"], width, generator=gen) * (3.0 / math.sqrt(width))
    logits = (h @ router.T).float()
    want_e, want_w = plain.route(h.to(F), router.to(F), r)
    groups = r.get("groups") or {"count": 1, "keep": 1}
    rule = ops.RouterRule("sigmoid", 2, False, r["scale"])
    chosen, weight = ops.route_topk(logits.to(DEV), None, r["top"], groups["count"], groups["keep"], rule)
    chosen, weight = chosen.cpu(), weight.cpu()
    want_scores = torch.sigmoid((h.to(F) @ router.to(F).T))
    for row in range(rows):
        have, want = sorted(chosen[row].tolist()), sorted(want_e[row].tolist())
        if have != want:                                   # only where two scores lie within float rounding
            odd = set(have) ^ set(want)
            spread = [float(want_scores[row, e]) for e in odd]
            assert max(spread) - min(spread) < 1e-5, (row, have, want)
            continue
        order = {e: n for n, e in enumerate(want_e[row].tolist())}
        for n, e in enumerate(chosen[row].tolist()):
            assert abs(float(weight[row, n]) - float(want_w[row, order[e]])) < 1e-5, (row, e)


@pytest.mark.parametrize("rows", [3, 40, 300])
@pytest.mark.parametrize("dtype_name", list(DTYPES))
def test_mixture_with_limited_experts_alone(rows, dtype_name):
    """The mixture part: router, choice, experts whose gate and up values are held to a limit (inputs large enough
    that both bounds bite), weighted sum; few rows (choice and tiles in one launch), some more, and many."""
    from leone_amd.parts import FEED_FORWARDS, PartSpec
    dtype = DTYPES[dtype_name]
    width = 64
    mlp = fu.moe(6, 2, 40, limit=1.5, scale=1.7, groups=(3, 2))
    gen = torch.Generator().manual_seed(rows)
    w = {"router": (torch.randn(6, width, generator=gen) * 3 / 8).to(dtype)}
    for e in range(6):
        w[f"e{e}.gate"] = (torch.randn(40, width, generator=gen) * 3 / 8).to(dtype)
        w[f"e{e}.up"] = (torch.randn(40, width, generator=gen) * 3 / 8).to(dtype)
        w[f"e{e}.down"] = (torch.randn(width, 40, generator=gen) / 6).to(dtype)
    part = FEED_FORWARDS.build(PartSpec("routed_glu", {"hidden": width, "experts": 6, "identity": 0, "top": 2, "group_count": 3,
                                                       "group_keep": 2, "intermediate": 40, "activation": "clamped_swish",
                                                       "limit": 1.5, "score": "sigmoid", "group_best": 2, "renormalize": False,
                                                       "weight_scale": 1.7, "router": "router", "correction": None,
                                                       "expert": "e{e}", "shared": None}))
    part.bind({k: v.to(DEV) for k, v in w.items()})
    h = torch.randn(rows, width, generator=gen).to(dtype)
    out = part.forward(h.to(DEV), step_of([(0, i) for i in range(rows)], dtype, [0]))
    assert out.dtype == torch.float32
    want = plain.mixture(h.to(F), mlp, {k: v.to(F) for k, v in w.items()}, "")
    err = fu.relative_error(out.cpu().numpy(), want.numpy())
    if dtype_name == "float32":
        assert err.max() <= 2e-5, (int(err.argmax()), float(err.max()))
    else:
        assert np.median(err) <= 2e-2 and (err > 0.1).sum() <= max(1, rows // 12), (float(np.median(err)), float(err.max()))
    g = h.to(F) @ w["e0.gate"].to(F).T
    assert (g > 1.5).any() and ((h.to(F) @ w["e0.up"].to(F).T).abs() > 1.5).any(), "the limits must bite in this test"


def test_scaled_residual_norm_and_stream_mixed_over_depth():
    """x += scale * delta with the norm that follows in one kernel (planes, picked rows); the stream as the weighted sum
    of the kept results of all layers so far."""
    from leone_amd import ops
    gen = torch.Generator().manual_seed(5)
    for hidden in (37, 40, 192, 1000, 5000):       # single elements and runs of four; rows longer than a thread holds
        rows, eps = 9, 1e-5
        x = torch.randn(rows, hidden, generator=gen)
        planes = torch.randn(3, rows, hidden, generator=gen)
        gain = 1 + 0.3 * torch.randn(hidden, generator=gen)
        want = x.double() + 0.3 * planes.double().sum(0)
        stream = x.to(DEV)
        y = ops.residual_norm(stream, planes.to(DEV), 0.3, gain.to(DEV), eps, torch.float32)
        close(stream, want, 2e-6, "stream")
        close(y, plain.rms_norm(want, gain.double(), eps), 3e-6, "normed rows")
        stream = x.to(DEV)
        picked = torch.tensor([7, 0, 3], dtype=torch.int32, device=DEV)
        y = ops.residual_norm(stream, planes[0].to(DEV), -2.0, gain.to(DEV).bfloat16(), eps, torch.bfloat16, rows=picked)
        close(y.float(), plain.rms_norm(x.double() - 2.0 * planes[0].double(), gain.bfloat16().double(), eps)[[7, 0, 3]], 1e-2, "picked rows")
        assert torch.equal(stream.cpu(), x), "with picked rows the stream is left alone"
        # depth: three results kept, the fourth arrives as stream + scale * delta
        history = torch.randn(6, rows, hidden, generator=gen)
        weight = torch.randn(4, generator=gen)
        stream, kept = x.to(DEV), history.to(DEV)
        ops.depth_mix(stream, planes[1].to(DEV), 0.5, kept, 4, weight.to(DEV))
        own = x.double() + 0.5 * planes[1].double()
        close(kept[3], own, 2e-6, "kept result")
        close(stream, sum(weight[j].double() * history[j].double() for j in range(3)) + weight[3].double() * own, 3e-6, "mixed stream")
        assert torch.equal(kept[4:].cpu(), history[4:]) and torch.equal(kept[:3].cpu(), history[:3])


@pytest.mark.parametrize("dtype_name", list(DTYPES))
@pytest.mark.parametrize("taps", [2, 4, 5])
def test_block_with_input_convolution_across_steps(taps, dtype_name):
    """One whole block (norm, convolution in residual form, mixer, factor, norm, mixture, factor) in cuts of every
    size against the plain functions put together by hand: the convolution's inputs are carried from step to step."""
    raw = fu.config(64, 50, [fu.layer(fu.memory(2, 16, 24), fu.moe(4, 2, 16, scale=1.3))], mult=0.4, embed_scale=3.0, taps=taps)
    dtype = DTYPES[dtype_name]
    weights = fu.make_weights(raw, taps, dtype)
    tokens = np.random.default_rng(taps).integers(0, 50, size=70).tolist()
    want = plain.forward(raw, widened(weights), tokens).numpy()
    with tempfile.TemporaryDirectory() as folder:
        fu.write_dir(folder, raw, weights)
        for sizes in ((1,), (2, 1, 3, taps - 1, taps, taps + 1, 30)):
            engine = make_engine(folder, dtype_name, max_tokens=128, poison_freed=True)
            steps = schedules.portions({"a": tokens}, sizes=sizes)
            compare(steps, run_steps(engine, steps), {"a": want}, dtype_name, f"{taps} taps, portions {sizes}")
