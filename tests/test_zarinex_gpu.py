"""Zarinex in the engine against the plain model of tests/plain/zarinex_plain.py: every mechanism
alone, prompts against token-by-token decoding, prompts cut into portions, batches of unequal
requests, slots and pages that are used again, far keys at page borders and at the first places,
prompts long enough for the chunked walk of the states, long decoding through recorded steps, and
greedy generation through the entry points.

The configurations are those of tests/zarinex_tiny.py; the plain model computes a whole sequence
from scratch in double precision, so every schedule has one truth: the function of the sequence."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import zarinex_tiny as zt

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]


def tokens_for(cfg, n, seed):
    rng = np.random.default_rng(seed)
    return [int(t) for t in rng.integers(0, cfg["vocab"], size=n)]


_MODELS, _TRUTH = {}, {}


def model_of(which, dtype, seed=0):
    key = (which, dtype, seed)
    if key not in _MODELS:
        cfg = zt.CONFIGS[which]
        w = zt.make_weights(cfg, seed)
        _MODELS[key] = (cfg, w, zt.load(cfg, w, dtype))
    return _MODELS[key]


def truth_of(which, seed, tokens):
    key = (which, seed, tuple(tokens))
    if key not in _TRUTH:
        cfg = zt.CONFIGS[which]
        _TRUTH[key] = zt.Truth(cfg, zt.make_weights(cfg, seed), tokens)
    return _TRUTH[key]


def new_session(model, max_tokens=4096, **kw):
    from picolm_amd.engine import Session
    return Session(model, max_tokens=max_tokens, **kw)


def run_whole(session, tokens):
    [slot] = session.begin(1)
    got = session.step([slot], [tokens], [list(range(len(tokens)))]).double().cpu().numpy()
    session.release([slot])
    return got


def test_the_models_tensors_are_the_designs():
    from picolm_amd.engine.builder import build_from_config_dict
    for cfg in zt.CONFIGS.values():
        specs = {s.name: tuple(s.shape) for s in build_from_config_dict(cfg).tensor_specs() if not s.optional}
        assert specs == zt.tensor_shapes(cfg)


# ------------------------------------------------------------------------------ each mechanism alone
def one_layer(mixer, mlp=None, **kw):
    return zt.config(61, 48, [zt.layer(mixer, mlp)], **kw)


ALONE = {
    "selective scan": one_layer(zt.mamba(40, 12, 5, 3)),
    "selective scan, a state of 200": one_layer(zt.mamba(24, 200, 4, 2)),      # sixteen lanes a column
    "selective scan, a state of one, one tap": one_layer(zt.mamba(72, 1, 1, 1)),
    "selective scan, 300 channels": one_layer(zt.mamba(300, 20, 9, 4)),        # more than a workgroup's columns
    "latent attention": one_layer(zt.latent(3, 12, 20, 28, 36, 0.4)),
    # latents that the matrix-core attention takes in bfloat16 (64, 96, 128), all heads on the one key head
    "latent attention, latents of 64": one_layer(zt.latent(4, 24, 16, 64, 40, 0.3)),
    "latent attention, latents of 96, forty heads": one_layer(zt.latent(40, 8, 12, 96, 24, 0.5)),
    "latent attention, latents of 128": one_layer(zt.latent(2, 32, 48, 128, 64, 0.2)),
    "latent attention, latents of 288": one_layer(zt.latent(2, 16, 24, 288, 48, 0.25)),      # beyond what a thread's registers hold of a key
    "latent attention, one head, latents of 5": one_layer(zt.latent(1, 7, 3, 5, 6, 0.6)),
    "forget-gated state": one_layer(zt.hgrn(3, 12, 20)),
    "forget-gated state, keys of 144": one_layer(zt.hgrn(2, 144, 8)),
    "forget-gated state, keys as long as values": one_layer(zt.hgrn(4, 16, 16)),
    "routed experts": one_layer(zt.hgrn(1, 8, 8), zt.moe(6, 2, 24, 40)),
    "routed experts, one pick, no shared expert": one_layer(zt.hgrn(1, 8, 8), zt.moe(5, 1, 36)),
    "routed experts, every expert picked": one_layer(zt.hgrn(1, 8, 8), zt.moe(3, 3, 20, 12)),
    # in bfloat16 a prompt of 64 rows and more sorts its picks by expert for the matrix cores: tiles that are partly
    # empty, experts without a row, hidden units and outputs that end inside a tile of 32
    "routed experts, widths in multiples of 16": one_layer(zt.hgrn(1, 8, 8), zt.moe(6, 2, 32, 48)),
    "routed experts, more experts than rows a tile": one_layer(zt.hgrn(1, 8, 8), zt.moe(40, 3, 48)),
    "routed experts, widths that are no multiples of 8": zt.config(61, 45, [zt.layer(zt.hgrn(1, 9, 5), zt.moe(4, 2, 13, 7))]),
    "alpha and eps": one_layer(zt.hgrn(2, 8, 12), zt.moe(2, 1, 16, 8), alpha=5.0, eps=1e-2),
}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("what", list(ALONE))
def test_each_mechanism_alone(what, dtype):
    cfg = ALONE[what]
    w = zt.make_weights(cfg, 11)
    tokens = tokens_for(cfg, 70, 3)            # past a page's end
    want = zt.Truth(cfg, w, tokens)
    s = new_session(zt.load(cfg, w, dtype), 256)
    assert zt.near(run_whole(s, tokens), want, slice(None), dtype)
    # and the same decoded token by token
    [slot] = s.begin(1)
    for i, t in enumerate(tokens):
        got = s.step([slot], [[t]]).double().cpu().numpy()
        assert zt.near(got, want, i, dtype), (what, "token", i)
    s.release([slot])


def test_every_mechanism_shows_in_the_plain_model():
    """The tests above would pass a model that ignored what they isolate, if the plain model did."""
    cfg = zt.CONFIGS["A"]
    w = zt.make_weights(cfg, 0)
    tokens = tokens_for(cfg, 30, 3)
    base = zt.plain_logits(cfg, w, tokens)
    for name in ("l0.shift", "l0.rg1.b", "l0.rg2", "l0.mix.lower", "l0.mix.f.b", "l2.mix.A_log", "l2.mix.dt.b", "l2.mix.D", "l2.mix.conv",
                 "l3.mix.g", "l3.mix.dq.norm", "l3.mlp.router.b", "l3.mlp.shared.down", "l0.mlp.e1.up"):
        changed = dict(w)
        changed[name] = torch.zeros_like(w[name])
        assert zt.distance(zt.plain_logits(cfg, changed, tokens), base) > 0.01, name
    other = dict(cfg, postln_alpha=1.0)
    assert zt.distance(zt.plain_logits(other, w, tokens), base) > 0.01
    no_positions = zt.plain_logits(cfg, w, tokens[:1] + tokens[:1])
    assert zt.distance(no_positions[1], no_positions[0]) > 0.01


# ------------------------------------------------------------------------------ prompts, decoding, portions
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", ["A", "B", "C"])
def test_prompt_decoding_and_portions(which, dtype):
    cfg, w, model = model_of(which, dtype)
    tokens = tokens_for(cfg, 150, 1)
    want = truth_of(which, 0, tokens)
    s = new_session(model, 1024)
    assert zt.near(run_whole(s, tokens), want, slice(None), dtype)
    # most of it at once, the rest one by one (past the page border at 128)
    [slot] = s.begin(1)
    got = s.step([slot], [tokens[:101]], [[0, 1, 2, 63, 64, 100]]).double().cpu().numpy()
    assert zt.near(got, want, [0, 1, 2, 63, 64, 100], dtype)
    for i in range(101, 150):
        got = s.step([slot], [[tokens[i]]]).double().cpu().numpy()
        assert zt.near(got, want, i, dtype), ("decoded", i)
    s.release([slot])
    # portions of several sizes, down to two tokens and one, every row wanted
    for sizes in ([2, 2, 3, 57, 1, 64, 21], [64, 64, 22], [1, 1, 2, 146], [149, 1]):
        assert sum(sizes) == 150
        [slot] = s.begin(1)
        at = 0
        for n in sizes:
            got = s.step([slot], [tokens[at:at + n]], [list(range(n))]).double().cpu().numpy()
            assert zt.near(got, want, slice(at, at + n), dtype), (sizes, "portion at", at)
            at += n
        s.release([slot])


@pytest.mark.parametrize("dtype", DTYPES)
def test_portions_equal_the_whole_prompt_beyond_rounding(dtype):
    """How a prompt is cut does not show in the logits: against each other, not only against the
    plain model, and much closer than the limit that bfloat16 needs there."""
    cfg, w, model = model_of("A", dtype)
    tokens = tokens_for(cfg, 131, 5)
    s = new_session(model, 1024)
    whole = run_whole(s, tokens)
    [slot] = s.begin(1)
    parts, at = [], 0
    for n in (2, 63, 2, 61, 3):
        parts.append(s.step([slot], [tokens[at:at + n]], [list(range(n))]).double().cpu().numpy())
        at += n
    s.release([slot])
    assert zt.distance(np.concatenate(parts), whole) <= (1e-5 if dtype == "float32" else 0.03)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", ["A", "B", "C"])
def test_long_prompts_walked_in_chunks(which, dtype):
    """From 256 new tokens of a sequence on, the states are walked in chunks of 64 side by side
    (every chunk's effect on a state first, then the states from chunk to chunk, then the outputs):
    a long prompt whole, in two long portions onto each other, and in a batch with a short one and
    one that is a token over the threshold, then decoded on."""
    cfg, w, model = model_of(which, dtype)
    tokens = tokens_for(cfg, 645, 8)
    want = truth_of(which, 0, tokens)
    s = new_session(model, 2048)
    assert zt.near(run_whole(s, tokens[:641]), want, slice(0, 641), dtype)
    [slot] = s.begin(1)
    rows = [0, 63, 64, 255, 256, 299]
    got = s.step([slot], [tokens[:300]], [rows]).double().cpu().numpy()
    assert zt.near(got, want, rows, dtype)
    got = s.step([slot], [tokens[300:641]], [list(range(341))]).double().cpu().numpy()
    assert zt.near(got, want, slice(300, 641), dtype)
    for i in range(641, 645):
        got = s.step([slot], [[tokens[i]]]).double().cpu().numpy()
        assert zt.near(got, want, i, dtype), ("decoded", i)
    s.release([slot])
    others = [tokens_for(cfg, n, 30 + n) for n in (10, 257)]
    slots = s.begin(3)
    got = s.step(slots, [tokens[:400]] + others).double().cpu().numpy()
    assert zt.near(got[0], want, 399, dtype)
    for i, q in enumerate(others):
        assert zt.near(got[1 + i], truth_of(which, 0, q), len(q) - 1, dtype), ("beside the long one", i)
    got = s.step(slots[:1], [[tokens[400]]]).double().cpu().numpy()
    assert zt.near(got, want, 400, dtype)
    s.release(slots)


# ------------------------------------------------------------------------------ batches
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", ["A", "C"])
def test_a_batch_of_unequal_requests_equals_each_alone(which, dtype):
    cfg, w, model = model_of(which, dtype)
    lens, n_dec = [1, 2, 65, 37, 64, 130], 5
    seqs = [tokens_for(cfg, n + n_dec, 20 + i) for i, n in enumerate(lens)]
    truth = [truth_of(which, 0, q) for q in seqs]
    s = new_session(model, 2048)
    slots = s.begin(len(seqs))
    got = s.step(slots, [q[:n] for q, n in zip(seqs, lens)], [list(range(n)) for n in lens]).double().cpu().numpy()
    at = 0
    for i, n in enumerate(lens):
        assert zt.near(got[at:at + n], truth[i], slice(0, n), dtype), ("prompt", i)
        at += n
    # the shorter ones end earlier: after two steps the first two leave the batch
    live = list(range(len(seqs)))
    for j in range(n_dec):
        if j == 2:
            s.release([slots[0], slots[1]])
            live = live[2:]
        got = s.step([slots[i] for i in live], [[seqs[i][lens[i] + j]] for i in live]).double().cpu().numpy()
        for row, i in enumerate(live):
            assert zt.near(got[row], truth[i], lens[i] + j, dtype), ("step", j, "sequence", i)
    s.release([slots[i] for i in live])


@pytest.mark.parametrize("dtype", DTYPES)
def test_slots_and_pages_that_are_used_again(dtype):
    """A slot's states and its row before the first start at zero again, and a page's old latents are
    not seen: sequences run one after another through a session that has room for little more than
    one of them."""
    cfg, w, model = model_of("A", dtype)
    s = new_session(model, 256, n_slots=2)
    for k, n in enumerate([130, 5, 70, 130, 1, 64]):
        tokens = tokens_for(cfg, n, 40 + k)
        want = truth_of("A", 0, tokens)
        [slot] = s.begin(1)
        cut = max(1, n - 3)
        rows = [0, cut - 1]
        got = s.step([slot], [tokens[:cut]], [rows]).double().cpu().numpy()
        assert zt.near(got, want, rows, dtype), ("prompt", k)
        for i in range(cut, n):
            got = s.step([slot], [[tokens[i]]]).double().cpu().numpy()
            assert zt.near(got, want, i, dtype), ("sequence", k, "token", i)
        s.release([slot])
    # two sequences that swap slots between uses
    a, b = tokens_for(cfg, 40, 90), tokens_for(cfg, 66, 91)
    for order in ((a, b), (b, a)):
        slots = s.begin(2)
        got = s.step(slots, list(order)).double().cpu().numpy()
        for i, q in enumerate(order):
            assert zt.near(got[i], truth_of("A", 0, q), len(q) - 1, dtype)
        s.release(slots)


# ------------------------------------------------------------------------------ far keys, page borders, the first places
def lookup_model(kv_rank=48, dim=64, vdim=16, heads=2):
    """One layer of latent attention that looks a token's partner up.  All but the last eight entries
    of a latent read the first half of the width, the last eight (kept small, so that the others
    decide the latent's norm) the second half; queries and keys read the first part through one
    matrix that nearly keeps lengths, values the last eight; token t + 700 has the first half of
    token t's embedding, and the embedding outweighs the positions.  So the score of t against
    t + 700 is as high as against itself, wherever the partner stands, and far above the chance
    products of hundreds of other keys, while the partner's value is its own."""
    keys = kv_rank - 8
    cfg = zt.config(1400, 64, [zt.layer(zt.latent(heads, dim, vdim, kv_rank, kv_rank, 30.0 / kv_rank), None)])
    w = zt.make_weights(cfg, 5)
    p = "l0.mix."
    w["embed"] = (6.0 * w["embed"].double()).to(torch.bfloat16)
    w["embed"][700:, :32] = w["embed"][:700, :32]
    w["l0.shift"] = torch.zeros_like(w["l0.shift"])
    w[p + "dkv"][:keys, 32:] = 0
    w[p + "dkv"][keys:, :32] = 0
    w[p + "dkv"][keys:] = (0.25 * w[p + "dkv"][keys:].double()).to(torch.bfloat16)
    w[p + "dq"] = w[p + "dkv"].clone()
    w[p + "dq.norm"] = w[p + "dkv.norm"] = torch.ones(kv_rank, dtype=torch.bfloat16)
    uk = torch.randn(heads * dim, kv_rank, generator=torch.Generator().manual_seed(2), dtype=torch.float64) / dim ** 0.5
    uk[:, keys:] = 0
    w[p + "uk"] = w[p + "uq"] = uk.to(torch.bfloat16)
    w[p + "uv"][:, :keys] = 0
    w[p + "uv"] = (4.0 * w[p + "uv"].double()).to(torch.bfloat16)
    w[p + "o"] = (16.0 * w[p + "o"].double()).to(torch.bfloat16)          # the branch outweighs the rows it is added to
    return cfg, w


def distinct_tokens(n, needle_at, vocab, seed):
    """n unrelated tokens, except that the last one's partner stands at `needle_at`."""
    rng = np.random.default_rng(seed)
    tokens = [int(t) for t in rng.permutation(vocab // 2)[:n]]
    tokens[needle_at] = tokens[-1] + vocab // 2
    return tokens


_FAR = {}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kv_rank", [48, 64])
def test_one_far_key_among_hundreds(kv_rank, dtype):
    """The asking token is the last; the key it asks for lies hundreds back, at the first places of
    the sequence, and just before and after page borders.  Both in a prompt and decoded.  (Latents
    of 64 go through the matrix-core kernel in bfloat16.)"""
    cfg, w = lookup_model(kv_rank)
    model = zt.load(cfg, w, dtype)
    s = new_session(model, 2048)
    n = 500
    for needle_at in (0, 1, 63, 64, 65, 128, 383, 498):
        tokens = distinct_tokens(n, needle_at, cfg["vocab"], needle_at)
        if (kv_rank, needle_at) not in _FAR:
            other = list(tokens)
            other[needle_at] = next(t for t in range(cfg["vocab"] // 2) if t not in tokens)
            _FAR[(kv_rank, needle_at)] = (zt.plain_logits(cfg, w, tokens)[-1], zt.plain_logits(cfg, w, other)[-1])
        want, missed = _FAR[(kv_rank, needle_at)]
        assert zt.distance(missed, want) > 0.12, "the key must count"
        [slot] = s.begin(1)
        got = s.step([slot], [tokens]).double().cpu().numpy()
        assert zt.distance(got, want) <= zt.LIMIT[dtype], ("prompt", needle_at)
        s.release([slot])
        [slot] = s.begin(1)
        s.step([slot], [tokens[:-1]], [[]])
        got = s.step([slot], [tokens[-1:]]).double().cpu().numpy()
        assert zt.distance(got, want) <= zt.LIMIT[dtype], ("decoded", needle_at)
        s.release([slot])


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_first_tokens_of_a_sequence(dtype):
    """Sequences of one, two and three tokens, alone and in one batch: the row before the first is
    zeros, the convolution's first inputs are zeros, the states start at zero."""
    cfg, w, model = model_of("C", dtype)
    s = new_session(model, 512)
    seqs = [tokens_for(cfg, n, 60 + n) for n in (1, 2, 3, 1)]
    for q in seqs:
        assert zt.near(run_whole(s, q), truth_of("C", 0, q), slice(None), dtype)
    slots = s.begin(len(seqs))
    got = s.step(slots, seqs).double().cpu().numpy()
    for i, q in enumerate(seqs):
        assert zt.near(got[i], truth_of("C", 0, q), len(q) - 1, dtype)
    s.release(slots)


# ------------------------------------------------------------------------------ long decoding
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", ["A", "B"])
def test_long_decoding_through_recorded_steps(which, dtype):
    """Three sequences decoded 200 tokens, over page borders; from the second step of a shape on the
    engine replays its recording."""
    cfg, w, model = model_of(which, dtype)
    lens, n_dec = [3, 60, 120], 200
    seqs = [tokens_for(cfg, n + n_dec, 70 + i) for i, n in enumerate(lens)]
    truth = [truth_of(which, 0, q) for q in seqs]
    s = new_session(model, 2048)
    slots = s.begin(3)
    s.step(slots, [q[:n] for q, n in zip(seqs, lens)])
    for j in range(n_dec):
        got = s.step(slots, [[q[n + j]] for q, n in zip(seqs, lens)]).double().cpu().numpy()
        for i, n in enumerate(lens):
            assert zt.near(got[i], truth[i], n + j, dtype), ("step", j, "sequence", i)
    assert s.recorded_steps() >= 1
    s.release(slots)


# ------------------------------------------------------------------------------ the entry points
@pytest.fixture(scope="module")
def folder_a(tmp_path_factory):
    cfg = zt.CONFIGS["A"]
    return zt.write_folder(str(tmp_path_factory.mktemp("zarinex") / "a"), cfg, zt.make_weights(cfg, 0))


@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_generation_through_the_entry_point(dtype, folder_a):
    import picolm_amd
    cfg = zt.CONFIGS["A"]
    prompts = [tokens_for(cfg, n, 50 + n) for n in (4, 9, 66)]
    got = picolm_amd.generate(folder_a, prompts, max_new_tokens=10, stop_ids=(), dtype=dtype)
    for p, r in zip(prompts, got):
        assert len(r.tokens) == 10 and r.finish == "length"
        seq = list(p)
        for k in range(10):
            lg = truth_of("A", 0, seq).logits[-1]
            top2 = np.sort(lg)[-2:]
            if top2[1] - top2[0] < 4 * zt.LIMIT[dtype] * lg.std():
                break                              # a near tie: either choice is right
            assert r.tokens[k] == int(np.argmax(lg)), (k, r.tokens)
            seq.append(r.tokens[k])


def test_trace_replay_and_command_line(folder_a, tmp_path):
    """bin/trace_run on a folder: a prompt, single tokens and a second request that joins later in a
    slot that was given back; bin/picolm generates from the same folder."""
    cfg = zt.CONFIGS["A"]
    a, b = tokens_for(cfg, 20, 1), tokens_for(cfg, 9, 2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:17], "want": [0, 16]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[17:18], "want": [0]}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": a[18:19], "want": []}], "end": []},
             {"step": 3, "entries": [{"id": "a", "tokens": a[19:20], "want": [0]}], "end": ["a"]},
             {"step": 4, "entries": [{"id": "b", "tokens": b, "want": [8]}], "end": ["b"]}]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = str(tmp_path / "out")
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder_a, "--dtype", "float32", "--out", out,
                        "--max-tokens", "128"], input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True,
                       timeout=300)
    assert r.returncode == 0, r.stderr
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(5)]
    ta, tb = truth_of("A", 0, a), truth_of("A", 0, b)
    read = lambda i: np.fromfile(os.path.join(out, f"{i}.f32"), dtype="<f4").reshape(-1, cfg["vocab"])
    assert zt.near(read(0), ta, [0, 16], "float32")
    assert zt.near(read(1), ta, 17, "float32")
    assert not os.path.exists(os.path.join(out, "2.f32"))
    assert zt.near(read(3), ta, 19, "float32")
    assert zt.near(read(4), tb, 8, "float32")
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "picolm"), folder_a, "-p", " ".join(map(str, b)), "-n", "4", "-t", "0",
                        "--dtype", "float32"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    assert len(r.stdout.split()) == 4
    assert int(r.stdout.split()[0]) == int(np.argmax(tb.logits[-1]))
