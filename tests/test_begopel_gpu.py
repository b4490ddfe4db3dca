"""Begopel in the engine against the plain model of tests/plain/begopel_plain.py: every mechanism
alone, prompts against token-by-token decoding, prompts cut into portions, batches of unequal
requests, slots and pages that are used again, far keys and the edges of the distance table and of
pages, long decoding through recorded steps, and greedy generation through the entry point.

The configurations are those of tests/begopel_tiny.py; the plain model computes a whole sequence
from scratch in double precision, so every schedule has one truth: the function of the sequence."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import begopel_tiny as bt

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]


def tokens_for(cfg, n, seed):
    rng = np.random.default_rng(seed)
    return [int(t) for t in rng.integers(0, cfg["vocab"], size=n)]


_MODELS = {}


def model_of(which, dtype, seed=0):
    """(configuration, weights, loaded model), made once per precision."""
    key = (which, dtype, seed)
    if key not in _MODELS:
        cfg = bt.CONFIGS[which]
        w = bt.make_weights(cfg, seed)
        _MODELS[key] = (cfg, w, bt.load(cfg, w, dtype))
    return _MODELS[key]


_TRUTH = {}


def truth_of(which, seed, tokens):
    key = (which, seed, tuple(tokens))
    if key not in _TRUTH:
        cfg = bt.CONFIGS[which]
        _TRUTH[key] = bt.plain_logits(cfg, bt.make_weights(cfg, seed), tokens)
    return _TRUTH[key]


def new_session(model, max_tokens=4096, **kw):
    from picolm_amd.engine import Session
    return Session(model, max_tokens=max_tokens, **kw)


def run_whole(session, tokens):
    [slot] = session.begin(1)
    got = session.step([slot], [tokens], [list(range(len(tokens)))]).double().cpu().numpy()
    session.release([slot])
    return got


# ------------------------------------------------------------------------------ the library's list
def test_the_models_tensors_are_the_designs():
    from picolm_amd.engine.builder import build_from_config_dict
    for cfg in bt.CONFIGS.values():
        specs = {s.name: tuple(s.shape) for s in build_from_config_dict(cfg).tensor_specs() if not s.optional}
        assert specs == bt.tensor_shapes(cfg)


# ------------------------------------------------------------------------------ each mechanism alone
def one_layer(layer, **kw):
    return bt.config(61, 48, [layer], **kw)


ALONE = {
    "attention": (one_layer(bt.parallel(bt.attention(4, 2, 12, 20, 0.6, 25.0, 10), bt.delta(2, 1, 8, 12, 2), None)), "right.out"),
    "delta": (one_layer(bt.parallel(bt.attention(2, 1, 8, 8, 0.3, 9.0, 4), bt.delta(6, 2, 20, 12, 3), None)), "left.out"),
    "both": (one_layer(bt.parallel(bt.attention(3, 1, 16, 24, 0.4, 12.0, 8), bt.delta(3, 3, 12, 28, 4), None)), None),
    # head sizes that the matrix-core attention takes in bfloat16 (64, 96, 128 on either side), with more than 32 heads a group
    "attention, sizes of real heads": (one_layer(bt.parallel(bt.attention(4, 2, 96, 64, 0.2, 25.0, 10), bt.delta(2, 1, 8, 12, 2), None)), "right.out"),
    "attention, forty heads a group": (one_layer(bt.parallel(bt.attention(40, 1, 64, 128, 0.25, 70.0, 16), bt.delta(2, 1, 8, 12, 2), None)), "right.out"),
    "attention, heads of 128": (one_layer(bt.parallel(bt.attention(4, 1, 128, 128, 0.1, 33.0, 12), bt.delta(2, 1, 8, 12, 2), None)), "right.out"),
    # keys beyond 128 lie in sixteen lanes a column
    "delta, keys of 144": (one_layer(bt.parallel(bt.attention(2, 1, 8, 8, 0.3, 9.0, 4), bt.delta(2, 1, 144, 8, 2), None)), "left.out"),
    "mamba, a state of 200": (one_layer(bt.mamba(2, 8, 200, 1, 1, 2, None)), None),
    "mamba": (one_layer(bt.mamba(6, 8, 12, 3, 2, 3, None)), None),
    "mamba, a wide norm": (one_layer(bt.mamba(20, 64, 8, 1, 1, 2, None)), None),
    "mamba, one tap": (one_layer(bt.mamba(2, 24, 20, 1, 3, 1, None)), None),
    "feed-forward": (one_layer(bt.mamba(1, 16, 8, 1, 1, 2, 80)), None),
    "loop": (one_layer(bt.mamba(2, 8, 8, 2, 1, 2, 24), loop=(0, 1, 3)), None),
    "scale and cap": (one_layer(bt.mamba(2, 8, 8, 1, 2, 2, None), scale=7.0, softcap=2.0, eps=1e-3), None),
}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("what", list(ALONE))
def test_each_mechanism_alone(what, dtype):
    """One layer with one mechanism that counts: a branch of the parallel mixer is silenced through
    the weight of the norm that it leaves by, so that the other's faults are not averaged away."""
    cfg, silenced = ALONE[what]
    w = bt.make_weights(cfg, 11)
    if silenced:
        w["l0.mix." + silenced] = torch.zeros_like(w["l0.mix." + silenced])
    tokens = tokens_for(cfg, 70, 3)            # past a page's end
    want = bt.plain_logits(cfg, w, tokens)
    s = new_session(bt.load(cfg, w, dtype), 256)
    assert bt.distance(run_whole(s, tokens), want) <= bt.LIMIT[dtype]
    # and the same decoded token by token
    [slot] = s.begin(1)
    for i, t in enumerate(tokens):
        got = s.step([slot], [[t]]).double().cpu().numpy()
        assert bt.distance(got, want[i]) <= bt.LIMIT[dtype], (what, "token", i)
    s.release([slot])


def test_a_silenced_branch_and_a_cap_show_in_the_plain_model():
    """The tests above would pass a model that ignored what they isolate, if the plain model did."""
    cfg, _ = ALONE["both"]
    w = bt.make_weights(cfg, 11)
    tokens = tokens_for(cfg, 30, 3)
    base = bt.plain_logits(cfg, w, tokens)
    for name in ("l0.mix.left.out", "l0.mix.right.out", "l0.mix.left.sink", "l0.mix.left.rel", "l0.mix.right.A_log"):
        changed = dict(w)
        changed[name] = torch.zeros_like(w[name])
        assert bt.distance(bt.plain_logits(cfg, changed, tokens), base) > 0.02, name


# ------------------------------------------------------------------------------ prompts, decoding, portions
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", ["P", "Q", "R", "S"])
def test_prompt_decoding_and_portions(which, dtype):
    cfg, w, model = model_of(which, dtype)
    tokens = tokens_for(cfg, 150, 1)
    want = truth_of(which, 0, tokens)
    s = new_session(model, 1024)
    assert bt.distance(run_whole(s, tokens), want) <= bt.LIMIT[dtype]
    # most of it at once, the rest one by one (past the page border at 128)
    [slot] = s.begin(1)
    got = s.step([slot], [tokens[:101]], [[0, 1, 2, 63, 64, 100]]).double().cpu().numpy()
    assert bt.distance(got, want[[0, 1, 2, 63, 64, 100]]) <= bt.LIMIT[dtype]
    for i in range(101, 150):
        got = s.step([slot], [[tokens[i]]]).double().cpu().numpy()
        assert bt.distance(got, want[i]) <= bt.LIMIT[dtype], ("decoded", i)
    s.release([slot])
    # portions of several sizes, down to two tokens and one, every row wanted
    for sizes in ([2, 2, 3, 57, 1, 64, 21], [64, 64, 22], [1, 1, 2, 146], [149, 1]):
        assert sum(sizes) == 150
        [slot] = s.begin(1)
        at = 0
        for n in sizes:
            got = s.step([slot], [tokens[at:at + n]], [list(range(n))]).double().cpu().numpy()
            assert bt.distance(got, want[at:at + n]) <= bt.LIMIT[dtype], (sizes, "portion at", at)
            at += n
        s.release([slot])


@pytest.mark.parametrize("dtype", DTYPES)
def test_portions_equal_the_whole_prompt_beyond_rounding(dtype):
    """How a prompt is cut does not show in the logits: against each other, not only against the
    plain model, and much closer than the limit that bfloat16 needs there."""
    cfg, w, model = model_of("P", dtype)
    tokens = tokens_for(cfg, 131, 5)
    s = new_session(model, 1024)
    whole = run_whole(s, tokens)
    [slot] = s.begin(1)
    parts, at = [], 0
    for n in (2, 63, 2, 61, 3):
        parts.append(s.step([slot], [tokens[at:at + n]], [list(range(n))]).double().cpu().numpy())
        at += n
    s.release([slot])
    assert bt.distance(np.concatenate(parts), whole) <= (1e-5 if dtype == "float32" else 0.03)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", ["P", "Q", "R"])
def test_long_prompts_walked_in_chunks(which, dtype):
    """From 256 new tokens of a sequence on, the matrix states are walked in chunks of 64 side by
    side (every chunk's effect on a state first, then the states from chunk to chunk, then the
    outputs): a long prompt whole, in two long portions onto each other, and in a batch with a short
    one and one that is a token over the threshold, then decoded on."""
    cfg, w, model = model_of(which, dtype)
    tokens = tokens_for(cfg, 645, 8)
    want = truth_of(which, 0, tokens)
    s = new_session(model, 2048)
    assert bt.distance(run_whole(s, tokens[:641]), want[:641]) <= bt.LIMIT[dtype]
    [slot] = s.begin(1)
    rows = [0, 63, 64, 255, 256, 299]
    got = s.step([slot], [tokens[:300]], [rows]).double().cpu().numpy()
    assert bt.distance(got, want[rows]) <= bt.LIMIT[dtype]
    got = s.step([slot], [tokens[300:641]], [list(range(341))]).double().cpu().numpy()
    assert bt.distance(got, want[300:641]) <= bt.LIMIT[dtype]
    for i in range(641, 645):
        got = s.step([slot], [[tokens[i]]]).double().cpu().numpy()
        assert bt.distance(got, want[i]) <= bt.LIMIT[dtype], ("decoded", i)
    s.release([slot])
    others = [tokens_for(cfg, n, 30 + n) for n in (10, 257)]
    slots = s.begin(3)
    got = s.step(slots, [tokens[:400]] + others).double().cpu().numpy()
    assert bt.distance(got[0], want[399]) <= bt.LIMIT[dtype]
    for i, q in enumerate(others):
        assert bt.distance(got[1 + i], truth_of(which, 0, q)[-1]) <= bt.LIMIT[dtype], ("beside the long one", i)
    got = s.step(slots[:1], [[tokens[400]]]).double().cpu().numpy()
    assert bt.distance(got, want[400]) <= bt.LIMIT[dtype]
    s.release(slots)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_prefill_step_wide_enough_for_a_head_a_wave(dtype):
    """With four or more query heads a KV group and at least 256 workgroups of (32 queries, four
    heads), the matrix-core attention gives each wave of a workgroup a head of its own instead of
    a share of one head's keys: 18 prompts of 100 to 160 tokens and 16 heads over 4 groups make
    such a step (bfloat16; the 32-bit runtime takes the vector-ALU kernel through the same test)."""
    cfg = bt.config(83, 64, [bt.parallel(bt.attention(16, 4, 64, 64, 0.3, 90.0, 16), bt.delta(2, 1, 8, 12, 2), None)], scale=2.0)
    w = bt.make_weights(cfg, 21)
    w["l0.mix.right.out"] = torch.zeros_like(w["l0.mix.right.out"])
    lens = [100 + (37 * i) % 61 for i in range(18)]
    assert sum((n + 31) // 32 for n in lens) * (16 // 4) >= 256
    seqs = [tokens_for(cfg, n + 2, 300 + i) for i, n in enumerate(lens)]
    s = new_session(bt.load(cfg, w, dtype), 4096)
    slots = s.begin(len(seqs))
    got = s.step(slots, [q[:n] for q, n in zip(seqs, lens)], [list(range(n)) for n in lens]).double().cpu().numpy()
    truth = [bt.plain_logits(cfg, w, q) for q in seqs]
    at = 0
    for i, n in enumerate(lens):
        assert bt.distance(got[at:at + n], truth[i][:n]) <= bt.LIMIT[dtype], ("prompt", i)
        at += n
    for j in range(2):
        got = s.step(slots, [[q[n + j]] for q, n in zip(seqs, lens)]).double().cpu().numpy()
        for i, n in enumerate(lens):
            assert bt.distance(got[i], truth[i][n + j]) <= bt.LIMIT[dtype], ("step", j, "sequence", i)
    s.release(slots)


# ------------------------------------------------------------------------------ batches
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", ["P", "Q"])
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
        assert bt.distance(got[at:at + n], truth[i][:n]) <= bt.LIMIT[dtype], ("prompt", i)
        at += n
    # the shorter ones end earlier: after two steps the first two leave the batch
    live = list(range(len(seqs)))
    for j in range(n_dec):
        if j == 2:
            s.release([slots[0], slots[1]])
            live = live[2:]
        got = s.step([slots[i] for i in live], [[seqs[i][lens[i] + j]] for i in live]).double().cpu().numpy()
        for row, i in enumerate(live):
            assert bt.distance(got[row], truth[i][lens[i] + j]) <= bt.LIMIT[dtype], ("step", j, "sequence", i)
    s.release([slots[i] for i in live])


@pytest.mark.parametrize("dtype", DTYPES)
def test_slots_and_pages_that_are_used_again(dtype):
    """A slot's state starts at zero again and a page's old keys are not seen: sequences run one
    after another through a session that has room for little more than one of them."""
    cfg, w, model = model_of("P", dtype)
    s = new_session(model, 256, n_slots=2)
    first = None
    for k, n in enumerate([130, 5, 70, 130, 1, 64]):
        tokens = tokens_for(cfg, n, 40 + k)
        want = truth_of("P", 0, tokens)
        [slot] = s.begin(1)
        first = slot if first is None else first
        cut = max(1, n - 3)
        rows = [0, cut - 1]
        got = s.step([slot], [tokens[:cut]], [rows]).double().cpu().numpy()
        assert bt.distance(got, want[rows]) <= bt.LIMIT[dtype], ("prompt", k)
        for i in range(cut, n):
            got = s.step([slot], [[tokens[i]]]).double().cpu().numpy()
            assert bt.distance(got, want[i]) <= bt.LIMIT[dtype], ("sequence", k, "token", i)
        s.release([slot])
    # two sequences that swap slots between uses
    a, b = tokens_for(cfg, 40, 90), tokens_for(cfg, 66, 91)
    for order in ((a, b), (b, a)):
        slots = s.begin(2)
        got = s.step(slots, list(order)).double().cpu().numpy()
        for i, q in enumerate(order):
            assert bt.distance(got[i], truth_of("P", 0, q)[-1]) <= bt.LIMIT[dtype]
        s.release(slots)


# ------------------------------------------------------------------------------ far keys, edges of the table and of pages
def lookup_model(bias_max, bias_rows, heads=2, kv_heads=1, dim=32, vdim=16):
    """One attention layer that looks a token's partner up.  Queries and keys share their matrix and
    read the first half of the width only, values read the second half, and token t + 700 has the
    first half of token t's embedding: so the score of t against t + 700 is as high as against
    itself, wherever the partner stands, while the partner's value is its own.  The delta branch is
    silenced.  In a sequence of otherwise unrelated tokens, about half of the last token's attention
    rests on the one key of its partner, more or less by the bias of that distance."""
    cfg = bt.config(1400, 64, [bt.parallel(bt.attention(heads, kv_heads, dim, vdim, 32.0 / dim, bias_max, bias_rows), bt.delta(2, 2, 8, 8, 2),
                                           None)], scale=2.0)
    w = bt.make_weights(cfg, 5)
    w["embed"][700:, :32] = w["embed"][:700, :32]
    w["l0.mix.left.k"][:, 32:] = 0
    w["l0.mix.left.v"][:, :32] = 0
    w["l0.mix.left.q"] = w["l0.mix.left.k"].repeat(heads // kv_heads, 1)
    w["l0.mix.left.q.norm"] = w["l0.mix.left.k.norm"] = torch.ones(dim, dtype=torch.bfloat16)
    w["l0.mix.right.out"] = torch.zeros_like(w["l0.mix.right.out"])
    w["l0.mix.left.sink"] = torch.full_like(w["l0.mix.left.sink"], 31.0)       # of the size of a match's score (32): it counts
    w["l0.mix.left.rel"] = (0.7 * torch.randn(bias_rows, heads, generator=torch.Generator().manual_seed(1))).to(torch.bfloat16)
    return cfg, w


def distinct_tokens(n, needle_at, vocab, seed):
    """n unrelated tokens, except that the last one's partner stands at `needle_at`."""
    rng = np.random.default_rng(seed)
    tokens = [int(t) for t in rng.permutation(vocab // 2)[:n]]
    tokens[needle_at] = tokens[-1] + vocab // 2
    return tokens


_FAR, _EDGES = {}, {}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("dims", [(32, 16), (64, 64)])
def test_one_far_key_among_hundreds(dims, dtype):
    """The asking token is the last; the key it asks for lies hundreds back, at the first places of
    the sequence, and just before and after page borders.  Both in a prompt and decoded.  (Heads of
    64 go through the matrix-core kernel in bfloat16.)"""
    cfg, w = lookup_model(40.0, 8, dim=dims[0], vdim=dims[1])
    model = bt.load(cfg, w, dtype)
    s = new_session(model, 2048)
    n = 500
    for needle_at in (0, 1, 63, 64, 65, 128, 383, 498):
        tokens = distinct_tokens(n, needle_at, cfg["vocab"], needle_at)
        if (dims, needle_at) not in _FAR:
            other = list(tokens)
            other[needle_at] = next(t for t in range(cfg["vocab"] // 2) if t not in tokens)
            _FAR[(dims, needle_at)] = (bt.plain_logits(cfg, w, tokens)[-1], bt.plain_logits(cfg, w, other)[-1])
        want, missed = _FAR[(dims, needle_at)]
        assert bt.distance(missed, want) > 0.1, "the key must count"
        [slot] = s.begin(1)
        got = s.step([slot], [tokens]).double().cpu().numpy()
        assert bt.distance(got, want) <= bt.LIMIT[dtype], ("prompt", needle_at)
        s.release([slot])
        [slot] = s.begin(1)
        s.step([slot], [tokens[:-1]], [[]])
        got = s.step([slot], [tokens[-1:]]).double().cpu().numpy()
        assert bt.distance(got, want) <= bt.LIMIT[dtype], ("decoded", needle_at)
        s.release([slot])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("bias_max,bias_rows,dims", [(40.0, 8, (32, 16)), (17.5, 6, (32, 16)), (100.0, 32, (32, 16)), (40.0, 8, (128, 64))])
def test_every_distance_across_the_tables_edges(bias_max, bias_rows, dims, dtype):
    """The asked key at every distance from 0 to beyond the table's reach: each row's first and last
    distance is among them.  The rows differ by about 0.5 in the score, which moves the logits by far
    more than the limit."""
    cfg, w = lookup_model(bias_max, bias_rows, dim=dims[0], vdim=dims[1])
    model = bt.load(cfg, w, dtype)
    s = new_session(model, 1024)
    n = int(bias_max) + 12
    from plain import begopel_plain as P
    rows_seen = set()
    for back in range(1, n):
        tokens = distinct_tokens(n, n - 1 - back, cfg["vocab"], back)
        rows_seen.add(P.distance_bucket(back, bias_rows, bias_max))
        key = (bias_max, bias_rows, dims, back)
        if key not in _EDGES:
            _EDGES[key] = bt.plain_logits(cfg, w, tokens)[-1]
        want = _EDGES[key]
        if back % 2:
            got = run_whole(s, tokens)[-1]
        else:
            [slot] = s.begin(1)
            s.step([slot], [tokens[:-1]], [[]])
            got = s.step([slot], [tokens[-1:]]).double().cpu().numpy()
            s.release([slot])
        assert bt.distance(got, want) <= bt.LIMIT[dtype], ("key back by", back)
    assert rows_seen == set(range(1, bias_rows))


def test_neighbouring_rows_of_the_table_differ_in_the_plain_model():
    from plain import begopel_plain as P
    cfg, w = lookup_model(40.0, 8)
    n = 60
    row = lambda back: P.distance_bucket(back, 8, 40.0)
    assert [row(b) for b in (0, 3, 4, 39, 40, 1000)] == [0, 3, 4, 7, 7, 7]
    last_edge = max(b for b in range(1, 40) if row(b) != row(b + 1))         # the last row's first distance is last_edge + 1
    for back in (3, last_edge):       # the last distance with a row of its own; the last two rows
        near, far = (bt.plain_logits(cfg, w, distinct_tokens(n, n - 1 - d, cfg["vocab"], 7))[-1] for d in (back, back + 1))
        assert bt.distance(near, far) > 0.01, back


# ------------------------------------------------------------------------------ long decoding
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", ["P", "R"])
def test_long_decoding_through_recorded_steps(which, dtype):
    """Three sequences decoded 200 tokens, over page borders and beyond the distance tables' reach;
    from the second step of a shape on the engine replays its recording."""
    cfg, w, model = model_of(which, dtype)
    lens, n_dec = [3, 60, 120], 200
    seqs = [tokens_for(cfg, n + n_dec, 70 + i) for i, n in enumerate(lens)]
    truth = [truth_of(which, 0, q) for q in seqs]
    s = new_session(model, 2048)
    slots = s.begin(3)
    s.step(slots, [q[:n] for q, n in zip(seqs, lens)])
    worst = 0.0
    for j in range(n_dec):
        got = s.step(slots, [[q[n + j]] for q, n in zip(seqs, lens)]).double().cpu().numpy()
        for i, n in enumerate(lens):
            worst = max(worst, bt.distance(got[i], truth[i][n + j]))
    assert worst <= bt.LIMIT[dtype]
    assert s.recorded_steps() >= 1
    s.release(slots)


# ------------------------------------------------------------------------------ the entry points
@pytest.fixture(scope="module")
def folder_p(tmp_path_factory):
    cfg = bt.CONFIGS["P"]
    return bt.write_folder(str(tmp_path_factory.mktemp("begopel") / "p"), cfg, bt.make_weights(cfg, 0))


@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_generation_through_the_entry_point(dtype, folder_p):
    import picolm_amd
    cfg = bt.CONFIGS["P"]
    prompts = [tokens_for(cfg, n, 50 + n) for n in (4, 9, 66)]
    got = picolm_amd.generate(folder_p, prompts, max_new_tokens=10, stop_ids=(), dtype=dtype)
    for p, r in zip(prompts, got):
        assert len(r.tokens) == 10 and r.finish == "length"
        seq = list(p)
        for k in range(10):
            lg = truth_of("P", 0, seq)[-1]
            top2 = np.sort(lg)[-2:]
            if top2[1] - top2[0] < 4 * bt.LIMIT[dtype] * lg.std():
                break                              # a near tie: either choice is right
            assert r.tokens[k] == int(np.argmax(lg)), (k, r.tokens)
            seq.append(r.tokens[k])


def test_trace_replay_and_command_line(folder_p, tmp_path):
    """bin/trace_run on a folder: a prompt, single tokens and a second request that joins later in a
    slot that was given back; bin/picolm generates from the same folder."""
    cfg = bt.CONFIGS["P"]
    a, b = tokens_for(cfg, 20, 1), tokens_for(cfg, 9, 2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:17], "want": [0, 16]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[17:18], "want": [0]}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": a[18:19], "want": []}], "end": []},
             {"step": 3, "entries": [{"id": "a", "tokens": a[19:20], "want": [0]}], "end": ["a"]},
             {"step": 4, "entries": [{"id": "b", "tokens": b, "want": [8]}], "end": ["b"]}]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = str(tmp_path / "out")
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder_p, "--dtype", "float32", "--out", out,
                        "--max-tokens", "128"], input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True,
                       timeout=300)
    assert r.returncode == 0, r.stderr
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(5)]
    ta, tb = truth_of("P", 0, a), truth_of("P", 0, b)
    read = lambda i: np.fromfile(os.path.join(out, f"{i}.f32"), dtype="<f4").reshape(-1, cfg["vocab"])
    assert bt.distance(read(0), ta[[0, 16]]) <= bt.LIMIT["float32"]
    assert bt.distance(read(1), ta[17]) <= bt.LIMIT["float32"]
    assert not os.path.exists(os.path.join(out, "2.f32"))
    assert bt.distance(read(3), ta[19]) <= bt.LIMIT["float32"]
    assert bt.distance(read(4), tb[8]) <= bt.LIMIT["float32"]
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "picolm"), folder_p, "-p", " ".join(map(str, b)), "-n", "4", "-t", "0",
                        "--dtype", "float32"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    assert len(r.stdout.split()) == 4
    assert int(r.stdout.split()[0]) == int(np.argmax(tb[-1]))
