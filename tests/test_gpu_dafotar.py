"""Dafotar models through the engine against the plain implementation (tests/plain/dafotar_plain.py):
every way of cutting the work, batches, pages and state slots used again, the edges of the
attention window in prompts and in decoding, keys far back, the first tokens, long decoding, and
greedy generation through ``Engine.generate``.  Small configurations of the tests' own, random
weights; where random weights would hide a fault the scores are made sharp."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

from conftest import ROOT
from dafotar_util import (CFG_A, CFG_B, CFG_C, attention_layer, config, mlstm_layer, random_weights, write_model)
from gpu_util import chunked_steps, make_runner, mixed_steps, run_steps, tail_decode_steps, whole_steps
from plain import dafotar_plain as P

pytestmark = pytest.mark.gpu

CONFIGS = {"A": (CFG_A, 11), "B": (CFG_B, 12), "C": (CFG_C, 13)}
LENGTHS = {"A": [70, 1, 45, 2, 90, 33, 58], "B": [40, 75, 3, 52, 21], "C": [30, 64, 17, 49, 5]}
PAGE = {"A": 4, "B": 8, "C": 16}


def tokens_of(vocab, n, seed):
    return np.random.default_rng(seed).integers(0, vocab, n).tolist()


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name, (cfg, seed) in CONFIGS.items():
        w = random_weights(cfg, seed)
        streams = {f"r{i}": tokens_of(cfg["vocab"], n, 50 + i) for i, n in enumerate(LENGTHS[name])}
        refs = {r: P.forward(cfg, w, t, np.float64) for r, t in streams.items()}
        for dtype in ("float32", "bfloat16"):
            folder = write_model(str(tmp_path_factory.mktemp(f"dafotar{name}_{dtype}")), cfg, w, dtype)
            out[(name, dtype)] = (folder, streams, refs)
    return out


def assert_close(got, want, dtype, what=""):
    """Against the float64 values, relative to the largest logit.  float32 differs by the order of
    its sums alone (these models' logits reach 10 and more).  bfloat16 rounds every product's inputs,
    and these narrow random models amplify that: one layer alone shows 0.3 to 3 % of the largest
    logit, five of them 7 %, a single touchy position 20 %.  So in bfloat16 nine rows in ten must lie
    within 5 % and every row within 30 %; a wrong key, state or stream moves most rows by the
    logits' own size."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    assert got.shape == want.shape, f"{what}: shape {got.shape} vs {want.shape}"
    err = np.abs(got - want).reshape(len(want), -1).max(axis=1) / max(1.0, np.abs(want).max())
    if dtype == "float32":
        ok = err.max() <= 2e-5
    else:
        ok = err.max() <= 0.30 and np.quantile(err, 0.9) <= 0.05
    if not ok:
        raise AssertionError(f"{what}: largest relative error {err.max():.3e} at row {int(np.argmax(err))}, "
                             f"nine in ten below {np.quantile(err, 0.9):.3e}")


def check(rows, refs, dtype, what):
    assert set(rows) == set(refs)
    for r in refs:
        assert_close(rows[r], refs[r], dtype, f"{what} {r}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_every_split_matches_the_plain_implementation(models, name, dtype):
    folder, streams, refs = models[(name, dtype)]
    runner = make_runner(folder, dtype, page_size=PAGE[name], cache_tokens=128, max_seqs=2, max_batch_tokens=128,
                         max_model_len=128)
    whole = run_steps(runner, streams, whole_steps(streams))
    check(whole, refs, dtype, "whole")
    tail = run_steps(runner, streams, tail_decode_steps(streams, tail=40))
    check(tail, refs, dtype, "last 40 one by one")
    one = run_steps(runner, streams, tail_decode_steps(streams, tail=1000))
    check(one, refs, dtype, "token by token")
    chunk = run_steps(runner, streams, chunked_steps(streams))
    check(chunk, refs, dtype, "portions")
    pairs = run_steps(runner, streams, chunked_steps(streams, sizes=(2,)))
    check(pairs, refs, dtype, "portions of two")
    if dtype == "float32":
        # every sum runs in an order fixed by positions alone: the cuts change nothing
        for r in streams:
            for other in (tail, one, chunk, pairs):
                assert np.array_equal(whole[r], other[r]), r
    assert all(p.free_pages == p.num_pages for p in runner.manager.pools)
    assert runner.manager.slots.free_slots == 2


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_mixed_batches_with_pages_and_slots_used_again(models, name, dtype):
    folder, streams, refs = models[(name, dtype)]
    page = PAGE[name]
    pages_of = lambda n: -(-n // page)
    room = sum(sorted((pages_of(len(t)) for t in streams.values()), reverse=True)[:3])
    runner = make_runner(folder, dtype, page_size=page, num_pages=room, max_seqs=3, max_batch_tokens=128,
                         max_model_len=128)
    alone = run_steps(runner, streams, whole_steps(streams))
    for seed in (0, 1):
        steps = mixed_steps(streams, seed=seed, max_live=3, room=room, page=page, decode_tail=9)
        assert any(any(n > 1 for _, n in e) and any(n == 1 for _, n in e) for e, _ in steps)
        slots_seen = {}

        def observe(_):
            for r in runner.manager.live():
                slots_seen.setdefault(runner.manager.slot(r), set()).add(r)

        rows = run_steps(runner, streams, steps, observe)
        check(rows, refs, dtype, f"mixed seed {seed}")
        assert any(len(v) >= 2 for v in slots_seen.values()), "no state slot was used again"
        if dtype == "float32":
            for r in streams:
                assert np.array_equal(rows[r], alone[r]), f"{r} differs from its run alone"
    assert all(p.free_pages == p.num_pages for p in runner.manager.pools)


# ---------------------------------------------------------------- the window's edges, and keys far back
def sharp_attention_model(tmp_path, window, dtype, page=None):
    """One attention layer and nothing else that looks back: no convolution, no recurrence.
    The numbers per head are large, so the softmax is close to a choice of one key and a key
    that is wrongly seen or missed changes the logits by much."""
    cfg = config([attention_layer(heads=2, kv_heads=1, dim=16, vdim=16, window=window, rot_dims=8, base=50.0, ff=32)],
                 vocab=40, width=32, streams=2, taps=None)
    w = random_weights(cfg, 5, temp=12.0)
    return cfg, w, write_model(str(tmp_path / f"sharp_{window}_{dtype}"), cfg, w, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("window", [21, 32])      # not a multiple of the page, and a whole number of pages
def test_keys_just_inside_and_just_outside_the_window(tmp_path, window, dtype):
    cfg, w, folder = sharp_attention_model(tmp_path, window, dtype)
    n = 3 * window + 5
    base = tokens_of(cfg["vocab"], n, 3)
    last = n - 1
    inside, outside = last - window + 1, last - window
    # the two tokens which, standing at the window's first place, pull the last logits furthest apart
    at_edge = []
    for v in range(cfg["vocab"]):
        t = list(base)
        t[inside] = v
        at_edge.append(P.forward(cfg, w, t, np.float64)[last])
    at_edge = np.stack(at_edge)
    gap = np.abs(at_edge[:, None, :] - at_edge[None, :, :]).max(axis=-1)
    va, vb = np.unravel_index(np.argmax(gap), gap.shape)
    base[inside] = int(va)
    changed_in, changed_out = list(base), list(base)
    changed_in[inside] = int(vb)
    changed_out[outside] = (base[outside] + 1) % cfg["vocab"]
    ref = {k: P.forward(cfg, w, t, np.float64) for k, t in (("base", base), ("in", changed_in), ("out", changed_out))}
    # the test's own premise: the key at the edge matters, the one before it cannot
    assert np.abs(ref["in"][last] - ref["base"][last]).max() > 0.05 * np.abs(ref["base"][last]).max()
    assert np.array_equal(ref["out"][last], ref["base"][last])
    runner = make_runner(folder, dtype, page_size=8, cache_tokens=2 * n, max_seqs=2, max_batch_tokens=128, max_model_len=128)
    streams = {"base": base, "in": changed_in, "out": changed_out}
    for how, steps in (("prompt", whole_steps(streams)), ("decoded", tail_decode_steps(streams, tail=window + 3)),
                       ("portions", chunked_steps(streams, sizes=(5, 2, 9)))):
        rows = run_steps(runner, streams, steps)
        for k in streams:
            assert_close(rows[k], ref[k], dtype, f"{how} {k}")
        tol = 0 if dtype == "float32" else 1e-6
        assert np.abs(rows["out"][last] - rows["base"][last]).max() <= tol, f"{how}: a key outside the window was seen"
        assert np.abs(rows["in"][last] - rows["base"][last]).max() > 0.02 * np.abs(ref["base"][last]).max(), how


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_key_hundreds_of_tokens_back(tmp_path, dtype):
    """No mask: the last token's sharp attention picks one key among some three hundred.  The key is
    found through the test's own reading of the plain scores; changing that token changes the logits."""
    cfg = config([attention_layer(heads=1, kv_heads=1, dim=16, vdim=24, window=None, rot_dims=4, base=30.0)],
                 vocab=50, width=32, streams=None, taps=None)
    w = random_weights(cfg, 8, temp=25.0)
    folder = write_model(str(tmp_path / f"far_{dtype}"), cfg, w, dtype)
    n = 330
    base = tokens_of(cfg["vocab"], n, 21)
    ref = P.forward(cfg, w, base, np.float64)
    # the early token whose change moves the last logits most is the far key
    moved = {}
    for j in range(5, 40):
        t = list(base)
        t[j] = (t[j] + 7) % cfg["vocab"]
        moved[j] = np.abs(P.forward(cfg, w, t, np.float64)[-1] - ref[-1]).max()
    far = max(moved, key=moved.get)
    assert moved[far] > 0.05 * np.abs(ref[-1]).max(), "no far key matters in this draw"
    other = list(base)
    other[far] = (other[far] + 7) % cfg["vocab"]
    ref_other = P.forward(cfg, w, other, np.float64)
    runner = make_runner(folder, dtype, page_size=16, cache_tokens=2 * 384, max_seqs=2, max_batch_tokens=512, max_model_len=384)
    streams = {"base": base, "other": other}
    for how, steps in (("prompt", whole_steps(streams)), ("decoded", tail_decode_steps(streams, tail=20)),
                       ("portions", chunked_steps(streams, sizes=(64, 3, 31, 2)))):
        rows = run_steps(runner, streams, steps)
        assert_close(rows["base"], ref, dtype, f"{how} base")
        assert_close(rows["other"], ref_other, dtype, f"{how} other")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_through_every_kind_of_state(models, dtype):
    cfg, seed = CONFIGS["A"]
    folder = models[("A", dtype)][0]
    w = random_weights(cfg, seed)
    toks = tokens_of(cfg["vocab"], 240, 77)
    ref = P.forward(cfg, w, toks, np.float64)
    # every group of this model has a window (7, and 33 for the keys that a later layer reads through
    # a wider window than their owner's): a pool of 64 tokens serves 240 only because pages come back
    runner = make_runner(folder, dtype, page_size=4, cache_tokens=64, max_seqs=1, max_batch_tokens=64, max_model_len=256)
    assert [g.window for g in runner.manager.groups] == [7, 33]
    rows = run_steps(runner, {"r": toks}, tail_decode_steps({"r": toks}, tail=230))
    assert_close(rows["r"], ref, dtype, "230 tokens one by one")


def test_the_first_tokens_of_a_sequence(models):
    """Positions 0, 1, 2: the convolution reads rows before the sequence (zeros), the recurrence
    starts from a zero state with its running maximum at 0, the window holds fewer keys than its size."""
    for name in ("A", "C"):
        cfg, seed = CONFIGS[name]
        folder = models[(name, "float32")][0]
        w = random_weights(cfg, seed)
        runner = make_runner(folder, "float32", page_size=4, cache_tokens=64, max_seqs=2, max_batch_tokens=64, max_model_len=64)
        for n in (1, 2, 3, 4):
            toks = tokens_of(cfg["vocab"], n, 200 + n)
            ref = P.forward(cfg, w, toks, np.float64)
            for steps in (whole_steps({"r": toks}), tail_decode_steps({"r": toks}, tail=10)):
                rows = run_steps(runner, {"r": toks}, steps)
                assert_close(rows["r"], ref, "float32", f"{name}: {n} tokens")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_slot_taken_over_starts_from_zero(models, dtype):
    """One slot, two requests one after the other: the second must not see the first's state."""
    folder, streams, refs = models[("A", dtype)]
    runner = make_runner(folder, dtype, page_size=4, cache_tokens=128, max_seqs=1, max_batch_tokens=128, max_model_len=128)
    for r in ("r0", "r4", "r2", "r0"):
        rows = run_steps(runner, {r: streams[r]}, chunked_steps({r: streams[r]}, sizes=(9, 1, 4)))
        assert_close(rows[r], refs[r], dtype, r)


# ---------------------------------------------------------------- the engine's own entry point
def plain_greedy(cfg, w, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(np.argmax(P.forward(cfg, w, toks, np.float64)[-1])))
    return toks[len(prompt):]


def test_greedy_generation_through_the_engine(models):
    from zse_amd.engine.engine import Engine
    from zse_amd.sampling.sampler import SamplingParams
    cfg, seed = CONFIGS["A"]
    folder = models[("A", "float32")][0]
    w = random_weights(cfg, seed)
    prompts = [tokens_of(cfg["vocab"], n, 300 + n) for n in (5, 23, 1, 40, 12, 31)]
    want = [plain_greedy(cfg, w, p, 12) for p in prompts]
    # four places for six requests, portions of 16: prompts are cut, requests wait for a slot
    with Engine(folder, dtype="float32", block_size=4, num_blocks=64, max_batch_tokens=32, max_batch_seqs=4,
                prefill_chunk_size=16, max_seq_len=128) as eng:
        got = eng.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0))
        assert got == want
        again = eng.generate(prompts[:2], SamplingParams(max_tokens=12, temperature=0.0))
        assert again == want[:2]
    with Engine(folder, dtype="float32", block_size=4, num_blocks=64, max_batch_tokens=32, max_batch_seqs=4,
                prefill_chunk_size=16, max_seq_len=128, use_graphs=False) as eng:
        assert eng.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0)) == want


def test_the_engine_at_its_default_limits(models):
    """No limits given: the longest sequence is the architecture's own default, the pools follow from the
    free memory; a model with windows only, and one that keeps every key."""
    from zse_amd.engine.engine import Engine
    from zse_amd.sampling.sampler import SamplingParams
    for name in ("A", "B"):
        cfg, seed = CONFIGS[name]
        folder = models[(name, "float32")][0]
        w = random_weights(cfg, seed)
        prompt = tokens_of(cfg["vocab"], 19, 500)
        with Engine(folder, dtype="float32") as eng:
            assert eng.generate([prompt], SamplingParams(max_tokens=6, temperature=0.0)) == [plain_greedy(cfg, w, prompt, 6)]
        with Engine(models[(name, "bfloat16")][0], dtype="bfloat16") as eng:
            assert len(eng.generate([prompt], SamplingParams(max_tokens=6, temperature=0.7, top_k=10, seed=1))[0]) == 6


def test_generation_in_bfloat16_does_not_depend_on_the_company(models):
    from zse_amd.engine.engine import Engine
    from zse_amd.sampling.sampler import SamplingParams
    cfg, _ = CONFIGS["A"]
    folder = models[("A", "bfloat16")][0]
    prompts = [tokens_of(cfg["vocab"], n, 400 + n) for n in (9, 30, 17)]
    sp = SamplingParams(max_tokens=10, temperature=0.0)
    with Engine(folder, dtype="bfloat16", block_size=4, num_blocks=64, max_batch_tokens=64, max_batch_seqs=4,
                prefill_chunk_size=64, max_seq_len=128) as eng:
        together = eng.generate(prompts, sp)
        alone = [eng.generate([p], sp)[0] for p in prompts]
    assert together == alone


def test_the_trace_program_serves_the_design(models, tmp_path):
    cfg, seed = CONFIGS["C"]
    folder, streams, refs = models[("C", "float32")]
    out = tmp_path / "out"
    a, b = streams["r0"], streams["r1"]
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:7], "want": [0, 6]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[7:9], "want": []}, {"id": "b", "tokens": b[:40], "want": [39]}], "end": []},
        {"step": 2, "entries": [{"id": "b", "tokens": b[40:41], "want": [0]}, {"id": "a", "tokens": a[9:], "want": [len(a) - 10]}],
         "end": ["a"]},
        {"step": 3, "entries": [{"id": "b", "tokens": b[41:], "want": [len(b) - 42]}], "end": ["b"]},
    ]
    p = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out", str(out),
                        "--max-tokens", "128"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                       capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(4)]
    V = cfg["vocab"]
    read = lambda i: np.fromfile(str(out / f"{i}.f32"), dtype="<f4").reshape(-1, V)
    assert_close(read(0), refs["r0"][[0, 6]], "float32", "step 0")
    assert_close(read(1), refs["r1"][[39]], "float32", "step 1")
    assert_close(read(2), np.stack([refs["r1"][40], refs["r0"][len(a) - 1]]), "float32", "step 2")
    assert_close(read(3), refs["r1"][[len(b) - 1]], "float32", "step 3")
