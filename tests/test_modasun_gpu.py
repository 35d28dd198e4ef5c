"""The Modasun decoder through the engine against the plain implementation: whole prompts, decoding
through cache and state, portions down to two tokens, unequal batches, slots and pages used again, sizes
of several kinds, far keys and long memories, the edges of the positions at which a query grows and of
the expert groups, greedy generation through the entry point, the trace program and the command line;
float32 and bfloat16."""
import numpy as np
import pytest
import torch

import herbert_rs_amd as hb
from herbert_rs_amd.engine import StepEntry

from . import replay_util as ru
from .bounds import BF16_REL_RMS, close
from .modasun_tiny import CONFIGS, make_folder, plain_folder, plain_logits, random_tokens
from .plain import modasun as plain

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]

# In bfloat16 the router sees rows that differ from the plain ones by their rounding, and of a few hundred
# choices among close scores some fall the other way: such a token then runs through another expert, which
# no bound on rounding covers, and a delta layer's state and the keys carry it on to later tokens. Float32 is
# compared row by row without exception. In bfloat16 a share of the rows may be off where experts are chosen
# (the mechanisms alone, where nothing is chosen, are held to the rounding of their kernels in
# test_modasun_kernels_gpu.py); where every expert runs (F, R) one row in fifty may pass the bound, by half of it
# at most: the tail of the rounding of rows as narrow as 64.
FLIPPED_SHARE = 0.25
TAIL_SHARE, TAIL_FACTOR = 0.02, 1.5


def compare(rows, folder, tokens, positions, dtype, label):
    ref = plain_logits(folder, tokens)
    name = label.split()[0]
    raw = CONFIGS[name][0]
    every = all(l["mlp"] is None or l["mlp"]["kind"] == "dense" or l["mlp"]["router"]["top"] == l["mlp"]["router"]["experts"]
                for l in raw["layers"])
    off = []
    for row, p in zip(rows, positions):
        assert np.isfinite(np.asarray(row)).all(), f"{label}: position {p} is not finite"
        ok, err = close(np.asarray(row), ref[p], dtype, "mod", label)
        if not ok:
            off.append((p, err))
    n = len(list(positions))
    if dtype == "float32":
        assert not off, f"{label}: positions and errors {off[:5]}"
    elif every:
        assert len(off) <= max(1, TAIL_SHARE * n) and all(e <= TAIL_FACTOR * BF16_REL_RMS["mod"] for _, e in off), \
            f"{label}: positions and errors {off[:5]}"
    else:
        assert len(off) <= max(3, FLIPPED_SHARE * n), f"{label}: {len(off)} of {n} rows off: {off[:5]}"


def feed(engine, slot, tokens, cuts):
    """The tokens of one sequence in portions that end at `cuts`; every position's logits, in order."""
    rows, at = [], 0
    for end in list(cuts) + [len(tokens)]:
        if end <= at:
            continue
        part = tokens[at:end]
        rows.append(engine.step([StepEntry(slot, part, list(range(len(part))))]).cpu().numpy())
        at = end
    return np.concatenate(rows)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["P", "Q", "R", "S", "N"])
def test_whole_prompts_and_token_by_token(name, dtype, model_root):
    folder = make_folder(model_root, name, dtype)
    vocab = CONFIGS[name][0]["vocab"]
    engine = hb.load(folder, dtype=dtype, cache_tokens=1024)
    for n, seed in ((1, 1), (2, 2), (67, 3), (150, 4)):
        tokens = random_tokens(vocab, n, seed)
        slot = engine.alloc_slot()
        compare(feed(engine, slot, tokens, []), folder, tokens, range(n), dtype, f"{name} whole")
        engine.free_slot(slot)
    # the first tokens of a sequence one by one, then on through a page's edge: the state of a fresh slot,
    # the filter's empty past, the first keys, the first positions at which a query grows
    tokens = random_tokens(vocab, 70, 5)
    slot = engine.alloc_slot()
    compare(feed(engine, slot, tokens, range(1, 70)), folder, tokens, range(70), dtype, f"{name} one by one")
    engine.free_slot(slot)
    engine.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["P", "Q"])
def test_portions_of_several_sizes_and_slots_used_again(name, dtype, model_root):
    folder = make_folder(model_root, name, dtype)
    vocab = CONFIGS[name][0]["vocab"]
    engine = hb.load(folder, dtype=dtype, cache_tokens=512)
    tokens = random_tokens(vocab, 200, 21)
    for cuts in ([2, 4, 7], [64, 128], [63, 65, 127, 129, 192], [1, 3, 100, 102, 199], [150]):
        slot = engine.alloc_slot()
        compare(feed(engine, slot, tokens, cuts), folder, tokens, range(200), dtype, f"{name} portions")
        engine.free_slot(slot)           # the next pass takes the same slot and pages: nothing of this one may stay
    engine.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["P", "Q", "R", "S", "N"])
def test_unequal_batches_against_each_alone(name, dtype, model_root):
    folder = make_folder(model_root, name, dtype)
    vocab = CONFIGS[name][0]["vocab"]
    engine = hb.load(folder, dtype=dtype, cache_tokens=1024)
    lengths = [1, 90, 33, 140, 64]
    seqs = [random_tokens(vocab, n + 12, 40 + i) for i, n in enumerate(lengths)]
    for again in range(2):               # twice: the second time the slots and pages were used before
        slots = [engine.alloc_slot() for _ in seqs]
        out = engine.step([StepEntry(s, t[:n], list(range(n))) for s, t, n in zip(slots, seqs, lengths)]).cpu().numpy()
        at = 0
        for t, n in zip(seqs, lengths):
            compare(out[at:at + n], folder, t, range(n), dtype, f"{name} batch prompts")
            at += n
        live = list(range(len(seqs)))
        for step in range(12):
            if step == 5:                # a sequence ends early; its slot goes back while the others go on
                engine.free_slot(slots[live.pop(1)])
            out = engine.step([StepEntry(slots[i], [seqs[i][lengths[i] + step]], [0]) for i in live]).cpu().numpy()
            for row, i in zip(out, live):
                compare([row], folder, seqs[i], [lengths[i] + step], dtype, f"{name} batch decode")
        for i in live:
            engine.free_slot(slots[i])
        engine.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding(dtype, model_root):
    """300 tokens one by one: the decode steps replayed as graphs, the query's factor stepping up every 32
    positions, the pages' edges, the state carried on."""
    folder = make_folder(model_root, "Q", dtype)
    vocab = CONFIGS["Q"][0]["vocab"]
    engine = hb.load(folder, dtype=dtype, cache_tokens=512)
    tokens = random_tokens(vocab, 330, 77)
    slot = engine.alloc_slot()
    compare(feed(engine, slot, tokens, [30] + list(range(31, 330))), folder, tokens, range(330), dtype, "Q long decode")
    engine.free_slot(slot)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_far_key_and_a_long_memory_show(dtype, model_root):
    """Scores three times as sharp as a random model's, so that few keys hold a query's weight, and decays near
    one, so that the state remembers the sequence's start: the logits then depend on tokens hundreds back, in
    the prompt and in decoding, across the pages' edges. That they do is checked on the plain implementation."""
    folder = make_folder(model_root, "F", dtype, set_to={".mix.A_log": -6.0}, tag="_long")
    vocab = CONFIGS["F"][0]["vocab"]
    tokens = random_tokens(vocab, 400, 91)
    cfg, w = plain_folder(folder)
    a = plain_logits(folder, tokens)[-1]
    for changed in (3, 70):
        other = list(tokens)
        other[changed] = (other[changed] + 1) % vocab
        b = plain.forward(cfg, w, other, rows=[399])[0].numpy()
        assert np.abs(a - b).max() > 0.005 * np.abs(a).max(), f"token {changed} does not show in the plain logits"
    engine = hb.load(folder, dtype=dtype, cache_tokens=1024)
    for cuts in ([], [128, 256], [360] + list(range(361, 400))):
        slot = engine.alloc_slot()
        compare(feed(engine, slot, tokens, cuts), folder, tokens, range(400), dtype, "F far")
        engine.free_slot(slot)


@pytest.mark.parametrize("dtype", DTYPES)
def test_wider_layers(dtype, model_root):
    """Heads of 128 and sixteen experts of 256: the sizes of a larger model's layers."""
    folder = make_folder(model_root, "W", dtype)
    vocab = CONFIGS["W"][0]["vocab"]
    engine = hb.load(folder, dtype=dtype, cache_tokens=1024)
    tokens = random_tokens(vocab, 300, 5)
    rows = [0, 1, 63, 64, 100, 126, 127, 128, 255, 256, 279]
    slot = engine.alloc_slot()
    out = engine.step([StepEntry(slot, tokens[:280], rows)]).cpu().numpy()
    compare(out, folder, tokens, rows, dtype, "W prompt")
    for p in range(280, 300):
        out = engine.step([StepEntry(slot, [tokens[p]], [0])]).cpu().numpy()
        compare(out, folder, tokens, [p], dtype, "W decode")
    engine.free_slot(slot)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["P", "Q"])
def test_greedy_generation_through_the_entry_point(name, dtype, model_root):
    folder = make_folder(model_root, name, dtype)
    vocab = CONFIGS[name][0]["vocab"]
    cfg, w = plain_folder(folder)
    prompts = [random_tokens(vocab, n, 60 + n) for n in (9, 1, 70)]
    got = hb.generate(folder, prompts, temperature=0.0, max_tokens=10, ignore_eos=True, no_repeat_check=True, dtype=dtype)
    for p, g in zip(prompts, got):
        assert len(g) == 10
        if dtype == "float32":
            assert g == plain.greedy(cfg, w, p, 10)
            continue
        seq = list(p)                    # bfloat16 may flip a near-tie: the token must then be close to the best
        for tok in g:
            logits = plain.forward(cfg, w, seq, rows=[len(seq) - 1])[0]
            assert float(logits.max() - logits[tok]) <= 0.05 * float(logits.std()) + 1e-6
            seq.append(tok)


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_trace_program(dtype, model_root, tmp_path):
    folder = make_folder(model_root, "P", dtype)
    vocab = CONFIGS["P"][0]["vocab"]
    reqs = {f"r{i}": random_tokens(vocab, n, 200 + i) for i, n in enumerate([5, 130, 1, 66, 40])}
    for label, steps in (("whole", ru.trace_whole(reqs)), ("tail", ru.trace_tail(reqs, 20)),
                         ("batches", ru.trace_batches(reqs, 3, 0.6))):
        held = max(sum(len(t) for t in reqs.values()), 1)
        out = ru.run_trace(folder, dtype, steps, str(tmp_path / label), held, vocab)
        got = ru.collect(steps, out)
        assert len(got) == sum(len(t) for t in reqs.values())
        for (rid, pos), row in got.items():
            compare([row], folder, reqs[rid], [pos], dtype, f"P trace {label}")


def test_a_folder_whose_configuration_leaves_sizes_to_the_tensors(model_root, tmp_path):
    """The narrow middles of a delta layer's two-step projections need not be named: the stored tensors give them."""
    import json
    import os
    import shutil
    folder = make_folder(model_root, "P", "float32")
    bare = str(tmp_path / "bare")
    shutil.copytree(folder, bare)
    raw = json.load(open(os.path.join(bare, "config.json")))
    for layer in raw["layers"]:
        layer["mixer"].pop("low_rank", None)
    json.dump(raw, open(os.path.join(bare, "config.json"), "w"))
    tokens = random_tokens(raw["vocab"], 40, 8)
    engine = hb.load(bare, dtype="float32", cache_tokens=256)
    slot = engine.alloc_slot()
    compare(feed(engine, slot, tokens, [17]), folder, tokens, range(40), "float32", "P bare")


def test_the_command_line_generates_token_ids(model_root):
    """The command line serves the family as it serves any other: token ids in, token ids out (--max-tokens 6 gives
    seven tokens: it counts the decode steps after the prompt's own token), with sampling parameters too."""
    import os
    import subprocess
    import sys
    folder = make_folder(model_root, "P", "float32")
    cfg, w = plain_folder(folder)
    cli = os.path.join(ru.ROOT, "bin", "herbert-cli")
    out = subprocess.run([sys.executable, cli, "--model", folder, "--prompt", "5,17,3,190", "--temperature", "0",
                          "--max-tokens", "6", "--dtype", "float32", "--ignore-eos", "--no-repeat-check", "--verbose"],
                         capture_output=True, text=True, timeout=240)
    assert out.returncode == 0, out.stderr
    assert [int(t) for t in out.stdout.strip().split(",")] == plain.greedy(cfg, w, [5, 17, 3, 190], 7)
    drawn = [subprocess.run([sys.executable, cli, "--model", folder, "--prompt", "5,17,3,190", "--temperature", "0.8",
                             "--top-k", "20", "--top-p", "0.9", "--seed", "3", "--max-tokens", "6", "--dtype", "float32",
                             "--ignore-eos", "--no-repeat-check"], capture_output=True, text=True, timeout=240)
             for _ in range(2)]
    assert all(d.returncode == 0 for d in drawn), drawn[0].stderr
    assert drawn[0].stdout == drawn[1].stdout and len(drawn[0].stdout.strip().split(",")) == 7
