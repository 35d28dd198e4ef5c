"""The Vipalorn decoder through the engine against the plain implementation: whole prompts, decoding
through cache and state, portions, unequal batches, slots used again, sizes of several kinds, greedy
generation through the entry point and the trace program; float32 and bfloat16."""
import numpy as np
import pytest
import torch

import herbert_rs_amd as hb
from herbert_rs_amd.engine import StepEntry

from . import replay_util as ru
from .bounds import close
from .plain import vipalorn as plain
from .vipalorn_tiny import CONFIGS, make_folder, plain_folder, plain_logits, random_tokens

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]


# In bfloat16 the router sees rows that differ from the plain ones by their rounding, and of a few hundred
# choices among close logits some fall the other way: such a token then runs through another expert,
# which no bound on rounding covers. Float32 is compared row by row without exception, and so is
# bfloat16 where every expert is chosen (R); elsewhere a small share of the bfloat16 rows may be off,
# and the rest must be as close as ever.
FLIPPED_SHARE = {"S": 0.25}          # (twelve experts in four layers: more close calls, and the state carries one on)


def compare(rows, folder, tokens, positions, dtype, label):
    ref = plain_logits(folder, tokens)
    name = label.split()[0]
    raw = CONFIGS[name][0]
    every = all(l["mlp"] is None or l["mlp"]["router"]["top"] == l["mlp"]["router"]["experts"] for l in raw["layers"])
    off = []
    for row, p in zip(rows, positions):
        assert np.isfinite(np.asarray(row)).all(), f"{label}: position {p} is not finite"
        ok, err = close(np.asarray(row), ref[p], dtype, "vip", label)
        if not ok:
            off.append((p, err))
    if dtype == "float32" or every:
        assert not off, f"{label}: positions and errors {off[:5]}"
    else:
        assert len(off) <= max(3, FLIPPED_SHARE.get(name, 0.06) * len(list(positions))), f"{label}: {len(off)} rows off: {off[:5]}"


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
@pytest.mark.parametrize("name", ["P", "Q", "R", "S"])
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
    # the filter's empty past, the first keys
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
        engine.free_slot(slot)           # the next round takes the same slot and pages: nothing of this one may stay
    engine.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["P", "Q", "R", "S"])
def test_unequal_batches_against_each_alone(name, dtype, model_root):
    folder = make_folder(model_root, name, dtype)
    vocab = CONFIGS[name][0]["vocab"]
    engine = hb.load(folder, dtype=dtype, cache_tokens=1024)
    lengths = [1, 90, 33, 140, 64]
    seqs = [random_tokens(vocab, n + 12, 40 + i) for i, n in enumerate(lengths)]
    for round_ in range(2):              # twice: the second round's slots and pages were used before
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
    folder = make_folder(model_root, "Q", dtype)
    vocab = CONFIGS["Q"][0]["vocab"]
    engine = hb.load(folder, dtype=dtype, cache_tokens=512)
    tokens = random_tokens(vocab, 330, 77)
    slot = engine.alloc_slot()
    compare(feed(engine, slot, tokens, [30] + list(range(31, 330))), folder, tokens, range(330), dtype, "Q long decode")
    engine.free_slot(slot)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_far_key_and_a_long_memory_show(dtype, model_root):
    """Queries and latents scaled up so that few keys hold a query's weight, decays near one so that the
    state remembers the sequence's start: the logits then depend on tokens hundreds back, in the prompt
    and in decoding, across the pages' edges. That they do is checked on the plain implementation."""
    folder = make_folder(model_root, "Q", dtype, scale={".mix.q": 6.0, ".mix.uk": 3.0}, set_to={".mix.A_log": -5.0},
                         tag="_sharp")
    vocab = CONFIGS["Q"][0]["vocab"]
    tokens = random_tokens(vocab, 400, 91)
    other = list(tokens)
    other[3] = (other[3] + 1) % vocab
    cfg, w = plain_folder(folder)
    a, b = plain_logits(folder, tokens)[-1], plain.forward(cfg, w, other, rows=[399])[0].numpy()
    assert np.abs(a - b).max() > 0.005 * np.abs(a).max(), "the far token does not show in the plain logits"   # (fifty times the float32 bound)
    engine = hb.load(folder, dtype=dtype, cache_tokens=1024)
    for cuts in ([], [128, 256], [360] + list(range(361, 400))):
        slot = engine.alloc_slot()
        compare(feed(engine, slot, tokens, cuts), folder, tokens, range(400), dtype, "Q sharp")
        engine.free_slot(slot)


@pytest.mark.parametrize("dtype", DTYPES)
def test_wider_layers(dtype, model_root):
    """Keys of 128 a head and a latent of 256 + 64: the sizes of a larger model's layers."""
    folder = make_folder(model_root, "W", dtype)
    vocab = CONFIGS["W"][0]["vocab"]
    engine = hb.load(folder, dtype=dtype, cache_tokens=1024)
    tokens = random_tokens(vocab, 300, 5)
    rows = [0, 1, 63, 64, 100, 255, 256, 280, 299]
    slot = engine.alloc_slot()
    out = engine.step([StepEntry(slot, tokens[:280], [r for r in rows if r < 280])]).cpu().numpy()
    compare(out, folder, tokens, [r for r in rows if r < 280], dtype, "W prompt")
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


def test_configuration_errors_and_the_registry(model_root):
    from herbert_rs_amd.config import load_config
    from herbert_rs_amd.errors import ConfigError
    folder = make_folder(model_root, "R", "float32")
    arch, cfg = load_config(folder)
    assert arch.name == "Vipalorn" and cfg.layers[0].type == "delta" and cfg.layers[0].mlp is None
    assert type(cfg).from_dict(cfg.to_dict()) == cfg
    raw = cfg.to_dict()
    raw["layers"][0]["type"] = "other"
    with pytest.raises(ConfigError):
        type(cfg).from_dict(raw)
