"""Vobotar on the GPU: whole models through the engine's step function, cache and
state manager against the plain implementation: whole prompts, token-by-token
decoding, portions down to two tokens, mixed batches with pages and state slots
used again, random schedules, long decoding past every window, keys far back
and at the windows' edges, the first tokens of a sequence, other orders and
sizes, and greedy generation through the entry point and the scheduler."""
import os
import random
import subprocess
import sys

import numpy as np
import pytest
import torch

from conftest import ROOT
from trace_util import Trace, compare, compare_with_alone, random_tokens, random_trace, replay
from vobotar_util import (BLOCK_SIZE, CONFIGS, RANKS, attention, config, dense, edit, pair, pair2, plain_greedy, plain_logits,
                          plain_sensitivity, random_config, write_model)

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]

# bfloat16 against the 64-bit plain model on the same rounded weights.  The test models' weights are
# wide (peaked attention, decays and gates that reach their limits); the bounds are per row, of the
# largest logit.  Every branch is normed after its product, and single rows in which a divisor is
# small enlarge their rounding many times: such a row gets an allowance of its own (``check_folder``).
TOL16 = dict(rtol=0.0, atol=1.5e-1, median=4e-2)


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for name, cfg in CONFIGS.items():
        out[name] = {dt: write_model(str(tmp_path_factory.mktemp(f"vobotar{name}_{dt}")), cfg, seed=31 + ord(name), dtype=dt,
                                     rank=RANKS[name]) for dt in DTYPES}
    return out


LENGTHS = {"a": 1, "b": 7, "c": 33, "d": 70, "e": 130}


def requests_for(name, extra=None):
    lens = dict(LENGTHS, **(extra or {}))
    return {rid: random_tokens(n, CONFIGS[name]["vocab"], seed=500 + i) for i, (rid, n) in enumerate(sorted(lens.items()))}


def run(folders, name, dtype, t, **kw):
    return replay(folders[name][dtype], dtype, t, block_size=BLOCK_SIZE[name], **kw)


def check_folder(t, got, folder, dtype, label):
    """32-bit: against the plain model as it is.  16-bit: a row is also allowed sixteen times what its
    logits move by when the weights are changed by one 16-bit rounding step (``plain_sensitivity``: one
    change of every matrix, where the engine rounds a dozen times a layer); the median over a trace's
    rows gets no such allowance."""
    if dtype == "float32":
        compare(t, got, plain_logits(folder, t.requests), dtype, label)
    else:
        slack = {rid: 16.0 * s.numpy() for rid, s in plain_sensitivity(folder, t.requests).items()}
        compare(t, got, plain_logits(folder, t.requests), dtype, label, tol=TOL16, slack=slack)


def check(t, got, folders, name, dtype, label):
    check_folder(t, got, folders[name][dtype], dtype, label)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_whole_prompts(folders, name, dtype):
    for rid, toks in requests_for(name).items():
        t = Trace({rid: toks})
        t.step([(rid, len(toks))], end=[rid])
        check(t, run(folders, name, dtype, t), folders, name, dtype, f"whole {name} {rid}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_prefill_then_token_by_token(folders, name, dtype):
    for rid, toks in requests_for(name).items():
        if len(toks) < 33:
            continue
        t = Trace({rid: toks})
        t.step([(rid, len(toks) - 30)], want="last")
        for _ in range(30):
            t.step([(rid, 1)])
        got = run(folders, name, dtype, t)
        check(t, got, folders, name, dtype, f"decode {name} {rid}")
        if dtype == "float32":
            compare_with_alone(t, got, folders[name][dtype], dtype, f"decode {name} {rid}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_every_token_alone_from_the_first(folders, name, dtype):
    """The first tokens of a sequence one by one: states that start at zero (the row before the
    first, the convolution's inputs, the matrices), a first page, windows that are not yet full."""
    toks = requests_for(name)["d"]
    t = Trace({"d": toks})
    for _ in toks:
        t.step([("d", 1)])
    check(t, run(folders, name, dtype, t), folders, name, dtype, f"one by one {name}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_portions_down_to_two_tokens(folders, name, dtype):
    sizes = [7, 2, 5, 3, 16, 2, 31, 4, 2, 9]
    for rid, toks in requests_for(name).items():
        if len(toks) < 9:
            continue
        t = Trace({rid: toks})
        left, i = len(toks), 0
        while left:
            n = min(sizes[i % len(sizes)], left)
            if left - n == 1:
                n += 1
            t.step([(rid, n)])
            left -= n
            i += 1
        got = run(folders, name, dtype, t)
        check(t, got, folders, name, dtype, f"portions {name} {rid}")
        if dtype == "float32":
            compare_with_alone(t, got, folders[name][dtype], dtype, f"portions {name} {rid}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_mixed_batches_with_pages_and_slots_used_again(folders, name, dtype):
    reqs = requests_for(name, {"f": 90, "g": 12, "h": 50})
    t = Trace(reqs)
    t.step([("d", 40), ("a", 1)], end=["a"])
    t.step([("d", 2), ("b", 4), ("c", 20)])
    t.step([("d", 1), ("b", 1), ("c", 2), ("e", 30)])
    t.step([("b", 1), ("c", 1), ("e", 7)])                              # d sits this one out
    t.step([("d", 27), ("b", 1), ("c", 10)], end=["b", "c"])
    t.step([("e", 1), ("f", 64), ("g", 3)], end=["d"])                  # f and g take the slots and pages of b, c
    t.step([("e", 2), ("f", 1), ("g", 2), ("h", 33)])
    for _ in range(5):
        t.step([("e", 1), ("f", 1), ("g", 1), ("h", 1)])
    t.step([("e", 85), ("f", 20), ("g", 2), ("h", 12)], end=["e", "f", "g", "h"])
    total = sum(64 * -(-len(v) // 64) for v in reqs.values())
    assert t.max_tokens < total, "the pool is meant to be too small for all requests at once"
    got = run(folders, name, dtype, t, num_state_slots=4)
    check(t, got, folders, name, dtype, f"mixed {name}")
    if dtype == "float32":
        compare_with_alone(t, got, folders[name][dtype], dtype, f"mixed {name}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "C"])
def test_random_schedules(folders, name, dtype):
    for seed in range(5):
        rng = random.Random(77 * seed + ord(name))
        reqs, t = random_trace(rng, CONFIGS[name]["vocab"], 150)
        got = run(folders, name, dtype, t, num_state_slots=4)
        check(t, got, folders, name, dtype, f"random schedule {name} {seed}")
        if dtype == "float32":
            compare_with_alone(t, got, folders[name][dtype], dtype, f"random schedule {name} {seed}")


def test_a_slot_used_again_starts_from_zero(folders):
    """One state slot: every request takes the slot the one before it left, with its matrices, its
    convolution inputs and its previous row still in it."""
    name, dtype = "A", "float32"
    reqs = {rid: random_tokens(n, CONFIGS[name]["vocab"], seed=40 + n) for rid, n in (("p", 37), ("q", 5), ("r", 21))}
    t = Trace(reqs)
    t.step([("p", 30)])
    for _ in range(7):
        t.step([("p", 1)])
    t.step([], end=["p"])
    t.step([("q", 1)])
    t.step([("q", 4)], end=["q"])
    t.step([("r", 2)])
    t.step([("r", 19)], end=["r"])
    check(t, run(folders, name, dtype, t, num_state_slots=1), folders, name, dtype, "one slot")


@pytest.mark.parametrize("name", ["A", "C"])
def test_long_decoding_past_every_window(folders, name):
    """400 tokens: most as portions that end inside pages, the last 150 one by one, so that every
    window moves over decoded tokens and pages behind it are given back; the recurrences' matrices
    carry what the first tokens wrote all the way."""
    dtype = "float32"
    toks = random_tokens(400, CONFIGS[name]["vocab"], seed=1)
    t = Trace({"x": toks})
    t.step([("x", 131)], want="last")
    t.step([("x", 119)], want="last")
    for _ in range(150):
        t.step([("x", 1)])
    check(t, run(folders, name, dtype, t), folders, name, dtype, "long decoding")


def sharpen(folder, factor, ends=(".q", ".k", ".q.b", ".k.b")):
    """Multiply the query and key projections of a written model, so that attention singles out few keys."""
    def change(tensors):
        for k in list(tensors):
            if k.endswith(tuple(ends)) and ".right." not in k:
                tensors[k] = (tensors[k].float() * factor).to(tensors[k].dtype)
    edit(folder, change)


@pytest.mark.parametrize("dtype", DTYPES)
def test_far_keys_in_several_partitions(tmp_path, dtype):
    """1,300 tokens through attention on the matrix cores and attention row by row, with scales
    large enough that a query's weight lies on a few keys anywhere in its sight (a thousand tokens
    back too, where there is no window); portions that end inside pages and tiles, then single tokens."""
    cfg = config(211, 96, [attention(4, 2, 32, 32, 1.2, rot=(1e4, 16), softcap=25.0, v_mix=True, mlp=dense(80)),
                           pair((2, 1, 48, 1.0, 300), (2, 16), 1.0, 0.3, mlp=dense(64)),
                           attention(2, 1, 24, 40, 1.0, rot=(1e6, 24), v_mix=False),
                           pair2((4, 2, 16, 16, 1.5, 700, (5e4, 8)), (2, 16, 16, 1, 4, 1), 0.9, 0.4)], side=8)
    folder = write_model(str(tmp_path / "m"), cfg, seed=13, dtype=dtype)
    toks = random_tokens(1300, 211, seed=6)
    t = Trace({"x": toks})
    for n in (511, 3, 258, 490):
        t.step([("x", n)], want="last")
    for _ in range(38):
        t.step([("x", 1)])
    check_folder(t, replay(folder, dtype, t, block_size=16), folder, dtype, "far keys")


def _attention_only(tmp_path, layer, width=64, vocab=97, seed=3):
    """A model whose only path between tokens is one attention layer: what stands beside it is
    silenced (a right branch's scale of zero)."""
    cfg = config(vocab, width, [layer])
    folder = write_model(str(tmp_path / "m"), cfg, seed=seed, dtype="float32")
    return cfg, folder


@pytest.mark.parametrize("kind", ["values are keys", "normed projections"])
@pytest.mark.parametrize("window", [9, 16, 40, 70])
def test_a_token_counts_exactly_while_the_window_holds_it(tmp_path, kind, window):
    """Only attention carries anything between tokens here (the other side of the pair has scale 0).
    Changing one token changes the logits of the positions whose window still holds it, in a portion
    and decoded alone, and of no position beyond: in the engine exactly as in the plain model."""
    dtype = "float32"
    if kind == "values are keys":
        layer = pair((2, 1, 16, 0.6, window), (1, 8), 1.0, 0.0)
    else:
        layer = pair2((2, 2, 16, 16, 0.6, window, (1e4, 8)), (1, 8, 8, 1, 2, 1), 1.0, 0.0)
    cfg, folder = _attention_only(tmp_path, layer)
    n, at = 150, 60
    toks = random_tokens(n, 97, seed=2)
    other = list(toks)
    other[at] = (toks[at] + 5) % 97
    outs = []
    for seq in (toks, other):
        t = Trace({"x": seq})
        t.step([("x", at + window - 3)])            # the portion ends three positions before the window lets go
        for _ in range(8):
            t.step([("x", 1)])
        t.step([("x", n - (at + window - 3) - 8)], end=["x"])
        got = replay(folder, dtype, t, block_size=16)
        check_folder(t, got, folder, dtype, f"window {window}")
        rows = {}
        for step, pairs in t.rows.items():
            for i, (_, pos) in enumerate(pairs):
                rows[pos] = got[step][i]
        outs.append(rows)
    for pos in range(n):
        moved = float(np.abs(outs[0][pos] - outs[1][pos]).max())
        if at <= pos < at + window:
            assert moved > 1e-4, f"position {pos} holds the changed token in its window of {window}"
        else:
            assert moved == 0.0, f"position {pos} cannot see the changed token (window {window}); its logits moved by {moved:.2e}"


def test_attention_depends_on_a_token_far_back(tmp_path):
    """The first token is changed and the last logits of 900 tokens change with it, in the engine as
    in the plain model: full attention with flat weights is the only path from far back."""
    dtype = "float32"
    cfg, folder = _attention_only(tmp_path, attention(2, 1, 16, 16, 0.05, rot=(1e4, 16), softcap=10.0))
    toks = random_tokens(900, 97, seed=2)
    other = [(toks[0] + 5) % 97] + toks[1:]
    outs = []
    for seq in (toks, other):
        t = Trace({"x": seq})
        t.step([("x", 880)], want="last")
        for _ in range(20):
            t.step([("x", 1)])
        got = replay(folder, dtype, t, block_size=16)
        check_folder(t, got, folder, dtype, "a token far back")
        outs.append(got[max(got)][0])
    want = plain_logits(folder, {"a": toks, "b": other})
    moved = float((want["a"][-1] - want["b"][-1]).abs().max())
    assert moved > 1e-4, "the test's model must carry the first token to the end"
    assert abs(float(np.abs(outs[0] - outs[1]).max()) - moved) < 0.05 * moved + 5e-5


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_sink_that_takes_nearly_all_weight_and_one_that_takes_none(tmp_path, dtype):
    cfg = config(131, 48, [pair((2, 2, 16, 0.4, 24), (2, 8), 1.0, 0.5, mlp=dense(64))])
    for value in (12.0, -30.0):
        folder = write_model(str(tmp_path / f"m{int(value)}"), cfg, seed=17, dtype=dtype)
        edit(folder, lambda ts: ts.update({"l0.mix.left.sink": torch.full_like(ts["l0.mix.left.sink"], value)}))
        toks = random_tokens(60, 131, seed=9)
        t = Trace({"x": toks})
        t.step([("x", 31)])
        t.step([("x", 2)])
        for _ in range(27):
            t.step([("x", 1)])
        check_folder(t, replay(folder, dtype, t, block_size=8), folder, dtype, f"sink {value}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_given_shape_of_things_is_not_assumed(tmp_path, dtype):
    """Sizes that are equal, or 1, in one model and not in another: a single layer of each kind with
    one head, keys larger than values and the other way round, fewer key heads than heads where
    another model has as many, a window of one, one tap and six, groups as many as heads, a rotation
    of two values, no feed-forward, no side input and a side input wider than the heads."""
    cases = [
        [attention(1, 1, 8, 24, 1.1, rot=(50.0, 2), softcap=2.0)],
        [attention(6, 2, 12, 4, 0.4, rot=(1e3, 12), v_mix=True, mlp=dense(16)), attention(4, 2, 6, 4, 0.4, v_mix=True)],
        [pair((1, 1, 24, 0.7, 1), (1, 24), 0.5, 2.0)],
        [pair((6, 3, 4, 0.9, 5), (5, 4), 1.0, 1.0, mlp=dense(24)), pair((2, 2, 20, 0.3, None), (2, 12))],
        [pair2((1, 1, 4, 20, 0.8, 3, None), (1, 4, 20, 1, 6, 1), 1.0, 1.0)],
        [pair2((4, 1, 20, 4, 0.5, None, (10.0, 20)), (4, 6, 5, 4, 1, 4), 2.0, 0.5, mlp=dense(20)),
         pair2((2, 2, 8, 8, 0.5, 64, (1e4, 2)), (6, 2, 3, 2, 2, 3), 0.5, 0.5)],
    ]
    for n, layers in enumerate(cases):
        cfg = config(97, 40, layers, eps=1e-4, scale=(1.0, 0.3, 2.0)[n % 3], side=(0, 3, 24)[n % 3])
        folder = write_model(str(tmp_path / f"m{n}"), cfg, seed=5 + n, dtype=dtype, rank=(3, 9, 2)[n % 3])
        toks = random_tokens(45, 97, seed=3)
        t = Trace({"x": toks})
        t.step([("x", 20)])
        t.step([("x", 2)])
        for _ in range(23):
            t.step([("x", 1)])
        check_folder(t, replay(folder, dtype, t, block_size=8), folder, dtype, f"one of everything {n}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("layers", ["heads of 128 and of 80", "rows of no whole 16 bytes", "recurrences of 256", "pairs first",
                                    "matrix cores everywhere", "many heads"])
def test_other_orders_and_sizes(tmp_path, dtype, layers):
    width = 64
    if layers == "heads of 128 and of 80":
        width = 128
        cfg = [attention(2, 1, 128, 128, 0.09, rot=(1e4, 64), softcap=15.0, v_mix=True, mlp=dense(64)),
               pair((2, 2, 80, 0.1, 50), (1, 64), 0.5, 0.5, mlp=dense(64)),
               pair2((2, 1, 128, 128, 0.09, 100, (1e5, 128)), (2, 32, 64, 1, 4, 2), 0.7, 0.7)]
    elif layers == "rows of no whole 16 bytes":
        width = 100
        cfg = [attention(5, 5, 6, 7, 0.5, rot=(100.0, 6), softcap=7.0, v_mix=True, mlp=dense(52)),
               pair((5, 5, 12, 0.5, 9), (5, 7), 0.9, 1.1, mlp=dense(36)),
               pair2((3, 3, 10, 14, 0.4, 11, (1e3, 6)), (5, 3, 7, 5, 3, 5), 1.0, 1.0)]
    elif layers == "recurrences of 256":
        cfg = [pair((1, 1, 16, 0.5, 30), (1, 256), 0.5, 1.0, mlp=dense(32)),
               pair2((1, 1, 16, 16, 0.5, 30, None), (2, 8, 200, 1, 2, 1), 0.5, 1.0), pair((2, 1, 16, 0.5, 20), (2, 72))]
    elif layers == "pairs first":
        cfg = [pair2((4, 4, 16, 16, 0.5, 40, (1e4, 16)), (4, 8, 16, 2, 4, 2), 1.0, 1.0, mlp=dense(40)),
               pair((4, 4, 16, 0.5, 33), (4, 8), 1.0, 1.0, mlp=dense(40)),
               attention(2, 1, 32, 32, 0.3, rot=(1e4, 32), softcap=10.0, v_mix=True, mlp=dense(40)),
               pair((2, 1, 32, 0.3, 50), (2, 16), 0.5, 1.5)]
    elif layers == "matrix cores everywhere":
        cfg = [attention(4, 2, 16, 16, 0.5, rot=(1e4, 8), softcap=6.0, v_mix=True, mlp=dense(48)),
               pair((4, 1, 48, 0.25, 37), (2, 16), 0.7, 0.7, mlp=dense(48)),
               attention(2, 2, 16, 16, 0.5, v_mix=True),
               pair2((2, 1, 48, 48, 0.25, 19, (1e4, 48)), (2, 16, 16, 2, 3, 1), 0.7, 0.7)]
    else:
        cfg = [attention(32, 2, 16, 16, 0.4, rot=(1e4, 16), softcap=8.0, mlp=dense(32)),
               pair((20, 20, 16, 0.4, 25), (8, 8), 1.0, 1.0)]
    cfg = config(111, width, cfg, side=4)
    folder = write_model(str(tmp_path / "m"), cfg, seed=9, dtype=dtype)
    reqs = {"x": random_tokens(80, 111, seed=1), "y": random_tokens(21, 111, seed=2)}
    t = Trace(reqs)
    t.step([("x", 30)])
    t.step([("x", 3), ("y", 19)])
    for _ in range(2):
        t.step([("x", 1), ("y", 1)])
    t.step([("x", 45)], end=["x", "y"])
    check_folder(t, replay(folder, dtype, t, block_size=16 if "heads of" in layers else 8), folder, dtype, layers)


@pytest.mark.parametrize("seed", range(12))
def test_random_configurations_under_random_schedules(tmp_path, seed):
    """Configurations and schedules drawn at random, in 32-bit, where the engine must agree with the
    plain model to 1e-4 of the largest logit and what a row's own sensitivity explains (a 32-bit
    rounding step is 2^-15 of the 16-bit one that ``plain_sensitivity`` measures)."""
    rng = random.Random(9000 + seed)
    cfg = random_config(rng)
    folder = write_model(str(tmp_path / "m"), cfg, seed=seed, dtype="float32", rank=rng.choice([3, 8, 16]))
    reqs, t = random_trace(rng, cfg["vocab"], rng.choice([60, 150, 300]))
    got = replay(folder, "float32", t, block_size=rng.choice([4, 8, 16]), num_state_slots=4)
    slack = {rid: 16.0 * 2.0 ** -15 * s.numpy() for rid, s in plain_sensitivity(folder, t.requests).items()}
    compare(t, got, plain_logits(folder, t.requests), "float32", f"random configuration {seed}", tol=dict(rtol=1e-4, atol=1e-4),
            slack=slack)


# ------------------------------------------------------------------- generation
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "C"])
def test_greedy_generation_through_the_entry_point(folders, name, dtype):
    import lyapunov_engine_amd as L

    folder = folders[name][dtype]
    prompts = [random_tokens(n, CONFIGS[name]["vocab"], seed=60 + n) for n in (3, 19, 40)]
    llm = L.LLM(folder, dtype=dtype, num_blocks=96, block_size=BLOCK_SIZE[name], max_num_batched_tokens=32)
    outs = llm.generate(prompts, L.SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True))
    for prompt, o in zip(prompts, outs):
        assert o.finished and o.prompt_tokens == prompt and len(o.output_tokens) == 12
        want, margins = plain_greedy(folder, prompt, 12)
        close = [i for i, m in enumerate(margins) if m < (1e-3 if dtype == "float32" else 0.3)]
        upto = close[0] if close else 12
        assert o.output_tokens[:upto] == want[:upto]


def test_generation_with_and_without_recorded_steps_and_with_preemption(folders):
    import lyapunov_engine_amd as L

    folder = folders["C"]["float32"]
    prompts = [random_tokens(n, CONFIGS["C"]["vocab"], seed=80 + n) for n in (5, 30, 61, 12)]
    sp = L.SamplingParams(temperature=0.0, max_tokens=20, ignore_eos=True)
    want = [plain_greedy(folder, p, 20)[0] for p in prompts]
    for kw in (dict(enable_graphs=True, num_blocks=64), dict(enable_graphs=False, num_blocks=64),
               dict(enable_graphs=True, num_blocks=12, max_num_batched_tokens=24)):   # few pages: preemption
        outs = L.LLM(folder, dtype="float32", block_size=16, **kw).generate(prompts, sp)
        assert [o.output_tokens for o in outs] == want, kw


def test_command_line_generate(folders):
    folder = folders["A"]["float32"]
    prompt = random_tokens(9, CONFIGS["A"]["vocab"], seed=8)
    want, _ = plain_greedy(folder, prompt, 8)
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "lyapunov"), "generate", "--model", folder,
                           "--prompt-ids", ",".join(map(str, prompt)), "--max-tokens", "8", "--temperature", "0",
                           "--dtype", "float32", "--block-size", "4", "--num-blocks", "32"],
                          capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert proc.stdout.strip().splitlines()[-1].split() == [str(t) for t in want]


def test_trace_runner_as_a_program(folders, tmp_path):
    import json

    folder = folders["A"]["float32"]
    toks = random_tokens(30, CONFIGS["A"]["vocab"], seed=4)
    steps = [{"step": 0, "entries": [{"id": "r", "tokens": toks[:17], "want": [0, 16]}], "end": []},
             {"step": 1, "entries": [{"id": "r", "tokens": toks[17:18], "want": [0]}], "end": []},
             {"step": 2, "entries": [{"id": "r", "tokens": toks[18:], "want": [11]}], "end": ["r"]}]
    out = tmp_path / "out"
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32",
                           "--out", str(out), "--max-tokens", "64"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                          capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    want = plain_logits(folder, {"r": toks})["r"].numpy()
    for step, rows in ((0, [0, 16]), (1, [17]), (2, [29])):
        got = np.fromfile(out / f"{step}.f32", dtype="<f4").reshape(len(rows), -1)
        assert np.abs(got - want[rows]).max() < 5e-4 * max(1.0, np.abs(want[rows]).max())
