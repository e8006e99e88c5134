"""Tonilix on the GPU: whole models through the engine's step function, cache and
state manager against the plain implementation: whole prompts, token-by-token
decoding, portions down to two tokens, mixed batches with pages and state slots
used again, random schedules, long decoding, keys far back, the positions where
the query multiplier steps, and greedy generation through the entry point and
the scheduler."""
import os
import random
import subprocess
import sys

import numpy as np
import pytest
import torch

from conftest import ROOT
from tonilix_util import (BLOCK_SIZE, CONFIGS, RANKS, RouterLog, config, delta, dense, moe, pair, plain_greedy, plain_logits,
                          plain_logits_routed_alike, write_model)
from trace_util import Trace, compare, compare_with_alone, random_tokens, random_trace, replay

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]
DEV = "cuda:0"


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for name, cfg in CONFIGS.items():
        out[name] = {dt: write_model(str(tmp_path_factory.mktemp(f"tonilix{name}_{dt}")), cfg, seed=31 + ord(name), dtype=dt,
                                     ranks=RANKS[name]) for dt in DTYPES}
    return out


LENGTHS = {"a": 1, "b": 7, "c": 33, "d": 70, "e": 130}


def requests_for(name, extra=None):
    lens = dict(LENGTHS, **(extra or {}))
    return {rid: random_tokens(n, CONFIGS[name]["vocab"], seed=500 + i) for i, (rid, n) in enumerate(sorted(lens.items()))}


def run_folder(folder, dtype, t, **kw):
    """Replay the trace; the engine's router choices go along with it (``t.routing``)."""
    with RouterLog() as log:
        got = replay(folder, dtype, t, **kw)
    t.routing = log.by_request(t)
    return got


def run(folders, name, dtype, t):
    return run_folder(folders[name][dtype], dtype, t, block_size=BLOCK_SIZE[name])


# bfloat16 against the 64-bit plain model on the same rounded weights.  The test models' weights are
# wide (peaked attention, decays and gates that reach their limits, routers that decide clearly), so
# rounding shows more than in a trained model; the bounds are per row, of the largest logit.
TOL16 = dict(rtol=0.0, atol=1.5e-1, median=4e-2)


def check_folder(t, got, folder, dtype, label):
    """32-bit: against the plain model as it is.  16-bit: against the plain model with the engine's
    router choices (a close call decided the other way is no fault of a kernel; a clear one is, and
    is asserted), on the same rounded weights."""
    if dtype == "float32":
        compare(t, got, plain_logits(folder, t.requests), dtype, label)
    else:
        compare(t, got, plain_logits_routed_alike(folder, t.requests, t.routing), dtype, label, tol=TOL16)


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
    """The first tokens of a sequence one by one: states that start at zero (the shift's previous
    token, the convolution's inputs, the matrices), a first page, the first steps of the multiplier."""
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
    got = run_folder(folders[name][dtype], dtype, t, block_size=BLOCK_SIZE[name], num_state_slots=4)
    check(t, got, folders, name, dtype, f"mixed {name}")
    if dtype == "float32":
        compare_with_alone(t, got, folders[name][dtype], dtype, f"mixed {name}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B"])
def test_random_schedules(folders, name, dtype):
    for seed in range(5):
        rng = random.Random(77 * seed + ord(name))
        reqs, t = random_trace(rng, CONFIGS[name]["vocab"], 150)
        got = run_folder(folders[name][dtype], dtype, t, block_size=BLOCK_SIZE[name], num_state_slots=4)
        check(t, got, folders, name, dtype, f"random schedule {name} {seed}")
        if dtype == "float32":
            compare_with_alone(t, got, folders[name][dtype], dtype, f"random schedule {name} {seed}")


def test_a_slot_used_again_starts_from_zero(folders):
    """One state slot: every request takes the slot the one before it left, with its matrices, its
    convolution inputs and its previous token still in it."""
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
    got = run_folder(folders[name][dtype], dtype, t, block_size=BLOCK_SIZE[name], num_state_slots=1)
    check(t, got, folders, name, dtype, "one slot")


@pytest.mark.parametrize("name", ["B", "C"])
def test_long_decoding(folders, name):
    """400 tokens: most as portions that end inside pages, the last 150 one by one; the recurrences'
    matrices carry what the first tokens wrote all the way."""
    dtype = "float32"
    toks = random_tokens(400, CONFIGS[name]["vocab"], seed=1)
    t = Trace({"x": toks})
    t.step([("x", 131)], want="last")
    t.step([("x", 119)], want="last")
    for _ in range(150):
        t.step([("x", 1)])
    check(t, run(folders, name, dtype, t), folders, name, dtype, "long decoding")


def sharpen(folder, factor, names=("left.q", "left.k")):
    """Multiply some matrices of a written model, so that attention singles out few keys."""
    from lyapunov_engine_amd.weights.safetensors_io import write_safetensors
    from plain.tonilix_plain import read_safetensors

    path = os.path.join(folder, "model.safetensors")
    tensors = dict(read_safetensors(path))
    for k in list(tensors):
        if k.endswith(tuple(names)):
            tensors[k] = (tensors[k].float() * factor).to(tensors[k].dtype)
    write_safetensors(path, tensors, metadata={"format": "pt"})


@pytest.mark.parametrize("dtype", DTYPES)
def test_far_keys_in_several_partitions(tmp_path, dtype):
    """1,300 tokens through attention on the matrix cores and attention row by row, both with queries
    and keys made large so that every query's weight lies on a few keys anywhere in the past (a
    thousand tokens back too); portions that end inside pages and tiles, then single tokens."""
    cfg = config(211, 96, [pair((4, 2, 32, 32, 0.35, 0.4, 64), (2, 24, 16, 8.0), 1.0, 0.3, mlp=dense(80)),
                           pair((2, 1, 24, 40, 0.3, 0.6, 100), (3, 16, 32, 2.0), 0.9, 0.4, mlp=moe(6, 2, 40, 2, 1, 2.0))],
                 groups=2)
    folder = write_model(str(tmp_path / "m"), cfg, seed=13, dtype=dtype)
    sharpen(folder, 3.0)
    toks = random_tokens(1300, 211, seed=6)
    t = Trace({"x": toks})
    for n in (511, 3, 258, 490):
        t.step([("x", n)], want="last")
    for _ in range(38):
        t.step([("x", 1)])
    check_folder(t, run_folder(folder, dtype, t, block_size=16), folder, dtype, "far keys")


def test_attention_depends_on_a_token_far_back(tmp_path):
    """The first token is changed and the last logits of 900 tokens change with it, in the engine as
    in the plain model: a model whose only path from far back is attention (no shift, a linear
    attention that forgets at once and counts for nothing)."""
    dtype = "float32"
    cfg = config(97, 64, [pair((2, 1, 16, 16, 0.5, 0.5, 7), (1, 16, 16, 1.0), 1.0, 1.0)])
    folder = write_model(str(tmp_path / "m"), cfg, seed=3, dtype=dtype)
    from lyapunov_engine_amd.weights.safetensors_io import write_safetensors
    from plain.tonilix_plain import read_safetensors

    path = os.path.join(folder, "model.safetensors")
    tensors = dict(read_safetensors(path))
    tensors["l0.shift"] = torch.zeros_like(tensors["l0.shift"])
    tensors["l0.mix.right.a2.b"] = torch.full_like(tensors["l0.mix.right.a2.b"], -40.0)   # decays of nearly 0
    tensors["l0.mix.right.a2"] = torch.zeros_like(tensors["l0.mix.right.a2"])
    tensors["l0.mix.left.q"] = tensors["l0.mix.left.q"] * 0.2    # flat weights: every key counts, the first too
    tensors["l0.mix.left.q.b"] = tensors["l0.mix.left.q.b"] * 0.2
    write_safetensors(path, tensors, metadata={"format": "pt"})
    toks = random_tokens(900, 97, seed=2)
    other = [(toks[0] + 5) % 97] + toks[1:]
    outs = []
    for seq in (toks, other):
        t = Trace({"x": seq})
        t.step([("x", 880)], want="last")
        for _ in range(20):
            t.step([("x", 1)])
        got = run_folder(folder, dtype, t, block_size=16)
        check_folder(t, got, folder, dtype, "a token far back")
        outs.append(got[max(got)][0])
    want = plain_logits(folder, {"a": toks, "b": other})
    moved = float((want["a"][-1] - want["b"][-1]).abs().max())
    assert moved > 1e-4, "the test's model must carry the first token to the end"
    assert abs(float(np.abs(outs[0] - outs[1]).max()) - moved) < 0.05 * moved + 5e-5


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_multiplier_steps_inside_portions_and_between_single_tokens(tmp_path, dtype):
    """A multiplier that steps every 13 positions with a large factor: a portion that ends on the last
    position before a step, one that starts on the step, single tokens over the next step."""
    cfg = config(131, 48, [pair((2, 2, 16, 16, 0.4, 2.5, 13), (2, 8, 8, 3.0), 1.0, 0.5, mlp=dense(64)),
                           pair((3, 1, 8, 12, 0.5, 1.5, 13), (1, 16, 24, 6.0), 0.7, 1.2)], groups=2)
    folder = write_model(str(tmp_path / "m"), cfg, seed=17, dtype=dtype)
    toks = random_tokens(60, 131, seed=9)
    t = Trace({"x": toks})
    t.step([("x", 12)])          # positions 0..11: (p + 1) // 13 is 0 throughout
    t.step([("x", 2)])           # 12 is the first with 1
    t.step([("x", 10)])          # ..23
    for _ in range(6):           # 24, 25 (the step to 2), ...
        t.step([("x", 1)])
    t.step([("x", 30)], end=["x"])
    check_folder(t, run_folder(folder, dtype, t, block_size=8), folder, dtype, "multiplier")


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_given_shape_of_things_is_not_assumed(tmp_path, dtype):
    """Sizes that are equal, or 1, in one model and not in another: a single layer of each kind with
    one head, keys larger than values and the other way round, one expert, no feed-forward, two
    taps, groups of one expert of which one group is kept."""
    for n, layers in enumerate([[delta(1, 1, 8, 24, 2, mlp=moe(1, 1, 56, 1, 1, 0.9))],
                                [pair((1, 1, 24, 8, 1.1, 0.9, 3), (1, 24, 8, 2.0), 0.5, 2.0)],
                                [delta(3, 3, 20, 4, 5, mlp=moe(5, 1, 16, 5, 1, 1.0)), delta(6, 2, 4, 20, 2, mlp=dense(16))]]):
        cfg = config(97, 40, layers, eps=1e-4, groups=(1, 5, 2)[n])
        folder = write_model(str(tmp_path / f"m{n}"), cfg, seed=5 + n, dtype=dtype, ranks=(3, 9, 2))
        toks = random_tokens(45, 97, seed=3)
        t = Trace({"x": toks})
        t.step([("x", 20)])
        t.step([("x", 2)])
        for _ in range(23):
            t.step([("x", 1)])
        check_folder(t, run_folder(folder, dtype, t, block_size=8), folder, dtype, f"one of everything {n}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("layers", ["many experts", "keys of 256", "heads of 128 and of 80", "rows of no whole 16 bytes",
                                    "recurrences only", "attention first"])
def test_other_orders_and_sizes(tmp_path, dtype, layers):
    if layers == "many experts":
        cfg = config(111, 64, [delta(2, 1, 16, 16, 4, mlp=moe(72, 5, 8, 9, 4, 3.0)),
                               pair((2, 1, 16, 16, 0.5, 0.2, 4), (2, 16, 16, 4.0), mlp=moe(64, 8, 8, 8, 2, 1.0))], groups=2)
    elif layers == "keys of 256":
        cfg = config(111, 64, [delta(1, 1, 256, 8, 2, mlp=dense(32)), pair((1, 1, 16, 16, 0.5, 0.2, 4), (1, 200, 8, 4.0)),
                               delta(2, 1, 72, 24, 3)])
    elif layers == "heads of 128 and of 80":
        cfg = config(111, 128, [pair((2, 1, 128, 128, 0.2, 0.3, 10), (2, 32, 64, 4.0), mlp=dense(64)),
                                pair((2, 2, 80, 80, 0.25, 0.3, 10), (1, 64, 128, 8.0), 0.5, 0.5, mlp=moe(4, 2, 64, 2, 2, 2.0))],
                     groups=8)
    elif layers == "rows of no whole 16 bytes":
        cfg = config(111, 100, [delta(5, 5, 6, 7, 3, mlp=moe(3, 2, 36, 1, 1, 2.0)),
                                pair((5, 5, 12, 20, 0.5, 0.3, 9), (5, 7, 9, 3.0), 0.9, 1.1, mlp=dense(52))], groups=5)
    elif layers == "recurrences only":
        cfg = config(111, 64, [delta(4, 2, 16, 32, 4, mlp=dense(96)), delta(2, 2, 32, 16, 2, mlp=moe(4, 2, 24, 2, 1, 2.0))])
    else:
        cfg = config(111, 64, [pair((4, 4, 16, 16, 0.5, 1.0, 2), (4, 8, 16, 2.0), 1.0, 1.0, mlp=moe(4, 2, 24, 4, 2, 2.0)),
                               delta(2, 1, 32, 32, 4, mlp=dense(40)),
                               pair((2, 1, 32, 32, 0.3, 0.1, 50), (2, 16, 16, 16.0), 0.5, 1.5)], groups=4)
    folder = write_model(str(tmp_path / "m"), cfg, seed=9, dtype=dtype)
    reqs = {"x": random_tokens(80, 111, seed=1), "y": random_tokens(21, 111, seed=2)}
    t = Trace(reqs)
    t.step([("x", 30)])
    t.step([("x", 3), ("y", 19)])
    for _ in range(2):
        t.step([("x", 1), ("y", 1)])
    t.step([("x", 45)], end=["x", "y"])
    check_folder(t, run_folder(folder, dtype, t, block_size=16 if "heads of" in layers else 8), folder, dtype, layers)


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
        if dtype == "float32":
            want, margins = plain_greedy(folder, prompt, 12)
            close = [i for i, m in enumerate(margins) if m < 1e-3]
            upto = close[0] if close else 12
            assert o.output_tokens[:upto] == want[:upto]
            continue
        # 16-bit: every token is the largest logit of the same tokens replayed step by step (a router's
        # close call may send the plain model down another path, so it is no yardstick here)
        toks = prompt + o.output_tokens
        t = Trace({"g": toks})
        t.step([("g", len(prompt))], want="last")
        for _ in range(11):
            t.step([("g", 1)])
        got = replay(folder, dtype, t, block_size=BLOCK_SIZE[name])
        for i in range(12):
            row = got[i][0]
            best = np.sort(row)[-2:]
            assert int(row.argmax()) == o.output_tokens[i] or best[1] - best[0] < 0.3, f"token {i}"


def test_generation_with_and_without_recorded_steps_and_with_preemption(folders):
    import lyapunov_engine_amd as L

    folder = folders["B"]["float32"]
    prompts = [random_tokens(n, CONFIGS["B"]["vocab"], seed=80 + n) for n in (5, 30, 61, 12)]
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
