"""Ronupel on the GPU: whole models through the engine's step function and cache
manager against the plain implementation: whole prompts, token-by-token
decoding, portions down to two tokens, mixed batches with pages used again,
random schedules, long decoding past every window, and greedy generation
through the entry point and the scheduler."""
import os
import random
import subprocess
import sys

import numpy as np
import pytest
import torch

from conftest import ROOT
from ronupel_util import (BLOCK_SIZE, CONFIGS, RouterLog, attn, config, moe, plain_greedy, plain_logits,
                          plain_logits_routed_alike, write_model)
from trace_util import Trace, compare, compare_with_alone, random_tokens, random_trace, replay

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]
DEV = "cuda:0"


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for name, cfg in CONFIGS.items():
        out[name] = {dt: write_model(str(tmp_path_factory.mktemp(f"ronupel{name}_{dt}")), cfg, seed=21 + ord(name), dtype=dt)
                     for dt in DTYPES}
    return out


LENGTHS = {"a": 1, "b": 7, "c": 33, "d": 70, "e": 130}


def requests_for(name, extra=None):
    lens = dict(LENGTHS, **(extra or {}))
    return {rid: random_tokens(n, CONFIGS[name]["vocab"], seed=400 + i) for i, (rid, n) in enumerate(sorted(lens.items()))}


def run_folder(folder, dtype, t, **kw):
    """Replay the trace; the engine's router choices go along with it (``t.routing``)."""
    with RouterLog() as log:
        got = replay(folder, dtype, t, **kw)
    t.routing = log.by_request(t)
    return got


def run(folders, name, dtype, t):
    return run_folder(folders[name][dtype], dtype, t, block_size=BLOCK_SIZE[name])


def check_folder(t, got, folder, dtype, label):
    """32-bit: against the plain model as it is.  16-bit: against the plain model with the engine's
    router choices (a close call decided the other way is no fault of a kernel; a clear one is,
    and is asserted), on the same rounded weights."""
    if dtype == "float32":
        compare(t, got, plain_logits(folder, t.requests), dtype, label)
    else:
        compare(t, got, plain_logits_routed_alike(folder, t.requests, t.routing), dtype, label, tol=TOL16)


# bfloat16 against the 64-bit plain model on the same rounded weights: these models are made with
# wide weights so that attention is peaked, gates reach their limits and routers decide clearly,
# which also makes rounding show; the bounds are per row, of the largest logit.
TOL16 = dict(rtol=0.0, atol=1.5e-1, median=4e-2)


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
    """The first tokens of a sequence one by one: a first page, windows that are not full yet, kept
    first tokens that are still inside the window."""
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
def test_mixed_batches_with_pages_used_again(folders, name, dtype):
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
    got = run(folders, name, dtype, t)
    check(t, got, folders, name, dtype, f"mixed {name}")
    if dtype == "float32":
        compare_with_alone(t, got, folders[name][dtype], dtype, f"mixed {name}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B"])
def test_random_schedules(folders, name, dtype):
    for seed in range(5):
        rng = random.Random(91 * seed + ord(name))
        reqs, t = random_trace(rng, CONFIGS[name]["vocab"], 150)
        got = run(folders, name, dtype, t)
        check(t, got, folders, name, dtype, f"random schedule {name} {seed}")
        if dtype == "float32":
            compare_with_alone(t, got, folders[name][dtype], dtype, f"random schedule {name} {seed}")


@pytest.mark.parametrize("name", ["B", "C"])
def test_long_decoding_past_every_window(folders, name):
    """400 tokens: most as portions that end inside pages, the last 150 one by one: every window has
    long passed the first tokens, whose pages the windowed layers gave back except the kept ones."""
    dtype = "float32"
    toks = random_tokens(400, CONFIGS[name]["vocab"], seed=1)
    t = Trace({"x": toks})
    t.step([("x", 131)], want="last")
    t.step([("x", 119)], want="last")
    for _ in range(150):
        t.step([("x", 1)])
    check(t, run(folders, name, dtype, t), folders, name, dtype, "long decoding")


@pytest.mark.parametrize("dtype", DTYPES)
def test_far_keys_and_windows_longer_than_a_partition(tmp_path, dtype):
    """1,300 tokens through a layer that sees everything (keys a thousand tokens back, in a prompt's
    portion and for single tokens, in several partitions) and one whose window of 300 spans
    partitions and keeps 33 first tokens; portions that end inside pages and tiles."""
    cfg = config(211, 96, [attn(4, 2, 32, 32, dims=16, base=5000.0, factor=2.0, scale=0.35, mlp=moe(6, 2, 40, 3.0, shared=(40, 3.0))),
                           attn(2, 1, 64, 64, window=300, keep=33, dims=64, scale=0.25, mlp=moe(3, 1, 24, 1.0))],
                 loop=(0, 2, 2))
    folder = write_model(str(tmp_path / "m"), cfg, seed=13, dtype=dtype)
    toks = random_tokens(1300, 211, seed=6)
    t = Trace({"x": toks})
    for n in (511, 3, 258, 490):
        t.step([("x", n)], want="last")
    for _ in range(38):
        t.step([("x", 1)])
    check_folder(t, run_folder(folder, dtype, t, block_size=16), folder, dtype, "far keys")


def test_windowed_layers_give_pages_back_and_keep_the_first(folders):
    """A model whose layers are all windowed runs a request far longer than its pool: pages behind
    the window return, those of the kept first tokens stay."""
    from lyapunov_engine_amd.engine.replay import TraceReplayer

    name, dtype = "B", "float32"
    toks = random_tokens(600, CONFIGS[name]["vocab"], seed=4)
    t = Trace({"x": toks})
    for n in (100, 100, 100, 100, 100, 99):
        t.step([("x", n)], want="last")
    t.step([("x", 1)])
    rp = TraceReplayer(folders[name][dtype], dtype, 384, block_size=16, max_model_len=1024)   # 24 pages a group for 600 tokens
    got = {s["step"]: rp.run(s) for s in t.steps}
    c = rp.core.cache.counters()
    assert c["window_returns"] > 0
    compare(t, got, plain_logits(folders[name][dtype], t.requests), dtype, "a request longer than the pool")


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_given_shape_of_things_is_not_assumed(tmp_path, dtype):
    """Sizes that are equal, or 1, in one model and not in another: one layer, one head, a loop over
    everything that runs once, one expert, a window of one token, more kept tokens than the window is
    long, rotated dimensions fewer than the head's, a value size larger than the key size."""
    cfg = config(97, 40, [attn(1, 1, 8, 24, window=1, keep=5, dims=4, base=9.0, factor=2.0, scale=1.1,
                               mlp=moe(1, 1, 56, 0.9))], loop=(0, 1, 1))
    folder = write_model(str(tmp_path / "m"), cfg, seed=5, dtype=dtype)
    toks = random_tokens(45, 97, seed=3)
    t = Trace({"x": toks})
    t.step([("x", 20)])
    t.step([("x", 2)])
    for _ in range(23):
        t.step([("x", 1)])
    check_folder(t, run_folder(folder, dtype, t, block_size=8), folder, dtype, "one of everything")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("layers", ["many experts", "no feed-forward at all", "looped four times from the start", "heads of 128",
                                    "rows of no whole 16 bytes", "heads of 80 and of 256"])
def test_other_orders_and_sizes(tmp_path, dtype, layers):
    if layers == "many experts":
        cfg = config(111, 64, [attn(2, 1, 16, 16, window=17, keep=2, dims=8, scale=0.5, mlp=moe(70, 5, 8, 3.0, shared=(24, 3.0)))])
    elif layers == "no feed-forward at all":
        cfg = config(111, 48, [attn(2, 2, 12, 12, window=6, keep=1, scale=0.6), attn(3, 1, 16, 16, window=44, keep=5, scale=0.5)])
    elif layers == "looped four times from the start":
        cfg = config(111, 64, [attn(4, 4, 16, 16, window=8, keep=8, dims=16, factor=8.0, scale=0.5, mlp=moe(4, 2, 24, 2.0)),
                               attn(2, 1, 32, 32, window=30, keep=0, dims=2, scale=0.3, mlp=moe(2, 1, 16, 2.0, shared=(8, 2.0)))],
                     loop=(0, 2, 4))
    elif layers == "rows of no whole 16 bytes":
        cfg = config(111, 100, [attn(5, 5, 12, 20, window=11, keep=3, dims=6, factor=2.0, scale=0.5, mlp=moe(3, 2, 36, 2.0, shared=(52, 1.0))),
                                attn(2, 1, 18, 18, window=25, keep=2, dims=18, scale=0.4, mlp=moe(5, 1, 44, 3.0))])
    elif layers == "heads of 80 and of 256":
        cfg = config(111, 64, [attn(2, 2, 80, 80, window=19, keep=2, dims=40, factor=4.0, scale=0.2, mlp=moe(3, 1, 32, 2.0)),
                               attn(1, 1, 256, 256, window=70, keep=1, dims=128, scale=0.1)])
    else:
        cfg = config(111, 128, [attn(2, 1, 128, 128, window=50, keep=4, dims=64, factor=2.0, scale=0.2, mlp=moe(4, 2, 64, 2.0))])
    folder = write_model(str(tmp_path / "m"), cfg, seed=9, dtype=dtype)
    reqs = {"x": random_tokens(80, 111, seed=1), "y": random_tokens(21, 111, seed=2)}
    t = Trace(reqs)
    t.step([("x", 30)])
    t.step([("x", 3), ("y", 19)])
    for _ in range(2):
        t.step([("x", 1), ("y", 1)])
    t.step([("x", 45)], end=["x", "y"])
    check_folder(t, run_folder(folder, dtype, t, block_size=8 if "heads of" not in layers else 16), folder, dtype, layers)


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
            want, _ = plain_greedy(folder, prompt, 12)
            assert o.output_tokens == want
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
