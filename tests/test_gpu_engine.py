"""The engine in-process on the GPU: the step function under many cuts, generation through
the entry point, the scheduler under page pressure."""

import numpy as np
import pytest
import torch

import plain_lfm2 as plain
from gpu_common import Loaded, feed
from helpers import assert_close, make_model, random_tokens

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("models")
    return {name: make_model(str(root / name), name, seed=21) for name in ("A", "B")}


@pytest.fixture(scope="module")
def loaded(folders):
    cache = {}

    def get(name, dtype):
        if (name, dtype) not in cache:
            cache[(name, dtype)] = Loaded(folders[name], dtype)
        return cache[(name, dtype)]
    return get


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B"])
def test_first_tokens_and_lengths_across_every_boundary(loaded, name, dtype):
    # prompt lengths of the reference's path-parity test (tests/test_v2_path_parity.py:129), whole and cut
    m = loaded(name, dtype)
    stepper = m.stepper(num_pages=6, max_requests=2)
    for length in (1, 2, 3, 9, 40, 300):
        tokens = random_tokens(m.config.vocab_size, length, seed=length)
        want = m.expected(tokens)
        for cuts in ([length], [1] * min(length, 5), [2, 1, 3, 64, 63, 1, 65]):
            stepper.admit("r")
            assert_close(feed(stepper, "r", tokens, cuts), want, dtype, f"length {length} cuts {cuts[:4]}")
            stepper.release("r")
    stepper.cache.check_invariants()


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding(loaded, dtype):
    m = loaded("B", dtype)
    tokens = random_tokens(m.config.vocab_size, 330, seed=8)
    stepper = m.stepper(num_pages=6, max_requests=1)
    stepper.admit("r")
    assert_close(feed(stepper, "r", tokens, [30] + [1] * 300), m.expected(tokens), dtype, "300 decoded tokens")


@pytest.mark.parametrize("dtype", DTYPES)
def test_cuts_agree_with_each_other(loaded, dtype):
    """Whole, token by token and in portions differ by rounding only. In float32 every kernel
    sums in an order fixed by the row alone, so that is far below the distance to the float64
    model. In bfloat16 a decode step and a prompt portion run different kernels that round
    their activations at different points (the fused decode product rounds x * w before the
    row's scale, the norm kernel after it), so two cuts are two independent bfloat16
    evaluations and differ as much as either does from the float64 model."""
    from helpers import MAX_TOL
    m = loaded("A", dtype)
    tokens = random_tokens(m.config.vocab_size, 150, seed=4)
    stepper = m.stepper(num_pages=3, max_requests=1)
    runs = []
    for cuts in ([150], [1] * 150, [7, 2, 16, 3, 2, 64, 5]):
        stepper.admit("r")
        runs.append(feed(stepper, "r", tokens, cuts))
        stepper.release("r")
    scale = np.abs(runs[0]).max()
    limit = {"float32": 2e-6, "bfloat16": MAX_TOL["bfloat16"]}[dtype] * scale
    assert np.abs(runs[1] - runs[0]).max() <= limit and np.abs(runs[2] - runs[0]).max() <= limit


@pytest.mark.parametrize("dtype", DTYPES)
def test_pages_and_slots_that_are_used_again_carry_nothing_over(loaded, dtype):
    """After a request ends its pages and state slot are filled with NaN; the next request
    gets exactly those (the pools are LIFO) and must not be touched by what they hold."""
    m = loaded("B", dtype)
    stepper = m.stepper(num_pages=4, max_requests=1)
    first = random_tokens(m.config.vocab_size, 200, seed=1)
    stepper.admit("a")
    feed(stepper, "a", first, [200])
    held = list(stepper.cache.groups[0].tables["a"])
    stepper.release("a")
    for pages in list(stepper.cache.k_pages.values()) + list(stepper.cache.v_pages.values()):
        pages.fill_(float("nan"))
    for state in stepper.cache.state.values():
        state.fill_(float("nan"))
    second = random_tokens(m.config.vocab_size, 130, seed=2)
    stepper.admit("b")
    got = feed(stepper, "b", second, [70, 3, 1, 1, 55])
    assert set(stepper.cache.groups[0].tables["b"]) <= set(held)
    assert_close(got, m.expected(second), dtype, "second request on poisoned pages")


@pytest.mark.parametrize("dtype", ["float32"])
def test_a_far_key_among_hundreds_decides_the_output(loaded, dtype, tmp_path):
    """The query of the last token is made to match the key of token 3 (of 400) far better
    than any other, by scaling the q- and k-norm weights of the attention layers: if a step
    dropped or misplaced one key, the logits would move by far more than the tolerance. The
    plain model sees the same weights, so this is an ordinary comparison with a sharp
    attention pattern. In 32-bit only: so sharp a softmax magnifies bfloat16's rounding of
    the scores just as it magnifies a fault (the bfloat16 kernels are given single dominant
    keys in their own tests instead)."""
    import os
    from flyweight_amd.weights import SafetensorsFile, write_file
    m = loaded("A", dtype)
    with SafetensorsFile(os.path.join(m.folder, "model.safetensors")) as handle:
        tensors = {n: handle.tensor(n) for n in handle.names()}
    for n in tensors:
        if n.endswith("k_layernorm.weight") or n.endswith("q_layernorm.weight"):
            tensors[n] = tensors[n] * 3.0       # scores nine times larger: softmax picks single keys
    folder = str(tmp_path / "sharp")
    os.makedirs(folder)
    write_file(os.path.join(folder, "model.safetensors"), tensors)
    m.config.save(folder)
    sharp = Loaded(folder, dtype)
    tokens = random_tokens(sharp.config.vocab_size, 380, seed=9)
    want = sharp.expected(tokens)
    stepper = sharp.stepper(num_pages=6, max_requests=1)
    stepper.admit("r")
    assert_close(feed(stepper, "r", tokens, [100, 1, 1, 150, 2, 126]), want, dtype, "sharp attention")


def _runtime(m, **kw):
    from flyweight_amd.engine import Model, Runtime
    model = Model.__new__(Model)
    model.path, model.dtype, model.config, model.model = m.folder, m.model.dtype, m.config, m.model
    return Runtime(model, **kw).prepare()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_through_the_entry_point(folders, name, dtype):
    import flyweight_amd
    model = flyweight_amd.Model(folders[name], dtype=dtype)
    config, weights = plain.read_folder(folders[name])
    with flyweight_amd.Runtime(model, parallel_sequences=2, prefill_rows=16, max_batch_tokens=24) as runtime:
        for length in (5, 17, 31):
            prompt = random_tokens(config["vocab_size"], length, seed=length)
            seen = []
            produced = runtime.generate(prompt, 8, callback=seen.append)
            assert produced == seen
            if dtype == "float32":
                assert produced == plain.greedy(config, weights, prompt, 8)
            else:   # bfloat16 may legitimately pick another of two near-equal logits; check each choice instead
                context = list(prompt)
                for token in produced:
                    logits = plain.forward(config, weights, context)[-1]
                    assert logits[token] >= logits.max() - 2e-2 * np.abs(logits).max()
                    context.append(token)
        # decode(token) -> token, the reference's single-sequence call
        runtime.reset()
        prompt = random_tokens(config["vocab_size"], 6, seed=1)
        token = None
        for t in prompt:
            token = runtime.decode(t)
        if dtype == "float32":
            assert token == plain.greedy(config, weights, prompt, 1)[0]
        assert runtime.info["decode_calls"] >= 6


def test_engine_tasks_equal_blocking_generation_and_survive_preemption(loaded):
    m = loaded("B", "float32")
    config, weights = m.plain_config, m.plain_weights
    prompts = [random_tokens(m.config.vocab_size, n, seed=n) for n in (1, 9, 64, 100)]
    expected = [plain.greedy(config, weights, p, 16) for p in prompts]
    # a roomy engine, portions of 16 beside decode rows
    runtime = _runtime(m, parallel_sequences=4, prefill_rows=16, max_batch_tokens=32)
    ids = [runtime.task_submit(p, 16) for p in prompts]
    events = []
    while runtime.scheduler.has_work():
        events += runtime.engine_step()
    for task, want in zip(ids, expected):
        assert [e[1] for e in events if e[0] == task and e[2] == 0] == want
        assert [e[2] for e in events if e[0] == task][-1] == 1
    # so few pages that the newest request must give way while decoding and be recomputed: same tokens
    tight = _runtime(m, parallel_sequences=4, prefill_rows=32, max_batch_tokens=64, num_pages=3)
    pressed = [(prompts[2], 40), (random_tokens(m.config.vocab_size, 60, seed=77), 80)]    # 104 and 140 tokens: 2 + 3 pages
    ids = [tight.task_submit(p, n) for p, n in pressed]
    result = tight.run()
    assert tight.info["preemptions"] >= 1
    for task, (prompt, n) in zip(ids, pressed):
        assert result[task] == plain.greedy(config, weights, prompt, n)
    assert tight.info["pages_free"] == 3 and tight.info["live_requests"] == 0
    tight.stepper.cache.check_invariants()


@pytest.mark.parametrize("dtype", DTYPES)
def test_decode_steps_that_run_ahead_of_the_host_give_the_same_tokens(loaded, dtype):
    """With several decode steps per turn the device feeds each step's tokens to the next and
    the host reads them in bursts: the same tokens in the same order as one step per turn (float32:
    the plain model's), bursts that go on past the requests that end in them (their last token, a stop token),
    across page edges, and also while somebody waits for a slot that none of them has given up yet."""
    m = loaded("B", dtype)
    config, weights = m.plain_config, m.plain_weights
    prompts = [random_tokens(m.config.vocab_size, n, seed=40 + n) for n in (3, 60, 9, 30)]
    budgets = [70, 9, 23, 41]

    def run(steps_per_turn, stop_tokens=(), parallel=4):
        runtime = _runtime(m, parallel_sequences=parallel, prefill_rows=64, max_batch_tokens=128,
                           decode_steps_per_turn=steps_per_turn)
        ids = [runtime.task_submit(p, n, stop_tokens=stop_tokens if i == 0 else ()) for i, (p, n) in enumerate(zip(prompts, budgets))]
        events, bursts = [], []
        while runtime.scheduler.has_work():
            got = runtime.engine_step()
            bursts.append(max([sum(1 for e in got if e[0] == task and e[2] == 0) for task in ids] + [0]))
            events += got
        runtime.stepper.cache.check_invariants()
        assert runtime.info["pages_free"] == runtime.num_pages and runtime.info["live_requests"] == 0
        return [[e[1] for e in events if e[0] == task and e[2] == 0] for task in ids], max(bursts), events

    single, burst, _ = run(1)
    assert burst == 1
    ahead, burst, events = run(4)
    assert ahead == single and burst == 4
    assert [len(tokens) for tokens in ahead] == budgets
    for task_events in ([e for e in events if e[0] == task] for task in {e[0] for e in events}):
        assert task_events[-1][2] == 1 and all(e[2] != 1 for e in task_events[:-1]), "finished is a request's last event"
    if dtype == "float32":
        assert ahead == [plain.greedy(config, weights, p, n) for p, n in zip(prompts, budgets)]
    # a request that may stop on a token runs ahead like the others; when it draws that token, wherever
    # in a turn, it ends there, what its row drew after it is dropped, and the others go on in order
    for place in (17, 18, 19, 20):
        stop = single[0][place]
        stopped, burst, events = run(4, stop_tokens=(stop,))
        cut = single[0].index(stop) + 1
        assert stopped[0] == single[0][:cut] and stopped[1:] == single[1:] and burst == 4
        for task_events in ([e for e in events if e[0] == task] for task in {e[0] for e in events}):
            assert task_events[-1][2] == 1 and all(e[2] != 1 for e in task_events[:-1])
    # two slots for four requests: the two that run do so in bursts while the others wait for their slots
    queued, burst, _ = run(4, parallel=2)
    assert burst == 4 and [len(tokens) for tokens in queued] == budgets
    if dtype == "float32":          # (in bfloat16 a prompt that runs beside other rows may round to another of two near-equal tokens)
        assert queued == single


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_turn_reserves_pages_only_up_to_each_requests_last_token(loaded, dtype):
    """Two pages for two requests. One of them ends with the turn's first step, two tokens short
    of its page's end; its row runs on beside the other for three more steps. Pages for those
    steps would be a second page for it, which the pool does not have: the turn reserves up to its
    last token only, names the spare page behind the one it holds, and runs ahead all the same.
    The other request's tokens are what it draws one step per turn."""
    m = loaded("B", dtype)
    prompts = [random_tokens(m.config.vocab_size, n, seed=70 + n) for n in (62, 10)]
    budgets = [2, 30]

    def run(steps_per_turn):
        runtime = _runtime(m, parallel_sequences=2, num_pages=2, prefill_rows=64, max_batch_tokens=128,
                           decode_steps_per_turn=steps_per_turn)
        ids = [runtime.task_submit(p, n) for p, n in zip(prompts, budgets)]
        events, bursts = [], []
        while runtime.scheduler.has_work():
            got = runtime.engine_step()
            bursts.append(sum(1 for e in got if e[0] == ids[1] and e[2] == 0))
            events += got
        runtime.stepper.cache.check_invariants()
        assert runtime.info["pages_free"] == 2 and runtime.info["live_requests"] == 0 and runtime.scheduler.preemptions == 0
        return [[e[1] for e in events if e[0] == task and e[2] == 0] for task in ids], bursts

    single, bursts = run(1)
    assert max(bursts) == 1 and [len(tokens) for tokens in single] == budgets
    ahead, bursts = run(4)
    assert ahead == single
    assert bursts[:2] == [1, 4], "the first decode turn ran four steps although one request ended in its first"
    if dtype == "float32":
        assert ahead == [plain.greedy(m.plain_config, m.plain_weights, p, n) for p, n in zip(prompts, budgets)]


@pytest.mark.parametrize("dtype", DTYPES)
def test_decode_steps_are_filled_up_to_the_sizes_that_are_kept(loaded, dtype):
    """Eleven requests that end one by one: the engine's decode steps run at the kept sizes (16,
    then 8, then every size below), the rows behind the plan's filled up with a token of nobody's
    in the cache's spare page and slot. Every request gets the tokens it gets alone."""
    from flyweight_amd.engine.step import Stepper
    assert [Stepper.kept_batch(n) for n in (1, 7, 8, 9, 16, 17, 64, 65, 81, 128)] == [1, 7, 8, 16, 16, 24, 64, 80, 96, 128]
    m = loaded("A", dtype)
    config, weights = m.plain_config, m.plain_weights
    prompts = [random_tokens(m.config.vocab_size, 2 + 5 * i, seed=70 + i) for i in range(11)]
    budgets = [6 + 3 * i for i in range(11)]
    for steps_per_turn in (1, 4):
        runtime = _runtime(m, parallel_sequences=11, prefill_rows=64, max_batch_tokens=128, decode_steps_per_turn=steps_per_turn)
        ids = [runtime.task_submit(p, n) for p, n in zip(prompts, budgets)]
        tokens = runtime.run()
        sizes = {batch for batch, _ in runtime.stepper._graphs}
        # (a turn of four steps goes on past the requests that end in it, so it need not meet every size)
        assert 16 in sizes and (8 in sizes or steps_per_turn > 1) and not sizes & {9, 10, 11, 12, 13, 14, 15}, sizes
        runtime.stepper.cache.check_invariants()
        assert runtime.info["pages_free"] == runtime.num_pages and runtime.info["live_requests"] == 0
        # the same requests with every decode step at its exact size: rows are independent in every
        # kernel, so a row that only fills a step up changes nothing of the others, in bfloat16 with
        # its fused kernels as in float32
        exact = _runtime(m, parallel_sequences=11, prefill_rows=64, max_batch_tokens=128, decode_steps_per_turn=steps_per_turn)
        exact.stepper.kept_batch = lambda rows: rows
        exact_ids = [exact.task_submit(p, n) for p, n in zip(prompts, budgets)]
        exact_tokens = exact.run()
        assert {batch for batch, _ in exact.stepper._graphs} >= {9, 10, 11}
        for task, exact_task, prompt, budget in zip(ids, exact_ids, prompts, budgets):
            assert len(tokens[task]) == budget
            assert tokens[task] == exact_tokens[exact_task]
            if dtype == "float32":
                assert tokens[task] == plain.greedy(config, weights, prompt, budget)


def test_generate_stops_at_the_token_its_callback_refuses_even_inside_a_burst(loaded):
    """With several decode steps per turn a turn brings several tokens of a request: the callback
    that returns False ends the generation at its token; the tokens of the same turn behind it are
    dropped, the request's pages and slot are given back."""
    m = loaded("A", "float32")
    prompt = random_tokens(m.config.vocab_size, 11, seed=5)
    whole = _runtime(m, parallel_sequences=2, prefill_rows=64, max_batch_tokens=128).generate(prompt, 24)
    assert len(whole) == 24
    for stop_after in (1, 6, 7, 10):
        runtime = _runtime(m, parallel_sequences=2, prefill_rows=64, max_batch_tokens=128, decode_steps_per_turn=4)
        seen = []

        def callback(token):
            seen.append(token)
            return len(seen) < stop_after

        got = runtime.generate(prompt, 24, callback)
        assert got == whole[:stop_after] and seen == got
        while runtime.scheduler.has_work():
            runtime.engine_step()
        runtime.stepper.cache.check_invariants()
        assert runtime.info["pages_free"] == runtime.num_pages and runtime.info["live_requests"] == 0


def test_seeded_sampling_does_not_depend_on_the_batch(loaded):
    """Temperature 0.8, seed 7, portions of 16 mixed with decode rows: a request draws the
    same tokens alone and among others, and they are the plain sampler's tokens given the
    plain model's logits."""
    m = loaded("B", "float32")
    prompts = [random_tokens(m.config.vocab_size, n, seed=n + 3) for n in (1, 9, 64, 200)]
    settings = dict(temperature=0.8, top_k=40, top_p=0.95, min_p=0.05, seed=7)
    together = _runtime(m, parallel_sequences=4, prefill_rows=16, max_batch_tokens=40)
    ids = [together.task_submit(p, 16, **settings) for p in prompts]
    batch = together.run()
    for task, prompt in zip(ids, prompts):
        alone = _runtime(m, parallel_sequences=1, prefill_rows=512)
        assert alone.generate(prompt, 16, **settings) == batch[task]
    rng = plain.XorShift64Star(7)
    context, want = list(prompts[1]), []
    for _ in range(16):
        logits = plain.forward(m.plain_config, m.plain_weights, context)[-1]
        want.append(plain.sample(logits.astype(np.float32), 0.8, 40, 0.95, 0.05, rng))
        context.append(want[-1])
    assert batch[ids[1]] == want
    # top_k = 0: the whole vocabulary; also the plain sampler's tokens
    full = _runtime(m, parallel_sequences=1)
    a = full.generate(prompts[1], 6, temperature=1.0, top_k=0, top_p=1.0, min_p=0.0, seed=3)
    b = full.generate(prompts[1], 6, temperature=1.0, top_k=0, top_p=1.0, min_p=0.0, seed=3)
    rng = plain.XorShift64Star(3)
    context, want = list(prompts[1]), []
    for _ in range(6):
        logits = plain.forward(m.plain_config, m.plain_weights, context)[-1]
        want.append(plain.sample(logits.astype(np.float32), 1.0, 0, 1.0, 0.0, rng))
        context.append(want[-1])
    assert a == b == want


@pytest.mark.parametrize("dtype", DTYPES)
def test_drawn_tokens_come_from_recorded_steps_and_turns_like_the_most_likely_ones(loaded, dtype):
    """Requests that draw their tokens (each with its own settings and seed, one of them greedy) run
    through the recorded decode steps with the sampler behind them, one step or four per turn: the
    same tokens either way, the same as each request alone, and in float32 the plain sampler's
    given the plain model's logits. The generators end where the host's copies say."""
    m = loaded("B", dtype)
    prompts = [random_tokens(m.config.vocab_size, n, seed=70 + n) for n in (5, 33, 12, 64)]
    settings = [dict(temperature=0.8, top_k=40, top_p=0.95, min_p=0.05, seed=11), dict(temperature=1.3, top_k=0, top_p=0.7, min_p=0.0, seed=12),
                dict(temperature=0.0), dict(temperature=0.5, top_k=3, top_p=1.0, min_p=0.3, seed=14)]
    budgets = [21, 30, 17, 26]

    def run(steps_per_turn):
        runtime = _runtime(m, parallel_sequences=4, prefill_rows=64, max_batch_tokens=128, decode_steps_per_turn=steps_per_turn)
        ids = [runtime.task_submit(p, n, **kw) for p, n, kw in zip(prompts, budgets, settings)]
        states = {}
        bursts = []
        while runtime.scheduler.has_work():
            for task in ids:
                request = runtime.scheduler.requests.get(task)
                if request is not None:
                    states[task] = request.rng.state
            got = runtime.engine_step()
            bursts.append(max([sum(1 for e in got if e[0] == task and e[2] == 0) for task in ids] + [0]))
            for task, token, kind in got:
                if kind == 0:
                    states.setdefault(("tokens", task), []).append(token)
        return [states[("tokens", task)] for task in ids], max(bursts), runtime.stepper.graph_replays

    single, burst, replays = run(1)
    assert burst == 1 and replays > 20, "the drawing requests ran through recorded steps"
    ahead, burst, _ = run(4)
    assert ahead == single and burst == 4
    assert [len(tokens) for tokens in single] == budgets
    for prompt, budget, kw, tokens in zip(prompts, budgets, settings, single):
        alone = _runtime(m, parallel_sequences=1, prefill_rows=64)
        if dtype == "float32":          # (in bfloat16 a prompt beside other rows may round to another of two near-equal logits)
            assert alone.generate(prompt, budget, **kw) == tokens
        if dtype == "float32" and kw.get("temperature", 0) > 0:
            rng = plain.XorShift64Star(kw["seed"])
            context, want = list(prompt), []
            for _ in range(budget):
                logits = plain.forward(m.plain_config, m.plain_weights, context)[-1]
                want.append(plain.sample(logits.astype(np.float32), kw["temperature"], kw["top_k"], kw["top_p"], kw["min_p"], rng))
                context.append(want[-1])
            assert tokens == want


def test_draws_over_a_whole_vocabulary_beyond_a_batch_of_candidates(tmp_path):
    """A vocabulary of 3,001 drawn from without top_k (and with one above 1,024): the sampler's path for
    long lists, through recorded decode steps, one step or four per turn; the plain sampler's tokens
    given the plain model's logits, in float32."""
    from flyweight_amd.config import config_from_dict
    from flyweight_amd.weights import write_random_model
    from gpu_common import Loaded
    from helpers import TINY_A
    folder = write_random_model(str(tmp_path / "wide"), config_from_dict(dict(TINY_A, vocab_size=3001)), 5, scale="fan_in")
    m = Loaded(folder, "float32")
    prompts = [random_tokens(3001, n, seed=90 + n) for n in (7, 20, 3)]
    settings = [dict(temperature=1.0, top_k=0, top_p=1.0, min_p=0.0, seed=21), dict(temperature=0.9, top_k=0, top_p=0.8, min_p=0.0005, seed=22),
                dict(temperature=1.4, top_k=2000, top_p=0.95, min_p=0.0, seed=23)]
    results = []
    for steps_per_turn in (1, 4):
        runtime = _runtime(m, parallel_sequences=4, prefill_rows=64, max_batch_tokens=128, decode_steps_per_turn=steps_per_turn)
        ids = [runtime.task_submit(p, 14, **kw) for p, kw in zip(prompts, settings)]
        finished = runtime.run()
        results.append([finished[task] for task in ids])
        assert runtime.stepper.graph_replays > 8
    assert results[0] == results[1]
    for prompt, kw, tokens in zip(prompts, settings, results[0]):
        rng = plain.XorShift64Star(kw["seed"])
        context, want = list(prompt), []
        for _ in range(14):
            logits = plain.forward(m.plain_config, m.plain_weights, context)[-1]
            want.append(plain.sample(logits.astype(np.float32), kw["temperature"], kw["top_k"], kw["top_p"], kw["min_p"], rng))
            context.append(want[-1])
        assert tokens == want


def test_errors_are_reported_not_hidden(loaded):
    from flyweight_amd.engine import EngineError, StepEntry, StepError
    from flyweight_amd.cache import OutOfPages
    m = loaded("A", "float32")
    runtime = _runtime(m, parallel_sequences=2, num_pages=2)
    with pytest.raises(EngineError, match="exceeds the context"):
        runtime.task_submit([1] * 300, 200)
    with pytest.raises(EngineError, match="empty"):
        runtime.task_submit([], 2)
    task = runtime.task_submit([1] * 100, 100)       # needs 4 pages, the pool has 2
    events = runtime.engine_step()
    assert (task, 0, 2) in events and "pages" in runtime.task_error(task)
    stepper = m.stepper(num_pages=1, max_requests=2)
    stepper.admit("a")
    with pytest.raises(StepError, match="outside the vocabulary"):
        stepper.step([StepEntry("a", [m.config.vocab_size], [0])])
    with pytest.raises(StepError, match="not admitted"):
        stepper.step([StepEntry("zz", [1], [0])])
    with pytest.raises(StepError, match="twice"):
        stepper.step([StepEntry("a", [1], [0]), StepEntry("a", [2], [0])])
    with pytest.raises(OutOfPages):
        stepper.step([StepEntry("a", [1] * 65, [])])
    assert stepper.cache.length_of("a") == 0 and stepper.cache.groups[0].pool.in_use == 0   # nothing half-done
    assert stepper.step([StepEntry("a", [1] * 64, [63])]).shape == (1, m.config.vocab_size)


def _run_to_the_end(runtime):
    events = []
    while runtime.scheduler.has_work():
        events += runtime.engine_step()
    return events


@pytest.mark.parametrize("bad_place", [3, 21])
def test_a_request_the_step_refuses_ends_alone_and_the_others_go_on(loaded, bad_place):
    """Three tasks, the middle one with a token id outside the vocabulary in its first portion or
    in its second (the scheduler here does not know the vocabulary, so only the step finds it):
    it ends with an error event and its text, the other two generate the plain model's tokens,
    and every page and slot is back."""
    from flyweight_amd.engine import EVENT_ERROR, EVENT_FINISHED, EVENT_TOKEN, EngineError, Scheduler
    m = loaded("A", "float32")
    config, weights = m.plain_config, m.plain_weights
    vocab = m.config.vocab_size
    good = [random_tokens(vocab, 30, seed=5), random_tokens(vocab, 19, seed=6)]
    bad = random_tokens(vocab, 40, seed=7)
    bad[bad_place] = vocab
    runtime = _runtime(m, parallel_sequences=4, prefill_rows=16, max_batch_tokens=40, num_pages=6)
    with pytest.raises(EngineError, match=f"token id {vocab} at place {bad_place} of the prompt is outside the vocabulary"):
        runtime.task_submit(bad, 5)
    with pytest.raises(EngineError, match="stop token"):
        runtime.task_submit(good[0], 5, stop_tokens=[vocab + 7])
    assert not runtime.scheduler.has_work()
    runtime.scheduler = Scheduler(runtime.stepper.cache, max_positions=runtime.context_limit, max_batch_tokens=40,
                                  chunk_size=16, max_live=4)      # no vocabulary: nothing is checked at submit
    first = runtime.task_submit(good[0], 8)
    middle = runtime.task_submit(bad, 8)
    last = runtime.task_submit(good[1], 8)
    events = _run_to_the_end(runtime)
    assert [e[2] for e in events if e[0] == middle and e[2] != 3] == [EVENT_ERROR]
    assert any(e[0] == middle and e[2] == 3 for e in events) == (bad_place >= 16)      # its first portion ran
    assert "outside the vocabulary" in runtime.task_error(middle) and runtime.task_error(first) is None
    for task, prompt in ((first, good[0]), (last, good[1])):
        assert [e[1] for e in events if e[0] == task and e[2] == EVENT_TOKEN] == plain.greedy(config, weights, prompt, 8)
        assert [e[2] for e in events if e[0] == task][-1] == EVENT_FINISHED
    assert runtime.info["pages_free"] == 6 and runtime.info["slots_free"] == 4 and runtime.info["live_requests"] == 0
    runtime.stepper.cache.check_invariants()
    assert not runtime.scheduler.requests, "finished tasks are forgotten once their last event is handed out"


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_step_that_fails_while_it_runs_ends_its_requests_only(loaded, dtype, monkeypatch):
    """A kernel refuses in the middle of a step (forced here from the host: the third forward pass
    raises before it launches anything): the requests of that step end with an error, their pages
    and slots come back, and the request that was still waiting runs to the plain model's tokens."""
    from flyweight_amd.engine import EVENT_ERROR, EVENT_TOKEN
    from flyweight_amd.kernels.ops import KernelError
    m = loaded("B", dtype)
    vocab = m.config.vocab_size
    prompts = [random_tokens(vocab, n, seed=40 + n) for n in (20, 33, 25)]
    runtime = _runtime(m, parallel_sequences=2, prefill_rows=16, max_batch_tokens=32, num_pages=5)
    tasks = [runtime.task_submit(p, 6) for p in prompts]      # two slots: the third waits
    calls = {"n": 0}
    forward = m.model.forward

    def failing(ctx, cache):
        calls["n"] += 1
        if calls["n"] == 3:
            raise KernelError("forced: a kernel refused its operands")
        return forward(ctx, cache)
    monkeypatch.setattr(m.model, "forward", failing)
    events = _run_to_the_end(runtime)
    monkeypatch.undo()
    for task in tasks[:2]:
        assert [e[2] for e in events if e[0] == task][-1] == EVENT_ERROR
        assert "KernelError" in runtime.task_error(task) and "forced" in runtime.task_error(task)
    got = [e[1] for e in events if e[0] == tasks[2] and e[2] == EVENT_TOKEN]
    if dtype == "float32":
        assert got == plain.greedy(m.plain_config, m.plain_weights, prompts[2], 6)
    assert len(got) == 6 and runtime.info["failed_steps"] == 1
    assert runtime.info["pages_free"] == 5 and runtime.info["slots_free"] == 2
    runtime.stepper.cache.check_invariants()
    # the runtime is as good as new: the same prompts again, nothing forced
    again = [runtime.task_submit(p, 6) for p in prompts]
    result = runtime.run()
    if dtype == "float32":
        for task, prompt in zip(again, prompts):
            assert result[task] == plain.greedy(m.plain_config, m.plain_weights, prompt, 6)
    assert sorted(result) == sorted(again)


def test_generate_beside_other_tasks_keeps_their_events(loaded):
    from flyweight_amd.engine import EVENT_FINISHED, EVENT_TOKEN
    m = loaded("A", "float32")
    vocab = m.config.vocab_size
    other_prompt, own_prompt = random_tokens(vocab, 12, seed=1), random_tokens(vocab, 7, seed=2)
    runtime = _runtime(m, parallel_sequences=2)
    other = runtime.task_submit(other_prompt, 9)
    own = runtime.generate(own_prompt, 4)
    assert own == plain.greedy(m.plain_config, m.plain_weights, own_prompt, 4)
    events = _run_to_the_end(runtime) + runtime.engine_step()
    assert [e[1] for e in events if e[0] == other and e[2] == EVENT_TOKEN] == plain.greedy(m.plain_config, m.plain_weights, other_prompt, 9)
    assert [e[2] for e in events if e[0] == other][-1] == EVENT_FINISHED
    assert not runtime.scheduler.requests


@pytest.mark.parametrize("dtype", DTYPES)
def test_captured_decode_steps_replay_to_the_eager_result(loaded, dtype):
    """Decode steps are recorded in a HIP graph per batch size and replayed. Every replay,
    with eager prompt portions and synchronisations between them and with the batch changing
    size, must give what the eager step gives."""
    from flyweight_amd.engine import StepEntry
    m = loaded("B", dtype)
    vocab = m.config.vocab_size
    runs = []
    for use_graphs in (False, True):
        stepper = m.stepper(num_pages=12, max_requests=4)
        assert stepper.use_graphs
        stepper.use_graphs = use_graphs
        rng = np.random.default_rng(5)
        out = []
        for request in ("a", "b", "c"):
            stepper.admit(request)
        stepper.step([StepEntry("a", rng.integers(0, vocab, 70).tolist(), []), StepEntry("b", rng.integers(0, vocab, 3).tolist(), [])])
        for step in range(40):
            entries = [StepEntry("a", [int(rng.integers(0, vocab))], [0]), StepEntry("b", [int(rng.integers(0, vocab))], [0])]
            if step % 7 == 3:       # an eager step between replays: a prompt portion of a third request
                out.append(stepper.step([StepEntry("c", rng.integers(0, vocab, 5).tolist(), [4])]).cpu().numpy())
            if step >= 20:          # the batch grows: another graph
                entries.append(StepEntry("c", [int(rng.integers(0, vocab))], [] if step % 2 else [0]))
            logits = stepper.step(entries)
            out.append(logits.cpu().numpy())
        runs.append(out)
        if use_graphs:
            assert stepper.graph_replays >= 30 and {batch for batch, _ in stepper._graphs} == {2, 3}
    for eager, replayed in zip(*runs):
        assert eager.shape == replayed.shape and np.array_equal(eager, replayed)


@pytest.mark.parametrize("dtype", DTYPES)
def test_captured_decode_steps_are_sized_by_the_run_not_by_the_model(folders, tmp_path, dtype):
    """The same weights under ``max_position_embeddings`` 128,000 and 512: the captured decode
    steps are sized by the contexts that are live (block-table rows and split-key grid of the
    next power of two of their pages), so the large limit costs nothing, and a sequence that
    grows past a bucket moves to the next recorded step; the logits are the same bit for bit."""
    import json
    import shutil
    from flyweight_amd.engine import StepEntry, Stepper, load_model
    wide = str(tmp_path / "wide")
    shutil.copytree(folders["B"], wide)
    with open(f"{wide}/config.json") as handle:
        raw = json.load(handle)
    raw["max_position_embeddings"] = 128000
    with open(f"{wide}/config.json", "w") as handle:
        json.dump(raw, handle)
    vocab = raw["vocab_size"]
    runs, keys = [], []
    for folder, limit in ((folders["B"], None), (wide, None), (wide, 4096)):
        _, model = load_model(folder, dtype=dtype)
        stepper = Stepper(model, num_pages=16, max_requests=3, context_limit=limit)
        rng = np.random.default_rng(11)
        for request in ("a", "b"):
            stepper.admit(request)
        stepper.step([StepEntry("a", rng.integers(0, vocab, 250).tolist(), []), StepEntry("b", rng.integers(0, vocab, 40).tolist(), [])])
        out = []
        for step in range(12):      # "a" goes from 250 to 262 tokens: past the first bucket of 256
            out.append(stepper.step([StepEntry("a", [int(rng.integers(0, vocab))], [0]),
                                     StepEntry("b", [int(rng.integers(0, vocab))], [0, 0])]).cpu().numpy())
        assert out[0].shape == (3, vocab)       # a place named twice gives two rows, recorded step or not
        runs.append(out)
        keys.append(sorted(stepper._graphs))
        assert stepper.cache.max_pages_per_request == {None: raw["max_position_embeddings"] if folder == wide else 512, 4096: 4096}[limit] // 64
    assert keys[0] == keys[1] == keys[2] == [(2, 4), (2, 8)]
    for other in runs[1:]:
        for small, large in zip(runs[0], other):
            assert np.array_equal(small, large)
    with pytest.raises(Exception, match="context limit is 4096"):
        stepper.step([StepEntry("a", [1] * 4000, [])])


@pytest.mark.parametrize("dtype", DTYPES)
def test_equal_logits_give_the_lowest_id_through_the_engine(folders, tmp_path, dtype):
    """With a tied head a copy of an embedding row has that row's logit bit for bit, in either
    precision: the engine must generate the lower of the two ids, as the plain model does."""
    import shutil
    from safetensors.torch import load_file, save_file
    import flyweight_amd
    config, weights = plain.read_folder(folders["A"])
    prompt = random_tokens(config["vocab_size"], 9, seed=2)
    with flyweight_amd.Runtime(flyweight_amd.Model(folders["A"], dtype=dtype)) as runtime:
        winner = runtime.generate(prompt, 1)[0]
    free = [t for t in range(config["vocab_size"]) if t not in prompt and t != winner]
    for copy, expected in ((max(free), winner), (min(free), min(free))):
        folder = str(tmp_path / f"copy{copy}")
        shutil.copytree(folders["A"], folder)
        tensors = load_file(f"{folder}/model.safetensors")
        tensors["model.embed_tokens.weight"][copy] = tensors["model.embed_tokens.weight"][winner]
        save_file(tensors, f"{folder}/model.safetensors")
        with flyweight_amd.Runtime(flyweight_amd.Model(folder, dtype=dtype)) as runtime:
            assert runtime.generate(prompt, 1) == [expected]
        if dtype == "float32":
            changed_config, changed = plain.read_folder(folder)
            assert plain.greedy(changed_config, changed, prompt, 1) == [expected]


@pytest.mark.parametrize("name,seed", [("A", 0), ("A", 1), ("A", 2), ("B", 3)])
def test_a_random_load_under_every_setting_gives_each_request_what_it_gets_alone(loaded, name, seed):
    """Forty requests (greedy ones, drawing ones, some with stop tokens, a few cancelled on the way)
    arrive while others run, on few slots and so few pages that requests give way, in turns of one
    and of four decode steps: every request that runs to its end gets the tokens it gets alone with
    pages to spare, each has one last event, and the cache is whole after every step and empty at the
    end. (float32, whose logits differ between ways of cutting and batching in the last bits only: a
    request that takes the most likely token is never moved by that; one that draws is, once in
    thousands of draws, when a candidate sits on the edge of a cut, so one of the forty may differ.)"""
    m = loaded(name, "float32")
    rng = np.random.default_rng(100 + seed)
    vocab = m.config.vocab_size
    count = 40
    prompts = [random_tokens(vocab, int(rng.integers(1, 90)), seed=500 + 50 * seed + i) for i in range(count)]
    budgets = [int(rng.integers(1, 40)) for _ in range(count)]
    settings = []
    for i in range(count):
        kind = int(rng.integers(0, 4))
        drawn = {} if kind == 0 else dict(temperature=float(rng.choice([0.7, 1.0, 1.5])), top_k=int(rng.choice([0, 1, 5, 40])),
                                          top_p=float(rng.choice([1.0, 0.9, 0.5])), min_p=float(rng.choice([0.0, 0.1])), seed=1000 + i)
        settings.append(drawn)
    alone = _runtime(m, parallel_sequences=1, prefill_rows=64)
    wanted = [alone.generate(p, n, **kw) for p, n, kw in zip(prompts, budgets, settings)]
    # a stop token for every third request: a token it will draw, where it draws one more than once
    stops = [(wanted[i][len(wanted[i]) // 2],) if i % 3 == 0 and len(wanted[i]) > 2 else () for i in range(count)]
    for i, stop in enumerate(stops):
        if stop:
            wanted[i] = wanted[i][:wanted[i].index(stop[0]) + 1]
    cancel_at = {int(i): int(rng.integers(1, 6)) for i in rng.choice(count, 4, replace=False)}
    gave_way = 0
    for steps_per_turn in (1, 4):
        runtime = _runtime(m, parallel_sequences=5, num_pages=6, prefill_rows=32, max_batch_tokens=48, decode_steps_per_turn=steps_per_turn)
        todo = list(range(count))
        ids, got, last, seen_tokens = {}, {}, {}, {}
        engine_steps = 0
        while todo or runtime.scheduler.has_work():
            for _ in range(int(rng.integers(0, 3))):
                if todo:
                    i = todo.pop(0)
                    ids[runtime.task_submit(prompts[i], budgets[i], stop_tokens=stops[i], **settings[i])] = i
            for task, i in ids.items():
                if i in cancel_at and seen_tokens.get(i, 0) >= cancel_at[i] and task not in last:
                    runtime.task_cancel(task)
            for task, value, kind in runtime.engine_step():
                i = ids[task]
                assert task not in last, "an event behind a request's last one"
                if kind == 0:
                    got.setdefault(i, []).append(value)
                    seen_tokens[i] = seen_tokens.get(i, 0) + 1
                elif kind in (1, 2):
                    last[task] = kind
            runtime.stepper.cache.check_invariants()
            engine_steps += 1
            assert engine_steps < 5000, "the load does not come to an end"
        assert len(last) == count and all(kind == 1 for kind in last.values())
        assert runtime.info["pages_free"] == runtime.num_pages and runtime.info["live_requests"] == 0
        gave_way += runtime.info["preemptions"]
        moved = []
        for i in range(count):
            mine = got.get(i, [])
            same = mine == wanted[i][:len(mine)] and (len(mine) >= min(cancel_at[i], len(wanted[i])) if i in cancel_at else len(mine) == len(wanted[i]))
            if not same:
                assert settings[i], (i, "a request that takes the most likely token", mine, wanted[i])
                assert len(mine) >= 1, "a request that ran got no token"
                moved.append(i)
        assert len(moved) <= 1, (moved, [settings[i] for i in moved])
    assert gave_way > 0, "the pages were meant to run out"
