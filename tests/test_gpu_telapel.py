"""Telapel through the engine against the plain float64 model (tests/plain_telapel.py): whole prompts,
token-by-token decoding, portions down to two tokens, mixed batches on few pages and slots, each mixer
alone, long decoding, greedy generation through the scheduler, trace replay and the command line. In
32-bit and bfloat16."""

import json
import subprocess

import numpy as np
import pytest

import plain_telapel as plain
from telapel_common import (CONFIGS, assert_close, attention, latent, layer, make_folder, model, moe, only_mixer, random_tokens,
                            rglru)

pytestmark = pytest.mark.gpu

DTYPES = ("float32", "bfloat16")


class Loaded:
    def __init__(self, folder, config, dtype, seed=0):
        from flyweight_amd.engine import load_model
        self.config = config
        self.weights = make_folder(folder, config, seed=seed)
        self.folder, self.dtype = folder, dtype
        _, self.model = load_model(folder, dtype=dtype)
        self._expected = {}

    def stepper(self, num_pages, max_requests=4):
        from flyweight_amd.engine import Stepper
        return Stepper(self.model, num_pages=num_pages, max_requests=max_requests, context_limit=num_pages * 64)

    def expected(self, tokens):
        key = tuple(tokens)
        if key not in self._expected:
            self._expected[key] = plain.forward(self.config, self.weights, list(tokens))
        return self._expected[key]


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    root = tmp_path_factory.mktemp("telapel")
    made = {}

    def get(name, dtype, variant=""):
        key = (name, dtype, variant)
        if key not in made:
            config = CONFIGS[name] if not variant else only_mixer(CONFIGS[name], variant)
            made[key] = Loaded(str(root / f"{name}{variant}_{dtype}"), config, dtype, seed=len(name) + len(variant))
        return made[key]
    return get


def feed(stepper, request, tokens, cuts):
    """Feeds ``tokens`` in portions of the given sizes (cycled) and returns the logits at every position."""
    from flyweight_amd.engine import StepEntry
    out, at, i = [], 0, 0
    while at < len(tokens):
        n = min(cuts[i % len(cuts)], len(tokens) - at)
        out.append(stepper.step([StepEntry(request, list(tokens[at:at + n]), list(range(n)))]).cpu().numpy())
        at, i = at + n, i + 1
    return np.concatenate(out)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["X", "Y", "Z"])
def test_whole_prompt(models, name, dtype):
    loaded = models(name, dtype)
    tokens = random_tokens(loaded.config["vocab"], 200, seed=1)
    stepper = loaded.stepper(num_pages=8)
    stepper.admit("a")
    assert_close(feed(stepper, "a", tokens, [len(tokens)]), loaded.expected(tokens), dtype, f"{name} whole")
    # the first tokens of a sequence alone (a prompt of one, of two): convolutions that reach before the start,
    # a recurrence from nothing, a softmax of one key beside the term of 1
    for count in (1, 2):
        stepper.admit(("short", count))
        assert_close(feed(stepper, ("short", count), tokens[:count], [count]), loaded.expected(tokens[:count]), dtype, f"{name} first {count}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["X", "Y", "Z"])
def test_token_by_token_against_prefill(models, name, dtype):
    """Every token decoded alone, 170 steps: the windows (1, 33, 50, 64 keys) pass over decoded tokens and page
    borders, the query factor steps up, the recurrences and every convolution run on what the slot carries, recorded
    steps are replayed."""
    loaded = models(name, dtype)
    tokens = random_tokens(loaded.config["vocab"], 170, seed=2)
    stepper = loaded.stepper(num_pages=6)
    stepper.admit(0)
    assert_close(feed(stepper, 0, tokens, [1]), loaded.expected(tokens), dtype, f"{name} decoded")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["X", "Y", "Z"])
@pytest.mark.parametrize("cuts", [[2], [3, 2, 64, 5, 2, 33, 65, 9], [63, 1, 1, 64, 2], [7]])
def test_portions(models, name, dtype, cuts):
    loaded = models(name, dtype)
    tokens = random_tokens(loaded.config["vocab"], 150, seed=3)
    stepper = loaded.stepper(num_pages=6)
    stepper.admit("p")
    assert_close(feed(stepper, "p", tokens, cuts), loaded.expected(tokens), dtype, f"{name} portions {cuts}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding(models, dtype):
    """A short prompt and 330 tokens decoded one by one: five pages, ten windows of the shorter mask, pages of the
    windowed layers handed back, a recurrence whose slowest channels barely forget."""
    loaded = models("Y", dtype)
    tokens = random_tokens(loaded.config["vocab"], 340, seed=9)
    stepper = loaded.stepper(num_pages=6)
    stepper.admit("long")
    head = feed(stepper, "long", tokens[:10], [10])
    tail = feed(stepper, "long", tokens[10:], [1])
    assert_close(np.concatenate([head, tail]), loaded.expected(tokens), dtype, "Y long decoding")
    stepper.cache.check_invariants()


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_wider_model_through_the_prompt_kernels(models, dtype):
    """600 tokens of a model of width 512: whole (the tiled products, the matrix-core attention over a latent of
    128 + 64 channels and over keys that are the values, the grouped products of sixteen experts), cut at odd places,
    and its last 40 tokens decoded one by one beside a second request's portions."""
    from flyweight_amd.engine import StepEntry
    loaded = models("W", dtype)
    tokens = random_tokens(loaded.config["vocab"], 600, seed=7)
    other = random_tokens(loaded.config["vocab"], 300, seed=8)
    expected = loaded.expected(tokens)
    stepper = loaded.stepper(num_pages=26)
    stepper.admit("whole")
    assert_close(feed(stepper, "whole", tokens, [600]), expected, dtype, "W whole")
    stepper.release("whole")
    stepper.admit("cut")
    assert_close(feed(stepper, "cut", tokens, [257, 17, 200, 63, 63]), expected, dtype, "W cut")
    stepper.release("cut")
    stepper.admit("a")
    stepper.admit("b")
    head = feed(stepper, "a", tokens[:560], [560])
    rows, at = [], 0
    for i in range(560, 600):
        entries = [StepEntry("a", [tokens[i]], [0])]
        if at < len(other):
            entries.append(StepEntry("b", other[at:at + 9], []))
            at += 9
        rows.append(stepper.step(entries).cpu().numpy())
    assert_close(np.concatenate([head] + rows), expected, dtype, "W decoded beside another request")
    stepper.release("a")
    stepper.release("b")
    # and alone, so that decode steps are recorded and replayed
    stepper.admit("c")
    head = feed(stepper, "c", tokens[:580], [580])
    assert_close(np.concatenate([head, feed(stepper, "c", tokens[580:], [1])]), expected, dtype, "W decoded alone")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("variant", ["attention", "latent_attention", "rglru"])
@pytest.mark.parametrize("name", ["X", "Y", "Z"])
def test_each_mixer_alone(models, name, variant, dtype):
    loaded = models(name, dtype, variant)
    tokens = random_tokens(loaded.config["vocab"], 140, seed=4)
    stepper = loaded.stepper(num_pages=6)
    stepper.admit("w")
    assert_close(feed(stepper, "w", tokens, [len(tokens)]), loaded.expected(tokens), dtype, f"{name} {variant} whole")
    stepper.admit("c")
    assert_close(feed(stepper, "c", tokens, [5, 2, 70, 1, 1]), loaded.expected(tokens), dtype, f"{name} {variant} cut")


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_latent_wider_than_the_matrix_core_kernels_take(dtype, tmp_path):
    """A latent of 512 channels with a rotated part of 64: keys of 576 channels go to the plain attention kernel in
    both dtypes; whole, cut, and with a decoded tail."""
    config = model(150, 64, [layer(latent(2, 32, 64, 16, 24, 512, 0.1), None), layer(rglru(32, 2, 3), moe(4, 2, 2, 1, 16, 1.0))])
    loaded = Loaded(str(tmp_path / dtype), config, dtype, seed=3)
    tokens = random_tokens(config["vocab"], 100, seed=5)
    for cuts in ([100], [33, 2, 65], [80] + [1] * 20):
        stepper = loaded.stepper(num_pages=3, max_requests=2)
        stepper.admit("a")
        assert_close(feed(stepper, "a", tokens, cuts), loaded.expected(tokens), dtype, f"wide latent cut {cuts[:3]}")


def random_config(seed):
    """Two to six layers of any mixer in any order, every size drawn: heads and groups of 1..4, head sizes on and off
    the matrix cores' steps of 16, windows of 1 token to longer than the prompt or none, with and without a cap and a
    query factor, convolutions of 1 to 6 taps, latents with rotated parts of 2 to 64 channels, recurrences of 1 to 8
    blocks, experts in 1 to 4 groups with or without a shared unit or no feed-forward, layers that run an earlier
    layer's weights, widths of 40..320."""
    rng = np.random.default_rng(seed)
    pick = lambda *xs: xs[int(rng.integers(len(xs)))]
    layers = []
    for index in range(int(rng.integers(2, 7))):
        owners = [i for i, entry in enumerate(layers) if entry.get("weights_of") is None]
        if owners and rng.random() < 0.25:
            source = int(pick(*owners))
            layers.append(layer({"type": layers[source]["type"], "mixer": layers[source]["mixer"]}, layers[source]["mlp"], weights_of=source))
            continue
        kind = pick("attention", "latent_attention", "rglru")
        if kind == "attention":
            kv, dim = int(pick(1, 2, 3, 4)), int(pick(16, 20, 32, 48, 64, 96, 128))
            mixer = attention(kv * int(pick(1, 2, 3, 4)), kv, dim, int(pick(1, 2, 3, 4, 6)), pick(None, 1, 7, 50, 64, 100, 128, 1000),
                              pick(None, 5.0, 30.0), float(pick(dim ** -0.5, 0.1, 0.2)), temp=pick(None, (0.5, 16), (0.1, 1), (0.7, 100)))
        elif kind == "latent_attention":
            dim, rot = int(pick(8, 16, 24, 32, 64)), int(pick(2, 8, 16, 32, 64))
            mixer = latent(int(pick(1, 2, 3, 5, 8)), dim, rot, int(pick(8, 16, 40, 64)), int(pick(8, 24, 48)), int(pick(16, 32, 48, 100, 128)),
                           float(pick((dim + rot) ** -0.5, 0.2)), base=float(pick(100.0, 10000.0, 1e6)))
        else:
            blocks = int(pick(1, 2, 4, 8))
            mixer = rglru(blocks * int(pick(4, 16, 24, 40)), blocks, int(pick(1, 2, 4, 5)))
        mlp = pick(None, "moe", "moe", "moe")
        if mlp == "moe":
            groups = int(pick(1, 2, 4))
            per_group = int(pick(1, 2, 3, 8))
            keep = int(pick(*range(1, groups + 1)))
            top = int(pick(*[t for t in (1, 2, 4, 8) if t <= keep * per_group]))
            mlp = moe(groups * per_group, top, groups, keep, int(pick(12, 40, 64, 100)), float(pick(0.5, 1.5, 7.0)),
                      shared=pick(None, (24, 1.0), (64, 2.0)))
        layers.append(layer(mixer, mlp))
    return model(int(pick(97, 300, 512, 1000)), int(pick(40, 64, 96, 100, 128, 160, 192, 256, 320)), layers, eps=float(pick(1e-5, 1e-6)))


@pytest.mark.parametrize("seed", range(10))
def test_random_configurations(seed, tmp_path):
    """Whatever config.json gives is read from there: ten drawn models, whole, token by token, in odd portions and
    with a decoded tail, in both dtypes, against the plain model."""
    config = random_config(seed)
    tokens = random_tokens(config["vocab"], 150, seed=seed)
    for dtype in DTYPES:
        loaded = Loaded(str(tmp_path / dtype), config, dtype, seed=seed)
        for cuts in ([150], [1], [3, 2, 64, 5, 2, 33, 65, 9], [130] + [1] * 20):
            stepper = loaded.stepper(num_pages=4, max_requests=2)
            stepper.admit("a")
            assert_close(feed(stepper, "a", tokens, cuts), loaded.expected(tokens), dtype, f"drawn model {seed} cut {cuts[:3]}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["X", "Y", "Z"])
def test_mixed_batches_on_few_pages_and_slots(models, name, dtype):
    """Eight requests of unequal length through four slots and a pool that holds four of them at most: portions
    of some beside single tokens of others, requests left out of steps, pages and slots handed on. Every row must
    equal the request run alone."""
    from flyweight_amd.engine import StepEntry
    loaded = models(name, dtype)
    rng = np.random.default_rng(5)
    vocab = loaded.config["vocab"]
    prompts = {i: random_tokens(vocab, n, seed=10 + i) for i, n in enumerate([130, 1, 67, 200, 2, 64, 97, 33])}
    stepper = loaded.stepper(num_pages=9, max_requests=4)
    waiting, live, at = list(prompts), [], {}
    got = {i: [] for i in prompts}
    steps = 0
    while waiting or live:
        while waiting and len(live) < 4:
            need = (len(prompts[waiting[0]]) + 63) // 64
            held = sum((len(prompts[r]) + 63) // 64 for r in live)
            if held + need > 9:
                break
            request = waiting.pop(0)
            stepper.admit(request)
            live.append(request)
            at[request] = 0
        entries = []
        for request in live:
            if len(live) > 1 and rng.random() < 0.25:
                continue
            left = len(prompts[request]) - at[request]
            n = 1 if left <= 20 else int(min(left - 20, rng.choice([2, 3, 17, 64, 40])))
            entries.append(StepEntry(request, prompts[request][at[request]:at[request] + n], list(range(n))))
        if not entries:
            continue
        if rng.random() < 0.5:
            entries.sort(key=lambda e: len(e.tokens) != 1)      # the scheduler's order: single tokens first
        logits = stepper.step(entries).cpu().numpy()
        row = 0
        for entry in entries:
            n = len(entry.tokens)
            got[entry.request].append(logits[row:row + n])
            row += n
            at[entry.request] += n
            if at[entry.request] == len(prompts[entry.request]):
                stepper.release(entry.request)
                live.remove(entry.request)
        steps += 1
        stepper.cache.check_invariants()
    assert steps > 40
    for request, tokens in prompts.items():
        assert_close(np.concatenate(got[request]), loaded.expected(tokens), dtype, f"{name} mixed request {request}")


def test_a_batch_does_not_change_a_request(models):
    """float32: a request's logits beside three others, cut in portions, on pages and slots that others have used
    before, are bit for bit those of the request alone on a fresh cache."""
    from flyweight_amd.engine import StepEntry
    loaded = models("X", "float32")
    vocab = loaded.config["vocab"]
    mine = random_tokens(vocab, 120, seed=50)
    others = [random_tokens(vocab, n, seed=51 + n) for n in (90, 40, 75)]
    fresh = loaded.stepper(num_pages=4)
    fresh.admit("m")
    alone = feed(fresh, "m", mine, [120])
    stepper = loaded.stepper(num_pages=8)
    for i, tokens in enumerate(others):         # use pages and slots, then give them back
        stepper.admit(("old", i))
        feed(stepper, ("old", i), tokens, [len(tokens)])
    for i in range(len(others)):
        stepper.release(("old", i))
    for name in ("m", "o0", "o1", "o2"):
        stepper.admit(name)
    rows, at = [], 0
    for n in (50, 1, 1, 30, 38):
        entries = [StepEntry(f"o{i}", others[i][at:at + n], []) for i in range(3) if at + n <= len(others[i])]
        entries.insert(1 if entries else 0, StepEntry("m", mine[at:at + n], list(range(n))))
        rows.append(stepper.step(entries).cpu().numpy())
        at += n
    assert np.array_equal(np.concatenate(rows), alone)


@pytest.mark.parametrize("name", ["X", "Y"])
def test_greedy_generation_through_the_scheduler(models, name, tmp_path):
    """Several prompts at once through Runtime (admission, portions, decode steps, recorded steps): in float32 the
    tokens are the plain model's; in bfloat16 every chosen token is among the plain model's best."""
    import flyweight_amd
    from flyweight_amd.engine import EVENT_TOKEN
    loaded = models(name, "float32")
    vocab = loaded.config["vocab"]
    prompts = [random_tokens(vocab, n, seed=20 + n) for n in (37, 5, 90)]
    new = 12
    want = [plain.greedy(loaded.config, loaded.weights, prompt, new) for prompt in prompts]
    with flyweight_amd.Runtime(flyweight_amd.Model(loaded.folder, dtype="float32"), context_limit=256, parallel_sequences=3,
                               prefill_rows=16, max_batch_tokens=24) as runtime:
        tasks = [runtime.task_submit(prompt, new) for prompt in prompts]
        outputs = {task: [] for task in tasks}
        while runtime.scheduler.has_work():
            for task, value, kind in runtime.engine_step():
                if kind == EVENT_TOKEN:
                    outputs[task].append(value)
    for task, expected in zip(tasks, want):
        assert outputs[task] == expected
    with flyweight_amd.Runtime(flyweight_amd.Model(loaded.folder, dtype="bfloat16"), context_limit=256, parallel_sequences=2) as runtime:
        got = runtime.generate(prompts[0], new)
    context = list(prompts[0])
    for token in got:
        logits = plain.forward(loaded.config, loaded.weights, context)[-1]
        assert logits[token] >= logits.max() - 0.1 * np.abs(logits).max()
        context.append(token)


def test_serving_more_requests_than_slots_on_few_pages(models):
    """Seven requests through three slots and four pages a group, several decode steps per turn on the device:
    requests wait for a slot, slots and pages are handed on, recorded decode steps are replayed at changing batch
    sizes. The tokens are the plain model's (float32)."""
    import flyweight_amd
    loaded = models("Y", "float32")
    vocab = loaded.config["vocab"]
    prompts = [random_tokens(vocab, n, seed=60 + n) for n in (90, 3, 150, 64, 65, 1, 120)]
    new = [9, 14, 6, 11, 5, 16, 8]
    want = [plain.greedy(loaded.config, loaded.weights, p, n) for p, n in zip(prompts, new)]
    with flyweight_amd.Runtime(flyweight_amd.Model(loaded.folder, dtype="float32"), context_limit=192, parallel_sequences=3,
                               num_pages=4, prefill_rows=48, max_batch_tokens=56, decode_steps_per_turn=4) as runtime:
        tasks = [runtime.task_submit(p, n) for p, n in zip(prompts, new)]
        result = runtime.run()
        assert runtime.info["live_requests"] == 0
        runtime.stepper.cache.check_invariants()
    for task, expected in zip(tasks, want):
        assert result[task] == expected


def test_trace_replay(models, tmp_path):
    """bin/trace_run chooses the model class by config.json and replays a mixed trace on four slots."""
    from helpers import TRACE_RUN
    loaded = models("X", "float32")
    vocab = loaded.config["vocab"]
    a, b = random_tokens(vocab, 70, seed=31), random_tokens(vocab, 9, seed=32)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:40], "want": [0, 39]}], "end": []},
        {"step": 1, "entries": [{"id": "b", "tokens": b[:8], "want": []}, {"id": "a", "tokens": a[40:69], "want": [28]}], "end": []},
        {"step": 2, "entries": [{"id": "a", "tokens": a[69:], "want": [0]}, {"id": "b", "tokens": b[8:], "want": [0]}], "end": ["a", "b"]},
        {"step": 3, "entries": [{"id": "c", "tokens": b, "want": [8]}], "end": ["c"]},
    ]
    out = tmp_path / "out"
    process = subprocess.run([TRACE_RUN, "--model", loaded.folder, "--dtype", "float32", "--out", str(out), "--max-tokens", "192"],
                             input="".join(json.dumps(step) + "\n" for step in steps), capture_output=True, text=True, timeout=300)
    assert process.returncode == 0, process.stderr
    assert [line for line in process.stdout.splitlines() if line.startswith("done")] == [f"done {i}" for i in range(4)]
    full_a, full_b = loaded.expected(a), loaded.expected(b)
    read = lambda i: np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, vocab)
    assert_close(read(0), full_a[[0, 39]], "float32", "step 0")
    assert_close(read(1), full_a[[68]], "float32", "step 1")
    assert_close(read(2), np.stack([full_a[69], full_b[8]]), "float32", "step 2")
    assert_close(read(3), full_b[[8]], "float32", "step 3")


def test_command_line(models, capsys, tmp_path):
    """generate prints the plain model's greedy tokens; inspect names the architecture and its tensors;
    random-weights writes a folder from the configuration alone."""
    from flyweight_amd.cli import main
    from flyweight_amd.config import load_config
    loaded = models("Y", "float32")
    prompt = random_tokens(loaded.config["vocab"], 13, seed=40)
    expected = plain.greedy(loaded.config, loaded.weights, prompt, 5)
    assert main(["generate", loaded.folder, "--tokens", ",".join(map(str, prompt)), "--max-tokens", "5", "--temperature", "0",
                 "--dtype", "float32", "--ignore-eos", "--context", "128"]) == 0
    assert [int(t) for t in capsys.readouterr().out.split()] == expected
    assert main(["inspect", loaded.folder]) == 0
    shown = json.loads(capsys.readouterr().out)
    assert shown["architecture"] == "Telapel" and set(shown["tensors"]) == set(plain.tensor_shapes(loaded.config))
    (tmp_path / "config.json").write_text(json.dumps(load_config(loaded.folder).to_dict()))
    assert main(["random-weights", "--config", str(tmp_path / "config.json"), "--seed", "3", "--out", str(tmp_path / "drawn")]) == 0
    capsys.readouterr()
    assert main(["generate", str(tmp_path / "drawn"), "--tokens", "1,2,3", "--max-tokens", "4", "--temperature", "0",
                 "--ignore-eos", "--context", "128"]) == 0
    assert len(capsys.readouterr().out.split()) == 4
