"""Dalerax on the CPU: its configuration and tensor names, the cache entries it asks for (pages of kept first keys
stay, a cache entry read through two masks keeps what either sees), and the plain model held against itself (a
sequence in one piece against token by token with carried state, the mask's edges, the sink, the router)."""

import copy

import numpy as np
import pytest

import plain_dalerax as plain
from dalerax_common import CONFIG_X, CONFIG_Y, CONFIG_Z, make_folder, random_tokens


def test_config_lowers_to_parts_and_names(tmp_path):
    from flyweight_amd.config import ConfigError, DaleraxConfig, load_config
    from flyweight_amd.engine.model import declared_tensors
    for name, raw in (("X", CONFIG_X), ("Y", CONFIG_Y), ("Z", CONFIG_Z)):
        folder = str(tmp_path / name)
        make_folder(folder, raw, decay_rank=5 + len(name))
        config = load_config(folder)                         # the model class by config.json, the decay maps' width by the checkpoint
        assert isinstance(config, DaleraxConfig)
        spec = config.model_spec()
        declared = declared_tensors(spec)
        assert {n: tuple(d.shape) for n, d in declared.items()} == plain.tensor_shapes(raw, decay_rank=5 + len(name))
        assert [layer.mixer.kind for layer in config.layers] == [entry["type"] for entry in raw["layers"]]
        assert spec.lm_head_name == "head" and spec.position_table_name == "pos" and spec.max_positions == raw["max_positions"]
        assert all(layer.arrangement == "parallel_residual" and layer.ffn_norm is None for layer in spec.layers)
        again = DaleraxConfig.from_dict(config.to_dict())
        assert again == config
    spec = DaleraxConfig.from_dict(CONFIG_X).model_spec()
    assert spec.embedding_scale == 3.0 and spec.logit_scale == 0.7
    second, third, last = spec.layers[1], spec.layers[2], spec.layers[4]
    assert second.mixer.kind == "gqa_attention" and second.mixer["window"] == 40 and second.mixer["keep_first"] == 3 and second.mixer["sink"]
    assert second.mixer["position"]["wavelength_scaling"] == (4.0, 1.0, 4.0, 64.0) and not second.mixer["shared_kv"]
    assert third.mixer["shared_kv"] and third.ffn is None and last.mixer["window"] is None and last.mixer["position"].get("wavelength_scaling") is None
    assert second.ffn.kind == "moe_swiglu" and second.ffn["num_experts"] == 7 and second.ffn["top"] == 3 and second.ffn["shared_intermediate_size"] == 56
    assert spec.layers[3].ffn["shared_intermediate_size"] is None and spec.layers[0].ffn.kind == "swiglu" and spec.layers[0].mixer.kind == "wkv"
    # a layer that reads another's keys and values names that layer's cache entry and does not write it
    assert [(entry.layer, entry.cache, entry.writes_cache) for entry in spec.schedule] == [(0, 0, True), (1, 1, True), (2, 1, False), (3, 3, True), (4, 4, True)]
    for path, value, match in ((("layers", 0, "type"), "serial", "type"), (("layers", 1, "mixer", "heads"), 3, "multiple"),
                               (("layers", 1, "mixer", "rot", "dims"), 34, "dims"), (("norm", "eps"), 0, "eps"),
                               (("layers", 0, "mlp", "kind"), "sparse", "kind"), (("layers", 1, "mlp", "router", "top"), 8, "chooses"),
                               (("layers", 2, "mixer", "kv_from"), 0, "kv_from"), (("layers", 2, "mixer", "kv_from"), 4, "kv_from"),
                               (("layers", 2, "mixer", "dim"), 48, "kv_from"), (("layers", 1, "mixer", "rot", "scaling", "high"), 0.5, "high"),
                               (("max_positions",), None, "max_positions"), (("layers", 3, "mixer", "dim"), 0, "dim")):
        broken = copy.deepcopy(CONFIG_X)
        at = broken
        for key in path[:-1]:
            at = at[key]
        at[path[-1]] = value
        with pytest.raises(ConfigError, match=match):
            DaleraxConfig.from_dict(broken)
    chained = copy.deepcopy(CONFIG_X)
    chained["layers"][4]["mixer"] = dict(chained["layers"][2]["mixer"], kv_from=2)      # the layer it names has none of its own
    with pytest.raises(ConfigError, match="kv_from"):
        DaleraxConfig.from_dict(chained)


def test_cache_entries():
    """A recurrence asks for its matrix state and its last input in the request's slot; attention layers for paged keys
    and values; an entry that two layers read through different masks keeps what either of them sees."""
    from flyweight_amd.cache import CacheManager
    from flyweight_amd.config import DaleraxConfig
    from flyweight_amd.engine.model import CausalLM
    model = CausalLM(DaleraxConfig.from_dict(CONFIG_X).model_spec())
    needs = model.cache_needs()
    assert set(needs) == {0, 1, 3, 4}
    assert set(needs[0]) == {"state", "shift"} and needs[0]["state"].shape == (4, 24, 24) and needs[0]["shift"].shape == (96,)
    assert (needs[1].window, needs[1].keep_first, needs[1].v_head_dim) == (70, 5, 48)       # the wider window, the more kept keys
    assert needs[4].window is None and needs[4].keep_first == 0
    needs_y = CausalLM(DaleraxConfig.from_dict(CONFIG_Y).model_spec()).cache_needs()
    assert (needs_y[0].window, needs_y[0].keep_first) == (64, 1) and (needs_y[2].window, needs_y[2].keep_first) == (33, 70)
    cache = CacheManager(needs_y, num_pages=6, max_requests=2)
    windowed = {group.need.window: index for index, group in enumerate(cache.groups)}
    cache.admit("a")
    for length in (50, 130, 131, 200, 330):
        cache.reserve("a", length)
        cache.commit("a", length)
        cache.check_invariants()
    # window 33 with 70 kept keys: the two pages of the kept keys stay, then only the window's; window 64 with one kept
    # key: its first page stays
    held = lambda window: [page != -1 for page in cache.groups[windowed[window]].tables["a"]]
    assert held(33) == [True, True, False, False, True, True]
    assert held(64) == [True, False, False, False, True, True]
    cache.admit("b")
    cache.reserve("b", 128)         # the pages that "a" gave back serve "b"
    cache.commit("b", 128)
    cache.check_invariants()
    cache.release("a")
    cache.release("b")
    assert all(group.pool.free_count == 6 for group in cache.groups) and cache.slots.free_count == 2
    # two masks over one entry: no window on one side keeps every key
    from flyweight_amd.cache.needs import PagedKV
    assert PagedKV(2, 32, 40, 48, None, 3).shared_with(PagedKV(2, 32, None, 48)).window is None
    assert PagedKV(2, 32, 40, 48, None, 3).shared_with(PagedKV(2, 32, 20, 48, None, 9)) == PagedKV(2, 32, 40, 48, None, 9)
    with pytest.raises(ValueError):
        PagedKV(2, 32, 40).shared_with(PagedKV(2, 64, 40))


def test_plain_recurrence_in_one_piece_and_token_by_token():
    rng = np.random.default_rng(0)
    m = {"heads": 3, "dim": 8}
    shapes = {name[len("l0.mix."):]: shape for name, shape in plain.tensor_shapes(
        {"width": 20, "vocab": 5, "max_positions": 4, "layers": [{"type": "wkv", "mixer": m, "mlp": None}]}, 4).items() if name.startswith("l0.mix.")}
    w = {name: rng.normal(0.0, 0.5, shape) for name, shape in shapes.items()}
    h = rng.normal(size=(30, 20))
    whole, (S, last) = plain.wkv_mixer(h, w, m, 1e-5)
    state, rows = None, []
    for t in range(30):
        row, state = plain.wkv_step(h[t], w, m, 1e-5, state)
        rows.append(row)
    assert np.allclose(np.stack(rows), whole, atol=1e-12) and np.allclose(state[0], S, atol=1e-12) and np.array_equal(state[1], last)
    # in two runs of tokens with the state handed on
    first, state = plain.wkv_mixer(h[:13], w, m, 1e-5)
    second, _ = plain.wkv_mixer(h[13:], w, m, 1e-5, state)
    assert np.allclose(np.concatenate([first, second]), whole, atol=1e-12)
    # the bonus counts for the current token only: with an empty state the read-out is (r . (u k)) v
    r, k, v, decay, u = (rng.normal(size=8) for _ in range(5))
    o, S1 = plain.wkv_read_write(np.zeros((8, 8)), r, k, v, np.exp(-np.exp(decay)), u)
    assert np.allclose(o, (r * u * k).sum() * v) and np.allclose(S1, np.outer(k, v))
    o2, _ = plain.wkv_read_write(S1, r, k, v, np.exp(-np.exp(decay)), np.zeros(8))
    assert np.allclose(o2, (r * k).sum() * v)


def test_plain_mask_sink_and_rotation():
    # which keys a row sees: itself and the size - 1 before it, and the first keep_first wherever it stands
    assert [j for j in range(12) if plain.may_see(9, j, 4, 2)] == [0, 1, 6, 7, 8, 9]
    assert [j for j in range(12) if plain.may_see(3, j, 4, 2)] == [0, 1, 2, 3]
    assert [j for j in range(12) if plain.may_see(9, j, None, 0)] == list(range(10))
    assert [j for j in range(12) if plain.may_see(5, j, 1, 0)] == [5]
    rng = np.random.default_rng(1)
    q, k, v = rng.normal(size=(6, 2, 4)), rng.normal(size=(6, 1, 4)), rng.normal(size=(6, 1, 3))
    without = plain.sink_heads(q, k, v, 0.5, None, 0, None)
    low = plain.sink_heads(q, k, v, 0.5, None, 0, np.array([-60.0, -60.0]))
    high = plain.sink_heads(q, k, v, 0.5, None, 0, np.array([60.0, -60.0]))
    assert np.allclose(low, without) and np.abs(high[:, 0]).max() < 1e-20 and np.allclose(high[:, 1], without[:, 1])
    # the first row sees itself alone: its weight is 1 / (1 + exp(sink - score))
    sink = np.array([0.3, -0.2])
    first = plain.sink_heads(q, k, v, 0.5, 3, 1, sink)[0]
    for head in range(2):
        score = 0.5 * q[0, head] @ k[0, 0]
        assert np.allclose(first[head], v[0, 0] / (1.0 + np.exp(sink[head] - score)))
    # the three ranges of the frequencies' stretching
    f = 10000.0 ** (-2.0 * np.arange(16) / 32)
    g = plain.rotary_frequencies(32, 10000.0, {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 100})
    wavelength = 2 * np.pi / f
    assert np.array_equal(g[wavelength < 25], f[wavelength < 25]) and np.allclose(g[wavelength > 100], f[wavelength > 100] / 8.0)
    between = (wavelength >= 25) & (wavelength <= 100)
    assert between.any() and (g[between] < f[between]).all() and (g[between] > f[between] / 8.0).all()
    x = rng.normal(size=(5, 2, 8))
    turned = plain.rotate_halves(x, np.arange(5), 4, np.array([0.5, 0.1]))
    assert np.array_equal(turned[..., 4:], x[..., 4:]) and np.array_equal(turned[0], x[0])
    assert np.allclose(turned[3, 1, 0], x[3, 1, 0] * np.cos(1.5) - x[3, 1, 2] * np.sin(1.5))
    assert np.allclose(turned[3, 1, 3], x[3, 1, 3] * np.cos(0.3) + x[3, 1, 1] * np.sin(0.3))


def test_plain_router():
    h = np.array([[1.0, 0.0], [0.0, 1.0], [0.0, 0.0]])
    router = np.array([[1.0, 0.0], [2.0, 0.0], [0.0, 3.0], [2.0, 3.0]])
    chosen, weight = plain.route(h, router, np.array([0.0, 0.0, 0.5, 0.0]), 2)
    assert chosen.tolist() == [[1, 3], [2, 3], [2, 0]]          # equal logits: the lower id first
    assert np.allclose(weight.sum(-1), 1.0) and np.allclose(weight[0], [0.5, 0.5]) and np.allclose(weight[1, 0], 1 / (1 + np.exp(-0.5)))


def test_plain_model_is_causal_and_every_part_counts():
    for raw in (CONFIG_X, CONFIG_Z):
        weights = plain.random_weights(raw, 3)
        tokens = random_tokens(raw["vocab"], 60, seed=5)
        full = plain.forward(raw, weights, tokens)
        assert np.allclose(plain.forward(raw, weights, tokens[:45]), full[:45], atol=1e-10)
        for name in weights:
            if name in ("embed", "pos", "head") or ".mlp.e" in name:       # rows that the tokens or the router may not reach
                continue
            changed = dict(weights)
            changed[name] = weights[name] + 0.05 * np.sign(weights[name] + 1e-9)
            assert np.abs(plain.forward(raw, changed, tokens) - full).max() > 1e-7, name
