"""Telapel on the CPU: its configuration and tensor names, the schedule of a layer that runs another's weights, the
cache entries it asks for, and the plain model held against itself (a sequence in one piece against pieces with
carried state, the window's edges, the term of 1 in the softmax, the bias by distance, the query factor, the router's
groups, the clamps)."""

import copy

import numpy as np
import pytest

import plain_telapel as plain
from telapel_common import CONFIG_X, CONFIG_Y, CONFIG_Z, make_folder, random_tokens


def test_config_lowers_to_parts_and_names(tmp_path):
    from flyweight_amd.config import ConfigError, TelapelConfig, load_config
    from flyweight_amd.engine.model import declared_tensors
    for name, raw in (("X", CONFIG_X), ("Y", CONFIG_Y), ("Z", CONFIG_Z)):
        folder = str(tmp_path / name)
        make_folder(folder, raw)
        config = load_config(folder)                         # the model class by config.json
        assert isinstance(config, TelapelConfig)
        spec = config.model_spec()
        assert {n: tuple(d.shape) for n, d in declared_tensors(spec).items()} == plain.tensor_shapes(raw)
        assert [layer.mixer.kind for layer in config.layers] == [entry["type"] for entry in raw["layers"]]
        assert spec.lm_head_name is None and spec.embedding_name == "embed"
        assert all(layer.arrangement == "output_norm_residual" for layer in spec.layers)
        assert TelapelConfig.from_dict(config.to_dict()) == config and config.to_dict() == raw
    spec = TelapelConfig.from_dict(CONFIG_X).model_spec()
    # layers 3 and 4 run the weights of layers 0 and 2, each on a cache entry of its own
    assert len(spec.layers) == 3
    assert [(entry.layer, entry.cache, entry.writes_cache) for entry in spec.schedule] == [(0, 0, True), (1, 1, True), (2, 2, True), (0, 3, True), (2, 4, True)]
    first, second, third = spec.layers
    assert first.mixer.kind == "rglru" and (first.mixer["width"], first.mixer["blocks"], first.mixer["taps"], first.mixer["decay_rate"]) == (120, 3, 4, 8.0)
    assert second.mixer.kind == "gqa_attention" and second.mixer["values"] == "keys" and second.mixer["sink"] == "unit"
    assert (second.mixer["window"], second.mixer["score_softcap"], second.mixer["qk_conv"], second.mixer["softmax_scale"]) == (50, 20.0, 3, 0.2)
    assert second.mixer["query_temperature"] == (0.4, 48) and second.mixer["distance_slope_exponent"] == 8.0 and second.mixer["qk_norm"]
    assert third.mixer.kind == "latent_attention" and (third.mixer["rot_dim"], third.mixer["kv_rank"], third.mixer["q_rank"]) == (16, 48, 40)
    assert third.mixer["position"].kind == "rotary_interleaved" and third.mixer["position"]["rotary_dim"] == 16 and not third.mixer["output_gate"]
    assert first.ffn.kind == "moe_glu" and (first.ffn["num_experts"], first.ffn["top"], first.ffn["router_groups"]) == (12, 3, (3, 2))
    assert (first.ffn["limit"], first.ffn["shared_limit"], first.ffn["shared_intermediate_size"], first.ffn["router_scores"]) == (1.2, 1.7, 56, "softmax_all")
    assert second.ffn["shared_intermediate_size"] is None and first.mixer_norm["tensor"] == "l0.norm1" and third.ffn_norm["tensor"] == "l2.norm2"
    spec_y = TelapelConfig.from_dict(CONFIG_Y).model_spec()
    assert spec_y.layers[2].ffn is None and spec_y.layers[0].mixer["score_softcap"] is None and spec_y.layers[3].mixer["query_temperature"] is None
    for path, value, match in ((("layers", 0, "type"), "serial", "type"), (("layers", 1, "mixer", "heads"), 5, "multiple"),
                               (("layers", 2, "mixer", "rot", "dims"), 18, "rot"), (("norm", "eps"), 0, "eps"),
                               (("layers", 0, "mlp", "kind"), "dense", "kind"), (("layers", 0, "mlp", "router", "top"), 9, "groups"),
                               (("layers", 0, "mlp", "router", "groups", "count"), 5, "groups"), (("layers", 0, "mixer", "blocks"), 7, "blocks"),
                               (("layers", 3, "weights_of"), 3, "weights_of"), (("layers", 4, "weights_of"), 3, "weights_of"),
                               (("layers", 3, "weights_of"), 1, "sizes"), (("layers", 1, "mixer", "vdim"), 48, "vdim"),
                               (("layers", 1, "mlp", "expert", "limit"), 0.0, "limit"), (("vocab",), None, "vocab")):
        broken = copy.deepcopy(CONFIG_X)
        at = broken
        for key in path[:-1]:
            at = at[key]
        at[path[-1]] = value
        with pytest.raises(ConfigError, match=match):
            TelapelConfig.from_dict(broken)


def test_cache_entries():
    """A recurrent layer asks for its state and its convolution's memory in the request's slot; a latent layer for pages
    of one head whose keys hold the latent and the rotated part, its values the latent alone; an attention layer for
    pages of its keys (which are its values) within its window, and for the memory of its two convolutions. A layer that
    runs another's weights has entries of its own."""
    from flyweight_amd.cache import CacheManager
    from flyweight_amd.config import TelapelConfig
    from flyweight_amd.engine.model import CausalLM
    needs = CausalLM(TelapelConfig.from_dict(CONFIG_X).model_spec()).cache_needs()
    assert set(needs) == {0, 1, 2, 3, 4}
    assert set(needs[0]) == {"state", "conv"} and needs[0]["state"].shape == (120,) and needs[0]["conv"].shape == (120, 3)
    assert needs[3] == needs[0] and needs[4] == needs[2]
    assert set(needs[1]) == {"kv", "conv"} and needs[1]["conv"].shape == ((6 + 2) * 32, 2)
    assert (needs[1]["kv"].num_kv_heads, needs[1]["kv"].head_dim, needs[1]["kv"].window, needs[1]["kv"].v_head_dim) == (2, 32, 50, None)
    assert (needs[2].num_kv_heads, needs[2].head_dim, needs[2].v_head_dim, needs[2].window) == (1, 48 + 16, 48, None)
    needs_z = CausalLM(TelapelConfig.from_dict(CONFIG_Z).model_spec()).cache_needs()
    assert set(needs_z[1]) == {"state"}                      # one tap: nothing to remember
    assert needs_z[4]["kv"].window is None and needs_z[0]["kv"].window == 1
    cache = CacheManager(needs, num_pages=6, max_requests=2)
    cache.admit("a")
    for length in (50, 130, 131, 200, 330):
        cache.reserve("a", length)
        cache.commit("a", length)
        cache.check_invariants()
    windowed = [group for group in cache.groups if group.need.window == 50][0]
    assert [page != -1 for page in windowed.tables["a"]] == [False, False, False, False, True, True]    # the window's pages alone
    cache.release("a")
    assert all(group.pool.free_count == 6 for group in cache.groups) and cache.slots.free_count == 2


def _mix(config, index):
    entry = config["layers"][index]
    return entry, {name[len(f"l{index}.mix."):]: value for name, value in plain.random_weights(config, 3).items() if name.startswith(f"l{index}.mix.")}


def test_plain_mixers_in_one_piece_and_in_pieces():
    """Each mixer over 90 tokens at once equals the same tokens in pieces of 1, 2, 7 and 40 on the carried state."""
    rng = np.random.default_rng(0)
    for config, index in ((CONFIG_X, 0), (CONFIG_X, 1), (CONFIG_X, 2), (CONFIG_Z, 3), (CONFIG_Z, 5), (CONFIG_Y, 2)):
        entry, w = _mix(config, index)
        h = rng.normal(size=(90, config["width"]))
        eps = config["norm"]["eps"]

        def run(rows, state):
            if entry["type"] == "rglru":
                return plain.rglru(rows, w, entry["mixer"]["blocks"], state)
            if entry["type"] == "latent_attention":
                return plain.latent_attention(rows, w, plain._mixer_sizes(entry), eps, state)
            return plain.key_value_attention(rows, w, plain._mixer_sizes(entry), eps, state)
        whole, _ = run(h, None)
        for piece in (1, 2, 7, 40):
            state, parts = None, []
            for at in range(0, 90, piece):
                out, state = run(h[at:at + piece], state)
                parts.append(out)
            assert np.allclose(np.concatenate(parts), whole, rtol=1e-10, atol=1e-10), (entry["type"], piece)


def test_plain_attention_window_sink_distance_and_factor():
    """One head, identity-like weights: a key just inside the window counts, the one just outside does not; with no key
    that scores above zero the term of 1 takes most of the weight; the bias by distance grows with the distance; the
    query factor steps up where floor((p + 1) / every) does."""
    d, T = 8, 12
    eye = np.eye(d)
    w = {"q": eye, "k": eye, "q.b": np.zeros(d), "k.b": np.zeros(d), "q.conv": np.ones((d, 1)), "k.conv": np.ones((d, 1)),
         "q.norm": np.ones(d), "k.norm": np.ones(d), "o": eye}
    sizes = {"heads": 1, "kv_heads": 1, "dim": d, "scale": 1.0, "softcap": None, "window": 4, "temp_coef": 0.0, "temp_every": None}
    h = np.full((T, d), 1e-3)
    h[5] = 10.0 * np.eye(d)[0]      # a value that stands out, at position 5
    out, _ = plain.key_value_attention(h, w, sizes, 1e-6)
    seen = np.abs(out[:, 0]) > 0.01
    assert seen.tolist() == [False] * 5 + [True] * 4 + [False] * 3         # rows 5..8 see key 5 (window 4), row 9 does not
    # a row whose keys all score far below zero gives nearly everything to the term of 1: the output nearly vanishes
    far = dict(sizes, scale=-50.0, window=None)
    out, _ = plain.key_value_attention(np.ones((3, d)), w, far, 1e-6)
    assert np.abs(out).max() < 1e-6
    # equal keys: the weights fall with the distance by exp(-slope * distance), slope = 2^-8 for one head
    level = dict(sizes, window=None, scale=1e-9)
    h = np.ones((6, d))
    h[0] = 2.0                      # only row 0's value differs: its weight in the last row is exp(-5 slope) / (1 + sum)
    out, _ = plain.key_value_attention(h, w, level, 1e-6)
    slope = 2.0 ** -8
    weights = np.exp(-slope * np.arange(5, -1, -1))
    expected = (weights[0] * 2.0 + weights[1:].sum()) / (1.0 + weights.sum())
    assert abs(out[5, 0] - expected) < 1e-6
    # the query factor multiplies the score: with every = 3 rows 0..1 have factor 1, rows 2..4 1 + c ln 2, rows 5..7 1 + c ln 3
    factor = lambda p: 1.0 + 0.5 * np.log((p + 1) // 3 + 1)
    assert [round(factor(p), 6) for p in (0, 1, 2, 4, 5)] == [1.0, 1.0, round(1 + 0.5 * np.log(2), 6), round(1 + 0.5 * np.log(2), 6), round(1 + 0.5 * np.log(3), 6)]
    warm = dict(sizes, window=1, temp_coef=0.5, temp_every=3, scale=1.0)
    out, _ = plain.key_value_attention(np.ones((6, d)), w, warm, 1e-6)
    for p in (0, 2, 5):             # a row sees itself alone: weight e^s / (1 + e^s) with s = d * factor (unit vectors times sqrt(d) each)
        s = d * factor(p)
        assert abs(out[p, 0] - np.exp(s) / (1.0 + np.exp(s))) < 1e-7      # (eps under the norms' roots)


def test_plain_router_and_unit():
    h = np.eye(8)[:3]
    router = np.zeros((8, 8))
    router[:, 0] = [1.0, 0.9, 0.0, 0.0, 5.0, -1.0, -1.0, -1.0]     # row 0: the best expert is 4, in the second group
    router[:, 1] = [2.0, 1.0, 0.5, 0.1, 0.0, 1.9, 1.8, 1.7]        # row 1: the best expert is 0, in the first group
    router[:, 2] = 0.0                                               # row 2: all equal, the lowest ids win
    chosen, weight = plain.route(h, router, top=2, groups=2, keep=1)
    assert chosen.tolist() == [[4, 5], [0, 1], [0, 1]]               # never across the two groups, though 5..7 beat 1 in row 1
    free, _ = plain.route(h, router, top=2, groups=2, keep=2)
    assert free.tolist() == [[4, 0], [0, 5], [0, 1]]
    assert np.allclose(weight.sum(axis=1), 1.0) and np.allclose(weight[1], np.exp([2.0, 1.0]) / np.exp([2.0, 1.0]).sum())
    # the unit's clamps: a gate above the limit counts as the limit, an up value beyond it as the limit with its sign
    one = np.ones((1, 1))
    unit = lambda g, u: plain.clamped_unit(one, np.array([[g]]), np.array([[u]]), one, 1.5)[0, 0]
    assert unit(9.0, 0.3) == unit(1.5, 0.3) and unit(0.7, 8.0) == unit(0.7, 1.5) and unit(0.7, -8.0) == unit(0.7, -1.5)
    assert unit(-9.0, 0.3) != unit(-1.5, 0.3)                        # no limit below on the gate
    assert abs(unit(1.0, 0.5) - 1.0 / (1.0 + np.exp(-1.702)) * 1.5) < 1e-12


def test_plain_model_is_causal_and_every_part_counts():
    for config in (CONFIG_X, CONFIG_Y, CONFIG_Z):
        weights = plain.random_weights(config, 5)
        tokens = random_tokens(config["vocab"], 80, seed=6)
        full = plain.forward(config, weights, tokens)
        assert np.isfinite(full).all()
        assert np.allclose(plain.forward(config, weights, tokens[:50]), full[:50], rtol=1e-9, atol=1e-9)
        model, states = plain.PlainTelapel(config, weights), None
        states = model.start()
        pieces = [model.forward(tokens[at:at + n], states) for at, n in ((0, 33), (33, 1), (34, 2), (36, 44))]
        assert np.allclose(np.concatenate(pieces), full, rtol=1e-9, atol=1e-9)
        assert plain.greedy(config, weights, tokens[:20], 3) == [int(np.argmax(plain.forward(config, weights, tokens[:20])[-1]))] + \
            plain.greedy(config, weights, tokens[:20] + [int(np.argmax(plain.forward(config, weights, tokens[:20])[-1]))], 2)
        for name in weights:
            changed = dict(weights)
            # (a router of which one expert is chosen gives the same choice and the weight 1 whatever its size: its rows are moved on instead)
            changed[name] = np.roll(weights[name], 1, axis=0) if name.endswith(".router") else weights[name] * 1.3 + 0.05
            assert not np.allclose(plain.forward(config, changed, tokens), full, rtol=1e-7, atol=1e-7), f"{name} changes nothing"
