"""A plain, slow Dalerax in float64 numpy, one function per mechanism, written from the design's
equations. It shares no code with the package: the tests hold the engine against it.

Notation: T tokens, D model width; a weight W is stored [out, in] and applied as x @ W.T. Every
mixer takes a whole sequence (position 0 first); ``wkv_step`` takes one token and the state before it,
so that a sequence can also be walked token by token.

The design: x = embed[token] * scale + pos[position]; every layer is parallel, with h = N(x) (an RMS
norm whose weight is stored around zero) it adds mixer(h) + ff(h) to x. Mixers: ``wkv`` (a linear
recurrence over a matrix state per head with a decay per key channel formed from the token, a bonus for
the current token, inputs mixed with the token before) and ``attention`` (grouped softmax attention with
rotary positions whose frequencies are stretched by wavelength, a sliding window that also keeps the
first tokens of the sequence, one more term exp(sink) per head in the softmax's denominator, and
optionally the keys and values of an earlier layer). Feed-forwards: a gated unit, or a mixture of
such units chosen per token by a router, with one unit shared by all tokens.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional, Tuple

import numpy as np


# ----- small pieces -------------------------------------------------------------------------
def rms(x: np.ndarray, eps: float) -> np.ndarray:
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def norm_around_zero(x: np.ndarray, weight: np.ndarray, eps: float) -> np.ndarray:
    return rms(x, eps) * (1.0 + weight)


def sigmoid(x: np.ndarray) -> np.ndarray:
    return 1.0 / (1.0 + np.exp(-x))


def silu(x: np.ndarray) -> np.ndarray:
    return x * sigmoid(x)


def gated_unit(h: np.ndarray, gate: np.ndarray, up: np.ndarray, down: np.ndarray) -> np.ndarray:
    return (silu(h @ gate.T) * (h @ up.T)) @ down.T


# ----- rotary positions with stretched frequencies ------------------------------------------------
def rotary_frequencies(dims: int, base: float, scaling: Optional[Dict]) -> np.ndarray:
    """f_i = base^(-2i / dims) for i < dims / 2. With ``scaling`` (factor, low, high, original): a
    frequency whose wavelength 2 pi / f is shorter than original / high stays, one whose wavelength is
    longer than original / low is divided by factor, and between the two the frequency is the blend
    (1 - s) f / factor + s f with s = (original / wavelength - low) / (high - low)."""
    f = base ** (-2.0 * np.arange(dims // 2) / dims)
    if not scaling:
        return f
    factor, low, high, original = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
    out = f.copy()
    for i, fi in enumerate(f):
        wavelength = 2.0 * math.pi / fi
        if wavelength < original / high:
            continue
        if wavelength > original / low:
            out[i] = fi / factor
        else:
            s = (original / wavelength - low) / (high - low)
            out[i] = (1.0 - s) * fi / factor + s * fi
    return out


def rotate_halves(x: np.ndarray, positions: np.ndarray, dims: int, freq: np.ndarray) -> np.ndarray:
    """x [T, heads, dim]: channel i < dims / 2 of a head turns together with channel i + dims / 2 by the
    angle position * freq[i]; channels from ``dims`` on stay."""
    out = x.copy()
    half = dims // 2
    if half == 0:
        return out
    angle = positions[:, None].astype(np.float64) * freq[None, :]
    c, s = np.cos(angle)[:, None, :], np.sin(angle)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


# ----- mixer: attention -------------------------------------------------------------------------
def may_see(i: int, j: int, size: Optional[int], keep_first: int) -> bool:
    return j <= i and (size is None or i - j < size or j < keep_first)


def sink_heads(q: np.ndarray, k: np.ndarray, v: np.ndarray, scale: float, size: Optional[int], keep_first: int,
               sink: Optional[np.ndarray]) -> np.ndarray:
    """q [T, H, d], k [T, G, d], v [T, G, dv] of one sequence from position 0 -> [T, H, dv]. Row i sees
    key j if ``may_see``; the weights are exp(score) over the sum of the seen keys' exponentials plus
    exp(sink[head]), a term with no value of its own."""
    T, H = q.shape[:2]
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    for head in range(H):
        g = head // (H // G)
        for i in range(T):
            seen = [j for j in range(i + 1) if may_see(i, j, size, keep_first)]
            score = k[seen, g] @ q[i, head] * scale
            top = max(score.max(), sink[head]) if sink is not None else score.max()
            weight = np.exp(score - top)
            total = weight.sum() + (math.exp(sink[head] - top) if sink is not None else 0.0)
            out[i, head] = (weight / total) @ v[seen, g]
    return out


def attention_keys_values(h: np.ndarray, w: Dict[str, np.ndarray], m: Dict) -> Tuple[np.ndarray, np.ndarray]:
    """What an attention layer leaves in its cache for a sequence from position 0: keys after rotation, values."""
    T = h.shape[0]
    G = m.get("kv_heads", m["heads"])
    d, dv = m["dim"], m.get("vdim", m["dim"])
    rot = m.get("rot")
    k = (h @ w["k"].T).reshape(T, G, d)
    if rot:
        k = rotate_halves(k, np.arange(T), rot["dims"], rotary_frequencies(rot["dims"], rot["base"], rot.get("scaling")))
    return k, (h @ w["v"].T).reshape(T, G, dv)


def attention_mixer(h: np.ndarray, w: Dict[str, np.ndarray], m: Dict, shared: Optional[Tuple[np.ndarray, np.ndarray]] = None):
    """-> (output [T, D], (keys, values)). ``shared``: the keys and values of the layer named by kv_from."""
    T = h.shape[0]
    H, d = m["heads"], m["dim"]
    rot, mask = m.get("rot"), m.get("mask")
    q = (h @ w["q"].T).reshape(T, H, d)
    if rot:
        q = rotate_halves(q, np.arange(T), rot["dims"], rotary_frequencies(rot["dims"], rot["base"], rot.get("scaling")))
    k, v = shared if shared is not None else attention_keys_values(h, w, m)
    size = mask["size"] if mask else None
    keep = mask.get("keep_first", 0) if mask else 0
    o = sink_heads(q, k, v, m.get("scale", d ** -0.5), size, keep, w.get("sink"))
    return o.reshape(T, -1) @ w["o"].T, (k, v)


# ----- mixer: wkv --------------------------------------------------------------------------------
def wkv_inputs(h: np.ndarray, before: np.ndarray, w: Dict[str, np.ndarray]):
    """Rows h [T, D] and the row before each (``before`` [T, D]) -> r, k, v [T, H d], gate [T, H d], decay
    [T, H d] in (0, 1)."""
    mixed = {s: h + (before - h) * w["mu." + s] for s in "rkvgw"}
    r, k, v = (mixed[s] @ w[s].T for s in "rkv")
    gate = silu(mixed["g"] @ w["g"].T)
    decay = np.exp(-np.exp(np.tanh(mixed["w"] @ w["w1"].T) @ w["w2"].T + w["w0"]))
    return r, k, v, gate, decay


def wkv_read_write(S: np.ndarray, r: np.ndarray, k: np.ndarray, v: np.ndarray, decay: np.ndarray, u: np.ndarray):
    """One token, one head: S [d, d] (key channel, value channel). The read-out sees the state before
    this token plus the token's own outer product weighted by the bonus u per key channel; then the state
    decays per key channel and takes the outer product."""
    o = (S + (u * k)[:, None] * v[None, :]).T @ r
    return o, decay[:, None] * S + k[:, None] * v[None, :]


def wkv_finish(o: np.ndarray, gate: np.ndarray, w: Dict[str, np.ndarray], heads: int, eps: float) -> np.ndarray:
    """o [T, H d]: each head divided by its root mean square, times the norm weight, times the gate, then W_o."""
    T = o.shape[0]
    normed = rms(o.reshape(T, heads, -1), eps).reshape(T, -1)
    return (normed * w["norm"] * gate) @ w["o"].T


def wkv_mixer(h: np.ndarray, w: Dict[str, np.ndarray], m: Dict, eps: float, state=None):
    """A run of tokens from ``state`` = (matrix state [H, d, d], the last h) or from the start -> (output, state)."""
    T, D = h.shape
    H, d = m["heads"], m["dim"]
    S, last = state if state is not None else (np.zeros((H, d, d)), np.zeros(D))
    S = S.copy()
    before = np.concatenate([last[None, :], h[:-1]], axis=0)
    r, k, v, gate, decay = wkv_inputs(h, before, w)
    o = np.zeros((T, H * d))
    for t in range(T):
        for head in range(H):
            span = slice(head * d, (head + 1) * d)
            o[t, span], S[head] = wkv_read_write(S[head], r[t, span], k[t, span], v[t, span], decay[t, span], w["u"][head])
    return wkv_finish(o, gate, w, H, eps), (S, h[-1].copy())


def wkv_step(h_row: np.ndarray, w, m, eps, state):
    out, state = wkv_mixer(h_row[None, :], w, m, eps, state)
    return out[0], state


# ----- feed-forwards ------------------------------------------------------------------------------
def route(h: np.ndarray, router: np.ndarray, bias: np.ndarray, top: int):
    """-> (chosen experts [T, top], their weights [T, top]): the ``top`` largest logits, softmax over those only."""
    logits = h @ router.T + bias
    chosen = np.argsort(-logits, axis=-1, kind="stable")[:, :top]
    picked = np.take_along_axis(logits, chosen, axis=-1)
    weight = np.exp(picked - picked.max(axis=-1, keepdims=True))
    return chosen, weight / weight.sum(axis=-1, keepdims=True)


def mixture(h: np.ndarray, w: Dict[str, np.ndarray], mlp: Dict) -> np.ndarray:
    experts, top = mlp["router"]["experts"], mlp["router"]["top"]
    chosen, weight = route(h, w["router"], w["router.b"], top)
    out = np.zeros((h.shape[0], w["e0.down"].shape[0]))
    for t in range(h.shape[0]):
        for e, share in zip(chosen[t], weight[t]):
            out[t] += share * gated_unit(h[t], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"])
    if mlp.get("shared"):
        out += gated_unit(h, w["shared.gate"], w["shared.up"], w["shared.down"])
    assert experts == sum(1 for name in w if name.endswith(".gate") and name.startswith("e"))
    return out


def feed_forward(h: np.ndarray, w: Dict[str, np.ndarray], mlp: Optional[Dict]) -> np.ndarray:
    if mlp is None:
        return np.zeros_like(h)
    if mlp["kind"] == "dense":
        return gated_unit(h, w["gate"], w["up"], w["down"])
    return mixture(h, w, mlp)


# ----- the model ----------------------------------------------------------------------------------
def part(weights: Dict[str, np.ndarray], prefix: str) -> Dict[str, np.ndarray]:
    return {name[len(prefix):]: value for name, value in weights.items() if name.startswith(prefix)}


def forward(config: Dict, weights: Dict[str, np.ndarray], tokens: List[int], layers_out: Optional[List[np.ndarray]] = None) -> np.ndarray:
    """One sequence from position 0 -> logits [T, vocab]. ``layers_out``: receives x after every layer."""
    T = len(tokens)
    eps = config["norm"]["eps"]
    x = weights["embed"][np.asarray(tokens)] * config.get("embedding", {}).get("scale", 1.0) + weights["pos"][:T]
    caches: Dict[int, Tuple[np.ndarray, np.ndarray]] = {}
    for index, layer in enumerate(config["layers"]):
        base = f"l{index}."
        h = norm_around_zero(x, weights[base + "norm1"], eps)
        mix, m = part(weights, base + "mix."), layer["mixer"]
        if layer["type"] == "wkv":
            mixed, _ = wkv_mixer(h, mix, m, eps)
        else:
            source = m.get("kv_from")
            mixed, caches[index] = attention_mixer(h, mix, m, caches[source] if source is not None else None)
        x = x + (mixed + feed_forward(h, part(weights, base + "mlp."), layer.get("mlp")))
        if layers_out is not None:
            layers_out.append(x.copy())
    return norm_around_zero(x, weights["final.norm"], eps) @ weights["head"].T * config.get("logit_scale", 1.0)


def greedy(config: Dict, weights: Dict[str, np.ndarray], prompt: List[int], new: int) -> List[int]:
    tokens, out = list(prompt), []
    for _ in range(new):
        out.append(int(np.argmax(forward(config, weights, tokens)[-1])))
        tokens.append(out[-1])
    return out


# ----- tensors of a model --------------------------------------------------------------------------------
def tensor_shapes(config: Dict, decay_rank: int = 8) -> Dict[str, Tuple[int, ...]]:
    D, V = config["width"], config["vocab"]
    shapes: Dict[str, Tuple[int, ...]] = {"embed": (V, D), "pos": (config["max_positions"], D), "final.norm": (D,), "head": (V, D)}
    for index, layer in enumerate(config["layers"]):
        base, m = f"l{index}.", layer["mixer"]
        shapes[base + "norm1"] = (D,)
        if layer["type"] == "wkv":
            W = m["heads"] * m["dim"]
            for s in "rkvgw":
                shapes[base + "mix.mu." + s] = (D,)
            for s in "rkvg":
                shapes[base + "mix." + s] = (W, D)
            rank = m.get("decay_rank", decay_rank)
            shapes.update({base + "mix.w1": (rank, D), base + "mix.w2": (W, rank), base + "mix.w0": (W,), base + "mix.u": (m["heads"], m["dim"]),
                           base + "mix.norm": (W,), base + "mix.o": (D, W)})
        else:
            H, G, d = m["heads"], m.get("kv_heads", m["heads"]), m["dim"]
            dv = m.get("vdim", d)
            shapes.update({base + "mix.q": (H * d, D), base + "mix.sink": (H,), base + "mix.o": (D, H * dv)})
            if m.get("kv_from") is None:
                shapes.update({base + "mix.k": (G * d, D), base + "mix.v": (G * dv, D)})
        mlp = layer.get("mlp")
        if mlp is None:
            continue
        units = {"": mlp["ff"]} if mlp["kind"] == "dense" else {f"e{e}.": mlp["expert"]["ff"] for e in range(mlp["router"]["experts"])}
        if mlp["kind"] == "moe":
            shapes.update({base + "mlp.router": (mlp["router"]["experts"], D), base + "mlp.router.b": (mlp["router"]["experts"],)})
            if mlp.get("shared"):
                units["shared."] = mlp["shared"]["ff"]
        for unit, ff in units.items():
            shapes.update({base + f"mlp.{unit}gate": (ff, D), base + f"mlp.{unit}up": (ff, D), base + f"mlp.{unit}down": (D, ff)})
    return shapes


def random_weights(config: Dict, seed: int, decay_rank: int = 8) -> Dict[str, np.ndarray]:
    """Weights that make every part count: matrices keep the size of what passes through them, sinks of about one,
    decays from barely forgetting to forgetting at once, a bonus and mixing weights of visible size."""
    rng = np.random.default_rng(seed)
    weights: Dict[str, np.ndarray] = {}
    for name, shape in tensor_shapes(config, decay_rank).items():
        leaf = name.split(".")[-1]
        if name.endswith("norm1") or name == "final.norm":
            value = rng.uniform(-0.3, 0.3, shape)
        elif ".mu." in name:
            value = rng.uniform(0.0, 1.0, shape)
        elif leaf == "w0":
            value = rng.uniform(-6.0, 0.5, shape)
        elif leaf == "u":
            value = rng.normal(0.0, 0.5, shape)
        elif leaf == "norm":
            value = rng.uniform(0.7, 1.3, shape)
        elif leaf == "sink":
            value = rng.normal(0.0, 1.5, shape)
        elif leaf == "b":
            value = rng.normal(0.0, 0.5, shape)
        elif name == "pos":
            value = rng.normal(0.0, 0.5, shape)
        elif name == "embed":
            value = rng.normal(0.0, 1.0, shape)
        else:
            value = rng.normal(0.0, 1.0, shape) / math.sqrt(shape[-1])
        weights[name] = value
    return weights
