"""A plain, slow Telapel in float64 numpy, one function per mechanism, written from the design's
equations. It shares no code with the package: the tests hold the engine against it.

Notation: T tokens, D model width; a weight W is stored [out, in] and applied as x @ W.T. Every mixer
takes a whole sequence (position 0 first) and can also be walked in pieces: a piece gets the ``state``
that the piece before it returned (None at the start of a sequence).

The design: x = embed[token]; a layer does x += N1(mixer(x)), then x += N2(ff(x)): the sublayers read x
itself and the RMS norm (plain weight) stands on a sublayer's output. Mixers: ``rglru`` (two branches,
one through a short causal convolution and a gated linear recurrence per channel, the other a gelu gate),
``latent_attention`` (softmax attention whose keys and values are maps of one cached latent per token, plus a
rotated key part shared by all heads) and ``attention`` (grouped heads whose values are the keys, short
convolutions on queries and keys, a per-head norm, a query factor that grows with the position, capped
scores, a bias by distance, a sliding window, and a softmax with one more term of 1 in its denominator).
The feed-forward is a mixture of clamped gated units chosen per token among a few groups of experts, with
one unit that every token runs. A layer may use another layer's weights with a state of its own. The head
is the embedding table behind a final norm.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional, Tuple

import numpy as np


# ----- small pieces -------------------------------------------------------------------------
def rms(x: np.ndarray, eps: float) -> np.ndarray:
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def rms_norm(x: np.ndarray, weight: np.ndarray, eps: float) -> np.ndarray:
    return rms(x, eps) * weight


def sigmoid(x: np.ndarray) -> np.ndarray:
    return 1.0 / (1.0 + np.exp(-x))


def softplus(x: np.ndarray) -> np.ndarray:
    return np.logaddexp(0.0, x)


def gelu_tanh(z: np.ndarray) -> np.ndarray:
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def causal_conv(u: np.ndarray, taps: np.ndarray, before: Optional[np.ndarray]) -> Tuple[np.ndarray, np.ndarray]:
    """u [T, C], taps [C, K] whose last column multiplies the current token: y_t = sum_j taps[:, j] *
    u_(t - K + 1 + j). ``before`` [K - 1, C] are the inputs ahead of this piece (zeros at a sequence's
    start). Returns y and the last K - 1 inputs."""
    K = taps.shape[1]
    if before is None:
        before = np.zeros((K - 1, u.shape[1]))
    full = np.concatenate([before, u], axis=0)
    y = np.zeros_like(u)
    for t in range(u.shape[0]):
        for j in range(K):
            y[t] += taps[:, j] * full[t + j]
    return y, full[full.shape[0] - (K - 1):].copy()


# ----- the recurrent mixer --------------------------------------------------------------------
def rglru(h: np.ndarray, w: Dict[str, np.ndarray], blocks: int, state=None):
    """y = gelu_tanh(W_y h + b_y); u = conv(W_x h + b_x) + b_conv; per block of channels r = sigmoid(A_b u_b +
    a_b), i = sigmoid(I_b u_b + i_b); a = exp(-8 r softplus(lam)); S_t = a S_(t-1) + sqrt(1 - a^2) i u;
    out = W_o (S * y). The state is (S, the convolution's last inputs)."""
    S, before = state if state is not None else (None, None)
    y = gelu_tanh(h @ w["y"].T + w["y.b"])
    u, before = causal_conv(h @ w["x"].T + w["x.b"], w["conv"], before)
    u = u + w["conv.b"]
    T, C = u.shape
    size = C // blocks
    r, i = np.zeros_like(u), np.zeros_like(u)
    for b in range(blocks):
        part = u[:, b * size:(b + 1) * size]
        r[:, b * size:(b + 1) * size] = sigmoid(part @ w["ra"][b].T + w["ra.b"][b])
        i[:, b * size:(b + 1) * size] = sigmoid(part @ w["ri"][b].T + w["ri.b"][b])
    out, S = gated_recurrence(u, r, i, w["lam"], S)
    return (out * y) @ w["o"].T, (S, before)


def gated_recurrence(u: np.ndarray, r: np.ndarray, i: np.ndarray, lam: np.ndarray, S: Optional[np.ndarray], rate: float = 8.0):
    """a = exp(-rate r softplus(lam)); S_t = a_t S_(t-1) + sqrt(1 - a_t^2) i_t u_t, from S (zeros if None). Returns
    every S_t [T, C] and the last one."""
    a = np.exp(-rate * r * softplus(lam))
    S = np.zeros(u.shape[1]) if S is None else S
    out = np.zeros_like(u)
    for t in range(u.shape[0]):
        S = a[t] * S + np.sqrt(1.0 - a[t] ** 2) * i[t] * u[t]
        out[t] = S
    return out, S


# ----- rotation of neighbouring channels ------------------------------------------------------------
def rotate_pairs(x: np.ndarray, positions: np.ndarray, dims: int, base: float) -> np.ndarray:
    """x [T, ..., dim]: channels (2i, 2i + 1), i < dims / 2, turn by position * base^(-2i / dims)."""
    out = x.copy()
    half = dims // 2
    if half == 0:
        return out
    freq = base ** (-2.0 * np.arange(half) / dims)
    angle = positions.astype(np.float64)[:, None] * freq[None, :]
    shape = (x.shape[0],) + (1,) * (x.ndim - 2) + (half,)
    c, s = np.cos(angle).reshape(shape), np.sin(angle).reshape(shape)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


# ----- attention over a latent --------------------------------------------------------------------
def latent_attention(h: np.ndarray, w: Dict[str, np.ndarray], sizes: Dict, eps: float, state=None):
    """sizes: heads, dim, rot_dim, vdim, kv_rank, scale, rot_base. The state is (latents so far, rotated key
    parts so far): nothing else of a token is kept."""
    H, d, dr, dv, rk = sizes["heads"], sizes["dim"], sizes["rot_dim"], sizes["vdim"], sizes["kv_rank"]
    past_c, past_kr = state if state is not None else (np.zeros((0, rk)), np.zeros((0, dr)))
    T, start = h.shape[0], past_c.shape[0]
    positions = np.arange(start, start + T)
    q = (rms_norm(h @ w["dq"].T, w["dq.norm"], eps) @ w["uq"].T).reshape(T, H, d + dr)
    q_plain, q_rot = q[..., :d], rotate_pairs(q[..., d:], positions, dr, sizes["rot_base"])
    down = h @ w["dkv"].T
    c = np.concatenate([past_c, rms_norm(down[:, :rk], w["dkv.norm"], eps)], axis=0)
    kr = np.concatenate([past_kr, rotate_pairs(down[:, rk:], positions, dr, sizes["rot_base"])], axis=0)
    k_plain = (c @ w["uk"].T).reshape(-1, H, d)
    v = (c @ w["uv"].T).reshape(-1, H, dv)
    out = np.zeros((T, H, dv))
    for t in range(T):
        n = start + t + 1
        for head in range(H):
            s = (k_plain[:n, head] @ q_plain[t, head] + kr[:n] @ q_rot[t, head]) * sizes["scale"]
            p = np.exp(s - s.max())
            out[t, head] = (p / p.sum()) @ v[:n, head]
    return out.reshape(T, H * dv) @ w["o"].T, (c, kr)


# ----- attention whose values are its keys ----------------------------------------------------------
def key_value_attention(h: np.ndarray, w: Dict[str, np.ndarray], sizes: Dict, eps: float, state=None):
    """sizes: heads, kv_heads, dim, scale, softcap (0: none), window (None: every key), temp_coef, temp_every.
    The state is (values so far, normed keys so far, the convolutions' last inputs of q and of k)."""
    H, G, d = sizes["heads"], sizes["kv_heads"], sizes["dim"]
    if state is None:
        past_v, past_k, before_q, before_k = np.zeros((0, G, d)), np.zeros((0, G, d)), None, None
    else:
        past_v, past_k, before_q, before_k = state
    T, start = h.shape[0], past_v.shape[0]
    q, before_q = causal_conv(h @ w["q"].T + w["q.b"], w["q.conv"], before_q)
    k, before_k = causal_conv(h @ w["k"].T + w["k.b"], w["k.conv"], before_k)
    values = np.concatenate([past_v, k.reshape(T, G, d)], axis=0)             # the keys before their norm
    keys = np.concatenate([past_k, rms_norm(k.reshape(T, G, d), w["k.norm"], eps)], axis=0)
    q = rms_norm(q.reshape(T, H, d), w["q.norm"], eps)
    for t in range(T):
        q[t] *= query_factor(start + t, sizes["temp_coef"], sizes.get("temp_every"))
    out = biased_heads(q, keys, values, start, sizes["scale"], sizes.get("window"), sizes.get("softcap"))
    return out.reshape(T, H * d) @ w["o"].T, (values, keys, before_q, before_k)


def query_factor(position: int, coef: float, every: Optional[int]) -> float:
    """1 + coef ln(floor((p + 1) / every) + 1); 1 where the design has none."""
    return 1.0 + coef * math.log(math.floor((position + 1) / every) + 1.0) if every else 1.0


def biased_heads(q: np.ndarray, keys: np.ndarray, values: np.ndarray, start: int, scale: float, window: Optional[int],
                 softcap: Optional[float], exponent: float = 8.0) -> np.ndarray:
    """q [T, H, d] are the rows at positions start .. start + T - 1 of a sequence whose keys [N, G, d] and values
    [N, G, dv] are given from position 0 on. score = q . k * scale, capped (cap tanh(score / cap)), less slope_h *
    distance with slope_h = 2^(-exponent (h + 1) / H); row i sees keys j with 0 <= i - j < window; the weights are
    e^s / (1 + sum e^s). Returns [T, H, dv]."""
    T, H, _ = q.shape
    G = keys.shape[1]
    out = np.zeros((T, H, values.shape[2]))
    for t in range(T):
        p = start + t
        first = 0 if window is None else max(0, p - window + 1)
        js = np.arange(first, p + 1)
        for head in range(H):
            g = head // (H // G)
            s = (keys[first:p + 1, g] @ q[t, head]) * scale
            if softcap:
                s = softcap * np.tanh(s / softcap)
            s = s - 2.0 ** (-exponent * (head + 1) / H) * (p - js)
            top = max(s.max(), 0.0)
            e = np.exp(s - top)
            out[t, head] = (e / (np.exp(-top) + e.sum())) @ values[first:p + 1, g]
    return out


# ----- the feed-forward -------------------------------------------------------------------------
def clamped_unit(h: np.ndarray, gate: np.ndarray, up: np.ndarray, down: np.ndarray, limit: float) -> np.ndarray:
    g = np.minimum(h @ gate.T, limit)
    u = np.clip(h @ up.T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ down.T


def route(h: np.ndarray, router: np.ndarray, top: int, groups: int, keep: int) -> Tuple[np.ndarray, np.ndarray]:
    """(chosen [T, top], weight [T, top]): softmax over all experts; experts outside the ``keep`` groups (of
    neighbours) with the largest best score cannot be chosen; the chosen scores are divided by their sum."""
    z = h @ router.T
    s = np.exp(z - z.max(axis=-1, keepdims=True))
    s = s / s.sum(axis=-1, keepdims=True)
    T, E = s.shape
    chosen, weight = np.zeros((T, top), dtype=np.int64), np.zeros((T, top))
    for t in range(T):
        best = s[t].reshape(groups, E // groups).max(axis=1)
        kept = np.argsort(-best, kind="stable")[:keep]
        allowed = np.full(E, -np.inf)
        for g in kept:
            allowed[g * (E // groups):(g + 1) * (E // groups)] = s[t, g * (E // groups):(g + 1) * (E // groups)]
        chosen[t] = np.argsort(-allowed, kind="stable")[:top]
        weight[t] = s[t, chosen[t]] / (s[t, chosen[t]].sum() + 1e-20)
    return chosen, weight


def mixture(h: np.ndarray, w: Dict[str, np.ndarray], sizes: Dict) -> np.ndarray:
    """sizes: experts, top, groups, keep, limit, and shared_limit where there is a shared unit."""
    chosen, weight = route(h, w["router"], sizes["top"], sizes["groups"], sizes["keep"])
    out = np.zeros((h.shape[0], w["e0.down"].shape[0]))
    for t in range(h.shape[0]):
        for e, a in zip(chosen[t], weight[t]):
            out[t] += a * clamped_unit(h[t:t + 1], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"], sizes["limit"])[0]
    if "shared.gate" in w:
        out += clamped_unit(h, w["shared.gate"], w["shared.up"], w["shared.down"], sizes["shared_limit"])
    return out


# ----- the model ------------------------------------------------------------------------------
def _under(tensors: Dict[str, np.ndarray], prefix: str) -> Dict[str, np.ndarray]:
    return {name[len(prefix):]: value for name, value in tensors.items() if name.startswith(prefix)}


def _mixer_sizes(entry: Dict) -> Dict:
    m = entry["mixer"]
    if entry["type"] == "latent_attention":
        return {"heads": m["heads"], "dim": m["dim"], "rot_dim": m["rot_dim"], "vdim": m["vdim"], "kv_rank": m["kv_rank"],
                "scale": m["scale"], "rot_base": m["rot"]["base"]}
    if entry["type"] == "attention":
        return {"heads": m["heads"], "kv_heads": m.get("kv_heads", m["heads"]), "dim": m["dim"], "scale": m["scale"],
                "softcap": m.get("softcap"), "window": (m.get("mask") or {}).get("size"),
                "temp_coef": (m.get("q_temp") or {}).get("coef", 0.0), "temp_every": (m.get("q_temp") or {}).get("every")}
    return {}


def _ff_sizes(mlp: Dict) -> Dict:
    router = mlp["router"]
    groups = router.get("groups") or {"count": 1, "keep": 1}
    sizes = {"experts": router["experts"], "top": router["top"], "groups": groups["count"], "keep": groups["keep"],
             "limit": mlp["expert"]["limit"]}
    if mlp.get("shared"):
        sizes["shared_limit"] = mlp["shared"]["limit"]
    return sizes


class PlainTelapel:
    """``config``: the model's configuration as a dict; ``tensors``: name -> float64 array."""

    def __init__(self, config: Dict, tensors: Dict[str, np.ndarray]):
        self.config, self.tensors = config, {k: np.asarray(v, dtype=np.float64) for k, v in tensors.items()}
        self.eps = float(config["norm"]["eps"])

    def start(self) -> List:
        return [None] * len(self.config["layers"])

    def forward(self, tokens, states: Optional[List] = None, keep_layers: bool = False):
        """Logits [T, vocab] of the next ``tokens`` of one sequence; ``states`` (from ``start`` or an earlier
        call) is brought up to date in place."""
        if states is None:
            states = self.start()
        x = self.tensors["embed"][np.asarray(tokens, dtype=np.int64)]
        after = []
        for index, entry in enumerate(self.config["layers"]):
            owner = entry.get("weights_of", index)
            w = _under(self.tensors, f"l{owner}.")
            mix = _under(w, "mix.")
            if entry["type"] == "rglru":
                y, states[index] = rglru(x, mix, entry["mixer"]["blocks"], states[index])
            elif entry["type"] == "latent_attention":
                y, states[index] = latent_attention(x, mix, _mixer_sizes(entry), self.eps, states[index])
            else:
                y, states[index] = key_value_attention(x, mix, _mixer_sizes(entry), self.eps, states[index])
            x = x + rms_norm(y, w["norm1"], self.eps)
            if entry.get("mlp") is not None:
                x = x + rms_norm(mixture(x, _under(w, "mlp."), _ff_sizes(entry["mlp"])), w["norm2"], self.eps)
            after.append(x.copy())
        logits = rms_norm(x, self.tensors["final.norm"], self.eps) @ self.tensors["embed"].T
        return (logits, after) if keep_layers else logits


def forward(config: Dict, weights: Dict[str, np.ndarray], tokens) -> np.ndarray:
    """Logits [T, vocab] of a whole sequence."""
    return PlainTelapel(config, weights).forward(list(tokens))


def greedy(config: Dict, weights: Dict[str, np.ndarray], prompt: List[int], new: int) -> List[int]:
    """The prompt once, then token by token on the carried states."""
    model = PlainTelapel(config, weights)
    states = model.start()
    logits = model.forward(list(prompt), states)
    out = []
    for _ in range(new):
        out.append(int(np.argmax(logits[-1])))
        logits = model.forward([out[-1]], states)
    return out


# ----- tensors of a model --------------------------------------------------------------------------------
def tensor_shapes(config: Dict) -> Dict[str, Tuple[int, ...]]:
    D, V = config["width"], config["vocab"]
    shapes: Dict[str, Tuple[int, ...]] = {"embed": (V, D), "final.norm": (D,)}
    for index, layer in enumerate(config["layers"]):
        if layer.get("weights_of") is not None:
            continue
        base, m = f"l{index}.", layer["mixer"]
        shapes[base + "norm1"] = (D,)
        mix = base + "mix."
        if layer["type"] == "rglru":
            C, B, L = m["width"], m["blocks"], m["conv"]
            shapes.update({mix + "y": (C, D), mix + "y.b": (C,), mix + "x": (C, D), mix + "x.b": (C,), mix + "conv": (C, L),
                           mix + "conv.b": (C,), mix + "ra": (B, C // B, C // B), mix + "ra.b": (B, C // B),
                           mix + "ri": (B, C // B, C // B), mix + "ri.b": (B, C // B), mix + "lam": (C,), mix + "o": (D, C)})
        elif layer["type"] == "latent_attention":
            H, d, dr, dv, rq, rk = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["q_rank"], m["kv_rank"]
            shapes.update({mix + "dq": (rq, D), mix + "dq.norm": (rq,), mix + "uq": (H * (d + dr), rq), mix + "dkv": (rk + dr, D),
                           mix + "dkv.norm": (rk,), mix + "uk": (H * d, rk), mix + "uv": (H * dv, rk), mix + "o": (D, H * dv)})
        else:
            H, G, d, L = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m["conv"]
            shapes.update({mix + "q": (H * d, D), mix + "q.b": (H * d,), mix + "k": (G * d, D), mix + "k.b": (G * d,),
                           mix + "q.norm": (d,), mix + "k.norm": (d,), mix + "q.conv": (H * d, L), mix + "k.conv": (G * d, L),
                           mix + "o": (D, H * d)})
        mlp = layer.get("mlp")
        if mlp is not None:
            shapes[base + "norm2"] = (D,)
            ff = base + "mlp."
            shapes[ff + "router"] = (mlp["router"]["experts"], D)
            units = [(f"e{e}.", mlp["expert"]["ff"]) for e in range(mlp["router"]["experts"])]
            if mlp.get("shared"):
                units.append(("shared.", mlp["shared"]["ff"]))
            for unit, width in units:
                shapes.update({ff + unit + "gate": (width, D), ff + unit + "up": (width, D), ff + unit + "down": (D, width)})
    return shapes


def random_weights(config: Dict, seed: int, experts_alike: float = 0.9) -> Dict[str, np.ndarray]:
    """Weights that make every part count: matrices keep the size of what passes through them (the router's and the
    units' somewhat more, so that the clamps bite), decays from barely forgetting to forgetting at once, biases and
    taps of visible size. The experts of a layer share ``experts_alike`` of their weights: where bfloat16 rounding turns
    a close call of the router the output then moves by a part of an expert, not by all of it, while in float32 any
    wrong choice still shows far above the comparison's limit."""
    rng = np.random.default_rng(seed)
    weights: Dict[str, np.ndarray] = {}
    common: Dict[Tuple[str, str], np.ndarray] = {}
    for name, shape in tensor_shapes(config).items():
        leaf = name.split(".")[-1]
        parts = name.split(".")
        if len(parts) == 4 and parts[1] == "mlp" and parts[2].startswith("e") and experts_alike:
            if (parts[0], leaf) not in common:
                common[parts[0], leaf] = rng.normal(0.0, 1.5 if leaf != "down" else 1.0, shape) / math.sqrt(shape[-1])
            own = rng.normal(0.0, 1.5 if leaf != "down" else 1.0, shape) / math.sqrt(shape[-1])
            weights[name] = experts_alike * common[parts[0], leaf] + (1.0 - experts_alike) * own
            continue
        if leaf in ("norm1", "norm2", "norm") or name == "final.norm":
            value = rng.uniform(0.6, 1.4, shape)
        elif leaf == "lam":
            value = rng.uniform(-5.0, 1.0, shape)
        elif leaf == "b":
            value = rng.normal(0.0, 0.5, shape)
        elif leaf == "conv":
            value = rng.normal(0.0, 0.6, shape)
        elif name == "embed":
            value = rng.normal(0.0, 1.0, shape)
        elif leaf == "router" or leaf in ("gate", "up"):
            value = rng.normal(0.0, 1.5, shape) / math.sqrt(shape[-1])
        else:
            value = rng.normal(0.0, 1.0, shape) / math.sqrt(shape[-1])
        weights[name] = value
    return weights
