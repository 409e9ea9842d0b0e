"""Shared by the Telapel tests: small configurations that differ from each other in every size and option,
model folders with random weights that make every part count, and the comparison's limits."""

from __future__ import annotations

import copy
import json
import os
from typing import List, Optional

import numpy as np

import plain_telapel as plain


def rglru(width, blocks, conv):
    return {"type": "rglru", "mixer": {"blocks": blocks, "conv": conv, "width": width}}


def latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, base=10000.0):
    return {"type": "latent_attention", "mixer": {"dim": dim, "heads": heads, "kv_rank": kv_rank, "q_rank": q_rank,
                                                  "rot": {"base": base, "dims": rot_dim}, "rot_dim": rot_dim, "scale": scale, "vdim": vdim}}


def attention(heads, kv_heads, dim, conv, window, softcap, scale, temp=None):
    out = {"conv": conv, "dim": dim, "heads": heads, "kv_heads": kv_heads, "scale": scale, "vdim": dim}
    if window is not None:
        out["mask"] = {"size": window}
    if softcap is not None:
        out["softcap"] = softcap
    if temp is not None:
        out["q_temp"] = {"coef": temp[0], "every": temp[1]}
    return {"type": "attention", "mixer": out}


def moe(experts, top, groups, keep, ff, limit, shared=None):
    out = {"expert": {"ff": ff, "limit": limit}, "kind": "moe",
           "router": {"experts": experts, "groups": {"count": groups, "keep": keep}, "top": top}}
    if shared is not None:
        out["shared"] = {"ff": shared[0], "limit": shared[1]}
    return out


def layer(mixer, mlp, weights_of=None):
    out = {**copy.deepcopy(mixer), "mlp": copy.deepcopy(mlp)}
    if weights_of is not None:
        out["weights_of"] = weights_of
    return out


def model(vocab, width, layers, eps=1e-5):
    return {"architecture": "Telapel", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}


# X: every mixer, a layer that runs another's weights on a state of its own, a window of 50 that crosses page
# borders, a cap, a query factor that steps up every 48 positions, two key heads under six, three taps; a latent
# of 48 channels with a rotated part of 16, values wider than keys; twelve experts in three groups of which two
# are kept, three chosen, a shared unit; a recurrence of three blocks with four taps.
_X_MIX = moe(12, 3, 3, 2, 40, 1.2, shared=(56, 1.7))
CONFIG_X = model(300, 96, [
    layer(rglru(120, 3, 4), _X_MIX),
    layer(attention(6, 2, 32, 3, 50, 20.0, 0.2, temp=(0.4, 48)), moe(8, 2, 4, 2, 48, 0.9)),
    layer(latent(4, 16, 16, 32, 40, 48, 0.2), _X_MIX),
    layer(rglru(120, 3, 4), _X_MIX, weights_of=0),
    layer(latent(4, 16, 16, 32, 40, 48, 0.2), _X_MIX, weights_of=2),
])

# Y: a window of 64 and one of 33, one key head, two taps and one, no cap in one layer, a query
# factor from the second position on, a latent of 32 with a rotated part of 32 and few heads, one group (every
# expert can be chosen), one expert chosen, as many chosen as there are, no shared unit, a layer without feed-forward,
# a recurrence of one block and two taps.
CONFIG_Y = model(200, 64, [
    layer(attention(2, 1, 48, 2, 64, None, 0.3, temp=(0.25, 2)), moe(4, 1, 1, 1, 64, 2.5, shared=(32, 0.8))),
    layer(rglru(64, 1, 2), moe(3, 3, 1, 1, 32, 1.0)),
    layer(latent(2, 32, 32, 16, 24, 32, 0.35, base=100.0), None),
    layer(attention(4, 4, 16, 1, 33, 8.0, 0.6), moe(6, 2, 3, 1, 24, 1.5)),
    layer(attention(2, 1, 48, 2, 64, None, 0.3, temp=(0.25, 2)), moe(4, 1, 1, 1, 64, 2.5, shared=(32, 0.8)), weights_of=0),
], eps=1e-6)

# Z: the corners. A window of one key (a row sees itself and the term of 1), a window longer than any prompt here,
# no window, heads of 8 and of 20 channels (off the matrix cores' steps), a latent of 24 with a rotated part of 2,
# one head, a recurrence of as many blocks as channels and one of a single tap, a width that is no multiple of eight,
# two experts in two groups.
CONFIG_Z = model(97, 44, [
    layer(attention(1, 1, 8, 4, 1, 5.0, 1.0), None),
    layer(rglru(12, 12, 1), moe(2, 1, 2, 1, 50, 3.0)),
    layer(latent(1, 12, 2, 20, 9, 24, 0.5), moe(9, 4, 3, 2, 12, 0.5, shared=(12, 0.5))),
    layer(attention(6, 3, 20, 5, 500, None, 0.25, temp=(0.2, 7)), None),
    layer(attention(3, 1, 20, 2, None, 50.0, 0.3), moe(2, 2, 1, 1, 20, 1.0)),
    layer(rglru(50, 5, 7), None),
])

# W: wide enough that a prompt of some hundred tokens goes through the tiled prompt products and the matrix-core
# attention (a latent of 128 + 64 channels; eight heads of 64 on two key heads), sixteen experts in four groups.
_W_MIX = moe(16, 4, 4, 2, 256, 1.5, shared=(384, 2.0))
CONFIG_W = model(1000, 512, [
    layer(rglru(640, 5, 4), _W_MIX),
    layer(latent(8, 64, 64, 64, 192, 128, 0.09), _W_MIX),
    layer(attention(8, 2, 64, 3, 150, 30.0, 0.125, temp=(0.5, 128)), moe(8, 2, 2, 1, 512, 1.0)),
    layer(rglru(640, 5, 4), _W_MIX, weights_of=0),
])

CONFIGS = {"X": CONFIG_X, "Y": CONFIG_Y, "Z": CONFIG_Z, "W": CONFIG_W}

# Largest difference from the plain float64 model, as a fraction of the largest logit compared, and the same for the
# root mean square. float32 shows the logic right; the bfloat16 limits have to tell rounding (2e-3 at every stored
# activation) from a fault, and the configurations make faults large. In bfloat16 a router's choice between two
# experts (or two groups) of nearly equal scores can fall the other way; the experts of a layer are drawn alike in most
# of their weights, so that such a row moves by a part of an expert: one row in twenty may pass the largest difference,
# the root mean square over all rows has to hold.
MAX_TOL = {"float32": 3e-5, "bfloat16": 8e-2}
RMS_TOL = {"float32": 6e-6, "bfloat16": 2e-2}
ROWS_OVER = {"float32": 0.0, "bfloat16": 0.05}


def only_mixer(config: dict, kind: str) -> dict:
    """The same model with the layers of one mixer alone and no feed-forward: one mechanism behind its norm."""
    out = copy.deepcopy(config)
    kept = [index for index, entry in enumerate(out["layers"]) if entry["type"] == kind]
    layers = []
    for index in kept:
        entry = dict(out["layers"][index], mlp=None)
        if entry.get("weights_of") is not None:
            entry["weights_of"] = kept.index(entry["weights_of"])
        layers.append(entry)
    out["layers"] = layers
    return out


def make_folder(folder: str, config: dict, seed: int = 0):
    """Writes config.json and model.safetensors (bfloat16 matrices) and returns the weights as the plain model
    reads them: the stored values, in float64."""
    import torch
    from safetensors.torch import save_file
    weights = plain.random_weights(config, seed)
    stored = {name: torch.from_numpy(value).to(torch.bfloat16) for name, value in weights.items()}
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as handle:
        json.dump(config, handle)
    save_file({name: value.contiguous() for name, value in stored.items()}, os.path.join(folder, "model.safetensors"))
    return {name: value.to(torch.float64).numpy() for name, value in stored.items()}


def random_tokens(vocab: int, count: int, seed: int) -> List[int]:
    return np.random.default_rng(seed).integers(0, vocab, size=count).tolist()


def assert_close(found: np.ndarray, expected: np.ndarray, dtype: str, what: str = "", scale: Optional[float] = None) -> None:
    assert found.shape == expected.shape, f"{what}: shape {found.shape} vs {expected.shape}"
    assert np.isfinite(found).all(), f"{what}: non-finite values"
    scale = max(1.0, float(np.abs(expected).max())) if scale is None else scale
    error = np.abs(found.astype(np.float64) - expected)
    worst, rms = float(error.max()), float(np.sqrt(np.mean(error ** 2)))
    over = error.reshape(error.shape[0], -1).max(axis=-1) > MAX_TOL[dtype] * scale
    allowed = int(ROWS_OVER[dtype] * error.shape[0])
    assert int(over.sum()) <= allowed, (f"{what}: largest difference {worst:.3e} exceeds {MAX_TOL[dtype] * scale:.3e} in {int(over.sum())} rows "
                                        f"({allowed} allowed; first row over: {int(np.argmax(over))})")
    assert rms <= RMS_TOL[dtype] * scale, f"{what}: rms difference {rms:.3e} exceeds {RMS_TOL[dtype] * scale:.3e}"
