"""Shared by the Dalerax tests: small configurations that differ from each other in every size and option,
model folders with random weights that make every part count, and the comparison's limits."""

from __future__ import annotations

import copy
import json
import os
from typing import Dict, List, Optional

import numpy as np

import plain_dalerax as plain


def attention(heads, kv_heads, dim, vdim, window, keep_first, rot_dims, base, scale, scaling=None, kv_from=None):
    rot = {"base": base, "dims": rot_dims}
    if scaling is not None:
        rot["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    out = {"dim": dim, "heads": heads, "kv_heads": kv_heads, "rot": rot, "scale": scale, "vdim": vdim}
    if window is not None:
        out["mask"] = {"size": window, "keep_first": keep_first}
    if kv_from is not None:
        out["kv_from"] = kv_from
    return {"type": "attention", "mixer": out}


def wkv(heads, dim):
    return {"type": "wkv", "mixer": {"dim": dim, "heads": heads}}


def dense(ff):
    return {"ff": ff, "kind": "dense"}


def moe(experts, top, ff, shared):
    out = {"expert": {"ff": ff}, "kind": "moe", "router": {"experts": experts, "top": top}}
    if shared is not None:
        out["shared"] = {"ff": shared}
    return out


def layer(mixer, mlp):
    return {**mixer, "mlp": mlp}


def model(vocab, width, layers, eps=1e-5, positions=512, embedding_scale=3.0, logit_scale=0.7):
    return {"architecture": "Dalerax", "vocab": vocab, "width": width, "max_positions": positions, "norm": {"eps": eps},
            "embedding": {"scale": embedding_scale}, "logit_scale": logit_scale, "layers": layers}


# X: both mixers, every feed-forward. A window of 40 that crosses page borders with three kept keys, partial
# rotation with stretched frequencies, values wider than keys, a layer that reads its keys and values through a
# wider window and keeps more first keys than their owner, a recurrence of heads of 24 channels, seven experts of
# which three are chosen with a shared unit, a dense unit, a layer without feed-forward.
CONFIG_X = model(300, 96, [
    layer(wkv(4, 24), dense(160)),
    layer(attention(4, 2, 32, 48, 40, 3, 16, 10000.0, 0.25, scaling=(4.0, 1.0, 4.0, 64)), moe(7, 3, 40, 56)),
    layer(attention(4, 2, 32, 48, 70, 5, 16, 10000.0, 0.2, scaling=(4.0, 1.0, 4.0, 64), kv_from=1), None),
    layer(wkv(2, 40), moe(5, 2, 48, None)),
    layer(attention(2, 2, 64, 64, None, 0, 64, 500000.0, 0.125), dense(96)),
])

# Y: pointed softmaxes (score spreads of about three), a window of 64 and one of 33 tokens with one kept key and with
# seventy (more than a page of them), a single kv head, a head of 16 channels, experts of which one is chosen,
# as many chosen as there are, no shared unit, a recurrence with one head, no scaling of the embedding or the logits.
CONFIG_Y = model(200, 64, [
    layer(attention(2, 1, 48, 32, 64, 1, 24, 1000.0, 0.45), moe(4, 1, 64, 32)),
    layer(wkv(1, 64), moe(3, 3, 32, None)),
    layer(attention(4, 4, 16, 16, 33, 70, 8, 100.0, 0.7, scaling=(8.0, 1.0, 2.0, 32)), dense(128)),
    layer(attention(2, 1, 48, 32, 20, 0, 24, 1000.0, 0.45, kv_from=0), dense(64)),
    layer(wkv(4, 16), None),
], eps=1e-6, positions=400, embedding_scale=1.0, logit_scale=1.0)

# Z: the corners. A window of one key (a row sees itself and the kept keys), a window longer than any prompt here, no
# rotation, heads of 8 and of 20 channels (off the matrix cores' steps), one head on one key head and six on three, a
# recurrence of heads of 100 channels and one of 4, a feed-forward width that is no multiple of eight, two experts.
CONFIG_Z = model(97, 40, [
    layer(attention(1, 1, 8, 24, 1, 2, 0, 10000.0, 1.0), None),
    layer(wkv(1, 100), dense(50)),
    layer(attention(6, 3, 20, 8, 500, 4, 20, 10000.0, 0.25), moe(2, 1, 50, 20)),
    layer(wkv(3, 4), None),
    layer(attention(6, 3, 20, 8, 7, 0, 20, 10000.0, 0.3, kv_from=2), moe(9, 4, 12, 12)),
], positions=384)

# W: wide enough that a prompt of some hundred tokens goes through the tiled prompt products and the matrix-core
# attention (keys of 64 and values of 128 channels), a recurrence of heads of 64 channels, sixteen experts.
CONFIG_W = model(1000, 512, [
    layer(wkv(8, 64), dense(1344)),
    layer(attention(8, 2, 64, 128, 150, 6, 48, 100000.0, 0.11, scaling=(4.0, 1.0, 4.0, 256)), moe(16, 4, 256, 384)),
    layer(attention(8, 2, 64, 128, 100, 70, 48, 100000.0, 0.11, scaling=(4.0, 1.0, 4.0, 256), kv_from=1), moe(8, 2, 512, None)),
    layer(wkv(4, 128), dense(1024)),
], positions=4096)

CONFIGS = {"X": CONFIG_X, "Y": CONFIG_Y, "Z": CONFIG_Z, "W": CONFIG_W}

# Largest difference from the plain float64 model, as a fraction of the largest logit compared, and the same for the
# root mean square. float32 shows the logic right; the bfloat16 limits have to tell rounding (2e-3 at every stored
# activation) from a fault, and the configurations make faults large. In bfloat16 a router's choice between two
# experts of nearly equal logits can fall the other way, and a read-out is divided by its own size, which now and then
# is nearly nothing: one row in fifty may pass the largest difference, the root mean square over all rows has to hold.
MAX_TOL = {"float32": 3e-5, "bfloat16": 8e-2}
RMS_TOL = {"float32": 6e-6, "bfloat16": 2e-2}
ROWS_OVER = {"float32": 0.0, "bfloat16": 0.02}


def only_mixer(config: dict, kind: str) -> dict:
    """The same model with the layers of one mixer alone and no feed-forward: one mechanism behind its norm."""
    out = copy.deepcopy(config)
    kept = [index for index, entry in enumerate(out["layers"]) if entry["type"] == kind]
    layers = []
    for index in kept:
        entry = dict(out["layers"][index], mlp=None)
        if entry["mixer"].get("kv_from") is not None:
            entry["mixer"] = dict(entry["mixer"], kv_from=kept.index(entry["mixer"]["kv_from"]))
        layers.append(entry)
    out["layers"] = layers
    return out


def make_folder(folder: str, config: dict, seed: int = 0, decay_rank: int = 8):
    """Writes config.json and model.safetensors (bfloat16 matrices) and returns the weights as the plain model
    reads them: the stored values, in float64."""
    import torch
    from safetensors.torch import save_file
    weights = plain.random_weights(config, seed, decay_rank)
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
