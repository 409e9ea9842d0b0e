"""A linear recurrence over a matrix state per head whose decay the token itself forms ("wkv").

With h' the input of the token before (zeros before a sequence's first token), each of r, k, v, g, w reads a
mix of its own, h + (h' - h) * mu_s. r, k, v = W_r, W_k, W_v of their mixes (heads of ``dim`` channels),
gate = silu(W_g mix_g), and the decay per head and key channel is w = exp(-exp(W_w2 tanh(W_w1 mix_w) + w0)).
Per head, with the state S [key channel, value channel] (zero at the start):

    o_t = (S + diag(u) k_t v_t^T)^T r_t;      S <- diag(w_t) S + k_t v_t^T

(u, the bonus, counts for the current token only). Each head's o is divided by its root mean square, times a
weight per head and channel, times the gate; out = W_o of the heads side by side. The mixes, the decay with
its exponentials, the state, the read-out and the heads' norm are float32 whatever the run's dtype; a request
keeps S and its last h. The inner width of the decay's low-rank map is ``decay_rank``.
"""

from __future__ import annotations

from typing import Dict

import torch

from ..cache.needs import FixedState
from ..config.spec import ConfigError
from ..kernels import ops
from ..weights.loader import TensorDecl
from .base import Mixer, register_mixer
from .linear import Linear
from .norm import LazyNorm

_DEFAULT_NAMES = {"r": "r", "k": "k", "v": "v", "g": "g", "w1": "w1", "w2": "w2", "w0": "w0", "u": "u", "norm": "norm", "o": "o",
                  "mu_r": "mu.r", "mu_k": "mu.k", "mu_v": "mu.v", "mu_g": "mu.g", "mu_w": "mu.w"}
_MIXES = ("r", "k", "v", "g", "w")


@register_mixer("wkv")
class Wkv(Mixer):
    graph_safe = True
    accepts_lazy_norm = True        # the norm in front is taken into the kernel that forms the mixes
    wants_unnormed_rows = True      # ... in float32, from the residual rows themselves: it asks for them also where the normed rows exist

    def __init__(self, spec):
        super().__init__(spec)
        self.hidden = int(spec["hidden_size"])
        self.heads = int(spec["num_heads"])
        self.dim = int(spec["head_dim"])
        self.rank = int(spec["decay_rank"])
        self.eps = float(spec["norm_eps"])
        self.names = {**_DEFAULT_NAMES, **dict(spec.get("names", {}))}
        if not 1 <= self.dim <= 256:
            raise ConfigError(f"the recurrence's head size {self.dim} must lie in 1..256")
        if self.heads < 1 or self.rank < 1:
            raise ConfigError("the recurrence needs at least one head and a decay map of at least one inner channel")
        self.width = self.heads * self.dim

    def cache_need(self):
        return {"state": FixedState((self.heads, self.dim, self.dim), torch.float32),
                "shift": FixedState((self.hidden,), torch.float32)}

    def _name(self, which: str) -> str:
        return self.prefix + self.names[which]

    def mixing_flops(self, rows: int, keys_before: int = 0) -> int:
        """Flops of the recurrence itself: per token and head a read and a write of the state, a multiply and an add each
        (the write two)."""
        return 5 * self.heads * self.dim * self.dim * rows

    def tensors(self) -> Dict[str, TensorDecl]:
        D, W = self.hidden, self.width
        declared = {self._name("mu_" + s): TensorDecl((D,), "vector", "bias") for s in _MIXES}
        for s in ("r", "k", "v", "g"):
            declared[self._name(s)] = TensorDecl((W, D))
        declared[self._name("w1")] = TensorDecl((self.rank, D))
        declared[self._name("w2")] = TensorDecl((W, self.rank))
        declared[self._name("w0")] = TensorDecl((W,), "vector", "bias")
        declared[self._name("u")] = TensorDecl((self.heads, self.dim), "vector", "bias")
        declared[self._name("norm")] = TensorDecl((W,), "vector", "norm")
        declared[self._name("o")] = TensorDecl((D, W))
        return declared

    def bind(self, tensors, dtype, device) -> None:
        super().bind(tensors, dtype, device)
        t = {which: tensors[self._name(which)] for which in self.names}
        self.mu = torch.stack([t["mu_" + s] for s in _MIXES]).contiguous()
        self.r, self.k, self.v, self.g = (Linear(t[s]) for s in ("r", "k", "v", "g"))
        self.w1, self.w2 = Linear(t["w1"]), Linear(t["w2"])
        self.w0, self.u, self.norm_weight = t["w0"], t["u"].reshape(-1).contiguous(), t["norm"]
        self.out = Linear(t["o"])

    def heads_output(self, h, ctx, cache) -> torch.Tensor:
        """The heads' normed and gated read-outs [rows, heads * dim] in the activation dtype; the request's state
        and last input move on by the step's rows."""
        if isinstance(h, LazyNorm) and h.row_index is None and h.rms_parameters() is not None:
            weight, eps, one_centered = h.rms_parameters()
            x = h.x
        else:       # rows that are normed already: mixed in float32 as they are
            x, weight, eps, one_centered = (h.tensor() if isinstance(h, LazyNorm) else h).to(torch.float32), None, 0.0, False
        mixes = ops.token_shift_mix(x, weight, eps, one_centered, self.mu, cache["shift"].state, ctx.row_seg, ctx.seg_row0,
                                    ctx.seg_slot, ctx.num_segments, self.dtype)
        r, k, v, gate = (linear.forward(mixes[i], out_dtype=torch.float32) for i, linear in enumerate((self.r, self.k, self.v, self.g)))
        inner = ops.tanh_rows(self.w1.forward(mixes[4], out_dtype=torch.float32), self.dtype)
        a = self.w2.forward(inner, out_dtype=torch.float32)
        o = ops.wkv_recurrence(r, k, v, a, self.w0, self.u, cache["state"].state, ctx.seg_row0, ctx.seg_slot, ctx.num_segments,
                               self.heads, self.dim)
        return ops.gated_head_norm(o, gate, self.norm_weight, self.heads, self.dim, self.eps, self.dtype, gate_silu=True)

    def output(self, h, ctx, cache) -> torch.Tensor:
        return self.out.forward(self.heads_output(h, ctx, cache), out_dtype=torch.float32)

    def forward(self, h, residual, ctx, cache):
        return self.out.accumulate(self.heads_output(h, ctx, cache), residual, then=getattr(ctx, "upcoming_norm", None))
