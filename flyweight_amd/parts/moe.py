"""A mixture of gated feed-forward units chosen per token.

Router logits z = W_router h + b in float32 (h as the products read it); the ``top`` experts with the largest
logits are chosen (ties: the lowest id) and weighted by the softmax over the chosen logits alone. An expert is
W_down (silu(W_gate h) * (W_up h)) without biases; the output is the weighted sum of the chosen experts'
outputs, summed in the order of the choices. ``shared_intermediate_size``: one more unit of that width runs for
every token and is added. The experts' weights lie stacked ([experts, 2 ff, hidden] gate rows then up rows,
[experts, hidden, ff]); a step sorts its (token, choice) pairs by expert on the device and runs each expert's
pairs as tiles of one grouped product, so nothing crosses to the host and a decode step can be recorded.

``router_scores`` "softmax_all": the scores are the softmax over all experts, and the chosen experts' scores divided by
their sum (+ 1e-20) are the weights (the choice is the same: the largest scores are the largest logits).
``router_groups`` (count, keep): the experts form ``count`` equal groups of neighbours, a group's score is its best
expert's, and only experts of the ``keep`` best groups can be chosen. ``unit`` "clamped" with ``limit`` (and ``alpha``,
``shift``): an expert is W_down (g sigmoid(alpha g) (u + shift)) with g = min(W_gate h, limit), u = clamp(W_up h, -limit,
limit); the shared unit is then of the same form with ``shared_limit``. Registered as ``moe_swiglu`` and ``moe_glu``.
"""

from __future__ import annotations

from typing import Dict

import torch

from ..config.spec import ConfigError, PartSpec
from ..kernels import ops
from ..weights.loader import TensorDecl
from .base import FeedForward, build_part, register_feed_forward
from .linear import Linear
from .norm import LazyNorm

_DEFAULT_NAMES = {"router": "router", "router_bias": "router.b", "expert": "e{index}.", "gate": "gate", "up": "up", "down": "down",
                  "shared": "shared."}


@register_feed_forward("moe_glu")
@register_feed_forward("moe_swiglu")
class MoeSwiGLU(FeedForward):
    graph_safe = True
    accepts_lazy_norm = True        # handed on to the shared unit, whose first product can take the norm

    def __init__(self, spec):
        super().__init__(spec)
        self.hidden = int(spec["hidden_size"])
        self.experts = int(spec["num_experts"])
        self.top = int(spec["top"])
        self.intermediate = int(spec["intermediate_size"])
        self.shared_intermediate = int(spec.get("shared_intermediate_size") or 0)
        self.router_bias = bool(spec.get("router_bias", True))
        self.score_all = spec.get("router_scores", "softmax_chosen") == "softmax_all"
        self.groups, self.keep_groups = (int(n) for n in (spec.get("router_groups") or (1, 1)))
        self.clamped = spec.get("unit", "swiglu") == "clamped"
        self.glu = (float(spec["limit"]), float(spec.get("alpha", 1.702)), float(spec.get("shift", 1.0))) if self.clamped else None
        self.names = {**_DEFAULT_NAMES, **dict(spec.get("names", {}))}
        if spec.get("router_scores", "softmax_chosen") not in ("softmax_chosen", "softmax_all") or spec.get("unit", "swiglu") not in ("swiglu", "clamped"):
            raise ConfigError("a mixture's router scores are 'softmax_chosen' or 'softmax_all', its units 'swiglu' or 'clamped'")
        if self.groups < 1 or self.groups > 64 or self.experts % self.groups or not 1 <= self.keep_groups <= self.groups \
                or self.top > self.keep_groups * (self.experts // self.groups):
            raise ConfigError(f"{self.experts} experts in {self.groups} groups (equal ones, at most 64) of which {self.keep_groups} "
                              f"are kept cannot give {self.top} experts a token")
        if self.clamped and not self.glu[0] > 0:
            raise ConfigError("a clamped unit needs a positive limit")
        if not 1 <= self.top <= self.experts or self.experts > 1024 or self.top > 64:
            raise ConfigError(f"a mixture of {self.experts} experts (at most 1,024) with {self.top} a token (at most 64)")
        self.shared = None
        if self.shared_intermediate:
            shared = {"hidden_size": self.hidden, "intermediate_size": self.shared_intermediate,
                      "names": {which: self.names[which] for which in ("gate", "up", "down")}, "weight_suffix": ""}
            if self.clamped:
                shared.update(limit=float(spec.get("shared_limit", self.glu[0])), alpha=self.glu[1], shift=self.glu[2])
            self.shared = build_part("ffn", PartSpec("clamped_glu" if self.clamped else "swiglu", shared,
                                                     prefix=self.prefix + self.names["shared"]))

    def sub_parts(self):
        return (self.shared,) if self.shared is not None else ()

    def _expert(self, index: int, which: str) -> str:
        return self.prefix + self.names["expert"].format(index=index) + self.names[which]

    def tensors(self) -> Dict[str, TensorDecl]:
        D, F = self.hidden, self.intermediate
        # the router's product sums in float32 (its operands' products are exact there) and leaves float32 logits
        declared = {self.prefix + self.names["router"]: TensorDecl((self.experts, D))}
        if self.router_bias:
            declared[self.prefix + self.names["router_bias"]] = TensorDecl((self.experts,), "vector", "bias")
        for index in range(self.experts):
            declared[self._expert(index, "gate")] = TensorDecl((F, D))
            declared[self._expert(index, "up")] = TensorDecl((F, D))
            declared[self._expert(index, "down")] = TensorDecl((D, F))
        if self.shared is not None:
            declared.update(self.shared.tensors())
        return declared

    def bind(self, tensors, dtype, device) -> None:
        super().bind(tensors, dtype, device)
        self.router = Linear(tensors[self.prefix + self.names["router"]])
        self.bias = tensors[self.prefix + self.names["router_bias"]] if self.router_bias else None
        self.gate_up = torch.stack([torch.cat([tensors[self._expert(e, "gate")], tensors[self._expert(e, "up")]], dim=0)
                                    for e in range(self.experts)]).contiguous()
        self.down = torch.stack([tensors[self._expert(e, "down")] for e in range(self.experts)]).contiguous()
        if self.shared is not None:
            self.shared.bind(tensors, dtype, device)

    # ----- what a step reads and computes (the experts' weights are read only where tokens chose them) --------
    def gathered_tensors(self):
        return (self.gate_up, self.down)

    def chosen_weight_bytes(self, rows: int) -> float:
        """Bytes of the experts that ``rows`` tokens are expected to choose, each ``top`` different ones and
        every expert as likely as any other: experts * (1 - (1 - top / experts) ** rows) of them."""
        per_expert = (self.gate_up[0].numel() + self.down[0].numel()) * self.gate_up.element_size()
        return self.experts * (1.0 - (1.0 - self.top / self.experts) ** max(int(rows), 0)) * per_expert

    def chosen_flops_per_token(self) -> int:
        return 2 * self.top * 3 * self.hidden * self.intermediate

    def route(self, h: torch.Tensor):
        """(chosen [rows, top], weight [rows, top]) of the rows ``h``."""
        logits = self.router.forward(h, out_dtype=torch.float32)
        return ops.moe_route(logits, self.bias, self.top, self.groups, self.keep_groups, self.score_all)

    def forward(self, h, residual, ctx):
        rows = (h.tensor() if isinstance(h, LazyNorm) else h)
        chosen, weight = self.route(rows)
        begin, place_row, pair_place = ops.moe_arrange(chosen, self.experts)
        places = rows.shape[0] * self.top
        hidden = ops.grouped_gemm(rows, place_row, self.gate_up, begin, places, gated=True, out_dtype=rows.dtype, glu=self.glu)
        outputs = ops.grouped_gemm(hidden, None, self.down, begin, places, gated=False, out_dtype=torch.float32)
        ops.moe_combine_(residual, outputs, weight, pair_place)
        if self.shared is not None:
            return self.shared.forward(h if getattr(self.shared, "accepts_lazy_norm", False) else rows, residual, ctx)
        return None

    def output(self, h, ctx) -> torch.Tensor:
        out = torch.empty((h.shape[0], self.hidden), dtype=torch.float32, device=h.device)
        ops.fill_zero(out)
        self.forward(h, out, ctx)
        return out
