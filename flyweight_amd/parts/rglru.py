"""A recurrent block around a real-gated linear recurrent unit (the recurrent block of Griffin: De, Smith et al.,
"Griffin: Mixing Gated Linear Recurrences with Local Attention for Efficient Language Models").

Two branches of ``width`` channels read the same input: y = gelu_tanh(W_y h + b_y), and u = conv(W_x h + b_x) + b_c, a short
causal convolution per channel. The channels of u form ``blocks`` equal blocks; in block b the recurrence gate is
r = sigmoid(A_b u_b + a_b) and the input gate i = sigmoid(I_b u_b + i_b) (square maps [out, in] per block). With
a = exp(-rate * r * softplus(lam)) the state moves as S <- a S + sqrt(1 - a^2) * (i * u), from S = 0, and the block's output
is W_o (S * y). Per request the slot keeps S (float32 [width]) and the convolution's last taps - 1 inputs.

Everything behind the two projections is float32 in either run dtype: the convolution, both gates' maps, the decay
and the state; S * y is rounded once, for the output product.
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

_DEFAULT_NAMES = {"y": "y", "y_bias": "y.b", "x": "x", "x_bias": "x.b", "conv": "conv", "conv_bias": "conv.b", "ra": "ra",
                  "ra_bias": "ra.b", "ri": "ri", "ri_bias": "ri.b", "lam": "lam", "o": "o"}


@register_mixer("rglru")
class RGLRU(Mixer):
    graph_safe = True

    def __init__(self, spec):
        super().__init__(spec)
        self.hidden = int(spec["hidden_size"])
        self.width = int(spec["width"])
        self.blocks = int(spec["blocks"])
        self.taps_count = int(spec["taps"])
        self.rate = float(spec.get("decay_rate", 8.0))
        self.names = {**_DEFAULT_NAMES, **dict(spec.get("names", {}))}
        if self.blocks < 1 or self.width % self.blocks:
            raise ConfigError(f"{self.width} recurrent channels are not {self.blocks} equal blocks")
        if not 1 <= self.taps_count <= 16:
            raise ConfigError(f"a short convolution of {self.taps_count} taps (1..16)")
        if not self.rate > 0:
            raise ConfigError("the decay's rate must be positive")
        self.block_width = self.width // self.blocks

    def cache_need(self):
        need = {"state": FixedState((self.width,), torch.float32)}
        if self.taps_count > 1:
            need["conv"] = FixedState((self.width, self.taps_count - 1), torch.float32)
        return need

    def _name(self, which: str) -> str:
        return self.prefix + self.names[which]

    def mixing_flops(self, rows: int, keys_before: int = 0) -> int:
        """The two gates' maps per block, the convolution and the recurrence's few operations per channel."""
        return rows * (4 * self.width * self.block_width + 2 * self.width * self.taps_count + 12 * self.width)

    def tensors(self) -> Dict[str, TensorDecl]:
        D, C, B, w, L = self.hidden, self.width, self.blocks, self.block_width, self.taps_count
        return {
            self._name("y"): TensorDecl((C, D)), self._name("y_bias"): TensorDecl((C,), "vector", "bias"),
            self._name("x"): TensorDecl((C, D)), self._name("x_bias"): TensorDecl((C,), "vector", "bias"),
            self._name("conv"): TensorDecl((C, L), "vector", "conv"), self._name("conv_bias"): TensorDecl((C,), "vector", "bias"),
            self._name("ra"): TensorDecl((B, w, w)), self._name("ra_bias"): TensorDecl((B, w), "vector", "bias"),
            self._name("ri"): TensorDecl((B, w, w)), self._name("ri_bias"): TensorDecl((B, w), "vector", "bias"),
            self._name("lam"): TensorDecl((C,), "vector", "bias"),
            self._name("o"): TensorDecl((D, C)),
        }

    def bind(self, tensors, dtype, device) -> None:
        super().bind(tensors, dtype, device)
        t = {which: tensors[self._name(which)] for which in self.names}
        # one operand for both branches (float32 sums out: the gelu and the convolution read them as they are)
        self.in_proj = Linear(torch.cat([t["y"], t["x"]], dim=0), torch.cat([t["y_bias"], t["x_bias"]]))
        # per block one map for both gates: the rows of A_b, then those of I_b
        self.gate_maps = torch.cat([t["ra"], t["ri"]], dim=1).contiguous()          # [blocks][2 w][w]
        self.r_bias, self.i_bias = t["ra_bias"].reshape(-1).contiguous(), t["ri_bias"].reshape(-1).contiguous()
        self.taps, self.conv_bias, self.lam = t["conv"], t["conv_bias"], t["lam"]
        self.out = Linear(t["o"])
        self._no_conv_state = None

    def _conv_state(self, cache):
        if "conv" in cache:
            return cache["conv"].state
        slots = cache["state"].state.shape[0]
        if self._no_conv_state is None or self._no_conv_state.shape[0] != slots:
            self._no_conv_state = torch.zeros((slots, self.width, 0), dtype=torch.float32, device=self.device)
        return self._no_conv_state

    def gated_state(self, h, ctx, cache) -> torch.Tensor:
        """S * y [rows, width] in the activation dtype; the request's state and convolution memory move on."""
        both = self.in_proj.forward(h, out_dtype=torch.float32)
        y, x = both[:, :self.width], both[:, self.width:]
        u = ops.causal_conv(x, self.taps, self.conv_bias, self._conv_state(cache), ctx.row_seg, ctx.seg_row0, ctx.seg_slot,
                            ctx.num_segments, single_rows=ctx.all_decode)
        gates = ops.head_linear(u, self.gate_maps, torch.float32)
        return ops.rglru_scan(u, gates, y, self.r_bias, self.i_bias, self.lam, self.rate, cache["state"].state, ctx.seg_row0,
                              ctx.seg_slot, ctx.num_segments, self.block_width, self.dtype)

    def output(self, h, ctx, cache) -> torch.Tensor:
        return self.out.forward(self.gated_state(h, ctx, cache), out_dtype=torch.float32)

    def forward(self, h, residual, ctx, cache):
        return self.out.accumulate(self.gated_state(h, ctx, cache), residual, then=getattr(ctx, "upcoming_norm", None))
