"""A recurrent block around a real-gated linear recurrent unit (the recurrent block of Griffin).

Two branches of ``width`` channels read the layer's input: y = gelu_tanh(W_y h + b_y) and u = conv(W_x h + b_x), a
short causal convolution over time for every channel (``conv`` taps with a bias, the last tap the token's own,
zeros before a request's start, no activation).  u is cut into ``blocks`` equal parts; in part b, with square
matrices A_b and I_b:

    r = sigmoid(A_b u_b + a_b);   i = sigmoid(I_b u_b + c_b);   log a = -rate * r * softplus(lam);   a = e^(log a)
    S' = a S + sqrt(1 - a^2) * i * u          for the tokens of a request in their order, S starting at zero

(no special case for a request's first token), and the mixer's output is W_o (S' * y).

What a request keeps between steps is one float32 slot: the convolution's last ``conv - 1`` inputs and S.  The
gates, the decays with their logarithms and exponentials and S are 32-bit whatever the activations' type.

Parameters: ``width``, ``blocks``, ``conv``, ``rate`` (8 if absent), and ``names``: role (``y``, ``y_bias``, ``x``,
``x_bias``, ``conv``, ``conv_bias``, ``ra``, ``ra_bias``, ``ri``, ``ri_bias``, ``lam``, ``o``) -> the tensor's whole
name under the layer's prefix.
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import Mixer, ParamSpec, StateNeed, StateView
from .linear import decode_weight, linear, linear_unrounded, tensor_names
from .registry import MIXERS
from .spec import PartSpec


class GatedLinearRecurrence(Mixer):
    NAMES = {"y": "mix.y", "y_bias": "mix.y.b", "x": "mix.x", "x_bias": "mix.x.b", "conv": "mix.conv",
             "conv_bias": "mix.conv.b", "ra": "mix.ra", "ra_bias": "mix.ra.b", "ri": "mix.ri", "ri_bias": "mix.ri.b",
             "lam": "mix.lam", "o": "mix.o"}
    RATE = 8.0  # what the kernel multiplies r * softplus(lam) by

    def __init__(self, spec: PartSpec, *, hidden_size: int):
        self.hidden_size = int(hidden_size)
        self.width = int(spec["width"])
        self.blocks = int(spec["blocks"])
        self.taps = int(spec["conv"])
        if min(self.width, self.blocks, self.taps) < 1 or self.width % self.blocks:
            raise ValueError(f"a recurrent unit of {self.width} channels in {self.blocks} equal blocks")
        if float(spec.get("rate", self.RATE)) != self.RATE:
            raise ValueError(f"the recurrent unit's kernel has the rate {self.RATE} built in")
        self.block = self.width // self.blocks
        self.names = tensor_names(self.NAMES, spec.get("names"))
        self.s_off = (self.taps - 1) * self.width
        self.state_size = self.s_off + self.width
        self.w_in = self.b_in = self.w_gates = self.w_o = None
        self.conv_w = self.conv_b = self.r_bias = self.i_bias = self.lam = None

    def param_specs(self, prefix: str) -> list[ParamSpec]:
        at = {role: f"{prefix}.{name}" for role, name in self.names.items()}
        H, W, B, S = self.hidden_size, self.width, self.blocks, self.block
        return [
            ParamSpec(at["y"], (W, H)), ParamSpec(at["y_bias"], (W,), init=("normal", 0.1)),
            ParamSpec(at["x"], (W, H)), ParamSpec(at["x_bias"], (W,), init=("normal", 0.1)),
            ParamSpec(at["conv"], (W, self.taps), init=("normal", 0.5)),
            ParamSpec(at["conv_bias"], (W,), init=("normal", 0.1)),
            ParamSpec(at["ra"], (B, S, S), init=("normal", 0.1)), ParamSpec(at["ra_bias"], (B, S), init=("normal", 0.5)),
            ParamSpec(at["ri"], (B, S, S), init=("normal", 0.1)), ParamSpec(at["ri_bias"], (B, S), init=("normal", 0.5)),
            ParamSpec(at["lam"], (W,), init=("normal", 1.0)),
            ParamSpec(at["o"], (H, W)),
        ]

    def bind(self, tensors, prefix, device, dtype) -> None:
        at = {role: f"{prefix}.{name}" for role, name in self.names.items()}

        def get(role, to=dtype):
            return tensors[at[role]].to(device=device, dtype=to).contiguous()

        f32 = torch.float32
        self.w_in = decode_weight(torch.cat([get("x"), get("y")], dim=0).contiguous(), self.tiled_weights)  # [x | y]
        self.b_in = torch.cat([get("x_bias", f32), get("y_bias", f32)]).contiguous()
        # a block's two matrices one after the other: one product by blocks leaves g_r and g_i of a block side by side
        self.w_gates = torch.cat([get("ra"), get("ri")], dim=1).contiguous()  # [blocks, 2 block, block]
        self.w_o = decode_weight(get("o"), self.tiled_weights)
        self.conv_w, self.conv_b = get("conv", f32), get("conv_bias", f32)
        self.r_bias = get("ra_bias", f32).reshape(-1).contiguous()
        self.i_bias = get("ri_bias", f32).reshape(-1).contiguous()
        self.lam = get("lam", f32)

    def cache_need(self) -> StateNeed:
        return StateNeed((self.state_size,), torch.float32)

    def forward(self, x: torch.Tensor, step, cache: StateView) -> torch.Tensor:
        if not cache.writes:
            raise ValueError("a recurrent layer moves its state on with every token and cannot read another's")
        n = x.shape[0]
        W = self.width
        slots = cache.slots
        proj = ops.add_bias(linear(x, self.w_in, sliced_ok=True), self.b_in)  # [n, x | y]
        u = torch.empty((n, W), dtype=x.dtype, device=x.device)
        moves = ops.conv_moves_state(step)  # single tokens: the convolution moves its state on itself
        ops.causal_conv(proj, 0, W, self.conv_w, self.conv_b, slots, 0, step, u, move_state=moves, act="none")
        if not moves:
            ops.conv_state_update(proj, 0, W, self.taps, slots, 0, step)
        gates = ops.gemm_blocks_f32(u, self.w_gates)  # [n, per block: g_r | g_i], 32-bit
        out = ops.gated_linear_scan(u, gates, self.block, self.r_bias, self.i_bias, self.lam, proj, W, slots,
                                    self.s_off, step)
        return linear_unrounded(out, self.w_o)


MIXERS.register("gated_linear_recurrence", GatedLinearRecurrence)
