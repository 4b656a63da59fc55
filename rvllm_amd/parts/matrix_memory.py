"""A matrix memory with exponential gates (the mLSTM of xLSTM): a mixer that keeps a matrix, a vector and a
running maximum a head instead of keys and values.

q = W_q h * dim^(-1/2) and k = W_k h (``heads`` heads of ``dim``), v = W_v h (``heads`` heads of ``vdim``).  A head
has a log input gate i = cap * tanh((w_i . h + b_i) / cap) and a log forget gate
f = logsigmoid(cap * tanh((w_f . h + b_f) / cap)).  For the tokens of a request in their order, with S [dim, vdim],
n [dim] and m starting at zero (m at 0, not at minus infinity):

    m' = max(f + m, i);   S' = e^(f + m - m') S + e^(i - m') k v^T;   n' = e^(f + m - m') n + e^(i - m') k
    o = S'^T q / (max(|n' . q|, e^(-m')) + 1e-6)

Every head's o is divided by its root mean square (``eps`` inside the root), the heads side by side are multiplied
by a weight of all heads' size and by sigmoid(W_g h), and W_o projects the result.

What a request keeps between steps is one float32 slot: S of every head, then n, then m.  The gates, their
exponentials, S, n, m and the output norm are 32-bit whatever the activations' type.

Parameters: ``heads``, ``dim``, ``vdim``, ``gate_cap``, ``eps``, ``divisor_eps`` (1e-6 if absent), and ``names``:
role (``q``, ``k``, ``v``, ``g``, ``i``, ``f``, ``i_bias``, ``f_bias``, ``norm``, ``o``) -> the tensor's whole name
under the layer's prefix.
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import Mixer, ParamSpec, StateNeed, StateView
from .linear import decode_weight, linear, linear_unrounded, tensor_names
from .registry import MIXERS
from .spec import PartSpec


class MatrixMemory(Mixer):
    NAMES = {"q": "mix.q", "k": "mix.k", "v": "mix.v", "g": "mix.g", "i": "mix.i", "f": "mix.f", "i_bias": "mix.i.b",
             "f_bias": "mix.f.b", "norm": "mix.norm", "o": "mix.o"}
    DIVISOR_EPS = 1e-6  # built into the kernel

    def __init__(self, spec: PartSpec, *, hidden_size: int):
        self.hidden_size = int(hidden_size)
        self.heads = int(spec["heads"])
        self.dim = int(spec["dim"])
        self.vdim = int(spec["vdim"])
        self.cap = float(spec["gate_cap"])
        self.eps = float(spec["eps"])
        if float(spec.get("divisor_eps", self.DIVISOR_EPS)) != self.DIVISOR_EPS:
            raise ValueError(f"the matrix memory's kernel raises its divisor by {self.DIVISOR_EPS}")
        if min(self.heads, self.dim, self.vdim) < 1 or not self.cap > 0.0:
            raise ValueError("a matrix memory needs positive sizes and a positive cap of its gates")
        self.names = tensor_names(self.NAMES, spec.get("names"))
        self.qk_size = self.heads * self.dim
        self.v_size = self.heads * self.vdim
        # columns of the fused projection: q | k | v | g | i | f
        self.k_col = self.qk_size
        self.v_col = 2 * self.qk_size
        self.g_col = self.v_col + self.v_size
        self.i_col = self.g_col + self.v_size
        self.f_col = self.i_col + self.heads
        # the slot: S [heads, vdim, dim], n [heads, dim], m [heads]
        self.n_off = self.heads * self.dim * self.vdim
        self.m_off = self.n_off + self.qk_size
        self.state_size = self.m_off + self.heads
        self.w_in = self.w_o = self.i_bias = self.f_bias = self.norm_w = None

    def param_specs(self, prefix: str) -> list[ParamSpec]:
        at = {role: f"{prefix}.{name}" for role, name in self.names.items()}
        H = self.hidden_size
        return [
            ParamSpec(at["q"], (self.qk_size, H)), ParamSpec(at["k"], (self.qk_size, H)),
            ParamSpec(at["v"], (self.v_size, H)), ParamSpec(at["g"], (self.v_size, H)),
            ParamSpec(at["i"], (self.heads, H)), ParamSpec(at["f"], (self.heads, H)),
            ParamSpec(at["i_bias"], (self.heads,), init=("normal", 0.5)),
            ParamSpec(at["f_bias"], (self.heads,), init=("normal_about", 2.0, 0.5)),
            ParamSpec(at["norm"], (self.v_size,), init=("normal_about", 1.0, 0.1)),
            ParamSpec(at["o"], (H, self.v_size)),
        ]

    def bind(self, tensors, prefix, device, dtype) -> None:
        at = {role: f"{prefix}.{name}" for role, name in self.names.items()}

        def get(role, to=dtype):
            return tensors[at[role]].to(device=device, dtype=to)

        rows = [get(role) for role in ("q", "k", "v", "g", "i", "f")]
        self.w_in = decode_weight(torch.cat(rows, dim=0).contiguous(), self.tiled_weights)
        self.w_o = decode_weight(get("o").contiguous(), self.tiled_weights)
        f32 = torch.float32  # what enters the recurrence is 32-bit
        self.i_bias, self.f_bias = get("i_bias", f32).contiguous(), get("f_bias", f32).contiguous()
        self.norm_w = get("norm", f32).contiguous()

    def cache_need(self) -> StateNeed:
        return StateNeed((self.state_size,), torch.float32)

    def forward(self, x: torch.Tensor, step, cache: StateView) -> torch.Tensor:
        if not cache.writes:
            raise ValueError("a matrix-memory layer moves its state on with every token and cannot read another's")
        proj = linear(x, self.w_in)  # [n, q | k | v | g | i | f]
        o, divisor = ops.matrix_memory(proj, 0, self.k_col, self.v_col, self.i_col, self.f_col, self.i_bias, self.f_bias,
                              self.cap, self.dim ** -0.5, cache.slots, 0, self.n_off, self.m_off, step, self.heads,
                              self.dim, self.vdim)
        y = ops.head_norm_gate(o, proj, self.g_col, self.norm_w, self.eps, self.heads, self.vdim, x.dtype,
                               act="sigmoid", divisor=divisor)
        return linear_unrounded(y, self.w_o)


MIXERS.register("matrix_memory", MatrixMemory)
