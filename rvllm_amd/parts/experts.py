"""A mixture of experts: each token's feed-forward is the weighted sum of a few small gated feed-forwards.

Which experts a token uses is the router's matter.  ``token_table``: a stored
integer table ``[vocab, top]`` gives each token id its ``top`` experts (the
entries of a row differ), each with weight 1 / top; nothing is learned from
the activations.  The step's (token, choice) pairs are sorted by expert on the
device (``ops.moe_route``), each expert's rows are multiplied against its own
matrices in one launch for all experts (``ops.gemm_experts``), and the results
return to their tokens (``ops.moe_combine``): no launch depends on which
experts the tokens chose, so a step can be replayed from a graph.

``sigmoid_topk``: a learned router ``[experts, hidden]`` gives every token 32-bit
logits; the ``top`` experts with the largest logits are chosen (of equal ones
the lower index), each with the weight sigmoid(logit), not renormalized.  With
``weight_on`` = ``input`` (the only form this router has) a choice's weight
multiplies the expert's input, not its output: the token's result is
sum_k expert_k(w_k * x).  The choice is made on the device (``ops.moe_topk``)
and sorted by the same kernel as a table's.

An expert computes down(act(gate(x), up(x))) without biases.  ``activation``:
``clamped_glu`` with ``limit`` and ``alpha``: g = min(gate, limit), u =
clamp(up, -limit, limit), act = g * sigmoid(alpha g) * (u + 1); ``silu_glu``:
act = gate * sigmoid(gate) * up.
``shared`` (optional: ``intermediate_size``, ``limit``, ``alpha``) is one more
expert of the same form that every token uses with weight 1.

``names``: ``expert`` (a pattern with ``{}`` for the expert's number),
``table``, ``router``, ``shared`` under the layer's prefix; ``gate``, ``up``, ``down``
under an expert's name.
"""

from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops
from .base import FeedForward, ParamSpec
from .linear import decode_weight, linear, tensor_names
from .registry import FEED_FORWARDS
from .spec import PartSpec


class RoutedExperts(FeedForward):
    NAMES = {"expert": "mlp.e{}", "table": "mlp.table", "router": "mlp.router", "shared": "mlp.shared", "gate": "gate",
             "up": "up", "down": "down"}
    ROUTERS = ("token_table", "sigmoid_topk")
    ACTIVATIONS = ("clamped_glu", "silu_glu")

    def __init__(self, spec: PartSpec, *, hidden_size: int):
        self.hidden_size = int(hidden_size)
        self.num_experts = int(spec["experts"])
        self.top = int(spec["top"])
        self.intermediate_size = int(spec["intermediate_size"])
        self.router = str(spec.get("router", "token_table"))
        self.activation = str(spec.get("activation", "clamped_glu"))
        if self.router not in self.ROUTERS:
            raise ValueError(f"unknown router {self.router!r}; known: {self.ROUTERS}")
        if self.activation not in self.ACTIVATIONS:
            raise ValueError(f"unknown expert activation {self.activation!r}; known: {self.ACTIVATIONS}")
        if not 1 <= self.top <= self.num_experts:
            raise ValueError(f"{self.top} of {self.num_experts} experts a token")
        self.learned = self.router == "sigmoid_topk"
        self.weight_on = str(spec.get("weight_on", "input" if self.learned else "output"))
        if self.weight_on != ("input" if self.learned else "output"):
            raise ValueError(f"router {self.router!r} with its weights on the experts' {self.weight_on}s is not built")
        self.vocab_size = 0 if self.learned else int(spec["vocab_size"])
        self.plain_glu = self.activation == "silu_glu"
        self.limit = 0.0 if self.plain_glu else float(spec["limit"])
        self.alpha = float(spec.get("alpha", 1.702))
        shared = spec.get("shared")
        self.shared = None if shared is None else {
            "intermediate_size": int(shared["intermediate_size"]), "limit": float(shared["limit"]),
            "alpha": float(shared.get("alpha", self.alpha))}
        self.names = tensor_names(self.NAMES, spec.get("names"))
        self.table = self.w_router = self.w_gate_up = self.w_down = self.shared_gate_up = self.shared_down = None

    # ---- weights -----------------------------------------------------
    def _expert_names(self, prefix: str, e: Optional[int]) -> dict:
        base = f"{prefix}.{self.names['shared']}" if e is None else f"{prefix}.{self.names['expert'].format(e)}"
        return {role: f"{base}.{self.names[role]}" for role in ("gate", "up", "down")}

    def param_specs(self, prefix: str) -> list[ParamSpec]:
        H, I = self.hidden_size, self.intermediate_size
        specs = []
        for e in range(self.num_experts):
            at = self._expert_names(prefix, e)
            specs += [ParamSpec(at["gate"], (I, H)), ParamSpec(at["up"], (I, H)), ParamSpec(at["down"], (H, I))]
        if self.learned:
            specs.append(ParamSpec(f"{prefix}.{self.names['router']}", (self.num_experts, H), init=("normal", 0.5)))
        else:
            specs.append(ParamSpec(f"{prefix}.{self.names['table']}", (self.vocab_size, self.top),
                                   init=("distinct", self.num_experts), integer=True))
        if self.shared is not None:
            at, S = self._expert_names(prefix, None), self.shared["intermediate_size"]
            specs += [ParamSpec(at["gate"], (S, H)), ParamSpec(at["up"], (S, H)), ParamSpec(at["down"], (H, S))]
        return specs

    def bind(self, tensors, prefix, device, dtype) -> None:
        def get(name):
            return tensors[name].to(device=device, dtype=dtype)

        ats = [self._expert_names(prefix, e) for e in range(self.num_experts)]
        # [experts, 2 I, H]: an expert's gates, then its ups; [experts, H, I]
        self.w_gate_up = torch.stack([torch.cat([get(at["gate"]), get(at["up"])], dim=0) for at in ats]).contiguous()
        self.w_down = torch.stack([get(at["down"]) for at in ats]).contiguous()
        if self.learned:
            self.w_router = get(f"{prefix}.{self.names['router']}").contiguous()
        else:
            self.table = tensors[f"{prefix}.{self.names['table']}"].to(device=device, dtype=torch.int32).contiguous()
        if self.shared is not None:
            at = self._expert_names(prefix, None)
            self.shared_gate_up = decode_weight(torch.cat([get(at["gate"]), get(at["up"])], dim=0).contiguous(),
                                                self.tiled_weights)
            self.shared_down = decode_weight(get(at["down"]).contiguous(), self.tiled_weights)

    # ---- run ---------------------------------------------------------
    def forward(self, x: torch.Tensor, step) -> torch.Tensor:
        n = x.shape[0]
        shared = None
        if self.shared is not None:
            # products of few rows stay unreduced K slices; the kernels that take them add them up
            act = ops.clamped_glu(linear(x, self.shared_gate_up, sliced_ok=True), self.shared["limit"],
                                  self.shared["alpha"])
            shared = linear(act, self.shared_down, sliced_ok=True)
        tile, mfma = ops.moe_plan(x.dtype, n * self.top, self.hidden_size, self.intermediate_size)
        if self.learned:
            # 32-bit logits from the activations as they are; the token's row stands for its id in the routing
            logits = linear(x, self.w_router, out_dtype=torch.float32)
            chosen, weights = ops.moe_topk(logits, self.top)
            rows = torch.arange(n, dtype=torch.int32, device=x.device)
            slot_of, row_token, tile_group = ops.moe_route(rows, n, chosen, self.num_experts, tile)
            # a choice's weight multiplies the expert's input: the sorted rows are made scaled
            x, row_token, combine = ops.moe_scale_rows(x, slot_of, weights, self.top, row_token.numel()), None, 1.0
        else:
            slot_of, row_token, tile_group = ops.moe_route(step.token_ids, n, self.table, self.num_experts, tile)
            combine = 1.0 / self.top
        if mfma:  # bf16: the product of gates and ups applies the activation itself
            act = ops.gemm_experts(x, self.w_gate_up, tile_group, row_index=row_token, tile=tile, mfma=True,
                                   glu="silu" if self.plain_glu else (self.limit, self.alpha))
        else:
            gate_up = ops.gemm_experts(x, self.w_gate_up, tile_group, row_index=row_token, tile=tile)
            act = (ops.gated_act(gate_up, "silu") if self.plain_glu
                   else ops.clamped_glu(gate_up, self.limit, self.alpha))
        y = ops.gemm_experts(act, self.w_down, tile_group, tile=tile, mfma=mfma)
        return ops.moe_combine(y, slot_of, self.top, combine, n, shared)


FEED_FORWARDS.register("routed_experts", RoutedExperts)
