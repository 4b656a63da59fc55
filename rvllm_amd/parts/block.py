"""Arrangements of norm, mixer, feed-forward and residual sum in a layer.

``sandwich``: a norm before and after each branch; the normed branch output
is added to the residual stream
(v3/crates/rvllm-loader/src/metal_host.rs:501,606-628; the order of launches:
v3/crates/rvllm-runtime/src/gemma4_layer_exec.rs:1-28):

    x = x + post_attention_layernorm(mixer(input_layernorm(x)))
    x = x + post_feedforward_layernorm(ff(pre_feedforward_layernorm(x)))

A block may hand the next block its entry norm already applied (``then``),
which lets the kernel that adds the feed-forward branch also write the next
layer's normed input.  Parameters of ``sandwich``: ``norm_names`` (the four
norms' names under the layer's prefix, the Gemma names if absent) and
``layer_scale`` = (name, name) or None: one learned number a channel that the
normed mixer branch, and one that the normed feed-forward branch, is multiplied
by before it is added (x = x + ls1 * norm(mixer(..))).  A layer whose
feed-forward is ``none`` has the first sublayer only and asks for the first two
norms only.  The residual stream may be 32-bit under bf16 activations
(``ModelSpec.residual_float32``); the norms then read the one and write the other.

``parallel``: one norm, both branches read its output, and their sum is added
with a multiplier; the residual stream is 32-bit whatever the activations' type:

    h = norm(x);  X = x + residual_mult * (mixer(h) + ff(h))

With ``depth_average`` = {"name", "terms", "slots"} what goes on to the next
layer is a learned average over depth, x = sum_j w[j] * X_j over the first
``terms`` of: the first layer's input and every layer's X so far (``slots`` in
all; the tensor ``<layer>.<name>`` holds the ``terms`` weights).  The X_j of a
step live in ``step.shared`` and end with it.

``streams``: the residual stream is kept in S copies x_1 .. x_S (32-bit, all equal to the embedding's output at the
first layer) that learned weights mix; there is no plain residual sum.  For sublayer q (1: the mixer, 2: the
feed-forward) with the layer's tensors ``<hc_q>.in [S]``, ``<hc_q>.out [S]``, ``<hc_q>.mix [S, S]`` (from, to):

    u = sum_s in[s] x_s;   y = sublayer(norm_q(u));   x_t <- sum_s mix[s, t] x_s + mult * out[t] * (ls_q * y)

all streams at once from the old ones.  After the last layer the stream handed to the final norm is sum_s x_s.
Parameters: ``streams``, ``residual_mult``, ``norm_names`` (two), ``connection_names`` (two, ``hc1`` / ``hc2`` if
absent), ``layer_scale`` = (name, name) or None.  The streams of a step live in ``step.shared`` and end with it; one
kernel a sublayer moves them on and writes the next sublayer's normed input.
"""

from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops
from .base import Block, Norm, ParamSpec, tensor_path
from .norm import ScalarRMSNorm
from .registry import BLOCKS, FEED_FORWARDS, MIXERS, NORMS
from .spec import LayerSpec, PartSpec


class SandwichBlock(Block):
    NORM_NAMES = ("input_layernorm", "post_attention_layernorm", "pre_feedforward_layernorm",
                  "post_feedforward_layernorm")

    def __init__(self, spec: PartSpec, *, layer: LayerSpec, hidden_size: int):
        self.hidden_size = hidden_size
        self.mixer = MIXERS.build(layer.mixer, hidden_size=hidden_size)
        self.feed_forward = FEED_FORWARDS.build(layer.feed_forward, hidden_size=hidden_size)
        self.has_feed_forward = layer.feed_forward.kind != "none"
        names = tuple(spec.get("norm_names") or self.NORM_NAMES)
        if len(names) != 4:
            raise ValueError("a sandwich has four norms: before and after the mixer, before and after the feed-forward")
        if not self.has_feed_forward:
            names = names[:2]
        self.norms = [NORMS.build(layer.norm, width=hidden_size, name=name) for name in names]
        self.norm_in, self.norm_post_mixer = self.norms[:2]
        self.norm_pre_ff, self.norm_post_ff = self.norms[2:] if self.has_feed_forward else (None, None)
        scale_names = spec.get("layer_scale")
        self.scale_names = None if scale_names is None else tuple(str(n) for n in scale_names)
        if self.scale_names is not None and len(self.scale_names) != 2:
            raise ValueError("layer_scale names two tensors: the mixer branch's and the feed-forward branch's")
        self.scale_mixer: Optional[torch.Tensor] = None
        self.scale_ff: Optional[torch.Tensor] = None

    def parts(self):
        return (self.mixer, self.feed_forward, *self.norms)

    def param_specs(self, prefix: str) -> list[ParamSpec]:
        specs = [s for part in self.parts() for s in part.param_specs(prefix)]
        if self.scale_names is not None:
            used = self.scale_names if self.has_feed_forward else self.scale_names[:1]
            specs += [ParamSpec(tensor_path(prefix, name), (self.hidden_size,), init=("normal_about", 1.0, 0.1))
                      for name in used]
        return specs

    def bind(self, tensors, prefix, device, dtype) -> None:
        for part in self.parts():
            part.bind(tensors, prefix, device, dtype)
        if self.scale_names is not None:  # applied in 32-bit with the norm
            self.scale_mixer = tensors[tensor_path(prefix, self.scale_names[0])].to(
                device=device, dtype=torch.float32).contiguous()
            if self.has_feed_forward:
                self.scale_ff = tensors[tensor_path(prefix, self.scale_names[1])].to(
                    device=device, dtype=torch.float32).contiguous()

    def entry_norm(self) -> Optional[Norm]:
        return self.norm_in

    @staticmethod
    def _add(norm: Norm, branch, x, then, scale):
        if scale is None:
            return norm.add_into(branch, x, then=then)
        return norm.add_into(branch, x, then=then, scale=scale)

    def forward(self, x: torch.Tensor, step, cache, entered: Optional[torch.Tensor] = None,
                then: Optional[Norm] = None) -> Optional[torch.Tensor]:
        h = entered if entered is not None else self.norm_in.forward(x)
        a = self.mixer.forward(h, step, cache)
        if not self.has_feed_forward:
            return self._add(self.norm_post_mixer, a, x, then, self.scale_mixer)
        h = self._add(self.norm_post_mixer, a, x, self.norm_pre_ff, self.scale_mixer)
        f = self.feed_forward.forward(h, step)
        return self._add(self.norm_post_ff, f, x, then, self.scale_ff)


class ParallelBlock(Block):
    HISTORY = "parallel_block.depth_history"  # key in step.shared: (the X_j, how many are written)

    def __init__(self, spec: PartSpec, *, layer: LayerSpec, hidden_size: int):
        self.hidden_size = hidden_size
        self.residual_mult = float(spec.get("residual_mult", 1.0))
        self.norm_name = str(spec.get("norm_name", "norm"))
        depth = spec.get("depth_average")
        self.depth = None if depth is None else {"name": str(depth["name"]), "terms": int(depth["terms"]),
                                                 "slots": int(depth["slots"])}
        if self.depth is not None and not 2 <= self.depth["terms"] <= self.depth["slots"]:
            raise ValueError(f"a depth average over {self.depth['terms']} of {self.depth['slots']} streams")
        self.mixer = MIXERS.build(layer.mixer, hidden_size=hidden_size)
        self.feed_forward = FEED_FORWARDS.build(layer.feed_forward, hidden_size=hidden_size)
        self.norm = NORMS.build(layer.norm, width=hidden_size, name=self.norm_name)
        self.depth_weights: Optional[torch.Tensor] = None

    def parts(self):
        return (self.mixer, self.feed_forward, self.norm)

    def param_specs(self, prefix: str) -> list[ParamSpec]:
        specs = [s for part in self.parts() for s in part.param_specs(prefix)]
        if self.depth is not None:
            specs.append(ParamSpec(tensor_path(prefix, self.depth["name"]), (self.depth["terms"],),
                                   init=("normal_about", 1.0 / self.depth["terms"], 0.05)))
        return specs

    def bind(self, tensors, prefix, device, dtype) -> None:
        for part in self.parts():
            part.bind(tensors, prefix, device, dtype)
        if self.depth is not None:  # averaged in 32-bit
            self.depth_weights = tensors[tensor_path(prefix, self.depth["name"])].to(
                device=device, dtype=torch.float32).contiguous()

    def entry_norm(self) -> Optional[Norm]:
        return self.norm

    def forward(self, x: torch.Tensor, step, cache, entered: Optional[torch.Tensor] = None,
                then: Optional[Norm] = None) -> Optional[torch.Tensor]:
        h = entered if entered is not None else self.norm.forward(x)
        a = self.mixer.forward(h, step, cache)
        f = self.feed_forward.forward(h, step)
        history, terms, seed = None, 0, False
        if self.depth is not None:
            terms = self.depth["terms"]
            kept = step.shared.get(self.HISTORY)
            if kept is None:  # the first layer of the step: its input is the first of the streams
                kept = [torch.empty((self.depth["slots"], *x.shape), dtype=torch.float32, device=x.device), 1]
                step.shared[self.HISTORY] = kept
                seed = True
            history = kept[0]
            if kept[1] != terms - 1:
                raise ValueError(f"a depth average over {terms} streams, but the step has written {kept[1]}")
            kept[1] = terms
        fused = isinstance(then, ScalarRMSNorm)
        nxt = ops.residual_mix(x, a, f, self.residual_mult, history, terms, self.depth_weights, seed,
                               then.gain if fused else None, then.eps if fused else 0.0,
                               then.out_dtype if fused else None)
        if then is not None and not fused:
            return then.forward(x)
        return nxt


class StreamsInput(Norm):
    """What a ``streams`` block applies to the streams first: the weighted sum of the copies, then its first norm.
    The block before gets it as ``then`` and lets the kernel that moves the streams on write this block's input."""

    def __init__(self, norm: Norm):
        self.norm = norm
        self.weights: Optional[torch.Tensor] = None  # [S], the block's, set when it binds

    def forward(self, x: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        raise ValueError("the input of a streams block is made from the streams, not from one residual stream")


class StreamsBlock(Block):
    STREAMS = "streams_block.streams"  # key in step.shared: the step's [S, tokens, width]

    def __init__(self, spec: PartSpec, *, layer: LayerSpec, hidden_size: int):
        self.hidden_size = hidden_size
        self.num_streams = int(spec["streams"])
        if self.num_streams < 1:
            raise ValueError("a residual stream is kept in one copy at least")
        self.residual_mult = float(spec.get("residual_mult", 1.0))
        self.mixer = MIXERS.build(layer.mixer, hidden_size=hidden_size)
        self.feed_forward = FEED_FORWARDS.build(layer.feed_forward, hidden_size=hidden_size)
        self.has_feed_forward = layer.feed_forward.kind != "none"
        count = 2 if self.has_feed_forward else 1
        names = tuple(spec.get("norm_names") or ("norm1", "norm2"))
        self.connection_names = tuple(str(n) for n in (spec.get("connection_names") or ("hc1", "hc2")))
        scale_names = spec.get("layer_scale")
        self.scale_names = None if scale_names is None else tuple(str(n) for n in scale_names)
        if len(names) != 2 or len(self.connection_names) != 2 or (self.scale_names and len(self.scale_names) != 2):
            raise ValueError("a streams block names two norms, two connections and two layer scales or none")
        self.norms = [NORMS.build(layer.norm, width=hidden_size, name=name) for name in names[:count]]
        self.connection_names = self.connection_names[:count]
        self.entry = StreamsInput(self.norms[0])
        self.w_in: list = [None] * count
        self.w_out: list = [None] * count
        self.w_mix: list = [None] * count
        self.scales: list = [None] * count

    def parts(self):
        return (self.mixer, self.feed_forward, *self.norms)

    def param_specs(self, prefix: str) -> list[ParamSpec]:
        S = self.num_streams
        specs = [s for part in self.parts() for s in part.param_specs(prefix)]
        for name in self.connection_names:
            at = tensor_path(prefix, name)
            specs += [ParamSpec(f"{at}.in", (S,), init=("normal_about", 1.0 / S, 0.1)),
                      ParamSpec(f"{at}.out", (S,), init=("normal_about", 1.0, 0.2)),
                      ParamSpec(f"{at}.mix", (S, S), init=("normal_about", 1.0 / S, 0.2))]
        if self.scale_names is not None:
            specs += [ParamSpec(tensor_path(prefix, name), (self.hidden_size,), init=("normal_about", 1.0, 0.1))
                      for name in self.scale_names[:len(self.norms)]]
        return specs

    def bind(self, tensors, prefix, device, dtype) -> None:
        for part in self.parts():
            part.bind(tensors, prefix, device, dtype)

        def f32(name):  # the streams are mixed in 32-bit
            return tensors[name].to(device=device, dtype=torch.float32).contiguous()

        for q, name in enumerate(self.connection_names):
            at = tensor_path(prefix, name)
            self.w_in[q], self.w_out[q], self.w_mix[q] = f32(f"{at}.in"), f32(f"{at}.out"), f32(f"{at}.mix")
            if self.scale_names is not None:
                self.scales[q] = f32(tensor_path(prefix, self.scale_names[q]))
        self.entry.weights = self.w_in[0]
        self.out_dtype = dtype

    def entry_norm(self) -> Optional[Norm]:
        return self.entry

    def _move_on(self, q: int, branch, streams, x, then, in_w=None, norm=None):
        """Sublayer q's result joins the streams; returns the next sublayer's input, this block's (``in_w``,
        ``norm``) or the next block's (``then``), or None after writing the streams' sum into ``x``."""
        total = None
        if in_w is None and isinstance(then, StreamsInput) and then.weights is not None \
                and then.weights.shape[0] == self.num_streams:
            in_w, norm = then.weights, then.norm
        elif in_w is None:
            total = x  # the last block of the step, or a block of another kind follows
        nxt = ops.streams_update(
            streams, self.out_dtype, branch=branch, layer_scale=self.scales[q], mix=self.w_mix[q], out_w=self.w_out[q],
            mult=self.residual_mult, in_w=in_w, norm_w=None if norm is None else norm.weight,
            norm_b=None if norm is None else norm.bias, eps=0.0 if norm is None else norm.eps, total=total)
        if total is not None and then is not None:
            return then.forward(x)
        return nxt

    def forward(self, x: torch.Tensor, step, cache, entered: Optional[torch.Tensor] = None,
                then: Optional[Norm] = None) -> Optional[torch.Tensor]:
        for norm in self.norms:
            if not hasattr(norm, "bias"):
                raise ValueError("the kernel that moves the streams on applies a layer norm with weight and bias")
        streams = step.shared.get(self.STREAMS)
        if streams is None:  # the first layer of the step: every copy is the embedding's output
            if x.dtype != torch.float32:
                raise ValueError("the streams are 32-bit: the model keeps a 32-bit residual stream")
            streams = torch.empty((self.num_streams, *x.shape), dtype=torch.float32, device=x.device)
            step.shared[self.STREAMS] = streams
            entered = ops.streams_update(streams, self.out_dtype, seed=x, in_w=self.w_in[0],
                                         norm_w=self.norms[0].weight, norm_b=self.norms[0].bias, eps=self.norms[0].eps)
        elif entered is None:
            entered = ops.streams_update(streams, self.out_dtype, in_w=self.w_in[0], norm_w=self.norms[0].weight,
                                         norm_b=self.norms[0].bias, eps=self.norms[0].eps)
        a = self.mixer.forward(entered, step, cache)
        if not self.has_feed_forward:
            return self._move_on(0, a, streams, x, then)
        h = self._move_on(0, a, streams, x, then, in_w=self.w_in[1], norm=self.norms[1])
        f = self.feed_forward.forward(h, step)
        return self._move_on(1, f, streams, x, then)


BLOCKS.register("sandwich", SandwichBlock)
BLOCKS.register("streams", StreamsBlock)
BLOCKS.register("parallel", ParallelBlock)
