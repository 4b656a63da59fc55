"""The Dafalix decoder as a ``ModelSpec``.

What the design fixes (not read from config.json):
  * the embedding is the token's vector as stored; the head is the embedding table; the model's norm and every
    layer's norms are layer norms with weight and bias;
  * the residual stream is kept in ``streams`` copies that learned weights mix (hyper-connections), 32-bit:
    for sublayer q, u = sum_s in_q[s] x_s, y = sublayer(norm_q(u)), x_t <- sum_s mix_q[s, t] x_s +
    residual_mult * out_q[t] * (ls_q * y) with one learned number a channel ls_q; the final norm reads sum_s x_s;
  * a stretch of layers (``loop``) runs several times in a row with the same weights, each pass with keys and
    states of its own;
  * mixer ``mlstm``: a matrix memory with capped log gates and a running maximum that starts at 0, an output norm
    per head without a weight, then a weight over all heads, a sigmoid gate and the output projection;
  * mixer ``parallel``: two mixers on the same input, weighted by ``left_scale`` and ``right_scale``.  Left:
    grouped-query attention over a sliding window, values of their own size, an RMS norm with a plain weight that
    the heads share on queries and keys before the rotation, a rotation of the first ``rot.dims`` dimensions of a
    head in halves with frequencies base^(-2i/dims) / factor, ordinary softmax.  Right: a recurrent block around
    a gated linear recurrent unit with a biased short convolution and block-diagonal gates;
  * the feed-forward is a mixture of experts with a learned router: sigmoid scores, the ``top`` largest chosen,
    not renormalized, a choice's score multiplying the expert's input; an expert is gated with silu, no biases.
Tensor names: ``embed``, ``l<i>.norm1`` / ``norm2`` (biases ``.b``), ``l<i>.ls1`` / ``ls2``, ``l<i>.hc1.*`` /
``hc2.*`` (``in``, ``out``, ``mix``), ``l<i>.mix.*`` (``mix.left.*`` and ``mix.right.*`` in a parallel layer),
``l<i>.mlp.router`` and ``l<i>.mlp.e<j>.gate`` / ``up`` / ``down``, ``final.norm``; weights have no suffix, biases
end in ``.b``.
"""

from __future__ import annotations

from ..config.dafalix import ARCHITECTURE, MAX_CONTEXT, DafalixConfig
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
from .registry import Architecture, register_architecture

DIVISOR_EPS = 1e-6  # what the matrix memory's divisor is raised by
RECURRENCE_RATE = 8.0  # log a = -rate * r * softplus(lam)


def _memory(m, eps: float) -> PartSpec:
    return PartSpec("matrix_memory", {"heads": m.heads, "dim": m.dim, "vdim": m.vdim, "gate_cap": m.gate_cap,
                                      "eps": eps, "divisor_eps": DIVISOR_EPS})


def _window_attention(a, eps: float) -> PartSpec:
    names = {"q": "mix.left.q", "k": "mix.left.k", "v": "mix.left.v", "o": "mix.left.o",
             "q_norm": "mix.left.q.norm", "k_norm": "mix.left.k.norm"}
    return PartSpec("attention", {
        "num_heads": a.heads, "num_kv_heads": a.kv_heads, "head_dim": a.dim, "value_dim": a.vdim, "scale": a.scale,
        "window": a.window, "qk_norm": {"eps": eps},
        "position": PartSpec("rope", {"theta": a.rot_base, "factor": a.rot_factor, "rotary_dim": a.rot_dims,
                                      "exponent_over": "rotary_dim", "pairing": "rotary_half"})
        if a.rot_dims else PartSpec("none"),
        "names": names, "weight_suffix": "", "bias_suffix": ".b", "norm_suffix": "",
    })


def _recurrence(s) -> PartSpec:
    names = {"y": "y", "y_bias": "y.b", "x": "x", "x_bias": "x.b", "conv": "conv", "conv_bias": "conv.b", "ra": "ra",
             "ra_bias": "ra.b", "ri": "ri", "ri_bias": "ri.b", "lam": "lam", "o": "o"}
    return PartSpec("gated_linear_recurrence", {
        "width": s.width, "blocks": s.blocks, "conv": s.conv, "rate": RECURRENCE_RATE,
        "names": {role: f"mix.right.{name}" for role, name in names.items()},
    })


def build_spec(cfg: DafalixConfig) -> ModelSpec:
    eps = cfg.norm_eps
    norm = PartSpec("layernorm", {"eps": eps, "suffix": "", "bias_suffix": ".b"})
    block = PartSpec("streams", {"streams": cfg.streams, "residual_mult": cfg.residual_mult,
                                 "norm_names": ("norm1", "norm2"), "connection_names": ("hc1", "hc2"),
                                 "layer_scale": ("ls1", "ls2")})
    layers = []
    for i, layer in enumerate(cfg.layers):
        if layer.type == "mlstm":
            mixer = _memory(layer.mixer, eps)
        else:
            m = layer.mixer
            mixer = PartSpec("side_by_side", {"members": [
                {"mixer": _window_attention(m.left, eps), "scale": m.left_scale},
                {"mixer": _recurrence(m.right), "scale": m.right_scale},
            ]})
        if layer.mlp is None:
            ff = PartSpec("none")
        else:
            ff = PartSpec("routed_experts", {
                "experts": layer.mlp.experts, "top": layer.mlp.top, "intermediate_size": layer.mlp.ff,
                "router": "sigmoid_topk", "weight_on": "input", "activation": "silu_glu",
                "names": {"expert": "mlp.e{}", "router": "mlp.router"},
            })
        layers.append(LayerSpec(prefix=f"l{i}", block=block, mixer=mixer, feed_forward=ff, norm=norm))
    return ModelSpec(
        architecture=cfg.architecture,
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        max_position=MAX_CONTEXT,
        embedding=PartSpec("scaled_embedding", {"scale": 1.0, "name": "embed", "suffix": ""}),
        layers=tuple(layers),
        schedule=tuple(ScheduleEntry(layer, copy=copy) for layer, copy in cfg.layer_runs()),
        final_norm=norm,
        head=PartSpec("lm_head", {"tied": True}),
        prefix="",
        final_norm_name="final.norm",
        residual_float32=True,
    )


register_architecture(Architecture(
    name=ARCHITECTURE,
    read_config=DafalixConfig.from_dict,
    build_spec=build_spec,
    write_config=DafalixConfig.to_dict,
))
