"""Small Dafalix configurations for the tests.  They differ from one another in every size and constant, and use
what a given checkpoint may happen to make equal or 1.

A  four layers, a matrix memory first; the middle two run twice; three streams; experts with two choices of five and
   one of four, layers without a feed-forward; attention heads of 32 with values of 16 and a window of 21, a rotation
   of 16 of 32 dimensions with scaled frequencies, and heads of 16 rotated whole with values of 32; recurrent units in
   three blocks and in one
B  widths that are no multiple of 8, one stream, no loop; a window of 1 (a token sees itself only) without rotation,
   one key/value head a query head; a recurrent unit whose blocks are single channels with a convolution of one tap
   (no state) and one of five taps; all experts chosen; a matrix memory of one head; scales that are negative or 1
C  layers wide enough for long sequences: four streams, the first two layers twice, windows of 100 and 64 that end
   inside pages, no rotation in one layer, four of sixteen experts
"""

from __future__ import annotations

import json
from pathlib import Path

import torch


def _memory(heads, dim, vdim, cap, mlp=None):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}, "mlp": mlp}


def _parallel(left, right, left_scale, right_scale, mlp=None):
    return {"type": "parallel", "mlp": mlp,
            "mixer": {"left": left, "right": right, "left_scale": left_scale, "right_scale": right_scale}}


def _left(heads, kv_heads, dim, vdim, scale, window, dims, base, factor):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "mask": {"size": window},
            "rot": {"dims": dims, "base": base, "scaling": {"factor": factor}}}


def _right(width, blocks, conv):
    return {"width": width, "blocks": blocks, "conv": conv}


def _moe(ff, experts, top):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


CONFIG_A = {
    "architecture": "Dafalix", "vocab": 211, "width": 64, "norm": {"eps": 1e-5}, "residual_mult": 0.7, "streams": 3,
    "loop": {"start": 1, "stop": 3, "times": 2},
    "layers": [
        _memory(2, 16, 24, 10.0, _moe(32, 5, 2)),
        _parallel(_left(4, 2, 32, 16, 0.2, 21, 16, 10000.0, 4.0), _right(48, 3, 3), 0.7, 1.3, _moe(40, 4, 1)),
        _memory(3, 8, 8, 15.0),
        _parallel(_left(6, 1, 16, 32, 0.3, 5, 16, 500.0, 1.0), _right(80, 1, 4), 1.1, 0.6),
    ],
}

CONFIG_B = {
    "architecture": "Dafalix", "vocab": 97, "width": 100, "norm": {"eps": 1e-6}, "residual_mult": 1.0, "streams": 1,
    "layers": [
        _parallel(_left(3, 3, 20, 20, 0.25, 1, 0, 100.0, 1.0), _right(36, 36, 1), -0.8, 1.0, _moe(50, 3, 3)),
        _memory(1, 40, 36, 5.0, _moe(44, 7, 2)),
        _parallel(_left(5, 1, 12, 28, 0.4, 7, 6, 37.5, 2.5), _right(50, 5, 5), 1.0, 0.45),
        _memory(5, 12, 20, 20.0),
    ],
}

CONFIG_C = {
    "architecture": "Dafalix", "vocab": 1500, "width": 256, "norm": {"eps": 1e-6}, "residual_mult": 0.4, "streams": 4,
    "loop": {"start": 0, "stop": 2, "times": 2},
    "layers": [
        _parallel(_left(8, 2, 64, 64, 0.125, 100, 32, 1000000.0, 8.0), _right(384, 6, 4), 1.2, 0.9, _moe(128, 8, 2)),
        _memory(4, 64, 64, 15.0),
        _parallel(_left(4, 4, 48, 80, 0.15, 64, 0, 10000.0, 1.0), _right(256, 8, 2), 0.8, 1.0, _moe(96, 16, 4)),
    ],
}

CONFIGS = {"A": (CONFIG_A, 31), "B": (CONFIG_B, 32), "C": (CONFIG_C, 33)}


def write_model(folder, name: str, seed=None, loud: bool = False) -> Path:
    """Writes configuration ``name`` with random weights through the framework's random-weights mode, then rescales
    them so that every part matters: a matrix keeps its input's size (rows of variance 1 / inputs), the embedding
    is of order one, norm weights and layer scales lie about one, the recurrent units decay slowly, the routers'
    logits stay where a sigmoid tells them apart in 32-bit.
    ``loud``: the weights of the query and key norms are scaled up so that a softmax hangs on single keys, so that a
    key just inside or just outside a window shows in the logits."""
    from safetensors.torch import load_file

    from rvllm_amd.models.registry import architecture_of
    from rvllm_amd.weights.random_init import write_random_model
    from rvllm_amd.weights.safetensors_io import write_safetensors

    doc, default_seed = CONFIGS[name]
    config = architecture_of(doc).read_config(doc, f"tiny config {name}")
    out = write_random_model(Path(folder), config, default_seed if seed is None else seed, torch.bfloat16)
    (out / "config.json").write_text(json.dumps(doc, indent=2))
    tensors = load_file(str(out / "model.safetensors"))
    for key, t in list(tensors.items()):
        x = t.float()
        last = key.split(".")[-1]
        if key == "embed":
            x = x * 50.0
        elif key.endswith((".q.norm", ".k.norm")):
            x = (1.0 + x * 2.0) * (2.5 if loud else 1.0)  # written about zero with a deviation of 0.1
        elif key.endswith(".right.lam"):
            x = x - 3.0  # decays near one, as trained units have them
        elif last == "router":
            x = x * (4.0 / x.shape[1] ** 0.5)  # written with a deviation of 0.5: logits of a deviation of two
        elif last in ("ra", "ri"):
            x = x * (10.0 / x.shape[-1] ** 0.5)  # written with a deviation of 0.1
        elif x.dim() == 2 and last not in ("conv", "mix"):
            x = x * (50.0 / x.shape[1] ** 0.5)
        tensors[key] = x.to(torch.bfloat16)
    write_safetensors(out / "model.safetensors", tensors, metadata={"format": "pt"})
    return out
