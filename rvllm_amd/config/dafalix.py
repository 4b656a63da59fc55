"""Typed configuration of the Dafalix decoder, read from config.json.

The file gives every size and every constant that differs between models of
the design:

    architecture       "Dafalix"
    vocab, width
    norm.eps           of every norm (the layer norms and the per-head RMS norms)
    residual_mult      what a sublayer's result is multiplied by before it joins the streams
    streams            how many copies of the residual stream the hyper-connections keep
    loop               {start, stop, times}: layers start .. stop-1 run `times` times in a row with the same
                       weights, each pass with a cache of its own (absent: every layer once)
    layers[i]          type ("mlstm" or "parallel"), mixer (its sizes), mlp (null: none; kind "moe")
      mlstm            heads, dim, vdim, gate_cap
      parallel         left {heads, kv_heads, dim, vdim, scale, mask.size, rot.dims, rot.base, rot.scaling.factor},
                       left_scale, right {width, blocks, conv}, right_scale
      mlp              kind "moe", expert.ff, router.experts, router.top

What the design fixes is stated in ``models/dafalix.py``.  As with the other
readers, every problem of a file is reported in one ``ConfigError``.
"""

from __future__ import annotations

import dataclasses
from typing import Any, Optional, Union

from .errors import ConfigError
from .fields import FieldReader

ARCHITECTURE = "Dafalix"
MAX_LAYERS = 1024
MAX_WIDTH = 1 << 20
MAX_VOCAB = 1 << 22
MAX_CONTEXT = 1 << 20  # the design has no table of positions; a request is held to this many tokens
MAX_TAPS = 16
MAX_STREAMS = 8
MAX_EXPERTS = 1024
MIXER_TYPES = ("mlstm", "parallel")
MLP_KINDS = ("moe",)


@dataclasses.dataclass(frozen=True)
class MatrixMemorySizes:
    heads: int
    dim: int
    vdim: int
    gate_cap: float


@dataclasses.dataclass(frozen=True)
class WindowAttentionSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int        # mask.size: a token sees itself and the window - 1 before it
    rot_dims: int      # rot.dims
    rot_base: float    # rot.base
    rot_factor: float  # rot.scaling.factor: every frequency is divided by it


@dataclasses.dataclass(frozen=True)
class RecurrentUnitSizes:
    width: int
    blocks: int
    conv: int


@dataclasses.dataclass(frozen=True)
class ParallelSizes:
    left: WindowAttentionSizes
    right: RecurrentUnitSizes
    left_scale: float
    right_scale: float


@dataclasses.dataclass(frozen=True)
class ExpertsMlp:
    ff: int
    experts: int
    top: int
    kind: str = "moe"


@dataclasses.dataclass(frozen=True)
class Loop:
    start: int
    stop: int
    times: int


@dataclasses.dataclass(frozen=True)
class DafalixLayer:
    type: str
    mixer: Union[MatrixMemorySizes, ParallelSizes]
    mlp: Optional[ExpertsMlp]


@dataclasses.dataclass(frozen=True)
class DafalixConfig:
    vocab: int
    width: int
    norm_eps: float
    residual_mult: float
    streams: int
    loop: Optional[Loop]
    layers: tuple[DafalixLayer, ...]
    architecture: str = ARCHITECTURE

    def layer_runs(self) -> list[tuple[int, int]]:
        """(layer, pass) in the order the layers run."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, 0) for i in range(n)]
        lo, hi = self.loop.start, self.loop.stop
        runs = [(i, 0) for i in range(lo)]
        for p in range(self.loop.times):
            runs += [(i, p) for i in range(lo, hi)]
        return runs + [(i, 0) for i in range(hi, n)]

    @classmethod
    def from_dict(cls, doc: dict, source: str = "config.json") -> "DafalixConfig":
        r = FieldReader(doc)
        problems = r.problems
        vocab = r.integer("vocab", lo=1, hi=MAX_VOCAB)
        width = r.integer("width", lo=1, hi=MAX_WIDTH)
        mult = r.real("residual_mult")
        streams = r.integer("streams", lo=1, hi=MAX_STREAMS)
        eps = _sub(doc, "norm", problems, lambda f: f.real("eps", positive=True), 1.0)
        raw_layers = r.raw("layers")
        layers = []
        if not isinstance(raw_layers, list) or not raw_layers:
            problems.append("missing or invalid required list layers")
        elif len(raw_layers) > MAX_LAYERS:
            problems.append(f"{len(raw_layers)} layers, at most {MAX_LAYERS}")
        else:
            for i, entry in enumerate(raw_layers):
                layer, found = _read_layer(entry)
                problems += [f"layers[{i}]: {p}" for p in found]
                layers.append(layer)
        loop = None
        if doc.get("loop") is not None:
            loop = _sub(doc, "loop", problems, lambda f: Loop(f.integer("start", lo=0, hi=MAX_LAYERS),
                                                              f.integer("stop", lo=0, hi=MAX_LAYERS),
                                                              f.integer("times", lo=1, hi=MAX_LAYERS)), None)
            if loop is not None and layers and not loop.start <= loop.stop <= len(layers):
                problems.append(f"loop: start={loop.start} .. stop={loop.stop} must lie within the {len(layers)} layers")
        if problems:
            raise ConfigError(source, problems)
        return cls(vocab, width, eps, mult, streams, loop, tuple(layers))

    def to_dict(self) -> dict:
        layers = []
        for layer in self.layers:
            m = layer.mixer
            if layer.type == "mlstm":
                mixer: Any = dataclasses.asdict(m)
            else:
                a, s = m.left, m.right
                mixer = {"left": {"heads": a.heads, "kv_heads": a.kv_heads, "dim": a.dim, "vdim": a.vdim,
                                  "scale": a.scale, "mask": {"size": a.window},
                                  "rot": {"dims": a.rot_dims, "base": a.rot_base,
                                          "scaling": {"factor": a.rot_factor}}},
                         "left_scale": m.left_scale, "right": dataclasses.asdict(s), "right_scale": m.right_scale}
            mlp = None if layer.mlp is None else {"kind": layer.mlp.kind, "expert": {"ff": layer.mlp.ff},
                                                  "router": {"experts": layer.mlp.experts, "top": layer.mlp.top}}
            layers.append({"type": layer.type, "mixer": mixer, "mlp": mlp})
        doc = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
               "norm": {"eps": self.norm_eps}, "residual_mult": self.residual_mult, "streams": self.streams,
               "layers": layers}
        if self.loop is not None:
            doc["loop"] = dataclasses.asdict(self.loop)
        return doc


def _sub(doc: dict, key: str, problems: list, read, fallback):
    """``read(FieldReader(doc[key]))``, with the sub-object's problems filed under its key."""
    obj = doc.get(key)
    if not isinstance(obj, dict):
        problems.append(f"missing or invalid required object {key}")
        return fallback
    f = FieldReader(obj)
    value = read(f)
    problems += [f"{key}: {p}" for p in f.problems]
    return fallback if f.problems else value


def _read_matrix_memory(obj: dict, problems: list) -> MatrixMemorySizes:
    m = FieldReader(obj)
    sizes = MatrixMemorySizes(m.integer("heads", lo=1, hi=4096), m.integer("dim", lo=1, hi=1024),
                              m.integer("vdim", lo=1, hi=4096), m.real("gate_cap", positive=True))
    problems += [f"mixer: {p}" for p in m.problems]
    return sizes


def _read_left(raw: dict) -> tuple[Optional[WindowAttentionSizes], list]:
    a = FieldReader(raw)
    heads, kv_heads = a.integer("heads", lo=1, hi=4096), a.integer("kv_heads", lo=1, hi=4096)
    dim, vdim = a.integer("dim", lo=1, hi=512), a.integer("vdim", lo=1, hi=512)
    scale = a.real("scale", positive=True)
    found = list(a.problems)
    window = _sub(raw, "mask", found, lambda f: f.integer("size", lo=1, hi=MAX_CONTEXT), 1)
    dims, base, factor = 0, 1.0, 1.0
    rot = raw.get("rot")
    if not isinstance(rot, dict):
        found.append("missing or invalid required object rot")
    else:
        f = FieldReader(rot)
        dims, base = f.integer("dims", lo=0, hi=512), f.real("base", positive=True)
        sub = [f"rot: {p}" for p in f.problems]
        if rot.get("scaling") is not None:  # absent: the frequencies are left as they are
            factor = _sub(rot, "scaling", sub, lambda g: g.real("factor", positive=True), 1.0)
            sub = [p if p.startswith("rot: ") else f"rot: {p}" for p in sub]
        found += sub
    if not found:
        if heads % kv_heads:
            found.append(f"heads={heads} must be a multiple of kv_heads={kv_heads}")
        if dims % 2 or dims > dim:
            found.append(f"rot.dims={dims} must be even and at most dim={dim}")
    if found:
        return None, found
    return WindowAttentionSizes(heads, kv_heads, dim, vdim, scale, window, dims, base, factor), []


def _read_parallel(obj: dict, problems: list) -> Optional[ParallelSizes]:
    m = FieldReader(obj)
    left_scale, right_scale = m.real("left_scale"), m.real("right_scale")
    found = list(m.problems)
    left = right = None
    raw_left = obj.get("left")
    if not isinstance(raw_left, dict):
        found.append("missing or invalid required object left")
    else:
        left, bad = _read_left(raw_left)
        found += [f"left: {p}" for p in bad]
    raw_right = obj.get("right")
    if not isinstance(raw_right, dict):
        found.append("missing or invalid required object right")
    else:
        s = FieldReader(raw_right)
        right = RecurrentUnitSizes(s.integer("width", lo=1, hi=MAX_WIDTH), s.integer("blocks", lo=1, hi=MAX_WIDTH),
                                   s.integer("conv", lo=1, hi=MAX_TAPS))
        if not s.problems and right.width % right.blocks:
            s.problem(f"width={right.width} must be a multiple of blocks={right.blocks}")
        found += [f"right: {p}" for p in s.problems]
    problems += [f"mixer: {p}" for p in found]
    if found:
        return None
    return ParallelSizes(left, right, left_scale, right_scale)


def _read_mlp(raw: dict, problems: list) -> Optional[ExpertsMlp]:
    f = FieldReader(raw)
    kind = f.string("kind")
    found = list(f.problems)
    if kind and kind not in MLP_KINDS:
        found.append(f"unknown kind {kind!r}; known: {', '.join(MLP_KINDS)}")
    ff = _sub(raw, "expert", found, lambda g: g.integer("ff", lo=1, hi=MAX_WIDTH), 1)
    experts, top = 1, 1
    router = raw.get("router")
    if not isinstance(router, dict):
        found.append("missing or invalid required object router")
    else:
        g = FieldReader(router)
        experts, top = g.integer("experts", lo=1, hi=MAX_EXPERTS), g.integer("top", lo=1, hi=MAX_EXPERTS)
        if not g.problems and top > experts:
            g.problem(f"top={top} of experts={experts}")
        found += [f"router: {p}" for p in g.problems]
    problems += [f"mlp: {p}" for p in found]
    return None if found else ExpertsMlp(ff, experts, top)


def _read_layer(entry: Any) -> tuple[Optional[DafalixLayer], list]:
    problems: list = []
    if not isinstance(entry, dict):
        return None, ["must be an object"]
    r = FieldReader(entry)
    kind = r.string("type")
    if kind and kind not in MIXER_TYPES:
        r.problem(f"unknown mixer type {kind!r}; known: {', '.join(MIXER_TYPES)}")
    mixer = None
    raw_mixer = r.raw("mixer")
    if not isinstance(raw_mixer, dict):
        r.problem("missing or invalid required object mixer")
    elif kind == "mlstm":
        mixer = _read_matrix_memory(raw_mixer, problems)
    elif kind == "parallel":
        mixer = _read_parallel(raw_mixer, problems)
    mlp = None
    raw_mlp = entry.get("mlp")
    if raw_mlp is not None:
        if not isinstance(raw_mlp, dict):
            r.problem("mlp must be an object or null")
        else:
            mlp = _read_mlp(raw_mlp, problems)
    problems = r.problems + problems
    if problems:
        return None, problems
    return DafalixLayer(kind, mixer, mlp), []
