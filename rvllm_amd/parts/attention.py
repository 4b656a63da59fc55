"""Grouped-query attention over the paged cache.

Order of work for the tokens of a step (v3/crates/rvllm-runtime/src/gemma4_layer_exec.rs:1-28,
steps 2 to 7): one fused projection to q|k|v, per-head RMSNorm of queries and
keys, rotation, write of keys and values into the cache, attention over the
cache, output projection.  The score scale, the window, the head counts and
sizes, the norm's constants and the position encoding are parameters of the
part.  ``window`` None means every earlier key is visible; otherwise a token at
position p sees the keys p - window + 1 .. p.

Where the checkpoint keeps the part's tensors is a parameter too: ``names`` maps a
role (``q``, ``k``, ``v``, ``o``, ``q_norm``, ``k_norm``) to the tensor's name under
the layer's prefix, without ``.weight`` (the Gemma names if absent); a role ``qkv``
names one stored matrix that holds the rows of q, k and v in this order.  ``bias``
lists the projections that have a ``.bias`` beside their ``.weight`` (True: all).
``weight_suffix`` / ``bias_suffix`` are what a projection's name is followed by
(``.weight`` / ``.bias`` if absent).

Variants, all parameters: ``values`` = ``"keys"``: there is no value projection, a
token's values are its keys as projected, before norm and rotation.  ``gate`` =
``"sigmoid"``: the concatenated heads are multiplied by sigmoid of one more
projection of the layer's input (role ``g``) before the output projection.
``qk_norm`` may say ``"weight": False`` (a norm without a learned weight) and
``"after_rotation": True`` (rotate first, then norm).  A position encoding may pair
dimension i with i + rotary_dim/2 (``rope``'s ``pairing``).  ``value_dim``: the size
of a value head where it differs from ``head_dim``, the size of a query and key head;
the cache and the kernels then hold every head at the larger of the two sizes, the
shorter ones with zeros behind (zero rows of the projections, zero columns of the
output projection), which changes no score and no output.  Any of these takes the
step through ``ops.rotate_norm_write`` instead of the fused kernel of the plain case.
"""

from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops
from .base import KVCacheView, KVNeed, Mixer, ParamSpec
from .linear import bias_roles, decode_weight, linear, linear_unrounded, tensor_names
from .registry import MIXERS, POSITION_ENCODINGS
from .spec import PartSpec


class PagedAttention(Mixer):
    NAMES = {"q": "self_attn.q_proj", "k": "self_attn.k_proj", "v": "self_attn.v_proj", "o": "self_attn.o_proj",
             "q_norm": "self_attn.q_norm", "k_norm": "self_attn.k_norm"}

    def __init__(self, spec: PartSpec, *, hidden_size: int):
        self.hidden_size = int(hidden_size)
        self.num_heads = int(spec["num_heads"])
        self.num_kv_heads = int(spec["num_kv_heads"])
        self.qk_dim = int(spec["head_dim"])  # a query or key head as the checkpoint has it
        self.value_dim = int(spec.get("value_dim") or self.qk_dim)
        self.head_dim = max(self.qk_dim, self.value_dim)  # a head as the cache and the kernels hold it
        self.scale = float(spec["scale"])
        window = spec.get("window")
        self.window: Optional[int] = None if window is None else int(window)
        self.qk_norm: Optional[dict] = spec.get("qk_norm")  # {"eps":, "unit_offset":} or None
        if self.num_heads % self.num_kv_heads:
            raise ValueError(f"{self.num_heads} query heads cannot share {self.num_kv_heads} key/value heads")
        pos_spec = spec.get("position") or PartSpec("none")
        self.position = POSITION_ENCODINGS.build(pos_spec, head_dim=self.qk_dim)
        self.q_size = self.num_heads * self.head_dim
        self.kv_size = self.num_kv_heads * self.head_dim
        self.names = tensor_names(self.NAMES, spec.get("names"))
        self.w_suffix = str(spec.get("weight_suffix", ".weight"))
        self.norm_suffix = str(spec.get("norm_suffix", ".weight"))
        self.b_suffix = str(spec.get("bias_suffix", ".bias"))
        values = str(spec.get("values", "projected"))
        if values not in ("projected", "keys"):
            raise ValueError(f"attention: values {values!r}; known: 'projected', 'keys'")
        self.values_from_keys = values == "keys"
        gate = spec.get("gate")
        if gate not in (None, "sigmoid"):
            raise ValueError(f"attention: gate {gate!r}; known: None, 'sigmoid'")
        self.gate = gate
        self.norm_weight = bool((self.qk_norm or {}).get("weight", True))
        self.norm_after_rotation = bool((self.qk_norm or {}).get("after_rotation", False))
        # the projections as the checkpoint stores them: role -> rows
        if "qkv" in self.names:
            if self.values_from_keys or self.gate or self.value_dim != self.qk_dim:
                raise ValueError("attention: a stored q|k|v matrix goes with projected values of the keys' size and "
                                 "no gate")
            self.stored = {"qkv": self.q_size + 2 * self.kv_size}
        else:
            self.stored = {"q": self.q_size, "k": self.kv_size}
            if not self.values_from_keys:
                self.stored["v"] = self.kv_size
            elif self.value_dim != self.qk_dim:
                raise ValueError("attention: values that are the keys have the keys' size")
            if self.gate:
                self.names.setdefault("g", "self_attn.g_proj")
                self.stored["g"] = self.q_size
        self.bias = bias_roles(spec.get("bias"), [*self.stored, "o"])
        # the step's kernel for queries and keys: the fused one of the plain case, or the general one
        partial_halves = (self.position.rotary_dim not in (0, self.qk_dim)
                          and getattr(self.position, "pairing", "head_half") == "rotary_half")
        self.general_path = bool(self.values_from_keys or self.gate or partial_halves or self.norm_after_rotation
                                 or (self.qk_norm is not None and not self.norm_weight)
                                 or self.value_dim != self.qk_dim)
        if self.general_path and self.position.rotary_dim not in (0, self.qk_dim) \
                and getattr(self.position, "pairing", "head_half") != "rotary_half":
            raise ValueError("attention: with these variants a partial rotation pairs i with i + rotary_dim/2")
        self.w_qkv = self.w_o = self.q_norm_w = self.k_norm_w = self.b_qkv = self.b_o = None

    # ---- weights -----------------------------------------------------
    def _own(self, role: str, held: int) -> int:
        """How many rows (columns, for ``o``) of a projection the checkpoint has where the part holds ``held``."""
        own = {"q": self.qk_dim, "k": self.qk_dim, "v": self.value_dim, "g": self.value_dim, "o": self.value_dim}
        return held if role not in own else held // self.head_dim * own[role]

    def _widen(self, t: torch.Tensor, role: str) -> torch.Tensor:
        """A projection's rows (or a bias) head by head at the held size, zeros behind each head's own."""
        own = self._own(role, self.head_dim)
        if own == self.head_dim:
            return t
        heads = t.shape[0] // own
        wide = torch.zeros((heads, self.head_dim, *t.shape[1:]), dtype=t.dtype, device=t.device)
        wide[:, :own] = t.reshape(heads, own, *t.shape[1:])
        return wide.reshape(heads * self.head_dim, *t.shape[1:])

    def param_specs(self, prefix: str) -> list[ParamSpec]:
        at = {role: f"{prefix}.{name}" for role, name in self.names.items()}
        ws, bs = self.w_suffix, self.b_suffix
        specs = [ParamSpec(f"{at[role]}{ws}", (self._own(role, rows), self.hidden_size))
                 for role, rows in self.stored.items()]
        specs.append(ParamSpec(f"{at['o']}{ws}", (self.hidden_size, self._own("o", self.q_size))))
        specs += [ParamSpec(f"{at[role]}{bs}", (self._own(role, rows),)) for role, rows in self.stored.items()
                  if role in self.bias]
        if "o" in self.bias:
            specs.append(ParamSpec(f"{at['o']}{bs}", (self.hidden_size,)))
        if self.qk_norm is not None and self.norm_weight:
            specs += [
                ParamSpec(f"{at['q_norm']}{self.norm_suffix}", (self.qk_dim,), init=("normal", 0.1)),
                ParamSpec(f"{at['k_norm']}{self.norm_suffix}", (self.qk_dim,), init=("normal", 0.1)),
            ]
        return specs

    def bind(self, tensors, prefix, device, dtype) -> None:
        at = {role: f"{prefix}.{name}" for role, name in self.names.items()}
        # q, k and v rows are joined into one matrix, as the reference's loader
        # joins them (v3/crates/rvllm-loader/src/gemma4_load.rs:522,621-625).
        ws, bs = self.w_suffix, self.b_suffix
        parts = [self._widen(tensors[f"{at[role]}{ws}"].to(device=device, dtype=dtype), role) for role in self.stored]
        self.w_qkv = decode_weight(torch.cat(parts, dim=0).contiguous(), self.tiled_weights)
        w_o = tensors[f"{at['o']}{ws}"].to(device=device, dtype=dtype)
        self.w_o = decode_weight(self._widen(w_o.t(), "o").t().contiguous(), self.tiled_weights)
        if self.bias & set(self.stored):  # projections without a bias of their own add zeros
            self.b_qkv = torch.cat([
                self._widen(tensors[f"{at[role]}{bs}"].to(device=device, dtype=torch.float32), role) if role in self.bias
                else torch.zeros(rows, dtype=torch.float32, device=device) for role, rows in self.stored.items()])
        if "o" in self.bias:
            self.b_o = tensors[f"{at['o']}{bs}"].to(device=device, dtype=torch.float32).contiguous()
        if self.qk_norm is not None and self.norm_weight:
            self.q_norm_w = tensors[f"{at['q_norm']}{self.norm_suffix}"].to(device).contiguous()
            self.k_norm_w = tensors[f"{at['k_norm']}{self.norm_suffix}"].to(device).contiguous()
            if self.q_norm_w.dtype != self.k_norm_w.dtype:
                self.k_norm_w = self.k_norm_w.to(self.q_norm_w.dtype)

    # ---- cache -------------------------------------------------------
    def cache_need(self) -> KVNeed:
        return KVNeed(self.num_kv_heads, self.head_dim, self.window)

    # ---- run ---------------------------------------------------------
    def forward(self, x: torch.Tensor, step, cache: KVCacheView) -> torch.Tensor:
        if self.general_path:
            return self._forward_general(x, step, cache)
        n = x.shape[0]
        qkv = linear(x, self.w_qkv, sliced_ok=True)
        if self.b_qkv is not None:
            qkv = ops.add_bias(qkv, self.b_qkv)
        q = torch.empty((n, self.q_size), dtype=x.dtype, device=x.device)
        table = step.block_tables[cache.group]
        norm = self.qk_norm or {}
        # prompt portions: values go into their pages a page at a time, in wide stores, by blocks of the same launch
        by_page = (cache.writes and isinstance(qkv, torch.Tensor)
                   and step.max_portion >= ops.VALUES_BY_PAGE_MIN_PORTION)
        ops.qk_norm_rope_kv_write(
            qkv, q, self.q_norm_w, self.k_norm_w, float(norm.get("eps", 0.0)),
            1.0 if norm.get("unit_offset", False) else 0.0, self.position.tables(step),
            self.position.rotary_dim, step.positions, step.token_req, table, cache.k_pages, cache.v_pages,
            self.num_heads, self.num_kv_heads, self.head_dim, write_kv=cache.writes,
            values_by_page=step if by_page else None)
        attn = torch.empty_like(q)
        ops.paged_attention(q, cache.k_pages, cache.v_pages, table, step, attn, self.num_heads, self.scale,
                            self.window)
        out = linear(attn, self.w_o, sliced_ok=True)
        return out if self.b_o is None else ops.add_bias(out, self.b_o)


    def _forward_general(self, x: torch.Tensor, step, cache: KVCacheView) -> torch.Tensor:
        """The variants: the rows of the fused projection hold q | k | (v) | (g)."""
        n = x.shape[0]
        proj = linear(x, self.w_qkv)
        bias = self.b_qkv
        if bias is not None and "g" in self.bias:  # the gate reads its columns from the rows: its bias goes in there
            proj, bias = ops.add_bias(proj, bias), None
        q = torch.empty((n, self.q_size), dtype=x.dtype, device=x.device)
        table = step.block_tables[cache.group]
        norm = self.qk_norm or {}
        mode = ops.NORM_NONE if self.qk_norm is None else (
            ops.NORM_AFTER_ROTATION if self.norm_after_rotation else ops.NORM_BEFORE_ROTATION)
        k_col = self.q_size
        v_col = None if self.values_from_keys else k_col + self.kv_size
        ops.rotate_norm_write(
            proj, 0, k_col, v_col, q, self.q_norm_w, self.k_norm_w, float(norm.get("eps", 0.0)),
            1.0 if norm.get("unit_offset", False) else 0.0, mode, self.position.tables(step),
            self.position.rotary_dim, step.positions, step.token_req, table, cache.k_pages, cache.v_pages,
            self.num_heads, self.num_kv_heads, self.head_dim, write_kv=cache.writes, bias=bias,
            norm_dim=self.qk_dim)
        attn = torch.empty_like(q)
        ops.paged_attention(q, cache.k_pages, cache.v_pages, table, step, attn, self.num_heads, self.scale,
                            self.window)
        if self.gate:
            ops.gate_mul_(attn, proj, proj.shape[1] - self.q_size, self.gate)
        if self.b_o is None:
            return linear_unrounded(attn, self.w_o)
        return ops.add_bias(linear(attn, self.w_o, sliced_ok=True), self.b_o)


MIXERS.register("attention", PagedAttention)
