"""The Dafalix design written plainly: whole sequences, no cache, no state carried between calls, 64-bit, a loop
over tokens wherever the design has a recurrence.  One function a mechanism; the GPU tests hold the engine's
kernels, parts and whole models against these.  Nothing here is shared with the product path.

Notation: T tokens, h the normed input of a sublayer, W a matrix stored [out, in] and applied as h @ W.T.
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch

F = torch.float64

# What the design allows in 16 bits (the inputs and outputs of matrix products, the short convolution, gated
# outputs) passes through ``r``; with ``rounded()`` it is rounded to bfloat16 there and nowhere else, so that the
# difference to the unrounded run is the error that rounding alone causes in this model at every position.
_ROUND = False


def r(t):
    return t.to(torch.bfloat16).to(F) if _ROUND else t


class rounded:
    def __enter__(self):
        global _ROUND
        _ROUND = True

    def __exit__(self, *exc):
        global _ROUND
        _ROUND = False


def read_config(folder) -> dict:
    return json.loads((Path(folder) / "config.json").read_text())


def load_weights(folder) -> dict:
    from safetensors.torch import load_file

    return {k: (v.to(F) if v.is_floating_point() else v) for k, v in load_file(str(Path(folder) / "model.safetensors")).items()}


# ---- pieces ------------------------------------------------------------------
def layer_norm(x, eps, weight, bias):
    """(x - mean) / sqrt(mean of squared deviations + eps) * weight + bias."""
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * weight + bias


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(x):
    return x * torch.sigmoid(x)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def softplus(x):
    return torch.clamp(x, min=0) + torch.log1p(torch.exp(-x.abs()))


def log_sigmoid(x):
    return -softplus(-x)


def causal_conv(x, taps_w, bias):
    """y[t, c] = bias[c] + sum_j taps_w[c, j] * x[t - (K - 1) + j, c], zeros before the first row."""
    T, C = x.shape
    K = taps_w.shape[1]
    xp = torch.cat([torch.zeros(K - 1, C, dtype=x.dtype), x], 0)
    y = torch.zeros_like(x)
    for t in range(T):
        for j in range(K):
            y[t] += taps_w[:, j] * xp[t + j]
    return y + bias


# ---- matrix memory ------------------------------------------------------------
def capped(x, cap):
    return cap * torch.tanh(x / cap)


def matrix_memory_recurrence(q, k, v, log_in, log_forget):
    """One head.  q, k [T, d], v [T, dv], the two log gates [T].  A running maximum m (from 0) keeps the
    exponentials in range:  m' = max(f + m, i);  S' = e^(f + m - m') S + e^(i - m') k v^T;  n likewise with k;
    o = S'^T q / (max(|n' . q|, e^(-m')) + 1e-6)."""
    T, d = k.shape
    S = torch.zeros(d, v.shape[1], dtype=F)
    n = torch.zeros(d, dtype=F)
    m = torch.zeros((), dtype=F)
    o = torch.zeros(T, v.shape[1], dtype=F)
    for t in range(T):
        m_new = torch.maximum(log_forget[t] + m, log_in[t])
        keep, take = torch.exp(log_forget[t] + m - m_new), torch.exp(log_in[t] - m_new)
        S = keep * S + take * torch.outer(k[t], v[t])
        n = keep * n + take * k[t]
        m = m_new
        o[t] = (S.T @ q[t]) / (torch.maximum((n @ q[t]).abs(), torch.exp(-m)) + 1e-6)
    return o


def matrix_memory_mixer(h, W, p, m, eps):
    T = h.shape[0]
    H, d, dv, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = r(h @ W[p + "q"].T).view(T, H, d) * d ** -0.5
    k = r(h @ W[p + "k"].T).view(T, H, d)
    v = r(h @ W[p + "v"].T).view(T, H, dv)
    log_in = capped(r(h @ W[p + "i"].T) + W[p + "i.b"], cap)
    log_forget = log_sigmoid(capped(r(h @ W[p + "f"].T) + W[p + "f.b"], cap))
    o = torch.stack([matrix_memory_recurrence(q[:, i], k[:, i], v[:, i], log_in[:, i], log_forget[:, i])
                     for i in range(H)], 1)
    o = rms(o, eps).reshape(T, H * dv) * W[p + "norm"]
    return r(o * torch.sigmoid(r(h @ W[p + "g"].T))) @ W[p + "o"].T


# ---- windowed attention --------------------------------------------------------
def rotate_halves(x, positions, dims, base, factor):
    """x [T, heads, d]: the first ``dims`` dimensions turn, i with i + dims/2, by position * base^(-2i/dims) / factor."""
    if dims == 0:
        return x
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) / factor for i in range(half)], dtype=F)
    ang = positions.to(F)[:, None] * freq
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    a, b = x[..., :half], x[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., dims:]], -1)


def window_softmax_attention(q, k, v, scale, window):
    """q [T, H, d], k [T, G, d], v [T, G, dv]: position i sees j with 0 <= i - j < window."""
    T, H, _ = q.shape
    G = k.shape[1]
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    seen = (i - j >= 0) & (i - j < window)
    out = torch.zeros(T, H, v.shape[2], dtype=F)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        s = s.masked_fill(~seen, float("-inf"))
        out[:, h] = torch.softmax(s, -1) @ v[:, g]
    return out


def window_attention_mixer(h, W, p, m, eps):
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    rot = m["rot"]
    q = rms(r(h @ W[p + "q"].T).view(T, H, d), eps) * W[p + "q.norm"]
    k = rms(r(h @ W[p + "k"].T).view(T, G, d), eps) * W[p + "k.norm"]
    v = r(h @ W[p + "v"].T).view(T, G, dv)
    pos = torch.arange(T)
    q = r(rotate_halves(q, pos, rot["dims"], rot["base"], rot["scaling"]["factor"]))
    k = r(rotate_halves(k, pos, rot["dims"], rot["base"], rot["scaling"]["factor"]))
    out = r(window_softmax_attention(q, k, v, m["scale"], m["mask"]["size"]).reshape(T, H * dv))
    return out @ W[p + "o"].T


# ---- gated linear recurrent unit --------------------------------------------------
def gated_linear_recurrence(u, gate_a, gate_in, lam):
    """u, gate_a, gate_in [T, C], lam [C]:  a = exp(-8 gate_a softplus(lam));  S' = a S + sqrt(1 - a^2) gate_in u,
    from S = 0 for the first token too."""
    T, C = u.shape
    S = torch.zeros(C, dtype=F)
    out = torch.zeros(T, C, dtype=F)
    for t in range(T):
        a = torch.exp(-8.0 * gate_a[t] * softplus(lam))
        S = a * S + torch.sqrt(1.0 - a * a) * gate_in[t] * u[t]
        out[t] = S
    return out


def block_diagonal(u, mats, bias):
    """u [T, C] cut into len(mats) equal parts; part b times mats[b] ([out, in]) plus bias[b]."""
    T, C = u.shape
    B = mats.shape[0]
    parts = u.view(T, B, C // B)
    return (torch.einsum("tbi,boi->tbo", parts, mats) + bias).reshape(T, C)


def recurrent_unit_mixer(h, W, p, m):
    y = r(gelu_tanh(r(h @ W[p + "y"].T + W[p + "y.b"])))
    u = r(causal_conv(r(h @ W[p + "x"].T + W[p + "x.b"]), W[p + "conv"], W[p + "conv.b"]))
    gate_a = torch.sigmoid(block_diagonal(u, W[p + "ra"], W[p + "ra.b"]))
    gate_in = torch.sigmoid(block_diagonal(u, W[p + "ri"], W[p + "ri.b"]))
    S = gated_linear_recurrence(u, gate_a, gate_in, W[p + "lam"])
    return r(S * y) @ W[p + "o"].T


# ---- experts -----------------------------------------------------------------------
def routed_experts(h, W, p, mlp, margins=None, forced=None, lead=0.2):
    """Scores sigmoid(W_router h); the ``top`` largest choose the experts; an expert's input is score * h.
    ``margins`` collects, for every token, by how much the last chosen logit leads the first one left out.
    ``forced`` [T, top] gives the experts instead (what an engine chose): each must be one of the largest or fall
    short of them by less than ``lead``, the room that rounding has, but for one token in fifty (or one), whose
    router may have got an input that an ill-conditioned read-out before it moved far; everything else is computed
    as ever."""
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    scores = torch.sigmoid(r(h) @ W[p + "router"].T)
    if margins is not None:
        z = torch.sort(r(h) @ W[p + "router"].T, dim=-1, descending=True).values
        margins.append(z[:, top - 1] - z[:, top] if top < E else torch.full((h.shape[0],), float("inf"), dtype=F))
    chosen = torch.topk(scores, top, dim=-1).indices
    if forced is not None:
        z = r(h) @ W[p + "router"].T
        chosen = torch.as_tensor(forced, dtype=torch.long)
        assert chosen.shape == (h.shape[0], top) and all(len(set(row)) == top for row in chosen.tolist())
        short = torch.sort(z, dim=-1, descending=True).values[:, top - 1:top] - z.gather(1, chosen)
        far = int((short.max(-1).values >= lead).sum())
        assert far <= max(1, h.shape[0] // 50), f"{far} of {h.shape[0]} tokens chose an expert far from the largest"
    out = torch.zeros(h.shape[0], W[p + "e0.down"].shape[0], dtype=F)
    for t in range(h.shape[0]):
        for e in chosen[t].tolist():
            x = r(scores[t, e] * h[t])
            out[t] += r(silu(x @ W[p + f"e{e}.gate"].T) * (x @ W[p + f"e{e}.up"].T)) @ W[p + f"e{e}.down"].T
    return out


def mixer(h, W, p, layer, eps):
    if layer["type"] == "mlstm":
        return matrix_memory_mixer(h, W, p + "mix.", layer["mixer"], eps)
    m = layer["mixer"]
    return (m["left_scale"] * window_attention_mixer(h, W, p + "mix.left.", m["left"], eps)
            + m["right_scale"] * recurrent_unit_mixer(h, W, p + "mix.right.", m["right"]))


# ---- the model -----------------------------------------------------------------
def layer_runs(cfg) -> list[int]:
    """The layers in the order they run: the looped stretch ``times`` times in a row, the rest once."""
    n = len(cfg["layers"])
    loop = cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}
    inside = list(range(loop["start"], loop["stop"]))
    return list(range(loop["start"])) + inside * loop["times"] + list(range(loop["stop"], n))


def forward(W, cfg, ids, streams=None, margins=None, forced=None):
    """Logits [T, vocab] of one sequence; ``streams`` collects the summed residual streams after every layer run,
    ``margins`` the routers' leads (``routed_experts``), one entry for every run of a layer with experts;
    ``forced`` gives the experts of every such run, in their order."""
    forced = None if forced is None else list(forced)
    eps = cfg["norm"]["eps"]
    mult, S = cfg["residual_mult"], cfg["streams"]
    xs = [W["embed"][torch.tensor(ids, dtype=torch.long)].clone() for _ in range(S)]
    for i in layer_runs(cfg):
        layer, p = cfg["layers"][i], f"l{i}."
        for q, sub in ((1, "mixer"), (2, "mlp")):
            if sub == "mlp" and layer["mlp"] is None:
                continue
            hc = p + f"hc{q}."
            u = sum(W[hc + "in"][s] * xs[s] for s in range(S))
            h = r(layer_norm(u, eps, W[p + f"norm{q}"], W[p + f"norm{q}.b"]))
            y = mixer(h, W, p, layer, eps) if sub == "mixer" else routed_experts(
                h, W, p + "mlp.", layer["mlp"], margins, None if forced is None else forced.pop(0))
            y = y * W[p + f"ls{q}"]
            xs = [sum(W[hc + "mix"][s, t] * xs[s] for s in range(S)) + mult * W[hc + "out"][t] * y for t in range(S)]
        if streams is not None:
            streams.append(sum(xs))
    x = sum(xs)
    return r(layer_norm(x, eps, W["final.norm"], W["final.norm.b"])) @ W["embed"].T


def rounding_error(W, cfg, ids, exact=None, forced=None):
    """For every position, the largest difference that rounding alone (``rounded``) makes to a logit."""
    exact = forward(W, cfg, ids, forced=forced) if exact is None else exact
    with rounded():
        coarse = forward(W, cfg, ids, forced=forced)
    return (coarse - exact).abs().max(-1).values


def float32_error(W, cfg, ids, exact, forced=None):
    """For every position, the largest difference to ``exact`` of this same implementation run in 32-bit throughout:
    what 32-bit arithmetic alone costs there (a read-out that all but cancels, a norm that blows a remainder up)."""
    global F
    F = torch.float32
    try:
        W32 = {k: (v.float() if v.is_floating_point() else v) for k, v in W.items()}
        got = forward(W32, cfg, ids, forced=forced).double()
    finally:
        F = torch.float64
    return (got - exact).abs().max(-1).values


def close_calls(W, cfg, ids, lead=0.2):
    """For every position whether some router chose there by less than ``lead``: 16-bit rounding of the router's
    input may then choose another expert, and every later position of the sequence may hear of it."""
    margins = []
    forward(W, cfg, ids, margins=margins)
    if not margins:
        return torch.zeros(len(ids), dtype=torch.bool)
    return torch.stack(margins).min(0).values < lead


def greedy(W, cfg, prompt, count):
    ids = list(prompt)
    for _ in range(count):
        ids.append(int(forward(W, cfg, ids)[-1].argmax()))
    return ids[len(prompt):]
