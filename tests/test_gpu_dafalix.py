"""The Dafalix design on the GPU against the plain implementation (``plain_dafalix``): each mechanism alone at the
level of its kernels and parts, then whole models through the step function under every way of cutting the work,
through ``bin/trace_run`` and through the engine's scheduler."""

import numpy as np
import pytest
import torch

import plain_dafalix as PD
import tiny_dafalix
import trace_tools as tt
from rvllm_amd.cache.manager import CacheManager, group_name
from rvllm_amd.cache.storage import CacheStorage
from rvllm_amd.config.engine_config import EngineConfig
from rvllm_amd.engine.batch import BatchBuilder, Portion
from rvllm_amd.engine.runner import ModelRunner
from rvllm_amd.kernels import ops
from rvllm_amd.parts.block import StreamsBlock
from rvllm_amd.parts.registry import FEED_FORWARDS, MIXERS
from rvllm_amd.parts.spec import PartSpec

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def dev(t):
    return t.to(DEV).contiguous()


def close(got, want, dtype, what="", f32=2e-5, bf16=2e-2):
    """Against the values' own size: 32-bit to a few roundings, bf16 to a few of its."""
    got, want = got.detach().double().cpu(), want.detach().double().cpu()
    assert got.shape == want.shape, f"{what}: {tuple(got.shape)} against {tuple(want.shape)}"
    assert bool(torch.isfinite(got).all()), f"{what}: not finite"
    scale = float(want.abs().max()) or 1.0
    worst = float((got - want).abs().max())
    assert worst <= (f32 if dtype == torch.float32 else bf16) * scale, f"{what}: {worst:.3e} against {scale:.3e}"


def make_step(portions, slots):
    """A step of ``portions`` = [(first position, tokens)], request b in state slot ``slots[b]``; no page groups."""
    total = sum(n for _, n in portions)
    builder = BatchBuilder(torch.device(DEV), max(total, 1), max(len(portions), 1), {})
    return builder.build([Portion(b, [0] * n, start) for b, (start, n) in enumerate(portions)], {}, slots)


def cuts_of(total, sizes):
    """(first, count) pieces of ``total`` tokens, sizes taken in turn."""
    out, at, i = [], 0, 0
    while at < total:
        n = min(sizes[i % len(sizes)], total - at)
        out.append((at, n))
        at += n
        i += 1
    return out


# --------------------------------------------------------------------------
# mechanisms alone
# --------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width", [64, 100, 1030, 4100, 4500])
def test_layer_norm(dtype, width):
    g = torch.Generator().manual_seed(width)
    x = torch.randn(7, width, generator=g) * 3 + 1.5
    w, b = torch.randn(width, generator=g), torch.randn(width, generator=g)
    want = PD.layer_norm(x.double(), 1e-5, w.double(), b.double())
    close(ops.layernorm(dev(x), dev(w), dev(b), 1e-5, dtype), want, dtype, "32-bit rows")
    close(ops.layernorm(dev(x.to(dtype)), dev(w), dev(b), 1e-5, dtype),
          PD.layer_norm(x.to(dtype).double(), 1e-5, w.double(), b.double()), dtype, "rows of the activations' type")
    rows = torch.tensor([5, 0, 5, 2], dtype=torch.int32)
    close(ops.layernorm(dev(x), dev(w), dev(b), 1e-5, dtype, rows=dev(rows)), want[rows.long()], dtype, "chosen rows")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("streams,width", [(1, 64), (2, 100), (3, 300), (4, 1100), (8, 4100), (2, 4500)])
def test_streams_move_on_as_the_equations_say(dtype, streams, width):
    """The seeding, a branch of every kind (a tensor, unreduced partial sums, two weighted branches), the layer scale,
    the next input with its norm, and the streams' sum."""
    g = torch.Generator().manual_seed(streams * 7 + width)
    n = 5
    seed = torch.randn(n, width, generator=g) * 2
    mix, out_w, in_w = torch.randn(streams, streams, generator=g), torch.randn(streams, generator=g), torch.randn(streams, generator=g)
    ls, nw, nb = torch.randn(width, generator=g), torch.randn(width, generator=g), torch.randn(width, generator=g)
    xs = torch.empty(streams, n, width, device=DEV)
    first = ops.streams_update(xs, dtype, seed=dev(seed), in_w=dev(in_w), norm_w=dev(nw), norm_b=dev(nb), eps=1e-5)
    want_xs = [seed.double().clone() for _ in range(streams)]
    close(xs, torch.stack(want_xs), torch.float32, "seeded")
    u = sum(in_w[s].double() * want_xs[s] for s in range(streams))
    close(first, PD.layer_norm(u, 1e-5, nw.double(), nb.double()), dtype, "first input")
    y1 = torch.randn(n, width, generator=g).to(dtype)
    parts = torch.randn(3, n, width, generator=g)
    y2 = torch.randn(n, width, generator=g).to(dtype)
    branches = [
        (dev(y1), y1.double()),
        (ops.SlicedSums(dev(parts), dtype), parts.double().sum(0)),
        (ops.BranchSum(dev(y1), ops.SlicedSums(dev(parts), dtype), 0.8, -1.1), 0.8 * y1.double() - 1.1 * parts.double().sum(0)),
        (ops.BranchSum(dev(y2), dev(y1), 1.0, 0.5), y2.double() + 0.5 * y1.double()),
    ]
    for i, (branch, y) in enumerate(branches):
        last = i == len(branches) - 1
        total = torch.empty(n, width, device=DEV) if last else None
        scale = None if i == 1 else dev(ls)
        nxt = ops.streams_update(xs, dtype, branch=branch, layer_scale=scale, mix=dev(mix), out_w=dev(out_w), mult=0.6,
                                 in_w=None if last else dev(in_w), norm_w=None if last else dev(nw),
                                 norm_b=None if last else dev(nb), eps=1e-5, total=total)
        ys = y if scale is None else y * ls.double()
        want_xs = [sum(mix[s, t].double() * want_xs[s] for s in range(streams)) + 0.6 * out_w[t].double() * ys
                   for t in range(streams)]
        close(xs, torch.stack(want_xs), torch.float32, f"streams after branch {i}", f32=1e-5)
        if last:
            assert nxt is None
            close(total, sum(want_xs), torch.float32, "the streams' sum", f32=1e-5)
        else:
            u = sum(in_w[s].double() * want_xs[s] for s in range(streams))
            close(nxt, PD.layer_norm(u, 1e-5, nw.double(), nb.double()), dtype, f"input after branch {i}", f32=1e-4)
    # only reading: the streams stay as they are
    before = xs.clone()
    again = ops.streams_update(xs, dtype, in_w=dev(in_w), norm_w=dev(nw), norm_b=dev(nb), eps=1e-5)
    assert torch.equal(xs, before)
    u = sum(in_w[s].double() * want_xs[s] for s in range(streams))
    close(again, PD.layer_norm(u, 1e-5, nw.double(), nb.double()), dtype, "read only", f32=1e-4)


def memory_read(*args):
    """``ops.matrix_memory`` with the division that it leaves to the kernel behind it."""
    o, (dots, gates) = ops.matrix_memory(*args)
    heads = dots.shape[1]
    den = torch.maximum(dots.abs(), gates[..., 2]) + 1e-6
    return (o.view(o.shape[0], heads, -1) / den[..., None]).reshape(o.shape[0], -1)


def _memory_case(heads, dk, dv, T, g, dtype, cap, far=False):
    """Rows q | pad | k | v | i | f of type ``dtype`` and what the plain recurrence makes of them."""
    pad = 3
    width = 2 * heads * dk + pad + heads * dv + 2 * heads
    rows = torch.randn(T, width, generator=g)
    k_col, v_col = heads * dk + pad, 2 * heads * dk + pad
    i_col = v_col + heads * dv
    f_col = i_col + heads
    rows[:, i_col:] *= 3.0
    i_bias, f_bias = torch.randn(heads, generator=g), torch.randn(heads, generator=g) + 2.0
    if far:  # one token early on is taken with a large gate and hardly forgotten; the last query asks for its key
        rows[:, f_col:f_col + heads] = 40.0
        rows[:, i_col:i_col + heads] = -6.0
        rows[3, i_col:i_col + heads] = 9.0
        rows[-1, :heads * dk] = rows[3, k_col:k_col + heads * dk] * 4.0
    rows = rows.to(dtype)
    r64 = rows.double()
    log_in = PD.capped(r64[:, i_col:i_col + heads] + i_bias.double(), cap)
    log_forget = PD.log_sigmoid(PD.capped(r64[:, f_col:f_col + heads] + f_bias.double(), cap))
    want = torch.cat([PD.matrix_memory_recurrence(
        r64[:, h * dk:(h + 1) * dk] * dk ** -0.5, r64[:, k_col + h * dk:k_col + (h + 1) * dk],
        r64[:, v_col + h * dv:v_col + (h + 1) * dv], log_in[:, h], log_forget[:, h]) for h in range(heads)], 1)
    return rows, (k_col, v_col, i_col, f_col), i_bias, f_bias, want


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,dk,dv", [(2, 16, 24), (1, 40, 12), (6, 7, 70), (2, 128, 64), (3, 300, 5), (1, 5, 130),
                                         (2, 64, 64), (1, 520, 8)])
def test_matrix_memory_whole_and_cut_give_the_same_bits(dtype, heads, dk, dv):
    g = torch.Generator().manual_seed(heads * 100 + dk)
    T, cap = 41, 6.0
    rows, (k_col, v_col, i_col, f_col), i_bias, f_bias, want = _memory_case(heads, dk, dv, T, g, dtype, cap)
    s_off = 5
    n_off = s_off + heads * dk * dv + 2
    m_off = n_off + heads * dk + 1
    results = []
    for sizes in ([T], [1], [2, 3, 1, 7, 16]):
        slots = torch.zeros(3, m_off + heads + 4, device=DEV)
        got = []
        for start, n in cuts_of(T, sizes):
            step = make_step([(start, n)], [1])
            got.append(memory_read(dev(rows[start:start + n]), 0, k_col, v_col, i_col, f_col, dev(i_bias),
                                         dev(f_bias), cap, dk ** -0.5, slots, s_off, n_off, m_off, step, heads, dk, dv))
        results.append(torch.cat(got))
        close(results[-1], want, torch.float32, f"cut {sizes}", f32=1e-4)
        assert float(slots[[0, 2]].abs().max()) == 0.0 and float(slots[1, :s_off].abs().max()) == 0.0
    assert torch.equal(results[0], results[1]) and torch.equal(results[0], results[2])


@pytest.mark.parametrize("dtype", DTYPES)
def test_matrix_memory_keeps_a_token_taken_long_ago(dtype):
    """520 tokens in portions, two requests in a step: the last query's answer is the value taken at position 3."""
    g = torch.Generator().manual_seed(11)
    heads, dk, dv, T, cap = 2, 32, 16, 520, 50.0
    cases = [_memory_case(heads, dk, dv, T, g, dtype, cap, far=True), _memory_case(heads, dk, dv, 77, g, dtype, cap)]
    cols = cases[0][1]
    i_bias, f_bias = cases[0][2] * 0, cases[0][3] * 0
    for case in cases:  # the biases are shared by the requests of a step: taken as zero
        r64 = case[0].double()
        k_col, v_col, i_col, f_col = cols
        log_in = PD.capped(r64[:, i_col:i_col + heads], cap)
        log_forget = PD.log_sigmoid(PD.capped(r64[:, f_col:f_col + heads], cap))
        case_want = torch.cat([PD.matrix_memory_recurrence(
            r64[:, h * dk:(h + 1) * dk] * dk ** -0.5, r64[:, k_col + h * dk:k_col + (h + 1) * dk],
            r64[:, v_col + h * dv:v_col + (h + 1) * dv], log_in[:, h], log_forget[:, h]) for h in range(heads)], 1)
        case[4].copy_(case_want)
    far_rows, want = cases[0][0], cases[0][4]
    v3 = far_rows[3, cols[1]:cols[1] + heads * dv].double()
    assert float((want[-1] - v3).abs().max()) < 0.05 * float(v3.abs().max())  # the plain recurrence recalls it
    n_off = heads * dk * dv
    slots = torch.zeros(4, n_off + heads * dk + heads, device=DEV)
    cuts = [cuts_of(T, [64, 2, 100, 1, 33]), cuts_of(77, [5, 1, 1, 30])]
    got = [[], []]
    for i in range(max(len(c) for c in cuts)):
        live = [r for r in range(2) if i < len(cuts[r])]
        step = make_step([cuts[r][i] for r in live], [3 if r == 0 else 0 for r in live])
        rows = torch.cat([cases[r][0][cuts[r][i][0]:cuts[r][i][0] + cuts[r][i][1]] for r in live])
        o = memory_read(dev(rows), 0, *cols, dev(i_bias), dev(f_bias), cap, dk ** -0.5, slots, 0, n_off,
                              n_off + heads * dk, step, heads, dk, dv)
        at = 0
        for r in live:
            got[r].append(o[at:at + cuts[r][i][1]])
            at += cuts[r][i][1]
    # a query that happens to stand across the one key the memory holds divides a small sum by a small sum: such
    # rows carry the roundings of a 32-bit dot product at a thousand times their size; the far query does not
    for r in range(2):
        close(torch.cat(got[r]), cases[r][4], torch.float32, f"request {r}", f32=5e-3)
    close(torch.cat(got[0])[-1], want[-1], torch.float32, "the far query", f32=2e-5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("channels,blocks", [(48, 3), (36, 36), (80, 1), (200, 5), (64, 4), (130, 2)])
def test_gated_linear_unit_whole_and_cut_give_the_same_bits(dtype, channels, blocks):
    g = torch.Generator().manual_seed(channels + blocks)
    T = 45
    block = channels // blocks
    u = (torch.randn(T, channels, generator=g) * 2).to(dtype)
    y = torch.randn(T, channels + 9, generator=g).to(dtype)
    ra, ri = (torch.randn(blocks, block, block, generator=g) * 0.5).to(dtype), (torch.randn(blocks, block, block, generator=g) * 0.5).to(dtype)
    ra_b, ri_b = torch.randn(blocks, block, generator=g), torch.randn(blocks, block, generator=g)
    lam = torch.randn(channels, generator=g) - 2.0
    gate_a = torch.sigmoid(PD.block_diagonal(u.double(), ra.double(), ra_b.double()))
    gate_in = torch.sigmoid(PD.block_diagonal(u.double(), ri.double(), ri_b.double()))
    S = PD.gated_linear_recurrence(u.double(), gate_a, gate_in, lam.double())
    want = S * PD.gelu_tanh(y[:, 9:].double()).to(dtype).double()
    w_gates = dev(torch.cat([ra, ri], dim=1))
    results = []
    for sizes in ([T], [1], [2, 3, 1, 7, 16]):
        slots = torch.zeros(3, 4 + channels, device=DEV)
        got = []
        for start, n in cuts_of(T, sizes):
            step = make_step([(start, n)], [2])
            rows = dev(u[start:start + n])
            gates = ops.gemm_blocks_f32(rows, w_gates)
            got.append(ops.gated_linear_scan(rows, gates, block, dev(ra_b.reshape(-1)), dev(ri_b.reshape(-1)), dev(lam),
                                             dev(y[start:start + n]), 9, slots, 4, step))
        results.append(torch.cat(got))
        close(results[-1], want, dtype, f"cut {sizes}", f32=1e-4)
        close(slots[2, 4:], S[-1], torch.float32, "the state left behind", f32=1e-4)
        assert float(slots[:2].abs().max()) == 0.0 and float(slots[2, :4].abs().max()) == 0.0
    assert torch.equal(results[0], results[1]) and torch.equal(results[0], results[2])


@pytest.mark.parametrize("experts,top", [(5, 2), (12, 1), (3, 3), (130, 4), (64, 8), (1, 1)])
def test_the_router_chooses_the_largest_and_breaks_ties_downwards(experts, top):
    g = torch.Generator().manual_seed(experts)
    logits = torch.randn(37, experts, generator=g) * 2
    if experts > 2:
        logits[5, :] = 0.25            # all equal: the lowest indices
        logits[6, experts - 1] = logits[6].max() + 1.0
        logits[7, 0] = logits[7, experts - 1] = 9.0
    chosen, weights = ops.moe_topk(dev(logits), top)
    chosen, weights = chosen.cpu().long(), weights.cpu()
    for t in range(logits.shape[0]):
        order = sorted(range(experts), key=lambda e: (-float(logits[t, e]), e))[:top]
        assert chosen[t].tolist() == order, f"row {t}"
    close(weights, torch.sigmoid(logits.double()).gather(1, chosen), torch.float32)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden,ff,experts,top,tokens", [(64, 32, 5, 2, 19), (100, 50, 3, 3, 7), (48, 40, 12, 1, 300),
                                                          (72, 24, 130, 4, 33), (64, 16, 4, 2, 1)])
def test_experts_with_a_learned_router(dtype, hidden, ff, experts, top, tokens):
    g = torch.Generator().manual_seed(hidden + experts)
    spec = PartSpec("routed_experts", {"experts": experts, "top": top, "intermediate_size": ff, "router": "sigmoid_topk",
                                       "weight_on": "input", "activation": "silu_glu"})
    part = FEED_FORWARDS.build(spec, hidden_size=hidden)
    W = {s.name: (torch.randn(s.shape, generator=g) * (1.0 / s.shape[-1] ** 0.5)).to(dtype) for s in part.param_specs("L")}
    W["L.mlp.router"] = (torch.randn(experts, hidden, generator=g) * 0.3).to(dtype)
    part.bind(W, "L", torch.device(DEV), dtype)
    h = torch.randn(tokens, hidden, generator=g).to(dtype)
    plain = {k[len("L.mlp."):]: v.double() for k, v in W.items()}
    mlp = {"router": {"experts": experts, "top": top}}
    want = PD.routed_experts(h.double(), plain, "", mlp)
    got = part.forward(dev(h), make_step([(0, tokens)], [0]))
    close(got, want, dtype, "experts", bf16=3e-2)


# --------------------------------------------------------------------------
# whole models through the step function
# --------------------------------------------------------------------------
LENGTHS = {"A": [70, 1, 33, 2, 45, 17], "B": [40, 3, 25, 1, 18], "A-loud": [70, 29, 48, 5]}
MODES = {"whole": tt.trace_whole, "tail": tt.trace_tail, "portions": tt.trace_portions, "mixed": tt.trace_mixed}
# By model and request, the error at every position that rounding to bfloat16 alone causes in the plain
# implementation, where the design allows 16 bits.  Nothing norms a branch before it joins the streams, and a
# router's close call changes an expert; the bf16 engine is held to three times that error or the flat share of the
# largest logit, whichever is larger; from a router's first close call on, a tenth of the positions may be over
# (``trace_tools.compare_where_routers_may_differ``).
ROUNDING: dict = {}
CLOSE: dict = {}


@pytest.fixture(scope="module")
def dafalix_dirs(tmp_path_factory):
    root = tmp_path_factory.mktemp("dafalix")
    return {"A": tiny_dafalix.write_model(root / "A", "A"), "B": tiny_dafalix.write_model(root / "B", "B"),
            "A-loud": tiny_dafalix.write_model(root / "A-loud", "A", seed=5, loud=True)}


@pytest.fixture(scope="module")
def references(dafalix_dirs):
    out = {}
    for name, folder in dafalix_dirs.items():
        weights, cfg = PD.load_weights(folder), PD.read_config(folder)
        seqs = tt.make_sequences(cfg["vocab"], LENGTHS[name], seed=len(name) + ord(name[0]))
        refs = {rid: PD.forward(weights, cfg, ids) for rid, ids in seqs.items()}
        out[name] = (seqs, refs, cfg["vocab"])
        ROUNDING[name] = {rid: PD.rounding_error(weights, cfg, ids, refs[rid]) for rid, ids in seqs.items()}
        CLOSE[name] = {rid: PD.close_calls(weights, cfg, ids).numpy() for rid, ids in seqs.items()}
    return out


def compare(got, ref, dtype, what, model=None, rid=None):
    if dtype == "bfloat16" and model in ROUNDING:
        allowed = np.maximum(tt.TOLERANCE[dtype] * float(ref.abs().max()), 3.0 * ROUNDING[model][rid].numpy())
        tt.compare_where_routers_may_differ(got, ref, allowed, CLOSE[model][rid], what)
        return
    tt.compare(got, ref, dtype, what)


def make_runner(model_dir, dtype, max_tokens, page_size=16, **more):
    cfg = EngineConfig(dtype=dtype, page_size=page_size, max_model_len=max_tokens, max_num_seqs=4,
                       max_num_batched_tokens=max_tokens, max_prefill_chunk=max_tokens, max_cache_tokens=max_tokens,
                       **more)
    return ModelRunner.from_model_dir(model_dir, cfg)


def check_with_the_engines_choices(folder, steps, outputs, choices, seqs, vocab, what):
    """The 16-bit engine against the plain implementation made to use the experts that the engine chose (each of
    them one of the largest or short of them by less than rounding moves a logit): every position is then held to
    three times the error that rounding alone causes there, or the flat share of the largest logit."""
    weights, cfg = PD.load_weights(folder), PD.read_config(folder)
    got = tt.collect(steps, outputs, vocab)
    forced = choices.by_request(steps)
    prefix = steps[0]["entries"][0]["id"].split("-")[0]
    for name, ids in seqs.items():
        rid = f"{prefix}-{name}"
        ref = PD.forward(weights, cfg, ids, forced=forced.get(rid))
        rounding = PD.rounding_error(weights, cfg, ids, ref, forced=forced.get(rid)).numpy()
        arr = np.asarray(got[rid], dtype=np.float64)
        assert arr.shape == tuple(ref.shape) and np.isfinite(arr).all(), f"{what} {name}"
        err = np.abs(arr - ref.numpy()).max(-1)
        allowed = np.maximum(tt.TOLERANCE["bfloat16"] * float(ref.abs().max()), 3.0 * rounding)
        worst = int((err / allowed).argmax())
        assert err[worst] <= allowed[worst], f"{what} {name}: position {worst}: {err[worst]:.3e} > {allowed[worst]:.3e}"


def check(steps, outputs, refs, vocab, dtype, what, model=None):
    got = tt.collect(steps, outputs, vocab)
    prefix = steps[0]["entries"][0]["id"].split("-")[0]
    assert len(got) == len(refs)
    for name, ref in refs.items():
        compare(got[f"{prefix}-{name}"], ref, dtype, f"{what} {name}", model, name)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_the_streams_sum_after_every_layer_run(dafalix_dirs, name, dtype):
    """Layer by layer, a looped layer every time it runs: the first run that differs names the mechanism."""
    folder = dafalix_dirs[name]
    weights, cfg = PD.load_weights(folder), PD.read_config(folder)
    ids = tt.make_sequences(cfg["vocab"], [50], seed=2)["r0"]
    want = []
    PD.forward(weights, cfg, ids, want)
    runner = make_runner(folder, dtype, 64)
    got = []
    for block in runner.model.blocks:
        inner = block.forward

        def spy(x, step, cache, entered=None, then=None, inner=inner):
            out = inner(x, step, cache, entered=entered, then=then)
            got.append(step.shared[StreamsBlock.STREAMS].sum(0).float().cpu())
            return out

        block.forward = spy
    runner.add_request("a")
    runner.step([("a", ids, [len(ids) - 1])])
    assert len(got) == len(want) == len(PD.layer_runs(cfg))
    calls = PD.close_calls(weights, cfg, ids).numpy()
    for i, (g_, w_) in enumerate(zip(got, want)):
        if dtype == "float32":
            close(g_, w_, torch.float32, f"after layer run {i}")
        else:  # up to a router's first close call: behind it another expert may have spoken
            first = int(np.argmax(calls)) if calls.any() else len(calls)
            assert first >= 5, "the sequence is to have a stretch without close calls"
            close(g_[:first], w_[:first], torch.bfloat16, f"after layer run {i}", bf16=3e-2)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "A-loud"])
@pytest.mark.parametrize("mode", list(MODES))
def test_cuttings(dafalix_dirs, references, name, dtype, mode):
    """Whole prompts; prefill and then token-by-token decoding; portions down to two tokens and single tokens;
    unequal requests mixed in a batch, with a pool so small that pages and slots are used again."""
    seqs, refs, vocab = references[name]
    steps = MODES[mode](seqs)
    if dtype == "bfloat16":  # kernel by kernel, so that every choice of a router is seen
        runner = make_runner(dafalix_dirs[name], dtype, tt.required_tokens(steps), use_graphs=False)
        with tt.RecordedChoices() as choices:
            outputs = tt.run_in_process(runner, steps, choices)
        check_with_the_engines_choices(dafalix_dirs[name], steps, outputs, choices, seqs, vocab, f"{name} {mode}")
    else:
        runner = make_runner(dafalix_dirs[name], dtype, tt.required_tokens(steps))
        check(steps, tt.run_in_process(runner, steps), refs, vocab, dtype, f"{name} {dtype} {mode}", name)
    assert all(g.pool.free_count == g.pool.num_pages for g in runner.cache.groups.values())
    assert runner.cache.slots.free_count == 4


@pytest.mark.parametrize("name", ["A", "B"])
def test_cuttings_agree_bit_for_bit_in_32_bit(dafalix_dirs, references, name):
    """No logit depends on how the prompt was cut, on what else is in the batch or on the pages and slots used."""
    seqs, refs, vocab = references[name]
    runner = make_runner(dafalix_dirs[name], "float32", 4 * 192)
    results = {}
    for mode, make in MODES.items():
        steps = make(seqs)
        got = tt.collect(steps, tt.run_in_process(runner, steps), vocab)
        results[mode] = {rid.split("-", 1)[1]: arr for rid, arr in got.items()}
    for mode in ("tail", "portions", "mixed"):
        for rid in seqs:
            assert np.array_equal(results[mode][rid], results["whole"][rid]), f"{name} {mode} {rid}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mode", ["tail", "mixed"])
def test_what_a_page_or_slot_held_before_reaches_no_logit(dafalix_dirs, references, dtype, mode):
    """Pages full of NaN and state slots full of large numbers before the first request: pages are never read
    past a request's own tokens, and a slot is cleared when it is handed out; every pass of a looped layer has
    pages and a slot of its own."""
    seqs, refs, vocab = references["A-loud"]
    steps = MODES[mode](seqs)
    runner = make_runner(dafalix_dirs["A-loud"], dtype, tt.required_tokens(steps))
    assert len(runner.storage.views) == 6  # four layers, two of them a second time

    def spoil(view):
        if isinstance(view, tuple):
            for member in view:
                spoil(member)
        elif hasattr(view, "k_pages"):
            view.k_pages.fill_(float("nan"))
            view.v_pages.fill_(float("nan"))
        elif view is not None:
            view.slots.fill_(1e4)

    for view in runner.storage.views:
        spoil(view)
    check(steps, tt.run_in_process(runner, steps), refs, vocab, dtype, f"spoiled {dtype} {mode}", "A-loud")


@pytest.mark.parametrize("page_size", [32, 64])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_other_page_sizes(dafalix_dirs, references, page_size, dtype):
    seqs, refs, vocab = references["A"]
    steps = tt.trace_mixed(seqs, seed=3)
    runner = make_runner(dafalix_dirs["A"], dtype, tt.required_tokens(steps), page_size=page_size)
    check(steps, tt.run_in_process(runner, steps), refs, vocab, dtype, f"page {page_size}", "A")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(dafalix_dirs, references, tmp_path, dtype):
    seqs, refs, vocab = references["B"]
    steps, n = [], 0
    for make in MODES.values():
        part = make(seqs, first_step=n)
        steps += part
        n += len(part)
    outputs = tt.run_trace_program(dafalix_dirs["B"], dtype, steps, tmp_path / "out", max_tokens=tt.required_tokens(steps))
    got = tt.collect(steps, outputs, vocab)
    for prefix in ("w", "t", "p", "m"):
        for name, ref in refs.items():
            compare(got[f"{prefix}-{name}"], ref, dtype, f"trace_run {dtype} {prefix}-{name}", "B", name)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_sequences_window_edges_and_long_decoding(tmp_path_factory, dtype):
    """Wide layers with loud keys over 700 tokens, windows of 100 and 64 that end inside pages: a prompt in one
    step, one in portions that end inside pages and windows, and the last 200 tokens decoded one by one (in bf16
    from recorded graphs), so that both windows pass wholly over decoded tokens."""
    folder = tiny_dafalix.write_model(tmp_path_factory.mktemp("C") / "C", "C", loud=True)
    weights, cfg = PD.load_weights(folder), PD.read_config(folder)
    ids = tt.make_sequences(cfg["vocab"], [700], seed=77)["r0"]
    want = PD.forward(weights, cfg, ids)
    rounding = PD.rounding_error(weights, cfg, ids, want).numpy()
    calls = PD.close_calls(weights, cfg, ids).numpy()

    def held(got, what):
        if dtype == "float32":
            return tt.compare(got, want, dtype, what)
        allowed = np.maximum(tt.TOLERANCE[dtype] * float(want.abs().max()), 3.0 * rounding)
        tt.compare_where_routers_may_differ(got, want, allowed, calls, what)

    runner = make_runner(folder, dtype, 1024)
    runner.add_request("whole")
    got = runner.step([("whole", ids, list(range(len(ids))))]).float().cpu().numpy()
    runner.release("whole")
    held(got, "whole")
    runner.add_request("cut")
    rows, at = [], 0
    for size in (63, 2, 36, 99, 1, 100, 130, 69):
        rows.append(runner.step([("cut", ids[at:at + size], list(range(size)))]).float().cpu().numpy())
        at += size
    while at < len(ids):
        rows.append(runner.step([("cut", ids[at:at + 1], [0])]).float().cpu().numpy().copy())
        at += 1
    runner.release("cut")
    held(np.concatenate(rows), "portions, then token by token")


def test_a_key_just_inside_and_just_outside_the_window_shows(dafalix_dirs):
    """The loud model's attention output moves when the token at the window's far edge changes, and does not when
    the token one further back does: checked on the plain implementation's attention, which the engine is held
    against at every position by the tests above."""
    folder = dafalix_dirs["A-loud"]
    weights, cfg = PD.load_weights(folder), PD.read_config(folder)
    m = cfg["layers"][1]["mixer"]["left"]
    window = m["mask"]["size"]
    g = torch.Generator().manual_seed(4)
    T = window + 6
    h = torch.randn(T, cfg["width"], generator=g, dtype=PD.F)
    base = PD.window_attention_mixer(h, weights, "l1.mix.left.", m, cfg["norm"]["eps"])
    for back, moves in ((window - 1, True), (window, False)):
        changed = h.clone()
        changed[T - 1 - back] += 3.0
        out = PD.window_attention_mixer(changed, weights, "l1.mix.left.", m, cfg["norm"]["eps"])
        assert bool((out[-1] - base[-1]).abs().max() > 1e-9) == moves


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_windows_edge_in_prompts_and_in_decoding(dafalix_dirs, dtype):
    """One layer's attention alone through the engine's part, with values of another size than the keys and norm
    weights so large that a softmax hangs on few keys, so that a key just inside or just outside the window of 19
    shows: a key written in a prompt's portion and asked for by a decoded token, and the other way round, the whole
    window over decoded tokens, portions that end inside it."""

    hidden, heads, dim, vdim, window = 64, 2, 16, 24, 19
    spec = PartSpec("attention", {
        "num_heads": heads, "num_kv_heads": 1, "head_dim": dim, "value_dim": vdim, "scale": 1.0, "window": window,
        "qk_norm": {"eps": 1e-6}, "position": PartSpec("none"), "weight_suffix": "", "norm_suffix": "",
        "names": {"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm"}})
    torch_dtype = torch.float32 if dtype == "float32" else torch.bfloat16
    g = torch.Generator().manual_seed(8)
    T = 60
    h = torch.randn(T, hidden, generator=g).to(torch_dtype)
    W = {"L.q": torch.randn(heads * dim, hidden, generator=g) / 8, "L.k": torch.randn(dim, hidden, generator=g) / 8,
         "L.v": torch.randn(vdim, hidden, generator=g) / 8, "L.o": torch.randn(hidden, heads * vdim, generator=g) / 5,
         "L.q.norm": torch.full((dim,), 4.0), "L.k.norm": torch.full((dim,), 4.0)}
    W = {k: v.to(torch_dtype) for k, v in W.items()}
    m = {"heads": heads, "kv_heads": 1, "dim": dim, "vdim": vdim, "scale": 1.0, "mask": {"size": window},
         "rot": {"dims": 0, "base": 1.0, "scaling": {"factor": 1.0}}}
    plain_w = {k[2:]: v.double() for k, v in W.items()}
    want = PD.window_attention_mixer(h.double(), plain_w, "", m, 1e-6)
    with PD.rounded():  # what rounding alone does to a softmax that hangs on few keys
        coarse = PD.window_attention_mixer(h.double(), plain_w, "", m, 1e-6)
    allowed = torch.maximum(3.0 * (coarse - want).abs().max(-1).values, 3e-2 * want.abs().max())
    for cuts in ([T], [T - 1, 1], [T - window, 1] + [1] * (window - 1), [7, 2, 30, 1, 1, 19]):
        part = MIXERS.build(spec, hidden_size=hidden)
        part.bind(W, "L", torch.device(DEV), torch_dtype)
        manager = CacheManager([part.cache_need()], 16, {group_name(window): 8}, 2)
        storage = CacheStorage(manager, torch.device(DEV), torch_dtype)
        manager.add_request("r")
        builder = BatchBuilder(torch.device(DEV), T, 2, {name: 8 for name in manager.groups})
        got, at = [], 0
        for n in cuts:
            manager.extend_all([("r", at + n)])
            tables = {name: [manager.table("r", name)] for name in manager.groups}
            step = builder.build([Portion("r", [0] * n, at)], tables, [manager.slot("r")])
            got.append(ops.as_tensor(part.forward(dev(h[at:at + n]), step, storage.views[0])).float().cpu())
            manager.commit("r", at + n)
            at += n
        if dtype == "float32":
            close(torch.cat(got), want, torch_dtype, f"cuts {cuts}", f32=1e-4)
        else:
            err = (torch.cat(got).double() - want).abs().max(-1).values
            assert bool((err <= allowed).all()), f"cuts {cuts}: rows {(err > allowed).nonzero().flatten().tolist()}"


# --------------------------------------------------------------------------
# through the engine: scheduler, batching, sampling
# --------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_through_the_entry_point(dafalix_dirs, name, dtype):
    """Five prompts for two places, prompts in portions of five tokens, a pool of two requests' worth: requests
    wait, pages and slots change hands.  Every token is the plain model's choice (in bf16: within the
    tolerance of its largest logit)."""
    import rvllm_amd

    folder = dafalix_dirs[name]
    weights, cfg = PD.load_weights(folder), PD.read_config(folder)
    prompts = [[3, 1, 4, 1, 5, 9, 2, 6, 5, 3, 5], [27, 18, 28], [7], [11, 12, 13, 14, 15, 16, 17], [90, 2]]
    outs = rvllm_amd.generate(str(folder), prompts, max_tokens=12, dtype=dtype, max_model_len=64, max_num_seqs=2,
                              max_num_batched_tokens=16, max_prefill_chunk=5, max_cache_tokens=128)
    for prompt, out in zip(prompts, outs):
        assert len(out) == 12
        logits = PD.forward(weights, cfg, prompt + out)
        scale = float(logits.abs().max())
        slack = 2 * tt.TOLERANCE[dtype] * scale
        calls = torch.zeros(len(prompt) + len(out), dtype=torch.bool)
        if dtype == "bfloat16":  # from a router's first close call on another expert may speak
            slack = max(slack, 6.0 * float(PD.rounding_error(weights, cfg, prompt + out, logits).max()))
            calls = PD.close_calls(weights, cfg, prompt + out)
        for j, token in enumerate(out):
            if bool(calls[:len(prompt) + j].any()):
                break
            row = logits[len(prompt) - 1 + j]
            assert row[token] >= row.max() - slack, f"token {j} of {prompt}"


def test_sampled_generation_runs_and_is_repeatable(dafalix_dirs):
    import rvllm_amd

    kw = dict(max_tokens=10, temperature=0.8, top_k=20, top_p=0.9, seed=4, dtype="bfloat16", max_model_len=64,
              max_num_seqs=3)
    prompts = [[1, 2, 3], [50, 60], [9, 9, 9, 9]]
    first = rvllm_amd.generate(str(dafalix_dirs["A"]), prompts, **kw)
    assert first == rvllm_amd.generate(str(dafalix_dirs["A"]), prompts, **kw)
    assert all(len(out) == 10 and all(0 <= t < 211 for t in out) for out in first)
