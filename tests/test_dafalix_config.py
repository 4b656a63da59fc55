"""The Dafalix design without a GPU: the configuration reader and its errors, the order in which a looped stretch of
layers runs, the tensors the model asks for, the needs its layers declare to the cache manager (every pass of a
looped layer its own), and pins on the plain implementation (``plain_dafalix``) that the GPU tests compare against."""

import copy
import math

import pytest
import torch

import plain_dafalix as PD
import tiny_dafalix
from rvllm_amd.cache.manager import CacheManager
from rvllm_amd.config.dafalix import DafalixConfig
from rvllm_amd.config.errors import ConfigError
from rvllm_amd.models import DecoderModel
from rvllm_amd.models.registry import architecture_of
from rvllm_amd.parts.base import KVNeed, StateNeed
from rvllm_amd.parts.spec import ScheduleEntry


def model_of(doc):
    return DecoderModel(architecture_of(doc).build_spec(DafalixConfig.from_dict(doc)))


@pytest.mark.parametrize("name", list(tiny_dafalix.CONFIGS))
def test_the_reader_takes_every_size_from_the_file_and_writes_it_back(name):
    doc = tiny_dafalix.CONFIGS[name][0]
    arch = architecture_of(doc)
    cfg = arch.read_config(doc, "test")
    assert isinstance(cfg, DafalixConfig) and arch.write_config(cfg) == doc
    assert [layer.type for layer in cfg.layers] == [layer["type"] for layer in doc["layers"]]


def test_every_problem_of_a_file_is_reported_at_once():
    doc = copy.deepcopy(tiny_dafalix.CONFIG_A)
    doc["vocab"] = 0
    del doc["norm"]
    doc["streams"] = 0
    doc["loop"] = {"start": 3, "stop": 9, "times": 2}
    doc["layers"][0]["mixer"]["gate_cap"] = -1.0
    doc["layers"][0]["mlp"]["router"]["top"] = 6            # of 5 experts
    doc["layers"][1]["mixer"]["left"]["heads"] = 3          # not a multiple of kv_heads 2
    doc["layers"][1]["mixer"]["right"]["blocks"] = 5        # 48 channels
    doc["layers"][2]["type"] = "conv"
    doc["layers"][3]["mixer"]["left"]["rot"]["dims"] = 7
    doc["layers"][3]["mlp"] = {"kind": "dense"}
    with pytest.raises(ConfigError) as e:
        DafalixConfig.from_dict(doc, "test")
    text = str(e.value)
    for piece in ("vocab", "norm", "streams", "loop", "layers[0]", "gate_cap", "top=6", "layers[1]", "kv_heads",
                  "blocks", "layers[2]", "unknown mixer type", "layers[3]", "rot.dims", "unknown kind"):
        assert piece in text, piece


def test_what_a_file_may_leave_out():
    doc = copy.deepcopy(tiny_dafalix.CONFIG_A)
    del doc["loop"]
    del doc["layers"][1]["mixer"]["left"]["rot"]["scaling"]
    cfg = DafalixConfig.from_dict(doc)
    assert cfg.loop is None and cfg.layer_runs() == [(0, 0), (1, 0), (2, 0), (3, 0)]
    assert cfg.layers[1].mixer.left.rot_factor == 1.0


def test_a_looped_stretch_runs_in_a_row_and_every_pass_has_a_cache_of_its_own():
    cfg = DafalixConfig.from_dict(tiny_dafalix.CONFIG_A)
    assert cfg.layer_runs() == [(0, 0), (1, 0), (2, 0), (1, 1), (2, 1), (3, 0)]
    assert [i for i, _ in cfg.layer_runs()] == PD.layer_runs(tiny_dafalix.CONFIG_A)
    model = model_of(tiny_dafalix.CONFIG_A)
    assert model.spec.schedule[3] == ScheduleEntry(1, copy=1)
    assert model.cache_index == {(0, 0): 0, (1, 0): 1, (2, 0): 2, (3, 0): 3, (1, 1): 4, (2, 1): 5}
    needs = model.cache_needs()
    assert len(needs) == 6 and needs[4] == needs[1] and needs[5] == needs[2]
    whole = model_of(tiny_dafalix.CONFIG_C)  # the loop starts at the first layer
    assert [(e.layer, e.copy) for e in whole.spec.schedule] == [(0, 0), (1, 0), (0, 1), (1, 1), (2, 0)]
    once = copy.deepcopy(tiny_dafalix.CONFIG_A)
    once["loop"] = {"start": 2, "stop": 2, "times": 5}  # an empty stretch
    assert DafalixConfig.from_dict(once).layer_runs() == [(0, 0), (1, 0), (2, 0), (3, 0)]


def test_the_model_asks_for_the_designs_tensors():
    shapes = {s.name: tuple(s.shape) for s in model_of(tiny_dafalix.CONFIG_A).param_specs()}
    assert shapes["embed"] == (211, 64) and shapes["final.norm"] == (64,) and shapes["final.norm.b"] == (64,)
    assert "head" not in shapes  # the head is the embedding table
    # a matrix memory with experts: two norms with biases, two scales, two connections of three streams
    for name, shape in {"l0.norm1": (64,), "l0.norm1.b": (64,), "l0.norm2": (64,), "l0.norm2.b": (64,), "l0.ls1": (64,),
                        "l0.ls2": (64,), "l0.hc1.in": (3,), "l0.hc1.out": (3,), "l0.hc1.mix": (3, 3), "l0.hc2.mix": (3, 3),
                        "l0.mix.q": (32, 64), "l0.mix.k": (32, 64), "l0.mix.v": (48, 64), "l0.mix.g": (48, 64),
                        "l0.mix.i": (2, 64), "l0.mix.i.b": (2,), "l0.mix.f": (2, 64), "l0.mix.f.b": (2,),
                        "l0.mix.norm": (48,), "l0.mix.o": (64, 48), "l0.mlp.router": (5, 64),
                        "l0.mlp.e4.gate": (32, 64), "l0.mlp.e4.up": (32, 64), "l0.mlp.e0.down": (64, 32)}.items():
        assert shapes[name] == shape, name
    assert "l0.mlp.e5.gate" not in shapes and "l0.mlp.table" not in shapes
    # a parallel layer: values of their own size, norm weights of the keys' size, block-diagonal gates
    for name, shape in {"l1.mix.left.q": (128, 64), "l1.mix.left.k": (64, 64), "l1.mix.left.v": (32, 64),
                        "l1.mix.left.o": (64, 64), "l1.mix.left.q.norm": (32,), "l1.mix.left.k.norm": (32,),
                        "l1.mix.right.y": (48, 64), "l1.mix.right.y.b": (48,), "l1.mix.right.x": (48, 64),
                        "l1.mix.right.x.b": (48,), "l1.mix.right.conv": (48, 3), "l1.mix.right.conv.b": (48,),
                        "l1.mix.right.ra": (3, 16, 16), "l1.mix.right.ra.b": (3, 16), "l1.mix.right.ri": (3, 16, 16),
                        "l1.mix.right.ri.b": (3, 16), "l1.mix.right.lam": (48,), "l1.mix.right.o": (64, 48),
                        "l3.mix.left.v": (32, 64), "l3.mix.left.o": (64, 192)}.items():
        assert shapes[name] == shape, name
    # a layer without a feed-forward: the first sublayer's tensors only
    assert not {"l2.norm2", "l2.norm2.b", "l2.ls2", "l2.hc2.in", "l2.mlp.router"} & set(shapes)


def test_a_layer_may_need_pages_and_a_state_at_once():
    model = model_of(tiny_dafalix.CONFIG_A)
    needs = model.cache_needs()
    # a head is held at the larger of its key and value sizes
    assert needs[1][0] == KVNeed(2, 32, 21) and needs[3][0] == KVNeed(1, 32, 5)
    # the convolution's rows and the unit's state; S, n and m of every head
    assert needs[1][1] == StateNeed(((3 - 1) * 48 + 48,), torch.float32)
    assert needs[0] == StateNeed((2 * 16 * 24 + 2 * 16 + 2,), torch.float32)
    manager = CacheManager(needs, 16, 8, 3)
    assert set(manager.groups) == {"window21", "window5"} and manager.state_layers == [0, 1, 2, 3, 4, 5]
    assert manager.groups["window21"].layers == [1, 4]
    a = manager.add_request("a")
    manager.extend("a", 40)
    manager.commit("a", 40)
    manager.release("a")
    assert manager.add_request("b").slot == a.slot
    manager.check()


# ---- pins on the plain implementation ------------------------------------------------------------------------
def test_plain_layer_norm_takes_the_mean_off_and_divides_by_the_deviation():
    x = torch.tensor([[1.0, 3.0, 5.0, 7.0]], dtype=PD.F)
    w, b = torch.tensor([1.0, 2.0, 1.0, 1.0], dtype=PD.F), torch.tensor([0.0, 0.0, 0.0, 10.0], dtype=PD.F)
    sd = math.sqrt(5.0)
    assert torch.allclose(PD.layer_norm(x, 0.0, w, b), torch.tensor([[-3 / sd, -2 / sd, 1 / sd, 3 / sd + 10.0]], dtype=PD.F))


def test_plain_convolution_sees_the_token_itself_last_and_zeros_before_the_start():
    x = torch.tensor([[1.0], [10.0], [100.0], [1000.0]], dtype=PD.F)
    w = torch.tensor([[3.0, 2.0, 1.0]], dtype=PD.F)  # the last tap is the token's own
    assert PD.causal_conv(x, w, torch.tensor([0.5], dtype=PD.F)).flatten().tolist() == [1.5, 12.5, 123.5, 1230.5]


def test_plain_matrix_memory_starts_its_maximum_at_zero():
    """A first token with a log input gate below zero is taken with e^i, not with 1: the running maximum starts at 0."""
    k = torch.tensor([[1.0, 0.0]], dtype=PD.F)
    v = torch.tensor([[4.0]], dtype=PD.F)
    q = torch.tensor([[1.0, 0.0]], dtype=PD.F)
    log_in, log_forget = torch.tensor([-2.0], dtype=PD.F), torch.tensor([-0.1], dtype=PD.F)
    o = PD.matrix_memory_recurrence(q, k, v, log_in, log_forget)
    # m' = max(-0.1 + 0, -2) = -0.1; take = e^(-1.9); S = take * 4, n . q = take; divisor max(take, e^0.1) + 1e-6
    take = math.exp(-1.9)
    assert abs(float(o) - take * 4.0 / (math.exp(0.1) + 1e-6)) < 1e-12
    # a large gate later: the answer is the value itself, whatever the exponentials' size
    k2 = torch.tensor([[1.0, 0.0], [0.0, 1.0]], dtype=PD.F)
    v2 = torch.tensor([[4.0], [7.0]], dtype=PD.F)
    o2 = PD.matrix_memory_recurrence(k2, k2, v2, torch.tensor([-2.0, 300.0], dtype=PD.F), torch.tensor([-0.1, -0.1], dtype=PD.F))
    assert abs(float(o2[1]) - 7.0) < 1e-4


def test_plain_recurrent_unit_has_no_special_first_token():
    u = torch.ones(3, 1, dtype=PD.F)
    half = torch.full((3, 1), 0.5, dtype=PD.F)
    lam = torch.zeros(1, dtype=PD.F)
    S = PD.gated_linear_recurrence(u, half, half, lam).flatten().tolist()
    a = math.exp(-8.0 * 0.5 * math.log(2.0))
    x = math.sqrt(1.0 - a * a) * 0.5
    assert abs(S[0] - x) < 1e-12 and abs(S[1] - (a * x + x)) < 1e-12 and abs(S[2] - (a * (a * x + x) + x)) < 1e-12
    mats = torch.tensor([[[1.0, 0.0], [1.0, 1.0]], [[2.0, 0.0], [0.0, 3.0]]], dtype=PD.F)  # [out, in] in every block
    got = PD.block_diagonal(torch.tensor([[1.0, 2.0, 3.0, 4.0]], dtype=PD.F), mats, torch.zeros(2, 2, dtype=PD.F))
    assert got.flatten().tolist() == [1.0, 3.0, 6.0, 12.0]


def test_plain_experts_weigh_their_input_and_do_not_renormalize():
    W = {"router": torch.tensor([[10.0, 0.0], [0.0, 0.0], [-10.0, 0.0]], dtype=PD.F)}
    for e in range(3):
        W[f"e{e}.gate"] = torch.eye(2, dtype=PD.F) * (e + 1)
        W[f"e{e}.up"] = torch.eye(2, dtype=PD.F)
        W[f"e{e}.down"] = torch.eye(2, dtype=PD.F)
    h = torch.tensor([[1.0, 2.0]], dtype=PD.F)
    got = PD.routed_experts(h, W, "", {"router": {"experts": 3, "top": 2}})
    want = torch.zeros(1, 2, dtype=PD.F)
    for e, score in ((0, torch.sigmoid(torch.tensor(10.0, dtype=PD.F))), (1, torch.tensor(0.5, dtype=PD.F))):
        x = score * h
        want += PD.silu(x * (e + 1)) * x
    assert torch.allclose(got, want)


def test_plain_window_rotation_and_scaled_frequencies():
    T, d = 9, 4
    g = torch.Generator().manual_seed(0)
    q = torch.randn(T, 1, d, generator=g, dtype=PD.F)
    k = torch.randn(T, 1, d, generator=g, dtype=PD.F)
    v = torch.eye(T, dtype=PD.F)[:, None, :]  # value j is the j-th unit vector: the output is the weights themselves
    w = PD.window_softmax_attention(q, k, v, 1.0, 3)[:, 0]
    for i in range(T):
        seen = [j for j in range(T) if w[i, j] > 0]
        assert seen == list(range(max(0, i - 2), i + 1)) and abs(float(w[i].sum()) - 1.0) < 1e-12
    x = torch.randn(T, 2, 6, generator=g, dtype=PD.F)
    r = PD.rotate_halves(x, torch.arange(T), 4, 100.0, 2.0)
    assert torch.equal(r[..., 4:], x[..., 4:]) and torch.allclose(r.norm(dim=-1), x.norm(dim=-1))
    assert torch.equal(r[0], x[0])  # position 0 turns nothing
    ang = torch.tensor(5 * 100.0 ** (-2.0 * 1 / 4) / 2.0)  # every frequency divided by the factor
    assert torch.allclose(r[5, 0, 1], x[5, 0, 1] * torch.cos(ang) - x[5, 0, 3] * torch.sin(ang))
    assert torch.allclose(r[5, 0, 3], x[5, 0, 3] * torch.cos(ang) + x[5, 0, 1] * torch.sin(ang))
    # position 2p with factor 2 is position p with factor 1
    assert torch.allclose(PD.rotate_halves(x, 2 * torch.arange(T), 4, 100.0, 2.0), PD.rotate_halves(x, torch.arange(T), 4, 100.0, 1.0))
