"""Dafalix configurations drawn at random against the plain implementation: 1-5 layers of either kind in any order,
with experts or none, a looped stretch anywhere or none, 1-5 streams; matrix memories of 1-6 heads with key sizes
4-140 and value sizes 4-96 and any cap; attention with 1-16 query heads a key/value head, key and value sizes 8-136
that are equal or not, windows of 1-150, rotations of none, a part or all of a head with any base and factor;
recurrent units of 8-200 channels in 1 to as many blocks, 1-5 taps; 1-20 experts of which 1 to all are chosen;
sequences of 1-260 tokens under the four cuttings, pages of 16 / 32 / 64, both dtypes.  Either dtype is held to the
larger of its flat share of the largest logit and three times the error that its rounding alone causes at the position
in the plain implementation (``plain_dafalix.rounding_error`` with bf16's roundings, ``float32_error`` for a run in
32-bit throughout: a matrix memory's read-out can all but cancel, and the norm behind it blows the remainder up).
Where a router's choice hangs on less than rounding moves it, the engine may choose another expert: its choices are
recorded, checked to be such close calls, and given to the plain implementation, so that every position is held to
the same measure.  A few seeds are committed; ``draw`` serves a longer run by hand."""

import json
import random

import numpy as np
import pytest

import plain_dafalix as PD
import tiny_dafalix
import trace_tools as tt
from rvllm_amd.config.engine_config import EngineConfig
from rvllm_amd.engine.runner import ModelRunner

pytestmark = pytest.mark.gpu


def draw(seed: int) -> dict:
    rng = random.Random(seed)
    eights = rng.random() < 0.6  # sizes the matrix-core kernels take, or any

    def size(lo, hi):
        return rng.randrange(lo, hi + 1, 8) if eights else rng.randint(lo, hi)

    def mlp():
        if rng.random() < 0.3:
            return None
        experts = rng.choice([1, 2, 3, 5, 8, 12, 20])
        return {"kind": "moe", "expert": {"ff": size(8, 120)},
                "router": {"experts": experts, "top": min(experts, rng.choice([1, 1, 2, experts, rng.randint(1, experts)]))}}

    layers = []
    for _ in range(rng.randint(1, 5)):
        if rng.random() < 0.5:
            layers.append({"type": "mlstm", "mlp": mlp(), "mixer": {
                "heads": rng.choice([1, 2, 3, 4, 6]), "dim": size(8, 136) if eights else rng.randint(4, 140),
                "vdim": size(8, 96) if eights else rng.randint(4, 96), "gate_cap": rng.choice([15.0, rng.uniform(1.0, 30.0)])}})
        else:
            kv_heads = rng.choice([1, 1, 2, 3, 4])
            heads = kv_heads * rng.choice([1, 2, 4, 8, 16] if kv_heads == 1 else [1, 2, 4])
            dim = rng.choice([16, 32, 48, 64, 96, 128]) if rng.random() < 0.6 else 2 * rng.randint(4, 68)
            vdim = rng.choice([dim, dim, rng.choice([16, 32, 64, 128]), 2 * rng.randint(4, 68)])
            dims = rng.choice([0, dim, 2 * rng.randint(1, dim // 2)])
            left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": rng.uniform(0.02, 0.4),
                    "mask": {"size": rng.choice([1, 2, 15, 16, 17, 33, rng.randint(3, 150)])},
                    "rot": {"dims": dims, "base": rng.choice([37.5, 10000.0, 1000000.0]),
                            "scaling": {"factor": rng.choice([1.0, 8.0, rng.uniform(0.5, 40.0)])}}}
            width = size(8, 200)
            blocks = rng.choice([b for b in (1, 2, 3, 4, 5, 8, width) if width % b == 0])
            right = {"width": width, "blocks": blocks, "conv": rng.randint(1, 5)}
            layers.append({"type": "parallel", "mlp": mlp(), "mixer": {
                "left": left, "right": right, "left_scale": rng.choice([1.0, rng.uniform(-1.5, 1.5)]),
                "right_scale": rng.choice([1.0, rng.uniform(0.2, 1.5)])}})
    doc = {"architecture": "Dafalix", "vocab": rng.randint(5, 700), "width": size(16, 160),
           "norm": {"eps": rng.choice([1e-6, 1e-5, 1e-3])}, "residual_mult": rng.choice([1.0, rng.uniform(0.2, 1.2)]),
           "streams": rng.choice([1, 2, 2, 3, 4, 5]), "layers": layers}
    if rng.random() < 0.7:
        start = rng.randint(0, len(layers) - 1)
        doc["loop"] = {"start": start, "stop": rng.randint(start, len(layers)), "times": rng.randint(1, 3)}
    return doc


@pytest.mark.parametrize("seed", [3, 7, 12, 19, 40, 46, 51, 65])
def test_a_configuration_drawn_at_random(tmp_path, seed):
    doc = draw(seed)
    tiny_dafalix.CONFIGS["random"] = (doc, seed)
    try:
        folder = tiny_dafalix.write_model(tmp_path / "m", "random", loud=seed % 2 == 0)
    finally:
        del tiny_dafalix.CONFIGS["random"]
    weights, cfg = PD.load_weights(folder), PD.read_config(folder)
    rng = random.Random(seed + 1000)
    lengths = [rng.choice([1, 2, 15, 16, 17, 33]), rng.randint(3, 120), rng.randint(100, 260)]
    seqs = tt.make_sequences(cfg["vocab"], lengths, seed=seed)
    measured: dict = {}
    page_size = rng.choice([16, 32, 64])
    for dtype in ("float32", "bfloat16"):
        for mode, make in (("whole", tt.trace_whole), ("tail", tt.trace_tail), ("portions", tt.trace_portions),
                           ("mixed", tt.trace_mixed)):
            steps = make(seqs, seed=seed) if mode in ("portions", "mixed") else make(seqs)
            most = max(tt.required_tokens(steps), page_size)
            runner = ModelRunner.from_model_dir(folder, EngineConfig(
                dtype=dtype, page_size=page_size, max_model_len=most, max_num_seqs=4, max_num_batched_tokens=most,
                max_prefill_chunk=most, max_cache_tokens=most, use_graphs=dtype != "bfloat16"))
            with tt.RecordedChoices() as choices:
                got = tt.collect(steps, tt.run_in_process(runner, steps, choices), cfg["vocab"])
            forced = choices.by_request(steps)
            prefix = steps[0]["entries"][0]["id"].split("-")[0]
            for name, ids in seqs.items():
                what = f"seed {seed} {dtype} {mode} {name}: {json.dumps(doc)}"
                # against the plain implementation with the experts that the engine chose (each a close call or the
                # plain choice); the allowance is three times what the dtype's rounding alone does at the position
                chosen = forced.get(f"{prefix}-{name}") or []
                key = (name, dtype, b"".join(c.tobytes() for c in chosen))
                if key not in measured:  # the cuttings mostly choose alike
                    ref = PD.forward(weights, cfg, ids, forced=chosen)
                    noise = (PD.rounding_error(weights, cfg, ids, ref, forced=chosen) if dtype == "bfloat16"
                             else PD.float32_error(weights, cfg, ids, ref, forced=chosen)).numpy()
                    measured[key] = (ref, noise)
                ref, noise = measured[key]
                allowed = np.maximum(tt.TOLERANCE[dtype] * float(ref.abs().max()), 3.0 * noise)
                tt.held_to_rounding(got[f"{prefix}-{name}"], ref, allowed, what)
