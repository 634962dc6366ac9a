"""Tarulix models of random shapes (layer order, head counts and sizes that are no multiple of eight, windows, block
lengths, rotated channels, taps, state places, expert counts with and without identity and shared experts, table
rows) through the engine on the GPU, in float32 and bfloat16, a whole prompt per step and a mixed schedule of portions
and decode tokens of two requests, against the float64 oracle."""

import os
import random
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, os.path.join(ROOT, "tests"))
import tarulix_oracle as O  # noqa: E402

from colossalai_amd.inference import ContinuousBatchEngine, InferenceConfig  # noqa: E402
from colossalai_amd.models import TarulixForCausalLM  # noqa: E402

pytestmark = pytest.mark.gpu


def random_config(rng):
    def attention():
        G = rng.choice([1, 2, 3, 4])
        a = dict(bias_max=rng.choice([20, 64, 100, 300]), dim=rng.choice([16, 24, 40, 64, 128]), heads=G * rng.choice([1, 2, 3, 4]),
                 kv_heads=G, mask=dict(size=rng.choice([5, 17, 64, 100, 1000])), v_mix=rng.random() < 0.7,
                 vdim=rng.choice([16, 24, 40, 64, 128]))
        a["scale"] = rng.choice([4.0, 8.0, 10.0]) / a["dim"]
        return a

    def parallel():
        G, D = rng.choice([1, 2, 4]), rng.choice([16, 32, 48, 64, 96, 128])
        left = dict(dim=D, heads=G * rng.choice([1, 2, 4]), kv_heads=G,
                    mask=dict(pool=rng.choice([1, 3, 8, 16, 32, 50]), size=rng.choice([4, 20, 33, 72, 130])),
                    rot=dict(base=rng.choice([100.0, 10000.0, 500000.0]), dims=rng.choice([2, D // 4 * 2, D])),
                    scale=rng.choice([4.0, 8.0, 10.0]) / D, softcap=rng.choice([5.0, 20.0, 50.0]),
                    vdim=rng.choice([16, 32, 56, 96, 128]))
        right = dict(conv=rng.choice([1, 2, 3, 4, 5]), dt_rank=rng.choice([1, 4, 7, 16]), inner=rng.choice([48, 100, 256]),
                     state=rng.choice([1, 4, 16, 20, 40]))
        return dict(left=left, right=right, left_scale=rng.choice([1.0, 0.6, 1.4]), right_scale=rng.choice([1.0, 0.3, 0.9]))

    def mlp():
        if rng.random() < 0.2:
            return None
        E, I = rng.choice([2, 4, 7, 8, 16]), rng.choice([0, 1, 2, 3])
        return dict(kind="moe", expert=dict(ff=rng.choice([8, 24, 32, 64, 100])),
                    router=dict(experts=E, identity=I, top=rng.randint(1, min(E + I, 5))),
                    shared=dict(ff=rng.choice([16, 40, 96])) if rng.random() < 0.8 else None)

    layers, mixed = [], None
    for _ in range(rng.randint(2, 5)):
        if rng.random() < 0.5:
            a = attention()
            if a["v_mix"]:
                if mixed is None:
                    mixed = (a["kv_heads"], a["vdim"])
                else:  # layers that mix values share the value sizes of the first
                    a["kv_heads"], a["vdim"] = mixed
                    a["heads"] = a["kv_heads"] * rng.choice([1, 2])
            layers.append(dict(type="attention", mixer=a, mlp=mlp()))
        else:
            layers.append(dict(type="parallel", mixer=parallel(), mlp=mlp()))
    return dict(architecture="Tarulix", vocab=rng.choice([50, 333]), width=rng.choice([64, 96, 160, 256]),
                norm=dict(eps=rng.choice([1e-6, 1e-5])), layers=layers)


def run(cfg, P, toks, dtype, plan):
    model = TarulixForCausalLM.from_checkpoint(cfg, P, dtype=dtype, device="cuda")
    eng = ContinuousBatchEngine(model, InferenceConfig(max_batch_size=4, dtype=dtype), num_blocks=64, block_size=16)
    outs, at = {k: [] for k in toks}, {k: 0 for k in toks}
    for step in plan:
        items = []
        for k, n in step:
            n = min(n, len(toks[k]) - at[k])
            if n > 0:
                items.append((k, toks[k][at[k] : at[k] + n], list(range(n))))
                at[k] += n
        if items:
            logits, o = eng.run_ragged(items), 0
            for k, t, _ in items:
                outs[k].append(logits[o : o + len(t)].float().cpu())
                o += len(t)
    assert all(at[k] == len(toks[k]) for k in toks)
    return {k: torch.cat(v) for k, v in outs.items()}


@pytest.mark.parametrize("seed", range(8))
def test_random_configuration(seed):
    rng = random.Random(seed)
    cfg = random_config(rng)
    P = {k: v.float() for k, v in O.random_checkpoint(cfg, seed, rel_rows=rng.choice([6, 9, 16, 20])).items()}
    g = torch.Generator().manual_seed(seed)
    toks = {"a": torch.randint(0, cfg["vocab"], (rng.choice([90, 150, 300]),), generator=g).tolist(),   # 300: the chunked scan
            "b": torch.randint(0, cfg["vocab"], (rng.choice([3, 40, 70]),), generator=g).tolist()}
    want = {k: O.forward(cfg, P, v).float() for k, v in toks.items()}
    whole = [[("a", 10 ** 6), ("b", 10 ** 6)]]
    mixed = ([[("a", 37)], [("a", 2), ("b", 5)], [("a", 64), ("b", 1)], [("a", 1), ("b", 30)], [("a", 130), ("b", 1)]]
             + [[("a", 1), ("b", 1)]] * 30 + [[("a", 10 ** 6), ("b", 2)], [("b", 10 ** 6)]])
    for dtype in (torch.float32, torch.bfloat16):
        for plan in (whole, mixed):
            got = run(cfg, P, toks, dtype, plan)
            err = torch.cat([(got[k] - want[k]).pow(2).mean(-1).sqrt() / want[k].pow(2).mean().sqrt() for k in toks])
            if dtype == torch.float32:
                assert err.max().item() < 3e-4, (cfg, err.max().item())
            else:  # single positions may sit on a close router call; most must be at rounding level
                assert err.median().item() < 0.03 and (err > 0.1).float().mean().item() < 0.1, (cfg, err.median().item())
