"""The continuous-batching engine's ragged step on Vitinex (latent attention over paged latents,
state-space layers with slots, a looped block whose passes keep caches of their own): logits must
not depend on how a prompt is cut, on what shares the step, or on which pages and slots are used.
The float64 oracle (tests/vitinex_oracle.py) gives the expected logits; bin/trace_run is run as a
user runs it."""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, os.path.join(ROOT, "tests"))
import vitinex_oracle as O  # noqa: E402

from colossalai_amd.inference import ContinuousBatchEngine, GenerationConfig, InferenceConfig  # noqa: E402
from colossalai_amd.models import VitinexForCausalLM  # noqa: E402

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]

LAT = dict(dim=8, heads=3, kv_rank=20, q_rank=12, rot=dict(base=1000.0, dims=6), rot_dim=6, scale=0.6, vdim=10)
SSM = dict(conv=3, groups=2, heads=4, norm_groups=2, state=10, vdim=6)
MOE = dict(kind="moe", expert=dict(ff=12), router=dict(experts=6, top=2), shared=dict(ff=6))
CFG = dict(architecture="Vitinex", vocab=40, width=24, norm=dict(eps=1e-5), residual_mult=0.5,
           loop=dict(start=1, stop=3, times=2),
           layers=[dict(type="mamba2", mixer=SSM, mlp=dict(kind="dense", ff=32)),
                   dict(type="latent_attention", mixer=LAT, mlp=MOE),
                   dict(type="mamba2", mixer=dict(SSM, groups=1, conv=4), mlp=None),
                   dict(type="latent_attention", mixer=dict(LAT, heads=2, scale=1.5), mlp=MOE)])
P = {k: v.float() for k, v in O.random_checkpoint(CFG, seed=3).items()}
_oracle_cache = {}


def oracle(tokens):
    key = tuple(tokens)
    if key not in _oracle_cache:
        _oracle_cache[key] = O.forward(CFG, P, list(tokens)).float()
    return _oracle_cache[key]


def engine(device, slots=4, pages=64, page=4):
    model = VitinexForCausalLM.from_checkpoint(CFG, P, dtype=torch.float32, device=device)
    return ContinuousBatchEngine(model, InferenceConfig(max_batch_size=slots, dtype=torch.float32),
                                 num_blocks=pages, block_size=page)


def prompt(n, seed):
    return torch.randint(0, CFG["vocab"], (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def close(got, want, tol=3e-4):
    err = (got.cpu().float() - want).abs().max().item()
    assert err <= tol * max(1.0, want.abs().max().item()), f"max abs error {err}"


def run_cut(eng, sid, toks, cuts):
    """Feed toks to sequence sid in portions of the given sizes; all logits."""
    out, at = [], 0
    for n in cuts:
        out.append(eng.run_ragged([(sid, toks[at : at + n], list(range(n)))]))
        at += n
    assert at == len(toks)
    return torch.cat(out, 0)


@pytest.mark.parametrize("device", DEVICES)
def test_prefill_then_token_by_token(device):
    toks = prompt(30, 0)
    eng = engine(device)
    close(run_cut(eng, "a", toks, [12] + [1] * 18), oracle(toks))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cuts", [[2] * 15, [3, 2, 7, 2, 5, 11], [1, 29], [29, 1], [5, 5, 5, 5, 5, 5], [4, 4, 8, 14]])
def test_portions_of_any_size(device, cuts):
    toks = prompt(30, 1)
    eng = engine(device)
    close(run_cut(eng, "a", toks, cuts), oracle(toks))


@pytest.mark.parametrize("device", DEVICES)
def test_first_tokens_one_by_one(device):
    toks = prompt(9, 2)
    eng = engine(device)
    close(run_cut(eng, "a", toks, [1] * 9), oracle(toks))


@pytest.mark.parametrize("device", DEVICES)
def test_unequal_requests_share_steps(device):
    """A prompt portion next to decode tokens of other requests, requests that
    sit out a step, and a late joiner."""
    A, B, C = prompt(26, 3), prompt(9, 4), prompt(17, 5)
    eng = engine(device)
    got = {"A": [], "B": [], "C": []}
    plan = [
        [("A", 7), ("B", 2)],
        [("A", 1), ("B", 5), ("C", 3)],
        [("C", 2)],
        [("A", 10), ("B", 1), ("C", 1)],
        [("A", 1), ("B", 1), ("C", 11)],
        [("A", 7)],
    ]
    src, at = {"A": A, "B": B, "C": C}, {"A": 0, "B": 0, "C": 0}
    for step in plan:
        items = []
        for name, n in step:
            items.append((name, src[name][at[name] : at[name] + n], list(range(n))))
            at[name] += n
        logits = eng.run_ragged(items)
        o = 0
        for name, n in step:
            got[name].append(logits[o : o + n])
            o += n
    for name in got:
        assert at[name] == len(src[name])
        close(torch.cat(got[name], 0), oracle(src[name]))


@pytest.mark.parametrize("device", DEVICES)
def test_pages_and_slots_are_used_again(device):
    """Two slots and a pool that holds two requests at most: later requests run
    in slots and pages that earlier ones filled and gave back."""
    eng = engine(device, slots=2, pages=12, page=4)
    reqs = [prompt(n, 10 + i) for i, n in enumerate([22, 13, 24, 5, 19])]
    first = eng.run_ragged([("r0", reqs[0], list(range(22))), ("r1", reqs[1][:6], list(range(6)))])
    close(first[:22], oracle(reqs[0]))
    eng.close_sequence("r0")
    assert eng.state.free_slots == 1
    second = eng.run_ragged([("r1", reqs[1][6:], list(range(7))), ("r2", reqs[2], list(range(24)))])
    close(torch.cat([first[22:], second[:7]], 0), oracle(reqs[1]))
    close(second[7:], oracle(reqs[2]))
    eng.close_sequence("r1")
    eng.close_sequence("r2")
    assert eng.kv.free_blocks == 12 and eng.state.free_slots == 2
    third = eng.run_ragged([("r3", reqs[3], list(range(5))), ("r4", reqs[4], list(range(19)))])
    close(third[:5], oracle(reqs[3]))
    close(third[5:], oracle(reqs[4]))
    with pytest.raises(AssertionError):
        eng.run_ragged([("r5", prompt(3, 99), [0])])  # no third slot


@pytest.mark.parametrize("device", DEVICES)
def test_long_decode_over_many_pages(device):
    toks = prompt(90, 6)
    eng = engine(device)
    close(run_cut(eng, "a", toks, [4] + [1] * 86), oracle(toks), 5e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_large_step_and_small_step_agree(device, monkeypatch):
    """A prompt long enough for the sorted per-expert products next to the same prompt in small steps
    (matrix-vector experts on the GPU)."""
    from colossalai_amd.ops import routed_experts

    monkeypatch.setattr(routed_experts, "GEMV_MAX_PAIRS", 64)
    monkeypatch.setattr(routed_experts, "GEMV_FALLBACK_PAIRS", 64)
    toks = prompt(120, 8)
    big = run_cut(engine(device), "a", toks, [120])
    small = run_cut(engine(device), "a", toks, [100] + [4] * 5)
    close(big, oracle(toks), 5e-4)
    close(small, oracle(toks), 5e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_a_late_query_reads_an_early_token(device):
    """With sharp scores (a large score scale) a query's weight sits on single keys far back, across many pages;
    whole, cut at page borders and inside pages, and decoded."""
    cfg = dict(CFG, layers=[dict(type="latent_attention", mixer=dict(LAT, scale=6.0), mlp=None),
                            dict(type="latent_attention", mixer=dict(LAT, scale=6.0, heads=1), mlp=None)], loop=None)
    cfg.pop("loop")
    W = {k: v.float() for k, v in O.random_checkpoint(cfg, seed=12).items()}
    toks = torch.randint(0, 40, (150,), generator=torch.Generator().manual_seed(3)).tolist()
    want = O.forward(cfg, W, toks).float()
    for cuts in ([150], [64, 64, 22], [63, 2, 63, 1, 21], [128] + [1] * 22):
        model = VitinexForCausalLM.from_checkpoint(cfg, W, dtype=torch.float32, device=device)
        eng = ContinuousBatchEngine(model, InferenceConfig(max_batch_size=1, dtype=torch.float32), num_blocks=10,
                                    block_size=16)
        close(run_cut(eng, "a", toks, cuts), want, 5e-4)


@pytest.mark.gpu
def test_bfloat16_paths_agree_with_each_other_and_the_oracle():
    """bfloat16 serving: a whole prompt against the same prompt in small steps."""
    lat = dict(dim=32, heads=4, kv_rank=64, q_rank=48, rot=dict(base=10000.0, dims=16), rot_dim=16, scale=0.15, vdim=24)
    ssm = dict(conv=4, groups=2, heads=4, norm_groups=2, state=16, vdim=16)
    moe = dict(kind="moe", expert=dict(ff=32), router=dict(experts=6, top=2), shared=dict(ff=32))
    cfg = dict(architecture="Vitinex", vocab=64, width=64, norm=dict(eps=1e-5), residual_mult=0.5,
               loop=dict(start=0, stop=2, times=2),
               layers=[dict(type="latent_attention", mixer=lat, mlp=moe),
                       dict(type="mamba2", mixer=ssm, mlp=dict(kind="dense", ff=96))])
    W = {k: v.float() for k, v in O.random_checkpoint(cfg, seed=4).items()}
    toks = torch.randint(0, 64, (70,), generator=torch.Generator().manual_seed(9)).tolist()
    want = O.forward(cfg, W, toks).float()

    def run(cuts):
        model = VitinexForCausalLM.from_checkpoint(cfg, W, dtype=torch.bfloat16, device="cuda")
        eng = ContinuousBatchEngine(model, InferenceConfig(max_batch_size=2, dtype=torch.bfloat16), num_blocks=16,
                                    block_size=16)
        return run_cut(eng, "a", toks, cuts).float().cpu()

    whole, stepped = run([70]), run([40] + [3] * 10)
    scale = want.pow(2).mean().sqrt()
    for got in (whole, stepped):
        err = (got - want).pow(2).mean(-1).sqrt() / scale
        assert err.median().item() < 0.03 and (err < 0.1).float().mean().item() > 0.8
    both = (whole - stepped).pow(2).mean(-1).sqrt() / scale
    assert both.median().item() < 0.03


@pytest.mark.parametrize("device", DEVICES)
def test_only_wanted_rows_come_back(device):
    toks = prompt(12, 7)
    eng = engine(device)
    got = eng.run_ragged([("a", toks, [11, 0, 5])])
    close(got, oracle(toks)[[11, 0, 5]])
    assert eng.run_ragged([("a", prompt(2, 8), [])]).shape[0] == 0


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_scheduler(device):
    """generate(): the engine's own scheduler cuts prompts into portions (token
    budget 8 per step) and batches them with decoding requests."""
    model = VitinexForCausalLM.from_checkpoint(CFG, P, dtype=torch.float32, device=device)
    eng = ContinuousBatchEngine(model, InferenceConfig(max_batch_size=2, max_input_len=64, max_output_len=8,
                                                       dtype=torch.float32),
                                num_blocks=40, block_size=4, max_step_tokens=8)
    prompts = [prompt(19, 20), prompt(3, 21), prompt(11, 22)]
    outs = eng.generate(prompts, GenerationConfig(max_new_tokens=5))
    for p, o in zip(prompts, outs):
        seq = list(p)
        for _ in range(5):
            seq.append(int(oracle(seq)[-1].argmax()))
        assert o == seq
    assert eng.kv.free_blocks == 40 and eng.state.free_slots == 2


def checkpoint_folder(tmp_path):
    """A checkpoint folder on disk, bfloat16 tensors as a checkpoint holds them."""
    from safetensors.torch import save_file

    cfg = dict(CFG, vocab=30)
    W = O.random_checkpoint(cfg, seed=11)
    model_dir = tmp_path / "model"
    model_dir.mkdir()
    (model_dir / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in W.items()}, str(model_dir / "model.safetensors"))
    return cfg, {k: v.float() for k, v in W.items()}, model_dir


def test_command_line_lists_and_generates(tmp_path):
    """`models` names the architecture; `generate` loads the folder through the
    registry and decodes greedily through the engine's scheduler."""
    cfg, Wf, model_dir = checkpoint_folder(tmp_path)
    env = dict(os.environ, PYTHONPATH=ROOT, CUDA_VISIBLE_DEVICES="", HIP_VISIBLE_DEVICES="")
    cli = [sys.executable, "-m", "colossalai_amd.cli.cli"]
    r = subprocess.run(cli + ["models"], capture_output=True, text=True, env=env, timeout=300)
    assert r.returncode == 0 and "vitinex" in r.stdout.split()
    r = subprocess.run(cli + ["generate", "--model", str(model_dir), "--prompt-ids", "3,9,27,1,4;5,6", "--max-new-tokens", "4",
                              "--dtype", "float32", "--max-step-tokens", "3"], capture_output=True, text=True, env=env,
                       timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [json.loads(l) for l in r.stdout.splitlines() if l.startswith("{")]
    assert [l["prompt_ids"] for l in lines] == [[3, 9, 27, 1, 4], [5, 6]]
    for l in lines:
        seq = list(l["prompt_ids"])
        for _ in range(4):
            seq.append(int(O.forward(cfg, Wf, seq)[-1].argmax()))
        assert l["output_ids"] == seq[len(l["prompt_ids"]):]


def test_replay_writes_the_oracles_logits(tmp_path):
    """bin/trace_run on a checkpoint folder on disk, float32 serving on the CPU."""
    cfg, Wf, model_dir = checkpoint_folder(tmp_path)
    out_dir = tmp_path / "out"
    a = torch.randint(0, 30, (21,), generator=torch.Generator().manual_seed(0)).tolist()
    b = torch.randint(0, 30, (9,), generator=torch.Generator().manual_seed(1)).tolist()
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:8], "want": [7]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[8:9], "want": []}, {"id": "b", "tokens": b[:9], "want": [0, 8]}],
         "end": ["b"]},
        {"step": 2, "entries": [{"id": "a", "tokens": a[9:], "want": [11, 2]}, {"id": "c", "tokens": b[:2], "want": [1]}],
         "end": ["a", "c"]},
    ]
    env = dict(os.environ, PYTHONPATH=ROOT)
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", str(model_dir), "--dtype", "float32",
                        "--out", str(out_dir), "--max-tokens", "64", "--device", "cpu"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, env=env,
                       timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    ya, yb = O.forward(cfg, Wf, a).float().numpy(), O.forward(cfg, Wf, b).float().numpy()
    got = {n: np.fromfile(out_dir / f"{n}.f32", dtype="<f4").reshape(-1, 30) for n in range(3)}
    np.testing.assert_allclose(got[0], ya[[7]], atol=3e-4)
    np.testing.assert_allclose(got[1], yb[[0, 8]], atol=3e-4)
    np.testing.assert_allclose(got[2], np.concatenate([ya[[20, 11]], yb[[1]]]), atol=3e-4)
