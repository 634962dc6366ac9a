"""The continuous-batching engine's ragged step on Tarulix (windowed attention over paged keys, block summaries in a
pool of their own, selective-scan state and convolution tails in slots, values shared between layers inside a step):
logits must not depend on how a prompt is cut, on what shares the step, or on which pages and slots are used. The
float64 oracle (tests/tarulix_oracle.py) gives the expected logits; bin/trace_run is run as a user runs it."""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, os.path.join(ROOT, "tests"))
import tarulix_oracle as O  # noqa: E402

from colossalai_amd.inference import ContinuousBatchEngine, GenerationConfig, InferenceConfig  # noqa: E402
from colossalai_amd.models import TarulixForCausalLM  # noqa: E402

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]

ATT = dict(bias_max=11, dim=8, heads=4, kv_heads=2, mask=dict(size=9), scale=0.9, v_mix=True, vdim=6)
LEFT = dict(dim=6, heads=4, kv_heads=2, mask=dict(pool=3, size=5), rot=dict(base=300.0, dims=4), scale=1.1, softcap=4.0,
            vdim=10)
RIGHT = dict(conv=3, dt_rank=2, inner=14, state=5)
MOE = dict(kind="moe", expert=dict(ff=12), router=dict(experts=5, identity=2, top=3), shared=dict(ff=6))
CFG = dict(architecture="Tarulix", vocab=40, width=24, norm=dict(eps=1e-5),
           layers=[dict(type="parallel", mixer=dict(left=LEFT, right=RIGHT, left_scale=0.7, right_scale=0.6), mlp=MOE),
                   dict(type="attention", mixer=ATT, mlp=MOE),
                   dict(type="parallel", mixer=dict(left=dict(LEFT, kv_heads=4, mask=dict(pool=6, size=4)),
                                                    right=dict(RIGHT, conv=4, state=3), left_scale=1.0, right_scale=0.4),
                        mlp=None),
                   dict(type="attention", mixer=dict(ATT, mask=dict(size=14)), mlp=MOE)])
P = {k: v.float() for k, v in O.random_checkpoint(CFG, seed=3).items()}
_oracle_cache = {}


def oracle(tokens):
    key = tuple(tokens)
    if key not in _oracle_cache:
        _oracle_cache[key] = O.forward(CFG, P, list(tokens)).float()
    return _oracle_cache[key]


def engine(device, slots=4, pages=64, page=4):
    model = TarulixForCausalLM.from_checkpoint(CFG, P, dtype=torch.float32, device=device)
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
    toks = prompt(36, 0)
    eng = engine(device)
    close(run_cut(eng, "a", toks, [12] + [1] * 24), oracle(toks))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cuts", [[2] * 18, [3, 2, 7, 2, 5, 17], [1, 35], [35, 1], [6] * 6, [4, 4, 8, 20], [5, 9, 3, 19]])
def test_portions_of_any_size(device, cuts):
    toks = prompt(36, 1)
    eng = engine(device)
    close(run_cut(eng, "a", toks, cuts), oracle(toks))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("page", [2, 16])
def test_first_tokens_one_by_one(device, page):
    toks = prompt(11, 2)
    eng = engine(device, page=page)
    close(run_cut(eng, "a", toks, [1] * 11), oracle(toks))


@pytest.mark.parametrize("device", DEVICES)
def test_unequal_requests_share_steps(device):
    """A prompt portion next to decode tokens of other requests, requests that sit out a step, and a late joiner."""
    A, B, C = prompt(30, 3), prompt(9, 4), prompt(19, 5)
    eng = engine(device)
    got = {"A": [], "B": [], "C": []}
    plan = [
        [("A", 7), ("B", 2)],
        [("A", 1), ("B", 5), ("C", 3)],
        [("C", 2)],
        [("A", 12), ("B", 1), ("C", 1)],
        [("A", 1), ("B", 1), ("C", 13)],
        [("A", 9)],
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
    """Two slots and a pool that holds two requests at most: later requests run in slots, pages and summary rows that
    earlier ones filled and gave back."""
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
    """Windows and block summaries pass over decoded tokens many times."""
    toks = prompt(110, 6)
    eng = engine(device)
    close(run_cut(eng, "a", toks, [4] + [1] * 106), oracle(toks), 5e-4)


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
def test_a_late_query_reads_far_tokens_through_summaries(device):
    """With sharp scores a query's weight sits on single keys and summaries; a prompt of many pages, whole, cut at
    page borders and inside pages, and decoded."""
    left = dict(LEFT, scale=5.0, softcap=50.0, mask=dict(pool=4, size=6))
    cfg = dict(CFG, layers=[dict(type="parallel", mixer=dict(left=left, right=RIGHT, left_scale=1.0, right_scale=0.1), mlp=None),
                            dict(type="attention", mixer=dict(ATT, scale=5.0, mask=dict(size=40), bias_max=30), mlp=None)])
    W = {k: v.float() for k, v in O.random_checkpoint(cfg, seed=12).items()}
    toks = torch.randint(0, 40, (150,), generator=torch.Generator().manual_seed(3)).tolist()
    want = O.forward(cfg, W, toks).float()
    for cuts in ([150], [64, 64, 22], [63, 2, 63, 1, 21], [128] + [1] * 22):
        model = TarulixForCausalLM.from_checkpoint(cfg, W, dtype=torch.float32, device=device)
        eng = ContinuousBatchEngine(model, InferenceConfig(max_batch_size=1, dtype=torch.float32), num_blocks=10,
                                    block_size=16)
        close(run_cut(eng, "a", toks, cuts), want, 5e-4)


@pytest.mark.gpu
def test_bfloat16_paths_agree_with_each_other_and_the_oracle():
    """bfloat16 serving: a whole prompt against the same prompt in small steps."""
    att = dict(bias_max=40, dim=32, heads=4, kv_heads=2, mask=dict(size=24), scale=0.2, v_mix=True, vdim=24)
    left = dict(dim=32, heads=4, kv_heads=2, mask=dict(pool=8, size=20), rot=dict(base=10000.0, dims=16), scale=0.2,
                softcap=20.0, vdim=32)
    right = dict(conv=4, dt_rank=4, inner=96, state=16)
    moe = dict(kind="moe", expert=dict(ff=32), router=dict(experts=6, identity=1, top=2), shared=dict(ff=32))
    cfg = dict(architecture="Tarulix", vocab=64, width=64, norm=dict(eps=1e-5),
               layers=[dict(type="attention", mixer=att, mlp=moe),
                       dict(type="parallel", mixer=dict(left=left, right=right, left_scale=0.9, right_scale=0.4), mlp=moe),
                       dict(type="attention", mixer=att, mlp=None)])
    W = {k: v.float() for k, v in O.random_checkpoint(cfg, seed=4).items()}
    toks = torch.randint(0, 64, (70,), generator=torch.Generator().manual_seed(9)).tolist()
    want = O.forward(cfg, W, toks).float()

    def run(cuts):
        model = TarulixForCausalLM.from_checkpoint(cfg, W, dtype=torch.bfloat16, device="cuda")
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
    """generate(): the engine's own scheduler cuts prompts into portions (token budget 8 per step) and batches them
    with decoding requests."""
    model = TarulixForCausalLM.from_checkpoint(CFG, P, dtype=torch.float32, device=device)
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
    """`models` names the architecture; `generate` loads the folder through the registry and decodes greedily through
    the engine's scheduler."""
    cfg, Wf, model_dir = checkpoint_folder(tmp_path)
    env = dict(os.environ, PYTHONPATH=ROOT, CUDA_VISIBLE_DEVICES="", HIP_VISIBLE_DEVICES="")
    cli = [sys.executable, "-m", "colossalai_amd.cli.cli"]
    r = subprocess.run(cli + ["models"], capture_output=True, text=True, env=env, timeout=300)
    assert r.returncode == 0 and "tarulix" in r.stdout.split()
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
