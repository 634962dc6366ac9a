"""Vitinex against the float64 oracle (tests/vitinex_oracle.py): every mechanism alone, then whole
models of several shapes, on the CPU (reference path of every op) and on the GPU (HIP kernels)."""

import copy
import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, os.path.join(ROOT, "tests"))
import vitinex_oracle as O  # noqa: E402

from colossalai_amd.inference.kv_cache import KVCacheManager  # noqa: E402
from colossalai_amd.inference.state_cache import StateCacheManager  # noqa: E402
from colossalai_amd.models import VitinexForCausalLM, model_class_for  # noqa: E402
from colossalai_amd.ops import group_norm, latent_attention, linear_recurrence, pair_rotary, routed_experts, short_conv  # noqa: E402
from colossalai_amd.ops.activation import gelu_tanh_mul  # noqa: E402
from colossalai_amd.ops.ragged import RaggedBatch  # noqa: E402

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
F64 = torch.float64

LAT = dict(dim=10, heads=3, kv_rank=24, q_rank=14, rot=dict(base=10000.0, dims=6), rot_dim=6, scale=0.3, vdim=12)
SSM = dict(conv=3, groups=1, heads=4, norm_groups=2, state=12, vdim=6)
MOE = dict(kind="moe", expert=dict(ff=12), router=dict(experts=7, top=3), shared=dict(ff=10))


def cfg_of(layers, loop=None, width=28, vocab=50, mult=0.4, eps=1e-5):
    c = dict(architecture="Vitinex", layers=layers, norm=dict(eps=eps), residual_mult=mult, vocab=vocab, width=width)
    if loop is not None:
        c["loop"] = loop
    return c


SHAPES = {
    # a looped middle block, every feed-forward kind, a layer without one
    "looped_middle": cfg_of([dict(type="mamba2", mixer=SSM, mlp=dict(kind="dense", ff=20)),
                             dict(type="latent_attention", mixer=LAT, mlp=MOE),
                             dict(type="mamba2", mixer=dict(SSM, groups=2, norm_groups=1, conv=2), mlp=None),
                             dict(type="latent_attention", mixer=dict(LAT, heads=2, vdim=5, rot_dim=8), mlp=dict(kind="dense", ff=9))],
                            loop=dict(start=1, stop=3, times=3)),
    # no loop at all; groups = heads, one expert chosen, no shared expert, one tap, part of the rotated channels fixed
    "plain": cfg_of([dict(type="latent_attention", mixer=dict(LAT, rot=dict(base=50.0, dims=4)),
                          mlp=dict(kind="moe", expert=dict(ff=6), router=dict(experts=3, top=1))),
                     dict(type="mamba2", mixer=dict(SSM, groups=4, norm_groups=4, conv=1, heads=4), mlp=MOE)], width=20),
    # the whole model is the loop, run once; a loop from layer 0 run twice follows
    "loop_once": cfg_of([dict(type="mamba2", mixer=dict(SSM, heads=2, groups=2, state=5, vdim=3, norm_groups=3), mlp=None),
                         dict(type="latent_attention", mixer=dict(LAT, heads=1, kv_rank=9, q_rank=5, dim=3), mlp=None)],
                        loop=dict(start=0, stop=2, times=1), width=18, mult=1.0),
    "loop_head": cfg_of([dict(type="latent_attention", mixer=LAT, mlp=dict(kind="dense", ff=16)),
                         dict(type="mamba2", mixer=SSM, mlp=MOE)], loop=dict(start=0, stop=1, times=2), width=24),
}


def close(got, want, tol=3e-4):
    got, want = got.detach().cpu().to(F64), want.to(F64)
    err = (got - want).abs().max().item()
    assert err <= tol * max(1.0, want.abs().max().item()), f"max abs error {err}"


def one_sequence(T, device, page=4, start=0, pages_first=0):
    pages = (start + T + page - 1) // page
    table = list(range(pages_first + pages - 1, pages_first - 1, -1))
    return RaggedBatch.build([T], [start], [0], device, [table], page), pages_first + pages


# ------------------------------------------------------------------- mechanisms alone
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("W", [20, 64, 200])
def test_centred_norm_in_and_out(device, W):
    g = torch.Generator().manual_seed(W)
    x, y = torch.randn(9, W, generator=g) * 2 + 1.5, torch.randn(9, W, generator=g) - 0.7
    w_out, w_next = torch.randn(W, generator=g), torch.randn(W, generator=g)
    want_x = x.to(F64) + 0.3 * O.layer_norm(y.to(F64), w_out, 1e-5)
    xr = x.clone().to(device)
    h = group_norm.add_layer_norm(xr, y.to(device), w_out.to(device), 0.3, w_next.to(device), 1e-5, torch.float32)
    close(xr, want_x, 1e-5)
    close(h, O.layer_norm(want_x, w_next, 1e-5), 1e-5)
    close(group_norm.layer_norm(x.to(device), w_next.to(device), 1e-5), O.layer_norm(x.to(F64), w_next, 1e-5), 1e-5)
    # a row of equal entries has no deviation: eps alone keeps the root apart from zero
    flat = torch.full((2, W), 3.25)
    assert float(group_norm.layer_norm(flat.to(device), w_next.to(device), 1e-5).abs().max()) < 1e-3


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("R,dims,base", [(6, 6, 10000.0), (8, 4, 50.0), (16, 16, 250000.0)])
def test_pair_rotation(device, R, dims, base):
    g = torch.Generator().manual_seed(R)
    x = torch.randn(11, 3, R, generator=g)
    pos = torch.tensor([0, 1, 2, 3, 15, 16, 17, 255, 256, 1000, 4095], dtype=torch.int32)
    f = pair_rotary.pair_frequencies(base, dims)
    got = pair_rotary.rotate_pairs(x.to(device), pos.to(device), f.to(device))
    close(got, O.rotate_pairs(x.to(F64), pos, base, dims), 5e-4)
    assert torch.equal(got[0].cpu(), x[0])  # position 0 turns nothing


def latent_inputs(T, c, seed, spike=None):
    """Random projections of T tokens; with ``spike=(i, j)`` query i's plain part points at key j's."""
    g = torch.Generator().manual_seed(seed)
    H, D, R, Dv, rank = c["heads"], c["dim"], c["rot_dim"], c["vdim"], c["kv_rank"]
    q = torch.randn(T, H, D + R, generator=g)
    dkv = torch.randn(T, rank + R, generator=g)
    w_uk, w_uv = torch.randn(H * D, rank, generator=g) / rank ** 0.5, torch.randn(H * Dv, rank, generator=g) / rank ** 0.5
    norm_w = 1 + 0.1 * torch.randn(rank, generator=g)
    gate = torch.randn(T, H, generator=g)
    if spike is not None:
        i, j = spike
        lat_j = O.rms_unit(dkv[j : j + 1, :rank].to(F64), 1e-5) * norm_w.to(F64)
        q[i, :, :D] = 12.0 * O.lin(lat_j, w_uk).view(H, D).float()
    return q, dkv, w_uk, w_uv, norm_w, gate


def oracle_latent(q, dkv, w_uk, w_uv, norm_w, gate, c, pos):
    D, rank = c["dim"], c["kv_rank"]
    lat = O.rms_unit(dkv[:, :rank].to(F64), 1e-5) * norm_w.to(F64)
    k_rot = O.rotate_pairs(dkv[:, rank:].to(F64), pos, c["rot"]["base"], c["rot"]["dims"])
    q_rot = O.rotate_pairs(q[..., D:].to(F64), pos, c["rot"]["base"], c["rot"]["dims"])
    o = O.latent_attention_core(q[..., :D].to(F64), q_rot, lat, k_rot, w_uk, w_uv, c["scale"], pos, pos)
    return (o * torch.sigmoid(gate.to(F64))[:, :, None]).reshape(q.shape[0], -1)


def framework_latent(q, dkv, w_uk, w_uv, norm_w, gate, c, device, cuts, page=4):
    """The framework's ops on one sequence fed in portions of the sizes ``cuts``."""
    H, D, R, Dv, rank = c["heads"], c["dim"], c["rot_dim"], c["vdim"], c["kv_rank"]
    T = q.shape[0]
    f = pair_rotary.pair_frequencies(c["rot"]["base"], c["rot"]["dims"]).to(device)
    pool = torch.full(((T + page - 1) // page + 2, page, 1, rank + R), float("nan"), device=device)
    table = list(range(pool.shape[0] - 1, -1, -1))
    out, at = [], 0
    for n in cuts:
        batch = RaggedBatch.build([n], [at], [0], device, [table[: (at + n + page - 1) // page]], page)
        sl = slice(at, at + n)
        latent_attention.latent_kv_write(dkv[sl].to(device), norm_w.to(device), 1e-5, f, pool, batch)
        out.append(latent_attention.latent_attention(q[sl].to(device), w_uk.view(H, D, rank).to(device),
                                                     w_uv.view(H, Dv, rank).to(device), pool, batch, c["scale"], f, rank,
                                                     gate[sl].to(device)))
        at += n
    return torch.cat(out, 0)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("c", [LAT, dict(LAT, heads=5, dim=4, vdim=3, kv_rank=16, rot_dim=8, rot=dict(base=77.0, dims=8))])
def test_latent_attention_alone(device, c):
    T = 37
    args = latent_inputs(T, c, 1)
    want = oracle_latent(*args, c, torch.arange(T))
    close(framework_latent(*args, c, device, [T]), want)
    close(framework_latent(*args, c, device, [20] + [1] * 17), want)
    close(framework_latent(*args, c, device, [2, 3, 5, 2, 9, 16]), want)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("far", [0, 1, 3, 4, 63, 64, 127, 128, 300, 417, 418])
def test_one_key_far_back_takes_the_weight(device, far):
    """Among several hundred keys the last query's score stands out at one place: the first tokens, both sides of
    a page border, the query itself. In a prompt portion and as a decoded token."""
    T, c = 419, dict(LAT, scale=1.0, dim=32, kv_rank=48)
    args = latent_inputs(T, c, 2, spike=(T - 1, far))
    want = oracle_latent(*args, c, torch.arange(T))
    lat = O.rms_unit(args[1][:, : c["kv_rank"]].to(F64), 1e-5) * args[4].to(F64)
    value_far = (O.lin(lat[far : far + 1], args[3]).view(c["heads"], -1) * torch.sigmoid(args[5][T - 1].to(F64))[:, None])
    assert (want[T - 1] - value_far.reshape(-1)).abs().max() < 1e-3, "the test's spike does not stand out"
    close(framework_latent(*args, c, device, [T], page=64)[T - 1], want[T - 1])          # in a prompt
    close(framework_latent(*args, c, device, [T - 1, 1], page=64)[T - 1], want[T - 1])   # decoded alone
    close(framework_latent(*args, c, device, [400, 19], page=64)[T - 1], want[T - 1])    # in a later portion


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,G,N,V,K", [(4, 1, 12, 6, 3), (4, 4, 5, 3, 1), (6, 3, 16, 8, 4), (3, 3, 9, 7, 2)])
def test_convolution_and_state_space_scan(device, H, G, N, V, K):
    """conv + silu + scan on one sequence whole, token by token and in odd portions, through slots whose contents
    are garbage before the first token."""
    T = 41
    g = torch.Generator().manual_seed(H * 100 + N)
    inner, C = H * V, H * V + 2 * G * N
    xbc_in = torch.randn(T, C, generator=g)
    dt_raw = torch.randn(T, H, generator=g) * 2
    taps, bias = torch.randn(C, K, generator=g) * 0.5, torch.randn(C, generator=g) * 0.2
    A_log, dt_bias, skip = torch.randn(H, generator=g) * 0.5, torch.randn(H, generator=g), torch.randn(H, generator=g)
    conv, _ = O.causal_conv(xbc_in.to(F64), taps, bias)
    conv = O.silu(conv)
    dt = O.softplus(dt_raw.to(F64) + dt_bias.to(F64))
    want, S_end = O.ssd_scan(conv[:, :inner].reshape(T, H, V), conv[:, inner : inner + G * N].reshape(T, G, N),
                             conv[:, inner + G * N:].reshape(T, G, N), dt, A_log, skip, G)
    for cuts in ([T], [1] * T, [2, 7, 1, 16, 2, 13]):
        state = torch.full((2, H, N, V), 1e3, device=device)
        tail = torch.full((2, max(K - 1, 1), C), -1e3, device=device)[:, : K - 1]
        out, at = [], 0
        for n in cuts:
            batch = RaggedBatch.build([n], [at], [1], device)
            xbc = short_conv.short_conv(xbc_in[at : at + n].to(device), taps.to(device), tail if K > 1 else None, batch,
                                        True, torch.float32, bias.to(device))
            out.append(linear_recurrence.ssd_recurrence(
                xbc[:, :inner].view(n, H, V), xbc[:, inner : inner + G * N].view(n, G, N),
                xbc[:, inner + G * N:].view(n, G, N), dt_raw[at : at + n].to(device), A_log.to(device),
                dt_bias.to(device), skip.to(device), state, batch))
            at += n
        close(torch.cat(out, 0), want, 2e-4)
        close(state[1], S_end, 2e-4)
        assert float(state[0].min()) == 1e3  # the other slot is untouched


@pytest.mark.parametrize("device", DEVICES)
def test_large_steps_are_not_clamped(device):
    """softplus of a large argument is the argument itself: the decay then wipes the state."""
    H, N, V = 2, 4, 3
    batch = RaggedBatch.build([3], [0], [0], device)
    x, B, C = torch.ones(3, H, V, device=device), torch.ones(3, 1, N, device=device), torch.ones(3, 1, N, device=device)
    dt_raw = torch.tensor([[0.0, 0.0], [40.0, -40.0], [0.0, 0.0]], device=device)
    zeros = torch.zeros(H, device=device)
    state = torch.zeros(1, H, N, V, device=device)
    y = linear_recurrence.ssd_recurrence(x, B, C, dt_raw, zeros, zeros, zeros, state, batch)
    dt = O.softplus(dt_raw.cpu().to(F64))
    want, _ = O.ssd_scan(x.cpu().to(F64), B.cpu().to(F64), C.cpu().to(F64), dt, zeros.cpu(), zeros.cpu(), 1)
    close(y, want, 1e-5)
    assert abs(float(y[1, 0, 0]) - 40.0 * N) < 1e-2 and abs(float(y[1, 1, 0]) - float(want[1, 1, 0])) < 1e-5


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("groups", [1, 2, 5])
def test_gate_comes_before_the_grouped_norm(device, groups):
    g = torch.Generator().manual_seed(groups)
    y, z, w = torch.randn(7, 40, generator=g), torch.randn(7, 40, generator=g) * 2, torch.randn(40, generator=g)
    want = O.rms_unit((y.to(F64) * O.silu(z.to(F64))).view(7, groups, -1), 1e-5).reshape(7, 40) * w.to(F64)
    close(group_norm.gated_grouped_rms_norm(y.to(device), z.to(device), w.to(device), groups, 1e-5, torch.float32), want, 1e-5)


@pytest.mark.parametrize("device", DEVICES)
def test_dense_feed_forward_activation(device):
    g = torch.Generator().manual_seed(0)
    packed = torch.randn(9, 2 * 21, generator=g) * 3
    want = O.gelu_tanh(packed[:, :21].to(F64)) * packed[:, 21:].to(F64)
    close(gelu_tanh_mul(packed.to(device)), want, 1e-5)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("E,top,shared", [(7, 3, True), (3, 1, False), (12, 12, True), (40, 5, False)])
def test_softmax_router_and_experts(device, E, top, shared):
    """Scores are the softmax over all experts, the chosen ones are not renormalised; the shared expert is scaled by
    one sigmoid per token."""
    W, F, N = 16, 6, 23
    cfg = cfg_of([dict(type="mamba2", mixer=SSM, mlp=dict(kind="moe", expert=dict(ff=F), router=dict(experts=E, top=top),
                                                          **({"shared": dict(ff=5)} if shared else {})))], width=W)
    P = {k: v.float() for k, v in O.random_checkpoint(cfg, seed=E).items()}
    h = torch.randn(N, W, generator=torch.Generator().manual_seed(1))
    want = O.moe_ff(h.to(F64), P, "l0.mlp.", cfg["layers"][0]["mlp"])
    idx, w = O.route(h.to(F64), P["l0.mlp.router"], top)
    assert top == E or float(w.sum(-1).max()) < 1.0  # the kept scores do not sum to one
    model = VitinexForCausalLM.from_checkpoint(cfg, P, dtype=torch.float32, device=device)
    close(model.layers[0].mlp(h.to(device)), want, 1e-4)
    ids, wts = routed_experts.grouped_topk_route(O.lin(h.to(F64), P["l0.mlp.router"]).float().to(device), None, top,
                                                 score="softmax", renorm=False)
    assert torch.equal(ids.cpu().long(), idx)
    close(wts, w, 1e-5)


# -------------------------------------------------------------------- whole models
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("shape", sorted(SHAPES))
def test_whole_model_and_every_layer_run(device, shape):
    cfg = SHAPES[shape]
    P = {k: v.float() for k, v in O.random_checkpoint(cfg, seed=5).items()}
    toks = torch.randint(0, cfg["vocab"], (33,), generator=torch.Generator().manual_seed(7)).tolist()
    want_res = []
    want = O.forward(cfg, P, toks, want_res)
    assert model_class_for(cfg) is VitinexForCausalLM
    model = VitinexForCausalLM.from_checkpoint(cfg, P, dtype=torch.float32, device=device)
    assert len(model.runs) == len(want_res) == len(model.kv_layer_shapes()) == len(model.state_layer_buffers())
    page = 8
    kv = KVCacheManager(len(model.runs), 0, 0, num_blocks=6, block_size=page, device=device, dtype=torch.float32,
                        layer_shapes=model.kv_layer_shapes())
    state = StateCacheManager(model.state_layer_buffers(), 1, device=device)
    batch, _ = one_sequence(len(toks), device, page)
    got_res = []
    with torch.no_grad():
        got = model.forward_ragged(torch.tensor(toks, device=device), batch, kv, state, None, got_res)
    for r, (a, b) in enumerate(zip(got_res, want_res)):
        close(a, b, 2e-4)
    close(got, want)
    with torch.no_grad():
        close(model(torch.tensor([toks, toks[::-1]], device=device))[1], O.forward(cfg, P, toks[::-1]))


def test_loader_refuses_stray_and_missing_tensors():
    cfg = SHAPES["looped_middle"]
    P = O.random_checkpoint(cfg, seed=1)
    with pytest.raises(ValueError):
        VitinexForCausalLM.from_checkpoint(cfg, dict(P, extra=torch.zeros(3)), dtype=torch.float32)
    Q = dict(P)
    del Q["l1.mlp.shared.sg"]
    with pytest.raises(KeyError):
        VitinexForCausalLM.from_checkpoint(cfg, Q, dtype=torch.float32)
    bad = copy.deepcopy(cfg)
    bad["layers"][0]["type"] = "something_else"
    with pytest.raises(ValueError):
        VitinexForCausalLM.from_checkpoint(bad, P, dtype=torch.float32)


@pytest.mark.gpu
def test_bfloat16_serving_stays_near_the_oracle():
    """bfloat16 matrices and activations, float32 residual, norms, scores, router and state."""
    lat = dict(dim=32, heads=4, kv_rank=64, q_rank=48, rot=dict(base=10000.0, dims=16), rot_dim=16, scale=0.15, vdim=24)
    ssm = dict(conv=4, groups=2, heads=4, norm_groups=2, state=16, vdim=16)
    moe = dict(kind="moe", expert=dict(ff=32), router=dict(experts=6, top=2), shared=dict(ff=32))
    cfg = cfg_of([dict(type="latent_attention", mixer=lat, mlp=dict(kind="dense", ff=96)),
                  dict(type="mamba2", mixer=ssm, mlp=moe)], loop=dict(start=0, stop=2, times=2), width=64, vocab=80)
    P = {k: v.float() for k, v in O.random_checkpoint(cfg, seed=4).items()}
    toks = torch.randint(0, 80, (70,), generator=torch.Generator().manual_seed(9)).tolist()
    want = O.forward(cfg, P, toks).float()
    model = VitinexForCausalLM.from_checkpoint(cfg, P, dtype=torch.bfloat16, device="cuda")
    with torch.no_grad():
        got = model(torch.tensor([toks], device="cuda"))[0].float().cpu()
    err = (got - want).pow(2).mean(-1).sqrt() / want.pow(2).mean().sqrt()
    assert err.median().item() < 0.03 and (err < 0.1).float().mean().item() > 0.9


@pytest.mark.gpu
@pytest.mark.parametrize("shape", sorted(SHAPES))
def test_bfloat16_serving_of_odd_sizes(shape):
    """Sizes that are no multiples of 8 (strided, unaligned rows everywhere) in bfloat16: whole prompt and small
    steps agree with each other and, loosely, with the oracle."""
    from colossalai_amd.inference import ContinuousBatchEngine, InferenceConfig

    cfg = SHAPES[shape]
    P = {k: v.float() for k, v in O.random_checkpoint(cfg, seed=6).items()}
    toks = torch.randint(0, cfg["vocab"], (45,), generator=torch.Generator().manual_seed(8)).tolist()
    want = O.forward(cfg, P, toks).float()

    def run(cuts):
        model = VitinexForCausalLM.from_checkpoint(cfg, P, dtype=torch.bfloat16, device="cuda")
        eng = ContinuousBatchEngine(model, InferenceConfig(max_batch_size=1, dtype=torch.bfloat16), num_blocks=8,
                                    block_size=16)
        out, at = [], 0
        for n in cuts:
            out.append(eng.run_ragged([("a", toks[at : at + n], list(range(n)))]))
            at += n
        return torch.cat(out, 0).float().cpu()

    whole, stepped = run([45]), run([30, 2, 5] + [1] * 8)
    scale = want.pow(2).mean().sqrt()
    for got in (whole, stepped):
        err = (got - want).pow(2).mean(-1).sqrt() / scale
        assert err.median().item() < 0.06 and (err < 0.2).float().mean().item() > 0.8
