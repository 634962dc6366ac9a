"""Tarulix against the float64 oracle (tests/tarulix_oracle.py): every mechanism alone, driven through a real page
pool and state slots with prompts cut in several ways, with inputs made so that an off-by-one shows (a spiked key
just inside and just outside a window, a block summary that is just seen and not yet seen, a sink that takes all the
weight), and whole models of several shapes."""

import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, os.path.join(ROOT, "tests"))
import tarulix_oracle as O  # noqa: E402

from colossalai_amd.inference.kv_cache import KVCacheManager  # noqa: E402
from colossalai_amd.inference.state_cache import StateCacheManager  # noqa: E402
from colossalai_amd.models import TarulixForCausalLM  # noqa: E402
from colossalai_amd.ops.paged_attention import distance_bias_table  # noqa: E402
from colossalai_amd.ops.ragged import RaggedBatch  # noqa: E402

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
EPS = 1e-5
W = 16

ATT = dict(bias_max=9, dim=8, heads=4, kv_heads=2, mask=dict(size=13), scale=3.0, v_mix=False, vdim=6)
LEFT = dict(dim=8, heads=4, kv_heads=2, mask=dict(pool=3, size=7), rot=dict(base=100.0, dims=4), scale=3.0, softcap=10.0,
            vdim=6)
RIGHT = dict(conv=3, dt_rank=2, inner=12, state=5)
MOE = dict(kind="moe", expert=dict(ff=10), router=dict(experts=5, identity=2, top=3), shared=dict(ff=6))


def one_layer(kind, mixer, mlp=None):
    return dict(architecture="Tarulix", vocab=20, width=W, norm=dict(eps=EPS), layers=[dict(type=kind, mixer=mixer, mlp=mlp)])


def close(got, want, tol=2e-4):
    err = (got.detach().cpu().double() - want).abs().max().item()
    assert err <= tol * max(1.0, want.abs().max().item()), f"max abs error {err}"


def drive(call, h, cuts, device, kv_shape=None, summary=None, state_buf=None, page=4):
    """Run ``call(rows, batch, pools, state)`` over the rows of h in portions of the given sizes, on one sequence that
    owns scattered pages of a pool and the second of two state slots."""
    kv = KVCacheManager(1, 0, 0, num_blocks=64, block_size=page, device=device, dtype=torch.float32,
                        layer_shapes=[kv_shape], layer_summaries=[summary])
    state = StateCacheManager([state_buf], 2, device=device)
    for pool in (kv.k_pools[0], kv.v_pools[0], kv.k_summaries[0], kv.v_summaries[0]):
        if pool is not None:
            pool.normal_()          # whatever earlier owners left must not matter
    state.arena.normal_()
    state.allocate("other")
    slot = state.allocate("s")
    kv.allocate("other", 9)
    kv.allocate("s", 0)
    out, at = [], 0
    for n in cuts:
        kv.extend("s", at + n)
        kv.extend("other", kv.block_size * (len(kv.table("other")) + 1))   # interleave the pages of the two
        batch = RaggedBatch.build([n], [at], [slot], device, [kv.table("s")], page)
        pools = (kv.k_pools[0], kv.v_pools[0], kv.k_summaries[0], kv.v_summaries[0])
        with torch.no_grad():
            out.append(call(h[at : at + n].to(device), batch, pools, state.layers[0]))
        at += n
    assert at == h.shape[0]
    return torch.cat(out, 0)


def cut_sets(T, special):
    """Whole; the special position decoded alone after a long portion; pairs; a cut right at the special position."""
    pairs = [2] * (T // 2) + ([1] if T % 2 else [])
    return [[T], [special] + [1] * (T - special), pairs, [special - 1, 3, T - special - 2]]


# ------------------------------------------------------------------ distance table
@pytest.mark.parametrize("rows,far,length", [(10, 9.0, 13), (24, 90.0, 100), (9, 40.0, 60), (4, 100.0, 7), (2, 5.0, 12)])
def test_distance_table_follows_the_buckets(rows, far, length):
    rel = torch.randn(rows, 3, generator=torch.Generator().manual_seed(rows))
    table = distance_bias_table(rel, far, length)
    assert table.shape == (length, 3)
    for d in range(length):
        assert torch.equal(table[d], rel[O.distance_bucket(d, rows, far)]), d
    # the buckets themselves: exact below half, the last row from `far` on
    assert [O.distance_bucket(d, 16, 50.0) for d in (0, 7, 8, 49, 50, 500)] == [0, 7, 8, 15, 15, 15]


# ------------------------------------------------- windowed attention with table and sink
def spiked_attention(seed, T, i, j, cfg_mixer, kind="attention"):
    """A one-layer model whose keys repeat the queries' first head of each group, without q/k biases, and an input
    whose rows i and j are the same strong vector: query i's weight sits on key j (and on itself) if it sees it."""
    cfg = one_layer(kind, cfg_mixer)
    P = O.random_checkpoint(cfg, seed)
    pre = "l0.mix." if kind == "attention" else "l0.mix.left."
    c = cfg_mixer if kind == "attention" else cfg_mixer["left"]
    H, G, D = c["heads"], c["kv_heads"], c["dim"]
    q = P[pre + "q"].view(H, D, W)
    P[pre + "k"] = q[:: H // G].reshape(G * D, W).clone()
    P[pre + "q.b"].zero_()
    P[pre + "k.b"].zero_()
    g = torch.Generator().manual_seed(seed + 1)
    h = torch.randn(T, W, generator=g)
    s = torch.randn(W, generator=g) * 3
    if isinstance(j, int):
        j = [j]
    for t in [i] + list(j):
        h[t] = s
    return cfg, {k: v.float() for k, v in P.items()}, h


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("offset", [12, 13, 1, 5])        # window 13: distance 12 is its last place, 13 is outside
def test_window_edge_in_prompt_and_decode(device, offset):
    T, i = 40, 31
    cfg, P, h = spiked_attention(offset, T, i, i - offset, ATT)
    want, _ = O.biased_window_attention(h.double(), O.sub(P, "l0.mix."), ATT, EPS)
    mix = TarulixForCausalLM.from_checkpoint(cfg, P, dtype=torch.float32, device=device).layers[0].mix
    for cuts in cut_sets(T, i):
        got = drive(lambda x, b, pools, st: mix(x, b, pools, None, {}), h, cuts, device, kv_shape=mix.kv_shape())
        close(got, want)
    # the spike matters: without key j the row differs
    h2 = h.clone()
    h2[i - offset] = torch.randn(W, generator=torch.Generator().manual_seed(5))
    other, _ = O.biased_window_attention(h2.double(), O.sub(P, "l0.mix."), ATT, EPS)
    assert ((other[i] - want[i]).abs().max() > 1e-2) == (offset < 13)


@pytest.mark.parametrize("device", DEVICES)
def test_sink_takes_the_weight_and_first_tokens(device):
    cfg = one_layer("attention", ATT)
    P = {k: v.float() for k, v in O.random_checkpoint(cfg, 3).items()}
    P["l0.mix.sink"] = torch.tensor([25.0, -25.0, 0.0, 3.0])
    h = torch.randn(9, W, generator=torch.Generator().manual_seed(0))
    want, _ = O.biased_window_attention(h.double(), O.sub(P, "l0.mix."), ATT, EPS)
    mix = TarulixForCausalLM.from_checkpoint(cfg, P, dtype=torch.float32, device=device).layers[0].mix
    for cuts in ([9], [1] * 9, [2, 2, 2, 3]):
        got = drive(lambda x, b, pools, st: mix(x, b, pools, None, {}), h, cuts, device, kv_shape=mix.kv_shape())
        close(got, want)


@pytest.mark.parametrize("device", DEVICES)
def test_values_mix_with_the_first_mixing_layers(device):
    """Three attention layers: the first mixes nothing and is not the source, the second is the source, the third
    caches a blend of its values with the source's."""
    layers = [dict(type="attention", mixer=dict(ATT, v_mix=False), mlp=None),
              dict(type="attention", mixer=dict(ATT, v_mix=True), mlp=None),
              dict(type="attention", mixer=dict(ATT, v_mix=True, heads=2, dim=4), mlp=None)]
    cfg = dict(architecture="Tarulix", vocab=20, width=W, norm=dict(eps=EPS), layers=layers)
    P = {k: v.float() for k, v in O.random_checkpoint(cfg, 8).items()}
    toks = torch.randint(0, 20, (30,), generator=torch.Generator().manual_seed(2)).tolist()
    want, res = O.model_forward(cfg, P, toks)
    model = TarulixForCausalLM.from_checkpoint(cfg, P, dtype=torch.float32, device=device)
    close(model(torch.tensor([toks], device=device))[0], want, 3e-4)
    P2 = dict(P)
    P2["l2.mix.vmix"] = torch.tensor(0.0)
    assert (O.forward(cfg, P2, toks) - want).abs().max() > 1e-3


# ------------------------------------------- window + block summaries + talking heads
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("delta", [0, -1, 2])
def test_block_summary_just_seen_and_not_yet(device, delta):
    """Window 7, blocks of 3: block b = 4 (positions 12..14) is seen from query 21 on. The block's three inputs are
    the query's own strong vector, so its summary carries the spike; at query 20 the block's tokens have left the
    window and the block is not yet seen."""
    T, b = 40, 4
    i = b * 3 + 2 + 7 + delta
    mixer = dict(left=LEFT, right=RIGHT, left_scale=0.9, right_scale=0.4)
    cfg, P, h = spiked_attention(11 + delta, T, i, [12, 13, 14], mixer, kind="parallel")
    want = O.pooled_window_attention(h.double(), O.sub(P, "l0.mix.left."), LEFT, EPS)
    left = TarulixForCausalLM.from_checkpoint(cfg, P, dtype=torch.float32, device=device).layers[0].mix.left
    for cuts in cut_sets(T, i) + [[14, 1, 25], [15, 25], [13, 2, 25]]:      # the block completes inside / at the end of a portion
        got = drive(lambda x, bt, pools, st: left(x, bt, pools, None, {}), h, cuts, device, kv_shape=left.kv_shape(),
                    summary=LEFT["mask"]["pool"])
        close(got, want)
    h2 = h.clone()     # positions 12 and 13 have left query 20's window; it sees them again, pooled, from 21 on
    h2[12:14] = torch.randn(2, W, generator=torch.Generator().manual_seed(5))
    other = O.pooled_window_attention(h2.double(), O.sub(P, "l0.mix.left."), LEFT, EPS)
    assert ((other[i] - want[i]).abs().max() > 1e-2) == (delta >= 0)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("left", [dict(LEFT, mask=dict(pool=1, size=1)), dict(LEFT, mask=dict(pool=5, size=3), kv_heads=4),
                                  dict(LEFT, mask=dict(pool=9, size=4), kv_heads=1, rot=dict(base=7.0, dims=8)),
                                  dict(LEFT, mask=dict(pool=2, size=50), heads=2, kv_heads=2, dim=6, vdim=10,
                                       rot=dict(base=50.0, dims=2))])
def test_pooled_attention_of_other_sizes(device, left):
    cfg = one_layer("parallel", dict(left=left, right=RIGHT, left_scale=1.0, right_scale=1.0))
    P = {k: v.float() for k, v in O.random_checkpoint(cfg, 21).items()}
    h = torch.randn(33, W, generator=torch.Generator().manual_seed(1))
    want = O.pooled_window_attention(h.double(), O.sub(P, "l0.mix.left."), left, EPS)
    mod = TarulixForCausalLM.from_checkpoint(cfg, P, dtype=torch.float32, device=device).layers[0].mix.left
    for cuts, page in (([33], 4), ([20] + [1] * 13, 16), ([2] * 16 + [1], 2), ([7, 11, 15], 8)):
        got = drive(lambda x, b, pools, st: mod(x, b, pools, None, {}), h, cuts, device, kv_shape=mod.kv_shape(),
                    summary=left["mask"]["pool"], page=page)
        close(got, want)


def test_rotate_half_layout_and_unit_norm():
    from colossalai_amd.ops.half_rotary import rotate_halves_unit_norm
    from colossalai_amd.ops.pair_rotary import pair_frequencies

    x = torch.randn(7, 3, 10, generator=torch.Generator().manual_seed(0))
    pos = torch.tensor([0, 1, 5, 100, 1000, 3, 2], dtype=torch.int32)
    want = O.unit_rms(O.rotate_half_layout(x.double(), pos, 6, 50.0), 1e-6)
    # float32 angles: position 1000 times a frequency carries about 1e-4 of rounding
    close(rotate_halves_unit_norm(x, pos, pair_frequencies(50.0, 6), 1e-6), want, 3e-4)
    assert torch.equal(rotate_halves_unit_norm(x, pos, None, None), x)


# ------------------------------------------------------------------ selective scan
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("right", [RIGHT, dict(conv=1, dt_rank=1, inner=7, state=1), dict(conv=4, dt_rank=3, inner=20, state=9),
                                   dict(conv=2, dt_rank=5, inner=4, state=40)])
def test_selective_scan_carries_state_and_tail(device, right):
    cfg = one_layer("parallel", dict(left=LEFT, right=right, left_scale=1.0, right_scale=1.0))
    P = {k: v.float() for k, v in O.random_checkpoint(cfg, 5).items()}
    h = torch.randn(29, W, generator=torch.Generator().manual_seed(4))
    want = O.selective_scan_mixer(h.double(), O.sub(P, "l0.mix.right."), right)
    mod = TarulixForCausalLM.from_checkpoint(cfg, P, dtype=torch.float32, device=device).layers[0].mix.right
    for cuts in ([29], [1] * 29, [2] * 14 + [1], [3, 1, 1, 24], [28, 1]):
        got = drive(lambda x, b, pools, st: mod(x, b, st), h, cuts, device, state_buf=mod.state_buffers())
        close(got, want)


# ------------------------------------------------------------------ routed experts
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("moe", [MOE, dict(MOE, router=dict(experts=4, identity=0, top=1), shared=None),
                                 dict(MOE, router=dict(experts=2, identity=5, top=4)),
                                 dict(kind="moe", expert=dict(ff=3), router=dict(experts=3, top=3), shared=dict(ff=20))])
def test_routed_experts_identity_and_shared(device, moe):
    cfg = one_layer("attention", ATT, moe)
    P = {k: v.float() for k, v in O.random_checkpoint(cfg, 9).items()}
    h = torch.randn(37, W, generator=torch.Generator().manual_seed(6))
    want = O.routed_mlp(h.double(), O.sub(P, "l0.mlp."), moe)
    mlp = TarulixForCausalLM.from_checkpoint(cfg, P, dtype=torch.float32, device=device).layers[0].mlp
    with torch.no_grad():
        close(mlp(h.to(device)), want)
        close(mlp(h[:2].to(device)), want[:2])
    # the weights are the plain softmax scores: they do not sum to one
    r = moe["router"]
    if r["top"] < r["experts"] + r.get("identity", 0):
        s = torch.softmax(h.double() @ P["l0.mlp.router"].double().T, -1)
        chosen = torch.topk(s + P["l0.mlp.correction"].double(), r["top"]).indices
        assert (s.gather(1, chosen).sum(-1) < 0.99).any()


def test_output_norm_with_one_number():
    from colossalai_amd.ops.group_norm import add_scaled_unit_norm

    g = torch.Generator().manual_seed(0)
    x, a, b = torch.randn(5, W, generator=g), torch.randn(5, W, generator=g), torch.randn(5, W, generator=g)
    want = x.double() + O.scalar_norm(0.9 * a.double() + 0.4 * b.double(), 1.3, EPS)
    got = x.clone()
    cast = add_scaled_unit_norm(got, a, b, 0.9, 0.4, 1.3, EPS, torch.bfloat16)
    close(got, want, 1e-5)
    assert cast.dtype == torch.bfloat16 and torch.equal(cast, got.to(torch.bfloat16))


# ------------------------------------------------------------------ whole models
SHAPES = {
    "both mixers, experts everywhere": [
        dict(type="attention", mixer=dict(ATT, v_mix=True), mlp=MOE),
        dict(type="parallel", mixer=dict(left=LEFT, right=RIGHT, left_scale=0.9, right_scale=0.4), mlp=MOE),
        dict(type="attention", mixer=dict(ATT, v_mix=True), mlp=MOE)],
    "parallel first, no feed-forward in places, one key head": [
        dict(type="parallel", mixer=dict(left=dict(LEFT, kv_heads=1, mask=dict(pool=4, size=5)), right=dict(RIGHT, conv=2),
                                         left_scale=1.0, right_scale=2.0), mlp=None),
        dict(type="attention", mixer=dict(ATT, kv_heads=4, mask=dict(size=3), bias_max=30), mlp=None),
        dict(type="parallel", mixer=dict(left=dict(LEFT, heads=2, kv_heads=2, softcap=2.0), right=dict(RIGHT, state=1, conv=1),
                                         left_scale=0.3, right_scale=0.1),
             mlp=dict(MOE, router=dict(experts=3, identity=0, top=1)))],
    "window longer than the prompt": [
        dict(type="attention", mixer=dict(ATT, mask=dict(size=500), bias_max=20, dim=6, vdim=8, v_mix=True), mlp=MOE),
        dict(type="parallel", mixer=dict(left=dict(LEFT, mask=dict(pool=2, size=400)), right=RIGHT, left_scale=1.0,
                                         right_scale=1.0), mlp=None)],
}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("shape", sorted(SHAPES))
def test_whole_models(device, shape):
    cfg = dict(architecture="Tarulix", vocab=23, width=W, norm=dict(eps=EPS), layers=SHAPES[shape])
    P = {k: v.float() for k, v in O.random_checkpoint(cfg, len(shape), rel_rows=7).items()}
    toks = torch.randint(0, 23, (2, 35), generator=torch.Generator().manual_seed(1))
    model = TarulixForCausalLM.from_checkpoint(cfg, P, dtype=torch.float32, device=device)
    got = model(toks.to(device))
    for b in range(2):
        want, res = O.model_forward(cfg, P, toks[b].tolist())
        close(got[b], want, 3e-4)
    # the residual stream after every layer
    from colossalai_amd.inference.kv_cache import KVCacheManager as KV

    kv = KV(len(cfg["layers"]), 0, 0, num_blocks=3, block_size=16, device=device, dtype=torch.float32,
            layer_shapes=model.kv_layer_shapes(), layer_summaries=model.kv_layer_summaries())
    st = StateCacheManager(model.state_layer_buffers(), 1, device=device)
    batch = RaggedBatch.build([35], [0], [0], device, [[2, 0, 1]], 16)
    seen = []
    with torch.no_grad():
        model.forward_ragged(toks[1].to(device), batch, kv, st, residuals=seen)
    assert len(seen) == len(res)
    for g, w in zip(seen, res):
        close(g, w, 3e-4)


def test_checkpoint_names_are_checked():
    cfg = one_layer("attention", ATT, MOE)
    P = {k: v.float() for k, v in O.random_checkpoint(cfg, 0).items()}
    with pytest.raises(ValueError):
        TarulixForCausalLM.from_checkpoint(cfg, dict(P, stray=torch.zeros(1)), dtype=torch.float32)
    P.pop("l0.mlp.e1.up")
    with pytest.raises(KeyError):
        TarulixForCausalLM.from_checkpoint(cfg, P, dtype=torch.float32)
    with pytest.raises(ValueError):
        TarulixForCausalLM.from_checkpoint(one_layer("conv", ATT), {}, dtype=torch.float32)
