"""HIP kernels of the latent-attention / state-space serving path against their float32 PyTorch
references (same op, run on CPU copies of the inputs), on ragged batches that mix fresh sequences,
continued portions and single decode tokens, in bfloat16 and float32."""

import pytest
import torch

from colossalai_amd.ops import group_norm, latent_attention, linear_recurrence, pair_rotary, routed_experts, short_conv
from colossalai_amd.ops.activation import gelu_tanh_mul
from colossalai_amd.ops.paged_attention import paged_attention, paged_attention_ref
from colossalai_amd.ops.ragged import RaggedBatch

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def tol(dtype):
    return dict(rtol=2e-5, atol=2e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)


def make_batch(device, page=16):
    counts = [37, 5, 1, 1, 1, 70]
    starts = [0, 21, 63, 64, 0, 130]
    slots = [3, 0, 5, 1, 4, 2]
    tables, nxt = [], 0
    for c, s in zip(counts, starts):
        need = (c + s + page - 1) // page
        tables.append(list(range(nxt + need - 1, nxt - 1, -1)))  # pages in descending order: not contiguous
        nxt += need
    return (RaggedBatch.build(counts, starts, slots, device, tables, page),
            RaggedBatch.build(counts, starts, slots, "cpu", tables, page), nxt)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("W", [96, 200, 2048, 4104, 6144])
def test_add_layer_norm(dtype, W):
    torch.manual_seed(W)
    N = 23
    x = torch.randn(N, W) * 3 + 0.7
    y = (torch.randn(N, W) * 2 - 1.5).to(dtype)
    wo, wn = torch.randn(W), torch.randn(W)
    xg, xc = x.cuda(), x.clone()
    hg = group_norm.add_layer_norm(xg, y.cuda(), wo.cuda(), 0.3, wn.cuda(), 1e-6, dtype)
    hc = group_norm.add_layer_norm_ref(xc, y, wo, 0.3, wn, 1e-6, dtype)
    torch.testing.assert_close(xg.cpu(), xc, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(hg.cpu().float(), hc.float(), **tol(dtype))
    # the sum alone, and the plain norm
    xg2, xc2 = x.cuda(), x.clone()
    assert group_norm.add_layer_norm(xg2, y.cuda(), wo.cuda(), 1.7, None, 1e-6, dtype) is None
    group_norm.add_layer_norm_ref(xc2, y, wo, 1.7, None, 1e-6, dtype)
    torch.testing.assert_close(xg2.cpu(), xc2, rtol=1e-5, atol=1e-5)
    pg = group_norm.layer_norm(x.cuda(), wn.cuda(), 1e-6, dtype)
    torch.testing.assert_close(pg.cpu().float(), group_norm.layer_norm_ref(x, wn, 1e-6, dtype).float(), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("groups,W", [(1, 96), (2, 160), (3, 600), (8, 4096)])
def test_gated_grouped_rms_norm(dtype, groups, W):
    torch.manual_seed(2)
    x = torch.randn(19, W)
    wide = torch.randn(19, W + 24).to(dtype)
    gate = wide[:, 8 : 8 + W]
    w = torch.randn(W)
    out = group_norm.gated_grouped_rms_norm(x.cuda(), wide.cuda()[:, 8 : 8 + W], w.cuda(), groups, 1e-6, dtype)
    ref = group_norm.gated_grouped_rms_norm_ref(x, gate, w, groups, 1e-6, dtype)
    torch.testing.assert_close(out.cpu().float(), ref.float(), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
def test_strided_rms_norm(dtype):
    torch.manual_seed(3)
    wide = torch.randn(11, 300).to(dtype)
    w = torch.randn(128)
    out = group_norm.grouped_rms_norm(wide.cuda()[:, 40:168], w.cuda(), 1, 1e-6)
    ref = group_norm.grouped_rms_norm_ref(wide[:, 40:168], w, 1, 1e-6)
    torch.testing.assert_close(out.cpu().float(), ref.float(), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("F", [96, 77])
def test_gelu_tanh_mul(dtype, F):
    torch.manual_seed(4)
    packed = (torch.randn(13, 2 * F) * 3).to(dtype)
    out = gelu_tanh_mul(packed.cuda())
    g, u = packed[:, :F].float(), packed[:, F:].float()
    ref = torch.nn.functional.gelu(g, approximate="tanh") * u
    torch.testing.assert_close(out.cpu().float(), ref.to(dtype).float(), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("R,dims", [(32, 32), (24, 16), (7, 4)])
def test_rotate_pairs(dtype, R, dims):
    torch.manual_seed(5)
    N, H = 29, 3
    wide = torch.randn(N, H, R + 10).to(dtype)
    pos = torch.randint(0, 5000, (N,), dtype=torch.int32)
    f = pair_rotary.pair_frequencies(250000.0, dims)
    out_wide = torch.zeros(N, H, R + 6, dtype=dtype, device="cuda")
    pair_rotary.rotate_pairs(wide.cuda()[:, :, 10:], pos.cuda(), f.cuda(), out=out_wide[:, :, 6:])
    ref = pair_rotary.rotate_pairs_ref(wide[:, :, 10:], pos, f)
    torch.testing.assert_close(out_wide[:, :, 6:].cpu().float(), ref.float(), **tol(dtype))
    assert float(out_wide[:, :, :6].abs().max()) == 0.0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rank,R,dims", [(64, 16, 16), (40, 24, 16)])
def test_latent_kv_write(dtype, rank, R, dims):
    torch.manual_seed(6)
    gb, cb, pages = make_batch("cuda")
    N = gb.num_tokens
    wide = torch.randn(N, rank + R + 16).to(dtype)
    w = torch.randn(rank)
    f = pair_rotary.pair_frequencies(10000.0, dims)
    pg = torch.zeros(pages, 16, 1, rank + R, dtype=dtype, device="cuda")
    pc = torch.zeros(pages, 16, 1, rank + R, dtype=dtype)
    latent_attention.latent_kv_write(wide.cuda()[:, 8 : 8 + rank + R], w.cuda(), 1e-6, f.cuda(), pg, gb)
    latent_attention.latent_kv_write_ref(wide[:, 8 : 8 + rank + R], w, 1e-6, f, pc, cb)
    torch.testing.assert_close(pg.cpu().float(), pc.float(), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,rank,R", [(8, 128, 64), (3, 40, 24), (5, 256, 64), (2, 512, 64), (4, 96, 16), (3, 320, 32), (2, 44, 12), (2, 27, 6)])
def test_attention_over_latent_view(dtype, H, rank, R):
    """Multi-query attention whose values are the leading channels of the keys (a view of the key pool)."""
    torch.manual_seed(7)
    gb, cb, pages = make_batch("cuda")
    N = gb.num_tokens
    pool = (torch.randn(pages, 16, 1, rank + R) * 0.5).to(dtype)
    q = (torch.randn(N, H, rank + R) * 0.5).to(dtype)
    gate = torch.randn(N, H).to(dtype)
    pg = pool.cuda()
    out = paged_attention(q.cuda(), pg, pg[..., :rank], gb, 0.11, gate=gate.cuda())
    ref = paged_attention_ref(q, pool, pool[..., :rank], cb, 0.11, gate=gate)
    torch.testing.assert_close(out.cpu().float(), ref.float(), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,Dv,K", [(8, 2, 64, 32, 4), (4, 1, 128, 64, 4), (3, 3, 20, 24, 2), (8, 4, 64, 16, 1)])
def test_conv_and_ssd_recurrence(dtype, H, G, D, Dv, K):
    torch.manual_seed(8)
    gb, cb, _ = make_batch("cuda")
    N = gb.num_tokens
    inner, C = H * Dv, H * Dv + 2 * G * D
    proj = (torch.randn(N, 2 * inner + 2 * G * D + H) * 0.7).to(dtype)
    taps, bias = torch.randn(C, K) * 0.5, torch.randn(C) * 0.1
    A_log, dt_bias, skip = torch.randn(H) * 0.5 - 0.5, torch.randn(H) * 0.5 - 1.0, torch.randn(H)
    tail = torch.randn(6, max(K - 1, 1), C)[:, : K - 1]
    state = torch.randn(6, H, D, Dv)

    def run(dev, batch, conv_fn, scan_fn):
        p, tl, st = proj.to(dev), tail.to(dev).clone(), state.to(dev).clone()
        xbc = conv_fn(p[:, inner : inner + C], taps.to(dev), tl if K > 1 else None, batch, True, torch.float32,
                      bias.to(dev))
        y = scan_fn(xbc[:, :inner].view(N, H, Dv), xbc[:, inner : inner + G * D].view(N, G, D),
                    xbc[:, inner + G * D:].view(N, G, D), p[:, inner + C:], A_log.to(dev), dt_bias.to(dev),
                    skip.to(dev), st, batch)
        return xbc.cpu(), y.cpu(), tl.cpu(), st.cpu()

    got = run("cuda", gb, short_conv.short_conv, linear_recurrence.ssd_recurrence)
    ref = run("cpu", cb, short_conv.short_conv_ref, linear_recurrence.ssd_recurrence_ref)
    for a, b in zip(got, ref):
        torch.testing.assert_close(a, b, rtol=3e-5, atol=3e-5)


@pytest.mark.parametrize("E,top", [(10, 3), (5, 5), (64, 6), (130, 1)])
def test_softmax_route(E, top):
    torch.manual_seed(9)
    wide = torch.randn(37, E + 1) * 3
    ids, w = routed_experts.grouped_topk_route(wide.cuda()[:, :E], None, top, score="softmax", renorm=False)
    rid, rw = routed_experts.grouped_topk_route_ref(wide[:, :E], None, top, score="softmax", renorm=False)
    assert torch.equal(ids.cpu(), rid)
    torch.testing.assert_close(w.cpu(), rw, rtol=1e-5, atol=1e-7)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("N", [3, 40, 700])
def test_experts_with_gated_base(dtype, N):
    torch.manual_seed(10)
    E, F, W, top = 10, 48, 160, 3
    h = torch.randn(N, W).to(dtype)
    up, down = (torch.randn(E, F, W) * W ** -0.5).to(dtype), (torch.randn(E, W, F) * F ** -0.5).to(dtype)
    wide = torch.randn(N, E + 1) * 2
    base = torch.randn(N, W).to(dtype)
    ids, wt = routed_experts.grouped_topk_route_ref(wide[:, :E], None, top, score="softmax", renorm=False)
    out = routed_experts.routed_expert_ffn(h.cuda(), up.cuda(), down.cuda(), ids.cuda(), wt.cuda(), base.cuda(),
                                           "relu_squared", wide.cuda()[:, E])
    ref = routed_experts.routed_expert_ffn_ref(h, up, down, ids, wt, base, "relu_squared", wide[:, E])
    torch.testing.assert_close(out.cpu(), ref, **(dict(rtol=1e-4, atol=1e-4) if dtype == torch.float32 else tol(dtype)))


@pytest.mark.parametrize("window,keep", [(0, 0), (70, 5)])
@pytest.mark.parametrize("D,Dv", [(64, 32), (128, 128), (48, 24)])
def test_one_query_head_per_key_head_prompt_tiles(window, keep, D, Dv):
    """Multi-head attention without grouping in bfloat16: the matrix-core kernel's blocks take four token tiles of
    one head. Portions longer and shorter than a block, from position 0 and continued, next to a decode token."""
    torch.manual_seed(11)
    counts, starts, page = [200, 37, 1, 130, 128], [0, 50, 9, 300, 64], 16
    tables, nxt = [], 0
    for c, s in zip(counts, starts):
        need = (c + s + page - 1) // page
        tables.append(list(range(nxt + need - 1, nxt - 1, -1)))
        nxt += need
    gb = RaggedBatch.build(counts, starts, list(range(5)), "cuda", tables, page)
    cb = RaggedBatch.build(counts, starts, list(range(5)), "cpu", tables, page)
    H = 3
    kpool = (torch.randn(nxt, page, H, D) * 0.5).to(torch.bfloat16)
    vpool = torch.randn(nxt, page, H, Dv).to(torch.bfloat16)
    q = (torch.randn(gb.num_tokens, H, D) * 0.5).to(torch.bfloat16)
    gate = torch.randn(gb.num_tokens, H).to(torch.bfloat16)
    out = paged_attention(q.cuda(), kpool.cuda(), vpool.cuda(), gb, 0.3, window, keep, None, gate.cuda())
    ref = paged_attention_ref(q, kpool, vpool, cb, 0.3, window, keep, None, gate)
    torch.testing.assert_close(out.cpu().float(), ref.float(), rtol=2e-2, atol=2e-2)


def test_decode_steps_of_the_state_space_scan_match_prompt_steps():
    """Single-token steps take a launch shape of their own: same results, same state, as one portion."""
    torch.manual_seed(12)
    H, G, D, Dv, T = 8, 2, 128, 64, 6
    x, Bm, Cm = torch.randn(T, H, Dv).cuda(), torch.randn(T, G, D).cuda(), torch.randn(T, G, D).cuda()
    dt = torch.randn(T, H).cuda()
    A_log, dt_bias, skip = (torch.randn(H) * 0.3).cuda(), torch.randn(H).cuda(), torch.randn(H).cuda()
    st1, st2 = torch.randn(3, H, D, Dv).cuda(), None
    st2 = st1.clone()
    whole = linear_recurrence.ssd_recurrence(x, Bm, Cm, dt, A_log, dt_bias, skip, st1,
                                             RaggedBatch.build([T], [5], [1], "cuda"))
    steps = [linear_recurrence.ssd_recurrence(x[t : t + 1], Bm[t : t + 1], Cm[t : t + 1], dt[t : t + 1], A_log, dt_bias,
                                              skip, st2, RaggedBatch.build([1], [5 + t], [1], "cuda")) for t in range(T)]
    torch.testing.assert_close(torch.cat(steps, 0), whole, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(st2, st1, rtol=1e-5, atol=1e-5)
