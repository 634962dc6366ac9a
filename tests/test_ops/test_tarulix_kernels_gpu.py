"""HIP kernels of the Tarulix serving path against their float32 PyTorch references (same op, run on CPU copies of
the inputs), on ragged batches that mix fresh sequences, continued portions and single decode tokens, in bfloat16
and float32."""

import pytest
import torch

from colossalai_amd.ops import group_norm, half_rotary, routed_experts, selective_scan as scan_ops
from colossalai_amd.ops.pair_rotary import pair_frequencies
from colossalai_amd.ops.paged_attention import (distance_bias_table, mix_values, paged_attention, paged_attention_ref,
                                                paged_pool_write, paged_pool_write_ref, summary_rows_per_page)
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
@pytest.mark.parametrize("W", [96, 200, 1024, 2048, 4104])
@pytest.mark.parametrize("two", [False, True])
def test_add_scaled_unit_norm(dtype, W, two):
    torch.manual_seed(W)
    N = 19
    res = torch.randn(N, W)
    a = (torch.randn(N, W) * 2).to(dtype)
    b = (torch.randn(N, W) * 0.5).to(dtype) if two else None
    want_res = res.clone()
    want = group_norm.add_scaled_unit_norm_ref(want_res, a, b, 0.9, 0.4, 1.7, 1e-6, dtype)
    got_res = res.cuda()
    got = group_norm.add_scaled_unit_norm(got_res, a.cuda(), None if b is None else b.cuda(), 0.9, 0.4, 1.7, 1e-6, dtype)
    torch.testing.assert_close(got_res.cpu(), want_res, rtol=2e-5, atol=2e-5)
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dtype))
    assert group_norm.add_scaled_unit_norm(got_res, a.cuda(), None, 1.0, 0.0, 1.0, 1e-6, None) is None


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,D,dims", [(8, 64, 0), (4, 80, 24), (3, 40, 40), (2, 136, 64), (1, 320, 6)])
@pytest.mark.parametrize("eps", [1e-6, None])
def test_rotate_halves_unit_norm(dtype, H, D, dims, eps):
    torch.manual_seed(D)
    N = 29
    packed = (torch.randn(N, H * D + 24) * 2).to(dtype)   # heads side by side inside a wider row
    x = packed[:, 8 : 8 + H * D].view(N, H, D)
    pos = torch.randint(0, 5000, (N,), dtype=torch.int32)
    freqs = pair_frequencies(40000.0, dims) if dims else None
    want = half_rotary.rotate_halves_unit_norm_ref(x, pos, freqs, eps)
    xg = packed.cuda()[:, 8 : 8 + H * D].view(N, H, D)
    got = half_rotary.rotate_halves_unit_norm(xg, pos.cuda(), None if freqs is None else freqs.cuda(), eps)
    assert got.is_contiguous() and got.dtype == dtype
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
def test_mix_values(dtype):
    torch.manual_seed(0)
    N, C = 33, 136
    a = torch.randn(N, 3 * C).to(dtype)
    b = torch.randn(N, C).to(dtype)
    want = torch.lerp(a[:, C : 2 * C].float(), b.float(), 0.3).to(dtype)
    got = mix_values(a.cuda()[:, C : 2 * C], b.cuda(), 0.3)
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dtype))


def fill_pools(batch_cpu, pages, page, G, D, Dv, dtype, P=None):
    kpool = torch.randn(pages, page, G, D).to(dtype)
    vpool = torch.randn(pages, page, G, Dv).to(dtype)
    if P is None:
        return kpool, vpool, None, None
    R = summary_rows_per_page(page, P)
    ksum = torch.randn(pages, R, G, D).to(dtype)      # stale rows everywhere: only refreshed summaries may count
    vsum = torch.randn(pages, R, G, Dv).to(dtype)
    return kpool, vpool, ksum, vsum


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("P", [16, 4, 6, 40])
def test_paged_pool_write(dtype, P):
    torch.manual_seed(P)
    dev, cpu, pages = make_batch("cuda")
    kpool, vpool, ksum, vsum = fill_pools(cpu, pages, 16, 2, 24, 40, dtype, P)
    got_k, got_v = ksum.cuda(), vsum.cuda()
    paged_pool_write(kpool.cuda(), vpool.cuda(), got_k, got_v, dev, P)
    paged_pool_write_ref(kpool, vpool, ksum, vsum, cpu, P)
    torch.testing.assert_close(got_k.cpu().float(), ksum.float(), **tol(dtype))
    torch.testing.assert_close(got_v.cpu().float(), vsum.float(), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,Dv", [(8, 2, 64, 32), (4, 4, 40, 24), (6, 2, 96, 136), (2, 1, 20, 6)])
@pytest.mark.parametrize("window", [0, 7, 50])
def test_attention_distance_table_and_learned_sink(dtype, H, G, D, Dv, window):
    torch.manual_seed(H * D + window)
    dev, cpu, pages = make_batch("cuda")
    N = cpu.num_tokens
    kpool, vpool, _, _ = fill_pools(cpu, pages, 16, G, D, Dv, dtype)
    q = torch.randn(N, H, D).to(dtype)
    rel = torch.randn(12, H)
    table = distance_bias_table(rel, 37.0, window if window else 38)
    sink = torch.randn(H) * 2
    want = paged_attention_ref(q, kpool, vpool, cpu, 0.2, window=window, sink_logits=sink, dist_bias=table)
    got = paged_attention(q.cuda(), kpool.cuda(), vpool.cuda(), dev, 0.2, window=window, sink_logits=sink.cuda(),
                          dist_bias=table.cuda())
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,Dv", [(8, 4, 96, 64), (4, 1, 40, 24), (6, 6, 24, 136), (3, 3, 20, 6)])
@pytest.mark.parametrize("window,P", [(20, 16), (9, 4), (33, 6), (16, 40), (1, 1)])
def test_attention_block_summaries_and_talking_heads(dtype, H, G, D, Dv, window, P):
    torch.manual_seed(H * D + window)
    dev, cpu, pages = make_batch("cuda")
    N = cpu.num_tokens
    kpool, vpool, ksum, vsum = fill_pools(cpu, pages, 16, G, D, Dv, dtype, P)
    # summaries of every complete block of every sequence, as earlier steps would have left them
    for i in range(cpu.num_seqs):
        whole = RaggedBatch.build([cpu.start_host[i] + cpu.cu_host[i + 1] - cpu.cu_host[i]], [0], [0], "cpu",
                                  [cpu.block_tables[i].tolist()], 16)
        paged_pool_write_ref(kpool, vpool, ksum, vsum, whole, P)
    q = torch.randn(N, H, D).to(dtype)
    talk = torch.randn(H, H) * 0.5 + torch.eye(H)
    for tk in (None, talk):
        want = paged_attention_ref(q, kpool, vpool, cpu, 0.3, window=window, softcap=5.0, pooled=(ksum, vsum, P), talk=tk)
        got = paged_attention(q.cuda(), kpool.cuda(), vpool.cuda(), dev, 0.3, window=window, softcap=5.0,
                              pooled=(ksum.cuda(), vsum.cuda(), P), talk=None if tk is None else tk.cuda())
        torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dtype))


def make_long_batch(device):
    """A portion long enough for the chunked form (not a multiple of the chunk), beside a decode token, a short
    continued portion and a second long, continued one."""
    counts, starts, slots = [300, 1, 7, 257], [0, 63, 130, 40], [3, 0, 5, 1]
    return (RaggedBatch.build(counts, starts, slots, device), RaggedBatch.build(counts, starts, slots, "cpu"), 0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C,S", [(192, 20), (64, 16), (100, 3), (48, 70), (8, 1)])
@pytest.mark.parametrize("long", [False, True])
def test_selective_scan(dtype, C, S, long):
    torch.manual_seed(C + S)
    dev, cpu, _ = make_long_batch("cuda") if long else make_batch("cuda")
    N = cpu.num_tokens
    x = torch.randn(N, C)
    packed = torch.randn(N, 2 * S + 5).to(dtype)
    dt_raw = (torch.randn(N, C) * 2).to(dtype)
    z = torch.randn(N, 2 * C).to(dtype)
    A_log = torch.randn(C, S) * 0.5
    D_skip, dt_bias = torch.randn(C), torch.randn(C)
    state = torch.randn(6, C, S)
    want_state = state.clone()
    want = scan_ops.selective_scan_ref(x, dt_raw, A_log, packed[:, 5 : 5 + S], packed[:, 5 + S :], D_skip, dt_bias,
                                       z[:, C:], want_state, cpu)
    got_state = state.cuda()
    pg, zg = packed.cuda(), z.cuda()
    got = scan_ops.selective_scan(x.cuda(), dt_raw.cuda(), A_log.cuda(), pg[:, 5 : 5 + S], pg[:, 5 + S :], D_skip.cuda(),
                                  dt_bias.cuda(), zg[:, C:], got_state, dev)
    torch.testing.assert_close(got.cpu().float(), want.float(), **(tol(dtype) if not long or dtype == torch.bfloat16
                                                                     else dict(rtol=2e-4, atol=2e-4)))
    torch.testing.assert_close(got_state.cpu(), want_state, rtol=2e-4, atol=2e-4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("N", [5, 40, 700, 3000])
@pytest.mark.parametrize("W,F_", [(64, 32), (96, 40)])
def test_gated_experts_with_identity(dtype, N, W, F_):
    torch.manual_seed(N + W)
    E, I, top = 6, 3, 4
    h = torch.randn(N, W).to(dtype)
    w_up = (torch.randn(E, 2 * F_, W) * W ** -0.5).to(dtype)
    w_down = (torch.randn(E, W, F_) * F_ ** -0.5).to(dtype)
    logits = torch.randn(N, E + I)
    corr = torch.randn(E + I) * 0.1
    ids, weights = routed_experts.grouped_topk_route_ref(logits, corr, top, score="softmax", renorm=False)
    assert (ids >= E).any() and (ids < E).any()
    base = torch.randn(N, W).to(dtype)
    want = routed_experts.routed_expert_ffn_ref(h, w_up, w_down, ids, weights, base, "silu_gated", identity=True)
    gi, gw = routed_experts.grouped_topk_route(logits.cuda(), corr.cuda(), top, score="softmax", renorm=False)
    assert torch.equal(gi.cpu(), ids)
    got = routed_experts.routed_expert_ffn(h.cuda(), w_up.cuda(), w_down.cuda(), gi, gw, base.cuda(), "silu_gated",
                                           identity=True, num_ids=E + I)
    torch.testing.assert_close(got.cpu(), want, **(dict(rtol=1e-4, atol=1e-4) if dtype == torch.float32
                                                    else dict(rtol=3e-2, atol=3e-2)))
