"""HIP serving kernels against their float32 PyTorch references (same op,
run on CPU copies of the inputs): ragged batches that mix fresh sequences,
continued sequences and single decode tokens, in bfloat16 and float32."""

import pytest
import torch

from colossalai_amd.ops import group_norm, linear_recurrence, paged_attention, routed_experts, short_conv, token_shift
from colossalai_amd.ops.activation import relu_squared, silu_mul, softcap
from colossalai_amd.ops.ragged import RaggedBatch

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def tol(dtype):
    return dict(rtol=2e-5, atol=2e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)


def make_batch(device, page=16):
    # a fresh prompt, a continued portion, two decode tokens (one at a page border), a fresh single token
    counts = [37, 5, 1, 1, 1]
    starts = [0, 21, 63, 64, 0]
    slots = [3, 0, 5, 1, 4]
    tables, nxt = [], 0
    for c, s in zip(counts, starts):
        need = (c + s + page - 1) // page
        tables.append(list(range(nxt + need - 1, nxt - 1, -1)))  # pages in descending order: not contiguous
        nxt += need
    return (RaggedBatch.build(counts, starts, slots, device, tables, page),
            RaggedBatch.build(counts, starts, slots, "cpu", tables, page), nxt)


def both(t):
    return t.cuda(), t.clone()


@pytest.mark.parametrize("dtype", DTYPES)
def test_token_shift(dtype):
    torch.manual_seed(0)
    gb, cb, _ = make_batch("cuda")
    W = 200
    x = torch.randn(gb.num_tokens, W)
    mu = torch.rand(W)
    arena = torch.randn(6, W + 8)
    pg, pc = arena.cuda()[:, 4 : 4 + W], arena.clone()[:, 4 : 4 + W]
    out = token_shift.token_shift(x.cuda(), mu.cuda(), pg, gb, dtype)
    ref = token_shift.token_shift_ref(x, mu, pc, cb, dtype)
    torch.testing.assert_close(out.cpu().float(), ref.float(), **tol(dtype))
    torch.testing.assert_close(pg.cpu(), pc)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("groups,W", [(1, 96), (4, 352), (3, 600)])
def test_grouped_rms_norm(dtype, groups, W):
    torch.manual_seed(1)
    x = torch.randn(19, W).to(dtype)
    w = torch.randn(W)
    out = group_norm.grouped_rms_norm(x.cuda(), w.cuda(), groups, 1e-5)
    torch.testing.assert_close(out.cpu().float(), group_norm.grouped_rms_norm_ref(x, w, groups, 1e-5).float(), **tol(dtype))
    res = torch.randn(19, W)
    rg = res.cuda()
    group_norm.grouped_rms_norm(x.cuda(), w.cuda(), groups, 1e-5, rg)
    group_norm.grouped_rms_norm_ref(x, w, groups, 1e-5, res)
    torch.testing.assert_close(rg.cpu(), res, rtol=2e-5, atol=2e-5)


@pytest.mark.parametrize("dtype", DTYPES)
def test_head_norm_gate_and_merge(dtype):
    torch.manual_seed(2)
    N, H, D, pad = 11, 3, 40, 8
    wide = torch.randn(N, H * D + pad).to(dtype)
    gate = torch.randn(N, H * D + pad).to(dtype)
    w = torch.randn(D)
    out = group_norm.head_rms_norm_gate(wide.cuda()[:, : H * D].view(N, H, D), w.cuda(), 1e-6,
                                        gate.cuda()[:, pad:], torch.float32)
    ref = group_norm.head_rms_norm_gate_ref(wide[:, : H * D].view(N, H, D), w, 1e-6, gate[:, pad:], torch.float32)
    torch.testing.assert_close(out.cpu(), ref, **tol(dtype))
    W = 120
    a, b = torch.randn(N, W).to(dtype), (torch.randn(N, W) * 3).to(dtype)
    wa, wb, wo = torch.randn(W), torch.randn(W), torch.randn(W)
    res = torch.randn(N, W)
    rg = res.cuda()
    group_norm.merge_rms_norm(a.cuda(), wa.cuda(), b.cuda(), wb.cuda(), 1e-6, wo.cuda(), 3, rg)
    group_norm.merge_rms_norm_ref(a, wa, b, wb, 1e-6, wo, 3, res)
    torch.testing.assert_close(rg.cpu(), res, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("K", [1, 2, 4, 7])
def test_short_conv(dtype, K):
    torch.manual_seed(3)
    gb, cb, _ = make_batch("cuda")
    C, pad = 72, 5
    wide = torch.randn(gb.num_tokens, C + pad).to(dtype)
    taps = torch.randn(C, K)
    arena = torch.randn(6, max(K - 1, 1) * C + 4)
    tg = arena.cuda()[:, : (K - 1) * C].view(6, K - 1, C) if K > 1 else None
    tc = arena.clone()[:, : (K - 1) * C].view(6, K - 1, C) if K > 1 else None
    out = short_conv.short_conv(wide.cuda()[:, :C], taps.cuda(), tg, gb, True)
    ref = short_conv.short_conv_ref(wide[:, :C], taps, tc, cb, True)
    assert out.dtype == dtype
    torch.testing.assert_close(out.cpu().float(), ref.float(), **tol(dtype))
    if K > 1:  # float32 output of the same inputs (the slot's tail is refreshed again: same values)
        wide32 = short_conv.short_conv(wide.cuda()[:, :C], taps.cuda(), tg.clone(), gb, True, torch.float32)
        assert wide32.dtype == torch.float32
        torch.testing.assert_close(wide32.cpu(), short_conv.short_conv_ref(wide[:, :C], taps, tc.clone(), cb, True, torch.float32),
                                   rtol=2e-5, atol=2e-5)
    if K > 1:
        torch.testing.assert_close(tg.cpu(), tc, **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,Dv", [(4, 2, 32, 24), (3, 3, 20, 64), (2, 1, 128, 70), (2, 2, 8, 8)])
@pytest.mark.parametrize("qkv32", [False, True])
def test_gated_delta_rule(dtype, H, G, D, Dv, qkv32):
    """qkv32: q/k/v arrive in float32 (an unrounded convolution output) next to logits in ``dtype``."""
    torch.manual_seed(4)
    gb, cb, _ = make_batch("cuda")
    N = gb.num_tokens
    qd = torch.float32 if qkv32 else dtype
    q, k, v = (torch.randn(N, G, D).to(qd), torch.randn(N, G, D).to(qd), torch.randn(N, H, Dv).to(qd))
    bl, dt = torch.randn(N, H).to(dtype), torch.randn(N, H * D).to(dtype)
    A, bias = torch.randn(H) - 1, torch.randn(H * D)
    state = torch.randn(6, H, D, Dv)
    sg = state.cuda()
    out = linear_recurrence.gated_delta_rule(q.cuda(), k.cuda(), v.cuda(), bl.cuda(), dt.cuda(), A.cuda(), bias.cuda(),
                                             sg, gb, 1e-6, D ** -0.5)
    ref = linear_recurrence.gated_delta_rule_ref(q, k, v, bl, dt, A, bias, state, cb, 1e-6, D ** -0.5)
    torch.testing.assert_close(out.cpu(), ref, rtol=2e-4, atol=2e-4)
    live = sorted(gb.slots_host)
    torch.testing.assert_close(sg.cpu()[live], state[live], rtol=2e-4, atol=2e-4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,D,Dv", [(4, 32, 32), (3, 48, 20), (1, 256, 64)])
def test_tied_gate_recurrence(dtype, H, D, Dv):
    torch.manual_seed(5)
    gb, cb, _ = make_batch("cuda")
    N = gb.num_tokens
    q, f, v = torch.randn(N, H, D).to(dtype), torch.randn(N, H, D).to(dtype), torch.randn(N, H, Dv).to(dtype)
    fb, low = torch.randn(H * D), torch.rand(H * D)
    state = torch.randn(6, H, D, Dv)
    sg = state.cuda()
    out = linear_recurrence.tied_gate_recurrence(q.cuda(), f.cuda(), v.cuda(), fb.cuda(), low.cuda(), sg, gb)
    ref = linear_recurrence.tied_gate_recurrence_ref(q, f, v, fb, low, state, cb)
    torch.testing.assert_close(out.cpu(), ref, rtol=2e-4, atol=2e-4)
    live = sorted(gb.slots_host)
    torch.testing.assert_close(sg.cpu()[live], state[live], rtol=2e-4, atol=2e-4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("page", [16, 64])
@pytest.mark.parametrize("H,G,D,Dv,window,keep", [(4, 2, 32, 32, 9, 3), (6, 3, 24, 40, 0, 0), (2, 2, 64, 16, 70, 0),
                                                  (4, 1, 16, 130, 5, 30), (8, 2, 64, 64, 37, 11), (5, 5, 128, 128, 0, 0),
                                                  (4, 2, 128, 64, 33, 2), (2, 1, 64, 128, 31, 40), (8, 1, 64, 64, 12, 1)])
def test_paged_attention(dtype, H, G, D, Dv, window, keep, page):
    """Scalar kernel (float32, odd head sizes) and matrix-core kernel (bfloat16
    with head sizes it tiles) on the same ragged batch; the pool's other rows
    hold large values that a wrong page lookup or mask would pick up."""
    torch.manual_seed(6)
    gb, cb, pages = make_batch("cuda", page)
    N = gb.num_tokens
    kpool, vpool = (torch.randn(pages, page, G, D) * 3).to(dtype), (torch.randn(pages, page, G, Dv) * 50).to(dtype)
    kg, vg = kpool.cuda(), vpool.cuda()
    q, k, v = torch.randn(N, H, D).to(dtype), torch.randn(N, G, D).to(dtype), torch.randn(N, G, Dv).to(dtype)
    gate = torch.randn(N, H).to(dtype)
    slopes = paged_attention.distance_slopes(H)
    paged_attention.paged_kv_write(k.cuda(), v.cuda(), kg, vg, gb)
    paged_attention.paged_kv_write(k, v, kpool, vpool, cb)
    torch.testing.assert_close(kg.cpu(), kpool)
    out = paged_attention.paged_attention(q.cuda(), kg, vg, gb, 0.2, window, keep, slopes.cuda(), gate.cuda())
    ref = paged_attention.paged_attention_ref(q, kpool, vpool, cb, 0.2, window, keep, slopes, gate)
    if dtype == torch.bfloat16:  # decode-only step: the scalar kernel on the same pages
        dec = RaggedBatch.build([1] * 3, [36, 25, 63], [3, 0, 5], "cuda", [t.tolist() for t in gb.block_tables[:3]], page)
        qd = q[[36, 41, 42]]
        one = paged_attention.paged_attention(qd.cuda(), kg, vg, dec, 0.2, window, keep, slopes.cuda(), None)
        dec_c = RaggedBatch.build([1] * 3, [36, 25, 63], [3, 0, 5], "cpu", [t.tolist() for t in gb.block_tables[:3]], page)
        torch.testing.assert_close(one.cpu().float(),
                                   paged_attention.paged_attention_ref(qd, kpool, vpool, dec_c, 0.2, window, keep, slopes, None).float(),
                                   rtol=2e-2, atol=0.5)
    # values are ~50 in size: absolute tolerances scale with them
    torch.testing.assert_close(out.cpu().float(), ref.float(), **(dict(rtol=2e-2, atol=0.5) if dtype == torch.bfloat16
                                                                 else dict(rtol=1e-4, atol=2e-3)))


def test_activations():
    x = torch.randn(1000)
    torch.testing.assert_close(relu_squared(x.cuda()).cpu(), torch.relu(x).square())
    xb = x.bfloat16()
    torch.testing.assert_close(relu_squared(xb.cuda()).cpu(), torch.relu(xb).square())
    torch.testing.assert_close(softcap(x.cuda() * 20, 15.0).cpu(), 15.0 * torch.tanh(x * 20 / 15.0), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("counts", [[200, 100], [90, 60], [7, 3]])
def test_paged_attention_heads_per_block(counts):
    """The scalar kernel picks how many query heads of a group share a block
    from the size of the step (4, 2 or 1): all three must agree with the
    reference (float32, 4 query heads on one kv head)."""
    torch.manual_seed(8)
    H, G, D, Dv, page = 4, 1, 24, 20, 16
    starts = [5, 0]
    tables, nxt = [], 0
    for c, s in zip(counts, starts):
        need = (c + s + page - 1) // page
        tables.append(list(range(nxt, nxt + need)))
        nxt += need
    gb = RaggedBatch.build(counts, starts, [0, 1], "cuda", tables, page)
    cb = RaggedBatch.build(counts, starts, [0, 1], "cpu", tables, page)
    kpool, vpool = torch.randn(nxt, page, G, D), torch.randn(nxt, page, G, Dv)
    q = torch.randn(gb.num_tokens, H, D)
    slopes = paged_attention.distance_slopes(H)
    out = paged_attention.paged_attention(q.cuda(), kpool.cuda(), vpool.cuda(), gb, 0.3, 50, 3, slopes.cuda(), None)
    ref = paged_attention.paged_attention_ref(q, kpool, vpool, cb, 0.3, 50, 3, slopes, None)
    torch.testing.assert_close(out.cpu(), ref, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("page", [16, 64])
@pytest.mark.parametrize("H,G,D,Dv,cap", [(6, 2, 48, 96, 8.0), (4, 2, 40, 80, 0.0), (2, 1, 96, 72, 3.0), (8, 2, 64, 64, 40.0),
                                          (3, 3, 24, 44, 5.0), (4, 4, 128, 128, 30.0), (4, 2, 16, 8, 1.0),
                                          (2, 2, 104, 120, 12.0)])
def test_paged_attention_softcap_and_sink(dtype, H, G, D, Dv, cap, page):
    """Soft-capped scores and the sink's place in the denominator, in the scalar
    kernel and in the matrix-core kernel (bfloat16; head sizes that are
    multiples of 8 ride zero-padded in the next larger tiling)."""
    torch.manual_seed(9)
    gb, cb, pages = make_batch("cuda", page)
    N = gb.num_tokens
    kpool, vpool = (torch.randn(pages, page, G, D) * 3).to(dtype), (torch.randn(pages, page, G, Dv) * 50).to(dtype)
    kg, vg = kpool.cuda(), vpool.cuda()
    q, k, v = torch.randn(N, H, D).to(dtype), torch.randn(N, G, D).to(dtype), torch.randn(N, G, Dv).to(dtype)
    paged_attention.paged_kv_write(k.cuda(), v.cuda(), kg, vg, gb)
    paged_attention.paged_kv_write(k, v, kpool, vpool, cb)
    loose = dict(rtol=2e-2, atol=0.5) if dtype == torch.bfloat16 else dict(rtol=1e-4, atol=2e-3)
    for sink in (True, False):
        out = paged_attention.paged_attention(q.cuda(), kg, vg, gb, 0.3, softcap=cap, sink=sink)
        ref = paged_attention.paged_attention_ref(q, kpool, vpool, cb, 0.3, softcap=cap, sink=sink)
        torch.testing.assert_close(out.cpu().float(), ref.float(), **loose)
    # decode-only step: the scalar kernel on the same pages
    tabs = [t.tolist() for t in gb.block_tables[:3]]
    dec = RaggedBatch.build([1] * 3, [36, 25, 63], [3, 0, 5], "cuda", tabs, page)
    dec_c = RaggedBatch.build([1] * 3, [36, 25, 63], [3, 0, 5], "cpu", tabs, page)
    qd = q[[36, 41, 42]]
    one = paged_attention.paged_attention(qd.cuda(), kg, vg, dec, 0.3, softcap=cap, sink=True)
    torch.testing.assert_close(one.cpu().float(),
                               paged_attention.paged_attention_ref(qd, kpool, vpool, dec_c, 0.3, softcap=cap, sink=True).float(),
                               **loose)


@pytest.mark.parametrize("cap", [2.0, 60.0, 66.0, 70.0])
def test_saturated_softcap_with_sink(cap):
    """Scores pushed against both ends of the cap. With a sink and a cap the matrix-core kernel takes its
    weights against the fixed reference 0 as long as exp2 of the cap cannot overflow (cap <= 66.5) and against
    a running maximum beyond; either way keys at -cap vanish beside keys at +cap and beside the sink."""
    torch.manual_seed(16)
    H, G, D, Dv, page = 4, 2, 64, 64, 16
    gb, cb, pages = make_batch("cuda", page)
    N = gb.num_tokens
    kpool, vpool = torch.randn(pages, page, G, D).bfloat16(), torch.randn(pages, page, G, Dv).bfloat16()
    kg, vg = kpool.cuda(), vpool.cuda()
    q, k, v = (torch.randn(N, H, D) * 40).bfloat16(), torch.randn(N, G, D).bfloat16(), torch.randn(N, G, Dv).bfloat16()
    q[::3] = -q[::3].abs() * k[::3].repeat_interleave(H // G, 1).sign()   # these tokens score themselves near -cap
    paged_attention.paged_kv_write(k.cuda(), v.cuda(), kg, vg, gb)
    paged_attention.paged_kv_write(k, v, kpool, vpool, cb)
    out = paged_attention.paged_attention(q.cuda(), kg, vg, gb, 1.0, softcap=cap, sink=True)
    ref = paged_attention.paged_attention_ref(q, kpool, vpool, cb, 1.0, softcap=cap, sink=True)
    assert torch.isfinite(out).all()
    torch.testing.assert_close(out.cpu().float(), ref.float(), rtol=3e-2, atol=3e-2)


def test_sink_with_tiny_scores_halves_nothing_by_accident():
    """Scores of exactly 0 for t visible keys: every weight is 1 / (t + 1)."""
    page, T, D, Dv = 16, 40, 32, 32
    b = RaggedBatch.build([T], [0], [0], "cuda", [[2, 0, 1]], page)
    kpool = torch.zeros(3, page, 1, D, dtype=torch.bfloat16, device="cuda")
    vpool = torch.ones(3, page, 1, Dv, dtype=torch.bfloat16, device="cuda")
    q = torch.randn(T, 2, D, dtype=torch.bfloat16, device="cuda")
    out = paged_attention.paged_attention(q, kpool, vpool, b, 1.0, softcap=7.0, sink=True).float().cpu()
    want = torch.arange(1, T + 1).float() / torch.arange(2, T + 2).float()
    torch.testing.assert_close(out[:, 0, 0], want, rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("W", [96, 1000, 2600, 5000, 100, 9000])  # rows held in registers (1, 2, 4 chunks), re-read rows
def test_add_rms_norm(dtype, W):
    torch.manual_seed(10)
    x, w = torch.randn(19, W) * 4, torch.randn(W)
    a, b = torch.randn(19, W).to(dtype), torch.randn(19, W)  # the second addend may be float32
    rg, rc = x.clone().cuda(), x.clone()
    hg = group_norm.add_rms_norm(rg, a.cuda(), b.cuda(), w.cuda(), 1e-5, dtype)
    hc = group_norm.add_rms_norm_ref(rc, a, b, w, 1e-5, dtype)
    torch.testing.assert_close(rg.cpu(), rc, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(hg.cpu().float(), hc.float(), **tol(dtype))
    rg2, rc2 = x.clone().cuda(), x.clone()
    assert group_norm.add_rms_norm(rg2, a.cuda(), None, None, 1e-5) is None
    group_norm.add_rms_norm_ref(rc2, a, None, None, 1e-5)
    torch.testing.assert_close(rg2.cpu(), rc2, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("dtype", DTYPES)
def test_silu_mul(dtype):
    torch.manual_seed(11)
    y = (torch.randn(33, 2 * 150 + 10) * 3).to(dtype)
    out = silu_mul(y.cuda()[:, 10:])
    g, u = y[:, 10:160].float(), y[:, 160:].float()
    torch.testing.assert_close(out.cpu().float(), (g * torch.sigmoid(g) * u).to(dtype).float(), **tol(dtype))


@pytest.mark.parametrize("E,top,groups,keep", [(12, 2, 3, 2), (64, 6, 8, 3), (256, 8, 8, 4), (7, 3, 1, 1), (9, 2, 9, 5),
                                               (160, 6, 1, 1)])
def test_grouped_topk_route(E, top, groups, keep):
    torch.manual_seed(12)
    z = torch.randn(301, E) * 2
    corr = torch.randn(E) * 0.4
    ids, w = routed_experts.grouped_topk_route(z.cuda(), corr.cuda(), top, groups, keep, 2, 1e-20)
    ids_r, w_r = routed_experts.grouped_topk_route_ref(z, corr, top, groups, keep, 2, 1e-20)
    same = (ids.cpu() == ids_r).all(-1)
    assert same.float().mean().item() > 0.99  # a sigmoid that differs in its last bit may swap a near-tie
    torch.testing.assert_close(w.cpu()[same], w_r[same], rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("N,W,Fe,E,top,shared", [(7, 256, 96, 8, 2, True), (3, 100, 36, 5, 3, False), (1, 512, 200, 4, 4, True),
                                               (300, 256, 128, 6, 2, True), (200, 96, 40, 16, 1, False),
                                               (700, 64, 32, 6, 2, True), (1100, 40, 24, 3, 1, False),
                                               (2200, 40, 24, 3, 1, False), (900, 160, 96, 40, 4, True)])
def test_routed_expert_ffn(dtype, N, W, Fe, E, top, shared):
    """Few pairs: matrix-vector kernels. Many: in bfloat16 with sizes that are multiples of 32 the grouped
    matrix-core product (device-side sort, no host round trip), else matrix-vector kernels again and, past their
    limit, sorted per-expert library products."""
    torch.manual_seed(13)
    h = torch.randn(N, W).to(dtype)
    w_up = (torch.randn(E, Fe, W) / W ** 0.5).to(dtype)
    w_down = (torch.randn(E, W, Fe) / Fe ** 0.5).to(dtype)
    ids = torch.stack([torch.randperm(E)[:top] for _ in range(N)]).int()
    wts = torch.rand(N, top)
    base = torch.randn(N, W).to(dtype) if shared else None
    out = routed_experts.routed_expert_ffn(h.cuda(), w_up.cuda(), w_down.cuda(), ids.cuda(), wts.cuda(),
                                           None if base is None else base.cuda())
    ref = routed_experts.routed_expert_ffn_ref(h.float(), w_up.float(), w_down.float(), ids, wts,
                                               None if base is None else base.float())
    assert out.dtype == torch.float32
    torch.testing.assert_close(out.cpu(), ref, **(dict(rtol=3e-2, atol=3e-2) if dtype == torch.bfloat16
                                                  else dict(rtol=1e-4, atol=1e-4)))


@pytest.mark.parametrize("M,K", [(128, 64), (96, 32), (200, 160), (384, 1024)])
def test_expert_grouped_gemm(M, K):
    """Row ranges of very different sizes, experts without rows at both ends and in the middle, output widths that
    are no multiple of the tile, with and without the row gather and the squared-ReLU epilogue."""
    from colossalai_amd.ops._kernels import serving_kernels

    torch.manual_seed(14)
    counts = [0, 5, 0, 300, 1, 129, 0, 128, 64, 0]
    E, P = len(counts), sum(counts)
    offsets = torch.tensor([0] + torch.tensor(counts).cumsum(0).tolist(), dtype=torch.int32)
    w = (torch.randn(E, M, K) / K ** 0.5).bfloat16()
    src_rows = torch.randint(0, 50, (P,), dtype=torch.int32)
    a_small, a_full = torch.randn(50, K).bfloat16(), torch.randn(P, K).bfloat16()
    for a, rows, act in ((a_small, src_rows, True), (a_full, None, False)):
        out = serving_kernels().expert_grouped_gemm(a.cuda(), None if rows is None else rows.cuda(), w.cuda(),
                                                    offsets.cuda(), P, act)
        x = a.float() if rows is None else a.float()[rows.long()]
        ref = torch.empty(P, M)
        for e in range(E):
            lo, hi = int(offsets[e]), int(offsets[e + 1])
            ref[lo:hi] = x[lo:hi] @ w[e].float().t()
        if act:
            ref = torch.relu(ref).square()
        torch.testing.assert_close(out.cpu().float(), ref, rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("N,top,E", [(1, 1, 1), (40, 3, 7), (1000, 6, 32), (2048, 4, 200), (77, 1, 3)])
def test_expert_sort(N, top, E):
    from colossalai_amd.ops._kernels import serving_kernels

    torch.manual_seed(15)
    ids = torch.randint(0, E, (N, top), dtype=torch.int32)
    if E > 2:
        ids[ids == 1] = 2  # an expert without rows
    offsets, src, inv = (t.cpu() for t in serving_kernels().expert_sort(ids.cuda(), E))
    order, inv_ref, offsets_ref = routed_experts._sort_pairs(ids, E)
    assert offsets.tolist() == offsets_ref.tolist()
    assert src.tolist() == (order // top).tolist()
    assert inv.reshape(-1).tolist() == inv_ref.tolist()
