"""HIP serving kernels against their float32 PyTorch references (same op,
run on CPU copies of the inputs): ragged batches that mix fresh sequences,
continued sequences and single decode tokens, in bfloat16 and float32."""

import pytest
import torch

from colossalai_amd.ops import group_norm, linear_recurrence, paged_attention, short_conv, token_shift
from colossalai_amd.ops.activation import relu_squared, softcap
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
