"""Kipirax against the slow float64 oracle (tests/kipirax_oracle.py): each
mechanism alone, then whole models of several small shapes. The CPU runs use
the library's PyTorch reference ops, the GPU runs its HIP kernels."""

import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import kipirax_oracle as O  # noqa: E402

from colossalai_amd.models import KipiraxForCausalLM, model_class_for  # noqa: E402
from colossalai_amd.ops import group_norm, linear_recurrence, paged_attention, short_conv, token_shift  # noqa: E402
from colossalai_amd.ops.ragged import RaggedBatch  # noqa: E402

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
F64 = torch.float64


def one_seq(T, device, page=4, slot=1):
    pages = (T + page - 1) // page
    return RaggedBatch.build([T], [0], [slot], device, [list(range(pages))[::-1]], page), pages


def close(got, want, tol=2e-4):
    want = want.to(torch.float32)
    err = (got.detach().cpu().float() - want).abs().max().item()
    assert err <= tol * max(1.0, want.abs().max().item()), f"max abs error {err}"


# ------------------------------------------------------------- mechanisms
@pytest.mark.parametrize("device", DEVICES)
def test_token_shift_alone(device):
    torch.manual_seed(0)
    x, mu = torch.randn(9, 24), torch.rand(24)
    b, _ = one_seq(9, device)
    prev = torch.full((3, 24), 7.0, device=device)  # stale slot contents must not be seen at position 0
    got = token_shift.token_shift(x.to(device), mu.to(device), prev, b, torch.float32)
    close(got, O.token_shift(x.to(F64), mu))
    close(prev[1], x[-1])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("groups", [1, 2, 5])
def test_grouped_norm_alone(device, groups):
    torch.manual_seed(1)
    x, w = torch.randn(6, 40) * 3, torch.randn(40)
    got = group_norm.grouped_rms_norm(x.to(device), w.to(device), groups, 1e-3)
    close(got, O.grouped_rms_norm(x.to(F64), w, groups, 1e-3))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("K", [2, 4])
def test_short_conv_alone(device, K):
    torch.manual_seed(2)
    x, taps = torch.randn(11, 10), torch.randn(10, K)
    b, _ = one_seq(11, device)
    tail = torch.full((3, K - 1, 10), 5.0, device=device)
    got = short_conv.short_conv(x.to(device), taps.to(device), tail, b, True)
    close(got, O.silu(O.causal_short_conv(x.to(F64), taps.to(F64))))
    close(tail[1], x[-(K - 1):])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,G", [(4, 2), (3, 3), (2, 1)])
def test_gated_delta_alone(device, H, G):
    torch.manual_seed(3)
    T, D, Dv = 13, 12, 10
    q, k, v = torch.randn(T, G, D), torch.randn(T, G, D), torch.randn(T, H, Dv)
    bl, dt, A, bias = torch.randn(T, H), torch.randn(T, H * D), torch.randn(H) - 1, torch.randn(H * D)
    b, _ = one_seq(T, device)
    state = torch.full((3, H, D, Dv), 9.0, device=device)
    got = linear_recurrence.gated_delta_rule(*(t.to(device) for t in (q, k, v, bl, dt, A, bias)), state, b,
                                             1e-6, D ** -0.5)
    q64, k64 = q.to(F64), k.to(F64)
    qn = (q64 / torch.sqrt((q64 * q64).sum(-1, keepdim=True) + 1e-6) * D ** -0.5).repeat_interleave(H // G, 1)
    kn = (k64 / torch.sqrt((k64 * k64).sum(-1, keepdim=True) + 1e-6)).repeat_interleave(H // G, 1)
    g = torch.exp(-torch.exp(A.to(F64))[None, :, None] * O.softplus(dt.to(F64).reshape(T, H, D) + bias.to(F64).reshape(H, D)))
    close(got, O.gated_delta_scan(qn, kn, v.to(F64), O.sigmoid(bl.to(F64)), g))


@pytest.mark.parametrize("device", DEVICES)
def test_tied_gate_alone(device):
    torch.manual_seed(4)
    T, H, D, Dv = 13, 3, 20, 6
    q, f, v, fb, low = torch.randn(T, H, D), torch.randn(T, H, D), torch.randn(T, H, Dv), torch.randn(H * D), torch.rand(H * D)
    b, _ = one_seq(T, device)
    state = torch.full((3, H, D, Dv), 9.0, device=device)
    got = linear_recurrence.tied_gate_recurrence(*(t.to(device) for t in (q, f, v, fb, low)), state, b)
    l64 = low.to(F64).reshape(H, D)
    f64 = l64 + (1 - l64) * O.sigmoid(f.to(F64) + fb.to(F64).reshape(H, D))
    close(got, O.hgrn2_scan(O.silu(q.to(F64)), f64, v.to(F64)))


def attention_case(device, T, H, G, D, Dv, window, keep, q, k, v, page=4):
    b, pages = one_seq(T, device, page)
    kpool = torch.zeros(pages, page, G, D, device=device)
    vpool = torch.zeros(pages, page, G, Dv, device=device)
    paged_attention.paged_kv_write(k.to(device), v.to(device), kpool, vpool, b)
    return paged_attention.paged_attention(q.to(device), kpool, vpool, b, 0.3, window, keep,
                                           paged_attention.distance_slopes(H, device), None)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("window,keep", [(5, 2), (5, 0), (1, 3), (0, 0), (40, 4)])
def test_window_attention_alone(device, window, keep):
    torch.manual_seed(5)
    T, H, G, D, Dv = 23, 4, 2, 8, 6
    q, k, v = torch.randn(T, H, D), torch.randn(T, G, D), torch.randn(T, G, Dv)
    got = attention_case(device, T, H, G, D, Dv, window, keep, q, k, v)
    want = O.windowed_bias_attention(q.to(F64), k.to(F64), v.to(F64), 0.3, window if window else T + 1, keep)
    close(got, want)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("spike", ["window_in", "window_out", "keep_in", "keep_out", "page_edge"])
def test_window_edges_stand_out(device, spike):
    """One key is made to dominate the scores of the last query; whether it is
    seen decides the output, so an edge that is one token off cannot hide."""
    torch.manual_seed(6)
    T, H, G, D, Dv, window, keep = 40, 2, 1, 8, 4, 9, 3
    j = {"window_in": T - window, "window_out": T - 1 - window, "keep_in": keep - 1, "keep_out": keep,
         "page_edge": T - 1 - 4}[spike]
    q, k, v = torch.randn(T, H, D) * 0.1, torch.randn(T, G, D) * 0.1, torch.randn(T, G, Dv)
    k[j] = 0.0
    k[j, :, 0] = 30.0
    q[T - 1, :, 0] = 30.0
    got = attention_case(device, T, H, G, D, Dv, window, keep, q, k, v)
    want = O.windowed_bias_attention(q.to(F64), k.to(F64), v.to(F64), 0.3, window, keep)
    seen = spike in ("window_in", "keep_in", "page_edge")
    dominated = (want[T - 1, 0] - v[j, 0].to(F64)).abs().max().item() < 1e-3
    assert dominated == seen
    close(got, want)


# ------------------------------------------------------------------ models
def cfg_small(order, width=24, groups=3, left=None, right=None, delta=None, ff=40, softcap=7.0, no_mlp_at=()):
    left = left or dict(dim=8, heads=4, kv_heads=2, vdim=6, scale=0.4, mask=dict(size=7, keep_first=2))
    right = right or dict(dim=6, heads=2, vdim=10)
    delta = delta or dict(conv=3, dim=6, heads=4, kv_heads=2, vdim=8)
    layers = []
    for i, t in enumerate(order):
        mixer = dict(left=left, right=right) if t == "parallel" else delta
        layers.append(dict(type=t, mixer=mixer, mlp=None if i in no_mlp_at else dict(kind="dense", ff=ff)))
    return dict(architecture="Kipirax", vocab=50, width=width, max_positions=128, layers=layers,
                norm=dict(eps=1e-5, groups=groups), logit_softcap=softcap)


CONFIGS = {
    "mixed-order": cfg_small(["channel_delta", "parallel", "parallel", "channel_delta"]),
    "one-group-one-kv-head": cfg_small(["parallel", "channel_delta"], groups=1,
                                       left=dict(dim=4, heads=3, kv_heads=1, vdim=12, scale=1.0,
                                                 mask=dict(size=3, keep_first=0)),
                                       right=dict(dim=16, heads=1, vdim=4),
                                       delta=dict(conv=2, dim=20, heads=2, kv_heads=1, vdim=4), no_mlp_at=(0,)),
    "wide-window-many-taps": cfg_small(["channel_delta", "channel_delta", "parallel"], width=40, groups=5,
                                       left=dict(dim=8, heads=2, kv_heads=2, vdim=8, scale=0.2,
                                                 mask=dict(size=64, keep_first=9)),
                                       delta=dict(conv=6, dim=8, heads=3, kv_heads=3, vdim=4), softcap=30.0),
}


def build(name, device, dtype=torch.float32, seed=0):
    cfg = CONFIGS[name]
    P = O.random_weights(cfg, seed)
    assert model_class_for(cfg) is KipiraxForCausalLM
    return cfg, P, KipiraxForCausalLM.from_checkpoint(cfg, P, dtype=dtype, device=device)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_whole_prompt_matches_oracle(device, name):
    cfg, P, model = build(name, device)
    torch.manual_seed(7)
    toks = torch.randint(0, cfg["vocab"], (2, 29))
    got = model(toks.to(device))
    for b in range(2):
        want, layers = O.forward(cfg, P, toks[b].tolist(), return_layers=True)
        close(got[b], want, 3e-4)


@pytest.mark.gpu
def test_bfloat16_model_close_to_oracle():
    cfg, P, model = build("mixed-order", "cuda", torch.bfloat16)
    toks = torch.randint(0, cfg["vocab"], (1, 29), generator=torch.Generator().manual_seed(1))
    got = model(toks.cuda())[0].cpu()
    want = O.forward(cfg, P, toks[0].tolist()).float()
    d = got - want
    assert ((d - d.mean(-1, keepdim=True)).pow(2).mean().sqrt() / want.std()).item() < 0.06


def test_checkpoint_names_are_all_used_and_required():
    cfg, P, _ = build("mixed-order", "cpu")
    extra = dict(P, **{"l0.mix.unknown": torch.zeros(1)})
    with pytest.raises(ValueError):
        KipiraxForCausalLM.from_checkpoint(cfg, extra, dtype=torch.float32)
    fewer = {k: v for k, v in P.items() if k != "l1.mix.left.q.norm"}
    with pytest.raises(KeyError):
        KipiraxForCausalLM.from_checkpoint(cfg, fewer, dtype=torch.float32)
