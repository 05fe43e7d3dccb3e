"""Mubutar against the slow float64 oracle (tests/mubutar_oracle.py): each
mechanism alone, then whole models of several small shapes. The CPU runs use
the library's PyTorch reference ops, the GPU runs its HIP kernels."""

import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import mubutar_oracle as O  # noqa: E402

from colossalai_amd.inference.kv_cache import KVCacheManager  # noqa: E402
from colossalai_amd.models import MubutarForCausalLM, model_class_for  # noqa: E402
from colossalai_amd.ops import activation, group_norm, paged_attention, routed_experts  # noqa: E402
from colossalai_amd.ops.ragged import RaggedBatch  # noqa: E402

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
F64 = torch.float64


def close(got, want, tol=2e-4):
    want = want.to(torch.float32)
    err = (got.detach().cpu().float() - want).abs().max().item()
    assert err <= tol * max(1.0, want.abs().max().item()), f"max abs error {err}"


def paged(k, v, device, page, cut=None, dtype=torch.float32):
    """Put k [T, G, D] / v [T, G, Dv] of one sequence into pools whose pages lie
    in reverse order; the batch describes the last ``T - cut`` tokens as new
    (all of them when cut is None)."""
    T = k.shape[0]
    pages = (T + page - 1) // page
    table = list(range(pages))[::-1]
    start = 0 if cut is None else cut
    b = RaggedBatch.build([T - start], [start], [0], device, [table], page)
    kpool = torch.zeros(pages, page, *k.shape[1:], device=device, dtype=dtype)
    vpool = torch.zeros(pages, page, *v.shape[1:], device=device, dtype=dtype)
    full = RaggedBatch.build([T], [0], [0], device, [table], page)
    paged_attention.paged_kv_write(k.to(device, dtype), v.to(device, dtype), kpool, vpool, full)
    return b, kpool, vpool, start


# ------------------------------------------------------------- mechanisms
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,G,D,Dv,cap", [(4, 2, 8, 6, 3.0), (3, 3, 5, 9, 0.0), (6, 1, 16, 4, 0.7), (2, 2, 64, 64, 20.0)])
def test_sink_softcap_attention_alone(device, H, G, D, Dv, cap):
    torch.manual_seed(0)
    T = 21
    q, k, v = torch.randn(T, H, D), torch.randn(T, G, D), torch.randn(T, G, Dv)
    b, kpool, vpool, _ = paged(k, v, device, 4)
    got = paged_attention.paged_attention(q.to(device), kpool, vpool, b, 0.6, softcap=cap, sink=True)
    close(got, O.sink_softcap_attention(q.to(F64), k.to(F64), v.to(F64), 0.6, cap))


@pytest.mark.parametrize("device", DEVICES)
def test_sink_takes_the_weight_when_no_key_fits(device):
    """All scores far below 0: the sink's place in the denominator takes nearly
    all the weight and the output shrinks towards zero; an ordinary softmax
    would return an average of the values instead."""
    torch.manual_seed(1)
    T, H, D, Dv = 9, 2, 8, 8
    k = torch.randn(T, H, D)
    q = -4.0 * k  # q . k = -4 |k|^2
    v = torch.ones(T, H, Dv)
    b, kpool, vpool, _ = paged(k, v, device, 4)
    got = paged_attention.paged_attention(q.to(device), kpool, vpool, b, 1.0, softcap=0.0, sink=True)
    want = O.sink_softcap_attention(q.to(F64), k.to(F64), v.to(F64), 1.0, 0.0)
    close(got, want, 1e-5)
    plain = paged_attention.paged_attention(q.to(device), kpool, vpool, b, 1.0)
    assert plain.min().item() > 0.99  # the values' average, as every value is 1
    # the causal mask is part of it: only keys j <= i count, and for late tokens some
    # earlier key can score high by chance, so test the first token alone
    assert got[0].abs().max().item() < 0.5


@pytest.mark.parametrize("device", DEVICES)
def test_softcap_bounds_a_spiked_score(device):
    """One huge score: without the cap its key takes everything, with the cap
    it only leads by exp(cap - others)."""
    torch.manual_seed(2)
    T, D, Dv, cap = 12, 8, 4, 2.0
    q, k, v = torch.randn(T, 1, D) * 0.1, torch.randn(T, 1, D) * 0.1, torch.randn(T, 1, Dv)
    q[-1, 0], k[3, 0] = 30.0, 30.0
    b, kpool, vpool, _ = paged(k, v, device, 4)
    got = paged_attention.paged_attention(q.to(device), kpool, vpool, b, 1.0, softcap=cap, sink=True)
    close(got, O.sink_softcap_attention(q.to(F64), k.to(F64), v.to(F64), 1.0, cap))
    free = paged_attention.paged_attention(q.to(device), kpool, vpool, b, 1.0, sink=True)
    close(free[-1, 0], v[3, 0], 1e-4)
    assert (got[-1, 0].cpu() - v[3, 0]).abs().max().item() > 0.05


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("far", [0, 3, 4, 63, 64, 255, 256, 300])
@pytest.mark.parametrize("decode", [False, True])
def test_far_key_among_hundreds(device, far, decode):
    """The last query matches exactly one key (scaled so that its score stands
    out): at the very start, at page borders, hundreds of tokens back. The
    output must be that key's value, in a prompt and when decoded alone."""
    torch.manual_seed(3)
    T, H, G, D, Dv = 310, 2, 1, 8, 6
    q, k, v = torch.randn(T, H, D) * 0.05, torch.randn(T, G, D) * 0.05, torch.randn(T, G, Dv)
    unit = torch.zeros(D)
    unit[far % D] = 1.0
    q[-1, :], k[far, 0] = unit * 6.0, unit * 6.0   # score 36 * scale against ~0 elsewhere
    b, kpool, vpool, start = paged(k, v, device, 64 if far >= 63 else 4, cut=T - 1 if decode else None)
    got = paged_attention.paged_attention(q[start:].to(device), kpool, vpool, b, 0.5, softcap=30.0, sink=True)
    for h in range(H):
        close(got[-1, h], v[far, 0], 2e-3)


@pytest.mark.parametrize("device", DEVICES)
def test_add_rms_norm_alone(device):
    torch.manual_seed(4)
    x, a, b, w = torch.randn(7, 40) * 3, torch.randn(7, 40), torch.randn(7, 40), torch.randn(40)
    res = x.clone().to(device)
    h = group_norm.add_rms_norm(res, a.to(device), b.to(device), w.to(device), 1e-3, torch.float32)
    s = (x + a + b).to(F64)
    close(res, s, 1e-6)
    close(h, O.rms_norm(s, w, 1e-3))
    res2 = x.clone().to(device)
    assert group_norm.add_rms_norm(res2, a.to(device), None, None, 1e-3) is None
    close(res2, (x + a).to(F64), 1e-6)


@pytest.mark.parametrize("device", DEVICES)
def test_gated_silu_alone(device):
    torch.manual_seed(5)
    y = torch.randn(5, 2 * 12) * 2
    wide = torch.randn(5, 30)
    wide[:, 3:27] = y  # a column view: rows are strided
    got = activation.silu_mul(wide.to(device)[:, 3:27])
    g, u = y[:, :12].to(F64), y[:, 12:].to(F64)
    close(got, g * O.sigmoid(g) * u, 1e-5)


ROUTER_CASES = [
    # E, top, groups, keep
    (12, 2, 3, 2), (8, 3, 1, 1), (6, 2, 6, 3), (16, 4, 4, 4), (10, 1, 5, 1), (64, 6, 8, 3), (130, 5, 2, 1),
]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("E,top,groups,keep", ROUTER_CASES)
def test_router_alone(device, E, top, groups, keep):
    torch.manual_seed(6)
    z = torch.randn(9, E) * 2
    corr = torch.randn(E) * 0.5
    ids, w = routed_experts.grouped_topk_route(z.to(device), corr.to(device), top, groups, keep, 2, 1e-20)
    for t in range(z.shape[0]):
        chosen, weights = O.route(z[t].to(F64), corr, top, groups, keep)
        assert ids[t].tolist() == chosen
        close(w[t], torch.tensor(weights, dtype=F64), 1e-5)


@pytest.mark.parametrize("device", DEVICES)
def test_router_negative_choice_scores_stay_in_their_group(device):
    """A correction that pushes every choice score below zero: a dropped group
    counts as minus infinity, not 0, so the choice still falls inside the kept
    groups; the weights come from the scores without the correction."""
    E, top, groups, keep = 8, 2, 4, 1
    z = torch.tensor([[0.1, 0.2, 2.0, 1.5, -1.0, 0.3, 0.0, 0.4]])
    corr = torch.full((E,), -3.0)
    ids, w = routed_experts.grouped_topk_route(z.to(device), corr.to(device), top, groups, keep, 2, 1e-20)
    assert ids[0].tolist() == [2, 3]
    s = torch.sigmoid(z[0, [2, 3]].to(F64))
    close(w[0], s / s.sum(), 1e-6)
    # a correction can move the choice without moving the weights
    corr2 = torch.zeros(E)
    corr2[4] = 5.0
    ids2, w2 = routed_experts.grouped_topk_route(z.to(device), corr2.to(device), 1, 1, 1, 2, 1e-20)
    assert ids2[0].tolist() == [4]
    close(w2[0], torch.ones(1, dtype=F64), 1e-6)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("N,W,Fe,E,top,shared", [(5, 24, 16, 6, 2, True), (3, 20, 7, 4, 3, False),
                                               (150, 32, 24, 5, 2, True), (200, 24, 8, 3, 1, False)])
def test_expert_feed_forward_alone(device, N, W, Fe, E, top, shared):
    """Few pairs take the matrix-vector kernels on the GPU, many the sorted
    per-expert products; both against the per-token loop."""
    torch.manual_seed(7)
    h = torch.randn(N, W)
    P = {f"e{e}.up": torch.randn(Fe, W) / W ** 0.5 for e in range(E)}
    P.update({f"e{e}.down": torch.randn(W, Fe) / Fe ** 0.5 for e in range(E)})
    ids = torch.stack([torch.randperm(E)[:top] for _ in range(N)]).int()
    wts = torch.rand(N, top)
    base = torch.randn(N, W) if shared else None
    w_up = torch.stack([P[f"e{e}.up"] for e in range(E)])
    w_down = torch.stack([P[f"e{e}.down"] for e in range(E)])
    got = routed_experts.routed_expert_ffn(h.to(device), w_up.to(device), w_down.to(device), ids.to(device),
                                           wts.to(device), None if base is None else base.to(device))
    want = torch.zeros(N, W, dtype=F64) if base is None else base.to(F64).clone()
    for n in range(N):
        for j in range(top):
            want[n] += wts[n, j].to(F64) * O.expert_ff(h[n].to(F64), P, f"e{int(ids[n, j])}.")
    close(got, want, 1e-4)


# ------------------------------------------------------------ whole models
ATT = dict(dim=8, heads=4, kv_heads=2, vdim=6, scale=0.4, softcap=5.0)
MOE = dict(kind="moe", expert=dict(ff=12), router=dict(experts=6, top=2, groups=dict(count=3, keep=2)),
           shared=dict(ff=10))
SHAPES = {
    "shared-keys-moe": dict(vocab=50, width=24, embedding=dict(scale=3.0), logit_scale=0.5, norm=dict(eps=1e-5),
                            layers=[dict(type="attention", mixer=ATT, mlp=dict(kind="dense", ff=40)),
                                    dict(type="attention", mixer=dict(ATT, kv_from=0), mlp=MOE),
                                    dict(type="attention", mixer=dict(ATT, kv_from=0), mlp=None)]),
    # one kv head, equal key/value sizes, no cap, top 1 without groups or shared expert, scales of 1
    "plain": dict(vocab=31, width=16, embedding=dict(scale=1.0), logit_scale=1.0, norm=dict(eps=1e-6),
                  layers=[dict(type="attention", mixer=dict(dim=4, heads=3, kv_heads=1, vdim=4, scale=0.5, softcap=0),
                               mlp=dict(kind="moe", expert=dict(ff=8), router=dict(experts=4, top=1), shared=None)),
                          dict(type="attention", mixer=dict(dim=4, heads=3, kv_heads=3, vdim=4, scale=0.5),
                               mlp=dict(kind="dense", ff=8))]),
    # every group kept, groups of one expert, layers that differ in head sizes, sharing from a middle layer
    "mixed-sizes": dict(vocab=40, width=32, embedding=dict(scale=0.5), logit_scale=3.0, norm=dict(eps=1e-4),
                        layers=[dict(type="attention", mixer=dict(dim=16, heads=2, kv_heads=2, vdim=8, scale=0.3, softcap=2.0),
                                     mlp=dict(kind="moe", expert=dict(ff=16),
                                              router=dict(experts=5, top=3, groups=dict(count=5, keep=4)),
                                              shared=dict(ff=8))),
                                dict(type="attention", mixer=dict(dim=8, heads=4, kv_heads=1, vdim=24, scale=0.6, softcap=9.0),
                                     mlp=None),
                                dict(type="attention", mixer=dict(dim=8, heads=4, kv_heads=1, vdim=24, scale=0.2, softcap=1.5,
                                                                  kv_from=1),
                                     mlp=dict(kind="dense", ff=24))]),
    # nothing a multiple of 8 or of the wave: scalar loads everywhere, three query heads on one kv head
    "odd-sizes": dict(vocab=37, width=36, embedding=dict(scale=1.7), logit_scale=0.9, norm=dict(eps=1e-6),
                      layers=[dict(type="attention", mixer=dict(dim=6, heads=3, kv_heads=1, vdim=5, scale=0.41, softcap=11.0),
                                   mlp=dict(kind="moe", expert=dict(ff=10), shared=dict(ff=7),
                                            router=dict(experts=9, top=4, groups=dict(count=3, keep=2)))),
                              dict(type="attention", mixer=dict(dim=6, heads=3, kv_heads=1, vdim=5, scale=0.41, softcap=11.0,
                                                                kv_from=0),
                                   mlp=dict(kind="dense", ff=21))]),
}


def full(cfg):
    return dict(cfg, architecture="Mubutar")


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", sorted(SHAPES))
def test_whole_model_matches_the_oracle(device, name):
    cfg = full(SHAPES[name])
    P = O.random_weights(cfg, seed=len(name))
    toks = torch.randint(0, cfg["vocab"], (2, 19), generator=torch.Generator().manual_seed(1))
    model = MubutarForCausalLM.from_checkpoint(cfg, P, dtype=torch.float32, device=device)
    got = model(toks.to(device))
    for b in range(2):
        close(got[b], O.forward(cfg, P, toks[b].tolist()), 3e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_residual_stream_after_every_layer(device):
    cfg = full(SHAPES["shared-keys-moe"])
    P = O.random_weights(cfg, seed=5)
    toks = list(range(3, 16))
    model = MubutarForCausalLM.from_checkpoint(cfg, P, dtype=torch.float32, device=device)
    kv = KVCacheManager(3, 0, 0, num_blocks=4, block_size=4, device=device, dtype=torch.float32,
                        layer_shapes=model.kv_layer_shapes(), layer_sources=model.kv_layer_sources())
    assert kv.k_pools[1] is kv.k_pools[0] and kv.v_pools[2] is kv.v_pools[0]
    b = RaggedBatch.build([len(toks)], [0], [0], device, [[2, 0, 3, 1]], 4)
    taps = []
    with torch.no_grad():
        model.forward_ragged(torch.tensor(toks, device=device), b, kv, None, None, taps)
    _, layers = O.forward(cfg, P, toks, return_layers=True)
    assert len(taps) == len(layers)
    for got, want in zip(taps, layers):
        close(got, want, 3e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(SHAPES))
def test_bfloat16_model_stays_near_the_oracle(name):
    """bfloat16 serving: matrices, keys and values in bfloat16, residual, norms,
    scores and router in float32."""
    cfg = full(SHAPES[name])
    P = {k: v.to(torch.bfloat16).float() for k, v in O.random_weights(cfg, seed=2).items()}
    toks = torch.randint(0, cfg["vocab"], (1, 40), generator=torch.Generator().manual_seed(2))
    model = MubutarForCausalLM.from_checkpoint(cfg, P, dtype=torch.bfloat16, device="cuda")
    got = model(toks.cuda())[0].float().cpu()
    want = O.forward(cfg, P, toks[0].tolist()).float()
    # a near-tie of the router may flip an expert under bfloat16 inputs: judge the bulk of the rows
    err = (got - want).pow(2).mean(-1).sqrt() / want.pow(2).mean().sqrt()
    assert err.median().item() < 0.03 and (err < 0.08).float().mean().item() > 0.8


def test_registry_and_config_round_trip():
    cfg = full(SHAPES["mixed-sizes"])
    assert model_class_for(cfg) is MubutarForCausalLM
    model = MubutarForCausalLM.from_checkpoint(cfg, O.random_weights(cfg), dtype=torch.float32)
    d = model.config.to_dict()
    assert d["architecture"] == "Mubutar" and d["embedding"]["scale"] == 0.5 and d["logit_scale"] == 3.0
    assert model.kv_layer_shapes() == [(2, 16, 8), (1, 8, 24), None]
    assert model.kv_layer_sources() == [None, None, 1]
    for layer in model.layers:  # the router stays float32 whatever the serving dtype
        if hasattr(layer.mlp, "router"):
            assert layer.mlp.router.dtype == torch.float32


def test_checkpoint_with_a_stray_or_missing_tensor_is_refused():
    cfg = full(SHAPES["plain"])
    P = O.random_weights(cfg)
    with pytest.raises(ValueError):
        MubutarForCausalLM.from_checkpoint(cfg, dict(P, **{"l0.mix.extra": torch.zeros(2)}), dtype=torch.float32)
    Q = dict(P)
    del Q["l1.mix.k.b"]
    with pytest.raises(KeyError):
        MubutarForCausalLM.from_checkpoint(cfg, Q, dtype=torch.float32)


def test_key_sharing_must_point_back_at_a_layer_with_keys():
    cfg = full(SHAPES["shared-keys-moe"])
    bad = dict(cfg, layers=[cfg["layers"][1], cfg["layers"][0]])
    with pytest.raises(ValueError):
        MubutarForCausalLM.from_checkpoint(bad, {}, dtype=torch.float32)
