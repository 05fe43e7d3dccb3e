"""Mixture-of-experts feed-forward of the serving path: a group-limited top-k
router and the experts' two-matrix feed-forward over a flat token batch.

``grouped_topk_route`` turns float32 router logits into expert ids and mixing
weights:

* score ``s = sigmoid(z)``; the *choice* score is ``s + correction`` (a
  per-expert selection bias), the mixing weights use ``s`` alone;
* the ``E`` experts form ``group_count`` runs of neighbours; a group is worth the
  sum of its ``group_top`` largest choice scores and only the ``group_keep``
  best groups stay in the running (the others count as minus infinity, so a
  negative choice score inside a kept group still beats them);
* the ``top`` largest remaining choice scores are chosen (ties go to the lower
  index) and their plain scores are divided by their sum plus ``renorm_eps``.

``routed_expert_ffn`` runs ``down_e(act(up_e(h)))`` for each token's chosen
experts and forms ``base + sum_j weight_j * y_j`` in float32. On the GPU a small
step (decode tokens) streams just the chosen experts' weights through a
matrix-vector kernel without touching the host; a large step (prompt portions)
sorts the (token, expert) pairs by expert and runs one matrix product per expert.
"""

from typing import Optional

import torch
import torch.nn.functional as F

from ._kernels import serving_kernels, use_serving_hip as use_hip
from .activation import relu_squared

__all__ = ["grouped_topk_route", "grouped_topk_route_ref", "routed_expert_ffn", "routed_expert_ffn_ref"]

# (token, expert) pairs up to which the matrix-vector kernels beat sorting + per-expert GEMMs
GEMV_MAX_PAIRS = 256


def grouped_topk_route_ref(logits, correction, top: int, group_count: int = 1, group_keep: int = 1,
                           group_top: int = 2, renorm_eps: float = 1e-20):
    N, E = logits.shape
    s = torch.sigmoid(logits.float())
    choice = s + correction.float()
    if group_count > 1:
        per = E // group_count
        grouped = choice.view(N, group_count, per)
        worth = grouped.topk(min(group_top, per), dim=-1).values.sum(-1)
        # stable descending order: ties go to the lower group
        kept = torch.sort(worth, dim=-1, descending=True, stable=True).indices[:, :group_keep]
        allowed = torch.zeros(N, group_count, dtype=torch.bool, device=logits.device)
        allowed.scatter_(1, kept, True)
        choice = grouped.masked_fill(~allowed[:, :, None], float("-inf")).reshape(N, E)
    idx = torch.sort(choice, dim=-1, descending=True, stable=True).indices[:, :top]
    w = s.gather(1, idx)
    return idx.int(), w / (w.sum(-1, keepdim=True) + renorm_eps)


def grouped_topk_route(logits, correction, top: int, group_count: int = 1, group_keep: int = 1,
                       group_top: int = 2, renorm_eps: float = 1e-20):
    """logits [N, E] float32, correction [E] -> (ids [N, top] int32, weights [N, top] float32)."""
    N, E = logits.shape
    assert E % group_count == 0 and 0 < group_keep <= group_count
    assert 0 < top <= (E // group_count) * group_keep, "fewer experts in the kept groups than are to be chosen"
    if use_hip(logits):
        return serving_kernels().grouped_topk_route(logits.float().contiguous(), correction, top, group_count,
                                                    group_keep, group_top, renorm_eps)
    return grouped_topk_route_ref(logits, correction, top, group_count, group_keep, group_top, renorm_eps)


def _act(x, activation: str):
    if activation == "relu_squared":
        return relu_squared(x)
    raise ValueError(f"unknown expert activation {activation!r}")


def routed_expert_ffn_ref(h, w_up, w_down, ids, weights, base=None, activation: str = "relu_squared"):
    N, top = ids.shape
    out = torch.zeros(N, w_down.shape[1], dtype=torch.float32, device=h.device) if base is None else base.float().clone()
    for e in range(w_up.shape[0]):
        rows, slot = (ids == e).nonzero(as_tuple=True)
        if rows.numel():
            y = F.linear(_act(F.linear(h[rows], w_up[e]), activation), w_down[e])
            out.index_add_(0, rows, y.float() * weights[rows, slot][:, None])
    return out


def _sorted_expert_ffn(h, w_up, w_down, ids, weights, base, activation):
    """Pairs sorted by expert, one up and one down product per expert that got
    rows, then every token gathers its ``top`` results in slot order."""
    N, top = ids.shape
    E = w_up.shape[0]
    flat = ids.reshape(-1).long()
    order = torch.argsort(flat, stable=True)
    counts = torch.bincount(flat, minlength=E).tolist()  # host: the products below are launched per expert
    x = h.index_select(0, order // top)
    hidden = torch.empty(x.shape[0], w_up.shape[1], dtype=h.dtype, device=h.device)
    at = 0
    for e, n in enumerate(counts):
        if n:
            torch.mm(x[at : at + n], w_up[e].t(), out=hidden[at : at + n])
            at += n
    hidden = _act(hidden, activation)
    y = torch.empty(x.shape[0], w_down.shape[1], dtype=h.dtype, device=h.device)
    at = 0
    for e, n in enumerate(counts):
        if n:
            torch.mm(hidden[at : at + n], w_down[e].t(), out=y[at : at + n])
            at += n
    inv = torch.empty_like(order)
    inv[order] = torch.arange(order.numel(), device=order.device)
    return serving_kernels().expert_combine(y, inv.int().view(N, top), weights, base)


def routed_expert_ffn(h, w_up, w_down, ids, weights, base: Optional[torch.Tensor] = None,
                      activation: str = "relu_squared"):
    """h [N, W]; w_up [E, F, W]; w_down [E, W, F]; ids [N, top] int32; weights
    [N, top] float32; ``base`` [N, W] (any activation type) is added, e.g. a
    shared expert's output. Returns float32 [N, W]."""
    if not use_hip(h):
        return routed_expert_ffn_ref(h, w_up, w_down, ids, weights, base, activation)
    if activation != "relu_squared":
        raise ValueError(f"unknown expert activation {activation!r}")
    if ids.numel() <= GEMV_MAX_PAIRS:
        return serving_kernels().expert_ffn_gemv(h.contiguous(), w_up, w_down, ids, weights, base)
    return _sorted_expert_ffn(h, w_up, w_down, ids, weights, base, activation)
