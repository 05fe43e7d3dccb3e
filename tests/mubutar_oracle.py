"""Slow, plain re-statement of the Mubutar layer mathematics, used as the
numerics oracle by the tests. Everything runs in float64 on the CPU, one
function per mechanism, with explicit loops where a vectorised form could hide
an off-by-one; none of it is imported by the library.

Notation: ``T`` tokens of one sequence, ``W`` model width, weights are
``[out, in]`` matrices applied as ``x @ M.T``. ``P`` is a flat dict of tensors
with the checkpoint's names ("l0.mix.q", "l1.mlp.e3.up", ...).
"""

import math

import torch

F64 = torch.float64


def lin(x, m, b=None):
    y = x @ m.to(F64).T
    return y if b is None else y + b.to(F64)


def sigmoid(x):
    return 1.0 / (1.0 + torch.exp(-x))


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w.to(F64)


def sink_softcap_attention(q, k, v, scale, softcap):
    """q [T, H, D], k [T, G, D], v [T, G, Dv]. Query i sees every key j <= i.
    The scaled score is squashed to (-softcap, softcap) by a tanh (no squashing
    when softcap is 0), and the softmax has one more place in its denominator:
    a sink of score 0 that carries no value,
    ``p_j = exp(s_j) / (1 + sum_j' exp(s_j'))``."""
    T, H, D = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[-1], dtype=F64)
    for h in range(H):
        g = h // (H // G)
        for i in range(T):
            s = (k[: i + 1, g] @ q[i, h]) * scale       # keys 0..i and no others
            if softcap:
                s = softcap * torch.tanh(s / softcap)
            e = torch.exp(s)
            p = e / (1.0 + e.sum())
            out[i, h] = p @ v[: i + 1, g]
    return out


def attention_keys_values(h, P, pre):
    """The key/value projections (with biases) of the layer whose tensors start with ``pre``."""
    return lin(h, P[pre + "k"], P[pre + "k.b"]), lin(h, P[pre + "v"], P[pre + "v.b"])


def mixer_attention(h, P, pre, c, kv):
    """``kv`` is the (k, v) pair this layer reads: its own, or another layer's."""
    T = h.shape[0]
    H, G, D, Dv = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    q = lin(h, P[pre + "q"], P[pre + "q.b"]).view(T, H, D)
    k, v = kv
    o = sink_softcap_attention(q, k.view(T, G, D), v.view(T, G, Dv), c["scale"], c.get("softcap") or 0.0)
    return lin(o.reshape(T, H * Dv), P[pre + "o"])


def dense_ff(h, P, pre):
    g = lin(h, P[pre + "gate"])
    return lin(g * sigmoid(g) * lin(h, P[pre + "up"]), P[pre + "down"])


def expert_ff(h, P, pre):
    return lin(torch.relu(lin(h, P[pre + "up"])) ** 2, P[pre + "down"])


def route(z, correction, top, group_count, group_keep):
    """z [E] router logits of one token -> (chosen expert ids, their weights).
    Scores are sigmoids; the *choice* uses score + correction, the weights the
    plain scores. Experts form ``group_count`` runs of neighbours; a group is
    worth the sum of its two best choice scores, and only the ``group_keep``
    best groups take part in the top-``top`` choice."""
    E = z.shape[0]
    s = sigmoid(z)
    choice = s + correction.to(F64)
    per = E // group_count
    worth = []
    for g in range(group_count):
        members = sorted((float(choice[e]) for e in range(g * per, (g + 1) * per)), reverse=True)
        worth.append(sum(members[:2]))
    kept = sorted(range(group_count), key=lambda g: (-worth[g], g))[:group_keep]
    allowed = [e for e in range(E) if e // per in kept]
    chosen = sorted(allowed, key=lambda e: (-float(choice[e]), e))[:top]
    total = sum(float(s[e]) for e in chosen) + 1e-20
    return chosen, [float(s[e]) / total for e in chosen]


def moe_ff(h, P, pre, c):
    r = c["router"]
    groups = r.get("groups") or {"count": 1, "keep": 1}
    out = torch.zeros(h.shape[0], P[pre + "e0.down"].shape[0], dtype=F64)
    logits = lin(h, P[pre + "router"])
    for t in range(h.shape[0]):
        chosen, weights = route(logits[t], P[pre + "correction"], r["top"], groups["count"], groups["keep"])
        for e, w in zip(chosen, weights):
            out[t] += w * expert_ff(h[t], P, f"{pre}e{e}.")
    if c.get("shared"):
        out = out + expert_ff(h, P, pre + "shared.")
    return out


def feed_forward(h, P, pre, c):
    if c["kind"] == "dense":
        return dense_ff(h, P, pre)
    if c["kind"] == "moe":
        return moe_ff(h, P, pre, c)
    raise ValueError(c["kind"])


def forward(cfg, P, tokens, return_layers=False):
    """Logits [T, vocab] (float64) of one sequence from position 0."""
    eps = cfg["norm"]["eps"]
    x = P["embed"].to(F64)[torch.tensor(tokens)] * cfg["embedding"]["scale"]
    kept, layers = {}, []
    for i, spec in enumerate(cfg["layers"]):
        assert spec["type"] == "attention"
        pre = f"l{i}."
        h = rms_norm(x, P[pre + "norm1"], eps)
        c = spec["mixer"]
        if c.get("kv_from") is None:
            kept[i] = attention_keys_values(h, P, pre + "mix.")
            kv = kept[i]
        else:
            kv = kept[c["kv_from"]]
        y = mixer_attention(h, P, pre + "mix.", c, kv)
        if spec.get("mlp") is not None:
            y = y + feed_forward(h, P, pre + "mlp.", spec["mlp"])
        x = x + y
        layers.append(x.clone())
    y = lin(rms_norm(x, P["final.norm"], eps), P["head"]) * cfg.get("logit_scale", 1.0)
    return (y, layers) if return_layers else y


def random_weights(cfg, seed=0, scale=1.0):
    """A checkpoint's tensors for ``cfg`` (float32 values, names as on disk)."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def mat(o, i, gain=1.0):
        return torch.randn(o, i, generator=g) * (gain * scale / math.sqrt(i))

    def vec(n, spread=0.1, mean=0.0):
        return mean + torch.randn(n, generator=g) * spread

    P = {"embed": torch.randn(cfg["vocab"], W, generator=g) * 0.5, "final.norm": vec(W, 0.1, 1.0),
         "head": mat(cfg["vocab"], W)}
    for i, spec in enumerate(cfg["layers"]):
        p, c = f"l{i}.", spec["mixer"]
        H, G, D, Dv = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
        P[p + "norm1"] = vec(W, 0.1, 1.0)
        P[p + "mix.q"], P[p + "mix.q.b"] = mat(H * D, W, 2.0), vec(H * D, 0.3)
        if c.get("kv_from") is None:
            P[p + "mix.k"], P[p + "mix.k.b"] = mat(G * D, W, 2.0), vec(G * D, 0.3)
            P[p + "mix.v"], P[p + "mix.v.b"] = mat(G * Dv, W), vec(G * Dv, 0.3)
        P[p + "mix.o"] = mat(W, H * Dv)
        m = spec.get("mlp")
        if m is None:
            continue
        if m["kind"] == "dense":
            P[p + "mlp.gate"], P[p + "mlp.up"], P[p + "mlp.down"] = mat(m["ff"], W), mat(m["ff"], W), mat(W, m["ff"])
        else:
            E = m["router"]["experts"]
            for e in range(E):
                P[p + f"mlp.e{e}.up"], P[p + f"mlp.e{e}.down"] = mat(m["expert"]["ff"], W), mat(W, m["expert"]["ff"])
            P[p + "mlp.router"] = mat(E, W, 3.0)
            P[p + "mlp.correction"] = vec(E, 0.3)
            if m.get("shared"):
                P[p + "mlp.shared.up"], P[p + "mlp.shared.down"] = mat(m["shared"]["ff"], W), mat(W, m["shared"]["ff"])
    return P
