"""Slow, plain re-statement of the Kipirax layer mathematics, used as the
numerics oracle by the tests. Everything runs token by token in float64 on the
CPU, one function per mechanism, and none of it is imported by the library.

Notation: ``T`` tokens of one sequence, ``W`` model width, weights are
``[out, in]`` matrices applied as ``x @ M.T``. ``P`` is a flat dict of tensors
with the checkpoint's names ("l0.mix.left.q", ...).
"""

import math

import torch

F64 = torch.float64


def lin(x, m):
    return x @ m.to(F64).T


def sigmoid(x):
    return 1.0 / (1.0 + torch.exp(-x))


def silu(x):
    return x * sigmoid(x)


def softplus(x):
    return torch.log1p(torch.exp(-x.abs())) + x.clamp(min=0)


def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def grouped_rms_norm(x, w, groups, eps):
    """Split the last axis into ``groups`` consecutive parts, scale each part
    to unit RMS by itself, then apply the element-wise weight."""
    shp = x.shape
    y = rms_unit(x.reshape(*shp[:-1], groups, shp[-1] // groups), eps).reshape(shp)
    return y * w.to(F64)


def token_shift(h, mu):
    """h_t + (h_{t-1} - h_t) * mu, with h_{-1} = 0 and the *unshifted* h on
    the right-hand side."""
    out = torch.empty_like(h)
    prev = torch.zeros_like(h[0])
    for t in range(h.shape[0]):
        out[t] = h[t] + (prev - h[t]) * mu.to(F64)
        prev = h[t]
    return out


def causal_short_conv(x, taps):
    """x [T, C], taps [C, K]; tap K-1 multiplies the current token, tap K-1-d
    the token d steps back; nothing before the start."""
    T, C = x.shape
    K = taps.shape[1]
    y = torch.zeros_like(x)
    for t in range(T):
        for d in range(K):
            if t - d >= 0:
                y[t] += taps[:, K - 1 - d].to(F64) * x[t - d]
    return y


def windowed_bias_attention(q, k, v, scale, window, keep_first):
    """q [T, H, D], k [T, G, D], v [T, G, Dv]; query i sees key j <= i when
    i - j < window or j < keep_first; the score loses slope_h * (i - j) with
    slope_h = 2^(-8 (h + 1) / H)."""
    T, H, D = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[-1], dtype=F64)
    for h in range(H):
        g = h // (H // G)
        slope = 2.0 ** (-8.0 * (h + 1) / H)
        for i in range(T):
            js = [j for j in range(i + 1) if (i - j < window or j < keep_first)]
            s = torch.stack([(q[i, h] * k[j, g]).sum() * scale - slope * (i - j) for j in js])
            p = torch.softmax(s, 0)
            out[i, h] = (p[:, None] * torch.stack([v[j, g] for j in js])).sum(0)
    return out


def hgrn2_scan(q, f, v):
    """q, f [T, H, D], v [T, H, Dv]: S <- diag(f) S + (1 - f) v^T, o = S^T q."""
    T, H, D = q.shape
    S = torch.zeros(H, D, v.shape[-1], dtype=F64)
    out = torch.zeros(T, H, v.shape[-1], dtype=F64)
    for t in range(T):
        S = f[t][:, :, None] * S + (1.0 - f[t])[:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", S, q[t])
    return out


def gated_delta_scan(q, k, v, beta, g):
    """q, k, g [T, H, D] (already expanded to the value heads), v [T, H, Dv],
    beta [T, H]. Per step: decay rows, delta-rule write, read with the write
    included."""
    T, H, D = q.shape
    S = torch.zeros(H, D, v.shape[-1], dtype=F64)
    out = torch.zeros(T, H, v.shape[-1], dtype=F64)
    for t in range(T):
        S = g[t][:, :, None] * S
        pred = torch.einsum("hdv,hd->hv", S, k[t])
        u = beta[t][:, None] * (v[t] - pred)
        S = S + k[t][:, :, None] * u[:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", S, q[t])
    return out


# ----------------------------------------------------------------- mixers
def parallel_left(h, P, pre, c, eps):
    T = h.shape[0]
    H, G, D, Dv = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    q = lin(h, P[pre + "q"]).reshape(T, H, D)
    k = lin(h, P[pre + "k"]).reshape(T, G, D)
    v = lin(h, P[pre + "v"]).reshape(T, G, Dv)
    q = rms_unit(q, eps) * P[pre + "q.norm"].to(F64)
    k = rms_unit(k, eps) * P[pre + "k.norm"].to(F64)
    o = windowed_bias_attention(q, k, v, c["scale"], c["mask"]["size"], c["mask"]["keep_first"])
    gate = sigmoid(lin(h, P[pre + "g"]))  # [T, H]
    o = o * gate[:, :, None]
    return lin(o.reshape(T, H * Dv), P[pre + "o"])


def parallel_right(h, P, pre, c, eps):
    T = h.shape[0]
    H, D, Dv = c["heads"], c["dim"], c["vdim"]
    q = silu(lin(h, P[pre + "q"])).reshape(T, H, D)
    v = lin(h, P[pre + "v"]).reshape(T, H, Dv)
    low = P[pre + "lower"].to(F64)
    f = low + (1.0 - low) * sigmoid(lin(h, P[pre + "f"]) + P[pre + "f.b"].to(F64))
    o = hgrn2_scan(q, f.reshape(T, H, D), v)
    o = rms_unit(o, eps) * P[pre + "norm"].to(F64)
    return lin(o.reshape(T, H * Dv), P[pre + "o"])


def mixer_parallel(h, P, pre, c, eps):
    a = rms_unit(parallel_left(h, P, pre + "left.", c["left"], eps), eps) * P[pre + "left.out"].to(F64)
    b = rms_unit(parallel_right(h, P, pre + "right.", c["right"], eps), eps) * P[pre + "right.out"].to(F64)
    return 0.5 * (a + b)


def mixer_channel_delta(h, P, pre, c, eps):
    T = h.shape[0]
    H, G, D, Dv = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    q = silu(causal_short_conv(lin(h, P[pre + "q"]), P[pre + "q.conv"].to(F64))).reshape(T, G, D)
    k = silu(causal_short_conv(lin(h, P[pre + "k"]), P[pre + "k.conv"].to(F64))).reshape(T, G, D)
    v = silu(causal_short_conv(lin(h, P[pre + "v"]), P[pre + "v.conv"].to(F64))).reshape(T, H, Dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    rep = H // G
    q = q.repeat_interleave(rep, dim=1)
    k = k.repeat_interleave(rep, dim=1)
    beta = sigmoid(lin(h, P[pre + "b"]))  # [T, H]
    dt = softplus(lin(lin(h, P[pre + "a1"]), P[pre + "a2"]) + P[pre + "dt_bias"].to(F64)).reshape(T, H, D)
    g = torch.exp(-torch.exp(P[pre + "A_log"].to(F64))[None, :, None] * dt)
    o = gated_delta_scan(q, k, v, beta, g)
    gate = sigmoid(lin(lin(h, P[pre + "g1"]), P[pre + "g2"])).reshape(T, H, Dv)
    o = rms_unit(o, eps) * P[pre + "norm"].to(F64) * gate
    return lin(o.reshape(T, H * Dv), P[pre + "o"])


def feed_forward(x, P, pre, c):
    assert c["kind"] == "dense"
    a = lin(x, P[pre + "up"]).clamp(min=0)
    return lin(a * a, P[pre + "down"])


# ------------------------------------------------------------------ model
def forward(cfg, P, tokens, return_layers=False):
    """Logits [T, vocab] of one sequence (float64)."""
    eps, groups = cfg["norm"]["eps"], cfg["norm"]["groups"]
    T = len(tokens)
    x = P["embed"].to(F64)[torch.tensor(tokens)] + P["pos"].to(F64)[:T]
    per_layer = []
    for i, L in enumerate(cfg["layers"]):
        pre = "l%d." % i
        h = token_shift(x, P[pre + "shift"])
        if L["type"] == "parallel":
            m = mixer_parallel(h, P, pre + "mix.", L["mixer"], eps)
        elif L["type"] == "channel_delta":
            m = mixer_channel_delta(h, P, pre + "mix.", L["mixer"], eps)
        else:
            raise ValueError(L["type"])
        x = x + grouped_rms_norm(m, P[pre + "norm1"], groups, eps)
        if L.get("mlp") is not None:
            x = x + grouped_rms_norm(feed_forward(x, P, pre + "mlp.", L["mlp"]), P[pre + "norm2"], groups, eps)
        per_layer.append(x.clone())
    y = lin(grouped_rms_norm(x, P["final.norm"], groups, eps), P["head"])
    cap = cfg["logit_softcap"]
    y = cap * torch.tanh(y / cap)
    return (y, torch.stack(per_layer)) if return_layers else y


def random_weights(cfg, seed=0, scale=1.0):
    """Random bf16-representable weights with the checkpoint's names/shapes."""
    gen = torch.Generator().manual_seed(seed)
    W = cfg["width"]
    P = {}

    def mat(name, o, i, s=None):
        P[name] = (torch.randn(o, i, generator=gen) * (s if s is not None else scale / math.sqrt(i))).bfloat16()

    def vec(name, n, base=1.0, s=0.1):
        P[name] = (base + torch.randn(n, generator=gen) * s).bfloat16()

    mat("embed", cfg["vocab"], W, 1.0)
    mat("pos", cfg["max_positions"], W, 0.5)
    for i, L in enumerate(cfg["layers"]):
        p = "l%d." % i
        vec(p + "norm1", W)
        vec(p + "norm2", W)
        P[p + "shift"] = torch.rand(W, generator=gen).bfloat16()
        c = L["mixer"]
        if L["type"] == "parallel":
            a, b = c["left"], c["right"]
            q = p + "mix.left."
            mat(q + "q", a["heads"] * a["dim"], W)
            mat(q + "k", a["kv_heads"] * a["dim"], W)
            mat(q + "v", a["kv_heads"] * a["vdim"], W)
            vec(q + "q.norm", a["dim"])
            vec(q + "k.norm", a["dim"])
            mat(q + "g", a["heads"], W)
            mat(q + "o", W, a["heads"] * a["vdim"])
            vec(q + "out", W)
            r = p + "mix.right."
            mat(r + "q", b["heads"] * b["dim"], W)
            mat(r + "f", b["heads"] * b["dim"], W)
            vec(r + "f.b", b["heads"] * b["dim"], 0.0, 1.0)
            P[r + "lower"] = torch.rand(b["heads"] * b["dim"], generator=gen).mul(0.9).bfloat16()
            mat(r + "v", b["heads"] * b["vdim"], W)
            vec(r + "norm", b["vdim"])
            mat(r + "o", W, b["heads"] * b["vdim"])
            vec(r + "out", W)
        else:
            q = p + "mix."
            K = c["conv"]
            low = max(4, W // 8)
            for n, ch in (("q", c["kv_heads"] * c["dim"]), ("k", c["kv_heads"] * c["dim"]), ("v", c["heads"] * c["vdim"])):
                mat(q + n, ch, W)
                mat(q + n + ".conv", ch, K, 0.5)
            mat(q + "b", c["heads"], W)
            vec(q + "A_log", c["heads"], -1.0, 1.0)
            vec(q + "norm", c["vdim"])
            mat(q + "a1", low, W)
            mat(q + "a2", c["heads"] * c["dim"], low)
            vec(q + "dt_bias", c["heads"] * c["dim"], -1.0, 1.0)
            mat(q + "g1", low, W)
            mat(q + "g2", c["heads"] * c["vdim"], low)
            mat(q + "o", W, c["heads"] * c["vdim"])
        if L.get("mlp") is not None:
            mat(p + "mlp.up", L["mlp"]["ff"], W)
            mat(p + "mlp.down", W, L["mlp"]["ff"])
    vec("final.norm", W)
    mat("head", cfg["vocab"], W)
    return P
