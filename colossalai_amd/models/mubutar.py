"""Mubutar: a decoder-only language model of *parallel* pre-norm layers with
sink-softmax attention, cross-layer key/value sharing and a group-routed
mixture of experts.

Every layer is ``x <- x + mixer(h) + ff(h)`` with ``h = rms_norm(x) * w``: one
norm per layer, both sublayers read it, the residual ``x`` is float32. The
embedding is scaled by a constant on the way in and the logits on the way out.

* Mixer ``attention``: grouped-query attention with biased q/k/v projections,
  no positional rotation (positions reach the scores through the causal mask
  only), a configured score scale, a tanh soft cap on the scaled score and a
  softmax whose denominator has one extra place of score 0 without a value
  (``p_j = exp(s_j) / (1 + sum exp(s_j))``). Key and value head sizes differ. A
  layer with ``kv_from: j`` projects only queries and attends over the keys and
  values that layer ``j`` put into its pages.
* Feed-forward ``dense``: ``down(silu(gate h) * up h)``.
* Feed-forward ``moe``: bias-free experts ``down(relu(up h)^2)``; float32
  sigmoid router with a per-expert correction that only steers the choice,
  group-limited top-k, chosen scores renormalised to sum to one; an optional
  shared expert of the same form runs for every token.

The module holds the packed layout the kernels want: q/k/v (with biases) of a
layer are one matrix, gate/up of a dense feed-forward another, the experts'
matrices are stacked ``[E, out, in]``. Serving goes through ``forward_ragged``
(a ragged step over paged keys; the model keeps no recurrent state, so its
state slots are empty); ``forward`` runs whole sequences through the same path
with throw-away caches.
"""

from dataclasses import dataclass
from typing import Dict, List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from ..ops.activation import relu_squared, silu_mul
from ..ops.group_norm import add_rms_norm, grouped_rms_norm
from ..ops.paged_attention import paged_attention, paged_kv_write
from ..ops.ragged import RaggedBatch
from ..ops.routed_experts import grouped_topk_route, routed_expert_ffn
from .packed import PackedLinear
from .registry import register_model

__all__ = ["MubutarConfig", "MubutarForCausalLM"]

GROUP_TOP = 2         # a router group is worth the sum of this many of its best choice scores
RENORM_EPS = 1e-20    # added to the sum of the chosen scores before dividing


@dataclass
class MubutarConfig:
    vocab: int
    width: int
    layers: List[dict]
    norm_eps: float = 1e-6
    embedding_scale: float = 1.0
    logit_scale: float = 1.0

    @classmethod
    def from_dict(cls, d: dict) -> "MubutarConfig":
        return cls(vocab=int(d["vocab"]), width=int(d["width"]), layers=list(d["layers"]),
                   norm_eps=float(d["norm"]["eps"]),
                   embedding_scale=float((d.get("embedding") or {}).get("scale", 1.0)),
                   logit_scale=float(d.get("logit_scale", 1.0)))

    def to_dict(self) -> dict:
        return {"architecture": "Mubutar", "embedding": {"scale": self.embedding_scale}, "layers": self.layers,
                "logit_scale": self.logit_scale, "norm": {"eps": self.norm_eps}, "vocab": self.vocab,
                "width": self.width}


def _vec(n, value=1.0):
    return nn.Parameter(torch.full((n,), value, dtype=torch.float32))


class MubutarAttention(nn.Module):
    def __init__(self, width: int, c: dict):
        super().__init__()
        self.H, self.G, self.D, self.Dv = int(c["heads"]), int(c["kv_heads"]), int(c["dim"]), int(c["vdim"])
        assert self.H % self.G == 0
        self.scale = float(c["scale"])
        self.softcap = float(c.get("softcap") or 0.0)
        self.kv_from = None if c.get("kv_from") is None else int(c["kv_from"])
        parts = {"q": self.H * self.D}
        if self.kv_from is None:
            parts.update(k=self.G * self.D, v=self.G * self.Dv)
        self.in_proj = PackedLinear(width, parts, bias=True)
        self.o = nn.Linear(self.H * self.Dv, width, bias=False)

    def kv_shape(self):
        return (self.G, self.D, self.Dv) if self.kv_from is None else None

    def forward(self, h, batch: RaggedBatch, kpool, vpool):
        N = h.shape[0]
        p, _ = self.in_proj(h)
        if self.kv_from is None:
            paged_kv_write(p["k"].view(N, self.G, self.D), p["v"].view(N, self.G, self.Dv), kpool, vpool, batch)
        o = paged_attention(p["q"].view(N, self.H, self.D), kpool, vpool, batch, self.scale,
                            softcap=self.softcap, sink=True)
        return self.o(o.reshape(N, self.H * self.Dv))


class MubutarDenseMLP(nn.Module):
    def __init__(self, width: int, c: dict):
        super().__init__()
        ff = int(c["ff"])
        self.in_proj = PackedLinear(width, {"gate": ff, "up": ff})
        self.down = nn.Linear(ff, width, bias=False)

    def forward(self, h):
        _, y = self.in_proj(h)
        return self.down(silu_mul(y))


class MubutarExpert(nn.Module):
    """down(relu(up h)^2), no biases."""

    def __init__(self, width: int, ff: int):
        super().__init__()
        self.up = nn.Linear(width, ff, bias=False)
        self.down = nn.Linear(ff, width, bias=False)

    def forward(self, h):
        return self.down(relu_squared(self.up(h)))


class MubutarMoE(nn.Module):
    def __init__(self, width: int, c: dict):
        super().__init__()
        r = c["router"]
        self.E, self.top = int(r["experts"]), int(r["top"])
        groups = r.get("groups") or {}
        self.group_count, self.group_keep = int(groups.get("count", 1)), int(groups.get("keep", 1))
        ff = int(c["expert"]["ff"])
        self.router = nn.Parameter(torch.randn(self.E, width, dtype=torch.float32) * width ** -0.5)  # float32 always
        self.correction = _vec(self.E, 0.0)
        self.w_up = nn.Parameter(torch.randn(self.E, ff, width) * width ** -0.5)
        self.w_down = nn.Parameter(torch.randn(self.E, width, ff) * ff ** -0.5)
        self.shared = MubutarExpert(width, int(c["shared"]["ff"])) if c.get("shared") else None

    def forward(self, h):
        logits = F.linear(h.float(), self.router)
        ids, weights = grouped_topk_route(logits, self.correction, self.top, self.group_count, self.group_keep,
                                          GROUP_TOP, RENORM_EPS)
        base = self.shared(h) if self.shared is not None else None
        return routed_expert_ffn(h, self.w_up, self.w_down, ids, weights, base, "relu_squared")


MIXERS = {"attention": MubutarAttention}
MLPS = {"dense": MubutarDenseMLP, "moe": MubutarMoE}


class MubutarLayer(nn.Module):
    def __init__(self, cfg: MubutarConfig, spec: dict):
        super().__init__()
        if spec["type"] not in MIXERS:
            raise ValueError(f"unknown mixer type {spec['type']!r}")
        self.kind = spec["type"]
        self.norm1 = _vec(cfg.width)
        self.mix = MIXERS[spec["type"]](cfg.width, spec["mixer"])
        m = spec.get("mlp")
        if m is not None and m.get("kind", "dense") not in MLPS:
            raise ValueError(f"unknown feed-forward kind {m.get('kind')!r}")
        self.mlp = MLPS[m.get("kind", "dense")](cfg.width, m) if m is not None else None


@register_model("Mubutar")
class MubutarForCausalLM(nn.Module):
    config_class = MubutarConfig
    serves_ragged = True  # the serving engines drive forward_ragged

    def __init__(self, cfg: MubutarConfig):
        super().__init__()
        self.config = cfg
        self.embed = nn.Embedding(cfg.vocab, cfg.width)
        self.layers = nn.ModuleList([MubutarLayer(cfg, s) for s in cfg.layers])
        self.final_norm = _vec(cfg.width)
        self.head = nn.Linear(cfg.width, cfg.vocab, bias=False)
        for i, layer in enumerate(self.layers):
            j = layer.mix.kv_from
            if j is None:
                continue
            if not 0 <= j < i or self.layers[j].mix.kv_from is not None:
                raise ValueError(f"layer {i} reads keys of layer {j}, which must come earlier and project its own")
            a, b = layer.mix, self.layers[j].mix
            if (a.G, a.D, a.Dv) != (b.G, b.D, b.Dv):
                raise ValueError(f"layer {i} and the layer {j} whose keys it reads differ in key/value head sizes")

    # ------------------------------------------------------------ cache plan
    def kv_layer_shapes(self):
        """Per layer ``(kv_heads, key_dim, value_dim)``, None for a layer that reads another's keys."""
        return [l.mix.kv_shape() for l in self.layers]

    def kv_layer_sources(self):
        """Per layer the layer whose pools it reads, None for its own."""
        return [l.mix.kv_from for l in self.layers]

    def state_layer_buffers(self):
        """No layer keeps fixed-size state; a sequence's slot is empty."""
        return [None for _ in self.layers]

    @property
    def act_dtype(self):
        return self.head.weight.dtype

    # ---------------------------------------------------------------- serve
    def forward_ragged(self, tokens: torch.Tensor, batch: RaggedBatch, kv, state=None,
                       want: Optional[torch.Tensor] = None, residuals: Optional[list] = None) -> torch.Tensor:
        """tokens [N] (flat, sequence after sequence as ``batch`` says); ``kv`` a
        KVCacheManager laid out by ``kv_layer_shapes`` / ``kv_layer_sources``.
        Returns float32 logits of the rows ``want`` (indices into the flat token
        axis; all rows if None). ``residuals``, when a list, receives a copy of
        the float32 residual stream after every layer."""
        cfg, act = self.config, self.act_dtype
        x = self.embed(tokens).float() * cfg.embedding_scale
        n = len(self.layers)
        h = grouped_rms_norm(x, self.layers[0].norm1, 1, cfg.norm_eps, None, act) if n else None
        for i, layer in enumerate(self.layers):
            a = layer.mix(h, batch, kv.k_pools[i], kv.v_pools[i])
            b = layer.mlp(h) if layer.mlp is not None else None
            next_w = self.layers[i + 1].norm1 if i + 1 < n else None
            h = add_rms_norm(x, a, b, next_w, cfg.norm_eps, act)  # x += a + b; h = norm of the next layer
            if residuals is not None:
                residuals.append(x.clone())
        if want is not None:
            x = x.index_select(0, want)
        y = self.head(grouped_rms_norm(x, self.final_norm, 1, cfg.norm_eps, None, act)).float()
        return y * cfg.logit_scale if cfg.logit_scale != 1.0 else y

    def forward(self, input_ids: torch.Tensor) -> torch.Tensor:
        """input_ids [B, S] -> logits [B, S, vocab] (float32), every sequence
        from position 0 with caches that live for this call only."""
        from ..inference.kv_cache import KVCacheManager

        B, S = input_ids.shape
        dev = input_ids.device
        page = 16
        pages = (S + page - 1) // page
        kv = KVCacheManager(len(self.layers), 0, 0, num_blocks=B * pages, block_size=page, device=dev,
                            dtype=self.act_dtype, layer_shapes=self.kv_layer_shapes(),
                            layer_sources=self.kv_layer_sources())
        tables = [list(range(b * pages, (b + 1) * pages)) for b in range(B)]
        batch = RaggedBatch.build([S] * B, [0] * B, list(range(B)), dev, tables, page)
        with torch.no_grad():
            return self.forward_ragged(input_ids.reshape(-1), batch, kv).view(B, S, -1)

    # -------------------------------------------------------------- weights
    def load_checkpoint_tensors(self, tensors: Dict[str, torch.Tensor]) -> None:
        """Pack a checkpoint's per-projection tensors (``embed``, ``l<i>.norm1``,
        ``l<i>.mix.{q,k,v}[.b]``, ``l<i>.mix.o``, ``l<i>.mlp.*``, ``final.norm``,
        ``head``) into this module's fused parameters. Every tensor must be used
        and every parameter filled."""
        used = set()

        def get(name):
            used.add(name)
            return tensors[name]

        def put(param, value):
            assert tuple(param.shape) == tuple(value.shape), (tuple(param.shape), tuple(value.shape))
            param.data.copy_(value.to(param.dtype))

        put(self.embed.weight, get("embed"))
        put(self.final_norm, get("final.norm"))
        put(self.head.weight, get("head"))
        for i, layer in enumerate(self.layers):
            p, m = f"l{i}.", layer.mix
            put(layer.norm1, get(p + "norm1"))
            put(m.in_proj.weight, torch.cat([get(p + "mix." + part) for part in m.in_proj.parts], 0))
            put(m.in_proj.bias, torch.cat([get(p + "mix." + part + ".b") for part in m.in_proj.parts], 0))
            put(m.o.weight, get(p + "mix.o"))
            f = layer.mlp
            if isinstance(f, MubutarDenseMLP):
                put(f.in_proj.weight, torch.cat([get(p + "mlp.gate"), get(p + "mlp.up")], 0))
                put(f.down.weight, get(p + "mlp.down"))
            elif isinstance(f, MubutarMoE):
                put(f.router, get(p + "mlp.router"))
                put(f.correction, get(p + "mlp.correction"))
                put(f.w_up, torch.stack([get(p + f"mlp.e{e}.up") for e in range(f.E)], 0))
                put(f.w_down, torch.stack([get(p + f"mlp.e{e}.down") for e in range(f.E)], 0))
                if f.shared is not None:
                    put(f.shared.up.weight, get(p + "mlp.shared.up"))
                    put(f.shared.down.weight, get(p + "mlp.shared.down"))
        missing = set(tensors) - used
        if missing:
            raise ValueError(f"checkpoint tensors without a place in the model: {sorted(missing)[:8]}")

    @classmethod
    def from_checkpoint(cls, config: dict, tensors: Dict[str, torch.Tensor], dtype=torch.bfloat16, device="cpu"):
        """Build from a parsed config.json and a name -> tensor mapping.
        Matrices and projection biases take ``dtype``; norm weights, the router
        and its correction stay float32."""
        model = cls(MubutarConfig.from_dict(config))
        keep32 = {id(l.mlp.router) for l in model.layers if isinstance(l.mlp, MubutarMoE)}
        for p in model.parameters():
            if p.dim() >= 2 and id(p) not in keep32:
                p.data = p.data.to(dtype)
        for layer in model.layers:
            layer.mix.in_proj.bias.data = layer.mix.in_proj.bias.data.to(dtype)
        model.load_checkpoint_tensors(tensors)
        return model.to(device).eval()
