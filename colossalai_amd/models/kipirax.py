"""Kipirax: a hybrid decoder-only language model served from fixed-size state
plus a paged window of keys.

Every layer is ``x <- x + norm1(mixer(shift(x)))`` then ``x <- x + norm2(ff(x))``
(norms on the sublayer *outputs*, grouped RMS; the residual ``x`` is float32
and the sublayers read it un-normalised). ``shift`` is a token shift. Two
mixers exist and a checkpoint's ``layers`` list picks one per layer:

* ``parallel`` — two branches on the same input, averaged after a full-width
  RMS norm each: a grouped-query softmax attention with per-head q/k RMS norm,
  a sliding window that keeps the first tokens, a linear distance penalty and
  a per-head sigmoid output gate (no rotation); and an HGRN2 matrix-state
  recurrence whose forget gate also scales the write.
* ``channel_delta`` — a gated delta rule with a decay per key channel, short
  causal convolutions on q/k/v, unit-length q/k, a low-rank decay projection
  and a low-rank output gate.

The feed-forward is dense with squared-ReLU. Positions enter through a learned
table added to the embedding and through the attention's distance penalty.
Logits are soft-capped.

The module holds the *packed* layout the kernels want (all input projections
of a mixer in one matrix, so a layer's input is read by one GEMM); a
checkpoint's per-projection tensors are packed by ``load_checkpoint_tensors``.
Serving goes through ``forward_ragged`` (a ragged step over paged keys and
state slots); ``forward`` runs whole sequences through the same path with
throw-away caches.
"""

import json
import os
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from ..ops.group_norm import grouped_rms_norm, head_rms_norm_gate, merge_rms_norm
from ..ops.linear_recurrence import gated_delta_rule, tied_gate_recurrence
from ..ops.paged_attention import distance_slopes, paged_attention, paged_kv_write
from ..ops.ragged import RaggedBatch
from ..ops.short_conv import short_conv
from ..ops.token_shift import token_shift
from ..ops.activation import relu_squared, softcap
from .packed import PackedLinear as _Packed
from .registry import register_model

__all__ = ["KipiraxConfig", "KipiraxForCausalLM"]

UNIT_EPS = 1e-6  # inside the root of the delta rule's q/k unit-length scaling


@dataclass
class KipiraxConfig:
    vocab: int
    width: int
    max_positions: int
    layers: List[dict]
    norm_eps: float = 1e-6
    norm_groups: int = 1
    logit_softcap: float = 0.0

    @classmethod
    def from_dict(cls, d: dict) -> "KipiraxConfig":
        return cls(vocab=int(d["vocab"]), width=int(d["width"]), max_positions=int(d["max_positions"]),
                   layers=list(d["layers"]), norm_eps=float(d["norm"]["eps"]), norm_groups=int(d["norm"]["groups"]),
                   logit_softcap=float(d.get("logit_softcap") or 0.0))

    def to_dict(self) -> dict:
        return {"architecture": "Kipirax", "layers": self.layers, "logit_softcap": self.logit_softcap,
                "max_positions": self.max_positions, "norm": {"eps": self.norm_eps, "groups": self.norm_groups},
                "vocab": self.vocab, "width": self.width}


def _vec(n, value=1.0):
    return nn.Parameter(torch.full((n,), value, dtype=torch.float32))


class KipiraxParallelMixer(nn.Module):
    def __init__(self, width: int, c: dict, eps: float):
        super().__init__()
        a, b = c["left"], c["right"]
        self.eps = eps
        self.H, self.G, self.D, self.Dv = int(a["heads"]), int(a["kv_heads"]), int(a["dim"]), int(a["vdim"])
        assert self.H % self.G == 0
        self.scale = float(a["scale"])
        mask = a.get("mask") or {}
        self.window, self.keep_first = int(mask.get("size", 0)), int(mask.get("keep_first", 0))
        self.rH, self.rD, self.rDv = int(b["heads"]), int(b["dim"]), int(b["vdim"])
        self.in_proj = _Packed(width, {
            "lq": self.H * self.D, "lk": self.G * self.D, "lv": self.G * self.Dv,
            "rq": self.rH * self.rD, "rf": self.rH * self.rD, "rv": self.rH * self.rDv, "lg": self.H,
        })
        self.q_norm, self.k_norm = _vec(self.D), _vec(self.D)
        self.left_o = nn.Linear(self.H * self.Dv, width, bias=False)
        self.left_out = _vec(width)
        self.f_bias, self.lower = _vec(self.rH * self.rD, 0.0), _vec(self.rH * self.rD, 0.0)
        self.right_norm = _vec(self.rDv)
        self.right_o = nn.Linear(self.rH * self.rDv, width, bias=False)
        self.right_out = _vec(width)
        self.register_buffer("slopes", distance_slopes(self.H), persistent=False)

    def kv_shape(self):
        return (self.G, self.D, self.Dv)

    def state_buffers(self):
        return {"S": (self.rH, self.rD, self.rDv)}

    def forward(self, h, batch: RaggedBatch, kpool, vpool, state, norm_w, groups, residual):
        N = h.shape[0]
        p, _ = self.in_proj(h)
        # left: windowed softmax attention over the pages
        q = head_rms_norm_gate(p["lq"].view(N, self.H, self.D), self.q_norm, self.eps)
        k = head_rms_norm_gate(p["lk"].view(N, self.G, self.D), self.k_norm, self.eps)
        paged_kv_write(k, p["lv"].view(N, self.G, self.Dv), kpool, vpool, batch)
        left = paged_attention(q, kpool, vpool, batch, self.scale, self.window, self.keep_first,
                               self.slopes, p["lg"])
        left = self.left_o(left.reshape(N, self.H * self.Dv))
        # right: matrix-state recurrence with a tied forget/write gate
        o = tied_gate_recurrence(p["rq"].view(N, self.rH, self.rD), p["rf"].view(N, self.rH, self.rD),
                                 p["rv"].view(N, self.rH, self.rDv), self.f_bias, self.lower, state["S"], batch)
        o = head_rms_norm_gate(o, self.right_norm, self.eps, None, h.dtype)
        right = self.right_o(o.reshape(N, self.rH * self.rDv))
        return merge_rms_norm(left, self.left_out, right, self.right_out, self.eps, norm_w, groups, residual)


class KipiraxChannelDeltaMixer(nn.Module):
    def __init__(self, width: int, c: dict, eps: float):
        super().__init__()
        self.eps = eps
        self.H, self.G, self.D, self.Dv = int(c["heads"]), int(c["kv_heads"]), int(c["dim"]), int(c["vdim"])
        assert self.H % self.G == 0
        self.K = int(c["conv"])
        # ranks of the two low-rank projections: not in a checkpoint's config (its tensors' shapes give them)
        self.decay_rank = int(c.get("decay_rank", max(4, width // 8)))
        self.gate_rank = int(c.get("gate_rank", max(4, width // 8)))
        self.Cq, self.Cv = self.G * self.D, self.H * self.Dv
        self.C = 2 * self.Cq + self.Cv
        self.in_proj = _Packed(width, {"q": self.Cq, "k": self.Cq, "v": self.Cv, "a1": self.decay_rank, "g1": self.gate_rank,
                                       "b": self.H})
        self.conv = nn.Parameter(torch.randn(self.C, self.K, dtype=torch.float32) * 0.5)
        self.a2 = nn.Linear(self.decay_rank, self.H * self.D, bias=False)
        self.g2 = nn.Linear(self.gate_rank, self.H * self.Dv, bias=False)
        self.A_log, self.dt_bias = _vec(self.H, 0.0), _vec(self.H * self.D, 0.0)
        self.norm = _vec(self.Dv)
        self.o = nn.Linear(self.H * self.Dv, width, bias=False)

    def kv_shape(self):
        return None

    def state_buffers(self):
        buf = {"S": (self.H, self.D, self.Dv)}
        if self.K > 1:
            buf["tail"] = (self.K - 1, self.C)
        return buf

    def forward(self, h, batch: RaggedBatch, kpool, vpool, state, norm_w, groups, residual):
        N = h.shape[0]
        p, y = self.in_proj(h)
        # the convolution feeds a recurrence: its activated output stays float32
        qkv = short_conv(y[:, : self.C], self.conv, state.get("tail"), batch, True, torch.float32)
        q = qkv[:, : self.Cq].view(N, self.G, self.D)
        k = qkv[:, self.Cq : 2 * self.Cq].view(N, self.G, self.D)
        v = qkv[:, 2 * self.Cq :].view(N, self.H, self.Dv)
        dt = self.a2(p["a1"])
        gate = self.g2(p["g1"])
        o = gated_delta_rule(q, k, v, p["b"], dt, self.A_log, self.dt_bias, state["S"], batch,
                             UNIT_EPS, self.D ** -0.5)
        o = head_rms_norm_gate(o, self.norm, self.eps, gate, h.dtype)
        out = self.o(o.reshape(N, self.H * self.Dv))
        return grouped_rms_norm(out, norm_w, groups, self.eps, residual)


class KipiraxMLP(nn.Module):
    def __init__(self, width: int, c: dict):
        super().__init__()
        if c.get("kind", "dense") != "dense":
            raise ValueError(f"unknown feed-forward kind {c.get('kind')!r}")
        self.up = nn.Linear(width, int(c["ff"]), bias=False)
        self.down = nn.Linear(int(c["ff"]), width, bias=False)

    def forward(self, x):
        return self.down(relu_squared(self.up(x)))


MIXERS = {"parallel": KipiraxParallelMixer, "channel_delta": KipiraxChannelDeltaMixer}


class KipiraxLayer(nn.Module):
    def __init__(self, cfg: KipiraxConfig, spec: dict):
        super().__init__()
        if spec["type"] not in MIXERS:
            raise ValueError(f"unknown mixer type {spec['type']!r}")
        self.kind = spec["type"]
        self.mix = MIXERS[spec["type"]](cfg.width, spec["mixer"], cfg.norm_eps)
        self.shift = _vec(cfg.width, 0.5)
        self.norm1 = _vec(cfg.width)
        self.mlp = KipiraxMLP(cfg.width, spec["mlp"]) if spec.get("mlp") is not None else None
        self.norm2 = _vec(cfg.width) if self.mlp is not None else None

    def state_buffers(self, width: int):
        return dict(self.mix.state_buffers(), shift=(width,))


@register_model("Kipirax")
class KipiraxForCausalLM(nn.Module):
    config_class = KipiraxConfig
    serves_ragged = True  # the serving engines drive forward_ragged

    def __init__(self, cfg: KipiraxConfig):
        super().__init__()
        self.config = cfg
        self.embed = nn.Embedding(cfg.vocab, cfg.width)
        self.pos = nn.Embedding(cfg.max_positions, cfg.width)
        self.layers = nn.ModuleList([KipiraxLayer(cfg, s) for s in cfg.layers])
        self.final_norm = _vec(cfg.width)
        self.head = nn.Linear(cfg.width, cfg.vocab, bias=False)

    # ------------------------------------------------------------ cache plan
    def kv_layer_shapes(self):
        """Per layer ``(kv_heads, key_dim, value_dim)`` or None."""
        return [l.mix.kv_shape() for l in self.layers]

    def state_layer_buffers(self):
        """Per layer ``{name: shape}`` of float32 state kept per sequence."""
        return [l.state_buffers(self.config.width) for l in self.layers]

    @property
    def act_dtype(self):
        return self.head.weight.dtype

    # ---------------------------------------------------------------- serve
    def forward_ragged(self, tokens: torch.Tensor, batch: RaggedBatch, kv, state,
                       want: Optional[torch.Tensor] = None) -> torch.Tensor:
        """tokens [N] (flat, sequence after sequence as ``batch`` says); ``kv`` a
        KVCacheManager and ``state`` a StateCacheManager laid out by
        ``kv_layer_shapes`` / ``state_layer_buffers``. Returns float32 logits of
        the rows ``want`` (indices into the flat token axis; all rows if None)."""
        cfg, act = self.config, self.act_dtype
        if batch.max_total > cfg.max_positions:
            raise ValueError(f"sequence of {batch.max_total} tokens exceeds max_positions {cfg.max_positions}")
        x = self.embed(tokens).float() + self.pos(batch.positions.long()).float()
        for i, layer in enumerate(self.layers):
            st = state.layers[i]
            h = token_shift(x, layer.shift, st["shift"], batch, act)
            x = layer.mix(h, batch, kv.k_pools[i], kv.v_pools[i], st, layer.norm1, cfg.norm_groups, x)
            if layer.mlp is not None:
                x = grouped_rms_norm(layer.mlp(x.to(act)), layer.norm2, cfg.norm_groups, cfg.norm_eps, x)
        if want is not None:
            x = x.index_select(0, want)
        y = self.head(grouped_rms_norm(x, self.final_norm, cfg.norm_groups, cfg.norm_eps, None, act)).float()
        return softcap(y, cfg.logit_softcap) if cfg.logit_softcap > 0 else y

    def forward(self, input_ids: torch.Tensor) -> torch.Tensor:
        """input_ids [B, S] -> logits [B, S, vocab] (float32), every sequence
        from position 0 with caches that live for this call only."""
        from ..inference.kv_cache import KVCacheManager
        from ..inference.state_cache import StateCacheManager

        B, S = input_ids.shape
        dev = input_ids.device
        page = 16
        pages = (S + page - 1) // page
        kv = KVCacheManager(len(self.layers), 0, 0, num_blocks=B * pages, block_size=page, device=dev,
                            dtype=self.act_dtype, layer_shapes=self.kv_layer_shapes())
        state = StateCacheManager(self.state_layer_buffers(), B, device=dev)
        tables = [list(range(b * pages, (b + 1) * pages)) for b in range(B)]
        batch = RaggedBatch.build([S] * B, [0] * B, list(range(B)), dev, tables, page)
        with torch.no_grad():
            return self.forward_ragged(input_ids.reshape(-1), batch, kv, state).view(B, S, -1)

    # -------------------------------------------------------------- weights
    def load_checkpoint_tensors(self, tensors: Dict[str, torch.Tensor]) -> None:
        """Pack a checkpoint's per-projection tensors (names ``l<i>.mix.*``,
        ``l<i>.mlp.*``, ``embed``, ``pos``, ``final.norm``, ``head``) into this
        module's fused parameters. Every tensor must be used and every
        parameter filled."""
        used = set()

        def get(name):
            used.add(name)
            return tensors[name]

        def put(param, value):
            assert tuple(param.shape) == tuple(value.shape), (tuple(param.shape), tuple(value.shape))
            param.data.copy_(value.to(param.dtype))

        def pack(mod: _Packed, names: Dict[str, str]):
            put(mod.weight, torch.cat([get(names[part]) for part in mod.parts], 0))

        put(self.embed.weight, get("embed"))
        put(self.pos.weight, get("pos"))
        put(self.final_norm, get("final.norm"))
        put(self.head.weight, get("head"))
        for i, layer in enumerate(self.layers):
            p, m = f"l{i}.", layer.mix
            put(layer.shift, get(p + "shift"))
            put(layer.norm1, get(p + "norm1"))
            if layer.mlp is not None:
                put(layer.norm2, get(p + "norm2"))
                put(layer.mlp.up.weight, get(p + "mlp.up"))
                put(layer.mlp.down.weight, get(p + "mlp.down"))
            else:
                used.add(p + "norm2")  # a layer without a feed-forward may still carry its unused norm weight
            if layer.kind == "parallel":
                a, b = p + "mix.left.", p + "mix.right."
                pack(m.in_proj, {"lq": a + "q", "lk": a + "k", "lv": a + "v", "lg": a + "g",
                                 "rq": b + "q", "rf": b + "f", "rv": b + "v"})
                put(m.q_norm, get(a + "q.norm"))
                put(m.k_norm, get(a + "k.norm"))
                put(m.left_o.weight, get(a + "o"))
                put(m.left_out, get(a + "out"))
                put(m.f_bias, get(b + "f.b"))
                put(m.lower, get(b + "lower"))
                put(m.right_norm, get(b + "norm"))
                put(m.right_o.weight, get(b + "o"))
                put(m.right_out, get(b + "out"))
            else:
                a = p + "mix."
                pack(m.in_proj, {"q": a + "q", "k": a + "k", "v": a + "v", "a1": a + "a1", "g1": a + "g1",
                                 "b": a + "b"})
                put(m.conv, torch.cat([get(a + "q.conv"), get(a + "k.conv"), get(a + "v.conv")], 0))
                put(m.a2.weight, get(a + "a2"))
                put(m.g2.weight, get(a + "g2"))
                put(m.A_log, get(a + "A_log"))
                put(m.dt_bias, get(a + "dt_bias"))
                put(m.norm, get(a + "norm"))
                put(m.o.weight, get(a + "o"))
        missing = set(tensors) - used
        if missing:
            raise ValueError(f"checkpoint tensors without a place in the model: {sorted(missing)[:8]}")

    @classmethod
    def from_checkpoint(cls, config: dict, tensors: Dict[str, torch.Tensor], dtype=torch.bfloat16, device="cpu"):
        """Build from a parsed config.json and a name -> tensor mapping. Sizes
        that the config leaves to the tensors (the low rank of the decay and
        gate projections) are read from their shapes. Matrices take ``dtype``;
        vectors (norm weights, gates' biases, taps, decays) stay float32."""
        cfg = KipiraxConfig.from_dict(config)
        layers = []
        for i, spec in enumerate(cfg.layers):
            spec = json.loads(json.dumps(spec))
            if spec["type"] == "channel_delta":
                spec["mixer"]["decay_rank"] = int(tensors[f"l{i}.mix.a1"].shape[0])
                spec["mixer"]["gate_rank"] = int(tensors[f"l{i}.mix.g1"].shape[0])
            layers.append(spec)
        cfg.layers = layers
        model = cls(cfg)
        for p in model.parameters():
            if p.dim() >= 2:
                p.data = p.data.to(dtype)
        for layer in model.layers:
            if layer.kind == "channel_delta":
                layer.mix.conv.data = layer.mix.conv.data.float()
        model.load_checkpoint_tensors(tensors)
        return model.to(device).eval()
