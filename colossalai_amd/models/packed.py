"""Several projections of one input stored as one matrix, so that a layer's
input is read by a single GEMM."""

from typing import Dict

import torch
import torch.nn as nn
import torch.nn.functional as F

__all__ = ["PackedLinear"]


class PackedLinear(nn.Module):
    """``parts`` maps a name to its output size; the ``[out_i, in]`` matrices are
    stacked in that order (with their biases, when ``bias``). ``forward`` hands
    back column views of the single product's output and the output itself."""

    def __init__(self, in_features: int, parts: Dict[str, int], bias: bool = False):
        super().__init__()
        self.parts = dict(parts)
        self.offsets, at = {}, 0
        for name, n in parts.items():
            self.offsets[name] = (at, at + n)
            at += n
        self.weight = nn.Parameter(torch.empty(at, in_features))
        nn.init.normal_(self.weight, std=in_features ** -0.5)
        self.bias = nn.Parameter(torch.zeros(at)) if bias else None

    def forward(self, h):
        y = F.linear(h, self.weight, self.bias)
        return {name: y[:, lo:hi] for name, (lo, hi) in self.offsets.items()}, y
