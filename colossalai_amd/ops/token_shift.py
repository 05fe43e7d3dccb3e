"""Token shift over a ragged serving batch.

``h_t = x_t + (x_{t-1} - x_t) * mu`` element-wise, where ``x_{t-1}`` is the
previous token of the same sequence *before* shifting (zeros ahead of position
0). The last row of each sequence's portion is kept in ``prev`` (one row per
state slot) so the next step continues where this one stopped.
"""

import torch

from ._kernels import serving_kernels, use_serving_hip as use_hip
from .ragged import RaggedBatch

__all__ = ["token_shift", "token_shift_ref"]


def token_shift_ref(x, mu, prev, batch: RaggedBatch, out_dtype=None):
    xf = x.float()
    before = torch.empty_like(xf)
    before[1:] = xf[:-1]
    for i in range(batch.num_seqs):
        lo, hi, slot = batch.cu_host[i], batch.cu_host[i + 1], batch.slots_host[i]
        before[lo] = prev[slot] if batch.start_host[i] > 0 else 0.0
        prev[slot] = xf[hi - 1]
    return (xf + (before - xf) * mu.float()).to(out_dtype or x.dtype)


def token_shift(x, mu, prev, batch: RaggedBatch, out_dtype=None):
    """x [N, W] float32 residual rows, mu [W], prev [slots, W] float32 (rows
    may be strided); returns the mixer input [N, W] in ``out_dtype``."""
    if use_hip(x):
        return serving_kernels().token_shift(x, mu, prev, batch.cu, batch.start, batch.slots, batch.tok_seq,
                                             out_dtype or x.dtype)
    return token_shift_ref(x, mu, prev, batch, out_dtype)
