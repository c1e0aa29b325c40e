"""Short causal convolutions over time with carried inputs (the depthwise "conv1d" in front of linear-attention
and state-space mixers), on packed variable-length batches.

``y_t = sum_j w[:, j] * u_(t - taps + 1 + j)`` per channel, zeros before a sequence's start; the last ``taps - 1``
inputs of every sequence are its state (``[slots, taps - 1, C]``, the input's dtype, updated in place), so a prompt
continued in a later step — or decoded token by token — sees the same window.  The channels are cut into up to three
segments of equal-width heads, each with what follows the convolution: nothing (0), RMS norm with a weight shared by
the heads (1), SiLU (2), SiLU then unit length times a scale (3).  One wave per (token, head); HIP kernels in
csrc/kernels/seq/seq_scan.hip.
"""
from __future__ import annotations

import torch

from . import reference as ref
from ._native import native_seq, use_seq

PLAIN, RMS, SILU, SILU_UNIT = 0, 1, 2, 3


def short_conv(u: torch.Tensor, weight: torch.Tensor, state: torch.Tensor | None, segments, sb, eps: float,
               out_f32: bool = False, bias: torch.Tensor | None = None) -> torch.Tensor:
    """``u`` ``[T, C]`` (a column slice of a wider matrix is fine), ``weight`` float ``[C, taps]``, ``segments`` a list
    of ``(first channel, heads, head width, mode, norm weight | None, scale)``, ``sb`` the step's ``SeqBatch``;
    ``bias`` float ``[C]`` is added before the segment's activation."""
    segs = [[int(s[0]), int(s[1]), int(s[2]), int(s[3])] for s in segments]
    sw = [s[4] for s in segments]
    sc = [float(s[5]) for s in segments]
    if use_seq(u):
        return native_seq().short_conv(u, weight, state, segs, sw, sc, sb.desc, sb.live, eps, out_f32, bias)
    return ref.short_conv(u, weight, state, segs, sw, sc, sb, eps, out_f32, bias)
