"""Two mixers side by side on the same normed input, for models on the fp32
stream: softmax attention over the paged pool (models/paged_attention.py)
and a recurrent matrix-state mixer (models/state_mixers.py). Each output is
RMS-normed over the model width with a weight of its own and the two are
averaged (ops.dual_rms_mix, statistics in fp32):

    out = (rmsnorm(left(h)) * w_left + rmsnorm(right(h)) * w_right) / 2

A layer run of this kind holds both a paged key/value pool and a state slot;
the two halves are built from their own specs, so any attention variant can
sit beside any recurrence.
"""
from __future__ import annotations

import torch
from torch import nn

from .. import ops
from ..engine.config import ParallelMixerSpec
from .paged_attention import PagedRotaryAttention
from .state_mixers import build_scan_mixer


class ParallelMixer(nn.Module):
    def __init__(self, width: int, m: ParallelMixerSpec, eps: float, dtype,
                 comm=None):
        super().__init__()
        self.eps = eps
        self.left = PagedRotaryAttention(width, m.left, eps, dtype, comm)
        self.right = build_scan_mixer(width, m.right, eps, dtype, comm)
        f32 = lambda: nn.Parameter(torch.empty(width, dtype=torch.float32),
                                   requires_grad=False)
        self.left_out, self.right_out = f32(), f32()

    def post_load(self) -> None:
        for half in (self.left, self.right):
            if hasattr(half, "post_load"):
                half.post_load()

    def forward(self, h, meta, k_cache, v_cache, ssm_state, conv_state):
        a = self.left(h, meta, k_cache, v_cache)
        b = self.right(h, meta, ssm_state, conv_state)
        out = torch.empty_like(a)
        ops.dual_rms_mix(out, a, self.left_out, b, self.right_out, self.eps)
        return out
