"""Recurrent mixers with one matrix state per head and sequence, for models
on the fp32 stream (ModelSpec.fp32_residual). Both run the same recurrence

    S_t = a_t S_(t-1) + b_t k_t v_t^T,    y_t = S_t^T q_t (+ skip * v_t)

(ops.state_scan) with the state [state x vdim] in fp32 in the sequence's
slot of the engine's state pool (engine/kv_cache.py): a step reads the slot
— or starts from zero when its first row sits at position 0 —, walks this
step's rows of the sequence in order and writes the slot back, so a prompt
cut into portions, a single decoded token and a whole prompt give the same
states. Nothing is kept per token.

* Mamba2Mixer: one projection gives z | x | B | C | dt; x, B and C pass a
  short causal convolution per channel and SiLU (ops.causal_conv_silu; its
  last taps - 1 inputs live in the slot too); a_t = exp(-exp(A_log) dt_t),
  b_t = dt_t = softplus(dt + dt_bias) per head, k = B and q = C shared by
  the heads of a group, v = x, skip = D. The output is gated by silu(z) and
  then RMS-normed in equal parts (ops.gated_group_norm).
* LightningMixer: one projection gives q | k | v | g; q, k, v go through
  SiLU on their way into the scan; a_t is a constant per head, b_t = 1. The
  output is RMS-normed over all heads and multiplied by sigmoid(g).

* GatedDeltaMixer runs the gated delta rule instead (ops.delta_scan),
      S_t = g_t S_(t-1) + k_t u_t^T,  u_t = beta_t (v_t - (g_t S_(t-1))^T k_t),
  y_t = S_t^T q_t: one projection gives q | k | v | gate | a | b; q, k, v
  pass the convolution and SiLU, q and k are scaled to unit length inside
  the scan, g_t = exp(-exp(A_log) softplus(a + dt_bias)), beta_t =
  sigmoid(b); each head's output is RMS-normed, weighted and multiplied by
  silu(gate).

Decays, step sizes, the recurrence and both norms are fp32; the
projections (library GEMMs) and the convolution run in the engine dtype.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F
from torch import nn

from .. import ops
from ..engine.config import ScanMixerSpec


def _mk(*shape, dt):
    return nn.Parameter(torch.empty(*shape, dtype=dt), requires_grad=False)


class Mamba2Mixer(nn.Module):
    def __init__(self, width: int, m: ScanMixerSpec, eps: float, dtype,
                 comm=None):
        super().__init__()
        if comm is not None and comm.tp_size > 1:
            raise NotImplementedError(
                "recurrent mixers are not sharded for tensor parallelism yet")
        self.m, self.eps, self.comm = m, eps, comm
        f32 = torch.float32
        gn = m.groups * m.state
        self.col_x = m.inner                   # columns of the projection
        self.col_dt = 2 * m.inner + 2 * gn
        self.in_w = _mk(self.col_dt + m.heads, width, dt=dtype)
        self.conv_w = _mk(m.conv_channels, m.conv, dt=f32)
        self.conv_b = _mk(m.conv_channels, dt=f32)
        self.dt_bias = _mk(m.heads, dt=f32)
        self.a_log = _mk(m.heads, dt=f32)
        self.skip = _mk(m.heads, dt=f32)
        self.norm = _mk(m.inner, dt=f32)
        self.o_w = _mk(width, m.inner, dt=dtype)

    def forward(self, h, meta, ssm_state, conv_state):
        m = self.m
        rg = meta.ragged
        T = h.shape[0]
        u = F.linear(h, self.in_w)
        xbc = torch.empty(T, m.conv_channels, dtype=h.dtype, device=h.device)
        ops.causal_conv_silu(xbc, u, self.col_x, self.conv_w, self.conv_b,
                             conv_state, rg.seq_first, rg.seq_rows,
                             rg.state_slots, rg.row_seq, rg.pos32)
        gn = m.groups * m.state
        y = torch.empty(T, m.inner, dtype=torch.float32, device=h.device)
        ops.state_scan(y, xbc, 0, m.inner, m.inner + gn, u, self.col_dt,
                       m.heads, m.groups, m.state, m.vdim, False,
                       self.dt_bias, self.a_log, self.skip, None, ssm_state,
                       rg.seq_first, rg.seq_rows, rg.state_slots, rg.pos32,
                       single=max(rg.seq_news, default=1) <= 1)
        g = torch.empty(T, m.inner, dtype=h.dtype, device=h.device)
        ops.gated_group_norm(g, y, u[:, :m.inner], self.norm, m.norm_groups,
                             self.eps, True)
        out = F.linear(g, self.o_w)
        return self.comm.all_reduce(out) if self.comm is not None else out


class LightningMixer(nn.Module):
    def __init__(self, width: int, m: ScanMixerSpec, eps: float, dtype,
                 comm=None):
        super().__init__()
        if comm is not None and comm.tp_size > 1:
            raise NotImplementedError(
                "recurrent mixers are not sharded for tensor parallelism yet")
        self.m, self.eps, self.comm = m, eps, comm
        f32 = torch.float32
        self.nqk = m.heads * m.state
        # rows: q | k | v | g
        self.qkvg_w = _mk(2 * self.nqk + 2 * m.inner, width, dt=dtype)
        self.norm = _mk(m.inner, dt=f32)
        self.o_w = _mk(width, m.inner, dt=dtype)
        self.register_buffer(
            "decay", torch.tensor(m.decay, dtype=torch.float64).to(f32),
            persistent=False)

    def forward(self, h, meta, ssm_state, conv_state=None):
        m = self.m
        rg = meta.ragged
        T = h.shape[0]
        u = F.linear(h, self.qkvg_w)
        y = torch.empty(T, m.inner, dtype=torch.float32, device=h.device)
        ops.state_scan(y, u, 2 * self.nqk, self.nqk, 0, None, 0, m.heads,
                       m.heads, m.state, m.vdim, True, None, None, None,
                       self.decay, ssm_state, rg.seq_first, rg.seq_rows,
                       rg.state_slots, rg.pos32,
                       single=max(rg.seq_news, default=1) <= 1)
        g = torch.empty(T, m.inner, dtype=h.dtype, device=h.device)
        ops.gated_group_norm(g, y, u[:, 2 * self.nqk + m.inner:], self.norm,
                             1, self.eps, False)
        out = F.linear(g, self.o_w)
        return self.comm.all_reduce(out) if self.comm is not None else out


class GatedDeltaMixer(nn.Module):
    def __init__(self, width: int, m: ScanMixerSpec, eps: float, dtype,
                 comm=None):
        super().__init__()
        if comm is not None and comm.tp_size > 1:
            raise NotImplementedError(
                "recurrent mixers are not sharded for tensor parallelism yet")
        self.m, self.eps, self.comm = m, eps, comm
        f32 = torch.float32
        self.nqk = m.groups * m.state
        # columns of the projection: q | k | v | gate | a | b
        self.col_gate = 2 * self.nqk + m.inner
        self.col_a = self.col_gate + m.inner
        self.col_b = self.col_a + m.heads
        self.in_w = _mk(self.col_b + m.heads, width, dt=dtype)
        self.conv_w = _mk(m.conv_channels, m.conv, dt=f32)   # q | k | v
        self.register_buffer("conv_b", torch.zeros(m.conv_channels, dtype=f32),
                             persistent=False)
        self.dt_bias = _mk(m.heads, dt=f32)
        self.a_log = _mk(m.heads, dt=f32)
        self.norm = _mk(m.vdim, dt=f32)          # one weight vector, all heads
        self.register_buffer("norm_rows", torch.ones(m.inner, dtype=f32),
                             persistent=False)
        self.o_w = _mk(width, m.inner, dt=dtype)

    def post_load(self) -> None:
        self.norm_rows.copy_(self.norm.repeat(self.m.heads))

    def forward(self, h, meta, ssm_state, conv_state):
        m = self.m
        rg = meta.ragged
        T = h.shape[0]
        u = F.linear(h, self.in_w)
        qkv = torch.empty(T, m.conv_channels, dtype=h.dtype, device=h.device)
        ops.causal_conv_silu(qkv, u, 0, self.conv_w, self.conv_b, conv_state,
                             rg.seq_first, rg.seq_rows, rg.state_slots,
                             rg.row_seq, rg.pos32)
        y = torch.empty(T, m.inner, dtype=torch.float32, device=h.device)
        ops.delta_scan(y, qkv, 0, self.nqk, 2 * self.nqk, u, self.col_a,
                       self.col_b, m.heads, m.groups, m.state, m.vdim,
                       self.dt_bias, self.a_log, ssm_state, rg.seq_first,
                       rg.seq_rows, rg.state_slots, rg.pos32,
                       single=max(rg.seq_news, default=1) <= 1)
        g = torch.empty(T, m.inner, dtype=h.dtype, device=h.device)
        ops.gated_group_norm(g, y, u[:, self.col_gate:self.col_a],
                             self.norm_rows, m.heads, self.eps, 2)
        out = F.linear(g, self.o_w)
        return self.comm.all_reduce(out) if self.comm is not None else out


def build_scan_mixer(width: int, m: ScanMixerSpec, eps: float, dtype,
                     comm=None):
    if m.kind == "delta":
        return GatedDeltaMixer(width, m, eps, dtype, comm)
    if m.kind == "mamba2":
        return Mamba2Mixer(width, m, eps, dtype, comm)
    if m.kind == "lightning":
        return LightningMixer(width, m, eps, dtype, comm)
    raise NotImplementedError(f"recurrent mixer kind {m.kind!r}")
