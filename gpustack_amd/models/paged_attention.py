"""Rotary softmax attention over a paged key/value pool, for models on the
fp32 stream (ModelSpec.fp32_residual). One module covers a family of
variants, every one a parameter of PagedMixerSpec:

* grouped-query heads with own key and value widths, projection biases;
* pairwise rotary on the first channels of each head, with optional
  wavelength-dependent frequency scaling; angles are pos * f in fp32;
* weighted RMS norm over the whole q / k projection before rotation;
* values tied to the keys (the raw key projection: not normed, not rotated);
* a sliding window that also keeps the first keys of the sequence;
* a per-head sink logit in the softmax denominator;
* differential scores: two score maps per head share one value stream,
  out = unit_rms(a1 - lambda * a2) * (1 - diff), lambda = exp(lq1.lk1) -
  exp(lq2.lk2) + diff;
* without rotation, positions entering through the scores instead: a
  weighted RMS norm per q / k head (one weight vector shared by the heads),
  a query temperature growing with the logarithm of the position, a
  per-head slope times the distance taken off every score, and values
  blended with those the first such layer of the stack computed for the
  same token (ops.head_norm_store prepares q and writes the pool);
* the per-head q / k norm FOLLOWED by a rotation (either pairing layout,
  optionally with a cos / sin amplitude) and with projection biases
  (ops.head_rope_store), and a tanh cap on the scaled scores.

Flow per step: one fused q/k/v GEMM -> ops.rotary_norm_store (norm, rotary,
cache write, all fp32 inside) -> ops.paged_attention over the block tables
of the batch (prompt portions and decode rows alike; every score map is a
"head" of the kernel) -> ops.diff_combine where there are two maps -> output
GEMM. This step's rows are read back from the pool like older positions.
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F
from torch import nn

from .. import ops
from ..engine.config import PagedMixerSpec


class PagedRotaryAttention(nn.Module):
    def __init__(self, width: int, m: PagedMixerSpec, eps: float, dtype,
                 comm=None, v_mix_first: bool = False):
        super().__init__()
        # per-head norm, then rotation: the generic per-head row kernel
        self.rope_rows = bool(m.head_norm and (m.rot.dims or m.bias)) \
            or m.rot.layout == "half"
        if self.rope_rows and (m.qk_norm_full or m.tied_values or m.maps != 1
                               or m.q_temp or m.v_mix or m.distance_bias):
            raise NotImplementedError(
                "the per-head norm + rotation row kernel serves one score "
                "map with its own values, without whole-row norms, query "
                "temperature, distance bias or value mixing")
        if m.head_norm and not self.rope_rows and (
                m.qk_norm_full or m.tied_values or m.maps != 1):
            raise NotImplementedError(
                "per-head q/k norm is served without whole-row norms, tied "
                "values or a second score map")
        if (m.q_temp or m.v_mix) and not m.head_norm:
            raise NotImplementedError(
                "query temperature and value mixing come with the per-head "
                "norm row kernel")
        # the first value-mixing layer of a stack lends its values to the
        # later ones and keeps its own unmixed
        self.v_mix_first = bool(m.v_mix and v_mix_first)
        if comm is not None and comm.tp_size > 1:
            raise NotImplementedError(
                "paged rotary attention is not sharded for tensor "
                "parallelism yet")
        if m.maps not in (1, 2):
            raise ValueError("one or two score maps per head")
        self.m, self.eps, self.comm = m, eps, comm
        self.nq = m.heads * m.maps * m.qk_dim
        self.nk = m.kv_heads * m.maps * m.qk_dim
        self.nv = 0 if m.tied_values else m.kv_heads * m.v_dim
        self.vw = m.v_width
        mk = lambda *shape, dt=dtype: nn.Parameter(
            torch.empty(*shape, dtype=dt), requires_grad=False)
        n = self.nq + self.nk + self.nv
        self.qkv_w = mk(n, width)
        self.qkv_b = mk(n) if m.bias else None
        self.o_w = mk(width, m.heads * self.vw)
        f32 = torch.float32
        self.q_norm = mk(self.nq, dt=f32) if m.qk_norm_full else None
        self.k_norm = mk(self.nk, dt=f32) if m.qk_norm_full else None
        self.sinks = mk(m.heads, dt=f32) if m.sink else None
        if m.head_norm:
            self.q_head_norm = mk(m.qk_dim, dt=f32)
            self.k_head_norm = mk(m.qk_dim, dt=f32)
        else:
            self.q_head_norm = self.k_head_norm = None
        self.v_lam = mk(1, dt=f32) if m.v_mix else None
        self.register_buffer(
            "slopes", torch.tensor(m.slopes(), dtype=torch.float64).to(f32)
            if m.distance_bias else None, persistent=False)
        # rows: lq1, lk1, lq2, lk2
        self.lam_vecs = mk(4, m.qk_dim, dt=f32) if m.maps == 2 else None
        self.register_buffer(
            "inv_freq", torch.tensor(m.rot.inv_freq(), dtype=torch.float64)
            .to(f32), persistent=False)
        self.register_buffer("lam", torch.zeros(1, dtype=f32),
                             persistent=False)

    def post_load(self) -> None:
        """Constants derived from loaded weights."""
        if self.lam_vecs is not None:
            v = self.lam_vecs.float()
            lam = (math.exp(float((v[0] * v[1]).sum()))
                   - math.exp(float((v[2] * v[3]).sum())) + self.m.diff)
            self.lam.fill_(lam)

    def forward(self, h, meta, k_cache, v_cache, shared=None):
        """`shared`: a dict that lives for one model step; value-mixing
        layers pass the first layer's values through it."""
        m = self.m
        T = h.shape[0]
        rg = meta.ragged
        qkv = F.linear(h, self.qkv_w, self.qkv_b)
        q = torch.empty(T, self.nq, dtype=h.dtype, device=h.device)
        groups = (rg.page_groups(k_cache.shape[2])
                  if h.is_cuda and k_cache.shape[2] == 16 else None)
        if self.rope_rows:
            rot0 = 0 if m.rot.dims else -1
            ops.head_rope_store(
                q, qkv, 0, m.heads, m.qk_dim, self.q_head_norm, m.qk_dim,
                rot0, self.nq, m.kv_heads, m.qk_dim, self.k_head_norm,
                m.qk_dim, rot0, self.nq + self.nk, self.inv_freq,
                m.rot.layout == "half", m.rot.amplitude, rg.pos32, k_cache,
                v_cache, meta.slot_mapping, self.eps, page_groups=groups)
        elif m.head_norm:
            v_first = None
            if m.v_mix and not self.v_mix_first:
                v_first = shared["v_first"]
            coef, every = m.q_temp or (0.0, 0.0)
            ops.head_norm_store(q, qkv, self.nq, self.nk, self.q_head_norm,
                                self.k_head_norm, m.qk_dim, coef, every,
                                rg.pos32, v_first, self.v_lam, k_cache,
                                v_cache, meta.slot_mapping, self.eps,
                                page_groups=groups)
            if self.v_mix_first:
                shared["v_first"] = qkv[:, self.nq + self.nk:]
        else:
            ops.rotary_norm_store(q, qkv, self.nq, self.nk, self.q_norm,
                                  self.k_norm, self.inv_freq, rg.pos32,
                                  m.qk_dim, k_cache, v_cache,
                                  meta.slot_mapping, self.eps, m.tied_values,
                                  page_groups=groups)
        A = m.heads * m.maps
        # two maps meet again in fp32 (their difference cancels digits)
        a = torch.empty(T, A, self.vw, device=h.device,
                        dtype=torch.float32 if m.maps == 2 else h.dtype)
        ops.paged_attention(
            a, q.view(T, A, m.qk_dim), k_cache, v_cache, rg.block_tables,
            rg.row_seq, rg.pos32, m.scale, maps=m.maps, window=m.window,
            keep_first=m.keep_first, sinks=self.sinks,
            tiles=rg.attn_tiles(m.heads, m.kv_heads, m.maps) if h.is_cuda
            else None, max_ctx=rg.max_ctx, slopes=self.slopes,
            softcap=m.softcap)
        if m.maps == 2:
            o = torch.empty(T, m.heads * self.vw, dtype=h.dtype,
                            device=h.device)
            ops.diff_combine(o, a.view(T, m.heads, 2, self.vw), self.lam,
                             m.diff, self.eps)
        else:
            o = a.view(T, A * self.vw)
        out = F.linear(o, self.o_w)
        return self.comm.all_reduce(out) if self.comm is not None else out
