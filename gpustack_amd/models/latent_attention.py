"""Position-free latent attention mixer.

Every token leaves ONE RMS-normalised latent c (width R) in the paged pool;
head a's keys and values are the linear images U_k[a] c and U_v[a] c. No
rotation or other positional signal enters the scores, so — unlike the
DeepSeek-style MLAAttention in models/llama.py — there is no rope slice in
the cache row and the absorbed form is exact for the whole score:

    q~[t,a] = U_k[a]^T q[t,a]                       (width R, fp32)
    ctx[t,a] = softmax_{j<=pos(t)}(scale * q~[t,a] . c_j) . C
    out[t]   = W_o concat_a(U_v[a] ctx[t,a])

Only c is ever read per cached token (R values instead of
heads * (Dq + Dv)), by all heads of a row at once: ops.latent_attention
streams a sequence's latents once per 16 (row, head) pairs. Scores, the
softmax and the latent norm are fp32 in every engine dtype; head sizes,
latent width and score scale are constructor parameters.

RotaryLatentAttention is the variant with positions: every query head has a
rotated part beside the unrotated one and every token ONE rotated key part
shared by all heads, so a cache row is [latent c (R) | rotated key part]
and the score is q~ . c + q_rot . k_rot with q~ = U_k^T q_unrotated. To
the attention kernel that is multi-query attention with one key "head" of
width R + rot_dim whose first R channels are also the value, which is how
it is served: ops.head_rope_store norms the latent, turns the key part and
writes the row (and the latent again into the transposed value pages),
ops.paged_attention streams it for all heads of a row at once — behind a
sliding window and with a sink logit per head where the layer has them.
The queries come through a normed latent of their own; each head's output
is multiplied by a sigmoid gate read from the mixer's input; a layer may
own no down-projection and read the rows an earlier layer cached.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F
from torch import nn

from .. import ops
from ..engine.config import LatentMixerSpec


class LatentAttention(nn.Module):
    def __init__(self, width: int, m: LatentMixerSpec, eps: float, dtype,
                 comm=None):
        super().__init__()
        if comm is not None and comm.tp_size > 1:
            raise NotImplementedError(
                "latent attention is not sharded for tensor parallelism yet")
        self.comm = comm
        self.h, self.dq, self.dv, self.r = m.heads, m.qk_dim, m.v_dim, m.kv_rank
        self.scale = float(m.scale)
        self.eps = eps
        mk = lambda *shape, dt=dtype: nn.Parameter(
            torch.empty(*shape, dtype=dt), requires_grad=False)
        # q and the latent down-projection fused: one GEMM per layer entry
        self.qd_w = mk(self.h * self.dq + self.r, width)
        self.lat_norm = mk(self.r, dt=torch.float32)
        # absorbed factors, head-major, in the GEMM dtype (fp32 engines keep
        # every product fp32; bf16 engines feed the MFMA kernel, which
        # rounds q~ to bf16 anyway)
        self.uk = mk(self.h, self.dq, self.r)
        self.uv_t = mk(self.h, self.r, self.dv)
        self.o_w = mk(width, self.h * self.dv)

    def forward(self, h, meta, cache):
        T = h.shape[0]
        rg = meta.ragged
        nq = self.h * self.dq
        qd = F.linear(h, self.qd_w)                        # [T, H*Dq + R]
        # norm + cache write first: this step's rows are read back from
        # the pool like every earlier position
        ops.latent_norm_store(cache, qd, nq, self.lat_norm,
                              meta.slot_mapping, self.eps)
        q = qd[:, :nq].unflatten(1, (self.h, self.dq))     # [T, H, Dq]
        q_hts = torch.bmm(q.transpose(0, 1), self.uk)      # [H, T, R]
        if ops.latent_attention_mfma_ok(cache):
            # bf16 in, bf16 out, head-major buffers handed to the kernel as
            # strided [T, H, R] views: no transposing or casting passes
            # between the two batched projections and the kernel
            q_lat = q_hts.transpose(0, 1)
            ctx_hts = torch.empty(self.h, T, self.r, dtype=h.dtype,
                                  device=h.device)
            ctx = ctx_hts.transpose(0, 1)
        else:
            q_lat = q_hts.transpose(0, 1).float().contiguous()
            ctx = torch.empty(T, self.h, self.r, dtype=torch.float32,
                              device=h.device)
            ctx_hts = None
        ops.latent_attention(ctx, q_lat, cache, rg.block_tables, rg.row_seq,
                             rg.pos32, self.scale,
                             tiles=rg.latent_tiles(self.h) if h.is_cuda
                             else None, max_ctx=rg.max_ctx)
        if ctx_hts is None:
            ctx_hts = ctx.transpose(0, 1).to(self.uv_t.dtype)
        o = torch.bmm(ctx_hts, self.uv_t)                  # [H, T, Dv]
        o = o.transpose(0, 1).reshape(T, self.h * self.dv)  # [T, H*Dv]
        out = F.linear(o, self.o_w)
        return self.comm.all_reduce(out) if self.comm is not None else out


class RotaryLatentAttention(nn.Module):
    def __init__(self, width: int, m: LatentMixerSpec, eps: float, dtype,
                 comm=None):
        super().__init__()
        if comm is not None and comm.tp_size > 1:
            raise NotImplementedError(
                "latent attention is not sharded for tensor parallelism yet")
        if not (m.rot_dim and m.q_rank and m.rot is not None):
            raise NotImplementedError(
                "the rotary latent mixer needs a rotated part and a query "
                "latent")
        self.m, self.eps, self.comm = m, eps, comm
        self.h, self.dq, self.dv, self.r = m.heads, m.qk_dim, m.v_dim, m.kv_rank
        self.rd, self.qr = m.rot_dim, m.q_rank
        self.own_kv = m.kv_from < 0
        f32 = torch.float32
        mk = lambda *shape, dt=dtype: nn.Parameter(
            torch.empty(*shape, dtype=dt), requires_grad=False)
        # one GEMM on the mixer's input: query latent | key/value latent +
        # key part to rotate (when the layer owns them) | one gate per head
        self.n_kv = (self.r + self.rd) if self.own_kv else 0
        self.col_g = self.qr + self.n_kv
        self.in_w = mk(self.col_g + (self.h if m.out_gate else 0), width)
        self.q_norm = mk(self.qr, dt=f32)
        self.kv_norm = mk(self.r, dt=f32) if self.own_kv else None
        self.uq_w = mk(self.h * (self.dq + self.rd), self.qr)
        # absorbed key factor per head, extended by an identity block that
        # carries the rotated query part through the same batched product
        self.uk_ext = mk(self.h, self.dq + self.rd, self.r + self.rd)
        self.uv_t = mk(self.h, self.r, self.dv)
        self.sinks = mk(self.h, dt=f32) if m.sink else None
        self.o_w = mk(width, self.h * self.dv)
        self.register_buffer(
            "inv_freq", torch.tensor(m.rot.inv_freq(), dtype=torch.float64)
            .to(f32), persistent=False)

    def extend_uk(self, t):
        """Checkpoint U_k [heads * dim, R] -> [heads, dim + rot, R + rot]."""
        ext = torch.zeros(self.h, self.dq + self.rd, self.r + self.rd,
                          dtype=t.dtype, device=t.device)
        ext[:, :self.dq, :self.r] = t.view(self.h, self.dq, self.r)
        ext[:, self.dq:, self.r:] = torch.eye(self.rd, dtype=t.dtype,
                                              device=t.device)
        return ext

    def forward(self, h, meta, k_cache, v_cache):
        """k_cache / v_cache: this layer's pools, or those of the layer it
        borrows its keys from (then nothing is written)."""
        m = self.m
        T = h.shape[0]
        rg = meta.ragged
        H, dqr = self.h, self.dq + self.rd
        half = m.rot.layout == "half"
        amp = m.rot.amplitude
        u = F.linear(h, self.in_w)
        cq = torch.empty(T, self.qr, dtype=h.dtype, device=h.device)
        groups = (rg.page_groups(k_cache.shape[2])
                  if self.own_kv and h.is_cuda and k_cache.shape[2] == 16
                  else None)
        # query latent normed; latent normed + key part turned -> the pool.
        # This step's rows are read back from the pool like older ones
        ops.head_rope_store(
            cq, u, 0, 1, self.qr, self.q_norm, self.qr, -1,
            self.qr, 1 if self.own_kv else 0, self.r + self.rd, self.kv_norm,
            self.r, self.r, -1, self.inv_freq, half, amp, rg.pos32,
            k_cache if self.own_kv else None,
            v_cache if self.own_kv else None,
            meta.slot_mapping if self.own_kv else None, self.eps,
            page_groups=groups)
        qh = F.linear(cq, self.uq_w)                          # [T, H*(dq+rd)]
        qt = torch.empty_like(qh)
        ops.head_rope_store(
            qt, qh, 0, H, dqr, None, 0, self.dq, 0, 0, 0, None, 0, -1, -1,
            self.inv_freq, half, amp, rg.pos32, None, None, None, self.eps)
        q_lat = torch.bmm(qt.view(T, H, dqr).transpose(0, 1), self.uk_ext)
        ctx_hts = torch.empty(H, T, self.r, dtype=h.dtype, device=h.device)
        ops.paged_attention(
            ctx_hts.transpose(0, 1), q_lat.transpose(0, 1), k_cache, v_cache,
            rg.block_tables, rg.row_seq, rg.pos32, float(m.scale),
            window=m.window, sinks=self.sinks,
            tiles=rg.attn_tiles(H, 1, 1) if h.is_cuda else None,
            max_ctx=rg.max_ctx)
        o_hts = torch.bmm(ctx_hts, self.uv_t)                  # [H, T, dv]
        if m.out_gate:
            o = torch.empty(T, H * self.dv, dtype=h.dtype, device=h.device)
            ops.head_gate(o, o_hts, u, self.col_g)
        else:
            o = o_hts.transpose(0, 1).reshape(T, H * self.dv)
        out = F.linear(o, self.o_w)
        return self.comm.all_reduce(out) if self.comm is not None else out
