"""Feed-forward blocks of the layer-listed models: dense, and a routed
expert bank.

Both compute W_down act(W_up h) with a selectable activation; the dense
block also has a gated form, W_down (act(W_gate h) * W_up h), with gate and
up fused into one GEMM (the gated SiLU blocks of the llama lineage live in
models/llama.py). The bank routes
with full-softmax scores and group-limited top-k — experts sit in equal
groups of neighbours, a group is ranked by its best member, only the best
`keep_groups` groups stay eligible — and weights the chosen experts by
score * route_scale without renormalising. An optional shared expert runs
for every token and is scaled by a per-token sigmoid gate. Variants, all
parameters of FeedForwardSpec (ops.route_topk): sigmoid scores, a learned
per-expert correction that counts for the choice only, groups ranked by the
sum of their best few choice scores, chosen weights divided by their sum,
an ungated shared expert.

Router logits, scores, the gate and the weighted sum are fp32; the router
and gate rows are fused into one fp32 GEMM on the fp32 stream.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F
from torch import nn

from .. import ops
from ..engine.config import FeedForwardSpec


class DenseFF(nn.Module):
    def __init__(self, width: int, f: FeedForwardSpec, dtype, comm=None):
        super().__init__()
        if comm is not None and comm.tp_size > 1:
            raise NotImplementedError("ungated FF is not TP-sharded yet")
        self.act, self.gated, self.ff = f.act, f.gated, f.ff
        # gated: rows [0, ff) are the gate, [ff, 2 ff) the up projection
        self.up_w = nn.Parameter(
            torch.empty(f.ff * (2 if f.gated else 1), width, dtype=dtype),
            requires_grad=False)
        self.down_w = nn.Parameter(torch.empty(width, f.ff, dtype=dtype),
                                   requires_grad=False)

    def forward(self, h, x32=None):
        u = F.linear(h, self.up_w)
        if self.gated:
            g = torch.empty(h.shape[0], self.ff, dtype=h.dtype,
                            device=h.device)
            ops.act_and_mul(g, u, self.act)
            u = g
        else:
            ops.act_inplace(u, self.act)
        return F.linear(u, self.down_w)


class RoutedFF(nn.Module):
    def __init__(self, width: int, f: FeedForwardSpec, dtype, comm=None):
        super().__init__()
        if comm is not None and comm.tp_size > 1:
            raise NotImplementedError("ungated expert bank is not TP-sharded yet")
        if f.experts % max(f.groups, 1):
            raise ValueError("experts must divide evenly into groups")
        self.f = f
        self.e, self.top = f.experts, f.top
        mk = lambda *shape, dt=dtype: nn.Parameter(
            torch.empty(*shape, dtype=dt), requires_grad=False)
        self.gated = bool(f.shared_ff and f.shared_gated)
        # rows [0, E): router; row E (when gated): the shared expert's gate
        self.router_w = mk(self.e + (1 if self.gated else 0), width,
                           dt=torch.float32)
        self.correction = (mk(self.e, dt=torch.float32)
                           if f.route_correction else None)
        # the plain softmax / best-member routing keeps its own kernel
        self.scored = (f.route_scores != "softmax" or f.route_correction
                       or f.group_top != 1 or f.renorm)
        if f.route_scores not in ("softmax", "sigmoid"):
            raise ValueError(f"route_scores {f.route_scores!r}")
        self.up_w = mk(self.e, f.ff, width)
        self.down_w = mk(self.e, width, f.ff)
        if f.shared_ff:
            self.shared_up_w = mk(f.shared_ff, width)
            self.shared_down_w = mk(width, f.shared_ff)
        else:
            self.shared_up_w = self.shared_down_w = None

    def fused_ok(self, h) -> bool:
        import os

        return (ops.grouped_ff_available(h, h.shape[1], self.f.ff)
                and os.environ.get("GPUSTACK_AMD_FUSED_MOE", "1") == "1")

    def _consts(self, TK: int, dev):
        """Per-size constant tensors, kept for the module's lifetime: a
        captured graph refers to them by address."""
        cache = self.__dict__.setdefault("_const_cache", {})
        c = cache.get(TK)
        if c is None:
            c = (torch.ones(TK, dtype=torch.int32, device=dev),
                 torch.arange(TK, dtype=torch.int32, device=dev))
            if TK <= 4096:
                cache[TK] = c
        return c

    def forward(self, h, x32):
        T, W = h.shape
        dev = h.device
        # x32 None: the router reads h itself (fp32 product of its values)
        logits = F.linear(x32 if x32 is not None else h.float(),
                          self.router_w)                    # fp32 [T, E(+1)]
        experts = torch.empty(T, self.top, dtype=torch.int32, device=dev)
        weights = torch.empty(T, self.top, dtype=torch.float32, device=dev)
        if self.scored:
            ops.route_topk(experts, weights, logits, self.correction, self.e,
                           self.f.groups, self.f.keep_groups,
                           self.f.group_top,
                           self.f.route_scores == "sigmoid", self.f.renorm,
                           self.f.route_scale)
        else:
            ops.route_grouped_topk(experts, weights, logits, self.e,
                                   self.f.groups, self.f.keep_groups,
                                   self.f.route_scale)
        # sort the T*top assignments by expert; each expert then owns one
        # contiguous row range of the gathered activations
        TK = T * self.top
        flat = experts.reshape(-1).long()
        order = torch.argsort(flat, stable=True)
        u = torch.empty(TK, self.f.ff, dtype=h.dtype, device=dev)
        y = torch.empty(TK, W, dtype=h.dtype, device=dev)
        capturing = h.is_cuda and torch.cuda.is_current_stream_capturing()
        if self.fused_ok(h) and (TK <= 32 * self.e or capturing):
            # decode-sized: grouped MFMA kernels, no host sync, fixed grids
            ones, ar = self._consts(TK, dev)
            counts = torch.zeros(self.e, dtype=torch.int32, device=dev)
            counts.scatter_add_(0, flat, ones)
            offs = (counts.cumsum(0, dtype=torch.int32) - counts).to(torch.int32)
            s_tok = (order // self.top).to(torch.int32)
            ops.grouped_up_act(u, h, self.up_w, s_tok, offs, counts, self.f.act)
            ops.grouped_down(y, u, self.down_w, offs, counts)
        else:
            # prompt-sized (or unaligned sizes, fp32, CPU): per-expert
            # library GEMMs on contiguous row ranges; one host sync
            counts = torch.bincount(flat, minlength=self.e).tolist()
            xs = h.index_select(0, order // self.top)       # [T*top, W]
            off = 0
            for e, n in enumerate(counts):
                if n:
                    torch.mm(xs[off:off + n], self.up_w[e].t(),
                             out=u[off:off + n])
                off += n
            ops.act_inplace(u, self.f.act)
            off = 0
            for e, n in enumerate(counts):
                if n:
                    torch.mm(u[off:off + n], self.down_w[e].t(),
                             out=y[off:off + n])
                off += n
            ar = torch.arange(TK, dtype=torch.int32, device=dev)
        inv = torch.empty(TK, dtype=torch.int32, device=dev)
        inv[order] = ar
        shared = None
        if self.shared_up_w is not None:
            su = F.linear(h, self.shared_up_w)
            ops.act_inplace(su, self.f.act)
            shared = F.linear(su, self.shared_down_w)
        out = torch.empty(T, W, dtype=torch.float32, device=dev)
        ops.moe_combine(out, y, inv.view(T, self.top), weights, shared,
                        logits if self.gated else None, self.e)
        return out
