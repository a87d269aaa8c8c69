"""Livasun: a layer-listed pre-norm decoder on an fp32 stream whose layers
mix tokens in three different ways.

    x <- x + mixer(ln1(x));   x <- x + ff(ln2(x))

with layer norms that have a weight and a bias, scaled token embeddings, and
a final layer norm before the head. A layer's mixer is windowed softmax
attention without rotation (models/paged_attention.py: per-head q/k norm,
query temperature, distance bias, values blended with the first such
layer's) or one of two recurrent matrix-state mixers
(models/state_mixers.py); its feed-forward is the gated dense block, a
routed expert bank with a shared expert (models/experts.py), or absent.
Attention layers keep keys and values in the paged pools, recurrent layers
keep one state slot per live sequence (engine/kv_cache.py); both are driven
by the ragged batch view, so prompt portions, decode rows and mixed batches
take the same path.

One row kernel (ops.add_layer_norm) closes a sublayer and opens the next:
residual add on the fp32 stream and the next layer norm in the GEMM dtype.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F
from torch import nn

from .. import ops
from ..engine.config import EngineConfig, PagedMixerSpec
from ..parallel import Communicator
from .experts import DenseFF, RoutedFF
from .paged_attention import PagedRotaryAttention
from .state_mixers import build_scan_mixer


class LivasunLayer(nn.Module):
    def __init__(self, width, ls, eps, dtype, comm, v_mix_first):
        super().__init__()
        f32 = lambda: nn.Parameter(torch.empty(width, dtype=torch.float32),
                                   requires_grad=False)
        self.kind = ls.mixer_type
        if ls.mixer_type == "paged_attention":
            self.mixer = PagedRotaryAttention(width, ls.mixer, eps, dtype,
                                              comm, v_mix_first=v_mix_first)
        elif ls.mixer_type == "scan":
            self.mixer = build_scan_mixer(width, ls.mixer, eps, dtype, comm)
        else:
            raise NotImplementedError(ls.mixer_type)
        self.norm1_w, self.norm1_b = f32(), f32()
        if ls.mlp is None:
            self.mlp = None
        else:
            cls = RoutedFF if ls.mlp.kind == "moe" else DenseFF
            self.mlp = cls(width, ls.mlp, dtype, comm)
            self.norm2_w, self.norm2_b = f32(), f32()


class LivasunForCausalLM(nn.Module):
    uses_ragged_meta = True

    def __init__(self, cfg: EngineConfig, comm: Communicator, device):
        super().__init__()
        spec = cfg.spec
        if comm.pp_size > 1 or comm.tp_size > 1:
            raise NotImplementedError(
                "Livasun serves on one GPU per replica (no TP/PP sharding yet)")
        self.spec, self.cfg, self.comm = spec, cfg, comm
        self.device = torch.device(device)
        dtype = getattr(torch, cfg.dtype)
        self.dtype = dtype
        self.layer_offset = 0
        self.num_local_layers = spec.num_layers
        W = spec.hidden_size
        mk = lambda *shape, dt=dtype: nn.Parameter(
            torch.empty(*shape, dtype=dt), requires_grad=False)
        self.embed = mk(spec.vocab_size, W)
        layers, seen_mix = [], False
        for ls in spec.layers:
            first = (isinstance(ls.mixer, PagedMixerSpec) and ls.mixer.v_mix
                     and not seen_mix)
            seen_mix = seen_mix or first
            layers.append(LivasunLayer(W, ls, spec.rms_norm_eps, dtype, comm,
                                       first))
        self.layers = nn.ModuleList(layers)
        self.final_norm = mk(W, dt=torch.float32)
        self.final_norm_b = mk(W, dt=torch.float32)
        self.lm_head = mk(spec.vocab_size, W)
        self.lm_head_pack = None
        self.offload = None
        self.to(device)

    def graph_capturable(self) -> bool:
        """A decode step can be captured when nothing in it waits for the
        host: every routed feed-forward must take the grouped expert
        kernels (models/experts.py)."""
        import os

        for layer in self.layers:
            m = layer.mlp
            if isinstance(m, RoutedFF) and not (
                    self.dtype == torch.bfloat16
                    and self.spec.hidden_size % 64 == 0 and m.f.ff % 64 == 0
                    and os.environ.get("GPUSTACK_AMD_FUSED_MOE", "1") == "1"):
                return False
        return True

    @torch.inference_mode()
    def forward(self, token_ids, meta, kv, return_hidden: bool = False,
                return_both: bool = False):
        spec = self.spec
        eps = spec.rms_norm_eps
        T = token_ids.shape[0]
        dev = token_ids.device
        W = spec.hidden_size
        x = torch.empty(T, W, dtype=torch.float32, device=dev)
        h = torch.empty(T, W, dtype=self.dtype, device=dev)
        ops.embed_rows_scaled(x, token_ids, self.embed,
                              spec.embed_scale or 1.0)
        shared: dict = {}
        n = len(self.layers)
        if n:
            first = self.layers[0]
            ops.add_layer_norm(x, None, first.norm1_w, first.norm1_b, eps, h)
        for i, layer in enumerate(self.layers):
            if layer.kind == "paged_attention":
                a = layer.mixer(h, meta, kv.k_caches[i], kv.v_caches[i],
                                shared)
            else:
                a = layer.mixer(h, meta, kv.ssm_states[i], kv.conv_states[i])
            # the norm the stream meets next: this layer's second one, the
            # next layer's first, or none (the final norm runs on the
            # chosen rows only)
            nxt = self.layers[i + 1] if i + 1 < n else None
            nw, nb = (nxt.norm1_w, nxt.norm1_b) if nxt is not None \
                else (None, None)
            if layer.mlp is not None:
                ops.add_layer_norm(x, a, layer.norm2_w, layer.norm2_b, eps, h)
                f = layer.mlp(h, None)
                ops.add_layer_norm(x, f, nw, nb, eps, h)
            else:
                ops.add_layer_norm(x, a, nw, nb, eps, h)
        rows = x if return_hidden else x[meta.logits_indices].contiguous()
        y = torch.empty(rows.shape, dtype=self.dtype, device=dev)
        ops.add_layer_norm(rows, None, self.final_norm, self.final_norm_b,
                           eps, y)
        if return_hidden:
            return y
        logits = F.linear(y, self.lm_head).float()
        if return_both:
            return logits, y
        return logits
