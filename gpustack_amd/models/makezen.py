"""Makezen: a layer-listed decoder on an fp32 stream whose sublayers sit
between two weight-only layer norms,

    x <- x + ln1b(mixer(ln1(x)));   x <- x + ln2b(ff(ln2(x)))

with the embedding output layer-normed before the first layer and the
embedding table as the head. A layer's mixer is rotary latent attention
(models/latent_attention.py RotaryLatentAttention: sliding window, sink
logits, output gate, optionally the cached rows of an earlier layer), the
gated delta rule (models/state_mixers.py GatedDeltaMixer) or softmax
attention and a gated delta rule side by side (models/parallel_mixer.py);
its feed-forward is the ungated dense block of models/experts.py or absent.
Attention keeps its rows in the paged pools, the delta rule one state slot
per live sequence (engine/kv_cache.py); both follow the ragged batch view,
so prompt portions, decode rows and mixed batches take the same path.

One row kernel (ops.sandwich_add_norm, centred) closes a sublayer and opens
the next: the norm after, the residual add on the fp32 stream and the next
norm before in the GEMM dtype.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F
from torch import nn

from .. import ops
from ..engine.config import EngineConfig
from ..parallel import Communicator
from .experts import DenseFF
from .latent_attention import RotaryLatentAttention
from .parallel_mixer import ParallelMixer
from .state_mixers import build_scan_mixer


class MakezenLayer(nn.Module):
    def __init__(self, width, ls, eps, dtype, comm):
        super().__init__()
        f32 = lambda: nn.Parameter(torch.empty(width, dtype=torch.float32),
                                   requires_grad=False)
        self.kind = ls.mixer_type
        if ls.mixer_type == "latent_attention":
            self.mixer = RotaryLatentAttention(width, ls.mixer, eps, dtype,
                                               comm)
        elif ls.mixer_type == "scan":
            self.mixer = build_scan_mixer(width, ls.mixer, eps, dtype, comm)
        elif ls.mixer_type == "parallel":
            self.mixer = ParallelMixer(width, ls.mixer, eps, dtype, comm)
        else:
            raise NotImplementedError(ls.mixer_type)
        self.pre1, self.post1 = f32(), f32()
        if ls.mlp is None:
            self.mlp = None
        else:
            if ls.mlp.kind != "dense":
                raise NotImplementedError(ls.mlp.kind)
            self.mlp = DenseFF(width, ls.mlp, dtype, comm)
            self.pre2, self.post2 = f32(), f32()


class MakezenForCausalLM(nn.Module):
    uses_ragged_meta = True
    tied_head = True

    def __init__(self, cfg: EngineConfig, comm: Communicator, device):
        super().__init__()
        spec = cfg.spec
        if comm.pp_size > 1 or comm.tp_size > 1:
            raise NotImplementedError(
                "Makezen serves on one GPU per replica (no TP/PP sharding yet)")
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
        self.embed_norm = mk(W, dt=torch.float32)
        self.layers = nn.ModuleList(
            [MakezenLayer(W, ls, spec.rms_norm_eps, dtype, comm)
             for ls in spec.layers])
        self.final_norm = mk(W, dt=torch.float32)
        self.lm_head = self.embed           # the head is the embedding table
        self.lm_head_pack = None
        self.offload = None
        self.to(device)

    def post_load(self) -> None:
        for layer in self.layers:
            if hasattr(layer.mixer, "post_load"):
                layer.mixer.post_load()

    def graph_capturable(self) -> bool:
        return True

    def _mix(self, i, layer, h, meta, kv):
        if layer.kind == "latent_attention":
            return layer.mixer(h, meta, kv.k_caches[i], kv.v_caches[i])
        if layer.kind == "scan":
            return layer.mixer(h, meta, kv.ssm_states[i], kv.conv_states[i])
        return layer.mixer(h, meta, kv.k_caches[i], kv.v_caches[i],
                           kv.ssm_states[i], kv.conv_states[i])

    @torch.inference_mode()
    def forward(self, token_ids, meta, kv, return_hidden: bool = False,
                return_both: bool = False):
        spec = self.spec
        eps = spec.rms_norm_eps
        T = token_ids.shape[0]
        dev = token_ids.device
        W = spec.hidden_size
        e = torch.empty(T, W, dtype=torch.float32, device=dev)
        ops.embed_rows_f32(e, token_ids, self.embed)
        # the stream starts as the normed embedding rows
        x = torch.zeros(T, W, dtype=torch.float32, device=dev)
        h = torch.empty(T, W, dtype=self.dtype, device=dev)
        layers = self.layers
        n = len(layers)
        ops.sandwich_add_norm(x, e, self.embed_norm, 1.0, eps, None,
                              layers[0].pre1 if n else None, h, center=True)
        for i, layer in enumerate(layers):
            a = self._mix(i, layer, h, meta, kv)
            nxt = layers[i + 1].pre1 if i + 1 < n else None
            if layer.mlp is not None:
                ops.sandwich_add_norm(x, a, layer.post1, 1.0, eps, None,
                                      layer.pre2, h, center=True)
                f = layer.mlp(h)
                ops.sandwich_add_norm(x, f, layer.post2, 1.0, eps, None, nxt,
                                      h, center=True)
            else:
                ops.sandwich_add_norm(x, a, layer.post1, 1.0, eps, None, nxt,
                                      h, center=True)
        rows = x if return_hidden else x[meta.logits_indices].contiguous()
        y = torch.empty(rows.shape, dtype=self.dtype, device=dev)
        ops.sandwich_add_norm(rows, None, None, 0.0, eps, None,
                              self.final_norm, y, center=True)
        if return_hidden:
            return y
        logits = F.linear(y, self.lm_head).float()
        if return_both:
            return logits, y
        return logits
