"""Layer-level comparison bench: a Vunitar, Fusipel, Livasun or Makezen stack (`family`) at
real-model layer sizes beside the closest llama-lineage stack of equal
width, depth and heads (random weights, synthetic tokens). Reports end-to-end prefill and decode
throughput through LLMEngine for both, and per-kernel rates of the new
kernels next to their counterparts with the fraction of the MI355X
roofline each reaches (2.5 PFLOP/s dense bf16, 8 TB/s HBM3E).

Run through `python bench.py --layer-bench [--layer-family fusipel]
[--layer-sizes small,medium]`; bench.py's default workload is untouched.
"""
from __future__ import annotations

import json
import time

import torch

PEAK_FLOPS = 2.5e15
PEAK_BW = 8.0e12

SIZES = {
    # width, heads, latent width, dense ff, experts, expert ff, layers
    "small": dict(width=1024, heads=8, rank=256, ff=4096, experts=16, eff=512, layers=4),
    "medium": dict(width=2048, heads=16, rank=512, ff=8192, experts=32, eff=1024, layers=4),
    "large": dict(width=4096, heads=32, rank=512, ff=14336, experts=32, eff=2048, layers=2),
}


def vunitar_spec(s, moe: bool):
    from ..engine.config import (FeedForwardSpec, LatentMixerSpec, LayerSpec,
                                 ModelSpec)

    mixer = LatentMixerSpec(heads=s["heads"], qk_dim=128, v_dim=128,
                            kv_rank=s["rank"], scale=128 ** -0.5)
    if moe:
        ff = FeedForwardSpec(kind="moe", ff=s["eff"], act="gelu",
                             experts=s["experts"], top=4, groups=4,
                             keep_groups=2, route_scale=2.0,
                             shared_ff=s["eff"], shared_gated=True)
    else:
        ff = FeedForwardSpec(kind="dense", ff=s["ff"], act="relu2")
    return ModelSpec(
        architecture="Vunitar", vocab_size=32000, hidden_size=s["width"],
        num_layers=s["layers"],
        layers=tuple(LayerSpec("latent_attention", mixer, ff)
                     for _ in range(s["layers"])),
        num_heads=1, num_kv_heads=1, head_dim=8, intermediate_size=0,
        rms_norm_eps=1e-6, max_position_embeddings=1 << 20, eos_token_id=-1,
        norm_after=True, layer_scale=True, fp32_residual=True,
        final_logit_softcap=30.0, bigram_buckets=4093, bigram_mul_prev=131,
        bigram_mul_cur=17)


def fusipel_spec(s, moe: bool = False):
    """Alternating mixers at head size 128: values tied to the keys with a
    sink (heads/4 kv heads), and two-map differential attention behind a
    512-key window that keeps 4 first keys (half the heads, two maps each);
    gated tanh-GELU feed-forward of the llama stack's width."""
    from ..engine.config import (FeedForwardSpec, LayerSpec, ModelSpec,
                                 PagedMixerSpec, RotarySpec)

    H = s["heads"]
    rot = RotarySpec(dims=64, base=10000.0, scaling=(8.0, 1.0, 4.0, 8192.0))
    tied = PagedMixerSpec(heads=H, kv_heads=max(1, H // 4), qk_dim=128,
                          v_dim=128, scale=128 ** -0.5, rot=rot, bias=True,
                          sink=True, qk_norm_full=True, tied_values=True)
    diff = PagedMixerSpec(heads=max(1, H // 2), kv_heads=max(1, H // 8),
                          qk_dim=128, v_dim=128, scale=128 ** -0.5, rot=rot,
                          bias=True, maps=2, diff=0.4, window=512,
                          keep_first=4)
    ff = FeedForwardSpec(kind="dense", ff=s["ff"], act="gelu_tanh", gated=True)
    return ModelSpec(
        architecture="Fusipel", vocab_size=32000, hidden_size=s["width"],
        num_layers=s["layers"],
        layers=tuple(LayerSpec("paged_attention", diff if i % 2 else tied, ff)
                     for i in range(s["layers"])),
        num_heads=1, num_kv_heads=1, head_dim=8, intermediate_size=0,
        rms_norm_eps=1e-6, max_position_embeddings=1 << 20, eos_token_id=-1,
        sandwich_norms=True, fp32_residual=True, residual_multiplier=0.7)


def livasun_spec(s, moe: bool = False):
    """Layers cycle windowed attention (head size 128, heads/4 kv heads,
    window 1024, query temperature, value blend), a mamba2 mixer (inner =
    2 x width in heads of 64, state 128, 8 groups, 4 taps), attention again
    and a lightning mixer (heads x 128 x 128); gated SiLU feed-forward of
    the llama stack's width, or a sigmoid-routed expert bank with a shared
    expert."""
    from ..engine.config import (FeedForwardSpec, LayerSpec, ModelSpec,
                                 PagedMixerSpec, ScanMixerSpec)

    H, W = s["heads"], s["width"]
    attn = PagedMixerSpec(heads=H, kv_heads=max(1, H // 4), qk_dim=128,
                          v_dim=128, scale=128 ** -0.5, window=1024,
                          head_norm=True, q_temp=(0.1, 1024),
                          distance_bias=True, v_mix=True)
    mamba = ScanMixerSpec(kind="mamba2", heads=2 * W // 64, state=128, vdim=64,
                          groups=8, conv=4, norm_groups=8)
    light = ScanMixerSpec(kind="lightning", heads=H, state=128, vdim=128,
                          groups=H, decay=tuple(
                              1.0 - 2.0 ** (-5.0 - 5.0 * h / max(H - 1, 1))
                              for h in range(H)))
    if moe:
        ff = FeedForwardSpec(kind="moe", ff=s["eff"], act="relu2",
                             experts=s["experts"], top=4, groups=4,
                             keep_groups=2, route_scale=2.5,
                             shared_ff=s["eff"], route_scores="sigmoid",
                             route_correction=True, group_top=2, renorm=True)
    else:
        ff = FeedForwardSpec(kind="dense", ff=s["ff"], act="silu", gated=True)
    cycle = [("paged_attention", attn), ("scan", mamba),
             ("paged_attention", attn), ("scan", light)]
    return ModelSpec(
        architecture="Livasun", vocab_size=32000, hidden_size=W,
        num_layers=s["layers"],
        layers=tuple(LayerSpec(*cycle[i % 4], ff) for i in range(s["layers"])),
        num_heads=1, num_kv_heads=1, head_dim=8, intermediate_size=0,
        rms_norm_eps=1e-5, max_position_embeddings=1 << 20, eos_token_id=-1,
        fp32_residual=True, norm_type="layernorm_bias", embed_scale=4.0)


def makezen_spec(s, moe: bool = False):
    """Layers cycle rotary latent attention (head sizes 128 + 64 rotated,
    latent 384 — 256 at the small size —, query latent 3/4 of the width,
    window 1024, sinks, output gates), a gated delta rule (heads x 128 x
    128, half as many key heads, 4 taps), softmax attention (head size 128,
    heads/4 kv heads, 64 rotated channels, capped scores) beside a delta
    rule of half the heads, and latent attention on the first layer's
    cache; ungated tanh-GELU feed-forward of the llama stack's width."""
    from ..engine.config import (FeedForwardSpec, LatentMixerSpec, LayerSpec,
                                 ModelSpec, PagedMixerSpec, ParallelMixerSpec,
                                 RotarySpec, ScanMixerSpec)

    H, W = s["heads"], s["width"]
    R = makezen_rank(s)
    rot = RotarySpec(dims=64, base=10000.0, layout="half",
                     ramp=(4.0, 4096.0, 32.0, 1.0))
    lat = dict(heads=H, qk_dim=128, v_dim=128, kv_rank=R,
               scale=192 ** -0.5, rot_dim=64, rot=rot, q_rank=3 * W // 4,
               window=1024, sink=True, out_gate=True)
    delta = ScanMixerSpec(kind="delta", heads=H, state=128, vdim=128,
                          groups=max(1, H // 2), conv=4)
    left = PagedMixerSpec(heads=H, kv_heads=max(1, H // 4), qk_dim=128,
                          v_dim=128, scale=128 ** -0.5, rot=rot, bias=True,
                          head_norm=True, softcap=30.0)
    right = ScanMixerSpec(kind="delta", heads=max(1, H // 2), state=128,
                          vdim=128, groups=max(1, H // 4), conv=4)
    ff = FeedForwardSpec(kind="dense", ff=s["ff"], act="gelu_tanh")
    cycle = [("latent_attention", LatentMixerSpec(**lat)), ("scan", delta),
             ("parallel", ParallelMixerSpec(left=left, right=right)),
             ("latent_attention", LatentMixerSpec(**lat, kv_from=0))]
    return ModelSpec(
        architecture="Makezen", vocab_size=32000, hidden_size=W,
        num_layers=s["layers"],
        layers=tuple(LayerSpec(*cycle[i % 4], ff) for i in range(s["layers"])),
        num_heads=1, num_kv_heads=1, head_dim=8, intermediate_size=0,
        rms_norm_eps=1e-5, max_position_embeddings=1 << 20, eos_token_id=-1,
        sandwich_norms=True, fp32_residual=True, norm_type="layernorm",
        embed_norm=True, tie_word_embeddings=True)


def makezen_rank(s) -> int:
    return 256 if s["width"] <= 1024 else 384


def llama_spec(s, moe: bool):
    from ..engine.config import ModelSpec

    kw = dict(vocab_size=32000, hidden_size=s["width"],
              intermediate_size=s["ff"], num_layers=s["layers"],
              num_heads=s["heads"], num_kv_heads=max(1, s["heads"] // 4),
              head_dim=128, max_position_embeddings=1 << 20, eos_token_id=-1)
    if moe:
        kw.update(architecture="Qwen3MoeForCausalLM", qk_norm=True,
                  num_experts=s["experts"], num_experts_per_tok=4,
                  moe_intermediate_size=s["eff"])
    return ModelSpec(**kw)


def _engine(spec, device, max_seqs, max_len):
    from ..engine import EngineConfig, LLMEngine

    cfg = EngineConfig(model="layer-bench", device=device, max_num_seqs=max_seqs,
                       max_model_len=max_len, max_prefill_tokens=8192,
                       gpu_memory_utilization=0.5, admission_min_seqs=1)
    cfg.spec = spec
    cfg.max_model_len = max_len
    return LLMEngine(cfg)


def _sync():
    if torch.cuda.is_available():
        torch.cuda.synchronize()


def engine_rates(spec, device, B_pre=8, L=1024, B_dec=64, n_dec=32):
    from ..engine import SamplingParams

    eng = _engine(spec, device, max(B_dec, B_pre), L + n_dec + 8)
    g = torch.Generator().manual_seed(0)
    mk = lambda n: torch.randint(2, spec.vocab_size, (n,), generator=g).tolist()

    def prefill_once():
        for _ in range(B_pre):
            eng.add_request(mk(L), SamplingParams(max_tokens=1, ignore_eos=True))
        while eng.has_unfinished():
            eng.step()

    prefill_once()
    _sync()
    t0 = time.perf_counter()
    reps = 3
    for _ in range(reps):
        prefill_once()
    _sync()
    pre = reps * B_pre * L / (time.perf_counter() - t0)

    for _ in range(B_dec):
        eng.add_request(mk(L), SamplingParams(max_tokens=n_dec + 8,
                                              ignore_eos=True))
    while eng.num_running < B_dec and eng.has_unfinished():
        eng.step()
    for _ in range(4):
        eng.step()
    _sync()
    t0 = time.perf_counter()
    steps = n_dec - 8
    for _ in range(steps):
        eng.step()
    _sync()
    dec = steps * B_dec / (time.perf_counter() - t0)
    while eng.has_unfinished():
        eng.step()
    del eng
    if torch.cuda.is_available():
        torch.cuda.empty_cache()
    return pre, dec


def _time(fn, iters=20):
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(True), torch.cuda.Event(True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / iters * 1e-3


def kernel_rates(s, device):
    """Per-kernel rates: (name, seconds, achieved, unit, roofline share)."""
    from .. import ops

    bf = torch.bfloat16
    H, R, W, D, BS = s["heads"], s["rank"], s["width"], 128, 16
    out = []

    def rec(name, sec, flops=None, nbytes=None):
        if flops is not None:
            out.append(dict(kernel=name, us=round(sec * 1e6, 1),
                            tflops=round(flops / sec / 1e12, 1),
                            roofline=round(flops / sec / PEAK_FLOPS, 4)))
        else:
            out.append(dict(kernel=name, us=round(sec * 1e6, 1),
                            gbps=round(nbytes / sec / 1e9, 1),
                            roofline=round(nbytes / sec / PEAK_BW, 4)))

    # ---- prefill attention: 4 prompts x 2048 ----
    nseq, L = 4, 2048
    T = nseq * L
    pairs = nseq * L * (L + 1) // 2
    nblk = T // BS + 1
    pool = torch.randn(nblk, 2, BS, R, device=device).to(bf)
    bt = torch.arange(nseq * (L // BS), dtype=torch.int32, device=device).view(nseq, -1)
    row_seq = torch.arange(nseq, dtype=torch.int32, device=device).repeat_interleave(L)
    pos = torch.arange(L, dtype=torch.int32, device=device).repeat(nseq)
    q = torch.randn(T, H, R, device=device) * R ** -0.5
    ctx = torch.empty_like(q)
    tiles = ops.build_latent_tiles([i * L for i in range(nseq)], [0] * nseq,
                                   [L] * nseq, H, device)
    rec("latent_attention prefill (mfma)",
        _time(lambda: ops.latent_attention(ctx, q, pool, bt, row_seq, pos, 1.0,
                                           tiles=tiles), 5),
        flops=4.0 * R * H * pairs)
    qf = torch.randn(T, H, D, device=device).to(bf)
    kf = torch.randn(T, max(1, H // 4), D, device=device).to(bf)
    vf = torch.randn_like(kf)
    of = torch.empty_like(qf)
    ptiles = ops.build_prefill_tiles([L] * nseq, device)
    rec("flash_prefill (llama graph)",
        _time(lambda: ops.varlen_prefill_attn(of, qf, kf, vf, [L] * nseq,
                                              D ** -0.5, tiles=ptiles), 5),
        flops=4.0 * D * H * pairs)

    # ---- decode attention: 64 sequences x 2048 cached ----
    B, Lc = 64, 2048
    nblk = B * (Lc // BS) + 1
    pool = torch.randn(nblk, 2, BS, R, device=device).to(bf)
    bt = torch.arange(B * (Lc // BS), dtype=torch.int32, device=device).view(B, -1)
    row_seq = torch.arange(B, dtype=torch.int32, device=device)
    pos = torch.full((B,), Lc - 1, dtype=torch.int32, device=device)
    q = torch.randn(B, H, R, device=device) * R ** -0.5
    ctx = torch.empty_like(q)
    tiles = ops.build_latent_tiles(list(range(B)), [Lc - 1] * B, [1] * B, H, device)
    rec("latent_attention decode (mfma)",
        _time(lambda: ops.latent_attention(ctx, q, pool, bt, row_seq, pos, 1.0,
                                           tiles=tiles, max_ctx=Lc)),
        nbytes=B * Lc * R * 2 * 2)
    hkv = max(1, H // 4)
    kc = torch.randn(nblk, hkv, BS, D, device=device).to(bf)
    vc = torch.randn_like(kc)
    qd = torch.randn(B, H, D, device=device).to(bf)
    od = torch.empty_like(qd)
    lens = torch.full((B,), Lc, dtype=torch.int32, device=device)
    rec("paged_attn_decode (llama graph)",
        _time(lambda: ops.paged_attn_decode(od, qd, kc, vc, bt, lens, D ** -0.5)),
        nbytes=B * Lc * hkv * D * 2 * 2)

    # ---- row kernels at T = 8192 ----
    T = 8192
    x = torch.randn(T, W, device=device)
    a = torch.randn(T, W, device=device).to(bf)
    w32 = torch.ones(W, device=device)
    hb = torch.empty(T, W, dtype=bf, device=device)
    rec("rms_scale_add (fp32 stream + bf16 copy)",
        _time(lambda: ops.rms_scale_add(x, a, w32, w32, 1e-6, hb)),
        nbytes=T * W * 12)
    xb, rb = a.clone(), a.clone()
    wb = torch.ones(W, dtype=bf, device=device)
    rec("fused_add_rms_norm (llama graph)",
        _time(lambda: ops.fused_add_rms_norm(xb, rb, wb, 1e-6)),
        nbytes=T * W * 8)
    u = torch.randn(T, s["ff"], device=device).to(bf)
    rec("act_inplace relu2", _time(lambda: ops.act_inplace(u, "relu2")),
        nbytes=T * s["ff"] * 4)
    gu = torch.randn(T, 2 * s["ff"], device=device).to(bf)
    ao = torch.empty(T, s["ff"], dtype=bf, device=device)
    rec("silu_and_mul (llama graph)", _time(lambda: ops.silu_and_mul(ao, gu)),
        nbytes=T * s["ff"] * 6)
    nblk = T // BS + 1
    pool = torch.zeros(nblk, 2, BS, R, dtype=bf, device=device)
    src = torch.randn(T, H * D + R, device=device).to(bf)
    slots = torch.arange(T, device=device)      # a prompt: consecutive slots
    rec("latent_norm_store (norm + both planes)",
        _time(lambda: ops.latent_norm_store(pool, src, H * D, w32[:R].contiguous()
                                            if R <= W else torch.ones(R, device=device),
                                            slots, 1e-6)),
        nbytes=T * R * 6)
    hkv = max(1, H // 4)
    kk = torch.randn(T, hkv, D, device=device).to(bf)
    kc = torch.zeros(nblk, hkv, BS, D, dtype=bf, device=device)
    vc = torch.zeros_like(kc)
    rec("reshape_and_cache (llama graph)",
        _time(lambda: ops.reshape_and_cache(kk, kk, kc, vc, slots)),
        nbytes=T * hkv * D * 8)
    return out


def fusipel_kernel_rates(s, device):
    """Per-kernel rates of the paged rotary attention family next to the
    llama graph's counterparts."""
    from .. import ops

    bf = torch.bfloat16
    H, W, D, BS = s["heads"], s["width"], 128, 16
    G = max(1, H // 4)
    out = []

    def rec(name, sec, flops=None, nbytes=None):
        if flops is not None:
            out.append(dict(kernel=name, us=round(sec * 1e6, 1),
                            tflops=round(flops / sec / 1e12, 1),
                            roofline=round(flops / sec / PEAK_FLOPS, 4)))
        else:
            out.append(dict(kernel=name, us=round(sec * 1e6, 1),
                            gbps=round(nbytes / sec / 1e9, 1),
                            roofline=round(nbytes / sec / PEAK_BW, 4)))

    def pools(nblk, g, kw, vw):
        return (torch.randn(nblk, g, BS, kw, device=device).to(bf),
                torch.randn(nblk, g, vw, BS, device=device).to(bf))

    # ---- prefill attention: 4 prompts x 2048 ----
    nseq, L = 4, 2048
    T = nseq * L
    pairs = nseq * L * (L + 1) // 2
    nblk = T // BS + 1
    bt = torch.arange(nseq * (L // BS), dtype=torch.int32, device=device).view(nseq, -1)
    row_seq = torch.arange(nseq, dtype=torch.int32, device=device).repeat_interleave(L)
    pos = torch.arange(L, dtype=torch.int32, device=device).repeat(nseq)
    starts = [i * L for i in range(nseq)]
    kc, vc = pools(nblk, G, D, D)
    q = torch.randn(T, H, D, device=device).to(bf)
    o = torch.empty_like(q)
    sinks = torch.zeros(H, device=device)
    tiles = ops.build_attn_tiles(starts, [0] * nseq, [L] * nseq, H, G, 1, device)
    rec("paged_attention prefill, causal + sink (mfma)",
        _time(lambda: ops.paged_attention(o, q, kc, vc, bt, row_seq, pos,
                                          D ** -0.5, sinks=sinks, tiles=tiles), 5),
        flops=4.0 * D * H * pairs)
    # two maps, window 512 + 4 kept: H/2 heads x 2 maps = H score maps
    Gd = max(1, H // 8)
    kc2, vc2 = pools(nblk, Gd, 2 * D, D)
    o32 = torch.empty(T, H, D, device=device)
    tiles2 = ops.build_attn_tiles(starts, [0] * nseq, [L] * nseq,
                                  max(1, H // 2), Gd, 2, device)
    wpairs = nseq * sum(min(i + 1, 512 + 4) for i in range(L))
    rec("paged_attention prefill, 2 maps, window 512 (mfma)",
        _time(lambda: ops.paged_attention(o32, q, kc2, vc2, bt, row_seq, pos,
                                          D ** -0.5, maps=2, window=512,
                                          keep_first=4, tiles=tiles2), 5),
        flops=4.0 * D * H * wpairs)
    kf = torch.randn(T, G, D, device=device).to(bf)
    vf = torch.randn_like(kf)
    of = torch.empty_like(q)
    ptiles = ops.build_prefill_tiles([L] * nseq, device)
    rec("flash_prefill (llama graph)",
        _time(lambda: ops.varlen_prefill_attn(of, q, kf, vf, [L] * nseq,
                                              D ** -0.5, tiles=ptiles), 5),
        flops=4.0 * D * H * pairs)

    # ---- decode attention: 64 sequences x 2048 cached ----
    B, Lc = 64, 2048
    nblk = B * (Lc // BS) + 1
    bt = torch.arange(B * (Lc // BS), dtype=torch.int32, device=device).view(B, -1)
    row_seq = torch.arange(B, dtype=torch.int32, device=device)
    pos = torch.full((B,), Lc - 1, dtype=torch.int32, device=device)
    kc, vc = pools(nblk, G, D, D)
    qd = torch.randn(B, H, D, device=device).to(bf)
    od = torch.empty_like(qd)
    tiles = ops.build_attn_tiles(list(range(B)), [Lc - 1] * B, [1] * B, H, G, 1,
                                 device)
    rec("paged_attention decode, causal + sink (mfma)",
        _time(lambda: ops.paged_attention(od, qd, kc, vc, bt, row_seq, pos,
                                          D ** -0.5, sinks=sinks, tiles=tiles,
                                          max_ctx=Lc)),
        nbytes=B * Lc * G * D * 2 * 2)
    kl = torch.randn(nblk, G, BS, D, device=device).to(bf)
    vl = torch.randn_like(kl)
    lens = torch.full((B,), Lc, dtype=torch.int32, device=device)
    rec("paged_attn_decode (llama graph)",
        _time(lambda: ops.paged_attn_decode(od, qd, kl, vl, bt, lens, D ** -0.5)),
        nbytes=B * Lc * G * D * 2 * 2)

    # ---- row kernels at T = 8192 ----
    T = 8192
    x = torch.randn(T, W, device=device)
    a = torch.randn(T, W, device=device).to(bf)
    w32 = torch.ones(W, device=device)
    hb = torch.empty(T, W, dtype=bf, device=device)
    rec("sandwich_add_norm (post-norm + add + pre-norm, fp32 stream)",
        _time(lambda: ops.sandwich_add_norm(x, a, w32, 0.5, 1e-6, None, w32, hb)),
        nbytes=T * W * 12)
    xb, rb = a.clone(), a.clone()
    wb = torch.ones(W, dtype=bf, device=device)
    rec("fused_add_rms_norm (llama graph)",
        _time(lambda: ops.fused_add_rms_norm(xb, rb, wb, 1e-6)),
        nbytes=T * W * 8)
    gu = torch.randn(T, 2 * s["ff"], device=device).to(bf)
    ao = torch.empty(T, s["ff"], dtype=bf, device=device)
    rec("act_and_mul gelu_tanh", _time(lambda: ops.act_and_mul(ao, gu, "gelu_tanh")),
        nbytes=T * s["ff"] * 6)
    rec("silu_and_mul (llama graph)", _time(lambda: ops.silu_and_mul(ao, gu)),
        nbytes=T * s["ff"] * 6)
    nblk = T // BS + 1
    nq, nk = H * D, G * D
    kc, vc = pools(nblk, G, D, D)
    qkv = torch.randn(T, nq + nk, device=device).to(bf)
    qo = torch.empty(T, nq, dtype=bf, device=device)
    qw, kw = torch.ones(nq, device=device), torch.ones(nk, device=device)
    inv = torch.tensor([10000.0 ** (-i / 32) for i in range(32)], device=device)
    slots = torch.arange(T, device=device)
    p32 = torch.arange(T, dtype=torch.int32, device=device)
    rec("rotary_norm_store, values row by row (decode's way)",
        _time(lambda: ops.rotary_norm_store(qo, qkv, nq, nk, qw, kw, inv, p32, D,
                                            kc, vc, slots, 1e-6, True)),
        nbytes=T * (2 * nq + 3 * nk) * 2)
    pg = ops.build_page_groups([0], [0], [T], BS, device)
    rec("rotary_norm_store (q/k norm + rotary + cache write, values by page)",
        _time(lambda: ops.rotary_norm_store(qo, qkv, nq, nk, qw, kw, inv, p32, D,
                                            kc, vc, slots, 1e-6, True,
                                            page_groups=pg)),
        nbytes=T * (2 * nq + 3 * nk) * 2)
    kk = torch.randn(T, G, D, device=device).to(bf)
    kl = torch.zeros(nblk, G, BS, D, dtype=bf, device=device)
    vl = torch.zeros_like(kl)
    rec("reshape_and_cache (llama graph)",
        _time(lambda: ops.reshape_and_cache(kk, kk, kl, vl, slots)),
        nbytes=T * G * D * 8)
    # the same function as the llama graph runs it (its q/k-normed models):
    # per-head norm of q, of k, rotary, cache write — four launches; priced
    # with the fused kernel's byte count, so the shares compare times
    qh = torch.randn(T, H, D, device=device).to(bf)
    wn = torch.ones(D, dtype=bf, device=device)
    cs = ops.build_cos_sin_cache(D, 64, T, 10000.0, None, device)
    p64 = torch.arange(T, device=device)

    def llama_chain():
        ops.rms_norm(qh.view(-1, D), qh.view(-1, D), wn, 1e-6)
        ops.rms_norm(kk.view(-1, D), kk.view(-1, D), wn, 1e-6)
        ops.rotary_embedding(p64, qh, kk, cs, D, 64)
        ops.reshape_and_cache(kk, kk, kl, vl, slots)

    rec("rms_norm q, k + rotary_embedding + reshape_and_cache (llama graph)",
        _time(llama_chain), nbytes=T * (2 * nq + 3 * nk) * 2)
    a4 = torch.randn(T, max(1, H // 2), 2, D, device=device)
    oc = torch.empty(T, max(1, H // 2) * D, dtype=bf, device=device)
    lam = torch.tensor([0.7], device=device)
    rec("diff_combine (a1 - lambda a2, unit rms)",
        _time(lambda: ops.diff_combine(oc, a4, lam, 0.4, 1e-6)),
        nbytes=T * H * D * 4 + T * (H // 2) * D * 2)
    return out


PEAK_VALU = 157.3e12     # fp32 vector ALU


def livasun_kernel_rates(s, device):
    """Per-kernel rates of the Livasun kernels next to the llama graph's
    counterparts (the recurrent mixers have none there: their like is the
    attention kernel of the same phase)."""
    from .. import ops

    bf = torch.bfloat16
    H, W, D, BS = s["heads"], s["width"], 128, 16
    G = max(1, H // 4)
    out = []

    def rec(name, sec, flops=None, nbytes=None, peak=PEAK_FLOPS):
        if flops is not None:
            out.append(dict(kernel=name, us=round(sec * 1e6, 1),
                            tflops=round(flops / sec / 1e12, 1),
                            roofline=round(flops / sec / peak, 4)))
        else:
            out.append(dict(kernel=name, us=round(sec * 1e6, 1),
                            gbps=round(nbytes / sec / 1e9, 1),
                            roofline=round(nbytes / sec / PEAK_BW, 4)))

    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=device)
    # ---- prefill attention: 4 prompts x 2048, window 1024 ----
    nseq, L, win = 4, 2048, 1024
    T = nseq * L
    nblk = T // BS + 1
    bt = torch.arange(nseq * (L // BS), dtype=torch.int32, device=device).view(nseq, -1)
    row_seq = torch.arange(nseq, dtype=torch.int32, device=device).repeat_interleave(L)
    pos = torch.arange(L, dtype=torch.int32, device=device).repeat(nseq)
    starts = [i * L for i in range(nseq)]
    kc = torch.randn(nblk, G, BS, D, device=device).to(bf)
    vc = torch.randn(nblk, G, D, BS, device=device).to(bf)
    q = torch.randn(T, H, D, device=device).to(bf)
    o = torch.empty_like(q)
    slopes = torch.tensor([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)],
                          device=device)
    tiles = ops.build_attn_tiles(starts, [0] * nseq, [L] * nseq, H, G, 1, device)
    wpairs = nseq * sum(min(i + 1, win) for i in range(L))
    rec("paged_attention prefill, window 1024 + slopes (mfma, useful pairs)",
        _time(lambda: ops.paged_attention(o, q, kc, vc, bt, row_seq, pos,
                                          D ** -0.5, window=win, tiles=tiles,
                                          slopes=slopes), 5),
        flops=4.0 * D * H * wpairs)
    kf = torch.randn(T, G, D, device=device).to(bf)
    vf = torch.randn_like(kf)
    ptiles = ops.build_prefill_tiles([L] * nseq, device)
    rec("flash_prefill (llama graph, causal)",
        _time(lambda: ops.varlen_prefill_attn(o, q, kf, vf, [L] * nseq,
                                              D ** -0.5, tiles=ptiles), 5),
        flops=4.0 * D * H * nseq * L * (L + 1) // 2)

    # ---- decode attention: 64 sequences x 2048 cached, window 1024 ----
    B, Lc = 64, 2048
    nblk = B * (Lc // BS) + 1
    bt = torch.arange(B * (Lc // BS), dtype=torch.int32, device=device).view(B, -1)
    row_seq = torch.arange(B, dtype=torch.int32, device=device)
    pos = torch.full((B,), Lc - 1, dtype=torch.int32, device=device)
    kc = torch.randn(nblk, G, BS, D, device=device).to(bf)
    vc = torch.randn(nblk, G, D, BS, device=device).to(bf)
    qd = torch.randn(B, H, D, device=device).to(bf)
    od = torch.empty_like(qd)
    tiles = ops.build_attn_tiles(list(range(B)), [Lc - 1] * B, [1] * B, H, G, 1,
                                 device)
    rec("paged_attention decode, window 1024 + slopes (mfma)",
        _time(lambda: ops.paged_attention(od, qd, kc, vc, bt, row_seq, pos,
                                          D ** -0.5, window=win, tiles=tiles,
                                          max_ctx=Lc, slopes=slopes)),
        nbytes=B * win * G * D * 2 * 2)
    kl = torch.randn(nblk, G, BS, D, device=device).to(bf)
    vl = torch.randn_like(kl)
    lens = torch.full((B,), Lc, dtype=torch.int32, device=device)
    rec("paged_attn_decode (llama graph, 2048 keys)",
        _time(lambda: ops.paged_attn_decode(od, qd, kl, vl, bt, lens, D ** -0.5)),
        nbytes=B * Lc * G * D * 2 * 2)

    # ---- row kernels at T = 8192 ----
    T = 8192
    x = torch.randn(T, W, device=device)
    a = torch.randn(T, W, device=device).to(bf)
    w32 = torch.ones(W, device=device)
    hb = torch.empty(T, W, dtype=bf, device=device)
    rec("add_layer_norm (add + layer norm, fp32 stream)",
        _time(lambda: ops.add_layer_norm(x, a, w32, w32, 1e-5, hb)),
        nbytes=T * W * 12)
    xb, rb = a.clone(), a.clone()
    wb = torch.ones(W, dtype=bf, device=device)
    rec("fused_add_rms_norm (llama graph)",
        _time(lambda: ops.fused_add_rms_norm(xb, rb, wb, 1e-6)),
        nbytes=T * W * 8)
    nblk = T // BS + 1
    nq, nk = H * D, G * D
    kc = torch.zeros(nblk, G, BS, D, dtype=bf, device=device)
    vc = torch.zeros(nblk, G, D, BS, dtype=bf, device=device)
    qkv = torch.randn(T, nq + 2 * nk, device=device).to(bf)
    vfirst = torch.randn(T, nq + 2 * nk, device=device).to(bf)[:, nq + nk:]
    qo = torch.empty(T, nq, dtype=bf, device=device)
    wd = torch.ones(D, device=device)
    lam = torch.tensor([0.3], device=device)
    slots = torch.arange(T, device=device)
    p32 = torch.arange(T, dtype=torch.int32, device=device)
    pg = ops.build_page_groups([0], [0], [T], BS, device)
    nb_store = T * (2 * nq + 2 * nk + 4 * nk) * 2   # q in/out, k in/out, v in, blend, back, page
    rec("head_norm_store (head norms + temperature + blend + cache write, values by page)",
        _time(lambda: ops.head_norm_store(qo, qkv, nq, nk, wd, wd, D, 0.1, 1024,
                                          p32, vfirst, lam, kc, vc, slots, 1e-5,
                                          page_groups=pg)),
        nbytes=nb_store)
    rec("head_norm_store, values row by row (decode's way)",
        _time(lambda: ops.head_norm_store(qo, qkv, nq, nk, wd, wd, D, 0.1, 1024,
                                          p32, vfirst, lam, kc, vc, slots, 1e-5)),
        nbytes=T * (2 * nq + 2 * nk + 3 * nk) * 2)
    qh = torch.randn(T, H, D, device=device).to(bf)
    kk = torch.randn(T, G, D, device=device).to(bf)
    kl = torch.zeros(nblk, G, BS, D, dtype=bf, device=device)
    vl = torch.zeros_like(kl)
    wn = torch.ones(D, dtype=bf, device=device)
    cs = ops.build_cos_sin_cache(D, 64, T, 10000.0, None, device)
    p64 = torch.arange(T, device=device)

    def llama_chain():
        ops.rms_norm(qh.view(-1, D), qh.view(-1, D), wn, 1e-6)
        ops.rms_norm(kk.view(-1, D), kk.view(-1, D), wn, 1e-6)
        ops.rotary_embedding(p64, qh, kk, cs, D, 64)
        ops.reshape_and_cache(kk, kk, kl, vl, slots)

    rec("rms_norm q, k + rotary_embedding + reshape_and_cache (llama graph)",
        _time(llama_chain), nbytes=T * (2 * nq + 2 * nk + 3 * nk) * 2)
    gu = torch.randn(T, 2 * s["ff"], device=device).to(bf)
    ao = torch.empty(T, s["ff"], dtype=bf, device=device)
    rec("act_and_mul silu", _time(lambda: ops.act_and_mul(ao, gu, "silu")),
        nbytes=T * s["ff"] * 6)
    rec("silu_and_mul (llama graph)", _time(lambda: ops.silu_and_mul(ao, gu)),
        nbytes=T * s["ff"] * 6)

    # ---- recurrent mixers ----
    Hm, N, P, Gm, taps = 2 * W // 64, 128, 64, 8, 4
    inner, gn = Hm * P, Gm * N
    C = inner + 2 * gn
    for label, nseq, L in (("prefill 8 x 1024", 8, 1024), ("decode 64 x 1", 64, 1)):
        T = nseq * L
        sf, sr = i32([i * L for i in range(nseq)]), i32([L] * nseq)
        ss = i32(list(range(nseq)))
        rs = torch.arange(nseq, dtype=torch.int32, device=device).repeat_interleave(L)
        ps = (torch.arange(L, dtype=torch.int32, device=device) + 5).repeat(nseq)
        u = torch.randn(T, 2 * inner + 2 * gn + Hm, device=device).to(bf)
        xbc = torch.empty(T, C, dtype=bf, device=device)
        cw, cb = torch.randn(C, taps, device=device), torch.zeros(C, device=device)
        cst = torch.zeros(nseq + 1, taps - 1, C, dtype=bf, device=device)
        rec(f"causal_conv_silu {label}",
            _time(lambda: ops.causal_conv_silu(xbc, u, inner, cw, cb, cst, sf, sr,
                                               ss, rs, ps)),
            nbytes=T * C * 4)
        y = torch.empty(T, inner, device=device)
        st = torch.zeros(nseq + 1, Hm, N, P, device=device)
        hv = torch.zeros(Hm, device=device)
        sec = _time(lambda: ops.state_scan(y, xbc, 0, inner, inner + gn, u,
                                           2 * inner + 2 * gn, Hm, Gm, N, P,
                                           False, hv - 1, hv, hv + 1, None, st,
                                           sf, sr, ss, ps, single=L == 1), 5)
        if L > 1:
            rec(f"state_scan mamba2 {label} (fp32 vector ALU)", sec,
                flops=4.0 * T * Hm * N * P, peak=PEAK_VALU)
        else:
            rec(f"state_scan mamba2 {label} (state read + write)", sec,
                nbytes=nseq * Hm * N * P * 8)
        # lightning: H heads of 128 x 128
        ul = torch.randn(T, 4 * H * 128, device=device).to(bf)
        yl = torch.empty(T, H * 128, device=device)
        stl = torch.zeros(nseq + 1, H, 128, 128, device=device)
        dec = torch.full((H,), 0.99, device=device)
        sec = _time(lambda: ops.state_scan(yl, ul, 2 * H * 128, H * 128, 0, None,
                                           0, H, H, 128, 128, True, None, None,
                                           None, dec, stl, sf, sr, ss, ps,
                                           single=L == 1), 5)
        if L > 1:
            rec(f"state_scan lightning {label} (fp32 vector ALU)", sec,
                flops=4.0 * T * H * 128 * 128, peak=PEAK_VALU)
        else:
            rec(f"state_scan lightning {label} (state read + write)", sec,
                nbytes=nseq * H * 128 * 128 * 8)
        g = torch.empty(T, inner, dtype=bf, device=device)
        wi = torch.ones(inner, device=device)
        rec(f"gated_group_norm {label}",
            _time(lambda: ops.gated_group_norm(g, y, u[:, :inner], wi, 8, 1e-5,
                                               True)),
            nbytes=T * inner * 8)
    # ---- routing at T = 8192 ----
    T, E = 8192, s["experts"]
    lg = torch.randn(T, E, device=device)
    ex = torch.empty(T, 4, dtype=torch.int32, device=device)
    wt = torch.empty(T, 4, device=device)
    corr = torch.zeros(E, device=device)
    rec("route_topk (sigmoid + correction + top-2 group rank)",
        _time(lambda: ops.route_topk(ex, wt, lg, corr, E, 4, 2, 2, True, True,
                                     2.0)), nbytes=T * (E * 4 + 32))
    rec("route_grouped_topk (softmax, best member)",
        _time(lambda: ops.route_grouped_topk(ex, wt, lg, E, 4, 2, 2.0)),
        nbytes=T * (E * 4 + 32))
    return out


def makezen_kernel_rates(s, device):
    """Per-kernel rates of the Makezen kernels next to their likes in the
    Livasun stack (windowed attention, the matrix-state scan and step, its
    row kernels)."""
    from .. import ops

    bf = torch.bfloat16
    H, W, D, BS = s["heads"], s["width"], 128, 16
    G = max(1, H // 4)
    R = makezen_rank(s)
    KW = R + 64
    out = []

    def rec(name, sec, flops=None, nbytes=None, peak=PEAK_FLOPS):
        if flops is not None:
            out.append(dict(kernel=name, us=round(sec * 1e6, 1),
                            tflops=round(flops / sec / 1e12, 1),
                            roofline=round(flops / sec / peak, 4)))
        else:
            out.append(dict(kernel=name, us=round(sec * 1e6, 1),
                            gbps=round(nbytes / sec / 1e9, 1),
                            roofline=round(nbytes / sec / PEAK_BW, 4)))

    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=device)
    # ---- prefill attention: 4 prompts x 2048 ----
    nseq, L, win = 4, 2048, 1024
    T = nseq * L
    nblk = T // BS + 1
    bt = torch.arange(nseq * (L // BS), dtype=torch.int32, device=device).view(nseq, -1)
    row_seq = torch.arange(nseq, dtype=torch.int32, device=device).repeat_interleave(L)
    pos = torch.arange(L, dtype=torch.int32, device=device).repeat(nseq)
    starts = [i * L for i in range(nseq)]
    wpairs = nseq * sum(min(i + 1, win) for i in range(L))
    pairs = nseq * L * (L + 1) // 2
    sinks = torch.zeros(H, device=device)
    # latent rows: one key "head" of R + 64 channels, values its first R
    kc = torch.randn(nblk, 1, BS, KW, device=device).to(bf)
    vc = torch.randn(nblk, 1, R, BS, device=device).to(bf)
    q_hts = torch.randn(H, T, KW, device=device).to(bf)
    c_hts = torch.empty(H, T, R, dtype=bf, device=device)
    tiles = ops.build_attn_tiles(starts, [0] * nseq, [L] * nseq, H, 1, 1, device)
    rec("paged_attention prefill, latent rows, window 1024 + sink (mfma, useful pairs)",
        _time(lambda: ops.paged_attention(c_hts.transpose(0, 1),
                                          q_hts.transpose(0, 1), kc, vc, bt,
                                          row_seq, pos, 0.07, window=win,
                                          sinks=sinks, tiles=tiles), 5),
        flops=2.0 * (KW + R) * H * wpairs)
    kc = torch.randn(nblk, G, BS, D, device=device).to(bf)
    vc = torch.randn(nblk, G, D, BS, device=device).to(bf)
    q = torch.randn(T, H, D, device=device).to(bf)
    o = torch.empty_like(q)
    tiles = ops.build_attn_tiles(starts, [0] * nseq, [L] * nseq, H, G, 1, device)
    rec("paged_attention prefill, causal + score cap (mfma)",
        _time(lambda: ops.paged_attention(o, q, kc, vc, bt, row_seq, pos,
                                          D ** -0.5, tiles=tiles, softcap=30.0), 5),
        flops=4.0 * D * H * pairs)
    slopes = torch.tensor([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)],
                          device=device)
    rec("paged_attention prefill, window 1024 + slopes (Livasun, useful pairs)",
        _time(lambda: ops.paged_attention(o, q, kc, vc, bt, row_seq, pos,
                                          D ** -0.5, window=win, tiles=tiles,
                                          slopes=slopes), 5),
        flops=4.0 * D * H * wpairs)

    # ---- decode attention: 64 sequences x 2048 cached ----
    B, Lc = 64, 2048
    nblk = B * (Lc // BS) + 1
    bt = torch.arange(B * (Lc // BS), dtype=torch.int32, device=device).view(B, -1)
    row_seq = torch.arange(B, dtype=torch.int32, device=device)
    pos = torch.full((B,), Lc - 1, dtype=torch.int32, device=device)
    kc = torch.randn(nblk, 1, BS, KW, device=device).to(bf)
    vc = torch.randn(nblk, 1, R, BS, device=device).to(bf)
    q_hts = torch.randn(H, B, KW, device=device).to(bf)
    c_hts = torch.empty(H, B, R, dtype=bf, device=device)
    tiles = ops.build_attn_tiles(list(range(B)), [Lc - 1] * B, [1] * B, H, 1, 1,
                                 device)
    rec("paged_attention decode, latent rows, window 1024 + sink (mfma)",
        _time(lambda: ops.paged_attention(c_hts.transpose(0, 1),
                                          q_hts.transpose(0, 1), kc, vc, bt,
                                          row_seq, pos, 0.07, window=win,
                                          sinks=sinks, tiles=tiles, max_ctx=Lc)),
        nbytes=B * win * (KW + R) * 2)
    kc = torch.randn(nblk, G, BS, D, device=device).to(bf)
    vc = torch.randn(nblk, G, D, BS, device=device).to(bf)
    qd = torch.randn(B, H, D, device=device).to(bf)
    od = torch.empty_like(qd)
    tiles = ops.build_attn_tiles(list(range(B)), [Lc - 1] * B, [1] * B, H, G, 1,
                                 device)
    rec("paged_attention decode, causal + score cap (mfma)",
        _time(lambda: ops.paged_attention(od, qd, kc, vc, bt, row_seq, pos,
                                          D ** -0.5, tiles=tiles, max_ctx=Lc,
                                          softcap=30.0)),
        nbytes=B * Lc * G * D * 2 * 2)
    rec("paged_attention decode, window 1024 + slopes (Livasun)",
        _time(lambda: ops.paged_attention(od, qd, kc, vc, bt, row_seq, pos,
                                          D ** -0.5, window=win, tiles=tiles,
                                          max_ctx=Lc, slopes=slopes)),
        nbytes=B * win * G * D * 2 * 2)

    # ---- row kernels at T = 8192 ----
    T = 8192
    x = torch.randn(T, W, device=device)
    a = torch.randn(T, W, device=device).to(bf)
    w32 = torch.ones(W, device=device)
    hb = torch.empty(T, W, dtype=bf, device=device)
    rec("sandwich_add_norm, centred (layer norm + add + layer norm, fp32 stream)",
        _time(lambda: ops.sandwich_add_norm(x, a, w32, 1.0, 1e-5, None, w32, hb,
                                            center=True)),
        nbytes=T * W * 12)
    rec("add_layer_norm (Livasun: add + layer norm)",
        _time(lambda: ops.add_layer_norm(x, a, w32, w32, 1e-5, hb)),
        nbytes=T * W * 12)
    b2 = torch.randn(T, W, device=device).to(bf)
    rec("dual_rms_mix (two RMS norms, mean)",
        _time(lambda: ops.dual_rms_mix(hb, a, w32, b2, w32, 1e-5)),
        nbytes=T * W * 6)
    nblk = T // BS + 1
    nq, nk = H * D, G * D
    kc = torch.zeros(nblk, G, BS, D, dtype=bf, device=device)
    vc = torch.zeros(nblk, G, D, BS, dtype=bf, device=device)
    qkv = torch.randn(T, nq + 2 * nk, device=device).to(bf)
    qo = torch.empty(T, nq, dtype=bf, device=device)
    wd = torch.ones(D, device=device)
    inv = torch.tensor([10000.0 ** (-i / 32) for i in range(32)], device=device)
    slots = torch.arange(T, device=device)
    p32 = torch.arange(T, dtype=torch.int32, device=device)
    pg = ops.build_page_groups([0], [0], [T], BS, device)
    nb_rows = T * (2 * nq + 2 * nk + 2 * nk) * 2      # q, k in/out; v in/out
    for label, groups in (("values by page", pg), ("values row by row", None)):
        rec(f"head_rope_store (head norms + rotation + cache write, {label})",
            _time(lambda: ops.head_rope_store(
                qo, qkv, 0, H, D, wd, D, 0, nq, G, D, wd, D, 0, nq + nk, inv,
                True, 1.1, p32, kc, vc, slots, 1e-5, page_groups=groups)),
            nbytes=nb_rows)
    vfirst = torch.randn(T, nk, device=device).to(bf)
    lam = torch.tensor([0.3], device=device)
    rec("head_norm_store (Livasun: head norms + temperature + blend + cache write, values by page)",
        _time(lambda: ops.head_norm_store(qo, qkv, nq, nk, wd, wd, D, 0.1, 1024,
                                          p32, vfirst, lam, kc, vc, slots, 1e-5,
                                          page_groups=pg)),
        nbytes=nb_rows + T * nk * 2)
    # latent rows: query latent normed, latent normed + key part turned,
    # key row and value pages written
    QR = 3 * W // 4
    u = torch.randn(T, QR + KW + H, device=device).to(bf)
    cq = torch.empty(T, QR, dtype=bf, device=device)
    kc1 = torch.zeros(nblk, 1, BS, KW, dtype=bf, device=device)
    vc1 = torch.zeros(nblk, 1, R, BS, dtype=bf, device=device)
    wq, wr = torch.ones(QR, device=device), torch.ones(R, device=device)
    rec("head_rope_store, latent rows (two norms + rotation + key row + value pages)",
        _time(lambda: ops.head_rope_store(
            cq, u, 0, 1, QR, wq, QR, -1, QR, 1, KW, wr, R, R, -1, inv, True,
            1.1, p32, kc1, vc1, slots, 1e-5)),
        nbytes=T * (2 * QR + 2 * KW + R) * 2)
    qh = torch.randn(T, H * 192, device=device).to(bf)
    qt = torch.empty_like(qh)
    rec("head_rope_store, query heads (rotation of the last 64 of 192 channels)",
        _time(lambda: ops.head_rope_store(
            qt, qh, 0, H, 192, None, 0, 128, 0, 0, 0, None, 0, -1, -1, inv,
            True, 1.1, p32, None, None, None, 1e-5)),
        nbytes=T * H * 192 * 4)
    o_hts = torch.randn(H, T, D, device=device).to(bf)
    og = torch.empty(T, H * D, dtype=bf, device=device)
    rec("head_gate (head-major -> rows, sigmoid gate per head)",
        _time(lambda: ops.head_gate(og, o_hts, u, QR + KW)),
        nbytes=T * H * D * 4)
    uf = torch.randn(T, s["ff"], device=device).to(bf)
    rec("act_inplace gelu_tanh", _time(lambda: ops.act_inplace(uf, "gelu_tanh")),
        nbytes=T * s["ff"] * 4)
    gu = torch.randn(T, 2 * s["ff"], device=device).to(bf)
    ao = torch.empty(T, s["ff"], dtype=bf, device=device)
    rec("act_and_mul silu (Livasun)", _time(lambda: ops.act_and_mul(ao, gu, "silu")),
        nbytes=T * s["ff"] * 6)

    # ---- recurrent mixers: H heads of 128 x 128, H/2 key heads ----
    N = P = 128
    Gk, taps = max(1, H // 2), 4
    nqk, inner = Gk * N, H * P
    C = 2 * nqk + inner
    for label, nseq, L in (("prefill 8 x 1024", 8, 1024), ("decode 64 x 1", 64, 1)):
        T = nseq * L
        sf, sr = i32([i * L for i in range(nseq)]), i32([L] * nseq)
        ss = i32(list(range(nseq)))
        rs = torch.arange(nseq, dtype=torch.int32, device=device).repeat_interleave(L)
        ps = (torch.arange(L, dtype=torch.int32, device=device) + 5).repeat(nseq)
        u = torch.randn(T, C + inner + 2 * H, device=device).to(bf)
        qkv = torch.empty(T, C, dtype=bf, device=device)
        cw, cb = torch.randn(C, taps, device=device), torch.zeros(C, device=device)
        cst = torch.zeros(nseq + 1, taps - 1, C, dtype=bf, device=device)
        rec(f"causal_conv_silu {label}",
            _time(lambda: ops.causal_conv_silu(qkv, u, 0, cw, cb, cst, sf, sr,
                                               ss, rs, ps)),
            nbytes=T * C * 4)
        y = torch.empty(T, inner, device=device)
        st = torch.zeros(nseq + 1, H, N, P, device=device)
        hv = torch.zeros(H, device=device)
        sec = _time(lambda: ops.delta_scan(y, qkv, 0, nqk, 2 * nqk, u,
                                           C + inner, C + inner + H, H, Gk, N, P,
                                           hv - 1, hv, st, sf, sr, ss, ps,
                                           single=L == 1), 5)
        if L > 1:
            rec(f"delta_scan {label} (fp32 vector ALU, 7 flops per state element)",
                sec, flops=7.0 * T * H * N * P, peak=PEAK_VALU)
        else:
            rec(f"delta_scan {label} (state read + write)", sec,
                nbytes=nseq * H * N * P * 8)
        ul = torch.randn(T, 4 * H * 128, device=device).to(bf)
        stl = torch.zeros(nseq + 1, H, 128, 128, device=device)
        dec = torch.full((H,), 0.99, device=device)
        sec = _time(lambda: ops.state_scan(y, ul, 2 * H * 128, H * 128, 0, None,
                                           0, H, H, 128, 128, True, None, None,
                                           None, dec, stl, sf, sr, ss, ps,
                                           single=L == 1), 5)
        if L > 1:
            rec(f"state_scan lightning {label} (Livasun, 4 flops per state element)",
                sec, flops=4.0 * T * H * 128 * 128, peak=PEAK_VALU)
        else:
            rec(f"state_scan lightning {label} (Livasun, state read + write)",
                sec, nbytes=nseq * H * 128 * 128 * 8)
        g = torch.empty(T, inner, dtype=bf, device=device)
        wi = torch.ones(inner, device=device)
        rec(f"gated_group_norm per head, SiLU gate {label}",
            _time(lambda: ops.gated_group_norm(g, y, u[:, C:C + inner], wi, H,
                                               1e-5, 2)),
            nbytes=T * inner * 8)
    return out


def run(sizes: list[str], device: str, family: str = "vunitar",
        solo: bool = False) -> None:
    """`solo`: only the family's own stack end to end (no comparison stack,
    no per-kernel rates) — the run to put under a profiler."""
    for name in sizes:
        s = SIZES[name]
        if family in ("livasun", "makezen"):
            s = dict(s, layers=4)       # one full cycle of the mixers
        for moe in ((False, True) if family in ("vunitar", "livasun")
                    else (False,)):
            row = {"size": name, **s, "ff_kind": "moe" if moe else "dense"}
            mine = {"vunitar": vunitar_spec, "fusipel": fusipel_spec,
                    "livasun": livasun_spec, "makezen": makezen_spec}[family]
            # Makezen's closest existing model is the other hybrid of
            # attention and recurrent layers; the llama graph for scale
            others = ((("livasun", livasun_spec),) if family == "makezen"
                      else ()) + (("llama_graph", llama_spec),)
            for label, mk in ((family, mine),) + (() if solo else others):
                pre, dec = engine_rates(mk(s, moe), device)
                row[label] = {"prefill_tok_s": round(pre), "decode_tok_s": round(dec)}
            print(json.dumps({"layer_bench": row}), flush=True)
        if torch.cuda.is_available() and not solo:
            rates = {"vunitar": kernel_rates, "fusipel": fusipel_kernel_rates,
                     "livasun": livasun_kernel_rates,
                     "makezen": makezen_kernel_rates}[family]
            for k in rates(s, device):
                print(json.dumps({"kernel_bench": {"size": name, **k}}), flush=True)
