"""Plain-PyTorch fp32 reference implementations of every HIP op.

These are the numerics oracle for the GPU kernel tests (tests compare the
HIP kernels against these at fp32), and the CPU execution path that keeps
the whole serving stack testable without a GPU (the reference
tests everything host-only; we do the same for the control plane + engine
logic and add real kernel tests on-device).
"""
from __future__ import annotations

import torch
import torch.nn.functional as F


def rms_norm(out: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, eps: float) -> None:
    xf = x.float()
    inv = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    out.copy_((xf * inv * weight.float()).to(out.dtype))


def fused_add_rms_norm(x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float) -> None:
    summed = (x.float() + residual.float()).to(residual.dtype)
    residual.copy_(summed)
    sf = summed.float()
    inv = torch.rsqrt(sf.pow(2).mean(-1, keepdim=True) + eps)
    x.copy_((sf * inv * weight.float()).to(x.dtype))


def build_cos_sin_cache(
    head_dim: int,
    rot_dim: int,
    max_pos: int,
    base: float = 10000.0,
    scaling: dict | None = None,
    device: torch.device | str = "cpu",
) -> torch.Tensor:
    """[max_pos, rot_dim] f32: first rot_dim/2 cos then rot_dim/2 sin.

    `scaling` supports llama3-style rope scaling (keys: factor,
    low_freq_factor, high_freq_factor, original_max_position_embeddings).
    """
    half = rot_dim // 2
    inv_freq = 1.0 / (base ** (torch.arange(0, half, dtype=torch.float64) * 2 / rot_dim))
    attention_factor = 1.0
    if scaling and scaling.get("rope_type", scaling.get("type")) == "yarn":
        # YaRN (arXiv 2309.00071; HF _compute_yarn_parameters): blend
        # interpolated and extrapolated inverse frequencies over a linear
        # ramp between the beta_fast/beta_slow correction dims, and scale
        # cos/sin by the attention factor (mscale)
        import math

        factor = scaling.get("factor")
        orig = scaling["original_max_position_embeddings"]
        if factor is None:
            factor = max_pos / orig
        beta_fast = scaling.get("beta_fast") or 32
        beta_slow = scaling.get("beta_slow") or 1
        truncate = scaling.get("truncate", True)

        def get_mscale(scale, m=1):
            return 1.0 if scale <= 1 else 0.1 * m * math.log(scale) + 1.0

        attention_factor = scaling.get("attention_factor")
        if attention_factor is None:
            ms, msd = scaling.get("mscale"), scaling.get("mscale_all_dim")
            if ms and msd:
                attention_factor = float(get_mscale(factor, ms)
                                         / get_mscale(factor, msd))
            else:
                attention_factor = get_mscale(factor)

        def corr_dim(nrot):
            return (rot_dim * math.log(orig / (nrot * 2 * math.pi))
                    / (2 * math.log(base)))

        low, high = corr_dim(beta_fast), corr_dim(beta_slow)
        if truncate:
            low, high = math.floor(low), math.ceil(high)
        low, high = max(low, 0), min(high, rot_dim - 1)
        if low == high:
            high += 0.001
        ramp = ((torch.arange(half, dtype=torch.float64) - low)
                / (high - low)).clamp(0, 1)
        extrap_f = 1 - ramp
        inv_freq = (inv_freq / factor) * (1 - extrap_f) + inv_freq * extrap_f
    elif scaling and scaling.get("rope_type", scaling.get("type")) == "longrope":
        # LongRoPE (Phi-3/4; HF _compute_longrope_parameters): per-dim
        # frequency rescale factors, long vs short chosen by the cache's
        # target length vs the pretraining length — a single static cache
        # per engine (vLLM-style), not HF's per-forward dynamic switch
        import math

        orig = scaling["original_max_position_embeddings"]
        factors = (scaling["long_factor"] if max_pos > orig
                   else scaling["short_factor"])
        inv_freq = inv_freq / torch.tensor(factors, dtype=torch.float64)[:half]
        factor = scaling.get("factor") or (max_pos / orig)
        attention_factor = scaling.get("attention_factor")
        if attention_factor is None:
            attention_factor = (1.0 if factor <= 1.0 else
                                math.sqrt(1 + math.log(factor)
                                          / math.log(orig)))
    elif scaling and scaling.get("rope_type", scaling.get("type")) == "linear":
        # linear position interpolation (Gemma-3 global layers: factor 8)
        inv_freq = inv_freq / scaling["factor"]
    elif scaling and scaling.get("rope_type", scaling.get("type")) == "llama3":
        factor = scaling["factor"]
        lo = scaling["low_freq_factor"]
        hi = scaling["high_freq_factor"]
        orig = scaling["original_max_position_embeddings"]
        wavelen = 2 * torch.pi / inv_freq
        lo_wl = orig / lo
        hi_wl = orig / hi
        new = torch.where(wavelen > lo_wl, inv_freq / factor, inv_freq)
        smooth = (orig / wavelen - lo) / (hi - lo)
        mid = (1 - smooth) * inv_freq / factor + smooth * inv_freq
        is_mid = (wavelen <= lo_wl) & (wavelen >= hi_wl)
        inv_freq = torch.where(is_mid, mid, new)
    t = torch.arange(max_pos, dtype=torch.float64)
    freqs = torch.outer(t, inv_freq)
    cache = torch.cat([freqs.cos(), freqs.sin()], dim=-1).float()
    if attention_factor != 1.0:
        cache = cache * attention_factor
    return cache.to(device)


def rotary_embedding(
    positions: torch.Tensor,
    q: torch.Tensor,
    k: torch.Tensor,
    cos_sin: torch.Tensor,
    head_dim: int,
    rot_dim: int,
    mode: str = "neox",
) -> None:
    """In-place rotation. q: [T, Hq*D] or [T, Hq, D]; same for k.
    mode "neox" rotates the two halves (llama lineage); "pairwise"
    rotates adjacent (even, odd) pairs by one frequency each (GPT-J
    layout; Ernie-4.5 / Hunyuan / MiniMax checkpoints)."""
    half = rot_dim // 2
    cs = cos_sin[positions]  # [T, rot]
    cos = cs[:, :half].unsqueeze(1)  # [T, 1, half]
    sin = cs[:, half:].unsqueeze(1)
    for x in (q, k):
        T = x.shape[0]
        xs = x if x.dim() == 3 else x.view(T, -1, head_dim)
        if mode == "pairwise":
            x1 = xs[..., 0:rot_dim:2].float()
            x2 = xs[..., 1:rot_dim:2].float()
            o1 = x1 * cos - x2 * sin
            o2 = x2 * cos + x1 * sin
            xs[..., 0:rot_dim:2] = o1.to(x.dtype)
            xs[..., 1:rot_dim:2] = o2.to(x.dtype)
            continue
        x1 = xs[..., :half].float()
        x2 = xs[..., half : 2 * half].float()
        o1 = x1 * cos - x2 * sin
        o2 = x2 * cos + x1 * sin
        xs[..., :half] = o1.to(x.dtype)
        xs[..., half : 2 * half] = o2.to(x.dtype)


def silu_and_mul(out: torch.Tensor, x: torch.Tensor) -> None:
    d = out.shape[-1]
    xf = x.float()
    out.copy_((torch.nn.functional.silu(xf[..., :d]) * xf[..., d:]).to(out.dtype))


def reshape_and_cache(
    k: torch.Tensor,
    v: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    slots: torch.Tensor,
) -> None:
    """k/v: [T, Hkv, D]; caches: [B, Hkv, BS, D]; slots: [T] int64 (-1 skip)."""
    bs = k_cache.shape[2]
    mask = slots >= 0
    idx = slots[mask]
    blk = torch.div(idx, bs, rounding_mode="floor")
    off = idx % bs
    k_cache[blk, :, off] = k[mask].to(k_cache.dtype)
    v_cache[blk, :, off] = v[mask].to(v_cache.dtype)


def greedy_sample(out: torch.Tensor, logits: torch.Tensor) -> None:
    out.copy_(logits.float().argmax(dim=-1))


def _sink_softmax(att: torch.Tensor, sinks: torch.Tensor | None):
    """softmax over the kv axis with optional per-head SINK logits joining
    the denominator only (GPT-OSS: probability mass the sinks absorb is
    dropped — no value contribution). att: [Hq, Tq, L]."""
    if sinks is None:
        return torch.softmax(att, dim=-1)
    s = sinks.float().view(-1, 1, 1).expand(att.shape[0], att.shape[1], 1)
    combined = torch.cat([att, s], dim=-1)
    probs = torch.softmax(combined, dim=-1)
    return probs[..., :-1]


def _softcap(att: torch.Tensor, cap: float):
    """Gemma-2 attention logit softcapping: tanh(att/cap)*cap applied to
    the SCALED scores before the mask (HF eager semantics)."""
    if cap:
        return torch.tanh(att / cap) * cap
    return att


def _window_mask(qpos: torch.Tensor, kpos: torch.Tensor, window: int):
    """Causal (+ optional sliding-window) additive mask [Tq, L]."""
    m = torch.where(kpos.unsqueeze(0) <= qpos.unsqueeze(1), 0.0, float("-inf"))
    if window:
        m = torch.where(kpos.unsqueeze(0) > qpos.unsqueeze(1) - window,
                        m, torch.tensor(float("-inf")))
    return m


def paged_attn_decode(
    out: torch.Tensor,
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    block_tables: torch.Tensor,
    seq_lens: torch.Tensor,
    scale: float,
    sinks: torch.Tensor | None = None,
    window: int = 0,
    softcap: float = 0.0,
) -> None:
    """q/out: [N, Hq, D]; caches [B, Hkv, BS, D]."""
    N, Hq, D = q.shape
    Hkv = k_cache.shape[1]
    BS = k_cache.shape[2]
    GQ = Hq // Hkv
    for i in range(N):
        L = int(seq_lens[i])
        nblk = (L + BS - 1) // BS
        blocks = block_tables[i, :nblk].long()
        keys = k_cache[blocks].float().permute(1, 0, 2, 3).reshape(Hkv, -1, D)[:, :L]
        vals = v_cache[blocks].float().permute(1, 0, 2, 3).reshape(Hkv, -1, D)[:, :L]
        keys = keys.repeat_interleave(GQ, dim=0)  # [Hq, L, D]
        vals = vals.repeat_interleave(GQ, dim=0)
        qi = q[i].float().unsqueeze(1)  # [Hq, 1, D]
        att = _softcap((qi @ keys.transpose(1, 2)) * scale, softcap)
        att = att + _window_mask(torch.tensor([L - 1], device=q.device),
                                 torch.arange(L, device=q.device), window)
        att = _sink_softmax(att, sinks)
        out[i] = (att @ vals).squeeze(1).to(out.dtype)


def varlen_prefill_attn(
    out: torch.Tensor,
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    seq_lens: list[int],
    scale: float,
    sinks: torch.Tensor | None = None,
    window: int = 0,
    softcap: float = 0.0,
) -> None:
    """q: [T, Hq, D]; k/v: [T, Hkv, D]; causal within each sequence."""
    Hq = q.shape[1]
    Hkv = k.shape[1]
    GQ = Hq // Hkv
    start = 0
    for L in seq_lens:
        qs = q[start : start + L].float().permute(1, 0, 2)  # [Hq, L, D]
        ks = k[start : start + L].float().permute(1, 0, 2).repeat_interleave(GQ, dim=0)
        vs = v[start : start + L].float().permute(1, 0, 2).repeat_interleave(GQ, dim=0)
        att = _softcap((qs @ ks.transpose(1, 2)) * scale, softcap)
        pos = torch.arange(L, device=q.device)
        att = att + _window_mask(pos, pos, window)
        att = _sink_softmax(att, sinks)
        out[start : start + L] = (att @ vs).permute(1, 0, 2).to(out.dtype)
        start += L


def paged_prefill_attn(
    out: torch.Tensor,
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    block_tables: torch.Tensor,
    seq_starts: list[int],
    seq_hists: list[int],
    seq_news: list[int],
    scale: float,
    sinks: torch.Tensor | None = None,
    window: int = 0,
    softcap: float = 0.0,
) -> None:
    """Prefill-with-history: q/out hold only the NEW (suffix) rows of each
    sequence; K/V for positions [0, hist+new) are gathered from the paged
    pool. Row r of sequence i attends causally to positions [0, hist+r].

    q/out: [T, Hq, D]; caches [B, Hkv, BS, D]; block_tables [nseq, maxb].
    """
    Hq = q.shape[1]
    D = q.shape[2]
    Hkv = k_cache.shape[1]
    BS = k_cache.shape[2]
    GQ = Hq // Hkv
    row = 0
    for i, (hist, new) in enumerate(zip(seq_hists, seq_news)):
        L = hist + new
        nblk = (L + BS - 1) // BS
        blocks = block_tables[i, :nblk].long()
        keys = k_cache[blocks].float().permute(1, 0, 2, 3).reshape(Hkv, -1, D)[:, :L]
        vals = v_cache[blocks].float().permute(1, 0, 2, 3).reshape(Hkv, -1, D)[:, :L]
        keys = keys.repeat_interleave(GQ, dim=0)  # [Hq, L, D]
        vals = vals.repeat_interleave(GQ, dim=0)
        start = seq_starts[i]
        qs = q[start:start + new].float().permute(1, 0, 2)  # [Hq, new, D]
        att = _softcap((qs @ keys.transpose(1, 2)) * scale,
                       softcap)                             # [Hq, new, L]
        pos = torch.arange(L, device=q.device)
        qpos = hist + torch.arange(new, device=q.device)
        att = att + _window_mask(qpos, pos, window)
        att = _sink_softmax(att, sinks)
        out[start:start + new] = (att @ vals).permute(1, 0, 2).to(out.dtype)
        row += new


# --- fp32-residual op family (heterogeneous latent-attention stacks) -------
# The residual stream is fp32; GEMM operands take the model dtype. These are
# the CPU execution path and the numerics oracle of ops/csrc/resid32.hip and
# ops/csrc/latent_attn.hip.

def embed_pair_hash(x: torch.Tensor, h: torch.Tensor | None,
                    tokens: torch.Tensor, prev: torch.Tensor,
                    embed: torch.Tensor, pair_table: torch.Tensor | None,
                    buckets: int, mul_prev: int, mul_cur: int) -> None:
    """x[t] = embed[tok] + pair_table[(prev*mul_prev + tok*mul_cur) %
    buckets] in fp32; prev < 0 marks a sequence's first token, which reads
    row `buckets`. h (optional) receives x rounded to the GEMM dtype."""
    v = embed[tokens].float()
    if pair_table is not None:
        row = (prev * mul_prev + tokens * mul_cur) % buckets
        row = torch.where(prev < 0, torch.full_like(row, buckets), row)
        v = v + pair_table[row].float()
    x.copy_(v)
    if h is not None:
        h.copy_(v.to(h.dtype))


def rms_scale_add(x: torch.Tensor, a: torch.Tensor, weight: torch.Tensor,
                  scale: torch.Tensor | None, eps: float,
                  h: torch.Tensor | None) -> None:
    """x += a / sqrt(mean(a^2) + eps) * weight [* scale], all in fp32 on the
    fp32 stream x; h (optional) receives the new x in the GEMM dtype."""
    af = a.float()
    y = af * torch.rsqrt(af.pow(2).mean(-1, keepdim=True) + eps) * weight.float()
    if scale is not None:
        y = y * scale.float()
    x.add_(y)
    if h is not None:
        h.copy_(x.to(h.dtype))


def rms_norm_f32(out: torch.Tensor, x: torch.Tensor, weight: torch.Tensor,
                 eps: float) -> None:
    xf = x.float()
    out.copy_((xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
               * weight.float()).to(out.dtype))


def latent_norm_store(cache: torch.Tensor, src: torch.Tensor, col0: int,
                      weight: torch.Tensor, slots: torch.Tensor,
                      eps: float) -> None:
    """RMS-normalise src[:, col0:col0+R] in fp32 and write each row into
    its slot of the paged latent pool [nblocks, P, BS, R] (slot < 0: skip):
    plane 0 row-major, plane 1 (if present) the page transposed [R][BS]."""
    nb, P, BS, R = cache.shape
    lat = src[:, col0:col0 + R].float()
    c = (lat * torch.rsqrt(lat.pow(2).mean(-1, keepdim=True) + eps)
         * weight.float()).to(cache.dtype)
    ok = slots >= 0
    blk, off = slots[ok] // BS, slots[ok] % BS
    cache[blk, 0, off] = c[ok]
    if P == 2:
        tr = cache.view(nb, P, BS * R)[:, 1].unflatten(-1, (R, BS))
        tr[blk, :, off] = c[ok]


def latent_attention(ctx: torch.Tensor, q_lat: torch.Tensor,
                     cache: torch.Tensor, block_tables: torch.Tensor,
                     row_seq: torch.Tensor, positions: torch.Tensor,
                     scale: float) -> None:
    """ctx[t, h] = softmax_j<=pos(t)(q_lat[t, h] . c_j * scale) . C for the
    latents c_j of row t's sequence, read through its block table."""
    T, H, R = q_lat.shape
    BS = cache.shape[2]
    for t in range(T):
        L = int(positions[t]) + 1
        bt = block_tables[int(row_seq[t])]
        j = torch.arange(L, device=cache.device)
        C = cache[bt[j // BS].long(), 0, j % BS].float()     # [L, R]
        s = (q_lat[t].float() @ C.T) * scale                 # [H, L]
        p = torch.softmax(s, dim=-1)
        ctx[t] = p @ C


def act_inplace(x: torch.Tensor, mode: str) -> None:
    xf = x.float()
    if mode == "relu2":
        y = torch.relu(xf) ** 2
    elif mode == "gelu":
        y = torch.nn.functional.gelu(xf)
    elif mode == "gelu_tanh":
        y = torch.nn.functional.gelu(xf, approximate="tanh")
    elif mode == "silu":
        y = torch.nn.functional.silu(xf)
    else:
        raise ValueError(mode)
    x.copy_(y.to(x.dtype))


def route_grouped_topk(experts: torch.Tensor, weights: torch.Tensor,
                       logits: torch.Tensor, n_experts: int, groups: int,
                       keep: int, scale: float) -> None:
    """Softmax over logits[:, :n_experts]; experts outside the `keep`
    groups with the largest best-member score are masked; the top-k of the
    rest are written with weight score * scale."""
    T = logits.shape[0]
    top = experts.shape[1]
    s = torch.softmax(logits[:, :n_experts].float(), dim=-1)
    choice = s
    if groups > 1 and keep < groups:
        g = s.view(T, groups, n_experts // groups).amax(-1)
        gi = torch.topk(g, keep, dim=-1)[1]
        gm = torch.zeros_like(g, dtype=torch.bool).scatter_(1, gi, True)
        em = gm.unsqueeze(-1).expand(T, groups, n_experts // groups)
        choice = s.masked_fill(~em.reshape(T, n_experts), -1.0)
    idx = torch.topk(choice, top, dim=-1)[1]
    experts.copy_(idx.to(experts.dtype))
    weights.copy_(s.gather(1, idx) * scale)


def moe_combine(out: torch.Tensor, y: torch.Tensor, inv: torch.Tensor,
                weights: torch.Tensor, shared: torch.Tensor | None,
                gate_logits: torch.Tensor | None, gate_col: int) -> None:
    """out[t] = sum_k weights[t, k] * y[inv[t, k]] (+ sigmoid(gate) *
    shared[t]) in fp32."""
    T, top = inv.shape
    acc = (y[inv.reshape(-1).long()].float().view(T, top, -1)
           * weights.unsqueeze(-1)).sum(1)
    if shared is not None:
        sh = shared.float()
        if gate_logits is not None:
            sh = sh * torch.sigmoid(gate_logits[:, gate_col:gate_col + 1].float())
        acc = acc + sh
    out.copy_(acc)


def softcap_(logits: torch.Tensor, cap: float) -> None:
    logits.copy_(cap * torch.tanh(logits / cap))


# --- paged rotary attention family (ops/csrc/rowmix32.hip, ragged_attn.hip) --
# fp32 stream with pre- and post-norms around every sublayer; rotary keys
# in a paged pool with transposed value pages; scores, softmax and norms in
# fp32 whatever the GEMM dtype.

def embed_rows_f32(x: torch.Tensor, tokens: torch.Tensor,
                   embed: torch.Tensor) -> None:
    x.copy_(embed[tokens].float())


def sandwich_add_norm(x: torch.Tensor, a: torch.Tensor | None,
                      post_w: torch.Tensor | None, mult: float, eps: float,
                      extra: torch.Tensor | None,
                      next_w: torch.Tensor | None,
                      h: torch.Tensor | None, center: bool = False) -> None:
    """x += mult * rmsnorm(a) * post_w  (+ extra), in fp32 on the fp32
    stream x; then h = rmsnorm(x) * next_w in h's dtype. Either half may be
    absent (a is None: no sublayer output; next_w is None: no next norm).
    `center`: both norms take the row's mean off first (weight-only layer
    norms: deviations over the root of their mean square + eps)."""
    def unit(t):
        if center:
            t = t - t.mean(-1, keepdim=True)
        return t * torch.rsqrt(t.pow(2).mean(-1, keepdim=True) + eps)

    if a is not None:
        x.add_(unit(a.float()) * post_w.float() * mult)
    if extra is not None:
        x.add_(extra.float())
    if next_w is not None:
        h.copy_((unit(x) * next_w.float()).to(h.dtype))


def rotary_norm_store(q_out: torch.Tensor, qkv: torch.Tensor, nq: int,
                      nk: int, q_norm_w: torch.Tensor | None,
                      k_norm_w: torch.Tensor | None, inv_freq: torch.Tensor,
                      pos32: torch.Tensor, head_dim: int,
                      k_cache: torch.Tensor, v_cache: torch.Tensor,
                      slots: torch.Tensor, eps: float, tied: bool) -> None:
    """Row kernel between the fused q/k/v projection and attention.
    qkv[:, :nq] are the queries, [nq:nq+nk] the keys, the rest the values
    (tied: none — the raw key projection serves as the value). Optionally a weighted
    RMS norm over the WHOLE q and k rows, then pairwise rotary on the first
    2*len(inv_freq) channels of every head_dim-wide head (angle = pos * f in
    fp32). q goes to q_out [T, nq]; k to its slot of k_cache [nb, G, BS, KW];
    v to its slot of the transposed pages v_cache [nb, G, VW, BS]."""
    T = qkv.shape[0]
    nb, G, BS, KW = k_cache.shape
    VW = v_cache.shape[2]
    q = qkv[:, :nq].float()
    k = qkv[:, nq:nq + nk].float()
    v = k if tied else qkv[:, nq + nk:].float()
    if q_norm_w is not None:
        q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + eps) * q_norm_w.float()
        k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + eps) * k_norm_w.float()
    half = inv_freq.numel()

    def turn(t):
        if half == 0:
            return t
        t = t.reshape(T, -1, head_dim).clone()
        ang = pos32.to(torch.float32)[:, None] * inv_freq.float()[None, :]
        c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
        u, w = t[..., 0:2 * half:2].clone(), t[..., 1:2 * half:2].clone()
        t[..., 0:2 * half:2] = u * c - w * s
        t[..., 1:2 * half:2] = w * c + u * s
        return t.reshape(T, -1)

    q_out.copy_(turn(q).to(q_out.dtype))
    k = turn(k).to(k_cache.dtype).view(T, G, KW)
    v = v.to(v_cache.dtype).view(T, G, VW)
    ok = slots >= 0
    blk, off = slots[ok] // BS, slots[ok] % BS
    k_cache[blk, :, off] = k[ok]
    v_cache[blk, :, :, off] = v[ok]


def paged_attention(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor,
                    v_cache: torch.Tensor, block_tables: torch.Tensor,
                    row_seq: torch.Tensor, positions: torch.Tensor,
                    scale: float, maps: int = 1, window: int = 0,
                    keep_first: int = 0,
                    sinks: torch.Tensor | None = None,
                    slopes: torch.Tensor | None = None,
                    softcap: float = 0.0) -> None:
    """out[t, a] = softmax_j(scale * q[t, a] . k_j) . V over the visible
    keys j of row t's sequence: j <= pos(t), and with window > 0 also
    (pos(t) - j < window or j < keep_first). q: [T, A, D] with A = heads *
    maps score maps (a = head * maps + map); map m of a head reads channels
    [m*D, (m+1)*D) of its kv head's key row and all maps weight the same
    values. sinks (per head, or None) add exp(sink) to the denominator;
    slopes (per head, or None) take slope * (pos(t) - j) off the scaled
    score; softcap > 0 turns a scaled score s into softcap * tanh(s /
    softcap) first."""
    T, A, D = q.shape
    nb, G, BS, KW = k_cache.shape
    VW = v_cache.shape[2]
    H = A // maps
    rep = H // G
    for t in range(T):
        p = int(positions[t])
        bt = block_tables[int(row_seq[t])]
        j = torch.arange(p + 1, device=q.device)
        if window > 0:
            j = j[(p - j < window) | (j < keep_first)]
        blk = bt[j // BS].long()
        K = k_cache[blk, :, j % BS].float()                  # [L, G, KW]
        V = v_cache[blk, :, :, j % BS].float()               # [L, G, VW]
        for a in range(A):
            g = (a // maps) // rep
            m = a % maps
            s = (K[:, g, m * D:(m + 1) * D] @ q[t, a].float()) * scale
            if softcap:
                s = softcap * torch.tanh(s / softcap)
            if slopes is not None:
                s = s - slopes[a // maps].float() * (p - j).float()
            mx = s.max()
            if sinks is not None:
                mx = torch.maximum(mx, sinks[a // maps].float())
            e = torch.exp(s - mx)
            den = e.sum()
            if sinks is not None:
                den = den + torch.exp(sinks[a // maps].float() - mx)
            out[t, a] = ((e / den) @ V[:, g]).to(out.dtype)


def diff_combine(out: torch.Tensor, a: torch.Tensor, lam: torch.Tensor,
                 diff: float, eps: float) -> None:
    """a: [T, H, 2, VW] (two maps' outputs per head, fp32); out[t, h] =
    unit_rms(a1 - lam * a2) * (1 - diff), RMS over the head's VW values."""
    o = a[:, :, 0].float() - lam.float() * a[:, :, 1].float()
    o = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps) * (1.0 - diff)
    out.copy_(o.reshape(out.shape).to(out.dtype))


def act_and_mul(out: torch.Tensor, gu: torch.Tensor, mode: str) -> None:
    """out = act(gu[:, :F]) * gu[:, F:] (the gate in fp32 through the
    activation, the product rounded once)."""
    F_ = out.shape[1]
    g = gu[:, :F_].float().clone()
    act_inplace(g, mode)
    out.copy_((g * gu[:, F_:].float()).to(out.dtype))


# --- layer-norm fp32 stream, windowed attention prep, recurrent mixers ------
# (ops/csrc/lnrows32.hip, state_scan.hip). fp32: the stream, both norms'
# statistics, q/k head norms, the query temperature, step sizes, decays and
# the matrix states, whatever the GEMM dtype.

def embed_rows_scaled(x: torch.Tensor, tokens: torch.Tensor,
                      embed: torch.Tensor, scale: float) -> None:
    x.copy_(embed[tokens].float() * scale)


def add_layer_norm(x: torch.Tensor, a: torch.Tensor | None,
                   w: torch.Tensor | None, b: torch.Tensor | None,
                   eps: float, h: torch.Tensor | None) -> None:
    """x += a (fp32 stream, in place); h = (x - mean) / sqrt(var + eps) * w
    + b in h's dtype, var the mean squared deviation. Either half may be
    left out (a None / w None)."""
    if a is not None:
        x.add_(a.float())
    if w is not None:
        mu = x.mean(-1, keepdim=True)
        d = x - mu
        var = (d * d).mean(-1, keepdim=True)
        h.copy_((d * torch.rsqrt(var + eps) * w.float() + b.float())
                .to(h.dtype))


def head_norm_store(q_out: torch.Tensor, qkv: torch.Tensor, nq: int, nk: int,
                    q_w: torch.Tensor, k_w: torch.Tensor, head_dim: int,
                    temp_coef: float, temp_every: float, pos32: torch.Tensor,
                    v_first: torch.Tensor | None, lam: torch.Tensor | None,
                    k_cache: torch.Tensor, v_cache: torch.Tensor,
                    slots: torch.Tensor, eps: float) -> None:
    """Row kernel between a fused q/k/v projection and windowed attention
    without rotation. Every q and k head is RMS-normed over its head_dim
    channels with one shared weight vector each; q is then multiplied by
    1 + temp_coef * ln(floor((pos + 1) / temp_every) + 1) (temp_every 0:
    off); v blends with v_first, (1 - lam) v + lam v_first, when given.
    q -> q_out [T, nq]; k and v -> their slots of k_cache [nb, G, BS, D]
    and of the transposed pages v_cache [nb, G, VW, BS]."""
    T = qkv.shape[0]
    nb, G, BS, KW = k_cache.shape
    VW = v_cache.shape[2]
    q = qkv[:, :nq].float().reshape(T, -1, head_dim)
    k = qkv[:, nq:nq + nk].float().reshape(T, -1, head_dim)
    v = qkv[:, nq + nk:].float()
    q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + eps) * q_w.float()
    k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + eps) * k_w.float()
    if temp_every > 0:
        p = pos32.to(torch.float32)
        temp = 1.0 + temp_coef * torch.log(
            torch.floor((p + 1.0) / float(temp_every)) + 1.0)
        q = q * temp[:, None, None]
    if v_first is not None:
        lm = lam.float().reshape(())
        v = (1.0 - lm) * v + lm * v_first.float()
    q_out.copy_(q.reshape(T, nq).to(q_out.dtype))
    k = k.to(k_cache.dtype).view(T, G, KW)
    v = v.to(v_cache.dtype).view(T, G, VW)
    ok = slots >= 0
    blk, off = slots[ok] // BS, slots[ok] % BS
    k_cache[blk, :, off] = k[ok]
    v_cache[blk, :, :, off] = v[ok]


def causal_conv_silu(out: torch.Tensor, src: torch.Tensor, col0: int,
                     w: torch.Tensor, b: torch.Tensor,
                     conv_state: torch.Tensor, seq_first: torch.Tensor,
                     seq_rows: torch.Tensor, state_slots: torch.Tensor,
                     pos32: torch.Tensor) -> None:
    """out[t, c] = silu(b[c] + sum_k w[c, k] * in_c(t - (taps - 1 - k)))
    per channel c of src[:, col0:col0 + C], within each sequence; inputs
    before this step's rows come from conv_state[slot] (the sequence's last
    taps - 1 inputs, oldest first), inputs before position 0 are zero. The
    state then takes the last taps - 1 inputs including this step's."""
    C, taps = w.shape
    keep = taps - 1
    for s in range(seq_first.numel()):
        r0, n, slot = int(seq_first[s]), int(seq_rows[s]), int(state_slots[s])
        hist = int(pos32[r0])
        x = src[r0:r0 + n, col0:col0 + C].float()
        if keep:
            old = (conv_state[slot].float() if hist > 0
                   else torch.zeros(keep, C, device=src.device))
            if 0 < hist < keep:
                old = old.clone()
                old[:keep - hist] = 0
            full = torch.cat([old, x], 0)
        else:
            full = x
        acc = b.float()[None, :].repeat(n, 1)
        for k in range(taps):
            acc = acc + full[k:k + n] * w[:, k].float()[None, :]
        out[r0:r0 + n] = (acc * torch.sigmoid(acc)).to(out.dtype)
        if keep:
            conv_state[slot] = full[full.shape[0] - keep:].to(conv_state.dtype)


def state_scan(y: torch.Tensor, src: torch.Tensor, col_x: int, col_b: int,
               col_c: int, dt_src: torch.Tensor | None, col_dt: int,
               heads: int, groups: int, n_state: int, vdim: int,
               act_silu: bool, dt_bias: torch.Tensor | None,
               a_log: torch.Tensor | None, skip: torch.Tensor | None,
               decay: torch.Tensor | None, state: torch.Tensor,
               seq_first: torch.Tensor, seq_rows: torch.Tensor,
               state_slots: torch.Tensor, pos32: torch.Tensor) -> None:
    """Per sequence and head, over this step's rows in order:
        S <- a_t S + b_t k_t v_t^T;  y_t = S^T q_t + skip * v_t
    with S [n_state, vdim] fp32 read from state[slot] (zero when the first
    row sits at position 0) and written back at the end. v = src[:, col_x +
    h * vdim ...], k = src[:, col_b + g * n_state ...], q = src[:, col_c +
    g * n_state ...] with g = h // (heads / groups), all through SiLU when
    act_silu. With dt_src: b_t = dt = softplus(dt_src[t, col_dt + h] +
    dt_bias[h]), a_t = exp(-exp(a_log[h]) * dt); otherwise a_t = decay[h]
    and b_t = 1. y: [T, heads * vdim] fp32."""
    rep = heads // groups

    def act(t):
        t = t.float()
        return t * torch.sigmoid(t) if act_silu else t

    for s in range(seq_first.numel()):
        r0, n, slot = int(seq_first[s]), int(seq_rows[s]), int(state_slots[s])
        hist = int(pos32[r0])
        rows = src[r0:r0 + n]
        v = act(rows[:, col_x:col_x + heads * vdim]).view(n, heads, vdim)
        k = act(rows[:, col_b:col_b + groups * n_state]).view(n, groups, n_state)
        q = act(rows[:, col_c:col_c + groups * n_state]).view(n, groups, n_state)
        k = k.repeat_interleave(rep, 1)
        q = q.repeat_interleave(rep, 1)
        if dt_src is not None:
            raw = (dt_src[r0:r0 + n, col_dt:col_dt + heads].float()
                   + dt_bias.float())
            # softplus without a switch-over: max(x, 0) + log1p(exp(-|x|))
            dt = raw.clamp(min=0) + torch.log1p(torch.exp(-raw.abs()))
            a = torch.exp(-torch.exp(a_log.float()) * dt)
        else:
            dt = torch.ones(n, heads, device=src.device)
            a = decay.float()[None, :].expand(n, heads)
        S = (state[slot].clone() if hist > 0
             else torch.zeros_like(state[slot]))
        for t in range(n):
            S = a[t][:, None, None] * S + (dt[t][:, None] * k[t])[:, :, None] \
                * v[t][:, None, :]
            o = torch.einsum("hnp,hn->hp", S, q[t])
            if skip is not None:
                o = o + skip.float()[:, None] * v[t]
            y[r0 + t] = o.reshape(-1)
        state[slot] = S


def gated_group_norm(out: torch.Tensor, y: torch.Tensor, gate: torch.Tensor,
                     w: torch.Tensor, groups: int, eps: float,
                     gate_first) -> None:
    """gate_first True (1): u = y * silu(gate), then RMS norm of each of
    `groups` equal parts of the row by its own root mean square, times w.
    False (0): RMS norm of y in parts, times w, times sigmoid(gate). 2: the
    same with silu(gate) in place of the sigmoid. y fp32 [T, C]."""
    T, C = y.shape
    mode = int(gate_first)
    g = gate.float()
    u = y * (g * torch.sigmoid(g)) if mode == 1 else y
    u = u.view(T, groups, C // groups)
    u = (u * torch.rsqrt(u.pow(2).mean(-1, keepdim=True) + eps)).view(T, C)
    u = u * w.float()
    if mode == 0:
        u = u * torch.sigmoid(g)
    elif mode == 2:
        u = u * (g * torch.sigmoid(g))
    out.copy_(u.to(out.dtype))


def route_topk(experts: torch.Tensor, weights: torch.Tensor,
               logits: torch.Tensor, correction: torch.Tensor | None,
               n_experts: int, groups: int, keep: int, group_top: int,
               sigmoid: bool, renorm: bool, scale: float) -> None:
    """Scores s = sigmoid(z) or softmax(z) over logits[:, :n_experts];
    choice scores c = s + correction. Experts sit in `groups` equal groups
    of neighbours; a group ranks by the sum of its group_top largest choice
    scores and only the `keep` best groups stay eligible. The top-k by
    choice score are written with weight s (divided by the chosen scores'
    sum + 1e-20 when renorm) * scale."""
    T = logits.shape[0]
    top = experts.shape[1]
    z = logits[:, :n_experts].float()
    s = torch.sigmoid(z) if sigmoid else torch.softmax(z, -1)
    c = s + correction.float() if correction is not None else s
    if groups > 1 and keep < groups:
        per = n_experts // groups
        cg = c.view(T, groups, per)
        gs = torch.topk(cg, min(group_top, per), -1)[0].sum(-1)
        gi = torch.topk(gs, keep, -1)[1]
        gm = torch.zeros_like(gs, dtype=torch.bool).scatter_(1, gi, True)
        c = cg.masked_fill(~gm[:, :, None], -float("inf")).reshape(T, n_experts)
    idx = torch.topk(c, top, -1)[1]
    wt = s.gather(1, idx)
    if renorm:
        wt = wt / (wt.sum(-1, keepdim=True) + 1e-20)
    experts.copy_(idx.to(experts.dtype))
    weights.copy_(wt * scale)


# --- rotary row kernel with per-head norms, gated delta rule, row mixes -----
# (ops/csrc/roperows32.hip, delta_scan.hip)

def head_rope_store(q_out: torch.Tensor | None, src: torch.Tensor, col_q: int,
                    q_heads: int, q_dim: int, q_w: torch.Tensor | None,
                    q_norm_dims: int, q_rot0: int, col_k: int, k_heads: int,
                    k_dim: int, k_w: torch.Tensor | None, k_norm_dims: int,
                    k_rot0: int, col_v: int, inv_freq: torch.Tensor,
                    half_layout: bool, amplitude: float, pos32: torch.Tensor,
                    k_cache: torch.Tensor | None,
                    v_cache: torch.Tensor | None,
                    slots: torch.Tensor | None, eps: float) -> None:
    """Row kernel between a projection and attention. The q side: q_heads
    heads of q_dim channels at src[:, col_q:]; the k side: k_heads heads of
    k_dim channels at src[:, col_k:] (k_heads 0: none). Per head, in fp32:
    the first *_norm_dims channels are RMS-normed over themselves and
    multiplied by *_w (None: no norm); then the 2 * len(inv_freq) channels
    from *_rot0 on turn by pos * f (rot0 < 0: no rotation) — channel i with
    i + half (half_layout) or 2i with 2i+1 — with cos and sin multiplied by
    `amplitude`. q heads go to q_out [T, q_heads * q_dim]; k heads to their
    slot of k_cache [nb, G, BS, k_dim]; values to the transposed pages
    v_cache [nb, G, VW, BS]: src[:, col_v:] (G heads of VW channels), or,
    with col_v < 0, the first VW channels of each finished key head."""
    T = src.shape[0]
    half = inv_freq.numel()
    ang = pos32.to(torch.float32)[:, None] * inv_freq.float()[None, :]
    c = (torch.cos(ang) * amplitude)[:, None, :]
    sn = (torch.sin(ang) * amplitude)[:, None, :]

    def prep(col, heads, dim, w, nd, rot0):
        t = src[:, col:col + heads * dim].float().reshape(T, heads, dim).clone()
        if w is not None:
            part = t[..., :nd]
            t[..., :nd] = part * torch.rsqrt(
                part.pow(2).mean(-1, keepdim=True) + eps) * w.float()
        if rot0 >= 0 and half:
            r = t[..., rot0:rot0 + 2 * half]
            if half_layout:
                u, v = r[..., :half].clone(), r[..., half:].clone()
                r[..., :half] = u * c - v * sn
                r[..., half:] = v * c + u * sn
            else:
                u, v = r[..., 0::2].clone(), r[..., 1::2].clone()
                r[..., 0::2] = u * c - v * sn
                r[..., 1::2] = v * c + u * sn
        return t

    if q_out is not None and q_heads:
        q = prep(col_q, q_heads, q_dim, q_w, q_norm_dims, q_rot0)
        q_out.copy_(q.reshape(T, q_heads * q_dim).to(q_out.dtype))
    if k_heads and k_cache is not None:
        nb, G, BS, KW = k_cache.shape
        VW = v_cache.shape[2]
        k = prep(col_k, k_heads, k_dim, k_w, k_norm_dims, k_rot0)
        k = k.to(k_cache.dtype)
        if col_v >= 0:
            v = src[:, col_v:col_v + G * VW].reshape(T, G, VW).to(v_cache.dtype)
        else:
            v = k[..., :VW]
        ok = slots >= 0
        blk, off = slots[ok] // BS, slots[ok] % BS
        k_cache[blk, :, off] = k[ok]
        v_cache[blk, :, :, off] = v[ok]


def delta_scan(y: torch.Tensor, src: torch.Tensor, col_q: int, col_k: int,
               col_v: int, gate_src: torch.Tensor, col_a: int, col_b: int,
               heads: int, groups: int, n_state: int, vdim: int,
               dt_bias: torch.Tensor, a_log: torch.Tensor,
               state: torch.Tensor, seq_first: torch.Tensor,
               seq_rows: torch.Tensor, state_slots: torch.Tensor,
               pos32: torch.Tensor) -> None:
    """Gated delta rule, per sequence and head over this step's rows in
    order, all in fp32:
        S <- g_t S;  u = beta_t (v_t - S^T k_t);  S <- S + k_t u^T;
        y_t = S^T q_t
    S [n_state, vdim] is read from state[slot] (zero when the first row
    sits at position 0) and written back. q = src[:, col_q + g * n_state
    ...] and k likewise (g = h // (heads / groups)), each scaled to unit
    length, x / sqrt(sum x^2 + 1e-6), q also by n_state^(-1/2); v =
    src[:, col_v + h * vdim ...]; g_t = exp(-exp(a_log[h]) *
    softplus(gate_src[t, col_a + h] + dt_bias[h])), beta_t =
    sigmoid(gate_src[t, col_b + h]). y: [T, heads * vdim] fp32."""
    rep = heads // groups
    for s in range(seq_first.numel()):
        r0, n, slot = int(seq_first[s]), int(seq_rows[s]), int(state_slots[s])
        hist = int(pos32[r0])
        rows = src[r0:r0 + n].float()
        q = rows[:, col_q:col_q + groups * n_state].view(n, groups, n_state)
        k = rows[:, col_k:col_k + groups * n_state].view(n, groups, n_state)
        v = rows[:, col_v:col_v + heads * vdim].view(n, heads, vdim)
        q = q * torch.rsqrt(q.pow(2).sum(-1, keepdim=True) + 1e-6) \
            * float(n_state) ** -0.5
        k = k * torch.rsqrt(k.pow(2).sum(-1, keepdim=True) + 1e-6)
        q = q.repeat_interleave(rep, 1)
        k = k.repeat_interleave(rep, 1)
        gs = gate_src[r0:r0 + n].float()
        raw = gs[:, col_a:col_a + heads] + dt_bias.float()
        dt = raw.clamp(min=0) + torch.log1p(torch.exp(-raw.abs()))
        g = torch.exp(-torch.exp(a_log.float()) * dt)          # [n, H]
        beta = torch.sigmoid(gs[:, col_b:col_b + heads])
        S = (state[slot].clone() if hist > 0
             else torch.zeros_like(state[slot]))
        for t in range(n):
            S = g[t][:, None, None] * S
            u = beta[t][:, None] * (v[t] - torch.einsum("hnp,hn->hp", S, k[t]))
            S = S + k[t][:, :, None] * u[:, None, :]
            y[r0 + t] = torch.einsum("hnp,hn->hp", S, q[t]).reshape(-1)
        state[slot] = S


def dual_rms_mix(out: torch.Tensor, a: torch.Tensor, wa: torch.Tensor,
                 b: torch.Tensor, wb: torch.Tensor, eps: float) -> None:
    """out = (rmsnorm(a) * wa + rmsnorm(b) * wb) / 2 over the rows, fp32
    inside."""
    def unit(t):
        t = t.float()
        return t * torch.rsqrt(t.pow(2).mean(-1, keepdim=True) + eps)

    out.copy_((0.5 * (unit(a) * wa.float() + unit(b) * wb.float()))
              .to(out.dtype))


def head_gate(out: torch.Tensor, o_hts: torch.Tensor, gate_src: torch.Tensor,
              col: int) -> None:
    """out[t, h * VD + c] = o_hts[h, t, c] * sigmoid(gate_src[t, col + h]):
    head-major mixer outputs become rows, each head times its gate."""
    H, T, VD = o_hts.shape
    g = torch.sigmoid(gate_src[:, col:col + H].float())          # [T, H]
    o = o_hts.float().transpose(0, 1) * g[:, :, None]
    out.copy_(o.reshape(T, H * VD).to(out.dtype))
