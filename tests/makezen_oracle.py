"""Plain float64 implementation of the Makezen design, written from its
equations: whole sequences, no cache, no state pool, no batching. One
function per mechanism; the engine is compared with these in
tests/test_makezen.py and tests/test_makezen_gpu.py. Nothing here imports
the product path.

`cfg` is the dict of a checkpoint's config.json, `w` maps checkpoint tensor
names to tensors (any float dtype; converted to float64 on use).
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def f64(t):
    return t.to(F64)


def layer_norm(x, w, eps):
    """(x - mean) / sqrt(var + eps) * w with var the mean squared deviation."""
    mu = x.mean(-1, keepdim=True)
    d = x - mu
    return d / torch.sqrt((d * d).mean(-1, keepdim=True) + eps) * f64(w)


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi)
                                       * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.clamp(z, min=0) + torch.log1p(torch.exp(-z.abs()))


def rot_freqs(rot):
    """(frequencies [dims/2], amplitude) of a rotation entry: base
    frequencies base^(-2i/dims); with a `scaling` entry, slow waves are
    divided by `factor` behind a linear ramp between two cut-off channels,
    and cos / sin grow by 0.1 ln(factor) + 1."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if not sc:
        return torch.tensor(f, dtype=F64), 1.0
    factor, orig = float(sc["factor"]), float(sc["original"])

    def chan(turns):
        return dims * math.log(orig / (2.0 * math.pi * turns)) \
            / (2.0 * math.log(base))

    lo = max(math.floor(chan(float(sc["fast"]))), 0)
    hi = min(math.ceil(chan(float(sc["slow"]))), dims - 1)
    out = []
    for i, fi in enumerate(f):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fi / factor * ramp + fi * (1.0 - ramp))
    return torch.tensor(out, dtype=F64), 0.1 * math.log(factor) + 1.0


def rotate_half_layout(x, pos, freqs, amp):
    """x [..., T, dims]: channel i pairs with i + dims/2; the pair turns by
    pos * f_i. pos [T]."""
    half = freqs.numel()
    # angles in 32-bit as the design computes them
    ang = (pos.to(torch.float32)[:, None] * freqs.to(torch.float32)[None, :])
    c, s = f64(torch.cos(ang)) * amp, f64(torch.sin(ang)) * amp
    u, v = x[..., :half], x[..., half:2 * half]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., 2 * half:]], -1)


def causal_conv_silu(x, w):
    """x [T, C], w [C, taps] (last column = the current token's): zeros
    before the sequence starts, then SiLU."""
    T, C = x.shape
    taps = w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, C, dtype=F64), x], 0)
    acc = torch.zeros(T, C, dtype=F64)
    for k in range(taps):
        acc = acc + pad[k:k + T] * f64(w)[:, k][None, :]
    return silu(acc)


def delta_recurrence(q, k, v, beta, g):
    """One head. q, k [T, N], v [T, P], beta, g [T]. S <- g S; u = beta (v -
    S^T k); S <- S + k u^T; o = S^T q."""
    T, N = q.shape
    P = v.shape[1]
    S = torch.zeros(N, P, dtype=F64)
    out = torch.zeros(T, P, dtype=F64)
    for t in range(T):
        S = g[t] * S
        u = beta[t] * (v[t] - S.t() @ k[t])
        S = S + torch.outer(k[t], u)
        out[t] = S.t() @ q[t]
    return out


def delta_mixer(h, m, w, p, eps):
    """Gated delta rule mixer on h [T, W]; tensors p + name."""
    T = h.shape[0]
    H, G, N, P = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    W = lambda n: f64(w[p + n])
    q = causal_conv_silu(h @ W("q").t(), w[p + "q.conv"]).view(T, G, N)
    k = causal_conv_silu(h @ W("k").t(), w[p + "k.conv"]).view(T, G, N)
    v = causal_conv_silu(h @ W("v").t(), w[p + "v.conv"]).view(T, H, P)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * N ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ W("b").t())                       # [T, H]
    g = torch.exp(-torch.exp(W("A_log"))
                  * softplus(h @ W("a").t() + W("dt_bias")))   # [T, H]
    gate = silu(h @ W("g").t()).view(T, H, P)
    rep = H // G
    outs = []
    for hd in range(H):
        o = delta_recurrence(q[:, hd // rep], k[:, hd // rep], v[:, hd],
                             beta[:, hd], g[:, hd])
        outs.append(rms_unit(o, eps) * W("norm") * gate[:, hd])
    return torch.cat(outs, -1) @ W("o").t()


def visible(i, j, window):
    return j <= i and (window <= 0 or i - j < window)


def attend(q, k, v, scale, window=0, sink=None, softcap=0.0):
    """One head: q, k [T, D], v [T, VD]; optional sliding window, sink logit
    in the denominator, tanh cap on the scaled scores."""
    T = q.shape[0]
    s = (q @ k.t()) * scale
    if softcap:
        s = softcap * torch.tanh(s / softcap)
    i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
    mask = (j <= i) & ((i - j < window) if window > 0 else (j <= i))
    if T <= 8:      # the table above is `visible`, element by element
        assert all(bool(mask[a, b]) == visible(a, b, window)
                   for a in range(T) for b in range(T))
    s = s.masked_fill(~mask, -float("inf"))
    mx = s.max(-1, keepdim=True)[0]
    if sink is not None:
        mx = torch.maximum(mx, sink.reshape(1, 1))
    e = torch.exp(s - mx)
    den = e.sum(-1, keepdim=True)
    if sink is not None:
        den = den + torch.exp(sink - mx)
    return (e / den) @ v


def softmax_mixer(h, m, w, p, eps):
    """Grouped-query softmax attention with biases, per-head q/k RMS norm,
    rotation on the first rot.dims channels, capped scores."""
    T = h.shape[0]
    H, G, D, VD = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    W = lambda n: f64(w[p + n])
    pos = torch.arange(T)
    q = (h @ W("q").t() + W("q.b")).view(T, H, D)
    k = (h @ W("k").t() + W("k.b")).view(T, G, D)
    v = (h @ W("v").t() + W("v.b")).view(T, G, VD)
    q = rms_unit(q, eps) * W("q.norm")
    k = rms_unit(k, eps) * W("k.norm")
    freqs, amp = rot_freqs(m["rot"])
    q = rotate_half_layout(q.transpose(0, 1), pos, freqs, amp)   # [H, T, D]
    k = rotate_half_layout(k.transpose(0, 1), pos, freqs, amp)
    rep = H // G
    outs = [attend(q[hd], k[hd // rep], v[:, hd // rep], float(m["scale"]),
                   softcap=float(m.get("softcap") or 0.0)) for hd in range(H)]
    return torch.cat(outs, -1) @ W("o").t()


def parallel_mixer(h, m, w, p, eps):
    a = softmax_mixer(h, m["left"], w, p + "left.", eps)
    b = delta_mixer(h, m["right"], w, p + "right.", eps)
    return 0.5 * (rms_unit(a, eps) * f64(w[p + "left.out"])
                  + rms_unit(b, eps) * f64(w[p + "right.out"]))


def latent_kv(h, m, w, p, eps):
    """(latent c [T, R], rotated shared key part [T, rot_dim]) of a layer
    that owns a down-projection."""
    T = h.shape[0]
    R = int(m["kv_rank"])
    d = h @ f64(w[p + "dkv"]).t()
    c = rms_unit(d[:, :R], eps) * f64(w[p + "dkv.norm"])
    freqs, amp = rot_freqs(m["rot"])
    kr = rotate_half_layout(d[:, R:], torch.arange(T), freqs, amp)
    return c, kr


def latent_mixer(h, m, w, p, eps, kv):
    """Latent attention; kv = (c, rotated key part) of this layer or of the
    layer it borrows them from."""
    T = h.shape[0]
    H, D, RD, VD = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"])
    W = lambda n: f64(w[p + n])
    c, kr = kv
    cq = rms_unit(h @ W("dq").t(), eps) * W("dq.norm")
    q = (cq @ W("uq").t()).view(T, H, D + RD)
    freqs, amp = rot_freqs(m["rot"])
    qr = rotate_half_layout(q[:, :, D:].transpose(0, 1), torch.arange(T),
                            freqs, amp)                          # [H, T, RD]
    kn = (c @ W("uk").t()).view(T, H, D)
    vv = (c @ W("uv").t()).view(T, H, VD)
    gate = torch.sigmoid(h @ W("g").t())                         # [T, H]
    window = int((m.get("mask") or {}).get("size", 0) or 0)
    outs = []
    for hd in range(H):
        qh = torch.cat([q[:, hd, :D], qr[hd]], -1)
        kh = torch.cat([kn[:, hd], kr], -1)
        o = attend(qh, kh, vv[:, hd], float(m["scale"]), window=window,
                   sink=W("sink")[hd])
        outs.append(o * gate[:, hd:hd + 1])
    return torch.cat(outs, -1) @ W("o").t()


def dense_ff(h, w, p):
    return gelu_tanh(h @ f64(w[p + "up"]).t()) @ f64(w[p + "down"]).t()


def forward(cfg, w, tokens, return_layers=False):
    """Logits [T, vocab] of one sequence (and the stream after every layer)."""
    eps = float(cfg["norm"]["eps"])
    E = f64(w["embed"])
    x = layer_norm(E[torch.as_tensor(tokens)], w["embed.norm"], eps)
    kvs, stream = {}, []
    for i, ent in enumerate(cfg["layers"]):
        p, m = f"l{i}.", ent["mixer"]
        h = layer_norm(x, w[p + "norm1"], eps)
        if ent["type"] == "delta":
            a = delta_mixer(h, m, w, p + "mix.", eps)
        elif ent["type"] == "parallel":
            a = parallel_mixer(h, m, w, p + "mix.", eps)
        elif ent["type"] == "latent_attention":
            src = m.get("kv_from")
            if src is None:
                kvs[i] = latent_kv(h, m, w, p + "mix.", eps)
                src = i
            a = latent_mixer(h, m, w, p + "mix.", eps, kvs[int(src)])
        else:
            raise ValueError(ent["type"])
        x = x + layer_norm(a, w[p + "norm1b"], eps)
        if ent.get("mlp"):
            h = layer_norm(x, w[p + "norm2"], eps)
            x = x + layer_norm(dense_ff(h, w, p + "mlp."), w[p + "norm2b"], eps)
        stream.append(x)
    logits = layer_norm(x, w["final.norm"], eps) @ E.t()
    if return_layers:
        return logits, torch.stack(stream)
    return logits


def greedy(cfg, w, prompt, n):
    """n greedy tokens after `prompt`, recomputing the whole sequence."""
    toks, out = list(prompt), []
    for _ in range(n):
        nxt = int(forward(cfg, w, toks)[-1].argmax())
        out.append(nxt)
        toks.append(nxt)
    return out


# ---- small configurations and random checkpoints for the tests ----------------

def rot_entry(dims, base=100.0, factor=4.0, original=16, fast=4.0, slow=1.0,
              scaling=True):
    r = {"dims": dims, "base": base}
    if scaling:
        r["scaling"] = {"factor": factor, "original": original, "fast": fast,
                        "slow": slow}
    return r


def latent_layer(heads=3, dim=6, rot_dim=4, vdim=5, kv_rank=10, q_rank=7,
                 window=9, scale=0.4, ff=20, kv_from=None, **rot):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim,
         "kv_rank": kv_rank, "q_rank": q_rank, "scale": scale,
         "mask": {"size": window}, "rot": rot_entry(rot_dim, **rot)}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m,
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def delta_mixer_entry(heads=4, kv_heads=2, dim=6, vdim=5, conv=3):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
            "conv": conv}


def delta_layer(ff=0, **kw):
    return {"type": "delta", "mixer": delta_mixer_entry(**kw),
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def softmax_entry(heads=4, kv_heads=2, dim=8, vdim=6, rot_dims=4, scale=0.5,
                  softcap=3.0, **rot):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
            "scale": scale, "softcap": softcap,
            "rot": rot_entry(rot_dims, **rot)}


def parallel_layer(left=None, right=None, ff=16):
    return {"type": "parallel",
            "mixer": {"left": left or softmax_entry(),
                      "right": right or delta_mixer_entry(heads=2, kv_heads=1,
                                                          dim=4, vdim=6,
                                                          conv=4)},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def make_config(width=24, vocab=50, layers=None, eps=1e-5):
    if layers is None:
        layers = [latent_layer(), delta_layer(), parallel_layer(),
                  latent_layer(window=5, kv_from=0, ff=12)]
    return {"architecture": "Makezen", "vocab": vocab, "width": width,
            "norm": {"eps": eps}, "layers": layers}


def make_weights(cfg, seed=0):
    """Random bf16 checkpoint of a configuration (norm weights, sinks,
    biases and decay constants spread enough to matter)."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]
    w = {}

    def lin(name, out, inp, gain=1.0):
        w[name] = (torch.randn(out, inp, generator=g) * gain * inp ** -0.5
                   ).to(torch.bfloat16)

    def vec(name, n, base=1.0, std=0.2):
        w[name] = (base + std * torch.randn(n, generator=g)).to(torch.bfloat16)

    def delta(p, m):
        H, G, N, P = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        for nm, rows in (("q", G * N), ("k", G * N), ("v", H * P)):
            lin(p + nm, rows, W, 1.5)
            w[p + nm + ".conv"] = (torch.randn(rows, m["conv"], generator=g)
                                   * 0.6).to(torch.bfloat16)
        lin(p + "b", H, W, 2.0)
        lin(p + "a", H, W, 2.0)
        lin(p + "g", H * P, W, 1.5)
        vec(p + "A_log", H, -1.0, 1.0)
        vec(p + "dt_bias", H, 0.0, 1.0)
        vec(p + "norm", P)
        lin(p + "o", W, H * P)

    def softmax(p, m):
        H, G, D, VD = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        for nm, rows in (("q", H * D), ("k", G * D), ("v", G * VD)):
            lin(p + nm, rows, W, 1.5)
            vec(p + nm + ".b", rows, 0.0, 0.3)
        vec(p + "q.norm", D, 1.0, 0.3)
        vec(p + "k.norm", D, 1.0, 0.3)
        lin(p + "o", W, H * VD)

    w["embed"] = torch.randn(cfg["vocab"], W, generator=g).to(torch.bfloat16)
    vec("embed.norm", W)
    vec("final.norm", W)
    for i, ent in enumerate(cfg["layers"]):
        p, m = f"l{i}.", ent["mixer"]
        vec(p + "norm1", W)
        vec(p + "norm1b", W)
        if ent["type"] == "delta":
            delta(p + "mix.", m)
        elif ent["type"] == "parallel":
            softmax(p + "mix.left.", m["left"])
            delta(p + "mix.right.", m["right"])
            vec(p + "mix.left.out", W)
            vec(p + "mix.right.out", W)
        else:
            H, D, RD, VD = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
            R, QR = m["kv_rank"], m["q_rank"]
            lin(p + "mix.dq", QR, W)
            vec(p + "mix.dq.norm", QR)
            lin(p + "mix.uq", H * (D + RD), QR, 1.5)
            if m.get("kv_from") is None:
                lin(p + "mix.dkv", R + RD, W, 1.5)
                vec(p + "mix.dkv.norm", R)
            lin(p + "mix.uk", H * D, R, 1.5)
            lin(p + "mix.uv", H * VD, R, 1.5)
            vec(p + "mix.sink", H, 0.0, 1.0)
            lin(p + "mix.g", H, W, 2.0)
            lin(p + "mix.o", W, H * VD)
        if ent.get("mlp"):
            vec(p + "norm2", W)
            vec(p + "norm2b", W)
            lin(p + "mlp.up", ent["mlp"]["ff"], W)
            lin(p + "mlp.down", W, ent["mlp"]["ff"])
    return w


def save_model(path, cfg, weights):
    import json
    from pathlib import Path

    from safetensors.torch import save_file

    path = Path(path)
    path.mkdir(parents=True, exist_ok=True)
    (path / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in weights.items()},
              str(path / "model.safetensors"))
    return str(path)
