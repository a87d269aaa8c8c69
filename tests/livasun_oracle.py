"""Plain float64 oracle of the Livasun design, written from its equations:
one function per mechanism, whole sequences at once, no cache, no state
pool, no batching, nothing shared with gpustack_amd. Also the helpers that
make small random configurations and checkpoints for the tests.

Notation: x stream [T, W]; h a sublayer's input; for attention H query
heads, G kv heads, d score size, dv value size; for the recurrent mixers H
heads, N state rows, P value channels per head. Linear weights are
[out, in].
"""
import json
import math
from pathlib import Path

import torch

F64 = torch.float64
BF = torch.bfloat16


# ---- small pieces -------------------------------------------------------------

def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def unit_rms(x, eps, w=None):
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if w is None else y * w


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.clamp(z, min=0) + torch.log1p(torch.exp(-z.abs()))


def relu2(z):
    return torch.relu(z) ** 2


# ---- attention ------------------------------------------------------------------

def query_temperature(pos, qt):
    """1 + coef * ln(floor((p + 1) / every) + 1) per position; 1 without."""
    if not qt:
        return torch.ones_like(pos, dtype=F64)
    steps = torch.div(pos + 1, qt["every"], rounding_mode="floor")
    return 1.0 + qt["coef"] * torch.log(steps.to(F64) + 1.0)


def head_slopes(H):
    return torch.tensor([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)],
                        dtype=F64)


def visible(T, size=0):
    """[T, T] bool: row i sees column j when 0 <= i - j (< size, if any)."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    ok = j <= i
    if size:
        ok = ok & (i - j < size)
    return ok


def mixer_attention(W, p, m, h, eps, carry):
    """Softmax attention without rotation. `carry` passes the first
    value-mixing layer's values on to the later ones."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = unit_rms((h @ W[p + "q"].T).view(T, H, d), eps, W[p + "q.norm"])
    k = unit_rms((h @ W[p + "k"].T).view(T, G, d), eps, W[p + "k.norm"])
    v = (h @ W[p + "v"].T).view(T, G, dv)
    pos = torch.arange(T)
    q = q * query_temperature(pos, m.get("q_temp"))[:, None, None]
    if m.get("v_mix"):
        if "v_first" in carry:
            lam = W[p + "vmix"]
            v = (1.0 - lam) * v + lam * carry["v_first"]
        else:
            carry["v_first"] = v
    dist = (pos[:, None] - pos[None, :]).to(F64)
    ok = visible(T, (m.get("mask") or {}).get("size", 0))
    slopes = head_slopes(H)
    out = torch.zeros(T, H, dv, dtype=F64)
    for a in range(H):
        g = a // (H // G)
        s = (q[:, a] @ k[:, g].T) * m["scale"] - slopes[a] * dist
        s = s.masked_fill(~ok, -math.inf)
        out[:, a] = torch.softmax(s, -1) @ v[:, g]
    return out.reshape(T, H * dv) @ W[p + "o"].T


# ---- recurrent mixers -------------------------------------------------------------

def causal_conv(x, w, b):
    """x [T, C], w [C, taps] (last column weighs the current row), zeros
    before the first row."""
    T, taps = x.shape[0], w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, x.shape[1], dtype=F64), x])
    y = b[None, :].repeat(T, 1)
    for k in range(taps):
        y = y + pad[k:k + T] * w[:, k]
    return y


def matrix_recurrence(a, b, k, v, q, skip=None):
    """S_t = a_t S_(t-1) + b_t k_t v_t^T, y_t = S_t^T q_t (+ skip v_t) for
    one head: a, b [T]; k, q [T, N]; v [T, P]."""
    T, N, P = k.shape[0], k.shape[1], v.shape[1]
    S = torch.zeros(N, P, dtype=F64)
    y = torch.zeros(T, P, dtype=F64)
    for t in range(T):
        S = a[t] * S + b[t] * torch.outer(k[t], v[t])
        y[t] = S.T @ q[t]
        if skip is not None:
            y[t] = y[t] + skip * v[t]
    return y


def mixer_mamba2(W, p, m, h, eps, carry=None):
    T = h.shape[0]
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner, gn = H * P, G * N
    u = h @ W[p + "in"].T
    z, xbc, dt = u[:, :inner], u[:, inner:2 * inner + 2 * gn], u[:, 2 * inner + 2 * gn:]
    xbc = silu(causal_conv(xbc, W[p + "conv"], W[p + "conv.b"]))
    x = xbc[:, :inner].view(T, H, P)
    B = xbc[:, inner:inner + gn].view(T, G, N)
    C = xbc[:, inner + gn:].view(T, G, N)
    dt = softplus(dt + W[p + "dt_bias"])
    decay = torch.exp(-torch.exp(W[p + "A_log"]) * dt)
    y = torch.zeros(T, H, P, dtype=F64)
    for a in range(H):
        g = a // (H // G)
        y[:, a] = matrix_recurrence(decay[:, a], dt[:, a], B[:, g], x[:, a],
                                    C[:, g], W[p + "D"][a])
    y = y.reshape(T, inner) * silu(z)
    parts = m["norm_groups"]
    y = unit_rms(y.view(T, parts, inner // parts), eps).reshape(T, inner)
    return (y * W[p + "norm"]) @ W[p + "o"].T


def mixer_lightning(W, p, m, h, eps, carry=None):
    T = h.shape[0]
    H, N, P = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ W[p + "q"].T).view(T, H, N)
    k = silu(h @ W[p + "k"].T).view(T, H, N)
    v = silu(h @ W[p + "v"].T).view(T, H, P)
    ones = torch.ones(T, dtype=F64)
    y = torch.zeros(T, H, P, dtype=F64)
    for a in range(H):
        y[:, a] = matrix_recurrence(ones * m["decay"][a], ones, k[:, a],
                                    v[:, a], q[:, a])
    y = unit_rms(y.reshape(T, H * P), eps, W[p + "norm"])
    return (y * torch.sigmoid(h @ W[p + "g"].T)) @ W[p + "o"].T


# ---- feed-forward -------------------------------------------------------------------

def gated_ff(W, p, h):
    return (silu(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def route(z, correction, r):
    """Chosen experts [T, top] and their weights for router logits z."""
    E, top = r["experts"], r["top"]
    s = torch.sigmoid(z)
    c = s + correction
    gr = r.get("groups")
    if gr and gr["count"] > 1:
        per = E // gr["count"]
        cg = c.view(-1, gr["count"], per)
        rank = cg.topk(min(2, per), -1).values.sum(-1)
        kept = rank.topk(gr["keep"], -1).indices
        drop = torch.ones_like(rank, dtype=torch.bool).scatter_(1, kept, False)
        c = cg.masked_fill(drop[:, :, None], -math.inf).reshape(-1, E)
    idx = c.topk(top, -1).indices
    w = s.gather(1, idx)
    return idx, w / (w.sum(-1, keepdim=True) + 1e-20) * r["scale"]


def expert(W, p, h):
    return relu2(h @ W[p + "up"].T) @ W[p + "down"].T


def routed_ff(W, p, f, h):
    idx, wt = route(h @ W[p + "router"].T, W[p + "correction"], f["router"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(idx.shape[1]):
            out[t] += wt[t, j] * expert(W, f"{p}e{int(idx[t, j])}.", h[t])
    if f.get("shared"):
        out = out + expert(W, p + "shared.", h)
    return out


# ---- the model ------------------------------------------------------------------------

MIXERS = {"attention": mixer_attention, "mamba2": mixer_mamba2,
          "lightning": mixer_lightning}


def forward(cfg, weights, tokens, streams=None):
    """Logits [T, vocab] of one sequence; `streams` collects the stream
    after every layer."""
    W = {k: v.to(F64) for k, v in weights.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(tokens)] * cfg["embedding"]["scale"]
    carry = {}
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = layer_norm(x, W[p + "norm1"], W[p + "norm1.b"], eps)
        x = x + MIXERS[L["type"]](W, p + "mix.", L["mixer"], h, eps, carry)
        f = L.get("mlp")
        if f:
            h = layer_norm(x, W[p + "norm2"], W[p + "norm2.b"], eps)
            x = x + (gated_ff(W, p + "mlp.", h) if f["kind"] == "dense"
                     else routed_ff(W, p + "mlp.", f, h))
        if streams is not None:
            streams.append(x.clone())
    return layer_norm(x, W["final.norm"], W["final.norm.b"], eps) @ W["head"].T


def greedy(cfg, weights, prompt, n):
    toks = list(prompt)
    out = []
    for _ in range(n):
        out.append(int(forward(cfg, weights, toks)[-1].argmax()))
        toks.append(out[-1])
    return out


# ---- small configurations and checkpoints -------------------------------------------------

def attn_layer(heads=4, kv_heads=2, dim=8, vdim=6, window=9, temp=(0.4, 5),
               v_mix=True, scale=0.6, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
         "scale": scale, "v_mix": v_mix}
    if window:
        m["mask"] = {"size": window}
    if temp:
        m["q_temp"] = {"coef": temp[0], "every": temp[1]}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def mamba_layer(heads=4, groups=2, state=6, vdim=5, conv=3, norm_groups=2,
                mlp=None):
    return {"type": "mamba2", "mlp": mlp,
            "mixer": {"heads": heads, "groups": groups, "state": state,
                      "vdim": vdim, "conv": conv, "norm_groups": norm_groups}}


def lightning_layer(heads=3, dim=7, vdim=4, decay=(0.7, 0.93, 0.999), mlp=None):
    return {"type": "lightning", "mlp": mlp,
            "mixer": {"heads": heads, "dim": dim, "vdim": vdim,
                      "decay": list(decay)}}


def dense(ff=20):
    return {"kind": "dense", "ff": ff}


def moe(experts=6, count=3, keep=2, top=2, ff=10, shared=12, scale=1.5):
    r = {"experts": experts, "top": top, "scale": scale}
    if count:
        r["groups"] = {"count": count, "keep": keep}
    f = {"kind": "moe", "expert": {"ff": ff}, "router": r}
    if shared:
        f["shared"] = {"ff": shared}
    return f


def make_config(width=24, vocab=53, layers=None, embed_scale=3.0, eps=1e-6):
    if layers is None:
        layers = [attn_layer(mlp=dense()),
                  mamba_layer(mlp=moe()),
                  attn_layer(heads=2, dim=10, window=5, temp=None),
                  lightning_layer(mlp=dense(16)),
                  attn_layer(heads=6, kv_heads=2, dim=4, window=0,
                             temp=(0.2, 3), mlp=moe(experts=4, count=0, top=1,
                                                    shared=0))]
    return {"architecture": "Livasun", "vocab": vocab, "width": width,
            "embedding": {"scale": embed_scale}, "norm": {"eps": eps},
            "layers": layers}


def make_weights(cfg, seed=0):
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def lin(o, i, gain=1.0):
        return (torch.randn(o, i, generator=g) * gain / math.sqrt(i)).to(BF)

    def vec(n, base=1.0, spread=0.2):
        return (base + spread * torch.randn(n, generator=g)).to(BF)

    w = {"embed": torch.randn(cfg["vocab"], W, generator=g).to(BF),
         "final.norm": vec(W), "final.norm.b": vec(W, 0.0, 0.3),
         "head": lin(cfg["vocab"], W, 2.0)}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        w[p + "norm1"], w[p + "norm1.b"] = vec(W), vec(W, 0.0, 0.3)
        if L["type"] == "attention":
            H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            w[p + "mix.q"], w[p + "mix.k"] = lin(H * d, W, 2.0), lin(G * d, W, 2.0)
            w[p + "mix.v"], w[p + "mix.o"] = lin(G * dv, W), lin(W, H * dv)
            w[p + "mix.q.norm"], w[p + "mix.k.norm"] = vec(d, 1.5), vec(d, 1.5)
            w[p + "mix.vmix"] = (0.25 + 0.5 * torch.rand((), generator=g)).to(BF)
        elif L["type"] == "mamba2":
            H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
            ch = H * P + 2 * G * N
            w[p + "mix.in"] = lin(2 * H * P + 2 * G * N + H, W, 1.5)
            w[p + "mix.conv"] = lin(ch, m["conv"], 1.5)
            w[p + "mix.conv.b"] = vec(ch, 0.0, 0.3)
            w[p + "mix.dt_bias"] = vec(H, -0.5, 0.7)
            w[p + "mix.A_log"] = vec(H, -1.0, 0.8)
            w[p + "mix.D"] = vec(H, 1.0, 0.5)
            w[p + "mix.norm"] = vec(H * P)
            w[p + "mix.o"] = lin(W, H * P)
        else:
            H, N, P = m["heads"], m["dim"], m["vdim"]
            w[p + "mix.q"], w[p + "mix.k"] = lin(H * N, W, 1.5), lin(H * N, W, 1.5)
            w[p + "mix.v"], w[p + "mix.g"] = lin(H * P, W), lin(H * P, W, 2.0)
            w[p + "mix.norm"] = vec(H * P)
            w[p + "mix.o"] = lin(W, H * P)
        f = L.get("mlp")
        if not f:
            continue
        w[p + "norm2"], w[p + "norm2.b"] = vec(W), vec(W, 0.0, 0.3)
        if f["kind"] == "dense":
            w[p + "mlp.gate"], w[p + "mlp.up"] = lin(f["ff"], W, 1.5), lin(f["ff"], W)
            w[p + "mlp.down"] = lin(W, f["ff"])
            continue
        E = f["router"]["experts"]
        w[p + "mlp.router"] = lin(E, W, 3.0)
        w[p + "mlp.correction"] = vec(E, -0.3, 0.5)    # choice scores go negative
        for e in range(E):
            w[p + f"mlp.e{e}.up"] = lin(f["expert"]["ff"], W, 1.5)
            w[p + f"mlp.e{e}.down"] = lin(W, f["expert"]["ff"])
        if f.get("shared"):
            w[p + "mlp.shared.up"] = lin(f["shared"]["ff"], W, 1.5)
            w[p + "mlp.shared.down"] = lin(W, f["shared"]["ff"])
    return w


def save_model(path, cfg, weights):
    from safetensors.torch import save_file

    path = Path(path)
    path.mkdir(parents=True, exist_ok=True)
    (path / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in weights.items()},
              str(path / "model.safetensors"))
    return str(path)
