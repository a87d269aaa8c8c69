"""Makezen through the engine (scheduler, paged pools, state slots, model
runner, ops) against the plain float64 oracle in tests/makezen_oracle.py.

Every test writes its own small checkpoint (config.json + safetensors with
random bf16 weights) and loads it like a served model. The engine runs in
fp32 here so that a structural fault — a key one position off at the
window's edge, a lost sink, a state that is lost or carried into the wrong
request, a convolution input missing at a portion's start, a borrowed cache
read from the wrong layer — shows far above the rounding floor; one test
repeats the comparison in bf16. Windows are a few tokens wide, so every key
inside one carries weight.
"""
import io
import json
import math
import sys
from pathlib import Path

import pytest
import torch

sys.path.insert(0, str(Path(__file__).resolve().parent))
import makezen_oracle as oracle  # noqa: E402
from test_fusipel import err, make_engine, replay, tokens_for  # noqa: E402

from gpustack_amd.engine import SamplingParams  # noqa: E402
from gpustack_amd.engine.config import (LatentMixerSpec, ModelSpec,  # noqa: E402
                                        ParallelMixerSpec, RotarySpec,
                                        ScanMixerSpec)

TOL = 2e-4      # fp32 engine against the float64 oracle


@pytest.fixture(scope="module")
def model(tmp_path_factory):
    cfg = oracle.make_config()
    w = oracle.make_weights(cfg, seed=3)
    d = oracle.save_model(tmp_path_factory.mktemp("makezen"), cfg, w)
    return cfg, w, d


def _one(tmp_path, layers, n=41, seed=0, width=24, steps=None, dtype="float32"):
    """A model of the given layers: whole prompt (or `steps`) vs oracle."""
    cfg = oracle.make_config(width=width, layers=layers)
    w = oracle.make_weights(cfg, seed=seed)
    d = oracle.save_model(tmp_path, cfg, w)
    toks = tokens_for(cfg, n, seed + 11)
    got = replay(make_engine(d, dtype=dtype), {"a": toks},
                 steps or [[("a", n)]])["a"]
    return err(got, oracle.forward(cfg, w, toks))


# ---- configuration ------------------------------------------------------------

def test_config_is_read_from_the_file(model):
    cfg, _, d = model
    spec = ModelSpec.from_dir(d)
    assert spec.architecture == "Makezen" and spec.fp32_residual
    assert spec.vocab_size == cfg["vocab"] and spec.hidden_size == cfg["width"]
    assert spec.rms_norm_eps == cfg["norm"]["eps"]
    assert spec.tie_word_embeddings and spec.embed_norm
    kinds = [type(ls.mixer) for ls in spec.layers]
    assert kinds == [LatentMixerSpec, ScanMixerSpec, ParallelMixerSpec,
                     LatentMixerSpec]
    a0, c0 = spec.layers[0].mixer, cfg["layers"][0]["mixer"]
    assert (a0.heads, a0.qk_dim, a0.rot_dim, a0.v_dim, a0.kv_rank, a0.q_rank,
            a0.window, a0.scale, a0.kv_from) == (
        c0["heads"], c0["dim"], c0["rot_dim"], c0["vdim"], c0["kv_rank"],
        c0["q_rank"], c0["mask"]["size"], c0["scale"], -1)
    assert a0.sink and a0.out_gate and a0.rot.layout == "half"
    sc = c0["rot"]["scaling"]
    assert a0.rot.ramp == (sc["factor"], sc["original"], sc["fast"], sc["slow"])
    assert spec.layers[3].mixer.kv_from == 0
    assert spec.layers[3].mixer.window == cfg["layers"][3]["mixer"]["mask"]["size"]
    m1, c1 = spec.layers[1].mixer, cfg["layers"][1]["mixer"]
    assert (m1.kind, m1.heads, m1.groups, m1.state, m1.vdim, m1.conv) == (
        "delta", c1["heads"], c1["kv_heads"], c1["dim"], c1["vdim"], c1["conv"])
    m2, c2 = spec.layers[2].mixer, cfg["layers"][2]["mixer"]
    assert (m2.left.heads, m2.left.kv_heads, m2.left.qk_dim, m2.left.v_dim,
            m2.left.softcap, m2.left.rot.dims, m2.left.bias,
            m2.left.head_norm) == (
        c2["left"]["heads"], c2["left"]["kv_heads"], c2["left"]["dim"],
        c2["left"]["vdim"], c2["left"]["softcap"], c2["left"]["rot"]["dims"],
        True, True)
    assert m2.right.kind == "delta" and m2.right.conv == c2["right"]["conv"]
    assert spec.layers[1].mlp is None
    assert spec.layers[0].mlp.act == "gelu_tanh" and not spec.layers[0].mlp.gated
    # latent runs own a key row of latent + key part and the latent again as
    # value; the borrowing run owns nothing; the parallel run owns both kinds
    pools = spec.kv_pool_widths()
    assert pools[0] == ("kv", 1, c0["kv_rank"] + c0["rot_dim"], c0["kv_rank"])
    assert pools[1] == ("state",) and pools[3] == ("shared", 0)
    assert pools[2] == ("kv", c2["left"]["kv_heads"], c2["left"]["dim"],
                        c2["left"]["vdim"])
    shapes = spec.state_pool_shapes()
    assert shapes[0] is None and shapes[3] is None
    assert shapes[1] == (c1["heads"], c1["dim"], c1["vdim"], c1["conv"] - 1,
                         c1["heads"] * c1["vdim"] + 2 * c1["kv_heads"] * c1["dim"])
    r = c2["right"]
    assert shapes[2] == (r["heads"], r["dim"], r["vdim"], r["conv"] - 1,
                         r["heads"] * r["vdim"] + 2 * r["kv_heads"] * r["dim"])


def test_bad_configurations_are_refused():
    bad = [
        [oracle.latent_layer(), oracle.latent_layer(kv_from=0, kv_rank=8)],
        [oracle.latent_layer(kv_from=0)],                  # no earlier layer
        [oracle.delta_layer(), oracle.latent_layer(kv_from=0)],
        [oracle.latent_layer(), oracle.latent_layer(kv_from=0),
         oracle.latent_layer(kv_from=1)],                  # borrowed twice over
        [oracle.delta_layer(heads=3, kv_heads=2)],
        [oracle.parallel_layer(left=oracle.softmax_entry(heads=3, kv_heads=2))],
        [oracle.parallel_layer(left=oracle.softmax_entry(rot_dims=10, dim=8))],
    ]
    for layers in bad:
        with pytest.raises(ValueError):
            ModelSpec.from_hf_config(oracle.make_config(layers=layers))
    cfg = oracle.make_config(layers=[oracle.delta_layer()])
    cfg["layers"][0]["type"] = "other"
    with pytest.raises(NotImplementedError):
        ModelSpec.from_hf_config(cfg)


def test_state_models_refuse_prefix_caching_and_speculation(model):
    _, _, d = model
    with pytest.raises(ValueError):
        make_engine(d, enable_prefix_caching=True)
    with pytest.raises(ValueError):
        make_engine(d, speculative={"method": "ngram", "num_draft_tokens": 2})


# ---- each mechanism alone -----------------------------------------------------

@pytest.mark.parametrize("rot", [
    oracle.rot_entry(16, base=50.0, factor=8.0, original=40, fast=6.0, slow=1.0),
    oracle.rot_entry(32, base=1e4, factor=4.0, original=4096, fast=32.0, slow=1.0),
    oracle.rot_entry(8, base=10.0, factor=2.0, original=8, fast=1.0, slow=1.0),
    oracle.rot_entry(6, base=1000.0, factor=16.0, original=3, fast=2.0, slow=0.5),
    oracle.rot_entry(12, scaling=False),
])
def test_rotary_frequencies(rot):
    sc = rot.get("scaling")
    spec = RotarySpec(dims=rot["dims"], base=rot["base"], layout="half",
                      ramp=(sc["factor"], sc["original"], sc["fast"],
                            sc["slow"]) if sc else None)
    f, amp = oracle.rot_freqs(rot)
    assert torch.allclose(torch.tensor(spec.inv_freq(), dtype=torch.float64),
                          f, rtol=1e-12, atol=0)
    assert spec.amplitude == pytest.approx(amp, rel=1e-12)
    if sc:
        assert amp == pytest.approx(0.1 * math.log(sc["factor"]) + 1.0)


@pytest.mark.parametrize("half_layout", [True, False])
def test_head_norm_rotation_and_latent_rows_alone(half_layout):
    """ops.head_rope_store against the oracle's pieces: heads normed over
    all their channels and turned on the first ones; a latent row normed
    over its first channels, turned on its last ones and kept as key and
    value; queries turned on their last channels without a norm."""
    from gpustack_amd import ops

    eps, BS = 1e-5, 4
    rot = oracle.rot_entry(6, base=30.0, factor=3.0, original=20, fast=3.0)
    freqs, amp = oracle.rot_freqs(rot)
    invf = freqs.float()
    pos = torch.tensor([0, 1, 5, 6, 7, 40, 1000], dtype=torch.int32)
    T = pos.numel()
    g = torch.Generator().manual_seed(4)

    def turned(x, first):
        """x [T, heads, d]: rotation of channels first .. first + 5."""
        part = x[..., first:first + 6].transpose(0, 1)
        if half_layout:
            r = oracle.rotate_half_layout(part, pos.long(), freqs, amp)
        else:       # pairs (2i, 2i + 1): the same rotation on re-ordered channels
            order = [0, 2, 4, 1, 3, 5]
            back = [0, 3, 1, 4, 2, 5]
            r = oracle.rotate_half_layout(part[..., order], pos.long(), freqs,
                                          amp)[..., back]
        out = x.clone()
        out[..., first:first + 6] = r.transpose(0, 1)
        return out

    # softmax heads: H q heads and G k heads of d channels, values beside
    H, G, d, dv = 3, 2, 10, 7
    src = torch.randn(T, (H + G) * d + G * dv + 3, generator=g)
    qw, kw = torch.rand(d, generator=g) + 0.5, torch.rand(d, generator=g) + 0.5
    q = torch.zeros(T, H * d)
    kc, vc = torch.zeros(3, G, BS, d), torch.zeros(3, G, dv, BS)
    slots = torch.tensor([8, 9, 1, 2, 3, 4, 11])
    ops.head_rope_store(q, src, 0, H, d, qw, d, 0, H * d, G, d, kw, d, 0,
                        (H + G) * d, invf, half_layout, amp, pos, kc, vc,
                        slots, eps)
    x = src.double()
    rq = turned(oracle.rms_unit(x[:, :H * d].view(T, H, d), eps) * qw.double(), 0)
    rk = turned(oracle.rms_unit(x[:, H * d:(H + G) * d].view(T, G, d), eps)
                * kw.double(), 0)
    rv = x[:, (H + G) * d:(H + G) * d + G * dv].view(T, G, dv)
    assert (q.double() - rq.reshape(T, -1)).abs().max() < 1e-5
    assert (kc[slots // BS, :, slots % BS].double() - rk).abs().max() < 1e-5
    assert (vc[slots // BS, :, :, slots % BS].double() - rv).abs().max() < 1e-6
    # a latent row: query latent normed whole; key row = normed latent |
    # turned key part; the value pages repeat the latent
    QR, R = 5, 9
    src = torch.randn(T, QR + R + 6 + 2, generator=g)
    qn, kn = torch.rand(QR, generator=g) + 0.5, torch.rand(R, generator=g) + 0.5
    cq = torch.zeros(T, QR)
    kc, vc = torch.zeros(3, 1, BS, R + 6), torch.zeros(3, 1, R, BS)
    ops.head_rope_store(cq, src, 0, 1, QR, qn, QR, -1, QR, 1, R + 6, kn, R, R,
                        -1, invf, half_layout, amp, pos, kc, vc, slots, eps)
    x = src.double()
    rc = oracle.rms_unit(x[:, QR:QR + R], eps) * kn.double()
    row = turned(torch.cat([rc, x[:, QR + R:QR + R + 6]], -1)[:, None], R)[:, 0]
    assert (cq.double() - oracle.rms_unit(x[:, :QR], eps) * qn.double()
            ).abs().max() < 1e-5
    assert (kc[slots // BS, 0, slots % BS].double() - row).abs().max() < 1e-5
    assert (vc[slots // BS, 0, :, slots % BS].double() - rc).abs().max() < 1e-5
    # queries: no norm, last channels turned, no cache
    src = torch.randn(T, 2 * 11, generator=g)
    out = torch.zeros(T, 2 * 11)
    ops.head_rope_store(out, src, 0, 2, 11, None, 0, 5, 0, 0, 0, None, 0, -1,
                        -1, invf, half_layout, amp, pos, None, None, None, eps)
    assert (out.double() - turned(src.double().view(T, 2, 11), 5)
            .reshape(T, -1)).abs().max() < 1e-5


@pytest.mark.parametrize("H,G,N,P", [(4, 2, 6, 5), (2, 2, 16, 8), (3, 1, 5, 12)])
def test_delta_rule_alone(H, G, N, P):
    """ops.delta_scan against the oracle's recurrence: two sequences, one of
    them continuing from a state, slots out of order."""
    from gpustack_amd import ops

    g = torch.Generator().manual_seed(N)
    n0, n1 = 9, 6
    T = n0 + n1
    nqk = G * N
    src = torch.randn(T, 2 * nqk + H * P, generator=g)
    gates = torch.randn(T, 2 * H + 1, generator=g) * 2
    dt_bias, a_log = torch.randn(H, generator=g), torch.randn(H, generator=g) - 1
    state = torch.randn(3, H, N, P, generator=g)       # junk to be ignored
    y = torch.zeros(T, H * P)
    meta = lambda a: torch.tensor(a, dtype=torch.int32)
    pos = meta(list(range(n0)) + list(range(n1)))
    ops.delta_scan(y, src, 0, nqk, 2 * nqk, gates, 1, 1 + H, H, G, N, P,
                   dt_bias, a_log, state, meta([0, n0]), meta([n0, n1]),
                   meta([2, 0]), pos)
    # the second sequence goes on for 4 more rows from its slot
    src2 = torch.randn(4, 2 * nqk + H * P, generator=g)
    gates2 = torch.randn(4, 2 * H + 1, generator=g) * 2
    y2 = torch.zeros(4, H * P)
    ops.delta_scan(y2, src2, 0, nqk, 2 * nqk, gates2, 1, 1 + H, H, G, N, P,
                   dt_bias, a_log, state, meta([0]), meta([4]), meta([0]),
                   meta([n1, n1 + 1, n1 + 2, n1 + 3]))

    def ref(rows, gate_rows):
        x, gr = rows.double(), gate_rows.double()
        n = x.shape[0]
        q = x[:, :nqk].view(n, G, N)
        k = x[:, nqk:2 * nqk].view(n, G, N)
        v = x[:, 2 * nqk:].view(n, H, P)
        q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * N ** -0.5
        k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
        gg = torch.exp(-torch.exp(a_log.double())
                       * oracle.softplus(gr[:, 1:1 + H] + dt_bias.double()))
        beta = torch.sigmoid(gr[:, 1 + H:1 + 2 * H])
        rep = H // G
        return torch.cat([oracle.delta_recurrence(
            q[:, h // rep], k[:, h // rep], v[:, h], beta[:, h], gg[:, h])
            for h in range(H)], -1)

    assert (y[:n0].double() - ref(src[:n0], gates[:n0])).abs().max() < 1e-5
    both = ref(torch.cat([src[n0:], src2]), torch.cat([gates[n0:], gates2]))
    assert (y[n0:].double() - both[:n1]).abs().max() < 1e-5
    assert (y2.double() - both[n1:]).abs().max() < 1e-5


def test_centred_sandwich_norm_alone():
    from gpustack_amd import ops

    g = torch.Generator().manual_seed(2)
    T, W, eps = 5, 22, 1e-5
    x = torch.randn(T, W, generator=g) * 3 + 1.5
    a = torch.randn(T, W, generator=g) * 0.2 - 4.0      # a large common offset
    pw, nw = torch.rand(W, generator=g) + 0.5, torch.rand(W, generator=g) + 0.5
    h = torch.zeros(T, W)
    x0 = x.double().clone()
    ops.sandwich_add_norm(x, a, pw, 1.0, eps, None, nw, h, center=True)
    rx = x0 + oracle.layer_norm(a.double(), pw, eps)
    assert (x.double() - rx).abs().max() < 1e-5
    assert (h.double() - oracle.layer_norm(rx, nw, eps)).abs().max() < 1e-5


def test_latent_mixer_alone(tmp_path):
    assert _one(tmp_path, [oracle.latent_layer(ff=0)]) < TOL


def test_latent_mixer_borrowing_keys(tmp_path):
    layers = [oracle.latent_layer(ff=0, window=50), oracle.delta_layer(),
              oracle.latent_layer(ff=0, window=4, kv_from=0, heads=2, dim=3,
                                  vdim=7, q_rank=5),
              oracle.latent_layer(ff=8, window=6),
              oracle.latent_layer(ff=0, window=11, kv_from=3)]
    assert _one(tmp_path, layers, n=33) < TOL


def test_delta_mixer_alone(tmp_path):
    assert _one(tmp_path, [oracle.delta_layer()]) < TOL


def test_parallel_mixer_alone(tmp_path):
    assert _one(tmp_path, [oracle.parallel_layer(ff=0)]) < TOL


def test_large_sinks_and_caps(tmp_path):
    """Sinks that outweigh every score, and a cap that bends every score."""
    cfg = oracle.make_config(layers=[
        oracle.latent_layer(ff=0, scale=1.5),
        oracle.parallel_layer(left=oracle.softmax_entry(softcap=0.7, scale=2.0))])
    w = oracle.make_weights(cfg, seed=5)
    w["l0.mix.sink"] = torch.tensor([6.0, -6.0, 2.5], dtype=torch.bfloat16)
    d = oracle.save_model(tmp_path, cfg, w)
    toks = tokens_for(cfg, 30, 2)
    ref = oracle.forward(cfg, w, toks)
    got = replay(make_engine(d), {"a": toks}, [[("a", 30)]])["a"]
    assert err(got, ref) < TOL
    no_sink = dict(w)
    no_sink["l0.mix.sink"] = torch.full((3,), -40.0, dtype=torch.bfloat16)
    assert err(oracle.forward(cfg, no_sink, toks), ref) > 0.02
    flat = json.loads(json.dumps(cfg))
    flat["layers"][1]["mixer"]["left"]["softcap"] = 50.0
    assert err(oracle.forward(flat, w, toks), ref) > 0.02


@pytest.mark.parametrize("layers", [
    # kv heads == heads everywhere, value size == key size, full rotation
    [oracle.delta_layer(heads=2, kv_heads=2, dim=4, vdim=4, conv=2),
     oracle.parallel_layer(left=oracle.softmax_entry(heads=2, kv_heads=2, dim=6,
                                                     vdim=6, rot_dims=6),
                           right=oracle.delta_mixer_entry(heads=3, kv_heads=3,
                                                          dim=5, vdim=3,
                                                          conv=2))],
    # one head, one key head, one tap (no convolution state), window 1
    [oracle.latent_layer(heads=1, dim=4, rot_dim=2, vdim=3, kv_rank=5, q_rank=3,
                         window=1),
     oracle.delta_layer(heads=1, kv_heads=1, dim=3, vdim=9, conv=1),
     oracle.parallel_layer(left=oracle.softmax_entry(heads=1, kv_heads=1, dim=4,
                                                     vdim=5, rot_dims=2,
                                                     softcap=0.0),
                           right=oracle.delta_mixer_entry(heads=1, kv_heads=1,
                                                          dim=7, vdim=2,
                                                          conv=5))],
    # a window wider than the sequence, no frequency scaling, many heads per
    # key head, sizes that no vector path divides
    [oracle.latent_layer(heads=5, dim=3, rot_dim=6, vdim=4, kv_rank=7, q_rank=9,
                         window=500, scaling=False),
     oracle.parallel_layer(left=oracle.softmax_entry(heads=6, kv_heads=1, dim=10,
                                                     vdim=3, rot_dims=2,
                                                     scaling=False),
                           right=oracle.delta_mixer_entry(heads=6, kv_heads=2,
                                                          dim=3, vdim=5,
                                                          conv=3)),
     oracle.latent_layer(heads=2, dim=5, rot_dim=6, vdim=2, kv_rank=7, q_rank=4,
                         window=3, kv_from=0, scaling=False)],
])
def test_other_sizes(tmp_path, layers):
    steps = [[("a", 11)], [("a", 2)], [("a", 19)]] + [[("a", 1)]] * 5
    assert _one(tmp_path, layers, n=37, width=18, steps=steps) < TOL


# ---- schedules ------------------------------------------------------------------

def test_whole_prompts_and_first_tokens(model):
    cfg, w, d = model
    eng = make_engine(d)
    for n in (1, 2, 3, 17, 64):
        toks = tokens_for(cfg, n, n)
        got = replay(eng, {"a": toks}, [[("a", n)]])["a"]
        assert err(got, oracle.forward(cfg, w, toks)) < TOL, n


def test_prefill_equals_token_by_token(model):
    cfg, w, d = model
    toks = tokens_for(cfg, 50, 7)
    ref = oracle.forward(cfg, w, toks)
    eng = make_engine(d)
    whole = replay(eng, {"a": toks}, [[("a", 50)]])["a"]
    single = replay(eng, {"a": toks}, [[("a", 1)]] * 50)["a"]
    late = replay(eng, {"a": toks}, [[("a", 18)]] + [[("a", 1)]] * 32)["a"]
    for got in (whole, single, late):
        assert err(got, ref) < TOL
    assert err(single, whole) < 1e-5 and err(late, whole) < 1e-5


@pytest.mark.parametrize("sizes", [[2] * 20, [16, 16, 8], [15, 2, 17, 1, 5],
                                   [1, 2, 3, 31, 3], [33, 7], [9, 31]])
def test_portions(model, sizes):
    """Portions cut inside pages, windows and the convolutions' reach."""
    cfg, w, d = model
    toks = tokens_for(cfg, sum(sizes), 3)
    got = replay(make_engine(d), {"a": toks}, [[("a", n)] for n in sizes])["a"]
    assert err(got, oracle.forward(cfg, w, toks)) < TOL


def test_unequal_batch_equals_each_alone(model):
    cfg, w, d = model
    prompts = {"a": tokens_for(cfg, 40, 1), "b": tokens_for(cfg, 9, 2),
               "c": tokens_for(cfg, 23, 3), "d": tokens_for(cfg, 30, 4)}
    schedule = [
        [("a", 20), ("b", 2)],
        [("b", 1), ("a", 1), ("c", 12)],
        [("c", 2), ("d", 30), ("a", 1), ("b", 1)],
        [("a", 18), ("b", 5), ("c", 9)],
    ]
    eng = make_engine(d)
    got = replay(eng, prompts, schedule)
    for r, toks in prompts.items():
        assert err(got[r], oracle.forward(cfg, w, toks)) < TOL, r
        alone = replay(eng, {r: toks}, [[(r, len(toks))]])[r]
        assert err(got[r], alone) < 1e-5, r


def test_blocks_and_slots_are_used_again(model):
    """A pool of 7 usable blocks and 2 state slots: every request takes
    blocks and a slot that an ended one has just given back."""
    cfg, w, d = model
    eng = make_engine(d, blocks=8, max_seqs=2)
    kv = eng.scheduler.kv
    free0, slots0 = kv.allocator.num_free, kv.state_allocator.num_free
    prompts = {f"r{i}": tokens_for(cfg, n, 20 + i)
               for i, n in enumerate([50, 33, 17, 60, 40, 31])}
    schedule = [
        [("r0", 30), ("r1", 2)], [("r0", 20), ("r1", 31)],      # r0, r1 end
        [("r2", 16), ("r3", 40)], [("r2", 1), ("r3", 20)],      # r2, r3 end
        [("r4", 38), ("r5", 2)], [("r4", 2), ("r5", 29)],
    ]
    got = replay(eng, prompts, schedule)
    for r, toks in prompts.items():
        assert err(got[r], oracle.forward(cfg, w, toks)) < TOL, r
    assert kv.allocator.num_free == free0
    assert kv.state_allocator.num_free == slots0


def test_long_decoding_across_pages_and_windows(model):
    cfg, w, d = model
    toks = tokens_for(cfg, 5 + 140, 13)
    eng = make_engine(d)
    got = replay(eng, {"a": toks}, [[("a", 5)]] + [[("a", 1)]] * 140)["a"]
    assert err(got, oracle.forward(cfg, w, toks)) < TOL


def test_bf16_engine_is_close(model):
    cfg, w, d = model
    toks = tokens_for(cfg, 40, 5)
    eng = make_engine(d, dtype="bfloat16")
    got = replay(eng, {"a": toks}, [[("a", 23)], [("a", 16)], [("a", 1)]])["a"]
    assert err(got, oracle.forward(cfg, w, toks)) < 0.15


# ---- faults that random weights would hide ------------------------------------------

def standout_model(tmp_path, kind, far_pos, n, window=1000):
    """A one-mixer model and a prompt of one filler token in which the LAST
    token's scores single out the key at `far_pos`: the token put there is
    the one of the vocabulary whose presence changes the last row most (a
    short-prompt search with the oracle), and the score scale is large, so
    the softmax is nearly one-hot. Losing that key, or wrongly admitting
    it, changes the row wholly."""
    if kind == "latent":
        L = oracle.latent_layer(heads=2, dim=8, rot_dim=2, vdim=6, kv_rank=12,
                                q_rank=8, window=window, scale=6.0, ff=0,
                                scaling=False)
    else:
        L = oracle.parallel_layer(
            left=oracle.softmax_entry(heads=2, kv_heads=1, dim=12, vdim=6,
                                      rot_dims=2, scale=6.0, softcap=60.0,
                                      scaling=False), ff=0)
    cfg = oracle.make_config(width=16, vocab=40, layers=[L])
    w = oracle.make_weights(cfg, seed=9)
    if kind == "latent":
        w["l0.mix.sink"] = torch.zeros(2, dtype=torch.bfloat16)
    filler, last = 0, 39
    best, best_t = -1.0, 1
    base = oracle.forward(cfg, w, [filler] * 7 + [last])[-1:]
    for t in range(1, 39):
        e = err(oracle.forward(cfg, w, [filler] * 3 + [t] + [filler] * 3
                               + [last])[-1:], base)
        if e > best:
            best, best_t = e, t
    toks = [filler] * n
    toks[far_pos] = best_t
    toks[-1] = last
    return cfg, w, oracle.save_model(tmp_path, cfg, w), toks


@pytest.mark.parametrize("kind", ["latent", "softmax"])
@pytest.mark.parametrize("far_pos", [0, 15, 16, 31, 200])
@pytest.mark.parametrize("decode", [False, True])
def test_far_key_among_hundreds(tmp_path, kind, far_pos, decode):
    cfg, w, d, toks = standout_model(tmp_path, kind, far_pos, 300)
    ref = oracle.forward(cfg, w, toks)[-1:]
    # the key matters: without it the last row is another one altogether
    other = list(toks)
    other[far_pos] = 0
    assert err(oracle.forward(cfg, w, other)[-1:], ref) > 0.05
    eng = make_engine(d)
    n = len(toks)
    steps = [[("a", n - 1)], [("a", 1)]] if decode else [[("a", n)]]
    got = replay(eng, {"a": toks}, steps)["a"][-1:]
    assert err(got, ref) < TOL


@pytest.mark.parametrize("gap", [-1, 0, 1])   # just inside, at, just outside
@pytest.mark.parametrize("decode", [False, True])
def test_window_edge(tmp_path, gap, decode):
    n, window = 83, 19
    far_pos = (n - 1) - (window - 1) - gap        # gap <= 0: seen
    cfg, w, d, toks = standout_model(tmp_path, "latent", far_pos, n, window)
    ref = oracle.forward(cfg, w, toks)[-1:]
    eng = make_engine(d)
    steps = [[("a", n - 1)], [("a", 1)]] if decode \
        else [[("a", 40)], [("a", n - 40)]]
    got = replay(eng, {"a": toks}, steps)["a"][-1:]
    assert err(got, ref) < TOL
    # and the edge is where the oracle says: moving the mask by one key
    # changes this row
    moved = json.loads(json.dumps(cfg))
    mk = moved["layers"][0]["mixer"]["mask"]
    mk["size"] += 1 if gap == 1 else -1 if gap == 0 else 0
    if gap != -1:
        assert err(oracle.forward(moved, w, toks)[-1:], ref) > 0.02


def test_state_carries_the_first_token_to_the_last_row(tmp_path):
    """A delta rule that hardly decays: the first token still shapes the
    last row, through a prompt cut into portions and decoded tokens."""
    cfg = oracle.make_config(width=16, layers=[
        oracle.delta_layer(heads=2, kv_heads=1, dim=8, vdim=6, conv=2)])
    w = oracle.make_weights(cfg, seed=4)
    w["l0.mix.A_log"] = torch.full((2,), -9.0, dtype=torch.bfloat16)
    d = oracle.save_model(tmp_path, cfg, w)
    toks = tokens_for(cfg, 60, 8)
    ref = oracle.forward(cfg, w, toks)
    other = [(toks[0] + 1) % cfg["vocab"]] + toks[1:]
    assert err(oracle.forward(cfg, w, other)[-1:], ref[-1:]) > 0.01
    steps = [[("a", 3)], [("a", 20)], [("a", 2)], [("a", 20)]] + [[("a", 1)]] * 15
    got = replay(make_engine(d), {"a": toks}, steps)["a"]
    assert err(got, ref) < TOL


def test_convolution_across_portion_starts(tmp_path):
    """Portions shorter than the convolution's reach, in both delta mixers."""
    layers = [oracle.delta_layer(conv=5),
              oracle.parallel_layer(right=oracle.delta_mixer_entry(
                  heads=2, kv_heads=2, dim=4, vdim=4, conv=6))]
    steps = [[("a", 1)], [("a", 2)], [("a", 1)], [("a", 3)], [("a", 2)],
             [("a", 12)], [("a", 1)], [("a", 1)], [("a", 4)]]
    assert _one(tmp_path, layers, n=27, steps=steps) < TOL


# ---- the framework's own entry points -------------------------------------------

def test_greedy_generation_through_the_scheduler(model):
    cfg, w, d = model
    eng = make_engine(d)
    prompts = [tokens_for(cfg, n, 40 + n) for n in (3, 21, 9)]
    outs = eng.generate(prompts, SamplingParams(max_tokens=14, temperature=0.0,
                                                ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert o == oracle.greedy(cfg, w, p, 14)


def test_generation_with_chunked_prefill_and_small_pool(model):
    cfg, w, d = model
    eng = make_engine(d, blocks=14, max_prefill_tokens=16)
    prompts = [tokens_for(cfg, n, 60 + n) for n in (45, 7, 30)]
    outs = eng.generate(prompts, SamplingParams(max_tokens=10, temperature=0.0,
                                                ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert o == oracle.greedy(cfg, w, p, 10)


def test_replay_command(model, tmp_path):
    """The replay driver writes the wanted rows, step by step."""
    from gpustack_amd.engine.replay import run_trace

    cfg, w, d = model
    toks = tokens_for(cfg, 30, 77)
    lines = [json.dumps({"step": 0, "entries": [
                {"id": "x", "tokens": toks[:20], "want": [0, 19]}], "end": []}),
             json.dumps({"step": 1, "entries": [
                 {"id": "x", "tokens": toks[20:29], "want": []}], "end": []}),
             json.dumps({"step": 2, "entries": [
                 {"id": "x", "tokens": toks[29:], "want": [0]}], "end": ["x"]})]
    out = io.StringIO()
    assert run_trace(d, "float32", str(tmp_path / "o"), 64, lines=lines,
                     out=out, device="cpu") == 0
    assert out.getvalue().split() == ["done", "0", "done", "1", "done", "2"]
    import numpy as np

    ref = oracle.forward(cfg, w, toks)
    a = torch.from_numpy(np.fromfile(tmp_path / "o" / "0.f32", dtype="<f4")
                         ).view(2, -1)
    b = torch.from_numpy(np.fromfile(tmp_path / "o" / "2.f32", dtype="<f4")
                         ).view(1, -1)
    assert not (tmp_path / "o" / "1.f32").exists()
    assert err(a, ref[[0, 19]]) < TOL and err(b, ref[[29]]) < TOL
