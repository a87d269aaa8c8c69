"""Livasun through the engine (scheduler, paged pools, state slots, model
runner, ops) against the plain float64 oracle in tests/livasun_oracle.py.

Every test writes its own small checkpoint (config.json + safetensors with
random bf16 weights) and loads it like a served model. The engine runs in
fp32 here so that a structural fault — a key one position off at the
window's edge, a state that is lost or carried into the wrong request, a
convolution input missing at a portion's start, a group wrongly kept — shows
far above the rounding floor; one test repeats the comparison in bf16.
Windows are a few tokens wide, so every key inside one carries weight.
"""
import io
import json
import sys
from pathlib import Path

import pytest
import torch

sys.path.insert(0, str(Path(__file__).resolve().parent))
import livasun_oracle as oracle  # noqa: E402
from test_fusipel import err, make_engine, replay, tokens_for  # noqa: E402

from gpustack_amd.engine import SamplingParams  # noqa: E402
from gpustack_amd.engine.config import (ModelSpec, PagedMixerSpec,  # noqa: E402
                                        ScanMixerSpec)

TOL = 2e-4      # fp32 engine against the float64 oracle


def rows_over(got, ref, tol):
    """Share of rows whose centred RMS difference, relative to the row's
    own RMS, is above tol. In bf16 a router's near-tie may fall the other
    way and move a whole row; such rows are counted, not forbidden."""
    d = got.double() - ref
    d = d - d.mean(-1, keepdim=True)
    c = ref - ref.mean(-1, keepdim=True)
    e = d.pow(2).mean(-1).sqrt() / c.pow(2).mean(-1).sqrt()
    return float((e > tol).double().mean())


@pytest.fixture(scope="module")
def model(tmp_path_factory):
    cfg = oracle.make_config()
    w = oracle.make_weights(cfg, seed=3)
    d = oracle.save_model(tmp_path_factory.mktemp("livasun"), cfg, w)
    return cfg, w, d


def _one(tmp_path, layers, n=41, seed=0, width=24, steps=None, **kw):
    """A model of the given layers: whole prompt (or `steps`) vs oracle."""
    cfg = oracle.make_config(width=width, layers=layers, **kw)
    w = oracle.make_weights(cfg, seed=seed)
    d = oracle.save_model(tmp_path, cfg, w)
    toks = tokens_for(cfg, n, seed + 11)
    got = replay(make_engine(d), {"a": toks}, steps or [[("a", n)]])["a"]
    return err(got, oracle.forward(cfg, w, toks))


# ---- configuration ------------------------------------------------------------

def test_config_is_read_from_the_file(model):
    cfg, _, d = model
    spec = ModelSpec.from_dir(d)
    assert spec.architecture == "Livasun" and spec.fp32_residual
    assert spec.vocab_size == cfg["vocab"] and spec.hidden_size == cfg["width"]
    assert spec.embed_scale == cfg["embedding"]["scale"]
    assert spec.rms_norm_eps == cfg["norm"]["eps"]
    kinds = [type(ls.mixer) for ls in spec.layers]
    assert kinds == [PagedMixerSpec, ScanMixerSpec, PagedMixerSpec,
                     ScanMixerSpec, PagedMixerSpec]
    a0, c0 = spec.layers[0].mixer, cfg["layers"][0]["mixer"]
    assert (a0.heads, a0.kv_heads, a0.qk_dim, a0.v_dim, a0.window, a0.scale) == (
        c0["heads"], c0["kv_heads"], c0["dim"], c0["vdim"], c0["mask"]["size"],
        c0["scale"])
    assert a0.q_temp == (c0["q_temp"]["coef"], c0["q_temp"]["every"])
    assert a0.head_norm and a0.distance_bias and a0.v_mix and not a0.rot.dims
    assert spec.layers[2].mixer.q_temp is None
    assert spec.layers[4].mixer.window == 0
    m1, c1 = spec.layers[1].mixer, cfg["layers"][1]["mixer"]
    assert (m1.kind, m1.heads, m1.groups, m1.state, m1.vdim, m1.conv,
            m1.norm_groups) == ("mamba2", c1["heads"], c1["groups"], c1["state"],
                                c1["vdim"], c1["conv"], c1["norm_groups"])
    m3, c3 = spec.layers[3].mixer, cfg["layers"][3]["mixer"]
    assert (m3.kind, m3.state, m3.decay) == ("lightning", c3["dim"],
                                            tuple(c3["decay"]))
    f1, r1 = spec.layers[1].mlp, cfg["layers"][1]["mlp"]["router"]
    assert (f1.experts, f1.top, f1.groups, f1.keep_groups, f1.route_scale,
            f1.group_top, f1.renorm, f1.route_scores) == (
        r1["experts"], r1["top"], r1["groups"]["count"], r1["groups"]["keep"],
        r1["scale"], 2, True, "sigmoid")
    assert spec.layers[2].mlp is None
    # attention runs own paged pools, recurrent runs a state slot
    pools = spec.kv_pool_widths()
    assert pools[0] == ("kv", c0["kv_heads"], c0["dim"], c0["vdim"])
    assert pools[1] == ("state",) and pools[3] == ("state",)
    shapes = spec.state_pool_shapes()
    assert shapes[0] is None
    assert shapes[1] == (c1["heads"], c1["state"], c1["vdim"], c1["conv"] - 1,
                         c1["heads"] * c1["vdim"] + 2 * c1["groups"] * c1["state"])
    assert shapes[3] == (c3["heads"], c3["dim"], c3["vdim"], 0, 0)
    assert spec.state_bytes_per_slot(2) == (
        4 * c1["heads"] * c1["state"] * c1["vdim"]
        + 2 * (c1["conv"] - 1) * shapes[1][4]
        + 4 * c3["heads"] * c3["dim"] * c3["vdim"])


def test_bad_configurations_are_refused():
    cfg = oracle.make_config(layers=[oracle.attn_layer(heads=3, kv_heads=2)])
    with pytest.raises(ValueError):
        ModelSpec.from_hf_config(cfg)
    cfg = oracle.make_config(layers=[oracle.attn_layer(),
                                     oracle.attn_layer(vdim=8)])
    with pytest.raises(ValueError):
        ModelSpec.from_hf_config(cfg)
    cfg = oracle.make_config(layers=[oracle.lightning_layer(decay=(0.5,))])
    with pytest.raises(ValueError):
        ModelSpec.from_hf_config(cfg)
    cfg = oracle.make_config(layers=[oracle.mamba_layer(
        mlp=oracle.moe(experts=6, count=3, keep=1, top=3))])
    with pytest.raises(ValueError):
        ModelSpec.from_hf_config(cfg)


def test_state_models_refuse_prefix_caching_and_speculation(model):
    _, _, d = model
    with pytest.raises(ValueError):
        make_engine(d, enable_prefix_caching=True)
    with pytest.raises(ValueError):
        make_engine(d, speculative={"method": "ngram", "num_draft_tokens": 2})


# ---- each mechanism alone -----------------------------------------------------

def test_head_norm_temperature_and_value_blend_alone():
    """ops.head_norm_store against the oracle's pieces, at positions on
    both sides of every temperature step."""
    from gpustack_amd import ops

    H, G, d, dv, eps, BS = 3, 1, 10, 6, 1e-5, 4
    qt = {"coef": 0.7, "every": 6}
    pos = torch.tensor([0, 4, 5, 6, 10, 11, 12, 17, 18, 599, 600, 5000],
                       dtype=torch.int32)
    T = pos.numel()
    g = torch.Generator().manual_seed(4)
    qkv = torch.randn(T, (H + G) * d + G * dv, generator=g)
    vf = torch.randn(T, G * dv, generator=g)
    qw, kw = torch.rand(d, generator=g) + 0.5, torch.rand(d, generator=g) + 0.5
    lam = torch.tensor([0.35])
    q = torch.zeros(T, H * d)
    kc, vc = torch.zeros(3, G, BS, d), torch.zeros(3, G, dv, BS)
    slots = torch.arange(T)
    ops.head_norm_store(q, qkv.clone(), H * d, G * d, qw, kw, d, qt["coef"],
                        qt["every"], pos, vf, lam, kc, vc, slots, eps)
    x = qkv.double()
    rq = oracle.unit_rms(x[:, :H * d].view(T, H, d), eps, qw.double()) \
        * oracle.query_temperature(pos.long(), qt)[:, None, None]
    rk = oracle.unit_rms(x[:, H * d:(H + G) * d].view(T, G, d), eps, kw.double())
    rv = 0.65 * x[:, (H + G) * d:] + 0.35 * vf.double()
    assert (q.double() - rq.reshape(T, -1)).abs().max() < 1e-5
    assert (kc[slots // BS, :, slots % BS].double() - rk).abs().max() < 1e-5
    assert (vc[slots // BS, :, :, slots % BS].double()
            - rv.view(T, G, dv)).abs().max() < 1e-5
    # the temperature steps exactly where (p + 1) reaches a multiple
    t = oracle.query_temperature(pos.long(), qt)
    assert t[0] == 1.0 and t[1] == 1.0 and t[2] > 1.0 and t[2] == t[3]
    assert t[5] > t[4] and t[8] == t[7] and t[10] == t[9]


@pytest.mark.parametrize("E,count,keep,top", [(6, 3, 2, 2), (10, 5, 3, 3),
                                              (4, 0, 0, 1), (6, 6, 3, 2),
                                              (12, 2, 1, 5), (9, 3, 3, 4)])
def test_routing_alone(E, count, keep, top):
    """ops.route_topk against the oracle: negative choice scores, groups of
    one, every group kept, no groups."""
    from gpustack_amd import ops

    g = torch.Generator().manual_seed(E + top)
    z = torch.randn(64, E, generator=g) * 2
    corr = torch.randn(E, generator=g) * 0.6 - 0.8
    r = {"experts": E, "top": top, "scale": 1.7}
    if count:
        r["groups"] = {"count": count, "keep": keep}
    idx, wt = oracle.route(z.double(), corr.double(), r)
    ex = torch.zeros(64, top, dtype=torch.int32)
    w = torch.zeros(64, top)
    ops.route_topk(ex, w, z, corr, E, count or 1, keep or 1, 2, True, True, 1.7)
    assert torch.equal(ex.long().sort(-1)[0], idx.sort(-1)[0])
    assert (w.gather(1, ex.long().argsort(-1)).double()
            - wt.gather(1, idx.argsort(-1))).abs().max() < 1e-6
    assert (torch.sigmoid(z) + corr).min() < 0      # the case is exercised


def test_attention_mixer_alone(tmp_path):
    assert _one(tmp_path, [oracle.attn_layer()]) < TOL


def test_attention_without_window_temperature_and_blend(tmp_path):
    assert _one(tmp_path, [oracle.attn_layer(window=0, temp=None,
                                             v_mix=False)]) < TOL


def test_value_blend_starts_at_the_first_blending_layer(tmp_path):
    """The first blending layer is not the stack's first layer, a layer in
    between does not blend, and the lender's own weight is ignored."""
    layers = [oracle.attn_layer(v_mix=False, vdim=9), oracle.attn_layer(),
              oracle.lightning_layer(), oracle.attn_layer(v_mix=False, vdim=3),
              oracle.attn_layer(heads=2, dim=12), oracle.attn_layer(window=3)]
    assert _one(tmp_path, layers) < TOL
    cfg = oracle.make_config(layers=layers)
    w = oracle.make_weights(cfg, seed=0)
    toks = tokens_for(cfg, 20, 1)
    ref = oracle.forward(cfg, w, toks)
    w2 = dict(w)
    w2["l1.mix.vmix"] = torch.tensor(0.9).to(torch.bfloat16)
    assert err(oracle.forward(cfg, w2, toks), ref) == 0.0
    w2["l4.mix.vmix"] = torch.tensor(0.9).to(torch.bfloat16)
    assert err(oracle.forward(cfg, w2, toks), ref) > 1e-3


def test_mamba2_mixer_alone(tmp_path):
    assert _one(tmp_path, [oracle.mamba_layer()]) < TOL


def test_lightning_mixer_alone(tmp_path):
    assert _one(tmp_path, [oracle.lightning_layer()]) < TOL


def test_feed_forwards_alone(tmp_path):
    assert _one(tmp_path / "d", [oracle.lightning_layer(mlp=oracle.dense())]) < TOL
    assert _one(tmp_path / "m", [oracle.lightning_layer(mlp=oracle.moe())]) < TOL


@pytest.mark.parametrize("layers", [
    # kv heads == heads, value size == score size, one norm part
    [oracle.attn_layer(heads=3, kv_heads=3, dim=8, vdim=8),
     oracle.mamba_layer(heads=2, groups=2, state=9, vdim=3, conv=2,
                        norm_groups=1)],
    # one kv head, one head, one group, one tap, window of one key ...
    # ... and a temperature step that is no whole number
    [oracle.attn_layer(heads=5, kv_heads=1, dim=6, vdim=4, window=1,
                       temp=(0.7, 2.5)),
     oracle.mamba_layer(heads=1, groups=1, state=4, vdim=8, conv=1,
                        norm_groups=4),
     oracle.lightning_layer(heads=1, dim=5, vdim=9, decay=(1.0,))],
    # window wider than any prompt here, temperature stepping at every
    # position, many taps, parts == heads
    [oracle.attn_layer(window=500, temp=(1.5, 1), scale=0.2),
     oracle.mamba_layer(heads=6, groups=3, state=3, vdim=2, conv=6,
                        norm_groups=6, mlp=oracle.moe(experts=8, count=4,
                                                      keep=4, top=3, shared=5)),
     oracle.lightning_layer(heads=4, dim=3, vdim=6, decay=(0.1, 0.5, 0.9, 0.99),
                            mlp=oracle.moe(experts=5, count=5, keep=2, top=2,
                                           scale=0.5))],
])
def test_other_sizes(tmp_path, layers):
    steps = [[("a", 17)], [("a", 1)], [("a", 2)], [("a", 21)]]
    assert _one(tmp_path, layers, steps=steps, width=30, vocab=37,
                embed_scale=0.5, eps=1e-3) < TOL


# ---- schedules: whole, decoded, portions, batches, reuse ------------------------------------

def test_whole_prompts_and_first_tokens(model):
    cfg, w, d = model
    eng = make_engine(d)
    for n in (1, 2, 3, 4, 5, 16, 17, 50):
        toks = tokens_for(cfg, n, n)
        got = replay(eng, {"a": toks}, [[("a", n)]])["a"]
        assert err(got, oracle.forward(cfg, w, toks)) < TOL, n


def test_prefill_equals_token_by_token(model):
    cfg, w, d = model
    toks = tokens_for(cfg, 45, 8)
    eng = make_engine(d)
    whole = replay(eng, {"a": toks}, [[("a", 45)]])["a"]
    single = replay(eng, {"b": toks}, [[("b", 1)] for _ in toks])["b"]
    ref = oracle.forward(cfg, w, toks)
    assert err(whole, ref) < TOL and err(single, ref) < TOL
    assert err(single, whole) < 1e-5


@pytest.mark.parametrize("sizes", [
    [2] * 30, [3, 2, 5, 2, 16, 1, 1, 17, 2, 11], [1, 59], [59, 1], [7] * 8 + [4],
    [15, 1, 16, 17, 11]])
def test_portions(model, sizes):
    cfg, w, d = model
    n = sum(sizes)
    toks = tokens_for(cfg, n, 21)
    got = replay(make_engine(d), {"a": toks}, [[("a", s)] for s in sizes])["a"]
    assert err(got, oracle.forward(cfg, w, toks)) < TOL


def test_unequal_batch_equals_each_alone(model):
    cfg, w, d = model
    reqs = {"a": tokens_for(cfg, 70, 1), "b": tokens_for(cfg, 3, 2),
            "c": tokens_for(cfg, 33, 3), "d": tokens_for(cfg, 1, 4)}
    steps = [[("a", 40), ("b", 2)],
             [("a", 1), ("b", 1), ("c", 16), ("d", 1)],
             [("c", 1), ("a", 2)],          # order inside a step changes
             [("a", 27), ("c", 16)]]
    eng = make_engine(d)
    got = replay(eng, reqs, steps)
    for r, toks in reqs.items():
        ref = oracle.forward(cfg, w, toks)
        assert err(got[r], ref) < TOL, r
        alone = replay(eng, {r: toks}, [[(r, len(toks))]])[r]
        assert err(got[r], alone) < 1e-5, r


def test_blocks_and_slots_are_used_again(model):
    """A pool of a few blocks and two state slots serves request after
    request: every block and slot is reused, dirty, by a later request, and
    a request left out of a step keeps its state."""
    cfg, w, d = model
    eng = make_engine(d, blocks=9, max_seqs=2)
    kv = eng.runner.kv
    assert kv.state_allocator.num_slots == 2
    seen_slots = []
    for wave in range(4):
        a, b = f"a{wave}", f"b{wave}"
        reqs = {a: tokens_for(cfg, 50, 10 + wave), b: tokens_for(cfg, 37, 20 + wave)}
        steps = [[(a, 30)], [(b, 20), (a, 1)], [(b, 1)], [(a, 19), (b, 16)]]
        at = {r: 0 for r in reqs}
        got = {r: [] for r in reqs}
        for step in steps:
            entries, end = [], []
            for r, n in step:
                entries.append((r, reqs[r][at[r]:at[r] + n], list(range(n))))
                at[r] += n
                if at[r] == len(reqs[r]):
                    end.append(r)
            logits = eng.replay_step(entries, end)
            seen_slots += [q.state_slot for q in
                           getattr(eng, "_replay_seqs", {}).values()]
            off = 0
            for r, n in step:
                got[r].append(logits[off:off + n].double())
                off += n
        for r, toks in reqs.items():
            assert err(torch.cat(got[r]), oracle.forward(cfg, w, toks)) < TOL, r
        assert kv.state_allocator.num_free == 2
        assert kv.allocator.num_free == kv.allocator.num_blocks
    assert set(s for s in seen_slots if s >= 0) == {0, 1}
    with pytest.raises(RuntimeError):
        for i in range(3):                 # a third live request has no slot
            eng.replay_step([(f"x{i}", [1, 2], [])], [])


def test_long_decoding_across_pages_and_windows(model):
    cfg, w, d = model
    toks = tokens_for(cfg, 160, 5)
    steps = [[("a", 20)]] + [[("a", 1)]] * 140
    got = replay(make_engine(d), {"a": toks}, steps)["a"]
    assert err(got, oracle.forward(cfg, w, toks)) < TOL


def test_bf16_engine_is_close(model):
    cfg, w, d = model
    toks = tokens_for(cfg, 60, 6)
    steps = [[("a", 33)], [("a", 2)]] + [[("a", 1)]] * 25
    got = replay(make_engine(d, dtype="bfloat16"), {"a": toks}, steps)["a"]
    assert rows_over(got, oracle.forward(cfg, w, toks), 0.08) <= 0.1


# ---- faults that random weights would hide ------------------------------------------------

def standout_model(tmp_path, far_pos, n, window=0):
    """A one-mixer attention model in which the LAST token's query matches
    the key at `far_pos` far better than any other: W_k is W_q with its
    input channels shifted by one and the token at far_pos has the last
    token's embedding shifted back (the layer norm before the mixer has no
    weights here, so it commutes with the shift). The score scale is large
    enough that this one key outweighs the distance bias of the flatter
    heads: losing it, or wrongly admitting it, changes the row wholly."""
    L = oracle.attn_layer(heads=2, kv_heads=2, dim=32, vdim=6, window=window,
                          temp=(0.35, 50), v_mix=False, scale=1.0)
    cfg = oracle.make_config(width=32, vocab=40, layers=[L], embed_scale=2.0)
    w = oracle.make_weights(cfg, seed=9)
    w["l0.norm1"] = torch.ones_like(w["l0.norm1"])
    w["l0.norm1.b"] = torch.zeros_like(w["l0.norm1.b"])
    w["l0.mix.k"] = torch.roll(w["l0.mix.q"], -1, dims=1).contiguous()
    w["l0.mix.k.norm"] = w["l0.mix.q.norm"].clone()
    w["embed"][38] = torch.roll(w["embed"][39], -1, dims=0)
    toks = [t % 38 for t in tokens_for(cfg, n, 5)]
    toks[far_pos] = 38
    toks[-1] = 39
    return cfg, w, oracle.save_model(tmp_path, cfg, w), toks


@pytest.mark.parametrize("far_pos", [0, 15, 16, 31, 200])
@pytest.mark.parametrize("decode", [False, True])
def test_far_key_among_hundreds(tmp_path, far_pos, decode):
    cfg, w, d, toks = standout_model(tmp_path, far_pos, 420)
    ref = oracle.forward(cfg, w, toks)[-1:]
    other = list(toks)
    other[far_pos] = 1        # the key matters: without it the row differs
    assert err(oracle.forward(cfg, w, other)[-1:], ref) > 0.05
    n = len(toks)
    steps = [[("a", n - 1)], [("a", 1)]] if decode else [[("a", n)]]
    got = replay(make_engine(d), {"a": toks}, steps)["a"][-1:]
    assert err(got, ref) < TOL


@pytest.mark.parametrize("gap", [-1, 0, 1])   # just inside, at, just outside
@pytest.mark.parametrize("decode", [False, True])
def test_window_edge(tmp_path, gap, decode):
    n, window = 83, 19
    far_pos = (n - 1) - (window - 1) - gap        # gap <= 0: seen
    cfg, w, d, toks = standout_model(tmp_path, far_pos, n, window)
    ref = oracle.forward(cfg, w, toks)[-1:]
    steps = [[("a", n - 1)], [("a", 1)]] if decode \
        else [[("a", 40)], [("a", n - 40)]]
    got = replay(make_engine(d), {"a": toks}, steps)["a"][-1:]
    assert err(got, ref) < TOL
    # and the edge is where the oracle says: a mask moved by one key
    # changes this row
    moved = json.loads(json.dumps(cfg))
    moved["layers"][0]["mixer"]["mask"]["size"] += \
        1 if gap == 1 else -1 if gap == 0 else 0
    if gap != -1:
        assert err(oracle.forward(moved, w, toks)[-1:], ref) > 0.02


@pytest.mark.parametrize("kind", ["lightning", "mamba2"])
def test_state_reaches_far_back(tmp_path, kind):
    """A state that does not decay carries the first token to the last
    row, which depends on it, through portions and decoding alike."""
    if kind == "lightning":
        L = oracle.lightning_layer(heads=2, dim=6, vdim=5, decay=(0.9999, 1.0))
    else:
        L = oracle.mamba_layer(heads=2, groups=1, state=6, vdim=5)
    cfg = oracle.make_config(layers=[L])
    w = oracle.make_weights(cfg, seed=2)
    if kind == "mamba2":      # small steps and rates: a long memory
        w["l0.mix.dt_bias"] = torch.full((2,), -4.0).to(torch.bfloat16)
        w["l0.mix.A_log"] = torch.full((2,), -3.0).to(torch.bfloat16)
    d = oracle.save_model(tmp_path, cfg, w)
    toks = tokens_for(cfg, 120, 3)
    ref = oracle.forward(cfg, w, toks)
    other = [(toks[0] + 1) % cfg["vocab"]] + toks[1:]
    assert err(oracle.forward(cfg, w, other)[-1:], ref[-1:]) > 1e-3
    steps = [[("a", 50)], [("a", 2)], [("a", 50)]] + [[("a", 1)]] * 18
    got = replay(make_engine(d), {"a": toks}, steps)["a"]
    assert err(got, ref) < TOL


def test_convolution_across_portion_starts(tmp_path):
    """Portions shorter than the convolution: its inputs come from the slot
    for several steps in a row, and from before position 0 as zeros."""
    L = oracle.mamba_layer(heads=2, groups=1, state=4, vdim=6, conv=7)
    cfg = oracle.make_config(layers=[L])
    w = oracle.make_weights(cfg, seed=5)
    d = oracle.save_model(tmp_path, cfg, w)
    toks = tokens_for(cfg, 40, 3)
    sizes = [2, 1, 1, 3, 2, 6, 7, 8, 1, 9]
    got = replay(make_engine(d), {"a": toks}, [[("a", s)] for s in sizes])["a"]
    assert err(got, oracle.forward(cfg, w, toks)) < TOL


# ---- the framework's own entry points -----------------------------------------------------

def test_greedy_generation_through_the_scheduler(model):
    cfg, w, d = model
    eng = make_engine(d)
    prompts = [tokens_for(cfg, n, 40 + n) for n in (3, 21, 9)]
    outs = eng.generate(prompts, SamplingParams(max_tokens=14, temperature=0.0,
                                                ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert o == oracle.greedy(cfg, w, p, 14)
    assert eng.runner.kv.state_allocator.num_free == 4


def test_generation_with_chunked_prefill_and_small_pool(model):
    cfg, w, d = model
    eng = make_engine(d, blocks=14, max_prefill_tokens=16, max_seqs=2)
    prompts = [tokens_for(cfg, n, 60 + n) for n in (45, 7, 30)]
    outs = eng.generate(prompts, SamplingParams(max_tokens=10, temperature=0.0,
                                                ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert o == oracle.greedy(cfg, w, p, 10)
    assert eng.runner.kv.state_allocator.num_free == 2


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
