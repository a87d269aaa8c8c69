"""Livasun on the GPU: the engine with the HIP kernels (fp32 vector-ALU
attention, bf16 MFMA attention with key split, state scan, short
convolution, fused row kernels, grouped expert kernels, captured decode
graphs) against the float64 oracle, on the schedules and the crafted cases
of tests/test_livasun.py."""
import sys
from pathlib import Path

import pytest
import torch

sys.path.insert(0, str(Path(__file__).resolve().parent))
import livasun_oracle as oracle  # noqa: E402
import test_fusipel as tf  # noqa: E402
import test_livasun as tl  # noqa: E402

from gpustack_amd import ops  # noqa: E402
from gpustack_amd.engine import SamplingParams  # noqa: E402

pytestmark = pytest.mark.gpu

# sizes the MFMA attention and the grouped expert kernels accept (score size
# % 32, value size % 16, width and expert width % 64), still unlike each
# other
ALIGNED = dict(width=64, vocab=97, layers=[
    oracle.attn_layer(heads=4, kv_heads=2, dim=32, vdim=16, window=37,
                      temp=(0.25, 20), mlp=oracle.dense(80)),
    oracle.mamba_layer(heads=4, groups=2, state=16, vdim=24, conv=4,
                       norm_groups=3,
                       mlp=oracle.moe(experts=8, count=2, keep=1, top=3, ff=64,
                                      shared=40)),
    oracle.attn_layer(heads=6, kv_heads=2, dim=64, vdim=16, window=0,
                      temp=None),
    oracle.lightning_layer(heads=3, dim=40, vdim=12,
                           decay=(0.6, 0.95, 0.999),
                           mlp=oracle.moe(experts=4, count=0, top=2, ff=128,
                                          shared=0)),
    oracle.attn_layer(heads=2, kv_heads=2, dim=32, vdim=16, window=130,
                      temp=(0.1, 64), mlp=oracle.dense(48)),
])

REQS = {"a": 150, "b": 3, "c": 61, "d": 1}
STEPS = [[("a", 47), ("b", 2)], [("a", 1), ("b", 1), ("c", 16), ("d", 1)],
         [("a", 90), ("c", 1)], [("c", 43), ("a", 1)], [("a", 11), ("c", 1)]]


@pytest.fixture
def gpu_engine():
    """Engine factory whose engines are torn down when the test is over:
    an engine is a reference cycle (runner <-> graph runner), so without an
    explicit collection its captured graphs and pools would linger into
    whatever runs next in the process."""
    import gc

    made = []

    def make(model_dir, **kw):
        made.append(tf.make_engine(model_dir, device="cuda", **kw))
        return made[-1]

    yield make
    made.clear()
    gc.collect()
    torch.cuda.synchronize()
    torch.cuda.empty_cache()


def _model(tmp_path, kw, seed=3):
    cfg = oracle.make_config(**kw)
    w = oracle.make_weights(cfg, seed=seed)
    return cfg, w, oracle.save_model(tmp_path / "m", cfg, w)


@pytest.mark.parametrize("name", ["default", "aligned"])
def test_fp32_engine_matches_oracle(tmp_path, gpu_engine, name):
    cfg, w, d = _model(tmp_path, {} if name == "default" else ALIGNED)
    eng = gpu_engine(d)
    reqs = {i: tf.tokens_for(cfg, n, 70 + n) for i, n in REQS.items()}
    got = tf.replay(eng, reqs, STEPS)
    for i, t in reqs.items():
        assert tf.err(got[i], oracle.forward(cfg, w, t)) < 5e-4, i


@pytest.mark.parametrize("name", ["default", "aligned"])
def test_bf16_engine_with_block_and_slot_reuse(tmp_path, gpu_engine, name):
    """bf16 serving path (MFMA attention and grouped expert kernels for the
    aligned sizes, the fp32 vector path for the others) in a pool that every
    repetition refills, with as many state slots as live requests."""
    cfg, w, d = _model(tmp_path, {} if name == "default" else ALIGNED)
    eng = gpu_engine(d, dtype="bfloat16", blocks=18)
    kv = eng.runner.kv
    if name == "aligned":
        q = torch.empty(1, 4, 32, dtype=torch.bfloat16, device="cuda")
        assert ops._load_paged().paged_attention_uses_mfma(
            q, kv.k_caches[0], kv.v_caches[0])
        assert eng.runner.model.graph_capturable()
    for rnd in range(3):
        reqs = {i: tf.tokens_for(cfg, n, 80 + n + rnd) for i, n in REQS.items()}
        got = tf.replay(eng, reqs, STEPS)
        for i, t in reqs.items():
            assert tl.rows_over(got[i], oracle.forward(cfg, w, t), 0.15) \
                <= 0.1, (rnd, i)
        assert kv.state_allocator.num_free == 4


def test_bf16_logits_do_not_depend_on_the_schedule(tmp_path, gpu_engine):
    cfg, w, d = _model(tmp_path, ALIGNED)
    eng = gpu_engine(d, dtype="bfloat16")
    reqs = {i: tf.tokens_for(cfg, n, 90 + n) for i, n in REQS.items()}
    mixed = tf.replay(eng, reqs, STEPS)
    for i, t in reqs.items():
        whole = tf.replay(eng, {i: t}, [[(i, len(t))]])[i]
        ref = oracle.forward(cfg, w, t)
        # both are rounding away from the oracle, and no further from each
        # other than from it
        assert tl.rows_over(mixed[i], whole.double(), 0.15) <= 0.1, i
        assert tl.rows_over(whole, ref, 0.15) <= 0.1, i


@pytest.mark.parametrize("sizes", [[2] * 20, [3, 2, 5, 2, 16, 1, 1, 17, 2, 11],
                                   [1, 59], [15, 1, 16, 17, 11]])
def test_portions(tmp_path, gpu_engine, sizes):
    cfg, w, d = _model(tmp_path, ALIGNED)
    toks = tf.tokens_for(cfg, sum(sizes), 21)
    got = tf.replay(gpu_engine(d), {"a": toks}, [[("a", s)] for s in sizes])["a"]
    assert tf.err(got, oracle.forward(cfg, w, toks)) < 5e-4


@pytest.mark.parametrize("dtype,tol", [("float32", 5e-4), ("bfloat16", 0.12)])
@pytest.mark.parametrize("far_pos", [0, 16, 63, 64, 500])
def test_far_key_among_hundreds(tmp_path, gpu_engine, dtype, tol, far_pos):
    """One key stands out among 1100 (tests/test_livasun.py standout_model);
    as the last row of a prompt and as a decoded token, where the MFMA
    kernel splits the keys over workgroups."""
    cfg, w, d, toks = tl.standout_model(tmp_path, far_pos, 1100)
    ref = oracle.forward(cfg, w, toks)[-1:]
    eng = gpu_engine(d, dtype=dtype, blocks=80)
    n = len(toks)
    a = tf.replay(eng, {"a": toks}, [[("a", n)]])["a"][-1:]
    b = tf.replay(eng, {"a": toks}, [[("a", n - 1)], [("a", 1)]])["a"][-1:]
    assert tf.err(a, ref) < tol and tf.err(b, ref) < tol


@pytest.mark.parametrize("dtype,tol", [("float32", 5e-4), ("bfloat16", 0.12)])
@pytest.mark.parametrize("gap", [0, 1])
def test_window_edge(tmp_path, gpu_engine, dtype, tol, gap):
    n, window = 211, 70                 # the edge inside a page and a key tile
    far_pos = (n - 1) - (window - 1) - gap
    cfg, w, d, toks = tl.standout_model(tmp_path, far_pos, n, window)
    ref = oracle.forward(cfg, w, toks)[-1:]
    eng = gpu_engine(d, dtype=dtype)
    a = tf.replay(eng, {"a": toks}, [[("a", 100)], [("a", n - 100)]])["a"][-1:]
    b = tf.replay(eng, {"a": toks}, [[("a", n - 1)], [("a", 1)]])["a"][-1:]
    assert tf.err(a, ref) < tol and tf.err(b, ref) < tol


@pytest.mark.parametrize("layers", [
    [oracle.mamba_layer(heads=2, groups=1, state=128, vdim=64, conv=4,
                        norm_groups=1)],
    [oracle.mamba_layer(heads=3, groups=3, state=200, vdim=8, conv=2,
                        norm_groups=3)],
    [oracle.lightning_layer(heads=2, dim=96, vdim=100, decay=(0.9, 0.999))],
])
def test_wide_states(tmp_path, gpu_engine, layers):
    """State sizes on every lane split of the scan kernel."""
    cfg = oracle.make_config(width=32, layers=layers)
    w = oracle.make_weights(cfg, seed=1)
    d = oracle.save_model(tmp_path / "m", cfg, w)
    toks = tf.tokens_for(cfg, 70, 2)
    steps = [[("a", 33)], [("a", 1)], [("a", 30)]] + [[("a", 1)]] * 6
    got = tf.replay(gpu_engine(d), {"a": toks}, steps)["a"]
    assert tf.err(got, oracle.forward(cfg, w, toks)) < 5e-4


@pytest.mark.parametrize("routed", [False, True])
def test_generation_with_decode_graphs(tmp_path, gpu_engine, routed):
    """fp32 greedy decoding equals the oracle's token for token. Without
    routed layers every decode step is a captured graph (state slots and
    block tables in static buffers); an fp32 expert bank waits for the host
    and decodes eagerly."""
    kw = dict(ALIGNED)
    if not routed:
        kw["layers"] = [dict(L, mlp=oracle.dense(40) if (L["mlp"] or {}).get(
            "kind") == "moe" else L["mlp"]) for L in ALIGNED["layers"]]
    cfg, w, d = _model(tmp_path, kw)
    eng = gpu_engine(d)
    assert (eng.runner.graph_runner is not None) == (not routed)
    prompts = [tf.tokens_for(cfg, n, 40 + n) for n in (3, 70, 9)]
    outs = eng.generate(prompts, SamplingParams(max_tokens=40, temperature=0.0,
                                                ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert o == oracle.greedy(cfg, w, p, 40)
    assert eng.runner.kv.state_allocator.num_free == 4


def test_bf16_generation_runs_and_stays_close(tmp_path, gpu_engine):
    """bf16 greedy decoding (captured graphs, grouped expert kernels) may
    part from the oracle at a near-tie; the logits of the tokens it did
    choose must still be the oracle's."""
    cfg, w, d = _model(tmp_path, ALIGNED)
    eng = gpu_engine(d, dtype="bfloat16")
    assert eng.runner.graph_runner is not None
    prompt = tf.tokens_for(cfg, 30, 5)
    out = eng.generate([prompt], SamplingParams(max_tokens=24, temperature=0.0,
                                                ignore_eos=True))[0]
    assert len(out) == 24
    full = prompt + out
    got = tf.replay(eng, {"z": full}, [[("z", len(full))]])["z"]
    assert tl.rows_over(got, oracle.forward(cfg, w, full), 0.15) <= 0.1
