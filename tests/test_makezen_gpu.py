"""Makezen on the GPU: the engine with the HIP kernels (per-head norm and
rotation row kernel, fp32 vector-ALU and bf16 MFMA attention with window,
sink and score cap, delta rule scan and step kernels, short convolution,
centred row norms, captured decode graphs) against the float64 oracle, on
the schedules and the crafted cases of tests/test_makezen.py."""
import sys
from pathlib import Path

import pytest
import torch

sys.path.insert(0, str(Path(__file__).resolve().parent))
import makezen_oracle as oracle  # noqa: E402
import test_fusipel as tf  # noqa: E402
import test_makezen as tm  # noqa: E402

from gpustack_amd import ops  # noqa: E402
from gpustack_amd.engine import SamplingParams  # noqa: E402

pytestmark = pytest.mark.gpu

# sizes the MFMA attention and the 16-byte row paths accept (key row % 32,
# value size % 16, channels % 8), still unlike each other
ALIGNED = dict(width=64, vocab=97, layers=[
    oracle.latent_layer(heads=4, dim=16, rot_dim=16, vdim=24, kv_rank=48,
                        q_rank=40, window=37, ff=80, base=1000.0, factor=4.0,
                        original=64, fast=8.0),
    oracle.delta_layer(heads=4, kv_heads=2, dim=16, vdim=24, conv=4),
    oracle.parallel_layer(
        left=oracle.softmax_entry(heads=6, kv_heads=2, dim=32, vdim=16,
                                  rot_dims=8, softcap=4.0, base=500.0,
                                  original=32),
        right=oracle.delta_mixer_entry(heads=3, kv_heads=1, dim=40, vdim=12,
                                       conv=3), ff=48),
    oracle.latent_layer(heads=2, dim=8, rot_dim=16, vdim=16, kv_rank=48,
                        q_rank=24, window=130, kv_from=0, ff=0, base=1000.0,
                        factor=4.0, original=64, fast=8.0),
    oracle.delta_layer(heads=2, kv_heads=2, dim=64, vdim=32, conv=2, ff=64),
])

REQS = {"a": 150, "b": 3, "c": 61, "d": 1}
STEPS = [[("a", 47), ("b", 2)], [("a", 1), ("b", 1), ("c", 16), ("d", 1)],
         [("a", 90), ("c", 1)], [("c", 43), ("a", 1)], [("a", 11), ("c", 1)]]


def rows_over(got, ref, tol):
    """Share of rows whose centred RMS difference, relative to the row's
    own RMS, is above tol."""
    d = got.double() - ref
    d = d - d.mean(-1, keepdim=True)
    c = ref - ref.mean(-1, keepdim=True)
    e = d.pow(2).mean(-1).sqrt() / c.pow(2).mean(-1).sqrt()
    return float((e > tol).double().mean())


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
    """bf16 serving path (MFMA attention for the aligned sizes, the fp32
    vector path for the others) in a pool that every repetition refills,
    with as many state slots as live requests."""
    cfg, w, d = _model(tmp_path, {} if name == "default" else ALIGNED)
    eng = gpu_engine(d, dtype="bfloat16", blocks=18)
    kv = eng.runner.kv
    if name == "aligned":
        q = torch.empty(1, 4, 64, dtype=torch.bfloat16, device="cuda")
        assert ops._load_paged().paged_attention_uses_mfma(
            q, kv.k_caches[0], kv.v_caches[0])
        assert kv.k_caches[3] is kv.k_caches[0]
    for rnd in range(3):
        reqs = {i: tf.tokens_for(cfg, n, 80 + n + rnd) for i, n in REQS.items()}
        got = tf.replay(eng, reqs, STEPS)
        for i, t in reqs.items():
            assert rows_over(got[i], oracle.forward(cfg, w, t), 0.15) <= 0.1, \
                (rnd, i)
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
        assert rows_over(mixed[i], whole.double(), 0.15) <= 0.1, i
        assert rows_over(whole, ref, 0.15) <= 0.1, i


@pytest.mark.parametrize("sizes", [[2] * 20, [3, 2, 5, 2, 16, 1, 1, 17, 2, 11],
                                   [33, 1, 1, 40]])
@pytest.mark.parametrize("name", ["default", "aligned"])
def test_portions_fp32(tmp_path, gpu_engine, sizes, name):
    cfg, w, d = _model(tmp_path, {} if name == "default" else ALIGNED)
    toks = tf.tokens_for(cfg, sum(sizes), 3)
    got = tf.replay(gpu_engine(d), {"a": toks}, [[("a", n)] for n in sizes])["a"]
    assert tf.err(got, oracle.forward(cfg, w, toks)) < 5e-4


def test_other_sizes_fp32_and_bf16(tmp_path, gpu_engine):
    """One head, one tap, window 1, many heads per key head, sizes that no
    vector path divides."""
    layers = [
        oracle.latent_layer(heads=1, dim=4, rot_dim=2, vdim=3, kv_rank=5,
                            q_rank=3, window=1),
        oracle.delta_layer(heads=1, kv_heads=1, dim=3, vdim=9, conv=1),
        oracle.parallel_layer(
            left=oracle.softmax_entry(heads=6, kv_heads=1, dim=10, vdim=3,
                                      rot_dims=2, scaling=False),
            right=oracle.delta_mixer_entry(heads=6, kv_heads=2, dim=3, vdim=5,
                                           conv=5)),
        oracle.latent_layer(heads=5, dim=3, rot_dim=6, vdim=4, kv_rank=7,
                            q_rank=9, window=500, scaling=False),
        oracle.latent_layer(heads=2, dim=5, rot_dim=6, vdim=2, kv_rank=7,
                            q_rank=4, window=3, kv_from=3, scaling=False),
        # more heads on one key stream than a workgroup's tile holds
        oracle.latent_layer(heads=20, dim=2, rot_dim=4, vdim=3, kv_rank=6,
                            q_rank=5, window=9, ff=0),
        oracle.parallel_layer(
            left=oracle.softmax_entry(heads=36, kv_heads=2, dim=4, vdim=2,
                                      rot_dims=4),
            right=oracle.delta_mixer_entry(heads=2, kv_heads=1, dim=4, vdim=4,
                                           conv=2), ff=0),
    ]
    cfg, w, d = _model(tmp_path, dict(width=18, layers=layers))
    toks = tf.tokens_for(cfg, 37, 11)
    steps = [[("a", 11)], [("a", 2)], [("a", 19)]] + [[("a", 1)]] * 5
    ref = oracle.forward(cfg, w, toks)
    got = tf.replay(gpu_engine(d), {"a": toks}, steps)["a"]
    assert tf.err(got, ref) < 5e-4
    got = tf.replay(gpu_engine(d, dtype="bfloat16"), {"a": toks}, steps)["a"]
    assert rows_over(got, ref, 0.2) <= 0.1


def test_long_decoding_fp32(tmp_path, gpu_engine):
    cfg, w, d = _model(tmp_path, ALIGNED)
    toks = tf.tokens_for(cfg, 5 + 140, 13)
    got = tf.replay(gpu_engine(d), {"a": toks},
                    [[("a", 5)]] + [[("a", 1)]] * 140)["a"]
    assert tf.err(got, oracle.forward(cfg, w, toks)) < 5e-4


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_context_with_key_split(tmp_path, gpu_engine, dtype):
    """A context long enough for the attention kernels to split a decode
    row's keys over workgroups (MFMA path), behind a window of 600, with
    sinks, on latent rows and on capped softmax heads."""
    import copy

    kw = dict(ALIGNED, layers=copy.deepcopy(ALIGNED["layers"]))
    kw["layers"][0]["mixer"]["mask"]["size"] = 600
    kw["layers"][3]["mixer"]["mask"]["size"] = 530
    cfg, w, d = _model(tmp_path, kw)
    toks = tf.tokens_for(cfg, 650, 21)
    steps = [[("a", 300)], [("a", 340)]] + [[("a", 1)]] * 10
    ref = oracle.forward(cfg, w, toks)
    got = tf.replay(gpu_engine(d, dtype=dtype, blocks=60), {"a": toks},
                    steps)["a"]
    if dtype == "float32":
        assert tf.err(got, ref) < 5e-4
    else:
        assert rows_over(got, ref, 0.15) <= 0.1


@pytest.mark.parametrize("kind", ["latent", "softmax"])
@pytest.mark.parametrize("far_pos", [0, 16, 511, 700])
@pytest.mark.parametrize("decode", [False, True])
def test_far_key_among_a_thousand(tmp_path, gpu_engine, kind, far_pos, decode):
    cfg, w, d, toks = tm.standout_model(tmp_path, kind, far_pos, 1100)
    ref = oracle.forward(cfg, w, toks)[-1:]
    n = len(toks)
    steps = [[("a", n - 1)], [("a", 1)]] if decode else [[("a", n)]]
    got = tf.replay(gpu_engine(d, blocks=80), {"a": toks}, steps)["a"][-1:]
    assert tf.err(got, ref) < 5e-4


@pytest.mark.parametrize("gap", [-1, 0, 1])
@pytest.mark.parametrize("decode", [False, True])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_window_edge(tmp_path, gpu_engine, gap, decode, dtype):
    n, window = 83, 19
    far_pos = (n - 1) - (window - 1) - gap
    cfg, w, d, toks = tm.standout_model(tmp_path, "latent", far_pos, n, window)
    ref = oracle.forward(cfg, w, toks)[-1:]
    steps = [[("a", n - 1)], [("a", 1)]] if decode \
        else [[("a", 40)], [("a", n - 40)]]
    got = tf.replay(gpu_engine(d, dtype=dtype), {"a": toks}, steps)["a"][-1:]
    assert tf.err(got, ref) < (5e-4 if dtype == "float32" else 0.15)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_generation_with_graphs(tmp_path, gpu_engine, dtype):
    """Greedy generation through the scheduler, chunked prefill and the
    captured decode graphs; fp32 must reproduce the oracle's tokens."""
    cfg, w, d = _model(tmp_path, ALIGNED)
    eng = gpu_engine(d, dtype=dtype, blocks=40, max_prefill_tokens=32)
    prompts = [tf.tokens_for(cfg, n, 60 + n) for n in (45, 7, 30)]
    outs = eng.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0,
                                                ignore_eos=True))
    assert all(len(o) == 12 for o in outs)
    if dtype == "float32":
        for p, o in zip(prompts, outs):
            assert o == oracle.greedy(cfg, w, p, 12)
    # a second round re-uses blocks, slots and graphs
    outs2 = eng.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0,
                                                 ignore_eos=True))
    assert outs2 == outs
