"""gpustack_amd.ops — dispatch layer for the CDNA4 HIP kernels.

On a GPU box the in-tree `_hip_ops.so` (hand-written gfx950 kernels) is
REQUIRED: there is no silent eager fallback — a missing extension raises at
first use so a broken build can't masquerade as the native path. On CPU-only
hosts the fp32 torch reference implementations run instead, which keeps the
engine/control-plane logic testable without hardware.
"""
from __future__ import annotations

import os

import torch

from . import torch_ref

_HIP = None
_HIP_ERR: str | None = None


def _load_hip():
    global _HIP, _HIP_ERR
    if _HIP is not None or _HIP_ERR is not None:
        return _HIP
    try:
        import importlib.util
        from pathlib import Path

        so = Path(__file__).resolve().parent / "_hip_ops.so"
        if not so.exists():
            raise ImportError(
                f"{so} not found — build it with `python -m gpustack_amd.ops.build` "
                "(hipcc --offload-arch=gfx950)"
            )
        spec = importlib.util.spec_from_file_location("gpustack_amd.ops._hip_ops", so)
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        _HIP = mod
    except Exception as e:  # noqa: BLE001
        _HIP_ERR = str(e)
        raise
    return _HIP


def hip_available() -> bool:
    if not torch.cuda.is_available():
        return False
    try:
        return _load_hip() is not None
    except Exception:  # noqa: BLE001
        return False


def _backend(t: torch.Tensor):
    if t.is_cuda:
        return _load_hip()  # raises loudly if the native build is missing
    return None


def _oss_kernels_enabled() -> bool:
    """GPT-OSS CDNA4 kernel variants (head_dim-64 + attention sinks +
    sliding window in attn_decode/attn_prefill.hip) are written and
    compile-checked but not yet GPU-validated — opt in explicitly until
    the r3 numerics pass (tests/test_ops_gpu.py oss tests)."""
    return os.environ.get("GPUSTACK_AMD_OSS_KERNELS", "0") == "1"


def _mla_kernel_enabled() -> bool:
    return os.environ.get("GPUSTACK_AMD_MLA_KERNEL", "0") == "1"


def _sinks_f32(sinks):
    if sinks is not None and (sinks.dtype != torch.float32
                              or not sinks.is_contiguous()):
        sinks = sinks.float().contiguous()
    return sinks


# --- op surface -----------------------------------------------------------

def rms_norm(out, x, weight, eps: float) -> None:
    hip = _backend(x)
    if hip is not None:
        hip.rms_norm(out, x, weight, eps)
    else:
        torch_ref.rms_norm(out, x, weight, eps)


def fused_add_rms_norm(x, residual, weight, eps: float) -> None:
    hip = _backend(x)
    if hip is not None:
        hip.fused_add_rms_norm(x, residual, weight, eps)
    else:
        torch_ref.fused_add_rms_norm(x, residual, weight, eps)


def rotary_embedding(positions, q, k, cos_sin, head_dim: int, rot_dim: int,
                     mode: str = "neox") -> None:
    hip = _backend(q)
    if hip is not None:
        if mode != "neox":
            raise NotImplementedError(
                "pairwise (GPT-J style) rotary is not in the CDNA4 kernel "
                "yet (Ernie/Hunyuan/MiniMax GPU serving lands with it in "
                "r3); CPU serving is available")
        hip.rotary_embedding(positions, q, k, cos_sin, head_dim, rot_dim)
    else:
        torch_ref.rotary_embedding(positions, q, k, cos_sin, head_dim,
                                   rot_dim, mode=mode)


def silu_and_mul(out, x) -> None:
    hip = _backend(x)
    if hip is not None:
        hip.silu_and_mul(out, x)
    else:
        torch_ref.silu_and_mul(out, x)


def reshape_and_cache(k, v, k_cache, v_cache, slots) -> None:
    hip = _backend(k)
    if hip is not None:
        hip.reshape_and_cache(k, v, k_cache, v_cache, slots)
    else:
        torch_ref.reshape_and_cache(k, v, k_cache, v_cache, slots)


def greedy_sample_into(out, logits) -> None:
    if logits.is_cuda and logits.dtype == torch.float32:
        # fp32-logit models: whichever fp32-stream library is loaded
        (_PAGED if _PAGED is not None else _load_latent()).argmax_f32(
            out, logits)
        return
    hip = _backend(logits)
    if hip is not None:
        hip.greedy_sample(out, logits)
    else:
        torch_ref.greedy_sample(out, logits)


def greedy_sample(logits) -> torch.Tensor:
    out = torch.empty(logits.shape[0], dtype=torch.long, device=logits.device)
    if logits.is_cuda and logits.dtype == torch.float32:
        _load_latent().argmax_f32(out, logits)  # fp32-logit models
        return out
    hip = _backend(logits)
    if hip is not None:
        hip.greedy_sample(out, logits)
    else:
        torch_ref.greedy_sample(out, logits)
    return out


def paged_attn_decode(out, q, k_cache, v_cache, block_tables, seq_lens,
                      scale: float, sinks=None, window: int = 0,
                      softcap: float = 0.0) -> None:
    hip = _backend(q)
    if hip is not None:
        if (sinks is not None or window or softcap or q.shape[-1] != 128) \
                and not _oss_kernels_enabled():
            # the sinks/window/softcap and D!=128 kernel variants are
            # written but not yet GPU-validated — fail loudly rather than
            # silently mis-attend (opt in with GPUSTACK_AMD_OSS_KERNELS=1;
            # r3 flips the default after the validation pass)
            raise NotImplementedError(
                "sinks/window/softcap/D!=128 CDNA4 decode kernel variants "
                "are unvalidated — set GPUSTACK_AMD_OSS_KERNELS=1 to opt in")
        hip.paged_attn_decode(out, q, k_cache, v_cache, block_tables, seq_lens,
                              scale, sinks=_sinks_f32(sinks), window=window,
                              softcap=softcap)
    else:
        torch_ref.paged_attn_decode(out, q, k_cache, v_cache, block_tables,
                                    seq_lens, scale, sinks=sinks,
                                    window=window, softcap=softcap)


def mla_decode(ctx_out, q_cat, lat_cache, block_tables, seq_lens,
               scale: float) -> None:
    """MLA absorbed decode (DeepSeek): ctx_out[N,H,512] f32 = softmax
    (q_cat · lat) · lat[:, :512] over the paged latent pool. GPU-only —
    the CPU oracle lives in models/llama.py MLAAttention."""
    hip = _backend(q_cat)
    if hip is None:
        raise NotImplementedError("mla_decode is the CDNA4 kernel entry; "
                                  "CPU serving uses the torch MLA path")
    hip.mla_decode(ctx_out, q_cat, lat_cache, block_tables, seq_lens, scale)


_PREFILL_BQ = 64


def build_prefill_tiles(seq_lens: list[int], device) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Map varlen sequences to fixed 64-row q tiles for the MFMA kernel."""
    starts, q0s, lens = [], [], []
    tok = 0
    for L in seq_lens:
        for q0 in range(0, L, _PREFILL_BQ):
            starts.append(tok)
            q0s.append(q0)
            lens.append(L)
        tok += L
    mk = lambda a: torch.tensor(a, dtype=torch.int32, device=device)
    return mk(starts), mk(q0s), mk(lens)


def varlen_prefill_attn(out, q, k, v, seq_lens: list[int], scale: float,
                        tiles=None, sinks=None, window: int = 0,
                        softcap: float = 0.0) -> None:
    hip = _backend(q)
    if hip is not None:
        d_ok = (q.shape[-1] == 128
                or (q.shape[-1] == 192 and _mla_kernel_enabled()))
        if (sinks is not None or window or softcap or not d_ok) \
                and not _oss_kernels_enabled():
            raise NotImplementedError(
                "sinks/window/softcap/D!=128 CDNA4 prefill kernel variants "
                "are unvalidated — set GPUSTACK_AMD_OSS_KERNELS=1 (or "
                "GPUSTACK_AMD_MLA_KERNEL=1 for the 192/128 MLA expand "
                "shape) to opt in")
        if tiles is None or tiles[0] is None:
            tiles = build_prefill_tiles(seq_lens, q.device)
        hip.flash_prefill(out, q, k, v, tiles[0], tiles[1], tiles[2], scale,
                          sinks=_sinks_f32(sinks), window=window,
                          softcap=softcap)
    else:
        torch_ref.varlen_prefill_attn(out, q, k, v, seq_lens, scale,
                                      sinks=sinks, window=window,
                                      softcap=softcap)


def build_paged_prefill_tiles(seq_starts: list[int], seq_hists: list[int],
                              seq_news: list[int], device):
    """Map per-seq suffix rows to fixed 64-row q tiles for the paged
    prefill-with-history kernel (one entry set per (seq, q-tile))."""
    qstart, q0s, hists, news, seqi = [], [], [], [], []
    for i, (st, h, n) in enumerate(zip(seq_starts, seq_hists, seq_news)):
        for q0 in range(0, n, _PREFILL_BQ):
            qstart.append(st)
            q0s.append(q0)
            hists.append(h)
            news.append(n)
            seqi.append(i)
    mk = lambda a: torch.tensor(a, dtype=torch.int32, device=device)
    return mk(qstart), mk(q0s), mk(hists), mk(news), mk(seqi)


def paged_prefill_attn(out, q, k_cache, v_cache, block_tables,
                       seq_starts: list[int], seq_hists: list[int],
                       seq_news: list[int], scale: float, tiles=None,
                       sinks=None, window: int = 0,
                       softcap: float = 0.0) -> None:
    """Prefill-with-history: suffix/chunk rows attend to cached paged KV +
    their own freshly written positions through the MFMA flash kernel
    (removes the r1-measured ~3.5x paged-decode-row penalty)."""
    hip = _backend(q)
    if hip is not None:
        if (sinks is not None or window or softcap or q.shape[-1] != 128) \
                and not _oss_kernels_enabled():
            raise NotImplementedError(
                "sinks/window/softcap/D!=128 CDNA4 paged-prefill kernel "
                "variants are unvalidated — set GPUSTACK_AMD_OSS_KERNELS=1 "
                "to opt in")
        if tiles is None:
            tiles = build_paged_prefill_tiles(seq_starts, seq_hists,
                                              seq_news, q.device)
        hip.flash_prefill_paged(out, q, k_cache, v_cache, block_tables,
                                tiles[0], tiles[1], tiles[2], tiles[3],
                                tiles[4], scale, sinks=_sinks_f32(sinks),
                                window=window, softcap=softcap)
    else:
        torch_ref.paged_prefill_attn(out, q, k_cache, v_cache, block_tables,
                                     seq_starts, seq_hists, seq_news, scale,
                                     sinks=sinks, window=window,
                                     softcap=softcap)


_SG_WORKSPACES: dict = {}


def gemm8(x, w, out=None, safe: bool = False):
    """8-phase pipelined 256x256 MFMA GEMM: out[M,N] = x[M,K] @ w[N,K]^T
    (bf16, f32 accumulate). GPU-only; requires N%256==0, K%128==0 —
    falls back to F.linear otherwise. `safe=True` runs the fully-drained
    variant (race isolation for tests)."""
    import torch.nn.functional as F

    M, K = x.shape
    N = w.shape[0]
    if not x.is_cuda or N % 256 != 0 or K % 128 != 0:
        return F.linear(x, w, None)
    if out is None:
        out = torch.empty(M, N, dtype=x.dtype, device=x.device)
    hip = _backend(x)
    if hip is None:
        return F.linear(x, w, None)
    hip.gemm8(out, x.contiguous(), w, 1 if safe else 0)
    return out


def skinny_gemm(x, w, out=None, splitk: int | None = None, version: int = 1):
    """Split-K decode GEMM: out[M,N] = x[M,K] @ w[N,K]^T (bf16, f32 acc).
    GPU-only (falls back to F.linear elsewhere or for unsupported shapes)."""
    import torch.nn.functional as F

    M, K = x.shape
    N = w.shape[0]
    if not x.is_cuda or N % 128 != 0 or K % 64 != 0:
        return F.linear(x, w, None)
    if splitk is None:
        mt = (M + 255) // 256
        nt = N // 128
        splitk = 1
        while (mt * nt * splitk < 400 and splitk < 8
               and K % (64 * splitk * 2) == 0):
            splitk *= 2
    if out is None:
        out = torch.empty(M, N, dtype=x.dtype, device=x.device)
    ws = None
    if splitk > 1:
        key = (splitk, M, N, x.device.index)
        ws = _SG_WORKSPACES.get(key)
        if ws is None:
            ws = torch.empty(splitk * M * N, dtype=torch.float32, device=x.device)
            _SG_WORKSPACES[key] = ws
    _load_hip().skinny_gemm(out, x, w, ws, splitk, version)
    return out


def linear_auto(x, w):
    """Shape-gated GEMM dispatch: the split-K skinny kernel where it
    measured faster than hipBLASLt (scripts/bench_skinny_gemm.py on
    MI355X: down_proj-like N=4096 K>=8192 M>=384 at splitk=4, 824 TF vs
    hipBLASLt 680), F.linear everywhere else."""
    import os

    import torch.nn.functional as F

    if (x.is_cuda and x.dim() == 2
            and os.environ.get("GPUSTACK_AMD_SKINNY_GEMM", "1") == "1"):
        M, K = x.shape
        N = w.shape[0]
        if (N == 4096 and K >= 8192 and 384 <= M <= 1024
                and K % 256 == 0 and x.stride(1) == 1):
            return skinny_gemm(x, w, splitk=4)
    return F.linear(x, w)


def mfma_probe(a, b):
    return _load_hip().mfma_probe(a, b)


build_cos_sin_cache = torch_ref.build_cos_sin_cache


# --- fp32-residual op family ------------------------------------------------
# Kernels for models that keep the residual stream, norms, attention scores
# and routers in fp32 (ModelSpec.fp32_residual): ops/csrc/resid32.hip and
# ops/csrc/latent_attn.hip, built into their own small extension so a
# checkout that serves only such a model compiles nothing else. Activations
# entering GEMMs are bf16 or fp32 (the engine dtype); every kernel is
# instantiated for both.

_LATENT = None
_PAGED = None


def _load_paged():
    """Load `_hip_paged.so` (row kernels of the pre/post-norm fp32 stream
    and paged rotary attention), compiling it in-tree first when no built
    library is there."""
    global _PAGED
    if _PAGED is not None:
        return _PAGED
    import importlib.util

    from .build import PAGED_SO_PATH, build_paged

    if not PAGED_SO_PATH.exists():
        build_paged()
    spec = importlib.util.spec_from_file_location(
        "gpustack_amd.ops._hip_paged", PAGED_SO_PATH)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    _PAGED = mod
    return mod


def _paged_backend(t: torch.Tensor):
    return _load_paged() if t.is_cuda else None


def _load_latent():
    """Load `_hip_latent.so`, compiling it in-tree first when no built
    library is there (a fresh checkout on a GPU box)."""
    global _LATENT
    if _LATENT is not None:
        return _LATENT
    import importlib.util

    from .build import LATENT_SO_PATH, build_latent

    if not LATENT_SO_PATH.exists():
        build_latent()
    spec = importlib.util.spec_from_file_location(
        "gpustack_amd.ops._hip_latent", LATENT_SO_PATH)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    _LATENT = mod
    return mod


def _lat_backend(t: torch.Tensor):
    return _load_latent() if t.is_cuda else None


ACT_MODES = {"relu2": 0, "gelu": 1, "gelu_tanh": 2, "silu": 3}


def embed_pair_hash(x, h, tokens, prev, embed, pair_table, buckets: int,
                    mul_prev: int, mul_cur: int) -> None:
    k = _lat_backend(x)
    if k is not None:
        k.embed_pair_hash(x, h, tokens, prev, embed, pair_table,
                          buckets, mul_prev, mul_cur)
    else:
        torch_ref.embed_pair_hash(x, h, tokens, prev, embed, pair_table,
                                  buckets, mul_prev, mul_cur)


def rms_scale_add(x, a, weight, scale, eps: float, h) -> None:
    k = _lat_backend(x)
    if k is not None:
        k.rms_scale_add(x, a, weight, scale, eps, h)
    else:
        torch_ref.rms_scale_add(x, a, weight, scale, eps, h)


def rms_norm_f32(out, x, weight, eps: float) -> None:
    k = _lat_backend(x)
    if k is not None:
        k.rms_norm_f32(out, x, weight, eps)
    else:
        torch_ref.rms_norm_f32(out, x, weight, eps)


def latent_norm_store(cache, src, col0: int, weight, slots, eps: float) -> None:
    k = _lat_backend(src)
    if k is not None:
        k.latent_norm_store(cache, src, col0, weight, slots, eps)
    else:
        torch_ref.latent_norm_store(cache, src, col0, weight, slots, eps)


_LAT_GROUP = 16   # (row, head) pairs sharing one key stream per workgroup


def build_latent_tiles(seq_starts, seq_hists, seq_news, heads: int, device):
    """Group the batch's (row, head) pairs into tiles of at most 16 pairs
    that belong to ONE sequence, so a workgroup streams that sequence's
    latents once for all of them. Long portions tile as 16 rows x 1 head;
    short ones (decode rows above all) pack rows x heads. Returns int32
    [ntiles, 6]: row0, nrows, head0, nheads, seq, pos0."""
    import numpy as np

    G = _LAT_GROUP
    parts = []
    for i, (st, hist, new) in enumerate(zip(seq_starts, seq_hists, seq_news)):
        if new >= G:
            nh, nr = 1, G
        else:
            nh = min(heads, G)
            nr = max(1, min(new, G // nh))
        r0 = np.arange(0, new, nr, dtype=np.int32)
        h0 = np.arange(0, heads, nh, dtype=np.int32)
        rr, hh = np.meshgrid(r0, h0, indexing="ij")
        rr, hh = rr.reshape(-1), hh.reshape(-1)
        t = np.empty((rr.size, 6), dtype=np.int32)
        t[:, 0] = st + rr
        t[:, 1] = np.minimum(nr, new - rr)
        t[:, 2] = hh
        t[:, 3] = np.minimum(nh, heads - hh)
        t[:, 4] = i
        t[:, 5] = hist + rr
        parts.append(t)
    tiles = (np.concatenate(parts) if parts
             else np.empty((0, 6), dtype=np.int32))
    return torch.from_numpy(tiles).to(device)


def latent_attention_mfma_ok(cache) -> bool:
    """True when ops.latent_attention takes the MFMA kernel for this pool:
    bf16, both page planes, 16-token pages, width % 32 == 0 (<= 1024). Only
    then may q_lat / ctx be bf16 and arbitrarily strided."""
    return (cache.is_cuda and cache.dtype == torch.bfloat16
            and cache.shape[1] == 2 and cache.shape[2] == 16
            and cache.shape[3] % 32 == 0 and cache.shape[3] <= 1024)


def latent_attention(ctx, q_lat, cache, block_tables, row_seq, positions,
                     scale: float, tiles=None, exact: bool = False,
                     max_ctx: int = 0) -> None:
    """ctx / q_lat: [T, H, R] views (last axis contiguous). `exact` forces
    the fp32 vector-ALU kernel where the MFMA kernel would run. `max_ctx`
    (longest context in the batch, a host number) lets a batch of few tiles
    over long contexts split each tile's keys over several workgroups."""
    k = _lat_backend(q_lat)
    if k is not None:
        if tiles is None:
            raise ValueError("latent_attention on GPU needs the tile list "
                             "(build_latent_tiles)")
        nsplit = 1
        nt = tiles.shape[0]
        if not exact and max_ctx >= 512 and 0 < nt < 512:
            nsplit = max(1, min(16, 1024 // nt, max_ctx // 128))
        k.latent_attention(ctx, q_lat, cache, block_tables, tiles, positions,
                           scale, exact, nsplit)
    else:
        torch_ref.latent_attention(ctx, q_lat, cache, block_tables, row_seq,
                                   positions, scale)


def act_inplace(x, mode: str) -> None:
    # the kernel ships in both fp32-stream libraries: whichever is loaded
    k = _PAGED if (_PAGED is not None and x.is_cuda) else _lat_backend(x)
    if k is not None:
        k.act_inplace(x, ACT_MODES[mode])
    else:
        torch_ref.act_inplace(x, mode)


def route_grouped_topk(experts, weights, logits, n_experts: int, groups: int,
                       keep: int, scale: float) -> None:
    k = _lat_backend(logits)
    if k is not None:
        k.route_grouped_topk(experts, weights, logits, n_experts, groups,
                             keep, scale)
    else:
        torch_ref.route_grouped_topk(experts, weights, logits, n_experts,
                                     groups, keep, scale)


def moe_combine(out, y, inv, weights, shared, gate_logits, gate_col: int) -> None:
    k = _lat_backend(out)
    if k is not None:
        k.moe_combine(out, y, inv, weights, shared, gate_logits, gate_col)
    else:
        torch_ref.moe_combine(out, y, inv, weights, shared, gate_logits,
                              gate_col)


def grouped_ff_available(x, width: int, ff: int) -> bool:
    """The sync-free grouped expert kernels take bf16 on the GPU with
    width % 64 == 0 and ff % 64 == 0."""
    return (x.is_cuda and x.dtype == torch.bfloat16
            and width % 64 == 0 and ff % 64 == 0)


def grouped_up_act(u, x, up_w, s_tok, offs, counts, mode: str) -> None:
    _load_latent().grouped_up_act(u, x, up_w, s_tok, offs, counts,
                                  ACT_MODES[mode])


def grouped_down(y, u, down_w, offs, counts) -> None:
    _load_latent().grouped_down(y, u, down_w, offs, counts)


def softcap_(logits, cap: float) -> None:
    k = _lat_backend(logits)
    if k is not None:
        k.softcap(logits, cap)
    else:
        torch_ref.softcap_(logits, cap)


# --- pre/post-norm fp32 stream + paged rotary attention -------------------
# ops/csrc/rowmix32.hip and ops/csrc/ragged_attn.hip in `_hip_paged.so`.

def embed_rows_f32(x, tokens, embed) -> None:
    k = _paged_backend(x)
    if k is not None:
        k.embed_rows_f32(x, tokens, embed)
    else:
        torch_ref.embed_rows_f32(x, tokens, embed)


def rms_norm_rows(out, x, weight, eps: float) -> None:
    """fp32 rows -> weighted RMS norm in out's dtype."""
    k = _paged_backend(x)
    if k is not None:
        k.sandwich_add_norm(x, None, None, 0.0, eps, None, weight, out)
    else:
        torch_ref.rms_norm_f32(out, x, weight, eps)


def sandwich_add_norm(x, a, post_w, mult: float, eps: float, extra, next_w,
                      h, center: bool = False) -> None:
    """`center`: both norms are weight-only layer norms (the mean comes off
    first) instead of RMS norms."""
    k = _paged_backend(x)
    if k is not None:
        k.sandwich_add_norm(x, a, post_w, mult, eps, extra, next_w, h, center)
    else:
        torch_ref.sandwich_add_norm(x, a, post_w, mult, eps, extra, next_w, h,
                                    center)


def build_page_groups(seq_starts, seq_hists, seq_news, block_size: int,
                      device):
    """Runs of batch rows that fall into ONE cache page in order, for
    page-wise value stores: int32 [n, 2] = first row, rows. A sequence that
    brings rows for positions hist..hist+new-1 is cut at multiples of the
    page size."""
    import numpy as np

    parts = []
    for st, hist, new in zip(seq_starts, seq_hists, seq_news):
        first = np.arange(hist - hist % block_size, hist + new, block_size)
        lo = np.maximum(first, hist)
        hi = np.minimum(first + block_size, hist + new)
        parts.append(np.stack([st + lo - hist, hi - lo], axis=1))
    g = (np.concatenate(parts) if parts else np.empty((0, 2))).astype(np.int32)
    return torch.from_numpy(g).to(device)


def rotary_norm_store(q_out, qkv, nq: int, nk: int, q_norm_w, k_norm_w,
                      inv_freq, pos32, head_dim: int, k_cache, v_cache, slots,
                      eps: float, tied: bool, page_groups=None) -> None:
    """`page_groups` (build_page_groups; GPU, prompts): the value rows are
    written page by page instead of row by row."""
    k = _paged_backend(qkv)
    if k is not None:
        k.rotary_norm_store(q_out, qkv, nq, nk, q_norm_w, k_norm_w, inv_freq,
                            pos32, head_dim, k_cache, v_cache, slots, eps,
                            tied, page_groups)
    else:
        torch_ref.rotary_norm_store(q_out, qkv, nq, nk, q_norm_w, k_norm_w,
                                    inv_freq, pos32, head_dim, k_cache,
                                    v_cache, slots, eps, tied)


_ATT_GROUP = 16   # (row, score map) pairs sharing one key stream per workgroup


def build_attn_tiles(seq_starts, seq_hists, seq_news, heads: int,
                     kv_heads: int, maps: int, device):
    """Group the batch's (row, score map) pairs into tiles of at most 16
    pairs that share ONE key stream: same sequence, same kv head, same map.
    Long portions tile as 16 rows x 1 query head; short ones (decode rows
    above all) pack rows x the query heads of a kv group. Score map a =
    head * maps + map, so the heads of one kv group and one map are `maps`
    apart. Returns int32 [ntiles, 6]: row0, nrows, a0, n_a, seq, a_step."""
    import numpy as np

    G = _ATT_GROUP
    rep = heads // kv_heads
    parts = []
    for i, (st, hist, new) in enumerate(zip(seq_starts, seq_hists, seq_news)):
        if new >= G or rep == 1:
            nh, nr = 1, G
        else:
            nh = min(rep, G)
            nr = max(1, min(new, G // nh))
        r0 = np.arange(0, new, nr, dtype=np.int32)
        # first score map of every (kv head, chunk of nh heads, map)
        g0 = np.arange(0, rep, nh, dtype=np.int32)
        a0 = ((np.arange(kv_heads, dtype=np.int32)[:, None, None] * rep
               + g0[None, :, None]) * maps
              + np.arange(maps, dtype=np.int32)[None, None, :])
        na = np.broadcast_to(np.minimum(nh, rep - g0)[None, :, None],
                             a0.shape).reshape(-1)
        a0 = a0.reshape(-1)
        rr, ai = np.meshgrid(r0, np.arange(a0.size), indexing="ij")
        rr, ai = rr.reshape(-1), ai.reshape(-1)
        t = np.empty((rr.size, 6), dtype=np.int32)
        t[:, 0] = st + rr
        t[:, 1] = np.minimum(nr, new - rr)
        t[:, 2] = a0[ai]
        t[:, 3] = na[ai]
        t[:, 4] = i
        t[:, 5] = maps
        parts.append(t)
    tiles = (np.concatenate(parts) if parts
             else np.empty((0, 6), dtype=np.int32))
    return torch.from_numpy(tiles).to(device)


def paged_attention(out, q, k_cache, v_cache, block_tables, row_seq, positions,
                    scale: float, maps: int = 1, window: int = 0,
                    keep_first: int = 0, sinks=None, tiles=None,
                    exact: bool = False, max_ctx: int = 0,
                    slopes=None, softcap: float = 0.0) -> None:
    """q: [T, A, D], out: [T, A, VW] (A = heads * maps score maps; views
    whose last axis is contiguous). On the
    GPU the MFMA kernel runs for bf16 pools of fitting sizes, the fp32
    vector-ALU kernel otherwise (always for fp32 pools, or with `exact`).
    `max_ctx` (longest context in the batch, a host number) lets a batch of
    few tiles over long contexts split each tile's keys over workgroups.
    `slopes` (fp32, per head): slope * distance is taken off every scaled
    score. `softcap` > 0: scaled scores pass softcap * tanh(s / softcap)."""
    k = _paged_backend(q)
    if k is not None:
        if tiles is None:
            raise ValueError("paged_attention on GPU needs the tile list "
                             "(build_attn_tiles)")
        nsplit = 1
        nt = tiles.shape[0]
        span = min(max_ctx, window + keep_first) if window > 0 else max_ctx
        if span >= 512 and 0 < nt < 2048:
            # 1024 workgroups, or up to 2048 while the split stays <= 4 (a
            # wider split pays more for the merge than it gains in
            # occupancy), each of at least 128 keys
            nsplit = max(1, min(16, span // 128,
                                max(1024 // nt, min(4, 2048 // nt))))
        k.paged_attention(out, q, k_cache, v_cache, block_tables, tiles,
                          positions, scale, maps, window, keep_first, sinks,
                          exact, nsplit, slopes, softcap)
    else:
        torch_ref.paged_attention(out, q, k_cache, v_cache, block_tables,
                                  row_seq, positions, scale, maps, window,
                                  keep_first, sinks, slopes, softcap)


def head_rope_store(q_out, src, col_q: int, q_heads: int, q_dim: int, q_w,
                    q_norm_dims: int, q_rot0: int, col_k: int, k_heads: int,
                    k_dim: int, k_w, k_norm_dims: int, k_rot0: int, col_v: int,
                    inv_freq, half_layout: bool, amplitude: float, pos32,
                    k_cache, v_cache, slots, eps: float,
                    page_groups=None) -> None:
    """Per-head norm + rotation + cache write (torch_ref.head_rope_store
    has the semantics). `page_groups` (build_page_groups; GPU, prompts,
    values read from src): the value rows are written page by page."""
    k = _paged_backend(src)
    if k is not None:
        k.head_rope_store(q_out, src, col_q, q_heads, q_dim, q_w, q_norm_dims,
                          q_rot0, col_k, k_heads, k_dim, k_w, k_norm_dims,
                          k_rot0, col_v, inv_freq, half_layout, amplitude,
                          pos32, k_cache, v_cache, slots, eps, page_groups)
    else:
        torch_ref.head_rope_store(q_out, src, col_q, q_heads, q_dim, q_w,
                                  q_norm_dims, q_rot0, col_k, k_heads, k_dim,
                                  k_w, k_norm_dims, k_rot0, col_v, inv_freq,
                                  half_layout, amplitude, pos32, k_cache,
                                  v_cache, slots, eps)


def dual_rms_mix(out, a, wa, b, wb, eps: float) -> None:
    k = _paged_backend(a)
    if k is not None:
        k.dual_rms_mix(out, a, wa, b, wb, eps)
    else:
        torch_ref.dual_rms_mix(out, a, wa, b, wb, eps)


def head_gate(out, o_hts, gate_src, col: int) -> None:
    k = _paged_backend(o_hts)
    if k is not None:
        k.head_gate(out, o_hts, gate_src, col)
    else:
        torch_ref.head_gate(out, o_hts, gate_src, col)


def diff_combine(out, a, lam, diff: float, eps: float) -> None:
    k = _paged_backend(a)
    if k is not None:
        k.diff_combine(out, a, lam, diff, eps)
    else:
        torch_ref.diff_combine(out, a, lam, diff, eps)


def act_and_mul(out, gu, mode: str) -> None:
    k = _paged_backend(gu)
    if k is not None:
        k.act_and_mul(out, gu, ACT_MODES[mode])
    else:
        torch_ref.act_and_mul(out, gu, mode)


# --- layer-norm fp32 stream, attention without rotation, recurrent mixers ---
# ops/csrc/lnrows32.hip and ops/csrc/state_scan.hip in `_hip_state.so`.

_STATE = None


def _load_state():
    """Load `_hip_state.so` (layer-norm row kernels, head-norm cache write,
    short convolution, matrix-state scan, gated norms, scored routing),
    compiling it in-tree first when no built library is there."""
    global _STATE
    if _STATE is not None:
        return _STATE
    import importlib.util

    from .build import STATE_SO_PATH, build_state

    if not STATE_SO_PATH.exists():
        build_state()
    spec = importlib.util.spec_from_file_location(
        "gpustack_amd.ops._hip_state", STATE_SO_PATH)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    _STATE = mod
    return mod


def _state_backend(t: torch.Tensor):
    return _load_state() if t.is_cuda else None


def embed_rows_scaled(x, tokens, embed, scale: float) -> None:
    k = _state_backend(x)
    if k is not None:
        k.embed_rows_scaled(x, tokens, embed, scale)
    else:
        torch_ref.embed_rows_scaled(x, tokens, embed, scale)


def add_layer_norm(x, a, w, b, eps: float, h) -> None:
    k = _state_backend(x)
    if k is not None:
        k.add_layer_norm(x, a, w, b, eps, h)
    else:
        torch_ref.add_layer_norm(x, a, w, b, eps, h)


def head_norm_store(q_out, qkv, nq: int, nk: int, q_w, k_w, head_dim: int,
                    temp_coef: float, temp_every: float, pos32, v_first, lam,
                    k_cache, v_cache, slots, eps: float,
                    page_groups=None) -> None:
    """`page_groups` (build_page_groups; GPU, prompts): the value rows are
    written page by page instead of row by row."""
    k = _state_backend(qkv)
    if k is not None:
        k.head_norm_store(q_out, qkv, nq, nk, q_w, k_w, head_dim, temp_coef,
                          temp_every, pos32, v_first, lam, k_cache, v_cache,
                          slots, eps, page_groups)
    else:
        torch_ref.head_norm_store(q_out, qkv, nq, nk, q_w, k_w, head_dim,
                                  temp_coef, temp_every, pos32, v_first, lam,
                                  k_cache, v_cache, slots, eps)


def causal_conv_silu(out, src, col0: int, w, b, conv_state, seq_first,
                     seq_rows, state_slots, row_seq, pos32) -> None:
    k = _state_backend(src)
    if k is not None:
        k.causal_conv_silu(out, src, col0, w, b, conv_state, seq_first,
                           seq_rows, state_slots, row_seq, pos32)
    else:
        torch_ref.causal_conv_silu(out, src, col0, w, b, conv_state,
                                   seq_first, seq_rows, state_slots, pos32)


def state_scan(y, src, col_x: int, col_b: int, col_c: int, dt_src,
               col_dt: int, heads: int, groups: int, n_state: int, vdim: int,
               act_silu: bool, dt_bias, a_log, skip, decay, state, seq_first,
               seq_rows, state_slots, pos32, single: bool = False) -> None:
    """`single` (a host-side hint): every sequence brings one row, as in a
    decode step; the GPU then streams the states through its step kernel."""
    k = _state_backend(src)
    if k is not None:
        k.state_scan(y, src, col_x, col_b, col_c, dt_src, col_dt, heads,
                     groups, n_state, vdim, act_silu, dt_bias, a_log, skip,
                     decay, state, seq_first, seq_rows, state_slots, pos32,
                     single)
    else:
        torch_ref.state_scan(y, src, col_x, col_b, col_c, dt_src, col_dt,
                             heads, groups, n_state, vdim, act_silu, dt_bias,
                             a_log, skip, decay, state, seq_first, seq_rows,
                             state_slots, pos32)


def gated_group_norm(out, y, gate, w, groups: int, eps: float,
                     gate_first) -> None:
    """gate_first: True / 1 = silu gate, then norm; False / 0 = norm, then
    sigmoid gate; 2 = norm, then silu gate."""
    k = _state_backend(y)
    if k is not None:
        k.gated_group_norm(out, y, gate, w, groups, eps, int(gate_first))
    else:
        torch_ref.gated_group_norm(out, y, gate, w, groups, eps, gate_first)


def route_topk(experts, weights, logits, correction, n_experts: int,
               groups: int, keep: int, group_top: int, sigmoid: bool,
               renorm: bool, scale: float) -> None:
    k = _state_backend(logits)
    if k is not None:
        k.route_topk(experts, weights, logits, correction, n_experts, groups,
                     keep, group_top, sigmoid, renorm, scale)
    else:
        torch_ref.route_topk(experts, weights, logits, correction, n_experts,
                             groups, keep, group_top, sigmoid, renorm, scale)


def delta_scan(y, src, col_q: int, col_k: int, col_v: int, gate_src,
               col_a: int, col_b: int, heads: int, groups: int, n_state: int,
               vdim: int, dt_bias, a_log, state, seq_first, seq_rows,
               state_slots, pos32, single: bool = False) -> None:
    """Gated delta rule over the state pool (torch_ref.delta_scan has the
    semantics). `single`: every sequence brings one row (a decode step)."""
    k = _state_backend(src)
    if k is not None:
        k.delta_scan(y, src, col_q, col_k, col_v, gate_src, col_a, col_b,
                     heads, groups, n_state, vdim, dt_bias, a_log, state,
                     seq_first, seq_rows, state_slots, pos32, single)
    else:
        torch_ref.delta_scan(y, src, col_q, col_k, col_v, gate_src, col_a,
                             col_b, heads, groups, n_state, vdim, dt_bias,
                             a_log, state, seq_first, seq_rows, state_slots,
                             pos32)
