"""Engine + model configuration for the first-party CDNA4 inference engine.

ModelSpec mirrors the fields the reference reads out of HF config.json via
AutoConfig (reference: gpustack/scheduler/scheduler.py:216 evaluation path);
we parse config.json directly so random-init serving needs no checkpoint.
"""
from __future__ import annotations

import json
from dataclasses import dataclass, field
from pathlib import Path


@dataclass(frozen=True)
class LatentMixerSpec:
    """Position-free latent attention (models/latent_attention.py): keys
    and values of every head are linear images of ONE normalised latent of
    width kv_rank per token, which is all the paged cache holds."""
    heads: int
    qk_dim: int
    v_dim: int
    kv_rank: int
    scale: float
    # the rotary variant (models/latent_attention.py RotaryLatentAttention):
    # rot_dim > 0 adds a rotated part to every query head and ONE rotated
    # key part per token shared by all heads, cached beside the latent;
    # q_rank > 0 sends the queries through a normed latent of their own;
    # window > 0: a row sees the last `window` positions, itself included;
    # sink: a learned logit per head joins the softmax denominator;
    # out_gate: each head's output times a sigmoid gate read from the
    # mixer's input; kv_from >= 0: no down-projection and no pool of its
    # own — the layer reads the latent and rotated key part that layer
    # `kv_from` cached
    rot_dim: int = 0
    rot: "RotarySpec | None" = None
    q_rank: int = 0
    window: int = 0
    sink: bool = False
    out_gate: bool = False
    kv_from: int = -1


@dataclass(frozen=True)
class RotarySpec:
    """Rotary positions on the first `dims` channels of a head, the pair i
    turning by pos * f_i, f_i = base^(-2i/dims). `layout` "pairs": channel
    2i pairs with 2i+1; "half": channel i pairs with i + dims/2. Optional
    wavelength-dependent frequency scaling, one of
    * `scaling` (factor, low, high, original): long waves slowed by
      `factor`, short ones kept, a linear blend in the wavelength between;
    * `ramp` (factor, original, fast, slow): the blend is linear in the
      CHANNEL index between the channels that make `fast` and `slow` turns
      over `original` positions, and cos / sin are multiplied by
      `amplitude` = 0.1 ln(factor) + 1."""
    dims: int = 0
    base: float = 10000.0
    scaling: tuple | None = None        # (factor, low, high, original)
    layout: str = "pairs"               # "pairs" | "half"
    ramp: tuple | None = None           # (factor, original, fast, slow)

    @property
    def amplitude(self) -> float:
        import math

        return 0.1 * math.log(self.ramp[0]) + 1.0 if self.ramp else 1.0

    def inv_freq(self) -> list[float]:
        """f_i for i < dims/2, in double precision."""
        import math

        out = []
        if self.ramp is not None:
            factor, orig, fast, slow = self.ramp

            def chan(turns):
                return (self.dims * math.log(orig / (2.0 * math.pi * turns))
                        / (2.0 * math.log(self.base)))

            lo = max(math.floor(chan(fast)), 0)
            hi = min(math.ceil(chan(slow)), self.dims - 1)
        for i in range(self.dims // 2):
            f = self.base ** (-2.0 * i / self.dims)
            if self.ramp is not None:
                r = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
                f = f / factor * r + f * (1.0 - r)
            if self.scaling is not None:
                factor, low, high, orig = self.scaling
                wave = 2.0 * math.pi / f
                if wave > orig / low:
                    f = f / factor
                elif wave >= orig / high:
                    s = (orig / wave - low) / (high - low)
                    f = (1.0 - s) * f / factor + s * f
            out.append(f)
        return out


@dataclass(frozen=True)
class PagedMixerSpec:
    """Rotary softmax attention over a paged key/value pool
    (models/paged_attention.py). Every option is a parameter:

    * maps = 2: differential attention — q and k carry two score maps per
      head (a head's two maps adjacent, heads in order), both weight the same values, and
      the head's output is a1 - lambda * a2, unit-RMS-normalised and scaled
      by (1 - diff); lambda = exp(lq1.lk1) - exp(lq2.lk2) + diff.
    * window > 0: a row sees keys closer than `window` plus the first
      `keep_first` keys of its sequence, whose positions stay what they are.
    * sink: one learned logit per head joins the softmax denominator.
    * qk_norm_full: weighted RMS norm over the whole q (and k) projection,
      before rotation.
    * tied_values: no value projection of its own; the raw key projection
      (neither normed nor rotated) serves as the value.
    * head_norm: weighted RMS norm of every q and k head over its own
      channels, one weight vector of head size shared by all heads.
    * q_temp = (coef, every): the query at position p is multiplied by
      1 + coef * ln(floor((p + 1) / every) + 1).
    * distance_bias: slope_h * (i - j) is taken off the scaled score of
      query i and key j, slope_h = 2^(-8 (h + 1) / heads).
    * v_mix: the layer's values blend with the values the FIRST such layer
      of the stack computed for the same token, v <- (1 - l) v + l v_first
      with one learned l per layer; the blend is what the pool keeps.
    * softcap > 0: the scaled score s becomes softcap * tanh(s / softcap).
    * head_norm together with a rotation (rot.dims > 0) and biases: the
      per-head norm comes first, then the rotation."""
    heads: int
    kv_heads: int
    qk_dim: int
    v_dim: int
    scale: float
    rot: RotarySpec = RotarySpec()
    bias: bool = False
    maps: int = 1
    diff: float = 0.0
    window: int = 0
    keep_first: int = 0
    sink: bool = False
    qk_norm_full: bool = False
    tied_values: bool = False
    head_norm: bool = False
    q_temp: tuple | None = None         # (coef, every)
    distance_bias: bool = False
    v_mix: bool = False
    softcap: float = 0.0

    def slopes(self) -> list[float]:
        """Distance-bias slope of every head, in double precision."""
        return [2.0 ** (-8.0 * (h + 1) / self.heads)
                for h in range(self.heads)]

    @property
    def k_width(self) -> int:           # cached key channels per kv head
        return self.maps * self.qk_dim

    @property
    def v_width(self) -> int:
        return self.qk_dim if self.tied_values else self.v_dim


@dataclass(frozen=True)
class ScanMixerSpec:
    """Recurrent mixer with one matrix state per head and sequence
    (models/state_mixers.py), S_t = a_t S_(t-1) + b_t k_t v_t^T, y_t = S_t^T
    q_t (+ skip * v_t), the state [state x vdim] kept in fp32 in a slot of
    the engine's state pool.

    * kind "mamba2": a_t = exp(-exp(A_log) * dt_t), b_t = dt_t with dt_t =
      softplus(dt + dt_bias) per head and token; k / q (B / C) are shared
      by the heads of a group; v (x), B and C pass a causal convolution of
      `conv` taps per channel and SiLU first; a per-head skip D; the output
      is gated by silu(z), then RMS-normed in `norm_groups` parts.
    * kind "lightning": a_t = decay[h] (constants), b_t = 1, q / k / v are
      SiLU of their projections (one k and q per head); the output is
      RMS-normed over all heads, then multiplied by a sigmoid gate.
    * kind "delta" (gated delta rule): S <- g_t S; u = beta_t (v_t - S^T
      k_t); S <- S + k_t u^T; y_t = S^T q_t with g_t = exp(-exp(A_log) *
      softplus(a_t + dt_bias)) and beta_t = sigmoid(b_t) per head and token;
      q, k (shared by the heads of a group) and v pass a causal convolution
      of `conv` taps and SiLU, then q and k are scaled to unit length (q
      also by state^(-1/2)); each head's output is RMS-normed, weighted and
      multiplied by a SiLU gate."""
    kind: str
    heads: int
    state: int                          # rows of the state = size of k and q
    vdim: int
    groups: int = 0                     # k/q groups (mamba2); heads otherwise
    conv: int = 0                       # taps of the causal convolution
    norm_groups: int = 1
    decay: tuple | None = None

    @property
    def inner(self) -> int:
        return self.heads * self.vdim

    @property
    def conv_channels(self) -> int:     # x | B | C
        return (self.inner + 2 * self.groups * self.state) if self.conv else 0


@dataclass(frozen=True)
class ParallelMixerSpec:
    """Two mixers side by side on the same input (models/parallel_mixer.py):
    softmax attention over the paged pool and a recurrent matrix-state
    mixer; each output is RMS-normed over the model width with its own
    weight and the two are averaged."""
    left: PagedMixerSpec
    right: ScanMixerSpec


@dataclass(frozen=True)
class FeedForwardSpec:
    """Feed-forward W_down act(W_up h) — with `gated`, W_down (act(W_gate h)
    * W_up h) — dense or as a bank of routed experts (models/experts.py). Routing: softmax scores over all
    experts, group-limited top-k (groups of neighbouring experts ranked by
    their best member, keep_groups stay eligible), weights = score *
    route_scale without renormalisation; shared_ff > 0 adds an always-on
    expert scaled by a per-token sigmoid gate when shared_gated."""
    kind: str = "dense"                  # "dense" | "moe"
    ff: int = 0                          # dense width / routed expert width
    act: str = "relu2"                   # "relu2" | "gelu" | "gelu_tanh" | "silu"
    experts: int = 0
    top: int = 0
    groups: int = 1
    keep_groups: int = 1
    route_scale: float = 1.0
    shared_ff: int = 0
    shared_gated: bool = False
    gated: bool = False
    # routing variants: scores from a softmax over all experts or from a
    # sigmoid per expert; a learned per-expert correction added to the
    # scores for the CHOICE only (weights use the plain scores); a group
    # ranked by the sum of its `group_top` best choice scores (1 = its best
    # member); chosen scores divided by their sum before the scale
    route_scores: str = "softmax"        # "softmax" | "sigmoid"
    route_correction: bool = False
    group_top: int = 1
    renorm: bool = False


@dataclass(frozen=True)
class LayerSpec:
    """One entry of a heterogeneous layer stack (ModelSpec.layers)."""
    # "latent_attention" | "paged_attention" | "scan" | "parallel"
    mixer_type: str
    mixer: "LatentMixerSpec | PagedMixerSpec | ScanMixerSpec | ParallelMixerSpec"
    mlp: FeedForwardSpec | None = None


@dataclass
class ModelSpec:
    architecture: str = "LlamaForCausalLM"
    vocab_size: int = 128256
    hidden_size: int = 4096
    intermediate_size: int = 14336
    num_layers: int = 32
    num_heads: int = 32
    num_kv_heads: int = 8
    head_dim: int = 128
    rope_theta: float = 500000.0
    rope_scaling: dict | None = None
    rms_norm_eps: float = 1e-5
    max_position_embeddings: int = 8192
    tie_word_embeddings: bool = False
    attention_bias: bool = False  # qwen2-style qkv bias
    qk_norm: bool = False         # qwen3-style per-head q/k RMSNorm
    eos_token_id: int = 128001
    # MoE (Qwen3-MoE / Mixtral): num_experts > 0 makes every decoder
    # layer's MLP a router + expert bank (models/llama.py MoEMLP)
    num_experts: int = 0
    num_experts_per_tok: int = 0
    moe_intermediate_size: int = 0
    norm_topk_prob: bool = True
    # GLM-4.5 / DeepSeek-style MoE extensions (Glm4MoeForCausalLM):
    # sigmoid router scores + learned correction bias + optional grouped
    # top-k; a SHARED dense expert added to every token; the first k
    # layers use a plain dense MLP
    router_mode: str = "softmax"          # "softmax" | "sigmoid_bias"
    n_shared_experts: int = 0
    shared_expert_gated: bool = False    # Qwen2-MoE: sigmoid(gate(x)) scales
                                         # the shared expert's output
    first_k_dense_replace: int = 0
    routed_scaling_factor: float = 1.0
    n_group: int = 1
    topk_group: int = 1
    # rotary applied to the first head_dim*partial_rotary_factor dims only
    partial_rotary_factor: float = 1.0
    # GPT-OSS extensions (GptOssForCausalLM):
    # - attention SINKS: per-head learned logit joining the softmax
    #   denominator only
    # - alternating sliding-window / full attention layers (layer_types)
    # - clamped-swiglu expert activation + expert/router biases
    # - bias on o_proj (attention_bias covers q/k/v)
    attention_sinks: bool = False
    sliding_window: int = 0
    layer_types: tuple | None = None     # ("sliding_attention"|"full_attention", ...)
    moe_act: str = "silu"                # "silu" | "clamped_swiglu"
    moe_bias: bool = False               # expert gate_up/down biases
    router_logit_bias: bool = False      # bias added to router logits
    o_proj_bias: bool = False
    # DeepSeek V2/V3/R1 MLA (DeepseekV3ForCausalLM, models/llama.py
    # MLAAttention): kv_lora_rank > 0 switches attention to the latent
    # formulation — the paged cache stores [kv_lora_rank + qk_rope]
    # per token per layer instead of 2 * kv_heads * head_dim
    q_lora_rank: int = 0
    kv_lora_rank: int = 0
    qk_nope_head_dim: int = 0
    qk_rope_head_dim: int = 0
    v_head_dim: int = 0
    rope_interleave: bool = True         # deepseek weights: paired dims
    # Gemma-2 (Gemma2ForCausalLM): sandwich layer norms (post-attn and
    # post-ffn norms applied BEFORE the residual adds), sqrt(h)-scaled
    # embeddings, tanh logit softcapping in attention and on the final
    # logits, custom attention scale, GeGLU MLP; sliding window
    # alternates via layer_types (even layers) like GPT-OSS
    sandwich_norms: bool = False
    # OLMo-2 (Olmo2ForCausalLM): NO input norms — RMSNorm applied to each
    # sublayer's OUTPUT before the residual add; qk-norm runs over the
    # FULL projected q/k vectors (num_heads*head_dim), not per head
    norm_after: bool = False
    qk_norm_full: bool = False
    # Granite (GraniteForCausalLM): llama graph + scalar multipliers —
    # embeddings (embed_scale above), attention scale (attn_scale above),
    # sublayer outputs before the residual adds, and a final logits
    # DIVISOR
    residual_multiplier: float = 0.0     # 0 = off (1.0)
    logits_scaling: float = 0.0          # 0 = off (divide logits by this)
    # rotary application layout: "neox" rotate-half (llama lineage) or
    # "pairwise" GPT-J-style adjacent-pair rotation (Ernie-4.5; Hunyuan
    # and MiniMax share it — SURVEY family matrix)
    rope_mode: str = "neox"
    # Hunyuan-dense: per-head qk-norm applied AFTER rope (Qwen3 norms
    # before rope)
    qk_norm_after_rope: bool = False
    # SmolLM3 (SmolLM3ForCausalLM): per-layer rope switch — entry 0 means
    # a NoPE layer (no rotary at all); None = rope everywhere
    no_rope_layers: tuple | None = None
    # Gemma-3: sliding layers rope at a LOCAL base frequency (10k) while
    # full-attention layers use rope_theta (1M, linearly scaled) — the
    # model holds two cos/sin caches and each layer picks by window
    rope_local_theta: float = 0.0
    embed_scale: float = 0.0             # 0 = no scaling
    attn_logit_softcap: float = 0.0      # 0 = off
    final_logit_softcap: float = 0.0
    attn_scale: float = 0.0              # 0 = 1/sqrt(head_dim)
    mlp_act: str = "silu"                # "silu" | "gelu_tanh" | "relu2"
    norm_type: str = "rmsnorm"           # "layernorm": Cohere mean-centered
    parallel_block: bool = False         # Cohere: x + attn(ln(x)) + mlp(ln(x))
    logits_multiplier: float = 0.0       # Cohere logit_scale (multiplies)
    mlp_no_gate: bool = False            # Arcee: down(act(up(x))), no gate
    # Heterogeneous stacks (Vunitar): one LayerSpec per layer — each layer
    # names its mixer and feed-forward with their own sizes, so nothing
    # above (num_heads, head_dim, intermediate_size, ...) describes them.
    # Such models keep the residual stream, norms, scores and routers in
    # fp32 (fp32_residual) and run norm-after layers with a learned
    # per-channel layer scale on each sublayer's normed output.
    layers: tuple | None = None
    fp32_residual: bool = False
    layer_scale: bool = False
    # hashed (previous token, token) embedding added to the token row:
    # row = (prev * mul_prev + tok * mul_cur) % buckets; a sequence's first
    # token reads the extra row `buckets`. 0 buckets = off
    bigram_buckets: int = 0
    bigram_mul_prev: int = 0
    bigram_mul_cur: int = 0
    # weight-shared loop over a span of a heterogeneous stack: layers
    # start..stop-1 run `times` times in a row with the same weights, every
    # pass with cache pools of its own; each pass but the first starts by
    # adding the embedding output to the stream. None = every layer once
    layer_loop: tuple | None = None      # (start, stop, times)
    # the embedding output passes a norm of its own before the first layer
    embed_norm: bool = False

    @property
    def gqa_ratio(self) -> int:
        return self.num_heads // self.num_kv_heads

    def layer_runs(self) -> list[tuple[int, bool]]:
        """Execution order of a heterogeneous stack: one (layer index,
        re-inject the embedding first) entry per layer RUN. A looped layer
        appears once per pass; cache pools are per run, weights per layer."""
        n = len(self.layers)
        if not self.layer_loop:
            return [(i, False) for i in range(n)]
        start, stop, times = self.layer_loop
        runs = [(i, False) for i in range(start)]
        for t in range(times):
            runs += [(i, t > 0 and i == start) for i in range(start, stop)]
        return runs + [(i, False) for i in range(stop, n)]

    def kv_pool_widths(self) -> list[tuple]:
        """Per layer run of a heterogeneous stack: ("latent", rank),
        ("kv", kv_heads, key width, value width), ("state",) for a run that
        keeps nothing per token, or ("shared", run) for a run that reads
        the pools of an earlier one."""
        out = []
        for i, _ in self.layer_runs():
            m = self.layers[i].mixer
            if isinstance(m, ParallelMixerSpec):
                m = m.left
            if isinstance(m, LatentMixerSpec):
                if m.kv_from >= 0:
                    out.append(("shared", m.kv_from))
                elif m.rot_dim:
                    # one key "head" per token: latent | rotated key part;
                    # the latent again, page-transposed, as the value
                    out.append(("kv", 1, m.kv_rank + m.rot_dim, m.kv_rank))
                else:
                    out.append(("latent", m.kv_rank))
            elif isinstance(m, ScanMixerSpec):
                out.append(("state",))      # nothing per token: a state slot
            else:
                out.append(("kv", m.kv_heads, m.k_width, m.v_width))
        return out

    def state_pool_shapes(self) -> list[tuple | None]:
        """Per layer run: None, or (heads, state, vdim, conv rows, conv
        channels) of the recurrent state one live sequence holds there."""
        out = []
        for i, _ in self.layer_runs():
            m = self.layers[i].mixer
            if isinstance(m, ParallelMixerSpec):
                m = m.right
            if isinstance(m, ScanMixerSpec):
                out.append((m.heads, m.state, m.vdim,
                            max(m.conv - 1, 0), m.conv_channels))
            else:
                out.append(None)
        return out

    def state_bytes_per_slot(self, dtype_size: int = 2) -> int:
        """Bytes one live sequence holds in the recurrent-state pool: fp32
        matrix states plus the convolutions' last inputs in the engine
        dtype, over all layer runs."""
        if self.layers is None:
            return 0
        return sum(sh[0] * sh[1] * sh[2] * 4 + sh[3] * sh[4] * dtype_size
                   for sh in self.state_pool_shapes() if sh is not None)

    @property
    def has_state(self) -> bool:
        return self.layers is not None and any(
            isinstance(ls.mixer, (ScanMixerSpec, ParallelMixerSpec))
            for ls in self.layers)

    def kv_bytes_per_token(self, dtype_size: int = 2) -> int:
        if self.layers is not None:
            return sum(w[1] if w[0] == "latent" else
                       0 if w[0] in ("state", "shared")
                       else w[1] * (w[2] + w[3])
                       for w in self.kv_pool_widths()) * dtype_size
        if self.kv_lora_rank:
            # MLA: one compressed latent row per token per layer
            return (self.num_layers
                    * (self.kv_lora_rank + self.qk_rope_head_dim)
                    * dtype_size)
        return 2 * self.num_layers * self.num_kv_heads * self.head_dim * dtype_size

    def weight_bytes(self, dtype_size: int = 2) -> int:
        h, i, v = self.hidden_size, self.intermediate_size, self.vocab_size
        if self.layers is not None:
            n = 2 * v * h + h
            if self.bigram_buckets:
                n += (self.bigram_buckets + 1) * h
            for ls in self.layers:
                m = ls.mixer
                if self.architecture == "Makezen":
                    n += self._mixer_weights(h, m) + 2 * h
                    if ls.mlp is not None:
                        n += 2 * h * ls.mlp.ff + 2 * h
                    continue
                if isinstance(m, ScanMixerSpec):
                    if m.kind == "mamba2":
                        n += (h * (2 * m.inner + 2 * m.groups * m.state
                                   + m.heads)
                              + m.conv_channels * (m.conv + 1)
                              + 3 * m.heads + m.inner)
                    else:
                        n += (h * (2 * m.heads * m.state + 2 * m.inner)
                              + m.inner)
                    n += m.inner * h + 4 * h
                    f = ls.mlp
                    if f is not None and f.kind == "moe":
                        n += f.experts * (2 * h * f.ff + h + 1)
                        n += 2 * h * f.shared_ff
                    elif f is not None:
                        n += (3 if f.gated else 2) * h * f.ff
                    continue
                if isinstance(m, PagedMixerSpec):
                    n += (h * m.maps * m.qk_dim * (m.heads + m.kv_heads)
                          + (0 if m.tied_values else h * m.kv_heads * m.v_dim)
                          + m.heads * m.v_dim * h + 4 * h)
                    f = ls.mlp
                    if f is not None and f.kind == "moe":
                        n += f.experts * (2 * h * f.ff + h + 1)
                        n += 2 * h * f.shared_ff
                    elif f is not None:
                        n += (3 if f.gated else 2) * h * f.ff
                    continue
                n += (h * m.heads * m.qk_dim + h * m.kv_rank + m.kv_rank
                      + m.kv_rank * m.heads * (m.qk_dim + m.v_dim)
                      + m.heads * m.v_dim * h + 2 * h)
                f = ls.mlp
                if f is None:
                    continue
                n += 2 * h
                if f.kind == "moe":
                    n += f.experts * (2 * h * f.ff + h)
                    if f.shared_ff:
                        n += 2 * h * f.shared_ff + h
                else:
                    n += 2 * h * f.ff
            return n * dtype_size
        if self.kv_lora_rank:
            dq = self.qk_nope_head_dim + self.qk_rope_head_dim
            qp = (self.q_lora_rank * (h + self.num_heads * dq)
                  if self.q_lora_rank else h * self.num_heads * dq)
            qkv = (qp + h * (self.kv_lora_rank + self.qk_rope_head_dim)
                   + self.kv_lora_rank * self.num_heads
                   * (self.qk_nope_head_dim + self.v_head_dim))
            o = self.num_heads * self.v_head_dim * h
        else:
            qkv = h * (self.num_heads + 2 * self.num_kv_heads) * self.head_dim
            o = self.num_heads * self.head_dim * h
        attn_norm = qkv + o + 2 * h
        dense_mlp = 3 * h * i
        if self.num_experts > 0:
            moe_mlp = (self.num_experts * 3 * h * self.moe_intermediate_size
                       + self.num_experts * h  # router
                       + 3 * h * self.moe_intermediate_size
                       * self.n_shared_experts)
            k_dense = min(self.first_k_dense_replace, self.num_layers)
            total_layers = (attn_norm * self.num_layers
                            + dense_mlp * k_dense
                            + moe_mlp * (self.num_layers - k_dense))
        else:
            total_layers = (attn_norm + dense_mlp) * self.num_layers
        emb = v * h * (1 if self.tie_word_embeddings else 2)
        return (total_layers + emb + h) * dtype_size

    @classmethod
    def _mixer_weights(cls, h: int, m) -> int:
        """Weight count of one mixer of a Makezen stack."""
        if isinstance(m, ParallelMixerSpec):
            return (cls._mixer_weights(h, m.left)
                    + cls._mixer_weights(h, m.right) + 2 * h)
        if isinstance(m, ScanMixerSpec):        # gated delta rule
            qk = 2 * m.groups * m.state
            return (h * (qk + 2 * m.inner + 2 * m.heads)
                    + (qk + m.inner) * m.conv + 2 * m.heads + m.vdim
                    + m.inner * h)
        if isinstance(m, PagedMixerSpec):
            return ((h + 1) * (m.qk_dim * (m.heads + m.kv_heads)
                               + m.kv_heads * m.v_dim)
                    + 2 * m.qk_dim + m.heads * m.v_dim * h)
        qd = m.qk_dim + m.rot_dim
        n = (h * m.q_rank + m.q_rank + m.q_rank * m.heads * qd
             + m.kv_rank * m.heads * (m.qk_dim + m.v_dim)
             + 2 * m.heads + m.heads * h + m.heads * m.v_dim * h)
        if m.kv_from < 0:
            n += h * (m.kv_rank + m.rot_dim) + m.kv_rank
        return n

    @staticmethod
    def _rope_scaling_from(cfg: dict) -> dict | None:
        sc = cfg.get("rope_scaling") or (
            (cfg.get("rope_parameters") or None)
            if (cfg.get("rope_parameters") or {}).get("rope_type", "default")
            not in ("default",) else None)
        if sc and sc.get("rope_type", sc.get("type")) == "longrope" \
                and "original_max_position_embeddings" not in sc:
            # Phi-3/4 keep the pretraining length top-level
            sc = dict(sc)
            sc["original_max_position_embeddings"] = cfg.get(
                "original_max_position_embeddings",
                cfg.get("max_position_embeddings", 4096))
        return sc

    @classmethod
    def _from_vunitar_config(cls, cfg: dict) -> "ModelSpec":
        """Vunitar checkpoints describe themselves layer by layer: `layers`
        is a list of {type, mixer{...}, mlp{...}|null}; every size and
        every per-model constant comes from there."""
        layers = []
        for ent in cfg["layers"]:
            if ent["type"] != "latent_attention":
                raise NotImplementedError(
                    f"Vunitar mixer type {ent['type']!r} is not implemented")
            m = ent["mixer"]
            mixer = LatentMixerSpec(
                heads=int(m["heads"]), qk_dim=int(m["dim"]),
                v_dim=int(m["vdim"]), kv_rank=int(m["kv_rank"]),
                scale=float(m["scale"]))
            f = ent.get("mlp")
            if not f:
                ff = None
            elif f["kind"] == "dense":
                ff = FeedForwardSpec(kind="dense", ff=int(f["ff"]),
                                     act="relu2")
            elif f["kind"] == "moe":
                r = f["router"]
                g = r.get("groups") or {}
                sh = f.get("shared") or None
                ff = FeedForwardSpec(
                    kind="moe", ff=int(f["expert"]["ff"]), act="gelu",
                    experts=int(r["experts"]), top=int(r["top"]),
                    groups=int(g.get("count", 1) or 1),
                    keep_groups=int(g.get("keep", g.get("count", 1)) or 1),
                    route_scale=float(r.get("scale", 1.0)),
                    shared_ff=int(sh["ff"]) if sh else 0,
                    shared_gated=bool(sh))
            else:
                raise NotImplementedError(
                    f"Vunitar feed-forward kind {f['kind']!r}")
            layers.append(LayerSpec("latent_attention", mixer, ff))
        bg = (cfg.get("embedding") or {}).get("bigram") or {}
        return cls(
            architecture="Vunitar",
            vocab_size=int(cfg["vocab"]),
            hidden_size=int(cfg["width"]),
            num_layers=len(layers),
            layers=tuple(layers),
            # filler for code that sizes things by head: one latent "head"
            num_heads=1, num_kv_heads=1, head_dim=8, intermediate_size=0,
            rms_norm_eps=float(cfg["norm"]["eps"]),
            # no positional signal anywhere: length is bounded by the
            # cache pool alone
            max_position_embeddings=int(
                cfg.get("max_position_embeddings", 1 << 20)),
            eos_token_id=int(cfg.get("eos_token_id", -1)),
            norm_after=True, layer_scale=True, fp32_residual=True,
            final_logit_softcap=float(cfg.get("logit_softcap") or 0.0),
            bigram_buckets=int(bg.get("buckets", 0) or 0),
            bigram_mul_prev=int(bg.get("mul_prev", 0) or 0),
            bigram_mul_cur=int(bg.get("mul_cur", 0) or 0),
        )

    @classmethod
    def _from_fusipel_config(cls, cfg: dict) -> "ModelSpec":
        """Fusipel checkpoints list their layers like Vunitar ones: every
        entry names its mixer — "attention" (two-map differential scores,
        sliding window with kept first keys, own value projection) or
        "attention_2" (whole-projection q/k norm, values tied to the keys,
        per-head sink) — with its sizes and constants, and an optional
        gated dense feed-forward. `loop` repeats a span of the stack."""
        def rotary(r):
            if not r or not int(r.get("dims", 0) or 0):
                return RotarySpec()
            sc = r.get("scaling") or None
            return RotarySpec(
                dims=int(r["dims"]), base=float(r["base"]),
                scaling=(float(sc["factor"]), float(sc["low"]),
                         float(sc["high"]), float(sc["original"]))
                if sc else None)

        layers = []
        for ent in cfg["layers"]:
            m = ent["mixer"]
            common = dict(
                heads=int(m["heads"]), kv_heads=int(m["kv_heads"]),
                qk_dim=int(m["dim"]), v_dim=int(m.get("vdim", m["dim"])),
                scale=float(m["scale"]), rot=rotary(m.get("rot")), bias=True)
            if ent["type"] == "attention":
                mask = m.get("mask") or {}
                mixer = PagedMixerSpec(
                    **common, maps=2, diff=float(m["diff"]),
                    window=int(mask.get("size", 0) or 0),
                    keep_first=int(mask.get("keep_first", 0) or 0))
            elif ent["type"] == "attention_2":
                mixer = PagedMixerSpec(
                    **common, sink=True, qk_norm_full=True, tied_values=True)
            else:
                raise NotImplementedError(
                    f"Fusipel mixer type {ent['type']!r} is not implemented")
            if mixer.heads % mixer.kv_heads:
                raise ValueError("heads must be a multiple of kv_heads")
            if mixer.rot.dims % 2 or mixer.rot.dims > mixer.qk_dim:
                raise ValueError("rotary dims must be even and fit the head")
            f = ent.get("mlp")
            if not f:
                ff = None
            elif f["kind"] == "dense":
                ff = FeedForwardSpec(kind="dense", ff=int(f["ff"]),
                                     act="gelu_tanh", gated=True)
            else:
                raise NotImplementedError(
                    f"Fusipel feed-forward kind {f['kind']!r}")
            layers.append(LayerSpec("paged_attention", mixer, ff))
        loop = cfg.get("loop") or None
        if loop:
            start, stop, times = (int(loop["start"]), int(loop["stop"]),
                                  int(loop["times"]))
            if not (0 <= start <= stop <= len(layers)) or times < 1:
                raise ValueError("loop span outside the layer list")
            loop = (start, stop, times) if stop > start else None
        return cls(
            architecture="Fusipel",
            vocab_size=int(cfg["vocab"]),
            hidden_size=int(cfg["width"]),
            num_layers=len(layers),
            layers=tuple(layers),
            layer_loop=loop,
            num_heads=1, num_kv_heads=1, head_dim=8, intermediate_size=0,
            rms_norm_eps=float(cfg["norm"]["eps"]),
            max_position_embeddings=int(
                cfg.get("max_position_embeddings", 1 << 20)),
            eos_token_id=int(cfg.get("eos_token_id", -1)),
            sandwich_norms=True, fp32_residual=True,
            residual_multiplier=float(cfg.get("residual_mult", 1.0)),
        )

    @classmethod
    def _from_livasun_config(cls, cfg: dict) -> "ModelSpec":
        """Livasun checkpoints list their layers one by one; an entry names
        its mixer — "attention" (windowed softmax attention without
        rotation: per-head q/k norm, query temperature, distance bias,
        values blended with the first such layer's), "mamba2" or
        "lightning" (recurrent matrix states) — and its feed-forward:
        gated dense, a routed expert bank with an always-on shared expert,
        or none. Layers are pre-norm with layer norms (weight and bias) on
        an fp32 stream; embeddings are scaled."""
        layers = []
        for ent in cfg["layers"]:
            m, kind = ent["mixer"], ent["type"]
            if kind == "attention":
                mask = m.get("mask") or {}
                qt = m.get("q_temp") or None
                mixer = PagedMixerSpec(
                    heads=int(m["heads"]), kv_heads=int(m["kv_heads"]),
                    qk_dim=int(m["dim"]), v_dim=int(m.get("vdim", m["dim"])),
                    scale=float(m["scale"]),
                    window=int(mask.get("size", 0) or 0), head_norm=True,
                    q_temp=(float(qt["coef"]), float(qt["every"]))
                    if qt else None,
                    distance_bias=True, v_mix=bool(m.get("v_mix", False)))
                if mixer.heads % mixer.kv_heads:
                    raise ValueError("heads must be a multiple of kv_heads")
                if mixer.q_temp is not None and not mixer.q_temp[1] > 0:
                    raise ValueError("q_temp.every must be positive")
                mtype = "paged_attention"
            elif kind == "mamba2":
                mixer = ScanMixerSpec(
                    kind="mamba2", heads=int(m["heads"]),
                    state=int(m["state"]), vdim=int(m["vdim"]),
                    groups=int(m.get("groups", 1) or 1),
                    conv=int(m["conv"]),
                    norm_groups=int(m.get("norm_groups", 1) or 1))
                if mixer.heads % mixer.groups or mixer.conv < 1 \
                        or mixer.inner % mixer.norm_groups:
                    raise ValueError("mamba2 sizes do not divide")
                mtype = "scan"
            elif kind == "lightning":
                mixer = ScanMixerSpec(
                    kind="lightning", heads=int(m["heads"]),
                    state=int(m["dim"]), vdim=int(m["vdim"]),
                    groups=int(m["heads"]),
                    decay=tuple(float(d) for d in m["decay"]))
                if len(mixer.decay) != mixer.heads:
                    raise ValueError("one decay per head")
                mtype = "scan"
            else:
                raise NotImplementedError(
                    f"Livasun mixer type {kind!r} is not implemented")
            f = ent.get("mlp")
            if not f:
                ff = None
            elif f["kind"] == "dense":
                ff = FeedForwardSpec(kind="dense", ff=int(f["ff"]),
                                     act="silu", gated=True)
            elif f["kind"] == "moe":
                r = f["router"]
                g = r.get("groups") or {}
                sh = f.get("shared") or None
                ff = FeedForwardSpec(
                    kind="moe", ff=int(f["expert"]["ff"]), act="relu2",
                    experts=int(r["experts"]), top=int(r["top"]),
                    groups=int(g.get("count", 1) or 1),
                    keep_groups=int(g.get("keep", g.get("count", 1)) or 1),
                    route_scale=float(r.get("scale", 1.0)),
                    shared_ff=int(sh["ff"]) if sh else 0,
                    route_scores="sigmoid", route_correction=True,
                    group_top=2, renorm=True)
                if ff.experts % ff.groups or ff.top > ff.experts \
                        or ff.keep_groups * (ff.experts // ff.groups) < ff.top:
                    raise ValueError("router sizes do not fit")
            else:
                raise NotImplementedError(
                    f"Livasun feed-forward kind {f['kind']!r}")
            layers.append(LayerSpec(mtype, mixer, ff))
        vm = [ls.mixer for ls in layers
              if isinstance(ls.mixer, PagedMixerSpec) and ls.mixer.v_mix]
        if any((m.kv_heads, m.v_dim) != (vm[0].kv_heads, vm[0].v_dim)
               for m in vm):
            raise ValueError("value-mixing layers must share a value shape")
        return cls(
            architecture="Livasun",
            vocab_size=int(cfg["vocab"]),
            hidden_size=int(cfg["width"]),
            num_layers=len(layers),
            layers=tuple(layers),
            num_heads=1, num_kv_heads=1, head_dim=8, intermediate_size=0,
            rms_norm_eps=float(cfg["norm"]["eps"]),
            max_position_embeddings=int(
                cfg.get("max_position_embeddings", 1 << 20)),
            eos_token_id=int(cfg.get("eos_token_id", -1)),
            fp32_residual=True, norm_type="layernorm_bias",
            embed_scale=float((cfg.get("embedding") or {}).get("scale", 1.0)),
        )

    @classmethod
    def _from_makezen_config(cls, cfg: dict) -> "ModelSpec":
        """Makezen checkpoints list their layers one by one; an entry names
        its mixer — "latent_attention" (rotary latent attention behind a
        sliding window, with sinks, an output gate and optionally the
        cached latents of an earlier layer), "delta" (gated delta rule) or
        "parallel" (softmax attention and a gated delta rule side by side)
        — and an ungated dense feed-forward or none. Every sublayer sits
        between two weight-only layer norms on an fp32 stream; the
        embedding output is normed and the head is the embedding table."""
        def rotary(r):
            if not r or not int(r.get("dims", 0) or 0):
                return RotarySpec(layout="half")
            sc = r.get("scaling") or None
            return RotarySpec(
                dims=int(r["dims"]), base=float(r["base"]), layout="half",
                ramp=(float(sc["factor"]), float(sc["original"]),
                      float(sc["fast"]), float(sc["slow"])) if sc else None)

        def delta(m):
            sp = ScanMixerSpec(
                kind="delta", heads=int(m["heads"]), state=int(m["dim"]),
                vdim=int(m["vdim"]), groups=int(m["kv_heads"]),
                conv=int(m["conv"]))
            if sp.heads % sp.groups or sp.conv < 1:
                raise ValueError("delta mixer sizes do not divide")
            return sp

        def softmax(m):
            sp = PagedMixerSpec(
                heads=int(m["heads"]), kv_heads=int(m["kv_heads"]),
                qk_dim=int(m["dim"]), v_dim=int(m.get("vdim", m["dim"])),
                scale=float(m["scale"]), rot=rotary(m.get("rot")), bias=True,
                head_norm=True, softcap=float(m.get("softcap") or 0.0),
                window=int((m.get("mask") or {}).get("size", 0) or 0))
            if sp.heads % sp.kv_heads:
                raise ValueError("heads must be a multiple of kv_heads")
            if sp.rot.dims % 2 or sp.rot.dims > sp.qk_dim:
                raise ValueError("rotary dims must be even and fit the head")
            return sp

        layers = []
        for i, ent in enumerate(cfg["layers"]):
            m, kind = ent["mixer"], ent["type"]
            if kind == "latent_attention":
                rot = rotary(m.get("rot"))
                src = m.get("kv_from")
                mixer = LatentMixerSpec(
                    heads=int(m["heads"]), qk_dim=int(m["dim"]),
                    v_dim=int(m["vdim"]), kv_rank=int(m["kv_rank"]),
                    scale=float(m["scale"]), rot_dim=int(m["rot_dim"]),
                    rot=rot, q_rank=int(m["q_rank"]),
                    window=int((m.get("mask") or {}).get("size", 0) or 0),
                    sink=True, out_gate=True,
                    kv_from=-1 if src is None else int(src))
                if rot.dims != mixer.rot_dim or rot.dims % 2 or not rot.dims:
                    raise ValueError("the rotated part is rot_dim wide")
                if mixer.kv_from >= 0:
                    own = layers[mixer.kv_from].mixer \
                        if mixer.kv_from < i else None
                    if not isinstance(own, LatentMixerSpec) \
                            or own.kv_from >= 0 \
                            or (own.kv_rank, own.rot_dim, own.rot) != (
                                mixer.kv_rank, mixer.rot_dim, mixer.rot):
                        raise ValueError(
                            "kv_from must name an earlier latent layer with "
                            "its own down-projection and the same latent "
                            "sizes and rotation")
                mtype = "latent_attention"
            elif kind == "delta":
                mixer, mtype = delta(m), "scan"
            elif kind == "parallel":
                mixer = ParallelMixerSpec(left=softmax(m["left"]),
                                          right=delta(m["right"]))
                mtype = "parallel"
            else:
                raise NotImplementedError(
                    f"Makezen mixer type {kind!r} is not implemented")
            f = ent.get("mlp")
            if not f:
                ff = None
            elif f["kind"] == "dense":
                ff = FeedForwardSpec(kind="dense", ff=int(f["ff"]),
                                     act="gelu_tanh")
            else:
                raise NotImplementedError(
                    f"Makezen feed-forward kind {f['kind']!r}")
            layers.append(LayerSpec(mtype, mixer, ff))
        return cls(
            architecture="Makezen",
            vocab_size=int(cfg["vocab"]),
            hidden_size=int(cfg["width"]),
            num_layers=len(layers),
            layers=tuple(layers),
            num_heads=1, num_kv_heads=1, head_dim=8, intermediate_size=0,
            rms_norm_eps=float(cfg["norm"]["eps"]),
            max_position_embeddings=int(
                cfg.get("max_position_embeddings", 1 << 20)),
            eos_token_id=int(cfg.get("eos_token_id", -1)),
            sandwich_norms=True, fp32_residual=True, norm_type="layernorm",
            embed_norm=True, tie_word_embeddings=True,
        )

    @classmethod
    def from_hf_config(cls, cfg: dict) -> "ModelSpec":
        if cfg.get("architecture") == "Makezen" and "architectures" not in cfg:
            return cls._from_makezen_config(cfg)
        if cfg.get("architecture") == "Livasun" and "architectures" not in cfg:
            return cls._from_livasun_config(cfg)
        if cfg.get("architecture") == "Vunitar" and "architectures" not in cfg:
            return cls._from_vunitar_config(cfg)
        if cfg.get("architecture") == "Fusipel" and "architectures" not in cfg:
            return cls._from_fusipel_config(cfg)
        arch = (cfg.get("architectures") or ["LlamaForCausalLM"])[0]
        if arch.startswith("Cohere") and cfg.get("use_qk_norm"):
            raise NotImplementedError(
                "Cohere use_qk_norm (per-head LayerNorm, Command-A) is "
                "not implemented yet")
        # OLMo-3 keys rope_parameters BY LAYER TYPE: full_attention
        # defines the main rope (theta + any scaling); sliding layers
        # rope unscaled at their own theta (the Gemma-3 dual-cache path).
        slide_theta = 0.0
        rp = cfg.get("rope_parameters")
        if isinstance(rp, dict) and "full_attention" in rp:
            cfg = dict(cfg)
            cfg["rope_parameters"] = rp.get("full_attention") or {}
            slide_theta = (rp.get("sliding_attention") or {}).get(
                "rope_theta", 0.0) or 0.0
        nh = cfg.get("num_attention_heads", 32)
        hd = cfg.get("head_dim") or cfg.get("hidden_size", 4096) // nh
        eos = cfg.get("eos_token_id", 2)
        if isinstance(eos, list):
            eos = eos[0]
        return cls(
            architecture=arch,
            vocab_size=cfg.get("vocab_size", 32000),
            hidden_size=cfg.get("hidden_size", 4096),
            intermediate_size=cfg.get("intermediate_size", 11008),
            num_layers=cfg.get("num_hidden_layers", 32),
            num_heads=nh,
            num_kv_heads=cfg.get("num_key_value_heads", nh),
            head_dim=hd,
            rope_theta=cfg.get("rope_theta")
            or (cfg.get("rope_parameters") or {}).get("rope_theta", 10000.0),
            rope_scaling=cls._rope_scaling_from(cfg),
            rms_norm_eps=(cfg.get("layer_norm_eps", 1e-5)
                          if arch.startswith("Cohere")
                          else cfg.get("rms_norm_eps", 1e-6)),
            max_position_embeddings=cfg.get("max_position_embeddings", 4096),
            tie_word_embeddings=cfg.get("tie_word_embeddings", False),
            attention_bias=(arch.startswith("Qwen2")
                            or arch.startswith("SeedOss")
                            or (arch in ("GlmForCausalLM",
                                         "Glm4ForCausalLM")
                                and bool(cfg.get("attention_bias", True)))
                            or (arch.startswith("Ernie4_5")
                                and bool(cfg.get("use_bias")))),
            qk_norm=(arch.startswith("Qwen3") or arch.startswith("Gemma3")
                     or arch.startswith(("Olmo2", "Olmo3", "Exaone4"))
                     or arch.startswith(("Olmoe", "MiniMaxM2", "Dots1"))
                     or arch.startswith("HunYuan")
                     or bool(cfg.get("use_qk_norm", False))),
            qk_norm_after_rope=arch.startswith("HunYuan"),
            eos_token_id=eos,
            num_experts=cfg.get("num_experts",
                                cfg.get("num_local_experts",
                                        cfg.get("n_routed_experts", 0))) or 0,
            num_experts_per_tok=cfg.get("num_experts_per_tok", 0) or 0,
            moe_intermediate_size=cfg.get("moe_intermediate_size",
                                          cfg.get("intermediate_size", 0))
            if (cfg.get("num_experts") or cfg.get("num_local_experts")
                or cfg.get("n_routed_experts")) else 0,
            norm_topk_prob=bool(cfg.get("norm_topk_prob", True)),
            router_mode=("sigmoid_bias"
                         if (arch.startswith("Glm4Moe")
                             or arch.startswith(("MiniMaxM2", "Dots1"))
                             or arch.startswith("Deepseek"))
                         else "softmax"),
            n_shared_experts=(cfg.get("n_shared_experts", 0) or 0)
            if not arch.startswith("Qwen2Moe")
            # Qwen2-MoE sizes the shared expert directly; express it as
            # a multiple of the routed intermediate (5632 = 4 x 1408)
            else (cfg.get("shared_expert_intermediate_size", 0)
                  // max(cfg.get("moe_intermediate_size", 1), 1)),
            shared_expert_gated=arch.startswith("Qwen2Moe"),
            first_k_dense_replace=cfg.get("first_k_dense_replace", 0) or 0,
            routed_scaling_factor=cfg.get("routed_scaling_factor", 1.0) or 1.0,
            n_group=cfg.get("n_group", 1) or 1,
            topk_group=cfg.get("topk_group", 1) or 1,
            partial_rotary_factor=(cfg.get("partial_rotary_factor")
                                   or (cfg.get("rope_parameters") or {})
                                   .get("partial_rotary_factor")
                                   # MiniMax checkpoints name it rotary_dim
                                   or (cfg["rotary_dim"] / hd
                                       if cfg.get("rotary_dim") else 1.0)),
            attention_sinks=arch.startswith("GptOss"),
            sliding_window=(cfg.get("sliding_window") or 0)
            if (arch.startswith("GptOss") or arch.startswith("Gemma")
                or arch.startswith(("Olmo3", "Exaone4", "Cohere2")))
            else 0,
            layer_types=tuple(cfg["layer_types"])
            if cfg.get("layer_types") else (
                tuple("sliding_attention"
                      if (i + 1) % int(cfg.get("sliding_window_pattern", 6))
                      else "full_attention"
                      for i in range(cfg.get("num_hidden_layers", 0)))
                if arch.startswith("Gemma3") else None),
            moe_act="clamped_swiglu" if arch.startswith("GptOss") else "silu",
            moe_bias=arch.startswith("GptOss"),
            router_logit_bias=arch.startswith("GptOss"),
            o_proj_bias=bool(cfg.get("attention_bias"))
            if arch.startswith("GptOss") else False,
            q_lora_rank=(cfg.get("q_lora_rank") or 0)
            if arch.startswith("Deepseek") else 0,
            kv_lora_rank=(cfg.get("kv_lora_rank") or 0)
            if arch.startswith("Deepseek") else 0,
            qk_nope_head_dim=cfg.get("qk_nope_head_dim", 0) or 0,
            qk_rope_head_dim=cfg.get("qk_rope_head_dim", 0) or 0,
            v_head_dim=cfg.get("v_head_dim", 0) or 0,
            rope_interleave=bool(cfg.get("rope_interleave", True)),
            sandwich_norms=(arch.startswith("Gemma2")
                            or arch.startswith("Gemma3")
                            # GLM-4 dense: same four-norm layer flow,
                            # plain RMSNorm weights (no (1+w) offset)
                            or arch == "Glm4ForCausalLM"),
            norm_after=arch.startswith(("Olmo2", "Olmo3", "Exaone4")),
            qk_norm_full=arch.startswith(("Olmo2", "Olmo3", "Olmoe",
                                          "MiniMaxM2")),
            embed_scale=(cfg.get("hidden_size", 4096) ** 0.5
                         if arch.startswith("Gemma")
                         else (cfg.get("embedding_multiplier") or 0.0)
                         if arch.startswith("Granite") else 0.0),
            attn_logit_softcap=(cfg.get("attn_logit_softcapping") or 0.0)
            if arch.startswith("Gemma") else 0.0,
            final_logit_softcap=(cfg.get("final_logit_softcapping") or 0.0)
            if arch.startswith("Gemma") else 0.0,
            attn_scale=((cfg.get("query_pre_attn_scalar") or 0) ** -0.5
                        if (arch.startswith("Gemma")
                            and cfg.get("query_pre_attn_scalar"))
                        else (cfg.get("attention_multiplier") or 0.0)
                        if arch.startswith("Granite") else 0.0),
            residual_multiplier=(cfg.get("residual_multiplier") or 0.0)
            if arch.startswith("Granite") else 0.0,
            logits_scaling=(cfg.get("logits_scaling") or 0.0)
            if arch.startswith("Granite") else 0.0,
            rope_mode=("pairwise"
                       if (arch.startswith(("Ernie4_5", "Cohere",
                                            "Helium"))
                           or arch in ("GlmForCausalLM",
                                       "Glm4ForCausalLM"))
                       else "neox"),
            norm_type=("layernorm" if arch.startswith("Cohere")
                       else "rmsnorm"),
            parallel_block=arch.startswith("Cohere"),
            logits_multiplier=(cfg.get("logit_scale") or 0.0)
            if arch.startswith("Cohere") else 0.0,
            no_rope_layers=(tuple(cfg["no_rope_layers"])
                            if cfg.get("no_rope_layers") else (
                                # EXAONE-4 hybrid: global-NoPE — rope on
                                # sliding layers only, full layers unroped
                                tuple(1 if lt == "sliding_attention" else 0
                                      for lt in cfg["layer_types"])
                                if (arch.startswith(("Exaone4", "Cohere2"))
                                    and cfg.get("sliding_window")
                                    and cfg.get("layer_types")) else
                                tuple(0 if (i + 1) % 4 == 0 else 1
                                      for i in range(
                                          cfg.get("num_hidden_layers", 0)))
                                if arch.startswith("SmolLM3") else None)),
            rope_local_theta=(cfg.get("rope_local_base_freq") or 0.0)
            if arch.startswith("Gemma3")
            else (slide_theta if arch.startswith("Olmo3") else 0.0),
            mlp_act=("gelu_tanh" if arch.startswith("Gemma")
                     else "relu2" if arch.startswith("Arcee")
                     else "silu"),
            mlp_no_gate=arch.startswith("Arcee"),
        )

    @classmethod
    def from_dir(cls, model_dir: str | Path) -> "ModelSpec":
        with open(Path(model_dir) / "config.json") as f:
            return cls.from_hf_config(json.load(f))


# Named presets so the bench / tests / control plane can run with
# random-init weights and no network (BASELINE.json: synthetic data).
PRESETS: dict[str, ModelSpec] = {
    # DeepSeek-V3/R1 671B: MLA latent attention + 256-expert sigmoid+bias
    # grouped MoE (the R1 checkpoints share this architecture)
    "deepseek-v3": ModelSpec(
        architecture="DeepseekV3ForCausalLM", vocab_size=129280,
        hidden_size=7168, intermediate_size=18432, num_layers=61,
        num_heads=128, num_kv_heads=128, head_dim=192,
        rope_theta=10000.0, max_position_embeddings=163840,
        rope_scaling={"rope_type": "yarn", "factor": 40.0,
                      "beta_fast": 32.0, "beta_slow": 1.0,
                      "mscale": 1.0, "mscale_all_dim": 1.0,
                      "original_max_position_embeddings": 4096},
        eos_token_id=1, num_experts=256, num_experts_per_tok=8,
        moe_intermediate_size=2048, router_mode="sigmoid_bias",
        n_shared_experts=1, first_k_dense_replace=3,
        routed_scaling_factor=2.5, n_group=8, topk_group=4,
        norm_topk_prob=True,
        q_lora_rank=1536, kv_lora_rank=512, qk_nope_head_dim=128,
        qk_rope_head_dim=64, v_head_dim=128,
    ),

    "llama-3-8b": ModelSpec(),
    "llama-3-70b": ModelSpec(
        hidden_size=8192, intermediate_size=28672, num_layers=80,
        num_heads=64, num_kv_heads=8,
    ),
    # Llama-3.1: same graph as 3.0 plus llama3 rope scaling and 128k context
    "llama-3.1-8b": ModelSpec(
        rope_scaling={"rope_type": "llama3", "factor": 8.0,
                      "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                      "original_max_position_embeddings": 8192},
        max_position_embeddings=131072,
    ),
    "llama-3.1-70b": ModelSpec(
        hidden_size=8192, intermediate_size=28672, num_layers=80,
        num_heads=64, num_kv_heads=8,
        rope_scaling={"rope_type": "llama3", "factor": 8.0,
                      "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                      "original_max_position_embeddings": 8192},
        max_position_embeddings=131072,
    ),
    "qwen3-32b": ModelSpec(
        architecture="Qwen3ForCausalLM", vocab_size=151936, hidden_size=5120,
        intermediate_size=25600, num_layers=64, num_heads=64, num_kv_heads=8,
        rope_theta=1000000.0, max_position_embeddings=40960, qk_norm=True,
        eos_token_id=151645,
    ),
    "qwen3-14b": ModelSpec(
        architecture="Qwen3ForCausalLM", vocab_size=151936, hidden_size=5120,
        intermediate_size=17408, num_layers=40, num_heads=40, num_kv_heads=8,
        rope_theta=1000000.0, max_position_embeddings=40960, qk_norm=True,
        eos_token_id=151645,
    ),
    "qwen2.5-7b": ModelSpec(
        architecture="Qwen2ForCausalLM", vocab_size=152064, hidden_size=3584,
        intermediate_size=18944, num_layers=28, num_heads=28, num_kv_heads=4,
        rope_theta=1000000.0, attention_bias=True, eos_token_id=151645,
    ),
    # Qwen3-30B-A3B: 128-expert top-8 MoE, 3B active params
    "qwen3-30b-a3b": ModelSpec(
        architecture="Qwen3MoeForCausalLM", vocab_size=151936,
        hidden_size=2048, intermediate_size=6144, num_layers=48,
        num_heads=32, num_kv_heads=4, head_dim=128, rope_theta=1000000.0,
        max_position_embeddings=40960, qk_norm=True, eos_token_id=151645,
        num_experts=128, num_experts_per_tok=8, moe_intermediate_size=768,
    ),
    # Qwen3-235B-A22B (the BASELINE.md 8-GPU MoE row): same Qwen3-MoE
    # graph as 30B-A3B, bigger dims — serves TP8 over xGMI
    "qwen3-235b-a22b": ModelSpec(
        architecture="Qwen3MoeForCausalLM", vocab_size=151936,
        hidden_size=4096, intermediate_size=12288, num_layers=94,
        num_heads=64, num_kv_heads=4, head_dim=128, rope_theta=1000000.0,
        max_position_embeddings=40960, qk_norm=True, eos_token_id=151645,
        num_experts=128, num_experts_per_tok=8, moe_intermediate_size=1536,
    ),
    # GLM-4.5-Air: Glm4Moe graph — sigmoid+bias
    # router, 1 shared expert, first layer dense, partial rotary 0.5
    "glm-4.5-air": ModelSpec(
        architecture="Glm4MoeForCausalLM", vocab_size=151552,
        hidden_size=4096, intermediate_size=10944, num_layers=46,
        num_heads=96, num_kv_heads=8, head_dim=128, rope_theta=1000000.0,
        max_position_embeddings=131072, qk_norm=True, eos_token_id=151329,
        num_experts=128, num_experts_per_tok=8, moe_intermediate_size=1408,
        router_mode="sigmoid_bias", n_shared_experts=1,
        first_k_dense_replace=1, partial_rotary_factor=0.5,
    ),
    # GPT-OSS 20B / 120B: 128/32-expert top-4 MoE,
    # alternating sliding(128)/full attention with sinks, clamped swiglu,
    # YaRN rope, head_dim 64. CPU-exact; CDNA4 kernels are an r3 item
    # (the GPU ops fail loudly on D=64/sinks/window).
    "gpt-oss-20b": ModelSpec(
        architecture="GptOssForCausalLM", vocab_size=201088,
        hidden_size=2880, intermediate_size=2880, num_layers=24,
        num_heads=64, num_kv_heads=8, head_dim=64, rope_theta=150000.0,
        rope_scaling={"rope_type": "yarn", "factor": 32.0,
                      "beta_fast": 32.0, "beta_slow": 1.0, "truncate": False,
                      "original_max_position_embeddings": 4096},
        max_position_embeddings=131072, eos_token_id=200002,
        attention_bias=True, o_proj_bias=True, attention_sinks=True,
        sliding_window=128, num_experts=32, num_experts_per_tok=4,
        moe_intermediate_size=2880, moe_act="clamped_swiglu", moe_bias=True,
        router_logit_bias=True, norm_topk_prob=True,
    ),
    "gpt-oss-120b": ModelSpec(
        architecture="GptOssForCausalLM", vocab_size=201088,
        hidden_size=2880, intermediate_size=2880, num_layers=36,
        num_heads=64, num_kv_heads=8, head_dim=64, rope_theta=150000.0,
        rope_scaling={"rope_type": "yarn", "factor": 32.0,
                      "beta_fast": 32.0, "beta_slow": 1.0, "truncate": False,
                      "original_max_position_embeddings": 4096},
        max_position_embeddings=131072, eos_token_id=200002,
        attention_bias=True, o_proj_bias=True, attention_sinks=True,
        sliding_window=128, num_experts=128, num_experts_per_tok=4,
        moe_intermediate_size=2880, moe_act="clamped_swiglu", moe_bias=True,
        router_logit_bias=True, norm_topk_prob=True,
    ),
    # Mixtral 8x7B: 8-expert top-2 MoE on the llama graph
    "mixtral-8x7b": ModelSpec(
        architecture="MixtralForCausalLM", vocab_size=32000,
        hidden_size=4096, intermediate_size=14336, num_layers=32,
        num_heads=32, num_kv_heads=8, rope_theta=1000000.0,
        max_position_embeddings=32768, eos_token_id=2,
        num_experts=8, num_experts_per_tok=2, moe_intermediate_size=14336,
    ),
    # tiny MoE (CPU-testable routing/dispatch plumbing)
    "tiny-moe": ModelSpec(
        vocab_size=512, hidden_size=128, intermediate_size=256, num_layers=2,
        num_heads=4, num_kv_heads=2, head_dim=32, max_position_embeddings=512,
        rope_theta=10000.0, eos_token_id=1,
        num_experts=8, num_experts_per_tok=2, moe_intermediate_size=64,
    ),
    # Mistral v0.3: llama-compatible compute graph (no SWA since v0.1;
    # GQA 32/8, theta 1e6) — runs on the same CDNA4 kernel set
    "mistral-7b": ModelSpec(
        architecture="MistralForCausalLM", vocab_size=32768, hidden_size=4096,
        intermediate_size=14336, num_layers=32, num_heads=32, num_kv_heads=8,
        rope_theta=1000000.0, max_position_embeddings=32768,
    ),
    # tiny CPU-testable model (OPT-125m-scale plumbing per BASELINE.json cfg 1)
    "tiny": ModelSpec(
        vocab_size=512, hidden_size=128, intermediate_size=256, num_layers=2,
        num_heads=4, num_kv_heads=2, head_dim=32, max_position_embeddings=512,
        rope_theta=10000.0, eos_token_id=1,
    ),
    # OLMo-2 13B (norm-after layers + full-projection qk-norm)
    "olmo-2-13b": ModelSpec(
        architecture="Olmo2ForCausalLM", vocab_size=100352,
        hidden_size=5120, intermediate_size=13824, num_layers=40,
        num_heads=40, num_kv_heads=40, head_dim=128,
        rope_theta=500000.0, max_position_embeddings=4096,
        rms_norm_eps=1e-6, eos_token_id=100257, qk_norm=True,
        norm_after=True, qk_norm_full=True,
    ),
    # Phi-4 14B (Phi3ForCausalLM graph: fused qkv/gate_up, plain rope)
    "phi-4": ModelSpec(
        architecture="Phi3ForCausalLM", vocab_size=100352,
        hidden_size=5120, intermediate_size=17920, num_layers=40,
        num_heads=40, num_kv_heads=10, head_dim=128, rope_theta=250000.0,
        max_position_embeddings=16384, eos_token_id=100257,
    ),
    # DeepSeek-R1: identical architecture/dims to V3 (reasoning ckpt)
    "deepseek-r1": ModelSpec(
        architecture="DeepseekV3ForCausalLM", vocab_size=129280,
        hidden_size=7168, intermediate_size=18432, num_layers=61,
        num_heads=128, num_kv_heads=128, head_dim=192,
        rope_theta=10000.0, max_position_embeddings=163840,
        rope_scaling={"rope_type": "yarn", "factor": 40.0,
                      "beta_fast": 32.0, "beta_slow": 1.0,
                      "mscale": 1.0, "mscale_all_dim": 1.0,
                      "original_max_position_embeddings": 4096},
        eos_token_id=1, num_experts=256, num_experts_per_tok=8,
        moe_intermediate_size=2048, router_mode="sigmoid_bias",
        n_shared_experts=1, first_k_dense_replace=3,
        routed_scaling_factor=2.5, n_group=8, topk_group=4,
        norm_topk_prob=True,
        q_lora_rank=1536, kv_lora_rank=512, qk_nope_head_dim=128,
        qk_rope_head_dim=64, v_head_dim=128,
    ),
    # Kimi-K2 1T: DeepseekV3 architecture at larger expert count
    "kimi-k2": ModelSpec(
        architecture="DeepseekV3ForCausalLM", vocab_size=163840,
        hidden_size=7168, intermediate_size=18432, num_layers=61,
        num_heads=64, num_kv_heads=64, head_dim=192,
        rope_theta=50000.0, max_position_embeddings=131072,
        eos_token_id=163585, num_experts=384, num_experts_per_tok=8,
        moe_intermediate_size=2048, router_mode="sigmoid_bias",
        n_shared_experts=1, first_k_dense_replace=1,
        routed_scaling_factor=2.827, n_group=1, topk_group=1,
        norm_topk_prob=True,
        q_lora_rank=1536, kv_lora_rank=512, qk_nope_head_dim=128,
        qk_rope_head_dim=64, v_head_dim=128,
    ),
    # Gemma-2: sandwich norms, GeGLU, softcapping, alternating SWA,
    # scaled tied embeddings (CPU-oracle family; GPU kernels share the
    # GPT-OSS r3 window work — head_dim 256 needs a D-template too)
    "gemma-2-9b": ModelSpec(
        architecture="Gemma2ForCausalLM", vocab_size=256000,
        hidden_size=3584, intermediate_size=14336, num_layers=42,
        num_heads=16, num_kv_heads=8, head_dim=256, rope_theta=10000.0,
        max_position_embeddings=8192, tie_word_embeddings=True,
        rms_norm_eps=1e-6, eos_token_id=1, sliding_window=4096,
        sandwich_norms=True, embed_scale=3584 ** 0.5,
        attn_logit_softcap=50.0, final_logit_softcap=30.0,
        attn_scale=224 ** -0.5, mlp_act="gelu_tanh",
    ),
    # Gemma-3: dual rope (local 10k on sliding layers, linear-scaled 1M
    # global), (1+w) qk-norm, 5:1 SWA pattern, no softcapping
    "gemma-3-27b": ModelSpec(
        architecture="Gemma3ForCausalLM", vocab_size=262208,
        hidden_size=5376, intermediate_size=21504, num_layers=62,
        num_heads=32, num_kv_heads=16, head_dim=128,
        rope_theta=1000000.0, rope_local_theta=10000.0,
        rope_scaling={"rope_type": "linear", "factor": 8.0},
        max_position_embeddings=131072, tie_word_embeddings=True,
        rms_norm_eps=1e-6, eos_token_id=1, sliding_window=1024,
        layer_types=tuple("sliding_attention" if (i + 1) % 6 else
                          "full_attention" for i in range(62)),
        sandwich_norms=True, qk_norm=True, embed_scale=5376 ** 0.5,
        attn_scale=168 ** -0.5, mlp_act="gelu_tanh",
    ),
    # CPU-test preset: Gemma-shaped sandwich-norm layers (tests the
    # residual-None PP handoff + softcap/GeGLU paths on gloo)
    "tiny-gemma": ModelSpec(
        architecture="Gemma2ForCausalLM", vocab_size=512, hidden_size=128,
        intermediate_size=256, num_layers=4, num_heads=4, num_kv_heads=2,
        head_dim=32, max_position_embeddings=512, rope_theta=10000.0,
        rms_norm_eps=1e-6, eos_token_id=1, tie_word_embeddings=True,
        sliding_window=8, sandwich_norms=True, embed_scale=128 ** 0.5,
        attn_logit_softcap=50.0, final_logit_softcap=30.0,
        attn_scale=24 ** -0.5, mlp_act="gelu_tanh",
    ),
    # CPU-test preset: DeepSeek-shaped MLA + MoE (tests/test_deepseek.py,
    # TP exactness on gloo)
    "tiny-mla": ModelSpec(
        architecture="DeepseekV3ForCausalLM", vocab_size=512,
        hidden_size=128, intermediate_size=256, num_layers=2,
        num_heads=4, num_kv_heads=4, head_dim=48,
        max_position_embeddings=256, rope_theta=10000.0, eos_token_id=1,
        num_experts=8, num_experts_per_tok=2, moe_intermediate_size=64,
        router_mode="sigmoid_bias", n_shared_experts=1,
        first_k_dense_replace=1, routed_scaling_factor=1.5, n_group=2,
        topk_group=1, q_lora_rank=64, kv_lora_rank=96,
        qk_nope_head_dim=32, qk_rope_head_dim=16, v_head_dim=32,
    ),
}


@dataclass
class EngineConfig:
    model: str = "llama-3-8b"              # preset name or model dir
    dtype: str = "bfloat16"
    kv_cache_dtype: str = "bf16"           # bf16 | fp8 (e4m3, halves KV bytes)
    block_size: int = 16
    gpu_memory_utilization: float = 0.90
    max_num_seqs: int = 256
    max_prefill_tokens: int = 8192         # per-step prefill token budget
    max_model_len: int = 8192
    kv_cache_blocks: int | None = None     # override (CPU tests)
    tp_size: int = 1
    tp_rank: int = 0
    device: str = "cuda"
    seed: int = 0
    enforce_random_weights: bool = True    # no checkpoint: random init
    model_dir: str | None = None
    # host-DRAM KV offload tier (extended_kv_cache in the reference schema)
    kv_offload_gb: float = 0.0
    # automatic prefix caching: cache-hit prompts recompute only the suffix
    # through the paged prefill-with-history MFMA kernel; the r1 cap (the
    # old paged-decode-row fallback cost ~3.5x per token) is retired — any
    # suffix length now runs at flash-prefill efficiency
    enable_prefix_caching: bool = False
    prefix_cache_suffix_cap: int = 1 << 30
    # chunked prefill (reference: vLLM --enable-chunked-prefill): a prompt
    # longer than max_prefill_tokens is split into budget-sized chunks
    # (chunk 0 = capped prefill batch, continuations = paged prefill-with-
    # history tiles), alternating 1:1 with decode steps so running
    # sequences keep a bounded time-between-tokens during long-prompt
    # admission. Default ON since r2: continuations run at flash-prefill
    # efficiency (the r1 3.5x continuation penalty is gone)
    enable_chunked_prefill: bool = True
    # speculative decoding (reference speculative_config schema):
    # {"method": "ngram", "num_draft_tokens": 3, "ngram_max": 3, "ngram_min": 1}
    speculative: dict | None = None
    # W4 runtime quantization ("w4"): the big serving weights are packed
    # int4 in HBM after load and decode GEMMs dequantize in-register
    # (ops/csrc/w4_gemm.hip) — 70B-class models stay resident packed
    # instead of inflating to bf16 (reference: vLLM --quantization)
    quantize_runtime: str | None = None
    # CPU weight offload (reference: vLLM --cpu-offload-gb, the GGUF
    # partial-offload placement): ~this many GiB of trailing layers'
    # weights live pinned in host DRAM and stream to a double-buffered
    # device staging area one layer ahead of use (engine/offload.py)
    cpu_offload_gb: float = 0.0
    # uneven pipeline-stage layer counts (len == pp_size, sums to
    # num_layers) — the native analog of the reference's per-GPU GGUF
    # tensor_split proportions; None = even split (remainder to early
    # stages so the sampling stage carries less)
    pp_partition: list[int] | None = None
    # LoRA adapters merged into the weights at load (reference lora_list)
    lora_dirs: list[str] = field(default_factory=list)
    # GGUF checkpoint execution: dequantized to bf16 at load (utils/gguf.py)
    gguf_path: str | None = None
    # admission hysteresis: open a prefill step only when this many requests
    # wait, one has waited admission_max_wait_s, or nothing is running —
    # keeps steady-state decode on the hipGraph path instead of degrading
    # every step to a tiny eager mixed batch
    admission_min_seqs: int = 16
    admission_max_wait_s: float = 0.1

    spec: ModelSpec = field(default_factory=ModelSpec)

    def __post_init__(self):
        if self.model in PRESETS:
            import dataclasses

            # copy: configs may tweak their spec (tests shrink num_layers,
            # qk_norm overrides) and must not mutate the shared preset
            self.spec = dataclasses.replace(PRESETS[self.model])
        elif self.model_dir:
            self.spec = ModelSpec.from_dir(self.model_dir)
        elif self.model.endswith(".gguf") and Path(self.model).is_file():
            from ..utils.gguf import spec_from_gguf

            self.gguf_path = self.model
            self.spec = spec_from_gguf(self.model)
        elif Path(self.model).is_dir():
            self.model_dir = self.model
            self.spec = ModelSpec.from_dir(self.model)
        self.max_model_len = min(self.max_model_len, self.spec.max_position_embeddings)
        if self.enable_chunked_prefill and self.speculative and \
                self.speculative.get("method") in ("eagle", "eagle3", "mtp"):
            # draft-model speculation seeds from full-prompt prefill hiddens,
            # which chunked admission does not produce in one step; chunked
            # prefill (default-on since r2) yields to the explicit
            # speculative config
            import logging

            logging.getLogger(__name__).info(
                "disabling chunked prefill: incompatible with draft-model "
                "speculative decoding")
            self.enable_chunked_prefill = False
