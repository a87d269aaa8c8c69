// Torch bindings for the layer-norm row kernels, the head-norm cache write,
// scored routing (lnrows32.hip) and the recurrent mixers (state_scan.hip,
// delta_scan.hip);
// page-wise value stores come from rowmix32.hip. Every shape a kernel or its
// grid assumes is checked here on the host before the launch; VALUES inside
// index tensors are bounded in the kernels.
#include <torch/extension.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime.h>

void embed_rows_scaled_launch(float*, const long*, const void*, int, int, long, float, int, hipStream_t);
void add_layer_norm_launch(float*, const void*, const float*, const float*, void*, int, int, float, int, int, hipStream_t);
void head_norm_store_launch(void*, void*, long, int, int, int, const float*, const float*, int, float, float, const int*, const void*, long, const float*, void*, void*, const long*, long, int, int, int, float, int, int, int, hipStream_t);
void value_page_store_launch(const void*, long, int, void*, const long*, long, const int*, int, int, int, int, int, int, hipStream_t);
void route_topk_launch(int*, float*, const float*, int, const float*, int, int, int, int, int, int, int, int, float, hipStream_t);
void causal_conv_silu_launch(void*, const void*, long, int, int, int, const float*, const float*, void*, const int*, const int*, const int*, const int*, const int*, int, int, int, int, hipStream_t);
int state_scan_launch(float*, const void*, long, int, int, int, const void*, long, int, int, int, int, int, int, const float*, const float*, const float*, const float*, float*, const int*, const int*, const int*, const int*, int, int, int, int, int, hipStream_t);
void gated_group_norm_launch(void*, const float*, const void*, long, const float*, int, int, int, float, int, int, int, hipStream_t);
int delta_scan_launch(float*, const void*, long, int, int, int, const void*, long, int, int, int, int, int, int, const float*, const float*, float*, const int*, const int*, const int*, const int*, int, int, int, int, int, hipStream_t);
int delta_scan_max_state();
int state_scan_max_state();
int conv_max_taps();

#define HIP_CHECK_LAST()                                                     \
  do {                                                                       \
    hipError_t e_ = hipGetLastError();                                       \
    TORCH_CHECK(e_ == hipSuccess, "HIP kernel launch failed: ",              \
                hipGetErrorString(e_));                                      \
  } while (0)

namespace {

using at::Tensor;
using OptTensor = c10::optional<Tensor>;

hipStream_t cur_stream(const Tensor& t) {
  return c10::hip::getCurrentHIPStream(t.device().index()).stream();
}

void chk(const Tensor& t, const char* name, at::ScalarType ty) {
  TORCH_CHECK(t.is_cuda(), name, " must be on GPU");
  TORCH_CHECK(t.scalar_type() == ty, name, " has the wrong dtype");
  TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
}

// bf16 -> 1, fp32 -> 0
int act_kind(const Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda(), name, " must be on GPU");
  TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
  if (t.scalar_type() == at::kBFloat16) return 1;
  TORCH_CHECK(t.scalar_type() == at::kFloat, name, " must be bf16 or fp32");
  return 0;
}

// a [T, C] view whose rows may be strided (a column slice of a projection)
int view_kind(const Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda(), name, " must be on GPU");
  TORCH_CHECK(t.dim() == 2 && (t.size(1) == 1 || t.stride(1) == 1) &&
              t.stride(0) >= t.size(1), name, " must be a row-major 2-d view");
  if (t.scalar_type() == at::kBFloat16) return 1;
  TORCH_CHECK(t.scalar_type() == at::kFloat, name, " must be bf16 or fp32");
  return 0;
}

void embed_rows_scaled(Tensor x, Tensor tokens, Tensor embed, double scale) {
  chk(x, "x", at::kFloat);
  chk(tokens, "tokens", at::kLong);
  const int bf = act_kind(embed, "embed");
  TORCH_CHECK(x.dim() == 2 && embed.dim() == 2 && embed.size(1) == x.size(1));
  TORCH_CHECK(tokens.numel() == x.size(0) && embed.size(0) >= 1);
  embed_rows_scaled_launch(x.data_ptr<float>(), tokens.data_ptr<long>(),
                           embed.data_ptr(), (int)x.size(0), (int)x.size(1),
                           embed.size(0), (float)scale, bf, cur_stream(x));
  HIP_CHECK_LAST();
}

void add_layer_norm(Tensor x, OptTensor a, OptTensor w, OptTensor b, double eps,
                    OptTensor h) {
  chk(x, "x", at::kFloat);
  TORCH_CHECK(x.dim() == 2);
  const int T = x.size(0), W = x.size(1);
  const void* ap = nullptr;
  const float *wp = nullptr, *bp = nullptr;
  void* hp = nullptr;
  int a_bf = 0, h_bf = 0;
  if (a.has_value()) {
    a_bf = act_kind(*a, "a");
    TORCH_CHECK(a->sizes() == x.sizes());
    ap = a->data_ptr();
  }
  if (w.has_value()) {
    TORCH_CHECK(b.has_value() && h.has_value());
    chk(*w, "w", at::kFloat);
    chk(*b, "b", at::kFloat);
    TORCH_CHECK(w->numel() == W && b->numel() == W);
    h_bf = act_kind(*h, "h");
    TORCH_CHECK(h->sizes() == x.sizes());
    wp = w->data_ptr<float>();
    bp = b->data_ptr<float>();
    hp = h->data_ptr();
  }
  add_layer_norm_launch(x.data_ptr<float>(), ap, wp, bp, hp, T, W, (float)eps,
                        a_bf, h_bf, cur_stream(x));
  HIP_CHECK_LAST();
}

void head_norm_store(Tensor q_out, Tensor qkv, long nq, long nk, Tensor q_w,
                     Tensor k_w, long head_dim, double temp_coef,
                     double temp_every, Tensor pos32, OptTensor v_first,
                     OptTensor lam, Tensor k_cache, Tensor v_cache, Tensor slots,
                     double eps, OptTensor page_groups) {
  const int bf = act_kind(q_out, "q_out");
  TORCH_CHECK(act_kind(qkv, "qkv") == bf && act_kind(k_cache, "k_cache") == bf &&
              act_kind(v_cache, "v_cache") == bf,
              "q, qkv and the pools must share a dtype");
  chk(q_w, "q_w", at::kFloat);
  chk(k_w, "k_w", at::kFloat);
  chk(pos32, "pos32", at::kInt);
  chk(slots, "slots", at::kLong);
  TORCH_CHECK(qkv.dim() == 2 && q_out.dim() == 2 && k_cache.dim() == 4 &&
              v_cache.dim() == 4);
  const int T = qkv.size(0);
  const int G = k_cache.size(1), BS = k_cache.size(2), D = k_cache.size(3);
  const int VW = v_cache.size(2);
  TORCH_CHECK(v_cache.size(0) == k_cache.size(0) && v_cache.size(1) == G &&
              v_cache.size(3) == BS, "value pool must be [nblocks, G, VW, BS]");
  const long nv = (long)G * VW;
  TORCH_CHECK(head_dim == D && nq >= D && nq % D == 0 && nk == (long)G * D &&
              qkv.size(1) == nq + nk + nv,
              "projection width does not fit the pools");
  TORCH_CHECK(q_out.size(0) == T && q_out.size(1) == nq);
  TORCH_CHECK(q_w.numel() == D && k_w.numel() == D);
  TORCH_CHECK(pos32.numel() == T && slots.numel() == T && temp_every >= 0);
  const void* vf = nullptr;
  const float* lp = nullptr;
  long ld_vf = 0;
  if (v_first.has_value()) {
    TORCH_CHECK(lam.has_value());
    chk(*lam, "lam", at::kFloat);
    TORCH_CHECK(lam->numel() >= 1);
    TORCH_CHECK(view_kind(*v_first, "v_first") == bf);
    TORCH_CHECK(v_first->size(0) == T && v_first->size(1) == nv);
    vf = v_first->data_ptr();
    ld_vf = v_first->stride(0);
    lp = lam->data_ptr<float>();
  }
  // slots outside [0, nblocks*BS) are skipped inside the kernels
  head_norm_store_launch(q_out.data_ptr(), qkv.data_ptr(), qkv.stride(0),
                         (int)nq, (int)nk, (int)nv, q_w.data_ptr<float>(),
                         k_w.data_ptr<float>(), D, (float)temp_coef,
                         (float)temp_every, pos32.data_ptr<int>(), vf, ld_vf, lp,
                         k_cache.data_ptr(), v_cache.data_ptr(),
                         slots.data_ptr<long>(), k_cache.size(0) * (long)BS, G,
                         BS, VW, (float)eps, page_groups.has_value() ? 1 : 0, T,
                         bf, cur_stream(qkv));
  HIP_CHECK_LAST();
  if (page_groups.has_value()) {
    // the value rows leave page by page (runs of rows inside one page)
    chk(*page_groups, "page_groups", at::kInt);
    TORCH_CHECK(BS == 16, "page-wise value stores need 16-token pages");
    TORCH_CHECK(page_groups->dim() == 2 && page_groups->size(1) == 2);
    value_page_store_launch(qkv.data_ptr(), qkv.stride(0), (int)(nq + nk),
                            v_cache.data_ptr(), slots.data_ptr<long>(),
                            k_cache.size(0) * (long)BS,
                            page_groups->data_ptr<int>(),
                            (int)page_groups->size(0), T, G, VW, bf, 0,
                            cur_stream(qkv));
    HIP_CHECK_LAST();
  }
}

void route_topk(Tensor experts, Tensor weights, Tensor logits,
                OptTensor correction, long n_experts, long groups, long keep,
                long group_top, bool use_sigmoid, bool renorm, double scale) {
  chk(experts, "experts", at::kInt);
  chk(weights, "weights", at::kFloat);
  chk(logits, "logits", at::kFloat);
  TORCH_CHECK(logits.dim() == 2 && experts.dim() == 2 &&
              experts.sizes() == weights.sizes());
  const int T = logits.size(0), top = experts.size(1);
  TORCH_CHECK(experts.size(0) == T && n_experts >= 1 &&
              n_experts <= logits.size(1) && n_experts <= 4096);
  TORCH_CHECK(groups >= 1 && n_experts % groups == 0 && keep >= 1 &&
              keep <= groups && group_top >= 1);
  TORCH_CHECK(top >= 1 && top <= keep * (n_experts / groups),
              "not enough eligible experts for top-k");
  const float* cp = nullptr;
  if (correction.has_value()) {
    chk(*correction, "correction", at::kFloat);
    TORCH_CHECK(correction->numel() == n_experts);
    cp = correction->data_ptr<float>();
  }
  route_topk_launch(experts.data_ptr<int>(), weights.data_ptr<float>(),
                    logits.data_ptr<float>(), (int)logits.size(1), cp, T,
                    (int)n_experts, (int)groups, (int)keep, (int)group_top, top,
                    use_sigmoid ? 1 : 0, renorm ? 1 : 0, (float)scale,
                    cur_stream(logits));
  HIP_CHECK_LAST();
}

// the per-sequence view: first row, rows, state slot of every sequence
int seq_view(const Tensor& seq_first, const Tensor& seq_rows,
             const Tensor& state_slots, const Tensor& pos32, int T) {
  chk(seq_first, "seq_first", at::kInt);
  chk(seq_rows, "seq_rows", at::kInt);
  chk(state_slots, "state_slots", at::kInt);
  chk(pos32, "pos32", at::kInt);
  const int nseq = seq_first.numel();
  TORCH_CHECK(seq_rows.numel() == nseq && state_slots.numel() == nseq &&
              pos32.numel() == T);
  return nseq;
}

void causal_conv_silu(Tensor out, Tensor src, long col0, Tensor w, Tensor b,
                      Tensor conv_state, Tensor seq_first, Tensor seq_rows,
                      Tensor state_slots, Tensor row_seq, Tensor pos32) {
  const int bf = act_kind(out, "out");
  TORCH_CHECK(view_kind(src, "src") == bf &&
              act_kind(conv_state, "conv_state") == bf,
              "out, src and the state must share a dtype");
  chk(w, "w", at::kFloat);
  chk(b, "b", at::kFloat);
  chk(row_seq, "row_seq", at::kInt);
  TORCH_CHECK(out.dim() == 2 && w.dim() == 2 && conv_state.dim() == 3);
  const int T = out.size(0), C = out.size(1), taps = w.size(1);
  TORCH_CHECK(src.size(0) == T && col0 >= 0 && col0 + C <= src.size(1));
  TORCH_CHECK(w.size(0) == C && b.numel() == C && taps >= 1 &&
              taps <= conv_max_taps());
  TORCH_CHECK(taps == 1 || (conv_state.size(1) == taps - 1 &&
                            conv_state.size(2) == C && conv_state.size(0) >= 1),
              "state must be [slots, taps - 1, channels]");
  const int nseq = seq_view(seq_first, seq_rows, state_slots, pos32, T);
  TORCH_CHECK(row_seq.numel() == T);
  causal_conv_silu_launch(out.data_ptr(), src.data_ptr(), src.stride(0),
                          (int)col0, C, taps, w.data_ptr<float>(),
                          b.data_ptr<float>(), conv_state.data_ptr(),
                          seq_first.data_ptr<int>(), seq_rows.data_ptr<int>(),
                          state_slots.data_ptr<int>(), row_seq.data_ptr<int>(),
                          pos32.data_ptr<int>(), nseq, (int)conv_state.size(0),
                          T, bf, cur_stream(src));
  HIP_CHECK_LAST();
}

void state_scan(Tensor y, Tensor src, long col_x, long col_b, long col_c,
                OptTensor dt_src, long col_dt, long heads, long groups,
                long n_state, long vdim, bool act_silu, OptTensor dt_bias,
                OptTensor a_log, OptTensor skip, OptTensor decay, Tensor state,
                Tensor seq_first, Tensor seq_rows, Tensor state_slots,
                Tensor pos32, bool single) {
  chk(y, "y", at::kFloat);
  chk(state, "state", at::kFloat);
  const int bf = view_kind(src, "src");
  const int T = src.size(0);
  TORCH_CHECK(heads >= 1 && groups >= 1 && heads % groups == 0 &&
              n_state >= 1 && n_state <= state_scan_max_state() && vdim >= 1);
  TORCH_CHECK(y.dim() == 2 && y.size(0) == T && y.size(1) == heads * vdim);
  TORCH_CHECK(state.dim() == 4 && state.size(0) >= 1 && state.size(1) == heads &&
              state.size(2) == n_state && state.size(3) == vdim,
              "state must be [slots, heads, state, vdim]");
  const long W = src.size(1);
  TORCH_CHECK(col_x >= 0 && col_x + heads * vdim <= W && col_b >= 0 &&
              col_b + groups * n_state <= W && col_c >= 0 &&
              col_c + groups * n_state <= W, "columns outside the source");
  const void* dtp = nullptr;
  long ld_dt = 0;
  const float *bp = nullptr, *ap = nullptr, *sp = nullptr, *dp = nullptr;
  if (dt_src.has_value()) {
    TORCH_CHECK(view_kind(*dt_src, "dt_src") == bf && dt_src->size(0) == T &&
                col_dt >= 0 && col_dt + heads <= dt_src->size(1));
    TORCH_CHECK(dt_bias.has_value() && a_log.has_value());
    chk(*dt_bias, "dt_bias", at::kFloat);
    chk(*a_log, "a_log", at::kFloat);
    TORCH_CHECK(dt_bias->numel() == heads && a_log->numel() == heads);
    dtp = dt_src->data_ptr();
    ld_dt = dt_src->stride(0);
    bp = dt_bias->data_ptr<float>();
    ap = a_log->data_ptr<float>();
  } else {
    TORCH_CHECK(decay.has_value(), "either step sizes or constant decays");
    chk(*decay, "decay", at::kFloat);
    TORCH_CHECK(decay->numel() == heads);
    dp = decay->data_ptr<float>();
  }
  if (skip.has_value()) {
    chk(*skip, "skip", at::kFloat);
    TORCH_CHECK(skip->numel() == heads);
    sp = skip->data_ptr<float>();
  }
  const int nseq = seq_view(seq_first, seq_rows, state_slots, pos32, T);
  const int ok = state_scan_launch(
      y.data_ptr<float>(), src.data_ptr(), src.stride(0), (int)col_x,
      (int)col_b, (int)col_c, dtp, ld_dt, (int)col_dt, (int)heads, (int)groups,
      (int)n_state, (int)vdim, act_silu ? 1 : 0, bp, ap, sp, dp,
      state.data_ptr<float>(), seq_first.data_ptr<int>(),
      seq_rows.data_ptr<int>(), state_slots.data_ptr<int>(),
      pos32.data_ptr<int>(), nseq, (int)state.size(0), T, bf, single ? 1 : 0,
      cur_stream(src));
  TORCH_CHECK(ok, "state size unsupported");
  HIP_CHECK_LAST();
}

void delta_scan(Tensor y, Tensor src, long col_q, long col_k, long col_v,
                Tensor gate_src, long col_a, long col_b, long heads,
                long groups, long n_state, long vdim, Tensor dt_bias,
                Tensor a_log, Tensor state, Tensor seq_first, Tensor seq_rows,
                Tensor state_slots, Tensor pos32, bool single) {
  chk(y, "y", at::kFloat);
  chk(state, "state", at::kFloat);
  chk(dt_bias, "dt_bias", at::kFloat);
  chk(a_log, "a_log", at::kFloat);
  const int bf = view_kind(src, "src");
  const int T = src.size(0);
  TORCH_CHECK(heads >= 1 && groups >= 1 && heads % groups == 0 &&
              n_state >= 1 && n_state <= delta_scan_max_state() && vdim >= 1);
  TORCH_CHECK(y.dim() == 2 && y.size(0) == T && y.size(1) == heads * vdim);
  TORCH_CHECK(state.dim() == 4 && state.size(0) >= 1 && state.size(1) == heads &&
              state.size(2) == n_state && state.size(3) == vdim,
              "state must be [slots, heads, state, vdim]");
  const long W = src.size(1);
  TORCH_CHECK(col_v >= 0 && col_v + heads * vdim <= W && col_q >= 0 &&
              col_q + groups * n_state <= W && col_k >= 0 &&
              col_k + groups * n_state <= W, "columns outside the source");
  TORCH_CHECK(view_kind(gate_src, "gate_src") == bf && gate_src.size(0) == T &&
              col_a >= 0 && col_a + heads <= gate_src.size(1) && col_b >= 0 &&
              col_b + heads <= gate_src.size(1), "gate columns outside");
  TORCH_CHECK(dt_bias.numel() == heads && a_log.numel() == heads);
  const int nseq = seq_view(seq_first, seq_rows, state_slots, pos32, T);
  const int ok = delta_scan_launch(
      y.data_ptr<float>(), src.data_ptr(), src.stride(0), (int)col_q,
      (int)col_k, (int)col_v, gate_src.data_ptr(), gate_src.stride(0),
      (int)col_a, (int)col_b, (int)heads, (int)groups, (int)n_state, (int)vdim,
      dt_bias.data_ptr<float>(), a_log.data_ptr<float>(),
      state.data_ptr<float>(), seq_first.data_ptr<int>(),
      seq_rows.data_ptr<int>(), state_slots.data_ptr<int>(),
      pos32.data_ptr<int>(), nseq, (int)state.size(0), T, bf, single ? 1 : 0,
      cur_stream(src));
  TORCH_CHECK(ok, "state size unsupported");
  HIP_CHECK_LAST();
}

void gated_group_norm(Tensor out, Tensor y, Tensor gate, Tensor w, long groups,
                      double eps, long gate_first) {
  chk(y, "y", at::kFloat);
  chk(w, "w", at::kFloat);
  const int out_bf = act_kind(out, "out");
  const int gate_bf = view_kind(gate, "gate");
  TORCH_CHECK(y.dim() == 2 && out.sizes() == y.sizes() &&
              gate.size(0) == y.size(0) && gate.size(1) == y.size(1));
  const int T = y.size(0), C = y.size(1);
  TORCH_CHECK(groups >= 1 && C % groups == 0 && w.numel() == C);
  TORCH_CHECK(gate_first >= 0 && gate_first <= 2);
  gated_group_norm_launch(out.data_ptr(), y.data_ptr<float>(), gate.data_ptr(),
                          gate.stride(0), w.data_ptr<float>(), T, C,
                          (int)groups, (float)eps, (int)gate_first, gate_bf,
                          out_bf, cur_stream(y));
  HIP_CHECK_LAST();
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("embed_rows_scaled", &embed_rows_scaled);
  m.def("add_layer_norm", &add_layer_norm);
  m.def("head_norm_store", &head_norm_store);
  m.def("route_topk", &route_topk);
  m.def("causal_conv_silu", &causal_conv_silu);
  m.def("state_scan", &state_scan);
  m.def("delta_scan", &delta_scan);
  m.def("gated_group_norm", &gated_group_norm);
}
