// Torch bindings for the pre/post-norm fp32-stream row kernels and paged
// rotary attention (rowmix32.hip, ragged_attn.hip; argmax from resid32.hip).
// Every shape a kernel or its grid assumes is checked here on the host
// before the launch; VALUES inside index tensors are bounded in the kernels.
#include <torch/extension.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime.h>

void embed_rows_f32_launch(float*, const long*, const void*, int, int, long, int, hipStream_t);
void sandwich_add_norm_launch(float*, const void*, const float*, float, const float*, const float*, void*, int, int, float, int, int, int, hipStream_t);
void rotary_norm_store_launch(void*, const void*, long, int, int, int, const float*, const float*, const float*, int, const int*, int, void*, void*, const long*, long, int, int, int, int, float, int, int, int, hipStream_t);
void value_page_store_launch(const void*, long, int, void*, const long*, long, const int*, int, int, int, int, int, int, hipStream_t);
void diff_combine_launch(void*, const float*, const float*, float, float, long, int, int, hipStream_t);
void act_and_mul_launch(void*, const void*, long, int, int, int, hipStream_t);
void argmax_f32_launch(long*, const float*, int, int, hipStream_t);
void paged_attention_launch(void*, const void*, const void*, const void*, const int*, const int*, const int*, const float*, const float*, float, float, long, long, long, long, int, int, int, int, int, int, int, int, int, int, int, int, int, int, int, int, int, int, int, float*, float*, hipStream_t);
void head_rope_store_launch(void*, const void*, long, int, int, int, const float*, int, int, int, int, int, const float*, int, int, int, const float*, int, int, float, const int*, void*, void*, const long*, long, int, int, float, int, int, int, hipStream_t);
void dual_rms_mix_launch(void*, const void*, const float*, const void*, const float*, int, int, float, int, hipStream_t);
void head_gate_launch(void*, const void*, const void*, long, int, int, int, int, int, hipStream_t);
void act_inplace_launch(void*, long, int, int, hipStream_t);
int paged_attn_max_dim();
int paged_attn_uses_mfma(int, int, int, int);

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

// the same for a [T, A, C] view: any row / head strides, channels contiguous
// (the attention kernels read q and write out element by element)
int view_kind(const Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda(), name, " must be on GPU");
  TORCH_CHECK(t.dim() == 3 && (t.size(2) == 1 || t.stride(2) == 1), name,
              " must be [T, A, C] with contiguous channels");
  TORCH_CHECK(t.stride(0) >= 0 && t.stride(1) >= 0, name, " strides");
  const bool bf = t.scalar_type() == at::kBFloat16;
  TORCH_CHECK(bf || t.scalar_type() == at::kFloat, name,
              " must be bf16 or fp32");
  return bf ? 1 : 0;
}

void embed_rows_f32(Tensor x, Tensor tokens, Tensor embed) {
  chk(x, "x", at::kFloat);
  chk(tokens, "tokens", at::kLong);
  const int bf = act_kind(embed, "embed");
  TORCH_CHECK(x.dim() == 2 && embed.dim() == 2 && embed.size(1) == x.size(1));
  TORCH_CHECK(tokens.numel() == x.size(0) && embed.size(0) >= 1);
  embed_rows_f32_launch(x.data_ptr<float>(), tokens.data_ptr<long>(),
                        embed.data_ptr(), (int)x.size(0), (int)x.size(1),
                        embed.size(0), bf, cur_stream(x));
  HIP_CHECK_LAST();
}

void sandwich_add_norm(Tensor x, OptTensor a, OptTensor post_w, double mult,
                       double eps, OptTensor extra, OptTensor next_w,
                       OptTensor h, bool center) {
  chk(x, "x", at::kFloat);
  TORCH_CHECK(x.dim() == 2);
  const int T = x.size(0), W = x.size(1);
  const void* ap = nullptr;
  const float *pw = nullptr, *ep = nullptr, *nw = nullptr;
  void* hp = nullptr;
  int a_bf = 0, h_bf = 0;
  if (a.has_value()) {
    a_bf = act_kind(*a, "a");
    TORCH_CHECK(a->sizes() == x.sizes() && post_w.has_value());
    chk(*post_w, "post_w", at::kFloat);
    TORCH_CHECK(post_w->numel() == W);
    ap = a->data_ptr();
    pw = post_w->data_ptr<float>();
  }
  if (extra.has_value()) {
    chk(*extra, "extra", at::kFloat);
    TORCH_CHECK(extra->sizes() == x.sizes());
    ep = extra->data_ptr<float>();
  }
  if (next_w.has_value()) {
    chk(*next_w, "next_w", at::kFloat);
    TORCH_CHECK(next_w->numel() == W && h.has_value());
    h_bf = act_kind(*h, "h");
    TORCH_CHECK(h->sizes() == x.sizes());
    nw = next_w->data_ptr<float>();
    hp = h->data_ptr();
  }
  sandwich_add_norm_launch(x.data_ptr<float>(), ap, pw, (float)mult, ep, nw, hp,
                           T, W, (float)eps, a_bf, h_bf, center ? 1 : 0,
                           cur_stream(x));
  HIP_CHECK_LAST();
}

void rotary_norm_store(Tensor q_out, Tensor qkv, long nq, long nk,
                       OptTensor q_norm_w, OptTensor k_norm_w, Tensor inv_freq,
                       Tensor pos32, long head_dim, Tensor k_cache,
                       Tensor v_cache, Tensor slots, double eps, bool tied,
                       OptTensor page_groups) {
  const int bf = act_kind(q_out, "q_out");
  TORCH_CHECK(act_kind(qkv, "qkv") == bf && act_kind(k_cache, "k_cache") == bf &&
              act_kind(v_cache, "v_cache") == bf,
              "q, qkv and the pools must share a dtype");
  chk(inv_freq, "inv_freq", at::kFloat);
  chk(pos32, "pos32", at::kInt);
  chk(slots, "slots", at::kLong);
  TORCH_CHECK(qkv.dim() == 2 && q_out.dim() == 2 && k_cache.dim() == 4 &&
              v_cache.dim() == 4);
  const int T = qkv.size(0);
  const int G = k_cache.size(1), BS = k_cache.size(2), KW = k_cache.size(3);
  const int VW = v_cache.size(2);
  TORCH_CHECK(v_cache.size(0) == k_cache.size(0) && v_cache.size(1) == G &&
              v_cache.size(3) == BS, "value pool must be [nblocks, G, VW, BS]");
  const long nv = tied ? 0 : (long)G * VW;
  TORCH_CHECK(nq >= 1 && nk == (long)G * KW && qkv.size(1) == nq + nk + nv,
              "projection width does not fit the pools");
  TORCH_CHECK(!tied || VW * (long)G == nk, "tied values need VW == KW");
  TORCH_CHECK(q_out.size(0) == T && q_out.size(1) == nq);
  TORCH_CHECK(pos32.numel() == T && slots.numel() == T);
  const int half = inv_freq.numel();
  TORCH_CHECK(head_dim >= 1 && nq % head_dim == 0 && KW % head_dim == 0 &&
              2 * half <= head_dim, "rotary dims must fit the head");
  TORCH_CHECK(half == 0 || head_dim % 2 == 0,
              "rotary needs an even head size");
  const float *qw = nullptr, *kw = nullptr;
  if (q_norm_w.has_value()) {
    TORCH_CHECK(k_norm_w.has_value());
    chk(*q_norm_w, "q_norm_w", at::kFloat);
    chk(*k_norm_w, "k_norm_w", at::kFloat);
    TORCH_CHECK(q_norm_w->numel() == nq && k_norm_w->numel() == nk);
    qw = q_norm_w->data_ptr<float>();
    kw = k_norm_w->data_ptr<float>();
  }
  // slots outside [0, nblocks*BS) are skipped inside the kernel
  rotary_norm_store_launch(q_out.data_ptr(), qkv.data_ptr(), qkv.stride(0),
                           (int)nq, (int)nk, (int)nv, qw, kw,
                           inv_freq.data_ptr<float>(), half,
                           pos32.data_ptr<int>(), (int)head_dim,
                           k_cache.data_ptr(), v_cache.data_ptr(),
                           slots.data_ptr<long>(), k_cache.size(0) * (long)BS,
                           G, BS, KW, VW, (float)eps,
                           (tied ? 1 : 0) | (page_groups.has_value() ? 2 : 0),
                           T, bf, cur_stream(qkv));
  HIP_CHECK_LAST();
  if (page_groups.has_value()) {
    // the value rows leave page by page (runs of rows inside one page)
    chk(*page_groups, "page_groups", at::kInt);
    TORCH_CHECK(BS == 16, "page-wise value stores need 16-token pages");
    TORCH_CHECK(page_groups->dim() == 2 && page_groups->size(1) == 2);
    value_page_store_launch(qkv.data_ptr(), qkv.stride(0),
                            (int)(tied ? nq : nq + nk), v_cache.data_ptr(),
                            slots.data_ptr<long>(), k_cache.size(0) * (long)BS,
                            page_groups->data_ptr<int>(),
                            (int)page_groups->size(0), T, G, VW, bf, 0,
                            cur_stream(qkv));
    HIP_CHECK_LAST();
  }
}

void paged_attention(Tensor out, Tensor q, Tensor k_cache, Tensor v_cache,
                     Tensor block_tables, Tensor tiles, Tensor pos32,
                     double scale, long maps, long window, long keep_first,
                     OptTensor sinks, bool exact, long nsplit,
                     OptTensor slopes, double softcap) {
  chk(block_tables, "block_tables", at::kInt);
  chk(tiles, "tiles", at::kInt);
  chk(pos32, "pos32", at::kInt);
  const int q_bf = view_kind(q, "q");
  const int out_bf = view_kind(out, "out");
  TORCH_CHECK(act_kind(k_cache, "k_cache") == q_bf &&
              act_kind(v_cache, "v_cache") == q_bf,
              "q and the pools must share a dtype");
  TORCH_CHECK(q_bf || !out_bf, "fp32 q gives fp32 out");
  TORCH_CHECK(q.dim() == 3 && out.dim() == 3 && k_cache.dim() == 4 &&
              v_cache.dim() == 4);
  const int T = q.size(0), A = q.size(1), D = q.size(2);
  const int G = k_cache.size(1), BS = k_cache.size(2), KW = k_cache.size(3);
  const int VW = v_cache.size(2);
  TORCH_CHECK(v_cache.size(0) == k_cache.size(0) && v_cache.size(1) == G &&
              v_cache.size(3) == BS, "value pool must be [nblocks, G, VW, BS]");
  TORCH_CHECK(out.size(0) == T && out.size(1) == A && out.size(2) == VW);
  TORCH_CHECK((maps == 1 || maps == 2) && A % maps == 0 && KW == maps * D);
  const int H = A / maps;
  TORCH_CHECK(G >= 1 && H % G == 0, "heads must be a multiple of kv heads");
  const bool mfma = !exact && paged_attn_uses_mfma(q_bf, BS, D, VW);
  TORCH_CHECK(D >= 1 && VW >= 1 &&
              (mfma || (D <= paged_attn_max_dim() && VW <= paged_attn_max_dim())),
              "head size unsupported");
  TORCH_CHECK(block_tables.dim() == 2 && block_tables.size(1) >= 1 &&
              tiles.dim() == 2 && tiles.size(1) == 6 && pos32.numel() == T);
  TORCH_CHECK(window >= 0 && keep_first >= 0);
  const float* sp = nullptr;
  if (sinks.has_value()) {
    chk(*sinks, "sinks", at::kFloat);
    TORCH_CHECK(sinks->numel() == H);
    sp = sinks->data_ptr<float>();
  }
  const float* slp = nullptr;
  if (slopes.has_value()) {
    chk(*slopes, "slopes", at::kFloat);
    TORCH_CHECK(slopes->numel() == H);
    slp = slopes->data_ptr<float>();
  }
  if (!mfma) nsplit = 1;
  TORCH_CHECK(nsplit >= 1 && nsplit <= 64);
  const int ntiles = tiles.size(0);
  Tensor ws_acc, ws_ml;
  float *wa = nullptr, *wm = nullptr;
  if (nsplit > 1 && ntiles > 0) {
    auto opt = at::TensorOptions().dtype(at::kFloat).device(q.device());
    ws_acc = at::empty({(long)ntiles * nsplit * 16 * VW}, opt);
    ws_ml = at::empty({(long)ntiles * nsplit * 16 * 2}, opt);
    wa = ws_acc.data_ptr<float>();
    wm = ws_ml.data_ptr<float>();
  }
  paged_attention_launch(out.data_ptr(), q.data_ptr(), k_cache.data_ptr(),
                         v_cache.data_ptr(), block_tables.data_ptr<int>(),
                         tiles.data_ptr<int>(), pos32.data_ptr<int>(), sp, slp,
                         (float)scale, (float)softcap, q.stride(0), q.stride(1),
                         out.stride(0), out.stride(1), ntiles, T, A, D, VW, KW,
                         G, BS,
                         (int)maps, H / G, (int)block_tables.size(0),
                         (int)block_tables.size(1), (int)k_cache.size(0),
                         (int)window, (int)keep_first, q_bf, out_bf,
                         exact ? 1 : 0, (int)nsplit, wa, wm, cur_stream(q));
  HIP_CHECK_LAST();
}

bool paged_attention_uses_mfma(Tensor q, Tensor k_cache, Tensor v_cache) {
  return paged_attn_uses_mfma(q.scalar_type() == at::kBFloat16 ? 1 : 0,
                              (int)k_cache.size(2), (int)q.size(2),
                              (int)v_cache.size(2)) != 0;
}

void diff_combine(Tensor out, Tensor a, Tensor lam, double diff, double eps) {
  chk(a, "a", at::kFloat);
  chk(lam, "lam", at::kFloat);
  const int out_bf = act_kind(out, "out");
  TORCH_CHECK(a.dim() == 4 && a.size(2) == 2 && lam.numel() >= 1);
  const long n_heads = a.size(0) * a.size(1);
  const int VW = a.size(3);
  TORCH_CHECK(out.numel() == n_heads * VW);
  diff_combine_launch(out.data_ptr(), a.data_ptr<float>(),
                      lam.data_ptr<float>(), (float)diff, (float)eps, n_heads,
                      VW, out_bf, cur_stream(a));
  HIP_CHECK_LAST();
}

void act_and_mul(Tensor out, Tensor gu, long mode) {
  const int bf = act_kind(gu, "gu");
  TORCH_CHECK(act_kind(out, "out") == bf && gu.dim() == 2 && out.dim() == 2);
  TORCH_CHECK(out.size(0) == gu.size(0) && gu.size(1) == 2 * out.size(1));
  TORCH_CHECK(mode >= 0 && mode <= 3);
  act_and_mul_launch(out.data_ptr(), gu.data_ptr(), out.size(0),
                     (int)out.size(1), (int)mode, bf, cur_stream(gu));
  HIP_CHECK_LAST();
}

// one side (q or k) of head_rope_store: heads x dim channels from column col
void chk_rope_side(const char* name, long col, long heads, long dim,
                   const OptTensor& w, long nd, long rot0, long half,
                   long width) {
  TORCH_CHECK(heads >= 0 && (heads == 0 || (dim >= 1 && col >= 0 &&
              col + heads * dim <= width)), name, " columns outside the row");
  if (heads == 0) return;
  if (w.has_value()) {
    chk(*w, name, at::kFloat);
    TORCH_CHECK(nd >= 1 && nd <= dim && w->numel() == nd, name,
                " norm weight does not fit the normed channels");
  }
  TORCH_CHECK(rot0 < 0 || half == 0 || rot0 + 2 * half <= dim, name,
              " rotated channels outside the head");
}

void head_rope_store(OptTensor q_out, Tensor src, long col_q, long q_heads,
                     long q_dim, OptTensor q_w, long q_nd, long q_rot0,
                     long col_k, long k_heads, long k_dim, OptTensor k_w,
                     long k_nd, long k_rot0, long col_v, Tensor inv_freq,
                     bool half_layout, double amplitude, Tensor pos32,
                     OptTensor k_cache, OptTensor v_cache, OptTensor slots,
                     double eps, OptTensor page_groups) {
  TORCH_CHECK(src.is_cuda() && src.dim() == 2 && src.stride(1) == 1,
              "src must be [T, C] rows on GPU");
  const int bf = src.scalar_type() == at::kBFloat16 ? 1 : 0;
  TORCH_CHECK(bf || src.scalar_type() == at::kFloat, "src must be bf16 or fp32");
  chk(inv_freq, "inv_freq", at::kFloat);
  chk(pos32, "pos32", at::kInt);
  const int T = src.size(0);
  const long width = src.size(1), half = inv_freq.numel();
  TORCH_CHECK(pos32.numel() == T);
  if (!q_out.has_value()) q_heads = 0;
  if (!k_cache.has_value()) k_heads = 0;
  chk_rope_side("q side", col_q, q_heads, q_dim, q_w, q_nd, q_rot0, half, width);
  chk_rope_side("k side", col_k, k_heads, k_dim, k_w, k_nd, k_rot0, half, width);
  void *qp = nullptr, *kp = nullptr, *vp = nullptr;
  const long* sp = nullptr;
  long nslots = 0;
  int BS = 1, VW = 0;
  if (q_heads > 0) {
    TORCH_CHECK(act_kind(*q_out, "q_out") == bf && q_out->dim() == 2 &&
                q_out->size(0) == T && q_out->size(1) == q_heads * q_dim);
    TORCH_CHECK(q_out->data_ptr() != src.data_ptr(), "q_out must not alias src");
    qp = q_out->data_ptr();
  }
  if (k_heads > 0) {
    TORCH_CHECK(v_cache.has_value() && slots.has_value());
    TORCH_CHECK(act_kind(*k_cache, "k_cache") == bf &&
                act_kind(*v_cache, "v_cache") == bf,
                "src and the pools must share a dtype");
    chk(*slots, "slots", at::kLong);
    TORCH_CHECK(k_cache->dim() == 4 && v_cache->dim() == 4 &&
                slots->numel() == T);
    BS = k_cache->size(2);
    VW = v_cache->size(2);
    TORCH_CHECK(k_cache->size(1) == k_heads && k_cache->size(3) == k_dim,
                "key pool must be [nblocks, k_heads, BS, k_dim]");
    TORCH_CHECK(v_cache->size(0) == k_cache->size(0) &&
                v_cache->size(1) == k_heads && v_cache->size(3) == BS,
                "value pool must be [nblocks, k_heads, VW, BS]");
    TORCH_CHECK(col_v < 0 ? VW <= k_dim
                          : col_v + k_heads * (long)VW <= width,
                "value columns outside the row");
    kp = k_cache->data_ptr();
    vp = v_cache->data_ptr();
    sp = slots->data_ptr<long>();
    nslots = k_cache->size(0) * (long)BS;
  }
  // values page by page: from the projection's value columns, or — one key
  // head whose first channels are the values — from the key pool's rows
  // this launch has just written
  const bool by_page = page_groups.has_value() && k_heads > 0 &&
                       (col_v >= 0 || k_heads == 1);
  head_rope_store_launch(
      qp, src.data_ptr(), src.stride(0), (int)col_q, (int)q_heads, (int)q_dim,
      q_w.has_value() && q_heads > 0 ? q_w->data_ptr<float>() : nullptr,
      (int)q_nd, (int)q_rot0, (int)col_k, (int)k_heads, (int)k_dim,
      k_w.has_value() && k_heads > 0 ? k_w->data_ptr<float>() : nullptr,
      (int)k_nd, (int)k_rot0, (int)col_v, inv_freq.data_ptr<float>(),
      (int)half, half_layout ? 1 : 0, (float)amplitude, pos32.data_ptr<int>(),
      kp, vp, sp, nslots, BS, VW, (float)eps, by_page ? 1 : 0, T, bf,
      cur_stream(src));
  HIP_CHECK_LAST();
  if (by_page) {
    chk(*page_groups, "page_groups", at::kInt);
    TORCH_CHECK(BS == 16, "page-wise value stores need 16-token pages");
    TORCH_CHECK(page_groups->dim() == 2 && page_groups->size(1) == 2);
    if (col_v >= 0)
      value_page_store_launch(src.data_ptr(), src.stride(0), (int)col_v, vp,
                              sp, nslots, page_groups->data_ptr<int>(),
                              (int)page_groups->size(0), T, (int)k_heads, VW,
                              bf, 0, cur_stream(src));
    else
      value_page_store_launch(kp, k_dim, 0, vp, sp, nslots,
                              page_groups->data_ptr<int>(),
                              (int)page_groups->size(0), T, 1, VW, bf, 1,
                              cur_stream(src));
    HIP_CHECK_LAST();
  }
}

void dual_rms_mix(Tensor out, Tensor a, Tensor wa, Tensor b, Tensor wb,
                  double eps) {
  const int bf = act_kind(a, "a");
  TORCH_CHECK(act_kind(b, "b") == bf && act_kind(out, "out") == bf);
  chk(wa, "wa", at::kFloat);
  chk(wb, "wb", at::kFloat);
  TORCH_CHECK(a.dim() == 2 && b.sizes() == a.sizes() && out.sizes() == a.sizes());
  TORCH_CHECK(wa.numel() == a.size(1) && wb.numel() == a.size(1));
  dual_rms_mix_launch(out.data_ptr(), a.data_ptr(), wa.data_ptr<float>(),
                      b.data_ptr(), wb.data_ptr<float>(), (int)a.size(0),
                      (int)a.size(1), (float)eps, bf, cur_stream(a));
  HIP_CHECK_LAST();
}

void head_gate(Tensor out, Tensor o_hts, Tensor gate_src, long col) {
  const int bf = act_kind(o_hts, "o_hts");
  TORCH_CHECK(act_kind(out, "out") == bf && gate_src.is_cuda() &&
              gate_src.scalar_type() == o_hts.scalar_type() &&
              gate_src.dim() == 2 && gate_src.stride(1) == 1);
  TORCH_CHECK(o_hts.dim() == 3 && out.dim() == 2);
  const int H = o_hts.size(0), T = o_hts.size(1), VD = o_hts.size(2);
  TORCH_CHECK(out.size(0) == T && out.size(1) == (long)H * VD);
  TORCH_CHECK(gate_src.size(0) == T && col >= 0 && col + H <= gate_src.size(1));
  head_gate_launch(out.data_ptr(), o_hts.data_ptr(), gate_src.data_ptr(),
                   gate_src.stride(0), (int)col, H, T, VD, bf,
                   cur_stream(o_hts));
  HIP_CHECK_LAST();
}

void act_inplace(Tensor x, long mode) {
  const int bf = act_kind(x, "x");
  TORCH_CHECK(mode >= 0 && mode <= 3);
  act_inplace_launch(x.data_ptr(), x.numel(), (int)mode, bf, cur_stream(x));
  HIP_CHECK_LAST();
}

void argmax_f32(Tensor out, Tensor logits) {
  chk(out, "out", at::kLong);
  chk(logits, "logits", at::kFloat);
  TORCH_CHECK(logits.dim() == 2 && out.numel() == logits.size(0));
  argmax_f32_launch(out.data_ptr<long>(), logits.data_ptr<float>(),
                    (int)logits.size(0), (int)logits.size(1),
                    cur_stream(logits));
  HIP_CHECK_LAST();
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("embed_rows_f32", &embed_rows_f32);
  m.def("sandwich_add_norm", &sandwich_add_norm, py::arg("x"), py::arg("a"),
        py::arg("post_w"), py::arg("mult"), py::arg("eps"), py::arg("extra"),
        py::arg("next_w"), py::arg("h"), py::arg("center") = false);
  m.def("rotary_norm_store", &rotary_norm_store);
  m.def("paged_attention", &paged_attention, py::arg("out"), py::arg("q"),
        py::arg("k_cache"), py::arg("v_cache"), py::arg("block_tables"),
        py::arg("tiles"), py::arg("pos32"), py::arg("scale"), py::arg("maps"),
        py::arg("window"), py::arg("keep_first"), py::arg("sinks"),
        py::arg("exact"), py::arg("nsplit"), py::arg("slopes") = py::none(),
        py::arg("softcap") = 0.0);
  m.def("paged_attention_uses_mfma", &paged_attention_uses_mfma);
  m.def("diff_combine", &diff_combine);
  m.def("head_rope_store", &head_rope_store);
  m.def("dual_rms_mix", &dual_rms_mix);
  m.def("head_gate", &head_gate);
  m.def("act_inplace", &act_inplace);
  m.def("act_and_mul", &act_and_mul);
  m.def("argmax_f32", &argmax_f32);
}
