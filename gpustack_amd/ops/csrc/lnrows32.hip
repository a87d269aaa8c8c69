// Row kernels of the pre-norm fp32 stream with layer norms, of attention
// without rotation, and of scored expert routing (gfx950).
//
// The stream x [T, W] is fp32 and updated in place; statistics, norms, the
// query temperature and router scores are fp32 whatever the GEMM dtype is,
// and every kernel emits its GEMM operand in that dtype directly.
//
//   embed_rows_scaled : x = embed[token] * scale
//   add_layer_norm    : x += a;  h = (x - mean) / sqrt(var + eps) * w + b
//                       (closes one sublayer and opens the next in one
//                       pass; the row stays in registers between the two)
//   head_norm_store   : weighted RMS norm of every q / k head, query
//                       temperature, value blend, q out, k (and v) into
//                       their paged pools
//   route_topk        : sigmoid / softmax scores, choice correction,
//                       groups ranked by their best few, top-k, weights
#include "common.h"

namespace {

template <typename T> DEVICE_INLINE float ld(const T* p);
template <> DEVICE_INLINE float ld<float>(const float* p) { return *p; }
template <> DEVICE_INLINE float ld<unsigned short>(const unsigned short* p) {
  return bf2f(*p);
}
template <typename T> DEVICE_INLINE void st(T* p, float v);
template <> DEVICE_INLINE void st<float>(float* p, float v) { *p = v; }
template <> DEVICE_INLINE void st<unsigned short>(unsigned short* p, float v) {
  *p = f2bf(v);
}

constexpr int ROW_THREADS = 256;

DEVICE_INLINE float block_sum(float v, float* red) {
  v = wave_reduce_sum(v);
  const int w = threadIdx.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[w] = v;
  __syncthreads();
  return red[0] + red[1] + red[2] + red[3];
}

template <typename TW>
__global__ __launch_bounds__(ROW_THREADS) void embed_rows_scaled_kernel(
    float* __restrict__ x, const long* __restrict__ tokens,
    const TW* __restrict__ embed, int W, long vocab, float scale) {
  const long t = blockIdx.x;
  const long tok = min(max(tokens[t], 0L), vocab - 1);   // never read outside
  const TW* e = embed + tok * W;
  for (int i = threadIdx.x; i < W; i += ROW_THREADS)
    x[t * W + i] = ld(e + i) * scale;
}

// NV: row values each lane keeps in registers (W <= NV * 256); wider rows
// re-read x. Mean first, then the mean of the squared deviations.
template <typename TA, typename TH, int NV>
__global__ __launch_bounds__(ROW_THREADS) void add_layer_norm_kernel(
    float* __restrict__ x, const TA* __restrict__ a,
    const float* __restrict__ w, const float* __restrict__ b,
    TH* __restrict__ h, int W, float eps) {
  __shared__ float red[4];
  const long t = blockIdx.x;
  float* xr = x + t * W;
  float keep[NV];
  float sum = 0.f;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int i = threadIdx.x + j * ROW_THREADS;
    float v = 0.f;
    if (i < W) {
      v = xr[i];
      if (a != nullptr) {
        v += ld(a + t * W + i);
        xr[i] = v;
      }
    }
    keep[j] = v;
    sum += v;
  }
  for (int i = threadIdx.x + NV * ROW_THREADS; i < W; i += ROW_THREADS) {
    float v = xr[i];
    if (a != nullptr) {
      v += ld(a + t * W + i);
      xr[i] = v;
    }
    sum += v;
  }
  if (w == nullptr) return;
  const float mean = block_sum(sum, red) / (float)W;
  float sq = 0.f;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int i = threadIdx.x + j * ROW_THREADS;
    if (i < W) {
      const float d = keep[j] - mean;
      sq += d * d;
    }
  }
  for (int i = threadIdx.x + NV * ROW_THREADS; i < W; i += ROW_THREADS) {
    const float d = xr[i] - mean;
    sq += d * d;
  }
  const float inv = 1.0f / sqrtf(block_sum(sq, red) / (float)W + eps);
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int i = threadIdx.x + j * ROW_THREADS;
    if (i < W) st(h + t * W + i, (keep[j] - mean) * inv * w[i] + b[i]);
  }
  for (int i = threadIdx.x + NV * ROW_THREADS; i < W; i += ROW_THREADS)
    st(h + t * W + i, (xr[i] - mean) * inv * w[i] + b[i]);
}

// One workgroup per row; a wave takes one head at a time. Heads 0..HQ-1 are
// the queries, HQ..HQ+G-1 the keys; then the values, channel by channel.
// flags bit 0: values are stored by a later page-wise pass (the blend, if
// any, is written back into qkv for it).
template <typename TS, typename TC>
__global__ __launch_bounds__(ROW_THREADS) void head_norm_store_kernel(
    TS* __restrict__ q_out, TS* __restrict__ qkv, long ld_qkv, int nq, int nk,
    int nv, const float* __restrict__ q_w, const float* __restrict__ k_w,
    int D, float temp_coef, float temp_every, const int* __restrict__ pos32,
    const TS* __restrict__ v_first, long ld_vf, const float* __restrict__ lam,
    TC* __restrict__ k_cache, TC* __restrict__ v_cache,
    const long* __restrict__ slots, long nslots, int G, int BS, int VW,
    float eps, int flags) {
  const long t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  TS* row = qkv + t * ld_qkv;
  const long slot = slots[t];
  const bool keep = slot >= 0 && slot < nslots;
  const long blk = keep ? slot / BS : 0;
  const int off = keep ? (int)(slot % BS) : 0;
  float temp = 1.f;
  if (temp_every > 0.f) {
    // exact for whole-numbered steps while the position is below 2^24
    const int p = max(pos32[t], 0);
    temp = 1.f + temp_coef * logf(floorf((float)(p + 1) / temp_every) + 1.f);
  }
  const int HQ = nq / D;
  for (int hd = wave; hd < HQ + G; hd += 4) {
    const bool is_q = hd < HQ;
    const TS* src = row + (long)hd * D;      // q heads then k heads, in order
    float ss = 0.f;
    for (int c = lane; c < D; c += 64) {
      const float v = ld(src + c);
      ss += v * v;
    }
    ss = wave_reduce_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)D + eps);
    if (is_q) {
      TS* dst = q_out + t * nq + (long)hd * D;
      for (int c = lane; c < D; c += 64)
        st(dst + c, ld(src + c) * inv * q_w[c] * temp);
    } else if (keep) {
      TC* dst = k_cache + ((blk * G + (hd - HQ)) * BS + off) * (long)D;
      for (int c = lane; c < D; c += 64) st(dst + c, ld(src + c) * inv * k_w[c]);
    }
  }
  const bool later = flags & 1;
  if (later && v_first == nullptr) return;
  const float l = v_first != nullptr ? lam[0] : 0.f;
  TS* vr = row + nq + nk;
  for (int c = threadIdx.x; c < nv; c += ROW_THREADS) {
    float v = ld(vr + c);
    if (v_first != nullptr)
      v = (1.f - l) * v + l * ld(v_first + t * ld_vf + c);
    if (later) {
      st(vr + c, v);
    } else if (keep) {
      st(v_cache + ((blk * G + c / VW) * (long)VW + c % VW) * BS + off, v);
    }
  }
}

// (value, index) argmax over a wave; ties go to the lower index
DEVICE_INLINE void wave_argmax(float& v, int& idx) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) {
    const float ov = __shfl_xor(v, m, WAVE_SIZE);
    const int oi = __shfl_xor(idx, m, WAVE_SIZE);
    if (ov > v || (ov == v && oi < idx)) { v = ov; idx = oi; }
  }
}

constexpr int NONE = 0x7fffffff;

// One wave per token. smem: score[E], choice[E], gscore[G], then flags
// taken[E] and gkept[G] (ints). Choice scores may be negative, so taken
// experts and groups carry flags instead of marker values.
__global__ __launch_bounds__(64) void route_topk_kernel(
    int* __restrict__ experts, float* __restrict__ weights,
    const float* __restrict__ logits, int ld_logits,
    const float* __restrict__ correction, int E, int G, int keep,
    int group_top, int top, int use_sigmoid, int renorm, float scale) {
  extern __shared__ float sm[];
  float* score = sm;
  float* choice = score + E;
  float* gscore = choice + E;
  int* taken = reinterpret_cast<int*>(gscore + G);
  int* gkept = taken + E;
  const long t = blockIdx.x;
  const int lane = threadIdx.x;
  const float* z = logits + t * ld_logits;
  if (use_sigmoid) {
    for (int e = lane; e < E; e += 64) score[e] = 1.0f / (1.0f + expf(-z[e]));
  } else {
    float mx = -INFINITY;
    for (int e = lane; e < E; e += 64) mx = fmaxf(mx, z[e]);
    mx = wave_reduce_max(mx);
    float sum = 0.f;
    for (int e = lane; e < E; e += 64) {
      const float p = expf(z[e] - mx);
      score[e] = p;
      sum += p;
    }
    sum = wave_reduce_sum(sum);
    const float inv = 1.0f / sum;
    for (int e = lane; e < E; e += 64) score[e] *= inv;
  }
  for (int e = lane; e < E; e += 64) {
    choice[e] = score[e] + (correction != nullptr ? correction[e] : 0.f);
    taken[e] = 0;
  }
  __syncthreads();
  const int per = E / G;
  if (G > 1 && keep < G) {
    for (int g = lane; g < G; g += 64) {
      // sum of the group's group_top largest choice scores: repeated
      // selection with a "used below this rank" bound on (value, index)
      float total = 0.f;
      float pv = INFINITY;
      int pi = -1;
      const int n = min(group_top, per);
      for (int it = 0; it < n; ++it) {
        float bv = -INFINITY;
        int bi = NONE;
        for (int j = 0; j < per; ++j) {
          const float c = choice[g * per + j];
          const bool after = c < pv || (c == pv && j > pi);
          if (after && (c > bv || (c == bv && j < bi) || bi == NONE)) {
            bv = c;
            bi = j;
          }
        }
        if (bi == NONE) break;
        total += bv;
        pv = bv;
        pi = bi;
      }
      gscore[g] = total;
      gkept[g] = 0;
    }
    __syncthreads();
    for (int it = 0; it < keep; ++it) {
      float v = -INFINITY;
      int gi = NONE;
      for (int g = lane; g < G; g += 64)
        if (!gkept[g] && (gi == NONE || gscore[g] > v)) { v = gscore[g]; gi = g; }
      wave_argmax(v, gi);
      // lanes without a candidate carry (-inf, NONE); a real candidate of
      // value -inf still wins by its lower index
      if (lane == 0 && gi != NONE) gkept[gi] = 1;
      __syncthreads();
    }
  } else {
    for (int g = lane; g < G; g += 64) gkept[g] = 1;
    __syncthreads();
  }
  float wsum = 0.f;
  for (int it = 0; it < top; ++it) {
    float v = -INFINITY;
    int ei = NONE;
    for (int e = lane; e < E; e += 64)
      if (!taken[e] && gkept[e / per] && (ei == NONE || choice[e] > v)) {
        v = choice[e];
        ei = e;
      }
    wave_argmax(v, ei);
    const bool ok = ei != NONE;       // host checks keep * per >= top
    const float s = ok ? score[ei] : 0.f;
    wsum += s;
    if (lane == 0) {
      experts[t * top + it] = ok ? ei : 0;
      weights[t * top + it] = s;
      if (ok) taken[ei] = 1;
    }
    __syncthreads();
  }
  const float mul = renorm ? scale / (wsum + 1e-20f) : scale;
  for (int it = lane; it < top; it += 64) weights[t * top + it] *= mul;
}

template <typename TA, typename TH>
void aln_pick(float* x, const void* a, const float* w, const float* b, void* h,
              int T, int W, float eps, hipStream_t s) {
  if (W <= 1024)
    add_layer_norm_kernel<TA, TH, 4><<<T, ROW_THREADS, 0, s>>>(
        x, (const TA*)a, w, b, (TH*)h, W, eps);
  else if (W <= 2048)
    add_layer_norm_kernel<TA, TH, 8><<<T, ROW_THREADS, 0, s>>>(
        x, (const TA*)a, w, b, (TH*)h, W, eps);
  else
    add_layer_norm_kernel<TA, TH, 16><<<T, ROW_THREADS, 0, s>>>(
        x, (const TA*)a, w, b, (TH*)h, W, eps);
}

}  // namespace

// ---- launchers: `bf` flags say which operands are bf16 (else fp32) ----------

void embed_rows_scaled_launch(float* x, const long* tokens, const void* embed,
                              int T, int W, long vocab, float scale, int bf,
                              hipStream_t s) {
  if (T <= 0) return;
  if (bf)
    embed_rows_scaled_kernel<unsigned short><<<T, ROW_THREADS, 0, s>>>(
        x, tokens, (const unsigned short*)embed, W, vocab, scale);
  else
    embed_rows_scaled_kernel<float><<<T, ROW_THREADS, 0, s>>>(
        x, tokens, (const float*)embed, W, vocab, scale);
}

void add_layer_norm_launch(float* x, const void* a, const float* w,
                           const float* b, void* h, int T, int W, float eps,
                           int a_bf, int h_bf, hipStream_t s) {
  if (T <= 0) return;
  if (a_bf) {
    if (h_bf) aln_pick<unsigned short, unsigned short>(x, a, w, b, h, T, W, eps, s);
    else aln_pick<unsigned short, float>(x, a, w, b, h, T, W, eps, s);
  } else {
    if (h_bf) aln_pick<float, unsigned short>(x, a, w, b, h, T, W, eps, s);
    else aln_pick<float, float>(x, a, w, b, h, T, W, eps, s);
  }
}

void head_norm_store_launch(void* q_out, void* qkv, long ld_qkv, int nq, int nk,
                            int nv, const float* q_w, const float* k_w, int D,
                            float temp_coef, float temp_every, const int* pos32,
                            const void* v_first, long ld_vf, const float* lam,
                            void* k_cache, void* v_cache, const long* slots,
                            long nslots, int G, int BS, int VW, float eps,
                            int flags, int T, int bf, hipStream_t s) {
  if (T <= 0) return;
  if (bf)
    head_norm_store_kernel<unsigned short, unsigned short>
        <<<T, ROW_THREADS, 0, s>>>(
            (unsigned short*)q_out, (unsigned short*)qkv, ld_qkv, nq, nk, nv,
            q_w, k_w, D, temp_coef, temp_every, pos32,
            (const unsigned short*)v_first, ld_vf, lam,
            (unsigned short*)k_cache, (unsigned short*)v_cache, slots, nslots,
            G, BS, VW, eps, flags);
  else
    head_norm_store_kernel<float, float><<<T, ROW_THREADS, 0, s>>>(
        (float*)q_out, (float*)qkv, ld_qkv, nq, nk, nv, q_w, k_w, D, temp_coef,
        temp_every, pos32, (const float*)v_first, ld_vf, lam, (float*)k_cache,
        (float*)v_cache, slots, nslots, G, BS, VW, eps, flags);
}

void route_topk_launch(int* experts, float* weights, const float* logits,
                       int ld_logits, const float* correction, int T, int E,
                       int G, int keep, int group_top, int top, int use_sigmoid,
                       int renorm, float scale, hipStream_t s) {
  if (T <= 0) return;
  const size_t smem = (size_t)(3 * E + 2 * G) * sizeof(float);
  route_topk_kernel<<<T, 64, smem, s>>>(experts, weights, logits, ld_logits,
                                        correction, E, G, keep, group_top, top,
                                        use_sigmoid, renorm, scale);
}
