// Row kernels for models with an fp32 residual stream (gfx950).
//
// The stream x [T, W] is fp32 and updated in place; every kernel that
// changes it can also emit the row in the GEMM dtype (bf16), so the next
// projection needs no separate cast pass. Sums of squares, softmax scores,
// gates and weighted sums are fp32 whatever the GEMM dtype is. One
// workgroup of 256 lanes (4 waves) handles one row; rows of a few hundred
// to a few thousand channels keep every lane busy and the two passes over
// the row stay in L1/L2.
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

// sum over the 256-lane workgroup; every lane gets the result
DEVICE_INLINE float block_sum(float v, float* red) {
  v = wave_reduce_sum(v);
  const int w = threadIdx.x >> 6;
  __syncthreads();               // red may still be read from a previous use
  if ((threadIdx.x & 63) == 0) red[w] = v;
  __syncthreads();
  return red[0] + red[1] + red[2] + red[3];
}

template <typename TW, typename TH>
__global__ __launch_bounds__(ROW_THREADS) void embed_pair_hash_kernel(
    float* __restrict__ x, TH* __restrict__ h, const long* __restrict__ tokens,
    const long* __restrict__ prev, const TW* __restrict__ embed,
    const TW* __restrict__ pair, int W, long vocab, long buckets,
    long mul_prev, long mul_cur) {
  const long t = blockIdx.x;
  const long tok = min(max(tokens[t], 0L), vocab - 1);   // never read outside
  const TW* e = embed + tok * W;
  const TW* b = nullptr;
  if (pair != nullptr) {
    const long p = prev[t];
    const long row = p < 0 ? buckets : (p * mul_prev + tok * mul_cur) % buckets;
    b = pair + row * W;
  }
  for (int i = threadIdx.x; i < W; i += ROW_THREADS) {
    float v = ld(e + i);
    if (b != nullptr) v += ld(b + i);
    x[t * W + i] = v;
    if (h != nullptr) st(h + t * W + i, v);
  }
}

// x += a * rsqrt(mean(a^2) + eps) * w [* s];  h = cast(x)
template <typename TA, typename TH>
__global__ __launch_bounds__(ROW_THREADS) void rms_scale_add_kernel(
    float* __restrict__ x, const TA* __restrict__ a,
    const float* __restrict__ w, const float* __restrict__ s,
    TH* __restrict__ h, int W, float eps) {
  __shared__ float red[4];
  const long t = blockIdx.x;
  const TA* ar = a + t * W;
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += ROW_THREADS) {
    const float v = ld(ar + i);
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += ROW_THREADS) {
    float y = ld(ar + i) * inv * w[i];
    if (s != nullptr) y *= s[i];
    const float v = x[t * W + i] + y;
    x[t * W + i] = v;
    if (h != nullptr) st(h + t * W + i, v);
  }
}

template <typename TO>
__global__ __launch_bounds__(ROW_THREADS) void rms_norm_f32_kernel(
    TO* __restrict__ out, const float* __restrict__ x,
    const float* __restrict__ w, int W, float eps) {
  __shared__ float red[4];
  const long t = blockIdx.x;
  const float* xr = x + t * W;
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += ROW_THREADS) ss += xr[i] * xr[i];
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += ROW_THREADS)
    st(out + t * W + i, xr[i] * inv * w[i]);
}

// Second pool plane for a group of 16 rows whose normalised values sit in
// LDS (tile[r * LS + i]). The usual case inside a prompt — the 16 rows fill
// one whole 16-token page in order — writes each channel's 16 offsets as 32
// bytes per lane; otherwise one two-byte store per (row, channel), row index
// fastest over the lanes so neighbours still share 32-byte segments.
template <typename TC>
DEVICE_INLINE void store_transposed_plane(TC* __restrict__ cache,
                                          const TC* tile, int LS,
                                          const long* s_slot, int R, int BS,
                                          long page_stride, int tid) {
  bool whole_page = BS == 16 && s_slot[0] >= 0 && s_slot[0] % 16 == 0;
#pragma unroll
  for (int r = 1; r < 16; ++r) whole_page = whole_page && s_slot[r] == s_slot[0] + r;
  if (sizeof(TC) == 2 && whole_page) {           // uniform over the workgroup
    unsigned short* tp = reinterpret_cast<unsigned short*>(
        cache + (s_slot[0] / 16) * page_stride + (long)BS * R);
    const unsigned short* tl = reinterpret_cast<const unsigned short*>(tile);
    for (int i = tid; i < R; i += ROW_THREADS) {
      u16x8 lo, hi;
#pragma unroll
      for (int r = 0; r < 8; ++r) {
        lo[r] = tl[r * LS + i];
        hi[r] = tl[(r + 8) * LS + i];
      }
      *reinterpret_cast<u16x8*>(tp + (long)i * 16) = lo;
      *reinterpret_cast<u16x8*>(tp + (long)i * 16 + 8) = hi;
    }
    return;
  }
  for (int idx = tid; idx < 16 * R; idx += ROW_THREADS) {
    const int r = idx & 15, i = idx >> 4;
    const long slot = s_slot[r];
    if (slot < 0) continue;
    cache[(slot / BS) * page_stride + (long)BS * R + (long)i * BS + slot % BS] =
        tile[r * LS + i];
  }
}

// Normalise src[t, col0:col0+R] and write it to its pool slot: plane 0 of
// the page row-major, plane 1 (when the pool has it) transposed [R][BS].
// A workgroup takes 16 consecutive rows (one wave normalises four of them)
// and keeps the results in LDS, so the transposed plane is written with the
// ROW index running fastest over the lanes: rows of a prompt portion sit at
// consecutive offsets of one page, and their 16 two-byte stores per channel
// then fill whole 32-byte segments instead of one segment each.
template <typename TS, typename TC>
__global__ __launch_bounds__(ROW_THREADS) void latent_norm_store_kernel(
    TC* __restrict__ cache, const TS* __restrict__ src, long ld_src, int col0,
    const float* __restrict__ w, const long* __restrict__ slots, int T, int R,
    int BS, int planes, long nslots, float eps) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lraw[];
  TC* tile = reinterpret_cast<TC*>(lraw);       // [16][R + 2] when planes == 2
  const int LS = R + 2;
  __shared__ long s_slot[16];
  const int t0 = blockIdx.x * 16;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const long page_stride = (long)planes * BS * R;
  if (tid < 16) {
    long sl = -1;
    if (t0 + tid < T) {
      sl = slots[t0 + tid];
      if (sl < 0 || sl >= nslots) sl = -1;      // skipped, never written
    }
    s_slot[tid] = sl;
  }
  __syncthreads();
  for (int rr = wave; rr < 16; rr += 4) {
    const long slot = s_slot[rr];
    if (slot < 0) continue;                     // uniform over the wave
    const TS* sr = src + (long)(t0 + rr) * ld_src + col0;
    float ss = 0.f;
    for (int i = lane; i < R; i += 64) {
      const float v = ld(sr + i);
      ss += v * v;
    }
    ss = wave_reduce_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)R + eps);
    TC* row = cache + (slot / BS) * page_stride + (slot % BS) * R;
    for (int i = lane; i < R; i += 64) {
      const float v = ld(sr + i) * inv * w[i];
      st(row + i, v);
      if (planes == 2) st(tile + rr * LS + i, v);
    }
  }
  if (planes != 2) return;
  __syncthreads();
  store_transposed_plane(cache, tile, LS, s_slot, R, BS, page_stride, tid);
}

// bf16 rows whose latent slice is 16-byte aligned (R, col0, row stride all
// multiples of 8): 16 lanes per row, all 16 rows of the group at once, eight
// channels per load — the whole group's loads are in flight together.
__global__ __launch_bounds__(ROW_THREADS) void latent_norm_store_vec_kernel(
    unsigned short* __restrict__ cache, const unsigned short* __restrict__ src,
    long ld_src, int col0, const float* __restrict__ w,
    const long* __restrict__ slots, int T, int R, int BS, int planes,
    long nslots, float eps) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lraw[];
  unsigned short* tile = reinterpret_cast<unsigned short*>(lraw);  // [16][R + 8]
  const int LS = R + 8;
  __shared__ long s_slot[16];
  const int t0 = blockIdx.x * 16;
  const int tid = threadIdx.x;
  const int r = tid >> 4, l16 = tid & 15;
  const long page_stride = (long)planes * BS * R;
  if (tid < 16) {
    long sl = -1;
    if (t0 + tid < T) {
      sl = slots[t0 + tid];
      if (sl < 0 || sl >= nslots) sl = -1;
    }
    s_slot[tid] = sl;
  }
  __syncthreads();
  const long slot = s_slot[r];
  const bool valid = slot >= 0;
  const unsigned short* sr = src + (long)(t0 + r) * ld_src + col0;
  const int nvec = R / 8;
  u16x8 xs[8];                       // R <= 1024: at most 8 vectors per lane
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int v = l16 + 16 * j;
    xs[j] = u16x8{0, 0, 0, 0, 0, 0, 0, 0};
    if (valid && v < nvec) xs[j] = *reinterpret_cast<const u16x8*>(sr + v * 8);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const float f = bf2f(xs[j][k]);
      ss += f * f;
    }
  }
  ss = group16_reduce_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)R + eps);
  if (valid) {
    unsigned short* row = cache + (slot / BS) * page_stride + (slot % BS) * R;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int v = l16 + 16 * j;
      if (v < nvec) {
        u16x8 y;
#pragma unroll
        for (int k = 0; k < 8; ++k)
          y[k] = f2bf(bf2f(xs[j][k]) * inv * w[v * 8 + k]);
        *reinterpret_cast<u16x8*>(row + v * 8) = y;
        if (planes == 2) *reinterpret_cast<u16x8*>(tile + r * LS + v * 8) = y;
      }
    }
  }
  if (planes != 2) return;
  __syncthreads();
  store_transposed_plane(cache, tile, LS, s_slot, R, BS, page_stride, tid);
}

// The same for a handful of rows (decode): one workgroup per row keeps
// every load of the row in flight at once; the transposed plane takes one
// two-byte store per channel, which is all a single new token can fill.
template <typename TS, typename TC>
__global__ __launch_bounds__(ROW_THREADS) void latent_norm_store_row_kernel(
    TC* __restrict__ cache, const TS* __restrict__ src, long ld_src, int col0,
    const float* __restrict__ w, const long* __restrict__ slots, int R,
    int BS, int planes, long nslots, float eps) {
  __shared__ float red[4];
  const long t = blockIdx.x;
  const long slot = slots[t];
  if (slot < 0 || slot >= nslots) return;   // uniform over the workgroup
  const TS* sr = src + t * ld_src + col0;
  float ss = 0.f;
  for (int i = threadIdx.x; i < R; i += ROW_THREADS) {
    const float v = ld(sr + i);
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)R + eps);
  TC* page = cache + (slot / BS) * ((long)planes * BS * R);
  const int off = (int)(slot % BS);
  for (int i = threadIdx.x; i < R; i += ROW_THREADS) {
    const float v = ld(sr + i) * inv * w[i];
    st(page + (long)off * R + i, v);
    if (planes == 2) st(page + (long)BS * R + (long)i * BS + off, v);
  }
}

DEVICE_INLINE float act_apply(float z, int mode) {
  switch (mode) {
    case 0: { const float r = fmaxf(z, 0.f); return r * r; }          // relu^2
    case 1: return 0.5f * z * (1.0f + erff(z * 0.70710678118654752f)); // gelu
    case 2: {                                                        // tanh gelu
      const float u = 0.7978845608028654f * (z + 0.044715f * z * z * z);
      return 0.5f * z * (1.0f + tanhf(u));
    }
    default: return z / (1.0f + expf(-z));                            // silu
  }
}

template <typename T>
__global__ void act_inplace_kernel(T* __restrict__ x, long n, int mode) {
  const long stride = (long)gridDim.x * blockDim.x;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    st(x + i, act_apply(ld(x + i), mode));
}

// bf16, n % 8 == 0: 16 bytes per lane. The tanh form of GELU is
// z * sigmoid(2u), one exponential per element.
template <int MODE>
__global__ __launch_bounds__(256) void act_inplace_vec_kernel(
    unsigned short* __restrict__ x, long n8) {
  const long stride = (long)gridDim.x * blockDim.x;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n8; i += stride) {
    const u16x8 v = reinterpret_cast<const u16x8*>(x)[i];
    u16x8 o;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const float z = bf2f(v[k]);
      float r;
      if (MODE == 2) {
        const float u = 0.7978845608028654f * (z + 0.044715f * z * z * z);
        r = z / (1.0f + __expf(-2.0f * u));
      } else if (MODE == 3) {
        r = z / (1.0f + __expf(-z));
      } else {
        r = act_apply(z, MODE);
      }
      o[k] = f2bf(r);
    }
    reinterpret_cast<u16x8*>(x)[i] = o;
  }
}

__global__ void softcap_kernel(float* __restrict__ x, long n, float cap) {
  const long stride = (long)gridDim.x * blockDim.x;
  const float inv = 1.0f / cap;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    x[i] = cap * tanhf(x[i] * inv);
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

// One wave per token. smem: score[E] then group_best[G].
__global__ __launch_bounds__(64) void route_grouped_topk_kernel(
    int* __restrict__ experts, float* __restrict__ weights,
    const float* __restrict__ logits, int ld_logits, int E, int G, int keep,
    int top, float scale) {
  extern __shared__ float sm[];
  float* score = sm;
  float* gbest = sm + E;
  const long t = blockIdx.x;
  const int lane = threadIdx.x;
  const float* z = logits + t * ld_logits;
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
  __syncthreads();
  const int per = E / G;
  if (G > 1 && keep < G) {
    for (int g = lane; g < G; g += 64) {
      float b = -1.f;
      for (int j = 0; j < per; ++j) b = fmaxf(b, score[g * per + j]);
      gbest[g] = b;
    }
    __syncthreads();
    // take the `keep` best groups one at a time; a taken group's entry
    // becomes -2 (scores are >= 0, so the marker cannot collide)
    for (int it = 0; it < keep; ++it) {
      float v = -INFINITY;
      int gi = 0x7fffffff;
      for (int g = lane; g < G; g += 64)
        if (gbest[g] >= 0.f && (gbest[g] > v)) { v = gbest[g]; gi = g; }
      wave_argmax(v, gi);
      if (lane == 0 && gi != 0x7fffffff) gbest[gi] = -2.f;
      __syncthreads();
    }
  } else {
    for (int g = lane; g < G; g += 64) gbest[g] = -2.f;
    __syncthreads();
  }
  // top-k over experts of taken groups; a chosen expert's score is kept in
  // the output and its slot is negated so it cannot be chosen twice
  for (int it = 0; it < top; ++it) {
    float v = -INFINITY;
    int ei = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      const float sc = score[e];
      if (sc >= 0.f && gbest[e / per] == -2.f && sc > v) { v = sc; ei = e; }
    }
    wave_argmax(v, ei);
    if (lane == 0) {
      const bool ok = ei != 0x7fffffff;   // host checks keep*per >= top
      experts[t * top + it] = ok ? ei : 0;
      weights[t * top + it] = ok ? v * scale : 0.f;
      if (ok) score[ei] = -1.f;
    }
    __syncthreads();
  }
}

// out[t] = sum_k wt[t,k] * y[inv[t,k]] + sigmoid(gate[t]) * shared[t]
template <typename TY>
__global__ __launch_bounds__(ROW_THREADS) void moe_combine_kernel(
    float* __restrict__ out, const TY* __restrict__ y,
    const int* __restrict__ inv, const float* __restrict__ wt,
    const TY* __restrict__ shared, const float* __restrict__ gate,
    int ld_gate, int gate_col, int W, int top, int ny) {
  const long t = blockIdx.x;
  float g = 1.f;
  if (shared != nullptr && gate != nullptr) {
    const float z = gate[t * ld_gate + gate_col];
    g = 1.0f / (1.0f + expf(-z));
  }
  for (int i = threadIdx.x; i < W; i += ROW_THREADS) {
    float acc = 0.f;
    for (int k = 0; k < top; ++k)
      acc += wt[t * top + k] *
             ld(y + (long)min(max(inv[t * top + k], 0), ny - 1) * W + i);
    if (shared != nullptr) acc += g * ld(shared + t * W + i);
    out[t * W + i] = acc;
  }
}

__global__ __launch_bounds__(ROW_THREADS) void argmax_f32_kernel(
    long* __restrict__ out, const float* __restrict__ logits, int V) {
  __shared__ float bv[4];
  __shared__ int bi[4];
  const long t = blockIdx.x;
  const float* z = logits + t * V;
  float v = -INFINITY;
  int idx = 0x7fffffff;
  for (int i = threadIdx.x; i < V; i += ROW_THREADS)
    if (z[i] > v) { v = z[i]; idx = i; }
  wave_argmax(v, idx);
  if ((threadIdx.x & 63) == 0) { bv[threadIdx.x >> 6] = v; bi[threadIdx.x >> 6] = idx; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; ++w)
      if (bv[w] > v || (bv[w] == v && bi[w] < idx)) { v = bv[w]; idx = bi[w]; }
    out[t] = idx == 0x7fffffff ? 0 : idx;
  }
}

}  // namespace

// ---- launchers: `bf` flags say which operands are bf16 (else fp32) ----------

void embed_pair_hash_launch(float* x, void* h, const long* tokens,
                            const long* prev, const void* embed,
                            const void* pair, int T, int W, long vocab,
                            long buckets, long mul_prev, long mul_cur,
                            int table_bf, hipStream_t s) {
  if (T == 0) return;
  if (table_bf)
    embed_pair_hash_kernel<unsigned short, unsigned short>
        <<<T, ROW_THREADS, 0, s>>>(x, (unsigned short*)h, tokens, prev,
                                   (const unsigned short*)embed,
                                   (const unsigned short*)pair, W, vocab,
                                   buckets, mul_prev, mul_cur);
  else
    embed_pair_hash_kernel<float, float><<<T, ROW_THREADS, 0, s>>>(
        x, (float*)h, tokens, prev, (const float*)embed, (const float*)pair,
        W, vocab, buckets, mul_prev, mul_cur);
}

void rms_scale_add_launch(float* x, const void* a, const float* w,
                          const float* sc, void* h, int T, int W, float eps,
                          int a_bf, hipStream_t s) {
  if (T == 0) return;
  // h, when given, is bf16 (an fp32 engine reads the stream itself)
  if (a_bf)
    rms_scale_add_kernel<unsigned short, unsigned short>
        <<<T, ROW_THREADS, 0, s>>>(x, (const unsigned short*)a, w, sc,
                                   (unsigned short*)h, W, eps);
  else
    rms_scale_add_kernel<float, unsigned short><<<T, ROW_THREADS, 0, s>>>(
        x, (const float*)a, w, sc, (unsigned short*)h, W, eps);
}

void rms_norm_f32_launch(void* out, const float* x, const float* w, int T,
                         int W, float eps, int out_bf, hipStream_t s) {
  if (T == 0) return;
  if (out_bf)
    rms_norm_f32_kernel<unsigned short><<<T, ROW_THREADS, 0, s>>>(
        (unsigned short*)out, x, w, W, eps);
  else
    rms_norm_f32_kernel<float><<<T, ROW_THREADS, 0, s>>>((float*)out, x, w, W,
                                                         eps);
}

void latent_norm_store_launch(void* cache, const void* src, long ld_src,
                              int col0, const float* w, const long* slots,
                              int T, int R, int BS, int planes, long nslots,
                              float eps, int bf, hipStream_t s) {
  if (T == 0) return;
  if (T < 128) {
    if (bf)
      latent_norm_store_row_kernel<unsigned short, unsigned short>
          <<<T, ROW_THREADS, 0, s>>>((unsigned short*)cache,
                                     (const unsigned short*)src, ld_src, col0,
                                     w, slots, R, BS, planes, nslots, eps);
    else
      latent_norm_store_row_kernel<float, float><<<T, ROW_THREADS, 0, s>>>(
          (float*)cache, (const float*)src, ld_src, col0, w, slots, R, BS,
          planes, nslots, eps);
    return;
  }
  const int groups = (T + 15) / 16;
  if (bf && R % 8 == 0 && R <= 1024 && col0 % 8 == 0 && ld_src % 8 == 0 &&
      ((uintptr_t)src & 15) == 0 && ((uintptr_t)cache & 15) == 0) {
    const size_t vsmem = planes == 2 ? (size_t)16 * (R + 8) * 2 : 0;
    latent_norm_store_vec_kernel<<<groups, ROW_THREADS, vsmem, s>>>(
        (unsigned short*)cache, (const unsigned short*)src, ld_src, col0, w,
        slots, T, R, BS, planes, nslots, eps);
    return;
  }
  const size_t smem = planes == 2 ? (size_t)16 * (R + 2) * (bf ? 2 : 4) : 0;
  if (bf)
    latent_norm_store_kernel<unsigned short, unsigned short>
        <<<groups, ROW_THREADS, smem, s>>>((unsigned short*)cache,
                                           (const unsigned short*)src, ld_src,
                                           col0, w, slots, T, R, BS, planes,
                                           nslots, eps);
  else
    latent_norm_store_kernel<float, float><<<groups, ROW_THREADS, smem, s>>>(
        (float*)cache, (const float*)src, ld_src, col0, w, slots, T, R, BS,
        planes, nslots, eps);
}

void act_inplace_launch(void* x, long n, int mode, int bf, hipStream_t s) {
  if (n == 0) return;
  const int blocks = (int)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096);
  if (bf && n % 8 == 0 && ((uintptr_t)x % 16) == 0) {
    const long n8 = n / 8;
    const int b8 = (int)((n8 + 255) / 256 < 16384 ? (n8 + 255) / 256 : 16384);
    auto* xp = (unsigned short*)x;
    switch (mode) {
      case 0: act_inplace_vec_kernel<0><<<b8, 256, 0, s>>>(xp, n8); break;
      case 1: act_inplace_vec_kernel<1><<<b8, 256, 0, s>>>(xp, n8); break;
      case 2: act_inplace_vec_kernel<2><<<b8, 256, 0, s>>>(xp, n8); break;
      default: act_inplace_vec_kernel<3><<<b8, 256, 0, s>>>(xp, n8); break;
    }
    return;
  }
  if (bf)
    act_inplace_kernel<unsigned short><<<blocks, 256, 0, s>>>(
        (unsigned short*)x, n, mode);
  else
    act_inplace_kernel<float><<<blocks, 256, 0, s>>>((float*)x, n, mode);
}

void softcap_launch(float* x, long n, float cap, hipStream_t s) {
  if (n == 0) return;
  const int blocks = (int)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096);
  softcap_kernel<<<blocks, 256, 0, s>>>(x, n, cap);
}

void route_grouped_topk_launch(int* experts, float* weights,
                               const float* logits, int ld_logits, int T,
                               int E, int G, int keep, int top, float scale,
                               hipStream_t s) {
  if (T == 0) return;
  const size_t smem = (size_t)(E + G) * sizeof(float);
  route_grouped_topk_kernel<<<T, 64, smem, s>>>(experts, weights, logits,
                                                ld_logits, E, G, keep, top,
                                                scale);
}

void moe_combine_launch(float* out, const void* y, const int* inv,
                        const float* wt, const void* shared, const float* gate,
                        int ld_gate, int gate_col, int T, int W, int top,
                        int bf, hipStream_t s) {
  if (T == 0) return;
  if (bf)
    moe_combine_kernel<unsigned short><<<T, ROW_THREADS, 0, s>>>(
        out, (const unsigned short*)y, inv, wt, (const unsigned short*)shared,
        gate, ld_gate, gate_col, W, top, T * top);
  else
    moe_combine_kernel<float><<<T, ROW_THREADS, 0, s>>>(
        out, (const float*)y, inv, wt, (const float*)shared, gate, ld_gate,
        gate_col, W, top, T * top);
}

void argmax_f32_launch(long* out, const float* logits, int N, int V,
                       hipStream_t s) {
  if (N == 0) return;
  argmax_f32_kernel<<<N, ROW_THREADS, 0, s>>>(out, logits, V);
}
