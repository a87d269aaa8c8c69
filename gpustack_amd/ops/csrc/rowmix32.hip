// Row kernels of the pre/post-norm fp32 stream and of paged rotary
// attention (gfx950).
//
// The stream x [T, W] is fp32 and updated in place. One workgroup of 256
// lanes (4 waves) handles one row; sums of squares, angles, rotations and
// norms are fp32 whatever the GEMM dtype is, and every kernel emits its
// GEMM operand in that dtype directly, so no cast pass runs between a row
// kernel and the projection that follows.
//
//   sandwich_add_norm : x += mult * rmsnorm(a) * post_w (+ extra);
//                       h = rmsnorm(x) * next_w          (closes one
//                       sublayer and opens the next in one pass; RMS norms
//                       or, centred, weight-only layer norms)
//   rotary_norm_store : optional whole-row RMS norm of q and k, pairwise
//                       rotary, q out, k and v into their paged pools
//   diff_combine      : unit_rms(a1 - lambda * a2) * (1 - diff) per head
//   act_and_mul       : act(gate) * up on the fused gate/up GEMM output
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
__global__ __launch_bounds__(ROW_THREADS) void embed_rows_kernel(
    float* __restrict__ x, const long* __restrict__ tokens,
    const TW* __restrict__ embed, int W, long vocab) {
  const long t = blockIdx.x;
  const long tok = min(max(tokens[t], 0L), vocab - 1);   // never read outside
  const TW* e = embed + tok * W;
  for (int i = threadIdx.x; i < W; i += ROW_THREADS) x[t * W + i] = ld(e + i);
}

// NV: row values each lane keeps in registers between the two halves
// (W <= NV * 256); wider rows re-read x. center: both norms take the row's
// mean off first (weight-only layer norms).
template <typename TA, typename TH, int NV>
__global__ __launch_bounds__(ROW_THREADS) void sandwich_add_norm_kernel(
    float* __restrict__ x, const TA* __restrict__ a,
    const float* __restrict__ post_w, float mult,
    const float* __restrict__ extra, const float* __restrict__ next_w,
    TH* __restrict__ h, int W, float eps, int center) {
  __shared__ float red[4];
  const long t = blockIdx.x;
  float* xr = x + t * W;
  float inv_a = 0.f, mean_a = 0.f;
  if (a != nullptr) {
    const TA* ar = a + t * W;
    if (center) {
      float s1 = 0.f;
      for (int i = threadIdx.x; i < W; i += ROW_THREADS) s1 += ld(ar + i);
      mean_a = block_sum(s1, red) / (float)W;
    }
    float ss = 0.f;
    for (int i = threadIdx.x; i < W; i += ROW_THREADS) {
      const float v = ld(ar + i) - mean_a;
      ss += v * v;
    }
    ss = block_sum(ss, red);
    inv_a = 1.0f / sqrtf(ss / (float)W + eps);
  }
  float keep[NV];
  float sx = 0.f, s1x = 0.f;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int i = threadIdx.x + j * ROW_THREADS;
    float v = 0.f;
    if (i < W) {
      v = xr[i];
      if (a != nullptr)
        v += ((ld(a + t * W + i) - mean_a) * inv_a * post_w[i]) * mult;
      if (extra != nullptr) v += extra[t * W + i];
      if (a != nullptr || extra != nullptr) xr[i] = v;
    }
    keep[j] = v;
    sx += v * v;
    s1x += v;
  }
  for (int i = threadIdx.x + NV * ROW_THREADS; i < W; i += ROW_THREADS) {
    float v = xr[i];
    if (a != nullptr)
      v += ((ld(a + t * W + i) - mean_a) * inv_a * post_w[i]) * mult;
    if (extra != nullptr) v += extra[t * W + i];
    if (a != nullptr || extra != nullptr) xr[i] = v;
    sx += v * v;
    s1x += v;
  }
  if (next_w == nullptr) return;
  float mean_x = 0.f;
  if (center) {
    // the deviations' squares, summed as such (no E[x^2] - mean^2)
    mean_x = block_sum(s1x, red) / (float)W;
    sx = 0.f;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int i = threadIdx.x + j * ROW_THREADS;
      if (i < W) sx += (keep[j] - mean_x) * (keep[j] - mean_x);
    }
    for (int i = threadIdx.x + NV * ROW_THREADS; i < W; i += ROW_THREADS)
      sx += (xr[i] - mean_x) * (xr[i] - mean_x);
  }
  sx = block_sum(sx, red);
  const float inv_x = 1.0f / sqrtf(sx / (float)W + eps);
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int i = threadIdx.x + j * ROW_THREADS;
    if (i < W) st(h + t * W + i, (keep[j] - mean_x) * inv_x * next_w[i]);
  }
  for (int i = threadIdx.x + NV * ROW_THREADS; i < W; i += ROW_THREADS)
    st(h + t * W + i, (xr[i] - mean_x) * inv_x * next_w[i]);
}

// W % 4 == 0 and W <= NV * 1024: four consecutive channels per lane and
// step (16-byte accesses on the fp32 stream, 8-byte ones on bf16 operands).
template <typename T> struct Vec4;
template <> struct Vec4<float> {
  static DEVICE_INLINE void load(const float* p, float* o) {
    const f32x4 v = *reinterpret_cast<const f32x4*>(p);
    o[0] = v[0]; o[1] = v[1]; o[2] = v[2]; o[3] = v[3];
  }
  static DEVICE_INLINE void store(float* p, const float* o) {
    *reinterpret_cast<f32x4*>(p) = f32x4{o[0], o[1], o[2], o[3]};
  }
};
template <> struct Vec4<unsigned short> {
  static DEVICE_INLINE void load(const unsigned short* p, float* o) {
    const u16x4 v = *reinterpret_cast<const u16x4*>(p);
    o[0] = bf2f(v[0]); o[1] = bf2f(v[1]); o[2] = bf2f(v[2]); o[3] = bf2f(v[3]);
  }
  static DEVICE_INLINE void store(unsigned short* p, const float* o) {
    *reinterpret_cast<u16x4*>(p) = u16x4{f2bf(o[0]), f2bf(o[1]), f2bf(o[2]), f2bf(o[3])};
  }
};

template <typename TA, typename TH, int NV>
__global__ __launch_bounds__(ROW_THREADS) void sandwich_add_norm_vec_kernel(
    float* __restrict__ x, const TA* __restrict__ a,
    const float* __restrict__ post_w, float mult,
    const float* __restrict__ extra, const float* __restrict__ next_w,
    TH* __restrict__ h, int W, float eps, int center) {
  __shared__ float red[4];
  const long t = blockIdx.x;
  float* xr = x + t * W;
  float av[NV][4];
  float inv_a = 0.f;
  if (a != nullptr) {
    float s1 = 0.f;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int i = (threadIdx.x + j * ROW_THREADS) * 4;
      if (i < W) {
        Vec4<TA>::load(a + t * W + i, av[j]);
        s1 += av[j][0] + av[j][1] + av[j][2] + av[j][3];
      }
    }
    const float mean_a = center ? block_sum(s1, red) / (float)W : 0.f;
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int i = (threadIdx.x + j * ROW_THREADS) * 4;
      if (i < W) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          av[j][k] -= mean_a;
          ss += av[j][k] * av[j][k];
        }
      }
    }
    ss = block_sum(ss, red);
    inv_a = 1.0f / sqrtf(ss / (float)W + eps);
  }
  float keep[NV][4];
  float sx = 0.f, s1x = 0.f;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int i = (threadIdx.x + j * ROW_THREADS) * 4;
    if (i < W) {
      Vec4<float>::load(xr + i, keep[j]);
      if (a != nullptr) {
        float w[4];
        Vec4<float>::load(post_w + i, w);
#pragma unroll
        for (int k = 0; k < 4; ++k) keep[j][k] += (av[j][k] * inv_a * w[k]) * mult;
      }
      if (extra != nullptr) {
        float e[4];
        Vec4<float>::load(extra + t * W + i, e);
#pragma unroll
        for (int k = 0; k < 4; ++k) keep[j][k] += e[k];
      }
      if (a != nullptr || extra != nullptr) Vec4<float>::store(xr + i, keep[j]);
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        sx += keep[j][k] * keep[j][k];
        s1x += keep[j][k];
      }
    }
  }
  if (next_w == nullptr) return;
  float mean_x = 0.f;
  if (center) {
    mean_x = block_sum(s1x, red) / (float)W;
    sx = 0.f;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int i = (threadIdx.x + j * ROW_THREADS) * 4;
      if (i < W) {
#pragma unroll
        for (int k = 0; k < 4; ++k)
          sx += (keep[j][k] - mean_x) * (keep[j][k] - mean_x);
      }
    }
  }
  sx = block_sum(sx, red);
  const float inv_x = 1.0f / sqrtf(sx / (float)W + eps);
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int i = (threadIdx.x + j * ROW_THREADS) * 4;
    if (i < W) {
      float w[4], o[4];
      Vec4<float>::load(next_w + i, w);
#pragma unroll
      for (int k = 0; k < 4; ++k) o[k] = (keep[j][k] - mean_x) * inv_x * w[k];
      Vec4<TH>::store(h + t * W + i, o);
    }
  }
}

// One workgroup per row. Lanes walk channel PAIRS (2i, 2i+1) of q, then of
// k, so a rotation needs no exchange between lanes. The value row (the
// raw key projection when tied) goes into the transposed value pages.
template <typename TS, typename TC>
__global__ __launch_bounds__(ROW_THREADS) void rotary_norm_store_kernel(
    TS* __restrict__ q_out, const TS* __restrict__ qkv, long ld_qkv, int nq,
    int nk, int nv, const float* __restrict__ q_norm_w,
    const float* __restrict__ k_norm_w, const float* __restrict__ inv_freq,
    int half, const int* __restrict__ pos32, int head_dim,
    TC* __restrict__ k_cache, TC* __restrict__ v_cache,
    const long* __restrict__ slots, long nslots, int G, int BS, int KW, int VW,
    float eps, int flags) {
  const bool tied = flags & 1, skip_v = flags & 2;
  __shared__ float red[4];
  extern __shared__ float cs_tab[];          // [half] cos, [half] sin
  const long t = blockIdx.x;
  const TS* row = qkv + t * ld_qkv;
  const float pos = (float)pos32[t];
  // every head turns by the same angles: one sin/cos pair per frequency
  for (int i = threadIdx.x; i < half; i += ROW_THREADS) {
    float sn, cs;
    sincosf(pos * inv_freq[i], &sn, &cs);
    cs_tab[i] = cs;
    cs_tab[half + i] = sn;
  }
  if (q_norm_w == nullptr) __syncthreads();   // block_sum syncs otherwise
  float inv_q = 1.f, inv_k = 1.f;
  if (q_norm_w != nullptr) {
    float sq = 0.f, sk = 0.f;
    for (int i = threadIdx.x; i < nq; i += ROW_THREADS) {
      const float v = ld(row + i);
      sq += v * v;
    }
    for (int i = threadIdx.x; i < nk; i += ROW_THREADS) {
      const float v = ld(row + nq + i);
      sk += v * v;
    }
    sq = block_sum(sq, red);
    sk = block_sum(sk, red);
    inv_q = 1.0f / sqrtf(sq / (float)nq + eps);
    inv_k = 1.0f / sqrtf(sk / (float)nk + eps);
  }
  const long slot = slots[t];
  const bool store = slot >= 0 && slot < nslots;
  const long blk = store ? slot / BS : 0;
  const int off = store ? (int)(slot % BS) : 0;
  // head_dim is even or carries no rotation: pairs never straddle heads
  const int npq = nq / 2, npk = nk / 2;
  for (int p = threadIdx.x; p < npq + npk; p += ROW_THREADS) {
    const bool is_k = p >= npq;
    const int c = 2 * (is_k ? p - npq : p);          // channel in q or k
    const TS* src = row + (is_k ? nq : 0) + c;
    float u = ld(src), v = ld(src + 1);
    if (q_norm_w != nullptr) {
      const float* w = is_k ? k_norm_w : q_norm_w;
      const float inv = is_k ? inv_k : inv_q;
      u = u * inv * w[c];
      v = v * inv * w[c + 1];
    }
    const int d = c % head_dim;
    if (d < 2 * half) {
      const float cs = cs_tab[d >> 1], sn = cs_tab[half + (d >> 1)];
      const float u2 = u * cs - v * sn;
      v = v * cs + u * sn;
      u = u2;
    }
    if (!is_k) {
      st(q_out + t * nq + c, u);
      st(q_out + t * nq + c + 1, v);
    } else if (store) {
      const int g = c / KW, kc = c % KW;
      TC* dst = k_cache + ((blk * G + g) * BS + off) * (long)KW + kc;
      st(dst, u);
      st(dst + 1, v);
    }
  }
  if (nq & 1) {   // odd widths carry no rotation; copy the last channel
    if (threadIdx.x == 0) {
      float u = ld(row + nq - 1);
      if (q_norm_w != nullptr) u = u * inv_q * q_norm_w[nq - 1];
      st(q_out + t * nq + nq - 1, u);
    }
  }
  if ((nk & 1) && store && threadIdx.x == 0) {
    const int c = nk - 1;
    float u = ld(row + nq + c);
    if (k_norm_w != nullptr) u = u * inv_k * k_norm_w[c];
    st(k_cache + ((blk * G + c / KW) * BS + off) * (long)KW + c % KW, u);
  }
  if (store && !skip_v) {
    const TS* vs = tied ? row + nq : row + nq + nk;
    const int n = G * VW;
    for (int i = threadIdx.x; i < n; i += ROW_THREADS) {
      const int g = i / VW, c = i % VW;
      st(v_cache + ((blk * G + g) * (long)VW + c) * BS + off, ld(vs + i));
    }
  }
}

// bf16 with every width a multiple of 8: 16 bytes per lane, ONE WAVE per
// row (four rows per workgroup): the sums of squares reduce with shuffles,
// so a row costs no workgroup barrier besides the one behind the sin/cos
// table. A lane takes 8 consecutive channels (4 rotation pairs) of q or k,
// then 8 of v.
__global__ __launch_bounds__(ROW_THREADS) void rotary_norm_store_vec_kernel(
    unsigned short* __restrict__ q_out, const unsigned short* __restrict__ qkv,
    long ld_qkv, int nq, int nk, const float* __restrict__ q_norm_w,
    const float* __restrict__ k_norm_w, const float* __restrict__ inv_freq,
    int half, const int* __restrict__ pos32, int head_dim,
    unsigned short* __restrict__ k_cache, unsigned short* __restrict__ v_cache,
    const long* __restrict__ slots, long nslots, int G, int BS, int KW, int VW,
    float eps, int flags, int T) {
  const bool tied = flags & 1, skip_v = flags & 2;
  extern __shared__ float cs_all[];              // [4][2 * half]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const long t = (long)blockIdx.x * 4 + wave;
  const bool live = t < T;
  float* cs_tab = cs_all + wave * 2 * half;
  const unsigned short* row = qkv + (live ? t : 0) * ld_qkv;
  const float pos = live ? (float)pos32[t] : 0.f;
  for (int i = lane; i < half; i += 64) {
    float sn, cs;
    sincosf(pos * inv_freq[i], &sn, &cs);
    cs_tab[i] = cs;
    cs_tab[half + i] = sn;
  }
  __syncthreads();
  if (!live) return;
  float inv_q = 1.f, inv_k = 1.f;
  if (q_norm_w != nullptr) {
    float sq = 0.f, sk = 0.f;
    for (int c = lane * 8; c < nq + nk; c += 64 * 8) {
      const u16x8 v = *reinterpret_cast<const u16x8*>(row + c);
      float ss = 0.f;
#pragma unroll
      for (int k = 0; k < 8; ++k) { const float f = bf2f(v[k]); ss += f * f; }
      if (c < nq) sq += ss; else sk += ss;
    }
    sq = wave_reduce_sum(sq);
    sk = wave_reduce_sum(sk);
    inv_q = 1.0f / sqrtf(sq / (float)nq + eps);
    inv_k = 1.0f / sqrtf(sk / (float)nk + eps);
  }
  const long slot = slots[t];
  const bool store = slot >= 0 && slot < nslots;
  const long blk = store ? slot / BS : 0;
  const int off = store ? (int)(slot % BS) : 0;
  for (int c0 = lane * 8; c0 < nq + nk; c0 += 64 * 8) {
    const bool is_k = c0 >= nq;
    const int c = is_k ? c0 - nq : c0;
    const u16x8 raw = *reinterpret_cast<const u16x8*>(row + c0);
    float f[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) f[k] = bf2f(raw[k]);
    if (q_norm_w != nullptr) {
      const float* w = (is_k ? k_norm_w : q_norm_w) + c;
      const float inv = is_k ? inv_k : inv_q;
      const f32x4 w0 = *reinterpret_cast<const f32x4*>(w);
      const f32x4 w1 = *reinterpret_cast<const f32x4*>(w + 4);
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        f[k] = f[k] * inv * w0[k];
        f[4 + k] = f[4 + k] * inv * w1[k];
      }
    }
    const int d = c % head_dim;
#pragma unroll
    for (int k = 0; k < 8; k += 2) {
      if (d + k < 2 * half) {
        const int i = (d + k) >> 1;
        const float cs = cs_tab[i], sn = cs_tab[half + i];
        const float u2 = f[k] * cs - f[k + 1] * sn;
        f[k + 1] = f[k + 1] * cs + f[k] * sn;
        f[k] = u2;
      }
    }
    u16x8 o;
#pragma unroll
    for (int k = 0; k < 8; ++k) o[k] = f2bf(f[k]);
    if (!is_k) {
      *reinterpret_cast<u16x8*>(q_out + t * nq + c) = o;
    } else if (store) {
      const int g = c / KW, kc = c % KW;
      *reinterpret_cast<u16x8*>(
          k_cache + ((blk * G + g) * BS + off) * (long)KW + kc) = o;
    }
  }
  if (store && !skip_v) {
    const unsigned short* vs = tied ? row + nq : row + nq + nk;
    const int n = G * VW;
    for (int i = lane * 8; i < n; i += 64 * 8) {
      const u16x8 v = *reinterpret_cast<const u16x8*>(vs + i);
      const int g = i / VW, c = i % VW;
      unsigned short* dst = v_cache + ((blk * G + g) * (long)VW + c) * BS + off;
#pragma unroll
      for (int k = 0; k < 8; ++k) dst[(long)k * BS] = v[k];
    }
  }
}

// Value rows of a prompt into the transposed value pages, a page at a
// time. groups: int32 [n, 2] = first row, rows (<= 16) of runs that fall into
// ONE page in order (host-built from the batch's sequences). The source is
// the projection (row = batch row) or, by_slot, a row-major pool (row =
// slot). A run that
// fills its whole page leaves as 16 keys per channel in one piece (32 bytes
// of bf16 per lane, neighbouring lanes neighbouring channels); any other
// run falls back to one store per (row, channel). CH channels at a time go
// through LDS, which turns the row-major projection into page columns.
template <typename TS, int CH>
__global__ __launch_bounds__(ROW_THREADS) void value_page_store_kernel(
    const TS* __restrict__ qkv, long ld_qkv, int v_col0,
    TS* __restrict__ v_cache, const long* __restrict__ slots, long nslots,
    const int* __restrict__ groups, int T, int G, int VW, int by_slot) {
  constexpr int BS = 16;
  __shared__ TS tile[BS][CH + 8];
  __shared__ long s_slot[BS];
  const int row0 = groups[2 * blockIdx.x], nrows = groups[2 * blockIdx.x + 1];
  if (row0 < 0 || nrows < 1 || nrows > BS || row0 + nrows > T) return;
  const int tid = threadIdx.x;
  if (tid < BS) s_slot[tid] = tid < nrows ? slots[row0 + tid] : -1;
  __syncthreads();
  bool fast = nrows == BS && s_slot[0] >= 0 && s_slot[0] % BS == 0 &&
              s_slot[0] + BS <= nslots;
#pragma unroll
  for (int r = 1; r < BS; ++r) fast = fast && s_slot[r] == s_slot[0] + r;
  const int C = G * VW;
  for (int c0 = 0; c0 < C; c0 += CH) {
    const int cw = min(CH, C - c0);
    __syncthreads();
    for (int i = tid; i < nrows * cw; i += ROW_THREADS) {
      const int r = i / cw, c = i % cw;
      // by_slot: the source is a row-major pool indexed like the slots (a
      // key pool whose rows' first channels are the values)
      long srow = row0 + r;
      if (by_slot) srow = min(max(s_slot[r], 0L), nslots - 1);
      tile[r][c] = qkv[srow * ld_qkv + v_col0 + c0 + c];
    }
    __syncthreads();
    if (fast) {
      const long blk = s_slot[0] / BS;
      for (int c = tid; c < cw; c += ROW_THREADS) {
        const int cc = c0 + c;
        TS* dst = v_cache + ((blk * G + cc / VW) * (long)VW + cc % VW) * BS;
        TS col[BS];
#pragma unroll
        for (int r = 0; r < BS; ++r) col[r] = tile[r][c];
        constexpr int PER = 16 / sizeof(TS);       // elements per 16 bytes
        typedef TS vec_t __attribute__((ext_vector_type(PER)));
#pragma unroll
        for (int v = 0; v < BS / PER; ++v) {
          vec_t o;
#pragma unroll
          for (int k = 0; k < PER; ++k) o[k] = col[v * PER + k];
          reinterpret_cast<vec_t*>(dst)[v] = o;
        }
      }
    } else {
      for (int i = tid; i < nrows * cw; i += ROW_THREADS) {
        const int r = i % nrows, c = i / nrows;
        const long slot = s_slot[r];
        if (slot < 0 || slot >= nslots) continue;
        const int cc = c0 + c;
        v_cache[(((slot / BS) * G + cc / VW) * (long)VW + cc % VW) * BS +
                slot % BS] = tile[r][c];
      }
    }
  }
}

// One wave per (row, head): a [T, H, 2, VW] fp32 -> out [T, H*VW].
template <typename TO>
__global__ __launch_bounds__(ROW_THREADS) void diff_combine_kernel(
    TO* __restrict__ out, const float* __restrict__ a,
    const float* __restrict__ lam_p, float diff, float eps, long n_heads,
    int VW) {
  const long e = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (e >= n_heads) return;
  const int lane = threadIdx.x & 63;
  const float lam = lam_p[0];
  const float* a1 = a + e * 2 * VW;
  const float* a2 = a1 + VW;
  float ss = 0.f;
  for (int i = lane; i < VW; i += 64) {
    const float o = a1[i] - lam * a2[i];
    ss += o * o;
  }
  ss = wave_reduce_sum(ss);
  const float inv = (1.0f / sqrtf(ss / (float)VW + eps)) * (1.0f - diff);
  for (int i = lane; i < VW; i += 64)
    st(out + e * VW + i, (a1[i] - lam * a2[i]) * inv);
}

DEVICE_INLINE float act_fn(float z, int mode) {
  switch (mode) {
    case 0: { const float r = fmaxf(z, 0.f); return r * r; }
    case 1: return 0.5f * z * (1.0f + erff(z * 0.70710678118654752f));
    case 2: {
      const float u = 0.7978845608028654f * (z + 0.044715f * z * z * z);
      return 0.5f * z * (1.0f + tanhf(u));
    }
    default: return z / (1.0f + expf(-z));
  }
}

template <typename T>
__global__ void act_and_mul_kernel(T* __restrict__ out, const T* __restrict__ gu,
                                   long rows, int F, int mode) {
  const long n = rows * F;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (long)gridDim.x * blockDim.x) {
    const long r = i / F;
    const int c = (int)(i % F);
    const float g = ld(gu + r * 2 * F + c);
    const float u = ld(gu + r * 2 * F + F + c);
    st(out + i, act_fn(g, mode) * u);
  }
}

// bf16, F % 8 == 0: 16 bytes per lane and operand. The tanh form of GELU
// is z * sigmoid(2u), one exponential per element.
DEVICE_INLINE float act_fast(float z, int mode) {
  if (mode == 2) {
    const float u = 0.7978845608028654f * (z + 0.044715f * z * z * z);
    return z / (1.0f + __expf(-2.0f * u));
  }
  if (mode == 3) return z / (1.0f + __expf(-z));
  return act_fn(z, mode);
}

template <int MODE>
__global__ __launch_bounds__(256) void act_and_mul_vec_kernel(
    unsigned short* __restrict__ out, const unsigned short* __restrict__ gu,
    long rows, int F8) {
  const long n = rows * F8;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (long)gridDim.x * blockDim.x) {
    const long r = i / F8;
    const int c = (int)(i % F8);
    const u16x8* gp = reinterpret_cast<const u16x8*>(gu) + r * 2 * F8 + c;
    const u16x8 g = gp[0], u = gp[F8];
    u16x8 o;
#pragma unroll
    for (int k = 0; k < 8; ++k)
      o[k] = f2bf(act_fast(bf2f(g[k]), MODE) * bf2f(u[k]));
    reinterpret_cast<u16x8*>(out)[i] = o;
  }
}

}  // namespace

void embed_rows_f32_launch(float* x, const long* tokens, const void* embed,
                           int T, int W, long vocab, int bf, hipStream_t s) {
  if (T <= 0) return;
  if (bf)
    embed_rows_kernel<unsigned short><<<T, ROW_THREADS, 0, s>>>(
        x, tokens, (const unsigned short*)embed, W, vocab);
  else
    embed_rows_kernel<float><<<T, ROW_THREADS, 0, s>>>(
        x, tokens, (const float*)embed, W, vocab);
}

template <typename TA, typename TH>
static void sandwich_pick(float* x, const void* a, const float* post_w,
                          float mult, const float* extra, const float* next_w,
                          void* h, int T, int W, float eps, int center,
                          hipStream_t s) {
#define SW_ARGS x, (const TA*)a, post_w, mult, extra, next_w, (TH*)h, W, eps, center
  if (W % 4 == 0 && W <= 8 * 1024) {
    if (W <= 1024)
      sandwich_add_norm_vec_kernel<TA, TH, 1><<<T, ROW_THREADS, 0, s>>>(SW_ARGS);
    else if (W <= 2048)
      sandwich_add_norm_vec_kernel<TA, TH, 2><<<T, ROW_THREADS, 0, s>>>(SW_ARGS);
    else if (W <= 4096)
      sandwich_add_norm_vec_kernel<TA, TH, 4><<<T, ROW_THREADS, 0, s>>>(SW_ARGS);
    else
      sandwich_add_norm_vec_kernel<TA, TH, 8><<<T, ROW_THREADS, 0, s>>>(SW_ARGS);
  } else if (W <= 4 * ROW_THREADS) {
    sandwich_add_norm_kernel<TA, TH, 4><<<T, ROW_THREADS, 0, s>>>(SW_ARGS);
  } else {
    sandwich_add_norm_kernel<TA, TH, 16><<<T, ROW_THREADS, 0, s>>>(SW_ARGS);
  }
#undef SW_ARGS
}

// a_bf / h_bf: element type of a and h (1 = bf16, 0 = fp32)
void sandwich_add_norm_launch(float* x, const void* a, const float* post_w,
                              float mult, const float* extra,
                              const float* next_w, void* h, int T, int W,
                              float eps, int a_bf, int h_bf, int center,
                              hipStream_t s) {
  if (T <= 0) return;
  if (a_bf && h_bf)
    sandwich_pick<unsigned short, unsigned short>(x, a, post_w, mult, extra, next_w, h, T, W, eps, center, s);
  else if (a_bf)
    sandwich_pick<unsigned short, float>(x, a, post_w, mult, extra, next_w, h, T, W, eps, center, s);
  else if (h_bf)
    sandwich_pick<float, unsigned short>(x, a, post_w, mult, extra, next_w, h, T, W, eps, center, s);
  else
    sandwich_pick<float, float>(x, a, post_w, mult, extra, next_w, h, T, W, eps, center, s);
}

void rotary_norm_store_launch(void* q_out, const void* qkv, long ld_qkv, int nq,
                              int nk, int nv, const float* q_norm_w,
                              const float* k_norm_w, const float* inv_freq,
                              int half, const int* pos32, int head_dim,
                              void* k_cache, void* v_cache, const long* slots,
                              long nslots, int G, int BS, int KW, int VW,
                              float eps, int flags, int T, int bf,
                              hipStream_t s) {
  const int tied = flags;   // bit 0: tied values, bit 1: values stored elsewhere
  if (T <= 0) return;
  const size_t tab = (size_t)2 * half * sizeof(float);
  if (bf && nq % 8 == 0 && nk % 8 == 0 && nv % 8 == 0 && head_dim % 8 == 0 &&
      KW % 8 == 0 && VW % 8 == 0 && ld_qkv % 8 == 0) {
    rotary_norm_store_vec_kernel<<<(T + 3) / 4, ROW_THREADS, 4 * tab, s>>>(
        (unsigned short*)q_out, (const unsigned short*)qkv, ld_qkv, nq, nk,
        q_norm_w, k_norm_w, inv_freq, half, pos32, head_dim,
        (unsigned short*)k_cache, (unsigned short*)v_cache, slots, nslots, G,
        BS, KW, VW, eps, tied, T);
    return;
  }
  if (bf)
    rotary_norm_store_kernel<unsigned short, unsigned short>
        <<<T, ROW_THREADS, tab, s>>>(
            (unsigned short*)q_out, (const unsigned short*)qkv, ld_qkv, nq, nk,
            nv, q_norm_w, k_norm_w, inv_freq, half, pos32, head_dim,
            (unsigned short*)k_cache, (unsigned short*)v_cache, slots, nslots,
            G, BS, KW, VW, eps, tied);
  else
    rotary_norm_store_kernel<float, float><<<T, ROW_THREADS, tab, s>>>(
        (float*)q_out, (const float*)qkv, ld_qkv, nq, nk, nv, q_norm_w,
        k_norm_w, inv_freq, half, pos32, head_dim, (float*)k_cache,
        (float*)v_cache, slots, nslots, G, BS, KW, VW, eps, tied);
}

void value_page_store_launch(const void* qkv, long ld_qkv, int v_col0,
                             void* v_cache, const long* slots, long nslots,
                             const int* groups, int ngroups, int T, int G,
                             int VW, int bf, int by_slot, hipStream_t s) {
  if (ngroups <= 0) return;
  if (bf)
    value_page_store_kernel<unsigned short, 1024><<<ngroups, ROW_THREADS, 0, s>>>(
        (const unsigned short*)qkv, ld_qkv, v_col0, (unsigned short*)v_cache,
        slots, nslots, groups, T, G, VW, by_slot);
  else
    value_page_store_kernel<float, 512><<<ngroups, ROW_THREADS, 0, s>>>(
        (const float*)qkv, ld_qkv, v_col0, (float*)v_cache, slots, nslots,
        groups, T, G, VW, by_slot);
}

void diff_combine_launch(void* out, const float* a, const float* lam,
                         float diff, float eps, long n_heads, int VW,
                         int out_bf, hipStream_t s) {
  if (n_heads <= 0) return;
  const int grid = (int)((n_heads + 3) / 4);
  if (out_bf)
    diff_combine_kernel<unsigned short><<<grid, ROW_THREADS, 0, s>>>(
        (unsigned short*)out, a, lam, diff, eps, n_heads, VW);
  else
    diff_combine_kernel<float><<<grid, ROW_THREADS, 0, s>>>(
        (float*)out, a, lam, diff, eps, n_heads, VW);
}

void act_and_mul_launch(void* out, const void* gu, long rows, int F, int mode,
                        int bf, hipStream_t s) {
  const long n = rows * F;
  if (n <= 0) return;
  if (bf && F % 8 == 0) {
    const long n8 = n / 8;
    const int g8 = (int)min((n8 + 255) / 256, (long)(256 * 64));
    auto* o = (unsigned short*)out;
    auto* g = (const unsigned short*)gu;
    switch (mode) {
      case 0: act_and_mul_vec_kernel<0><<<g8, 256, 0, s>>>(o, g, rows, F / 8); break;
      case 1: act_and_mul_vec_kernel<1><<<g8, 256, 0, s>>>(o, g, rows, F / 8); break;
      case 2: act_and_mul_vec_kernel<2><<<g8, 256, 0, s>>>(o, g, rows, F / 8); break;
      default: act_and_mul_vec_kernel<3><<<g8, 256, 0, s>>>(o, g, rows, F / 8); break;
    }
    return;
  }
  const int grid = (int)min((n + 255) / 256, (long)(256 * 32));
  if (bf)
    act_and_mul_kernel<unsigned short><<<grid, 256, 0, s>>>(
        (unsigned short*)out, (const unsigned short*)gu, rows, F, mode);
  else
    act_and_mul_kernel<float><<<grid, 256, 0, s>>>(
        (float*)out, (const float*)gu, rows, F, mode);
}
