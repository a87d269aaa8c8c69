// Row kernels around attention mixers whose heads are normed and rotated
// one by one (gfx950).
//
//   head_rope_store : per head of a q side and a k side of one projection
//                     row: RMS norm of the head's first channels with a
//                     weight vector shared by the heads, then rotation of a
//                     channel range (pairs (i, i + half) or (2i, 2i + 1),
//                     cos / sin times an amplitude); q heads out, k heads
//                     into their page rows, values into the transposed
//                     value pages — from the projection, or the first
//                     channels of the finished key head (a latent that is
//                     key and value at once)
//   dual_rms_mix    : (rmsnorm(a) * wa + rmsnorm(b) * wb) / 2 per row
//   head_gate       : head-major outputs -> rows, each head times the
//                     sigmoid of its gate logit
//
// Sums of squares, angles, rotations and gates are fp32 whatever the GEMM
// dtype; every kernel emits its operand in that dtype directly.
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

struct RopeArgs {
  long ld_src;
  int col_q, q_heads, q_dim, q_nd, q_rot0;
  int col_k, k_heads, k_dim, k_nd, k_rot0;
  int col_v;                 // < 0: values are the key heads' first VW channels
  const float* q_w;          // [q_nd] or null
  const float* k_w;          // [k_nd] or null
  const float* inv_freq;     // [half]
  int half, half_layout;
  float amp, eps;
  const int* pos32;
  const long* slots;
  long nslots;
  int BS, VW, skip_v, T;
};

// grid (T, ceil((q_heads + k_heads) / 4)): one wave per (row, head). The
// sin / cos table of the row is built once per workgroup in LDS.
template <typename TS>
__global__ __launch_bounds__(ROW_THREADS) void head_rope_store_kernel(
    TS* __restrict__ q_out, const TS* __restrict__ src,
    TS* __restrict__ k_cache, TS* __restrict__ v_cache, RopeArgs p) {
  extern __shared__ float cs_tab[];            // [half] cos, [half] sin
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int half = p.half;
  const float pos = (float)p.pos32[t];
  for (int i = threadIdx.x; i < half; i += ROW_THREADS) {
    float sn, cs;
    sincosf(pos * p.inv_freq[i], &sn, &cs);
    cs_tab[i] = cs * p.amp;
    cs_tab[half + i] = sn * p.amp;
  }
  __syncthreads();
  const int unit = blockIdx.y * 4 + wave;
  if (unit >= p.q_heads + p.k_heads) return;
  const bool is_k = unit >= p.q_heads;
  const int hd = is_k ? unit - p.q_heads : unit;
  const int dim = is_k ? p.k_dim : p.q_dim;
  const int nd = is_k ? p.k_nd : p.q_nd;
  const int rot0 = is_k ? p.k_rot0 : p.q_rot0;
  const float* w = is_k ? p.k_w : p.q_w;
  const TS* row = src + (long)t * p.ld_src + (is_k ? p.col_k : p.col_q) +
                  (long)hd * dim;
  float inv = 1.f;
  if (w != nullptr) {
    float ss = 0.f;
    for (int c = lane; c < nd; c += 64) {
      const float v = ld(row + c);
      ss += v * v;
    }
    ss = wave_reduce_sum(ss);
    inv = 1.0f / sqrtf(ss / (float)nd + p.eps);
  }
  long blk = 0;
  int off = 0;
  bool store = false;
  if (is_k) {
    const long slot = p.slots[t];
    store = slot >= 0 && slot < p.nslots;
    if (!store) return;
    blk = slot / p.BS;
    off = (int)(slot % p.BS);
  }
  const int G = p.k_heads;
  for (int c = lane; c < dim; c += 64) {
    float v = ld(row + c);
    if (w != nullptr && c < nd) v = v * inv * w[c];
    const int r = c - rot0;
    if (rot0 >= 0 && r >= 0 && r < 2 * half) {
      int i, pc;
      bool lower;
      if (p.half_layout) {
        lower = r < half;
        i = lower ? r : r - half;
        pc = lower ? c + half : c - half;
      } else {
        lower = (r & 1) == 0;
        i = r >> 1;
        pc = lower ? c + 1 : c - 1;
      }
      float o = ld(row + pc);
      if (w != nullptr && pc < nd) o = o * inv * w[pc];
      const float cs = cs_tab[i], sn = cs_tab[half + i];
      v = lower ? v * cs - o * sn : v * cs + o * sn;
    }
    if (!is_k) {
      st(q_out + ((long)t * p.q_heads + hd) * dim + c, v);
    } else {
      st(k_cache + ((blk * G + hd) * p.BS + off) * (long)dim + c, v);
      if (p.col_v < 0 && !p.skip_v && c < p.VW)
        st(v_cache + ((blk * G + hd) * (long)p.VW + c) * p.BS + off, v);
    }
  }
  if (is_k && p.col_v >= 0 && !p.skip_v) {
    const TS* vs = src + (long)t * p.ld_src + p.col_v + (long)hd * p.VW;
    for (int c = lane; c < p.VW; c += 64)
      v_cache[((blk * G + hd) * (long)p.VW + c) * p.BS + off] = vs[c];
  }
}


// bf16 with every size, column and rotation boundary a multiple of 8: a lane
// takes 8 consecutive channels of its head (16 bytes) per step, LPH lanes
// share a head (the smallest power of two that covers the widest head in
// one step, at most a wave) and a wave takes 64 / LPH heads. A rotated piece
// in the (i, i + half) layout fetches its partner piece as well, in the
// (2i, 2i + 1) layout the partners sit in the same piece.
template <int LPH>
__global__ __launch_bounds__(ROW_THREADS) void head_rope_store_vec_kernel(
    unsigned short* __restrict__ q_out, const unsigned short* __restrict__ src,
    unsigned short* __restrict__ k_cache, unsigned short* __restrict__ v_cache,
    RopeArgs p) {
  constexpr int HPW = 64 / LPH;                // heads per wave
  extern __shared__ float cs_tab[];            // [half] cos, [half] sin
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int sub = lane % LPH;
  const int half = p.half;
  const float pos = (float)p.pos32[t];
  for (int i = threadIdx.x; i < half; i += ROW_THREADS) {
    float sn, cs;
    sincosf(pos * p.inv_freq[i], &sn, &cs);
    cs_tab[i] = cs * p.amp;
    cs_tab[half + i] = sn * p.amp;
  }
  __syncthreads();
  const int unit = (blockIdx.y * 4 + wave) * HPW + lane / LPH;
  const bool active = unit < p.q_heads + p.k_heads;
  const bool is_k = unit >= p.q_heads;
  const int hd = is_k ? unit - p.q_heads : unit;
  const int dim = !active ? 0 : is_k ? p.k_dim : p.q_dim;
  const int nd = is_k ? p.k_nd : p.q_nd;
  const int rot0 = is_k ? p.k_rot0 : p.q_rot0;
  const float* w = is_k ? p.k_w : p.q_w;
  const unsigned short* row = src + (long)t * p.ld_src +
                              (is_k ? p.col_k : p.col_q) + (long)hd * dim;
  float inv = 1.f;
  {
    // every lane walks the shuffles; heads without a norm add nothing
    float ss = 0.f;
    if (w != nullptr)
      for (int c = sub * 8; c < min(nd, dim); c += LPH * 8) {
        const u16x8 v = *reinterpret_cast<const u16x8*>(row + c);
#pragma unroll
        for (int k = 0; k < 8; ++k) { const float f = bf2f(v[k]); ss += f * f; }
      }
#pragma unroll
    for (int m = LPH / 2; m >= 1; m >>= 1) ss += __shfl_xor(ss, m, WAVE_SIZE);
    if (w != nullptr) inv = 1.0f / sqrtf(ss / (float)nd + p.eps);
  }
  if (!active) return;
  long blk = 0;
  int off = 0;
  if (is_k) {
    const long slot = p.slots[t];
    if (slot < 0 || slot >= p.nslots) return;
    blk = slot / p.BS;
    off = (int)(slot % p.BS);
  }
  const int G = p.k_heads;
  auto piece = [&](int c, float* f) {
    const u16x8 v = *reinterpret_cast<const u16x8*>(row + c);
#pragma unroll
    for (int k = 0; k < 8; ++k) f[k] = bf2f(v[k]);
    if (w != nullptr && c < nd) {
      const f32x4 w0 = *reinterpret_cast<const f32x4*>(w + c);
      const f32x4 w1 = *reinterpret_cast<const f32x4*>(w + c + 4);
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        f[k] = f[k] * inv * w0[k];
        f[4 + k] = f[4 + k] * inv * w1[k];
      }
    }
  };
  for (int c = sub * 8; c < dim; c += LPH * 8) {
    float f[8];
    piece(c, f);
    const int r = c - rot0;
    if (rot0 >= 0 && r >= 0 && r < 2 * half) {
      if (p.half_layout) {
        const bool lower = r < half;
        const int i0 = lower ? r : r - half;
        float o[8];
        piece(lower ? c + half : c - half, o);
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          const float cs = cs_tab[i0 + k], sn = cs_tab[half + i0 + k];
          f[k] = lower ? f[k] * cs - o[k] * sn : f[k] * cs + o[k] * sn;
        }
      } else {
#pragma unroll
        for (int k = 0; k < 8; k += 2) {
          const int i = (r + k) >> 1;
          const float cs = cs_tab[i], sn = cs_tab[half + i];
          const float u2 = f[k] * cs - f[k + 1] * sn;
          f[k + 1] = f[k + 1] * cs + f[k] * sn;
          f[k] = u2;
        }
      }
    }
    u16x8 o8;
#pragma unroll
    for (int k = 0; k < 8; ++k) o8[k] = f2bf(f[k]);
    if (!is_k) {
      *reinterpret_cast<u16x8*>(q_out + ((long)t * p.q_heads + hd) * dim + c) = o8;
    } else {
      *reinterpret_cast<u16x8*>(
          k_cache + ((blk * G + hd) * p.BS + off) * (long)dim + c) = o8;
      if (p.col_v < 0 && !p.skip_v && c < p.VW) {
        unsigned short* dst =
            v_cache + ((blk * G + hd) * (long)p.VW + c) * p.BS + off;
#pragma unroll
        for (int k = 0; k < 8; ++k) dst[(long)k * p.BS] = o8[k];
      }
    }
  }
  if (is_k && p.col_v >= 0 && !p.skip_v) {
    const unsigned short* vs = src + (long)t * p.ld_src + p.col_v + (long)hd * p.VW;
    for (int c = sub * 8; c < p.VW; c += LPH * 8) {
      const u16x8 v = *reinterpret_cast<const u16x8*>(vs + c);
      unsigned short* dst =
          v_cache + ((blk * G + hd) * (long)p.VW + c) * p.BS + off;
#pragma unroll
      for (int k = 0; k < 8; ++k) dst[(long)k * p.BS] = v[k];
    }
  }
}

DEVICE_INLINE float block_sum(float v, float* red) {
  v = wave_reduce_sum(v);
  const int w = threadIdx.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[w] = v;
  __syncthreads();
  return red[0] + red[1] + red[2] + red[3];
}

// One workgroup per row; NV values of each input stay in registers between
// the sums of squares and the store (W <= NV * 256), wider rows re-read.
template <typename TS, int NV>
__global__ __launch_bounds__(ROW_THREADS) void dual_rms_mix_kernel(
    TS* __restrict__ out, const TS* __restrict__ a, const float* __restrict__ wa,
    const TS* __restrict__ b, const float* __restrict__ wb, int W, float eps) {
  __shared__ float red[4];
  const long t = blockIdx.x;
  const TS* ar = a + t * W;
  const TS* br = b + t * W;
  float ka[NV], kb[NV];
  float sa = 0.f, sb = 0.f;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int i = threadIdx.x + j * ROW_THREADS;
    ka[j] = i < W ? ld(ar + i) : 0.f;
    kb[j] = i < W ? ld(br + i) : 0.f;
    sa += ka[j] * ka[j];
    sb += kb[j] * kb[j];
  }
  for (int i = threadIdx.x + NV * ROW_THREADS; i < W; i += ROW_THREADS) {
    const float x = ld(ar + i), y = ld(br + i);
    sa += x * x;
    sb += y * y;
  }
  sa = block_sum(sa, red);
  sb = block_sum(sb, red);
  const float ia = 1.0f / sqrtf(sa / (float)W + eps);
  const float ib = 1.0f / sqrtf(sb / (float)W + eps);
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int i = threadIdx.x + j * ROW_THREADS;
    if (i < W)
      st(out + t * W + i, 0.5f * (ka[j] * ia * wa[i] + kb[j] * ib * wb[i]));
  }
  for (int i = threadIdx.x + NV * ROW_THREADS; i < W; i += ROW_THREADS)
    st(out + t * W + i,
       0.5f * (ld(ar + i) * ia * wa[i] + ld(br + i) * ib * wb[i]));
}

// W % 4 == 0 and W <= NV * 1024: four consecutive channels per lane and step,
// both rows in registers between the sums of squares and the store.
template <typename T> struct V4;
template <> struct V4<float> {
  static DEVICE_INLINE void load(const float* p, float* o) {
    const f32x4 v = *reinterpret_cast<const f32x4*>(p);
    o[0] = v[0]; o[1] = v[1]; o[2] = v[2]; o[3] = v[3];
  }
  static DEVICE_INLINE void store(float* p, const float* o) {
    *reinterpret_cast<f32x4*>(p) = f32x4{o[0], o[1], o[2], o[3]};
  }
};
template <> struct V4<unsigned short> {
  static DEVICE_INLINE void load(const unsigned short* p, float* o) {
    const u16x4 v = *reinterpret_cast<const u16x4*>(p);
    o[0] = bf2f(v[0]); o[1] = bf2f(v[1]); o[2] = bf2f(v[2]); o[3] = bf2f(v[3]);
  }
  static DEVICE_INLINE void store(unsigned short* p, const float* o) {
    *reinterpret_cast<u16x4*>(p) = u16x4{f2bf(o[0]), f2bf(o[1]), f2bf(o[2]), f2bf(o[3])};
  }
};

template <typename TS, int NV>
__global__ __launch_bounds__(ROW_THREADS) void dual_rms_mix_vec_kernel(
    TS* __restrict__ out, const TS* __restrict__ a, const float* __restrict__ wa,
    const TS* __restrict__ b, const float* __restrict__ wb, int W, float eps) {
  __shared__ float red[4];
  const long t = blockIdx.x;
  float ka[NV][4], kb[NV][4];
  float sa = 0.f, sb = 0.f;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int i = (threadIdx.x + j * ROW_THREADS) * 4;
    if (i < W) {
      V4<TS>::load(a + t * W + i, ka[j]);
      V4<TS>::load(b + t * W + i, kb[j]);
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        sa += ka[j][k] * ka[j][k];
        sb += kb[j][k] * kb[j][k];
      }
    }
  }
  sa = block_sum(sa, red);
  sb = block_sum(sb, red);
  const float ia = 0.5f / sqrtf(sa / (float)W + eps);
  const float ib = 0.5f / sqrtf(sb / (float)W + eps);
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int i = (threadIdx.x + j * ROW_THREADS) * 4;
    if (i < W) {
      float x[4], yv[4], o[4];
      V4<float>::load(wa + i, x);
      V4<float>::load(wb + i, yv);
#pragma unroll
      for (int k = 0; k < 4; ++k)
        o[k] = ka[j][k] * ia * x[k] + kb[j][k] * ib * yv[k];
      V4<TS>::store(out + t * W + i, o);
    }
  }
}

// bf16, VD % 8 == 0: 16 bytes per lane.
__global__ __launch_bounds__(256) void head_gate_vec_kernel(
    unsigned short* __restrict__ out, const unsigned short* __restrict__ o_hts,
    const unsigned short* __restrict__ gate_src, long ld_gate, int col, int H,
    int T, int VD8) {
  const long n = (long)T * H * VD8;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (long)gridDim.x * blockDim.x) {
    const int c = (int)(i % VD8);
    const long th = i / VD8;
    const int h = (int)(th % H);
    const long t = th / H;
    const float g = bf2f(gate_src[t * ld_gate + col + h]);
    const float sg = 1.0f / (1.0f + __expf(-g));
    const u16x8 v = reinterpret_cast<const u16x8*>(o_hts)[((long)h * T + t) * VD8 + c];
    u16x8 o;
#pragma unroll
    for (int k = 0; k < 8; ++k) o[k] = f2bf(bf2f(v[k]) * sg);
    reinterpret_cast<u16x8*>(out)[i] = o;
  }
}

template <typename TS>
__global__ __launch_bounds__(256) void head_gate_kernel(
    TS* __restrict__ out, const TS* __restrict__ o_hts,
    const TS* __restrict__ gate_src, long ld_gate, int col, int H, int T,
    int VD) {
  const long n = (long)T * H * VD;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (long)gridDim.x * blockDim.x) {
    const int c = (int)(i % VD);
    const long th = i / VD;
    const int h = (int)(th % H);
    const long t = th / H;
    const float g = ld(gate_src + t * ld_gate + col + h);
    const float v = ld(o_hts + ((long)h * T + t) * VD + c);
    st(out + i, v / (1.0f + expf(-g)));
  }
}

}  // namespace

void head_rope_store_launch(void* q_out, const void* src, long ld_src,
                            int col_q, int q_heads, int q_dim,
                            const float* q_w, int q_nd, int q_rot0, int col_k,
                            int k_heads, int k_dim, const float* k_w, int k_nd,
                            int k_rot0, int col_v, const float* inv_freq,
                            int half, int half_layout, float amp,
                            const int* pos32, void* k_cache, void* v_cache,
                            const long* slots, long nslots, int BS, int VW,
                            float eps, int skip_v, int T, int bf,
                            hipStream_t s) {
  if (T <= 0 || q_heads + k_heads <= 0) return;
  RopeArgs p;
  p.ld_src = ld_src; p.col_q = col_q; p.q_heads = q_heads; p.q_dim = q_dim;
  p.q_nd = q_nd; p.q_rot0 = q_rot0; p.col_k = col_k; p.k_heads = k_heads;
  p.k_dim = k_dim; p.k_nd = k_nd; p.k_rot0 = k_rot0; p.col_v = col_v;
  p.q_w = q_w; p.k_w = k_w; p.inv_freq = inv_freq; p.half = half;
  p.half_layout = half_layout; p.amp = amp; p.eps = eps; p.pos32 = pos32;
  p.slots = slots; p.nslots = nslots; p.BS = BS; p.VW = VW; p.skip_v = skip_v;
  p.T = T;
  const dim3 grid(T, (q_heads + k_heads + 3) / 4);
  const size_t tab = (size_t)2 * half * sizeof(float);
  auto m8 = [](long v) { return v % 8 == 0; };
  const bool q_ok = q_heads == 0 ||
      (m8(col_q) && m8(q_dim) && (q_w == nullptr || m8(q_nd)) &&
       (q_rot0 < 0 || m8(q_rot0)) && (uintptr_t)q_out % 16 == 0);
  const bool k_ok = k_heads == 0 ||
      (m8(col_k) && m8(k_dim) && (k_w == nullptr || m8(k_nd)) &&
       (k_rot0 < 0 || m8(k_rot0)) && m8(VW) && (col_v < 0 || m8(col_v)) &&
       (uintptr_t)k_cache % 16 == 0);
  if (bf && q_ok && k_ok && m8(ld_src) && (uintptr_t)src % 16 == 0 &&
      (half == 0 || (half_layout ? m8(half) : m8(2 * half)))) {
    const int widest = max(q_heads ? q_dim : 0, k_heads ? max(k_dim, VW) : 0);
    int lph = 1;
    while (lph < 64 && lph * 8 < widest) lph *= 2;
    const int hpw = 64 / lph;
    const dim3 vgrid(T, (q_heads + k_heads + 4 * hpw - 1) / (4 * hpw));
#define HRS(L)                                                              \
  head_rope_store_vec_kernel<L><<<vgrid, ROW_THREADS, tab, s>>>(            \
      (unsigned short*)q_out, (const unsigned short*)src,                   \
      (unsigned short*)k_cache, (unsigned short*)v_cache, p)
    switch (lph) {
      case 1: HRS(1); break;
      case 2: HRS(2); break;
      case 4: HRS(4); break;
      case 8: HRS(8); break;
      case 16: HRS(16); break;
      case 32: HRS(32); break;
      default: HRS(64); break;
    }
#undef HRS
    return;
  }
  if (bf)
    head_rope_store_kernel<unsigned short><<<grid, ROW_THREADS, tab, s>>>(
        (unsigned short*)q_out, (const unsigned short*)src,
        (unsigned short*)k_cache, (unsigned short*)v_cache, p);
  else
    head_rope_store_kernel<float><<<grid, ROW_THREADS, tab, s>>>(
        (float*)q_out, (const float*)src, (float*)k_cache, (float*)v_cache, p);
}

void dual_rms_mix_launch(void* out, const void* a, const float* wa,
                         const void* b, const float* wb, int T, int W,
                         float eps, int bf, hipStream_t s) {
  if (T <= 0) return;
  if (W % 4 == 0 && W <= 8 * 1024) {
#define DRV(TS, NV)                                                         \
  dual_rms_mix_vec_kernel<TS, NV><<<T, ROW_THREADS, 0, s>>>(                \
      (TS*)out, (const TS*)a, wa, (const TS*)b, wb, W, eps)
    if (bf) {
      if (W <= 1024) DRV(unsigned short, 1);
      else if (W <= 2048) DRV(unsigned short, 2);
      else if (W <= 4096) DRV(unsigned short, 4);
      else DRV(unsigned short, 8);
    } else {
      if (W <= 1024) DRV(float, 1);
      else if (W <= 2048) DRV(float, 2);
      else if (W <= 4096) DRV(float, 4);
      else DRV(float, 8);
    }
#undef DRV
    return;
  }
#define DRM(TS, NV)                                                         \
  dual_rms_mix_kernel<TS, NV><<<T, ROW_THREADS, 0, s>>>(                    \
      (TS*)out, (const TS*)a, wa, (const TS*)b, wb, W, eps)
  if (bf) {
    if (W <= 4 * ROW_THREADS) DRM(unsigned short, 4);
    else DRM(unsigned short, 16);
  } else {
    if (W <= 4 * ROW_THREADS) DRM(float, 4);
    else DRM(float, 16);
  }
#undef DRM
}

void head_gate_launch(void* out, const void* o_hts, const void* gate_src,
                      long ld_gate, int col, int H, int T, int VD, int bf,
                      hipStream_t s) {
  const long n = (long)T * H * VD;
  if (n <= 0) return;
  const int grid = (int)min((n + 255) / 256, (long)(256 * 32));
  if (bf && VD % 8 == 0) {
    const int g8 = (int)min((n / 8 + 255) / 256, (long)(256 * 32));
    head_gate_vec_kernel<<<g8, 256, 0, s>>>(
        (unsigned short*)out, (const unsigned short*)o_hts,
        (const unsigned short*)gate_src, ld_gate, col, H, T, VD / 8);
    return;
  }
  if (bf)
    head_gate_kernel<unsigned short><<<grid, 256, 0, s>>>(
        (unsigned short*)out, (const unsigned short*)o_hts,
        (const unsigned short*)gate_src, ld_gate, col, H, T, VD);
  else
    head_gate_kernel<float><<<grid, 256, 0, s>>>(
        (float*)out, (const float*)o_hts, (const float*)gate_src, ld_gate, col,
        H, T, VD);
}
