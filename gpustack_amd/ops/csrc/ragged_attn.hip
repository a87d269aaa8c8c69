// Paged rotary attention over a ragged batch (gfx950).
//
//   out[t, a, :] = sum_j softmax_j(scale * q[t, a, :] . k_j) * v_j
//
// over the visible keys j of row t's sequence, read through its block
// table: j <= pos(t), and with a window also (pos(t) - j < window or
// j < keep_first). a runs over heads * maps SCORE MAPS (a = head * maps +
// map): map m of a head reads channels [m*D, (m+1)*D) of its kv head's key
// row, and all maps of a head weight the same value rows — two maps per
// head are the two halves of differential attention, combined afterwards.
// A per-head sink logit may join the denominator (no key, no value), and a
// per-head slope times the distance pos(t) - j may be taken off the scaled
// score (positions without rotation); a tanh cap may bound the scaled
// score. q and out are [T, A, *] views with a contiguous last axis.
//
// Pools: keys [nblocks, G, BS, KW] with KW = maps * D (rotated at write
// time), values with every page transposed, [nblocks, G, VW, BS], so both
// matrix products find their reduction axis contiguous: scores reduce over
// channels, the weighted sum over keys.
//
// A workgroup takes a tile of up to 16 (row, map) pairs that share one key
// stream — same sequence, same kv head, same map (host-built list: 16 rows
// x 1 map inside prompts, rows x the query heads of a kv group for decode
// rows) — and walks that stream once for all of them. Key tiles that lie
// wholly outside every pair's window (and past the kept first keys) are
// skipped, so a windowed layer costs its window, not its context.
//
// Two paths. The MFMA path (bf16 q and pools, BS = 16, D % 32 == 0, VW %
// 16 == 0) runs both products on v_mfma_f32_16x16x32_bf16 with fp32
// accumulation; scores are scaled, masked and soft-maxed in fp32 and only
// the weights are rounded to bf16 for the second product. Per 64-key tile:
// wave w multiplies the 16 pairs with keys 16w..16w+15 (B operand straight
// from the key pool, 16 B per lane), scores meet in LDS for the online
// softmax, then wave w owns the output channels of n-tiles w, w+4, ... and
// multiplies P (A operand, LDS) with the transposed value pages. With few
// tiles over long contexts (decode) gridDim.y workgroups split a tile's
// keys and a merge kernel joins the partial (acc, m, l) triples. The exact
// path keeps everything fp32 on the vector ALUs, for pools of bf16 or fp32
// and any sizes; it is the path of fp32 engines and the reference the MFMA
// kernel is tested against.
#include "common.h"

namespace {

constexpr int G16 = 16;       // (row, map) pairs per workgroup
constexpr int THREADS = 256;

template <typename T> DEVICE_INLINE float ldf(const T* p);
template <> DEVICE_INLINE float ldf<float>(const float* p) { return *p; }
template <> DEVICE_INLINE float ldf<unsigned short>(const unsigned short* p) {
  return bf2f(*p);
}
template <typename T> DEVICE_INLINE void stf(T* p, float v);
template <> DEVICE_INLINE void stf<float>(float* p, float v) { *p = v; }
template <> DEVICE_INLINE void stf<unsigned short>(unsigned short* p, float v) {
  *p = f2bf(v);
}

struct AttnArgs {
  const int* block_tables;   // [nseq, maxb]
  const int* tiles;          // [ntiles, 6] row0, nrows, a0, n_a, seq, a_step
  const int* pos32;          // [T]
  const float* sinks;        // [A / maps] or null
  const float* slopes;       // [A / maps] or null
  float scale;
  float softcap;             // > 0: scaled scores pass cap * tanh(s / cap)
  long q_st, q_sa;           // element strides of q [T, A, D]: row, score map
  long o_st, o_sa;           // and of out [T, A, VW]
  int T, A, D, VW, KW, G, BS, maps, rep;   // rep = heads / kv heads
  int nseq, maxb, nblocks, window, keep_first;
};

// Decodes and validates a tile; false = skip the tile untouched.
DEVICE_INLINE bool tile_setup(const AttnArgs& p, int tile, int* e_pos,
                              int* e_row, int* e_a, int& n_ent, int& seq,
                              int& g, int& koff) {
  const int* tl = p.tiles + (long)tile * 6;
  const int row0 = tl[0], nrows = tl[1], a0 = tl[2], n_a = tl[3];
  const int a_step = tl[5];
  seq = tl[4];
  if (row0 < 0 || nrows < 1 || row0 + nrows > p.T || a0 < 0 || n_a < 1 ||
      a_step < 1 || a0 + (long)(n_a - 1) * a_step >= p.A ||
      (long)nrows * n_a > G16 || seq < 0 || seq >= p.nseq)
    return false;
  n_ent = nrows * n_a;
  g = (a0 / p.maps) / p.rep;
  koff = (a0 % p.maps) * p.D;
  if (g >= p.G) return false;
  if (threadIdx.x < G16) {
    int ps = -1, row = 0, a = 0;
    if ((int)threadIdx.x < n_ent) {
      row = row0 + threadIdx.x / n_a;
      a = a0 + (threadIdx.x % n_a) * a_step;
      ps = min(max(p.pos32[row], 0), p.maxb * p.BS - 1);
    }
    e_pos[threadIdx.x] = ps;
    e_row[threadIdx.x] = row;
    e_a[threadIdx.x] = a;
  }
  return true;
}

DEVICE_INLINE bool key_visible(int j, int pos, int window, int keep_first) {
  return j <= pos && (window <= 0 || pos - j < window || j < keep_first);
}

DEVICE_INLINE float scaled_score(float dot, const AttnArgs& p) {
  const float s = dot * p.scale;
  return p.softcap > 0.f ? p.softcap * tanhf(s / p.softcap) : s;
}

// ---- exact path ----------------------------------------------------------

template <typename TQ, typename TC, typename TO, int NJ, int KT>
__global__ __launch_bounds__(THREADS) void paged_attn_exact_kernel(
    TO* __restrict__ out, const TQ* __restrict__ q,
    const TC* __restrict__ k_cache, const TC* __restrict__ v_cache,
    AttnArgs p) {
  extern __shared__ float sm[];
  const int D = p.D, VW = p.VW, KS = p.D + 1, VS = p.VW + 1;
  float* qs = sm;                     // [16][D]
  float* ks = qs + G16 * D;           // [KT][KS]
  float* vs = ks + KT * KS;           // [KT][VS]
  float* ps = vs + KT * VS;           // [16][KT]
  float* als = ps + G16 * KT;         // [16]
  float* lsum = als + G16;            // [16]
  __shared__ int e_pos[G16], e_row[G16], e_a[G16];

  int n_ent, seq, g, koff;
  if (!tile_setup(p, blockIdx.x, e_pos, e_row, e_a, n_ent, seq, g, koff))
    return;
  __syncthreads();
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int jmax = -1, jmin = 1 << 30;
#pragma unroll
  for (int e = 0; e < G16; ++e) {
    jmax = max(jmax, e_pos[e]);
    if (e_pos[e] >= 0) jmin = min(jmin, e_pos[e]);
  }
  const int lo = p.window > 0 ? max(0, jmin - p.window + 1) : 0;
  for (int e = wave; e < G16; e += 4) {
    const bool ok = e < n_ent;
    const TQ* qp = q + (long)e_row[e] * p.q_st + (long)e_a[e] * p.q_sa;
    for (int r = lane; r < D; r += 64) qs[e * D + r] = ok ? ldf(qp + r) : 0.f;
  }
  const int e_s = tid >> 4, kk = tid & 15;
  const int my_pos = e_pos[e_s];
  float m_run = -INFINITY, l_run = 0.f;
  if (p.sinks != nullptr && my_pos >= 0) {
    m_run = p.sinks[e_a[e_s] / p.maps];
    l_run = 1.f;
  }
  const float slope = p.slopes != nullptr ? p.slopes[e_a[e_s] / p.maps] : 0.f;
  float acc[4][NJ];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j) acc[i][j] = 0.f;

  const int* bt = p.block_tables + (long)seq * p.maxb;
  const int BS = p.BS;
  for (int k0 = 0; k0 <= jmax; k0 += KT) {
    if (p.window > 0 && k0 >= p.keep_first && k0 + KT - 1 < lo) continue;
    __syncthreads();   // previous tile fully consumed (and qs written)
    for (int k = wave; k < KT; k += 4) {
      const int j = k0 + k;
      float* dst = ks + k * KS;
      if (j <= jmax) {
        const long blk = min(max(bt[j / BS], 0), p.nblocks - 1);
        const TC* src =
            k_cache + ((blk * p.G + g) * BS + j % BS) * (long)p.KW + koff;
        for (int r = lane; r < D; r += 64) dst[r] = ldf(src + r);
      } else {
        for (int r = lane; r < D; r += 64) dst[r] = 0.f;
      }
    }
    for (int i = tid; i < KT * VW; i += THREADS) {
      const int k = i % KT, c = i / KT;
      const int j = k0 + k;
      float v = 0.f;
      if (j <= jmax) {
        const long blk = min(max(bt[j / BS], 0), p.nblocks - 1);
        v = ldf(v_cache + ((blk * p.G + g) * (long)VW + c) * BS + j % BS);
      }
      vs[k * VS + c] = v;
    }
    __syncthreads();
    float s[KT / 16];
#pragma unroll
    for (int u = 0; u < KT / 16; ++u) s[u] = 0.f;
    {
      const float* qp = qs + e_s * D;
      for (int r = 0; r < D; ++r) {
        const float qv = qp[r];
#pragma unroll
        for (int u = 0; u < KT / 16; ++u) s[u] += qv * ks[(kk + 16 * u) * KS + r];
      }
    }
    float mx = -INFINITY;
#pragma unroll
    for (int u = 0; u < KT / 16; ++u) {
      const int j = k0 + kk + 16 * u;
      s[u] = key_visible(j, my_pos, p.window, p.keep_first)
                 ? scaled_score(s[u], p) - slope * (float)(my_pos - j)
                 : -INFINITY;
      mx = fmaxf(mx, s[u]);
    }
#pragma unroll
    for (int m = 8; m >= 1; m >>= 1) mx = fmaxf(mx, __shfl_xor(mx, m, WAVE_SIZE));
    const float m_new = fmaxf(m_run, mx);
    float alpha = 1.f, psum = 0.f;
    if (m_new == -INFINITY) {
#pragma unroll
      for (int u = 0; u < KT / 16; ++u) ps[e_s * KT + kk + 16 * u] = 0.f;
    } else {
      alpha = expf(m_run - m_new);
#pragma unroll
      for (int u = 0; u < KT / 16; ++u) {
        const float pv = expf(s[u] - m_new);
        ps[e_s * KT + kk + 16 * u] = pv;
        psum += pv;
      }
    }
    psum = group16_reduce_sum(psum);
    l_run = l_run * alpha + psum;
    m_run = m_new;
    if (kk == 0) als[e_s] = alpha;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float al = als[wave + 4 * i];
#pragma unroll
      for (int j = 0; j < NJ; ++j) acc[i][j] *= al;
    }
    for (int k = 0; k < KT; ++k) {
      float vv[NJ];
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int c = lane + 64 * j;
        vv[j] = c < VW ? vs[k * VS + c] : 0.f;
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float pv = ps[(wave + 4 * i) * KT + k];
#pragma unroll
        for (int j = 0; j < NJ; ++j) acc[i][j] += pv * vv[j];
      }
    }
  }
  if (kk == 0) lsum[e_s] = l_run;
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int e = wave + 4 * i;
    if (e >= n_ent) continue;
    const float l = lsum[e];
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    TO* op = out + (long)e_row[e] * p.o_st + (long)e_a[e] * p.o_sa;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int c = lane + 64 * j;
      if (c < VW) stf(op + c, acc[i][j] * inv);
    }
  }
}

// ---- MFMA path -------------------------------------------------------------

typedef __attribute__((ext_vector_type(8))) short ra_s16x8;

DEVICE_INLINE f32x4 ra_mfma(u16x8 a, u16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(
      __builtin_bit_cast(ra_s16x8, a), __builtin_bit_cast(ra_s16x8, b), c, 0, 0, 0);
}

constexpr int MKT = 64;            // keys per tile (16 per wave)
constexpr int MSS = MKT + 4;       // fp32 score row stride
constexpr int MPS = MKT + 8;       // bf16 weight row stride (16 B aligned)

// NT: 16-channel n-tiles per wave (wave w owns n-tiles w, w+4, ...).
template <int NT, typename TO>
__global__ __launch_bounds__(THREADS) void paged_attn_mfma_kernel(
    TO* __restrict__ out, const unsigned short* __restrict__ q,
    const unsigned short* __restrict__ k_cache,
    const unsigned short* __restrict__ v_cache, AttnArgs p,
    float* __restrict__ ws_acc, float* __restrict__ ws_ml) {
  constexpr int BS = 16;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  const int D = p.D, VW = p.VW;
  const int QS = D + 8;                               // bf16 row stride
  unsigned short* Ql = reinterpret_cast<unsigned short*>(smem_raw);  // [16][QS]
  unsigned short* Pl = Ql + G16 * QS;                 // [16][MPS]
  float* Ss = reinterpret_cast<float*>(Pl + G16 * MPS);  // [16][MSS]
  float* als = Ss + G16 * MSS;                        // [16]
  float* lsum = als + G16;                            // [16]
  __shared__ int e_pos[G16], e_row[G16], e_a[G16];

  int n_ent, seq, g, koff;
  if (!tile_setup(p, blockIdx.x, e_pos, e_row, e_a, n_ent, seq, g, koff))
    return;
  __syncthreads();
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lc = lane & 15, lg = lane >> 4;
  int jmax = -1, jmin = 1 << 30;
#pragma unroll
  for (int e = 0; e < G16; ++e) {
    jmax = max(jmax, e_pos[e]);
    if (e_pos[e] >= 0) jmin = min(jmin, e_pos[e]);
  }
  const int lo = p.window > 0 ? max(0, jmin - p.window + 1) : 0;
  for (int e = wave; e < G16; e += 4) {
    const bool ok = e < n_ent;
    const unsigned short* qp =
        q + (long)e_row[e] * p.q_st + (long)e_a[e] * p.q_sa;
    for (int r = lane; r < D; r += 64)
      Ql[e * QS + r] = ok ? qp[r] : (unsigned short)0;
  }

  const int e_s = tid >> 4, kk = tid & 15;    // softmax role
  const int my_pos = e_pos[e_s];
  const int nsplit = gridDim.y, split = blockIdx.y;
  float m_run = -INFINITY, l_run = 0.f;
  if (p.sinks != nullptr && my_pos >= 0 && split == 0) {
    m_run = p.sinks[e_a[e_s] / p.maps];
    l_run = 1.f;
  }
  const float slope = p.slopes != nullptr ? p.slopes[e_a[e_s] / p.maps] : 0.f;
  f32x4 acc[NT];
#pragma unroll
  for (int i = 0; i < NT; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int* bt = p.block_tables + (long)seq * p.maxb;
  const int last_page = jmax >> 4;
  const int ntk = jmax / MKT + 1;                       // key tiles
  const int per = (ntk + nsplit - 1) / nsplit;
  const int t_end = min(ntk, (split + 1) * per);
  for (int kt = split * per; kt < t_end; ++kt) {
    const int k0 = kt * MKT;
    if (p.window > 0 && k0 >= p.keep_first && k0 + MKT - 1 < lo) continue;
    __syncthreads();   // Ql staged / previous tile's Pl and als consumed
    {
      // scores: this wave's 16 keys; keys past jmax re-read key jmax (their
      // weights are masked to zero below)
      const int key = min(k0 + wave * 16 + lc, jmax);
      const long blk = min(max(bt[key >> 4], 0), p.nblocks - 1);
      const unsigned short* rowp =
          k_cache + ((blk * p.G + g) * BS + (key & 15)) * (long)p.KW + koff;
      const unsigned short* qrow = Ql + lc * QS;
      f32x4 sacc{0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
      for (int r = 0; r < D; r += 32) {
        const u16x8 a = *reinterpret_cast<const u16x8*>(qrow + r + lg * 8);
        const u16x8 b = *reinterpret_cast<const u16x8*>(rowp + r + lg * 8);
        sacc = ra_mfma(a, b, sacc);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r)
        Ss[(lg * 4 + r) * MSS + wave * 16 + lc] = sacc[r];
    }
    __syncthreads();
    {
      float sv[4];
      float mx = -INFINITY;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int j = k0 + kk + 16 * u;
        sv[u] = key_visible(j, my_pos, p.window, p.keep_first)
                    ? scaled_score(Ss[e_s * MSS + kk + 16 * u], p) -
                          slope * (float)(my_pos - j)
                    : -INFINITY;
        mx = fmaxf(mx, sv[u]);
      }
#pragma unroll
      for (int m = 8; m >= 1; m >>= 1) mx = fmaxf(mx, __shfl_xor(mx, m, WAVE_SIZE));
      const float m_new = fmaxf(m_run, mx);
      float alpha = 1.f, psum = 0.f;
      if (m_new == -INFINITY) {
#pragma unroll
        for (int u = 0; u < 4; ++u) Pl[e_s * MPS + kk + 16 * u] = 0;
      } else {
        alpha = __expf(m_run - m_new);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const float pv = __expf(sv[u] - m_new);
          Pl[e_s * MPS + kk + 16 * u] = f2bf(pv);
          psum += pv;
        }
      }
      psum = group16_reduce_sum(psum);
      l_run = l_run * alpha + psum;
      m_run = m_new;
      if (kk == 0) als[e_s] = alpha;
    }
    __syncthreads();
    {
      float ar[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) ar[r] = als[lg * 4 + r];
#pragma unroll
      for (int i = 0; i < NT; ++i)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[i][r] *= ar[r];
#pragma unroll
      for (int ks = 0; ks < MKT; ks += 32) {
        const u16x8 a =
            *reinterpret_cast<const u16x8*>(Pl + lc * MPS + ks + lg * 8);
        // 8 consecutive keys of one page; groups wholly past jmax read the
        // last valid page (weights there are zero)
        const int keyb = k0 + ks + lg * 8;
        const int pg = min(keyb >> 4, last_page);
        const long blk = min(max(bt[pg], 0), p.nblocks - 1);
        const unsigned short* pt =
            v_cache + (blk * p.G + g) * (long)VW * BS + (keyb & 15);
#pragma unroll
        for (int i = 0; i < NT; ++i) {
          const int ch = (wave + 4 * i) * 16 + lc;
          if ((wave + 4 * i) * 16 < VW) {       // uniform over the wave
            const u16x8 b = *reinterpret_cast<const u16x8*>(pt + (long)ch * BS);
            acc[i] = ra_mfma(a, b, acc[i]);
          }
        }
      }
    }
  }
  if (nsplit > 1) {
    const long slot = (long)blockIdx.x * nsplit + split;
    if (kk == 0) {
      ws_ml[(slot * G16 + e_s) * 2] = m_run;
      ws_ml[(slot * G16 + e_s) * 2 + 1] = l_run;
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int e = lg * 4 + r;
      float* wp = ws_acc + (slot * G16 + e) * VW;
#pragma unroll
      for (int i = 0; i < NT; ++i) {
        const int ch = (wave + 4 * i) * 16 + lc;
        if (ch < VW) wp[ch] = acc[i][r];
      }
    }
    return;
  }
  if (kk == 0) lsum[e_s] = l_run;
  __syncthreads();
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int e = lg * 4 + r;
    if (e >= n_ent) continue;
    const float l = lsum[e];
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    TO* op = out + (long)e_row[e] * p.o_st + (long)e_a[e] * p.o_sa;
#pragma unroll
    for (int i = 0; i < NT; ++i) {
      const int ch = (wave + 4 * i) * 16 + lc;
      if (ch < VW) stf(op + ch, acc[i][r] * inv);
    }
  }
}

// out = sum_s acc_s exp(m_s - M) / sum_s l_s exp(m_s - M) over a tile's
// splits; one workgroup of 128 lanes per (tile, pair)
constexpr int MERGE_THREADS = 128;

template <typename TO>
__global__ __launch_bounds__(MERGE_THREADS) void paged_attn_merge_kernel(
    TO* __restrict__ out, AttnArgs p, const float* __restrict__ ws_acc,
    const float* __restrict__ ws_ml, int nsplit) {
  const int* tl = p.tiles + (long)blockIdx.x * 6;
  const int row0 = tl[0], nrows = tl[1], a0 = tl[2], n_a = tl[3];
  const int seq = tl[4], a_step = tl[5];
  const int e = blockIdx.y;
  // the same test the attention kernel applies: skipped tiles left nothing
  if (row0 < 0 || nrows < 1 || row0 + nrows > p.T || a0 < 0 || n_a < 1 ||
      a_step < 1 || a0 + (long)(n_a - 1) * a_step >= p.A ||
      (long)nrows * n_a > G16 || seq < 0 || seq >= p.nseq ||
      (a0 / p.maps) / p.rep >= p.G || e >= nrows * n_a)
    return;
  const int VW = p.VW;
  const long base = (long)blockIdx.x * nsplit;
  float M = -INFINITY;
  for (int s = 0; s < nsplit; ++s)
    M = fmaxf(M, ws_ml[((base + s) * G16 + e) * 2]);
  float L = 0.f;
  for (int s = 0; s < nsplit; ++s) {
    const float* ml = ws_ml + ((base + s) * G16 + e) * 2;
    if (ml[0] != -INFINITY) L += ml[1] * __expf(ml[0] - M);
  }
  const float inv = L > 0.f ? 1.0f / L : 0.f;
  const int row = row0 + e / n_a, a = a0 + (e % n_a) * a_step;
  TO* op = out + (long)row * p.o_st + (long)a * p.o_sa;
  for (int ch = threadIdx.x; ch < VW; ch += MERGE_THREADS) {
    float v = 0.f;
    for (int s = 0; s < nsplit; ++s) {
      const float m = ws_ml[((base + s) * G16 + e) * 2];
      if (m != -INFINITY)
        v += ws_acc[((base + s) * G16 + e) * VW + ch] * __expf(m - M);
    }
    stf(op + ch, v * inv);
  }
}

template <int NT, typename TO>
void launch_mfma(void* out, const void* q, const void* kc, const void* vc,
                 const AttnArgs& p, int ntiles, int nsplit, float* ws_acc,
                 float* ws_ml, hipStream_t s) {
  const size_t smem = (size_t)G16 * (p.D + 8) * 2 + (size_t)G16 * MPS * 2 +
                      (size_t)(G16 * MSS + 2 * G16) * sizeof(float);
  paged_attn_mfma_kernel<NT, TO><<<dim3(ntiles, nsplit), THREADS, smem, s>>>(
      (TO*)out, (const unsigned short*)q, (const unsigned short*)kc,
      (const unsigned short*)vc, p, ws_acc, ws_ml);
  if (nsplit > 1)
    paged_attn_merge_kernel<TO><<<dim3(ntiles, G16), MERGE_THREADS, 0, s>>>(
        (TO*)out, p, ws_acc, ws_ml, nsplit);
}

template <typename TO>
void dispatch_mfma(void* out, const void* q, const void* kc, const void* vc,
                   const AttnArgs& p, int ntiles, int nsplit, float* ws_acc,
                   float* ws_ml, hipStream_t s) {
  const int nt = (p.VW / 16 + 3) / 4;
  if (nt <= 1) launch_mfma<1, TO>(out, q, kc, vc, p, ntiles, nsplit, ws_acc, ws_ml, s);
  else if (nt <= 2) launch_mfma<2, TO>(out, q, kc, vc, p, ntiles, nsplit, ws_acc, ws_ml, s);
  else if (nt <= 4) launch_mfma<4, TO>(out, q, kc, vc, p, ntiles, nsplit, ws_acc, ws_ml, s);
  else launch_mfma<8, TO>(out, q, kc, vc, p, ntiles, nsplit, ws_acc, ws_ml, s);
}

template <typename TQ, typename TC, typename TO, int NJ, int KT>
void launch_exact(void* out, const void* q, const void* kc, const void* vc,
                  const AttnArgs& p, int ntiles, hipStream_t s) {
  const size_t smem = (size_t)(G16 * p.D + KT * (p.D + 1) + KT * (p.VW + 1) +
                               G16 * KT + 2 * G16) * sizeof(float);
  auto kern = paged_attn_exact_kernel<TQ, TC, TO, NJ, KT>;
  if (smem > 48 * 1024)
    (void)hipFuncSetAttribute((const void*)kern,
                              hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)smem);
  kern<<<ntiles, THREADS, smem, s>>>((TO*)out, (const TQ*)q, (const TC*)kc,
                                     (const TC*)vc, p);
}

template <typename TQ, typename TC, typename TO>
void dispatch_exact(void* out, const void* q, const void* kc, const void* vc,
                    const AttnArgs& p, int ntiles, hipStream_t s) {
  // wide heads take shorter key tiles so the staging fits the LDS
  const bool small = p.D + p.VW <= 320;   // KT = 32 within 64 KB
  if (p.VW <= 64) {
    if (small) launch_exact<TQ, TC, TO, 1, 32>(out, q, kc, vc, p, ntiles, s);
    else launch_exact<TQ, TC, TO, 1, 16>(out, q, kc, vc, p, ntiles, s);
  } else if (p.VW <= 128) {
    if (small) launch_exact<TQ, TC, TO, 2, 32>(out, q, kc, vc, p, ntiles, s);
    else launch_exact<TQ, TC, TO, 2, 16>(out, q, kc, vc, p, ntiles, s);
  } else if (p.VW <= 256) {
    if (small) launch_exact<TQ, TC, TO, 4, 32>(out, q, kc, vc, p, ntiles, s);
    else launch_exact<TQ, TC, TO, 4, 16>(out, q, kc, vc, p, ntiles, s);
  } else {
    launch_exact<TQ, TC, TO, 8, 16>(out, q, kc, vc, p, ntiles, s);
  }
}

}  // namespace

// largest head sizes the exact path's LDS tiling covers (the MFMA path
// takes score sizes up to 1024 and value sizes up to 512)
int paged_attn_max_dim() { return 512; }

// 1 when (q / pool dtype, page size, head sizes) take the MFMA path
int paged_attn_uses_mfma(int io_bf, int BS, int D, int VW) {
  return io_bf && BS == 16 && D % 32 == 0 && D <= 1024 && VW % 16 == 0 &&
         VW <= 512;
}

// q_bf: q and the pools are bf16, else fp32. out_bf: out is bf16, else fp32.
// nsplit > 1 (MFMA path only) needs ws_acc [ntiles*nsplit*16*VW] and ws_ml
// [ntiles*nsplit*16*2] fp32.
void paged_attention_launch(void* out, const void* q, const void* k_cache,
                            const void* v_cache, const int* block_tables,
                            const int* tiles, const int* pos32,
                            const float* sinks, const float* slopes,
                            float scale, float softcap, long q_st, long q_sa,
                            long o_st, long o_sa, int ntiles, int T,
                            int A, int D, int VW, int KW, int G, int BS,
                            int maps, int rep, int nseq, int maxb, int nblocks,
                            int window, int keep_first, int q_bf, int out_bf,
                            int force_exact, int nsplit, float* ws_acc,
                            float* ws_ml, hipStream_t s) {
  if (ntiles == 0) return;
  AttnArgs p;
  p.block_tables = block_tables; p.tiles = tiles; p.pos32 = pos32;
  p.softcap = softcap; p.q_st = q_st; p.q_sa = q_sa; p.o_st = o_st;
  p.o_sa = o_sa;
  p.sinks = sinks; p.slopes = slopes; p.scale = scale; p.T = T; p.A = A; p.D = D; p.VW = VW;
  p.KW = KW; p.G = G; p.BS = BS; p.maps = maps; p.rep = rep; p.nseq = nseq;
  p.maxb = maxb; p.nblocks = nblocks; p.window = window;
  p.keep_first = keep_first;
  if (!force_exact && paged_attn_uses_mfma(q_bf, BS, D, VW)) {
    if (out_bf)
      dispatch_mfma<unsigned short>(out, q, k_cache, v_cache, p, ntiles, nsplit, ws_acc, ws_ml, s);
    else
      dispatch_mfma<float>(out, q, k_cache, v_cache, p, ntiles, nsplit, ws_acc, ws_ml, s);
    return;
  }
  if (q_bf) {
    if (out_bf)
      dispatch_exact<unsigned short, unsigned short, unsigned short>(out, q, k_cache, v_cache, p, ntiles, s);
    else
      dispatch_exact<unsigned short, unsigned short, float>(out, q, k_cache, v_cache, p, ntiles, s);
  } else {
    dispatch_exact<float, float, float>(out, q, k_cache, v_cache, p, ntiles, s);
  }
}
