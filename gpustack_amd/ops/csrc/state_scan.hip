// Recurrent mixers with one matrix state per head and sequence (gfx950).
//
//   S_t = a_t S_(t-1) + b_t k_t v_t^T,    y_t = S_t^T q_t + skip * v_t
//
// S [N x P] is fp32 and lives in the sequence's slot of a state pool
// [slots, H, N, P]. A batch is ragged: sequence s brings rows seq_first[s]
// .. seq_first[s] + seq_rows[s] - 1 (a prompt portion, or one decoded
// token); its first row's position says whether the slot is read (> 0) or
// the state starts from zero (== 0). Every kernel here walks or indexes
// rows through that per-sequence view, so a prompt cut anywhere, a decode
// row and a mixed batch give the same states.
//
//   causal_conv_silu : short causal convolution per channel + SiLU; the
//                      inputs before this step's rows come from the slot's
//                      last taps - 1 inputs; a second launch moves the
//                      slot on (it must not race with the reads)
//   state_scan       : the recurrence. A wave owns PL value channels of one
//                      (sequence, head); the N state rows are split over
//                      TPP lanes per channel, NR rows each, in registers.
//                      Rows are staged CH at a time through LDS (k, q, v,
//                      decay, step), then walked in order. Step sizes and
//                      decays are computed here in fp32: a = exp(-exp(A_log)
//                      * dt), b = dt = softplus(raw + bias), or constants.
//   gated_group_norm : gate (SiLU or sigmoid) and RMS norm in equal parts of
//                      the row, in either order
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

DEVICE_INLINE float silu_f(float z) { return z / (1.0f + expf(-z)); }
DEVICE_INLINE float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }
// softplus without a switch-over: max(x, 0) + log1p(exp(-|x|))
DEVICE_INLINE float softplus_f(float x) {
  return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x)));
}

constexpr int MAX_TAPS = 16;

// grid (T, ceil(C / 256)): one lane per (row, channel).
template <typename TS>
__global__ __launch_bounds__(256) void causal_conv_silu_kernel(
    TS* __restrict__ out, const TS* __restrict__ src, long ld_src, int col0,
    int C, int taps, const float* __restrict__ w, const float* __restrict__ b,
    const TS* __restrict__ conv_state, const int* __restrict__ seq_first,
    const int* __restrict__ state_slots, const int* __restrict__ row_seq,
    const int* __restrict__ pos32, int nseq, int nslots, int T) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int s = min(max(row_seq[t], 0), nseq - 1);
  const int first = min(max(seq_first[s], 0), t);
  const int i = t - first;                   // row index inside the portion
  const int pos = max(pos32[t], 0);
  const int slot = min(max(state_slots[s], 0), nslots - 1);
  const int keep = taps - 1;
  const TS* stp = conv_state + (long)slot * keep * C;
  float acc = b[c];
  for (int k = 0; k < taps; ++k) {
    const int d = keep - k;                  // how far back this tap looks
    float v = 0.f;
    if (i - d >= 0)
      v = ld(src + (long)(t - d) * ld_src + col0 + c);
    else if (pos - d >= 0)
      v = ld(stp + (long)(keep + i - d) * C + c);
    acc += w[(long)c * taps + k] * v;
  }
  st(out + (long)t * C + c, silu_f(acc));
}

// The same for bf16 rows whose channel count, first column and row stride
// are multiples of 8: a lane takes 8 neighbouring channels of RB rows in a
// row with 16-byte loads, its TAPS x 8 weights in registers.
// grid (ceil(T / RB), ceil(C / 8 / 256)).
constexpr int RB = 8;

template <int TAPS>
__global__ __launch_bounds__(256) void causal_conv_silu_vec_kernel(
    unsigned short* __restrict__ out, const unsigned short* __restrict__ src,
    long ld_src, int col0, int C, const float* __restrict__ w,
    const float* __restrict__ b, const unsigned short* __restrict__ conv_state,
    const int* __restrict__ seq_first, const int* __restrict__ state_slots,
    const int* __restrict__ row_seq, const int* __restrict__ pos32, int nseq,
    int nslots, int T) {
  const int c = (blockIdx.y * 256 + threadIdx.x) * 8;
  if (c >= C) return;
  constexpr int keep = TAPS - 1;
  float wr[TAPS][8], br[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    br[e] = b[c + e];
#pragma unroll
    for (int k = 0; k < TAPS; ++k) wr[k][e] = w[(long)(c + e) * TAPS + k];
  }
  const int t_end = min(T, (int)(blockIdx.x + 1) * RB);
  for (int t = blockIdx.x * RB; t < t_end; ++t) {
    const int s = min(max(row_seq[t], 0), nseq - 1);
    const int first = min(max(seq_first[s], 0), t);
    const int i = t - first;
    const int pos = max(pos32[t], 0);
    const int slot = min(max(state_slots[s], 0), nslots - 1);
    const unsigned short* stp = conv_state + (long)slot * keep * C;
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = br[e];
#pragma unroll
    for (int k = 0; k < TAPS; ++k) {
      const int d = keep - k;
      u16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
      if (i - d >= 0)
        v = *reinterpret_cast<const u16x8*>(src + (long)(t - d) * ld_src + col0 + c);
      else if (pos - d >= 0)
        v = *reinterpret_cast<const u16x8*>(stp + (long)(keep + i - d) * C + c);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] += wr[k][e] * bf2f(v[e]);
    }
    u16x8 o;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = f2bf(silu_f(acc[e]));
    *reinterpret_cast<u16x8*>(out + (long)t * C + c) = o;
  }
}

// grid (nseq, ceil(C / 256)): the slot's new last inputs, after every read
// of the old ones (stream order).
template <typename TS>
__global__ __launch_bounds__(256) void conv_state_update_kernel(
    const TS* __restrict__ src, long ld_src, int col0, int C, int taps,
    TS* __restrict__ conv_state, const int* __restrict__ seq_first,
    const int* __restrict__ seq_rows, const int* __restrict__ state_slots,
    const int* __restrict__ pos32, int nslots, int T) {
  const int s = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int first = seq_first[s], n = seq_rows[s];
  if (first < 0 || n < 1 || first + n > T) return;
  const int hist = max(pos32[first], 0);
  const int slot = min(max(state_slots[s], 0), nslots - 1);
  const int keep = taps - 1;
  TS* stp = conv_state + (long)slot * keep * C;
  TS fresh[MAX_TAPS];
  for (int j = 0; j < keep; ++j) {
    const int i = n - (keep - j);            // local row of new entry j
    TS v = 0;
    if (i >= 0)
      v = src[(long)(first + i) * ld_src + col0 + c];
    else if (hist + i >= 0)
      v = stp[(long)(keep + i) * C + c];
    fresh[j] = v;
  }
  for (int j = 0; j < keep; ++j) stp[(long)j * C + c] = fresh[j];
}

struct ScanArgs {
  long ld_src, ld_dt;
  int col_x, col_b, col_c, col_dt;
  int H, G, N, P, act;
  const float* dt_bias;    // [H] with dt
  const float* a_log;      // [H] with dt
  const float* skip;       // [H] or null
  const float* decay;      // [H] without dt
  float* state;            // [nslots, H, N, P]
  const int* seq_first;
  const int* seq_rows;
  const int* state_slots;
  const int* pos32;
  int nslots, T;
};

constexpr int CH = 16;     // rows staged per pass

// One wave per (sequence, head, block of PL = 64 / TPP value channels).
// lane = ns * PL + pl: channel p0 + pl, state rows n = r * TPP + ns. CHG rows
// are staged per pass (fewer for the widest states, to fit the LDS).
template <typename TS, typename TD, int NR, int TPP, int CHG>
__global__ __launch_bounds__(64) void state_scan_kernel(
    float* __restrict__ y, const TS* __restrict__ src,
    const TD* __restrict__ dt_src, ScanArgs p) {
  constexpr int PL = 64 / TPP;
  constexpr int NP = NR * TPP;               // padded state rows
  __shared__ float ks[CHG][NP];
  __shared__ float qs[CHG][NP];
  __shared__ float vs[CHG][PL];
  __shared__ float a_s[CHG], b_s[CHG];
  const int s = blockIdx.x, h = blockIdx.y, p0 = blockIdx.z * PL;
  const int lane = threadIdx.x;
  const int pl = lane % PL, ns = lane / PL;
  const int first = p.seq_first[s], n = p.seq_rows[s];
  if (first < 0 || n < 1 || first + n > p.T) return;
  const int slot = min(max(p.state_slots[s], 0), p.nslots - 1);
  const int hist = p.pos32[first];
  const int N = p.N, P = p.P;
  const int g = h / (p.H / p.G);
  const int pc = p0 + pl;
  const bool live = pc < P;
  float* sp = p.state + ((long)slot * p.H + h) * N * P;
  float S[NR];
#pragma unroll
  for (int r = 0; r < NR; ++r) {
    const int nn = r * TPP + ns;
    S[r] = (hist > 0 && live && nn < N) ? sp[(long)nn * P + pc] : 0.f;
  }
  const float skip = p.skip != nullptr ? p.skip[h] : 0.f;
  const float a_rate = dt_src != nullptr ? expf(p.a_log[h]) : 0.f;
  const float dtb = dt_src != nullptr ? p.dt_bias[h] : 0.f;
  const float a_const = dt_src == nullptr ? p.decay[h] : 0.f;

  for (int c0 = 0; c0 < n; c0 += CHG) {
    const int rows = min(CHG, n - c0);
    __syncthreads();
    for (int i = lane; i < rows * NP; i += 64) {
      const int r = i / NP, nn = i % NP;
      float kv = 0.f, qv = 0.f;
      if (nn < N) {
        const TS* rp = src + (long)(first + c0 + r) * p.ld_src;
        kv = ld(rp + p.col_b + g * N + nn);
        qv = ld(rp + p.col_c + g * N + nn);
        if (p.act) { kv = silu_f(kv); qv = silu_f(qv); }
      }
      ks[r][nn] = kv;
      qs[r][nn] = qv;
    }
    for (int i = lane; i < rows * PL; i += 64) {
      const int r = i / PL, c = i % PL;
      float v = 0.f;
      if (p0 + c < P) {
        v = ld(src + (long)(first + c0 + r) * p.ld_src + p.col_x + h * P + p0 + c);
        if (p.act) v = silu_f(v);
      }
      vs[r][c] = v;
    }
    if (lane < rows) {
      if (dt_src != nullptr) {
        const float dt = softplus_f(
            ld(dt_src + (long)(first + c0 + lane) * p.ld_dt + p.col_dt + h) + dtb);
        a_s[lane] = expf(-a_rate * dt);
        b_s[lane] = dt;
      } else {
        a_s[lane] = a_const;
        b_s[lane] = 1.f;
      }
    }
    __syncthreads();
    for (int r = 0; r < rows; ++r) {
      const float a = a_s[r];
      const float v = vs[r][pl];
      const float bv = b_s[r] * v;
      float acc = 0.f;
#pragma unroll
      for (int j = 0; j < NR; ++j) {
        const int nn = j * TPP + ns;
        S[j] = a * S[j] + ks[r][nn] * bv;
        acc += S[j] * qs[r][nn];
      }
#pragma unroll
      for (int m = PL; m < 64; m <<= 1) acc += __shfl_xor(acc, m, WAVE_SIZE);
      if (ns == 0 && live)
        y[(long)(first + c0 + r) * p.H * P + h * P + pc] = acc + skip * v;
    }
  }
#pragma unroll
  for (int r = 0; r < NR; ++r) {
    const int nn = r * TPP + ns;
    if (live && nn < N) sp[(long)nn * P + pc] = S[r];
  }
}


// The same recurrence for bf16 sources whose sizes and columns are multiples
// of 8: four waves share one (sequence, head) and 4 * PL value channels, so
// k and q are staged once for all of them with 16-byte loads; the next
// CH rows are fetched into registers while the current ones are walked
// (two LDS buffers, one barrier per pass). A lane owns the state rows
// ns * NR .. ns * NR + NR - 1 and reads its k / q slice from LDS in 16-byte
// pieces; slices of different ns sit NR + 4 floats apart, on other banks.
template <int NR, int TPP>
__global__ __launch_bounds__(256) void state_scan_vec_kernel(
    float* __restrict__ y, const unsigned short* __restrict__ src,
    const unsigned short* __restrict__ dt_src, ScanArgs p) {
  constexpr int PL = 64 / TPP;
  constexpr int NP = NR * TPP;
  constexpr int NS = NR + 4;                 // floats between two ns slices
  constexpr int ROW = TPP * NS;              // floats per staged k / q row
  constexpr int PB = 4 * PL;                 // value channels per workgroup
  constexpr int KV = (CH * NP / 8 + 255) / 256;   // 16-byte loads per lane
  constexpr int VV = (CH * PB / 8 + 255) / 256;
  __shared__ __attribute__((aligned(16))) float ks[2][CH][ROW];
  __shared__ __attribute__((aligned(16))) float qs[2][CH][ROW];
  __shared__ float vs[2][CH][PB];
  __shared__ float a_s[2][CH], b_s[2][CH];
  const int s = blockIdx.x, h = blockIdx.y, pb0 = blockIdx.z * PB;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int pl = lane % PL, ns = lane / PL;
  const int first = p.seq_first[s], n = p.seq_rows[s];
  if (first < 0 || n < 1 || first + n > p.T) return;
  const int slot = min(max(p.state_slots[s], 0), p.nslots - 1);
  const int hist = p.pos32[first];
  const int N = p.N, P = p.P;
  const int g = h / (p.H / p.G);
  const int pc = pb0 + wave * PL + pl;
  const bool live = pc < P;
  float* sp = p.state + ((long)slot * p.H + h) * N * P;
  float S[NR];
#pragma unroll
  for (int j = 0; j < NR; ++j) {
    const int nn = ns * NR + j;
    S[j] = (hist > 0 && live && nn < N) ? sp[(long)nn * P + pc] : 0.f;
  }
  const float skip = p.skip != nullptr ? p.skip[h] : 0.f;
  const float a_rate = dt_src != nullptr ? expf(p.a_log[h]) : 0.f;
  const float dtb = dt_src != nullptr ? p.dt_bias[h] : 0.f;
  const float a_const = dt_src == nullptr ? p.decay[h] : 0.f;
  const int nvec = N / 8;                    // 16-byte pieces per k / q row
  const u16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};

  u16x8 kreg[KV], qreg[KV], vreg[VV];
  float dreg = 0.f;
  auto fetch = [&](int c0) {
    const int rows = min(CH, n - c0);
#pragma unroll
    for (int u = 0; u < KV; ++u) {
      const int i = tid + u * 256;
      kreg[u] = zero8;
      qreg[u] = zero8;
      if (i < rows * nvec) {
        const int r = i / nvec, e = (i % nvec) * 8;
        const unsigned short* rp = src + (long)(first + c0 + r) * p.ld_src;
        kreg[u] = *reinterpret_cast<const u16x8*>(rp + p.col_b + g * N + e);
        qreg[u] = *reinterpret_cast<const u16x8*>(rp + p.col_c + g * N + e);
      }
    }
#pragma unroll
    for (int u = 0; u < VV; ++u) {
      const int i = tid + u * 256;
      vreg[u] = zero8;
      if (i < rows * (PB / 8)) {
        const int r = i / (PB / 8), c = (i % (PB / 8)) * 8;
        if (pb0 + c < P)
          vreg[u] = *reinterpret_cast<const u16x8*>(
              src + (long)(first + c0 + r) * p.ld_src + p.col_x + h * P + pb0 + c);
      }
    }
    if (dt_src != nullptr && tid < rows)
      dreg = bf2f(dt_src[(long)(first + c0 + tid) * p.ld_dt + p.col_dt + h]);
  };
  auto stage = [&](int buf, int c0) {
    const int rows = min(CH, n - c0);
#pragma unroll
    for (int u = 0; u < KV; ++u) {
      const int i = tid + u * 256;
      if (i < rows * nvec) {
        const int r = i / nvec, e = (i % nvec) * 8;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          float kv = bf2f(kreg[u][k]), qv = bf2f(qreg[u][k]);
          if (p.act) { kv = silu_f(kv); qv = silu_f(qv); }
          const int nn = e + k;
          const int at = (nn / NR) * NS + nn % NR;
          ks[buf][r][at] = kv;
          qs[buf][r][at] = qv;
        }
      }
    }
#pragma unroll
    for (int u = 0; u < VV; ++u) {
      const int i = tid + u * 256;
      if (i < rows * (PB / 8)) {
        const int r = i / (PB / 8), c = (i % (PB / 8)) * 8;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          float v = bf2f(vreg[u][k]);
          if (p.act) v = silu_f(v);
          vs[buf][r][c + k] = v;
        }
      }
    }
    if (tid < rows) {
      if (dt_src != nullptr) {
        const float dt = softplus_f(dreg + dtb);
        a_s[buf][tid] = expf(-a_rate * dt);
        b_s[buf][tid] = dt;
      } else {
        a_s[buf][tid] = a_const;
        b_s[buf][tid] = 1.f;
      }
    }
  };
  // state rows past N (padding up to NP) keep k = q = 0: zero them once
  for (int i = tid; i < 2 * CH * ROW; i += 256) {
    (&ks[0][0][0])[i] = 0.f;
    (&qs[0][0][0])[i] = 0.f;
  }
  __syncthreads();
  fetch(0);
  int buf = 0;
  for (int c0 = 0; c0 < n; c0 += CH, buf ^= 1) {
    const int rows = min(CH, n - c0);
    stage(buf, c0);
    __syncthreads();
    if (c0 + CH < n) fetch(c0 + CH);
    const float* kb = &ks[buf][0][ns * NS];
    const float* qb = &qs[buf][0][ns * NS];
    for (int r = 0; r < rows; ++r) {
      const float a = a_s[buf][r];
      const float v = vs[buf][r][wave * PL + pl];
      const float bv = b_s[buf][r] * v;
      float acc = 0.f;
#pragma unroll
      for (int j = 0; j < NR; j += 4) {
        const f32x4 k4 = *reinterpret_cast<const f32x4*>(kb + r * ROW + j);
        const f32x4 q4 = *reinterpret_cast<const f32x4*>(qb + r * ROW + j);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          S[j + k] = a * S[j + k] + k4[k] * bv;
          acc += S[j + k] * q4[k];
        }
      }
#pragma unroll
      for (int m = PL; m < 64; m <<= 1) acc += __shfl_xor(acc, m, WAVE_SIZE);
      if (ns == 0 && live)
        y[(long)(first + c0 + r) * p.H * P + h * P + pc] = acc + skip * v;
    }
  }
#pragma unroll
  for (int j = 0; j < NR; ++j) {
    const int nn = ns * NR + j;
    if (live && nn < N) sp[(long)nn * P + pc] = S[j];
  }
}

// Single rows (decode): the state itself is the traffic, so one workgroup
// per (sequence, head) streams it once with 16-byte accesses — a lane
// owns 4 neighbouring value channels of every RP-th state row — updates it
// in place and reduces y over the rows through LDS. More rows of a
// sequence, should a batch bring them, are walked one after the other.
template <typename TS>
__global__ __launch_bounds__(256) void state_step_kernel(
    float* __restrict__ y, const TS* __restrict__ src,
    const TS* __restrict__ dt_src, ScanArgs p) {
  extern __shared__ __attribute__((aligned(16))) float sm[];
  const int N = p.N, P = p.P, P4 = P / 4, RP = 256 / P4;
  float* vs = sm;                 // [P]      (16-byte reads: P % 4 == 0)
  float* part = vs + P;           // [RP][P]
  float* ks = part + RP * P;      // [N]
  float* qs = ks + N;             // [N]
  __shared__ float ab[2];
  const int s = blockIdx.x, h = blockIdx.y;
  const int tid = threadIdx.x;
  const int cg = tid % P4, r0 = tid / P4;
  const int first = p.seq_first[s], n = p.seq_rows[s];
  if (first < 0 || n < 1 || first + n > p.T) return;
  const int slot = min(max(p.state_slots[s], 0), p.nslots - 1);
  const int hist = p.pos32[first];
  const int g = h / (p.H / p.G);
  float* sp = p.state + ((long)slot * p.H + h) * N * P;
  const float skip = p.skip != nullptr ? p.skip[h] : 0.f;
  for (int r = 0; r < n; ++r) {
    const TS* rp = src + (long)(first + r) * p.ld_src;
    __syncthreads();
    for (int i = tid; i < N; i += 256) {
      float kv = ld(rp + p.col_b + g * N + i), qv = ld(rp + p.col_c + g * N + i);
      if (p.act) { kv = silu_f(kv); qv = silu_f(qv); }
      ks[i] = kv;
      qs[i] = qv;
    }
    for (int i = tid; i < P; i += 256) {
      float v = ld(rp + p.col_x + h * P + i);
      vs[i] = p.act ? silu_f(v) : v;
    }
    if (tid == 0) {
      if (dt_src != nullptr) {
        const float dt = softplus_f(
            ld(dt_src + (long)(first + r) * p.ld_dt + p.col_dt + h) + p.dt_bias[h]);
        ab[0] = expf(-expf(p.a_log[h]) * dt);
        ab[1] = dt;
      } else {
        ab[0] = p.decay[h];
        ab[1] = 1.f;
      }
    }
    __syncthreads();
    const float a = ab[0], b = ab[1];
    const bool fresh = hist <= 0 && r == 0;      // start from a zero state
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    if (r0 < RP) {
      const f32x4 v4 = *reinterpret_cast<const f32x4*>(vs + cg * 4);
      for (int nn = r0; nn < N; nn += RP) {
        f32x4* at = reinterpret_cast<f32x4*>(sp + (long)nn * P + cg * 4);
        f32x4 S = fresh ? f32x4{0.f, 0.f, 0.f, 0.f} : *at;
        const float bk = b * ks[nn], qn = qs[nn];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          S[k] = a * S[k] + bk * v4[k];
          acc[k] += S[k] * qn;
        }
        *at = S;
      }
      *reinterpret_cast<f32x4*>(part + r0 * P + cg * 4) = acc;
    }
    __syncthreads();
    for (int i = tid; i < P; i += 256) {
      float o = skip * vs[i];
      for (int k = 0; k < RP; ++k) o += part[k * P + i];
      y[(long)(first + r) * p.H * P + h * P + i] = o;
    }
  }
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

// grid (T, groups): one workgroup per (row, part). gate_first 1: u = y *
// silu(gate), out = u / rms(u) * w; 0: out = y / rms(y) * w * sigmoid(gate);
// 2: out = y / rms(y) * w * silu(gate).
template <typename TG, typename TO>
__global__ __launch_bounds__(ROW_THREADS) void gated_group_norm_kernel(
    TO* __restrict__ out, const float* __restrict__ y,
    const TG* __restrict__ gate, long ld_gate, const float* __restrict__ w,
    int C, int gs, float eps, int gate_first) {
  __shared__ float red[4];
  const long t = blockIdx.x;
  const int c0 = blockIdx.y * gs;
  const float* yr = y + t * C + c0;
  const TG* gr = gate + t * ld_gate + c0;
  float ss = 0.f;
  for (int i = threadIdx.x; i < gs; i += ROW_THREADS) {
    float u = yr[i];
    if (gate_first == 1) u *= silu_f(ld(gr + i));
    ss += u * u;
  }
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)gs + eps);
  for (int i = threadIdx.x; i < gs; i += ROW_THREADS) {
    const float gv = ld(gr + i);
    float u = yr[i];
    if (gate_first == 1) u = u * silu_f(gv) * inv * w[c0 + i];
    else if (gate_first == 2) u = u * inv * w[c0 + i] * silu_f(gv);
    else u = u * inv * w[c0 + i] * sigmoid_f(gv);
    st(out + t * C + c0 + i, u);
  }
}

// The same for bf16 gates and outputs with parts of a multiple of 4 and at
// most 4096 channels: a lane keeps its 4 x NV channels in registers between
// the sum of squares and the store (one pass over y and the gate).
template <int NV>
__global__ __launch_bounds__(ROW_THREADS) void gated_group_norm_vec_kernel(
    unsigned short* __restrict__ out, const float* __restrict__ y,
    const unsigned short* __restrict__ gate, long ld_gate,
    const float* __restrict__ w, int C, int gs, float eps, int gate_first) {
  __shared__ float red[4];
  const long t = blockIdx.x;
  const int c0 = blockIdx.y * gs;
  const float* yr = y + t * C + c0;
  const unsigned short* gr = gate + t * ld_gate + c0;
  float u[NV][4], gv[NV][4];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int i = (threadIdx.x + j * ROW_THREADS) * 4;
    if (i < gs) {
      const f32x4 yv = *reinterpret_cast<const f32x4*>(yr + i);
      const u16x4 g4 = *reinterpret_cast<const u16x4*>(gr + i);
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        gv[j][k] = bf2f(g4[k]);
        u[j][k] = gate_first == 1 ? yv[k] * silu_f(gv[j][k]) : yv[k];
        ss += u[j][k] * u[j][k];
      }
    }
  }
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)gs + eps);
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int i = (threadIdx.x + j * ROW_THREADS) * 4;
    if (i < gs) {
      const f32x4 wv = *reinterpret_cast<const f32x4*>(w + c0 + i);
      u16x4 o;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        float r = u[j][k] * inv * wv[k];
        if (gate_first == 0) r *= sigmoid_f(gv[j][k]);
        else if (gate_first == 2) r *= silu_f(gv[j][k]);
        o[k] = f2bf(r);
      }
      *reinterpret_cast<u16x4*>(out + t * C + c0 + i) = o;
    }
  }
}

// bf16 gates and outputs, parts of a multiple of 4 and at most 256
// channels (per-head norms): LPG lanes share a part, 4 channels each in one
// step, a wave takes 64 / LPG parts of a row and a workgroup four times that.
template <int LPG>
__global__ __launch_bounds__(ROW_THREADS) void gated_group_norm_small_kernel(
    unsigned short* __restrict__ out, const float* __restrict__ y,
    const unsigned short* __restrict__ gate, long ld_gate,
    const float* __restrict__ w, int C, int gs, int groups, float eps,
    int gate_first) {
  constexpr int GPW = 64 / LPG;
  const long t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int grp = (blockIdx.y * 4 + wave) * GPW + lane / LPG;
  const int c = (lane % LPG) * 4;
  const bool live = grp < groups && c < gs;
  const int c0 = grp * gs + c;
  float u[4] = {0.f, 0.f, 0.f, 0.f}, gv[4] = {0.f, 0.f, 0.f, 0.f};
  float ss = 0.f;
  if (live) {
    const f32x4 yv = *reinterpret_cast<const f32x4*>(y + t * C + c0);
    const u16x4 g4 = *reinterpret_cast<const u16x4*>(gate + t * ld_gate + c0);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      gv[k] = bf2f(g4[k]);
      u[k] = gate_first == 1 ? yv[k] * silu_f(gv[k]) : yv[k];
      ss += u[k] * u[k];
    }
  }
#pragma unroll
  for (int m = LPG / 2; m >= 1; m >>= 1) ss += __shfl_xor(ss, m, WAVE_SIZE);
  if (!live) return;
  const float inv = 1.0f / sqrtf(ss / (float)gs + eps);
  const f32x4 wv = *reinterpret_cast<const f32x4*>(w + c0);
  u16x4 o;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    float r = u[k] * inv * wv[k];
    if (gate_first == 0) r *= sigmoid_f(gv[k]);
    else if (gate_first == 2) r *= silu_f(gv[k]);
    o[k] = f2bf(r);
  }
  *reinterpret_cast<u16x4*>(out + t * C + c0) = o;
}

template <typename TS, typename TD, int NR, int TPP>
void scan_launch(float* y, const void* src, const void* dt, const ScanArgs& p,
                 int nseq, hipStream_t s) {
  constexpr int PL = 64 / TPP;
  dim3 grid(nseq, p.H, (p.P + PL - 1) / PL);
  state_scan_kernel<TS, TD, NR, TPP, (NR * TPP > 256 ? 8 : 16)>
      <<<grid, 64, 0, s>>>(y, (const TS*)src, (const TD*)dt, p);
}

// Rows of the state per lane (NR) and lanes per value channel (TPP): the
// fewest lanes per channel that keep NR <= 32, but no more channels per wave
// than the head has.
template <typename TS, typename TD>
bool scan_pick(float* y, const void* src, const void* dt, const ScanArgs& p,
               int nseq, hipStream_t s) {
  int tpp = 1;
  while (tpp < 8 && ((p.N + tpp - 1) / tpp > 32 || 64 / tpp > max(p.P, 8)))
    tpp *= 2;
  // 16-byte staging: bf16 rows whose sizes and columns are multiples of 8
  const bool vec = p.N % 8 == 0 && p.P % 8 == 0 &&
                   p.ld_src % 8 == 0 && p.col_x % 8 == 0 && p.col_b % 8 == 0 &&
                   p.col_c % 8 == 0;
  // few workgroups (long portions of few sequences): more lanes per channel
  // make more, smaller ones, so that every SIMD holds two waves
  while (vec && sizeof(TS) == 2 && tpp < 8 && (p.N + tpp - 1) / tpp >= 16 &&
         (long)nseq * p.H * ((p.P + 4 * (64 / tpp) - 1) / (4 * (64 / tpp))) < 512)
    tpp *= 2;
  const int nr = (p.N + tpp - 1) / tpp;
#define SCAN_CASE(NRV, TPPV)                                              \
  if (tpp == TPPV && nr <= NRV) {                                         \
    constexpr bool fits = sizeof(TS) == 2 &&                              \
        (4 * CH * TPPV * (NRV + 4) + 2 * CH * 4 * (64 / TPPV) + 4 * CH) * 4 \
            <= 60 * 1024;                                                 \
    if constexpr (fits) if (vec) {                                        \
      constexpr int PBV = 4 * (64 / TPPV);                                \
      dim3 grid(nseq, p.H, (p.P + PBV - 1) / PBV);                        \
      state_scan_vec_kernel<NRV, TPPV><<<grid, 256, 0, s>>>(              \
          y, (const unsigned short*)src, (const unsigned short*)dt, p);   \
      return true;                                                        \
    }                                                                     \
    scan_launch<TS, TD, NRV, TPPV>(y, src, dt, p, nseq, s);               \
    return true;                                                          \
  }
#define SCAN_TPP(TPPV) \
  SCAN_CASE(4, TPPV) SCAN_CASE(8, TPPV) SCAN_CASE(16, TPPV) SCAN_CASE(32, TPPV)
  SCAN_TPP(1) SCAN_TPP(2) SCAN_TPP(4) SCAN_TPP(8) SCAN_CASE(64, 8)
#undef SCAN_TPP
#undef SCAN_CASE
  return false;
}

}  // namespace

int state_scan_max_state() { return 8 * 64; }
int conv_max_taps() { return MAX_TAPS; }

void causal_conv_silu_launch(void* out, const void* src, long ld_src, int col0,
                             int C, int taps, const float* w, const float* b,
                             void* conv_state, const int* seq_first,
                             const int* seq_rows, const int* state_slots,
                             const int* row_seq, const int* pos32, int nseq,
                             int nslots, int T, int bf, hipStream_t s) {
  if (T <= 0 || nseq <= 0) return;
  dim3 grid(T, (C + 255) / 256), sgrid(nseq, (C + 255) / 256);
  if (bf) {
    // few rows (decode): one lane per (row, channel) makes more workgroups
    const bool vec = C % 8 == 0 && col0 % 8 == 0 && ld_src % 8 == 0 &&
                     (long)T * C >= (1 << 20);
    const dim3 vgrid((T + RB - 1) / RB, (C / 8 + 255) / 256);
#define CONV_VEC(TAPSV)                                                        \
  causal_conv_silu_vec_kernel<TAPSV><<<vgrid, 256, 0, s>>>(                    \
      (unsigned short*)out, (const unsigned short*)src, ld_src, col0, C, w, b, \
      (const unsigned short*)conv_state, seq_first, state_slots, row_seq,      \
      pos32, nseq, nslots, T)
    if (vec && taps == 4) CONV_VEC(4);
    else if (vec && taps == 3) CONV_VEC(3);
    else if (vec && taps == 2) CONV_VEC(2);
#undef CONV_VEC
    else
      causal_conv_silu_kernel<unsigned short><<<grid, 256, 0, s>>>(
          (unsigned short*)out, (const unsigned short*)src, ld_src, col0, C,
          taps, w, b, (const unsigned short*)conv_state, seq_first, state_slots,
          row_seq, pos32, nseq, nslots, T);
    if (taps > 1)
      conv_state_update_kernel<unsigned short><<<sgrid, 256, 0, s>>>(
          (const unsigned short*)src, ld_src, col0, C, taps,
          (unsigned short*)conv_state, seq_first, seq_rows, state_slots, pos32,
          nslots, T);
  } else {
    causal_conv_silu_kernel<float><<<grid, 256, 0, s>>>(
        (float*)out, (const float*)src, ld_src, col0, C, taps, w, b,
        (const float*)conv_state, seq_first, state_slots, row_seq, pos32, nseq,
        nslots, T);
    if (taps > 1)
      conv_state_update_kernel<float><<<sgrid, 256, 0, s>>>(
          (const float*)src, ld_src, col0, C, taps, (float*)conv_state,
          seq_first, seq_rows, state_slots, pos32, nslots, T);
  }
}

// src_bf: src and dt_src are bf16 (else fp32). single: the caller expects
// one row per sequence (a hint: any batch is still computed correctly).
// Returns 0 when no instantiation covers the sizes.
int state_scan_launch(float* y, const void* src, long ld_src, int col_x,
                      int col_b, int col_c, const void* dt_src, long ld_dt,
                      int col_dt, int H, int G, int N, int P, int act,
                      const float* dt_bias, const float* a_log,
                      const float* skip, const float* decay, float* state,
                      const int* seq_first, const int* seq_rows,
                      const int* state_slots, const int* pos32, int nseq,
                      int nslots, int T, int src_bf, int single,
                      hipStream_t s) {
  if (T <= 0 || nseq <= 0) return 1;
  ScanArgs p;
  p.ld_src = ld_src; p.ld_dt = ld_dt; p.col_x = col_x; p.col_b = col_b;
  p.col_c = col_c; p.col_dt = col_dt; p.H = H; p.G = G; p.N = N; p.P = P;
  p.act = act; p.dt_bias = dt_bias; p.a_log = a_log; p.skip = skip;
  p.decay = decay; p.state = state; p.seq_first = seq_first;
  p.seq_rows = seq_rows; p.state_slots = state_slots; p.pos32 = pos32;
  p.nslots = nslots; p.T = T;
  // batches of single rows: the streaming step kernel, when the value size
  // splits a workgroup evenly into 16-byte columns
  const int P4 = P / 4;
  if (single && P % 4 == 0 && P4 >= 1 && P4 <= 256 && 256 % P4 == 0 &&
      (size_t)(2 * N + P + (256 / P4) * P) * sizeof(float) <= 48 * 1024) {
    const size_t smem = (size_t)(2 * N + P + (256 / P4) * P) * sizeof(float);
    if (src_bf)
      state_step_kernel<unsigned short><<<dim3(nseq, H), 256, smem, s>>>(
          y, (const unsigned short*)src, (const unsigned short*)dt_src, p);
    else
      state_step_kernel<float><<<dim3(nseq, H), 256, smem, s>>>(
          y, (const float*)src, (const float*)dt_src, p);
    return 1;
  }
  if (src_bf)
    return scan_pick<unsigned short, unsigned short>(y, src, dt_src, p, nseq, s);
  return scan_pick<float, float>(y, src, dt_src, p, nseq, s);
}

void gated_group_norm_launch(void* out, const float* y, const void* gate,
                             long ld_gate, const float* w, int T, int C,
                             int groups, float eps, int gate_first, int gate_bf,
                             int out_bf, hipStream_t s) {
  if (T <= 0) return;
  dim3 grid(T, groups);
  const int gs = C / groups;
  if (gate_bf && out_bf && gs % 4 == 0 && C % 4 == 0 && ld_gate % 4 == 0 &&
      gs <= 256 && groups > 1 && ((uintptr_t)gate % 8) == 0) {
    int lpg = 1;
    while (lpg * 4 < gs) lpg *= 2;
    const int gpb = 4 * (64 / lpg);
    const dim3 sgrid(T, (groups + gpb - 1) / gpb);
#define GGN(L)                                                               \
  gated_group_norm_small_kernel<L><<<sgrid, ROW_THREADS, 0, s>>>(            \
      (unsigned short*)out, y, (const unsigned short*)gate, ld_gate, w, C,   \
      gs, groups, eps, gate_first)
    switch (lpg) {
      case 1: GGN(1); break;
      case 2: GGN(2); break;
      case 4: GGN(4); break;
      case 8: GGN(8); break;
      case 16: GGN(16); break;
      case 32: GGN(32); break;
      default: GGN(64); break;
    }
#undef GGN
    return;
  }
  if (gate_bf && out_bf && gs % 4 == 0 && C % 4 == 0 && ld_gate % 4 == 0 &&
      gs <= 4096 && ((uintptr_t)gate % 8) == 0) {
    if (gs <= 1024)
      gated_group_norm_vec_kernel<1><<<grid, ROW_THREADS, 0, s>>>(
          (unsigned short*)out, y, (const unsigned short*)gate, ld_gate, w, C,
          gs, eps, gate_first);
    else
      gated_group_norm_vec_kernel<4><<<grid, ROW_THREADS, 0, s>>>(
          (unsigned short*)out, y, (const unsigned short*)gate, ld_gate, w, C,
          gs, eps, gate_first);
    return;
  }
  if (gate_bf) {
    if (out_bf)
      gated_group_norm_kernel<unsigned short, unsigned short>
          <<<grid, ROW_THREADS, 0, s>>>((unsigned short*)out, y,
                                        (const unsigned short*)gate, ld_gate, w,
                                        C, gs, eps, gate_first);
    else
      gated_group_norm_kernel<unsigned short, float><<<grid, ROW_THREADS, 0, s>>>(
          (float*)out, y, (const unsigned short*)gate, ld_gate, w, C, gs, eps,
          gate_first);
  } else {
    if (out_bf)
      gated_group_norm_kernel<float, unsigned short><<<grid, ROW_THREADS, 0, s>>>(
          (unsigned short*)out, y, (const float*)gate, ld_gate, w, C, gs, eps,
          gate_first);
    else
      gated_group_norm_kernel<float, float><<<grid, ROW_THREADS, 0, s>>>(
          (float*)out, y, (const float*)gate, ld_gate, w, C, gs, eps,
          gate_first);
  }
}
