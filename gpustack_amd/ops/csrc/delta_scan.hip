// Gated delta rule over the recurrent-state pool (gfx950).
//
//   S <- g_t S;   u_t = beta_t (v_t - S^T k_t);   S <- S + k_t u_t^T;
//   y_t = S^T q_t
//
// per (sequence, head), S [N x P] fp32 in the sequence's slot of the state
// pool [slots, H, N, P]; the batch is ragged exactly as for the other
// recurrent mixers (state_scan.hip): sequence s brings rows seq_first[s] ..
// seq_first[s] + seq_rows[s] - 1, and its first row's position says whether
// the slot is read (> 0) or the state starts from zero (== 0).
//
// k and q arrive raw (after the short convolution) and are scaled to unit
// length here, x / sqrt(sum x^2 + 1e-6), q also by N^(-1/2); with the scales
// c_k, c_q and the raw rows in LDS a token costs one pass for both products
// with the decayed state and one for the update:
//
//   d_k = (g S)^T k,  d_q = (g S)^T q            (one pass, two sums)
//   u   = beta (v - c_k d_k);   S = g S + k (c_k u)^T
//   y   = c_q d_q + u (c_k c_q k.q)              (= S_new^T q_hat)
//
// g_t = exp(-exp(A_log) softplus(a_t + dt_bias)) and beta_t = sigmoid(b_t)
// are computed here in fp32 from the projection's columns.
//
//   delta_scan_kernel : a wave owns PL value channels of one (sequence,
//                       head); the N state rows are split over TPP lanes per
//                       channel, NR rows each, in registers; rows are staged
//                       CHG at a time through LDS and walked in order
//   delta_step_kernel : single rows (decode): one workgroup per (sequence,
//                       head) holds the whole state in registers — a lane
//                       owns 4 neighbouring value channels of every RP-th
//                       state row —, streams it in and out once with 16-byte
//                       accesses and reduces the two products through LDS
#include "common.h"

namespace {

template <typename T> DEVICE_INLINE float ld(const T* p);
template <> DEVICE_INLINE float ld<float>(const float* p) { return *p; }
template <> DEVICE_INLINE float ld<unsigned short>(const unsigned short* p) {
  return bf2f(*p);
}

DEVICE_INLINE float softplus_f(float x) {
  return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x)));
}

struct DeltaArgs {
  long ld_src, ld_gate;
  int col_q, col_k, col_v, col_a, col_b;
  int H, G, N, P;
  const float* dt_bias;    // [H]
  const float* a_log;      // [H]
  float* state;            // [nslots, H, N, P]
  const int* seq_first;
  const int* seq_rows;
  const int* state_slots;
  const int* pos32;
  int nslots, T;
  float q_scale;           // N^(-1/2)
};

// lane = ns * PL + pl: channel p0 + pl, state rows n = j * TPP + ns.
template <typename TS, int NR, int TPP, int CHG>
__global__ __launch_bounds__(64) void delta_scan_kernel(
    float* __restrict__ y, const TS* __restrict__ src,
    const TS* __restrict__ gate_src, DeltaArgs p) {
  constexpr int PL = 64 / TPP;
  constexpr int NP = NR * TPP;               // padded state rows
  constexpr int LPR = 64 / CHG;              // lanes per staged row (norms)
  __shared__ float ks[CHG][NP];
  __shared__ float qs[CHG][NP];
  __shared__ float vs[CHG][PL];
  __shared__ float g_s[CHG], b_s[CHG], ck_s[CHG], cq_s[CHG], kq_s[CHG];
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
  for (int j = 0; j < NR; ++j) {
    const int nn = j * TPP + ns;
    S[j] = (hist > 0 && live && nn < N) ? sp[(long)nn * P + pc] : 0.f;
  }
  const float a_rate = expf(p.a_log[h]);
  const float dtb = p.dt_bias[h];

  for (int c0 = 0; c0 < n; c0 += CHG) {
    const int rows = min(CHG, n - c0);
    __syncthreads();
    for (int i = lane; i < rows * NP; i += 64) {
      const int r = i / NP, nn = i % NP;
      float kv = 0.f, qv = 0.f;
      if (nn < N) {
        const TS* rp = src + (long)(first + c0 + r) * p.ld_src;
        kv = ld(rp + p.col_k + g * N + nn);
        qv = ld(rp + p.col_q + g * N + nn);
      }
      ks[r][nn] = kv;
      qs[r][nn] = qv;
    }
    for (int i = lane; i < rows * PL; i += 64) {
      const int r = i / PL, c = i % PL;
      vs[r][c] = p0 + c < P ? ld(src + (long)(first + c0 + r) * p.ld_src +
                                 p.col_v + h * P + p0 + c)
                            : 0.f;
    }
    if (lane < rows) {
      const TS* gp = gate_src + (long)(first + c0 + lane) * p.ld_gate;
      const float dt = softplus_f(ld(gp + p.col_a + h) + dtb);
      g_s[lane] = expf(-a_rate * dt);
      b_s[lane] = 1.0f / (1.0f + expf(-ld(gp + p.col_b + h)));
    }
    __syncthreads();
    {
      // lengths of k and q and their product, LPR lanes per staged row
      const int r = lane / LPR, sub = lane % LPR;
      float kk = 0.f, qq = 0.f, kq = 0.f;
      if (r < rows) {
        for (int nn = sub; nn < N; nn += LPR) {
          const float kv = ks[r][nn], qv = qs[r][nn];
          kk += kv * kv;
          qq += qv * qv;
          kq += kv * qv;
        }
      }
#pragma unroll
      for (int m = 1; m < LPR; m <<= 1) {
        kk += __shfl_xor(kk, m, WAVE_SIZE);
        qq += __shfl_xor(qq, m, WAVE_SIZE);
        kq += __shfl_xor(kq, m, WAVE_SIZE);
      }
      if (r < rows && sub == 0) {
        const float ck = 1.0f / sqrtf(kk + 1e-6f);
        const float cq = p.q_scale / sqrtf(qq + 1e-6f);
        ck_s[r] = ck;
        cq_s[r] = cq;
        kq_s[r] = ck * cq * kq;
      }
    }
    __syncthreads();
    for (int r = 0; r < rows; ++r) {
      const float a = g_s[r];
      float dk = 0.f, dq = 0.f;
#pragma unroll
      for (int j = 0; j < NR; ++j) {
        const int nn = j * TPP + ns;
        S[j] *= a;
        dk += S[j] * ks[r][nn];
        dq += S[j] * qs[r][nn];
      }
#pragma unroll
      for (int m = PL; m < 64; m <<= 1) {
        dk += __shfl_xor(dk, m, WAVE_SIZE);
        dq += __shfl_xor(dq, m, WAVE_SIZE);
      }
      const float ck = ck_s[r];
      const float u = b_s[r] * (vs[r][pl] - ck * dk);
      const float cu = ck * u;
#pragma unroll
      for (int j = 0; j < NR; ++j) S[j] += ks[r][j * TPP + ns] * cu;
      if (ns == 0 && live)
        y[(long)(first + c0 + r) * p.H * P + h * P + pc] =
            cq_s[r] * dq + u * kq_s[r];
    }
  }
#pragma unroll
  for (int j = 0; j < NR; ++j) {
    const int nn = j * TPP + ns;
    if (live && nn < N) sp[(long)nn * P + pc] = S[j];
  }
}


// The same recurrence for bf16 sources whose sizes and columns are multiples
// of 8: four waves share one (sequence, head) and 4 * PL value channels, so
// k and q are staged once for all of them with 16-byte loads; the next CH
// rows are fetched into registers while the current ones are walked (two LDS
// buffers). A lane owns the state rows ns * NR .. ns * NR + NR - 1 and reads
// its k / q slice from LDS in 16-byte pieces; slices of different ns sit
// NR + 4 floats apart, on other banks. The lengths of k and q and their
// product are summed from the staged rows, 16 lanes per row.
constexpr int CH = 16;     // rows staged per pass

template <int NR, int TPP>
__global__ __launch_bounds__(256) void delta_scan_vec_kernel(
    float* __restrict__ y, const unsigned short* __restrict__ src,
    const unsigned short* __restrict__ gate_src, DeltaArgs p) {
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
  __shared__ float g_s[2][CH], b_s[2][CH], ck_s[2][CH], cq_s[2][CH], kq_s[2][CH];
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
  const float a_rate = expf(p.a_log[h]);
  const float dtb = p.dt_bias[h];
  const int nvec = N / 8;                    // 16-byte pieces per k / q row
  const u16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};

  u16x8 kreg[KV], qreg[KV], vreg[VV];
  float areg = 0.f, breg = 0.f;
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
        kreg[u] = *reinterpret_cast<const u16x8*>(rp + p.col_k + g * N + e);
        qreg[u] = *reinterpret_cast<const u16x8*>(rp + p.col_q + g * N + e);
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
              src + (long)(first + c0 + r) * p.ld_src + p.col_v + h * P + pb0 + c);
      }
    }
    if (tid < rows) {
      const unsigned short* gp = gate_src + (long)(first + c0 + tid) * p.ld_gate;
      areg = bf2f(gp[p.col_a + h]);
      breg = bf2f(gp[p.col_b + h]);
    }
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
          const int nn = e + k;
          const int at = (nn / NR) * NS + nn % NR;
          ks[buf][r][at] = bf2f(kreg[u][k]);
          qs[buf][r][at] = bf2f(qreg[u][k]);
        }
      }
    }
#pragma unroll
    for (int u = 0; u < VV; ++u) {
      const int i = tid + u * 256;
      if (i < rows * (PB / 8)) {
        const int r = i / (PB / 8), c = (i % (PB / 8)) * 8;
#pragma unroll
        for (int k = 0; k < 8; ++k) vs[buf][r][c + k] = bf2f(vreg[u][k]);
      }
    }
    if (tid < rows) {
      const float dt = softplus_f(areg + dtb);
      g_s[buf][tid] = expf(-a_rate * dt);
      b_s[buf][tid] = 1.0f / (1.0f + expf(-breg));
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
    {
      // 16 lanes per staged row: sum over the padded row (zeros add nothing)
      const int r = tid >> 4, sub = tid & 15;
      float kk = 0.f, qq = 0.f, kq = 0.f;
      for (int i = sub; i < ROW; i += 16) {
        const float kv = ks[buf][r][i], qv = qs[buf][r][i];
        kk += kv * kv;
        qq += qv * qv;
        kq += kv * qv;
      }
#pragma unroll
      for (int m = 8; m >= 1; m >>= 1) {
        kk += __shfl_xor(kk, m, WAVE_SIZE);
        qq += __shfl_xor(qq, m, WAVE_SIZE);
        kq += __shfl_xor(kq, m, WAVE_SIZE);
      }
      if (sub == 0) {
        const float ck = 1.0f / sqrtf(kk + 1e-6f);
        const float cq = p.q_scale / sqrtf(qq + 1e-6f);
        ck_s[buf][r] = ck;
        cq_s[buf][r] = cq;
        kq_s[buf][r] = ck * cq * kq;
      }
    }
    __syncthreads();
    if (c0 + CH < n) fetch(c0 + CH);
    const float* kb = &ks[buf][0][ns * NS];
    const float* qb = &qs[buf][0][ns * NS];
    for (int r = 0; r < rows; ++r) {
      const float a = g_s[buf][r];
      float dk = 0.f, dq = 0.f;
      f32x4 k4[NR / 4];
#pragma unroll
      for (int j = 0; j < NR; j += 4) {
        k4[j / 4] = *reinterpret_cast<const f32x4*>(kb + r * ROW + j);
        const f32x4 q4 = *reinterpret_cast<const f32x4*>(qb + r * ROW + j);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          S[j + k] *= a;
          dk += S[j + k] * k4[j / 4][k];
          dq += S[j + k] * q4[k];
        }
      }
#pragma unroll
      for (int m = PL; m < 64; m <<= 1) {
        dk += __shfl_xor(dk, m, WAVE_SIZE);
        dq += __shfl_xor(dq, m, WAVE_SIZE);
      }
      const float ck = ck_s[buf][r];
      const float u = b_s[buf][r] * (vs[buf][r][wave * PL + pl] - ck * dk);
      const float cu = ck * u;
#pragma unroll
      for (int j = 0; j < NR; j += 4)
#pragma unroll
        for (int k = 0; k < 4; ++k) S[j + k] += k4[j / 4][k] * cu;
      if (ns == 0 && live)
        y[(long)(first + c0 + r) * p.H * P + h * P + pc] =
            cq_s[buf][r] * dq + u * kq_s[buf][r];
    }
  }
#pragma unroll
  for (int j = 0; j < NR; ++j) {
    const int nn = ns * NR + j;
    if (live && nn < N) sp[(long)nn * P + pc] = S[j];
  }
}

DEVICE_INLINE float block_sum3(float v, float* red, int slot) {
  v = wave_reduce_sum(v);
  if ((threadIdx.x & 63) == 0) red[slot * 4 + (threadIdx.x >> 6)] = v;
  return v;
}

// P % 4 == 0, P / 4 divides 256, N <= NI * (256 / (P / 4)). Thread (r0, cg):
// value channels 4 cg .. 4 cg + 3 of state rows r0, r0 + RP, ...
template <typename TS, int NI>
__global__ __launch_bounds__(256) void delta_step_kernel(
    float* __restrict__ y, const TS* __restrict__ src,
    const TS* __restrict__ gate_src, DeltaArgs p) {
  extern __shared__ __attribute__((aligned(16))) float sm[];
  const int N = p.N, P = p.P, P4 = P / 4, RP = 256 / P4;
  float* vs = sm;                    // [P]
  float* pk = vs + P;                // [RP][P] partial d_k
  float* pq = pk + RP * P;           // [RP][P] partial d_q
  float* ks = pq + RP * P;           // [N]
  float* qs = ks + N;                // [N]
  __shared__ float red[12];
  __shared__ float gb[2];
  const int s = blockIdx.x, h = blockIdx.y;
  const int tid = threadIdx.x;
  const int cg = tid % P4, r0 = tid / P4;
  const int first = p.seq_first[s], n = p.seq_rows[s];
  if (first < 0 || n < 1 || first + n > p.T) return;
  const int slot = min(max(p.state_slots[s], 0), p.nslots - 1);
  const int hist = p.pos32[first];
  const int g = h / (p.H / p.G);
  float* sp = p.state + ((long)slot * p.H + h) * N * P;
  f32x4 S[NI];
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const int nn = r0 + i * RP;
    S[i] = (hist > 0 && nn < N)
               ? *reinterpret_cast<const f32x4*>(sp + (long)nn * P + cg * 4)
               : f32x4{0.f, 0.f, 0.f, 0.f};
  }
  for (int r = 0; r < n; ++r) {
    const TS* rp = src + (long)(first + r) * p.ld_src;
    __syncthreads();
    float kk = 0.f, qq = 0.f, kq = 0.f;
    for (int i = tid; i < N; i += 256) {
      const float kv = ld(rp + p.col_k + g * N + i);
      const float qv = ld(rp + p.col_q + g * N + i);
      ks[i] = kv;
      qs[i] = qv;
      kk += kv * kv;
      qq += qv * qv;
      kq += kv * qv;
    }
    for (int i = tid; i < P; i += 256) vs[i] = ld(rp + p.col_v + h * P + i);
    block_sum3(kk, red, 0);
    block_sum3(qq, red, 1);
    block_sum3(kq, red, 2);
    if (tid == 0) {
      const TS* gp = gate_src + (long)(first + r) * p.ld_gate;
      const float dt = softplus_f(ld(gp + p.col_a + h) + p.dt_bias[h]);
      gb[0] = expf(-expf(p.a_log[h]) * dt);
      gb[1] = 1.0f / (1.0f + expf(-ld(gp + p.col_b + h)));
    }
    __syncthreads();
    kk = red[0] + red[1] + red[2] + red[3];
    qq = red[4] + red[5] + red[6] + red[7];
    kq = red[8] + red[9] + red[10] + red[11];
    const float ck = 1.0f / sqrtf(kk + 1e-6f);
    const float cq = p.q_scale / sqrtf(qq + 1e-6f);
    const float a = gb[0], beta = gb[1];
    f32x4 dk = {0.f, 0.f, 0.f, 0.f}, dq = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int nn = r0 + i * RP;
      const float kn = nn < N ? ks[nn] : 0.f, qn = nn < N ? qs[nn] : 0.f;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        S[i][k] *= a;
        dk[k] += S[i][k] * kn;
        dq[k] += S[i][k] * qn;
      }
    }
    if (r0 < RP) {
      *reinterpret_cast<f32x4*>(pk + r0 * P + cg * 4) = dk;
      *reinterpret_cast<f32x4*>(pq + r0 * P + cg * 4) = dq;
    }
    __syncthreads();
    dk = f32x4{0.f, 0.f, 0.f, 0.f};
    dq = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int k = 0; k < RP; ++k) {
      const f32x4 a4 = *reinterpret_cast<const f32x4*>(pk + k * P + cg * 4);
      const f32x4 b4 = *reinterpret_cast<const f32x4*>(pq + k * P + cg * 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) { dk[e] += a4[e]; dq[e] += b4[e]; }
    }
    const f32x4 v4 = *reinterpret_cast<const f32x4*>(vs + cg * 4);
    f32x4 u, cu;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      u[e] = beta * (v4[e] - ck * dk[e]);
      cu[e] = ck * u[e];
    }
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int nn = r0 + i * RP;
      const float kn = nn < N ? ks[nn] : 0.f;
#pragma unroll
      for (int e = 0; e < 4; ++e) S[i][e] += kn * cu[e];
    }
    if (r0 == 0) {
      const float kqs = ck * cq * kq;
      f32x4 o;
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = cq * dq[e] + u[e] * kqs;
      *reinterpret_cast<f32x4*>(y + (long)(first + r) * p.H * P + h * P +
                                cg * 4) = o;
    }
  }
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const int nn = r0 + i * RP;
    if (nn < N && r0 < RP)
      *reinterpret_cast<f32x4*>(sp + (long)nn * P + cg * 4) = S[i];
  }
}

template <typename TS, int NR, int TPP>
void delta_launch(float* y, const void* src, const void* gate,
                  const DeltaArgs& p, int nseq, hipStream_t s) {
  constexpr int PL = 64 / TPP;
  dim3 grid(nseq, p.H, (p.P + PL - 1) / PL);
  delta_scan_kernel<TS, NR, TPP, (NR * TPP > 256 ? 8 : 16)>
      <<<grid, 64, 0, s>>>(y, (const TS*)src, (const TS*)gate, p);
}

// Rows of the state per lane (NR) and lanes per value channel (TPP): the
// fewest lanes per channel that keep NR <= 32, but no more channels per wave
// than the head has; more lanes per channel when that leaves few waves.
template <typename TS>
bool delta_pick(float* y, const void* src, const void* gate,
                const DeltaArgs& p, int nseq, hipStream_t s) {
  int tpp = 1;
  while (tpp < 8 && ((p.N + tpp - 1) / tpp > 32 || 64 / tpp > max(p.P, 8)))
    tpp *= 2;
  while (tpp < 8 && (p.N + tpp - 1) / tpp >= 16 &&
         (long)nseq * p.H * ((p.P + 64 / tpp - 1) / (64 / tpp)) < 1024)
    tpp *= 2;
  // 16-byte staging: bf16 rows whose sizes and columns are multiples of 8
  const bool vec = sizeof(TS) == 2 && p.N % 8 == 0 && p.P % 8 == 0 &&
                   p.ld_src % 8 == 0 && p.col_q % 8 == 0 && p.col_k % 8 == 0 &&
                   p.col_v % 8 == 0;
  const int nr = (p.N + tpp - 1) / tpp;
#define DELTA_CASE(NRV, TPPV)                                                \
  if (tpp == TPPV && nr <= NRV) {                                            \
    constexpr bool fits = sizeof(TS) == 2 && NRV % 4 == 0 &&                 \
        (4 * CH * TPPV * (NRV + 4) + 2 * CH * 4 * (64 / TPPV) + 10 * CH) * 4 \
            <= 60 * 1024;                                                    \
    if constexpr (fits) if (vec) {                                           \
      constexpr int PBV = 4 * (64 / TPPV);                                   \
      dim3 grid(nseq, p.H, (p.P + PBV - 1) / PBV);                           \
      delta_scan_vec_kernel<NRV, TPPV><<<grid, 256, 0, s>>>(                 \
          y, (const unsigned short*)src, (const unsigned short*)gate, p);    \
      return true;                                                           \
    }                                                                        \
    delta_launch<TS, NRV, TPPV>(y, src, gate, p, nseq, s);                   \
    return true;                                                             \
  }
#define DELTA_TPP(TPPV) \
  DELTA_CASE(4, TPPV) DELTA_CASE(8, TPPV) DELTA_CASE(16, TPPV) DELTA_CASE(32, TPPV)
  DELTA_TPP(1) DELTA_TPP(2) DELTA_TPP(4) DELTA_TPP(8) DELTA_CASE(64, 8)
#undef DELTA_TPP
#undef DELTA_CASE
  return false;
}

template <typename TS>
bool delta_step_pick(float* y, const void* src, const void* gate,
                     const DeltaArgs& p, int nseq, hipStream_t s) {
  const int P4 = p.P / 4;
  if (p.P % 4 != 0 || P4 < 1 || P4 > 256 || 256 % P4 != 0) return false;
  const int RP = 256 / P4;
  const int ni = (p.N + RP - 1) / RP;
  const size_t smem = (size_t)(p.P + 2 * RP * p.P + 2 * p.N) * sizeof(float);
  if (smem > 48 * 1024) return false;
  const dim3 grid(nseq, p.H);
#define STEP_CASE(NIV)                                                       \
  if (ni <= NIV) {                                                           \
    delta_step_kernel<TS, NIV><<<grid, 256, smem, s>>>(                      \
        y, (const TS*)src, (const TS*)gate, p);                              \
    return true;                                                             \
  }
  STEP_CASE(1) STEP_CASE(2) STEP_CASE(4) STEP_CASE(8) STEP_CASE(16) STEP_CASE(32)
#undef STEP_CASE
  return false;
}

}  // namespace

int delta_scan_max_state() { return 8 * 64; }

// src_bf: src and gate_src are bf16 (else fp32). single: the caller expects
// one row per sequence (a hint: any batch is still computed correctly).
// Returns 0 when no instantiation covers the sizes.
int delta_scan_launch(float* y, const void* src, long ld_src, int col_q,
                      int col_k, int col_v, const void* gate_src, long ld_gate,
                      int col_a, int col_b, int H, int G, int N, int P,
                      const float* dt_bias, const float* a_log, float* state,
                      const int* seq_first, const int* seq_rows,
                      const int* state_slots, const int* pos32, int nseq,
                      int nslots, int T, int src_bf, int single,
                      hipStream_t s) {
  if (T <= 0 || nseq <= 0) return 1;
  DeltaArgs p;
  p.ld_src = ld_src; p.ld_gate = ld_gate; p.col_q = col_q; p.col_k = col_k;
  p.col_v = col_v; p.col_a = col_a; p.col_b = col_b; p.H = H; p.G = G;
  p.N = N; p.P = P; p.dt_bias = dt_bias; p.a_log = a_log; p.state = state;
  p.seq_first = seq_first; p.seq_rows = seq_rows; p.state_slots = state_slots;
  p.pos32 = pos32; p.nslots = nslots; p.T = T;
  p.q_scale = 1.0f / sqrtf((float)N);
  if (single) {
    const bool ok = src_bf ? delta_step_pick<unsigned short>(y, src, gate_src, p, nseq, s)
                           : delta_step_pick<float>(y, src, gate_src, p, nseq, s);
    if (ok) return 1;
  }
  if (src_bf) return delta_pick<unsigned short>(y, src, gate_src, p, nseq, s);
  return delta_pick<float>(y, src, gate_src, p, nseq, s);
}
