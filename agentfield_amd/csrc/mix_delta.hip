// Kernels of delta-rule decoders with the norm after the residual sum:
//
//   delta_scan          gated delta rule, token by token in fp32, with the
//                       unit-length q / k, the write strength and the decay
//                       evaluated on the way in
//   qk_rope_cache       bias, per-head RMSNorm, partial rotate-half rotary
//                       positions, K/V page append
//   postnorm_sum        x <- norm(alpha x + sublayer output); the sublayer
//                       output may be the mean of two separately normed
//                       branches
//   gate_gather         act(z) * rows of a per-token table
//
// Storage dtype S is bf16 (raw u16) or fp32; statistics, angles, decays, the
// recurrent state and the residual are fp32.
#include "common.h"

namespace {

template <typename S> __device__ __forceinline__ float ldf(const S* p);
template <> __device__ __forceinline__ float ldf<u16>(const u16* p) { return bf2f(*p); }
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <typename S> __device__ __forceinline__ void stf(S* p, float v);
template <> __device__ __forceinline__ void stf<u16>(u16* p, float v) { *p = f2bf(v); }
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }

template <typename S> __device__ __forceinline__ void ld4(const S* p, float (&o)[4]);
template <> __device__ __forceinline__ void ld4<u16>(const u16* p, float (&o)[4]) {
  const s16x4 v = *reinterpret_cast<const s16x4*>(p);
#pragma unroll
  for (int j = 0; j < 4; ++j) o[j] = bf2f((u16)v[j]);
}
template <> __device__ __forceinline__ void ld4<float>(const float* p, float (&o)[4]) {
  const f32x4 v = *reinterpret_cast<const f32x4*>(p);
#pragma unroll
  for (int j = 0; j < 4; ++j) o[j] = v[j];
}
template <typename S> __device__ __forceinline__ void st4(S* p, const float (&o)[4]);
template <> __device__ __forceinline__ void st4<u16>(u16* p, const float (&o)[4]) {
  s16x4 v;
#pragma unroll
  for (int j = 0; j < 4; ++j) v[j] = (short)f2bf(o[j]);
  *reinterpret_cast<s16x4*>(p) = v;
}
template <> __device__ __forceinline__ void st4<float>(float* p, const float (&o)[4]) {
  *reinterpret_cast<f32x4*>(p) = f32x4{o[0], o[1], o[2], o[3]};
}
template <typename S, int V>
__device__ __forceinline__ void ldv(const S* p, float (&o)[4]) {
  if (V == 4) ld4<S>(p, o);
  else { o[0] = ldf<S>(p); o[1] = o[2] = o[3] = 0.f; }
}
template <typename S, int V>
__device__ __forceinline__ void stv(S* p, const float (&o)[4]) {
  if (V == 4) st4<S>(p, o);
  else stf<S>(p, o[0]);
}

template <int N>
__device__ __forceinline__ void block_sum(float (&v)[N], float* red) {
#pragma unroll
  for (int n = 0; n < N; ++n) v[n] = wave_sum_f32(v[n]);
  const int wave = threadIdx.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) {
#pragma unroll
    for (int n = 0; n < N; ++n) red[n * 4 + wave] = v[n];
  }
  __syncthreads();
#pragma unroll
  for (int n = 0; n < N; ++n)
    v[n] = red[n * 4] + red[n * 4 + 1] + red[n * 4 + 2] + red[n * 4 + 3];
}

template <typename... P>
inline bool aligned16(P... p) {
  return ((((uintptr_t)p) % 16 == 0) && ...);
}

inline int grid_for(i64 n) {
  i64 g = (n + 255) / 256;
  return (int)(g < 1 ? 1 : (g > 8192 ? 8192 : g));
}

// exp / softplus / sigmoid on the way into the recurrence.  fp32 storage:
// the library forms.  bf16 storage: hardware exponential and logarithm (the
// inputs already carry 2^-9 rounding); softplus switches to e^z below -8 so
// that 1 + e^z does not swallow it.
template <typename S> __device__ __forceinline__ float exp_s(float v);
template <> __device__ __forceinline__ float exp_s<u16>(float v) { return __expf(v); }
template <> __device__ __forceinline__ float exp_s<float>(float v) { return expf(v); }
template <typename S> __device__ __forceinline__ float softplus_s(float z);
template <> __device__ __forceinline__ float softplus_s<u16>(float z) {
  const float e = __expf(z);
  return z > 20.f ? z : (z < -8.f ? e : __logf(1.0f + e));
}
template <> __device__ __forceinline__ float softplus_s<float>(float z) {
  return z > 20.f ? z : log1pf(expf(z));
}

template <typename S, int N, bool VEC>
__device__ __forceinline__ void load_run(const S* p, int e0, int n, float (&o)[N]) {
  // N consecutive elements from p + e0, zero past n
  if constexpr (VEC && N >= 4) {
#pragma unroll
    for (int j = 0; j < N; j += 4) {
      float t[4] = {0.f, 0.f, 0.f, 0.f};
      if (e0 + j < n) ld4<S>(p + e0 + j, t);
#pragma unroll
      for (int i = 0; i < 4; ++i) o[j + i] = t[i];
    }
  } else {
#pragma unroll
    for (int j = 0; j < N; ++j) o[j] = (e0 + j < n) ? ldf<S>(p + e0 + j) : 0.f;
  }
}

__device__ __forceinline__ float row16_sum(float v) {
  v += __shfl_xor(v, 1, 64);
  v += __shfl_xor(v, 2, 64);
  v += __shfl_xor(v, 4, 64);
  v += __shfl_xor(v, 8, 64);
  return v;
}

// ------------------------------------------------------------ delta scan
// Workgroup = (sequence, head, 64 state columns); each of its 4 waves owns
// 16 columns and walks alone between the staging barriers.  Lane = (row
// group rg = lane >> 4, column c = lane & 15); a thread keeps the RP rows
// rg*RP .. rg*RP+RP-1 of its column in registers (4*RP >= dk, rows past dk
// stay zero).  Per token, with the decayed column d = g * s:
//     kd = k . d,  qd = q . d        (partial sums, then 2 cross-lane steps)
//     u  = beta (v - kd);  s = d + k u;  o = qd + (q . k) u
// which is S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q with the
// read-out taken after the write.  Tokens advance in blocks of 16: sixteen
// lanes per token fetch the block's q, k, decay logits and values into
// registers while the previous block is being walked; after the walk they
// turn them into unit-length q and k (q also times q_scale), q . k, decays
// and write strengths in LDS.  The order of every sum is fixed, so the state
// does not depend on where a sequence is cut into chunks.
constexpr int DS_TB = 16;

template <typename S, int RP, bool CH, bool VEC>
__global__ void __launch_bounds__(256) delta_scan_kernel(
    float* __restrict__ out, float* __restrict__ state,
    const S* __restrict__ q, i64 ldq, const S* __restrict__ k, i64 ldk,
    const S* __restrict__ v, i64 ldv, const S* __restrict__ beta, i64 ldb,
    const S* __restrict__ dec, i64 ldd, const float* __restrict__ dec_bias,
    const float* __restrict__ rate, const i32* __restrict__ cu,
    const i32* __restrict__ q_start, const i32* __restrict__ sslot, int H,
    int G, int dk, int dv, float q_scale) {
  constexpr int RS = RP + 4;              // padded row-group segment
  constexpr int ROW = 4 * RS;             // one token's k (or q, or g) in LDS
  constexpr int EL = RP / 4;              // staged elements per lane
  __shared__ __attribute__((aligned(16))) float k_s[DS_TB * ROW];
  __shared__ __attribute__((aligned(16))) float q_s[DS_TB * ROW];
  __shared__ __attribute__((aligned(16))) float g_s[CH ? DS_TB * ROW : 4];
  __shared__ __attribute__((aligned(16))) float v_s[DS_TB * 64];
  __shared__ float sc_s[DS_TB * 4];       // per token: beta, q.k, scalar decay

  const int b = blockIdx.x, h = blockIdx.y, col0 = blockIdx.z * 64;
  const int r0 = cu[b], r1 = cu[b + 1];
  if (r1 == r0) return;
  const int g = h / (H / G);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int rg = lane >> 4;
  const int col = col0 + wave * 16 + (lane & 15);
  const bool live = col < dv;
  float* sp = state + ((size_t)sslot[b] * H + h) * (size_t)dk * dv;

  float s[RP];
#pragma unroll
  for (int i = 0; i < RP; ++i) {
    const int row = rg * RP + i;
    s[i] = (q_start[b] > 0 && live && row < dk) ? sp[(size_t)row * dv + col] : 0.f;
  }
  const float rt = rate[h];

  // staging role: token st of the block, elements e0 .. e0 + EL - 1
  const int st = threadIdx.x >> 4, sub = threadIdx.x & 15;
  const int e0 = sub * EL;
  float bias_r[CH ? EL : 1];
  if (CH) {
#pragma unroll
    for (int j = 0; j < EL; ++j)
      bias_r[j] = e0 + j < dk ? dec_bias[(size_t)h * dk + e0 + j] : 0.f;
  } else {
    bias_r[0] = dec_bias[h];
  }
  float fq[EL], fk[EL], fz[CH ? EL : 1], fv[4], fb = 0.f;
  auto fetch = [&](int t0) {
    const int tt = t0 + st;
    if (tt < r1) {
      const size_t t = (size_t)tt;
      load_run<S, EL, VEC>(q + t * ldq + (size_t)g * dk, e0, dk, fq);
      load_run<S, EL, VEC>(k + t * ldk + (size_t)g * dk, e0, dk, fk);
      if (CH) load_run<S, CH ? EL : 1, VEC>(dec + t * ldd + (size_t)h * dk, e0, dk, fz);
      else fz[0] = ldf<S>(dec + t * ldd + h);
      load_run<S, 4, VEC>(v + t * ldv + (size_t)h * dv, col0 + sub * 4, dv, fv);
      fb = ldf<S>(beta + t * ldb + h);
    }
  };
  fetch(r0);

  for (int t0 = r0; t0 < r1; t0 += DS_TB) {
    const int nb = min(DS_TB, r1 - t0);
    __syncthreads();                       // the previous block is consumed
    // ---- fetched values -> LDS ----
    if (st < nb) {
      float sq = 0.f, sk = 0.f, qk = 0.f;
#pragma unroll
      for (int j = 0; j < EL; ++j) {
        sq += fq[j] * fq[j];
        sk += fk[j] * fk[j];
        qk += fq[j] * fk[j];
      }
      sq = row16_sum(sq);
      sk = row16_sum(sk);
      qk = row16_sum(qk);
      const float rq = q_scale / sqrtf(sq + 1e-6f), rk = 1.0f / sqrtf(sk + 1e-6f);
      // EL divides RP: a lane's run lies inside one row group's segment
      const int o = st * ROW + (e0 / RP) * RS + (e0 % RP);
#pragma unroll
      for (int j = 0; j < EL; ++j) {
        q_s[o + j] = fq[j] * rq;
        k_s[o + j] = fk[j] * rk;
        if (CH)
          g_s[o + j] = e0 + j < dk
              ? exp_s<S>(-rt * softplus_s<S>(fz[j] + bias_r[j])) : 1.f;
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) v_s[st * 64 + sub * 4 + j] = fv[j];
      if (sub == 0) {
        sc_s[st * 4 + 0] = 1.0f / (1.0f + exp_s<S>(-fb));
        sc_s[st * 4 + 1] = qk * rq * rk;
        if (!CH) sc_s[st * 4 + 2] = exp_s<S>(-rt * softplus_s<S>(fz[0] + bias_r[0]));
      }
    }
    __syncthreads();
    fetch(t0 + DS_TB);                     // in flight during the walk
    // ---- walk the block: every wave on its own 16 columns ----
    for (int tt = 0; tt < nb; ++tt) {
      const float* kp = k_s + tt * ROW + rg * RS;
      const float* qp = q_s + tt * ROW + rg * RS;
      const float* gp = g_s + tt * ROW + rg * RS;
      const float bt = sc_s[tt * 4 + 0], qk = sc_s[tt * 4 + 1];
      const float gsc = CH ? 1.f : sc_s[tt * 4 + 2];
      float kd = 0.f, qd = 0.f;
      float kk[RP];
#pragma unroll
      for (int i = 0; i < RP; i += 4) {
        const f32x4 k4 = *reinterpret_cast<const f32x4*>(kp + i);
        const f32x4 q4 = *reinterpret_cast<const f32x4*>(qp + i);
        f32x4 g4 = f32x4{gsc, gsc, gsc, gsc};
        if (CH) g4 = *reinterpret_cast<const f32x4*>(gp + i);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float d = s[i + j] * g4[j];
          s[i + j] = d;
          kk[i + j] = k4[j];
          kd += k4[j] * d;
          qd += q4[j] * d;
        }
      }
      kd += __shfl_xor(kd, 16, 64);
      qd += __shfl_xor(qd, 16, 64);
      kd += __shfl_xor(kd, 32, 64);
      qd += __shfl_xor(qd, 32, 64);
      const float u = bt * (v_s[tt * 64 + wave * 16 + (lane & 15)] - kd);
#pragma unroll
      for (int i = 0; i < RP; ++i) s[i] += kk[i] * u;
      if (rg == 0 && live)
        out[(size_t)(t0 + tt) * ((size_t)H * dv) + (size_t)h * dv + col] = qd + qk * u;
    }
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < RP; ++i) {
      const int row = rg * RP + i;
      if (row < dk) sp[(size_t)row * dv + col] = s[i];
    }
  }
}

// Sum over the 16 lanes of a DPP row; every lane gets the total.
__device__ __forceinline__ float row16_sum_dpp(float v) {
  // quad_perm [1,0,3,2], [2,3,0,1]: xor 1, xor 2; then rotate the row by 4, 8
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
      0, __builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
      0, __builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
      0, __builtin_bit_cast(int, v), 0x124, 0xf, 0xf, false));   // row_ror:4
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
      0, __builtin_bit_cast(int, v), 0x128, 0xf, 0xf, false));   // row_ror:8
  return v;
}

// The same recurrence for long chunks (prompts).  Lane = (row group rg =
// lane & 15, column set lane >> 4): a thread keeps the RP rows rg*RP ..
// rg*RP+RP-1 (16*RP >= dk) of CPT adjacent columns, so the sums over rows
// end in four DPP steps inside a 16-lane row and every q / k / decay value
// read from LDS feeds CPT columns.  A wave covers 4*CPT columns, the
// workgroup 16*CPT; the host picks CPT so that the launch fills the chip.
// Staging is the one of delta_scan_kernel: lane `sub` of a token's sixteen
// stages exactly row group `sub`.
template <typename S, int RP, bool CH, bool VEC, int CPT>
__global__ void __launch_bounds__(256) delta_scan_long_kernel(
    float* __restrict__ out, float* __restrict__ state,
    const S* __restrict__ q, i64 ldq, const S* __restrict__ k, i64 ldk,
    const S* __restrict__ v, i64 ldv, const S* __restrict__ beta, i64 ldb,
    const S* __restrict__ dec, i64 ldd, const float* __restrict__ dec_bias,
    const float* __restrict__ rate, const i32* __restrict__ cu,
    const i32* __restrict__ q_start, const i32* __restrict__ sslot, int H,
    int G, int dk, int dv, float q_scale) {
  constexpr int ROW = 16 * RP;            // one token's k (or q, or g) in LDS
  constexpr int NC = 16 * CPT;            // columns of the workgroup
  __shared__ __attribute__((aligned(16))) float k_s[DS_TB * ROW];
  __shared__ __attribute__((aligned(16))) float q_s[DS_TB * ROW];
  __shared__ __attribute__((aligned(16))) float g_s[CH ? DS_TB * ROW : 4];
  __shared__ __attribute__((aligned(16))) float v_s[DS_TB * NC];
  __shared__ float sc_s[DS_TB * 4];       // per token: beta, q.k, scalar decay

  const int b = blockIdx.x, h = blockIdx.y, col0 = blockIdx.z * NC;
  const int r0 = cu[b], r1 = cu[b + 1];
  if (r1 == r0) return;
  const int g = h / (H / G);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int rg = lane & 15;
  const int cl = (wave * 4 + (lane >> 4)) * CPT;   // first column in the tile
  float* sp = state + ((size_t)sslot[b] * H + h) * (size_t)dk * dv;

  float s[CPT][RP];
#pragma unroll
  for (int c = 0; c < CPT; ++c)
#pragma unroll
    for (int i = 0; i < RP; ++i) {
      const int row = rg * RP + i, col = col0 + cl + c;
      s[c][i] = (q_start[b] > 0 && col < dv && row < dk)
          ? sp[(size_t)row * dv + col] : 0.f;
    }
  const float rt = rate[h];

  // staging role: token st of the block, row group sub
  const int st = threadIdx.x >> 4, sub = threadIdx.x & 15;
  const int e0 = sub * RP;
  float bias_r[CH ? RP : 1];
  if (CH) {
#pragma unroll
    for (int j = 0; j < RP; ++j)
      bias_r[j] = e0 + j < dk ? dec_bias[(size_t)h * dk + e0 + j] : 0.f;
  } else {
    bias_r[0] = dec_bias[h];
  }
  float fq[RP], fk[RP], fz[CH ? RP : 1], fv[CPT], fb = 0.f;
  auto fetch = [&](int t0) {
    const int tt = t0 + st;
    if (tt < r1) {
      const size_t t = (size_t)tt;
      load_run<S, RP, VEC>(q + t * ldq + (size_t)g * dk, e0, dk, fq);
      load_run<S, RP, VEC>(k + t * ldk + (size_t)g * dk, e0, dk, fk);
      if (CH) load_run<S, CH ? RP : 1, VEC>(dec + t * ldd + (size_t)h * dk, e0, dk, fz);
      else fz[0] = ldf<S>(dec + t * ldd + h);
      load_run<S, CPT, VEC>(v + t * ldv + (size_t)h * dv, col0 + sub * CPT, dv, fv);
      fb = ldf<S>(beta + t * ldb + h);
    }
  };
  fetch(r0);

  for (int t0 = r0; t0 < r1; t0 += DS_TB) {
    const int nb = min(DS_TB, r1 - t0);
    __syncthreads();                       // the previous block is consumed
    if (st < nb) {
      float sq = 0.f, sk = 0.f, qk = 0.f;
#pragma unroll
      for (int j = 0; j < RP; ++j) {
        sq += fq[j] * fq[j];
        sk += fk[j] * fk[j];
        qk += fq[j] * fk[j];
      }
      sq = row16_sum(sq);
      sk = row16_sum(sk);
      qk = row16_sum(qk);
      const float rq = q_scale / sqrtf(sq + 1e-6f), rk = 1.0f / sqrtf(sk + 1e-6f);
      const int o = st * ROW + e0;
#pragma unroll
      for (int j = 0; j < RP; ++j) {
        q_s[o + j] = fq[j] * rq;
        k_s[o + j] = fk[j] * rk;
        if (CH)
          g_s[o + j] = e0 + j < dk
              ? exp_s<S>(-rt * softplus_s<S>(fz[j] + bias_r[j])) : 1.f;
      }
#pragma unroll
      for (int j = 0; j < CPT; ++j) v_s[st * NC + sub * CPT + j] = fv[j];
      if (sub == 0) {
        sc_s[st * 4 + 0] = 1.0f / (1.0f + exp_s<S>(-fb));
        sc_s[st * 4 + 1] = qk * rq * rk;
        if (!CH) sc_s[st * 4 + 2] = exp_s<S>(-rt * softplus_s<S>(fz[0] + bias_r[0]));
      }
    }
    __syncthreads();
    fetch(t0 + DS_TB);                     // in flight during the walk
    // the next token's LDS values are read while the current one computes
    float kr[RP], qr[RP], gr[RP], sc[3], vv[CPT];
    auto read_tok = [&](int tt, float (&kx)[RP], float (&qx)[RP],
                        float (&gx)[RP], float (&sx)[3], float (&vx)[CPT]) {
      sx[0] = sc_s[tt * 4 + 0];
      sx[1] = sc_s[tt * 4 + 1];
      sx[2] = CH ? 1.f : sc_s[tt * 4 + 2];
      if constexpr (RP >= 4) {
#pragma unroll
        for (int i = 0; i < RP; i += 4) {
          const f32x4 k4 = *reinterpret_cast<const f32x4*>(k_s + tt * ROW + rg * RP + i);
          const f32x4 q4 = *reinterpret_cast<const f32x4*>(q_s + tt * ROW + rg * RP + i);
          f32x4 g4 = f32x4{sx[2], sx[2], sx[2], sx[2]};
          if (CH) g4 = *reinterpret_cast<const f32x4*>(g_s + tt * ROW + rg * RP + i);
#pragma unroll
          for (int j = 0; j < 4; ++j) { kx[i + j] = k4[j]; qx[i + j] = q4[j]; gx[i + j] = g4[j]; }
        }
      } else {
#pragma unroll
        for (int i = 0; i < RP; ++i) {
          kx[i] = k_s[tt * ROW + rg * RP + i];
          qx[i] = q_s[tt * ROW + rg * RP + i];
          gx[i] = CH ? g_s[tt * ROW + rg * RP + i] : sx[2];
        }
      }
#pragma unroll
      for (int c = 0; c < CPT; ++c) vx[c] = v_s[tt * NC + cl + c];
    };
    float kn[RP], qn[RP], gn[RP], sn[3], vn[CPT];
    auto step = [&](int tt, const float (&kx)[RP], const float (&qx)[RP],
                    const float (&gx)[RP], const float (&sx)[3],
                    const float (&vx)[CPT], float (&ky)[RP], float (&qy)[RP],
                    float (&gy)[RP], float (&sy)[3], float (&vy)[CPT]) {
      read_tok(min(tt + 1, DS_TB - 1), ky, qy, gy, sy, vy);
      const float bt = sx[0], qk = sx[1];
      float kd[CPT], qd[CPT];
#pragma unroll
      for (int c = 0; c < CPT; ++c) {
        kd[c] = 0.f;
        qd[c] = 0.f;
#pragma unroll
        for (int i = 0; i < RP; ++i) {
          const float d = s[c][i] * gx[i];
          s[c][i] = d;
          kd[c] += kx[i] * d;
          qd[c] += qx[i] * d;
        }
      }
#pragma unroll
      for (int c = 0; c < CPT; ++c) {
        kd[c] = row16_sum_dpp(kd[c]);
        qd[c] = row16_sum_dpp(qd[c]);
      }
      float o[CPT];
#pragma unroll
      for (int c = 0; c < CPT; ++c) {
        const float u = bt * (vx[c] - kd[c]);
#pragma unroll
        for (int i = 0; i < RP; ++i) s[c][i] += kx[i] * u;
        o[c] = qd[c] + qk * u;
      }
      if (rg == 0) {
        float* op = out + (size_t)(t0 + tt) * ((size_t)H * dv) + (size_t)h * dv + col0 + cl;
#pragma unroll
        for (int c = 0; c < CPT; ++c)
          if (col0 + cl + c < dv) op[c] = o[c];
      }
    };
    read_tok(0, kr, qr, gr, sc, vv);
    for (int tt = 0; tt < nb; tt += 2) {
      step(tt, kr, qr, gr, sc, vv, kn, qn, gn, sn, vn);
      if (tt + 1 < nb) step(tt + 1, kn, qn, gn, sn, vn, kr, qr, gr, sc, vv);
    }
  }
#pragma unroll
  for (int c = 0; c < CPT; ++c)
#pragma unroll
    for (int i = 0; i < RP; ++i) {
      const int row = rg * RP + i, col = col0 + cl + c;
      if (row < dk && col < dv) sp[(size_t)row * dv + col] = s[c][i];
    }
}

// ------------------------------------------------ q/k prep for attention
// cos | sin of position * f_i per row, the product and the functions taken
// in double precision: tab [T, 2*half] fp32.  One table serves every layer
// of a step that rotates with the same frequencies.
__global__ void __launch_bounds__(256) rotary_table_kernel(
    float* __restrict__ tab, const i32* __restrict__ positions,
    const double* __restrict__ inv_freq, i64 n, int half) {
  for (i64 i = (i64)blockIdx.x * 256 + threadIdx.x; i < n;
       i += (i64)gridDim.x * 256) {
    const i64 t = i / half;
    const int j = (int)(i % half);
    const double a = (double)positions[t] * inv_freq[j];
    tab[t * 2 * half + j] = (float)cos(a);
    tab[t * 2 * half + half + j] = (float)sin(a);
  }
}

// 2 consecutive elements (V2) or one
template <typename S, bool V2>
__device__ __forceinline__ void ld2(const S* p, float& a, float& b) {
  if constexpr (!V2) { a = ldf<S>(p); b = 0.f; }
  else if constexpr (sizeof(S) == 2) {
    const uint32_t w = *reinterpret_cast<const uint32_t*>(p);
    a = bf2f((u16)(w & 0xffffu));
    b = bf2f((u16)(w >> 16));
  } else {
    const f32x2 w = *reinterpret_cast<const f32x2*>(p);
    a = w[0];
    b = w[1];
  }
}
template <typename S, bool V2>
__device__ __forceinline__ void st2(S* p, float a, float b) {
  if constexpr (!V2) stf<S>(p, a);
  else if constexpr (sizeof(S) == 2)
    *reinterpret_cast<uint32_t*>(p) = (uint32_t)f2bf(a) | ((uint32_t)f2bf(b) << 16);
  else *reinterpret_cast<f32x2*>(p) = f32x2{a, b};
}

// One workgroup per row, one wave per head at a time.  Every q head and k
// head: + bias, RMSNorm over the head with a weight shared by heads,
// rotate-half rotary positions on the first `rot` dims (dim i pairs with
// i + rot/2) with the row's cos | sin from `tab`.  q goes to a contiguous
// [T, H*dk] buffer, k and v (+ bias) to their pages.  V2: two adjacent
// elements per lane and access (even sizes, 4- / 8-byte aligned rows).
template <typename S, bool V2>
__global__ void __launch_bounds__(256) qk_rope_cache_kernel(
    S* __restrict__ qo, const S* __restrict__ q, i64 ldq,
    const S* __restrict__ k, i64 ldk, const S* __restrict__ v, i64 ldv,
    const S* __restrict__ qb, const S* __restrict__ kb,
    const S* __restrict__ vb, const S* __restrict__ qw,
    const S* __restrict__ kw, const float* __restrict__ tab, int rot,
    S* __restrict__ kc, S* __restrict__ vc, const i64* __restrict__ slots,
    float eps, int H, int G, int dk, int dv, int page) {
  extern __shared__ float sm[];            // [4][dk]
  constexpr int E = V2 ? 2 : 1;
  const int half = rot / 2;
  const int t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const float* cs = tab + (size_t)t * rot;  // [half] cos, [half] sin
  const i64 sl = slots[t];
  const i64 pg = sl / page, off = sl % page;
  float* nb = sm + wave * dk;
  for (int u = wave; u < H + G; u += 4) {
    const bool isq = u < H;
    const int hh = isq ? u : u - H;
    const S* src = isq ? q + (size_t)t * ldq + (size_t)hh * dk
                       : k + (size_t)t * ldk + (size_t)hh * dk;
    const S* bias = isq ? qb : kb;
    const S* w = isq ? qw : kw;
    float ss = 0.f;
    for (int d = lane * E; d < dk; d += 64 * E) {
      float x0, x1, b0 = 0.f, b1 = 0.f;
      ld2<S, V2>(src + d, x0, x1);
      if (bias) ld2<S, V2>(bias + (size_t)hh * dk + d, b0, b1);
      x0 += b0;
      x1 += b1;
      nb[d] = x0;
      if (V2) nb[d + 1] = x1;
      ss += x0 * x0 + x1 * x1;
    }
    ss = wave_sum_f32(ss);
    const float r = w ? 1.0f / sqrtf(ss / (float)dk + eps) : 1.0f;
    for (int d = lane * E; d < dk; d += 64 * E) {
      float w0 = 1.f, w1 = 1.f;
      if (w) ld2<S, V2>(w + d, w0, w1);
      nb[d] = nb[d] * r * w0;              // each lane rewrites its own slots
      if (V2) nb[d + 1] = nb[d + 1] * r * w1;
    }
    __builtin_amdgcn_wave_barrier();       // partners come from other lanes
    S* dst = isq ? qo + ((size_t)t * H + hh) * dk
                 : kc + (((size_t)pg * G + hh) * page + off) * dk;
    if (isq || sl >= 0) {
      for (int d = lane * E; d < dk; d += 64 * E) {
        float o[2];
#pragma unroll
        for (int e = 0; e < E; ++e) {
          const int dd = d + e;
          float x = nb[dd];
          if (dd < half) x = x * cs[dd] - nb[dd + half] * cs[half + dd];
          else if (dd < rot) x = x * cs[dd - half] + nb[dd - half] * cs[dd];
          o[e] = x;
        }
        st2<S, V2>(dst + d, o[0], V2 ? o[1] : 0.f);
      }
    }
    __builtin_amdgcn_wave_barrier();       // the buffer is reused
  }
  if (sl < 0) return;
  for (int i = threadIdx.x * E; i < G * dv; i += 256 * E) {
    float x0, x1, b0 = 0.f, b1 = 0.f;
    ld2<S, V2>(v + (size_t)t * ldv + i, x0, x1);
    if (vb) ld2<S, V2>(vb + i, b0, b1);
    st2<S, V2>(vc + (((size_t)pg * G + i / dv) * page + off) * dv + (i % dv),
               x0 + b0, x1 + b1);
  }
}

// The same for even head sizes up to 128 * NP with aligned rows: a lane owns
// NP element pairs of every head, so its norm weights, cos / sin factors and
// rotation partners are fixed for the row and sit in registers; the next
// head's values are loaded while the current head is reduced and rotated.
template <typename S, int NP>
__global__ void __launch_bounds__(256) qk_rope_cache_pairs_kernel(
    S* __restrict__ qo, const S* __restrict__ q, i64 ldq,
    const S* __restrict__ k, i64 ldk, const S* __restrict__ v, i64 ldv,
    const S* __restrict__ qb, const S* __restrict__ kb,
    const S* __restrict__ vb, const S* __restrict__ qw,
    const S* __restrict__ kw, const float* __restrict__ tab, int rot,
    S* __restrict__ kc, S* __restrict__ vc, const i64* __restrict__ slots,
    float eps, int H, int G, int dk, int dv, int page) {
  extern __shared__ float sm[];            // [4][dk]
  const int half = rot / 2;
  const int t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const float* cs = tab + (size_t)t * rot;
  const i64 sl = slots[t];
  const i64 pg = sl / page, off = sl % page;
  float* nb = sm + wave * dk;
  // per-lane constants of the row: o = n[d] * cc + n[pi] * sn
  float cc[NP][2], sn[NP][2], wq[NP][2], wk[NP][2];
  int pi[NP][2];
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int d = lane * 2 + 128 * p;
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const int dd = d + e;
      cc[p][e] = 1.f; sn[p][e] = 0.f; pi[p][e] = dd < dk ? dd : 0;
      if (dd < half) { cc[p][e] = cs[dd]; sn[p][e] = -cs[half + dd]; pi[p][e] = dd + half; }
      else if (dd < rot) { cc[p][e] = cs[dd - half]; sn[p][e] = cs[dd]; pi[p][e] = dd - half; }
    }
    wq[p][0] = wq[p][1] = wk[p][0] = wk[p][1] = 1.f;
    if (d < dk) {
      if (qw) ld2<S, true>(qw + d, wq[p][0], wq[p][1]);
      if (kw) ld2<S, true>(kw + d, wk[p][0], wk[p][1]);
    }
  }
  auto fetch = [&](int u, float (&x)[NP][2]) {
    const bool isq = u < H;
    const int hh = isq ? u : u - H;
    const S* src = isq ? q + (size_t)t * ldq + (size_t)hh * dk
                       : k + (size_t)t * ldk + (size_t)hh * dk;
    const S* bias = isq ? qb : kb;
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      const int d = lane * 2 + 128 * p;
      x[p][0] = x[p][1] = 0.f;
      if (d < dk) {
        ld2<S, true>(src + d, x[p][0], x[p][1]);
        if (bias) {
          float b0, b1;
          ld2<S, true>(bias + (size_t)hh * dk + d, b0, b1);
          x[p][0] += b0;
          x[p][1] += b1;
        }
      }
    }
  };
  float cur[NP][2], nxt[NP][2];
  if (wave < H + G) fetch(wave, cur);
  for (int u = wave; u < H + G; u += 4) {
    if (u + 4 < H + G) fetch(u + 4, nxt);
    const bool isq = u < H;
    const int hh = isq ? u : u - H;
    float ss = 0.f;
#pragma unroll
    for (int p = 0; p < NP; ++p) ss += cur[p][0] * cur[p][0] + cur[p][1] * cur[p][1];
    ss = wave_sum_f32(ss);
    const float r = (isq ? qw : kw) ? 1.0f / sqrtf(ss / (float)dk + eps) : 1.0f;
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      const int d = lane * 2 + 128 * p;
      if (d < dk) {
        nb[d] = cur[p][0] * r * (isq ? wq[p][0] : wk[p][0]);
        nb[d + 1] = cur[p][1] * r * (isq ? wq[p][1] : wk[p][1]);
      }
    }
    __builtin_amdgcn_wave_barrier();       // partners come from other lanes
    S* dst = isq ? qo + ((size_t)t * H + hh) * dk
                 : kc + (((size_t)pg * G + hh) * page + off) * dk;
    if (isq || sl >= 0) {
#pragma unroll
      for (int p = 0; p < NP; ++p) {
        const int d = lane * 2 + 128 * p;
        if (d < dk)
          st2<S, true>(dst + d, nb[d] * cc[p][0] + nb[pi[p][0]] * sn[p][0],
                       nb[d + 1] * cc[p][1] + nb[pi[p][1]] * sn[p][1]);
      }
    }
    __builtin_amdgcn_wave_barrier();       // the buffer is reused
#pragma unroll
    for (int p = 0; p < NP; ++p) { cur[p][0] = nxt[p][0]; cur[p][1] = nxt[p][1]; }
  }
  if (sl < 0) return;
  for (int i = threadIdx.x * 2; i < G * dv; i += 512) {
    float x0, x1, b0 = 0.f, b1 = 0.f;
    ld2<S, true>(v + (size_t)t * ldv + i, x0, x1);
    if (vb) ld2<S, true>(vb + i, b0, b1);
    st2<S, true>(vc + (((size_t)pg * G + i / dv) * page + off) * dv + (i % dv),
                 x0 + b0, x1 + b1);
  }
}

// --------------------------------------------------------- postnorm sum
// x <- (alpha x + u) / rms(alpha x + u) * w in place on the fp32 residual,
// also written as h in the storage dtype.  u = y, or with a second branch
// u = (y / rms(y) * wy + y2 / rms(y2) * wy2) / 2.
// REG: the row fits 8 passes of the workgroup and waits in registers
// between the sum and the norm; otherwise it waits in x itself.
constexpr int PNS_IT = 8;

template <typename S, typename YT, int V, bool REG>
__global__ void __launch_bounds__(256) postnorm_sum_kernel(
    float* __restrict__ x, S* __restrict__ h, const YT* __restrict__ y,
    i64 ldy, const YT* __restrict__ y2, i64 ldy2, const S* __restrict__ wy,
    const S* __restrict__ wy2, const S* __restrict__ w, float alpha,
    float eps, int W) {
  __shared__ float red[8];
  const int t = blockIdx.x;
  float* xr = x + (size_t)t * W;
  const YT* yr = y + (size_t)t * ldy;
  const YT* y2r = y2 ? y2 + (size_t)t * ldy2 : nullptr;
  float r1 = 1.f, r2 = 0.f;
  if (y2r) {
    float ss[2] = {0.f, 0.f};
    for (int i = threadIdx.x * V; i < W; i += 256 * V) {
      float a[4], b[4];
      ldv<YT, V>(yr + i, a);
      ldv<YT, V>(y2r + i, b);
#pragma unroll
      for (int j = 0; j < V; ++j) { ss[0] += a[j] * a[j]; ss[1] += b[j] * b[j]; }
    }
    block_sum<2>(ss, red);
    r1 = 0.5f / sqrtf(ss[0] / (float)W + eps);
    r2 = 0.5f / sqrtf(ss[1] / (float)W + eps);
  }
  float sv[1] = {0.f};
  float keep[REG ? PNS_IT : 1][4];
  auto sum_at = [&](int i, float (&xv)[4]) {
    float a[4];
    ldv<YT, V>(yr + i, a);
    ldv<float, V>(xr + i, xv);
    if (y2r) {
      float b[4], wa[4], wb[4];
      ldv<YT, V>(y2r + i, b);
      ldv<S, V>(wy + i, wa);
      ldv<S, V>(wy2 + i, wb);
#pragma unroll
      for (int j = 0; j < V; ++j) a[j] = a[j] * r1 * wa[j] + b[j] * r2 * wb[j];
    }
#pragma unroll
    for (int j = 0; j < V; ++j) {
      xv[j] = alpha * xv[j] + a[j];
      sv[0] += xv[j] * xv[j];
    }
  };
  if constexpr (REG) {
#pragma unroll
    for (int it = 0; it < PNS_IT; ++it) {
      const int i = (it * 256 + threadIdx.x) * V;
      if (i < W) sum_at(i, keep[it]);
    }
  } else {
    for (int i = threadIdx.x * V; i < W; i += 256 * V) {
      float xv[4];
      sum_at(i, xv);
      stv<float, V>(xr + i, xv);          // re-read below by the same thread
    }
  }
  block_sum<1>(sv, red);
  const float r = 1.0f / sqrtf(sv[0] / (float)W + eps);
  auto norm_at = [&](int i, float (&xv)[4]) {
    float wv[4];
    ldv<S, V>(w + i, wv);
#pragma unroll
    for (int j = 0; j < V; ++j) xv[j] = xv[j] * r * wv[j];
    stv<float, V>(xr + i, xv);
    if (h) stv<S, V>(h + (size_t)t * W + i, xv);
  };
  if constexpr (REG) {
#pragma unroll
    for (int it = 0; it < PNS_IT; ++it) {
      const int i = (it * 256 + threadIdx.x) * V;
      if (i < W) norm_at(i, keep[it]);
    }
  } else {
    for (int i = threadIdx.x * V; i < W; i += 256 * V) {
      float xv[4];
      ldv<float, V>(xr + i, xv);
      norm_at(i, xv);
    }
  }
}

// out[t, c] = gelu_tanh(z[t, c]) * table[ids[t], off + c]
template <typename S>
__global__ void __launch_bounds__(256) gate_gather_kernel(
    S* __restrict__ out, const S* __restrict__ z, i64 ldz,
    const S* __restrict__ table, i64 ldt, int off,
    const i32* __restrict__ ids, i64 n, int C) {
  for (i64 i = (i64)blockIdx.x * 256 + threadIdx.x; i < n;
       i += (i64)gridDim.x * 256) {
    const i64 t = i / C;
    const int c = (int)(i % C);
    const float a = ldf<S>(z + t * ldz + c);
    const float gl = 0.5f * a * (1.0f + tanhf(0.7978845608028654f *
                                              (a + 0.044715f * a * a * a)));
    stf<S>(out + i, gl * ldf<S>(table + (size_t)ids[t] * ldt + off + c));
  }
}

}  // namespace

#define MIX_DISPATCH(dt, CALL_BF, CALL_F32) \
  do {                                      \
    if ((dt) == 0) { CALL_BF; }             \
    else if ((dt) == 1) { CALL_F32; }       \
    else return 9002;                       \
  } while (0)

AF_EXPORT int afm_delta_scan(
    void* out, void* state, const void* q, i64 ldq, const void* k, i64 ldk,
    const void* v, i64 ldv, const void* beta, i64 ldb, const void* dec,
    i64 ldd, const void* dec_bias, const void* rate, const void* cu,
    const void* q_start, const void* sslot, int B, int H, int G, int dk,
    int dv, int per_channel, float q_scale, int long_chunks, int dt,
    void* stream) {
  if (B == 0) return 0;
  if (H < 1 || G < 1 || H % G != 0 || dk < 1 || dv < 1) return 9003;
  if (dk > 256) return 9004;
  hipStream_t s = (hipStream_t)stream;
  if (long_chunks) {
    // prompts: rows over the lanes of a DPP row; as many columns per thread
    // as still leave two waves per SIMD
    const bool vecl = dk % 4 == 0 && dv % 4 == 0 && ldq % 4 == 0 &&
                      ldk % 4 == 0 && ldv % 4 == 0 && ldd % 4 == 0 &&
                      aligned16(q, k, v, dec);
    const i64 bh = (i64)B * H;
    const int cpt = bh * ((dv + 63) / 64) >= 512 ? 4
                  : bh * ((dv + 31) / 32) >= 512 ? 2 : 1;
    const dim3 gl(B, H, (dv + 16 * cpt - 1) / (16 * cpt));
#define DLV(ST, RPV, CHV, VECV, CP)                                         \
  delta_scan_long_kernel<ST, RPV, CHV, VECV, CP><<<gl, 256, 0, s>>>(        \
      (float*)out, (float*)state, (const ST*)q, ldq, (const ST*)k, ldk,     \
      (const ST*)v, ldv, (const ST*)beta, ldb, (const ST*)dec, ldd,         \
      (const float*)dec_bias, (const float*)rate, (const i32*)cu,           \
      (const i32*)q_start, (const i32*)sslot, H, G, dk, dv, q_scale)
#define DL_CP(ST, RPV, CHV, VECV)                                           \
  do {                                                                      \
    if (cpt == 4) DLV(ST, RPV, CHV, VECV, 4);                               \
    else if (cpt == 2) DLV(ST, RPV, CHV, VECV, 2);                          \
    else DLV(ST, RPV, CHV, VECV, 1);                                        \
  } while (0)
#define DL_CH(ST, RPV)                                                      \
  do {                                                                      \
    if (per_channel) { if (vecl) DL_CP(ST, RPV, true, true); else DL_CP(ST, RPV, true, false); } \
    else { if (vecl) DL_CP(ST, RPV, false, true); else DL_CP(ST, RPV, false, false); } \
  } while (0)
#define DL_RP(ST)                                    \
  do {                                               \
    if (dk <= 16) DL_CH(ST, 1);                      \
    else if (dk <= 32) DL_CH(ST, 2);                 \
    else if (dk <= 64) DL_CH(ST, 4);                 \
    else if (dk <= 128) DL_CH(ST, 8);                \
    else DL_CH(ST, 16);                              \
  } while (0)
    MIX_DISPATCH(dt, DL_RP(u16), DL_RP(float));
#undef DL_RP
#undef DL_CH
#undef DL_CP
#undef DLV
    return af_last_err();
  }
  const dim3 grid(B, H, (dv + 63) / 64);
  // 4-element vector loads: every head's run of q / k / v / decay logits
  // starts on an 8- or 16-byte boundary
  const bool vec = dk % 4 == 0 && dv % 4 == 0 && ldq % 4 == 0 &&
                   ldk % 4 == 0 && ldv % 4 == 0 && ldd % 4 == 0 &&
                   aligned16(q, k, v, dec);
#define DSK(ST, RPV, CHV)                                                   \
  do {                                                                      \
    if (vec) DSKV(ST, RPV, CHV, true); else DSKV(ST, RPV, CHV, false);      \
  } while (0)
#define DSKV(ST, RPV, CHV, VECV)                                            \
  delta_scan_kernel<ST, RPV, CHV, VECV><<<grid, 256, 0, s>>>((float*)out,   \
      (float*)state, (const ST*)q, ldq, (const ST*)k, ldk, (const ST*)v,    \
      ldv, (const ST*)beta, ldb, (const ST*)dec, ldd,                       \
      (const float*)dec_bias, (const float*)rate, (const i32*)cu,           \
      (const i32*)q_start, (const i32*)sslot, H, G, dk, dv, q_scale)
#define DSK_CH(ST, RPV)                              \
  do {                                               \
    if (per_channel) DSK(ST, RPV, true);             \
    else DSK(ST, RPV, false);                        \
  } while (0)
#define DSK_RP(ST)                                   \
  do {                                               \
    if (dk <= 16) DSK_CH(ST, 4);                     \
    else if (dk <= 32) DSK_CH(ST, 8);                \
    else if (dk <= 64) DSK_CH(ST, 16);               \
    else if (dk <= 128) DSK_CH(ST, 32);              \
    else DSK_CH(ST, 64);                             \
  } while (0)
  MIX_DISPATCH(dt, DSK_RP(u16), DSK_RP(float));
#undef DSK_RP
#undef DSK_CH
#undef DSK
#undef DSKV
  return af_last_err();
}

AF_EXPORT int afm_rotary_table(void* tab, const void* positions,
                               const void* inv_freq, int T, int half,
                               void* stream) {
  if (T == 0 || half == 0) return 0;
  const i64 n = (i64)T * half;
  rotary_table_kernel<<<grid_for(n), 256, 0, (hipStream_t)stream>>>(
      (float*)tab, (const i32*)positions, (const double*)inv_freq, n, half);
  return af_last_err();
}

AF_EXPORT int afm_qk_rope_cache(
    void* qo, const void* q, i64 ldq, const void* k, i64 ldk, const void* v,
    i64 ldv, const void* qb, const void* kb, const void* vb, const void* qw,
    const void* kw, const void* tab, int rot, void* kc, void* vc,
    const void* slots, float eps, int T, int H, int G, int dk, int dv,
    int page, int dt, void* stream) {
  if (T == 0) return 0;
  if (rot < 0 || rot > dk || rot % 2 != 0 || (rot > 0 && !tab)) return 9003;
  const size_t smem = (size_t)(4 * dk) * sizeof(float);
  if (smem > 60000) return 9004;
  hipStream_t s = (hipStream_t)stream;
  const size_t al = dt == 0 ? 4 : 8;       // bytes of an element pair
  auto ok = [&](const void* p) { return (uintptr_t)p % al == 0; };
  const bool v2 = dk % 2 == 0 && dv % 2 == 0 && ldq % 2 == 0 && ldk % 2 == 0 &&
                  ldv % 2 == 0 && ok(qo) && ok(q) && ok(k) && ok(v) && ok(qb) &&
                  ok(kb) && ok(vb) && ok(qw) && ok(kw) && ok(kc) && ok(vc);
#define QRC(ST, V2)                                                          \
  qk_rope_cache_kernel<ST, V2><<<T, 256, smem, s>>>((ST*)qo, (const ST*)q,   \
      ldq, (const ST*)k, ldk, (const ST*)v, ldv, (const ST*)qb,              \
      (const ST*)kb, (const ST*)vb, (const ST*)qw, (const ST*)kw,            \
      (const float*)tab, rot, (ST*)kc, (ST*)vc, (const i64*)slots, eps, H,   \
      G, dk, dv, page)
#define QRP(ST, NPV)                                                         \
  qk_rope_cache_pairs_kernel<ST, NPV><<<T, 256, smem, s>>>((ST*)qo,          \
      (const ST*)q, ldq, (const ST*)k, ldk, (const ST*)v, ldv,               \
      (const ST*)qb, (const ST*)kb, (const ST*)vb, (const ST*)qw,            \
      (const ST*)kw, (const float*)tab, rot, (ST*)kc, (ST*)vc,               \
      (const i64*)slots, eps, H, G, dk, dv, page)
  if (v2 && dk <= 128) MIX_DISPATCH(dt, (QRP(u16, 1)), (QRP(float, 1)));
  else if (v2 && dk <= 256) MIX_DISPATCH(dt, (QRP(u16, 2)), (QRP(float, 2)));
  else if (v2) MIX_DISPATCH(dt, (QRC(u16, true)), (QRC(float, true)));
  else MIX_DISPATCH(dt, (QRC(u16, false)), (QRC(float, false)));
#undef QRP
#undef QRC
  return af_last_err();
}

AF_EXPORT int afm_postnorm_sum(void* x, void* h, const void* y, i64 ldy,
                               int y_f32, const void* y2, i64 ldy2,
                               const void* wy, const void* wy2, const void* w,
                               float alpha, float eps, int T, int W, int dt,
                               void* stream) {
  if (T == 0) return 0;
  if (y2 && (!wy || !wy2)) return 9003;
  hipStream_t s = (hipStream_t)stream;
  const bool vec = W % 4 == 0 && ldy % 4 == 0 && ldy2 % 4 == 0 &&
                   aligned16(x, h, y, y2, wy, wy2, w);
  const bool reg = W <= PNS_IT * 256 * (vec ? 4 : 1);
#define PNSK(ST, YT, V, R)                                                   \
  postnorm_sum_kernel<ST, YT, V, R><<<T, 256, 0, s>>>((float*)x, (ST*)h,     \
      (const YT*)y, ldy, (const YT*)y2, ldy2, (const ST*)wy, (const ST*)wy2, \
      (const ST*)w, alpha, eps, W)
#define PNS(ST, YT)                                                          \
  do {                                                                       \
    if (vec) { if (reg) PNSK(ST, YT, 4, true); else PNSK(ST, YT, 4, false); } \
    else { if (reg) PNSK(ST, YT, 1, true); else PNSK(ST, YT, 1, false); }    \
  } while (0)
  if (dt == 0) {
    if (y_f32) PNS(u16, float);
    else PNS(u16, u16);
  } else if (dt == 1) {
    PNS(float, float);
  } else {
    return 9002;
  }
#undef PNS
#undef PNSK
  return af_last_err();
}

AF_EXPORT int afm_gate_gather(void* out, const void* z, i64 ldz,
                              const void* table, i64 ldt, int off,
                              const void* ids, int T, int C, int dt,
                              void* stream) {
  if (T == 0 || C == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const i64 n = (i64)T * C;
  const int grid = grid_for(n);
  MIX_DISPATCH(dt,
      (gate_gather_kernel<u16><<<grid, 256, 0, s>>>((u16*)out, (const u16*)z,
          ldz, (const u16*)table, ldt, off, (const i32*)ids, n, C)),
      (gate_gather_kernel<float><<<grid, 256, 0, s>>>((float*)out,
          (const float*)z, ldz, (const float*)table, ldt, off,
          (const i32*)ids, n, C)));
  return af_last_err();
}
