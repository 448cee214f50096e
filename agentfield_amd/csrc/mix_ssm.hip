// Selective state-space mixer (Mamba-1 form) over packed row chunks: the
// token-serial selective scan with one fp32 state matrix [channels, N] per
// sequence slot (its depthwise causal convolution lives in mix_conv.hip).
//
// Storage dtype S is bf16 (raw u16) or fp32.  Step sizes (softplus), decays
// (exp), the state and its update are fp32; the scan walks tokens strictly
// in order, so results do not depend on where a sequence was cut.
#include "common.h"
#include <stdlib.h>

namespace {

template <typename S> __device__ __forceinline__ float ldf(const S* p);
template <> __device__ __forceinline__ float ldf<u16>(const u16* p) { return bf2f(*p); }
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <typename S> __device__ __forceinline__ void stf(S* p, float v);
template <> __device__ __forceinline__ void stf<u16>(u16* p, float v) { *p = f2bf(v); }
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }

// exp for decays: hardware exp2 when the inputs already carry bf16 rounding,
// the precise library form for fp32 storage
template <typename S> __device__ __forceinline__ float decay_exp(float v);
template <> __device__ __forceinline__ float decay_exp<u16>(float v) { return __expf(v); }
template <> __device__ __forceinline__ float decay_exp<float>(float v) { return expf(v); }
// softplus and silu of staged values, same split: hardware exp / log / rcp
// behind bf16 inputs, library forms for fp32 storage
template <typename S> __device__ __forceinline__ float softplus_f(float v);
template <> __device__ __forceinline__ float softplus_f<u16>(float v) {
  // far below zero log(1 + e^v) = e^v to rounding; 1 + e^v would lose it
  return v > 20.f ? v : (v < -8.f ? __expf(v) : __logf(1.0f + __expf(v)));
}
template <> __device__ __forceinline__ float softplus_f<float>(float v) {
  return v > 20.f ? v : log1pf(expf(v));
}
template <typename S> __device__ __forceinline__ float silu_f(float v);
template <> __device__ __forceinline__ float silu_f<u16>(float v) {
  return v * __frcp_rn(1.0f + __expf(-v));
}
template <> __device__ __forceinline__ float silu_f<float>(float v) {
  return v / (1.0f + expf(-v));
}

// ---------------------------------------------------------- selective scan
// Workgroup = (block of CB channels, sequence); 256 threads = CB channels x
// NL state lanes (NL = 4, CB = 64, or NL = 16, CB = 16 for large N or few
// sequences),
// lane l keeping the PER consecutive states n = l*PER .. l*PER+PER-1 of its
// channel in registers.  Tokens are staged TB at a time into LDS (step size
// after softplus, input, silu(z), B and C rows), then walked serially:
//   S[c,n] = exp(dt_c A[c,n]) S[c,n] + dt_c x_c B_n ;  y_c = sum_n S[c,n] C_n
// with the sum over the NL lanes taken by DPP / shuffles.  The outputs of a
// token block, (y + D x) * silu(z), leave through LDS as contiguous row
// segments in the storage dtype.
constexpr int SCAN_TB = 16;

template <int NL>
__device__ __forceinline__ float lanes_sum(float v) {
#pragma unroll
  for (int o = NL / 2; o >= 4; o >>= 1) v += __shfl_xor(v, o, 64);
  // quad_perm [2,3,0,1] and [1,0,3,2]: xor 2, xor 1 inside a quad
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
      0, __builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
      0, __builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, false));
  return v;
}

template <typename S, int NL, int PER>
__global__ void __launch_bounds__(256) selective_scan_kernel(
    S* __restrict__ out, float* __restrict__ state, const S* __restrict__ x,
    const S* __restrict__ dtp, const S* __restrict__ dt_bias,
    const S* __restrict__ bc, i64 ldbc, const S* __restrict__ z, i64 ldz,
    const float* __restrict__ A, const float* __restrict__ D,
    const i32* __restrict__ cu, const i32* __restrict__ q_start,
    const i32* __restrict__ sslot, int C, int N) {
  constexpr int CB = 256 / NL;
  extern __shared__ float sh[];
  float* s_dt = sh;                              // [TB][CB]
  float* s_x = s_dt + SCAN_TB * CB;              // [TB][CB]
  float* s_z = s_x + SCAN_TB * CB;               // [TB][CB], silu(z)
  float* s_y = s_z + SCAN_TB * CB;               // [TB][CB]
  float* s_b = s_y + SCAN_TB * CB;               // [TB][N]
  float* s_c = s_b + SCAN_TB * N;                // [TB][N]
  const int b = blockIdx.y;
  const int r0 = cu[b], L = cu[b + 1] - r0;
  if (L == 0) return;
  const int c0 = blockIdx.x * CB;
  const int cl = threadIdx.x / NL, lane = threadIdx.x % NL;
  const int c = c0 + cl;
  const bool okc = c < C;
  float* sb = state + ((size_t)sslot[b] * C + (okc ? c : 0)) * N;
  float st[PER], a[PER];
  const bool fresh = q_start[b] == 0;
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int n = lane * PER + j;
    const bool ok = okc && n < N;
    st[j] = (ok && !fresh) ? sb[n] : 0.f;
    a[j] = ok ? A[(size_t)c * N + n] : 0.f;
  }
  const float dcoef = okc ? D[c] : 0.f;
  for (int tb = 0; tb < L; tb += SCAN_TB) {
    const int nt = min(SCAN_TB, L - tb);
    __syncthreads();                   // previous block fully consumed
    for (int i = threadIdx.x; i < nt * CB; i += 256) {
      const int tt = i / CB, cc = i % CB;
      if (c0 + cc < C) {
        const size_t row = (size_t)(r0 + tb + tt);
        const float v = ldf<S>(dtp + row * C + c0 + cc) +
                        ldf<S>(dt_bias + c0 + cc);
        s_dt[i] = softplus_f<S>(v);
        s_x[i] = ldf<S>(x + row * C + c0 + cc);
        const float zv = ldf<S>(z + row * ldz + c0 + cc);
        s_z[i] = silu_f<S>(zv);
      }
    }
    for (int i = threadIdx.x; i < nt * N; i += 256) {
      const int t2 = i / N, n = i % N;
      const S* rowp = bc + (size_t)(r0 + tb + t2) * ldbc;
      s_b[i] = ldf<S>(rowp + n);
      s_c[i] = ldf<S>(rowp + N + n);
    }
    __syncthreads();
    auto step = [&](int tt) {
      const float dt = s_dt[tt * CB + cl];
      const float xv = s_x[tt * CB + cl];
      const float dx = dt * xv;
      float y = 0.f;
#pragma unroll
      for (int j = 0; j < PER; ++j) {
        const int n = lane * PER + j;
        if (n < N) {
          st[j] = decay_exp<S>(dt * a[j]) * st[j] + dx * s_b[tt * N + n];
          y += st[j] * s_c[tt * N + n];
        }
      }
      y = lanes_sum<NL>(y);
      if (lane == 0)
        s_y[tt * CB + cl] = (y + dcoef * xv) * s_z[tt * CB + cl];
    };
    for (int tt = 0; tt < nt; ++tt) step(tt);
    __syncthreads();
    for (int i = threadIdx.x; i < nt * CB; i += 256) {
      const int tt = i / CB, cc = i % CB;
      if (c0 + cc < C)
        stf<S>(out + (size_t)(r0 + tb + tt) * C + c0 + cc, s_y[i]);
    }
  }
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int n = lane * PER + j;
    if (okc && n < N) sb[n] = st[j];
  }
}

inline int grid_for(i64 n) {
  i64 g = (n + 255) / 256;
  return (int)(g < 1 ? 1 : (g > 8192 ? 8192 : g));
}

}  // namespace

AF_EXPORT int afm_selective_scan(void* out, void* state, const void* x,
                                 const void* dtp, const void* dt_bias,
                                 const void* bc, i64 ldbc, const void* z,
                                 i64 ldz, const void* A, const void* D,
                                 const void* cu, const void* q_start,
                                 const void* sslot, int B, int C, int N,
                                 int dt, void* stream) {
  if (B == 0) return 0;
  if (N < 1 || N > 256) return 9003;
  hipStream_t s = (hipStream_t)stream;
  // 4 state lanes per channel (64 channels per workgroup) when that still
  // gives the chip enough workgroups, else 16 lanes (16 channels)
  // (AFM_SCAN_MIN_WGS moves the switch-over, for tuning)
  static const long min_wgs = [] {
    const char* e = getenv("AFM_SCAN_MIN_WGS");
    return e ? atol(e) : 1024L;
  }();
  const int nl = (N <= 64 && (i64)B * ((C + 63) / 64) >= min_wgs) ? 4 : 16;
  const int cb = 256 / nl;
  const size_t sm = (size_t)SCAN_TB * (4 * cb + 2 * N) * sizeof(float);
  dim3 grid((C + cb - 1) / cb, B);
  const int per = (N + nl - 1) / nl;
#define SCAN(ST, NL, P)                                                       \
  selective_scan_kernel<ST, NL, P><<<grid, 256, sm, s>>>((ST*)out,            \
      (float*)state, (const ST*)x, (const ST*)dtp, (const ST*)dt_bias,        \
      (const ST*)bc, ldbc, (const ST*)z, ldz, (const float*)A,                \
      (const float*)D, (const i32*)cu, (const i32*)q_start,                   \
      (const i32*)sslot, C, N)
#define SCAN_NL(ST, NL)                             \
  do {                                              \
    if (per <= 1) SCAN(ST, NL, 1);                  \
    else if (per <= 2) SCAN(ST, NL, 2);             \
    else if (per <= 4) SCAN(ST, NL, 4);             \
    else if (per <= 8) SCAN(ST, NL, 8);             \
    else SCAN(ST, NL, 16);                          \
  } while (0)
#define SCAN_PER(ST)                                \
  do {                                              \
    if (nl == 4) SCAN_NL(ST, 4);                    \
    else SCAN_NL(ST, 16);                           \
  } while (0)
  if (dt == 0) SCAN_PER(u16);
  else if (dt == 1) SCAN_PER(float);
  else return 9002;
#undef SCAN_PER
#undef SCAN_NL
#undef SCAN
  return af_last_err();
}
