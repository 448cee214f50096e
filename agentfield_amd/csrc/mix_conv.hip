// Depthwise causal convolution over packed row chunks with the inputs it
// carries from step to step: the short convolution in front of state-space
// and delta-rule mixers.
//
// Storage dtype S is bf16 (raw u16) or fp32; products and sums are fp32.
#include "common.h"

namespace {

template <typename S> __device__ __forceinline__ float ldf(const S* p);
template <> __device__ __forceinline__ float ldf<u16>(const u16* p) { return bf2f(*p); }
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <typename S> __device__ __forceinline__ void stf(S* p, float v);
template <> __device__ __forceinline__ void stf<u16>(u16* p, float v) { *p = f2bf(v); }
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }

// bf16 storage: hardware exponential and reciprocal (the result is rounded
// to 8 bits of mantissa anyway); fp32 storage: the library forms
template <typename S> __device__ __forceinline__ float silu_f(float v);
template <> __device__ __forceinline__ float silu_f<u16>(float v) {
  return v * __frcp_rn(1.0f + __expf(-v));
}
template <> __device__ __forceinline__ float silu_f<float>(float v) {
  return v / (1.0f + expf(-v));
}

inline int grid_for(i64 n) {
  i64 g = (n + 255) / 256;
  return (int)(g < 1 ? 1 : (g > 8192 ? 8192 : g));
}

// ------------------------------------------------------------- convolution
// out[t, c] = silu(b[c] + sum_j w[j, c] * in[t - (taps-1-j), c]), weights
// tap-major [taps, C] so that neighbouring channels load together.  Inputs
// before the chunk come from the sequence's slot of `state`
// [slots, taps-1, C] (the taps-1 inputs before the chunk, oldest first),
// inputs before position 0 are zero.  One workgroup per (row, 256*V
// channels), V channels per thread.
// V consecutive channels per thread (V = 4: 8- or 16-byte accesses).
template <typename S, int V>
__device__ __forceinline__ void ldc(const S* p, float (&o)[4]) {
  if constexpr (V == 1) {
    o[0] = ldf<S>(p);
  } else if constexpr (sizeof(S) == 2) {
    const s16x4 v = *reinterpret_cast<const s16x4*>(p);
#pragma unroll
    for (int j = 0; j < 4; ++j) o[j] = bf2f((u16)v[j]);
  } else {
    const f32x4 v = *reinterpret_cast<const f32x4*>(p);
#pragma unroll
    for (int j = 0; j < 4; ++j) o[j] = v[j];
  }
}
template <typename S, int V>
__device__ __forceinline__ void stc(S* p, const float (&o)[4]) {
  if constexpr (V == 1) {
    stf<S>(p, o[0]);
  } else if constexpr (sizeof(S) == 2) {
    s16x4 v;
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = (short)f2bf(o[j]);
    *reinterpret_cast<s16x4*>(p) = v;
  } else {
    *reinterpret_cast<f32x4*>(p) = f32x4{o[0], o[1], o[2], o[3]};
  }
}

template <typename S, int V>
__global__ void __launch_bounds__(256) causal_conv_kernel(
    S* __restrict__ out, const S* __restrict__ in, i64 ldi,
    const S* __restrict__ w, const S* __restrict__ bias,
    const S* __restrict__ state, const i32* __restrict__ row_seq,
    const i32* __restrict__ cu, const i32* __restrict__ q_start,
    const i32* __restrict__ sslot, int C, int taps, int silu) {
  const int t = blockIdx.x;
  const int c = (blockIdx.y * 256 + threadIdx.x) * V;
  if (c >= C) return;
  const int b = row_seq[t];
  const int k = t - cu[b];                // row inside the chunk
  const int pos = q_start[b] + k;
  const S* st = state + (size_t)sslot[b] * (taps - 1) * C;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  if (bias) ldc<S, V>(bias + c, acc);
  for (int l = 0; l < taps; ++l) {        // lag
    if (pos - l < 0) break;
    float v[4], wv[4];
    if (l <= k) ldc<S, V>(in + (size_t)(t - l) * ldi + c, v);
    else ldc<S, V>(st + (size_t)(taps - 1 - (l - k)) * C + c, v);
    ldc<S, V>(w + (size_t)(taps - 1 - l) * C + c, wv);
#pragma unroll
    for (int j = 0; j < V; ++j) acc[j] += wv[j] * v[j];
  }
  if (silu) {
#pragma unroll
    for (int j = 0; j < V; ++j) acc[j] = silu_f<S>(acc[j]);
  }
  stc<S, V>(out + (size_t)t * C + c, acc);
}

// After the chunk: the slot keeps the last taps-1 inputs of the sequence.
// One thread per (sequence, channel); entry i takes old entry i + L when
// the chunk (L rows) is shorter than the history, read before it is written.
template <typename S>
__global__ void __launch_bounds__(256) conv_state_kernel(
    S* __restrict__ state, const S* __restrict__ in, i64 ldi,
    const i32* __restrict__ cu, const i32* __restrict__ q_start,
    const i32* __restrict__ sslot, int B, int C, int taps) {
  const i64 n = (i64)B * C;
  for (i64 i = (i64)blockIdx.x * 256 + threadIdx.x; i < n;
       i += (i64)gridDim.x * 256) {
    const int b = (int)(i / C), c = (int)(i % C);
    const int r0 = cu[b], L = cu[b + 1] - r0;
    if (L == 0) continue;
    const int start = q_start[b];
    S* st = state + (size_t)sslot[b] * (taps - 1) * C;
    const int hist = taps - 1;
    for (int j = 0; j < hist; ++j) {
      // entry j holds position end - hist + j
      const int k = L - hist + j;         // row inside the chunk
      float v = 0.f;
      if (k >= 0) v = ldf<S>(in + (size_t)(r0 + k) * ldi + c);
      else if (start + k >= 0) v = ldf<S>(st + (size_t)(j + L) * C + c);
      stf<S>(st + (size_t)j * C + c, v);
    }
  }
}

}  // namespace

AF_EXPORT int afm_causal_conv(void* out, const void* in, i64 ldi,
                              const void* w, const void* bias, void* state,
                              const void* row_seq, const void* cu,
                              const void* q_start, const void* sslot, int T,
                              int B, int C, int taps, int silu, int dt,
                              void* stream) {
  if (T == 0) return 0;
  if (taps < 1 || (taps > 1 && !state)) return 9003;
  hipStream_t s = (hipStream_t)stream;
  const bool vec = C % 4 == 0 && ldi % 4 == 0 && (uintptr_t)out % 16 == 0 &&
                   (uintptr_t)in % 16 == 0 && (uintptr_t)bias % 16 == 0 &&
                   (uintptr_t)w % 16 == 0 &&
                   (uintptr_t)state % 16 == 0;
  const int vw = vec ? 4 : 1;
  dim3 grid(T, (C / vw + 255) / 256);
#define CONVK(ST, V)                                                         \
  causal_conv_kernel<ST, V><<<grid, 256, 0, s>>>((ST*)out,                   \
      (const ST*)in, ldi, (const ST*)w, (const ST*)bias, (const ST*)state,   \
      (const i32*)row_seq, (const i32*)cu, (const i32*)q_start,              \
      (const i32*)sslot, C, taps, silu)
#define CONV(ST)                                                             \
  do {                                                                       \
    if (vec) CONVK(ST, 4); else CONVK(ST, 1);                                \
    if (taps > 1)                                                            \
      conv_state_kernel<ST><<<grid_for((i64)B * C), 256, 0, s>>>(            \
          (ST*)state, (const ST*)in, ldi, (const i32*)cu,                    \
          (const i32*)q_start, (const i32*)sslot, B, C, taps);               \
  } while (0)
  if (dt == 0) CONV(u16);
  else if (dt == 1) CONV(float);
  else return 9002;
#undef CONVK
#undef CONV
  return af_last_err();
}
